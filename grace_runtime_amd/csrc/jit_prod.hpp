// Model-specialised kernels of the channel-wise Clebsch-Gordan products, generated as straight-line HIP code from the
// model's own term lists and compiled with hiprtc when the engine is created.
//
// A product acts on every (atom, channel) column independently: out[o] = sum_t c_t L[l_t] R[r_t].  With the term list
// known, a thread owns one column, keeps the operands it needs in registers and runs the terms as an unrolled
// instruction stream with literal coefficients and literal addresses: no index tables, no address arithmetic, every
// function read once.  The reference specialises the same products at build time for the shapes of its registry
// models (libgrace/include/grace/kk/cg_tables.h, `ShapeProd_*` in kk/grace_1l_fused_kk_impl.h:828-856) and runs a
// table-driven kernel otherwise (kk/fused_dense.h:610-645); here the specialisation happens for whatever model is
// loaded, and the table-driven kernels (k_prod_fwd / k_prod_bwd) remain as the path when hiprtc is unavailable.
#pragma once

#include "npz.hpp"

#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <set>
#include <sstream>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

namespace grhip {

struct ProdTerm {
  int l, r, o;
  double c;
};

struct JitKernels {
  hipModule_t mod = nullptr;
  hipFunction_t fwd = nullptr, bwd = nullptr;
  bool ok() const { return mod != nullptr; }
  void release()
  {
    if (mod) (void) hipModuleUnload(mod);
    mod = nullptr;
    fwd = bwd = nullptr;
  }
};

namespace jit_detail {

constexpr int kRegMax = 32;    // operand functions of one side kept (with their adjoints) in registers

inline std::string lit(double v, bool f32)
{
  char b[64];
  if (f32) std::snprintf(b, sizeof b, "%.9gf", v);
  else std::snprintf(b, sizeof b, "%.17g", v);
  std::string s(b);
  if (s.find('.') == std::string::npos && s.find('e') == std::string::npos && s.find("inf") == std::string::npos) {
    if (f32) s.insert(s.size() - 1, ".0");
    else s += ".0";
  }
  return s;
}

// Source of the forward and reverse kernels of one product.
//   self: both operands are the same tensor (then nfl == nfr and the adjoints are one tensor too)
//   C: channels per function (the thread's column stride is C elements between functions)
inline std::string generate(const std::vector<ProdTerm> &terms, int nfl, int nfr, int nout, bool self, int C, bool f32)
{
  std::ostringstream s;
  s << "typedef " << (f32 ? "float" : "double") << " T;\n";
  s << "#define C " << C << "\n";
  std::set<int> liveL, liveR;
  for (const auto &t : terms) {
    liveL.insert(t.l);
    (self ? liveL : liveR).insert(t.r);
  }
  if (self) liveR = liveL;
  const bool regL = (int) liveL.size() <= kRegMax, regR = (int) liveR.size() <= kRegMax;
  auto Lv = [&](int a) { return regL ? "l" + std::to_string(a) : "L[" + std::to_string(a) + " * C]"; };
  auto Rv = [&](int b) {
    if (self) return Lv(b);
    return regR ? "r" + std::to_string(b) : "R[" + std::to_string(b) + " * C]";
  };
  std::map<int, std::vector<const ProdTerm *>> by_o, by_l, by_r;
  for (const auto &t : terms) {
    by_o[t.o].push_back(&t);
    by_l[t.l].push_back(&t);
    by_r[t.r].push_back(&t);
  }
  // keeps the compiler from hoisting the loads of later statements to the top (register pressure)
  const char *fence = "  __asm__ volatile(\"\" ::: \"memory\");\n";
  auto header = [&](const char *name, const char *args) {
    s << "extern \"C\" __global__ __launch_bounds__(256) void " << name << "(" << args << ", int natoms, int one)\n{\n"
      << "  const long long col = (long long) blockIdx.x * blockDim.x + threadIdx.x;\n"
      << "  const long long at = col / C;\n  const int k = (int) (col % C);\n  if (at >= natoms) return;\n";
  };
  auto load_regs = [&]() {
    if (regL)
      for (int a : liveL) s << "  const T l" << a << " = L[" << a << " * C];\n";
    if (!self && regR)
      for (int b : liveR) s << "  const T r" << b << " = R[" << b << " * C];\n";
  };
  // ---- forward
  header("prod_fwd", "const T *__restrict__ L, const T *__restrict__ R, T *__restrict__ O");
  s << "  L += at * " << nfl << " * C + k;\n  R += at * " << nfr << " * C + k;\n  O += at * " << nout << " * C + k;\n";
  load_regs();
  for (const auto &kv : by_o) {
    s << "  O[" << kv.first << " * C] = ";
    bool first = true;
    for (const ProdTerm *t : kv.second) {
      s << (first ? "" : " + ") << "(T) " << lit(t->c, f32) << " * " << Lv(t->l) << " * " << Rv(t->r);
      first = false;
    }
    s << ";\n" << fence;
  }
  s << "}\n\n";
  // ---- reverse.  accL / accR: add to the stored adjoint (1) or overwrite it (0)
  header("prod_bwd", "const T *__restrict__ L, const T *__restrict__ R, const T *__restrict__ G, T *gL, T *gR, int accL, int accR");
  s << "  L += at * " << nfl << " * C + k;\n  R += at * " << nfr << " * C + k;\n  G += at * " << nout << " * C + k;\n"
    << "  gL += at * " << nfl << " * C + k;\n  gR += at * " << nfr << " * C + k;\n";
  load_regs();
  if (regL)
    for (int a : liveL) s << "  T gl" << a << " = (T) 0;\n";
  if (!self && regR)
    for (int b : liveR) s << "  T gr" << b << " = (T) 0;\n";
  auto gLn = [&](int a) { return "gl" + std::to_string(a); };
  auto gRn = [&](int b) { return self ? "gl" + std::to_string(b) : "gr" + std::to_string(b); };
  const bool accumL = regL, accumR = self ? regL : regR;
  if (accumL || accumR) {
    // Stream over the outputs once, in batches of 8: the batch's adjoints g are loaded together, then its terms
    // update the register-held operand adjoints.  Every batch is the body of a loop that runs `one` (= 1, a kernel
    // argument) times: separate basic blocks, so the compiler schedules batch by batch instead of interleaving the
    // whole kernel (which spills hundreds of temporaries).
    std::vector<int> outs;
    for (const auto &kv : by_o) outs.push_back(kv.first);
    for (size_t b0 = 0; b0 < outs.size(); b0 += 4) {
      const size_t b1 = std::min(outs.size(), b0 + 4);
      s << "  for (int it = 0; it < one; it++) {\n";
      for (size_t q = b0; q < b1; q++) s << "    const T g" << q - b0 << " = G[" << outs[q] << " * C];\n";
      for (size_t q = b0; q < b1; q++)
        for (const ProdTerm *t : by_o[outs[q]]) {
          s << "    { const T cg = (T) " << lit(t->c, f32) << " * g" << q - b0 << ";";
          if (accumL) s << " " << gLn(t->l) << " += cg * " << Rv(t->r) << ";";
          if (accumR) s << " " << gRn(t->r) << " += cg * " << Lv(t->l) << ";";
          s << " }\n";
        }
      s << "  }\n";
    }
  }
  if (self) {
    if (regL) {
      for (int a : liveL) s << "  gL[" << a << " * C] = accL ? gL[" << a << " * C] + gl" << a << " : gl" << a << ";\n";
    } else {
      // gather per operand function, both sides merged
      for (int a : liveL) {
        s << "  {\n    T v = (T) 0;\n";
        if (by_l.count(a))
          for (const ProdTerm *t : by_l[a]) s << "    v += (T) " << lit(t->c, f32) << " * G[" << t->o << " * C] * " << Lv(t->r) << ";\n";
        if (by_r.count(a))
          for (const ProdTerm *t : by_r[a]) s << "    v += (T) " << lit(t->c, f32) << " * G[" << t->o << " * C] * " << Lv(t->l) << ";\n";
        s << "    gL[" << a << " * C] = accL ? gL[" << a << " * C] + v : v;\n  }\n" << fence;
      }
    }
  } else {
    if (regL) {
      for (int a : liveL) s << "  gL[" << a << " * C] = accL ? gL[" << a << " * C] + gl" << a << " : gl" << a << ";\n";
    } else {
      for (int a : liveL) {
        s << "  {\n    T v = (T) 0;\n";
        for (const ProdTerm *t : by_l[a]) s << "    v += (T) " << lit(t->c, f32) << " * G[" << t->o << " * C] * " << Rv(t->r) << ";\n";
        s << "    gL[" << a << " * C] = accL ? gL[" << a << " * C] + v : v;\n  }\n" << fence;
      }
    }
    if (regR) {
      for (int b : liveR) s << "  gR[" << b << " * C] = accR ? gR[" << b << " * C] + gr" << b << " : gr" << b << ";\n";
    } else {
      for (int b : liveR) {
        s << "  {\n    T v = (T) 0;\n";
        for (const ProdTerm *t : by_r[b]) s << "    v += (T) " << lit(t->c, f32) << " * G[" << t->o << " * C] * " << Lv(t->l) << ";\n";
        s << "    gR[" << b << " * C] = accR ? gR[" << b << " * C] + v : v;\n  }\n" << fence;
      }
    }
  }
  s << "}\n";
  return s.str();
}

}    // namespace jit_detail

// Compiles the two kernels of a product for the current device.  Returns false (with the reason in `why`) when hiprtc
// cannot be used; the caller then keeps the table-driven kernels.  GRACE_HIP_JIT=0 switches the specialisation off,
// GRACE_HIP_JIT_DUMP=<dir> writes the generated sources there.
inline bool jit_compile_product(const char *name, const std::vector<ProdTerm> &terms, int nfl, int nfr, int nout, bool self,
                                int C, bool f32, const std::string &arch, JitKernels &out, std::string &why)
{
  const char *sw = std::getenv("GRACE_HIP_JIT");
  if (sw && sw[0] == '0') {
    why = "switched off by GRACE_HIP_JIT=0";
    return false;
  }
  if (terms.empty()) {
    why = "no terms";
    return false;
  }
  const std::string src = jit_detail::generate(terms, nfl, nfr, nout, self, C, f32);
  if (const char *dir = std::getenv("GRACE_HIP_JIT_DUMP")) {
    const std::string p = std::string(dir) + "/" + name + (f32 ? "_f32" : "_f64") + ".hip";
    if (FILE *f = std::fopen(p.c_str(), "w")) {
      std::fputs(src.c_str(), f);
      std::fclose(f);
    }
  }
  // compiled code objects of the process by (architecture, source): a second engine of the same model, or a fresh one
  // after a reset, loads the code without compiling it again
  static std::mutex cache_mu;
  static std::map<std::string, std::shared_ptr<const std::vector<char>>> cache;
  const std::string key = arch + "\n" + src;
  std::shared_ptr<const std::vector<char>> obj;
  {
    std::lock_guard<std::mutex> lk(cache_mu);
    auto it = cache.find(key);
    if (it != cache.end()) obj = it->second;
  }
  if (!obj) {
    hiprtcProgram prog;
    if (hiprtcCreateProgram(&prog, src.c_str(), name, 0, nullptr, nullptr) != HIPRTC_SUCCESS) {
      why = "hiprtcCreateProgram failed";
      return false;
    }
    const std::string a = "--offload-arch=" + arch;
    const char *opts[] = {a.c_str(), "-O3", "-ffp-contract=fast"};
    const hiprtcResult rc = hiprtcCompileProgram(prog, 3, opts);
    if (rc != HIPRTC_SUCCESS) {
      size_t ls = 0;
      hiprtcGetProgramLogSize(prog, &ls);
      std::string log(ls, ' ');
      if (ls) hiprtcGetProgramLog(prog, &log[0]);
      why = "hiprtc: " + log.substr(0, 400);
      hiprtcDestroyProgram(&prog);
      return false;
    }
    size_t cs = 0;
    hiprtcGetCodeSize(prog, &cs);
    std::vector<char> code(cs);
    hiprtcGetCode(prog, code.data());
    hiprtcDestroyProgram(&prog);
    obj = std::make_shared<const std::vector<char>>(std::move(code));
    std::lock_guard<std::mutex> lk(cache_mu);
    cache[key] = obj;
  }
  if (hipModuleLoadData(&out.mod, obj->data()) != hipSuccess) {
    (void) hipGetLastError();
    out.mod = nullptr;
    why = "hipModuleLoadData failed";
    return false;
  }
  if (hipModuleGetFunction(&out.fwd, out.mod, "prod_fwd") != hipSuccess || hipModuleGetFunction(&out.bwd, out.mod, "prod_bwd") != hipSuccess) {
    (void) hipGetLastError();
    out.release();
    why = "kernel not found in the compiled module";
    return false;
  }
  return true;
}

}    // namespace grhip
