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

#include <cstring>
#include <sys/stat.h>
#include <unistd.h>

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
    // whole kernel (which spills hundreds of temporaries).  The adjoints are read through a pointer that depends on the
    // loop counter: loads the compiler can prove invariant are moved in front of the loop together with the products
    // that use them, which leaves an addition per term in the loop and a register per product in front of it.
    std::vector<int> outs;
    for (const auto &kv : by_o) outs.push_back(kv.first);
    for (size_t b0 = 0; b0 < outs.size(); b0 += 4) {
      const size_t b1 = std::min(outs.size(), b0 + 4);
      s << "  for (int it = 0; it < one; it++) {\n    const T *Gv = G + it;\n";
      for (size_t q = b0; q < b1; q++) s << "    const T g" << q - b0 << " = Gv[" << outs[q] << " * C];\n";
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

// Block-structured source for a product whose operands do not fit the registers of a thread.  The functions of each
// side come in groups (the rows of one irreducible representation: 2 l + 1 functions); the terms that couple left
// group a with right group b form a block, and every output function belongs to exactly one block.  A thread still owns
// one (atom, channel) column and runs all blocks in turn: the block's operand rows and their adjoints live in registers,
// every term is register arithmetic, and memory sees the operands, the outputs (forward) or their adjoints (reverse)
// and the operand adjoints once per block.  Blocks are ordered by left group, so the left rows and their adjoints stay
// in registers over all blocks of the group.  Returns an empty string when the term list has no such structure (an
// output fed by two blocks, a group with more than kBlockRows functions); the caller then keeps its other kernels.
constexpr int kBlockRows = 16;

inline std::string generate_blocked(const std::vector<ProdTerm> &terms, const std::vector<int> &group_l, const std::vector<int> &group_r, int nfl,
                                    int nfr, int nout, int C, bool f32)
{
  if ((int) group_l.size() != nfl || (int) group_r.size() != nfr || terms.empty()) return "";
  struct Block {
    int a, b;
    std::vector<int> lrows, rrows, outs;
    std::vector<const ProdTerm *> terms;
  };
  std::map<std::pair<int, int>, Block> bm;
  for (const auto &t : terms) {
    if (t.l < 0 || t.l >= nfl || t.r < 0 || t.r >= nfr || t.o < 0 || t.o >= nout) return "";
    Block &B = bm[{group_l[t.l], group_r[t.r]}];
    B.a = group_l[t.l];
    B.b = group_r[t.r];
    B.terms.push_back(&t);
  }
  // rows of a group: every function of the group that any term uses, so that the registers of a left group serve all
  // of its blocks
  std::map<int, std::vector<int>> rows_l, rows_r;
  {
    std::map<int, std::set<int>> sl, sr;
    for (const auto &t : terms) {
      sl[group_l[t.l]].insert(t.l);
      sr[group_r[t.r]].insert(t.r);
    }
    for (auto &kv : sl) rows_l[kv.first].assign(kv.second.begin(), kv.second.end());
    for (auto &kv : sr) rows_r[kv.first].assign(kv.second.begin(), kv.second.end());
  }
  int maxl = 0, maxr = 0;
  for (auto &kv : rows_l) maxl = std::max(maxl, (int) kv.second.size());
  for (auto &kv : rows_r) maxr = std::max(maxr, (int) kv.second.size());
  if (maxl > kBlockRows || maxr > kBlockRows) return "";
  std::vector<int> owner(nout, -1);
  std::vector<Block *> order;
  for (auto &kv : bm) order.push_back(&kv.second);    // map order: by a, then by b
  for (size_t q = 0; q < order.size(); q++) {
    Block &B = *order[q];
    B.lrows = rows_l[B.a];
    B.rrows = rows_r[B.b];
    std::set<int> seen;
    for (const ProdTerm *t : B.terms) {
      if (owner[t->o] >= 0 && owner[t->o] != (int) q) return "";
      owner[t->o] = (int) q;
      if (seen.insert(t->o).second) B.outs.push_back(t->o);
    }
    std::sort(B.outs.begin(), B.outs.end());
  }
  // within a left group the right groups run up and down in turn: neighbouring blocks then share rows in the caches
  {
    size_t q0 = 0;
    int flip = 0;
    while (q0 < order.size()) {
      size_t q1 = q0;
      while (q1 < order.size() && order[q1]->a == order[q0]->a) q1++;
      if (flip) std::reverse(order.begin() + q0, order.begin() + q1);
      flip ^= 1;
      q0 = q1;
    }
  }
  auto index_of = [](const std::vector<int> &v, int x) { return (int) (std::lower_bound(v.begin(), v.end(), x) - v.begin()); };
  std::ostringstream s;
  s << "typedef " << (f32 ? "float" : "double") << " T;\n";
  s << "#define C " << C << "\n";
  auto header = [&](const char *name, const char *args) {
    s << "extern \"C\" __global__ __launch_bounds__(256) void " << name << "(" << args << ", int natoms, int one)\n{\n"
      << "  const long long col = (long long) blockIdx.x * blockDim.x + threadIdx.x;\n"
      << "  const long long at = col / C;\n  const int k = (int) (col % C);\n  if (at >= natoms) return;\n";
  };
  auto declare = [&](const char *stem, int n) {
    s << "  T";
    for (int i = 0; i < n; i++) s << (i ? ", " : " ") << stem << i << " = (T) 0";
    s << ";\n";
  };
  // Every group of statements is the body of a loop that runs `one` (= 1, a kernel argument) times, so that the compiler
  // schedules group by group; the loads of a body go through pointers that depend on the loop counter, or the
  // compiler moves them, and the products that follow them, in front of the loop and keeps every product in a register.
  std::string vary = "    const T *Lv = L + it, *Rv = R + it;\n";
  // ---- forward
  header("prod_fwd", "const T *__restrict__ L, const T *__restrict__ R, T *__restrict__ O");
  s << "  L += at * " << nfl << " * C + k;\n  R += at * " << nfr << " * C + k;\n  O += at * " << nout << " * C + k;\n";
  declare("l", maxl);
  declare("r", maxr);
  {
    bool any = false;
    for (int o = 0; o < nout; o++)
      if (owner[o] < 0) {
        s << "  O[" << o << " * C] = (T) 0;\n";
        any = true;
      }
    if (any) s << "  __asm__ volatile(\"\" ::: \"memory\");\n";
  }
  int cur_a = -1;
  bool have_a = false;
  for (Block *Bp : order) {
    const Block &B = *Bp;
    s << "  for (int it = 0; it < one; it++) {\n" << vary;
    if (!have_a || B.a != cur_a) {
      for (size_t i = 0; i < B.lrows.size(); i++) s << "    l" << i << " = Lv[" << B.lrows[i] << " * C];\n";
      cur_a = B.a;
      have_a = true;
    }
    for (size_t j = 0; j < B.rrows.size(); j++) s << "    r" << j << " = Rv[" << B.rrows[j] << " * C];\n";
    s << "  }\n";
    std::map<int, std::vector<const ProdTerm *>> by_o;
    for (const ProdTerm *t : B.terms) by_o[t->o].push_back(t);
    for (size_t b0 = 0; b0 < B.outs.size(); b0 += 8) {
      // the operands pass through an empty asm statement: the compiler then neither moves the products in front of the
      // loop nor keeps products that two batches share in registers from one batch to the next
      s << "  for (int it = 0; it < one; it++) {\n    T *Ov = O + it;\n    __asm__ volatile(\"\" :";
      for (size_t i = 0; i < B.lrows.size(); i++) s << (i ? ", " : " ") << "\"+v\"(l" << i << ")";
      s << ");\n    __asm__ volatile(\"\" :";
      for (size_t j = 0; j < B.rrows.size(); j++) s << (j ? ", " : " ") << "\"+v\"(r" << j << ")";
      s << ");\n";
      for (size_t x = b0; x < std::min(B.outs.size(), b0 + 8); x++) {
        s << "    Ov[" << B.outs[x] << " * C] = ";
        bool first = true;
        for (const ProdTerm *t : by_o[B.outs[x]]) {
          s << (first ? "" : " + ") << "(T) " << lit(t->c, f32) << " * l" << index_of(B.lrows, t->l) << " * r" << index_of(B.rrows, t->r);
          first = false;
        }
        s << ";\n";
      }
      s << "  }\n";
    }
  }
  s << "}\n\n";
  vary = "    const T *Lv = L + it, *Rv = R + it, *Gv = G + it, *gLv = gL + it, *gRv = gR + it;\n";
  // ---- reverse.  accL / accR: add to the stored adjoint (1) or overwrite it (0)
  header("prod_bwd", "const T *__restrict__ L, const T *__restrict__ R, const T *__restrict__ G, T *__restrict__ gL, T *__restrict__ gR, int accL, int accR");
  s << "  L += at * " << nfl << " * C + k;\n  R += at * " << nfr << " * C + k;\n  G += at * " << nout << " * C + k;\n"
    << "  gL += at * " << nfl << " * C + k;\n  gR += at * " << nfr << " * C + k;\n";
  declare("l", maxl);
  declare("r", maxr);
  declare("gl", maxl);
  declare("gr", maxr);
  {
    // operand rows that no term uses get a zero adjoint when the caller asked for an overwrite
    std::vector<char> usedl(nfl, 0), usedr(nfr, 0);
    for (const auto &t : terms) usedl[t.l] = usedr[t.r] = 1;
    for (int a = 0; a < nfl; a++)
      if (!usedl[a]) s << "  if (!accL) gL[" << a << " * C] = (T) 0;\n";
    for (int b = 0; b < nfr; b++)
      if (!usedr[b]) s << "  if (!accR) gR[" << b << " * C] = (T) 0;\n";
  }
  std::set<int> visited_r;
  for (size_t q = 0; q < order.size(); q++) {
    const Block &B = *order[q];
    const bool first_of_a = q == 0 || order[q - 1]->a != B.a, last_of_a = q + 1 == order.size() || order[q + 1]->a != B.a;
    s << "  for (int it = 0; it < one; it++) {\n" << vary;
    if (first_of_a)
      for (size_t i = 0; i < B.lrows.size(); i++)
        s << "    l" << i << " = Lv[" << B.lrows[i] << " * C]; gl" << i << " = accL ? gLv[" << B.lrows[i] << " * C] : (T) 0;\n";
    const bool again = visited_r.count(B.b) != 0;
    visited_r.insert(B.b);
    for (size_t j = 0; j < B.rrows.size(); j++) {
      s << "    r" << j << " = Rv[" << B.rrows[j] << " * C]; gr" << j << " = ";
      if (again) s << "gRv[" << B.rrows[j] << " * C];\n";
      else s << "accR ? gRv[" << B.rrows[j] << " * C] : (T) 0;\n";
    }
    s << "  }\n";
    std::map<int, std::vector<const ProdTerm *>> by_o;
    for (const ProdTerm *t : B.terms) by_o[t->o].push_back(t);
    for (size_t b0 = 0; b0 < B.outs.size(); b0 += 8) {
      const size_t b1 = std::min(B.outs.size(), b0 + 8);
      s << "  for (int it = 0; it < one; it++) {\n" << vary;
      for (size_t x = b0; x < b1; x++) s << "    const T g" << x - b0 << " = Gv[" << B.outs[x] << " * C];\n";
      for (size_t x = b0; x < b1; x++)
        for (const ProdTerm *t : by_o[B.outs[x]]) {
          const int i = index_of(B.lrows, t->l), j = index_of(B.rrows, t->r);
          s << "    { const T cg = (T) " << lit(t->c, f32) << " * g" << x - b0 << "; gl" << i << " += cg * r" << j << "; gr" << j << " += cg * l" << i << "; }\n";
        }
      s << "  }\n";
    }
    s << "  for (int it = 0; it < one; it++) {\n";
    for (size_t j = 0; j < B.rrows.size(); j++) s << "    gR[" << B.rrows[j] << " * C] = gr" << j << ";\n";
    if (last_of_a)
      for (size_t i = 0; i < B.lrows.size(); i++) s << "    gL[" << B.lrows[i] << " * C] = gl" << i << ";\n";
    s << "  }\n";
  }
  s << "}\n";
  return s.str();
}

// ---- code objects on disk
inline std::string cache_dir()
{
  const char *e = std::getenv("GRACE_HIP_CACHE");
  if (e && e[0] == '0' && e[1] == 0) return "";
  if (e && e[0]) return e;
  const char *x = std::getenv("XDG_CACHE_HOME");
  if (x && x[0]) return std::string(x) + "/grace_hip";
  const char *h = std::getenv("HOME");
  if (h && h[0]) return std::string(h) + "/.cache/grace_hip";
  return "";
}
// file of the code object of `key` (architecture, options and source): two independent 64-bit FNV-1a digests of the key
// and of the compiler's version in its name; "" when there is no cache directory
inline std::string cache_file(const std::string &key)
{
  const std::string dir = cache_dir();
  if (dir.empty()) return "";
  int major = 0, minor = 0;
  (void) hiprtcVersion(&major, &minor);
  const std::string full = "hiprtc " + std::to_string(major) + "." + std::to_string(minor) + "\n" + key;
  unsigned long long h1 = 1469598103934665603ULL, h2 = 0x9E3779B97F4A7C15ULL;
  for (unsigned char ch : full) {
    h1 = (h1 ^ ch) * 1099511628211ULL;
    h2 = (h2 ^ (ch + 0x5bULL)) * 0x100000001B3ULL + (h2 >> 29);
  }
  char name[64];
  std::snprintf(name, sizeof name, "%016llx%016llx_%zu.co", h1, h2, full.size());
  return dir + "/" + name;
}
// A cache file is the code object followed by 24 bytes: a tag, the length of the code object and an FNV-1a digest of its
// bytes.  A file without them (cut short, damaged, of another layout) is not handed to the driver.
constexpr unsigned long long kCacheTag = 0x4f43504948524721ULL;
inline unsigned long long bytes_digest(const char *p, size_t n)
{
  unsigned long long h = 1469598103934665603ULL;
  for (size_t q = 0; q < n; q++) h = (h ^ (unsigned char) p[q]) * 1099511628211ULL;
  return h;
}
inline void seal(std::vector<char> &data)
{
  const unsigned long long t[3] = {kCacheTag, (unsigned long long) data.size(), bytes_digest(data.data(), data.size())};
  const char *b = reinterpret_cast<const char *>(t);
  data.insert(data.end(), b, b + sizeof t);
}
// true and the trailer removed when `data` is a whole sealed file
inline bool unseal(std::vector<char> &data)
{
  unsigned long long t[3];
  if (data.size() < sizeof t + 64) return false;
  std::memcpy(t, data.data() + data.size() - sizeof t, sizeof t);
  const size_t n = data.size() - sizeof t;
  if (t[0] != kCacheTag || t[1] != n || t[2] != bytes_digest(data.data(), n)) return false;
  data.resize(n);
  return true;
}
inline bool read_file(const std::string &path, std::vector<char> &out)
{
  FILE *f = std::fopen(path.c_str(), "rb");
  if (!f) return false;
  std::fseek(f, 0, SEEK_END);
  const long n = std::ftell(f);
  std::fseek(f, 0, SEEK_SET);
  bool ok = n > 0;
  if (ok) {
    out.resize((size_t) n);
    ok = std::fread(out.data(), 1, (size_t) n, f) == (size_t) n;
  }
  std::fclose(f);
  return ok;
}
// written under a temporary name and renamed: a reader never sees half a file, two writers of the same key write the same bytes
inline void write_file_atomically(const std::string &path, const std::vector<char> &data)
{
  const size_t slash = path.rfind('/');
  if (slash != std::string::npos) {
    std::string dir = path.substr(0, slash), cmd;
    for (size_t q = 1; q <= dir.size(); q++)    // the directories on the way, one by one
      if (q == dir.size() || dir[q] == '/') (void) ::mkdir(dir.substr(0, q).c_str(), 0700);
  }
  const std::string tmp = path + ".tmp" + std::to_string((long long) ::getpid());
  FILE *f = std::fopen(tmp.c_str(), "wb");
  if (!f) return;
  const bool ok = std::fwrite(data.data(), 1, data.size(), f) == data.size();
  if (std::fclose(f) != 0 || !ok || std::rename(tmp.c_str(), path.c_str()) != 0) (void) std::remove(tmp.c_str());
}

}    // namespace jit_detail

// Compiles the two kernels of a generated source for the current device.  Returns false (with the reason in `why`)
// when hiprtc cannot be used; the caller then keeps the table-driven kernels.  GRACE_HIP_JIT=0 switches the
// specialisation off, GRACE_HIP_JIT_DUMP=<dir> writes the generated sources there.
inline bool jit_compile_source(const char *name, const std::string &src, bool f32, const std::string &arch, JitKernels &out, std::string &why,
                               bool in_order = false, const char *fwd_name = "prod_fwd", const char *bwd_name = "prod_bwd")
{
  const char *sw = std::getenv("GRACE_HIP_JIT");
  if (sw && sw[0] == '0') {
    why = "switched off by GRACE_HIP_JIT=0";
    return false;
  }
  if (src.empty()) {
    why = "no source";
    return false;
  }
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
  const std::string key = arch + (in_order ? "\nin order\n" : "\n") + src;
  out.release();
  std::shared_ptr<const std::vector<char>> obj;
  {
    std::lock_guard<std::mutex> lk(cache_mu);
    auto it = cache.find(key);
    if (it != cache.end()) obj = it->second;
  }
  // and across processes: a directory of code objects keyed by a digest of (architecture, compiler version, options, source);
  // the reference ships its product tables compiled (libgrace/include/grace/kk/cg_tables.h), here the second process that
  // loads a model finds its kernels on disk.  GRACE_HIP_CACHE=<dir> names the directory (default ~/.cache/grace_hip),
  // GRACE_HIP_CACHE=0 switches the disk cache off.
  const std::string disk = jit_detail::cache_file(key);
  bool from_disk = false;
  if (!obj && !disk.empty()) {
    std::vector<char> code;
    if (jit_detail::read_file(disk, code)) {
      if (jit_detail::unseal(code)) {
        obj = std::make_shared<const std::vector<char>>(std::move(code));
        from_disk = true;
      } else {
        (void) std::remove(disk.c_str());    // cut short or damaged: compiled again below and written anew
      }
    }
  }
  // a whole file that the driver does not load (written for another driver) is dropped as well and the source compiled
  if (from_disk) {
    if (hipModuleLoadData(&out.mod, obj->data()) == hipSuccess) {
      std::lock_guard<std::mutex> lk(cache_mu);
      cache[key] = obj;
    } else {
      (void) hipGetLastError();
      out.mod = nullptr;
      obj.reset();
      (void) std::remove(disk.c_str());
    }
  }
  if (!obj) {
    hiprtcProgram prog;
    if (hiprtcCreateProgram(&prog, src.c_str(), name, 0, nullptr, nullptr) != HIPRTC_SUCCESS) {
      why = "hiprtcCreateProgram failed";
      return false;
    }
    const std::string a = "--offload-arch=" + arch;
    // no packed fp32 instructions (as in the Makefile of the library).  in_order: the generated statements are already
    // in the order they should run in, and the machine scheduler would take most of the compile time of a long list
    const char *opts[] = {a.c_str(), "-O3", "-ffp-contract=fast", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-mllvm", "-enable-misched=false"};
    const hiprtcResult rc = hiprtcCompileProgram(prog, in_order ? 9 : 7, opts);
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
    if (!disk.empty()) {
      std::vector<char> sealed(*obj);
      jit_detail::seal(sealed);
      jit_detail::write_file_atomically(disk, sealed);
    }
    std::lock_guard<std::mutex> lk(cache_mu);
    cache[key] = obj;
  }
  if (!out.mod && hipModuleLoadData(&out.mod, obj->data()) != hipSuccess) {
    (void) hipGetLastError();
    out.mod = nullptr;
    why = "hipModuleLoadData failed";
    return false;
  }
  if (hipModuleGetFunction(&out.fwd, out.mod, fwd_name) != hipSuccess || hipModuleGetFunction(&out.bwd, out.mod, bwd_name) != hipSuccess) {
    (void) hipGetLastError();
    out.release();
    why = "kernel not found in the compiled module";
    return false;
  }
  return true;
}

inline bool jit_compile_product(const char *name, const std::vector<ProdTerm> &terms, int nfl, int nfr, int nout, bool self,
                                int C, bool f32, const std::string &arch, JitKernels &out, std::string &why)
{
  if (terms.empty()) {
    why = "no terms";
    return false;
  }
  return jit_compile_source(name, jit_detail::generate(terms, nfl, nfr, nout, self, C, f32), f32, arch, out, why);
}

// The block-structured kernels of a product between two different tensors whose functions come in groups
// (group_l[f], group_r[f]: the group of every left and right function).
inline bool jit_compile_blocked(const char *name, const std::vector<ProdTerm> &terms, const std::vector<int> &group_l, const std::vector<int> &group_r,
                                int nfl, int nfr, int nout, int C, bool f32, const std::string &arch, JitKernels &out, std::string &why)
{
  const std::string src = jit_detail::generate_blocked(terms, group_l, group_r, nfl, nfr, nout, C, f32);
  if (src.empty()) {
    why = "the term list has no block structure";
    return false;
  }
  return jit_compile_source(name, src, f32, arch, out, why, true);
}

}    // namespace grhip
