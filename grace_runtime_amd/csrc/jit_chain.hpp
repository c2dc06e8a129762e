// The per-atom dense chain of a GRACE layer as TWO generated kernels (forward, reverse) instead of one launch per FC
// layer and product:
//
//   X1  = FC1 (X0, X0)                      (A1 = fc_A1(A, A))
//   P2  = X1 x X1                           (AA: channel-wise Clebsch-Gordan product)
//   P21 = FC21(P2, X0), P22 = FC22(P2, X0)  (AA1, AA2)
//   P3  = P21 x (X1 | X0)                   (AAA)
//   P4  = P22 x P22                         (AAAA)
//
// (stage order of libgrace/src/fused_1l.cpp:260-300, reverse :306-349; FC libgrace/include/grace/fused_cpu.h:349-364,
// products :409-475).  Launched stage by stage, every tensor of the chain makes a round trip through HBM per stage (P2
// alone is 36 kB per atom in fp64); the stages themselves are cheap, so the chain is bound by that traffic.  Here a block
// of 256 threads owns NA = 256 / C atoms and keeps the chain on chip:
//
// * a thread is one (atom, channel) column, as in the generated product kernels: X1 (and in the reverse its adjoint) of the
//   column live in registers, the products are straight-line code with literal coefficients;
// * the FC layers mix the channels of a column, so they run on the matrix cores: the columns of a 16x16x4 MFMA are
//   "items" = (atom, function) pairs that share a weight tile (the 2 L + 1 functions of one coupling path of all NA
//   atoms), the A operand is the weight tile in fragment order (read from global memory once per path and wave, into
//   registers, before the barrier that precedes its use), the B operand an LDS row of the item, the result goes back to
//   an LDS row.  The column threads hand a path's product values to the matrix cores through LDS and take the FC
//   results back from it: per path two barriers;
// * P2 is never stored (the reduce's functions excepted); P21 and P22 are written for the reverse, P3 and P4 for the
//   reduce; the reverse never materialises the adjoints of P2, P21, P22 and X1;
// * P4 couples functions of different paths: paths are joined into groups (connected components of the P4 term list:
//   the paths of one L), a group's P22 functions stay in registers until the group's P4 outputs are formed.
//
// The generator refuses (returns false with a reason) what it does not cover: channel widths other than 32, FC
// functions with other than one right connection, groups too large for the register file.  The engine then keeps its
// stage-by-stage kernels.
#pragma once

#include "jit_prod.hpp"
#include "model.hpp"

#include <functional>
#include <numeric>

namespace grhip {

struct ChainFcSpec {
  int nfunc = 0;                       // output functions (= functions of the left input)
  int n_out = 0, n_in_l = 0, n_in_r = 0, ntiles = 0;    // real widths of the file's weight arrays
  std::vector<char> live;              // outputs that are computed
  std::vector<int> tile_l;             // weight tile of the left segment of function f
  std::vector<int> from, tile_r;       // right-input function of f and the weight tile of that connection
  std::vector<double> nof;             // norm_out_factor
  const std::vector<double> *w_left = nullptr, *w_right = nullptr;    // [n_out][n_in][tiles]
  double norm_l = 1.0, norm_r = 1.0;
  bool ok = true;                      // false: a function with other than one right connection
  std::string why;
};

struct ChainSpec {
  int C = 32;
  bool f32 = false;
  int nf0 = 0;                  // functions of X0
  ChainFcSpec fc1;
  int nP2 = 0;
  std::vector<ProdTerm> prod2;
  ChainFcSpec fc21, fc22;
  bool have22 = false;
  int nP3 = 0;
  std::vector<ProdTerm> prod3;
  bool prod3_right_x0 = false;
  // P3 inside the kernels (its outputs are accumulated in registers: for the few scalar outputs of a readout chain) or left to
  // the product kernels of the caller (many outputs): the forward kernel then only writes P21, the reverse kernel reads the
  // adjoint of P21 from gP21, and the adjoint of X0 that the reverse of P3 leaves in gX0 is added to, for every function
  bool fuse3 = true;
  int nP4 = 0;
  std::vector<ProdTerm> prod4;
  std::vector<char> keepP2;     // P2 functions read outside the chain (reduce, UQ): written forward, adjoint read in the reverse
  std::vector<char> keepX0;     // X0 functions whose adjoint holds a contribution from outside the chain when the reverse starts
  int drow[16];                 // accumulator row of (lane / 16, register) of the 16x16x4 MFMA
};

struct ChainCode {
  std::string src;
  std::vector<double> weights;    // fragment-ordered weight units of both kernels
  std::string why;
  int atoms_per_block = 0;
  double flops_per_atom = 0.0;    // of the FC layers of one direction (live functions, padded widths; 2 per multiply-add)
};

struct ChainKernels {
  hipModule_t mod = nullptr;
  hipFunction_t fwd = nullptr, bwd = nullptr;
  int atoms_per_block = 0;
  double flops_per_atom = 0.0;
  bool ok() const { return mod != nullptr; }
  void release()
  {
    if (mod) (void) hipModuleUnload(mod);
    mod = nullptr;
    fwd = bwd = nullptr;
  }
};

namespace chain_detail {

using jit_detail::lit;

struct Path {
  int f0 = 0, M = 0;
  bool l21 = false, l22 = false, any = false;    // any: some function of the path is computed at all
  int tl21 = -1, tr21 = -1, r21 = -1, tl22 = -1, tr22 = -1, r22 = -1;
  int group = -1;
};

struct Fc1Path {
  int f0 = 0, M = 0, tl = -1, tr = -1, r0 = -1;
};

inline double tile_w(const std::vector<double> &w, double norm, int nin, int nt, int k, int n, int t)
{
  return norm * w[((size_t) k * nin + n) * nt + t];
}

// one weight unit [k-steps][lane]: the A operand of the MFMAs of one (matrix, 16-row block): lane (g, i) of step s holds
// M(rb * 16 + i, 4 s + g)
inline void pack_unit(std::vector<double> &out, const std::function<double(int, int)> &M, int rb, int ksteps)
{
  for (int s = 0; s < ksteps; s++)
    for (int lane = 0; lane < 64; lane++) out.push_back(M(rb * 16 + (lane & 15), 4 * s + (lane >> 4)));
}

}    // namespace chain_detail

inline ChainFcSpec chain_fc_spec(const FCWeights &w, const std::vector<char> &live, int nf_right)
{
  ChainFcSpec s;
  s.nfunc = w.n_funcs;
  s.n_out = w.n_out;
  s.n_in_l = w.n_in_left;
  s.n_in_r = w.n_in_right;
  s.ntiles = w.tiles_left;
  s.live = live;
  s.tile_l = w.w_tile_left;
  s.from.assign(w.n_funcs, -1);
  s.tile_r.assign(w.n_funcs, -1);
  s.nof = w.norm_out_factor;
  s.w_left = &w.w_left;
  s.w_right = &w.w_right;
  s.norm_l = w.norm_left;
  s.norm_r = w.norm_right;
  if (w.tiles_left != w.tiles_right) {
    s.ok = false;
    s.why = "left and right weight arrays hold different numbers of tiles";
    return s;
  }
  std::vector<int> nconn(w.n_funcs, 0);
  for (int c = 0; c < w.n_conn; c++) {
    const int f = w.collect_to[c];
    if (f < 0 || f >= w.n_funcs || w.collect_from[c] < 0 || w.collect_from[c] >= nf_right) {
      s.ok = false;
      s.why = "connection out of range";
      return s;
    }
    nconn[f]++;
    s.from[f] = w.collect_from[c];
    s.tile_r[f] = w.w_tile_right[c];
  }
  for (int f = 0; f < w.n_funcs; f++)
    if (live[f] && nconn[f] != 1) {
      s.ok = false;
      s.why = "a function with " + std::to_string(nconn[f]) + " right connections";
      return s;
    }
  return s;
}

// Source of chain_fwd / chain_bwd and their weight units.
inline bool generate_chain(const ChainSpec &sp, ChainCode &out)
{
  using namespace chain_detail;
  const int C = sp.C;
  if (C != 32) { out.why = "channel width " + std::to_string(C) + " (the fused chain covers 32)"; return false; }
  if (!sp.fc1.ok) { out.why = "fc1: " + sp.fc1.why; return false; }
  if (!sp.fc21.ok) { out.why = "fc21: " + sp.fc21.why; return false; }
  if (sp.have22 && !sp.fc22.ok) { out.why = "fc22: " + sp.fc22.why; return false; }
  if (sp.fc1.nfunc != sp.nf0 || sp.fc21.nfunc != sp.nP2 || (sp.have22 && sp.fc22.nfunc != sp.nP2)) { out.why = "function counts differ"; return false; }
  const int NA = 256 / C, KS = C / 4, RB = C / 16;
  const int PAD = sp.f32 ? 4 : 2, S = C + PAD;    // LDS row stride: 16 bytes over the row, so the 16 items of an MFMA column block fall on different banks
  const int maxM = 9;
  const bool f32 = sp.f32;
  const int nf0 = sp.nf0, nP2 = sp.nP2, nP3 = sp.nP3, nP4 = sp.have22 ? sp.nP4 : 0;

  // ---- functions that are computed
  std::vector<char> live21 = sp.fc21.live, live22 = sp.have22 ? sp.fc22.live : std::vector<char>(nP2, 0);
  std::vector<char> keep2 = sp.keepP2;
  keep2.resize(nP2, 0);
  std::map<int, std::vector<const ProdTerm *>> p2_by_o, p3_by_o, p3_by_l, p4_by_o, p4_by_l, p4_by_r;
  for (const auto &t : sp.prod2) {
    if (t.o < 0 || t.o >= nP2 || t.l < 0 || t.l >= nf0 || t.r < 0 || t.r >= nf0) { out.why = "prod2 term out of range"; return false; }
    if (!sp.fc1.live[t.l] || !sp.fc1.live[t.r]) { out.why = "prod2 reads a function fc1 does not compute"; return false; }
    p2_by_o[t.o].push_back(&t);
  }
  for (const auto &t : sp.prod3) {
    if (t.o < 0 || t.o >= nP3 || t.l < 0 || t.l >= nP2 || t.r < 0 || t.r >= nf0) { out.why = "prod3 term out of range"; return false; }
    if (!live21[t.l]) { out.why = "prod3 reads a function fc21 does not compute"; return false; }
    p3_by_o[t.o].push_back(&t);
    p3_by_l[t.l].push_back(&t);
  }
  if (sp.have22)
    for (const auto &t : sp.prod4) {
      if (t.o < 0 || t.o >= nP4 || t.l < 0 || t.l >= nP2 || t.r < 0 || t.r >= nP2) { out.why = "prod4 term out of range"; return false; }
      if (!live22[t.l] || !live22[t.r]) { out.why = "prod4 reads a function fc22 does not compute"; return false; }
      p4_by_o[t.o].push_back(&t);
      p4_by_l[t.l].push_back(&t);
      p4_by_r[t.r].push_back(&t);
    }

  // ---- paths of P2: runs of functions with one weight signature and contiguous right inputs
  std::vector<Path> paths;
  std::vector<int> path_of(nP2, -1);
  {
    auto sig = [&](int f) {
      std::vector<int> v;
      v.push_back(live21[f]);
      v.push_back(live21[f] ? sp.fc21.tile_l[f] : -1);
      v.push_back(live21[f] ? sp.fc21.tile_r[f] : -1);
      v.push_back(live21[f] ? sp.fc21.from[f] - f : 0);
      v.push_back(live22[f]);
      v.push_back(live22[f] ? sp.fc22.tile_l[f] : -1);
      v.push_back(live22[f] ? sp.fc22.tile_r[f] : -1);
      v.push_back(live22[f] ? sp.fc22.from[f] - f : 0);
      return v;
    };
    for (int f = 0; f < nP2; f++) {
      const bool fresh = paths.empty() || paths.back().M >= maxM || sig(f) != sig(f - 1);
      if (fresh) {
        Path p;
        p.f0 = f;
        p.l21 = live21[f];
        p.l22 = live22[f];
        if (p.l21) { p.tl21 = sp.fc21.tile_l[f]; p.tr21 = sp.fc21.tile_r[f]; p.r21 = sp.fc21.from[f]; }
        if (p.l22) { p.tl22 = sp.fc22.tile_l[f]; p.tr22 = sp.fc22.tile_r[f]; p.r22 = sp.fc22.from[f]; }
        paths.push_back(p);
      }
      Path &p = paths.back();
      p.M++;
      p.any = p.any || live21[f] || live22[f] || keep2[f];
      path_of[f] = (int) paths.size() - 1;
    }
    for (const Path &p : paths) {
      if ((p.l21 && (p.r21 < 0 || p.r21 + p.M > nf0)) || (p.l22 && (p.r22 < 0 || p.r22 + p.M > nf0))) { out.why = "right inputs of a path out of range"; return false; }
      if ((p.l21 && (p.tl21 < 0 || p.tl21 >= sp.fc21.ntiles || p.tr21 < 0 || p.tr21 >= sp.fc21.ntiles)) ||
          (p.l22 && (p.tl22 < 0 || p.tl22 >= sp.fc22.ntiles || p.tr22 < 0 || p.tr22 >= sp.fc22.ntiles))) { out.why = "weight tile out of range"; return false; }
    }
  }
  // ---- groups: paths joined by P4 terms
  std::vector<int> grp(paths.size());
  std::iota(grp.begin(), grp.end(), 0);
  std::function<int(int)> find = [&](int x) { return grp[x] == x ? x : grp[x] = find(grp[x]); };
  if (sp.have22)
    for (const auto &t : sp.prod4) grp[find(path_of[t.l])] = find(path_of[t.r]);
  std::map<int, std::vector<int>> groups;    // root -> paths (ascending)
  for (size_t q = 0; q < paths.size(); q++) groups[find((int) q)].push_back((int) q);
  std::vector<std::vector<int>> order;
  for (auto &kv : groups) order.push_back(kv.second);
  std::sort(order.begin(), order.end(), [](const std::vector<int> &a, const std::vector<int> &b) { return a[0] < b[0]; });
  for (const auto &g : order) {
    int regs = 0;
    for (int q : g)
      if (paths[q].l22) regs += paths[q].M;
    if (regs > 72) { out.why = "a group of " + std::to_string(regs) + " coupled functions does not fit the registers"; return false; }
  }
  std::vector<int> group_of_p4(nP4, -1);
  for (size_t gi = 0; gi < order.size(); gi++)
    for (int q : order[gi]) paths[q].group = (int) gi;
  for (const auto &kv : p4_by_o) group_of_p4[kv.first] = paths[path_of[kv.second[0]->l]].group;

  // ---- paths of FC1
  std::vector<Fc1Path> f1;
  for (int f = 0; f < nf0; f++) {
    if (!sp.fc1.live[f]) continue;    // a function no product reads: not computed, its adjoint is zero
    const bool fresh = f1.empty() || f1.back().f0 + f1.back().M != f || f1.back().M >= maxM || sp.fc1.tile_l[f] != f1.back().tl || sp.fc1.tile_r[f] != f1.back().tr ||
                       sp.fc1.from[f] != f1.back().r0 + f1.back().M;
    if (fresh) {
      Fc1Path p;
      p.f0 = f; p.tl = sp.fc1.tile_l[f]; p.tr = sp.fc1.tile_r[f]; p.r0 = sp.fc1.from[f];
      if (p.tl < 0 || p.tl >= sp.fc1.ntiles || p.tr < 0 || p.tr >= sp.fc1.ntiles || p.r0 < 0) { out.why = "fc1 tile out of range"; return false; }
      f1.push_back(p);
    }
    f1.back().M++;
  }
  for (const Fc1Path &p : f1)
    if (p.r0 + p.M > nf0) { out.why = "fc1 right inputs out of range"; return false; }

  // ---- weight units
  std::vector<double> &W = out.weights;
  W.clear();
  auto mat = [&](const ChainFcSpec &fc, bool right, int t) {
    const std::vector<double> *w = right ? fc.w_right : fc.w_left;
    const double norm = right ? fc.norm_r : fc.norm_l;
    const int nin = right ? fc.n_in_r : fc.n_in_l, nt = fc.ntiles, no = fc.n_out;
    return [w, norm, nin, nt, no, t](int k, int n) { return (k < no && n < nin) ? tile_w(*w, norm, nin, nt, k, n, t) : 0.0; };
  };
  // forward unit: rows = output channels, columns = input channels; reverse unit: the transpose
  auto unit_fwd = [&](const ChainFcSpec &fc, bool right, int t, int rb) {
    auto m = mat(fc, right, t);
    pack_unit(W, [&](int r, int c) { return m(r, c); }, rb, KS);
  };
  auto unit_bwd = [&](const ChainFcSpec &fc, bool right, int t, int rb) {
    auto m = mat(fc, right, t);
    pack_unit(W, [&](int r, int c) { return m(c, r); }, rb, KS);
  };
  struct WaveUnits { long long off[4]; int nseg; };
  // forward FC1: pairs (rb), two segments
  std::vector<WaveUnits> wu_f1(f1.size()), wu_f1b(f1.size());
  for (size_t q = 0; q < f1.size(); q++) {
    for (int rb = 0; rb < RB; rb++) {
      wu_f1[q].off[rb] = wu_f1[q].off[rb + 2] = (long long) W.size();
      unit_fwd(sp.fc1, false, f1[q].tl, rb);
      unit_fwd(sp.fc1, true, f1[q].tr, rb);
    }
    wu_f1[q].nseg = 2;
  }
  // forward paths: pairs (out, rb), two segments each
  std::vector<WaveUnits> wu_p(paths.size()), wu_pb(paths.size());
  for (size_t q = 0; q < paths.size(); q++) {
    const Path &p = paths[q];
    wu_p[q].nseg = 2;
    if (p.l21 && p.l22) {
      for (int o = 0; o < 2; o++)
        for (int rb = 0; rb < RB; rb++) {
          wu_p[q].off[o * 2 + rb] = (long long) W.size();
          unit_fwd(o ? sp.fc22 : sp.fc21, false, o ? p.tl22 : p.tl21, rb);
          unit_fwd(o ? sp.fc22 : sp.fc21, true, o ? p.tr22 : p.tr21, rb);
        }
    } else if (p.l21 || p.l22) {
      const ChainFcSpec &fc = p.l22 ? sp.fc22 : sp.fc21;
      for (int rb = 0; rb < RB; rb++) {
        wu_p[q].off[rb] = wu_p[q].off[rb + 2] = (long long) W.size();
        unit_fwd(fc, false, p.l22 ? p.tl22 : p.tl21, rb);
        unit_fwd(fc, true, p.l22 ? p.tr22 : p.tr21, rb);
      }
    }
  }
  // reverse paths: pairs (left -> adjoint of P2 | right -> adjoint of X0, rb); segments: the live layers
  for (size_t q = 0; q < paths.size(); q++) {
    const Path &p = paths[q];
    wu_pb[q].nseg = (p.l21 ? 1 : 0) + (p.l22 ? 1 : 0);
    if (!wu_pb[q].nseg) continue;
    for (int side = 0; side < 2; side++)
      for (int rb = 0; rb < RB; rb++) {
        wu_pb[q].off[side * 2 + rb] = (long long) W.size();
        if (p.l21) unit_bwd(sp.fc21, side == 1, side ? p.tr21 : p.tl21, rb);
        if (p.l22) unit_bwd(sp.fc22, side == 1, side ? p.tr22 : p.tl22, rb);
      }
  }
  // reverse FC1: left and right rows coincide -> pairs (rb) with two segments; else pairs (side, rb) with one
  for (size_t q = 0; q < f1.size(); q++) {
    const bool same = f1[q].r0 == f1[q].f0;
    wu_f1b[q].nseg = same ? 2 : 1;
    if (same) {
      for (int rb = 0; rb < RB; rb++) {
        wu_f1b[q].off[rb] = wu_f1b[q].off[rb + 2] = (long long) W.size();
        unit_bwd(sp.fc1, false, f1[q].tl, rb);
        unit_bwd(sp.fc1, true, f1[q].tr, rb);
      }
    } else {
      for (int side = 0; side < 2; side++)
        for (int rb = 0; rb < RB; rb++) {
          wu_f1b[q].off[side * 2 + rb] = (long long) W.size();
          unit_bwd(sp.fc1, side == 1, side ? f1[q].tr : f1[q].tl, rb);
        }
    }
  }

  int XM = 1;
  for (const Path &p : paths) XM = std::max(XM, p.M);
  for (const Fc1Path &p : f1) XM = std::max(XM, p.M);
  const int XR = XM * NA;    // rows of a hand-over buffer

  // ---- source
  std::ostringstream s;
  s << "typedef " << (f32 ? "float" : "double") << " T;\n";
  s << "typedef T v4 __attribute__((ext_vector_type(4)));\n";
  s << "#define ST(dst, val) dst = val\n";
  s << "#define LDW(p, q) (p)[(q) * 64]\n";
  s << "#define MMA(a, b, c) " << (f32 ? "__builtin_amdgcn_mfma_f32_16x16x4f32" : "__builtin_amdgcn_mfma_f64_16x16x4f64") << "(a, b, c, 0, 0, 0)\n";
  s << "#define C " << C << "\n#define NA " << NA << "\n#define S " << S << "\n#define KS " << KS << "\n";
  // The barrier between the column phase and the matrix phase of a path orders LDS traffic only: the weight requests of the
  // next step and the stores of the results to global memory stay in flight across it (__syncthreads would wait for them).
  s << "#define SYNC() __asm__ volatile(\"s_waitcnt lgkmcnt(0)\\n\\ts_barrier\" ::: \"memory\")\n";
  s << "__device__ const int DROW[16] = {";
  for (int q = 0; q < 16; q++) s << (q ? ", " : "") << sp.drow[q];
  s << "};\n";
  // One wave, one 16-row block of the output: D[row][item] = sum over the segments of W_seg (16 x C) B_seg (C x items),
  // items in column blocks of 16 from cb0 in steps of cbstep.  wf: the weight fragments of the segments (KS each); B0 / B1 /
  // Y: LDS rows of item 0; acc: add to the row instead of writing it.
  s << R"(
// One wave, one 16-row block of the output: D[row][item] = sum over the segments of W_seg (16 x C) B_seg (C x items), items
// in column blocks of 16 from cb0 in steps of CBSTEP.  wf: the weight fragments of the segments (KS each); B0 / B1 / Y: LDS
// rows of item 0; acc: add to the row instead of writing it.  wn / wq / NNEXT: the buffer, the lane's source pointer and the
// count of the NEXT step's weight fragments, requested one per matrix instruction of the first column block: the
// vector-memory pipe of the CU takes 8 cycles per request, and 16 requests per wave issued in one burst (next to the burst
// of stores of the column phase) hold the issuing waves up.
template<int NSEG, int NITEMS, int CBSTEP, int NNEXT, int PIPE>
__device__ inline __attribute__((always_inline)) void fc_rows(const T (&wf)[2 * KS], T (&wn)[2 * KS], const T *wq, const T *B0, const T *B1, T *Y, int cb0,
                                                              int rb, int acc, int lane)
{
  constexpr int NCB = (NITEMS + 15) / 16, MAXT = (NCB + CBSTEP - 1) / CBSTEP, NK = NSEG * KS;
  const int g = lane >> 4, c = lane & 15;
  const int d0 = DROW[4 * g], d1 = DROW[4 * g + 1], d2 = DROW[4 * g + 2], d3 = DROW[4 * g + 3];
  // PIPE: the B fragments of a column block and (acc) the old values of its output rows are requested while the matrix
  // instructions of the block before it run, so that nothing but arithmetic and writes is left for the end of a block (the
  // reverse kernel, whose output rows are read, added to and written); else at the start of the block itself (fewer registers)
  T b[2][NK], o[2][4];
  auto request = [&](int cb, T (&dst)[NK], T (&old)[4]) {
    const int item = cb * 16 + c, it = item < NITEMS ? item : NITEMS - 1;
    const T *p0 = B0 + it * S + g;
#pragma unroll
    for (int q = 0; q < KS; q++) dst[q] = p0[4 * q];
    if (NSEG == 2) {
      const T *p1 = B1 + it * S + g;
#pragma unroll
      for (int q = 0; q < KS; q++) dst[KS + q] = p1[4 * q];
    }
    if (acc) {
      const T *y = Y + it * S + rb * 16;
      old[0] = y[d0]; old[1] = y[d1]; old[2] = y[d2]; old[3] = y[d3];
    } else {
      old[0] = old[1] = old[2] = old[3] = (T) 0;
    }
  };
  if (cb0 >= NCB) {    // a wave without a column block in this step
#pragma unroll
    for (int q = 0; q < NNEXT; q++) wn[q] = LDW(wq, q);
  } else if (PIPE) {
    request(cb0, b[0], o[0]);
  }
#pragma unroll
  for (int t = 0; t < MAXT; t++) {
    const int cb = cb0 + t * CBSTEP;
    if (cb < NCB) {
      if (PIPE) {
        if (t + 1 < MAXT && cb + CBSTEP < NCB) request(cb + CBSTEP, b[(t + 1) & 1], o[(t + 1) & 1]);
      } else {
        request(cb, b[t & 1], o[t & 1]);
      }
      __builtin_amdgcn_sched_barrier(0);
      v4 d = {0, 0, 0, 0};
      if (t == 0) {
#pragma unroll
        for (int q = 0; q < NK; q++) {
          d = MMA(wf[q], b[0][q], d);    // t == 0
          if (q < NNEXT) wn[q] = LDW(wq, q);
        }
#pragma unroll
        for (int q = NK; q < NNEXT; q++) wn[q] = LDW(wq, q);
#pragma unroll
        for (int q = 0; q < NK; q++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
        }
      } else {
#pragma unroll
        for (int q = 0; q < NK; q++) d = MMA(wf[q], b[t & 1][q], d);
      }
      __builtin_amdgcn_sched_barrier(0);
      const int item = cb * 16 + c;
      if (item < NITEMS) {
        T *y = Y + item * S + rb * 16;
        y[d0] = o[t & 1][0] + d[0]; y[d1] = o[t & 1][1] + d[1]; y[d2] = o[t & 1][2] + d[2]; y[d3] = o[t & 1][3] + d[3];
      }
    }
  }
}
)";
  auto woff = [&](const WaveUnits &u) {
    std::ostringstream o;
    o << "(wave == 0 ? " << u.off[0] << "LL : wave == 1 ? " << u.off[1] << "LL : wave == 2 ? " << u.off[2] << "LL : " << u.off[3] << "LL)";
    return o.str();
  };
  // The weight fragments of a step (one path's FC phase) are requested one step ahead, into the buffer the current step
  // does not use: a request issued right before its barrier is answered after ~2 us, longer than the products of a path take.
  std::vector<const WaveUnits *> steps;    // the steps of the kernel being written, in execution order
  size_t step = 0;
  // the first step's fragments are requested at the start of the kernel; every step requests the next one's
  auto request_wf = [&](size_t k) {
    if (k >= steps.size()) return;
    const WaveUnits &u = *steps[k];
    s << "    { const T *wq = W + " << woff(u) << " + lane;\n";
    s << "#pragma unroll\n      for (int q = 0; q < " << u.nseg * KS << "; q++) wf" << (k & 1) << "[q] = LDW(wq, q); }\n";
  };
  // begin_step: template and call arguments of fc_rows that name this step's buffer and the next step's request
  struct StepArgs { std::string nnext, bufs; };
  auto begin_step = [&]() {
    StepArgs a;
    const bool more = step + 1 < steps.size();
    a.nnext = std::to_string(more ? steps[step + 1]->nseg * KS : 0);
    const std::string cur = (step & 1) ? "wf1" : "wf0", nxt = (step & 1) ? "wf0" : "wf1";
    a.bufs = cur + ", " + nxt + ", W + " + (more ? woff(*steps[step + 1]) : std::string("0")) + " + lane";
    step++;
    return a;
  };
  auto common_head = [&](const char *lds_decl) {
    s << "  " << lds_decl << "\n";
    s << "  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);\n";
    s << "  const int a = tid / C, n = tid % C;\n";
    // every tensor holds rows for a whole number of blocks (the caller pads the atom count to a multiple of NA): the
    // columns of the atoms past the end compute on whatever those rows hold and write rows nobody reads, so no load or
    // store is guarded and the column phases are branch-free (a guarded store ends a scheduling region: the LDS reads of
    // a phase then wait for each other)
    s << "  const long long at = (long long) blockIdx.x * NA + a;\n";
    s << "  (void) natoms;\n";
    s << "  const int col = a * S + n;    // this thread's element of row 0 of a buffer whose rows are (function, atom)\n";
    s << "  T wf0[2 * KS], wf1[2 * KS];\n";
  };
  auto sum_terms = [&](const std::vector<const ProdTerm *> &ts, const std::function<std::string(const ProdTerm *)> &f) {
    std::ostringstream o;
    if (ts.empty()) return std::string("(T) 0");
    bool first = true;
    for (const ProdTerm *t : ts) {
      o << (first ? "" : " + ") << "(T) " << lit(t->c, f32) << " * " << f(t);
      first = false;
    }
    return o.str();
  };
  auto x1 = [](int f) { return "x1_" + std::to_string(f); };
  auto xr = [&](int f) { return (sp.prod3_right_x0 ? "x0_" : "x1_") + std::to_string(f); };
  auto v2 = [](int f) { return "v2_" + std::to_string(f); };

  // =========================================================== forward
  s << "extern \"C\" __global__ __launch_bounds__(256) void chain_fwd(const T *__restrict__ X0, T *__restrict__ X1, T *__restrict__ P2, "
       "T *__restrict__ P21, T *__restrict__ P22, T *__restrict__ P3, T *__restrict__ P4, const T *__restrict__ W, int natoms, int one)\n{\n";
  {
    std::ostringstream d;
    d << "__shared__ T L0[" << nf0 * NA * S << "], LX[" << XR * S << "], LY1[" << XR * S << "], LY2[" << XR * S << "];";
    common_head(d.str().c_str());
  }
  s << "  X0 += at * " << nf0 << " * C + n; X1 += at * " << nf0 << " * C + n; P2 += at * " << nP2 << " * C + n; P21 += at * " << nP2
    << " * C + n; P22 += at * " << nP2 << " * C + n; P3 += at * " << std::max(nP3, 1) << " * C + n; P4 += at * " << std::max(nP4, 1) << " * C + n;\n";
  for (int f = 0; f < nf0; f++) s << "  L0[" << f * NA * S << " + col] = X0[" << f << " * C];\n";
  for (int f = 0; f < nf0; f++) s << "  T " << x1(f) << ";\n";
  if (sp.fuse3)
    for (int o = 0; o < nP3; o++) s << "  T p3_" << o << " = (T) 0;\n";
  // the steps of the forward kernel: FC1 paths, then the paths of P2 with an FC phase, group by group
  steps.clear();
  step = 0;
  for (size_t q = 0; q < f1.size(); q++) steps.push_back(&wu_f1[q]);
  for (const auto &g : order)
    for (int q : g)
      if (paths[q].any && (paths[q].l21 || paths[q].l22)) steps.push_back(&wu_p[q]);
  request_wf(0);
  // FC1
  for (size_t q = 0; q < f1.size(); q++) {
    const Fc1Path &p = f1[q];
    s << "  {    // FC1, functions " << p.f0 << " .. " << p.f0 + p.M - 1 << "\n";
    const StepArgs wf = begin_step();
    s << "    SYNC();\n";
    s << "    fc_rows<2, " << p.M * NA << ", 2, " << wf.nnext << ", 0>(" << wf.bufs << ", L0 + " << p.f0 * NA * S << ", L0 + " << p.r0 * NA * S << ", LY1, wave >> 1, wave & 1, 0, lane);\n";
    s << "    SYNC();\n";
    for (int i = 0; i < p.M; i++) {
      const int f = p.f0 + i;
      s << "    " << x1(f) << " = (T) " << lit(sp.fc1.nof[f], f32) << " * LY1[" << i * NA * S << " + col]; X1[" << f << " * C] = " << x1(f) << ";\n";
    }
    s << "  }\n";
  }
  // P2 paths, group by group
  for (const auto &g : order) {
    bool any = false;
    for (int q : g) any = any || paths[q].any;
    if (!any) continue;
    s << "  {    // group of paths";
    for (int q : g) s << " " << q;
    s << "\n";
    for (int q : g)
      if (paths[q].l22)
        for (int i = 0; i < paths[q].M; i++) s << "    T " << v2(paths[q].f0 + i) << ";\n";
    std::set<int> outs4;
    for (int q : g) {
      const Path &p = paths[q];
      if (!p.any) continue;
      const bool gemm = p.l21 || p.l22;
      s << "    {    // path " << q << ": functions " << p.f0 << " .. " << p.f0 + p.M - 1 << "\n";
      const StepArgs wf = gemm ? begin_step() : StepArgs();
      for (int i = 0; i < p.M; i++) {
        const int f = p.f0 + i;
        const auto it = p2_by_o.find(f);
        const std::string e = sum_terms(it == p2_by_o.end() ? std::vector<const ProdTerm *>() : it->second,
                                        [&](const ProdTerm *t) { return x1(t->l) + " * " + x1(t->r); });
        s << "      { const T v = " << e << ";";
        if (gemm) s << " LX[" << i * NA * S << " + col] = v;";
        if (keep2[f]) s << " ST(P2[" << f << " * C], v);";
        s << " }\n";
      }
      if (gemm) {
        s << "      SYNC();\n";
        if (p.l21 && p.l22)
          s << "      fc_rows<2, " << p.M * NA << ", 1, " << wf.nnext << ", 0>(" << wf.bufs << ", LX, L0 + (wave < 2 ? " << p.r21 * NA * S << " : " << p.r22 * NA * S
            << "), wave < 2 ? LY1 : LY2, 0, wave & 1, 0, lane);\n";
        else
          s << "      fc_rows<2, " << p.M * NA << ", 2, " << wf.nnext << ", 0>(" << wf.bufs << ", LX, L0 + " << (p.l22 ? p.r22 : p.r21) * NA * S << ", " << (p.l22 ? "LY2" : "LY1")
            << ", wave >> 1, wave & 1, 0, lane);\n";
        s << "      SYNC();\n";
        for (int i = 0; i < p.M; i++) {
          const int f = p.f0 + i;
          if (live21[f]) {
            s << "      { const T v = (T) " << lit(sp.fc21.nof[f], f32) << " * LY1[" << i * NA * S << " + col]; ST(P21[" << f << " * C], v);";
            const auto it = p3_by_l.find(f);
            if (sp.fuse3 && it != p3_by_l.end())
              for (const ProdTerm *t : it->second)
                s << " p3_" << t->o << " += (T) " << lit(t->c, f32) << " * v * "
                  << (sp.prod3_right_x0 ? "L0[" + std::to_string(t->r * NA * S) + " + col]" : x1(t->r)) << ";";    // X0 is resident in LDS
            s << " }\n";
          }
          if (live22[f]) {
            s << "      " << v2(f) << " = (T) " << lit(sp.fc22.nof[f], f32) << " * LY2[" << i * NA * S << " + col]; ST(P22[" << f << " * C], " << v2(f)
              << ");\n";
            for (const auto *m : {&p4_by_l, &p4_by_r}) {
              const auto it = m->find(f);
              if (it != m->end())
                for (const ProdTerm *t : it->second) outs4.insert(t->o);
            }
          }
        }
      }
      s << "    }\n";
    }
    if (!outs4.empty()) {
      s << "    {\n";
      for (int o : outs4)
        s << "      ST(P4[" << o << " * C], " << sum_terms(p4_by_o[o], [&](const ProdTerm *t) { return v2(t->l) + " * " + v2(t->r); }) << ");\n";
      s << "    }\n";
    }
    s << "  }\n";
  }
  s << "  {\n";
  if (sp.fuse3)
    for (int o = 0; o < nP3; o++) s << "    P3[" << o << " * C] = p3_" << o << ";\n";
  for (int o = 0; o < nP4; o++)
    if (!p4_by_o.count(o)) s << "    P4[" << o << " * C] = (T) 0;\n";
  s << "  }\n}\n\n";

  // =========================================================== reverse
  s << "extern \"C\" __global__ __launch_bounds__(256) void chain_bwd(const T *__restrict__ X0, const T *__restrict__ X1, const T *__restrict__ P21, "
       "const T *__restrict__ P22, const T *__restrict__ gP2, const T *__restrict__ gP3, const T *__restrict__ gP4, const T *__restrict__ gP21, "
       "T *__restrict__ gX0, "
       "const T *__restrict__ W, int natoms, int one)\n{\n";
  {
    std::ostringstream d;
    d << "__shared__ T LG[" << nf0 * NA * S << "], LX1[" << XR * S << "], LX2[" << XR * S << "], LY[" << XR * S << "];";
    common_head(d.str().c_str());
  }
  s << "  X0 += at * " << nf0 << " * C + n; X1 += at * " << nf0 << " * C + n; P21 += at * " << nP2 << " * C + n; P22 += at * " << nP2
    << " * C + n; gP2 += at * " << nP2 << " * C + n; gP3 += at * " << std::max(nP3, 1) << " * C + n; gP4 += at * " << std::max(nP4, 1)
    << " * C + n; gX0 += at * " << nf0 << " * C + n; gP21 += at * " << nP2 << " * C + n;\n";

  for (int f = 0; f < nf0; f++)
    if (sp.fc1.live[f]) s << "  const T " << x1(f) << " = X1[" << f << " * C];\n";
  if (sp.prod3_right_x0 && sp.fuse3)
    for (int f = 0; f < nf0; f++) s << "  const T x0_" << f << " = X0[" << f << " * C];\n";
  for (int f = 0; f < nf0; f++) s << "  T g1_" << f << " = (T) 0;\n";
  if (sp.fuse3)
    for (int o = 0; o < nP3; o++) s << "  const T g3_" << o << " = gP3[" << o << " * C];\n";
  auto gr = [&](int f) { return (sp.prod3_right_x0 ? "gx0_" : "g1_") + std::to_string(f); };
  // the reverse of P3 with respect to its right operand needs P21 only here: all of it up front, with every load in flight
  // at once, instead of a load per path whose latency nothing hides (one wave per SIMD)
  // (when the right operand is X0 the sums are the initial values of the LDS rows in which the adjoint of X0 is gathered)
  s << "  {\n";
  if (sp.fuse3) {
    if (sp.prod3_right_x0)
      for (int f = 0; f < nf0; f++) s << "    T gx0_" << f << " = (T) 0;\n";
    for (const auto &kv : p3_by_l) s << "    const T p_" << kv.first << " = P21[" << kv.first << " * C];\n";
    for (const auto &kv : p3_by_l)
      for (const ProdTerm *t : kv.second) s << "    " << gr(t->r) << " += (T) " << lit(t->c, f32) << " * g3_" << t->o << " * p_" << kv.first << ";\n";
  }
  for (int f = 0; f < nf0; f++)
    s << "    LG[" << f * NA * S << " + col] = " << (sp.prod3_right_x0 && sp.fuse3 ? "gx0_" + std::to_string(f) : std::string("(T) 0")) << ";\n";
  s << "  }\n";
  // the P22 rows and the P4 adjoints of a group are requested one path ahead of the group (behind the column phase of the
  // last path of the group before it, whose own rows are dead by then), so that they arrive during that path's matrix phase
  for (int f = 0; f < nP2; f++)
    if (live22[f]) s << "  T " << v2(f) << ";\n";
  for (int o = 0; o < nP4; o++)
    if (p4_by_o.count(o)) s << "  T g4_" << o << ";\n";
  std::vector<size_t> live_groups;
  for (size_t gi = 0; gi < order.size(); gi++) {
    bool any = false;
    for (int q : order[gi]) any = any || paths[q].any;
    if (any) live_groups.push_back(gi);
  }
  auto group_loads = [&](size_t gi, const char *p22, const char *g4p, const char *indent) {
    std::set<int> outs4;
    for (int q : order[gi])
      if (paths[q].l22)
        for (int i = 0; i < paths[q].M; i++) {
          const int f = paths[q].f0 + i;
          s << indent << v2(f) << " = " << p22 << "[" << f << " * C];\n";
          for (const auto *m : {&p4_by_l, &p4_by_r}) {
            const auto it = m->find(f);
            if (it != m->end())
              for (const ProdTerm *t : it->second) outs4.insert(t->o);
          }
        }
    for (int o : outs4) s << indent << "g4_" << o << " = " << g4p << "[" << o << " * C];\n";
  };
  if (!live_groups.empty()) {
    s << "  for (int it = 0; it < one; it++) {\n    const T *P22v = P22 + it, *gP4v = gP4 + it;\n";
    group_loads(live_groups[0], "P22v", "gP4v", "    ");
    s << "  }\n";
  }
  // the steps of the reverse kernel: the paths of P2 with an FC phase, group by group, then the FC1 paths
  steps.clear();
  step = 0;
  for (const auto &g : order)
    for (int q : g)
      if (paths[q].any && (paths[q].l21 || paths[q].l22)) steps.push_back(&wu_pb[q]);
  for (size_t q = 0; q < f1.size(); q++) steps.push_back(&wu_f1b[q]);
  request_wf(0);
  for (const auto &g : order) {
    bool any = false;
    for (int q : g) any = any || paths[q].any;
    if (!any) continue;
    // every group is the body of a loop that runs `one` (= 1, a kernel argument) times and reads global memory through
    // pointers that depend on the loop counter: the compiler then keeps the loads of a group inside it (it otherwise
    // starts them groups ahead and spills what they return)
    s << "  for (int it = 0; it < one; it++) {    // group of paths";
    for (int q : g) s << " " << q;
    s << "\n";
    s << "    const T *P22v = P22 + it, *gP4v = gP4 + it;\n";
    // the last path of this group with a matrix phase requests the next group's rows
    int last_gemm = -1;
    for (int q : g)
      if (paths[q].any && (paths[q].l21 || paths[q].l22)) last_gemm = q;
    size_t next_group = order.size();
    for (size_t k = 0; k + 1 < live_groups.size(); k++)
      if (&order[live_groups[k]] == &g) next_group = live_groups[k + 1];
    bool next_requested = false;
    for (int q : g) {
      const Path &p = paths[q];
      if (!p.any) continue;
      const bool gemm = p.l21 || p.l22;
      s << "    for (int ip = 0; ip < one; ip++) {    // path " << q << ": functions " << p.f0 << " .. " << p.f0 + p.M - 1 << "\n";
      s << "      const T *P22w = P22v + ip, *gP4w = gP4v + ip, *gP2w = gP2 + it + ip, *gP21w = gP21 + it + ip;\n";
      // the adjoints that the reduces left on this path's functions: requested here, used behind the matrix phase
      for (int i = 0; i < p.M; i++)
        if (keep2[p.f0 + i] && p2_by_o.count(p.f0 + i)) s << "      const T gk_" << p.f0 + i << " = gP2w[" << p.f0 + i << " * C];\n";
      const StepArgs wf = gemm ? begin_step() : StepArgs();
      if (gemm) {
        for (int i = 0; i < p.M; i++) {
          const int f = p.f0 + i;
          if (p.l21) {
            if (live21[f]) {
              const auto it = p3_by_l.find(f);
              const std::vector<const ProdTerm *> none;
              const auto &ts = it == p3_by_l.end() ? none : it->second;
              if (sp.fuse3)
                s << "      LX1[" << i * NA * S << " + col] = (T) " << lit(sp.fc21.nof[f], f32) << " * ("
                  << sum_terms(ts, [&](const ProdTerm *t) { return "g3_" + std::to_string(t->o) + " * " + xr(t->r); }) << ");\n";
              else
                s << "      LX1[" << i * NA * S << " + col] = (T) " << lit(sp.fc21.nof[f], f32) << " * gP21w[" << f << " * C];\n";
            } else {
              s << "      LX1[" << i * NA * S << " + col] = (T) 0;\n";
            }
          }
          if (p.l22) {
            if (live22[f]) {
              std::ostringstream e;
              bool first = true;
              const auto il = p4_by_l.find(f), ir = p4_by_r.find(f);
              if (il != p4_by_l.end())
                for (const ProdTerm *t : il->second) {
                  e << (first ? "" : " + ") << "(T) " << lit(t->c, f32) << " * (g4_" << t->o << " * " << v2(t->r) << ")";
                  first = false;
                }
              if (ir != p4_by_r.end())
                for (const ProdTerm *t : ir->second) {
                  e << (first ? "" : " + ") << "(T) " << lit(t->c, f32) << " * (g4_" << t->o << " * " << v2(t->l) << ")";
                  first = false;
                }
              if (first) e << "(T) 0";
              s << "      LX2[" << i * NA * S << " + col] = (T) " << lit(sp.fc22.nof[f], f32) << " * (" << e.str() << ");\n";
            } else {
              s << "      LX2[" << i * NA * S << " + col] = (T) 0;\n";
            }
          }
        }
        if (q == last_gemm && next_group < order.size()) {
          group_loads(next_group, "P22w", "gP4w", "      ");
          next_requested = true;
        }
        s << "      SYNC();\n";
        // waves 0, 1: adjoint of P2 (left weights) into LY; waves 2, 3: adjoint of X0 (right weights) added to its rows
        const char *b0 = p.l21 ? "LX1" : "LX2";
        const int rr = p.l21 ? p.r21 : p.r22;
        if (p.l21 && p.l22 && p.r21 != p.r22) { out.why = "the two layers of a path read different right inputs"; return false; }
        s << "      fc_rows<" << wu_pb[q].nseg << ", " << p.M * NA << ", 1, " << wf.nnext << ", 1>(" << wf.bufs << ", " << b0 << ", LX2, wave < 2 ? LY : LG + " << rr * NA * S
          << ", 0, wave & 1, wave >> 1, lane);\n";
        s << "      SYNC();\n";
      }
      for (int i = 0; i < p.M; i++) {
        const int f = p.f0 + i;
        const auto it = p2_by_o.find(f);
        if (it == p2_by_o.end()) continue;
        if (!gemm && !keep2[f]) continue;
        s << "      { const T g = ";
        if (gemm) s << "LY[" << i * NA * S << " + col]";
        if (gemm && keep2[f]) s << " + ";
        if (keep2[f]) s << "gk_" << f;
        s << ";";
        for (const ProdTerm *t : it->second) {
          s << " { const T cg = (T) " << lit(t->c, f32) << " * g; g1_" << t->l << " += cg * " << x1(t->r) << "; g1_" << t->r << " += cg * " << x1(t->l)
            << "; }";
        }
        s << " }\n";
      }
      s << "    }\n";
    }
    if (!next_requested && next_group < order.size()) group_loads(next_group, "P22v", "gP4v", "    ");
    s << "  }\n";
  }
  // reverse of FC1
  for (size_t q = 0; q < f1.size(); q++) {
    const Fc1Path &p = f1[q];
    const bool same = p.r0 == p.f0;
    s << "  {    // FC1 reverse, functions " << p.f0 << " .. " << p.f0 + p.M - 1 << "\n";
    const StepArgs wf = begin_step();
    for (int i = 0; i < p.M; i++) {
      const int f = p.f0 + i;
      s << "    LX1[" << i * NA * S << " + col] = (T) " << lit(sp.fc1.nof[f], f32) << " * g1_" << f << ";\n";
    }
    s << "    SYNC();\n";
    if (same)
      s << "    fc_rows<2, " << p.M * NA << ", 2, " << wf.nnext << ", 1>(" << wf.bufs << ", LX1, LX1, LG + " << p.f0 * NA * S << ", wave >> 1, wave & 1, 1, lane);\n";
    else
      s << "    fc_rows<1, " << p.M * NA << ", 1, " << wf.nnext << ", 1>(" << wf.bufs << ", LX1, LX1, LG + (wave < 2 ? " << p.f0 * NA * S << " : " << p.r0 * NA * S << "), 0, wave & 1, 1, lane);\n";
    s << "    SYNC();\n";
    s << "  }\n";
  }
  // when left and right rows of FC1 differ, two waves may add to one row in the same phase only if the rows of a path's two
  // sides are disjoint
  for (const Fc1Path &p : f1)
    if (p.r0 != p.f0 && p.r0 < p.f0 + p.M && p.f0 < p.r0 + p.M) { out.why = "fc1: left and right rows of a path overlap"; return false; }
  s << "  {\n";
  std::vector<char> keep0 = sp.keepX0;
  keep0.resize(nf0, 0);
  for (int f = 0; f < nf0; f++) {
    s << "    gX0[" << f << " * C] = LG[" << f * NA * S << " + col]";
    if (keep0[f] || !sp.fuse3) s << " + gX0[" << f << " * C]";
    s << ";\n";
  }
  s << "  }\n}\n";
  out.src = s.str();
  out.atoms_per_block = NA;
  {
    double nfun = 0.0;    // live output functions, each with a left and a right segment of C x C
    for (int f = 0; f < nf0; f++) nfun += sp.fc1.live[f] ? 1.0 : 0.0;
    for (int f = 0; f < nP2; f++) nfun += (live21[f] ? 1.0 : 0.0) + (live22[f] ? 1.0 : 0.0);
    out.flops_per_atom = nfun * 2.0 * 2.0 * C * C;
  }
  return true;
}

// Generates, compiles and loads the two kernels.  false (with the reason) when the model is outside what the generator
// covers or hiprtc is unavailable; GRACE_HIP_CHAIN=0 switches the fused chain off.
inline bool jit_compile_chain(const char *name, const ChainSpec &sp, const std::string &arch, ChainKernels &k, std::vector<double> &weights,
                              std::string &why)
{
  const char *sw = std::getenv("GRACE_HIP_CHAIN");
  if (sw && sw[0] == '0') {
    why = "switched off by GRACE_HIP_CHAIN=0";
    return false;
  }
  ChainCode code;
  if (!generate_chain(sp, code)) {
    why = code.why;
    return false;
  }
  JitKernels jk;
  if (!jit_compile_source(name, code.src, sp.f32, arch, jk, why, false, "chain_fwd", "chain_bwd")) return false;
  k.mod = jk.mod;
  k.fwd = jk.fwd;
  k.bwd = jk.bwd;
  k.atoms_per_block = code.atoms_per_block;
  k.flops_per_atom = code.flops_per_atom;
  weights = std::move(code.weights);
  return true;
}

}    // namespace grhip
