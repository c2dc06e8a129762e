// GRACE-3L engine for gfx950: three message-passing layers on one GPU, whole structure resident.
// Dataflow after libgrace/src/fused_3l.cpp:1550-1637 of the reference (layer 1, 2, 3 forward with the normalised
// messages I1, I2 of every atom kept; readout; layer 3, 2, 1 reverse with dE/dI_j added to the neighbours), without
// the recompute of layers 1-2: the forward tensors the reverse reads stay in device memory.
//
// Per layer (names of libgrace/src/model_3l.cpp:28-36):
//   radial functions  R[e][l][n] = MLP([T_k(2x-1), emb_i, emb_j]) env(x) fac[mu_j][n]          k_radial, species form
//   SPBF              layer 1: X[lm][n] = sum_b Y_lm R_l                                       k_scatter_a*
//                     layers 2-3: P[li][ly][n] = sum_b Y_ly R_l(ly) M_j[li][n],               k_pair_fwd
//                     A = cg_W^T P (sparse), X = reduce(A)                                     k_lincomb, job GEMM
//   cp_l product q    Lp = U[g] XL, Rp = V[g] XR (job GEMMs), P = sum cg Lp Rp (product kernel), R_q = reduce(P) (job GEMM)
//   FCRight2Left      out[f] = nof[f] (left[f] + W[t] right[from])                             k_scale_rows + job GEMM
//   eq / rho          reduces of (X, R2, R3, R4); EquivariantRMSNorm -> message; rho -> readout kernel
// Every dense contraction over (source function, destination function, weight tile) connections is one list of tile
// GEMM jobs on the matrix cores (k_gemm_jobs), forward by destination and reverse by source.
#include "engine_common.hpp"
#include "kernels_3l.hpp"
#include "model_3l.hpp"

namespace grhip {

namespace {

inline int pad_width(int c) { return c <= 16 ? 16 : c <= 32 ? 32 : c <= 64 ? 64 : -1; }
constexpr size_t kCoupleLdsMax = 158 * 1024;    // projections of one atom staged in LDS by the couple kernels

// out[dst][k] (+)= dscale[dst] sum over connections (src, dst, tile) of sum_n W[tile][n][k] in[src][n]; reverse:
// gin[src][n] += sum over its connections of dscale[dst] sum_k W[tile][n][k] gout[dst][k]   (fused_3l_cpu.h:84-221)
template<class T> struct DevContract {
  struct Conn {
    int src, dst, tile;
  };
  DevBuf WF, WT;
  DevJobs<T> fwd, bwd;
  int nel = 1;                                  // weight sets: 1, or one per element (wget(el * nt + t, n, k))
  size_t wstride = 0, wtstride = 0;             // values of one weight set, forward / transposed
  int kin = 0, kout = 0, nsrc = 0, ndst = 0;    // padded widths, functions of the source and destination tensors
  bool all_dst = false, all_src = false;        // every destination / source function has a connection
  template<class WGet>
  void build(int nin, int nout, int nt, const std::vector<Conn> &conns, WGet wget, const std::vector<double> &dscale, int nsrc_, int ndst_,
             const int *drow, const std::string &what, int nel_ = 1)
  {
    nel = nel_;
    kin = pad_width(nin);
    kout = pad_width(nout);
    nsrc = nsrc_;
    ndst = ndst_;
    if (kin < 0 || kout < 0) throw Error("GRACE-3L: " + what + ": channel widths above 64 are not supported by the GPU kernels");
    std::vector<T> F, Ft;
    std::vector<double> M((size_t) nin * nout), Mt((size_t) nout * nin);
    for (int t = 0; t < nel * nt; t++) {
      if (t == nt) { wstride = F.size(); wtstride = Ft.size(); }
      for (int n = 0; n < nin; n++)
        for (int k = 0; k < nout; k++) {
          const double v = wget(t, n, k);
          M[(size_t) n * nout + k] = v;
          Mt[(size_t) k * nin + n] = v;
        }
      pack_fragments<T>(M, nin, nout, kin, kout, F);
      pack_fragments<T>(Mt, nout, nin, kout, kin, Ft);
    }
    upload_vec(WF, F);
    upload_vec(WT, Ft);
    std::vector<std::vector<int>> by_dst(ndst), by_src(nsrc);
    for (size_t c = 0; c < conns.size(); c++) {
      if (conns[c].src < 0 || conns[c].src >= nsrc || conns[c].dst < 0 || conns[c].dst >= ndst || conns[c].tile < 0 || conns[c].tile >= nt)
        throw Error("GRACE-3L: " + what + ": connection index out of range");
      by_dst[conns[c].dst].push_back((int) c);
      by_src[conns[c].src].push_back((int) c);
    }
    all_dst = all_src = true;
    for (const auto &v : by_dst) all_dst = all_dst && !v.empty();
    for (const auto &v : by_src) all_src = all_src && !v.empty();
    auto sc = [&](int d) { return dscale.empty() ? 1.0 : dscale[d]; };
    typename DevJobs<T>::Host hf, hb;
    for (int d = 0; d < ndst; d++) {
      if (by_dst[d].empty()) continue;
      hf.job(d, sc(d));
      for (int c : by_dst[d]) hf.seg(0, conns[c].src, conns[c].tile, 1.0);
      hf.end_job();
    }
    for (int s = 0; s < nsrc; s++) {
      if (by_src[s].empty()) continue;
      hb.job(s, 1.0);
      for (int c : by_src[s]) hb.seg(0, conns[c].dst, conns[c].tile, sc(conns[c].dst));
      hb.end_job();
    }
    fwd.build(hf, WF.as<T>(), WF.as<T>());
    bwd.build(hb, WT.as<T>(), WT.as<T>());
    fwd.set_rows(drow);
    bwd.set_rows(drow);
  }
};

// sparse matrix in CSR form on the device (k_lincomb)
struct DevCsr {
  DevBuf off, idx, rowof, val;
  int nrow = 0, ncol = 0, rows = 8;    // rows: output rows per wave
  void build(int nrow_, int ncol_, const std::vector<int> &row, const std::vector<int> &col, const std::vector<double> &v)
  {
    nrow = nrow_;
    ncol = ncol_;
    rows = lincomb_rows((int) row.size(), nrow_);
    std::vector<int> o(nrow + 1, 0), ix(row.size()), rw(row.size());
    std::vector<double> vv(row.size());
    for (int r : row) o[r + 1]++;
    for (int r = 0; r < nrow; r++) o[r + 1] += o[r];
    std::vector<int> pos(o.begin(), o.end() - 1);
    for (size_t t = 0; t < row.size(); t++) {
      const int q = pos[row[t]]++;
      ix[q] = col[t];
      rw[q] = row[t];
      vv[q] = v[t];
    }
    if (ix.empty()) { ix.push_back(0); rw.push_back(0); vv.push_back(0.0); }
    upload_vec(off, o);
    upload_vec(idx, ix);
    upload_vec(rowof, rw);
    upload_vec(val, vv);
  }
};

// a per-atom tensor [atom][nf][w]
struct Ten {
  DevBuf buf;
  int nf = 0, w = 0;
  size_t bytes(size_t na, size_t s) const { return na * nf * w * s; }
};

template<class T> struct ProdStage {
  DevContract<T> U, V, red;
  DevProd cp;
  DevBuf tl, tr, to, tc;    // the terms sorted by output, for the LDS couple kernels
  CoupleDev cd{};
  int nfunc = 0, rankP = 0;
  bool jit = false;
  bool jit_sets = false;    // the specialised reverse kernel writes every row of both adjoints: nothing to clear before it
};

template<class T> struct FcStage {
  DevContract<T> right;
  DevBuf nof;
  int nf = 0;
};

template<class T> struct Layer3 {
  bool equiv = false, has_eq = false;
  int C = 0, CP = 0;                  // radial channels and their padded width
  DevRadial<T> rad;
  DevBuf fac;
  // equivariant SPBF
  int nlmi = 0, nfA = 0;
  DevBuf zproj, mask;
  DevCsr cg, cgt;                     // A = cg P (rows: A functions), gP = cgt gA (rows: pair functions slot * nlm + lm)
  DevContract<T> redA;
  ProdStage<T> p2, p3, p4;
  FcStage<T> fa, fb;
  std::vector<std::unique_ptr<DevContract<T>>> eq;    // sources X, R2, R3, R4
  DevBuf eq_dw, eq_mask, eq_aff, eq_grp;
  EqNormDev eqn{};
  DevReduce<T> rho;
  // forward tensors kept for the reverse
  DevBuf R, dR;
  Ten X, L2, R2p, L3, R3p, L4, R4p, EQ, I;
  DevBuf rho_raw, grho;
  int nR2 = 0, nR3 = 0, nR4 = 0, wR = 0;    // functions of the product reduces, their common padded width
  // UQ head: the rows of this layer's basis block (inputs of the rho reduce in the model's instruction order)
  UqDev<T> uq{};
  int uqSlot[4] = {0, 0, 0, 0};             // tensor of each instruction: 0 X, 1 R2, 2 R3, 3 R4
  DevBuf uqCi[4];
};

template<class T> class Engine3L final : public EngineBase {
 public:
  Engine3L(std::shared_ptr<const Model3L> m, int ntypes, const std::vector<int> &type2mu, int device) :
      EngineBase(device, "GRACE-3L", ntypes, type2mu, m->n_elements), model_(std::move(m))
  {
    this->template probe_mfma_both<T>();
    build();
    end_build();    // buffers allocated from here on are work buffers (release_buffers)
    chunks_ = true;
    ordered_ok_ = true;
  }
  int layers() const override { return 3; }
  // radial tables per ordered pair of species and per layer: n / 2 intervals for layers 1 and 2 (at least 16), n for layer 3
  // (spline_n_3l, libgrace/include/grace/system.h:95-103); tables that would exceed the memory they may take are not built
  // and the MLPs stay (the reference's spline_mb, libgrace/src/fused_3l.cpp:405-418)
  void apply_spline(int n) override
  {
    double total = 0.0;
    for (int k = 0; k < 3; k++) {
      L_[k].rad.spline_n = n > 0 ? (k < 2 ? std::max(16, n / 2) : n) : 0;
      total += L_[k].rad.table_bytes(L_[k].rad.spline_n);
    }
    // the three layers' tables together against the limit (2048 MB as Grace3LKK::spline_mb, libgrace/include/grace/kk/
    // grace_3l_kk.h:1264; GRACE_HIP_TABLE_MB sets another)
    double limit_mb = 2048.0;
    if (const char *e = std::getenv("GRACE_HIP_TABLE_MB")) limit_mb = std::atof(e);
    const bool fits = total <= limit_mb * 1048576.0;
    for (int k = 0; k < 3; k++) L_[k].rad.tables_allowed = fits;
    if (n > 0 && !fits)
      log_message(0, who_ + ": the radial MLPs are evaluated for every bond: tables for " + std::to_string(L_[0].rad.species_mu.size() *
                         L_[0].rad.species_mu.size()) + " species pairs would need " + std::to_string((long long) (total / 1048576.0)) +
                         " MB > " + std::to_string((long long) limit_mb) + " MB");
  }
  void run(const RunFlags &fl) override;
  void debug_radial(int, const double *, const int *, double *, double *) override
  {
    throw Error("GRACE-3L: debug_radial is available for GRACE-1L engines");
  }
  // two messages: the normalised equivariant outputs of layers 1 and 2 (libgrace/include/grace/kk/grace_3l_kk.h:313-324)
  int comm_layers() const override { return 2; }
  int comm_width(int layer) const override { return layer == 1 || layer == 2 ? L_[layer].nlmi * L_[layer].C : 0; }
  void comm_rows(int mode, int layer, int n, const int *list, int first, double *buf, bool host) override
  {
    if (layer != 1 && layer != 2) throw InvalidArgument("GRACE-3L exchanges the messages of layers 1 and 2");
    const Layer3<T> &L = L_[layer];    // the layer that gathers the message
    if (mode < 2) {
      move_rows<T>(mode, L_[layer - 1].I.buf.template as<T>(), (long long) L.nlmi * L.CP, L.nlmi, L.C, L.CP, n, list, first, buf, host);
    } else {
      // the adjoint rows live in scratch shared by the layers: they are this layer's only inside its reverse exchange
      if (comm_reverse_layer_ != layer) throw Error("GRACE-3L: the adjoint rows of a message exist only inside its reverse exchange");
      move_rows<T>(mode, gM_.as<T>(), (long long) L.nlmi * L.CP, L.nlmi, L.C, L.CP, n, list, first, buf, host);
    }
  }

 private:
  std::shared_ptr<const Model3L> model_;
  int lmax_ = 0, nl_ = 0, nlm_ = 0, nel_ = 0, nrho_ = 0;
  ShCoef sh_{};
  Layer3<T> L_[3];
  DevBuf shift_, eW0_, eW1_, escale_[3], sink_, emi_, YG_;
  Energy3Dev en_{};
  DevBuf uqR_, uqCen_, uqIcov_, uqNcl_, uqThr_, uqZ_, uqN2_;    // UQ head arrays; raw projection and block norms carried over the layers
  bool uq_on_ = false;
  int comm_reverse_layer_ = 0;    // the message whose adjoint rows gM_ holds while its reverse exchange runs
  // scratch shared by the layers (largest size over the layers): temporaries of the forward pass and all adjoints
  DevBuf M_, gM_, pairP_, gpairP_, A_, gA_, P_, gP_, R2_, R3_, R4_, FA_, FB_, gX_, gR2_, gR3_, gR4_, gFA_, gFB_, gLp_, gRp_, gEQ_;
  // ordered sums: the message adjoints of a chunk's bonds [bond][nlmi][CP]; the forces and per-atom sums of the slot groups
  // of a pair kernel, [bond][group][3] and [atom][group][9]; ordered_first_: no layer of this pass has stored its bond forces yet
  DevBuf gMe_, fpart_, cpart_;
  bool ordered_first_ = true;
  DevBuf gMin_;    // adjoint of the message the layer in reverse SENT (filled by the layer above); gM_: of the one it gathers
  // the chunk of atoms the layer functions act on: atoms [a0_, a0_ + cn_), their bonds [eb_, eb_ + ecnt_) (ecnt_ < 0: all
  // bonds), the capacities the chunk buffers are sized for, the chunk's element tiles (atoms counted from a0_)
  int cn_ = 0, a0_ = 0;
  size_t cap_ = 0, ecap_ = 1;
  long long eb_ = 0, ecnt_ = -1;
  const int *cur_tiles_ = nullptr, *cur_tile_el_ = nullptr;
  int cur_ntiles_ = 0;

  void build();
  void build_layer(int k);
  void gemm(DevJobs<T> &J, int kin, int kout, const T *X, int nfx, T *out, int nfo, int accumulate)
  {
    EngineBase::launch_gemm<T>(J, kin / 16, kin / 16, kout / 16, X, nfx, X, nfx, out, nfo, accumulate, cur_tiles_, cur_ntiles_);
  }
  // element-dependent weights: one launch per element over its tiles (tiles hold atoms of one element, elements in order)
  void gemm_el(DevJobs<T> &J, size_t wstride, int nel, int kin, int kout, const T *X, int nfx, T *out, int nfo, int accumulate)
  {
    if (nel == 1) return gemm(J, kin, kout, X, nfx, out, nfo, accumulate);
    const T *w0 = J.d.WF0, *w1 = J.d.WF1;
    for (int e = 0; e < nel; e++) {
      const int t0 = cur_tile_el_[e], nt = cur_tile_el_[e + 1] - t0;
      if (nt == 0) continue;
      J.d.WF0 = w0 + e * wstride;
      J.d.WF1 = w1 + e * wstride;
      EngineBase::launch_gemm<T>(J, kin / 16, kin / 16, kout / 16, X, nfx, X, nfx, out, nfo, accumulate, cur_tiles_ + (size_t) 16 * t0, nt);
    }
    J.d.WF0 = w0;
    J.d.WF1 = w1;
  }
  void cfwd(DevContract<T> &c, const T *X, T *out, int accumulate) { gemm_el(c.fwd, c.wstride, c.nel, c.kin, c.kout, X, c.nsrc, out, c.ndst, accumulate); }
  void cbwd(DevContract<T> &c, const T *gout, T *gX, int accumulate) { gemm_el(c.bwd, c.wtstride, c.nel, c.kout, c.kin, gout, c.ndst, gX, c.nsrc, accumulate); }
  void zero(void *p, size_t bytes) { if (bytes) HIP_CHECK(hipMemsetAsync(p, 0, bytes, stream_)); }
  // out = contraction (not accumulated): functions without a connection are cleared
  void cfwd_set(DevContract<T> &c, const T *X, T *out)
  {
    if (!c.all_dst) zero(out, (size_t) cn_ * c.ndst * c.kout * sizeof(T));
    cfwd(c, X, out, c.all_dst ? 0 : 1);
  }
  void cbwd_set(DevContract<T> &c, const T *gout, T *gX)
  {
    if (!c.all_src) zero(gX, (size_t) cn_ * c.nsrc * c.kin * sizeof(T));
    cbwd(c, gout, gX, c.all_src ? 0 : 1);
  }
  void couple_fwd(ProdStage<T> &p, const T *Lp, int nfl, const T *Rp, int nfr, T *out);
  void couple_bwd(ProdStage<T> &p, const T *Lp, int nfl, const T *Rp, int nfr, const T *g, T *gL, T *gR);
  void scale_rows(const T *in, const DevBuf &s, T *out, int nf, int w, int accumulate)
  {
    const long long tot = (long long) cn_ * nf * w;
    if (tot == 0) return;
    hipLaunchKernelGGL(k_scale_rows<T>, dim3((unsigned) ((tot + 255) / 256)), dim3(256), 0, stream_, in, s.as<T>(), out, cn_, nf, w, accumulate);
  }
  void layer_messages(int k);
  void layer_forward(int k, bool forces, int yw, bool again);
  void layer_backward(int k, int yw);
  double chunk_bytes_per_atom() const;
  std::string tg(int k, const char *name) { return std::string(name) + "_L" + std::to_string(k + 1); }
};

template<class T> void Engine3L<T>::build()
{
  const Model3L &m = *model_;
  lmax_ = m.lmax;
  if (lmax_ > kKernMaxL) throw Error("GRACE-3L: lmax > " + std::to_string(kKernMaxL) + " not supported");
  nl_ = lmax_ + 1;
  nlm_ = nl_ * nl_;
  nel_ = m.n_elements;
  nrho_ = m.rho_width;
  std::memset(&sh_, 0, sizeof(sh_));
  sh_.lmax = lmax_;
  for (int l = 2; l <= lmax_; l++) {
    for (int mm = 0; mm < l - 1; mm++) {
      const double l2 = l * l, m2 = mm * mm, lm1 = l - 1;
      sh_.a[l * (l + 1) / 2 + mm] = std::sqrt((4.0 * l2 - 1.0) / (l2 - m2));
      sh_.b[l * (l + 1) / 2 + mm] = -std::sqrt((lm1 * lm1 - m2) / (4.0 * lm1 * lm1 - 1.0));
    }
    sh_.c[l] = -std::sqrt(1.0 + 0.5 / l);
    sh_.d[l] = std::sqrt(2.0 * l + 1.0);
  }
  {
    std::vector<double> cut((size_t) nel_ * nel_);
    for (int a = 0; a < nel_; a++)
      for (int b = 0; b < nel_; b++) cut[(size_t) a * nel_ + b] = m.pair_cutoff(a, b);
    set_cutoffs(cut);
  }
  upload_vec(shift_, m.shift_values);
  sink_.ensure(64);
  for (int k = 0; k < 3; k++) build_layer(k);
  // ---- UQ head (libgrace/src/fused_3l.cpp:845-866): basis = inputs of the rho1 | rho2 | rho3 reduces, one block per layer
  if (m.uq.has_uq) {
    try {
      if (m.uq.rp_dim > 256 || m.uq.feature_dim > 256) throw Error("GRACE-3L UQ: feature widths above 256 are not supported");
      upload_vec(uqR_, m.uq.rp_matrix); upload_vec(uqCen_, m.uq.centroids); upload_vec(uqIcov_, m.uq.inv_cov);
      upload_vec(uqNcl_, m.uq.n_clusters); upload_vec(uqThr_, m.uq.interp_thresholds);
      int off = 0;
      for (int k = 0; k < 3; k++) {
        Layer3<T> &L = L_[k];
        const std::string K = "A" + std::to_string(k + 1);
        const std::string names[4] = {L.equiv ? K + "_red" : K, K + "_2_red", K + "_3_red", K + "_4_red"};
        const int nf[4] = {L.X.nf, L.nR2, L.nR3, L.nR4};
        const Model3L::Reduce &r = Model3L::by_name(m.reduce, "rho" + std::to_string(k + 1));
        if (r.instr.size() != 4) throw Error("GRACE-3L UQ: rho" + std::to_string(k + 1) + " does not have four inputs");
        UqDev<T> &u = L.uq;
        u = UqDev<T>{};
        int loc = 0;
        for (int q = 0; q < 4; q++) {
          const Model3L::Instr &ins = r.instr[q];
          int slot = -1;
          for (int s = 0; s < 4; s++)
            if (ins.name == names[s]) slot = s;
          if (slot < 0) throw Error("GRACE-3L UQ: rho input " + ins.name + " is not a tensor of the layer");
          for (int c : ins.collect_ind)
            if (c < 0 || c >= nf[slot]) throw Error("GRACE-3L UQ: rho input " + ins.name + " collects a function it does not have");
          L.uqSlot[q] = slot;
          upload_vec(L.uqCi[q], ins.collect_ind);
          u.ci[q] = L.uqCi[q].template as<int>();
          u.nfun[q] = nf[slot];
          u.cpad[q] = slot == 0 ? L.X.w : L.wR;
          u.nin[q] = ins.n_in;
          u.nc[q] = (int) ins.collect_ind.size();
          u.off[q] = loc;
          u.blk[q] = k;
          if (u.nin[q] > u.cpad[q]) throw Error("GRACE-3L UQ: rho input " + ins.name + " is wider than its tensor");
          loc += u.nin[q] * u.nc[q];
        }
        u.nsrc = 4; u.nblk = 3; u.row0 = off; u.d_basis = loc;
        u.carry_in = k > 0 ? 1 : 0; u.carry_out = k < 2 ? 1 : 0;
        u.rp = m.uq.rp_dim; u.D = m.uq.feature_dim; u.K = m.uq.max_clusters;
        u.density_scale = m.uq.density_scale;
        u.R = uqR_.template as<double>(); u.cen = uqCen_.template as<double>(); u.icov = uqIcov_.template as<double>();
        u.ncl = uqNcl_.template as<int>(); u.thr = uqThr_.template as<double>();
        if ((size_t) (u.d_basis + 4 * u.rp + 2 * u.D) * sizeof(double) > 150 * 1024) throw Error("GRACE-3L UQ: the basis does not fit the kernel's LDS");
        off += loc;
      }
      if (off != m.uq.d_basis) throw Error("GRACE-3L UQ: basis width " + std::to_string(off) + " != uq_rp_matrix rows " + std::to_string(m.uq.d_basis));
      has_uq_head_ = true;
    } catch (const std::exception &e) {
      uq_why_ = e.what();
    }
  } else {
    uq_why_ = "the model file carries none";
  }
  for (int k = 0; k < 2; k++) {
    const Layer3<T> &a = L_[k], &b = L_[k + 1];
    if (a.I.nf != b.nlmi || a.eqn.Creal != b.C) throw Error("GRACE-3L: the message of layer " + std::to_string(k + 1) + " does not fit the next SPBF");
  }
  // ---- readout: 2-layer MLP on the summed normalised densities (fused_3l.cpp:833-843)
  const auto &e = m.energy_mlp.layers;
  if (e.size() != 2 || e[0].n_in != nrho_ - 1 || e[1].n_out != 1)
    throw Error("GRACE-3L: the GPU readout implements a 2-layer energy MLP on rho[1:]");
  for (const auto &b : m.energy_mlp.bias)
    if (!b.empty()) throw Error("GRACE-3L: a bias in the energy MLP is not supported");
  if (nrho_ > 256 || e[0].n_out > 1024) throw Error("GRACE-3L: energy MLP too wide for the readout kernel");
  upload_vec(eW0_, e[0].W);
  upload_vec(eW1_, e[1].W);
  en_.W0 = eW0_.as<double>();
  en_.W1 = eW1_.as<double>();
  en_.norm0 = e[0].norm;
  en_.norm1 = e[1].norm;
  en_.nin = e[0].n_in;
  en_.nh = e[0].n_out;
  en_.act = m.energy_mlp_activation;
  en_.nrho = nrho_;
  en_.out_scale = m.output_scale;
  en_.eps = Model3L::rms_norm_eps;
  en_.shift = shift_.as<double>();
  for (int k = 0; k < 3; k++) {
    const auto &r = Model3L::by_name(m.rmsnorm, "rho" + std::to_string(k + 1) + "_norm");
    upload_vec(escale_[k], r.scale);
    en_.scale[k] = escale_[k].as<double>();
    en_.type[k] = r.type;
  }
}

template<class T> void Engine3L<T>::build_layer(int k)
{
  const Model3L &m = *model_;
  Layer3<T> &L = L_[k];
  const std::string ks = std::to_string(k + 1), K = "A" + ks;
  const Model3L::Spbf &sp = Model3L::by_name(m.spbf, K);
  L.equiv = sp.equivariant;
  L.C = sp.n_rad_max;
  L.CP = pad_width(L.C);
  if (L.CP < 0) throw Error("GRACE-3L: more than 64 radial channels are not supported by the GPU kernels");
  for (int lm = 0; lm < nlm_; lm++) {
    int l = 0;
    while ((l + 1) * (l + 1) <= lm) l++;
    if (sp.l_tile[lm] != l) throw Error("GRACE-3L: " + K + "_l_tile is not the l of each (l, m) function; not supported by the GPU kernels");
  }
  // ---- radial MLP; fac[mu_j][n] = inv_avg (z_tr[mu_j][n] in layer 1): fused_3l.cpp:441-460
  const int ne = m.embedding_size;
  L.rad.build_species(sp.mlp.layers, sp.mlp.bias, m.chem_embedding, ne, m.nradbase, sp.p, L.C, L.CP, nl_, nel_, drow_, "GRACE-3L");
  L.rad.build_species_double(sp.mlp.layers, sp.mlp.bias, m.chem_embedding, ne, m.nradbase, sp.p, L.C, L.CP, nl_, nel_, drow64_, "GRACE-3L");
  {
    // the species of this engine: the elements its atom types map to (tables per ordered pair of them, fused_3l.cpp:381-398)
    std::vector<int> present;
    for (int t = 1; t <= ntypes_; t++) {
      const int mu = type2mu_[(size_t) t];
      if (mu >= 0 && std::find(present.begin(), present.end(), mu) == present.end()) present.push_back(mu);
    }
    L.rad.set_species(present, nel_, "GRACE-3L layer " + std::to_string(k + 1));
  }
  auto species_table = [&](const std::vector<double> &W, double norm) {
    std::vector<double> z((size_t) nel_ * L.C);
    for (int mu = 0; mu < nel_; mu++)
      for (int n = 0; n < L.C; n++) {
        double v = 0.0;
        for (int e = 0; e < ne; e++) v += m.chem_embedding[(size_t) mu * ne + e] * W[(size_t) e * L.C + n];
        z[(size_t) mu * L.C + n] = v * norm;
      }
    return z;
  };
  {
    std::vector<T> fac((size_t) nel_ * L.CP, (T) 0);
    std::vector<double> ztr;
    if (!L.equiv) ztr = species_table(sp.lin_transform_W, sp.lin_transform_norm);
    for (int mu = 0; mu < nel_; mu++)
      for (int n = 0; n < L.C; n++) fac[(size_t) mu * L.CP + n] = (T) (sp.inv_avg_n_neigh * (L.equiv ? 1.0 : ztr[(size_t) mu * L.C + n]));
    upload_vec(L.fac, fac);
  }
  typedef typename DevContract<T>::Conn Conn;
  // a reduce instruction as a contraction; W: [n_elements |] [n_out][n_in][w_shape]
  auto instr_contract = [&](DevContract<T> &c, const Model3L::Reduce &r, const Model3L::Instr &ins, int nsrc, const std::string &what) {
    std::vector<Conn> conns;
    for (size_t q = 0; q < ins.collect_ind.size(); q++) conns.push_back({ins.collect_ind[q], r.only_invar ? 0 : ins.total_sum_ind[q], ins.w_l_tile[q]});
    const size_t per = (size_t) r.n_out * ins.n_in * ins.w_shape;
    c.build(ins.n_in, r.n_out, ins.w_shape, conns,
            [&](int t, int n, int kk) {
              const int el = t / ins.w_shape, tt = t % ins.w_shape;
              return ins.norm * ins.W[el * per + ((size_t) kk * ins.n_in + n) * ins.w_shape + tt];
            },
            r.norm_map, nsrc, r.nfo(), drow_, what, r.elem_dep ? nel_ : 1);
  };
  L.X.nf = nlm_;
  if (L.equiv) {
    L.nlmi = sp.n_lm_ind;
    L.nfA = sp.nfunc;
    {
      const std::vector<double> zp = species_table(sp.chem_linear_W, sp.chem_linear_norm);
      std::vector<T> z((size_t) nel_ * L.CP, (T) 0), mk(sp.chem_l0_mask.begin(), sp.chem_l0_mask.end());
      for (int mu = 0; mu < nel_; mu++)
        for (int n = 0; n < L.C; n++) z[(size_t) mu * L.CP + n] = (T) zp[(size_t) mu * L.C + n];
      upload_vec(L.zproj, z);
      upload_vec(L.mask, mk);
    }
    // cg_W rows p = ly * nlmi + li (fused_3l.cpp:523-549); the pair tensor of k_pair_fwd has functions li * nlm + ly
    std::vector<int> rf, cf;
    std::vector<double> vv;
    const int np = nlm_ * L.nlmi;
    for (int p = 0; p < np; p++)
      for (int f = 0; f < L.nfA; f++) {
        const double v = sp.cg_W[(size_t) p * L.nfA + f];
        if (v == 0.0) continue;
        const int ly = p / L.nlmi, li = p % L.nlmi;
        rf.push_back(f);
        cf.push_back(li * nlm_ + ly);
        vv.push_back(v);
      }
    L.cg.build(L.nfA, np, rf, cf, vv);
    L.cgt.build(np, L.nfA, cf, rf, vv);
    const Model3L::Reduce &r = Model3L::by_name(m.reduce, K + "_red");
    if (r.instr.size() != 1 || r.only_invar) throw Error("GRACE-3L: " + K + "_red must be one instruction on " + K);
    instr_contract(L.redA, r, r.instr[0], L.nfA, K + "_red");
    L.X.nf = r.nfo();
    L.X.w = L.redA.kout;
  } else
    L.X.w = L.CP;
  const int nX = L.X.nf;
  // ---- cp_l products with their reduces
  auto build_prod = [&](ProdStage<T> &P, const std::string &q, int nfl, int wl, int nfr, int wr, Ten &Lp, Ten &Rp, int &nfred) {
    const Model3L::Cpl &c = Model3L::by_name(m.prod, K + "_" + q);
    const Model3L::Reduce &r = Model3L::by_name(m.reduce, K + "_" + q + "_red");
    if (r.instr.size() != 1 || r.only_invar) throw Error("GRACE-3L: " + r.name + " must be one instruction on the product");
    if (pad_width(c.n_left) != wl || pad_width(c.n_right) != wr) throw Error("GRACE-3L: " + c.name + ": input widths");
    std::vector<Conn> cl, cr;
    for (int f = 0; f < nfl; f++) cl.push_back({f, f, c.group_left[f]});
    for (int f = 0; f < nfr; f++) cr.push_back({f, f, c.group_right[f]});
    P.U.build(c.n_left, c.rank, c.n_groups_left, cl, [&](int t, int n, int kk) { return c.norm_u * c.U[((size_t) t * c.rank + kk) * c.n_left + n]; }, {}, nfl,
              nfl, drow_, c.name + "_U");
    P.V.build(c.n_right, c.rank, c.n_groups_right, cr, [&](int t, int n, int kk) { return c.norm_v * c.V[((size_t) t * c.rank + kk) * c.n_right + n]; }, {},
              nfr, nfr, drow_, c.name + "_V");
    P.nfunc = c.nfunc;
    P.rankP = P.U.kout;
    const HostProd h = grhip::build_prod(c.cg, std::vector<char>(c.nfunc, 1), nfl, nfr);
    P.cp.build(h);
    // The shorter term lists run with the operands of both sides in registers (that generator writes only outputs with
    // terms, so it needs a list that feeds every output), the longer ones block by block.
    bool every_output = true;
    {
      std::vector<char> fed(c.nfunc, 0);
      for (const ProdTerm &t : h.terms) fed[t.o] = 1;
      for (char x : fed) every_output = every_output && x;
    }
    if (h.terms.size() <= 1500 && every_output)
      jit_compile_product((c.name + "_cp").c_str(), h.terms, nfl, nfr, c.nfunc, false, P.rankP, sizeof(T) == 4, arch_, P.cp.jit, P.cp.jit_note);
    else
      P.jit_sets = jit_compile_blocked((c.name + "_cp").c_str(), h.terms, c.group_left, c.group_right, nfl, nfr, c.nfunc, P.rankP, sizeof(T) == 4,
                                       arch_, P.cp.jit, P.cp.jit_note);
    P.jit = P.cp.jit.ok();
    {
      std::vector<int> tl, tr, to;
      std::vector<double> tc;
      for (const ProdTerm &t : h.terms) { tl.push_back(t.l); tr.push_back(t.r); to.push_back(t.o); tc.push_back(t.c); }
      if (tl.empty()) { tl.push_back(0); tr.push_back(0); to.push_back(0); tc.push_back(0.0); }
      upload_vec(P.tl, tl); upload_vec(P.tr, tr); upload_vec(P.to, to); upload_vec(P.tc, tc);
      P.cd.l = P.tl.template as<int>(); P.cd.r = P.tr.template as<int>(); P.cd.o = P.to.template as<int>(); P.cd.c = P.tc.template as<double>();
      P.cd.off = P.cp.off.template as<int>();
      P.cd.nout = c.nfunc;
      P.cd.nterms = (int) h.terms.size();
    }
    instr_contract(P.red, r, r.instr[0], c.nfunc, r.name);
    Lp.nf = nfl;
    Rp.nf = nfr;
    Lp.w = Rp.w = P.rankP;
    nfred = r.nfo();
    if (L.wR == 0) L.wR = P.red.kout;
    if (P.red.kout != L.wR) throw Error("GRACE-3L: the product reduces of a layer must have one channel width");
  };
  auto build_fc = [&](FcStage<T> &F, const std::string &name) {
    const Model3L::Fc &f = Model3L::by_name(m.fc, name);
    if (f.n_funcs_left != L.nR2 || pad_width(f.n_out) != L.wR || pad_width(f.n_in_right) != L.X.w) throw Error("GRACE-3L: FC " + name + ": shapes");
    std::vector<Conn> conns;
    for (size_t q = 0; q < f.collect_from.size(); q++) conns.push_back({f.collect_from[q], f.collect_to[q], f.w_tile_right[q]});
    F.right.build(f.n_in_right, f.n_out, f.w_shape_right, conns,
                  [&](int t, int n, int kk) { return f.norm_right * f.w_right[((size_t) kk * f.n_in_right + n) * f.w_shape_right + t]; }, f.norm_out_factor,
                  nX, f.n_funcs_left, drow_, "fc_" + name);
    F.nf = f.n_funcs_left;
    upload_vec(F.nof, std::vector<T>(f.norm_out_factor.begin(), f.norm_out_factor.end()));
  };
  build_prod(L.p2, "2", nX, L.X.w, nX, L.X.w, L.L2, L.R2p, L.nR2);
  build_fc(L.fa, K + "_2a");
  build_prod(L.p3, "3", L.nR2, L.wR, nX, L.X.w, L.L3, L.R3p, L.nR3);
  build_fc(L.fb, K + "_2b");
  build_prod(L.p4, "4", L.nR2, L.wR, L.nR2, L.wR, L.L4, L.R4p, L.nR4);
  // ---- eq (layers 1-2) and rho reduces of (X, R2, R3, R4)
  const std::string xname = L.equiv ? K + "_red" : K;
  const std::string srcs[4] = {xname, K + "_2_red", K + "_3_red", K + "_4_red"};
  const int src_nf[4] = {nX, L.nR2, L.nR3, L.nR4};
  L.has_eq = k < 2;
  if (L.has_eq) {
    const Model3L::Reduce &r = Model3L::by_name(m.reduce, "eq" + ks);
    if (r.only_invar) throw Error("GRACE-3L: eq" + ks + " is marked invariant");
    for (int s = 0; s < 4; s++) {
      L.eq.emplace_back(new DevContract<T>());
      instr_contract(*L.eq.back(), r, Model3L::by_name(r.instr, srcs[s]), src_nf[s], "eq" + ks);
    }
    const Model3L::EqNorm &e = Model3L::by_name(m.eqnorm, "eq" + ks + "_norm");
    L.EQ.nf = L.I.nf = e.M;
    L.EQ.w = L.I.w = L.eq[0]->kout;
    upload_vec(L.eq_dw, e.degree_weights);
    upload_vec(L.eq_mask, e.l0_mask);
    upload_vec(L.eq_grp, e.expand_index);
    std::vector<double> aff((size_t) e.n_groups * L.EQ.w, 0.0);
    for (int g = 0; g < e.n_groups; g++)
      for (int n = 0; n < e.n_out; n++) aff[(size_t) g * L.EQ.w + n] = e.affine_weight[(size_t) g * e.n_out + n];
    upload_vec(L.eq_aff, aff);
    L.eqn.dw = L.eq_dw.template as<double>();
    L.eqn.mask = L.eq_mask.template as<double>();
    L.eqn.aff = L.eq_aff.template as<double>();
    L.eqn.grp = L.eq_grp.template as<int>();
    L.eqn.M = e.M;
    L.eqn.C = L.EQ.w;
    L.eqn.Creal = e.n_out;
    L.eqn.center = e.center_l0 ? 1 : 0;
    L.eqn.eps = e.eps;
  }
  {
    const Model3L::Reduce &r = Model3L::by_name(m.reduce, "rho" + ks);
    if (!r.only_invar) throw Error("GRACE-3L: rho" + ks + " must be an invariant reduce");
    if (r.n_out != nrho_) throw Error("GRACE-3L: rho widths differ between the layers");
    // element-independent weights are replicated per element for the reduce kernel
    std::vector<std::vector<double>> Wrep(4);
    std::vector<ReduceSrc> v;
    for (int s = 0; s < 4; s++) {
      const Model3L::Instr &ins = Model3L::by_name(r.instr, srcs[s]);
      const std::vector<double> *W = &ins.W;
      if (!r.elem_dep) {
        for (int mu = 0; mu < nel_; mu++) Wrep[s].insert(Wrep[s].end(), ins.W.begin(), ins.W.end());
        W = &Wrep[s];
      }
      v.push_back({W, ins.norm, ins.n_in, ins.w_shape, &ins.collect_ind, &ins.w_l_tile, nullptr, src_nf[s], s == 0 ? L.X.w : L.wR});
    }
    L.rho.build(v, nel_, nrho_, -1, nrho_, 0, drow_);
  }
}

template<class T> void Engine3L<T>::couple_fwd(ProdStage<T> &p, const T *Lp, int nfl, const T *Rp, int nfr, T *out)
{
  const int n = cn_, KP = p.rankP;
  int one = 1, nat = n;
  if (p.jit) {
    void *args[] = {(void *) &Lp, (void *) &Rp, (void *) &out, (void *) &nat, (void *) &one};
    const long long cols = (long long) n * KP;
    HIP_CHECK(hipModuleLaunchKernel(p.cp.jit.fwd, (unsigned) ((cols + 255) / 256), 1, 1, 256, 1, 1, 0, stream_, args, nullptr));
    return;
  }
  const int ATl = 64 / KP;
  const size_t lds = (size_t) ATl * (nfl + nfr) * KP * sizeof(T);
  if (lds <= kCoupleLdsMax && p.cd.nterms > 0) {
    auto kern = k_couple_fwd_lds<T>;
    if (lds > 48 * 1024) HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds));
    hipLaunchKernelGGL(kern, dim3((n + ATl - 1) / ATl), dim3(p.cd.nout >= 256 ? 1024 : 256), lds, stream_, p.cd, Lp, Rp, out, KP, nfl, nfr, n);
    return;
  }
  const int AT = std::max(1, 256 / KP);
  hipLaunchKernelGGL(k_prod_fwd<T>, dim3(p.cp.d.nout * 8 * (((n + AT - 1) / AT + 7) / 8)), dim3(KP * AT), 0, stream_, p.cp.d, Lp, Rp, out, n, KP, nfl, nfr);
}

// gL, gR are accumulated into (zeroed by the caller), or set when the stage says jit_sets
template<class T> void Engine3L<T>::couple_bwd(ProdStage<T> &p, const T *Lp, int nfl, const T *Rp, int nfr, const T *g, T *gL, T *gR)
{
  const int n = cn_, KP = p.rankP;
  int one = 1, nat = n, acc = p.jit_sets ? 0 : 1;
  if (p.jit) {
    void *args[] = {(void *) &Lp, (void *) &Rp, (void *) &g, (void *) &gL, (void *) &gR, (void *) &acc, (void *) &acc, (void *) &nat, (void *) &one};
    const long long cols = (long long) n * KP;
    HIP_CHECK(hipModuleLaunchKernel(p.cp.jit.bwd, (unsigned) ((cols + 255) / 256), 1, 1, 256, 1, 1, 0, stream_, args, nullptr));
    return;
  }
  const int ATl = 64 / KP;
  const size_t lds = (size_t) ATl * (nfl + nfr) * KP * (sizeof(T) + sizeof(double));
  if (!ordered_ && lds <= kCoupleLdsMax && p.cd.nterms > 0) {    // ordered sums: the gather form below has no atomics
    auto kern = k_couple_bwd_lds<T>;
    if (lds > 48 * 1024) HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds));
    hipLaunchKernelGGL(kern, dim3((n + ATl - 1) / ATl), dim3(p.cd.nout >= 256 ? 1024 : 256), lds, stream_, p.cd, Lp, Rp, g, gL, gR, KP, nfl, nfr, n);
    return;
  }
  const int AT = std::max(1, 256 / KP);
  hipLaunchKernelGGL(k_prod_bwd<T>, dim3(p.cp.d.nleft * 8 * (((n + AT - 1) / AT + 7) / 8)), dim3(KP * AT), 0, stream_, p.cp.d, 0, Rp, g, gL, n, KP, nfr, nfl);
  hipLaunchKernelGGL(k_prod_bwd<T>, dim3(p.cp.d.nright * 8 * (((n + AT - 1) / AT + 7) / 8)), dim3(KP * AT), 0, stream_, p.cp.d, 1, Lp, g, gR, n, KP, nfl, nfr);
}

// Slots (message functions) of one block of the pair kernels, in blocks of at most max_threads threads; when spreading the
// slots evenly over the same number of groups saves whole rounds of waves on the four SIMDs (36 slots of 64 channels: 3 x 12
// instead of 16 + 16 + 4), the even split, else the full blocks (72 slots: 4 x 16 + 8 ran faster than 5 x 15).  The forward
// kernel runs in blocks of 512 threads (config 4, layers 2 / 3: 6.3 / 11.3 ms against 7.2 / 13.2 with 1024; fp32 3.8 / 6.8
// against 3.6 / 9.9; 256 threads 6.0 / 11.7), the vector reverse kernels in blocks of 1024.
static int slots_per_block(int nslot, int CP, int max_threads)
{
  const int smax = std::max(1, std::min(nslot, max_threads / CP)), ngrp = (nslot + smax - 1) / smax, even = (nslot + ngrp - 1) / ngrp;
  auto rounds = [&](int spb) { return (spb * CP / 64 + 3) / 4; };
  return rounds(even) < rounds(smax) ? even : smax;
}

#define GR_PAIR1(K_, N_, grid_, block_, lds_, ...)                                                                       \
  {                                                                                                                      \
    auto kern = K_<T, N_>;                                                                                               \
    if (lds_ > 48 * 1024)                                                                                                \
      HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds_)); \
    hipLaunchKernelGGL(kern, grid_, block_, lds_, __VA_ARGS__);                                                          \
  }
#define GR_PAIR(K_, ...)                                     \
  switch (nl_) {                                             \
    case 1: GR_PAIR1(K_, 1, __VA_ARGS__) break;              \
    case 2: GR_PAIR1(K_, 4, __VA_ARGS__) break;              \
    case 3: GR_PAIR1(K_, 9, __VA_ARGS__) break;              \
    case 4: GR_PAIR1(K_, 16, __VA_ARGS__) break;             \
    case 5: GR_PAIR1(K_, 25, __VA_ARGS__) break;             \
    case 6: GR_PAIR1(K_, 36, __VA_ARGS__) break;             \
    default: GR_PAIR1(K_, 49, __VA_ARGS__) break;            \
  }
// the staged reverse kernel in its form without floating-point atomics
#define GR_PAIR_ORD1(N_, grid_, block_, lds_, ...)                                                                       \
  {                                                                                                                      \
    auto kern = k_pair_bwd<T, N_, true>;                                                                                 \
    if (lds_ > 48 * 1024)                                                                                                \
      HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds_)); \
    hipLaunchKernelGGL(kern, grid_, block_, lds_, __VA_ARGS__);                                                          \
  }
#define GR_PAIR_ORD(...)                                     \
  switch (nl_) {                                             \
    case 1: GR_PAIR_ORD1(1, __VA_ARGS__) break;              \
    case 2: GR_PAIR_ORD1(4, __VA_ARGS__) break;              \
    case 3: GR_PAIR_ORD1(9, __VA_ARGS__) break;              \
    case 4: GR_PAIR_ORD1(16, __VA_ARGS__) break;             \
    case 5: GR_PAIR_ORD1(25, __VA_ARGS__) break;             \
    case 6: GR_PAIR_ORD1(36, __VA_ARGS__) break;             \
    default: GR_PAIR_ORD1(49, __VA_ARGS__) break;            \
  }
// the reverse kernel with asynchronous staging and chunks of CH_ bonds
#define GR_PAIR_ASYNC1(N_, CH_, grid_, block_, lds_, ...)                                                                \
  {                                                                                                                      \
    auto kern = k_pair_bwd_async<T, N_, CH_>;                                                                            \
    if (lds_ > 48 * 1024)                                                                                                \
      HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds_)); \
    hipLaunchKernelGGL(kern, grid_, block_, lds_, __VA_ARGS__);                                                          \
  }
#define GR_PAIR_ASYNC(CH_, ...)                              \
  switch (nl_) {                                             \
    case 1: GR_PAIR_ASYNC1(1, CH_, __VA_ARGS__) break;       \
    case 2: GR_PAIR_ASYNC1(4, CH_, __VA_ARGS__) break;       \
    case 3: GR_PAIR_ASYNC1(9, CH_, __VA_ARGS__) break;       \
    case 4: GR_PAIR_ASYNC1(16, CH_, __VA_ARGS__) break;      \
    case 5: GR_PAIR_ASYNC1(25, CH_, __VA_ARGS__) break;      \
    case 6: GR_PAIR_ASYNC1(36, CH_, __VA_ARGS__) break;      \
    default: GR_PAIR_ASYNC1(49, CH_, __VA_ARGS__) break;     \
  }

// The message layer k gathers, for every atom and ghost: the normalised output of the layer below plus the species term
// (once per layer, before the chunks of its forward pass and again before those of its reverse: M_ is shared scratch).
template<class T> void Engine3L<T>::layer_messages(int k)
{
  Layer3<T> &L = L_[k];
  const Layer3<T> &Lm = L_[k - 1];
  M_.ensure((size_t) n_nodes_ * L.nlmi * L.CP * sizeof(T));
  stage(tg(k, "message").c_str(), [&] {
    const long long tot = (long long) n_nodes_ * L.nlmi * L.CP;
    hipLaunchKernelGGL(k_message<T>, dim3((unsigned) ((tot + 255) / 256)), dim3(256), 0, stream_, Lm.I.buf.template as<T>(), mu_.as<int>(),
                       L.zproj.template as<T>(), L.mask.template as<T>(), M_.as<T>(), n_nodes_, L.nlmi, L.CP);
  });
}

// Forward pass of layer k over the atoms of the current chunk.  Per-atom tensors hold the chunk's atoms from row 0 and the
// radial rows the chunk's bonds from row 0 (kernels index bonds by their number in the structure: the pointers are moved
// back); the messages, the raw densities and their adjoints are kept for the whole structure.  again: the forward pass
// repeated before the layer's reverse (a structure evaluated in several chunks keeps no layer tensors between the sweeps).
template<class T> void Engine3L<T>::layer_forward(int k, bool forces, int yw, bool again)
{
  Layer3<T> &L = L_[k];
  const int n = cn_;
  const size_t na = cap_, s = sizeof(T);
  const long long *n_edges = eoff_.as<long long>() + n_;
  const long long *eoff = eoff_.as<long long>() + a0_;
  const int *mu = mu_.as<int>() + a0_;
  L.R.ensure(ecap_ * L.rad.noutp * s);
  L.dR.ensure(ecap_ * L.rad.noutp * s);
  T *Rl = moved_back(L.R.template as<T>(), eb_ * L.rad.noutp), *dRl = moved_back(L.dR.template as<T>(), eb_ * L.rad.noutp);
  stage(tg(k, "radial").c_str(), [&] {
    L.rad.launch(stream_, ncu_, L.fac.template as<T>(), eb_, ecnt_, xr_.as<double>(), emu_.as<int>(), Rl, dRl, n_edges, emi_.as<int>(), true);
  });
  L.X.buf.ensure(L.X.bytes(na, s));
  T *X = L.X.buf.template as<T>();
  if (!L.equiv) {
    ScatterArgs<T> sa{};
    sa.eoff = eoff_.as<long long>(); sa.rh = rh_.as<double>(); sa.Rz = Rl; sa.A = X;
    sa.a0 = a0_; sa.C = L.CP; sa.nl = nl_; sa.nlm = nlm_; sa.noutp = L.rad.noutp; sa.sh = sh_;
    stage(tg(k, "scatter_A").c_str(), [&] { launch_scatter<T>(sa, n, lmax_); });
  } else {
    const int npf = L.nlmi * nlm_;
    pairP_.ensure(na * npf * L.CP * s);
    A_.ensure(na * L.nfA * L.CP * s);
    const int spb = slots_per_block(L.nlmi, L.CP, 512), ngrp = (L.nlmi + spb - 1) / spb;
    stage(tg(k, "pair_fwd").c_str(), [&] {
      const int pt = round_up(spb * L.CP, 64);
      // rows of CP values and of noutp values go to LDS 16 bytes at a time
      if ((L.CP * s) % 16 || (L.rad.noutp * s) % 16) throw Error("GRACE-3L: pair kernels need rows that are multiples of 16 bytes");
      const size_t lds = (size_t) 2 * kAsyncChunkFwd * (pt + L.rad.noutp) * s;
      GR_PAIR(k_pair_fwd, dim3((unsigned) ((n + 7) / 8 * 8 * ngrp)), dim3(pt), lds, stream_, eoff, ej_.as<int>(), YG_.as<T>(), (const T *) Rl,
              (const T *) M_.as<T>(), pairP_.as<T>(), L.nlmi, L.CP, nl_, L.rad.noutp, yw, sink_.as<T>(), ngrp, n, spb);
    });
    stage(tg(k, "couple_YI").c_str(), [&] {
      const int AT = 64 / L.CP;
      const int ngrp = (L.nfA + 4 * L.cg.rows - 1) / (4 * L.cg.rows);
      hipLaunchKernelGGL(k_lincomb<T>, dim3((unsigned) (((n + AT - 1) / AT + 7) / 8 * 8 * ngrp)), dim3(256), 0, stream_,
                         L.cg.off.template as<int>(), L.cg.idx.template as<int>(), L.cg.rowof.template as<int>(), L.cg.val.template as<double>(),
                         (const T *) pairP_.as<T>(), A_.as<T>(), npf, L.nfA, L.CP, n, L.cg.rows, ngrp);
    });
    stage(tg(k, "reduce_A").c_str(), [&] { cfwd_set(L.redA, A_.as<T>(), X); });
  }
  // ---- chain (fused_3l.cpp:970-990)
  const int nX = L.X.nf, wX = L.X.w, wR = L.wR;
  size_t maxP = 0;
  for (ProdStage<T> *p : {&L.p2, &L.p3, &L.p4}) maxP = std::max(maxP, (size_t) p->nfunc * p->rankP);
  P_.ensure(na * maxP * s);
  R2_.ensure(na * L.nR2 * wR * s);
  R3_.ensure(na * L.nR3 * wR * s);
  R4_.ensure(na * L.nR4 * wR * s);
  FA_.ensure(na * L.nR2 * wR * s);
  FB_.ensure(na * L.nR2 * wR * s);
  for (Ten *t : {&L.L2, &L.R2p, &L.L3, &L.R3p, &L.L4, &L.R4p}) t->buf.ensure(t->bytes(na, s));
  T *P = P_.as<T>(), *R2 = R2_.as<T>(), *R3 = R3_.as<T>(), *R4 = R4_.as<T>(), *FA = FA_.as<T>(), *FB = FB_.as<T>();
  auto prod = [&](const char *name, ProdStage<T> &p, const T *XL, const T *XR, Ten &Lp, Ten &Rp, T *Rout, int nfred) {
    (void) nfred;
    T *lp = Lp.buf.template as<T>(), *rp = Rp.buf.template as<T>();
    stage(tg(k, (std::string("proj_") + name).c_str()).c_str(), [&] {
      cfwd(p.U, XL, lp, 0);
      cfwd(p.V, XR, rp, 0);
    });
    stage(tg(k, (std::string("couple_") + name).c_str()).c_str(), [&] { couple_fwd(p, lp, Lp.nf, rp, Rp.nf, P); });
    stage(tg(k, (std::string("reduce_") + name).c_str()).c_str(), [&] { cfwd_set(p.red, P, Rout); });
  };
  auto fc = [&](const char *name, FcStage<T> &F, T *out) {
    stage(tg(k, name).c_str(), [&] {
      scale_rows(R2, F.nof, out, F.nf, wR, 0);
      cfwd(F.right, X, out, 1);
    });
  };
  prod("2", L.p2, X, X, L.L2, L.R2p, R2, L.nR2);
  fc("fc_2a", L.fa, FA);
  prod("3", L.p3, FA, X, L.L3, L.R3p, R3, L.nR3);
  fc("fc_2b", L.fb, FB);
  prod("4", L.p4, FB, FB, L.L4, L.R4p, R4, L.nR4);
  const T *srcs[4] = {X, R2, R3, R4};
  if (L.has_eq) {
    L.EQ.buf.ensure(L.EQ.bytes(na, s));
    L.I.buf.ensure(L.I.bytes((size_t) n_nodes_, s));    // rows of the ghost atoms too: the exchange fills them
    stage(tg(k, "reduce_eq").c_str(), [&] {
      zero(L.EQ.buf.p, L.EQ.bytes((size_t) n, s));
      for (int q = 0; q < 4; q++) cfwd(*L.eq[q], srcs[q], L.EQ.buf.template as<T>(), 1);
    });
    if (!again)    // the message rows exist already (and the layer above has read them)
      stage(tg(k, "eqnorm").c_str(), [&] {
        hipLaunchKernelGGL(k_eqnorm<T>, dim3(n), dim3(256), (size_t) L.eqn.M * sizeof(double), stream_, L.eqn, (const T *) L.EQ.buf.template as<T>(),
                           L.I.buf.template as<T>() + (size_t) a0_ * L.eqn.M * L.eqn.C, (const T *) nullptr, (T *) nullptr, 0);
      });
  }
  L.rho_raw.ensure((size_t) n_ * nrho_ * sizeof(double));
  L.grho.ensure((size_t) n_ * nrho_ * sizeof(double));
  (void) nX;
  if (again) return;    // the densities, the energy and the UQ rows come from the first forward pass
  stage(tg(k, "reduce_rho").c_str(), [&] {
    const int *tiles = cur_tiles_;
#define GR_RED(KA, KF) hipLaunchKernelGGL((k_reduce_fwd<T, KA, KF>), dim3(cur_ntiles_), dim3(64 * kReduceWaves), 0, stream_, L.rho.d, mu, tiles, srcs[0], srcs[1], \
                                          srcs[2], srcs[3], L.rho_raw.template as<double>() + (size_t) a0_ * nrho_)
    switch ((wX / 16) * 10 + wR / 16) {
      case 11: GR_RED(1, 1); break;
      case 12: GR_RED(1, 2); break;
      case 14: GR_RED(1, 4); break;
      case 21: GR_RED(2, 1); break;
      case 22: GR_RED(2, 2); break;
      case 24: GR_RED(2, 4); break;
      case 41: GR_RED(4, 1); break;
      case 42: GR_RED(4, 2); break;
      case 44: GR_RED(4, 4); break;
      default: throw Error("unsupported channel widths");
    }
#undef GR_RED
  });
  if (uq_on_) {    // this layer's rows of the basis while its tensors exist; the last layer finishes the GMM (fused_3l.cpp:1158-1201)
    stage(tg(k, "uq").c_str(), [&] {
      UqDev<T> u = L.uq;
      for (int q = 0; q < u.nsrc; q++) u.X[q] = srcs[L.uqSlot[q]];
      u.zacc = uqZ_.as<double>() + (size_t) a0_ * u.rp;
      u.n2acc = uqN2_.as<double>() + (size_t) a0_ * kUqMaxBlk;
      const size_t lds = (size_t) (u.d_basis + 4 * u.rp + 2 * u.D) * sizeof(double);
      auto kern = k_uq<T>;
      if (lds > 48 * 1024)
        HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds));
      hipLaunchKernelGGL(kern, dim3(n), dim3(256), lds, stream_, u, mu, n, uq_gamma_.as<double>() + a0_, uq_sigma_.as<double>() + a0_,
                         uq_cluster_.as<double>() + a0_);
    });
  }
  (void) forces;
}

// Reverse of layer k over the atoms of the current chunk.  In: L.grho (adjoint of the raw density) and, for layers 1-2,
// gMin_ (adjoint of the message this layer sent: dE/dI, accumulated by the pair kernel of the layer above).  Out: forces of
// the layer's bonds and, for layers 2-3, the adjoint of the message of the layer below added to gM_ (cleared by the caller
// before the first chunk).
template<class T> void Engine3L<T>::layer_backward(int k, int yw)
{
  Layer3<T> &L = L_[k];
  const int n = cn_;
  const size_t na = cap_, s = sizeof(T);
  const long long *eoff = eoff_.as<long long>() + a0_;
  const int *mu = mu_.as<int>() + a0_;
  T *Rl = moved_back(L.R.template as<T>(), eb_ * L.rad.noutp), *dRl = moved_back(L.dR.template as<T>(), eb_ * L.rad.noutp);
  const int nX = L.X.nf, wX = L.X.w, wR = L.wR;

  size_t maxP = 0, maxLp = 0;
  for (ProdStage<T> *p : {&L.p2, &L.p3, &L.p4}) maxP = std::max(maxP, (size_t) p->nfunc * p->rankP);
  for (Ten *t : {&L.L2, &L.R2p, &L.L3, &L.R3p, &L.L4, &L.R4p}) maxLp = std::max(maxLp, (size_t) t->nf * t->w);
  gP_.ensure(na * maxP * s);
  gLp_.ensure(na * maxLp * s);
  gRp_.ensure(na * maxLp * s);
  gX_.ensure(na * nX * wX * s);
  gR2_.ensure(na * L.nR2 * wR * s);
  gR3_.ensure(na * L.nR3 * wR * s);
  gR4_.ensure(na * L.nR4 * wR * s);
  gFA_.ensure(na * L.nR2 * wR * s);
  gFB_.ensure(na * L.nR2 * wR * s);
  T *gP = gP_.as<T>(), *gLp = gLp_.as<T>(), *gRp = gRp_.as<T>(), *gX = gX_.as<T>(), *gR2 = gR2_.as<T>(), *gR3 = gR3_.as<T>(), *gR4 = gR4_.as<T>(),
    *gFA = gFA_.as<T>(), *gFB = gFB_.as<T>();
  T *gsrc[4] = {gX, gR2, gR3, gR4};
  const size_t nn = (size_t) n;
  stage(tg(k, "zero_grads").c_str(), [&] {
    zero(gX, nn * nX * wX * s);
    zero(gR2, nn * L.nR2 * wR * s);
    zero(gR3, nn * L.nR3 * wR * s);
    zero(gR4, nn * L.nR4 * wR * s);
    zero(gFA, nn * L.nR2 * wR * s);
    zero(gFB, nn * L.nR2 * wR * s);
  });
  if (L.has_eq) {
    gEQ_.ensure(L.EQ.bytes(na, s));
    stage(tg(k, "eqnorm_bwd").c_str(), [&] {
      hipLaunchKernelGGL(k_eqnorm<T>, dim3(n), dim3(256), (size_t) L.eqn.M * sizeof(double), stream_, L.eqn, (const T *) L.EQ.buf.template as<T>(), (T *) nullptr,
                         (const T *) gMin_.as<T>() + (size_t) a0_ * L.eqn.M * L.eqn.C, gEQ_.as<T>(), 0);
    });
    stage(tg(k, "reduce_eq_bwd").c_str(), [&] {
      for (int q = 0; q < 4; q++) cbwd(*L.eq[q], gEQ_.as<T>(), gsrc[q], 1);
    });
  }
  stage(tg(k, "reduce_rho_bwd").c_str(), [&] {
    if (L.rho.njobs)
      hipLaunchKernelGGL(k_reduce_bwd<T>, dim3(cur_ntiles_, L.rho.njobs), dim3(64), 0, stream_, L.rho.d, mu, cur_tiles_,
                         (const double *) L.grho.template as<double>() + (size_t) a0_ * nrho_, gX, gR2, gR3, gR4);
  });
  // gXL / gXR: where the adjoints of the product's inputs are added
  auto prod_bwd = [&](const char *name, ProdStage<T> &p, Ten &Lp, Ten &Rp, const T *gR, T *gXL, T *gXR) {
    const T *lp = Lp.buf.template as<T>(), *rp = Rp.buf.template as<T>();
    stage(tg(k, (std::string("reduce_") + name + "_bwd").c_str()).c_str(), [&] { cbwd_set(p.red, gR, gP); });
    stage(tg(k, (std::string("couple_") + name + "_bwd").c_str()).c_str(), [&] {
      if (!p.jit_sets) {
        zero(gLp, Lp.bytes(nn, s));
        zero(gRp, Rp.bytes(nn, s));
      }
      couple_bwd(p, lp, Lp.nf, rp, Rp.nf, gP, gLp, gRp);
    });
    stage(tg(k, (std::string("proj_") + name + "_bwd").c_str()).c_str(), [&] {
      cbwd(p.U, gLp, gXL, 1);
      cbwd(p.V, gRp, gXR, 1);
    });
  };
  auto fc_bwd = [&](const char *name, FcStage<T> &F, const T *gout) {
    stage(tg(k, name).c_str(), [&] {
      scale_rows(gout, F.nof, gR2, F.nf, wR, 1);
      cbwd(F.right, gout, gX, 1);
    });
  };
  prod_bwd("4", L.p4, L.L4, L.R4p, gR4, gFB, gFB);
  fc_bwd("fc_2b_bwd", L.fb, gFB);
  prod_bwd("3", L.p3, L.L3, L.R3p, gR3, gFA, gX);
  fc_bwd("fc_2a_bwd", L.fa, gFA);
  prod_bwd("2", L.p2, L.L2, L.R2p, gR2, gX, gX);
  if (!L.equiv) {
    BondBwdArgs<T> ba{};
    ba.eoff = eoff_.as<long long>(); ba.ej = ej_.as<int>(); ba.rh = rh_.as<double>(); ba.r = r_.as<double>(); ba.rc = rc_.as<double>();
    ba.Rz = Rl; ba.dRz = dRl; ba.gA = gX;
    ba.f = f_.as<double>(); ba.virial = scal_.as<double>() + 1; ba.sid = sid_ptr(); ba.vatom = vatom_ptr();
    ba.a0 = a0_; ba.C = L.CP; ba.nl = nl_; ba.nlm = nlm_; ba.noutp = L.rad.noutp; ba.sh = sh_;
    if (ordered_) {
      ba.fedge = fedge_.as<double>(); ba.fcen = fcen_.as<double>(); ba.ordered_add = ordered_first_ ? 0 : 1;
    }
    stage(tg(k, "bond_bwd").c_str(), [&] { launch_bond_bwd<T>(ba, n); });
    return;
  }
  const int npf = L.nlmi * nlm_;
  gA_.ensure(na * L.nfA * L.CP * s);
  gpairP_.ensure(na * npf * L.CP * s);
  stage(tg(k, "reduce_A_bwd").c_str(), [&] { cbwd_set(L.redA, gX, gA_.as<T>()); });
  stage(tg(k, "couple_YI_bwd").c_str(), [&] {
    const int AT = 64 / L.CP;
    const int ngrp = (npf + 4 * L.cgt.rows - 1) / (4 * L.cgt.rows);
    hipLaunchKernelGGL(k_lincomb<T>, dim3((unsigned) (((n + AT - 1) / AT + 7) / 8 * 8 * ngrp)), dim3(256), 0, stream_,
                       L.cgt.off.template as<int>(), L.cgt.idx.template as<int>(), L.cgt.rowof.template as<int>(), L.cgt.val.template as<double>(),
                       (const T *) gA_.as<T>(), gpairP_.as<T>(), L.nfA, npf, L.CP, n, L.cgt.rows, ngrp);
  });
  const int spb = slots_per_block(L.nlmi, L.CP, 1024), ngrp = (L.nlmi + spb - 1) / spb, pthreads = round_up(spb * L.CP, 64);
  stage(tg(k, "pair_bwd").c_str(), [&] {
    // fp32: the next chunk is copied to a second LDS buffer while this one is worked on (chunks of 8 bonds in the large
    // blocks that fill a CU alone, of 4 otherwise); fp64 runs faster with one chunk staged through registers
    const size_t row = (size_t) (pthreads + 2 * L.rad.noutp) * s;
    const int ch = s != 4 ? 0 : (pthreads >= 512 && 16 * row <= kPairLdsMax) ? 8 : 8 * row <= kPairLdsMax ? 4 : 0;
    const size_t lds = ch && !ordered_ ? 2 * ch * row : kPairChunk * row;
    // ordered sums: the staged kernel without atomics; per slot group the bond forces and the per-atom sums, added in the
    // order of the groups afterwards; the message adjoints of the chunk's bonds gathered by neighbour atom afterwards
    PairOrdered<T> po{};
    if (ordered_) {
      gMe_.ensure(ecap_ * L.nlmi * L.CP * s);
      fpart_.ensure((size_t) 3 * std::max<int64_t>(nb_, 1) * ngrp * sizeof(double));
      cpart_.ensure((size_t) 9 * n_ * ngrp * sizeof(double));
      po.gMe = gMe_.as<T>(); po.fedge = fpart_.as<double>(); po.fcen = cpart_.as<double>(); po.e_base = eb_; po.ngrp = ngrp;
    }
#define GR_ARGS                                                                                                                          \
  dim3((unsigned) ((n + 7) / 8 * 8 * ngrp)), dim3(pthreads), lds, stream_, eoff, ej_.as<int>(), YG_.as<T>(), (const T *) Rl, (const T *) dRl,     \
      (const T *) M_.as<T>(), (const T *) gpairP_.as<T>(), rh_.as<double>(), r_.as<double>(), rc_.as<double>(), gM_.as<T>(), f_.as<double>(),   \
      scal_.as<double>() + 1, L.nlmi, L.nlmi, L.CP, nl_, L.rad.noutp, sink_.as<T>(), 1, sid_ptr(), spb, ngrp, n, a0_, vatom_ptr(), yw
    const PairMfmaPlan mp = pair_mfma_plan(L.nlmi, L.CP, nl_, s, pair_mfma_waves(s, pair_waves_));
    if (!ordered_ && mp.ok && pair_mfma_ != 0) {
      PairMfmaArgs<T> pa{};
      pa.eoff = eoff; pa.ej = ej_.as<int>(); pa.YG = YG_.as<T>(); pa.R1 = Rl; pa.dR1 = dRl; pa.M = M_.as<T>(); pa.gP = gpairP_.as<T>();
      pa.rh = rh_.as<double>(); pa.rlen = r_.as<double>(); pa.rcut = rc_.as<double>();
      pa.gM = gM_.as<T>(); pa.f = f_.as<double>(); pa.virial = scal_.as<double>() + 1; pa.vatom = vatom_ptr(); pa.sid = sid_ptr();
      pa.nslot = pa.nI = L.nlmi; pa.C = L.CP; pa.noutp = L.rad.noutp; pa.natoms = n; pa.a0 = a0_;
      for (int q = 0; q < 16; q++) pa.drow[q] = drow_[q];
      launch_pair_bwd_mfma(mp, pa, nl_, stream_);
    } else if (ordered_) {
      GR_PAIR_ORD(GR_ARGS, po)
      const long long nwork = 3 * (long long) (ecnt_ >= 0 ? ecnt_ : std::max<int64_t>(nb_, 1)) + 9ll * n;
      hipLaunchKernelGGL(k_ordered_combine, dim3((unsigned) ((nwork + 255) / 256)), dim3(256), 0, stream_, (const double *) fpart_.as<double>(),
                         (const double *) cpart_.as<double>(), ngrp, eb_, (const long long *) (eoff_.as<long long>() + n_), ecnt_, a0_, n, ordered_first_ ? 0 : 1, fedge_.as<double>(),
                         fcen_.as<double>());
      hipLaunchKernelGGL(k_ordered_gm<T>, dim3((unsigned) n_nodes_), dim3(std::min(1024, round_up(L.nlmi * L.CP, 64))), 0, stream_,
                         toff_.as<long long>(), tsorted_.as<int>(), (const T *) gMe_.as<T>(), eb_, (const long long *) (eoff_.as<long long>() + n_), ecnt_, L.nlmi * L.CP, gM_.as<T>());
    } else if (ch == 8) {
      GR_PAIR_ASYNC(8, GR_ARGS)
    } else if (ch == 4) {
      GR_PAIR_ASYNC(4, GR_ARGS)
    } else {
      GR_PAIR(k_pair_bwd, GR_ARGS, po)
    }
#undef GR_ARGS
  });
}

// bytes of chunk-sized work buffers per atom of a chunk (per-atom tensors of the forward and the reverse pass and, per bond
// of an atom, the radial rows of the three layers), largest layer
template<class T> double Engine3L<T>::chunk_bytes_per_atom() const
{
  const double bonds = (double) std::max<int64_t>(nb_, 1) / std::max(n_, 1);
  double shared = 0.0, kept = 0.0;
  for (int k = 0; k < 3; k++) {
    const Layer3<T> &L = L_[k];
    double maxP = 0, maxLp = 0, proj = 0;
    for (const ProdStage<T> *p : {&L.p2, &L.p3, &L.p4}) maxP = std::max(maxP, (double) p->nfunc * p->rankP);
    for (const Ten *t : {&L.L2, &L.R2p, &L.L3, &L.R3p, &L.L4, &L.R4p}) {
      maxLp = std::max(maxLp, (double) t->nf * t->w);
      proj += (double) t->nf * t->w;
    }
    const double X = (double) L.X.nf * L.X.w, R = (double) (L.nR2 + L.nR3 + L.nR4) * L.wR, F = 2.0 * L.nR2 * L.wR;
    const double spbf = L.equiv ? 2.0 * ((double) L.nlmi * nlm_ + L.nfA) * L.CP : 0.0;    // pair tensor and coupled functions, with adjoints
    const double eq = L.has_eq ? 2.0 * L.EQ.nf * L.EQ.w : 0.0;
    shared = std::max(shared, spbf + 2.0 * maxP + 2.0 * maxLp + X + 2.0 * R + 2.0 * F + (L.has_eq ? (double) L.EQ.nf * L.EQ.w : 0.0));
    kept += X + proj + eq / 2.0 + 2.0 * bonds * L.rad.noutp;    // every layer keeps its own inputs of the reverse
  }
  if (ordered_) {    // ordered sums: the message adjoints of the chunk's bonds, widest layer
    double rows = 0.0;
    for (int k = 0; k < 3; k++)
      if (L_[k].equiv) rows = std::max(rows, (double) L_[k].nlmi * L_[k].CP);
    shared += bonds * rows;
  }
  return (shared + kept) * sizeof(T);
}

template<class T> void Engine3L<T>::run(const RunFlags &fl)
{
  const int n = n_;
  ordered_check(fl);
  if (!begin_pass(fl)) return;
  const size_t ecap = (size_t) std::max<int64_t>(nb_, 1);
  const long long *n_edges = eoff_.as<long long>() + n;
  const bool forces = !fl.energy_only;
  if (ordered_ && forces) ordered_begin();
  emi_.ensure(ecap * sizeof(int));
  stage("edge_center", [&] { hipLaunchKernelGGL(k_edge_center, dim3(n), dim3(64), 0, stream_, eoff_.as<long long>(), mu_.as<int>(), emi_.as<int>()); });
  // row of an edge: Y[nlm] and, for forces, the two tangential gradients D1[nlm], D2[nlm] and padding (pair_row_stride)
  const int yw = forces ? pair_row_stride(nlm_, sizeof(T)) : nlm_;
  YG_.ensure(ecap * yw * sizeof(T));
  stage("sh_edges", [&] {
    const size_t lds = (size_t) 64 * ((forces ? 3 * nlm_ : nlm_) + 1) * sizeof(T);
    auto kern = k_sh_edges<T>;
    if (lds > 48 * 1024) HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds));
    hipLaunchKernelGGL(kern, dim3((unsigned) ((ecap + 63) / 64)), dim3(64), lds, stream_, sh_, rh_.as<double>(), n_edges, nlm_, forces ? 1 : 0,
                       YG_.as<T>(), yw);
  });
  uq_on_ = fl.uq;
  if (fl.uq) {
    const size_t na = (size_t) n;
    uq_gamma_.ensure(na * sizeof(double)); uq_sigma_.ensure(na * sizeof(double)); uq_cluster_.ensure(na * sizeof(double));
    uqZ_.ensure(na * L_[0].uq.rp * sizeof(double));
    uqN2_.ensure(na * kUqMaxBlk * sizeof(double));
  }

  // ---- chunks of atoms.  A layer needs the messages of ALL atoms of the layer below, so the forward pass goes layer by
  // layer over the chunks, and so does the reverse from the top.  What is kept for the whole structure: the harmonics and
  // the compact bonds, per layer the message, the raw density and its adjoint, and two arrays of message adjoints.  Every
  // other tensor (the radial rows of a layer included) exists for one chunk: with more than one chunk the reverse of a
  // layer repeats that layer's forward pass for the chunk first (the reference's store_l1 = false, libgrace/include/grace/
  // system.h:79-80, extended to every layer).
  const double bonds_per_atom = (double) ecap / n;
  double kept = bonds_per_atom * (60.0 + yw * sizeof(T)) + 64.0;
  for (int k = 0; k < 3; k++) kept += 3.0 * (double) L_[k].I.nf * L_[k].I.w * sizeof(T) + 16.0 * nrho_;
  const int cs = plan_chunk(n, chunk_bytes_per_atom(), kept);
  const int nchunks = (n + cs - 1) / cs;
  chunk_used_ = nchunks > 1 ? cs : 0;
  std::vector<long long> ebound;
  cap_ = (size_t) cs;
  ecap_ = ecap;
  if (nchunks > 1) {
    layout_chunks(cs);
    ebound = chunk_edge_bounds(cs);
    ecap_ = 1;
    for (int q = 0; q < nchunks; q++) ecap_ = std::max(ecap_, (size_t) (ebound[(size_t) q + 1] - ebound[(size_t) q]));
  }
  auto set_chunk = [&](int q) {
    if (nchunks == 1) {
      a0_ = 0; cn_ = n; eb_ = 0; ecnt_ = -1;
      cur_tiles_ = tiles_.as<int>(); cur_ntiles_ = ntiles_; cur_tile_el_ = tile_el_.data();
      return;
    }
    a0_ = q * cs;
    cn_ = std::min(n, a0_ + cs) - a0_;
    eb_ = ebound[(size_t) q];
    ecnt_ = ebound[(size_t) q + 1] - eb_;
    cur_tiles_ = chunk_tiles_.as<int>() + (size_t) 16 * chunk_tile_off_[(size_t) q];
    cur_ntiles_ = chunk_tile_off_[(size_t) q + 1] - chunk_tile_off_[(size_t) q];
    cur_tile_el_ = chunk_tile_el_[(size_t) q].data();
  };
  for (int k = 0; k < 3; k++) {
    if (L_[k].equiv) {
      exchange_forward(k);    // the message of layer k (counted from 1) reaches the ghost atoms
      layer_messages(k);
    }
    for (int q = 0; q < nchunks; q++) {
      set_chunk(q);
      layer_forward(k, forces, yw, false);
    }
  }
  set_chunk(0);
  if (fl.uq) ran_uq_ = true;
  stage("energy_mlp", [&] {
    hipLaunchKernelGGL(k_energy_3l, dim3(n), dim3(64), (size_t) (nrho_ + 2 * en_.nh) * sizeof(double), stream_, en_, mu_.as<int>(),
                       (const double *) L_[0].rho_raw.template as<double>(), (const double *) L_[1].rho_raw.template as<double>(),
                       (const double *) L_[2].rho_raw.template as<double>(), L_[0].grho.template as<double>(), L_[1].grho.template as<double>(),
                       L_[2].grho.template as<double>(), fl.eatom || ordered_ ? eatom_.as<double>() : nullptr, ordered_ ? nullptr : scal_.as<double>(),
                       forces ? 1 : 0, sid_ptr());
  });
  if (!forces) {
    if (ordered_) ordered_finish(fl);
    return;
  }
  ordered_first_ = true;
  for (int k = 2; k >= 0; k--) {
    Layer3<T> &L = L_[k];
    if (L.equiv) {
      layer_messages(k);    // M_ holds the message of the layer that ran last
      gM_.ensure((size_t) n_nodes_ * L.nlmi * L.CP * sizeof(T));
      stage(tg(k, "message_bwd").c_str(), [&] { zero(gM_.p, (size_t) n_nodes_ * L.nlmi * L.CP * sizeof(T)); });
    }
    for (int q = 0; q < nchunks; q++) {
      set_chunk(q);
      if (nchunks > 1) layer_forward(k, forces, yw, true);
      layer_backward(k, yw);
    }
    ordered_first_ = false;    // the layers below add to the bond forces this one stored
    if (L.equiv) {
      comm_reverse_layer_ = k;
      exchange_reverse(k);    // the ghosts' adjoint rows of the message of layer k go to their owners
      comm_reverse_layer_ = 0;
      std::swap(gM_.p, gMin_.p);    // what this layer gathered is what the layer below sent
      std::swap(gM_.bytes, gMin_.bytes);
    }
  }
  set_chunk(0);
  if (ordered_) ordered_finish(fl);
}

#undef GR_PAIR_ASYNC
#undef GR_PAIR_ASYNC1
#undef GR_PAIR_ORD
#undef GR_PAIR_ORD1
#undef GR_PAIR
#undef GR_PAIR1

}    // namespace

std::unique_ptr<Engine> make_engine_3l(std::shared_ptr<const Model3L> model, int ntypes, const std::vector<int> &type2mu, int precision,
                                       int device)
{
  if (precision == 64) return std::make_unique<Engine3L<double>>(std::move(model), ntypes, type2mu, device);
  if (precision == 32) return std::make_unique<Engine3L<float>>(std::move(model), ntypes, type2mu, device);
  throw InvalidArgument("precision must be 64 or 32");
}

}    // namespace grhip
