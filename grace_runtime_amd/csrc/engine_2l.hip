// GRACE-2L engine for gfx950: two message-passing layers on one GPU, whole structure resident.
// Phases after libgrace/src/fused_2l.cpp:849-1099 of the reference (P1 layer 1 forward -> message I and rho of every
// atom; P3 layer 2, readout, layer-2 reverse with dE/dI_j added to the neighbours; P5 layer 1 reverse), without the
// layer-1 recompute: the layer-1 tensors of all atoms stay in device memory between P1 and P5.
// Dense chains (FC, CG products, reduces) reuse the GRACE-1L kernels; liveness pruning after fused_2l.cpp:296-345.
#include "engine_common.hpp"
#include "jit_chain.hpp"
#include "kernels_2l.hpp"
#include "model_2l.hpp"

namespace grhip {

namespace {

// One dense chain X -> X1 = FC(X, X) -> XX = X1 x X1 -> XX1 = FC(XX, X) -> XXX = XX1 x X [-> XX2 = FC(XX, X) ->
// XXXX = XX2 x XX2] of a layer (X = A or B), all tensors of one padded channel width.
template<class T> struct Chain {
  int nf = 0, nXX = 0, nXXX = 0, nXXXX = 0, kb = 0;    // functions of X, XX, XXX, XXXX; 16-channel blocks
  bool order4 = false, jit_all = false;
  DevFc<T> fc1, fc2, fc3;
  DevFcPairBwd<T> fc23;    // reverse of fc2 and fc3 in one pass over their shared inputs (order 4)
  DevProd p2, p3, p4;
  // the whole chain as one generated kernel per direction (jit_chain.hpp); not ok(): the stage-by-stage kernels run
  ChainKernels fused;
  DevBuf fusedW, keepXX;    // fragment-ordered weights; the functions of XX the reduces collect (their adjoint rows are cleared)
  int nkeepXX = 0;
  bool fuse3 = true;        // P3 = XX1 x X inside the chain kernels (few outputs) or as the product kernels below (many)
  std::string fused_note;
  ~Chain() { fused.release(); }
  DevBuf X1, XX, XX1, XXX, XX2, XXXX, gX, gX1, gXX, gXX1, gXXX, gXX2, gXXXX;
  const T *src(int s, const T *X) const
  {
    return s == 0 ? X : s == 1 ? XX.as<T>() : s == 2 ? XXX.as<T>() : XXXX.as<T>();
  }
  T *gsrc(int s) const { return s == 0 ? gX.as<T>() : s == 1 ? gXX.as<T>() : s == 2 ? gXXX.as<T>() : gXXXX.as<T>(); }
  int nfun(int s) const { return s == 0 ? nf : s == 1 ? nXX : s == 2 ? nXXX : nXXXX; }
};

template<class T> class Engine2L final : public EngineBase {
 public:
  Engine2L(std::shared_ptr<const Model2L> m, int ntypes, const std::vector<int> &type2mu, int device) :
      EngineBase(device, "GRACE-2L", ntypes, type2mu, m->n_elements), model_(std::move(m))
  {
    this->template probe_mfma_both<T>();
    build();
    end_build();    // buffers allocated from here on are work buffers (release_buffers)
    chunks_ = true;
    ordered_ok_ = true;
  }
  int layers() const override { return 2; }
  void apply_spline(int n) override { radR_.spline_n = radR1_.spline_n = n; }
  void run(const RunFlags &fl) override;
  void debug_radial(int, const double *, const int *, double *, double *) override
  {
    throw Error("GRACE-2L: debug_radial is available for GRACE-1L engines");
  }
  // one message: the functions I of layer 1 (libgrace/include/grace/kk/grace_2l_kk.h:141: I_n_funcs x I_n_out doubles per atom)
  int comm_layers() const override { return 1; }
  int comm_width(int layer) const override { return layer == 1 ? nI_ * model_->CR : 0; }
  void comm_rows(int mode, int layer, int n, const int *list, int first, double *buf, bool host) override
  {
    if (layer != 1) throw InvalidArgument("GRACE-2L exchanges the message of layer 1 only");
    if (mode < 2) move_rows<T>(mode, M_.as<T>(), (long long) nslot_ * CRP_, nI_, model_->CR, CRP_, n, list, first, buf, host);
    else move_rows<T>(mode, gM_.as<T>(), (long long) nI_ * CRP_, nI_, model_->CR, CRP_, n, list, first, buf, host);
  }

 private:
  std::shared_ptr<const Model2L> model_;
  int lmax_ = 0, nl_ = 0, nlm_ = 0, nel_ = 0, C1P_ = 0, CRP_ = 0, C2P_ = 0, PI1_ = 0, nI1_ = 0, nI_ = 0, nslot_ = 0, nB_ = 0, nrho_ = 0;
  bool order4_ = false;
  ShCoef sh_{};
  DevBuf zA_, zB0_, ones_, shift_, lnI_, ln0_, eW_[7];
  DevRadial<T> radR_, radR1_;
  Chain<T> c1_, c2_;
  DevReduce<T> redrho_, redI2_;
  UqDev<T> uq_{};             // UQ head: blocks [I2 (layer 2), rho (layer 1)]
  DevBuf uqR_, uqCen_, uqIcov_, uqNcl_, uqThr_, uqCi_[kUqMaxSrc];
  std::vector<std::unique_ptr<DevReduce<T>>> redI1_;    // one per output function of I1
  DevBuf WI_, WIT_, WB_, WBT_;
  DevJobs<T> jI_, jIb_, jB_, jBb_;
  Energy2Dev en_{};
  // pass buffers
  DevBuf sink_, Rz_, dRz_, R1_, dR1_, YG_, A_, rho_, grho_, I1_, gI1_, I1t_, gI1t_, M_, gM_, P_, gP_, B_, I2_, gI2_;
  DevBuf gMe_;    // ordered sums: the message adjoints of a chunk's bonds, [bond][nI][CRP]
  // the chunk of atoms the chain and reduce functions act on: cn_ atoms from a0_, the chunk's element tiles (atoms counted
  // from a0_), the capacity the chunk buffers are sized for
  int cn_ = 0, a0_ = 0;
  size_t cap_ = 0;
  const int *cur_tiles_ = nullptr;
  int cur_ntiles_ = 0;

  void build();
  void build_chain(Chain<T> &c, const char *tag, int nf, int KP, const FCWeights *fc[3], const CGProduct *pr[3],
                   const std::vector<const ReduceEq *> reds[4]);
  void gemm(DevJobs<T> &J, int kb0, int nb, const T *X0, int nf0, T *out, int nfo, int accumulate)
  {
    EngineBase::launch_gemm<T>(J, kb0, kb0, nb, X0, nf0, X0, nf0, out, nfo, accumulate, cur_tiles_, cur_ntiles_);
  }
  void chain_forward(Chain<T> &c, const char *tag, const T *X);
  void chain_zero(Chain<T> &c, const char *tag);
  void chain_backward(Chain<T> &c, const char *tag, const T *X, const std::function<void()> &reduces_x_xx);
  void reduce_fwd(DevReduce<T> &R, int kb, const Chain<T> &c, const T *X, double *out);
  void reduce_bwd(DevReduce<T> &R, const Chain<T> &c, const double *g, bool high);
  std::string tagged(const char *tag, const char *name) { return std::string(name) + tag; }
};

template<class T>
void Engine2L<T>::build_chain(Chain<T> &c, const char *tag, int nf, int KP, const FCWeights *fc[3], const CGProduct *pr[3],
                              const std::vector<const ReduceEq *> reds[4])
{
  c.nf = nf;
  c.kb = KP / 16;
  c.order4 = order4_;
  c.nXX = pr[0]->n_out;
  c.nXXX = pr[1]->n_out;
  c.nXXXX = order4_ ? pr[2]->n_out : 0;
  auto collected = [&](int s, int n) {
    std::vector<char> v(n, 0);
    for (const ReduceEq *r : reds[s])
      for (int q : r->collect_ind) v[q] = 1;
    return v;
  };
  HostProd h3 = build_prod(*pr[1], collected(2, c.nXXX), c.nXX, nf);
  std::vector<char> live2(c.nXX, 0), live3(c.nXX, 0), live1(nf, 0);
  for (int q : h3.l) live2[q] = 1;
  HostProd h4;
  if (order4_) {
    h4 = build_prod(*pr[2], collected(3, c.nXXXX), c.nXX, c.nXX);
    for (int q : h4.l) live3[q] = 1;
    for (int q : h4.r) live3[q] = 1;
  }
  std::vector<char> need2 = collected(1, c.nXX);
  for (int q = 0; q < c.nXX; q++) need2[q] = need2[q] || live2[q] || live3[q];
  HostProd h2 = build_prod(*pr[0], need2, nf, nf);
  for (int q : h2.l) live1[q] = 1;
  for (int q : h2.r) live1[q] = 1;
  c.p2.build(h2);
  c.p3.build(h3);
  if (order4_) c.p4.build(h4);
  const bool f32 = sizeof(T) == 4;
  const std::string t(tag);
  jit_compile_product(("prod2" + t).c_str(), h2.terms, nf, nf, c.nXX, true, KP, f32, arch_, c.p2.jit, c.p2.jit_note);
  jit_compile_product(("prod3" + t).c_str(), h3.terms, c.nXX, nf, c.nXXX, false, KP, f32, arch_, c.p3.jit, c.p3.jit_note);
  if (order4_) jit_compile_product(("prod4" + t).c_str(), h4.terms, c.nXX, c.nXX, c.nXXXX, true, KP, f32, arch_, c.p4.jit, c.p4.jit_note);
  c.jit_all = c.p2.jit.ok() && c.p3.jit.ok() && (!order4_ || c.p4.jit.ok());
  {
    // the fused chain: same liveness, same pruned term lists; P3 = XX1 x X (the right operand is the chain's input)
    ChainSpec sp;
    sp.C = KP;
    sp.f32 = f32;
    sp.nf0 = nf;
    sp.fc1 = chain_fc_spec(*fc[0], live1, nf);
    sp.nP2 = c.nXX;
    sp.prod2 = h2.terms;
    sp.fc21 = chain_fc_spec(*fc[1], live2, nf);
    sp.have22 = order4_;
    if (order4_) sp.fc22 = chain_fc_spec(*fc[2], live3, nf);
    sp.nP3 = c.nXXX;
    sp.prod3 = h3.terms;
    sp.prod3_right_x0 = true;
    {
      std::set<int> outs;
      for (const ProdTerm &q : h3.terms) outs.insert(q.o);
      c.fuse3 = sp.fuse3 = outs.size() <= 24;    // the outputs of a fused P3 are accumulated in registers
    }
    sp.nP4 = c.nXXXX;
    if (order4_) sp.prod4 = h4.terms;
    sp.keepP2 = collected(1, c.nXX);
    sp.keepX0 = collected(0, nf);
    for (int q = 0; q < 16; q++) sp.drow[q] = drow_[q];
    std::vector<double> w;
    if (jit_compile_chain(("chain" + t).c_str(), sp, arch_, c.fused, w, c.fused_note)) {
      std::vector<T> wt(w.begin(), w.end());
      upload_vec(c.fusedW, wt);
      std::vector<int> keep;
      for (int q = 0; q < c.nXX; q++)
        if (sp.keepP2[q]) keep.push_back(q);
      c.nkeepXX = (int) keep.size();
      if (keep.empty()) keep.push_back(0);
      upload_vec(c.keepXX, keep);
    } else {
      log_message(1, std::string("GRACE-2L: the dense chain") + tag + " runs stage by stage (" + c.fused_note + ")");
    }
  }
  c.fc1.build(*fc[0], live1, nf, KP, KP, KP, drow_, false, true);    // both inputs are X: one reverse launch
  // the reverse of fc2 (with the fourth-order stage: of fc2 and fc3 in one pass) WRITES the adjoint of XX: a job per function
  c.fc2.build(*fc[1], live2, nf, KP, KP, KP, drow_, true);
  if (order4_) {
    c.fc3.build(*fc[2], live3, nf, KP, KP, KP, drow_);
    c.fc23.build(*fc[1], live2, c.fc2, *fc[2], live3, c.fc3, nf, drow_, true);
  }
}

template<class T> void Engine2L<T>::build()
{
  const Model2L &m = *model_;
  lmax_ = m.lmax;
  if (lmax_ > kKernMaxL) throw Error("GRACE-2L: lmax > " + std::to_string(kKernMaxL) + " not supported");
  nl_ = lmax_ + 1;
  nlm_ = nl_ * nl_;
  nel_ = m.n_elements;
  order4_ = m.max_order == 4;
  nrho_ = m.rho_n_out;
  nI1_ = m.I1_n_funcs;
  nI_ = m.I_n_funcs;
  nslot_ = nI_ + 1;
  nB_ = m.B_n_funcs;
  auto pad_width = [](int c) { return c <= 16 ? 16 : c <= 32 ? 32 : c <= 64 ? 64 : -1; };
  C1P_ = pad_width(m.C1);
  CRP_ = pad_width(m.CR);
  C2P_ = pad_width(m.C2);
  PI1_ = pad_width(m.I1_n_out);
  if (C1P_ < 0 || CRP_ < 0 || C2P_ < 0 || PI1_ < 0) throw Error("GRACE-2L: channel widths above 64 are not supported by the GPU kernels");
  if (nrho_ > 32 || m.I1_n_out > 32) throw Error("GRACE-2L: rho_n_out or I1_n_out > 32 not supported by the GPU reduce kernels");
  if (nslot_ * CRP_ > 1024) throw Error("GRACE-2L: (I_n_funcs + 1) x message width exceeds one block");

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
  // ---- pair cutoffs, species weights zA, zB0 (fused_2l.cpp:176-192), unit weights for the bare layer-2 radial functions
  {
    std::vector<double> cut((size_t) nel_ * nel_);
    for (int a = 0; a < nel_; a++)
      for (int b = 0; b < nel_; b++) cut[(size_t) a * nel_ + b] = m.pair_cutoff(a, b);
    set_cutoffs(cut);
    auto ztab = [&](const std::vector<double> &W, double norm, double inv, int C, int CP) {
      std::vector<T> z((size_t) nel_ * CP, (T) 0);
      for (int mu = 0; mu < nel_; mu++)
        for (int n = 0; n < C; n++) {
          double v = 0.0;
          for (int e = 0; e < m.embedding_size; e++) v += W[(size_t) e * C + n] * m.chem_embedding[(size_t) mu * m.embedding_size + e];
          z[(size_t) mu * CP + n] = (T) (v * norm * inv);
        }
      return z;
    };
    upload_vec(zA_, ztab(m.A_lin_transform_W, m.A_lin_transform_norm, m.A_inv_avg_n_neigh, m.C1, C1P_));
    upload_vec(zB0_, ztab(m.B0_lin_transform_W, m.B0_lin_transform_norm, m.B0_inv_avg_n_neigh, m.CR, CRP_));
    upload_vec(ones_, std::vector<T>((size_t) nel_ * CRP_, (T) 1));
    upload_vec(shift_, m.shift_values);
  }
  sink_.ensure(64);
  radR_.build(m.mlp_R, m.nradbase, m.radial_basis_p, m.radial_activation, m.C1, C1P_, nl_, nel_, drow_, "GRACE-2L");
  radR1_.build(m.mlp_R1, m.nradbase, m.radial_basis_p, m.radial_activation, m.CR, CRP_, nl_, nel_, drow_, "GRACE-2L");
  radR_.build_double(m.mlp_R, m.nradbase, m.radial_basis_p, m.radial_activation, m.C1, C1P_, nl_, nel_, drow64_, "GRACE-2L");
  radR1_.build_double(m.mlp_R1, m.nradbase, m.radial_basis_p, m.radial_activation, m.CR, CRP_, nl_, nel_, drow64_, "GRACE-2L");

  // ---- the two dense chains
  const int ns = m.nsrc();
  {
    const FCWeights *fc[3] = {&m.fc_A1, &m.fc_AA1, &m.fc_AA2};
    const CGProduct *pr[3] = {&m.prod_AA, &m.prod_AAA, &m.prod_AAAA};
    std::vector<const ReduceEq *> reds[4];
    for (int s = 0; s < ns; s++) reds[s] = {&m.I1_red[s], &m.rho_red[s]};
    build_chain(c1_, "_L1", nlm_, C1P_, fc, pr, reds);
  }
  {
    const FCWeights *fc[3] = {&m.fc_B1, &m.fc_BB1, &m.fc_BB2};
    const CGProduct *pr[3] = {&m.prod_BB, &m.prod_BBB, &m.prod_BBBB};
    std::vector<const ReduceEq *> reds[4];
    for (int s = 0; s < ns; s++) reds[s] = {&m.I2_red[s]};
    build_chain(c2_, "_L2", nB_, C2P_, fc, pr, reds);
  }
  // ---- element-dependent reduces: rho, I1 (one per output function), I2
  auto sources = [&](const ReduceEq *r, const Chain<T> &c, int KP, bool with_fo) {
    std::vector<ReduceSrc> v;
    for (int s = 0; s < ns; s++)
      v.push_back({&r[s].W, r[s].norm, r[s].n_in, r[s].w_shape, &r[s].collect_ind, &r[s].w_l_tile, with_fo ? &r[s].total_sum_ind : nullptr,
                   c.nfun(s), KP});
    return v;
  };
  redrho_.build(sources(m.rho_red, c1_, C1P_, false), nel_, nrho_, -1, nrho_, 0, drow_);
  redI2_.build(sources(m.I2_red, c2_, C2P_, false), nel_, nrho_, -1, nrho_, 0, drow_);
  // ---- UQ head: a head that does not validate leaves the model usable without UQ (libgrace/src/model_2l.cpp:404-478)
  if (m.uq.has_uq) {
    try {
      m.validate_uq();
      if (m.uq.rp_dim > 256 || m.uq.feature_dim > 256) throw Error("GRACE-2L UQ: feature widths above 256 are not supported");
      int off = 0, q = 0;
      for (int b = 0; b < 2; b++) {    // block 0: I2 over (B, BB, BBB, BBBB); block 1: rho over (A, AA, AAA, AAAA)
        const ReduceEq *r = b == 0 ? m.I2_red : m.rho_red;
        const Chain<T> &c = b == 0 ? c2_ : c1_;
        for (int s = 0; s < ns; s++, q++) {
          upload_vec(uqCi_[q], r[s].collect_ind);
          uq_.ci[q] = uqCi_[q].template as<int>();
          uq_.nfun[q] = c.nfun(s);
          uq_.cpad[q] = b == 0 ? C2P_ : C1P_;
          uq_.nin[q] = r[s].n_in;
          uq_.nc[q] = (int) r[s].collect_ind.size();
          uq_.off[q] = off;
          uq_.blk[q] = b;
          off += uq_.nin[q] * uq_.nc[q];
        }
      }
      uq_.nsrc = q; uq_.nblk = 2; uq_.d_basis = off; uq_.row0 = 0; uq_.carry_in = uq_.carry_out = 0;
      uq_.rp = m.uq.rp_dim; uq_.D = m.uq.feature_dim; uq_.K = m.uq.max_clusters;
      uq_.density_scale = m.uq.density_scale;
      upload_vec(uqR_, m.uq.rp_matrix); upload_vec(uqCen_, m.uq.centroids); upload_vec(uqIcov_, m.uq.inv_cov);
      upload_vec(uqNcl_, m.uq.n_clusters); upload_vec(uqThr_, m.uq.interp_thresholds);
      uq_.R = uqR_.template as<double>(); uq_.cen = uqCen_.template as<double>(); uq_.icov = uqIcov_.template as<double>();
      uq_.ncl = uqNcl_.template as<int>(); uq_.thr = uqThr_.template as<double>();
      if ((size_t) (uq_.d_basis + 4 * uq_.rp + 2 * uq_.D) * sizeof(double) > 150 * 1024) throw Error("GRACE-2L UQ: the basis does not fit the kernel's LDS");
      has_uq_head_ = true;
    } catch (const std::exception &e) {
      uq_why_ = e.what();
    }
  } else {
    uq_why_ = "the model file carries none";
  }
  for (int fo = 0; fo < nI1_; fo++) {
    redI1_.emplace_back(new DevReduce<T>());
    redI1_.back()->build(sources(m.I1_red, c1_, C1P_, true), nel_, m.I1_n_out, fo, nI1_ * PI1_, fo * PI1_, drow_);
  }
  // ---- I from I1 and B from (YI, B0): tile-GEMM job lists (weights not element dependent).  W: [n_out][n_in][w_shape]
  auto tile_frags = [&](const ReduceEq &r, int nout, int KinP, int NoutP, std::vector<T> &F, std::vector<T> &Ft) {
    std::vector<double> Mx((size_t) r.n_in * nout), Mt((size_t) nout * r.n_in);
    for (int t = 0; t < r.w_shape; t++) {
      for (int k = 0; k < nout; k++)
        for (int n = 0; n < r.n_in; n++) {
          const double v = r.norm * r.W[((size_t) k * r.n_in + n) * r.w_shape + t];
          Mx[(size_t) n * nout + k] = v;
          Mt[(size_t) k * r.n_in + n] = v;
        }
      pack_fragments<T>(Mx, r.n_in, nout, KinP, NoutP, F);
      pack_fragments<T>(Mt, nout, r.n_in, NoutP, KinP, Ft);
    }
  };
  {
    const ReduceEq &r = m.I_red;
    std::vector<T> F, Ft;
    tile_frags(r, m.CR, PI1_, CRP_, F, Ft);
    upload_vec(WI_, F);
    upload_vec(WIT_, Ft);
    typename DevJobs<T>::Host hf, hb;
    for (int fo = 0; fo < nI_; fo++) {
      hf.job(fo, 1.0);
      for (size_t c = 0; c < r.collect_ind.size(); c++)
        if (r.total_sum_ind[c] == fo) hf.seg(0, r.collect_ind[c], r.w_l_tile[c], 1.0);
      hf.end_job();
    }
    for (int fi = 0; fi < nI1_; fi++) {
      hb.job(fi, 1.0);
      for (size_t c = 0; c < r.collect_ind.size(); c++)
        if (r.collect_ind[c] == fi) hb.seg(0, r.total_sum_ind[c], r.w_l_tile[c], 1.0);
      hb.end_job();
    }
    jI_.build(hf, WI_.as<T>(), WI_.as<T>());
    jIb_.build(hb, WIT_.as<T>(), WIT_.as<T>());
    jI_.set_rows(drow_);
    jIb_.set_rows(drow_);
  }
  {
    // B[fo] = sum over YI connections c -> fo of W_YI[tile c] YI[ci c]  +  sum over B0 connections of W_B0[tile c] B0[ci c],
    // YI[o] = inv_avg sum_t cg_t P[(I_t, y_t)] (fused_2l.cpp:228-276, 655-665) folded in: one segment per coupling term.
    // The pair tensor P has functions slot * nlm + lm; slot nI is B0.
    const ReduceEq &ry = m.B_red_YI, &r0 = m.B_red_B0;
    std::vector<T> F, Ft;
    tile_frags(ry, m.C2, CRP_, C2P_, F, Ft);
    tile_frags(r0, m.C2, CRP_, C2P_, F, Ft);
    upload_vec(WB_, F);
    upload_vec(WBT_, Ft);
    struct Seg { int fo, pair, tile; double scale; };
    std::vector<Seg> segs;
    for (size_t c = 0; c < ry.collect_ind.size(); c++)
      for (int t = 0; t < m.yi.n_terms; t++)
        if (m.yi.m_sum_ind[t] == ry.collect_ind[c])
          segs.push_back({ry.total_sum_ind[c], m.yi.i[t] * nlm_ + m.yi.y[t], ry.w_l_tile[c], m.yi.cg_coeff[t] * m.yi.inv_avg_n_neigh});
    for (size_t c = 0; c < r0.collect_ind.size(); c++)
      segs.push_back({r0.total_sum_ind[c], nI_ * nlm_ + r0.collect_ind[c], ry.w_shape + r0.w_l_tile[c], 1.0});
    typename DevJobs<T>::Host hf, hb;
    for (int fo = 0; fo < nB_; fo++) {
      hf.job(fo, 1.0);
      for (const Seg &s : segs)
        if (s.fo == fo) hf.seg(0, s.pair, s.tile, s.scale);
      hf.end_job();
    }
    for (int p = 0; p < nslot_ * nlm_; p++) {
      hb.job(p, 1.0);    // a job for every pair function, without segments when no term reads it: the launch writes all of gP
      for (const Seg &s : segs)
        if (s.pair == p) hb.seg(0, s.fo, s.tile, s.scale);
      hb.end_job();
    }
    jB_.build(hf, WB_.as<T>(), WB_.as<T>());
    jBb_.build(hb, WBT_.as<T>(), WBT_.as<T>());
    jB_.set_rows(drow_);
    jBb_.set_rows(drow_);
  }
  // ---- readout
  {
    en_.nlay = (int) m.energy_mlp.size();
    for (int L = 0; L < en_.nlay; L++) {
      upload_vec(eW_[L], m.energy_mlp[L].W);
      en_.W[L] = eW_[L].template as<double>();
      en_.norm[L] = m.energy_mlp[L].norm;
      en_.nin[L] = m.energy_mlp[L].n_in;
      en_.nout[L] = m.energy_mlp[L].n_out;
    }
    upload_vec(lnI_, m.I_nl_LN_scale);
    upload_vec(ln0_, m.I_0_LN_scale);
    en_.act = m.energy_mlp_activation;
    en_.ln = m.energy_mlp_ln;
    en_.nrho = nrho_;
    en_.width = nrho_;
    for (int L = 0; L < en_.nlay; L++) en_.width = std::max({en_.width, en_.nin[L], en_.nout[L]});
    en_.rms = m.energy_rms_norm;
    en_.eps = Model2L::rms_norm_eps;
    en_.out_scale = m.output_scale;
    en_.shift = shift_.as<double>();
    en_.lnI = lnI_.as<double>();
    en_.ln0 = ln0_.as<double>();
  }
}

template<class T> void Engine2L<T>::chain_forward(Chain<T> &c, const char *tag, const T *X)
{
  const int n = cn_, KP = c.kb * 16;
  const size_t na = cap_;
  c.X1.ensure(na * c.nf * KP * sizeof(T));
  c.XX.ensure(na * c.nXX * KP * sizeof(T));
  c.XX1.ensure(na * c.nXX * KP * sizeof(T));
  c.XXX.ensure(na * c.nXXX * KP * sizeof(T));
  if (c.order4) {
    c.XX2.ensure(na * c.nXX * KP * sizeof(T));
    c.XXXX.ensure(na * std::max(c.nXXXX, 1) * KP * sizeof(T));
  }
  int one = 1, nat = n;
  auto prod = [&](const std::string &name, DevProd &P, const T *L, const T *R, T *out, int sl, int sr) {
    if (P.jit.ok()) {
      stage(name.c_str(), [&] {
        void *args[] = {(void *) &L, (void *) &R, (void *) &out, (void *) &nat, (void *) &one};
        const long long cols = (long long) n * KP;
        HIP_CHECK(hipModuleLaunchKernel(P.jit.fwd, (unsigned) ((cols + 255) / 256), 1, 1, 256, 1, 1, 0, stream_, args, nullptr));
      });
      return;
    }
    const int AT = std::max(1, 256 / KP);
    stage(name.c_str(), [&] {
      hipLaunchKernelGGL(k_prod_fwd<T>, dim3(P.d.nout * 8 * (((n + AT - 1) / AT + 7) / 8)), dim3(KP * AT), 0, stream_, P.d, L, R, out, n, KP, sl, sr);
    });
  };
  T *X1 = c.X1.template as<T>(), *XX = c.XX.template as<T>(), *XX1 = c.XX1.template as<T>(), *XXX = c.XXX.template as<T>(),
    *XX2 = c.XX2.template as<T>(), *XXXX = c.XXXX.template as<T>();
  if (c.fused.ok()) {
    // X -> X1 -> XX -> XX1 / XX2 -> XXX / XXXX in one kernel; XX is written for the functions the reduces collect only
    stage(tagged(tag, "chain_fwd").c_str(), [&] {
      const T *w = c.fusedW.template as<T>();
      void *args[] = {(void *) &X, (void *) &X1, (void *) &XX, (void *) &XX1, (void *) &XX2, (void *) &XXX, (void *) &XXXX, (void *) &w, (void *) &nat,
                      (void *) &one};
      const unsigned blocks = (unsigned) ((n + c.fused.atoms_per_block - 1) / c.fused.atoms_per_block);
      HIP_CHECK(hipModuleLaunchKernel(c.fused.fwd, blocks, 1, 1, 256, 1, 1, 0, stream_, args, nullptr));
      cur_flops_ += c.fused.flops_per_atom * n;
    });
    if (!c.fuse3) prod(tagged(tag, "prod_3"), c.p3, XX1, X, XXX, c.nXX, c.nf);
    return;
  }
  stage(tagged(tag, "fc_1").c_str(), [&] { launch_gemm<T>(c.fc1.fwd, c.kb, c.kb, c.kb, X, c.nf, X, c.nf, X1, c.nf, 0, cur_tiles_, cur_ntiles_); });
  prod(tagged(tag, "prod_2"), c.p2, X1, X1, XX, c.nf, c.nf);
  stage(tagged(tag, "fc_2").c_str(), [&] { launch_gemm<T>(c.fc2.fwd, c.kb, c.kb, c.kb, XX, c.nXX, X, c.nf, XX1, c.nXX, 0, cur_tiles_, cur_ntiles_); });
  prod(tagged(tag, "prod_3"), c.p3, XX1, X, XXX, c.nXX, c.nf);
  if (c.order4) {
    stage(tagged(tag, "fc_3").c_str(), [&] { launch_gemm<T>(c.fc3.fwd, c.kb, c.kb, c.kb, XX, c.nXX, X, c.nf, XX2, c.nXX, 0, cur_tiles_, cur_ntiles_); });
    prod(tagged(tag, "prod_4"), c.p4, XX2, XX2, XXXX, c.nXX, c.nXX);
  }
}

template<class T> void Engine2L<T>::chain_zero(Chain<T> &c, const char *tag)
{
  const size_t nc = cap_, KP = c.kb * 16;
  if (c.fused.ok()) {
    // the reduces add their adjoints to gX, gXXX, gXXXX and to the collected rows of gXX; the chain kernel reads those rows
    // only and writes gX
    c.gX.ensure(nc * c.nf * KP * sizeof(T));
    c.gXX.ensure(nc * c.nXX * KP * sizeof(T));
    c.gXXX.ensure(nc * c.nXXX * KP * sizeof(T));
    if (c.order4) c.gXXXX.ensure(nc * std::max(c.nXXXX, 1) * KP * sizeof(T));
    if (!c.fuse3) c.gXX1.ensure(nc * c.nXX * KP * sizeof(T));
    const size_t na = (size_t) cn_;
    stage(tagged(tag, "zero_grads").c_str(), [&] {
      HIP_CHECK(hipMemsetAsync(c.gX.p, 0, na * c.nf * KP * sizeof(T), stream_));
      if (!c.fuse3 && !c.jit_all) HIP_CHECK(hipMemsetAsync(c.gXX1.p, 0, na * c.nXX * KP * sizeof(T), stream_));
      HIP_CHECK(hipMemsetAsync(c.gXXX.p, 0, na * c.nXXX * KP * sizeof(T), stream_));
      if (c.order4) HIP_CHECK(hipMemsetAsync(c.gXXXX.p, 0, na * std::max(c.nXXXX, 1) * KP * sizeof(T), stream_));
      const long long total = (long long) na * c.nkeepXX * (long long) KP;
      if (total > 0)
        hipLaunchKernelGGL(k_clear_functions<T>, dim3((unsigned) ((total + 255) / 256)), dim3(256), 0, stream_, c.gXX.template as<T>(), c.nXX, (int) KP,
                           c.keepXX.template as<int>(), c.nkeepXX, total);
    });
    return;
  }
  c.gX.ensure(nc * c.nf * KP * sizeof(T));
  c.gX1.ensure(nc * c.nf * KP * sizeof(T));
  c.gXX.ensure(nc * c.nXX * KP * sizeof(T));
  c.gXX1.ensure(nc * c.nXX * KP * sizeof(T));
  c.gXXX.ensure(nc * c.nXXX * KP * sizeof(T));
  if (c.order4) {
    c.gXX2.ensure(nc * c.nXX * KP * sizeof(T));
    c.gXXXX.ensure(nc * std::max(c.nXXXX, 1) * KP * sizeof(T));
  }
  const size_t na = (size_t) cn_;
  stage(tagged(tag, "zero_grads").c_str(), [&] {
    HIP_CHECK(hipMemsetAsync(c.gX.p, 0, na * c.nf * KP * sizeof(T), stream_));
    HIP_CHECK(hipMemsetAsync(c.gX1.p, 0, na * c.nf * KP * sizeof(T), stream_));
    // gXX is not filled: the FC reverse writes every row of it, and the reduces add their XX parts afterwards
    // with the specialised product kernels gXX1 and gXX2 are written (not accumulated) by their producer
    if (!c.jit_all) HIP_CHECK(hipMemsetAsync(c.gXX1.p, 0, na * c.nXX * KP * sizeof(T), stream_));
    HIP_CHECK(hipMemsetAsync(c.gXXX.p, 0, na * c.nXXX * KP * sizeof(T), stream_));
    if (c.order4) {
      if (!c.jit_all) HIP_CHECK(hipMemsetAsync(c.gXX2.p, 0, na * c.nXX * KP * sizeof(T), stream_));
      HIP_CHECK(hipMemsetAsync(c.gXXXX.p, 0, na * std::max(c.nXXXX, 1) * KP * sizeof(T), stream_));
    }
  });
}

// reverse of the chain; the reduces have added their adjoints to gXXX and gXXXX.  The FC reverse WRITES gXX (no fill, no
// read of the largest adjoint); reduces_x_xx then adds the reduces' adjoints of X and XX.  Result in c.gX.
template<class T> void Engine2L<T>::chain_backward(Chain<T> &c, const char *tag, const T *X, const std::function<void()> &reduces_x_xx)
{
  const int n = cn_, KP = c.kb * 16;
  int one = 1, nat = n;
  auto prod_bwd = [&](const std::string &name, DevProd &P, const T *L, const T *R, const T *g, T *gL, T *gR, int sl, int sr, int accL, int accR) {
    if (P.jit.ok()) {
      if (!c.jit_all) accL = accR = 1;
      stage(name.c_str(), [&] {
        void *args[] = {(void *) &L, (void *) &R, (void *) &g, (void *) &gL, (void *) &gR, (void *) &accL, (void *) &accR, (void *) &nat, (void *) &one};
        const long long cols = (long long) n * KP;
        HIP_CHECK(hipModuleLaunchKernel(P.jit.bwd, (unsigned) ((cols + 255) / 256), 1, 1, 256, 1, 1, 0, stream_, args, nullptr));
      });
      return;
    }
    const int AT = std::max(1, 256 / KP);
    stage(name.c_str(), [&] {
      hipLaunchKernelGGL(k_prod_bwd<T>, dim3(P.d.nleft * 8 * (((n + AT - 1) / AT + 7) / 8)), dim3(KP * AT), 0, stream_, P.d, 0, R, g, gL, n, KP, sr, sl);
      hipLaunchKernelGGL(k_prod_bwd<T>, dim3(P.d.nright * 8 * (((n + AT - 1) / AT + 7) / 8)), dim3(KP * AT), 0, stream_, P.d, 1, L, g, gR, n, KP, sl, sr);
    });
  };
  auto fc_bwd = [&](const std::string &name, DevFc<T> &F, const T *g, T *gXl, T *gXr, int nfl, int acc_left) {
    stage(name.c_str(), [&] {
      if (F.have_lr && gXl == gXr && nfl == c.nf && acc_left) {
        launch_gemm<T>(F.bwd_lr, c.kb, c.kb, c.kb, g, nfl, g, nfl, gXl, nfl, 1, cur_tiles_, cur_ntiles_);
        return;
      }
      launch_gemm<T>(F.bwd_l, c.kb, c.kb, c.kb, g, nfl, g, nfl, gXl, nfl, acc_left, cur_tiles_, cur_ntiles_);
      launch_gemm<T>(F.bwd_r, c.kb, c.kb, c.kb, g, nfl, g, nfl, gXr, c.nf, 1, cur_tiles_, cur_ntiles_);
    });
  };
  const T *X1 = c.X1.template as<T>(), *XX1 = c.XX1.template as<T>(), *XX2 = c.XX2.template as<T>();
  T *gX = c.gX.template as<T>(), *gX1 = c.gX1.template as<T>(), *gXX = c.gXX.template as<T>(), *gXX1 = c.gXX1.template as<T>(),
    *gXXX = c.gXXX.template as<T>(), *gXX2 = c.gXX2.template as<T>(), *gXXXX = c.gXXXX.template as<T>();
  if (c.fused.ok()) {
    reduces_x_xx();    // the adjoints the reduces leave on X and on the collected functions of XX come first
    if (!c.fuse3) prod_bwd(tagged(tag, "prod_3_bwd"), c.p3, XX1, X, gXXX, gXX1, gX, c.nXX, c.nf, 0, 1);
    stage(tagged(tag, "chain_bwd").c_str(), [&] {
      const T *w = c.fusedW.template as<T>(), *g2 = gXX, *g3 = gXXX, *g4 = gXXXX, *g21 = gXX1;
      void *args[] = {(void *) &X, (void *) &X1, (void *) &XX1, (void *) &XX2, (void *) &g2, (void *) &g3, (void *) &g4, (void *) &g21, (void *) &gX,
                      (void *) &w, (void *) &nat, (void *) &one};
      const unsigned blocks = (unsigned) ((n + c.fused.atoms_per_block - 1) / c.fused.atoms_per_block);
      HIP_CHECK(hipModuleLaunchKernel(c.fused.bwd, blocks, 1, 1, 256, 1, 1, 0, stream_, args, nullptr));
      cur_flops_ += c.fused.flops_per_atom * n;
    });
    return;
  }
  if (c.order4) prod_bwd(tagged(tag, "prod_4_bwd"), c.p4, XX2, XX2, gXXXX, gXX2, gXX2, c.nXX, c.nXX, 0, 0);
  prod_bwd(tagged(tag, "prod_3_bwd"), c.p3, XX1, X, gXXX, gXX1, gX, c.nXX, c.nf, 0, 1);
  if (c.order4) {
    // fc2 and fc3 share their inputs: one pass over gXX and gX for both
    stage(tagged(tag, "fc_23_bwd").c_str(), [&] {
      launch_gemm<T>(c.fc23.bwd_l, c.kb, c.kb, c.kb, gXX1, c.nXX, gXX2, c.nXX, gXX, c.nXX, 0, cur_tiles_, cur_ntiles_);
      launch_gemm<T>(c.fc23.bwd_r, c.kb, c.kb, c.kb, gXX1, c.nXX, gXX2, c.nXX, gX, c.nf, 1, cur_tiles_, cur_ntiles_);
    });
  } else {
    fc_bwd(tagged(tag, "fc_2_bwd"), c.fc2, gXX1, gXX, gX, c.nXX, 0);
  }
  reduces_x_xx();
  prod_bwd(tagged(tag, "prod_2_bwd"), c.p2, X1, X1, gXX, gX1, gX1, c.nf, c.nf, 1, 1);
  fc_bwd(tagged(tag, "fc_1_bwd"), c.fc1, gX1, gX, gX, c.nf, 1);
}

template<class T> void Engine2L<T>::reduce_fwd(DevReduce<T> &R, int kb, const Chain<T> &c, const T *X, double *out)
{
  const int *tiles = cur_tiles_;
#define GR_RED(KA) hipLaunchKernelGGL((k_reduce_fwd<T, KA, KA>), dim3(cur_ntiles_), dim3(64 * kReduceWaves), 0, stream_, R.d, mu_.as<int>() + a0_, tiles, \
                                      c.src(0, X), c.src(1, X), c.src(2, X), c.src(3, X), out)
  switch (kb) {
    case 1: GR_RED(1); break;
    case 2: GR_RED(2); break;
    case 4: GR_RED(4); break;
    default: throw Error("unsupported channel widths");
  }
#undef GR_RED
}

// high: the sources XXX and XXXX (before the chain's reverse reads their adjoints); else X and XX (after the FC reverse
// has written the adjoint of XX)
template<class T> void Engine2L<T>::reduce_bwd(DevReduce<T> &R, const Chain<T> &c, const double *g, bool high)
{
  const int low = R.d.ncol[0] + R.d.ncol[1], first = high ? low : 0, count = high ? R.njobs - low : low;
  if (count <= 0) return;
  hipLaunchKernelGGL(k_reduce_bwd<T>, dim3(cur_ntiles_, count), dim3(64), 0, stream_, R.d, mu_.as<int>() + a0_, cur_tiles_, g, c.gsrc(0), c.gsrc(1),
                     c.gsrc(2), c.gsrc(3), first);
}

template<class T> void Engine2L<T>::run(const RunFlags &fl)
{
  const int n = n_;
  ordered_check(fl);
  if (!begin_pass(fl)) return;
  const size_t ecap_all = (size_t) std::max<int64_t>(nb_, 1);
  const long long *n_edges = eoff_.as<long long>() + n;
  const bool forces = !fl.energy_only;
  if (ordered_ && forces) ordered_begin();
  // row of an edge: Y[nlm] and, for forces, the two tangential gradients D1[nlm], D2[nlm] and padding (pair_row_stride)
  const int yw = forces ? pair_row_stride(nlm_, sizeof(T)) : nlm_;
  YG_.ensure(ecap_all * yw * sizeof(T));
  stage("sh_edges", [&] {
    const size_t lds = (size_t) 64 * ((forces ? 3 * nlm_ : nlm_) + 1) * sizeof(T);
    auto kern = k_sh_edges<T>;
    if (lds > 48 * 1024) HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds));
    hipLaunchKernelGGL(kern, dim3((unsigned) ((ecap_all + 63) / 64)), dim3(64), lds, stream_, sh_, rh_.as<double>(), n_edges, nlm_, forces ? 1 : 0,
                       YG_.as<T>(), yw);
  });

  // ---- chunks of atoms.  Layer 2 gathers the messages of ALL atoms, so the pass is three sweeps over the chunks: layer 1
  // forward (the message rows of the chunk's atoms); layer 2 forward, the readout and layer 2 reverse (the message
  // adjoints, added to the rows of the neighbours); layer 1 reverse.  Kept for the whole structure: the harmonics and the
  // compact bonds, the message and its adjoint, rho and its adjoint.  Every other tensor, the radial rows of both layers
  // included, exists for one chunk; with more than one chunk the third sweep repeats the chunk's layer-1 forward pass
  // first (the reference's store_l1 = false, libgrace/include/grace/system.h:79-80).
  const double bonds_per_atom = (double) ecap_all / n;
  auto chain_values = [](const Chain<T> &c) {    // forward tensors and adjoints of a chain, values per atom
    return 2.0 * c.kb * 16 * (2.0 * c.nf + (c.order4 ? 3.0 : 2.0) * c.nXX + c.nXXX + (c.order4 ? std::max(c.nXXXX, 1) : 0));
  };
  const int npf = nslot_ * nlm_;
  const double per_atom = sizeof(T) * (chain_values(c1_) + chain_values(c2_) + (double) nlm_ * C1P_ + 2.0 * npf * CRP_ + (double) nB_ * C2P_ +
                                       bonds_per_atom * 2.0 * (radR_.noutp + radR1_.noutp)) +
                          (2.0 * nI1_ * PI1_ + 2.0 * nrho_) * sizeof(double) + 2.0 * nI1_ * PI1_ * (sizeof(T) == 4 ? 4.0 : 0.0);
  const double kept = bonds_per_atom * (60.0 + yw * sizeof(T)) + (double) (nslot_ + nI_) * CRP_ * sizeof(T) + 32.0 * nrho_ + 64.0;
  const int cs = plan_chunk(n, per_atom, kept);
  const int nchunks = (n + cs - 1) / cs;
  chunk_used_ = nchunks > 1 ? cs : 0;
  std::vector<long long> ebound;
  size_t ecap = ecap_all;
  cap_ = (size_t) round_up(cs, 16);    // the generated chain kernels run whole blocks of atoms: rows up to the end of the last block
  if (nchunks > 1) {
    layout_chunks(cs);
    ebound = chunk_edge_bounds(cs);
    ecap = 1;
    for (int q = 0; q < nchunks; q++) ecap = std::max(ecap, (size_t) (ebound[(size_t) q + 1] - ebound[(size_t) q]));
  }
  long long eb = 0, ecnt = -1;
  auto set_chunk = [&](int q) {
    if (nchunks == 1) {
      a0_ = 0; cn_ = n; eb = 0; ecnt = -1;
      cur_tiles_ = tiles_.as<int>(); cur_ntiles_ = ntiles_;
      return;
    }
    a0_ = q * cs;
    cn_ = std::min(n, a0_ + cs) - a0_;
    eb = ebound[(size_t) q];
    ecnt = ebound[(size_t) q + 1] - eb;
    cur_tiles_ = chunk_tiles_.as<int>() + (size_t) 16 * chunk_tile_off_[(size_t) q];
    cur_ntiles_ = chunk_tile_off_[(size_t) q + 1] - chunk_tile_off_[(size_t) q];
  };
  const size_t na = cap_, nnodes = (size_t) n_nodes_;

  // buffers of the whole structure
  rho_.ensure((size_t) n * nrho_ * sizeof(double));
  grho_.ensure((size_t) n * nrho_ * sizeof(double));
  M_.ensure(nnodes * nslot_ * CRP_ * sizeof(T));    // the message rows exist for the ghost atoms too: the exchange fills them
  T *M = M_.as<T>();
  if (fl.uq) {
    uq_gamma_.ensure((size_t) n * sizeof(double)); uq_sigma_.ensure((size_t) n * sizeof(double)); uq_cluster_.ensure((size_t) n * sizeof(double));
  }
  // buffers of a chunk
  // radial tables asked for: the A basis and the bond reverse of layer 1 evaluate them themselves, and the rows of R are
  // neither written nor read (GRACE_HIP_TABLE_ROWS=1: rows from the table kernel, as without tables).  The pair kernels of
  // layer 2 read the rows of R1 in either case.
  const char *rows_env = std::getenv("GRACE_HIP_TABLE_ROWS");
  const bool tab_inside = radR_.has_tables() && !(rows_env && rows_env[0] == '1') && nl_ * (C1P_ / 16) <= 10;
  if (!tab_inside) {
    Rz_.ensure(ecap * radR_.noutp * sizeof(T));
    dRz_.ensure(ecap * radR_.noutp * sizeof(T));
  }
  RadialTable<T> tbR{};
  if (tab_inside) tbR = radR_.table(stream_, ncu_, xr_.as<double>(), emu_.as<int>(), zA_.as<T>());
  A_.ensure(na * nlm_ * C1P_ * sizeof(T));
  T *A = A_.as<T>();
  if (I1_.bytes < na * nI1_ * PI1_ * sizeof(double)) {
    I1_.ensure(na * nI1_ * PI1_ * sizeof(double));
    HIP_CHECK(hipMemsetAsync(I1_.p, 0, I1_.bytes, stream_));    // the padding channels stay zero
  }
  if constexpr (sizeof(T) == 4) I1t_.ensure(na * nI1_ * PI1_ * sizeof(T));

  // layer 1 of the current chunk up to its chain (radial rows from row 0 of Rz_ / dRz_; kernels index bonds by their number
  // in the structure)
  auto layer1_chain = [&] {
    T *Rz = moved_back(Rz_.as<T>(), eb * radR_.noutp), *dRz = moved_back(dRz_.as<T>(), eb * radR_.noutp);
    if (!tab_inside)
      stage("radial_R", [&] { radR_.launch(stream_, ncu_, zA_.as<T>(), eb, ecnt, xr_.as<double>(), emu_.as<int>(), Rz, dRz, n_edges, nullptr, true); });
    ScatterArgs<T> sa{};
    sa.tb = tbR;
    sa.eoff = eoff_.as<long long>(); sa.rh = rh_.as<double>(); sa.Rz = Rz; sa.A = A;
    sa.a0 = a0_; sa.C = C1P_; sa.nl = nl_; sa.nlm = nlm_; sa.noutp = radR_.noutp; sa.sh = sh_;
    stage("scatter_A", [&] { launch_scatter<T>(sa, cn_, lmax_); });
    chain_forward(c1_, "_L1", A);
  };

  // ---- sweep 1: layer 1 forward
  for (int q = 0; q < nchunks; q++) {
    set_chunk(q);
    layer1_chain();
    stage("reduce_rho", [&] { reduce_fwd(redrho_, c1_.kb, c1_, A, rho_.as<double>() + (size_t) a0_ * nrho_); });
    stage("reduce_I1", [&] {
      for (auto &r : redI1_) reduce_fwd(*r, c1_.kb, c1_, A, I1_.as<double>());
    });
    // I1 leaves the scalar reduce in fp64; the fp32 engine hands the GEMM a copy in fp32
    const long long nI1v = (long long) cn_ * nI1_ * PI1_;
    const T *I1t = I1_.as<T>();
    if constexpr (sizeof(T) == 4) I1t = I1t_.as<T>();
    stage("reduce_I", [&] {
      if constexpr (sizeof(T) == 4)
        hipLaunchKernelGGL((k_convert<double, T>), dim3((unsigned) ((nI1v + 255) / 256)), dim3(256), 0, stream_, I1_.as<double>(), I1t_.as<T>(), nI1v);
      gemm(jI_, PI1_ / 16, CRP_ / 16, I1t, nI1_, M + (size_t) a0_ * nslot_ * CRP_, nslot_, 0);
    });
  }
  stage("fill_slot", [&] {
    hipLaunchKernelGGL(k_fill_slot<T>, dim3((unsigned) ((nnodes * CRP_ + 255) / 256)), dim3(256), 0, stream_, mu_.as<int>(), zB0_.as<T>(), M, n_nodes_,
                       nslot_, nI_, CRP_);
  });
  exchange_forward(1);

  // ---- sweep 2: layer 2 forward, readout, layer 2 reverse
  R1_.ensure(ecap * radR1_.noutp * sizeof(T));
  dR1_.ensure(ecap * radR1_.noutp * sizeof(T));
  P_.ensure(na * npf * CRP_ * sizeof(T));
  B_.ensure(na * nB_ * C2P_ * sizeof(T));
  I2_.ensure(na * nrho_ * sizeof(double));
  gI2_.ensure(na * nrho_ * sizeof(double));
  T *P = P_.as<T>(), *B = B_.as<T>();
  const int pthreads = round_up(nslot_ * CRP_, 64);
  // the pair kernels copy rows of CRP_ values and of noutp values to LDS 16 bytes at a time
  if ((CRP_ * sizeof(T)) % 16 || (radR1_.noutp * sizeof(T)) % 16) throw Error("GRACE-2L: pair kernels need rows that are multiples of 16 bytes");
  if (forces) {
    gP_.ensure(na * npf * CRP_ * sizeof(T));
    gM_.ensure(nnodes * nI_ * CRP_ * sizeof(T));
    if (ordered_) gMe_.ensure(ecap * nI_ * CRP_ * sizeof(T));
    stage("zero_gM", [&] { HIP_CHECK(hipMemsetAsync(gM_.p, 0, nnodes * nI_ * CRP_ * sizeof(T), stream_)); });
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
  for (int q = 0; q < nchunks; q++) {
    set_chunk(q);
    const int nc = cn_;
    const long long *eoff = eoff_.as<long long>() + a0_;
    const int *mu = mu_.as<int>() + a0_;
    T *R1 = moved_back(R1_.as<T>(), eb * radR1_.noutp), *dR1 = moved_back(dR1_.as<T>(), eb * radR1_.noutp);
    stage("radial_R1", [&] { radR1_.launch(stream_, ncu_, ones_.as<T>(), eb, ecnt, xr_.as<double>(), emu_.as<int>(), R1, dR1, n_edges, nullptr, true); });
    stage("pair_fwd", [&] {
      const size_t lds = (size_t) 2 * kAsyncChunkFwd * (pthreads + radR1_.noutp) * sizeof(T);
      GR_PAIR(k_pair_fwd, dim3(nc), dim3(pthreads), lds, stream_, eoff, ej_.as<int>(), YG_.as<T>(), (const T *) R1, (const T *) M, P, nslot_, CRP_,
              nl_, radR1_.noutp, yw, sink_.as<T>(), 0, nc, nslot_);
    });
    stage("reduce_B", [&] { gemm(jB_, CRP_ / 16, C2P_ / 16, P, npf, B, nB_, 0); });
    chain_forward(c2_, "_L2", B);
    stage("reduce_I2", [&] { reduce_fwd(redI2_, c2_.kb, c2_, B, I2_.as<double>()); });
    if (fl.uq) {
      if (nchunks > 1) layer1_chain();    // the head reads layer 1's tensors of these atoms as well
      stage("uq", [&] {
        UqDev<T> u = uq_;
        for (int k = 0; k < u.nsrc; k++) u.X[k] = u.blk[k] == 0 ? c2_.src(k, B) : c1_.src(k - u.nsrc / 2, A);
        const size_t lds = (size_t) (u.d_basis + 4 * u.rp + 2 * u.D) * sizeof(double);
        auto kern = k_uq<T>;
        if (lds > 48 * 1024)
          HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds));
        hipLaunchKernelGGL(kern, dim3(nc), dim3(256), lds, stream_, u, mu, nc, uq_gamma_.as<double>() + a0_, uq_sigma_.as<double>() + a0_,
                           uq_cluster_.as<double>() + a0_);
      });
      ran_uq_ = true;
    }
    stage("energy_mlp", [&] {
      hipLaunchKernelGGL(k_energy_2l, dim3(nc), dim3(64), (size_t) (2 * en_.nlay + 4) * en_.width * sizeof(double), stream_, en_, mu, nc,
                         (const double *) rho_.as<double>() + (size_t) a0_ * nrho_, (const double *) I2_.as<double>(),
                         grho_.as<double>() + (size_t) a0_ * nrho_, gI2_.as<double>(), fl.eatom || ordered_ ? eatom_.as<double>() + a0_ : nullptr,
                         ordered_ ? nullptr : scal_.as<double>(), forces ? 1 : 0, sid_ptr() ? sid_ptr() + a0_ : nullptr);
    });
    if (!forces) continue;
    // layer 2 reverse: dE/dB -> dE/dP -> bond forces of layer 2 and dE/dI of the neighbours
    chain_zero(c2_, "_L2");
    stage("reduce_I2_bwd", [&] { reduce_bwd(redI2_, c2_, gI2_.as<double>(), true); });
    chain_backward(c2_, "_L2", B, [&] { stage("reduce_I2_bwd_X_XX", [&] { reduce_bwd(redI2_, c2_, gI2_.as<double>(), false); }); });
    stage("reduce_B_bwd", [&] { gemm(jBb_, C2P_ / 16, CRP_ / 16, c2_.gX.template as<T>(), nB_, gP_.as<T>(), npf, 0); });    // gP: every row is written
    stage("pair_bwd", [&] {
      // fp32: the next chunk is copied to a second LDS buffer while this one is worked on (chunks of 8 bonds in the large
      // blocks that fill a CU alone, of 4 otherwise); fp64 runs faster with one chunk staged through registers
      const size_t row = (size_t) (pthreads + 2 * radR1_.noutp) * sizeof(T);
      const int ch = sizeof(T) != 4 ? 0 : (pthreads >= 512 && 16 * row <= kPairLdsMax) ? 8 : 8 * row <= kPairLdsMax ? 4 : 0;
      const size_t lds = ch && !ordered_ ? 2 * ch * row : kPairChunk * row;
#define GR_ARGS_ASYNC                                                                                                                   \
  dim3(nc), dim3(pthreads), lds, stream_, eoff, ej_.as<int>(), YG_.as<T>(), (const T *) R1, (const T *) dR1, (const T *) M, (const T *) gP_.as<T>(),        \
      rh_.as<double>(), r_.as<double>(), rc_.as<double>(), gM_.as<T>(), f_.as<double>(), scal_.as<double>() + 1, nslot_, nI_, CRP_, nl_, radR1_.noutp, \
      sink_.as<T>(), 1, sid_ptr(), nslot_, 0, nc, a0_, vatom_ptr(), yw
#define GR_ARGS GR_ARGS_ASYNC, po
      // ordered sums: the staged kernel without atomics; the message adjoints of the chunk's bonds are gathered afterwards
      PairOrdered<T> po{};
      if (ordered_) {
        po.gMe = gMe_.as<T>(); po.fedge = fedge_.as<double>(); po.fcen = fcen_.as<double>(); po.e_base = eb; po.ngrp = 1;
      }
      const PairMfmaPlan mp = pair_mfma_plan(nslot_, CRP_, nl_, sizeof(T), pair_mfma_waves(sizeof(T), pair_waves_));
      if (!ordered_ && mp.ok && pair_mfma_ != 0) {
        PairMfmaArgs<T> pa{};
        pa.eoff = eoff; pa.ej = ej_.as<int>(); pa.YG = YG_.as<T>(); pa.R1 = R1; pa.dR1 = dR1; pa.M = M; pa.gP = gP_.as<T>();
        pa.rh = rh_.as<double>(); pa.rlen = r_.as<double>(); pa.rcut = rc_.as<double>();
        pa.gM = gM_.as<T>(); pa.f = f_.as<double>(); pa.virial = scal_.as<double>() + 1; pa.vatom = vatom_ptr(); pa.sid = sid_ptr();
        pa.nslot = nslot_; pa.nI = nI_; pa.C = CRP_; pa.noutp = radR1_.noutp; pa.natoms = nc; pa.a0 = a0_;
        for (int q = 0; q < 16; q++) pa.drow[q] = drow_[q];
        launch_pair_bwd_mfma(mp, pa, nl_, stream_);
      } else if (ordered_) {
        GR_PAIR_ORD(GR_ARGS)
      } else if (ch == 8) {
        GR_PAIR_ASYNC(8, GR_ARGS_ASYNC)
      } else if (ch == 4) {
        GR_PAIR_ASYNC(4, GR_ARGS_ASYNC)
      } else {
        GR_PAIR(k_pair_bwd, GR_ARGS)
      }
#undef GR_ARGS
#undef GR_ARGS_ASYNC
    });
    if (ordered_)
      stage("ordered_gM", [&] {
        hipLaunchKernelGGL(k_ordered_gm<T>, dim3((unsigned) n_nodes_), dim3(std::min(1024, round_up(nI_ * CRP_, 64))), 0, stream_, toff_.as<long long>(),
                           tsorted_.as<int>(), (const T *) gMe_.as<T>(), eb, n_edges, ecnt, nI_ * CRP_, gM_.as<T>());
      });
  }
#undef GR_PAIR_ASYNC
#undef GR_PAIR_ASYNC1
#undef GR_PAIR_ORD
#undef GR_PAIR_ORD1
#undef GR_PAIR
#undef GR_PAIR1
  if (!forces) {
    set_chunk(0);
    if (ordered_) ordered_finish(fl);
    return;
  }
  exchange_reverse(1);

  // ---- sweep 3: layer 1 reverse
  gI1_.ensure(na * nI1_ * PI1_ * sizeof(double));
  if constexpr (sizeof(T) == 4) gI1t_.ensure(na * nI1_ * PI1_ * sizeof(T));
  for (int q = 0; q < nchunks; q++) {
    set_chunk(q);
    if (nchunks > 1) layer1_chain();
    const long long nI1v = (long long) cn_ * nI1_ * PI1_;
    const T *gMc = gM_.as<T>() + (size_t) a0_ * nI_ * CRP_;
    const double *grho = grho_.as<double>() + (size_t) a0_ * nrho_;
    chain_zero(c1_, "_L1");
    stage("reduce_I_bwd", [&] {
      if constexpr (sizeof(T) == 4) {
        gemm(jIb_, CRP_ / 16, PI1_ / 16, gMc, nI_, gI1t_.as<T>(), nI1_, 0);
        hipLaunchKernelGGL((k_convert<T, double>), dim3((unsigned) ((nI1v + 255) / 256)), dim3(256), 0, stream_, gI1t_.as<T>(), gI1_.as<double>(), nI1v);
      } else {
        gemm(jIb_, CRP_ / 16, PI1_ / 16, gMc, nI_, gI1_.as<T>(), nI1_, 0);
      }
    });
    stage("reduce_rho_bwd", [&] { reduce_bwd(redrho_, c1_, grho, true); });
    stage("reduce_I1_bwd", [&] {
      for (auto &r : redI1_) reduce_bwd(*r, c1_, gI1_.as<double>(), true);
    });
    chain_backward(c1_, "_L1", A, [&] {
      stage("reduce_rho_bwd_X_XX", [&] { reduce_bwd(redrho_, c1_, grho, false); });
      stage("reduce_I1_bwd_X_XX", [&] {
        for (auto &r : redI1_) reduce_bwd(*r, c1_, gI1_.as<double>(), false);
      });
    });
    BondBwdArgs<T> ba{};
    ba.eoff = eoff_.as<long long>(); ba.ej = ej_.as<int>(); ba.rh = rh_.as<double>(); ba.r = r_.as<double>(); ba.rc = rc_.as<double>();
    ba.Rz = moved_back(Rz_.as<T>(), eb * radR_.noutp); ba.dRz = moved_back(dRz_.as<T>(), eb * radR_.noutp); ba.gA = c1_.gX.template as<T>();
    ba.f = f_.as<double>(); ba.virial = scal_.as<double>() + 1; ba.sid = sid_ptr(); ba.vatom = vatom_ptr();
    ba.tb = tbR;
    ba.a0 = a0_; ba.C = C1P_; ba.nl = nl_; ba.nlm = nlm_; ba.noutp = radR_.noutp; ba.sh = sh_;
    if (ordered_) {    // added to what the pair kernel of layer 2 stored for the same bonds and atoms
      ba.fedge = fedge_.as<double>(); ba.fcen = fcen_.as<double>(); ba.ordered_add = 1;
    }
    stage("bond_bwd", [&] { launch_bond_bwd<T>(ba, cn_); });
  }
  set_chunk(0);
  if (ordered_) ordered_finish(fl);
}

}    // namespace

std::unique_ptr<Engine> make_engine_2l(std::shared_ptr<const Model2L> model, int ntypes, const std::vector<int> &type2mu, int precision,
                                       int device)
{
  if (precision == 64) return std::make_unique<Engine2L<double>>(std::move(model), ntypes, type2mu, device);
  if (precision == 32) return std::make_unique<Engine2L<float>>(std::move(model), ntypes, type2mu, device);
  throw InvalidArgument("precision must be 64 or 32");
}

}    // namespace grhip
