// GRACE-1L engine for gfx950: device tables built from the model, and the staged pass over a CSR structure.
// Driver skeleton after libgrace/src/fused_1l.cpp:474-582 (type map, bond filter, forward, readout, reverse, forces)
// and the staged GPU pipeline of libgrace/include/grace/kk/grace_1l_kk.h:449-454; liveness pruning of FC outputs and
// CG terms after libgrace/src/fused_1l.cpp:176-216.
#include "engine_common.hpp"
#include "jit_chain.hpp"

#include <mutex>

namespace grhip {

namespace {

// ---------------------------------------------------------------------------------------------------------------
// Fixed device memory of the radial call that allocates nothing (radial_noalloc): a header (error flag), the checked
// neighbour elements and the padded rows the radial kernel writes.  Every GPU the library runs on holds its own copy
// of the array until the process ends.  In host code the array's name is only a handle for hipGetSymbolAddress: the
// address of a device's copy is looked up once per device (with that device current, when the first GRACE-1L engine
// of the device is built) and kept in scratch_ptr; host code uses that pointer and never the name.
// ---------------------------------------------------------------------------------------------------------------
constexpr size_t kScratchBytes = (size_t) 32 << 20;
constexpr size_t kScratchHeader = 256;
constexpr int kScratchMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
static void *scratch_ptr[kScratchMaxDevices] = {};
static std::mutex scratch_mutex;
// one call at a time per GPU uses the array: held by radial_noalloc from its first launch until its results are written
static std::mutex scratch_in_use[kScratchMaxDevices];

// address of the current device's copy of `scratch`
static unsigned char *scratch_of_device(int device)
{
  if (device < 0 || device >= kScratchMaxDevices) throw Error("device index " + std::to_string(device) + " out of range");
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (!scratch_ptr[device]) {
    void *p = nullptr;
    HIP_CHECK(hipSetDevice(device));
    HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) throw Error("hipGetSymbolAddress gave no address for the library's fixed device array");
    scratch_ptr[device] = p;
  }
  return static_cast<unsigned char *>(scratch_ptr[device]);
}

// neighbour elements of the caller checked into the fixed array: an element outside 0 .. nel-1 is replaced by 0 (so that
// the radial kernel stays inside its tables) and reported through *bad
static __global__ void k_stage_elements(const int *mu, int m, int nel, int *out, int *bad)
{
  const int q = blockIdx.x * blockDim.x + threadIdx.x;
  if (q >= m) return;
  const int v = mu[q];
  const bool ok = v >= 0 && v < nel;
  out[q] = ok ? v : 0;
  if (!ok) atomicMax(bad, 1);
}
// the flag starts at zero on every call (a fill kernel: a memset node would not survive a graph capture by the caller)
static __global__ void k_clear_flag(int *bad)
{
  if (threadIdx.x == 0 && blockIdx.x == 0) *bad = 0;
}
// padded rows [m][noutp] (column l * CP + n) -> caller's [m][nl][C] doubles
template<class T> static __global__ void k_unpack_radial(const T *R, const T *dR, long long total, int nl, int C, int CP, int noutp, double *oR, double *odR)
{
  for (long long i = blockIdx.x * (long long) blockDim.x + threadIdx.x; i < total; i += (long long) gridDim.x * blockDim.x) {
    const long long q = i / (nl * C);
    const int rest = (int) (i - q * (nl * C)), l = rest / C, n = rest - l * C;
    const long long src = q * noutp + l * CP + n;
    oR[i] = (double) R[src];
    odR[i] = (double) dR[src];
  }
}

template<class T> class Engine1L final : public EngineBase {
 public:
  Engine1L(std::shared_ptr<const Model1L> m, int ntypes, const std::vector<int> &type2mu, int device) :
      EngineBase(device, "GRACE-1L", ntypes, type2mu, m->n_elements), model_(std::move(m))
  {
    this->template probe_mfma_both<T>();
    chunks_ = true;
    ordered_ok_ = true;
    if (const char *e = std::getenv("GRACE_HIP_TABLE_ROWS")) tables_inside_ = !(e[0] == '1');
    build();
    scratch_dev_ = scratch_of_device(device);    // set-up: the device is current (EngineBase)
    end_build();    // buffers allocated from here on are work buffers (release_buffers)
  }

  ~Engine1L() override { chain_.release(); }
  int layers() const override { return 1; }
  void run(const RunFlags &fl) override;
  void debug_radial(int m, const double *x, const int *mu_j, double *Rz, double *dRz) override;
  void radial_noalloc(int m, const double *x, const int *mu_j, double *Rz, double *dRz) override;

 private:
  unsigned char *scratch_dev_ = nullptr;    // this device's copy of the fixed array (hipGetSymbolAddress)
  std::shared_ptr<const Model1L> model_;
  bool jit_all_ = false;

  // model dimensions
  int CP_ = 0, CFP_ = 0;    // channel widths padded to 16 / 32 / 64: the widths of every per-atom tensor on the device
  int lmax_ = 0, nl_ = 0, nlm_ = 0, C_ = 0, CF_ = 0, nAA_ = 0, nAAA_ = 0, nAAAA_ = 0, nrho_ = 0, nel_ = 0;
  bool order4_ = true, aaa_a_ = false;
  int noutp_ = 0;
  ShCoef sh_{};

  // device tables
  DevBuf z_, shift_;
  DevRadial<T> rad_;
  DevFc<T> fcA1_, fcAA1_, fcAA2_;
  DevFcPairBwd<T> fcAA12_;    // reverse of fc_AA1 and fc_AA2 in one pass over their shared inputs (models with the AAAA stage)
  DevProd pAA_, pAAA_, pAAAA_;
  // the whole chain A -> A1 -> AA -> AA1 / AA2 -> AAA / AAAA as one generated kernel per direction (jit_chain.hpp); not
  // ok(): the stage-by-stage kernels above run
  ChainKernels chain_;
  DevBuf chainW_;
  std::string chain_note_;
  bool tables_inside_ = true;  // radial tables evaluated by the kernels that use the radial functions
  bool red_writes_ = false;    // the reverse of the rho reduce may overwrite the adjoints (every function collected at most once)
  DevReduce<T> redrho_;
  UqDev<T> uq_{};             // UQ head (models that carry a valid one)
  DevBuf uqR_, uqCen_, uqIcov_, uqNcl_, uqThr_, uqCi_[4];
  DevBuf eW_[7];
  EnergyDev en_{};

  // pass buffers
  DevBuf Rz_, dRz_;
  DevBuf A_, A1_, AA_, AA1_, AA2_, AAA_, AAAA_, gA_, gA1_, gAA_, gAA1_, gAA2_, gAAA_, gAAAA_, rho_, grho_;

  void build();
  // the atom tiles of the chunk that is being evaluated (all atoms when there is one chunk)
  const int *cur_tiles_ = nullptr;
  int cur_ntiles_ = 0;
  void run_chunk(const RunFlags &fl, int a0, int nc, long long e_begin, long long e_count);
  void launch_gemm(DevJobs<T> &J, int kb0, int kb1, int nb, const T *X0, int nf0, const T *X1, int nf1, T *out, int nfo, int accumulate)
  {
    EngineBase::launch_gemm<T>(J, kb0, kb1, nb, X0, nf0, X1, nf1, out, nfo, accumulate, cur_tiles_, cur_ntiles_);
  }
  void launch_radial(long long e_begin, long long e_count, const double *x, const int *emu, T *Rz, T *dRz,
                     const long long *n_edges, bool tables = false);
  void apply_spline(int n) override { rad_.spline_n = n; }
};

template<class T> void Engine1L<T>::build()
{
  const Model1L &m = *model_;
  lmax_ = m.lmax;
  if (lmax_ > kKernMaxL) throw Error("GRACE-1L: lmax > " + std::to_string(kKernMaxL) + " not supported");
  nl_ = lmax_ + 1;
  nlm_ = nl_ * nl_;
  C_ = m.nradmax;
  CF_ = m.fc_A1.n_out;
  nel_ = m.n_elements;
  order4_ = m.max_order == 4;
  aaa_a_ = m.AAA_right_A;
  nrho_ = m.rho_n_out;
  if (nrho_ > 32) throw Error("GRACE-1L: rho_n_out > 32 not supported by the GPU reduce kernels");
  auto pad_width = [](int c) { return c <= 16 ? 16 : c <= 32 ? 32 : c <= 64 ? 64 : -1; };
  CP_ = pad_width(C_);
  CFP_ = pad_width(CF_);
  // the same limit as the reference's fused GPU engines (FC widths up to 64)
  if (CP_ < 0 || CFP_ < 0) throw Error("GRACE-1L: channel widths above 64 are not supported by the GPU kernels");
  nAA_ = m.prod_AA.n_out;
  nAAA_ = m.prod_AAA.n_out;
  nAAAA_ = order4_ ? m.prod_AAAA.n_out : 0;

  // ---- spherical harmonics coefficients (fused_cpu.h:686-704)
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

  // ---- pair cutoffs and species weights z[mu][n] (fused_1l.cpp:150-162)
  {
    std::vector<double> cut((size_t) nel_ * nel_);
    for (int a = 0; a < nel_; a++)
      for (int b = 0; b < nel_; b++) cut[(size_t) a * nel_ + b] = m.pair_cutoff(a, b);
    set_cutoffs(cut);
    std::vector<T> z((size_t) nel_ * CP_, (T) 0);
    for (int mu = 0; mu < nel_; mu++)
      for (int n = 0; n < C_; n++) {
        double v = 0.0;
        for (int e = 0; e < m.embedding_size; e++)
          v += m.A_lin_transform_W[(size_t) e * C_ + n] * m.chem_embedding[(size_t) mu * m.embedding_size + e];
        z[(size_t) mu * CP_ + n] = (T) (v * m.A_lin_transform_norm * m.A_inv_avg_n_neigh);
      }
    upload_vec(z_, z);
    upload_vec(shift_, m.shift_values);
  }

  // ---- radial MLP in MFMA fragment order
  rad_.build(m.mlp_rad, m.nradbase, m.radial_basis_p, m.radial_activation, C_, CP_, nl_, nel_, drow_, "GRACE-1L");
  rad_.build_double(m.mlp_rad, m.nradbase, m.radial_basis_p, m.radial_activation, C_, CP_, nl_, nel_, drow64_, "GRACE-1L");
  noutp_ = rad_.noutp;

  // ---- liveness, products, FCs (fused_1l.cpp:176-216)
  {
    auto collected = [](const ReduceWeights &r, int nf) {
      std::vector<char> v(nf, 0);
      for (int c : r.collect_ind) v[c] = 1;
      return v;
    };
    std::vector<char> needAAA = collected(m.red_AAA, nAAA_);
    HostProd hAAA = build_prod(m.prod_AAA, needAAA, nAA_, nlm_);
    std::vector<char> liveAA1(nAA_, 0), liveAA2(nAA_, 0), liveA1(nlm_, 0);
    for (int q : hAAA.l) liveAA1[q] = 1;
    if (!aaa_a_) for (int q : hAAA.r) liveA1[q] = 1;
    HostProd hAAAA;
    if (order4_) {
      std::vector<char> needAAAA = collected(m.red_AAAA, nAAAA_);
      hAAAA = build_prod(m.prod_AAAA, needAAAA, nAA_, nAA_);
      for (int q : hAAAA.l) liveAA2[q] = 1;
      for (int q : hAAAA.r) liveAA2[q] = 1;
    }
    std::vector<char> needAA = collected(m.red_AA, nAA_);
    for (int q = 0; q < nAA_; q++) needAA[q] = needAA[q] || liveAA1[q] || liveAA2[q];
    HostProd hAA = build_prod(m.prod_AA, needAA, nlm_, nlm_);
    for (int q : hAA.l) liveA1[q] = 1;
    for (int q : hAA.r) liveA1[q] = 1;
    pAA_.build(hAA);
    pAAA_.build(hAAA);
    if (order4_) pAAAA_.build(hAAAA);
    {
      const bool f32 = sizeof(T) == 4;
      jit_compile_product("prod_AA", hAA.terms, nlm_, nlm_, nAA_, true, CFP_, f32, arch_, pAA_.jit, pAA_.jit_note);
      if (!(aaa_a_ && CP_ != CFP_))
        jit_compile_product("prod_AAA", hAAA.terms, nAA_, nlm_, nAAA_, false, CFP_, f32, arch_, pAAA_.jit, pAAA_.jit_note);
      if (order4_) jit_compile_product("prod_AAAA", hAAAA.terms, nAA_, nAA_, nAAAA_, true, CFP_, f32, arch_, pAAAA_.jit, pAAAA_.jit_note);
      jit_all_ = pAA_.jit.ok() && pAAA_.jit.ok() && (!order4_ || pAAAA_.jit.ok());
    }
    // ---- the fused chain (same liveness, same pruned term lists)
    if (CP_ == CFP_ && !(aaa_a_ && CP_ != CFP_)) {
      ChainSpec sp;
      sp.C = CFP_;
      sp.f32 = sizeof(T) == 4;
      sp.nf0 = nlm_;
      sp.fc1 = chain_fc_spec(m.fc_A1, liveA1, nlm_);
      sp.nP2 = nAA_;
      sp.prod2 = hAA.terms;
      sp.fc21 = chain_fc_spec(m.fc_AA1, liveAA1, nlm_);
      sp.have22 = order4_;
      if (order4_) sp.fc22 = chain_fc_spec(m.fc_AA2, liveAA2, nlm_);
      sp.nP3 = nAAA_;
      sp.prod3 = hAAA.terms;
      sp.prod3_right_x0 = aaa_a_;
      sp.nP4 = nAAAA_;
      if (order4_) sp.prod4 = hAAAA.terms;
      sp.keepP2 = collected(m.red_AA, nAA_);
      sp.keepX0 = collected(m.red_A, nlm_);
      for (int q = 0; q < 16; q++) sp.drow[q] = drow_[q];
      std::vector<double> w;
      if (jit_compile_chain("chain_1l", sp, arch_, chain_, w, chain_note_)) {
        std::vector<T> wt(w.begin(), w.end());
        upload_vec(chainW_, wt);
      } else {
        log_message(1, "GRACE-1L: the dense chain runs stage by stage (" + chain_note_ + ")");
      }
      // the reverse of the rho reduce may write its rows instead of adding to cleared ones when no function is collected twice
      red_writes_ = true;
      for (const ReduceWeights *rw : {&m.red_A, &m.red_AA, &m.red_AAA, &m.red_AAAA}) {
        std::set<int> seen;
        for (int c : rw->collect_ind) red_writes_ = red_writes_ && seen.insert(c).second;
      }
    }
    fcA1_.build(m.fc_A1, liveA1, nlm_, CP_, CP_, CFP_, drow_, false, true);    // both inputs are A: one reverse launch
    fcAA1_.build(m.fc_AA1, liveAA1, nlm_, CFP_, CP_, CFP_, drow_);
    if (order4_) {
      fcAA2_.build(m.fc_AA2, liveAA2, nlm_, CFP_, CP_, CFP_, drow_);
      fcAA12_.build(m.fc_AA1, liveAA1, fcAA1_, m.fc_AA2, liveAA2, fcAA2_, nlm_, drow_, true);
    }
  }

  // ---- rho reduce: weights per collected function in MFMA fragment order (fused_cpu.h:1202-1273)
  {
    const ReduceWeights *rw[4] = {&m.red_A, &m.red_AA, &m.red_AAA, &m.red_AAAA};
    const int nfun[4] = {nlm_, nAA_, nAAA_, nAAAA_};
    std::vector<ReduceSrc> src;
    for (int s = 0; s < (order4_ ? 4 : 3); s++)
      src.push_back({&rw[s]->W, rw[s]->norm, rw[s]->n_in, rw[s]->w_shape, &rw[s]->collect_ind, &rw[s]->w_l_tile, nullptr, nfun[s],
                     s == 0 ? CP_ : CFP_});
    redrho_.build(src, nel_, nrho_, -1, nrho_, 0, drow_);
  }

  // ---- UQ head: a head that does not validate leaves the model usable without UQ (libgrace/src/model_1l.cpp:216-271)
  if (m.uq.has_uq) {
    try {
      m.validate_uq();
      if (m.uq.rp_dim > 256 || m.uq.feature_dim > 256) throw Error("GRACE-1L UQ: feature widths above 256 are not supported");
      const ReduceWeights *rw[4] = {&m.red_A, &m.red_AA, &m.red_AAA, &m.red_AAAA};
      const int nfun[4] = {nlm_, nAA_, nAAA_, nAAAA_};
      uq_.nsrc = order4_ ? 4 : 3;
      int off = 0;
      for (int s = 0; s < uq_.nsrc; s++) {
        upload_vec(uqCi_[s], rw[s]->collect_ind);
        uq_.ci[s] = uqCi_[s].template as<int>();
        uq_.nfun[s] = nfun[s];
        uq_.cpad[s] = s == 0 ? CP_ : CFP_;
        uq_.nin[s] = rw[s]->n_in;
        uq_.nc[s] = (int) rw[s]->collect_ind.size();
        uq_.off[s] = off;
        uq_.blk[s] = 0;
        off += uq_.nin[s] * uq_.nc[s];
      }
      uq_.d_basis = off; uq_.row0 = 0; uq_.carry_in = uq_.carry_out = 0;
      uq_.nblk = 1;
      uq_.rp = m.uq.rp_dim; uq_.D = m.uq.feature_dim; uq_.K = m.uq.max_clusters;
      uq_.density_scale = m.uq.density_scale;
      upload_vec(uqR_, m.uq.rp_matrix); upload_vec(uqCen_, m.uq.centroids); upload_vec(uqIcov_, m.uq.inv_cov);
      upload_vec(uqNcl_, m.uq.n_clusters); upload_vec(uqThr_, m.uq.interp_thresholds);
      uq_.R = uqR_.template as<double>(); uq_.cen = uqCen_.template as<double>(); uq_.icov = uqIcov_.template as<double>();
      uq_.ncl = uqNcl_.template as<int>(); uq_.thr = uqThr_.template as<double>();
      if ((size_t) (uq_.d_basis + 4 * uq_.rp + 2 * uq_.D) * sizeof(double) > 150 * 1024) throw Error("GRACE-1L UQ: the basis does not fit the kernel's LDS");
      has_uq_head_ = true;
    } catch (const std::exception &e) {
      uq_why_ = e.what();
    }
  } else {
    uq_why_ = "the model file carries none";
  }

  // ---- energy MLP
  {
    en_.nlay = (int) m.energy_mlp.size();
    for (int L = 0; L < en_.nlay; L++) {
      upload_vec(eW_[L], m.energy_mlp[L].W);
      en_.W[L] = eW_[L].template as<double>();
      en_.norm[L] = m.energy_mlp[L].norm;
      en_.nin[L] = m.energy_mlp[L].n_in;
      en_.nout[L] = m.energy_mlp[L].n_out;
    }
    en_.act = m.energy_mlp_activation;
    en_.ln = m.energy_mlp_ln;
    en_.nrho = nrho_;
    en_.width = nrho_;
    for (int L = 0; L < en_.nlay; L++) en_.width = std::max({en_.width, en_.nin[L], en_.nout[L]});
    en_.wlds = 0;
    for (int L = 0; L < en_.nlay; L++) en_.wlds += 2 * en_.nin[L] * en_.nout[L];
    if (en_.wlds > 4096) en_.wlds = 0;    // 32 kB: larger networks read their weights from global memory
    en_.out_scale = m.output_scale;
    en_.shift = shift_.as<double>();
  }
}

template<class T>
void Engine1L<T>::launch_radial(long long e_begin, long long e_count, const double *x, const int *emu, T *Rz, T *dRz,
                                const long long *n_edges, bool tables)
{
  rad_.launch(stream_, ncu_, z_.as<T>(), e_begin, e_count, x, emu, Rz, dRz, n_edges, nullptr, tables);
}

template<class T> void Engine1L<T>::run(const RunFlags &fl)
{
  const int n = n_;
  ordered_check(fl);
  if (!begin_pass(fl)) return;
  if (ordered_ && !fl.energy_only) ordered_begin();

  // ---- chunks of atoms: every stage after the bond filter acts on the atoms of a chunk and on their bonds only, so the
  // radial rows and the per-atom tensors are sized for one chunk; forces, per-atom energies and the compact bonds are
  // kept for the whole structure
  const double bonds_per_atom = (double) std::max<int64_t>(nb_, 1) / n;
  const double per_atom = sizeof(T) * (2.0 * nlm_ * CP_ + (double) CFP_ * (2.0 * nlm_ + (order4_ ? 6.0 : 4.0) * nAA_ + 2.0 * nAAA_ + 2.0 * nAAAA_)) +
                          16.0 * nrho_ + bonds_per_atom * 2.0 * noutp_ * sizeof(T);
  const int cs = plan_chunk(n, per_atom, 64.0 * bonds_per_atom + 64.0);
  const int nchunks = (n + cs - 1) / cs;
  chunk_used_ = nchunks > 1 ? cs : 0;
  std::vector<long long> ebound;
  size_t ecap = (size_t) std::max<int64_t>(nb_, 1);
  if (nchunks > 1) {
    layout_chunks(cs);
    ebound = chunk_edge_bounds(cs);
    ecap = 1;
    for (int k = 0; k < nchunks; k++) ecap = std::max(ecap, (size_t) (ebound[(size_t) k + 1] - ebound[(size_t) k]));
  }
  // rows of the per-atom tensors: the generated chain kernels run whole blocks of atoms and neither guard their loads nor
  // their stores, so the tensors hold rows up to the end of the last block
  const size_t na = (size_t) round_up(cs, 16);
  if (!(rad_.has_tables() && tables_inside_)) {    // with tables evaluated inside the kernels the rows do not exist
    Rz_.ensure(ecap * noutp_ * sizeof(T));
    dRz_.ensure(ecap * noutp_ * sizeof(T));
  }
  A_.ensure(na * nlm_ * CP_ * sizeof(T));
  A1_.ensure(na * nlm_ * CFP_ * sizeof(T));
  AA_.ensure(na * nAA_ * CFP_ * sizeof(T));
  AA1_.ensure(na * nAA_ * CFP_ * sizeof(T));
  AAA_.ensure(na * nAAA_ * CFP_ * sizeof(T));
  if (order4_) {
    AA2_.ensure(na * nAA_ * CFP_ * sizeof(T));
    AAAA_.ensure(na * nAAAA_ * CFP_ * sizeof(T));
  }
  rho_.ensure(na * nrho_ * sizeof(double));
  grho_.ensure(na * nrho_ * sizeof(double));
  if (fl.uq) {
    uq_gamma_.ensure((size_t) n * sizeof(double)); uq_sigma_.ensure((size_t) n * sizeof(double)); uq_cluster_.ensure((size_t) n * sizeof(double));
    ran_uq_ = true;
  }
  if (!fl.energy_only) {
    gA_.ensure(na * nlm_ * CP_ * sizeof(T));
    gA1_.ensure(na * nlm_ * CFP_ * sizeof(T));
    gAA_.ensure(na * nAA_ * CFP_ * sizeof(T));
    gAA1_.ensure(na * nAA_ * CFP_ * sizeof(T));
    gAAA_.ensure(na * nAAA_ * CFP_ * sizeof(T));
    if (order4_) {
      gAA2_.ensure(na * nAA_ * CFP_ * sizeof(T));
      gAAAA_.ensure(na * nAAAA_ * CFP_ * sizeof(T));
    }
  }
  if (aaa_a_ && CP_ != CFP_) throw Error("GRACE-1L: AAA = AA1 x A needs equal A and FC widths");
  for (int k = 0; k < nchunks; k++) {
    const int a0 = k * cs, nc = std::min(n, a0 + cs) - a0;
    if (nchunks == 1) {
      cur_tiles_ = tiles_.as<int>();
      cur_ntiles_ = ntiles_;
      run_chunk(fl, 0, n, 0, -1);
    } else {
      cur_tiles_ = chunk_tiles_.as<int>() + (size_t) 16 * chunk_tile_off_[(size_t) k];
      cur_ntiles_ = chunk_tile_off_[(size_t) k + 1] - chunk_tile_off_[(size_t) k];
      run_chunk(fl, a0, nc, ebound[(size_t) k], ebound[(size_t) k + 1] - ebound[(size_t) k]);
    }
  }
  if (ordered_) ordered_finish(fl);
}

// One chunk: atoms [a0, a0 + nc) and their bonds [e_begin, e_begin + e_count) (e_count < 0: all bonds, counted on the
// device).  Per-atom tensors hold the chunk's atoms from row 0; cur_tiles_ names them by that row.
template<class T> void Engine1L<T>::run_chunk(const RunFlags &fl, int a0, int nc, long long e_begin, long long e_count)
{
  const int n = nc;
  const int ntiles = cur_ntiles_;
  const int *tiles = cur_tiles_;
  const int *mu = mu_.as<int>() + a0;
  const size_t na = (size_t) nc;
  // the radial rows of the chunk start at row 0 of Rz_ / dRz_; the kernels index them by the bond's number in the structure
  T *Rz = moved_back(Rz_.as<T>(), e_begin * noutp_), *dRz = moved_back(dRz_.as<T>(), e_begin * noutp_);

  // radial tables asked for: the A basis and the bond reverse evaluate them themselves, no radial row is written or read
  // (GRACE_HIP_TABLE_ROWS=1: the rows are written by the table kernel and read back, as without tables)
  const bool tab_inside = rad_.has_tables() && tables_inside_ && (nl_ * (CP_ / 16) <= 10 || (nl_ <= 7 && CP_ == 16));
  RadialTable<T> tb{};
  if (tab_inside) tb = rad_.table(stream_, ncu_, xr_.as<double>(), emu_.as<int>(), z_.as<T>());
  else stage("radial_mlp", [&] { launch_radial(e_begin, e_count, xr_.as<double>(), emu_.as<int>(), Rz, dRz, eoff_.as<long long>() + n_, true); });

  ScatterArgs<T> sa{};
  sa.tb = tb;
  sa.eoff = eoff_.as<long long>(); sa.rh = rh_.as<double>(); sa.Rz = Rz; sa.A = A_.as<T>();
  sa.a0 = a0; sa.C = CP_; sa.nl = nl_; sa.nlm = nlm_; sa.noutp = noutp_; sa.sh = sh_;
  stage("scatter_A", [&] { launch_scatter<T>(sa, n, lmax_); });

  const int ka = CP_ / 16, kf = CFP_ / 16;
  auto jit_launch = [&](hipFunction_t f, std::vector<void *> args) {
    const long long cols = (long long) n * CFP_;
    HIP_CHECK(hipModuleLaunchKernel(f, (unsigned) ((cols + 255) / 256), 1, 1, 256, 1, 1, 0, stream_, args.data(), nullptr));
  };
  int one = 1, nat = n;
  auto prod_fwd = [&](const char *name, DevProd &P, const T *L, const T *R, T *out, int sl, int sr) {
    const int AT = std::max(1, 256 / CFP_);
    if (P.jit.ok()) {
      stage(name, [&] { jit_launch(P.jit.fwd, {(void *) &L, (void *) &R, (void *) &out, (void *) &nat, (void *) &one}); });
      return;
    }
    stage(name, [&] {
      hipLaunchKernelGGL(k_prod_fwd<T>, dim3(P.d.nout * 8 * (((n + AT - 1) / AT + 7) / 8)), dim3(CFP_ * AT), 0, stream_, P.d, L, R, out, n, CFP_, sl, sr);
    });
  };
  T *A = A_.as<T>(), *A1 = A1_.as<T>(), *AA = AA_.as<T>(), *AA1 = AA1_.as<T>(), *AA2 = AA2_.as<T>(), *AAA = AAA_.as<T>(),
    *AAAA = AAAA_.as<T>();
  const T *Ar = aaa_a_ ? A : A1;
  const bool fused = chain_.ok();
  const T *chainW = chainW_.as<T>();
  const unsigned chain_blocks = fused ? (unsigned) ((n + chain_.atoms_per_block - 1) / chain_.atoms_per_block) : 0;
  if (fused) {
    // A -> A1 -> AA -> AA1 / AA2 -> AAA / AAAA in one kernel: AA is written for the functions the rho reduce collects only
    stage("chain_fwd", [&] {
      const T *x0 = A;
      void *args[] = {(void *) &x0, (void *) &A1, (void *) &AA, (void *) &AA1, (void *) &AA2, (void *) &AAA, (void *) &AAAA, (void *) &chainW, (void *) &nat,
                      (void *) &one};
      HIP_CHECK(hipModuleLaunchKernel(chain_.fwd, chain_blocks, 1, 1, 256, 1, 1, 0, stream_, args, nullptr));
      cur_flops_ += chain_.flops_per_atom * n;
    });
  } else {
    stage("fc_A1", [&] { launch_gemm(fcA1_.fwd, ka, ka, kf, A, nlm_, A, nlm_, A1, nlm_, 0); });
    prod_fwd("prod_AA", pAA_, A1, A1, AA, nlm_, nlm_);
    stage("fc_AA1", [&] { launch_gemm(fcAA1_.fwd, kf, ka, kf, AA, nAA_, A, nlm_, AA1, nAA_, 0); });
    prod_fwd("prod_AAA", pAAA_, AA1, Ar, AAA, nAA_, nlm_);
    if (order4_) {
      stage("fc_AA2", [&] { launch_gemm(fcAA2_.fwd, kf, ka, kf, AA, nAA_, A, nlm_, AA2, nAA_, 0); });
      prod_fwd("prod_AAAA", pAAAA_, AA2, AA2, AAAA, nAA_, nAA_);
    }
  }
  stage("reduce_rho", [&] {
#define GR_RED(KA, KF) hipLaunchKernelGGL((k_reduce_fwd<T, KA, KF>), dim3(ntiles), dim3(64 * kReduceWaves), 0, stream_, redrho_.d, mu, tiles, \
                                          (const T *) A, (const T *) AA, (const T *) AAA, (const T *) AAAA, rho_.as<double>())
    switch (ka * 10 + kf) {
      case 11: GR_RED(1, 1); break; case 12: GR_RED(1, 2); break; case 14: GR_RED(1, 4); break;
      case 21: GR_RED(2, 1); break; case 22: GR_RED(2, 2); break; case 24: GR_RED(2, 4); break;
      case 41: GR_RED(4, 1); break; case 42: GR_RED(4, 2); break; case 44: GR_RED(4, 4); break;
      default: throw Error("unsupported channel widths");
    }
#undef GR_RED
  });
  stage("energy_mlp", [&] {
    const size_t lds = (size_t) (4 * (2 * en_.nlay + 4) * en_.width + en_.wlds) * sizeof(double);
    const dim3 grid((unsigned) ((n + kEnergyAtomsPerBlock - 1) / kEnergyAtomsPerBlock));
    auto kern = en_.wlds > 0 ? k_energy<true> : k_energy<false>;
    if (lds > 48 * 1024)
      HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds));
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream_, en_, mu_.as<int>(), a0, n, rho_.as<double>(), grho_.as<double>(),
                       fl.eatom || ordered_ ? eatom_.as<double>() + a0 : nullptr, ordered_ ? nullptr : scal_.as<double>(), fl.energy_only ? 0 : 1,
                       sid_ptr());
  });
  if (fl.uq) {
    stage("uq", [&] {
      UqDev<T> u = uq_;
      u.X[0] = A; u.X[1] = AA; u.X[2] = AAA; u.X[3] = AAAA;
      const size_t lds = (size_t) (u.d_basis + 4 * u.rp + 2 * u.D) * sizeof(double);
      auto kern = k_uq<T>;
      if (lds > 48 * 1024)
        HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds));
      hipLaunchKernelGGL(kern, dim3(n), dim3(256), lds, stream_, u, mu, n, uq_gamma_.as<double>() + a0, uq_sigma_.as<double>() + a0,
                         uq_cluster_.as<double>() + a0);
    });
  }
  if (fl.energy_only) return;

  // ---- reverse
  T *gA = gA_.as<T>(), *gA1 = gA1_.as<T>(), *gAA = gAA_.as<T>(), *gAA1 = gAA1_.as<T>(), *gAA2 = gAA2_.as<T>(),
    *gAAA = gAAA_.as<T>(), *gAAAA = gAAAA_.as<T>();
  if (fused) {
    // the reverse of the rho reduce leaves the adjoints of AAA, AAAA and of the collected functions of A and AA; the chain
    // kernel takes them to the adjoint of A.  Rows the reduce does not visit are not read by it, so nothing is cleared
    // when the reduce may write its rows.
    if (!red_writes_)
      stage("zero_grads", [&] {
        HIP_CHECK(hipMemsetAsync(gA, 0, na * nlm_ * CP_ * sizeof(T), stream_));
        HIP_CHECK(hipMemsetAsync(gAA, 0, na * nAA_ * CFP_ * sizeof(T), stream_));
        HIP_CHECK(hipMemsetAsync(gAAA, 0, na * nAAA_ * CFP_ * sizeof(T), stream_));
        if (order4_) HIP_CHECK(hipMemsetAsync(gAAAA, 0, na * nAAAA_ * CFP_ * sizeof(T), stream_));
      });
    stage("reduce_rho_bwd", [&] {
      if (redrho_.njobs > 0)
        hipLaunchKernelGGL(k_reduce_bwd<T>, dim3(ntiles, redrho_.njobs), dim3(64), 0, stream_, redrho_.d, mu, tiles, grho_.as<double>(), gA, gAA,
                           gAAA, gAAAA, 0, red_writes_ ? 1 : 0);
    });
    stage("chain_bwd", [&] {
      const T *x0 = A, *x1 = A1, *p21 = AA1, *p22 = AA2, *g2 = gAA, *g3 = gAAA, *g4 = gAAAA, *g21 = nullptr;    // P3 is inside the kernel
      void *args[] = {(void *) &x0, (void *) &x1, (void *) &p21, (void *) &p22, (void *) &g2, (void *) &g3, (void *) &g4, (void *) &g21, (void *) &gA,
                      (void *) &chainW,
                      (void *) &nat, (void *) &one};
      HIP_CHECK(hipModuleLaunchKernel(chain_.bwd, chain_blocks, 1, 1, 256, 1, 1, 0, stream_, args, nullptr));
      cur_flops_ += chain_.flops_per_atom * n;
    });
  } else {
  stage("zero_grads", [&] {
    HIP_CHECK(hipMemsetAsync(gA, 0, na * nlm_ * CP_ * sizeof(T), stream_));
    HIP_CHECK(hipMemsetAsync(gA1, 0, na * nlm_ * CFP_ * sizeof(T), stream_));
    // with the AAAA stage the merged FC reverse WRITES every row of gAA (a job per function) and the rho reverse of the
    // sources A and AA runs after it: no fill of the largest adjoint, and no read of it by the FC reverse
    if (!order4_) HIP_CHECK(hipMemsetAsync(gAA, 0, na * nAA_ * CFP_ * sizeof(T), stream_));
    // with the specialised product kernels gAA1 and gAA2 are written (not accumulated) by their first producer
    if (!jit_all_) HIP_CHECK(hipMemsetAsync(gAA1, 0, na * nAA_ * CFP_ * sizeof(T), stream_));
    HIP_CHECK(hipMemsetAsync(gAAA, 0, na * nAAA_ * CFP_ * sizeof(T), stream_));
    if (order4_) {
      if (!jit_all_) HIP_CHECK(hipMemsetAsync(gAA2, 0, na * nAA_ * CFP_ * sizeof(T), stream_));
      HIP_CHECK(hipMemsetAsync(gAAAA, 0, na * nAAAA_ * CFP_ * sizeof(T), stream_));
    }
  });
  const int jobs_a_aa = redrho_.d.ncol[0] + redrho_.d.ncol[1];    // jobs of the sources A and AA (the first two)
  stage("reduce_rho_bwd", [&] {
    const int first = order4_ ? jobs_a_aa : 0;
    if (redrho_.njobs > first)
      hipLaunchKernelGGL(k_reduce_bwd<T>, dim3(ntiles, redrho_.njobs - first), dim3(64), 0, stream_, redrho_.d, mu, tiles, grho_.as<double>(),
                         gA, gAA, gAAA, gAAAA, first);
  });
  // accL / accR: add to the stored adjoint or overwrite it (specialised kernels; the table-driven ones always add)
  auto prod_bwd = [&](const char *name, DevProd &P, const T *L, const T *R, const T *g, T *gL, T *gR, int sl, int sr, int accL, int accR) {
    const int AT = std::max(1, 256 / CFP_);
    if (P.jit.ok()) {
      if (!jit_all_) accL = accR = 1;
      stage(name, [&] {
        jit_launch(P.jit.bwd, {(void *) &L, (void *) &R, (void *) &g, (void *) &gL, (void *) &gR, (void *) &accL, (void *) &accR, (void *) &nat,
                               (void *) &one});
      });
      return;
    }
    stage(name, [&] {
      hipLaunchKernelGGL(k_prod_bwd<T>, dim3(P.d.nleft * 8 * (((n + AT - 1) / AT + 7) / 8)), dim3(CFP_ * AT), 0, stream_, P.d, 0, R, g, gL, n, CFP_, sr, sl);
      hipLaunchKernelGGL(k_prod_bwd<T>, dim3(P.d.nright * 8 * (((n + AT - 1) / AT + 7) / 8)), dim3(CFP_ * AT), 0, stream_, P.d, 1, L, g, gR, n, CFP_, sl, sr);
    });
  };
  // FC reverse: left input (same functions as the output), then right input (functions of A)
  auto fc_bwd = [&](const char *name, DevFc<T> &F, const T *g, T *gXl, T *gXr, int nfl, int kl) {
    stage(name, [&] {
      if (F.have_lr && gXl == gXr && kl == ka && nfl == nlm_) {
        launch_gemm(F.bwd_lr, kf, kf, ka, g, nfl, g, nfl, gXl, nlm_, 1);
        return;
      }
      launch_gemm(F.bwd_l, kf, kf, kl, g, nfl, g, nfl, gXl, nfl, 1);
      launch_gemm(F.bwd_r, kf, kf, ka, g, nfl, g, nfl, gXr, nlm_, 1);
    });
  };
  if (order4_) prod_bwd("prod_AAAA_bwd", pAAAA_, AA2, AA2, gAAAA, gAA2, gAA2, nAA_, nAA_, 0, 0);
  prod_bwd("prod_AAA_bwd", pAAA_, AA1, Ar, gAAA, gAA1, aaa_a_ ? gA : gA1, nAA_, nlm_, 0, 1);
  if (order4_) {
    // fc_AA1 and fc_AA2 share their inputs: one pass over gAA and gA for both
    stage("fc_AA12_bwd", [&] {
      launch_gemm(fcAA12_.bwd_l, kf, kf, kf, gAA1, nAA_, gAA2, nAA_, gAA, nAA_, 0);
      launch_gemm(fcAA12_.bwd_r, kf, kf, ka, gAA1, nAA_, gAA2, nAA_, gA, nlm_, 1);
    });
    stage("reduce_rho_bwd_A_AA", [&] {
      if (jobs_a_aa > 0)
        hipLaunchKernelGGL(k_reduce_bwd<T>, dim3(ntiles, jobs_a_aa), dim3(64), 0, stream_, redrho_.d, mu, tiles, grho_.as<double>(), gA, gAA,
                           gAAA, gAAAA, 0);
    });
  } else {
    fc_bwd("fc_AA1_bwd", fcAA1_, gAA1, gAA, gA, nAA_, kf);
  }
  prod_bwd("prod_AA_bwd", pAA_, A1, A1, gAA, gA1, gA1, nlm_, nlm_, 1, 1);
  fc_bwd("fc_A1_bwd", fcA1_, gA1, gA, gA, nlm_, ka);
  }

  BondBwdArgs<T> ba{};
  ba.eoff = eoff_.as<long long>(); ba.ej = ej_.as<int>(); ba.rh = rh_.as<double>(); ba.r = r_.as<double>(); ba.rc = rc_.as<double>();
  ba.Rz = Rz; ba.dRz = dRz; ba.gA = gA;
  ba.tb = tb;
  ba.f = f_.as<double>(); ba.virial = scal_.as<double>() + 1; ba.sid = sid_ptr(); ba.vatom = vatom_ptr();
  ba.fedge = ordered_ ? fedge_.as<double>() : nullptr; ba.fcen = ordered_ ? fcen_.as<double>() : nullptr;
  ba.a0 = a0; ba.C = CP_; ba.nl = nl_; ba.nlm = nlm_; ba.noutp = noutp_; ba.sh = sh_;
  stage("bond_bwd", [&] { launch_bond_bwd<T>(ba, n); });
}

template<class T> void Engine1L<T>::debug_radial(int m, const double *x, const int *mu_j, double *Rz, double *dRz)
{
  HIP_CHECK(hipSetDevice(device_));
  if (m <= 0) return;
  for (int q = 0; q < m; q++)
    if (mu_j[q] < 0 || mu_j[q] >= nel_) throw InvalidArgument("neighbour element out of range");
  DevBuf dx, dmu, dR, ddR, dn;
  dx.ensure(sizeof(double) * m); dmu.ensure(sizeof(int) * m);
  dR.ensure(sizeof(T) * (size_t) m * noutp_); ddR.ensure(sizeof(T) * (size_t) m * noutp_);
  dn.ensure(sizeof(long long));
  HIP_CHECK(hipMemcpy(dx.p, x, sizeof(double) * m, hipMemcpyHostToDevice));
  HIP_CHECK(hipMemcpy(dmu.p, mu_j, sizeof(int) * m, hipMemcpyHostToDevice));
  launch_radial(0, m, dx.as<double>(), dmu.as<int>(), dR.as<T>(), ddR.as<T>(), dn.as<long long>());
  HIP_CHECK(hipGetLastError());
  HIP_CHECK(hipStreamSynchronize(stream_));
  std::vector<T> hR((size_t) m * noutp_), hdR((size_t) m * noutp_);
  HIP_CHECK(hipMemcpy(hR.data(), dR.p, hR.size() * sizeof(T), hipMemcpyDeviceToHost));
  HIP_CHECK(hipMemcpy(hdR.data(), ddR.p, hdR.size() * sizeof(T), hipMemcpyDeviceToHost));
  for (int q = 0; q < m; q++)
    for (int l = 0; l < nl_; l++)
      for (int c = 0; c < C_; c++) {
        Rz[((size_t) q * nl_ + l) * C_ + c] = (double) hR[(size_t) q * noutp_ + l * CP_ + c];
        dRz[((size_t) q * nl_ + l) * C_ + c] = (double) hdR[(size_t) q * noutp_ + l * CP_ + c];
      }
}

// The radial functions of debug_radial for device arrays, without any device allocation: the staging rows live in the
// fixed array.  Calls on one GPU share that array (also calls of different engines and of different threads): a mutex per
// GPU lets one call at a time use it.  The caller's arrays may still be in flight on another stream (x written by a
// kernel of the caller's library just before the call), so the call first waits for the device, as the other entry
// points that take device arrays do.
template<class T> void Engine1L<T>::radial_noalloc(int m, const double *x, const int *mu_j, double *Rz, double *dRz)
{
  HIP_CHECK(hipSetDevice(device_));
  if (m < 0) throw InvalidArgument("negative number of radial arguments");
  if (m == 0) return;
  if (!x || !mu_j || !Rz || !dRz) throw InvalidArgument("x, mu_j, Rz and dRz are required");
  for (const void *p : {(const void *) x, (const void *) mu_j, (const void *) Rz, (const void *) dRz}) {
    hipPointerAttribute_t at{};
    if (hipPointerGetAttributes(&at, p) != hipSuccess || at.type != hipMemoryTypeDevice || at.device != device_) {
      (void) hipGetLastError();
      throw InvalidArgument("x, mu_j, Rz and dRz must be device memory of the engine's GPU");
    }
  }
  auto align = [](size_t b) { return (b + 255) / 256 * 256; };
  const size_t mu_bytes = align((size_t) m * sizeof(int)), row_bytes = align((size_t) m * noutp_ * sizeof(T));
  const size_t need = kScratchHeader + mu_bytes + 2 * row_bytes;
  if (need > kScratchBytes) {
    const size_t per = sizeof(int) + 2 * (size_t) noutp_ * sizeof(T);
    throw InvalidArgument("radial call without allocations: " + std::to_string(m) + " arguments need " + std::to_string(need) +
                          " bytes of the fixed " + std::to_string(kScratchBytes) + "-byte device array (at most " +
                          std::to_string((kScratchBytes - kScratchHeader - 768) / per) + " arguments for this model and precision)");
  }
  std::lock_guard<std::mutex> in_use(scratch_in_use[device_]);
  HIP_CHECK(hipDeviceSynchronize());
  unsigned char *base = scratch_dev_;
  int *bad = reinterpret_cast<int *>(base);
  long long *nedges = reinterpret_cast<long long *>(base + 8);    // not read: the count is passed by value
  int *mu = reinterpret_cast<int *>(base + kScratchHeader);
  T *R = reinterpret_cast<T *>(base + kScratchHeader + mu_bytes), *dR = reinterpret_cast<T *>(base + kScratchHeader + mu_bytes + row_bytes);
  hipLaunchKernelGGL(k_clear_flag, dim3(1), dim3(64), 0, stream_, bad);
  hipLaunchKernelGGL(k_stage_elements, dim3((unsigned) ((m + 255) / 256)), dim3(256), 0, stream_, mu_j, m, nel_, mu, bad);
  HIP_CHECK(hipGetLastError());
  launch_radial(0, m, x, mu, R, dR, nedges);
  HIP_CHECK(hipGetLastError());
  const long long total = (long long) m * nl_ * C_;
  hipLaunchKernelGGL(k_unpack_radial<T>, dim3((unsigned) std::min<long long>((total + 255) / 256, 4096)), dim3(256), 0, stream_, (const T *) R,
                     (const T *) dR, total, nl_, C_, CP_, noutp_, Rz, dRz);
  HIP_CHECK(hipGetLastError());
  int flag = 0;
  HIP_CHECK(hipMemcpyAsync(&flag, bad, sizeof(int), hipMemcpyDeviceToHost, stream_));
  HIP_CHECK(hipStreamSynchronize(stream_));
  if (flag) throw InvalidArgument("neighbour element out of range");
}

}    // namespace

std::unique_ptr<Engine> make_engine_1l(std::shared_ptr<const Model1L> model, int ntypes, const std::vector<int> &type2mu,
                                       int precision, int device)
{
  if (precision == 64) return std::make_unique<Engine1L<double>>(std::move(model), ntypes, type2mu, device);
  if (precision == 32) return std::make_unique<Engine1L<float>>(std::move(model), ntypes, type2mu, device);
  throw InvalidArgument("precision must be 64 or 32");
}

}    // namespace grhip
