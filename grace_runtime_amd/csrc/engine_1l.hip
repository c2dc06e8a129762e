// GRACE-1L engine for gfx950: device tables built from the model, and the staged pass over a CSR structure.
// Driver skeleton after libgrace/src/fused_1l.cpp:474-582 (type map, bond filter, forward, readout, reverse, forces)
// and the staged GPU pipeline of libgrace/include/grace/kk/grace_1l_kk.h:449-454; liveness pruning of FC outputs and
// CG terms after libgrace/src/fused_1l.cpp:176-216.
#include "engine.hpp"
#include "jit_prod.hpp"
#include "kernels_1l.hpp"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <numeric>

namespace grhip {

#define HIP_CHECK(expr)                                                                                         \
  do {                                                                                                          \
    hipError_t e_ = (expr);                                                                                     \
    if (e_ != hipSuccess)                                                                                       \
      throw Error(std::string("HIP error: ") + hipGetErrorString(e_) + " in " #expr " (" __FILE__ ":" + std::to_string(__LINE__) + ")"); \
  } while (0)

namespace {

// device allocation owned by the engine
struct DevBuf {
  void *p = nullptr;
  size_t bytes = 0;
  DevBuf() = default;
  DevBuf(const DevBuf &) = delete;
  DevBuf &operator=(const DevBuf &) = delete;
  ~DevBuf() { release(); }
  void release()
  {
    if (p) (void) hipFree(p);
    p = nullptr;
    bytes = 0;
  }
  // at least `need` bytes (grown with head room; contents are not kept)
  void ensure(size_t need)
  {
    if (need <= bytes && p) return;
    release();
    const size_t want = std::max<size_t>(need + need / 8, 256);
    hipError_t e = hipMalloc(&p, want);
    if (e != hipSuccess) {
      p = nullptr;
      (void) hipGetLastError();
      throw std::bad_alloc();
    }
    bytes = want;
  }
  template<class U> U *as() const { return static_cast<U *>(p); }
};

template<class U> void upload_vec(DevBuf &b, const std::vector<U> &v)
{
  b.ensure(std::max<size_t>(v.size(), 1) * sizeof(U));
  if (!v.empty()) HIP_CHECK(hipMemcpy(b.p, v.data(), v.size() * sizeof(U), hipMemcpyHostToDevice));
}

inline int round_up(int a, int b) { return (a + b - 1) / b * b; }

struct HostProd {
  std::vector<int> off, l, r;
  std::vector<double> c;
  std::vector<int> loff, l_o, l_r, roff, r_o, r_l;
  std::vector<double> l_c, r_c;
  std::vector<ProdTerm> terms;    // the kept terms, for the specialised kernels
  int nout = 0, nleft = 0, nright = 0;
};

// terms of outputs with need[o] set, sorted by output; operand-major copies for the reverse
HostProd build_prod(const CGProduct &p, const std::vector<char> &need, int nleft, int nright)
{
  HostProd h;
  h.nout = p.n_out;
  h.nleft = nleft;
  h.nright = nright;
  std::vector<int> ord;
  for (int t = 0; t < p.n_terms; t++)
    if (need[p.m_sum_ind[t]]) ord.push_back(t);
  std::stable_sort(ord.begin(), ord.end(), [&](int a, int b) { return p.m_sum_ind[a] < p.m_sum_ind[b]; });
  h.off.assign(h.nout + 1, 0);
  for (int t : ord) {
    h.l.push_back(p.left_ind[t]);
    h.r.push_back(p.right_ind[t]);
    h.c.push_back(p.cg_coeff[t]);
    h.off[p.m_sum_ind[t] + 1]++;
    h.terms.push_back({p.left_ind[t], p.right_ind[t], p.m_sum_ind[t], p.cg_coeff[t]});
  }
  for (int o = 0; o < h.nout; o++) h.off[o + 1] += h.off[o];
  auto by_operand = [&](const std::vector<int> &key, int nkey, std::vector<int> &off, std::vector<int> &oo,
                        std::vector<int> &other, std::vector<double> &cc, const std::vector<int> &oth) {
    std::vector<int> o2 = ord;
    std::stable_sort(o2.begin(), o2.end(), [&](int a, int b) { return key[a] < key[b]; });
    off.assign(nkey + 1, 0);
    for (int t : o2) {
      oo.push_back(p.m_sum_ind[t]);
      other.push_back(oth[t]);
      cc.push_back(p.cg_coeff[t]);
      off[key[t] + 1]++;
    }
    for (int q = 0; q < nkey; q++) off[q + 1] += off[q];
  };
  by_operand(p.left_ind, nleft, h.loff, h.l_o, h.l_r, h.l_c, p.right_ind);
  by_operand(p.right_ind, nright, h.roff, h.r_o, h.r_l, h.r_c, p.left_ind);
  return h;
}

struct DevProd {
  DevBuf off, l, r, c, loff, l_o, l_r, l_c, roff, r_o, r_l, r_c;
  ProdDev d{};
  JitKernels jit;        // model-specialised kernels (jit_prod.hpp); not ok(): the table-driven kernels run
  std::string jit_note;
  ~DevProd() { jit.release(); }
  void build(const HostProd &h)
  {
    upload_vec(off, h.off); upload_vec(l, h.l); upload_vec(r, h.r); upload_vec(c, h.c);
    upload_vec(loff, h.loff); upload_vec(l_o, h.l_o); upload_vec(l_r, h.l_r); upload_vec(l_c, h.l_c);
    upload_vec(roff, h.roff); upload_vec(r_o, h.r_o); upload_vec(r_l, h.r_l); upload_vec(r_c, h.r_c);
    d.off = off.as<int>(); d.l = l.as<int>(); d.r = r.as<int>(); d.c = c.as<double>();
    d.loff = loff.as<int>(); d.l_o = l_o.as<int>(); d.l_r = l_r.as<int>(); d.l_c = l_c.as<double>();
    d.roff = roff.as<int>(); d.r_o = r_o.as<int>(); d.r_l = r_l.as<int>(); d.r_c = r_c.as<double>();
    d.nout = h.nout; d.nleft = h.nleft; d.nright = h.nright;
  }
};

// weights W[K][N] (row-major) of a tile GEMM in MFMA fragment order [cb][s][lane]: lane (g, c) holds
// W[g * (K / 4) + s][cb * 16 + c]
template<class T> void pack_fragments(const std::vector<double> &W, int K, int N, int Kp, int Np, std::vector<T> &out)
{
  const int ks = Kp / 4, nb = Np / 16;
  const size_t base = out.size();
  out.resize(base + (size_t) nb * ks * 64, (T) 0);
  for (int cb = 0; cb < nb; cb++)
    for (int s = 0; s < ks; s++)
      for (int lane = 0; lane < 64; lane++) {
        const int g = lane >> 4, c = lane & 15, k = g * ks + s, n = cb * 16 + c;
        if (k < K && n < N) out[base + ((size_t) cb * ks + s) * 64 + lane] = (T) W[(size_t) k * N + n];
      }
}

template<class T> struct DevJobs {
  DevBuf job_out, job_scale, seg_off, seg_src, seg_fn, seg_w, seg_scale;
  GemmJobs<T> d{};
  struct Host {
    std::vector<int> job_out, seg_off{0}, seg_src, seg_fn, seg_w;
    std::vector<T> job_scale, seg_scale;
    void job(int out, double scale) { job_out.push_back(out); job_scale.push_back((T) scale); }
    void seg(int src, int fn, int w, double scale) { seg_src.push_back(src); seg_fn.push_back(fn); seg_w.push_back(w); seg_scale.push_back((T) scale); }
    void end_job() { seg_off.push_back((int) seg_src.size()); }
  };
  void build(const Host &h, const T *WF0, const T *WF1)
  {
    upload_vec(job_out, h.job_out); upload_vec(job_scale, h.job_scale); upload_vec(seg_off, h.seg_off);
    upload_vec(seg_src, h.seg_src); upload_vec(seg_fn, h.seg_fn); upload_vec(seg_w, h.seg_w); upload_vec(seg_scale, h.seg_scale);
    d.job_out = job_out.as<int>(); d.job_scale = job_scale.as<T>(); d.seg_off = seg_off.as<int>();
    d.seg_src = seg_src.as<int>(); d.seg_fn = seg_fn.as<int>(); d.seg_w = seg_w.as<int>(); d.seg_scale = seg_scale.as<T>();
    d.WF0 = WF0; d.WF1 = WF1;
    d.njobs = (int) h.job_out.size();
  }
  void set_rows(const int *drow) { for (int q = 0; q < 16; q++) d.drow[q] = drow[q]; }
};

// One FC layer as three job lists (forward, reverse into the left input, reverse into the right input) over
// fragment-ordered weight tiles.  Widths are the padded ones (multiples of 16; padding weights are zero).
template<class T> struct DevFc {
  DevBuf WlF, WrF, WlTF, WrTF;
  DevJobs<T> fwd, bwd_l, bwd_r;
  int nil = 0, nir = 0, no = 0;    // padded widths
  // nfr: functions of the right-input tensor; livef: outputs that are computed
  void build(const FCWeights &w, const std::vector<char> &livef, int nfr, int nil_p, int nir_p, int no_p, const int *drow)
  {
    nil = nil_p; nir = nir_p; no = no_p;
    const int nt = w.tiles_left;
    std::vector<T> fl, fr, flt, frt;
    std::vector<double> M, Mt;
    auto tile_mats = [&](const std::vector<double> &W, double norm, int nin, int t) {
      M.assign((size_t) nin * w.n_out, 0.0);     // [n][k]
      Mt.assign((size_t) w.n_out * nin, 0.0);    // [k][n]
      for (int k = 0; k < w.n_out; k++)
        for (int n = 0; n < nin; n++) {
          const double v = norm * W[((size_t) k * nin + n) * nt + t];
          M[(size_t) n * w.n_out + k] = v;
          Mt[(size_t) k * nin + n] = v;
        }
    };
    for (int t = 0; t < nt; t++) {
      tile_mats(w.w_left, w.norm_left, w.n_in_left, t);
      pack_fragments<T>(M, w.n_in_left, w.n_out, nil, no, fl);
      pack_fragments<T>(Mt, w.n_out, w.n_in_left, no, nil, flt);
      tile_mats(w.w_right, w.norm_right, w.n_in_right, t);
      pack_fragments<T>(M, w.n_in_right, w.n_out, nir, no, fr);
      pack_fragments<T>(Mt, w.n_out, w.n_in_right, no, nir, frt);
    }
    upload_vec(WlF, fl); upload_vec(WrF, fr); upload_vec(WlTF, flt); upload_vec(WrTF, frt);
    typename DevJobs<T>::Host hf, hl, hr;
    std::vector<std::vector<int>> conn_of(w.n_funcs), conn_from(nfr);
    for (int c = 0; c < w.n_conn; c++) {
      conn_of[w.collect_to[c]].push_back(c);
      if (livef[w.collect_to[c]]) conn_from[w.collect_from[c]].push_back(c);
    }
    for (int f = 0; f < w.n_funcs; f++) {
      if (!livef[f]) continue;
      hf.job(f, w.norm_out_factor[f]);
      hf.seg(0, f, w.w_tile_left[f], 1.0);
      for (int c : conn_of[f]) hf.seg(1, w.collect_from[c], w.w_tile_right[c], 1.0);
      hf.end_job();
      hl.job(f, w.norm_out_factor[f]);
      hl.seg(0, f, w.w_tile_left[f], 1.0);
      hl.end_job();
    }
    for (int r = 0; r < nfr; r++) {
      if (conn_from[r].empty()) continue;
      hr.job(r, 1.0);
      for (int c : conn_from[r]) hr.seg(0, w.collect_to[c], w.w_tile_right[c], w.norm_out_factor[w.collect_to[c]]);
      hr.end_job();
    }
    fwd.build(hf, WlF.as<T>(), WrF.as<T>());
    bwd_l.build(hl, WlTF.as<T>(), WlTF.as<T>());
    bwd_r.build(hr, WrTF.as<T>(), WrTF.as<T>());
    fwd.set_rows(drow); bwd_l.set_rows(drow); bwd_r.set_rows(drow);
  }
};

template<class T> class Engine1L final : public Engine {
 public:
  Engine1L(std::shared_ptr<const Model1L> m, int ntypes, const std::vector<int> &type2mu, int device) :
      model_(std::move(m)), ntypes_(ntypes), type2mu_(type2mu), device_(device)
  {
    check_type2mu(type2mu_, ntypes_, model_->n_elements, "GRACE-1L");
    HIP_CHECK(hipSetDevice(device_));
    hipDeviceProp_t prop;
    HIP_CHECK(hipGetDeviceProperties(&prop, device_));
    if (std::string(prop.gcnArchName).rfind("gfx950", 0) != 0 && std::string(prop.gcnArchName).rfind("gfx942", 0) != 0)
      throw Error(std::string("this library is built for gfx950 (MI355X); device is ") + prop.gcnArchName);
    ncu_ = prop.multiProcessorCount;
    arch_ = prop.gcnArchName;
    HIP_CHECK(hipStreamCreate(&stream_));
    probe_mfma();
    build();
  }
  ~Engine1L() override
  {
    (void) hipSetDevice(device_);
    for (auto &e : events_) { (void) hipEventDestroy(e.first); (void) hipEventDestroy(e.second); }
    if (stream_) (void) hipStreamDestroy(stream_);
  }

  int layers() const override { return 1; }
  double cutoff(int t1, int t2) const override
  {
    if (t1 < 1 || t1 > ntypes_ || t2 < 1 || t2 > ntypes_) return 0.0;
    return model_->pair_cutoff(type2mu_[t1], type2mu_[t2]);
  }
  double max_cutoff() const override
  {
    double m = 0.0;
    for (int a = 1; a <= ntypes_; a++)
      for (int b = 1; b <= ntypes_; b++) m = std::max(m, cutoff(a, b));
    return m;
  }

  void upload(const CsrInput &in) override;
  void run(const RunFlags &fl) override;
  void fetch(double *energy, double *forces, double *virial, double *eatom) override;
  void synchronize() override { HIP_CHECK(hipSetDevice(device_)); HIP_CHECK(hipStreamSynchronize(stream_)); }
  void set_profile(bool on) override { profile_ = on; }
  const std::vector<StageTime> &stage_times() override;
  int64_t last_edge_count() override
  {
    synchronize();
    long long e = 0;
    if (n_ > 0) HIP_CHECK(hipMemcpy(&e, eoff_.as<long long>() + n_, sizeof(e), hipMemcpyDeviceToHost));
    return e;
  }
  void debug_radial(int m, const double *x, const int *mu_j, double *Rz, double *dRz) override;
  void debug_copy(int64_t bytes) override
  {
    HIP_CHECK(hipSetDevice(device_));
    const long long nd = std::max<int64_t>(bytes / 8, 1);
    DevBuf a, b;
    a.ensure(nd * 8);
    b.ensure(nd * 8);
    HIP_CHECK(hipMemsetAsync(a.p, 0, nd * 8, stream_));
    hipLaunchKernelGGL(k_copy_calibration, dim3(4096), dim3(256), 0, stream_, a.as<double>(), b.as<double>(), nd);
    HIP_CHECK(hipGetLastError());
    HIP_CHECK(hipStreamSynchronize(stream_));
  }

 private:
  std::shared_ptr<const Model1L> model_;
  int ntypes_;
  std::vector<int> type2mu_;
  int device_, ncu_ = 256;
  std::string arch_;
  bool jit_all_ = false;
  hipStream_t stream_ = nullptr;
  bool profile_ = false;
  std::vector<std::pair<hipEvent_t, hipEvent_t>> events_;
  std::vector<std::string> ev_names_;
  size_t ev_used_ = 0;
  std::vector<StageTime> times_;

  // model dimensions
  int CP_ = 0, CFP_ = 0;    // channel widths padded to 16 / 32 / 64: the widths of every per-atom tensor on the device
  int lmax_ = 0, nl_ = 0, nlm_ = 0, C_ = 0, CF_ = 0, nAA_ = 0, nAAA_ = 0, nAAAA_ = 0, nrho_ = 0, nel_ = 0;
  bool order4_ = true, aaa_a_ = false;
  int hb_ = 4, ks0_ = 2, nob_ = 0, noutp_ = 0, w2_in_lds_ = 1;
  size_t rad_lds_ = 0;
  int drow_[16];
  ShCoef sh_{};

  // device tables
  DevBuf cut_, z_, w0_, w1_, w2_, shift_;
  DevFc<T> fcA1_, fcAA1_, fcAA2_;
  DevProd pAA_, pAAA_, pAAAA_;
  DevBuf redWF_[4], redWB_[4], redFn_[4];
  ReduceDev<T> red_{};
  DevBuf eW_[7];
  EnergyDev en_{};

  // structure
  int n_ = 0;
  int64_t nb_ = 0;
  bool have_rij_ = false;
  DevBuf mu_, offset_, j_, rij_, x_, image_, shifts_, tiles_;
  int ntiles_ = 0;
  // pass buffers
  DevBuf count_, eoff_, zero_, ei_, ej_, emu_, rh_, r_, xr_, rc_, Rz_, dRz_;
  DevBuf A_, A1_, AA_, AA1_, AA2_, AAA_, AAAA_, gA_, gA1_, gAA_, gAA1_, gAA2_, gAAA_, gAAAA_, rho_, grho_;
  DevBuf f_, eatom_, scal_;    // scal: energy, virial[6]
  bool ran_ = false, ran_forces_ = false, ran_eatom_ = false;

  void probe_mfma();
  void build();
  void prof_begin(const char *name);
  void prof_end();
  template<class F> void stage(const char *name, F &&f)
  {
    prof_begin(name);
    f();
    HIP_CHECK(hipGetLastError());
    prof_end();
  }
  void launch_gemm(DevJobs<T> &J, int kb0, int kb1, int nb, const T *X0, int nf0, const T *X1, int nf1, T *out, int nfo, int accumulate);
  void launch_radial(long long e_begin, long long e_count, const double *x, const int *emu, T *Rz, T *dRz,
                     const long long *n_edges);
};

template<class T> void Engine1L<T>::prof_begin(const char *name)
{
  if (!profile_) return;
  if (ev_used_ == events_.size()) {
    hipEvent_t a, b;
    HIP_CHECK(hipEventCreate(&a));
    HIP_CHECK(hipEventCreate(&b));
    events_.push_back({a, b});
    ev_names_.push_back("");
  }
  ev_names_[ev_used_] = name;
  HIP_CHECK(hipEventRecord(events_[ev_used_].first, stream_));
}

template<class T> void Engine1L<T>::prof_end()
{
  if (!profile_) return;
  HIP_CHECK(hipEventRecord(events_[ev_used_].second, stream_));
  ev_used_++;
}

template<class T> const std::vector<StageTime> &Engine1L<T>::stage_times()
{
  synchronize();
  times_.clear();
  for (size_t q = 0; q < ev_used_; q++) {
    float ms = 0.f;
    HIP_CHECK(hipEventElapsedTime(&ms, events_[q].first, events_[q].second));
    auto it = std::find_if(times_.begin(), times_.end(), [&](const StageTime &s) { return s.name == ev_names_[q]; });
    if (it == times_.end()) {
      times_.push_back({ev_names_[q], 0.0, 0});
      it = times_.end() - 1;
    }
    it->ms += ms;
    it->launches++;
  }
  return times_;
}

// which accumulator row each (lane / 16, register) of a 16x16x4 MFMA holds; the column must be lane % 16
template<class T> void Engine1L<T>::probe_mfma()
{
  std::vector<T> A(64), B(64), D(256);
  for (int i = 0; i < 16; i++)
    for (int k = 0; k < 4; k++) {
      A[i * 4 + k] = (T) (1 + i + 16 * k);
      B[k * 16 + i] = (T) ((k == 0 ? 1 : k == 1 ? 3 : k == 2 ? 7 : 11) * (i + 1));
    }
  DevBuf dA, dB, dD;
  upload_vec(dA, A);
  upload_vec(dB, B);
  dD.ensure(256 * sizeof(T));
  hipLaunchKernelGGL(k_mfma_probe<T>, dim3(1), dim3(64), 0, stream_, dA.as<T>(), dB.as<T>(), dD.as<T>());
  HIP_CHECK(hipGetLastError());
  HIP_CHECK(hipStreamSynchronize(stream_));
  HIP_CHECK(hipMemcpy(D.data(), dD.p, 256 * sizeof(T), hipMemcpyDeviceToHost));
  double ref[16][16];
  for (int i = 0; i < 16; i++)
    for (int j = 0; j < 16; j++) {
      double s = 0;
      for (int k = 0; k < 4; k++) s += (double) A[i * 4 + k] * (double) B[k * 16 + j];
      ref[i][j] = s;
    }
  for (int g = 0; g < 4; g++)
    for (int v = 0; v < 4; v++) {
      int row = -1;
      for (int i = 0; i < 16 && row < 0; i++) {
        bool ok = true;
        for (int c = 0; c < 16 && ok; c++) ok = (double) D[(g * 16 + c) * 4 + v] == ref[i][c];
        if (ok) row = i;
      }
      if (row < 0) throw Error("MFMA 16x16x4 accumulator layout of this device is not the one the kernels assume");
      drow_[g * 4 + v] = row;
    }
  // the 16 (group, register) pairs must cover the 16 rows
  int seen = 0;
  for (int q = 0; q < 16; q++) seen |= 1 << drow_[q];
  if (seen != 0xFFFF) throw Error("MFMA 16x16x4 accumulator layout probe failed");
}

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
    upload_vec(cut_, cut);
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
  {
    if (m.mlp_rad.size() != 3) throw Error("GRACE-1L: the GPU radial kernel implements 3-layer radial MLPs (file has " +
                                           std::to_string(m.mlp_rad.size()) + ")");
    const MLPLayer &L0 = m.mlp_rad[0], &L1 = m.mlp_rad[1], &L2 = m.mlp_rad[2];
    const int H1 = L0.n_out, H2 = L1.n_out;
    if (m.nradbase > kMaxRadBasis) throw Error("GRACE-1L: nradbase > 16 not supported");
    const int hmax = std::max(H1, H2);
    if (hmax <= 64) hb_ = 4;
    else if (hmax <= 128) hb_ = 8;
    else throw Error("GRACE-1L: radial MLP hidden width > 128 not supported");
    ks0_ = round_up(m.nradbase, 4) / 4;
    const int nout = CP_ * nl_;
    noutp_ = round_up(nout, 16);
    nob_ = noutp_ / 16;
    std::vector<T> w0((size_t) hb_ * ks0_ * 64, (T) 0), w1((size_t) hb_ * hb_ * 4 * 64, (T) 0),
        w2((size_t) nob_ * hb_ * 4 * 64, (T) 0);
    for (int rb = 0; rb < hb_; rb++)
      for (int s = 0; s < ks0_; s++)
        for (int lane = 0; lane < 64; lane++) {
          const int g = lane >> 4, r = lane & 15, kin = 4 * s + g, out = rb * 16 + r;
          if (kin < L0.n_in && out < H1) w0[((size_t) rb * ks0_ + s) * 64 + lane] = (T) (L0.norm * L0.W[(size_t) kin * H1 + out]);
        }
    for (int rb = 0; rb < hb_; rb++)
      for (int kb = 0; kb < hb_; kb++)
        for (int s = 0; s < 4; s++)
          for (int lane = 0; lane < 64; lane++) {
            const int g = lane >> 4, r = lane & 15, in = kb * 16 + drow_[g * 4 + s], out = rb * 16 + r;
            if (in < H1 && out < H2)
              w1[(((size_t) rb * hb_ + kb) * 4 + s) * 64 + lane] = (T) (L1.norm * L1.W[(size_t) in * H2 + out]);
          }
    for (int cb = 0; cb < nob_; cb++)
      for (int kb = 0; kb < hb_; kb++)
        for (int s = 0; s < 4; s++)
          for (int lane = 0; lane < 64; lane++) {
            const int g = lane >> 4, cc = lane & 15, in = kb * 16 + drow_[g * 4 + s], col = cb * 16 + cc;
            const int l = col / CP_, n = col % CP_, o = n * nl_ + l;    // file order o = n nl + l (fused_1l.cpp:123)
            if (in < H2 && col < nout && n < C_) {
              w2[(((size_t) cb * hb_ + kb) * 4 + s) * 64 + lane] = (T) (L2.norm * L2.W[(size_t) in * L2.n_out + o]);
            }
          }
    upload_vec(w0_, w0); upload_vec(w1_, w1); upload_vec(w2_, w2);
    const size_t base = (w0.size() + w1.size()) * sizeof(T);
    w2_in_lds_ = base + w2.size() * sizeof(T) <= 150 * 1024;
    rad_lds_ = base + (w2_in_lds_ ? w2.size() * sizeof(T) : 0);
  }

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
    fcA1_.build(m.fc_A1, liveA1, nlm_, CP_, CP_, CFP_, drow_);
    fcAA1_.build(m.fc_AA1, liveAA1, nlm_, CFP_, CP_, CFP_, drow_);
    if (order4_) fcAA2_.build(m.fc_AA2, liveAA2, nlm_, CFP_, CP_, CFP_, drow_);
  }

  // ---- rho reduce: weights per collected function in MFMA fragment order (fused_cpu.h:1202-1273)
  {
    const ReduceWeights *rw[4] = {&m.red_A, &m.red_AA, &m.red_AAA, &m.red_AAAA};
    const int nfun[4] = {nlm_, nAA_, nAAA_, nAAAA_};
    red_.nsrc = order4_ ? 4 : 3;
    red_.nrho = nrho_;
    red_.nbr = (nrho_ + 15) / 16;
    red_.ksr = (nrho_ + 3) / 4;
    for (int q = 0; q < 16; q++) red_.drow[q] = drow_[q];
    const int krp = red_.ksr * 4;
    for (int s = 0; s < red_.nsrc; s++) {
      const ReduceWeights &w = *rw[s];
      std::vector<int> fn(w.collect_ind);
      std::sort(fn.begin(), fn.end());
      fn.erase(std::unique(fn.begin(), fn.end()), fn.end());
      const int nc = (int) fn.size(), nin = w.n_in, ninp = s == 0 ? CP_ : CFP_;
      std::vector<T> WF, WB;
      std::vector<double> M((size_t) nin * nrho_), Mt((size_t) nrho_ * nin);
      for (int mu = 0; mu < nel_; mu++)
        for (int u = 0; u < nc; u++) {
          std::fill(M.begin(), M.end(), 0.0);
          for (size_t c = 0; c < w.collect_ind.size(); c++) {
            if (w.collect_ind[c] != fn[u]) continue;
            const int tile = w.w_l_tile[c];
            for (int k = 0; k < nrho_; k++)
              for (int n = 0; n < nin; n++)
                M[(size_t) n * nrho_ + k] += w.norm * w.W[(((size_t) mu * nrho_ + k) * nin + n) * w.w_shape + tile];
          }
          for (int k = 0; k < nrho_; k++)
            for (int n = 0; n < nin; n++) Mt[(size_t) k * nin + n] = M[(size_t) n * nrho_ + k];
          pack_fragments<T>(M, nin, nrho_, ninp, red_.nbr * 16, WF);      // X[atom][n] . M[n][k]
          pack_fragments<T>(Mt, nrho_, nin, krp, ninp, WB);               // grho[atom][k] . Mt[k][n]
        }
      upload_vec(redWF_[s], WF);
      upload_vec(redWB_[s], WB);
      upload_vec(redFn_[s], fn);
      red_.WF[s] = redWF_[s].template as<T>();
      red_.WB[s] = redWB_[s].template as<T>();
      red_.fn[s] = redFn_[s].template as<int>();
      red_.ncol[s] = nc;
      red_.nin[s] = ninp;
      red_.stride[s] = nfun[s];
    }
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
    en_.out_scale = m.output_scale;
    en_.shift = shift_.as<double>();
  }
  scal_.ensure(8 * sizeof(double));
  zero_.ensure(2 * sizeof(int));
}

template<class T> void Engine1L<T>::upload(const CsrInput &in)
{
  HIP_CHECK(hipSetDevice(device_));
  if (in.n < 0) throw InvalidArgument("negative atom count");
  const bool table = in.x && in.image && in.shifts;
  if ((in.rij != nullptr) == (in.x || in.image || in.shifts) || (!in.rij && !table))
    throw InvalidArgument("give rij or positions, image and shifts");
  const int n = in.n;
  std::vector<int> mu(n);
  for (int a = 0; a < n; a++) {
    if (in.types[a] < 1 || in.types[a] > ntypes_) throw InvalidArgument("types must be 1 .. len(species)");
    mu[a] = type2mu_[in.types[a]];
    if (mu[a] < 0)
      throw Error("GRACE-1L: atom " + std::to_string(a) + " of unmapped type " + std::to_string(in.types[a]) + " in the atom list");
  }
  if (in.offset[0] != 0) throw InvalidArgument("offset[0] must be 0 and offset[-1] == len(j)");
  for (int a = 0; a < n; a++)
    if (in.offset[a + 1] < in.offset[a]) throw InvalidArgument("offset must be non-decreasing");
  const int64_t nb = in.offset[n];
  for (int64_t q = 0; q < nb; q++) {
    if (in.j[q] < 0 || in.j[q] >= n) throw InvalidArgument("j must index atoms 0 .. len(types)-1");
    if (in.image && (in.image[q] < 0 || in.image[q] >= in.nimages)) throw InvalidArgument("image must index rows of shifts");
  }
  HIP_CHECK(hipStreamSynchronize(stream_));
  n_ = n;
  nb_ = nb;
  have_rij_ = in.rij != nullptr;
  auto put = [&](DevBuf &b, const void *src, size_t bytes) {
    b.ensure(std::max<size_t>(bytes, 8));
    if (bytes) HIP_CHECK(hipMemcpyAsync(b.p, src, bytes, hipMemcpyHostToDevice, stream_));
  };
  put(mu_, mu.data(), sizeof(int) * n);
  // tiles of 16 atoms of one element, in atom order within an element
  std::vector<int> tiles;
  {
    std::vector<int> ord(n);
    std::iota(ord.begin(), ord.end(), 0);
    std::stable_sort(ord.begin(), ord.end(), [&](int a, int b) { return mu[a] < mu[b]; });
    for (int q = 0; q < n;) {
      int cnt = 0;
      const int m0 = mu[ord[q]];
      while (cnt < 16 && q < n && mu[ord[q]] == m0) { tiles.push_back(ord[q]); q++; cnt++; }
      while (cnt < 16) { tiles.push_back(-1); cnt++; }
    }
  }
  ntiles_ = (int) tiles.size() / 16;
  put(tiles_, tiles.data(), sizeof(int) * tiles.size());
  static_assert(sizeof(long long) == sizeof(int64_t), "offset type");
  put(offset_, in.offset, sizeof(int64_t) * (n + 1));
  put(j_, in.j, sizeof(int) * nb);
  if (have_rij_) put(rij_, in.rij, sizeof(double) * 3 * nb);
  else {
    put(x_, in.x, sizeof(double) * 3 * n);
    put(image_, in.image, sizeof(int) * nb);
    put(shifts_, in.shifts, sizeof(double) * 3 * in.nimages);
  }
  HIP_CHECK(hipStreamSynchronize(stream_));    // the host copies (mu) go out of scope
  ran_ = false;
}

template<class T>
void Engine1L<T>::launch_gemm(DevJobs<T> &J, int kb0, int kb1, int nb, const T *X0, int nf0, const T *X1, int nf1, T *out, int nfo,
                              int accumulate)
{
  if (J.d.njobs == 0 || ntiles_ == 0) return;
  const int ksm = std::max(kb0, kb1) * 4;
  const size_t lds = (size_t) kGemmMaxSeg * nb * ksm * 64 * sizeof(T);
  const dim3 grid(J.d.njobs, (ntiles_ + 4 * kGemmTilesPerWave - 1) / (4 * kGemmTilesPerWave));
#define GR_GEMM(A_, B_, C_)                                                                                            \
  {                                                                                                                    \
    auto kern = k_gemm_jobs<T, A_, B_, C_>;                                                                            \
    if (lds > 48 * 1024)                                                                                               \
      HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds)); \
    hipLaunchKernelGGL(kern, grid, dim3(256), lds, stream_, J.d, X0, nf0, X1, nf1, out, nfo, tiles_.as<int>(), ntiles_, accumulate); \
  }
#define GR_GEMM_C(A_, B_)                                                                                              \
  switch (nb) {                                                                                                        \
    case 1: GR_GEMM(A_, B_, 1) break;                                                                                  \
    case 2: GR_GEMM(A_, B_, 2) break;                                                                                  \
    case 4: GR_GEMM(A_, B_, 4) break;                                                                                  \
    default: throw Error("unsupported channel widths");                                                                \
  }
  switch (kb0 * 10 + kb1) {
    case 11: GR_GEMM_C(1, 1) break;
    case 12: GR_GEMM_C(1, 2) break;
    case 14: GR_GEMM_C(1, 4) break;
    case 21: GR_GEMM_C(2, 1) break;
    case 22: GR_GEMM_C(2, 2) break;
    case 24: GR_GEMM_C(2, 4) break;
    case 41: GR_GEMM_C(4, 1) break;
    case 42: GR_GEMM_C(4, 2) break;
    case 44: GR_GEMM_C(4, 4) break;
    default: throw Error("unsupported channel widths");
  }
#undef GR_GEMM_C
#undef GR_GEMM
}

template<class T>
void Engine1L<T>::launch_radial(long long e_begin, long long e_count, const double *x, const int *emu, T *Rz, T *dRz,
                                const long long *n_edges)
{
  RadialArgs<T> ra{};
  ra.n_edges = n_edges;
  ra.e_begin = e_begin;
  ra.e_count = e_count;
  ra.x = x;
  ra.emu = emu;
  ra.w0 = w0_.as<T>(); ra.w1 = w1_.as<T>(); ra.w2 = w2_.as<T>();
  ra.z = z_.as<T>();
  ra.Rz = Rz; ra.dRz = dRz;
  ra.nrb = model_->nradbase; ra.p = model_->radial_basis_p; ra.ks0 = ks0_;
  ra.nob = nob_; ra.noutp = noutp_;
  ra.C = CP_; ra.nel = nel_; ra.act = model_->radial_activation;
  ra.w2_in_lds = w2_in_lds_;
  for (int q = 0; q < 16; q++) ra.drow[q] = drow_[q];
  const int threads = hb_ == 4 ? 512 : 256;
  const int act = model_->radial_activation;
  auto kern = hb_ == 4 ? (act == 1 ? k_radial<T, 4, 1> : k_radial<T, 4, 0>) : (act == 1 ? k_radial<T, 8, 1> : k_radial<T, 8, 0>);
  HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
  hipLaunchKernelGGL(kern, dim3(ncu_), dim3(threads), rad_lds_, stream_, ra);
}

template<class T> void Engine1L<T>::run(const RunFlags &fl)
{
  HIP_CHECK(hipSetDevice(device_));
  ev_used_ = 0;
  const int n = n_;
  // ---- outputs
  f_.ensure(std::max<size_t>((size_t) 3 * n, 1) * sizeof(double));
  eatom_.ensure(std::max<size_t>(n, 1) * sizeof(double));
  HIP_CHECK(hipMemsetAsync(f_.p, 0, (size_t) 3 * n * sizeof(double), stream_));
  HIP_CHECK(hipMemsetAsync(scal_.p, 0, 8 * sizeof(double), stream_));
  ran_ = true;
  ran_forces_ = !fl.energy_only;
  ran_eatom_ = fl.eatom;
  if (n == 0) return;
  // ---- bond filter and compaction
  count_.ensure(sizeof(int) * n);
  eoff_.ensure(sizeof(long long) * (n + 1));
  {
    const int init[2] = {-1, -1};
    HIP_CHECK(hipMemcpyAsync(zero_.p, init, sizeof(init), hipMemcpyHostToDevice, stream_));
  }
  BondSrc src{};
  src.mu = mu_.as<int>(); src.offset = offset_.as<long long>(); src.j = j_.as<int>();
  src.rij = have_rij_ ? rij_.as<double>() : nullptr;
  src.x = have_rij_ ? nullptr : x_.as<double>();
  src.image = have_rij_ ? nullptr : image_.as<int>();
  src.shifts = have_rij_ ? nullptr : shifts_.as<double>();
  src.cut = cut_.as<double>(); src.nel = nel_;
  const size_t ecap = (size_t) std::max<int64_t>(nb_, 1);
  ei_.ensure(ecap * sizeof(int)); ej_.ensure(ecap * sizeof(int)); emu_.ensure(ecap * sizeof(int));
  rh_.ensure(ecap * 3 * sizeof(double)); r_.ensure(ecap * sizeof(double)); xr_.ensure(ecap * sizeof(double));
  rc_.ensure(ecap * sizeof(double));
  Edges ed{ei_.as<int>(), ej_.as<int>(), emu_.as<int>(), rh_.as<double>(), r_.as<double>(), xr_.as<double>(), rc_.as<double>()};
  const int wpb = 4;
  stage("edge_count", [&] { hipLaunchKernelGGL(k_edge_count, dim3((n + wpb - 1) / wpb), dim3(64 * wpb), 0, stream_, src, n, count_.as<int>(), zero_.as<int>()); });
  stage("edge_scan", [&] { hipLaunchKernelGGL(k_scan, dim3(1), dim3(1024), 0, stream_, count_.as<int>(), n, eoff_.as<long long>()); });
  stage("edge_fill", [&] { hipLaunchKernelGGL(k_edge_fill, dim3((n + wpb - 1) / wpb), dim3(64 * wpb), 0, stream_, src, n, eoff_.as<long long>(), ed); });

  // ---- radial functions of all edges
  Rz_.ensure(ecap * noutp_ * sizeof(T));
  if (!fl.energy_only) dRz_.ensure(ecap * noutp_ * sizeof(T));
  else dRz_.ensure(ecap * noutp_ * sizeof(T));
  stage("radial_mlp", [&] {
    launch_radial(0, -1, xr_.as<double>(), emu_.as<int>(), Rz_.as<T>(), dRz_.as<T>(), eoff_.as<long long>() + n);
  });

  // ---- per-atom tensors (whole structure in one chunk), channel widths padded
  const size_t na = (size_t) n;
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

  const int sthreads = round_up(nl_ * CP_, 64);
  ScatterArgs<T> sa{};
  sa.eoff = eoff_.as<long long>(); sa.rh = rh_.as<double>(); sa.Rz = Rz_.as<T>(); sa.A = A_.as<T>();
  sa.a0 = 0; sa.C = CP_; sa.nl = nl_; sa.nlm = nlm_; sa.noutp = noutp_; sa.sh = sh_;
  stage("scatter_A", [&] {
    if (lmax_ <= 4) hipLaunchKernelGGL((k_scatter_a<T, 9>), dim3(n), dim3(sthreads), 0, stream_, sa);
    else hipLaunchKernelGGL((k_scatter_a<T, 13>), dim3(n), dim3(sthreads), 0, stream_, sa);
  });

  const int *tiles = tiles_.as<int>();
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
  if (aaa_a_ && CP_ != CFP_) throw Error("GRACE-1L: AAA = AA1 x A needs equal A and FC widths");
  const T *Ar = aaa_a_ ? A : A1;
  stage("fc_A1", [&] { launch_gemm(fcA1_.fwd, ka, ka, kf, A, nlm_, A, nlm_, A1, nlm_, 0); });
  prod_fwd("prod_AA", pAA_, A1, A1, AA, nlm_, nlm_);
  stage("fc_AA1", [&] { launch_gemm(fcAA1_.fwd, kf, ka, kf, AA, nAA_, A, nlm_, AA1, nAA_, 0); });
  prod_fwd("prod_AAA", pAAA_, AA1, Ar, AAA, nAA_, nlm_);
  if (order4_) {
    stage("fc_AA2", [&] { launch_gemm(fcAA2_.fwd, kf, ka, kf, AA, nAA_, A, nlm_, AA2, nAA_, 0); });
    prod_fwd("prod_AAAA", pAAAA_, AA2, AA2, AAAA, nAA_, nAA_);
  }
  stage("reduce_rho", [&] {
#define GR_RED(KA, KF) hipLaunchKernelGGL((k_reduce_fwd<T, KA, KF>), dim3(ntiles_), dim3(256), 0, stream_, red_, mu_.as<int>(), tiles, \
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
    hipLaunchKernelGGL(k_energy, dim3(n), dim3(64), 0, stream_, en_, mu_.as<int>(), 0, n, rho_.as<double>(), grho_.as<double>(),
                       fl.eatom ? eatom_.as<double>() : nullptr, scal_.as<double>(), fl.energy_only ? 0 : 1);
  });
  if (fl.energy_only) return;

  // ---- reverse
  gA_.ensure(na * nlm_ * CP_ * sizeof(T));
  gA1_.ensure(na * nlm_ * CFP_ * sizeof(T));
  gAA_.ensure(na * nAA_ * CFP_ * sizeof(T));
  gAA1_.ensure(na * nAA_ * CFP_ * sizeof(T));
  gAAA_.ensure(na * nAAA_ * CFP_ * sizeof(T));
  if (order4_) {
    gAA2_.ensure(na * nAA_ * CFP_ * sizeof(T));
    gAAAA_.ensure(na * nAAAA_ * CFP_ * sizeof(T));
  }
  T *gA = gA_.as<T>(), *gA1 = gA1_.as<T>(), *gAA = gAA_.as<T>(), *gAA1 = gAA1_.as<T>(), *gAA2 = gAA2_.as<T>(),
    *gAAA = gAAA_.as<T>(), *gAAAA = gAAAA_.as<T>();
  stage("zero_grads", [&] {
    HIP_CHECK(hipMemsetAsync(gA, 0, na * nlm_ * CP_ * sizeof(T), stream_));
    HIP_CHECK(hipMemsetAsync(gA1, 0, na * nlm_ * CFP_ * sizeof(T), stream_));
    HIP_CHECK(hipMemsetAsync(gAA, 0, na * nAA_ * CFP_ * sizeof(T), stream_));
    // with the specialised product kernels gAA1 and gAA2 are written (not accumulated) by their first producer
    if (!jit_all_) HIP_CHECK(hipMemsetAsync(gAA1, 0, na * nAA_ * CFP_ * sizeof(T), stream_));
    HIP_CHECK(hipMemsetAsync(gAAA, 0, na * nAAA_ * CFP_ * sizeof(T), stream_));
    if (order4_) {
      if (!jit_all_) HIP_CHECK(hipMemsetAsync(gAA2, 0, na * nAA_ * CFP_ * sizeof(T), stream_));
      HIP_CHECK(hipMemsetAsync(gAAAA, 0, na * nAAAA_ * CFP_ * sizeof(T), stream_));
    }
  });
  stage("reduce_rho_bwd", [&] {
    int njobs = 0;
    for (int s = 0; s < red_.nsrc; s++) njobs += red_.ncol[s];
    hipLaunchKernelGGL(k_reduce_bwd<T>, dim3(ntiles_, njobs), dim3(64), 0, stream_, red_, mu_.as<int>(), tiles, grho_.as<double>(), gA, gAA,
                       gAAA, gAAAA);
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
      launch_gemm(F.bwd_l, kf, kf, kl, g, nfl, g, nfl, gXl, nfl, 1);
      launch_gemm(F.bwd_r, kf, kf, ka, g, nfl, g, nfl, gXr, nlm_, 1);
    });
  };
  if (order4_) {
    prod_bwd("prod_AAAA_bwd", pAAAA_, AA2, AA2, gAAAA, gAA2, gAA2, nAA_, nAA_, 0, 0);
    fc_bwd("fc_AA2_bwd", fcAA2_, gAA2, gAA, gA, nAA_, kf);
  }
  prod_bwd("prod_AAA_bwd", pAAA_, AA1, Ar, gAAA, gAA1, aaa_a_ ? gA : gA1, nAA_, nlm_, 0, 1);
  fc_bwd("fc_AA1_bwd", fcAA1_, gAA1, gAA, gA, nAA_, kf);
  prod_bwd("prod_AA_bwd", pAA_, A1, A1, gAA, gA1, gA1, nlm_, nlm_, 1, 1);
  fc_bwd("fc_A1_bwd", fcA1_, gA1, gA, gA, nlm_, ka);

  BondBwdArgs<T> ba{};
  ba.eoff = eoff_.as<long long>(); ba.ej = ej_.as<int>(); ba.rh = rh_.as<double>(); ba.r = r_.as<double>(); ba.rc = rc_.as<double>();
  ba.Rz = Rz_.as<T>(); ba.dRz = dRz_.as<T>(); ba.gA = gA;
  ba.f = f_.as<double>(); ba.virial = scal_.as<double>() + 1;
  ba.a0 = 0; ba.C = CP_; ba.nl = nl_; ba.nlm = nlm_; ba.noutp = noutp_; ba.sh = sh_;
  for (int q = 0; q < 16; q++) ba.drow[q] = drow_[q];
  stage("bond_bwd", [&] {
    const size_t lds = ((size_t) nl_ * (CP_ / 4) * 64 + (size_t) 4 * 16 * nlm_ * 4) * sizeof(T);
    switch (CP_ / 16) {
      case 1: hipLaunchKernelGGL((k_bond_bwd<T, 1>), dim3(n), dim3(256), lds, stream_, ba); break;
      case 2: hipLaunchKernelGGL((k_bond_bwd<T, 2>), dim3(n), dim3(256), lds, stream_, ba); break;
      default: hipLaunchKernelGGL((k_bond_bwd<T, 4>), dim3(n), dim3(256), lds, stream_, ba); break;
    }
  });
}

template<class T> void Engine1L<T>::fetch(double *energy, double *forces, double *virial, double *eatom)
{
  HIP_CHECK(hipSetDevice(device_));
  if (!ran_) throw Error("fetch() before run()");
  HIP_CHECK(hipStreamSynchronize(stream_));
  if (n_ > 0) {
    int zb[2];
    HIP_CHECK(hipMemcpy(zb, zero_.p, sizeof(zb), hipMemcpyDeviceToHost));
    if (zb[0] >= 0)    // bonds.h:49-62
      throw Error("two atoms at the same position (a bond of length 0 between atoms " + std::to_string(zb[0]) + " and " +
                  std::to_string(zb[1]) + " of the neighbour list): not a physical structure");
  }
  double s[8];
  HIP_CHECK(hipMemcpy(s, scal_.p, sizeof(s), hipMemcpyDeviceToHost));
  if (energy) *energy = s[0];
  if (virial && ran_forces_)
    for (int k = 0; k < 6; k++) virial[k] = s[1 + k];
  if (forces && ran_forces_ && n_ > 0) HIP_CHECK(hipMemcpy(forces, f_.p, sizeof(double) * 3 * n_, hipMemcpyDeviceToHost));
  if (eatom && ran_eatom_ && n_ > 0) HIP_CHECK(hipMemcpy(eatom, eatom_.p, sizeof(double) * n_, hipMemcpyDeviceToHost));
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

}    // namespace

std::unique_ptr<Engine> make_engine_1l(std::shared_ptr<const Model1L> model, int ntypes, const std::vector<int> &type2mu,
                                       int precision, int device)
{
  if (precision == 64) return std::make_unique<Engine1L<double>>(std::move(model), ntypes, type2mu, device);
  if (precision == 32) return std::make_unique<Engine1L<float>>(std::move(model), ntypes, type2mu, device);
  throw InvalidArgument("precision must be 64 or 32");
}

}    // namespace grhip
