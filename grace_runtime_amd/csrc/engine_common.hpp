// Host-side building blocks shared by the engines: device buffers, the CG-product tables, MFMA fragment packing, the
// tile-GEMM job lists of the FC layers, and the stream / profiling base of an engine.
#pragma once

#include "engine.hpp"
#include "jit_prod.hpp"
#include "kernels_1l.hpp"

#include <algorithm>
#include <atomic>
#include <functional>
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

// Messages of the library (choice of a chunk, retries after a failed allocation, kernels that fall back to their
// table-driven form) go to a callback the caller installs, as the reference's grace::Logger (libgrace/include/grace/
// error.h:10-15): fn(user, level, message), level 0 information, 1 warning.  Without a callback they are dropped.
typedef void (*LogCallback)(void *user, int level, const char *message);
struct LogSink {
  std::atomic<LogCallback> fn{nullptr};
  std::atomic<void *> user{nullptr};
};
inline LogSink &log_sink()
{
  static LogSink s;
  return s;
}
inline void log_message(int level, const std::string &m)
{
  const LogCallback f = log_sink().fn.load();
  if (f) f(log_sink().user.load(), level, m.c_str());
}

// Device memory held by the library's buffers and an optional cap on it (0: none).  With a cap an allocation that would
// pass it fails like one the device refuses (std::bad_alloc), which lets a GPU be shared by budget and lets the
// retry paths be exercised without exhausting the device.
inline std::atomic<long long> &dev_bytes_in_use()
{
  static std::atomic<long long> v{0};
  return v;
}
inline std::atomic<long long> &dev_bytes_limit()
{
  static std::atomic<long long> v{0};
  return v;
}

// The buffers of the engine under construction on this thread register themselves here (BufRegistry below): the engine
// can then give back the memory of its work buffers without knowing each of them.
struct DevBuf;
inline std::vector<DevBuf *> *&building_registry()
{
  static thread_local std::vector<DevBuf *> *r = nullptr;
  return r;
}

// device allocation owned by the engine
struct DevBuf {
  void *p = nullptr;
  size_t bytes = 0;
  bool model_data = false;              // allocated while the engine was built (weights, tables): kept by release_work()
  std::vector<DevBuf *> *reg = nullptr;
  DevBuf() : reg(building_registry())
  {
    if (reg) reg->push_back(this);
  }
  DevBuf(const DevBuf &) = delete;
  DevBuf &operator=(const DevBuf &) = delete;
  ~DevBuf()
  {
    release();
    if (reg) {
      auto it = std::find(reg->begin(), reg->end(), this);
      if (it != reg->end()) reg->erase(it);
    }
  }
  void release()
  {
    if (p) {
      (void) hipFree(p);
      dev_bytes_in_use() -= (long long) bytes;
    }
    p = nullptr;
    bytes = 0;
  }
  // at least `need` bytes (grown with head room; contents are not kept)
  void ensure(size_t need)
  {
    if (need <= bytes && p) return;
    release();
    const size_t want = std::max<size_t>(need + need / 8, 256);
    const long long cap = dev_bytes_limit().load();
    if (cap > 0 && dev_bytes_in_use().load() + (long long) want > cap) throw std::bad_alloc();
    hipError_t e = hipMalloc(&p, want);
    if (e != hipSuccess) {
      p = nullptr;
      (void) hipGetLastError();
      throw std::bad_alloc();
    }
    bytes = want;
    model_data = building_registry() != nullptr;
    dev_bytes_in_use() += (long long) want;
  }
  template<class U> U *as() const { return static_cast<U *>(p); }
};

// pinned host memory of the engine (allocated, never registered): staging of the small per-call transfers, so that they are
// asynchronous copies on the engine's stream with one wait instead of one blocking copy each
struct PinnedBuf {
  void *p = nullptr;
  size_t bytes = 0;
  PinnedBuf() = default;
  PinnedBuf(const PinnedBuf &) = delete;
  PinnedBuf &operator=(const PinnedBuf &) = delete;
  ~PinnedBuf() { release(); }
  void release()
  {
    if (p) (void) hipHostFree(p);
    p = nullptr;
    bytes = 0;
  }
  void ensure(size_t need)
  {
    if (need <= bytes && p) return;
    release();
    const size_t want = std::max<size_t>(need + need / 8, 4096);
    if (hipHostMalloc(&p, want, hipHostMallocDefault) != hipSuccess) {
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
inline HostProd build_prod(const CGProduct &p, const std::vector<char> &need, int nleft, int nright)
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
  long long nseg[2] = {0, 0};    // segments that read source 0 / source 1
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
    nseg[0] = nseg[1] = 0;
    for (int src : h.seg_src) nseg[src ? 1 : 0]++;
    d.max_seg = 0;
    for (size_t q = 0; q + 1 < h.seg_off.size(); q++) d.max_seg = std::max(d.max_seg, h.seg_off[q + 1] - h.seg_off[q]);
  }
  void set_rows(const int *drow) { for (int q = 0; q < 16; q++) d.drow[q] = drow[q]; }
};

// One FC layer as three job lists (forward, reverse into the left input, reverse into the right input) over
// fragment-ordered weight tiles.  Widths are the padded ones (multiples of 16; padding weights are zero).
template<class T> struct DevFc {
  DevBuf WlF, WrF, WlTF, WrTF;
  DevJobs<T> fwd, bwd_l, bwd_r;
  // the reverse of a layer whose two inputs are ONE tensor (A1 = FC(A, A)): a job per input function that takes the left
  // segment and the right segments together (source 0: left weights, source 1: right weights; both sources are the output
  // adjoint), one launch and one read-add-write of the input adjoint instead of two; empty unless build() was asked for it
  DevJobs<T> bwd_lr;
  bool have_lr = false;
  int nil = 0, nir = 0, no = 0;    // padded widths
  // nfr: functions of the right-input tensor; livef: outputs that are computed; cover_left: the reverse into the left
  // input has a job for EVERY function (without segments for outputs that are not computed), so that a launch that
  // overwrites instead of accumulating leaves no row of the adjoint unwritten
  void build(const FCWeights &w, const std::vector<char> &livef, int nfr, int nil_p, int nir_p, int no_p, const int *drow,
             bool cover_left = false, bool same_input = false)
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
      if (!livef[f]) {
        if (cover_left) { hl.job(f, 1.0); hl.end_job(); }
        continue;
      }
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
    have_lr = same_input && nil == nir && nfr == w.n_funcs;
    if (have_lr) {
      typename DevJobs<T>::Host hlr;
      for (int r = 0; r < nfr; r++) {
        if (!livef[r] && conn_from[r].empty()) continue;
        hlr.job(r, 1.0);
        if (livef[r]) hlr.seg(0, r, w.w_tile_left[r], w.norm_out_factor[r]);
        for (int c : conn_from[r]) hlr.seg(1, w.collect_to[c], w.w_tile_right[c], w.norm_out_factor[w.collect_to[c]]);
        hlr.end_job();
      }
      bwd_lr.build(hlr, WlTF.as<T>(), WrTF.as<T>());
      bwd_lr.set_rows(drow);
    }
  }
};

// The reverse of two FC layers that read the same two inputs (AA1 = FC1(AA, A), AA2 = FC2(AA, A)) as ONE pair of job
// lists: the adjoint of the shared left input is read, added to and written once instead of twice, and so is the
// adjoint of the right input.  Source 0 of a segment is the output adjoint of the first layer, source 1 of the second.
template<class T> struct DevFcPairBwd {
  DevJobs<T> bwd_l, bwd_r;
  // cover_left: the reverse into the left input has a job for EVERY function (those no live output reads get one without
  // segments), so that a launch that overwrites instead of accumulating leaves no row of the adjoint unwritten
  void build(const FCWeights &w1, const std::vector<char> &live1, const DevFc<T> &F1, const FCWeights &w2, const std::vector<char> &live2,
             const DevFc<T> &F2, int nfr, const int *drow, bool cover_left = false)
  {
    if (w1.n_funcs != w2.n_funcs || F1.nil != F2.nil || F1.nir != F2.nir || F1.no != F2.no) throw Error("FC pair: the two layers differ in shape");
    typename DevJobs<T>::Host hl, hr;
    for (int f = 0; f < w1.n_funcs; f++) {
      if (!live1[f] && !live2[f] && !cover_left) continue;
      hl.job(f, 1.0);
      if (live1[f]) hl.seg(0, f, w1.w_tile_left[f], w1.norm_out_factor[f]);
      if (live2[f]) hl.seg(1, f, w2.w_tile_left[f], w2.norm_out_factor[f]);
      hl.end_job();
    }
    std::vector<std::vector<std::pair<int, int>>> from(nfr);    // (layer, connection)
    for (int c = 0; c < w1.n_conn; c++)
      if (live1[w1.collect_to[c]]) from[w1.collect_from[c]].push_back({0, c});
    for (int c = 0; c < w2.n_conn; c++)
      if (live2[w2.collect_to[c]]) from[w2.collect_from[c]].push_back({1, c});
    for (int r = 0; r < nfr; r++) {
      if (from[r].empty()) continue;
      hr.job(r, 1.0);
      for (const auto &lc : from[r]) {
        const FCWeights &w = lc.first ? w2 : w1;
        const int c = lc.second;
        hr.seg(lc.first, w.collect_to[c], w.w_tile_right[c], w.norm_out_factor[w.collect_to[c]]);
      }
      hr.end_job();
    }
    bwd_l.build(hl, F1.WlTF.template as<T>(), F2.WlTF.template as<T>());
    bwd_r.build(hr, F1.WrTF.template as<T>(), F2.WrTF.template as<T>());
    bwd_l.set_rows(drow); bwd_r.set_rows(drow);
  }
};


// A 3-layer radial MLP in MFMA fragment order and the launch of the persistent radial kernel (radial_x.h:11-60 of the
// reference; its spline tables are replaced by the exact network).  Output column l * CP + n of an edge holds
// R_{n,l}(x) z[mu_j][n] (file order of the last layer: o = n nl + l, libgrace/src/fused_1l.cpp:123).
template<class T> struct DevRadial {
  DevBuf w0, w1, w2, bias_i, bias_j, bias1;
  // radial tables (the reference's spline_n, libgrace/include/grace/system.h:78): intervals asked for (0: the MLP itself is
  // evaluated for every bond) and the table that exists: value and d/dx at the knots, [N + 1][noutp] each
  int spline_n = 0, table_n = 0;
  DevBuf tabF, tabD, knots, knot_mu, knot_mi, unit_z, knotF, knotD;
  // species form: the species of the engine (elements that atom types map to), element -> species, and the memory the pair
  // tables may take (the reference's spline_mb, libgrace/include/grace/system.h:85: beyond it the MLP itself is evaluated)
  std::vector<int> species_mu;
  DevBuf sp_of_mu;
  bool tables_allowed = true;
  std::string who_tables = "radial tables";
  void set_species(const std::vector<int> &present_mu, int n_elements, const std::string &who)
  {
    species_mu = present_mu;
    std::vector<int> map((size_t) n_elements, 0);
    for (size_t q = 0; q < species_mu.size(); q++) map[(size_t) species_mu[q]] = (int) q;
    upload_vec(sp_of_mu, map);
    who_tables = who;
  }
  // bytes of the tables of `n` intervals for the engine's species pairs
  double table_bytes(int n) const
  {
    const double pairs = mode == 1 ? (double) species_mu.size() * species_mu.size() : 1.0;
    return sizeof(T) == 8 ? pairs * (n + 1.0) * noutp * 16.0 : pairs * n * 4.0 * noutp * 4.0;
  }
  // fp32 engines: the same MLP in fp64, which evaluates the knots of the tables (build_double)
  std::unique_ptr<DevRadial<double>> dbl;
  template<class... A> void build_double(A &&...a)
  {
    if constexpr (sizeof(T) == 4) {
      dbl = std::make_unique<DevRadial<double>>();
      dbl->build(std::forward<A>(a)...);
    }
  }
  template<class... A> void build_species_double(A &&...a)
  {
    if constexpr (sizeof(T) == 4) {
      dbl = std::make_unique<DevRadial<double>>();
      dbl->build_species(std::forward<A>(a)...);
    }
  }
  int mode = 0;    // 1: species form (build_species)
  int hb = 4, ks0 = 2, nob = 0, noutp = 0, w2_in_lds = 1, nrb = 0, p = 0, act = 0, CP = 0, nel = 0;
  size_t lds = 0;
  int drow[16];
  void build(const std::vector<MLPLayer> &mlp, int nradbase, int basis_p, int activation, int C, int CP_, int nl, int nel_,
             const int *drow_, const std::string &who)
  {
    if (mlp.size() != 3)
      throw Error(who + ": the GPU radial kernel implements 3-layer radial MLPs (file has " + std::to_string(mlp.size()) + ")");
    const MLPLayer &L0 = mlp[0], &L1 = mlp[1], &L2 = mlp[2];
    const int H1 = L0.n_out, H2 = L1.n_out;
    if (nradbase > kMaxRadBasis) throw Error(who + ": nradbase > 16 not supported");
    const int hmax = std::max(H1, H2);
    if (hmax <= 64) hb = 4;
    else if (hmax <= 128) hb = 8;
    else throw Error(who + ": radial MLP hidden width > 128 not supported");
    nrb = nradbase; p = basis_p; act = activation; CP = CP_; nel = nel_;
    for (int q = 0; q < 16; q++) drow[q] = drow_[q];
    ks0 = round_up(nradbase, 4) / 4;
    const int nout = CP * nl;
    noutp = round_up(nout, 16);
    nob = noutp / 16;
    std::vector<T> v0((size_t) hb * ks0 * 64, (T) 0), v1((size_t) hb * hb * 4 * 64, (T) 0), v2(((size_t) nob * hb * 4 + kRadialPrefetch) * 64, (T) 0);
    for (int rb = 0; rb < hb; rb++)
      for (int s = 0; s < ks0; s++)
        for (int lane = 0; lane < 64; lane++) {
          const int g = lane >> 4, r = lane & 15, kin = 4 * s + g, out = rb * 16 + r;
          if (kin < L0.n_in && out < H1) v0[((size_t) rb * ks0 + s) * 64 + lane] = (T) (L0.norm * L0.W[(size_t) kin * H1 + out]);
        }
    for (int rb = 0; rb < hb; rb++)
      for (int kb = 0; kb < hb; kb++)
        for (int s = 0; s < 4; s++)
          for (int lane = 0; lane < 64; lane++) {
            const int g = lane >> 4, r = lane & 15, in = kb * 16 + drow[g * 4 + s], out = rb * 16 + r;
            if (in < H1 && out < H2) v1[(((size_t) rb * hb + kb) * 4 + s) * 64 + lane] = (T) (L1.norm * L1.W[(size_t) in * H2 + out]);
          }
    for (int cb = 0; cb < nob; cb++)
      for (int kb = 0; kb < hb; kb++)
        for (int s = 0; s < 4; s++)
          for (int lane = 0; lane < 64; lane++) {
            const int g = lane >> 4, cc = lane & 15, in = kb * 16 + drow[g * 4 + s], col = cb * 16 + cc;
            const int l = col / CP, n = col % CP, o = n * nl + l;
            if (in < H2 && col < nout && n < C)
              v2[(((size_t) cb * hb + kb) * 4 + s) * 64 + lane] = (T) (L2.norm * L2.W[(size_t) in * L2.n_out + o]);
          }
    upload_vec(w0, v0); upload_vec(w1, v1); upload_vec(w2, v2);
    const size_t base = (v0.size() + v1.size()) * sizeof(T);
    w2_in_lds = base + v2.size() * sizeof(T) <= 150 * 1024;
    lds = base + (w2_in_lds ? v2.size() * sizeof(T) : 0);
  }
  // Species form of GRACE-3L (libgrace/src/fused_3l.cpp:299-346, :462-493): the MLP input is [T_1..T_nrb(2x - 1),
  // emb(mu_i), emb(mu_j)], hidden layers carry a bias, and the envelope multiplies the output.  The embedding rows of
  // layer 0 become per-element tables added to its pre-activation: tab_i[mu] = norm0 (b0 + emb[mu] W0[nrb : nrb + ne]),
  // tab_j[mu] = norm0 emb[mu] W0[nrb + ne : nrb + 2 ne].
  void build_species(const std::vector<MLPLayer> &mlp, const std::vector<std::vector<double>> &bias, const std::vector<double> &emb, int ne,
                     int nradbase, int basis_p, int C, int CP_, int nl, int nel_, const int *drow_, const std::string &who)
  {
    if (mlp.size() != 3)
      throw Error(who + ": the GPU radial kernel implements 3-layer radial MLPs (file has " + std::to_string(mlp.size()) + ")");
    std::vector<MLPLayer> cut = mlp;
    const int H1 = mlp[0].n_out, H2 = mlp[1].n_out;
    cut[0].n_in = nradbase;
    cut[0].W.assign(mlp[0].W.begin(), mlp[0].W.begin() + (size_t) nradbase * H1);
    build(cut, nradbase, basis_p, 0, C, CP_, nl, nel_, drow_, who);
    mode = 1;
    const int HP = hb * 16;
    std::vector<T> ti((size_t) nel_ * HP, (T) 0), tj((size_t) nel_ * HP, (T) 0), t1((size_t) HP, (T) 0);
    for (int mu = 0; mu < nel_; mu++)
      for (int o = 0; o < H1; o++) {
        double vi = bias.size() > 0 && !bias[0].empty() ? bias[0][o] : 0.0, vj = 0.0;
        for (int e = 0; e < ne; e++) {
          const double zz = emb[(size_t) mu * ne + e];
          vi += zz * mlp[0].W[(size_t) (nradbase + e) * H1 + o];
          vj += zz * mlp[0].W[(size_t) (nradbase + ne + e) * H1 + o];
        }
        ti[(size_t) mu * HP + o] = (T) (mlp[0].norm * vi);
        tj[(size_t) mu * HP + o] = (T) (mlp[0].norm * vj);
      }
    for (int o = 0; o < H2; o++) t1[o] = (T) (bias.size() > 1 && !bias[1].empty() ? mlp[1].norm * bias[1][o] : 0.0);
    if (bias.size() > 2 && !bias[2].empty()) throw Error(who + ": a bias on the output layer of the radial MLP is not supported");
    upload_vec(bias_i, ti); upload_vec(bias_j, tj); upload_vec(bias1, t1);
  }
  // z: [nel][CP] species weights of the neighbour; e_count < 0: the edge count is read from *n_edges on the device;
  // emi: element of the central atom of every edge (species form only)
  // tables: use the radial tables when the engine was asked for them (the plain form only); otherwise, and for the debug
  // entry points, the MLP is evaluated for every bond
  void launch(hipStream_t stream, int ncu, const T *z, long long e_begin, long long e_count, const double *x, const int *emu, T *Rz, T *dRz,
              const long long *n_edges, const int *emi = nullptr, bool tables = false)
  {
    if (tables && has_tables()) {
      ensure_tables(stream, ncu);
      const long long bound = e_count >= 0 ? e_count : (long long) 1 << 40;
      const unsigned grid = (unsigned) std::max<long long>(1, std::min<long long>(bound, (long long) ncu * 32));
      hipLaunchKernelGGL((k_radial_spline<T, sizeof(T) == 4>), dim3(grid), dim3(round_up(noutp, 64)), 0, stream, n_edges, e_begin, e_count, x, emu,
                         (const T *) tabF.template as<T>(), (const T *) tabD.template as<T>(), table_n, z, CP, noutp, Rz, dRz,
                         mode == 1 ? emi : (const int *) nullptr, (const int *) sp_of_mu.as<int>(), (int) species_mu.size());
      return;
    }
    launch_mlp(stream, ncu, z, e_begin, e_count, x, emu, Rz, dRz, n_edges, emi);
  }
  // tables requested (spline_n > 0) and, in the species form, within the memory they may take
  bool has_tables()
  {
    if (spline_n <= 0) return false;
    if (mode == 0) return true;
    if (species_mu.empty()) return false;
    return tables_allowed;
  }
  // the tables as the kernels that evaluate them take them (built on first use and again after release_buffers)
  RadialTable<T> table(hipStream_t stream, int ncu, const double *x, const int *emu, const T *z)
  {
    ensure_tables(stream, ncu);
    RadialTable<T> t{};
    t.F = tabF.template as<T>();
    t.D = tabD.template as<T>();
    t.N = table_n;
    t.x = x;
    t.emu = emu;
    t.z = z;
    return t;
  }
  void ensure_tables(hipStream_t stream, int ncu)
  {
    {
      const int N = spline_n;
      if (table_n != N || !tabF.p || (sizeof(T) == 8 && !tabD.p)) {    // the MLP at the knots x = k / N, unit species weights (again after release_buffers)
        // species form: the knots of every ordered pair of species, pair after pair
        const size_t nsp = mode == 1 ? species_mu.size() : 1, npair = nsp * nsp;
        std::vector<double> xs(((size_t) N + 1) * npair);
        std::vector<int> kmi(xs.size(), 0), kmj(xs.size(), 0);
        for (size_t pr = 0; pr < npair; pr++)
          for (int k = 0; k <= N; k++) {
            const size_t q = pr * ((size_t) N + 1) + k;
            xs[q] = (double) k / N;
            if (mode == 1) { kmi[q] = species_mu[pr / nsp]; kmj[q] = species_mu[pr % nsp]; }
          }
        upload_vec(knots, xs);
        upload_vec(knot_mu, kmj);
        upload_vec(knot_mi, kmi);
        const long long nknots = (long long) xs.size();
        const size_t rows = xs.size() * noutp;
        if constexpr (sizeof(T) == 8) {
          upload_vec(unit_z, std::vector<T>((size_t) CP * std::max(nel, 1), (T) 1));
          tabF.ensure(rows * sizeof(T));
          tabD.ensure(rows * sizeof(T));
          launch_mlp(stream, ncu, unit_z.template as<T>(), 0, nknots, knots.as<double>(), knot_mu.as<int>(), tabF.template as<T>(),
                     tabD.template as<T>(), nullptr, mode == 1 ? knot_mi.as<int>() : nullptr);
        } else {
          if (!dbl) throw Error("radial tables of an fp32 engine need the fp64 form of its radial MLP");
          upload_vec(unit_z, std::vector<double>((size_t) CP * std::max(nel, 1), 1.0));
          knotF.ensure(rows * sizeof(double));
          knotD.ensure(rows * sizeof(double));
          tabF.ensure(npair * (size_t) N * 4 * noutp * sizeof(T));
          dbl->launch_mlp(stream, ncu, unit_z.as<double>(), 0, nknots, knots.as<double>(), knot_mu.as<int>(), knotF.as<double>(),
                          knotD.as<double>(), nullptr, mode == 1 ? knot_mi.as<int>() : nullptr);
          const long long tot = (long long) N * noutp;
          for (size_t pr = 0; pr < npair; pr++)
            hipLaunchKernelGGL(k_spline_coef, dim3((unsigned) ((tot + 255) / 256)), dim3(256), 0, stream,
                               (const double *) knotF.as<double>() + pr * ((size_t) N + 1) * noutp,
                               (const double *) knotD.as<double>() + pr * ((size_t) N + 1) * noutp, N, noutp,
                               tabF.as<float>() + pr * (size_t) N * 4 * noutp);
          knotF.release();    // the fp64 knots are needed for the coefficients only
          knotD.release();
        }
        table_n = N;
      }
    }
  }
  // the radial MLP itself for every edge of the range
  void launch_mlp(hipStream_t stream, int ncu, const T *z, long long e_begin, long long e_count, const double *x, const int *emu, T *Rz, T *dRz,
                  const long long *n_edges, const int *emi)
  {
    RadialArgs<T> ra{};
    ra.n_edges = n_edges;
    ra.e_begin = e_begin;
    ra.e_count = e_count;
    ra.x = x;
    ra.emu = emu;
    ra.w0 = w0.as<T>(); ra.w1 = w1.as<T>(); ra.w2 = w2.as<T>();
    ra.z = z;
    ra.Rz = Rz; ra.dRz = dRz;
    ra.nrb = nrb; ra.p = p; ra.ks0 = ks0;
    ra.nob = nob; ra.noutp = noutp;
    ra.C = CP; ra.nel = nel; ra.act = act;
    ra.w2_in_lds = w2_in_lds;
    for (int q = 0; q < 16; q++) ra.drow[q] = drow[q];
    ra.emi = emi; ra.bias_i = bias_i.as<T>(); ra.bias_j = bias_j.as<T>(); ra.bias1 = bias1.as<T>();
    if (mode == 1 && !emi) throw Error("radial kernel: the species form needs the central element of every edge");
    const int threads = radial_threads(hb, mode, w2_in_lds != 0);
    // <T, 16-row blocks of the hidden width, activation, species form, layer-2 weights in LDS>
    void (*kern)(RadialArgs<T>);
    if (w2_in_lds)
      kern = mode == 1 ? (hb == 4 ? k_radial<T, 4, 0, 1, true> : k_radial<T, 8, 0, 1, true>)
                       : hb == 4 ? (act == 1 ? k_radial<T, 4, 1, 0, true> : k_radial<T, 4, 0, 0, true>)
                                 : (act == 1 ? k_radial<T, 8, 1, 0, true> : k_radial<T, 8, 0, 0, true>);
    else
      kern = mode == 1 ? (hb == 4 ? k_radial<T, 4, 0, 1, false> : k_radial<T, 8, 0, 1, false>)
                       : hb == 4 ? (act == 1 ? k_radial<T, 4, 1, 0, false> : k_radial<T, 4, 0, 0, false>)
                                 : (act == 1 ? k_radial<T, 8, 1, 0, false> : k_radial<T, 8, 0, 0, false>);
    HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    hipLaunchKernelGGL(kern, dim3(ncu), dim3(threads), lds, stream, ra);
  }
};

// One source of an element-dependent reduce, as the host containers give it (weights [nel][nout][nin][w_shape])
struct ReduceSrc {
  const std::vector<double> *W;
  double norm;
  int n_in, w_shape;
  const std::vector<int> *collect_ind, *w_l_tile, *out_fn;    // out_fn: output function per connection, or null (one function)
  int nfun, ninp;                                            // functions of the source tensor, its padded channel width
};

// Element-dependent reduce of up to 4 sources into `nout` channels of ONE output function (fused_cpu.h:1202-1273 of the
// reference): weights per collected function in MFMA fragment order, for k_reduce_fwd / k_reduce_bwd.
// fo >= 0 keeps the connections whose output function is fo.
template<class T> struct DevReduce {
  DevBuf WF[4], WB[4], Fn[4];
  ReduceDev<T> d{};
  int njobs = 0;
  void build(const std::vector<ReduceSrc> &src, int nel, int nout, int fo, int ostride, int ooff, const int *drow)
  {
    d.nsrc = (int) src.size();
    d.nrho = nout;
    d.nbr = (nout + 15) / 16;
    d.ksr = (nout + 3) / 4;
    d.ostride = ostride;
    d.ooff = ooff;
    if (nout > 32) throw Error("reduce widths above 32 are not supported by the GPU reduce kernels");
    for (int q = 0; q < 16; q++) d.drow[q] = drow[q];
    const int krp = d.ksr * 4;
    njobs = 0;
    for (int s = 0; s < d.nsrc; s++) {
      const ReduceSrc &w = src[s];
      std::vector<int> fn;
      for (size_t c = 0; c < w.collect_ind->size(); c++)
        if (fo < 0 || !w.out_fn || (*w.out_fn)[c] == fo) fn.push_back((*w.collect_ind)[c]);
      std::sort(fn.begin(), fn.end());
      fn.erase(std::unique(fn.begin(), fn.end()), fn.end());
      const int nc = (int) fn.size(), nin = w.n_in;
      std::vector<T> vF, vB;
      std::vector<double> M((size_t) nin * nout), Mt((size_t) nout * nin);
      for (int mu = 0; mu < nel; mu++)
        for (int u = 0; u < nc; u++) {
          std::fill(M.begin(), M.end(), 0.0);
          for (size_t c = 0; c < w.collect_ind->size(); c++) {
            if ((*w.collect_ind)[c] != fn[u]) continue;
            if (fo >= 0 && w.out_fn && (*w.out_fn)[c] != fo) continue;
            const int tile = (*w.w_l_tile)[c];
            for (int k = 0; k < nout; k++)
              for (int n = 0; n < nin; n++)
                M[(size_t) n * nout + k] += w.norm * (*w.W)[(((size_t) mu * nout + k) * nin + n) * w.w_shape + tile];
          }
          for (int k = 0; k < nout; k++)
            for (int n = 0; n < nin; n++) Mt[(size_t) k * nin + n] = M[(size_t) n * nout + k];
          pack_fragments<T>(M, nin, nout, w.ninp, d.nbr * 16, vF);      // X[atom][n] . M[n][k]
          pack_fragments<T>(Mt, nout, nin, krp, w.ninp, vB);             // g[atom][k] . Mt[k][n]
        }
      upload_vec(WF[s], vF);
      upload_vec(WB[s], vB);
      upload_vec(Fn[s], fn);
      d.WF[s] = WF[s].template as<T>();
      d.WB[s] = WB[s].template as<T>();
      d.fn[s] = Fn[s].template as<int>();
      d.ncol[s] = nc;
      d.nin[s] = w.ninp;
      d.stride[s] = w.nfun;
      njobs += nc;
    }
  }
};

// Device, stream, per-stage GPU timing and the MFMA accumulator-row probe of an engine.
// First base of an engine: from its construction until end_build() every DevBuf made on this thread (members of the
// engine and of the structures it holds) is listed in bufs_, and what they allocate in that time is model data.
struct BufRegistry {
  std::vector<DevBuf *> bufs_;
  BufRegistry() { building_registry() = &bufs_; }
  ~BufRegistry()
  {
    if (building_registry() == &bufs_) building_registry() = nullptr;    // a constructor that threw
  }
  void end_build()
  {
    if (building_registry() == &bufs_) building_registry() = nullptr;
  }
};

class EngineBase : public Engine, protected BufRegistry {
 public:
  // Frees every buffer that was allocated after the engine was built (per-atom and per-bond work buffers, the uploaded
  // structure); weights, tables and compiled kernels stay.  The engine then holds no structure: upload before the next
  // run.  The reference's engines: release_buffers() (kk/grace_1l_kk.h:72-113).
  void release_buffers() override
  {
    HIP_CHECK(hipSetDevice(device_));
    HIP_CHECK(hipStreamSynchronize(stream_));
    for (DevBuf *b : bufs_)
      if (!b->model_data) b->release();
    scal_.ensure(8 * sizeof(double));    // grown by a batch upload: an empty pass still clears and reads one record
    chunk_laid_out_ = 0;
    n_peak_ = 0;
    n_ = 0;
    n_nodes_ = 0;
    nb_ = 0;
    nstruct_ = 1;
    ran_ = ran_forces_ = ran_eatom_ = ran_uq_ = ran_vatom_ = false;
    upload_serial_++;
  }
  void synchronize() override { check(hipSetDevice(device_), "hipSetDevice"); check(hipStreamSynchronize(stream_), "hipStreamSynchronize"); }
  void set_chunksize(int atoms) override
  {
    if (!chunks_ && atoms > 0)
      throw InvalidArgument(who_ + ": this engine evaluates a structure in one pass; chunksize must be 0 (one pass) or -1 (auto), got " +
                            std::to_string(atoms));
    chunk_request_ = atoms;
  }
  int chunksize_used() const override { return chunk_used_; }
  void set_spline(int n) override
  {
    if (n < 0 || (n > 0 && n < 16) || n > (1 << 20)) throw InvalidArgument(who_ + ": spline must be 0 (the radial MLP itself) or 16 .. 1048576 intervals");
    apply_spline(n);
    spline_n_ = n;
  }
  int spline() const override { return spline_n_; }
  void set_ordered_sums(bool on) override
  {
    if (on && !ordered_ok_) throw InvalidArgument(who_ + ": this engine has no ordered (atomic-free) sums");
    ordered_ = on;
  }
  bool ordered_sums() const override { return ordered_; }
  void set_exchange(const ExchangeCallbacks &cb) override { exchange_ = cb; }
  int comm_layers() const override { return 0; }
  int comm_width(int) const override { return 0; }
  void comm_rows(int, int, int, const int *, int, double *, bool) override { throw Error(who_ + ": this model kind has no message rows to exchange"); }
  int64_t atoms_that_fit() override
  {
    HIP_CHECK(hipSetDevice(device_));
    if (chunks_ && chunk_request_ < 0) return INT64_MAX;    // the engine splits a pass that does not fit by itself
    if (n_peak_ <= 0 || chunk_used_ > 0) return layers() == 3 ? 16384 : layers() == 2 ? 131072 : 262144;
    double held = 0.0;
    for (const DevBuf *b : bufs_)
      if (!b->model_data) held += (double) b->bytes;
    size_t free_b = 0, total_b = 0;
    HIP_CHECK(hipMemGetInfo(&free_b, &total_b));
    double avail = (double) free_b;
    const long long cap = dev_bytes_limit().load();
    if (cap > 0) avail = std::min(avail, (double) (cap - dev_bytes_in_use().load()));
    // the buffers grew to the largest pass since they were last released: that pass fits, and sets the bytes per atom
    const double per_atom = std::max(held / n_peak_, 1.0);
    return std::max<int64_t>(n_peak_, (int64_t) (0.7 * (avail + held) / per_atom));
  }
  void set_profile(bool on) override { profile_ = on; }
  const std::vector<StageTime> &stage_times() override
  {
    synchronize();
    times_.clear();
    for (size_t q = 0; q < ev_used_; q++) {
      float ms = 0.f;
      check(hipEventElapsedTime(&ms, events_[q].first, events_[q].second), "hipEventElapsedTime");
      auto it = std::find_if(times_.begin(), times_.end(), [&](const StageTime &s) { return s.name == ev_names_[q]; });
      if (it == times_.end()) {
        times_.push_back({ev_names_[q], 0.0, 0});
        it = times_.end() - 1;
      }
      it->ms += ms;
      it->launches++;
      it->flops += ev_flops_[q];
    }
    return times_;
  }
  void debug_copy(int64_t bytes) override
  {
    check(hipSetDevice(device_), "hipSetDevice");
    const long long nd = std::max<int64_t>(bytes / 8, 1);
    DevBuf a, b;
    a.ensure(nd * 8);
    b.ensure(nd * 8);
    check(hipMemsetAsync(a.p, 0, nd * 8, stream_), "hipMemsetAsync");
    hipLaunchKernelGGL(k_copy_calibration, dim3(4096), dim3(256), 0, stream_, a.as<double>(), b.as<double>(), nd);
    check(hipGetLastError(), "copy kernel");
    check(hipStreamSynchronize(stream_), "hipStreamSynchronize");
  }
  // GB/s of the copy kernel (bytes read + bytes written) and of a read-only stream kernel over `bytes` bytes, best of 5
  void stream_rates(int64_t bytes, double *copy_gbs, double *read_gbs) override
  {
    check(hipSetDevice(device_), "hipSetDevice");
    const long long nd = std::max<int64_t>(bytes / 16, 1) * 2;
    DevBuf a, b, part;
    a.ensure(nd * 8);
    b.ensure(nd * 8);
    part.ensure(4096 * 8);
    check(hipMemsetAsync(a.p, 0, nd * 8, stream_), "hipMemsetAsync");
    check(hipMemsetAsync(part.p, 0, 4096 * 8, stream_), "hipMemsetAsync");
    hipEvent_t e0, e1;
    check(hipEventCreate(&e0), "hipEventCreate");
    check(hipEventCreate(&e1), "hipEventCreate");
    double best[2] = {1e30, 1e30};
    for (int rep = 0; rep < 6; rep++)
      for (int k = 0; k < 2; k++) {
        check(hipEventRecord(e0, stream_), "hipEventRecord");
        if (k == 0) hipLaunchKernelGGL(k_copy_calibration, dim3(4096), dim3(256), 0, stream_, a.as<double>(), b.as<double>(), nd);
        else hipLaunchKernelGGL(k_read_calibration, dim3(4096), dim3(256), 0, stream_, a.as<double>(), part.as<double>(), nd);
        check(hipEventRecord(e1, stream_), "hipEventRecord");
        check(hipEventSynchronize(e1), "hipEventSynchronize");
        float ms = 0.f;
        check(hipEventElapsedTime(&ms, e0, e1), "hipEventElapsedTime");
        if (rep > 0) best[k] = std::min(best[k], (double) ms);
      }
    (void) hipEventDestroy(e0);
    (void) hipEventDestroy(e1);
    if (copy_gbs) *copy_gbs = 2.0 * nd * 8 / (best[0] * 1e-3) * 1e-9;
    if (read_gbs) *read_gbs = 1.0 * nd * 8 / (best[1] * 1e-3) * 1e-9;
  }

  // copies a CSR structure to the device after the argument checks of the reference's CSR entry
  // (python/src/core.cpp:292-396); atoms are grouped into tiles of 16 of one element for the tile GEMMs
  void upload(const CsrInput &in) override
  {
    HIP_CHECK(hipSetDevice(device_));
    if (in.n < 0) throw InvalidArgument("negative atom count");
    const bool table = in.x && in.image && in.shifts;
    if ((in.rij != nullptr) == (in.x || in.image || in.shifts) || (!in.rij && !table))
      throw InvalidArgument("give rij or positions, image and shifts");
    const int n = in.n, nn = std::max(in.n, in.n_nodes);
    if (nn > n && (in.sid || !in.rij)) throw InvalidArgument("a list with ghost atoms holds one structure and gives its bond vectors");
    std::vector<int> mu(nn);
    for (int a = 0; a < nn; a++) {
      if (in.types[a] < 1 || in.types[a] > ntypes_) throw InvalidArgument("types must be 1 .. len(species)");
      mu[a] = type2mu_[in.types[a]];
      if (mu[a] < 0)
        throw Error(who_ + ": atom " + std::to_string(a) + " of unmapped type " + std::to_string(in.types[a]) + " in the atom list");
    }
    if (in.offset[0] != 0) throw InvalidArgument("offset[0] must be 0 and offset[-1] == len(j)");
    for (int a = 0; a < n; a++)
      if (in.offset[a + 1] < in.offset[a]) throw InvalidArgument("offset must be non-decreasing");
    const int64_t nb = in.offset[n];
    for (int64_t q = 0; q < nb; q++) {
      if (in.j[q] < 0 || in.j[q] >= nn) throw InvalidArgument("j must index atoms 0 .. len(types)-1");
      if (in.image && (in.image[q] < 0 || in.image[q] >= in.nimages)) throw InvalidArgument("image must index rows of shifts");
    }
    if (in.nstruct < 1) throw InvalidArgument("the number of structures must be positive");
    if (in.sid)
      for (int a = 0; a < n; a++)
        if (in.sid[a] < 0 || in.sid[a] >= in.nstruct) throw InvalidArgument("structure index of an atom out of range");
    if (in.sid)
      for (int a = 0; a < n; a++)
        for (int64_t q = in.offset[a]; q < in.offset[a + 1]; q++)
          if (in.sid[in.j[q]] != in.sid[a]) throw InvalidArgument("a bond joins atoms of two structures");
    HIP_CHECK(hipStreamSynchronize(stream_));
    n_ = n;
    n_nodes_ = nn;
    nb_ = nb;
    nstruct_ = in.sid ? in.nstruct : 1;
    have_sid_ = in.sid != nullptr;
    sid_sorted_ = !in.sid || std::is_sorted(in.sid, in.sid + n);
    scal_.ensure((size_t) 8 * nstruct_ * sizeof(double));
    have_rij_ = in.rij != nullptr;
    auto put = [&](DevBuf &b, const void *src, size_t bytes) {
      b.ensure(std::max<size_t>(bytes, 8));
      if (bytes) HIP_CHECK(hipMemcpyAsync(b.p, src, bytes, hipMemcpyHostToDevice, stream_));
    };
    put(mu_, mu.data(), sizeof(int) * nn);
    if (have_sid_) put(sid_, in.sid, sizeof(int) * n);
    mu_host_.assign(mu.begin(), mu.begin() + n);    // the central atoms: they make the element tiles
    chunk_laid_out_ = 0;
    const std::vector<int> tiles = element_tiles(mu_host_, nelem_, tile_el_);
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
    HIP_CHECK(hipStreamSynchronize(stream_));    // the host copies (mu, tiles) go out of scope
    ran_ = false;
    upload_serial_++;
  }
  void upload_device(const DeviceCsr &in) override
  {
    HIP_CHECK(hipSetDevice(device_));
    if (in.n < 0) throw InvalidArgument("negative atom count");
    const int n = in.n, nn = std::max(in.n, in.n_nodes);
    if (nn > n && (in.sid || !in.rij)) throw InvalidArgument("a list with ghost atoms holds one structure and gives its bond vectors");
    std::vector<int> mu(nn);
    for (int a = 0; a < nn; a++) {
      if (in.types[a] < 1 || in.types[a] > ntypes_) throw InvalidArgument("types must be 1 .. len(species)");
      mu[a] = type2mu_[in.types[a]];
      if (mu[a] < 0)
        throw Error(who_ + ": atom " + std::to_string(a) + " of unmapped type " + std::to_string(in.types[a]) + " in the atom list");
    }
    HIP_CHECK(hipStreamSynchronize(stream_));
    if (in.nstruct < 1) throw InvalidArgument("the number of structures must be positive");
    if (in.sid)
      for (int a = 0; a < n; a++)
        if (in.sid[a] < 0 || in.sid[a] >= in.nstruct) throw InvalidArgument("structure index of an atom out of range");
    n_ = n;
    n_nodes_ = nn;
    nb_ = in.nb;
    nstruct_ = in.sid ? in.nstruct : 1;
    have_sid_ = in.sid != nullptr;
    sid_sorted_ = !in.sid || std::is_sorted(in.sid, in.sid + n);
    have_rij_ = in.rij != nullptr;
    scal_.ensure((size_t) 8 * nstruct_ * sizeof(double));
    auto put = [&](DevBuf &b, const void *src, size_t bytes, hipMemcpyKind kind) {
      b.ensure(std::max<size_t>(bytes, 8));
      if (bytes) HIP_CHECK(hipMemcpyAsync(b.p, src, bytes, kind, stream_));
    };
    put(mu_, mu.data(), sizeof(int) * nn, hipMemcpyHostToDevice);
    mu_host_.assign(mu.begin(), mu.begin() + n);    // the central atoms: they make the element tiles
    chunk_laid_out_ = 0;
    const std::vector<int> tiles = element_tiles(mu_host_, nelem_, tile_el_);
    ntiles_ = (int) tiles.size() / 16;
    put(tiles_, tiles.data(), sizeof(int) * tiles.size(), hipMemcpyHostToDevice);
    put(offset_, in.offset, sizeof(int64_t) * (n + 1), hipMemcpyDeviceToDevice);
    put(j_, in.j, sizeof(int) * in.nb, hipMemcpyDeviceToDevice);
    if (have_sid_) put(sid_, in.sid, sizeof(int) * n, hipMemcpyHostToDevice);
    if (have_rij_) put(rij_, in.rij, sizeof(double) * 3 * in.nb, hipMemcpyDeviceToDevice);
    else {
      put(image_, in.image, sizeof(int) * in.nb, hipMemcpyDeviceToDevice);
      put(x_, in.x, sizeof(double) * 3 * n, hipMemcpyDeviceToDevice);
      put(shifts_, in.shifts, sizeof(double) * 3 * in.nimages, hipMemcpyHostToDevice);
    }
    HIP_CHECK(hipStreamSynchronize(stream_));
    ran_ = false;
    upload_serial_++;
  }
  void update_positions(const double *x) override
  {
    HIP_CHECK(hipSetDevice(device_));
    if (have_rij_) throw Error("update_positions: the uploaded list holds bond vectors, not positions");
    HIP_CHECK(hipStreamSynchronize(stream_));    // no pass of the stream still reads the staging memory or x_
    if (n_ > 0) {
      const size_t bytes = sizeof(double) * 3 * (size_t) n_;
      pin_in_.ensure(bytes);
      std::memcpy(pin_in_.p, x, bytes);
      HIP_CHECK(hipMemcpyAsync(x_.p, pin_in_.p, bytes, hipMemcpyHostToDevice, stream_));    // ordered before the pass on the same stream
    }
    ran_ = false;
  }
  double *bond_vectors_device() override
  {
    if (!have_rij_) throw Error("bond_vectors_device: the uploaded list holds positions, not bond vectors");
    HIP_CHECK(hipSetDevice(device_));
    HIP_CHECK(hipStreamSynchronize(stream_));
    ran_ = false;
    return rij_.as<double>();
  }
  uint64_t upload_serial() const override { return upload_serial_; }
  int device_index() const override { return device_; }
  void radial_noalloc(int, const double *, const int *, double *, double *) override
  {
    throw Error(who_ + ": the radial call without allocations is available for GRACE-1L engines");
  }
  // tiles of 16 atoms of one element (-1 padded), in atom order within an element, elements ascending;
  // el_off[e] .. el_off[e + 1]: the tiles of element e
  static std::vector<int> element_tiles(const std::vector<int> &mu, int nel, std::vector<int> &el_off)
  {
    // a counting pass per element (the elements are few): atoms per element, the tiles each element needs, then every atom
    // to the next free slot of its element, in atom order
    const int n = (int) mu.size();
    std::vector<int> count((size_t) nel, 0);
    for (int a = 0; a < n; a++) {
      if (mu[a] < 0 || mu[a] >= nel) throw Error("element of a central atom out of range");
      count[(size_t) mu[a]]++;
    }
    el_off.assign(nel + 1, 0);
    for (int e = 0; e < nel; e++) el_off[e + 1] = el_off[e] + (count[(size_t) e] + 15) / 16;
    std::vector<int> tiles((size_t) 16 * el_off[nel], -1), next((size_t) nel);
    for (int e = 0; e < nel; e++) next[(size_t) e] = 16 * el_off[e];
    for (int a = 0; a < n; a++) tiles[(size_t) next[(size_t) mu[a]]++] = a;
    return tiles;
  }
  void fetch(double *energy, double *forces, double *virial, double *eatom) override
  {
    if (have_sid_) throw Error("the uploaded list holds several structures: use fetch_batch()");
    fetch_batch(1, energy, forces, virial, eatom);
  }
  void fetch_batch(int nstruct, double *energy, double *forces, double *virial, double *eatom) override
  {
    HIP_CHECK(hipSetDevice(device_));
    if (!ran_) throw Error("fetch() before run()");
    if (nstruct != nstruct_) throw InvalidArgument("fetch_batch: the uploaded list holds " + std::to_string(nstruct_) + " structures");
    // everything the call returns goes to pinned memory as asynchronous copies behind the pass, with one wait:
    // [records 8 nstruct][forces 3 n_nodes][per-atom energies n]; the zero-bond flag of the pass is in pin_flag_ already
    const bool wf = forces && ran_forces_ && n_nodes_ > 0, we = eatom && ran_eatom_ && n_ > 0;
    const size_t nrec = (size_t) 8 * nstruct_, nf = wf ? (size_t) 3 * n_nodes_ : 0, ne = we ? (size_t) n_ : 0;
    pin_out_.ensure((nrec + nf + ne) * sizeof(double));
    double *rec = pin_out_.as<double>(), *pf = rec + nrec, *pe = pf + nf;
    HIP_CHECK(hipMemcpyAsync(rec, scal_.p, nrec * sizeof(double), hipMemcpyDeviceToHost, stream_));
    if (wf) HIP_CHECK(hipMemcpyAsync(pf, f_.p, nf * sizeof(double), hipMemcpyDeviceToHost, stream_));
    if (we) HIP_CHECK(hipMemcpyAsync(pe, eatom_.p, ne * sizeof(double), hipMemcpyDeviceToHost, stream_));
    HIP_CHECK(hipStreamSynchronize(stream_));
    check_zero_bond();
    for (int q = 0; q < nstruct_; q++) {
      if (energy) energy[q] = rec[8 * (size_t) q];
      if (virial && ran_forces_)
        for (int k = 0; k < 6; k++) virial[6 * (size_t) q + k] = rec[8 * (size_t) q + 1 + k];
    }
    if (wf) std::memcpy(forces, pf, nf * sizeof(double));
    if (we) std::memcpy(eatom, pe, ne * sizeof(double));
  }
  void fetch_batch_device(int nstruct, double *energy, double *forces, double *virial, double *eatom) override
  {
    HIP_CHECK(hipSetDevice(device_));
    if (!ran_) throw Error("fetch() before run()");
    if (nstruct != nstruct_) throw InvalidArgument("fetch_batch: the uploaded list holds " + std::to_string(nstruct_) + " structures");
    HIP_CHECK(hipStreamSynchronize(stream_));
    check_zero_bond();    // before anything is written to the caller's arrays
    hipLaunchKernelGGL(k_unpack_records, dim3((unsigned) ((nstruct_ + 255) / 256)), dim3(256), 0, stream_, scal_.as<double>(), nstruct_, energy,
                       ran_forces_ ? virial : nullptr);
    if (forces && ran_forces_ && n_ > 0) HIP_CHECK(hipMemcpyAsync(forces, f_.p, sizeof(double) * 3 * n_, hipMemcpyDeviceToDevice, stream_));
    if (eatom && ran_eatom_ && n_ > 0) HIP_CHECK(hipMemcpyAsync(eatom, eatom_.p, sizeof(double) * n_, hipMemcpyDeviceToDevice, stream_));
    HIP_CHECK(hipStreamSynchronize(stream_));
  }
  // two atoms at one position make a bond of length 0 (bonds.h:49-62 of the reference): reported by the pass in zero_
  void check_zero_bond()
  {
    if (n_ == 0) return;
    // the pass sent the flag to pinned memory right after its bond filter; every caller has waited for the stream
    const int *zb = pin_flag_.as<int>();
    if (!zb) return;
    if (zb[0] >= 0)
      throw Error("two atoms at the same position (a bond of length 0 between atoms " + std::to_string(zb[0]) + " and " + std::to_string(zb[1]) +
                  " of the neighbour list): not a physical structure");
  }
  void fetch_add_device(const int *atom, double *energy, double *forces, double *virial, double *eatom) override
  {
    HIP_CHECK(hipSetDevice(device_));
    if (!ran_) throw Error("fetch() before run()");
    if (have_sid_) throw Error("the uploaded list holds several structures: use fetch_batch()");
    HIP_CHECK(hipStreamSynchronize(stream_));
    check_zero_bond();    // before anything is added to the caller's arrays
    const bool wf = forces && ran_forces_, we = eatom && ran_eatom_;
    if (n_nodes_ > n_ && atom) throw Error("fetch_add_device: a list with ghost atoms keeps the caller's atom order");
    if (n_ > 0 && (wf || we))
      hipLaunchKernelGGL(k_add_results, dim3((unsigned) ((n_nodes_ + 255) / 256)), dim3(256), 0, stream_, atom, n_nodes_, n_, f_.as<double>(),
                         wf ? forces : nullptr, eatom_.as<double>(), we ? eatom : nullptr);
    double s[8];
    HIP_CHECK(hipMemcpyAsync(s, scal_.p, sizeof(s), hipMemcpyDeviceToHost, stream_));
    HIP_CHECK(hipStreamSynchronize(stream_));
    if (energy) *energy = s[0];
    if (virial && ran_forces_)
      for (int k = 0; k < 6; k++) virial[k] = s[1 + k];
  }
  void fetch_vatom(double *vatom, int ncomp, long long expect_rows = -1) override
  {
    HIP_CHECK(hipSetDevice(device_));
    if (ncomp != 6 && ncomp != 9) throw InvalidArgument("per-atom virials have 6 or 9 components");
    if (!ran_ || !ran_vatom_) throw Error("fetch_vatom() needs a run with the per-atom virial flag (and forces)");
    if (expect_rows >= 0 && expect_rows != n_nodes_)
      throw Error("fetch_vatom(): the engine holds " + std::to_string(n_nodes_) + " rows, the caller expects " + std::to_string(expect_rows));
    HIP_CHECK(hipStreamSynchronize(stream_));
    check_zero_bond();
    if (!vatom || n_nodes_ <= 0) return;
    std::vector<double> rows((size_t) 9 * n_nodes_);
    HIP_CHECK(hipMemcpy(rows.data(), vatom_.p, sizeof(double) * rows.size(), hipMemcpyDeviceToHost));
    for (size_t q = 0; q < (size_t) n_nodes_; q++)
      for (int k = 0; k < ncomp; k++) vatom[(size_t) ncomp * q + k] = rows[9 * q + k];
  }
  void add_vatom_device(const int *atom, double *vatom, int ncomp) override
  {
    if (ncomp != 6 && ncomp != 9) throw InvalidArgument("per-atom virials have 6 or 9 components");
    HIP_CHECK(hipSetDevice(device_));
    if (!ran_ || !ran_vatom_) throw Error("per-atom virials need a run with the per-atom virial flag (and forces)");
    if (n_nodes_ > n_ && atom) throw Error("add_vatom_device: a list with ghost atoms keeps the caller's atom order");
    HIP_CHECK(hipStreamSynchronize(stream_));
    check_zero_bond();
    const long long tot = (long long) ncomp * n_nodes_;
    if (tot > 0)
      hipLaunchKernelGGL(k_add_rows, dim3((unsigned) ((tot + 255) / 256)), dim3(256), 0, stream_, atom, n_nodes_, (const double *) vatom_.as<double>(), 9,
                         ncomp, vatom);
    HIP_CHECK(hipStreamSynchronize(stream_));
  }
  void fetch_uq(double *gamma, double *sigma, double *cluster) override
  {
    HIP_CHECK(hipSetDevice(device_));
    if (!ran_ || !ran_uq_) throw Error("fetch_uq() needs a run with the UQ flag");
    HIP_CHECK(hipStreamSynchronize(stream_));
    if (n_ == 0) return;
    // host or device destinations (the batch call on device arrays hands in device pointers)
    if (gamma) HIP_CHECK(hipMemcpy(gamma, uq_gamma_.p, sizeof(double) * n_, hipMemcpyDefault));
    if (sigma) HIP_CHECK(hipMemcpy(sigma, uq_sigma_.p, sizeof(double) * n_, hipMemcpyDefault));
    if (cluster) HIP_CHECK(hipMemcpy(cluster, uq_cluster_.p, sizeof(double) * n_, hipMemcpyDefault));
  }
  int64_t last_edge_count() override
  {
    synchronize();
    long long e = 0;
    if (n_ > 0) HIP_CHECK(hipMemcpy(&e, eoff_.as<long long>() + n_, sizeof(e), hipMemcpyDeviceToHost));
    return e;
  }
  double cutoff(int t1, int t2) const override
  {
    if (t1 < 1 || t1 > ntypes_ || t2 < 1 || t2 > ntypes_) return 0.0;
    const int a = type2mu_[t1], b = type2mu_[t2];
    return (a < 0 || b < 0) ? 0.0 : cut_host_[(size_t) a * nelem_ + b];
  }
  double max_cutoff() const override
  {
    double m = 0.0;
    for (int a = 1; a <= ntypes_; a++)
      for (int b = 1; b <= ntypes_; b++) m = std::max(m, cutoff(a, b));
    return m;
  }

 protected:
  // pair cutoffs [nel][nel] of the model
  void set_cutoffs(const std::vector<double> &cut)
  {
    cut_host_ = cut;
    upload_vec(cut_, cut);
  }
  // start of a pass: clears the outputs, filters the bonds of the uploaded list (r^2 < rc^2, bonds.h:120-162 of the
  // reference) into the compact edge arrays.  false: no atoms, nothing to do.
  bool begin_pass(const RunFlags &fl)
  {
    HIP_CHECK(hipSetDevice(device_));
    // argument checks first: a refused call leaves the state of the last good run (fetch() after it returns that run)
    if (fl.uq && !has_uq_head_) throw InvalidArgument(who_ + ": the model has no usable UQ head (" + uq_why_ + ")");
    ev_used_ = 0;
    const int n = n_;
    f_.ensure(std::max<size_t>((size_t) 3 * n_nodes_, 1) * sizeof(double));
    eatom_.ensure(std::max<size_t>(n, 1) * sizeof(double));
    HIP_CHECK(hipMemsetAsync(f_.p, 0, (size_t) 3 * n_nodes_ * sizeof(double), stream_));
    HIP_CHECK(hipMemsetAsync(scal_.p, 0, (size_t) 8 * nstruct_ * sizeof(double), stream_));
    ran_ = true;
    n_peak_ = std::max(n_peak_, n_);
    ran_forces_ = !fl.energy_only;
    ran_vatom_ = fl.vatom && !fl.energy_only;
    if (ran_vatom_) {
      vatom_.ensure(std::max<size_t>((size_t) 9 * n_nodes_, 1) * sizeof(double));
      HIP_CHECK(hipMemsetAsync(vatom_.p, 0, (size_t) 9 * n_nodes_ * sizeof(double), stream_));
    }
    ran_eatom_ = fl.eatom;
    ran_uq_ = false;    // set by the engine that evaluates a UQ head
    if (n == 0) return false;
    count_.ensure(sizeof(int) * n);
    eoff_.ensure(sizeof(long long) * (n + 1));
    HIP_CHECK(hipMemsetAsync(zero_.p, 0xFF, 2 * sizeof(int), stream_));    // (-1, -1): no bond of length zero seen
    BondSrc src{};
    src.mu = mu_.as<int>(); src.offset = offset_.as<long long>(); src.j = j_.as<int>();
    src.rij = have_rij_ ? rij_.as<double>() : nullptr;
    src.x = have_rij_ ? nullptr : x_.as<double>();
    src.image = have_rij_ ? nullptr : image_.as<int>();
    src.shifts = have_rij_ ? nullptr : shifts_.as<double>();
    src.cut = cut_.as<double>(); src.nel = nelem_;
    const size_t ecap = (size_t) std::max<int64_t>(nb_, 1);
    ei_.ensure(ecap * sizeof(int)); ej_.ensure(ecap * sizeof(int)); emu_.ensure(ecap * sizeof(int));
    rh_.ensure(ecap * 3 * sizeof(double)); r_.ensure(ecap * sizeof(double)); xr_.ensure(ecap * sizeof(double));
    rc_.ensure(ecap * sizeof(double));
    Edges ed{ei_.as<int>(), ej_.as<int>(), emu_.as<int>(), rh_.as<double>(), r_.as<double>(), xr_.as<double>(), rc_.as<double>()};
    const int wpb = 4;
    stage("edge_count", [&] { hipLaunchKernelGGL(k_edge_count, dim3((n + wpb - 1) / wpb), dim3(64 * wpb), 0, stream_, src, n, count_.as<int>(), zero_.as<int>()); });
    stage("edge_scan", [&] { hipLaunchKernelGGL(k_scan, dim3(1), dim3(1024), 0, stream_, count_.as<int>(), n, eoff_.as<long long>()); });
    stage("edge_fill", [&] { hipLaunchKernelGGL(k_edge_fill, dim3((n + wpb - 1) / wpb), dim3(64 * wpb), 0, stream_, src, n, eoff_.as<long long>(), ed); });
    pin_flag_.ensure(2 * sizeof(int));
    HIP_CHECK(hipMemcpyAsync(pin_flag_.p, zero_.p, 2 * sizeof(int), hipMemcpyDeviceToHost, stream_));    // read by check_zero_bond()
    return true;
  }
  EngineBase(int device, const char *who, int ntypes, const std::vector<int> &type2mu, int n_elements) :
      device_(device), who_(who), ntypes_(ntypes), type2mu_(type2mu), nelem_(n_elements)
  {
    check_type2mu(type2mu_, ntypes_, n_elements, who);
    check(hipSetDevice(device_), "hipSetDevice");
    hipDeviceProp_t prop;
    check(hipGetDeviceProperties(&prop, device_), "hipGetDeviceProperties");
    if (std::string(prop.gcnArchName).rfind("gfx950", 0) != 0 && std::string(prop.gcnArchName).rfind("gfx942", 0) != 0)
      throw Error(std::string(who) + ": this library is built for gfx950 (MI355X); device is " + prop.gcnArchName);
    ncu_ = prop.multiProcessorCount;
    arch_ = prop.gcnArchName;
    check(hipStreamCreate(&stream_), "hipStreamCreate");
    scal_.ensure(8 * sizeof(double));
    zero_.ensure(2 * sizeof(int));
  }
  ~EngineBase() override
  {
    (void) hipSetDevice(device_);
    for (auto &e : events_) { (void) hipEventDestroy(e.first); (void) hipEventDestroy(e.second); }
    if (stream_) (void) hipStreamDestroy(stream_);
  }
  static void check(hipError_t e, const char *what)
  {
    if (e != hipSuccess) throw Error(std::string("HIP error: ") + hipGetErrorString(e) + " in " + what);
  }
  void prof_begin(const char *name)
  {
    if (!profile_) return;
    if (ev_used_ == events_.size()) {
      hipEvent_t a, b;
      check(hipEventCreate(&a), "hipEventCreate");
      check(hipEventCreate(&b), "hipEventCreate");
      events_.push_back({a, b});
      ev_names_.push_back("");
      ev_flops_.push_back(0.0);
    }
    cur_flops_ = 0.0;
    ev_names_[ev_used_] = name;
    check(hipEventRecord(events_[ev_used_].first, stream_), "hipEventRecord");
  }
  void prof_end()
  {
    if (!profile_) return;
    check(hipEventRecord(events_[ev_used_].second, stream_), "hipEventRecord");
    ev_flops_[ev_used_] = cur_flops_;
    ev_used_++;
  }
  template<class F> void stage(const char *name, F &&f)
  {
    prof_begin(name);
    f();
    check(hipGetLastError(), name);
    prof_end();
  }
  // which accumulator row each (lane / 16, register) of a 16x16x4 MFMA holds; the column must be lane % 16
  template<class T> void probe_mfma()
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
    check(hipGetLastError(), "k_mfma_probe");
    check(hipStreamSynchronize(stream_), "hipStreamSynchronize");
    check(hipMemcpy(D.data(), dD.p, 256 * sizeof(T), hipMemcpyDeviceToHost), "hipMemcpy");
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
    int seen = 0;    // the 16 (group, register) pairs must cover the 16 rows
    for (int q = 0; q < 16; q++) seen |= 1 << drow_[q];
    if (seen != 0xFFFF) throw Error("MFMA 16x16x4 accumulator layout probe failed");
  }
  // A[atom][lm][n] = sum over the atom's edges of Y_lm Rz_l[n]: on the matrix cores where the register tiles fit
  template<class T> void launch_scatter(ScatterArgs<T> sa, int n, int lmax)
  {
    sa.natoms = n;
    for (int q = 0; q < 16; q++) sa.drow[q] = drow_[q];
    const int kb = sa.C / 16;
    const size_t lds = (size_t) 4 * 16 * sa.nlm * sizeof(T);
    const dim3 grid((n + 3) / 4), block(256);
#define GR_SCAT(NL_, KB_)                                                                       \
  do {                                                                                          \
    if (sa.tb.F) hipLaunchKernelGGL((k_scatter_a_tab<T, NL_, KB_>), grid, block, lds, stream_, sa); \
    else hipLaunchKernelGGL((k_scatter_a_mfma<T, NL_, KB_>), grid, block, lds, stream_, sa);    \
  } while (0)
    const int key = sa.nl * 10 + kb;    // register tiles of the kernel: nl * kb <= 10
    if (key == 11) GR_SCAT(1, 1); else if (key == 12) GR_SCAT(1, 2); else if (key == 14) GR_SCAT(1, 4);
    else if (key == 21) GR_SCAT(2, 1); else if (key == 22) GR_SCAT(2, 2); else if (key == 24) GR_SCAT(2, 4);
    else if (key == 31) GR_SCAT(3, 1); else if (key == 32) GR_SCAT(3, 2);
    else if (key == 41) GR_SCAT(4, 1); else if (key == 42) GR_SCAT(4, 2);
    else if (key == 51) GR_SCAT(5, 1); else if (key == 52) GR_SCAT(5, 2);
    else if (key == 61) GR_SCAT(6, 1); else if (key == 71) GR_SCAT(7, 1);
#undef GR_SCAT
    else {
      if (sa.tb.F) throw Error("A basis from radial tables: the channel widths of this model have no matrix-core kernel");
      const int sthreads = round_up(sa.nl * sa.C, 64);
      if (lmax <= 4) hipLaunchKernelGGL((k_scatter_a<T, 9>), dim3(n), dim3(sthreads), 0, stream_, sa);
      else hipLaunchKernelGGL((k_scatter_a<T, 13>), dim3(n), dim3(sthreads), 0, stream_, sa);
    }
  }
  // per-bond forces of a layer from the adjoint of its A basis (k_bond_bwd); ba.drow is filled here
  template<class T> void launch_bond_bwd(BondBwdArgs<T> ba, int n)
  {
    for (int q = 0; q < 16; q++) ba.drow[q] = drow_[q];
    const int kb = ba.C / 16;
    const size_t lds = ((size_t) ba.nlm * (ba.C + 2) + (size_t) 4 * 16 * ba.nlm * 3) * sizeof(T);
    if (kb != 1 && kb != 2 && kb != 4) throw Error("bond backward: channel width must be 16, 32 or 64");
#define GR_BB(KB, NL)                                                                                  \
  do {                                                                                                 \
    if (ba.tb.F) hipLaunchKernelGGL((k_bond_bwd<T, KB, NL, true>), dim3(n), dim3(256), lds, stream_, ba); \
    else hipLaunchKernelGGL((k_bond_bwd<T, KB, NL, false>), dim3(n), dim3(256), lds, stream_, ba);     \
  } while (0)
#define GR_BB_NL(NL) case NL: if (kb == 1) GR_BB(1, NL); else if (kb == 2) GR_BB(2, NL); else GR_BB(4, NL); break
    switch (ba.nl) {
      GR_BB_NL(1); GR_BB_NL(2); GR_BB_NL(3); GR_BB_NL(4); GR_BB_NL(5); GR_BB_NL(6); GR_BB_NL(7);
      default: throw Error("bond backward: lmax above " + std::to_string(kKernMaxL));
    }
#undef GR_BB_NL
#undef GR_BB
  }
  // out[tile atoms][job output] = GEMM jobs over X0 (kb0 16-channel blocks) and X1 (kb1), nb output blocks
  static constexpr size_t kGemmLdsBudget = 24 * 1024;    // measured on the benchmarks: 24 kB beats 16, 40 and 64 kB (blocks per CU)
  template<class T>
  void launch_gemm(DevJobs<T> &J, int kb0, int kb1, int nb, const T *X0, int nf0, const T *X1, int nf1, T *out, int nfo, int accumulate,
                   const int *tiles, int ntiles)
  {
    if (J.d.njobs == 0 || ntiles == 0) return;
    // multiply-adds of the launch: every segment is a [16 atoms x K] . [K x N] product per atom tile
    cur_flops_ += 2.0 * 16.0 * ntiles * (double) (nb * 16) * ((double) J.nseg[0] * kb0 * 16 + (double) J.nseg[1] * kb1 * 16);
    const int ksm = std::max(kb0, kb1) * 4;
    // weight tiles staged at a time: as many as fit kGemmLdsBudget, so that the wide tiles of 64-channel models (32 kB
    // in fp64) leave room for several blocks per CU
    const size_t tile_bytes = (size_t) nb * ksm * 64 * sizeof(T);
    const int mseg = std::max(1, std::min(kGemmMaxSeg, (int) (kGemmLdsBudget / tile_bytes)));
    const size_t lds = (size_t) mseg * tile_bytes;
    // single-segment jobs (one weight tile each: projections, reverse of the product reduces) walk several groups of
    // atom tiles per block when the grid is large: the staging of the tile is what they spend their time on
    const bool widest = kb0 == 4 && kb1 == 4 && nb == 4;
    const int tpw = widest ? 1 : 2;      // = gemm_tiles_per_wave<kb0, kb1, nb>()
    // waves of a block: a staged weight set is shared by 8 waves at fp64 and for the widest tiles, by 4 at fp32 with
    // narrower tiles (measured: 8 instead of 4 gives -1.3 % of a pass on the fp64 benchmarks, +1.8 % at fp32)
    const int nwave = widest || sizeof(T) == 8 ? 8 : 4;
    const int groups = (ntiles + nwave * tpw - 1) / (nwave * tpw);
    const int reps = J.d.max_seg == 1 ? std::max(1, std::min(8, (int) ((long long) J.d.njobs * groups / 8192))) : 1;
    const dim3 grid(J.d.njobs, (groups + reps - 1) / reps);
#define GR_GEMM(A_, B_, C_)                                                                                            \
  {                                                                                                                    \
    auto kern = k_gemm_jobs<T, A_, B_, C_, gemm_tiles_per_wave<A_, B_, C_>()>;                                         \
    if (lds > 48 * 1024)                                                                                               \
      HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds)); \
    hipLaunchKernelGGL(kern, grid, dim3(64 * nwave), lds, stream_, J.d, X0, nf0, X1, nf1, out, nfo, tiles, ntiles, accumulate, reps, mseg); \
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

  // ---- exchange with ghost atoms ------------------------------------------------------------------------------
  void exchange_forward(int layer)
  {
    if (!exchange_.forward || n_nodes_ == n_) return;
    HIP_CHECK(hipStreamSynchronize(stream_));
    exchange_.forward(exchange_.user, layer);
  }
  void exchange_reverse(int layer)
  {
    if (!exchange_.reverse || n_nodes_ == n_) return;
    HIP_CHECK(hipStreamSynchronize(stream_));
    exchange_.reverse(exchange_.user, layer);
  }
  // The four row movers on rows [atom][function][CP] of which the first nf functions and C channels travel
  // (nf C doubles per atom); stride: elements per atom.
  template<class T> void move_rows(int mode, T *rows, long long stride, int nf, int C, int CP, int n, const int *list, int first, double *buf, bool host)
  {
    HIP_CHECK(hipSetDevice(device_));
    if (n <= 0) return;
    if (!rows) throw Error(who_ + ": the message rows do not exist yet (the exchange runs inside a pass)");
    const bool by_list = mode == 0 || mode == 3;
    if (by_list && !list) throw InvalidArgument("the atom list of the exchange is missing");
    if (!buf) throw InvalidArgument("the buffer of the exchange is missing");
    const size_t count = (size_t) n * nf * C;
    const int *dl = list;
    double *db = buf;
    if (host) {
      comm_buf_.ensure(count * sizeof(double));
      db = comm_buf_.as<double>();
      if (by_list) {
        for (int k = 0; k < n; k++)
          if (list[k] < 0 || list[k] >= n_nodes_) throw InvalidArgument("the atom list of the exchange names an atom outside the owned and ghost atoms");
        comm_list_.ensure((size_t) n * sizeof(int));
        HIP_CHECK(hipMemcpyAsync(comm_list_.p, list, (size_t) n * sizeof(int), hipMemcpyHostToDevice, stream_));
        dl = comm_list_.as<int>();
      }
      if (mode == 1 || mode == 3) HIP_CHECK(hipMemcpyAsync(db, buf, count * sizeof(double), hipMemcpyHostToDevice, stream_));
    }
    if (!by_list && (first < 0 || first + n > n_nodes_)) throw InvalidArgument("the atom range of the exchange lies outside the owned and ghost atoms");
    const dim3 grid((unsigned) ((count + 255) / 256)), block(256);
    if (mode == 0 || mode == 2)
      hipLaunchKernelGGL(k_comm_pack<T>, grid, block, 0, stream_, (const T *) rows, stride, nf, C, CP, by_list ? dl : nullptr, first, n, db);
    else
      hipLaunchKernelGGL(k_comm_unpack<T>, grid, block, 0, stream_, rows, stride, nf, C, CP, by_list ? dl : nullptr, first, n, (const double *) db,
                         mode == 3 ? 1 : 0);
    HIP_CHECK(hipGetLastError());
    if (host && (mode == 0 || mode == 2)) HIP_CHECK(hipMemcpyAsync(buf, db, count * sizeof(double), hipMemcpyDeviceToHost, stream_));
    HIP_CHECK(hipStreamSynchronize(stream_));
  }

  // ---- chunks of atoms ---------------------------------------------------------------------------------------
  // Atoms per pass for a structure whose work buffers take `per_atom` bytes per atom of a chunk and `kept` bytes per atom
  // of the structure, after the reference's policy (libgrace/include/grace/kk/support.h:425-450): everything in one pass
  // while that fits 70 % of the memory this engine can have (the free device memory, or what the library's own cap
  // leaves, plus what its work buffers hold already), else the largest power of two >= 512 that fits.  Returns n for one pass.
  int plan_chunk(int n, double per_atom, double kept)
  {
    if (n <= 0 || chunk_request_ == 0) return n;
    if (chunk_request_ > 0) return std::min(n, chunk_request_);
    size_t free_b = 0, total_b = 0;
    HIP_CHECK(hipMemGetInfo(&free_b, &total_b));
    double avail = (double) free_b;
    const long long cap = dev_bytes_limit().load();
    if (cap > 0) avail = std::min(avail, (double) (cap - dev_bytes_in_use().load()));
    double held = 0.0;
    for (const DevBuf *b : bufs_)
      if (!b->model_data) held += (double) b->bytes;
    const double budget = 0.7 * (avail + held);
    if (per_atom * 1.125 * n + kept * n <= budget) return n;
    int c = std::min(n, kChunkFloor);
    while (2 * c < n && per_atom * 1.125 * 2.0 * c + kept * n <= budget) c *= 2;
    log_message(0, who_ + ": chunksize auto: " + std::to_string(c) + " atoms per pass for " + std::to_string(n) + " atoms (" +
                       std::to_string((long long) (per_atom * 1000 / 1048576)) + " MB of work buffers and " +
                       std::to_string((long long) (kept * 1000 / 1048576)) + " MB kept per 1000 atoms, " + std::to_string((long long) (avail / 1048576)) +
                       " MB of device memory available)");
    return c;
  }
  static constexpr int kChunkFloor = 512;    // smallest chunk of the automatic choice and of the retries after a failed allocation
  // Tiles of 16 atoms of one element for every chunk of `cs` atoms, with atom indices counted from the chunk's first atom:
  // chunk k owns tiles [chunk_tile_off_[k], chunk_tile_off_[k + 1]) of chunk_tiles_.
  void layout_chunks(int cs)
  {
    if (chunk_laid_out_ == cs) return;
    const int n = n_, nch = (n + cs - 1) / cs;
    std::vector<int> all, el;
    chunk_tile_off_.assign(1, 0);
    chunk_tile_el_.clear();
    for (int k = 0; k < nch; k++) {
      const int a0 = k * cs, a1 = std::min(n, a0 + cs);
      const std::vector<int> sub(mu_host_.begin() + a0, mu_host_.begin() + a1);
      const std::vector<int> t = element_tiles(sub, nelem_, el);
      all.insert(all.end(), t.begin(), t.end());
      chunk_tile_off_.push_back((int) all.size() / 16);
      chunk_tile_el_.push_back(el);    // tiles of element e within the chunk: [el[e], el[e + 1])
    }
    upload_vec(chunk_tiles_, all);
    chunk_laid_out_ = cs;
  }
  // first edge of every chunk (and the end of the last): eoff at the chunk boundaries, read back after the bond filter
  std::vector<long long> chunk_edge_bounds(int cs)
  {
    const int nch = (n_ + cs - 1) / cs;
    std::vector<long long> b((size_t) nch + 1);
    for (int k = 0; k <= nch; k++)
      HIP_CHECK(hipMemcpyAsync(&b[(size_t) k], eoff_.as<long long>() + std::min(n_, k * cs), sizeof(long long), hipMemcpyDeviceToHost, stream_));
    HIP_CHECK(hipStreamSynchronize(stream_));
    return b;
  }
  // a pointer moved back by `count` elements: kernels that index a chunk's buffer with structure-wide indices (edges)
  template<class U> static U *moved_back(U *p, long long count)
  {
    return reinterpret_cast<U *>(reinterpret_cast<intptr_t>(p) - (intptr_t) (count * (long long) sizeof(U)));
  }
  bool chunks_ = false;          // the engine can evaluate a structure in chunks of atoms
  int chunk_request_ = -1, chunk_used_ = 0, chunk_laid_out_ = 0;
  std::vector<int> mu_host_, chunk_tile_off_;
  std::vector<std::vector<int>> chunk_tile_el_;
  DevBuf chunk_tiles_;

  int device_, ncu_ = 256;
  std::string arch_, who_;
  int ntypes_;
  std::vector<int> type2mu_;
  int nelem_;
  std::vector<double> cut_host_;
  // uploaded structure
  int n_nodes_ = 0;           // central atoms and ghosts (= n_ without ghosts)
  uint64_t upload_serial_ = 0;
  PinnedBuf pin_in_, pin_out_;    // staging of the positions of a call and of what a call returns
  PinnedBuf pin_flag_;            // the zero-bond flag of the last pass (two ints)
  DevBuf vatom_;              // per-atom virials [n_nodes][9] (xx yy zz xy xz yz yx zx zy) of a pass with the vatom flag
  bool ran_vatom_ = false;
  double *vatom_ptr() { return ran_vatom_ ? vatom_.as<double>() : nullptr; }
  ExchangeCallbacks exchange_{};
  DevBuf comm_list_, comm_buf_;    // staging of the host forms of the row movers
  int n_ = 0, n_peak_ = 0;    // atoms of the uploaded structure; of the largest pass since the work buffers were released
  int64_t nb_ = 0;
  bool have_rij_ = false;
  DevBuf cut_, mu_, sid_, offset_, j_, rij_, x_, image_, shifts_, tiles_;
  int ntiles_ = 0, nstruct_ = 1;
  std::vector<int> tile_el_;    // [nel + 1] tile range of every element
  bool have_sid_ = false, sid_sorted_ = true;    // sid_sorted_: the atoms of every structure are one range of rows

  // ---- ordered sums (engines that set ordered_ok_): the reverse kernels store the force of every bond on its central atom
  // (fedge_[e][3]) and, per atom, the sums over its own bonds (fcen_[i][9]: force, then the six virial sums) instead of
  // adding with atomics; the forces on the neighbours are gathered through the bonds listed by neighbour atom (rebuilt every
  // pass: the bonds inside the cutoff change with the positions); energy and virial records are summed per structure in a
  // fixed order from the per-atom energies and fcen_
  bool ordered_ok_ = false, ordered_ = false;
  int spline_n_ = 0;
  // the engine's radial kernels take the setting (engines without radial tables say so and stay exact)
  virtual void apply_spline(int n)
  {
    if (n > 0) log_message(0, who_ + ": radial tables are not used by this engine; the radial MLPs are evaluated for every bond");
  }
  DevBuf fedge_, fcen_, tcount_, toff_, traw_, tsorted_;
  // before begin_pass(): what the mode cannot do
  void ordered_check(const RunFlags &fl) const
  {
    if (!ordered_) return;
    if (fl.vatom && !fl.energy_only) throw InvalidArgument(who_ + ": per-atom virials are not available with ordered sums");
    if (!sid_sorted_) throw InvalidArgument(who_ + ": ordered sums need the atoms of every structure in one range of rows");
    if (nb_ >= INT32_MAX) throw InvalidArgument(who_ + ": ordered sums number the bonds with 32 bits");
  }
  // after begin_pass() of a pass with forces: the per-bond and per-atom stores, and the bonds by neighbour atom, each row
  // in ascending order
  void ordered_begin()
  {
    const int n = n_, nn = n_nodes_;
    const size_t ne = (size_t) std::max<int64_t>(nb_, 1);
    fedge_.ensure(3 * ne * sizeof(double));
    fcen_.ensure((size_t) 9 * std::max(n, 1) * sizeof(double));
    tcount_.ensure((size_t) 2 * nn * sizeof(int));    // bonds per neighbour atom, then the fill cursors
    toff_.ensure(((size_t) nn + 1) * sizeof(long long));
    traw_.ensure(ne * sizeof(int));
    tsorted_.ensure(ne * sizeof(int));
    stage("ordered_list", [&] {
      HIP_CHECK(hipMemsetAsync(tcount_.p, 0, (size_t) 2 * nn * sizeof(int), stream_));
      const long long *n_edges = eoff_.as<long long>() + n;
      const dim3 egrid((unsigned) ((ne + 255) / 256)), agrid((unsigned) ((nn + 3) / 4));
      hipLaunchKernelGGL(k_tlist_count, egrid, dim3(256), 0, stream_, n_edges, ej_.as<int>(), tcount_.as<int>());
      hipLaunchKernelGGL(k_scan, dim3(1), dim3(1024), 0, stream_, tcount_.as<int>(), nn, toff_.as<long long>());
      hipLaunchKernelGGL(k_tlist_fill, egrid, dim3(256), 0, stream_, n_edges, ej_.as<int>(), toff_.as<long long>(), tcount_.as<int>() + nn,
                         traw_.as<int>());
      hipLaunchKernelGGL(k_tlist_sort, agrid, dim3(256), 0, stream_, nn, toff_.as<long long>(), traw_.as<int>(), tsorted_.as<int>());
    });
  }
  // end of the pass: forces of all rows (ghosts included) and the records of the structures
  void ordered_finish(const RunFlags &fl)
  {
    const int n = n_, nn = n_nodes_;
    stage("ordered_sums", [&] {
      if (!fl.energy_only)
        hipLaunchKernelGGL(k_ordered_forces, dim3((unsigned) ((nn + 3) / 4)), dim3(256), 0, stream_, nn, n, toff_.as<long long>(), tsorted_.as<int>(),
                           fedge_.as<double>(), fcen_.as<double>(), f_.as<double>());
      hipLaunchKernelGGL(k_ordered_records, dim3((unsigned) nstruct_), dim3(256), 0, stream_, n, sid_ptr(), eatom_.as<double>(), fcen_.as<double>(),
                         fl.energy_only ? 0 : 1, scal_.as<double>());
    });
  }
  const int *sid_ptr() const { return have_sid_ ? sid_.as<int>() : nullptr; }
  // edges of the pass and its outputs (scal: energy, virial[6])
  DevBuf count_, eoff_, zero_, ei_, ej_, emu_, rh_, r_, xr_, rc_, f_, eatom_, scal_;
  bool ran_ = false, ran_forces_ = false, ran_eatom_ = false, ran_uq_ = false;
  bool has_uq_head_ = false;      // set by an engine whose model carries a valid UQ head
  std::string uq_why_ = "this engine evaluates none";
  DevBuf uq_gamma_, uq_sigma_, uq_cluster_;
  hipStream_t stream_ = nullptr;
  bool profile_ = false;
  std::vector<std::pair<hipEvent_t, hipEvent_t>> events_;
  std::vector<std::string> ev_names_;
  std::vector<double> ev_flops_;
  double cur_flops_ = 0.0;
  size_t ev_used_ = 0;
  std::vector<StageTime> times_;
  // the reverse pair kernel on the matrix cores wherever it applies; GRACE_HIP_PAIR_MFMA=0: the vector kernels
  int pair_mfma_ = pair_mfma_switch();
  static int pair_mfma_switch()
  {
    const char *e = std::getenv("GRACE_HIP_PAIR_MFMA");
    return e && e[0] == '0' ? 0 : 1;
  }
  int pair_waves_ = pair_waves_switch();    // waves of a block of that kernel; 0: 8 in fp64, 4 in fp32 (pair_mfma_waves)
  static int pair_waves_switch()
  {
    const char *e = std::getenv("GRACE_HIP_PAIR_WAVES");
    const int w = e ? std::atoi(e) : 0;
    return w >= 1 && w <= 8 ? w : 0;
  }
  int drow_[16];
  int drow64_[16];    // fp32 engines: the accumulator rows of the fp64 MFMA (the fp64 radial MLP that fills the radial tables)
  // probes the MFMA accumulator layout of the engine's precision; an fp32 engine probes the fp64 one first and keeps it
  template<class T> void probe_mfma_both()
  {
    if constexpr (sizeof(T) == 4) {
      probe_mfma<double>();
      for (int q = 0; q < 16; q++) drow64_[q] = drow_[q];
    }
    probe_mfma<T>();
    if constexpr (sizeof(T) == 8)
      for (int q = 0; q < 16; q++) drow64_[q] = drow_[q];
  }
};

}    // namespace grhip
