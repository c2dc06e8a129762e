// HIP kernels of the GRACE-1L energy/forces/virial pass for gfx950 (wave64, MFMA).  Included by engine_1l.hip only.
//
// Stage map (reference stages in libgrace/src/fused_1l.cpp:260-372 and the staged pipeline of
// libgrace/include/grace/kk/grace_1l_kk.h:449-454):
//   k_edge_count / k_edge_fill   bond filter r^2 < rc^2, unit vectors, x = r / rc        (bonds.h:120-162)
//   k_radial                     Chebyshev x envelope basis + radial MLP value/tangent on MFMA, times z[mu_j]
//                                (radial_x.h:11-60; spline tables of the CPU path replaced by the exact MLP)
//   k_scatter_a                  A[lm][n] = sum_b Y_lm R_nl z                            (fused_cpu.h:947-982)
//   k_gemm_jobs                  FC forward / reverse as tile GEMMs on MFMA               (fused_cpu.h:349-364)
//   k_prod_fwd / k_prod_bwd      channel-wise CG products                                 (fused_cpu.h:409-475)
//   k_reduce_fwd / k_reduce_bwd  rho reduce with per-element weights                      (fused_cpu.h:637-649)
//   k_energy                     fp64 readout MLP and its reverse                         (fused_1l.cpp:378-427)
//   k_bond_bwd                   per-bond force, pair scatter, virial                     (fused_cpu.h:836-860,1027-1050)
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace grhip {

constexpr int kKernMaxL = 6;                                // largest lmax of the kernels
constexpr int kMaxNlm = (kKernMaxL + 1) * (kKernMaxL + 1);
constexpr int kMaxPlm = (kKernMaxL + 1) * (kKernMaxL + 2) / 2;
constexpr int kBondChunk = 32;                          // bonds staged per pass of the per-atom kernels
constexpr int kMaxRadBasis = 16;
constexpr int kRadialPrefetch = 16;                     // weight fragments the radial kernel reads ahead: padding of the layer-2 weights                        // radial basis functions (padded to a multiple of 4)

// spherical-harmonics recursion coefficients (fused_cpu.h:686-704), by index l (l + 1) / 2 + m
struct ShCoef {
  double a[kMaxPlm], b[kMaxPlm], c[kKernMaxL + 1], d[kKernMaxL + 1];
  int lmax;
};

// Real spherical harmonics Y[lm] (stride ys) of the unit vector (rx, ry, rz) and, with GRAD, the gradient
// G[lm][3] of their polynomial extension.  Same recursion as fused_cpu.h:712-798, one bond per thread, fp64.
// LMAX: compile-time bound of co.lmax (the register arrays of the recursion are sized by it).
// With e1, e2 and D2 given, the gradient is stored as its two components along e1 and e2 instead: G[lm] = grad . e1,
// D2[lm] = grad . e2.
template<bool GRAD, class TY, int LMAX = kKernMaxL>
__device__ inline void sh_eval(const ShCoef &co, double rx, double ry, double rz, TY *Y, TY *G, const double *e1 = nullptr,
                               const double *e2 = nullptr, TY *D2 = nullptr)
{
  auto put = [&](int lm, double gx, double gy, double gz) {
    if (e1) {
      G[lm] = (TY) (gx * e1[0] + gy * e1[1] + gz * e1[2]);
      D2[lm] = (TY) (gx * e2[0] + gy * e2[1] + gz * e2[2]);
    } else {
      G[3 * lm] = (TY) gx; G[3 * lm + 1] = (TY) gy; G[3 * lm + 2] = (TY) gz;
    }
  };
  double plm[(LMAX + 1) * (LMAX + 2) / 2], dplm[(LMAX + 1) * (LMAX + 2) / 2];
  const int lmax = co.lmax < LMAX ? co.lmax : LMAX;
  plm[0] = 1.0;
  dplm[0] = 0.0;
  if (LMAX > 0 && lmax > 0) {
    const double s3 = 1.7320508075688772, s15 = -1.224744871391589;
    plm[LMAX > 0 ? 1 : 0] = s3 * rz; dplm[LMAX > 0 ? 1 : 0] = s3;
    plm[LMAX > 0 ? 2 : 0] = s15;     dplm[LMAX > 0 ? 2 : 0] = 0.0;
#pragma unroll
    for (int l = 2; l <= LMAX; l++) {
      if (l <= lmax) {
#pragma unroll
        for (int mm = 0; mm < l - 1; mm++) {
          const int id = l * (l + 1) / 2 + mm, i1 = (l - 1) * l / 2 + mm, i2 = (l - 2) * (l - 1) / 2 + mm;
          const double ca = co.a[id], cb = co.b[id];
          plm[id] = ca * (rz * plm[i1] + cb * plm[i2]);
          if (GRAD) dplm[id] = ca * (plm[i1] + rz * dplm[i1] + cb * dplm[i2]);
        }
        const int prev = (l - 1) * l / 2 + l - 1, i0 = l * (l + 1) / 2 + l - 1, i1 = l * (l + 1) / 2 + l;
        const double sd = co.d[l], sc = co.c[l];
        plm[i0] = sd * plm[prev] * rz;
        plm[i1] = sc * plm[prev];
        if (GRAD) {
          dplm[i0] = sd * (dplm[prev] * rz + plm[prev]);
          dplm[i1] = sc * dplm[prev];
        }
      }
    }
  }
  const double sq2 = 1.4142135623730951;
#pragma unroll
  for (int l = 0; l <= LMAX; l++) {
    if (l <= lmax) {
      const int c = l * (l + 1), p0 = l * (l + 1) / 2;
      Y[c] = (TY) plm[p0];
      if (GRAD) put(c, 0.0, 0.0, dplm[p0]);
      double pr = rx, pi = ry, prx = 1.0, pry = 0.0, pix = 0.0, piy = 1.0;
#pragma unroll
      for (int mm = 1; mm <= l; mm++) {
        const double sg = (mm % 2 == 0) ? sq2 : -sq2;
        const double pv = plm[p0 + mm];
        Y[c + mm] = (TY) (sg * pr * pv);
        Y[c - mm] = (TY) (sg * pi * pv);
        if (GRAD) {
          const double dpv = dplm[p0 + mm];
          put(c + mm, sg * prx * pv, sg * pry * pv, sg * pr * dpv);
          put(c - mm, sg * pix * pv, sg * piy * pv, sg * pi * dpv);
          const double nrx = prx * rx + pr - pix * ry, nry = pry * rx - piy * ry - pi;
          const double nix = prx * ry + pix * rx + pi, niy = pry * ry + pr + piy * rx;
          prx = nrx; pry = nry; pix = nix; piy = niy;
        }
        const double nr = pr * rx - pi * ry, ni = pr * ry + pi * rx;
        pr = nr; pi = ni;
      }
    }
  }
}

// Message rows to and from an exchange buffer (the pack / unpack kernels of the reference's GPU engines,
// libgrace/include/grace/kk/grace_2l_kk.h:141-157): rows[atom][function][CP], of which nf functions x C channels travel
// as doubles; the atoms are list[0 .. n) or first .. first + n.  add: the buffer is added to the rows (reverse exchange).
template<class T>
__global__ void k_comm_pack(const T *rows, long long stride, int nf, int C, int CP, const int *list, int first, int n, double *buf)
{
  const long long e = blockIdx.x * (long long) blockDim.x + threadIdx.x;
  if (e >= (long long) n * nf * C) return;
  const int c = (int) (e % C), fn = (int) ((e / C) % nf), k = (int) (e / ((long long) C * nf));
  const int atom = list ? list[k] : first + k;
  buf[e] = (double) rows[atom * stride + (long long) fn * CP + c];
}
template<class T>
__global__ void k_comm_unpack(T *rows, long long stride, int nf, int C, int CP, const int *list, int first, int n, const double *buf, int add)
{
  const long long e = blockIdx.x * (long long) blockDim.x + threadIdx.x;
  if (e >= (long long) n * nf * C) return;
  const int c = (int) (e % C), fn = (int) ((e / C) % nf), k = (int) (e / ((long long) C * nf));
  const int atom = list ? list[k] : first + k;
  T *dst = rows + atom * stride + (long long) fn * CP + c;
  // several entries of a send list may name one atom (an atom with several images): atomic add
  if (add) atomicAdd(dst, (T) buf[e]);
  else *dst = (T) buf[e];
}

// plain copy of n doubles: the calibration kernel for the HBM counters (FETCH_SIZE / WRITE_SIZE per byte moved)
static __global__ void k_copy_calibration(const double *src, double *dst, long long n)
{
  for (long long i = blockIdx.x * (long long) blockDim.x + threadIdx.x; i < n; i += (long long) gridDim.x * blockDim.x) dst[i] = src[i];
}

// read-only stream over n doubles (16 bytes per lane and step, one partial sum written per block): what a kernel that
// only reads can draw from HBM, next to the copy kernel's rate for one that reads and writes as much
static __global__ void k_read_calibration(const double *src, double *partial, long long n)
{
  const double2 *s2 = reinterpret_cast<const double2 *>(src);
  double acc = 0.0;
  for (long long i = blockIdx.x * (long long) blockDim.x + threadIdx.x; i < n / 2; i += (long long) gridDim.x * blockDim.x) {
    const double2 v = s2[i];
    acc += v.x + v.y;
  }
  for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
  if ((threadIdx.x & 63) == 0) atomicAdd(&partial[blockIdx.x], acc);
}

// ---------------------------------------------------------------------------------------------------------------
// bond filter
// ---------------------------------------------------------------------------------------------------------------
struct BondSrc {
  const int *mu;              // [n] model element of each atom
  const long long *offset;    // [n + 1]
  const int *j;               // [nb]
  const double *rij;          // [nb][3] or null
  const double *x;            // [n][3]      (with rij null)
  const int *image;           // [nb]
  const double *shifts;       // [nimg][3]
  const double *cut;          // [nel][nel] pair cutoffs
  int nel;
};

__device__ inline void bond_vec(const BondSrc &s, int i, long long q, double &dx, double &dy, double &dz)
{
  if (s.rij) {
    dx = s.rij[3 * q]; dy = s.rij[3 * q + 1]; dz = s.rij[3 * q + 2];
  } else {    // x_j - x_i + shift, in this order (system.h:36-42)
    const int jj = s.j[q];
    const double *xi = s.x + 3 * (long long) i, *xj = s.x + 3 * (long long) jj, *sh = s.shifts + 3 * (long long) s.image[q];
    dx = xj[0] - xi[0] + sh[0];
    dy = xj[1] - xi[1] + sh[1];
    dz = xj[2] - xi[2] + sh[2];
  }
}

// one wave per atom: number of bonds with r^2 < rc^2; a bond of length 0 is recorded in zero_bond (i, j) and skipped
static __global__ void k_edge_count(BondSrc s, int n, int *count, int *zero_bond)
{
  const int lane = threadIdx.x & 63;
  const int i = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (i >= n) return;
  const int mi = s.mu[i];
  int c = 0;
  for (long long q = s.offset[i] + lane; q < s.offset[i + 1]; q += 64) {
    double dx, dy, dz;
    bond_vec(s, i, q, dx, dy, dz);
    const double rsq = dx * dx + dy * dy + dz * dz;
    const int jj = s.j[q];
    const double rc = s.cut[mi * s.nel + s.mu[jj]];
    if (!(rsq < rc * rc)) continue;
    if (rsq == 0.0) {
      if (atomicCAS(zero_bond, -1, i) == -1) zero_bond[1] = jj;
      continue;
    }
    c++;
  }
  for (int o = 32; o > 0; o >>= 1) c += __shfl_down(c, o, 64);
  if (lane == 0) count[i] = c;
}

// exclusive scan of count[n] into eoff[n + 1] (single block; n up to a few million is a few passes of 1024)
static __global__ void k_scan(const int *count, int n, long long *eoff)
{
  __shared__ long long part[1024];
  __shared__ long long carry;
  if (threadIdx.x == 0) carry = 0;
  __syncthreads();
  for (int base = 0; base < n; base += 1024) {
    const int i = base + threadIdx.x;
    long long v = i < n ? count[i] : 0;
    part[threadIdx.x] = v;
    __syncthreads();
    for (int o = 1; o < 1024; o <<= 1) {
      long long t = threadIdx.x >= o ? part[threadIdx.x - o] : 0;
      __syncthreads();
      part[threadIdx.x] += t;
      __syncthreads();
    }
    if (i < n) eoff[i] = carry + part[threadIdx.x] - v;
    __syncthreads();
    if (threadIdx.x == 1023) carry += part[1023];
    __syncthreads();
  }
  if (threadIdx.x == 0) eoff[n] = carry;
}

// (energy, virial[6], unused) records of the structures -> energy [nstruct], virial [nstruct][6] (null: skipped)
static __global__ void k_unpack_records(const double *rec, int nstruct, double *energy, double *virial)
{
  const int s = blockIdx.x * blockDim.x + threadIdx.x;
  if (s >= nstruct) return;
  if (energy) energy[s] = rec[8 * (long long) s];
  if (virial)
    for (int k = 0; k < 6; k++) virial[6 * (long long) s + k] = rec[8 * (long long) s + 1 + k];
}

// f[atom[q]] += fe[q], eatom[atom[q]] += ee[q] for the n rows of the engine (null pointers are skipped)
// adds the pass's forces (rows 0 .. nf) and atom energies (rows 0 .. ne) to the caller's arrays; atom: caller's index of row q,
// null when the rows are in the caller's order
static __global__ void k_add_results(const int *atom, int nf, int ne, const double *fe, double *f, const double *ee, double *eatom)
{
  const int q = blockIdx.x * blockDim.x + threadIdx.x;
  if (q >= nf && q >= ne) return;
  const long long i = atom ? atom[q] : q;
  if (f && q < nf) {
    f[3 * i] += fe[3 * (long long) q];
    f[3 * i + 1] += fe[3 * (long long) q + 1];
    f[3 * i + 2] += fe[3 * (long long) q + 2];
  }
  if (eatom && q < ne) eatom[i] += ee[q];
}

// dst[atom[q]][k] += src[q][k], k < ncomp, for rows of sstride values in src and ncomp values in dst (atom null: row q)
static __global__ void k_add_rows(const int *atom, int n, const double *src, int sstride, int ncomp, double *dst)
{
  const long long t = blockIdx.x * (long long) blockDim.x + threadIdx.x;
  if (t >= (long long) ncomp * n) return;
  const long long q = t / ncomp;
  const int k = (int) (t % ncomp);
  dst[ncomp * (atom ? (long long) atom[q] : q) + k] += src[sstride * q + k];
}

struct Edges {
  int *ei, *ej, *emu;         // central atom, neighbour, neighbour element
  double *rh;                 // [E][3] unit vectors
  double *r, *x, *rc;         // length, r / rc, rc
};

// one wave per atom: in-cutoff bonds in list order -> compact edge arrays at eoff[i]
static __global__ void k_edge_fill(BondSrc s, int n, const long long *eoff, Edges e)
{
  const int lane = threadIdx.x & 63;
  const int i = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (i >= n) return;
  const int mi = s.mu[i];
  long long w = eoff[i];
  const long long q0 = s.offset[i], q1 = s.offset[i + 1];
  for (long long base = q0; base < q1; base += 64) {
    const long long q = base + lane;
    bool keep = false;
    double dx = 0, dy = 0, dz = 0, rsq = 0, rc = 0;
    int jj = 0;
    if (q < q1) {
      bond_vec(s, i, q, dx, dy, dz);
      rsq = dx * dx + dy * dy + dz * dz;
      jj = s.j[q];
      rc = s.cut[mi * s.nel + s.mu[jj]];
      keep = (rsq < rc * rc) && rsq != 0.0;
    }
    const unsigned long long m = __ballot(keep);
    if (keep) {
      const long long p = w + __popcll(m & ((1ull << lane) - 1ull));
      const double r = sqrt(rsq), ir = 1.0 / r;
      e.ei[p] = i;
      e.ej[p] = jj;
      e.emu[p] = s.mu[jj];
      e.rh[3 * p] = dx * ir; e.rh[3 * p + 1] = dy * ir; e.rh[3 * p + 2] = dz * ir;
      e.r[p] = r;
      e.rc[p] = rc;
      e.x[p] = r / rc;
    }
    w += __popcll(m);
  }
}

// ---------------------------------------------------------------------------------------------------------------
// radial MLP on the matrix cores
// ---------------------------------------------------------------------------------------------------------------
template<class T> struct Mfma;
template<> struct Mfma<double> {
  typedef double v4 __attribute__((ext_vector_type(4)));
  __device__ static inline v4 mma(double a, double b, v4 c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
};
template<> struct Mfma<float> {
  typedef float v4 __attribute__((ext_vector_type(4)));
  __device__ static inline v4 mma(float a, float b, v4 c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
};

// D = A B for one wave with A[i][k], B[k][j] held as (i or j = lane % 16, k = lane / 16): every lane writes its four
// accumulator values; the host derives which (row, column) each (lane, register) holds
template<class T> __global__ void k_mfma_probe(const T *A, const T *B, T *D)
{
  const int lane = threadIdx.x;
  typename Mfma<T>::v4 acc = {0, 0, 0, 0};
  acc = Mfma<T>::mma(A[(lane & 15) * 4 + (lane >> 4)], B[(lane >> 4) * 16 + (lane & 15)], acc);
  for (int v = 0; v < 4; v++) D[lane * 4 + v] = acc[v];
}

template<class T> struct RadialArgs {
  const long long *n_edges;   // device scalar: edges of this pass are [e_begin, e_begin + count)
  long long e_begin, e_count; // e_count < 0: take *n_edges - e_begin
  const double *x;            // [E] r / rc
  const int *emu;             // [E] neighbour element
  const T *w0, *w1, *w2;      // fragment-ordered weights (norms folded in)
  const T *z;                 // [nel][C]
  T *Rz, *dRz;                // [E][noutp]  columns l * C + n
  int nrb, p, ks0;            // basis functions, envelope order, k-steps of layer 0
  int nob, noutp;             // 16-column blocks and padded width of the output
  int C, nel, act;            // radial channels, elements, activation (0 SiLU, 1 tanh)
  int w2_in_lds;
  int drow[16];               // accumulator row of (lane / 16, register)
  // species form (MODE 1 of k_radial): the basis is the bare T_k(2x - 1); layer 0 adds bias_i[element of the central
  // atom] + bias_j[element of the neighbour], layer 1 adds bias1, and the envelope multiplies the output
  const int *emi;             // [E] element of the central atom
  const T *bias_i, *bias_j;   // [nel][HB * 16]
  const T *bias1;             // [HB * 16]
};

// reciprocal: hardware estimate + Newton steps (2 in fp64: full precision; 1 in fp32)
__device__ inline double fast_rcp(double x)
{
  double r = __builtin_amdgcn_rcp(x);
  r = fma(fma(-x, r, 1.0), r, r);
  r = fma(fma(-x, r, 1.0), r, r);
  return r;
}
__device__ inline float fast_rcp(float x)
{
  float r = __builtin_amdgcn_rcpf(x);
  return fmaf(fmaf(-x, r, 1.0f), r, r);
}

template<class T, int ACT> __device__ inline void act_pair(T &s, T &ds)
{
  if (ACT == 1) {
    const T t = tanh(s);
    ds = ds * ((T) 1 - t * t);
    s = t;
  } else {
    const T sg = fast_rcp((T) 1 + exp(-s));
    ds = sg * ((T) 1 + s * ((T) 1 - sg)) * ds;
    s = s * sg;
  }
}

// x^n for a non-negative integer n by squaring
__device__ inline double ipow(double x, int n)
{
  double r = 1.0, b = x;
  while (n > 0) {
    if (n & 1) r *= b;
    b *= b;
    n >>= 1;
  }
  return r;
}

// One wave = 16 edges.  Layers 0 and 1 run as D[feature][edge] = W^T H with the weights as the A operand, so the
// accumulator registers of one layer are exactly the B operand of the next (no data movement between layers: the
// k index of a step is the accumulator row held by that lane, and the weight fragments are stored in that order).
// Layer 2 swaps the operands, D[edge][column], so that 16 lanes write 16 consecutive columns of one edge row.
// Every k-step feeds all row blocks of the value and the tangent stream (2 HB independent accumulator chains).
// ACT: 0 SiLU, 1 tanh (compile-time: the fp64 tanh is large, and both activations inlined 32 times overflow the
// instruction cache).
// Radial functions from tables, as the reference's engines evaluate them (spline_eval, libgrace/include/grace/fused_cpu.h:
// 1052-1074; tables of Grace1LFused::build_splines, libgrace/src/fused_1l.cpp:102-129): N intervals over x = r / rc in
// [0, 1], per interval the cubic through the values and derivatives of the radial MLP at its two ends,
//   R(t) = f0 + t (d0 + t (c2 + t c3)),  c2 = -3 f0 - 2 d0 + 3 f1 - d1,  c3 = 2 f0 + d0 - 2 f1 + d1,  d = f' / N,
//   dR/dx = N (d0 + t (2 c2 + 3 c3 t)),  k = min(int(x N), N - 1),  t = x N - k.
// COEF false (fp64): F, D are [N + 1][noutp] value and d/dx at the knots (what k_radial returns for x = k / N and unit
// species weights) and the cubic's coefficients are formed per use, so the table is half the size of stored coefficients
// and stays in the L2.  COEF true (fp32): F is [N][4][noutp] coefficients formed in fp64 by k_spline_coef (c2 and c3 are
// differences of nearly equal values: formed in fp32 they would cost four digits of dR/dx), D unused.
// One block = noutp threads rounded up to a wave, a thread per column, blocks stride over the edges; rows as k_radial.
// Species form (GRACE-3L: the MLP takes the embeddings of both atoms of the bond; per-pair tables of the reference,
// libgrace/src/fused_3l.cpp:487-520): emi set: one table per ordered pair of species, table number sp[emi[e]] nsp +
// sp[emu[e]] (sp: element -> species of the engine), the tables one after the other in F and D.
template<class T, bool COEF>
__global__ void k_radial_spline(const long long *__restrict__ n_edges, long long e_begin, long long e_count, const double *__restrict__ x,
                                const int *__restrict__ emu, const T *__restrict__ F, const T *__restrict__ D, int N, const T *__restrict__ z, int C,
                                int noutp, T *__restrict__ Rz, T *__restrict__ dRz, const int *__restrict__ emi = nullptr,
                                const int *__restrict__ sp = nullptr, int nsp = 1)
{
  const long long cnt = e_count >= 0 ? e_count : *n_edges - e_begin;
  const int col = threadIdx.x;
  if (col >= noutp) return;
  const int n = col % C;
  const T h = (T) (1.0 / N);
  constexpr int U = 4;    // edges of one step: their table reads are in flight together
  for (long long el0 = (long long) blockIdx.x * U; el0 < cnt; el0 += (long long) gridDim.x * U) {
    T c0[U], c1[U], c2[U], c3[U], t[U], zc[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      const long long e = e_begin + (el0 + u < cnt ? el0 + u : cnt - 1);
      const double sx = x[e] * N;
      int k = (int) sx;
      k = k > N - 1 ? N - 1 : (k < 0 ? 0 : k);
      t[u] = (T) (sx - k);
      zc[u] = z[emu[e] * C + n];
      const long long pair = emi ? (long long) sp[emi[e]] * nsp + sp[emu[e]] : 0;
      if (COEF) {
        const T *c = F + (pair * N + k) * 4 * noutp + col;
        c0[u] = c[0]; c1[u] = c[noutp]; c2[u] = c[2 * noutp]; c3[u] = c[3 * noutp];
      } else {
        const T *f = F + (pair * (N + 1) + k) * noutp + col, *d = D + (pair * (N + 1) + k) * noutp + col;
        c0[u] = f[0]; c1[u] = d[0]; c2[u] = f[noutp]; c3[u] = d[noutp];    // f0, f0', f1, f1'
      }
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      if (el0 + u >= cnt) break;
      const long long e = e_begin + el0 + u;
      T a0 = c0[u], a1 = c1[u], a2 = c2[u], a3 = c3[u];
      if (!COEF) {
        const T f1 = a2, d1 = a3 * h;
        a1 *= h;
        a2 = (T) -3 * a0 - (T) 2 * a1 + (T) 3 * f1 - d1;
        a3 = (T) 2 * a0 + a1 - (T) 2 * f1 + d1;
      }
      const T tt = t[u];
      __builtin_nontemporal_store((a0 + tt * (a1 + tt * (a2 + tt * a3))) * zc[u], &Rz[e * noutp + col]);
      __builtin_nontemporal_store((a1 + tt * ((T) 2 * a2 + tt * (T) 3 * a3)) * (T) N * zc[u], &dRz[e * noutp + col]);
    }
  }
}
// coefficients [N][4][noutp] of the cubics in fp32 from the knot values and derivatives in fp64
static __global__ void k_spline_coef(const double *__restrict__ F, const double *__restrict__ D, int N, int noutp, float *__restrict__ coef)
{
  const long long q = blockIdx.x * (long long) blockDim.x + threadIdx.x;
  if (q >= (long long) N * noutp) return;
  const long long k = q / noutp;
  const int col = (int) (q % noutp);
  const double f0 = F[k * noutp + col], f1 = F[(k + 1) * noutp + col], d0 = D[k * noutp + col] / N, d1 = D[(k + 1) * noutp + col] / N;
  float *c = coef + k * 4 * noutp + col;
  c[0] = (float) f0;
  c[noutp] = (float) d0;
  c[2 * noutp] = (float) (-3.0 * f0 - 2.0 * d0 + 3.0 * f1 - d1);
  c[3 * noutp] = (float) (2.0 * f0 + d0 - 2.0 * f1 + d1);
}

// Threads of a block: hidden width 64 with every weight in LDS runs three waves per SIMD (168 registers; two waves at 180
// were 2 % slower in fp64, 6 % in fp32), the other forms would spill at that size; width 128 runs one wave per SIMD.
constexpr int radial_threads(int hb, int mode, bool w2l) { return hb <= 4 ? (w2l && mode == 0 ? 768 : 512) : 256; }

template<class T, int HB, int ACT, int MODE, bool W2L> __global__ __launch_bounds__((radial_threads(HB, MODE, W2L))) void k_radial(RadialArgs<T> a)
{
  typedef typename Mfma<T>::v4 v4;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  T *w0s = reinterpret_cast<T *>(smem_raw);
  T *w1s = w0s + HB * a.ks0 * 64;
  T *w2s = w1s + HB * HB * 4 * 64;
  {
    const int n0 = HB * a.ks0 * 64, n1 = HB * HB * 4 * 64, n2 = W2L ? (a.nob * HB * 4 + kRadialPrefetch) * 64 : 0;
    for (int q = threadIdx.x; q < n0; q += blockDim.x) w0s[q] = a.w0[q];
    for (int q = threadIdx.x; q < n1; q += blockDim.x) w1s[q] = a.w1[q];
    for (int q = threadIdx.x; q < n2; q += blockDim.x) w2s[q] = a.w2[q];
  }
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const int c = lane & 15, g = lane >> 4;
  const long long cnt = a.e_count >= 0 ? a.e_count : *a.n_edges - a.e_begin;
  const long long ntiles = (cnt + 15) / 16;
  const int p = a.p;
  const double cf0 = 0.5 * (p + 1) * (p + 2), cf1 = (double) p * (p + 2), cf2 = 0.5 * p * (p + 1), cfd = 0.5 * p * (p + 1) * (p + 2);
  // The memory counter of a wave retires loads and stores in order: a load issued behind a store waits for that store
  // to complete.  The per-edge inputs of the NEXT tile (x of this lane's column, element and x of this lane's four
  // output rows) are therefore requested before the first store of the current tile.
  const int KZ = a.C >> 4;                        // distinct columns n = (16 cb + c) mod C of a lane: c + 16 k, k < KZ <= 4
  const long long tstep = (long long) gridDim.x * nw;
  long long tile = (long long) blockIdx.x * nw + wave;
  double x_n = 0.5, xv_n[4] = {0.5, 0.5, 0.5, 0.5};
  int emu_n[4] = {0, 0, 0, 0};
  auto fetch_edge_inputs = [&](long long tl) {
    const long long el = tl * 16 + c;
    x_n = (tl < ntiles && el < cnt) ? a.x[a.e_begin + el] : 0.5;
#pragma unroll
    for (int v = 0; v < 4; v++) {
      const long long er = tl * 16 + a.drow[g * 4 + v];
      const bool ok = tl < ntiles && er < cnt;
      emu_n[v] = ok ? a.emu[a.e_begin + er] : 0;
      if (MODE == 1) xv_n[v] = ok ? a.x[a.e_begin + er] : 0.5;
    }
  };
  fetch_edge_inputs(tile);
  for (; tile < ntiles; tile += tstep) {
    const long long eloc = tile * 16 + c;
    const long long e = a.e_begin + eloc;
    const double x = x_n;
    double xv[4];
#pragma unroll
    for (int v = 0; v < 4; v++) xv[v] = xv_n[v];
    // basis g_k = T_k(2x - 1) fcut_p(x), k = 1..nrb, and d/dx (radial_x.h:11-26); this lane supplies k = 4 s + g
    T h0[kMaxRadBasis / 4], dh0[kMaxRadBasis / 4];
    {
      const double xpm = ipow(x, p - 1), xp = xpm * x, xp1 = xp * x, xp2 = xp1 * x;
      const double fc = 1.0 - cf0 * xp + cf1 * xp1 - cf2 * xp2;
      const double dfc = cfd * (-xpm + 2.0 * xp - xp1);
      const double t = 2.0 * x - 1.0;
      double Tp = 1.0, Tc = t, dTp = 0.0, dTc = 2.0;
#pragma unroll
      for (int s = 0; s < kMaxRadBasis / 4; s++) { h0[s] = (T) 0; dh0[s] = (T) 0; }
      for (int k = 0; k < a.nrb; k++) {
        const double gk = MODE == 1 ? Tc : Tc * fc, dgk = MODE == 1 ? dTc : dTc * fc + Tc * dfc;
        if ((k & 3) == g) {
#pragma unroll
          for (int s = 0; s < kMaxRadBasis / 4; s++)
            if (s == (k >> 2)) { h0[s] = (T) gk; dh0[s] = (T) dgk; }
        }
        const double Tn = 2.0 * t * Tc - Tp, dTn = 2.0 * (2.0 * Tc + t * dTc) - dTp;
        Tp = Tc; dTp = dTc; Tc = Tn; dTc = dTn;
      }
    }
    // ---- layer 0
    v4 h1[HB], dh1[HB];
#pragma unroll
    for (int rb = 0; rb < HB; rb++) { h1[rb] = v4{0, 0, 0, 0}; dh1[rb] = v4{0, 0, 0, 0}; }
#pragma unroll
    for (int s = 0; s < kMaxRadBasis / 4; s++)
      if (s < a.ks0) {
#pragma unroll
        for (int rb = 0; rb < HB; rb++) {
          const T w = w0s[(rb * a.ks0 + s) * 64 + lane];
          h1[rb] = Mfma<T>::mma(w, h0[s], h1[rb]);
          dh1[rb] = Mfma<T>::mma(w, dh0[s], dh1[rb]);
        }
      }
    if (MODE == 1) {
      const long long ee = eloc < cnt ? e : a.e_begin;
      const T *bi = a.bias_i + (long long) a.emi[ee] * (HB * 16), *bj = a.bias_j + (long long) a.emu[ee] * (HB * 16);
#pragma unroll
      for (int rb = 0; rb < HB; rb++)
#pragma unroll
        for (int v = 0; v < 4; v++) h1[rb][v] += bi[rb * 16 + a.drow[g * 4 + v]] + bj[rb * 16 + a.drow[g * 4 + v]];
    }
#pragma unroll
    for (int rb = 0; rb < HB; rb++)
#pragma unroll
      for (int v = 0; v < 4; v++) {
        T s_ = h1[rb][v], d_ = dh1[rb][v];
        act_pair<T, ACT>(s_, d_);
        h1[rb][v] = s_; dh1[rb][v] = d_;
      }
    // ---- layer 1
    // An fp64 MFMA holds its wave for the 64 cycles it runs, and nothing else of the wave issues meanwhile: what hides
    // the latency of a weight fragment is to request it a few steps (2 MFMAs each) before its use.  The scheduling
    // barriers keep the compiler from moving the request back next to the use.
    v4 h2[HB], dh2[HB];
#pragma unroll
    for (int rb = 0; rb < HB; rb++) { h2[rb] = v4{0, 0, 0, 0}; dh2[rb] = v4{0, 0, 0, 0}; }
    {
      constexpr int NS = HB * 4 * HB;
      // step q = (kb, s, rb): fragment ((rb HB + kb) 4 + s) of w1
      auto frag = [&](int q) { return w1s[(((q % HB) * HB + q / (4 * HB)) * 4 + (q / HB) % 4) * 64 + lane]; };
      T wa_ = frag(0), wb_ = frag(1);
#pragma unroll
      for (int q = 0; q < NS; q++) {
        const int kb = q / (4 * HB), s_ = (q / HB) % 4, rb = q % HB;
        const T w = wa_;
        wa_ = wb_;
        if (q + 2 < NS) wb_ = frag(q + 2);
        __builtin_amdgcn_sched_barrier(0);
        h2[rb] = Mfma<T>::mma(w, h1[kb][s_], h2[rb]);
        dh2[rb] = Mfma<T>::mma(w, dh1[kb][s_], dh2[rb]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if (MODE == 1) {
#pragma unroll
      for (int rb = 0; rb < HB; rb++)
#pragma unroll
        for (int v = 0; v < 4; v++) h2[rb][v] += a.bias1[rb * 16 + a.drow[g * 4 + v]];
    }
#pragma unroll
    for (int rb = 0; rb < HB; rb++)
#pragma unroll
      for (int v = 0; v < 4; v++) {
        T s_ = h2[rb][v], d_ = dh2[rb][v];
        act_pair<T, ACT>(s_, d_);
        h2[rb][v] = s_; dh2[rb][v] = d_;
      }
    // ---- layer 2 (linear), operands swapped: rows = edges, columns = outputs; one block of 16 columns at a time (a
    // single dependent accumulator chain keeps the matrix pipe full, and one block's weights are all that is in flight)
    // The z values of a column block are requested one block ahead and the inputs of the next tile before the first
    // store of this one: no load is issued behind a store whose completion it would then wait for.
    // rows of the tile as 32-bit offsets from its first row (the tile is wave-uniform), -1: no such edge
    T *const Rt = a.Rz + (a.e_begin + tile * 16) * a.noutp, *const dRt = a.dRz + (a.e_begin + tile * 16) * a.noutp;
    int zrow[4], row_v[4];
    T env_v[4], denv_v[4], zc[4];
#pragma unroll
    for (int v = 0; v < 4; v++) {
      const int rl = a.drow[g * 4 + v];
      row_v[v] = tile * 16 + rl < cnt ? rl * a.noutp : -1;
      zrow[v] = emu_n[v] * a.C + c;
      zc[v] = a.z[zrow[v]];
      if (MODE == 1) {
        const double xpm = ipow(xv[v], p - 1), xp = xpm * xv[v], xp1 = xp * xv[v], xp2 = xp1 * xv[v];
        env_v[v] = (T) (1.0 - cf0 * xp + cf1 * xp1 - cf2 * xp2);
        denv_v[v] = (T) (cfd * (-xpm + 2.0 * xp - xp1));
      }
    }
    fetch_edge_inputs(tile + tstep);
    // weight fragments of layer 2 run PF steps ahead of their use, across the column blocks (the fragments of
    // consecutive steps are consecutive in memory): LDS when they fit, else global memory, hence the depth
    constexpr int PF = W2L ? 2 : 16, NQ = HB * 4;
    static_assert(PF <= kRadialPrefetch, "padding of the layer-2 weights");
    // two separate pointers: one pointer that may be either would make every read a flat load, which waits for the
    // stores of the block before it
    const T *wl = (W2L ? (const T *) w2s : a.w2) + lane;
    T wq[PF];
#pragma unroll
    for (int i = 0; i < PF; i++) wq[i] = wl[i * 64];
    for (int cb = 0; cb < a.nob; cb++) {
      T zn[4];
      const int kn = ((cb + 1) & (KZ - 1)) * 16;       // column n = c + 16 k of z in the next block
#pragma unroll
      for (int v = 0; v < 4; v++) zn[v] = a.z[zrow[v] + kn];
      v4 acc = {0, 0, 0, 0}, dacc = {0, 0, 0, 0};
      const T *wc = wl + (long long) cb * NQ * 64;
#pragma unroll
      for (int q = 0; q < NQ; q++) {
        const T w_ = wq[q % PF];
        wq[q % PF] = wc[(q + PF) * 64];               // beyond the last block: the zero padding of the weights
        __builtin_amdgcn_sched_barrier(0);
        acc = Mfma<T>::mma(h2[q / 4][q % 4], w_, acc);
        dacc = Mfma<T>::mma(dh2[q / 4][q % 4], w_, dacc);
        __builtin_amdgcn_sched_barrier(0);
      }
      const int col = cb * 16 + c;
#pragma unroll
      for (int v = 0; v < 4; v++) {
        if (row_v[v] >= 0) {
          // streaming stores: the rows are read by other kernels after the whole array has been written
          if (MODE == 1) {
            __builtin_nontemporal_store((T) (acc[v] * env_v[v] * zc[v]), &Rt[row_v[v] + col]);
            __builtin_nontemporal_store((T) ((dacc[v] * env_v[v] + acc[v] * denv_v[v]) * zc[v]), &dRt[row_v[v] + col]);
          } else {
            __builtin_nontemporal_store((T) (acc[v] * zc[v]), &Rt[row_v[v] + col]);
            __builtin_nontemporal_store((T) (dacc[v] * zc[v]), &dRt[row_v[v] + col]);
          }
        }
        zc[v] = zn[v];
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// A basis
// ---------------------------------------------------------------------------------------------------------------
// The radial tables for kernels that evaluate them themselves instead of reading rows another kernel wrote (the bond
// loops of the reference's fused GPU engines read their table in the same place, libgrace/include/grace/kk/
// grace_1l_fused_kk_impl.h:405-440; CPU: spline_eval, libgrace/include/grace/fused_cpu.h:1052-1074).  F == nullptr: no
// tables, the kernel reads rows.  Layouts and formulas are those of k_radial_spline.
template<class T> struct RadialTable {
  const T *F, *D;     // fp64: value and d/dx at the knots, [N + 1][noutp] each; fp32: F = coefficients [N][4][noutp], D unused
  int N;              // intervals over x = r / rc in [0, 1]
  const double *x;    // [E] r / rc
  const int *emu;     // [E] neighbour element
  const T *z;         // [nel][C] species weights (all ones where the rows carry none)
};
// interval and offset of x in a table of N intervals
__device__ inline int table_interval(double x, int N, double &t)
{
  const double sx = x * N;
  int k = (int) sx;
  k = k > N - 1 ? N - 1 : (k < 0 ? 0 : k);
  t = sx - k;
  return k;
}
// the four table entries of column col in interval k (requested here, used by table_value)
template<class T> __device__ inline void table_request(const RadialTable<T> &tb, int k, int col, int noutp, T (&raw)[4])
{
  if constexpr (sizeof(T) == 4) {
    const T *c = tb.F + (long long) k * 4 * noutp + col;
    raw[0] = c[0]; raw[1] = c[noutp]; raw[2] = c[2 * noutp]; raw[3] = c[3 * noutp];
  } else {
    const T *f = tb.F + (long long) k * noutp + col, *d = tb.D + (long long) k * noutp + col;
    raw[0] = f[0]; raw[1] = d[0]; raw[2] = f[noutp]; raw[3] = d[noutp];    // f0, f0', f1, f1'
  }
}
// R(t) and, with DERIV, dR/dx of the cubic of the interval
template<class T, bool DERIV> __device__ inline void table_value(const T (&raw)[4], T t, T h, T fN, T &R, T &dR)
{
  T a0 = raw[0], a1 = raw[1], a2 = raw[2], a3 = raw[3];
  if constexpr (sizeof(T) == 8) {
    const T f1 = a2, d1 = a3 * h;
    a1 *= h;
    a2 = (T) -3 * a0 - (T) 2 * a1 + (T) 3 * f1 - d1;
    a3 = (T) 2 * a0 + a1 - (T) 2 * f1 + d1;
  }
  R = a0 + t * (a1 + t * (a2 + t * a3));
  if (DERIV) dR = (a1 + t * ((T) 2 * a2 + t * (T) 3 * a3)) * fN;
}

template<class T> struct ScatterArgs {
  const long long *eoff;      // [n + 1]
  const double *rh;           // [E][3]
  const T *Rz;                // [E][noutp]
  RadialTable<T> tb;          // tb.F set: the radial functions come from the tables, Rz is not read
  T *A;                       // [chunk atoms][nlm][C]
  int a0, natoms;             // first atom of the chunk, atoms in it
  int C, nl, nlm, noutp;
  int drow[16];               // accumulator row of (lane / 16, register)
  ShCoef sh;
};

// One block per atom, thread = (l, n).  The harmonics of up to kScatterBonds bonds are computed by all threads into LDS,
// then the radial rows stream through registers in groups of kScatterGroup bonds, the loads of the next group in flight
// while the current one is accumulated.
constexpr int kScatterBonds = 64, kScatterGroup = 16;

template<class T, int MAXM> __device__ inline void scatter_group(const T *Ysh, int b0, int nb, int lm0, int nm, const T *r, T *acc)
{
#pragma unroll
  for (int u = 0; u < kScatterGroup; u++)
    if (b0 + u < nb) {
      // no branch per m (the lanes of a wave hold two values of l): entries beyond 2l+1 read a valid address and add 0
      const T *y = Ysh + (b0 + u) * kMaxNlm + lm0;
      T yv[MAXM];
#pragma unroll
      for (int m = 0; m < MAXM; m++) yv[m] = y[m < nm ? m : 0];
#pragma unroll
      for (int m = 0; m < MAXM; m++) acc[m] += (m < nm ? yv[m] : (T) 0) * r[u];
    }
}

template<class T, int MAXM> __global__ void k_scatter_a(ScatterArgs<T> a)
{
  __shared__ T Ysh[kScatterBonds * kMaxNlm];
  const int t = threadIdx.x;
  const int i = a.a0 + blockIdx.x;
  const long long e0 = a.eoff[i], e1 = a.eoff[i + 1];
  const int ncol = a.nl * a.C;
  const int l = t < ncol ? t / a.C : 0, n = t % a.C;
  const int nm = 2 * l + 1, lm0 = l * l;
  T acc[MAXM];
#pragma unroll
  for (int m = 0; m < MAXM; m++) acc[m] = (T) 0;
  for (long long base = e0; base < e1; base += kScatterBonds) {
    const int nb = (int) (e1 - base < kScatterBonds ? e1 - base : kScatterBonds);
    const T *rp = a.Rz + base * a.noutp + (t < ncol ? t : 0);
    T r0[kScatterGroup], r1[kScatterGroup];
#pragma unroll
    for (int u = 0; u < kScatterGroup; u++) r0[u] = rp[(long long) (u < nb ? u : 0) * a.noutp];
    __syncthreads();
    for (int b = t; b < nb; b += blockDim.x) {
      const double *u = a.rh + 3 * (base + b);
      sh_eval<false, T>(a.sh, u[0], u[1], u[2], Ysh + b * kMaxNlm, nullptr);
    }
    __syncthreads();
    for (int b0 = 0; b0 < nb; b0 += 2 * kScatterGroup) {
      const int b1 = b0 + kScatterGroup, b2 = b1 + kScatterGroup;
#pragma unroll
      for (int u = 0; u < kScatterGroup; u++) r1[u] = rp[(long long) (b1 + u < nb ? b1 + u : 0) * a.noutp];
      scatter_group<T, MAXM>(Ysh, b0, nb, lm0, nm, r0, acc);
#pragma unroll
      for (int u = 0; u < kScatterGroup; u++) r0[u] = rp[(long long) (b2 + u < nb ? b2 + u : 0) * a.noutp];
      scatter_group<T, MAXM>(Ysh, b1, nb, lm0, nm, r1, acc);
    }
  }
  if (t < ncol) {
    T *Ai = a.A + (long long) blockIdx.x * a.nlm * a.C;
#pragma unroll
    for (int m = 0; m < MAXM; m++)
      if (m < nm) Ai[(lm0 + m) * a.C + n] = acc[m];
  }
}

// A[lm][n] = sum_b Y_lm(b) Rz[b][l][n] on the matrix cores.  One wave per atom (4 atoms per block); per tile of 16
// bonds and per l:  D_l[m][n] += Y_l^T[m][b] . Rz_l[b][n]  with K = bonds (4 per MFMA step), rows m padded to 16.
// The B operand (Rz) comes straight from memory, 16 lanes reading 128 consecutive bytes of one bond row; the B operands
// of a tile are requested before the harmonics of the tile are evaluated, and each half of the next tile as soon as the
// MFMAs have consumed that half of the current one.  The A operand (Y) comes from the wave's LDS tile.  The
// accumulators of the wave are the atom's A.
// The grid walks the atoms from the LAST to the first: the radial kernel, which runs right before, writes the edge rows
// in ascending order, so the rows it wrote last are the ones still held by the memory-side cache.
// NL = lmax + 1, KB = channels / 16.   dynamic LDS: 4 * 16 * nlm values.
template<class T, int NL, int KB> __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void k_scatter_a_mfma(ScatterArgs<T> a)
{
  typedef typename Mfma<T>::v4 v4;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 15, g = lane >> 4;
  T *Yw = reinterpret_cast<T *>(smem_raw) + wave * 16 * a.nlm;     // [16 bonds][nlm]
  const int ia = a.natoms - 1 - (blockIdx.x * 4 + wave);
  if (ia < 0) return;
  const int i = a.a0 + ia;
  const long long w0 = a.eoff[i], w1 = a.eoff[i + 1];
  const int C = a.C;
  v4 acc[NL][KB];
#pragma unroll
  for (int l = 0; l < NL; l++)
#pragma unroll
    for (int cb = 0; cb < KB; cb++) acc[l][cb] = v4{0, 0, 0, 0};
  T breg[4][NL][KB];
  auto request = [&](long long eb, int h) {
    const int nb = (int) (w1 - eb < 16 ? w1 - eb : 16);
#pragma unroll
    for (int s = 2 * h; s < 2 * h + 2; s++) {
      if (4 * s >= nb) continue;                      // a step with no bond: neither loaded nor multiplied
      const int b = 4 * s + g;                        // k index of this lane in step s = bond of the tile
      const T *row = a.Rz + (eb + (b < nb ? b : 0)) * a.noutp + c;      // rows beyond the range: any valid row (Y = 0 there)
#pragma unroll
      for (int l = 0; l < NL; l++)
#pragma unroll
        for (int cb = 0; cb < KB; cb++) breg[s][l][cb] = row[l * C + cb * 16];
    }
  };
  if (w0 < w1) { request(w0, 0); request(w0, 1); }
  for (long long eb = w0; eb < w1; eb += 16) {
    const int nb = (int) (w1 - eb < 16 ? w1 - eb : 16);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    if (lane < 16) {
      if (lane < nb) {
        const double *u = a.rh + 3 * (eb + lane);
        sh_eval<false, T, NL - 1>(a.sh, u[0], u[1], u[2], Yw + lane * a.nlm, nullptr);
      } else {
        for (int q = 0; q < a.nlm; q++) Yw[lane * a.nlm + q] = (T) 0;
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const bool more = eb + 16 < w1;
#pragma unroll
    for (int h = 0; h < 2; h++) {
#pragma unroll
      for (int s = 2 * h; s < 2 * h + 2; s++) {
        if (4 * s >= nb) continue;
        const T *yb = Yw + (4 * s + g) * a.nlm;
#pragma unroll
        for (int l = 0; l < NL; l++) {
          const T y = c < 2 * l + 1 ? yb[l * l + c] : (T) 0;       // A operand: row m = c
#pragma unroll
          for (int cb = 0; cb < KB; cb++) acc[l][cb] = Mfma<T>::mma(y, breg[s][l][cb], acc[l][cb]);
        }
      }
      if (more) request(eb + 16, h);
    }
  }
  T *Ai = a.A + (long long) ia * a.nlm * C;
#pragma unroll
  for (int l = 0; l < NL; l++) {
#pragma unroll
      for (int v = 0; v < 4; v++) {
        const int m = a.drow[4 * g + v];
        if (m < 2 * l + 1) {
#pragma unroll
          for (int cb = 0; cb < KB; cb++) Ai[(l * l + m) * C + cb * 16 + c] = acc[l][cb][v];
        }
      }
  }
}

// k_scatter_a_mfma with the B operand formed from the radial tables: lane (g, c) supplies, in step s, the columns
// l C + cb 16 + c of bond 4 s + g, i.e. per (l, cb) four table entries of the bond's interval (16 lanes read 128
// consecutive bytes of a table row; the 2.6 MB table of a 32-channel lmax-4 model stays in the L2), the cubic in t, times
// the species weight.  The entries of step s + 1 are requested when those of step s have been turned into operands, and
// arrive while the matrix instructions of step s run; x and the element of the lane's four bonds of the NEXT tile are
// requested a tile ahead.  No radial row is read: the rows need not exist.
template<class T, int NL, int KB> __global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void k_scatter_a_tab(ScatterArgs<T> a)
{
  typedef typename Mfma<T>::v4 v4;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 15, g = lane >> 4;
  T *Yw = reinterpret_cast<T *>(smem_raw) + wave * 16 * a.nlm;     // [16 bonds][nlm]
  const int ia = a.natoms - 1 - (blockIdx.x * 4 + wave);
  if (ia < 0) return;
  const int i = a.a0 + ia;
  const long long w0 = a.eoff[i], w1 = a.eoff[i + 1];
  const int C = a.C;
  const RadialTable<T> tb = a.tb;
  const T h = (T) (1.0 / tb.N), fN = (T) tb.N;
  v4 acc[NL][KB];
#pragma unroll
  for (int l = 0; l < NL; l++)
#pragma unroll
    for (int cb = 0; cb < KB; cb++) acc[l][cb] = v4{0, 0, 0, 0};
  double xs[4], xn[4] = {0, 0, 0, 0};
  int ms[4], mn[4] = {0, 0, 0, 0};
  auto geometry = [&](long long eb, double (&x)[4], int (&m)[4]) {
    const int nb = (int) (w1 - eb < 16 ? w1 - eb : 16);
#pragma unroll
    for (int s = 0; s < 4; s++) {
      const int b = 4 * s + g;
      const long long e = eb + (b < nb ? b : 0);
      x[s] = tb.x[e];
      m[s] = tb.emu[e];
    }
  };
  // one (step, 16-column block) at a time: NL x 4 entries in flight per lane
  T raw[NL][4], zc = (T) 0, tt = (T) 0;
  auto request = [&](int q) {    // q = s KB + cb
    const int s = q / KB, cb = q % KB;
    double t;
    const int k = table_interval(xs[s], tb.N, t);
    tt = (T) t;
    zc = tb.z[ms[s] * C + cb * 16 + c];
#pragma unroll
    for (int l = 0; l < NL; l++) table_request(tb, k, l * C + cb * 16 + c, a.noutp, raw[l]);
  };
  if (w0 < w1) geometry(w0, xs, ms);
  for (long long eb = w0; eb < w1; eb += 16) {
    const int nb = (int) (w1 - eb < 16 ? w1 - eb : 16);
    request(0);
    const bool more = eb + 16 < w1;
    if (more) geometry(eb + 16, xn, mn);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    if (lane < 16) {
      if (lane < nb) {
        const double *u = a.rh + 3 * (eb + lane);
        sh_eval<false, T, NL - 1>(a.sh, u[0], u[1], u[2], Yw + lane * a.nlm, nullptr);
      } else {
        for (int q = 0; q < a.nlm; q++) Yw[lane * a.nlm + q] = (T) 0;
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int q = 0; q < 4 * KB; q++) {
      const int s = q / KB, cb = q % KB;
      if (4 * s >= nb) continue;                      // a step with no bond: neither evaluated nor multiplied
      T bv[NL];
#pragma unroll
      for (int l = 0; l < NL; l++) {
        T R, dR;
        table_value<T, false>(raw[l], tt, h, fN, R, dR);
        bv[l] = R * zc;
      }
      if (q + 1 < 4 * KB && 4 * ((q + 1) / KB) < nb) request(q + 1);
      const T *yb = Yw + (4 * s + g) * a.nlm;
#pragma unroll
      for (int l = 0; l < NL; l++) {
        const T y = c < 2 * l + 1 ? yb[l * l + c] : (T) 0;       // A operand: row m = c
        acc[l][cb] = Mfma<T>::mma(y, bv[l], acc[l][cb]);
      }
    }
#pragma unroll
    for (int s = 0; s < 4; s++) { xs[s] = xn[s]; ms[s] = mn[s]; }
  }
  T *Ai = a.A + (long long) ia * a.nlm * C;
#pragma unroll
  for (int l = 0; l < NL; l++) {
#pragma unroll
      for (int v = 0; v < 4; v++) {
        const int m = a.drow[4 * g + v];
        if (m < 2 * l + 1) {
#pragma unroll
          for (int cb = 0; cb < KB; cb++) Ai[(l * l + m) * C + cb * 16 + c] = acc[l][cb][v];
        }
      }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// per-atom dense chain.  Per-atom tensors are [atom][function][channel].
// ---------------------------------------------------------------------------------------------------------------
// Atoms are processed in tiles of 16 (one MFMA tile): tile_atoms[tile * 16 + r] is the atom of row r, or -1.  Tiles
// hold atoms of one element, so that element-dependent weights (rho reduce) are uniform per tile.
//
// Job / segment GEMM of the FC layers on the matrix cores.  Job = one output function; its value for a tile is
//   out[atom][fo][0:N] (+)= scale_job * sum_seg  seg_scale * X_src(seg)[atom][fn(seg)][0:K] . W[wtile(seg)][0:K][0:N]
// FC forward:        job f,  segments (Xl, f, Wl[tile_l f]) and (Xr, from c, Wr[tile c]) for every connection c -> f
// FC reverse, left:  job f,  segment  (g, f, Wl^T[tile_l f]), accumulated into gXl
// FC reverse, right: job r,  segments (g, to c, nof[to c] Wr^T[tile c]) for the connections c from r, accumulated
// Rows of the A operand are the 16 atoms (lane % 16), its k index g * (K / 4) + s (g = lane / 16), so that a lane
// reads K / 4 consecutive channels; weights are stored in that fragment order ([tile][cb][s][lane]) and staged in LDS.
template<class T> struct GemmJobs {
  const int *job_out;         // [njobs] output function
  const T *job_scale;         // [njobs]
  const int *seg_off;         // [njobs + 1]
  const int *seg_src;         // [nseg] 0: X0 (K0 channels), 1: X1 (K1 channels)
  const int *seg_fn;          // [nseg] function of the source tensor
  const int *seg_w;           // [nseg] weight tile
  const T *seg_scale;         // [nseg]
  const T *WF0, *WF1;         // fragments of the weights used with X0 / X1
  int njobs;
  int max_seg;                // most segments of one job
  int drow[16];               // accumulator row of (lane / 16, register), probed on the device
};

constexpr int kGemmMaxSeg = 4;      // most weight tiles staged in LDS at a time (the launch passes the number, mseg)
// atom tiles of a wave (TPW): 2, and 1 for the widest tiles (64 channels in, 64 out), whose accumulators and operands
// of two atom tiles would leave two waves per SIMD
template<int KB0, int KB1, int NB> constexpr int gemm_tiles_per_wave() { return KB0 == 4 && KB1 == 4 && NB == 4 ? 1 : 2; }

template<class T, int KB0, int KB1, int NB, int TPW>
__global__ __launch_bounds__(512) void k_gemm_jobs(GemmJobs<T> J, const T *X0, int nf0, const T *X1, int nf1, T *out, int nfo,
                                                   const int *tile_atoms, int ntiles, int accumulate, int reps, int mseg)
{
  // mseg <= kGemmMaxSeg weight tiles are staged at a time (dynamic LDS: mseg tiles; wide tiles are staged fewer at a
  // time so that several blocks fit a CU).  reps > 1 (only when every job has one segment): the block stages its
  // weight tile once and walks `reps` groups of atom tiles with it
  typedef typename Mfma<T>::v4 v4;
  constexpr int KS0 = KB0 * 4, KS1 = KB1 * 4, KSM = KS0 > KS1 ? KS0 : KS1, K0 = KB0 * 16, K1 = KB1 * 16, N = NB * 16;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  T *wl = reinterpret_cast<T *>(smem_raw);      // [mseg][NB][KSM][64]
  __shared__ int s_src[kGemmMaxSeg], s_fn[kGemmMaxSeg];
  __shared__ T s_scale[kGemmMaxSeg];
  const int job = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwave = blockDim.x >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int sg0 = J.seg_off[job], sg1 = J.seg_off[job + 1];
  const int fo = J.job_out[job];
  const T js = J.job_scale[job];
  for (int rep = 0; rep < reps; rep++) {
    const int tile0 = ((blockIdx.y * reps + rep) * nwave + wave) * TPW;
    if (rep > 0 && (blockIdx.y * reps + rep) * nwave * TPW >= ntiles) break;    // uniform over the block
    v4 acc[TPW][NB];
    int arow[TPW];            // atom of this lane's A row
#pragma unroll
    for (int i = 0; i < TPW; i++) {
      const int tile = tile0 + i;
      arow[i] = tile < ntiles ? tile_atoms[tile * 16 + c] : -1;
#pragma unroll
      for (int cb = 0; cb < NB; cb++) acc[i][cb] = v4{0, 0, 0, 0};
    }
    for (int sg = sg0; sg < sg1; sg += mseg) {
      const int ns = sg1 - sg < mseg ? sg1 - sg : mseg;
      if (rep == 0) {
        __syncthreads();
        for (int q = 0; q < ns; q++) {
          const int src = J.seg_src[sg + q];
          const int ks = src == 0 ? KS0 : KS1;
          const T *wf = (src == 0 ? J.WF0 : J.WF1) + (long long) J.seg_w[sg + q] * NB * ks * 64;
          for (int e = threadIdx.x; e < NB * ks * 64; e += blockDim.x) {
            const int cb = e / (ks * 64), rem = e % (ks * 64);
            wl[(q * NB + cb) * KSM * 64 + rem] = wf[e];
          }
          if (threadIdx.x == 0) { s_src[q] = src; s_fn[q] = J.seg_fn[sg + q]; s_scale[q] = J.seg_scale[sg + q]; }
        }
        __syncthreads();
      }
#pragma unroll
      for (int i = 0; i < TPW; i++) {
        for (int q = 0; q < ns; q++) {
          const T sc = s_scale[q];
          const T *wq = wl + q * NB * KSM * 64 + lane;
          if (s_src[q] == 0) {
            T x[KS0];
            if (arow[i] >= 0) {
              const T *xp = X0 + ((long long) arow[i] * nf0 + s_fn[q]) * K0 + g * KS0;
#pragma unroll
              for (int s = 0; s < KS0; s++) x[s] = xp[s] * sc;
            } else {
#pragma unroll
              for (int s = 0; s < KS0; s++) x[s] = (T) 0;
            }
#pragma unroll
            for (int cb = 0; cb < NB; cb++)
#pragma unroll
              for (int s = 0; s < KS0; s++) acc[i][cb] = Mfma<T>::mma(x[s], wq[(cb * KSM + s) * 64], acc[i][cb]);
          } else {
            T x[KS1];
            if (arow[i] >= 0) {
              const T *xp = X1 + ((long long) arow[i] * nf1 + s_fn[q]) * K1 + g * KS1;
#pragma unroll
              for (int s = 0; s < KS1; s++) x[s] = xp[s] * sc;
            } else {
#pragma unroll
              for (int s = 0; s < KS1; s++) x[s] = (T) 0;
            }
#pragma unroll
            for (int cb = 0; cb < NB; cb++)
#pragma unroll
              for (int s = 0; s < KS1; s++) acc[i][cb] = Mfma<T>::mma(x[s], wq[(cb * KSM + s) * 64], acc[i][cb]);
          }
        }
      }
    }
    // accumulator (g, v) holds row drow[4 g + v] of the tile, column cb * 16 + c
#pragma unroll
    for (int i = 0; i < TPW; i++) {
      const int tile = tile0 + i;
      if (tile >= ntiles) continue;
#pragma unroll
      for (int v = 0; v < 4; v++) {
        const int at = tile_atoms[tile * 16 + J.drow[4 * g + v]];
        if (at < 0) continue;
        T *o = out + ((long long) at * nfo + fo) * N + c;
#pragma unroll
        for (int cb = 0; cb < NB; cb++) {
          const T val = js * acc[i][cb][v];
          o[cb * 16] = accumulate ? o[cb * 16] + val : val;
        }
      }
    }
  }
}

// Block index -> (function q, atom group) for grids of nq * 8 * ceil(groups / 8) blocks.  Workgroups go to the 8 XCDs
// round-robin by linear index and every XCD has its own L2: the blocks of one atom group (all its functions q) are
// given consecutive indices on ONE XCD, so that the per-atom tensors they share are fetched into one L2 once.
__device__ inline void xcd_block(int nq, int &q, int &group)
{
  const int L = blockIdx.x, xcd = L & 7, rest = L >> 3;
  q = rest % nq;
  group = (rest / nq) * 8 + xcd;
}

struct ProdDev {
  // forward: terms sorted by output (CSR off over nout; only live outputs have terms)
  const int *off, *l, *r;
  const double *c;
  // reverse: terms by left operand (loff over nleft) and by right operand (roff over nright)
  const int *loff, *l_o, *l_r;
  const double *l_c;
  const int *roff, *r_o, *r_l;
  const double *r_c;
  int nout, nleft, nright;
};

// out[a][o][k] = sum_t c_t L[a][l_t][k] R[a][r_t][k]      grid: xcd_block over (nout, atom groups), block = C x AT
template<class T> __global__ void k_prod_fwd(ProdDev P, const T *L, const T *R, T *out, int natoms, int C, int sl, int sr)
{
  const int k = threadIdx.x % C, al = threadIdx.x / C;
  int o, ag;
  xcd_block(P.nout, o, ag);
  const int at = ag * (blockDim.x / C) + al;
  if (at >= natoms) return;
  const T *La = L + (long long) at * sl * C + k, *Ra = R + (long long) at * sr * C + k;
  T acc = (T) 0;
  for (int t = P.off[o]; t < P.off[o + 1]; t++) acc += (T) P.c[t] * La[(long long) P.l[t] * C] * Ra[(long long) P.r[t] * C];
  out[((long long) at * P.nout + o) * C + k] = acc;
}

// gL[a][q][k] += sum_{t: l_t = q} c_t g[a][o_t][k] R[a][r_t][k]   (side 0), gR likewise with L (side 1)
// grid (nleft or nright, atom groups)
template<class T> __global__ void k_prod_bwd(ProdDev P, int side, const T *other, const T *g, T *gX, int natoms, int C, int so,
                                             int sx)
{
  const int k = threadIdx.x % C, al = threadIdx.x / C;
  int q, ag;
  xcd_block(side == 0 ? P.nleft : P.nright, q, ag);
  const int at = ag * (blockDim.x / C) + al;
  if (at >= natoms) return;
  const int *off = side == 0 ? P.loff : P.roff, *oo = side == 0 ? P.l_o : P.r_o, *ot = side == 0 ? P.l_r : P.r_l;
  const double *cc = side == 0 ? P.l_c : P.r_c;
  if (off[q] == off[q + 1]) return;
  const T *Oa = other + (long long) at * so * C + k, *ga = g + (long long) at * P.nout * C + k;
  T acc = (T) 0;
  for (int t = off[q]; t < off[q + 1]; t++) acc += (T) cc[t] * ga[(long long) oo[t] * C] * Oa[(long long) ot[t] * C];
  gX[((long long) at * sx + q) * C + k] += acc;
}

template<class T> struct ReduceDev {
  // per source s: collected functions fn[s][c] (unique), weights in fragment order
  //   forward WF[s][mu][c][cb][ks][lane]  = W_s[mu][c][n = g KS + ks][k = cb 16 + lane % 16]    (norm folded, k >= nrho zero)
  //   reverse WB[s][mu][c][cb][ks][lane]  = W_s[mu][c][n = cb 16 + lane % 16][k = g KSR + ks]
  const T *WF[4], *WB[4];
  const int *fn[4];
  int ncol[4], nin[4], stride[4];    // collected functions, (padded) channels, functions per atom of the source
  int nsrc, nrho, nbr, ksr;          // rho width, its 16-column blocks, k-steps of the reverse (ceil(nrho / 4))
  int ostride, ooff;                 // output row of an atom: rho[atom * ostride + ooff + k]
  int drow[16];                      // accumulator row of (lane / 16, register)
};

// rho[atom][k] = sum_s sum_c sum_n W_s[mu][c][n][k] X_s[atom][fn c][n] on the matrix cores: one block per tile of
// 16 atoms, its kReduceWaves waves split the (s, c) list, partial tiles summed through LDS.  KBA / KBF: 16-channel blocks of
// source 0 (A) and of the other sources.
constexpr int kReduceWaves = 8;    // waves of a k_reduce_fwd block: each takes every eighth collected function
template<class T, int KBA, int KBF>
__global__ __launch_bounds__(64 * kReduceWaves) void k_reduce_fwd(ReduceDev<T> R, const int *mu, const int *tile_atoms, const T *X0, const T *X1,
                                                    const T *X2, const T *X3, double *rho)
{
  typedef typename Mfma<T>::v4 v4;
  __shared__ double part[kReduceWaves][2][16][17];
  const int tile = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int arow = tile_atoms[tile * 16 + c];
  const int a0 = tile_atoms[tile * 16];
  const int m = mu[a0];
  const T *X[4] = {X0, X1, X2, X3};
  v4 acc[2] = {v4{0, 0, 0, 0}, v4{0, 0, 0, 0}};
  int job = 0;
  for (int s = 0; s < R.nsrc; s++) {
    const int ks = (s == 0 ? KBA : KBF) * 4, K = ks * 4;
    for (int cc = 0; cc < R.ncol[s]; cc++, job++) {
      if (job % kReduceWaves != wave) continue;
      const T *wf = R.WF[s] + ((long long) m * R.ncol[s] + cc) * R.nbr * ks * 64 + lane;
      T x[(KBA > KBF ? KBA : KBF) * 4];
      if (arow >= 0) {
        const T *xp = X[s] + ((long long) arow * R.stride[s] + R.fn[s][cc]) * K + g * ks;
#pragma unroll
        for (int q = 0; q < (KBA > KBF ? KBA : KBF) * 4; q++) x[q] = q < ks ? xp[q] : (T) 0;
      } else {
#pragma unroll
        for (int q = 0; q < (KBA > KBF ? KBA : KBF) * 4; q++) x[q] = (T) 0;
      }
#pragma unroll
      for (int cb = 0; cb < 2; cb++)
        if (cb < R.nbr) {
#pragma unroll
          for (int q = 0; q < (KBA > KBF ? KBA : KBF) * 4; q++)
            if (q < ks) acc[cb] = Mfma<T>::mma(x[q], wf[(cb * ks + q) * 64], acc[cb]);
        }
    }
  }
#pragma unroll
  for (int cb = 0; cb < 2; cb++)
#pragma unroll
    for (int v = 0; v < 4; v++) part[wave][cb][R.drow[4 * g + v]][c] = (double) acc[cb][v];
  __syncthreads();
  for (int e = threadIdx.x; e < 16 * R.nrho; e += 64 * kReduceWaves) {
    const int r = e / R.nrho, k = e % R.nrho;
    const int at = tile_atoms[tile * 16 + r];
    if (at < 0) continue;
    double v = 0.0;
    for (int w = 0; w < kReduceWaves; w++) v += part[w][k >> 4][r][k & 15];
    rho[(long long) at * R.ostride + R.ooff + k] = v;
  }
}

// gX_s[atom][fn c][n] += sum_k grho[atom][k] W_s[mu][c][n][k]: grid (tiles, jobs), one wave per block; the jobs are all
// (s, c) in the order of the sources, this launch takes those from job_first on.  overwrite: the rows are written, not
// added to (for callers that know every row is visited once and read no row that is not visited)
template<class T>
__global__ __launch_bounds__(64) void k_reduce_bwd(ReduceDev<T> R, const int *mu, const int *tile_atoms, const double *grho, T *G0, T *G1,
                                                   T *G2, T *G3, int job_first = 0, int overwrite = 0)
{
  typedef typename Mfma<T>::v4 v4;
  const int tile = blockIdx.x;
  int job = blockIdx.y + job_first, s = 0;
  while (job >= R.ncol[s]) { job -= R.ncol[s]; s++; }
  const int lane = threadIdx.x, c = lane & 15, g = lane >> 4;
  const int arow = tile_atoms[tile * 16 + c];
  const int m = mu[tile_atoms[tile * 16]];
  T *G[4] = {G0, G1, G2, G3};
  T x[8];
#pragma unroll
  for (int q = 0; q < 8; q++) {
    const int k = g * R.ksr + q;
    x[q] = (arow >= 0 && q < R.ksr && k < R.nrho) ? (T) grho[(long long) arow * R.ostride + R.ooff + k] : (T) 0;
  }
  const int nb = R.nin[s] / 16;
  const T *wb = R.WB[s] + ((long long) m * R.ncol[s] + job) * nb * R.ksr * 64 + lane;
  const int fn = R.fn[s][job];
  for (int cb = 0; cb < nb; cb++) {
    v4 acc = {0, 0, 0, 0};
#pragma unroll
    for (int q = 0; q < 8; q++)
      if (q < R.ksr) acc = Mfma<T>::mma(x[q], wb[(cb * R.ksr + q) * 64], acc);
#pragma unroll
    for (int v = 0; v < 4; v++) {
      const int at = tile_atoms[tile * 16 + R.drow[4 * g + v]];
      if (at >= 0) {
        T *out = &G[s][((long long) at * R.stride[s] + fn) * R.nin[s] + cb * 16 + c];
        *out = overwrite ? acc[v] : *out + acc[v];
      }
    }
  }
}


struct EnergyDev {
  const double *W[7];         // [n_in][n_out]
  double norm[7];
  int nin[7], nout[7];
  int nlay, act, ln, nrho, width;    // width: largest layer width (LDS row of the kernel)
  int wlds;                   // weights staged in LDS (sum of n_in n_out values, twice: as stored and transposed), or 0
  double out_scale;
  const double *shift;        // [nel]
};

constexpr int kEnergyAtomsPerBlock = 16;    // atoms of one block of k_energy (4 waves, 4 atoms each)

// E_i = (MLP(rho[1:]) + rho[0]) out_scale + shift[mu_i] and dE/drho, fp64, one wave per atom (fused_1l.cpp:378-427;
// legacy RMS layer norm fused_cpu.h:666-682).  A block of 4 waves shares the staged weights and walks
// kEnergyAtomsPerBlock atoms; WLDS: the weights of the network sit in LDS (as stored and transposed), else they are
// read from global memory.  A layer with fewer than 33 outputs splits each dot product over 64 / outputs lanes (the
// last layer's single output: all 64).  Without structure records the block adds its energies to the total with one
// atomic.  dynamic LDS: M.wlds + 4 x (2 nlay + 4) x width doubles.
template<bool WLDS>
static __global__ __launch_bounds__(256) void k_energy(EnergyDev M, const int *mu, int a0, int natoms, const double *rho, double *grho,
                                                         double *eatom_chunk, double *energy, int want_grad, const int *sid)
{
  // LDS rows of W = M.width values per wave: nlay + 1 activations, nlay pre-activations, 2 adjoint buffers, x0
  extern __shared__ __align__(16) unsigned char smem_raw[];
  const int W = M.width;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  double *wl0 = reinterpret_cast<double *>(smem_raw);
  double *act_ = wl0 + (WLDS ? M.wlds : 0) + wave * (2 * M.nlay + 4) * W, *pre_ = act_ + (M.nlay + 1) * W, *gbuf_ = pre_ + M.nlay * W,
         *x0 = gbuf_ + 2 * W;
#define act(L_, k_) act_[(L_) * W + (k_)]
#define pre(L_, k_) pre_[(L_) * W + (k_)]
#define gbuf(L_, k_) gbuf_[(L_) * W + (k_)]
  // the rows of a wave are its own: a wave-level barrier orders its LDS writes before the reads of its other lanes
#define GR_WAVE_SYNC()                                        \
  do {                                                        \
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");    \
    __builtin_amdgcn_wave_barrier();                          \
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");    \
  } while (0)
  // as stored [a][c] for the forward pass and transposed [c][a] for the reverse: one round of coalesced loads per block
  // instead of a dependent chain of them per layer and atom
  const double *wf[7], *wt[7];
  {
    double *wl = wl0;
    for (int L = 0; L < M.nlay; L++) {
      const int sz = M.nin[L] * M.nout[L];
      if (WLDS) {
        for (int e = threadIdx.x; e < sz; e += 256) {
          const double v = M.W[L][e];
          wl[e] = v;
          wl[sz + (e % M.nout[L]) * M.nin[L] + e / M.nout[L]] = v;
        }
        wf[L] = wl;
        wt[L] = wl + sz;
        wl += 2 * sz;
      } else {
        wf[L] = M.W[L];
        wt[L] = nullptr;
      }
    }
  }
  __syncthreads();
  const int n0 = M.nrho - 1;
  // lanes that share one output of a layer: the largest power of two g with outputs x g <= 64
  auto group = [](int nout_) {
    int g = 1;
    while (g < 64 && nout_ * (g * 2) <= 64) g *= 2;
    return g;
  };
  double esum = 0.0;                                // lane 0: energies of this wave's atoms (no structure records)
  for (int k4 = 0; k4 < kEnergyAtomsPerBlock / 4; k4++) {
    const int at = blockIdx.x * kEnergyAtomsPerBlock + k4 * 4 + wave;
    if (at >= natoms) break;                        // uniform over the wave; no block barrier inside the loop
    const double *r = rho + (long long) at * M.nrho;
    GR_WAVE_SYNC();                                 // the rows of the previous atom are no longer read
    for (int k = lane; k < n0; k += 64) act(0, k) = r[k + 1];
    GR_WAVE_SYNC();
    double q = 0.0;
    if (M.ln) {
      double ms = 0.0;
      for (int k = lane; k < n0; k += 64) { x0[k] = act(0, k); ms += act(0, k) * act(0, k); }
      for (int o = 32; o > 0; o >>= 1) ms += __shfl_xor(ms, o, 64);
      q = 1.0 / sqrt(ms / n0 + 1e-16);
      for (int k = lane; k < n0; k += 64) act(0, k) *= q;
      GR_WAVE_SYNC();
    }
    for (int L = 0; L < M.nlay; L++) {
      const int no = M.nout[L], ni = M.nin[L], g = group(no), p = lane % g;
      for (int c0 = 0; c0 < no; c0 += 64 / g) {     // every lane walks the loop: the exchanges below need the whole wave
        const int c = c0 + lane / g;
        double s = 0.0;
        if (c < no) {
#pragma unroll 4
          for (int a = p; a < ni; a += g) s += act(L, a) * wf[L][a * no + c];
        }
        for (int o = g >> 1; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
        if (c < no && p == 0) {
          s *= M.norm[L];
          pre(L, c) = s;
          act(L + 1, c) = (L < M.nlay - 1) ? (M.act == 1 ? tanh(s) : s / (1.0 + exp(-s))) : s;
        }
      }
      GR_WAVE_SYNC();
    }
    const double Ei = (act(M.nlay, 0) + r[0]) * M.out_scale + M.shift[mu[a0 + at]];
    if (lane == 0) {
      if (eatom_chunk) eatom_chunk[at] = Ei;
      if (!energy) {}    // ordered mode: the records are summed from the per-atom energies afterwards
      else if (sid) atomicAdd(energy + 8 * sid[a0 + at], Ei);    // one (energy, virial[6]) record of 8 doubles per structure
      else esum += Ei;
    }
    if (!want_grad) continue;
    int cur = 0;
    if (lane == 0) gbuf(0, 0) = M.out_scale;
    GR_WAVE_SYNC();
    for (int L = M.nlay - 1; L >= 0; L--) {
      if (L < M.nlay - 1) {
        for (int c = lane; c < M.nout[L]; c += 64) {
          const double v = pre(L, c);
          if (M.act == 1) {
            const double t = act(L + 1, c);
            gbuf(cur, c) *= 1.0 - t * t;
          } else {
            const double sg = 1.0 / (1.0 + exp(-v));
            gbuf(cur, c) *= sg * (1.0 + v * (1.0 - sg));
          }
        }
        GR_WAVE_SYNC();
      }
      {
        const int no = M.nout[L], ni = M.nin[L], g = group(ni), p = lane % g;
        for (int b0 = 0; b0 < ni; b0 += 64 / g) {
          const int a = b0 + lane / g;
          double s = 0.0;
          if (a < ni) {
            if (WLDS) {
#pragma unroll 4
              for (int c = p; c < no; c += g) s += gbuf(cur, c) * wt[L][c * ni + a];
            } else {
#pragma unroll 4
              for (int c = p; c < no; c += g) s += gbuf(cur, c) * wf[L][(long long) a * no + c];
            }
          }
          for (int o = g >> 1; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
          if (a < ni && p == 0) gbuf(cur ^ 1, a) = s * M.norm[L];
        }
      }
      cur ^= 1;
      GR_WAVE_SYNC();
    }
    if (M.ln) {
      double t = 0.0;
      for (int k = lane; k < n0; k += 64) t += gbuf(cur, k) * x0[k];
      for (int o = 32; o > 0; o >>= 1) t += __shfl_xor(t, o, 64);
      for (int k = lane; k < n0; k += 64) gbuf(cur, k) = q * (gbuf(cur, k) - x0[k] * t * q * q / n0);
      GR_WAVE_SYNC();
    }
    double *g = grho + (long long) at * M.nrho;
    if (lane == 0) g[0] = M.out_scale;
    for (int k = lane; k < n0; k += 64) g[k + 1] = gbuf(cur, k);
  }
  if (!sid && energy) {    // one atomic per block (every wave leaves the loop above and arrives here)
    __shared__ double eblk[4];
    if (lane == 0) eblk[wave] = esum;
    __syncthreads();
    if (threadIdx.x == 0) {
      const double e = eblk[0] + eblk[1] + eblk[2] + eblk[3];
      if (e != 0.0) atomicAdd(energy, e);
    }
  }
#undef GR_WAVE_SYNC
#undef act
#undef pre
#undef gbuf
}

// ---------------------------------------------------------------------------------------------------------------
// UQ head (uqv6, gamma only)
// ---------------------------------------------------------------------------------------------------------------
constexpr int kUqMaxSrc = 8, kUqMaxBlk = 3;
template<class T> struct UqDev {
  const T *X[kUqMaxSrc];      // per-atom tensors of the reduces' sources [atom][function][channel]
  const int *ci[kUqMaxSrc];   // collected functions of each source
  int nfun[kUqMaxSrc], cpad[kUqMaxSrc], nin[kUqMaxSrc], nc[kUqMaxSrc], off[kUqMaxSrc];    // functions per atom, padded / real channels, collected, first basis index
  int blk[kUqMaxSrc];         // invariant block of the source (1L: rho = 0; 2L: I2 = 0, rho = 1; 3L: layer)
  int nsrc, nblk, rp, D, K;
  int row0, d_basis;          // this launch holds rows row0 .. row0 + d_basis of the basis (off[] counts from row0)
  int carry_in, carry_out;    // 3L, one launch per layer: add the projection and block norms kept by the earlier layers / keep them and stop
  double *zacc, *n2acc;       // [atom][rp], [atom][kUqMaxBlk]: the kept raw projection and squared block norms
  double density_scale;
  const double *R;            // [d_basis][rp]
  const double *cen;          // [nel][K][D]
  const double *icov;         // [nel][K][D][D]
  const int *ncl;             // [nel]
  const double *thr;          // [nel][K]
};

// gamma, sigma, cluster of one atom per block (libgrace/include/grace/fused_cpu.h:1290-1312 basis, :1375-1412 GMM;
// libgrace/src/fused_1l.cpp:616-636, fused_2l.cpp:1156-1186): basis B = per invariant block the collected functions of
// the reduce's sources, n-outer and c-inner per source; phi = ((B / |B|) R, log |B| scale, log |B_block| scale ...);
// nearest centroid of the atom's element, Mahalanobis distance over the cluster's threshold.  fp64 throughout.
// GRACE-3L (libgrace/src/fused_3l.cpp:1156-1201) evaluates the rows of one layer per launch, right after that layer's
// rho reduce while its tensors exist: raw projection and squared block norms are carried in zacc / n2acc.
// block: 256 threads; dynamic LDS: d_basis + 4 rp + 2 D doubles.
template<class T>
__global__ __launch_bounds__(256) void k_uq(UqDev<T> U, const int *mu, int natoms, double *gamma, double *sigma, double *cluster)
{
  extern __shared__ __align__(16) unsigned char smem_raw[];
  double *Bsh = reinterpret_cast<double *>(smem_raw);       // [d_basis]
  double *Zp = Bsh + U.d_basis;                             // [4][rp] partial projections
  double *f = Zp + 4 * U.rp;                                // [D]
  double *dl = f + U.D;                                     // [D]
  __shared__ double wsum[4], bsum[4][kUqMaxBlk];
  __shared__ int kstar;
  const int at = blockIdx.x, t = threadIdx.x, lane = t & 63, wave = t >> 6;
  if (at >= natoms) return;
  // ---- basis and the norms of its blocks
  double n2[kUqMaxBlk];
#pragma unroll
  for (int b = 0; b < kUqMaxBlk; b++) n2[b] = 0.0;
  for (int s = 0; s < U.nsrc; s++) {
    const T *x = U.X[s] + (long long) at * U.nfun[s] * U.cpad[s];
    const int w = U.nin[s] * U.nc[s];
    double acc = 0.0;
    for (int r = t; r < w; r += 256) {
      const int n = r / U.nc[s], c = r % U.nc[s];
      const double v = (double) x[U.ci[s][c] * U.cpad[s] + n];
      Bsh[U.off[s] + r] = v;
      acc += v * v;
    }
#pragma unroll
    for (int b = 0; b < kUqMaxBlk; b++)
      if (U.blk[s] == b) n2[b] += acc;
  }
#pragma unroll
  for (int b = 0; b < kUqMaxBlk; b++) {
    for (int o = 32; o > 0; o >>= 1) n2[b] += __shfl_xor(n2[b], o, 64);
    if (lane == 0) bsum[wave][b] = n2[b];
  }
  __syncthreads();
  double nb2[kUqMaxBlk], tot = 0.0;
#pragma unroll
  for (int b = 0; b < kUqMaxBlk; b++) {
    nb2[b] = bsum[0][b] + bsum[1][b] + bsum[2][b] + bsum[3][b];
    if (U.carry_in) nb2[b] += U.n2acc[(long long) at * kUqMaxBlk + b];
    tot += nb2[b];
  }
  const double nrm = sqrt(tot);
  // ---- projection Z = B R: column d = t mod rp, rows split over the 256 / rp (at most 4 used) thread groups
  {
    const int ng = 256 / U.rp > 4 ? 4 : 256 / U.rp, gq = t / U.rp, d = t % U.rp;
    if (gq < ng) {
      double z = 0.0;
      for (int b = gq; b < U.d_basis; b += ng) z += Bsh[b] * U.R[(long long) (U.row0 + b) * U.rp + d];
      Zp[gq * U.rp + d] = z;
    }
    __syncthreads();
    if (t < U.D) {
      if (t < U.rp) {
        double z = 0.0;
        for (int q = 0; q < ng; q++) z += Zp[q * U.rp + t];
        if (U.carry_in) z += U.zacc[(long long) at * U.rp + t];
        if (U.carry_out) U.zacc[(long long) at * U.rp + t] = z;
        f[t] = z / (nrm + 1.0e-12);
      } else {    // density channels: the whole basis, then its blocks (one block: the same norm again)
        const int p = t - U.rp;
        double dn = nrm;
#pragma unroll
        for (int b = 0; b < kUqMaxBlk; b++)
          if (p == 1 + b) dn = sqrt(nb2[b]);
        f[t] = log(dn + 1.0e-12) * U.density_scale;
      }
    }
    if (U.carry_out) {    // the same for every thread of the block
#pragma unroll
      for (int b = 0; b < kUqMaxBlk; b++)
        if (t == b) U.n2acc[(long long) at * kUqMaxBlk + b] = nb2[b];
      return;
    }
    __syncthreads();
  }
  // ---- nearest centroid of the element (the first of equal distances)
  const int m = mu[at];
  if (t == 0) {
    int kb = 0;
    double best = 1.0e300;
    for (int q = 0; q < U.ncl[m]; q++) {
      const double *c = U.cen + ((long long) m * U.K + q) * U.D;
      double d2 = 0.0;
      for (int p = 0; p < U.D; p++) d2 += (f[p] - c[p]) * (f[p] - c[p]);
      if (d2 < best) { best = d2; kb = q; }
    }
    kstar = kb;
  }
  __syncthreads();
  const int kq = kstar;
  for (int p = t; p < U.D; p += 256) dl[p] = f[p] - U.cen[((long long) m * U.K + kq) * U.D + p];
  __syncthreads();
  // ---- sigma^2 = delta^T S delta
  const double *S = U.icov + ((long long) m * U.K + kq) * U.D * U.D;
  double part = 0.0;
  for (int p = t; p < U.D; p += 256) {
    double y = 0.0;
    for (int q = 0; q < U.D; q++) y += S[(long long) p * U.D + q] * dl[q];
    part += dl[p] * y;
  }
  for (int o = 32; o > 0; o >>= 1) part += __shfl_xor(part, o, 64);
  __syncthreads();
  if (lane == 0) wsum[wave] = part;
  __syncthreads();
  if (t == 0) {
    const double sg = sqrt(wsum[0] + wsum[1] + wsum[2] + wsum[3] + 1.0e-8);
    const double th = U.thr[(long long) m * U.K + kq];
    sigma[at] = sg;
    gamma[at] = sg / (th > 1.0e-10 ? th : 1.0e-10);
    cluster[at] = (double) kq;
  }
}

// Two unit vectors that span the plane normal to the unit vector u: e1 = a x u / |a x u| with a the coordinate axis on
// which u has its smallest component, e2 = u x e1.  A pure function of u: the kernel that stores tangential gradients
// and the kernel that turns their adjoints into a force compute the same pair.
__device__ inline void tangent_basis(const double *u, double *e1, double *e2)
{
  const double ax = fabs(u[0]), ay = fabs(u[1]), az = fabs(u[2]);
  double a[3] = {0.0, 0.0, 0.0};
  if (ax <= ay && ax <= az) a[0] = 1.0;
  else if (ay <= az) a[1] = 1.0;
  else a[2] = 1.0;
  const double c0 = a[1] * u[2] - a[2] * u[1], c1 = a[2] * u[0] - a[0] * u[2], c2 = a[0] * u[1] - a[1] * u[0];
  const double inv = 1.0 / sqrt(c0 * c0 + c1 * c1 + c2 * c2);
  e1[0] = c0 * inv; e1[1] = c1 * inv; e1[2] = c2 * inv;
  e2[0] = u[1] * e1[2] - u[2] * e1[1]; e2[1] = u[2] * e1[0] - u[0] * e1[2]; e2[2] = u[0] * e1[1] - u[1] * e1[0];
}

// ---------------------------------------------------------------------------------------------------------------
// bond backward: forces and virial
// ---------------------------------------------------------------------------------------------------------------
template<class T> struct BondBwdArgs {
  const long long *eoff;
  const int *ej;
  const double *rh, *r, *rc;
  const T *Rz, *dRz;          // [E][noutp]
  RadialTable<T> tb;          // tb.F set: value and derivative of the radial functions come from the tables, Rz / dRz are not read
  const T *gA;                // [chunk atoms][nlm][C]
  double *f;                  // [n][3]  (+=, atomics)
  double *virial;             // [6]     (+=, atomics); with sid: record 8 sid[i] of the atom's structure
  const int *sid;             // [n] structure of each atom, or null
  double *vatom;              // [n][9] per-atom virial xx yy zz xy xz yz yx zx zy (+=, atomics), or null: half of a bond's (-r rhat) (x) fv to each of its atoms
  // ordered mode (both set, no atomics, vatom null): fedge[e][3] = force of bond e on its central atom; fcen[i][9] = sum of
  // these over the bonds of atom i, then the six virial sums of its bonds; k_ordered_forces / k_ordered_records finish
  double *fedge, *fcen;
  int ordered_add;            // ordered mode: add to what fedge / fcen hold (a later layer of the same pass) instead of storing
  int a0;
  int C, nl, nlm, noutp;
  int drow[16];               // accumulator row of (lane / 16, register)
  ShCoef sh;
};

// One block (4 waves) per atom; a wave takes tiles of 16 bonds.  Per tile and l two tile GEMMs on the matrix cores,
//   P[m][b] = sum_n gA[l*l + m][n] Rz[b][l][n],   Q[m][b] = sum_n gA[l*l + m][n] dRz[b][l][n]      (K = channels)
// with the bonds as columns: lane (g, c) of the wave ends up with the rows m = drow[4 g + v] of bond c, so the sums over
// m are four terms in the lane and two exchanges between the lane groups, and lane c < 16 -- the lane that evaluated
// the harmonics of bond c and holds its geometry in registers -- finishes the bond:
//   g_d = sum_lm G[b][lm][d] P[lm][b],  dE/dx = sum_lm Y[b][lm] Q[lm][b],
//   fv = dE/dx / rc rhat + (g - (g . rhat) rhat) / r;  f_i += fv, f_j -= fv, virial += (-r rhat) (x) fv
// (fused_cpu.h:836-860,1027-1050; fused_1l.cpp:46-51 of the reference).  Only the part of g normal to the bond enters,
// g - (g . rhat) rhat = (g . e1) e1 + (g . e2) e2 for an orthonormal pair e1, e2 normal to the bond (tangent_basis), so
// the harmonics' gradients are kept as their two components along e1 and e2: two sums per bond instead of three, and a
// third less LDS per block (three blocks per CU instead of two).  gA of the atom sits in LDS as [lm][C + 2]
// (the pad spreads the rows over the banks); the radial rows of l + 1 are requested before the products of l.
// KB = channels / 16, NL = lmax + 1.  dynamic LDS: nlm (C + 2) + 4 waves x 16 bonds x 3 nlm values.
// TAB: the B operands are formed from the radial tables (lane (g, c): the eight columns l C + 8 g + s of bond c, four table
// entries each, value and derivative from the same four; requested for l + 1 before the products of l).
template<class T, int KB, int NL, bool TAB> __global__ __launch_bounds__(256) void k_bond_bwd(BondBwdArgs<T> a)
{
  typedef typename Mfma<T>::v4 v4;
  constexpr int KS = KB * 4, C = KB * 16, CS = C + 2, NLM = NL * NL;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  T *gAl = reinterpret_cast<T *>(smem_raw);                          // [NLM][CS]
  T *Ysh = gAl + NLM * CS;                                           // [4 waves][16][NLM]
  T *Gsh = Ysh + 4 * 16 * NLM;                                       // [4 waves][16][2][NLM]: gradient . e1, gradient . e2
  __shared__ double red[4][9];
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
  const int c = lane & 15, g = lane >> 4;
  const int i = a.a0 + blockIdx.x;
  const long long e0 = a.eoff[i], e1 = a.eoff[i + 1];
  {
    const T *gAi = a.gA + (long long) blockIdx.x * NLM * C;
    for (int q = t; q < NLM * C; q += 256) gAl[(q / C) * CS + q % C] = gAi[q];
  }
  __syncthreads();
  T *Yw = Ysh + wave * 16 * NLM, *Gw = Gsh + wave * 16 * 2 * NLM;
  int mrow[4];
#pragma unroll
  for (int v = 0; v < 4; v++) mrow[v] = a.drow[4 * g + v];
  double fi[3] = {0, 0, 0}, vir[6] = {0, 0, 0, 0, 0, 0};
  const int ntile = (int) ((e1 - e0 + 15) / 16);
  for (int tile = wave; tile < ntile; tile += 4) {
    const long long eb = e0 + (long long) tile * 16;
    const int nb = (int) (e1 - eb < 16 ? e1 - eb : 16);
    const bool colok = c < nb;                      // B operand column = bond c of the tile
    // rows read by this lane: without tables step s of lane group g is channel 8 (s / 2) + 2 g + s % 2 (CH), so that the
    // four lane groups read 64 consecutive bytes of a bond's row in one instruction; with tables channel g KS + s
    const T *rp = a.Rz + (eb + (colok ? c : 0)) * a.noutp + (TAB ? g * KS : 2 * g);
    const T *dp = a.dRz + (eb + (colok ? c : 0)) * a.noutp + (TAB ? g * KS : 2 * g);
#define CH(s_) (TAB ? (s_) : 8 * ((s_) >> 1) + ((s_) & 1))
    T x[2][KS], dx[2][KS];
    // tables: interval, offset and species weights of bond c, and the entries of l = 0
    // (four columns at a time: the entries of the next four are requested before the products of these four)
    constexpr int KH = 4;
    T raw[TAB ? KH : 1][4], zc[TAB ? KS : 1], tt = (T) 0;
    int tk = 0;
    const T th = TAB ? (T) (1.0 / a.tb.N) : (T) 0, tN = TAB ? (T) a.tb.N : (T) 0;
    if constexpr (TAB) {
      const long long e = eb + (colok ? c : 0);
      double t;
      tk = table_interval(a.tb.x[e], a.tb.N, t);
      tt = (T) t;
      const int mu = a.tb.emu[e];
#pragma unroll
      for (int s = 0; s < KS; s++) zc[s] = a.tb.z[mu * C + g * KS + s];
    } else {
#pragma unroll
      for (int s = 0; s < KS; s++) { x[0][s] = rp[CH(s)]; dx[0][s] = dp[CH(s)]; }
    }
    // geometry of bond `lane` (lanes below nb), kept for the end of the tile
    double u0 = 0, u1 = 0, u2 = 1, br = 1, brc = 1;
    double e1[3] = {1, 0, 0}, e2[3] = {0, 1, 0};
    int jj = 0;
    if (lane < nb) {
      const long long e = eb + lane;
      u0 = a.rh[3 * e]; u1 = a.rh[3 * e + 1]; u2 = a.rh[3 * e + 2];
      br = a.r[e]; brc = a.rc[e]; jj = a.ej[e];
      const double u[3] = {u0, u1, u2};
      tangent_basis(u, e1, e2);
      sh_eval<true, T, NL - 1>(a.sh, u0, u1, u2, Yw + lane * NLM, Gw + lane * 2 * NLM, e1, e2, Gw + lane * 2 * NLM + NLM);
    }
    if constexpr (TAB) {
#pragma unroll
      for (int s = 0; s < KH; s++) table_request(a.tb, tk, g * KS + s, a.noutp, raw[s]);
    }
    // LDS writes of this wave visible to its other lanes (the Y / G region is private to the wave)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    double px = 0, p1 = 0, p2 = 0;
#pragma unroll
    for (int l = 0; l < NL; l++) {
      const int cur = TAB ? 0 : (l & 1), nxt = cur ^ 1;
      if constexpr (!TAB) {
        if (l + 1 < NL) {
#pragma unroll
          for (int s = 0; s < KS; s++) { x[nxt][s] = rp[(l + 1) * C + CH(s)]; dx[nxt][s] = dp[(l + 1) * C + CH(s)]; }
        }
      }
      v4 aP = {0, 0, 0, 0}, aQ = {0, 0, 0, 0};
      // A operand: row m = c of gA_l^T, k = g KS + s
      const T *ga = gAl + (l * l + (c < 2 * l + 1 ? c : 0)) * CS + (TAB ? g * KS : 2 * g);
      if constexpr (TAB) {
#pragma unroll
        for (int hb = 0; hb < KS; hb += KH) {
          T xv[KH], dxv[KH];
#pragma unroll
          for (int s = 0; s < KH; s++) {
            T R, dR;
            table_value<T, true>(raw[s], tt, th, tN, R, dR);
            xv[s] = R * zc[hb + s];
            dxv[s] = dR * zc[hb + s];
          }
          // the next four columns: of this l, or the first four of l + 1
          if (hb + KH < KS) {
#pragma unroll
            for (int s = 0; s < KH; s++) table_request(a.tb, tk, l * C + g * KS + hb + KH + s, a.noutp, raw[s]);
          } else if (l + 1 < NL) {
#pragma unroll
            for (int s = 0; s < KH; s++) table_request(a.tb, tk, (l + 1) * C + g * KS + s, a.noutp, raw[s]);
          }
#pragma unroll
          for (int s = 0; s < KH; s++) {
            const T w = c < 2 * l + 1 ? ga[hb + s] : (T) 0;
            aP = Mfma<T>::mma(w, xv[s], aP);
            aQ = Mfma<T>::mma(w, dxv[s], aQ);
          }
        }
      } else {
#pragma unroll
        for (int s = 0; s < KS; s++) {
          const T w = c < 2 * l + 1 ? ga[CH(s)] : (T) 0;
          aP = Mfma<T>::mma(w, x[cur][s], aP);
          aQ = Mfma<T>::mma(w, dx[cur][s], aQ);
        }
      }
      if (colok) {
#pragma unroll
        for (int v = 0; v < 4; v++) {
          if (mrow[v] < 2 * l + 1) {
            const int lm = l * l + mrow[v];
            const T *G = Gw + c * 2 * NLM + lm;
            px += (double) (Yw[c * NLM + lm] * aQ[v]);
            p1 += (double) (G[0] * aP[v]);
            p2 += (double) (G[NLM] * aP[v]);
          }
        }
      }
    }
    // sum over the four lane groups (the rows m of a bond are spread over them)
    px += __shfl_xor(px, 16, 64); p1 += __shfl_xor(p1, 16, 64); p2 += __shfl_xor(p2, 16, 64);
    px += __shfl_xor(px, 32, 64); p1 += __shfl_xor(p1, 32, 64); p2 += __shfl_xor(p2, 32, 64);
    if (lane < nb) {
      const double dEdr = px / brc, t1 = p1 / br, t2 = p2 / br;
      const double fv[3] = {dEdr * u0 + t1 * e1[0] + t2 * e2[0], dEdr * u1 + t1 * e1[1] + t2 * e2[1], dEdr * u2 + t1 * e1[2] + t2 * e2[2]};
      for (int d = 0; d < 3; d++) {
        fi[d] += fv[d];
        if (a.fedge) a.fedge[3 * (eb + lane) + d] = (a.ordered_add ? a.fedge[3 * (eb + lane) + d] : 0.0) + fv[d];
        else atomicAdd(&a.f[3 * (long long) jj + d], -fv[d]);
      }
      const double ddx = -u0 * br, ddy = -u1 * br, ddz = -u2 * br;
      vir[0] += ddx * fv[0]; vir[1] += ddy * fv[1]; vir[2] += ddz * fv[2];
      vir[3] += ddx * fv[1]; vir[4] += ddx * fv[2]; vir[5] += ddy * fv[2];
      if (a.vatom) {    // the neighbour's half (add_vatom, libgrace/include/grace/fused_cpu.h:1075-1087); the atom's own below
        double *vj = a.vatom + 9 * (long long) jj;
        atomicAdd(vj, 0.5 * ddx * fv[0]); atomicAdd(vj + 1, 0.5 * ddy * fv[1]); atomicAdd(vj + 2, 0.5 * ddz * fv[2]);
        atomicAdd(vj + 3, 0.5 * ddx * fv[1]); atomicAdd(vj + 4, 0.5 * ddx * fv[2]); atomicAdd(vj + 5, 0.5 * ddy * fv[2]);
        // the components below the diagonal (the centroid form, kk/grace_1l_kk_impl.h:1344-1349), for both atoms of the bond
        double *vi = a.vatom + 9 * (long long) i;
        const double yx = 0.5 * ddy * fv[0], zx = 0.5 * ddz * fv[0], zy = 0.5 * ddz * fv[1];
        atomicAdd(vj + 6, yx); atomicAdd(vj + 7, zx); atomicAdd(vj + 8, zy);
        atomicAdd(vi + 6, yx); atomicAdd(vi + 7, zx); atomicAdd(vi + 8, zy);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  double vsum[9] = {fi[0], fi[1], fi[2], vir[0], vir[1], vir[2], vir[3], vir[4], vir[5]};
#pragma unroll
  for (int k = 0; k < 9; k++)
    for (int o = 32; o > 0; o >>= 1) vsum[k] += __shfl_xor(vsum[k], o, 64);
  if (lane == 0)
    for (int k = 0; k < 9; k++) red[wave][k] = vsum[k];
  __syncthreads();
  if (t < 9) {
    const double s = red[0][t] + red[1][t] + red[2][t] + red[3][t];
    if (a.fcen) a.fcen[9 * (long long) i + t] = (a.ordered_add ? a.fcen[9 * (long long) i + t] : 0.0) + s;
    else if (e1 > e0) {
      if (t < 3) atomicAdd(&a.f[3 * (long long) i + t], s);
      else {
        atomicAdd(&a.virial[(a.sid ? 8 * a.sid[i] : 0) + t - 3], s);
        if (a.vatom) atomicAdd(&a.vatom[9 * (long long) i + t - 3], 0.5 * s);
      }
    }
  }
}
#undef CH

// ---------------------------------------------------------------------------------------------------------------
// ordered (atomic-free) sums of the forces, the virial and the energy: same bits on every run
// ---------------------------------------------------------------------------------------------------------------
// bonds per neighbour atom: count[ej[e]] += 1 (integer atomics: the result does not depend on their order)
static __global__ void k_tlist_count(const long long *n_edges, const int *ej, int *count)
{
  const long long e = blockIdx.x * (long long) blockDim.x + threadIdx.x;
  if (e < *n_edges) atomicAdd(&count[ej[e]], 1);
}
// bond numbers by neighbour atom, in arrival order (k_tlist_sort orders every row)
static __global__ void k_tlist_fill(const long long *n_edges, const int *ej, const long long *toff, int *cursor, int *raw)
{
  const long long e = blockIdx.x * (long long) blockDim.x + threadIdx.x;
  if (e < *n_edges) {
    const int j = ej[e];
    raw[toff[j] + atomicAdd(&cursor[j], 1)] = (int) e;
  }
}
// One wave per atom k (owned atoms, then ghosts): its row of bond numbers in ascending order, by counting for every
// entry the entries below it (a row is a few hundred entries at most).
static __global__ void k_tlist_sort(int n_nodes, const long long *toff, const int *raw, int *sorted)
{
  const int lane = threadIdx.x & 63;
  const int k = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (k >= n_nodes) return;
  const long long t0 = toff[k];
  const int *row = raw + t0;
  const int len = (int) (toff[k + 1] - t0);
  for (int p = lane; p < len; p += 64) {
    const int mine = row[p];
    int rank = 0;
    for (int q = 0; q < len; q++) rank += row[q] < mine;
    sorted[t0 + rank] = mine;
  }
}
// One wave per atom k: f[k] = fcen[k] (owned atoms) - sum of fedge over the bonds that have k as their neighbour, the
// sorted row taken by the lanes in turn and the lane sums added in a fixed tree.
static __global__ void k_ordered_forces(int n_nodes, int n, const long long *toff, const int *sorted, const double *fedge, const double *fcen, double *f)
{
  const int lane = threadIdx.x & 63;
  const int k = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (k >= n_nodes) return;
  const long long t0 = toff[k];
  const int len = (int) (toff[k + 1] - t0);
  double s[3] = {0, 0, 0};
  for (int p = lane; p < len; p += 64) {
    const double *fe = fedge + 3 * (long long) sorted[t0 + p];
    s[0] += fe[0]; s[1] += fe[1]; s[2] += fe[2];
  }
#pragma unroll
  for (int d = 0; d < 3; d++)
    for (int o = 32; o > 0; o >>= 1) s[d] += __shfl_xor(s[d], o, 64);
  if (lane < 3) f[3 * (long long) k + lane] = (k < n ? fcen[9 * (long long) k + lane] : 0.0) - s[lane];
}
// One block per structure: record (energy, virial[6]) = sums of eatom[i] and fcen[i][3 .. 9] over its atoms, which are
// the range [lower_bound(s), lower_bound(s + 1)) of the non-decreasing sid (null: one structure, all atoms); every
// thread adds its atoms in ascending order, the thread sums are added in a fixed tree.
static __global__ __launch_bounds__(256) void k_ordered_records(int n, const int *sid, const double *eatom, const double *fcen, int with_virial, double *rec)
{
  __shared__ double part[256][7];
  const int s = blockIdx.x, t = threadIdx.x;
  int lo = 0, hi = n;
  if (sid) {
    auto lower = [&](int key) {
      int a = 0, b = n;
      while (a < b) {
        const int m = (a + b) >> 1;
        if (sid[m] < key) a = m + 1;
        else b = m;
      }
      return a;
    };
    lo = lower(s);
    hi = lower(s + 1);
  }
  double v[7] = {0, 0, 0, 0, 0, 0, 0};
  for (int i = lo + t; i < hi; i += 256) {
    v[0] += eatom[i];
    if (with_virial)
      for (int k = 0; k < 6; k++) v[1 + k] += fcen[9 * (long long) i + 3 + k];
  }
  for (int k = 0; k < 7; k++) part[t][k] = v[k];
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if (t < o)
      for (int k = 0; k < 7; k++) part[t][k] += part[t + o][k];
    __syncthreads();
  }
  if (t < 7) rec[8 * (long long) s + t] = part[0][t];
}

}    // namespace grhip
