// HIP kernels of the GRACE-3L layers for gfx950 that the GRACE-1L / 2L kernels do not already provide.
//
//   k_edge_center      element of the central atom of every edge (input of the species form of the radial kernel)
//   k_message          M[atom][li][n] = I[atom][li][n] + chem_l0_mask[li] zproj[mu_atom][n]: what a neighbour contributes to
//                      the equivariant SPBF (bond_vectors, libgrace/src/fused_3l.cpp:1049-1083)
//   k_lincomb          out[atom][f][n] = sum_t v_t in[atom][p_t][n]: the sparse Clebsch-Gordan matrix cg_W of the equivariant
//                      SPBF and its transpose (fused_3l.cpp:1266-1272, :1443-1449)
//   k_scale_rows       out[atom][f][n] (+)= s[f] in[atom][f][n]: the left input of an FCRight2Left layer (fused_3l.cpp:955-969)
//   k_couple_*_lds     cp_l couple and its reverse with the atom's projections in LDS (fused_3l_cpu.h:223-276)
//   k_eqnorm           EquivariantRMSNorm and its reverse (libgrace/include/grace/fused_3l_cpu.h:335-414)
//   k_energy_3l        InvariantLayerRMSNorm of the three densities, their sum, fp64 readout MLP and the reverse of all of it
//                      (fused_3l_cpu.h:416-444, fused_3l.cpp:1300-1360)
#pragma once

#include "kernels_2l.hpp"

namespace grhip {

__device__ inline double readlane_f64(double v, int k)
{
  const int lo = __builtin_amdgcn_readlane(__double2loint(v), k), hi = __builtin_amdgcn_readlane(__double2hiint(v), k);
  return __hiloint2double(hi, lo);
}

// grid: atoms; block: 64
static __global__ void k_edge_center(const long long *eoff, const int *mu, int *emi)
{
  const int i = blockIdx.x;
  const int m = mu[i];
  for (long long e = eoff[i] + threadIdx.x; e < eoff[i + 1]; e += blockDim.x) emi[e] = m;
}

// grid: ceil(natoms * nf * C / 256)
template<class T>
__global__ void k_message(const T *I, const int *mu, const T *zproj, const T *mask, T *M, int natoms, int nf, int C)
{
  const long long q = blockIdx.x * (long long) blockDim.x + threadIdx.x;
  if (q >= (long long) natoms * nf * C) return;
  const int n = (int) (q % C), f = (int) ((q / C) % nf), at = (int) (q / ((long long) C * nf));
  M[q] = I[q] + mask[f] * zproj[(long long) mu[at] * C + n];
}

// Sparse matrix times the per-atom tensor: out[atom][f][n] = sum_{t in row f} val[t] in[atom][idx[t]][n].  CSR by output
// row: terms [off[f], off[f + 1]), row[t] = f.  A wave spans the channels of AT = 64 / C atoms and takes `rows`
// consecutive output rows (lincomb_rows: about 64 terms per wave); it reads its terms 64 at a time, one per lane, and
// walks them with lane reads, the source rows of 8 terms requested before the first is used.
// grid: 8 ceil(ceil(atoms / AT) / 8) ngrp blocks, ngrp = ceil(nout / (4 rows)), in the order of pair_block: the row groups
// of one atom run on one XCD shortly after each other, so a source row that several groups read comes from HBM once.
// block 256.
inline int lincomb_rows(int nterms, int nout)
{
  const int per = nout > 0 ? (nterms + nout - 1) / nout : 1;
  int rows = 8;
  while (rows < 64 && rows * 2 * per <= 64) rows *= 2;
  return rows;
}
template<class T>
__global__ __launch_bounds__(256) void k_lincomb(const int *__restrict__ off, const int *__restrict__ idx, const int *__restrict__ row,
                                                 const double *__restrict__ val, const T *__restrict__ in, T *__restrict__ out, int nin, int nout,
                                                 int C, int natoms, int rows, int ngrp)
{
  const int AT = 64 / C, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int ab, grp;
  if (!pair_block(ngrp, (natoms + AT - 1) / AT, ab, grp)) return;
  const int a0 = ab * AT, sub = lane / C, n = lane % C;
  const bool live = a0 + sub < natoms;
  const int r0 = (grp * 4 + wave) * rows, r1 = r0 + rows < nout ? r0 + rows : nout;
  if (r0 >= nout) return;
  const T *src = in + (long long) (a0 + (live ? sub : 0)) * nin * C + n;
  T *dst = out + (long long) (a0 + (live ? sub : 0)) * nout * C + n;
  const int t0 = off[r0], t1 = off[r1];
  for (int f = r0; f < r1; f++)                        // rows without terms
    if (live && off[f] == off[f + 1]) dst[(long long) f * C] = (T) 0;
  int cur = -1;
  T acc = (T) 0;
  for (int base = t0; base < t1; base += 64) {
    const int q = base + lane < t1 ? base + lane : t1 - 1;
    const int iv = idx[q], rv = row[q];
    const double cv = val[q];
    const int cnt = t1 - base < 64 ? t1 - base : 64;
    for (int k0 = 0; k0 < cnt; k0 += 8) {
      T x[8];
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const int k = k0 + u < cnt ? k0 + u : cnt - 1;
        x[u] = src[(long long) __builtin_amdgcn_readlane(iv, k) * C];
      }
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const int k = k0 + u;
        if (k < cnt) {
          const int f = __builtin_amdgcn_readlane(rv, k);
          if (f != cur) {
            if (cur >= 0 && live) dst[(long long) cur * C] = acc;
            acc = (T) 0;
            cur = f;
          }
          acc += (T) readlane_f64(cv, k) * x[u];
        }
      }
    }
  }
  if (cur >= 0 && live) dst[(long long) cur * C] = acc;
}

// grid: ceil(natoms * nf * C / 256)
template<class T> __global__ void k_scale_rows(const T *in, const T *s, T *out, int natoms, int nf, int C, int accumulate)
{
  const long long q = blockIdx.x * (long long) blockDim.x + threadIdx.x;
  if (q >= (long long) natoms * nf * C) return;
  const int f = (int) ((q / C) % nf);
  const T v = s[f] * in[q];
  out[q] = accumulate ? out[q] + v : v;
}

// Term list of a cp_l couple sorted by output function: left, right, output function and coefficient of every term.
struct CoupleDev {
  const int *l, *r, *o;
  const double *c;
  const int *off;             // [nout + 1] terms of output o are [off[o], off[o + 1])
  int nout, nterms;
};

// cp_l couple with the projections staged in LDS: out[o][n] = sum_t c_t Lp[l_t][n] Rp[r_t][n]
// (couple_row_fwd, libgrace/include/grace/fused_3l_cpu.h:232-255).  A block works on AT = 64 / C atoms (a wave spans the
// channels of AT atoms); wave w takes the outputs [w nout / nw, (w + 1) nout / nw).  The terms of a wave are read 64 at
// a time, one per lane, and then walked with lane reads, so that no memory access sits between two terms but the LDS
// reads of the operands.  grid: ceil(atoms / AT); dynamic LDS: AT (nfl + nfr) C values.
template<class T>
__global__ __launch_bounds__(1024) void k_couple_fwd_lds(CoupleDev P, const T *__restrict__ L, const T *__restrict__ R, T *__restrict__ out, int C,
                                                         int nfl, int nfr, int natoms)
{
  extern __shared__ __align__(16) unsigned char smem_raw[];
  const int AT = 64 / C, t = threadIdx.x, lane = t & 63, wave = t >> 6, nw = blockDim.x >> 6;
  T *Ls = reinterpret_cast<T *>(smem_raw), *Rs = Ls + AT * nfl * C;
  const int a0 = blockIdx.x * AT, na = natoms - a0 < AT ? natoms - a0 : AT;
  {
    const T *La = L + (long long) a0 * nfl * C, *Ra = R + (long long) a0 * nfr * C;
    for (int q = t; q < na * nfl * C; q += blockDim.x) Ls[q] = La[q];
    for (int q = t; q < na * nfr * C; q += blockDim.x) Rs[q] = Ra[q];
  }
  __syncthreads();
  const int sub = lane / C, n = lane % C;
  const bool live = sub < na;
  const T *Lm = Ls + sub * nfl * C + n, *Rm = Rs + sub * nfr * C + n;
  T *om = out + (long long) (a0 + (live ? sub : 0)) * P.nout * C + n;
  const int o0 = (int) ((long long) wave * P.nout / nw), o1 = (int) ((long long) (wave + 1) * P.nout / nw);
  const int t0 = P.off[o0], t1 = P.off[o1];
  for (int o = o0; o < o1; o++)                       // outputs without terms
    if (live && P.off[o] == P.off[o + 1]) om[(long long) o * C] = (T) 0;
  int cur = -1;
  T acc = (T) 0;
  for (int base = t0; base < t1; base += 64) {
    const int idx = base + lane < t1 ? base + lane : t1 - 1;
    const int lv = P.l[idx], rv = P.r[idx], ov = P.o[idx];
    const double cv = P.c[idx];
    const int cnt = t1 - base < 64 ? t1 - base : 64;
    for (int k = 0; k < cnt; k++) {
      const int o = __builtin_amdgcn_readlane(ov, k);
      if (o != cur) {
        if (cur >= 0 && live) om[(long long) cur * C] = acc;
        acc = (T) 0;
        cur = o;
      }
      const int l = __builtin_amdgcn_readlane(lv, k), r = __builtin_amdgcn_readlane(rv, k);
      acc += (T) readlane_f64(cv, k) * Lm[l * C] * Rm[r * C];
    }
  }
  if (cur >= 0 && live) om[(long long) cur * C] = acc;
}

// Its reverse in scatter form: for every term gLp[l][n] += c g[o][n] Rp[r][n], gRp[r][n] += c g[o][n] Lp[l][n]
// (couple_row_bwd, fused_3l_cpu.h:258-276), the two adjoints accumulated in LDS with LDS atomics (the waves of a block
// share them) and added to gL / gR at the end; g is read once, row by row.  The LDS accumulators are fp64 for both
// precisions (ds_add_f32 runs several times slower than ds_add_f64 on this hardware).  Same grid; dynamic LDS:
// AT (nfl + nfr) C (sizeof(T) + 8) bytes.
template<class T>
__global__ __launch_bounds__(1024) void k_couple_bwd_lds(CoupleDev P, const T *__restrict__ L, const T *__restrict__ R, const T *__restrict__ g,
                                                         T *__restrict__ gL, T *__restrict__ gR, int C, int nfl, int nfr, int natoms)
{
  extern __shared__ __align__(16) unsigned char smem_raw[];
  const int AT = 64 / C, t = threadIdx.x, lane = t & 63, wave = t >> 6, nw = blockDim.x >> 6;
  double *gLs = reinterpret_cast<double *>(smem_raw), *gRs = gLs + AT * nfl * C;
  T *Ls = reinterpret_cast<T *>(gRs + AT * nfr * C), *Rs = Ls + AT * nfl * C;
  const int a0 = blockIdx.x * AT, na = natoms - a0 < AT ? natoms - a0 : AT;
  {
    const T *La = L + (long long) a0 * nfl * C, *Ra = R + (long long) a0 * nfr * C;
    for (int q = t; q < AT * nfl * C; q += blockDim.x) {
      Ls[q] = q < na * nfl * C ? La[q] : (T) 0;
      gLs[q] = 0.0;
    }
    for (int q = t; q < AT * nfr * C; q += blockDim.x) {
      Rs[q] = q < na * nfr * C ? Ra[q] : (T) 0;
      gRs[q] = 0.0;
    }
  }
  __syncthreads();
  const int sub = lane / C, n = lane % C;
  const bool live = sub < na;
  const int lo = sub * nfl * C + n, ro = sub * nfr * C + n;
  const T *gm = g + (long long) (a0 + (live ? sub : 0)) * P.nout * C + n;
  const int o0 = (int) ((long long) wave * P.nout / nw), o1 = (int) ((long long) (wave + 1) * P.nout / nw);
  const int t0 = P.off[o0], t1 = P.off[o1];
  int cur = -1;
  T gcur = (T) 0, gnext = (T) 0;
  int onext = -1;
  for (int base = t0; base < t1; base += 64) {
    const int idx = base + lane < t1 ? base + lane : t1 - 1;
    const int lv = P.l[idx], rv = P.r[idx], ov = P.o[idx];
    const double cv = P.c[idx];
    const int cnt = t1 - base < 64 ? t1 - base : 64;
    for (int k = 0; k < cnt; k++) {
      const int o = __builtin_amdgcn_readlane(ov, k);
      if (o != cur) {
        gcur = o == onext ? gnext : (live ? gm[(long long) o * C] : (T) 0);
        onext = o + 1 < o1 ? o + 1 : o;
        gnext = live ? gm[(long long) onext * C] : (T) 0;    // the row of the next output, in flight during this one
        cur = o;
      }
      const int l = __builtin_amdgcn_readlane(lv, k), r = __builtin_amdgcn_readlane(rv, k);
      const T cg = (T) readlane_f64(cv, k) * gcur;
      atomicAdd(&gLs[lo + l * C], (double) (cg * Rs[ro + r * C]));
      atomicAdd(&gRs[ro + r * C], (double) (cg * Ls[lo + l * C]));
    }
  }
  __syncthreads();
  {
    T *ga = gL + (long long) a0 * nfl * C, *gb = gR + (long long) a0 * nfr * C;
    for (int q = t; q < na * nfl * C; q += blockDim.x) ga[q] += (T) gLs[q];
    for (int q = t; q < na * nfr * C; q += blockDim.x) gb[q] += (T) gRs[q];
  }
}

struct EqNormDev {
  const double *dw, *mask, *aff;    // [M], [M], [groups][C] (C = padded channel width, padding columns zero)
  const int *grp;                   // [M]
  int M, C, Creal, center;
  double eps;
};

__device__ inline double block_sum(double v, double *red)
{
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  double s = 0.0;
  for (int w = 0; w < nw; w++) s += red[w];
  return s;
}

// xc = x - l0_mask mean_n x;  r = 1 / sqrt(mean_n sum_f dw[f] xc^2 + eps);  y = xc r aff[e(f)][n].
// One block of 256 threads per atom; a wave per function row for the means.  With gy != nullptr also the reverse:
// gx[f][n] = r g - r^3 / C (sum g xc) dw[f] xc, minus its channel mean on the centred rows, g = gy aff.
template<class T>
__global__ void k_eqnorm(EqNormDev E, const T *X, T *Y, const T *gY, T *gX, int accumulate)
{
  extern __shared__ __align__(16) unsigned char smem_raw[];
  double *mean = reinterpret_cast<double *>(smem_raw);    // [M]
  __shared__ double red[16];
  const int at = blockIdx.x, t = threadIdx.x, lane = t & 63, wave = t >> 6, nw = blockDim.x >> 6;
  const int M = E.M, C = E.C, Cr = E.Creal;
  const T *x = X + (long long) at * M * C;
  for (int f = wave; f < M; f += nw) {
    double m = 0.0;
    if (E.center && E.mask[f] != 0.0) {
      for (int n = lane; n < Cr; n += 64) m += (double) x[(long long) f * C + n];
      for (int o = 32; o > 0; o >>= 1) m += __shfl_xor(m, o, 64);
      m = m / Cr * E.mask[f];
    }
    if (lane == 0) mean[f] = m;
  }
  __syncthreads();
  double s = 0.0;
  for (int q = t; q < M * C; q += blockDim.x) {
    const int f = q / C, n = q % C;
    if (n < Cr) {
      const double c = (double) x[q] - mean[f];
      s += E.dw[f] * c * c;
    }
  }
  const double S = block_sum(s, red);
  const double r = 1.0 / sqrt(S / Cr + E.eps);
  if (!gY) {
    T *y = Y + (long long) at * M * C;
    for (int q = t; q < M * C; q += blockDim.x) {
      const int f = q / C, n = q % C;
      y[q] = n < Cr ? (T) (((double) x[q] - mean[f]) * r * E.aff[(long long) E.grp[f] * C + n]) : (T) 0;
    }
    return;
  }
  const T *gy = gY + (long long) at * M * C;
  double gx = 0.0;
  for (int q = t; q < M * C; q += blockDim.x) {
    const int f = q / C, n = q % C;
    if (n < Cr) gx += (double) gy[q] * E.aff[(long long) E.grp[f] * C + n] * ((double) x[q] - mean[f]);
  }
  const double k3 = r * r * r * block_sum(gx, red) / Cr;
  T *go = gX + (long long) at * M * C;
  for (int f = wave; f < M; f += nw) {
    const double kf = k3 * E.dw[f];
    const bool cen = E.center && E.mask[f] != 0.0;
    double vsum = 0.0;
    for (int n = lane; n < Cr; n += 64) {
      const long long q = (long long) f * C + n;
      vsum += r * (double) gy[q] * E.aff[(long long) E.grp[f] * C + n] - kf * ((double) x[q] - mean[f]);
    }
    for (int o = 32; o > 0; o >>= 1) vsum += __shfl_xor(vsum, o, 64);
    const double mg = cen ? vsum / Cr * E.mask[f] : 0.0;
    for (int n = lane; n < Cr; n += 64) {
      const long long q = (long long) f * C + n;
      const double v = r * (double) gy[q] * E.aff[(long long) E.grp[f] * C + n] - kf * ((double) x[q] - mean[f]) - mg;
      go[q] = accumulate ? go[q] + (T) v : (T) v;
    }
  }
}

struct Energy3Dev {
  const double *W0, *W1;      // [nin][nh], [nh]
  double norm0, norm1, out_scale, eps;
  int nin, nh, act, nrho;
  const double *shift;        // [nel]
  const double *scale[3];     // RMSNorm scales of rho1, rho2, rho3: [nrho - type]
  int type[3];                // 1: only_nonlin (channel 0 passes)
};

// rho_k -> y_k = RMSNorm_k(rho_k), h = y_1 + y_2 + y_3, E_i = (MLP(h[1:]) + h[0]) out_scale + shift[mu_i]; with want_grad
// the adjoints grho_k of the raw densities.  One wave per atom, fp64.  Dynamic LDS: (nrho + 2 nh) doubles.
static __global__ void k_energy_3l(Energy3Dev M, const int *mu, const double *rho1, const double *rho2, const double *rho3, double *g1, double *g2,
                                   double *g3, double *eatom, double *energy, int want_grad, const int *sid)
{
  extern __shared__ __align__(16) unsigned char smem_raw[];
  double *h = reinterpret_cast<double *>(smem_raw), *pre = h + M.nrho, *gs = pre + M.nh;
  const int at = blockIdx.x, lane = threadIdx.x, nr = M.nrho;
  const double *rho[3] = {rho1 + (long long) at * nr, rho2 + (long long) at * nr, rho3 + (long long) at * nr};
  double rinv[3];
  for (int k = 0; k < 3; k++) {
    const int n0 = M.type[k];
    double s = 0.0;
    for (int n = n0 + lane; n < nr; n += 64) s += rho[k][n] * rho[k][n];
    for (int o = 32; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
    rinv[k] = 1.0 / sqrt(s / (nr - n0) + M.eps);
  }
  for (int n = lane; n < nr; n += 64) {
    double v = 0.0;
    for (int k = 0; k < 3; k++) v += n < M.type[k] ? rho[k][n] : rho[k][n] * rinv[k] * M.scale[k][n - M.type[k]];
    h[n] = v;
  }
  __syncthreads();
  double e = 0.0;
  for (int j = lane; j < M.nh; j += 64) {
    double s = 0.0;
    for (int c = 0; c < M.nin; c++) s += h[c + 1] * M.W0[(long long) c * M.nh + j];
    s *= M.norm0;
    pre[j] = s;
    e += M.W1[j] * (M.act == 1 ? tanh(s) : s / (1.0 + exp(-s)));
  }
  for (int o = 32; o > 0; o >>= 1) e += __shfl_xor(e, o, 64);
  const double Ei = (e * M.norm1 + h[0]) * M.out_scale + M.shift[mu[at]];
  if (lane == 0) {
    if (eatom) eatom[at] = Ei;
    if (energy) atomicAdd(energy + (sid ? 8 * sid[at] : 0), Ei);    // null: ordered sums, the records are added from eatom afterwards
  }
  if (!want_grad) return;
  for (int j = lane; j < M.nh; j += 64) {
    const double s = pre[j];
    double da;
    if (M.act == 1) {
      const double tt = tanh(s);
      da = 1.0 - tt * tt;
    } else {
      const double sg = 1.0 / (1.0 + exp(-s));
      da = sg * (1.0 + s * (1.0 - sg));
    }
    gs[j] = M.out_scale * M.norm1 * M.W1[j] * da * M.norm0;
  }
  __syncthreads();
  // dE/dh: channel 0 the linear skip, channels 1.. through the MLP
  double gh_mine[4];    // nrho <= 256: up to 4 channels per lane
  for (int q = 0; q < 4; q++) {
    const int n = lane + 64 * q;
    double v = 0.0;
    if (n == 0) v = M.out_scale;
    else if (n < nr) {
      for (int j = 0; j < M.nh; j++) v += M.W0[(long long) (n - 1) * M.nh + j] * gs[j];
    }
    gh_mine[q] = v;
  }
  double *gout[3] = {g1 + (long long) at * nr, g2 + (long long) at * nr, g3 + (long long) at * nr};
  for (int k = 0; k < 3; k++) {
    const int n0 = M.type[k], nn = nr - n0;
    double gx = 0.0;
    for (int q = 0; q < 4; q++) {
      const int n = lane + 64 * q;
      if (n >= n0 && n < nr) gx += gh_mine[q] * M.scale[k][n - n0] * rho[k][n];
    }
    for (int o = 32; o > 0; o >>= 1) gx += __shfl_xor(gx, o, 64);
    const double r = rinv[k], kk = r * r * r * gx / nn;
    for (int q = 0; q < 4; q++) {
      const int n = lane + 64 * q;
      if (n >= nr) continue;
      gout[k][n] = n < n0 ? gh_mine[q] : r * gh_mine[q] * M.scale[k][n - n0] - kk * rho[k][n];
    }
  }
}

}    // namespace grhip
