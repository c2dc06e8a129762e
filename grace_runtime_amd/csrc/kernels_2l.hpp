// HIP kernels of the second message-passing layer of GRACE-2L for gfx950.
//
//   k_sh_edges     Y_lm and the gradient of its polynomial extension for every edge, once per pass, written coalesced
//   k_fill_slot    the species weights zB0[mu_j] as one more "message function" of every atom
//   k_pair_fwd     P[slot][lm][n] = sum_b Y_lm(b) R1_l(b)[n] M_jb[slot][n]: the neighbour gather of the messages
//                  (slots 0 .. nI-1: the equivariant message I_j; slot nI: zB0, which gives B0)
//                  (atom_yi / atom_scatter, libgrace/include/grace/fused_cpu.h:947-1025)
//   k_pair_bwd_mfma, k_pair_bwd[_async]  its reverse: per-bond force of layer 2, dE/dI_j added to the neighbour's row
//                  (bond_yi_bwd_g, bond_yi_commit, bond_scatter_bwd_t, bond_force: fused_cpu.h:836-942,1027-1050); the first
//                  forms the sums over m on the matrix cores, the others on the vector unit
//   k_energy_2l    readout with the two RMSNorms, fp64 (libgrace/src/fused_2l.cpp:548-615)
//
// The vector gather kernels run one block per atom with one thread per (slot, channel): a thread keeps its 2l+1 .. nlm
// accumulators (or adjoints) in registers and walks the atom's bonds; everything that is the same for the whole block
// (neighbour index, Y, G of the bond) is read through uniform addresses.
#pragma once

#include "kernels_1l.hpp"

namespace grhip {

// rows (atom, listed function) of a per-atom tensor [atom][nfun][KP] set to zero; total = atoms x listed functions x KP
template<class T> __global__ void k_clear_functions(T *G, int nfun, int KP, const int *list, int nlist, long long total)
{
  const long long i = (long long) blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const int n = (int) (i % KP), q = (int) ((i / KP) % nlist);
  const long long a = i / ((long long) KP * nlist);
  G[(a * nfun + list[q]) * KP + n] = (T) 0;
}


// One thread per edge: YG[e] = (Y[nlm], D1[nlm], D2[nlm]) (row width W = 3 nlm), or Y[nlm] alone (W = nlm, no
// gradients), in rows of `stride` >= W values, the rest of a row zero.  D1 = G . e1, D2 = G . e2 are the components of the gradient G of the polynomial extension of Y along the
// tangent vectors of the bond (tangent_basis): the bond force only uses the part of sum_lm gY_lm G_lm normal to the bond,
// g - (g . rhat) rhat = (g . e1) e1 + (g . e2) e2, so two components per harmonic carry all of it.
// The lanes write their rows into an LDS tile, the block copies the tile out in consecutive addresses.
// block: 64 threads; dynamic LDS: 64 * (W + 1) values.
template<class T> __global__ void k_sh_edges(ShCoef sh, const double *rh, const long long *n_edges, int nlm, int grad, T *YG, int stride)
{
  extern __shared__ __align__(16) unsigned char smem_raw[];
  T *tile = reinterpret_cast<T *>(smem_raw);
  const int W = grad ? 3 * nlm : nlm, t = threadIdx.x;
  const long long ne = *n_edges, e0 = blockIdx.x * 64ll, e = e0 + t;
  if (e0 >= ne) return;
  if (e < ne) {
    const double *u = rh + 3 * e;
    T *row = tile + t * (W + 1);
    if (grad) {
      double e1[3], e2[3];
      tangent_basis(u, e1, e2);
      sh_eval<true, T>(sh, u[0], u[1], u[2], row, row + nlm, e1, e2, row + 2 * nlm);
    } else {
      sh_eval<false, T>(sh, u[0], u[1], u[2], row, nullptr);
    }
  }
  __syncthreads();
  const int rows = (int) (ne - e0 < 64 ? ne - e0 : 64);
  T *out = YG + e0 * stride;
  for (int q = t; q < rows * stride; q += 64) {
    const int r = q / stride, col = q % stride;
    out[q] = col < W ? tile[r * (W + 1) + col] : (T) 0;
  }
}

// M[atom][slot][n] = z[mu_atom][n]
template<class T> __global__ void k_fill_slot(const int *mu, const T *z, T *M, int natoms, int nslot, int slot, int C)
{
  const long long q = blockIdx.x * (long long) blockDim.x + threadIdx.x;
  if (q >= (long long) natoms * C) return;
  const int at = (int) (q / C), n = (int) (q % C);
  M[((long long) at * nslot + slot) * C + n] = z[mu[at] * C + n];
}

// dst[q] = src[q] in another precision (the fp32 engine: the scalar reduces write and read fp64 rows, the GEMMs fp32 rows)
template<class S, class D> __global__ void k_convert(const S *src, D *dst, long long count)
{
  const long long q = blockIdx.x * (long long) blockDim.x + threadIdx.x;
  if (q < count) dst[q] = (D) src[q];
}

constexpr int kPairChunk = 8;    // bonds staged in LDS at a time by the pair kernel that stages through registers
constexpr size_t kPairLdsMax = 158 * 1024;    // dynamic LDS a pair kernel may ask for

// Block -> (atom, slot group).  ngrp == 0: a (atoms, groups) grid.  ngrp > 0: a 1-d grid of 8 ceil(atoms / 8) ngrp
// blocks laid out so that the groups of one atom are blocks b, b + 8, b + 16 ...: workgroups go to the 8 XCDs in turn,
// so those blocks run on ONE XCD shortly after each other and find the atom's radial rows and harmonics in its L2.
__device__ inline bool pair_block(int ngrp, int natoms, int &atom, int &grp)
{
  if (ngrp == 0) {
    atom = blockIdx.x;
    grp = blockIdx.y;
    return true;
  }
  const int b = blockIdx.x, q = b >> 3;
  grp = q % ngrp;
  atom = (q / ngrp) * 8 + (b & 7);
  return atom < natoms;
}

// Stages what a chunk of nb bonds (edges base .. base + nb) needs into LDS with all loads in flight at once: the
// neighbour rows M_j[slot][n] of this thread, the radial rows (contiguous in memory), and touches the harmonics of the
// chunk (the first yuse values of every row of ylen) so that the uniform (scalar) reads of the bond loop find them in
// the L2.
template<class T>
__device__ inline T pair_stage(const int *__restrict__ ej, const T *__restrict__ M, const T *__restrict__ R1, const T *__restrict__ dR1,
                               const T *__restrict__ Yu, int ylen, int yuse, long long base, int nb, int nslot, int C, int nrow, bool active, int slot,
                               int n, T *Msh, T *Rsh, T *dRsh, int NT)
{
  const int t = threadIdx.x;
  T mv[kPairChunk];
#pragma unroll
  for (int b = 0; b < kPairChunk; b++) {
    const int j = b < nb ? ej[base + b] : 0;
    mv[b] = (active && b < nb) ? M[((long long) j * nslot + slot) * C + n] : (T) 0;
  }
  const T *rs = R1 + base * nrow, *drs = dR1 ? dR1 + base * nrow : nullptr;
  for (int q = t; q < nb * nrow; q += blockDim.x) {
    Rsh[q] = rs[q];
    if (drs) dRsh[q] = drs[q];
  }
  T touch = (T) 0;
  const T *yu = Yu + base * ylen;
  const int per = (yuse + 7) / 8;    // 64-byte pieces of a row that the bond loop reads
  for (int q = t; q < nb * per; q += blockDim.x) touch += yu[(q / per) * ylen + (q % per) * 8];
#pragma unroll
  for (int b = 0; b < kPairChunk; b++) Msh[b * NT + t] = mv[b];
  return touch;
}

// sums of 4 values per lane over the wave with 7 exchanges: afterwards lanes 0, 1, 2, 3 hold the totals of
// v0, v2, v1, v3
__device__ inline double wave_sum4(double v0, double v1, double v2, double v3, int lane)
{
  const bool b0 = lane & 1, b1 = lane & 2;
  double a = b0 ? v2 : v0, b = b0 ? v3 : v1;
  const double sa = b0 ? v0 : v2, sb = b0 ? v1 : v3;
  a += __shfl_xor(sa, 1, 64);
  b += __shfl_xor(sb, 1, 64);
  double c = b1 ? b : a;
  const double sc = b1 ? a : b;
  c += __shfl_xor(sc, 2, 64);
#pragma unroll
  for (int o = 4; o < 64; o <<= 1) c += __shfl_xor(c, o, 64);
  return c;
}

// grid: (atoms, slot groups); block: spb * C threads rounded up to a wave, spb slots per block (a kernel argument);
// dynamic LDS: kPairChunk * (NT + 2 nl C) values.  Every block adds the force of its slots to the bond's two atoms.
// The atoms are a chunk of the structure: eoff, gP start at the chunk's first atom a0; ej, M, gM, f, sid, the harmonics
// and the radial rows are indexed by the atom's or the bond's number in the structure.
// gP: adjoint of P of the atom.
//   S_l = sum_m Y_lm gP[lm],  T_l,k = sum_m D_k,lm gP[lm], k = 1, 2 (tangential gradients)   (per thread: slot, n)
//   dE/dI_j[slot][n] += sum_l R1_l S_l                                        (slots < nI)
//   dE/dx = sum_{slot,n,l} S_l dR1_l M_j,   g_k = sum_{slot,n,l} T_l,k R1_l M_j
//   fv = dE/dx / rc rhat + (g_1 e1 + g_2 e2) / r  (= the reference's dE/dx / rc rhat + (g - (g . rhat) rhat) / r with
//   g the Cartesian sum);  f_i += fv, f_j -= fv, virial += (-r rhat) (x) fv
// ORD (ordered sums): no floating-point atomics.  The message adjoint of bond e goes to ord.gMe[e - ord.e_base][slot][n],
// the force that the block's slot group gives the bond to ord.fedge[e][group][3], the sums over the atom's bonds to
// ord.fcen[a0 + i][group][9] (ord.ngrp groups: with one group these are the engine's per-bond and per-atom stores, with
// several k_ordered_combine adds the groups in turn); the sums over the waves of a block are added in the order of the waves.
template<class T> struct PairOrdered {
  T *gMe;
  double *fedge, *fcen;
  long long e_base;
  int ngrp;
};
template<class T, int NLM, bool ORD = false>
__global__ void k_pair_bwd(const long long *__restrict__ eoff, const int *__restrict__ ej, const T *__restrict__ YG,
                           const T *__restrict__ R1, const T *__restrict__ dR1, const T *__restrict__ M, const T *__restrict__ gP,
                           const double *__restrict__ rh, const double *__restrict__ rlen, const double *__restrict__ rcut,
                           T *__restrict__ gM, double *__restrict__ f, double *__restrict__ virial, int nslot, int nI, int C, int nl,
                           int noutp, T *__restrict__ sink, int one, const int *__restrict__ sid, int spb, int ngrp, int natoms, int a0,
                           double *__restrict__ vatom, int ystr, PairOrdered<T> ord)
{
  extern __shared__ __align__(16) unsigned char smem_raw[];
  __shared__ double bsum[kPairChunk][4];
  __shared__ double bwave[ORD ? kPairChunk : 1][ORD ? 16 : 1][4];    // ORD: the sums of every wave (at most 16 waves)
  int i, grp;
  if (!pair_block(ngrp, natoms, i, grp)) return;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6, NT = blockDim.x;
  T *Msh = reinterpret_cast<T *>(smem_raw), *Rsh = Msh + kPairChunk * NT, *dRsh = Rsh + kPairChunk * noutp;
  const int slot_raw = grp * spb + t / C;
  const bool active = t < spb * C && slot_raw < nslot;
  const int slot = active ? slot_raw : 0, n = t % C;
  const int nlm = nl * nl;
  const long long e0 = eoff[i], e1 = eoff[i + 1];
  T g[NLM];
  {
    const T *gp = gP + ((long long) i * nslot + slot) * nlm * C + n;
#pragma unroll
    for (int q = 0; q < NLM; q++) g[q] = (active && q < nlm) ? gp[(long long) q * C] : (T) 0;
  }
  double fi[3] = {0, 0, 0}, vir[6] = {0, 0, 0, 0, 0, 0};
  T touch = (T) 0;
  for (long long base = e0; base < e1; base += kPairChunk) {
    const int nb = (int) (e1 - base < kPairChunk ? e1 - base : kPairChunk);
    __syncthreads();
    touch += pair_stage<T>(ej, M, R1, dR1, YG, ystr, nlm * 3, base, nb, nslot, C, noutp, active, slot, n, Msh, Rsh, dRsh, NT);
    if (t < kPairChunk * 4) bsum[t >> 2][t & 3] = 0.0;
    __syncthreads();
    for (int b = 0; b < nb; b++) {
      const long long e = base + b;
      const T m = Msh[b * NT + t];
      const T *r = Rsh + b * noutp + n, *dr = dRsh + b * noutp + n;
      const T *yg = YG + e * ystr;
      T sI = (T) 0, dE = (T) 0, t1 = (T) 0, t2 = (T) 0;
      // every l is the body of a loop that runs `one` (= 1, a kernel argument) times: its uniform loads then stay inside
      // it (all harmonics of a bond at once need more scalar registers than there are)
#pragma unroll
      for (int l = 0; l <= kKernMaxL; l++)
        if (l * l < NLM) for (int it = 0; it < one; it++) {
          T S = (T) 0, a1 = (T) 0, a2 = (T) 0;
#pragma unroll
          for (int mm = 0; mm < 2 * l + 1; mm++) {
            const T gv = g[l * l + mm];
            S += yg[l * l + mm] * gv; a1 += yg[nlm + l * l + mm] * gv; a2 += yg[2 * nlm + l * l + mm] * gv;
          }
          const T rl = r[l * C], drl = dr[l * C];
          sI += rl * S;
          dE += drl * S;
          t1 += rl * a1; t2 += rl * a2;
        }
      if (active && slot < nI) {
        if (ORD) ord.gMe[((e - ord.e_base) * nI + slot) * C + n] = sI;
        else atomicAdd(&gM[((long long) ej[e] * nI + slot) * C + n], sI);
      }
      const double c = wave_sum4((double) (dE * m), (double) (t1 * m), (double) (t2 * m), 0.0, lane);
      if (lane < 3) {    // lanes 0..2: dE/dx, g . e2, g . e1  (order v0, v2, v1, v3)
        if (ORD) bwave[b][wave][lane] = c;
        else atomicAdd(&bsum[b][lane], c);
      }
    }
    __syncthreads();
    if (ORD && t < nb)
      for (int k = 0; k < 3; k++) {
        double sw = 0.0;
        for (int w = 0; w < (NT >> 6); w++) sw += bwave[t][w][k];
        bsum[t][k] = sw;
      }
    if (t < nb) {
      const long long e = base + t;
      const double *u = rh + 3 * e;
      const double r = rlen[e], rc = rcut[e];
      const double dEdr = bsum[t][0] / rc, g1 = bsum[t][2] / r, g2 = bsum[t][1] / r;
      double e1[3], e2[3], fv[3];
      tangent_basis(u, e1, e2);
      for (int d = 0; d < 3; d++) fv[d] = dEdr * u[d] + g1 * e1[d] + g2 * e2[d];
      const int jj = ej[e];
      for (int d = 0; d < 3; d++) {
        fi[d] += fv[d];
        if (ORD) ord.fedge[3 * (e * ord.ngrp + grp) + d] = fv[d];
        else atomicAdd(&f[3 * (long long) jj + d], -fv[d]);
      }
      const double ddx = -u[0] * r, ddy = -u[1] * r, ddz = -u[2] * r;
      vir[0] += ddx * fv[0]; vir[1] += ddy * fv[1]; vir[2] += ddz * fv[2];
      vir[3] += ddx * fv[1]; vir[4] += ddx * fv[2]; vir[5] += ddy * fv[2];
      if (!ORD && vatom) {    // per-atom virial: the neighbour's half of this bond (fused_cpu.h:1075-1087 of the reference)
        double *vj = vatom + 9 * (long long) jj;
        atomicAdd(vj, 0.5 * ddx * fv[0]); atomicAdd(vj + 1, 0.5 * ddy * fv[1]); atomicAdd(vj + 2, 0.5 * ddz * fv[2]);
        atomicAdd(vj + 3, 0.5 * ddx * fv[1]); atomicAdd(vj + 4, 0.5 * ddx * fv[2]); atomicAdd(vj + 5, 0.5 * ddy * fv[2]);
        // the components below the diagonal (the centroid form, kk/grace_1l_kk_impl.h:1344-1349), for both atoms of the bond
        double *vi = vatom + 9 * (long long) (a0 + i);
        const double yx = 0.5 * ddy * fv[0], zx = 0.5 * ddz * fv[0], zy = 0.5 * ddz * fv[1];
        atomicAdd(vj + 6, yx); atomicAdd(vj + 7, zx); atomicAdd(vj + 8, zy);
        atomicAdd(vi + 6, yx); atomicAdd(vi + 7, zx); atomicAdd(vi + 8, zy);
      }
    }
  }
  // the finishing threads t < kPairChunk sit in wave 0
  if (wave == 0) {
    double vsum[9] = {fi[0], fi[1], fi[2], vir[0], vir[1], vir[2], vir[3], vir[4], vir[5]};
#pragma unroll
    for (int k = 0; k < 9; k++)
      for (int o = 32; o > 0; o >>= 1) vsum[k] += __shfl_xor(vsum[k], o, 64);
    if (ORD) {
      if (lane == 0)
        for (int k = 0; k < 9; k++) ord.fcen[9 * ((long long) (a0 + i) * ord.ngrp + grp) + k] = vsum[k];
    } else if (lane == 0 && e1 > e0) {
      for (int k = 0; k < 3; k++) atomicAdd(&f[3 * (long long) (a0 + i) + k], vsum[k]);
      for (int k = 0; k < 6; k++) atomicAdd(&virial[(sid ? 8 * sid[a0 + i] : 0) + k], vsum[3 + k]);
      if (vatom)
        for (int k = 0; k < 6; k++) atomicAdd(&vatom[9 * (long long) (a0 + i) + k], 0.5 * vsum[3 + k]);
    }
  }
  if (touch == (T) 1.2345e300) sink[0] = touch;    // keeps the touching loads alive
}

// Ordered sums with several slot groups per atom: fedge[e][3] (=, or += with add) the sum over the groups, in their order, of
// fpart[e][group][3] for the bonds [e_base, e_end), and fcen[i][9] likewise of cpart[i][group][9] for the atoms [a0, a0 + natoms).
static __global__ void k_ordered_combine(const double *__restrict__ fpart, const double *__restrict__ cpart, int ngrp, long long e_base,
                                         const long long *__restrict__ e_end_dev, long long e_count, int a0, int natoms, int add,
                                         double *__restrict__ fedge, double *__restrict__ fcen)
{
  const long long e_end = e_count >= 0 ? e_base + e_count : *e_end_dev;
  const long long ne3 = 3 * (e_end - e_base), t = blockIdx.x * (long long) blockDim.x + threadIdx.x;
  if (t < ne3) {
    const long long e = e_base + t / 3;
    const int d = (int) (t % 3);
    double s = add ? fedge[3 * e + d] : 0.0;
    for (int g = 0; g < ngrp; g++) s += fpart[3 * (e * ngrp + g) + d];
    fedge[3 * e + d] = s;
  } else if (t < ne3 + 9ll * natoms) {
    const long long q = t - ne3, i = a0 + q / 9;
    const int k = (int) (q % 9);
    double s = add ? fcen[9 * i + k] : 0.0;
    for (int g = 0; g < ngrp; g++) s += cpart[9 * (i * ngrp + g) + k];
    fcen[9 * i + k] = s;
  }
}

// Ordered sums: gM[j][slot][n] += sum of gMe[e - e_base][slot][n] over the bonds e in [e_base, e_end) that have j as their
// neighbour, in ascending order of e (sorted: the bonds by neighbour atom, each row ascending; ncol = nI C columns).
// One block per atom j; a thread owns columns, so no two threads add to one value.
template<class T>
__global__ void k_ordered_gm(const long long *__restrict__ toff, const int *__restrict__ sorted, const T *__restrict__ gMe, long long e_base,
                             const long long *__restrict__ e_end_dev, long long e_count, int ncol, T *__restrict__ gM)
{
  const int j = blockIdx.x;
  const long long t0 = toff[j], t1 = toff[j + 1];
  const long long e_end = e_count >= 0 ? e_base + e_count : *e_end_dev;
  for (int col = threadIdx.x; col < ncol; col += blockDim.x) {
    T s = (T) 0;
    for (long long p = t0; p < t1; p++) {
      const long long e = sorted[p];
      if (e >= e_base && e < e_end) s += gMe[(e - e_base) * ncol + col];
    }
    gM[(long long) j * ncol + col] += s;
  }
}

// ---- the pair kernels with asynchronous staging
// The chunk after the one being worked on is copied from global memory straight into a second LDS buffer while the
// waves compute (global_load_lds: no registers, no wait until the end of the chunk), so the memory latency of the
// neighbour rows no longer stands between two chunks.
constexpr int kAsyncChunkFwd = 4;    // bonds per chunk of the gather; two chunks are resident

__device__ inline void lds_load_word(const void *src, void *lds_wave_base)
{
  __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *) src, (void __attribute__((address_space(3))) *) lds_wave_base, 4, 0, 0);
}

// The waves of a block copy nbytes (a multiple of 16, both ends 16-byte aligned) from global memory to LDS: pieces of
// 1 kB are dealt to the waves, a lane moves 16 bytes; the data lands at dst in the order it has at src.
__device__ inline void block_copy_async(const void *src, void *dst, int nbytes, int wave, int nw, int lane)
{
  for (int p = wave; p * 1024 < nbytes; p += nw) {
    const int q = p * 64 + lane;
    if (q * 16 < nbytes)
      __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *) (reinterpret_cast<const char *>(src) + 16 * (size_t) q),
                                       (void __attribute__((address_space(3))) *) (reinterpret_cast<char *>(dst) + 1024 * (size_t) p), 16, 0, 0);
  }
}

__device__ inline void wait_async_loads() { __asm__ volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// The neighbour gather: spb slots per block, spb C threads rounded up to whole waves (a copy is the work
// of all 64 lanes of a wave).  dynamic LDS: 2 kAsyncChunkFwd (NT + noutp) values.
template<class T, int NLM>
__global__ void k_pair_fwd(const long long *__restrict__ eoff, const int *__restrict__ ej, const T *__restrict__ Y,
                           const T *__restrict__ R1, const T *__restrict__ M, T *__restrict__ P, int nslot, int C, int nl, int noutp,
                           int ystride, T *__restrict__ sink, int ngrp, int natoms, int spb)
{
  constexpr int CH = kAsyncChunkFwd;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  int i, grp;
  if (!pair_block(ngrp, natoms, i, grp)) return;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6, NT = blockDim.x, nw = NT >> 6;
  T *Msh = reinterpret_cast<T *>(smem_raw), *Rsh = Msh + 2 * CH * NT;
  const int slot_raw = grp * spb + t / C, n = t % C;
  const bool active = t < spb * C && slot_raw < nslot;
  const int slot = active ? slot_raw : 0;
  const int nlm = nl * nl;
  const int nact = (nslot - grp * spb < spb ? nslot - grp * spb : spb) * C;
  const long long e0 = eoff[i], e1 = eoff[i + 1];
  const int nchunk = (int) ((e1 - e0 + CH - 1) / CH);
  T acc[NLM];
#pragma unroll
  for (int q = 0; q < NLM; q++) acc[q] = (T) 0;
  for (int q = t; q < 2 * CH * NT; q += NT) Msh[q] = (T) 0;
  __syncthreads();
  auto stage = [&](int c) {
    const long long base = e0 + (long long) c * CH;
    const int nb = (int) (e1 - base < CH ? e1 - base : CH), buf = c & 1;
    // the rows of the block's slots are contiguous in M_j and in the buffer: nact values per bond
    for (int b = 0; b < nb; b++)
      block_copy_async(M + ((long long) ej[base + b] * nslot + grp * spb) * C, Msh + (size_t) (buf * CH + b) * NT, nact * (int) sizeof(T), (wave + b) % nw,
                       nw, lane);
    block_copy_async(R1 + base * noutp, Rsh + (size_t) buf * CH * noutp, nb * noutp * (int) sizeof(T), wave, nw, lane);
  };
  T touch = (T) 0;
  const bool works = __ballot(active) != 0;      // a wave without a slot (the last group of an atom) only copies
  // round c stages chunk c + 1 and works on chunk c (round -1 only stages)
  for (int c = -1; c < nchunk; c++) {
    const long long base = e0 + (long long) c * CH;
    const int nb = c < 0 ? 0 : (int) (e1 - base < CH ? e1 - base : CH), buf = c & 1;
    T tv = (T) 0;
    if (c + 1 < nchunk) {
      stage(c + 1);
      const long long nbase = base + CH;
      const int nnb = (int) (e1 - nbase < CH ? e1 - nbase : CH), per = (nlm + 7) / 8;
      if (t < nnb * per) tv = Y[(nbase + t / per) * ystride + (t % per) * 8];
    }
    for (int b = 0; b < (works ? nb : 0); b++) {
      const T m = Msh[(size_t) (buf * CH + b) * NT + t];
      const T *r = Rsh + (size_t) (buf * CH + b) * noutp + n;
      const T *y = Y + (base + b) * ystride;
#pragma unroll
      for (int l = 0; l <= kKernMaxL; l++)
        if (l * l < NLM) {
          const T rm = r[l * C] * m;
#pragma unroll
          for (int mm = 0; mm < 2 * l + 1; mm++) acc[l * l + mm] += y[l * l + mm] * rm;
        }
    }
    touch += tv;
    wait_async_loads();
    __syncthreads();
  }
  T *o = P + ((long long) i * nslot + slot) * nlm * C + n;
#pragma unroll
  for (int q = 0; q < NLM; q++)
    if (active && q < nlm) __builtin_nontemporal_store(acc[q], &o[(long long) q * C]);
  if (touch == (T) 1.2345e300) sink[0] = touch;    // keeps the touching loads alive
}

// k_pair_bwd with asynchronous staging and chunks of CH bonds; same arguments, grid and block.
// dynamic LDS: 2 CH (NT + 2 noutp) values.
template<class T, int NLM, int CH>
__global__ void k_pair_bwd_async(const long long *__restrict__ eoff, const int *__restrict__ ej, const T *__restrict__ YG,
                                 const T *__restrict__ R1, const T *__restrict__ dR1, const T *__restrict__ M, const T *__restrict__ gP,
                                 const double *__restrict__ rh, const double *__restrict__ rlen, const double *__restrict__ rcut,
                                 T *__restrict__ gM, double *__restrict__ f, double *__restrict__ virial, int nslot, int nI, int C, int nl,
                                 int noutp, T *__restrict__ sink, int one, const int *__restrict__ sid, int spb, int ngrp, int natoms, int a0,
                                 double *__restrict__ vatom, int ystr)
{
  extern __shared__ __align__(16) unsigned char smem_raw[];
  __shared__ double bsum[2][CH][4];
  __shared__ __align__(16) double g_rh[2][CH * 3], g_r[2][CH], g_rc[2][CH];
  __shared__ __align__(16) int g_j[2][CH];
  int i, grp;
  if (!pair_block(ngrp, natoms, i, grp)) return;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6, NT = blockDim.x, nw = NT >> 6;
  T *Msh = reinterpret_cast<T *>(smem_raw), *Rsh = Msh + 2 * CH * NT, *dRsh = Rsh + 2 * CH * noutp;
  const int slot_raw = grp * spb + t / C;
  const bool active = t < spb * C && slot_raw < nslot;
  const int slot = active ? slot_raw : 0, n = t % C;
  const int nlm = nl * nl;
  // threads of the block with a slot: the first nact (slots grp spb .. of the atom's rows, C values each)
  const int nact = (nslot - grp * spb < spb ? nslot - grp * spb : spb) * C;
  const long long e0 = eoff[i], e1 = eoff[i + 1];
  const int nchunk = (int) ((e1 - e0 + CH - 1) / CH);
  T g[NLM];
  {
    const T *gp = gP + ((long long) i * nslot + slot) * nlm * C + n;
#pragma unroll
    for (int q = 0; q < NLM; q++) g[q] = (active && q < nlm) ? gp[(long long) q * C] : (T) 0;
  }
  for (int q = t; q < 2 * CH * NT; q += NT) Msh[q] = (T) 0;
  if (t < 2 * CH * 4) (&bsum[0][0][0])[t] = 0.0;
  __syncthreads();
  // stage(c): everything chunk c needs, into buffer c & 1
  auto stage = [&](int c) {
    const long long base = e0 + (long long) c * CH;
    const int nb = (int) (e1 - base < CH ? e1 - base : CH), buf = c & 1;
    // the rows of the block's slots are contiguous in M_j and in the buffer: nact values per bond
    for (int b = 0; b < nb; b++)
      block_copy_async(M + ((long long) ej[base + b] * nslot + grp * spb) * C, Msh + (size_t) (buf * CH + b) * NT, nact * (int) sizeof(T), (wave + b) % nw,
                       nw, lane);
    block_copy_async(R1 + base * noutp, Rsh + (size_t) buf * CH * noutp, nb * noutp * (int) sizeof(T), (wave + 1) % nw, nw, lane);
    block_copy_async(dR1 + base * noutp, dRsh + (size_t) buf * CH * noutp, nb * noutp * (int) sizeof(T), (wave + 2) % nw, nw, lane);
    if (wave == 0) {
      if (lane < nb * 6) lds_load_word(reinterpret_cast<const char *>(rh + 3 * base) + 4 * lane, &g_rh[buf][0]);
      if (lane < nb * 2) lds_load_word(reinterpret_cast<const char *>(rlen + base) + 4 * lane, &g_r[buf][0]);
      if (lane < nb * 2) lds_load_word(reinterpret_cast<const char *>(rcut + base) + 4 * lane, &g_rc[buf][0]);
      if (lane < nb) lds_load_word(reinterpret_cast<const char *>(ej + base) + 4 * lane, &g_j[buf][0]);
    }
  };
  double fi[3] = {0, 0, 0}, vir[6] = {0, 0, 0, 0, 0, 0};
  T touch = (T) 0;
  // round c stages chunk c + 1 and works on chunk c (round -1 only stages)
  for (int c = -1; c < nchunk; c++) {
    const long long base = e0 + (long long) c * CH;
    const int nb = c < 0 ? 0 : (int) (e1 - base < CH ? e1 - base : CH), buf = c & 1;
    T tv = (T) 0;
    if (c + 1 < nchunk) {
      stage(c + 1);
      // the harmonics of the next chunk, one 64-byte piece per thread, so that its uniform reads find them in the L2
      const long long nbase = base + CH;
      const int nnb = (int) (e1 - nbase < CH ? e1 - nbase : CH), per = (nlm * 3 + 7) / 8;
      if (t < nnb * per) tv = YG[(nbase + t / per) * ystr + (t % per) * 8];
    }
    for (int b = 0; b < nb; b++) {
      const long long e = base + b;
      const T m = Msh[(size_t) (buf * CH + b) * NT + t];
      const T *r = Rsh + (size_t) (buf * CH + b) * noutp + n, *dr = dRsh + (size_t) (buf * CH + b) * noutp + n;
      const T *yg = YG + e * ystr;
      T sI = (T) 0, dE = (T) 0, t1 = (T) 0, t2 = (T) 0;
#pragma unroll
      for (int l = 0; l <= kKernMaxL; l++)
        if (l * l < NLM) for (int it = 0; it < one; it++) {
          T S = (T) 0, a1 = (T) 0, a2 = (T) 0;
#pragma unroll
          for (int mm = 0; mm < 2 * l + 1; mm++) {
            const T gv = g[l * l + mm];
            S += yg[l * l + mm] * gv; a1 += yg[nlm + l * l + mm] * gv; a2 += yg[2 * nlm + l * l + mm] * gv;
          }
          const T rl = r[l * C], drl = dr[l * C];
          sI += rl * S;
          dE += drl * S;
          t1 += rl * a1; t2 += rl * a2;
        }
      if (active && slot < nI) atomicAdd(&gM[((long long) g_j[buf][b] * nI + slot) * C + n], sI);
      const double cs = wave_sum4((double) (dE * m), (double) (t1 * m), (double) (t2 * m), 0.0, lane);
      if (lane < 3) atomicAdd(&bsum[buf][b][lane], cs);    // lanes 0..2: dE/dx, g . e2, g . e1  (order v0, v2, v1, v3)
    }
    touch += tv;
    wait_async_loads();
    __syncthreads();
    // the forces of the chunk: threads 0 .. nb - 1 while the other waves go on; bsum[buf] is clear again before the
    // chunk after the next adds to it (a barrier lies between)
    if (t < nb) {
      const double *u = &g_rh[buf][3 * t];
      const double r = g_r[buf][t], rc = g_rc[buf][t];
      const double dEdr = bsum[buf][t][0] / rc, g1 = bsum[buf][t][2] / r, g2 = bsum[buf][t][1] / r;
      bsum[buf][t][0] = bsum[buf][t][1] = bsum[buf][t][2] = 0.0;
      double e1v[3], e2v[3], fv[3];
      tangent_basis(u, e1v, e2v);
      for (int d = 0; d < 3; d++) fv[d] = dEdr * u[d] + g1 * e1v[d] + g2 * e2v[d];
      const int jj = g_j[buf][t];
      for (int d = 0; d < 3; d++) {
        fi[d] += fv[d];
        atomicAdd(&f[3 * (long long) jj + d], -fv[d]);
      }
      const double ddx = -u[0] * r, ddy = -u[1] * r, ddz = -u[2] * r;
      vir[0] += ddx * fv[0]; vir[1] += ddy * fv[1]; vir[2] += ddz * fv[2];
      vir[3] += ddx * fv[1]; vir[4] += ddx * fv[2]; vir[5] += ddy * fv[2];
      if (vatom) {    // per-atom virial: the neighbour's half of this bond (fused_cpu.h:1075-1087 of the reference)
        double *vj = vatom + 9 * (long long) jj;
        atomicAdd(vj, 0.5 * ddx * fv[0]); atomicAdd(vj + 1, 0.5 * ddy * fv[1]); atomicAdd(vj + 2, 0.5 * ddz * fv[2]);
        atomicAdd(vj + 3, 0.5 * ddx * fv[1]); atomicAdd(vj + 4, 0.5 * ddx * fv[2]); atomicAdd(vj + 5, 0.5 * ddy * fv[2]);
        // the components below the diagonal (the centroid form, kk/grace_1l_kk_impl.h:1344-1349), for both atoms of the bond
        double *vi = vatom + 9 * (long long) (a0 + i);
        const double yx = 0.5 * ddy * fv[0], zx = 0.5 * ddz * fv[0], zy = 0.5 * ddz * fv[1];
        atomicAdd(vj + 6, yx); atomicAdd(vj + 7, zx); atomicAdd(vj + 8, zy);
        atomicAdd(vi + 6, yx); atomicAdd(vi + 7, zx); atomicAdd(vi + 8, zy);
      }
    }
  }
  if (wave == 0) {
    double vsum[9] = {fi[0], fi[1], fi[2], vir[0], vir[1], vir[2], vir[3], vir[4], vir[5]};
#pragma unroll
    for (int k = 0; k < 9; k++)
      for (int o = 32; o > 0; o >>= 1) vsum[k] += __shfl_xor(vsum[k], o, 64);
    if (lane == 0 && e1 > e0) {
      for (int k = 0; k < 3; k++) atomicAdd(&f[3 * (long long) (a0 + i) + k], vsum[k]);
      for (int k = 0; k < 6; k++) atomicAdd(&virial[(sid ? 8 * sid[a0 + i] : 0) + k], vsum[3 + k]);
      if (vatom)
        for (int k = 0; k < 6; k++) atomicAdd(&vatom[9 * (long long) (a0 + i) + k], 0.5 * vsum[3 + k]);
    }
  }
  if (touch == (T) 1.2345e300) sink[0] = touch;    // keeps the touching loads alive
}

// ---- the reverse pair kernel on the matrix cores
// For one atom the adjoints gP[slot][lm][n] are fixed while the bonds change, so per l the three sums over m
//   S_l, T_l,1, T_l,2 [bond][column] = sum_m (Y, D1, D2)[bond][l, m] gP[l, m][column],   column = (slot, n),
// are products of a [16 bonds][2l + 1] tile of the harmonics with a [2l + 1][16 columns] tile of the adjoints: MFMA
// 16x16x4 with the bonds as rows, K = 2l + 1 in steps of 4 (the unused k of the last step are zero in the adjoint
// tile).  A wave owns 16 channels (n0 .. n0 + 15) of TPW slots: its adjoint tiles stay in registers for all bonds of
// the atom.  The harmonics of a chunk of 16 bonds (rows padded to `ystr` values in memory, so that a chunk is one range
// of 16-byte pieces and its LDS rows fall into different banks) and the neighbours' message rows are copied to LDS
// asynchronously one chunk ahead, a thread issuing a few 16-byte pieces; the neighbour indices of the chunk after that
// wait in registers.  The radial rows come from memory, 16 lanes reading 128 consecutive bytes of a bond's row.
// Per accumulator value (bond, column, l) four multiply-adds remain for the vector unit:
//   sI += R_l S_l;  U_l += S_l m,  V_l,k += T_l,k m  (m = the neighbour's message value; summed over the wave's slots)
// and per (bond, n, l) three:  dE/dx += dR_l U_l,  g_k += R_l V_l,k.
// Blocks are small (at most 4 waves by default, 16 tiles of 16 columns) so that two or three of them share a CU and the
// copies, barriers and force sums of one overlap the matrix work of another.
// grid: as k_pair_bwd (pair_block); block: 64 (C / 16) ceil(spb / TPW) threads;
// dynamic LDS: 2 * 16 * (spb C + ystr) values.
template<class T> struct PairMfmaArgs {
  const long long *eoff;
  const int *ej;
  const T *YG, *R1, *dR1, *M, *gP;
  const double *rh, *rlen, *rcut;
  T *gM;
  double *f, *virial, *vatom;
  const int *sid;
  int nslot, nI, C, noutp, spb, ngrp, natoms, a0, ystr;
  int one;         // 1
  int drow[16];    // accumulator row of (lane / 16, register)
};

constexpr int pair_mfma_steps(int l) { return (2 * l + 1 + 3) / 4; }
constexpr int pair_mfma_step0(int l) { return l == 0 ? 0 : pair_mfma_step0(l - 1) + pair_mfma_steps(l - 1); }
constexpr int kPairMfmaPieces = 4;    // 16-byte pieces of the neighbour rows of a chunk that one thread may have to copy

// nwords 4-byte words from global memory to LDS, in order: pieces of 64 words dealt to the waves
__device__ inline void block_copy_async_words(const void *src, void *dst, int nwords, int wave, int nw, int lane)
{
  for (int p = wave; p * 64 < nwords; p += nw)
    if (p * 64 + lane < nwords)
      lds_load_word(reinterpret_cast<const char *>(src) + 4 * (size_t) (p * 64 + lane), reinterpret_cast<char *>(dst) + 256 * (size_t) p);
}
// one 16-byte piece per lane: lane's source address, the wave's destination (the lanes' pieces land one after another)
__device__ inline void lds_load_piece(const void *src, void *lds_wave_base)
{
  __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *) src, (void __attribute__((address_space(3))) *) lds_wave_base, 16, 0, 0);
}

template<class T, int NL, int TPW>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(sizeof(T) == 4 ? 3 : 2))) void k_pair_bwd_mfma(PairMfmaArgs<T> a)
{
  typedef typename Mfma<T>::v4 v4;
  constexpr int NLM = NL * NL, STEPS = pair_mfma_step0(NL), VPP = 16 / (int) sizeof(T);    // VPP: values per 16-byte piece
  extern __shared__ __align__(16) unsigned char smem_raw[];
  __shared__ double bsum[2][16][4], fsum[16][9];    // fsum: what thread t < 16 has summed over its bonds (3 force, 6 virial)
  __shared__ __align__(16) double g_rh[2][48], g_r[2][16], g_rc[2][16];
  __shared__ __align__(16) int g_j[2][16];
  int i, grp;
  if (!pair_block(a.ngrp, a.natoms, i, grp)) return;
  const int t = threadIdx.x, lane = t & 63, wave = t >> 6, NT = blockDim.x;
  const int c = lane & 15, g = lane >> 4;
  const int C = a.C, nbk = C >> 4, mrow = a.spb * C;
  T *Msh = reinterpret_cast<T *>(smem_raw), *Ysh = Msh + 2 * 16 * mrow;
  const int n0 = (wave % nbk) * 16, ls0 = (wave / nbk) * TPW;       // channels and first local slot of the wave
  const int nloc = a.nslot - grp * a.spb < a.spb ? a.nslot - grp * a.spb : a.spb;    // slots of this block
  const long long e0 = a.eoff[i], e1 = a.eoff[i + 1];
  const int nchunk = (int) ((e1 - e0 + 15) / 16);
  // the pieces of the neighbour rows that this thread copies: piece id = t + k NT of the chunk, ppr pieces per row
  const int ppr = nloc * C / VPP;
  int prow[kPairMfmaPieces], poff[kPairMfmaPieces], jn[kPairMfmaPieces];
#pragma unroll
  for (int k = 0; k < kPairMfmaPieces; k++) {
    const int id = t + k * NT;
    prow[k] = ppr > 0 ? id / ppr : 16;
    poff[k] = ppr > 0 ? (id % ppr) * VPP : 0;
  }
  auto neighbours = [&](int ch) {      // of the rows this thread copies in chunk ch
    const long long base = e0 + (long long) ch * 16;
#pragma unroll
    for (int k = 0; k < kPairMfmaPieces; k++) jn[k] = (prow[k] < 16 && base + prow[k] < e1) ? a.ej[base + prow[k]] : -1;
  };
  if (nchunk > 0) neighbours(0);
  int rows[4];
#pragma unroll
  for (int v = 0; v < 4; v++) rows[v] = a.drow[4 * g + v];
  // the adjoint tiles of the wave: B operand, lane (g, c) holds k = 4 s + g of column c
  T B[TPW][STEPS];
  bool any = false;
#pragma unroll
  for (int q = 0; q < TPW; q++) {
    const bool ok = ls0 + q < nloc;
    any = any || ok;
    const T *gp = a.gP + ((long long) i * a.nslot + grp * a.spb + (ok ? ls0 + q : 0)) * NLM * C + n0 + c;
#pragma unroll
    for (int l = 0; l < NL; l++)
#pragma unroll
      for (int s = 0; s < pair_mfma_steps(l); s++) {
        const int kk = 4 * s + g;
        B[q][pair_mfma_step0(l) + s] = (ok && kk < 2 * l + 1) ? gp[(long long) (l * l + kk) * C] : (T) 0;
      }
  }
  for (int q = t; q < 2 * 16 * 4; q += NT) (&bsum[0][0][0])[q] = 0.0;
  for (int q = t; q < 16 * 9; q += NT) (&fsum[0][0])[q] = 0.0;
  __syncthreads();
  // stage(ch): the copies of chunk ch into buffer ch & 1 (jn: its neighbours), then the neighbours of chunk ch + 1
  auto stage = [&](int ch) {
    const long long base = e0 + (long long) ch * 16;
    const int nb = (int) (e1 - base < 16 ? e1 - base : 16), buf = ch & 1;
    char *mdst = reinterpret_cast<char *>(Msh + (size_t) buf * 16 * mrow) + 16 * (size_t) (t & ~63);
#pragma unroll
    for (int k = 0; k < kPairMfmaPieces; k++)
      if (jn[k] >= 0) lds_load_piece(a.M + ((long long) jn[k] * a.nslot + grp * a.spb) * C + poff[k], mdst + 16 * (size_t) k * NT);
    // the rows of the harmonics: one range of memory, rows of ystr values here as there
    const int ypieces = nb * a.ystr / VPP;
    const char *ysrc = reinterpret_cast<const char *>(a.YG + base * a.ystr);
    char *ydst = reinterpret_cast<char *>(Ysh + (size_t) buf * 16 * a.ystr);
    for (int id0 = t & ~63; id0 < ypieces; id0 += NT)
      if (id0 + lane < ypieces) lds_load_piece(ysrc + 16 * (size_t) (id0 + lane), ydst + 16 * (size_t) id0);
    if (wave == 0) {    // the wave that reads them for the forces of the chunk before: its reads come first
      block_copy_async_words(a.rh + 3 * base, &g_rh[buf][0], nb * 6, 0, 1, lane);
      if (lane < nb * 2) lds_load_word(reinterpret_cast<const char *>(a.rlen + base) + 4 * lane, &g_r[buf][0]);
      if (lane < nb * 2) lds_load_word(reinterpret_cast<const char *>(a.rcut + base) + 4 * lane, &g_rc[buf][0]);
      if (lane < nb) lds_load_word(reinterpret_cast<const char *>(a.ej + base) + 4 * lane, &g_j[buf][0]);
    }
    if (ch + 1 < nchunk) neighbours(ch + 1);
  };
  // round ch stages chunk ch + 1 and works on chunk ch (round -1 only stages)
  for (int ch = -1; ch < nchunk; ch++) {
    const long long base = e0 + (long long) ch * 16;
    const int nb = ch < 0 ? 0 : (int) (e1 - base < 16 ? e1 - base : 16), buf = ch & 1;
    if (ch + 1 < nchunk) stage(ch + 1);
    if (nb > 0 && any) {
      const T *Yc = Ysh + (size_t) (buf * 16 + c) * a.ystr + g;          // A operand: row = bond c of the chunk, k = 4 s + g
      const T *Mc = Msh + (size_t) buf * 16 * mrow + n0 + c;
      // the radial rows of the lane's four bonds (rows beyond the chunk: its last bond; their results are not used)
      int ro[4];
#pragma unroll
      for (int v = 0; v < 4; v++) ro[v] = (int) ((rows[v] < nb ? rows[v] : nb - 1) * a.noutp) + n0 + c;
      const T *Rb = a.R1 + base * a.noutp, *dRb = a.dR1 + base * a.noutp;
      T sI[TPW][4], pE[4], p1[4], p2[4];
      // the message values of the lane's bonds: rows of nloc C values, as copied (a row beyond the chunk: its last bond;
      // what it gives is not used)
      int mo[4];
#pragma unroll
      for (int v = 0; v < 4; v++) mo[v] = (rows[v] < nb ? rows[v] : nb - 1) * (nloc * C) + (ls0 < nloc ? ls0 : 0) * C;
#pragma unroll
      for (int q = 0; q < TPW; q++)
#pragma unroll
        for (int v = 0; v < 4; v++) sI[q][v] = (T) 0;
#pragma unroll
      for (int v = 0; v < 4; v++) pE[v] = p1[v] = p2[v] = (T) 0;
      // every l is the body of a loop that runs `one` (= 1, a kernel argument) times, so that its loads stay inside it
#pragma unroll
      for (int l = 0; l < NL; l++)
        for (int it = 0; it < a.one; it++) {
          T rc[4], dc[4];
#pragma unroll
          for (int v = 0; v < 4; v++) { rc[v] = Rb[ro[v] + l * C]; dc[v] = dRb[ro[v] + l * C]; }
          T aS[3], a1[3], a2[3];
#pragma unroll
          for (int s = 0; s < pair_mfma_steps(l); s++) {
            aS[s] = Yc[l * l + 4 * s];
            a1[s] = Yc[NLM + l * l + 4 * s];
            a2[s] = Yc[2 * NLM + l * l + 4 * s];
          }
          // the matrix products of all tiles of the wave first (a tile without a slot: its adjoint tile is zero), then
          // the vector work on their results: while that runs, the matrix unit works for the other wave of the SIMD
          v4 accS[TPW], acc1[TPW], acc2[TPW];
#pragma unroll
          for (int q = 0; q < TPW; q++) accS[q] = acc1[q] = acc2[q] = v4{0, 0, 0, 0};
#pragma unroll
          for (int s = 0; s < pair_mfma_steps(l); s++)
#pragma unroll
            for (int q = 0; q < TPW; q++) {
              const T b = B[q][pair_mfma_step0(l) + s];
              accS[q] = Mfma<T>::mma(aS[s], b, accS[q]);
              acc1[q] = Mfma<T>::mma(a1[s], b, acc1[q]);
              acc2[q] = Mfma<T>::mma(a2[s], b, acc2[q]);
            }
          T U[4] = {0, 0, 0, 0}, V1[4] = {0, 0, 0, 0}, V2[4] = {0, 0, 0, 0};
#pragma unroll
          for (int q = 0; q < TPW; q++)
#pragma unroll
            for (int v = 0; v < 4; v++) {
              const T m = ls0 + q < nloc ? Mc[mo[v] + q * C] : (T) 0;
              sI[q][v] += rc[v] * accS[q][v];
              U[v] += accS[q][v] * m;
              V1[v] += acc1[q][v] * m;
              V2[v] += acc2[q][v] * m;
            }
#pragma unroll
          for (int v = 0; v < 4; v++) {
            pE[v] += dc[v] * U[v];
            p1[v] += rc[v] * V1[v];
            p2[v] += rc[v] * V2[v];
          }
        }
      // dE/dI of the neighbours
#pragma unroll
      for (int q = 0; q < TPW; q++) {
        const int slot = grp * a.spb + ls0 + q;
        if (ls0 + q < nloc && slot < a.nI) {
#pragma unroll
          for (int v = 0; v < 4; v++)
            if (rows[v] < nb) atomicAdd(&a.gM[((long long) g_j[buf][rows[v]] * a.nI + slot) * C + n0 + c], sI[q][v]);
        }
      }
      // the three sums of the lane's four bonds over the 16 columns: 12 values, halved twice while exchanged, so that
      // lane c holds the sums of register v = c % 4
      double w[12];
#pragma unroll
      for (int v = 0; v < 4; v++) { w[v] = (double) pE[v]; w[4 + v] = (double) p1[v]; w[8 + v] = (double) p2[v]; }
      const bool b0 = c & 1, b1 = c & 2;
      double h[6];
#pragma unroll
      for (int q = 0; q < 6; q++) {
        const double keep = b0 ? w[2 * q + 1] : w[2 * q], give = b0 ? w[2 * q] : w[2 * q + 1];
        h[q] = keep + __shfl_xor(give, 1, 64);
      }
      double z[3];
#pragma unroll
      for (int q = 0; q < 3; q++) {
        const double keep = b1 ? h[2 * q + 1] : h[2 * q], give = b1 ? h[2 * q] : h[2 * q + 1];
        z[q] = keep + __shfl_xor(give, 2, 64);
        z[q] += __shfl_xor(z[q], 4, 64);
        z[q] += __shfl_xor(z[q], 8, 64);
      }
      if (c < 4) {
        const int row = a.drow[4 * g + c];
        if (row < nb) {
#pragma unroll
          for (int q = 0; q < 3; q++) atomicAdd(&bsum[buf][row][q], z[q]);
        }
      }
    }
    wait_async_loads();
    __syncthreads();
    // the forces of the chunk: threads 0 .. nb - 1 while the other waves go on; bsum[buf] is clear again before the
    // chunk after the next adds to it (a barrier lies between)
    if (t < nb) {
      const double *u = &g_rh[buf][3 * t];
      const double r = g_r[buf][t], rcv = g_rc[buf][t];
      const double dEdr = bsum[buf][t][0] / rcv, g1 = bsum[buf][t][1] / r, g2 = bsum[buf][t][2] / r;
      bsum[buf][t][0] = bsum[buf][t][1] = bsum[buf][t][2] = 0.0;
      double e1v[3], e2v[3], fv[3];
      tangent_basis(u, e1v, e2v);
      for (int d = 0; d < 3; d++) fv[d] = dEdr * u[d] + g1 * e1v[d] + g2 * e2v[d];
      const int jj = g_j[buf][t];
      double *fs = fsum[t];
      for (int d = 0; d < 3; d++) {
        fs[d] += fv[d];
        atomicAdd(&a.f[3 * (long long) jj + d], -fv[d]);
      }
      const double ddx = -u[0] * r, ddy = -u[1] * r, ddz = -u[2] * r;
      fs[3] += ddx * fv[0]; fs[4] += ddy * fv[1]; fs[5] += ddz * fv[2];
      fs[6] += ddx * fv[1]; fs[7] += ddx * fv[2]; fs[8] += ddy * fv[2];
      if (a.vatom) {    // per-atom virial, as k_pair_bwd
        double *vj = a.vatom + 9 * (long long) jj;
        atomicAdd(vj, 0.5 * ddx * fv[0]); atomicAdd(vj + 1, 0.5 * ddy * fv[1]); atomicAdd(vj + 2, 0.5 * ddz * fv[2]);
        atomicAdd(vj + 3, 0.5 * ddx * fv[1]); atomicAdd(vj + 4, 0.5 * ddx * fv[2]); atomicAdd(vj + 5, 0.5 * ddy * fv[2]);
        double *vi = a.vatom + 9 * (long long) (a.a0 + i);
        const double yx = 0.5 * ddy * fv[0], zx = 0.5 * ddz * fv[0], zy = 0.5 * ddz * fv[1];
        atomicAdd(vj + 6, yx); atomicAdd(vj + 7, zx); atomicAdd(vj + 8, zy);
        atomicAdd(vi + 6, yx); atomicAdd(vi + 7, zx); atomicAdd(vi + 8, zy);
      }
    }
  }
  if (t < 9 && e1 > e0) {
    double sum = 0.0;
    for (int q = 0; q < 16; q++) sum += fsum[q][t];      // written by threads of this wave
    if (t < 3) atomicAdd(&a.f[3 * (long long) (a.a0 + i) + t], sum);
    else {
      atomicAdd(&a.virial[(a.sid ? 8 * a.sid[a.a0 + i] : 0) + t - 3], sum);
      if (a.vatom) atomicAdd(&a.vatom[9 * (long long) (a.a0 + i) + t - 3], 0.5 * sum);
    }
  }
}

// Values per row of the harmonics and their two gradient components in memory: at least 3 nlm + 3 (the last MFMA step of
// the largest l reads up to three values past the row's third part: zeros), a whole number of 16-byte pieces, and 16
// consecutive rows in different LDS banks (fp64: rows 2 (mod 4) values apart, fp32: 4 (mod 8))
inline int pair_row_stride(int nlm, size_t value_bytes)
{
  int v = 3 * nlm + 3;
  if (value_bytes == 8) while (v % 4 != 2) v++;
  else while (v % 8 != 4) v++;
  return v;
}

// Shape of a k_pair_bwd_mfma launch for nslot message functions of C channels (TPW = 2) in blocks of at most `waves`
// waves: ok = false where the kernel does not apply (channels not in blocks of 16 or more of them than 16 waves' worth,
// lmax above 6, a thread would copy more than kPairMfmaPieces pieces of the neighbour rows)
struct PairMfmaPlan {
  bool ok = false;
  int spb = 0, ngrp = 0, threads = 0, ystr = 0;
  size_t lds = 0;
};
inline PairMfmaPlan pair_mfma_plan(int nslot, int C, int nl, size_t value_bytes, int waves)
{
  PairMfmaPlan p;
  if (C % 16 != 0 || nl > 7 || nslot < 1) return p;
  const int nbk = C / 16, wsmax = waves / nbk;
  if (wsmax < 1) return p;
  const int spbmax = wsmax * 2;
  p.ngrp = (nslot + spbmax - 1) / spbmax;
  p.spb = (nslot + p.ngrp - 1) / p.ngrp;
  p.threads = 64 * nbk * ((p.spb + 1) / 2);
  p.ystr = pair_row_stride(nl * nl, value_bytes);
  p.lds = (size_t) 2 * 16 * (p.spb * C + p.ystr) * value_bytes;
  const int pieces = 16 * (p.spb * C * (int) value_bytes / 16);
  p.ok = p.lds <= kPairLdsMax && p.threads <= 512 && pieces <= kPairMfmaPieces * p.threads;
  return p;
}
// Where the matrix-core kernel is the faster one of the reverse pair kernels (measured, fp64 / fp32, vector kernel ->
// this one): 72 slots x 64 channels 43.6 -> 37.2 ms / 31.8 -> 24.8 ms; 36 x 64: 24.5 -> 18.9 / 16.6 -> 12.4; 5 x 32:
// 6.9 -> 5.3 / 4.0 -> 3.4: everywhere it applies.  Waves of a block: 8 in fp64 (250 registers: two waves per SIMD, one
// block per CU; blocks of 4 were 5 % slower), 4 in fp32, where the kernel is compiled for three waves per SIMD (168
// registers, 8 of them spilled) and three blocks share a CU (blocks of 8: 27.2 / 13.8 / 4.3 ms).
inline int pair_mfma_waves(size_t value_bytes, int asked) { return asked > 0 ? asked : value_bytes == 4 ? 4 : 8; }

template<class T> inline void launch_pair_bwd_mfma(const PairMfmaPlan &p, PairMfmaArgs<T> a, int nl, hipStream_t stream)
{
  void (*kern)(PairMfmaArgs<T>) = nl == 1 ? k_pair_bwd_mfma<T, 1, 2> : nl == 2 ? k_pair_bwd_mfma<T, 2, 2> : nl == 3 ? k_pair_bwd_mfma<T, 3, 2>
                                : nl == 4 ? k_pair_bwd_mfma<T, 4, 2> : nl == 5 ? k_pair_bwd_mfma<T, 5, 2> : nl == 6 ? k_pair_bwd_mfma<T, 6, 2>
                                                                                                            : k_pair_bwd_mfma<T, 7, 2>;
  if (p.lds > 48 * 1024)
    HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int) p.lds));
  a.spb = p.spb;
  a.ngrp = p.ngrp;
  a.ystr = p.ystr;
  a.one = 1;
  hipLaunchKernelGGL(kern, dim3((unsigned) ((a.natoms + 7) / 8 * 8 * p.ngrp)), dim3(p.threads), p.lds, stream, a);
}

struct Energy2Dev {
  const double *W[7];         // [n_in][n_out]
  double norm[7];
  int nin[7], nout[7];
  int nlay, act, ln, nrho, rms, width;    // width: largest layer width (LDS row of the kernel)
  double out_scale, eps;
  const double *shift;        // [nel]
  const double *lnI;          // [nrho - 1] scale of the only_nonlin RMSNorm of rho
  const double *ln0;          // [nrho]     scale of the full RMSNorm of I2
};

// E_i = (MLP(x) + rho[0] + I2[0] ln0[0] / s0) out_scale + shift,  x_k = rho[k] lnI[k-1] / s1 + I2[k] ln0[k] / s0,
// s1 = sqrt(mean rho[1:]^2 + eps), s0 = sqrt(mean I2^2 + eps); dE/drho, dE/dI2.  One wave per atom, fp64; a layer with
// fewer than 33 outputs splits each dot product over 64 / outputs lanes.
static __global__ void k_energy_2l(Energy2Dev M, const int *mu, int natoms, const double *rho, const double *I2, double *grho, double *gI2,
                            double *eatom, double *energy, int want_grad, const int *sid)
{
  // LDS rows of W = M.width values: nlay + 1 activations, nlay pre-activations, 2 adjoint buffers, x0
  extern __shared__ __align__(16) unsigned char smem_raw[];
  const int W = M.width;
  double *act_ = reinterpret_cast<double *>(smem_raw), *pre_ = act_ + (M.nlay + 1) * W, *gbuf_ = pre_ + M.nlay * W, *x0 = gbuf_ + 2 * W;
#define act(L_, k_) act_[(L_) * W + (k_)]
#define pre(L_, k_) pre_[(L_) * W + (k_)]
#define gbuf(L_, k_) gbuf_[(L_) * W + (k_)]
  const int at = blockIdx.x, lane = threadIdx.x;
  const double *r = rho + (long long) at * M.nrho, *i2 = I2 + (long long) at * M.nrho;
  const int nr = M.nrho, n0 = nr - 1;
  double ms1 = 0.0, ms0 = 0.0;
  for (int k = lane; k < nr; k += 64) {
    if (k > 0) ms1 += r[k] * r[k];
    ms0 += i2[k] * i2[k];
  }
  for (int o = 32; o > 0; o >>= 1) { ms1 += __shfl_xor(ms1, o, 64); ms0 += __shfl_xor(ms0, o, 64); }
  const double s1 = M.rms ? sqrt(ms1 / n0 + M.eps) : 1.0, s0 = M.rms ? sqrt(ms0 / nr + M.eps) : 1.0;
  for (int k = lane; k < n0; k += 64) act(0, k) = r[k + 1] / s1 * M.lnI[k] + i2[k + 1] / s0 * M.ln0[k + 1];
  __syncthreads();
  double q = 0.0;
  if (M.ln) {
    double ms = 0.0;
    for (int k = lane; k < n0; k += 64) { x0[k] = act(0, k); ms += act(0, k) * act(0, k); }
    for (int o = 32; o > 0; o >>= 1) ms += __shfl_xor(ms, o, 64);
    q = 1.0 / sqrt(ms / n0 + 1e-16);
    for (int k = lane; k < n0; k += 64) act(0, k) *= q;
    __syncthreads();
  }
  // lanes that share one output of a layer: the largest power of two g with outputs x g <= 64
  auto group = [](int nout_) {
    int g = 1;
    while (g < 64 && nout_ * (g * 2) <= 64) g *= 2;
    return g;
  };
  for (int L = 0; L < M.nlay; L++) {
    const int no = M.nout[L], ni = M.nin[L], g = group(no), p = lane % g;
    for (int c0 = 0; c0 < no; c0 += 64 / g) {    // every lane walks the loop: the exchanges need the whole wave
      const int c = c0 + lane / g;
      double s = 0.0;
      if (c < no) {
#pragma unroll 4
        for (int a = p; a < ni; a += g) s += act(L, a) * M.W[L][(long long) a * no + c];
      }
      for (int o = g >> 1; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
      if (c < no && p == 0) {
        s *= M.norm[L];
        pre(L, c) = s;
        act(L + 1, c) = (L < M.nlay - 1) ? (M.act == 1 ? tanh(s) : s / (1.0 + exp(-s))) : s;
      }
    }
    __syncthreads();
  }
  const double Ei = (act(M.nlay, 0) + r[0] + i2[0] / s0 * M.ln0[0]) * M.out_scale + M.shift[mu[at]];
  if (lane == 0) {
    if (eatom) eatom[at] = Ei;
    if (energy) atomicAdd(energy + (sid ? 8 * sid[at] : 0), Ei);    // null: ordered sums, the records are added from eatom afterwards
  }
  if (!want_grad) return;
  int cur = 0;
  if (lane == 0) gbuf(0, 0) = M.out_scale;
  __syncthreads();
  for (int L = M.nlay - 1; L >= 0; L--) {
    if (L < M.nlay - 1) {
      for (int c = lane; c < M.nout[L]; c += 64) {
        const double v = pre(L, c);
        if (M.act == 1) {
          const double tt = act(L + 1, c);
          gbuf(cur, c) *= 1.0 - tt * tt;
        } else {
          const double sg = 1.0 / (1.0 + exp(-v));
          gbuf(cur, c) *= sg * (1.0 + v * (1.0 - sg));
        }
      }
      __syncthreads();
    }
    {
      const int no = M.nout[L], ni = M.nin[L], g = group(ni), p = lane % g;
      for (int b0 = 0; b0 < ni; b0 += 64 / g) {
        const int a = b0 + lane / g;
        double s = 0.0;
        if (a < ni) {
#pragma unroll 4
          for (int c = p; c < no; c += g) s += gbuf(cur, c) * M.W[L][(long long) a * no + c];
        }
        for (int o = g >> 1; o > 0; o >>= 1) s += __shfl_xor(s, o, 64);
        if (a < ni && p == 0) gbuf(cur ^ 1, a) = s * M.norm[L];
      }
    }
    cur ^= 1;
    __syncthreads();
  }
  if (M.ln) {
    double tt = 0.0;
    for (int k = lane; k < n0; k += 64) tt += gbuf(cur, k) * x0[k];
    for (int o = 32; o > 0; o >>= 1) tt += __shfl_xor(tt, o, 64);
    for (int k = lane; k < n0; k += 64) gbuf(cur, k) = q * (gbuf(cur, k) - x0[k] * tt * q * q / n0);
    __syncthreads();
  }
  // gbuf(cur, k-1) = dE/dx_k; RMSNorm reverses (y_k = x_k s_k / sigma)
  double t1 = 0.0, t0 = 0.0;
  if (M.rms) {
    for (int k = lane; k < nr; k += 64) {
      const double gy = k == 0 ? M.out_scale : gbuf(cur, k - 1);
      if (k > 0) t1 += gy * M.lnI[k - 1] * r[k];
      t0 += gy * M.ln0[k] * i2[k];
    }
    for (int o = 32; o > 0; o >>= 1) { t1 += __shfl_xor(t1, o, 64); t0 += __shfl_xor(t0, o, 64); }
  }
  double *gr = grho + (long long) at * nr, *gi = gI2 + (long long) at * nr;
  for (int k = lane; k < nr; k += 64) {
    const double gy = k == 0 ? M.out_scale : gbuf(cur, k - 1);
    gr[k] = k == 0 ? M.out_scale : gy * M.lnI[k - 1] / s1 - r[k] * t1 / (n0 * s1 * s1 * s1);
    gi[k] = gy * M.ln0[k] / s0 - i2[k] * t0 / (nr * s0 * s0 * s0);
  }
#undef act
#undef pre
#undef gbuf
}

}    // namespace grhip
