// Neighbour lists of many structures at once, built on the GPU from positions that already live there: the list of
// Batch::compute_device of the reference's GPU module (python/kk/kk_api.h:141-146; its own device list is
// libgrace/include/grace/kk/neighbors_kk.h BatchNeighborListKK).  Positions never visit the host; cells, periodic flags
// and atom counts come from the host as in the reference.
//
// The batches this serves hold hundreds of small cells, so the search is the direct one: per structure the atoms are
// wrapped into the cell along its periodic directions, and one wave per atom walks the (neighbour, image) candidates
// of its own structure 64 at a time -- count, scan, fill.  A row lists its bonds by (neighbour, image) in ascending
// order and keeps the caller's atom order, so no permutation is involved.  The bond vectors
// r_ij = xw_j + S cell - xw_i go out with the list (the engines take them in place of positions + shift table).
// Cost: natoms(s)^2 x images(s) distance tests per structure.
#pragma once

#include "engine_common.hpp"

#include <cmath>
#include <vector>

namespace grhip {

struct BnlStruct {
  int first, n;          // atoms first .. first + n of the packed atom list
  int reach[3];          // images -reach .. reach along each cell vector (0: open direction)
  int nimg;              // (2 reach0 + 1)(2 reach1 + 1)(2 reach2 + 1)
  double cell[9];        // rows: the cell vectors (open directions: any completion to full rank)
  double inv[9];         // inverse of `cell`: fractional coordinate k = sum_d x_d inv[3 d + k]
};

// xw[a] = x[a] - sum_k floor(frac_k) cell_k over the periodic directions k
static __global__ void k_bnl_wrap(const BnlStruct *S, const int *sid, const double *x, double *xw, int n)
{
  const int a = blockIdx.x * blockDim.x + threadIdx.x;
  if (a >= n) return;
  const BnlStruct &s = S[sid[a]];
  double p[3] = {x[3 * (long long) a], x[3 * (long long) a + 1], x[3 * (long long) a + 2]};
  double w[3] = {p[0], p[1], p[2]};
  for (int k = 0; k < 3; k++) {
    if (s.reach[k] == 0) continue;
    const double f = p[0] * s.inv[k] + p[1] * s.inv[3 + k] + p[2] * s.inv[6 + k];
    const double fl = floor(f);
    for (int d = 0; d < 3; d++) w[d] -= fl * s.cell[3 * k + d];
  }
  for (int d = 0; d < 3; d++) xw[3 * (long long) a + d] = w[d];
}

// One wave per atom.  FILL = false: count[a] = bonds of atom a within rc.  FILL = true: j and rij of those bonds from
// offset[a] on, in candidate order (neighbour ascending, then image ascending).
template<bool FILL>
__global__ __launch_bounds__(256) void k_bnl_pairs(const BnlStruct *S, const int *sid, const double *xw, double rc2, int n, int *count,
                                                   const long long *offset, int *j, double *rij)
{
  const int lane = threadIdx.x & 63;
  const int a = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (a >= n) return;
  const BnlStruct &s = S[sid[a]];
  const double xa[3] = {xw[3 * (long long) a], xw[3 * (long long) a + 1], xw[3 * (long long) a + 2]};
  const int w1 = 2 * s.reach[1] + 1, w2 = 2 * s.reach[2] + 1;
  const long long ncand = (long long) s.n * s.nimg;
  long long w = FILL ? offset[a] : 0;
  int c = 0;
  for (long long q0 = 0; q0 < ncand; q0 += 64) {
    const long long q = q0 + lane;
    bool hit = false;
    int b = 0;
    double d[3] = {0, 0, 0};
    if (q < ncand) {
      const int nbr = (int) (q / s.nimg), im = (int) (q % s.nimg);
      const int s0 = im / (w1 * w2) - s.reach[0], s1 = (im / w2) % w1 - s.reach[1], s2 = im % w2 - s.reach[2];
      b = s.first + nbr;
      for (int k = 0; k < 3; k++)
        d[k] = (xw[3 * (long long) b + k] - xa[k]) + (s0 * s.cell[k] + s1 * s.cell[3 + k] + s2 * s.cell[6 + k]);
      const double r2 = d[0] * d[0] + d[1] * d[1] + d[2] * d[2];
      hit = r2 < rc2 && !(b == a && s0 == 0 && s1 == 0 && s2 == 0);
    }
    const unsigned long long m = __ballot(hit);
    if (FILL) {
      if (hit) {
        const long long at = w + __popcll(m & ((1ull << lane) - 1ull));
        j[at] = b;
        rij[3 * at] = d[0]; rij[3 * at + 1] = d[1]; rij[3 * at + 2] = d[2];
      }
      w += __popcll(m);
    } else {
      c += __popcll(m);
    }
  }
  if (!FILL && lane == 0) count[a] = c;
}

class BatchDeviceNeighbors {
 public:
  int64_t nb = 0;
  DevBuf offset, j, rij;          // [N + 1] i64, [nb] i32, [nb][3] f64
  std::vector<int> sid;           // structure of every atom (host)

  // natoms [nstruct] (host), pos [N][3] (device), cells [nstruct][3][3] and pbc [nstruct][3] (host).  A direction is
  // periodic when its flag is set and its cell vector is not zero; the other cell vectors are not read.
  void build(int nstruct, const int *natoms, const double *pos, const double *cells, const unsigned char *pbc, double cutoff,
             hipStream_t stream)
  {
    if (!(cutoff > 0.0) || !std::isfinite(cutoff)) throw InvalidArgument("cutoff must be positive");
    std::vector<BnlStruct> tab((size_t) nstruct);
    int64_t N = 0;
    for (int s = 0; s < nstruct; s++) {
      if (natoms[s] < 0) throw InvalidArgument("negative atom count");
      BnlStruct &b = tab[s];
      b.first = (int) N;
      b.n = natoms[s];
      N += natoms[s];
      if (N >= INT32_MAX) throw InvalidArgument("atom count out of range");
      fill_cell(cells + 9 * (size_t) s, pbc + 3 * (size_t) s, cutoff, b);
    }
    sid.resize((size_t) N);
    for (int s = 0; s < nstruct; s++) std::fill(sid.begin() + tab[s].first, sid.begin() + tab[s].first + tab[s].n, s);
    nb = 0;
    offset.ensure(sizeof(long long) * (size_t) (N + 1));
    if (N == 0) {
      const long long z = 0;
      HIP_CHECK(hipMemcpy(offset.p, &z, sizeof(z), hipMemcpyHostToDevice));
      return;
    }
    tab_.ensure(sizeof(BnlStruct) * tab.size());
    sid_.ensure(sizeof(int) * (size_t) N);
    xw_.ensure(sizeof(double) * 3 * (size_t) N);
    count_.ensure(sizeof(int) * (size_t) N);
    HIP_CHECK(hipMemcpyAsync(tab_.p, tab.data(), sizeof(BnlStruct) * tab.size(), hipMemcpyHostToDevice, stream));
    HIP_CHECK(hipMemcpyAsync(sid_.p, sid.data(), sizeof(int) * (size_t) N, hipMemcpyHostToDevice, stream));
    const int n = (int) N;
    hipLaunchKernelGGL(k_bnl_wrap, dim3((unsigned) ((n + 255) / 256)), dim3(256), 0, stream, tab_.as<BnlStruct>(), sid_.as<int>(), pos,
                       xw_.as<double>(), n);
    const dim3 grid((unsigned) ((n + 3) / 4)), block(256);
    hipLaunchKernelGGL(k_bnl_pairs<false>, grid, block, 0, stream, tab_.as<BnlStruct>(), sid_.as<int>(), xw_.as<double>(), cutoff * cutoff, n,
                       count_.as<int>(), (const long long *) nullptr, (int *) nullptr, (double *) nullptr);
    hipLaunchKernelGGL(k_scan, dim3(1), dim3(1024), 0, stream, count_.as<int>(), n, offset.as<long long>());
    long long total = 0;
    HIP_CHECK(hipMemcpyAsync(&total, offset.as<long long>() + n, sizeof(total), hipMemcpyDeviceToHost, stream));
    HIP_CHECK(hipStreamSynchronize(stream));    // also: the host tables above are free to go
    nb = total;
    j.ensure(sizeof(int) * (size_t) std::max<int64_t>(nb, 1));
    rij.ensure(sizeof(double) * 3 * (size_t) std::max<int64_t>(nb, 1));
    hipLaunchKernelGGL(k_bnl_pairs<true>, grid, block, 0, stream, tab_.as<BnlStruct>(), sid_.as<int>(), xw_.as<double>(), cutoff * cutoff, n,
                       (int *) nullptr, (const long long *) offset.as<long long>(), j.as<int>(), rij.as<double>());
    HIP_CHECK(hipGetLastError());
  }

 private:
  DevBuf tab_, sid_, xw_, count_;

  static void fill_cell(const double *cell, const unsigned char *pbc, double cutoff, BnlStruct &b)
  {
    bool per[3];
    double a[9];
    int nper = 0;
    for (int k = 0; k < 3; k++) {
      const double *v = cell + 3 * k;
      per[k] = pbc[k] && !(v[0] == 0.0 && v[1] == 0.0 && v[2] == 0.0);
      for (int d = 0; d < 3; d++) {
        if (per[k] && !std::isfinite(v[d])) throw InvalidArgument("cell vectors must be finite");
        a[3 * k + d] = per[k] ? v[d] : 0.0;
      }
      nper += per[k];
    }
    // unit vectors normal to the periodic ones complete the matrix (they carry no images and no wrap)
    auto cross = [](const double *u, const double *v, double *o) {
      o[0] = u[1] * v[2] - u[2] * v[1]; o[1] = u[2] * v[0] - u[0] * v[2]; o[2] = u[0] * v[1] - u[1] * v[0];
    };
    auto unit = [](double *u) {
      const double l = std::sqrt(u[0] * u[0] + u[1] * u[1] + u[2] * u[2]);
      if (!(l > 0.0)) throw InvalidArgument("the periodic cell vectors are linearly dependent");
      for (int d = 0; d < 3; d++) u[d] /= l;
    };
    int open[3], no = 0, given[3], ng = 0;
    for (int k = 0; k < 3; k++) (per[k] ? given[ng++] : open[no++]) = k;
    if (nper == 0) {
      for (int k = 0; k < 3; k++) a[3 * k + k] = 1.0;
    } else if (nper == 2) {
      cross(a + 3 * given[0], a + 3 * given[1], a + 3 * open[0]);
      unit(a + 3 * open[0]);
    } else if (nper == 1) {
      double u[3] = {a[3 * given[0]], a[3 * given[0] + 1], a[3 * given[0] + 2]};
      unit(u);
      int kmin = 0;
      for (int d = 1; d < 3; d++)
        if (std::fabs(u[d]) < std::fabs(u[kmin])) kmin = d;
      double e[3] = {0, 0, 0};
      e[kmin] = 1.0;
      cross(u, e, a + 3 * open[0]);
      unit(a + 3 * open[0]);
      cross(u, a + 3 * open[0], a + 3 * open[1]);
      unit(a + 3 * open[1]);
    }
    const double det = a[0] * (a[4] * a[8] - a[5] * a[7]) - a[1] * (a[3] * a[8] - a[5] * a[6]) + a[2] * (a[3] * a[7] - a[4] * a[6]);
    const double na = std::sqrt(a[0] * a[0] + a[1] * a[1] + a[2] * a[2]), nb_ = std::sqrt(a[3] * a[3] + a[4] * a[4] + a[5] * a[5]),
                 nc = std::sqrt(a[6] * a[6] + a[7] * a[7] + a[8] * a[8]);
    if (!std::isfinite(det) || !(std::fabs(det) > 1e-12 * na * nb_ * nc)) throw InvalidArgument("neighbour search needs a full-rank cell");
    const double dd = 1.0 / det;
    const double inv[9] = {(a[4] * a[8] - a[5] * a[7]) * dd, (a[2] * a[7] - a[1] * a[8]) * dd, (a[1] * a[5] - a[2] * a[4]) * dd,
                           (a[5] * a[6] - a[3] * a[8]) * dd, (a[0] * a[8] - a[2] * a[6]) * dd, (a[2] * a[3] - a[0] * a[5]) * dd,
                           (a[3] * a[7] - a[4] * a[6]) * dd, (a[1] * a[6] - a[0] * a[7]) * dd, (a[0] * a[4] - a[1] * a[3]) * dd};
    int64_t nimg = 1;
    for (int k = 0; k < 3; k++) {
      b.reach[k] = 0;
      if (per[k]) {
        // height of the cell along direction k = 1 / |column k of the inverse|
        const double h = 1.0 / std::sqrt(inv[k] * inv[k] + inv[3 + k] * inv[3 + k] + inv[6 + k] * inv[6 + k]);
        const double r = std::ceil(cutoff / h);
        if (!(r < 1024.0)) throw InvalidArgument("a periodic cell vector is shorter than 1/1000 of the cutoff");
        b.reach[k] = std::max(1, (int) r);
      }
      nimg *= 2 * b.reach[k] + 1;
    }
    if (nimg > (int64_t(1) << 24)) throw InvalidArgument("the cutoff spans too many periodic images of a cell");
    b.nimg = (int) nimg;
    for (int k = 0; k < 9; k++) { b.cell[k] = a[k]; b.inv[k] = inv[k]; }
  }
};

}    // namespace grhip
