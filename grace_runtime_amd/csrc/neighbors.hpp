// Host neighbour list that reproduces the reference list bond for bond (same permutation, CSR rows, (j, image)
// order and shift table): fractional-coordinate binning with bin edge >= cutoff / 2, stable counting sort by bin,
// per atom the bins in lexicographic offset order and inside a bin by slot.  Algorithm of
// libgrace/include/grace/cell_list.h:39-152,216-241 and python/src/neighbors.cpp:15-95; the floating-point
// expressions are written in the same operation order so that the r^2 < rc^2 decisions agree bit for bit.
#pragma once

#include "npz.hpp"

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

namespace grhip {

struct NeighborList {
  std::vector<int64_t> perm, offset;
  std::vector<int32_t> j, image;
  std::vector<double> shifts;
};

namespace nl_detail {
inline int64_t floordiv(int64_t a, int64_t b) { return a >= 0 ? a / b : -((-a + b - 1) / b); }
inline int64_t bin_reach(double rc, double w, int64_t nbin, bool pbc)
{
  const int64_t r = (int64_t) std::ceil(rc / w - 1e-12);
  return pbc ? r : std::min(r, nbin - 1);
}

struct Cells {
  int64_t n = 0;
  double cell[9];
  bool pbc[3];
  int64_t nbin[3] = {1, 1, 1};
  double width[3] = {1, 1, 1};
  std::vector<int64_t> perm, start, b3, img;
  std::vector<double> xw;

  void build(const double *pos, int64_t n_, const double *cell_, const bool *pbc_, double bin_size)
  {
    n = n_;
    for (int k = 0; k < 9; k++) cell[k] = cell_[k];
    for (int k = 0; k < 3; k++) pbc[k] = pbc_[k];
    perm.assign(n, 0);
    xw.assign(3 * n, 0.0);
    b3.assign(3 * n, 0);
    img.assign(3 * n, 0);
    const double *a = cell;
    const double det = a[0] * (a[4] * a[8] - a[5] * a[7]) - a[1] * (a[3] * a[8] - a[5] * a[6]) + a[2] * (a[3] * a[7] - a[4] * a[6]);
    {
      const double na = std::sqrt(a[0] * a[0] + a[1] * a[1] + a[2] * a[2]);
      const double nb = std::sqrt(a[3] * a[3] + a[4] * a[4] + a[5] * a[5]);
      const double nc = std::sqrt(a[6] * a[6] + a[7] * a[7] + a[8] * a[8]);
      if (!std::isfinite(det) || !(std::abs(det) > 1e-12 * na * nb * nc))
        throw InvalidArgument("neighbour search needs a full-rank cell");
    }
    const double d = 1.0 / det;
    const double inv[9] = {(a[4] * a[8] - a[5] * a[7]) * d, (a[2] * a[7] - a[1] * a[8]) * d, (a[1] * a[5] - a[2] * a[4]) * d,
                           (a[5] * a[6] - a[3] * a[8]) * d, (a[0] * a[8] - a[2] * a[6]) * d, (a[2] * a[3] - a[0] * a[5]) * d,
                           (a[3] * a[7] - a[4] * a[6]) * d, (a[1] * a[6] - a[0] * a[7]) * d, (a[0] * a[4] - a[1] * a[3]) * d};
    double h[3], lo[3] = {0, 0, 0}, span[3] = {1, 1, 1};
    for (int k = 0; k < 3; k++) h[k] = 1.0 / std::sqrt(inv[k] * inv[k] + inv[3 + k] * inv[3 + k] + inv[6 + k] * inv[6 + k]);
    std::vector<double> frac(3 * n);
    for (int64_t i = 0; i < n; i++)
      for (int k = 0; k < 3; k++) {
        const double f = pos[3 * i] * inv[k] + pos[3 * i + 1] * inv[3 + k] + pos[3 * i + 2] * inv[6 + k];
        if (!std::isfinite(f)) throw InvalidArgument("positions must be finite");
        const double fl = pbc[k] ? std::floor(f) : 0.0;
        img[3 * i + k] = (int64_t) fl;
        frac[3 * i + k] = f - fl;
      }
    for (int k = 0; k < 3; k++)
      if (!pbc[k]) {
        double mn = frac[k], mx = frac[k];
        for (int64_t i = 1; i < n; i++) {
          mn = std::min(mn, frac[3 * i + k]);
          mx = std::max(mx, frac[3 * i + k]);
        }
        lo[k] = mn;
        span[k] = std::max(mx - mn, 1e-12);
      }
    const int64_t max_bins = 8 * n + 64;
    for (int k = 0; k < 3; k++) {
      const double nb = std::floor(span[k] * h[k] / bin_size);
      nbin[k] = (int64_t) std::min<double>(std::max(nb, 1.0), (double) max_bins);
    }
    while ((double) nbin[0] * (double) nbin[1] * (double) nbin[2] > (double) max_bins) {
      const int k = (int) (std::max_element(nbin, nbin + 3) - nbin);
      nbin[k] = std::max<int64_t>(1, nbin[k] / 2);
    }
    for (int k = 0; k < 3; k++) width[k] = span[k] * h[k] / (double) nbin[k];
    const int64_t nbt = nbin[0] * nbin[1] * nbin[2];
    std::vector<int64_t> bin(n);
    start.assign(nbt + 1, 0);
    for (int64_t i = 0; i < n; i++) {
      for (int k = 0; k < 3; k++) {
        const int64_t b = (int64_t) std::floor((frac[3 * i + k] - lo[k]) / span[k] * (double) nbin[k]);
        b3[3 * i + k] = std::min(std::max<int64_t>(b, 0), nbin[k] - 1);
      }
      bin[i] = (b3[3 * i] * nbin[1] + b3[3 * i + 1]) * nbin[2] + b3[3 * i + 2];
      start[bin[i] + 1]++;
    }
    for (int64_t b = 0; b < nbt; b++) start[b + 1] += start[b];
    std::vector<int64_t> fill(start.begin(), start.end() - 1);
    for (int64_t i = 0; i < n; i++) {
      const int64_t s = fill[bin[i]]++;
      perm[s] = i;
      for (int dd = 0; dd < 3; dd++)
        xw[3 * s + dd] = frac[3 * i] * cell[dd] + frac[3 * i + 1] * cell[3 + dd] + frac[3 * i + 2] * cell[6 + dd];
    }
  }

  // fn(p, s0, s1, s2) for every neighbour slot p of slot q within rc, images S in the wrapped frame
  template<class F> void visit(int64_t q, double rc, F &&fn) const
  {
    const double rc2 = rc * rc;
    const double *xq = &xw[3 * q];
    int64_t reach[3];
    for (int k = 0; k < 3; k++) reach[k] = bin_reach(rc, width[k], nbin[k], pbc[k]);
    const int64_t *bq = &b3[3 * perm[q]];
    for (int64_t o0 = -reach[0]; o0 <= reach[0]; o0++) {
      int64_t c0 = bq[0] + o0, s0 = 0;
      if (pbc[0]) { s0 = floordiv(c0, nbin[0]); c0 -= s0 * nbin[0]; }
      else if (c0 < 0 || c0 >= nbin[0]) continue;
      for (int64_t o1 = -reach[1]; o1 <= reach[1]; o1++) {
        int64_t c1 = bq[1] + o1, s1 = 0;
        if (pbc[1]) { s1 = floordiv(c1, nbin[1]); c1 -= s1 * nbin[1]; }
        else if (c1 < 0 || c1 >= nbin[1]) continue;
        for (int64_t o2 = -reach[2]; o2 <= reach[2]; o2++) {
          int64_t c2 = bq[2] + o2, s2 = 0;
          if (pbc[2]) { s2 = floordiv(c2, nbin[2]); c2 -= s2 * nbin[2]; }
          else if (c2 < 0 || c2 >= nbin[2]) continue;
          const int64_t c = (c0 * nbin[1] + c1) * nbin[2] + c2;
          const double sx = s0 * cell[0] + s1 * cell[3] + s2 * cell[6];
          const double sy = s0 * cell[1] + s1 * cell[4] + s2 * cell[7];
          const double sz = s0 * cell[2] + s1 * cell[5] + s2 * cell[8];
          const bool own = o0 == 0 && o1 == 0 && o2 == 0;
          for (int64_t p = start[c]; p < start[c + 1]; p++) {
            if (own && p == q) continue;
            const double dx = xw[3 * p] + sx - xq[0];
            const double dy = xw[3 * p + 1] + sy - xq[1];
            const double dz = xw[3 * p + 2] + sz - xq[2];
            const double r2 = dx * dx + dy * dy + dz * dz;
            if (r2 < rc2) fn(p, s0, s1, s2);
          }
        }
      }
    }
  }
};
}    // namespace nl_detail

inline NeighborList neighbor_search(const double *pos, int64_t n, const double *cell, const bool *pbc, double cutoff, int nthreads)
{
  using namespace nl_detail;
  if (!(cutoff > 0.0) || !std::isfinite(cutoff)) throw InvalidArgument("cutoff must be positive");
  if (n < 0 || n >= INT32_MAX) throw InvalidArgument("atom count out of range");
  NeighborList r;
  r.offset.assign(n + 1, 0);
  if (n == 0) return r;
  Cells cl;
  cl.build(pos, n, cell, pbc, 0.5 * cutoff);
  r.perm = cl.perm;
  constexpr int64_t kB = int64_t(1) << 20;
  bool far = false;
  auto key = [&](int64_t a, int64_t b, int64_t s0, int64_t s1, int64_t s2, bool &far_) {
    const int64_t *ia = &cl.img[3 * a], *ib = &cl.img[3 * b];
    const int64_t t0 = s0 - ib[0] + ia[0], t1 = s1 - ib[1] + ia[1], t2 = s2 - ib[2] + ia[2];
    if (std::max({std::abs(t0), std::abs(t1), std::abs(t2)}) >= kB) {
      far_ = true;
      return int64_t(0);
    }
    return ((t0 + kB) << 42) | ((t1 + kB) << 21) | (t2 + kB);
  };
  std::vector<int64_t> nn(n), keys;
  const int nth = std::max(1, nthreads);
#pragma omp parallel num_threads(nth)
  {
    std::vector<int64_t> seen;
    int64_t last = -1;
    bool myfar = false;
#pragma omp for schedule(dynamic, 64)
    for (int64_t q = 0; q < n; q++) {
      const int64_t a = r.perm[q];
      int64_t c = 0;
      cl.visit(q, cutoff, [&](int64_t p, int64_t s0, int64_t s1, int64_t s2) {
        c++;
        const int64_t k = key(a, r.perm[p], s0, s1, s2, myfar);
        if (k != last) seen.push_back(last = k);
      });
      nn[q] = c;
      if (seen.size() > 4096) {
        std::sort(seen.begin(), seen.end());
        seen.erase(std::unique(seen.begin(), seen.end()), seen.end());
      }
    }
#pragma omp critical
    {
      keys.insert(keys.end(), seen.begin(), seen.end());
      far = far || myfar;
    }
  }
  if (far) throw InvalidArgument("atoms a million cells or more apart: wrap the positions");
  std::sort(keys.begin(), keys.end());
  keys.erase(std::unique(keys.begin(), keys.end()), keys.end());
  r.shifts.resize(3 * keys.size());
  for (size_t u = 0; u < keys.size(); u++) {
    const int64_t m = (int64_t(1) << 21) - 1, k = keys[u];
    const double t0 = (double) (((k >> 42) & m) - kB), t1 = (double) (((k >> 21) & m) - kB), t2 = (double) ((k & m) - kB);
    // fused multiply-adds in the order an FMA-contracting compiler gives the reference's expression
    // t0 a_d + t1 b_d + t2 c_d (the reference builds with -march=native), so that the table agrees to the bit
    for (int d = 0; d < 3; d++) r.shifts[3 * u + d] = std::fma(t2, cell[6 + d], std::fma(t1, cell[3 + d], t0 * cell[d]));
  }
  for (int64_t q = 0; q < n; q++) r.offset[q + 1] = r.offset[q] + nn[q];
  const int64_t nb = r.offset[n];
  r.j.resize(nb);
  r.image.resize(nb);
#pragma omp parallel for schedule(dynamic, 64) num_threads(nth)
  for (int64_t q = 0; q < n; q++) {
    int64_t w = r.offset[q], last = -1;
    int32_t u = 0;
    bool f2 = false;
    const int64_t a = r.perm[q];
    cl.visit(q, cutoff, [&](int64_t p, int64_t s0, int64_t s1, int64_t s2) {
      const int64_t k = key(a, r.perm[p], s0, s1, s2, f2);
      if (k != last) u = (int32_t) (std::lower_bound(keys.begin(), keys.end(), last = k) - keys.begin());
      r.j[w] = (int32_t) p;
      r.image[w] = u;
      w++;
    });
  }
  return r;
}

}    // namespace grhip
