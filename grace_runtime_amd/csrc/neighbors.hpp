// Host neighbour list: the list the reference's search returns (python/src/neighbors.cpp:15-95 over the cell list of
// libgrace/include/grace/cell_list.h:39-152), bond for bond: the same permutation (atoms in bin order, a bin's atoms in
// input order), the same rows (bins in ascending offset order, a bin's atoms by slot), the same shift table (distinct
// image differences in ascending order).
//
// Layout of this implementation: a Frame (cell, inverse, plane spacings), a Grid (bins per direction and the map atom ->
// bin), and a search in which every thread walks a contiguous range of slots ONCE, appending (neighbour, image key) pairs
// to its own arrays; rows are then laid out by prefix sums and the image keys are ranked.  Only the floating-point
// expressions that decide a result are fixed by the reference and keep its operation order: the fractional coordinate,
// the bin index, the wrapped position and the squared distance (marked "order matters" below).
#pragma once

#include "npz.hpp"

#include <algorithm>
#include <array>
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

namespace nl {

constexpr int64_t kFarImages = int64_t(1) << 20;    // image differences must stay below this in every direction

// The periodic frame: rows of `a` are the cell vectors, columns of `inv` the reciprocal ones, `gap[k]` the distance
// between the lattice planes normal to reciprocal vector k.
struct Frame {
  double a[9], inv[9], gap[3];
  bool periodic[3];

  Frame(const double *cell, const bool *pbc)
  {
    for (int k = 0; k < 9; k++) a[k] = cell[k];
    for (int k = 0; k < 3; k++) periodic[k] = pbc[k];
    const double c00 = a[4] * a[8] - a[5] * a[7], c01 = a[3] * a[8] - a[5] * a[6], c02 = a[3] * a[7] - a[4] * a[6];
    const double volume = a[0] * c00 - a[1] * c01 + a[2] * c02;    // order matters (threshold below, and 1 / volume)
    double edge[3];
    for (int k = 0; k < 3; k++) edge[k] = std::sqrt(a[3 * k] * a[3 * k] + a[3 * k + 1] * a[3 * k + 1] + a[3 * k + 2] * a[3 * k + 2]);
    if (!std::isfinite(volume) || !(std::abs(volume) > 1e-12 * edge[0] * edge[1] * edge[2]))
      throw InvalidArgument("the neighbour search needs three linearly independent cell vectors (a full-rank cell)");
    const double s = 1.0 / volume;
    // adjugate times 1 / volume, element by element: order matters (fractional coordinates)
    inv[0] = c00 * s;
    inv[1] = (a[2] * a[7] - a[1] * a[8]) * s;
    inv[2] = (a[1] * a[5] - a[2] * a[4]) * s;
    inv[3] = (a[5] * a[6] - a[3] * a[8]) * s;
    inv[4] = (a[0] * a[8] - a[2] * a[6]) * s;
    inv[5] = (a[2] * a[3] - a[0] * a[5]) * s;
    inv[6] = c02 * s;
    inv[7] = (a[1] * a[6] - a[0] * a[7]) * s;
    inv[8] = (a[0] * a[4] - a[1] * a[3]) * s;
    for (int k = 0; k < 3; k++) gap[k] = 1.0 / std::sqrt(inv[k] * inv[k] + inv[3 + k] * inv[3 + k] + inv[6 + k] * inv[6 + k]);
  }
  // order matters
  double fractional(const double *x, int k) const { return x[0] * inv[k] + x[1] * inv[3 + k] + x[2] * inv[6 + k]; }
  double cartesian(const double *u, int d) const { return u[0] * a[d] + u[1] * a[3 + d] + u[2] * a[6 + d]; }
  double image_shift(int64_t s0, int64_t s1, int64_t s2, int d) const { return s0 * a[d] + s1 * a[3 + d] + s2 * a[6 + d]; }
};

// Bins of edge >= bin_edge along every direction over the span of the fractional coordinates (the whole cell along
// periodic directions, the occupied range along open ones), at most 8 n + 64 bins in all.
struct Grid {
  int64_t count[3] = {1, 1, 1};
  double origin[3] = {0.0, 0.0, 0.0}, extent[3] = {1.0, 1.0, 1.0}, width[3] = {1.0, 1.0, 1.0};

  void choose(const Frame &fr, const std::vector<double> &u, int64_t n, double bin_edge)
  {
    double low[3], high[3];
    for (int k = 0; k < 3; k++) {
      low[k] = high[k] = u[k];
      for (int64_t i = 1; i < n; i++) {
        low[k] = std::min(low[k], u[3 * i + k]);
        high[k] = std::max(high[k], u[3 * i + k]);
      }
    }
    choose(fr, low, high, n, bin_edge);
  }
  // low / high: smallest and largest fractional coordinate of the atoms per direction (used along open directions)
  void choose(const Frame &fr, const double *low, const double *high, int64_t n, double bin_edge)
  {
    for (int k = 0; k < 3; k++) {
      if (fr.periodic[k]) continue;
      origin[k] = low[k];
      extent[k] = std::max(high[k] - low[k], 1e-12);
    }
    const double budget = (double) (8 * n + 64);
    for (int k = 0; k < 3; k++) count[k] = (int64_t) std::min(std::max(std::floor(extent[k] * fr.gap[k] / bin_edge), 1.0), budget);    // order matters
    while ((double) count[0] * (double) count[1] * (double) count[2] > budget) {
      int widest = 0;
      for (int k = 1; k < 3; k++)
        if (count[k] > count[widest]) widest = k;
      count[widest] = std::max<int64_t>(1, count[widest] / 2);
    }
    for (int k = 0; k < 3; k++) width[k] = extent[k] * fr.gap[k] / (double) count[k];
  }
  int64_t total() const { return count[0] * count[1] * count[2]; }
  int64_t along(double u, int k) const    // order matters
  {
    const int64_t b = (int64_t) std::floor((u - origin[k]) / extent[k] * (double) count[k]);
    return std::min(std::max<int64_t>(b, 0), count[k] - 1);
  }
  // bins to visit on either side so that nothing within `cutoff` is missed
  int64_t reach(double cutoff, int k, bool periodic) const
  {
    const int64_t r = (int64_t) std::ceil(cutoff / width[k] - 1e-12);
    return periodic ? r : std::min(r, count[k] - 1);
  }
};

// The atoms sorted into bins: slot q holds atom perm[q]; per slot the wrapped Cartesian position, the bin triple and the
// image the atom was wrapped by.
struct Binned {
  Frame frame;
  Grid grid;
  int64_t n = 0;
  std::vector<int64_t> perm, first;     // first[b] .. first[b + 1]: slots of bin b
  std::vector<double> x;                // [n][3] wrapped positions by slot
  std::vector<int32_t> bin3, wrap3;     // [n][3] by slot

  Binned(const double *pos, int64_t n_, const double *cell, const bool *pbc, double bin_edge) : frame(cell, pbc), n(n_)
  {
    std::vector<double> u((size_t) 3 * n);
    std::vector<int64_t> wrapped((size_t) 3 * n);
    for (int64_t i = 0; i < n; i++)
      for (int k = 0; k < 3; k++) {
        const double f = frame.fractional(pos + 3 * i, k);
        if (!std::isfinite(f)) throw InvalidArgument("atom " + std::to_string(i) + " has a position that is not finite");
        const double whole = frame.periodic[k] ? std::floor(f) : 0.0;
        wrapped[3 * i + k] = (int64_t) whole;
        u[3 * i + k] = f - whole;
      }
    grid.choose(frame, u, n, bin_edge);
    // counting sort by bin, atoms of a bin in input order
    std::vector<int64_t> bin_of((size_t) n);
    first.assign((size_t) grid.total() + 1, 0);
    for (int64_t i = 0; i < n; i++) {
      bin_of[i] = (grid.along(u[3 * i], 0) * grid.count[1] + grid.along(u[3 * i + 1], 1)) * grid.count[2] + grid.along(u[3 * i + 2], 2);
      first[bin_of[i] + 1]++;
    }
    for (size_t b = 1; b < first.size(); b++) first[b] += first[b - 1];
    std::vector<int64_t> cursor(first.begin(), first.end() - 1);
    perm.resize((size_t) n);
    x.resize((size_t) 3 * n);
    bin3.resize((size_t) 3 * n);
    wrap3.resize((size_t) 3 * n);
    for (int64_t i = 0; i < n; i++) {
      const int64_t q = cursor[bin_of[i]]++;
      perm[q] = i;
      for (int k = 0; k < 3; k++) {
        if (std::abs(wrapped[3 * i + k]) >= (int64_t(1) << 30)) throw InvalidArgument("atoms a million cells or more from the cell: wrap the positions first");
        x[3 * q + k] = frame.cartesian(&u[3 * i], k);
        bin3[3 * q + k] = (int32_t) grid.along(u[3 * i + k], k);
        wrap3[3 * q + k] = (int32_t) wrapped[3 * i + k];
      }
    }
  }

  // One direction of the walk over neighbouring bins: the bins at offsets -reach .. reach of bin b, folded back into
  // the grid along a periodic direction (with the image they lie in) and clipped along an open one.
  struct Step {
    int64_t bin, image;
    bool home;
  };
  void steps(int k, int64_t b, int64_t reach, std::vector<Step> &out) const
  {
    out.clear();
    const int64_t m = grid.count[k];
    for (int64_t o = -reach; o <= reach; o++) {
      int64_t c = b + o, s = 0;
      if (frame.periodic[k]) {
        s = c >= 0 ? c / m : -((m - 1 - c) / m);    // floor division
        c -= s * m;
      } else if (c < 0 || c >= m) {
        continue;
      }
      out.push_back({c, s, o == 0});
    }
  }
};

inline int64_t pack_image(int64_t t0, int64_t t1, int64_t t2)
{
  return ((t0 + kFarImages) << 42) | ((t1 + kFarImages) << 21) | (t2 + kFarImages);
}
inline void unpack_image(int64_t key, int64_t t[3])
{
  const int64_t mask = (int64_t(1) << 21) - 1;
  t[0] = ((key >> 42) & mask) - kFarImages;
  t[1] = ((key >> 21) & mask) - kFarImages;
  t[2] = (key & mask) - kFarImages;
}
// row of the shift table for an image difference: t0 a + t1 b + t2 c accumulated with fused multiply-adds from the
// first term on, the form the reference's optimised build evaluates, so that the table agrees to the last bit
inline void shift_row(const double *cell, const int64_t t[3], double *out)
{
  for (int d = 0; d < 3; d++) out[d] = std::fma((double) t[2], cell[6 + d], std::fma((double) t[1], cell[3 + d], (double) t[0] * cell[d]));
}

}    // namespace nl

inline NeighborList neighbor_search(const double *pos, int64_t n, const double *cell, const bool *pbc, double cutoff, int nthreads)
{
  if (!(cutoff > 0.0) || !std::isfinite(cutoff)) throw InvalidArgument("the neighbour search needs a cutoff: cutoff must be positive and finite");
  if (n < 0 || n >= INT32_MAX) throw InvalidArgument("the neighbour search handles fewer than 2^31 atoms");
  NeighborList out;
  out.offset.assign((size_t) n + 1, 0);
  if (n == 0) return out;
  const nl::Binned B(pos, n, cell, pbc, 0.5 * cutoff);
  out.perm = B.perm;
  const double cut2 = cutoff * cutoff;
  int64_t reach[3];
  for (int k = 0; k < 3; k++) reach[k] = B.grid.reach(cutoff, k, B.frame.periodic[k]);

  // every thread owns a contiguous range of slots and collects their rows in its own arrays
  const int threads = (int) std::max<int64_t>(1, std::min<int64_t>(nthreads, (n + 255) / 256));
  struct Part {
    std::vector<int32_t> j;
    std::vector<int64_t> key;
    bool far = false;
  };
  std::vector<Part> part((size_t) threads);
  std::vector<int64_t> row_len((size_t) n);
#pragma omp parallel num_threads(threads)
  {
#ifdef _OPENMP
    const int me = omp_get_thread_num(), team = omp_get_num_threads();
#else
    const int me = 0, team = 1;
#endif
    // with fewer threads than planned (team < threads) the ranges still cover every slot
    Part &mine = part[(size_t) me];
    std::vector<nl::Binned::Step> s0, s1, s2;
    for (int64_t q = n * me / team; q < n * (me + 1) / team; q++) {
      const double *xq = &B.x[3 * q];
      const int32_t *wq = &B.wrap3[3 * q];
      const size_t before = mine.j.size();
      B.steps(0, B.bin3[3 * q], reach[0], s0);
      B.steps(1, B.bin3[3 * q + 1], reach[1], s1);
      B.steps(2, B.bin3[3 * q + 2], reach[2], s2);
      for (const auto &a : s0)
        for (const auto &b : s1)
          for (const auto &c : s2) {
            const int64_t bin = (a.bin * B.grid.count[1] + b.bin) * B.grid.count[2] + c.bin;
            const double shift[3] = {B.frame.image_shift(a.image, b.image, c.image, 0), B.frame.image_shift(a.image, b.image, c.image, 1),
                                     B.frame.image_shift(a.image, b.image, c.image, 2)};
            const bool home = a.home && b.home && c.home;
            for (int64_t p = B.first[bin]; p < B.first[bin + 1]; p++) {
              if (home && p == q) continue;
              // order matters: (x_p + shift) - x_q, then the sum of squares from the first term on
              const double dx = B.x[3 * p] + shift[0] - xq[0], dy = B.x[3 * p + 1] + shift[1] - xq[1], dz = B.x[3 * p + 2] + shift[2] - xq[2];
              const double d2 = dx * dx + dy * dy + dz * dz;
              if (!(d2 < cut2)) continue;
              // image of the bond in the caller's frame: both atoms un-wrapped
              const int32_t *wp = &B.wrap3[3 * p];
              const int64_t t0 = a.image - wp[0] + wq[0], t1 = b.image - wp[1] + wq[1], t2 = c.image - wp[2] + wq[2];
              if (std::max({std::abs(t0), std::abs(t1), std::abs(t2)}) >= nl::kFarImages) mine.far = true;
              mine.j.push_back((int32_t) p);
              mine.key.push_back(nl::pack_image(t0, t1, t2));
            }
          }
      row_len[q] = (int64_t) (mine.j.size() - before);
    }
  }
  for (const Part &p : part)
    if (p.far) throw InvalidArgument("atoms a million cells or more apart: wrap the positions first");

  // rows: the parts are in slot order already
  for (int64_t q = 0; q < n; q++) out.offset[q + 1] = out.offset[q] + row_len[q];
  std::vector<int64_t> keys;
  for (const Part &p : part) {
    std::vector<int64_t> seen(p.key);
    std::sort(seen.begin(), seen.end());
    seen.erase(std::unique(seen.begin(), seen.end()), seen.end());
    keys.insert(keys.end(), seen.begin(), seen.end());
  }
  std::sort(keys.begin(), keys.end());
  keys.erase(std::unique(keys.begin(), keys.end()), keys.end());
  out.shifts.resize(3 * keys.size());
  for (size_t r = 0; r < keys.size(); r++) {
    int64_t t[3];
    nl::unpack_image(keys[r], t);
    nl::shift_row(cell, t, &out.shifts[3 * r]);
  }
  out.j.resize((size_t) out.offset[n]);
  out.image.resize((size_t) out.offset[n]);
  size_t at = 0;
  for (const Part &p : part) {
    std::copy(p.j.begin(), p.j.end(), out.j.begin() + (std::ptrdiff_t) at);
    int64_t last = -1;
    int32_t rank = 0;
    for (size_t w = 0; w < p.key.size(); w++) {
      if (p.key[w] != last) rank = (int32_t) (std::lower_bound(keys.begin(), keys.end(), last = p.key[w]) - keys.begin());
      out.image[at + w] = rank;
    }
    at += p.j.size();
  }
  return out;
}

}    // namespace grhip
