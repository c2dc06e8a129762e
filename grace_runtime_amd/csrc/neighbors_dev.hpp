// Neighbour list built on the GPU: wrap, bin, sort into bins, count, scan and fill all run as kernels; the host sizes the
// grid from twelve reduced numbers and ranks the image differences that occur (a table of at most 2^20 entries).
// The list equals the host list of neighbors.hpp, and with it the reference's list (libgrace/include/grace/
// cell_list.h:39-152,216-241, python/src/neighbors.cpp:15-95; its own device list is libgrace/include/grace/kk/
// neighbors_kk.h), bond for bond: atoms in bin order with a bin's atoms in input order, a row's bonds by ascending bin
// offset and slot.  The kernels evaluate the deciding expressions (fractional coordinate, bin index, wrapped position,
// squared distance) without floating-point contraction and in the host code's operation order.
#pragma once

#include "engine_common.hpp"
#include "neighbors.hpp"

namespace grhip {

struct NlGrid {
  int n;
  int count[3], reach[3], periodic[3];
  double a[9], inv[9], origin[3], extent[3], cut2;
  int tmin[3], tdim[3];    // table of image differences t: index ((t0 - tmin0) tdim1 + t1 - tmin1) tdim2 + t2 - tmin2
};

constexpr int kNlBlock = 256;

// fractional coordinates u (wrapped along periodic directions) and the wrap of every atom; per block the smallest and
// largest u and wrap per direction and whether a coordinate was not finite: [block][13] doubles
static __global__ void k_nl_wrap(NlGrid G, const double *pos, double *u, int *wrap, double *partial)
{
#pragma clang fp contract(off)
  __shared__ double red[kNlBlock];
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  double v[13];
  for (int k = 0; k < 3; k++) {
    v[k] = v[6 + k] = 1e300;
    v[3 + k] = v[9 + k] = -1e300;
  }
  v[12] = 0.0;
  if (i < G.n) {
    const double x = pos[3 * i], y = pos[3 * i + 1], z = pos[3 * i + 2];
    for (int k = 0; k < 3; k++) {
      const double f = x * G.inv[k] + y * G.inv[3 + k] + z * G.inv[6 + k];
      const bool finite = f - f == 0.0;
      const double whole = G.periodic[k] && finite ? floor(f) : 0.0;
      const double w = fabs(whole) < 2e9 ? whole : 0.0;
      u[3 * i + k] = f - whole;
      wrap[3 * i + k] = (int) w;
      if (!finite || fabs(whole) >= 1073741824.0) v[12] = 1.0;
      v[k] = v[3 + k] = f - whole;
      v[6 + k] = v[9 + k] = w;
    }
  }
  for (int c = 0; c < 13; c++) {
    const bool smallest = c < 3 || (c >= 6 && c < 9);
    red[threadIdx.x] = v[c];
    __syncthreads();
    for (int o = kNlBlock / 2; o > 0; o >>= 1) {
      if ((int) threadIdx.x < o) {
        const double p = red[threadIdx.x], q = red[threadIdx.x + o];
        red[threadIdx.x] = smallest ? (q < p ? q : p) : (q > p ? q : p);
      }
      __syncthreads();
    }
    if (threadIdx.x == 0) partial[13 * blockIdx.x + c] = red[0];
    __syncthreads();
  }
}

__device__ inline int nl_bin_along(const NlGrid &G, double u, int k)
{
#pragma clang fp contract(off)
  const double b = floor((u - G.origin[k]) / G.extent[k] * (double) G.count[k]);
  return b < 0.0 ? 0 : b > (double) (G.count[k] - 1) ? G.count[k] - 1 : (int) b;
}

// bin of every atom and the population of every bin
static __global__ void k_nl_bin(NlGrid G, const double *u, int *bin, int *population)
{
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= G.n) return;
  const int b = (nl_bin_along(G, u[3 * i], 0) * G.count[1] + nl_bin_along(G, u[3 * i + 1], 1)) * G.count[2] + nl_bin_along(G, u[3 * i + 2], 2);
  bin[i] = b;
  atomicAdd(&population[b], 1);
}
// atoms into the slots of their bin, in whatever order the atomics give ...
static __global__ void k_nl_scatter(int n, const int *bin, const long long *first, int *cursor, int *slot_atom)
{
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int b = bin[i];
  slot_atom[first[b] + atomicAdd(&cursor[b], 1)] = i;
}
// ... and every bin's atoms into ascending order (bins hold a handful of atoms: insertion sort by one thread)
static __global__ void k_nl_order_bins(int nbins, const long long *first, int *slot_atom)
{
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= nbins) return;
  const long long lo = first[b], hi = first[b + 1];
  for (long long q = lo + 1; q < hi; q++) {
    const int a = slot_atom[q];
    long long w = q;
    while (w > lo && slot_atom[w - 1] > a) {
      slot_atom[w] = slot_atom[w - 1];
      w--;
    }
    slot_atom[w] = a;
  }
}
// per slot: wrapped Cartesian position, bin triple and wrap of its atom
static __global__ void k_nl_place(NlGrid G, const int *slot_atom, const double *u, const int *wrap, double *x, int *bin3, int *wrap3)
{
#pragma clang fp contract(off)
  const int q = blockIdx.x * blockDim.x + threadIdx.x;
  if (q >= G.n) return;
  const int i = slot_atom[q];
  const double u0 = u[3 * i], u1 = u[3 * i + 1], u2 = u[3 * i + 2];
  for (int d = 0; d < 3; d++) {
    x[3 * q + d] = u0 * G.a[d] + u1 * G.a[3 + d] + u2 * G.a[6 + d];
    wrap3[3 * q + d] = wrap[3 * i + d];
  }
  bin3[3 * q] = nl_bin_along(G, u0, 0);
  bin3[3 * q + 1] = nl_bin_along(G, u1, 1);
  bin3[3 * q + 2] = nl_bin_along(G, u2, 2);
}

__device__ inline int nl_fold(int c, int m, int &image)
{
  image = c >= 0 ? c / m : -((m - 1 - c) / m);
  return c - image * m;
}

// FILL = false: count[q] = neighbours of slot q, present[t] = 1 for every image difference met;
// FILL = true: j and image of the bonds of slot q from offset[q] on, image = rank[t]
template<bool FILL>
__global__ void k_nl_pairs(NlGrid G, const double *x, const int *bin3, const int *wrap3, const long long *first, int *count,
                           unsigned char *present, const long long *offset, const int *rank, int *j, int *image)
{
#pragma clang fp contract(off)
  const int q = blockIdx.x * blockDim.x + threadIdx.x;
  if (q >= G.n) return;
  const double xq0 = x[3 * q], xq1 = x[3 * q + 1], xq2 = x[3 * q + 2];
  const int w0 = wrap3[3 * q], w1 = wrap3[3 * q + 1], w2 = wrap3[3 * q + 2];
  int found = 0;
  long long at = FILL ? offset[q] : 0;
  for (int o0 = -G.reach[0]; o0 <= G.reach[0]; o0++) {
    int s0 = 0, c0 = bin3[3 * q] + o0;
    if (G.periodic[0]) c0 = nl_fold(c0, G.count[0], s0);
    else if (c0 < 0 || c0 >= G.count[0]) continue;
    for (int o1 = -G.reach[1]; o1 <= G.reach[1]; o1++) {
      int s1 = 0, c1 = bin3[3 * q + 1] + o1;
      if (G.periodic[1]) c1 = nl_fold(c1, G.count[1], s1);
      else if (c1 < 0 || c1 >= G.count[1]) continue;
      for (int o2 = -G.reach[2]; o2 <= G.reach[2]; o2++) {
        int s2 = 0, c2 = bin3[3 * q + 2] + o2;
        if (G.periodic[2]) c2 = nl_fold(c2, G.count[2], s2);
        else if (c2 < 0 || c2 >= G.count[2]) continue;
        const int b = (c0 * G.count[1] + c1) * G.count[2] + c2;
        const double sx = s0 * G.a[0] + s1 * G.a[3] + s2 * G.a[6];
        const double sy = s0 * G.a[1] + s1 * G.a[4] + s2 * G.a[7];
        const double sz = s0 * G.a[2] + s1 * G.a[5] + s2 * G.a[8];
        const bool home = o0 == 0 && o1 == 0 && o2 == 0;
        for (long long p = first[b]; p < first[b + 1]; p++) {
          if (home && p == q) continue;
          const double dx = x[3 * p] + sx - xq0, dy = x[3 * p + 1] + sy - xq1, dz = x[3 * p + 2] + sz - xq2;
          const double d2 = dx * dx + dy * dy + dz * dz;
          if (!(d2 < G.cut2)) continue;
          const int t0 = s0 - wrap3[3 * p] + w0, t1 = s1 - wrap3[3 * p + 1] + w1, t2 = s2 - wrap3[3 * p + 2] + w2;
          const int t = ((t0 - G.tmin[0]) * G.tdim[1] + (t1 - G.tmin[1])) * G.tdim[2] + (t2 - G.tmin[2]);
          if (FILL) {
            j[at] = (int) p;
            image[at] = rank[t];
            at++;
          } else {
            found++;
            present[t] = 1;
          }
        }
      }
    }
  }
  if (!FILL) count[q] = found;
}

// x[q] = pos[perm[q]]
static __global__ void k_nl_gather(const double *pos, const int *perm, double *x, int n)
{
  const int q = blockIdx.x * blockDim.x + threadIdx.x;
  if (q >= n) return;
  const int a = perm[q];
  x[3 * q] = pos[3 * a];
  x[3 * q + 1] = pos[3 * a + 1];
  x[3 * q + 2] = pos[3 * a + 2];
}

// The list of one structure in device memory (perm and the shift table also on the host).
class DeviceNeighbors {
 public:
  std::vector<int64_t> perm;       // slot -> atom
  std::vector<double> shifts;      // [nimages][3]
  int64_t nb = 0;
  DevBuf offset, j, image;         // [n + 1] i64, [nb] i32, [nb] i32
  // false: the structure does not fit the device tables (atoms thousands of cells apart, more than 2^31 bins) and the
  // caller falls back to the host list
  bool build(const double *pos, int64_t n, const double *cell, const bool *pbc, double cutoff, hipStream_t stream)
  {
    if (!(cutoff > 0.0) || !std::isfinite(cutoff)) throw InvalidArgument("the neighbour search needs a cutoff: cutoff must be positive and finite");
    if (n < 0 || n >= INT32_MAX) throw InvalidArgument("the neighbour search handles fewer than 2^31 atoms");
    perm.clear();
    shifts.clear();
    nb = 0;
    offset.ensure(sizeof(long long) * (size_t) (n + 1));
    if (n == 0) {
      const long long z = 0;
      HIP_CHECK(hipMemcpy(offset.p, &z, sizeof(z), hipMemcpyHostToDevice));
      return true;
    }
    const nl::Frame frame(cell, pbc);
    NlGrid G{};
    G.n = (int) n;
    G.cut2 = cutoff * cutoff;
    for (int k = 0; k < 9; k++) {
      G.a[k] = frame.a[k];
      G.inv[k] = frame.inv[k];
    }
    for (int k = 0; k < 3; k++) G.periodic[k] = frame.periodic[k] ? 1 : 0;
    const unsigned blocks = (unsigned) ((n + kNlBlock - 1) / kNlBlock);
    const size_t n3 = (size_t) 3 * n;
    pos_.ensure(n3 * sizeof(double)); u_.ensure(n3 * sizeof(double)); wrap_.ensure(n3 * sizeof(int));
    partial_.ensure((size_t) blocks * 13 * sizeof(double));
    HIP_CHECK(hipMemcpyAsync(pos_.p, pos, n3 * sizeof(double), hipMemcpyHostToDevice, stream));
    hipLaunchKernelGGL(k_nl_wrap, dim3(blocks), dim3(kNlBlock), 0, stream, G, pos_.as<double>(), u_.as<double>(), wrap_.as<int>(), partial_.as<double>());
    std::vector<double> part((size_t) blocks * 13);
    HIP_CHECK(hipMemcpyAsync(part.data(), partial_.p, part.size() * sizeof(double), hipMemcpyDeviceToHost, stream));
    HIP_CHECK(hipStreamSynchronize(stream));
    double lo[3], hi[3], wlo[3], whi[3];
    for (int k = 0; k < 3; k++) {
      lo[k] = part[k]; hi[k] = part[3 + k]; wlo[k] = part[6 + k]; whi[k] = part[9 + k];
    }
    for (unsigned b = 0; b < blocks; b++) {
      if (part[13 * (size_t) b + 12] != 0.0) {
        for (int64_t i = 0; i < n; i++)
          for (int d = 0; d < 3; d++)
            if (!std::isfinite(pos[3 * i + d])) throw InvalidArgument("atom " + std::to_string(i) + " has a position that is not finite");
        return false;    // finite, but a million cells from the cell: the host search reports it
      }
      for (int k = 0; k < 3; k++) {
        lo[k] = std::min(lo[k], part[13 * (size_t) b + k]); hi[k] = std::max(hi[k], part[13 * (size_t) b + 3 + k]);
        wlo[k] = std::min(wlo[k], part[13 * (size_t) b + 6 + k]); whi[k] = std::max(whi[k], part[13 * (size_t) b + 9 + k]);
      }
    }
    nl::Grid grid;
    grid.choose(frame, lo, hi, n, 0.5 * cutoff);
    const int64_t nbins = grid.total();
    if (nbins >= INT32_MAX / 2) return false;
    for (int k = 0; k < 3; k++) {
      G.count[k] = (int) grid.count[k];
      G.origin[k] = grid.origin[k];
      G.extent[k] = grid.extent[k];
      G.reach[k] = (int) grid.reach(cutoff, k, frame.periodic[k]);
      // image differences that can occur: the images the bin walk reaches, shifted by the spread of the atoms' wraps
      const int64_t spread = (int64_t) (whi[k] - wlo[k]);
      if (spread >= (int64_t(1) << 19)) return false;
      const int64_t m = grid.count[k];
      const int64_t smin = frame.periodic[k] ? -((m - 1 + G.reach[k]) / m) : 0, smax = frame.periodic[k] ? (m - 1 + G.reach[k]) / m : 0;
      G.tmin[k] = (int) (smin - spread);
      G.tdim[k] = (int) (smax + spread - G.tmin[k] + 1);
    }
    const int64_t tsize = (int64_t) G.tdim[0] * G.tdim[1] * G.tdim[2];
    if (tsize > (int64_t(1) << 20)) return false;

    // ---- atoms into bins
    bin_.ensure((size_t) n * sizeof(int)); slot_atom_.ensure((size_t) n * sizeof(int));
    population_.ensure((size_t) nbins * sizeof(int)); cursor_.ensure((size_t) nbins * sizeof(int)); first_.ensure((size_t) (nbins + 1) * sizeof(long long));
    x_.ensure(n3 * sizeof(double)); bin3_.ensure(n3 * sizeof(int)); wrap3_.ensure(n3 * sizeof(int));
    HIP_CHECK(hipMemsetAsync(population_.p, 0, (size_t) nbins * sizeof(int), stream));
    HIP_CHECK(hipMemsetAsync(cursor_.p, 0, (size_t) nbins * sizeof(int), stream));
    hipLaunchKernelGGL(k_nl_bin, dim3(blocks), dim3(kNlBlock), 0, stream, G, u_.as<double>(), bin_.as<int>(), population_.as<int>());
    hipLaunchKernelGGL(k_scan, dim3(1), dim3(1024), 0, stream, population_.as<int>(), (int) nbins, first_.as<long long>());
    hipLaunchKernelGGL(k_nl_scatter, dim3(blocks), dim3(kNlBlock), 0, stream, (int) n, bin_.as<int>(), first_.as<long long>(), cursor_.as<int>(),
                       slot_atom_.as<int>());
    hipLaunchKernelGGL(k_nl_order_bins, dim3((unsigned) ((nbins + kNlBlock - 1) / kNlBlock)), dim3(kNlBlock), 0, stream, (int) nbins, first_.as<long long>(),
                       slot_atom_.as<int>());
    hipLaunchKernelGGL(k_nl_place, dim3(blocks), dim3(kNlBlock), 0, stream, G, slot_atom_.as<int>(), u_.as<double>(), wrap_.as<int>(), x_.as<double>(),
                       bin3_.as<int>(), wrap3_.as<int>());
    std::vector<int> perm32((size_t) n);
    HIP_CHECK(hipMemcpyAsync(perm32.data(), slot_atom_.p, (size_t) n * sizeof(int), hipMemcpyDeviceToHost, stream));

    // ---- pairs: count, scan, rank the image differences met, fill
    count_.ensure(sizeof(int) * (size_t) n);
    present_.ensure((size_t) tsize);
    rank_.ensure(sizeof(int) * (size_t) tsize);
    HIP_CHECK(hipMemsetAsync(present_.p, 0, (size_t) tsize, stream));
    const dim3 grid64((unsigned) ((n + 63) / 64)), block64(64);
    hipLaunchKernelGGL(k_nl_pairs<false>, grid64, block64, 0, stream, G, x_.as<double>(), bin3_.as<int>(), wrap3_.as<int>(), first_.as<long long>(),
                       count_.as<int>(), present_.as<unsigned char>(), (const long long *) nullptr, (const int *) nullptr, (int *) nullptr, (int *) nullptr);
    hipLaunchKernelGGL(k_scan, dim3(1), dim3(1024), 0, stream, count_.as<int>(), (int) n, offset.as<long long>());
    std::vector<unsigned char> met((size_t) tsize);
    long long total = 0;
    HIP_CHECK(hipMemcpyAsync(met.data(), present_.p, (size_t) tsize, hipMemcpyDeviceToHost, stream));
    HIP_CHECK(hipMemcpyAsync(&total, offset.as<long long>() + n, sizeof(total), hipMemcpyDeviceToHost, stream));
    HIP_CHECK(hipGetLastError());
    HIP_CHECK(hipStreamSynchronize(stream));
    nb = total;
    perm.assign(perm32.begin(), perm32.end());
    // the table index ascends with (t0, t1, t2), which is the order of the shift table
    std::vector<int> rank((size_t) tsize, -1);
    int rows = 0;
    for (int64_t t = 0; t < tsize; t++) {
      if (!met[(size_t) t]) continue;
      rank[(size_t) t] = rows++;
      const int64_t tt[3] = {t / ((int64_t) G.tdim[2] * G.tdim[1]) + G.tmin[0], (t / G.tdim[2]) % G.tdim[1] + G.tmin[1], t % G.tdim[2] + G.tmin[2]};
      if (std::max({std::abs(tt[0]), std::abs(tt[1]), std::abs(tt[2])}) >= nl::kFarImages)
        throw InvalidArgument("atoms a million cells or more apart: wrap the positions first");
      shifts.resize(shifts.size() + 3);
      nl::shift_row(cell, tt, &shifts[shifts.size() - 3]);
    }
    HIP_CHECK(hipMemcpyAsync(rank_.p, rank.data(), sizeof(int) * (size_t) tsize, hipMemcpyHostToDevice, stream));
    j.ensure(sizeof(int) * (size_t) std::max<int64_t>(nb, 1));
    image.ensure(sizeof(int) * (size_t) std::max<int64_t>(nb, 1));
    hipLaunchKernelGGL(k_nl_pairs<true>, grid64, block64, 0, stream, G, x_.as<double>(), bin3_.as<int>(), wrap3_.as<int>(), first_.as<long long>(),
                       (int *) nullptr, (unsigned char *) nullptr, (const long long *) offset.as<long long>(), (const int *) rank_.as<int>(), j.as<int>(),
                       image.as<int>());
    HIP_CHECK(hipGetLastError());
    HIP_CHECK(hipStreamSynchronize(stream));    // the host staging vectors go out of scope
    return true;
  }
  const int *perm_dev() const { return slot_atom_.as<int>(); }

 private:
  DevBuf pos_, u_, wrap_, partial_, bin_, slot_atom_, population_, cursor_, first_, x_, bin3_, wrap3_, count_, present_, rank_;
};

}    // namespace grhip
