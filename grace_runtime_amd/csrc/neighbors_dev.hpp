// Neighbour list with the pair search on the GPU.  The binning of the atoms (fractional coordinates, wrap, stable
// counting sort by bin: O(n)) is the host code of neighbors.hpp, so the permutation and the wrapped coordinates are
// the reference's by construction; the O(n x neighbours) part -- per atom the bins in lexicographic offset order, inside
// a bin by slot, r^2 < rc^2 -- runs on the device, one thread per atom, in two passes (count, fill).  The distance
// expressions are compiled without floating-point contraction and in the operation order of the host code, so the list
// (offset, j, image, shift table) equals the host list, and with it the reference list
// (libgrace/include/grace/cell_list.h:39-152,216-241, python/src/neighbors.cpp:15-95), bond for bond.
// The reference's own device list is libgrace/include/grace/kk/neighbors_kk.h.
#pragma once

#include "engine_common.hpp"
#include "neighbors.hpp"

namespace grhip {

struct NlDev {
  int n;
  int nbin[3], reach[3], pbc[3];
  double cell[9], rc2;
  const double *xw;      // [n][3] wrapped coordinates, slot order
  const int *b3;         // [n][3] bin of the atom in slot q
  const int *img;        // [n][3] image of the atom in slot q (floor of its fractional coordinates)
  const int *start;      // [nbins + 1]
  int tmin[3], tdim[3];  // table of the image differences t = s - img_b + img_a: index ((t0 - tmin0) T1 + t1 - tmin1) T2 + t2 - tmin2
};

__device__ inline int nl_floordiv(int a, int b) { return a >= 0 ? a / b : -((-a + b - 1) / b); }

// FILL = false: count[q] = neighbours of slot q, present[t] = 1 for every image difference met;
// FILL = true: j and image of the bonds of slot q from offset[q] on, image = rank[t]
template<bool FILL>
__global__ void k_nl_pairs(NlDev A, int *count, unsigned char *present, const long long *offset, const int *rank, int *j, int *image)
{
#pragma clang fp contract(off)
  const int q = blockIdx.x * blockDim.x + threadIdx.x;
  if (q >= A.n) return;
  const double xq0 = A.xw[3 * q], xq1 = A.xw[3 * q + 1], xq2 = A.xw[3 * q + 2];
  const int b0 = A.b3[3 * q], b1 = A.b3[3 * q + 1], b2 = A.b3[3 * q + 2];
  const int i0 = A.img[3 * q], i1 = A.img[3 * q + 1], i2 = A.img[3 * q + 2];
  int c = 0;
  long long w = FILL ? offset[q] : 0;
  for (int o0 = -A.reach[0]; o0 <= A.reach[0]; o0++) {
    int c0 = b0 + o0, s0 = 0;
    if (A.pbc[0]) { s0 = nl_floordiv(c0, A.nbin[0]); c0 -= s0 * A.nbin[0]; }
    else if (c0 < 0 || c0 >= A.nbin[0]) continue;
    for (int o1 = -A.reach[1]; o1 <= A.reach[1]; o1++) {
      int c1 = b1 + o1, s1 = 0;
      if (A.pbc[1]) { s1 = nl_floordiv(c1, A.nbin[1]); c1 -= s1 * A.nbin[1]; }
      else if (c1 < 0 || c1 >= A.nbin[1]) continue;
      for (int o2 = -A.reach[2]; o2 <= A.reach[2]; o2++) {
        int c2 = b2 + o2, s2 = 0;
        if (A.pbc[2]) { s2 = nl_floordiv(c2, A.nbin[2]); c2 -= s2 * A.nbin[2]; }
        else if (c2 < 0 || c2 >= A.nbin[2]) continue;
        const int cb = (c0 * A.nbin[1] + c1) * A.nbin[2] + c2;
        const double sx = s0 * A.cell[0] + s1 * A.cell[3] + s2 * A.cell[6];
        const double sy = s0 * A.cell[1] + s1 * A.cell[4] + s2 * A.cell[7];
        const double sz = s0 * A.cell[2] + s1 * A.cell[5] + s2 * A.cell[8];
        const bool own = o0 == 0 && o1 == 0 && o2 == 0;
        for (int p = A.start[cb]; p < A.start[cb + 1]; p++) {
          if (own && p == q) continue;
          const double dx = A.xw[3 * p] + sx - xq0;
          const double dy = A.xw[3 * p + 1] + sy - xq1;
          const double dz = A.xw[3 * p + 2] + sz - xq2;
          const double r2 = dx * dx + dy * dy + dz * dz;
          if (!(r2 < A.rc2)) continue;
          const int t0 = s0 - A.img[3 * p] + i0, t1 = s1 - A.img[3 * p + 1] + i1, t2 = s2 - A.img[3 * p + 2] + i2;
          const int t = ((t0 - A.tmin[0]) * A.tdim[1] + (t1 - A.tmin[1])) * A.tdim[2] + (t2 - A.tmin[2]);
          if (FILL) {
            j[w] = p;
            image[w] = rank[t];
            w++;
          } else {
            c++;
            present[t] = 1;
          }
        }
      }
    }
  }
  if (!FILL) count[q] = c;
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
  // false: the image differences of this structure do not fit the device table (atoms thousands of cells apart) --
  // the caller falls back to the host list
  bool build(const double *pos, int64_t n, const double *cell, const bool *pbc, double cutoff, hipStream_t stream)
  {
    using namespace nl_detail;
    if (!(cutoff > 0.0) || !std::isfinite(cutoff)) throw InvalidArgument("cutoff must be positive");
    if (n < 0 || n >= INT32_MAX) throw InvalidArgument("atom count out of range");
    perm.clear();
    shifts.clear();
    nb = 0;
    offset.ensure(sizeof(long long) * (size_t) (n + 1));
    if (n == 0) {
      const long long z = 0;
      HIP_CHECK(hipMemcpy(offset.p, &z, sizeof(z), hipMemcpyHostToDevice));
      return true;
    }
    Cells cl;
    cl.build(pos, n, cell, pbc, 0.5 * cutoff);
    perm = cl.perm;
    NlDev A{};
    A.n = (int) n;
    A.rc2 = cutoff * cutoff;
    int64_t nbt = 1;
    int imin[3], imax[3];
    for (int k = 0; k < 3; k++) {
      if (cl.nbin[k] > INT32_MAX / 4) return false;
      A.nbin[k] = (int) cl.nbin[k];
      A.reach[k] = (int) bin_reach(cutoff, cl.width[k], cl.nbin[k], cl.pbc[k]);
      A.pbc[k] = cl.pbc[k] ? 1 : 0;
      nbt *= cl.nbin[k];
      int64_t lo = cl.img[k], hi = cl.img[k];
      for (int64_t i = 1; i < n; i++) {
        lo = std::min(lo, cl.img[3 * i + k]);
        hi = std::max(hi, cl.img[3 * i + k]);
      }
      if (hi - lo >= (int64_t(1) << 19) || std::abs(lo) >= (int64_t(1) << 30) || std::abs(hi) >= (int64_t(1) << 30)) return false;
      imin[k] = (int) lo;
      imax[k] = (int) hi;
      const int64_t smin = cl.pbc[k] ? floordiv(-A.reach[k], cl.nbin[k]) : 0, smax = cl.pbc[k] ? floordiv(cl.nbin[k] - 1 + A.reach[k], cl.nbin[k]) : 0;
      A.tmin[k] = (int) (smin - (imax[k] - imin[k]));
      A.tdim[k] = (int) (smax + (imax[k] - imin[k]) - A.tmin[k] + 1);
    }
    for (int k = 0; k < 9; k++) A.cell[k] = cl.cell[k];
    const int64_t tsize = (int64_t) A.tdim[0] * A.tdim[1] * A.tdim[2];
    if (tsize > (int64_t(1) << 20) || nbt >= INT32_MAX) return false;
    std::vector<int> b3s((size_t) 3 * n), imgs((size_t) 3 * n), st((size_t) nbt + 1), perm32((size_t) n);
    for (int64_t q = 0; q < n; q++) {
      const int64_t a = cl.perm[q];
      perm32[q] = (int) a;
      for (int k = 0; k < 3; k++) {
        b3s[3 * q + k] = (int) cl.b3[3 * a + k];
        imgs[3 * q + k] = (int) cl.img[3 * a + k];
      }
    }
    for (int64_t b = 0; b <= nbt; b++) st[b] = (int) cl.start[b];
    auto put = [&](DevBuf &b, const void *src, size_t bytes) {
      b.ensure(std::max<size_t>(bytes, 8));
      HIP_CHECK(hipMemcpyAsync(b.p, src, bytes, hipMemcpyHostToDevice, stream));
    };
    put(xw_, cl.xw.data(), sizeof(double) * 3 * n);
    put(b3_, b3s.data(), sizeof(int) * 3 * n);
    put(img_, imgs.data(), sizeof(int) * 3 * n);
    put(start_, st.data(), sizeof(int) * (nbt + 1));
    put(perm_, perm32.data(), sizeof(int) * n);
    count_.ensure(sizeof(int) * n);
    present_.ensure((size_t) tsize);
    rank_.ensure(sizeof(int) * (size_t) tsize);
    HIP_CHECK(hipMemsetAsync(present_.p, 0, (size_t) tsize, stream));
    A.xw = xw_.as<double>(); A.b3 = b3_.as<int>(); A.img = img_.as<int>(); A.start = start_.as<int>();
    const dim3 grid((unsigned) ((n + 63) / 64)), block(64);
    hipLaunchKernelGGL(k_nl_pairs<false>, grid, block, 0, stream, A, count_.as<int>(), present_.as<unsigned char>(), (const long long *) nullptr,
                       (const int *) nullptr, (int *) nullptr, (int *) nullptr);
    hipLaunchKernelGGL(k_scan, dim3(1), dim3(1024), 0, stream, count_.as<int>(), (int) n, offset.as<long long>());
    std::vector<unsigned char> pres((size_t) tsize);
    long long total = 0;
    HIP_CHECK(hipMemcpyAsync(pres.data(), present_.p, (size_t) tsize, hipMemcpyDeviceToHost, stream));
    HIP_CHECK(hipMemcpyAsync(&total, offset.as<long long>() + n, sizeof(total), hipMemcpyDeviceToHost, stream));
    HIP_CHECK(hipStreamSynchronize(stream));
    nb = total;
    // shift table: the distinct image differences in the order of the reference's packed keys = lexicographic (t0, t1, t2)
    std::vector<int> rank((size_t) tsize, -1);
    int u = 0;
    for (int64_t t = 0; t < tsize; t++) {
      if (!pres[t]) continue;
      rank[t] = u++;
      const int t2 = (int) (t % A.tdim[2]) + A.tmin[2], t1 = (int) ((t / A.tdim[2]) % A.tdim[1]) + A.tmin[1],
                t0 = (int) (t / ((int64_t) A.tdim[2] * A.tdim[1])) + A.tmin[0];
      if (std::max({std::abs(t0), std::abs(t1), std::abs(t2)}) >= (1 << 20))
        throw InvalidArgument("atoms a million cells or more apart: wrap the positions");
      for (int d = 0; d < 3; d++)
        shifts.push_back(std::fma((double) t2, cell[6 + d], std::fma((double) t1, cell[3 + d], (double) t0 * cell[d])));
    }
    put(rank_, rank.data(), sizeof(int) * (size_t) tsize);
    j.ensure(sizeof(int) * (size_t) std::max<int64_t>(nb, 1));
    image.ensure(sizeof(int) * (size_t) std::max<int64_t>(nb, 1));
    hipLaunchKernelGGL(k_nl_pairs<true>, grid, block, 0, stream, A, (int *) nullptr, (unsigned char *) nullptr, (const long long *) offset.as<long long>(),
                       (const int *) rank_.as<int>(), j.as<int>(), image.as<int>());
    HIP_CHECK(hipStreamSynchronize(stream));    // the host staging vectors go out of scope
    return true;
  }
  const int *perm_dev() const { return perm_.as<int>(); }

 private:
  DevBuf xw_, b3_, img_, start_, perm_, count_, present_, rank_;
};

}    // namespace grhip
