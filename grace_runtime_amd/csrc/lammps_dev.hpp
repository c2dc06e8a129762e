// The LAMMPS pair-style call with every per-atom array in device memory (the RunInput of the reference's GPU engines,
// libgrace/include/grace/kk/grace_1l_kk.h:80-103: x, f, type, ilist, numneigh and the 2-d neighbour view of a KOKKOS
// pair style).  The full neighbour list is turned into the engine's CSR list with bond vectors by two kernels (count,
// fill) without leaving the device; the owner map stands in for the exchange of the reference on one rank, with an
// exchange installed the ghosts stay atoms of their own.
#pragma once

#include "engine_common.hpp"

namespace grhip {

struct LmpListDev {
  const int *type;         // [nall] 1-based atom types
  const double *x;         // [nall][3]
  const int *numneigh;     // [nlocal], by atom
  const int *neighbors;    // element (i, k) at i stride_i + k stride_k
  long long stride_i, stride_k;
  const int *owner;        // [nall] owned atom of every ghost, or null
  const int *idx;          // [nlocal] engine row of an owned atom of a mapped type, else -1
  const int *atom;         // [n] owned atom of engine row q
  const unsigned char *mapped;    // [ntypes + 1] type has a model element
  int n, nlocal, nall, neighmask;
  int nodes;               // 1: ghosts are atoms of their own (an exchange moves their rows): a neighbour keeps its index
};

// FILL = false: count[q] = bonds of row q to atoms of mapped types; *err = 1: neighbour index outside the atoms,
// 2: a ghost without a usable owner.  FILL = true: j and rij of those bonds from offset[q] on, in list order.
template<bool FILL>
__global__ void k_lmp_rows(LmpListDev L, int *count, int *err, const long long *offset, int *j, double *rij)
{
  const int q = blockIdx.x * blockDim.x + threadIdx.x;
  if (q >= L.n) return;
  const int i = L.atom[q];
  const double xi0 = L.x[3 * (long long) i], xi1 = L.x[3 * (long long) i + 1], xi2 = L.x[3 * (long long) i + 2];
  const int nn = L.numneigh[i];
  const int *row = L.neighbors + i * L.stride_i;
  long long w = FILL ? offset[q] : 0;
  int c = 0;
  for (int k = 0; k < nn; k++) {
    const int a = row[k * L.stride_k] & L.neighmask;
    if (a < 0 || a >= L.nall) {
      if (!FILL) *err = 1;
      continue;
    }
    const int ta = L.type[a];
    if (!L.mapped[ta]) continue;
    int o = a;
    if (!L.nodes) {
      if (a >= L.nlocal) o = L.owner ? L.owner[a] : -1;
      if (o < 0 || o >= L.nlocal || L.idx[o] < 0 || L.type[o] != ta) {
        if (!FILL) *err = 2;
        continue;
      }
      o = L.idx[o];
    }
    if (FILL) {
      j[w] = o;
      rij[3 * w] = L.x[3 * (long long) a] - xi0;
      rij[3 * w + 1] = L.x[3 * (long long) a + 1] - xi1;
      rij[3 * w + 2] = L.x[3 * (long long) a + 2] - xi2;
      w++;
    } else {
      c++;
    }
  }
  if (!FILL) count[q] = c;
}

// buffers of the converted list, kept between calls
struct LammpsDeviceList {
  DevBuf idx, atom, mapped, count, err, offset, j, rij;
  int64_t nb = 0;
  // what the kept list was made for: a call that says "same list" and matches it only renews the bond vectors
  bool kept = false;
  int n = 0, nlocal = 0, nall = 0, inum = 0, nodes = 0, neighmask = 0;
  long long stride_i = 0, stride_k = 0;
  const void *neighbors = nullptr, *type = nullptr, *numneigh = nullptr, *owner = nullptr;
  uint64_t serial = 0;
};

}    // namespace grhip
