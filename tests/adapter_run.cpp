// A pair style's use of the C++ adapter (include/grace_hip_lammps.hpp), driven by the tests: reads one rank's arrays from a
// file, puts them in device memory, runs two passes (the second with same_list after moving x) and prints the results.
//   adapter_run model.npz input.bin  ->  "energy virial[6]" then nall lines "fx fy fz eatom", once per pass
#include <hip/hip_runtime_api.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

#include "grace_hip_lammps.hpp"

template<class T> static std::vector<T> take(FILE *f, size_t n)
{
  std::vector<T> v(n);
  if (n && fread(v.data(), sizeof(T), n, f) != n) { fprintf(stderr, "short input\n"); exit(2); }
  return v;
}
template<class T> static T *to_device(const std::vector<T> &v)
{
  void *p = nullptr;
  if (hipMalloc(&p, v.size() * sizeof(T) + 8) != hipSuccess || hipMemcpy(p, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice) != hipSuccess) {
    fprintf(stderr, "device copy failed\n");
    exit(2);
  }
  return (T *) p;
}

int main(int argc, char **argv)
{
  if (argc != 3) return 2;
  FILE *f = fopen(argv[2], "rb");
  if (!f) return 2;
  const std::vector<int> head = take<int>(f, 4);    // nlocal, nall, maxneigh, ntypes
  const int nlocal = head[0], nall = head[1], maxn = head[2], ntypes = head[3];
  const std::vector<int> type2mu = take<int>(f, ntypes + 1), type = take<int>(f, nall), numneigh = take<int>(f, nlocal),
                         neigh = take<int>(f, (size_t) nlocal * maxn), owner = take<int>(f, nall);
  std::vector<double> x = take<double>(f, 3 * (size_t) nall), dx = take<double>(f, 3 * (size_t) nall);
  fclose(f);
  std::vector<int> ilist(nlocal);
  for (int i = 0; i < nlocal; i++) ilist[i] = i;
  try {
    grace_hip::Engine eng;
    eng.set_model(argv[1], type2mu);
    eng.setup();
    grace_hip::RunInput in;
    double *d_x = to_device(x);
    in.x = d_x;
    in.f = to_device(std::vector<double>(3 * (size_t) nall, 0.0));
    in.eatom = to_device(std::vector<double>(nall, 0.0));
    in.type = to_device(type);
    in.ilist = to_device(ilist);
    in.numneigh = to_device(numneigh);
    in.neighbors = to_device(neigh);
    in.stride_i = maxn;
    in.owner = to_device(owner);
    in.inum = in.nlocal = nlocal;
    in.nall = nall;
    in.ntypes = ntypes;
    in.eflag_atom = 1;
    for (int pass = 0; pass < 2; pass++) {
      if (pass == 1) {
        for (size_t k = 0; k < x.size(); k++) x[k] += dx[k];
        if (hipMemcpy(d_x, x.data(), x.size() * sizeof(double), hipMemcpyHostToDevice) != hipSuccess) return 2;
        if (hipMemset(in.f, 0, 3 * (size_t) nall * sizeof(double)) != hipSuccess || hipMemset(in.eatom, 0, nall * sizeof(double)) != hipSuccess) return 2;
        in.same_list = true;
      }
      const grace_hip::RunOutput out = eng.run(in);
      std::vector<double> fo(3 * (size_t) nall), ea(nall);
      if (hipMemcpy(fo.data(), in.f, fo.size() * sizeof(double), hipMemcpyDeviceToHost) != hipSuccess ||
          hipMemcpy(ea.data(), in.eatom, ea.size() * sizeof(double), hipMemcpyDeviceToHost) != hipSuccess)
        return 2;
      printf("%.17g", out.eng_vdwl);
      for (int k = 0; k < 6; k++) printf(" %.17g", out.virial[k]);
      printf("\n");
      for (int a = 0; a < nall; a++) printf("%.17g %.17g %.17g %.17g\n", fo[3 * a], fo[3 * a + 1], fo[3 * a + 2], ea[a]);
    }
    printf("cutoff %.17g chunk %d layers %d\n", eng.cutoff(1, 1), eng.auto_chunk_size(), eng.comm_layers());
    eng.release_buffers();
  } catch (const std::exception &e) {
    fprintf(stderr, "error: %s\n", e.what());
    return 1;
  }
  return 0;
}
