// C++ adapter over the C ABI of libgrace_hip.so with the shape of the reference's GPU engines, for a pair style that holds
// its atoms in device memory: what `pair_style grace/runtime/kk` calls on Grace1LKK / Grace2LKK / Grace3LKK
// (libgrace/include/grace/kk/grace_1l_kk.h:72-113, grace_2l_kk.h:81-157, grace_3l_kk.h:232-324): set_model, setup,
// cutoff, run(RunInput) -> RunOutput, chunksize, release_buffers, and the comm surface (Exchange, comm_width, pack / unpack
// of the message rows).  Plain device pointers stand where the reference has Kokkos views.  Header only; link libgrace_hip.so.
//
//   grace_hip::Engine eng;
//   eng.set_model("model/kokkos.npz", type2mu);         // type2mu[t], t = 1 .. ntypes: model element of atom type t or -1
//   eng.setup();
//   grace_hip::RunInput in; in.x = d_x; in.f = d_f; ...   // the views of atomKK and of the KOKKOS neighbour list
//   grace_hip::RunOutput out = eng.run(in);
#ifndef GRACE_HIP_LAMMPS_HPP
#define GRACE_HIP_LAMMPS_HPP

#include "grace_hip.h"

#include <stdexcept>
#include <string>
#include <vector>

namespace grace_hip {

// Message exchange of one layer between owned atoms and ghosts (libgrace/include/grace/system.h:53-60; LAMMPS: the pair
// style's forward_comm / reverse_comm, which call Engine::pack_forward ... below).
struct Exchange {
  virtual ~Exchange() = default;
  virtual void forward(int layer) = 0;    // message rows of the owners -> their ghost images
  virtual void reverse(int layer) = 0;    // adjoint rows of the ghost images summed into their owners
};

// The arguments of a pass (kk/grace_1l_kk.h:80-100): every pointer is device memory of the engine's GPU.
struct RunInput {
  const double *x = nullptr;          // [nall][3] positions, owned atoms then ghosts
  double *f = nullptr;                // [nall][3], forces are ADDED
  const int *type = nullptr;          // [nall] atom types, 1-based
  const int *ilist = nullptr;         // [inum] owned atoms of mapped types
  const int *numneigh = nullptr;      // [nlocal]
  const int *neighbors = nullptr;     // the 2-d neighbour view: element (i, k) at neighbors[i * stride_i + k * stride_k]
  long long stride_i = 0, stride_k = 1;
  int neighmask = 0x1FFFFFFF;         // LAMMPS NEIGHMASK: the special-bond bits of a neighbour index are dropped
  const int *owner = nullptr;         // [nall] owned atom each ghost is an image of (atom->map(tag)); one rank without Exchange
  int inum = 0, nlocal = 0, nall = 0, ntypes = 0;
  int eflag_atom = 0;
  bool energy_only = false;
  bool same_list = false;             // neighbor->ago > 0: the arrays are those of the previous run, only x has changed
  double *eatom = nullptr;            // [nall], per-atom energies are ADDED (with eflag_atom)
  int vflag_atom = 0;
  double *vatom = nullptr;            // [nall][6] xx yy zz xy xz yz, per-atom virials are ADDED (with vflag_atom)
  int cvflag_atom = 0;
  double *cvatom = nullptr;           // [nall][9] xx yy zz xy xz yz yx zx zy, centroid form, ADDED (with cvflag_atom)
};
struct RunOutput {
  double eng_vdwl = 0.0;
  double virial[6] = {0, 0, 0, 0, 0, 0};    // xx yy zz xy xz yz
};

class Engine {
 public:
  Engine() = default;
  Engine(const Engine &) = delete;
  Engine &operator=(const Engine &) = delete;
  ~Engine()
  {
    if (engine_) gr_engine_free(engine_);
    if (model_) gr_model_free(model_);
  }
  // precision 64 or 32 (fp32 network, fp64 geometry and sums); device: HIP device index
  int precision = 64, device = 0;
  // atoms per pass: > 0 fixed, 0 one pass, -1 from the free device memory (kk/grace_1l_kk.h: chunksize)
  int chunksize = -1;
  // forces, virial and energy added in a fixed order (same bits on every run) instead of with floating-point atomics;
  // no per-atom virials in this mode (gr_engine_set_ordered_sums)
  bool ordered_sums = false;

  void set_model(const std::string &npz_path, const std::vector<int> &type2mu)
  {
    if (model_) gr_model_free(model_);
    model_ = nullptr;
    check(gr_model_load(npz_path.c_str(), &model_));
    type2mu_ = type2mu;
  }
  void setup()
  {
    if (!model_) throw std::runtime_error("grace_hip::Engine::setup() before set_model()");
    if (engine_) gr_engine_free(engine_);
    engine_ = nullptr;
    check(gr_engine_create(model_, (int) type2mu_.size() - 1, type2mu_.data(), precision, device, &engine_));
    check(gr_engine_set_chunksize(engine_, chunksize));
    if (ordered_sums) check(gr_engine_set_ordered_sums(engine_, 1));
    if (exchange_) install_exchange();
  }
  double cutoff(int type_i, int type_j) const { return engine_ ? gr_engine_cutoff(engine_, type_i, type_j) : 0.0; }
  int auto_chunk_size() const { return engine_ ? gr_engine_chunksize(engine_) : 0; }
  void release_buffers() { if (engine_) check(gr_engine_release_buffers(engine_)); }

  RunOutput run(const RunInput &in)
  {
    RunOutput out;
    unsigned flags = 0;
    if (in.energy_only) flags |= GR_FLAG_ENERGY_ONLY;
    if (in.eflag_atom && in.eatom) flags |= GR_FLAG_EATOM;
    if (in.same_list) flags |= GR_FLAG_SAME_LIST;
    const bool vatom = in.vflag_atom && in.vatom && !in.energy_only, cvatom = in.cvflag_atom && in.cvatom && !in.energy_only;
    if (vatom || cvatom) flags |= GR_FLAG_VATOM;
    check(gr_compute_lammps_device(engine_, in.nlocal, in.nall, in.ntypes, in.type, in.x, in.inum, in.ilist, in.numneigh, in.neighbors,
                                   in.stride_i, in.stride_k, in.neighmask, in.owner, flags, &out.eng_vdwl, in.f, out.virial, in.eatom));
    if (vatom) check(gr_lammps_add_vatom_device(engine_, in.nall, in.vatom));
    if (cvatom) check(gr_lammps_add_cvatom_device(engine_, in.nall, in.cvatom));
    return out;
  }

  // ---- comm surface (kk/grace_2l_kk.h:141-157): layers 1 .. comm_layers() have a message of comm_width(layer) doubles
  void set_exchange(Exchange *x)
  {
    exchange_ = x;
    if (engine_) install_exchange();
  }
  int comm_layers() const { return engine_ ? gr_engine_comm_layers(engine_) : 0; }
  int comm_width(int layer) const { return engine_ ? gr_engine_comm_width(engine_, layer) : 0; }
  int pack_forward(int layer, int n, const int *sendlist, double *buf) { check(gr_engine_pack_forward(engine_, layer, n, sendlist, buf)); return n * comm_width(layer); }
  void unpack_forward(int layer, int n, int first, const double *buf) { check(gr_engine_unpack_forward(engine_, layer, n, first, buf)); }
  int pack_reverse(int layer, int n, int first, double *buf) { check(gr_engine_pack_reverse(engine_, layer, n, first, buf)); return n * comm_width(layer); }
  void unpack_reverse(int layer, int n, const int *sendlist, const double *buf) { check(gr_engine_unpack_reverse(engine_, layer, n, sendlist, buf)); }
  int pack_forward_host(int layer, int n, const int *list, double *buf) { check(gr_engine_pack_forward_host(engine_, layer, n, list, buf)); return n * comm_width(layer); }
  void unpack_forward_host(int layer, int n, int first, const double *buf) { check(gr_engine_unpack_forward_host(engine_, layer, n, first, buf)); }
  int pack_reverse_host(int layer, int n, int first, double *buf) { check(gr_engine_pack_reverse_host(engine_, layer, n, first, buf)); return n * comm_width(layer); }
  void unpack_reverse_host(int layer, int n, const int *list, const double *buf) { check(gr_engine_unpack_reverse_host(engine_, layer, n, list, buf)); }

  gr_engine *handle() const { return engine_; }

 private:
  gr_model *model_ = nullptr;
  gr_engine *engine_ = nullptr;
  std::vector<int> type2mu_;
  Exchange *exchange_ = nullptr;

  static void check(int status)
  {
    if (status == GR_OK) return;
    const std::string what = gr_last_error();
    if (status == GR_INVALID) throw std::invalid_argument(what);
    if (status == GR_NOMEM) throw std::bad_alloc();
    throw std::runtime_error(what);
  }
  static void forward_thunk(void *user, int layer) { static_cast<Exchange *>(user)->forward(layer); }
  static void reverse_thunk(void *user, int layer) { static_cast<Exchange *>(user)->reverse(layer); }
  void install_exchange()
  {
    if (!exchange_) {
      check(gr_engine_set_exchange(engine_, nullptr));
      return;
    }
    gr_exchange x{forward_thunk, reverse_thunk, exchange_};
    check(gr_engine_set_exchange(engine_, &x));
  }
};

}    // namespace grace_hip

#endif
