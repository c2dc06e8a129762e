// Engine interface behind the C ABI: one engine = one model on one GPU for one type -> element map.
// The call pattern mirrors the reference GPU engines (libgrace/include/grace/kk/grace_1l_kk.h:72-113: set_model /
// setup / run) and the CSR entry of the Python module (python/src/core.cpp:292-396).
#pragma once

#include "model.hpp"
#include "model_2l.hpp"
#include "model_3l.hpp"

#include <cstdint>
#include <memory>
#include <string>
#include <vector>

namespace grhip {

struct CsrInput {
  int n = 0;
  const int *types = nullptr;         // [n] 1-based atom types
  const int64_t *offset = nullptr;    // [n + 1]
  const int *j = nullptr;             // [nb]
  const double *rij = nullptr;        // [nb][3], or null with (x, image, shifts)
  const double *x = nullptr;          // [n][3]
  const int *image = nullptr;         // [nb]
  const double *shifts = nullptr;     // [nimages][3]
  int64_t nimages = 0;
  // several independent structures in one list (no bonds between them): structure of every atom, or null for one
  int nstruct = 1;
  const int *sid = nullptr;           // [n] in 0 .. nstruct-1
  // atoms with and without a row of bonds (a LAMMPS rank: owned atoms, then ghosts): n_nodes >= n atoms in all, the
  // first n are central atoms; types (and positions) have n_nodes entries, j indexes 0 .. n_nodes - 1, forces are
  // returned for all n_nodes.  0: every atom is central (n_nodes = n)
  int n_nodes = 0;
};

// Exchange of the message rows between the central atoms and the ghost atoms of a layer, as the reference's Exchange
// (libgrace/include/grace/system.h:53-60): forward(layer) is called when the layer's message rows of the central atoms
// are complete and must fill the rows of the ghosts; reverse(layer) when the adjoint rows are complete and must add the
// ghosts' rows to their owners'.  layer counts from 1.  The callbacks use Engine::comm_rows to move rows.
struct ExchangeCallbacks {
  void (*forward)(void *user, int layer) = nullptr;
  void (*reverse)(void *user, int layer) = nullptr;
  void *user = nullptr;
};

// A structure whose neighbour list is already in device memory: the engine copies it into its own buffers.
struct DeviceCsr {
  int n = 0;
  const int *types = nullptr;         // host [n] 1-based atom types, in the order of the list
  int64_t nb = 0;
  const int64_t *offset = nullptr;    // device [n + 1]
  const int *j = nullptr;             // device [nb]
  const int *image = nullptr;         // device [nb]
  const double *x = nullptr;          // device [n][3]
  const double *shifts = nullptr;     // host [nimages][3]
  int64_t nimages = 0;
  const double *rij = nullptr;        // device [nb][3] bond vectors, in place of (image, x, shifts)
  int nstruct = 1;                    // several independent structures in one list:
  const int *sid = nullptr;           // host [n] structure of every atom, or null for one structure
  int n_nodes = 0;                    // as CsrInput::n_nodes: types has n_nodes entries, j indexes 0 .. n_nodes - 1
};

struct StageTime {
  std::string name;
  double ms = 0.0;       // summed over the launches of the stage in the last run
  int launches = 0;
  double flops = 0.0;    // floating-point operations of the stage's tile GEMMs in the last run (2 per multiply-add; 0: not counted)
};

struct RunFlags {
  bool energy_only = false;
  bool eatom = false;
  bool uq = false;    // UQ head (ComputeFlags::uq, libgrace/include/grace/system.h:117): gamma, sigma, cluster per atom
  bool vatom = false; // per-atom virials (ComputeFlags::vflag_atom, system.h:115): half of every bond's virial to each of its atoms
};

class Engine {
 public:
  virtual ~Engine() = default;
  virtual int layers() const = 0;
  virtual double cutoff(int t1, int t2) const = 0;    // atom types, 1-based
  virtual double max_cutoff() const = 0;
  // copy a structure to the GPU (validates types, offsets and neighbour indices)
  virtual void upload(const CsrInput &in) = 0;
  // the same from a list in device memory (indices are trusted: the list comes from the library's own search)
  virtual void upload_device(const DeviceCsr &in) = 0;
  // new positions [n][3] (host) for the uploaded list (a list given as positions + image + shifts)
  virtual void update_positions(const double *x) = 0;
  // the device array [nb][3] that holds the bond vectors of the uploaded list (a list given with bond vectors), for a
  // caller that writes new vectors for the same bonds; the results of the last pass are dropped
  virtual double *bond_vectors_device() = 0;
  // counts the uploads of this engine: tells a caller whether the list it uploaded is still the one held
  virtual uint64_t upload_serial() const = 0;
  virtual int device_index() const = 0;
  // one energy / forces / virial pass over the uploaded structure; results stay on the GPU
  virtual void run(const RunFlags &fl) = 0;
  // wait for the pass and copy results out (null pointers are skipped); forces [n][3], virial [6], eatom [n]
  virtual void fetch(double *energy, double *forces, double *virial, double *eatom) = 0;
  // the same for a list of several structures: energy [nstruct], virial [nstruct][6]
  virtual void fetch_batch(int nstruct, double *energy, double *forces, double *virial, double *eatom) = 0;
  // the same with every output in device memory (the engine's GPU); null pointers are skipped
  virtual void fetch_batch_device(int nstruct, double *energy, double *forces, double *virial, double *eatom) = 0;
  // one structure: energy and virial [6] to the host; forces and per-atom energies ADDED to device arrays of the
  // caller, row q of the engine to row atom[q] (atom: device [n]); null pointers are skipped
  virtual void fetch_add_device(const int *atom, double *energy, double *forces, double *virial, double *eatom) = 0;
  // UQ outputs of the last run with RunFlags::uq, [n] each in the order of the uploaded list (null pointers are skipped)
  // per-atom virials [n_nodes][6] (xx yy zz xy xz yz) of a run with the vatom flag, in the order of the uploaded list; host memory
  // ncomp 9: the centroid form, the six components followed by yx zx zy (cvatom of kk/grace_1l_kk.h:94)
  // expect_rows >= 0: the rows the caller's buffer holds; a different count held by the engine is an error
  virtual void fetch_vatom(double *vatom, int ncomp = 6, long long expect_rows = -1) = 0;
  // the same rows added to a device array: row q of the list goes to row atom[q] (null: row q) of vatom
  virtual void add_vatom_device(const int *atom, double *vatom, int ncomp = 6) = 0;
  virtual void fetch_uq(double *gamma, double *sigma, double *cluster) = 0;
  // atoms per engine pass (python/kk/kk_api.h:72-75): 0 all atoms in one pass, < 0 chosen from the free device memory
  // (one pass while it fits, else the largest power of two >= 512 that fits), > 0 as given.  chunksize_used(): atoms per
  // pass of the last run (0: one pass).  Engines that do not chunk refuse values other than 0 and -1.
  // message exchange with ghost atoms (LAMMPS comm): the callbacks, the layers that have a message (0 for GRACE-1L, 1 for
  // 2L, 2 for 3L), the doubles per atom of a layer's message, and the four row movers of the reference's GPU engines
  // (libgrace/include/grace/kk/grace_2l_kk.h:141-157): mode 0 pack_forward (rows of the atoms list[0 .. n) -> buf),
  // 1 unpack_forward (buf -> rows of atoms first .. first + n), 2 pack_reverse (adjoint rows of first .. first + n -> buf),
  // 3 unpack_reverse (buf ADDED to the adjoint rows of list[0 .. n)); list and buf in device memory, or, with host = true,
  // in host memory
  virtual void set_exchange(const ExchangeCallbacks &cb) = 0;
  virtual int comm_layers() const = 0;
  virtual int comm_width(int layer) const = 0;
  virtual void comm_rows(int mode, int layer, int n, const int *list, int first, double *buf, bool host) = 0;
  // atoms of one pass whose work buffers fit 70 % of the memory the library may use, from the bytes per atom that the
  // buffers of the last pass hold; before the first pass: a bound by model kind.  The batch entry points size their
  // passes with it (the reference sizes the first pass from the free memory: libgrace/include/grace/kk/support.h:425-450)
  virtual int64_t atoms_that_fit() = 0;
  virtual void set_chunksize(int atoms) = 0;
  // radial tables (spline_n of the reference's engines, libgrace/include/grace/system.h:78; `spline` of Model / System /
  // Batch, python/kk/kk_api.h:53,75): n > 0: the radial functions of GRACE-1L and 2L engines come from cubic tables of n
  // intervals, as in the reference; 0 (the engines' default): the radial MLP is evaluated for every bond
  virtual void set_spline(int n) = 0;
  virtual int spline() const = 0;
  // ordered sums: forces, virial, energy and message adjoints are added in a fixed order instead of with floating-point
  // atomics, so that two runs on the same input give the same bits (the reference's GPU engines accept last-bit variation
  // from run to run: python/tests/test_gpu_several_calculators.py).
  virtual void set_ordered_sums(bool on) = 0;
  virtual bool ordered_sums() const = 0;
  virtual int chunksize_used() const = 0;
  virtual void release_buffers() = 0;    // frees the work buffers and the uploaded structure; weights stay
  virtual void synchronize() = 0;
  virtual void set_profile(bool on) = 0;
  virtual const std::vector<StageTime> &stage_times() = 0;
  virtual int64_t last_edge_count() = 0;
  // a plain device-to-device copy kernel over `bytes` bytes (calibration of the memory-traffic counters)
  virtual void debug_copy(int64_t bytes) = 0;
  // measured rates (GB/s) of that copy kernel and of a read-only stream kernel: the ceilings HBM-bound kernels are compared with
  virtual void stream_rates(int64_t bytes, double *copy_gbs, double *read_gbs) = 0;
  // radial functions of the device kernel for the given x = r / rc and neighbour elements: R z and dR/dx z,
  // [m][nl][C] (tests of the MFMA kernel against the CPU restatement)
  virtual void debug_radial(int m, const double *x, const int *mu_j, double *Rz, double *dRz) = 0;
  // the same functions for callers that must not allocate device memory: x [m], mu_j [m], Rz, dRz [m][nl][C] are device
  // arrays of the engine's GPU, the staging rows come from a fixed device array of the library (bounded m)
  virtual void radial_noalloc(int m, const double *x, const int *mu_j, double *Rz, double *dRz) = 0;
};

// precision: 64 (network arithmetic in fp64) or 32 (fp32 network, fp64 geometry and sums)
std::unique_ptr<Engine> make_engine_1l(std::shared_ptr<const Model1L> model, int ntypes, const std::vector<int> &type2mu,
                                       int precision, int device);

// GRACE-2L: the same two precisions (fp32: the scalar reduces, the two RMSNorms and the readout stay in fp64)
std::unique_ptr<Engine> make_engine_2l(std::shared_ptr<const Model2L> model, int ntypes, const std::vector<int> &type2mu,
                                       int precision, int device);

// GRACE-3L: the same two precisions (fp32: the scalar reduces, the norms and the readout stay in fp64)
std::unique_ptr<Engine> make_engine_3l(std::shared_ptr<const Model3L> model, int ntypes, const std::vector<int> &type2mu,
                                       int precision, int device);

}    // namespace grhip
