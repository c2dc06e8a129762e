// extern "C" layer of libgrace_hip.so (declarations and the reference interfaces they replace: include/grace_hip.h).
// Exceptions never cross the ABI: they become a status code and a thread-local message.
#include "../../include/grace_hip.h"

#include "engine.hpp"
#include "neighbors.hpp"
#include "neighbors_dev.hpp"
#include "neighbors_batch_dev.hpp"
#include "lammps_dev.hpp"

#include <hip/hip_runtime_api.h>

#include <array>
#include <cmath>
#include <cstring>
#include <memory>
#include <new>
#include <string>

struct gr_model {
  grhip::ModelKind kind;
  std::shared_ptr<grhip::Model1L> m1;
  std::shared_ptr<grhip::Model2L> m2;
  std::shared_ptr<grhip::Model3L> m3;
  std::string path;
};
struct gr_engine {
  std::unique_ptr<grhip::Engine> eng;
  // what the engine was made from: reset() makes a fresh one after a failed allocation left this one half grown
  std::shared_ptr<grhip::Model1L> m1;
  std::shared_ptr<grhip::Model2L> m2;
  std::shared_ptr<grhip::Model3L> m3;
  std::vector<int> type2mu;
  int ntypes = 0, precision = 64, device = 0;
  int generation = 0;                                  // counts reset(): holders of uploaded state (gr_system) upload again
  int64_t nall_cap = INT64_MAX;                        // atoms per batch pass after an allocation failure (kept for later calls)
  bool has_exchange = false;                           // an exchange is installed: ghosts of the LAMMPS call stay atoms of their own
  grhip::ExchangeCallbacks exchange;                   // kept for the engine a reset makes
  int chunk_request = -1;                              // the caller's chunk size, kept for the engine a reset makes
  bool ordered = false;                                // ordered sums requested, kept for the engine a reset makes
  int spline = 0;                                      // radial-table intervals requested, kept for the engine a reset makes
  grhip::PinnedBuf pin_types;                          // gr_compute_batch_device: the atom types of a pass on their way to the host
  std::vector<int> lmp_rows;                           // gr_compute_lammps: LAMMPS index of engine row q (empty: rows are LAMMPS indices)
  int lmp_nall = -1;                                   // atoms of the last gr_compute_lammps[_device] call
  uint64_t lmp_serial = 0;                             // the engine's upload count at that call: its list is still the one held
  bool lmp_on_device = false;                          // that call was the device form (its row map is lmp->atom)
  // the state of the last LAMMPS call names rows of a structure the engine no longer holds (the new engine of a reset
  // counts its uploads from zero again, so the old count could match a later, unrelated upload)
  void forget_lammps_call()
  {
    lmp_rows.clear();
    lmp_nall = -1;
    lmp_serial = 0;
    lmp_on_device = false;
  }
  void make()
  {
    if (m1) eng = grhip::make_engine_1l(m1, ntypes, type2mu, precision, device);
    else if (m2) eng = grhip::make_engine_2l(m2, ntypes, type2mu, precision, device);
    else eng = grhip::make_engine_3l(m3, ntypes, type2mu, precision, device);
  }
  void reset()
  {
    bnl.reset();
    lmp.reset();
    forget_lammps_call();
    eng.reset();    // frees every device buffer of the engine before the new one allocates
    generation++;
    make();
    if (has_exchange) eng->set_exchange(exchange);
    eng->set_chunksize(chunk_request);
    if (ordered) eng->set_ordered_sums(true);
    if (spline > 0) eng->set_spline(spline);
  }
  std::vector<grhip::StageTime> times;
  std::unique_ptr<grhip::BatchDeviceNeighbors> bnl;    // lists of gr_compute_batch_device (buffers kept between calls)
  std::unique_ptr<grhip::LammpsDeviceList> lmp;       // converted list of gr_compute_lammps_device
  hipStream_t bnl_stream = nullptr;                    // stream of the list builds of the device entry points
  ~gr_engine()
  {
    if (bnl_stream) (void) hipStreamDestroy(bnl_stream);
  }
};
struct gr_nlist {
  grhip::NeighborList nl;
};
// One structure resident on the device with a Verlet list at cutoff + skin (System of the reference's GPU module,
// python/kk/kk_api.h:66-93): the pair search of a rebuild runs on the device, calls between rebuilds send positions only.
struct gr_system {
  gr_engine *eng = nullptr;
  double skin = 0.0, cutoff = 0.0;
  int rebuilds = 0, generation = 0;
  bool have = false, on_device = false;
  bool auto_chunk = true;    // the chunk is the engine's choice (and may be halved after an allocation failure)
  int n = 0;
  std::vector<int> types;
  std::vector<double> x0, cell;
  unsigned char pbc[3] = {0, 0, 0};
  std::vector<int64_t> perm;
  grhip::DeviceNeighbors nl;
  grhip::NeighborList host_nl;    // the list when the device search declined the structure
  grhip::DevBuf pos_dev, x_dev;
  hipStream_t stream = nullptr;
  ~gr_system()
  {
    if (stream) (void) hipStreamDestroy(stream);
  }
};

namespace {
// the engine behind a handle; a handle whose engine was dropped by a reset that could not build the new one says so
grhip::Engine &live(const gr_engine *e)
{
  if (!e) throw grhip::InvalidArgument("null engine");
  if (!e->eng) throw grhip::Error("the engine was lost when a reset could not allocate its replacement; call gr_engine_reset");
  return *e->eng;
}
void padded_cell(const double *cell, const unsigned char *pbc, const double *pos, int64_t n, double reach, double *out, double *shift);
thread_local std::string g_err;

template<class F> int guarded(F &&f)
{
  try {
    f();
    g_err.clear();
    return GR_OK;
  } catch (const grhip::InvalidArgument &e) {
    g_err = e.what();
    return GR_INVALID;
  } catch (const std::invalid_argument &e) {
    g_err = e.what();
    return GR_INVALID;
  } catch (const std::bad_alloc &) {
    g_err = "out of memory";
    return GR_NOMEM;
  } catch (const std::exception &e) {
    g_err = e.what();
    return GR_ERROR;
  } catch (...) {
    g_err = "unknown error";
    return GR_ERROR;
  }
}

grhip::CsrInput make_input(int n, const int *types, const int64_t *offset, const int *j, const double *rij,
                           const double *positions, const int *image, const double *shifts, int64_t nimages)
{
  if (n > 0 && (!types || !offset)) throw grhip::InvalidArgument("types and offset are required");
  grhip::CsrInput in;
  in.n = n;
  in.types = types;
  in.offset = offset;
  in.j = j;
  in.rij = rij;
  in.x = positions;
  in.image = image;
  in.shifts = shifts;
  in.nimages = nimages;
  return in;
}
}    // namespace

extern "C" {

const char *gr_last_error(void) { return g_err.c_str(); }
int gr_abi_version(void) { return 7; }
void gr_set_logger(gr_log_fn fn, void *user)
{
  grhip::log_sink().user.store(user);
  grhip::log_sink().fn.store(fn);
}

int gr_device_count(void)
{
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void) hipGetLastError();
    return 0;
  }
  return n;
}

int gr_device_arch(int device, char *buf, int len)
{
  if (buf && len > 0) buf[0] = 0;
  return guarded([&] {
    hipDeviceProp_t p;
    if (hipGetDeviceProperties(&p, device) != hipSuccess) {
      (void) hipGetLastError();
      throw grhip::Error("no such HIP device");
    }
    if (buf && len > 0) {
      std::strncpy(buf, p.gcnArchName, (size_t) len - 1);
      buf[len - 1] = 0;
    }
  });
}

int gr_model_load(const char *npz_path, gr_model **out)
{
  return guarded([&] {
    if (!npz_path || !out) throw grhip::InvalidArgument("null argument");
    *out = nullptr;
    const grhip::Npz z = grhip::npz_load(npz_path);
    auto m = std::make_unique<gr_model>();
    m->path = npz_path;
    m->kind = grhip::model_kind(z, npz_path);
    if (m->kind == grhip::ModelKind::Grace1L) {
      m->m1 = std::make_shared<grhip::Model1L>();
      m->m1->load(z);
    } else if (m->kind == grhip::ModelKind::Grace2L) {
      m->m2 = std::make_shared<grhip::Model2L>();
      m->m2->load(z);
    } else {
      m->m3 = std::make_shared<grhip::Model3L>();
      m->m3->load(z);
    }
    *out = m.release();
  });
}

int gr_model_get_info(const gr_model *m, gr_model_info *info)
{
  return guarded([&] {
    if (!m || !info) throw grhip::InvalidArgument("null argument");
    std::memset(info, 0, sizeof(*info));
    info->layers = (int) m->kind;
    if (m->m1) {
      info->n_elements = m->m1->n_elements;
      info->lmax = m->m1->lmax;
      info->n_radial = m->m1->nradmax;
      info->n_radbase = m->m1->nradbase;
      info->max_order = m->m1->max_order;
      double rc = 0.0;
      for (double c : m->m1->bond_cutoff_map) rc = std::max(rc, c);
      info->rcut = m->m1->has_bond_specific_cutoff ? rc : m->m1->rcut;
    } else if (m->m2) {
      info->n_elements = m->m2->n_elements;
      info->lmax = m->m2->lmax;
      info->n_radial = m->m2->C1;
      info->n_radbase = m->m2->nradbase;
      info->max_order = m->m2->max_order;
      double rc = 0.0;
      for (double c : m->m2->bond_cutoff_map) rc = std::max(rc, c);
      info->rcut = m->m2->has_bond_specific_cutoff ? rc : m->m2->rcut;
    } else if (m->m3) {
      info->n_elements = m->m3->n_elements;
      info->lmax = m->m3->lmax;
      info->n_radial = m->m3->spbf.empty() ? 0 : m->m3->spbf[0].n_rad_max;
      info->n_radbase = m->m3->nradbase;
      info->max_order = 4;
      double rc = 0.0;
      for (double c : m->m3->bond_cutoff_map) rc = std::max(rc, c);
      info->rcut = m->m3->has_bond_specific_cutoff ? rc : m->m3->rcut;
    }
  });
}

const char *gr_model_element_name(const gr_model *m, int k)
{
  if (!m || k < 0) return "";
  const std::vector<std::string> &names = m->m1 ? m->m1->element_names : m->m2 ? m->m2->element_names : m->m3->element_names;
  return k < (int) names.size() ? names[k].c_str() : "";
}

void gr_model_free(gr_model *m) { delete m; }

int gr_engine_create(const gr_model *m, int ntypes, const int *type2mu, int precision, int device, gr_engine **out)
{
  return guarded([&] {
    if (!m || !type2mu || !out) throw grhip::InvalidArgument("null argument");
    *out = nullptr;
    if (ntypes < 1) throw grhip::InvalidArgument("ntypes must be positive");
    auto e = std::make_unique<gr_engine>();
    e->m1 = m->m1; e->m2 = m->m2; e->m3 = m->m3;
    e->type2mu.assign(type2mu, type2mu + ntypes + 1);
    e->ntypes = ntypes; e->precision = precision; e->device = device;
    e->make();
    *out = e.release();
  });
}

int gr_engine_release_buffers(gr_engine *e)
{
  return guarded([&] {
    if (!e) throw grhip::InvalidArgument("null engine");
    e->bnl.reset();
    e->lmp.reset();
    e->forget_lammps_call();
    live(e).release_buffers();
    e->generation++;    // a gr_system on this engine uploads its structure again
  });
}

int gr_engine_reset(gr_engine *e)
{
  return guarded([&] {
    if (!e) throw grhip::InvalidArgument("null engine");
    e->reset();
  });
}

void gr_set_memory_limit(int64_t bytes) { grhip::dev_bytes_limit().store(bytes > 0 ? bytes : 0); }
int64_t gr_memory_in_use(void) { return grhip::dev_bytes_in_use().load(); }

void gr_engine_free(gr_engine *e) { delete e; }

double gr_engine_cutoff(const gr_engine *e, int t1, int t2) { return e && e->eng ? e->eng->cutoff(t1, t2) : 0.0; }

int gr_engine_upload(gr_engine *e, int n, const int *types, const int64_t *offset, const int *j, const double *rij,
                     const double *positions, const int *image, const double *shifts, int64_t nimages)
{
  return guarded([&] {
    if (!e) throw grhip::InvalidArgument("null engine");
    live(e).upload(make_input(n, types, offset, j, rij, positions, image, shifts, nimages));
  });
}

int gr_engine_run(gr_engine *e, unsigned flags)
{
  return guarded([&] {
    if (!e) throw grhip::InvalidArgument("null engine");
    grhip::RunFlags fl;
    fl.energy_only = (flags & GR_FLAG_ENERGY_ONLY) != 0;
    fl.eatom = (flags & GR_FLAG_EATOM) != 0;
    fl.vatom = (flags & GR_FLAG_VATOM) != 0;
    fl.uq = (flags & GR_FLAG_UQ) != 0;
    live(e).run(fl);
  });
}

int gr_engine_fetch_uq(gr_engine *e, double *gamma, double *sigma, double *cluster)
{
  return guarded([&] {
    if (!e) throw grhip::InvalidArgument("null engine");
    live(e).fetch_uq(gamma, sigma, cluster);
  });
}

int gr_engine_fetch_vatom(gr_engine *e, double *vatom)
{
  return guarded([&] {
    if (!e || !vatom) throw grhip::InvalidArgument("null argument");
    live(e).fetch_vatom(vatom);
  });
}

int gr_engine_fetch_cvatom(gr_engine *e, double *cvatom)
{
  return guarded([&] {
    if (!e || !cvatom) throw grhip::InvalidArgument("null argument");
    live(e).fetch_vatom(cvatom, 9);
  });
}

int gr_model_has_uq(const gr_model *m)
{
  return m && ((m->m1 && m->m1->uq.has_uq) || (m->m2 && m->m2->uq.has_uq) || (m->m3 && m->m3->uq.has_uq)) ? 1 : 0;
}

int gr_model_validate_uq(const gr_model *m)
{
  return guarded([&] {
    if (!m) throw grhip::InvalidArgument("null model");
    try {
      if (m->m1) m->m1->validate_uq();
      else if (m->m2) m->m2->validate_uq();
      else if (!m->m3->uq.has_uq)    // a GRACE-3L file with a broken head does not load (libgrace/src/fused_3l.cpp:269-274)
        throw grhip::Error("GRACE-3L: the model has no UQ head (kokkos.npz exported without UQ artifacts)");
    } catch (const grhip::Error &e) {
      throw grhip::InvalidArgument(e.what());    // python/kk/kk_core.cpp: std::invalid_argument (unsupported model)
    }
  });
}

int gr_engine_sync(gr_engine *e)
{
  return guarded([&] {
    if (!e) throw grhip::InvalidArgument("null engine");
    live(e).synchronize();
  });
}

int gr_engine_fetch(gr_engine *e, double *energy, double *forces, double *virial, double *eatom)
{
  return guarded([&] {
    if (!e) throw grhip::InvalidArgument("null engine");
    live(e).fetch(energy, forces, virial, eatom);
  });
}

int64_t gr_engine_edge_count(gr_engine *e)
{
  int64_t r = -1;
  guarded([&] { r = live(e).last_edge_count(); });
  return r;
}

int gr_compute_csr(gr_engine *e, int n, const int *types, const int64_t *offset, const int *j, const double *rij,
                   const double *positions, const int *image, const double *shifts, int64_t nimages, unsigned flags,
                   double *energy, double *forces, double *virial, double *eatom)
{
  return guarded([&] {
    if (!e) throw grhip::InvalidArgument("null engine");
    live(e).upload(make_input(n, types, offset, j, rij, positions, image, shifts, nimages));
    grhip::RunFlags fl;
    fl.energy_only = (flags & GR_FLAG_ENERGY_ONLY) != 0;
    fl.eatom = (flags & GR_FLAG_EATOM) != 0 && eatom;
    fl.vatom = (flags & GR_FLAG_VATOM) != 0;
    live(e).run(fl);
    if (!(flags & GR_FLAG_ACCUMULATE)) {
      live(e).fetch(energy, forces, virial, eatom);
      return;
    }
    // Outputs of the reference accumulate (libgrace/include/grace/system.h:66-75): add to what the caller's arrays hold
    double en = 0.0, vir[6] = {0, 0, 0, 0, 0, 0};
    std::vector<double> f(forces && !fl.energy_only ? (size_t) 3 * n : 0), ea(fl.eatom ? (size_t) n : 0);
    live(e).fetch(&en, f.empty() ? nullptr : f.data(), vir, ea.empty() ? nullptr : ea.data());
    if (energy) *energy += en;
    if (virial && !fl.energy_only)
      for (int k = 0; k < 6; k++) virial[k] += vir[k];
    for (size_t q = 0; q < f.size(); q++) forces[q] += f[q];
    for (size_t q = 0; q < ea.size(); q++) eatom[q] += ea[q];
  });
}

int gr_engine_set_profile(gr_engine *e, int on)
{
  return guarded([&] {
    if (!e) throw grhip::InvalidArgument("null engine");
    live(e).set_profile(on != 0);
  });
}

int gr_engine_stage_count(gr_engine *e)
{
  int n = -1;
  guarded([&] {
    e->times = live(e).stage_times();
    n = (int) e->times.size();
  });
  return n;
}

int gr_engine_stage_get(gr_engine *e, int k, char *name, int name_len, double *ms, int *launches)
{
  return guarded([&] {
    if (!e || k < 0 || k >= (int) e->times.size()) throw grhip::InvalidArgument("no such stage");
    if (name && name_len > 0) {
      std::strncpy(name, e->times[k].name.c_str(), (size_t) name_len - 1);
      name[name_len - 1] = 0;
    }
    if (ms) *ms = e->times[k].ms;
    if (launches) *launches = e->times[k].launches;
  });
}

int gr_engine_stage_flops(gr_engine *e, int k, double *flops)
{
  return guarded([&] {
    if (!e || k < 0 || k >= (int) e->times.size()) throw grhip::InvalidArgument("no such stage");
    if (flops) *flops = e->times[k].flops;
  });
}

int gr_engine_debug_radial(gr_engine *e, int m, const double *x, const int *mu_j, double *Rz, double *dRz)
{
  return guarded([&] {
    if (!e) throw grhip::InvalidArgument("null engine");
    live(e).debug_radial(m, x, mu_j, Rz, dRz);
  });
}

int gr_engine_radial_noalloc(gr_engine *e, int m, const double *x, const int *mu_j, double *Rz, double *dRz)
{
  return guarded([&] {
    if (!e || !e->eng) throw grhip::InvalidArgument("null engine");
    live(e).radial_noalloc(m, x, mu_j, Rz, dRz);
  });
}

int gr_engine_debug_copy(gr_engine *e, int64_t bytes)
{
  return guarded([&] {
    if (!e) throw grhip::InvalidArgument("null engine");
    live(e).debug_copy(bytes);
  });
}

int gr_engine_stream_rates(gr_engine *e, int64_t bytes, double *copy_gbs, double *read_gbs)
{
  return guarded([&] {
    if (!e || bytes < 16) throw grhip::InvalidArgument("null engine or no bytes");
    live(e).stream_rates(bytes, copy_gbs, read_gbs);
  });
}

int gr_neighbor_build(int64_t n, const double *positions, const double *cell, const unsigned char *pbc, double cutoff,
                      int nthreads, gr_nlist **out)
{
  return guarded([&] {
    if (!out || !cell || !pbc || (n > 0 && !positions)) throw grhip::InvalidArgument("null argument");
    *out = nullptr;
    const bool p[3] = {pbc[0] != 0, pbc[1] != 0, pbc[2] != 0};
    auto l = std::make_unique<gr_nlist>();
    l->nl = grhip::neighbor_search(positions, n, cell, p, cutoff, nthreads);
    *out = l.release();
  });
}

int64_t gr_nlist_nbonds(const gr_nlist *l) { return l ? (int64_t) l->nl.j.size() : 0; }
int64_t gr_nlist_nimages(const gr_nlist *l) { return l ? (int64_t) l->nl.shifts.size() / 3 : 0; }

int gr_nlist_get(const gr_nlist *l, int64_t *perm, int64_t *offset, int32_t *j, int32_t *image, double *shifts)
{
  return guarded([&] {
    if (!l) throw grhip::InvalidArgument("null list");
    const auto &r = l->nl;
    if (perm) std::memcpy(perm, r.perm.data(), r.perm.size() * sizeof(int64_t));
    if (offset) std::memcpy(offset, r.offset.data(), r.offset.size() * sizeof(int64_t));
    if (j) std::memcpy(j, r.j.data(), r.j.size() * sizeof(int32_t));
    if (image) std::memcpy(image, r.image.data(), r.image.size() * sizeof(int32_t));
    if (shifts) std::memcpy(shifts, r.shifts.data(), r.shifts.size() * sizeof(double));
  });
}

void gr_nlist_free(gr_nlist *l) { delete l; }

int gr_compute(gr_engine *e, int n, const int *types, const double *positions, const double *cell,
               const unsigned char *pbc, unsigned flags, double *energy, double *forces, double *virial, double *eatom)
{
  return guarded([&] {
    if (!e || !cell || !pbc || (n > 0 && (!types || !positions))) throw grhip::InvalidArgument("null argument");
    const bool p[3] = {pbc[0] != 0, pbc[1] != 0, pbc[2] != 0};
    double rc = 0.0;
    {
      // largest cutoff over the types present
      rc = live(e).max_cutoff();
      if (!(rc > 0.0)) throw grhip::Error("the engine has no positive cutoff");
    }
    grhip::NeighborList nl = grhip::neighbor_search(positions, n, cell, p, rc, 8);
    std::vector<int> ty(n);
    std::vector<double> x((size_t) 3 * n);
    for (int q = 0; q < n; q++) {
      const int64_t a = nl.perm[q];
      ty[q] = types[a];
      for (int d = 0; d < 3; d++) x[3 * (size_t) q + d] = positions[3 * a + d];
    }
    std::vector<double> dummy(3, 0.0);
    const int64_t nimg = (int64_t) nl.shifts.size() / 3;
    live(e).upload(make_input(n, ty.data(), nl.offset.data(), nl.j.data(), nullptr, x.data(), nl.image.data(),
                              nimg ? nl.shifts.data() : dummy.data(), nimg));
    grhip::RunFlags fl;
    fl.energy_only = (flags & GR_FLAG_ENERGY_ONLY) != 0;
    fl.eatom = (flags & GR_FLAG_EATOM) != 0 && eatom;
    fl.vatom = (flags & GR_FLAG_VATOM) != 0;
    live(e).run(fl);
    std::vector<double> f((size_t) 3 * n), ea(fl.eatom ? n : 0);
    live(e).fetch(energy, forces ? f.data() : nullptr, virial, fl.eatom ? ea.data() : nullptr);
    for (int q = 0; q < n; q++) {
      const int64_t a = nl.perm[q];
      if (forces && !fl.energy_only)
        for (int d = 0; d < 3; d++) forces[3 * a + d] = f[3 * (size_t) q + d];
      if (fl.eatom) eatom[a] = ea[q];
    }
  });
}

int gr_compute_lammps(gr_engine *e, int nlocal, int nall, const int *type, const double *x, int inum, const int *ilist, const int *numneigh,
                      const int *const *firstneigh, int neighmask, const int *owner, unsigned flags, double *energy, double *f,
                      double *virial, double *eatom)
{
  return guarded([&] {
    if (!e || (nall > 0 && (!type || !x)) || (inum > 0 && (!ilist || !numneigh || !firstneigh))) throw grhip::InvalidArgument("null argument");
    if (nlocal < 0 || nall < nlocal || inum < 0) throw grhip::InvalidArgument("atom counts out of range");
    grhip::Engine &eng = live(e);
    // atoms of types the engine has no element for take no part (pair_style hybrid): neither central atoms nor neighbours
    auto mapped = [&](int a) { return eng.cutoff(type[a], type[a]) > 0.0; };
    grhip::RunFlags fl;
    fl.energy_only = (flags & GR_FLAG_ENERGY_ONLY) != 0;
    fl.eatom = (flags & GR_FLAG_EATOM) != 0 && eatom;
    fl.vatom = (flags & GR_FLAG_VATOM) != 0;
    if (!owner && nall > nlocal && (e->has_exchange || eng.comm_layers() == 0)) {
      // Ghosts stay atoms of their own (the way of the reference's drivers): bonds name them by their LAMMPS index, their
      // message rows come through the exchange, and what the pass leaves on them (forces, adjoint rows) goes back through
      // the reverse exchange and LAMMPS' reverse communication of f.  Every atom must have a model element here.
      for (int a = 0; a < nall; a++)
        if (!mapped(a)) throw grhip::InvalidArgument("with an exchange every owned and ghost atom needs a type with a model element");
      std::vector<char> listed(nlocal, 0);
      for (int q = 0; q < inum; q++) {
        if (ilist[q] < 0 || ilist[q] >= nlocal) throw grhip::InvalidArgument("ilist must index owned atoms");
        listed[ilist[q]] = 1;
      }
      for (int i = 0; i < nlocal; i++)
        if (!listed[i]) throw grhip::InvalidArgument("every owned atom of a mapped type must be in ilist (sub-lists are not supported)");
      std::vector<int64_t> offset((size_t) nlocal + 1, 0);
      std::vector<int> jj;
      std::vector<double> rij;
      for (int i = 0; i < nlocal; i++) {
        const int *nb = firstneigh[i];
        for (int k = 0; k < numneigh[i]; k++) {
          const int j = nb[k] & neighmask;
          if (j < 0 || j >= nall) throw grhip::InvalidArgument("neighbour index outside the owned and ghost atoms");
          jj.push_back(j);
          for (int d = 0; d < 3; d++) rij.push_back(x[3 * (size_t) j + d] - x[3 * (size_t) i + d]);
        }
        offset[(size_t) i + 1] = (int64_t) jj.size();
      }
      const std::vector<double> dummy(3, 0.0);
      grhip::CsrInput in = make_input(nlocal, type, offset.data(), jj.data(), rij.empty() ? dummy.data() : rij.data(), nullptr, nullptr, nullptr, 0);
      in.n_nodes = nall;
      eng.upload(in);
      eng.run(fl);
      e->lmp_rows.clear();    // rows are LAMMPS indices
      e->lmp_nall = nall;
      e->lmp_serial = eng.upload_serial();
      e->lmp_on_device = false;
      std::vector<double> fo((size_t) 3 * nall), ea(fl.eatom ? nlocal : 0);
      double en = 0.0, vir[6] = {0, 0, 0, 0, 0, 0};
      eng.fetch(&en, f ? fo.data() : nullptr, vir, fl.eatom ? ea.data() : nullptr);
      if (energy) *energy = en;
      if (virial && !fl.energy_only)
        for (int k = 0; k < 6; k++) virial[k] = vir[k];
      if (f && !fl.energy_only)
        for (size_t q = 0; q < fo.size(); q++) f[q] += fo[q];
      for (int i = 0; i < (fl.eatom ? nlocal : 0); i++) eatom[i] += ea[(size_t) i];
      return;
    }
    std::vector<int> idx(nlocal, -1), atom;
    std::vector<char> central(nlocal, 0);
    for (int q = 0; q < inum; q++) {
      const int i = ilist[q];
      if (i < 0 || i >= nlocal) throw grhip::InvalidArgument("ilist must index owned atoms");
      if (!mapped(i)) throw grhip::Error("atom " + std::to_string(i) + " of unmapped type " + std::to_string(type[i]) + " in the atom list");
      central[i] = 1;
    }
    for (int i = 0; i < nlocal; i++) {
      if (!mapped(i)) continue;
      if (!central[i]) throw grhip::InvalidArgument("every owned atom of a mapped type must be in ilist (sub-lists are not supported)");
      idx[i] = (int) atom.size();
      atom.push_back(i);
    }
    const int n = (int) atom.size();
    std::vector<int> ty(n), jj;
    std::vector<int64_t> offset(n + 1, 0);
    std::vector<double> rij;
    for (int q = 0; q < n; q++) {
      const int i = atom[q];
      ty[q] = type[i];
      const int *nb = firstneigh[i];
      for (int k = 0; k < numneigh[i]; k++) {
        const int j = nb[k] & neighmask;
        if (j < 0 || j >= nall) throw grhip::InvalidArgument("neighbour index outside the owned and ghost atoms");
        if (!mapped(j)) continue;
        int o = j;
        if (j >= nlocal) {
          if (!owner) throw grhip::InvalidArgument("ghost neighbours need the owner map (the owned atom each ghost is an image of) or an exchange");
          o = owner[j];
        }
        if (o < 0 || o >= nlocal || idx[o] < 0 || type[o] != type[j])
          throw grhip::InvalidArgument("owner of ghost atom " + std::to_string(j) + " is not an owned atom of the same type");
        jj.push_back(idx[o]);
        for (int d = 0; d < 3; d++) rij.push_back(x[3 * (size_t) j + d] - x[3 * (size_t) i + d]);
      }
      offset[q + 1] = (int64_t) jj.size();
    }
    const std::vector<double> dummy(3, 0.0);
    eng.upload(make_input(n, ty.data(), offset.data(), jj.data(), rij.empty() ? dummy.data() : rij.data(), nullptr, nullptr, nullptr, 0));
    eng.run(fl);
    e->lmp_rows = atom;
    e->lmp_nall = nall;
    e->lmp_serial = eng.upload_serial();
    e->lmp_on_device = false;
    std::vector<double> fo((size_t) 3 * n), ea(fl.eatom ? n : 0);
    double en = 0.0, vir[6] = {0, 0, 0, 0, 0, 0};
    eng.fetch(&en, f ? fo.data() : nullptr, vir, fl.eatom ? ea.data() : nullptr);
    if (energy) *energy = en;
    if (virial && !fl.energy_only)
      for (int k = 0; k < 6; k++) virial[k] = vir[k];
    for (int q = 0; q < n; q++) {
      const int i = atom[q];
      if (f && !fl.energy_only)
        for (int d = 0; d < 3; d++) f[3 * (size_t) i + d] += fo[3 * (size_t) q + d];
      if (fl.eatom) eatom[i] += ea[q];
    }
  });
}

// ---- message exchange with ghost atoms (LAMMPS comm) ----------------------------------------------------------------
int gr_engine_set_exchange(gr_engine *e, const gr_exchange *x)
{
  return guarded([&] {
    grhip::ExchangeCallbacks cb;
    if (x) {
      cb.forward = x->forward;
      cb.reverse = x->reverse;
      cb.user = x->user;
    }
    live(e).set_exchange(cb);
    e->has_exchange = x && (x->forward || x->reverse);
    e->exchange = cb;
  });
}
int gr_engine_comm_layers(gr_engine *e)
{
  int r = -1;
  guarded([&] { r = live(e).comm_layers(); });
  return r;
}
int gr_engine_comm_width(gr_engine *e, int layer)
{
  int r = -1;
  guarded([&] { r = live(e).comm_width(layer); });
  return r;
}
int gr_engine_pack_forward(gr_engine *e, int layer, int n, const int *sendlist, double *buf)
{
  return guarded([&] { live(e).comm_rows(0, layer, n, sendlist, 0, buf, false); });
}
int gr_engine_unpack_forward(gr_engine *e, int layer, int n, int first, const double *buf)
{
  return guarded([&] { live(e).comm_rows(1, layer, n, nullptr, first, const_cast<double *>(buf), false); });
}
int gr_engine_pack_reverse(gr_engine *e, int layer, int n, int first, double *buf)
{
  return guarded([&] { live(e).comm_rows(2, layer, n, nullptr, first, buf, false); });
}
int gr_engine_unpack_reverse(gr_engine *e, int layer, int n, const int *sendlist, const double *buf)
{
  return guarded([&] { live(e).comm_rows(3, layer, n, sendlist, 0, const_cast<double *>(buf), false); });
}
int gr_engine_pack_forward_host(gr_engine *e, int layer, int n, const int *sendlist, double *buf)
{
  return guarded([&] { live(e).comm_rows(0, layer, n, sendlist, 0, buf, true); });
}
int gr_engine_unpack_forward_host(gr_engine *e, int layer, int n, int first, const double *buf)
{
  return guarded([&] { live(e).comm_rows(1, layer, n, nullptr, first, const_cast<double *>(buf), true); });
}
int gr_engine_pack_reverse_host(gr_engine *e, int layer, int n, int first, double *buf)
{
  return guarded([&] { live(e).comm_rows(2, layer, n, nullptr, first, buf, true); });
}
int gr_engine_unpack_reverse_host(gr_engine *e, int layer, int n, const int *sendlist, const double *buf)
{
  return guarded([&] { live(e).comm_rows(3, layer, n, sendlist, 0, const_cast<double *>(buf), true); });
}

int gr_compute_lammps_device(gr_engine *e, int nlocal, int nall, int ntypes, const int *type, const double *x, int inum, const int *ilist,
                             const int *numneigh, const int *neighbors, int64_t stride_i, int64_t stride_k, int neighmask, const int *owner,
                             unsigned flags, double *energy, double *f, double *virial, double *eatom)
{
  return guarded([&] {
    if (!e || (nall > 0 && (!type || !x)) || (inum > 0 && (!ilist || !numneigh || !neighbors))) throw grhip::InvalidArgument("null argument");
    if (nlocal < 0 || nall < nlocal || inum < 0 || ntypes < 0) throw grhip::InvalidArgument("atom counts out of range");
    grhip::Engine &eng = live(e);
    if (hipSetDevice(eng.device_index()) != hipSuccess) throw grhip::Error("hipSetDevice failed");
    auto on_device = [&](const void *p, const char *name) {
      if (!p) return;
      hipPointerAttribute_t at;
      if (hipPointerGetAttributes(&at, p) != hipSuccess || at.type != hipMemoryTypeDevice || at.device != eng.device_index()) {
        (void) hipGetLastError();
        throw grhip::InvalidArgument(std::string(name) + " must be memory of the engine's GPU");
      }
    };
    on_device(type, "type"); on_device(x, "x"); on_device(ilist, "ilist"); on_device(numneigh, "numneigh");
    on_device(neighbors, "neighbors"); on_device(owner, "owner"); on_device(f, "f"); on_device(eatom, "eatom");
    if (!e->bnl_stream && hipStreamCreateWithFlags(&e->bnl_stream, hipStreamNonBlocking) != hipSuccess) throw grhip::Error("hipStreamCreate failed");
    if (!e->lmp) e->lmp = std::make_unique<grhip::LammpsDeviceList>();
    grhip::LammpsDeviceList &W = *e->lmp;
    hipStream_t st = e->bnl_stream;
    // work queued by the caller on other streams (the arrays that hold the inputs) is finished first
    if (hipDeviceSynchronize() != hipSuccess) throw grhip::Error("hipDeviceSynchronize failed");
    grhip::RunFlags fl;
    fl.energy_only = (flags & GR_FLAG_ENERGY_ONLY) != 0;
    fl.eatom = (flags & GR_FLAG_EATOM) != 0 && eatom;
    fl.vatom = (flags & GR_FLAG_VATOM) != 0;
    const bool nodes = !owner && nall > nlocal && (e->has_exchange || eng.comm_layers() == 0);
    grhip::LmpListDev L{};
    L.type = type; L.x = x; L.numneigh = numneigh; L.neighbors = neighbors; L.stride_i = stride_i; L.stride_k = stride_k;
    L.owner = owner; L.nlocal = nlocal; L.nall = nall; L.neighmask = neighmask; L.nodes = nodes ? 1 : 0;
    if ((flags & GR_FLAG_SAME_LIST) && W.kept && W.serial == eng.upload_serial() && W.nlocal == nlocal && W.nall == nall && W.inum == inum &&
        W.nodes == L.nodes && W.neighmask == neighmask && W.stride_i == stride_i && W.stride_k == stride_k && W.neighbors == neighbors &&
        W.type == type && W.numneigh == numneigh && W.owner == owner) {
      // the steps between two reneighbourings: same rows, same bonds, new bond vectors written into the engine's array
      L.idx = W.idx.as<int>(); L.atom = W.atom.as<int>(); L.mapped = W.mapped.as<unsigned char>(); L.n = W.n;
      if (W.n > 0 && W.nb > 0) {
        double *rij = eng.bond_vectors_device();
        hipLaunchKernelGGL(grhip::k_lmp_rows<true>, dim3((unsigned) ((W.n + 127) / 128)), dim3(128), 0, st, L, (int *) nullptr, (int *) nullptr,
                           (const long long *) W.offset.as<long long>(), W.j.as<int>(), rij);
        if (hipStreamSynchronize(st) != hipSuccess) throw grhip::Error("the renewal of the bond vectors failed");
      }
      eng.run(fl);
      eng.fetch_add_device(nodes ? nullptr : W.atom.as<int>(), energy, f, virial, fl.eatom ? eatom : nullptr);
      e->lmp_nall = nall;
      e->lmp_serial = eng.upload_serial();
      e->lmp_on_device = true;
      return;
    }
    W.kept = false;
    // atom types and the atom list: 4 bytes per atom to the host, where the rows of the engine and its element tiles are laid out
    std::vector<int> ty((size_t) nall), il((size_t) inum);
    if (nall > 0 && hipMemcpy(ty.data(), type, sizeof(int) * (size_t) nall, hipMemcpyDeviceToHost) != hipSuccess) throw grhip::Error("copy of the atom types failed");
    if (inum > 0 && hipMemcpy(il.data(), ilist, sizeof(int) * (size_t) inum, hipMemcpyDeviceToHost) != hipSuccess) throw grhip::Error("copy of ilist failed");
    std::vector<unsigned char> mapped((size_t) ntypes + 1, 0);
    for (int t = 1; t <= ntypes; t++) mapped[t] = eng.cutoff(t, t) > 0.0;
    for (int a = 0; a < nall; a++)
      if (ty[a] < 1 || ty[a] > ntypes) throw grhip::InvalidArgument("types must be 1 .. ntypes");
    // ghosts as atoms of their own, as in gr_compute_lammps: the engine's rows are the owned atoms in LAMMPS order
    if (nodes)
      for (int a = 0; a < nall; a++)
        if (!mapped[ty[a]]) throw grhip::InvalidArgument("with an exchange every owned and ghost atom needs a type with a model element");
    std::vector<int> idx((size_t) nlocal, -1), atom, tq;
    std::vector<char> central((size_t) nlocal, 0);
    for (int q = 0; q < inum; q++) {
      const int i = il[q];
      if (i < 0 || i >= nlocal) throw grhip::InvalidArgument("ilist must index owned atoms");
      if (!mapped[ty[i]]) throw grhip::Error("atom " + std::to_string(i) + " of unmapped type " + std::to_string(ty[i]) + " in the atom list");
      central[i] = 1;
    }
    for (int i = 0; i < nlocal; i++) {
      if (!mapped[ty[i]]) continue;
      if (!central[i]) throw grhip::InvalidArgument("every owned atom of a mapped type must be in ilist (sub-lists are not supported)");
      idx[i] = (int) atom.size();
      atom.push_back(i);
      tq.push_back(ty[i]);
    }
    const int n = (int) atom.size();
    if (nodes) tq.insert(tq.end(), ty.begin() + nlocal, ty.end());    // n = nlocal here: the types of all nall atoms
    auto put = [&](grhip::DevBuf &b, const void *src, size_t bytes) {
      b.ensure(std::max<size_t>(bytes, 8));
      if (bytes && hipMemcpyAsync(b.p, src, bytes, hipMemcpyHostToDevice, st) != hipSuccess) throw grhip::Error("copy to the device failed");
    };
    put(W.idx, idx.data(), sizeof(int) * (size_t) nlocal);
    put(W.atom, atom.data(), sizeof(int) * (size_t) n);
    put(W.mapped, mapped.data(), mapped.size());
    const int zero = 0;
    put(W.err, &zero, sizeof(int));
    W.count.ensure(sizeof(int) * (size_t) std::max(n, 1));
    W.offset.ensure(sizeof(long long) * (size_t) (n + 1));
    L.idx = W.idx.as<int>(); L.atom = W.atom.as<int>(); L.mapped = W.mapped.as<unsigned char>(); L.n = n;
    W.nb = 0;
    if (n > 0) {
      const dim3 grid((unsigned) ((n + 127) / 128)), block(128);
      hipLaunchKernelGGL(grhip::k_lmp_rows<false>, grid, block, 0, st, L, W.count.as<int>(), W.err.as<int>(), (const long long *) nullptr, (int *) nullptr,
                         (double *) nullptr);
      hipLaunchKernelGGL(grhip::k_scan, dim3(1), dim3(1024), 0, st, W.count.as<int>(), n, W.offset.as<long long>());
      long long total = 0;
      int err = 0;
      if (hipMemcpyAsync(&total, W.offset.as<long long>() + n, sizeof(total), hipMemcpyDeviceToHost, st) != hipSuccess ||
          hipMemcpyAsync(&err, W.err.p, sizeof(err), hipMemcpyDeviceToHost, st) != hipSuccess || hipStreamSynchronize(st) != hipSuccess)
        throw grhip::Error("the conversion of the neighbour list failed");
      if (err == 1) throw grhip::InvalidArgument("neighbour index outside the owned and ghost atoms");
      if (err == 2) throw grhip::InvalidArgument(owner ? "the owner of a ghost atom is not an owned atom of the same type"
                                                       : "ghost neighbours need the owner map (the owned atom each ghost is an image of) or an exchange");
      W.nb = total;
      W.j.ensure(sizeof(int) * (size_t) std::max<int64_t>(W.nb, 1));
      W.rij.ensure(sizeof(double) * 3 * (size_t) std::max<int64_t>(W.nb, 1));
      hipLaunchKernelGGL(grhip::k_lmp_rows<true>, grid, block, 0, st, L, (int *) nullptr, (int *) nullptr, (const long long *) W.offset.as<long long>(),
                         W.j.as<int>(), W.rij.as<double>());
    } else {
      const long long z = 0;
      put(W.offset, &z, sizeof(z));
    }
    if (hipStreamSynchronize(st) != hipSuccess) throw grhip::Error("the conversion of the neighbour list failed");
    grhip::DeviceCsr in;
    in.n = n;
    in.types = tq.data();
    in.nb = W.nb;
    in.offset = W.offset.as<int64_t>();
    in.j = W.j.as<int>();
    in.rij = W.rij.as<double>();
    in.n_nodes = nodes ? nall : 0;
    eng.upload_device(in);
    W.kept = true;
    W.serial = eng.upload_serial();
    W.n = n; W.nlocal = nlocal; W.nall = nall; W.inum = inum; W.nodes = L.nodes; W.neighmask = neighmask;
    W.stride_i = stride_i; W.stride_k = stride_k; W.neighbors = neighbors; W.type = type; W.numneigh = numneigh; W.owner = owner;
    eng.run(fl);
    eng.fetch_add_device(nodes ? nullptr : W.atom.as<int>(), energy, f, virial, fl.eatom ? eatom : nullptr);
    e->lmp_nall = nall;
    e->lmp_serial = eng.upload_serial();
    e->lmp_on_device = true;
  });
}

namespace {
// rows of ncomp components (6: vatom, 9: cvatom) of the last LAMMPS call added to the caller's array
void lammps_add_virials(gr_engine *e, int nall, double *vatom, int ncomp, bool device)
{
  if (!e || !vatom) throw grhip::InvalidArgument("null argument");
  grhip::Engine &eng = live(e);
  if (device) {
    if (e->lmp_nall != nall || !e->lmp_on_device || e->lmp_serial != eng.upload_serial() || !e->lmp)
      throw grhip::Error("the per-atom virials of the device call follow a gr_compute_lammps_device call with GR_FLAG_VATOM on the same atoms");
    eng.add_vatom_device(e->lmp->nodes ? nullptr : e->lmp->atom.as<int>(), vatom, ncomp);
    return;
  }
  if (e->lmp_nall != nall || e->lmp_on_device || e->lmp_serial != eng.upload_serial())
    throw grhip::Error("the per-atom virials follow a gr_compute_lammps call with GR_FLAG_VATOM on the same atoms");
  const bool nodes = e->lmp_rows.empty();
  const size_t rows = nodes ? (size_t) nall : e->lmp_rows.size();
  std::vector<double> v((size_t) ncomp * std::max<size_t>(rows, 1));
  eng.fetch_vatom(v.data(), ncomp, (long long) rows);
  for (size_t q = 0; q < rows; q++) {
    const size_t a = nodes ? q : (size_t) e->lmp_rows[q];
    for (int k = 0; k < ncomp; k++) vatom[(size_t) ncomp * a + k] += v[(size_t) ncomp * q + k];
  }
}
}    // namespace

int gr_lammps_add_vatom(gr_engine *e, int nall, double *vatom)
{
  return guarded([&] { lammps_add_virials(e, nall, vatom, 6, false); });
}
int gr_lammps_add_cvatom(gr_engine *e, int nall, double *cvatom)
{
  return guarded([&] { lammps_add_virials(e, nall, cvatom, 9, false); });
}
int gr_lammps_add_vatom_device(gr_engine *e, int nall, double *vatom)
{
  return guarded([&] { lammps_add_virials(e, nall, vatom, 6, true); });
}
int gr_lammps_add_cvatom_device(gr_engine *e, int nall, double *cvatom)
{
  return guarded([&] { lammps_add_virials(e, nall, cvatom, 9, true); });
}

int gr_system_create(gr_engine *e, double skin, gr_system **out)
{
  return guarded([&] {
    if (!e || !out) throw grhip::InvalidArgument("null argument");
    *out = nullptr;
    if (!(std::isfinite(skin) && skin >= 0.0)) throw grhip::InvalidArgument("skin must be a finite number >= 0");
    auto s = std::make_unique<gr_system>();
    s->eng = e;
    s->skin = skin;
    s->cutoff = live(e).max_cutoff();
    if (hipSetDevice(live(e).device_index()) != hipSuccess || hipStreamCreate(&s->stream) != hipSuccess)
      throw grhip::Error("gr_system_create: cannot create a stream on the engine's device");
    *out = s.release();
  });
}

void gr_system_free(gr_system *s) { delete s; }
int gr_system_rebuilds(const gr_system *s) { return s ? s->rebuilds : 0; }
int gr_system_list_on_device(const gr_system *s) { return s && s->have && s->on_device ? 1 : 0; }

int gr_system_compute(gr_system *s, int n, const int *types, const double *positions, const double *cell, const unsigned char *pbc,
                      unsigned flags, double *energy, double *forces, double *virial, double *eatom)
{
  // one attempt; an allocation failure inside leaves as std::bad_alloc
  auto attempt = [&] {
    if (!s || !cell || !pbc || (n > 0 && (!types || !positions))) throw grhip::InvalidArgument("null argument");
    if (n < 0) throw grhip::InvalidArgument("negative atom count");
    if (!(s->cutoff > 0.0)) throw grhip::Error("the engine has no positive cutoff");
    grhip::Engine &eng = live(s->eng);
    if (hipSetDevice(eng.device_index()) != hipSuccess) throw grhip::Error("hipSetDevice failed");
    // list policy of the reference (python/grace_runtime/neighbors.py:68-89): rebuild when the atoms, the cell or the
    // boundary conditions change or an atom moved more than skin / 2 since the last build
    if (s->generation != s->eng->generation) {    // the engine was reset: what was uploaded is gone
      s->have = false;
      s->generation = s->eng->generation;
    }
    bool rebuild = !s->have || n != s->n || std::memcmp(pbc, s->pbc, 3) != 0 || std::memcmp(cell, s->cell.data(), 9 * sizeof(double)) != 0 ||
                   (n > 0 && std::memcmp(types, s->types.data(), sizeof(int) * (size_t) n) != 0);
    if (!rebuild) {
      const double lim = 0.25 * s->skin * s->skin;
      for (int a = 0; a < n && !rebuild; a++) {
        const double dx = positions[3 * a] - s->x0[3 * (size_t) a], dy = positions[3 * a + 1] - s->x0[3 * (size_t) a + 1],
                     dz = positions[3 * a + 2] - s->x0[3 * (size_t) a + 2];
        rebuild = dx * dx + dy * dy + dz * dz > lim;
      }
    }
    std::vector<double> x((size_t) 3 * n);
    if (rebuild) {
      s->have = false;
      const double reach = s->cutoff + s->skin;
      double pc[9], sh[3];
      padded_cell(cell, pbc, positions, n, reach, pc, sh);
      std::vector<double> xs((size_t) 3 * n);
      for (int a = 0; a < n; a++)
        for (int d = 0; d < 3; d++) xs[3 * (size_t) a + d] = positions[3 * a + d] + sh[d];
      const bool p[3] = {pbc[0] != 0, pbc[1] != 0, pbc[2] != 0};
      s->on_device = s->nl.build(xs.data(), n, pc, p, reach, s->stream);
      if (!s->on_device) s->host_nl = grhip::neighbor_search(xs.data(), n, pc, p, reach, 8);
      s->perm = s->on_device ? s->nl.perm : s->host_nl.perm;
      std::vector<int> ty(n);
      for (int q = 0; q < n; q++) {
        const int64_t a = s->perm[q];
        ty[q] = types[a];
        for (int d = 0; d < 3; d++) x[3 * (size_t) q + d] = positions[3 * a + d];
      }
      const std::vector<double> dummy(3, 0.0);
      if (s->on_device) {
        s->x_dev.ensure(std::max<size_t>(sizeof(double) * 3 * (size_t) n, 8));
        if (n > 0 && hipMemcpy(s->x_dev.p, x.data(), sizeof(double) * 3 * (size_t) n, hipMemcpyHostToDevice) != hipSuccess)
          throw grhip::Error("copy of the positions to the device failed");
        grhip::DeviceCsr in;
        in.n = n;
        in.types = ty.data();
        in.nb = s->nl.nb;
        in.offset = s->nl.offset.as<int64_t>();
        in.j = s->nl.j.as<int>();
        in.image = s->nl.image.as<int>();
        in.x = s->x_dev.as<double>();
        in.nimages = (int64_t) s->nl.shifts.size() / 3;
        in.shifts = in.nimages ? s->nl.shifts.data() : dummy.data();
        eng.upload_device(in);
      } else {
        const grhip::NeighborList &nl = s->host_nl;
        const int64_t nimg = (int64_t) nl.shifts.size() / 3;
        eng.upload(make_input(n, ty.data(), nl.offset.data(), nl.j.data(), nullptr, x.data(), nl.image.data(), nimg ? nl.shifts.data() : dummy.data(), nimg));
      }
      s->n = n;
      s->types.assign(types, types + n);
      s->x0.assign(positions, positions + 3 * (size_t) n);
      s->cell.assign(cell, cell + 9);
      std::memcpy(s->pbc, pbc, 3);
      s->have = true;
      s->rebuilds++;
    } else {
      for (int q = 0; q < n; q++) {
        const int64_t a = s->perm[q];
        for (int d = 0; d < 3; d++) x[3 * (size_t) q + d] = positions[3 * a + d];
      }
      eng.update_positions(x.data());
    }
    grhip::RunFlags fl;
    fl.energy_only = (flags & GR_FLAG_ENERGY_ONLY) != 0;
    fl.eatom = (flags & GR_FLAG_EATOM) != 0 && eatom;
    fl.vatom = (flags & GR_FLAG_VATOM) != 0;
    fl.uq = (flags & GR_FLAG_UQ) != 0;
    eng.run(fl);
    std::vector<double> f((size_t) 3 * n), ea(fl.eatom ? n : 0);
    eng.fetch(energy, forces ? f.data() : nullptr, virial, fl.eatom ? ea.data() : nullptr);
    for (int q = 0; q < n; q++) {
      const int64_t a = s->perm[q];
      if (forces && !fl.energy_only)
        for (int d = 0; d < 3; d++) forces[3 * a + d] = f[3 * (size_t) q + d];
      if (fl.eatom) eatom[a] = ea[q];
    }
  };
  // Allocation failure with the automatic chunk (python/kk/kk_api.h:72-75, kk_core.cpp:453-497): the work buffers go back,
  // the chunk is halved (never below 512 atoms) and kept for later calls, and the call starts again; when 512 atoms per
  // pass do not fit either, or the chunk was fixed by the caller, the failure is reported and the engine stays usable.
  return guarded([&] {
    for (;;) {
      try {
        attempt();
        return;
      } catch (const std::bad_alloc &) {
        grhip::Engine &eng = live(s->eng);
        const int used = eng.chunksize_used() > 0 ? eng.chunksize_used() : n;
        s->have = false;
        eng.release_buffers();
        if (!s->auto_chunk || used <= 512)
          throw grhip::Error("the structure (" + std::to_string(n) + " atoms) does not fit the GPU memory " +
                             (s->auto_chunk ? "even in chunks of 512 atoms" : "with the chunk size that was asked for") +
                             "; use a GPU with more memory or a smaller chunksize");
        int next = 512;
        while (2 * next < used) next *= 2;
        grhip::log_message(1, "device allocation failed with " + std::to_string(used) + " atoms per pass; trying again with " + std::to_string(next));
        try {
          eng.set_chunksize(next);
          s->eng->chunk_request = next;
        } catch (const grhip::InvalidArgument &) {    // an engine that evaluates structures in one pass only
          throw grhip::Error("the structure (" + std::to_string(n) + " atoms) does not fit the GPU memory in one pass, and this model kind is "
                             "not evaluated in chunks");
        }
      }
    }
  });
}

int gr_system_set_chunksize(gr_system *s, int atoms)
{
  return guarded([&] {
    if (!s) throw grhip::InvalidArgument("null system");
    live(s->eng).set_chunksize(atoms);
    s->eng->chunk_request = atoms;
    s->auto_chunk = atoms < 0;
  });
}

int gr_system_chunksize(const gr_system *s) { return s && s->eng && s->eng->eng ? s->eng->eng->chunksize_used() : 0; }

int64_t gr_engine_atoms_that_fit(gr_engine *e)
{
  int64_t r = 0;
  guarded([&] { r = live(e).atoms_that_fit(); });
  return r;
}

int gr_engine_set_chunksize(gr_engine *e, int atoms)
{
  return guarded([&] {
    live(e).set_chunksize(atoms);
    e->chunk_request = atoms;
  });
}

int gr_engine_chunksize(const gr_engine *e) { return e && e->eng ? e->eng->chunksize_used() : 0; }

int gr_engine_set_ordered_sums(gr_engine *e, int on)
{
  return guarded([&] {
    live(e).set_ordered_sums(on != 0);
    e->ordered = on != 0;
  });
}

int gr_engine_ordered_sums(const gr_engine *e) { return e && e->eng && e->eng->ordered_sums() ? 1 : 0; }

int gr_engine_set_spline(gr_engine *e, int intervals)
{
  return guarded([&] {
    live(e).set_spline(intervals);
    e->spline = intervals;
  });
}

int gr_engine_spline(const gr_engine *e) { return e && e->eng ? e->eng->spline() : 0; }

int gr_system_fetch_uq(gr_system *s, double *gamma, double *sigma, double *cluster)
{
  return guarded([&] {
    if (!s || !s->have) throw grhip::Error("gr_system_fetch_uq: no structure has been computed");
    const int n = s->n;
    std::vector<double> g((size_t) n), sg((size_t) n), cl((size_t) n);
    live(s->eng).fetch_uq(g.data(), sg.data(), cl.data());
    for (int q = 0; q < n; q++) {
      const int64_t a = s->perm[q];
      if (gamma) gamma[a] = g[q];
      if (sigma) sigma[a] = sg[q];
      if (cluster) cluster[a] = cl[q];
    }
  });
}

namespace {
void system_fetch_virials(gr_system *s, double *vatom, int ncomp)
{
  if (!s || !s->have) throw grhip::Error("the per-atom virials of a system: no structure has been computed");
  if (!vatom) throw grhip::InvalidArgument("null argument");
  const int n = s->n;
  std::vector<double> v((size_t) ncomp * n);
  live(s->eng).fetch_vatom(v.data(), ncomp);
  for (int q = 0; q < n; q++)
    for (int k = 0; k < ncomp; k++) vatom[(size_t) ncomp * s->perm[q] + k] = v[(size_t) ncomp * q + k];
}
}    // namespace

int gr_system_fetch_vatom(gr_system *s, double *vatom)
{
  return guarded([&] { system_fetch_virials(s, vatom, 6); });
}
int gr_system_fetch_cvatom(gr_system *s, double *cvatom)
{
  return guarded([&] { system_fetch_virials(s, cvatom, 9); });
}

// the list of the last rebuild: sizes, then the arrays (perm [n], offset [n + 1], j [nb], image [nb], shifts [nimages][3])
int gr_system_list_sizes(gr_system *s, int64_t *nbonds, int64_t *nimages)
{
  return guarded([&] {
    if (!s || !s->have) throw grhip::Error("gr_system_list_sizes: no list has been built");
    if (nbonds) *nbonds = s->on_device ? s->nl.nb : (int64_t) s->host_nl.j.size();
    if (nimages) *nimages = (int64_t) (s->on_device ? s->nl.shifts.size() : s->host_nl.shifts.size()) / 3;
  });
}

int gr_system_list_get(gr_system *s, int64_t *perm, int64_t *offset, int32_t *j, int32_t *image, double *shifts)
{
  return guarded([&] {
    if (!s || !s->have) throw grhip::Error("gr_system_list_get: no list has been built");
    std::memcpy(perm, s->perm.data(), sizeof(int64_t) * s->perm.size());
    if (s->on_device) {
      if (hipSetDevice(live(s->eng).device_index()) != hipSuccess) throw grhip::Error("hipSetDevice failed");
      bool ok = hipMemcpy(offset, s->nl.offset.p, sizeof(int64_t) * (size_t) (s->n + 1), hipMemcpyDeviceToHost) == hipSuccess;
      if (s->nl.nb > 0) {
        ok = ok && hipMemcpy(j, s->nl.j.p, sizeof(int32_t) * (size_t) s->nl.nb, hipMemcpyDeviceToHost) == hipSuccess;
        ok = ok && hipMemcpy(image, s->nl.image.p, sizeof(int32_t) * (size_t) s->nl.nb, hipMemcpyDeviceToHost) == hipSuccess;
      }
      if (!ok) throw grhip::Error("copy of the neighbour list from the device failed");
      std::memcpy(shifts, s->nl.shifts.data(), sizeof(double) * s->nl.shifts.size());
    } else {
      const grhip::NeighborList &nl = s->host_nl;
      std::memcpy(offset, nl.offset.data(), sizeof(int64_t) * nl.offset.size());
      std::memcpy(j, nl.j.data(), sizeof(int32_t) * nl.j.size());
      std::memcpy(image, nl.image.data(), sizeof(int32_t) * nl.image.size());
      std::memcpy(shifts, nl.shifts.data(), sizeof(double) * nl.shifts.size());
    }
  });
}

int gr_engine_upload_batch(gr_engine *e, int n, const int *types, const int64_t *offset, const int *j, const double *rij,
                           const double *positions, const int *image, const double *shifts, int64_t nimages, int nstruct,
                           const int *struct_of_atom)
{
  return guarded([&] {
    if (!e) throw grhip::InvalidArgument("null engine");
    if (n > 0 && !struct_of_atom) throw grhip::InvalidArgument("struct_of_atom is required");
    grhip::CsrInput in = make_input(n, types, offset, j, rij, positions, image, shifts, nimages);
    in.nstruct = nstruct;
    in.sid = struct_of_atom;
    live(e).upload(in);
  });
}

int gr_engine_fetch_batch(gr_engine *e, int nstruct, double *energy, double *forces, double *virial, double *eatom)
{
  return guarded([&] {
    if (!e) throw grhip::InvalidArgument("null engine");
    live(e).fetch_batch(nstruct, energy, forces, virial, eatom);
  });
}

namespace {
// Cell of a structure for the cell list: zero vectors and the vectors of open directions are replaced by unit
// directions normal to the periodic ones, long enough that no image is within reach; `shift` puts the atoms inside
// (python/grace_runtime/neighbors.py:27-47 of the reference).
void padded_cell(const double *cell, const unsigned char *pbc, const double *pos, int64_t n, double reach, double *out, double *shift)
{
  bool pad[3];
  std::vector<std::array<double, 3>> given;
  for (int k = 0; k < 3; k++) {
    const double *v = cell + 3 * k;
    pad[k] = !pbc[k] || (v[0] == 0.0 && v[1] == 0.0 && v[2] == 0.0);
    for (int d = 0; d < 3; d++) out[3 * k + d] = v[d];
    if (!pad[k]) given.push_back({v[0], v[1], v[2]});
  }
  shift[0] = shift[1] = shift[2] = 0.0;
  if (given.size() == 3) return;
  auto norm = [](std::array<double, 3> &a) {
    const double l = std::sqrt(a[0] * a[0] + a[1] * a[1] + a[2] * a[2]);
    if (!(l > 0.0)) throw grhip::InvalidArgument("the periodic cell vectors are linearly dependent");
    for (double &c : a) c /= l;
  };
  auto cross = [](const std::array<double, 3> &a, const std::array<double, 3> &b) {
    return std::array<double, 3>{a[1] * b[2] - a[2] * b[1], a[2] * b[0] - a[0] * b[2], a[0] * b[1] - a[1] * b[0]};
  };
  std::vector<std::array<double, 3>> dirs;
  if (given.empty()) dirs = {{1, 0, 0}, {0, 1, 0}, {0, 0, 1}};
  else if (given.size() == 2) {
    auto c = cross(given[0], given[1]);
    norm(c);
    dirs = {c};
  } else {
    std::array<double, 3> a = given[0];
    norm(a);
    int kmin = 0;
    for (int d = 1; d < 3; d++)
      if (std::fabs(a[d]) < std::fabs(a[kmin])) kmin = d;
    std::array<double, 3> ek{0, 0, 0};
    ek[kmin] = 1.0;
    auto b = cross(a, ek);
    norm(b);
    auto c = cross(a, b);
    norm(c);
    dirs = {b, c};
  }
  size_t q = 0;
  for (int k = 0; k < 3; k++) {
    if (!pad[k]) continue;
    const auto &d = dirs[q++];
    double lo = 0.0, hi = 0.0;
    for (int64_t a = 0; a < n; a++) {
      const double pr = pos[3 * a] * d[0] + pos[3 * a + 1] * d[1] + pos[3 * a + 2] * d[2];
      if (a == 0 || pr < lo) lo = pr;
      if (a == 0 || pr > hi) hi = pr;
    }
    const double len = (hi - lo) + 2.0 * reach + 1.0;
    for (int c = 0; c < 3; c++) {
      out[3 * k + c] = d[c] * len;
      if (n > 0) shift[c] += d[c] * (reach + 0.5 - lo);
    }
  }
}
}    // namespace

int gr_compute_batch(gr_engine *e, int nstruct, const int *natoms, const int *types, const double *positions, const double *cells,
                     const unsigned char *pbc, unsigned flags, int nthreads, double *energy, double *forces, double *virial,
                     double *eatom)
{
  return gr_compute_batch_uq(e, nstruct, natoms, types, positions, cells, pbc, flags, nthreads, energy, forces, virial, eatom, nullptr, nullptr,
                             nullptr);
}

int gr_compute_batch_uq(gr_engine *e, int nstruct, const int *natoms, const int *types, const double *positions, const double *cells,
                        const unsigned char *pbc, unsigned flags, int nthreads, double *energy, double *forces, double *virial,
                        double *eatom, double *gamma, double *sigma, double *cluster)
{
  return guarded([&] {
    if (!e || nstruct < 0 || (nstruct > 0 && (!natoms || !cells || !pbc))) throw grhip::InvalidArgument("null argument");
    if (nstruct == 0) return;
    const double rc = live(e).max_cutoff();
    if (!(rc > 0.0)) throw grhip::Error("the engine has no positive cutoff");
    std::vector<int64_t> start(nstruct + 1, 0);
    for (int s = 0; s < nstruct; s++) {
      if (natoms[s] < 0) throw grhip::InvalidArgument("negative atom count");
      start[s + 1] = start[s] + natoms[s];
    }
    const int64_t N = start[nstruct];
    if (N >= INT32_MAX) throw grhip::InvalidArgument("atom count out of range");
    if (N > 0 && (!types || !positions)) throw grhip::InvalidArgument("null argument");
    // one cell list per structure (they are independent: in parallel), then one list of all atoms
    std::vector<grhip::NeighborList> nls(nstruct);
    std::string err;
    bool invalid = false;
#pragma omp parallel for schedule(dynamic, 4) num_threads(nthreads > 0 ? nthreads : 1)
    for (int s = 0; s < nstruct; s++) {
      try {
        const int64_t n = natoms[s];
        const double *x = positions + 3 * start[s];
        double pc[9], sh[3];
        padded_cell(cells + 9 * (size_t) s, pbc + 3 * (size_t) s, x, n, rc, pc, sh);
        std::vector<double> xs((size_t) 3 * n);
        for (int64_t a = 0; a < n; a++)
          for (int d = 0; d < 3; d++) xs[3 * a + d] = x[3 * a + d] + sh[d];
        const bool p[3] = {pbc[3 * s] != 0, pbc[3 * s + 1] != 0, pbc[3 * s + 2] != 0};
        nls[s] = grhip::neighbor_search(xs.data(), n, pc, p, rc, 1);
      } catch (const grhip::InvalidArgument &ex) {
#pragma omp critical
        { err = ex.what(); invalid = true; }
      } catch (const std::exception &ex) {
#pragma omp critical
        { if (err.empty()) err = ex.what(); }
      }
    }
    if (!err.empty()) {
      if (invalid) throw grhip::InvalidArgument(err);
      throw grhip::Error(err);
    }
    std::vector<int64_t> offset(N + 1, 0), boff(nstruct + 1, 0), ioff(nstruct + 1, 0);
    for (int s = 0; s < nstruct; s++) {
      boff[s + 1] = boff[s] + (int64_t) nls[s].j.size();
      ioff[s + 1] = ioff[s] + (int64_t) nls[s].shifts.size() / 3;
    }
    const int64_t nb = boff[nstruct], nimg = ioff[nstruct];
    std::vector<int> ty(N), sid(N), jj(nb), img(nb);
    std::vector<double> x((size_t) 3 * N), shifts((size_t) 3 * std::max<int64_t>(nimg, 1), 0.0);
#pragma omp parallel for schedule(dynamic, 4) num_threads(nthreads > 0 ? nthreads : 1)
    for (int s = 0; s < nstruct; s++) {
      const grhip::NeighborList &nl = nls[s];
      const int64_t n = natoms[s], a0 = start[s];
      for (int64_t q = 0; q < n; q++) {
        const int64_t a = a0 + nl.perm[q];
        ty[a0 + q] = types[a];
        sid[a0 + q] = s;
        for (int d = 0; d < 3; d++) x[3 * (a0 + q) + d] = positions[3 * a + d];
        offset[a0 + q + 1] = boff[s] + nl.offset[q + 1];
      }
      for (size_t b = 0; b < nl.j.size(); b++) {
        jj[boff[s] + b] = (int) (a0 + nl.j[b]);
        img[boff[s] + b] = (int) (ioff[s] + nl.image[b]);
      }
      std::copy(nl.shifts.begin(), nl.shifts.end(), shifts.begin() + 3 * ioff[s]);
    }
    grhip::CsrInput in = make_input((int) N, ty.data(), offset.data(), jj.data(), nullptr, x.data(), img.data(), shifts.data(), nimg);
    in.nstruct = nstruct;
    in.sid = sid.data();
    live(e).upload(in);
    grhip::RunFlags fl;
    fl.energy_only = (flags & GR_FLAG_ENERGY_ONLY) != 0;
    fl.eatom = (flags & GR_FLAG_EATOM) != 0 && eatom;
    fl.vatom = (flags & GR_FLAG_VATOM) != 0;
    fl.uq = gamma || sigma || cluster;
    live(e).run(fl);
    std::vector<double> f((size_t) 3 * N), ea(fl.eatom ? N : 0);
    live(e).fetch_batch(nstruct, energy, forces ? f.data() : nullptr, virial, fl.eatom ? ea.data() : nullptr);
    std::vector<double> ug(gamma ? N : 0), us(sigma ? N : 0), uc(cluster ? N : 0);
    if (fl.uq) live(e).fetch_uq(gamma ? ug.data() : nullptr, sigma ? us.data() : nullptr, cluster ? uc.data() : nullptr);
    for (int s = 0; s < nstruct; s++)
      for (int64_t q = 0; q < natoms[s]; q++) {
        const int64_t a = start[s] + nls[s].perm[q], w = start[s] + q;
        if (forces && !fl.energy_only)
          for (int d = 0; d < 3; d++) forces[3 * a + d] = f[3 * (size_t) w + d];
        if (fl.eatom) eatom[a] = ea[w];
        if (gamma) gamma[a] = ug[w];
        if (sigma) sigma[a] = us[w];
        if (cluster) cluster[a] = uc[w];
      }
  });
}

int gr_compute_batch_device(gr_engine *e, int nstruct, const int *natoms, const int *types, const double *positions, const double *cells,
                            const unsigned char *pbc, unsigned flags, int64_t max_atoms, double *energy, double *forces, double *virial,
                            double *eatom, int *passes)
{
  return gr_compute_batch_device_uq(e, nstruct, natoms, types, positions, cells, pbc, flags, max_atoms, energy, forces, virial, eatom, nullptr,
                                    nullptr, nullptr, passes);
}

int gr_compute_batch_device_uq(gr_engine *e, int nstruct, const int *natoms, const int *types, const double *positions, const double *cells,
                               const unsigned char *pbc, unsigned flags, int64_t max_atoms, double *energy, double *forces, double *virial,
                               double *eatom, double *gamma, double *sigma, double *cluster, int *passes)
{
  return guarded([&] {
    if (passes) *passes = 0;
    if (!e || nstruct < 0 || (nstruct > 0 && (!natoms || !cells || !pbc))) throw grhip::InvalidArgument("null argument");
    if (max_atoms < 0) throw grhip::InvalidArgument("max_atoms must be >= 0");
    if (nstruct == 0) return;
    const double rc = live(e).max_cutoff();
    if (!(rc > 0.0)) throw grhip::Error("the engine has no positive cutoff");
    std::vector<int64_t> start((size_t) nstruct + 1, 0);
    for (int s = 0; s < nstruct; s++) {
      if (natoms[s] < 0) throw grhip::InvalidArgument("negative atom count");
      start[s + 1] = start[s] + natoms[s];
    }
    const int64_t N = start[nstruct];
    if (N >= INT32_MAX) throw grhip::InvalidArgument("atom count out of range");
    if (N > 0 && (!types || !positions)) throw grhip::InvalidArgument("null argument");
    if (!energy) throw grhip::InvalidArgument("the energy output is required");
    if (hipSetDevice(live(e).device_index()) != hipSuccess) throw grhip::Error("hipSetDevice failed");
    // the pointers must be memory of the engine's GPU: a host pointer here would fault in the kernels
    auto on_device = [&](const void *p, const char *name) {
      if (!p) return;
      hipPointerAttribute_t at;
      if (hipPointerGetAttributes(&at, p) != hipSuccess || at.type != hipMemoryTypeDevice || at.device != live(e).device_index()) {
        (void) hipGetLastError();
        throw grhip::InvalidArgument(std::string(name) + " must be memory of the engine's GPU");
      }
    };
    on_device(types, "types");
    on_device(positions, "positions");
    on_device(energy, "energy");
    on_device(forces, "forces");
    on_device(virial, "virial");
    on_device(eatom, "energies");
    on_device(gamma, "gamma");
    on_device(sigma, "atomic_sigma");
    on_device(cluster, "gmm_cluster");
    if (!e->bnl_stream && hipStreamCreateWithFlags(&e->bnl_stream, hipStreamNonBlocking) != hipSuccess) throw grhip::Error("hipStreamCreate failed");
    // work queued by the caller on the default stream (the tensors that hold the inputs) is finished first
    if (hipDeviceSynchronize() != hipSuccess) throw grhip::Error("hipDeviceSynchronize failed");
    grhip::RunFlags fl;
    fl.energy_only = (flags & GR_FLAG_ENERGY_ONLY) != 0;
    fl.eatom = (flags & GR_FLAG_EATOM) != 0 && eatom;
    fl.vatom = (flags & GR_FLAG_VATOM) != 0;
    fl.uq = gamma || sigma || cluster;
    // passes of whole structures with at most `limit` atoms (at least one structure each); every pass overwrites its outputs
    auto once = [&](int64_t limit) {
      if (passes) *passes = 0;
      if (!e->bnl) e->bnl = std::make_unique<grhip::BatchDeviceNeighbors>();
      grhip::BatchDeviceNeighbors &nl = *e->bnl;
      for (int g0 = 0; g0 < nstruct;) {
        int g1 = g0 + 1;
        const int64_t fit = std::min<int64_t>(limit, live(e).atoms_that_fit());    // what the device memory holds, once a pass has shown it
        while (g1 < nstruct && start[g1 + 1] - start[g0] <= fit) g1++;
        const int ns = g1 - g0;
        const int64_t a0 = start[g0], na = start[g1] - a0;
        nl.build(ns, natoms + g0, positions + 3 * a0, cells + 9 * (size_t) g0, pbc + 3 * (size_t) g0, rc, e->bnl_stream);
        // atom types: 4 bytes per atom to the host, where the element tiles of the tile GEMMs are laid out
        e->pin_types.ensure(sizeof(int) * (size_t) std::max<int64_t>(na, 1));    // pinned: the copy is a DMA, not a staged one
        int *ty_pinned = e->pin_types.as<int>();
        if (na > 0 && hipMemcpyAsync(ty_pinned, types + a0, sizeof(int) * (size_t) na, hipMemcpyDeviceToHost, e->bnl_stream) != hipSuccess)
          throw grhip::Error("copy of the atom types failed");
        if (hipStreamSynchronize(e->bnl_stream) != hipSuccess) throw grhip::Error("the device neighbour search failed");
        const std::vector<int> ty(ty_pinned, ty_pinned + na);
        grhip::DeviceCsr in;
        in.n = (int) na;
        in.types = ty.data();
        in.nb = nl.nb;
        in.offset = nl.offset.as<int64_t>();
        in.j = nl.j.as<int>();
        in.rij = nl.rij.as<double>();
        in.nstruct = ns;
        in.sid = nl.sid.data();
        live(e).upload_device(in);
        live(e).run(fl);
        live(e).fetch_batch_device(ns, energy + g0, forces ? forces + 3 * a0 : nullptr, virial ? virial + 6 * (size_t) g0 : nullptr,
                                   fl.eatom ? eatom + a0 : nullptr);
        if (fl.uq) live(e).fetch_uq(gamma ? gamma + a0 : nullptr, sigma ? sigma + a0 : nullptr, cluster ? cluster + a0 : nullptr);
        if (passes) ++*passes;
        g0 = g1;
      }
    };
    // After an allocation failure: a fresh engine (the failed one is half grown) and passes of half as many atoms, down
    // to 16384, from the first structure again; the limit found is kept for later calls (python/kk/kk_core.cpp:1452-1484)
    int64_t limit = std::min<int64_t>(max_atoms == 0 ? INT64_MAX : max_atoms, e->nall_cap);
    for (;;) {
      try {
        once(limit);
        return;
      } catch (const std::bad_alloc &) {
        const int64_t tried = std::min<int64_t>(limit, N);
        e->reset();
        if (tried <= 16384)
          throw grhip::Error("the batch (" + std::to_string(N) + " atoms) does not fit the GPU memory even in passes of " + std::to_string(tried) +
                             " atoms; use a GPU with more memory");
        limit = e->nall_cap = std::max<int64_t>(16384, tried / 2);
        grhip::log_message(1, "device allocation failed with batch passes of " + std::to_string(tried) + " atoms; trying again with " + std::to_string(limit));
      }
    }
  });
}
}
