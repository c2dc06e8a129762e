// C entry points over the *compiled reference* CPU drivers (TEST INFRASTRUCTURE, not product code).
//
// This file is our own glue; it contains no reference code.  oracle/Makefile compiles it together with the
// reference's own sources, read where they lie in the reference checkout, into oracle/_ref/libgrace_ref.so.
// The shared object is used (a) to validate the numpy restatement in oracle/grace_oracle.py and (b) as the CPU
// baseline that the benchmark times beside the GPU path.  Nothing in the shipped library links or loads it.
//
// Calls mirror python/src/core.cpp:292-396 of the reference (Model.compute on CSR bonds) and
// python/src/neighbors.cpp:15-95 (neighbor_search).
#include "grace/fused_1l.h"
#include "grace/fused_2l.h"
#include "grace/fused_3l.h"
#include "grace/model_kind.h"
#include "neighbors.h"

#include <cstring>
#include <memory>
#include <string>
#include <vector>

namespace {
struct Ref {
  int layers = 0;
  std::shared_ptr<grace::GRACE1LModel> m1;
  std::shared_ptr<grace::GRACE2LModel> m2;
  std::shared_ptr<grace::GRACE3LModel> m3;
  std::unique_ptr<grace::Grace1LFused> d1;
  std::unique_ptr<grace::Grace2LFused> d2;
  std::unique_ptr<grace::Grace3LFused> d3;
  grace::FusedSettings fs;
};
thread_local std::string g_err;
struct NL {
  grace_runtime::NeighborResult r;
};
}    // namespace

extern "C" {

const char *ref_last_error() { return g_err.c_str(); }

void *ref_open(const char *path, int spline_n)
{
  try {
    auto h = std::make_unique<Ref>();
    if (spline_n > 0) h->fs.spline_n = spline_n;
    const grace::ModelKind k = grace::model_kind(path);
    if (k == grace::ModelKind::Grace1L) {
      h->layers = 1;
      h->m1 = std::make_shared<grace::GRACE1LModel>();
      h->m1->load(path);
    } else if (k == grace::ModelKind::Grace2L) {
      h->layers = 2;
      h->m2 = std::make_shared<grace::GRACE2LModel>();
      h->m2->load(path);
    } else if (k == grace::ModelKind::Grace3L) {
      h->layers = 3;
      h->m3 = std::make_shared<grace::GRACE3LModel>();
      h->m3->load(path);
    } else {
      g_err = "not a GRACE kokkos.npz";
      return nullptr;
    }
    return h.release();
  } catch (const std::exception &e) {
    g_err = e.what();
    return nullptr;
  }
}

int ref_layers(void *hv) { return static_cast<Ref *>(hv)->layers; }

int ref_n_elements(void *hv)
{
  Ref *h = static_cast<Ref *>(hv);
  return h->m1 ? h->m1->n_elements : h->m2 ? h->m2->n_elements : h->m3->n_elements;
}

// type2mu has ntypes + 1 entries (types are 1-based), as Grace*LFused::setup_types
int ref_setup_types(void *hv, int ntypes, const int *type2mu)
{
  Ref *h = static_cast<Ref *>(hv);
  try {
    std::vector<int> t(type2mu, type2mu + ntypes + 1);
    grace::Logger log;
    if (h->m1) {
      h->d1 = std::make_unique<grace::Grace1LFused>(h->m1, h->fs, log);
      h->d1->setup_types(ntypes, t);
    } else if (h->m2) {
      h->d2 = std::make_unique<grace::Grace2LFused>(h->m2, h->fs, log);
      h->d2->setup_types(ntypes, t);
    } else {
      h->d3 = std::make_unique<grace::Grace3LFused>(h->m3, h->fs, log);
      h->d3->setup_types(ntypes, t);
    }
    return 0;
  } catch (const std::exception &e) {
    g_err = e.what();
    return 1;
  }
}

double ref_cutoff(void *hv, int t1, int t2)
{
  Ref *h = static_cast<Ref *>(hv);
  return h->d1 ? h->d1->cutoff(t1, t2) : h->d2 ? h->d2->cutoff(t1, t2) : h->d3->cutoff(t1, t2);
}

// CSR bonds; rij != null, or (x, image, shifts).  f [n][3], eatom [n] (may be null), virial [6] are OVERWRITTEN.
int ref_compute(void *hv, int n, const int *types, const int64_t *offset, const int *j, const double *rij,
                const double *x, const int *image, const double *shifts, int nthreads, int energy_only,
                double *energy, double *eatom, double *f, double *virial)
{
  Ref *h = static_cast<Ref *>(hv);
  try {
    grace::CsrBonds src{types, offset, j, rij, x, image, shifts};
    grace::Outputs out;
    std::memset(f, 0, sizeof(double) * 3 * (size_t) n);
    if (eatom) std::memset(eatom, 0, sizeof(double) * (size_t) n);
    out.f = f;
    out.eatom = eatom;
    grace::ComputeFlags fl;
    fl.eflag_atom = eatom != nullptr;
    fl.virial = !energy_only;
    fl.energy_only = energy_only != 0;
    grace::NoExchange ex;
    if (h->d1) h->d1->compute(n, nullptr, n, n, src, out, fl, nthreads);
    else if (h->d2) h->d2->compute(n, nullptr, n, n, src, ex, out, fl, nthreads);
    else if (h->d3) h->d3->compute(n, nullptr, n, n, src, ex, out, fl, nthreads);
    else {
      g_err = "setup_types not called";
      return 1;
    }
    *energy = out.energy;
    for (int k = 0; k < 6; k++) virial[k] = out.virial[k];
    return 0;
  } catch (const std::exception &e) {
    g_err = e.what();
    return 1;
  }
}

// The same call with per-atom virials: vatom [n][6] is OVERWRITTEN (Outputs::vatom, ComputeFlags::vflag_atom).
int ref_compute_vatom(void *hv, int n, const int *types, const int64_t *offset, const int *j, const double *rij, int nthreads, double *energy,
                      double *f, double *virial, double *vatom)
{
  Ref *h = static_cast<Ref *>(hv);
  try {
    grace::CsrBonds src{types, offset, j, rij, nullptr, nullptr, nullptr};
    grace::Outputs out;
    std::memset(f, 0, sizeof(double) * 3 * (size_t) n);
    std::memset(vatom, 0, sizeof(double) * 6 * (size_t) n);
    std::vector<double *> rows((size_t) n);
    for (int a = 0; a < n; a++) rows[(size_t) a] = vatom + 6 * (size_t) a;
    out.f = f;
    out.vatom = rows.data();
    grace::ComputeFlags fl;
    fl.virial = true;
    fl.vflag_atom = true;
    grace::NoExchange ex;
    if (h->d1) h->d1->compute(n, nullptr, n, n, src, out, fl, nthreads);
    else if (h->d2) h->d2->compute(n, nullptr, n, n, src, ex, out, fl, nthreads);
    else if (h->d3) h->d3->compute(n, nullptr, n, n, src, ex, out, fl, nthreads);
    else {
      g_err = "setup_types not called";
      return 1;
    }
    *energy = out.energy;
    for (int k = 0; k < 6; k++) virial[k] = out.virial[k];
    return 0;
  } catch (const std::exception &e) {
    g_err = e.what();
    return 1;
  }
}

// GRACE-1L / 2L / 3L with the UQ head (uqv6): forward only; gamma, sigma, cluster [n] per atom (Grace{1,2,3}LFused::enable_uq)
int ref_compute_uq(void *hv, int n, const int *types, const int64_t *offset, const int *j, const double *rij, const double *x,
                   const int *image, const double *shifts, int nthreads, double *energy, double *gamma, double *sigma, double *cluster)
{
  Ref *h = static_cast<Ref *>(hv);
  try {
    if (!h->d1 && !h->d2 && !h->d3) {
      g_err = "UQ: setup_types first";
      return 1;
    }
    if (h->d1) h->d1->enable_uq();
    else if (h->d2) h->d2->enable_uq();
    else h->d3->enable_uq();
    grace::CsrBonds src{types, offset, j, rij, x, image, shifts};
    grace::Outputs out;
    std::vector<double> f((size_t) 3 * n, 0.0);
    out.f = f.data();
    out.gamma = gamma;
    out.atomic_sigma = sigma;
    out.gmm_cluster = cluster;
    grace::ComputeFlags fl;
    fl.energy_only = true;
    fl.uq = true;
    grace::NoExchange ex;
    if (h->d1) h->d1->compute(n, nullptr, n, n, src, out, fl, nthreads);
    else if (h->d2) h->d2->compute(n, nullptr, n, n, src, ex, out, fl, nthreads);
    else h->d3->compute(n, nullptr, n, n, src, ex, out, fl, nthreads);
    *energy = out.energy;
    return 0;
  } catch (const std::exception &e) {
    g_err = e.what();
    return 1;
  }
}

void ref_close(void *hv) { delete static_cast<Ref *>(hv); }

// ---- neighbour list of the reference (python/src/neighbors.cpp)
void *ref_nl_build(const double *pos, int64_t n, const double *cell, const unsigned char *pbc, double cutoff,
                   int nthreads)
{
  try {
    const bool p[3] = {pbc[0] != 0, pbc[1] != 0, pbc[2] != 0};
    auto nl = std::make_unique<NL>();
    nl->r = grace_runtime::neighbor_search(pos, n, cell, p, cutoff, nthreads);
    return nl.release();
  } catch (const std::exception &e) {
    g_err = e.what();
    return nullptr;
  }
}
int64_t ref_nl_nbonds(void *v) { return (int64_t) static_cast<NL *>(v)->r.j.size(); }
int64_t ref_nl_nimages(void *v) { return (int64_t) static_cast<NL *>(v)->r.shifts.size() / 3; }
void ref_nl_get(void *v, int64_t *perm, int64_t *offset, int32_t *j, int32_t *image, double *shifts)
{
  const auto &r = static_cast<NL *>(v)->r;
  std::memcpy(perm, r.perm.data(), r.perm.size() * sizeof(int64_t));
  std::memcpy(offset, r.offset.data(), r.offset.size() * sizeof(int64_t));
  std::memcpy(j, r.j.data(), r.j.size() * sizeof(int32_t));
  std::memcpy(image, r.image.data(), r.image.size() * sizeof(int32_t));
  std::memcpy(shifts, r.shifts.data(), r.shifts.size() * sizeof(double));
}
void ref_nl_free(void *v) { delete static_cast<NL *>(v); }
}
