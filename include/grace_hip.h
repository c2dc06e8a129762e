/* C ABI of libgrace_hip.so: GRACE energy + forces + virial on one AMD MI355X (gfx950).
 *
 * Plain C types only; every call returns a status and never throws.  The entry points are what a binding of the
 * reference would call for this path; each comment names the reference interface it stands in for (paths relative
 * to the reference checkout).
 *
 * Threading: a gr_engine is not re-entrant (one call at a time per engine, as the reference's per-driver mutex,
 * python/src/core.cpp:343-344).  gr_last_error() is thread-local.
 */
#ifndef GRACE_HIP_H
#define GRACE_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct gr_model gr_model;
typedef struct gr_engine gr_engine;
typedef struct gr_nlist gr_nlist;
typedef struct gr_system gr_system;

enum {
  GR_OK = 0,
  GR_INVALID = 1, /* bad argument: the Python layer raises ValueError (nb::value_error / std::invalid_argument) */
  GR_ERROR = 2,   /* grace::Error / RuntimeError of the reference */
  GR_NOMEM = 3    /* std::bad_alloc of the reference: the engine stays usable */
};

enum {
  GR_FLAG_ENERGY_ONLY = 1, /* ComputeFlags::energy_only (libgrace/include/grace/system.h:118): no forces / virial */
  GR_FLAG_EATOM = 2,       /* ComputeFlags::eflag_atom (system.h:114): per-atom energies */
  GR_FLAG_UQ = 4,          /* ComputeFlags::uq (system.h:117): the UQ head; gr_engine_run and gr_system_compute */
  GR_FLAG_ACCUMULATE = 8,  /* gr_compute_csr: energy, forces, virial and per-atom energies are ADDED to the caller's values, as
                              the reference's Outputs accumulate (system.h:66-75); without it they are overwritten */
  GR_FLAG_VATOM = 32,      /* ComputeFlags::vflag_atom (system.h:115): per-atom virials, Outputs::vatom (system.h:71): every bond's
                              virial (x_i - x_j) (x) f_i goes half to each of its two atoms (add_vatom, libgrace/include/grace/
                              fused_cpu.h:1075-1087), so the rows add up to the total virial.  Needs forces.  The rows are read
                              with gr_engine_fetch_vatom / gr_system_fetch_vatom / gr_lammps_add_vatom after the call, or in
                              the nine-component centroid form with the _cvatom calls */
  GR_FLAG_SAME_LIST = 16   /* gr_compute_lammps_device: atom counts, types, ilist, neighbour list and owner map are those of the
                              previous call on this engine and only x has changed (LAMMPS: neighbor->ago > 0, the steps between
                              two reneighbourings): the converted list is kept, only the bond vectors are renewed and no array
                              makes a trip to the host.  The reference's engines walk the whole list in every run; this flag has
                              no counterpart there.  A hint: when the engine no longer holds that list the call converts anew */
};

typedef struct gr_model_info {
  int layers;     /* 1, 2, 3: GRACE-1L / 2L / 3L */
  int n_elements;
  int lmax;
  int n_radial;   /* radial channels of the first layer */
  int n_radbase;
  int max_order;  /* 3 or 4 */
  double rcut;    /* largest cutoff */
} gr_model_info;

/* message of the last failed call on this thread ("" if none).  grace::Error::what(). */
const char *gr_last_error(void);
/* Messages of the library (the automatic chunk, retries after a failed allocation): fn(user, level, message) with level 0
 * information, 1 warning -- the callback of grace::Logger (libgrace/include/grace/error.h:10-15).  NULL: dropped (default).
 * The callback may be called from any thread that calls into the library. */
typedef void (*gr_log_fn)(void *user, int level, const char *message);
void gr_set_logger(gr_log_fn fn, void *user);
/* library ABI version (the Python plug-in contract uses ABI = 7: python/grace_runtime/_gpu.py:18) */
int gr_abi_version(void);
/* number of HIP devices; gfx arch name of a device into buf ("" on failure).  _kk.arch(), _kk.initialize(device):
 * python/kk/kk_api.h:16-27 */
int gr_device_count(void);
int gr_device_arch(int device, char *buf, int len);

/* Load a kokkos.npz model: GRACE1LModel::load (libgrace/src/model_1l.cpp:16), GRACE2LModel::load
 * (libgrace/src/model_2l.cpp:26), GRACE3LModel::load (libgrace/src/model_3l.cpp:163); kind by grace::model_kind,
 * libgrace/include/grace/model_kind.h:19.  The same validation errors as the reference loaders. */
int gr_model_load(const char *npz_path, gr_model **out);
int gr_model_get_info(const gr_model *m, gr_model_info *info);
/* element name k (0 <= k < n_elements), "" when the file has none: Model.element_names, python/kk/kk_api.h:56 */
const char *gr_model_element_name(const gr_model *m, int k);
void gr_model_free(gr_model *m);

/* An engine for one type map: type2mu has ntypes + 1 entries, types are 1-based, type2mu[t] = model element or -1.
 * Grace1LFused(model, settings, log) + setup_types(ntypes, type2mu): libgrace/include/grace/fused_1l.h:28-31, likewise
 * Grace2LFused (fused_2l.h:32-39) and Grace3LFused (fused_3l.h:26-34); Grace1LKK::set_model / setup:
 * libgrace/include/grace/kk/grace_1l_kk.h:72-79.
 * precision 64: network arithmetic in fp64; 32: fp32 network, fp64 geometry, norms, readout and sums
 * (docs/advanced.md:37-38), for GRACE-1L, 2L and 3L models; any other value: GR_INVALID. */
int gr_engine_create(const gr_model *m, int ntypes, const int *type2mu, int precision, int device, gr_engine **out);
void gr_engine_free(gr_engine *e);
/* Drops the engine and every device buffer it holds and makes a fresh one from the same model, types, precision and
 * device: what the reference's GPU module does with an engine that an allocation failure left half grown
 * (python/kk/kk_core.cpp:478-497 poison / drop, the next compute attaches a fresh engine).  A structure uploaded before
 * is gone; a gr_system on this engine notices and uploads its structure again. */
int gr_engine_reset(gr_engine *e);
/* Frees the engine's work buffers (per-atom and per-bond arrays, the uploaded structure, the lists of the device entry
 * points); weights, tables and compiled kernels stay, the next call allocates again.  System.release_buffers() /
 * Batch.release_buffers() of the reference's GPU module (python/kk/kk_api.h:66-156; engines: release_buffers(),
 * kk/grace_1l_kk.h:72-113). */
int gr_engine_release_buffers(gr_engine *e);
/* Bytes of device memory the library's buffers hold (all engines of the process), and a cap on them: with a cap an
 * allocation that would pass it fails as one the device refuses (GR_NOMEM, or the retry of gr_compute_batch_device).
 * 0: no cap.  The part of the reference module's memory_info() / chunk-by-free-memory policy (kk/support.h:415-450) that
 * the caller controls; it also lets the allocation-failure paths be tested without exhausting a GPU. */
void gr_set_memory_limit(int64_t bytes);
int64_t gr_memory_in_use(void);
/* Grace1LFused::cutoff(t1, t2): fused_1l.h:32 */
double gr_engine_cutoff(const gr_engine *e, int t1, int t2);

/* One call on caller-supplied CSR bonds = _core.Model.compute (python/src/core.cpp:292-396) =
 * Grace1LFused::compute<CsrBonds>(n, nullptr, n, n, src, out, flags, nthreads) (fused_1l.h:41):
 * bonds of atom i are [offset[i], offset[i+1]); give rij [nb][3] or (positions [n][3], image [nb], shifts [nimages][3]).
 * types are 1-based.  Outputs: energy, forces [n][3], virial[6] = xx yy zz xy xz yz, eatom [n] (with GR_FLAG_EATOM);
 * overwritten, or added to with GR_FLAG_ACCUMULATE; null outputs are skipped.  Same argument errors as the reference binding. */
int gr_compute_csr(gr_engine *e, int n, const int *types, const int64_t *offset, const int *j, const double *rij,
                   const double *positions, const int *image, const double *shifts, int64_t nimages, unsigned flags,
                   double *energy, double *forces, double *virial, double *eatom);

/* The same call in three steps, for callers that keep the structure on the GPU between passes (System.compute
 * without a list rebuild, python/kk/kk_core.cpp:802-958): upload copies the CSR structure to the device, run
 * queues one pass on the engine's stream, fetch waits and copies results out. */
int gr_engine_upload(gr_engine *e, int n, const int *types, const int64_t *offset, const int *j, const double *rij,
                     const double *positions, const int *image, const double *shifts, int64_t nimages);
int gr_engine_run(gr_engine *e, unsigned flags);
int gr_engine_sync(gr_engine *e);
int gr_engine_fetch(gr_engine *e, double *energy, double *forces, double *virial, double *eatom);
/* in-cutoff bonds of the last pass */
int64_t gr_engine_edge_count(gr_engine *e);

/* Per-stage GPU times (HIP events on the engine's stream) of the last gr_engine_run, when profiling is on.
 * The reference's counterpart is the G2LF_PROF category table (libgrace/include/grace/fused_cpu.h:171-213). */
int gr_engine_set_profile(gr_engine *e, int on);
int gr_engine_stage_count(gr_engine *e);
int gr_engine_stage_get(gr_engine *e, int k, char *name, int name_len, double *ms, int *launches);
/* floating-point operations (2 per multiply-add) of the tile GEMMs stage k launched in that run: the channel-mixing
 * GEMMs of the FC layers and equivariant reduces over the functions the engine keeps live (the reference prunes the same
 * functions, libgrace/src/fused_1l.cpp:176-216); 0 for stages that are not tile GEMMs */
int gr_engine_stage_flops(gr_engine *e, int k, double *flops);

/* Radial functions of the GPU kernel: Rz, dRz [m][lmax+1][n_radial] = R_nl(x) z[mu_j][n] and d/dx, for x = r / rc.
 * Test hook for the radial-MLP kernel (the reference's counterpart is radial_x.h:29-60 evaluated on the host). */
int gr_engine_debug_radial(gr_engine *e, int m, const double *x, const int *mu_j, double *Rz, double *dRz);

/* gr_engine_debug_radial for callers that cannot allocate device memory (tight serving loops, harnesses that forbid
 * hipMalloc, code that runs between the captures of a HIP graph and must leave the allocator alone).  No counterpart in
 * the reference.  The call itself synchronises (it waits for the device on entry, so arrays that another stream is
 * still writing are complete, and for its own stream before it returns): it cannot be recorded INTO a graph.  x [m], mu_j [m], Rz and dRz [m][lmax+1]
 * [n_radial] are DEVICE arrays of the engine's GPU.  The staging rows of the radial kernel live in a fixed 32 MiB
 * device array of the library (one per GPU, held until the process ends), so the call makes no hipMalloc / hipFree:
 * m is bounded by 256 + 4 m + 2 m nl CP s <= 32 MiB (CP = n_radial padded to 16 / 32 / 64, s = 8 or 4 bytes; 13 000
 * arguments for a 32-channel lmax-4 model in fp64), a larger m gives GR_INVALID with the limit in the message.
 * GRACE-1L engines only.  The call returns when Rz and dRz are written.  All calls on one GPU share the array: the
 * library serialises them with one lock per GPU (calls of two threads or two engines wait for each other). */
int gr_engine_radial_noalloc(gr_engine *e, int m, const double *x, const int *mu_j, double *Rz, double *dRz);

/* Runs a plain device-to-device copy kernel (k_copy_calibration) over `bytes` bytes: the known-size kernel that the
 * rocprof memory counters (FETCH_SIZE, WRITE_SIZE) are scaled by.  No counterpart in the reference. */
int gr_engine_debug_copy(gr_engine *e, int64_t bytes);
/* Times that copy kernel and a read-only stream kernel over `bytes` bytes with HIP events and returns their rates in
 * GB/s (copy: bytes read + bytes written): the ceilings this GPU shows to a kernel bound by HBM, which the published peak
 * is not.  Measurement support of bench.py; no counterpart in the reference. */
int gr_engine_stream_rates(gr_engine *e, int64_t bytes, double *copy_gbs, double *read_gbs);

/* Neighbour list at `cutoff`, the exact list of grace_runtime::neighbor_search (python/src/neighbors.cpp:15-95):
 * perm [n] (new -> original index), offset [n+1], j [nb] (new indices), image [nb], shifts [nimages][3]. */
int gr_neighbor_build(int64_t n, const double *positions, const double *cell, const unsigned char *pbc, double cutoff,
                      int nthreads, gr_nlist **out);
int64_t gr_nlist_nbonds(const gr_nlist *l);
int64_t gr_nlist_nimages(const gr_nlist *l);
int gr_nlist_get(const gr_nlist *l, int64_t *perm, int64_t *offset, int32_t *j, int32_t *image, double *shifts);
void gr_nlist_free(gr_nlist *l);

/* Energy, forces (caller's atom order), virial of a periodic structure: neighbour list at the engine's largest
 * cutoff, permutation to bin order, one pass, forces permuted back.  The engine part of GRACERuntimeCalculator.
 * calculate -> _CpuEngine.compute (python/grace_runtime/calculator.py:204-224) without the Verlet skin. */
int gr_compute(gr_engine *e, int n, const int *types, const double *positions, const double *cell,
               const unsigned char *pbc, unsigned flags, double *energy, double *forces, double *virial, double *eatom);

/* UQ head (uqv6, gamma only) of GRACE-1L, GRACE-2L and GRACE-3L models: replaces GRACE1LModel::has_uq / validate_uq (libgrace/src/
 * model_1l.cpp:216-285) and GRACE2LModel's (libgrace/src/model_2l.cpp:404-478), Grace1LFused::enable_uq / uq_batch /
 * uq_flush (libgrace/src/fused_1l.cpp:584-636), Grace2LFused's UQ stage (libgrace/src/fused_2l.cpp:1156-1186: basis
 * blocks [I2 inputs, rho inputs], density channels total / I2 / rho), Grace3LFused::enable_uq / uq_layer (libgrace/src/
 * fused_3l.cpp:269-274, 1156-1201: one block per layer, the inputs of rho1, rho2, rho3, evaluated layer by layer; a
 * GRACE-3L file with a broken head does not load, libgrace/src/model_3l.cpp:453-463) and the gamma, atomic_sigma,
 * gmm_cluster outputs of Outputs (libgrace/include/grace/system.h:72-73).  A run with GR_FLAG_UQ (gr_engine_run,
 * gr_system_compute) evaluates per atom the extrapolation grade gamma, the Mahalanobis distance sigma to the nearest GMM
 * centroid of the atom's element and that cluster's index; the fetch calls copy them out ([n] each, NULL: skipped):
 * gr_engine_fetch_uq in the order of the uploaded list, gr_system_fetch_uq in the caller's atom order.
 * gr_model_has_uq: 1 when the file carries a UQ head; gr_model_validate_uq: GR_OK when it can be evaluated, else
 * GR_INVALID with the reason (no head, max_order 3, another schema, sizes that do not fit the model).  A run with
 * GR_FLAG_UQ on a model without a usable head gives GR_INVALID. */
int gr_model_has_uq(const gr_model *m);
int gr_model_validate_uq(const gr_model *m);
int gr_engine_fetch_uq(gr_engine *e, double *gamma, double *sigma, double *cluster);
/* Per-atom virials [atoms][6] = xx yy zz xy xz yz of the last pass with GR_FLAG_VATOM (gr_engine_run, gr_compute_csr):
 * rows in the order of the uploaded list (with ghost atoms as nodes: all of them); Outputs::vatom of the reference
 * (libgrace/include/grace/system.h:71).  GR_ERROR when that pass did not compute them. */
int gr_engine_fetch_vatom(gr_engine *e, double *vatom);
/* The same pass in the centroid form [atoms][9] = xx yy zz xy xz yz yx zx zy: the tensor (x_i - x_j) (x) f_i of every
 * bond is not symmetric, and this form keeps the components below the diagonal as well (RunInput::cvatom of the
 * reference's GPU engines, libgrace/include/grace/kk/grace_1l_kk.h:94, accumulated in kk/grace_1l_kk_impl.h:1344-1362).
 * The first six columns are those of gr_engine_fetch_vatom. */
int gr_engine_fetch_cvatom(gr_engine *e, double *cvatom);
int gr_system_fetch_uq(gr_system *s, double *gamma, double *sigma, double *cluster);
/* Per-atom virials [n][6] of the last gr_system_compute with GR_FLAG_VATOM, in the caller's atom order. */
int gr_system_fetch_vatom(gr_system *s, double *vatom);
/* The same in the centroid form [n][9] (gr_engine_fetch_cvatom). */
int gr_system_fetch_cvatom(gr_system *s, double *cvatom);

/* The call of a LAMMPS pair style on one MPI rank: owned and ghost atoms with LAMMPS' full neighbour list.  Replaces
 * Grace{1,2,3}LFused::compute<LammpsBonds>(inum, ilist, n_nodes, nmax_nodes, LammpsBonds{x, type, numneigh, firstneigh,
 * neighmask}, Exchange&, Outputs&, flags, nthreads) (libgrace/include/grace/system.h:14-20, fused_1l.h:41, fused_2l.h:49,
 * fused_3l.h:44) and the RunInput / RunOutput of the reference's GPU engines (kk/grace_1l_kk.h:80-113).
 * x [nall][3], type [nall] (1-based); neighbour indices are masked with neighmask (0x1FFFFFFF in LAMMPS); atoms of types
 * without a model element take no part.  owner [nall]: for a ghost atom the owned atom it is a periodic image of (LAMMPS:
 * atom->map(tag[j])); it stands in for the Exchange of the reference: the message of a ghost is its owner's, and what
 * the reference leaves on the ghosts for the reverse communication (forces, message adjoints) is added to the owner here.
 * May be NULL when no neighbour is a ghost.  Ghosts owned by another rank are not supported (one GPU, one rank).
 * As the reference's Outputs (system.h:66-75): forces are ADDED to f [nall][3], per-atom energies to eatom [nall];
 * energy and virial (xx yy zz xy xz yz) are returned.  ilist must hold every owned atom of a mapped type. */
int gr_compute_lammps(gr_engine *e, int nlocal, int nall, const int *type, const double *x, int inum, const int *ilist, const int *numneigh,
                      const int *const *firstneigh, int neighmask, const int *owner, unsigned flags, double *energy, double *f,
                      double *virial, double *eatom);

/* Message exchange between owned atoms and ghosts, for ghosts that are NOT images of this rank's atoms (several MPI
 * ranks): replaces the Exchange of the reference's drivers (libgrace/include/grace/system.h:53-60) and the comm surface of
 * its GPU engines (comm_width, pack_forward / unpack_forward / pack_reverse / unpack_reverse and their _host forms,
 * libgrace/include/grace/kk/grace_2l_kk.h:141-157, grace_3l_kk.h:313-324).
 * With an exchange installed (or a GRACE-1L engine, which has no message) gr_compute_lammps with owner = NULL keeps the
 * ghosts as atoms of their own: during the call forward(user, layer) is called when the message rows of the owned atoms of
 * `layer` (1 .. gr_engine_comm_layers: 0 for GRACE-1L, 1 for 2L, 2 for 3L) are complete -- it must fill the ghosts' rows,
 * as LAMMPS' comm->forward_comm does through pack_forward / unpack_forward -- and reverse(user, layer) when the adjoint rows
 * are complete -- it must add the ghosts' rows to their owners' (pack_reverse / unpack_reverse).  Forces left on ghosts
 * are added to f [nall][3] for LAMMPS' reverse communication of f.  Every owned and ghost atom needs a mapped type.
 * Row movers: gr_engine_comm_width doubles per atom; atoms by LAMMPS index (owned 0 .. nlocal-1, ghosts after);
 * pack_forward: rows of sendlist[0 .. n) -> buf; unpack_forward: buf -> rows of first .. first + n; pack_reverse: adjoint
 * rows of first .. first + n -> buf; unpack_reverse: buf ADDED to the adjoint rows of sendlist[0 .. n).  sendlist and buf
 * are device memory of the engine's GPU, host memory for the _host forms.  They may only be called from inside the
 * callbacks of the matching direction and layer; each returns when its copy is done. */
typedef struct gr_exchange {
  void (*forward)(void *user, int layer);
  void (*reverse)(void *user, int layer);
  void *user;
} gr_exchange;
int gr_engine_set_exchange(gr_engine *e, const gr_exchange *x);    /* NULL: none */
int gr_engine_comm_layers(gr_engine *e);
int gr_engine_comm_width(gr_engine *e, int layer);
int gr_engine_pack_forward(gr_engine *e, int layer, int n, const int *sendlist, double *buf);
int gr_engine_unpack_forward(gr_engine *e, int layer, int n, int first, const double *buf);
int gr_engine_pack_reverse(gr_engine *e, int layer, int n, int first, double *buf);
int gr_engine_unpack_reverse(gr_engine *e, int layer, int n, const int *sendlist, const double *buf);
int gr_engine_pack_forward_host(gr_engine *e, int layer, int n, const int *sendlist, double *buf);
int gr_engine_unpack_forward_host(gr_engine *e, int layer, int n, int first, const double *buf);
int gr_engine_pack_reverse_host(gr_engine *e, int layer, int n, int first, double *buf);
int gr_engine_unpack_reverse_host(gr_engine *e, int layer, int n, const int *sendlist, const double *buf);

/* The same call with every per-atom array in DEVICE memory of the engine's GPU: the RunInput / RunOutput of the
 * reference's GPU engines (libgrace/include/grace/kk/grace_1l_kk.h:80-103, grace_2l_kk.h:81-157, grace_3l_kk.h:232-324),
 * i.e. what a KOKKOS pair style holds.  type [nall], x [nall][3], ilist [inum], numneigh [nlocal] (by atom), owner [nall]
 * (or NULL), f [nall][3] and eatom [nall] (added to) are device pointers; the neighbour list is the 2-d view of the KOKKOS
 * list, element (i, k) at neighbors[i * stride_i + k * stride_k] (either layout).  ntypes: atom types of the run (the
 * engine's type map covers 1 .. ntypes).  The list is converted to the engine's rows on the device; the atom types and
 * ilist make one 4-byte-per-atom trip to the host for the layout of the rows.  energy and virial [6] are returned to the
 * host, as RunOutput.  The call waits for work queued on the device before it reads the inputs.  Same restrictions as
 * gr_compute_lammps. */
int gr_compute_lammps_device(gr_engine *e, int nlocal, int nall, int ntypes, const int *type, const double *x, int inum, const int *ilist,
                             const int *numneigh, const int *neighbors, int64_t stride_i, int64_t stride_k, int neighmask, const int *owner,
                             unsigned flags, double *energy, double *f, double *virial, double *eatom);

/* Adds the per-atom virials of the last gr_compute_lammps (host array) / gr_compute_lammps_device (device array) call
 * that carried GR_FLAG_VATOM to vatom [nall][6] by LAMMPS atom index: RunInput::vatom of the reference's GPU engines
 * (libgrace/include/grace/kk/grace_1l_kk.h:93,101).  With an owner map the halves of ghost atoms are on their owners'
 * rows; without one (nodes) they stay on the ghosts for LAMMPS' reverse communication. */
int gr_lammps_add_vatom(gr_engine *e, int nall, double *vatom);
int gr_lammps_add_vatom_device(gr_engine *e, int nall, double *vatom);
/* The same for the centroid form, cvatom [nall][9] = xx yy zz xy xz yz yx zx zy (RunInput::cvatom,
 * libgrace/include/grace/kk/grace_1l_kk.h:94): host array / device array. */
int gr_lammps_add_cvatom(gr_engine *e, int nall, double *cvatom);
int gr_lammps_add_cvatom_device(gr_engine *e, int nall, double *cvatom);

/* One structure resident on the device with a Verlet list at cutoff + skin: System of the reference's GPU module
 * (python/kk/kk_api.h:66-93, System::compute python/kk/kk_core.cpp:802-958; list policy python/grace_runtime/
 * neighbors.py:68-89: rebuild when types, cell or pbc change or an atom moved more than skin / 2).  The pair search of
 * a rebuild runs on the device (the reference's device list: libgrace/include/grace/kk/neighbors_kk.h) and gives the
 * list of gr_neighbor_build bond for bond; between rebuilds a call sends the positions only.  Results in the caller's
 * atom order, as gr_compute.  The engine must outlive the system and serves one system at a time.
 * gr_system_list_*: the list of the last rebuild (perm [n], offset [n + 1], j [nb], image [nb], shifts [nimages][3]);
 * gr_system_list_on_device: 1 when that list was searched on the device, 0 when the structure was handed to the host
 * search (atoms many thousands of cells apart). */
int gr_system_create(gr_engine *e, double skin, gr_system **out);
void gr_system_free(gr_system *s);
int gr_system_compute(gr_system *s, int n, const int *types, const double *positions, const double *cell, const unsigned char *pbc,
                      unsigned flags, double *energy, double *forces, double *virial, double *eatom);
/* Atoms per engine pass, which bounds the device memory of a large structure (System(chunksize) and System::chunksize()
 * of the reference's GPU module, python/kk/kk_api.h:72-75,86; the engines' chunksize, kk/grace_1l_kk.h:72-113; automatic
 * choice libgrace/include/grace/kk/support.h:425-450).  atoms = 0: all atoms in one pass; < 0 (the default): chosen from
 * the free device memory: one pass while the work buffers fit 70 % of it, else the largest power of two >= 512 that
 * fits, and halved (down to 512) when an allocation still fails; > 0: as given.  gr_*_chunksize: atoms per pass of the last
 * call, 0 for one pass.  All three engine kinds evaluate chunks: GRACE-1L chunk after chunk; GRACE-2L and GRACE-3L sweep
 * layer by layer over the chunks and repeat a layer's forward pass for a chunk before its reverse. */
/* Atoms of one pass whose work buffers fit 70 % of the device memory the library may use, from the bytes per atom the
 * last pass held (before any pass: 262144 / 131072 / 16384 atoms for GRACE-1L / 2L / 3L).  The batch entry points bound
 * their passes by it, as the reference sizes a batch pass from the free memory (libgrace/include/grace/kk/support.h:425-450,
 * python/kk/kk_core.cpp:1311-1347). */
int64_t gr_engine_atoms_that_fit(gr_engine *e);
int gr_engine_set_chunksize(gr_engine *e, int atoms);
int gr_engine_chunksize(const gr_engine *e);
int gr_system_set_chunksize(gr_system *s, int atoms);
int gr_system_chunksize(const gr_system *s);

/* Ordered sums: with on != 0 the engine adds forces, virial, energy and (GRACE-2L / 3L) the message adjoints in a fixed
 * order instead of with floating-point atomics, so that two calls on the same input return the same bits.  The reverse
 * kernels store every bond's contribution; the forces and message adjoints of the neighbours are gathered through the
 * bonds listed by neighbour atom (rebuilt every pass, each row in ascending order), the energy and virial of every
 * structure are summed over its atoms in ascending order.  The reference's GPU engines have no such mode: they document
 * last-bit variation from run to run (python/tests/test_gpu_several_calculators.py).  A GRACE-1L result does not depend
 * on the chunk size; a GRACE-2L / 3L result is the same for the same chunk size.  With ordered sums a run with
 * GR_FLAG_VATOM gives GR_INVALID, and so does a batch whose atoms are not grouped by structure.  A few per cent slower;
 * the multi-layer engines hold one more array of nI x channels values per bond of a chunk.  gr_engine_ordered_sums: 1
 * when on. */
int gr_engine_set_ordered_sums(gr_engine *e, int on);
int gr_engine_ordered_sums(const gr_engine *e);

/* Radial tables: intervals > 0 makes an engine take its radial functions from cubic tables of that many
 * intervals over r / rc in [0, 1] (per interval the cubic through the values and derivatives of the radial MLP at its two
 * ends), which is how the reference's CPU and GPU engines evaluate them: FusedSettings::spline_n, default 1024
 * (libgrace/include/grace/system.h:78), `spline` of Model / System / Batch (python/kk/kk_api.h:53,75), tables of
 * Grace1LFused::build_splines (libgrace/src/fused_1l.cpp:102-129), evaluation spline_eval (fused_cpu.h:1052-1074); the
 * tables here hold the engine's precision where the reference's hold fp32.  0, the default of gr_engine_create: the
 * radial MLP itself is evaluated for every bond (no interpolation error).  16 .. 1048576, else GR_INVALID.  GRACE-3L
 * engines hold one table per ordered pair of the engine's species and per layer, of intervals / 2 (at least 16) for
 * layers 1 and 2 and of `intervals` for layer 3 (libgrace/src/fused_3l.cpp:491-533, spline_n_3l of libgrace/include/
 * grace/system.h:95-103); tables of the three layers that together exceed 2048 MB (Grace3LKK::spline_mb, libgrace/
 * include/grace/kk/grace_3l_kk.h:1264) are not built: the engine says so through the logger and keeps evaluating its
 * radial MLPs.  gr_engine_spline: the value set. */
int gr_engine_set_spline(gr_engine *e, int intervals);
int gr_engine_spline(const gr_engine *e);
int gr_system_rebuilds(const gr_system *s);
int gr_system_list_on_device(const gr_system *s);
int gr_system_list_sizes(gr_system *s, int64_t *nbonds, int64_t *nimages);
int gr_system_list_get(gr_system *s, int64_t *perm, int64_t *offset, int32_t *j, int32_t *image, double *shifts);

/* Several independent structures in one pass (the batched small-structure workload).  Replaces Batch::compute of the
 * reference GPU module (python/kk/kk_api.h:116-156, python/kk/kk_core.cpp:960-1160: structures packed into one atom
 * list, one engine pass, per-structure energies and virials).
 * gr_compute_batch: natoms [nstruct], types / positions of all atoms structure after structure, cells [nstruct][3][3],
 * pbc [nstruct][3]; per structure the list of gr_compute (open directions padded), all lists built on `nthreads` host
 * threads; energy [nstruct], virial [nstruct][6], forces [N][3] and eatom [N] in the caller's atom order.
 * gr_engine_upload_batch / gr_engine_fetch_batch: the resident form for a caller with its own lists: one CSR list over
 * all atoms (no bond may join two structures) and the structure of every atom. */
int gr_compute_batch(gr_engine *e, int nstruct, const int *natoms, const int *types, const double *positions, const double *cells,
                     const unsigned char *pbc, unsigned flags, int nthreads, double *energy, double *forces, double *virial,
                     double *eatom);
/* The same pass with the atoms and the results in device memory: replaces Batch::compute_device of the reference GPU
 * module (python/kk/kk_api.h:107-120,141-146; binding python/kk/kk_module.cpp:142-193, which hands over DLPack arrays of
 * the module's GPU).  types [N] (int32) and positions [N][3] are DEVICE pointers of the engine's GPU, as are the outputs
 * energy [nstruct], forces [N][3], virial [nstruct][6], eatom [N] (NULL: not wanted); natoms, cells, pbc are host arrays
 * as in gr_compute_batch.  A direction is periodic when its flag is set and its cell vector is not zero.  The neighbour
 * lists are built on the device (the reference: kk/neighbors_kk.h BatchNeighborListKK); positions, forces and per-atom
 * energies never visit the host (the atom types do, 4 bytes per atom, for the layout of the element tiles).  Results in
 * the caller's atom order.  The call waits for work queued on the device before it reads the inputs and returns when
 * the outputs are written.  A pointer that is not memory of the engine's GPU gives GR_INVALID.
 * max_atoms: the structures go through the engine in passes of whole structures with at most max_atoms atoms (at least
 * one structure per pass), which bounds the engine's device memory as max_nall does in the reference
 * (python/kk/kk_core.cpp:1311-1347; this list holds no ghost images, so atoms stand for the reference's atoms + images);
 * 0: one pass.  *passes (may be NULL): engine passes made.
 * Allocation failure (python/kk/kk_core.cpp:1452-1484 compute_with_retry): the engine is reset and the batch runs again
 * from its first structure in passes of half as many atoms, down to 16384; the limit found is kept by the engine for
 * later calls.  When 16384 atoms per pass do not fit either: GR_ERROR "... does not fit the GPU memory ...", the engine
 * reset and usable. */
int gr_compute_batch_device(gr_engine *e, int nstruct, const int *natoms, const int *types, const double *positions, const double *cells,
                            const unsigned char *pbc, unsigned flags, int64_t max_atoms, double *energy, double *forces, double *virial,
                            double *eatom, int *passes);
/* The two batch calls with the UQ head evaluated as well (Batch.compute(uq=True) and the gamma / atomic_sigma /
 * gmm_cluster outputs of Batch.compute_device, python/kk/kk_api.h:116-156): gamma, sigma, cluster [N] per atom in the
 * caller's order, host arrays for gr_compute_batch_uq and arrays of the engine's GPU for gr_compute_batch_device_uq;
 * each may be NULL, all NULL: the call without UQ.  A model without a usable head gives GR_INVALID. */
int gr_compute_batch_uq(gr_engine *e, int nstruct, const int *natoms, const int *types, const double *positions, const double *cells,
                        const unsigned char *pbc, unsigned flags, int nthreads, double *energy, double *forces, double *virial,
                        double *eatom, double *gamma, double *sigma, double *cluster);
int gr_compute_batch_device_uq(gr_engine *e, int nstruct, const int *natoms, const int *types, const double *positions, const double *cells,
                               const unsigned char *pbc, unsigned flags, int64_t max_atoms, double *energy, double *forces, double *virial,
                               double *eatom, double *gamma, double *sigma, double *cluster, int *passes);
int gr_engine_upload_batch(gr_engine *e, int n, const int *types, const int64_t *offset, const int *j, const double *rij,
                           const double *positions, const int *image, const double *shifts, int64_t nimages, int nstruct,
                           const int *struct_of_atom);
int gr_engine_fetch_batch(gr_engine *e, int nstruct, double *energy, double *forces, double *virial, double *eatom);

#ifdef __cplusplus
}
#endif
#endif
