// Host-side containers of GRACE models read from kokkos.npz and the GRACE-1L loader.  The keys, their meaning and the
// consistency rules are the file format's, as the reference loader reads it (libgrace/src/model_1l.cpp:18-273, container
// libgrace/include/grace/model_1l.h; kind of a file: libgrace/include/grace/model_kind.h:13-19).  Every array is
// requested through FileReader (schema.hpp) with the shape it must have, so it is checked at the moment it is read.
#pragma once

#include "schema.hpp"

#include <algorithm>
#include <string>
#include <vector>

namespace grhip {

enum class ModelKind { Grace1L = 1, Grace2L = 2, Grace3L = 3 };

// The kind a file declares, or, for files older than the declaration, the kind its members give away.
inline ModelKind model_kind(const Npz &z, const std::string &path)
{
  FileReader f(z, "GRACE");
  static const struct { const char *label; const char *telltale; ModelKind kind; } kinds[] = {
      {"GRACE-3L", "prod_names", ModelKind::Grace3L},
      {"GRACE-2L", "B0_lin_transform_W", ModelKind::Grace2L},
      {"GRACE-1L", "mlp_rad_W0", ModelKind::Grace1L},
  };
  if (f.present("grace_model_kind")) {
    const auto declared = f.labels("grace_model_kind");
    for (const auto &k : kinds)
      if (declared.size() == 1 && declared[0] == k.label) return k.kind;
    throw Error(path + ": grace_model_kind names no model family this library knows (GRACE-1L, GRACE-2L, GRACE-3L)");
  }
  for (const auto &k : kinds)
    if (f.present(k.telltale)) return k.kind;
  throw Error(path + " holds none of the arrays of a GRACE kokkos.npz export");
}

// What every loader checks first: the declared kind is the loader's, and the format revision is one it reads.
inline void check_declaration(const FileReader &f, const char *label)
{
  const long revision = f.whole_or("grace_format_version", 0, kSizeLimit, 0);
  if (f.present("grace_model_kind")) {
    const auto declared = f.labels("grace_model_kind");
    if (declared.size() != 1) f.reject("grace_model_kind", "must hold exactly one name");
    if (declared[0] != label) throw Error(std::string(label) + " loader: the file declares a " + declared[0] + " model");
    if (revision < 1) f.reject("grace_format_version", "must be at least 1 in a file that declares its kind");
  }
  if (revision > 2) f.reject("grace_format_version", "= " + std::to_string(revision) + " is newer than the revisions (up to 2) this library reads");
}

struct MLPLayer {
  std::vector<double> W;    // [n_in][n_out]
  double norm = 1.0;
  int n_in = 0, n_out = 0;
};

struct FCWeights {
  std::vector<double> w_left, w_right;    // [n_out][n_in][tiles]
  std::vector<int> w_tile_left, w_tile_right, collect_to, collect_from;
  std::vector<double> norm_out_factor;
  double norm_left = 1.0, norm_right = 1.0;
  int n_out = 0, n_in_left = 0, n_in_right = 0, n_funcs = 0, n_conn = 0, tiles_left = 0, tiles_right = 0;
};

struct CGProduct {
  std::vector<int> left_ind, right_ind, m_sum_ind;
  std::vector<double> cg_coeff;
  int n_out = 0, n_terms = 0;
};

struct ReduceWeights {
  std::vector<double> W;    // [n_elements][n_out][n_in][w_shape]
  double norm = 1.0;
  int n_in = 0, w_shape = 0;
  std::vector<int> collect_ind, w_l_tile;
};

// A stack of dense layers `<stem>_W0, <stem>_W1, ...` with scalar norms: `depth` matrices chained from `first_in` inputs
// to `last_out` outputs; the widths in between are whatever the file holds.
inline std::vector<MLPLayer> read_dense_stack(const FileReader &f, const std::string &stem, long depth, long first_in, long last_out)
{
  std::vector<MLPLayer> stack((size_t) depth);
  long width = first_in;
  for (long k = 0; k < depth; k++) {
    const std::string tag = std::to_string(k);
    MLPLayer &layer = stack[(size_t) k];
    long out = last_out;
    layer.W = k + 1 == depth ? f.reals(stem + "_W" + tag, {width, out}) : f.reals(stem + "_W" + tag, {width, Ext::any(out)});
    layer.n_in = (int) width;
    layer.n_out = (int) out;
    layer.norm = f.real_or(stem + "_norm" + tag, 1.0);
    width = out;
  }
  return stack;
}

// Channel-mixing layer `<name>_*`: per output function a left weight tile applied to the same function of the left input and
// right tiles applied to collected functions of the right input.
struct FcExtents {
  long functions;          // functions of the left input = of the output
  long right_functions;    // functions of the right input
  long left_width, right_width, out_width;
};
inline FCWeights read_fc(const FileReader &f, const std::string &name, const FcExtents &x)
{
  FCWeights fc;
  long tiles = 0, links = 0;
  f.must_be(name + "_n_out", x.out_width, x.out_width, "all FC layers of a chain have the width of its first one");
  f.must_be(name + "_left_coefs", 1, 1, "the engines of this model family apply a left weight in every FC layer");
  fc.w_left = f.reals(name + "_w_left", {x.out_width, x.left_width, Ext::any(tiles)});
  fc.w_right = f.reals(name + "_w_right", {x.out_width, x.right_width, tiles});
  fc.w_tile_left = f.indices(name + "_w_tile_left", {x.functions}, tiles);
  fc.norm_out_factor = f.reals(name + "_norm_out_factor", Flat{x.functions});
  fc.collect_from = f.indices(name + "_collect_from", {Ext::any(links)}, x.right_functions);
  fc.collect_to = f.indices(name + "_collect_to", {links}, x.functions);
  fc.w_tile_right = f.indices(name + "_w_tile_right", {links}, tiles);
  fc.norm_left = f.real_or(name + "_norm_left", 1.0);
  fc.norm_right = f.real_or(name + "_norm_right", 1.0);
  fc.n_out = (int) x.out_width;
  fc.n_in_left = (int) x.left_width;
  fc.n_in_right = (int) x.right_width;
  fc.n_funcs = (int) x.functions;
  fc.n_conn = (int) links;
  fc.tiles_left = fc.tiles_right = (int) tiles;
  return fc;
}

// Channel-wise Clebsch-Gordan product `<name>_*`: a list of (left function, right function, output function, coefficient).
inline CGProduct read_product(const FileReader &f, const std::string &name, long left_functions, long right_functions)
{
  CGProduct p;
  const long terms = f.whole(name + "_n_cg_terms", 1, kSizeLimit), outputs = f.whole(name + "_n_output_funcs", 1, kSizeLimit);
  p.cg_coeff = f.reals(name + "_cg_coeff", {terms});
  p.left_ind = f.indices(name + "_left_ind", {terms}, left_functions);
  p.right_ind = f.indices(name + "_right_ind", {terms}, right_functions);
  p.m_sum_ind = f.indices(name + "_m_sum_ind", {terms}, outputs);
  if (addressed(p.m_sum_ind) != outputs)
    f.reject(name + "_n_output_funcs", "= " + std::to_string(outputs) + " but " + name + "_m_sum_ind addresses " + std::to_string(addressed(p.m_sum_ind)) + " functions");
  p.n_terms = (int) terms;
  p.n_out = (int) outputs;
  return p;
}

// The uqv6 UQ head of a model file (libgrace/include/grace/uq_head.h, loader libgrace/src/uq_head.cpp:11-76): the GMM
// feature of an atom is phi = concat((B / |B|) R, n_density log-norm channels), B the invariant basis of the energy
// path (the raw l = 0 inputs of the rho reduce), R the stored random projection; gamma = Mahalanobis distance to the
// nearest centroid of the atom's element over the cluster's interpolation threshold.
struct UqHead {
  bool has_uq = false;
  int schema = 0, n_elements = 0, max_clusters = 0, feature_dim = 0, rp_dim = 0, n_density = 0, normalize = 0, d_basis = 0;
  double density_scale = 1.0;
  std::vector<double> centroids;            // [E][Kmax][D]
  std::vector<double> inv_cov;              // [E][Kmax][D][D]
  std::vector<int> n_clusters;              // [E]
  std::vector<double> interp_thresholds;    // [E][Kmax]
  std::vector<double> rp_matrix;            // [d_basis][rp_dim]
  std::string error;                        // what is wrong with the head (reported by validate_uq; the model stays usable)

  // A head that cannot be used leaves `error` set instead of failing the load: energies and forces do not need it.
  void load(const FileReader &f, int model_elements)
  {
    *this = UqHead();
    schema = (int) f.whole_or("uq_schema_version", 0, kSizeLimit, 0);
    has_uq = schema != 0;
    if (schema != 6) return;    // another schema: validate_uq() says so
    try {
      f.must_be("uq_n_elements", model_elements, model_elements, "the head must cover the elements of the model");
      n_elements = model_elements;
      max_clusters = (int) f.whole("uq_max_clusters", 1, kSizeLimit);
      rp_dim = (int) f.whole("uq_rp_dim", 1, kSizeLimit);
      feature_dim = (int) f.whole("uq_feature_dim", rp_dim, kSizeLimit);
      n_density = feature_dim - rp_dim;
      normalize = (int) f.whole_or("uq_rp_normalize", 0, 1, 0);
      const bool density = f.flag_or("uq_rp_add_density_channel", false);
      const long transform = f.whole_or("uq_feature_transform", 0, kSizeLimit, 0);
      if (!normalize || !density || transform != 0)
        throw Error("a uqv6 head is defined with a normalised projection, density channels and no feature transform; this file has "
                    "uq_rp_normalize = " + std::to_string(normalize) + ", uq_rp_add_density_channel = " + std::to_string((int) density) +
                    ", uq_feature_transform = " + std::to_string(transform));
      density_scale = f.real_or("uq_rp_density_scale", 1.0);
      long basis = 0;
      rp_matrix = f.reals("uq_rp_matrix", {Ext::any(basis), rp_dim});
      d_basis = (int) basis;
      const long E = n_elements, K = max_clusters, D = feature_dim;
      centroids = f.reals("uq_centroids", Flat{E * K * D});
      inv_cov = f.reals("uq_inv_cov", Flat{E * K * D * D});
      interp_thresholds = f.reals("uq_interp_thresholds", Flat{E * K});
      n_clusters = f.indices("uq_n_clusters", {E}, K + 1);
      for (long e = 0; e < E; e++)
        if (n_clusters[(size_t) e] == 0) throw Error("uq_n_clusters: element " + std::to_string(e) + " has no GMM cluster; a head must cover every element");
    } catch (const std::exception &e) {
      error = f.family() + " UQ head: " + e.what();
    }
  }
  // Shared part of validate_uq(): is there a head of the schema the kernels implement, loaded without complaint, sized
  // for this model (`basis` rows of the projection, `blocks` basis blocks -> 1 + blocks density channels)?
  void require_usable(const std::string &family, bool order4, long basis, int blocks) const
  {
    if (!has_uq) throw Error(family + ": the model has no UQ head");
    if (!order4) throw Error(family + ": a UQ head needs the fourth-order stage; this is a max_order 3 model");
    if (schema != 6) throw Error(family + ": UQ head of schema " + std::to_string(schema) + "; only schema 6 (uqv6) can be evaluated");
    if (!error.empty()) throw Error(error);
    if (basis != d_basis)
      throw Error(family + " UQ head: uq_rp_matrix projects " + std::to_string(d_basis) + " basis functions, the model has " + std::to_string(basis));
    if (n_density != 1 + blocks)
      throw Error(family + " UQ head: " + std::to_string(n_density) + " density channels where " + std::to_string(1 + blocks) + " belong to this model family");
  }
};

// Sizes and switches shared by the GRACE-1L and GRACE-2L files: key, accepted range, value of a file without the key.
struct SizeKey {
  const char *key;
  long lo, hi, absent;
};

struct Model1L {
  int n_elements = 0, embedding_size = 0, lmax = 0, nradbase = 0, nradmax = 0, radial_basis_p = 0;
  int max_order = 4;    // 3: the file has no AAAA stage (its contribution is exactly zero, the engine skips it)
  double rcut = 0.0;
  bool has_bond_specific_cutoff = false;
  std::vector<double> bond_cutoff_map;    // [nel][nel]
  std::vector<double> chem_embedding, A_lin_transform_W;
  double A_lin_transform_norm = 1.0, A_inv_avg_n_neigh = 1.0;
  std::vector<MLPLayer> mlp_rad, energy_mlp;
  FCWeights fc_A1, fc_AA1, fc_AA2;
  CGProduct prod_AA, prod_AAA, prod_AAAA;
  int rho_n_out = 0;
  ReduceWeights red_A, red_AA, red_AAA, red_AAAA;
  int energy_mlp_activation = 0, radial_activation = 0;
  bool AAA_right_A = false, energy_mlp_ln = false;
  std::vector<double> shift_values;
  double output_scale = 1.0;
  std::vector<std::string> element_names;
  UqHead uq;

  int nl() const { return lmax + 1; }
  int nlm() const { return (lmax + 1) * (lmax + 1); }
  // width of the UQ basis: the collected functions of the rho reduce's sources times their channels
  // (libgrace/include/grace/uq.h:31-48)
  int uq_basis_width() const
  {
    int w = 0;
    for (const ReduceWeights *r : {&red_A, &red_AA, &red_AAA, &red_AAAA}) w += r->n_in * (int) r->collect_ind.size();
    return w;
  }
  // can the head be evaluated (libgrace/src/model_1l.cpp:275-285, libgrace/src/uq.cpp:8-33)
  void validate_uq() const { uq.require_usable("GRACE-1L", max_order == 4, uq_basis_width(), 1); }
  double pair_cutoff(int mu_i, int mu_j) const    // libgrace/include/grace/type_map.h:23-28
  {
    if (mu_i < 0 || mu_j < 0) return 0.0;
    return has_bond_specific_cutoff ? bond_cutoff_map[(size_t) mu_i * n_elements + mu_j] : rcut;
  }

  void load(const Npz &z)
  {
    *this = Model1L();
    const FileReader f(z, "GRACE-1L");
    check_declaration(f, "GRACE-1L");

    // ---- sizes
    int *const into[] = {&n_elements, &embedding_size, &lmax, &nradbase, &nradmax, &radial_basis_p};
    static const SizeKey sizes[] = {{"n_elements", 1, kSizeLimit, 89}, {"embedding_size", 1, kSizeLimit, 128}, {"lmax", 0, kDegreeLimit, 4},
                                    {"nradbase", 1, kSizeLimit, 10},   {"nradmax", 1, kSizeLimit, 32},         {"radial_basis_p", 1, kEnvelopeLimit, 16}};
    for (size_t k = 0; k < sizeof(sizes) / sizeof(sizes[0]); k++) *into[k] = (int) f.whole_or(sizes[k].key, sizes[k].lo, sizes[k].hi, sizes[k].absent);
    const long harmonics = nlm(), channels = nradmax;

    // ---- which stages the file has: a file without the fourth-order product must not carry pieces of that stage
    const bool fourth = f.present("prod_AAAA_n_cg_terms");
    max_order = fourth ? 4 : 3;
    if (!fourth)
      for (const auto &member : z)
        if (member.first.find("AAAA") != std::string::npos || member.first.compare(0, 7, "fc_AA2_") == 0)
          f.reject(member.first, "belongs to the AAAA stage, which this file otherwise lacks (no prod_AAAA_n_cg_terms): the stage is incomplete");

    // ---- elements, cutoffs, species weights
    element_names = f.labels("element_names");
    if (!element_names.empty() && (long) element_names.size() != n_elements)
      f.reject("element_names", "lists " + std::to_string(element_names.size()) + " elements where n_elements = " + std::to_string(n_elements));
    chem_embedding = f.reals("chem_embedding", {n_elements, embedding_size});
    rcut = f.length_or("rcut", 6.0);
    has_bond_specific_cutoff = f.flag_or("has_bond_specific_cutoff", false);
    bond_cutoff_map = f.distances_or_none("bond_cutoff_map", n_elements, n_elements);
    if (bond_cutoff_map.empty()) bond_cutoff_map.assign((size_t) n_elements * n_elements, rcut);
    A_lin_transform_W = f.reals("A_lin_transform_W", {embedding_size, channels});
    A_lin_transform_norm = f.real_or("A_lin_transform_norm", 1.0);
    A_inv_avg_n_neigh = f.real_or("A_inv_avg_n_neigh", 1.0);

    // ---- radial network
    f.must_be("mlp_rad_has_chem_emb", 0, 0, "radial networks with species inputs belong to GRACE-3L");
    mlp_rad = read_dense_stack(f, "mlp_rad", f.whole_or("mlp_rad_n_layers", 1, kSizeLimit, 3), nradbase, channels * nl());
    radial_activation = (int) f.whole_or("radial_activation", 0, 1, 0);

    // ---- the chain A -> A1 -> AA -> AA1 / AA2 -> AAA / AAAA; the FC width is that of its first layer
    const long fcw = f.whole_or("fc_A1_n_out", 1, kSizeLimit, 64);
    fc_A1 = read_fc(f, "fc_A1", {harmonics, harmonics, channels, channels, fcw});
    prod_AA = read_product(f, "prod_AA", harmonics, harmonics);
    const long pairs = prod_AA.n_out;
    fc_AA1 = read_fc(f, "fc_AA1", {pairs, harmonics, fcw, channels, fcw});
    prod_AAA = read_product(f, "prod_AAA", pairs, harmonics);
    if (fourth) {
      fc_AA2 = read_fc(f, "fc_AA2", {pairs, harmonics, fcw, channels, fcw});
      prod_AAAA = read_product(f, "prod_AAAA", pairs, pairs);
    }
    AAA_right_A = f.flag_or("AAA_right_A", false);
    if (AAA_right_A && fcw != channels)
      f.reject("AAA_right_A", "is set (AAA = AA1 x A), which needs the FC width " + std::to_string(fcw) + " to equal nradmax = " + std::to_string(channels));

    // ---- density: one element-dependent projection per stage
    rho_n_out = (int) f.whole_or("rho_n_out", 2, kSizeLimit, 17);
    f.must_be("rho_is_central_atom_type_dependent", 1, 1, "the density weights of this model family depend on the central element");
    struct Stage { const char *tag; ReduceWeights *into; long width, functions; bool have; };
    const Stage stages[] = {{"A", &red_A, channels, harmonics, true}, {"AA", &red_AA, fcw, pairs, true}, {"AAA", &red_AAA, fcw, prod_AAA.n_out, true},
                            {"AAAA", &red_AAAA, fcw, prod_AAAA.n_out, fourth}};
    for (const Stage &s : stages) {
      if (!s.have) continue;
      const std::string tag = s.tag;
      ReduceWeights &r = *s.into;
      long tiles = 0, picked = 0;
      f.must_be("rho_n_in_" + tag, s.width, s.width, "it is the channel width of " + tag);
      r.W = f.reals("rho_reduce_" + tag + "_W", {n_elements, rho_n_out, s.width, Ext::any(tiles)});
      f.must_be("rho_w_shape_" + tag, tiles, tiles, "it counts the weight tiles stored in rho_reduce_" + tag + "_W");
      r.collect_ind = f.indices("rho_collect_ind_" + tag, {Ext::any(picked)}, s.functions);
      r.w_l_tile = f.indices("rho_w_l_tile_" + tag, {picked}, tiles);
      r.norm = f.real_or("rho_reduce_" + tag + "_norm", 1.0);
      r.n_in = (int) s.width;
      r.w_shape = (int) tiles;
    }

    // ---- readout
    read_readout(f, "GRACE-1L", rho_n_out, 0, energy_mlp, energy_mlp_activation, energy_mlp_ln);
    shift_values = f.reals_or("shift_values", Flat{n_elements}, 0.0);
    output_scale = f.real_or("output_scale", 1.0);
    uq.load(f, n_elements);
  }

  // The readout network on the non-linear density channels, shared with GRACE-2L: `energy_mlp_*`, an activation switch, and in
  // legacy files the scale of an RMS layer norm of its input, which is folded into the first matrix.  The engines hold at
  // most 7 layers of at most 256 units (libgrace/src/fused_1l.cpp:226-236).
  static void read_readout(const FileReader &f, const char *family, int density_width, int default_activation, std::vector<MLPLayer> &net,
                           int &activation, bool &layer_norm)
  {
    net = read_dense_stack(f, "energy_mlp", f.whole_or("energy_mlp_n_layers", 1, 7, 2), density_width - 1, 1);
    for (const MLPLayer &layer : net)
      if (layer.n_out > 256 || layer.n_in > 256) throw Error(std::string(family) + ": readout layers wider than 256 units do not fit the engines");
    activation = (int) f.whole_or("energy_mlp_activation", 0, 1, default_activation);
    layer_norm = f.present("energy_mlp_scale");
    if (layer_norm) {
      const std::vector<double> scale = f.reals("energy_mlp_scale", Flat{net[0].n_in});
      for (int row = 0; row < net[0].n_in; row++)
        for (int col = 0; col < net[0].n_out; col++) net[0].W[(size_t) row * net[0].n_out + col] *= scale[(size_t) row];
    }
  }
};

// type2mu has ntypes + 1 entries (types are 1-based), each -1 or a model element: libgrace/include/grace/type_map.h:31-39
inline void check_type2mu(const std::vector<int> &type2mu, int ntypes, int n_elements, const char *who)
{
  if ((int) type2mu.size() != ntypes + 1) throw Error(std::string(who) + ": the type map needs one entry per atom type plus the unused entry 0");
  for (int t = 1; t <= ntypes; t++)
    if (type2mu[t] < -1 || type2mu[t] >= n_elements)
      throw Error(std::string(who) + ": atom type " + std::to_string(t) + " is mapped to element " + std::to_string(type2mu[t]) + " of a model with " +
                  std::to_string(n_elements) + " elements");
}

}    // namespace grhip
