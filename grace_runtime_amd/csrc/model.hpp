// Host-side containers of GRACE models read from kokkos.npz, with the validation of the reference loaders:
// GRACE-1L keys and checks follow libgrace/src/model_1l.cpp:18-273 (container libgrace/include/grace/model_1l.h),
// the kind of a file libgrace/include/grace/model_kind.h:13-19.
#pragma once

#include "npz.hpp"

#include <algorithm>
#include <string>
#include <vector>

namespace grhip {

enum class ModelKind { Grace1L = 1, Grace2L = 2, Grace3L = 3 };

// grace_model_kind names the kind; files without it are told apart by their members
inline ModelKind model_kind(const Npz &z, const std::string &path)
{
  NpzView v(z);
  if (v.has("grace_model_kind")) {
    const auto k = v.names("grace_model_kind");
    if (k.size() == 1 && k[0] == "GRACE-1L") return ModelKind::Grace1L;
    if (k.size() == 1 && k[0] == "GRACE-2L") return ModelKind::Grace2L;
    if (k.size() == 1 && k[0] == "GRACE-3L") return ModelKind::Grace3L;
    throw Error("model file " + path + ": unknown grace_model_kind");
  }
  if (v.has("prod_names")) return ModelKind::Grace3L;
  if (v.has("B0_lin_transform_W")) return ModelKind::Grace2L;
  if (v.has("mlp_rad_W0")) return ModelKind::Grace1L;
  throw Error("model file " + path + " is not a GRACE kokkos.npz");
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

inline std::vector<MLPLayer> load_mlp(const NpzView &v, const std::string &pfx, int n, int64_t n_in, int64_t n_out,
                                      const std::string &in_why, const std::string &out_why)
{
  std::vector<MLPLayer> layers;
  int64_t prev = n_in;
  for (int i = 0; i < n; i++) {
    const std::string wk = pfx + "_W" + std::to_string(i);
    MLPLayer L;
    L.W = v.require_doubles(wk);
    const auto sh = v.shape_rank(wk, 2);
    require_eq(wk, (int64_t) sh[0], prev, i == 0 ? in_why : "the outputs of the layer before", "rows");
    if (i == n - 1) require_eq(wk, (int64_t) sh[1], n_out, out_why, "columns");
    L.n_in = (int) sh[0];
    L.n_out = (int) sh[1];
    L.norm = v.double_scalar(pfx + "_norm" + std::to_string(i), 1.0);
    prev = L.n_out;
    layers.push_back(std::move(L));
  }
  return layers;
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

  // who: "GRACE-1L/KK"; checks and messages of uq_head.cpp:11-76
  void load(const NpzView &v, int model_elements, const std::string &who)
  {
    *this = UqHead();
    schema = v.int_scalar("uq_schema_version", 0);
    has_uq = schema != 0;
    if (schema != 6) return;
    const std::string pre = who + " UQ: ";
    try {
      n_elements = v.int_scalar("uq_n_elements", model_elements);
      require_eq("uq_n_elements", n_elements, model_elements, "n_elements");
      max_clusters = v.int_in("uq_max_clusters", 0, 1, kMaxDim);
      rp_dim = v.int_in("uq_rp_dim", 0, 1, kMaxDim);
      feature_dim = v.int_in("uq_feature_dim", 0, rp_dim, kMaxDim);
      normalize = v.int_scalar("uq_rp_normalize", 0);
      const int add_density = v.int_scalar("uq_rp_add_density_channel", 0);
      density_scale = v.double_scalar("uq_rp_density_scale", 1.0);
      const int transform = v.int_scalar("uq_feature_transform", 0);
      centroids = v.require_doubles("uq_centroids");
      inv_cov = v.require_doubles("uq_inv_cov");
      n_clusters = v.require_ints("uq_n_clusters");
      interp_thresholds = v.require_doubles("uq_interp_thresholds");
      rp_matrix = v.require_doubles("uq_rp_matrix");
      if (normalize != 1 || add_density != 1 || transform != 0)
        throw Error("schema v6 expects normalize=1, add_density_channel=1, feature_transform=0 (identity); got normalize=" +
                    std::to_string(normalize) + ", add_density=" + std::to_string(add_density) + ", transform=" + std::to_string(transform) +
                    ". Artifact mislabeled or unsupported variant.");
      n_density = feature_dim - rp_dim;
      const auto rs = v.shape_rank("uq_rp_matrix", 2);
      require_eq("uq_rp_matrix", (int64_t) rs[1], rp_dim, "uq_rp_dim", "columns");
      d_basis = (int) rs[0];
      const size_t E = (size_t) n_elements, K = (size_t) max_clusters, D = (size_t) feature_dim;
      require_size("uq_centroids", centroids, E * K * D);
      require_size("uq_inv_cov", inv_cov, E * K * D * D);
      require_size("uq_n_clusters", n_clusters, E);
      require_size("uq_interp_thresholds", interp_thresholds, E * K);
      for (size_t e = 0; e < n_clusters.size(); e++) {
        if (n_clusters[e] <= 0)
          throw Error("element index " + std::to_string(e) + " has no GMM clusters; uqv6 artifacts must cover all elements. Re-export the "
                      "UQ artifacts with a current grace_utils.");
        if (n_clusters[e] > max_clusters)
          throw Error("element index " + std::to_string(e) + " has " + std::to_string(n_clusters[e]) + " GMM clusters, more than uq_max_clusters = " +
                      std::to_string(max_clusters));
      }
    } catch (const std::exception &e) {
      error = e.what();
      if (error.rfind(pre, 0) != 0) error = pre + error;
    }
  }
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
    int w = red_A.n_in * (int) red_A.collect_ind.size() + red_AA.n_in * (int) red_AA.collect_ind.size() +
            red_AAA.n_in * (int) red_AAA.collect_ind.size();
    if (max_order == 4) w += red_AAAA.n_in * (int) red_AAAA.collect_ind.size();
    return w;
  }
  // libgrace/src/model_1l.cpp:275-285, libgrace/src/uq.cpp:8-33
  void validate_uq() const
  {
    if (!uq.has_uq) throw Error("GRACE-1L: the model has no UQ head");
    if (max_order == 3) throw Error("GRACE-1L: UQ is not supported for max_order 3 models");
    if (uq.schema != 6)
      throw Error("GRACE-1L: UQ schema v" + std::to_string(uq.schema) + " unsupported (expects v6, uqv6 basis-RP normalize+density). Re-export the "
                  "UQ artifacts at schema v6 with a current grace_utils.");
    if (!uq.error.empty()) throw Error(uq.error);
    if (uq_basis_width() != uq.d_basis)
      throw Error("GRACE-1L UQ: uq_rp_matrix has " + std::to_string(uq.d_basis) + " rows, the model's invariant basis has " +
                  std::to_string(uq_basis_width()) + "; re-export the UQ artifacts for this model");
    if (uq.n_density != 2)
      throw Error("GRACE-1L UQ: " + std::to_string(uq.n_density) + " density channels, expected 2 (1 + basis blocks)");
  }
  double pair_cutoff(int mu_i, int mu_j) const    // libgrace/include/grace/type_map.h:23-28
  {
    if (mu_i < 0 || mu_j < 0) return 0.0;
    return has_bond_specific_cutoff ? bond_cutoff_map[(size_t) mu_i * n_elements + mu_j] : rcut;
  }

  void load(const Npz &z)
  {
    *this = Model1L();
    NpzView v(z);
    if (v.has("grace_model_kind")) {
      const auto k = v.names("grace_model_kind");
      if (k.size() != 1) throw bad_array("grace_model_kind", "must hold one name");
      if (k[0] != "GRACE-1L") throw Error("GRACE-1L: the file holds a " + k[0] + " model");
      if (v.int_scalar("grace_format_version", 0) < 1) throw bad_array("grace_format_version", "is missing or below 1 next to grace_model_kind");
    }
    if (v.int_scalar("grace_format_version", 0) > 2)
      throw Error("GRACE-1L: kokkos.npz format " + std::to_string(v.int_scalar("grace_format_version", 0)) + ", this build reads up to 2");
    // max_order 3: no AAAA stage; some but not all of its arrays is a broken file (libgrace/src/max_order3.h:104-134)
    const bool order4 = v.has("prod_AAAA_n_cg_terms");
    if (!order4)
      for (const auto &kv : z)
        if (kv.first.find("AAAA") != std::string::npos || kv.first.rfind("fc_AA2_", 0) == 0)
          throw bad_array(kv.first, "is present, but prod_AAAA_n_cg_terms is not: the AAAA stage is incomplete");
    max_order = order4 ? 4 : 3;

    n_elements = v.int_in("n_elements", 89, 1, kMaxDim);
    embedding_size = v.int_in("embedding_size", 128, 1, kMaxDim);
    lmax = v.int_in("lmax", 4, 0, kMaxL);
    nradbase = v.int_in("nradbase", 10, 1, kMaxDim);
    nradmax = v.int_in("nradmax", 32, 1, kMaxDim);
    radial_basis_p = v.int_in("radial_basis_p", 16, 1, kMaxP);
    rcut = v.cutoff_scalar("rcut", 6.0, "GRACE-1L/KK");
    has_bond_specific_cutoff = v.flag("has_bond_specific_cutoff", 0);
    require_eq("mlp_rad_has_chem_emb", v.int_scalar("mlp_rad_has_chem_emb", 0), 0, "chem-embedded radial MLPs are not supported");
    const int64_t nlm_ = (int64_t) (lmax + 1) * (lmax + 1);

    element_names = v.names("element_names");
    chem_embedding = v.require_doubles("chem_embedding");
    {
      const auto ce = v.shape_rank("chem_embedding", 2);
      if ((long) ce[0] != n_elements && (element_names.empty() || element_names.size() == ce[0]))
        throw bad_array("n_elements", "is " + std::to_string(n_elements) + ", but chem_embedding has " + std::to_string(ce[0]) + " rows");
      if (!element_names.empty()) require_size("element_names", element_names, n_elements);
      v.require_shape("chem_embedding", {n_elements, embedding_size});
    }
    bond_cutoff_map = v.cutoffs("bond_cutoff_map", "GRACE-1L/KK");
    v.require_shape("bond_cutoff_map", {n_elements, n_elements});
    if (bond_cutoff_map.empty()) bond_cutoff_map.assign((size_t) n_elements * n_elements, rcut);

    A_lin_transform_W = v.require_doubles("A_lin_transform_W");
    v.require_shape("A_lin_transform_W", {embedding_size, nradmax});
    A_lin_transform_norm = v.double_scalar("A_lin_transform_norm", 1.0);
    A_inv_avg_n_neigh = v.double_scalar("A_inv_avg_n_neigh", 1.0);

    mlp_rad = load_mlp(v, "mlp_rad", v.int_in("mlp_rad_n_layers", 3, 1, kMaxDim), nradbase, (int64_t) nradmax * (lmax + 1),
                       "nradbase", "nradmax x (lmax + 1)");

    auto load_fc = [&](const std::string &p, FCWeights &fc, int64_t n_funcs, int64_t n_in_left) {
      fc.w_left = v.require_doubles(p + "_w_left");
      fc.w_right = v.require_doubles(p + "_w_right");
      fc.w_tile_left = v.require_ints(p + "_w_tile_left");
      fc.w_tile_right = v.require_ints(p + "_w_tile_right");
      fc.collect_to = v.require_ints(p + "_collect_to");
      fc.collect_from = v.require_ints(p + "_collect_from");
      fc.norm_out_factor = v.require_doubles(p + "_norm_out_factor");
      fc.norm_left = v.double_scalar(p + "_norm_left", 1.0);
      fc.norm_right = v.double_scalar(p + "_norm_right", 1.0);
      fc.n_out = v.int_in(p + "_n_out", 64, 1, kMaxDim);
      require_eq(p + "_left_coefs", v.int_scalar(p + "_left_coefs", 1), 1, "the GRACE-1L engines apply left weights in every FC");
      fc.tiles_left = (int) v.shape_rank(p + "_w_left", 3)[2];
      fc.tiles_right = (int) v.shape_rank(p + "_w_right", 3)[2];
      require_eq(p + "_w_right", fc.tiles_right, fc.tiles_left, "the tiles of " + p + "_w_left", "tiles");
      v.require_shape(p + "_w_left", {fc.n_out, n_in_left, fc.tiles_left});
      v.require_shape(p + "_w_right", {fc.n_out, nradmax, fc.tiles_right});
      require_size(p + "_w_tile_left", fc.w_tile_left, (size_t) n_funcs);
      require_size(p + "_norm_out_factor", fc.norm_out_factor, (size_t) n_funcs);
      require_index(p + "_w_tile_left", fc.w_tile_left, fc.tiles_left);
      const size_t nc = fc.collect_from.size();
      require_size(p + "_collect_to", fc.collect_to, nc);
      require_size(p + "_w_tile_right", fc.w_tile_right, nc);
      require_index(p + "_collect_from", fc.collect_from, nlm_);
      require_index(p + "_collect_to", fc.collect_to, n_funcs);
      require_index(p + "_w_tile_right", fc.w_tile_right, fc.tiles_right);
      fc.n_in_left = (int) n_in_left;
      fc.n_in_right = nradmax;
      fc.n_funcs = (int) n_funcs;
      fc.n_conn = (int) nc;
    };
    auto load_prod = [&](const std::string &p, CGProduct &pr, int64_t n_left, int64_t n_right) {
      pr.left_ind = v.require_ints(p + "_left_ind");
      pr.right_ind = v.require_ints(p + "_right_ind");
      pr.m_sum_ind = v.require_ints(p + "_m_sum_ind");
      pr.cg_coeff = v.require_doubles(p + "_cg_coeff");
      pr.n_out = v.int_in(p + "_n_output_funcs", 0, 1, kMaxDim);
      pr.n_terms = v.int_in(p + "_n_cg_terms", 0, 1, kMaxDim);
      const size_t nt = (size_t) pr.n_terms;
      require_size(p + "_left_ind", pr.left_ind, nt);
      require_size(p + "_right_ind", pr.right_ind, nt);
      require_size(p + "_m_sum_ind", pr.m_sum_ind, nt);
      require_size(p + "_cg_coeff", pr.cg_coeff, nt);
      require_index(p + "_left_ind", pr.left_ind, n_left);
      require_index(p + "_right_ind", pr.right_ind, n_right);
      require_index(p + "_m_sum_ind", pr.m_sum_ind, pr.n_out);
      require_eq(p + "_n_output_funcs", pr.n_out, index_extent(pr.m_sum_ind), "1 + the largest " + p + "_m_sum_ind");
    };

    // the FC width is needed before the checks: read it first
    const int CF = v.int_in("fc_A1_n_out", 64, 1, kMaxDim);
    load_fc("fc_A1", fc_A1, nlm_, nradmax);
    load_prod("prod_AA", prod_AA, nlm_, nlm_);
    const int64_t nAA = prod_AA.n_out;
    load_fc("fc_AA1", fc_AA1, nAA, CF);
    require_eq("fc_AA1_n_out", fc_AA1.n_out, CF, "fc_A1_n_out");
    load_prod("prod_AAA", prod_AAA, nAA, nlm_);
    if (order4) {
      load_fc("fc_AA2", fc_AA2, nAA, CF);
      require_eq("fc_AA2_n_out", fc_AA2.n_out, CF, "fc_A1_n_out");
      load_prod("prod_AAAA", prod_AAAA, nAA, nAA);
    }

    rho_n_out = v.int_in("rho_n_out", 17, 2, kMaxDim);
    require_eq("rho_is_central_atom_type_dependent", v.int_scalar("rho_is_central_atom_type_dependent", 1), 1,
               "the GRACE-1L engines implement this layout only");
    auto load_reduce = [&](const std::string &s, ReduceWeights &rw, int64_t n_in, int64_t n_funcs) {
      const std::string wkey = "rho_reduce_" + s + "_W", ckey = "rho_collect_ind_" + s, tkey = "rho_w_l_tile_" + s;
      rw.W = v.require_doubles(wkey);
      rw.norm = v.double_scalar("rho_reduce_" + s + "_norm", 1.0);
      rw.collect_ind = v.require_ints(ckey);
      rw.w_l_tile = v.require_ints(tkey);
      rw.n_in = v.int_scalar("rho_n_in_" + s, 0);
      rw.w_shape = v.int_in("rho_w_shape_" + s, 0, 1, kMaxDim);
      require_eq("rho_n_in_" + s, rw.n_in, n_in, "the channels of " + s);
      v.require_shape(wkey, {n_elements, rho_n_out, rw.n_in, rw.w_shape});
      require_size(tkey, rw.w_l_tile, rw.collect_ind.size());
      require_index(ckey, rw.collect_ind, n_funcs);
      require_index(tkey, rw.w_l_tile, rw.w_shape);
    };
    load_reduce("A", red_A, nradmax, nlm_);
    load_reduce("AA", red_AA, CF, nAA);
    load_reduce("AAA", red_AAA, CF, prod_AAA.n_out);
    if (order4) load_reduce("AAAA", red_AAAA, CF, prod_AAAA.n_out);

    energy_mlp = load_mlp(v, "energy_mlp", v.int_in("energy_mlp_n_layers", 2, 1, kMaxDim), rho_n_out - 1, 1, "rho_n_out - 1", "one energy");
    energy_mlp_activation = v.int_in("energy_mlp_activation", 0, 0, 1);
    radial_activation = v.int_in("radial_activation", 0, 0, 1);
    AAA_right_A = v.flag("AAA_right_A", 0);
    if (AAA_right_A) require_eq("fc_AA1_n_out", fc_AA1.n_out, nradmax, "nradmax (AAA = AA1 x A)");
    {    // legacy: RMS layer norm of the energy-MLP input, its scale folded into layer 0 (libgrace/src/npz3.h:330-338)
      const auto s = v.doubles("energy_mlp_scale");
      if (!s.empty()) {
        MLPLayer &L = energy_mlp[0];
        require_size("energy_mlp_scale", s, (size_t) L.n_in);
        for (int k = 0; k < L.n_in; k++)
          for (int j = 0; j < L.n_out; j++) L.W[(size_t) k * L.n_out + j] *= s[k];
        energy_mlp_ln = true;
      }
    }
    // readout limits of the engines (libgrace/src/fused_1l.cpp:226-236)
    if (energy_mlp.size() > 7) throw Error("GRACE-1L: energy MLP has " + std::to_string(energy_mlp.size()) + " layers, at most 7 supported");
    for (const auto &L : energy_mlp)
      if (L.n_in > 256 || L.n_out > 256) throw Error("GRACE-1L: energy MLP layer widths above 256 are not supported");
    shift_values = v.doubles("shift_values");
    if (v.has("shift_values")) require_size("shift_values", shift_values, (size_t) n_elements);
    else shift_values.assign(n_elements, 0.0);
    output_scale = v.double_scalar("output_scale", 1.0);
    uq.load(v, n_elements, "GRACE-1L/KK");
  }
};

// type2mu has ntypes + 1 entries (types are 1-based), each -1 or a model element: libgrace/include/grace/type_map.h:31-39
inline void check_type2mu(const std::vector<int> &type2mu, int ntypes, int n_elements, const char *who)
{
  if ((int) type2mu.size() != ntypes + 1) throw Error(std::string(who) + ": type2mu must have ntypes + 1 entries");
  for (int t = 1; t <= ntypes; t++)
    if (type2mu[t] < -1 || type2mu[t] >= n_elements)
      throw Error(std::string(who) + ": atom type " + std::to_string(t) + " maps to model element " + std::to_string(type2mu[t]) +
                  " (the model has " + std::to_string(n_elements) + ")");
}

}    // namespace grhip
