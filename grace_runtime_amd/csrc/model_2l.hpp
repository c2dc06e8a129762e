// Host-side container of a GRACE-2L model read from kokkos.npz.  Keys, defaults and consistency checks follow the
// reference loader libgrace/src/model_2l.cpp:28-420 (container libgrace/include/grace/model_2l.h:22-175); files of
// max_order 3 (no AAAA / BBBB stage, libgrace/src/max_order3.h) are loaded with those stages absent.
#pragma once

#include "model.hpp"

namespace grhip {

// reduce with one output function per connection (equivariant) or a single one (scalar)
struct ReduceEq {
  std::vector<double> W;    // [n_elements (element dependent) | 1][n_out][n_in][w_shape]
  double norm = 1.0;
  int n_in = 0, w_shape = 0;
  bool elem = false;
  std::vector<int> collect_ind, w_l_tile, total_sum_ind;
};

struct YICoupling {
  std::vector<int> y, i, m_sum_ind;    // per term: harmonic index lm, message function, output function
  std::vector<double> cg_coeff;
  int n_out = 0, n_terms = 0;
  double inv_avg_n_neigh = 1.0;
};

struct Model2L {
  int n_elements = 0, embedding_size = 0, lmax = 0, nradbase = 0, radial_basis_p = 0;
  int max_order = 4;
  double rcut = 0.0;
  bool has_bond_specific_cutoff = false;
  std::vector<double> bond_cutoff_map, chem_embedding;
  int C1 = 0, CR = 0, C2 = 0;    // layer-1 channels, layer-2 radial channels (= message width), layer-2 channels
  std::vector<MLPLayer> mlp_R, mlp_R1, energy_mlp;
  std::vector<double> A_lin_transform_W, B0_lin_transform_W;
  double A_lin_transform_norm = 1.0, A_inv_avg_n_neigh = 1.0, B0_lin_transform_norm = 1.0, B0_inv_avg_n_neigh = 1.0;
  FCWeights fc_A1, fc_AA1, fc_AA2, fc_B1, fc_BB1, fc_BB2;
  CGProduct prod_AA, prod_AAA, prod_AAAA, prod_BB, prod_BBB, prod_BBBB;
  int I1_n_out = 0, I1_n_funcs = 0, I_n_funcs = 0, B_n_funcs = 0, rho_n_out = 0;
  ReduceEq I1_red[4], rho_red[4], I_red, B_red_YI, B_red_B0, I2_red[4];    // sources A..AAAA / B..BBBB
  YICoupling yi;
  bool energy_rms_norm = true, energy_mlp_ln = false;
  std::vector<double> I_nl_LN_scale, I_0_LN_scale;
  int energy_mlp_activation = 1, radial_activation = 0;
  std::vector<double> shift_values;
  double output_scale = 1.0;
  UqHead uq;    // the uqv6 UQ head: invariant blocks [I2 (B .. BBBB), rho (A .. AAAA)] (libgrace/src/model_2l.cpp:518-534)
  std::vector<std::string> element_names;
  static constexpr double rms_norm_eps = 1e-10;    // libgrace/include/grace/model_2l.h:156

  int nl() const { return lmax + 1; }
  int nlm() const { return (lmax + 1) * (lmax + 1); }
  int nsrc() const { return max_order == 4 ? 4 : 3; }
  // widths of the two blocks of the UQ basis (libgrace/include/grace/uq.h:31-48)
  int uq_block_width(const ReduceEq *r) const
  {
    int w = 0;
    for (int s = 0; s < nsrc(); s++) w += r[s].n_in * (int) r[s].collect_ind.size();
    return w;
  }
  // libgrace/src/model_2l.cpp:466-478, libgrace/src/uq.cpp:8-33
  void validate_uq() const
  {
    if (!uq.has_uq) throw Error("GRACE-2L: the model has no UQ head");
    if (max_order == 3) throw Error("GRACE-2L: UQ is not supported for max_order 3 models");
    if (uq.schema != 6)
      throw Error("GRACE-2L: UQ schema v" + std::to_string(uq.schema) + " unsupported (expects v6, uqv6 basis-RP normalize+density). Re-export the "
                  "UQ artifacts at schema v6 with a current grace_utils.");
    if (!uq.error.empty()) throw Error(uq.error);
    const int total = uq_block_width(I2_red) + uq_block_width(rho_red);
    if (total != uq.d_basis)
      throw Error("GRACE-2L UQ: uq_rp_matrix has " + std::to_string(uq.d_basis) + " rows, the model's invariant basis has " + std::to_string(total) +
                  "; re-export the UQ artifacts for this model");
    if (uq.n_density != 3) throw Error("GRACE-2L UQ: " + std::to_string(uq.n_density) + " density channels, expected 3 (1 + basis blocks)");
  }
  double pair_cutoff(int mu_i, int mu_j) const
  {
    if (mu_i < 0 || mu_j < 0) return 0.0;
    return has_bond_specific_cutoff ? bond_cutoff_map[(size_t) mu_i * n_elements + mu_j] : rcut;
  }

  void load(const Npz &z)
  {
    *this = Model2L();
    NpzView v(z);
    if (v.has("grace_model_kind")) {
      const auto k = v.names("grace_model_kind");
      if (k.size() != 1) throw bad_array("grace_model_kind", "must hold one name");
      if (k[0] != "GRACE-2L") throw Error("GRACE-2L: the file holds a " + k[0] + " model");
      if (v.int_scalar("grace_format_version", 0) < 1) throw bad_array("grace_format_version", "is missing or below 1 next to grace_model_kind");
    }
    if (v.int_scalar("grace_format_version", 0) > 2)
      throw Error("GRACE-2L: kokkos.npz format " + std::to_string(v.int_scalar("grace_format_version", 0)) + ", this build reads up to 2");
    const bool o4a = v.has("prod_AAAA_n_cg_terms"), o4b = v.has("prod_BBBB_n_cg_terms");
    if (o4a != o4b) throw bad_array(o4a ? "prod_BBBB_n_cg_terms" : "prod_AAAA_n_cg_terms", "is missing: the two layers must have the same max_order");
    const bool order4 = o4a;
    if (!order4)
      for (const auto &kv : z)
        if (kv.first.find("AAAA") != std::string::npos || kv.first.find("BBBB") != std::string::npos ||
            kv.first.rfind("fc_AA2_", 0) == 0 || kv.first.rfind("fc_BB2_", 0) == 0)
          throw bad_array(kv.first, "is present, but the order-4 product is not: the stage is incomplete");
    max_order = order4 ? 4 : 3;

    n_elements = v.int_in("n_elements", 89, 1, kMaxDim);
    embedding_size = v.int_in("embedding_size", 128, 1, kMaxDim);
    chem_embedding = v.require_doubles("chem_embedding");
    v.require_shape("chem_embedding", {n_elements, embedding_size});
    lmax = v.int_in("lmax", 4, 0, kMaxL);
    nradbase = v.int_in("nradbase", 10, 1, kMaxDim);
    radial_basis_p = v.int_in("radial_basis_p", 16, 1, kMaxP);
    rcut = v.cutoff_scalar("rcut", 6.0, "GRACE-2L/KK");
    has_bond_specific_cutoff = v.flag("has_bond_specific_cutoff", 0);
    bond_cutoff_map = v.cutoffs("bond_cutoff_map", "GRACE-2L/KK");
    v.require_shape("bond_cutoff_map", {n_elements, n_elements});
    if (bond_cutoff_map.empty()) bond_cutoff_map.assign((size_t) n_elements * n_elements, rcut);
    const int64_t nl_ = lmax + 1, nlm_ = nl_ * nl_;

    auto load_rad = [&](const std::string &p, std::vector<MLPLayer> &layers, int &nrad) {
      require_eq(p + "_has_chem_emb", v.int_scalar(p + "_has_chem_emb", 0), 0, "chem-embedded radial MLPs are not supported");
      nrad = v.int_in(p + "_n_rad_max", 32, 1, kMaxDim);
      layers = load_mlp(v, p, v.int_in(p + "_n_layers", 3, 1, kMaxDim), nradbase, (int64_t) nrad * nl_, "nradbase", "n_rad_max x (lmax + 1)");
    };
    load_rad("mlp_rad_R", mlp_R, C1);
    load_rad("mlp_rad_R1", mlp_R1, CR);
    A_lin_transform_W = v.require_doubles("A_lin_transform_W");
    v.require_shape("A_lin_transform_W", {embedding_size, C1});
    A_lin_transform_norm = v.double_scalar("A_lin_transform_norm", 1.0);
    A_inv_avg_n_neigh = v.double_scalar("A_inv_avg_n_neigh", 1.0);
    B0_lin_transform_W = v.require_doubles("B0_lin_transform_W");
    v.require_shape("B0_lin_transform_W", {embedding_size, CR});
    B0_lin_transform_norm = v.double_scalar("B0_lin_transform_norm", 1.0);
    B0_inv_avg_n_neigh = v.double_scalar("B0_inv_avg_n_neigh", 1.0);
    C2 = v.int_in("B_n_out", 64, 1, kMaxDim);
    B_n_funcs = v.int_in("B_n_funcs", 31, 1, kMaxDim);

    // FC of ch channels over nfl functions, right input with nfr functions
    auto load_fc = [&](const std::string &p, FCWeights &fc, int64_t nfl, int64_t nfr, int64_t ch, const std::string &ch_what) {
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
      require_eq(p + "_left_coefs", v.int_scalar(p + "_left_coefs", 1), 1, "the GRACE-2L engines apply left weights in every FC");
      require_eq(p + "_n_out", fc.n_out, ch, ch_what);
      fc.tiles_left = (int) v.shape_rank(p + "_w_left", 3)[2];
      fc.tiles_right = (int) v.shape_rank(p + "_w_right", 3)[2];
      v.require_shape(p + "_w_left", {fc.n_out, ch, fc.tiles_left});
      v.require_shape(p + "_w_right", {fc.n_out, ch, fc.tiles_right});
      require_size(p + "_w_tile_left", fc.w_tile_left, (size_t) nfl);
      require_index(p + "_w_tile_left", fc.w_tile_left, fc.tiles_left);
      require_size(p + "_norm_out_factor", fc.norm_out_factor, (size_t) nfl);
      const size_t nc = fc.collect_from.size();
      require_size(p + "_collect_to", fc.collect_to, nc);
      require_size(p + "_w_tile_right", fc.w_tile_right, nc);
      require_index(p + "_collect_to", fc.collect_to, nfl);
      require_index(p + "_collect_from", fc.collect_from, nfr);
      require_index(p + "_w_tile_right", fc.w_tile_right, fc.tiles_right);
      fc.n_in_left = fc.n_in_right = (int) ch;
      fc.n_funcs = (int) nfl;
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
      require_index(p + "_m_sum_ind", pr.m_sum_ind, pr.n_out);
      require_eq(p + "_n_output_funcs", pr.n_out, index_extent(pr.m_sum_ind), "1 + the largest " + p + "_m_sum_ind");
      require_index(p + "_left_ind", pr.left_ind, n_left);
      require_index(p + "_right_ind", pr.right_ind, n_right);
      return (int64_t) pr.n_out;
    };
    // reduce r of n_out channels into nfo output functions from source s (ch channels, nf functions)
    auto load_reduce = [&](const std::string &r, const std::string &s, ReduceEq &rw, bool elem, int64_t n_out, int64_t nfo, int64_t ch,
                           int64_t nf) {
      const std::string wkey = r + "_reduce_" + s + "_W";
      rw.elem = elem;
      rw.W = v.require_doubles(wkey);
      rw.norm = v.double_scalar(r + "_reduce_" + s + "_norm", 1.0);
      rw.collect_ind = v.require_ints(r + "_collect_ind_" + s);
      rw.w_l_tile = v.require_ints(r + "_w_l_tile_" + s);
      rw.total_sum_ind = v.require_ints(r + "_total_sum_ind_" + s);
      rw.n_in = v.int_scalar(r + "_n_in_" + s, 0);
      rw.w_shape = v.int_in(r + "_w_shape_" + s, 0, 1, kMaxDim);
      require_eq(r + "_n_in_" + s, rw.n_in, ch, "the channels of " + s);
      if (elem) v.require_shape(wkey, {n_elements, n_out, ch, rw.w_shape});
      else v.require_shape(wkey, {n_out, ch, rw.w_shape});
      const size_t nc = rw.collect_ind.size();
      require_size(r + "_w_l_tile_" + s, rw.w_l_tile, nc);
      require_size(r + "_total_sum_ind_" + s, rw.total_sum_ind, nc);
      require_index(r + "_collect_ind_" + s, rw.collect_ind, nf);
      require_index(r + "_w_l_tile_" + s, rw.w_l_tile, rw.w_shape);
      require_index(r + "_total_sum_ind_" + s, rw.total_sum_ind, nfo);
    };
    auto elem_dependent = [&](const std::string &p, int fixed) {
      require_eq(p + "_is_central_atom_type_dependent", v.int_scalar(p + "_is_central_atom_type_dependent", fixed), fixed,
                 "the GRACE-2L engines implement this layout only");
    };

    // ---- layer 1
    const std::string c1_what = "the layer-1 radial channels mlp_rad_R_n_rad_max";
    load_fc("fc_A1", fc_A1, nlm_, nlm_, C1, c1_what);
    const int64_t nAA = load_prod("prod_AA", prod_AA, nlm_, nlm_);
    load_fc("fc_AA1", fc_AA1, nAA, nlm_, C1, c1_what);
    const int64_t nAAA = load_prod("prod_AAA", prod_AAA, nAA, nlm_);
    int64_t nAAAA = 0;
    if (order4) {
      load_fc("fc_AA2", fc_AA2, nAA, nlm_, C1, c1_what);
      nAAAA = load_prod("prod_AAAA", prod_AAAA, nAA, nAA);
    }
    const char *s1[4] = {"A", "AA", "AAA", "AAAA"};
    const int64_t nf1[4] = {nlm_, nAA, nAAA, nAAAA};
    I1_n_out = v.int_in("I1_n_out", 12, 1, kMaxDim);
    I1_n_funcs = v.int_in("I1_n_funcs", 4, 1, kMaxDim);
    elem_dependent("I1", 1);
    rho_n_out = v.int_in("rho_n_out", 17, 2, kMaxDim);
    elem_dependent("rho", 1);
    for (int s = 0; s < nsrc(); s++) {
      load_reduce("I1", s1[s], I1_red[s], true, I1_n_out, I1_n_funcs, C1, nf1[s]);
      load_reduce("rho", s1[s], rho_red[s], true, rho_n_out, 1, C1, nf1[s]);
    }
    require_eq("I_n_out", v.int_in("I_n_out", 32, 1, kMaxDim), CR, "YI couples I with the layer-2 radial channels mlp_rad_R1_n_rad_max");
    I_n_funcs = v.int_in("I_n_funcs", 4, 1, kMaxDim);
    elem_dependent("I", 0);
    load_reduce("I", "I1", I_red, false, CR, I_n_funcs, I1_n_out, I1_n_funcs);

    // ---- layer 2
    {
      const auto lr = v.require_ints("YI_lr_inds");
      yi.m_sum_ind = v.require_ints("YI_m_sum_ind");
      yi.cg_coeff = v.require_doubles("YI_cg_coeff");
      yi.n_terms = v.int_in("YI_n_cg_terms", 0, 1, kMaxDim);
      yi.n_out = v.int_in("YI_n_output_funcs", 0, 1, kMaxDim);
      yi.inv_avg_n_neigh = v.double_scalar("YI_inv_avg_n_neigh", 1.0);
      require_eq("YI_n_rad_max", v.int_scalar("YI_n_rad_max", 32), CR, "the layer-2 radial channels mlp_rad_R1_n_rad_max");
      v.require_shape("YI_lr_inds", {yi.n_terms, 2});
      require_size("YI_m_sum_ind", yi.m_sum_ind, (size_t) yi.n_terms);
      require_size("YI_cg_coeff", yi.cg_coeff, (size_t) yi.n_terms);
      for (int t = 0; t < yi.n_terms; t++) {
        const int y = lr[2 * t], i = lr[2 * t + 1];
        if (y < 0 || y >= nlm_ || i < 0 || i >= I_n_funcs)
          throw bad_array("YI_lr_inds", "has (" + std::to_string(y) + ", " + std::to_string(i) + ") at " + std::to_string(t) + ", outside [0, " +
                                            std::to_string(nlm_) + ") x [0, I_n_funcs = " + std::to_string(I_n_funcs) + ")");
        yi.y.push_back(y);
        yi.i.push_back(i);
      }
      require_index("YI_m_sum_ind", yi.m_sum_ind, yi.n_out);
      require_eq("YI_n_output_funcs", yi.n_out, index_extent(yi.m_sum_ind), "1 + the largest YI_m_sum_ind");
    }
    elem_dependent("B", 0);
    load_reduce("B", "YI", B_red_YI, false, C2, B_n_funcs, CR, yi.n_out);
    load_reduce("B", "B0", B_red_B0, false, C2, B_n_funcs, CR, nlm_);
    const int64_t nB = B_n_funcs;
    load_fc("fc_B1", fc_B1, nB, nB, C2, "B_n_out");
    const int64_t nBB = load_prod("prod_BB", prod_BB, nB, nB);
    load_fc("fc_BB1", fc_BB1, nBB, nB, C2, "B_n_out");
    const int64_t nBBB = load_prod("prod_BBB", prod_BBB, nBB, nB);
    int64_t nBBBB = 0;
    if (order4) {
      load_fc("fc_BB2", fc_BB2, nBB, nB, C2, "B_n_out");
      nBBBB = load_prod("prod_BBBB", prod_BBBB, nBB, nBB);
    }
    const char *s2[4] = {"B", "BB", "BBB", "BBBB"};
    const int64_t nf2[4] = {nB, nBB, nBBB, nBBBB};
    require_eq("I2_n_out", v.int_in("I2_n_out", 17, 1, kMaxDim), rho_n_out, "the energy adds rho and I2 function by function: rho_n_out");
    elem_dependent("I2", 1);
    for (int s = 0; s < nsrc(); s++) load_reduce("I2", s2[s], I2_red[s], true, rho_n_out, 1, C2, nf2[s]);

    // ---- readout
    energy_rms_norm = v.flag("energy_rms_norm", 1);
    if (energy_rms_norm) {
      I_nl_LN_scale = v.require_doubles("I_nl_LN_scale");
      require_eq("I_nl_LN_type", v.int_scalar("I_nl_LN_type", 1), 1, "the GRACE-2L engines implement the only_nonlin RMSNorm here");
      require_eq("I_nl_LN_n_out", v.int_scalar("I_nl_LN_n_out", 17), rho_n_out, "rho_n_out");
      require_size("I_nl_LN_scale", I_nl_LN_scale, (size_t) rho_n_out - 1);
      I_0_LN_scale = v.require_doubles("I_0_LN_scale");
      require_eq("I_0_LN_type", v.int_scalar("I_0_LN_type", 0), 0, "the GRACE-2L engines implement the full RMSNorm here");
      require_eq("I_0_LN_n_out", v.int_scalar("I_0_LN_n_out", 17), rho_n_out, "I2_n_out");
      require_size("I_0_LN_scale", I_0_LN_scale, (size_t) rho_n_out);
    } else {
      I_nl_LN_scale.assign(rho_n_out - 1, 1.0);
      I_0_LN_scale.assign(rho_n_out, 1.0);
    }
    energy_mlp = load_mlp(v, "energy_mlp", v.int_in("energy_mlp_n_layers", 2, 1, kMaxDim), rho_n_out - 1, 1, "rho_n_out - 1", "one energy");
    energy_mlp_activation = v.int_in("energy_mlp_activation", 1, 0, 1);
    radial_activation = v.int_in("radial_activation", 0, 0, 1);
    {
      const auto s = v.doubles("energy_mlp_scale");
      if (!s.empty()) {
        MLPLayer &L = energy_mlp[0];
        require_size("energy_mlp_scale", s, (size_t) L.n_in);
        for (int k = 0; k < L.n_in; k++)
          for (int j = 0; j < L.n_out; j++) L.W[(size_t) k * L.n_out + j] *= s[k];
        energy_mlp_ln = true;
      }
    }
    if (energy_mlp.size() > 7) throw Error("GRACE-2L: energy MLP has " + std::to_string(energy_mlp.size()) + " layers, at most 7 supported");
    for (const auto &L : energy_mlp)
      if (L.n_in > 256 || L.n_out > 256) throw Error("GRACE-2L: energy MLP layer widths above 256 are not supported");
    shift_values = v.doubles("shift_values");
    if (v.has("shift_values")) require_size("shift_values", shift_values, (size_t) n_elements);
    else shift_values.assign(n_elements, 0.0);
    output_scale = v.double_scalar("output_scale", 1.0);
    uq.load(v, n_elements, "GRACE-2L/KK");
    element_names = v.names("element_names");
    if (v.has("element_names")) require_size("element_names", element_names, (size_t) n_elements);
  }
};

}    // namespace grhip
