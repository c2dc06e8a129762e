// Host-side container of a GRACE-3L model read from kokkos.npz.  The file names its components (SPBF layers, cp_l
// products, reduces, FCs, norms) in index lists; keys, defaults and the dataflow check follow the reference loader
// libgrace/src/model_3l.cpp:36-464 (container libgrace/include/grace/model_3l.h:38-190).
#pragma once

#include "model.hpp"

#include <map>

namespace grhip {

struct Model3L {
  struct Mlp {
    std::vector<MLPLayer> layers;
    std::vector<std::vector<double>> bias;    // per layer, empty: none
  };
  struct Spbf {
    std::string name;
    bool equivariant = false;
    int n_rad_max = 0, p = 5, nfunc = 0, n_lm_ind = 0;
    double inv_avg_n_neigh = 1.0, lin_transform_norm = 1.0, chem_linear_norm = 1.0;
    std::vector<int> l_tile;
    Mlp mlp;
    std::vector<double> lin_transform_W, chem_linear_W, chem_l0_mask, cg_W;
  };
  struct Cpl {
    std::string name;
    int rank = 0, nfunc = 0, n_left = 0, n_right = 0, n_groups_left = 0, n_groups_right = 0;
    double norm_u = 1.0, norm_v = 1.0;
    std::vector<double> U, V;    // [groups][rank][n_in]
    std::vector<int> group_left, group_right;
    CGProduct cg;
  };
  struct Instr {
    std::string name;
    std::vector<double> W;    // [n_elements |] [n_out][n_in][w_shape]
    double norm = 1.0;
    int n_in = 0, w_shape = 0;
    std::vector<int> collect_ind, w_l_tile, total_sum_ind;
  };
  struct Reduce {
    std::string name;
    int n_out = 0, n_funcs = 0;
    bool only_invar = false, elem_dep = false;
    std::vector<Instr> instr;
    std::vector<double> norm_map;    // per output function, empty: none
    int nfo() const { return only_invar ? 1 : n_funcs; }
  };
  struct Fc {
    std::string name;
    int n_out = 0, n_funcs_left = 0, n_in_right = 0, w_shape_right = 0;
    double norm_right = 1.0;
    std::vector<double> w_right, norm_out_factor;
    std::vector<int> w_tile_right, collect_to, collect_from;
  };
  struct EqNorm {
    std::string name;
    int n_groups = 0, n_out = 0, M = 0;
    bool center_l0 = true;
    double eps = 1e-8;
    std::vector<double> affine_weight, degree_weights, l0_mask;
    std::vector<int> expand_index;
  };
  struct RmsNorm {
    std::string name;
    int type = 0, n_out = 0;
    std::vector<double> scale;
  };

  int n_elements = 0, embedding_size = 0, lmax = 0, nradbase = 0, radial_basis_p = 5;
  double rcut = 0.0, output_scale = 1.0;
  bool has_bond_specific_cutoff = false;
  std::vector<double> bond_cutoff_map, chem_embedding, shift_values;
  std::vector<std::string> element_names;
  std::vector<Spbf> spbf;
  std::vector<Cpl> prod;
  std::vector<Reduce> reduce;
  std::vector<Fc> fc;
  std::vector<EqNorm> eqnorm;
  std::vector<RmsNorm> rmsnorm;
  Mlp energy_mlp;
  int energy_mlp_activation = 0, rho_width = 0;
  UqHead uq;    // uqv6 UQ head; a file whose head is broken does not load (libgrace/src/model_3l.cpp:453-463)
  static constexpr double rms_norm_eps = 1e-10;    // libgrace/include/grace/fused_3l_cpu.h:424

  int nl() const { return lmax + 1; }
  int nlm() const { return (lmax + 1) * (lmax + 1); }
  double pair_cutoff(int mu_i, int mu_j) const
  {
    if (mu_i < 0 || mu_j < 0) return 0.0;
    return has_bond_specific_cutoff ? bond_cutoff_map[(size_t) mu_i * n_elements + mu_j] : rcut;
  }
  template<class V> static const typename V::value_type &by_name(const V &v, const std::string &name)
  {
    for (const auto &x : v)
      if (x.name == name) return x;
    throw Error("GRACE-3L: no component '" + name + "'");
  }

  void load(const Npz &z)
  {
    *this = Model3L();
    NpzView v(z);
    if (v.has("grace_model_kind")) {
      const auto k = v.names("grace_model_kind");
      if (k.size() != 1) throw bad_array("grace_model_kind", "must hold one name");
      if (k[0] != "GRACE-3L") throw Error("GRACE-3L: the file holds a " + k[0] + " model");
      if (v.int_scalar("grace_format_version", 0) < 1) throw bad_array("grace_format_version", "is missing or below 1 next to grace_model_kind");
    }
    if (v.int_scalar("grace_format_version", 0) > 2)
      throw Error("GRACE-3L: kokkos.npz format " + std::to_string(v.int_scalar("grace_format_version", 0)) + ", this build reads up to 2");
    for (const char *k : {"energy_mlp_scale", "radial_activation", "energy_rms_norm", "AAA_right_A"})
      if (v.has(k)) throw bad_array(k, "is a legacy GRACE-1L/2L key, not supported in GRACE-3L");
    auto size = [&](const std::string &k) { return v.int_in(k, 0, 1, kMaxDim); };

    n_elements = size("n_elements");
    embedding_size = v.int_in("embedding_size", 64, 1, kMaxDim);
    nradbase = v.int_in("nradbase", 10, 1, kMaxDim);
    lmax = v.int_in("lmax", v.int_in("A1_lmax", 4, 0, kMaxL), 0, kMaxL);
    const int nl_ = lmax + 1, nlm_ = nl_ * nl_;
    rcut = v.cutoff_scalar("rcut", 6.0, "GRACE-3L/KK");
    has_bond_specific_cutoff = v.flag("has_bond_specific_cutoff", 0);
    chem_embedding = v.require_doubles("chem_embedding");
    v.require_shape("chem_embedding", {n_elements, embedding_size});
    shift_values = v.require_doubles("shift_values");
    require_size("shift_values", shift_values, n_elements);
    output_scale = v.double_scalar("output_scale", 1.0);
    element_names = v.names("element_names");
    require_size("element_names", element_names, n_elements);
    bond_cutoff_map = v.cutoffs("bond_cutoff_map", "GRACE-3L/KK");
    v.require_shape("bond_cutoff_map", {n_elements, n_elements});
    if (bond_cutoff_map.empty()) bond_cutoff_map.assign((size_t) n_elements * n_elements, rcut);

    auto load_net = [&](const std::string &p, Mlp &m, int64_t n_in, int64_t n_out, const std::string &in_why, const std::string &out_why) {
      const int n = v.int_in(p + "_n_layers", 0, 1, kMaxDim);
      if (v.has(p + "_W" + std::to_string(n))) throw bad_array(p + "_n_layers", "is " + std::to_string(n) + ", but the file has " + p + "_W" + std::to_string(n));
      m.layers = load_mlp(v, p, n, n_in, n_out, in_why, out_why);
      for (int i = 0; i < n; i++) {
        const std::string bk = p + "_b" + std::to_string(i);
        m.bias.push_back(v.doubles(bk));
        if (v.has(bk)) require_size(bk, m.bias.back(), m.layers[i].n_out);
      }
    };

    for (const auto &nm : v.names("spbf_names")) {
      Spbf s;
      s.name = nm;
      s.equivariant = v.flag(nm + "_equivariant", 0);
      s.n_rad_max = size(nm + "_n_rad_max");
      require_eq(nm + "_n_rad_basis", v.int_scalar(nm + "_n_rad_basis", nradbase), nradbase, "nradbase, the radial MLP's Chebyshev inputs");
      require_eq(nm + "_lmax", v.int_scalar(nm + "_lmax", 4), lmax, "the model's lmax");
      (void) v.int_in(nm + "_Lmax", 4, 0, kMaxL);
      s.p = v.int_in(nm + "_p", 5, 1, kMaxP);
      (void) v.cutoff_scalar(nm + "_rcut", rcut, "GRACE-3L/KK");
      s.inv_avg_n_neigh = v.double_scalar(nm + "_inv_avg_n_neigh", 1.0);
      s.l_tile = v.require_ints(nm + "_l_tile");
      require_size(nm + "_l_tile", s.l_tile, nlm_);
      require_index(nm + "_l_tile", s.l_tile, nl_);
      load_net(nm + "_mlp", s.mlp, nradbase + 2 * embedding_size, (int64_t) s.n_rad_max * nl_, "nradbase + 2 embedding_size", "n_rad_max (lmax+1)");
      if (!s.equivariant) {
        s.lin_transform_W = v.require_doubles(nm + "_lin_transform_W");
        v.require_shape(nm + "_lin_transform_W", {embedding_size, s.n_rad_max});
        s.lin_transform_norm = v.double_scalar(nm + "_lin_transform_norm", 1.0);
      } else {
        s.nfunc = size(nm + "_nfunc");
        s.n_lm_ind = size(nm + "_n_lm_ind");
        s.chem_linear_W = v.require_doubles(nm + "_chem_linear_W");
        v.require_shape(nm + "_chem_linear_W", {embedding_size, s.n_rad_max});
        s.chem_linear_norm = v.double_scalar(nm + "_chem_linear_norm", 1.0);
        s.chem_l0_mask = v.require_doubles(nm + "_chem_l0_mask");
        require_size(nm + "_chem_l0_mask", s.chem_l0_mask, s.n_lm_ind);
        s.cg_W = v.require_doubles(nm + "_cg_W");
        v.require_shape(nm + "_cg_W", {(int64_t) nlm_ * s.n_lm_ind, s.nfunc});
      }
      spbf.push_back(std::move(s));
    }
    if (!spbf.empty()) radial_basis_p = spbf[0].p;
    for (const auto &s : spbf)
      if (s.p != radial_basis_p)
        throw bad_array(s.name + "_p", "is " + std::to_string(s.p) + ", the envelope order of " + spbf[0].name + " is " + std::to_string(radial_basis_p) +
                                           "; layers with different orders are not supported");

    for (const auto &nm : v.names("prod_names")) {
      Cpl c;
      c.name = nm;
      c.rank = size(nm + "_rank");
      c.nfunc = size(nm + "_nfunc");
      c.n_left = size(nm + "_n_left");
      c.n_right = size(nm + "_n_right");
      c.n_groups_left = size(nm + "_n_groups_left");
      c.n_groups_right = size(nm + "_n_groups_right");
      c.norm_u = v.double_scalar(nm + "_norm_u", 1.0);
      c.norm_v = v.double_scalar(nm + "_norm_v", 1.0);
      c.U = v.require_doubles(nm + "_U");
      v.require_shape(nm + "_U", {c.n_groups_left, c.rank, c.n_left});
      c.V = v.require_doubles(nm + "_V");
      v.require_shape(nm + "_V", {c.n_groups_right, c.rank, c.n_right});
      c.cg.cg_coeff = v.require_doubles(nm + "_cg");
      c.cg.n_terms = (int) c.cg.cg_coeff.size();
      c.cg.n_out = c.nfunc;
      c.group_left = v.require_ints(nm + "_group_left");
      require_index(nm + "_group_left", c.group_left, c.n_groups_left);
      c.group_right = v.require_ints(nm + "_group_right");
      require_index(nm + "_group_right", c.group_right, c.n_groups_right);
      c.cg.left_ind = v.require_ints(nm + "_left_ind");
      require_size(nm + "_left_ind", c.cg.left_ind, c.cg.n_terms);
      require_index(nm + "_left_ind", c.cg.left_ind, (int64_t) c.group_left.size());
      c.cg.right_ind = v.require_ints(nm + "_right_ind");
      require_size(nm + "_right_ind", c.cg.right_ind, c.cg.n_terms);
      require_index(nm + "_right_ind", c.cg.right_ind, (int64_t) c.group_right.size());
      c.cg.m_sum_ind = v.require_ints(nm + "_m_sum_ind");
      require_size(nm + "_m_sum_ind", c.cg.m_sum_ind, c.cg.n_terms);
      require_index(nm + "_m_sum_ind", c.cg.m_sum_ind, c.nfunc);
      const auto out_l = v.require_ints(nm + "_out_l");
      require_size(nm + "_out_l", out_l, c.nfunc);
      require_index(nm + "_out_l", out_l, kMaxL + 1);
      prod.push_back(std::move(c));
    }

    for (const auto &nm : v.names("reduce_names")) {
      Reduce r;
      r.name = nm;
      r.n_out = size(nm + "_n_out");
      r.n_funcs = size(nm + "_n_funcs");
      r.only_invar = v.flag(nm + "_only_invar", 0);
      r.elem_dep = v.flag(nm + "_is_central_atom_type_dependent", 0);
      for (const auto &cn : v.names(nm + "_instruction_names")) {
        Instr ri;
        ri.name = cn;
        ri.n_in = size(nm + "_n_in_" + cn);
        ri.w_shape = size(nm + "_w_shape_" + cn);
        const std::string wk = nm + "_reduce_" + cn + "_W";
        ri.W = v.require_doubles(wk);
        if (r.elem_dep) v.require_shape(wk, {n_elements, r.n_out, ri.n_in, ri.w_shape});
        else v.require_shape(wk, {r.n_out, ri.n_in, ri.w_shape});
        ri.norm = v.double_scalar(nm + "_reduce_" + cn + "_norm", 1.0);
        ri.collect_ind = v.require_ints(nm + "_collect_ind_" + cn);
        const size_t nc = ri.collect_ind.size();
        ri.w_l_tile = v.require_ints(nm + "_w_l_tile_" + cn);
        require_size(nm + "_w_l_tile_" + cn, ri.w_l_tile, nc);
        require_index(nm + "_w_l_tile_" + cn, ri.w_l_tile, ri.w_shape);
        ri.total_sum_ind = v.require_ints(nm + "_total_sum_ind_" + cn);
        require_size(nm + "_total_sum_ind_" + cn, ri.total_sum_ind, nc);
        require_index(nm + "_total_sum_ind_" + cn, ri.total_sum_ind, r.nfo());
        r.instr.push_back(std::move(ri));
      }
      r.norm_map = v.doubles(nm + "_norm_map");
      if (v.has(nm + "_norm_map")) require_size(nm + "_norm_map", r.norm_map, r.nfo());
      reduce.push_back(std::move(r));
    }

    for (const auto &nm : v.names("fc_names")) {
      Fc f;
      f.name = nm;
      const std::string p = "fc_" + nm;
      f.n_out = size(p + "_n_out");
      if (v.flag(p + "_left_coefs", 0)) throw bad_array(p + "_left_coefs", "is 1: FCs with left weights are not a part of the GRACE-3L architecture");
      f.w_right = v.require_doubles(p + "_w_right");
      const auto wr = v.shape_rank(p + "_w_right", 3);
      require_eq(p + "_w_right", (int64_t) wr[0], f.n_out, p + "_n_out", "rows");
      f.n_in_right = (int) wr[1];
      f.w_shape_right = (int) wr[2];
      f.norm_right = v.double_scalar(p + "_norm_right", 1.0);
      f.n_funcs_left = (int) v.shape_rank(p + "_w_tile_left", 1)[0];
      f.norm_out_factor = v.require_doubles(p + "_norm_out_factor");
      require_size(p + "_norm_out_factor", f.norm_out_factor, f.n_funcs_left);
      f.collect_from = v.require_ints(p + "_collect_from");
      f.collect_to = v.require_ints(p + "_collect_to");
      require_size(p + "_collect_to", f.collect_to, f.collect_from.size());
      require_index(p + "_collect_to", f.collect_to, f.n_funcs_left);
      f.w_tile_right = v.require_ints(p + "_w_tile_right");
      require_size(p + "_w_tile_right", f.w_tile_right, f.collect_from.size());
      require_index(p + "_w_tile_right", f.w_tile_right, f.w_shape_right);
      fc.push_back(std::move(f));
    }

    for (const auto &nm : v.names("eqnorm_names")) {
      EqNorm e;
      e.name = nm;
      e.affine_weight = v.require_doubles(nm + "_affine_weight");
      const auto aw = v.shape_rank(nm + "_affine_weight", 2);
      e.n_groups = (int) aw[0];
      e.n_out = (int) aw[1];
      e.degree_weights = v.require_doubles(nm + "_degree_weights");
      e.M = (int) e.degree_weights.size();
      e.l0_mask = v.require_doubles(nm + "_l0_mask");
      require_size(nm + "_l0_mask", e.l0_mask, e.M);
      e.expand_index = v.require_ints(nm + "_expand_index");
      require_size(nm + "_expand_index", e.expand_index, e.M);
      require_index(nm + "_expand_index", e.expand_index, e.n_groups);
      e.eps = v.double_scalar(nm + "_eps", 1e-8);
      if (e.eps < 0.0) throw bad_array(nm + "_eps", "is negative");
      e.center_l0 = v.flag(nm + "_center_l0", 1);
      eqnorm.push_back(std::move(e));
    }
    for (const auto &nm : v.names("rmsnorm_names")) {
      RmsNorm r;
      r.name = nm;
      r.scale = v.require_doubles(nm + "_scale");
      r.type = v.flag(nm + "_type", 0) ? 1 : 0;
      r.n_out = v.int_in(nm + "_n_out", (int) std::min<size_t>(r.scale.size() + r.type, kMaxDim), 1, kMaxDim);
      require_size(nm + "_scale", r.scale, r.n_out - r.type);
      rmsnorm.push_back(std::move(r));
    }
    const auto origins = v.names("out1_origins");
    require_eq("energy_mlp_n_origins", v.int_scalar("energy_mlp_n_origins", (int) origins.size()), (int64_t) origins.size(), "the names in out1_origins");
    rho_width = check_dataflow(origins);
    if (v.has("energy_mlp_origin_n_out")) require_eq("energy_mlp_origin_n_out", v.int_scalar("energy_mlp_origin_n_out", 0), rho_width, "the channels of out1_origins");
    load_net("energy_mlp", energy_mlp, rho_width - 1, 1, "the channels of out1_origins but the linear channel 0", "one energy per atom");
    energy_mlp_activation = v.int_in("energy_mlp_activation", 0, 0, 1);
    // ---- UQ head (optional): the GMM feature projects the inputs of the rho1 | rho2 | rho3 reduces
    uq.load(v, n_elements, "GRACE-3L");
    if (uq.has_uq) {
      if (uq.schema != 6)
        throw Error("GRACE-3L UQ: schema v" + std::to_string(uq.schema) + " unsupported (expects v6, uqv6 basis-RP normalize+density). Re-export the "
                    "UQ artifacts at schema v6 with a current grace_utils.");
      if (!uq.error.empty()) throw Error(uq.error);
      if (uq.n_density > 4)
        throw Error("GRACE-3L UQ: uq_n_density (" + std::to_string(uq.n_density) + ") > 4, the number of density channels this model's UQ kernels "
                    "write. Artifact has an unexpected invariant-block count.");
      int64_t width = 0;
      for (int k = 1; k <= 3; k++)
        for (const auto &ins : by_name(reduce, "rho" + std::to_string(k)).instr) width += (int64_t) ins.n_in * (int64_t) ins.collect_ind.size();
      require_eq("uq_rp_matrix", uq.d_basis, width, "the inputs of the rho1, rho2, rho3 reduces", "rows");
    }
  }

 private:
  // Every component against the functions and channels of its inputs, in the order the engines evaluate them
  // (libgrace/src/model_3l.cpp:36-154); a component outside the three-layer graph, or a missing one, is an error.
  int check_dataflow(const std::vector<std::string> &origins)
  {
    struct Shape {
      int nf, nc;
    };
    std::map<std::string, Shape> T;
    std::map<std::string, int> used;
    auto find = [&](auto &vec, const char *list, const std::string &name) -> auto & {
      int at = -1;
      for (size_t i = 0; i < vec.size(); i++)
        if (vec[i].name == name) {
          if (at >= 0) throw bad_array(list, "lists '" + name + "' twice");
          at = (int) i;
        }
      if (at < 0) throw bad_array(list, "has no '" + name + "', a part of the GRACE-3L architecture");
      used[std::string(list) + "/" + name] = 1;
      return vec[at];
    };
    auto unused = [&](auto &vec, const char *list) {
      for (const auto &x : vec)
        if (!used.count(std::string(list) + "/" + x.name)) throw bad_array(list, "lists '" + x.name + "', not a part of the GRACE-3L architecture");
    };
    auto red = [&](const std::string &name, std::vector<std::string> inputs) {
      auto &r = find(reduce, "reduce_names", name);
      std::vector<std::string> got;
      for (const auto &ins : r.instr) got.push_back(ins.name);
      std::vector<std::string> a = got, b = inputs;
      std::sort(a.begin(), a.end());
      std::sort(b.begin(), b.end());
      if (a != b) throw bad_array(name + "_instruction_names", "does not name the inputs of " + name + " in the GRACE-3L architecture");
      for (const auto &ins : r.instr) {
        const Shape in = T.at(ins.name);
        require_eq(name + "_n_in_" + ins.name, ins.n_in, in.nc, "the channels of " + ins.name);
        require_index(name + "_collect_ind_" + ins.name, ins.collect_ind, in.nf);
      }
      T[name] = {r.nfo(), r.n_out};
    };
    auto cpl = [&](const std::string &name, const std::string &left, const std::string &right) {
      auto &c = find(prod, "prod_names", name);
      const Shape l = T.at(left), r = T.at(right);
      require_eq(name + "_group_left", (int64_t) c.group_left.size(), l.nf, "the functions of " + left, "values");
      require_eq(name + "_n_left", c.n_left, l.nc, "the channels of " + left);
      require_eq(name + "_group_right", (int64_t) c.group_right.size(), r.nf, "the functions of " + right, "values");
      require_eq(name + "_n_right", c.n_right, r.nc, "the channels of " + right);
      T[name] = {c.nfunc, c.rank};
    };
    auto fcl = [&](const std::string &name, const std::string &left, const std::string &right) {
      auto &f = find(fc, "fc_names", name);
      const std::string p = "fc_" + name;
      const Shape l = T.at(left), r = T.at(right);
      require_eq(p + "_w_tile_left", f.n_funcs_left, l.nf, "the functions of " + left, "values");
      require_eq(p + "_n_out", f.n_out, l.nc, "the channels of " + left);
      require_eq(p + "_w_right", f.n_in_right, r.nc, "the channels of " + right, "columns");
      require_index(p + "_collect_from", f.collect_from, r.nf);
      T[name] = {f.n_funcs_left, f.n_out};
    };
    if (spbf.size() != 3) throw bad_array("spbf_names", "has " + std::to_string(spbf.size()) + " names, expected 3 (A1, A2, A3)");
    for (int k = 1; k <= 3; k++) {
      const std::string ks = std::to_string(k), K = "A" + ks;
      auto &s = find(spbf, "spbf_names", K);
      if (s.name != spbf[k - 1].name) throw bad_array("spbf_names", "lists '" + K + "' out of order");
      std::string X = K;
      if (k == 1) {
        if (s.equivariant) throw bad_array(K + "_equivariant", "is 1, expected 0 (the first layer has no message to couple)");
        T[K] = {nlm(), s.n_rad_max};
      } else {
        if (!s.equivariant) throw bad_array(K + "_equivariant", "is 0, expected 1 (the layer couples the message of the one before)");
        const std::string msg = "eq" + std::to_string(k - 1) + "_norm";
        require_eq(K + "_n_lm_ind", s.n_lm_ind, T.at(msg).nf, "the functions of the message " + msg);
        require_eq(K + "_n_rad_max", s.n_rad_max, T.at(msg).nc, "the channels of the message " + msg);
        T[K] = {s.nfunc, s.n_rad_max};
        red(K + "_red", {K});
        X = K + "_red";
      }
      cpl(K + "_2", X, X);
      red(K + "_2_red", {K + "_2"});
      fcl(K + "_2a", K + "_2_red", X);
      cpl(K + "_3", K + "_2a", X);
      red(K + "_3_red", {K + "_3"});
      fcl(K + "_2b", K + "_2_red", X);
      cpl(K + "_4", K + "_2b", K + "_2b");
      red(K + "_4_red", {K + "_4"});
      const std::vector<std::string> collect = {X, K + "_2_red", K + "_3_red", K + "_4_red"};
      if (k < 3) {
        red("eq" + ks, collect);
        auto &e = find(eqnorm, "eqnorm_names", "eq" + ks + "_norm");
        const Shape in = T.at("eq" + ks);
        require_eq(e.name + "_degree_weights", e.M, in.nf, "the functions of eq" + ks, "values");
        require_eq(e.name + "_affine_weight", e.n_out, in.nc, "the channels of eq" + ks, "columns");
        T[e.name] = {e.M, e.n_out};
      }
      red("rho" + ks, collect);
      auto &n = find(rmsnorm, "rmsnorm_names", "rho" + ks + "_norm");
      const Shape in = T.at("rho" + ks);
      require_eq(n.name + "_n_out", n.n_out, in.nc, "the channels of rho" + ks);
      T[n.name] = {in.nf, n.n_out};
    }
    unused(spbf, "spbf_names");
    unused(prod, "prod_names");
    unused(reduce, "reduce_names");
    unused(fc, "fc_names");
    unused(eqnorm, "eqnorm_names");
    unused(rmsnorm, "rmsnorm_names");
    std::vector<std::string> want = {"rho1_norm", "rho2_norm", "rho3_norm"}, got = origins;
    std::sort(got.begin(), got.end());
    if (got != want) throw bad_array("out1_origins", "does not name rho1_norm, rho2_norm, rho3_norm");
    const int w = T.at(want[0]).nc;
    for (const auto &o : want) require_eq(o + "_n_out", T.at(o).nc, w, "the channels of " + want[0]);
    return w;
  }
};

}    // namespace grhip
