// Host-side container of a GRACE-3L model read from kokkos.npz and its loader.  The file lists its components (SPBF layers,
// cp_l products, reduces, FCs, norms) by name; keys and consistency rules are the file format's, as the reference loader
// reads it (libgrace/src/model_3l.cpp:36-464, container libgrace/include/grace/model_3l.h:38-190).  The architecture the
// engines evaluate is written down once, as a table of components and their inputs (kLayerPlan), and the file is
// checked against that table.
#pragma once

#include "model.hpp"

#include <map>
#include <set>

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
    throw Error("GRACE-3L: the model has no component named '" + name + "'");
  }

  void load(const Npz &z)
  {
    *this = Model3L();
    const FileReader f(z, "GRACE-3L");
    check_declaration(f, "GRACE-3L");
    for (const char *old : {"energy_mlp_scale", "radial_activation", "energy_rms_norm", "AAA_right_A"})
      if (f.present(old)) f.reject(old, "is a switch of the one- and two-layer formats; a GRACE-3L file must not carry it");

    n_elements = (int) f.whole("n_elements", 1, kSizeLimit);
    embedding_size = (int) f.whole_or("embedding_size", 1, kSizeLimit, 64);
    nradbase = (int) f.whole_or("nradbase", 1, kSizeLimit, 10);
    lmax = (int) f.whole_or("lmax", 0, kDegreeLimit, f.whole_or("A1_lmax", 0, kDegreeLimit, 4));
    rcut = f.length_or("rcut", 6.0);
    has_bond_specific_cutoff = f.flag_or("has_bond_specific_cutoff", false);
    bond_cutoff_map = f.distances_or_none("bond_cutoff_map", n_elements, n_elements);
    if (bond_cutoff_map.empty()) bond_cutoff_map.assign((size_t) n_elements * n_elements, rcut);
    chem_embedding = f.reals("chem_embedding", {n_elements, embedding_size});
    shift_values = f.reals("shift_values", Flat{n_elements});
    output_scale = f.real_or("output_scale", 1.0);
    element_names = f.labels("element_names");
    if ((long) element_names.size() != n_elements)
      f.reject("element_names", "lists " + std::to_string(element_names.size()) + " elements where n_elements = " + std::to_string(n_elements));

    for (const std::string &name : f.labels("spbf_names")) spbf.push_back(read_spbf(f, name));
    for (const std::string &name : f.labels("prod_names")) prod.push_back(read_couple(f, name));
    for (const std::string &name : f.labels("reduce_names")) reduce.push_back(read_projection(f, name));
    for (const std::string &name : f.labels("fc_names")) fc.push_back(read_right_fc(f, name));
    for (const std::string &name : f.labels("eqnorm_names")) eqnorm.push_back(read_eqnorm(f, name));
    for (const std::string &name : f.labels("rmsnorm_names")) rmsnorm.push_back(read_rmsnorm(f, name));

    // one envelope for all layers
    if (!spbf.empty()) radial_basis_p = spbf[0].p;
    for (const Spbf &s : spbf)
      if (s.p != radial_basis_p)
        f.reject(s.name + "_p", "= " + std::to_string(s.p) + " while " + spbf[0].name + " uses the envelope order " + std::to_string(radial_basis_p) +
                                    "; the engines evaluate one envelope for all layers");

    rho_width = check_against_plan(f);
    const std::vector<std::string> origins = f.labels("out1_origins");
    if (std::set<std::string>(origins.begin(), origins.end()) != std::set<std::string>{"rho1_norm", "rho2_norm", "rho3_norm"} || origins.size() != 3)
      f.reject("out1_origins", "must name the three normalised densities rho1_norm, rho2_norm, rho3_norm, whose sum the readout takes");
    f.must_be("energy_mlp_n_origins", 3, 3, "the readout sums three densities");
    f.must_be("energy_mlp_origin_n_out", rho_width, rho_width, "it is the channel width of the normalised densities");
    read_net(f, "energy_mlp", energy_mlp, rho_width - 1, 1);
    energy_mlp_activation = (int) f.whole_or("energy_mlp_activation", 0, 1, 0);

    // ---- UQ head (optional): the GMM feature projects the inputs of the rho1 | rho2 | rho3 reduces.  Unlike the one- and
    // two-layer loaders this one refuses a file whose head cannot be evaluated.
    uq.load(f, n_elements);
    if (uq.has_uq) {
      if (uq.schema != 6) throw Error("GRACE-3L: UQ head of schema " + std::to_string(uq.schema) + "; only schema 6 (uqv6) can be evaluated");
      if (!uq.error.empty()) throw Error(uq.error);
      if (uq.n_density > 4)
        throw Error("GRACE-3L UQ head: " + std::to_string(uq.n_density) + " density channels; the three-layer kernels write at most 4 (total, rho1, rho2, rho3)");
      long basis = 0;
      for (const char *rho : {"rho1", "rho2", "rho3"})
        for (const Instr &ins : by_name(reduce, rho).instr) basis += (long) ins.n_in * (long) ins.collect_ind.size();
      if (basis != uq.d_basis)
        f.reject("uq_rp_matrix", "projects " + std::to_string(uq.d_basis) + " basis functions; the inputs of rho1, rho2, rho3 hold " + std::to_string(basis));
    }
  }

 private:
  // ---- component readers --------------------------------------------------------------------------------------
  // dense stack with optional biases `<stem>_b<k>`; the declared depth must match the matrices in the file
  static void read_net(const FileReader &f, const std::string &stem, Mlp &net, long first_in, long last_out)
  {
    const long depth = f.whole(stem + "_n_layers", 1, kSizeLimit);
    if (f.present(stem + "_W" + std::to_string(depth)))
      f.reject(stem + "_n_layers", "= " + std::to_string(depth) + " but the file holds a further matrix " + stem + "_W" + std::to_string(depth));
    net.layers = read_dense_stack(f, stem, depth, first_in, last_out);
    for (long k = 0; k < depth; k++) {
      const std::string key = stem + "_b" + std::to_string(k);
      net.bias.push_back(f.present(key) ? f.reals(key, Flat{net.layers[(size_t) k].n_out}) : std::vector<double>());
    }
  }
  Spbf read_spbf(const FileReader &f, const std::string &name) const
  {
    Spbf s;
    s.name = name;
    s.equivariant = f.flag_or(name + "_equivariant", false);
    s.n_rad_max = (int) f.whole(name + "_n_rad_max", 1, kSizeLimit);
    s.p = (int) f.whole_or(name + "_p", 1, kEnvelopeLimit, 5);
    s.inv_avg_n_neigh = f.real_or(name + "_inv_avg_n_neigh", 1.0);
    f.must_be(name + "_n_rad_basis", nradbase, nradbase, "every layer's radial network takes the nradbase Chebyshev functions");
    f.must_be(name + "_lmax", 4, lmax, "every layer expands the bonds up to the model's lmax");
    (void) f.whole_or(name + "_Lmax", 0, kDegreeLimit, 4);
    (void) f.length_or(name + "_rcut", rcut);
    s.l_tile = f.indices(name + "_l_tile", {nlm()}, nl());
    read_net(f, name + "_mlp", s.mlp, nradbase + 2 * embedding_size, (long) s.n_rad_max * nl());
    if (s.equivariant) {
      s.nfunc = (int) f.whole(name + "_nfunc", 1, kSizeLimit);
      s.n_lm_ind = (int) f.whole(name + "_n_lm_ind", 1, kSizeLimit);
      s.chem_linear_W = f.reals(name + "_chem_linear_W", {embedding_size, s.n_rad_max});
      s.chem_linear_norm = f.real_or(name + "_chem_linear_norm", 1.0);
      s.chem_l0_mask = f.reals(name + "_chem_l0_mask", Flat{s.n_lm_ind});
      s.cg_W = f.reals(name + "_cg_W", {(long) nlm() * s.n_lm_ind, s.nfunc});
    } else {
      s.lin_transform_W = f.reals(name + "_lin_transform_W", {embedding_size, s.n_rad_max});
      s.lin_transform_norm = f.real_or(name + "_lin_transform_norm", 1.0);
    }
    return s;
  }
  static Cpl read_couple(const FileReader &f, const std::string &name)
  {
    Cpl c;
    c.name = name;
    int *const into[] = {&c.rank, &c.nfunc, &c.n_left, &c.n_right, &c.n_groups_left, &c.n_groups_right};
    const char *const keys[] = {"_rank", "_nfunc", "_n_left", "_n_right", "_n_groups_left", "_n_groups_right"};
    for (int k = 0; k < 6; k++) *into[k] = (int) f.whole(name + keys[k], 1, kSizeLimit);
    c.U = f.reals(name + "_U", {c.n_groups_left, c.rank, c.n_left});
    c.V = f.reals(name + "_V", {c.n_groups_right, c.rank, c.n_right});
    c.norm_u = f.real_or(name + "_norm_u", 1.0);
    c.norm_v = f.real_or(name + "_norm_v", 1.0);
    long lf = 0, rf = 0, terms = 0;
    c.group_left = f.indices(name + "_group_left", {Ext::any(lf)}, c.n_groups_left);
    c.group_right = f.indices(name + "_group_right", {Ext::any(rf)}, c.n_groups_right);
    c.cg.cg_coeff = f.reals(name + "_cg", {Ext::any(terms)});
    c.cg.left_ind = f.indices(name + "_left_ind", {terms}, lf);
    c.cg.right_ind = f.indices(name + "_right_ind", {terms}, rf);
    c.cg.m_sum_ind = f.indices(name + "_m_sum_ind", {terms}, c.nfunc);
    (void) f.indices(name + "_out_l", {c.nfunc}, kDegreeLimit + 1);
    c.cg.n_terms = (int) terms;
    c.cg.n_out = c.nfunc;
    return c;
  }
  Reduce read_projection(const FileReader &f, const std::string &name) const
  {
    Reduce r;
    r.name = name;
    r.n_out = (int) f.whole(name + "_n_out", 1, kSizeLimit);
    r.n_funcs = (int) f.whole(name + "_n_funcs", 1, kSizeLimit);
    r.only_invar = f.flag_or(name + "_only_invar", false);
    r.elem_dep = f.flag_or(name + "_is_central_atom_type_dependent", false);
    for (const std::string &source : f.labels(name + "_instruction_names")) {
      Instr in;
      in.name = source;
      in.n_in = (int) f.whole(name + "_n_in_" + source, 1, kSizeLimit);
      in.w_shape = (int) f.whole(name + "_w_shape_" + source, 1, kSizeLimit);
      const std::string W = name + "_reduce_" + source + "_W";
      in.W = r.elem_dep ? f.reals(W, {n_elements, r.n_out, in.n_in, in.w_shape}) : f.reals(W, {r.n_out, in.n_in, in.w_shape});
      in.norm = f.real_or(name + "_reduce_" + source + "_norm", 1.0);
      long picked = 0;
      in.collect_ind = f.indices(name + "_collect_ind_" + source, {Ext::any(picked)}, kSizeLimit);    // range: checked against the plan
      in.w_l_tile = f.indices(name + "_w_l_tile_" + source, {picked}, in.w_shape);
      in.total_sum_ind = f.indices(name + "_total_sum_ind_" + source, {picked}, r.nfo());
      r.instr.push_back(std::move(in));
    }
    if (f.present(name + "_norm_map")) r.norm_map = f.reals(name + "_norm_map", Flat{r.nfo()});
    return r;
  }
  static Fc read_right_fc(const FileReader &f, const std::string &name)
  {
    Fc c;
    c.name = name;
    const std::string p = "fc_" + name;
    c.n_out = (int) f.whole(p + "_n_out", 1, kSizeLimit);
    f.must_be(p + "_left_coefs", 0, 0, "the FC layers of the three-layer architecture carry weights on their right input only");
    long in_right = 0, tiles = 0, functions = 0, links = 0;
    c.w_right = f.reals(p + "_w_right", {c.n_out, Ext::any(in_right), Ext::any(tiles)});
    c.norm_right = f.real_or(p + "_norm_right", 1.0);
    (void) f.indices(p + "_w_tile_left", {Ext::any(functions)}, kSizeLimit);
    c.norm_out_factor = f.reals(p + "_norm_out_factor", Flat{functions});
    c.collect_from = f.indices(p + "_collect_from", {Ext::any(links)}, kSizeLimit);    // range: checked against the plan
    c.collect_to = f.indices(p + "_collect_to", {links}, functions);
    c.w_tile_right = f.indices(p + "_w_tile_right", {links}, tiles);
    c.n_in_right = (int) in_right;
    c.w_shape_right = (int) tiles;
    c.n_funcs_left = (int) functions;
    return c;
  }
  static EqNorm read_eqnorm(const FileReader &f, const std::string &name)
  {
    EqNorm e;
    e.name = name;
    long groups = 0, width = 0, functions = 0;
    e.affine_weight = f.reals(name + "_affine_weight", {Ext::any(groups), Ext::any(width)});
    e.degree_weights = f.reals(name + "_degree_weights", {Ext::any(functions)});
    e.l0_mask = f.reals(name + "_l0_mask", Flat{functions});
    e.expand_index = f.indices(name + "_expand_index", {functions}, groups);
    e.eps = f.real_or(name + "_eps", 1e-8);
    if (e.eps < 0.0) f.reject(name + "_eps", "is negative; it is added to a mean square");
    e.center_l0 = f.flag_or(name + "_center_l0", true);
    e.n_groups = (int) groups;
    e.n_out = (int) width;
    e.M = (int) functions;
    return e;
  }
  static RmsNorm read_rmsnorm(const FileReader &f, const std::string &name)
  {
    RmsNorm r;
    r.name = name;
    r.type = f.flag_or(name + "_type", false) ? 1 : 0;    // 1: the linear channel 0 is left out
    long scaled = 0;
    r.scale = f.reals(name + "_scale", {Ext::any(scaled)});
    r.n_out = (int) f.whole_or(name + "_n_out", 1, kSizeLimit, scaled + r.type);
    if (r.n_out - r.type != scaled)
      f.reject(name + "_scale", "holds " + std::to_string(scaled) + " values, expected " + std::to_string(r.n_out - r.type) + " for " + std::to_string(r.n_out) + " channels");
    return r;
  }

  // ---- the architecture ---------------------------------------------------------------------------------------
  // One row per component of a layer, in evaluation order.  '#' in a name stands for the layer number, "X" for the
  // layer's basis functions: the SPBF output A1 in layer 1, its projection A#_red in layers 2 and 3.
  enum class Part { Basis, Project, Couple, MixRight, MessageNorm, DensityNorm };
  struct PlanRow {
    Part part;
    const char *name;
    const char *in[4];     // inputs (Couple, MixRight: left, right; Project: up to four sources)
    int first, last;       // layers that have the row
  };
  static const std::vector<PlanRow> &layer_plan()
  {
    static const std::vector<PlanRow> kLayerPlan = {
        {Part::Basis, "A#", {}, 1, 3},
        {Part::Project, "A#_red", {"A#"}, 2, 3},
        {Part::Couple, "A#_2", {"X", "X"}, 1, 3},
        {Part::Project, "A#_2_red", {"A#_2"}, 1, 3},
        {Part::MixRight, "A#_2a", {"A#_2_red", "X"}, 1, 3},
        {Part::Couple, "A#_3", {"A#_2a", "X"}, 1, 3},
        {Part::Project, "A#_3_red", {"A#_3"}, 1, 3},
        {Part::MixRight, "A#_2b", {"A#_2_red", "X"}, 1, 3},
        {Part::Couple, "A#_4", {"A#_2b", "A#_2b"}, 1, 3},
        {Part::Project, "A#_4_red", {"A#_4"}, 1, 3},
        {Part::Project, "eq#", {"X", "A#_2_red", "A#_3_red", "A#_4_red"}, 1, 2},
        {Part::MessageNorm, "eq#_norm", {"eq#"}, 1, 2},
        {Part::Project, "rho#", {"X", "A#_2_red", "A#_3_red", "A#_4_red"}, 1, 3},
        {Part::DensityNorm, "rho#_norm", {"rho#"}, 1, 3},
    };
    return kLayerPlan;
  }
  struct Extent2 {
    long functions, channels;
  };
  // Walks the plan: every row must be in the file's inventory exactly once, sized for the tensors its inputs produce; and
  // the inventories must hold nothing else.  Returns the channel width of the normalised densities.
  long check_against_plan(const FileReader &f) const
  {
    std::map<std::string, Extent2> made;       // tensors produced so far
    std::set<std::string> visited;             // "<inventory>/<name>"
    auto locate = [&](const auto &inventory, const char *list, const std::string &name) {
      long hits = 0, at = -1;
      for (size_t k = 0; k < inventory.size(); k++)
        if (inventory[k].name == name) { hits++; at = (long) k; }
      if (hits == 0) f.reject(list, "does not list '" + name + "', which the three-layer architecture needs");
      if (hits > 1) f.reject(list, "lists '" + name + "' " + std::to_string(hits) + " times");
      visited.insert(std::string(list) + "/" + name);
      return (size_t) at;
    };
    auto same = [&](const std::string &key, long have, long want, const std::string &of) {
      if (have != want) f.reject(key, "is sized for " + std::to_string(have) + " where " + of + " gives " + std::to_string(want));
    };
    if (spbf.size() != 3) f.reject("spbf_names", "lists " + std::to_string(spbf.size()) + " layers; the architecture has three (A1, A2, A3)");
    for (int layer = 1; layer <= 3; layer++) {
      const std::string number = std::to_string(layer);
      auto spell = [&](const char *pattern) {
        std::string s = pattern ? pattern : "";
        if (s == "X") s = layer == 1 ? "A#" : "A#_red";
        for (size_t at; (at = s.find('#')) != std::string::npos;) s.replace(at, 1, number);
        return s;
      };
      for (const PlanRow &row : layer_plan()) {
        if (layer < row.first || layer > row.last) continue;
        const std::string name = spell(row.name);
        std::vector<std::string> inputs;
        for (const char *in : row.in)
          if (in) inputs.push_back(spell(in));
        switch (row.part) {
        case Part::Basis: {
          const size_t at = locate(spbf, "spbf_names", name);
          if (at != (size_t) layer - 1) f.reject("spbf_names", "must list the layers in the order A1, A2, A3");
          const Spbf &s = spbf[at];
          if (layer == 1) {
            if (s.equivariant) f.reject(name + "_equivariant", "is 1, expected 0: the first layer has no message to gather");
            made[name] = {nlm(), s.n_rad_max};
          } else {
            if (!s.equivariant) f.reject(name + "_equivariant", "is 0, expected 1: the layer gathers the message of the layer before");
            const std::string message = "eq" + std::to_string(layer - 1) + "_norm";
            same(name + "_n_lm_ind", s.n_lm_ind, made.at(message).functions, "the message " + message);
            same(name + "_n_rad_max", s.n_rad_max, made.at(message).channels, "the message " + message);
            made[name] = {s.nfunc, s.n_rad_max};
          }
          break;
        }
        case Part::Project: {
          const Reduce &r = reduce[locate(reduce, "reduce_names", name)];
          std::multiset<std::string> have, want(inputs.begin(), inputs.end());
          for (const Instr &in : r.instr) have.insert(in.name);
          if (have != want) f.reject(name + "_instruction_names", "must name exactly the inputs the architecture gives " + name);
          for (const Instr &in : r.instr) {
            const Extent2 src = made.at(in.name);
            same(name + "_n_in_" + in.name, in.n_in, src.channels, "the channel width of " + in.name);
            for (size_t q = 0; q < in.collect_ind.size(); q++)
              if (in.collect_ind[q] >= src.functions)
                f.reject(name + "_collect_ind_" + in.name, "[" + std::to_string(q) + "] = " + std::to_string(in.collect_ind[q]) + " points outside the " +
                                                                 std::to_string(src.functions) + " functions of " + in.name);
          }
          made[name] = {r.nfo(), r.n_out};
          break;
        }
        case Part::Couple: {
          const Cpl &c = prod[locate(prod, "prod_names", name)];
          const Extent2 l = made.at(inputs[0]), r = made.at(inputs[1]);
          same(name + "_group_left", (long) c.group_left.size(), l.functions, "the function count of " + inputs[0]);
          same(name + "_n_left", c.n_left, l.channels, "the channel width of " + inputs[0]);
          same(name + "_group_right", (long) c.group_right.size(), r.functions, "the function count of " + inputs[1]);
          same(name + "_n_right", c.n_right, r.channels, "the channel width of " + inputs[1]);
          made[name] = {c.nfunc, c.rank};
          break;
        }
        case Part::MixRight: {
          const Fc &c = fc[locate(fc, "fc_names", name)];
          const Extent2 l = made.at(inputs[0]), r = made.at(inputs[1]);
          same("fc_" + name + "_w_tile_left", c.n_funcs_left, l.functions, "the function count of " + inputs[0]);
          same("fc_" + name + "_n_out", c.n_out, l.channels, "the channel width of " + inputs[0]);
          same("fc_" + name + "_w_right", c.n_in_right, r.channels, "the channel width of " + inputs[1]);
          for (size_t q = 0; q < c.collect_from.size(); q++)
            if (c.collect_from[q] >= r.functions)
              f.reject("fc_" + name + "_collect_from", "[" + std::to_string(q) + "] = " + std::to_string(c.collect_from[q]) + " points outside the " +
                                                           std::to_string(r.functions) + " functions of " + inputs[1]);
          made[name] = {c.n_funcs_left, c.n_out};
          break;
        }
        case Part::MessageNorm: {
          const EqNorm &e = eqnorm[locate(eqnorm, "eqnorm_names", name)];
          const Extent2 src = made.at(inputs[0]);
          same(name + "_degree_weights", e.M, src.functions, "the function count of " + inputs[0]);
          same(name + "_affine_weight", e.n_out, src.channels, "the channel width of " + inputs[0]);
          made[name] = {e.M, e.n_out};
          break;
        }
        case Part::DensityNorm: {
          const RmsNorm &n = rmsnorm[locate(rmsnorm, "rmsnorm_names", name)];
          const Extent2 src = made.at(inputs[0]);
          same(name + "_n_out", n.n_out, src.channels, "the channel width of " + inputs[0]);
          made[name] = {src.functions, n.n_out};
          break;
        }
        }
      }
    }
    auto nothing_else = [&](const auto &inventory, const char *list) {
      for (const auto &x : inventory)
        if (!visited.count(std::string(list) + "/" + x.name)) f.reject(list, "lists '" + x.name + "', which the three-layer architecture does not contain");
    };
    nothing_else(spbf, "spbf_names");
    nothing_else(prod, "prod_names");
    nothing_else(reduce, "reduce_names");
    nothing_else(fc, "fc_names");
    nothing_else(eqnorm, "eqnorm_names");
    nothing_else(rmsnorm, "rmsnorm_names");
    const long width = made.at("rho1_norm").channels;
    for (const char *rho : {"rho2_norm", "rho3_norm"}) same(std::string(rho) + "_n_out", made.at(rho).channels, width, "rho1_norm");
    return width;
  }
};

}    // namespace grhip
