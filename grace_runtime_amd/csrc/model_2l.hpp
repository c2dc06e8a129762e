// Host-side container of a GRACE-2L model read from kokkos.npz and its loader.  Keys and consistency rules are the file
// format's, as the reference loader reads it (libgrace/src/model_2l.cpp:28-420, container libgrace/include/grace/
// model_2l.h:22-175); files of max_order 3 (no AAAA / BBBB stage, libgrace/src/max_order3.h) load with those stages absent.
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
  // can the head be evaluated (libgrace/src/model_2l.cpp:466-478, libgrace/src/uq.cpp:8-33)
  void validate_uq() const { uq.require_usable("GRACE-2L", max_order == 4, uq_block_width(I2_red) + uq_block_width(rho_red), 2); }
  double pair_cutoff(int mu_i, int mu_j) const
  {
    if (mu_i < 0 || mu_j < 0) return 0.0;
    return has_bond_specific_cutoff ? bond_cutoff_map[(size_t) mu_i * n_elements + mu_j] : rcut;
  }

  void load(const Npz &z)
  {
    *this = Model2L();
    const FileReader f(z, "GRACE-2L");
    check_declaration(f, "GRACE-2L");

    int *const into[] = {&n_elements, &embedding_size, &lmax, &nradbase, &radial_basis_p, &C1, &CR, &C2, &B_n_funcs, &I1_n_out, &I1_n_funcs, &I_n_funcs, &rho_n_out};
    static const SizeKey sizes[] = {{"n_elements", 1, kSizeLimit, 89},  {"embedding_size", 1, kSizeLimit, 128},       {"lmax", 0, kDegreeLimit, 4},
                                    {"nradbase", 1, kSizeLimit, 10},    {"radial_basis_p", 1, kEnvelopeLimit, 16},    {"mlp_rad_R_n_rad_max", 1, kSizeLimit, 32},
                                    {"mlp_rad_R1_n_rad_max", 1, kSizeLimit, 32}, {"B_n_out", 1, kSizeLimit, 64},      {"B_n_funcs", 1, kSizeLimit, 31},
                                    {"I1_n_out", 1, kSizeLimit, 12},    {"I1_n_funcs", 1, kSizeLimit, 4},             {"I_n_funcs", 1, kSizeLimit, 4},
                                    {"rho_n_out", 2, kSizeLimit, 17}};
    for (size_t k = 0; k < sizeof(sizes) / sizeof(sizes[0]); k++) *into[k] = (int) f.whole_or(sizes[k].key, sizes[k].lo, sizes[k].hi, sizes[k].absent);
    const long harmonics = nlm();

    // ---- both layers carry the fourth-order stage, or neither does
    const bool fourth = f.present("prod_AAAA_n_cg_terms");
    if (fourth != f.present("prod_BBBB_n_cg_terms"))
      f.reject(fourth ? "prod_BBBB_n_cg_terms" : "prod_AAAA_n_cg_terms", "is absent while the other layer has its fourth-order product: both layers must stop at the same order");
    max_order = fourth ? 4 : 3;
    if (!fourth)
      for (const auto &member : z)
        for (const char *piece : {"AAAA", "BBBB", "fc_AA2_", "fc_BB2_"})
          if (member.first.find(piece) != std::string::npos)
            f.reject(member.first, "belongs to the fourth-order stage, which this file otherwise lacks: the stage is incomplete");

    // ---- elements and cutoffs
    element_names = f.labels("element_names");
    if (f.present("element_names") && (long) element_names.size() != n_elements)
      f.reject("element_names", "lists " + std::to_string(element_names.size()) + " elements where n_elements = " + std::to_string(n_elements));
    chem_embedding = f.reals("chem_embedding", {n_elements, embedding_size});
    rcut = f.length_or("rcut", 6.0);
    has_bond_specific_cutoff = f.flag_or("has_bond_specific_cutoff", false);
    bond_cutoff_map = f.distances_or_none("bond_cutoff_map", n_elements, n_elements);
    if (bond_cutoff_map.empty()) bond_cutoff_map.assign((size_t) n_elements * n_elements, rcut);

    // ---- the two radial networks and the species weights of the two gathers
    for (const char *stem : {"mlp_rad_R", "mlp_rad_R1"}) {
      const bool first = std::string(stem) == "mlp_rad_R";
      f.must_be(std::string(stem) + "_has_chem_emb", 0, 0, "radial networks with species inputs belong to GRACE-3L");
      (first ? mlp_R : mlp_R1) =
          read_dense_stack(f, stem, f.whole_or(std::string(stem) + "_n_layers", 1, kSizeLimit, 3), nradbase, (long) (first ? C1 : CR) * nl());
    }
    radial_activation = (int) f.whole_or("radial_activation", 0, 1, 0);
    A_lin_transform_W = f.reals("A_lin_transform_W", {embedding_size, C1});
    A_lin_transform_norm = f.real_or("A_lin_transform_norm", 1.0);
    A_inv_avg_n_neigh = f.real_or("A_inv_avg_n_neigh", 1.0);
    B0_lin_transform_W = f.reals("B0_lin_transform_W", {embedding_size, CR});
    B0_lin_transform_norm = f.real_or("B0_lin_transform_norm", 1.0);
    B0_inv_avg_n_neigh = f.real_or("B0_inv_avg_n_neigh", 1.0);

    // ---- layer 1: chain over A, message I1 -> I, density rho
    long fun1[4] = {harmonics, 0, 0, 0};
    read_chain(f, "A", C1, fourth, fc_A1, prod_AA, fc_AA1, prod_AAA, fc_AA2, prod_AAAA, fun1);
    const char *tags1[4] = {"A", "AA", "AAA", "AAAA"};
    for (int s = 0; s < nsrc(); s++) {
      I1_red[s] = read_reduce(f, "I1", tags1[s], true, I1_n_out, I1_n_funcs, C1, fun1[s]);
      rho_red[s] = read_reduce(f, "rho", tags1[s], true, rho_n_out, 1, C1, fun1[s]);
    }
    f.must_be("I_n_out", 32, CR, "the message is coupled with the layer-2 radial functions, mlp_rad_R1_n_rad_max channels wide");
    I_red = read_reduce(f, "I", "I1", false, CR, I_n_funcs, I1_n_out, I1_n_funcs);

    // ---- layer 2: the neighbour gather coupled with the harmonics (YI), B, chain over B, I2
    {
      const long terms = f.whole("YI_n_cg_terms", 1, kSizeLimit), outputs = f.whole("YI_n_output_funcs", 1, kSizeLimit);
      f.must_be("YI_n_rad_max", 32, CR, "YI carries the layer-2 radial channels mlp_rad_R1_n_rad_max");
      // one (harmonic, message function) pair per term: read the two columns against their own ranges
      const std::vector<int> pairs = f.indices("YI_lr_inds", {terms, 2}, std::max<long>(harmonics, I_n_funcs));
      for (long t = 0; t < terms; t++) {
        const int y = pairs[(size_t) (2 * t)], fn = pairs[(size_t) (2 * t + 1)];
        if (y >= harmonics || fn >= I_n_funcs)
          f.reject("YI_lr_inds", "row " + std::to_string(t) + " = (" + std::to_string(y) + ", " + std::to_string(fn) + ") names a harmonic or a message function "
                                 "that does not exist (" + std::to_string(harmonics) + " harmonics, I_n_funcs = " + std::to_string(I_n_funcs) + ")");
        yi.y.push_back(y);
        yi.i.push_back(fn);
      }
      yi.cg_coeff = f.reals("YI_cg_coeff", {terms});
      yi.m_sum_ind = f.indices("YI_m_sum_ind", {terms}, outputs);
      if (addressed(yi.m_sum_ind) != outputs)
        f.reject("YI_n_output_funcs", "= " + std::to_string(outputs) + " but YI_m_sum_ind addresses " + std::to_string(addressed(yi.m_sum_ind)) + " functions");
      yi.n_terms = (int) terms;
      yi.n_out = (int) outputs;
      yi.inv_avg_n_neigh = f.real_or("YI_inv_avg_n_neigh", 1.0);
    }
    B_red_YI = read_reduce(f, "B", "YI", false, C2, B_n_funcs, CR, yi.n_out);
    B_red_B0 = read_reduce(f, "B", "B0", false, C2, B_n_funcs, CR, harmonics);
    long fun2[4] = {B_n_funcs, 0, 0, 0};
    read_chain(f, "B", C2, fourth, fc_B1, prod_BB, fc_BB1, prod_BBB, fc_BB2, prod_BBBB, fun2);
    f.must_be("I2_n_out", 17, rho_n_out, "the readout adds rho and I2 channel by channel, so I2 has rho_n_out channels");
    const char *tags2[4] = {"B", "BB", "BBB", "BBBB"};
    for (int s = 0; s < nsrc(); s++) I2_red[s] = read_reduce(f, "I2", tags2[s], true, rho_n_out, 1, C2, fun2[s]);

    // ---- readout: two RMS norms, the network on the non-linear channels
    energy_rms_norm = f.flag_or("energy_rms_norm", true);
    if (energy_rms_norm) {
      f.must_be("I_nl_LN_type", 1, 1, "the norm of the non-linear channels leaves the linear channel out");
      f.must_be("I_nl_LN_n_out", 17, rho_n_out, "it normalises the rho_n_out density channels");
      f.must_be("I_0_LN_type", 0, 0, "the norm of the second-layer density covers all its channels");
      f.must_be("I_0_LN_n_out", 17, rho_n_out, "it normalises the I2 channels, as many as rho_n_out");
      I_nl_LN_scale = f.reals("I_nl_LN_scale", Flat{rho_n_out - 1});
      I_0_LN_scale = f.reals("I_0_LN_scale", Flat{rho_n_out});
    } else {
      I_nl_LN_scale.assign((size_t) rho_n_out - 1, 1.0);
      I_0_LN_scale.assign((size_t) rho_n_out, 1.0);
    }
    Model1L::read_readout(f, "GRACE-2L", rho_n_out, 1, energy_mlp, energy_mlp_activation, energy_mlp_ln);
    shift_values = f.reals_or("shift_values", Flat{n_elements}, 0.0);
    output_scale = f.real_or("output_scale", 1.0);
    uq.load(f, n_elements);
  }

 private:
  // FC / product chain over the functions X of one layer (X = "A" or "B", all stages `width` channels wide):
  // X1 = fc_X1(X, X), XX = X1 x X1, XX1 = fc_XX1(XX, X), XXX = XX1 x X1, [XX2 = fc_XX2(XX, X), XXXX = XX2 x XX2].
  // functions[0] holds the functions of X on entry; the counts of XX, XXX, XXXX are filled in.
  static void read_chain(const FileReader &f, const std::string &X, long width, bool fourth, FCWeights &fc1, CGProduct &p2, FCWeights &fc21,
                         CGProduct &p3, FCWeights &fc22, CGProduct &p4, long functions[4])
  {
    const long base = functions[0];
    const std::string XX = X + X;
    fc1 = read_fc(f, "fc_" + X + "1", {base, base, width, width, width});
    p2 = read_product(f, "prod_" + XX, base, base);
    functions[1] = p2.n_out;
    fc21 = read_fc(f, "fc_" + XX + "1", {functions[1], base, width, width, width});
    p3 = read_product(f, "prod_" + XX + X, functions[1], base);
    functions[2] = p3.n_out;
    if (fourth) {
      fc22 = read_fc(f, "fc_" + XX + "2", {functions[1], base, width, width, width});
      p4 = read_product(f, "prod_" + XX + XX, functions[1], functions[1]);
      functions[3] = p4.n_out;
    }
  }
  // Projection `<target>_*_<source>` of a source tensor (`in_width` channels, `in_functions` functions) onto `out_width` channels
  // of `out_functions` output functions; `per_element`: one weight set per element of the central atom.
  ReduceEq read_reduce(const FileReader &f, const std::string &target, const std::string &source, bool per_element, long out_width, long out_functions,
                       long in_width, long in_functions) const
  {
    ReduceEq r;
    long tiles = 0, picked = 0;
    const std::string W = target + "_reduce_" + source + "_W";
    f.must_be(target + "_is_central_atom_type_dependent", per_element, per_element,
              per_element ? "this projection has one weight set per central element" : "this projection has one weight set for all elements");
    f.must_be(target + "_n_in_" + source, in_width, in_width, "it is the channel width of " + source);
    r.W = per_element ? f.reals(W, {n_elements, out_width, in_width, Ext::any(tiles)}) : f.reals(W, {out_width, in_width, Ext::any(tiles)});
    f.must_be(target + "_w_shape_" + source, tiles, tiles, "it counts the weight tiles stored in " + W);
    r.collect_ind = f.indices(target + "_collect_ind_" + source, {Ext::any(picked)}, in_functions);
    r.w_l_tile = f.indices(target + "_w_l_tile_" + source, {picked}, tiles);
    r.total_sum_ind = f.indices(target + "_total_sum_ind_" + source, {picked}, out_functions);
    r.norm = f.real_or(W.substr(0, W.size() - 2) + "_norm", 1.0);
    r.elem = per_element;
    r.n_in = (int) in_width;
    r.w_shape = (int) tiles;
    return r;
  }
};

}    // namespace grhip
