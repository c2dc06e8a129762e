// Prints the HIP source that the engine generates for one Clebsch-Gordan product, for tests that compile it for the host
// and compare it with a direct evaluation of the term list (host code only; no device is touched).
//
//   jit_source blocked|plain <terms.txt> <channels> <64|32>
//
// terms.txt: "nterms nfl nfr nout", the group of every left function, of every right function, then "l r o c" per term.
#include "../grace_runtime_amd/csrc/jit_prod.hpp"

#include <fstream>
#include <iostream>

int main(int argc, char **argv)
{
  if (argc != 5) {
    std::cerr << "usage: jit_source blocked|plain terms.txt channels 64|32\n";
    return 2;
  }
  std::ifstream f(argv[2]);
  int nt = 0, nfl = 0, nfr = 0, nout = 0;
  if (!(f >> nt >> nfl >> nfr >> nout) || nt < 0 || nt > 10000000 || nfl < 0 || nfl > 100000 || nfr < 0 || nfr > 100000) {
    std::cerr << "cannot read " << argv[2] << "\n";
    return 2;
  }
  std::vector<int> gl(nfl), gr(nfr);
  for (auto &x : gl) f >> x;
  for (auto &x : gr) f >> x;
  std::vector<grhip::ProdTerm> t(nt);
  for (auto &x : t) f >> x.l >> x.r >> x.o >> x.c;
  if (!f) {
    std::cerr << "short file " << argv[2] << "\n";
    return 2;
  }
  const int C = std::atoi(argv[3]);
  const bool f32 = std::string(argv[4]) == "32";
  const std::string src = std::string(argv[1]) == "blocked" ? grhip::jit_detail::generate_blocked(t, gl, gr, nfl, nfr, nout, C, f32)
                                                            : grhip::jit_detail::generate(t, nfl, nfr, nout, false, C, f32);
  if (src.empty()) {
    std::cerr << "no block structure\n";
    return 1;
  }
  std::cout << src;
  return 0;
}
