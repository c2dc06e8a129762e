// Validated access to the members of a model file.  A loader states, per key, what it needs: the kind of value, the
// shape as a list of extents (a number, or a slot that takes whatever extent the file has so later requests can be
// checked against it), and for index arrays the range the entries must stay in.  Every request is checked when it is
// made, so a loader never holds an unchecked array.  The rules are those of the kokkos.npz format as the reference reads
// it (libgrace/src/npz3.h:60-330): floats may be stored as float32 / float64 / any integer type, integers as any integer
// type, flags also as bool; NaN / Inf, column-major matrices and values outside the stated range are refused.
#pragma once

#include "npz.hpp"

#include <algorithm>
#include <climits>
#include <cmath>
#include <initializer_list>
#include <string>
#include <vector>

namespace grhip {

constexpr long kSizeLimit = 1 << 16;    // no size, count or extent read from a file may exceed this
constexpr long kDegreeLimit = 255;      // largest angular momentum
constexpr long kEnvelopeLimit = 46339;  // largest envelope order p: (p + 1)(p + 2) stays inside int

// One extent of a requested shape.
struct Ext {
  long fixed = -1;        // the extent the file must have ...
  long *slot = nullptr;   // ... or where to put the extent it has (1 .. kSizeLimit)
  Ext(long v) : fixed(v) {}
  Ext(int v) : fixed(v) {}
  static Ext any(long &into)
  {
    Ext e(0L);
    e.fixed = -1;
    e.slot = &into;
    return e;
  }
};
// `total` values in any arrangement (the exporter pads some vectors with unit dimensions)
struct Flat {
  long total;
};

class FileReader {
 public:
  FileReader(const Npz &members, std::string family) : z_(members), family_(std::move(family)) {}

  const std::string &family() const { return family_; }
  bool present(const std::string &key) const { return z_.count(key) != 0; }
  const Npz &members() const { return z_; }

  [[noreturn]] void reject(const std::string &key, const std::string &complaint) const
  {
    throw Error(family_ + " model file: '" + key + "' " + complaint);
  }

  // ---- scalars ------------------------------------------------------------------------------------------------
  // integer in lo .. hi; a key the file does not have takes `fallback`, or is an error when there is none
  long whole(const std::string &key, long lo, long hi) const
  {
    if (!present(key)) reject(key, "is absent; the format requires it");
    return whole_or(key, lo, hi, lo);
  }
  long whole_or(const std::string &key, long lo, long hi, long fallback) const
  {
    const NpyArray *a = single(key);
    const long v = a ? integer_at(*a, 0, key) : fallback;
    if (v < lo || v > hi) reject(key, "= " + std::to_string(v) + " lies outside " + std::to_string(lo) + " .. " + std::to_string(hi));
    return v;
  }
  bool flag_or(const std::string &key, bool fallback) const { return whole_or(key, 0, 1, fallback ? 1 : 0) != 0; }
  double real_or(const std::string &key, double fallback) const
  {
    const NpyArray *a = single(key);
    return a ? real_at(*a, 0, key) : fallback;
  }
  // a distance: positive
  double length_or(const std::string &key, double fallback) const
  {
    const double v = real_or(key, fallback);
    if (!(v > 0.0)) reject(key, "= " + std::to_string(v) + " is not a positive cutoff distance");
    return v;
  }
  // the file must agree with what the engine implements or with another key
  void must_be(const std::string &key, long fallback, long wanted, const std::string &because) const
  {
    const long v = whole_or(key, LONG_MIN / 2, LONG_MAX / 2, fallback);
    if (v != wanted) reject(key, "= " + std::to_string(v) + " but " + std::to_string(wanted) + " is needed: " + because);
  }

  // ---- arrays -------------------------------------------------------------------------------------------------
  std::vector<double> reals(const std::string &key, std::initializer_list<Ext> shape) const
  {
    const NpyArray &a = need(key);
    fit(a, key, shape);
    return all_reals(a, key);
  }
  std::vector<double> reals(const std::string &key, Flat n) const
  {
    const NpyArray &a = need(key);
    if ((long) a.count != n.total) reject(key, "holds " + std::to_string(a.count) + " values, expected " + std::to_string(n.total));
    return all_reals(a, key);
  }
  // the same for a key that may be absent: then `total` copies of `fill`
  std::vector<double> reals_or(const std::string &key, Flat n, double fill) const
  {
    if (!present(key)) return std::vector<double>((size_t) n.total, fill);
    return reals(key, n);
  }
  // non-negative distances [rows][cols], or empty when absent
  std::vector<double> distances_or_none(const std::string &key, long rows, long cols) const
  {
    if (!present(key)) return {};
    std::vector<double> v = reals(key, {rows, cols});
    for (size_t q = 0; q < v.size(); q++)
      if (v[q] < 0.0) reject(key, "holds the negative cutoff " + std::to_string(v[q]) + " at position " + std::to_string(q));
    return v;
  }
  // integers that index something of `range` entries
  std::vector<int> indices(const std::string &key, std::initializer_list<Ext> shape, long range) const
  {
    const NpyArray &a = need(key);
    fit(a, key, shape);
    std::vector<int> v(a.count);
    for (size_t q = 0; q < v.size(); q++) {
      const long x = integer_at(a, q, key);
      if (x < 0 || x >= range)
        reject(key, "[" + std::to_string(q) + "] = " + std::to_string(x) + " points outside the " + std::to_string(range) + " entries it indexes");
      v[q] = (int) x;
    }
    return v;
  }
  // byte-string names; a key the file does not have gives none
  std::vector<std::string> labels(const std::string &key) const
  {
    std::vector<std::string> out;
    const NpyArray *a = look(key);
    if (!a) return out;
    if (a->kind != 'S' || a->shape.size() > 1) reject(key, "is stored as '" + a->descr + "'; a list of byte strings is needed");
    const size_t n = a->shape.empty() ? 0 : a->shape[0];
    for (size_t i = 0; i < n; i++) {
      const char *s = (const char *) a->raw.data() + i * a->word;
      size_t len = a->word;
      while (len > 0 && s[len - 1] == '\0') len--;
      out.emplace_back(s, len);
    }
    return out;
  }
  // extents of a stored array without reading it (rank must match; every extent 1 .. kSizeLimit)
  std::vector<long> extents(const std::string &key, size_t rank) const
  {
    const NpyArray &a = need(key);
    if (a.shape.size() != rank) reject(key, "is stored as " + layout(a) + "; " + std::to_string(rank) + " dimensions are needed");
    std::vector<long> d;
    for (size_t x : a.shape) {
      if (x < 1 || x > (size_t) kSizeLimit) reject(key, "is stored as " + layout(a) + "; extents must lie in 1 .. " + std::to_string(kSizeLimit));
      d.push_back((long) x);
    }
    return d;
  }

 private:
  const Npz &z_;
  std::string family_;

  static std::string layout(const NpyArray &a)
  {
    if (a.shape.empty()) return "a scalar";
    std::string s;
    for (size_t i = 0; i < a.shape.size(); i++) s += (i ? " x " : "") + std::to_string(a.shape[i]);
    return s;
  }
  const NpyArray *look(const std::string &key) const
  {
    auto it = z_.find(key);
    if (it == z_.end()) return nullptr;
    const NpyArray &a = it->second;
    size_t wide = 0;
    for (size_t d : a.shape) wide += d > 1 ? 1 : 0;
    if (a.fortran && wide > 1) reject(key, "is laid out column-major (Fortran order); save it row-major");
    return &a;
  }
  const NpyArray &need(const std::string &key) const
  {
    const NpyArray *a = look(key);
    if (!a || a->count == 0) reject(key, "is absent or empty; the model cannot be evaluated without it");
    return *a;
  }
  const NpyArray *single(const std::string &key) const
  {
    const NpyArray *a = look(key);
    if (a && a->count != 1) reject(key, "holds " + std::to_string(a->count) + " values where a single number is needed");
    return a;
  }
  // The stored shape against the requested one.  Exporters pad some arrays with unit dimensions (a vector stored as n x 1):
  // when the ranks differ, extents of 1 are dropped on both sides before the comparison.
  void fit(const NpyArray &a, const std::string &key, std::initializer_list<Ext> shape) const
  {
    std::vector<size_t> have(a.shape);
    std::vector<Ext> want(shape);
    if (have.size() != want.size()) {
      have.erase(std::remove(have.begin(), have.end(), (size_t) 1), have.end());
      want.erase(std::remove_if(want.begin(), want.end(), [](const Ext &e) { return !e.slot && e.fixed == 1; }), want.end());
    }
    bool ok = have.size() == want.size();
    for (size_t k = 0; ok && k < want.size(); k++)
      ok = want[k].slot ? (have[k] >= 1 && have[k] <= (size_t) kSizeLimit) : (want[k].fixed >= 0 && have[k] == (size_t) want[k].fixed);
    if (!ok) {
      std::string text;
      for (const Ext &e : shape) text += (text.empty() ? "" : " x ") + (e.slot ? std::string("any") : std::to_string(e.fixed));
      if (shape.size() == 1 && shape.begin()->fixed >= 0)
        reject(key, "holds " + std::to_string(a.count) + " values, expected " + text);
      reject(key, "is stored as " + layout(a) + " where " + text + " is needed");
    }
    for (size_t k = 0; k < want.size(); k++)
      if (want[k].slot) *want[k].slot = (long) have[k];
  }
  static bool integral(const NpyArray &a)
  {
    return (a.kind == 'i' || a.kind == 'u') && (a.word == 1 || a.word == 2 || a.word == 4 || a.word == 8);
  }
  long integer_at(const NpyArray &a, size_t q, const std::string &key) const
  {
    if (a.kind == 'b' && a.word == 1) return a.as<uint8_t>()[q] ? 1 : 0;
    if (!integral(a)) reject(key, "is stored as '" + a.descr + "'; an integer type is needed");
    long long v = 0;
    if (a.kind == 'i') v = a.word == 1 ? a.as<int8_t>()[q] : a.word == 2 ? a.as<int16_t>()[q] : a.word == 4 ? a.as<int32_t>()[q] : a.as<int64_t>()[q];
    else {
      const unsigned long long u =
          a.word == 1 ? a.as<uint8_t>()[q] : a.word == 2 ? a.as<uint16_t>()[q] : a.word == 4 ? a.as<uint32_t>()[q] : a.as<uint64_t>()[q];
      if (u > (unsigned long long) INT_MAX) reject(key, "[" + std::to_string(q) + "] does not fit a 32-bit integer");
      v = (long long) u;
    }
    if (v < INT_MIN || v > INT_MAX) reject(key, "[" + std::to_string(q) + "] does not fit a 32-bit integer");
    return (long) v;
  }
  double real_at(const NpyArray &a, size_t q, const std::string &key) const
  {
    double v;
    if (a.kind == 'f' && a.word == 8) v = a.as<double>()[q];
    else if (a.kind == 'f' && a.word == 4) v = a.as<float>()[q];
    else if (integral(a)) v = (double) integer_at(a, q, key);
    else reject(key, "is stored as '" + a.descr + "'; float32, float64 or an integer type is needed");
    if (!std::isfinite(v)) reject(key, "[" + std::to_string(q) + "] is not a finite number (NaN or Inf)");
    return v;
  }
  std::vector<double> all_reals(const NpyArray &a, const std::string &key) const
  {
    std::vector<double> v(a.count);
    for (size_t q = 0; q < v.size(); q++) v[q] = real_at(a, q, key);
    return v;
  }
};

// 1 + the largest entry: how many things an index array addresses
inline long addressed(const std::vector<int> &idx)
{
  long m = 0;
  for (int x : idx) m = std::max<long>(m, (long) x + 1);
  return m;
}

}    // namespace grhip
