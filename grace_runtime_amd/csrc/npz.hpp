// Reader for uncompressed .npz archives (numpy.savez) and typed accessors with the validation rules of the model
// loaders.  Semantics follow the reference's private helpers (libgrace/src/npz3.h:22-330): every value is converted
// by its stored dtype or rejected, Fortran-ordered multi-dimensional arrays, compressed members, big-endian data
// and NaN/Inf are errors, a missing required array is an error naming it.
#pragma once

#include <climits>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <map>
#include <stdexcept>
#include <string>
#include <vector>

namespace grhip {

// errors the C ABI reports as "invalid input" (the Python layer raises ValueError) and as "runtime"
struct Error : std::runtime_error {
  using std::runtime_error::runtime_error;
};
struct InvalidArgument : std::invalid_argument {
  using std::invalid_argument::invalid_argument;
};

struct NpyArray {
  std::string descr;              // e.g. "<f8", "|S8"
  char kind = 0;                  // 'f', 'i', 'u', 'b', 'S'
  size_t word = 0;                // bytes per element
  bool fortran = false;
  std::vector<size_t> shape;
  size_t count = 0;
  std::vector<unsigned char> raw;
  template<class T> const T *as() const { return reinterpret_cast<const T *>(raw.data()); }
};
using Npz = std::map<std::string, NpyArray>;

namespace detail {
inline uint16_t rd16(const unsigned char *p) { return (uint16_t) (p[0] | (p[1] << 8)); }
inline uint32_t rd32(const unsigned char *p) { return (uint32_t) p[0] | ((uint32_t) p[1] << 8) | ((uint32_t) p[2] << 16) | ((uint32_t) p[3] << 24); }
inline uint64_t rd64(const unsigned char *p) { return (uint64_t) rd32(p) | ((uint64_t) rd32(p + 4) << 32); }

// one .npy member (header + data) -> NpyArray
inline NpyArray parse_npy(const unsigned char *p, size_t len, const std::string &name)
{
  auto bad = [&](const std::string &w) { return Error("npz member '" + name + "': " + w); };
  if (len < 10 || std::memcmp(p, "\x93NUMPY", 6) != 0) throw bad("not a .npy array");
  const int major = p[6];
  size_t hlen, hoff;
  if (major == 1) { hlen = rd16(p + 8); hoff = 10; }
  else if (major == 2 || major == 3) { if (len < 12) throw bad("truncated header"); hlen = rd32(p + 8); hoff = 12; }
  else throw bad("unknown .npy version");
  if (hoff + hlen > len) throw bad("truncated header");
  const std::string h((const char *) p + hoff, hlen);
  NpyArray a;
  auto find_val = [&](const char *key) -> size_t {
    const size_t k = h.find(std::string("'") + key + "'");
    if (k == std::string::npos) throw bad(std::string("header lacks ") + key);
    const size_t c = h.find(':', k);
    if (c == std::string::npos) throw bad("malformed header");
    size_t v = c + 1;
    while (v < h.size() && h[v] == ' ') v++;
    return v;
  };
  {
    size_t v = find_val("descr");
    if (h[v] != '\'') throw bad("structured dtypes are not supported");
    const size_t e = h.find('\'', v + 1);
    a.descr = h.substr(v + 1, e - v - 1);
  }
  a.fortran = h.compare(find_val("fortran_order"), 4, "True") == 0;
  {
    size_t v = find_val("shape");
    if (h[v] != '(') throw bad("malformed shape");
    const size_t e = h.find(')', v);
    std::string s = h.substr(v + 1, e - v - 1);
    size_t q = 0;
    while (q < s.size()) {
      while (q < s.size() && (s[q] == ' ' || s[q] == ',')) q++;
      if (q >= s.size()) break;
      size_t d = 0;
      bool any = false;
      while (q < s.size() && s[q] >= '0' && s[q] <= '9') { d = d * 10 + (size_t) (s[q] - '0'); q++; any = true; }
      if (!any) throw bad("malformed shape");
      a.shape.push_back(d);
    }
  }
  if (a.descr.size() < 3) throw bad("unsupported dtype '" + a.descr + "'");
  const char order = a.descr[0];
  a.kind = a.descr[1];
  a.word = (size_t) std::strtoul(a.descr.c_str() + 2, nullptr, 10);
  if (order == '>' && a.word > 1) throw bad("big-endian data is not supported");
  if (!(a.kind == 'f' || a.kind == 'i' || a.kind == 'u' || a.kind == 'b' || a.kind == 'S') || a.word == 0)
    throw bad("unsupported dtype '" + a.descr + "'");
  a.count = 1;
  for (size_t d : a.shape) {
    if (d != 0 && a.count > SIZE_MAX / d) throw bad("shape overflows");
    a.count *= d;
  }
  const size_t need = a.count * a.word;
  if (hoff + hlen + need > len) throw bad("truncated data");
  a.raw.assign(p + hoff + hlen, p + hoff + hlen + need);
  return a;
}
}    // namespace detail

// all members of an uncompressed .npz (ZIP, stored entries, ZIP64 sizes accepted)
inline Npz npz_load(const std::string &path)
{
  using namespace detail;
  FILE *f = std::fopen(path.c_str(), "rb");
  if (!f) throw Error("cannot read the model file " + path + ": cannot open");
  std::vector<unsigned char> buf;
  {
    std::fseek(f, 0, SEEK_END);
    const long sz = std::ftell(f);
    std::fseek(f, 0, SEEK_SET);
    if (sz < 22) { std::fclose(f); throw Error("cannot read the model file " + path + ": not a zip archive"); }
    buf.resize((size_t) sz);
    const size_t got = std::fread(buf.data(), 1, buf.size(), f);
    std::fclose(f);
    if (got != buf.size()) throw Error("cannot read the model file " + path + ": short read");
  }
  auto fail = [&](const std::string &w) { return Error("cannot read the model file " + path + ": " + w); };
  const size_t n = buf.size();
  // end of central directory (search backwards over a possible comment)
  size_t eocd = std::string::npos;
  for (size_t k = n - 22;; k--) {
    if (rd32(&buf[k]) == 0x06054b50u) { eocd = k; break; }
    if (k == 0 || n - k > 22 + 65535) break;
  }
  if (eocd == std::string::npos) throw fail("not a zip archive");
  uint64_t nent = rd16(&buf[eocd + 10]), cdoff = rd32(&buf[eocd + 16]);
  if (nent == 0xFFFF || cdoff == 0xFFFFFFFFu) {    // ZIP64: locator precedes the EOCD
    if (eocd < 20 || rd32(&buf[eocd - 20]) != 0x07064b50u) throw fail("broken zip64 locator");
    const uint64_t e64 = rd64(&buf[eocd - 20 + 8]);
    if (e64 + 56 > n || rd32(&buf[e64]) != 0x06064b50u) throw fail("broken zip64 record");
    nent = rd64(&buf[e64 + 32]);
    cdoff = rd64(&buf[e64 + 48]);
  }
  Npz out;
  size_t p = (size_t) cdoff;
  for (uint64_t e = 0; e < nent; e++) {
    if (p + 46 > n || rd32(&buf[p]) != 0x02014b50u) throw fail("broken central directory");
    const uint16_t method = rd16(&buf[p + 10]);
    uint64_t csize = rd32(&buf[p + 20]), usize = rd32(&buf[p + 24]);
    const uint16_t nlen = rd16(&buf[p + 28]), xlen = rd16(&buf[p + 30]), clen = rd16(&buf[p + 32]);
    uint64_t lho = rd32(&buf[p + 42]);
    if (p + 46 + nlen + xlen + clen > n) throw fail("broken central directory");
    std::string name((const char *) &buf[p + 46], nlen);
    // zip64 extra field: the values that overflowed, in the order usize, csize, offset
    size_t x = p + 46 + nlen;
    const size_t xe = x + xlen;
    while (x + 4 <= xe) {
      const uint16_t id = rd16(&buf[x]), sz = rd16(&buf[x + 2]);
      if (id == 0x0001) {
        size_t q = x + 4;
        if (usize == 0xFFFFFFFFu && q + 8 <= xe) { usize = rd64(&buf[q]); q += 8; }
        if (csize == 0xFFFFFFFFu && q + 8 <= xe) { csize = rd64(&buf[q]); q += 8; }
        if (lho == 0xFFFFFFFFu && q + 8 <= xe) { lho = rd64(&buf[q]); q += 8; }
      }
      x += 4 + sz;
    }
    p += 46 + nlen + xlen + clen;
    if (method != 0)
      throw fail("member '" + name + "' is compressed (np.savez_compressed); save the model with np.savez");
    if (lho + 30 > n || rd32(&buf[lho]) != 0x04034b50u) throw fail("broken local header of '" + name + "'");
    const size_t data = (size_t) lho + 30 + rd16(&buf[lho + 26]) + rd16(&buf[lho + 28]);
    if (data + csize > n || csize != usize) throw fail("member '" + name + "' is truncated");
    if (name.size() > 4 && name.compare(name.size() - 4, 4, ".npy") == 0) name.resize(name.size() - 4);
    out[name] = parse_npy(&buf[data], (size_t) usize, name);
  }
  return out;
}

// ---------------------------------------------------------------------------------------------------------------
// typed access
// ---------------------------------------------------------------------------------------------------------------
constexpr int kMaxDim = 1 << 16;    // any size or count read from a file
constexpr int kMaxL = 255;
constexpr int kMaxP = 46339;

inline Error bad_array(const std::string &key, const std::string &what)
{
  return Error("model array '" + key + "' " + what + "; re-export the model");
}

struct NpzView {
  const Npz &z;
  explicit NpzView(const Npz &z_) : z(z_) {}

  bool has(const std::string &k) const { return z.count(k) != 0; }

  const NpyArray *find(const std::string &key) const
  {
    auto it = z.find(key);
    if (it == z.end()) return nullptr;
    const NpyArray &a = it->second;
    if (a.fortran) {
      int dims = 0;
      for (size_t d : a.shape) dims += d > 1;
      if (dims > 1) throw Error("model array '" + key + "' is stored in Fortran order; re-export it in C order");
    }
    return &a;
  }

  static bool int_at(const NpyArray &a, size_t q, int64_t &v)
  {
    const bool u = a.kind == 'u';
    switch (a.word) {
    case 1: v = u ? (int64_t) a.as<uint8_t>()[q] : (int64_t) a.as<int8_t>()[q]; return true;
    case 2: v = u ? (int64_t) a.as<uint16_t>()[q] : (int64_t) a.as<int16_t>()[q]; return true;
    case 4: v = u ? (int64_t) a.as<uint32_t>()[q] : (int64_t) a.as<int32_t>()[q]; return true;
    case 8:
      if (!u) { v = a.as<int64_t>()[q]; return true; }
      v = (int64_t) a.as<uint64_t>()[q];
      return a.as<uint64_t>()[q] <= (uint64_t) INT64_MAX;
    default: return false;
    }
  }
  static bool is_int(const NpyArray &a) { return (a.kind == 'i' || a.kind == 'u') && (a.word == 1 || a.word == 2 || a.word == 4 || a.word == 8); }

  std::vector<double> doubles(const std::string &key) const
  {
    const NpyArray *a = find(key);
    if (!a) return {};
    std::vector<double> v(a->count);
    auto put = [&](size_t q, double x) {
      if (!std::isfinite(x)) throw bad_array(key, "has a non-finite value (NaN / Inf) at " + std::to_string(q));
      v[q] = x;
    };
    if (a->kind == 'f' && a->word == 4) for (size_t q = 0; q < v.size(); q++) put(q, a->as<float>()[q]);
    else if (a->kind == 'f' && a->word == 8) for (size_t q = 0; q < v.size(); q++) put(q, a->as<double>()[q]);
    else if (is_int(*a)) {
      for (size_t q = 0; q < v.size(); q++) {
        int64_t x;
        if (!int_at(*a, q, x)) throw bad_array(key, "has dtype '" + a->descr + "', expected a float32 or float64 array");
        v[q] = (double) x;
      }
    } else throw bad_array(key, "has dtype '" + a->descr + "', expected a float32 or float64 array");
    return v;
  }

  std::vector<int> ints(const std::string &key) const
  {
    const NpyArray *a = find(key);
    if (!a) return {};
    std::vector<int> v(a->count);
    if (a->kind == 'b' && a->word == 1) {
      for (size_t q = 0; q < v.size(); q++) v[q] = a->as<uint8_t>()[q] != 0;
      return v;
    }
    if (!is_int(*a)) throw bad_array(key, "has dtype '" + a->descr + "', expected an integer array");
    for (size_t q = 0; q < v.size(); q++) {
      int64_t x;
      if (!int_at(*a, q, x) || x < INT_MIN || x > INT_MAX) throw bad_array(key, "has a value outside the range of int");
      v[q] = (int) x;
    }
    return v;
  }

  void require_scalar(const std::string &key) const
  {
    auto it = z.find(key);
    if (it != z.end() && it->second.count != 1)
      throw bad_array(key, "has " + std::to_string(it->second.count) + " values, expected one");
  }
  int int_scalar(const std::string &key, int def = 0) const
  {
    require_scalar(key);
    auto v = ints(key);
    return v.empty() ? def : v[0];
  }
  double double_scalar(const std::string &key, double def = 0.0) const
  {
    require_scalar(key);
    auto v = doubles(key);
    return v.empty() ? def : v[0];
  }
  // an int scalar in [lo, hi]; def when absent (a def outside [lo, hi]: the key is required)
  int int_in(const std::string &key, int def, int lo, int hi) const
  {
    if (!has(key) && (def < lo || def > hi)) throw bad_array(key, "is missing from the .npz file");
    const int v = int_scalar(key, def);
    if (v < lo || v > hi)
      throw bad_array(key, "is " + std::to_string(v) + ", expected a value in [" + std::to_string(lo) + ", " + std::to_string(hi) + "]");
    return v;
  }
  bool flag(const std::string &key, int def) const { return int_in(key, def, 0, 1) != 0; }

  std::vector<double> require_doubles(const std::string &key) const
  {
    auto v = doubles(key);
    if (v.empty())
      throw Error("required weight '" + key + "' missing from the .npz file (an empty load would give zero forces); re-export the model");
    return v;
  }
  std::vector<int> require_ints(const std::string &key) const
  {
    auto v = ints(key);
    if (v.empty()) throw Error("required index array '" + key + "' missing from the .npz file; re-export the model");
    return v;
  }
  std::vector<double> cutoffs(const std::string &key, const char *style) const
  {
    auto v = doubles(key);
    for (double x : v)
      if (x < 0.0) throw Error(std::string(style) + ": invalid cutoff in '" + key + "'");
    return v;
  }
  double cutoff_scalar(const std::string &key, double def, const char *style) const
  {
    require_scalar(key);
    auto v = cutoffs(key, style);
    if (v.empty()) return def;
    if (!(v[0] > 0.0)) throw Error(std::string(style) + ": cutoff '" + key + "' is not positive");
    return v[0];
  }
  std::vector<std::string> names(const std::string &key) const
  {
    std::vector<std::string> out;
    const NpyArray *a = find(key);
    if (!a) return out;
    if (a->kind != 'S' || a->shape.size() > 1) throw bad_array(key, "has dtype '" + a->descr + "', expected a 1-d byte-string array (|S)");
    const size_t n = a->shape.empty() ? 0 : a->shape[0];
    for (size_t i = 0; i < n; i++) {
      std::string s((const char *) a->raw.data() + i * a->word, a->word);
      while (!s.empty() && s.back() == '\0') s.pop_back();
      out.push_back(s);
    }
    return out;
  }
  std::vector<size_t> shape(const std::string &key) const
  {
    auto it = z.find(key);
    return it == z.end() ? std::vector<size_t>{} : it->second.shape;
  }
  static std::string dims_str(const std::vector<size_t> &d)
  {
    std::string o = "(";
    for (size_t i = 0; i < d.size(); i++) o += (i ? ", " : "") + std::to_string(d[i]);
    return o + ")";
  }
  std::vector<size_t> shape_rank(const std::string &key, size_t rank) const
  {
    const auto d = shape(key);
    bool ok = d.size() == rank;
    for (size_t x : d) ok = ok && x >= 1 && x <= (size_t) kMaxDim;
    if (!ok) throw bad_array(key, "has shape " + dims_str(d) + ", expected " + std::to_string(rank) + " dimensions in [1, " + std::to_string(kMaxDim) + "]");
    return d;
  }
  // the stored shape is exactly `want` (an absent key passes)
  void require_shape(const std::string &key, const std::vector<int64_t> &want) const
  {
    const NpyArray *a = find(key);
    if (!a) return;
    bool ok = a->shape.size() == want.size();
    for (size_t i = 0; ok && i < want.size(); i++) ok = want[i] >= 0 && a->shape[i] == (size_t) want[i];
    if (!ok) {
      std::vector<size_t> w;
      std::string ws = "(";
      for (size_t i = 0; i < want.size(); i++) ws += (i ? ", " : "") + std::to_string(want[i]);
      throw bad_array(key, "has shape " + dims_str(a->shape) + ", expected " + ws + ")");
    }
  }
};

template<class V> inline void require_size(const std::string &key, const V &v, size_t n)
{
  if (v.size() != n) throw bad_array(key, "has " + std::to_string(v.size()) + " values, expected " + std::to_string(n));
}
inline void require_eq(const std::string &key, int64_t got, int64_t want, const std::string &why, const char *noun = nullptr)
{
  if (got != want)
    throw bad_array(key, (noun ? "has " + std::to_string(got) + " " + noun : "is " + std::to_string(got)) + ", expected " + std::to_string(want) + " (" + why + ")");
}
inline void require_index(const std::string &key, const std::vector<int> &v, int64_t n)
{
  for (size_t q = 0; q < v.size(); q++)
    if (v[q] < 0 || v[q] >= n)
      throw bad_array(key, "has " + std::to_string(v[q]) + " at " + std::to_string(q) + ", outside [0, " + std::to_string(n) + ")");
}
inline int64_t index_extent(const std::vector<int> &v)
{
  int64_t m = 0;
  for (int x : v) m = std::max<int64_t>(m, (int64_t) x + 1);
  return m;
}

}    // namespace grhip
