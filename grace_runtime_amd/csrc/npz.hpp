// Reader for uncompressed .npz archives (numpy.savez): the ZIP directory and the .npy members, as raw bytes with their
// dtype and shape.  Compressed members, big-endian data and dtypes other than float / int / bool / byte strings are
// errors (the reference's reader, libgrace/src/npz3.h:22-58, accepts and refuses the same files).  Typed, validated
// access to the members is schema.hpp.
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

}    // namespace grhip
