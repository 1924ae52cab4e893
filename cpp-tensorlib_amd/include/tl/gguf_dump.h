// A canonical text rendering of a parsed GGUF file: header, every metadata value (keys
// sorted, floats as hex so nothing is rounded) and the tensor directory with a CRC-32 of
// each tensor's bytes. Two readers that agree on this text agree on everything a loader
// can observe. Generic over the reader type: it touches only the surface the
// reference's reader and tl/gguf.h share (version, alignment, metadata, tensors).
#pragma once

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <string>
#include <vector>

namespace tl {
namespace gguf_dump {

inline uint32_t crc32(const void* data, size_t n) {
  static uint32_t table[256];
  static bool built = false;
  if (!built) {
    for (uint32_t i = 0; i < 256; i++) {
      uint32_t c = i;
      for (int k = 0; k < 8; k++) c = (c & 1u) ? 0xEDB88320u ^ (c >> 1) : c >> 1;
      table[i] = c;
    }
    built = true;
  }
  uint32_t c = 0xFFFFFFFFu;
  const uint8_t* p = static_cast<const uint8_t*>(data);
  for (size_t i = 0; i < n; i++) c = table[(c ^ p[i]) & 0xFFu] ^ (c >> 8);
  return c ^ 0xFFFFFFFFu;
}

inline void quoted(std::string& out, const std::string& s) {
  char buf[8];
  out += std::to_string(s.size()) + ":\"";
  for (unsigned char ch : s) {
    if (ch >= 0x20 && ch < 0x7f && ch != '"' && ch != '\\') out += (char)ch;
    else { std::snprintf(buf, sizeof buf, "\\x%02x", ch); out += buf; }
  }
  out += '"';
}

template <class Value>
void value(std::string& out, const Value& v) {
  char buf[64];
  const uint32_t t = static_cast<uint32_t>(v.type);
  out += "t" + std::to_string(t) + "=";
  switch (t) {
    case 0: case 2: case 4: case 7: case 10: out += std::to_string(v.u); break;       // unsigned, bool
    case 1: case 3: case 5: case 11: out += std::to_string(v.i); break;               // signed
    case 6: case 12: std::snprintf(buf, sizeof buf, "%a", v.f); out += buf; break;    // floats
    case 8: quoted(out, v.s); break;
    case 9:
      out += "[e" + std::to_string(static_cast<uint32_t>(v.arr_elem_type)) + " n" + std::to_string(v.arr.size());
      for (const auto& e : v.arr) { out += ' '; value(out, e); }
      out += ']';
      break;
    default: out += "?";
  }
}

template <class Model>
std::string render(const Model& m) {
  std::string out = "gguf v" + std::to_string(m.version()) + " alignment=" + std::to_string(m.alignment()) +
                    " tensors=" + std::to_string(m.tensor_count()) + " kv=" + std::to_string(m.metadata().size()) + "\n";
  std::vector<std::string> keys;
  for (const auto& kv : m.metadata()) keys.push_back(kv.first);
  std::sort(keys.begin(), keys.end());
  for (const auto& k : keys) {
    out += "kv ";
    quoted(out, k);
    out += ' ';
    value(out, m.kv(k));
    out += '\n';
  }
  char buf[32];
  for (const auto& t : m.tensors()) {
    out += "tensor ";
    quoted(out, t.name);
    out += " type=" + std::to_string(static_cast<uint32_t>(t.type)) + " dims=[";
    for (size_t i = 0; i < t.dims.size(); i++) out += (i ? "," : "") + std::to_string(t.dims[i]);
    out += "] rel_offset=" + std::to_string(t.rel_offset) + " nbytes=" + std::to_string(t.nbytes);
    std::snprintf(buf, sizeof buf, " crc=%08x", crc32(t.data, (size_t)t.nbytes));
    out += buf;
    out += " lookup=" + std::string(m.tensor(t.name) ? "ok" : "missing") + "\n";
  }
  return out;
}

}  // namespace gguf_dump
}  // namespace tl
