// Writer of the per-layer output file (safetensors): the container the reference's scheduler stores a quantized
// layer in (SafeTensorsWriter, src/safetensors.cpp:93-137) and the tensors of one QTIP linear as
// write_layer_file lays them out (src/pipeline.cpp:329-340), so that the reference's runtime loader
// (runtime/src/qtip.cpp:216-276) reads the result.  Host code only.
//
// File = u64 little-endian header length, JSON header padded with spaces to a multiple of 8 bytes, tensor bytes
// back to back in name order.  The header is written in the compact form with sorted keys that the reference's
// JSON library produces, so equal inputs give byte-identical files.
#include <algorithm>
#include <cstdio>
#include <cstring>
#include <map>

#include "qtip_internal.hpp"

struct qtip_st_writer {
  struct Entry {
    std::string dtype;
    std::vector<int64_t> shape;
    std::vector<uint8_t> data;
  };
  std::map<std::string, Entry> entries;
};

namespace qtipmi {
namespace {

size_t dtype_bytes(const std::string& d) {
  if (d == "F64" || d == "I64" || d == "U64") return 8;
  if (d == "F32" || d == "I32" || d == "U32") return 4;
  if (d == "F16" || d == "BF16" || d == "I16" || d == "U16") return 2;
  if (d == "F8_E4M3" || d == "F8_E5M2" || d == "I8" || d == "U8" || d == "BOOL") return 1;
  return 0;
}

void json_string(std::string& o, const std::string& s) {
  o.push_back('"');
  for (unsigned char ch : s) {
    switch (ch) {
      case '"': o += "\\\""; break;
      case '\\': o += "\\\\"; break;
      case '\b': o += "\\b"; break;
      case '\f': o += "\\f"; break;
      case '\n': o += "\\n"; break;
      case '\r': o += "\\r"; break;
      case '\t': o += "\\t"; break;
      default:
        if (ch < 0x20) {
          char b[8];
          snprintf(b, sizeof b, "\\u%04x", ch);
          o += b;
        } else {
          o.push_back(char(ch));
        }
    }
  }
  o.push_back('"');
}

}  // namespace

qtip_st_writer* st_new() { return new qtip_st_writer(); }
void st_delete(qtip_st_writer* w) { delete w; }

void st_add(qtip_st_writer* w, const char* name, const char* dtype, const int64_t* shape, int rank, const void* data,
            size_t bytes) {
  QTIP_REQUIRE(w && name && dtype && rank >= 0 && (rank == 0 || shape) && (bytes == 0 || data), "st_add: bad arguments");
  const size_t eb = dtype_bytes(dtype);
  QTIP_REQUIRE(eb != 0, "st_add: unknown dtype '%s'", dtype);
  size_t numel = 1;
  for (int i = 0; i < rank; ++i) {
    QTIP_REQUIRE(shape[i] >= 0, "st_add: negative dimension in '%s'", name);
    numel *= size_t(shape[i]);
  }
  QTIP_REQUIRE(numel * eb == bytes, "st_add: '%s' has %zu bytes, shape x dtype needs %zu", name, bytes, numel * eb);
  QTIP_REQUIRE(std::string(name) != "__metadata__", "st_add: reserved tensor name");
  qtip_st_writer::Entry e;
  e.dtype = dtype;
  e.shape.assign(shape, shape + rank);
  e.data.assign(static_cast<const uint8_t*>(data), static_cast<const uint8_t*>(data) + bytes);
  w->entries[name] = std::move(e);  // a second add under one name replaces the first, as in the reference
}

void st_add_qtip_linear(qtip_st_writer* w, const char* prefix, const qtip_linear_out* out, int m, int n,
                        const uint16_t* tlut_f16) {
  QTIP_REQUIRE(w && prefix && out && tlut_f16, "st_add_qtip_linear: bad arguments");
  QTIP_REQUIRE(m > 0 && n > 0 && m % 16 == 0 && n % 16 == 0 && out->trellis && out->su_bf16 && out->sv,
               "st_add_qtip_linear: incomplete linear (m=%d n=%d)", m, n);
  const std::string b(prefix);
  const int64_t tiles = int64_t(m / 16) * (n / 16);
  const int64_t sh_tr[2] = {tiles, kWords}, sh_n[1] = {n}, sh_m[1] = {m}, sh_lut[2] = {512, 2};
  st_add(w, (b + "trellis").c_str(), "I16", sh_tr, 2, out->trellis, size_t(tiles) * kWords * 2);
  st_add(w, (b + "SU").c_str(), "BF16", sh_n, 1, out->su_bf16, size_t(n) * 2);
  std::vector<float> sv(static_cast<size_t>(m), 0.0f);
  for (int i = 0; i < m; ++i) sv[size_t(i)] = out->sv[i] * out->wscale;  // SV <- SV * Wscale (rcp = 0)
  st_add(w, (b + "SV").c_str(), "F32", sh_m, 1, sv.data(), size_t(m) * 4);
  st_add(w, (b + "tlut").c_str(), "F16", sh_lut, 2, tlut_f16, 512 * 2 * 2);
  const int64_t zero = 0, eight = 8;
  st_add(w, (b + "rcp").c_str(), "I64", nullptr, 0, &zero, 8);
  st_add(w, (b + "tp_rank").c_str(), "I64", nullptr, 0, &eight, 8);
}

size_t st_write(const qtip_st_writer* w, const char* path, const char* const* meta_kv, int nmeta) {
  QTIP_REQUIRE(w && path && nmeta >= 0 && (nmeta == 0 || meta_kv), "st_write: bad arguments");
  std::map<std::string, std::string> meta;
  for (int i = 0; i < nmeta; ++i) meta[meta_kv[2 * i]] = meta_kv[2 * i + 1];
  // header: one object, keys sorted bytewise, "__metadata__" taking its sorted place among the tensor names
  std::string hs = "{";
  bool first = true, meta_done = meta.empty();
  auto put_meta = [&] {
    if (!first) hs.push_back(',');
    first = false;
    hs += "\"__metadata__\":{";
    bool f2 = true;
    for (auto& kv : meta) {
      if (!f2) hs.push_back(',');
      f2 = false;
      json_string(hs, kv.first);
      hs.push_back(':');
      json_string(hs, kv.second);
    }
    hs.push_back('}');
    meta_done = true;
  };
  uint64_t off = 0;
  for (auto& kv : w->entries) {
    if (!meta_done && std::string("__metadata__") < kv.first) put_meta();
    if (!first) hs.push_back(',');
    first = false;
    json_string(hs, kv.first);
    hs += ":{\"data_offsets\":[" + std::to_string(off) + "," + std::to_string(off + kv.second.data.size()) + "],\"dtype\":";
    json_string(hs, kv.second.dtype);
    hs += ",\"shape\":[";
    for (size_t i = 0; i < kv.second.shape.size(); ++i) {
      if (i) hs.push_back(',');
      hs += std::to_string(kv.second.shape[i]);
    }
    hs += "]}";
    off += kv.second.data.size();
  }
  if (!meta_done) put_meta();
  hs.push_back('}');
  while (hs.size() % 8) hs.push_back(' ');
  const std::string tmp = std::string(path) + ".tmp";
  FILE* f = fopen(tmp.c_str(), "wb");
  if (!f) fail(QTIP_E_ARG, "cannot write %s", tmp.c_str());
  const uint64_t hl = hs.size();
  bool ok = fwrite(&hl, 8, 1, f) == 1 && fwrite(hs.data(), 1, hs.size(), f) == hs.size();
  for (auto& kv : w->entries)
    if (ok && !kv.second.data.empty()) ok = fwrite(kv.second.data.data(), 1, kv.second.data.size(), f) == kv.second.data.size();
  ok = (fflush(f) == 0) && ok;
  ok = (fclose(f) == 0) && ok;
  if (!ok) {
    remove(tmp.c_str());
    fail(QTIP_E_ARG, "write failed: %s", tmp.c_str());
  }
  if (rename(tmp.c_str(), path) != 0) {
    remove(tmp.c_str());
    fail(QTIP_E_ARG, "cannot rename %s to %s", tmp.c_str(), path);
  }
  return size_t(8 + hs.size() + off);
}

}  // namespace qtipmi
