// The burnpack container format (crates/burn-pack), in plain C++ with no GPU dependency: header
// and limits (base.rs:13-60), the CBOR subset serde writes for the metadata, and the parser of
// header + metadata into tensor descriptors. Everything here takes untrusted bytes: a malformed
// container is answered with a status and a message, never with an exception escaping, an
// out-of-range read or unbounded memory -- the number of CBOR nodes is capped, and the tests build
// this file with the address and undefined-behaviour sanitizers and run a mutation fuzz over it.
#pragma once

#include <algorithm>
#include <cmath>
#include <new>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <utility>
#include <vector>

#include "burnq.h"

namespace bq {
namespace pack {

constexpr uint32_t kMagic = 0x4255524Eu;
constexpr uint16_t kVersion = 1;
constexpr size_t kHeader = 10;
constexpr uint64_t kAlign = 256;
constexpr uint64_t kMaxMetadata = 100ull << 20;      // MAX_METADATA_SIZE
constexpr uint64_t kMaxTensorBytes = 10ull << 30;    // MAX_TENSOR_SIZE (64-bit platforms)
constexpr size_t kMaxTensors = 100000;               // MAX_TENSOR_COUNT
constexpr int kMaxDepth = 128;                       // MAX_CBOR_RECURSION_DEPTH
// Upper bound on decoded CBOR nodes. A descriptor is about 25 nodes (40 with a quantization scheme),
// so this admits MAX_TENSOR_COUNT real tensors; what it refuses is metadata made of millions of
// one-byte items, each of which would otherwise cost a hundred bytes of tree.
constexpr size_t kMaxNodes = 48 * kMaxTensors + 4096;

inline uint64_t align_up(uint64_t v, uint64_t a) { return (v + a - 1) / a * a; }

// ---- CBOR (RFC 8949), the subset serde emits for the metadata -------------------------------------
struct Cbor {
  enum Kind { UInt, NInt, Bytes, Text, Array, Map, Float, Bool, Null } kind = Null;
  uint64_t u = 0;        // UInt value, NInt: -1 - u, Bool
  double f = 0;
  std::string s;         // Text / Bytes
  std::vector<Cbor> items;                          // Array
  std::vector<std::pair<Cbor, Cbor>> entries;       // Map, in file order
  const Cbor* get(const char* key) const {
    for (auto& e : entries)
      if (e.first.kind == Text && e.first.s == key) return &e.second;
    return nullptr;
  }
};

struct CborReader {
  const uint8_t* p;
  const uint8_t* end;
  bool ok = true;
  size_t nodes = 0;
  bool need(size_t n) {
    if (static_cast<size_t>(end - p) < n) ok = false;
    return ok;
  }
  uint64_t arg(uint8_t info) {
    if (info < 24) return info;
    const int n = info == 24 ? 1 : info == 25 ? 2 : info == 26 ? 4 : info == 27 ? 8 : 0;
    if (n == 0 || !need(static_cast<size_t>(n))) {
      ok = false;
      return 0;
    }
    uint64_t v = 0;
    for (int i = 0; i < n; ++i) v = (v << 8) | *p++;
    return v;
  }
  Cbor value(int depth) {
    Cbor c;
    if (depth > kMaxDepth || ++nodes > kMaxNodes || !need(1)) {
      ok = false;
      return c;
    }
    const uint8_t head = *p++;
    const uint8_t major = head >> 5, info = head & 31;
    if (info == 31 && major != 7) {  // indefinite lengths: serde never writes them here
      ok = false;
      return c;
    }
    switch (major) {
      case 0: c.kind = Cbor::UInt; c.u = arg(info); break;
      case 1: c.kind = Cbor::NInt; c.u = arg(info); break;
      case 2:
      case 3: {
        const uint64_t n = arg(info);
        if (!ok || !need(n)) { ok = false; break; }
        c.kind = major == 2 ? Cbor::Bytes : Cbor::Text;
        c.s.assign(reinterpret_cast<const char*>(p), n);
        p += n;
        break;
      }
      case 4: {
        const uint64_t n = arg(info);
        if (!ok || n > static_cast<uint64_t>(end - p)) { ok = false; break; }
        c.kind = Cbor::Array;
        for (uint64_t i = 0; i < n && ok; ++i) c.items.push_back(value(depth + 1));
        break;
      }
      case 5: {
        const uint64_t n = arg(info);
        if (!ok || n > static_cast<uint64_t>(end - p)) { ok = false; break; }
        c.kind = Cbor::Map;
        for (uint64_t i = 0; i < n && ok; ++i) {
          Cbor k = value(depth + 1);
          Cbor v = value(depth + 1);
          c.entries.emplace_back(std::move(k), std::move(v));
        }
        break;
      }
      case 6: (void)arg(info); c = value(depth + 1); break;  // a tag: the tagged value
      default:
        if (info == 20 || info == 21) { c.kind = Cbor::Bool; c.u = info == 21; }
        else if (info == 22 || info == 23) { c.kind = Cbor::Null; }
        else if (info == 25 || info == 26 || info == 27) {
          const uint64_t bits = arg(info);
          c.kind = Cbor::Float;
          if (info == 27) { memcpy(&c.f, &bits, 8); }
          else if (info == 26) { float t; const uint32_t b = static_cast<uint32_t>(bits); memcpy(&t, &b, 4); c.f = t; }
          else {  // half
            const uint32_t h = static_cast<uint32_t>(bits), ex = (h >> 10) & 31, man = h & 1023;
            double v = ex == 0 ? man * 5.9604644775390625e-8 : ex == 31 ? (man ? NAN : INFINITY) : (1024 + man) * std::pow(2.0, static_cast<int>(ex) - 25);
            c.f = (h & 0x8000) ? -v : v;
          }
        } else { ok = false; }
    }
    return c;
  }
};

struct CborWriter {
  std::vector<uint8_t> out;
  void head(uint8_t major, uint64_t v) {  // shortest form, as ciborium writes integers and lengths
    const uint8_t m = static_cast<uint8_t>(major << 5);
    if (v < 24) { out.push_back(m | static_cast<uint8_t>(v)); return; }
    const int n = v <= 0xFF ? 1 : v <= 0xFFFF ? 2 : v <= 0xFFFFFFFFull ? 4 : 8;
    out.push_back(m | static_cast<uint8_t>(n == 1 ? 24 : n == 2 ? 25 : n == 4 ? 26 : 27));
    for (int i = n - 1; i >= 0; --i) out.push_back(static_cast<uint8_t>(v >> (8 * i)));
  }
  void uint(uint64_t v) { head(0, v); }
  void text(const std::string& s) { head(3, s.size()); out.insert(out.end(), s.begin(), s.end()); }
  void array(uint64_t n) { head(4, n); }
  void map(uint64_t n) { head(5, n); }
};

// ---- dtypes ----------------------------------------------------------------------------------------
static const char* const kDtypeNames[] = {"F64", "F32", "Flex32", "F16", "BF16", "I64", "I32", "I16", "I8",
                                   "U64", "U32", "U16", "U8", "Bool", "QFloat"};
constexpr int kDtypeSizes[] = {8, 4, 4, 2, 2, 8, 4, 2, 1, 8, 4, 2, 1, 1, 0};

inline int dtype_from_name(const std::string& s) {
  for (int i = 0; i < BQ_PACK_QFLOAT; ++i)
    if (i != BQ_PACK_BOOL && s == kDtypeNames[i]) return i;
  return -1;
}

inline void write_scheme(CborWriter& w, const bq_scheme& s) {
  w.map(s.tensor_scale ? 6 : 5);
  static const char* const kValueNames[] = {"Q8S", "Q4S", "Q2S", "Q8F", "Q4F", "Q2F"};
  w.text("value"); w.text(kValueNames[s.value <= BQ_Q2F ? s.value : 0]);
  w.text("level");
  if (s.level == BQ_LEVEL_TENSOR) { w.text("Tensor"); }
  else { w.map(1); w.text("Block"); w.array(s.block_rank); for (int i = 0; i < s.block_rank; ++i) w.uint(s.block[i]); }
  w.text("store");
  if (s.store == BQ_STORE_NATIVE) { w.text("Native"); } else { w.map(1); w.text("PackedU32"); w.uint(0); }
  w.text("scale_dtype");
  w.text(s.scale_dtype == BQ_SCALE_F32 ? "F32" : s.scale_dtype == BQ_SCALE_F16 ? "F16" : s.scale_dtype == BQ_SCALE_BF16 ? "BF16" : "UE4M3");
  w.text("mode"); w.text("Symmetric");
  if (s.tensor_scale) { w.text("tensor_scale"); w.text("F32"); }  // two-level: a per-tensor f32 scale on top
}

inline bool read_scheme(const Cbor& c, bq_scheme* s) {
  if (c.kind != Cbor::Map) return false;
  memset(s, 0, sizeof(*s));
  const Cbor *value = c.get("value"), *level = c.get("level"), *store = c.get("store"), *sd = c.get("scale_dtype");
  if (!value || !level || !store || !sd || value->kind != Cbor::Text || sd->kind != Cbor::Text) return false;
  if (value->s == "Q8S") s->value = BQ_Q8S; else if (value->s == "Q4S") s->value = BQ_Q4S;
  else if (value->s == "Q2S") s->value = BQ_Q2S; else if (value->s == "Q8F") s->value = BQ_Q8F;
  else if (value->s == "Q4F") s->value = BQ_Q4F; else if (value->s == "Q2F") s->value = BQ_Q2F; else return false;
  if (const Cbor* ts = c.get("tensor_scale")) {
    if (ts->kind != Cbor::Text || ts->s != "F32") return false;
    s->tensor_scale = 1;
  }
  if (sd->s == "F32") s->scale_dtype = BQ_SCALE_F32; else if (sd->s == "F16") s->scale_dtype = BQ_SCALE_F16;
  else if (sd->s == "BF16") s->scale_dtype = BQ_SCALE_BF16; else if (sd->s == "UE4M3") s->scale_dtype = BQ_SCALE_UE4M3;
  else return false;
  if (level->kind == Cbor::Text && level->s == "Tensor") {
    s->level = BQ_LEVEL_TENSOR;
  } else if (level->kind == Cbor::Map && level->get("Block") && level->get("Block")->kind == Cbor::Array) {
    const auto& b = level->get("Block")->items;
    if (b.empty() || b.size() > BQ_MAX_RANK) return false;
    s->level = BQ_LEVEL_BLOCK;
    s->block_rank = static_cast<uint8_t>(b.size());
    for (size_t i = 0; i < b.size(); ++i) {
      if (b[i].kind != Cbor::UInt || b[i].u == 0 || b[i].u > 255) return false;
      s->block[i] = static_cast<uint8_t>(b[i].u);
    }
  } else {
    return false;
  }
  if (store->kind == Cbor::Text && store->s == "Native") s->store = BQ_STORE_NATIVE;
  else if (store->kind == Cbor::Map && store->get("PackedU32")) s->store = BQ_STORE_PACKED_U32;
  else return false;
  return true;
}

struct Entry {
  std::string name;
  int dtype = -1;
  bool has_scheme = false;
  bq_scheme scheme{};
  std::vector<size_t> shape;
  uint64_t begin = 0, end = 0;
  bool has_param = false;
  uint64_t param_id = 0;
};
// What header + metadata say: where the data section starts and one descriptor per tensor.
struct Index {
  size_t data_start = 0;
  std::vector<Entry> entries;      // sorted by name, as the reference's BTreeMap iterates
  std::vector<std::pair<std::string, std::string>> metadata;
};

struct Failure {
  bq_status status = BQ_OK;
  char message[256] = {0};
};

#define BQ_PACK_FAIL(code, ...)                                  \
  do {                                                           \
    fail->status = (code);                                       \
    snprintf(fail->message, sizeof(fail->message), __VA_ARGS__); \
    return (code);                                               \
  } while (0)

inline bq_status parse_container_unguarded(const uint8_t* base, size_t size, Index* pk, Failure* fail) {
  if (size < kHeader) BQ_PACK_FAIL(BQ_ERR_SIZE, "burnpack: InvalidHeader (%zu bytes)", size);
  const uint8_t* b = base;
  const uint32_t magic = b[0] | (b[1] << 8) | (b[2] << 16) | (static_cast<uint32_t>(b[3]) << 24);
  if (magic != kMagic) BQ_PACK_FAIL(BQ_ERR_DTYPE, "burnpack: InvalidMagicNumber 0x%08X", magic);
  const uint16_t version = static_cast<uint16_t>(b[4] | (b[5] << 8));
  if (version != kVersion) BQ_PACK_FAIL(BQ_ERR_DTYPE, "burnpack: InvalidVersion %u", version);
  const uint64_t msize = b[6] | (b[7] << 8) | (b[8] << 16) | (static_cast<uint64_t>(b[9]) << 24);
  if (msize > kMaxMetadata) BQ_PACK_FAIL(BQ_ERR_SIZE, "burnpack: metadata size %llu exceeds the maximum", static_cast<unsigned long long>(msize));
  if (size < kHeader + msize) BQ_PACK_FAIL(BQ_ERR_SIZE, "burnpack: InvalidHeader (metadata runs past the end)");
  CborReader r{b + kHeader, b + kHeader + msize};
  const Cbor root = r.value(0);
  if (!r.ok || root.kind != Cbor::Map) BQ_PACK_FAIL(BQ_ERR_DTYPE, "burnpack: MetadataDeserializationError");
  const Cbor* tensors = root.get("tensors");
  if (!tensors || tensors->kind != Cbor::Map) BQ_PACK_FAIL(BQ_ERR_DTYPE, "burnpack: metadata has no tensor map");
  if (tensors->entries.size() > kMaxTensors) BQ_PACK_FAIL(BQ_ERR_SIZE, "burnpack: %zu tensors exceed the maximum", tensors->entries.size());
  pk->data_start = static_cast<size_t>(align_up(kHeader + msize, kAlign));
  uint64_t max_end = 0;
  for (auto& kv : tensors->entries) {
    Entry e;
    if (kv.first.kind != Cbor::Text || kv.second.kind != Cbor::Map) BQ_PACK_FAIL(BQ_ERR_DTYPE, "burnpack: malformed tensor descriptor");
    e.name = kv.first.s;
    const Cbor *dt = kv.second.get("dtype"), *sh = kv.second.get("shape"), *off = kv.second.get("data_offsets"), *pid = kv.second.get("param_id");
    if (!dt || !sh || !off || sh->kind != Cbor::Array || off->kind != Cbor::Array || off->items.size() != 2 ||
        off->items[0].kind != Cbor::UInt || off->items[1].kind != Cbor::UInt)
      BQ_PACK_FAIL(BQ_ERR_DTYPE, "burnpack: tensor '%s' has a malformed descriptor", e.name.c_str());
    if (dt->kind == Cbor::Text) {
      e.dtype = dtype_from_name(dt->s);
    } else if (dt->kind == Cbor::Map && dt->entries.size() == 1 && dt->entries[0].first.kind == Cbor::Text) {
      if (dt->entries[0].first.s == "QFloat") {
        e.dtype = BQ_PACK_QFLOAT;
        e.has_scheme = read_scheme(dt->entries[0].second, &e.scheme);
      } else if (dt->entries[0].first.s == "Bool") {
        e.dtype = BQ_PACK_BOOL;
      }
    }
    if (e.dtype < 0) BQ_PACK_FAIL(BQ_ERR_DTYPE, "burnpack: tensor '%s' has an unknown dtype", e.name.c_str());
    for (auto& d : sh->items) {
      if (d.kind != Cbor::UInt) BQ_PACK_FAIL(BQ_ERR_DTYPE, "burnpack: tensor '%s' has a malformed shape", e.name.c_str());
      e.shape.push_back(static_cast<size_t>(d.u));
    }
    e.begin = off->items[0].u;
    e.end = off->items[1].u;
    if (e.end < e.begin) BQ_PACK_FAIL(BQ_ERR_SIZE, "burnpack: tensor '%s' has inverted offsets", e.name.c_str());
    if (e.end - e.begin > kMaxTensorBytes) BQ_PACK_FAIL(BQ_ERR_SIZE, "burnpack: tensor '%s' exceeds the maximum tensor size", e.name.c_str());
    if (pid && pid->kind == Cbor::UInt) { e.has_param = true; e.param_id = pid->u; }
    max_end = std::max(max_end, e.end);
    pk->entries.push_back(std::move(e));
  }
  // the container must hold every byte its descriptors claim (reader.rs validate_total_size)
  if (max_end > 0 && (pk->data_start > size || max_end > size - pk->data_start))
    BQ_PACK_FAIL(BQ_ERR_SIZE, "burnpack: ValidationError: the file is smaller than its tensors (%zu bytes, data section %zu + %llu)",
            size, pk->data_start, static_cast<unsigned long long>(max_end));
  std::sort(pk->entries.begin(), pk->entries.end(), [](const Entry& a, const Entry& c) { return a.name < c.name; });
  if (const Cbor* md = root.get("metadata"))
    if (md->kind == Cbor::Map)
      for (auto& kv : md->entries)
        if (kv.first.kind == Cbor::Text && kv.second.kind == Cbor::Text) pk->metadata.emplace_back(kv.first.s, kv.second.s);
  return BQ_OK;
}

// Reader::from_bytes (reader.rs): header, limits, metadata, and the check that the container holds
// every byte its descriptors claim. Touches no tensor data. Never throws: running out of memory while
// decoding is a refusal like any other.
inline bq_status parse_container(const uint8_t* base, size_t size, Index* pk, Failure* fail) {
  try {
    return parse_container_unguarded(base, size, pk, fail);
  } catch (...) {
    BQ_PACK_FAIL(BQ_ERR_SIZE, "burnpack: ValidationError: the metadata could not be decoded (out of memory)");
  }
}

#undef BQ_PACK_FAIL

}  // namespace pack
}  // namespace bq
