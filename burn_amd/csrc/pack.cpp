// burnpack containers (crates/burn-pack): reading quantized (and float) tensors of a .bpk file
// straight into device tensors, and writing device tensors out in the same format.
//
// File layout (crates/burn-pack/src/lib.rs:52-82, base.rs:13-60): a 10-byte header -- magic
// 0x4255524E little endian ("NRUB" on disk), u16 version 1, u32 byte length of the metadata --, the
// metadata as CBOR, zero padding up to the next multiple of 256 bytes, then the tensor data section
// in which every tensor starts on a 256-byte boundary. The metadata is the serde image of
//   { tensors: map name -> { dtype, shape: [u64], data_offsets: [start, end], param_id? },
//     metadata?: map string -> string, scalars?: map string -> scalar }
// with offsets relative to the data section (base.rs:286-312). A quantized tensor's bytes are its
// QuantizedBytes blob (writer.rs:310-340 takes the producer's length, burn-store's
// tensor_snapshot.rs:253-262 computes it with quantized_data_len): values || scales, i.e. exactly
// what bq_q_from_data takes, so a tensor loads with one host-to-device copy out of the mapped file.
//
// The dtype of a quantized entry is `QFloat(QuantScheme)`; how QuantScheme serializes is decided by
// a crate that is not part of the reference tree, so this reader does not depend on it: the caller
// passes the scheme (a module knows the scheme it was quantized with), and what this writer emits
// for it -- a map of the bq_scheme fields -- is only promised to be readable by this reader.
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cstring>
#include <memory>

#include "common.hpp"

using namespace bq;

namespace {

constexpr uint32_t kMagic = 0x4255524Eu;
constexpr uint16_t kVersion = 1;
constexpr size_t kHeader = 10;
constexpr uint64_t kAlign = 256;
constexpr uint64_t kMaxMetadata = 100ull << 20;      // MAX_METADATA_SIZE
constexpr uint64_t kMaxTensorBytes = 10ull << 30;    // MAX_TENSOR_SIZE (64-bit platforms)
constexpr size_t kMaxTensors = 100000;               // MAX_TENSOR_COUNT
constexpr int kMaxDepth = 128;                       // MAX_CBOR_RECURSION_DEPTH

uint64_t align_up(uint64_t v, uint64_t a) { return (v + a - 1) / a * a; }

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
    if (depth > kMaxDepth || !need(1)) {
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
const char* const kDtypeNames[] = {"F64", "F32", "Flex32", "F16", "BF16", "I64", "I32", "I16", "I8",
                                   "U64", "U32", "U16", "U8", "Bool", "QFloat"};
constexpr int kDtypeSizes[] = {8, 4, 4, 2, 2, 8, 4, 2, 1, 8, 4, 2, 1, 1, 0};

int dtype_from_name(const std::string& s) {
  for (int i = 0; i < BQ_PACK_QFLOAT; ++i)
    if (i != BQ_PACK_BOOL && s == kDtypeNames[i]) return i;
  return -1;
}

void write_scheme(CborWriter& w, const bq_scheme& s) {
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

bool read_scheme(const Cbor& c, bq_scheme* s) {
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

}  // namespace

struct bq_pack {
  const uint8_t* base = nullptr;   // the whole container
  size_t size = 0;
  void* mapped = nullptr;          // non-null: mmap'ed here, unmapped on close
  std::vector<uint8_t> owned;      // non-empty: a private copy (bq_pack_from_bytes with copy)
  size_t data_start = 0;
  std::vector<Entry> entries;      // sorted by name, as the reference's BTreeMap iterates
  std::vector<std::pair<std::string, std::string>> metadata;
};

static bq_status parse_pack(bq_pack* pk) {
  if (pk->size < kHeader) BQ_FAIL(BQ_ERR_SIZE, "burnpack: InvalidHeader (%zu bytes)", pk->size);
  const uint8_t* b = pk->base;
  const uint32_t magic = b[0] | (b[1] << 8) | (b[2] << 16) | (static_cast<uint32_t>(b[3]) << 24);
  if (magic != kMagic) BQ_FAIL(BQ_ERR_DTYPE, "burnpack: InvalidMagicNumber 0x%08X", magic);
  const uint16_t version = static_cast<uint16_t>(b[4] | (b[5] << 8));
  if (version != kVersion) BQ_FAIL(BQ_ERR_DTYPE, "burnpack: InvalidVersion %u", version);
  const uint64_t msize = b[6] | (b[7] << 8) | (b[8] << 16) | (static_cast<uint64_t>(b[9]) << 24);
  if (msize > kMaxMetadata) BQ_FAIL(BQ_ERR_SIZE, "burnpack: metadata size %llu exceeds the maximum", static_cast<unsigned long long>(msize));
  if (pk->size < kHeader + msize) BQ_FAIL(BQ_ERR_SIZE, "burnpack: InvalidHeader (metadata runs past the end)");
  CborReader r{b + kHeader, b + kHeader + msize};
  const Cbor root = r.value(0);
  if (!r.ok || root.kind != Cbor::Map) BQ_FAIL(BQ_ERR_DTYPE, "burnpack: MetadataDeserializationError");
  const Cbor* tensors = root.get("tensors");
  if (!tensors || tensors->kind != Cbor::Map) BQ_FAIL(BQ_ERR_DTYPE, "burnpack: metadata has no tensor map");
  if (tensors->entries.size() > kMaxTensors) BQ_FAIL(BQ_ERR_SIZE, "burnpack: %zu tensors exceed the maximum", tensors->entries.size());
  pk->data_start = static_cast<size_t>(align_up(kHeader + msize, kAlign));
  uint64_t max_end = 0;
  for (auto& kv : tensors->entries) {
    Entry e;
    if (kv.first.kind != Cbor::Text || kv.second.kind != Cbor::Map) BQ_FAIL(BQ_ERR_DTYPE, "burnpack: malformed tensor descriptor");
    e.name = kv.first.s;
    const Cbor *dt = kv.second.get("dtype"), *sh = kv.second.get("shape"), *off = kv.second.get("data_offsets"), *pid = kv.second.get("param_id");
    if (!dt || !sh || !off || sh->kind != Cbor::Array || off->kind != Cbor::Array || off->items.size() != 2 ||
        off->items[0].kind != Cbor::UInt || off->items[1].kind != Cbor::UInt)
      BQ_FAIL(BQ_ERR_DTYPE, "burnpack: tensor '%s' has a malformed descriptor", e.name.c_str());
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
    if (e.dtype < 0) BQ_FAIL(BQ_ERR_DTYPE, "burnpack: tensor '%s' has an unknown dtype", e.name.c_str());
    for (auto& d : sh->items) {
      if (d.kind != Cbor::UInt) BQ_FAIL(BQ_ERR_DTYPE, "burnpack: tensor '%s' has a malformed shape", e.name.c_str());
      e.shape.push_back(static_cast<size_t>(d.u));
    }
    e.begin = off->items[0].u;
    e.end = off->items[1].u;
    if (e.end < e.begin) BQ_FAIL(BQ_ERR_SIZE, "burnpack: tensor '%s' has inverted offsets", e.name.c_str());
    if (e.end - e.begin > kMaxTensorBytes) BQ_FAIL(BQ_ERR_SIZE, "burnpack: tensor '%s' exceeds the maximum tensor size", e.name.c_str());
    if (pid && pid->kind == Cbor::UInt) { e.has_param = true; e.param_id = pid->u; }
    max_end = std::max(max_end, e.end);
    pk->entries.push_back(std::move(e));
  }
  // the container must hold every byte its descriptors claim (reader.rs validate_total_size)
  if (max_end > 0 && (pk->data_start > pk->size || max_end > pk->size - pk->data_start))
    BQ_FAIL(BQ_ERR_SIZE, "burnpack: ValidationError: the file is smaller than its tensors (%zu bytes, data section %zu + %llu)",
            pk->size, pk->data_start, static_cast<unsigned long long>(max_end));
  std::sort(pk->entries.begin(), pk->entries.end(), [](const Entry& a, const Entry& c) { return a.name < c.name; });
  if (const Cbor* md = root.get("metadata"))
    if (md->kind == Cbor::Map)
      for (auto& kv : md->entries)
        if (kv.first.kind == Cbor::Text && kv.second.kind == Cbor::Text) pk->metadata.emplace_back(kv.first.s, kv.second.s);
  return BQ_OK;
}

extern "C" size_t bq_pack_data_section_start(size_t metadata_size) {
  return static_cast<size_t>(align_up(kHeader + metadata_size, kAlign));
}

extern "C" bq_status bq_pack_from_bytes(const uint8_t* bytes, size_t len, int32_t copy, bq_pack** out) {
  BQ_NOTNULL(bytes);
  BQ_NOTNULL(out);
  *out = nullptr;
  std::unique_ptr<bq_pack> pk(new bq_pack());
  if (copy) {
    pk->owned.assign(bytes, bytes + len);
    pk->base = pk->owned.data();
  } else {
    pk->base = bytes;
  }
  pk->size = len;
  BQ_TRY(parse_pack(pk.get()));
  *out = pk.release();
  return BQ_OK;
}

extern "C" bq_status bq_pack_open(const char* path, bq_pack** out) {
  BQ_NOTNULL(path);
  BQ_NOTNULL(out);
  *out = nullptr;
  std::string p(path);
  int fd = open(p.c_str(), O_RDONLY);
  if (fd < 0 && p.find('.', p.find_last_of('/') == std::string::npos ? 0 : p.find_last_of('/')) == std::string::npos) {
    p += ".bpk";  // no extension and no such file: the canonical one (reader.rs:62-67)
    fd = open(p.c_str(), O_RDONLY);
  }
  if (fd < 0) BQ_FAIL(BQ_ERR_SIZE, "burnpack: IoError: cannot open '%s'", path);
  struct stat st;
  if (fstat(fd, &st) != 0 || st.st_size < 0) {
    close(fd);
    BQ_FAIL(BQ_ERR_SIZE, "burnpack: IoError: cannot stat '%s'", p.c_str());
  }
  if (static_cast<uint64_t>(st.st_size) > (100ull << 30)) {
    close(fd);
    BQ_FAIL(BQ_ERR_SIZE, "burnpack: ValidationError: file size exceeds the maximum (MAX_FILE_SIZE)");
  }
  std::unique_ptr<bq_pack> pk(new bq_pack());
  pk->size = static_cast<size_t>(st.st_size);
  if (pk->size > 0) {
    void* m = mmap(nullptr, pk->size, PROT_READ, MAP_PRIVATE, fd, 0);
    if (m == MAP_FAILED) {
      close(fd);
      BQ_FAIL(BQ_ERR_SIZE, "burnpack: IoError: cannot map '%s'", p.c_str());
    }
    pk->mapped = m;
    pk->base = static_cast<const uint8_t*>(m);
  }
  close(fd);
  bq_status rc = parse_pack(pk.get());
  if (rc != BQ_OK) {
    if (pk->mapped) munmap(pk->mapped, pk->size);
    return rc;
  }
  *out = pk.release();
  return BQ_OK;
}

extern "C" bq_status bq_pack_close(bq_pack* pk) {
  BQ_NOTNULL(pk);
  if (pk->mapped) munmap(pk->mapped, pk->size);
  delete pk;
  return BQ_OK;
}

extern "C" int64_t bq_pack_num_tensors(const bq_pack* pk) { return pk ? static_cast<int64_t>(pk->entries.size()) : -1; }

static void fill_entry(const bq_pack* pk, const Entry& e, bq_pack_entry* out) {
  memset(out, 0, sizeof(*out));
  out->name = e.name.c_str();
  out->dtype = e.dtype;
  out->rank = static_cast<int32_t>(std::min<size_t>(e.shape.size(), BQ_MAX_RANK));
  for (int i = 0; i < out->rank; ++i) out->shape[i] = e.shape[i];
  out->data_begin = e.begin;
  out->data_end = e.end;
  out->has_param_id = e.has_param;
  out->param_id = e.param_id;
  out->has_scheme = e.has_scheme;
  out->scheme = e.scheme;
  out->data = pk->base + pk->data_start + e.begin;
}

extern "C" bq_status bq_pack_entry_at(const bq_pack* pk, int64_t index, bq_pack_entry* out) {
  BQ_NOTNULL(pk);
  BQ_NOTNULL(out);
  if (index < 0 || static_cast<size_t>(index) >= pk->entries.size()) BQ_FAIL(BQ_ERR_SHAPE, "burnpack: entry %lld of %zu", static_cast<long long>(index), pk->entries.size());
  fill_entry(pk, pk->entries[static_cast<size_t>(index)], out);
  return BQ_OK;
}

static const Entry* find_entry(const bq_pack* pk, const char* name) {
  for (auto& e : pk->entries)
    if (e.name == name) return &e;
  return nullptr;
}

extern "C" bq_status bq_pack_find(const bq_pack* pk, const char* name, bq_pack_entry* out) {
  BQ_NOTNULL(pk);
  BQ_NOTNULL(name);
  BQ_NOTNULL(out);
  const Entry* e = find_entry(pk, name);
  if (!e) BQ_FAIL(BQ_ERR_SHAPE, "burnpack: TensorNotFound '%s'", name);
  fill_entry(pk, *e, out);
  return BQ_OK;
}

extern "C" const char* bq_pack_metadata(const bq_pack* pk, const char* key) {
  if (!pk || !key) return nullptr;
  for (auto& kv : pk->metadata)
    if (kv.first == key) return kv.second.c_str();
  return nullptr;
}

extern "C" bq_status bq_pack_load(const bq_pack* pk, const char* name, const bq_scheme* scheme, bq_device* dev,
                                  bq_tensor** out) {
  BQ_NOTNULL(pk);
  BQ_NOTNULL(name);
  BQ_NOTNULL(dev);
  BQ_NOTNULL(out);
  *out = nullptr;
  const Entry* e = find_entry(pk, name);
  if (!e) BQ_FAIL(BQ_ERR_SHAPE, "burnpack: TensorNotFound '%s'", name);
  if (e->shape.empty() || e->shape.size() > BQ_MAX_RANK) BQ_FAIL(BQ_ERR_SHAPE, "burnpack: tensor '%s' has rank %zu", name, e->shape.size());
  const uint8_t* data = pk->base + pk->data_start + e->begin;
  const size_t len = static_cast<size_t>(e->end - e->begin);
  const int rank = static_cast<int>(e->shape.size());
  if (e->dtype == BQ_PACK_QFLOAT) {
    const bq_scheme* s = scheme ? scheme : (e->has_scheme ? &e->scheme : nullptr);
    if (!s) BQ_FAIL(BQ_ERR_UNSUPPORTED_SCHEME, "burnpack: tensor '%s' is quantized and its scheme was not written by this library: pass the scheme", name);
    // (a length that disagrees with the scheme and shape is the reference's TensorBytesSizeMismatch)
    return bq_q_from_data(dev, data, len, e->shape.data(), rank, s, out);
  }
  if (e->dtype != BQ_PACK_F32 && e->dtype != BQ_PACK_BF16)
    BQ_FAIL(BQ_ERR_DTYPE, "burnpack: tensor '%s' is %s; this backend holds f32, bf16 and quantized tensors", name, kDtypeNames[e->dtype]);
  size_t n = 1;
  for (size_t d : e->shape) n *= d;
  if (len != n * static_cast<size_t>(kDtypeSizes[e->dtype]))
    BQ_FAIL(BQ_ERR_SIZE, "burnpack: TensorBytesSizeMismatch for '%s': %zu bytes for %zu elements", name, len, n);
  return bq_float_from_data(dev, data, e->dtype == BQ_PACK_F32 ? BQ_F32 : BQ_BF16, e->shape.data(), rank, out);
}

// ================================================================================ writer
struct PendingTensor {
  std::string name;
  int dtype;
  bool quantized;
  bq_scheme scheme;
  std::vector<size_t> shape;
  std::vector<uint8_t> bytes;
  bool has_param;
  uint64_t param_id;
};

struct bq_pack_writer {
  std::vector<PendingTensor> tensors;                           // in the order they were added
  std::vector<std::pair<std::string, std::string>> metadata;
};

extern "C" bq_status bq_pack_writer_new(bq_pack_writer** out) {
  BQ_NOTNULL(out);
  *out = new bq_pack_writer();
  return BQ_OK;
}

extern "C" bq_status bq_pack_writer_free(bq_pack_writer* w) {
  BQ_NOTNULL(w);
  delete w;
  return BQ_OK;
}

extern "C" bq_status bq_pack_writer_set_metadata(bq_pack_writer* w, const char* key, const char* value) {
  BQ_NOTNULL(w);
  BQ_NOTNULL(key);
  BQ_NOTNULL(value);
  for (auto& kv : w->metadata)
    if (kv.first == key) {
      kv.second = value;
      return BQ_OK;
    }
  w->metadata.emplace_back(key, value);
  return BQ_OK;
}

extern "C" bq_status bq_pack_writer_add_bytes(bq_pack_writer* w, const char* name, int32_t dtype, const bq_scheme* scheme,
                                              const size_t* shape, int32_t rank, const uint8_t* data, size_t len,
                                              int32_t has_param_id, uint64_t param_id) {
  BQ_NOTNULL(w);
  BQ_NOTNULL(name);
  BQ_NOTNULL(shape);
  if (len) BQ_NOTNULL(data);
  if (rank < 0 || rank > BQ_MAX_RANK) BQ_FAIL(BQ_ERR_SHAPE, "rank %d outside 0..%d", rank, BQ_MAX_RANK);
  if (dtype < 0 || dtype > BQ_PACK_QFLOAT || dtype == BQ_PACK_BOOL) BQ_FAIL(BQ_ERR_DTYPE, "burnpack writer: dtype %d", dtype);
  for (auto& t : w->tensors)
    if (t.name == name) BQ_FAIL(BQ_ERR_SHAPE, "burnpack: ValidationError: Duplicate tensor name '%s'", name);
  PendingTensor t;
  t.name = name;
  t.dtype = dtype;
  t.quantized = dtype == BQ_PACK_QFLOAT;
  memset(&t.scheme, 0, sizeof(t.scheme));
  t.shape.assign(shape, shape + rank);
  size_t expect;
  if (t.quantized) {
    BQ_NOTNULL(scheme);
    t.scheme = *scheme;
    BQ_TRY(bq_quantized_data_len(scheme, shape, rank, &expect));
  } else {
    size_t n = 1;
    for (int i = 0; i < rank; ++i) n *= shape[i];
    expect = n * static_cast<size_t>(kDtypeSizes[dtype]);
  }
  // (writer.rs check_byte_len: a length that cannot describe the declared tensor is refused)
  if (len != expect) BQ_FAIL(BQ_ERR_SIZE, "burnpack: TensorBytesSizeMismatch for '%s': %zu bytes, dtype and shape need %zu", name, len, expect);
  t.bytes.assign(data, data + len);
  t.has_param = has_param_id != 0;
  t.param_id = param_id;
  w->tensors.push_back(std::move(t));
  return BQ_OK;
}

extern "C" bq_status bq_pack_writer_add_tensor(bq_pack_writer* w, const char* name, const bq_tensor* t,
                                               int32_t has_param_id, uint64_t param_id) {
  BQ_NOTNULL(w);
  BQ_NOTNULL(name);
  BQ_NOTNULL(t);
  size_t shape[BQ_MAX_RANK];
  BQ_TRY(bq_tensor_shape(t, shape));
  const int rank = bq_tensor_rank(t);
  std::vector<uint8_t> host;
  if (bq_tensor_dtype(t) == BQ_QFLOAT) {
    bq_scheme s;
    BQ_TRY(bq_tensor_scheme(t, &s));
    size_t len = 0;
    BQ_TRY(bq_quantized_data_len(&s, shape, rank, &len));
    host.resize(len ? len : 1);
    size_t got = 0;
    BQ_TRY(bq_q_into_data(t, host.data(), len, &got));
    return bq_pack_writer_add_bytes(w, name, BQ_PACK_QFLOAT, &s, shape, rank, host.data(), got, has_param_id, param_id);
  }
  size_t n = 1;
  for (int i = 0; i < rank; ++i) n *= shape[i];
  const bool f32 = bq_tensor_dtype(t) == BQ_F32;
  const size_t len = n * (f32 ? 4 : 2);
  host.resize(len ? len : 1);
  BQ_TRY(bq_float_into_data(t, host.data(), len));
  return bq_pack_writer_add_bytes(w, name, f32 ? BQ_PACK_F32 : BQ_PACK_BF16, nullptr, shape, rank, host.data(), len, has_param_id, param_id);
}

// Header, metadata, padding and data section of everything added so far.
static std::vector<uint8_t> build_container(const bq_pack_writer* w) {
  // offsets in insertion order (writer.rs:264-314), descriptors keyed and emitted in name order
  std::vector<uint64_t> begin(w->tensors.size()), end(w->tensors.size());
  uint64_t cur = 0;
  for (size_t i = 0; i < w->tensors.size(); ++i) {
    begin[i] = align_up(cur, kAlign);
    end[i] = begin[i] + w->tensors[i].bytes.size();
    cur = end[i];
  }
  std::vector<size_t> order(w->tensors.size());
  for (size_t i = 0; i < order.size(); ++i) order[i] = i;
  std::sort(order.begin(), order.end(), [&](size_t a, size_t b) { return w->tensors[a].name < w->tensors[b].name; });
  CborWriter c;
  c.map(w->metadata.empty() ? 1 : 2);
  c.text("tensors");
  c.map(order.size());
  for (size_t i : order) {
    const PendingTensor& t = w->tensors[i];
    c.text(t.name);
    c.map(t.has_param ? 4 : 3);
    c.text("dtype");
    if (t.quantized) { c.map(1); c.text("QFloat"); write_scheme(c, t.scheme); } else { c.text(kDtypeNames[t.dtype]); }
    c.text("shape");
    c.array(t.shape.size());
    for (size_t d : t.shape) c.uint(d);
    c.text("data_offsets");
    c.array(2);
    c.uint(begin[i]);
    c.uint(end[i]);
    if (t.has_param) { c.text("param_id"); c.uint(t.param_id); }
  }
  if (!w->metadata.empty()) {
    auto md = w->metadata;
    std::sort(md.begin(), md.end());
    c.text("metadata");
    c.map(md.size());
    for (auto& kv : md) { c.text(kv.first); c.text(kv.second); }
  }
  const size_t msize = c.out.size();
  const size_t data_start = static_cast<size_t>(align_up(kHeader + msize, kAlign));
  std::vector<uint8_t> out(data_start + static_cast<size_t>(cur), 0);
  const uint8_t header[kHeader] = {0x4E, 0x52, 0x55, 0x42, 0x01, 0x00, static_cast<uint8_t>(msize), static_cast<uint8_t>(msize >> 8),
                                   static_cast<uint8_t>(msize >> 16), static_cast<uint8_t>(msize >> 24)};
  memcpy(out.data(), header, kHeader);
  memcpy(out.data() + kHeader, c.out.data(), msize);
  for (size_t i = 0; i < w->tensors.size(); ++i)
    if (!w->tensors[i].bytes.empty()) memcpy(out.data() + data_start + begin[i], w->tensors[i].bytes.data(), w->tensors[i].bytes.size());
  return out;
}

extern "C" bq_status bq_pack_writer_size(const bq_pack_writer* w, size_t* size_out) {
  BQ_NOTNULL(w);
  BQ_NOTNULL(size_out);
  *size_out = build_container(w).size();
  return BQ_OK;
}

extern "C" bq_status bq_pack_writer_write_into(const bq_pack_writer* w, uint8_t* buffer, size_t capacity, size_t* size_out) {
  BQ_NOTNULL(w);
  BQ_NOTNULL(size_out);
  const std::vector<uint8_t> bytes = build_container(w);
  *size_out = bytes.size();
  if (capacity < bytes.size()) BQ_FAIL(BQ_ERR_SIZE, "burnpack: buffer of %zu bytes for a container of %zu", capacity, bytes.size());
  BQ_NOTNULL(buffer);
  memcpy(buffer, bytes.data(), bytes.size());
  return BQ_OK;
}

extern "C" bq_status bq_pack_writer_write_file(const bq_pack_writer* w, const char* path) {
  BQ_NOTNULL(w);
  BQ_NOTNULL(path);
  const std::vector<uint8_t> bytes = build_container(w);
  FILE* f = fopen(path, "wb");
  if (!f) BQ_FAIL(BQ_ERR_SIZE, "burnpack: IoError: cannot create '%s'", path);
  const size_t done = fwrite(bytes.data(), 1, bytes.size(), f);
  const int rc = fclose(f);
  if (done != bytes.size() || rc != 0) BQ_FAIL(BQ_ERR_SIZE, "burnpack: IoError: short write to '%s'", path);
  return BQ_OK;
}
