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

#include "pack_format.hpp"

using namespace bq;
using namespace bq::pack;

// No C++ exception leaves this file: the container parser, the writer's buffers and the strings all
// allocate, and the caller on the other side of the C ABI (C, ctypes, Rust) cannot unwind.
#define BQ_PACK_GUARD(...)                                                       \
  try {                                                                          \
    __VA_ARGS__                                                                  \
  } catch (const std::bad_alloc&) {                                              \
    BQ_FAIL(BQ_ERR_SIZE, "burnpack: out of memory in %s", __func__);            \
  } catch (const std::exception& e) {                                            \
    BQ_FAIL(BQ_ERR_SIZE, "burnpack: %s failed: %s", __func__, e.what());        \
  } catch (...) {                                                                \
    BQ_FAIL(BQ_ERR_SIZE, "burnpack: %s failed", __func__);                      \
  }

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
  Index index;
  Failure fail;
  if (parse_container(pk->base, pk->size, &index, &fail) != BQ_OK) BQ_FAIL(fail.status, "%s", fail.message);
  pk->data_start = index.data_start;
  pk->entries = std::move(index.entries);
  pk->metadata = std::move(index.metadata);
  return BQ_OK;
}

extern "C" size_t bq_pack_data_section_start(size_t metadata_size) {
  return static_cast<size_t>(align_up(kHeader + metadata_size, kAlign));
}

static bq_status bq_pack_from_bytes_impl(const uint8_t* bytes, size_t len, int32_t copy, bq_pack** out) {
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

static bq_status bq_pack_open_impl(const char* path, bq_pack** out) {
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
  out->data = e.end > e.begin ? pk->base + pk->data_start + e.begin : nullptr;  // (an empty tensor has no bytes to point at)
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

static bq_status bq_pack_load_impl(const bq_pack* pk, const char* name, const bq_scheme* scheme, bq_device* dev,
                                  bq_tensor** out) {
  BQ_NOTNULL(pk);
  BQ_NOTNULL(name);
  BQ_NOTNULL(dev);
  BQ_NOTNULL(out);
  *out = nullptr;
  const Entry* e = find_entry(pk, name);
  if (!e) BQ_FAIL(BQ_ERR_SHAPE, "burnpack: TensorNotFound '%s'", name);
  if (e->shape.empty() || e->shape.size() > BQ_MAX_RANK) BQ_FAIL(BQ_ERR_SHAPE, "burnpack: tensor '%s' has rank %zu", name, e->shape.size());
  const uint8_t* data = e->end > e->begin ? pk->base + pk->data_start + e->begin : pk->base;
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

static bq_status bq_pack_writer_new_impl(bq_pack_writer** out) {
  BQ_NOTNULL(out);
  *out = new bq_pack_writer();
  return BQ_OK;
}

extern "C" bq_status bq_pack_writer_free(bq_pack_writer* w) {
  BQ_NOTNULL(w);
  delete w;
  return BQ_OK;
}

static bq_status bq_pack_writer_set_metadata_impl(bq_pack_writer* w, const char* key, const char* value) {
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

static bq_status bq_pack_writer_add_bytes_impl(bq_pack_writer* w, const char* name, int32_t dtype, const bq_scheme* scheme,
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

static bq_status bq_pack_writer_add_tensor_impl(bq_pack_writer* w, const char* name, const bq_tensor* t,
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
    return bq_pack_writer_add_bytes_impl(w, name, BQ_PACK_QFLOAT, &s, shape, rank, host.data(), got, has_param_id, param_id);
  }
  size_t n = 1;
  for (int i = 0; i < rank; ++i) n *= shape[i];
  const bool f32 = bq_tensor_dtype(t) == BQ_F32;
  const size_t len = n * (f32 ? 4 : 2);
  host.resize(len ? len : 1);
  BQ_TRY(bq_float_into_data(t, host.data(), len));
  return bq_pack_writer_add_bytes_impl(w, name, f32 ? BQ_PACK_F32 : BQ_PACK_BF16, nullptr, shape, rank, host.data(), len, has_param_id, param_id);
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

static bq_status bq_pack_writer_size_impl(const bq_pack_writer* w, size_t* size_out) {
  BQ_NOTNULL(w);
  BQ_NOTNULL(size_out);
  *size_out = build_container(w).size();
  return BQ_OK;
}

static bq_status bq_pack_writer_write_into_impl(const bq_pack_writer* w, uint8_t* buffer, size_t capacity, size_t* size_out) {
  BQ_NOTNULL(w);
  BQ_NOTNULL(size_out);
  const std::vector<uint8_t> bytes = build_container(w);
  *size_out = bytes.size();
  if (capacity < bytes.size()) BQ_FAIL(BQ_ERR_SIZE, "burnpack: buffer of %zu bytes for a container of %zu", capacity, bytes.size());
  BQ_NOTNULL(buffer);
  memcpy(buffer, bytes.data(), bytes.size());
  return BQ_OK;
}

static bq_status bq_pack_writer_write_file_impl(const bq_pack_writer* w, const char* path) {
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

// ---- the exported entry points of everything above that allocates: guarded against exceptions
extern "C" bq_status bq_pack_from_bytes(const uint8_t* bytes, size_t len, int32_t copy, bq_pack** out) {
  BQ_PACK_GUARD(return bq_pack_from_bytes_impl(bytes, len, copy, out);)
}
extern "C" bq_status bq_pack_open(const char* path, bq_pack** out) {
  BQ_PACK_GUARD(return bq_pack_open_impl(path, out);)
}
extern "C" bq_status bq_pack_load(const bq_pack* pk, const char* name, const bq_scheme* scheme, bq_device* dev, bq_tensor** out) {
  BQ_PACK_GUARD(return bq_pack_load_impl(pk, name, scheme, dev, out);)
}
extern "C" bq_status bq_pack_writer_new(bq_pack_writer** out) {
  BQ_PACK_GUARD(return bq_pack_writer_new_impl(out);)
}
extern "C" bq_status bq_pack_writer_set_metadata(bq_pack_writer* w, const char* key, const char* value) {
  BQ_PACK_GUARD(return bq_pack_writer_set_metadata_impl(w, key, value);)
}
extern "C" bq_status bq_pack_writer_add_bytes(bq_pack_writer* w, const char* name, int32_t dtype, const bq_scheme* scheme, const size_t* shape, int32_t rank, const uint8_t* data, size_t len, int32_t has_param_id, uint64_t param_id) {
  BQ_PACK_GUARD(return bq_pack_writer_add_bytes_impl(w, name, dtype, scheme, shape, rank, data, len, has_param_id, param_id);)
}
extern "C" bq_status bq_pack_writer_add_tensor(bq_pack_writer* w, const char* name, const bq_tensor* t, int32_t has_param_id, uint64_t param_id) {
  BQ_PACK_GUARD(return bq_pack_writer_add_tensor_impl(w, name, t, has_param_id, param_id);)
}
extern "C" bq_status bq_pack_writer_size(const bq_pack_writer* w, size_t* size_out) {
  BQ_PACK_GUARD(return bq_pack_writer_size_impl(w, size_out);)
}
extern "C" bq_status bq_pack_writer_write_into(const bq_pack_writer* w, uint8_t* buffer, size_t capacity, size_t* size_out) {
  BQ_PACK_GUARD(return bq_pack_writer_write_into_impl(w, buffer, capacity, size_out);)
}
extern "C" bq_status bq_pack_writer_write_file(const bq_pack_writer* w, const char* path) {
  BQ_PACK_GUARD(return bq_pack_writer_write_file_impl(w, path);)
}
