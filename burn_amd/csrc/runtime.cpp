// Host side of libburnq_mi355.so: device contexts, reference-counted tensors, the TensorData
// wire format and the QTensorOps entry points (validation + kernel dispatch). No arithmetic on
// tensor contents happens on the host: every value is produced by a HIP kernel.
#include <algorithm>
#include <cstdint>
#include <chrono>
#include <cstring>

#include "common.hpp"

namespace bq {

// ---- thread-local error string ------------------------------------------------------------------
static thread_local std::string g_error;

void set_error(const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_error = buf;
}
const char* get_error() { return g_error.c_str(); }

bool fused_block_ok(int block, int value);

// ---- scheme helpers -----------------------------------------------------------------------------
// BlockSize::to_dim_vec(rank): extents aligned to the trailing dims, leading dims 1.
static void block_dims(const bq_scheme& s, int rank, size_t* out) {
  for (int d = 0; d < rank; ++d) out[d] = 1;
  if (s.level == BQ_LEVEL_BLOCK)
    for (int j = 0; j < s.block_rank && j < rank; ++j) out[rank - 1 - j] = s.block[s.block_rank - 1 - j];
}

static size_t num_elements(const size_t* shape, int rank) {
  size_t n = 1;
  for (int d = 0; d < rank; ++d) n *= shape[d];
  return n;
}

// Shapes come from the caller: every size derived from one (element counts, byte counts, the
// allocation) must fit comfortably in 64 bits before anything is multiplied. 2^44 elements is far
// beyond the device's memory and leaves room for the factors applied later.
static bq_status check_shape_size(const size_t* shape, int rank) {
  const size_t limit = static_cast<size_t>(1) << 44;
  size_t n = 1;
  for (int d = 0; d < rank; ++d) {
    if (shape[d] > limit || (shape[d] != 0 && n > limit / shape[d]))
      BQ_FAIL(BQ_ERR_SIZE, "a shape of more than 2^44 elements (dim %d = %zu) is not addressable", d, shape[d]);
    n *= shape[d];
  }
  return BQ_OK;
}

// params_shape (crates/burn-std/src/tensor/quantization.rs:141-146)
static size_t num_params(const bq_scheme& s, const size_t* shape, int rank) {
  if (s.level == BQ_LEVEL_TENSOR) return 1;
  size_t blk[BQ_MAX_RANK];
  block_dims(s, rank, blk);
  size_t n = 1;
  for (int d = 0; d < rank; ++d) n *= shape[d] / blk[d];
  return n;
}

// storage_elements * element size (quantization.rs:382-407): packed words divide only the
// innermost dim; native keeps one byte per value.
static size_t value_bytes(const bq_scheme& s, const size_t* shape, int rank) {
  size_t n = num_elements(shape, rank);
  if (s.store == BQ_STORE_NATIVE) return n;
  size_t nq = static_cast<size_t>(num_quants(s.value));
  if (rank == 0) return 4 * ((n + nq - 1) / nq);
  size_t lines = num_elements(shape, rank - 1);
  return 4 * lines * ((shape[rank - 1] + nq - 1) / nq);
}

// scale_size (crates/burn-std/src/tensor/quantization.rs:409-416): bytes per stored scale on the wire.
static size_t scale_size(const bq_scheme& s) {
  return s.scale_dtype == BQ_SCALE_F32 ? 4 : (s.scale_dtype == BQ_SCALE_UE4M3 ? 1 : 2);
}
// global_scale_size (same file): the f32 per-tensor scale a two-level scheme stores behind its block scales.
static size_t global_size(const bq_scheme& s) { return s.tensor_scale ? 4 : 0; }

// What the backend accepts: the same conditions under which the reference backends panic.
// `storable`: also require what a packed device tensor needs (whole words along the last dim). The
// length formula alone (quantized_data_len) pads a ragged last dim to whole words instead.
static bq_status check_scheme(const bq_scheme& s, const size_t* shape, int rank, bool storable = true) {
  if (rank < 1 || rank > BQ_MAX_RANK) BQ_FAIL(BQ_ERR_SHAPE, "rank %d outside 1..%d", rank, BQ_MAX_RANK);
  BQ_TRY(check_shape_size(shape, rank));
  if (!value_supported(s.value))
    BQ_FAIL(BQ_ERR_UNSUPPORTED_SCHEME, "Quantization not supported for value %d (Q8S, Q4S, Q2S, Q8F, Q4F and Q2F are)", s.value);
  if (s.scale_dtype > BQ_SCALE_UE4M3)
    BQ_FAIL(BQ_ERR_UNSUPPORTED_SCHEME, "scale dtype %d is not supported (f32, f16, bf16 and ue4m3 are)", s.scale_dtype);
  if (s.level != BQ_LEVEL_TENSOR && s.level != BQ_LEVEL_BLOCK)
    BQ_FAIL(BQ_ERR_UNSUPPORTED_SCHEME, "unknown quantization level %d", s.level);
  if (s.tensor_scale > 1 || (s.tensor_scale && s.level != BQ_LEVEL_BLOCK))
    BQ_FAIL(BQ_ERR_UNSUPPORTED_SCHEME, "a per-tensor scale on top (tensor_scale = %d) goes with block scales, as f32", s.tensor_scale);
  if (s.store == BQ_STORE_NATIVE) {
    // one i8 per value, sub-byte values included (what the reference's CPU backend keeps and saves)
  } else if (s.store == BQ_STORE_PACKED_U32) {
    if (storable && shape[rank - 1] % static_cast<size_t>(num_quants(s.value)))
      BQ_FAIL(BQ_ERR_SHAPE, "Can't store in u32: last dim %zu is not a multiple of %d", shape[rank - 1],
              num_quants(s.value));
  } else {
    BQ_FAIL(BQ_ERR_UNSUPPORTED_SCHEME, "unknown store %d", s.store);
  }
  if (s.level == BQ_LEVEL_BLOCK) {
    if (s.block_rank < 1 || s.block_rank > rank)
      BQ_FAIL(BQ_ERR_SHAPE, "block of rank %d on a tensor of rank %d", s.block_rank, rank);
    size_t blk[BQ_MAX_RANK];
    block_dims(s, rank, blk);
    for (int d = 0; d < rank; ++d)
      if (blk[d] == 0 || shape[d] % blk[d])
        BQ_FAIL(BQ_ERR_SHAPE, "Tensor dim %d (%zu) must be evenly divisible by block size %zu", d, shape[d], blk[d]);
  }
  return BQ_OK;
}

long run_block(const bq_scheme& s, const size_t* shape, int rank) {
  if (s.level == BQ_LEVEL_TENSOR) return 0;
  size_t blk[BQ_MAX_RANK];
  block_dims(s, rank, blk);
  // A block is a run of the flat storage iff it is 1 on the leading dims, anything on one
  // dim d, and spans every dim after d.
  int d = 0;
  while (d < rank && blk[d] == 1) ++d;
  if (d == rank) return 1;
  size_t run = blk[d];
  for (int i = d + 1; i < rank; ++i) {
    if (blk[i] != shape[i]) return -1;
    run *= shape[i];
  }
  return static_cast<long>(run);
}

}  // namespace bq

using namespace bq;

// ================================================================================ device context
bq_status bq_device::alloc(size_t bytes, void** out, size_t* actual) {
  bytes = round_up(bytes ? bytes : 1, 512);
  {
    std::lock_guard<std::mutex> lock(mu);
    if (cache.take(bytes, out, actual)) return BQ_OK;
  }
  BQ_HIP(hipSetDevice(ordinal));
  hipError_t e = hipMalloc(out, bytes);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    BQ_TRY(trim());  // return the cache to the driver and retry once
    BQ_HIP(hipMalloc(out, bytes));
  }
  *actual = bytes;
  std::lock_guard<std::mutex> lock(mu);
  cache.note_handed_out(*out);
  return BQ_OK;
}

void bq_device::release(void* ptr, size_t bytes) {
  if (!ptr) return;
  std::lock_guard<std::mutex> lock(mu);
  // Reuse is stream ordered: everything that touched this block was enqueued on `stream`
  // before whatever the next owner enqueues. Blocks a HIP graph may still address are parked
  // with that graph instead (block_cache.hpp).
  cache.put(ptr, bytes);
}

bq_status bq_device::trim() {
  std::vector<void*> blocks, retired;
  {
    std::lock_guard<std::mutex> lock(mu);
    if (cache.capturing()) BQ_FAIL(BQ_ERR_UNSUPPORTED_OP, "bq_device_trim while the stream is being captured");
    blocks = cache.drain();
    retired = cache.take_retired();
  }
  if (blocks.empty() && retired.empty()) return BQ_OK;
  BQ_HIP(hipSetDevice(ordinal));
  BQ_HIP(hipStreamSynchronize(stream));
  for (void* p : blocks) (void)hipFree(p);
  for (void* p : retired) (void)hipFree(p);
  return BQ_OK;
}

// Called with `mu` held. A workspace that a captured graph may address is never freed while that
// graph can still be replayed: it is retired and freed once no graph is left (trim / close).
bq_status bq_device::ensure_workspace(size_t bytes) {
  if (bytes <= workspace_bytes) return BQ_OK;
  BQ_HIP(hipSetDevice(ordinal));
  if (workspace) {
    if (cache.must_retire()) {
      cache.retire(workspace);  // (no synchronisation either: the stream may be capturing)
    } else {
      BQ_HIP(hipStreamSynchronize(stream));
      (void)hipFree(workspace);
    }
    workspace = nullptr;
    workspace_bytes = 0;
  }
  bytes = round_up(bytes, 1 << 20);
  BQ_HIP(hipMalloc(&workspace, bytes));
  workspace_bytes = bytes;
  return BQ_OK;
}

// ---- dynamic LDS requests ------------------------------------------------------------------------
namespace bq {

bq_status lds_request_status(size_t bytes, size_t device_limit, const char* what) {
  if (bytes > device_limit)
    BQ_FAIL(BQ_ERR_HIP, "%s asks for %zu bytes of LDS, the device grants %zu per workgroup: launch refused",
            what ? what : "kernel", bytes, device_limit);
  return BQ_OK;
}

static size_t device_lds_limit(int ordinal) {
  static std::mutex mu;
  static size_t limits[64] = {0};
  std::lock_guard<std::mutex> lock(mu);
  if (ordinal < 0 || ordinal >= 64) return 64 * 1024;
  if (limits[ordinal] == 0) {
    int plain = 0, optin = 0;
    if (hipDeviceGetAttribute(&plain, hipDeviceAttributeMaxSharedMemoryPerBlock, ordinal) != hipSuccess) plain = 0;
    if (hipDeviceGetAttribute(&optin, hipDeviceAttributeSharedMemPerBlockOptin, ordinal) != hipSuccess) optin = 0;
    (void)hipGetLastError();
    const int best = std::max(plain, optin);
    limits[ordinal] = best > 0 ? static_cast<size_t>(best) : 64 * 1024;
  }
  return limits[ordinal];
}

bq_status configure_dynamic_lds(const void* kernel, size_t bytes, const char* what) {
  int ordinal = 0;
  BQ_HIP(hipGetDevice(&ordinal));
  BQ_TRY(lds_request_status(bytes, device_lds_limit(ordinal), what));
  static std::mutex mu;
  static std::map<std::pair<int, const void*>, size_t> raised;  // (device, kernel) -> attribute set so far
  std::lock_guard<std::mutex> lock(mu);
  size_t& have = raised[std::make_pair(ordinal, kernel)];
  if (have < bytes) {
    BQ_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes)));
    have = bytes;
  }
  return BQ_OK;
}

}  // namespace bq

static std::mutex g_devices_mu;
static bq_device* g_devices[64] = {nullptr};

extern "C" const char* bq_last_error(void) { return get_error(); }

extern "C" bq_status bq_device_count(int32_t* count) {
  BQ_NOTNULL(count);
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess) {
    // no driver / no device: that is a count of zero, not a failure
    (void)hipGetLastError();
    n = 0;
  }
  *count = n;
  return BQ_OK;
}

// Host <-> device copies. hipMemcpy from pageable memory is fast only once the runtime has the
// host pages pinned (it does that for large buffers it sees again); a fresh 256 KiB buffer takes
// 107 us and a fresh 4 MiB one 560 us. Through two pinned 2 MiB halves -- the host copies into one
// while the DMA engine drains the other -- the same copies take 22 us and 144 us, and large ones run
// at the link's 29 GB/s either way (measured with a stand-alone probe: malloc'd host buffer, one
// stream, medians of 50).
bq_status bq_device::ensure_stage() {
  if (stage[0]) return BQ_OK;
  for (int i = 0; i < 2; ++i) {
    hipError_t e = hipHostMalloc(reinterpret_cast<void**>(&stage[i]), kStageBytes, hipHostMallocDefault);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&stage_ev[i], hipEventDisableTiming);
    if (e != hipSuccess) {
      for (int j = 0; j < 2; ++j) {
        if (stage[j]) (void)hipHostFree(stage[j]);
        if (stage_ev[j]) (void)hipEventDestroy(stage_ev[j]);
        stage[j] = nullptr;
        stage_ev[j] = nullptr;
      }
      BQ_FAIL(BQ_ERR_HIP, "allocating the pinned staging buffers failed: %s", hipGetErrorString(e));
    }
  }
  return BQ_OK;
}

// Host transfers go through the shared pinned halves and wait on events: recorded into a HIP graph
// they would replay whatever the halves hold at that moment, so both are refused while the device's
// stream is being captured (the header's rule for *_from_data / *_into_data, enforced).
static bq_status refuse_while_capturing(bq_device* dev, const char* what) {
  std::lock_guard<std::mutex> lock(dev->mu);
  if (dev->cache.capturing())
    BQ_FAIL(BQ_ERR_UNSUPPORTED_OP, "%s copies through host memory and cannot be recorded into a HIP graph: make it before "
            "bq_graph_begin_capture or after bq_graph_end_capture", what);
  return BQ_OK;
}

// A word the device writes, read until it has reached `want` (sequence numbers wrap: compare the difference)
// or `budget_us` have passed. The wait is a read of host memory: no runtime call, no event.
static bool word_reached(const uint32_t* word, uint32_t want, double budget_us) {
  auto reached = [&] { return static_cast<int32_t>(__atomic_load_n(word, __ATOMIC_ACQUIRE) - want) >= 0; };
  if (reached()) return true;
  const auto t0 = std::chrono::steady_clock::now();
  for (;;) {
    for (int i = 0; i < 64; ++i) {
      if (reached()) return true;
      __builtin_ia32_pause();
    }
    if (std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count() > budget_us) return reached();
  }
}

bq_status bq_device::upload(void* dst, const void* src_host, size_t bytes) {
  BQ_TRY(refuse_while_capturing(this, "a host-to-device transfer (*_from_data)"));
  if (bytes == 0) return BQ_OK;
  std::lock_guard<std::mutex> lock(stage_mu);
  if (bytes <= kSmallUpload && small_stage && (reinterpret_cast<uintptr_t>(dst) & 15u) == 0) {
    // one of a few pinned slots (they stay in the host's cache) and a copy kernel that reports when it has
    // read the slot: 16 KiB reach the device 6 us sooner than through hipMemcpyAsync and an event
    const int slot = small_next;
    small_next = (slot + 1) % kSmallSlots;
    if (!word_reached(host_words + slot, small_issued[slot], 1000.0)) BQ_HIP(hipStreamSynchronize(stream));
    char* at = small_stage + static_cast<size_t>(slot) * kSmallUpload;
    std::memcpy(at, src_host, bytes);
    const uint32_t seq = ++small_seq;
    BQ_TRY(launch_copy_small(at, dst, bytes, false, host_words + slot, seq, stream));
    small_issued[slot] = seq;
    return BQ_OK;
  }
  BQ_TRY(ensure_stage());
  const char* src = static_cast<const char*>(src_host);
  char* to = static_cast<char*>(dst);
  for (size_t off = 0; off < bytes;) {
    const int half = stage_next;
    stage_next ^= 1;
    const size_t c = std::min(kStageBytes, bytes - off);
    if (stage_pending[half]) BQ_HIP(hipEventSynchronize(stage_ev[half]));  // its previous chunk has left the buffer
    std::memcpy(stage[half], src + off, c);
    BQ_HIP(hipMemcpyAsync(to + off, stage[half], c, hipMemcpyHostToDevice, stream));
    BQ_HIP(hipEventRecord(stage_ev[half], stream));
    stage_pending[half] = true;
    off += c;
  }
  // (no synchronisation: the caller's buffer has been read, and whatever uses `dst` next is queued
  // on the same stream behind the transfer)
  return BQ_OK;
}

bq_status bq_device::download(void* dst_host, const void* src, size_t bytes) {
  BQ_TRY(refuse_while_capturing(this, "a device-to-host transfer (*_into_data)"));
  if (bytes == 0) {
    BQ_HIP(hipStreamSynchronize(stream));
    return BQ_OK;
  }
  std::lock_guard<std::mutex> lock(stage_mu);
  if (bytes <= kSmallUpload && small_stage && (reinterpret_cast<uintptr_t>(src) & 15u) == 0) {
    // the small uploads' slots the other way round: a copy kernel fills the slot and reports, the host reads
    // the word instead of waiting for an event
    const int slot = small_next;
    small_next = (slot + 1) % kSmallSlots;
    if (!word_reached(host_words + slot, small_issued[slot], 1000.0)) BQ_HIP(hipStreamSynchronize(stream));
    char* at = small_stage + static_cast<size_t>(slot) * kSmallUpload;
    const uint32_t seq = ++small_seq;
    BQ_TRY(launch_copy_small(src, at, bytes, true, host_words + slot, seq, stream));
    small_issued[slot] = seq;
    if (!word_reached(host_words + slot, seq, 50.0)) BQ_HIP(hipStreamSynchronize(stream));
    std::memcpy(dst_host, at, bytes);
    return BQ_OK;
  }
  BQ_TRY(ensure_stage());
  char* to = static_cast<char*>(dst_host);
  const char* from = static_cast<const char*>(src);
  // the DMA engine fills one half while the host empties the other
  size_t issued = 0, drained = 0, len[2] = {0, 0};
  auto fill = [&](int h) -> bq_status {
    const size_t c = std::min(kStageBytes, bytes - issued);
    BQ_HIP(hipMemcpyAsync(stage[h], from + issued, c, hipMemcpyDeviceToHost, stream));
    BQ_HIP(hipEventRecord(stage_ev[h], stream));
    len[h] = c;
    issued += c;
    return BQ_OK;
  };
  // (an upload still leaving a half is ahead of these transfers on the stream)
  BQ_TRY(fill(0));
  if (issued < bytes) BQ_TRY(fill(1));
  for (int h = 0; drained < bytes; h ^= 1) {
    BQ_HIP(hipEventSynchronize(stage_ev[h]));
    std::memcpy(to + drained, stage[h], len[h]);
    drained += len[h];
    if (issued < bytes) BQ_TRY(fill(h));
  }
  stage_pending[0] = stage_pending[1] = false;  // everything queued before the last transfer has finished
  return BQ_OK;
}

extern "C" bq_status bq_device_open(int32_t ordinal, bq_device** out) {
  BQ_NOTNULL(out);
  *out = nullptr;
  if (ordinal < 0 || ordinal >= 64) BQ_FAIL(BQ_ERR_SHAPE, "device ordinal %d out of range", ordinal);
  std::lock_guard<std::mutex> lock(g_devices_mu);
  if (g_devices[ordinal]) {
    *out = g_devices[ordinal];
    return BQ_OK;
  }
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess || ordinal >= n) {
    (void)hipGetLastError();
    BQ_FAIL(BQ_ERR_HIP, "no HIP device %d (%d visible): this library has no CPU path", ordinal, n);
  }
  BQ_HIP(hipSetDevice(ordinal));
  bq_device* dev = new bq_device();
  dev->ordinal = ordinal;
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, ordinal) == hipSuccess) dev->num_cus = prop.multiProcessorCount;
  dev->lds_limit = device_lds_limit(ordinal);
  {  // set-up of the allocation-free entry point: this device's address of its static scratch array
    void* scratch_ptr = nullptr;
    if (static_scratch_ptr(&scratch_ptr) != BQ_OK) {
      delete dev;
      return BQ_ERR_HIP;
    }
  }
  hipError_t se = hipStreamCreateWithFlags(&dev->stream, hipStreamNonBlocking);
  if (se == hipSuccess) se = hipHostMalloc(reinterpret_cast<void**>(&dev->small_stage), bq_device::kSmallSlots * bq_device::kSmallUpload, hipHostMallocDefault);
  if (se == hipSuccess) se = hipHostMalloc(reinterpret_cast<void**>(&dev->host_words), 64, hipHostMallocDefault);
  if (se == hipSuccess) {
    // The sequence numbers start 256 short of the 32-bit wrap, so that every process that makes a few
    // hundred calls goes through it (a server that waits every few microseconds gets there in hours).
    constexpr uint32_t kFirst = 0xFFFFFF00u;
    for (int i = 0; i < 16; ++i) dev->host_words[i] = kFirst;
    for (int i = 0; i < bq_device::kSmallSlots; ++i) dev->small_issued[i] = kFirst;
    dev->small_seq = dev->sync_seq = kFirst;
  }
  // the ticket counters of the single-launch split-K sum: zero from here on, every launch leaves them so
  if (se == hipSuccess) se = hipMalloc(reinterpret_cast<void**>(&dev->tickets), kTicketBytes);
  if (se == hipSuccess) se = hipMemset(dev->tickets, 0, kTicketBytes);
  if (se == hipSuccess) se = hipDeviceSynchronize();
  if (se == hipSuccess) se = hipEventCreate(&dev->ev_start);
  if (se == hipSuccess) se = hipEventCreate(&dev->ev_stop);
  if (se != hipSuccess) {
    if (dev->small_stage) (void)hipHostFree(dev->small_stage);
    if (dev->host_words) (void)hipHostFree(dev->host_words);
    delete dev;
    BQ_FAIL(BQ_ERR_HIP, "creating the device stream/events failed: %s", hipGetErrorString(se));
  }
  g_devices[ordinal] = dev;
  *out = dev;
  return BQ_OK;
}

extern "C" bq_status bq_device_close(bq_device* dev) {
  BQ_NOTNULL(dev);
  std::lock_guard<std::mutex> lock(g_devices_mu);
  BQ_HIP(hipSetDevice(dev->ordinal));
  BQ_HIP(hipStreamSynchronize(dev->stream));
  BQ_TRY(dev->trim());
  if (dev->workspace) (void)hipFree(dev->workspace);
  if (dev->tickets) (void)hipFree(dev->tickets);
  if (dev->validate_cells) (void)hipFree(dev->validate_cells);
  for (int i = 0; i < 2; ++i) {
    if (dev->stage[i]) (void)hipHostFree(dev->stage[i]);
    if (dev->stage_ev[i]) (void)hipEventDestroy(dev->stage_ev[i]);
  }
  if (dev->small_stage) (void)hipHostFree(dev->small_stage);
  if (dev->host_words) (void)hipHostFree(dev->host_words);
  (void)hipEventDestroy(dev->ev_start);
  (void)hipEventDestroy(dev->ev_stop);
  (void)hipStreamDestroy(dev->stream);
  g_devices[dev->ordinal] = nullptr;
  delete dev;
  return BQ_OK;
}

// hipStreamSynchronize behind one short kernel returns 10.8 us after the launch on this part; a kernel that
// writes a pinned word which the host reads is seen after 6.0 us, and behind another kernel after 8.4 us. So a
// wait first queues that kernel and reads the word for a short while -- the stream is in order, the word
// arrives when everything before it has finished -- and only then blocks in the runtime, which is also
// where a failed kernel reports its error (the word of a stream that has faulted never arrives).
bq_status bq_device::wait_idle() {
  bool capturing;
  {
    std::lock_guard<std::mutex> lock(mu);
    capturing = cache.capturing();
  }
  if (host_words && !capturing) {
    // (asking the runtime first whether the stream is idle, hipStreamQuery, costs a busy stream 13 us: not done;
    // a wait on an idle stream therefore takes the 6 us of the kernel too)
    uint32_t want = 0;
    bq_status rc;
    {
      std::lock_guard<std::mutex> lock(sync_mu);
      want = ++sync_seq;
      rc = launch_host_word(host_words + kSmallSlots, want, stream);
    }
    if (rc == BQ_OK && word_reached(host_words + kSmallSlots, want, 50.0)) return BQ_OK;
  }
  BQ_HIP(hipStreamSynchronize(stream));
  return BQ_OK;
}

extern "C" bq_status bq_device_sync(bq_device* dev) {
  BQ_NOTNULL(dev);
  return dev->wait_idle();
}

extern "C" void* bq_device_stream(bq_device* dev) { return dev ? dev->stream : nullptr; }

extern "C" bq_status bq_device_trim(bq_device* dev) {
  BQ_NOTNULL(dev);
  return dev->trim();
}

extern "C" bq_status bq_device_set_validate(bq_device* dev, int32_t on) {
  BQ_NOTNULL(dev);
  dev->validate.store(on != 0);
  return BQ_OK;
}

extern "C" bq_status bq_device_set_f32_matmul_exact(bq_device* dev, int32_t on) {
  BQ_NOTNULL(dev);
  dev->f32_matmul_exact.store(on != 0);
  return BQ_OK;
}

extern "C" bq_status bqk_lds_request_status(size_t bytes, size_t device_limit) {
  return lds_request_status(bytes, device_limit, "kernel");
}

extern "C" bq_status bq_timer_start(bq_device* dev) {
  BQ_NOTNULL(dev);
  BQ_HIP(hipEventRecord(dev->ev_start, dev->stream));
  return BQ_OK;
}

extern "C" bq_status bq_timer_stop(bq_device* dev, float* elapsed_ms) {
  BQ_NOTNULL(dev);
  BQ_NOTNULL(elapsed_ms);
  BQ_HIP(hipEventRecord(dev->ev_stop, dev->stream));
  BQ_HIP(hipEventSynchronize(dev->ev_stop));
  BQ_HIP(hipEventElapsedTime(elapsed_ms, dev->ev_start, dev->ev_stop));
  return BQ_OK;
}

// ================================================================================ HIP graphs
struct bq_graph {
  bq_device* dev = nullptr;
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  bq::GraphBlocks blocks;  // allocations the captured kernels address (block_cache.hpp)
};

extern "C" bq_status bq_graph_begin_capture(bq_device* dev) {
  BQ_NOTNULL(dev);
  {
    std::lock_guard<std::mutex> lock(dev->mu);
    if (dev->cache.capturing()) BQ_FAIL(BQ_ERR_UNSUPPORTED_OP, "a capture is already open on this device");
  }
  // relaxed: an allocation-cache miss inside the captured region may still call hipMalloc
  BQ_HIP(hipStreamBeginCapture(dev->stream, hipStreamCaptureModeRelaxed));
  std::lock_guard<std::mutex> lock(dev->mu);
  dev->cache.begin_capture();
  return BQ_OK;
}

extern "C" bq_status bq_graph_end_capture(bq_device* dev, bq_graph** out) {
  BQ_NOTNULL(dev);
  BQ_NOTNULL(out);
  *out = nullptr;
  hipGraph_t graph = nullptr;
  hipError_t e = hipStreamEndCapture(dev->stream, &graph);
  hipGraphExec_t exec = nullptr;
  if (e == hipSuccess) {
    e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    if (e != hipSuccess) (void)hipGraphDestroy(graph);
  }
  if (e != hipSuccess) {
    (void)hipGetLastError();
    std::lock_guard<std::mutex> lock(dev->mu);
    dev->cache.end_capture(nullptr);
    BQ_FAIL(BQ_ERR_HIP, "ending the capture / instantiating the graph failed: %s", hipGetErrorString(e));
  }
  bq_graph* g = new bq_graph();
  g->dev = dev;
  g->graph = graph;
  g->exec = exec;
  {
    std::lock_guard<std::mutex> lock(dev->mu);
    dev->cache.end_capture(&g->blocks);
  }
  *out = g;
  return BQ_OK;
}

extern "C" bq_status bq_graph_launch(bq_graph* g) {
  BQ_NOTNULL(g);
  BQ_HIP(hipGraphLaunch(g->exec, g->dev->stream));
  return BQ_OK;
}

extern "C" bq_status bq_graph_release(bq_graph* g) {
  BQ_NOTNULL(g);
  (void)hipStreamSynchronize(g->dev->stream);  // the last replay has finished
  (void)hipGraphExecDestroy(g->exec);
  (void)hipGraphDestroy(g->graph);
  {
    std::lock_guard<std::mutex> lock(g->dev->mu);
    g->dev->cache.release_graph(&g->blocks);
  }
  delete g;
  return BQ_OK;
}

// ================================================================================ handles
static size_t dtype_size(int32_t dtype) { return dtype == BQ_BF16 ? 2 : (dtype == BQ_I64 ? 8 : 4); }

static bq_status new_float(bq_device* dev, int32_t dtype, const size_t* shape, int32_t rank,
                           bq_tensor** out) {
  // (the same dense row-major layout carries the i32 / i64 index tensors of q_select, q_gather, q_argmax)
  if (dtype != BQ_F32 && dtype != BQ_BF16 && dtype != BQ_I32 && dtype != BQ_I64) BQ_FAIL(BQ_ERR_DTYPE, "dtype must be f32, bf16, i32 or i64");
  if (rank < 1 || rank > BQ_MAX_RANK) BQ_FAIL(BQ_ERR_SHAPE, "rank %d outside 1..%d", rank, BQ_MAX_RANK);
  BQ_TRY(check_shape_size(shape, rank));
  bq_tensor* t = new bq_tensor();
  t->dev = dev;
  t->dtype = dtype;
  t->rank = rank;
  for (int d = 0; d < rank; ++d) t->shape[d] = shape[d];
  t->value_bytes = t->numel() * dtype_size(dtype);
  bq_status s = dev->alloc(round_up(t->value_bytes ? t->value_bytes : 1, 512), &t->data, &t->alloc_bytes);
  if (s != BQ_OK) {
    delete t;
    return s;
  }
  *out = t;
  return BQ_OK;
}

// values region, then (256-byte aligned) the scales; BQ_ABSMAX_CELLS spare words behind the scales
// are the absmax cells of a per-tensor quantize_dynamic.
static bq_status new_quantized(bq_device* dev, const bq_scheme& scheme, const size_t* shape,
                               int32_t rank, bq_tensor** out) {
  BQ_TRY(check_scheme(scheme, shape, rank));
  bq_tensor* t = new bq_tensor();
  t->dev = dev;
  t->dtype = BQ_QFLOAT;
  t->rank = rank;
  for (int d = 0; d < rank; ++d) t->shape[d] = shape[d];
  t->scheme = scheme;
  t->value_bytes = value_bytes(scheme, shape, rank);
  t->num_scales = num_params(scheme, shape, rank);
  t->scales_offset = round_up(t->value_bytes, 256);
  size_t bytes = t->scales_offset + 4 * (t->num_scales + 1 + BQ_ABSMAX_CELLS);
  if (scheme.tensor_scale) {
    // two-level: the kernels read global * s_block at scales(); what the blob stores -- the
    // per-tensor scale, then the block scales -- is kept beside them
    t->wire_offset = round_up(bytes, 256);
    bytes = t->wire_offset + 4 * (1 + t->num_scales);
  }
  bq_status s = dev->alloc(round_up(bytes, 512), &t->data, &t->alloc_bytes);
  if (s != BQ_OK) {
    delete t;
    return s;
  }
  *out = t;
  return BQ_OK;
}

extern "C" bq_status bq_tensor_retain(bq_tensor* t) {
  BQ_NOTNULL(t);
  t->refs.fetch_add(1);
  return BQ_OK;
}

extern "C" bq_status bq_tensor_release(bq_tensor* t) {
  BQ_NOTNULL(t);
  if (t->refs.fetch_sub(1) == 1) {
    if (t->base) {
      bq_tensor_release(t->base);
    } else if (t->alloc_bytes) {
      t->dev->release(t->data, t->alloc_bytes);
    }
    delete t;
  }
  return BQ_OK;
}

extern "C" int32_t bq_tensor_rank(const bq_tensor* t) { return t ? t->rank : -1; }
extern "C" int32_t bq_tensor_dtype(const bq_tensor* t) { return t ? t->dtype : -1; }
extern "C" bq_status bq_tensor_shape(const bq_tensor* t, size_t* shape_out) {
  BQ_NOTNULL(t);
  BQ_NOTNULL(shape_out);
  for (int d = 0; d < t->rank; ++d) shape_out[d] = t->shape[d];
  return BQ_OK;
}
extern "C" bq_status bq_tensor_scheme(const bq_tensor* t, bq_scheme* out) {
  BQ_NOTNULL(t);
  BQ_NOTNULL(out);
  if (t->dtype != BQ_QFLOAT) BQ_FAIL(BQ_ERR_DTYPE, "not a quantized tensor");
  *out = t->scheme;
  return BQ_OK;
}
extern "C" void* bq_tensor_data_ptr(const bq_tensor* t) { return t ? t->data : nullptr; }
extern "C" void* bq_tensor_scales_ptr(const bq_tensor* t) {
  return (t && t->dtype == BQ_QFLOAT) ? static_cast<void*>(t->scales()) : nullptr;
}
extern "C" size_t bq_tensor_num_scales(const bq_tensor* t) { return t ? t->num_scales : 0; }

// ================================================================================ float tensors
extern "C" bq_status bq_float_empty(bq_device* dev, int32_t dtype, const size_t* shape, int32_t rank,
                                    bq_tensor** out) {
  if (dtype != BQ_F32 && dtype != BQ_BF16) BQ_FAIL(BQ_ERR_DTYPE, "float dtype must be f32 or bf16");
  BQ_NOTNULL(dev);
  BQ_NOTNULL(shape);
  BQ_NOTNULL(out);
  return new_float(dev, dtype, shape, rank, out);
}

static bq_status plain_from_data(bq_device* dev, const void* host, int32_t dtype, const size_t* shape, int32_t rank, bq_tensor** out);

extern "C" bq_status bq_float_from_data(bq_device* dev, const void* host, int32_t dtype,
                                        const size_t* shape, int32_t rank, bq_tensor** out) {
  if (dtype != BQ_F32 && dtype != BQ_BF16) BQ_FAIL(BQ_ERR_DTYPE, "float dtype must be f32 or bf16");
  return plain_from_data(dev, host, dtype, shape, rank, out);
}

// IntTensorOps::int_from_data / int_into_data for the index tensors the quantized ops take and return.
extern "C" bq_status bq_int_from_data(bq_device* dev, const void* host, int32_t dtype, const size_t* shape, int32_t rank,
                                      bq_tensor** out) {
  if (dtype != BQ_I32 && dtype != BQ_I64) BQ_FAIL(BQ_ERR_DTYPE, "int dtype must be i32 or i64");
  return plain_from_data(dev, host, dtype, shape, rank, out);
}

extern "C" bq_status bq_int_into_data(const bq_tensor* t, void* host, size_t capacity_bytes) {
  BQ_NOTNULL(t);
  if (t->dtype != BQ_I32 && t->dtype != BQ_I64) BQ_FAIL(BQ_ERR_DTYPE, "bq_int_into_data takes an i32 or i64 tensor");
  return bq_float_into_data(t, host, capacity_bytes);
}

static bq_status plain_from_data(bq_device* dev, const void* host, int32_t dtype, const size_t* shape, int32_t rank, bq_tensor** out) {
  BQ_NOTNULL(dev);
  BQ_NOTNULL(shape);
  BQ_NOTNULL(out);
  bq_tensor* t = nullptr;
  BQ_TRY(new_float(dev, dtype, shape, rank, &t));
  if (t->value_bytes) {
    if (!host) {
      bq_tensor_release(t);
      BQ_FAIL(BQ_ERR_NULL, "bq_float_from_data: null host buffer");
    }
    const bq_status rc = dev->upload(t->data, host, t->value_bytes);  // (the host buffer is only borrowed: read before this returns)
    if (rc != BQ_OK) {
      bq_tensor_release(t);
      return rc;
    }
  }
  *out = t;
  return BQ_OK;
}

extern "C" bq_status bq_float_into_data(const bq_tensor* t, void* host, size_t capacity_bytes) {
  BQ_NOTNULL(t);
  if (t->dtype == BQ_QFLOAT) BQ_FAIL(BQ_ERR_DTYPE, "bq_float_into_data on a quantized tensor");
  if (capacity_bytes < t->value_bytes)
    BQ_FAIL(BQ_ERR_SIZE, "host buffer of %zu bytes for a tensor of %zu", capacity_bytes, t->value_bytes);
  if (t->value_bytes) BQ_NOTNULL(host);
  return t->dev->download(host, t->data, t->value_bytes);
}

extern "C" bq_status bq_float_from_device_ptr(bq_device* dev, void* device_ptr, int32_t dtype,
                                              const size_t* shape, int32_t rank, bq_tensor** out) {
  BQ_NOTNULL(dev);
  BQ_NOTNULL(device_ptr);
  BQ_NOTNULL(shape);
  BQ_NOTNULL(out);
  if (dtype != BQ_F32 && dtype != BQ_BF16) BQ_FAIL(BQ_ERR_DTYPE, "float dtype must be f32 or bf16");
  if (rank < 1 || rank > BQ_MAX_RANK) BQ_FAIL(BQ_ERR_SHAPE, "rank %d outside 1..%d", rank, BQ_MAX_RANK);
  BQ_TRY(check_shape_size(shape, rank));
  bq_tensor* t = new bq_tensor();
  t->dev = dev;
  t->dtype = dtype;
  t->rank = rank;
  for (int d = 0; d < rank; ++d) t->shape[d] = shape[d];
  t->value_bytes = t->numel() * dtype_size(dtype);
  t->data = device_ptr;
  t->alloc_bytes = 0;  // borrowed
  *out = t;
  return BQ_OK;
}

// ================================================================================ wire format
extern "C" bq_status bq_scheme_supported(const bq_scheme* scheme) {
  BQ_NOTNULL(scheme);
  const bq_scheme& s = *scheme;
  // the shape-independent half of check_scheme: a shape of block extents satisfies the other half
  size_t shape[BQ_MAX_RANK];
  int rank = 1;
  if (s.level == BQ_LEVEL_BLOCK) {
    if (s.block_rank < 1 || s.block_rank > BQ_MAX_RANK)
      BQ_FAIL(BQ_ERR_UNSUPPORTED_SCHEME, "block of rank %d (1..%d are supported)", s.block_rank, BQ_MAX_RANK);
    rank = s.block_rank;
    for (int d = 0; d < rank; ++d) shape[d] = s.block[d];
    if (s.block[rank - 1] == 0) BQ_FAIL(BQ_ERR_UNSUPPORTED_SCHEME, "a block extent of 0");
  } else {
    shape[0] = 1;
  }
  shape[rank - 1] *= 16;  // (whole packed words along the last dim for every value width)
  bq_status rc = check_scheme(s, shape, rank);
  if (rc != BQ_OK) return rc == BQ_ERR_SHAPE ? BQ_ERR_UNSUPPORTED_SCHEME : rc;
  // quantizable: normalize_scales needs block scales that f16's range holds
  if (s.tensor_scale && s.scale_dtype != BQ_SCALE_F16 && s.scale_dtype != BQ_SCALE_UE4M3)
    BQ_FAIL(BQ_ERR_UNSUPPORTED_SCHEME,
            "block scales of this dtype reach f32's range, which a per-tensor scale cannot absorb (f16 and ue4m3 block scales can)");
  return BQ_OK;
}

extern "C" bq_status bq_quantized_data_len(const bq_scheme* scheme, const size_t* shape, int32_t rank,
                                           size_t* len_out) {
  BQ_NOTNULL(scheme);
  BQ_NOTNULL(shape);
  BQ_NOTNULL(len_out);
  // (a zero block extent, a dim the block does not divide, an unknown store or level are refused
  // here; a ragged last dim is not: the formula pads it to whole words, burn-store's data_len cases)
  BQ_TRY(check_scheme(*scheme, shape, rank, false));
  *len_out = value_bytes(*scheme, shape, rank) + scale_size(*scheme) * num_params(*scheme, shape, rank) +
             global_size(*scheme);
  return BQ_OK;
}

extern "C" bq_status bq_q_from_data(bq_device* dev, const uint8_t* bytes, size_t len,
                                    const size_t* shape, int32_t rank, const bq_scheme* scheme,
                                    bq_tensor** out) {
  BQ_NOTNULL(dev);
  BQ_NOTNULL(shape);
  BQ_NOTNULL(scheme);
  BQ_NOTNULL(out);
  bq_tensor* t = nullptr;
  BQ_TRY(new_quantized(dev, *scheme, shape, rank, &t));
  const size_t ssz = scale_size(*scheme);
  const size_t need = t->value_bytes + ssz * t->num_scales + global_size(*scheme);
  if (len != need) {
    bq_tensor_release(t);
    BQ_FAIL(BQ_ERR_SIZE, "quantized tensor data is %zu bytes, its scheme and shape need %zu", len, need);
  }
  if (!bytes) {
    bq_tensor_release(t);
    BQ_FAIL(BQ_ERR_NULL, "bq_q_from_data: null bytes");
  }
  bq_status rc = BQ_OK;
  const bool two_level = scheme->tensor_scale != 0;
  // two-level: the block scales go to the stored copy, the kernels' scales are derived below
  float* const scales_dst = two_level ? t->wire_scales() : t->scales();
  // (every transfer is a bq_device::upload: it has read the host bytes when it returns, is ordered on
  // the stream like a kernel, and refuses to run inside a graph capture)
  if (!two_level && ssz == 4 && t->scales_offset == t->value_bytes) {
    // the device layout is the wire layout (values of a multiple of 256 bytes, f32 scales right
    // behind them): the whole blob arrives with one copy
    rc = dev->upload(t->data, bytes, need);
  } else {
    rc = dev->upload(t->data, bytes, t->value_bytes);
    if (rc == BQ_OK && ssz == 4) {
      rc = dev->upload(scales_dst, bytes + t->value_bytes, 4 * t->num_scales);
    } else if (rc == BQ_OK) {
      // 2- and 1-byte scales: staged in a device block, widened (exactly) to the f32 the kernels read
      void* stage = nullptr;
      size_t stage_bytes = 0;
      rc = dev->alloc(ssz * t->num_scales, &stage, &stage_bytes);
      if (rc == BQ_OK) {
        rc = dev->upload(stage, bytes + t->value_bytes, ssz * t->num_scales);
        if (rc == BQ_OK) rc = launch_scales_from_wire(stage, scales_dst, t->num_scales, scheme->scale_dtype, dev->stream);
        dev->release(stage, stage_bytes);  // (stream ordered: the next owner's work queues behind the kernel)
      }
    }
    if (two_level && rc == BQ_OK) {
      rc = dev->upload(t->wire_global(), bytes + t->value_bytes + ssz * t->num_scales, 4);
      if (rc == BQ_OK) rc = launch_scales_times_global(t->wire_scales(), t->wire_global(), t->num_scales, t->scales(), dev->stream);
    }
  }
  if (rc != BQ_OK) {
    bq_tensor_release(t);
    return rc;
  }
  *out = t;
  return BQ_OK;
}

extern "C" bq_status bq_q_into_data(const bq_tensor* t, uint8_t* bytes, size_t capacity, size_t* len_out) {
  BQ_NOTNULL(t);
  BQ_NOTNULL(len_out);
  if (t->dtype != BQ_QFLOAT) BQ_FAIL(BQ_ERR_DTYPE, "bq_q_into_data on a float tensor");
  const size_t ssz = scale_size(t->scheme);
  const size_t need = t->value_bytes + ssz * t->num_scales + global_size(t->scheme);
  *len_out = need;
  if (capacity < need) BQ_FAIL(BQ_ERR_SIZE, "host buffer of %zu bytes for a blob of %zu", capacity, need);
  BQ_NOTNULL(bytes);
  hipStream_t st = t->dev->stream;
  const bool two_level = t->scheme.tensor_scale != 0;
  const float* const scales_src = two_level ? t->wire_scales() : t->scales();
  if (!two_level && ssz == 4 && t->scales_offset == t->value_bytes) {  // dense on the device as on the wire: one copy
    return t->dev->download(bytes, t->data, need);
  }
  // (every transfer below goes through bq_device::download, which returns with the bytes in place and
  // refuses to run inside a graph capture; nothing is left in flight on an error return)
  BQ_TRY(t->dev->download(bytes, t->data, t->value_bytes));
  if (ssz == 4) {
    BQ_TRY(t->dev->download(bytes + t->value_bytes, scales_src, 4 * t->num_scales));
  } else {
    void* stage = nullptr;
    size_t stage_bytes = 0;
    BQ_TRY(t->dev->alloc(ssz * t->num_scales, &stage, &stage_bytes));
    bq_status rc = launch_scales_to_wire(scales_src, stage, t->num_scales, t->scheme.scale_dtype, st);
    if (rc == BQ_OK) rc = t->dev->download(bytes + t->value_bytes, stage, ssz * t->num_scales);
    t->dev->release(stage, stage_bytes);
    if (rc != BQ_OK) return rc;
  }
  if (two_level)  // the per-tensor scale comes last
    BQ_TRY(t->dev->download(bytes + t->value_bytes + ssz * t->num_scales, t->wire_global(), 4));
  return BQ_OK;
}

// ================================================================================ quantize
// Validate mode (bq_device_set_validate): the reference panics when a quotient x / scale is NaN
// (`Q::from(..).unwrap()`, crates/burn-ndarray/src/ops/quantization.rs:128-133). That happens for a
// NaN input, a NaN scale, and inf / inf: an infinite input against an infinite scale, which is every
// infinite input of a quantize_dynamic (its own range makes the scale infinite). The inputs are
// counted on the device and the call fails before anything is quantized. (With given scales an
// infinite input and an infinite scale anywhere are refused together, also when they belong to
// different blocks.) Synchronises the stream: a debugging aid, not for captured or timed loops.
static bq_status validate_quantize_inputs(bq_device* dev, const float* x, size_t n, const float* scales,
                                          size_t n_scales) {
  {
    std::lock_guard<std::mutex> lock(dev->mu);
    if (dev->cache.capturing())
      BQ_FAIL(BQ_ERR_UNSUPPORTED_OP, "the validate mode synchronises the stream and cannot be captured");
    if (dev->validate_cells == nullptr) {
      BQ_HIP(hipSetDevice(dev->ordinal));
      BQ_HIP(hipMalloc(reinterpret_cast<void**>(&dev->validate_cells), 4 * sizeof(uint32_t)));
    }
  }
  hipStream_t st = dev->stream;
  BQ_TRY(launch_fill_u32(dev->validate_cells, 4, 0u, st));
  BQ_TRY(launch_count_nonfinite(x, n, dev->validate_cells, st));
  if (scales != nullptr) BQ_TRY(launch_count_nonfinite(scales, n_scales, dev->validate_cells + 2, st));
  uint32_t host[4] = {0, 0, 0, 0};
  BQ_HIP(hipMemcpyAsync(host, dev->validate_cells, sizeof(host), hipMemcpyDeviceToHost, st));
  BQ_HIP(hipStreamSynchronize(st));
  const bool dynamic = scales == nullptr;
  if (host[0] || host[2] || (host[1] && (dynamic || host[3])))
    BQ_FAIL(BQ_ERR_NONFINITE,
            "quantize: x / scale is NaN for some element (%u NaN and %u infinite inputs, %u NaN and %u infinite "
            "scales); the reference panics here",
            host[0], host[1], host[2], host[3]);
  return BQ_OK;
}

static bq_status quantize_pass(const bq_tensor* x, const bq_scheme* scheme, bq_tensor* q, const bq_tensor* scales,
                               const bq_tensor* global, bool dynamic, bool params_ready, int sdt);

static bq_status quantize_impl(const bq_tensor* x, const bq_scheme* scheme, const bq_tensor* scales,
                               bq_tensor** out, const bq_tensor* global = nullptr) {
  BQ_NOTNULL(x);
  BQ_NOTNULL(scheme);
  BQ_NOTNULL(out);
  if (x->dtype != BQ_F32)
    BQ_FAIL(BQ_ERR_DTYPE, "quantize takes an f32 tensor (got dtype %d)", x->dtype);
  const bool dynamic = scales == nullptr;
  const bool two_level = scheme->tensor_scale != 0;
  // (the reference's messages: QuantizedBytes::new, crates/burn-std/src/tensor/quantization.rs:259-261)
  if (!dynamic && two_level && global == nullptr) BQ_FAIL(BQ_ERR_SHAPE, "a two-level scheme requires a per-tensor scale");
  if (global != nullptr && !two_level) BQ_FAIL(BQ_ERR_SHAPE, "this scheme does not take a per-tensor scale");
  if (global != nullptr && (global->dtype != BQ_F32 || global->numel() != 1 || global->dev != x->dev))
    BQ_FAIL(BQ_ERR_SHAPE, "the per-tensor scale must be an f32 tensor of one element on the input's device");
  // (normalize_scales, crates/burn-backend/src/quantization/scheme.rs:115-118)
  if (dynamic && two_level && scheme->scale_dtype != BQ_SCALE_F16 && scheme->scale_dtype != BQ_SCALE_UE4M3)
    BQ_FAIL(BQ_ERR_UNSUPPORTED_SCHEME,
            "block scales of this dtype reach f32's range, which a per-tensor scale cannot absorb (f16 and ue4m3 block scales can)");
  bq_tensor* q = nullptr;
  BQ_TRY(new_quantized(x->dev, *scheme, x->shape, x->rank, &q));
  if (!dynamic) {
    if (scales->dtype != BQ_F32 || scales->numel() != q->num_scales || scales->dev != x->dev) {
      bq_tensor_release(q);
      BQ_FAIL(BQ_ERR_SHAPE, "scales must be an f32 tensor of %zu entries on the input's device", q->num_scales);
    }
  }
  hipStream_t st = x->dev->stream;
  const size_t n = x->numel();
  const float* xin = static_cast<const float*>(x->data);
  bq_status rc = BQ_OK;
  if (x->dev->validate.load()) {
    rc = validate_quantize_inputs(x->dev, xin, n, dynamic ? nullptr : static_cast<const float*>(scales->data),
                                  dynamic ? 0 : q->num_scales);
    if (rc != BQ_OK) {
      bq_tensor_release(q);
      return rc;
    }
  }
  // Two-level: the kernels below always see the final f32 scale of a block, global * s_block. Given
  // parameters are combined first; a dynamic call computes plain f32 block scales in a first pass
  // over x (the values it writes are overwritten), splits them, and quantizes against the products.
  const int sdt = two_level ? BQ_SCALE_F32 : scheme->scale_dtype;
  bool dynamic_pass = dynamic;
  // Run blocks with a fused kernel need no first pass: the largest block scale follows from the
  // tensor's absmax alone, and the block kernel splits each scale as it computes it.
  const long run = scheme->level == BQ_LEVEL_BLOCK ? run_block(*scheme, x->shape, x->rank) : 0;
  if (two_level && dynamic && n > 0 && fused_value(scheme->value, scheme->store) && run > 0 && run <= 512 &&
      fused_block_ok(static_cast<int>(run), scheme->value)) {
    uint32_t* cells = reinterpret_cast<uint32_t*>(q->scales() + q->num_scales);
    rc = bqk_absmax_f32(xin, n, cells, st);
    if (rc == BQ_OK) rc = launch_two_level_global(cells, scheme->value, scheme->scale_dtype, q->wire_global(), st);
    if (rc == BQ_OK)
      rc = launch_quantize_run_block_two_level(xin, n, static_cast<int>(run), q->wire_global(), q->wire_scales(), q->scales(),
                                               scheme->value, scheme->store, q->data, scheme->scale_dtype, st);
    if (rc != BQ_OK) {
      bq_tensor_release(q);
      return rc;
    }
    *out = q;
    return BQ_OK;
  }
  for (int pass = 0; pass < 2; ++pass) {
    if (pass == 1) {
      if (!(two_level && dynamic) || rc != BQ_OK || n == 0) break;
      uint32_t* cells = reinterpret_cast<uint32_t*>(q->scales() + q->num_scales);
      rc = bqk_absmax_f32(q->scales(), q->num_scales, cells, st);
      if (rc == BQ_OK)
        rc = launch_two_level_split(q->scales(), q->num_scales, cells, scheme->scale_dtype, q->wire_global(), q->wire_scales(), st);
      if (rc != BQ_OK) break;
      dynamic_pass = false;
    }
    rc = quantize_pass(x, scheme, q, scales, global, dynamic_pass, pass == 1, sdt);
  }
  if (rc != BQ_OK) {
    bq_tensor_release(q);
    return rc;
  }
  *out = q;
  return BQ_OK;
}

// One pass of quantize_impl: parameters in place (unless they already are), then the value kernels.
static bq_status quantize_pass(const bq_tensor* x, const bq_scheme* scheme, bq_tensor* q, const bq_tensor* scales,
                               const bq_tensor* global, bool dynamic, bool params_ready, int sdt) {
  hipStream_t st = x->dev->stream;
  const size_t n = x->numel();
  const float* xin = static_cast<const float*>(x->data);
  const bool two_level = scheme->tensor_scale != 0;
  bq_status rc = BQ_OK;
  do {
    if (!dynamic && !params_ready && two_level) {
      // s_block rounded up to the scale dtype, kept as stored; the block's scale is global * that
      rc = launch_round_scales(static_cast<const float*>(scales->data), q->wire_scales(), q->num_scales, scheme->scale_dtype, st);
      if (rc != BQ_OK) break;
      hipError_t e = hipMemcpyAsync(q->wire_global(), global->data, 4, hipMemcpyDeviceToDevice, st);
      if (e != hipSuccess) {
        set_error("copying the per-tensor scale failed: %s", hipGetErrorString(e));
        rc = BQ_ERR_HIP;
        break;
      }
      rc = launch_scales_times_global(q->wire_scales(), q->wire_global(), q->num_scales, q->scales(), st);
      if (rc != BQ_OK) break;
    } else if (!dynamic && !params_ready) {
      // the stored scale is the given one, rounded up to the scale dtype first (scale_to_dtype,
      // crates/burn-ndarray/src/ops/qtensor.rs:90-95): the values are divided by what is stored
      if (sdt == BQ_SCALE_F32) {
        hipError_t e = hipMemcpyAsync(q->scales(), scales->data, 4 * q->num_scales, hipMemcpyDeviceToDevice, st);
        if (e != hipSuccess) {
          set_error("copying scales failed: %s", hipGetErrorString(e));
          rc = BQ_ERR_HIP;
          break;
        }
      } else {
        rc = launch_round_scales(static_cast<const float*>(scales->data), q->scales(), q->num_scales, sdt, st);
        if (rc != BQ_OK) break;
      }
    }
    if (n == 0) break;
    const long run = run_block(*scheme, x->shape, x->rank);
    if (!fused_value(scheme->value, scheme->store)) {
      // Q2S, and 4-bit values stored natively: the general kernels (any block shape). Per tensor, the range comes from the absmax
      // pass like every per-tensor quantize_dynamic.
      const bool per_tensor = scheme->level == BQ_LEVEL_TENSOR;
      if (per_tensor && dynamic) {
        uint32_t* cells = reinterpret_cast<uint32_t*>(q->scales() + 1);
        rc = bqk_absmax_f32(xin, n, cells, st);
        if (rc == BQ_OK) rc = launch_scale_from_cells(cells, scheme->value, sdt, q->scales(), st);
        if (rc != BQ_OK) break;
      }
      if (per_tensor && value_bits(scheme->value) == 2 && scheme->store == BQ_STORE_PACKED_U32 &&
          (reinterpret_cast<uintptr_t>(xin) & 15u) == 0) {
        // a per-tensor 2-bit quantize (a BitNet weight): the streaming per-tensor kernel, 16 values per word
        rc = launch_quantize_per_tensor(xin, n, q->scales(), false, nullptr, scheme->value, scheme->store, q->data, sdt, st);
        break;
      }
      size_t blk[BQ_MAX_RANK];
      block_dims(*scheme, x->rank, blk);
      rc = launch_quantize_rect(xin, x->shape, x->rank, per_tensor ? nullptr : blk, scheme->value, scheme->store,
                                dynamic && !per_tensor, sdt, q->data, q->scales(), st);
    } else if (scheme->level == BQ_LEVEL_TENSOR) {
      if (dynamic) {
        bool done = false;
        rc = launch_quantize_per_tensor_small(xin, n, q->scales(), scheme->value, scheme->store, q->data, sdt, st, &done);
        if (rc != BQ_OK || done) break;
        // the absmax cells sit right behind the scale (the first pass writes every cell)
        uint32_t* cells = reinterpret_cast<uint32_t*>(q->scales() + 1);
        rc = bqk_absmax_f32(xin, n, cells, st);
        if (rc != BQ_OK) break;
        rc = launch_quantize_per_tensor(xin, n, reinterpret_cast<const float*>(cells), true, q->scales(), scheme->value,
                                        scheme->store, q->data, sdt, st);
      } else {
        rc = launch_quantize_per_tensor(xin, n, q->scales(), false, nullptr, scheme->value, scheme->store, q->data, sdt, st);
      }
    } else if (run > 0 && fused_block_ok(static_cast<int>(run), scheme->value) && run <= 512) {
      rc = launch_quantize_run_block(xin, n, static_cast<int>(run), dynamic ? nullptr : q->scales(), q->scales(),
                                     scheme->value, scheme->store, q->data, sdt, st);
    } else {
      size_t blk[BQ_MAX_RANK];
      block_dims(*scheme, x->rank, blk);
      rc = launch_quantize_rect(xin, x->shape, x->rank, blk, scheme->value, scheme->store, dynamic, sdt,
                                q->data, q->scales(), st);
    }
  } while (false);
  return rc;
}

extern "C" bq_status bq_quantize(const bq_tensor* x, const bq_scheme* scheme, const bq_tensor* scales,
                                 bq_tensor** out) {
  BQ_NOTNULL(scales);
  return quantize_impl(x, scheme, scales, out);
}

extern "C" bq_status bq_quantize_two_level(const bq_tensor* x, const bq_scheme* scheme, const bq_tensor* scales,
                                           const bq_tensor* global, bq_tensor** out) {
  BQ_NOTNULL(scales);
  BQ_NOTNULL(global);
  return quantize_impl(x, scheme, scales, out, global);
}

extern "C" bq_status bq_quantize_dynamic(const bq_tensor* x, const bq_scheme* scheme, bq_tensor** out) {
  return quantize_impl(x, scheme, nullptr, out);
}

// compute_range under Calibration::AbsMean (crates/burn-backend/src/quantization/scheme.rs:57-69).
static bq_status abs_mean_impl(const bq_tensor* x, const bq_scheme* scheme, bq_tensor** gamma_out) {
  BQ_NOTNULL(x);
  BQ_NOTNULL(scheme);
  BQ_NOTNULL(gamma_out);
  *gamma_out = nullptr;
  if (x->dtype != BQ_F32) BQ_FAIL(BQ_ERR_DTYPE, "compute_range takes an f32 tensor (got dtype %d)", x->dtype);
  // (the reference's assert, scheme.rs:59-63)
  if (scheme->tensor_scale != 0)
    BQ_FAIL(BQ_ERR_UNSUPPORTED_SCHEME,
            "AbsMean calibration has no two-level form: gamma is a mean over the whole tensor or block, which a "
            "per-tensor scale cannot decompose");
  BQ_TRY(check_scheme(*scheme, x->shape, x->rank, false));
  const bool per_tensor = scheme->level == BQ_LEVEL_TENSOR;
  size_t blk[BQ_MAX_RANK], pshape[BQ_MAX_RANK];
  int prank = 1;
  pshape[0] = 1;
  if (!per_tensor) {
    block_dims(*scheme, x->rank, blk);
    prank = x->rank;
    for (int i = 0; i < x->rank; ++i) pshape[i] = x->shape[i] / blk[i];
  }
  bq_tensor* gamma = nullptr;
  BQ_TRY(new_float(x->dev, BQ_F32, pshape, prank, &gamma));
  bq_tensor* cells = nullptr;
  bq_status rc = BQ_OK;
  if (per_tensor) {
    const size_t ncells = BQ_ABSMAX_CELLS;
    rc = new_float(x->dev, BQ_F32, &ncells, 1, &cells);
  }
  if (rc == BQ_OK && x->numel() == 0) rc = launch_fill_u32(static_cast<uint32_t*>(gamma->data), gamma->numel(), 0u, x->dev->stream);
  if (rc == BQ_OK)
    rc = launch_abs_mean(static_cast<const float*>(x->data), x->shape, x->rank, per_tensor ? nullptr : blk,
                         cells ? static_cast<float*>(cells->data) : nullptr, static_cast<float*>(gamma->data), x->dev->stream);
  if (cells) bq_tensor_release(cells);
  if (rc != BQ_OK) {
    bq_tensor_release(gamma);
    return rc;
  }
  *gamma_out = gamma;
  return BQ_OK;
}

extern "C" bq_status bq_compute_range_abs_mean(const bq_tensor* x, const bq_scheme* scheme, bq_tensor** gamma_out) {
  return abs_mean_impl(x, scheme, gamma_out);
}

// The Quantizer's three steps (crates/burn-core/src/module/quantize.rs:47-49) with Calibration::AbsMean,
// all on the device: gamma, scale = (2 gamma) / (b - a), quantize against it.
extern "C" bq_status bq_quantize_abs_mean(const bq_tensor* x, const bq_scheme* scheme, bq_tensor** out) {
  BQ_NOTNULL(out);
  *out = nullptr;
  bq_tensor* gamma = nullptr;
  BQ_TRY(abs_mean_impl(x, scheme, &gamma));
  bq_status rc = launch_scales_from_range(static_cast<const float*>(gamma->data), gamma->numel(), scheme->value,
                                          static_cast<float*>(gamma->data), x->dev->stream);
  if (rc == BQ_OK) rc = quantize_impl(x, scheme, gamma, out);
  bq_tensor_release(gamma);
  return rc;
}

// ================================================================================ dequantize
extern "C" bq_status bq_dequantize(const bq_tensor* q, int32_t float_dtype, bq_tensor** out) {
  BQ_NOTNULL(q);
  BQ_NOTNULL(out);
  if (q->dtype != BQ_QFLOAT) BQ_FAIL(BQ_ERR_DTYPE, "dequantize takes a quantized tensor");
  bq_tensor* f = nullptr;
  BQ_TRY(new_float(q->dev, float_dtype, q->shape, q->rank, &f));
  hipStream_t st = q->dev->stream;
  const size_t n = q->numel();
  bq_status rc = BQ_OK;
  const long run = run_block(q->scheme, q->shape, q->rank);
  const int qv = stored_value(q->scheme.value, q->scheme.store);  // (natively stored values read as 8-bit ones)
  if (n == 0) {
  } else if (value_known(qv) && run >= 0 &&
             (run == 0 || (fused_block_ok(static_cast<int>(run), qv) && run <= 512))) {
    rc = bqk_dequantize(q->data, n, static_cast<int32_t>(run), q->scales(), qv,
                        q->scheme.store, float_dtype, f->data, st);
  } else {
    size_t blk[BQ_MAX_RANK];
    block_dims(q->scheme, q->rank, blk);
    rc = launch_dequantize_rect(q->data, q->shape, q->rank, q->scheme.level == BQ_LEVEL_TENSOR ? nullptr : blk,
                                q->scales(), qv, q->scheme.store, float_dtype, f->data, st);
  }
  if (rc != BQ_OK) {
    bq_tensor_release(f);
    return rc;
  }
  *out = f;
  return BQ_OK;
}

// ================================================================================ matmul
struct MatmulDims {
  size_t m, k, n;
  int rank;
  size_t out_shape[BQ_MAX_RANK];
  size_t batches;                 // product of the broadcast batch dims
  size_t lhs_batch_stride_sel[BQ_MAX_RANK];  // 0 where lhs broadcasts
  size_t rhs_batch_stride_sel[BQ_MAX_RANK];
};

// burn's matmul contract: equal rank >= 2, inner dims agree, batch dims broadcast
// (crates/burn-tensor/src/tensor/api/numeric.rs:817, check in ops).
static bq_status matmul_dims(const bq_tensor* lhs, const bq_tensor* rhs, MatmulDims* d) {
  if (lhs->rank != rhs->rank || lhs->rank < 2)
    BQ_FAIL(BQ_ERR_SHAPE, "matmul operands must have the same rank >= 2 (%d vs %d)", lhs->rank, rhs->rank);
  const int r = lhs->rank;
  d->rank = r;
  d->m = lhs->shape[r - 2];
  d->k = lhs->shape[r - 1];
  d->n = rhs->shape[r - 1];
  if (rhs->shape[r - 2] != d->k)
    BQ_FAIL(BQ_ERR_SHAPE, "matmul inner dimensions differ: %zu vs %zu", d->k, rhs->shape[r - 2]);
  d->batches = 1;
  size_t ls = 1, rs = 1;
  for (int i = r - 3; i >= 0; --i) {
    size_t a = lhs->shape[i], b = rhs->shape[i];
    if (a != b && a != 1 && b != 1) BQ_FAIL(BQ_ERR_SHAPE, "matmul batch dims %zu and %zu do not broadcast", a, b);
    d->out_shape[i] = std::max(a, b);
    d->lhs_batch_stride_sel[i] = (a == 1 && b != 1) ? 0 : ls;
    d->rhs_batch_stride_sel[i] = (b == 1 && a != 1) ? 0 : rs;
    ls *= a;
    rs *= b;
    d->batches *= d->out_shape[i];
  }
  d->out_shape[r - 2] = d->m;
  d->out_shape[r - 1] = d->n;
  return BQ_OK;
}

static void batch_offsets(const MatmulDims& d, size_t b, size_t* lhs_b, size_t* rhs_b) {
  size_t l = 0, r = 0;
  for (int i = d.rank - 3; i >= 0; --i) {
    size_t c = b % d.out_shape[i];
    b /= d.out_shape[i];
    l += c * d.lhs_batch_stride_sel[i];
    r += c * d.rhs_batch_stride_sel[i];
  }
  *lhs_b = l;
  *rhs_b = r;
}

extern "C" bq_status bq_float_matmul(const bq_tensor* lhs, const bq_tensor* rhs, bq_tensor** out) {
  BQ_NOTNULL(lhs);
  BQ_NOTNULL(rhs);
  BQ_NOTNULL(out);
  auto is_float = [](const bq_tensor* t) { return t->dtype == BQ_F32 || t->dtype == BQ_BF16; };
  if (!is_float(lhs) || !is_float(rhs)) BQ_FAIL(BQ_ERR_DTYPE, "float_matmul takes float tensors");
  if (lhs->dev != rhs->dev) BQ_FAIL(BQ_ERR_DTYPE, "float_matmul operands live on different devices");
  MatmulDims d;
  BQ_TRY(matmul_dims(lhs, rhs, &d));
  bq_tensor* o = nullptr;
  BQ_TRY(new_float(lhs->dev, lhs->dtype, d.out_shape, d.rank, &o));
  const size_t ls = dtype_size(lhs->dtype), rs = dtype_size(rhs->dtype), os = dtype_size(o->dtype);
  for (size_t b = 0; b < d.batches; ++b) {
    size_t lb, rb;
    batch_offsets(d, b, &lb, &rb);
    bq_status rc = launch_float_matmul(static_cast<char*>(lhs->data) + lb * d.m * d.k * ls, lhs->dtype,
                                       static_cast<char*>(rhs->data) + rb * d.k * d.n * rs, rhs->dtype,
                                       d.m, d.k, d.n, o->dtype,
                                       static_cast<char*>(o->data) + b * d.m * d.n * os, lhs->dev->stream);
    if (rc != BQ_OK) {
      bq_tensor_release(o);
      return rc;
    }
  }
  *out = o;
  return BQ_OK;
}

// `bias` (device f32, N entries, or null) is a linear layer's: added to every row of the product.
// quantized_out (optional): the caller wants the product quantized again with *requant_scheme (Propagate). Where
// the product ends in a reduction of K slices that can quantize what it sums, *quantized_out receives that
// tensor and *out stays null; otherwise *quantized_out stays null and *out is the float product as usual.
static bq_status q_matmul_impl(const bq_tensor* lhs, const bq_tensor* rhs, int32_t out_dtype_req,
                               const float* bias, bq_tensor** out, bq_tensor** quantized_out = nullptr,
                               const bq_scheme* requant_scheme = nullptr) {
  BQ_NOTNULL(lhs);
  BQ_NOTNULL(rhs);
  BQ_NOTNULL(out);
  const bool lq = lhs->dtype == BQ_QFLOAT, rq = rhs->dtype == BQ_QFLOAT;
  if (!lq && !rq) BQ_FAIL(BQ_ERR_DTYPE, "q_matmul needs at least one quantized operand");
  if ((!lq && lhs->dtype != BQ_F32 && lhs->dtype != BQ_BF16) || (!rq && rhs->dtype != BQ_F32 && rhs->dtype != BQ_BF16))
    BQ_FAIL(BQ_ERR_DTYPE, "q_matmul: the operand that is not quantized must be f32 or bf16");
  // dtype any dequantization targets: the float operand's, else f32 (qtensor.rs:507-512)
  const int32_t target = !lq ? lhs->dtype : (!rq ? rhs->dtype : BQ_F32);
  const int32_t out_dtype = out_dtype_req >= 0 ? out_dtype_req : target;
  if (out_dtype != BQ_F32 && out_dtype != BQ_BF16) BQ_FAIL(BQ_ERR_DTYPE, "out dtype must be f32 or bf16");
  MatmulDims d;
  BQ_TRY(matmul_dims(lhs, rhs, &d));
  bq_device* dev = lhs->dev;
  if (rhs->dev != dev) BQ_FAIL(BQ_ERR_DTYPE, "q_matmul operands live on different devices (%d and %d)", dev->ordinal, rhs->dev->ordinal);
  hipStream_t st = dev->stream;

  // Fused path: float lhs x quantized rhs whose scales are per tensor or runs along N.
  // Ternary fast path (crates/burn-ndarray/src/ops/qtensor.rs:442-517): f32 activations times a
  // per-tensor Q2S 2-D weight, no bias, f32 out. Every other Q2S product dequantizes first.
  if (!lq && rq && rhs->scheme.value == BQ_Q2S && rhs->scheme.store == BQ_STORE_PACKED_U32 &&
      rhs->scheme.level == BQ_LEVEL_TENSOR && lhs->dtype == BQ_F32 && out_dtype == BQ_F32 && rhs->rank == 2 && d.n % 16 == 0) {
    bq_tensor* o = nullptr;
    BQ_TRY(new_float(dev, BQ_F32, d.out_shape, d.rank, &o));
    bq_status rc = BQ_OK;
    if (!dev->f32_matmul_exact.load() && ternary_mfma_ok(d.m, d.k, d.n)) {
      // the same sums on the matrix cores, in another order (a fraction of the time; within 1e-5 of
      // the largest output). bq_device_set_f32_matmul_exact keeps the reference's order.
      std::unique_lock<std::mutex> lock(dev->mu);  // the split-K workspace is shared by the calls on this device
      rc = dev->ensure_workspace(ternary_workspace(d.m, d.k, d.n));
      unsigned slices = 0;
      if (rc == BQ_OK)
        rc = launch_ternary_mfma(static_cast<const float*>(lhs->data), static_cast<const uint32_t*>(rhs->data), rhs->scales(),
                                 d.m, d.k, d.n, static_cast<float*>(dev->workspace), &slices, st);
      if (rc == BQ_OK)
        rc = launch_splitk_reduce(static_cast<const float*>(dev->workspace), d.m * d.n, slices, bias, d.n, BQ_F32, o->data, st);
    } else {
      rc = launch_ternary_matmul(static_cast<const float*>(lhs->data), static_cast<const uint32_t*>(rhs->data),
                                 rhs->scales(), d.m, d.k, d.n, static_cast<float*>(o->data), st);
      if (rc == BQ_OK && bias != nullptr) rc = launch_add_bias(o->data, BQ_F32, bias, d.m, d.n, st);  // linear: matmul, then + bias
    }
    if (rc != BQ_OK) {
      bq_tensor_release(o);
      return rc;
    }
    *out = o;
    return BQ_OK;
  }
  // A quantized lhs is dequantized (to f32 when both operands are quantized, as the reference does)
  // and then multiplied like a float one: the weight stays packed and the matrix-core kernels run.
  // (More than 32 rows always take the tiled kernel, which rounds f32 activations to bf16 on the way in: there
  // the lhs is dequantized straight to bf16 -- the same bits as f32 and then bf16, one kernel and two passes
  // over the activations fewer.)
  const int32_t lhs_dtype = lq ? (target == BQ_F32 && rq && d.m > 32 ? BQ_BF16 : target) : lhs->dtype;
  long run = rq ? run_block(rhs->scheme, rhs->shape, rhs->rank) : -1;
  // (natively stored values of any width are i8s: they multiply as Q8S ones)
  const int rv = rq ? stored_value(rhs->scheme.value, rhs->scheme.store) : BQ_Q8S;
  bool fused = rq && run >= 0 && value_known(rv);
  if (fused && run > 0) {
    const size_t vpl = static_cast<size_t>(num_quants(rv));
    const size_t bw = static_cast<size_t>(run) / vpl;
    fused = (static_cast<size_t>(run) % vpl == 0) && bw && !(bw & (bw - 1)) && d.n % static_cast<size_t>(run) == 0;
  }
  if (fused && (d.n % static_cast<size_t>(num_quants(rv)))) fused = false;
  // (f32 activations, more than 32 rows: the fast kernels round to bf16; the device may ask for f32)
  // (more than 32 rows: the fast kernel rounds s * q -- and f32 activations -- to bf16; the device may ask
  // for the reference's arithmetic instead: weights dequantized to f32, f32 products)
  const bool exact = !lq && d.m > 32 && dev->f32_matmul_exact.load();
  if (fused && exact) fused = false;
  if (fused && !fused_matmul_ok(d.m, d.k, d.n, lhs_dtype, rv,
                                run > 0 ? d.n / static_cast<size_t>(run) : 0))
    fused = false;
  // The fused kernels take 16-byte aligned operands: with several batches every batch's slice of
  // the activations, the output and the weights has to start on such a boundary.
  if (fused && d.batches > 1) {
    const size_t vbytes = rhs->scheme.store == BQ_STORE_NATIVE
                              ? d.k * d.n
                              : 4 * d.k * (d.n / static_cast<size_t>(num_quants(rv)));
    if ((d.m * d.k * dtype_size(lhs_dtype)) % 16 || (d.m * d.n * dtype_size(out_dtype)) % 16 || vbytes % 16 ||
        (run > 0 && (d.k * (d.n / static_cast<size_t>(run)) * sizeof(float)) % 16))
      fused = false;
  }

  if (fused) {
    bq_tensor* lf = nullptr;
    if (lq) BQ_TRY(bq_dequantize(lhs, lhs_dtype, &lf));
    const bq_tensor* l = lq ? lf : lhs;
    bq_tensor* o = nullptr;
    bq_status rc = new_float(dev, out_dtype, d.out_shape, d.rank, &o);
    if (rc != BQ_OK) {
      if (lf) bq_tensor_release(lf);
      return rc;
    }
    // Propagate with a scheme of 32 or 64 columns per scale along the last dim (one level): the reduction of the
    // K slices, where the product has one, writes the quantized tensor
    RequantOut requant;
    bq_tensor* qt = nullptr;
    // (not in validate mode: quantize_dynamic then inspects the float product first)
    if (quantized_out != nullptr && requant_scheme != nullptr && d.batches == 1 && !dev->validate.load() &&
        requant_scheme->level == BQ_LEVEL_BLOCK &&
        !requant_scheme->tensor_scale && fused_value(requant_scheme->value, requant_scheme->store)) {
      const long out_run = run_block(*requant_scheme, d.out_shape, d.rank);
      if ((out_run == 32 || out_run == 64) && new_quantized(dev, *requant_scheme, d.out_shape, d.rank, &qt) == BQ_OK) {
        requant.value = requant_scheme->value;
        requant.store = requant_scheme->store;
        requant.block = static_cast<int>(out_run);
        requant.sdt = requant_scheme->scale_dtype;
        requant.from_bf16 = out_dtype == BQ_BF16;
        requant.values = qt->data;
        requant.scales = qt->scales();
      }
    }
    const size_t ws = bqk_q_matmul_workspace(d.m, d.k, d.n, lhs_dtype, rv);
    std::unique_lock<std::mutex> lock(dev->mu, std::defer_lock);
    if (ws) {
      lock.lock();  // the split-K workspace is shared by the calls on this device
      rc = dev->ensure_workspace(ws);
    }
    const size_t vbytes_per_batch = rhs->scheme.store == BQ_STORE_NATIVE
                                        ? d.k * d.n
                                        : 4 * d.k * (d.n / static_cast<size_t>(num_quants(rv)));
    const size_t scales_per_batch = run > 0 ? d.k * (d.n / static_cast<size_t>(run)) : 0;
    for (size_t b = 0; b < d.batches && rc == BQ_OK; ++b) {
      size_t lb, rb;
      batch_offsets(d, b, &lb, &rb);
      // (the ticket counters are shared like the workspace: only under its lock)
      rc = q_linear_with_tickets(static_cast<char*>(l->data) + lb * d.m * d.k * dtype_size(lhs_dtype), lhs_dtype,
                                 d.m, d.k, d.n, static_cast<char*>(rhs->data) + rb * vbytes_per_batch,
                                 rhs->scales() + rb * scales_per_batch, static_cast<int32_t>(run), rv,
                                 rhs->scheme.store, bias, out_dtype,
                                 static_cast<char*>(o->data) + b * d.m * d.n * dtype_size(out_dtype), dev->workspace,
                                 dev->workspace_bytes, lock.owns_lock() ? dev->tickets : nullptr, st,
                                 qt != nullptr ? &requant : nullptr);
    }
    if (lock.owns_lock()) lock.unlock();  // (releasing a tensor takes the same mutex)
    if (lf) bq_tensor_release(lf);         // (stream-ordered: the kernels above were enqueued first)
    if (rc != BQ_OK) {
      bq_tensor_release(o);
      if (qt) bq_tensor_release(qt);
      return rc;
    }
    if (qt != nullptr && requant.done) {  // the float product was never written
      bq_tensor_release(o);
      *quantized_out = qt;
      return BQ_OK;
    }
    if (qt) bq_tensor_release(qt);
    *out = o;
    return BQ_OK;
  }

  // General path, as the reference: dequantize whatever is quantized, then float_matmul.
  bq_tensor* lf = nullptr;
  bq_tensor* rf = nullptr;
  bq_status rc = BQ_OK;
  if (lq) rc = bq_dequantize(lhs, target, &lf);
  // (exact mode with bf16 activations: the weights still go to f32 -- dequantized to bf16, as the
  // reference's dtype rule has it, they would be rounded exactly as the fast kernel rounds them)
  if (rc == BQ_OK && rq) rc = bq_dequantize(rhs, exact ? BQ_F32 : target, &rf);
  bq_tensor* o = nullptr;
  if (rc == BQ_OK) rc = new_float(dev, out_dtype, d.out_shape, d.rank, &o);
  if (rc == BQ_OK) {
    const bq_tensor* l = lq ? lf : lhs;
    const bq_tensor* r = rq ? rf : rhs;
    for (size_t b = 0; b < d.batches && rc == BQ_OK; ++b) {
      size_t lb, rb;
      batch_offsets(d, b, &lb, &rb);
      rc = launch_float_matmul(static_cast<char*>(l->data) + lb * d.m * d.k * dtype_size(l->dtype), l->dtype,
                               static_cast<char*>(r->data) + rb * d.k * d.n * dtype_size(r->dtype), r->dtype,
                               d.m, d.k, d.n, out_dtype,
                               static_cast<char*>(o->data) + b * d.m * d.n * dtype_size(out_dtype), st);
      if (rc == BQ_OK && bias != nullptr)
        rc = launch_add_bias(static_cast<char*>(o->data) + b * d.m * d.n * dtype_size(out_dtype), out_dtype, bias,
                             d.m, d.n, st);
    }
  }
  if (lf) bq_tensor_release(lf);
  if (rf) bq_tensor_release(rf);
  if (rc != BQ_OK) {
    if (o) bq_tensor_release(o);
    return rc;
  }
  *out = o;
  return BQ_OK;
}

extern "C" bq_status bq_q_matmul(const bq_tensor* lhs, const bq_tensor* rhs, bq_tensor** out) {
  return q_matmul_impl(lhs, rhs, -1, nullptr, out);
}

extern "C" bq_status bq_q_matmul_as(const bq_tensor* lhs, const bq_tensor* rhs, int32_t out_dtype,
                                    bq_tensor** out) {
  if (out_dtype != BQ_F32 && out_dtype != BQ_BF16) BQ_FAIL(BQ_ERR_DTYPE, "out dtype must be f32 or bf16");
  return q_matmul_impl(lhs, rhs, out_dtype, nullptr, out);
}

// q_matmul under QuantPropagation::Propagate (crates/burn-ndarray/src/ops/qtensor.rs:262-265): the
// float product is quantized again, dynamically, with the scheme of the quantized operand (the
// rhs's when both are).
extern "C" bq_status bq_q_matmul_propagate(const bq_tensor* lhs, const bq_tensor* rhs, bq_tensor** out) {
  BQ_NOTNULL(lhs);
  BQ_NOTNULL(rhs);
  BQ_NOTNULL(out);
  const bool lq = lhs->dtype == BQ_QFLOAT, rq = rhs->dtype == BQ_QFLOAT;
  if (!lq && !rq) BQ_FAIL(BQ_ERR_DTYPE, "q_matmul needs at least one quantized operand");
  const int32_t target = !lq ? lhs->dtype : (!rq ? rhs->dtype : BQ_F32);
  const bq_scheme scheme = rq ? rhs->scheme : lhs->scheme;
  // The product has the float operand's dtype (qtensor.rs:234-239). A bf16 product is what gets
  // quantized: its values, widened exactly to the f32 the quantize kernels read.
  bq_tensor* f = nullptr;
  bq_tensor* quantized = nullptr;
  BQ_TRY(q_matmul_impl(lhs, rhs, target, nullptr, &f, &quantized, &scheme));
  if (quantized != nullptr) {  // quantized where the K slices were summed
    *out = quantized;
    return BQ_OK;
  }
  bq_status rc = BQ_OK;
  if (target == BQ_BF16) {
    bq_tensor* wide = nullptr;
    rc = new_float(f->dev, BQ_F32, f->shape, f->rank, &wide);
    if (rc == BQ_OK) rc = launch_bf16_to_f32(static_cast<const uint16_t*>(f->data), f->numel(), static_cast<float*>(wide->data), f->dev->stream);
    bq_tensor_release(f);
    f = wide;
    if (rc != BQ_OK) {
      if (f) bq_tensor_release(f);
      return rc;
    }
  }
  rc = bq_quantize_dynamic(f, &scheme, out);
  bq_tensor_release(f);
  return rc;
}

static bq_tensor* alias_of(const bq_tensor* t);

// linear (crates/burn-tensor/src/tensor/module.rs:527-567, quantized-weight branch): the leading
// dims of x fold into the rows of one [rows, d_in] x [d_in, d_out] product against the packed
// weight, then + bias. Here the bias is added by the kernel that writes the output.
extern "C" bq_status bq_q_linear(const bq_tensor* x, const bq_tensor* weight, const bq_tensor* bias,
                                 int32_t out_dtype, bq_tensor** out) {
  BQ_NOTNULL(x);
  BQ_NOTNULL(weight);
  BQ_NOTNULL(out);
  if (weight->dtype != BQ_QFLOAT || weight->rank != 2)
    BQ_FAIL(BQ_ERR_DTYPE, "q_linear takes a quantized [d_input, d_output] weight");
  if (x->dtype != BQ_F32 && x->dtype != BQ_BF16) BQ_FAIL(BQ_ERR_DTYPE, "q_linear input must be f32 or bf16");
  if (x->rank < 1 || x->shape[x->rank - 1] != weight->shape[0])
    BQ_FAIL(BQ_ERR_SHAPE, "q_linear input [.., %zu] does not match the weight's d_input %zu",
            x->rank >= 1 ? x->shape[x->rank - 1] : static_cast<size_t>(0), weight->shape[0]);
  if (out_dtype >= 0 && out_dtype != BQ_F32 && out_dtype != BQ_BF16)
    BQ_FAIL(BQ_ERR_DTYPE, "out dtype must be f32 or bf16");
  const size_t d_in = weight->shape[0], d_out = weight->shape[1];
  bq_device* dev = x->dev;
  if (weight->dev != dev || (bias != nullptr && bias->dev != dev))
    BQ_FAIL(BQ_ERR_DTYPE, "q_linear operands live on different devices");
  bq_tensor* bias32 = nullptr;  // f32 copy of a bf16 bias
  const float* bias_ptr = nullptr;
  if (bias != nullptr) {
    if ((bias->dtype != BQ_F32 && bias->dtype != BQ_BF16) || bias->rank != 1 || bias->shape[0] != d_out)
      BQ_FAIL(BQ_ERR_SHAPE, "q_linear bias must be a float [d_output = %zu] tensor", d_out);
    if (bias->dtype == BQ_BF16) {
      BQ_TRY(new_float(dev, BQ_F32, &d_out, 1, &bias32));
      bq_status rc = launch_bf16_to_f32(static_cast<const uint16_t*>(bias->data), d_out,
                                        static_cast<float*>(bias32->data), dev->stream);
      if (rc != BQ_OK) {
        bq_tensor_release(bias32);
        return rc;
      }
      bias_ptr = static_cast<const float*>(bias32->data);
    } else {
      bias_ptr = static_cast<const float*>(bias->data);
    }
  }
  size_t rows = 1;
  for (int d = 0; d + 1 < x->rank; ++d) rows *= x->shape[d];
  bq_tensor* x2 = alias_of(x);  // [rows, d_in] view of the same memory
  x2->rank = 2;
  x2->shape[0] = rows;
  x2->shape[1] = d_in;
  bq_tensor* o = nullptr;
  bq_status rc = q_matmul_impl(x2, weight, out_dtype, bias_ptr, &o);
  bq_tensor_release(x2);
  if (bias32) bq_tensor_release(bias32);
  if (rc != BQ_OK) return rc;
  // [rows, d_out] -> [.., d_out]
  o->rank = x->rank;
  for (int d = 0; d + 1 < x->rank; ++d) o->shape[d] = x->shape[d];
  o->shape[x->rank - 1] = d_out;
  *out = o;
  return BQ_OK;
}

// ================================================================================ layout ops
static bq_tensor* alias_of(const bq_tensor* t) {
  bq_tensor* a = new bq_tensor();
  a->dev = t->dev;
  a->dtype = t->dtype;
  a->rank = t->rank;
  for (int d = 0; d < t->rank; ++d) a->shape[d] = t->shape[d];
  a->scheme = t->scheme;
  a->data = t->data;
  a->alloc_bytes = 0;
  a->value_bytes = t->value_bytes;
  a->scales_offset = t->scales_offset;
  a->num_scales = t->num_scales;
  a->wire_offset = t->wire_offset;
  bq_tensor* root = const_cast<bq_tensor*>(t->base ? t->base : t);
  root->refs.fetch_add(1);
  a->base = root;
  return a;
}

extern "C" bq_status bq_q_to_device(const bq_tensor* t, bq_device* dev, bq_tensor** out) {
  BQ_NOTNULL(t);
  BQ_NOTNULL(dev);
  BQ_NOTNULL(out);
  if (t->dtype != BQ_QFLOAT) BQ_FAIL(BQ_ERR_DTYPE, "q_to_device takes a quantized tensor");
  if (dev == t->dev) {
    *out = alias_of(t);
    return BQ_OK;
  }
  // other GPU: values || scales is one allocation, so this is one peer copy
  bq_tensor* q = nullptr;
  BQ_TRY(new_quantized(dev, t->scheme, t->shape, t->rank, &q));
  BQ_HIP(hipStreamSynchronize(t->dev->stream));
  const size_t span = t->scheme.tensor_scale ? t->wire_offset + 4 * (1 + t->num_scales) : t->scales_offset + 4 * t->num_scales;
  hipError_t e = hipMemcpyPeerAsync(q->data, dev->ordinal, t->data, t->dev->ordinal, span, dev->stream);
  if (e != hipSuccess) {
    bq_tensor_release(q);
    BQ_FAIL(BQ_ERR_HIP, "peer copy failed: %s", hipGetErrorString(e));
  }
  *out = q;
  return BQ_OK;
}

extern "C" bq_status bq_q_reshape(const bq_tensor* t, const size_t* shape, int32_t rank, bq_tensor** out) {
  BQ_NOTNULL(t);
  BQ_NOTNULL(shape);
  BQ_NOTNULL(out);
  if (t->dtype != BQ_QFLOAT) BQ_FAIL(BQ_ERR_DTYPE, "q_reshape takes a quantized tensor");
  if (rank < 1 || rank > BQ_MAX_RANK) BQ_FAIL(BQ_ERR_SHAPE, "rank %d outside 1..%d", rank, BQ_MAX_RANK);
  BQ_TRY(check_shape_size(shape, rank));
  if (num_elements(shape, rank) != t->numel())
    BQ_FAIL(BQ_ERR_SHAPE, "reshape changes the number of elements (%zu -> %zu)", t->numel(),
            num_elements(shape, rank));
  bq_scheme s = t->scheme;
  const size_t nq = static_cast<size_t>(num_quants(s.value));
  if (s.store == BQ_STORE_PACKED_U32 && (shape[rank - 1] % nq))
    BQ_FAIL(BQ_ERR_UNSUPPORTED_OP, "reshape would split packed words: new last dim %zu, %zu values per word",
            shape[rank - 1], nq);
  if (s.level == BQ_LEVEL_BLOCK) {
    // Only metadata moves, so the blocks must stay the same runs of the flat storage.
    // The run is laid over the new trailing dims: whole dims while it is at least as long as they
    // are, then a divisor of the next one. (Block extents are bytes, as in the reference's
    // BlockSize, so a run of 256 or more has to be spread over several dims.)
    const long run = run_block(s, t->shape, t->rank);
    size_t rem = run > 0 ? static_cast<size_t>(run) : 0;
    uint8_t blk[BQ_MAX_RANK];
    int used = 0;
    for (int d = rank - 1; d >= 0 && rem > 1; --d) {
      const size_t ext = shape[d];
      size_t take;
      if (rem >= ext && ext > 0 && rem % ext == 0) {
        take = ext;
        rem /= ext;
      } else if (rem < ext && ext % rem == 0) {
        take = rem;
        rem = 1;
      } else {
        break;
      }
      if (take > 255) {
        rem = 0;
        break;
      }
      blk[used++] = static_cast<uint8_t>(take);
    }
    if (rem != 1)
      BQ_FAIL(BQ_ERR_UNSUPPORTED_OP,
              "reshape of a block-quantized tensor needs blocks that stay runs of the new trailing dims");
    if (used == 0) blk[used++] = 1;
    s.block_rank = static_cast<uint8_t>(used);
    for (int j = 0; j < used; ++j) s.block[j] = blk[used - 1 - j];  // (outermost of the used dims first)
  }
  bq_tensor* a = alias_of(t);
  a->rank = rank;
  for (int d = 0; d < rank; ++d) a->shape[d] = shape[d];
  a->scheme = s;
  *out = a;
  return BQ_OK;
}

// q_permute and q_flip in one gather: output dim a reads source dim axes[a], backwards where
// flip[axes[a]] is set. Block scales move with their blocks, as in
// crates/burn-ndarray/src/ops/qtensor.rs:310-336 (scheme.permute_block_dims).
// keep_params: the scales are copied as they are, whatever happens to the values (the reference's
// q_flip).
static bq_status q_gather_impl(const bq_tensor* t, const int32_t* axes, const uint8_t* flip, bq_tensor** out,
                               bool keep_params = false) {
  const int rank = t->rank;
  size_t new_shape[BQ_MAX_RANK], old_blk[BQ_MAX_RANK], old_params[BQ_MAX_RANK];
  block_dims(t->scheme, rank, old_blk);
  bq_scheme scheme = t->scheme;
  for (int a = 0; a < rank; ++a) {
    new_shape[a] = t->shape[axes[a]];
    old_params[a] = t->shape[a] / old_blk[a];
  }
  if (scheme.level == BQ_LEVEL_BLOCK) {
    scheme.block_rank = static_cast<uint8_t>(rank);
    for (int a = 0; a < rank; ++a) scheme.block[a] = static_cast<uint8_t>(old_blk[axes[a]]);
  }
  // Q8S words are the same bytes as native values, so a result whose last dim no longer fills whole
  // words is stored natively instead of being refused (the reference's CPU backend keeps one i8 per
  // value whatever the store says and permutes freely: ops/quantize.rs:406-431 of its tests ends
  // with a last dim of 2). Packed sub-byte values would have to be unpacked: those results are refused.
  if (scheme.store == BQ_STORE_PACKED_U32 && value_bits(scheme.value) == 8 && new_shape[rank - 1] % 4 != 0)
    scheme.store = BQ_STORE_NATIVE;
  bq_tensor* q = nullptr;
  BQ_TRY(new_quantized(t->dev, scheme, new_shape, rank, &q));  // also: "Can't store in u32" for the new last dim
  hipStream_t st = t->dev->stream;
  bq_status rc = launch_q_gather(t->data, q->data, t->shape, rank, axes, flip, stored_value(scheme.value, scheme.store),
                                 scheme.store == BQ_STORE_NATIVE, st);
  if (rc == BQ_OK) {
    if (scheme.tensor_scale) {  // two-level: what the blob stores moves like the scales the kernels use
      hipError_t e = hipMemcpyAsync(q->wire_global(), t->wire_global(), 4, hipMemcpyDeviceToDevice, st);
      if (e == hipSuccess && keep_params)
        e = hipMemcpyAsync(q->wire_scales(), t->wire_scales(), 4 * t->num_scales, hipMemcpyDeviceToDevice, st);
      if (e != hipSuccess) {
        set_error("copying scales failed: %s", hipGetErrorString(e));
        rc = BQ_ERR_HIP;
      } else if (!keep_params) {
        rc = launch_f32_gather(t->wire_scales(), q->wire_scales(), old_params, rank, axes, flip, st);
      }
    }
    if (rc != BQ_OK) {
    } else if (scheme.level == BQ_LEVEL_BLOCK && !keep_params) {
      rc = launch_f32_gather(t->scales(), q->scales(), old_params, rank, axes, flip, st);
    } else {
      hipError_t e = hipMemcpyAsync(q->scales(), t->scales(), 4 * t->num_scales, hipMemcpyDeviceToDevice, st);
      if (e != hipSuccess) {
        set_error("copying scales failed: %s", hipGetErrorString(e));
        rc = BQ_ERR_HIP;
      }
    }
  }
  if (rc != BQ_OK) {
    bq_tensor_release(q);
    return rc;
  }
  *out = q;
  return BQ_OK;
}

// ================================================================================ integer-domain ops
// q_slice / q_select / q_gather / q_expand / q_argmax / q_argmin on the stored integers, as the reference's CPU
// backend runs them (crates/burn-ndarray/src/ops/qtensor.rs:349-430): no dequantize, no new scales.
// One routine builds every result: the values through an index map over the source, the block
// scales through the same map in block units.
struct IndexPlan {
  int rank = 0;                        // of the output
  size_t out_shape[BQ_MAX_RANK] = {0};
  int64_t stride[BQ_MAX_RANK] = {0};   // source elements per step of output dim a
  int64_t base = 0;
  // block schemes: the same map over the params tensor
  size_t p_shape[BQ_MAX_RANK] = {0};
  int64_t p_stride[BQ_MAX_RANK] = {0};
  int64_t p_base = 0;
  int index_dim = -1, index_mode = 0;
  const bq_tensor* indices = nullptr;
  size_t index_limit = 0;
};

static bq_status index_map_impl(const bq_tensor* t, const IndexPlan& p, bq_tensor** out) {
  bq_scheme scheme = t->scheme;
  // (a Q8S result whose last dim no longer fills whole words is stored natively, as q_permute does)
  if (scheme.store == BQ_STORE_PACKED_U32 && value_bits(scheme.value) == 8 && p.out_shape[p.rank - 1] % 4 != 0)
    scheme.store = BQ_STORE_NATIVE;
  bq_tensor* q = nullptr;
  BQ_TRY(new_quantized(t->dev, scheme, p.out_shape, p.rank, &q));  // also: "Can't store in u32", dims against the block
  hipStream_t st = t->dev->stream;
  const void* idx = p.indices ? p.indices->data : nullptr;
  const int idx_dtype = p.indices ? p.indices->dtype : BQ_I32;
  bq_status rc = BQ_OK;
  bool fused = false;  // values and block scales in one launch where both are whole-row copies
  if (scheme.level == BQ_LEVEL_BLOCK)
    rc = launch_index_map_pair(t->data, q->data, p.out_shape, p.stride, p.base, stored_value(t->scheme.value, t->scheme.store),
                               t->scheme.store == BQ_STORE_NATIVE, scheme.store == BQ_STORE_NATIVE, t->scales(), q->scales(), p.p_shape,
                               p.p_stride, p.p_base, p.rank, p.index_dim, p.index_mode, idx, idx_dtype, p.index_limit, &fused, st);
  if (rc == BQ_OK && !fused)
    rc = launch_q_index_map(t->data, q->data, p.out_shape, p.rank, p.stride, p.base, p.index_dim, p.index_mode, idx, idx_dtype,
                            p.index_limit, stored_value(t->scheme.value, t->scheme.store), t->scheme.store == BQ_STORE_NATIVE,
                            scheme.store == BQ_STORE_NATIVE, st);
  if (rc == BQ_OK && scheme.level == BQ_LEVEL_BLOCK) {
    if (!fused)
      rc = launch_f32_index_map(t->scales(), q->scales(), p.p_shape, p.rank, p.p_stride, p.p_base, p.index_dim, p.index_mode, idx, idx_dtype,
                              p.index_limit, st);
    if (rc == BQ_OK && scheme.tensor_scale)
      rc = launch_f32_index_map(t->wire_scales(), q->wire_scales(), p.p_shape, p.rank, p.p_stride, p.p_base, p.index_dim, p.index_mode, idx,
                                idx_dtype, p.index_limit, st);
  } else if (rc == BQ_OK) {
    hipError_t e = hipMemcpyAsync(q->scales(), t->scales(), 4, hipMemcpyDeviceToDevice, st);
    if (e != hipSuccess) {
      set_error("copying the scale failed: %s", hipGetErrorString(e));
      rc = BQ_ERR_HIP;
    }
  }
  if (rc == BQ_OK && scheme.tensor_scale) {
    hipError_t e = hipMemcpyAsync(q->wire_global(), t->wire_global(), 4, hipMemcpyDeviceToDevice, st);
    if (e != hipSuccess) {
      set_error("copying the per-tensor scale failed: %s", hipGetErrorString(e));
      rc = BQ_ERR_HIP;
    }
  }
  if (rc != BQ_OK) {
    bq_tensor_release(q);
    return rc;
  }
  *out = q;
  return BQ_OK;
}

static void source_strides(const bq_tensor* t, const size_t* blk, int64_t* stride, int64_t* p_stride) {
  int64_t s = 1, ps = 1;
  for (int a = t->rank - 1; a >= 0; --a) {
    stride[a] = s;
    p_stride[a] = ps;
    s *= static_cast<int64_t>(t->shape[a]);
    ps *= static_cast<int64_t>(t->shape[a] / blk[a]);
  }
}

static bq_status check_quantized_for_index_op(const bq_tensor* t, const char* op) {
  if (t->dtype != BQ_QFLOAT) BQ_FAIL(BQ_ERR_DTYPE, "%s takes a quantized tensor", op);
  for (int a = 0; a < t->rank; ++a)
    if (t->shape[a] > 0xFFFFFFFFull) BQ_FAIL(BQ_ERR_SIZE, "%s: dim %d of %zu exceeds 32 bits", op, a, t->shape[a]);
  return BQ_OK;
}

// Slice::to_range / output_size (crates/burn-std/src/tensor/slice.rs:493-545): negative indices count
// from the end, everything is clamped into the dim, a negative step walks the range backwards.
extern "C" bq_status bq_q_slice(const bq_tensor* t, const int64_t* starts, const int64_t* ends, const int64_t* steps, int32_t n_slices,
                                bq_tensor** out) {
  BQ_NOTNULL(t);
  BQ_NOTNULL(out);
  BQ_TRY(check_quantized_for_index_op(t, "q_slice"));
  if (n_slices < 0 || n_slices > t->rank) BQ_FAIL(BQ_ERR_SHAPE, "%d slices for a tensor of rank %d", n_slices, t->rank);
  if (n_slices > 0) {
    BQ_NOTNULL(starts);
    BQ_NOTNULL(ends);
    BQ_NOTNULL(steps);
  }
  size_t blk[BQ_MAX_RANK];
  block_dims(t->scheme, t->rank, blk);
  int64_t stride[BQ_MAX_RANK], p_stride[BQ_MAX_RANK];
  source_strides(t, blk, stride, p_stride);
  auto signed_index = [](int64_t i, int64_t size) { return i < 0 ? std::max<int64_t>(size + i, 0) : std::min<int64_t>(i, size); };
  IndexPlan p;
  p.rank = t->rank;
  for (int a = 0; a < t->rank; ++a) {
    const int64_t size = static_cast<int64_t>(t->shape[a]);
    int64_t start = 0, end = size, step = 1;
    if (a < n_slices) {
      step = steps[a];
      if (step == 0 || step == INT64_MIN) BQ_FAIL(BQ_ERR_SHAPE, "Step cannot be zero");  // (INT64_MIN has no magnitude)
      start = signed_index(starts[a], size);
      end = ends[a] == INT64_MAX ? size : signed_index(ends[a], size);   // INT64_MAX: to the end of the dim
    }
    const int64_t len = end > start ? end - start : 0;
    const int64_t mag = step < 0 ? -step : step;
    const int64_t n_out = (len + mag - 1) / mag;
    const int64_t first = step > 0 ? start : end - 1;
    p.out_shape[a] = static_cast<size_t>(n_out);
    p.stride[a] = step * stride[a];
    p.base += (n_out > 0 ? first : 0) * stride[a];
    const int64_t b = static_cast<int64_t>(blk[a]);
    if (b > 1) {
      // whole blocks only: the scales of the result are the scales of the blocks it keeps
      if (step != 1 || start % b != 0 || len % b != 0)
        BQ_FAIL(BQ_ERR_UNSUPPORTED_OP, "q_slice: dim %d is cut inside its blocks of %lld (range %lld..%lld, step %lld)", a,
                static_cast<long long>(b), static_cast<long long>(start), static_cast<long long>(end), static_cast<long long>(step));
      p.p_shape[a] = static_cast<size_t>(len / b);
      p.p_stride[a] = p_stride[a];
      p.p_base += (start / b) * p_stride[a];
    } else {
      p.p_shape[a] = static_cast<size_t>(n_out);
      p.p_stride[a] = step * p_stride[a];
      p.p_base += (n_out > 0 ? first : 0) * p_stride[a];
    }
  }
  return index_map_impl(t, p, out);
}

static bq_status check_indices(const bq_tensor* t, const bq_tensor* indices, const char* op) {
  BQ_NOTNULL(indices);
  if (indices->dtype != BQ_I32 && indices->dtype != BQ_I64) BQ_FAIL(BQ_ERR_DTYPE, "%s takes i32 or i64 indices", op);
  if (indices->dev != t->dev) BQ_FAIL(BQ_ERR_DTYPE, "%s: the indices live on another device", op);
  return BQ_OK;
}

extern "C" bq_status bq_q_select(const bq_tensor* t, int32_t dim, const bq_tensor* indices, bq_tensor** out) {
  BQ_NOTNULL(t);
  BQ_NOTNULL(out);
  BQ_TRY(check_quantized_for_index_op(t, "q_select"));
  BQ_TRY(check_indices(t, indices, "q_select"));
  if (dim < 0 || dim >= t->rank) BQ_FAIL(BQ_ERR_SHAPE, "q_select: dim %d of a tensor of rank %d", dim, t->rank);
  if (indices->rank != 1) BQ_FAIL(BQ_ERR_SHAPE, "q_select takes a 1-D index tensor");
  size_t blk[BQ_MAX_RANK];
  block_dims(t->scheme, t->rank, blk);
  if (blk[dim] > 1) BQ_FAIL(BQ_ERR_UNSUPPORTED_OP, "q_select along dim %d would pick single values out of blocks of %zu", dim, blk[dim]);
  if (t->shape[dim] == 0 && indices->shape[0] > 0) BQ_FAIL(BQ_ERR_SHAPE, "q_select from an empty dim");
  IndexPlan p;
  p.rank = t->rank;
  source_strides(t, blk, p.stride, p.p_stride);
  for (int a = 0; a < t->rank; ++a) {
    p.out_shape[a] = a == dim ? indices->shape[0] : t->shape[a];
    p.p_shape[a] = p.out_shape[a] / blk[a];
  }
  p.index_dim = dim;
  p.index_mode = 1;
  p.indices = indices;
  p.index_limit = t->shape[dim];
  return index_map_impl(t, p, out);
}

extern "C" bq_status bq_q_gather(int32_t dim, const bq_tensor* t, const bq_tensor* indices, bq_tensor** out) {
  BQ_NOTNULL(t);
  BQ_NOTNULL(out);
  BQ_TRY(check_quantized_for_index_op(t, "q_gather"));
  BQ_TRY(check_indices(t, indices, "q_gather"));
  if (dim < 0 || dim >= t->rank) BQ_FAIL(BQ_ERR_SHAPE, "q_gather: dim %d of a tensor of rank %d", dim, t->rank);
  if (indices->rank != t->rank) BQ_FAIL(BQ_ERR_SHAPE, "q_gather: indices of rank %d for a tensor of rank %d", indices->rank, t->rank);
  // (the reference folds both operands to [batch, size]: every other dim must agree, base.rs:106-138)
  for (int a = 0; a < t->rank; ++a)
    if (a != dim && indices->shape[a] != t->shape[a])
      BQ_FAIL(BQ_ERR_SHAPE, "q_gather: indices dim %d is %zu, the tensor's is %zu", a, indices->shape[a], t->shape[a]);
  if (t->scheme.level == BQ_LEVEL_BLOCK) {
    size_t blk[BQ_MAX_RANK];
    block_dims(t->scheme, t->rank, blk);
    for (int a = 0; a < t->rank; ++a)
      if (blk[a] > 1) BQ_FAIL(BQ_ERR_UNSUPPORTED_OP, "q_gather picks single values: block scales cannot follow them");
  }
  if (t->shape[dim] == 0 && indices->numel() > 0) BQ_FAIL(BQ_ERR_SHAPE, "q_gather from an empty dim");
  size_t blk[BQ_MAX_RANK];
  block_dims(t->scheme, t->rank, blk);
  IndexPlan p;
  p.rank = t->rank;
  source_strides(t, blk, p.stride, p.p_stride);
  for (int a = 0; a < t->rank; ++a) p.out_shape[a] = p.p_shape[a] = indices->shape[a];
  p.index_dim = dim;
  p.index_mode = 2;
  p.indices = indices;
  p.index_limit = t->shape[dim];
  return index_map_impl(t, p, out);
}

// Broadcast: trailing dims aligned, a source dim of 1 repeats, new leading dims repeat the whole tensor.
extern "C" bq_status bq_q_expand(const bq_tensor* t, const size_t* shape, int32_t rank, bq_tensor** out) {
  BQ_NOTNULL(t);
  BQ_NOTNULL(shape);
  BQ_NOTNULL(out);
  BQ_TRY(check_quantized_for_index_op(t, "q_expand"));
  if (rank < t->rank || rank > BQ_MAX_RANK) BQ_FAIL(BQ_ERR_SHAPE, "q_expand: rank %d from a tensor of rank %d", rank, t->rank);
  size_t blk[BQ_MAX_RANK];
  block_dims(t->scheme, t->rank, blk);
  int64_t stride[BQ_MAX_RANK], p_stride[BQ_MAX_RANK];
  source_strides(t, blk, stride, p_stride);
  IndexPlan p;
  p.rank = rank;
  const int lead = rank - t->rank;
  for (int a = 0; a < rank; ++a) {
    if (shape[a] > 0xFFFFFFFFull) BQ_FAIL(BQ_ERR_SIZE, "q_expand: dim %d of %zu exceeds 32 bits", a, shape[a]);
    p.out_shape[a] = shape[a];
    const int s = a - lead;
    if (s < 0) {
      p.stride[a] = p.p_stride[a] = 0;
      p.p_shape[a] = shape[a];
    } else if (t->shape[s] == shape[a]) {
      p.stride[a] = stride[s];
      p.p_stride[a] = p_stride[s];
      p.p_shape[a] = shape[a] / blk[s];
    } else if (t->shape[s] == 1) {   // (a dim of 1 holds blocks of 1)
      p.stride[a] = p.p_stride[a] = 0;
      p.p_shape[a] = shape[a];
    } else {
      BQ_FAIL(BQ_ERR_SHAPE, "q_expand: dim %d of %zu cannot become %zu", s, t->shape[s], shape[a]);
    }
  }
  return index_map_impl(t, p, out);
}

static bq_status q_arg_impl(const bq_tensor* t, int32_t dim, int32_t out_dtype, bool want_max, bq_tensor** out) {
  BQ_NOTNULL(t);
  BQ_NOTNULL(out);
  const char* op = want_max ? "q_argmax" : "q_argmin";
  BQ_TRY(check_quantized_for_index_op(t, op));
  if (dim < 0 || dim >= t->rank) BQ_FAIL(BQ_ERR_SHAPE, "%s: dim %d of a tensor of rank %d", op, dim, t->rank);
  if (out_dtype != BQ_I32 && out_dtype != BQ_I64) BQ_FAIL(BQ_ERR_DTYPE, "%s returns i32 or i64 indices", op);
  // one scale for everything compared: the order of the integers is the order of the values
  if (t->scheme.level == BQ_LEVEL_BLOCK) {
    size_t blk[BQ_MAX_RANK];
    block_dims(t->scheme, t->rank, blk);
    bool whole = true;
    for (int a = 0; a < t->rank; ++a) whole = whole && (a == dim ? blk[a] == t->shape[a] : blk[a] == 1);
    if (!whole) BQ_FAIL(BQ_ERR_UNSUPPORTED_OP, "%s along dim %d compares values of different blocks: dequantize first", op, dim);
  }
  if (t->shape[dim] == 0) BQ_FAIL(BQ_ERR_SHAPE, "Cannot compute arg over an empty axis");
  size_t oshape[BQ_MAX_RANK], outer = 1, inner = 1;
  for (int a = 0; a < t->rank; ++a) {
    oshape[a] = a == dim ? 1 : t->shape[a];
    if (a < dim) outer *= t->shape[a];
    if (a > dim) inner *= t->shape[a];
  }
  bq_tensor* o = nullptr;
  BQ_TRY(new_float(t->dev, out_dtype, oshape, t->rank, &o));
  const bq_status rc = launch_q_arg(t->data, stored_value(t->scheme.value, t->scheme.store), t->scheme.store == BQ_STORE_NATIVE, outer,
                                    t->shape[dim], inner, want_max, out_dtype, o->data, t->dev->stream);
  if (rc != BQ_OK) {
    bq_tensor_release(o);
    return rc;
  }
  *out = o;
  return BQ_OK;
}

extern "C" bq_status bq_q_argmax(const bq_tensor* t, int32_t dim, int32_t out_dtype, bq_tensor** out) {
  return q_arg_impl(t, dim, out_dtype, true, out);
}

extern "C" bq_status bq_q_argmin(const bq_tensor* t, int32_t dim, int32_t out_dtype, bq_tensor** out) {
  return q_arg_impl(t, dim, out_dtype, false, out);
}

extern "C" bq_status bq_q_permute(const bq_tensor* t, const int32_t* axes, int32_t rank, bq_tensor** out) {
  BQ_NOTNULL(t);
  BQ_NOTNULL(axes);
  BQ_NOTNULL(out);
  if (t->dtype != BQ_QFLOAT) BQ_FAIL(BQ_ERR_DTYPE, "q_permute takes a quantized tensor");
  if (rank != t->rank) BQ_FAIL(BQ_ERR_SHAPE, "permute axes of rank %d on a tensor of rank %d", rank, t->rank);
  bool identity = true, seen[BQ_MAX_RANK] = {false};
  for (int d = 0; d < rank; ++d) {
    // (the reference panics on an axis out of bounds or repeated)
    if (axes[d] < 0 || axes[d] >= rank) BQ_FAIL(BQ_ERR_SHAPE, "permute axis %d out of bounds for rank %d", axes[d], rank);
    if (seen[axes[d]]) BQ_FAIL(BQ_ERR_SHAPE, "permute axis %d is repeated", axes[d]);
    seen[axes[d]] = true;
    identity = identity && axes[d] == d;
  }
  if (identity) {
    *out = alias_of(t);
    return BQ_OK;
  }
  return q_gather_impl(t, axes, nullptr, out);
}

extern "C" bq_status bq_q_swap_dims(const bq_tensor* t, int32_t dim1, int32_t dim2, bq_tensor** out) {
  BQ_NOTNULL(t);
  if (dim1 < 0 || dim2 < 0 || dim1 >= t->rank || dim2 >= t->rank)
    BQ_FAIL(BQ_ERR_SHAPE, "swap_dims(%d, %d) on a tensor of rank %d", dim1, dim2, t->rank);
  int32_t axes[BQ_MAX_RANK];
  for (int d = 0; d < t->rank; ++d) axes[d] = d;
  std::swap(axes[dim1], axes[dim2]);
  return bq_q_permute(t, axes, t->rank, out);
}

extern "C" bq_status bq_q_flip(const bq_tensor* t, const int32_t* axes, int32_t n_axes, bq_tensor** out) {
  BQ_NOTNULL(t);
  BQ_NOTNULL(out);
  if (t->dtype != BQ_QFLOAT) BQ_FAIL(BQ_ERR_DTYPE, "q_flip takes a quantized tensor");
  if (n_axes == 0) {
    *out = alias_of(t);
    return BQ_OK;
  }
  BQ_NOTNULL(axes);
  uint8_t flip[BQ_MAX_RANK] = {0};
  for (int i = 0; i < n_axes; ++i) {
    if (axes[i] < 0 || axes[i] >= t->rank) BQ_FAIL(BQ_ERR_SHAPE, "flip axis %d out of bounds for rank %d", axes[i], t->rank);
    if (flip[axes[i]]) BQ_FAIL(BQ_ERR_SHAPE, "flip axis %d is repeated", axes[i]);
    flip[axes[i]] = 1;
  }
  // The reference flips the values and keeps the parameters as they are, block scales included
  // (crates/burn-ndarray/src/ops/qtensor.rs:338-347): after a flip across blocks a value is
  // dequantized with the scale of the block it lands in. Reproduced as it is.
  int32_t ident[BQ_MAX_RANK];
  for (int d = 0; d < t->rank; ++d) ident[d] = d;
  return q_gather_impl(t, ident, flip, out, /*keep_params=*/true);
}
