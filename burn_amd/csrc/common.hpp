// Internal declarations shared by the host runtime and the kernel translation units.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <mutex>
#include <string>
#include <vector>

#include "block_cache.hpp"
#include "burnq.h"

namespace bq {

// ---- error reporting -------------------------------------------------------------------------
void set_error(const char* fmt, ...);
const char* get_error();

#define BQ_FAIL(code, ...)        \
  do {                            \
    ::bq::set_error(__VA_ARGS__); \
    return (code);                \
  } while (0)

#define BQ_HIP(expr)                                                                       \
  do {                                                                                     \
    hipError_t _e = (expr);                                                                \
    if (_e != hipSuccess) BQ_FAIL(BQ_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(_e)); \
  } while (0)

#define BQ_TRY(expr)                 \
  do {                               \
    bq_status _s = (expr);           \
    if (_s != BQ_OK) return _s;      \
  } while (0)

#define BQ_NOTNULL(p) \
  do {                \
    if ((p) == nullptr) BQ_FAIL(BQ_ERR_NULL, "%s: null argument '%s'", __func__, #p); \
  } while (0)

// ---- value helpers ---------------------------------------------------------------------------
// QuantValue::range(): symmetric Q8S (-127,127), Q4S (-7,7), Q2S (-1,1) (ternary: -1, 0, +1);
// full-range Q8F (-128,127), Q4F (-8,7), Q2F (-2,1). A full-range value has the bit layout of the
// symmetric value of the same width (two's complement fields): only the quantize kernels -- the
// span of the scale, the lower clamp -- tell them apart, everything else works on storage_value.
inline bool value_supported(int v) { return v >= BQ_Q8S && v <= BQ_Q2F; }
inline bool value_full(int v) { return v == BQ_Q8F || v == BQ_Q4F || v == BQ_Q2F; }
inline int storage_value(int v) { return value_full(v) ? v - BQ_Q8F : v; }
// value_known: what the fused kernels take (8- and 4-bit values). 2-bit values go through the
// general kernels, Q2S also through the ternary matmul.
inline bool value_known(int v) { return value_supported(v) && (storage_value(v) == BQ_Q8S || storage_value(v) == BQ_Q4S); }
inline int value_bits(int v) { return storage_value(v) == BQ_Q8S ? 8 : (storage_value(v) == BQ_Q4S ? 4 : 2); }
inline int value_qmax(int v) { return storage_value(v) == BQ_Q8S ? 127 : (storage_value(v) == BQ_Q4S ? 7 : 1); }  // b
inline int value_qmin(int v) { return -value_qmax(v) - (value_full(v) ? 1 : 0); }                                   // a
inline float value_span(int v) { return static_cast<float>(value_qmax(v) - value_qmin(v)); }                        // b - a
inline int num_quants(int v) { return 32 / value_bits(v); }
// The Native store keeps one i8 per value whatever the value's width (QuantizedBytes::new,
// crates/burn-std/src/tensor/quantization.rs:219-272; burn-store/src/tensor_snapshot.rs:545-557),
// so a 4- or 2-bit tensor stored natively reads exactly like a Q8S one with small values: every
// kernel that only reads values takes stored_value(). Quantizing to it clamps to the narrow range and
// goes through the general kernels (fused_value() is false).
inline int stored_value(int v, int store) { return store == BQ_STORE_NATIVE ? BQ_Q8S : v; }
inline bool fused_value(int v, int store) { return value_known(v) && !(store == BQ_STORE_NATIVE && value_bits(v) != 8); }

inline size_t round_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// Ticket counters of the single-launch split-K sum (splitk_tail.hpp): one counter per column tile
// of a launch, a 128-byte line apart.
constexpr unsigned kTicketStride = 32;     // words between two tiles' counters
constexpr unsigned kTicketCells = 2048;    // tiles a launch may have
constexpr size_t kTicketBytes = static_cast<size_t>(kTicketCells) * kTicketStride * sizeof(unsigned);

}  // namespace bq

// ---- opaque types ----------------------------------------------------------------------------
struct bq_device {
  int ordinal = 0;
  hipStream_t stream = nullptr;
  hipEvent_t ev_start = nullptr, ev_stop = nullptr;
  std::mutex mu;                                  // guards the allocation cache and workspace
  bq::BlockCache cache;                           // cached allocations, graph-capture bookkeeping
  void* workspace = nullptr;                      // split-K partials, bf16 copy of an f32 lhs
  size_t workspace_bytes = 0;
  unsigned* tickets = nullptr;                    // counters of the single-launch split-K sum (zero between launches)
  int num_cus = 256;
  size_t lds_limit = 64 * 1024;                   // largest dynamic LDS request a launch may make
  std::atomic<bool> validate{false};              // bq_device_set_validate
  std::atomic<bool> f32_matmul_exact{false};  // bq_device_set_f32_matmul_exact
  uint32_t* validate_cells = nullptr;             // 4 device counters of the validate mode
  // Two pinned halves that host <-> device copies go through (lazily allocated, see upload()).
  static constexpr size_t kStageBytes = 2u << 20;
  std::mutex stage_mu;
  char* stage[2] = {nullptr, nullptr};
  hipEvent_t stage_ev[2] = {nullptr, nullptr};
  bool stage_pending[2] = {false, false};         // a copy out of this half may still be in flight
  int stage_next = 0;
  // Small uploads and the short wait (set up when the device is opened). A copy of up to kSmallUpload bytes
  // leaves one of kSmallSlots pinned slots by a copy kernel that writes its sequence number to the slot's
  // pinned word once it holds the data: the host knows when it may refill a slot by reading memory, with no
  // event (recording one adds 5 us to a transfer of 3). The last word is written by the kernel bq_device_sync
  // queues behind everything else.
  static constexpr size_t kSmallUpload = 64u << 10;
  static constexpr int kSmallSlots = 4;
  char* small_stage = nullptr;                    // kSmallSlots * kSmallUpload bytes, pinned
  uint32_t* host_words = nullptr;                 // kSmallSlots + 1 pinned words the device writes
  uint32_t small_issued[kSmallSlots] = {};        // sequence number of the last copy queued out of each slot
  uint32_t small_seq = 0;
  int small_next = 0;
  std::mutex sync_mu;                             // orders the wait kernels of concurrent bq_device_sync calls
  uint32_t sync_seq = 0;

  // *actual receives the size of the block handed out (at least `bytes`); pass it to release().
  bq_status alloc(size_t bytes, void** out, size_t* actual);  // stream-ordered reuse is safe: one stream
  void release(void* ptr, size_t bytes);
  bq_status ensure_workspace(size_t bytes);
  // Copies between pageable host memory and this device, behind the work already queued on the
  // stream. upload() returns once the host buffer has been read (the transfer itself is stream
  // ordered like a kernel); download() returns with the data in place.
  bq_status upload(void* dst, const void* src_host, size_t bytes);
  bq_status download(void* dst_host, const void* src, size_t bytes);
  bq_status ensure_stage();
  bq_status wait_idle();                           // everything queued on the stream has finished
  bq_status trim();
};

struct bq_tensor {
  std::atomic<int> refs{1};
  bq_device* dev = nullptr;
  int32_t dtype = BQ_F32;
  int32_t rank = 0;
  size_t shape[BQ_MAX_RANK] = {0};
  bq_scheme scheme{};            // meaningful when dtype == BQ_QFLOAT
  // One allocation: values (or float data) at `data`, scales at data + scales_offset.
  void* data = nullptr;
  size_t alloc_bytes = 0;        // 0 => memory is borrowed (not returned to the cache)
  size_t value_bytes = 0;        // dense bytes of the values region (wire size)
  size_t scales_offset = 0;
  size_t num_scales = 0;
  size_t wire_offset = 0;        // two-level schemes: [per-tensor scale][block scales as stored], f32
  bq_tensor* base = nullptr;     // shares the memory of another handle (reshape / to_device)

  size_t numel() const {
    size_t n = 1;
    for (int d = 0; d < rank; ++d) n *= shape[d];
    return n;
  }
  float* scales() const {
    return reinterpret_cast<float*>(static_cast<char*>(data) + scales_offset);
  }
  float* wire_global() const { return reinterpret_cast<float*>(static_cast<char*>(data) + wire_offset); }
  float* wire_scales() const { return wire_global() + 1; }
};

// ---- kernel launchers implemented in the .hip files (all enqueue on `stream`) ------------------
namespace bq {

// Trailing run-block size if every block of `scheme` over `shape` is a run of the flat storage
// (0 for per-tensor), or -1 when blocks are general rectangles.
long run_block(const bq_scheme& scheme, const size_t* shape, int rank);

// Generic rectangle-block kernels (any block shape): slow, complete.
bq_status launch_quantize_rect(const float* x, const size_t* shape, int rank, const size_t* blk,
                               int value, int store, bool dynamic, int scale_dtype, void* values, float* scales,
                               hipStream_t stream);
// Fused quantize kernels with the scheme's scale dtype (quantize.hip). Per tensor: `scale_or_cells`
// is the scale, or (from_absmax) the absmax cells of pass 1, the derived scale then goes to
// scale_out. Run blocks: scales_in null = dynamic (scales_out receives them).
bq_status launch_quantize_per_tensor_small(const float* x, size_t n, float* scale_out, int value, int store, void* values,
                                           int sdt, hipStream_t stream, bool* done);
bq_status launch_quantize_per_tensor(const float* x, size_t n, const float* scale_or_cells, bool from_absmax,
                                     float* scale_out, int value, int store, void* values, int scale_dtype,
                                     hipStream_t stream);
bq_status launch_quantize_run_block(const float* x, size_t n, int block, const float* scales_in, float* scales_out,
                                    int value, int store, void* values, int scale_dtype, hipStream_t stream);
// Calibration::AbsMean: gamma = mean |x| per tensor (blk null; cells: BQ_ABSMAX_CELLS floats of scratch) or per
// rectangle block; and compute_q_params on a symmetric range, scales[i] = (2 range[i]) / (b - a).
bq_status launch_abs_mean(const float* x, const size_t* shape, int rank, const size_t* blk, float* cells, float* gamma,
                          hipStream_t stream);
bq_status launch_scales_from_range(const float* range, size_t n, int value, float* scales, hipStream_t stream);
// dst[i] = scale_to_dtype(src[i]); f32 scales <-> their 2-byte wire form (f16 / bf16).
bq_status launch_round_scales(const float* src, float* dst, size_t n, int scale_dtype, hipStream_t stream);
// Two-level schemes. split: `scales` holds the f32 block scales of a quantize_dynamic and `cells` the
// partial maxima over them (bqk_absmax_f32); on return scales[i] = global * stored[i], the scale
// the kernels use. times_global: the same product from a stored pair.
// Two-level quantize_dynamic in one pass over x: the per-tensor scale from the absmax cells of the whole
// tensor, then the run-block kernel that splits every block scale against it as it computes it.
bq_status launch_two_level_global(const uint32_t* cells, int value, int scale_dtype, float* global_out, hipStream_t stream);
bq_status launch_quantize_run_block_two_level(const float* x, size_t n, int block, const float* global, float* stored_out,
                                              float* scales_out, int value, int store, void* values, int scale_dtype,
                                              hipStream_t stream);
bq_status launch_two_level_split(float* scales, size_t n, const uint32_t* cells, int scale_dtype, float* global_out,
                                 float* stored, hipStream_t stream);
bq_status launch_scales_times_global(const float* stored, const float* global, size_t n, float* scales, hipStream_t stream);
bq_status launch_scales_to_wire(const float* src, void* dst, size_t n, int scale_dtype, hipStream_t stream);
bq_status launch_scales_from_wire(const void* src, float* dst, size_t n, int scale_dtype, hipStream_t stream);
bq_status launch_dequantize_rect(const void* values, const size_t* shape, int rank,
                                 const size_t* blk, const float* scales, int value, int store,
                                 int out_dtype, void* out, hipStream_t stream);

// Plain float GEMM (fallback when no operand stays quantized): C[M,N] = A[M,K] x B[K,N].
bq_status launch_float_matmul(const void* a, int a_dtype, const void* b, int b_dtype, size_t m,
                              size_t k, size_t n, int out_dtype, void* out, hipStream_t stream);

// Tiled MFMA q-GEMM (prefill): out[M,N] = a[M,K] x dequantize(w[K,N]).
bq_status launch_qgemm(const void* a, int a_dtype, const uint32_t* w, const float* scales, size_t m,
                       size_t k, size_t n, int value, unsigned block_words_log2, size_t scales_per_row,
                       bool per_tensor, const float* bias, int out_dtype, void* out, void* workspace,
                       size_t workspace_bytes, unsigned* slices_out, float** part_out, hipStream_t stream);
size_t qgemm_workspace(int a_dtype, size_t m, size_t k, size_t n);

// Small-batch MFMA kernel (2 <= M <= 32), split over K; partials are reduced by the caller.
// Layout ops (layout.hip): out = permute(flip(src)) of quantized values / of an f32 tensor.
bq_status launch_q_gather(const void* src, void* dst, const size_t* src_shape, int rank, const int32_t* axes,
                          const uint8_t* flip, int value, bool native, hipStream_t stream);
bq_status launch_f32_gather(const float* src, float* dst, const size_t* src_shape, int rank, const int32_t* axes,
                            const uint8_t* flip, hipStream_t stream);
// Integer-domain slice / select / gather / expand (layout.hip): output element e with coordinates c reads
// source element base + sum_a c[a] * stride[a], the coordinate of index_dim replaced by
// indices[c[index_dim]] (index_mode 1) or indices[e] (index_mode 2), clamped into [0, index_limit).
bq_status launch_q_index_map(const void* src, void* dst, const size_t* out_shape, int rank, const int64_t* stride, int64_t base,
                             int index_dim, int index_mode, const void* indices, int index_dtype, size_t index_limit, int value,
                             bool src_native, bool dst_native, hipStream_t stream);
bq_status launch_f32_index_map(const float* src, float* dst, const size_t* out_shape, int rank, const int64_t* stride, int64_t base,
                               int index_dim, int index_mode, const void* indices, int index_dtype, size_t index_limit,
                               hipStream_t stream);
bq_status launch_index_map_pair(const void* src, void* dst, const size_t* out_shape, const int64_t* stride, int64_t base, int value,
                                bool src_native, bool dst_native, const float* s_src, float* s_dst, const size_t* s_shape,
                                const int64_t* s_stride, int64_t s_base, int rank, int index_dim, int index_mode, const void* indices,
                                int index_dtype, size_t index_limit, bool* fused, hipStream_t stream);
bq_status launch_q_arg(const void* src, int value, bool native, size_t outer, size_t len, size_t inner, bool want_max, int out_dtype,
                       void* out, hipStream_t stream);
// out[r][c] += bias[c] (out f32 or bf16, in place), and a bf16 -> f32 copy (qmatmul.hip).
bq_status launch_add_bias(void* out, int out_dtype, const float* bias, size_t m, size_t n, hipStream_t stream);
bq_status launch_bf16_to_f32(const uint16_t* src, size_t n, float* dst, hipStream_t stream);
// Small batches of f32 activations on the bf16 matrix cores with split activations (qsplit.hip).
bool split_ok(size_t m, size_t k, size_t n, int x_dtype, int value, int block);
size_t split_workspace(size_t m, size_t k, size_t n);
bq_status launch_qsplit(const void* x, int x_dtype, const uint32_t* w, const float* scales, size_t m, size_t k, size_t n,
                        int value, int block, float* part, unsigned* slices_out, hipStream_t st);
bool skinny_ok(size_t m, size_t k, size_t n, int x_dtype, int value);
size_t skinny_workspace(size_t m, size_t k, size_t n, int x_dtype, int value);
bq_status launch_qskinny(const void* x, int x_dtype, const uint32_t* w, const float* scales, size_t m, size_t k,
                         size_t n, int value, unsigned block_words_log2, size_t scales_per_row, bool per_tensor,
                         float* part, unsigned* slices_out, hipStream_t stream);

bool qgemm_ok(int a_dtype, size_t k, size_t n, int value, size_t scales_per_row);
bool fused_matmul_ok(size_t m, size_t k, size_t n, int lhs_dtype, int value, size_t scales_per_row);

// Per-tensor scale from the absmax cells of bqk_absmax_f32, rounded up to the scale dtype (quantize.hip).
bq_status launch_scale_from_cells(const uint32_t* cells, int value, int scale_dtype, float* scale_out, hipStream_t stream);
// Ternary matmul (qmatmul.hip): out[M,N] = gamma * sum_k t[k][n] * x[m][k] with t in {-1, 0, +1} packed 16 per word.
bq_status launch_ternary_matmul(const float* x, const uint32_t* w, const float* scale, size_t m, size_t k, size_t n,
                                float* out, hipStream_t stream);

// The same product on the bf16 matrix cores, order of the sums given up (qternary.hip): partial products
// of `slices` K slices to `part`, summed by launch_splitk_reduce.
bool ternary_mfma_ok(size_t m, size_t k, size_t n);
size_t ternary_workspace(size_t m, size_t k, size_t n);
bq_status launch_ternary_mfma(const float* x, const uint32_t* w, const float* scale, size_t m, size_t k, size_t n,
                              float* part, unsigned* slices_out, hipStream_t stream);
// out[i] = sum over the slices of part[s][i] (+ bias[i % n]) in a fixed order, to f32 or bf16 (qmatmul.hip).
bq_status launch_splitk_reduce(const float* part, size_t mn, unsigned slices, const float* bias, size_t n,
                               int32_t out_dtype, void* out, hipStream_t stream);

// dst[0..n) = value, as a kernel (safe to record into a HIP graph, unlike a memset node).
bq_status launch_fill_u32(uint32_t* dst, size_t n, uint32_t value, hipStream_t stream);
// dst[0..bytes) = src[0..bytes) by one workgroup (both 16-byte aligned, bytes <= 64 KiB), then *done = seq
// at system scope. One side is pinned host memory: when the host sees seq, src has been read (an upload) or
// dst holds the data (to_host, a download).
bq_status launch_copy_small(const void* src, void* dst, size_t bytes, bool to_host, uint32_t* done, uint32_t seq,
                            hipStream_t stream);
// *word = seq at system scope, behind everything queued on the stream before it.
bq_status launch_host_word(uint32_t* word, uint32_t seq, hipStream_t stream);

// Host-side guard of a kernel's dynamic LDS request (runtime.cpp). A request beyond what the
// current device grants is refused here with BQ_ERR_HIP: it must never reach a launch. The first
// call for a (device, kernel) pair raises the kernel's dynamic-LDS attribute; later ones only check.
bq_status lds_request_status(size_t bytes, size_t device_limit, const char* what);
bq_status configure_dynamic_lds(const void* kernel, size_t bytes, const char* what);

// Device address of the static scratch array of bqk_q_linear_static on the current device
// (qmatmul.hip): resolved once per device.
bq_status static_scratch_ptr(void** out, unsigned** tickets_out = nullptr);
// bqk_q_linear plus the ticket counters that let the split-K kernels finish their own sum in one
// launch (qmatmul.hip, splitk_tail.hpp): `tickets` is kTicketBytes of device memory, zero between
// launches; calls sharing it must not overlap on the device.
// QuantPropagation::Propagate without a float product in memory: where a product ends in the reduction of its
// K slices, that kernel can quantize what it sums -- blocks of 32 or 64 output columns, the scale of each
// from its own absmax -- into `values` / `scales` of a quantized tensor. `done` says whether it did (the
// float output is then not written).
struct RequantOut {
  int value = 0, store = 0, block = 0, sdt = 0;
  bool from_bf16 = false;  // the product is a bf16 tensor: its values are rounded to bf16 before they are quantized
  void* values = nullptr;
  float* scales = nullptr;
  bool done = false;
};
bq_status q_linear_with_tickets(const void* x, int32_t x_dtype, size_t m, size_t k, size_t n, const void* w_values,
                                const float* w_scales, int32_t block, int32_t value, int32_t store, const float* bias,
                                int32_t out_dtype, void* out, void* workspace, size_t workspace_bytes, unsigned* tickets,
                                void* stream, RequantOut* requant = nullptr);

// Counts, over n floats, NaNs into counts[0] and infinities into counts[1] (device u32 cells that
// the kernel adds to; quantize.hip). Used by the validate mode.
bq_status launch_count_nonfinite(const float* x, size_t n, uint32_t* counts, hipStream_t stream);

}  // namespace bq
