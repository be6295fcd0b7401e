/*
 * burnq.h -- C ABI of libburnq_mi355.so: burn's quantized-tensor operations as hand-written
 * gfx950 (MI355X) HIP kernels.
 *
 * The library is what a burn backend crate binds with `extern "C"`: its `impl QTensorOps`
 * forwards each trait method to the function of the same name below.  Two layers:
 *
 *   bq_*   handle level.  Opaque, reference-counted device tensors and one function per
 *          QTensorOps method of the hot path (same names, same argument meaning).  Inputs are
 *          never modified; results are new handles returned through an out-parameter.
 *   bqk_*  kernel level.  Plain device pointers + sizes + a hipStream_t, no allocation, no
 *          handles: for callers that own their memory (another allocator, a torch tensor's
 *          data_ptr(), a captured HIP graph).
 *
 * Every function returns a bq_status (0 = ok).  Where the reference panics (unsupported scheme,
 * "Can't store in u32", shape not divisible by the block) the call returns an error code and
 * bq_last_error() holds the message for the calling thread.  No C++ exception crosses this
 * boundary.  All work is enqueued on the device context's stream and is asynchronous until
 * bq_device_sync / a *_into_data call, like a GPU backend's ops until Backend::sync.
 *
 * There is no CPU path in this library: without a HIP device every compute entry point fails
 * with BQ_ERR_HIP.
 *
 * Reference citations are paths inside the burn tree (crates/...).
 */
#ifndef BURNQ_H
#define BURNQ_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BQ_MAX_RANK 8

typedef int32_t bq_status;
enum {
  BQ_OK = 0,
  BQ_ERR_NULL = 1,               /* a required pointer argument was null */
  BQ_ERR_UNSUPPORTED_SCHEME = 2, /* reference: unimplemented!("Quantization not supported for scheme") */
  BQ_ERR_SHAPE = 3,              /* last dim % num_quants ("Can't store in u32"), dim % block, matmul inner dims */
  BQ_ERR_DTYPE = 4,              /* float/quantized mix-up or unsupported float dtype */
  BQ_ERR_HIP = 5,                /* a HIP runtime call failed (ExecutionError on the Rust side) */
  BQ_ERR_SIZE = 6,               /* host buffer too small / blob shorter than its scheme requires */
  BQ_ERR_UNSUPPORTED_OP = 7,     /* layout op this backend declines (reference: unimplemented!()) */
  BQ_ERR_NONFINITE = 8           /* validate mode: x / scale is NaN (reference: Q::from(NaN).unwrap() panics) */
};

/* DType of a handle. BQ_QFLOAT carries a bq_scheme, like DType::QFloat(scheme). BQ_I32 / BQ_I64 are the
 * index tensors that q_select / q_gather take and q_argmax / q_argmin return. */
enum { BQ_F32 = 0, BQ_BF16 = 1, BQ_QFLOAT = 2, BQ_I32 = 3, BQ_I64 = 4 };

/* QuantValue, QuantStore, quantization level (cubecl_common::quant::scheme, re-exported at
 * crates/burn-std/src/tensor/quantization.rs:4-6). The signed-integer values are implemented:
 * symmetric Q8S (-127,127), Q4S (-7,7), Q2S (-1,1), and full-range Q8F (-128,127) -- the value of
 * QuantScheme::default() -- Q4F (-8,7), Q2F (-2,1). A full-range value differs from its symmetric
 * twin in the quantizer only: scale = 2 absmax / (b - a) with b - a = 255 / 15 / 3, clamp to [a, b];
 * bits, packing, dequantize and q_matmul are the same.
 * Q2S is the ternary value type of BitNet-style weights (-1, 0, +1; 16 per u32, PackedU32 only):
 * quantize / dequantize / layout ops through the general kernels, and q_matmul's multiply-free
 * path for an f32 lhs times a per-tensor Q2S [K, N] weight
 * (crates/burn-ndarray/src/ops/qtensor.rs:431-517); every other 2-bit product dequantizes first, as
 * the reference does. The bqk_ kernel-level entry points take the 8- and 4-bit values. */
enum { BQ_Q8S = 0, BQ_Q4S = 1, BQ_Q2S = 2, BQ_Q8F = 3, BQ_Q4F = 4, BQ_Q2F = 5 };
enum { BQ_LEVEL_TENSOR = 0, BQ_LEVEL_BLOCK = 1 };
enum { BQ_STORE_NATIVE = 0, BQ_STORE_PACKED_U32 = 1 };
/* ScaleDtype. F16 / BF16 / UE4M3: the quantizer divides by the scale rounded UP to the scale dtype
 * (scale_to_dtype, crates/burn-std/src/tensor/quantization.rs:354-368) and the blob stores 2 bytes
 * (UE4M3: 1 byte, the non-negative half of OCP e4m3) per scale (encode_scales, same file). */
enum { BQ_SCALE_F32 = 0, BQ_SCALE_F16 = 1, BQ_SCALE_BF16 = 2, BQ_SCALE_UE4M3 = 3 };

/* The fields of QuantScheme this path reads. `block` holds block_rank extents aligned to the
 * trailing dims (BlockSize::to_dim_vec pads the leading dims with 1). PackedU32 always packs
 * the innermost dim (PackedU32(0)). */
typedef struct bq_scheme {
  uint8_t value;       /* BQ_Q8S | BQ_Q4S | BQ_Q2S | BQ_Q8F | BQ_Q4F | BQ_Q2F */
  uint8_t level;       /* BQ_LEVEL_TENSOR | BQ_LEVEL_BLOCK */
  uint8_t store;       /* BQ_STORE_NATIVE (one i8 per value, whatever its width) | BQ_STORE_PACKED_U32 */
  uint8_t scale_dtype; /* BQ_SCALE_F32 | BQ_SCALE_F16 | BQ_SCALE_BF16 | BQ_SCALE_UE4M3 */
  uint8_t block_rank;
  uint8_t tensor_scale; /* block level only: 1 = an f32 per-tensor scale on top of the block scales (below) */
  uint8_t reserved[2];
  uint8_t block[BQ_MAX_RANK];
} bq_scheme;
/* Two-level schemes (`.per_block(b, dtype).per_tensor(ScaleDtype::F32)`; global_scale_dtype,
 * crates/burn-std/src/tensor/quantization.rs:134-136): the scale of a block is global * s_block, the
 * block scales are stored in the scale dtype and the per-tensor scale as one f32 behind them
 * (QuantizedBytes::new, same file :245-266). quantize_dynamic splits the block scales so that the
 * largest lands on the scale dtype's largest value (normalize_scales,
 * crates/burn-backend/src/quantization/scheme.rs:106-134), which the reference allows for scale
 * dtypes whose largest value does not exceed f16's: BQ_SCALE_F16 and BQ_SCALE_UE4M3. */

typedef struct bq_device bq_device; /* one GPU: stream, allocation cache, workspace */
typedef struct bq_tensor bq_tensor; /* ref-counted device tensor: float, or values || scales */

/* ------------------------------------------------------------------ library / device */

/* Message of the last failing call on this thread ("" if none). */
const char* bq_last_error(void);
/* Backend::device_count -- crates/burn-backend/src/backend/base.rs:154-249. */
bq_status bq_device_count(int32_t* count);
/* Opens (or returns the already open) context of GPU `ordinal`. Contexts live until
 * bq_device_close; handles keep a pointer to theirs. */
bq_status bq_device_open(int32_t ordinal, bq_device** out);
bq_status bq_device_close(bq_device* dev);
/* Backend::sync(device) -- base.rs:154-249: blocks until everything enqueued has finished. (It queues one
 * small kernel of its own that reports through pinned memory, and reads that memory for a short while before
 * it blocks in the runtime: 4-5 us sooner than hipStreamSynchronize after short work. Not while a graph is
 * being captured: an error, as hipStreamSynchronize gives there.) */
bq_status bq_device_sync(bq_device* dev);
/* The hipStream_t all work of this context is enqueued on. */
void* bq_device_stream(bq_device* dev);
/* Returns cached, currently unused device allocations to the driver. */
bq_status bq_device_trim(bq_device* dev);
/* Validate mode (off by default). While on, bq_quantize / bq_quantize_dynamic first count the
 * NaN and infinite inputs (and scales) on the device and fail with BQ_ERR_NONFINITE where the
 * reference panics: a quotient x / scale that is NaN cannot become an integer
 * (crates/burn-ndarray/src/ops/quantization.rs:128-133, `Q::from(..).unwrap()`). That is a NaN input
 * or scale, or an infinite input against an infinite scale -- which includes every infinite input
 * of a quantize_dynamic, whose own range makes the scale infinite. The check synchronises the
 * stream (a debugging aid; refused during graph capture). Off, such inputs give unspecified
 * integers. */
bq_status bq_device_set_validate(bq_device* dev, int32_t on);
/* Activations against a quantized weight keep at least 16 significant bits per product up to 32
 * rows; from 33 rows on the fast kernel multiplies bf16(activation) by bf16(s * q), about 2e-3 of the
 * largest output, inside the 1e-2 the reference's own tests allow
 * (crates/burn-backend-tests/tests/tensor/float/quantization/ops/matmul.rs) but far from its f32
 * sgemm: on a 4096-deep product a few outputs in a million leave burn's elementwise rule
 * (|y - y'| < max(1e-2 max(|y|, |y'|), 1e-2)). on != 0 makes q_matmul / q_linear on this device
 * multiply such products the reference's way instead -- weights dequantized to f32, f32 matrix
 * product, for f32 and bf16 activations alike -- at a fraction of the speed, and makes the ternary
 * product (Q2S weights) keep the reference's order of additions bit for bit instead of running on
 * the matrix cores. Off by default. No counterpart in the reference. */
bq_status bq_device_set_f32_matmul_exact(bq_device* dev, int32_t on);
/* HIP-event stopwatch on the context's stream (what Backend::sync-bracketed benches measure,
 * without the host round trip): start, enqueue work, stop -> elapsed milliseconds. */
bq_status bq_timer_start(bq_device* dev);
bq_status bq_timer_stop(bq_device* dev, float* elapsed_ms);

/* HIP-graph capture of the context's stream: every bq_ and bqk_ call issued between begin and end
 * is recorded instead of executed, and bq_graph_launch replays the whole sequence with one
 * submission -- what a decode loop (a few ~10 us kernels per call) needs to stop being bound by
 * launch latency. No counterpart in the reference (its GPU backends batch through a lazy
 * op stream, crates/burn-fusion). Rules: run the sequence once eagerly first (so the allocation
 * cache and the split-K workspace exist), make no *_into_data / *_from_data / sync / timer call
 * while capturing, and keep every tensor created during capture alive for as long as the graph is
 * replayed (their memory is baked into it). The kernels clear their scratch with fill kernels,
 * never memset nodes.
 * What the library allocates for itself stays valid for the graph's lifetime: temporaries created
 * and released inside a captured call (the f32 copy of a bf16 bias, dequantized operands of the
 * general q_matmul path), tensors created during the capture and released afterwards, and the
 * split-K workspace (a larger one requested later does not free the one a graph addresses) all
 * return to the allocator only at bq_graph_release. Tensors that existed before the capture and
 * are read by it are the caller's to keep alive, with their contents. One capture per device at a
 * time; bq_device_trim is refused while one is open. */
typedef struct bq_graph bq_graph;
bq_status bq_graph_begin_capture(bq_device* dev);
bq_status bq_graph_end_capture(bq_device* dev, bq_graph** out);
bq_status bq_graph_launch(bq_graph* graph);
bq_status bq_graph_release(bq_graph* graph);

/* ------------------------------------------------------------------ handles */

bq_status bq_tensor_retain(bq_tensor* t);
bq_status bq_tensor_release(bq_tensor* t);
int32_t bq_tensor_rank(const bq_tensor* t);
/* Logical shape (of the unpacked values for a quantized tensor). */
bq_status bq_tensor_shape(const bq_tensor* t, size_t* shape_out /* [rank] */);
int32_t bq_tensor_dtype(const bq_tensor* t);
bq_status bq_tensor_scheme(const bq_tensor* t, bq_scheme* out);
/* Device pointers: float data or packed/native values; block or tensor scales (f32). */
void* bq_tensor_data_ptr(const bq_tensor* t);
void* bq_tensor_scales_ptr(const bq_tensor* t);
size_t bq_tensor_num_scales(const bq_tensor* t);

/* ------------------------------------------------------------------ float tensors
 * The slice of FloatTensorOps the path needs (float_from_data / float_into_data,
 * crates/burn-backend/src/backend/ops/tensor.rs). Row-major, contiguous. A host buffer is only
 * borrowed: bq_float_from_data / bq_q_from_data have read it when they return (the transfer to
 * the device is then queued on the device's stream, ahead of every later call), and
 * bq_float_into_data / bq_q_into_data return with the data in place. */
bq_status bq_float_from_data(bq_device* dev, const void* host, int32_t dtype, const size_t* shape,
                             int32_t rank, bq_tensor** out);
bq_status bq_float_into_data(const bq_tensor* t, void* host, size_t capacity_bytes);
/* Uninitialised float tensor (for callers that fill it on the device). */
bq_status bq_float_empty(bq_device* dev, int32_t dtype, const size_t* shape, int32_t rank,
                         bq_tensor** out);
/* Wraps device memory owned by the caller (not freed on release); must outlive the handle. */
bq_status bq_float_from_device_ptr(bq_device* dev, void* device_ptr, int32_t dtype,
                                   const size_t* shape, int32_t rank, bq_tensor** out);
/* float_matmul for 2-D (or [.., M, K] x [K, N]) operands; f32 accumulation. Used by q_matmul
 * when no operand stays quantized. */
bq_status bq_float_matmul(const bq_tensor* lhs, const bq_tensor* rhs, bq_tensor** out);

/* ------------------------------------------------------------------ QTensorOps
 * crates/burn-backend/src/backend/ops/qtensor.rs:123-1324; the CPU semantics these reproduce bit
 * for bit are burn-ndarray's (crates/burn-ndarray/src/ops/qtensor.rs, ops/quantization.rs). */

/* Whether this backend takes tensors of `scheme`, whatever their shape: what the binding answers
 * Backend::dtype_usage(DType::QFloat(scheme)) with (pattern: crates/burn-ndarray/src/backend.rs:98-119).
 * The values, stores and levels this library implements, under the reference's `quantizable` rule
 * (crates/burn-std/src/tensor/quantization.rs:113-128): a scale dtype with a round-up rule, and for a
 * two-level scheme block scales whose largest value does not exceed f16's (F16, UE4M3) under an f32
 * per-tensor scale. BQ_OK, or BQ_ERR_UNSUPPORTED_SCHEME with the reason in bq_last_error().
 * (bq_quantize_two_level with given parameters is laxer about the block scale dtype, as the
 * reference's quantize is; this is the answer for schemes to quantize dynamically against.) */
bq_status bq_scheme_supported(const bq_scheme* scheme);

/* Bytes of the TensorData blob for `shape` under `scheme`: values || block scales, dense.
 * quantized_data_len -- crates/burn-std/src/tensor/quantization.rs:400-407. */
bq_status bq_quantized_data_len(const bq_scheme* scheme, const size_t* shape, int32_t rank,
                                size_t* len_out);
/* QTensorOps::q_from_data (qtensor.rs:134). `bytes` is the QuantizedBytes blob
 * (burn-std .../quantization.rs:204-353); device layout == wire layout as on the packed backends
 * (crates/burn-cubecl/src/ops/qtensor.rs:219-250). Native-store blobs are accepted for Q8S. */
bq_status bq_q_from_data(bq_device* dev, const uint8_t* bytes, size_t len, const size_t* shape,
                         int32_t rank, const bq_scheme* scheme, bq_tensor** out);
/* QTensorOps::q_into_data (qtensor.rs:187): stream-ordered copy back + sync. */
bq_status bq_q_into_data(const bq_tensor* t, uint8_t* bytes, size_t capacity, size_t* len_out);
/* QTensorOps::quantize (qtensor.rs:137): `scales` is an f32 tensor of params_shape entries.
 * q = clamp(round_half_away(x / (s == 0 ? 0.1 : s)), a, b); the stored scale stays s
 * (burn-ndarray/src/ops/qtensor.rs:82-186, ops/quantization.rs:78-133). */
/* (A two-level scheme takes its parameters through bq_quantize_two_level.) */
bq_status bq_quantize(const bq_tensor* x, const bq_scheme* scheme, const bq_tensor* scales,
                      bq_tensor** out);
/* QTensorOps::quantize with QuantizationParametersPrimitive { scales, global: Some(..) }
 * (crates/burn-backend/src/quantization/parameters.rs:12-20) for a two-level scheme: `global` is an
 * f32 tensor of one element; every block is quantized against global * scale_to_dtype(s_block)
 * (quantize_per_block, crates/burn-ndarray/src/ops/qtensor.rs:519-538). */
bq_status bq_quantize_two_level(const bq_tensor* x, const bq_scheme* scheme, const bq_tensor* scales,
                                const bq_tensor* global, bq_tensor** out);
/* QTensorOps::quantize_dynamic (qtensor.rs:144-149), overridden as one fused pass per block
 * scheme / two passes per tensor: scale = (2 * max|x|) / (b - a)
 * (crates/burn-backend/src/quantization/scheme.rs:44-104), then quantize as above. */
bq_status bq_quantize_dynamic(const bq_tensor* x, const bq_scheme* scheme, bq_tensor** out);
/* compute_range under Calibration::AbsMean (crates/burn-backend/src/quantization/scheme.rs:57-69; the
 * calibration BitNet-style ternary weights are made with, crates/burn-std/src/tensor/quantization.rs:55-62):
 * gamma = mean(|x|) over the tensor or over each block; the range is [-gamma, +gamma]. gamma_out is
 * an f32 tensor of params_shape entries ([1], or dims / block) holding gamma, the range's maximum (its
 * minimum is the negation). A two-level scheme is refused, as the reference asserts. The mean is a
 * sum in a fixed order divided by the count (the reference's order is its backend's; its tests
 * compare within Tolerance::default(), 0.5 %). */
bq_status bq_compute_range_abs_mean(const bq_tensor* x, const bq_scheme* scheme, bq_tensor** gamma_out);
/* What Quantizer::map_float does under Calibration::AbsMean (crates/burn-core/src/module/quantize.rs:47-49):
 * compute_range -> compute_q_params -> quantize, i.e. scale = (2 gamma) / (b - a) -- gamma itself for
 * the ternary Q2S -- and q = clamp(round(x / scale), a, b), without leaving the device. */
bq_status bq_quantize_abs_mean(const bq_tensor* x, const bq_scheme* scheme, bq_tensor** out);
/* QTensorOps::dequantize (qtensor.rs:152): x = (s == 0 ? 0.1 : s) * q, to BQ_F32 or BQ_BF16
 * (bf16 = f32 result rounded to nearest even, TensorData::convert_dtype). */
bq_status bq_dequantize(const bq_tensor* q, int32_t float_dtype, bq_tensor** out);
/* QTensorOps::q_matmul (qtensor.rs:498-544) with QuantPropagation::Inhibit: either operand may be
 * float or quantized, the result is a float tensor. Output dtype = the float operand's dtype
 * (f32 if both are quantized), as burn-ndarray/src/ops/qtensor.rs:234-239. */
bq_status bq_q_matmul(const bq_tensor* lhs, const bq_tensor* rhs, bq_tensor** out);
/* Same with an explicit output dtype (the prefill config wants bf16 in, f32 out). */
bq_status bq_q_matmul_as(const bq_tensor* lhs, const bq_tensor* rhs, int32_t out_dtype,
                         bq_tensor** out);
/* q_matmul under QuantPropagation::Propagate (burn-ndarray/src/ops/qtensor.rs:262-265; the setting
 * is crates/burn-std/src/tensor/quantization.rs:28-75): the float product is quantized again,
 * quantize_dynamic with the scheme of the quantized operand (the rhs's when both are), and a
 * quantized tensor is returned. The product has the float operand's dtype, as there: with a bf16
 * operand it is the bf16 product whose values are quantized. */
bq_status bq_q_matmul_propagate(const bq_tensor* lhs, const bq_tensor* rhs, bq_tensor** out);
/* linear with a quantized weight (crates/burn-tensor/src/tensor/module.rs:527-567, what
 * nn::Linear::forward reaches after Module::quantize_weights,
 * crates/burn-core/src/module/quantize.rs:40-53): x [.., d_input] (f32 or bf16), weight a quantized
 * [d_input, d_output], bias NULL or a float [d_output]. The leading dims of x fold into the rows of
 * one product against the packed weight, as the reference does; out [.., d_output] = x @ weight +
 * bias, with the bias added in f32 by the kernel that writes the output (for an f32 output that is
 * the reference's own order of operations: the rounded sum, then one addition). out_dtype: BQ_F32,
 * BQ_BF16, or -1 for x's dtype. */
bq_status bq_q_linear(const bq_tensor* x, const bq_tensor* weight, const bq_tensor* bias,
                      int32_t out_dtype, bq_tensor** out);
/* QTensorOps::q_to_device (qtensor.rs:164). Same device: a new reference. */
bq_status bq_q_to_device(const bq_tensor* t, bq_device* dev, bq_tensor** out);
/* QTensorOps::q_reshape (qtensor.rs:176). Metadata-only; declined (BQ_ERR_UNSUPPORTED_OP) when
 * blocks or packed words would no longer be runs of the flat storage -- the same restriction as
 * crates/burn-cubecl/src/ops/base.rs:298-442. */
bq_status bq_q_reshape(const bq_tensor* t, const size_t* shape, int32_t rank, bq_tensor** out);
/* QTensorOps::q_swap_dims / q_permute / q_flip (qtensor.rs:240-262): values move and block
 * scales move with their blocks (burn-ndarray/src/ops/qtensor.rs:300-347). The result is a new
 * dense tensor (the block of the scheme is permuted with the axes, so a [1, 32] block becomes
 * [32, 1] under a transpose). An axis out of bounds or repeated, which the reference panics on,
 * returns BQ_ERR_SHAPE, as does a packed sub-byte result whose last dim is not a whole number of
 * words (a Q8S result of that kind is stored natively: same bytes, one per value; natively stored
 * tensors of any value width permute freely).
 * q_flip flips the values and keeps every parameter where it is, block scales included, as the
 * reference does (burn-ndarray/src/ops/qtensor.rs:338-347): a value flipped into another block
 * is dequantized with that block's scale. */
bq_status bq_q_swap_dims(const bq_tensor* t, int32_t dim1, int32_t dim2, bq_tensor** out);
bq_status bq_q_permute(const bq_tensor* t, const int32_t* axes, int32_t rank, bq_tensor** out);
bq_status bq_q_flip(const bq_tensor* t, const int32_t* axes, int32_t n_axes, bq_tensor** out);

/* ------------------------------------------------------------------ integer-domain ops
 * The QTensorOps methods the reference's CPU backend runs on the stored integers without
 * dequantizing (crates/burn-ndarray/src/ops/qtensor.rs:349-430; the trait's defaults,
 * crates/burn-backend/src/backend/ops/qtensor.rs:210-322 and :948-1041, dequantize, run the float op
 * and quantize again, which changes the scale). The result keeps the source's scheme and scales:
 * dequantize(op(q)) equals op(dequantize(q)) bit for bit. Block scales follow their blocks where the
 * op moves whole blocks; where it would cut into blocks the call returns BQ_ERR_UNSUPPORTED_OP and the
 * binding falls back to the trait's default. A Q8S result whose last dim no longer fills packed words
 * is stored natively (same bytes), as q_permute does; sub-byte results must fill their words
 * (BQ_ERR_SHAPE). */
/* IntTensorOps::int_from_data / int_into_data for index tensors (dtype BQ_I32 or BQ_I64, dense row-major). */
bq_status bq_int_from_data(bq_device* dev, const void* host, int32_t dtype, const size_t* shape, int32_t rank,
                           bq_tensor** out);
bq_status bq_int_into_data(const bq_tensor* t, void* host, size_t capacity_bytes);
/* QTensorOps::q_slice (qtensor.rs:296): slice a of n_slices is Slice { start: starts[a], end: ends[a] (INT64_MAX for
 * None), step: steps[a] } with burn's rules (crates/burn-std/src/tensor/slice.rs:493-545): negative indices count from
 * the end, ranges are clamped into the dim, the output holds ceil(len / |step|) values, a negative step walks the range
 * backwards from its last value. Dims past n_slices are kept whole. A dim with blocks wider than 1 takes step 1 and
 * ranges of whole blocks. */
bq_status bq_q_slice(const bq_tensor* t, const int64_t* starts, const int64_t* ends, const int64_t* steps, int32_t n_slices,
                     bq_tensor** out);
/* QTensorOps::q_select (qtensor.rs:274): out[.., i, ..] = t[.., indices[i], ..] along `dim`; indices 1-D. An index outside
 * the dim, which the reference panics on, is clamped into it. Blocks must be 1 wide along `dim`. */
bq_status bq_q_select(const bq_tensor* t, int32_t dim, const bq_tensor* indices, bq_tensor** out);
/* QTensorOps::q_gather (qtensor.rs:312): out[c] = t[c with c[dim] replaced by indices[c]]; indices has t's rank and t's
 * extents on every other dim (crates/burn-ndarray/src/ops/base.rs:106-138). Per-tensor schemes (or blocks of 1). */
bq_status bq_q_gather(int32_t dim, const bq_tensor* t, const bq_tensor* indices, bq_tensor** out);
/* QTensorOps::q_expand (qtensor.rs:210): broadcast to `shape` (trailing dims aligned; a dim of 1 repeats). */
bq_status bq_q_expand(const bq_tensor* t, const size_t* shape, int32_t rank, bq_tensor** out);
/* QTensorOps::q_argmax / q_argmin (qtensor.rs:948, :1037): index along `dim` of the largest / smallest value, the first one
 * on ties (crates/burn-ndarray/src/ops/base.rs:1727-1750), `dim` kept with extent 1; out_dtype BQ_I32 or BQ_I64. Compared
 * on the integers: per-tensor schemes, or blocks that span exactly the reduced dim. */
bq_status bq_q_argmax(const bq_tensor* t, int32_t dim, int32_t out_dtype, bq_tensor** out);
bq_status bq_q_argmin(const bq_tensor* t, int32_t dim, int32_t out_dtype, bq_tensor** out);

/* ------------------------------------------------------------------ burnpack containers
 * The on-disk format quantized modules are saved in (crates/burn-pack: base.rs:13-60 header and
 * alignment, lib.rs:52-82 layout, writer.rs:257-314 offsets, reader.rs validation). A quantized
 * tensor's bytes in the file are its QuantizedBytes blob (crates/burn-store/src/tensor_snapshot.rs:
 * 253-262, crates/burn-pack/src/writer.rs:310-340), i.e. what bq_q_from_data takes: a tensor loads
 * out of the mapped file with one host-to-device copy when its value bytes are a multiple of 256
 * (two otherwise). DType tags follow the order of burn's DType enum
 * (crates/burn-std/src/tensor/dtype.rs:10-26). */
enum {
  BQ_PACK_F64 = 0, BQ_PACK_F32, BQ_PACK_FLEX32, BQ_PACK_F16, BQ_PACK_BF16, BQ_PACK_I64, BQ_PACK_I32, BQ_PACK_I16,
  BQ_PACK_I8, BQ_PACK_U64, BQ_PACK_U32, BQ_PACK_U16, BQ_PACK_U8, BQ_PACK_BOOL, BQ_PACK_QFLOAT
};
typedef struct bq_pack bq_pack;               /* an open container (Reader) */
typedef struct bq_pack_writer bq_pack_writer; /* tensors collected for writing (Writer) */
typedef struct bq_pack_entry {                /* one TensorDescriptor + where its bytes are */
  const char* name;      /* owned by the bq_pack */
  int32_t dtype;         /* BQ_PACK_* */
  int32_t rank;
  size_t shape[BQ_MAX_RANK];
  uint64_t data_begin, data_end; /* data_offsets, relative to the data section */
  int32_t has_param_id;
  uint64_t param_id;
  int32_t has_scheme;    /* QFloat whose scheme this library wrote and could read back */
  bq_scheme scheme;
  const uint8_t* data;   /* the tensor's bytes inside the mapped / borrowed container */
} bq_pack_entry;
/* aligned_data_section_start (base.rs:52-60): where the data section begins for a metadata size. */
size_t bq_pack_data_section_start(size_t metadata_size);
/* Reader::from_file / from_bytes. Only header and metadata are parsed; the file is memory-mapped
 * and tensor bytes are touched when loaded. copy = 0 borrows `bytes` (must outlive the pack).
 * Rejections follow the reader's: bad magic / version (BQ_ERR_DTYPE), a short header, oversized
 * metadata, more tensors or bytes than the limits, a file smaller than its descriptors claim
 * (BQ_ERR_SIZE). */
bq_status bq_pack_open(const char* path, bq_pack** out);
bq_status bq_pack_from_bytes(const uint8_t* bytes, size_t len, int32_t copy, bq_pack** out);
bq_status bq_pack_close(bq_pack* pack);
int64_t bq_pack_num_tensors(const bq_pack* pack);
/* Entries in name order (the reference iterates a BTreeMap). */
bq_status bq_pack_entry_at(const bq_pack* pack, int64_t index, bq_pack_entry* out);
bq_status bq_pack_find(const bq_pack* pack, const char* name, bq_pack_entry* out);
/* A user metadata value, or NULL. */
const char* bq_pack_metadata(const bq_pack* pack, const char* key);
/* The named tensor as a device tensor. QFloat entries take their scheme from `scheme`; NULL is
 * accepted when the file was written by this library (how burn's own writer serializes a
 * QuantScheme is decided outside the reference tree and is not relied on). F32 / BF16 entries load
 * as float tensors; other dtypes are declined. */
bq_status bq_pack_load(const bq_pack* pack, const char* name, const bq_scheme* scheme, bq_device* dev, bq_tensor** out);
/* Writer: tensors are laid out in the order added, each at the next 256-byte boundary; descriptors
 * are emitted in name order; a duplicate name or a byte length that cannot describe the declared
 * dtype and shape is refused (writer.rs:264-330). add_tensor copies a device tensor back first. */
bq_status bq_pack_writer_new(bq_pack_writer** out);
bq_status bq_pack_writer_free(bq_pack_writer* w);
bq_status bq_pack_writer_set_metadata(bq_pack_writer* w, const char* key, const char* value);
bq_status bq_pack_writer_add_bytes(bq_pack_writer* w, const char* name, int32_t dtype, const bq_scheme* scheme,
                                   const size_t* shape, int32_t rank, const uint8_t* data, size_t len,
                                   int32_t has_param_id, uint64_t param_id);
bq_status bq_pack_writer_add_tensor(bq_pack_writer* w, const char* name, const bq_tensor* t, int32_t has_param_id,
                                    uint64_t param_id);
bq_status bq_pack_writer_size(const bq_pack_writer* w, size_t* size_out);
bq_status bq_pack_writer_write_into(const bq_pack_writer* w, uint8_t* buffer, size_t capacity, size_t* size_out);
bq_status bq_pack_writer_write_file(const bq_pack_writer* w, const char* path);

/* ------------------------------------------------------------------ kernel level
 * Plain pointers, no allocation. `stream` is a hipStream_t (NULL = the default stream).
 * A "run block" scheme is one whose blocks are `block` consecutive elements of the flat storage
 * (block = [B] on the last dim); `block` = 0 means per-tensor. `store`/`value` as in bq_scheme. */

/* No counterpart in the reference: a hardware self-check. The quantize kernels replace the IEEE
 * divisions of the reference arithmetic (x / s, 1 / s, (2*amax) / (b-a)) by reciprocal + fma
 * correction sequences that are exact; this launches exhaustive comparisons on the device and
 * leaves five mismatch counts in mismatches_dev[0..4] (device memory, 5 x u64):
 *   [0] reciprocal 1 / s, [1] Q8S scale, [2] Q4S scale: all 2^23 mantissas x every exponent the
 *       shortcut is used for;
 *   [3] quotient x / s, bit for bit, and [4] the integer it quantizes to: all 2^23 scale mantissas
 *       (lowest, middle and highest exponent of the shortcut) x every rounding tie (k + 1/2) * s,
 *       k in [-128, 127], with two neighbours of x on either side.
 * All five must read 0. */
bq_status bqk_selftest_division(uint64_t* mismatches_dev, void* stream);
/* No counterpart in the reference: a plain device-to-device streaming copy of `bytes` bytes
 * (16-byte aligned, multiple of 16). It is the kernel of known traffic that the HBM byte
 * counters of a profile are calibrated against, and the practical ceiling the streaming
 * kernels are compared with. */
bq_status bqk_copy(const void* src, void* dst, size_t bytes, void* stream);
/* No counterpart in the reference: the host-side check every kernel with a dynamic LDS request
 * goes through before it is launched. BQ_ERR_HIP when `bytes` exceeds `device_limit` (the launch
 * is refused; an over-sized request must never reach the GPU), BQ_OK otherwise. Exported so the
 * rule can be tested without a GPU. */
bq_status bqk_lds_request_status(size_t bytes, size_t device_limit);
/* max |x| over n floats, as BQ_ABSMAX_CELLS partial maxima (bit patterns of non-negative f32):
 * every cell of absmax_cells[0 .. BQ_ABSMAX_CELLS) is written, none needs initialising, and the
 * result is the largest cell (one cell per workgroup, so no atomics).
 * Replaces compute_range's float_min + float_max
 * (crates/burn-backend/src/quantization/scheme.rs:44-56). */
#define BQ_ABSMAX_CELLS 512
bq_status bqk_absmax_f32(const float* x, size_t n, uint32_t* absmax_cells, void* stream);
/* Second pass of a per-tensor quantize_dynamic: scale = (2 * max cell) / (b - a) is derived on
 * the device, stored to scale_out[0], and x is quantized against it (compute_q_params + quantize,
 * scheme.rs:75-93 and burn-ndarray/src/ops/qtensor.rs:126-136, without a host round trip). */
bq_status bqk_quantize_per_tensor_from_absmax(const float* x, size_t n,
                                              const uint32_t* absmax_cells, float* scale_out,
                                              int32_t value, int32_t store, void* values,
                                              void* stream);
/* scales[i] = (2 * absmax[i]) / (b - a): compute_q_params (scheme.rs:75-93) for n entries. */
bq_status bqk_scales_from_absmax(const float* absmax, size_t n, int32_t value, float* scales,
                                 void* stream);
/* Per-tensor quantize against the device-resident scale[0]. `values` is i8 (native) or u32 words. */
bq_status bqk_quantize_per_tensor(const float* x, size_t n, const float* scale, int32_t value,
                                  int32_t store, void* values, void* stream);
/* Fused range + q_params + quantize for run blocks: one pass over x. */
bq_status bqk_quantize_dynamic_block(const float* x, size_t n, int32_t block, int32_t value,
                                     int32_t store, void* values, float* scales, void* stream);
/* Quantize run blocks against given scales. */
bq_status bqk_quantize_block(const float* x, size_t n, int32_t block, const float* scales,
                             int32_t value, int32_t store, void* values, void* stream);
/* Dequantize n values; block = 0 reads scales[0]. out_dtype BQ_F32 | BQ_BF16. */
bq_status bqk_dequantize(const void* values, size_t n, int32_t block, const float* scales,
                         int32_t value, int32_t store, int32_t out_dtype, void* out, void* stream);
/* out[M,N] = lhs[M,K] (f32 or bf16) x dequantize(W[K,N]); W is Q8S/Q4S PackedU32 (or Q8S native)
 * with per-tensor (block = 0) or run-block scales along N. `workspace` (>= bqk_q_matmul_workspace
 * bytes, 256-byte aligned, may be NULL when that is 0) holds split-K partials.
 * Arithmetic: sums are f32 throughout. An f32 lhs with M <= 4, and a bf16 lhs with M <= 2 (widened
 * exactly), are multiplied in f32; up to M = 32 the products otherwise keep at least 16
 * significant bits of lhs x scale (exact integer weights on the bf16 matrix cores, or f32 where
 * that kernel does not apply); above that, and for layouts those kernels do not take, bf16(lhs)
 * is multiplied by bf16(scale x q). All within q_matmul's 1e-2. */
size_t bqk_q_matmul_workspace(size_t m, size_t k, size_t n, int32_t lhs_dtype, int32_t value);
bq_status bqk_q_matmul(const void* lhs, int32_t lhs_dtype, size_t m, size_t k, size_t n,
                       const void* w_values, const float* w_scales, int32_t block, int32_t value,
                       int32_t store, int32_t out_dtype, void* out, void* workspace,
                       size_t workspace_bytes, void* stream);

/* bqk_q_matmul plus a linear layer's bias (module.rs:564-567): out[r][c] = sum_k x[r][k] * w[k][c]
 * + bias[c]. bias: n f32 values, 16-byte aligned, or NULL. Same workspace as bqk_q_matmul. */
bq_status bqk_q_linear(const void* x, int32_t x_dtype, size_t m, size_t k, size_t n,
                       const void* w_values, const float* w_scales, int32_t block, int32_t value,
                       int32_t store, const float* bias, int32_t out_dtype, void* out, void* workspace,
                       size_t workspace_bytes, void* stream);

/* No counterpart in the reference: bqk_q_linear for callers that cannot allocate or bring a
 * workspace -- code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
 * Same arguments and same results (bit for bit: the same kernels in the same order) as
 * bqk_q_linear, minus the workspace: split-K partials and the bf16 copy of an f32 lhs go to a
 * static device array of BQK_STATIC_SCRATCH_BYTES that each GPU the library runs on holds until
 * the process ends. A product whose kernel needs more scratch than that is refused with
 * BQ_ERR_SIZE before anything is launched (16 MiB holds the partials of the decode and small-batch
 * kernels, M <= 32, on a [4096, 14336] weight; the need never exceeds bqk_q_matmul_workspace()).
 * The call allocates nothing (no hipMalloc / hipFree); the array's device address is looked up
 * once per device, at bq_device_open or at the first call on that device. All calls on one GPU
 * share the array: calls that overlap there (different streams or threads) race; calls on one
 * stream are ordered and need no clearing between them (every cell a call reads it has written). */
#define BQK_STATIC_SCRATCH_BYTES (16u << 20)
bq_status bqk_q_linear_static(const void* x, int32_t x_dtype, size_t m, size_t k, size_t n,
                              const void* w_values, const float* w_scales, int32_t block, int32_t value,
                              int32_t store, const float* bias, int32_t out_dtype, void* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* BURNQ_H */
