/*
 * CPU oracle for burn's quantized-tensor path.  TEST INFRASTRUCTURE ONLY.
 *
 * This is a plain-C restatement of what burn-ndarray (the reference CPU backend) computes
 * for quantize / quantize_dynamic / dequantize / q_matmul, plus the QuantizedBytes wire
 * format and PackedU32 word layout.  It exists so that the HIP kernels can be checked
 * bit for bit; it is never linked into, imported by, or called from the product library.
 * Only the tests, the smoke check and the benchmark's cpu_baseline leg may use it.
 *
 * Every function names the reference source it follows (paths relative to the burn tree).
 *
 * Pinning status (what fixes each function besides this restatement):
 *   bqo_value_range      Q8F (-128,127): burn-flex/src/ops/qtensor.rs:665-692; Q4F (-8,7), Q2F (-2,1): PARITY
 *                        UNPINNED (the same "full-range" rule, no reference-held number);
 *                        Q8S (-127,127): known answers in burn-ndarray/src/ops/quantization.rs:164-177;
 *                        Q4S (-7,7): the 16 packed words <-> 128 values vector in
 *                        burn-std/src/tensor/quantization.rs:581-602 (it is quantize(arange(128))).
 *   bqo_compute_range    burn-backend-tests .../quantization/calibration.rs:7-59
 *   bqo_compute_range_abs_mean  burn-backend-tests .../quantization/calibration.rs:62-125 (gamma 0.45 per
 *                        tensor; 0.45 and 0.25 per block of 4)
 *   bqo_compute_q_params burn-backend-tests .../quantization/scheme.rs:9-49, ops/quantize.rs:171-206
 *   bqo_quantize         quantization.rs:164-199 (ndarray), ops/quantize.rs:25-93
 *   bqo_dequantize       quantization.rs:164-216 (exact assert_eq on the dequantized floats)
 *   bqo_pack_u32/unpack  burn-std/src/tensor/quantization.rs:551-602
 *   bqo_quantized_data_len  burn-store/src/tensor_snapshot.rs:517-541
 *   bqo_encode/decode    burn-std/src/tensor/quantization.rs:605-625, tests .../quantization/data.rs:6-50
 *   bqo_block_of         ops/quantize.rs:171-206 + brute force against a reshape on small shapes
 *   bqo_q_matmul         ops/matmul.rs:141-168, :204-249 (known 3x4 and 3x16 products)
 *   bqo_ternary_matmul   burn-ndarray/src/ops/qtensor.rs:431-517 restated loop for loop; its values are
 *                        Q2S = {-1, 0, +1}: the range (-1, 1) is what that function's match arms and doc
 *                        comment state (QuantValue::range() itself lives in cubecl-common, absent).
 *                        Checked the way the reference checks it (ops/extended/ternary_matmul.rs, its
 *                        inputs): equal to dequantize-then-matmul within f32 rounding, and exactly 0
 *                        for an all-zero weight; the quantized ternary values of that test's weight
 *                        follow from the same round / clamp rule the Q8S / Q4S vectors pin.
 *   bqo_scale_to_dtype   f32 / f16 / bf16. The rule is the reference's doc comment (burn-std
 *                        .../quantization.rs:354-368: "the smallest value representable by the scale
 *                        dtype that is no smaller"); its arithmetic lives in cubecl-common (absent).
 *                        For IEEE f16 / bf16 the rule fixes the result: checked by brute force over
 *                        all 65 536 patterns of each format (representable values are fixed points,
 *                        the f32 neighbour above goes to the next representable value, the one
 *                        below stays) and by the reference test's own scales and properties
 *                        (:631-657: rounded >= scale, the codec leaves a rounded scale alone).
 *                        UE4M3 (one byte, the non-negative half of OCP e4m3: bias 7, 3 mantissa
 *                        bits, subnormals m * 2^-9, largest value 448, 0x7F NaN; decoded as the
 *                        reference does, e4m3::from_bits().to_f32(), :437): the same rule over its
 *                        127 values, brute force over all of them, and the inequalities the
 *                        reference's accuracy and two-level tests assert (accuracy.rs:88-139,
 *                        ops/quantize.rs:238-290, scheme.rs:50-123), which fail if scales are
 *                        rounded down, flushed below 2^-6 or left unsaturated.
 *                        PARITY UNPINNED: what a finite scale beyond the dtype's largest finite
 *                        value becomes (this restatement saturates to it, as the reference's test
 *                        comment says of e4m3), what the codec writes for a value the dtype does
 *                        not represent (never produced by quantize: scales are rounded up first;
 *                        here such a value is rounded up as well), and UE8M0 (unimplemented in the
 *                        reference itself, :439).
 *   bqo_encode/decode_scales  same test (:631-657) and the two-level layout test (:659-684).
 *   bqo_normalize_scales, bqo_two_level_scales  restated step for step from the reference's tensor
 *                        ops; no reference-held numbers exist. Pinned by what the mathematics
 *                        fixes (the largest stored block scale is exactly the dtype's largest
 *                        value, 65504, unless the clamp acts; global * stored >= the one-level
 *                        scale, within one f16 step of it) and by the reference's own properties
 *                        (burn-backend-tests .../ops/quantize.rs:213-293, 489-516: the blob round
 *                        trip reproduces the dequantized values exactly, they are within 1e-2 of
 *                        the input, and the error does not track the weights' magnitude). The
 *                        largest value of the block dtype is f16's by the reference's own assert
 *                        (scheme.rs:115-118), ue4m3's is 448 (its bit pattern 0x7E). The quotient
 *                        top / (top / dtype_max) is dtype_max or one f32 step above it, so this path takes
 *                        the saturating branch of bqo_scale_to_dtype about half of the time (PARITY
 *                        UNPINNED, see there). The reference's own two-level tests (ue4m3, same
 *                        arithmetic against 448) only pass if that branch saturates: on their input
 *                        arange(-128..128)/128 the quotient is one step above the dtype's top, and an
 *                        infinite block scale would quantize everything to zero.
 */
#ifndef BQ_ORACLE_H
#define BQ_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BQO_MAX_RANK 8

/* QuantValue: symmetric (Q2S = ternary) and full-range signed ints */
enum { BQO_Q8S = 0, BQO_Q4S = 1, BQO_Q2S = 2, BQO_Q8F = 3, BQO_Q4F = 4, BQO_Q2F = 5 };
enum { BQO_LEVEL_TENSOR = 0, BQO_LEVEL_BLOCK = 1 };
enum { BQO_STORE_NATIVE = 0, BQO_STORE_PACKED_U32 = 1 };
enum { BQO_SCALE_F32 = 0, BQO_SCALE_F16 = 1, BQO_SCALE_BF16 = 2, BQO_SCALE_UE4M3 = 3 };   /* ScaleDtype */

/* Mirrors the fields of cubecl_common::quant::scheme::QuantScheme that this path reads. */
typedef struct {
  uint8_t value;       /* BQO_Q8S .. BQO_Q2F */
  uint8_t level;       /* BQO_LEVEL_* */
  uint8_t store;       /* BQO_STORE_* ; PackedU32 always packs the innermost dim */
  uint8_t block_rank;  /* entries used in block[], aligned to the trailing dims */
  uint8_t block[BQO_MAX_RANK];
} bqo_scheme;

/* QuantValue::range() as f32 and bits / values per u32. Returns 0, or -1 for an unknown value. */
int bqo_value_range(int value, float* a, float* b);
int bqo_size_bits(int value);
int bqo_num_quants(int value);

/* params_shape: per-tensor -> [1]; per-block -> dim/block per axis. Returns the scale count. */
size_t bqo_params_shape(const size_t* shape, int rank, const bqo_scheme* s, size_t* out_shape);

/* BlockLayout::block_of: row-major block index of row-major element `index`. */
size_t bqo_block_of(const size_t* shape, int rank, const bqo_scheme* s, size_t index);

/* compute_range(MinMax): min and max per tensor or per block. Returns 0, -1 if not divisible. */
int bqo_compute_range(const float* x, const size_t* shape, int rank, const bqo_scheme* s,
                      float* min_out, float* max_out);

/* compute_range(AbsMean): gamma = mean |x| per tensor or per block; min = -gamma, max = +gamma. */
int bqo_compute_range_abs_mean(const float* x, const size_t* shape, int rank, const bqo_scheme* s,
                               float* min_out, float* max_out);

/* compute_q_params: scale = (max(|min|,|max|) * 2) / (b - a), elementwise over n entries. */
void bqo_compute_q_params(const float* min, const float* max, size_t n, int value, float* scales);

/* NdArray::quantize: q = (i8) clamp(round_half_away(x / valid(scale)), a, b); one i8 per value. */
int bqo_quantize(const float* x, const size_t* shape, int rank, const bqo_scheme* s,
                 const float* scales, int8_t* q_out);

/* QTensorOps::quantize_dynamic default body: range -> q_params -> quantize. */
int bqo_quantize_dynamic(const float* x, const size_t* shape, int rank, const bqo_scheme* s,
                         int8_t* q_out, float* scales_out);

/* NdArray::dequantize: x = valid(scale) * (f32) q. */
int bqo_dequantize(const int8_t* q, const size_t* shape, int rank, const bqo_scheme* s,
                   const float* scales, float* out);

/* PackedU32 word layout along the innermost dim: value j of a word sits in bits [j*w,(j+1)*w). */
size_t bqo_storage_elements(const size_t* shape, int rank, const bqo_scheme* s);
void bqo_pack_u32(const int8_t* q, const size_t* shape, int rank, int value, uint32_t* words);
void bqo_unpack_u32(const uint32_t* words, const size_t* shape, int rank, int value, int8_t* q);

/* quantized_data_len and the QuantizedBytes blob: values || block scales (dense, native endian). */
size_t bqo_quantized_data_len(const size_t* shape, int rank, const bqo_scheme* s);
size_t bqo_encode(const int8_t* q, const size_t* shape, int rank, const bqo_scheme* s,
                  const float* scales, uint8_t* bytes);
int bqo_decode(const uint8_t* bytes, size_t len, const size_t* shape, int rank,
               const bqo_scheme* s, int8_t* q_out, float* scales_out);

/* float_matmul on 2-D row-major f32 operands with f32 accumulation: c[M,N] = a[M,K] * b[K,N]. */
void bqo_matmul_f32(const float* a, const float* b, float* c, size_t m, size_t k, size_t n);

/* q_matmul with a float lhs and a quantized rhs: dequantize(rhs) -> f32 matmul. */
int bqo_q_matmul(const float* lhs, size_t m, const int8_t* rhs_q, const size_t* rhs_shape,
                 const bqo_scheme* s, const float* rhs_scales, float* out);

/* scale_to_dtype (burn-std/src/tensor/quantization.rs:354-368): the smallest value the scale dtype
 * represents that is no smaller than `scale`. NdArray::quantize applies it to every scale before
 * dividing (burn-ndarray/src/ops/qtensor.rs:90-95). */
float bqo_scale_to_dtype(float scale, int dtype);
/* scale_size / encode_scales / decode_scales (same file, :409-464): bytes per scale on the wire;
 * f16 and bf16 are written with round-to-nearest-even (half::from_f32), native endian. */
size_t bqo_scale_size(int dtype);
/* Two-level schemes (block scales in a narrow dtype + one f32 per-tensor scale; global_scale_dtype,
 * burn-std/src/tensor/quantization.rs:134-136). normalize_scales (burn-backend/src/quantization/
 * scheme.rs:106-134) divides the block scales in place by global = max / dtype_max and returns
 * global (NaN for a block dtype the reference refuses); two_level_scales gives what is stored and
 * what a block is quantized against (burn-ndarray/src/ops/qtensor.rs:90-101, 519-531). */
float bqo_normalize_scales(float* scales, size_t n, int block_dtype);
void bqo_two_level_scales(const float* block_scales, size_t n, int block_dtype, float global, float* stored,
                          float* effective);
void bqo_encode_scales(const float* scales, size_t n, int dtype, uint8_t* out);
void bqo_decode_scales(const uint8_t* in, size_t n, int dtype, float* out);

/* ternary_matmul (burn-ndarray/src/ops/qtensor.rs:431-517): out[m][n] = gamma * sum over k, in
 * ascending k, of +x (t = 1), -x (t = -1) or nothing (anything else); t = rhs_q[k][n]. */
void bqo_ternary_matmul(const float* lhs, size_t m, size_t k, size_t n, const int8_t* rhs_q, float gamma, float* out);

/* Threads used by the *_mt variants below (OpenMP), 1 when built without it. */
int bqo_max_threads(void);
/* Same arithmetic as bqo_quantize_dynamic / bqo_dequantize with rows split over host threads;
 * only for block schemes whose block is [32]-like on the last dim (or per-tensor). */
int bqo_quantize_dynamic_mt(const float* x, const size_t* shape, int rank, const bqo_scheme* s,
                            int8_t* q_out, float* scales_out);
int bqo_dequantize_mt(const int8_t* q, const size_t* shape, int rank, const bqo_scheme* s,
                      const float* scales, float* out);

#ifdef __cplusplus
}
#endif
#endif /* BQ_ORACLE_H */
