/*
 * CPU oracle for burn's quantized-tensor path.  TEST INFRASTRUCTURE ONLY -- see bq_oracle.h.
 *
 * Build with -O2 -ffp-contract=off and without -ffast-math: every step below is one correctly
 * rounded IEEE-754 binary32 operation, exactly as the Rust reference performs it, and the
 * compiler must neither fuse nor reassociate them.
 */
#include "bq_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* QuantValue::range() lives in cubecl-common (not vendored in the burn tree). Q8S = (-127,127)
 * is fixed by burn-ndarray/src/ops/quantization.rs:164-177; Q4S = (-7,7) by the packed vector in
 * burn-std/src/tensor/quantization.rs:581-602; Q8F = (-128,127) by burn-flex/src/ops/qtensor.rs:665-692
 * ("Q8F range: [-128, 127], so range = 255", scale = 2 * 7.5 / 255). Q4F = (-8,7) and Q2F = (-2,1)
 * are the same rule ("full-range", burn-book/src/performance/quantization.md:125-130) at 4 and 2 bits:
 * PARITY UNPINNED, no reference-held number covers them. */
int bqo_value_range(int value, float* a, float* b) {
  switch (value) {
    case BQO_Q8S: *a = -127.0f; *b = 127.0f; return 0;
    case BQO_Q4S: *a = -7.0f; *b = 7.0f; return 0;
    case BQO_Q2S: *a = -1.0f; *b = 1.0f; return 0;
    case BQO_Q8F: *a = -128.0f; *b = 127.0f; return 0;
    case BQO_Q4F: *a = -8.0f; *b = 7.0f; return 0;
    case BQO_Q2F: *a = -2.0f; *b = 1.0f; return 0;
    default: return -1;
  }
}

/* QuantValue::size_bits(), call site burn-std/src/tensor/quantization.rs:520. */
int bqo_size_bits(int value) {
  switch (value) {
    case BQO_Q8S: case BQO_Q8F: return 8;
    case BQO_Q4S: case BQO_Q4F: return 4;
    case BQO_Q2S: case BQO_Q2F: return 2;
    default: return -1;
  }
}

/* QuantScheme::num_quants() for a u32 store: burn-std/src/tensor/quantization.rs:383,519-521. */
int bqo_num_quants(int value) {
  int bits = bqo_size_bits(value);
  return bits > 0 ? 32 / bits : -1;
}

/* BlockSize::to_dim_vec(rank): block extents aligned to the trailing dims, leading dims 1
 * (call sites burn-backend/src/quantization/scheme.rs:23, burn-std/.../quantization.rs:163). */
static void block_dims(const bqo_scheme* s, int rank, size_t* out) {
  for (int d = 0; d < rank; ++d) out[d] = 1;
  if (s->level == BQO_LEVEL_BLOCK) {
    for (int j = 0; j < s->block_rank && j < rank; ++j)
      out[rank - 1 - j] = s->block[s->block_rank - 1 - j];
  }
}

static size_t num_elements(const size_t* shape, int rank) {
  size_t n = 1;
  for (int d = 0; d < rank; ++d) n *= shape[d];
  return n;
}

/* params_shape: burn-std/src/tensor/quantization.rs:141-146. */
size_t bqo_params_shape(const size_t* shape, int rank, const bqo_scheme* s, size_t* out_shape) {
  if (s->level == BQO_LEVEL_TENSOR) {
    if (out_shape) out_shape[0] = 1;
    return 1;
  }
  size_t blk[BQO_MAX_RANK];
  block_dims(s, rank, blk);
  size_t n = 1;
  for (int d = 0; d < rank; ++d) {
    size_t c = shape[d] / blk[d];
    if (out_shape) out_shape[d] = c;
    n *= c;
  }
  return n;
}

/* BlockLayout::block_of: burn-std/src/tensor/quantization.rs:182-192. */
size_t bqo_block_of(const size_t* shape, int rank, const bqo_scheme* s, size_t index) {
  size_t blk[BQO_MAX_RANK], blocks[BQO_MAX_RANK];
  block_dims(s, rank, blk);
  for (int d = 0; d < rank; ++d) blocks[d] = shape[d] / blk[d];
  size_t block = 0, stride = 1;
  for (int d = rank - 1; d >= 0; --d) {
    size_t coordinate = index % shape[d];
    index /= shape[d];
    block += coordinate / blk[d] * stride;
    stride *= blocks[d];
  }
  return block;
}

static int divides(const size_t* shape, int rank, const bqo_scheme* s) {
  size_t blk[BQO_MAX_RANK];
  block_dims(s, rank, blk);
  for (int d = 0; d < rank; ++d)
    if (blk[d] == 0 || shape[d] % blk[d] != 0) return 0;
  return 1;
}

/* compute_range(MinMax): burn-backend/src/quantization/scheme.rs:44-56; per block it is
 * reduce_blocks (:14-41), i.e. min and max over each block rectangle. */
int bqo_compute_range(const float* x, const size_t* shape, int rank, const bqo_scheme* s,
                      float* min_out, float* max_out) {
  size_t n = num_elements(shape, rank);
  if (s->level == BQO_LEVEL_TENSOR) {
    if (n == 0) return -1;
    float lo = x[0], hi = x[0];
    for (size_t i = 1; i < n; ++i) {
      if (x[i] < lo) lo = x[i];
      if (x[i] > hi) hi = x[i];
    }
    min_out[0] = lo;
    max_out[0] = hi;
    return 0;
  }
  if (!divides(shape, rank, s)) return -1;
  size_t nb = bqo_params_shape(shape, rank, s, NULL);
  unsigned char* seen = (unsigned char*)calloc(nb ? nb : 1, 1);
  if (!seen) return -1;
  for (size_t i = 0; i < n; ++i) {
    size_t b = bqo_block_of(shape, rank, s, i);
    if (!seen[b]) {
      seen[b] = 1;
      min_out[b] = x[i];
      max_out[b] = x[i];
    } else {
      if (x[i] < min_out[b]) min_out[b] = x[i];
      if (x[i] > max_out[b]) max_out[b] = x[i];
    }
  }
  free(seen);
  return 0;
}

/* compute_range(AbsMean): burn-backend/src/quantization/scheme.rs:57-69. gamma = mean(|x|) over the
 * tensor (float_mean of float_abs) or over each block rectangle (reduce_blocks with float_mean_dim);
 * the range is (-gamma, +gamma). The mean is a reassociable sum: the reference's order is its
 * backend's, and its tests compare within Tolerance::default(). Here the sum is taken in binary64
 * and rounded once, the value every f32 summation order approximates. */
int bqo_compute_range_abs_mean(const float* x, const size_t* shape, int rank, const bqo_scheme* s,
                               float* min_out, float* max_out) {
  size_t n = num_elements(shape, rank);
  if (n == 0) return -1;
  if (s->level == BQO_LEVEL_TENSOR) {
    double sum = 0.0;
    for (size_t i = 0; i < n; ++i) sum += fabs((double)x[i]);
    max_out[0] = (float)(sum / (double)n);
    min_out[0] = -max_out[0];
    return 0;
  }
  if (!divides(shape, rank, s)) return -1;
  size_t nb = bqo_params_shape(shape, rank, s, NULL);
  double* sums = (double*)calloc(nb ? nb : 1, sizeof(double));
  if (!sums) return -1;
  for (size_t i = 0; i < n; ++i) sums[bqo_block_of(shape, rank, s, i)] += fabs((double)x[i]);
  const double per_block = (double)(n / nb);
  for (size_t b = 0; b < nb; ++b) {
    max_out[b] = (float)(sums[b] / per_block);
    min_out[b] = -max_out[b];
  }
  free(sums);
  return 0;
}

/* compute_q_params: burn-backend/src/quantization/scheme.rs:75-93. `mask_where(min_abs, mask,
 * max_abs)` takes max_abs where min_abs < max_abs, then `* 2` and `/ (b - a)` in f32. */
void bqo_compute_q_params(const float* min, const float* max, size_t n, int value, float* scales) {
  float a, b;
  bqo_value_range(value, &a, &b);
  const float span = b - a;
  for (size_t i = 0; i < n; ++i) {
    float min_abs = fabsf(min[i]);
    float max_abs = fabsf(max[i]);
    float alpha = (min_abs < max_abs) ? max_abs : min_abs;
    float values_range = alpha * 2.0f;
    scales[i] = values_range / span;
  }
}

/* valid_scale: burn-ndarray/src/ops/quantization.rs:78-85. */
static inline float valid_scale(float s) { return s == 0.0f ? 0.1f : s; }

/* SymmetricQuantization::quantize_one: burn-ndarray/src/ops/quantization.rs:128-133.
 * Rust's f32::round is half away from zero == C roundf; clamp then truncating cast. */
static inline int8_t quantize_one(float x, float scale, float a, float b) {
  float q = roundf(x / scale);
  if (q < a) q = a;
  if (q > b) q = b;
  return (int8_t)q;
}

/* NdArray::quantize: burn-ndarray/src/ops/qtensor.rs:82-186 (scale_to_dtype(s, F32) is the
 * identity); per block it is quantize_per_block (:520-539) + QuantizationStrategy::quantize
 * (quantization.rs:21-33), which looks every element's block up with block_of. */
int bqo_quantize(const float* x, const size_t* shape, int rank, const bqo_scheme* s,
                 const float* scales, int8_t* q_out) {
  float a, b;
  if (bqo_value_range(s->value, &a, &b)) return -1;
  size_t n = num_elements(shape, rank);
  if (s->level == BQO_LEVEL_TENSOR) {
    float sc = valid_scale(scales[0]);
    for (size_t i = 0; i < n; ++i) q_out[i] = quantize_one(x[i], sc, a, b);
    return 0;
  }
  if (!divides(shape, rank, s)) return -1;
  for (size_t i = 0; i < n; ++i) {
    /* multiplier 1.0 * s for a one-level scheme: qtensor.rs:528-531 */
    float sc = valid_scale(1.0f * scales[bqo_block_of(shape, rank, s, i)]);
    q_out[i] = quantize_one(x[i], sc, a, b);
  }
  return 0;
}

/* QTensorOps::quantize_dynamic default: burn-backend/src/backend/ops/qtensor.rs:144-149. */
int bqo_quantize_dynamic(const float* x, const size_t* shape, int rank, const bqo_scheme* s,
                         int8_t* q_out, float* scales_out) {
  size_t np = bqo_params_shape(shape, rank, s, NULL);
  float* lo = (float*)malloc(sizeof(float) * (np ? np : 1));
  float* hi = (float*)malloc(sizeof(float) * (np ? np : 1));
  if (!lo || !hi) { free(lo); free(hi); return -1; }
  int rc = bqo_compute_range(x, shape, rank, s, lo, hi);
  if (rc == 0) {
    bqo_compute_q_params(lo, hi, np, s->value, scales_out);
    rc = bqo_quantize(x, shape, rank, s, scales_out, q_out);
  }
  free(lo);
  free(hi);
  return rc;
}

/* NdArray::dequantize: burn-ndarray/src/ops/qtensor.rs:188-210,541-554 with
 * NdArrayQTensor::strategy (tensor.rs:716-737, which re-applies valid_scale) and
 * dequantize_one (quantization.rs:135-138): scale * (f32) q. */
int bqo_dequantize(const int8_t* q, const size_t* shape, int rank, const bqo_scheme* s,
                   const float* scales, float* out) {
  size_t n = num_elements(shape, rank);
  if (s->level == BQO_LEVEL_TENSOR) {
    float sc = valid_scale(scales[0]);
    for (size_t i = 0; i < n; ++i) out[i] = sc * (float)q[i];
    return 0;
  }
  if (!divides(shape, rank, s)) return -1;
  for (size_t i = 0; i < n; ++i) {
    float sc = valid_scale(1.0f * scales[bqo_block_of(shape, rank, s, i)]);
    out[i] = sc * (float)q[i];
  }
  return 0;
}

/* storage_elements: burn-std/src/tensor/quantization.rs:382-396 (packed dim = innermost). */
size_t bqo_storage_elements(const size_t* shape, int rank, const bqo_scheme* s) {
  size_t n = num_elements(shape, rank);
  if (s->store == BQO_STORE_NATIVE) return n;
  size_t nq = (size_t)bqo_num_quants(s->value);
  if (rank == 0) return (n + nq - 1) / nq;
  size_t lines = 1;
  for (int d = 0; d + 1 < rank; ++d) lines *= shape[d];
  return lines * ((shape[rank - 1] + nq - 1) / nq);
}

/* pack along the innermost dim, zero padded per line. Word layout is what unpack_q_to_i8s reads:
 * burn-std/src/tensor/quantization.rs:514-542 (low bits first), :475-511 for the 8-bit case. */
void bqo_pack_u32(const int8_t* q, const size_t* shape, int rank, int value, uint32_t* words) {
  const int bits = bqo_size_bits(value);
  const size_t nq = (size_t)(32 / bits);
  const uint32_t mask = (bits == 32) ? 0xFFFFFFFFu : ((1u << bits) - 1u);
  size_t last = rank ? shape[rank - 1] : 1;
  size_t lines = rank ? num_elements(shape, rank - 1) : 1;
  size_t wpl = (last + nq - 1) / nq;
  for (size_t l = 0; l < lines; ++l) {
    for (size_t w = 0; w < wpl; ++w) {
      uint32_t word = 0;
      for (size_t j = 0; j < nq; ++j) {
        size_t c = w * nq + j;
        if (c < last) word |= ((uint32_t)(uint8_t)q[l * last + c] & mask) << (j * bits);
      }
      words[l * wpl + w] = word;
    }
  }
}

void bqo_unpack_u32(const uint32_t* words, const size_t* shape, int rank, int value, int8_t* q) {
  const int bits = bqo_size_bits(value);
  const size_t nq = (size_t)(32 / bits);
  const uint32_t mask = (1u << bits) - 1u;
  const int sign_shift = 8 - bits;
  size_t last = rank ? shape[rank - 1] : 1;
  size_t lines = rank ? num_elements(shape, rank - 1) : 1;
  size_t wpl = (last + nq - 1) / nq;
  for (size_t l = 0; l < lines; ++l) {
    for (size_t c = 0; c < last; ++c) {
      uint32_t packed = words[l * wpl + c / nq];
      uint8_t raw = (uint8_t)((packed >> ((c % nq) * bits)) & mask);
      q[l * last + c] = (int8_t)((int8_t)(raw << sign_shift) >> sign_shift);
    }
  }
}

/* quantized_data_len: burn-std/src/tensor/quantization.rs:400-407 (f32 scales, one level). */
size_t bqo_quantized_data_len(const size_t* shape, int rank, const bqo_scheme* s) {
  size_t value_bytes = bqo_storage_elements(shape, rank, s) *
                       (s->store == BQO_STORE_PACKED_U32 ? 4u : 1u);
  return value_bytes + 4u * bqo_params_shape(shape, rank, s, NULL);
}

/* The blob a backend hands to / takes from TensorData: values || block scales, dense.
 * Native store: one i8 per value (QuantizedBytes::new, :219-272). PackedU32: u32 words as the
 * packed backends keep them (burn-cubecl/src/ops/qtensor.rs:283-307) and as split_values_off
 * reads them (:317-352). */
size_t bqo_encode(const int8_t* q, const size_t* shape, int rank, const bqo_scheme* s,
                  const float* scales, uint8_t* bytes) {
  size_t n = num_elements(shape, rank);
  size_t off;
  if (s->store == BQO_STORE_NATIVE) {
    memcpy(bytes, q, n);
    off = n;
  } else {
    size_t words = bqo_storage_elements(shape, rank, s);
    uint32_t* tmp = (uint32_t*)malloc(4 * (words ? words : 1));
    bqo_pack_u32(q, shape, rank, s->value, tmp);
    memcpy(bytes, tmp, 4 * words);
    free(tmp);
    off = 4 * words;
  }
  size_t np = bqo_params_shape(shape, rank, s, NULL);
  memcpy(bytes + off, scales, 4 * np);
  return off + 4 * np;
}

/* QuantizedBytes::into_vec_i8: burn-std/src/tensor/quantization.rs:280-352. */
int bqo_decode(const uint8_t* bytes, size_t len, const size_t* shape, int rank,
               const bqo_scheme* s, int8_t* q_out, float* scales_out) {
  size_t np = bqo_params_shape(shape, rank, s, NULL);
  if (len < 4 * np) return -1;
  size_t split = len - 4 * np;
  memcpy(scales_out, bytes + split, 4 * np);
  size_t n = num_elements(shape, rank);
  if (s->store == BQO_STORE_NATIVE || bqo_size_bits(s->value) == 8) {
    /* 8-bit values read back as i8 whatever the store (:329-333); a padded packed line only
     * exists when the innermost dim is not a multiple of 4, which packed backends refuse. */
    if (s->store == BQO_STORE_NATIVE) {
      if (split < n) return -1;
      memcpy(q_out, bytes, n);
    } else {
      size_t words = bqo_storage_elements(shape, rank, s);
      if (split < 4 * words) return -1;
      uint32_t* tmp = (uint32_t*)malloc(4 * (words ? words : 1));
      memcpy(tmp, bytes, 4 * words);
      bqo_unpack_u32(tmp, shape, rank, s->value, q_out);
      free(tmp);
    }
    return 0;
  }
  size_t words = bqo_storage_elements(shape, rank, s);
  if (split < 4 * words) return -1;
  uint32_t* tmp = (uint32_t*)malloc(4 * (words ? words : 1));
  memcpy(tmp, bytes, 4 * words);
  bqo_unpack_u32(tmp, shape, rank, s->value, q_out);
  free(tmp);
  return 0;
}

/* float_matmul for 2-D f32 operands (burn-ndarray/src/ops/matmul.rs:9-69 ends in an sgemm whose
 * summation order is unspecified; this one accumulates in f32 over k ascending). */
void bqo_matmul_f32(const float* a, const float* b, float* c, size_t m, size_t k, size_t n) {
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
  for (size_t i = 0; i < m; ++i) {
    float* ci = c + i * n;
    for (size_t j = 0; j < n; ++j) ci[j] = 0.0f;
    for (size_t p = 0; p < k; ++p) {
      const float av = a[i * k + p];
      const float* bp = b + p * n;
      for (size_t j = 0; j < n; ++j) ci[j] = ci[j] + av * bp[j];
    }
  }
}

/* NdArray::q_matmul fallback path: burn-ndarray/src/ops/qtensor.rs:230-266 -- dequantize the
 * quantized operand to the float operand's dtype, then float_matmul; Inhibit => float out. */
int bqo_q_matmul(const float* lhs, size_t m, const int8_t* rhs_q, const size_t* rhs_shape,
                 const bqo_scheme* s, const float* rhs_scales, float* out) {
  size_t k = rhs_shape[0], n = rhs_shape[1];
  float* w = (float*)malloc(sizeof(float) * ((k * n) > 0 ? k * n : 1));
  if (!w) return -1;
  int rc = bqo_dequantize(rhs_q, rhs_shape, 2, s, rhs_scales, w);
  if (rc == 0) bqo_matmul_f32(lhs, w, out, m, k, n);
  free(w);
  return rc;
}

int bqo_max_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* True when every block is a run of `blk` consecutive elements of the flat storage. */
static int trailing_block(const size_t* shape, int rank, const bqo_scheme* s, size_t* blk_out) {
  if (s->level != BQO_LEVEL_BLOCK || rank < 1) return 0;
  size_t blk[BQO_MAX_RANK];
  block_dims(s, rank, blk);
  for (int d = 0; d + 1 < rank; ++d)
    if (blk[d] != 1) return 0;
  if (blk[rank - 1] == 0 || shape[rank - 1] % blk[rank - 1] != 0) return 0;
  *blk_out = blk[rank - 1];
  return 1;
}

/* Same arithmetic as bqo_quantize_dynamic, with the independent blocks (or, per tensor, the
 * elements of the second pass) spread over host threads. The per-element operations are the
 * ones above; max/min are order independent, so the result is bit identical. */
int bqo_quantize_dynamic_mt(const float* x, const size_t* shape, int rank, const bqo_scheme* s,
                            int8_t* q_out, float* scales_out) {
  float a, b;
  if (bqo_value_range(s->value, &a, &b)) return -1;
  const float span = b - a;
  size_t n = num_elements(shape, rank);
  if (s->level == BQO_LEVEL_TENSOR) {
    if (n == 0) return -1;
    float lo = x[0], hi = x[0];
#ifdef _OPENMP
#pragma omp parallel for reduction(min : lo) reduction(max : hi) schedule(static)
#endif
    for (size_t i = 0; i < n; ++i) {
      if (x[i] < lo) lo = x[i];
      if (x[i] > hi) hi = x[i];
    }
    bqo_compute_q_params(&lo, &hi, 1, s->value, scales_out);
    float sc = valid_scale(scales_out[0]);
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
    for (size_t i = 0; i < n; ++i) q_out[i] = quantize_one(x[i], sc, a, b);
    return 0;
  }
  size_t blk;
  if (!trailing_block(shape, rank, s, &blk)) return -1;
  size_t nb = n / blk;
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
  for (size_t bi = 0; bi < nb; ++bi) {
    const float* xb = x + bi * blk;
    float lo = xb[0], hi = xb[0];
    for (size_t j = 1; j < blk; ++j) {
      if (xb[j] < lo) lo = xb[j];
      if (xb[j] > hi) hi = xb[j];
    }
    float min_abs = fabsf(lo), max_abs = fabsf(hi);
    float alpha = (min_abs < max_abs) ? max_abs : min_abs;
    float sc = (alpha * 2.0f) / span;
    scales_out[bi] = sc;
    sc = valid_scale(sc);
    for (size_t j = 0; j < blk; ++j) q_out[bi * blk + j] = quantize_one(xb[j], sc, a, b);
  }
  return 0;
}

int bqo_dequantize_mt(const int8_t* q, const size_t* shape, int rank, const bqo_scheme* s,
                      const float* scales, float* out) {
  size_t n = num_elements(shape, rank);
  if (s->level == BQO_LEVEL_TENSOR) {
    float sc = valid_scale(scales[0]);
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
    for (size_t i = 0; i < n; ++i) out[i] = sc * (float)q[i];
    return 0;
  }
  size_t blk;
  if (!trailing_block(shape, rank, s, &blk)) return -1;
  size_t nb = n / blk;
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
  for (size_t bi = 0; bi < nb; ++bi) {
    float sc = valid_scale(scales[bi]);
    for (size_t j = 0; j < blk; ++j) out[bi * blk + j] = sc * (float)q[bi * blk + j];
  }
  return 0;
}

/* ---- scale dtypes --------------------------------------------------------------------------- */
static uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* f32 -> f16, round to nearest even (what half::f16::from_f32 does) */
static uint16_t f16_from_f32_rne(float f) {
  const uint32_t u = f32_bits(f), sign = (u >> 16) & 0x8000u, mag = u & 0x7FFFFFFFu;
  if (mag > 0x7F800000u) return (uint16_t)(sign | 0x7E00u);
  if (mag >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);           /* >= 65520 rounds to infinity */
  if (mag < 0x33000001u) return (uint16_t)sign;                          /* <= 2^-25 rounds to zero */
  int e = (int)(mag >> 23) - 127;
  uint32_t man = (mag & 0x7FFFFFu) | 0x800000u;                          /* 24-bit significand */
  int shift = e < -14 ? 13 + (-14 - e) : 13;                             /* bits dropped */
  uint32_t kept = man >> shift, rest = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
  if (rest > half || (rest == half && (kept & 1u))) ++kept;
  if (e < -14) return (uint16_t)(sign | kept);                           /* subnormal (a carry makes it 2^-14) */
  return (uint16_t)(sign | (((uint32_t)(e + 15) << 10) + (kept - 0x400u)));  /* a carry bumps the exponent */
}

static float f32_from_f16(uint16_t h) {
  const uint32_t sign = ((uint32_t)h & 0x8000u) << 16, ex = (h >> 10) & 0x1Fu, man = h & 0x3FFu;
  if (ex == 0) {
    float t = (float)man * 5.9604644775390625e-8f; /* man * 2^-24 */
    return bits_f32(sign | f32_bits(t));
  }
  if (ex == 31) return bits_f32(sign | 0x7F800000u | (man << 13));
  return bits_f32(sign | ((ex + 112u) << 23) | (man << 13));
}

static uint16_t bf16_from_f32_rne(float f) {
  uint32_t u = f32_bits(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/* e4m3 (OCP FP8 E4M3: 4 exponent bits, bias 7, 3 mantissa bits, no infinities, 0x7F = NaN, largest
 * value 0x7E = 448; subnormals m * 2^-9). "UE4M3" uses the non-negative half. */
static float f32_from_e4m3(uint8_t b) {
  const uint32_t ex = (b >> 3) & 0xFu, man = b & 7u;
  float v;
  if (ex == 0) v = (float)man * 0.001953125f;                       /* m * 2^-9 */
  else if (ex == 15 && man == 7) return NAN;
  else v = ldexpf(1.0f + (float)man * 0.125f, (int)ex - 7);
  return (b & 0x80u) ? -v : v;
}
/* bits of a value that e4m3 represents exactly (what the rounding below returns) */
static uint8_t e4m3_bits_exact(float v) {
  if (v != v) return 0x7Fu;
  if (v <= 0.0f) return 0;
  if (v < 0.015625f) return (uint8_t)(v * 512.0f);                  /* subnormal: m = v / 2^-9 */
  int e;
  const float m = frexpf(v, &e);                                    /* v = m * 2^e, m in [0.5, 1) */
  if (v > 448.0f) return 0x7Eu;
  return (uint8_t)(((unsigned)(e - 1 + 7) << 3) | (unsigned)((m * 2.0f - 1.0f) * 8.0f));
}
/* smallest non-negative e4m3 value that is no smaller than s (s > 0, finite) */
static float e4m3_round_up(float s) {
  if (s < 0.015625f) {                                              /* below the smallest normal, 2^-6 */
    return ceilf(s * 512.0f) * 0.001953125f;
  }
  int e;
  (void)frexpf(s, &e);                                              /* s in [2^(e-1), 2^e) */
  const float step = ldexpf(1.0f, e - 1 - 3);                       /* spacing of e4m3 values there */
  float r = ceilf(s / step) * step;                                 /* exact: s / step < 16 */
  return r > 448.0f ? 448.0f : r;                                   /* saturates (parity unpinned) */
}

float bqo_scale_to_dtype(float scale, int dtype) {
  if (dtype == BQO_SCALE_F32) return scale;
  if (dtype == BQO_SCALE_UE4M3) {
    if (scale != scale || scale == INFINITY) return scale;
    return scale > 0.0f ? e4m3_round_up(scale) : 0.0f;              /* unsigned: nothing below zero */
  }
  if (scale != scale || scale == INFINITY || scale == -INFINITY) return scale;
  /* start from the nearest representable value, step up while it is below the scale */
  if (dtype == BQO_SCALE_F16) {
    uint16_t h = f16_from_f32_rne(scale);
    float back = f32_from_f16(h);
    if (back < scale) {                      /* next representable value toward +infinity */
      if (h & 0x8000u) h = (uint16_t)((h & 0x7FFFu) == 0 ? 0x0001u : h - 1u); else h = (uint16_t)(h + 1u);
      back = f32_from_f16(h);
    }
    if (back == INFINITY) back = 65504.0f;   /* a finite scale saturates (parity unpinned) */
    if (back == -INFINITY) back = -65504.0f; /* (RNE of a finite value below -65504; -65504 is no smaller) */
    return back;
  }
  uint16_t b = bf16_from_f32_rne(scale);
  float back = bits_f32((uint32_t)b << 16);
  if (back < scale) {
    if (b & 0x8000u) b = (uint16_t)((b & 0x7FFFu) == 0 ? 0x0001u : b - 1u); else b = (uint16_t)(b + 1u);
    back = bits_f32((uint32_t)b << 16);
  }
  if (back == INFINITY) back = bits_f32(0x7F7F0000u);
  if (back == -INFINITY) back = bits_f32(0xFF7F0000u);
  return back;
}

size_t bqo_scale_size(int dtype) { return dtype == BQO_SCALE_F32 ? 4 : (dtype == BQO_SCALE_UE4M3 ? 1 : 2); }

/* normalize_scales (burn-backend/src/quantization/scheme.rs:106-134): the per-tensor scale of a
 * two-level scheme is the largest block scale over the block dtype's largest value, kept at or
 * above the smallest normal f32; every block scale is divided by it. One f32 operation per step,
 * as the tensor ops there (float_max, float_div_scalar, float_clamp_min, float_div). Returns the
 * per-tensor scale, or NaN for a block dtype the reference refuses (its largest value must not
 * exceed f16's: f16, largest value 65504, and ue4m3, largest value 448). */
float bqo_normalize_scales(float* scales, size_t n, int block_dtype) {
  if (block_dtype != BQO_SCALE_F16 && block_dtype != BQO_SCALE_UE4M3) return NAN;
  const float dtype_max = block_dtype == BQO_SCALE_F16 ? 65504.0f : 448.0f;
  float top = scales[0];
  for (size_t i = 1; i < n; ++i) top = scales[i] > top ? scales[i] : top;
  float global = top / dtype_max;
  if (global < 1.17549435e-38f) global = 1.17549435e-38f;   /* f32::MIN_POSITIVE */
  for (size_t i = 0; i < n; ++i) scales[i] = scales[i] / global;
  return global;
}

/* What NdArray::quantize makes of two-level parameters (burn-ndarray/src/ops/qtensor.rs:90-101,
 * 519-531): the block scales are rounded up to the block dtype (they are stored that way), the
 * per-tensor scale stays f32, and block i is quantized against global * stored[i]. */
void bqo_two_level_scales(const float* block_scales, size_t n, int block_dtype, float global, float* stored,
                          float* effective) {
  for (size_t i = 0; i < n; ++i) {
    stored[i] = bqo_scale_to_dtype(block_scales[i], block_dtype);
    effective[i] = global * stored[i];
  }
}

void bqo_encode_scales(const float* scales, size_t n, int dtype, uint8_t* out) {
  for (size_t i = 0; i < n; ++i) {
    if (dtype == BQO_SCALE_F32) {
      memcpy(out + 4 * i, scales + i, 4);
    } else if (dtype == BQO_SCALE_UE4M3) {
      /* (scales reach the codec already rounded up to the dtype, burn-ndarray/src/ops/qtensor.rs:90-95:
       * whatever rounding e4m3::from_f32 applies, it returns such a value unchanged) */
      out[i] = e4m3_bits_exact(bqo_scale_to_dtype(scales[i], dtype));
    } else {
      uint16_t h = dtype == BQO_SCALE_F16 ? f16_from_f32_rne(scales[i]) : bf16_from_f32_rne(scales[i]);
      memcpy(out + 2 * i, &h, 2);
    }
  }
}

void bqo_decode_scales(const uint8_t* in, size_t n, int dtype, float* out) {
  for (size_t i = 0; i < n; ++i) {
    if (dtype == BQO_SCALE_F32) {
      memcpy(out + i, in + 4 * i, 4);
    } else if (dtype == BQO_SCALE_UE4M3) {
      out[i] = f32_from_e4m3(in[i]);
    } else {
      uint16_t h;
      memcpy(&h, in + 2 * i, 2);
      out[i] = dtype == BQO_SCALE_F16 ? f32_from_f16(h) : bits_f32((uint32_t)h << 16);
    }
  }
}

void bqo_ternary_matmul(const float* lhs, size_t m, size_t k, size_t n, const int8_t* rhs_q, float gamma, float* out) {
  for (size_t i = 0; i < m; ++i) {
    float* orow = out + i * n;
    for (size_t j = 0; j < n; ++j) orow[j] = 0.0f;
    for (size_t kk = 0; kk < k; ++kk) {
      const float x = lhs[i * k + kk];
      const int8_t* wrow = rhs_q + kk * n;
      for (size_t j = 0; j < n; ++j) {
        if (wrow[j] == 1) orow[j] += x;
        else if (wrow[j] == -1) orow[j] -= x;
      }
    }
    for (size_t j = 0; j < n; ++j) orow[j] *= gamma;
  }
}
