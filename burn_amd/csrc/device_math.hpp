// Device-side arithmetic shared by the quantize / dequantize / matmul kernels (gfx950).
//
// Bit-exactness contract with burn-ndarray (crates/burn-ndarray/src/ops/quantization.rs:128-138):
//   q = (i8) clamp(round_half_away_from_zero(x / s), a, b)      x_hat = s * (f32) q
// where `/` and `*` are single correctly rounded binary32 operations. These translation units are
// compiled with -ffp-contract=off so nothing below is fused or reassociated by the compiler.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace bq {

constexpr int kWave = 64;

// Native 128-bit vectors (what global_load_dwordx4 / global_store_dwordx4 move).
typedef float vfloat4 __attribute__((ext_vector_type(4)));
typedef uint32_t vuint4 __attribute__((ext_vector_type(4)));
typedef uint32_t vuint2 __attribute__((ext_vector_type(2)));

// valid_scale: a zero scale (all-zero block) quantizes against 0.1; the stored scale stays 0.
__device__ __forceinline__ float valid_scale(float s) { return s == 0.0f ? 0.1f : s; }

// compute_q_params for one range: (2 * max|x|) / (b - a), with b - a = 2 * qmax exactly.
__device__ __forceinline__ float scale_from_absmax(float amax, float span) {
  return (amax * 2.0f) / span;
}

// scale_to_dtype (crates/burn-std/src/tensor/quantization.rs:354-368): the smallest value the scale
// dtype represents that is no smaller than s, as an f32. sdt: 0 f32 (identity), 1 f16, 2 bf16,
// 3 ue4m3 (BQ_SCALE_*). NaN and the infinities pass through; a finite scale past the dtype's largest
// finite value saturates to it.
__device__ __forceinline__ float scale_round_up(float s, int sdt) {
  if (sdt == 0) return s;
  const uint32_t u = __float_as_uint(s), mag = u & 0x7FFFFFFFu;
  if (mag >= 0x7F800000u) return s;
  if (sdt == 3) {  // ue4m3: 4 significant bits down to 2^-6, multiples of 2^-9 below; largest value 448; unsigned
    if (!(s > 0.0f)) return 0.0f;
    if (s < 0.015625f) return ceilf(s * 512.0f) * 0.001953125f;
    const uint32_t r = (u & 0xFFFFFu) ? ((u | 0xFFFFFu) + 1u) : u;   // magnitude up to a multiple of 2^(e - 3)
    return r > 0x43E00000u ? 448.0f : __uint_as_float(r);
  }
  if (sdt == 2) {  // bf16: the upper 16 bits; rounding the magnitude up (s > 0) or truncating it (s < 0)
    if ((u & 0xFFFFu) == 0u) return s;
    if (u & 0x80000000u) return __uint_as_float(u & 0xFFFF0000u);
    const uint32_t r = (u + 0xFFFFu) & 0xFFFF0000u;
    return __uint_as_float(r >= 0x7F800000u ? 0x7F7F0000u : r);
  }
  // f16: 11 significant bits down to 2^-14, multiples of 2^-24 below; largest finite value 65504
  int e = static_cast<int>(mag >> 23) - 127;
  if (e < -14) e = -14;
  if (e > 15) return s > 0.0f ? 65504.0f : -65504.0f;
  const float q = __uint_as_float(static_cast<uint32_t>(e - 10 + 127) << 23);   // the spacing, a power of two
  const float inv = __uint_as_float(static_cast<uint32_t>(10 - e + 127) << 23);
  const float r = ceilf(s * inv) * q;  // both products exact
  return r > 65504.0f ? 65504.0f : r;
}

// round half away from zero of a value already clamped to [-128, 128]. trunc(v + copysign(c, v))
// with c = pred(0.5): adding 0.5 itself would carry pred(0.5) up to 1.0, every other case is
// exact or rounds back below the next integer.
__device__ __forceinline__ int round_half_away_i32(float v) {
  const float c = __uint_as_float(0x3EFFFFFFu);  // 0.49999997
  float biased = v + copysignf(c, v);
  return static_cast<int>(biased);  // v_cvt_i32_f32 truncates toward zero
}

// Reference-order quantize of one value: IEEE divide, round half away, clamp.
__device__ __forceinline__ int quantize_div(float x, float s, float qmin, float qmax) {
  float q = x / s;
  q = fminf(fmaxf(q, qmin), qmax);  // clamping before rounding is equivalent: bounds are integers
  return round_half_away_i32(q);
}

// The same quotient without a divide per element. With r = RN(1/s) computed once per block:
//   q0 = RN(x * r), e = RN(x - s * q0) (exact: an fma residual), q = RN(q0 + e * r)
// is RN(x / s) (Markstein's correction step) whenever no intermediate under/overflows, which the
// callers guarantee by only taking this path for s in [2^-100, 2^100] and |x| <= 2^7 * 2 * s.
__device__ __forceinline__ float div_by_recip(float x, float s, float r) {
  float q0 = x * r;
  float e = __builtin_fmaf(-s, q0, x);
  return __builtin_fmaf(e, r, q0);
}

__device__ __forceinline__ bool recip_path_ok(float s) {
  // 2^-100 <= s < 2^101, tested on the exponent field
  uint32_t e = (__float_as_uint(s) >> 23) & 0xFFu;
  return e >= 27u && e <= 227u;
}

// RN(1/s) from the hardware approximation and one Newton step. bq_selftest_division checks on
// the device, for every mantissa and every exponent recip_path_ok admits, that this equals the
// IEEE quotient 1.0f / s.
__device__ __forceinline__ float recip_exact(float s) {
  const float r0 = __builtin_amdgcn_rcpf(s);
  const float e = __builtin_fmaf(-s, r0, 1.0f);
  return __builtin_fmaf(e, r0, r0);
}

// compute_q_params without a divide: (2 * amax) / (2 * QMAX) == amax / QMAX as real numbers, and
// the quotient by the constant is recovered exactly with the same correction step as above
// (c = RN(1 / QMAX)). Valid while nothing under/overflows: callers take it for
// 2^-87 <= amax < 2^94 only. Also checked exhaustively by bq_selftest_division.
template <int QMAX>
__device__ __forceinline__ float scale_from_absmax_fast(float amax) {
  constexpr float c = 1.0f / static_cast<float>(QMAX);
  const float q0 = amax * c;
  const float e = __builtin_fmaf(-static_cast<float>(QMAX), q0, amax);
  return __builtin_fmaf(e, c, q0);
}

__device__ __forceinline__ bool absmax_fast_ok(float amax) {
  const uint32_t e = __float_as_uint(amax) >> 23;  // amax >= 0
  return e >= 40u && e <= 220u;
}

__device__ __forceinline__ int quantize_recip(float x, float s, float r, float qmin, float qmax) {
  float q = div_by_recip(x, s, r);
  q = fminf(fmaxf(q, qmin), qmax);
  return round_half_away_i32(q);
}

// Low BITS of VPL integers into one word, field i at bits [i*BITS, (i+1)*BITS).
template <int VPL>
__device__ __forceinline__ uint32_t pack_fields(const int (&q)[VPL]) {
  if (VPL == 4) {
    // v_perm_b32 picks bytes out of {hi operand: selectors 4-7, lo operand: 0-3}; 0x0c yields 0
    const uint32_t lo = __builtin_amdgcn_perm(static_cast<uint32_t>(q[1]), static_cast<uint32_t>(q[0]), 0x0c0c0400u);
    const uint32_t hi = __builtin_amdgcn_perm(static_cast<uint32_t>(q[3]), static_cast<uint32_t>(q[2]), 0x04000c0cu);
    return lo | hi;
  } else if (VPL == 16) {
    uint32_t w = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) w |= (static_cast<uint32_t>(q[i]) & 0x3u) << (2 * i);
    return w;
  } else {
    uint32_t b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      b[i] = (static_cast<uint32_t>(q[2 * i]) & 0xFu) | (static_cast<uint32_t>(q[2 * i + 1]) << 4);
    const uint32_t lo = __builtin_amdgcn_perm(b[1], b[0], 0x0c0c0400u);
    const uint32_t hi = __builtin_amdgcn_perm(b[3], b[2], 0x04000c0cu);
    return lo | hi;
  }
}

// f32 -> bf16 round to nearest even (what TensorData::convert_dtype / half::bf16::from_f32 do).
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return static_cast<uint16_t>((u >> 16) | 0x40u);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return static_cast<uint16_t>(u >> 16);
}

// Two f32 -> two bf16 (round to nearest even) in one v_cvt_pk_bf16_f32: lo in bits 0..15. Same
// bits as f32_to_bf16 for every non-NaN input.
__device__ __forceinline__ uint32_t f32x2_to_bf16x2(float lo, float hi) {
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t));
}

__device__ __forceinline__ float bf16_to_f32(uint16_t h) {
  return __uint_as_float(static_cast<uint32_t>(h) << 16);
}

// Sign-extend field j (width BITS) of a packed word: value j sits in bits [j*BITS, (j+1)*BITS).
template <int BITS>
__device__ __forceinline__ int unpack_field(uint32_t word, int j) {
  return static_cast<int>(word << (32 - BITS - j * BITS)) >> (32 - BITS);
}

// One DPP-modified move: every lane reads the lane that `CTRL` names inside its row of 16.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_lane(uint32_t v) {
  return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), CTRL, 0xF, 0xF, true));
}

// max of a non-negative float (an absmax) over `WIDTH` consecutive lanes (a power of two <= 64),
// result in every lane. Non-negative floats order like their bit patterns, so every step is one
// v_max_u32 whose second operand is fetched by DPP inside the vector ALU -- no LDS crossbar
// (ds_bpermute), no canonicalising copies: quad_perm [1,0,3,2] and [2,3,0,1] inside a quad,
// row_half_mirror across the quads of 8 lanes, row_mirror across the halves of a row of 16, then
// v_permlane16_swap / v_permlane32_swap across rows and across the halves of the wave. max is
// order-free, so the result is the one any other reduction order gives.
template <int WIDTH>
__device__ __forceinline__ float group_max(float f) {
  static_assert(WIDTH >= 1 && WIDTH <= kWave && (WIDTH & (WIDTH - 1)) == 0, "a power of two up to the wave");
  uint32_t v = __float_as_uint(f);
  if (WIDTH >= 2) v = max(v, dpp_lane<0xB1>(v));    // quad_perm [1,0,3,2]
  if (WIDTH >= 4) v = max(v, dpp_lane<0x4E>(v));    // quad_perm [2,3,0,1]
  if (WIDTH >= 8) v = max(v, dpp_lane<0x141>(v));   // row_half_mirror
  if (WIDTH >= 16) v = max(v, dpp_lane<0x140>(v));  // row_mirror
  if (WIDTH >= 32) {  // rows 1, 3 of one copy <-> rows 0, 2 of the other
    const auto r = __builtin_amdgcn_permlane16_swap(v, v, false, false);
    v = max(r[0], r[1]);
  }
  if (WIDTH >= 64) {  // upper half of one copy <-> lower half of the other
    const auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    v = max(r[0], r[1]);
  }
  return __uint_as_float(v);
}

}  // namespace bq
