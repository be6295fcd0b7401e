// dequantize kernels for gfx950: a pure streaming unpack x scale.
//
// x_hat = (s == 0 ? 0.1 : s) * (f32) q, one correctly rounded multiply per value, exactly as
// crates/burn-ndarray/src/ops/quantization.rs:135-138 with the strategy of tensor.rs:716-737.
// One lane reads one packed word (4 x i8 or 8 x i4) and writes its VPL outputs as 128-bit stores.
#include "common.hpp"
#include "device_math.hpp"

namespace bq {

bool fused_block_ok(int block, int value);

namespace {

#ifndef BQ_DEQUANT_THREADS
#define BQ_DEQUANT_THREADS 256
#endif
#ifndef BQ_DEQUANT_UNROLL
#define BQ_DEQUANT_UNROLL 2
#endif
constexpr int kThreads = BQ_DEQUANT_THREADS;

// One lane-step produces one output "chunk": VPC consecutive values stored as a single vector
// (f32: 4 values = 16 B; bf16: a whole word's 4 or 8 values = 8 or 16 B), so every store
// instruction of a wave writes one contiguous run of full cache lines. For Q4S -> f32 a word
// holds two chunks: adjacent lanes read the same word and take one half each (the duplicate
// 4-byte read is served by the same cache line).
template <int VPC, bool BF16>
__device__ __forceinline__ void store_chunk(void* __restrict__ out, size_t chunk, const float* v) {
  if (BF16) {
    uint32_t packed[VPC / 2];
#pragma unroll
    for (int i = 0; i < VPC / 2; ++i)
      packed[i] = f32x2_to_bf16x2(v[2 * i], v[2 * i + 1]);
    if (VPC == 4) {
      vuint2 t = {packed[0], packed[1]};
      __builtin_nontemporal_store(t, reinterpret_cast<vuint2*>(out) + chunk);
    } else {
      vuint4 t = {packed[0], packed[1], packed[VPC == 8 ? 2 : 0], packed[VPC == 8 ? 3 : 1]};
      __builtin_nontemporal_store(t, reinterpret_cast<vuint4*>(out) + chunk);
    }
  } else {
    static_assert(BF16 || VPC == 4, "f32 chunks are one float4");
    vfloat4 t = {v[0], v[1], v[2], v[3]};
    __builtin_nontemporal_store(t, reinterpret_cast<vfloat4*>(out) + chunk);
  }
}

// A workgroup owns kThreads * U consecutive chunks; lane t takes chunks t, t + 256, ...
// block_words_log2 = log2(words per scale) for run-block schemes.
constexpr int kDequantUnroll = BQ_DEQUANT_UNROLL;  // measured on C2 / C1 / C3: 1 -> 60.9 / 17.9 / 49.4 us, 2 -> 53.7 / 16.1 / 47.5, 4 -> 57.3 / 16.4 / 48.9

template <int VPL, bool BF16>
__global__ void __launch_bounds__(kThreads)
dequantize_kernel(const uint32_t* __restrict__ words_in, size_t words, size_t n,
                  unsigned block_words_log2, bool per_tensor, const float* __restrict__ scales,
                  void* __restrict__ out) {
  constexpr int BITS = 32 / VPL;
  constexpr int SPLIT = (VPL == 8 && !BF16) ? 2 : 1;  // chunks per word
  constexpr int VPC = VPL / SPLIT;                     // values per chunk
  constexpr int U = kDequantUnroll * SPLIT;
  const size_t chunks = words * SPLIT;
  const size_t base = static_cast<size_t>(blockIdx.x) * (kThreads * U) + threadIdx.x;
  const float s_tensor = per_tensor ? valid_scale(scales[0]) : 0.0f;
  uint32_t word[U];
  float sc[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t c = base + static_cast<size_t>(u) * kThreads;
    const size_t w = c / SPLIT;
    word[u] = (c < chunks) ? __builtin_nontemporal_load(words_in + w) : 0u;
    sc[u] = per_tensor ? s_tensor : ((c < chunks) ? scales[w >> block_words_log2] : 0.0f);
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t c = base + static_cast<size_t>(u) * kThreads;
    if (c < chunks) {
      const float s = per_tensor ? s_tensor : valid_scale(sc[u]);
      // the half of the word this chunk covers, moved down to field 0
      const uint32_t bits = (SPLIT == 2) ? (word[u] >> (16 * static_cast<uint32_t>(c & 1))) : word[u];
      float v[VPC];
#pragma unroll
      for (int j = 0; j < VPC; ++j) v[j] = s * static_cast<float>(unpack_field<BITS>(bits, j));
      store_chunk<VPC, BF16>(out, c, v);
    }
  }
  // native i8 tail (n % 4 values), per-tensor only
  if (VPL == 4 && base == 0) {
    const int8_t* bytes = reinterpret_cast<const int8_t*>(words_in);
    for (size_t i = words * 4; i < n; ++i) {
      float r = s_tensor * static_cast<float>(bytes[i]);
      if (BF16)
        reinterpret_cast<uint16_t*>(out)[i] = f32_to_bf16(r);
      else
        reinterpret_cast<float*>(out)[i] = r;
    }
  }
}

// Q8S -> bf16: a word gives only 8 bytes of output, so a lane takes two adjacent words (one
// 8-byte load, one 16-byte store); an odd last word is stored as 8 bytes.
__global__ void __launch_bounds__(kThreads)
dequantize_q8_bf16_kernel(const uint32_t* __restrict__ words_in, size_t words, size_t n,
                          unsigned block_words_log2, bool per_tensor, const float* __restrict__ scales,
                          uint16_t* __restrict__ out) {
  constexpr int U = kDequantUnroll;
  const size_t pairs = (words + 1) / 2;
  const size_t base = static_cast<size_t>(blockIdx.x) * (kThreads * U) + threadIdx.x;
  const float s_tensor = per_tensor ? valid_scale(scales[0]) : 0.0f;
  vuint2 wp[U];
  float sc[U][2];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t c = base + static_cast<size_t>(u) * kThreads;
    const size_t w0 = 2 * c;
    wp[u] = vuint2{0u, 0u};
    sc[u][0] = sc[u][1] = 0.0f;
    if (c < pairs) {
      const bool both = w0 + 1 < words;
      if (both)
        wp[u] = __builtin_nontemporal_load(reinterpret_cast<const vuint2*>(words_in) + c);
      else
        wp[u].x = __builtin_nontemporal_load(words_in + w0);
      if (!per_tensor) {
        sc[u][0] = scales[w0 >> block_words_log2];
        sc[u][1] = scales[(both ? w0 + 1 : w0) >> block_words_log2];
      }
    }
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t c = base + static_cast<size_t>(u) * kThreads;
    if (c < pairs) {
      const size_t w0 = 2 * c;
      const float sa = per_tensor ? s_tensor : valid_scale(sc[u][0]);
      const float sb = per_tensor ? s_tensor : valid_scale(sc[u][1]);
      uint32_t packed[4];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        packed[i] = f32x2_to_bf16x2(sa * static_cast<float>(unpack_field<8>(wp[u].x, 2 * i)),
                                    sa * static_cast<float>(unpack_field<8>(wp[u].x, 2 * i + 1)));
        packed[2 + i] = f32x2_to_bf16x2(sb * static_cast<float>(unpack_field<8>(wp[u].y, 2 * i)),
                                        sb * static_cast<float>(unpack_field<8>(wp[u].y, 2 * i + 1)));
      }
      if (w0 + 1 < words)
        __builtin_nontemporal_store(vuint4{packed[0], packed[1], packed[2], packed[3]}, reinterpret_cast<vuint4*>(out) + c);
      else
        __builtin_nontemporal_store(vuint2{packed[0], packed[1]}, reinterpret_cast<vuint2*>(out) + w0);
    }
  }
  // native i8 tail (n % 4 values), per-tensor only
  if (base == 0) {
    const int8_t* bytes = reinterpret_cast<const int8_t*>(words_in);
    for (size_t i = words * 4; i < n; ++i) out[i] = f32_to_bf16(s_tensor * static_cast<float>(bytes[i]));
  }
}

// Unaligned pointers: one value per lane (native Q8S, per tensor).
template <bool BF16>
__global__ void __launch_bounds__(kThreads)
dequantize_scalar_kernel(const int8_t* __restrict__ q, size_t n, const float* __restrict__ scales,
                         void* __restrict__ out) {
  const float s = valid_scale(scales[0]);
  const size_t stride = static_cast<size_t>(gridDim.x) * kThreads;
  for (size_t i = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x; i < n; i += stride) {
    float r = s * static_cast<float>(q[i]);
    if (BF16)
      reinterpret_cast<uint16_t*>(out)[i] = f32_to_bf16(r);
    else
      reinterpret_cast<float*>(out)[i] = r;
  }
}

struct RectDims {
  int rank;
  size_t shape[BQ_MAX_RANK];
  size_t blk[BQ_MAX_RANK];
  size_t grid[BQ_MAX_RANK];
};

__device__ __forceinline__ size_t rect_block_of(const RectDims& d, size_t index) {
  size_t block = 0, stride = 1;
  for (int i = d.rank - 1; i >= 0; --i) {
    size_t c = index % d.shape[i];
    index /= d.shape[i];
    block += c / d.blk[i] * stride;
    stride *= d.grid[i];
  }
  return block;
}

// General rectangle blocks: one thread per value.
template <int BITS, bool BF16>
__global__ void rect_dequantize_kernel(const uint32_t* __restrict__ words_in, RectDims d,
                                       size_t n, size_t last, size_t words_per_line, bool native,
                                       const float* __restrict__ scales, void* __restrict__ out) {
  constexpr int NQ = 32 / BITS;
  size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  int q;
  if (native) {
    q = reinterpret_cast<const int8_t*>(words_in)[i];
  } else {
    size_t line = i / last, c = i % last;
    q = unpack_field<BITS>(words_in[line * words_per_line + c / NQ], static_cast<int>(c % NQ));
  }
  float s = valid_scale(scales[d.rank ? rect_block_of(d, i) : 0]);
  float r = s * static_cast<float>(q);
  if (BF16)
    reinterpret_cast<uint16_t*>(out)[i] = f32_to_bf16(r);
  else
    reinterpret_cast<float*>(out)[i] = r;
}

inline unsigned grid_for(size_t items, unsigned cap) {
  size_t g = (items + kThreads - 1) / kThreads;
  if (g < 1) g = 1;
  return static_cast<unsigned>(g < cap ? g : cap);
}

}  // namespace

bq_status launch_dequantize_rect(const void* values, const size_t* shape, int rank,
                                 const size_t* blk, const float* scales, int value, int store,
                                 int out_dtype, void* out, hipStream_t st) {
  value = storage_value(value);  // (a full-range value unpacks like its symmetric twin)
  RectDims d{};
  d.rank = blk ? rank : 0;
  size_t n = 1;
  for (int i = 0; i < rank; ++i) {
    d.shape[i] = shape[i];
    d.blk[i] = blk ? blk[i] : shape[i];
    d.grid[i] = blk ? shape[i] / blk[i] : 1;
    n *= shape[i];
  }
  if (n == 0) return BQ_OK;
  const size_t last = rank ? shape[rank - 1] : 1;
  const size_t nq = static_cast<size_t>(num_quants(value));
  const size_t wpl = (last + nq - 1) / nq;
  const bool native = store == BQ_STORE_NATIVE;
  const bool bf16 = out_dtype == BQ_BF16;
  dim3 grid((n + kThreads - 1) / kThreads), tb(kThreads);
  const uint32_t* w = static_cast<const uint32_t*>(values);
#define BQ_RECT(B, H)                                                                          \
  hipLaunchKernelGGL((rect_dequantize_kernel<B, H>), grid, tb, 0, st, w, d, n, last, wpl, native, \
                     scales, out)
  if (value == BQ_Q8S) {
    if (bf16) BQ_RECT(8, true); else BQ_RECT(8, false);
  } else if (value == BQ_Q4S) {
    if (bf16) BQ_RECT(4, true); else BQ_RECT(4, false);
  } else {
    if (bf16) BQ_RECT(2, true); else BQ_RECT(2, false);
  }
#undef BQ_RECT
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

}  // namespace bq

using namespace bq;

extern "C" bq_status bqk_dequantize(const void* values, size_t n, int32_t block,
                                    const float* scales, int32_t value, int32_t store,
                                    int32_t out_dtype, void* out, void* stream) {
  BQ_NOTNULL(values);
  BQ_NOTNULL(scales);
  BQ_NOTNULL(out);
  if (!value_known(value)) BQ_FAIL(BQ_ERR_UNSUPPORTED_SCHEME, "unknown quant value %d", value);
  value = storage_value(value);  // (a full-range value unpacks like its symmetric twin)
  if (out_dtype != BQ_F32 && out_dtype != BQ_BF16)
    BQ_FAIL(BQ_ERR_DTYPE, "dequantize target must be f32 or bf16");
  if (store == BQ_STORE_NATIVE && value != BQ_Q8S)
    BQ_FAIL(BQ_ERR_UNSUPPORTED_SCHEME, "Can't store native sub-byte values");
  const size_t nq = static_cast<size_t>(num_quants(value));
  if (store == BQ_STORE_PACKED_U32 && n % nq)
    BQ_FAIL(BQ_ERR_SHAPE, "Can't store in u32: %zu values, %zu per word", n, nq);
  if (block < 0 || (block > 0 && (n % static_cast<size_t>(block) || !fused_block_ok(block, value))))
    BQ_FAIL(BQ_ERR_SHAPE, "%zu values / run block %d has no fused dequantize kernel", n, block);
  if (n == 0) return BQ_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool bf16 = out_dtype == BQ_BF16;
  const bool aligned = (reinterpret_cast<uintptr_t>(values) & 3u) == 0 &&
                       (reinterpret_cast<uintptr_t>(out) & 15u) == 0;
  if (!aligned) {
    if (value != BQ_Q8S || block != 0)
      BQ_FAIL(BQ_ERR_SHAPE, "dequantize needs 4-byte aligned values and a 16-byte aligned output");
    dim3 grid(grid_for(n, 0x7FFFFFFFu)), tb(kThreads);
    if (bf16)
      hipLaunchKernelGGL(dequantize_scalar_kernel<true>, grid, tb, 0, st,
                         static_cast<const int8_t*>(values), n, scales, out);
    else
      hipLaunchKernelGGL(dequantize_scalar_kernel<false>, grid, tb, 0, st,
                         static_cast<const int8_t*>(values), n, scales, out);
    BQ_HIP(hipGetLastError());
    return BQ_OK;
  }
  const size_t words = n / nq;
  unsigned log2bw = 0;
  if (block > 0) {
    size_t bw = static_cast<size_t>(block) / nq;
    while ((static_cast<size_t>(1) << log2bw) < bw) ++log2bw;
  }
  const bool per_tensor = block == 0;
  // chunks per workgroup: see dequantize_kernel (Q4S -> f32 has two chunks per word)
  const size_t split = (value == BQ_Q4S && !bf16) ? 2 : 1;
  const size_t per_wg = static_cast<size_t>(kThreads) * kDequantUnroll * split;
  const size_t g = (words * split + per_wg - 1) / per_wg;
  dim3 grid(static_cast<unsigned>(g ? g : 1)), tb(kThreads);
  const uint32_t* w = static_cast<const uint32_t*>(values);
  if (value == BQ_Q8S && bf16 && (reinterpret_cast<uintptr_t>(values) & 7u) == 0) {
    const size_t pairs_per_wg = static_cast<size_t>(kThreads) * kDequantUnroll;
    const size_t gp = ((words + 1) / 2 + pairs_per_wg - 1) / pairs_per_wg;
    hipLaunchKernelGGL(dequantize_q8_bf16_kernel, dim3(static_cast<unsigned>(gp ? gp : 1)), tb, 0, st, w, words, n,
                       log2bw, per_tensor, scales, static_cast<uint16_t*>(out));
    BQ_HIP(hipGetLastError());
    return BQ_OK;
  }
#define BQ_DEQ(V, H)                                                                            \
  hipLaunchKernelGGL((dequantize_kernel<V, H>), grid, tb, 0, st, w, words, n, log2bw, per_tensor, \
                     scales, out)
  if (value == BQ_Q8S) {
    if (bf16) BQ_DEQ(4, true); else BQ_DEQ(4, false);
  } else {
    if (bf16) BQ_DEQ(8, true); else BQ_DEQ(8, false);
  }
#undef BQ_DEQ
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}
