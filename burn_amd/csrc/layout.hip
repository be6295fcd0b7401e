// Layout ops on quantized tensors for gfx950: q_permute / q_swap_dims / q_flip
// (crates/burn-ndarray/src/ops/qtensor.rs:301-347). The reference permutes the values and, for
// block schemes, the scales with their blocks (scheme.permute_block_dims); tensors here are
// always dense row-major, so the result is materialised by a gather: one thread per output word
// (4 x i8 or 8 x i4 along the new last dim), each element fetched from its source position.
// Complete rather than fast: these are set-up operations (a transposed weight), not the hot loop.
#include "common.hpp"
#include "device_math.hpp"

namespace bq {

namespace {

struct GatherDims {
  int rank;
  uint32_t shape[BQ_MAX_RANK];   // output shape
  uint64_t stride[BQ_MAX_RANK];  // source stride (in elements) of the source dim that output dim d reads
  uint32_t flip[BQ_MAX_RANK];    // output dim d runs backwards over its source dim
};

__device__ __forceinline__ size_t source_index(const GatherDims& d, size_t e) {
  size_t idx = 0;
  for (int a = d.rank - 1; a >= 0; --a) {
    size_t c = e % d.shape[a];
    e /= d.shape[a];
    if (d.flip[a]) c = d.shape[a] - 1 - c;
    idx += c * d.stride[a];
  }
  return idx;
}

// BITS-wide fields; `native`: one i8 per element (n need not be a multiple of 4), else u32 words.
template <int BITS>
__global__ void __launch_bounds__(256)
q_gather_kernel(const uint32_t* __restrict__ src, uint32_t* __restrict__ dst, size_t n, GatherDims d, bool native) {
  constexpr int EPW = 32 / BITS;
  const size_t unit = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  const size_t e0 = unit * EPW;
  if (e0 >= n) return;
  uint32_t word = 0;
#pragma unroll
  for (int j = 0; j < EPW; ++j) {
    const size_t e = e0 + j;
    if (e >= n) break;
    const size_t idx = source_index(d, e);
    uint32_t v;
    if (BITS == 8)
      v = reinterpret_cast<const uint8_t*>(src)[idx];
    else  // (rows are whole words, so flat element idx sits in word idx / EPW)
      v = (src[idx / EPW] >> (BITS * (idx % EPW))) & ((1u << BITS) - 1u);
    word |= v << (BITS * j);
  }
  if (!native || e0 + EPW <= n) {
    dst[unit] = word;
  } else {
    for (size_t e = e0; e < n; ++e) reinterpret_cast<uint8_t*>(dst)[e] = static_cast<uint8_t>(word >> (8 * (e - e0)));
  }
}

__global__ void __launch_bounds__(256)
f32_gather_kernel(const float* __restrict__ src, float* __restrict__ dst, size_t n, GatherDims d) {
  const size_t e = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (e < n) dst[e] = src[source_index(d, e)];
}

GatherDims make_dims(const size_t* src_shape, int rank, const int32_t* axes, const uint8_t* flip) {
  GatherDims d{};
  d.rank = rank;
  uint64_t src_stride[BQ_MAX_RANK];
  uint64_t s = 1;
  for (int a = rank - 1; a >= 0; --a) {
    src_stride[a] = s;
    s *= src_shape[a];
  }
  for (int a = 0; a < rank; ++a) {
    d.shape[a] = static_cast<uint32_t>(src_shape[axes[a]]);
    d.stride[a] = src_stride[axes[a]];
    d.flip[a] = flip ? flip[axes[a]] : 0;
  }
  return d;
}

}  // namespace

// out = permute(flip(src)): output dim a is source dim axes[a], reversed where flip[axes[a]] is set.
// Values are i8 (native) or packed u32 words along the last dim; shapes are element shapes.
bq_status launch_q_gather(const void* src, void* dst, const size_t* src_shape, int rank, const int32_t* axes,
                          const uint8_t* flip, int value, bool native, hipStream_t st) {
  size_t n = 1;
  for (int a = 0; a < rank; ++a) n *= src_shape[a];
  if (n == 0) return BQ_OK;
  const GatherDims d = make_dims(src_shape, rank, axes, flip);
  const int epw = num_quants(value);
  const size_t units = (n + epw - 1) / epw;
  dim3 grid(static_cast<unsigned>((units + 255) / 256)), tb(256);
  if (value == BQ_Q8S)
    hipLaunchKernelGGL(q_gather_kernel<8>, grid, tb, 0, st, static_cast<const uint32_t*>(src),
                       static_cast<uint32_t*>(dst), n, d, native);
  else if (value == BQ_Q4S)
    hipLaunchKernelGGL(q_gather_kernel<4>, grid, tb, 0, st, static_cast<const uint32_t*>(src),
                       static_cast<uint32_t*>(dst), n, d, false);
  else
    hipLaunchKernelGGL(q_gather_kernel<2>, grid, tb, 0, st, static_cast<const uint32_t*>(src),
                       static_cast<uint32_t*>(dst), n, d, false);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

// The same for an f32 tensor (the block scales, in params_shape order).
bq_status launch_f32_gather(const float* src, float* dst, const size_t* src_shape, int rank, const int32_t* axes,
                            const uint8_t* flip, hipStream_t st) {
  size_t n = 1;
  for (int a = 0; a < rank; ++a) n *= src_shape[a];
  if (n == 0) return BQ_OK;
  const GatherDims d = make_dims(src_shape, rank, axes, flip);
  hipLaunchKernelGGL(f32_gather_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, st, src, dst, n, d);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

}  // namespace bq
