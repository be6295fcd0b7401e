// Layout ops on quantized tensors for gfx950: q_permute / q_swap_dims / q_flip
// (crates/burn-ndarray/src/ops/qtensor.rs:301-347), and the ops the reference's CPU backend runs on
// the integers without dequantizing (same file, :349-430): q_slice, q_select, q_gather, q_expand,
// q_argmax, q_argmin (the index map and arg kernels at the end of this file). The reference permutes the values and, for
// block schemes, the scales with their blocks (scheme.permute_block_dims); tensors here are
// always dense row-major, so the result is materialised: by a tiled transpose when 8-bit values
// swap their last two dims (a transposed weight, the usual case), else by a gather, one thread per
// output word (4 x i8, 8 x i4 or 16 x i2 along the new last dim), each element fetched from its
// source position. These are set-up operations, not the hot loop.
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

// I: uint32_t when every element index fits 32 bits (a 64-bit division costs several times a
// 32-bit one, and there is one per dim and element).
template <typename I>
__device__ __forceinline__ size_t source_index(const GatherDims& d, I e) {
  I idx = 0;
  for (int a = d.rank - 1; a >= 0; --a) {
    I c = e % static_cast<I>(d.shape[a]);
    e /= static_cast<I>(d.shape[a]);
    if (d.flip[a]) c = static_cast<I>(d.shape[a]) - 1 - c;
    idx += c * static_cast<I>(d.stride[a]);
  }
  return idx;
}

// BITS-wide fields; `native`: one i8 per element (n need not be a multiple of 4), else u32 words.
template <int BITS, typename I>
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
    const size_t idx = source_index<I>(d, static_cast<I>(e));
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

template <typename I>
__global__ void __launch_bounds__(256)
f32_gather_kernel(const float* __restrict__ src, float* __restrict__ dst, size_t n, GatherDims d) {
  const size_t e = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (e < n) dst[e] = src[source_index<I>(d, static_cast<I>(e))];
}

// 8-bit values, last two dims swapped: dst[b][c][r] = src[b][r][c], R and C multiples of 4. A
// workgroup moves a tile of 128 x 128 bytes. A thread loads the same word column of 4 consecutive
// rows, transposes the 4 x 4 bytes in registers (8 byte permutes) and writes the 4 resulting words
// -- 4 output rows, one word each -- to LDS; the tile leaves as whole 128-byte output rows. LDS row
// of output row 4 w + j is 32 j + w and rows are 33 words apart, so both the writes (w varies over
// the lanes) and the reads (the word index does) are spread over all banks.
constexpr int kTile = 128;
constexpr int kTileWords = kTile / 4;

__global__ void __launch_bounds__(256)
q8_transpose_kernel(const uint32_t* __restrict__ src, uint32_t* __restrict__ dst, uint32_t R, uint32_t C) {
  __shared__ uint32_t tile[kTile][kTileWords + 1];
  const size_t plane = static_cast<size_t>(R) * C / 4;  // words per batch entry
  src += plane * blockIdx.z;
  dst += plane * blockIdx.z;
  // Workgroups go to the 8 XCDs round robin. When the tile count allows, each XCD takes a run of
  // consecutive tiles down a tile column, whose outputs are adjacent 128-byte pieces of the same
  // output rows, instead of every eighth tile of a tile row ([8192,8192]: 31.6 -> 29.2 us; runs
  // along a tile row, which share source rows instead: 30.8 us).
  uint32_t bx = blockIdx.x, by = blockIdx.y;
  const uint32_t total = gridDim.x * gridDim.y;
  if (total % 8 == 0) {
    const uint32_t lin = blockIdx.y * gridDim.x + blockIdx.x, t = (lin & 7u) * (total / 8) + (lin >> 3);
    by = t % gridDim.y;
    bx = t / gridDim.y;
  }
  const uint32_t r0 = by * kTile, c0 = bx * kTile;
  const uint32_t cw = C / 4, rw = R / 4;
  const uint32_t w = threadIdx.x % kTileWords, q0 = threadIdx.x / kTileWords;  // word column; first row quad (of 8 per pass)
#pragma unroll
  for (uint32_t pass = 0; pass < 4; ++pass) {
    const uint32_t g = q0 + 8 * pass;  // row quad of the tile: rows 4 g .. 4 g + 3
    uint32_t in[4];
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) {
      const uint32_t r = r0 + 4 * g + i, c = c0 / 4 + w;
      in[i] = (r < R && c < cw) ? __builtin_nontemporal_load(src + static_cast<size_t>(r) * cw + c) : 0u;
    }
    // bytes (row i, column j) -> word j holds rows 0..3 of column j, low byte first
    const uint32_t t0 = __builtin_amdgcn_perm(in[1], in[0], 0x05010400u), t1 = __builtin_amdgcn_perm(in[1], in[0], 0x07030602u);
    const uint32_t t2 = __builtin_amdgcn_perm(in[3], in[2], 0x05010400u), t3 = __builtin_amdgcn_perm(in[3], in[2], 0x07030602u);
    tile[0 * kTileWords + w][g] = __builtin_amdgcn_perm(t2, t0, 0x05040100u);
    tile[1 * kTileWords + w][g] = __builtin_amdgcn_perm(t2, t0, 0x07060302u);
    tile[2 * kTileWords + w][g] = __builtin_amdgcn_perm(t3, t1, 0x05040100u);
    tile[3 * kTileWords + w][g] = __builtin_amdgcn_perm(t3, t1, 0x07060302u);
  }
  __syncthreads();
  // output row c0 + cc, words r0 / 4 + (0 .. 31): a wave writes two whole 128-byte rows per store
  const uint32_t g = threadIdx.x % kTileWords;
#pragma unroll
  for (uint32_t pass = 0; pass < kTile / 8; ++pass) {
    const uint32_t cc = threadIdx.x / kTileWords + 8 * pass;
    const uint32_t c = c0 + cc, rq = r0 / 4 + g;
    if (c < C && rq < rw)
      __builtin_nontemporal_store(tile[(cc & 3u) * kTileWords + (cc >> 2)][g], dst + static_cast<size_t>(c) * rw + rq);
  }
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
  value = storage_value(value);  // (only the width of a field matters here)
  size_t n = 1;
  for (int a = 0; a < rank; ++a) n *= src_shape[a];
  if (n == 0) return BQ_OK;
  // 8-bit values whose last two dims trade places (leading dims in place, nothing flipped), both
  // in whole words: the tiled transpose
  if (value == BQ_Q8S && rank >= 2 && axes[rank - 1] == rank - 2 && axes[rank - 2] == rank - 1) {
    bool plain = true;
    size_t batch = 1;
    for (int a = 0; a < rank; ++a) plain = plain && !(flip && flip[a]);
    for (int a = 0; a + 2 < rank; ++a) {
      plain = plain && axes[a] == a;
      batch *= src_shape[a];
    }
    const size_t rows = src_shape[rank - 2], cols = src_shape[rank - 1];
    const size_t tr = (rows + kTile - 1) / kTile, tc = (cols + kTile - 1) / kTile;
    if (plain && rows % 4 == 0 && cols % 4 == 0 && rows < 0x7FFFFFFFu && cols < 0x7FFFFFFFu && tr <= 65535 && batch <= 65535 &&
        (reinterpret_cast<uintptr_t>(src) & 3u) == 0 && (reinterpret_cast<uintptr_t>(dst) & 3u) == 0) {
      hipLaunchKernelGGL(q8_transpose_kernel, dim3(static_cast<unsigned>(tc), static_cast<unsigned>(tr), static_cast<unsigned>(batch)),
                         dim3(256), 0, st, static_cast<const uint32_t*>(src), static_cast<uint32_t*>(dst),
                         static_cast<uint32_t>(rows), static_cast<uint32_t>(cols));
      BQ_HIP(hipGetLastError());
      return BQ_OK;
    }
  }
  const GatherDims d = make_dims(src_shape, rank, axes, flip);
  const int epw = num_quants(value);
  const size_t units = (n + epw - 1) / epw;
  if ((units + 255) / 256 > 0x7FFFFFFFu) BQ_FAIL(BQ_ERR_SIZE, "permute of %zu values exceeds the launch grid", n);
  dim3 grid(static_cast<unsigned>((units + 255) / 256)), tb(256);
  const uint32_t* s32 = static_cast<const uint32_t*>(src);
  uint32_t* d32 = static_cast<uint32_t*>(dst);
  const bool small = n <= 0xFFFFFFFFull;
#define BQ_GATHER(B, NATIVE)                                                                  \
  if (small) hipLaunchKernelGGL((q_gather_kernel<B, uint32_t>), grid, tb, 0, st, s32, d32, n, d, NATIVE); \
  else hipLaunchKernelGGL((q_gather_kernel<B, size_t>), grid, tb, 0, st, s32, d32, n, d, NATIVE)
  if (value == BQ_Q8S) { BQ_GATHER(8, native); }
  else if (value == BQ_Q4S) { BQ_GATHER(4, false); }
  else { BQ_GATHER(2, false); }
#undef BQ_GATHER
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
  if ((n + 255) / 256 > 0x7FFFFFFFu) BQ_FAIL(BQ_ERR_SIZE, "permute of %zu scales exceeds the launch grid", n);
  if (n <= 0xFFFFFFFFull)
    hipLaunchKernelGGL(f32_gather_kernel<uint32_t>, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, st, src, dst, n, d);
  else
    hipLaunchKernelGGL(f32_gather_kernel<size_t>, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, st, src, dst, n, d);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

// ---- integer-domain slice / select / gather / expand ---------------------------------------------
// One kernel for all four: output element e with coordinates c reads source element
//   base + sum over dims a != index_dim of c[a] * stride[a] + i * stride[index_dim],
// i = c[index_dim] (slice, expand: a negative stride runs backwards, a zero stride broadcasts),
// indices[c[index_dim]] (select) or indices[e] (gather). An index outside its dim, which the
// reference panics on, is clamped into it: never a fault.
namespace {

struct FastDiv {
  uint32_t m, s, d;
};
__device__ __forceinline__ uint32_t fast_div(uint32_t n, const FastDiv& f) {
  return static_cast<uint32_t>((static_cast<uint64_t>(n) * f.m) >> f.s);
}
struct IndexMap {
  int rank;
  int fast;                      // every element index is below 2^31: `div` holds the constants for the output extents
  FastDiv div[BQ_MAX_RANK];
  uint32_t shape[BQ_MAX_RANK];   // output shape
  int64_t stride[BQ_MAX_RANK];   // source elements per step of output dim a
  int64_t base;
  int index_dim;                 // -1: none
  int index_mode;                // 1: indices[c[index_dim]] (select), 2: indices[e] (gather)
  int index_i64;                 // indices are i64 (else i32)
  int64_t index_limit;           // extent of the source dim the indices address
};

__device__ __forceinline__ int64_t mapped_index(const IndexMap& d, size_t e, const void* __restrict__ indices) {
  int64_t idx = d.base;
  size_t rem = e;
  uint32_t rem32 = static_cast<uint32_t>(e);
  for (int a = d.rank - 1; a >= 0; --a) {
    size_t c;
    if (d.fast) {  // (uniform over the launch)
      const uint32_t q = fast_div(rem32, d.div[a]);
      c = rem32 - q * d.div[a].d;
      rem32 = q;
    } else {
      c = rem % d.shape[a];
      rem /= d.shape[a];
    }
    int64_t i = static_cast<int64_t>(c);
    if (a == d.index_dim) {
      const size_t at = d.index_mode == 2 ? e : c;
      i = d.index_i64 ? static_cast<const int64_t*>(indices)[at] : static_cast<int64_t>(static_cast<const int32_t*>(indices)[at]);
      i = i < 0 ? 0 : (i >= d.index_limit ? d.index_limit - 1 : i);
    }
    idx += i * d.stride[a];
  }
  return idx;
}

template <int BITS>
__global__ void __launch_bounds__(256)
q_index_map_kernel(const uint32_t* __restrict__ src, uint32_t* __restrict__ dst, size_t n, IndexMap d, bool src_native, bool dst_native,
                   const void* __restrict__ indices) {
  constexpr int EPW = 32 / BITS;
  const size_t unit = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  const size_t e0 = unit * EPW;
  if (e0 >= n) return;
  uint32_t word = 0;
#pragma unroll
  for (int j = 0; j < EPW; ++j) {
    const size_t e = e0 + j;
    if (e >= n) break;
    const size_t idx = static_cast<size_t>(mapped_index(d, e, indices));
    uint32_t v;
    if (BITS == 8 || src_native)
      v = reinterpret_cast<const uint8_t*>(src)[idx] & ((1u << BITS) - 1u);
    else  // (rows are whole words, so flat element idx sits in word idx / EPW)
      v = (src[idx / EPW] >> (BITS * (idx % EPW))) & ((1u << BITS) - 1u);
    word |= v << (BITS * j);
  }
  if (!dst_native) {
    dst[unit] = word;
  } else {  // one i8 per value: sign-extend the field
    for (int j = 0; j < EPW && e0 + j < n; ++j)
      reinterpret_cast<int8_t*>(dst)[e0 + j] = static_cast<int8_t>(static_cast<int32_t>(word << (32 - BITS * (j + 1))) >> (32 - BITS));
  }
}

__global__ void __launch_bounds__(256)
f32_index_map_kernel(const float* __restrict__ src, float* __restrict__ dst, size_t n, IndexMap d, const void* __restrict__ indices) {
  const size_t e = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (e < n) dst[e] = src[mapped_index(d, e, indices)];
}

// Fast path of the index maps: the innermost output dim walks the source with stride 1 and carries
// no index, so an output row is one contiguous run of source bytes (a slice, select or expand that
// leaves the last dim alone, or cuts it at word boundaries). A lane copies 16 (or 4) bytes; the
// row's coordinates come from divisions by constants the host prepared (q = (n * m) >> s, exact for
// n < 2^31), a few instructions per dim instead of a 64-bit division each.
struct RowMap {
  int rank;                        // outer dims (output rank - 1)
  FastDiv div[BQ_MAX_RANK];        // by the extent of outer dim a
  int64_t stride[BQ_MAX_RANK];     // source bytes per step of outer dim a
  int64_t base;                    // source byte offset of the first row
  FastDiv per_row;                 // by the vectors per row
  int index_dim;                   // outer dim whose coordinate goes through `indices`, or -1
  int index_i64;
  int64_t index_limit;
};

template <typename V>
__device__ __forceinline__ void row_copy_one(const unsigned char* __restrict__ src, unsigned char* __restrict__ dst, uint32_t u,
                                             const RowMap& d, const void* __restrict__ indices) {
  const uint32_t row = fast_div(u, d.per_row), v = u - row * d.per_row.d;
  int64_t off = d.base + static_cast<int64_t>(v) * static_cast<int64_t>(sizeof(V));
  uint32_t rem = row;
  for (int a = d.rank - 1; a >= 0; --a) {
    const uint32_t q = fast_div(rem, d.div[a]);
    int64_t i = static_cast<int64_t>(rem - q * d.div[a].d);
    rem = q;
    if (a == d.index_dim) {
      i = d.index_i64 ? static_cast<const int64_t*>(indices)[i] : static_cast<int64_t>(static_cast<const int32_t*>(indices)[i]);
      i = i < 0 ? 0 : (i >= d.index_limit ? d.index_limit - 1 : i);
    }
    off += i * d.stride[a];
  }
  const V val = __builtin_nontemporal_load(reinterpret_cast<const V*>(src + off));
  __builtin_nontemporal_store(val, reinterpret_cast<V*>(dst) + u);
}

template <typename V>
__global__ void __launch_bounds__(256)
row_copy_kernel(const unsigned char* __restrict__ src, unsigned char* __restrict__ dst, uint32_t total, RowMap d,
                const void* __restrict__ indices) {
  const uint32_t u = blockIdx.x * 256u + threadIdx.x;
  if (u < total) row_copy_one<V>(src, dst, u, d, indices);
}

// Values and block scales of one op in one launch: the first `blocks_a` workgroups move job a, the
// rest job b (a second launch for a few megabytes of scales costs more than it moves).
struct RowJob {
  const unsigned char* src;
  unsigned char* dst;
  uint32_t total;
  uint32_t wide;  // 16 bytes per lane (else 4)
  RowMap d;
};

__global__ void __launch_bounds__(256)
row_copy_pair_kernel(RowJob a, RowJob b, uint32_t blocks_a, const void* __restrict__ indices) {
  // (two spelled-out branches: picking one of the two argument structs through a reference would copy both to scratch)
  if (blockIdx.x < blocks_a) {
    const uint32_t u = blockIdx.x * 256u + threadIdx.x;
    if (u >= a.total) return;
    if (a.wide) row_copy_one<vuint4>(a.src, a.dst, u, a.d, indices);
    else row_copy_one<uint32_t>(a.src, a.dst, u, a.d, indices);
  } else {
    const uint32_t u = (blockIdx.x - blocks_a) * 256u + threadIdx.x;
    if (u >= b.total) return;
    if (b.wide) row_copy_one<vuint4>(b.src, b.dst, u, b.d, indices);
    else row_copy_one<uint32_t>(b.src, b.dst, u, b.d, indices);
  }
}

__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b) {
  typedef unsigned short ushort2v __attribute__((ext_vector_type(2)));
  const ushort2v x = __builtin_bit_cast(ushort2v, a), y = __builtin_bit_cast(ushort2v, b);
  const ushort2v r = {static_cast<unsigned short>(x.x > y.x ? x.x : y.x), static_cast<unsigned short>(x.y > y.y ? x.y : y.y)};
  return __builtin_bit_cast(uint32_t, r);
}

// Arg max / min along the last dim of 8-bit values: a wave per row. A lane walks the row 16 bytes at
// a time keeping its first best; the wave then takes the best of 64 (value, then lowest index) keys.
__global__ void __launch_bounds__(256)
q8_arg_last_kernel(const int8_t* __restrict__ src, size_t rows, size_t len, bool want_max, bool out_i64, void* __restrict__ out) {
  const size_t row = static_cast<size_t>(blockIdx.x) * 4 + threadIdx.x / kWave;
  if (row >= rows) return;
  const int lane = threadIdx.x & (kWave - 1);
  const int8_t* p = src + row * len;
  int best = want_max ? -129 : 128;
  uint32_t best_at = 0xFFFFFFFFu;
  auto take = [&](int v, uint32_t at) {
    if (want_max ? v > best : v < best) {
      best = v;
      best_at = at;
    }
  };
  const bool vec = (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
  const size_t whole = vec ? len / 16 * 16 : 0;
  // Sixteen values at a time without a compare per value: a byte u (the value with its sign bit
  // flipped: unsigned order is the signed order; all bits flipped for a minimum) becomes the 16-bit key
  // u << 8 | 15 - position, two keys to a register (one byte permute against a constant of position
  // codes), and packed 16-bit maxima leave the largest value at its lowest position.
  const uint32_t flip = want_max ? 0x80808080u : 0x7F7F7F7Fu;
  auto take16 = [&](const vuint4& w, size_t i) {
    const uint32_t ws[4] = {w.x ^ flip, w.y ^ flip, w.z ^ flip, w.w ^ flip};
    uint32_t m = 0;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      // position codes 15 - (4 q + j) of the word's four bytes
      const uint32_t codes = (15u - 4u * q) | ((14u - 4u * q) << 8) | ((13u - 4u * q) << 16) | ((12u - 4u * q) << 24);
      const uint32_t k01 = __builtin_amdgcn_perm(ws[q], codes, 0x05010400u);  // (u1, code1, u0, code0)
      const uint32_t k23 = __builtin_amdgcn_perm(ws[q], codes, 0x07030602u);  // (u3, code3, u2, code2)
      m = pk_max_u16(m, pk_max_u16(k01, k23));
    }
    const uint32_t lo = m & 0xFFFFu, hi = m >> 16;
    const uint32_t key = lo > hi ? lo : hi;
    // back to the value's own scale for the comparison with the running best
    const int v = want_max ? static_cast<int>(key >> 8) - 128 : 127 - static_cast<int>(key >> 8);
    take(v, static_cast<uint32_t>(i) + 15u - (key & 0xFFu));
  };
  size_t i = static_cast<size_t>(lane) * 16;
  for (; i + 3 * kWave * 16 < whole; i += 4 * kWave * 16) {   // four loads in flight per lane, taken in ascending order
    vuint4 w[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) w[u] = __builtin_nontemporal_load(reinterpret_cast<const vuint4*>(p + i + u * kWave * 16));
#pragma unroll
    for (int u = 0; u < 4; ++u) take16(w[u], i + u * kWave * 16);
  }
  for (; i < whole; i += kWave * 16) take16(*reinterpret_cast<const vuint4*>(p + i), i);
  for (size_t r = whole + lane; r < len; r += kWave) take(p[r], static_cast<uint32_t>(r));
  // key: the value in the high word (flipped for a minimum), the complement of the index below it:
  // the largest key is the best value at the lowest index
  uint64_t key = (static_cast<uint64_t>(static_cast<uint32_t>(want_max ? best + 129 : 128 - best)) << 32) | (0xFFFFFFFFu - best_at);
#pragma unroll
  for (int s = 32; s >= 1; s >>= 1) {
    const uint32_t hi = __shfl_xor(static_cast<uint32_t>(key >> 32), s), lo = __shfl_xor(static_cast<uint32_t>(key), s);
    const uint64_t other = (static_cast<uint64_t>(hi) << 32) | lo;
    key = other > key ? other : key;
  }
  if (lane == 0) {
    const uint32_t at = 0xFFFFFFFFu - static_cast<uint32_t>(key);
    if (out_i64) static_cast<int64_t*>(out)[row] = static_cast<int64_t>(at);
    else static_cast<int32_t*>(out)[row] = static_cast<int32_t>(at);
  }
}

// q_argmax / q_argmin on the stored integers: per output position, the first index along `dim` of the
// largest (smallest) value -- ties keep the lowest index, as the reference's fold with a strict
// comparison does (crates/burn-ndarray/src/ops/base.rs:1727-1750). One thread per output position.
template <int BITS>
__global__ void __launch_bounds__(256)
q_arg_kernel(const uint32_t* __restrict__ src, bool native, size_t outer, size_t len, size_t inner, bool want_max, bool out_i64,
             void* __restrict__ out) {
  constexpr int EPW = 32 / BITS;
  const size_t pos = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (pos >= outer * inner) return;
  const size_t o = pos / inner, in = pos % inner;
  int best = 0;
  size_t best_at = 0;
  for (size_t i = 0; i < len; ++i) {
    const size_t idx = (o * len + i) * inner + in;
    int v;
    if (BITS == 8 || native) v = reinterpret_cast<const int8_t*>(src)[idx];
    else v = static_cast<int32_t>(src[idx / EPW] << (32 - BITS - BITS * (idx % EPW))) >> (32 - BITS);
    if (i == 0 || (want_max ? v > best : v < best)) {
      best = v;
      best_at = i;
    }
  }
  if (out_i64) static_cast<int64_t*>(out)[pos] = static_cast<int64_t>(best_at);
  else static_cast<int32_t*>(out)[pos] = static_cast<int32_t>(best_at);
}

FastDiv make_fast_div(uint32_t d) {
  FastDiv f{};
  f.d = d;
  uint32_t l = 0;
  while ((1ull << l) < d) ++l;                       // ceil(log2 d)
  f.s = 31 + l;
  f.m = static_cast<uint32_t>(((1ull << f.s) + d - 1) / d);   // ceil(2^(31 + l) / d) <= 2^32 - 1 for d >= 1 ... (d = 1: 2^31)
  return f;
}

IndexMap make_index_map(const size_t* out_shape, int rank, const int64_t* stride, int64_t base, int index_dim, int index_mode,
                        int index_dtype, size_t index_limit) {
  IndexMap d{};
  d.rank = rank;
  size_t n = 1;
  for (int a = 0; a < rank; ++a) {
    d.shape[a] = static_cast<uint32_t>(out_shape[a]);
    d.stride[a] = stride[a];
    d.div[a] = make_fast_div(static_cast<uint32_t>(out_shape[a] ? out_shape[a] : 1));
    n *= out_shape[a];
  }
  d.fast = n < 0x7FFFFFFFull;
  d.base = base;
  d.index_dim = index_dim;
  d.index_mode = index_mode;
  d.index_i64 = index_dtype == BQ_I64;
  d.index_limit = static_cast<int64_t>(index_limit);
  return d;
}

// Plans the row-run copy when the map allows it; returns false otherwise.
// `elem_bits`: bits per element on both sides (8 for native and 8-bit values, 4, 2, or 32 for scales).
bool plan_row_copy(const void* src, void* dst, const size_t* out_shape, int rank, const int64_t* stride, int64_t base, int index_dim,
                   int index_mode, int index_dtype, size_t index_limit, int elem_bits, RowJob* job) {
  if (rank < 1 || stride[rank - 1] != 1 || index_dim == rank - 1 || (index_dim >= 0 && index_mode != 1)) return false;
  const size_t row_bits = out_shape[rank - 1] * static_cast<size_t>(elem_bits);
  size_t rows = 1;
  for (int a = 0; a + 1 < rank; ++a) rows *= out_shape[a];
  if (rows == 0 || row_bits == 0) return false;
  auto aligned = [&](size_t vb) {
    if (row_bits % (8 * vb) != 0 || (base * elem_bits) % static_cast<int64_t>(8 * vb) != 0) return false;
    for (int a = 0; a + 1 < rank; ++a)
      if ((stride[a] * elem_bits) % static_cast<int64_t>(8 * vb) != 0) return false;
    return (reinterpret_cast<uintptr_t>(src) % vb) == 0 && (reinterpret_cast<uintptr_t>(dst) % vb) == 0;
  };
  const size_t vb = aligned(16) ? 16 : (aligned(4) ? 4 : 0);
  if (vb == 0) return false;
  const size_t per_row = row_bits / (8 * vb), total = rows * per_row;
  if (total >= 0x7FFFFFFFull || rows >= 0x7FFFFFFFull) return false;
  RowMap& d = job->d;
  d = RowMap{};
  d.rank = rank - 1;
  for (int a = 0; a + 1 < rank; ++a) {
    d.div[a] = make_fast_div(static_cast<uint32_t>(out_shape[a]));
    d.stride[a] = stride[a] * elem_bits / 8;
  }
  d.base = base * elem_bits / 8;
  d.per_row = make_fast_div(static_cast<uint32_t>(per_row));
  d.index_dim = index_dim;
  d.index_i64 = index_dtype == BQ_I64;
  d.index_limit = static_cast<int64_t>(index_limit);
  job->src = static_cast<const unsigned char*>(src);
  job->dst = static_cast<unsigned char*>(dst);
  job->total = static_cast<uint32_t>(total);
  job->wide = vb == 16;
  return true;
}

// Launches the row-run copy when the map allows it; returns false (nothing launched) otherwise.
bool try_row_copy(const void* src, void* dst, const size_t* out_shape, int rank, const int64_t* stride, int64_t base, int index_dim,
                  int index_mode, const void* indices, int index_dtype, size_t index_limit, int elem_bits, hipStream_t st) {
  RowJob j{};
  if (!plan_row_copy(src, dst, out_shape, rank, stride, base, index_dim, index_mode, index_dtype, index_limit, elem_bits, &j)) return false;
  dim3 grid((j.total + 255u) / 256u), tb(256);
  if (j.wide) hipLaunchKernelGGL(row_copy_kernel<vuint4>, grid, tb, 0, st, j.src, j.dst, j.total, j.d, indices);
  else hipLaunchKernelGGL(row_copy_kernel<uint32_t>, grid, tb, 0, st, j.src, j.dst, j.total, j.d, indices);
  return true;
}

}  // namespace

// Values of `out_shape` (every extent below 2^32) gathered through the index map described above.
// `indices` (device memory, BQ_I32 or BQ_I64) is read when index_dim >= 0.
bq_status launch_q_index_map(const void* src, void* dst, const size_t* out_shape, int rank, const int64_t* stride, int64_t base,
                             int index_dim, int index_mode, const void* indices, int index_dtype, size_t index_limit, int value,
                             bool src_native, bool dst_native, hipStream_t st) {
  size_t n = 1;
  for (int a = 0; a < rank; ++a) n *= out_shape[a];
  if (n == 0) return BQ_OK;
  const int bits = value_bits(value);
  // whole rows of bytes when both sides store the values the same way (8-bit values: native bytes are the packed words' bytes)
  if ((src_native == dst_native || bits == 8) &&
      try_row_copy(src, dst, out_shape, rank, stride, base, index_dim, index_mode, indices, index_dtype, index_limit,
                   (src_native && dst_native) ? 8 : bits, st)) {
    BQ_HIP(hipGetLastError());
    return BQ_OK;
  }
  const IndexMap d = make_index_map(out_shape, rank, stride, base, index_dim, index_mode, index_dtype, index_limit);
  const size_t units = (n + 32 / bits - 1) / (32 / bits);
  if ((units + 255) / 256 > 0x7FFFFFFFu) BQ_FAIL(BQ_ERR_SIZE, "an index map over %zu values exceeds the launch grid", n);
  dim3 grid(static_cast<unsigned>((units + 255) / 256)), tb(256);
  const uint32_t* s32 = static_cast<const uint32_t*>(src);
  uint32_t* d32 = static_cast<uint32_t*>(dst);
  if (bits == 8) hipLaunchKernelGGL(q_index_map_kernel<8>, grid, tb, 0, st, s32, d32, n, d, src_native, dst_native, indices);
  else if (bits == 4) hipLaunchKernelGGL(q_index_map_kernel<4>, grid, tb, 0, st, s32, d32, n, d, src_native, dst_native, indices);
  else hipLaunchKernelGGL(q_index_map_kernel<2>, grid, tb, 0, st, s32, d32, n, d, src_native, dst_native, indices);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

// The same for an f32 tensor (the block scales, in params_shape order).
bq_status launch_f32_index_map(const float* src, float* dst, const size_t* out_shape, int rank, const int64_t* stride, int64_t base,
                               int index_dim, int index_mode, const void* indices, int index_dtype, size_t index_limit, hipStream_t st) {
  size_t n = 1;
  for (int a = 0; a < rank; ++a) n *= out_shape[a];
  if (n == 0) return BQ_OK;
  if (try_row_copy(src, dst, out_shape, rank, stride, base, index_dim, index_mode, indices, index_dtype, index_limit, 32, st)) {
    BQ_HIP(hipGetLastError());
    return BQ_OK;
  }
  const IndexMap d = make_index_map(out_shape, rank, stride, base, index_dim, index_mode, index_dtype, index_limit);
  if ((n + 255) / 256 > 0x7FFFFFFFu) BQ_FAIL(BQ_ERR_SIZE, "an index map over %zu scales exceeds the launch grid", n);
  hipLaunchKernelGGL(f32_index_map_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, st, src, dst, n, d, indices);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

// Values and f32 block scales of one op together, when both maps are whole-row copies: one launch,
// *fused set. Otherwise nothing is launched and the caller runs the two maps one after the other.
bq_status launch_index_map_pair(const void* src, void* dst, const size_t* out_shape, const int64_t* stride, int64_t base, int value,
                                bool src_native, bool dst_native, const float* s_src, float* s_dst, const size_t* s_shape,
                                const int64_t* s_stride, int64_t s_base, int rank, int index_dim, int index_mode, const void* indices,
                                int index_dtype, size_t index_limit, bool* fused, hipStream_t st) {
  *fused = false;
  const int bits = value_bits(value);
  if (!(src_native == dst_native || bits == 8)) return BQ_OK;
  RowJob a{}, b{};
  if (!plan_row_copy(src, dst, out_shape, rank, stride, base, index_dim, index_mode, index_dtype, index_limit,
                     (src_native && dst_native) ? 8 : bits, &a) ||
      !plan_row_copy(s_src, s_dst, s_shape, rank, s_stride, s_base, index_dim, index_mode, index_dtype, index_limit, 32, &b))
    return BQ_OK;
  const uint32_t blocks_a = (a.total + 255u) / 256u, blocks_b = (b.total + 255u) / 256u;
  hipLaunchKernelGGL(row_copy_pair_kernel, dim3(blocks_a + blocks_b), dim3(256), 0, st, a, b, blocks_a, indices);
  BQ_HIP(hipGetLastError());
  *fused = true;
  return BQ_OK;
}

// out[outer][1][inner] = arg max / min over the `len` values along the reduced dim (i32 or i64).
bq_status launch_q_arg(const void* src, int value, bool native, size_t outer, size_t len, size_t inner, bool want_max, int out_dtype,
                       void* out, hipStream_t st) {
  const size_t n = outer * inner;
  if (n == 0) return BQ_OK;
  if ((n + 255) / 256 > 0x7FFFFFFFu) BQ_FAIL(BQ_ERR_SIZE, "an arg reduction over %zu positions exceeds the launch grid", n);
  dim3 grid(static_cast<unsigned>((n + 255) / 256)), tb(256);
  const uint32_t* s32 = static_cast<const uint32_t*>(src);
  const int bits = value_bits(value);
  const bool i64 = out_dtype == BQ_I64;
  if ((bits == 8 || native) && inner == 1 && len >= 64 && len < 0xFFFFFFFFull && (outer + 3) / 4 <= 0x7FFFFFFFu) {
    hipLaunchKernelGGL(q8_arg_last_kernel, dim3(static_cast<unsigned>((outer + 3) / 4)), dim3(256), 0, st,
                       static_cast<const int8_t*>(src), outer, len, want_max, i64, out);
    BQ_HIP(hipGetLastError());
    return BQ_OK;
  }
  if (bits == 8) hipLaunchKernelGGL(q_arg_kernel<8>, grid, tb, 0, st, s32, native, outer, len, inner, want_max, i64, out);
  else if (bits == 4) hipLaunchKernelGGL(q_arg_kernel<4>, grid, tb, 0, st, s32, native, outer, len, inner, want_max, i64, out);
  else hipLaunchKernelGGL(q_arg_kernel<2>, grid, tb, 0, st, s32, native, outer, len, inner, want_max, i64, out);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

}  // namespace bq
