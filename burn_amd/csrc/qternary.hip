// Ternary weights on the bf16 matrix cores (gfx950): out[M,N] = gamma * X[M,K] x T[K,N], X f32,
// T a per-tensor Q2S weight -- values -1, 0, +1, sixteen 2-bit two's complement fields per packed
// word along N -- and gamma its scale.
//
// The reference multiplies such a weight without multiplications (crates/burn-ndarray/src/ops/
// qtensor.rs:442-517): per output it adds the activations whose weight is +1 and subtracts those
// whose weight is -1, in ascending k, then scales once. ternary_matmul_kernel (qmatmul.hip) keeps
// that order bit for bit, which makes every output one dependent chain of K additions: 100 us for
// a 4096 x 14336 weight that HBM delivers in 2 us. Nothing asks for that order (q_matmul is held
// to 1e-2, the reference's own ternary test to 2e-2), so by default the product runs here:
//   * the weights are exact in bf16; a field f becomes the bit pattern 0x4080 | (f ^ 2) << 5 =
//     4 + (f ^ 2) = t + 6 with one shift and one and-or per pair of rows (the 2 bits land in the
//     mantissa), and the 6 comes off through two more MFMAs per step against a constant -6
//     operand, into an accumulator of its own that is added at the end;
//   * gamma goes to the activations, xs = x * gamma in f32, split into two bf16 terms hi + lo
//     (16 significant bits; an output is off by about 1e-6 of the largest one) when the slice is
//     staged in LDS, once per workgroup;
//   * v_mfma_f32_16x16x32_bf16 multiplies 16 activation rows by 16 columns over 32 k rows, f32 sums.
// A workgroup of 8 waves owns a tile of 512 columns (32 packed words: 128 bytes of a weight row),
// 16 activation rows and a slice of up to 512 k rows. Its threads load the slice's weights as whole
// 128-byte rows (16 bytes per lane, every load in flight at once) and park them in LDS; wave v then
// multiplies columns 64 v .. 64 v + 63 over the whole slice: lane (c = lane % 16, kg = lane / 16)
// reads word c / 4 of its 8 k rows 8 kg .. 8 kg + 7 of a step and decodes that word's fields
// 4 (c % 4) .. + 3, one per MFMA, so an accumulator's 4 registers are rows 4 kg .. + 3 of 4
// adjacent columns and go to memory as 16-byte stores. No sum crosses waves; the K slices are
// added by the reduction kernel the other q_matmul kernels use, in a fixed order. An infinite or
// NaN activation sends its workgroup through a scalar loop that skips zero weights as the reference
// does (0 * inf would be NaN on the matrix cores).
#include <algorithm>

#include "common.hpp"
#include "device_math.hpp"

namespace bq {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));

constexpr int kTWaves = 8;
constexpr int kTThreads = kTWaves * kWave;   // 512
constexpr int kTRows = 16;                   // activation rows per workgroup (one MFMA tile)
constexpr int kTCols = 512;                  // columns per workgroup: 32 packed words, 128 bytes of a weight row
constexpr int kTWaveCols = kTCols / kTWaves; // 64 columns, 4 packed words per wave
constexpr int kTStep = 32;                   // k rows per MFMA
constexpr int kTMaxSlice = 512;              // k rows per workgroup
constexpr int kTChunks = kTMaxSlice * 8 / kTThreads;   // 16-byte weight loads per thread: 8
// LDS: the slice's activations as bf16 pairs, hi and lo planes, [16][slice / 2 + 4] words each (the
// pitch is 4 words past a multiple of 32: the 16 rows a quarter wave reads fall into distinct
// banks), then the weights, [slice][34] words (rows 8 apart -- the 4 row groups of a read -- land 16
// banks apart).
constexpr uint32_t kTWPitch = 34;
constexpr uint32_t kTLds = 2u * kTRows * (kTMaxSlice / 2 + 4) * 4u + kTMaxSlice * kTWPitch * 4u;   // 33 280 + 69 632 bytes

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2{lo, hi}, bf16x2));
}

// VEC: K % 4 == 0 and x 16-byte aligned (the activations are staged with 16-byte loads).
template <bool VEC>
__global__ void __launch_bounds__(kTThreads)
qternary_kernel(const float* __restrict__ x, const uint32_t* __restrict__ w, const float* __restrict__ scale,
                size_t M, size_t K, size_t N, uint32_t k_per_wg, float* __restrict__ part) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int c = lane & 15, kg = lane >> 4;
  const size_t NW = N / 16;
  const size_t col0 = static_cast<size_t>(blockIdx.x) * kTCols;
  const size_t m0 = static_cast<size_t>(blockIdx.z) * kTRows;
  const uint32_t rows = static_cast<uint32_t>(M - m0 < kTRows ? M - m0 : kTRows);
  const size_t k_begin = static_cast<size_t>(blockIdx.y) * k_per_wg;
  const uint32_t k_count = static_cast<uint32_t>(K - k_begin < k_per_wg ? K - k_begin : k_per_wg);  // rows of this slice that exist
  const float gamma = scale[0];
  float* const dst = part + (static_cast<size_t>(blockIdx.y) * M + m0) * N + col0;

  // ---- weights: chunk id = tid + 512 i is row id / 8 of the slice, 16-byte piece id % 8 of the tile's
  // 128 bytes. Every load goes out now. Rows past the slice's end and pieces past the row end (N is a
  // multiple of 64: a piece is in or out as a whole) get a lane offset outside the buffer: they read
  // as zero without touching memory, and a zero word decodes to t = 0.
  const __amdgpu_buffer_rsrc_t rsrc_w =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(w), 0, static_cast<int>(K * NW * 4), 0x00020000);
  const uint32_t w_row_bytes = static_cast<uint32_t>(NW) * 4u;
  vuint4 wl[kTChunks];
#pragma unroll
  for (int i = 0; i < kTChunks; ++i) {
    const uint32_t id = static_cast<uint32_t>(tid) + static_cast<uint32_t>(i) * kTThreads;
    const uint32_t row = id >> 3, piece = id & 7u;
    const bool ok = row < k_count && col0 / 16 + 4u * piece < NW;
    const uint32_t off = ok ? (static_cast<uint32_t>(k_begin) + row) * w_row_bytes + static_cast<uint32_t>(col0 / 16 + 4u * piece) * 4u : 0x80000000u;
    wl[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, off, 0, 0);
  }

  // ---- activations of the slice: xs = x * gamma as two bf16 terms, pairs (k, k + 1) per word
  uint32_t* const hi_plane = reinterpret_cast<uint32_t*>(smem);
  const uint32_t pitch = k_per_wg / 2u + 4u;                                   // words per row
  uint32_t* const lo_plane = hi_plane + kTRows * pitch;
  uint32_t* const w_lds = lo_plane + kTRows * pitch;
  int bad = 0;
  auto stage = [&](uint32_t r, uint32_t kk, float v0, float v1) {  // the pair (kk, kk + 1) of row r
    const uint32_t e = 0x7F800000u;
    bad |= (__float_as_uint(v0) & e) == e || (__float_as_uint(v1) & e) == e;
    const float t0 = v0 * gamma, t1 = v1 * gamma;
    const uint32_t hi = pack_bf16(t0, t1);
    const float d0 = t0 - __uint_as_float(hi << 16), d1 = t1 - __uint_as_float(hi & 0xFFFF0000u);  // exact
    hi_plane[r * pitch + kk / 2u] = hi;
    lo_plane[r * pitch + kk / 2u] = pack_bf16(d0, d1);
  };
  if (VEC) {
    // whole 16-byte groups: every load of the thread is in flight before the first is used. Rows the
    // batch does not have, and columns past K, stage zeros.
    constexpr int kMaxVecs = kTRows * (kTMaxSlice / 4) / kTThreads;   // 4
    const uint32_t vecs_per_row = k_per_wg / 4u;
    vfloat4 v[kMaxVecs];
#pragma unroll
    for (int i = 0; i < kMaxVecs; ++i) {
      const uint32_t idx = static_cast<uint32_t>(tid) + static_cast<uint32_t>(i) * kTThreads;
      const uint32_t r = idx / vecs_per_row, kk = (idx % vecs_per_row) * 4u;
      v[i] = (r < rows && kk < k_count) ? *reinterpret_cast<const vfloat4*>(x + (m0 + r) * K + k_begin + kk) : vfloat4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int i = 0; i < kMaxVecs; ++i) {
      const uint32_t idx = static_cast<uint32_t>(tid) + static_cast<uint32_t>(i) * kTThreads;
      const uint32_t r = idx / vecs_per_row, kk = (idx % vecs_per_row) * 4u;
      if (r < kTRows) {
        stage(r, kk, v[i].x, v[i].y);
        stage(r, kk + 2u, v[i].z, v[i].w);
      }
    }
  } else {
    const uint32_t pairs_per_row = k_per_wg / 2u;
    for (uint32_t idx = static_cast<uint32_t>(tid); idx < kTRows * pairs_per_row; idx += kTThreads) {
      const uint32_t r = idx / pairs_per_row, kk = (idx % pairs_per_row) * 2u;
      float v0 = 0.0f, v1 = 0.0f;
      if (r < rows) {
        const float* xr = x + (m0 + r) * K + k_begin;
        if (kk < k_count) v0 = xr[kk];
        if (kk + 1u < k_count) v1 = xr[kk + 1u];
      }
      stage(r, kk, v0, v1);
    }
  }
  // the weights into LDS (8-byte stores: the row pitch is not a multiple of 16 bytes)
#pragma unroll
  for (int i = 0; i < kTChunks; ++i) {
    const uint32_t id = static_cast<uint32_t>(tid) + static_cast<uint32_t>(i) * kTThreads;
    const uint32_t row = id >> 3, piece = id & 7u;
    if (row < k_per_wg) {
      vuint2* p = reinterpret_cast<vuint2*>(w_lds + row * kTWPitch + 4u * piece);
      p[0] = vuint2{wl[i].x, wl[i].y};
      p[1] = vuint2{wl[i].z, wl[i].w};
    }
  }
  const bool nonfinite = __syncthreads_or(bad) != 0;

  if (nonfinite) {
    // The reference's sum with its skips: a zero weight leaves the sum alone (no 0 * inf), +-1 adds
    // or subtracts the activation; then one multiply by gamma. Thread t owns column t of the tile.
    const size_t col = col0 + static_cast<size_t>(tid);
    if (col < N) {
      const unsigned shift = 2u * static_cast<unsigned>(col & 15u);
      for (uint32_t r = 0; r < rows; ++r) {
        const float* xr = x + (m0 + r) * K + k_begin;
        float sum = 0.0f;
        for (uint32_t k = 0; k < k_count; ++k) {
          const uint32_t f = (w_lds[k * kTWPitch + static_cast<uint32_t>(tid) / 16u] >> shift) & 3u;
          if (f == 1u) sum += xr[k];
          else if (f == 3u) sum -= xr[k];
        }
        dst[static_cast<size_t>(r) * N + tid] = sum * gamma;
      }
    }
    return;
  }

  // ---- multiply: wave v, columns 64 v .. + 63; MFMA jj (0..3) takes field 4 (c % 4) + jj of the
  // lane's word c / 4, i.e. column 16 (c / 4) + 4 (c % 4) + jj = 4 c + jj of the wave's 64
  floatx4 acc[4], off = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int jj = 0; jj < 4; ++jj) acc[jj] = floatx4{0.f, 0.f, 0.f, 0.f};
  const bf16x8 minus6 = __builtin_bit_cast(bf16x8, vuint4{0xC0C0C0C0u, 0xC0C0C0C0u, 0xC0C0C0C0u, 0xC0C0C0C0u});
  const uint32_t* const w_lane = w_lds + static_cast<uint32_t>(8 * kg) * kTWPitch + 4u * static_cast<uint32_t>(wave) + static_cast<uint32_t>(c >> 2);
  const uint32_t field_shift = 8u * static_cast<uint32_t>(c & 3);   // the lane's 4 fields to bits 0..7
  const int steps = static_cast<int>((k_count + kTStep - 1) / kTStep);
  for (int s = 0; s < steps; ++s) {
    const uint32_t kl = (static_cast<uint32_t>(s) * kTStep + 8u * kg) / 2u;   // word of the lane's first pair
    const bf16x8 a_hi = __builtin_bit_cast(bf16x8, *reinterpret_cast<const vuint4*>(hi_plane + c * pitch + kl));
    const bf16x8 a_lo = __builtin_bit_cast(bf16x8, *reinterpret_cast<const vuint4*>(lo_plane + c * pitch + kl));
    uint32_t z[4];   // rows (2 i, 2 i + 1): their 4 fields in bits 0..7 and 16..23, every field as f ^ 2
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t wa = w_lane[(static_cast<uint32_t>(s) * kTStep + 2 * i) * kTWPitch] >> field_shift;
      const uint32_t wb = w_lane[(static_cast<uint32_t>(s) * kTStep + 2 * i + 1) * kTWPitch] >> field_shift;
      z[i] = __builtin_amdgcn_perm(wb, wa, 0x0c040c00u) ^ 0x00AA00AAu;
    }
    bf16x8 bq[4];
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      uint32_t b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        // field jj of the low half to bits 5..6, of the high half to bits 21..22
        const int sh = 5 - 2 * jj;
        const uint32_t t = sh >= 0 ? z[i] << (sh & 31) : z[i] >> ((-sh) & 31);
        b[i] = (t & 0x00600060u) | 0x40804080u;   // bf16 pair: 4 + (f ^ 2) of row 2 i, of row 2 i + 1
      }
      bq[jj] = __builtin_bit_cast(bf16x8, vuint4{b[0], b[1], b[2], b[3]});
    }
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) acc[jj] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi, bq[jj], acc[jj], 0, 0, 0);
    off = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi, minus6, off, 0, 0, 0);
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) acc[jj] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_lo, bq[jj], acc[jj], 0, 0, 0);
    off = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_lo, minus6, off, 0, 0, 0);
  }
  // ---- element i of accumulator jj: row 4 kg + i, column 4 c + jj of the wave's 64: 16 bytes per row and lane
  const size_t wcol = static_cast<size_t>(wave) * kTWaveCols + 4u * static_cast<size_t>(c);
  if (col0 + wcol < N) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t r = 4u * static_cast<uint32_t>(kg) + static_cast<uint32_t>(i);
      // (every column of `off` holds -6 times the sum of the row's activations)
      if (r < rows)
        *reinterpret_cast<vfloat4*>(dst + static_cast<size_t>(r) * N + wcol) =
            vfloat4{acc[0][i] + off[i], acc[1][i] + off[i], acc[2][i] + off[i], acc[3][i] + off[i]};
    }
  }
}

struct TernaryPlan {
  unsigned tiles, row_tiles, slices;
  uint32_t k_per_wg;
};

// About one workgroup per CU of the 256-CU part, slices of 32 to 512 rows.
TernaryPlan ternary_plan(size_t m, size_t k, size_t n) {
  TernaryPlan p;
  p.tiles = static_cast<unsigned>((n + kTCols - 1) / kTCols);
  p.row_tiles = static_cast<unsigned>((m + kTRows - 1) / kTRows);
  const size_t columns = static_cast<size_t>(p.tiles) * p.row_tiles;
  const size_t want = std::max<size_t>(1, (256 + columns / 2) / columns);
  size_t kpw = ((k + want - 1) / want + kTStep - 1) / kTStep * kTStep;
  kpw = std::min<size_t>(std::max<size_t>(kpw, kTStep), kTMaxSlice);
  p.k_per_wg = static_cast<uint32_t>(kpw);
  p.slices = static_cast<unsigned>((k + kpw - 1) / kpw);
  return p;
}

}  // namespace

// Rows of whole 16-byte pieces (4 packed words, 64 columns), operands within 32-bit buffer offsets
// and launch limits.
bool ternary_mfma_ok(size_t m, size_t k, size_t n) {
  if (m == 0 || k == 0 || n == 0 || n % 64 != 0 || k * (n / 16) * 4 >= 0x7FFFFFFFull) return false;
  const TernaryPlan p = ternary_plan(m, k, n);
  return p.slices <= 65535u && p.row_tiles <= 65535u;
}

size_t ternary_workspace(size_t m, size_t k, size_t n) {
  return static_cast<size_t>(ternary_plan(m, k, n).slices) * m * n * sizeof(float);
}

// `part` receives slices x [M, N] partial products (gamma applied); the caller sums the slices.
bq_status launch_ternary_mfma(const float* x, const uint32_t* w, const float* scale, size_t m, size_t k, size_t n,
                              float* part, unsigned* slices_out, hipStream_t st) {
  const TernaryPlan p = ternary_plan(m, k, n);
  dim3 grid(p.tiles, p.slices, p.row_tiles), tb(kTThreads);
  if (k % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15u) == 0) {
    BQ_TRY(configure_dynamic_lds(reinterpret_cast<const void*>(qternary_kernel<true>), kTLds, "qternary_kernel"));
    hipLaunchKernelGGL(qternary_kernel<true>, grid, tb, kTLds, st, x, w, scale, m, k, n, p.k_per_wg, part);
  } else {
    BQ_TRY(configure_dynamic_lds(reinterpret_cast<const void*>(qternary_kernel<false>), kTLds, "qternary_kernel"));
    hipLaunchKernelGGL(qternary_kernel<false>, grid, tb, kTLds, st, x, w, scale, m, k, n, p.k_per_wg, part);
  }
  BQ_HIP(hipGetLastError());
  *slices_out = p.slices;
  return BQ_OK;
}

}  // namespace bq
