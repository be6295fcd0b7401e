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
// Lane (c = lane % 16, kg = lane / 16) loads 8 bytes -- packed words 2 c and 2 c + 1 of the tile's
// 32 -- of each of its 8 k rows 8 kg .. 8 kg + 7 of a step: every load instruction reads whole
// 128-byte rows, and MFMA j (0..31) multiplies field j % 16 of word j / 16 of every lane, i.e.
// column 32 c + j of the tile, straight from the registers. A workgroup of 8 waves owns a tile of
// 512 columns and 16 rows and a slice of K that its waves divide among themselves; they are added
// through LDS as a tree, the slices by the reduction kernel the other q_matmul kernels use, both
// in a fixed order. An infinite or NaN activation sends its workgroup through a scalar loop that
// skips zero weights as the reference does (0 * inf would be NaN on the matrix cores).
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
constexpr int kTStep = 32;                   // k rows per MFMA
constexpr int kTMaxSteps = 4;                // steps per wave: all of its weight loads are issued up front
constexpr int kTMaxSlice = kTWaves * kTMaxSteps * kTStep;   // 1024 k rows per workgroup
constexpr int kTOps = 32;                    // MFMA column operands per lane and step
// LDS: the slice's activations as bf16 pairs, hi and lo planes, [16][slice / 2 + 4] words each (the
// pitch is 4 words past a multiple of 32: the 16 rows a quarter wave reads fall into distinct
// banks); afterwards the same memory carries the tree sum of the waves (4 images of 32 KiB) and
// the output tile.
constexpr uint32_t kTImage = kTOps * kWave * 16;                 // one wave's accumulators: 32 KiB
constexpr uint32_t kTLds = 4 * kTImage;                          // 128 KiB
constexpr uint32_t kTOutPitch = kTCols + 64;                     // output tile pitch in floats (4 spare per 32 columns)
static_assert(2u * kTRows * (kTMaxSlice / 2 + 4) * 4u <= kTLds && kTRows * kTOutPitch * 4u <= kTLds, "LDS plan");

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2{lo, hi}, bf16x2));
}

__global__ void __launch_bounds__(kTThreads)
qternary_kernel(const float* __restrict__ x, const uint32_t* __restrict__ w, const float* __restrict__ scale,
                size_t M, size_t K, size_t N, uint32_t rows_per_wave, float* __restrict__ part) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int c = lane & 15, kg = lane >> 4;
  const size_t NW = N / 16;
  const size_t col0 = static_cast<size_t>(blockIdx.x) * kTCols;
  const size_t m0 = static_cast<size_t>(blockIdx.z) * kTRows;
  const uint32_t rows = static_cast<uint32_t>(M - m0 < kTRows ? M - m0 : kTRows);
  const uint32_t k_per_wg = rows_per_wave * kTWaves;
  const size_t k_begin = static_cast<size_t>(blockIdx.y) * k_per_wg;
  const uint32_t k_count = static_cast<uint32_t>(K - k_begin < k_per_wg ? K - k_begin : k_per_wg);  // rows of this slice that exist
  const float gamma = scale[0];
  float* const dst = part + (static_cast<size_t>(blockIdx.y) * M + m0) * N + col0;

  // ---- weights: every load of the wave goes out now (at most 4 steps x 8 rows x 8 bytes per lane).
  // Rows past K and words past the row end get a lane offset outside the buffer: they read as zero
  // without touching memory, and a zero word decodes to t = 0.
  const __amdgpu_buffer_rsrc_t rsrc_w =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(w), 0, static_cast<int>(K * NW * 4), 0x00020000);
  const uint32_t w_row_bytes = static_cast<uint32_t>(NW) * 4u;
  const uint32_t kw0 = static_cast<uint32_t>(wave) * rows_per_wave;            // first row of this wave inside the slice
  const int steps = kw0 < k_count ? static_cast<int>((std::min(k_count - kw0, rows_per_wave) + kTStep - 1) / kTStep) : 0;
  const size_t word0 = col0 / 16 + 2u * static_cast<size_t>(c);
  vuint2 wd[kTMaxSteps][8];
#pragma unroll
  for (int s = 0; s < kTMaxSteps; ++s)
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const size_t row = k_begin + kw0 + static_cast<size_t>(s) * kTStep + 8u * kg + r;
      const bool ok = s < steps && row < K && word0 < NW;
      const uint32_t off = ok ? static_cast<uint32_t>(row) * w_row_bytes + static_cast<uint32_t>(word0) * 4u : 0x80000000u;
      wd[s][r] = __builtin_amdgcn_raw_buffer_load_b64(rsrc_w, off, 0, 0);  // (N % 32 == 0: a pair of words is in or out as a whole)
    }

  // ---- activations of the slice: xs = x * gamma as two bf16 terms, pairs (k, k + 1) per word
  uint32_t* const hi_plane = reinterpret_cast<uint32_t*>(smem);
  const uint32_t pitch = k_per_wg / 2u + 4u;                                   // words per row
  uint32_t* const lo_plane = hi_plane + kTRows * pitch;
  int bad = 0;
  {
    const uint32_t pairs_per_row = k_per_wg / 2u;
    for (uint32_t idx = static_cast<uint32_t>(tid); idx < kTRows * pairs_per_row; idx += kTThreads) {
      const uint32_t r = idx / pairs_per_row, kk = (idx % pairs_per_row) * 2u;
      float v0 = 0.0f, v1 = 0.0f;
      if (r < rows) {
        const float* xr = x + (m0 + r) * K + k_begin;
        if (kk < k_count) v0 = xr[kk];
        if (kk + 1u < k_count) v1 = xr[kk + 1u];
      }
      const uint32_t e = 0x7F800000u;
      bad |= (__float_as_uint(v0) & e) == e || (__float_as_uint(v1) & e) == e;
      const float t0 = v0 * gamma, t1 = v1 * gamma;
      const uint32_t hi = pack_bf16(t0, t1);
      const float d0 = t0 - __uint_as_float(hi << 16), d1 = t1 - __uint_as_float(hi & 0xFFFF0000u);  // exact
      hi_plane[r * pitch + kk / 2u] = hi;
      lo_plane[r * pitch + kk / 2u] = pack_bf16(d0, d1);
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
          const uint32_t f = (w[(k_begin + k) * NW + col / 16] >> shift) & 3u;
          if (f == 1u) sum += xr[k];
          else if (f == 3u) sum -= xr[k];
        }
        dst[static_cast<size_t>(r) * N + tid] = sum * gamma;
      }
    }
    return;
  }

  // ---- multiply
  floatx4 acc[kTOps];
  floatx4 off = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < kTOps; ++j) acc[j] = floatx4{0.f, 0.f, 0.f, 0.f};
  const bf16x8 minus6 = __builtin_bit_cast(bf16x8, vuint4{0xC0C0C0C0u, 0xC0C0C0C0u, 0xC0C0C0C0u, 0xC0C0C0C0u});
#pragma unroll
  for (int s = 0; s < kTMaxSteps; ++s) {
    if (s < steps) {  // (wave-uniform)
      const uint32_t kl = (kw0 + static_cast<uint32_t>(s) * kTStep + 8u * kg) / 2u;   // word of the lane's first pair
      const vuint4 ah = *reinterpret_cast<const vuint4*>(hi_plane + c * pitch + kl);
      const vuint4 al = *reinterpret_cast<const vuint4*>(lo_plane + c * pitch + kl);
      const bf16x8 a_hi = __builtin_bit_cast(bf16x8, ah), a_lo = __builtin_bit_cast(bf16x8, al);
      off = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi, minus6, off, 0, 0, 0);
      off = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_lo, minus6, off, 0, 0, 0);
#pragma unroll
      for (int q = 0; q < 4; ++q) {  // word q / 2 of the lane, its fields 8 (q % 2) .. + 7
        // rows (2 i, 2 i + 1) side by side, 16 bits each, every field as f ^ 2
        uint32_t z[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t wa = q < 2 ? wd[s][2 * i].x : wd[s][2 * i].y, wb = q < 2 ? wd[s][2 * i + 1].x : wd[s][2 * i + 1].y;
          z[i] = __builtin_amdgcn_perm(wb, wa, (q & 1) ? 0x07060302u : 0x05040100u) ^ 0xAAAAAAAAu;
        }
#pragma unroll
        for (int f = 0; f < 8; ++f) {
          uint32_t b[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            // field f of the low half to bits 5..6, of the high half to bits 21..22
            const int sh = 5 - 2 * f;
            const uint32_t t = sh >= 0 ? z[i] << (sh & 31) : z[i] >> ((-sh) & 31);
            b[i] = (t & 0x00600060u) | 0x40804080u;   // bf16 pair: 4 + (f ^ 2) of row 2 i, of row 2 i + 1
          }
          const bf16x8 bq = __builtin_bit_cast(bf16x8, vuint4{b[0], b[1], b[2], b[3]});
          const int j = 8 * q + f;
          acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi, bq, acc[j], 0, 0, 0);
          acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_lo, bq, acc[j], 0, 0, 0);
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < kTOps; ++j) acc[j] += off;   // every column of `off` holds -6 * sum of the row's activations

  // ---- the 8 waves as a tree: 4..7 onto 0..3, 2..3 onto 0..1, 1 onto 0. An image is the accumulators
  // as the lanes hold them (16 bytes per lane and operand: conflict-free both ways).
  __syncthreads();  // the activations are no longer needed
  vuint4* const images = reinterpret_cast<vuint4*>(smem);
#pragma unroll
  for (int span = 4; span >= 1; span >>= 1) {
    if (wave >= span && wave < 2 * span) {
      vuint4* img = images + static_cast<uint32_t>(wave - span) * (kTImage / 16) + lane;
#pragma unroll
      for (int j = 0; j < kTOps; ++j) img[j * kWave] = __builtin_bit_cast(vuint4, acc[j]);
    }
    __syncthreads();
    if (wave < span) {
      const vuint4* img = images + static_cast<uint32_t>(wave) * (kTImage / 16) + lane;
#pragma unroll
      for (int j = 0; j < kTOps; ++j) acc[j] += __builtin_bit_cast(floatx4, img[j * kWave]);
    }
    __syncthreads();
  }
  // ---- wave 0 lays the tile out row-major in LDS (element i of operand j: row 4 kg + i, column
  // 32 c + j; 4 spare floats per 32 columns keep the 16-byte writes of a quarter wave apart), then
  // every thread stores whole 16-byte pieces of output rows.
  float* const tile = reinterpret_cast<float*>(smem);
  if (wave == 0) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j4 = 0; j4 < kTOps / 4; ++j4)
        *reinterpret_cast<vfloat4*>(tile + (4 * kg + i) * kTOutPitch + 36 * c + 4 * j4) =
            vfloat4{acc[4 * j4][i], acc[4 * j4 + 1][i], acc[4 * j4 + 2][i], acc[4 * j4 + 3][i]};
  }
  __syncthreads();
  for (uint32_t idx = static_cast<uint32_t>(tid); idx < rows * (kTCols / 4); idx += kTThreads) {
    const uint32_t r = idx / (kTCols / 4), c4 = (idx % (kTCols / 4)) * 4u;
    if (col0 + c4 < N)   // (N is a multiple of 32: a piece of 4 columns is in or out as a whole)
      *reinterpret_cast<vfloat4*>(dst + static_cast<size_t>(r) * N + c4) =
          *reinterpret_cast<const vfloat4*>(tile + r * kTOutPitch + 36 * (c4 / 32) + c4 % 32);
  }
}

struct TernaryPlan {
  unsigned tiles, row_tiles, slices;
  uint32_t rows_per_wave;
};

// About one workgroup per CU of the 256-CU part; a wave takes 1 to 4 steps of 32 rows.
TernaryPlan ternary_plan(size_t m, size_t k, size_t n) {
  TernaryPlan p;
  p.tiles = static_cast<unsigned>((n + kTCols - 1) / kTCols);
  p.row_tiles = static_cast<unsigned>((m + kTRows - 1) / kTRows);
  const size_t columns = static_cast<size_t>(p.tiles) * p.row_tiles;
  const size_t want = std::max<size_t>(1, (256 + columns / 2) / columns);
  size_t rpw = ((k + want * kTWaves - 1) / (want * kTWaves) + kTStep - 1) / kTStep * kTStep;
  rpw = std::min<size_t>(std::max<size_t>(rpw, kTStep), kTMaxSteps * kTStep);
  p.rows_per_wave = static_cast<uint32_t>(rpw);
  p.slices = static_cast<unsigned>((k + rpw * kTWaves - 1) / (rpw * kTWaves));
  return p;
}

}  // namespace

// Rows of whole pairs of packed words (a lane loads 8 bytes), operands within 32-bit buffer offsets
// and launch limits.
bool ternary_mfma_ok(size_t m, size_t k, size_t n) {
  if (m == 0 || k == 0 || n == 0 || n % 32 != 0 || k * (n / 16) * 4 >= 0x7FFFFFFFull) return false;
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
  BQ_TRY(configure_dynamic_lds(reinterpret_cast<const void*>(qternary_kernel), kTLds, "qternary_kernel"));
  dim3 grid(p.tiles, p.slices, p.row_tiles), tb(kTThreads);
  hipLaunchKernelGGL(qternary_kernel, grid, tb, kTLds, st, x, w, scale, m, k, n, p.rows_per_wave, part);
  BQ_HIP(hipGetLastError());
  *slices_out = p.slices;
  return BQ_OK;
}

}  // namespace bq
