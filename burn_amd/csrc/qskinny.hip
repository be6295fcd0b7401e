// Small-batch q_matmul for gfx950 (2 <= M <= 32): out[M,N] = X[M,K] x dequantize(W[K,N]).
//
// Same operation as the decode GEMV and the prefill GEMM
// (QTensorOps::q_matmul, crates/burn-backend/src/backend/ops/qtensor.rs:498-544; reference path
// crates/burn-ndarray/src/ops/qtensor.rs:223-267), for the batch sizes in between: the weights
// are streamed once from HBM (that is the bound), but M fused multiply-adds per decoded weight
// are too many for the vector ALU, so the products go to the matrix cores.
//
// The product is computed transposed, out^T = W^T X^T, with v_mfma_f32_32x32x16_bf16:
//   * MFMA rows are 32 packed word columns. Field j of the 32 words of one k row belongs to the
//     output columns VPL * c + j, so field j of every word feeds accumulator j: a lane loads the
//     8 words W[k0 + 8 g .. + 7][c] (its own word column, 8 consecutive k), decodes them to
//     bf16(s * q), and the 8 values of field j are exactly its A operand of MFMA j. No
//     transpose, no LDS for the weights; every load instruction reads full 128-byte row segments.
//   * MFMA columns are the M (<= 32, zero padded) rows of X; the workgroup's K slice of X is
//     rounded to bf16 once and kept in LDS in operand order.
//   * The 4 waves of a workgroup split the K slice; they are summed through LDS in a fixed
//     order, and the slices are summed by qgemv_reduce_kernel in a fixed order (no float
//     atomics: results are reproducible run to run).
#include <algorithm>

#include "common.hpp"
#include "device_math.hpp"

namespace bq {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx2 __attribute__((ext_vector_type(2)));

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / kWave;
constexpr int kTileWords = 32;  // word columns per workgroup = MFMA rows
constexpr int kStepK = 16;      // k per MFMA

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2{lo, hi}, bf16x2));
}

template <int VPL, bool X_BF16>
__global__ void __launch_bounds__(kThreads)
qskinny_kernel(const void* __restrict__ x, const uint32_t* __restrict__ w,
               const float* __restrict__ scales, size_t M, size_t K, size_t N, size_t NW,
               unsigned block_words_log2, size_t scales_per_row, bool per_tensor, size_t k_per_wg,
               float* __restrict__ part) {
  constexpr int BITS = 32 / VPL;
  constexpr float BIAS = (BITS == 8) ? 128.0f : 8.0f;
  constexpr uint32_t FLIP = (BITS == 8) ? 0x80808080u : 0x88888888u;
  constexpr int RED_STRIDE = kTileWords * VPL + 1;  // floats; odd, so a column of rows spreads over banks

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  vuint4* const xs = reinterpret_cast<vuint4*>(smem);  // [k chunk of 8][32 rows of X][8 bf16]
  float* const red = reinterpret_cast<float*>(smem);    // reused after the main loop: [32][RED_STRIDE]

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int c = lane & 31, g = lane >> 5;
  const size_t wc0 = static_cast<size_t>(blockIdx.x) * kTileWords;
  const size_t k_begin = static_cast<size_t>(blockIdx.y) * k_per_wg;

  // ---- the K slice of X, as bf16, in MFMA operand order (rows >= M and k >= K are zero)
  const size_t chunks = k_per_wg / 8;
  // (in batches of 4 chunks per thread, all loads of a batch issued before the first store: one
  // load-wait-store per chunk would put a memory latency on every chunk)
  for (size_t base = 0; base < chunks * 32; base += 4 * kThreads) {
    vuint4 lo[4], hi[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const size_t idx = base + u * kThreads + tid;
      const size_t kc = idx >> 5, m = idx & 31;
      const size_t k = k_begin + kc * 8;
      lo[u] = hi[u] = vuint4{0u, 0u, 0u, 0u};
      if (idx < chunks * 32 && m < M && k < K) {  // K is a multiple of 8: a chunk is inside or outside as a whole
        if (X_BF16) {
          lo[u] = *reinterpret_cast<const vuint4*>(static_cast<const uint16_t*>(x) + m * K + k);
        } else {
          lo[u] = *reinterpret_cast<const vuint4*>(static_cast<const float*>(x) + m * K + k);
          hi[u] = *reinterpret_cast<const vuint4*>(static_cast<const float*>(x) + m * K + k + 4);
        }
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const size_t idx = base + u * kThreads + tid;
      if (idx >= chunks * 32) continue;
      vuint4 v = lo[u];
      if (!X_BF16) {
        const vfloat4 a = __builtin_bit_cast(vfloat4, lo[u]), b = __builtin_bit_cast(vfloat4, hi[u]);
        v = vuint4{pack_bf16(a.x, a.y), pack_bf16(a.z, a.w), pack_bf16(b.x, b.y), pack_bf16(b.z, b.w)};
      }
      xs[idx] = v;
    }
  }
  __syncthreads();

  // ---- this wave's quarter of the slice
  const size_t k_per_wave = k_per_wg / kWaves;  // multiple of 16
  const size_t kw = k_begin + static_cast<size_t>(wave) * k_per_wave;
  const int steps = static_cast<int>(k_per_wave / kStepK);
  size_t wc = wc0 + c;
  if (wc >= NW) wc = NW - 1;  // N tail: re-read the last word column, its outputs are not stored
  const size_t sc = per_tensor ? 0 : (wc >> block_words_log2);
  const size_t k_last = K - 1;

  floatx16 acc[VPL];
#pragma unroll
  for (int j = 0; j < VPL; ++j)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[j][e] = 0.f;

  uint32_t words[2][8];
  float scl[2][8];
  auto load_step = [&](int buf, int s) {
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      size_t row = kw + static_cast<size_t>(s) * kStepK + 8 * g + r;
      row = row < k_last ? row : k_last;  // past K: any valid row, X is zero there
      words[buf][r] = __builtin_nontemporal_load(w + row * NW + wc);
      scl[buf][r] = per_tensor ? scales[0] : scales[row * scales_per_row + sc];
    }
  };
  auto compute_step = [&](int buf, int s) {
    // B operand: X[m = lane % 32][k = kstep + 8 g .. + 7]
    const size_t kc = (kw - k_begin) / 8 + static_cast<size_t>(s) * 2 + g;
    const bf16x8 xb = __builtin_bit_cast(bf16x8, xs[kc * 32 + c]);
    // Unsigned fields u = q + BIAS of (word ^ FLIP): s*q = s*u - BIAS*s, one fma (BIAS*s is
    // exact), rounded once to bf16.
    float v[8][VPL];
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const float s_ = valid_scale(scl[buf][r]);
      const float nb = -BIAS * s_;
      const uint32_t word = words[buf][r] ^ FLIP;
      if (BITS == 8) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          v[r][j] = __builtin_fmaf(static_cast<float>((word >> (8 * j)) & 0xFFu), s_, nb);
      } else {
        uint32_t even = word & 0x0F0F0F0Fu, odd = (word >> 4) & 0x0F0F0F0Fu;
        asm("" : "+v"(even));  // keep the nibble spread: each spread word feeds four v_cvt_f32_ubyteN
        asm("" : "+v"(odd));
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          v[r][2 * j] = __builtin_fmaf(static_cast<float>((even >> (8 * j)) & 0xFFu), s_, nb);
          v[r][2 * j + 1] = __builtin_fmaf(static_cast<float>((odd >> (8 * j)) & 0xFFu), s_, nb);
        }
      }
    }
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      const vuint4 a = {pack_bf16(v[0][j], v[1][j]), pack_bf16(v[2][j], v[3][j]),
                        pack_bf16(v[4][j], v[5][j]), pack_bf16(v[6][j], v[7][j])};
      acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), xb, acc[j], 0, 0, 0);
    }
  };

  // (scheduling barriers keep each step's loads ahead of the other step's arithmetic)
  if (steps > 0) load_step(0, 0);
  for (int s = 0; s < steps; s += 2) {
    if (s + 1 < steps) load_step(1, s + 1);
    __builtin_amdgcn_sched_barrier(0);
    compute_step(0, s);
    __builtin_amdgcn_sched_barrier(0);
    if (s + 2 < steps) load_step(0, s + 2);
    __builtin_amdgcn_sched_barrier(0);
    if (s + 1 < steps) compute_step(1, s + 1);
    __builtin_amdgcn_sched_barrier(0);
  }

  // ---- sum the 4 waves in a fixed order (X is no longer needed: its LDS is reused).
  // Element e of an accumulator is word column 8 * (e / 4) + 4 * g + e % 4, X row lane % 32.
  __syncthreads();
  for (int turn = 0; turn < kWaves; ++turn) {
    if (wave == turn && static_cast<size_t>(c) < M) {
#pragma unroll
      for (int j = 0; j < VPL; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int col = 8 * (e / 4) + 4 * g + (e % 4);
          float* cell = red + c * RED_STRIDE + col * VPL + j;
          *cell = turn == 0 ? acc[j][e] : *cell + acc[j][e];
        }
    }
    __syncthreads();
  }
  const size_t n0 = wc0 * VPL;
  float* dst = part + static_cast<size_t>(blockIdx.y) * M * N;
  for (size_t idx = tid; idx < M * (kTileWords * VPL); idx += kThreads) {
    const size_t m = idx / (kTileWords * VPL), nl = idx % (kTileWords * VPL);
    if (n0 + nl < N) dst[m * N + n0 + nl] = red[m * RED_STRIDE + nl];
  }
}

// ---- f32 activations, 2 <= M <= 16: the same transposed product on the FP32 matrix pipe --------
// v_mfma_f32_16x16x4_f32 takes one f32 of each operand per lane. Lane (c = lane % 16,
// kq = lane / 16) loads the four consecutive words W[k0 + kq][4c .. 4c + 3] (16 bytes: a wave
// reads 256 contiguous bytes of each of 4 rows per instruction; narrower row segments leave HBM
// at a third of its rate). Word t of every lane forms MFMA row tile t (word columns 4i + t), and
// field j of it, dequantized in f32 (s * q exactly as the reference computes it), is the lane's
// A value of MFMA (t, j); its B value is X[m = c][k0 + kq] from the workgroup's slice of X in
// LDS. Products and sums are f32, so the result matches an f32 sgemm to accumulation order. The
// FP32 matrix rate (4 * VPL MFMAs of 32 cycles per KiB of weights per wave) is about the HBM
// rate for Q8S. The 4 waves of a workgroup take consecutive quarters of its K slice and are
// summed through LDS in a fixed order.
typedef float floatx4 __attribute__((ext_vector_type(4)));
constexpr int kF32Batch = 8;    // k-steps (of 4 rows) whose loads are issued together
constexpr int kF32Words = 64;   // word columns per workgroup

template <int VPL>
__global__ void __launch_bounds__(kThreads)
qskinny_f32_kernel(const float* __restrict__ x, const uint32_t* __restrict__ w,
                   const float* __restrict__ scales, size_t M, size_t K, size_t N, size_t NW,
                   unsigned block_words_log2, size_t scales_per_row, bool per_tensor, size_t k_per_wg,
                   float* __restrict__ part) {
  constexpr int BITS = 32 / VPL;
  constexpr float BIAS = (BITS == 8) ? 128.0f : 8.0f;
  constexpr uint32_t FLIP = (BITS == 8) ? 0x80808080u : 0x88888888u;
  constexpr int RED_STRIDE = kF32Words * VPL + 1;  // floats per X row in the reduction buffer
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  // X slice as [16 rows][k_per_wg + 4]: the row pitch is 4 mod 32 banks, so both the coalesced
  // fill (a lane per k) and the operand reads (16 rows x 4 k per instruction) are conflict-free.
  // The same memory is the cross-wave reduction buffer afterwards.
  float* const xs = reinterpret_cast<float*>(smem);
  float* const red = reinterpret_cast<float*>(smem);
  const size_t xpitch = k_per_wg + 4;

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int c = lane & 15, kq = lane >> 4;
  const size_t wc0 = static_cast<size_t>(blockIdx.x) * kF32Words;
  const size_t k_begin = static_cast<size_t>(blockIdx.y) * k_per_wg;

  size_t wc = wc0 + 4 * c;
  if (wc >= NW) wc = NW - 4;  // N tail (NW is a multiple of 4): re-read the last group, not stored
  const size_t sc = per_tensor ? 0 : (wc >> block_words_log2);  // one block holds the 4 words
  const float s_tensor = per_tensor ? valid_scale(scales[0]) : 0.0f;
  // Buffer loads: a per-lane byte offset (row kq of the step, own word group) plus a scalar
  // offset per step, so that no per-lane address arithmetic is left in the loop. The scalar
  // part is not range-checked: steps past the end of K re-read the last four rows (and multiply
  // only what is theirs of them, see multiply).
  const __amdgpu_buffer_rsrc_t rsrc_w =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(w), 0, static_cast<int>(K * NW * 4), 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_s = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(scales), 0, static_cast<int>(per_tensor ? 4 : K * scales_per_row * 4), 0x00020000);
  const uint32_t w_lane = static_cast<uint32_t>((kq * NW + wc) * 4);
  const uint32_t s_lane = per_tensor ? 0u : static_cast<uint32_t>((kq * scales_per_row + sc) * 4);
  const uint32_t w_row_bytes = static_cast<uint32_t>(NW * 4);
  const uint32_t s_row_bytes = per_tensor ? 0u : static_cast<uint32_t>(scales_per_row * 4);
  const uint32_t row_cap = static_cast<uint32_t>(K - 4);

  floatx4 acc[4][VPL];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int j = 0; j < VPL; ++j) acc[t][j] = floatx4{0.f, 0.f, 0.f, 0.f};

  // this wave's quarter of the slice, in batches of kF32Batch steps: the loads of one batch are
  // all in flight while the other is multiplied. k_per_wg is a multiple of 4 waves x 4 rows x batch.
  const size_t k_per_wave = k_per_wg / kWaves;
  const uint32_t kw = static_cast<uint32_t>(k_begin + wave * k_per_wave);
  const int steps = static_cast<int>(k_per_wave / 4);
  vuint4 wq[2][kF32Batch];
  float sq[2][kF32Batch];
  auto fetch = [&](int buf, int s0) {
#pragma unroll
    for (int u = 0; u < kF32Batch; ++u) {
      uint32_t row = kw + static_cast<uint32_t>(s0 + u) * 4u;
      row = row < row_cap ? row : row_cap;
      wq[buf][u] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, w_lane, row * w_row_bytes, 0);
      sq[buf][u] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc_s, s_lane, row * s_row_bytes, 0));
    }
  };
  auto multiply = [&](int buf, int s0) {
#pragma unroll
    for (int u = 0; u < kF32Batch; ++u) {
      const float sv = per_tensor ? s_tensor : valid_scale(sq[buf][u]);
      const float nb = -BIAS * sv;  // s*q = s*u - BIAS*s with u = q + BIAS; BIAS*s is exact
      // The step's rows are r_eff .. r_eff + 3 (see fetch: a group that would pass the end of K is
      // moved back to the last four rows). Of those only the rows from the nominal start on are
      // this step's; the lanes of the others multiply by zero. (K % 4 != 0: the last group.)
      const uint32_t r_nom = kw + static_cast<uint32_t>(s0 + u) * 4u;
      const uint32_t r_eff = r_nom < row_cap ? r_nom : row_cap;
      const bool mine = r_eff + static_cast<uint32_t>(kq) >= r_nom;
      const float xb = mine ? xs[c * xpitch + (r_eff - static_cast<uint32_t>(k_begin) + static_cast<uint32_t>(kq))] : 0.0f;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const uint32_t word = wq[buf][u][t] ^ FLIP;
        if (BITS == 8) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float a = __builtin_fmaf(static_cast<float>((word >> (8 * j)) & 0xFFu), sv, nb);
            acc[t][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, xb, acc[t][j], 0, 0, 0);
          }
        } else {
          uint32_t even = word & 0x0F0F0F0Fu, odd = (word >> 4) & 0x0F0F0F0Fu;
          asm("" : "+v"(even));  // keep the nibble spread: each spread word feeds four v_cvt_f32_ubyteN
          asm("" : "+v"(odd));
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float a0 = __builtin_fmaf(static_cast<float>((even >> (8 * j)) & 0xFFu), sv, nb);
            const float a1 = __builtin_fmaf(static_cast<float>((odd >> (8 * j)) & 0xFFu), sv, nb);
            acc[t][2 * j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a0, xb, acc[t][2 * j], 0, 0, 0);
            acc[t][2 * j + 1] = __builtin_amdgcn_mfma_f32_16x16x4f32(a1, xb, acc[t][2 * j + 1], 0, 0, 0);
          }
        }
      }
    }
  };
  // (scheduling barriers: left alone, the compiler sinks a batch's loads below the MFMAs of the
  // other batch to save registers, which serialises load latency and compute)
  fetch(0, 0);  // both register sets are in flight while X is staged
  if (kF32Batch < steps) fetch(1, kF32Batch);
  __builtin_amdgcn_sched_barrier(0);
  // Fill: wave w takes rows w, w+4, w+8, w+12 of X; every load of the wave is issued before the
  // first LDS store (a load-wait-store per element would put a memory latency on each).
  if (K % 4 == 0) {
    constexpr int kMaxVec = 3;  // 16-byte loads per lane and row: k_per_wg <= 768
    vfloat4 v[4][kMaxVec];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t m = wave + 4 * i;
#pragma unroll
      for (int u = 0; u < kMaxVec; ++u) {
        const uint32_t kk = (u * kWave + lane) * 4;
        v[i][u] = vfloat4{0.f, 0.f, 0.f, 0.f};
        if (m < M && kk < k_per_wg && k_begin + kk < K)  // K % 4 == 0: a group is in or out as a whole
          v[i][u] = *reinterpret_cast<const vfloat4*>(x + static_cast<size_t>(m) * K + k_begin + kk);
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int u = 0; u < kMaxVec; ++u) {
        const uint32_t kk = (u * kWave + lane) * 4;
        if (kk < k_per_wg) *reinterpret_cast<vfloat4*>(xs + (wave + 4 * i) * xpitch + kk) = v[i][u];
      }
  } else {
    for (uint32_t m = wave; m < 16; m += kWaves) {
      const bool row_ok = m < M;
      const float* xr = x + static_cast<size_t>(row_ok ? m : 0) * K + k_begin;
      for (uint32_t kk0 = 0; kk0 < k_per_wg; kk0 += 8 * kWave) {
        float t8[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const uint32_t kk = kk0 + u * kWave + lane;
          t8[u] = (row_ok && kk < k_per_wg && k_begin + kk < K) ? xr[kk] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const uint32_t kk = kk0 + u * kWave + lane;
          if (kk < k_per_wg) xs[m * xpitch + kk] = t8[u];
        }
      }
    }
  }
  __syncthreads();

  for (int s0 = 0; s0 < steps; s0 += 2 * kF32Batch) {
    multiply(0, s0);
    __builtin_amdgcn_sched_barrier(0);
    if (s0 + 2 * kF32Batch < steps) fetch(0, s0 + 2 * kF32Batch);
    __builtin_amdgcn_sched_barrier(0);
    if (s0 + kF32Batch < steps) multiply(1, s0 + kF32Batch);
    __builtin_amdgcn_sched_barrier(0);
    if (s0 + 3 * kF32Batch < steps) fetch(1, s0 + 3 * kF32Batch);
    __builtin_amdgcn_sched_barrier(0);
  }

  // Sum the 4 waves in a fixed order (X is no longer needed: its LDS is reused). Element r of
  // accumulator (t, j): MFMA row 4 kq + r = word column 4 (4 kq + r) + t of the tile, X row c.
  __syncthreads();
  for (int turn = 0; turn < kWaves; ++turn) {
    if (wave == turn && static_cast<size_t>(c) < M) {
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int j = 0; j < VPL; ++j)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float* cell = red + c * RED_STRIDE + (4 * (4 * kq + r) + t) * VPL + j;
            *cell = turn == 0 ? acc[t][j][r] : *cell + acc[t][j][r];
          }
    }
    __syncthreads();
  }
  const size_t n0 = wc0 * VPL;
  float* dst = part + static_cast<size_t>(blockIdx.y) * M * N;
  for (size_t idx = tid; idx < M * (kF32Words * VPL); idx += kThreads) {
    const size_t m = idx / (kF32Words * VPL), nl = idx % (kF32Words * VPL);
    if (n0 + nl < N) dst[m * N + n0 + nl] = red[m * RED_STRIDE + nl];
  }
}

struct SkinnyPlan {
  unsigned tiles, slices;
  size_t k_per_wg;
};

// f32 kernel: 64 word columns per workgroup; K slices of a multiple of 4 waves x 4 rows x batch
SkinnyPlan skinny_f32_plan(size_t m, size_t k, size_t n, int value) {
  const size_t nw = n / static_cast<size_t>(num_quants(value));
  SkinnyPlan p;
  p.tiles = static_cast<unsigned>((nw + kF32Words - 1) / kF32Words);
  size_t want = std::max<size_t>(1, 1024 / p.tiles);
  want = std::min<size_t>(want, 8);  // keep the partials small beside the weights
  const size_t unit = kWaves * 4 * kF32Batch;
  size_t kpw = (k + want - 1) / want;
  kpw = (kpw + unit - 1) / unit * unit;
  kpw = std::min<size_t>(kpw, 768);  // the X slice (16 x kpw f32) in LDS; a multiple of `unit`
  p.k_per_wg = kpw;
  p.slices = static_cast<unsigned>((k + kpw - 1) / kpw);
  return p;
}

SkinnyPlan skinny_plan(size_t m, size_t k, size_t n, int value) {
  const size_t nw = n / static_cast<size_t>(num_quants(value));
  SkinnyPlan p;
  p.tiles = static_cast<unsigned>((nw + kTileWords - 1) / kTileWords);
  // about 4 workgroups per CU, but few enough slices that the partials stay small beside the weights
  size_t want = std::max<size_t>(1, 1024 / p.tiles);
  want = std::min<size_t>(want, m > 8 ? 4 : (m > 4 ? 8 : 16));
  size_t kpw = (k + want - 1) / want;
  kpw = (kpw + 63) / 64 * 64;                 // 4 waves x whole MFMA k-steps
  kpw = std::min<size_t>(kpw, 1024);          // the X slice (32 x kpw bf16 = 64 B per k) must fit in LDS
  p.k_per_wg = kpw;
  p.slices = static_cast<unsigned>((k + kpw - 1) / kpw);
  return p;
}

}  // namespace

// f32 activations with M <= 16 take the FP32-matrix kernel (any K); bf16 activations, and f32
// ones with 16 < M <= 32, the bf16 one (K a multiple of 8, so that X rows load as 16-byte chunks).
static bool use_f32_kernel(size_t m, int x_dtype) { return x_dtype == BQ_F32 && m <= 16; }

bool skinny_ok(size_t m, size_t k, size_t n, int x_dtype, int value) {
  const size_t nw = n / static_cast<size_t>(num_quants(value));
  if (m < 2 || m > 32 || nw < 1 || k < 4) return false;
  if (use_f32_kernel(m, x_dtype))  // 16-byte word groups, 32-bit buffer offsets
    return nw % 4 == 0 && k * nw * 4 < 0x7FFFFFFFull;
  return k % 8 == 0 && k >= 64;
}

size_t skinny_workspace(size_t m, size_t k, size_t n, int x_dtype, int value) {
  const SkinnyPlan p = use_f32_kernel(m, x_dtype) ? skinny_f32_plan(m, k, n, value) : skinny_plan(m, k, n, value);
  return static_cast<size_t>(p.slices) * m * n * sizeof(float);
}

// Launches the small-batch kernel; `part` receives slices x [M, N] partial sums. Returns the
// number of slices through *slices_out (the caller runs the fixed-order reduction).
bq_status launch_qskinny(const void* x, int x_dtype, const uint32_t* w, const float* scales, size_t m, size_t k,
                         size_t n, int value, unsigned block_words_log2, size_t scales_per_row, bool per_tensor,
                         float* part, unsigned* slices_out, hipStream_t st) {
  const size_t nw = n / static_cast<size_t>(num_quants(value));
  const int vpl = num_quants(value);
  if (use_f32_kernel(m, x_dtype)) {
    const SkinnyPlan p = skinny_f32_plan(m, k, n, value);
    const size_t lds = std::max<size_t>((p.k_per_wg + 4) * 16, 16 * (kF32Words * vpl + 1)) * sizeof(float);
    dim3 grid(p.tiles, p.slices), tb(kThreads);
#define BQ_SKINNY_F32(V)                                                                             \
  do {                                                                                               \
    auto kernel = qskinny_f32_kernel<V>;                                                             \
    /* refused on the host when the device grants less; the largest slices need the opt-in */        \
    BQ_TRY(configure_dynamic_lds(reinterpret_cast<const void*>(kernel), lds, "qskinny_f32_kernel"));  \
    hipLaunchKernelGGL(kernel, grid, tb, lds, st, static_cast<const float*>(x), w, scales, m, k, n,  \
                       nw, block_words_log2, scales_per_row, per_tensor, p.k_per_wg, part);          \
  } while (0)
    if (value == BQ_Q8S) BQ_SKINNY_F32(4); else BQ_SKINNY_F32(8);
#undef BQ_SKINNY_F32
    BQ_HIP(hipGetLastError());
    *slices_out = p.slices;
    return BQ_OK;
  }
  const SkinnyPlan p = skinny_plan(m, k, n, value);
  const size_t lds = std::max<size_t>(p.k_per_wg / 8 * 32 * 16, 32 * (kTileWords * vpl + 1) * sizeof(float));
  dim3 grid(p.tiles, p.slices), tb(kThreads);
  const bool xb = x_dtype == BQ_BF16;
#define BQ_SKINNY(V, XB)                                                                           \
  do {                                                                                             \
    auto kernel = qskinny_kernel<V, XB>;                                                           \
    /* refused on the host when the device grants less; the largest slices need the opt-in */      \
    BQ_TRY(configure_dynamic_lds(reinterpret_cast<const void*>(kernel), lds, "qskinny_kernel"));    \
    hipLaunchKernelGGL(kernel, grid, tb, lds, st, x, w, scales, m, k, n, nw, block_words_log2,     \
                       scales_per_row, per_tensor, p.k_per_wg, part);                              \
  } while (0)
  if (value == BQ_Q8S) {
    if (xb) BQ_SKINNY(4, true); else BQ_SKINNY(4, false);
  } else {
    if (xb) BQ_SKINNY(8, true); else BQ_SKINNY(8, false);
  }
#undef BQ_SKINNY
  BQ_HIP(hipGetLastError());
  *slices_out = p.slices;
  return BQ_OK;
}

}  // namespace bq
