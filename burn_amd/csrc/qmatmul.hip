// q_matmul kernels for gfx950: out[M,N] = lhs[M,K] x dequantize(W[K,N]).
//
// W is the quantized rhs of QTensorOps::q_matmul (crates/burn-backend/src/backend/ops/qtensor.rs:498-544):
// row-major [K, N], values packed along N (4 x i8 or 8 x i4 per u32, low field first), one f32
// scale per tensor or per run of `block` values along N (scales[k][n / block]). The reference
// (crates/burn-ndarray/src/ops/qtensor.rs:223-267) materialises dequantize(W) and calls an sgemm;
// here the dequantize is fused into the operand path:
//   * decode (f32 lhs: M <= 2 on 8-bit weights, M = 1 on 4-bit ones, one row more when the scales
//     are per 64 or 128 columns; bf16 lhs: M <= 2): a q-GEMV that unpacks in registers, split
//     over K; HBM bound.
//   * from there up to M = 32: the split-activation kernel of qsplit.hip (bf16 matrix cores, exact
//     integer weights, activations x scale as two bf16 terms); the weight layouts it does not take
//     fall back to the decode kernel (M <= 8), the kernels of qskinny.hip, or the general q-GEMV
//     below.
//   * prefill: packed words + scales -> registers -> bf16 in LDS -> v_mfma_f32_32x32x16_bf16,
//     f32 accumulation (qgemm.hip).
// Also here: the fixed-order reduction of the K slices, the f32 matrix-core GEMM of the general
// path (operands that are dequantized first), the multiply-free product of ternary weights, and
// the allocation-free entry point. Full-range values (Q8F, Q4F) are two's complement fields like
// their symmetric twins and take the same kernels.
#include <algorithm>

#include <type_traits>

#include "common.hpp"
#include "device_math.hpp"
#include "splitk_tail.hpp"

namespace bq {

namespace {

// ================================================================================ q-GEMV
constexpr int kGemvThreads = 256;
constexpr int kGemvWaves = kGemvThreads / kWave;

// One lane owns one packed word column (VPL output columns); the 4 waves of a workgroup take
// interleaved rows of the workgroup's K slice and are summed through LDS. Partials go to
// part[slice][m][n]; qgemv_reduce_kernel sums the slices in a fixed order (no float atomics, so
// results are reproducible run to run).
template <int VPL, int M>
__global__ void __launch_bounds__(kGemvThreads)
qgemv_kernel(const float* __restrict__ x, const uint32_t* __restrict__ w,
             const float* __restrict__ scales, size_t K, size_t NW, unsigned block_words_log2,
             size_t scales_per_row, bool per_tensor, size_t rows_per_slice,
             float* __restrict__ part) {
  constexpr int BITS = 32 / VPL;
  constexpr float BIAS = (BITS == 8) ? 128.0f : 8.0f;
  constexpr uint32_t FLIP = (BITS == 8) ? 0x80808080u : 0x88888888u;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const size_t col = static_cast<size_t>(blockIdx.x) * kWave + lane;  // word column
  const bool active = col < NW;
  const size_t k_begin = static_cast<size_t>(blockIdx.y) * rows_per_slice;
  size_t k_end = k_begin + rows_per_slice;
  if (k_end > K) k_end = K;

  float acc[M][VPL];
#pragma unroll
  for (int m = 0; m < M; ++m)
#pragma unroll
    for (int j = 0; j < VPL; ++j) acc[m][j] = 0.0f;

  const size_t scol = per_tensor ? 0 : (col >> block_words_log2);
  const float s_tensor = per_tensor ? valid_scale(scales[0]) : 0.0f;

  if (active) {
#pragma unroll 4
    for (size_t k = k_begin + wave; k < k_end; k += kGemvWaves) {
      const uint32_t word = __builtin_nontemporal_load(w + k * NW + col) ^ FLIP;
      const float s = per_tensor ? s_tensor : valid_scale(scales[k * scales_per_row + scol]);
      // unsigned fields u = q + BIAS: s*q = s*u - BIAS*s, and BIAS*s is exact (power of two)
      const float neg_bias_s = -BIAS * s;
      float wv[VPL];
      if (BITS == 8) {
#pragma unroll
        for (int j = 0; j < VPL; ++j)
          wv[j] = __builtin_fmaf(static_cast<float>((word >> (8 * j)) & 0xFFu), s, neg_bias_s);
      } else {
#pragma unroll
        for (int j = 0; j < VPL; ++j)
          wv[j] = __builtin_fmaf(static_cast<float>((word >> (4 * j)) & 0xFu), s, neg_bias_s);
      }
#pragma unroll
      for (int m = 0; m < M; ++m) {
        const float xv = x[static_cast<size_t>(m) * K + k];  // wave-uniform
#pragma unroll
        for (int j = 0; j < VPL; ++j) acc[m][j] = __builtin_fmaf(xv, wv[j], acc[m][j]);
      }
    }
  }

  // sum the 4 waves in a fixed order through LDS; wave 0 ends up with the slice partial
  __shared__ float red[M * VPL][kWave];
  for (int ww = 1; ww < kGemvWaves; ++ww) {
    if (wave == ww) {
#pragma unroll
      for (int m = 0; m < M; ++m)
#pragma unroll
        for (int j = 0; j < VPL; ++j) red[m * VPL + j][lane] = acc[m][j];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
      for (int m = 0; m < M; ++m)
#pragma unroll
        for (int j = 0; j < VPL; ++j) acc[m][j] += red[m * VPL + j][lane];
    }
    __syncthreads();
  }
  if (wave == 0 && active) {
    const size_t N = NW * VPL;
    float* dst = part + static_cast<size_t>(blockIdx.y) * M * N;
#pragma unroll
    for (int m = 0; m < M; ++m) {
      float r[VPL];
#pragma unroll
      for (int j = 0; j < VPL; ++j) r[j] = acc[m][j];
      vfloat4* p = reinterpret_cast<vfloat4*>(dst + static_cast<size_t>(m) * N + col * VPL);
#pragma unroll
      for (int i = 0; i < VPL / 4; ++i) {
        vfloat4 t = {r[4 * i], r[4 * i + 1], r[4 * i + 2], r[4 * i + 3]};
        p[i] = t;
      }
    }
  }
}

// ---- decode, a few activation rows (M <= 8) ----------------------------------------------------
// A lane owns 16 consecutive columns (16 bytes of Q8S, 8 bytes of Q4S), a wave 1024: it streams
// whole 1 KiB / 512-byte runs of a weight row, the waves of a workgroup on consecutive rows, a
// few rows in flight per wave, about one workgroup per CU. The unsigned fields u = q + BIAS go through
// v_cvt_f32_ubyte (once per weight, whatever M); sum_k xs*q = sum_k xs*u - BIAS * sum_k xs with
// xs = x[m][k] * s[k][n/block], the second sum kept per lane and row (a lane's columns share one
// scale). Vector-ALU work grows with M (one fma per weight and row): it stays below the memory
// time up to M = 3 or 4 and takes over from there.
constexpr int gemv1_words(int vpl) { return vpl == 4 ? 4 : 2; }  // packed words per lane and row: 16 columns
constexpr int gemv1_max_m(int vpl) { return vpl == 4 ? 8 : 4; }  // accumulators: M x 16 registers
// bf16 activations take this kernel for one or two rows (decode); from three rows on the
// split-activation MFMA kernel is as fast (measured on the 4096 x 14336 weight, Q8S / Q4S:
// M = 1 21.8 / 20.2 us there)
constexpr size_t kGemv1MaxMBf16 = 2;
// waves per workgroup: the cross-wave sum goes through WAVES * 16 * 64 floats of LDS, and 16
// waves leave 128 registers per lane
constexpr int gemv1_waves(int vpl, int m) { return m <= 4 ? 16 : 8; }
// rows per wave and loop trip (twice that in flight); Q4S rows are half as long, so more of them
constexpr int gemv1_unroll(int vpl, int m) { return (vpl == 8 && m <= 2) ? 4 : 2; }

template <int VPL>
__device__ __forceinline__ void gemv1_fields(uint32_t word, float* f) {
  if (VPL == 4) {
    const uint32_t u = word ^ 0x80808080u;
#pragma unroll
    for (int j = 0; j < 4; ++j) f[j] = static_cast<float>((u >> (8 * j)) & 0xFFu);
  } else {
    const uint32_t u = word ^ 0x88888888u;
    const uint32_t even = u & 0x0F0F0F0Fu, odd = (u >> 4) & 0x0F0F0F0Fu;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f[2 * j] = static_cast<float>((even >> (8 * j)) & 0xFFu);
      f[2 * j + 1] = static_cast<float>((odd >> (8 * j)) & 0xFFu);
    }
  }
}

// X_BF16: the activations are bf16 (instantiated for M <= 2). Their index is wave-uniform, so the
// aligned 32-bit word holding the element is a scalar load and the half is picked with scalar
// ALU; widened exactly to f32, everything after is the f32 kernel.
template <int VPL, bool PER_TENSOR, int M, bool X_BF16 = false>
__global__ void __launch_bounds__(gemv1_waves(VPL, M) * kWave)
qgemv1_kernel(const void* __restrict__ x, const uint32_t* __restrict__ w,
              const float* __restrict__ scales, size_t K, size_t NQ, unsigned scale_shift,
              size_t scales_per_row, size_t rows_per_wg, float* __restrict__ part,
              unsigned* __restrict__ tickets, const float* __restrict__ bias, int out_bf16, void* __restrict__ out) {
  constexpr int WPL = gemv1_words(VPL);
  constexpr int CPL = WPL * VPL;  // columns per lane: 16
  typedef uint32_t LoadT __attribute__((ext_vector_type(WPL)));  // one 16- or 8-byte load
  constexpr float BIAS = (VPL == 4) ? 128.0f : 8.0f;
  constexpr int U = gemv1_unroll(VPL, M);
  constexpr int WAVES = gemv1_waves(VPL, M);
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const size_t col = static_cast<size_t>(blockIdx.x) * kWave + lane;  // in units of one load
  const bool active = col < NQ;
  const size_t k_begin = static_cast<size_t>(blockIdx.y) * rows_per_wg;
  size_t k_end = k_begin + rows_per_wg;
  if (k_end > K) k_end = K;
  const float s_tensor = PER_TENSOR ? valid_scale(scales[0]) : 0.0f;
  const size_t scol = PER_TENSOR ? 0 : (col >> scale_shift);

  float acc[M][CPL];
  float corr[M];
#pragma unroll
  for (int m = 0; m < M; ++m) {
    corr[m] = 0.0f;
#pragma unroll
    for (int j = 0; j < CPL; ++j) acc[m][j] = 0.0f;
  }

  // rows of this wave: k_begin + wave + WAVES * i (wave-uniform, so x[m][k] is a scalar load).
  // The loads of the next U rows are issued before the current ones are multiplied.
  auto fetch = [&](size_t k, LoadT& q, float& s) {
    if (active && k < k_end) {
      q = __builtin_nontemporal_load(reinterpret_cast<const LoadT*>(w) + k * NQ + col);
      s = PER_TENSOR ? s_tensor : scales[k * scales_per_row + scol];
    } else {
#pragma unroll
      for (int i = 0; i < WPL; ++i) q[i] = 0u;
      s = 0.0f;
    }
  };
  // An infinity or a NaN among this workgroup's activations (rows_per_wg x M of them, read once
  // here, ahead of the weight loads) sends the whole workgroup through the guarded copy of the
  // loop: xs * u - BIAS * xs would be inf - inf there, and a padded row's x[k_begin] * 0 would be
  // NaN. Finite slices run the plain copy and pay one small load and a barrier for the test.
  int bad = 0;
  {
    const size_t rows = k_end > k_begin ? k_end - k_begin : 0;
    for (size_t i = threadIdx.x; i < rows * M; i += static_cast<size_t>(WAVES) * kWave) {
      const size_t e = (i / rows) * K + k_begin + i % rows;
      const uint32_t bits = X_BF16 ? static_cast<uint32_t>(static_cast<const uint16_t*>(x)[e]) << 16
                                   : static_cast<const uint32_t*>(x)[e];
      bad |= (bits & 0x7F800000u) == 0x7F800000u;
    }
  }
  LoadT q[U], qn[U];
  float sc[U], sn[U];
  size_t kb = k_begin + static_cast<size_t>(wave);
#pragma unroll
  for (int u = 0; u < U; ++u) fetch(kb + static_cast<size_t>(u) * WAVES, q[u], sc[u]);
  const bool nonfinite = __syncthreads_or(bad) != 0;
  auto run = [&](auto G) {
    constexpr bool guard = decltype(G)::value;
    while (kb < k_end) {
      const size_t kn = kb + static_cast<size_t>(WAVES) * U;
#pragma unroll
      for (int u = 0; u < U; ++u) fetch(kn + static_cast<size_t>(u) * WAVES, qn[u], sn[u]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const size_t k = kb + static_cast<size_t>(u) * WAVES;
        const size_t kx = k < k_end ? k : k_begin;  // rows past the slice: s is 0 there
        const float sv = (PER_TENSOR || !(active && k < k_end)) ? sc[u] : valid_scale(sc[u]);
        float xs[M];
#pragma unroll
        for (int m = 0; m < M; ++m) {
          const size_t e = static_cast<size_t>(m) * K + kx;
          float xe;
          if (X_BF16) {
            const uint32_t pair = static_cast<const uint32_t*>(x)[e >> 1];
            xe = __builtin_bit_cast(float, (e & 1) ? (pair & 0xFFFF0000u) : (pair << 16));
          } else {
            xe = static_cast<const float*>(x)[e];
          }
          if (guard) xe = k < k_end ? xe : 0.0f;
          xs[m] = xe * sv;
          if (!guard) corr[m] += xs[m];
        }
#pragma unroll
        for (int i = 0; i < WPL; ++i) {
          float f[VPL];
          gemv1_fields<VPL>(q[u][i], f);
#pragma unroll
          for (int m = 0; m < M; ++m)
#pragma unroll
            for (int j = 0; j < VPL; ++j)
              acc[m][i * VPL + j] = __builtin_fmaf(xs[m], guard ? f[j] - BIAS : f[j], acc[m][i * VPL + j]);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        q[u] = qn[u];
        sc[u] = sn[u];
      }
      kb = kn;
    }
  };
  if (!nonfinite) run(std::false_type{}); else run(std::true_type{});
  // Sum the waves in a fixed order through LDS, one activation row at a time. Every wave stores
  // its CPL x 64 partials; then each thread adds up, over the waves, the outputs t, t + THREADS,
  // ... of the workgroup's CPL * 64 consecutive columns, so the stores to `part` are contiguous.
  // Partial (j, lane) lives at j * 64 + (lane + (64 / CPL) * j) % 64: a rotation per j, which keeps
  // both the stores (lane varies) and the loads (j varies fastest) free of bank conflicts.
  constexpr int ELEMS = CPL * kWave, THREADS = WAVES * kWave;
  __shared__ float red[WAVES][ELEMS];
  const size_t N = NQ * CPL;
  const size_t n_base = static_cast<size_t>(blockIdx.x) * ELEMS;
#pragma unroll
  for (int m = 0; m < M; ++m) {
    if (m > 0) __syncthreads();
#pragma unroll
    for (int j = 0; j < CPL; ++j)
      red[wave][j * kWave + ((lane + (kWave / CPL) * j) & (kWave - 1))] = __builtin_fmaf(-BIAS, corr[m], acc[m][j]);
    __syncthreads();
    float* dst = part + (static_cast<size_t>(blockIdx.y) * M + m) * N + n_base;
#pragma unroll
    for (int i = 0; i < ELEMS / THREADS; ++i) {
      const int o = static_cast<int>(threadIdx.x) + i * THREADS;
      const int src_lane = o / CPL, j = o % CPL;
      const int at = j * kWave + ((src_lane + (kWave / CPL) * j) & (kWave - 1));
      float v = red[0][at];
#pragma unroll
      for (int ww = 1; ww < WAVES; ++ww) v += red[ww][at];
      if (n_base + o < N) {
        // (one launch: the partials are read by another workgroup, possibly on another XCD)
        if (tickets != nullptr) __hip_atomic_store(dst + o, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        else dst[o] = v;
      }
    }
  }
  // tickets: the last workgroup to finish a column strip sums the K slices and writes the output
  if (tickets != nullptr)
    splitk_reduce_tail<THREADS>(part, tickets + static_cast<size_t>(blockIdx.x) * kTicketStride, gridDim.y, M, N, n_base,
                                static_cast<unsigned>(N - n_base < ELEMS ? N - n_base : ELEMS), bias, out_bf16 != 0, out);
}

// out[i] = sum over slices of part[s][i]. A workgroup owns 256 / SL float4 columns; its SL "slice
// lanes" each add every SL-th slice in ascending order, then lane 0 adds the SL subtotals in
// ascending order: a fixed summation tree, so results are reproducible run to run. SL is the
// largest of 16, 8, 4 that does not exceed the slice count (no idle slice lanes).
template <int SL>
__device__ __forceinline__ bool reduce_slices(const float* __restrict__ part, size_t mn, unsigned slices,
                                              const float* __restrict__ bias, size_t n, size_t& i_out, vfloat4& v_out) {
  constexpr int COLS = 256 / SL;
  __shared__ vfloat4 sub[SL][COLS];
  const int c = threadIdx.x % COLS, sl = threadIdx.x / COLS;
  const size_t i = (static_cast<size_t>(blockIdx.x) * COLS + c) * 4;
  const bool vec = (mn & 3) == 0;
  vfloat4 v = {0.f, 0.f, 0.f, 0.f};
  if (i < mn) {
    for (unsigned s = sl; s < slices; s += SL) {
      const float* p = part + static_cast<size_t>(s) * mn + i;
      if (vec) {
        v += *reinterpret_cast<const vfloat4*>(p);
      } else {
        v.x += p[0];
        if (i + 1 < mn) v.y += p[1];
        if (i + 2 < mn) v.z += p[2];
        if (i + 3 < mn) v.w += p[3];
      }
    }
  }
  sub[sl][c] = v;
  __syncthreads();
  const bool mine = sl == 0 && i < mn;
  if (mine) {
#pragma unroll
    for (int t = 1; t < SL; ++t) v += sub[t][c];
    if (bias != nullptr) {  // the linear layer's bias, added last: (sum of products) + bias[column]
      const size_t col = i % n;
      if (vec && (n & 3) == 0) {
        v += *reinterpret_cast<const vfloat4*>(bias + col);
      } else {
        v.x += bias[col];
        v.y += bias[(i + 1) % n];
        v.z += bias[(i + 2) % n];
        v.w += bias[(i + 3) % n];
      }
    }
  }
  i_out = i;
  v_out = v;
  return mine;  // this thread holds outputs i .. i + 3
}

template <bool BF16, int SL>
__global__ void __launch_bounds__(256)
qgemv_reduce_kernel(const float* __restrict__ part, size_t mn, unsigned slices, const float* __restrict__ bias,
                    size_t n, void* __restrict__ out) {
  size_t i;
  vfloat4 v;
  if (reduce_slices<SL>(part, mn, slices, bias, n, i, v)) {
    const bool vec = (mn & 3) == 0;
    const float r[4] = {v.x, v.y, v.z, v.w};
    if (vec && !BF16) {
      *reinterpret_cast<vfloat4*>(static_cast<float*>(out) + i) = v;
    } else {
      for (int e = 0; e < 4 && i + e < mn; ++e) {
        if (BF16)
          static_cast<uint16_t*>(out)[i + e] = f32_to_bf16(r[e]);
        else
          static_cast<float*>(out)[i + e] = r[e];
      }
    }
  }
}

// The same sum, quantized where it is formed (QuantPropagation::Propagate, crates/burn-ndarray/src/ops/
// qtensor.rs:262-265, for a block scheme). A block of 4 * LANES consecutive outputs -- 32 or 64 columns of one
// row, n being a multiple of it -- lies in LANES consecutive lanes: absmax across them by DPP, the scale
// (2 * absmax) / (b - a) rounded up to the scale dtype, each value divided by it, rounded half away from
// zero and clamped: the arithmetic of quantize_dynamic on the float product, which is never written.
// VPL = 4: a lane's four values are one word (or four native bytes). VPL = 8: a word is two lanes' values.
template <int SL, int VPL, int LANES>
__global__ void __launch_bounds__(256)
qgemv_reduce_quant_kernel(const float* __restrict__ part, size_t mn, unsigned slices, const float* __restrict__ bias,
                          size_t n, float qmin, float qmax, int sdt, int from_bf16, uint32_t* __restrict__ values,
                          float* __restrict__ scales) {
  size_t i;
  vfloat4 v;
  const bool mine = reduce_slices<SL>(part, mn, slices, bias, n, i, v);
  // (mn is a multiple of the block: the lanes of a block hold outputs together or not at all; the
  // cross-lane steps below run in every lane)
  float r[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    if (!mine) r[e] = 0.0f;
    if (from_bf16) r[e] = bf16_to_f32(f32_to_bf16(r[e]));
  }
  const float m = group_max<LANES>(fmaxf(fmaxf(fabsf(r[0]), fabsf(r[1])), fmaxf(fabsf(r[2]), fabsf(r[3]))));
  const float s_stored = scale_round_up(scale_from_absmax(m, qmax - qmin), sdt);
  const float s = valid_scale(s_stored);
  int q[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) q[e] = quantize_div(r[e], s, qmin, qmax);
  const int c = threadIdx.x % (256 / SL);
  if (VPL == 4) {
    if (mine) values[i / 4] = pack_fields<4>(q);
  } else {
    const uint32_t half = static_cast<uint32_t>(q[0] & 15) | static_cast<uint32_t>(q[1] & 15) << 4 |
                          static_cast<uint32_t>(q[2] & 15) << 8 | static_cast<uint32_t>(q[3] & 15) << 12;
    const uint32_t next = dpp_lane<0xB1>(half);  // quad_perm [1,0,3,2]: the odd neighbour's half for an even lane
    if (mine && (c & 1) == 0) values[i / 8] = half | next << 16;
  }
  if (mine && (c & (LANES - 1)) == 0) scales[i / (4 * LANES)] = s_stored;
}

struct GemvPlan {
  unsigned strips;
  unsigned slices;
  size_t rows_per_slice;
};

GemvPlan gemv_plan(size_t k, size_t n, int value) {
  const size_t nw = n / static_cast<size_t>(num_quants(value));
  GemvPlan p;
  p.strips = static_cast<unsigned>((nw + kWave - 1) / kWave);
  size_t want = 2048 / (p.strips ? p.strips : 1);
  if (want < 1) want = 1;
  size_t max_slices = (k + 15) / 16;
  if (want > max_slices) want = max_slices;
  if (want < 1) want = 1;
  p.rows_per_slice = (k + want - 1) / want;
  p.rows_per_slice = (p.rows_per_slice + kGemvWaves - 1) / kGemvWaves * kGemvWaves;
  p.slices = static_cast<unsigned>((k + p.rows_per_slice - 1) / p.rows_per_slice);
  if (p.slices < 1) p.slices = 1;
  return p;
}

// Decode kernel: strips of 64 lanes x 16 bytes; the K slices are sized for a few workgroups per
// CU, all resident at once.
GemvPlan gemv1_plan(size_t m, size_t k, size_t n, int value) {
  const size_t cpl = static_cast<size_t>(gemv1_words(num_quants(value)) * num_quants(value));
  const size_t nq = n / cpl;
  GemvPlan p;
  p.strips = static_cast<unsigned>((nq + kWave - 1) / kWave);
  const size_t target = 224;  // workgroups: just under one per CU measured best on the 256-CU part
  size_t want = (target + p.strips / 2) / (p.strips ? p.strips : 1);
  const size_t max_slices = (k + 15) / 16;
  if (want > max_slices) want = max_slices;
  if (want < 1) want = 1;
  const size_t waves = static_cast<size_t>(gemv1_waves(num_quants(value), static_cast<int>(m)));
  p.rows_per_slice = ((k + want - 1) / want + waves - 1) / waves * waves;
  p.slices = static_cast<unsigned>((k + p.rows_per_slice - 1) / p.rows_per_slice);
  if (p.slices < 1) p.slices = 1;
  return p;
}

// The decode kernel needs rows of whole 16-column groups and one scale per group.
bool gemv1_ok(size_t m, size_t n, int lhs_dtype, int block, int value) {
  const size_t cpl = static_cast<size_t>(gemv1_words(num_quants(value)) * num_quants(value));
  const bool dtype_ok = lhs_dtype == BQ_F32 || (lhs_dtype == BQ_BF16 && m <= kGemv1MaxMBf16);
  return m >= 1 && m <= static_cast<size_t>(gemv1_max_m(num_quants(value))) && dtype_ok && n % cpl == 0 &&
         (block == 0 || static_cast<size_t>(block) % cpl == 0);
}

// ================================================================================ float GEMM
// f32-accurate GEMM on the matrix cores (v_mfma_f32_32x32x2_f32: full f32 products and sums) for the
// combinations where no operand stays packed: quantized lhs x float rhs, rectangle blocks, ternary
// weights outside the fast path. Both operands are dequantized first, as the reference does. A
// workgroup of 4 waves (2 x 2) owns a (64 * WT)^2 tile, 16 deep; the next slab is loaded into
// registers while the current one is multiplied out of LDS. Any shape, f32 or bf16 operands,
// element-wise guarded loads: sized for correctness at a fair speed, not tuned to the limit.
__device__ __forceinline__ float load_elem(const void* p, int dtype, size_t i) {
  return dtype == BQ_BF16 ? bf16_to_f32(static_cast<const uint16_t*>(p)[i])
                          : static_cast<const float*>(p)[i];
}

template <int WT>
__global__ void __launch_bounds__(256)
float_matmul_kernel(const void* __restrict__ a, int a_dtype, const void* __restrict__ b,
                    int b_dtype, size_t M, size_t K, size_t N, int out_dtype,
                    void* __restrict__ out) {
  constexpr int T = 64 * WT, TK = 16, LD = T + 4, PER = T * TK / 256;
  typedef float vfloat16 __attribute__((ext_vector_type(16)));
  __shared__ float As[TK][LD];  // [k][row]: a wave's 32 rows of one k are consecutive words
  __shared__ float Bs[TK][LD];  // [k][column]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const size_t m0 = static_cast<size_t>(blockIdx.y) * T, n0 = static_cast<size_t>(blockIdx.x) * T;
  vfloat16 acc[WT][WT];
#pragma unroll
  for (int i = 0; i < WT; ++i)
#pragma unroll
    for (int j = 0; j < WT; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  float ra[PER], rb[PER];
  auto gload = [&](size_t kt) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int idx = tid + i * 256;
      const size_t gr = m0 + idx / TK, gk = kt + idx % TK;   // A: k fastest, as in memory
      ra[i] = (gr < M && gk < K) ? load_elem(a, a_dtype, gr * K + gk) : 0.0f;
      const size_t gk2 = kt + idx / T, gn = n0 + idx % T;    // B: column fastest
      rb[i] = (gk2 < K && gn < N) ? load_elem(b, b_dtype, gk2 * N + gn) : 0.0f;
    }
  };
  gload(0);
  for (size_t kt = 0; kt < K; kt += TK) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int idx = tid + i * 256;
      As[idx % TK][idx / TK] = ra[i];
      Bs[idx / T][idx % T] = rb[i];
    }
    __syncthreads();
    if (kt + TK < K) gload(kt + TK);
#pragma unroll
    for (int kk = 0; kk < TK; kk += 2) {
      // operands of one 32x32x2 step: lane l holds A[row l % 32][k l / 32] and B[k l / 32][column l % 32]
      const int k = kk + (lane >> 5);
      float av[WT], bv[WT];
#pragma unroll
      for (int i = 0; i < WT; ++i) av[i] = As[k][(wm * WT + i) * 32 + (lane & 31)];
#pragma unroll
      for (int j = 0; j < WT; ++j) bv[j] = Bs[k][(wn * WT + j) * 32 + (lane & 31)];
#pragma unroll
      for (int i = 0; i < WT; ++i)
#pragma unroll
        for (int j = 0; j < WT; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[i], bv[j], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
  }
  // accumulator element r of lane l: row 8 * (r / 4) + 4 * (l / 32) + r % 4, column l % 32
#pragma unroll
  for (int i = 0; i < WT; ++i)
#pragma unroll
    for (int j = 0; j < WT; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const size_t row = m0 + (wm * WT + i) * 32 + 8 * (r / 4) + 4 * (lane >> 5) + r % 4;
        const size_t col = n0 + (wn * WT + j) * 32 + (lane & 31);
        if (row < M && col < N) {
          if (out_dtype == BQ_BF16)
            static_cast<uint16_t*>(out)[row * N + col] = f32_to_bf16(acc[i][j][r]);
          else
            static_cast<float*>(out)[row * N + col] = acc[i][j][r];
        }
      }
}

unsigned log2_exact(size_t v) {
  unsigned l = 0;
  while ((static_cast<size_t>(1) << l) < v) ++l;
  return l;
}

}  // namespace

__global__ void add_bias_kernel(void* __restrict__ out, int out_dtype, const float* __restrict__ bias, size_t mn,
                                size_t n) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= mn) return;
  if (out_dtype == BQ_BF16) {
    uint16_t* o = static_cast<uint16_t*>(out);
    o[i] = f32_to_bf16(bf16_to_f32(o[i]) + bias[i % n]);
  } else {
    static_cast<float*>(out)[i] += bias[i % n];
  }
}

__global__ void bf16_to_f32_kernel(const uint16_t* __restrict__ src, size_t n, float* __restrict__ dst) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = bf16_to_f32(src[i]);
}

// Ternary weights (Q2S: -1, 0, +1, 16 per word) times f32 activations, without a multiply in the
// sum: +1 adds the activation, -1 subtracts it, anything else leaves the sum alone, and the
// per-tensor scale multiplies the finished sum once -- crates/burn-ndarray/src/ops/qtensor.rs:431-517.
// An output's additions are made in ascending k, the reference's order, by one lane: the results
// are the reference's bit for bit, and the chain of K dependent additions is the kernel's time
// (an add per k, plus the field's decode off the chain). A lane owns one output column and one
// activation row (grid.y). The 16 lanes that share a packed word column load it for 16
// consecutive rows, one row each, and hand the rows round by DPP row broadcast; kTernaryDepth such
// loads are in flight per lane. The addend is built with bit operations -- x, its sign flipped
// when the field's high bit is set, masked to +0 when its low bit is clear -- and sum + (+0) is
// the sum itself here (a sum that starts at +0 never becomes -0), so a skipped field, an infinite
// or a NaN activation included, leaves the sum alone as the reference's `match` does.
constexpr int kTernaryDepth = 4;  // (8, 12, 16 measured the same: the chain of additions is the time)

template <int J>
__device__ __forceinline__ uint32_t ternary_row(uint32_t v) {  // the value lane J of this row of 16 lanes holds
  return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x150 + J, 0xF, 0xF, true));
}

__global__ void __launch_bounds__(256)
ternary_matmul_kernel(const float* __restrict__ x, const uint32_t* __restrict__ w, const float* __restrict__ scale,
                      size_t K, size_t NW, float* __restrict__ out) {
  constexpr int D = kTernaryDepth;
  const size_t N = NW * 16;
  const size_t col = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  const bool active = col < N;  // (N is a multiple of 16: the 16 lanes of a word are active together)
  const size_t wc = active ? col >> 4 : 0;
  const unsigned j = threadIdx.x & 15u, shift = 2u * j;
  const float* __restrict__ xr = x + static_cast<size_t>(blockIdx.y) * K;
  auto fetch = [&](size_t k0) {
    const size_t r = k0 + j;
    return (active && r < K) ? w[r * NW + wc] : 0u;  // rows past the end: zero fields add nothing
  };
  uint32_t ring[D];
#pragma unroll
  for (int d = 0; d < D; ++d) ring[d] = fetch(16u * d);
  float acc = 0.0f;
  for (size_t k0 = 0; k0 < K; k0 += 16 * D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const uint32_t cur = ring[d];
      ring[d] = fetch(k0 + 16u * (d + D));
      const size_t kb = k0 + 16u * d;
      if (kb >= K) break;  // (uniform)
      // rows kb .. kb + 15, in order; FULL: all of them exist (their activations are 16 contiguous
      // scalar loads), else the tail of K, row by row
#define BQ_TERNARY_STEP(JJ)                                                                          \
  {                                                                                                  \
    const uint32_t word = ternary_row<JJ>(cur);                                                      \
    const uint32_t xb = __builtin_bit_cast(uint32_t, (full || kb + JJ < K) ? xr[kb + JJ] : 0.0f);    \
    const uint32_t keep = static_cast<uint32_t>(__builtin_amdgcn_sbfe(static_cast<int>(word), shift, 1u));      /* +-1: all ones */ \
    const uint32_t flip = static_cast<uint32_t>(__builtin_amdgcn_sbfe(static_cast<int>(word), shift + 1u, 1u)) & 0x80000000u; /* -1: the sign */ \
    acc += __builtin_bit_cast(float, (xb ^ flip) & keep);                                            \
  }
      auto group = [&](auto FULL) {
        constexpr bool full = decltype(FULL)::value;
        BQ_TERNARY_STEP(0) BQ_TERNARY_STEP(1) BQ_TERNARY_STEP(2) BQ_TERNARY_STEP(3)
        BQ_TERNARY_STEP(4) BQ_TERNARY_STEP(5) BQ_TERNARY_STEP(6) BQ_TERNARY_STEP(7)
        BQ_TERNARY_STEP(8) BQ_TERNARY_STEP(9) BQ_TERNARY_STEP(10) BQ_TERNARY_STEP(11)
        BQ_TERNARY_STEP(12) BQ_TERNARY_STEP(13) BQ_TERNARY_STEP(14) BQ_TERNARY_STEP(15)
      };
      if (kb + 16 <= K) group(std::true_type{}); else group(std::false_type{});
#undef BQ_TERNARY_STEP
    }
  }
  if (active) out[static_cast<size_t>(blockIdx.y) * N + col] = acc * scale[0];
}

bq_status launch_ternary_matmul(const float* x, const uint32_t* w, const float* scale, size_t m, size_t k, size_t n,
                                float* out, hipStream_t st) {
  if (m == 0 || n == 0) return BQ_OK;
  const size_t nw = n / 16;
  for (size_t m0 = 0; m0 < m; m0 += 65535u) {  // (grid.y holds 65535 rows)
    const size_t rows = std::min<size_t>(65535u, m - m0);
    dim3 grid(static_cast<unsigned>((n + 255) / 256), static_cast<unsigned>(rows)), tb(256);
    hipLaunchKernelGGL(ternary_matmul_kernel, grid, tb, 0, st, x + m0 * k, w, scale, k, nw, out + m0 * n);
    BQ_HIP(hipGetLastError());
  }
  return BQ_OK;
}

bq_status launch_add_bias(void* out, int out_dtype, const float* bias, size_t m, size_t n, hipStream_t st) {
  if (m == 0 || n == 0) return BQ_OK;
  hipLaunchKernelGGL(add_bias_kernel, dim3(static_cast<unsigned>((m * n + 255) / 256)), dim3(256), 0, st, out,
                     out_dtype, bias, m * n, n);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

bq_status launch_bf16_to_f32(const uint16_t* src, size_t n, float* dst, hipStream_t st) {
  if (n == 0) return BQ_OK;
  hipLaunchKernelGGL(bf16_to_f32_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, st, src, n, dst);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

bq_status launch_float_matmul(const void* a, int a_dtype, const void* b, int b_dtype, size_t m,
                              size_t k, size_t n, int out_dtype, void* out, hipStream_t st) {
  if (m == 0 || n == 0) return BQ_OK;
  // 128 x 128 tiles once they fill the chip (more reuse per byte read), 64 x 64 below
  const bool big = ((m + 127) / 128) * ((n + 127) / 128) >= 256;
  const size_t t = big ? 128 : 64;
  if ((n + t - 1) / t > 0x7FFFFFFFu || (m + t - 1) / t > 65535u)
    BQ_FAIL(BQ_ERR_SIZE, "float matmul of %zu x %zu outputs exceeds the launch grid", m, n);
  dim3 grid(static_cast<unsigned>((n + t - 1) / t), static_cast<unsigned>((m + t - 1) / t)), tb(256);
  if (big)
    hipLaunchKernelGGL(float_matmul_kernel<2>, grid, tb, 0, st, a, a_dtype, b, b_dtype, m, k, n, out_dtype, out);
  else
    hipLaunchKernelGGL(float_matmul_kernel<1>, grid, tb, 0, st, a, a_dtype, b, b_dtype, m, k, n, out_dtype, out);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

}  // namespace bq

using namespace bq;

static bool use_gemv(size_t m, int32_t lhs_dtype) { return m <= 16 && lhs_dtype == BQ_F32; }
// Batch size from which the split-activation MFMA kernel beats the vector-ALU decode kernel on
// the 4096 x 14336 weight, one run (us per product, decode / matrix-core kernel). With the weights
// loaded directly (per-tensor scales or one scale per 32 columns), Q8S per tensor: M = 2 17.1 /
// 17.4, M = 3 18.6 / 17.3, M = 4 21.5 / 17.5; Q8S block-32: 19.5 / 19.8, 21.1 / 19.8, 23.5 / 19.9;
// Q4S per tensor: 16.0 / 15.9, 18.5 / 15.7, 20.7 / 15.7; Q4S block-32: 18.1 / 16.5, 22.1 / 16.5,
// 22.9 / 16.5. Through the LDS slot (one scale per 64 or 128 columns) the matrix-core kernel
// takes 22-24.5 us, and the decode kernel stays ahead one row longer.
static size_t split_from_m(int value, int block) {
  const bool direct = block == 0 || block == 32;
  if (value == BQ_Q8S) return direct ? 3 : 4;
  return direct ? 2 : 3;
}

namespace bq {
// Whether bqk_q_matmul has a fused kernel for this problem (else: dequantize + float matmul).
bool fused_matmul_ok(size_t m, size_t k, size_t n, int lhs_dtype, int value, size_t scales_per_row) {
  value = storage_value(value);
  // (one or two rows of bf16 activations: the decode kernel, whatever K's divisibility by 8)
  const int block = scales_per_row ? static_cast<int>(n / scales_per_row) : 0;
  const bool bf16_decode = lhs_dtype == BQ_BF16 && k % 2 == 0 && gemv1_ok(m, n, lhs_dtype, block, value);
  return use_gemv(m, lhs_dtype) || bf16_decode || skinny_ok(m, k, n, lhs_dtype, value) ||
         qgemm_ok(lhs_dtype, k, n, value, scales_per_row);
}
}  // namespace bq

extern "C" size_t bqk_q_matmul_workspace(size_t m, size_t k, size_t n, int32_t lhs_dtype,
                                         int32_t value) {
  if (!value_known(value) || m == 0 || n == 0 || k == 0) return 0;
  value = storage_value(value);  // (the products read two's complement fields: full-range values are their symmetric twins here)
  // the block size and the alignment (which pick the kernel) are not known here: cover every plan
  size_t bytes = 0;
  if (skinny_ok(m, k, n, lhs_dtype, value)) bytes = skinny_workspace(m, k, n, lhs_dtype, value);
  if (split_ok(m, k, n, lhs_dtype, value, 0)) bytes = std::max(bytes, split_workspace(m, k, n));
  if (use_gemv(m, lhs_dtype) || (lhs_dtype == BQ_BF16 && m <= kGemv1MaxMBf16)) {
    size_t slices = gemv_plan(k, n, value).slices;
    if (m <= static_cast<size_t>(gemv1_max_m(num_quants(value))))
      slices = std::max<size_t>(slices, gemv1_plan(m, k, n, value).slices);
    bytes = std::max(bytes, slices * m * n * sizeof(float));
  }
  return std::max(bytes, qgemm_workspace(lhs_dtype, m, k, n));
}

static bool requant_fits(const RequantOut* rq, size_t mn, size_t n) {
  if (rq == nullptr || rq->values == nullptr || rq->scales == nullptr) return false;
  const int bits = value_bits(rq->value);
  if (!(rq->block == 32 || rq->block == 64) || n % static_cast<size_t>(rq->block) || mn % static_cast<size_t>(rq->block)) return false;
  if (bits == 8) return rq->store == BQ_STORE_NATIVE || rq->store == BQ_STORE_PACKED_U32;
  return bits == 4 && rq->store == BQ_STORE_PACKED_U32;
}

static bq_status launch_gemv_reduce(const float* part, size_t mn, unsigned slices, const float* bias, size_t n,
                                    int32_t out_dtype, void* out, hipStream_t st, RequantOut* rq = nullptr) {
  const size_t cols4 = (mn + 3) / 4;
  const int sl = slices >= 16 ? 16 : (slices >= 8 ? 8 : 4);
  dim3 grid(static_cast<unsigned>((cols4 + 256 / sl - 1) / (256 / sl))), tb(256);
  if (requant_fits(rq, mn, n)) {
    const float qmax = static_cast<float>(value_qmax(rq->value)), qmin = static_cast<float>(value_qmin(rq->value));
    const int vpl = value_bits(rq->value) == 8 ? 4 : 8, lanes = rq->block / 4;
#define BQ_RQ(S, V, L)                                                                                              \
  hipLaunchKernelGGL((qgemv_reduce_quant_kernel<S, V, L>), grid, tb, 0, st, part, mn, slices, bias, n, qmin, qmax, \
                     rq->sdt, rq->from_bf16 ? 1 : 0, static_cast<uint32_t*>(rq->values), rq->scales)
#define BQ_RQ_S(V, L) \
  if (sl == 16) BQ_RQ(16, V, L); else if (sl == 8) BQ_RQ(8, V, L); else BQ_RQ(4, V, L)
    if (vpl == 4) { if (lanes == 8) { BQ_RQ_S(4, 8); } else { BQ_RQ_S(4, 16); } }
    else { if (lanes == 8) { BQ_RQ_S(8, 8); } else { BQ_RQ_S(8, 16); } }
#undef BQ_RQ_S
#undef BQ_RQ
    BQ_HIP(hipGetLastError());
    rq->done = true;
    return BQ_OK;
  }
#define BQ_REDUCE(B, S) hipLaunchKernelGGL((qgemv_reduce_kernel<B, S>), grid, tb, 0, st, part, mn, slices, bias, n, out)
  if (out_dtype == BQ_BF16) {
    if (sl == 16) BQ_REDUCE(true, 16); else if (sl == 8) BQ_REDUCE(true, 8); else BQ_REDUCE(true, 4);
  } else {
    if (sl == 16) BQ_REDUCE(false, 16); else if (sl == 8) BQ_REDUCE(false, 8); else BQ_REDUCE(false, 4);
  }
#undef BQ_REDUCE
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

namespace bq {
bq_status launch_splitk_reduce(const float* part, size_t mn, unsigned slices, const float* bias, size_t n,
                               int32_t out_dtype, void* out, hipStream_t stream) {
  return launch_gemv_reduce(part, mn, slices, bias, n, out_dtype, out, stream);
}
}  // namespace bq

// out[r][c] = bias[c], or 0 without a bias: the product over an empty K.
__global__ void empty_k_kernel(const float* __restrict__ bias, size_t mn, size_t n, int out_dtype,
                               void* __restrict__ out) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= mn) return;
  const float v = bias ? bias[i % n] : 0.0f;
  if (out_dtype == BQ_BF16)
    static_cast<uint16_t*>(out)[i] = f32_to_bf16(v);
  else
    static_cast<float*>(out)[i] = v;
}

static bq_status q_matmul_core(const void* lhs, int32_t lhs_dtype, size_t m, size_t k, size_t n,
                               const void* w_values, const float* w_scales, int32_t block,
                               int32_t value, int32_t store, const float* bias, int32_t out_dtype, void* out,
                               void* workspace, size_t workspace_bytes, void* stream, size_t* need_out = nullptr,
                               unsigned* tickets = nullptr, RequantOut* requant = nullptr) {
  if (requant != nullptr) tickets = nullptr;  // (the quantizing sum is the reduction kernel's: two launches)
  // tickets: kTicketBytes of device memory, zero between launches (splitk_tail.hpp), or null. With
  // them the decode kernel finishes its own split-K sum for one or two rows: one launch instead of two.
  // need_out: dry run. The arguments are validated and the kernel is chosen as usual, but nothing is
  // launched: *need_out receives the scratch bytes that kernel would use.
  if (need_out) *need_out = 0;
  BQ_NOTNULL(lhs);
  BQ_NOTNULL(w_values);
  BQ_NOTNULL(w_scales);
  BQ_NOTNULL(out);
  if (!value_known(value)) BQ_FAIL(BQ_ERR_UNSUPPORTED_SCHEME, "unknown quant value %d", value);
  value = storage_value(value);  // (the products read two's complement fields: full-range values are their symmetric twins here)
  if (lhs_dtype != BQ_F32 && lhs_dtype != BQ_BF16) BQ_FAIL(BQ_ERR_DTYPE, "lhs must be f32 or bf16");
  if (out_dtype != BQ_F32 && out_dtype != BQ_BF16) BQ_FAIL(BQ_ERR_DTYPE, "out must be f32 or bf16");
  if (store == BQ_STORE_NATIVE && value != BQ_Q8S)
    BQ_FAIL(BQ_ERR_UNSUPPORTED_SCHEME, "Can't store native sub-byte values");
  const size_t vpl = static_cast<size_t>(num_quants(value));
  if (n % vpl) BQ_FAIL(BQ_ERR_SHAPE, "Can't store in u32: N = %zu, %zu values per word", n, vpl);
  if (block < 0 || (block > 0 && (n % static_cast<size_t>(block) || static_cast<size_t>(block) % vpl ||
                                  ((block / vpl) & (block / vpl - 1)))))
    BQ_FAIL(BQ_ERR_SHAPE, "run block %d along N = %zu is not supported by the fused matmul", block, n);
  if ((reinterpret_cast<uintptr_t>(w_values) & 3u) || (reinterpret_cast<uintptr_t>(lhs) & 15u) ||
      (reinterpret_cast<uintptr_t>(out) & 15u))
    BQ_FAIL(BQ_ERR_SHAPE, "q_matmul operands must be 16-byte aligned");
  if (m == 0 || n == 0) return BQ_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const size_t nw = n / vpl;
  const bool per_tensor = block == 0;
  const unsigned bwl2 = per_tensor ? 0 : log2_exact(static_cast<size_t>(block) / vpl);
  const size_t spr = per_tensor ? 0 : n / static_cast<size_t>(block);
  const uint32_t* w = static_cast<const uint32_t*>(w_values);

  if (k == 0) {  // an empty sum, written by a kernel (a memset node must not enter a captured graph)
    if (need_out) return BQ_OK;
    hipLaunchKernelGGL(empty_k_kernel, dim3(static_cast<unsigned>((m * n + 255) / 256)), dim3(256), 0, st, bias,
                       m * n, n, out_dtype, out);
    BQ_HIP(hipGetLastError());
    return BQ_OK;
  }

  // (native Q8S bytes are the packed words' bytes, so either store takes the same kernels)
  // a few rows of activations (f32 from M = 5 or 3, bf16 from M = 3, or from M = 1 where the
  // decode kernel's layout does not apply): the split-activation kernel on the bf16 matrix cores
  const bool bf16_decode = lhs_dtype == BQ_BF16 && gemv1_ok(m, n, lhs_dtype, block, value) &&
                           (reinterpret_cast<uintptr_t>(w_values) & 15u) == 0 && (reinterpret_cast<uintptr_t>(lhs) & 3u) == 0 &&
                           k % 2 == 0;  // (whole 32-bit words of activations)
  if ((m >= split_from_m(value, block) || (lhs_dtype == BQ_BF16 && !bf16_decode)) && split_ok(m, k, n, lhs_dtype, value, block) &&
      (reinterpret_cast<uintptr_t>(w_values) & 15u) == 0 &&
      (per_tensor || (reinterpret_cast<uintptr_t>(w_scales) & 15u) == 0)) {
    const size_t need = split_workspace(m, k, n);
    if (need_out) return *need_out = need, BQ_OK;
    if (workspace == nullptr || workspace_bytes < need)
      BQ_FAIL(BQ_ERR_SIZE, "q_matmul workspace: need %zu bytes, got %zu", need, workspace_bytes);
    float* part = static_cast<float*>(workspace);
    unsigned slices = 0;
    // (the single-launch sum does not pay here: with 3 to 32 rows the partial sums are megabytes, which
    // the reduction kernel reads with the whole chip while a last workgroup per tile would read them
    // alone -- measured on the 4096 x 14336 weight, M = 4 / 16: 20.1 / 25.3 us against 19.8 / 22.5 us)
    BQ_TRY(launch_qsplit(lhs, lhs_dtype, w, w_scales, m, k, n, value, block, part, &slices, st));
    return launch_gemv_reduce(part, m * n, slices, bias, n, out_dtype, out, st, requant);
  }

  if (gemv1_ok(m, n, lhs_dtype, block, value) && (reinterpret_cast<uintptr_t>(w_values) & 15u) == 0 &&
      (lhs_dtype == BQ_F32 || bf16_decode)) {
    const size_t cpl = static_cast<size_t>(gemv1_words(static_cast<int>(vpl))) * vpl;
    GemvPlan p = gemv1_plan(m, k, n, value);
    const size_t need = static_cast<size_t>(p.slices) * m * n * sizeof(float);
    if (need_out) return *need_out = need, BQ_OK;
    if (workspace == nullptr || workspace_bytes < need)
      BQ_FAIL(BQ_ERR_SIZE, "q_matmul workspace: need %zu bytes, got %zu", need, workspace_bytes);
    float* part = static_cast<float*>(workspace);
    const size_t nq = n / cpl;
    const unsigned shift = per_tensor ? 0 : log2_exact(static_cast<size_t>(block) / cpl);
    dim3 grid(p.strips, p.slices), tb(gemv1_waves(static_cast<int>(vpl), static_cast<int>(m)) * kWave);
    // One launch when the caller brought ticket counters, for one or two rows: the last workgroup of a
    // strip reads slices x M x 4 KiB of partial sums by itself, which is less than a second launch costs
    // (4096 x 14336 weight, M = 1: 15.7 against 16.05 us per product) only while M is small.
    unsigned* const tk = (tickets != nullptr && m <= 2 && p.strips <= kTicketCells && need < 0x7FFFFFFFull) ? tickets : nullptr;
    const void* x = lhs;
    const uint32_t* w4 = static_cast<const uint32_t*>(w_values);
#define BQ_GEMV1B(V, MM)                                                                                         \
  if (per_tensor)                                                                                                \
    hipLaunchKernelGGL((qgemv1_kernel<V, true, MM, true>), grid, tb, 0, st, x, w4, w_scales, k, nq, shift, spr,  \
                       p.rows_per_slice, part, tk, bias, out_dtype == BQ_BF16, out);                             \
  else                                                                                                           \
    hipLaunchKernelGGL((qgemv1_kernel<V, false, MM, true>), grid, tb, 0, st, x, w4, w_scales, k, nq, shift, spr, \
                       p.rows_per_slice, part, tk, bias, out_dtype == BQ_BF16, out)
#define BQ_GEMV1(V, MM)                                                                                    \
  if (per_tensor)                                                                                          \
    hipLaunchKernelGGL((qgemv1_kernel<V, true, MM>), grid, tb, 0, st, x, w4, w_scales, k, nq, shift, spr,  \
                       p.rows_per_slice, part, tk, bias, out_dtype == BQ_BF16, out);                       \
  else                                                                                                     \
    hipLaunchKernelGGL((qgemv1_kernel<V, false, MM>), grid, tb, 0, st, x, w4, w_scales, k, nq, shift, spr, \
                       p.rows_per_slice, part, tk, bias, out_dtype == BQ_BF16, out)
    if (lhs_dtype == BQ_BF16) {  // m is 1 or 2
      if (value == BQ_Q8S) {
        if (m == 1) { BQ_GEMV1B(4, 1); } else { BQ_GEMV1B(4, 2); }
      } else {
        if (m == 1) { BQ_GEMV1B(8, 1); } else { BQ_GEMV1B(8, 2); }
      }
    } else if (value == BQ_Q8S) {
      switch (m) {
        case 1: BQ_GEMV1(4, 1); break;
        case 2: BQ_GEMV1(4, 2); break;
        case 3: BQ_GEMV1(4, 3); break;
        case 4: BQ_GEMV1(4, 4); break;
        case 5: BQ_GEMV1(4, 5); break;
        case 6: BQ_GEMV1(4, 6); break;
        case 7: BQ_GEMV1(4, 7); break;
        default: BQ_GEMV1(4, 8); break;
      }
    } else {
      switch (m) {
        case 1: BQ_GEMV1(8, 1); break;
        case 2: BQ_GEMV1(8, 2); break;
        case 3: BQ_GEMV1(8, 3); break;
        default: BQ_GEMV1(8, 4); break;
      }
    }
#undef BQ_GEMV1
#undef BQ_GEMV1B
    BQ_HIP(hipGetLastError());
    if (tk != nullptr) return BQ_OK;
    return launch_gemv_reduce(part, m * n, p.slices, bias, n, out_dtype, out, st, requant);
  }

  // f32 activations: the FP32-matrix kernel pays off from M = 7 (measured: 38-41 us flat against
  // 27 + 2.6 M us for the vector-ALU q-GEMV below); it reads 16-byte word groups sharing one scale.
  const bool f32_small = lhs_dtype == BQ_F32 && m <= 16;
  const bool skinny_layout_ok =
      !f32_small || (m >= 7 && (per_tensor || bwl2 >= 2) && (reinterpret_cast<uintptr_t>(w_values) & 15u) == 0);
  if (skinny_ok(m, k, n, lhs_dtype, value) && skinny_layout_ok) {
    const size_t need = skinny_workspace(m, k, n, lhs_dtype, value);
    if (need_out) return *need_out = need, BQ_OK;
    if (workspace == nullptr || workspace_bytes < need)
      BQ_FAIL(BQ_ERR_SIZE, "q_matmul workspace: need %zu bytes, got %zu", need, workspace_bytes);
    float* part = static_cast<float*>(workspace);
    unsigned slices = 0;
    BQ_TRY(launch_qskinny(lhs, lhs_dtype, w, w_scales, m, k, n, value, bwl2, spr, per_tensor, part, &slices, st));
    return launch_gemv_reduce(part, m * n, slices, bias, n, out_dtype, out, st, requant);
  }

  if (use_gemv(m, lhs_dtype)) {
    GemvPlan p = gemv_plan(k, n, value);
    const size_t need = static_cast<size_t>(p.slices) * m * n * sizeof(float);
    if (need_out) return *need_out = need, BQ_OK;
    if (workspace == nullptr || workspace_bytes < need)
      BQ_FAIL(BQ_ERR_SIZE, "q_matmul workspace: need %zu bytes, got %zu", need, workspace_bytes);
    float* part = static_cast<float*>(workspace);
    const float* x = static_cast<const float*>(lhs);
    dim3 grid(p.strips, p.slices), tb(kGemvThreads);
#define BQ_GEMV(V, MM)                                                                        \
  hipLaunchKernelGGL((qgemv_kernel<V, MM>), grid, tb, 0, st, x, w, w_scales, k, nw, bwl2, spr, \
                     per_tensor, p.rows_per_slice, part)
#define BQ_GEMV_M(V)                                       \
  switch (m) {                                             \
    case 1: BQ_GEMV(V, 1); break;                          \
    case 2: BQ_GEMV(V, 2); break;                          \
    case 3: BQ_GEMV(V, 3); break;                          \
    case 4: BQ_GEMV(V, 4); break;                          \
    case 5: BQ_GEMV(V, 5); break;                          \
    case 6: BQ_GEMV(V, 6); break;                          \
    case 7: BQ_GEMV(V, 7); break;                          \
    case 8: BQ_GEMV(V, 8); break;                          \
    case 9: BQ_GEMV(V, 9); break;                          \
    case 10: BQ_GEMV(V, 10); break;                        \
    case 11: BQ_GEMV(V, 11); break;                        \
    case 12: BQ_GEMV(V, 12); break;                        \
    case 13: BQ_GEMV(V, 13); break;                        \
    case 14: BQ_GEMV(V, 14); break;                        \
    case 15: BQ_GEMV(V, 15); break;                        \
    default: BQ_GEMV(V, 16); break;                        \
  }
    if (value == BQ_Q8S) {
      BQ_GEMV_M(4)
    } else {
      BQ_GEMV_M(8)
    }
#undef BQ_GEMV_M
#undef BQ_GEMV
    BQ_HIP(hipGetLastError());
    return launch_gemv_reduce(part, m * n, p.slices, bias, n, out_dtype, out, st, requant);
  }

  if (!qgemm_ok(lhs_dtype, k, n, value, spr))
    BQ_FAIL(BQ_ERR_SHAPE, "the tiled q_matmul needs K %% 8 == 0 and operands under 4 GiB (K = %zu)", k);
  if (need_out) return *need_out = qgemm_workspace(lhs_dtype, m, k, n), BQ_OK;
  unsigned slices = 1;
  float* part = nullptr;
  BQ_TRY(launch_qgemm(lhs, lhs_dtype, w, w_scales, m, k, n, value, bwl2, spr, per_tensor, bias, out_dtype, out,
                      workspace, workspace_bytes, &slices, &part, st));
  if (slices > 1) return launch_gemv_reduce(part, m * n, slices, bias, n, out_dtype, out, st, requant);
  return BQ_OK;
}

extern "C" bq_status bqk_q_matmul(const void* lhs, int32_t lhs_dtype, size_t m, size_t k, size_t n,
                                  const void* w_values, const float* w_scales, int32_t block,
                                  int32_t value, int32_t store, int32_t out_dtype, void* out,
                                  void* workspace, size_t workspace_bytes, void* stream) {
  return q_matmul_core(lhs, lhs_dtype, m, k, n, w_values, w_scales, block, value, store, nullptr, out_dtype, out,
                       workspace, workspace_bytes, stream);
}

extern "C" bq_status bqk_q_linear(const void* x, int32_t x_dtype, size_t m, size_t k, size_t n,
                                  const void* w_values, const float* w_scales, int32_t block,
                                  int32_t value, int32_t store, const float* bias, int32_t out_dtype,
                                  void* out, void* workspace, size_t workspace_bytes, void* stream) {
  if (bias != nullptr && (reinterpret_cast<uintptr_t>(bias) & 15u))
    BQ_FAIL(BQ_ERR_SHAPE, "q_linear bias must be 16-byte aligned");
  return q_matmul_core(x, x_dtype, m, k, n, w_values, w_scales, block, value, store, bias, out_dtype, out,
                       workspace, workspace_bytes, stream);
}

namespace bq {
// bqk_q_linear with the ticket counters of the single-launch split-K sum (the handle level passes its
// device context's; kTicketBytes, zero between launches, one call at a time per device).
bq_status q_linear_with_tickets(const void* x, int32_t x_dtype, size_t m, size_t k, size_t n, const void* w_values,
                                const float* w_scales, int32_t block, int32_t value, int32_t store, const float* bias,
                                int32_t out_dtype, void* out, void* workspace, size_t workspace_bytes, unsigned* tickets,
                                void* stream, RequantOut* requant) {
  if (bias != nullptr && (reinterpret_cast<uintptr_t>(bias) & 15u))
    BQ_FAIL(BQ_ERR_SHAPE, "q_linear bias must be 16-byte aligned");
  return q_matmul_core(x, x_dtype, m, k, n, w_values, w_scales, block, value, store, bias, out_dtype, out,
                       workspace, workspace_bytes, stream, nullptr, tickets, requant);
}
}  // namespace bq

// ================================================================================ no allocation
// bqk_q_linear for callers that cannot allocate (code under HIP graph capture, serving loops,
// harnesses that forbid hipMalloc): the split-K partials and the bf16 copy of an f32 lhs, which
// bqk_q_linear takes through its `workspace` argument, live in this file-scope device array
// instead. Every GPU the library runs on holds its own copy of the array at its own address
// until the process ends; the address is looked up once per device and the kernels only ever see
// that pointer (the array's name is a host-side stand-in, not a device address).
static __device__ __align__(256) unsigned char scratch[BQK_STATIC_SCRATCH_BYTES];
// The ticket counters of its single-launch split-K sum: zero when the module is loaded, left zero by
// every launch (splitk_tail.hpp). Like `scratch`, shared by all calls on one GPU.
static __device__ __align__(256) unsigned static_tickets[kTicketCells * kTicketStride];

namespace bq {

// The device address of `scratch` on the current device (looked up on first use, then cached), and
// of the ticket counters beside it.
bq_status static_scratch_ptr(void** out, unsigned** tickets_out) {
  static std::mutex mu;
  static void* ptrs[64] = {nullptr};
  static unsigned* tickets[64] = {nullptr};
  int ordinal = 0;
  BQ_HIP(hipGetDevice(&ordinal));
  if (ordinal < 0 || ordinal >= 64) BQ_FAIL(BQ_ERR_HIP, "device ordinal %d out of range", ordinal);
  std::lock_guard<std::mutex> lock(mu);
  if (ptrs[ordinal] == nullptr) {
    void* p = nullptr;
    BQ_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (p == nullptr || (reinterpret_cast<uintptr_t>(p) & 255u))
      BQ_FAIL(BQ_ERR_HIP, "the static scratch array resolved to %p", p);
    void* t = nullptr;
    BQ_HIP(hipGetSymbolAddress(&t, HIP_SYMBOL(static_tickets)));
    if (t == nullptr || (reinterpret_cast<uintptr_t>(t) & 255u))
      BQ_FAIL(BQ_ERR_HIP, "the static ticket counters resolved to %p", t);
    ptrs[ordinal] = p;
    tickets[ordinal] = static_cast<unsigned*>(t);
  }
  *out = ptrs[ordinal];
  if (tickets_out) *tickets_out = tickets[ordinal];
  return BQ_OK;
}

}  // namespace bq

extern "C" bq_status bqk_q_linear_static(const void* x, int32_t x_dtype, size_t m, size_t k, size_t n,
                                         const void* w_values, const float* w_scales, int32_t block,
                                         int32_t value, int32_t store, const float* bias, int32_t out_dtype,
                                         void* out, void* stream) {
  if (bias != nullptr && (reinterpret_cast<uintptr_t>(bias) & 15u))
    BQ_FAIL(BQ_ERR_SHAPE, "q_linear bias must be 16-byte aligned");
  // dry run first: the kernel this product takes and the scratch it uses, before anything is launched
  size_t need = 0;
  BQ_TRY(q_matmul_core(x, x_dtype, m, k, n, w_values, w_scales, block, value, store, bias, out_dtype, out, nullptr, 0,
                       stream, &need));
  if (need > BQK_STATIC_SCRATCH_BYTES)
    BQ_FAIL(BQ_ERR_SIZE,
            "bqk_q_linear_static: this product needs %zu bytes of scratch, the static array holds %zu; "
            "use bqk_q_linear with a workspace",
            need, static_cast<size_t>(BQK_STATIC_SCRATCH_BYTES));
  void* ws = nullptr;
  unsigned* tickets = nullptr;
  BQ_TRY(static_scratch_ptr(&ws, &tickets));
  return q_matmul_core(x, x_dtype, m, k, n, w_values, w_scales, block, value, store, bias, out_dtype, out, ws,
                       BQK_STATIC_SCRATCH_BYTES, stream, nullptr, tickets);
}
