// quantize / quantize_dynamic kernels for gfx950.
//
// Replaces, for a GPU tensor, what burn computes with compute_range + compute_q_params
// (crates/burn-backend/src/quantization/scheme.rs:44-104) followed by B::quantize
// (crates/burn-ndarray/src/ops/qtensor.rs:82-186 is the arithmetic reproduced bit for bit).
//
// Work decomposition: one lane owns one output word (4 x i8 or 8 x i4, i.e. VPL consecutive
// inputs read as 128-bit loads); a block of B = LANES * VPL elements is LANES adjacent lanes of
// one wavefront, so its absmax is a log2(LANES)-step cross-lane max and the whole
// range -> scale -> round -> clamp -> pack chain stays in registers: one read of x, one write of
// the words, one write of the scales.
#include "common.hpp"
#include "device_math.hpp"

namespace bq {

namespace {

// Tunables (the defaults are the measured best; overridable at compile time for sweeps).
#ifndef BQ_QUANT_THREADS
#define BQ_QUANT_THREADS 256
#endif
#ifndef BQ_BLOCK_THREADS
#define BQ_BLOCK_THREADS 64
#endif
#ifndef BQ_BLOCK_UNROLL
#define BQ_BLOCK_UNROLL 4
#endif
#ifndef BQ_TENSOR_UNROLL
#define BQ_TENSOR_UNROLL 4
#endif
#ifndef BQ_ABSMAX_UNROLL
#define BQ_ABSMAX_UNROLL 8
#endif
#ifndef BQ_ABSMAX_NT
#define BQ_ABSMAX_NT 0
#endif
#ifndef BQ_QUANT_QUAD_STORE
#define BQ_QUANT_QUAD_STORE 1
#endif
#ifndef BQ_QUANT_NT_STORE
#define BQ_QUANT_NT_STORE 1
#endif
constexpr int kThreads = BQ_QUANT_THREADS;

// b of QuantValue::range() by values per word: Q8S 127, Q4S 7, Q2S 1
constexpr float qmax_of(int vpl) { return vpl == 4 ? 127.0f : (vpl == 8 ? 7.0f : 1.0f); }

template <int VPL>
struct Vals {
  float v[VPL];
};

template <int VPL>
__device__ __forceinline__ Vals<VPL> load_vals(const float* __restrict__ x, size_t word) {
  Vals<VPL> r;
  const vfloat4* p = reinterpret_cast<const vfloat4*>(x) + word * (VPL / 4);
#pragma unroll
  for (int i = 0; i < VPL / 4; ++i) {
    vfloat4 t = __builtin_nontemporal_load(p + i);
    r.v[4 * i + 0] = t.x;
    r.v[4 * i + 1] = t.y;
    r.v[4 * i + 2] = t.z;
    r.v[4 * i + 3] = t.w;
  }
  return r;
}

template <int VPL>
__device__ __forceinline__ float absmax_vals(const Vals<VPL>& a) {
  float m = 0.0f;
#pragma unroll
  for (int i = 0; i < VPL; ++i) m = fmaxf(m, fabsf(a.v[i]));
  return m;
}

// Reference-order path: an IEEE divide per value. Taken for scales outside the exponent range
// the reciprocal path is proven for (subnormal / huge scales) -- rare, so speed is irrelevant.
// FULL: a full-range value (Q8F, Q4F): the lower clamp is -QMAX - 1.
template <int VPL, bool FULL = false>
__device__ __forceinline__ uint32_t quantize_pack_div(const Vals<VPL>& a, float s) {
  constexpr float QMAX = qmax_of(VPL), QMIN = FULL ? -QMAX - 1.0f : -QMAX;
  int q[VPL];
#pragma unroll
  for (int i = 0; i < VPL; ++i) q[i] = quantize_div(a.v[i], s, QMIN, QMAX);
  return pack_fields<VPL>(q);
}

// Fast path: quotients through r = RN(1/s) and one fma correction (== the IEEE quotient).
// CLAMP is dropped when s came from this block's own absmax: |x| <= amax and
// s = RN(amax / QMAX) is normal, so |x / s| < QMAX + 0.5 already.
// (A full-range value always clamps: absmax / s is QMAX + 0.5, which rounds to QMAX + 1.)
template <int VPL, bool CLAMP, bool FULL = false>
__device__ __forceinline__ uint32_t quantize_pack_recip(const Vals<VPL>& a, float s, float r) {
  constexpr float QMAX = qmax_of(VPL), QMIN = FULL ? -QMAX - 1.0f : -QMAX;
  int q[VPL];
#pragma unroll
  for (int i = 0; i < VPL; ++i) {
    float v = div_by_recip(a.v[i], s, r);
    if (CLAMP || FULL) v = fminf(fmaxf(v, QMIN), QMAX);
    q[i] = round_half_away_i32(v);
  }
  return pack_fields<VPL>(q);
}

// Quantize VPL values against a given (stored) scale.
template <int VPL, bool FULL = false>
__device__ __forceinline__ uint32_t quantize_pack(const Vals<VPL>& a, float s_stored) {
  const float s = valid_scale(s_stored);
  if (recip_path_ok(s)) return quantize_pack_recip<VPL, true, FULL>(a, s, recip_exact(s));
  return quantize_pack_div<VPL, FULL>(a, s);
}

// ---- run-block schemes: B = LANES * VPL consecutive elements per scale ------------------------
// A workgroup of T threads owns a contiguous chunk of T * U words; lane t takes words t, t + T, ...
// of the chunk, so every load/store instruction of a wave is one contiguous 1 KiB / 256 B run and
// U independent 128-bit loads are in flight per lane before any arithmetic starts. The packed
// words leave with non-temporal stores (like the loads: nothing here is read again by this
// kernel); with plain stores the same shapes are 5 % slower. Measured on the [8192, 8192] tensor
// (one box, graph replays, non-temporal stores), T x U: 64 x 1 73.2 us, 64 x 2 55.4, 64 x 4 55.1,
// 64 x 8 57.9, 128 x 2 57.5, 128 x 4 55.7, 128 x 8 57.9, 256 x 2 57.1, 256 x 4 56.2; with plain
// stores 256 x 2 took 60.0 us. A fixed grid of 1024-4096 workgroups that walk the chunks with a
// stride and load the next chunk ahead of the arithmetic is slower (63-67 us): many short
// workgroups keep more loads in flight.
constexpr int kBlockThreads = BQ_BLOCK_THREADS;      // run-block kernel
constexpr int kBlockUnroll = BQ_BLOCK_UNROLL;
constexpr int kTensorUnroll = BQ_TENSOR_UNROLL;      // per-tensor second pass

// Lane 4j + i of a workgroup of T threads holds words chunk + T u + 4j + i, u = 0..3. A 4 x 4
// transpose inside each quad of lanes (two DPP swaps) leaves lane 4j + i with the four
// consecutive words chunk + T i + 4j + {0..3}: one 16-byte store per lane instead of four 4-byte
// ones (1 % on the [8192, 8192] block quantize).
template <int T>
__device__ __forceinline__ void store_words_quad(uint32_t (&packed)[4], size_t chunk, uint32_t* __restrict__ out) {
  const bool b0 = threadIdx.x & 1, b1 = threadIdx.x & 2;
  auto swap1 = [](uint32_t v) { return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0xB1, 0xF, 0xF, false)); };
  auto swap2 = [](uint32_t v) { return static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x4E, 0xF, 0xF, false)); };
#pragma unroll
  for (int p = 0; p < 4; p += 2) {   // first: lanes i and i ^ 1 exchange across registers p, p + 1
    const uint32_t got = swap1(b0 ? packed[p] : packed[p + 1]);
    if (b0) packed[p] = got; else packed[p + 1] = got;
  }
#pragma unroll
  for (int p = 0; p < 2; ++p) {      // then: lanes i and i ^ 2 exchange across registers p, p + 2
    const uint32_t got = swap2(b1 ? packed[p] : packed[p + 2]);
    if (b1) packed[p] = got; else packed[p + 2] = got;
  }
  const size_t at = chunk + static_cast<size_t>(T) * (threadIdx.x & 3) + (threadIdx.x & ~3u);
  const vuint4 v = {packed[0], packed[1], packed[2], packed[3]};
  if (BQ_QUANT_NT_STORE) __builtin_nontemporal_store(v, reinterpret_cast<vuint4*>(out + at));
  else *reinterpret_cast<vuint4*>(out + at) = v;
}

// ---- the second of two passes goes to the XCD that read each chunk in the first -------------------
// A per-tensor scale (alone, or over block scales) needs max|x| of the whole tensor before a value
// can be quantized: absmax_kernel reads the tensor front to back, in chunks of kThreads *
// kAbsmaxUnroll float4s. Workgroups go to the 8 XCDs round robin, so chunk c was read by XCD
// c % 8. The pass that quantizes takes pieces of PPC to the chunk, and workgroup b, which lands
// on XCD b % 8, takes a piece of a chunk that XCD read, starting with the last ones. Measured on
// a 4096 x 4096 tensor, both passes, one run: 27.0 us with workgroup b on piece b, 26.8 us
// with the pieces merely reversed, 25.1 us on the first pass's XCD front to back, 24.7 us on
// the first pass's XCD back to front (the second pass by the profiler: 14.4 -> 12.4 us; alone on
// a cold tensor it takes 16.8 us under every mapping). What carries over is state of the XCD
// other than cached data: the L2 hit and miss counts and the bytes requested from the fabric are
// the same under all four mappings (every line of the input misses again). `grid` is a multiple
// of 8 * PPC; pieces past the end of the tensor find nothing to do. (Streaming loads in the
// first pass for all but the last 16-32 MB: 25.3-26.2 us. 1024 or 2048 first-pass workgroups
// instead of 512: 25.8-26.7 us.)
constexpr int kAbsmaxUnroll = BQ_ABSMAX_UNROLL;
template <unsigned PPC>
__device__ __forceinline__ size_t piece_back_to_front(unsigned b, unsigned grid) {
  const unsigned xcd = b & 7u, q = grid / 8u - 1u - b / 8u;  // q-th piece of this XCD, counted from the end
  return static_cast<size_t>(q / PPC) * (8u * PPC) + xcd * PPC + q % PPC;
}
template <unsigned PPC>
inline size_t grid_back_to_front(size_t pieces) { return (pieces + 8 * PPC - 1) / (8 * PPC) * (8 * PPC); }
// pieces of `threads` x `unroll` packed words (VPL floats each) to a first-pass chunk
template <int VPL>
constexpr unsigned pieces_per_chunk(int threads, int unroll) {
  return static_cast<unsigned>((kThreads * kAbsmaxUnroll * 4) / (threads * unroll * VPL));
}
static_assert((kThreads * kAbsmaxUnroll * 4) % (kBlockThreads * kBlockUnroll * 8) == 0 &&
              (kThreads * kAbsmaxUnroll * 4) % (kThreads * kTensorUnroll * 8) == 0, "a first-pass chunk is whole second-pass pieces");

// TWO (dynamic only): block scales relative to a per-tensor scale. `scales_in` then points at that
// one f32 (global), `stored_out` receives a block's scale as it is stored, scale_to_dtype(s / global)
// in the dtype `sdt`, and the block is quantized against global * that, which goes to `scales_out`
// -- normalize_scales (crates/burn-backend/src/quantization/scheme.rs:106-134) and what
// NdArray::quantize makes of its result, one IEEE operation per step as there.
// FULL: a full-range value: span b - a = 2 QMAX + 1 (no proven divide-free form: the scale takes
// the IEEE division, once per block), lower clamp -QMAX - 1.
template <int VPL, int LANES, bool DYNAMIC, bool TWO = false, bool FULL = false>
__global__ void __launch_bounds__(kBlockThreads)
quantize_block_kernel(const float* __restrict__ x, size_t words, uint32_t* __restrict__ out,
                      float* __restrict__ scales_out, const float* __restrict__ scales_in, int sdt,
                      float* __restrict__ stored_out = nullptr) {
  static_assert(!TWO || DYNAMIC, "two-level scales are split where the block scales are computed");
  constexpr int U = kBlockUnroll;
  constexpr int QMAX = (VPL == 4) ? 127 : 7;
  constexpr float SPAN = 2.0f * QMAX + (FULL ? 1.0f : 0.0f);
  // (TWO follows absmax_kernel over the same tensor)
  const size_t piece = TWO ? piece_back_to_front<pieces_per_chunk<VPL>(kBlockThreads, kBlockUnroll)>(blockIdx.x, gridDim.x) : blockIdx.x;
  const size_t base = piece * (kBlockThreads * U) + threadIdx.x;
  constexpr bool kQuadStore = BQ_QUANT_QUAD_STORE && U == 4;
  uint32_t packed[U];
  Vals<VPL> a[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t w = base + static_cast<size_t>(u) * kBlockThreads;
    if (w < words) {
      a[u] = load_vals<VPL>(x, w);
    } else {
#pragma unroll
      for (int i = 0; i < VPL; ++i) a[u].v[i] = 0.0f;
    }
  }
  // words is a multiple of LANES and kThreads is a multiple of 64, so the lanes of one block are
  // in range (or out of range) together; the cross-lane max runs in every lane either way.
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t w = base + static_cast<size_t>(u) * kBlockThreads;
    uint32_t word;
    float s;
    float stored = 0.0f;
    if (TWO) {
      const float m = group_max<LANES>(absmax_vals<VPL>(a[u]));
      const float one_level = (!FULL && absmax_fast_ok(m)) ? scale_from_absmax_fast<QMAX>(m) : scale_from_absmax(m, SPAN);
      const float global = scales_in[0];
      stored = scale_round_up(one_level / global, sdt);
      s = global * stored;
      word = quantize_pack<VPL, FULL>(a[u], s);
    } else if (DYNAMIC) {
      const float m = group_max<LANES>(absmax_vals<VPL>(a[u]));
      if (FULL) {
        s = scale_round_up(scale_from_absmax(m, SPAN), sdt);
        word = quantize_pack<VPL, true>(a[u], s);
      } else if (sdt != BQ_SCALE_F32) {  // f16 / bf16 scales: divide by the scale as it will be stored
        s = scale_round_up(absmax_fast_ok(m) ? scale_from_absmax_fast<QMAX>(m) : scale_from_absmax(m, SPAN), sdt);
        word = quantize_pack<VPL>(a[u], s);
      } else if (absmax_fast_ok(m)) {
        s = scale_from_absmax_fast<QMAX>(m);
        word = quantize_pack_recip<VPL, false>(a[u], s, recip_exact(s));
      } else {
        s = scale_from_absmax(m, SPAN);
        word = quantize_pack_div<VPL>(a[u], valid_scale(s));
      }
    } else {
      s = (w < words) ? scales_in[w / LANES] : 1.0f;
      word = quantize_pack<VPL, FULL>(a[u], s);
    }
    if (w < words) {
      if (DYNAMIC && (w & (LANES - 1)) == 0) scales_out[w / LANES] = s;
      if (TWO && (w & (LANES - 1)) == 0) stored_out[w / LANES] = stored;
      if (!kQuadStore) {
        if (BQ_QUANT_NT_STORE) __builtin_nontemporal_store(word, out + w); else out[w] = word;
      }
    }
    if (kQuadStore) packed[u] = word;
  }
  if (kQuadStore) {
    const size_t chunk = piece * (kBlockThreads * U);
    if (chunk + kBlockThreads * U <= words && (reinterpret_cast<uintptr_t>(out) & 15u) == 0) {
      store_words_quad<kBlockThreads>(reinterpret_cast<uint32_t (&)[4]>(packed), chunk, out);
    } else {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const size_t w = base + static_cast<size_t>(u) * kBlockThreads;
        if (w < words) out[w] = packed[u];
      }
    }
  }
}

// ---- per-tensor: pass 1, absmax -------------------------------------------------------------
// Exactly BQ_ABSMAX_CELLS workgroups; each walks chunks of kThreads * kAbsmaxUnroll float4s with
// a grid stride (plain loads: the second pass re-reads the tensor, so it is left in the caches;
// the next chunk's loads are issued before the current one is reduced) and stores max|x| of what
// it saw to its own cell. No atomics, so the cells need no initialisation.
// max over the workgroup, in every thread (one call per kernel: the LDS cells are not reused)
__device__ __forceinline__ float workgroup_max(float m) {
  __shared__ float part[kThreads / kWave];
  m = group_max<kWave>(m);
  if ((threadIdx.x & (kWave - 1)) == 0) part[threadIdx.x / kWave] = m;
  __syncthreads();
  float r = part[0];
#pragma unroll
  for (int i = 1; i < kThreads / kWave; ++i) r = fmaxf(r, part[i]);
  return r;
}

__global__ void __launch_bounds__(kThreads)
absmax_kernel(const float* __restrict__ x, size_t n, uint32_t* __restrict__ absmax_bits) {
  constexpr int U = kAbsmaxUnroll;
  const size_t n4 = n / 4;
  const size_t chunk = static_cast<size_t>(kThreads) * U;
  const size_t stride = static_cast<size_t>(gridDim.x) * chunk;
  const vfloat4* p = reinterpret_cast<const vfloat4*>(x);
  auto load = [&](size_t base, vfloat4* t) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t i = base + static_cast<size_t>(u) * kThreads;
      t[u] = (i < n4) ? (BQ_ABSMAX_NT ? __builtin_nontemporal_load(p + i) : p[i]) : vfloat4{0.f, 0.f, 0.f, 0.f};
    }
  };
  float m = 0.0f;
  size_t base = static_cast<size_t>(blockIdx.x) * chunk + threadIdx.x;
  vfloat4 t[U], t_next[U];
  load(base, t);
  while (base < n4) {  // (base - threadIdx.x is workgroup-uniform; a chunk past n4 loads zeros)
    load(base + stride, t_next);
#pragma unroll
    for (int u = 0; u < U; ++u)
      m = fmaxf(fmaxf(m, fabsf(t[u].x)), fmaxf(fabsf(t[u].y), fmaxf(fabsf(t[u].z), fabsf(t[u].w))));
#pragma unroll
    for (int u = 0; u < U; ++u) t[u] = t_next[u];
    base += stride;
  }
  if (blockIdx.x == 0 && threadIdx.x < (n & 3)) m = fmaxf(m, fabsf(x[n4 * 4 + threadIdx.x]));
  // Non-negative floats order like their bit patterns.
  const float r = workgroup_max(m);
  if (threadIdx.x == 0) absmax_bits[blockIdx.x] = __float_as_uint(r);
}

// max over the BQ_ABSMAX_CELLS cells, in every thread of a workgroup of kThreads threads.
__device__ __forceinline__ float absmax_from_cells(const uint32_t* __restrict__ cells) {
  float m = 0.0f;
#pragma unroll
  for (int i = static_cast<int>(threadIdx.x); i < BQ_ABSMAX_CELLS; i += kThreads) m = fmaxf(m, __uint_as_float(cells[i]));
  return workgroup_max(m);
}

// Unaligned input: same reduction with scalar loads.
__global__ void __launch_bounds__(kThreads)
absmax_scalar_kernel(const float* __restrict__ x, size_t n, uint32_t* __restrict__ absmax_bits) {
  const size_t stride = static_cast<size_t>(gridDim.x) * kThreads;
  float m = 0.0f;
  for (size_t i = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x; i < n; i += stride)
    m = fmaxf(m, fabsf(x[i]));
  const float r = workgroup_max(m);
  if (threadIdx.x == 0) absmax_bits[blockIdx.x] = __float_as_uint(r);
}

__global__ void __launch_bounds__(kThreads)
scale_from_cells_kernel(const uint32_t* __restrict__ cells, float span, int sdt, float* __restrict__ scale_out) {
  const float s = scale_round_up(scale_from_absmax(absmax_from_cells(cells), span), sdt);
  if (threadIdx.x == 0) scale_out[0] = s;
}

__global__ void scales_from_absmax_kernel(const float* __restrict__ amax, size_t n, float span,
                                          float* __restrict__ scales) {
  size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) scales[i] = scale_from_absmax(amax[i], span);
}

// ---- per-tensor: pass 2, quantize against the device-resident scale ---------------------------
// FROM_ABSMAX: `scale` points at the absmax cells (bit patterns of partial max|x|) instead of a
// scale; the scale is derived here, (2 * amax) / (b - a), and block 0 stores it to scale_out.
// Same chunked layout as the block kernel.
template <int VPL, bool FROM_ABSMAX, bool FULL = false>
__global__ void __launch_bounds__(kThreads)
quantize_tensor_kernel(const float* __restrict__ x, size_t n, const float* __restrict__ scale,
                       float* __restrict__ scale_out, uint32_t* __restrict__ out, int sdt) {
  constexpr int U = kTensorUnroll;
  constexpr float QMAX = qmax_of(VPL), QMIN = FULL ? -QMAX - 1.0f : -QMAX;
  constexpr float SPAN = QMAX - QMIN;
  const size_t words = n / VPL;
  // (2-bit values: a piece of 16 floats per lane and word is as large as two first-pass chunks; plain order)
  constexpr unsigned PPC = pieces_per_chunk<VPL>(kThreads, kTensorUnroll);
  const size_t piece = PPC == 0 ? static_cast<size_t>(blockIdx.x) : piece_back_to_front<(PPC == 0 ? 1u : PPC)>(blockIdx.x, gridDim.x);
  const size_t base = piece * (kThreads * U) + threadIdx.x;
  Vals<VPL> a[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t w = base + static_cast<size_t>(u) * kThreads;
    if (w < words) {
      a[u] = load_vals<VPL>(x, w);
    } else {
#pragma unroll
      for (int i = 0; i < VPL; ++i) a[u].v[i] = 0.0f;
    }
  }
  const float s_stored =
      FROM_ABSMAX ? scale_round_up(scale_from_absmax(absmax_from_cells(reinterpret_cast<const uint32_t*>(scale)), SPAN), sdt)
                  : scale[0];
  if (FROM_ABSMAX && piece == 0 && threadIdx.x == 0) scale_out[0] = s_stored;
  const float s = valid_scale(s_stored);
  const bool fast = recip_path_ok(s);
  const float r = recip_exact(s);
  constexpr bool kQuadStore = BQ_QUANT_QUAD_STORE && U == 4;
  const size_t chunk = piece * (kThreads * U);
  // (out is the values region of a tensor or a caller's buffer: 16-byte stores need it aligned)
  const bool quad = kQuadStore && chunk + kThreads * U <= words && (reinterpret_cast<uintptr_t>(out) & 15u) == 0;
  uint32_t packed[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t w = base + static_cast<size_t>(u) * kThreads;
    packed[u] = 0u;
    if (w < words)
    {
      packed[u] = fast ? quantize_pack_recip<VPL, true, FULL>(a[u], s, r) : quantize_pack_div<VPL, FULL>(a[u], s);
      if (!quad) {
        if (BQ_QUANT_NT_STORE) __builtin_nontemporal_store(packed[u], out + w); else out[w] = packed[u];
      }
    }
  }
  if (quad) store_words_quad<kThreads>(reinterpret_cast<uint32_t (&)[4]>(packed), chunk, out);
  // native i8 store with n % 4 != 0: the last 1..3 values, one byte each
  if (VPL == 4 && piece == 0 && threadIdx.x == 0) {
    int8_t* bytes = reinterpret_cast<int8_t*>(out);
    for (size_t i = words * 4; i < n; ++i) bytes[i] = static_cast<int8_t>(quantize_div(x[i], s, QMIN, QMAX));
  }
}

// Small tensors: one launch. One workgroup of 1024 threads loads the tensor once (16 floats a lane), takes
// the maximum through LDS, and quantizes what it holds: the same arithmetic as the two passes, in one
// dispatch. What a call of this size costs is the launches, not the bytes (a launch and the wait for it
// take 10.8 us on this part, every further launch 2.3 us, and the second pass cannot start before the first
// has left the chip): 4096 values 16.2 -> 12.7 us per synchronised call. The limit is where one compute
// unit's load bandwidth eats the gain: 65 536 values (64 floats a lane) took 16.7 us either way.
constexpr int kSmallThreads = 1024;
constexpr size_t kSmallValues = 16384;

template <int VPL, bool FULL>
__global__ void __launch_bounds__(kSmallThreads)
quantize_tensor_small_kernel(const float* __restrict__ x, size_t n, float* __restrict__ scale_out,
                             uint32_t* __restrict__ out, int sdt) {
  constexpr int U = static_cast<int>(kSmallValues / (kSmallThreads * VPL));
  constexpr float QMAX = qmax_of(VPL), QMIN = FULL ? -QMAX - 1.0f : -QMAX;
  __shared__ float part[kSmallThreads / kWave];
  const size_t words = n / VPL;
  Vals<VPL> a[U];
  float m = 0.0f;
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t w = threadIdx.x + static_cast<size_t>(u) * kSmallThreads;
    if (w < words) {
      a[u] = load_vals<VPL>(x, w);
    } else {
#pragma unroll
      for (int i = 0; i < VPL; ++i) a[u].v[i] = 0.0f;
    }
  }
#pragma unroll
  for (int u = 0; u < U; ++u) m = fmaxf(m, absmax_vals<VPL>(a[u]));
  if (VPL == 4 && threadIdx.x < (n & 3)) m = fmaxf(m, fabsf(x[words * 4 + threadIdx.x]));  // native i8: the last 1..3 values
  m = group_max<kWave>(m);
  if ((threadIdx.x & (kWave - 1)) == 0) part[threadIdx.x / kWave] = m;
  __syncthreads();
  float amax = part[0];
#pragma unroll
  for (int i = 1; i < kSmallThreads / kWave; ++i) amax = fmaxf(amax, part[i]);
  const float s_stored = scale_round_up(scale_from_absmax(amax, QMAX - QMIN), sdt);
  if (threadIdx.x == 0) scale_out[0] = s_stored;
  const float s = valid_scale(s_stored);
  const bool fast = recip_path_ok(s);
  const float r = recip_exact(s);
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t w = threadIdx.x + static_cast<size_t>(u) * kSmallThreads;
    if (w < words) out[w] = fast ? quantize_pack_recip<VPL, true, FULL>(a[u], s, r) : quantize_pack_div<VPL, FULL>(a[u], s);
  }
  if (VPL == 4 && threadIdx.x == 0) {
    int8_t* bytes = reinterpret_cast<int8_t*>(out);
    for (size_t i = words * 4; i < n; ++i) bytes[i] = static_cast<int8_t>(quantize_div(x[i], s, QMIN, QMAX));
  }
}

// 2-bit values against a given scale: 16 values to the word, so a lane that owned a whole word would
// read 64 bytes at a stride of 64 (the per-tensor kernel above does, at 3.6 TB/s). Here a lane takes
// one 16-byte piece per load, consecutive lanes consecutive pieces: the four lanes of a quad hold the
// four quarters of a word, put their bytes together with two DPP swaps, and lane i of the quad keeps
// the word of load i. n is a multiple of 16, x 16-byte aligned.
__global__ void __launch_bounds__(256)
quantize_tensor_2bit_kernel(const float* __restrict__ x, size_t n, const float* __restrict__ scale, float qmin,
                            uint32_t* __restrict__ out) {
  const float s = valid_scale(scale[0]);
  const bool fast = recip_path_ok(s);
  const float r = recip_exact(s);
  const size_t pieces = n / 4, first = static_cast<size_t>(blockIdx.x) * 1024 + threadIdx.x;
  vfloat4 v[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const size_t f = first + static_cast<size_t>(i) * 256;
    v[i] = f < pieces ? __builtin_nontemporal_load(reinterpret_cast<const vfloat4*>(x) + f) : vfloat4{0.f, 0.f, 0.f, 0.f};
  }
  uint32_t mine = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float e[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
    uint32_t b = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int q = fast ? quantize_recip(e[j], s, r, qmin, 1.0f) : quantize_div(e[j], s, qmin, 1.0f);
      b |= (static_cast<uint32_t>(q) & 3u) << (2 * j);
    }
    uint32_t w = b << (8u * (threadIdx.x & 3u));
    w |= static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(w), 0xB1, 0xF, 0xF, false));  // lanes 2p <-> 2p + 1
    w |= static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(w), 0x4E, 0xF, 0xF, false));  // pairs of a quad
    if ((threadIdx.x & 3u) == static_cast<unsigned>(i)) mine = w;
  }
  // load i of this quad was word 64 i + tid / 4 of the workgroup's 256
  const size_t word = static_cast<size_t>(blockIdx.x) * 256 + (threadIdx.x & 3u) * 64u + threadIdx.x / 4u;
  if (word * 16 < n) __builtin_nontemporal_store(mine, out + word);
}

// Unaligned input pointer: one value per lane, byte stores (native Q8S only).
__global__ void __launch_bounds__(kThreads)
quantize_tensor_scalar_kernel(const float* __restrict__ x, size_t n,
                              const float* __restrict__ scale, float qmin, int8_t* __restrict__ out) {
  const float s = valid_scale(scale[0]);
  const size_t stride = static_cast<size_t>(gridDim.x) * kThreads;
  for (size_t i = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x; i < n; i += stride)
    out[i] = static_cast<int8_t>(quantize_div(x[i], s, qmin, 127.0f));
}

// ---- general rectangle blocks (any block shape): complete, not fast ---------------------------
struct RectDims {
  int rank;
  size_t shape[BQ_MAX_RANK];
  size_t blk[BQ_MAX_RANK];
  size_t grid[BQ_MAX_RANK];  // blocks per dim
};

// BlockLayout::block_of (crates/burn-std/src/tensor/quantization.rs:182-192)
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

// One thread per block: max |x| over the block rectangle -> scale.
__global__ void rect_scales_kernel(const float* __restrict__ x, RectDims d, size_t nblocks,
                                   size_t block_elems, float span, int sdt, float* __restrict__ scales) {
  size_t b = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (b >= nblocks) return;
  // origin of block b
  size_t origin[BQ_MAX_RANK];
  size_t rem = b;
  for (int i = d.rank - 1; i >= 0; --i) {
    origin[i] = (rem % d.grid[i]) * d.blk[i];
    rem /= d.grid[i];
  }
  float m = 0.0f;
  for (size_t e = 0; e < block_elems; ++e) {
    size_t r = e, idx = 0, stride = 1;
    for (int i = d.rank - 1; i >= 0; --i) {
      size_t c = origin[i] + r % d.blk[i];
      r /= d.blk[i];
      idx += c * stride;
      stride *= d.shape[i];
    }
    m = fmaxf(m, fabsf(x[idx]));
  }
  scales[b] = scale_round_up(scale_from_absmax(m, span), sdt);
}

// One thread per output word; every value looks its own block up, so words may straddle blocks.
template <int BITS>
__global__ void rect_quantize_kernel(const float* __restrict__ x, RectDims d, size_t last,
                                     size_t words_per_line, size_t total_words, bool native, bool full,
                                     const float* __restrict__ scales, uint32_t* __restrict__ out) {
  constexpr int NQ = 32 / BITS;
  constexpr float QMAX = (BITS == 8) ? 127.0f : (BITS == 4 ? 7.0f : 1.0f);
  const float QMIN = full ? -QMAX - 1.0f : -QMAX;
  constexpr uint32_t MASK = (1u << BITS) - 1u;
  size_t w = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (w >= total_words) return;
  size_t line = w / words_per_line, col0 = (w % words_per_line) * NQ;
  uint32_t word = 0;
  for (int j = 0; j < NQ; ++j) {
    size_t c = col0 + j;
    if (c >= last) break;
    size_t idx = line * last + c;
    float s = valid_scale(scales[d.rank ? rect_block_of(d, idx) : 0]);
    int q = quantize_div(x[idx], s, QMIN, QMAX);
    if (native) {
      reinterpret_cast<int8_t*>(out)[idx] = static_cast<int8_t>(q);
    } else {
      word |= (static_cast<uint32_t>(q) & MASK) << (j * BITS);
    }
  }
  if (!native) out[w] = word;
}

inline unsigned grid_for(size_t items, unsigned cap) {
  size_t g = (items + kThreads - 1) / kThreads;
  if (g < 1) g = 1;
  return static_cast<unsigned>(g < cap ? g : cap);
}

template <int VPL, bool DYNAMIC, bool TWO = false, bool FULL = false>
bq_status launch_block(const float* x, size_t n, int block, uint32_t* out, float* scales_out,
                       const float* scales_in, int sdt, hipStream_t st, float* stored_out = nullptr) {
  const size_t words = n / VPL;
  const int lanes = block / VPL;
  size_t pieces = (words + kBlockThreads * kBlockUnroll - 1) / (kBlockThreads * kBlockUnroll);
  if (TWO) pieces = grid_back_to_front<pieces_per_chunk<VPL>(kBlockThreads, kBlockUnroll)>(pieces);
  if (pieces > 0x7FFFFFFFull) BQ_FAIL(BQ_ERR_SIZE, "quantize of %zu values exceeds the launch grid", n);
  const unsigned grid = static_cast<unsigned>(pieces);
#define BQ_CASE(L)                                                                         \
  case L:                                                                                  \
    hipLaunchKernelGGL((quantize_block_kernel<VPL, L, DYNAMIC, TWO, FULL>), dim3(grid), dim3(kBlockThreads), \
                       0, st, x, words, out, scales_out, scales_in, sdt, stored_out);      \
    break;
  switch (lanes) {
    BQ_CASE(1) BQ_CASE(2) BQ_CASE(4) BQ_CASE(8) BQ_CASE(16) BQ_CASE(32) BQ_CASE(64)
    default:
      BQ_FAIL(BQ_ERR_UNSUPPORTED_SCHEME, "run block %d has no fused kernel", block);
  }
#undef BQ_CASE
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace

// True when `block` has a fused run-block kernel for `value`.
bool fused_block_ok(int block, int value) {
  const int vpl = num_quants(value);
  if (block < vpl || block % vpl) return false;
  const int lanes = block / vpl;
  return lanes <= 64 && (lanes & (lanes - 1)) == 0;
}

__global__ void fill_u32_kernel(uint32_t* __restrict__ dst, size_t n, uint32_t value) {
  size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = value;
}

// ---- small host-to-device copies and the word a waiting host reads -----------------------------------------
// TO_HOST: dst is the pinned memory and the host reads it as soon as it sees seq, so every lane's stores are
// pushed out to system scope before the barrier.
template <bool TO_HOST>
__global__ void __launch_bounds__(1024)
copy_small_kernel(const vuint4* __restrict__ src, vuint4* __restrict__ dst, uint32_t bytes, uint32_t* __restrict__ done,
                  uint32_t seq) {
  const uint32_t n16 = bytes / 16;
  vuint4 v[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const uint32_t i = threadIdx.x + u * 1024u;
    if (i < n16) v[u] = src[i];
  }
  uint8_t last = 0;
  if (threadIdx.x < (bytes & 15u)) last = reinterpret_cast<const uint8_t*>(src)[n16 * 16 + threadIdx.x];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const uint32_t i = threadIdx.x + u * 1024u;
    if (i < n16) dst[i] = v[u];
  }
  if (threadIdx.x < (bytes & 15u)) reinterpret_cast<uint8_t*>(dst)[n16 * 16 + threadIdx.x] = last;
  // a lane's stores were issued with the data its loads brought: behind the barrier no lane reads src any more
  if (TO_HOST) __threadfence_system();
  __syncthreads();
  if (threadIdx.x == 0) __hip_atomic_store(done, seq, TO_HOST ? __ATOMIC_RELEASE : __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

__global__ void host_word_kernel(uint32_t* __restrict__ word, uint32_t seq) {
  if (threadIdx.x == 0) __hip_atomic_store(word, seq, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
}

bq_status launch_copy_small(const void* src, void* dst, size_t bytes, bool to_host, uint32_t* done, uint32_t seq,
                            hipStream_t st) {
  if (bytes > 4u * 1024u * 16u || ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15u))
    BQ_FAIL(BQ_ERR_SIZE, "small copy of %zu bytes: at most 64 KiB between 16-byte aligned buffers", bytes);
  if (to_host)
    hipLaunchKernelGGL(copy_small_kernel<true>, dim3(1), dim3(1024), 0, st, static_cast<const vuint4*>(src),
                       static_cast<vuint4*>(dst), static_cast<uint32_t>(bytes), done, seq);
  else
    hipLaunchKernelGGL(copy_small_kernel<false>, dim3(1), dim3(1024), 0, st, static_cast<const vuint4*>(src),
                       static_cast<vuint4*>(dst), static_cast<uint32_t>(bytes), done, seq);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

bq_status launch_host_word(uint32_t* word, uint32_t seq, hipStream_t st) {
  hipLaunchKernelGGL(host_word_kernel, dim3(1), dim3(64), 0, st, word, seq);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

bq_status launch_fill_u32(uint32_t* dst, size_t n, uint32_t value, hipStream_t st) {
  if (n == 0) return BQ_OK;
  hipLaunchKernelGGL(fill_u32_kernel, dim3((n + 255) / 256), dim3(256), 0, st, dst, n, value);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

// Validate mode: NaNs into counts[0], infinities into counts[1] (one atomic per workgroup that saw any).
__global__ void __launch_bounds__(256) count_nonfinite_kernel(const float* __restrict__ x, size_t n,
                                                              uint32_t* __restrict__ counts) {
  const size_t stride = static_cast<size_t>(gridDim.x) * 256;
  unsigned nan = 0, inf = 0;
  for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < n; i += stride) {
    const uint32_t mag = __float_as_uint(x[i]) & 0x7FFFFFFFu;
    nan += mag > 0x7F800000u;
    inf += mag == 0x7F800000u;
  }
  __shared__ unsigned tot[2];
  if (threadIdx.x == 0) tot[0] = tot[1] = 0;
  __syncthreads();
  if (nan) atomicAdd(&tot[0], nan);
  if (inf) atomicAdd(&tot[1], inf);
  __syncthreads();
  if (threadIdx.x == 0) {
    if (tot[0]) atomicAdd(counts + 0, tot[0]);
    if (tot[1]) atomicAdd(counts + 1, tot[1]);
  }
}

bq_status launch_count_nonfinite(const float* x, size_t n, uint32_t* counts, hipStream_t st) {
  if (n == 0) return BQ_OK;
  size_t g = (n + 255) / 256;
  if (g > 4096) g = 4096;
  hipLaunchKernelGGL(count_nonfinite_kernel, dim3(static_cast<unsigned>(g)), dim3(256), 0, st, x, n, counts);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

// Plain streaming copy: the known-traffic kernel the HBM counters are calibrated against, and the
// ceiling the streaming kernels are compared with. One 16-byte chunk per lane, 256 lanes per
// workgroup, non-temporal both ways: the best of the shapes measured on a 256 MiB copy (chunks per
// lane 1 / 2 / 4 / 8 at 256 threads: 6.51 / 6.12 / 6.18 / 4.29 TB/s; 1024 threads x 1: 6.45; 32
// contiguous bytes per lane: 4.0-5.1; persistent grids of 256-8192 workgroups with the next
// chunk's loads in flight: 5.5-6.3; plain instead of non-temporal accesses: 5.6; hipMemcpyAsync
// device to device: 5.4).
__global__ void __launch_bounds__(256) copy16_kernel(const vuint4* __restrict__ src, vuint4* __restrict__ dst,
                                                     size_t chunks) {
  const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (i < chunks) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

bq_status launch_quantize_rect(const float* x, const size_t* shape, int rank, const size_t* blk,
                               int value, int store, bool dynamic, int sdt, void* values, float* scales,
                               hipStream_t st) {
  RectDims d{};
  d.rank = blk ? rank : 0;
  size_t n = 1, nblocks = 1, block_elems = 1;
  for (int i = 0; i < rank; ++i) {
    d.shape[i] = shape[i];
    d.blk[i] = blk ? blk[i] : shape[i];
    d.grid[i] = blk ? shape[i] / blk[i] : 1;
    n *= shape[i];
    nblocks *= d.grid[i];
    block_elems *= d.blk[i];
  }
  if (n == 0) return BQ_OK;
  const float span = value_span(value);
  if (dynamic) {
    RectDims dd = d;
    dd.rank = rank;  // per-tensor: one block spanning everything
    hipLaunchKernelGGL(rect_scales_kernel, dim3((nblocks + 63) / 64), dim3(64), 0, st, x, dd,
                       nblocks, block_elems, span, sdt, scales);
    BQ_HIP(hipGetLastError());
  }
  const size_t last = rank ? shape[rank - 1] : 1;
  const size_t nq = static_cast<size_t>(num_quants(value));
  const size_t wpl = (last + nq - 1) / nq;
  const size_t total = (n / last) * wpl;
  const bool native = store == BQ_STORE_NATIVE;
  dim3 grid((total + kThreads - 1) / kThreads), tb(kThreads);
  const bool full = value_full(value);
  if (value_bits(value) == 8)
    hipLaunchKernelGGL(rect_quantize_kernel<8>, grid, tb, 0, st, x, d, last, wpl, total, native, full,
                       scales, static_cast<uint32_t*>(values));
  else if (value_bits(value) == 4)
    hipLaunchKernelGGL(rect_quantize_kernel<4>, grid, tb, 0, st, x, d, last, wpl, total, native, full,
                       scales, static_cast<uint32_t*>(values));
  else
    hipLaunchKernelGGL(rect_quantize_kernel<2>, grid, tb, 0, st, x, d, last, wpl, total, native, full,
                       scales, static_cast<uint32_t*>(values));
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

// ---- Calibration::AbsMean (crates/burn-backend/src/quantization/scheme.rs:57-69) ------------------
// gamma = mean(|x|) per tensor or per block; the range is [-gamma, +gamma], so compute_q_params
// gives scale = (2 gamma) / (b - a). The reference takes the mean with its float_mean / mean_dim
// (a sum in an order of its backend's choosing, divided by the count); here every sum has a fixed
// order, so results repeat run to run: per tensor, BQ_ABSMAX_CELLS workgroups each add the chunks
// they stride over (a per-thread f32 sum, then the threads of the workgroup pairwise through LDS),
// and one workgroup adds the cells in f64 and divides; per block, one thread adds its block's
// elements in ascending order (rectangles of any shape; calibration runs once per weight).
__device__ __forceinline__ float workgroup_sum(float v) {
  __shared__ float part[kThreads];
  part[threadIdx.x] = v;
  __syncthreads();
#pragma unroll
  for (int half = kThreads / 2; half > 0; half >>= 1) {
    if (static_cast<int>(threadIdx.x) < half) part[threadIdx.x] += part[threadIdx.x + half];
    __syncthreads();
  }
  return part[0];
}

__global__ void __launch_bounds__(kThreads)
abs_sum_kernel(const float* __restrict__ x, size_t n, float* __restrict__ cells) {
  // 16-byte loads, four in flight per lane, four independent vector sums per lane (a fixed
  // function of the element index, so the result repeats run to run); scalar loads when x is not
  // 16-byte aligned, and for the last n % 4 elements.
  const size_t stride = static_cast<size_t>(gridDim.x) * kThreads;
  const size_t first = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x;
  float sum = 0.0f;
  if ((reinterpret_cast<uintptr_t>(x) & 15u) == 0) {
    const size_t n4 = n / 4;
    const vfloat4* p = reinterpret_cast<const vfloat4*>(x);
    vfloat4 acc[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) acc[u] = vfloat4{0.f, 0.f, 0.f, 0.f};
    size_t i = first;
    for (; i + 3 * stride < n4; i += 4 * stride) {
      vfloat4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u] = __builtin_nontemporal_load(p + i + u * stride);
#pragma unroll
      for (int u = 0; u < 4; ++u) acc[u] += vfloat4{fabsf(v[u].x), fabsf(v[u].y), fabsf(v[u].z), fabsf(v[u].w)};
    }
    for (; i < n4; i += stride) {
      const vfloat4 v = __builtin_nontemporal_load(p + i);
      acc[0] += vfloat4{fabsf(v.x), fabsf(v.y), fabsf(v.z), fabsf(v.w)};
    }
    const vfloat4 a = (acc[0] + acc[1]) + (acc[2] + acc[3]);
    sum = (a.x + a.y) + (a.z + a.w);
    if (first == 0)
      for (size_t r = n4 * 4; r < n; ++r) sum += fabsf(x[r]);
  } else {
    for (size_t i = first; i < n; i += stride) sum += fabsf(x[i]);
  }
  const float total = workgroup_sum(sum);
  if (threadIdx.x == 0) cells[blockIdx.x] = total;
}

__global__ void __launch_bounds__(kThreads)
abs_mean_from_cells_kernel(const float* __restrict__ cells, size_t n, float* __restrict__ gamma) {
  __shared__ double part[kThreads];
  double sum = 0.0;
  for (int i = static_cast<int>(threadIdx.x); i < BQ_ABSMAX_CELLS; i += kThreads) sum += static_cast<double>(cells[i]);
  part[threadIdx.x] = sum;
  __syncthreads();
  for (int half = kThreads / 2; half > 0; half >>= 1) {
    if (static_cast<int>(threadIdx.x) < half) part[threadIdx.x] += part[threadIdx.x + half];
    __syncthreads();
  }
  if (threadIdx.x == 0) gamma[0] = static_cast<float>(part[0] / static_cast<double>(n));
}

// One thread per block: mean |x| over the block rectangle.
__global__ void rect_abs_mean_kernel(const float* __restrict__ x, RectDims d, size_t nblocks, size_t block_elems,
                                     float* __restrict__ gamma) {
  const size_t b = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (b >= nblocks) return;
  size_t origin[BQ_MAX_RANK];
  size_t rem = b;
  for (int i = d.rank - 1; i >= 0; --i) {
    origin[i] = (rem % d.grid[i]) * d.blk[i];
    rem /= d.grid[i];
  }
  float sum = 0.0f;
  for (size_t e = 0; e < block_elems; ++e) {
    size_t r = e, idx = 0, stride = 1;
    for (int i = d.rank - 1; i >= 0; --i) {
      const size_t c = origin[i] + r % d.blk[i];
      r /= d.blk[i];
      idx += c * stride;
      stride *= d.shape[i];
    }
    sum += fabsf(x[idx]);
  }
  gamma[b] = sum / static_cast<float>(block_elems);
}

// gamma[params] = mean |x| per tensor (blk null; `cells`: BQ_ABSMAX_CELLS floats of scratch) or per block.
bq_status launch_abs_mean(const float* x, const size_t* shape, int rank, const size_t* blk, float* cells, float* gamma,
                          hipStream_t st) {
  size_t n = 1;
  for (int i = 0; i < rank; ++i) n *= shape[i];
  if (n == 0) return BQ_OK;
  if (blk == nullptr) {
    hipLaunchKernelGGL(abs_sum_kernel, dim3(BQ_ABSMAX_CELLS), dim3(kThreads), 0, st, x, n, cells);
    BQ_HIP(hipGetLastError());
    hipLaunchKernelGGL(abs_mean_from_cells_kernel, dim3(1), dim3(kThreads), 0, st, cells, n, gamma);
    BQ_HIP(hipGetLastError());
    return BQ_OK;
  }
  RectDims d{};
  d.rank = rank;
  size_t nblocks = 1, block_elems = 1;
  for (int i = 0; i < rank; ++i) {
    d.shape[i] = shape[i];
    d.blk[i] = blk[i];
    d.grid[i] = shape[i] / blk[i];
    nblocks *= d.grid[i];
    block_elems *= d.blk[i];
  }
  hipLaunchKernelGGL(rect_abs_mean_kernel, dim3((nblocks + 63) / 64), dim3(64), 0, st, x, d, nblocks, block_elems, gamma);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

// scales[i] = (2 * range[i]) / (b - a) for any value type: compute_q_params on a symmetric range.
bq_status launch_scales_from_range(const float* range, size_t n, int value, float* scales, hipStream_t st) {
  if (n == 0) return BQ_OK;
  hipLaunchKernelGGL(scales_from_absmax_kernel, dim3((n + 255) / 256), dim3(256), 0, st, range, n, value_span(value), scales);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

// ---- scales in a 2-byte dtype ------------------------------------------------------------------
// Tensors keep their scales as f32 on the device, holding values the scale dtype represents exactly
// (rounded up at quantize time, or widened when a blob is loaded); the 2-byte form only exists on
// the wire.
__global__ void round_scales_kernel(const float* __restrict__ src, float* __restrict__ dst, size_t n, int sdt) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = scale_round_up(src[i], sdt);
}

// f32 -> f16 bits of a value f16 represents exactly (or an infinity / NaN)
__device__ __forceinline__ uint16_t f16_bits_exact(float v) {
  const uint32_t u = __float_as_uint(v), sign = (u >> 16) & 0x8000u, mag = u & 0x7FFFFFFFu;
  if (mag >= 0x7F800000u) return static_cast<uint16_t>(sign | 0x7C00u | (mag > 0x7F800000u ? 0x200u : 0u));
  if (mag < 0x38800000u) {  // below 2^-14: a multiple of 2^-24
    const float t = fabsf(v) * 16777216.0f;
    return static_cast<uint16_t>(sign | static_cast<uint32_t>(t));
  }
  return static_cast<uint16_t>(sign | ((mag - 0x38000000u) >> 13));
}

__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
  const uint32_t sign = (static_cast<uint32_t>(h) & 0x8000u) << 16, ex = (h >> 10) & 0x1Fu, man = h & 0x3FFu;
  if (ex == 0) {
    const float t = static_cast<float>(man) * 5.9604644775390625e-8f;  // man * 2^-24, exact
    return __uint_as_float(sign | __float_as_uint(t));
  }
  if (ex == 31) return __uint_as_float(sign | 0x7F800000u | (man << 13));
  return __uint_as_float(sign | ((ex + 112u) << 23) | (man << 13));
}

// e4m3 bits of a value the format represents exactly (non-negative half; NaN and infinities -> 0x7F)
__device__ __forceinline__ uint8_t e4m3_bits_exact(float v) {
  const uint32_t u = __float_as_uint(v);
  if ((u & 0x7FFFFFFFu) >= 0x7F800000u) return 0x7Fu;
  if (!(v > 0.0f)) return 0u;
  if (v < 0.015625f) return static_cast<uint8_t>(v * 512.0f);          // subnormal: m = v / 2^-9
  return static_cast<uint8_t>((((u >> 23) - 127u + 7u) << 3) | ((u >> 20) & 7u));
}
__device__ __forceinline__ float e4m3_bits_to_f32(uint8_t b) {
  const uint32_t ex = (b >> 3) & 0xFu, man = b & 7u;
  if (ex == 15u && man == 7u) return __uint_as_float(0x7FC00000u);
  const float v = ex == 0u ? static_cast<float>(man) * 0.001953125f : __uint_as_float(((ex + 120u) << 23) | (man << 20));
  return (b & 0x80u) ? -v : v;
}

// T: uint16_t (f16, bf16) or uint8_t (ue4m3)
template <typename T>
__global__ void scales_to_wire_kernel(const float* __restrict__ src, T* __restrict__ dst, size_t n, int sdt) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  // (a scale that did not pass through scale_round_up, e.g. given by hand: rounded up here as well)
  const float v = scale_round_up(src[i], sdt);
  if (sizeof(T) == 1)
    dst[i] = static_cast<T>(e4m3_bits_exact(v));
  else
    dst[i] = static_cast<T>(sdt == 2 ? static_cast<uint16_t>(__float_as_uint(v) >> 16) : f16_bits_exact(v));
}

template <typename T>
__global__ void scales_from_wire_kernel(const T* __restrict__ src, float* __restrict__ dst, size_t n, int sdt) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  if (sizeof(T) == 1)
    dst[i] = e4m3_bits_to_f32(static_cast<uint8_t>(src[i]));
  else
    dst[i] = sdt == 2 ? __uint_as_float(static_cast<uint32_t>(src[i]) << 16) : f16_bits_to_f32(static_cast<uint16_t>(src[i]));
}

bq_status launch_scale_from_cells(const uint32_t* cells, int value, int sdt, float* scale_out, hipStream_t st) {
  hipLaunchKernelGGL(scale_from_cells_kernel, dim3(1), dim3(kThreads), 0, st, cells, value_span(value),
                     sdt, scale_out);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

// ---- two-level schemes ---------------------------------------------------------------------------
namespace {

// normalize_scales (crates/burn-backend/src/quantization/scheme.rs:106-134) and what NdArray::quantize
// does with its result (crates/burn-ndarray/src/ops/qtensor.rs:90-101,519-531), one IEEE operation
// per step as there: global = max(scales) / dtype_max, not below the smallest normal f32; a block
// scale is stored as scale_to_dtype(scale / global) and the block is quantized against
// global * that. `cells` hold the partial maxima of the scales (they are not negative).
__global__ void __launch_bounds__(kThreads)
two_level_split_kernel(float* __restrict__ scales, size_t n, const uint32_t* __restrict__ cells, float dtype_max, int sdt,
                       float* __restrict__ global_out, float* __restrict__ stored) {
  const float top = absmax_from_cells(cells);
  const float global = fmaxf(top / dtype_max, 1.17549435e-38f);
  if (blockIdx.x == 0 && threadIdx.x == 0) global_out[0] = global;
  const size_t i = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i < n) {
    const float st = scale_round_up(scales[i] / global, sdt);
    stored[i] = st;
    scales[i] = global * st;
  }
}

// The per-tensor scale from the absmax cells of the whole tensor. The largest block scale is the
// scale of the largest block maximum (every step of scale = (2 absmax) / (b - a) is a correctly
// rounded, hence monotonic, operation), so no block scale has to exist yet.
__global__ void __launch_bounds__(kThreads)
two_level_global_kernel(const uint32_t* __restrict__ cells, float span, float dtype_max, float* __restrict__ global_out) {
  const float top = scale_from_absmax(absmax_from_cells(cells), span);
  if (threadIdx.x == 0) global_out[0] = fmaxf(top / dtype_max, 1.17549435e-38f);
}

__global__ void scales_times_global_kernel(const float* __restrict__ stored, const float* __restrict__ global, size_t n,
                                           float* __restrict__ scales) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) scales[i] = global[0] * stored[i];
}

}  // namespace

bq_status launch_two_level_split(float* scales, size_t n, const uint32_t* cells, int sdt, float* global_out, float* stored,
                                 hipStream_t st) {
  if (sdt != BQ_SCALE_F16 && sdt != BQ_SCALE_UE4M3)
    BQ_FAIL(BQ_ERR_UNSUPPORTED_SCHEME,
            "block scales of this dtype reach f32's range, which a per-tensor scale cannot absorb (f16 and ue4m3 block scales can)");
  if (n == 0) return BQ_OK;
  hipLaunchKernelGGL(two_level_split_kernel, dim3(static_cast<unsigned>((n + kThreads - 1) / kThreads)), dim3(kThreads), 0, st,
                     scales, n, cells, sdt == BQ_SCALE_F16 ? 65504.0f : 448.0f, sdt, global_out, stored);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

bq_status launch_two_level_global(const uint32_t* cells, int value, int sdt, float* global_out, hipStream_t st) {
  if (sdt != BQ_SCALE_F16 && sdt != BQ_SCALE_UE4M3)
    BQ_FAIL(BQ_ERR_UNSUPPORTED_SCHEME,
            "block scales of this dtype reach f32's range, which a per-tensor scale cannot absorb (f16 and ue4m3 block scales can)");
  hipLaunchKernelGGL(two_level_global_kernel, dim3(1), dim3(kThreads), 0, st, cells, value_span(value),
                     sdt == BQ_SCALE_F16 ? 65504.0f : 448.0f, global_out);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

bq_status launch_scales_times_global(const float* stored, const float* global, size_t n, float* scales, hipStream_t st) {
  if (n == 0) return BQ_OK;
  hipLaunchKernelGGL(scales_times_global_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, st, stored, global,
                     n, scales);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

bq_status launch_round_scales(const float* src, float* dst, size_t n, int sdt, hipStream_t st) {
  if (n == 0) return BQ_OK;
  hipLaunchKernelGGL(round_scales_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, st, src, dst, n, sdt);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

bq_status launch_scales_to_wire(const float* src, void* dst, size_t n, int sdt, hipStream_t st) {
  if (n == 0) return BQ_OK;
  const dim3 grid(static_cast<unsigned>((n + 255) / 256));
  if (sdt == BQ_SCALE_UE4M3)
    hipLaunchKernelGGL(scales_to_wire_kernel<uint8_t>, grid, dim3(256), 0, st, src, static_cast<uint8_t*>(dst), n, sdt);
  else
    hipLaunchKernelGGL(scales_to_wire_kernel<uint16_t>, grid, dim3(256), 0, st, src, static_cast<uint16_t*>(dst), n, sdt);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

bq_status launch_scales_from_wire(const void* src, float* dst, size_t n, int sdt, hipStream_t st) {
  if (n == 0) return BQ_OK;
  const dim3 grid(static_cast<unsigned>((n + 255) / 256));
  if (sdt == BQ_SCALE_UE4M3)
    hipLaunchKernelGGL(scales_from_wire_kernel<uint8_t>, grid, dim3(256), 0, st, static_cast<const uint8_t*>(src), dst, n, sdt);
  else
    hipLaunchKernelGGL(scales_from_wire_kernel<uint16_t>, grid, dim3(256), 0, st, static_cast<const uint16_t*>(src), dst, n, sdt);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

}  // namespace bq

using namespace bq;

// Exhaustive on-device comparison of the divide-free shortcuts with the IEEE divisions they
// replace: every mantissa, every exponent of the range each shortcut is used for.
__global__ void selftest_division_kernel(unsigned long long* __restrict__ mismatches) {
  const uint32_t m = blockIdx.x * blockDim.x + threadIdx.x;
  if (m >= (1u << 23)) return;
  unsigned bad_r = 0, bad_8 = 0, bad_4 = 0;
  for (uint32_t ex = 27; ex <= 227; ++ex) {
    const float s = __uint_as_float((ex << 23) | m);
    bad_r += __float_as_uint(1.0f / s) != __float_as_uint(recip_exact(s));
  }
  for (uint32_t ex = 40; ex <= 220; ++ex) {
    const float a = __uint_as_float((ex << 23) | m);
    bad_8 += __float_as_uint((a * 2.0f) / 254.0f) != __float_as_uint(scale_from_absmax_fast<127>(a));
    bad_4 += __float_as_uint((a * 2.0f) / 14.0f) != __float_as_uint(scale_from_absmax_fast<7>(a));
  }
  if (bad_r) atomicAdd(mismatches + 0, static_cast<unsigned long long>(bad_r));
  if (bad_8) atomicAdd(mismatches + 1, static_cast<unsigned long long>(bad_8));
  if (bad_4) atomicAdd(mismatches + 2, static_cast<unsigned long long>(bad_4));
}

// The quotient shortcut x / s (div_by_recip) where a misrounding could change an integer: around
// every rounding tie. For every scale mantissa (at the lowest, the middle and the highest exponent
// the shortcut is taken for) and every k in [-128, 127]: x = RN((k + 1/2) * s) and its two
// neighbours on either side. Counter 3: quotients whose bits differ from the IEEE division;
// counter 4: quantized integers (clamped to +-127, rounded half away) that differ.
__global__ void selftest_quotient_kernel(unsigned long long* __restrict__ mismatches) {
  const uint32_t m = blockIdx.x * blockDim.x + threadIdx.x;
  if (m >= (1u << 23)) return;
  unsigned bad_q = 0, bad_i = 0;
  const uint32_t exps[3] = {27u, 127u, 227u};
  for (int e = 0; e < 3; ++e) {
    const float s = __uint_as_float((exps[e] << 23) | m);
    const float r = recip_exact(s);
    for (int k = -128; k <= 127; ++k) {
      const float tie = (static_cast<float>(k) + 0.5f) * s;
      const uint32_t tb = __float_as_uint(tie);
#pragma unroll
      for (int d = -2; d <= 2; ++d) {
        const float x = __uint_as_float(tb + static_cast<uint32_t>(d));  // neighbours in magnitude
        const float exact = x / s, fast = div_by_recip(x, s, r);
        bad_q += __float_as_uint(exact) != __float_as_uint(fast);
        bad_i += quantize_div(x, s, -127.0f, 127.0f) != quantize_recip(x, s, r, -127.0f, 127.0f);
      }
    }
  }
  if (bad_q) atomicAdd(mismatches + 3, static_cast<unsigned long long>(bad_q));
  if (bad_i) atomicAdd(mismatches + 4, static_cast<unsigned long long>(bad_i));
}

extern "C" bq_status bqk_selftest_division(uint64_t* mismatches_dev, void* stream) {
  BQ_NOTNULL(mismatches_dev);
  hipStream_t st = static_cast<hipStream_t>(stream);
  BQ_TRY(launch_fill_u32(reinterpret_cast<uint32_t*>(mismatches_dev), 10, 0u, st));
  hipLaunchKernelGGL(selftest_division_kernel, dim3((1u << 23) / 256), dim3(256), 0, st,
                     reinterpret_cast<unsigned long long*>(mismatches_dev));
  BQ_HIP(hipGetLastError());
  hipLaunchKernelGGL(selftest_quotient_kernel, dim3((1u << 23) / 256), dim3(256), 0, st,
                     reinterpret_cast<unsigned long long*>(mismatches_dev));
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

extern "C" bq_status bqk_absmax_f32(const float* x, size_t n, uint32_t* absmax_bits, void* stream) {
  BQ_NOTNULL(x);
  BQ_NOTNULL(absmax_bits);
  if (n == 0) return BQ_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (aligned16(x))
    hipLaunchKernelGGL(absmax_kernel, dim3(BQ_ABSMAX_CELLS), dim3(kThreads), 0, st, x, n, absmax_bits);
  else
    hipLaunchKernelGGL(absmax_scalar_kernel, dim3(BQ_ABSMAX_CELLS), dim3(kThreads), 0, st, x, n, absmax_bits);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

extern "C" bq_status bqk_scales_from_absmax(const float* absmax, size_t n, int32_t value,
                                            float* scales, void* stream) {
  BQ_NOTNULL(absmax);
  BQ_NOTNULL(scales);
  if (!value_known(value)) BQ_FAIL(BQ_ERR_UNSUPPORTED_SCHEME, "unknown quant value %d", value);
  if (n == 0) return BQ_OK;
  const float span = value_span(value);
  hipLaunchKernelGGL(scales_from_absmax_kernel, dim3((n + 255) / 256), dim3(256), 0,
                     static_cast<hipStream_t>(stream), absmax, n, span, scales);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

static bq_status check_value_store(int32_t value, int32_t store, size_t n) {
  // (2-bit values: the per-tensor kernel takes them packed; the block kernels do not)
  if (!value_supported(value)) BQ_FAIL(BQ_ERR_UNSUPPORTED_SCHEME, "unknown quant value %d", value);
  if (store == BQ_STORE_NATIVE) {
    if (value_bits(value) != 8)
      BQ_FAIL(BQ_ERR_UNSUPPORTED_SCHEME, "Can't store native sub-byte values");
  } else if (store == BQ_STORE_PACKED_U32) {
    if (n % static_cast<size_t>(num_quants(value)))
      BQ_FAIL(BQ_ERR_SHAPE, "Can't store in u32: %zu values, %d per word", n, num_quants(value));
  } else {
    BQ_FAIL(BQ_ERR_UNSUPPORTED_SCHEME, "unknown store %d", store);
  }
  return BQ_OK;
}

// Pass 2 of the per-tensor path. from_absmax: `scale` is the absmax cell and scale_out receives
// the derived scale (saves the separate scales_from_absmax launch in quantize_dynamic).
static bq_status quantize_per_tensor_impl(const float* x, size_t n, const float* scale,
                                          bool from_absmax, float* scale_out, int32_t value,
                                          int32_t store, void* values, int sdt, hipStream_t st) {
  BQ_TRY(check_value_store(value, store, n));
  if (n == 0) return BQ_OK;
  const bool full = value_full(value), eight = value_bits(value) == 8;
  if (!aligned16(x) || (reinterpret_cast<uintptr_t>(values) & 3u)) {
    if (!eight)
      BQ_FAIL(BQ_ERR_SHAPE, "4-bit quantize needs a 16-byte aligned input and 4-byte aligned output");
    if (from_absmax) {
      hipLaunchKernelGGL(scale_from_cells_kernel, dim3(1), dim3(kThreads), 0, st,
                         reinterpret_cast<const uint32_t*>(scale), value_span(value), sdt, scale_out);
      scale = scale_out;
    }
    hipLaunchKernelGGL(quantize_tensor_scalar_kernel, dim3(grid_for(n, 65536u)), dim3(kThreads), 0, st, x,
                       n, scale, static_cast<float>(value_qmin(value)), static_cast<int8_t*>(values));
    BQ_HIP(hipGetLastError());
    return BQ_OK;
  }
  const size_t vpl = static_cast<size_t>(num_quants(value));
  const size_t per_wg = static_cast<size_t>(kThreads) * kTensorUnroll;
  size_t g = (n / vpl + per_wg - 1) / per_wg;
  if (g < 1) g = 1;
  const int bits = value_bits(value);
  if (bits == 2 && store != BQ_STORE_PACKED_U32) BQ_FAIL(BQ_ERR_UNSUPPORTED_SCHEME, "2-bit values are quantized per tensor as packed words only");
  if (bits != 2)
    g = eight ? grid_back_to_front<pieces_per_chunk<4>(kThreads, kTensorUnroll)>(g) : grid_back_to_front<pieces_per_chunk<8>(kThreads, kTensorUnroll)>(g);
  if (g > 0x7FFFFFFFull) BQ_FAIL(BQ_ERR_SIZE, "quantize of %zu values exceeds the launch grid", n);
  dim3 grid(static_cast<unsigned>(g)), tb(kThreads);
  uint32_t* out = static_cast<uint32_t*>(values);
#define BQ_TENSOR(V, A, F) hipLaunchKernelGGL((quantize_tensor_kernel<V, A, F>), grid, tb, 0, st, x, n, scale, scale_out, out, sdt)
  if (eight) {
    if (from_absmax) { if (full) BQ_TENSOR(4, true, true); else BQ_TENSOR(4, true, false); }
    else { if (full) BQ_TENSOR(4, false, true); else BQ_TENSOR(4, false, false); }
  } else if (bits == 2 && !from_absmax && n / 4 + 1023 < 0x7FFFFFFFull * 1024ull) {
    hipLaunchKernelGGL(quantize_tensor_2bit_kernel, dim3(static_cast<unsigned>((n / 4 + 1023) / 1024)), dim3(256), 0, st, x, n, scale,
                       static_cast<float>(value_qmin(value)), out);
  } else if (bits == 2) {
    if (from_absmax) { if (full) BQ_TENSOR(16, true, true); else BQ_TENSOR(16, true, false); }
    else { if (full) BQ_TENSOR(16, false, true); else BQ_TENSOR(16, false, false); }
  } else {
    if (from_absmax) { if (full) BQ_TENSOR(8, true, true); else BQ_TENSOR(8, true, false); }
    else { if (full) BQ_TENSOR(8, false, true); else BQ_TENSOR(8, false, false); }
  }
#undef BQ_TENSOR
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

extern "C" bq_status bqk_quantize_per_tensor_from_absmax(const float* x, size_t n,
                                                         const uint32_t* absmax_cells,
                                                         float* scale_out, int32_t value,
                                                         int32_t store, void* values, void* stream) {
  BQ_NOTNULL(x);
  BQ_NOTNULL(absmax_cells);
  BQ_NOTNULL(scale_out);
  BQ_NOTNULL(values);
  return quantize_per_tensor_impl(x, n, reinterpret_cast<const float*>(absmax_cells), true, scale_out,
                                  value, store, values, BQ_SCALE_F32, static_cast<hipStream_t>(stream));
}

extern "C" bq_status bqk_quantize_per_tensor(const float* x, size_t n, const float* scale,
                                             int32_t value, int32_t store, void* values,
                                             void* stream) {
  BQ_NOTNULL(x);
  BQ_NOTNULL(scale);
  BQ_NOTNULL(values);
  return quantize_per_tensor_impl(x, n, scale, false, nullptr, value, store, values, BQ_SCALE_F32,
                                  static_cast<hipStream_t>(stream));
}

static bq_status check_block_args(const float* x, size_t n, int32_t block, int32_t value,
                                  int32_t store, const void* values) {
  BQ_TRY(check_value_store(value, store, n));
  if (block <= 0 || n % static_cast<size_t>(block))
    BQ_FAIL(BQ_ERR_SHAPE, "%zu values are not a whole number of blocks of %d", n, block);
  if (!fused_block_ok(block, value))
    BQ_FAIL(BQ_ERR_UNSUPPORTED_SCHEME,
            "run block %d: the fused kernel needs a power-of-two multiple of %d up to %d", block,
            num_quants(value), 64 * num_quants(value));
  if (!aligned16(x) || (reinterpret_cast<uintptr_t>(values) & 3u))
    BQ_FAIL(BQ_ERR_SHAPE, "block quantize needs a 16-byte aligned input and 4-byte aligned output");
  return BQ_OK;
}

// The run-block kernel for a value: 8- or 4-bit fields, symmetric or full range.
template <bool DYNAMIC, bool TWO = false>
static bq_status launch_block_for(int value, const float* x, size_t n, int block, uint32_t* out, float* scales_out,
                                  const float* scales_in, int sdt, hipStream_t st, float* stored_out = nullptr) {
  const bool full = value_full(value);
  if (value_bits(value) == 8)
    return full ? launch_block<4, DYNAMIC, TWO, true>(x, n, block, out, scales_out, scales_in, sdt, st, stored_out)
                : launch_block<4, DYNAMIC, TWO, false>(x, n, block, out, scales_out, scales_in, sdt, st, stored_out);
  return full ? launch_block<8, DYNAMIC, TWO, true>(x, n, block, out, scales_out, scales_in, sdt, st, stored_out)
              : launch_block<8, DYNAMIC, TWO, false>(x, n, block, out, scales_out, scales_in, sdt, st, stored_out);
}

extern "C" bq_status bqk_quantize_dynamic_block(const float* x, size_t n, int32_t block,
                                                int32_t value, int32_t store, void* values,
                                                float* scales, void* stream) {
  BQ_NOTNULL(x);
  BQ_NOTNULL(values);
  BQ_NOTNULL(scales);
  BQ_TRY(check_block_args(x, n, block, value, store, values));
  if (n == 0) return BQ_OK;
  return launch_block_for<true>(value, x, n, block, static_cast<uint32_t*>(values), scales, nullptr, BQ_SCALE_F32,
                                static_cast<hipStream_t>(stream));
}

extern "C" bq_status bqk_quantize_block(const float* x, size_t n, int32_t block,
                                        const float* scales, int32_t value, int32_t store,
                                        void* values, void* stream) {
  BQ_NOTNULL(x);
  BQ_NOTNULL(values);
  BQ_NOTNULL(scales);
  BQ_TRY(check_block_args(x, n, block, value, store, values));
  if (n == 0) return BQ_OK;
  return launch_block_for<false>(value, x, n, block, static_cast<uint32_t*>(values), nullptr, scales, BQ_SCALE_F32,
                                 static_cast<hipStream_t>(stream));
}


extern "C" bq_status bqk_copy(const void* src, void* dst, size_t bytes, void* stream) {
  BQ_NOTNULL(src);
  BQ_NOTNULL(dst);
  if (bytes % 16 || (reinterpret_cast<uintptr_t>(src) & 15u) || (reinterpret_cast<uintptr_t>(dst) & 15u))
    BQ_FAIL(BQ_ERR_SHAPE, "bqk_copy needs 16-byte aligned pointers and a multiple of 16 bytes");
  if (bytes == 0) return BQ_OK;
  const size_t chunks = bytes / 16;
  if ((chunks + 255) / 256 > 0x7FFFFFFFull) BQ_FAIL(BQ_ERR_SIZE, "bqk_copy: %zu bytes is more than one launch copies", bytes);
  hipLaunchKernelGGL(copy16_kernel, dim3(static_cast<unsigned>((chunks + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const vuint4*>(src),
                     static_cast<vuint4*>(dst), chunks);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

namespace bq {

// The handle level's entry into the fused kernels, with the scheme's scale dtype.
// quantize_dynamic per tensor in one launch, where the tensor is small enough (*done says whether it was):
// 8-bit values or packed 4-bit ones, a 16-byte aligned input, at most kSmallValues values.
bq_status launch_quantize_per_tensor_small(const float* x, size_t n, float* scale_out, int value, int store, void* values,
                                           int sdt, hipStream_t st, bool* done) {
  *done = false;
  const int bits = value_bits(value);
  if (n == 0 || n > kSmallValues || bits == 2 || (bits == 4 && store != BQ_STORE_PACKED_U32) || !aligned16(x) ||
      (reinterpret_cast<uintptr_t>(values) & 3u))
    return BQ_OK;
  BQ_TRY(check_value_store(value, store, n));
  const bool full = value_full(value);
  uint32_t* out = static_cast<uint32_t*>(values);
#define BQ_SMALL(V, F) hipLaunchKernelGGL((quantize_tensor_small_kernel<V, F>), dim3(1), dim3(kSmallThreads), 0, st, x, n, scale_out, out, sdt)
  if (bits == 8) { if (full) BQ_SMALL(4, true); else BQ_SMALL(4, false); }
  else { if (full) BQ_SMALL(8, true); else BQ_SMALL(8, false); }
#undef BQ_SMALL
  BQ_HIP(hipGetLastError());
  *done = true;
  return BQ_OK;
}

bq_status launch_quantize_per_tensor(const float* x, size_t n, const float* scale_or_cells, bool from_absmax,
                                     float* scale_out, int value, int store, void* values, int sdt, hipStream_t st) {
  return quantize_per_tensor_impl(x, n, scale_or_cells, from_absmax, scale_out, value, store, values, sdt, st);
}

bq_status launch_quantize_run_block(const float* x, size_t n, int block, const float* scales_in, float* scales_out,
                                    int value, int store, void* values, int sdt, hipStream_t st) {
  BQ_TRY(check_block_args(x, n, block, value, store, values));
  if (n == 0) return BQ_OK;
  uint32_t* out = static_cast<uint32_t*>(values);
  if (scales_in == nullptr) return launch_block_for<true>(value, x, n, block, out, scales_out, nullptr, sdt, st);
  return launch_block_for<false>(value, x, n, block, out, nullptr, scales_in, sdt, st);
}

// quantize_dynamic of a two-level run-block scheme in one pass over x, given the per-tensor scale.
bq_status launch_quantize_run_block_two_level(const float* x, size_t n, int block, const float* global, float* stored_out,
                                              float* scales_out, int value, int store, void* values, int sdt, hipStream_t st) {
  BQ_TRY(check_block_args(x, n, block, value, store, values));
  if (n == 0) return BQ_OK;
  return launch_block_for<true, true>(value, x, n, block, static_cast<uint32_t*>(values), scales_out, global, sdt, st,
                                      stored_out);
}

}  // namespace bq
