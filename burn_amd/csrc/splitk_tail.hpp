// One launch instead of two for the split-K q_matmul kernels: the workgroup that finishes last on
// a column tile adds up the K slices itself, in the order qgemv_reduce_kernel uses (bit-identical
// results), adds the bias and writes the output.
//
// Protocol, all at device ("agent") scope so that it does not matter which XCD a workgroup runs
// on (each XCD has its own L2; only device-scope accesses are coherent between them):
//   1. every thread writes its partial sums with device-scope stores (written through);
//   2. it waits until those stores are acknowledged (s_waitcnt), then the workgroup meets at a
//      barrier: all partials of this workgroup are visible device-wide;
//   3. one thread takes a ticket on the tile's counter with a device-scope atomic add;
//   4. the workgroup that draws the last ticket knows every other workgroup of the tile has passed
//      step 2; it reads all partials with device-scope loads (never served from a stale line),
//      sums them in the fixed order, and puts the counter back to zero for the next launch.
// No wave ever waits for another workgroup: a workgroup that is not last simply leaves.
// The counters are `kTicketStride` words apart (one 128-byte line each) in memory that is zero
// before the first launch; every launch leaves them zero. Launches that share the counters must
// not overlap on the device (one stream, or one call at a time).
#pragma once

#include "common.hpp"
#include "device_math.hpp"

namespace bq {

// cache-policy operand of the raw buffer intrinsics: bit 4 = sc1, device scope on gfx950
constexpr int kDeviceScope = 16;

__device__ __forceinline__ __amdgpu_buffer_rsrc_t partials_rsrc(float* part, size_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(part, 0, static_cast<int>(bytes), 0x00020000);
}

// Steps 2-4. `part` holds slices x [M, N] floats (byte size below 2^31); this workgroup's tile is
// columns [col0, col0 + cols) of every row, cols a multiple of 4, N a multiple of 4. Called by all
// THREADS threads of the workgroup, after their partial stores (step 1).
template <int THREADS>
__device__ __forceinline__ void splitk_reduce_tail(float* part, unsigned* ticket, unsigned slices, size_t M, size_t N,
                                                   size_t col0, unsigned cols, const float* __restrict__ bias, bool out_bf16,
                                                   void* __restrict__ out) {
  __shared__ unsigned drawn;
  __builtin_amdgcn_s_waitcnt(0);  // this thread's partial stores have been acknowledged
  asm volatile("" ::: "memory");
  __syncthreads();
  if (threadIdx.x == 0) drawn = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  if (drawn != slices - 1u) return;
  asm volatile("" ::: "memory");
  if (threadIdx.x == 0) __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const __amdgpu_buffer_rsrc_t rsrc = partials_rsrc(part, static_cast<size_t>(slices) * M * N * sizeof(float));
  const size_t mn = M * N;
  const unsigned vecs = cols / 4u;
  const int SL = slices >= 16u ? 16 : (slices >= 8u ? 8 : 4);  // qgemv_reduce_kernel's slice lanes
  for (unsigned idx = threadIdx.x; idx < static_cast<unsigned>(M) * vecs; idx += THREADS) {
    const unsigned row = idx / vecs, c4 = (idx % vecs) * 4u;
    const size_t col = col0 + c4;
    if (col >= N) continue;
    const size_t at = static_cast<size_t>(row) * N + col;  // element index inside one slice
    // qgemv_reduce_kernel's order: sub[t] = 0 + slices t, t + SL, ... in ascending order; then
    // sub[0] + sub[1] + ... + sub[SL - 1].
    vfloat4 v;
    if (slices <= static_cast<unsigned>(SL)) {
      // every sub[t] is one partial (or zero): the sum is the plain ascending one, all loads in flight at once
      // (lane offset = the element, scalar offset = the slice; a slice past the end re-reads the last one and is not added)
      vuint4 p[16];
      const uint32_t lane_off = static_cast<uint32_t>(at * sizeof(float)), slice_bytes = static_cast<uint32_t>(mn * sizeof(float));
#pragma unroll
      for (int t = 0; t < 16; ++t) {
        const unsigned s = static_cast<unsigned>(t) < slices ? static_cast<unsigned>(t) : slices - 1u;
        p[t] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane_off, s * slice_bytes, kDeviceScope);
      }
      v = vfloat4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int t = 0; t < 16; ++t)
        if (static_cast<unsigned>(t) < slices) v += __builtin_bit_cast(vfloat4, p[t]);
      // (the reference order also adds the empty sub-sums, + 0.0f each: they change no bits of a sum that started from + 0.0f)
    } else {
      vfloat4 sub[16];
#pragma unroll
      for (int t = 0; t < 16; ++t) sub[t] = vfloat4{0.f, 0.f, 0.f, 0.f};
      for (unsigned s0 = 0; s0 < slices; s0 += static_cast<unsigned>(SL)) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {   // 4 loads in flight at a time: this path is rare, registers are not
          if (q * 4 >= SL) break;
          vuint4 p[4];
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const unsigned s = s0 + static_cast<unsigned>(q * 4 + t);
            const unsigned se = s < slices ? s : slices - 1u;
            p[t] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, static_cast<uint32_t>(at * sizeof(float)),
                                                         se * static_cast<uint32_t>(mn * sizeof(float)), kDeviceScope);
          }
#pragma unroll
          for (int t = 0; t < 4; ++t)
            if (s0 + static_cast<unsigned>(q * 4 + t) < slices) sub[q * 4 + t] += __builtin_bit_cast(vfloat4, p[t]);
        }
      }
      v = sub[0];
#pragma unroll
      for (int t = 1; t < 16; ++t)
        if (t < SL) v += sub[t];
    }
    if (bias != nullptr) v += *reinterpret_cast<const vfloat4*>(bias + col);
    if (!out_bf16) {
      *reinterpret_cast<vfloat4*>(static_cast<float*>(out) + at) = v;
    } else {
      vuint2 h = {f32x2_to_bf16x2(v.x, v.y), f32x2_to_bf16x2(v.z, v.w)};
      // (NaN payloads: f32_to_bf16 sets the quiet bit; the packed convert gives the same bits for every other input)
      if (v.x != v.x || v.y != v.y || v.z != v.z || v.w != v.w)
        h = vuint2{static_cast<uint32_t>(f32_to_bf16(v.x)) | static_cast<uint32_t>(f32_to_bf16(v.y)) << 16,
                   static_cast<uint32_t>(f32_to_bf16(v.z)) | static_cast<uint32_t>(f32_to_bf16(v.w)) << 16};
      *reinterpret_cast<vuint2*>(static_cast<uint16_t*>(out) + at) = h;
    }
  }
}

}  // namespace bq
