// Small-batch q_matmul on the bf16 matrix cores (gfx950) at better than bf16 accuracy, M <= 32:
// out[M,N] = X[M,K] x dequantize(W[K,N]), X f32 or bf16, W 8- or 4-bit with one scale per 32, 64
// or 128 columns (or per tensor).
//
// Same operation as the other q_matmul kernels (QTensorOps::q_matmul,
// crates/burn-backend/src/backend/ops/qtensor.rs:498-544; reference path
// crates/burn-ndarray/src/ops/qtensor.rs:223-267). The weights are streamed once from HBM, which
// is the bound; M fused multiply-adds per weight are too many for the vector ALU, and the FP32
// matrix pipe needs longer for them than HBM needs for the weights. So the products run on
// v_mfma_f32_16x16x32_bf16 without giving up the f32 activations:
//   * the integer weights are exact in bf16 (8 significant bits): they are converted, never rounded;
//   * the scale goes to the activations: xs[m][k] = X[m][k] * s[k][block], in f32, once per
//     (k, block of 32 columns), and xs is split into two bf16 terms hi + lo (16 significant bits:
//     a product is off by at most 2^-17 of its value, against 2^-9 for a bf16 rounding);
//   * out[m][n] = sum_k (hi + lo)[m][k] * q[k][n], accumulated in f32.
// One MFMA multiplies 16 activation rows by 16 columns that share their scales: for Q8S 8 packed
// words x 2 of their 4 byte fields, for Q4S 4 words x 4 of their 8 nibbles. A lane (c = lane %
// 16, kg = lane / 16) holds, for both operands, the 8 consecutive k rows 8 kg .. 8 kg + 7 of a
// 32-row step: as A operand the split xs of row m = c, as B operand one column of word c % 8
// (c % 4), field c / 8 (c / 4) in the first MFMA and that plus half the fields in the second.
// Q8S: the per-lane field choice is made by v_perm_b32 with a per-lane selector, which gathers
// the two fields of two rows into one register; sign-extending byte converts (SDWA) and a second
// v_perm_b32 (the upper halves of two floats are their bf16) finish the operand. Q4S: a per-lane
// rotation brings the lane's two nibbles to bits 3..6 of each 16-bit half, and and + xor turn
// them into the bf16 bit patterns 0x4180 | (nibble ^ 8) << 3 = 16 + (q + 8) = q + 24 (the nibble
// in the upper 4 of the 7 mantissa bits: exact); the 24 comes off through two more MFMAs per
// distinct A operand against a constant -24 operand, into an accumulator of their own that is
// added when the tile is stored (every column of it holds 24 times the sum of the row's
// activations). With the 0x4300 | (nibble ^ 8) = q + 136 patterns and the correction taken in
// every accumulator, the same kernels measured 1-4 us more and an error of 3.5e-6 to 7e-6 of
// the largest output instead of 2.9e-6 to 4.9e-6.
//
// A wave owns 4 adjacent blocks (128 columns: a row is 128 bytes of Q8S or 64 of Q4S) and a run
// of k rows; the 8 waves of a workgroup are 4 such column groups x 2 halves of the workgroup's K
// slice, whose activations sit in LDS. The weights are loaded as whole rows (16 bytes per lane)
// and handed to the lanes that multiply them through a small LDS slot private to the wave --
// unless any 16 columns of the group can share an A operand (per-tensor scales, or M <= 4 with
// the rows packed as below): then lane c loads the 8 columns 8 c .. 8 c + 7 of its own 8 k rows
// (8 or 4 bytes per row) and multiplies them straight from the registers, MFMA j taking column j
// of every lane. The two halves are added through LDS, the K slices by qgemv_reduce_kernel,
// both in a fixed order (no float atomics).
#include <algorithm>
#include <type_traits>

#include "common.hpp"
#include "device_math.hpp"

namespace bq {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));

constexpr int kGroups = 4;                          // waves across N
constexpr int kKWays = 2;                           // waves across K
constexpr int kSplitWaves = kGroups * kKWays;
constexpr int kSplitThreads = kSplitWaves * kWave;  // 512
constexpr int kUnits = 4;                           // blocks of 32 columns per wave
constexpr int kStepRows = 32;                       // k rows per MFMA
// steps of loads in flight per wave (3 and 4 were slower by 1.5 and 2 us: the burst of first loads
// is that much larger, and every wave's first step arrives behind all of it)
constexpr int kDepth = 2;
constexpr int kGroupCols = kUnits * 32;             // 128
constexpr int kTileCols = kGroups * kGroupCols;     // 512 columns per workgroup
constexpr int kMaxSlice = 512;                      // k rows per workgroup (activations in LDS: 16 x 516 floats)
constexpr int kSlotBytes = kStepRows * kGroupCols;   // one step of a wave's weights: 32 rows x 128 bytes
static_assert(kTileCols <= kMaxSlice, "the output tile is staged where the activation slice was");
// the largest request (two row tiles) must fit the 160 KiB of a CU
static_assert(16 * 2 * (kMaxSlice + 4) * 4 + kSplitWaves * kSlotBytes <= 160 * 1024, "LDS of the largest workgroup");
constexpr int kFillVecs = 16 * kMaxSlice / 4 / kSplitThreads;  // 16-byte loads per thread that fill the slice

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2{lo, hi}, bf16x2));
}
__device__ __forceinline__ float as_float(uint32_t v) { return __builtin_bit_cast(float, v); }
__device__ __forceinline__ uint32_t as_bits(float v) { return __builtin_bit_cast(uint32_t, v); }
__device__ __forceinline__ float byte_to_float(uint32_t v, int byte) {  // signed byte -> f32 (one SDWA convert)
  return static_cast<float>(static_cast<int>(static_cast<int8_t>(v >> (8 * byte))));
}

// The value lane R of the caller's row of 16 lanes holds (DPP row_newbcast:R).
template <int R>
__device__ __forceinline__ float row_lane(uint32_t v) {
  return as_float(static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), 0x150 + R, 0xF, 0xF, false)));
}
// The value lane R of the caller's quad of 4 lanes holds (DPP quad_perm:[R,R,R,R]).
template <int R>
__device__ __forceinline__ float quad_lane(uint32_t v) {
  return as_float(static_cast<uint32_t>(__builtin_amdgcn_update_dpp(0, static_cast<int>(v), R * 0x55, 0xF, 0xF, false)));
}

// MT: tiles of 16 activation rows (1 or 2): a lane prepares the split activations of rows c and
// c + 16 and multiplies both against the same weight operands.
// SB: log2 of (scale block / 32 columns): a scale serves 1, 2 or 4 of a wave's blocks of 32 columns.
// PK (M <= 4, one scale per 32 columns): the 16 rows of the A operand are 4 activation rows x the
// wave's 4 blocks of 32 columns -- lane c prepares row c % 4 against the scales of block c / 4 -- so
// the split activations are computed once per step instead of once per block (they are most of the
// vector-ALU work: 32 of 60 instructions per 1024 weights). Every MFMA of the wave then takes the
// same A operand, and of a column's 16 accumulator rows only the 4 of its own block b (rows 4 b ..
// 4 b + 3, held by the lanes with kg == b) are its product; the others multiply another block's
// scales and are dropped.
// DL (PK or PER_TENSOR): direct loads, no LDS slot. With the slot, the 16 columns of an MFMA must
// lie in one scale block, which fixes which word a lane needs; here every column of the group
// meets the same A operand (PK: its block's scales are rows 4 b .. 4 b + 3 of it), so a lane can
// multiply whatever columns it loaded. Measured on the 4096 x 14336 weight, whole product: Q8S
// block-32 M = 4 20.9 -> 20.1 us, per-tensor M = 4 / 16 / 32 20.0 / 21.3 / 27.1 -> 18.2 / 20.3 /
// 26.2 us; Q4S block-32 M = 3 / 4 18.6 / 19.5 -> 17.1 / 17.7 us.
template <int VPL, bool PER_TENSOR, bool X_BF16, int MT, int SB = 0, bool PK = false, bool DL = false>
__global__ void __launch_bounds__(kSplitThreads)
qsplit_kernel(const void* __restrict__ x, const uint32_t* __restrict__ w, const float* __restrict__ scales,
              size_t M, size_t K, size_t N, size_t k_per_wg, unsigned tiles, unsigned slices, float* __restrict__ part) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  // Workgroup -> (column tile, K slice). Workgroups reach the 8 XCDs round robin (workgroup b runs
  // on XCD b % 8) and each XCD has its own L2. A 128-byte line of scales serves kBundle adjacent
  // column tiles of one K slice: those tiles are given to consecutive workgroups of ONE XCD, so the
  // line comes from HBM once instead of once per XCD that holds one of its tiles (with the plain
  // (tile, slice) grid, neighbouring tiles sat on neighbouring XCDs and the scales were read twice:
  // 1.12 to 1.15 times the weights' bytes by the counters).
  constexpr unsigned kBundle = PER_TENSOR ? 1u : (2u << SB);
  unsigned tile_id, slice_id;
  {
    const unsigned b = blockIdx.x, xcd = b % 8u, local = b / 8u;
    const unsigned bundles = (tiles + kBundle - 1u) / kBundle;
    const unsigned unit = xcd + 8u * (local / kBundle);
    tile_id = (unit % bundles) * kBundle + local % kBundle;
    slice_id = unit / bundles;
    if (slice_id >= slices || tile_id >= tiles) return;  // padding of the grid (whole workgroup)
  }
  // Activation slice as [16 rows][k_per_wg + 4] f32: the pitch is 4 floats past a multiple of 64,
  // so the 16 rows read by a quarter wave (16 bytes each) fall into distinct banks. The same
  // memory carries the cross-wave sum afterwards.
  float* const xs = reinterpret_cast<float*>(smem);
  const uint32_t xpitch = static_cast<uint32_t>(k_per_wg) + 4u;
  constexpr uint32_t slot_base = 16u * MT * (kMaxSlice + 4) * 4u;  // the waves' slots follow the slice / the output tile

  constexpr int WPB = 32 / VPL;              // packed words per block of 32 columns: 8 (Q8S) or 4 (Q4S)
  constexpr uint32_t ROW_B = kUnits * WPB * 4;  // bytes of a weight row a wave owns: 128 or 64
  constexpr int LPR = ROW_B / 16;            // lanes (16-byte chunks) per row of a load instruction
  constexpr int RPI = kWave / LPR;           // rows per load instruction: 8 or 16
  constexpr int NLOAD = kStepRows / RPI;     // load instructions per step: 4 or 2
  constexpr uint32_t ROT = ROW_B / 4;        // slot rotation per 8 rows
  // Two measured choices for Q8S (the Q4S kernels move half the bytes and gain nothing from either):
  // the first weight loads wait for the activations, and a wave's priority falls with its progress.
  constexpr bool kLateFetch = VPL == 4;
  constexpr bool kProgressPriority = VPL == 4;
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int c = lane & 15, kg = lane >> 4;
  const int g = wave % kGroups, h = wave / kGroups;
  const size_t NW = N / VPL, spr = N / (32u << SB), groups_total = N / kGroupCols;
  const size_t group = static_cast<size_t>(tile_id) * kGroups + g;
  const bool live = group < groups_total;  // the last tile may hold fewer than 4 groups: the spare
  const size_t gc = live ? group : groups_total - 1;  // waves redo the last one and store nothing

  const size_t k_begin = static_cast<size_t>(slice_id) * k_per_wg;
  const uint32_t k_per_way = static_cast<uint32_t>(k_per_wg) / kKWays;
  const size_t kw0 = k_begin + static_cast<size_t>(h) * k_per_way;  // first row of this wave
  const int steps = kw0 < K ? static_cast<int>((K - kw0 < k_per_way ? K - kw0 : k_per_way) / kStepRows) : 0;

  // Buffer loads: lane offset + scalar offset (row of the step). Offsets are below 2^31 (checked
  // by the host). Weights: a load instruction reads whole rows of the group (Q8S: 8 rows of 128
  // bytes, lane l row l / 8, 16-byte chunk l % 8, 4 instructions a step; Q4S: 16 rows of 64
  // bytes, 2 instructions). They go through an LDS slot private to the wave, where lane (c, kg)
  // picks up the words it multiplies: with one word per lane and load, a wave could not keep
  // enough loads in flight (the counter they are waited on holds 63). Row r of a slot is rotated
  // by ROT (r / 8) bytes: the 4 kg groups of a read then fall into distinct banks.
  const __amdgpu_buffer_rsrc_t rsrc_w =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint32_t*>(w), 0, static_cast<int>(K * NW * 4), 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_s = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(scales), 0, static_cast<int>(PER_TENSOR ? 4 : K * spr * 4), 0x00020000);
  const uint32_t w_row_bytes = static_cast<uint32_t>(NW * 4), s_row_bytes = static_cast<uint32_t>(spr * 4);
  static_assert(DL == (PK || PER_TENSOR), "direct loads exactly where any 16 columns of the group share their activations");
  const uint32_t w_lane = DL ? static_cast<uint32_t>(8 * kg) * w_row_bytes + static_cast<uint32_t>(gc) * ROW_B + static_cast<uint32_t>(c) * (ROW_B / 16)
                             : static_cast<uint32_t>(lane / LPR) * w_row_bytes + static_cast<uint32_t>(gc) * ROW_B +
                                   static_cast<uint32_t>(lane % LPR) * 16u;
  static_assert(!PK || (MT == 1 && SB == 0 && !PER_TENSOR), "row packing: one tile of rows, one scale per 32 columns");
  // PK: lane (row c % 4, block c / 4) loads that block's scale for k rows 8 kg + c % 4 and + 4
  const uint32_t s_lane = PK ? static_cast<uint32_t>(8 * kg + (c & 3)) * s_row_bytes + static_cast<uint32_t>(gc * 4 + (c >> 2)) * 4u
                             : static_cast<uint32_t>(8 * kg + (c & 7)) * s_row_bytes + static_cast<uint32_t>(gc * (4 >> SB)) * 4u;
  unsigned char* const slot = smem + slot_base + static_cast<uint32_t>(wave) * kSlotBytes;
  uint32_t slot_wr[NLOAD], slot_rd[kUnits];  // byte offsets in the slot: store i of a step; unit u, row 8 kg
#pragma unroll
  for (int i = 0; i < NLOAD; ++i) {
    const uint32_t row = static_cast<uint32_t>(lane / LPR + RPI * i);
    slot_wr[i] = row * ROW_B + ((static_cast<uint32_t>(lane % LPR) * 16u + ROT * (row >> 3)) & (ROW_B - 1u));
  }
#pragma unroll
  for (int u = 0; u < kUnits; ++u)
    slot_rd[u] = static_cast<uint32_t>(8 * kg) * ROW_B + ((4u * WPB * u + 4u * (c % WPB) + ROT * kg) & (ROW_B - 1u));
  const float s_tensor = PER_TENSOR ? scales[0] : 0.0f;
  // Q8S: v_perm_b32 selector: bytes (f0 of row a, f0 of row b, f0 + 2 of row a, f0 + 2 of row b).
  // Q4S: the lane's two nibbles f0 and f0 + 4 of a word are 16 bits apart: one shift by 4 f0
  // brings them to the low nibble of each half (guarded loop), one rotation to bits 3..6.
  const uint32_t f0 = static_cast<uint32_t>(c / WPB);
  const uint32_t sel = f0 | ((4u + f0) << 8) | ((f0 + 2u) << 16) | ((6u + f0) << 24);
  const uint32_t nib_shift = 4u * f0;
  const uint32_t nib_rot = (4u * f0 + 29u) & 31u;  // rotate right: nibble f0 to bits 3..6, nibble f0 + 4 to bits 19..22

  floatx4 acc[MT][kUnits][2];
  // Q4S: the offset of the weight patterns times the sum of the activations, one accumulator per
  // distinct A operand (every column of it holds the same value)
  constexpr bool kSharedA = PK || PER_TENSOR;  // the wave's 4 units multiply the same A operand
  constexpr int kOffsetAccs = kSharedA ? 1 : kUnits;
  floatx4 off[MT][kOffsetAccs];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
#pragma unroll
    for (int u = 0; u < kUnits; ++u) acc[t][u][0] = acc[t][u][1] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < kOffsetAccs; ++u) off[t][u] = floatx4{0.f, 0.f, 0.f, 0.f};
  }

  // kDepth steps are in flight per wave. Scales: lane (c, kg) loads those of row 8 kg + c % 8 (four
  // blocks, 16 bytes); the multiply reads row r's from lane r of its row of 16 lanes (DPP broadcast).
  vuint4 wl[kDepth][NLOAD];
  vuint2 wd[kDepth][8];
  vuint4 sq[kDepth];
  // A step past the end of the wave's rows loads nothing: its lane offsets are out of the buffers'
  // range, so the loads return zeros without touching memory. Every fetch and multiply then runs
  // unconditionally, in one basic block per loop trip, and the compiler can count exactly how
  // many younger loads are in flight when it waits for a step's registers (with branches around
  // them it has to assume none and drains the whole pipeline at every step).
  auto fetch = [&](int buf, int s) {
    const bool ok = s < steps;
    const uint32_t row0 = ok ? static_cast<uint32_t>(kw0) + static_cast<uint32_t>(s) * kStepRows : 0u;
    const uint32_t wo = ok ? w_lane : 0x80000000u, so = ok ? s_lane : 0x80000000u;
    if (DL) {
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        const uint32_t row = (row0 + static_cast<uint32_t>(r)) * w_row_bytes;
        if (VPL == 4) wd[buf][r] = __builtin_amdgcn_raw_buffer_load_b64(rsrc_w, wo, row, 0);
        else wd[buf][r] = vuint2{__builtin_amdgcn_raw_buffer_load_b32(rsrc_w, wo, row, 0), 0u};
      }
    } else {
#pragma unroll
      for (int i = 0; i < NLOAD; ++i)
        wl[buf][i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, wo, (row0 + static_cast<uint32_t>(RPI * i)) * w_row_bytes, 0);
    }
    if (PK) {
      sq[buf] = vuint4{__builtin_amdgcn_raw_buffer_load_b32(rsrc_s, so, row0 * s_row_bytes, 0),
                       __builtin_amdgcn_raw_buffer_load_b32(rsrc_s, so, (row0 + 4u) * s_row_bytes, 0), 0u, 0u};
    } else if (!PER_TENSOR) {  // the 4, 2 or 1 scales of the group's row
      if (SB == 0) {
        sq[buf] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_s, so, row0 * s_row_bytes, 0);
      } else if (SB == 1) {
        const vuint2 t = __builtin_amdgcn_raw_buffer_load_b64(rsrc_s, so, row0 * s_row_bytes, 0);
        sq[buf] = vuint4{t.x, t.y, 0u, 0u};
      } else {
        sq[buf] = vuint4{__builtin_amdgcn_raw_buffer_load_b32(rsrc_s, so, row0 * s_row_bytes, 0), 0u, 0u, 0u};
      }
    }
  };
  // G (a std::bool_constant): the guarded variant, taken only by workgroups whose activation slice
  // holds an infinity or a NaN. There the second term of a non-finite product is dropped (inf - inf
  // would make every output of the row NaN, where the reference's sum has +-inf, and NaN only
  // against a zero weight), Q4S weights are converted to their true values instead of the offset
  // patterns (inf * (q + 24) - inf * 24 is NaN), and the padded step past the end is skipped
  // (inf * 0). Finite slices never execute any of it.
  // (-1, 0) and (0, -1) as bf16 pairs, kept in registers the compiler cannot see through: written
  // as constants, (-1, 0) becomes the inline operand -1.0, which this instruction reads as the 32-bit
  // float -- the pair (0, -1).
  uint32_t minus_lo = 0x0000BF80u, minus_hi = 0xBF800000u;
  asm volatile("" : "+s"(minus_lo), "+s"(minus_hi));
  auto split = [&](auto G, const float* t, uint32_t* hi, uint32_t* lo) {
    constexpr bool guard = decltype(G)::value;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      hi[i] = pack_bf16(t[2 * i], t[2 * i + 1]);
      float d0, d1;
      if (guard) {
        const float h0 = as_float(hi[i] << 16), h1 = as_float(hi[i] & 0xFFFF0000u);
        d0 = (as_bits(h0) & 0x7F800000u) == 0x7F800000u ? 0.0f : t[2 * i] - h0;
        d1 = (as_bits(h1) & 0x7F800000u) == 0x7F800000u ? 0.0f : t[2 * i + 1] - h1;
      } else {
        // t - hi straight from the packed pair: v_dot2_f32_bf16 against (-1, 0) and (0, -1) adds
        // -hi to t in one instruction each (the difference has at most 16 significant bits, so
        // it is exact), where unpacking the halves first costs a shift and a mask more per pair
        const bf16x2 h = __builtin_bit_cast(bf16x2, hi[i]);
        d0 = __builtin_amdgcn_fdot2_f32_bf16(h, __builtin_bit_cast(bf16x2, minus_lo), t[2 * i], false);
        d1 = __builtin_amdgcn_fdot2_f32_bf16(h, __builtin_bit_cast(bf16x2, minus_hi), t[2 * i + 1], false);
      }
      lo[i] = pack_bf16(d0, d1);
    }
  };
  auto multiply = [&](auto G, int buf, int s) {
    constexpr bool guard = decltype(G)::value;
    const int sx = s < steps ? s : 0;  // past the end the weights are zeros: any finite activations do
    const uint32_t kl = static_cast<uint32_t>(h) * k_per_way + static_cast<uint32_t>(sx) * kStepRows + 8u * kg;
    float xv[MT][8];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const vfloat4* xp = reinterpret_cast<const vfloat4*>(xs + ((PK ? (c & 3) : c) + 16 * t) * xpitch + kl);
      const vfloat4 x0 = xp[0], x1 = xp[1];
      xv[t][0] = x0.x; xv[t][1] = x0.y; xv[t][2] = x0.z; xv[t][3] = x0.w;
      xv[t][4] = x1.x; xv[t][5] = x1.y; xv[t][6] = x1.z; xv[t][7] = x1.w;
    }
    // through the wave's slot (LDS runs a wave's instructions in order: no barrier)
    if (!DL) {
#pragma unroll
      for (int i = 0; i < NLOAD; ++i) *reinterpret_cast<vuint4*>(slot + slot_wr[i]) = wl[buf][i];
    }
    const vuint4 sqv = sq[buf];
    uint32_t wq[kUnits][8];
#pragma unroll
    for (int u = 0; u < kUnits; ++u)
#pragma unroll
      for (int r = 0; r < 8; ++r)
        wq[u][r] = DL ? (VPL == 4 && u >> 1 ? wd[buf][r].y : wd[buf][r].x) : *reinterpret_cast<const uint32_t*>(slot + slot_rd[u] + ROW_B * r);
    uint32_t hi[MT][4], lo[MT][4];
    if (PK) {
      const uint32_t a = sqv.x, b = sqv.y;
      const float sr[8] = {quad_lane<0>(a), quad_lane<1>(a), quad_lane<2>(a), quad_lane<3>(a),
                           quad_lane<0>(b), quad_lane<1>(b), quad_lane<2>(b), quad_lane<3>(b)};
      float v[8];
#pragma unroll
      for (int r = 0; r < 8; ++r) v[r] = xv[0][r] * sr[r];
      split(G, v, hi[0], lo[0]);
    }
    if (PER_TENSOR) {
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        float v[8];
#pragma unroll
        for (int r = 0; r < 8; ++r) v[r] = xv[t][r] * (s < steps ? s_tensor : 0.0f);
        split(G, v, hi[t], lo[t]);
      }
    }
    // Q4S with direct loads: the lane's word of a row holds its 8 columns, one nibble each, and all
    // 4 units read the same words. Two byte permutes gather bytes 0, 2 (nibbles 0, 1, 4, 5) and
    // bytes 1, 3 (nibbles 2, 3, 6, 7) of two rows; after one xor (n ^ 8 in every nibble) a shift and
    // an and-or leave, per unit, the 4 bytes 0x80 | (n ^ 8) << 3 of (row a, row b) x (nibble u,
    // nibble u + 4): the low bytes of the bf16 patterns 0x4180 | (n ^ 8) << 3 = 16 + (q + 8) = q + 24.
    uint32_t nlo[4][kUnits];
    if (VPL == 8 && DL && !guard) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t wa = wd[buf][2 * i].x, wb = wd[buf][2 * i + 1].x;
        const uint32_t p01 = __builtin_amdgcn_perm(wb, wa, 0x06020400u) ^ 0x88888888u;
        const uint32_t p23 = __builtin_amdgcn_perm(wb, wa, 0x07030501u) ^ 0x88888888u;
        nlo[i][0] = ((p01 << 3) & 0x78787878u) | 0x80808080u;
        nlo[i][1] = ((p01 >> 1) & 0x78787878u) | 0x80808080u;
        nlo[i][2] = ((p23 << 3) & 0x78787878u) | 0x80808080u;
        nlo[i][3] = ((p23 >> 1) & 0x78787878u) | 0x80808080u;
      }
    }
    // the offset comes off through two MFMAs per distinct A operand against a constant -24
    const bf16x8 minus = __builtin_bit_cast(bf16x8, vuint4{0xC1C0C1C0u, 0xC1C0C1C0u, 0xC1C0C1C0u, 0xC1C0C1C0u});
    auto take_offset = [&](int u) {
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const bf16x8 a_hi = __builtin_bit_cast(bf16x8, vuint4{hi[t][0], hi[t][1], hi[t][2], hi[t][3]});
        const bf16x8 a_lo = __builtin_bit_cast(bf16x8, vuint4{lo[t][0], lo[t][1], lo[t][2], lo[t][3]});
        off[t][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi, minus, off[t][u], 0, 0, 0);
        off[t][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_lo, minus, off[t][u], 0, 0, 0);
      }
    };
    if (VPL == 8 && !guard && kSharedA) take_offset(0);
#pragma unroll
    for (int u = 0; u < kUnits; ++u) {
      if (!PER_TENSOR && !PK) {
        const uint32_t sv = sqv[u >> SB];
        const float sr[8] = {row_lane<0>(sv), row_lane<1>(sv), row_lane<2>(sv), row_lane<3>(sv),
                             row_lane<4>(sv), row_lane<5>(sv), row_lane<6>(sv), row_lane<7>(sv)};
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          float v[8];
#pragma unroll
          for (int r = 0; r < 8; ++r) v[r] = xv[t][r] * sr[r];
          split(G, v, hi[t], lo[t]);
        }
        if (VPL == 8 && !guard) take_offset(u);
      }
      uint32_t b0[4], b1[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (VPL == 4) {
          // DL: unit u multiplies bytes u % 2 and u % 2 + 2 of word u / 2 of the lane's 8 bytes
          const uint32_t p = __builtin_amdgcn_perm(wq[u][2 * i + 1], wq[u][2 * i], DL ? (u & 1 ? 0x07030501u : 0x06020400u) : sel);
          b0[i] = __builtin_amdgcn_perm(as_bits(byte_to_float(p, 1)), as_bits(byte_to_float(p, 0)), 0x07060302u);
          b1[i] = __builtin_amdgcn_perm(as_bits(byte_to_float(p, 3)), as_bits(byte_to_float(p, 2)), 0x07060302u);
        } else if (guard) {
          // the nibbles' own values (q = (n ^ 8) - 8, exact in bf16: the upper half of the f32)
          const uint32_t na = (wq[u][2 * i] >> (DL ? 4u * u : nib_shift)) & 0x000F000Fu, nb = (wq[u][2 * i + 1] >> (DL ? 4u * u : nib_shift)) & 0x000F000Fu;
          auto qf = [](uint32_t n) { return as_bits(static_cast<float>(static_cast<int>(n ^ 8u) - 8)); };
          b0[i] = __builtin_amdgcn_perm(qf(nb & 0xFu), qf(na & 0xFu), 0x07060302u);
          b1[i] = __builtin_amdgcn_perm(qf(nb >> 16), qf(na >> 16), 0x07060302u);
        } else if (DL) {
          // low bytes from above under the constant high byte 0x41: (row a, row b) of nibble u, of nibble u + 4
          b0[i] = __builtin_amdgcn_perm(0x41414141u, nlo[i][u], 0x04010400u);
          b1[i] = __builtin_amdgcn_perm(0x41414141u, nlo[i][u], 0x04030402u);
        } else {
          // the same pattern from the lane's own word of the unit: a rotation brings its nibbles f0
          // and f0 + 4 (16 bits apart) to bits 3..6 of each half, and and + xor finish both at once.
          // (Gathering the bytes of two rows first, as above, saves two instructions per pair here
          // too and was not faster: 22.3 against 21.8 us at M = 16.)
          const uint32_t ta = (__builtin_amdgcn_alignbit(wq[u][2 * i], wq[u][2 * i], nib_rot) & 0x00780078u) ^ 0x41C041C0u;
          const uint32_t tb = (__builtin_amdgcn_alignbit(wq[u][2 * i + 1], wq[u][2 * i + 1], nib_rot) & 0x00780078u) ^ 0x41C041C0u;
          b0[i] = __builtin_amdgcn_perm(tb, ta, 0x05040100u);
          b1[i] = __builtin_amdgcn_perm(tb, ta, 0x07060302u);
        }
      }
      const bf16x8 bq0 = __builtin_bit_cast(bf16x8, vuint4{b0[0], b0[1], b0[2], b0[3]});
      const bf16x8 bq1 = __builtin_bit_cast(bf16x8, vuint4{b1[0], b1[1], b1[2], b1[3]});
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const bf16x8 a_hi = __builtin_bit_cast(bf16x8, vuint4{hi[t][0], hi[t][1], hi[t][2], hi[t][3]});
        const bf16x8 a_lo = __builtin_bit_cast(bf16x8, vuint4{lo[t][0], lo[t][1], lo[t][2], lo[t][3]});
        acc[t][u][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi, bq0, acc[t][u][0], 0, 0, 0);
        acc[t][u][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_hi, bq1, acc[t][u][1], 0, 0, 0);
        acc[t][u][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_lo, bq0, acc[t][u][0], 0, 0, 0);
        acc[t][u][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_lo, bq1, acc[t][u][1], 0, 0, 0);
      }
    }
  };

  // The activations of the slice, through registers into LDS. (Buffer loads: rows past M and
  // columns past K read as zero through the range check.)
  int bad = 0;
  {
    constexpr uint32_t XB = X_BF16 ? 2u : 4u;  // bytes per activation
    const __amdgpu_buffer_rsrc_t rsrc_x =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(x), 0, static_cast<int>(M * K * XB), 0x00020000);
    const uint32_t vecs_per_row = static_cast<uint32_t>(k_per_wg) / 4u, total = 16u * MT * vecs_per_row;
    vuint4 v[kFillVecs * MT];
#pragma unroll
    for (int i = 0; i < kFillVecs * MT; ++i) {
      const uint32_t idx = static_cast<uint32_t>(tid) + static_cast<uint32_t>(i) * kSplitThreads;
      const uint32_t m = idx / vecs_per_row, kk = (idx % vecs_per_row) * 4u;
      const bool ok = idx < total && m < M && k_begin + kk < K;  // K % 4 == 0: a group of 4 is in or out as a whole
      const uint32_t off = ok ? (m * static_cast<uint32_t>(K) + static_cast<uint32_t>(k_begin) + kk) * XB : 0x80000000u;
      if (X_BF16) {  // 4 bf16 -> 4 f32 (exact)
        const vuint2 h = __builtin_amdgcn_raw_buffer_load_b64(rsrc_x, off, 0, 0);
        v[i] = vuint4{h.x << 16, h.x & 0xFFFF0000u, h.y << 16, h.y & 0xFFFF0000u};
      } else {
        v[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_x, off, 0, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (!kLateFetch) {
#pragma unroll
      for (int b = 0; b < kDepth; ++b) fetch(b, b);
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int i = 0; i < kFillVecs * MT; ++i) {
      const uint32_t idx = static_cast<uint32_t>(tid) + static_cast<uint32_t>(i) * kSplitThreads;
      const uint32_t m = idx / vecs_per_row, kk = (idx % vecs_per_row) * 4u;
      if (idx < total) *reinterpret_cast<vuint4*>(xs + m * xpitch + kk) = v[i];
      // an exponent field of all ones: an infinity or a NaN among this thread's activations
      const uint32_t e = 0x7F800000u;
      bad |= (v[i].x & e) == e || (v[i].y & e) == e || (v[i].z & e) == e || (v[i].w & e) == e;
    }
  }
  const bool nonfinite = __syncthreads_or(bad) != 0;
  // Q8S: the first weight loads go out only now, with the activations in LDS. Issued ahead of
  // them (to overlap the two round trips), the weights of all the workgroups fill the memory
  // system's queues and the small activation loads come back 3 us later instead of 1 us: the first
  // multiply of every wave waits for them, and the kernel took about 1 us longer that way (measured
  // with per-wave timestamps on the 4096 x 14336 weight, as are the other figures in this file).
  if (kLateFetch) {
#pragma unroll
    for (int b = 0; b < kDepth; ++b) fetch(b, b);
    __builtin_amdgcn_sched_barrier(0);
  }

  // (scheduling barriers: left alone, the compiler sinks a step's loads below the other step's
  // MFMAs to save registers, which puts the load latency in series with the arithmetic)
  if (!nonfinite) {
    for (int s0 = 0; s0 < steps; s0 += kDepth) {
#pragma unroll
      for (int b = 0; b < kDepth; ++b) {
        // Two waves share a SIMD (one of each half of the K slice), and the arbiter prefers the
        // older: left alone, that one runs ahead and the other finishes 3 us after it, alone on
        // the SIMD, with nothing to cover its waits. The priority falls with a wave's progress, so
        // the wave that is behind goes first and both finish together (1 us sooner).
        if (kProgressPriority) {
          const int quarter = (s0 + b) * 4 / steps;
          if (quarter <= 0) __builtin_amdgcn_s_setprio(3);
          else if (quarter == 1) __builtin_amdgcn_s_setprio(2);
          else if (quarter == 2) __builtin_amdgcn_s_setprio(1);
          else __builtin_amdgcn_s_setprio(0);
        }
        multiply(std::false_type{}, b, s0 + b);
        __builtin_amdgcn_sched_barrier(0);
        fetch(b, s0 + b + kDepth);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  } else {
    for (int s0 = 0; s0 < steps; s0 += kDepth) {
#pragma unroll
      for (int b = 0; b < kDepth; ++b) {
        if (s0 + b < steps) multiply(std::true_type{}, b, s0 + b);
        __builtin_amdgcn_sched_barrier(0);
        fetch(b, s0 + b + kDepth);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

  // Add the two halves of the K slice in LDS, laid out as the output tile (the activations are
  // no longer needed: their memory is reused), then store it row by row, 16 bytes per lane: every
  // store instruction of a wave writes 1 KB of one output row. Element i of accumulator (u, p)
  // is row 4 kg + i, column 32 u + VPL (c % WPB) + c / WPB + (VPL / 2) p of the group (word
  // c % WPB of the block, field c / WPB or that plus half the fields). (Stored straight from the
  // accumulators, as 4-byte pieces 16 bytes apart, the kernel took about 1 us longer.)
  __syncthreads();
  float* const stage = reinterpret_cast<float*>(smem);
  constexpr uint32_t SP = kTileCols + 4;  // pitch in floats
  // DL: the lane's columns are 8 c .. 8 c + 7 of the group (block c / 4), accumulator (u, p) being
  // byte u % 2 + 2 p of word u / 2 (Q4S: nibble u + 4 p). PK: a block's product sits in rows 4 b ..
  // 4 b + 3 of the accumulators, i.e. in the lanes with kg == b, element i = activation row i.
  auto cell = [&](int t, int u, int p, int i, bool& mine) -> uint32_t {
    const uint32_t col = static_cast<uint32_t>(g) * kGroupCols;
    mine = true;
    if (DL) {
      mine = !PK || kg == (c >> 2);
      return (PK ? i : 16 * t + 4 * kg + i) * SP + col + 8u * static_cast<uint32_t>(c) + (VPL == 4 ? 4 * (u >> 1) + (u & 1) + 2 * p : u + 4 * p);
    }
    const uint32_t in_block = static_cast<uint32_t>(VPL * (c % WPB) + c / WPB) + 32 * u + (VPL / 2) * p;
    return (16 * t + 4 * kg + i) * SP + col + in_block;
  };
  if (h == 1) {
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int u = 0; u < kUnits; ++u)
#pragma unroll
        for (int p = 0; p < 2; ++p)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            bool mine;
            const uint32_t at = cell(t, u, p, i, mine);
            if (mine) stage[at] = acc[t][u][p][i] + (VPL == 8 ? off[t][kSharedA ? 0 : u][i] : 0.0f);
          }
  }
  __syncthreads();
  if (h == 0) {
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int u = 0; u < kUnits; ++u)
#pragma unroll
        for (int p = 0; p < 2; ++p)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            bool mine;
            const uint32_t at = cell(t, u, p, i, mine);
            if (mine) stage[at] += acc[t][u][p][i] + (VPL == 8 ? off[t][kSharedA ? 0 : u][i] : 0.0f);
          }
  }
  __syncthreads();
  {
    float* dst = part + static_cast<size_t>(slice_id) * M * N;
    const size_t tile_col0 = static_cast<size_t>(tile_id) * kTileCols;
#pragma unroll
    for (int r = 0; r < 4 * MT; ++r) {
      const uint32_t idx = static_cast<uint32_t>(tid) + static_cast<uint32_t>(r) * kSplitThreads;
      const uint32_t row = idx / (kTileCols / 4), c4 = (idx % (kTileCols / 4)) * 4u;
      if (row < M && tile_col0 + c4 < N)
        *reinterpret_cast<vfloat4*>(dst + row * N + tile_col0 + c4) = *reinterpret_cast<const vfloat4*>(stage + row * SP + c4);
    }
  }
}

struct SplitPlan {
  unsigned tiles, slices;
  size_t k_per_wg;
};

// Just under one workgroup per CU of the 256-CU part (all resident at once), but few enough K
// slices that the partial sums stay small beside the weights.
SplitPlan split_plan(size_t k, size_t n) {
  SplitPlan p;
  p.tiles = static_cast<unsigned>((n + kTileCols - 1) / kTileCols);
  size_t want = std::max<size_t>(1, (224 + p.tiles / 2) / p.tiles);
  const size_t unit = kKWays * kStepRows;
  size_t kpw = ((k + want - 1) / want + unit - 1) / unit * unit;
  kpw = std::min<size_t>(kpw, kMaxSlice);
  p.k_per_wg = kpw;
  p.slices = static_cast<unsigned>((k + kpw - 1) / kpw);
  return p;
}

}  // namespace

// Weights whose rows split into whole 128-column groups and whose K into whole 32-row steps; one
// scale per 32, 64 or 128 columns or per tensor; 32-bit buffer offsets.
bool split_ok(size_t m, size_t k, size_t n, int x_dtype, int value, int block) {
  return (x_dtype == BQ_F32 || x_dtype == BQ_BF16) && (value == BQ_Q8S || value == BQ_Q4S) && m >= 1 && m <= 32 && n % kGroupCols == 0 && n > 0 &&
         k % kStepRows == 0 && k > 0 && (block == 0 || block == 32 || block == 64 || block == 128) && k * n < 0x7FFFFFFFull;
}

size_t split_workspace(size_t m, size_t k, size_t n) {
  return static_cast<size_t>(split_plan(k, n).slices) * m * n * sizeof(float);
}

// Launches the kernel; `part` receives slices x [M, N] partial sums, the number of slices goes to
// *slices_out (the caller runs the fixed-order reduction).
bq_status launch_qsplit(const void* x, int x_dtype, const uint32_t* w, const float* scales, size_t m, size_t k, size_t n,
                        int value, int block, float* part, unsigned* slices_out, hipStream_t st) {
  const SplitPlan p = split_plan(k, n);
  const bool per_tensor = block == 0;
  const size_t mt = m > 16 ? 2 : 1;
  const size_t lds = 16 * mt * (kMaxSlice + 4) * sizeof(float) + kSplitWaves * kSlotBytes;
  dim3 tb(kSplitThreads);
#define BQ_SPLIT3(V, PT, XB, T, S, P)                                                              \
  do {                                                                                            \
    auto kernel = qsplit_kernel<V, PT, XB, T, S, P, (P || PT)>;                                            \
    /* the kernel's workgroup map: bundles of adjacent tiles, dealt to the XCDs 8 at a time */    \
    const unsigned bundle = PT ? 1u : (2u << S), units = (p.tiles + bundle - 1u) / bundle * p.slices;  \
    dim3 grid(8u * bundle * ((units + 7u) / 8u));                                                 \
    /* more than the default 64 KiB: checked against what the device grants, else refused here */ \
    BQ_TRY(configure_dynamic_lds(reinterpret_cast<const void*>(kernel), lds, "qsplit_kernel"));   \
    hipLaunchKernelGGL(kernel, grid, tb, lds, st, x, w, scales, m, k, n, p.k_per_wg, p.tiles, p.slices, part);       \
  } while (0)
#define BQ_SPLIT(V, PT, XB, S)                  \
  if (mt == 2) BQ_SPLIT3(V, PT, XB, 2, S, false); else BQ_SPLIT3(V, PT, XB, 1, S, false)
#define BQ_SPLIT_B(V, XB)                                \
  if (per_tensor) BQ_SPLIT(V, true, XB, 0);              \
  else if (block == 32 && m <= 4) BQ_SPLIT3(V, false, XB, 1, 0, true); /* row packing */ \
  else if (block == 32) BQ_SPLIT(V, false, XB, 0);       \
  else if (block == 64) BQ_SPLIT(V, false, XB, 1);       \
  else BQ_SPLIT(V, false, XB, 2)
#define BQ_SPLIT_V(V)                                                    \
  if (x_dtype == BQ_BF16) { BQ_SPLIT_B(V, true); } else { BQ_SPLIT_B(V, false); }
  if (value == BQ_Q8S) { BQ_SPLIT_V(4) } else { BQ_SPLIT_V(8) }
#undef BQ_SPLIT_V
#undef BQ_SPLIT_B
#undef BQ_SPLIT3
#undef BQ_SPLIT
  BQ_HIP(hipGetLastError());
  *slices_out = p.slices;
  return BQ_OK;
}

}  // namespace bq
