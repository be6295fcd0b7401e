// Prefill q-GEMM for gfx950: out[M,N] = A[M,K] (bf16, or f32 rounded to bf16) x dequantize(W[K,N]).
//
// The quantized rhs of QTensorOps::q_matmul (crates/burn-backend/src/backend/ops/qtensor.rs:498-544)
// never exists as a float matrix: packed words and their scales go global -> registers, are
// dequantized to bf16(s * q) there, and are written k-contiguous into LDS, from where
// v_mfma_f32_32x32x16_bf16 consumes them with f32 accumulation. (The reference path,
// crates/burn-ndarray/src/ops/qtensor.rs:223-267, materialises dequantize(W) and calls an sgemm.)
//
// Tiling: a workgroup of 8 waves (2 x 4) owns a BM x 256 output tile, BM = 256 or 128; a wave
// holds its (BM / 2) x 64 part as 8 or 4 MFMA tiles of 32 x 32 in accumulator registers; K
// advances 64 per stage through a double-buffered LDS ring. Two waves per SIMD mean that little
// hides latency but the
// instruction order, so a stage is software-pipelined by hand: while the MFMAs of stage t
// issue, the same wave dequantizes the words of stage t+1 (loaded more than a stage earlier) in
// the issue slots the matrix pipe leaves free (about five plain instructions per 32x32x16 MFMA,
// measured), stores them to the other LDS stage, and issues the loads of stage t+3 (weights)
// and t+2 (activations). Each MFMA and the instructions that ride with it form a micro-step
// that a scheduling barrier pins in place.
//
// Global reads are buffer loads (scalar descriptor + 32-bit lane offset). Activation rows past M
// fall outside their descriptor and read as zero; weight rows past K are clamped to the last
// row (and zeroed in the K-tail variant), since the scalar part of a buffer address is not
// range-checked. Columns past N only ever feed output columns that are not stored.
// LDS rows are 128 bytes (64 bf16 along k); 16-byte chunk c of row r lives at chunk
// c ^ ((r ^ (r >> 3)) & 7), which keeps both the fragment reads (32 consecutive rows, one chunk)
// and the dequantize writes (rows 4 or 8 apart, one chunk) free of bank conflicts.
#include <type_traits>

#include <algorithm>

#include "common.hpp"
#include "device_math.hpp"

namespace bq {

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx2 __attribute__((ext_vector_type(2)));

constexpr int BN = 256;
constexpr int BK = 64;
constexpr int kRowBytes = BK * 2;  // one LDS row: 64 bf16

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(floatx2{lo, hi}, bf16x2));
}

__device__ __forceinline__ uint32_t lds_offset(int row, int chunk) {
  return static_cast<uint32_t>(row * kRowBytes + ((chunk ^ ((row ^ (row >> 3)) & 7)) << 4));
}

// Raw buffer descriptor over [base, base + bytes): lane offsets past the end read 0.
typedef uint32_t desc_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ desc_t make_desc(const void* base, size_t bytes) {
  const uint64_t addr = reinterpret_cast<uint64_t>(base);
  const uint32_t n = bytes > 0xFFFFFFFFull ? 0xFFFFFFFFu : static_cast<uint32_t>(bytes);
  return desc_t{static_cast<uint32_t>(addr), static_cast<uint32_t>(addr >> 32) & 0xFFFFu, n, 0x00020000u};
}

// Global loads the compiler does not track: it would drain the whole load queue (vmcnt(0)) at
// the loop header, which is exactly the prefetch distance this kernel lives on. The registers
// they write are not valid until a loads_landed() naming them has executed; loads return in
// issue order, so "at most N younger loads outstanding" is an exact condition.
__device__ __forceinline__ vuint4 load_b128(desc_t d, uint32_t lane_off) {
  vuint4 r;
  asm volatile("buffer_load_dwordx4 %0, %1, %2, 0 offen" : "=v"(r) : "v"(lane_off), "s"(d));
  return r;
}
__device__ __forceinline__ uint32_t load_b32(desc_t d, uint32_t lane_off, uint32_t scalar_off) {
  uint32_t r;
  asm volatile("buffer_load_dword %0, %1, %2, %3 offen" : "=v"(r) : "v"(lane_off), "s"(d), "s"(scalar_off));
  return r;
}
// Waits until at most N loads are outstanding. The values pass through the statement so that
// no use of them can be placed ahead of the wait.
template <int N>
__device__ __forceinline__ void loads_landed(vuint4& v) {
  asm volatile("s_waitcnt vmcnt(%1)" : "+v"(v) : "n"(N));
}
template <int N>
__device__ __forceinline__ void loads_landed(uint32_t (&w)[8], float (&f)[8]) {
  asm volatile("s_waitcnt vmcnt(%16)"
               : "+v"(w[0]), "+v"(w[1]), "+v"(w[2]), "+v"(w[3]), "+v"(w[4]), "+v"(w[5]), "+v"(w[6]), "+v"(w[7]),
                 "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]), "+v"(f[4]), "+v"(f[5]), "+v"(f[6]), "+v"(f[7])
               : "n"(N));
}

// f32 activations are rounded to bf16 (nearest even) once, ahead of the GEMM.
__global__ void __launch_bounds__(256) a_to_bf16_kernel(const float* __restrict__ a, size_t groups,
                                                        vuint4* __restrict__ out) {
  const size_t g = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
  if (g >= groups) return;
  const vfloat4 lo = reinterpret_cast<const vfloat4*>(a)[2 * g];
  const vfloat4 hi = reinterpret_cast<const vfloat4*>(a)[2 * g + 1];
  out[g] = vuint4{pack_bf16(lo.x, lo.y), pack_bf16(lo.z, lo.w), pack_bf16(hi.x, hi.y), pack_bf16(hi.z, hi.w)};
}

template <int N>
__device__ __forceinline__ void loads_landed(uint32_t (&w)[4], float (&f)[4]) {
  asm volatile("s_waitcnt vmcnt(%8)"
               : "+v"(w[0]), "+v"(w[1]), "+v"(w[2]), "+v"(w[3]), "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3])
               : "n"(N));
}

// Workgroup shape: 8 waves, 2 x 4 (wave tile BM/2 x 64): two waves per SIMD, so one wave's MFMAs
// issue while the other decodes, stores or waits; 128 + 128 registers per wave at BM = 256.
// Q8S holds twice the words per thread; to stay inside that budget it decodes straight from the
// registers its loads wrote (see DIRECT below). (BM = 128 with 4 waves of 64 x 128 was 5-9 %
// slower on 33 <= M <= 128.)
constexpr int gemm_waves(int bm, int vpl) { return (void)vpl, (void)bm, 8; }

// K_TAIL: K is not a multiple of 128; the last stage is masked beyond K, and an odd stage count
// is padded with a stage whose activations are all masked.
template <int VPL, int BM, bool OUT_BF16, bool K_TAIL>
__global__ void __launch_bounds__(gemm_waves(BM, VPL) * kWave, 1)
qgemm_kernel(const uint16_t* __restrict__ a, const uint32_t* __restrict__ w,
             const float* __restrict__ scales, size_t M, size_t K, size_t N, size_t NW,
             unsigned block_words_log2, size_t scales_per_row, bool per_tensor,
             uint32_t stages_per_slice, const float* __restrict__ bias, void* __restrict__ out) {
  constexpr int WAVES = gemm_waves(BM, VPL);
  constexpr int THREADS = WAVES * kWave;
  constexpr int WN = WAVES / 2;                             // waves across N (2 across M)
  constexpr int WAVE_N = BN / WN;                           // 64 or 128 columns per wave
  constexpr int BITS = 32 / VPL;
  constexpr float BIAS = (BITS == 8) ? 128.0f : 8.0f;
  constexpr uint32_t FLIP = (BITS == 8) ? 0x80808080u : 0x88888888u;
  constexpr int WORD_COLS = BN / VPL;                       // 32 (Q4S) or 64 (Q8S)
  constexpr int ROWS = WORD_COLS * BK / THREADS;            // weight rows (words) a thread decodes per stage: 4, 8 or 16
  constexpr int TASK_ROWS = ROWS < 8 ? ROWS : 8;            // consecutive k of one word column
  constexpr int B_TASKS = ROWS / TASK_ROWS;                 // 1 with 8 waves
  constexpr int A_CHUNKS = BM * (BK / 8) / THREADS;         // 16-byte chunks of A per thread: 4
  constexpr int A_ROWS_PER_PASS = THREADS / 8;              // A rows covered by chunk i of all threads
  constexpr int MT = BM / 64;                               // 32-row MFMA tiles per wave
  constexpr int NT = WAVE_N / 32;                           // 32-col MFMA tiles per wave
  constexpr int KSTEPS = BK / 16;                           // MFMA k-steps per stage
  constexpr uint32_t A_STAGE = BM * kRowBytes, B_STAGE = BN * kRowBytes;
  constexpr uint32_t LDS_B = 2 * A_STAGE;
  // Micro-step plan (one MFMA each). [0, PREP): row preparation. [PREP, SYNC_AT): field decodes
  // with a chunk store after every TASK_ROWS, and the activation chunks' store + reload. At
  // SYNC_AT the workgroup barrier: every LDS store of the step is before it and every LDS read of
  // the stage being multiplied has been issued (and is waited for) before it, so it is the only
  // barrier of the step. [SYNC_AT, U): the first operand fragments of the next step are read from
  // the stage just completed. Weight loads are spread over [PREP, U) and end the step.
  constexpr int U = KSTEPS * MT * NT;                       // MFMAs per wave and stage: 32 (BM = 256) or 16
  constexpr int GROUPS = U / NT;                            // A fragments per stage
  constexpr int PF = (NT == 2 && U >= 32) ? 3 : 2;                       // A fragments read this many groups ahead
  // DIRECT (Q8S on 8 waves): no per-row copies. A field is sign-extended straight out of the
  // loaded word and multiplied by the loaded scale, so the words stay live until the last field
  // is decoded and their registers are refilled only after that, in [SYNC_AT, U).
  constexpr bool DIRECT = BITS == 8 && WAVES == 8;
  constexpr int PREP = DIRECT ? 4 : (ROWS < 8 ? ROWS : 8);
  constexpr int ROWS_PER_PREP = ROWS / PREP;
  constexpr int SYNC_AT = U - U / 8;
  constexpr int FIELD_STEPS = SYNC_AT - PREP;
  constexpr int NFIELDS = ROWS * VPL;
  constexpr int NEXT_READS = NT + PF;                       // fragments fetched behind the barrier
  constexpr int LOADS_PER_STEP = A_CHUNKS + 2 * ROWS;
  static_assert(ROWS % PREP == 0 && FIELD_STEPS >= A_CHUNKS && NEXT_READS <= 2 * (U - SYNC_AT), "micro-step plan");
  // LDS reads of the stage being multiplied are issued before SYNC_AT: the last A fragment (PF
  // groups ahead) in group GROUPS - 1 - PF, the last B fragments during the k-step before the last
  static_assert((GROUPS - 1 - PF) * NT < SYNC_AT && (KSTEPS - 1) * MT * NT <= SYNC_AT, "reads before the barrier");

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];  // A: 2 stages, then B: 2 stages

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid / kWave;
  const int wm = wave / WN, wn = wave % WN;
  // Workgroups go to the 8 XCDs (each with its own L2) round robin in launch order. When the
  // tile grid divides evenly, XCD c multiplies the block of row tiles c / 4 and column tiles c % 4
  // of a 2 x 4 partition, so its L2 holds half of the activations and a quarter of the weights
  // instead of all of the activations.
  uint32_t tile_m = blockIdx.y, tile_n = blockIdx.x;
  if (gridDim.y % 2 == 0 && gridDim.x % 4 == 0) {
    const uint32_t id = blockIdx.x + gridDim.x * blockIdx.y;
    const uint32_t xcd = id & 7u, j = id >> 3;
    const uint32_t pm = gridDim.y / 2, pn = gridDim.x / 4;
    tile_m = (xcd >> 2) * pm + j % pm;
    tile_n = (xcd & 3u) * pn + j / pm;
  }
  const size_t m0 = static_cast<size_t>(tile_m) * BM;
  const size_t n0 = static_cast<size_t>(tile_n) * BN;

  // A: chunk i of a thread is row (tid >> 3) + A_ROWS_PER_PASS * i, k (tid & 7) * 8 of the stage.
  // One descriptor per i, based at that row block and ending with the matrix, so that one lane
  // offset serves all of them and rows past M read as zero.
  desc_t rsrc_a[A_CHUNKS];
  uint32_t a_wr[A_CHUNKS];
#pragma unroll
  for (int i = 0; i < A_CHUNKS; ++i) {
    const size_t row = m0 + static_cast<size_t>(A_ROWS_PER_PASS) * i;
    const size_t rows_left = row < M ? M - row : 0;
    rsrc_a[i] = make_desc(a + (row < M ? row : 0) * K, rows_left * K * 2);
    a_wr[i] = lds_offset((tid >> 3) + A_ROWS_PER_PASS * i, tid & 7);
  }
  const uint32_t a_off = (static_cast<uint32_t>(tid >> 3) * static_cast<uint32_t>(K) + static_cast<uint32_t>(tid & 7) * 8u) * 2u;

  // W / scales: task t of a thread is word column wc, k rows krow0 .. krow0 + TASK_ROWS - 1 of the stage
  const size_t w_skip = n0 / VPL;
  const desc_t rsrc_w = make_desc(w + w_skip, (K * NW - w_skip) * 4);
  const size_t n_scales = per_tensor ? 1 : K * scales_per_row;
  const desc_t rsrc_s = make_desc(scales, n_scales * 4);
  const uint32_t w_row_bytes = static_cast<uint32_t>(NW) * 4u;
  const uint32_t s_row_bytes = per_tensor ? 0u : static_cast<uint32_t>(scales_per_row) * 4u;
  uint32_t w_col[B_TASKS], s_col[B_TASKS], krow0[B_TASKS];
  // lane offsets of each row of the stage (Q4S), or of the task's first row only (Q8S decodes
  // twice the rows per thread and has no registers to spare: the row goes into the scalar offset)
  constexpr int OFF_ROWS = (BITS == 4) ? TASK_ROWS : 1;
  uint32_t w_off[B_TASKS][OFF_ROWS], s_off[B_TASKS][OFF_ROWS];
#pragma unroll
  for (int t = 0; t < B_TASKS; ++t) {
    const int task = tid + t * THREADS;
    int wc = task % WORD_COLS;
    // word columns past the row end (N tail) re-read the last one: their output columns are never stored
    if (w_skip + wc >= NW) wc = static_cast<int>(NW - 1 - w_skip);
    krow0[t] = static_cast<uint32_t>(task / WORD_COLS) * TASK_ROWS;
    w_col[t] = static_cast<uint32_t>(wc) * 4u;
    s_col[t] = per_tensor ? 0u : static_cast<uint32_t>((n0 / VPL + wc) >> block_words_log2) * 4u;
#pragma unroll
    for (int r = 0; r < OFF_ROWS; ++r) {
      w_off[t][r] = w_col[t] + (krow0[t] + r) * w_row_bytes;
      s_off[t][r] = s_col[t] + (krow0[t] + r) * s_row_bytes;
    }
  }
  const uint32_t k_last = static_cast<uint32_t>(K) - 1u;
  const uint32_t kt_last = (static_cast<uint32_t>((K + BK - 1) / BK) - 1u) * BK;
  // Split K (gridDim.z > 1): this workgroup multiplies stages [first_stage, first_stage +
  // num_stages) and writes an f32 partial result to slice blockIdx.z of `out`.
  const uint32_t total_stages = static_cast<uint32_t>((K + BK - 1) / BK);
  const uint32_t first_stage = blockIdx.z * stages_per_slice;
  const uint32_t num_stages = total_stages - first_stage < stages_per_slice ? total_stages - first_stage : stages_per_slice;
  const uint32_t kbase = first_stage * BK;

  // LDS byte offsets. With r0 a multiple of 8 (4) and j < 8 (4):
  //   lds_offset(r0 + j, c) == lds_offset(r0, c) ^ (j * 144),
  // and stepping a row by 32 only flips bit 6 of the chunk part, so a handful of bases plus
  // compile-time constants cover every access of the stage. A task of 4 rows fills half a chunk.
  const int task_k = (tid / WORD_COLS) * TASK_ROWS;  // first k row of task 0 (task 1: + THREADS / WORD_COLS * 8)
  const uint32_t b_wr = LDS_B + lds_offset((tid % WORD_COLS) * VPL, task_k >> 3) + static_cast<uint32_t>(task_k & 7) * 2u;
  // MFMA operand fragment: lane holds row (col) lane % 32, k = 8 * (lane / 32) .. + 7 of the k-step
  const int frow = lane & 31, fgroup = lane >> 5;
  uint32_t a_rd[4], b_rd[4];  // tile i of k-step kk: base[(kk ^ 2 (i & 1)) & 3] + 4096 i
  {
    const uint32_t ab = lds_offset(wm * (BM / 2) + frow, fgroup);
    const uint32_t bb = LDS_B + lds_offset(wn * WAVE_N + frow, fgroup);
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      a_rd[v] = ab ^ (static_cast<uint32_t>(v) << 5);
      b_rd[v] = bb ^ (static_cast<uint32_t>(v) << 5);
    }
  }

  floatx16 acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  vuint4 a_reg[A_CHUNKS];                  // activations of the stage after the one in LDS
  uint32_t b_word[2][B_TASKS][TASK_ROWS];  // weights of the next two stages
  float b_scale[2][B_TASKS][TASK_ROWS];
  // per-row decode state of the stage being dequantized
  float row_s[ROWS], row_nb[ROWS];
  uint32_t row_lo[ROWS], row_hi[ROWS];  // word ^ FLIP; Q4S: its even / odd nibbles spread to bytes
  uint32_t packed[TASK_ROWS / 2];       // bf16 pairs (k, k+1) of the chunk being assembled
  float held;                           // the even-k value waiting for its odd-k partner

  auto load_a = [&](int i, uint32_t kt) { a_reg[i] = load_b128(rsrc_a[i], a_off + kt * 2u); };
  // Stages past the end of K (prefetched by the last steps, never multiplied) re-read the last one.
  auto load_b = [&](auto P, int idx, uint32_t kt) {
    constexpr int p = decltype(P)::value;
    const int t = idx / TASK_ROWS, r = idx % TASK_ROWS;
    const uint32_t kc = kt < kt_last ? kt : kt_last;
    if (K_TAIL) {  // rows past K exist in the last stage: clamp per lane (and zero when decoding)
      uint32_t row = kc + krow0[t] + r;
      row = row < k_last ? row : k_last;
      b_word[p][t][r] = load_b32(rsrc_w, w_col[t] + row * w_row_bytes, 0u);
      b_scale[p][t][r] = __builtin_bit_cast(float, load_b32(rsrc_s, s_col[t] + row * s_row_bytes, 0u));
    } else {
      const int ro = OFF_ROWS == 1 ? 0 : r;
      const uint32_t krow = OFF_ROWS == 1 ? kc + r : kc;
      b_word[p][t][r] = load_b32(rsrc_w, w_off[t][ro], krow * w_row_bytes);
      b_scale[p][t][r] = __builtin_bit_cast(float, load_b32(rsrc_s, s_off[t][ro], krow * s_row_bytes));
    }
  };
  auto store_a = [&](int i, uint32_t stage_base, uint32_t kt) {
    vuint4 v = a_reg[i];
    if (K_TAIL && kt + static_cast<uint32_t>(tid & 7) * 8u >= K) v = vuint4{0u, 0u, 0u, 0u};
    *reinterpret_cast<vuint4*>(smem + stage_base + a_wr[i]) = v;
  };
  // Unsigned fields u = q + BIAS of (word ^ FLIP): s*q = s*u - BIAS*s, one fma (BIAS*s is exact),
  // rounded once to bf16. A zero word is u = BIAS everywhere and decodes to exactly 0.
  auto prep_row = [&](auto P, int idx, uint32_t kt) {
    constexpr int p = decltype(P)::value;
    const int t = idx / TASK_ROWS, r = idx % TASK_ROWS;
    if (DIRECT) {
      b_scale[p][t][r] = valid_scale(b_scale[p][t][r]);
      if (K_TAIL && kt + krow0[t] + r >= K) b_word[p][t][r] = 0u;
      return;
    }
    row_s[idx] = valid_scale(b_scale[p][t][r]);
    row_nb[idx] = -BIAS * row_s[idx];
    uint32_t word = b_word[p][t][r];
    if (K_TAIL && kt + krow0[t] + r >= K) word = 0u;
    word ^= FLIP;
    if (BITS == 4) {
      // (the empty asm keeps the compiler from folding the nibble spread back into one bit-field
      // extract per field: a spread word feeds four v_cvt_f32_ubyteN directly)
      row_hi[idx] = (word >> 4) & 0x0F0F0F0Fu;
      asm("" : "+v"(row_hi[idx]));
      word &= 0x0F0F0F0Fu;
      asm("" : "+v"(word));
    }
    row_lo[idx] = word;
  };
  // Field f of a task runs over its TASK_ROWS rows before the next field starts: after them one
  // chunk (TASK_ROWS consecutive k of one output column, 16 or 8 bytes) is complete and goes to LDS.
  auto decode_field = [&](auto P, int f, uint32_t stage_base) {
    constexpr int p = decltype(P)::value;
    const int t = f / (TASK_ROWS * VPL), j = (f / TASK_ROWS) % VPL, r = f % TASK_ROWS;
    const int idx = t * TASK_ROWS + r;
    const uint32_t src = (BITS == 8) ? row_lo[idx] : ((j & 1) ? row_hi[idx] : row_lo[idx]);
    const int byte = (BITS == 8) ? j : (j >> 1);
    float v;
    if (DIRECT)  // s * q, rounded once: the same value as the fma below
      v = static_cast<float>(static_cast<int8_t>(b_word[p][t][r] >> (8 * j))) * b_scale[p][t][r];
    else
      v = __builtin_fmaf(static_cast<float>((src >> (8 * byte)) & 0xFFu), row_s[idx], row_nb[idx]);
    if (r & 1)
      packed[r >> 1] = pack_bf16(held, v);
    else
      held = v;
    if (r == TASK_ROWS - 1) {
      unsigned char* dst = smem + stage_base + (b_wr ^ static_cast<uint32_t>((j * 144) ^ (t * 64)));
      if (TASK_ROWS == 8)
        *reinterpret_cast<vuint4*>(dst) = vuint4{packed[0], packed[1], packed[TASK_ROWS / 2 - 2], packed[TASK_ROWS / 2 - 1]};
      else
        *reinterpret_cast<vuint2*>(dst) = vuint2{packed[0], packed[1]};
    }
  };
  auto frag_a = [&](int i, int kk, uint32_t stage_base) {
    return *reinterpret_cast<const bf16x8*>(smem + stage_base + a_rd[(kk ^ (2 * (i & 1))) & 3] + 4096u * i);
  };
  auto frag_b = [&](int j, int kk, uint32_t stage_base) {
    return *reinterpret_cast<const bf16x8*>(smem + stage_base + b_rd[(kk ^ (2 * (j & 1))) & 3] + 4096u * j);
  };
  // Loads and activation stores of micro-step u: activation chunk c = its store (stage sa, k
  // offset kt_sa) and reload (k offset kt_la) at u = PREP + c * FIELD_STEPS / A_CHUNKS; weight
  // row n (word + scale) of set Q at u = PREP + (n + 1) * (U - PREP) / ROWS - 1, the last one in
  // the last micro-step (DIRECT: at u = SYNC_AT + n * (U - SYNC_AT) / ROWS, after the last
  // decode). Every step and the prologue issue these in this same order, which is what makes
  // the younger-load counts of the waits constants:
  //   before a chunk's store, its load is LOADS_PER_STEP - 1 loads old;
  //   at the start of a step, the last load of the set decoded there is LOADS_PER_STEP loads old.
  auto io_step = [&](auto Q, int u, bool store, uint32_t sa_base, uint32_t kt_sa, uint32_t kt_la, uint32_t kt_lb) {
#pragma unroll
    for (int c = 0; c < A_CHUNKS; ++c)
      if (PREP + c * FIELD_STEPS / A_CHUNKS == u) {
        if (store) {
          loads_landed<LOADS_PER_STEP - 1>(a_reg[c]);
          store_a(c, sa_base, kt_sa);
        }
        load_a(c, kt_la);
      }
#pragma unroll
    for (int n = 0; n < ROWS; ++n)
      if ((DIRECT ? SYNC_AT + n * (U - SYNC_AT) / ROWS : PREP + (n + 1) * (U - PREP) / ROWS - 1) == u)
        load_b(Q, n, kt_lb);
  };

  // first operand fragments of the next step, read after the barrier of the current one
  bf16x8 next_b[NT], next_a[PF];
  auto read_next = [&](int r, uint32_t a_base, uint32_t b_base) {
    if (r < NT)
      next_b[r] = frag_b(r, 0, b_base);
    else
      next_a[r - NT] = frag_a((r - NT) % MT, (r - NT) / MT, a_base);
  };

  // One pipeline step. p = t & 1 is the LDS stage being multiplied; the other LDS stage receives
  // stage t+1, decoded from register set p ^ 1, which is then refilled with stage t+3.
  auto step = [&](auto P, uint32_t t) {
    constexpr int p = decltype(P)::value;
    using Q = std::integral_constant<int, p ^ 1>;
    const uint32_t kt1 = kbase + (t + 1) * BK;
    // Operand fragments are read well ahead of their MFMAs (LDS latency under load is several
    // MFMAs long): B fragments of k-step kk+1 during k-step kk, spread over its groups of NT
    // MFMAs; the A fragment of group g+PF at the start of group g.
    bf16x8 bfr[2][NT], af[PF + 1];
#pragma unroll
    for (int j = 0; j < NT; ++j) bfr[0][j] = next_b[j];
#pragma unroll
    for (int i = 0; i < PF; ++i) af[i] = next_a[i];
#pragma unroll
    for (int tk = 0; tk < B_TASKS; ++tk) loads_landed<LOADS_PER_STEP>(b_word[p ^ 1][tk], b_scale[p ^ 1][tk]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int kk = u / (MT * NT), i = (u / NT) % MT, j = u % NT;
      const int g = u / NT;  // group = A fragment index: af[g % (PF + 1)] holds fragment (kk, i)
      if (u == SYNC_AT) {
        __syncthreads();
        __builtin_amdgcn_sched_barrier(0);
      }
      asm("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(af[g % (PF + 1)]), "v"(bfr[kk & 1][j]));
      if (j == 0 && g + PF < GROUPS) af[(g + PF) % (PF + 1)] = frag_a((g + PF) % MT, (g + PF) / MT, p * A_STAGE);
      if (j == 1 && kk + 1 < KSTEPS) {
#pragma unroll
        for (int f = 0; f < NT; ++f)
          if (f * MT / NT == i) bfr[(kk + 1) & 1][f] = frag_b(f, kk + 1, p * B_STAGE);
      }
      if (u < PREP) {
#pragma unroll
        for (int q = 0; q < ROWS_PER_PREP; ++q) prep_row(Q{}, u * ROWS_PER_PREP + q, kt1);
      } else {
        if (u < SYNC_AT) {
#pragma unroll
          for (int f = 0; f < NFIELDS; ++f)
            if (PREP + f * FIELD_STEPS / NFIELDS == u) decode_field(Q{}, f, (p ^ 1) * B_STAGE);
        } else {
#pragma unroll
          for (int r = 0; r < NEXT_READS; ++r)
            if (SYNC_AT + r * (U - SYNC_AT) / NEXT_READS == u) read_next(r, (p ^ 1) * A_STAGE, (p ^ 1) * B_STAGE);
        }
        io_step(Q{}, u, true, (p ^ 1) * A_STAGE, kt1, kbase + (t + 2) * BK, kbase + (t + 3) * BK);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // Prologue: stage 0 of the weights straight into LDS, then what the two steps before step 0
  // would have issued, in their order (see io_step): stage 1 weights into set 1 with the stage 0
  // activations, then stage 2 weights into set 0 with the activation store / reload.
  using P0 = std::integral_constant<int, 0>;
  using P1 = std::integral_constant<int, 1>;
#pragma unroll
  for (int idx = 0; idx < ROWS; ++idx) load_b(P0{}, idx, kbase);
#pragma unroll
  for (int tk = 0; tk < B_TASKS; ++tk) loads_landed<0>(b_word[0][tk], b_scale[0][tk]);
#pragma unroll
  for (int idx = 0; idx < ROWS; ++idx) prep_row(P0{}, idx, kbase);
#pragma unroll
  for (int f = 0; f < NFIELDS; ++f) decode_field(P0{}, f, 0);
#pragma unroll
  for (int u = PREP; u < U; ++u) io_step(P1{}, u, false, 0, 0, kbase, kbase + BK);
#pragma unroll
  for (int u = PREP; u < U; ++u) io_step(P0{}, u, true, 0, kbase, kbase + BK, kbase + 2 * BK);
  __syncthreads();
#pragma unroll
  for (int r = 0; r < NEXT_READS; ++r) read_next(r, 0, 0);
  // Steps run in pairs with no branch between them (a conditional second step makes every
  // accumulator a loop phi of two definitions, which the register allocator cannot untangle).
  for (uint32_t t = 0; t < num_stages; t += 2) {
    step(P0{}, t);
    step(P1{}, t + 1);
    // Before the loop is left: loads issued for stages past the end are still in flight and
    // their registers are about to be reused, and the MFMAs are opaque to the compiler's hazard
    // recognizer, so the last ones must have drained before anything reads an accumulator.
    // (Inside the loop, because the compiler may place copies right at the loop exit.)
    if (t + 2 >= num_stages) asm volatile("s_waitcnt vmcnt(0)\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
  }

  // epilogue: element e of a 32x32 tile is row 8 * (e / 4) + 4 * (lane / 32) + e % 4, column lane % 32
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      const size_t col = n0 + wn * WAVE_N + j * 32 + (lane & 31);
      // a linear layer's bias is added last (not to split-K partials: their sum gets it)
      const float bias_v = (bias != nullptr && col < N) ? bias[col] : 0.0f;
      // Neighbouring lanes hold neighbouring columns of the same rows. They swap one element of
      // every pair of rows (DPP, lanes 2p <-> 2p + 1): the even lane then stores columns
      // (c, c + 1) of the first row and the odd lane the same two columns of the second row, as
      // one 8-byte (f32) or 4-byte (bf16) store each instead of two of half the size. Measured on
      // [2048,4096] x [4096,14336]: f32 235.6 -> 221.7 us, bf16 244.6 -> 218.0 us; exchanging
      // among four lanes for 16-byte stores is no faster (223.1 us), and other orders of the
      // stores (the two column blocks of a row pair back to back, or column block outermost) are
      // 2-3 % slower than this one. N is even: rows are whole packed words.
      const bool odd = lane & 1;
      const size_t col0 = col & ~static_cast<size_t>(1);
#pragma unroll
      for (int t = 0; t < 8; ++t) {
        const float first = acc[i][j][2 * t] + bias_v, second = acc[i][j][2 * t + 1] + bias_v;
        const float give = odd ? first : second;
        const float got = __builtin_bit_cast(
            float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, give), 0xB1, 0xF, 0xF, false));
        const float left = odd ? got : first, right = odd ? second : got;
        const size_t row = m0 + wm * (BM / 2) + i * 32 + 8 * (t / 2) + 4 * (lane >> 5) + 2 * (t % 2) + (odd ? 1 : 0);
        if (row < M && col0 < N) {
          if (OUT_BF16)
            *reinterpret_cast<uint32_t*>(static_cast<uint16_t*>(out) + row * N + col0) = f32x2_to_bf16x2(left, right);
          else
            *reinterpret_cast<floatx2*>(static_cast<float*>(out) + static_cast<size_t>(blockIdx.z) * M * N + row * N + col0) =
                floatx2{left, right};
        }
      }
    }
}

template <int VPL, int BM, bool OUT_BF16>
bq_status launch_one(const uint16_t* a, const uint32_t* w, const float* scales, size_t m, size_t k, size_t n,
                     size_t nw, unsigned bwl2, size_t spr, bool per_tensor, unsigned slices, uint32_t stages_per_slice,
                     const float* bias, void* out, hipStream_t st) {
  constexpr size_t lds_bytes = 2 * (static_cast<size_t>(BM) + BN) * kRowBytes;
  const bool k_tail = k % (2 * BK) != 0;  // also pads an odd stage count (slices hold even counts)
  auto kernel = k_tail ? qgemm_kernel<VPL, BM, OUT_BF16, true> : qgemm_kernel<VPL, BM, OUT_BF16, false>;
  // (checked on the host against what the device grants per workgroup; refused, never launched, beyond it)
  BQ_TRY(configure_dynamic_lds(reinterpret_cast<const void*>(kernel), lds_bytes, "qgemm_kernel"));
  dim3 grid(static_cast<unsigned>((n + BN - 1) / BN), static_cast<unsigned>((m + BM - 1) / BM), slices), tb(gemm_waves(BM, VPL) * kWave);
  hipLaunchKernelGGL(kernel, grid, tb, lds_bytes, st, a, w, scales, m, k, n, nw, bwl2, spr, per_tensor, stages_per_slice, bias, out);
  BQ_HIP(hipGetLastError());
  return BQ_OK;
}

template <int VPL, int BM>
bq_status launch_dtype(bool o_bf16, const uint16_t* a, const uint32_t* w, const float* scales, size_t m,
                       size_t k, size_t n, size_t nw, unsigned bwl2, size_t spr, bool per_tensor, unsigned slices,
                       uint32_t stages_per_slice, const float* bias, void* out, hipStream_t st) {
  if (o_bf16) return launch_one<VPL, BM, true>(a, w, scales, m, k, n, nw, bwl2, spr, per_tensor, slices, stages_per_slice, bias, out, st);
  return launch_one<VPL, BM, false>(a, w, scales, m, k, n, nw, bwl2, spr, per_tensor, slices, stages_per_slice, bias, out, st);
}

}  // namespace

// True when the tiled kernel's 16-byte row alignment and 32-bit buffer offsets hold.
bool qgemm_ok(int a_dtype, size_t k, size_t n, int value, size_t scales_per_row) {
  (void)a_dtype;
  const size_t nw = n / static_cast<size_t>(num_quants(value));
  return k % 8 == 0 && 64 * k * 2 < 0xFFFFFFFFull && k * nw * 4 < 0xFFFFFFFFull &&
         k * (scales_per_row ? scales_per_row : 1) * 4 < 0xFFFFFFFFull;
}

// Few output tiles (M up to a few hundred) leave most CUs idle: K is then split over gridDim.z
// workgroups per tile, which write f32 partial results that the caller adds up in a fixed order.
struct GemmSplit {
  unsigned slices;
  uint32_t stages_per_slice;
};

GemmSplit gemm_split(size_t m, size_t k, size_t n) {
  const size_t bm = m > 128 ? 256 : 128;
  const size_t tiles = ((n + BN - 1) / BN) * ((m + bm - 1) / bm);
  const uint32_t total = static_cast<uint32_t>((k + BK - 1) / BK);
  GemmSplit g{1, total};
  if (tiles > 128 || total < 8) return g;
  size_t want = std::min<size_t>(8, 256 / tiles);
  uint32_t sps = static_cast<uint32_t>((total + want - 1) / want);
  sps = (sps + 1u) & ~1u;  // even: the kernel runs stages in pairs
  if (sps < 4) sps = 4;
  g.slices = (total + sps - 1) / sps;
  g.stages_per_slice = g.slices > 1 ? sps : total;
  return g;
}

// Bytes of scratch the tiled kernel needs: the bf16 copy of an f32 lhs, then the split-K partials.
static size_t a_copy_bytes(int a_dtype, size_t m, size_t k) {
  return a_dtype == BQ_F32 ? (m * k * 2 + 255) / 256 * 256 : 0;
}
size_t qgemm_workspace(int a_dtype, size_t m, size_t k, size_t n) {
  const GemmSplit g = gemm_split(m, k, n);
  return a_copy_bytes(a_dtype, m, k) + (g.slices > 1 ? static_cast<size_t>(g.slices) * m * n * sizeof(float) : 0);
}

// Tiled MFMA q-GEMM. BM = 256 once M fills such tiles, 128 below. With split K the result is left
// as *slices_out partial [M, N] f32 matrices at *part_out (inside the workspace) for the caller to
// reduce (and to add `bias` to); otherwise *slices_out is 1 and `out` is complete, bias included.
// `bias` (N floats, may be null) is a linear layer's: out[r][c] = sum + bias[c].
bq_status launch_qgemm(const void* a, int a_dtype, const uint32_t* w, const float* scales, size_t m,
                       size_t k, size_t n, int value, unsigned block_words_log2, size_t scales_per_row,
                       bool per_tensor, const float* bias, int out_dtype, void* out, void* workspace,
                       size_t workspace_bytes, unsigned* slices_out, float** part_out, hipStream_t st) {
  const uint16_t* a16 = static_cast<const uint16_t*>(a);
  const GemmSplit g = gemm_split(m, k, n);
  const size_t need = qgemm_workspace(a_dtype, m, k, n);
  if (need && (workspace == nullptr || workspace_bytes < need))
    BQ_FAIL(BQ_ERR_SIZE, "q_matmul workspace: need %zu bytes, got %zu", need, workspace_bytes);
  if (a_dtype == BQ_F32) {
    const size_t groups = m * k / 8;
    hipLaunchKernelGGL(a_to_bf16_kernel, dim3(static_cast<unsigned>((groups + 255) / 256)), dim3(256), 0, st,
                       static_cast<const float*>(a), groups, static_cast<vuint4*>(workspace));
    BQ_HIP(hipGetLastError());
    a16 = static_cast<const uint16_t*>(workspace);
  }
  float* part = reinterpret_cast<float*>(static_cast<unsigned char*>(workspace) + a_copy_bytes(a_dtype, m, k));
  *slices_out = g.slices;
  *part_out = part;
  const bool split = g.slices > 1;
  const bool o_bf16 = !split && out_dtype == BQ_BF16;
  void* dst = split ? static_cast<void*>(part) : out;
  const float* kb = split ? nullptr : bias;  // with split K the caller's reduction adds the bias
  const size_t nw = n / static_cast<size_t>(num_quants(value));
  const bool big = m > 128;
  if (value == BQ_Q8S) {
    if (big)
      return launch_dtype<4, 256>(o_bf16, a16, w, scales, m, k, n, nw, block_words_log2, scales_per_row,
                                  per_tensor, g.slices, g.stages_per_slice, kb, dst, st);
    return launch_dtype<4, 128>(o_bf16, a16, w, scales, m, k, n, nw, block_words_log2, scales_per_row,
                                per_tensor, g.slices, g.stages_per_slice, kb, dst, st);
  }
  if (big)
    return launch_dtype<8, 256>(o_bf16, a16, w, scales, m, k, n, nw, block_words_log2, scales_per_row,
                                per_tensor, g.slices, g.stages_per_slice, kb, dst, st);
  return launch_dtype<8, 128>(o_bf16, a16, w, scales, m, k, n, nw, block_words_log2, scales_per_row,
                              per_tensor, g.slices, g.stages_per_slice, kb, dst, st);
}

}  // namespace bq
