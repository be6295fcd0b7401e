/* Runs every function of the C oracle over ragged shapes with exactly sized heap buffers, so that
 * the address and undefined-behaviour sanitizers see any out-of-range access, signed overflow or
 * invalid shift.
 *
 *   gcc -std=c11 -O1 -g -fsanitize=address,undefined -fno-sanitize-recover=all -I oracle
 *       tests/cpp/oracle_sanitize.c oracle/bq_oracle.c -lm -o oracle_sanitize
 *
 * It checks little beyond "no sanitizer report" -- the known answers are in tests/test_oracle_kat.py --
 * except the round trips that cost nothing here: unpack(pack(q)) == q and decode(encode(q, s)) == (q, s). */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "bq_oracle.h"

static unsigned long long state = 0x2545F4914F6CDD1DULL;
static unsigned next_u32(void) {
  state ^= state << 13;
  state ^= state >> 7;
  state ^= state << 17;
  return (unsigned)(state >> 32);
}
static float next_float(void) { return ((float)(next_u32() % 200001) - 100000.0f) / 25000.0f; }

#define CHECK(cond)                                                          \
  do {                                                                       \
    if (!(cond)) {                                                           \
      fprintf(stderr, "oracle_sanitize: %s failed at line %d\n", #cond, __LINE__); \
      exit(1);                                                               \
    }                                                                        \
  } while (0)

static void* exact(size_t bytes) {
  void* p = malloc(bytes ? bytes : 1);
  CHECK(p != NULL);
  return p;
}

static void one_case(const size_t* shape, int rank, int value, int store, const unsigned char* block, int block_rank) {
  bqo_scheme s;
  memset(&s, 0, sizeof s);
  s.value = (uint8_t)value;
  s.store = (uint8_t)store;
  s.level = block ? BQO_LEVEL_BLOCK : BQO_LEVEL_TENSOR;
  s.block_rank = (uint8_t)block_rank;
  for (int i = 0; i < block_rank; ++i) s.block[i] = block[i];
  size_t n = 1;
  for (int i = 0; i < rank; ++i) n *= shape[i];
  size_t pshape[BQO_MAX_RANK];
  const size_t np = bqo_params_shape(shape, rank, &s, pshape);
  float* x = exact(n * sizeof(float));
  for (size_t i = 0; i < n; ++i) x[i] = (i % 97 == 0) ? 0.0f : next_float();
  float* lo = exact(np * sizeof(float));
  float* hi = exact(np * sizeof(float));
  float* scales = exact(np * sizeof(float));
  int8_t* q = exact(n);
  CHECK(bqo_compute_range(x, shape, rank, &s, lo, hi) == 0);
  bqo_compute_q_params(lo, hi, np, value, scales);
  CHECK(bqo_quantize(x, shape, rank, &s, scales, q) == 0);
  CHECK(bqo_compute_range_abs_mean(x, shape, rank, &s, lo, hi) == 0);
  for (size_t i = 0; i < np; ++i) CHECK(hi[i] >= 0.0f && lo[i] == -hi[i]);
  int8_t* q2 = exact(n);
  float* scales2 = exact(np * sizeof(float));
  CHECK(bqo_quantize_dynamic(x, shape, rank, &s, q2, scales2) == 0);
  CHECK(memcmp(q, q2, n) == 0 && memcmp(scales, scales2, np * sizeof(float)) == 0);
  /* (the threaded variants take per-tensor schemes and blocks along the last dim; -1 otherwise) */
  if (bqo_quantize_dynamic_mt(x, shape, rank, &s, q2, scales2) == 0)
    CHECK(memcmp(q, q2, n) == 0 && memcmp(scales, scales2, np * sizeof(float)) == 0);
  float* d = exact(n * sizeof(float));
  float* d2 = exact(n * sizeof(float));
  CHECK(bqo_dequantize(q, shape, rank, &s, scales, d) == 0);
  if (bqo_dequantize_mt(q, shape, rank, &s, scales, d2) == 0) CHECK(memcmp(d, d2, n * sizeof(float)) == 0);
  for (size_t i = 0; i < n; i += 13) (void)bqo_block_of(shape, rank, &s, i);
  const size_t nq = (size_t)bqo_num_quants(value);
  if (store == BQO_STORE_NATIVE || shape[rank - 1] % nq == 0) {
    const size_t len = bqo_quantized_data_len(shape, rank, &s);
    uint8_t* blob = exact(len);
    CHECK(bqo_encode(q, shape, rank, &s, scales, blob) == len);
    memset(q2, 0x55, n);
    CHECK(bqo_decode(blob, len, shape, rank, &s, q2, scales2) == 0);
    CHECK(memcmp(q, q2, n) == 0 && memcmp(scales, scales2, np * sizeof(float)) == 0);
    if (len > 0) CHECK(bqo_decode(blob, len - 1, shape, rank, &s, q2, scales2) != 0);
    free(blob);
  }
  if (shape[rank - 1] % nq == 0) {
    bqo_scheme packed = s;
    packed.store = BQO_STORE_PACKED_U32;
    const size_t words = bqo_storage_elements(shape, rank, &packed);
    uint32_t* w = exact(words * 4);
    bqo_pack_u32(q, shape, rank, value, w);
    bqo_unpack_u32(w, shape, rank, value, q2);
    CHECK(memcmp(q, q2, n) == 0);
    free(w);
  }
  if (rank == 2) {
    const size_t m = 3, k = shape[0], nn = shape[1];
    float* lhs = exact(m * k * sizeof(float));
    for (size_t i = 0; i < m * k; ++i) lhs[i] = next_float();
    float* out = exact(m * nn * sizeof(float));
    CHECK(bqo_q_matmul(lhs, m, q, shape, &s, scales, out) == 0);
    if (!block) bqo_ternary_matmul(lhs, m, k, nn, q, scales[0], out);
    free(lhs);
    free(out);
  }
  free(x); free(lo); free(hi); free(scales); free(scales2); free(q); free(q2); free(d); free(d2);
}

int main(void) {
  static const int values[] = {BQO_Q8S, BQO_Q4S, BQO_Q2S, BQO_Q8F, BQO_Q4F, BQO_Q2F};
  int cases = 0;
  for (unsigned vi = 0; vi < sizeof values / sizeof values[0]; ++vi) {
    const int value = values[vi];
    for (int store = 0; store < 2; ++store) {
      { const size_t sh[] = {1}; one_case(sh, 1, value, BQO_STORE_NATIVE, NULL, 0); ++cases; }
      { const size_t sh[] = {67}; one_case(sh, 1, value, BQO_STORE_NATIVE, NULL, 0); ++cases; }
      { const size_t sh[] = {3, 48}; one_case(sh, 2, value, store, NULL, 0); ++cases; }
      { const size_t sh[] = {5, 64}; const unsigned char b[] = {32}; one_case(sh, 2, value, store, b, 1); ++cases; }
      { const size_t sh[] = {6, 32}; const unsigned char b[] = {2, 16}; one_case(sh, 2, value, store, b, 2); ++cases; }
      { const size_t sh[] = {2, 9, 16}; const unsigned char b[] = {3, 8}; one_case(sh, 3, value, store, b, 2); ++cases; }
      { const size_t sh[] = {2, 3, 4, 16}; const unsigned char b[] = {1, 3, 2, 16}; one_case(sh, 4, value, store, b, 4); ++cases; }
    }
  }
  /* scale dtypes: every exponent, both signs, the specials */
  for (int dt = BQO_SCALE_F32; dt <= BQO_SCALE_UE4M3; ++dt) {
    float vals[600];
    size_t n = 0;
    for (int e = -149; e <= 127 && n < 590; e += 1) vals[n++] = ldexpf(1.0f + (float)(next_u32() % 1000) / 1000.0f, e);
    vals[n++] = 0.0f; vals[n++] = INFINITY; vals[n++] = 3.4e38f; vals[n++] = 65504.0f; vals[n++] = 448.0f; vals[n++] = 1e-45f;
    float* up = exact(n * sizeof(float));
    for (size_t i = 0; i < n; ++i) up[i] = bqo_scale_to_dtype(vals[i], dt);
    uint8_t* wire = exact(n * bqo_scale_size(dt));
    float* back = exact(n * sizeof(float));
    bqo_encode_scales(up, n, dt, wire);
    bqo_decode_scales(wire, n, dt, back);
    /* (a rounded finite scale is a fixed point of the codec; what the codec makes of an infinity is not checked) */
    for (size_t i = 0; i < n; ++i) CHECK(!isfinite(up[i]) || back[i] == up[i]);
    if (dt == BQO_SCALE_F16 || dt == BQO_SCALE_UE4M3) {
      float* stored = exact(n * sizeof(float));
      float* eff = exact(n * sizeof(float));
      float* copy = exact(n * sizeof(float));
      size_t m = 0;
      for (size_t i = 0; i < n; ++i) if (isfinite(vals[i]) && vals[i] < 1e30f) copy[m++] = vals[i];
      const float global = bqo_normalize_scales(copy, m, dt);
      CHECK(global > 0.0f);
      m = 0;
      for (size_t i = 0; i < n; ++i) if (isfinite(vals[i]) && vals[i] < 1e30f) copy[m++] = vals[i];
      bqo_two_level_scales(copy, m, dt, global, stored, eff);
      free(stored); free(eff); free(copy);
    }
    free(up); free(wire); free(back);
  }
  printf("oracle_sanitize: %d quantize cases and 4 scale dtypes, no report\n", cases);
  return 0;
}
