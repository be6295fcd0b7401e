/*
 * A caller of libburnq_mi355.so written in plain C (C99, no HIP headers, no Python): what a Rust
 * `extern "C"` binding sees. It walks the reference's own known-answer cases through the handle
 * level of the ABI and exits 0 when every one holds.
 *
 *   c_abi_driver            needs a GPU: quantize / dequantize / q_matmul / layout cases
 *   c_abi_driver --no-gpu   host-only entry points (sizes, refusals), runs anywhere
 *   c_abi_driver --latency  needs a GPU: the call latencies of the reference's own quantization benchmark
 *                           (crates/burn-backend-tests/benches/quantization_ops.rs:26-205), one JSON line
 *
 * Expected values are the literals of burn's tests:
 *   crates/burn-ndarray/src/ops/quantization.rs:164-177            (x -> q, q -> x^)
 *   crates/burn-backend-tests/tests/tensor/float/quantization/ops/quantize.rs:25-93
 *   crates/burn-std/src/tensor/quantization.rs:551-578              (packed word 2147287680)
 *   crates/burn-store/src/tensor_snapshot.rs:517-541               (packed Q4 data_len)
 *   crates/burn-backend-tests/tests/tensor/float/quantization/ops/matmul.rs:141-168
 */
#define _POSIX_C_SOURCE 200809L /* clock_gettime under -std=c99 */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

#include "burnq.h"

static int failures = 0;

#define CHECK(cond, ...)                        \
  do {                                          \
    if (!(cond)) {                              \
      ++failures;                               \
      fprintf(stderr, "FAIL %s:%d: ", __FILE__, __LINE__); \
      fprintf(stderr, __VA_ARGS__);             \
      fprintf(stderr, "\n");                    \
    }                                           \
  } while (0)

#define OK(call)                                                                   \
  do {                                                                             \
    bq_status st_ = (call);                                                        \
    if (st_ != BQ_OK) {                                                            \
      fprintf(stderr, "FAIL %s:%d: %s -> %d (%s)\n", __FILE__, __LINE__, #call, (int)st_, bq_last_error()); \
      exit(2);                                                                     \
    }                                                                              \
  } while (0)

static bq_scheme scheme_of(int value, int store, int block) {
  bq_scheme s;
  memset(&s, 0, sizeof s);
  s.value = (uint8_t)value;
  s.store = (uint8_t)store;
  s.scale_dtype = BQ_SCALE_F32;
  if (block > 0) {
    s.level = BQ_LEVEL_BLOCK;
    s.block_rank = 1;
    s.block[0] = (uint8_t)block;
  } else {
    s.level = BQ_LEVEL_TENSOR;
  }
  return s;
}

static void host_only(void) {
  /* packed Q4S blobs: [3,3] -> 16 bytes, [2,5,9] -> 84, [4,8] -> 20 */
  const size_t shapes[3][3] = {{3, 3, 0}, {2, 5, 9}, {4, 8, 0}};
  const int ranks[3] = {2, 3, 2};
  const size_t want[3] = {16, 84, 20};
  bq_scheme q4 = scheme_of(BQ_Q4S, BQ_STORE_PACKED_U32, 0);
  for (int i = 0; i < 3; ++i) {
    size_t len = 0;
    OK(bq_quantized_data_len(&q4, shapes[i], ranks[i], &len));
    CHECK(len == want[i], "data_len case %d: %zu, expected %zu", i, len, want[i]);
  }
  /* a block that does not divide the shape is refused with a message, not a crash */
  bq_scheme blk = scheme_of(BQ_Q8S, BQ_STORE_NATIVE, 32);
  const size_t bad[1] = {48};
  size_t len = 0;
  bq_status st = bq_quantized_data_len(&blk, bad, 1, &len);
  CHECK(st == BQ_ERR_SHAPE, "48 values in blocks of 32: status %d", (int)st);
  CHECK(strlen(bq_last_error()) > 0, "an error leaves a message");
  CHECK(bq_quantize_dynamic(NULL, &blk, NULL) == BQ_ERR_NULL, "null arguments are refused");
}

static void quantize_cases(bq_device* dev) {
  const float x[4] = {-1.8f, -1.0f, 0.0f, 0.5f};
  const size_t shape[1] = {4};
  bq_tensor *tx = NULL, *ts = NULL, *tq = NULL, *td = NULL;
  OK(bq_float_from_data(dev, x, BQ_F32, shape, 1, &tx));

  /* quantize with the given scale 0.014173228 -> [-127, -71, 0, 35]; blob = values || scale */
  const float scale[1] = {0.014173228f};
  const size_t one[1] = {1};
  OK(bq_float_from_data(dev, scale, BQ_F32, one, 1, &ts));
  bq_scheme native = scheme_of(BQ_Q8S, BQ_STORE_NATIVE, 0);
  OK(bq_quantize(tx, &native, ts, &tq));
  uint8_t blob[64];
  size_t len = 0;
  OK(bq_q_into_data(tq, blob, sizeof blob, &len));
  const int8_t want_q[4] = {-127, -71, 0, 35};
  CHECK(len == 8, "native per-tensor blob of 4 values: %zu bytes", len);
  CHECK(memcmp(blob, want_q, 4) == 0, "quantized values %d %d %d %d", (int8_t)blob[0], (int8_t)blob[1], (int8_t)blob[2], (int8_t)blob[3]);
  CHECK(memcmp(blob + 4, scale, 4) == 0, "the stored scale is the given one");

  /* dequantize -> [-1.8, -1.0062993, 0.0, 0.496063], exactly */
  const float want_d[4] = {-1.8f, -1.0062993f, 0.0f, 0.496063f};
  float d[4];
  OK(bq_dequantize(tq, BQ_F32, &td));
  OK(bq_float_into_data(td, d, sizeof d));
  CHECK(memcmp(d, want_d, sizeof d) == 0, "dequantized %.9g %.9g %.9g %.9g", d[0], d[1], d[2], d[3]);
  bq_tensor_release(td);
  bq_tensor_release(tq);

  /* the same through the packed store: one word, same bytes */
  bq_scheme packed = scheme_of(BQ_Q8S, BQ_STORE_PACKED_U32, 0);
  OK(bq_quantize(tx, &packed, ts, &tq));
  OK(bq_q_into_data(tq, blob, sizeof blob, &len));
  CHECK(len == 8 && memcmp(blob, want_q, 4) == 0, "packed blob");
  bq_tensor_release(tq);
  bq_tensor_release(ts);
  bq_tensor_release(tx);

  /* quantize_dynamic [5, 0, 4, -12.7] -> [50, 0, 40, -127], scale 0.1 */
  const float y[4] = {5.0f, 0.0f, 4.0f, -12.7f};
  OK(bq_float_from_data(dev, y, BQ_F32, shape, 1, &tx));
  OK(bq_quantize_dynamic(tx, &native, &tq));
  OK(bq_q_into_data(tq, blob, sizeof blob, &len));
  const int8_t want_y[4] = {50, 0, 40, -127};
  const float tenth = 0.1f;
  CHECK(memcmp(blob, want_y, 4) == 0 && memcmp(blob + 4, &tenth, 4) == 0, "quantize_dynamic blob");
  bq_tensor_release(tq);
  bq_tensor_release(tx);

  /* pack_i8s_to_u32: [-128, 2, -3, 127] is the word 2147287680; a blob loads and comes back unchanged */
  uint8_t in[8];
  const uint32_t word = 2147287680u;
  const float s1 = 1.0f;
  memcpy(in, &word, 4);
  memcpy(in + 4, &s1, 4);
  OK(bq_q_from_data(dev, in, 8, shape, 1, &packed, &tq));
  OK(bq_dequantize(tq, BQ_F32, &td));
  OK(bq_float_into_data(td, d, sizeof d));
  CHECK(d[0] == -128.0f && d[1] == 2.0f && d[2] == -3.0f && d[3] == 127.0f, "unpacked %g %g %g %g", d[0], d[1], d[2], d[3]);
  OK(bq_q_into_data(tq, blob, sizeof blob, &len));
  CHECK(len == 8 && memcmp(blob, in, 8) == 0, "blob -> tensor -> blob");
  bq_tensor_release(td);
  bq_tensor_release(tq);
}

static void matmul_case(bq_device* dev) {
  /* float lhs x quantized rhs (per-tensor Q8S), expected within rel 5e-3 / abs 1e-5 of the literals */
  const float lhs[12] = {1.0f, 6.35f, 2.0f, 3.0f, 2.0f, 3.0f, 4.0f, 5.0f, 1.0f, 3.0f, 5.0f, 7.0f};
  const float rhs[16] = {4.0f, 8.0f, 12.7f, 1.6f, 2.0f, 3.0f, 6.0f, 4.0f, 1.0f, 5.0f, 9.0f, 2.5f, 3.0f, 7.0f, 11.0f, 0.5f};
  const float want[12] = {27.7f, 58.05f, 101.8f, 33.5f, 33.0f, 80.0f, 134.4f, 27.7f, 36.0f, 91.0f, 152.7f, 29.6f};
  const size_t ls[2] = {3, 4}, rs[2] = {4, 4};
  for (int store = 0; store < 2; ++store) {
    bq_tensor *tl = NULL, *tr = NULL, *tq = NULL, *to = NULL, *tt = NULL, *td = NULL;
    OK(bq_float_from_data(dev, lhs, BQ_F32, ls, 2, &tl));
    OK(bq_float_from_data(dev, rhs, BQ_F32, rs, 2, &tr));
    bq_scheme s = scheme_of(BQ_Q8S, store ? BQ_STORE_PACKED_U32 : BQ_STORE_NATIVE, 0);
    OK(bq_quantize_dynamic(tr, &s, &tq));
    OK(bq_q_matmul(tl, tq, &to));
    float out[12];
    OK(bq_float_into_data(to, out, sizeof out));
    for (int i = 0; i < 12; ++i)
      CHECK(fabsf(out[i] - want[i]) <= 5e-3f * fabsf(want[i]) + 1e-5f, "q_matmul[%d] = %g, expected %g", i, out[i], want[i]);
    /* swap_dims twice is the identity on the dequantized values */
    float d0[16], d1[16];
    OK(bq_dequantize(tq, BQ_F32, &td));
    OK(bq_float_into_data(td, d0, sizeof d0));
    bq_tensor_release(td);
    OK(bq_q_swap_dims(tq, 0, 1, &tt));
    OK(bq_dequantize(tt, BQ_F32, &td));
    OK(bq_float_into_data(td, d1, sizeof d1));
    for (int r = 0; r < 4; ++r)
      for (int c = 0; c < 4; ++c) CHECK(d1[c * 4 + r] == d0[r * 4 + c], "transposed (%d, %d)", r, c);
    bq_tensor_release(td);
    bq_tensor_release(tt);
    bq_tensor_release(to);
    bq_tensor_release(tq);
    bq_tensor_release(tr);
    bq_tensor_release(tl);
  }
}

/* ---- the reference's benchmark, timed from C ----------------------------------------------------
 * Per-tensor Q8S, Native store, inputs (i % 1000) / 1000 - 0.5, every call followed by a device sync
 * (`bench_synced`): `quantize` builds the tensor from host data inside the timed call (make_tensor in
 * the closure, quantization_ops.rs:63-80), `dequantize` and `q_matmul` work on tensors made before.
 * Medians of 400 calls after 20 untimed ones, microseconds. */
static double now_us(void) {
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (double)ts.tv_sec * 1e6 + (double)ts.tv_nsec * 1e-3;
}

static int cmp_double(const void* a, const void* b) {
  const double x = *(const double*)a, y = *(const double*)b;
  return (x > y) - (x < y);
}

enum { LAT_REPS = 400, LAT_WARM = 20 };

typedef struct lat_case {
  bq_device* dev;
  const float* host;
  size_t shape[2];
  int rank;
  bq_scheme scheme;
  bq_tensor *x, *q, *q2;
} lat_case;

static void lat_sync(lat_case* c) { (void)c; }
static void lat_upload_quantize(lat_case* c) {
  bq_tensor *x = NULL, *q = NULL;
  OK(bq_float_from_data(c->dev, c->host, BQ_F32, c->shape, c->rank, &x));
  OK(bq_quantize_dynamic(x, &c->scheme, &q));
  OK(bq_tensor_release(x));
  OK(bq_tensor_release(q));
}
static void lat_quantize(lat_case* c) {
  bq_tensor* q = NULL;
  OK(bq_quantize_dynamic(c->x, &c->scheme, &q));
  OK(bq_tensor_release(q));
}
static void lat_dequantize(lat_case* c) {
  bq_tensor* y = NULL;
  OK(bq_dequantize(c->q, BQ_F32, &y));
  OK(bq_tensor_release(y));
}
static void lat_matmul(lat_case* c) {
  bq_tensor* y = NULL;
  OK(bq_q_matmul(c->q, c->q2, &y));
  OK(bq_tensor_release(y));
}

static double median_us(void (*fn)(lat_case*), lat_case* c) {
  static double t[LAT_REPS];
  for (int i = 0; i < LAT_WARM; ++i) {
    fn(c);
    OK(bq_device_sync(c->dev));
  }
  for (int i = 0; i < LAT_REPS; ++i) {
    const double t0 = now_us();
    fn(c);
    OK(bq_device_sync(c->dev));
    t[i] = now_us() - t0;
  }
  qsort(t, LAT_REPS, sizeof t[0], cmp_double);
  return 0.5 * (t[LAT_REPS / 2 - 1] + t[LAT_REPS / 2]);
}

static void latency(bq_device* dev) {
  static const struct { const char* name; size_t rows, cols; } sizes[] = {
      {"4K", 64, 64}, {"64K", 256, 256}, {"1M", 1024, 1024}, {"q_matmul", 64, 64}, {"q_matmul", 256, 256}, {"q_matmul", 512, 512}};
  lat_case c;
  memset(&c, 0, sizeof c);
  c.dev = dev;
  c.scheme = scheme_of(BQ_Q8S, BQ_STORE_NATIVE, 0);
  printf("{\"sync_only_us\": %.2f", median_us(lat_sync, &c));
  for (size_t s = 0; s < sizeof sizes / sizeof sizes[0]; ++s) {
    const size_t n = sizes[s].rows * sizes[s].cols;
    float* host = (float*)malloc(n * sizeof(float));
    for (size_t i = 0; i < n; ++i) host[i] = (float)(i % 1000) / 1000.0f - 0.5f;
    c.host = host;
    const int matmul = sizes[s].name[0] == 'q';
    c.rank = matmul ? 2 : 1;
    c.shape[0] = matmul ? sizes[s].rows : n;
    c.shape[1] = sizes[s].cols;
    OK(bq_float_from_data(dev, host, BQ_F32, c.shape, c.rank, &c.x));
    OK(bq_quantize_dynamic(c.x, &c.scheme, &c.q));
    OK(bq_quantize_dynamic(c.x, &c.scheme, &c.q2));
    if (matmul) {
      printf(", \"q_matmul_%zux%zu_us\": %.2f", sizes[s].rows, sizes[s].cols, median_us(lat_matmul, &c));
    } else {
      printf(", \"%s\": {\"quantize_with_upload_us\": %.2f, \"quantize_us\": %.2f, \"dequantize_us\": %.2f}", sizes[s].name,
             median_us(lat_upload_quantize, &c), median_us(lat_quantize, &c), median_us(lat_dequantize, &c));
    }
    OK(bq_tensor_release(c.x));
    OK(bq_tensor_release(c.q));
    OK(bq_tensor_release(c.q2));
    free(host);
  }
  printf("}\n");
}

int main(int argc, char** argv) {
  if (argc > 1 && strcmp(argv[1], "--latency") == 0) {
    bq_device* dev = NULL;
    OK(bq_device_open(0, &dev));
    latency(dev);
    OK(bq_device_close(dev));
    return 0;
  }
  host_only();
  if (argc > 1 && strcmp(argv[1], "--no-gpu") == 0) {
    printf(failures ? "c_abi_driver: %d failure(s)\n" : "c_abi_driver: host-only cases ok\n", failures);
    return failures ? 1 : 0;
  }
  bq_device* dev = NULL;
  OK(bq_device_open(0, &dev));
  quantize_cases(dev);
  matmul_case(dev);
  OK(bq_device_sync(dev));
  OK(bq_device_close(dev));
  printf(failures ? "c_abi_driver: %d failure(s)\n" : "c_abi_driver: all cases ok\n", failures);
  return failures ? 1 : 0;
}
