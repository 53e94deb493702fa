/* What one call of the library costs a caller that is not an interpreter: a plain C99 loop over
 * the C ABI, the way a JNA direct-mapped binding calls it.  Three calls are timed, each CALLS
 * times back to back on one stream:
 *   binary-op! :+  float [1024,1024] + [1024] row  (8 MiB: the kernel takes a few microseconds)
 *   unary-reduce! :sum over the rows of a [1024,1024] view (two launches)
 *   assign-constant! of a [64] vector (the smallest kernel there is)
 * For each it prints the host time per call (the loop alone, before the stream is waited for) and
 * the sustained time per call (loop plus the final wait), as one JSON object on stdout. */
#define _POSIX_C_SOURCE 199309L
#include <stdio.h>
#include <string.h>
#include <time.h>

#include "cortex_hip.h"

#define CHECK(call)                                                           \
  do {                                                                        \
    int rc_ = (call);                                                         \
    if (rc_ != CT_OK) {                                                       \
      fprintf(stderr, "%s failed (%d): %s\n", #call, rc_, ct_last_error());   \
      return 1;                                                               \
    }                                                                         \
  } while (0)

enum { ROWS = 1024, COLS = 1024, CALLS = 2000, WARMUP = 200 };

static double now_us(void) {
  struct timespec t;
  clock_gettime(CLOCK_MONOTONIC, &t);
  return (double)t.tv_sec * 1e6 + (double)t.tv_nsec * 1e-3;
}

static ct_dims dims(int ndim, int64_t s0, int64_t s1, int64_t st0, int64_t st1) {
  ct_dims d;
  memset(&d, 0, sizeof d);
  d.ndim = ndim;
  d.shape[0] = s0; d.shape[1] = s1;
  d.strides[0] = st0; d.strides[1] = st1;
  return d;
}

int main(void) {
  CHECK(ct_set_device(0));
  void* stream = NULL;
  CHECK(ct_stream_create(&stream));
  void *x = NULL, *b = NULL, *r = NULL, *s = NULL;
  CHECK(ct_malloc(&x, sizeof(float) * ROWS * COLS));
  CHECK(ct_malloc(&r, sizeof(float) * ROWS * COLS));
  CHECK(ct_malloc(&b, sizeof(float) * COLS));
  CHECK(ct_malloc(&s, sizeof(float) * COLS));
  CHECK(ct_memset(stream, x, CT_F32, 0.5, (int64_t)ROWS * COLS));
  CHECK(ct_memset(stream, b, CT_F32, 0.25, COLS));
  CHECK(ct_stream_reserve_scratch(stream, 16u << 20, 0));

  const ct_dims full = dims(2, ROWS, COLS, COLS, 1), row = dims(1, COLS, 0, 1, 0);
  const ct_dims cols_view = dims(2, COLS, ROWS, 1, COLS), col_out = dims(2, COLS, 1, 1, 1);
  const ct_dims small = dims(1, 64, 0, 1, 0);
  double host[3], sustained[3];
  for (int which = 0; which < 3; ++which) {
    double t0 = 0, t1 = 0, t2 = 0;
    for (int i = -WARMUP; i < CALLS; ++i) {
      if (i == 0) {
        CHECK(ct_stream_sync(stream));
        t0 = now_us();
      }
      if (which == 0)
        CHECK(ct_binary_op(stream, r, &full, x, &full, 1.0, b, &row, 1.0, (int64_t)ROWS * COLS, CT_BOP_ADD, CT_F32));
      else if (which == 1)
        CHECK(ct_unary_reduce(stream, s, &col_out, 1.0, x, &cols_view, CT_ROP_SUM, CT_F32));
      else
        CHECK(ct_assign_constant(stream, s, &small, CT_F32, 1.0, 64));
    }
    t1 = now_us();
    CHECK(ct_stream_sync(stream));
    t2 = now_us();
    host[which] = (t1 - t0) / CALLS;
    sustained[which] = (t2 - t0) / CALLS;
  }
  printf("{\"calls\": %d, \"binary_op_bias_add_1024x1024\": {\"host_us\": %.3f, \"sustained_us\": %.3f}, "
         "\"unary_reduce_columns_1024x1024\": {\"host_us\": %.3f, \"sustained_us\": %.3f}, "
         "\"assign_constant_64\": {\"host_us\": %.3f, \"sustained_us\": %.3f}}\n",
         CALLS, host[0], sustained[0], host[1], sustained[1], host[2], sustained[2]);
  CHECK(ct_free(x)); CHECK(ct_free(r)); CHECK(ct_free(b)); CHECK(ct_free(s));
  CHECK(ct_stream_destroy(stream));
  return 0;
}
