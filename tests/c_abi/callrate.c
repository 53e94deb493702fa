/* What one call of the library costs a caller that is not an interpreter: a plain C99 loop over
 * the C ABI, the way a JNA direct-mapped binding calls it.  Each call below is issued CALLS times
 * back to back on one stream; for each the program prints the host time per call (the loop alone,
 * before the stream is waited for) and the sustained time per call (loop plus the final wait), as
 * one JSON object on stdout.
 *
 * The first three are the launch-bound end of the benchmark's own shapes:
 *   binary-op! :+  float [1024,1024] + [1024] row  (8 MiB: the kernel takes a few microseconds)
 *   unary-reduce! :sum over the rows of a [1024,1024] view
 *   assign-constant! of a [64] vector (the smallest kernel there is)
 * The rest are the calls of one training step of the reference's own networks at their sizes
 * (src/cortex/verify/nn/train.clj:185-187: batches of 128 images of 784 pixels, ten classes; a
 * [64,32,7,7] activation for the spatial forms): bias add and bias gradient of a linear layer, a
 * sum over the batch, softmax, the batch-normalization update and its gradients in both forms,
 * and an Adam step over the 784 x 128 weights of a layer. */
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
enum { BATCH = 128, PIXELS = 784, CLASSES = 10, SB = 64, SC = 32, SE = 49, HIDDEN = 128 };

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

static void *g_stream, *g_x, *g_r, *g_b, *g_s, *g_g, *g_stat[8];

static int issue(int which) {
  const ct_dims full = dims(2, ROWS, COLS, COLS, 1), row = dims(1, COLS, 0, 1, 0);
  const ct_dims cols_view = dims(2, COLS, ROWS, 1, COLS), col_out = dims(2, COLS, 1, 1, 1);
  const ct_dims small = dims(1, 64, 0, 1, 0);
  const ct_dims act = dims(2, BATCH, PIXELS, PIXELS, 1), act_row = dims(1, PIXELS, 0, 1, 0);
  const ct_dims act_t = dims(2, PIXELS, BATCH, 1, PIXELS), act_out = dims(2, PIXELS, 1, 1, 1);
  const ct_dims logits = dims(2, BATCH, CLASSES, CLASSES, 1), logit_row = dims(1, CLASSES, 0, 1, 0);
  void* const* st = g_stat;
  switch (which) {
    case 0: return ct_binary_op(g_stream, g_r, &full, g_x, &full, 1.0, g_b, &row, 1.0, (int64_t)ROWS * COLS, CT_BOP_ADD, CT_F32);
    case 1: return ct_unary_reduce(g_stream, g_s, &col_out, 1.0, g_x, &cols_view, CT_ROP_SUM, CT_F32);
    case 2: return ct_assign_constant(g_stream, g_s, &small, CT_F32, 1.0, 64);
    case 3: return ct_binary_op(g_stream, g_r, &act, g_x, &act, 1.0, g_b, &act_row, 1.0, (int64_t)BATCH * PIXELS, CT_BOP_ADD, CT_F32);
    case 4: return ct_binary_accum(g_stream, g_s, &act_row, 1.0, g_x, &act, 1.0, (int64_t)BATCH * PIXELS, CT_BOP_ADD, 0, 1, CT_F32);
    case 5: return ct_binary_accum(g_stream, g_s, &logit_row, 1.0, g_x, &logits, 1.0, (int64_t)BATCH * CLASSES, CT_BOP_ADD, 0, 1, CT_F32);
    case 6: return ct_unary_reduce(g_stream, g_s, &act_out, 1.0, g_x, &act_t, CT_ROP_SUM, CT_F32);
    case 7: return ct_softmax_eltwise(g_stream, g_r, &logits, g_x, &logits, CT_F32);
    case 8: return ct_batch_normalize_update_and_apply_eltwise(g_stream, g_r, g_x, st[0], st[1], st[2], st[3], 0.9, st[4], st[5],
                                                               1e-3, BATCH, PIXELS, CT_F32);
    case 9: return ct_batch_normalize_gradients_eltwise(g_stream, g_r, st[6], st[7], g_g, g_r, g_x, st[0], st[1], st[4], st[5],
                                                        1e-3, BATCH, PIXELS, CT_F32);
    case 10: return ct_batch_normalize_update_and_apply_spatial(g_stream, g_r, g_x, st[0], st[1], st[2], st[3], 0.9, st[4], st[5],
                                                                1e-3, SB, SC, SE, CT_F32);
    case 11: return ct_batch_normalize_gradients_spatial(g_stream, g_r, st[6], st[7], g_g, g_r, g_x, st[0], st[1], st[4], st[5],
                                                         1e-3, SB, SC, SE, CT_F32);
    case 12: return ct_adam_step(g_stream, CT_F32, 1e-3, 0.9, 0.999, 1e-8, 0.34867844, 0.99004488, 1.0, g_g, g_x, g_r, g_b,
                                 (int64_t)PIXELS * HIDDEN);
    default: return CT_OK;
  }
}

static const char* const kNames[] = {
    "binary_op_bias_add_1024x1024", "unary_reduce_columns_1024x1024", "assign_constant_64",
    "bias_add_128x784", "bias_gradient_128x784", "bias_gradient_128x10", "sum_over_batch_128x784", "softmax_128x10",
    "bn_update_eltwise_128x784", "bn_gradients_eltwise_128x784", "bn_update_spatial_64x32x7x7",
    "bn_gradients_spatial_64x32x7x7", "adam_step_100352"};
enum { N_CASES = (int)(sizeof kNames / sizeof kNames[0]) };

int main(void) {
  CHECK(ct_set_device(0));
  CHECK(ct_stream_create(&g_stream));
  CHECK(ct_malloc(&g_x, sizeof(float) * ROWS * COLS));
  CHECK(ct_malloc(&g_r, sizeof(float) * ROWS * COLS));
  CHECK(ct_malloc(&g_g, sizeof(float) * ROWS * COLS));
  CHECK(ct_malloc(&g_b, sizeof(float) * ROWS * COLS));
  CHECK(ct_malloc(&g_s, sizeof(float) * COLS));
  CHECK(ct_memset(g_stream, g_x, CT_F32, 0.5, (int64_t)ROWS * COLS));
  CHECK(ct_memset(g_stream, g_g, CT_F32, 0.001, (int64_t)ROWS * COLS));
  CHECK(ct_memset(g_stream, g_r, CT_F32, 0.0, (int64_t)ROWS * COLS));
  CHECK(ct_memset(g_stream, g_b, CT_F32, 0.25, (int64_t)ROWS * COLS));
  for (int i = 0; i < 8; ++i) {
    CHECK(ct_malloc(&g_stat[i], sizeof(float) * COLS));
    CHECK(ct_memset(g_stream, g_stat[i], CT_F32, 1.0, COLS));
  }
  CHECK(ct_stream_reserve_scratch(g_stream, 16u << 20, 0));

  double host[N_CASES], sustained[N_CASES];
  for (int which = 0; which < N_CASES; ++which) {
    double t0 = 0, t1 = 0, t2 = 0;
    for (int i = -WARMUP; i < CALLS; ++i) {
      if (i == 0) {
        CHECK(ct_stream_sync(g_stream));
        t0 = now_us();
      }
      CHECK(issue(which));
    }
    t1 = now_us();
    CHECK(ct_stream_sync(g_stream));
    t2 = now_us();
    host[which] = (t1 - t0) / CALLS;
    sustained[which] = (t2 - t0) / CALLS;
  }
  printf("{\"calls\": %d", CALLS);
  for (int which = 0; which < N_CASES; ++which)
    printf(", \"%s\": {\"host_us\": %.3f, \"sustained_us\": %.3f}", kNames[which], host[which], sustained[which]);
  printf("}\n");
  CHECK(ct_free(g_x)); CHECK(ct_free(g_r)); CHECK(ct_free(g_g)); CHECK(ct_free(g_b)); CHECK(ct_free(g_s));
  for (int i = 0; i < 8; ++i) CHECK(ct_free(g_stat[i]));
  CHECK(ct_stream_destroy(g_stream));
  return 0;
}
