/* A caller of the C ABI written in plain C99 against include/cortex_hip.h alone,
 * the way a JNA / JavaCPP binding sees the library: no C++, no HIP headers.
 * It runs the bias add of a [rows, cols] matrix with a [cols] row vector, a
 * row reduction and an Adam step, copies the results back and checks them
 * against the same arithmetic on the host.  Exit status 0 and "ok" on success. */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "cortex_hip.h"

#define CHECK(call)                                                           \
  do {                                                                        \
    int rc_ = (call);                                                         \
    if (rc_ != CT_OK) {                                                       \
      fprintf(stderr, "%s failed (%d): %s\n", #call, rc_, ct_last_error());   \
      return 1;                                                               \
    }                                                                         \
  } while (0)

static ct_dims dims2(int64_t rows, int64_t cols, int64_t row_stride, int64_t col_stride) {
  ct_dims d;
  memset(&d, 0, sizeof d);
  d.ndim = 2;
  d.shape[0] = rows; d.shape[1] = cols;
  d.strides[0] = row_stride; d.strides[1] = col_stride;
  return d;
}

static ct_dims dims1(int64_t n) {
  ct_dims d;
  memset(&d, 0, sizeof d);
  d.ndim = 1;
  d.shape[0] = n;
  d.strides[0] = 1;
  return d;
}

int main(void) {
  enum { ROWS = 37, COLS = 1000, N = ROWS * COLS };
  int count = 0;
  CHECK(ct_device_count(&count));
  if (count < 1) { fprintf(stderr, "no device\n"); return 2; }
  CHECK(ct_set_device(0));
  void* stream = NULL;
  CHECK(ct_stream_create(&stream));

  float* h = NULL;   /* pinned staging: matrix, bias, result, row sums */
  CHECK(ct_host_alloc((void**)&h, sizeof(float) * (2 * N + COLS + ROWS)));
  float *hx = h, *hb = h + N, *hr = hb + COLS, *hs = hr + N;
  for (int i = 0; i < N; ++i) hx[i] = (float)((i * 37) % 101) * 0.125f - 6.0f;
  for (int j = 0; j < COLS; ++j) hb[j] = (float)(j % 17) * 0.5f;

  void *x = NULL, *b = NULL, *r = NULL, *s = NULL;
  CHECK(ct_malloc(&x, sizeof(float) * N));
  CHECK(ct_malloc(&b, sizeof(float) * COLS));
  CHECK(ct_malloc(&r, sizeof(float) * N));
  CHECK(ct_malloc(&s, sizeof(float) * ROWS));
  CHECK(ct_memcpy_async(x, hx, sizeof(float) * N, CT_COPY_HOST_TO_DEVICE, stream));
  CHECK(ct_memcpy_async(b, hb, sizeof(float) * COLS, CT_COPY_HOST_TO_DEVICE, stream));

  /* r = 1.0 * x + 2.0 * bias, the bias broadcast over the rows */
  const ct_dims m = dims2(ROWS, COLS, COLS, 1), v = dims1(COLS), col = dims2(ROWS, 1, 1, 1);
  CHECK(ct_binary_op(stream, r, &m, x, &m, 1.0, b, &v, 2.0, N, CT_BOP_ADD, CT_F32));
  /* s[i] = sum over the row of r */
  CHECK(ct_unary_reduce(stream, s, &col, 1.0, r, &m, CT_ROP_SUM, CT_F32));
  CHECK(ct_memcpy_async(hr, r, sizeof(float) * N, CT_COPY_DEVICE_TO_HOST, stream));
  CHECK(ct_memcpy_async(hs, s, sizeof(float) * ROWS, CT_COPY_DEVICE_TO_HOST, stream));
  CHECK(ct_stream_sync(stream));

  for (int i = 0; i < ROWS; ++i) {
    double sum = 0.0;
    for (int j = 0; j < COLS; ++j) {
      const float want = (float)((double)hx[i * COLS + j] + 2.0 * (double)hb[j]);
      if (hr[i * COLS + j] != want) {
        fprintf(stderr, "bias add mismatch at (%d,%d): %g != %g\n", i, j, hr[i * COLS + j], want);
        return 1;
      }
      sum += (double)want;
    }
    if (fabs((double)hs[i] - sum) > 2e-6 * fabs(sum) + 1e-3) {
      fprintf(stderr, "row sum mismatch at %d: %g != %g\n", i, hs[i], sum);
      return 1;
    }
  }

  /* one Adam step over the matrix as parameters, its own values as gradient */
  void *mm = NULL, *vv = NULL;
  CHECK(ct_malloc(&mm, sizeof(float) * N));
  CHECK(ct_malloc(&vv, sizeof(float) * N));
  CHECK(ct_memset(stream, mm, CT_F32, 0.0, N));
  CHECK(ct_memset(stream, vv, CT_F32, 0.0, N));
  CHECK(ct_adam_step(stream, CT_F32, 0.001, 0.9, 0.999, 1e-8, 0.9, 0.999, 1.0, r, x, mm, vv, N));
  float* hp = hr; /* reuse */
  float* hg = (float*)malloc(sizeof(float) * N);
  memcpy(hg, hr, sizeof(float) * N);
  CHECK(ct_memcpy_async(hp, x, sizeof(float) * N, CT_COPY_DEVICE_TO_HOST, stream));
  CHECK(ct_stream_sync(stream));
  for (int i = 0; i < N; ++i) {
    const double alpha = (double)0.001f, b1 = (double)0.9f, b2 = (double)0.999f, eps = (double)1e-8f;
    const double g = (double)hg[i];
    const double lm = b1 * 0.0 + (1.0 - b1) * g;
    const double lv = b2 * 0.0 + ((1.0 - b2) * g) * g;
    const double dx = alpha * (lm / ((1.0 - b1) * (sqrt(lv / (1.0 - b2)) + eps)));
    const float want = (float)((double)hx[i] - dx);
    if (hp[i] != want) {
      fprintf(stderr, "adam mismatch at %d: %.9g != %.9g\n", i, hp[i], want);
      return 1;
    }
  }
  free(hg);

  /* an invalid call reports through the status and the message, not by aborting */
  if (ct_binary_op(stream, r, &m, x, &m, 1.0, b, &v, 1.0, N, 999, CT_F32) == CT_OK || strlen(ct_last_error()) == 0) {
    fprintf(stderr, "an unknown operation code was accepted\n");
    return 1;
  }

  CHECK(ct_free(x)); CHECK(ct_free(b)); CHECK(ct_free(r)); CHECK(ct_free(s)); CHECK(ct_free(mm)); CHECK(ct_free(vv));
  CHECK(ct_host_free(h));
  CHECK(ct_stream_destroy(stream));
  printf("ok\n");
  return 0;
}
