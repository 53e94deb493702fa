// ops_gemv.hip -- gemv! (src/cortex/tensor/math.clj:115-123;
// src/cortex/compute/cpu/tensor_math.clj:700-726 through col->row-gemv,
// src/cortex/compute/math_util.clj:33-41):
//   y = alpha * op(A) x + beta * y      for a row-major A[rows, cols] with row pitch lda.
// A matrix-vector product reads every matrix element once and does two flops
// with it: it is bound by HBM, not by the matrix cores, so it is written here as
// the two reductions it is rather than handed to the BLAS library (whose gemv
// measured 45-63 % of the HBM peak on row-major A x and 16-35 % on A^T x):
//   gemv_rows_kernel   y[i] = sum_j A[i][j] x[j]: a group of 4 ... 256 lanes walks
//                      four rows at once with 128-bit loads, x comes from the
//                      caches once per four rows, double accumulators,
//                      shuffles (and LDS for 256 lanes)
//   gemv_cols_kernel   y[j] = sum_i A[i][j] x[i]: lanes own columns, the 16 waves
//                      of a block stride down the rows of the block's segment,
//                      partial sums per segment go to scratch memory and
//                      gemv_finish_kernel adds them in a fixed order
// Sums run in double whatever the tensor type (the products of two floats are
// exact in double), so the result is at least as close to the exact product as
// a BLAS in the tensor's own precision; beta == 0 does not read y.
#include <algorithm>

#include "elementwise.h"

using namespace cthip;

namespace {

constexpr int64_t kLim31 = int64_t(1) << 31;

struct GemvArgs {
  const void* a;
  const void* x;
  void* y;
  double* partials;   // [n_seg][cols], column form with more than one segment
  int64_t rows, cols, lda, incx, incy;
  double alpha, beta;  // already rounded to the tensor type
  uint32_t n_seg, rows_per_seg, n_strips;
};

template <class T> __device__ __forceinline__ T gemv_result(const GemvArgs& a, double acc, const T* y) {
  const double prev = a.beta == 0.0 ? 0.0 : a.beta * (double)*y;
  return (T)(a.alpha * acc + prev);
}

// A group of G lanes takes kRowsPerGroup consecutive rows at once, so that every
// vector of x it fetches serves that many rows (with one row per group x costs as
// many cache reads as the matrix).  VEC > 1 needs unit-stride x and rows on the
// 16-byte grid.
constexpr int kRowsPerGroup = 4;

template <class T, int VEC, int G>
__global__ void __launch_bounds__(kBlock) gemv_rows_kernel(const GemvArgs a) {
  using V = Vec<T, VEC>;
  constexpr int U = 2;  // vectors of x in flight per lane, each with kRowsPerGroup vectors of the matrix
  constexpr int R = kRowsPerGroup;
  __shared__ double lds[kBlock / 64][R];
  const int lane = threadIdx.x % G;
  const int64_t row0 = ((int64_t)blockIdx.x * (kBlock / G) + threadIdx.x / G) * R;
  const T* abase = reinterpret_cast<const T*>(a.a);
  const T* x = reinterpret_cast<const T*>(a.x);
  const uint32_t nv = (uint32_t)(a.cols / VEC);
  double acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = 0.0;
  if (row0 < a.rows) {
    // rows past the end read the last row again and are dropped at the store
    const T* arow[R];
#pragma unroll
    for (int r = 0; r < R; ++r) arow[r] = abase + (row0 + r < a.rows ? row0 + r : a.rows - 1) * a.lda;
    for (uint32_t v0 = lane; v0 < nv; v0 += G * U) {
      V av[U][R], xv[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const uint32_t v = v0 + u * G;
        if (v < nv) {
          if constexpr (VEC > 1) xv[u] = reinterpret_cast<const V*>(x)[v];
          else xv[u].v[0] = x[(int64_t)v * a.incx];
#pragma unroll
          for (int r = 0; r < R; ++r) av[u][r] = nt_load(reinterpret_cast<const V*>(arow[r]) + v);
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (v0 + u * G < nv) {
#pragma unroll
          for (int r = 0; r < R; ++r)
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[r] += (double)av[u][r].v[e] * (double)xv[u].v[e];
        }
      }
    }
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
#pragma unroll
    for (int s = (G < 64 ? G : 64) / 2; s >= 1; s >>= 1) acc[r] += __shfl_xor(acc[r], s, 64);
  }
  if constexpr (G == kBlock) {
    if ((threadIdx.x & 63) == 0) {
#pragma unroll
      for (int r = 0; r < R; ++r) lds[threadIdx.x >> 6][r] = acc[r];
    }
    __syncthreads();
    if (threadIdx.x == 0) {
#pragma unroll
      for (int r = 0; r < R; ++r)
#pragma unroll
        for (int w = 1; w < kBlock / 64; ++w) acc[r] += lds[w][r];
    }
  }
  if (lane == 0) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      if (row0 + r < a.rows) {
        T* y = reinterpret_cast<T*>(a.y) + (row0 + r) * a.incy;
        *y = gemv_result<T>(a, acc[r], y);
      }
    }
  }
}

constexpr int kColBlock = 1024;

// Lanes own VEC neighbouring columns; wave w of the block takes rows r0 + w, r0 + w + 16, ...
template <class T, int VEC>
__global__ void __launch_bounds__(kColBlock) gemv_cols_kernel(const GemvArgs a) {
  using V = Vec<T, VEC>;
  constexpr int WAVES = kColBlock / 64;
  constexpr int UN = 8;  // rows in flight per lane
  __shared__ double lds[WAVES - 1][64 * VEC];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t strip = blockIdx.x % a.n_strips, seg = blockIdx.x / a.n_strips;
  const int64_t col = ((int64_t)strip * 64 + lane) * VEC;
  const bool live = col < a.cols;
  const T* x = reinterpret_cast<const T*>(a.x);
  double acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) acc[e] = 0.0;
  const int64_t r0 = (int64_t)seg * a.rows_per_seg;
  const int64_t r1 = r0 + a.rows_per_seg < a.rows ? r0 + a.rows_per_seg : a.rows;
  if (live) {
    const T* p = reinterpret_cast<const T*>(a.a) + col;
    for (int64_t r = r0 + wave; r < r1; r += (int64_t)UN * WAVES) {
      V av[UN];
      T xr[UN];
#pragma unroll
      for (int j = 0; j < UN; ++j) {
        const int64_t rr = r + (int64_t)j * WAVES;
        if (rr < r1) {
          av[j] = nt_load(reinterpret_cast<const V*>(p + rr * a.lda));
          xr[j] = x[rr * a.incx];
        }
      }
#pragma unroll
      for (int j = 0; j < UN; ++j) {
        if (r + (int64_t)j * WAVES < r1) {
          const double xd = (double)xr[j];
#pragma unroll
          for (int e = 0; e < VEC; ++e) acc[e] += (double)av[j].v[e] * xd;
        }
      }
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) lds[wave - 1][e * 64 + lane] = acc[e];
  }
  __syncthreads();
  if (wave == 0 && live) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
#pragma unroll
      for (int w = 0; w < WAVES - 1; ++w) acc[e] += lds[w][e * 64 + lane];
      if (a.n_seg == 1) {
        T* y = reinterpret_cast<T*>(a.y) + (col + e) * a.incy;
        *y = gemv_result<T>(a, acc[e], y);
      } else {
        a.partials[(int64_t)seg * a.cols + col + e] = acc[e];
      }
    }
  }
}

template <class T>
__global__ void __launch_bounds__(kBlock) gemv_finish_kernel(const GemvArgs a) {
  const int64_t j = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (j >= a.cols) return;
  double acc = 0.0;
  for (uint32_t s = 0; s < a.n_seg; ++s) acc += a.partials[(int64_t)s * a.cols + j];
  T* y = reinterpret_cast<T*>(a.y) + j * a.incy;
  *y = gemv_result<T>(a, acc, y);
}

template <class T, int VEC>
void launch_rows(hipStream_t s, const GemvArgs& a) {
  const int64_t nv = a.cols / VEC;
#define CT_GEMV_ROWS(G_)                                                                                         \
  hipLaunchKernelGGL((gemv_rows_kernel<T, VEC, G_>),                                                              \
                     dim3((uint32_t)((a.rows + (kBlock / G_) * kRowsPerGroup - 1) / ((kBlock / G_) * kRowsPerGroup))),   \
                     dim3(kBlock), 0, s, a)
  if (nv >= 1024) CT_GEMV_ROWS(256);
  else if (nv >= 128) CT_GEMV_ROWS(64);
  else if (nv >= 16) CT_GEMV_ROWS(16);
  else CT_GEMV_ROWS(4);
#undef CT_GEMV_ROWS
}

template <class T>
int gemv_typed(hipStream_t s, void* y, int64_t incy, bool trans, double alpha, const void* a_ptr, int64_t rows,
               int64_t cols, int64_t lda, const void* x, int64_t incx, double beta) {
  constexpr int VMAX = 16 / (int)sizeof(T);
  GemvArgs a;
  std::memset(&a, 0, sizeof(a));
  a.a = a_ptr; a.x = x; a.y = y;
  a.rows = rows; a.cols = cols; a.lda = lda; a.incx = incx; a.incy = incy;
  a.alpha = (double)(T)alpha;
  a.beta = (double)(T)beta;
  const bool matrix_vec = (uintptr_t)a_ptr % 16 == 0 && lda % VMAX == 0 && cols % VMAX == 0;
  if (!trans) {
    const bool vec = matrix_vec && incx == 1 && (uintptr_t)x % 16 == 0;
    note_kernel(vec ? "gemv_rows_vec" : "gemv_rows");
    if (vec) launch_rows<T, VMAX>(s, a);
    else launch_rows<T, 1>(s, a);
    return after_launch(s);
  }
  const int vec = matrix_vec ? VMAX : 1;
  a.n_strips = (uint32_t)((cols + 64 * vec - 1) / (64 * vec));
  // rows are cut into segments until about two blocks per compute unit exist; a
  // segment is a whole number of load rounds (16 waves x 8 rows)
  constexpr int64_t kRowQuantum = 128;
  const int64_t want_seg = std::max<int64_t>(1, std::min<int64_t>(512 / a.n_strips, rows / kRowQuantum));
  int64_t per = ((rows + want_seg - 1) / want_seg + kRowQuantum - 1) / kRowQuantum * kRowQuantum;
  // eight rows more per segment, where that leaves their number alone: segment starts a power of
  // two apart advance in step through the same memory channels (see the column reduction)
  if (per < rows && (rows + per + 7) / (per + 8) == (rows + per - 1) / per) per += 8;
  a.rows_per_seg = (uint32_t)per;
  a.n_seg = (uint32_t)((rows + per - 1) / per);
  if (a.n_seg > 1) {
    void* scratch = nullptr;
    if (int rc = stream_scratch(s, (size_t)a.n_seg * cols * sizeof(double), &scratch)) return rc;
    a.partials = reinterpret_cast<double*>(scratch);
  }
  const int64_t grid = (int64_t)a.n_strips * a.n_seg;
  CT_REQUIRE(grid < kLim31, "gemv!: too many columns");
  note_kernel(matrix_vec ? "gemv_cols_vec" : "gemv_cols");
  if (matrix_vec) hipLaunchKernelGGL((gemv_cols_kernel<T, VMAX>), dim3((uint32_t)grid), dim3(kColBlock), 0, s, a);
  else hipLaunchKernelGGL((gemv_cols_kernel<T, 1>), dim3((uint32_t)grid), dim3(kColBlock), 0, s, a);
  if (a.n_seg > 1)
    hipLaunchKernelGGL((gemv_finish_kernel<T>), dim3((uint32_t)((cols + kBlock - 1) / kBlock)), dim3(kBlock), 0, s, a);
  return after_launch(s);
}

inline bool fits_int(int64_t v) { return v >= 0 && v <= 2147483647; }

}  // namespace

extern "C" int ct_gemv(void* stream, void* c, int64_t inc_c, int trans_a, double alpha, const void* a,
                       int64_t a_row_count, int64_t a_col_count, int64_t a_colstride, const void* x, int64_t inc_x,
                       double beta, int dtype) {
  CT_REQUIRE(dtype == CT_F32 || dtype == CT_F64, "gemv! is only defined for float and double tensors");
  CT_REQUIRE(a && x && c, "ct_gemv: null buffer");
  CT_REQUIRE(fits_int(a_row_count) && fits_int(a_col_count) && fits_int(a_colstride) && fits_int(inc_x) &&
                 fits_int(inc_c) && inc_x >= 1 && inc_c >= 1,
             "ct_gemv: a size or increment is out of range");
  CT_REQUIRE(a_colstride >= a_col_count, "ct_gemv: A column stride is shorter than its rows");
  if (a_row_count == 0 || a_col_count == 0) return CT_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == CT_F32)
    return gemv_typed<float>(s, c, inc_c, trans_a != 0, alpha, a, a_row_count, a_col_count, a_colstride, x, inc_x, beta);
  return gemv_typed<double>(s, c, inc_c, trans_a != 0, alpha, a, a_row_count, a_col_count, a_colstride, x, inc_x, beta);
}
