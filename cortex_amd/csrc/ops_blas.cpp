// ops_blas.cpp -- gemm! (src/cortex/tensor/math.clj:106-114) on rocBLAS.  It is
// a plain library matrix product (the reference's backends call netlib BLAS and
// cuBLAS for it, src/cortex/compute/cpu/tensor_math.clj:672-726,
// src/cortex/compute/cuda/tensor_math.clj:633-660), so the vendor library's MFMA
// kernels are the right tool; nothing is hand-written here.  gemv!, which is
// bound by memory rather than by the matrix cores, lives in ops_gemv.hip.
//
// The tensors are row-major and BLAS is column-major: a row-major matrix with
// row pitch ld is the column-major matrix of its transpose with leading
// dimension ld, and C^T = op(B)^T op(A)^T, which is the operand swap of
// col->row-gemm (src/cortex/compute/math_util.clj:17-31).
//
// rocBLAS is loaded on first use (dlopen), so the library loads, and every
// other entry point works, on a machine without it.  One handle per host thread
// and device, destroyed when the thread ends; atomics are switched off so results
// do not depend on scheduling.
#include <dlfcn.h>
#include <rocblas/rocblas.h>

#include <map>
#include <mutex>
#include <thread>

#include "common.h"

using namespace cthip;

namespace {

struct RocblasApi {
  decltype(&rocblas_create_handle) create_handle = nullptr;
  decltype(&rocblas_destroy_handle) destroy_handle = nullptr;
  decltype(&rocblas_set_stream) set_stream = nullptr;
  decltype(&rocblas_set_atomics_mode) set_atomics_mode = nullptr;
  decltype(&rocblas_set_pointer_mode) set_pointer_mode = nullptr;
  decltype(&rocblas_sgemm) sgemm = nullptr;
  decltype(&rocblas_dgemm) dgemm = nullptr;
  decltype(&rocblas_sgemm_strided_batched) sgemm_batched = nullptr;
  decltype(&rocblas_dgemm_strided_batched) dgemm_batched = nullptr;
  decltype(&rocblas_status_to_string) status_to_string = nullptr;
  bool ok = false;
  char why[256] = "";
};

RocblasApi* rocblas_api() {
  static RocblasApi api;
  static std::once_flag once;
  std::call_once(once, [] {
    void* h = nullptr;
    for (const char* name : {"librocblas.so.5", "librocblas.so", "/opt/rocm/lib/librocblas.so"}) {
      h = dlopen(name, RTLD_NOW | RTLD_LOCAL);
      if (h) break;
    }
    if (!h) {
      snprintf(api.why, sizeof(api.why), "cannot load librocblas.so: %s", dlerror());
      return;
    }
#define CT_SYM(field, sym)                                                            \
  api.field = reinterpret_cast<decltype(api.field)>(dlsym(h, #sym));                  \
  if (!api.field) { snprintf(api.why, sizeof(api.why), "librocblas.so lacks %s", #sym); return; }
    CT_SYM(create_handle, rocblas_create_handle)
    CT_SYM(destroy_handle, rocblas_destroy_handle)
    CT_SYM(set_stream, rocblas_set_stream)
    CT_SYM(set_atomics_mode, rocblas_set_atomics_mode)
    CT_SYM(set_pointer_mode, rocblas_set_pointer_mode)
    CT_SYM(sgemm, rocblas_sgemm)
    CT_SYM(dgemm, rocblas_dgemm)
    CT_SYM(sgemm_batched, rocblas_sgemm_strided_batched)
    CT_SYM(dgemm_batched, rocblas_dgemm_strided_batched)
    CT_SYM(status_to_string, rocblas_status_to_string)
#undef CT_SYM
    api.ok = true;
  });
  return &api;
}

#define CT_BLAS(api, expr)                                                                              \
  do {                                                                                                  \
    rocblas_status st__ = (expr);                                                                       \
    if (st__ != rocblas_status_success)                                                                 \
      return set_error(CT_ERR_HIP, "%s failed: %s", #expr, (api)->status_to_string(st__));              \
  } while (0)

// A host thread's handles, one per device, destroyed with the thread so that a
// pool that retires threads does not pile up rocBLAS workspaces.  The thread
// that loaded this library (normally the main one) keeps its handles until the
// process ends: its thread-local destructors run inside exit(), where tearing
// down a GPU library object is not worth the risk.
const std::thread::id g_loader_thread = std::this_thread::get_id();

struct HandleCache {
  std::map<int, rocblas_handle> handles;
  ~HandleCache() {
    if (std::this_thread::get_id() == g_loader_thread) return;
    RocblasApi* api = rocblas_api();
    if (!api->ok) return;
    for (auto& kv : handles)
      if (kv.second) api->destroy_handle(kv.second);
  }
};

// The calling thread's handle for the current device, bound to `s`.
int blas_handle(hipStream_t s, RocblasApi** api_out, rocblas_handle* out) {
  RocblasApi* api = rocblas_api();
  if (!api->ok) return set_error(CT_ERR_UNSUPPORTED, "gemm! needs rocBLAS: %s", api->why);
  int dev = 0;
  CT_HIP(hipGetDevice(&dev));
  thread_local HandleCache cache;
  rocblas_handle& h = cache.handles[dev];
  if (!h) {
    CT_BLAS(api, api->create_handle(&h));
    CT_BLAS(api, api->set_atomics_mode(h, rocblas_atomics_not_allowed));
    CT_BLAS(api, api->set_pointer_mode(h, rocblas_pointer_mode_host));
  }
  CT_BLAS(api, api->set_stream(h, s));
  *api_out = api;
  *out = h;
  return CT_OK;
}

inline rocblas_operation op_of(bool trans) { return trans ? rocblas_operation_transpose : rocblas_operation_none; }
inline bool fits_int(int64_t v) { return v >= 0 && v <= 2147483647; }

}  // namespace

namespace cthip {

// `batch_count` products of ct_gemm's form in one launch: product i reads
// a + i * a_stride, b + i * b_stride and writes c + i * c_stride (strides in
// elements; 0 shares an operand among the products).  Used by the convolution
// methods, whose per-image products are too small to fill the device one at a time.
int gemm_strided_batched(void* stream, void* c, int64_t c_colstride, int64_t c_stride, int trans_a, int trans_b,
                         double alpha, const void* a, int64_t a_row_count, int64_t a_col_count, int64_t a_colstride,
                         int64_t a_stride, const void* b, int64_t b_col_count, int64_t b_colstride, int64_t b_stride,
                         double beta, int64_t batch_count, int dtype) {
  CT_REQUIRE(dtype == CT_F32 || dtype == CT_F64, "gemm! is only defined for float and double tensors");
  CT_REQUIRE(a && b && c, "gemm: null buffer");
  CT_REQUIRE(fits_int(a_row_count) && fits_int(a_col_count) && fits_int(b_col_count) && fits_int(a_colstride) &&
                 fits_int(b_colstride) && fits_int(c_colstride) && fits_int(batch_count),
             "gemm: a size is negative or exceeds 2^31 - 1");
  if (a_row_count == 0 || b_col_count == 0 || batch_count == 0) return CT_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  RocblasApi* api;
  rocblas_handle h;
  if (int rc = blas_handle(s, &api, &h)) return rc;
  note_kernel("rocblas_gemm_strided_batched");
  const rocblas_int m = (rocblas_int)b_col_count, n = (rocblas_int)a_row_count, k = (rocblas_int)a_col_count;
  if (dtype == CT_F32) {
    const float al = (float)alpha, be = (float)beta;
    CT_BLAS(api, api->sgemm_batched(h, op_of(trans_b), op_of(trans_a), m, n, k, &al, (const float*)b,
                                    (rocblas_int)b_colstride, b_stride, (const float*)a, (rocblas_int)a_colstride,
                                    a_stride, &be, (float*)c, (rocblas_int)c_colstride, c_stride,
                                    (rocblas_int)batch_count));
  } else {
    CT_BLAS(api, api->dgemm_batched(h, op_of(trans_b), op_of(trans_a), m, n, k, &alpha, (const double*)b,
                                    (rocblas_int)b_colstride, b_stride, (const double*)a, (rocblas_int)a_colstride,
                                    a_stride, &beta, (double*)c, (rocblas_int)c_colstride, c_stride,
                                    (rocblas_int)batch_count));
  }
  return after_launch(s);
}

}  // namespace cthip

extern "C" {

int ct_gemm(void* stream, void* c, int64_t c_colstride, int trans_a, int trans_b, double alpha, const void* a,
            int64_t a_row_count, int64_t a_col_count, int64_t a_colstride, const void* b, int64_t b_col_count,
            int64_t b_colstride, double beta, int dtype) {
  CT_REQUIRE(dtype == CT_F32 || dtype == CT_F64, "gemm! is only defined for float and double tensors");
  CT_REQUIRE(a && b && c, "ct_gemm: null buffer");
  CT_REQUIRE(fits_int(a_row_count) && fits_int(a_col_count) && fits_int(b_col_count) && fits_int(a_colstride) &&
                 fits_int(b_colstride) && fits_int(c_colstride),
             "ct_gemm: a size is negative or exceeds 2^31 - 1");
  if (a_row_count == 0 || b_col_count == 0) return CT_OK;
  // leading dimensions must cover a stored row: the stored matrix is [rows, cols] before the transposition
  CT_REQUIRE(c_colstride >= b_col_count, "ct_gemm: C column stride %lld is shorter than its %lld columns",
             (long long)c_colstride, (long long)b_col_count);
  CT_REQUIRE(a_colstride >= (trans_a ? a_row_count : a_col_count), "ct_gemm: A column stride is shorter than its rows");
  CT_REQUIRE(b_colstride >= (trans_b ? a_col_count : b_col_count), "ct_gemm: B column stride is shorter than its rows");
  hipStream_t s = static_cast<hipStream_t>(stream);
  RocblasApi* api;
  rocblas_handle h;
  if (int rc = blas_handle(s, &api, &h)) return rc;
  note_kernel("rocblas_gemm");
  const rocblas_int m = (rocblas_int)b_col_count, n = (rocblas_int)a_row_count, k = (rocblas_int)a_col_count;
  if (dtype == CT_F32) {
    const float al = (float)alpha, be = (float)beta;
    CT_BLAS(api, api->sgemm(h, op_of(trans_b), op_of(trans_a), m, n, k, &al, (const float*)b, (rocblas_int)b_colstride,
                            (const float*)a, (rocblas_int)a_colstride, &be, (float*)c, (rocblas_int)c_colstride));
  } else {
    CT_BLAS(api, api->dgemm(h, op_of(trans_b), op_of(trans_a), m, n, k, &alpha, (const double*)b,
                            (rocblas_int)b_colstride, (const double*)a, (rocblas_int)a_colstride, &beta, (double*)c,
                            (rocblas_int)c_colstride));
  }
  return after_launch(s);
}

}  // extern "C"
