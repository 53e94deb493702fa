// ops_accum.hip -- binary-accum! (src/cortex/tensor/math.clj:53-65;
// src/cortex/compute/cpu/tensor_math.clj:386-420, 1439-1463).
//
//   dest[Ad(e)] = dest[Ad(e)]*dest_alpha op y[Ay(e)]*y_alpha     for e = 0 .. n-1
//
// Without dest_requires_cas every destination element is written once and the
// call is an ordinary in-place binary-op!.  With it, the destination is
// smaller than the operation (a broadcast target: "sum the rows into a
// vector", bias gradients) or indirectly indexed (scatter-add), so several e
// hit one address and the reference applies them serially in increasing e,
// rounding to the tensor datatype after every update.
//
// accum_owner_kernel reproduces exactly that for broadcast destinations:
// one lane owns one destination element and applies its updates in increasing
// e, so the result is bit-identical to the serial loop while all destination
// elements proceed in parallel.  For op :+ with dest_alpha 1 on float/double
// tensors, accum_sum_kernel instead splits each destination element's updates
// over a whole block and sums them in double: faster when the destination is
// tiny, and closer to the exact sum than the reference's float-by-float
// accumulation (which the reference itself only checks to 1e-4,
// src/cortex/verify/tensor.clj:188-191).
// Indirectly indexed destinations fall back to the serial kernel.
#include <algorithm>

#include "elementwise.h"
#include "functors.h"
#include "ops.h"

using namespace cthip;

namespace {

struct OwnerArgs {
  void* dest;
  const void* y;
  int64_t n_dest;   // destination elements (owners)
  int64_t n_red;    // updates per destination element
  int32_t n_kept, n_redax;
  FastDiv ksize[CT_MAX_DIMS];   // kept axes, fastest first
  int64_t kd_stride[CT_MAX_DIMS], ky_stride[CT_MAX_DIMS];
  FastDiv rsize[CT_MAX_DIMS];   // reduced axes, fastest first
  int64_t ry_stride[CT_MAX_DIMS];
  int32_t reverse;
};

template <class T, int OP>
__global__ void __launch_bounds__(kBlock) accum_owner_kernel(const BinaryF<T, OP> f, const OwnerArgs a) {
  const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (t >= a.n_dest) return;
  int64_t doff = 0, ybase = 0;
  uint32_t rem = (uint32_t)t;
  for (int d = 0; d < a.n_kept; ++d) {
    uint32_t q, r;
    a.ksize[d].divmod(rem, q, r);
    rem = q;
    doff += (int64_t)r * a.kd_stride[d];
    ybase += (int64_t)r * a.ky_stride[d];
  }
  T* dp = reinterpret_cast<T*>(a.dest) + doff;
  const T* yp = reinterpret_cast<const T*>(a.y) + ybase;
  T acc = *dp;
  for (uint32_t i = 0; i < (uint32_t)a.n_red; ++i) {
    int64_t yoff = 0;
    uint32_t rr = i;
    for (int d = 0; d < a.n_redax; ++d) {
      uint32_t q, r;
      a.rsize[d].divmod(rr, q, r);
      rr = q;
      yoff += (int64_t)r * a.ry_stride[d];
    }
    const T yv = yp[yoff];
    acc = a.reverse ? f(yv, acc, acc) : f(acc, yv, yv);
  }
  *dp = acc;
}

// One block per destination element: dest = (T)((double)dest + sum of y*ya).
template <class T>
__global__ void __launch_bounds__(kBlock) accum_sum_kernel(const OwnerArgs a, const double ya) {
  __shared__ double lds[kBlock / 64];
  const int64_t t = blockIdx.x;
  int64_t doff = 0, ybase = 0;
  uint32_t rem = (uint32_t)t;
  for (int d = 0; d < a.n_kept; ++d) {
    uint32_t q, r;
    a.ksize[d].divmod(rem, q, r);
    rem = q;
    doff += (int64_t)r * a.kd_stride[d];
    ybase += (int64_t)r * a.ky_stride[d];
  }
  const T* yp = reinterpret_cast<const T*>(a.y) + ybase;
  double acc = 0.0;
  // the fastest reduced axis is walked by the lanes: coalesced when it is unit-stride
  const uint32_t inner = a.rsize[0].d;
  const uint32_t outer = (uint32_t)(a.n_red / inner);
  for (uint32_t o = 0; o < outer; ++o) {
    int64_t yoff = 0;
    uint32_t rr = o;
    for (int d = 1; d < a.n_redax; ++d) {
      uint32_t q, r;
      a.rsize[d].divmod(rr, q, r);
      rr = q;
      yoff += (int64_t)r * a.ry_stride[d];
    }
    for (uint32_t i = threadIdx.x; i < inner; i += kBlock) acc += (double)yp[yoff + (int64_t)i * a.ry_stride[0]] * ya;
  }
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) acc += __shfl_xor(acc, m, 64);
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    double s = lds[0];
    for (int w = 1; w < kBlock / 64; ++w) s += lds[w];
    T* dp = reinterpret_cast<T*>(a.dest) + doff;
    *dp = (T)((double)*dp + s);
  }
}

// Splits the joint iteration space into axes the destination keeps and axes it
// broadcasts over.  Fails (returns false) unless both operands are direct,
// every axis of either operand is 1 or the full size, and n covers the space.
bool owner_structure(const ct_dims& dd, const ct_dims& yd, int64_t n, OwnerArgs* a) {
  if (!dims_direct(dd) || !dims_direct(yd)) return false;
  const int rank = std::max(dd.ndim, yd.ndim);
  int64_t dshape[CT_MAX_DIMS], dstr[CT_MAX_DIMS], yshape[CT_MAX_DIMS], ystr[CT_MAX_DIMS], mx[CT_MAX_DIMS];
  for (int i = 0; i < rank; ++i) {
    const int di = i - (rank - dd.ndim), yi = i - (rank - yd.ndim);
    dshape[i] = di >= 0 ? dd.shape[di] : 1;
    dstr[i] = di >= 0 ? dd.strides[di] : 0;
    yshape[i] = yi >= 0 ? yd.shape[yi] : 1;
    ystr[i] = yi >= 0 ? yd.strides[yi] : 0;
    mx[i] = std::max(dshape[i], yshape[i]);
  }
  int64_t total = 1, n_dest = 1, n_red = 1;
  a->n_kept = a->n_redax = 0;
  for (int i = rank - 1; i >= 0; --i) {  // fastest first
    if (mx[i] >= (int64_t(1) << 31)) return false;
    total *= mx[i];
    if (mx[i] == 1) continue;
    if ((dshape[i] != 1 && dshape[i] != mx[i]) || (yshape[i] != 1 && yshape[i] != mx[i])) return false;
    const int64_t ys = yshape[i] == 1 ? 0 : ystr[i];
    if (dshape[i] == mx[i]) {
      if (dstr[i] < 0) return false;
      a->ksize[a->n_kept] = FastDiv((uint32_t)mx[i]);
      a->kd_stride[a->n_kept] = dstr[i];
      a->ky_stride[a->n_kept] = ys;
      ++a->n_kept;
      n_dest *= mx[i];
    } else {
      a->rsize[a->n_redax] = FastDiv((uint32_t)mx[i]);
      a->ry_stride[a->n_redax] = ys;
      ++a->n_redax;
      n_red *= mx[i];
    }
  }
  if (total != n || n_dest >= (int64_t(1) << 31) || n_red >= (int64_t(1) << 31)) return false;
  if (a->n_redax == 0) { a->rsize[0] = FastDiv(1); a->ry_stride[0] = 0; a->n_redax = 1; }
  a->n_dest = n_dest;
  a->n_red = n_red;
  return true;
}

template <class T, int OP>
int accum_run(hipStream_t s, void* dest, const ct_dims* dd, double dest_alpha, const void* y, const ct_dims* yd,
              double y_alpha, int64_t n, bool reverse) {
  using A = typename acc_of<T>::type;
  BinaryF<T, OP> f;
  // f(first, second) = op(first * xa, second * ya)
  f.xa = reverse ? (A)jvm_cast<T>(y_alpha) : (A)jvm_cast<T>(dest_alpha);
  f.ya = reverse ? (A)jvm_cast<T>(dest_alpha) : (A)jvm_cast<T>(y_alpha);
  f.narrow = 0;  // every update is rounded to T; keep the reference's double route
  OwnerArgs a;
  std::memset(&a, 0, sizeof(a));
  if (owner_structure(*dd, *yd, n, &a)) {
    a.dest = dest;
    a.y = y;
    a.reverse = reverse ? 1 : 0;
    if constexpr (OP == CT_BOP_ADD && std::is_floating_point<T>::value) {
      // few owners, many updates each: sum in double across a block instead
      if (jvm_cast<T>(dest_alpha) == (T)1 && a.n_dest <= 4096 && a.n_red >= 4096) {
        note_kernel("accum_sum");
        hipLaunchKernelGGL((accum_sum_kernel<T>), dim3((uint32_t)a.n_dest), dim3(kBlock), 0, s, a,
                           (double)jvm_cast<T>(y_alpha));
        return after_launch(s);
      }
    }
    note_kernel("accum_owner");
    hipLaunchKernelGGL((accum_owner_kernel<T, OP>), dim3((uint32_t)((a.n_dest + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                       s, f, a);
    return after_launch(s);
  }
  EwOperand ops[3] = {{dest, dd, (int)sizeof(T), 0},
                      {reverse ? y : dest, reverse ? yd : dd, (int)sizeof(T), 0},
                      {reverse ? dest : y, reverse ? dd : yd, (int)sizeof(T), 0}};
  return launch_elementwise_serial(s, f, ops, n);
}

template <class T>
int accum_dispatch(hipStream_t s, void* dest, const ct_dims* dd, double da, const void* y, const ct_dims* yd, double ya,
                   int64_t n, int op, bool reverse) {
#define CT_CASE(OP) case OP: return accum_run<T, OP>(s, dest, dd, da, y, yd, ya, n, reverse)
  switch (op) {
    CT_CASE(CT_BOP_ADD); CT_CASE(CT_BOP_SUB); CT_CASE(CT_BOP_MUL); CT_CASE(CT_BOP_DIV);
    CT_CASE(CT_BOP_MIN); CT_CASE(CT_BOP_MAX); CT_CASE(CT_BOP_BIT_AND); CT_CASE(CT_BOP_BIT_XOR);
    CT_CASE(CT_BOP_EQ); CT_CASE(CT_BOP_GT); CT_CASE(CT_BOP_GE); CT_CASE(CT_BOP_LT); CT_CASE(CT_BOP_LE);
    default: return set_error(CT_ERR_INVALID, "unknown binary operation %d", op);
  }
#undef CT_CASE
}

}  // namespace

extern "C" int ct_binary_accum(void* stream, void* dest, const ct_dims* dest_dims, double dest_alpha, const void* y,
                               const ct_dims* y_dims, double y_alpha, int64_t n, int op, int reverse_operands,
                               int dest_requires_cas, int dtype) {
  CT_REQUIRE(dest && y, "ct_binary_accum: null buffer");
  CT_REQUIRE(n >= 0, "ct_binary_accum: negative count");
  if (n == 0) return CT_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (!dest_requires_cas) {
    // every destination element is written once: an in-place binary-op!
    // (cpu/tensor_math.clj:1451-1463)
    BinaryCall c = reverse_operands
                       ? BinaryCall{dest, dest_dims, y, y_dims, y_alpha, 0.0, dest, dest_dims, dest_alpha, 0.0, n, op}
                       : BinaryCall{dest, dest_dims, dest, dest_dims, dest_alpha, 0.0, y, y_dims, y_alpha, 0.0, n, op};
    return run_binary(s, dtype, c);
  }
  if (int rc = check_dims(dest_dims, "dest")) return rc;
  if (int rc = check_dims(y_dims, "y")) return rc;
  CT_DISPATCH_DTYPE(dtype, return accum_dispatch<T>(s, dest, dest_dims, dest_alpha, y, y_dims, y_alpha, n, op, reverse_operands != 0));
  return CT_OK;
}
