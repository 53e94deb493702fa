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
// elements proceed in parallel.  For op :+ with dest_alpha 1 and enough updates
// per destination element (bias gradients: [k] <- [b,k], [C,1,1] <- [N,C,H,W])
// the call instead runs as sum reductions of y over the broadcast axes into a
// stream-owned temporary, innermost group of axes first, followed by one
// in-place add into the destination: every pass streams at the reduce kernels'
// rate.  Integer results are unchanged by that (sums wrap modulo 2^bits either
// way); float/double results are sums formed in double, closer to the exact sum
// than the reference's value-by-value accumulation (which the reference itself
// only checks to 1e-4, src/cortex/verify/tensor.clj:188-191).
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
  uint32_t i = 0;
  if (a.n_redax == 1) {
    // one broadcast axis: fetch eight updates ahead, apply them in order
    constexpr int UN = 8;
    const int64_t st = a.ry_stride[0];
    for (; i + UN <= (uint32_t)a.n_red; i += UN) {
      T yv[UN];
#pragma unroll
      for (int j = 0; j < UN; ++j) yv[j] = yp[(int64_t)(i + j) * st];
#pragma unroll
      for (int j = 0; j < UN; ++j) acc = a.reverse ? f(yv[j], acc, acc) : f(acc, yv[j], yv[j]);
    }
  }
  for (; i < (uint32_t)a.n_red; ++i) {
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
      if (dstr[i] <= 0) return false;
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
  // two owners must never share an address: sorted by stride, each kept axis
  // has to step over everything the faster ones cover
  int order[CT_MAX_DIMS];
  for (int i = 0; i < a->n_kept; ++i) order[i] = i;
  std::sort(order, order + a->n_kept, [&](int l, int r) { return a->kd_stride[l] < a->kd_stride[r]; });
  int64_t span = 1;
  for (int i = 0; i < a->n_kept; ++i) {
    if (a->kd_stride[order[i]] < span) return false;
    span = a->kd_stride[order[i]] * ((int64_t)a->ksize[order[i]].d - 1) + span;
  }
  return true;
}

struct StageAxis {
  int64_t size, ystride, dstride;
  bool kept;
};

constexpr int64_t kStagedMinUpdates = 64;     // per destination element
constexpr int64_t kStagedMinElements = 16384;  // of y

// dest += sum over the broadcast axes of y*y_alpha, as staged unary-reduce!
// passes plus one in-place binary-op!.  Sets *handled to false (and does
// nothing) when y is itself broadcast along some axis.
int accum_sum_staged(hipStream_t s, const OwnerArgs& a, double y_alpha, int dtype, size_t elem_bytes, bool* handled) {
  *handled = false;
  StageAxis ax[CT_MAX_DIMS];
  int nax = 0;
  for (int d = 0; d < a.n_kept; ++d) {
    if (a.ky_stride[d] <= 0) return CT_OK;
    ax[nax++] = StageAxis{(int64_t)a.ksize[d].d, a.ky_stride[d], a.kd_stride[d], true};
  }
  for (int d = 0; d < a.n_redax; ++d) {
    if (a.rsize[d].d == 1) continue;
    if (a.ry_stride[d] <= 0) return CT_OK;
    ax[nax++] = StageAxis{(int64_t)a.rsize[d].d, a.ry_stride[d], 0, false};
  }
  if (nax > CT_MAX_DIMS) return CT_OK;
  std::sort(ax, ax + nax, [](const StageAxis& l, const StageAxis& r) { return l.ystride > r.ystride; });  // slowest first
  *handled = true;

  const void* cur = a.y;
  double alpha = y_alpha;
  int slot = kScratchAccumA;
  for (;;) {
    // innermost reduced axis, merged with the reduced axes that chain onto it
    int g = -1;
    for (int i = nax - 1; i >= 0; --i)
      if (!ax[i].kept) { g = i; break; }
    if (g < 0) break;
    int64_t gsize = ax[g].size;
    const int64_t gstride = ax[g].ystride;
    bool taken[CT_MAX_DIMS] = {false};
    taken[g] = true;
    for (int i = g - 1; i >= 0; --i) {
      if (ax[i].kept) continue;
      if (ax[i].ystride != gstride * gsize) break;
      gsize *= ax[i].size;
      taken[i] = true;
    }
    ct_dims id, od;
    std::memset(&id, 0, sizeof(id));
    std::memset(&od, 0, sizeof(od));
    StageAxis rest[CT_MAX_DIMS];
    int nrest = 0;
    for (int i = 0; i < nax; ++i)
      if (!taken[i]) rest[nrest++] = ax[i];
    int64_t n_out = 1;
    for (int i = 0; i < nrest; ++i) n_out *= rest[i].size;
    int64_t mul = 1;
    for (int i = nrest - 1; i >= 0; --i) {
      id.shape[i] = od.shape[i] = rest[i].size;
      id.strides[i] = rest[i].ystride;
      od.strides[i] = mul;
      rest[i].ystride = mul;  // the layout of the temporary the next pass reads
      mul *= rest[i].size;
    }
    id.ndim = od.ndim = nrest + 1;
    id.shape[nrest] = gsize;
    id.strides[nrest] = gstride;
    od.shape[nrest] = 1;
    od.strides[nrest] = 1;
    void* tmp = nullptr;
    if (int rc = stream_scratch(s, (size_t)n_out * elem_bytes, &tmp, slot)) return rc;
    if (int rc = ct_unary_reduce((void*)s, tmp, &od, alpha, cur, &id, CT_ROP_SUM, dtype)) return rc;
    cur = tmp;
    alpha = 1.0;
    slot = slot == kScratchAccumA ? kScratchAccumB : kScratchAccumA;
    nax = nrest;
    for (int i = 0; i < nrest; ++i) ax[i] = rest[i];
  }

  ct_dims dd, td;
  std::memset(&dd, 0, sizeof(dd));
  std::memset(&td, 0, sizeof(td));
  if (nax == 0) {
    dd.ndim = td.ndim = 1;
    dd.shape[0] = td.shape[0] = 1;
    dd.strides[0] = td.strides[0] = 1;
  } else {
    dd.ndim = td.ndim = nax;
    for (int i = 0; i < nax; ++i) {
      dd.shape[i] = td.shape[i] = ax[i].size;
      dd.strides[i] = ax[i].dstride;
      td.strides[i] = ax[i].ystride;
    }
  }
  const BinaryCall c{a.dest, &dd, a.dest, &dd, 1.0, 0.0, cur, &td, 1.0, 0.0, a.n_dest, CT_BOP_ADD};
  const int rc = run_binary(s, dtype, c);
  note_kernel("accum_staged_sum");
  return rc;
}

template <class T, int OP>
int accum_run(hipStream_t s, void* dest, const ct_dims* dd, double dest_alpha, const void* y, const ct_dims* yd,
              double y_alpha, int64_t n, bool reverse, int dtype) {
  using A = typename acc_of<T>::type;
  BinaryF<T, OP> f;
  // f(first, second) = op(first * xa, second * ya)
  f.xa = reverse ? (A)jvm_cast<T>(y_alpha) : (A)jvm_cast<T>(dest_alpha);
  f.ya = reverse ? (A)jvm_cast<T>(dest_alpha) : (A)jvm_cast<T>(y_alpha);
  OwnerArgs a;
  std::memset(&a, 0, sizeof(a));
  if (owner_structure(*dd, *yd, n, &a)) {
    a.dest = dest;
    a.y = y;
    a.reverse = reverse ? 1 : 0;
    if constexpr (OP == CT_BOP_ADD) {
      if (jvm_cast<T>(dest_alpha) == (T)1 && a.n_red >= kStagedMinUpdates && n >= kStagedMinElements) {
        bool handled = false;
        if (int rc = accum_sum_staged(s, a, y_alpha, dtype, sizeof(T), &handled)) return rc;
        if (handled) return CT_OK;
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
                   int64_t n, int op, bool reverse, int dtype) {
#define CT_CASE(OP) case OP: return accum_run<T, OP>(s, dest, dd, da, y, yd, ya, n, reverse, dtype)
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
  CT_DISPATCH_DTYPE(dtype, return accum_dispatch<T>(s, dest, dest_dims, dest_alpha, y, y_dims, y_alpha, n, op, reverse_operands != 0, dtype));
  return CT_OK;
}
