// reduce_impl.h -- the kernels and the per-datatype dispatch of unary-reduce!.  The six reductions of
// one datatype instantiate every kernel family; ops_reduce.hip instantiates the float and double
// tensors, ops_reduce_int.hip the integer ones, so that the two compile side by side.
//
// src/cortex/compute/cpu/tensor_math.clj:582-663).
//
// Reference semantics: output element p (in the output's own logical order)
// receives the reduction of input logical elements [p*k, (p+1)*k), where
// k = ecount(input) / ecount(output); the accumulator is a double (a long for
// integer tensors), seeded with the first element, and is rounded once at the
// store.  max and min are java.lang.Math.max/min: NaN propagates and +0 > -0.
//
// Kernels:
//   reduce_row_small_kernel  unit-stride rows of at most 256 vectors: a group
//                       of 4, 16 or 64 lanes inside one wave takes up to four
//                       consecutive rows, issues every load up front and
//                       combines with shuffles only
//   reduce_row_kernel   longer unit-stride rows: a group of 64 or 256 lanes
//                       owns one output, reads its row with 128-bit loads,
//                       accumulates in double and combines with wavefront
//                       shuffles (and LDS across the 4 waves); when there are
//                       too few rows to fill the chip each row is cut into
//                       chunks whose partial results reduce_finish_kernel
//                       combines
//   reduce_col_kernel   the reduced axis is strided and another axis is
//                       unit-stride (a transposed view): lanes own columns,
//                       the 16 waves of a block stride down the rows so every
//                       load stays coalesced; rows are split over blocks into
//                       segments whose partial results go to scratch memory and
//                       are combined by reduce_finish_kernel (deterministic, no
//                       atomics)
//   reduce_any_kernel   anything else (indirect dimensions, ragged segments):
//                       one lane per output walking the reference's address
//                       object
// The double accumulator makes the summation order immaterial after the final
// rounding to float (the tree order differs from the reference's sequential
// order by about k * 2^-53 relative to the sum of magnitudes).
#pragma once
#include <algorithm>
#include <cstdlib>
#include <limits>
#include <mutex>
#include "elementwise.h"
#include "ops.h"

namespace cthip {
namespace reduce_detail {

// The reduction is a template parameter (the values are the ct_reduce_op_t codes), so the
// kernels carry no run-time branch on it.
enum RedKind { RK_MAX = CT_ROP_MAX, RK_MIN = CT_ROP_MIN, RK_SUM = CT_ROP_SUM, RK_MEAN = CT_ROP_MEAN,
               RK_MAG = CT_ROP_MAGNITUDE, RK_SUMSQ = CT_ROP_MAGNITUDE_SQUARED };

__device__ __forceinline__ double jmax(double a, double b) {
  if (a != a) return a;
  if (b != b) return b;
  if (a == 0.0 && b == 0.0) return (__double_as_longlong(a) < 0) ? b : a;
  return a > b ? a : b;
}
__device__ __forceinline__ double jmin(double a, double b) {
  if (a != a) return a;
  if (b != b) return b;
  if (a == 0.0 && b == 0.0) return (__double_as_longlong(a) < 0) ? a : b;
  return a < b ? a : b;
}
__device__ __forceinline__ int64_t jmax(int64_t a, int64_t b) { return a > b ? a : b; }
__device__ __forceinline__ int64_t jmin(int64_t a, int64_t b) { return a < b ? a : b; }
__device__ __forceinline__ int32_t jmax(int32_t a, int32_t b) { return a > b ? a : b; }
__device__ __forceinline__ int32_t jmin(int32_t a, int32_t b) { return a < b ? a : b; }

// Reduction policy with the reference's accumulator: a double for float and
// double tensors, a long for integer tensors (cpu/tensor_math.clj:588-629).
// ACC = int: byte and short tensors whose reduction cannot leave 32 bits (the host checks: max
// and min always, sums, means and sums of squares while count * largest term stays below 2^31); the value is the
// one the long would hold, at a third of the instructions.
template <class T, int RK, class ACC = typename acc_of<T>::type> struct RedWide {
  using Elem = T;
  using Acc = ACC;
  using Alpha = Acc;
  __device__ __forceinline__ explicit RedWide(int) {}
  static __device__ __forceinline__ Acc identity() {
    if constexpr (RK == RK_MAX) {
      if constexpr (std::is_same<Acc, double>::value) return -__builtin_huge_val();
      else return std::numeric_limits<Acc>::min();
    } else if constexpr (RK == RK_MIN) {
      if constexpr (std::is_same<Acc, double>::value) return __builtin_huge_val();
      else return std::numeric_limits<Acc>::max();
    } else {
      // -0.0 is the additive identity that keeps a sum of negative zeros negative,
      // as the reference's first-element seed does
      if constexpr (std::is_same<Acc, double>::value) return -0.0;
      else return (Acc)0;
    }
  }
  static __device__ __forceinline__ Acc value(T x, Alpha alpha) {
    Acc v;
    if constexpr (std::is_same<Acc, int32_t>::value) v = w_mul((Acc)(T)alpha, (Acc)x);  // both in T's range: a 24-bit multiply
    else v = w_mul(alpha, (Acc)x);
    if constexpr (RK == RK_SUMSQ || RK == RK_MAG) return w_mul(v, v);
    else return v;
  }
  static __device__ __forceinline__ Acc combine(Acc a, Acc b) {
    if constexpr (RK == RK_MAX) return jmax(a, b);
    else if constexpr (RK == RK_MIN) return jmin(a, b);
    else return w_add(a, b);
  }
  // Final cast, with mean and magnitude applied (cpu/tensor_math.clj:610-622).
  static __device__ __forceinline__ T finish(Acc acc, int64_t count) {
    if constexpr (RK == RK_MEAN) {
      if constexpr (std::is_same<Acc, double>::value) return jvm_cast<T>(acc / (double)count);
      else return jvm_ratio_cast<T>((int64_t)acc, count);
    } else if constexpr (RK == RK_MAG) {
      return jvm_cast<T>(sqrt((double)acc));
    } else {
      return jvm_cast<T>(acc);
    }
  }
  static __device__ __forceinline__ Acc shfl(Acc v, int mask) {
    if constexpr (std::is_same<Acc, double>::value) return __shfl_xor(v, mask, 64);
    else if constexpr (std::is_same<Acc, int32_t>::value) return __shfl_xor(v, mask, 64);
    else return (Acc)__shfl_xor((long long)v, mask, 64);
  }
};

// max / min of float or double tensors with alpha == 1, without widening.
// The IEEE bit pattern is mapped to a signed integer key whose order is the
// numeric order with -0 below +0 (flip the magnitude bits of negative values).
// Positive NaNs map above +infinity and negative NaNs below -infinity, so
// keeping the largest and the smallest key seen tells whether any NaN took
// part; Math.max / Math.min then return NaN (cpu/tensor_math.clj:591-602).
template <class T, int RK> struct RedKeyed {
  using Elem = T;
  using K = typename std::conditional<sizeof(T) == 4, int32_t, int64_t>::type;
  struct Acc { K hi, lo; };
  using Alpha = typename acc_of<T>::type;  // unused: alpha is 1
  __device__ __forceinline__ explicit RedKeyed(int) {}
  static constexpr K kMag = sizeof(T) == 4 ? (K)0x7fffffff : (K)0x7fffffffffffffffLL;
  static constexpr K kPosInf = sizeof(T) == 4 ? (K)0x7f800000 : (K)0x7ff0000000000000LL;
  static constexpr K kNegInf = sizeof(T) == 4 ? (K)(int32_t)0x807fffff : (K)0x800fffffffffffffLL;
  static __device__ __forceinline__ K key_of(T x) {
    K b;
    __builtin_memcpy(&b, &x, sizeof(T));
    return b ^ ((b >> (sizeof(T) * 8 - 1)) & kMag);
  }
  static __device__ __forceinline__ Acc identity() {
    return Acc{sizeof(T) == 4 ? (K)INT32_MIN : (K)INT64_MIN, sizeof(T) == 4 ? (K)INT32_MAX : (K)INT64_MAX};
  }
  static __device__ __forceinline__ Acc value(T x, Alpha) {
    const K k = key_of(x);
    return Acc{k, k};
  }
  static __device__ __forceinline__ Acc combine(Acc a, Acc b) {
    return Acc{a.hi > b.hi ? a.hi : b.hi, a.lo < b.lo ? a.lo : b.lo};
  }
  static __device__ __forceinline__ T finish(Acc acc, int64_t) {
    if (acc.hi > kPosInf || acc.lo < kNegInf) return (T)__builtin_nanf("");
    const K k = RK == RK_MAX ? acc.hi : acc.lo;
    const K b = k ^ ((k >> (sizeof(T) * 8 - 1)) & kMag);
    T r;
    __builtin_memcpy(&r, &b, sizeof(T));
    return r;
  }
  static __device__ __forceinline__ Acc shfl(Acc v, int mask) {
    if constexpr (sizeof(T) == 4) return Acc{__shfl_xor(v.hi, mask, 64), __shfl_xor(v.lo, mask, 64)};
    else return Acc{(K)__shfl_xor((long long)v.hi, mask, 64), (K)__shfl_xor((long long)v.lo, mask, 64)};
  }
};

// Integer tensors choose the reduction at run time inside three policies, so that one set of kernels
// per (datatype, accumulator) serves two reductions instead of one (the integer reductions were a
// quarter of the library's code).  Both read the ct_reduce_op_t code the kernel's arguments
// carry; it is uniform over the launch, so the choices below are scalar selects.
//
// max / min: for two's-complement integers min(a, b) = ~max(~a, ~b), so :min complements every
// value on the way in and the result on the way out (one exclusive-or each) and both run as max.
template <class T, class ACC = typename acc_of<T>::type> struct RedIntExtreme {
  static_assert(std::is_integral<T>::value, "integer tensors only");
  using Elem = T;
  using Acc = ACC;
  using Alpha = Acc;
  Acc flip;
  __device__ __forceinline__ explicit RedIntExtreme(int rk) : flip(rk == RK_MIN ? (Acc)-1 : (Acc)0) {}
  __device__ __forceinline__ Acc identity() const { return std::numeric_limits<Acc>::min(); }
  __device__ __forceinline__ Acc value(T x, Alpha alpha) const {
    if constexpr (std::is_same<Acc, int32_t>::value) return w_mul((Acc)(T)alpha, (Acc)x) ^ flip;
    else return w_mul(alpha, (Acc)x) ^ flip;
  }
  __device__ __forceinline__ Acc combine(Acc a, Acc b) const { return a > b ? a : b; }
  __device__ __forceinline__ T finish(Acc acc, int64_t) const { return jvm_cast<T>((Acc)(acc ^ flip)); }
  static __device__ __forceinline__ Acc shfl(Acc v, int mask) {
    if constexpr (std::is_same<Acc, int32_t>::value) return __shfl_xor(v, mask, 64);
    else return (Acc)__shfl_xor((long long)v, mask, 64);
  }
};

// sum / mean (SQUARES false) and magnitude-squared / magnitude (true): wrapping sums of the values or
// of their squares, and the reference's final step per reduction (cpu/tensor_math.clj:610-622).
template <class T, bool SQUARES, class ACC = typename acc_of<T>::type> struct RedIntSum {
  static_assert(std::is_integral<T>::value, "integer tensors only");
  using Elem = T;
  using Acc = ACC;
  using Alpha = Acc;
  int rk;
  __device__ __forceinline__ explicit RedIntSum(int rk_) : rk(rk_) {}
  __device__ __forceinline__ Acc identity() const { return (Acc)0; }
  __device__ __forceinline__ Acc value(T x, Alpha alpha) const {
    Acc v;
    if constexpr (std::is_same<Acc, int32_t>::value) v = w_mul((Acc)(T)alpha, (Acc)x);  // both in T's range: a 24-bit multiply
    else v = w_mul(alpha, (Acc)x);
    if constexpr (SQUARES) return w_mul(v, v);
    else return v;
  }
  __device__ __forceinline__ Acc combine(Acc a, Acc b) const { return w_add(a, b); }
  __device__ __forceinline__ T finish(Acc acc, int64_t count) const {
    if constexpr (SQUARES) return rk == RK_MAG ? jvm_cast<T>(sqrt((double)acc)) : jvm_cast<T>(acc);
    else return rk == RK_MEAN ? jvm_ratio_cast<T>((int64_t)acc, count) : jvm_cast<T>(acc);
  }
  static __device__ __forceinline__ Acc shfl(Acc v, int mask) {
    if constexpr (std::is_same<Acc, int32_t>::value) return __shfl_xor(v, mask, 64);
    else return (Acc)__shfl_xor((long long)v, mask, 64);
  }
};

struct OutAddr {
  int32_t identity;  // output address == logical index
  int32_t accumulate;  // the result is added to what the output holds (the last pass of a staged binary-accum! :+)
  int32_t rk;          // the reduction's ct_reduce_op_t code, for the policies that choose it at run time
  int32_t nd;
  GenOperand op;
  int64_t rmax[CT_MAX_DIMS];
};
__device__ __forceinline__ int64_t out_address(const OutAddr& o, int64_t p) {
  return o.identity ? p : ref_address(o.op, o.nd, o.rmax, p);
}

// Stores output p.  With oa.accumulate the stored value is old + result, formed as binary-op! :+
// forms it (both widened, one rounding): what a separate in-place add of the result would leave.
template <class P>
__device__ __forceinline__ void store_output(const P& pol, void* out, const OutAddr& oa, int64_t p, const typename P::Acc& acc, int64_t k) {
  using T = typename P::Elem;
  using W = typename acc_of<T>::type;
  T* const o = reinterpret_cast<T*>(out) + out_address(oa, p);
  T r = pol.finish(acc, k);
  if (oa.accumulate) r = jvm_cast<T>(w_add((W)*o, (W)r));
  *o = r;
}

// Partial accumulators of a reduction split over several blocks:
// partials[seg * n_out + p], combined in increasing seg by reduce_finish_kernel.
struct FinishArgs {
  const void* partials;
  void* out;
  int64_t k, n_out;
  uint32_t n_seg;
  OutAddr oa;
};

struct RowArgs {
  const void* in;
  void* out;
  void* partials;       // [n_split][n_out] accumulators when n_split > 1
  int64_t k, n_out;
  int64_t chunk;        // elements of a row one lane group covers (k when n_split == 1)
  FastDiv split_fd;     // n_split
  uint32_t n_split;
  int32_t n_outer;
  FastDiv osize[CT_MAX_DIMS];   // kept axes, fastest first
  int64_t ostride[CT_MAX_DIMS];
  OutAddr oa;
  int32_t op;
};

// TPR lanes per output; kBlock / TPR outputs per block.  A long row may be cut
// into n_split chunks, each taken by its own lane group, when there are too
// few rows to fill the chip (the norm of a whole parameter vector).
template <class P, int VEC, int TPR, int BS = kBlock>
__global__ void __launch_bounds__(BS) reduce_row_kernel(const RowArgs a, const typename P::Alpha alpha) {
  const P pol(a.oa.rk);
  using T = typename P::Elem;
  using A = typename P::Acc;
  using V = Vec<T, VEC>;
  constexpr int RPB = BS / TPR;
  __shared__ A lds[BS / 64];
  // A block lives about as long as one trip to memory (a row is a few KiB), so the
  // arguments are fetched in one batch before the first branch: naming them in one
  // empty asm statement makes the compiler load them here rather than next to each use.
  asm volatile("" ::"s"(a.in), "s"(a.out), "s"(a.partials), "s"(a.k), "s"(a.n_out), "s"(a.chunk), "s"(a.split_fd.d),
               "s"(a.split_fd.m), "s"(a.split_fd.s), "s"(a.n_split), "s"(a.n_outer), "s"(a.osize[0].d), "s"(a.osize[0].m),
               "s"(a.osize[0].s), "s"(a.ostride[0]), "s"(a.osize[1].d), "s"(a.osize[1].m), "s"(a.osize[1].s),
               "s"(a.ostride[1]), "s"(a.oa.identity));
  const int lane = threadIdx.x % TPR;
  const int64_t vp = (int64_t)blockIdx.x * RPB + threadIdx.x / TPR;
  const bool live = vp < a.n_out * (int64_t)a.n_split;
  uint32_t p = (uint32_t)vp, seg = 0;
  if (a.n_split > 1) a.split_fd.divmod((uint32_t)vp, p, seg);
  A acc0 = pol.identity(), acc1 = pol.identity();
  if (live) {
    int64_t base = (int64_t)seg * a.chunk;
    int64_t len = a.k - base;
    if (len > a.chunk) len = a.chunk;
    // the first two kept axes with fixed indices (absent axes have size 1, stride 0)
    uint32_t rem, r0, r1, q0;
    a.osize[0].divmod(p, q0, r0);
    a.osize[1].divmod(q0, rem, r1);
    base += (int64_t)r0 * a.ostride[0] + (int64_t)r1 * a.ostride[1];
    for (int d = 2; d < a.n_outer; ++d) {
      uint32_t q, r;
      a.osize[d].divmod(rem, q, r);
      rem = q;
      base += (int64_t)r * a.ostride[d];
    }
    const V* row = reinterpret_cast<const V*>(reinterpret_cast<const T*>(a.in) + base);
    const int64_t nv = len / VEC;
    int64_t i = lane;
    for (; i + TPR < nv; i += 2 * TPR) {
      const V x0 = nt_load(row + i), x1 = nt_load(row + i + TPR);
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        acc0 = pol.combine(acc0, pol.value(x0.v[e], alpha));
        acc1 = pol.combine(acc1, pol.value(x1.v[e], alpha));
      }
    }
    if (i < nv) {
      const V x0 = nt_load(row + i);
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc0 = pol.combine(acc0, pol.value(x0.v[e], alpha));
    }
  }
  A acc = pol.combine(acc0, acc1);
  constexpr int W = TPR < 64 ? TPR : 64;
#pragma unroll
  for (int m = W / 2; m >= 1; m >>= 1) acc = pol.combine(acc, P::shfl(acc, m));
  if constexpr (TPR > 64) {
    if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
      acc = lds[0];
#pragma unroll
      for (int w = 1; w < BS / 64; ++w) acc = pol.combine(acc, lds[w]);
    }
  }
  if (live && lane == 0) {
    if (a.n_split == 1) store_output<P>(pol, a.out, a.oa, p, acc, a.k);
    else reinterpret_cast<A*>(a.partials)[(int64_t)seg * a.n_out + p] = acc;
  }
}

// Rows of at most L * TPR vectors (L <= 4, TPR <= 64): a group of TPR lanes
// inside one wave takes U = 4 / L rows, issues all of its loads before the
// first use, and combines with shuffles only (no LDS, no barrier).  For each
// of the U passes the groups of a block take consecutive rows, so one load
// instruction of a wave covers consecutive rows.
template <class P, int VEC, int TPR, int L>
__global__ void __launch_bounds__(kBlock) reduce_row_small_kernel(const RowArgs a, const typename P::Alpha alpha) {
  const P pol(a.oa.rk);
  using T = typename P::Elem;
  using A = typename P::Acc;
  using V = Vec<T, VEC>;
  constexpr int U = 4 / L;
  constexpr int GPB = kBlock / TPR;
  const int lane = threadIdx.x % TPR;
  const int64_t p0 = (int64_t)blockIdx.x * (GPB * U) + threadIdx.x / TPR;
  const int nv = (int)(a.k / VEC);
  V x[U][L];
#pragma unroll
  for (int r = 0; r < U; ++r) {
    const int64_t p = p0 + r * GPB;
    if (p < a.n_out) {
      int64_t base = 0;
      uint32_t rem = (uint32_t)p;
      for (int d = 0; d < a.n_outer; ++d) {
        uint32_t q, m;
        a.osize[d].divmod(rem, q, m);
        rem = q;
        base += (int64_t)m * a.ostride[d];
      }
      const V* row = reinterpret_cast<const V*>(reinterpret_cast<const T*>(a.in) + base);
#pragma unroll
      for (int j = 0; j < L; ++j)
        if (lane + j * TPR < nv) x[r][j] = nt_load(row + lane + j * TPR);
    }
  }
#pragma unroll
  for (int r = 0; r < U; ++r) {
    const int64_t p = p0 + r * GPB;
    A acc = pol.identity();
    if (p < a.n_out) {
#pragma unroll
      for (int j = 0; j < L; ++j)
        if (lane + j * TPR < nv) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) acc = pol.combine(acc, pol.value(x[r][j].v[e], alpha));
        }
    }
#pragma unroll
    for (int m = TPR / 2; m >= 1; m >>= 1) acc = pol.combine(acc, P::shfl(acc, m));
    if (p < a.n_out && lane == 0) store_output<P>(pol, a.out, a.oa, p, acc, a.k);
  }
}

struct ColArgs {
  const void* in;
  void* out;
  void* partials;       // [n_seg][n_out] accumulators
  int64_t k, n_out, rstride;
  uint32_t u;           // size of the unit-stride kept axis
  int64_t u_pmul;       // its multiplier in the output's logical index
  uint32_t n_strips, n_seg, rows_per_seg;
  FastDiv strips_fd, seg_fd;
  int32_t n_rest;       // other kept axes, fastest first
  FastDiv rsize[CT_MAX_DIMS];
  int64_t rstride_in[CT_MAX_DIMS], r_pmul[CT_MAX_DIMS];
  OutAddr oa;
  int32_t op;
};

// 16 waves per block: each wave-load is one 1 KiB row segment, 16 consecutive
// rows are in flight per block, 8 loads per lane.  Measured best among 1-16
// waves and 32-512 rows per block for a [16384, 4096] float input.
constexpr int kColBlock = 1024;
constexpr int64_t kNarrowColBytes = int64_t(4) << 20;  // largest input the one-launch narrow-strip column kernel takes
constexpr int64_t kRowSplitBytes = 16384;  // smallest chunk a split row is cut into

template <class P, int VEC>
__global__ void __launch_bounds__(kColBlock) reduce_col_kernel(const ColArgs a, const typename P::Alpha alpha) {
  const P pol(a.oa.rk);
  using T = typename P::Elem;
  using A = typename P::Acc;
  using V = Vec<T, VEC>;
  constexpr int WAVES = kColBlock / 64;
  __shared__ A lds[WAVES - 1][64 * VEC];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  uint32_t q0, strip, seg, rest;
  a.strips_fd.divmod(blockIdx.x, q0, strip);
  a.seg_fd.divmod(q0, rest, seg);
  int64_t base = 0, pbase = 0;
  for (int d = 0; d < a.n_rest; ++d) {
    uint32_t q, r;
    a.rsize[d].divmod(rest, q, r);
    rest = q;
    base += (int64_t)r * a.rstride_in[d];
    pbase += (int64_t)r * a.r_pmul[d];
  }
  const uint32_t col = (strip * 64 + lane) * VEC;
  const bool live = col < a.u;
  A acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) acc[e] = pol.identity();
  const int64_t r0 = (int64_t)seg * a.rows_per_seg;
  int64_t r1 = r0 + a.rows_per_seg;
  if (r1 > a.k) r1 = a.k;
  if (live) {
    // each wave owns rows r0+wave, r0+wave+WAVES, ...; UN loads are in flight per lane
    constexpr int UN = 8;
    const int64_t step = (int64_t)WAVES * a.rstride;
    const T* p = reinterpret_cast<const T*>(a.in) + base + col + (r0 + wave) * a.rstride;
    int64_t r = r0 + wave;
    for (; r + (UN - 1) * WAVES < r1; r += UN * WAVES, p += UN * step) {
      V x[UN];
#pragma unroll
      for (int j = 0; j < UN; ++j) x[j] = nt_load(reinterpret_cast<const V*>(p + j * step));
#pragma unroll
      for (int j = 0; j < UN; ++j)
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] = pol.combine(acc[e], pol.value(x[j].v[e], alpha));
    }
    if (r < r1) {  // the last, partial batch: same depth, rows past the end skipped
      V x[UN];
#pragma unroll
      for (int j = 0; j < UN; ++j)
        if (r + j * WAVES < r1) x[j] = nt_load(reinterpret_cast<const V*>(p + j * step));
#pragma unroll
      for (int j = 0; j < UN; ++j)
        if (r + j * WAVES < r1) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) acc[e] = pol.combine(acc[e], pol.value(x[j].v[e], alpha));
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
      for (int w = 0; w < WAVES - 1; ++w) acc[e] = pol.combine(acc[e], lds[w][e * 64 + lane]);
      const int64_t p = pbase + (int64_t)(col + e) * a.u_pmul;
      if (a.n_seg == 1) store_output<P>(pol, a.out, a.oa, p, acc[e], a.k);
      else reinterpret_cast<A*>(a.partials)[(int64_t)seg * a.n_out + p] = acc[e];
    }
  }
}

// A small matrix reduced down its columns (the [1024,1024] and [128,784] of a network's layer): cut
// into row segments it needs the finishing launch, which costs more than the reduction; left whole
// under 256-column strips it is four blocks.  Here a block owns a strip of LW * VEC columns (128
// bytes) over all rows, so there are blocks enough without segments: LW lanes across, 64 / LW rows
// per wave-load, eight loads in flight per lane; the lanes of a column combine with shuffles, the
// waves in LDS.  One launch.  (Strips this narrow stream at half the rate of the wide ones, which
// is why large matrices keep them.)
template <class P, int VEC, int LW>
__global__ void __launch_bounds__(kColBlock) reduce_col_narrow_kernel(const ColArgs a, const typename P::Alpha alpha) {
  const P pol(a.oa.rk);
  using T = typename P::Elem;
  using A = typename P::Acc;
  using V = Vec<T, VEC>;
  constexpr int WAVES = kColBlock / 64, RW = 64 / LW, RB = RW * WAVES, UN = 8;
  __shared__ A lds[WAVES - 1][LW * VEC];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int lc = lane % LW, lr = lane / LW;
  uint32_t rest, strip;
  a.strips_fd.divmod(blockIdx.x, rest, strip);
  int64_t base = 0, pbase = 0;
  for (int d = 0; d < a.n_rest; ++d) {
    uint32_t q, r;
    a.rsize[d].divmod(rest, q, r);
    rest = q;
    base += (int64_t)r * a.rstride_in[d];
    pbase += (int64_t)r * a.r_pmul[d];
  }
  const uint32_t col = (strip * LW + lc) * VEC;
  const bool live = col < a.u;
  A acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) acc[e] = pol.identity();
  if (live) {
    const T* p = reinterpret_cast<const T*>(a.in) + base + col;
    for (int64_t r = wave * RW + lr; r < a.k; r += (int64_t)RB * UN) {
      V x[UN];
#pragma unroll
      for (int j = 0; j < UN; ++j)
        if (r + j * RB < a.k) x[j] = nt_load(reinterpret_cast<const V*>(p + (r + j * RB) * a.rstride));
#pragma unroll
      for (int j = 0; j < UN; ++j)
        if (r + j * RB < a.k) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) acc[e] = pol.combine(acc[e], pol.value(x[j].v[e], alpha));
        }
    }
  }
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
#pragma unroll
    for (int m = LW; m < 64; m <<= 1) acc[e] = pol.combine(acc[e], P::shfl(acc[e], m));
  }
  if (wave > 0 && lr == 0) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) lds[wave - 1][lc * VEC + e] = acc[e];
  }
  __syncthreads();
  if (wave == 0 && lr == 0 && live) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
#pragma unroll
      for (int w = 0; w < WAVES - 1; ++w) acc[e] = pol.combine(acc[e], lds[w][lc * VEC + e]);
      store_output<P>(pol, a.out, a.oa, pbase + (int64_t)(col + e) * a.u_pmul, acc[e], a.k);
    }
  }
}

// Few rows under many columns ([16, 4194304] summed over its rows): every lane owns VEC columns
// and walks all k rows itself, first to last as the reference does, eight loads in flight.  No
// segments, no LDS, no second launch; a block of 256 lanes covers 256 * VEC consecutive columns.
// (With the kernel above a block of sixteen waves would meet for one row each: 30 % of the memory
// rate on that shape against 56-60 % here, and 66-78 % where the row pitch is no power of two:
// [16, 4198400], [64, 1050624], [32, 2000000].  Sixteen loads in flight change nothing.)  ColArgs as above with n_strips counted in blocks of 256 lanes;
// vec_out: the results of a lane are neighbours in the output and go out as one vector.
template <class P, int VEC>
__global__ void __launch_bounds__(kBlock) reduce_col_thin_kernel(const ColArgs a, const typename P::Alpha alpha, const int vec_out) {
  const P pol(a.oa.rk);
  using T = typename P::Elem;
  using A = typename P::Acc;
  using V = Vec<T, VEC>;
  uint32_t rest, strip;
  a.strips_fd.divmod(blockIdx.x, rest, strip);
  int64_t base = 0, pbase = 0;
  for (int d = 0; d < a.n_rest; ++d) {
    uint32_t q, r;
    a.rsize[d].divmod(rest, q, r);
    rest = q;
    base += (int64_t)r * a.rstride_in[d];
    pbase += (int64_t)r * a.r_pmul[d];
  }
  const uint32_t col = (strip * kBlock + threadIdx.x) * VEC;
  if (col >= a.u) return;
  A acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) acc[e] = pol.identity();
  const T* p = reinterpret_cast<const T*>(a.in) + base + col;
  constexpr int UN = 8;
  int64_t r = 0;
  for (; r + UN <= a.k; r += UN, p += UN * a.rstride) {
    V x[UN];
#pragma unroll
    for (int j = 0; j < UN; ++j) x[j] = nt_load(reinterpret_cast<const V*>(p + j * a.rstride));
#pragma unroll
    for (int j = 0; j < UN; ++j)
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc[e] = pol.combine(acc[e], pol.value(x[j].v[e], alpha));
  }
  if (r < a.k) {
    V x[UN];
#pragma unroll
    for (int j = 0; j < UN; ++j)
      if (r + j < a.k) x[j] = nt_load(reinterpret_cast<const V*>(p + j * a.rstride));
#pragma unroll
    for (int j = 0; j < UN; ++j)
      if (r + j < a.k) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] = pol.combine(acc[e], pol.value(x[j].v[e], alpha));
      }
  }
  if (vec_out) {
    V out;
#pragma unroll
    for (int e = 0; e < VEC; ++e) out.v[e] = pol.finish(acc[e], a.k);
    *reinterpret_cast<V*>(reinterpret_cast<T*>(a.out) + pbase + col) = out;
  } else {
#pragma unroll
    for (int e = 0; e < VEC; ++e) store_output<P>(pol, a.out, a.oa, pbase + (int64_t)(col + e) * a.u_pmul, acc[e], a.k);
  }
}

// Short rows stored back to back (a dense [rows, k] block of at most 128 bytes per row) whose
// length is no whole number of 16-byte vectors, ten classes say.  A block stages its 256 rows, one
// contiguous stretch of memory, through LDS with 128-bit accesses; one lane then owns a row in LDS
// and accumulates it from the first element to the last, the reference's order.  (With a lane
// group per row and 4-byte loads the same rows reach a sixth of the memory rate.)
struct ShortRowsArgs {
  const void* in;
  void* out;
  int64_t n_out;
  uint32_t k;
  OutAddr oa;
};

template <class P>
__global__ void __launch_bounds__(kBlock) reduce_short_rows_kernel(const ShortRowsArgs a, const typename P::Alpha alpha) {
  const P pol(a.oa.rk);
  using T = typename P::Elem;
  using A = typename P::Acc;
  constexpr int VEC = 16 / (int)sizeof(T);
  using V = Vec<T, VEC>;
  extern __shared__ __align__(16) char smem[];
  T* tile = reinterpret_cast<T*>(smem);
  const uint32_t k = a.k;
  const int64_t row0 = (int64_t)blockIdx.x * kBlock;
  const uint32_t n_rows = (uint32_t)(a.n_out - row0 < kBlock ? a.n_out - row0 : kBlock);
  const uint32_t count = n_rows * k;
  const T* in = reinterpret_cast<const T*>(a.in) + row0 * k;
  // a block's stretch starts on the 16-byte grid whenever the tensor does (256 * k elements per block)
  const uint32_t n_vec = count / VEC;
  for (uint32_t v = threadIdx.x; v < n_vec; v += kBlock)
    reinterpret_cast<V*>(tile)[v] = nt_load(reinterpret_cast<const V*>(in) + v);
  for (uint32_t e = n_vec * VEC + threadIdx.x; e < count; e += kBlock) tile[e] = in[e];
  __syncthreads();
  if (threadIdx.x < n_rows) {
    const T* row = tile + threadIdx.x * k;
    A acc = pol.identity();
    for (uint32_t j = 0; j < k; ++j) acc = pol.combine(acc, pol.value(row[j], alpha));
    store_output<P>(pol, a.out, a.oa, row0 + threadIdx.x, acc, (int64_t)k);
  }
}


// Combines the partial accumulators of a split reduction.  The launch is small
// (a few KiB to a MiB of partials) and sits on the critical path between two
// calls, so it is shaped for latency: LPO lanes share one output, every lane
// issues all of its loads (at most kFinishLoads) before the first combine when
// the segments allow, and the lanes of an output combine with shuffles.  The
// lanes of a wave are laid out output-fastest (lane = seg_lane * (64 / LPO) +
// output), so one load instruction reads runs of consecutive partials.
constexpr int kFinishLoads = 4;

template <class P, int LPO>
__global__ void __launch_bounds__(kBlock) reduce_finish_kernel(const FinishArgs a) {
  const P pol(a.oa.rk);
  using A = typename P::Acc;
  constexpr int PPW = 64 / LPO;  // outputs per wave
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sl = lane / PPW, pl = lane % PPW;
  const int64_t p = ((int64_t)blockIdx.x * (kBlock / 64) + wave) * PPW + pl;
  const bool live = p < a.n_out;
  const A* part = reinterpret_cast<const A*>(a.partials);
  A acc = pol.identity();
  if (live) {
    if (a.n_seg <= (uint32_t)(kFinishLoads * LPO)) {
      A x[kFinishLoads];
#pragma unroll
      for (int j = 0; j < kFinishLoads; ++j) {
        const uint32_t s = (uint32_t)(sl + j * LPO);
        if (s < a.n_seg) x[j] = part[(int64_t)s * a.n_out + p];
      }
#pragma unroll
      for (int j = 0; j < kFinishLoads; ++j)
        if ((uint32_t)(sl + j * LPO) < a.n_seg) acc = pol.combine(acc, x[j]);
    } else {
#pragma unroll 8
      for (uint32_t s = sl; s < a.n_seg; s += LPO) acc = pol.combine(acc, part[(int64_t)s * a.n_out + p]);
    }
  }
#pragma unroll
  for (int m = 32; m >= PPW; m >>= 1) acc = pol.combine(acc, P::shfl(acc, m));
  if (live && sl == 0) store_output<P>(pol, a.out, a.oa, p, acc, a.k);
}

template <class P>
void launch_finish(hipStream_t st, const FinishArgs& f) {
#define CT_FINISH(LPO)                                                                                              \
  hipLaunchKernelGGL((reduce_finish_kernel<P, LPO>),                                                                \
                     dim3((uint32_t)((f.n_out + (kBlock / 64) * (64 / LPO) - 1) / ((kBlock / 64) * (64 / LPO)))),   \
                     dim3(kBlock), 0, st, f)
  // as few lanes per output as keep every lane at kFinishLoads loads or fewer
  if (f.n_seg <= kFinishLoads) CT_FINISH(1);
  else if (f.n_seg <= 4 * kFinishLoads) CT_FINISH(4);
  else if (f.n_seg <= 16 * kFinishLoads) CT_FINISH(16);
  else CT_FINISH(64);
#undef CT_FINISH
}

struct AnyArgs {
  const void* in;
  void* out;
  int64_t k, n_out;
  int32_t in_nd;
  GenOperand in_op;
  int64_t in_rmax[CT_MAX_DIMS];
  OutAddr oa;
  int32_t op;
};

// One lane per output, in the reference's own order (sequential accumulation).
template <class P>
__global__ void __launch_bounds__(kBlock) reduce_any_kernel(const AnyArgs a, const typename P::Alpha alpha) {
  const P pol(a.oa.rk);
  using T = typename P::Elem;
  using A = typename P::Acc;
  const int64_t p = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (p >= a.n_out) return;
  const T* in = reinterpret_cast<const T*>(a.in);
  const int64_t start = p * a.k;
  A acc = pol.value(in[ref_address(a.in_op, a.in_nd, a.in_rmax, start)], alpha);
  for (int64_t i = 1; i < a.k; ++i)
    acc = pol.combine(acc, pol.value(in[ref_address(a.in_op, a.in_nd, a.in_rmax, start + i)], alpha));
  store_output<P>(pol, a.out, a.oa, p, acc, a.k);
}

// ------------------------------------------------------------------ host planning

struct RedShape {  // the input split into kept axes and one merged reduced axis
  bool fast;       // direct, non-negative strides, segment = trailing axes, single reduced axis
  int64_t k, rstride;
  int n_kept;      // slowest first
  int64_t ksize[CT_MAX_DIMS], kstride[CT_MAX_DIMS];
};

inline RedShape analyse(const ct_dims& in, int64_t k) {
  RedShape r;
  std::memset(&r, 0, sizeof(r));
  r.k = k;
  r.fast = dims_direct(in);
  for (int i = 0; r.fast && i < in.ndim; ++i)
    if (in.shape[i] > 1 && in.strides[i] < 0) r.fast = false;
  if (!r.fast) return r;
  int j = in.ndim;
  int64_t prod = 1;
  while (j > 0 && prod < k) prod *= in.shape[--j];
  if (prod != k) { r.fast = false; return r; }
  // merge the reduced axes j..nd-1 (size-1 axes dropped) into one
  int64_t rsize = 1, rstr = 1;
  bool have = false;
  for (int i = in.ndim - 1; i >= j; --i) {
    if (in.shape[i] == 1) continue;
    if (!have) { rsize = in.shape[i]; rstr = in.strides[i]; have = true; }
    else if (in.strides[i] == rstr * rsize) rsize *= in.shape[i];
    else { r.fast = false; return r; }
  }
  r.rstride = have ? rstr : 1;
  // kept axes, slowest first; neighbours that chain ([512, 7, 7] with strides [49, 7, 1]) are one axis
  for (int i = 0; i < j; ++i) {
    if (in.shape[i] == 1) continue;
    if (r.n_kept > 0 && r.kstride[r.n_kept - 1] == in.strides[i] * in.shape[i]) {
      r.ksize[r.n_kept - 1] *= in.shape[i];
      r.kstride[r.n_kept - 1] = in.strides[i];
      continue;
    }
    r.ksize[r.n_kept] = in.shape[i];
    r.kstride[r.n_kept] = in.strides[i];
    ++r.n_kept;
  }
  return r;
}

// Where a split reduction keeps its partial accumulators: the stream's growing
// scratch block (allocated on demand), or a fixed block that is never grown.
struct PartialStore {
  void* fixed;         // nullptr: use the stream's scratch
  size_t fixed_bytes;
  const char* who;
  bool accumulate = false;  // add the result to the output instead of replacing it
};

inline int partial_store(hipStream_t st, const PartialStore& ps, size_t bytes, void** out) {
  if (!ps.fixed) return stream_scratch(st, bytes, out);
  if (bytes > ps.fixed_bytes)
    return set_error(CT_ERR_INVALID,
                     "%s: this reduction needs %zu bytes of partial accumulators; the fixed scratch holds %zu "
                     "(use ct_unary_reduce, which allocates)",
                     ps.who, bytes, ps.fixed_bytes);
  *out = ps.fixed;
  return CT_OK;
}

template <class T> bool aligned_for(const void* p, int vec) { return ((uintptr_t)p % (uintptr_t)(vec * sizeof(T))) == 0; }

template <class P>
int reduce_run(hipStream_t st, const PartialStore& ps, void* out, const ct_dims* od, double alpha_d, const void* in,
               const ct_dims* id, int op) {
  using T = typename P::Elem;
  using A = typename P::Acc;
  const typename P::Alpha alpha = (typename P::Alpha)jvm_cast<T>(alpha_d);
  const int64_t n_out = dims_ecount(*od), total = dims_ecount(*id);
  const int64_t k = total / n_out;
  CT_REQUIRE(k >= 1, "unary-reduce!: input (%lld elements) is smaller than output (%lld)", (long long)total,
             (long long)n_out);

  OutAddr oa;
  std::memset(&oa, 0, sizeof(oa));
  int out_rank = 0;
  if (int rc = reference_operand_own(od, &oa.op, oa.rmax, &out_rank)) return rc;
  oa.nd = out_rank;
  oa.identity = oa.op.mode == 0;
  oa.accumulate = ps.accumulate ? 1 : 0;
  oa.rk = op;

  constexpr int VMAX = 16 / (int)sizeof(T);
  const RedShape rs = analyse(*id, k);
  const bool small_idx = n_out < (int64_t(1) << 31) && k < (int64_t(1) << 31);

  if (rs.fast && small_idx && rs.rstride == 1) {
    RowArgs a;
    std::memset(&a, 0, sizeof(a));
    a.in = in; a.out = out; a.k = k; a.n_out = n_out; a.oa = oa; a.op = op;
    a.n_outer = rs.n_kept;
    bool vec_ok = VMAX > 1 && k % VMAX == 0 && aligned_for<T>(in, VMAX);
    for (int d = 0; d < rs.n_kept; ++d) {  // fastest first
      const int src = rs.n_kept - 1 - d;
      a.osize[d] = FastDiv((uint32_t)rs.ksize[src]);
      a.ostride[d] = rs.kstride[src];
      if (rs.kstride[src] % VMAX != 0) vec_ok = false;
    }
    // too few rows for the chip and long ones: cut each row into chunks of at
    // least 16 KiB until about 4096 lane groups exist
    int64_t split = 1, chunk = k;
    if (n_out < 2048 && k * (int64_t)sizeof(T) >= 2 * kRowSplitBytes) {
      const int64_t quantum = kRowSplitBytes / (int64_t)sizeof(T);
      const int64_t want = (4096 + n_out - 1) / n_out;
      chunk = std::max<int64_t>(quantum, ((k + want - 1) / want + quantum - 1) / quantum * quantum);
      split = (k + chunk - 1) / chunk;
      if (split <= 1) { split = 1; chunk = k; }
    }
    a.chunk = chunk;
    a.n_split = (uint32_t)split;
    a.split_fd = FastDiv((uint32_t)split);
    if (split > 1) {
      if (int rc = partial_store(st, ps, (size_t)(split * n_out) * sizeof(A), &a.partials)) return rc;
    }
    const int64_t n_groups = n_out * split;
    const int64_t row_bytes = chunk * (int64_t)sizeof(T);
#define CT_ROW(VEC, TPR)                                                                                        \
  hipLaunchKernelGGL((reduce_row_kernel<P, VEC, TPR>), dim3((uint32_t)((n_groups + (kBlock / TPR) - 1) / (kBlock / TPR))), \
                     dim3(kBlock), 0, st, a, alpha)
#define CT_ROW_WIDE(VEC) \
  hipLaunchKernelGGL((reduce_row_kernel<P, VEC, 512, 512>), dim3((uint32_t)n_groups), dim3(512), 0, st, a, alpha)
#define CT_ROW_SMALL(VEC, TPR, L)                                                                                   \
  hipLaunchKernelGGL((reduce_row_small_kernel<P, VEC, TPR, L>),                                                     \
                     dim3((uint32_t)((n_out + (kBlock / TPR) * (4 / L) - 1) / ((kBlock / TPR) * (4 / L)))),          \
                     dim3(kBlock), 0, st, a, alpha)
#define CT_ROW_SMALL_SHAPES(VEC)                  \
  if (nv <= 1) CT_ROW_SMALL(VEC, 1, 1);           \
  else if (nv <= 2) CT_ROW_SMALL(VEC, 2, 1);      \
  else if (nv <= 4) CT_ROW_SMALL(VEC, 4, 1);      \
  else if (nv <= 8) CT_ROW_SMALL(VEC, 8, 1);      \
  else if (nv <= 16) CT_ROW_SMALL(VEC, 16, 1);    \
  else if (nv <= 32) CT_ROW_SMALL(VEC, 16, 2);    \
  else if (nv <= 64) CT_ROW_SMALL(VEC, 16, 4);    \
  else if (nv <= 128) CT_ROW_SMALL(VEC, 64, 2);   \
  else CT_ROW_SMALL(VEC, 64, 4)
    const int64_t nv = vec_ok ? k / VMAX : k;
    if (VMAX > 1 && !vec_ok && k % VMAX != 0 && k * (int64_t)sizeof(T) <= 128 && k >= 2 && rs.n_kept == 1 &&
        rs.kstride[0] == k && aligned_for<T>(in, VMAX) && n_out >= 1024) {
      ShortRowsArgs sa;
      std::memset(&sa, 0, sizeof(sa));
      sa.in = in; sa.out = out; sa.n_out = n_out; sa.k = (uint32_t)k; sa.oa = oa;
      note_kernel("reduce_short_rows");
      hipLaunchKernelGGL((reduce_short_rows_kernel<P>), dim3((uint32_t)((n_out + kBlock - 1) / kBlock)), dim3(kBlock),
                         (size_t)kBlock * k * sizeof(T), st, sa, alpha);
    } else if (split == 1 && nv <= 256) {
      note_kernel(vec_ok ? "reduce_row_small_vec" : "reduce_row_small");
      if (vec_ok) { CT_ROW_SMALL_SHAPES(VMAX); } else { CT_ROW_SMALL_SHAPES(1); }
    } else if (vec_ok && (row_bytes >= 32768 || (row_bytes >= 16384 && n_groups * row_bytes >= (int64_t(192) << 20)))) {
      // 512 lanes per row: a 16 KiB row is in flight at once, two loads per lane.  Measured on float
      // [16384,4096]: 92 % of peak against 85-89 % for 256 lanes (two rounds of two loads).  With a
      // quarter of the rows, [4096,4096], 256 lanes are ahead (10.4 us against 11.5), hence the
      // size condition on 16 KiB rows; rows of 32 KiB (double [4096,4096]) take 512 lanes at any size.
      note_kernel("reduce_row512_vec");
      CT_ROW_WIDE(VMAX);
    } else if (row_bytes >= 4096) {
      note_kernel(vec_ok ? "reduce_row256_vec" : "reduce_row256");
      if (vec_ok) CT_ROW(VMAX, 256); else CT_ROW(1, 256);
    } else {
      note_kernel("reduce_row64");
      CT_ROW(1, 64);
    }
#undef CT_ROW_WIDE
#undef CT_ROW_SMALL_SHAPES
#undef CT_ROW_SMALL
#undef CT_ROW
    if (split > 1) {
      const FinishArgs f{a.partials, out, k, n_out, (uint32_t)split, oa};
      launch_finish<P>(st, f);
    }
    return after_launch(st);
  }

  // the unit-stride kept axis the column kernels run along: at least 16 columns, or any number when the
  // input is small enough for the one-launch narrow-strip kernel (ten classes summed over a batch)
  const int64_t min_unit = total * (int64_t)sizeof(T) <= kNarrowColBytes ? 2 : 16;
  int unit = -1;
  if (rs.fast && small_idx)
    for (int d = 0; d < rs.n_kept; ++d)
      if (rs.kstride[d] == 1 && rs.ksize[d] >= min_unit) unit = d;
  if (unit >= 0) {
    ColArgs a;
    std::memset(&a, 0, sizeof(a));
    a.in = in; a.out = out; a.k = k; a.n_out = n_out; a.rstride = rs.rstride; a.oa = oa; a.op = op;
    a.u = (uint32_t)rs.ksize[unit];
    bool vec_ok = VMAX > 1 && a.u % VMAX == 0 && rs.rstride % VMAX == 0 && aligned_for<T>(in, VMAX);
    // logical multipliers of the kept axes in the output index (row-major, slowest first)
    int64_t pmul[CT_MAX_DIMS];
    int64_t m = 1;
    for (int d = rs.n_kept - 1; d >= 0; --d) { pmul[d] = m; m *= rs.ksize[d]; }
    a.u_pmul = pmul[unit];
    int64_t rest_count = 1;
    for (int d = rs.n_kept - 1; d >= 0; --d) {  // fastest first
      if (d == unit) continue;
      a.rsize[a.n_rest] = FastDiv((uint32_t)rs.ksize[d]);
      a.rstride_in[a.n_rest] = rs.kstride[d];
      a.r_pmul[a.n_rest] = pmul[d];
      if (rs.kstride[d] % VMAX != 0) vec_ok = false;
      rest_count *= rs.ksize[d];
      ++a.n_rest;
    }
    const int vec = vec_ok ? VMAX : 1;
    // few rows, and columns enough for four blocks per compute unit without cutting the rows
    const int64_t thin_strips = ((int64_t)a.u + kBlock * vec - 1) / (kBlock * vec);
    if (k <= 128 && thin_strips * rest_count >= 1024 && thin_strips * rest_count < (int64_t(1) << 31)) {
      a.n_strips = (uint32_t)thin_strips;
      a.n_seg = 1;
      a.strips_fd = FastDiv(a.n_strips);
      const int vec_out = oa.identity && !oa.accumulate && a.u_pmul == 1 && aligned_for<T>(out, vec) ? 1 : 0;
      note_kernel(vec_ok ? "reduce_col_thin_vec" : "reduce_col_thin");
      const dim3 grid((uint32_t)(thin_strips * rest_count));
      if (vec_ok) hipLaunchKernelGGL((reduce_col_thin_kernel<P, VMAX>), grid, dim3(kBlock), 0, st, a, alpha, vec_out);
      else hipLaunchKernelGGL((reduce_col_thin_kernel<P, 1>), grid, dim3(kBlock), 0, st, a, alpha, vec_out);
      return after_launch(st);
    }
    a.n_strips = (a.u + 64 * vec - 1) / (64 * vec);
    const int64_t base_blocks = (int64_t)a.n_strips * rest_count;
    // Rows are cut into segments until about two blocks per compute unit exist
    // (one round of resident blocks measured better than several shorter ones);
    // a segment is a whole number of load batches; partials capped at 16 MiB.
    constexpr int64_t kRowQuantum = 128;  // 16 waves x 8 loads in flight
    // Between one and two blocks per compute unit, segments of two load batches are preferred to
    // twice as many of one: float [4096,4096] 10.6 us with 16 segments against 11.6 with 32.
    const int64_t most = std::max<int64_t>(1, std::min<int64_t>(512 / base_blocks, k / kRowQuantum));
    const int64_t least = std::max<int64_t>(1, std::min<int64_t>(most, (256 + base_blocks - 1) / base_blocks));
    const int64_t want_seg = std::min(most, std::max(least, k / (2 * kRowQuantum)));
    int64_t rows = ((k + want_seg - 1) / want_seg + kRowQuantum - 1) / kRowQuantum * kRowQuantum;
    const int64_t seg_cap = std::max<int64_t>(1, (int64_t(16) << 20) / (n_out * (int64_t)sizeof(A)));
    if ((k + rows - 1) / rows > seg_cap) rows = (k + seg_cap - 1) / seg_cap;
    // Segments a power of two apart in memory advance in step through the same memory channels and
    // banks: eight rows more per segment moves every segment's start off that grid without changing
    // the number of segments (float [16384,4096]: 41.2 -> 38.5 us for the bare kernel, double
    // [4096,4096] 20.0 -> 19.5, float [4096,4096] 10.0 -> 9.2).
    if (rows < k && (k + rows + 7) / (rows + 8) == (k + rows - 1) / rows) rows += 8;
    int64_t seg = (k + rows - 1) / rows;
    // a small matrix that the wide strips have to cut into row segments: narrow strips, one launch
    constexpr int kNarrowLanes = 8;
    const int64_t narrow_strips = ((int64_t)a.u + kNarrowLanes * vec - 1) / (kNarrowLanes * vec);
    if (seg > 1 && total * (int64_t)sizeof(T) <= kNarrowColBytes) {
      a.n_strips = (uint32_t)narrow_strips;
      a.n_seg = 1;
      a.strips_fd = FastDiv(a.n_strips);
      note_kernel(vec_ok ? "reduce_col_narrow_vec" : "reduce_col_narrow");
      const dim3 grid((uint32_t)(narrow_strips * rest_count));
      if (vec_ok) hipLaunchKernelGGL((reduce_col_narrow_kernel<P, VMAX, kNarrowLanes>), grid, dim3(kColBlock), 0, st, a, alpha);
      else hipLaunchKernelGGL((reduce_col_narrow_kernel<P, 1, kNarrowLanes>), grid, dim3(kColBlock), 0, st, a, alpha);
      return after_launch(st);
    }
    a.n_seg = (uint32_t)seg;
    a.rows_per_seg = (uint32_t)rows;
    a.strips_fd = FastDiv(a.n_strips);
    a.seg_fd = FastDiv(a.n_seg);
    const int64_t grid = base_blocks * seg;
    if (grid < (int64_t(1) << 31)) {
      if (seg > 1) {
        if (int rc = partial_store(st, ps, (size_t)(seg * n_out) * sizeof(A), &a.partials)) return rc;
      }
      note_kernel(vec_ok ? "reduce_col_vec" : "reduce_col");
      if (vec_ok) hipLaunchKernelGGL((reduce_col_kernel<P, VMAX>), dim3((uint32_t)grid), dim3(kColBlock), 0, st, a, alpha);
      else hipLaunchKernelGGL((reduce_col_kernel<P, 1>), dim3((uint32_t)grid), dim3(kColBlock), 0, st, a, alpha);
      if (seg > 1) {
        const FinishArgs f{a.partials, out, k, n_out, (uint32_t)seg, oa};
        launch_finish<P>(st, f);
      }
      return after_launch(st);
    }
  }

  AnyArgs a;
  std::memset(&a, 0, sizeof(a));
  a.in = in; a.out = out; a.k = k; a.n_out = n_out; a.oa = oa; a.op = op;
  int in_rank = 0;
  if (int rc = reference_operand_own(id, &a.in_op, a.in_rmax, &in_rank)) return rc;
  a.in_nd = in_rank;
  CT_REQUIRE((n_out + kBlock - 1) / kBlock < (int64_t(1) << 31), "unary-reduce!: too many outputs");
  note_kernel("reduce_any");
  hipLaunchKernelGGL((reduce_any_kernel<P>), dim3((uint32_t)((n_out + kBlock - 1) / kBlock)), dim3(kBlock), 0, st,
                     a, alpha);
  return after_launch(st);
}

template <class T, int RK>
int reduce_typed(hipStream_t st, const PartialStore& ps, void* out, const ct_dims* od, double alpha, const void* in,
                 const ct_dims* id, int op) {
  if constexpr (std::is_floating_point<T>::value && (RK == RK_MAX || RK == RK_MIN)) {
    const T a = jvm_cast<T>(alpha);
    if (a == (T)1) return reduce_run<RedKeyed<T, RK>>(st, ps, out, od, alpha, in, id, op);
    // Any other finite, non-zero multiplier on a large input: x -> T(x * a) never reverses the order
    // of two values for a > 0 and always does for a < 0 (for float tensors the products are exact in
    // double; for double tensors the rounding is monotonic), so the extreme of the products is the
    // product of the extreme: the multiplier-free kernel above runs (on the opposite extreme for
    // a < 0) and one small launch multiplies its results.  Float [16384,4096] :max with alpha 0.5:
    // 76-86 us with the widening form, which multiplies and compares doubles per element.
    const int64_t total = dims_ecount(*id);
    if (a == a && a != (T)0 && a - a == (T)0 && total * (int64_t)sizeof(T) >= (int64_t(32) << 20) && dims_direct(*od) &&
        dims_dense(*od) && dims_access_increasing(*od)) {
      constexpr int kOpposite = RK == RK_MAX ? RK_MIN : RK_MAX;
      const int rc = a > (T)0 ? reduce_run<RedKeyed<T, RK>>(st, ps, out, od, 1.0, in, id, op)
                              : reduce_run<RedKeyed<T, kOpposite>>(st, ps, out, od, 1.0, in, id, op);
      if (rc) return rc;
      return ct_unary_op(st, out, od, out, od, (double)a, CT_UOP_NOOP, sizeof(T) == 4 ? CT_F32 : CT_F64, dims_ecount(*od));
    }
  }
  if constexpr (std::is_integral<T>::value) {
    constexpr bool kExtreme = RK == RK_MAX || RK == RK_MIN;
    constexpr bool kSquares = RK == RK_SUMSQ || RK == RK_MAG;
    if constexpr (sizeof(T) <= 2) {
      // the largest magnitude an element times the multiplier can have, and how many of them a sum adds
      const int64_t a_abs = std::llabs((long long)jvm_cast<T>(alpha));
      const int64_t x_abs = std::is_signed<T>::value ? (int64_t(1) << (8 * sizeof(T) - 1)) : (int64_t(1) << (8 * sizeof(T))) - 1;
      const int64_t n_out = dims_ecount(*od), total = dims_ecount(*id);
      const int64_t count = n_out > 0 ? total / n_out : 0;
      const int64_t term = (RK == RK_SUMSQ || RK == RK_MAG) ? (a_abs * x_abs) * (a_abs * x_abs) : a_abs * x_abs;  // < 2^62
      const bool fits = kExtreme ? term < (int64_t(1) << 31) : (count > 0 && term < (int64_t(1) << 31) / count);
      if (fits) {
        using Narrow = typename std::conditional<kExtreme, RedIntExtreme<T, int32_t>, RedIntSum<T, kSquares, int32_t>>::type;
        return reduce_run<Narrow>(st, ps, out, od, alpha, in, id, op);
      }
    }
    using Wide = typename std::conditional<kExtreme, RedIntExtreme<T>, RedIntSum<T, kSquares>>::type;
    return reduce_run<Wide>(st, ps, out, od, alpha, in, id, op);
  } else {
    return reduce_run<RedWide<T, RK>>(st, ps, out, od, alpha, in, id, op);
  }
}

template <class T>
int reduce_dispatch(hipStream_t st, const PartialStore& ps, void* out, const ct_dims* od, double alpha, const void* in,
                    const ct_dims* id, int op) {
  switch (op) {
    case CT_ROP_MAX: return reduce_typed<T, RK_MAX>(st, ps, out, od, alpha, in, id, op);
    case CT_ROP_MIN: return reduce_typed<T, RK_MIN>(st, ps, out, od, alpha, in, id, op);
    case CT_ROP_SUM: return reduce_typed<T, RK_SUM>(st, ps, out, od, alpha, in, id, op);
    case CT_ROP_MEAN: return reduce_typed<T, RK_MEAN>(st, ps, out, od, alpha, in, id, op);
    case CT_ROP_MAGNITUDE: return reduce_typed<T, RK_MAG>(st, ps, out, od, alpha, in, id, op);
    case CT_ROP_MAGNITUDE_SQUARED: return reduce_typed<T, RK_SUMSQ>(st, ps, out, od, alpha, in, id, op);
    default: return set_error(CT_ERR_INVALID, "unknown reduction operation %d", op);
  }
}

}  // namespace reduce_detail
}  // namespace cthip
