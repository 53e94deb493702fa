// ops_nn.hip -- activation-gradient!, softmax-eltwise!, softmax-spatial!
// (src/cortex/tensor/math.clj:176-189;
//  src/cortex/compute/cpu/tensor_math.clj:1037-1103, 1318-1362).
//
// activation-gradient! is one more elementwise functor over the shared
// launcher, so it accepts every access pattern the other elementwise ops do.
//
// softmax works on rows of k elements laid out as [outer, rows, k] with
// arbitrary (direct) strides per operand; the spatial form is the same thing
// with the channel axis taken as k.  Per row, as the CPU backend does it:
//   m   = max(x)                       (java.lang.Math.max: NaN propagates)
//   e_i = T(exp(double(x_i) - double(m)))
//   s   = T(sum of double(e_i))
//   y_i = e_i / s                      (a division in T)
// Four kernels cover the layouts:
//   softmax_wave_kernel   a group of 4, 16 or 64 lanes owns a row of up to 1024
//                         vectors, kept in registers (128-bit accesses when the
//                         rows are unit-stride and aligned)
//   softmax_block_kernel  longer rows: one block per row, exponentials parked
//                         in the output and scaled in a third pass
//   softmax_short_rows_kernel  dense rows of up to 128 bytes that are no whole
//                         number of vectors, staged through LDS
//   softmax_lane_kernel   one lane owns a row (or four neighbouring rows, as
//                         128-bit accesses) and walks k sequentially, the lanes
//                         of a wave take neighbouring rows (coalesced when the
//                         row axis is unit-stride: the spatial form, where k is
//                         the channel axis); rows of up to 32 elements stay in
//                         registers.  Its sum runs in the reference's order.
// y_i is formed as e_i * (1 / s): at most one ulp from the reference's e_i / s.
// The reference's maximum loop reads elements 1..k-1 of the input through the
// output's address object (cpu/tensor_math.clj:1067-1072); that only matters
// when the two layouts differ, and then only through rounding, because the
// result of a softmax does not depend on the value subtracted.  The kernels
// take the true row maximum.
#include <algorithm>

#include "elementwise.h"
#include "functors.h"

using namespace cthip;

namespace {

// act-backward-impl (cpu/tensor_math.clj:1318-1362): operands widen to double,
// the products run left to right, the store rounds once.
template <class T, int OP> struct ActGradF {
  static constexpr int NIN = 2;
  using Out = T;
  using In0 = T;  // output
  using In1 = T;  // output gradient
  using In2 = T;
  __device__ __forceinline__ T operator()(T out, T grad, T) const {
    const double o = (double)out, g = (double)grad;
    if constexpr (OP == CT_ACT_LOGISTIC) return (T)((o * (1.0 - o)) * g);
    else if constexpr (OP == CT_ACT_TANH) return (T)((1.0 - o * o) * g);
    else return (T)((o > 0.0 ? 1.0 : 0.0) * g);
  }
};

template <class T, int OP>
int act_grad_run(hipStream_t s, void* ig, const ct_dims* igd, const void* og, const ct_dims* ogd, const void* out,
                 const ct_dims* od, int64_t n) {
  ActGradF<T, OP> f;
  EwOperand ops[3] = {{ig, igd, (int)sizeof(T), 0}, {out, od, (int)sizeof(T), 0}, {og, ogd, (int)sizeof(T), 0}};
  return launch_elementwise(s, f, ops, n);
}

template <class T>
int act_grad_typed(hipStream_t s, void* ig, const ct_dims* igd, const void* og, const ct_dims* ogd, const void* out,
                   const ct_dims* od, int op, int64_t n) {
  switch (op) {
    case CT_ACT_LOGISTIC: return act_grad_run<T, CT_ACT_LOGISTIC>(s, ig, igd, og, ogd, out, od, n);
    case CT_ACT_TANH: return act_grad_run<T, CT_ACT_TANH>(s, ig, igd, og, ogd, out, od, n);
    case CT_ACT_RELU: return act_grad_run<T, CT_ACT_RELU>(s, ig, igd, og, ogd, out, od, n);
    default: return set_error(CT_ERR_INVALID, "Only :logistic :tanh and :relu are supported (got %d)", op);
  }
}

// ------------------------------------------------------------------ softmax

// The running maximum of a row.  java.lang.Math.max propagates NaN, the hardware's maximum
// returns the other operand.  The difference cannot reach the result: a NaN element has a NaN
// exponential whatever is subtracted from it, the row sum is NaN with it, and every element
// of the row comes out NaN, as it does in the reference (where the maximum itself is NaN).
// Nor can the sign of a zero maximum.  One instruction per element instead of four, in kernels
// whose arithmetic, not memory, sets the pace.
template <class T> __device__ __forceinline__ T jvm_max(T a, T b) {
  if constexpr (std::is_same<T, float>::value) return __builtin_fmaxf(a, b);
  else return __builtin_fmax(a, b);
}

// T(exp(double(x) - double(m))), x <= m.  For float: the difference and its product with
// log2(e) are formed in double (exact to 1e-16), split into an integer n and a fraction in
// [-0.5, 0.5]; the hardware's exp2 (1 ulp) takes the fraction as a float (its rounding moves
// the result by 1e-8 relative) and ldexp applies n.  About a dozen instructions against
// two dozen for an error-free float difference plus the library's expf; the result is
// within 1 ulp of the reference's.  n is clamped at -300 (the result is 0 long before), which
// also keeps it a number when the operand is NaN or -infinity: those reach exp2 through the
// fraction (NaN - n = NaN, -inf - n = -inf) and give NaN and 0.
template <class T> __device__ __forceinline__ T shifted_exp(T x, T m) {
  if constexpr (std::is_same<T, float>::value) {
    const double a = ((double)x - (double)m) * 1.4426950408889634;
    const double n = __builtin_fmax(__builtin_rint(a), -300.0);
    const float frac = (float)(a - n);
    return __builtin_ldexpf(__builtin_amdgcn_exp2f(frac), (int)n);
  } else {
    return exp(x - m);
  }
}

struct SoftmaxArgs {
  const void* in;
  void* out;
  int64_t n_rows;        // outer * rows
  uint32_t k;
  FastDiv rows_fd;       // rows per outer index
  int64_t in_outer, in_row, in_k;
  int64_t out_outer, out_row, out_k;
};

__device__ __forceinline__ void softmax_row_base(const SoftmaxArgs& a, int64_t r, int64_t* ib, int64_t* ob) {
  uint32_t o, p;
  a.rows_fd.divmod((uint32_t)r, o, p);
  *ib = (int64_t)o * a.in_outer + (int64_t)p * a.in_row;
  *ob = (int64_t)o * a.out_outer + (int64_t)p * a.out_row;
}

// TPR lanes (inside one wave) own a row of at most TPR * ITER vectors and keep
// it in registers: one read, one write.  VEC > 1 needs unit-stride, aligned rows.
// The division by the row sum is a multiplication by its reciprocal (at most
// one ulp from the quotient).
// NT: the call moves more than the last-level cache holds, and the loads and stores are non-temporal
// (rows of 1024 floats, 1 GiB: +2 % of peak for the loads, +2 to 3 for the stores; 128 MiB: -7 %).  The
// same stores did nothing for the lane-per-row kernel of the spatial form.
template <class T, int VEC, int TPR, int ITER, bool NT>
__global__ void __launch_bounds__(kBlock) softmax_wave_kernel(const SoftmaxArgs a) {
  using V = Vec<T, VEC>;
  const int lane = threadIdx.x % TPR;
  const int64_t r = (int64_t)blockIdx.x * (kBlock / TPR) + threadIdx.x / TPR;
  const bool live = r < a.n_rows;
  int64_t ib = 0, ob = 0;
  if (live) softmax_row_base(a, r, &ib, &ob);
  const T* in = reinterpret_cast<const T*>(a.in) + ib;
  T* out = reinterpret_cast<T*>(a.out) + ob;
  const uint32_t nv = a.k / VEC;
  V x[ITER];
  T m = -__builtin_huge_valf();  // identity of Math.max that lets NaN through
#pragma unroll
  for (int j = 0; j < ITER; ++j) {
    const uint32_t i = lane + j * TPR;
    if (live && i < nv) {
      if constexpr (VEC > 1) {
        const V* vp = reinterpret_cast<const V*>(in + (int64_t)i * VEC);
        if constexpr (NT) x[j] = nt_load(vp); else x[j] = *vp;
      }
      else x[j].v[0] = in[(int64_t)i * a.in_k];
#pragma unroll
      for (int e = 0; e < VEC; ++e) m = jvm_max(m, x[j].v[e]);
    }
  }
#pragma unroll
  for (int s = TPR / 2; s >= 1; s >>= 1) m = jvm_max(m, (T)__shfl_xor(m, s, 64));
  double sum = 0.0;
#pragma unroll
  for (int j = 0; j < ITER; ++j) {
    const uint32_t i = lane + j * TPR;
    if (live && i < nv) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) { x[j].v[e] = shifted_exp(x[j].v[e], m); sum += (double)x[j].v[e]; }
    }
  }
#pragma unroll
  for (int s = TPR / 2; s >= 1; s >>= 1) sum += __shfl_xor(sum, s, 64);
  const T inv = (T)1 / (T)sum;
#pragma unroll
  for (int j = 0; j < ITER; ++j) {
    const uint32_t i = lane + j * TPR;
    if (live && i < nv) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) x[j].v[e] *= inv;
      if constexpr (VEC > 1) {
        if constexpr (NT) nt_store(x[j], reinterpret_cast<V*>(out + (int64_t)i * VEC));
        else *reinterpret_cast<V*>(out + (int64_t)i * VEC) = x[j];
      } else {
        out[(int64_t)i * a.out_k] = x[j].v[0];
      }
    }
  }
}

// One block per row of any length: the exponentials are parked in the output
// (rounded to T, as the CPU backend stores them) and scaled in a third pass.
template <class T>
__global__ void __launch_bounds__(kBlock) softmax_block_kernel(const SoftmaxArgs a) {
  __shared__ double lds[kBlock / 64];
  int64_t ib, ob;
  softmax_row_base(a, blockIdx.x, &ib, &ob);
  const T* in = reinterpret_cast<const T*>(a.in) + ib;
  T* out = reinterpret_cast<T*>(a.out) + ob;
  const int wave = threadIdx.x >> 6;
  T m = -__builtin_huge_valf();
  for (uint32_t i = threadIdx.x; i < a.k; i += kBlock) m = jvm_max(m, in[(int64_t)i * a.in_k]);
#pragma unroll
  for (int s = 32; s >= 1; s >>= 1) m = jvm_max(m, (T)__shfl_xor(m, s, 64));
  if ((threadIdx.x & 63) == 0) lds[wave] = (double)m;
  __syncthreads();
  m = (T)lds[0];
#pragma unroll
  for (int w = 1; w < kBlock / 64; ++w) m = jvm_max(m, (T)lds[w]);
  __syncthreads();
  double sum = 0.0;
  for (uint32_t i = threadIdx.x; i < a.k; i += kBlock) {
    const T e = shifted_exp(in[(int64_t)i * a.in_k], m);
    out[(int64_t)i * a.out_k] = e;
    sum += (double)e;
  }
#pragma unroll
  for (int s = 32; s >= 1; s >>= 1) sum += __shfl_xor(sum, s, 64);
  if ((threadIdx.x & 63) == 0) lds[wave] = sum;
  __syncthreads();
  sum = lds[0];
#pragma unroll
  for (int w = 1; w < kBlock / 64; ++w) sum += lds[w];
  const T inv = (T)1 / (T)sum;
  for (uint32_t i = threadIdx.x; i < a.k; i += kBlock) out[(int64_t)i * a.out_k] *= inv;  // each lane re-reads its own stores
}

// One block per row of up to kBlock * ITER vectors, kept in registers like the wave kernel's rows
// (one read, one write), with the two reductions carried across the four waves through LDS.
// Unit-stride, aligned rows only.
template <class T, int VEC, int ITER>
__global__ void __launch_bounds__(kBlock) softmax_block_reg_kernel(const SoftmaxArgs a) {
  using V = Vec<T, VEC>;
  __shared__ double lds[kBlock / 64];
  int64_t ib, ob;
  softmax_row_base(a, blockIdx.x, &ib, &ob);
  const T* in = reinterpret_cast<const T*>(a.in) + ib;
  T* out = reinterpret_cast<T*>(a.out) + ob;
  const uint32_t nv = a.k / VEC;
  const int wave = threadIdx.x >> 6;
  V x[ITER];
  T m = -__builtin_huge_valf();
#pragma unroll
  for (int j = 0; j < ITER; ++j) {
    const uint32_t i = threadIdx.x + j * kBlock;
    if (i < nv) {
      x[j] = nt_load(reinterpret_cast<const V*>(in + (int64_t)i * VEC));
#pragma unroll
      for (int e = 0; e < VEC; ++e) m = jvm_max(m, x[j].v[e]);
    }
  }
#pragma unroll
  for (int s = 32; s >= 1; s >>= 1) m = jvm_max(m, (T)__shfl_xor(m, s, 64));
  if ((threadIdx.x & 63) == 0) lds[wave] = (double)m;
  __syncthreads();
  m = (T)lds[0];
#pragma unroll
  for (int w = 1; w < kBlock / 64; ++w) m = jvm_max(m, (T)lds[w]);
  __syncthreads();
  double sum = 0.0;
#pragma unroll
  for (int j = 0; j < ITER; ++j) {
    const uint32_t i = threadIdx.x + j * kBlock;
    if (i < nv) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) { x[j].v[e] = shifted_exp(x[j].v[e], m); sum += (double)x[j].v[e]; }
    }
  }
#pragma unroll
  for (int s = 32; s >= 1; s >>= 1) sum += __shfl_xor(sum, s, 64);
  if ((threadIdx.x & 63) == 0) lds[wave] = sum;
  __syncthreads();
  sum = lds[0];
#pragma unroll
  for (int w = 1; w < kBlock / 64; ++w) sum += lds[w];
  const T inv = (T)1 / (T)sum;
#pragma unroll
  for (int j = 0; j < ITER; ++j) {
    const uint32_t i = threadIdx.x + j * kBlock;
    if (i < nv) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) x[j].v[e] *= inv;
      *reinterpret_cast<V*>(out + (int64_t)i * VEC) = x[j];
    }
  }
}

// One lane per row, the lanes of a wave on neighbouring rows.  CMAX > 0: the row
// (k <= CMAX) stays in registers.  CMAX == 0: any k, exponentials parked in the
// output.  The sum runs in the reference's own order.
template <class T, int VEC, int CMAX>
__global__ void __launch_bounds__(kBlock) softmax_lane_kernel(const SoftmaxArgs a) {
  // VEC > 1: the lane owns VEC neighbouring rows (positions); the row axis is unit-stride
  // and every stride a multiple of VEC, so each channel is one aligned vector access.
  using V = Vec<T, VEC>;
  const int64_t r = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * VEC;
  if (r >= a.n_rows) return;
  int64_t ib, ob;
  softmax_row_base(a, r, &ib, &ob);
  const T* in = reinterpret_cast<const T*>(a.in) + ib;
  T* out = reinterpret_cast<T*>(a.out) + ob;
  auto load = [&](uint32_t i) { return *reinterpret_cast<const V*>(in + (int64_t)i * a.in_k); };
  auto store = [&](uint32_t i, const V& v) { *reinterpret_cast<V*>(out + (int64_t)i * a.out_k) = v; };
  T m[VEC];
  double sum[VEC];
  T inv[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) { m[e] = -__builtin_huge_valf(); sum[e] = 0.0; }  // identity of Math.max that lets NaN through
  if constexpr (CMAX > 0) {
    V x[CMAX];
#pragma unroll
    for (int i = 0; i < CMAX; ++i)
      if ((uint32_t)i < a.k) {
        x[i] = nt_load(reinterpret_cast<const V*>(in + (int64_t)i * a.in_k));  // read once
#pragma unroll
        for (int e = 0; e < VEC; ++e) m[e] = jvm_max(m[e], x[i].v[e]);
      }
#pragma unroll
    for (int i = 0; i < CMAX; ++i)
      if ((uint32_t)i < a.k) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) { x[i].v[e] = shifted_exp(x[i].v[e], m[e]); sum[e] += (double)x[i].v[e]; }
      }
#pragma unroll
    for (int e = 0; e < VEC; ++e) inv[e] = (T)1 / (T)sum[e];
#pragma unroll
    for (int i = 0; i < CMAX; ++i)
      if ((uint32_t)i < a.k) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) x[i].v[e] *= inv[e];
        store(i, x[i]);
      }
  } else {
    constexpr int U = 4;  // channels fetched ahead
    for (uint32_t i0 = 0; i0 < a.k; i0 += U) {
      V x[U];
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (i0 + u < a.k) x[u] = load(i0 + u);
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (i0 + u < a.k) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) m[e] = jvm_max(m[e], x[u].v[e]);
        }
    }
    for (uint32_t i0 = 0; i0 < a.k; i0 += U) {
      V x[U];
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (i0 + u < a.k) x[u] = load(i0 + u);
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (i0 + u < a.k) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) { x[u].v[e] = shifted_exp(x[u].v[e], m[e]); sum[e] += (double)x[u].v[e]; }
          store(i0 + u, x[u]);
        }
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) inv[e] = (T)1 / (T)sum[e];
    for (uint32_t i = 0; i < a.k; ++i) {
      V x = *reinterpret_cast<const V*>(out + (int64_t)i * a.out_k);  // the lane re-reads its own stores
#pragma unroll
      for (int e = 0; e < VEC; ++e) x.v[e] *= inv[e];
      store(i, x);
    }
  }
}

// The same for rows too long for registers: the lane's row sits in its own
// column of LDS (no other lane touches it, so no barrier), one read and one
// write of memory instead of the loop form's three and two.  One wave per
// block; k * 64 vectors of LDS, which is what bounds the waves per compute unit.
template <class T, int VEC>
__global__ void __launch_bounds__(64) softmax_lane_lds_kernel(const SoftmaxArgs a) {
  using V = Vec<T, VEC>;
  extern __shared__ __align__(16) char smem[];
  V* col = reinterpret_cast<V*>(smem) + threadIdx.x;  // channel i of this lane at col[i * 64]
  const int64_t r = ((int64_t)blockIdx.x * 64 + threadIdx.x) * VEC;
  if (r >= a.n_rows) return;
  int64_t ib, ob;
  softmax_row_base(a, r, &ib, &ob);
  const T* in = reinterpret_cast<const T*>(a.in) + ib;
  T* out = reinterpret_cast<T*>(a.out) + ob;
  T m[VEC];
  double sum[VEC];
  T inv[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) { m[e] = -__builtin_huge_valf(); sum[e] = 0.0; }
  constexpr int U = 16;  // channels fetched ahead
  for (uint32_t i0 = 0; i0 < a.k; i0 += U) {
    V x[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (i0 + u < a.k) x[u] = nt_load(reinterpret_cast<const V*>(in + (int64_t)(i0 + u) * a.in_k));
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (i0 + u < a.k) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) m[e] = jvm_max(m[e], x[u].v[e]);
        col[(i0 + u) * 64] = x[u];
      }
  }
  for (uint32_t i = 0; i < a.k; ++i) {
    V x = col[i * 64];
#pragma unroll
    for (int e = 0; e < VEC; ++e) { x.v[e] = shifted_exp(x.v[e], m[e]); sum[e] += (double)x.v[e]; }
    col[i * 64] = x;
  }
#pragma unroll
  for (int e = 0; e < VEC; ++e) inv[e] = (T)1 / (T)sum[e];
  for (uint32_t i = 0; i < a.k; ++i) {
    V x = col[i * 64];
#pragma unroll
    for (int e = 0; e < VEC; ++e) x.v[e] *= inv[e];
    *reinterpret_cast<V*>(out + (int64_t)i * a.out_k) = x;
  }
}

// Short rows stored back to back (a dense [rows, k] block) whose length is no
// whole number of 16-byte vectors, e.g. ten classes.  A block stages its 256
// rows, one contiguous stretch of memory, through LDS with 128-bit accesses;
// one lane then owns one row in LDS.  (With one lane per element the same rows
// move 4 bytes per lane and reach under a fifth of the memory rate.)
template <class T>
__global__ void __launch_bounds__(kBlock) softmax_short_rows_kernel(const SoftmaxArgs a) {
  constexpr int VEC = 16 / (int)sizeof(T);
  using V = Vec<T, VEC>;
  extern __shared__ __align__(16) char smem[];
  T* tile = reinterpret_cast<T*>(smem);
  const uint32_t k = a.k;
  const int64_t row0 = (int64_t)blockIdx.x * kBlock;
  const uint32_t n_rows = (uint32_t)(a.n_rows - row0 < kBlock ? a.n_rows - row0 : kBlock);
  const uint32_t count = n_rows * k;
  const T* in = reinterpret_cast<const T*>(a.in) + row0 * k;
  T* out = reinterpret_cast<T*>(a.out) + row0 * k;
  // a block's stretch starts on the 16-byte grid whenever the tensor does (256 * k elements per block)
  const uint32_t n_vec = count / VEC;
  for (uint32_t v = threadIdx.x; v < n_vec; v += kBlock)
    reinterpret_cast<V*>(tile)[v] = reinterpret_cast<const V*>(in)[v];
  for (uint32_t e = n_vec * VEC + threadIdx.x; e < count; e += kBlock) tile[e] = in[e];
  __syncthreads();
  if (threadIdx.x < n_rows) {
    T* row = tile + threadIdx.x * k;
    T m = -__builtin_huge_valf();
    for (uint32_t j = 0; j < k; ++j) m = jvm_max(m, row[j]);
    double sum = 0.0;
    for (uint32_t j = 0; j < k; ++j) {
      const T e = shifted_exp(row[j], m);
      row[j] = e;
      sum += (double)e;
    }
    const T inv = (T)1 / (T)sum;
    for (uint32_t j = 0; j < k; ++j) row[j] *= inv;
  }
  __syncthreads();
  for (uint32_t v = threadIdx.x; v < n_vec; v += kBlock)
    reinterpret_cast<V*>(out)[v] = reinterpret_cast<const V*>(tile)[v];
  for (uint32_t e = n_vec * VEC + threadIdx.x; e < count; e += kBlock) out[e] = tile[e];
}

struct RowLayout { int64_t outer, rows, k, s_outer, s_row, s_k; };

// [rows, k] or [outer, rows, k]; spatial swaps the last two axes (dimensions.clj:473-484 with [0 2 1]).
int row_layout(const ct_dims* d, bool spatial, const char* what, RowLayout* l) {
  if (int rc = check_dims(d, what)) return rc;
  CT_REQUIRE(dims_direct(*d), "softmax!: %s must have direct dimensions", what);
  CT_REQUIRE(d->ndim == 2 || d->ndim == 3, "softmax implementation only supports shapes of 2 or 3 dimensions");
  CT_REQUIRE(!spatial || d->ndim == 3, "softmax-spatial! needs [batch channels elements]");
  if (d->ndim == 2) {
    *l = RowLayout{1, d->shape[0], d->shape[1], 0, d->strides[0], d->strides[1]};
  } else if (!spatial) {
    *l = RowLayout{d->shape[0], d->shape[1], d->shape[2], d->strides[0], d->strides[1], d->strides[2]};
  } else {
    *l = RowLayout{d->shape[0], d->shape[2], d->shape[1], d->strides[0], d->strides[2], d->strides[1]};
  }
  return CT_OK;
}

template <class T>
int softmax_run(hipStream_t s, void* out, const RowLayout& ol, const void* in, const RowLayout& il) {
  SoftmaxArgs a;
  std::memset(&a, 0, sizeof(a));
  a.in = in; a.out = out;
  a.n_rows = il.outer * il.rows;
  a.k = (uint32_t)il.k;
  a.rows_fd = FastDiv((uint32_t)il.rows);
  a.in_outer = il.s_outer; a.in_row = il.s_row; a.in_k = il.s_k;
  a.out_outer = ol.s_outer; a.out_row = ol.s_row; a.out_k = ol.s_k;
  if (a.n_rows == 0) return CT_OK;
  // lanes along the row axis when that is the unit-stride one (spatial form) or the rows are tiny
  const bool row_major = il.s_k == 1 || il.k == 1;
  if (il.k < 8 || (!row_major && il.s_row == 1)) {
    constexpr int VL = 16 / (int)sizeof(T);
    // More than 16 float channels held four positions wide cost waves per compute unit: two
    // positions per lane measured 2.5 points of the HBM peak better at 21 and 32 channels, two
    // points worse at 4, the same at 10.
    const bool half_vec = sizeof(T) == 4 && il.k > 16;
    auto lanes_ok = [](const void* p, const RowLayout& l) {
      return l.s_row == 1 && l.rows % VL == 0 && l.s_k % VL == 0 && l.s_outer % VL == 0 && (uintptr_t)p % 16 == 0;
    };
    const bool vec_rows = lanes_ok(in, il) && lanes_ok(out, ol);
    const int64_t lanes = vec_rows ? a.n_rows / (half_vec ? 2 : VL) : a.n_rows;
    // Rows too long for registers are parked in LDS while at least five waves still fit a
    // compute unit.  One row per lane: four neighbouring rows per lane need four times the LDS
    // per wave and measured 32 % of peak against 56 % at 64 channels (24 % for the loop form).
    constexpr int64_t kLdsRowBytes = 32 << 10;
    if (il.k > 32 && il.k * 64 * (int64_t)sizeof(T) <= kLdsRowBytes && il.s_row == 1 && ol.s_row == 1) {
      note_kernel("softmax_lane_lds");
      hipLaunchKernelGGL((softmax_lane_lds_kernel<T, 1>), dim3((uint32_t)((a.n_rows + 63) / 64)), dim3(64),
                         (size_t)il.k * 64 * sizeof(T), s, a);
      return after_launch(s);
    }
    const dim3 grid((uint32_t)((lanes + kBlock - 1) / kBlock));
    note_kernel(il.k <= 32 ? (vec_rows ? "softmax_lane_vec" : "softmax_lane") : (vec_rows ? "softmax_lane_loop_vec" : "softmax_lane_loop"));
#define CT_SM_LANE(VEC_)                                                                                  \
  if (il.k <= 8) hipLaunchKernelGGL((softmax_lane_kernel<T, VEC_, 8>), grid, dim3(kBlock), 0, s, a);       \
  else if (il.k <= 16) hipLaunchKernelGGL((softmax_lane_kernel<T, VEC_, 16>), grid, dim3(kBlock), 0, s, a); \
  else if (il.k <= 24) hipLaunchKernelGGL((softmax_lane_kernel<T, VEC_, 24>), grid, dim3(kBlock), 0, s, a); \
  else if (il.k <= 32) hipLaunchKernelGGL((softmax_lane_kernel<T, VEC_, 32>), grid, dim3(kBlock), 0, s, a); \
  else hipLaunchKernelGGL((softmax_lane_kernel<T, VEC_, 0>), grid, dim3(kBlock), 0, s, a)
    if (vec_rows && half_vec) { CT_SM_LANE(2); } else if (vec_rows) { CT_SM_LANE(VL); } else { CT_SM_LANE(1); }
#undef CT_SM_LANE
    return after_launch(s);
  }
  constexpr int VMAX = 16 / (int)sizeof(T);
  auto aligned = [](const void* p, const RowLayout& l) {
    return l.s_k == 1 && l.k % VMAX == 0 && l.s_row % VMAX == 0 && l.s_outer % VMAX == 0 &&
           (uintptr_t)p % 16 == 0;
  };
  const bool vec_ok = aligned(in, il) && aligned(out, ol);
  const int64_t nv = vec_ok ? il.k / VMAX : il.k;
  // input plus output beyond the 256 MiB last-level cache: non-temporal loads
  const bool streams = 2.0 * (double)a.n_rows * (double)il.k * sizeof(T) > (double)(int64_t(256) << 20);
  auto dense_rows = [](const void* p, const RowLayout& l) {
    return l.s_k == 1 && l.s_row == l.k && (l.outer == 1 || l.s_outer == l.rows * l.k) && (uintptr_t)p % 16 == 0;
  };
  if (!vec_ok && il.k * (int64_t)sizeof(T) <= 128 && a.n_rows >= 4 * kBlock && dense_rows(in, il) && dense_rows(out, ol)) {
    note_kernel("softmax_short_rows");
    hipLaunchKernelGGL((softmax_short_rows_kernel<T>), dim3((uint32_t)((a.n_rows + kBlock - 1) / kBlock)), dim3(kBlock),
                       (size_t)kBlock * il.k * sizeof(T), s, a);
    return after_launch(s);
  }
#define CT_SM(VEC, TPR, ITER)                                                                                    \
  do {                                                                                                           \
    const dim3 grid((uint32_t)((a.n_rows + (kBlock / TPR) - 1) / (kBlock / TPR)));                               \
    if (streams) hipLaunchKernelGGL((softmax_wave_kernel<T, VEC, TPR, ITER, true>), grid, dim3(kBlock), 0, s, a); \
    else hipLaunchKernelGGL((softmax_wave_kernel<T, VEC, TPR, ITER, false>), grid, dim3(kBlock), 0, s, a);       \
  } while (0)
#define CT_SM_SHAPES(VEC)                     \
  if (nv <= 4) CT_SM(VEC, 4, 1);              \
  else if (nv <= 16) CT_SM(VEC, 16, 1);       \
  else if (nv <= 32) CT_SM(VEC, 16, 2);       \
  else if (nv <= 64) CT_SM(VEC, 16, 4);       \
  else if (nv <= 128) CT_SM(VEC, 64, 2);      \
  else if (nv <= 256) CT_SM(VEC, 64, 4);      \
  else if (nv <= 512) CT_SM(VEC, 64, 8);      \
  else CT_SM(VEC, 64, 16)
  if (nv <= 1024) {
    note_kernel(vec_ok ? "softmax_wave_vec" : "softmax_wave");
    if (vec_ok) { CT_SM_SHAPES(VMAX); } else { CT_SM_SHAPES(1); }
  } else if (vec_ok && VMAX > 1 && nv <= 16 * kBlock) {
    note_kernel("softmax_block_reg");
    if (nv <= 8 * kBlock) hipLaunchKernelGGL((softmax_block_reg_kernel<T, VMAX, 8>), dim3((uint32_t)a.n_rows), dim3(kBlock), 0, s, a);
    else hipLaunchKernelGGL((softmax_block_reg_kernel<T, VMAX, 16>), dim3((uint32_t)a.n_rows), dim3(kBlock), 0, s, a);
  } else {
    note_kernel("softmax_block");
    hipLaunchKernelGGL((softmax_block_kernel<T>), dim3((uint32_t)a.n_rows), dim3(kBlock), 0, s, a);
  }
#undef CT_SM_SHAPES
#undef CT_SM
  return after_launch(s);
}

int softmax_entry(void* stream, void* output, const ct_dims* od, const void* input, const ct_dims* id, int dtype,
                  bool spatial) {
  CT_REQUIRE(output && input, "softmax!: null buffer");
  RowLayout ol, il;
  if (int rc = row_layout(od, spatial, "output", &ol)) return rc;
  if (int rc = row_layout(id, spatial, "input", &il)) return rc;
  CT_REQUIRE(ol.outer == il.outer && ol.rows == il.rows && ol.k == il.k, "Input, output shapes do not match");
  CT_REQUIRE(il.outer * il.rows < (int64_t(1) << 31) && il.k < (int64_t(1) << 31), "softmax!: too many rows");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == CT_F32) return softmax_run<float>(s, output, ol, input, il);
  if (dtype == CT_F64) return softmax_run<double>(s, output, ol, input, il);
  return set_error(CT_ERR_INVALID, "softmax! is only defined for float and double tensors");
}

}  // namespace

extern "C" {

int ct_activation_gradient(void* stream, void* input_gradient, const ct_dims* input_gradient_dims,
                           const void* output_gradient, const ct_dims* output_gradient_dims, const void* output,
                           const ct_dims* output_dims, int op, int64_t n, int dtype) {
  CT_REQUIRE(input_gradient && output_gradient && output, "ct_activation_gradient: null buffer");
  CT_REQUIRE(n >= 0, "ct_activation_gradient: negative count");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == CT_F32)
    return act_grad_typed<float>(s, input_gradient, input_gradient_dims, output_gradient, output_gradient_dims, output,
                                 output_dims, op, n);
  if (dtype == CT_F64)
    return act_grad_typed<double>(s, input_gradient, input_gradient_dims, output_gradient, output_gradient_dims,
                                  output, output_dims, op, n);
  return set_error(CT_ERR_INVALID, "activation-gradient! is only defined for float and double tensors");
}

int ct_softmax_eltwise(void* stream, void* output, const ct_dims* output_dims, const void* input,
                       const ct_dims* input_dims, int dtype) {
  return softmax_entry(stream, output, output_dims, input, input_dims, dtype, false);
}

int ct_softmax_spatial(void* stream, void* output, const ct_dims* output_dims, const void* input,
                       const ct_dims* input_dims, int dtype) {
  return softmax_entry(stream, output, output_dims, input, input_dims, dtype, true);
}

}  // extern "C"
