// ops_optim.hip -- fused Adam and Adadelta steps over flat buffers.
//
// Adam follows cpu-adam-step-impl! (src/cortex/optimize/adam.clj:68-102): the
// seven scalars are cast to the buffer datatype first, then every operation
// runs in double with one rounding each, and m, v, p are rounded once at the
// store.  dx is computed from the unrounded m' and v'.
// Adadelta follows AdadeltaOptimizer.step_f / step_d
// (java/cortex/compute/optimize/AdadeltaOptimizer.java:29-64): the float
// variant forms gradient_alpha * gradient in float, widens, runs the
// micro-step in double and adds (float)dx to the parameter in float.
//
// Both kernels are pure streaming: 16 bytes read and 12 written per float
// parameter.  Each lane owns VEC consecutive elements per iteration so that
// every access is a 128-bit coalesced load or store when the four buffers are
// 16-byte aligned; m and v may sit at an arbitrary element offset of the flat
// optimizer state, in which case narrower vectors are used.
//
// Launch shape.  Four read streams and three write streams over the same four
// buffers are bound by how well the memory controllers can batch the mix, not
// by the kernel: with no arithmetic at all the same accesses run at the same
// rate.  Measured at 2^28 floats per buffer (percent of the 8 TB/s peak): one
// read stream 94, one write stream 84, copy 84, 2 reads + 1 write 83.5, 3 + 1
// 82, 4 + 1 80, 4 + 2 80, 4 + 3 78 (in place or into separate buffers alike),
// 4 + 4 76.  Within that, blocks of one wave in plain block order measured
// best: 79.0 against 77.3 for 256-lane blocks dealt to the dies in groups
// (256-lane blocks in plain order 77.4, 128-lane 76; two vectors per lane
// 74-76; a persistent grid-stride loop with prefetch 58-66; die groups of 16 /
// 32 / 64 blocks 63 / 67 / 69).  The non-temporal bit on loads and on stores
// is worth 9 points each (70 and 71.5 without); the scope bits change nothing.
#include "elementwise.h"

using namespace cthip;

namespace {

struct AdamScalars {
  double alpha, beta1, beta2, eps, one_minus_beta1, one_minus_beta2, one_minus_pb1, one_minus_pb2, ga;
};

constexpr int kOptBlock = 64;  // one wave per block
// The four buffers of a step together up to this size (the last-level cache) are read and written
// with plain accesses, larger ones with non-temporal ones.  Adam on float: 16 M parameters
// (256 MiB) 86 % of peak plain against 77 % non-temporal, 24 M (384 MiB) 70 % against 77 %.
constexpr int64_t kOptCacheBytes = int64_t(256) << 20;

template <class T, int VEC, int UNROLL, bool streaming>
__global__ void __launch_bounds__(kOptBlock) adam_kernel(const AdamScalars s, const T* g, T* p, T* m, T* v,
                                                         int64_t n_vecs) {
  using V = Vec<T, VEC>;
  constexpr int kBlock = kOptBlock;
  const int64_t first = (int64_t)blockIdx.x * (kBlock * UNROLL) + threadIdx.x;
  V gv[UNROLL], pv[UNROLL], mv[UNROLL], vv[UNROLL];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const int64_t i = first + (int64_t)u * kBlock;
    if (i < n_vecs) {
      gv[u] = streaming ? nt_load(reinterpret_cast<const V*>(g) + i) : reinterpret_cast<const V*>(g)[i];
      pv[u] = streaming ? nt_load(reinterpret_cast<const V*>(p) + i) : reinterpret_cast<const V*>(p)[i];
      mv[u] = streaming ? nt_load(reinterpret_cast<const V*>(m) + i) : reinterpret_cast<const V*>(m)[i];
      vv[u] = streaming ? nt_load(reinterpret_cast<const V*>(v) + i) : reinterpret_cast<const V*>(v)[i];
    }
  }
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const int64_t i = first + (int64_t)u * kBlock;
    if (i >= n_vecs) continue;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const double grad = s.ga * (double)gv[u].v[e];
      const double lm = s.beta1 * (double)mv[u].v[e] + s.one_minus_beta1 * grad;
      const double lv = s.beta2 * (double)vv[u].v[e] + (s.one_minus_beta2 * grad) * grad;
      const double dx = s.alpha * (lm / (s.one_minus_pb1 * (sqrt(lv / s.one_minus_pb2) + s.eps)));
      mv[u].v[e] = (T)lm;
      vv[u].v[e] = (T)lv;
      pv[u].v[e] = (T)((double)pv[u].v[e] - dx);
    }
    if (streaming) {
      nt_store(mv[u], reinterpret_cast<V*>(m) + i);
      nt_store(vv[u], reinterpret_cast<V*>(v) + i);
      nt_store(pv[u], reinterpret_cast<V*>(p) + i);
    } else {
      reinterpret_cast<V*>(m)[i] = mv[u];
      reinterpret_cast<V*>(v)[i] = vv[u];
      reinterpret_cast<V*>(p)[i] = pv[u];
    }
  }
}

template <class T> struct AdadeltaScalars { T ga; double decay, eps, one_minus_decay; };

template <class T, int VEC, int UNROLL, bool streaming>
__global__ void __launch_bounds__(kOptBlock) adadelta_kernel(const AdadeltaScalars<T> s, const T* g, T* p, T* gacc,
                                                             T* dacc, int64_t n_vecs) {
  using V = Vec<T, VEC>;
  constexpr int kBlock = kOptBlock;
  const int64_t first = (int64_t)blockIdx.x * (kBlock * UNROLL) + threadIdx.x;
  V gv[UNROLL], pv[UNROLL], av[UNROLL], dv[UNROLL];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const int64_t i = first + (int64_t)u * kBlock;
    if (i < n_vecs) {
      gv[u] = streaming ? nt_load(reinterpret_cast<const V*>(g) + i) : reinterpret_cast<const V*>(g)[i];
      pv[u] = streaming ? nt_load(reinterpret_cast<const V*>(p) + i) : reinterpret_cast<const V*>(p)[i];
      av[u] = streaming ? nt_load(reinterpret_cast<const V*>(gacc) + i) : reinterpret_cast<const V*>(gacc)[i];
      dv[u] = streaming ? nt_load(reinterpret_cast<const V*>(dacc) + i) : reinterpret_cast<const V*>(dacc)[i];
    }
  }
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const int64_t i = first + (int64_t)u * kBlock;
    if (i >= n_vecs) continue;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const double grad = (double)(T)(s.ga * gv[u].v[e]);  // product in the buffer type, then widened
      const double ga = grad * grad * s.decay + (double)av[u].v[e] * s.one_minus_decay;
      const double rms_g = sqrt(ga + s.eps);
      const double rms_dx = sqrt((double)dv[u].v[e] + s.eps);
      const double dx = (-1.0 * rms_dx * grad) / rms_g;
      const double da = dx * dx * s.decay + (double)dv[u].v[e] * s.one_minus_decay;
      av[u].v[e] = (T)ga;
      dv[u].v[e] = (T)da;
      pv[u].v[e] = (T)(pv[u].v[e] + (T)dx);
    }
    if (streaming) {
      nt_store(av[u], reinterpret_cast<V*>(gacc) + i);
      nt_store(dv[u], reinterpret_cast<V*>(dacc) + i);
      nt_store(pv[u], reinterpret_cast<V*>(p) + i);
    } else {
      reinterpret_cast<V*>(gacc)[i] = av[u];
      reinterpret_cast<V*>(dacc)[i] = dv[u];
      reinterpret_cast<V*>(p)[i] = pv[u];
    }
  }
}

// Largest power-of-two vector width (in elements, at most 16 bytes) at which
// all four buffers are aligned.
template <class T> int common_vec_width(const void* a, const void* b, const void* c, const void* d) {
  const uintptr_t bits = (uintptr_t)a | (uintptr_t)b | (uintptr_t)c | (uintptr_t)d;
  int vec = 16 / (int)sizeof(T);
  while (vec > 1 && (bits % (uintptr_t)(vec * sizeof(T))) != 0) vec >>= 1;
  return vec;
}

constexpr int kUnroll = 1;  // one vector per lane per buffer

template <class T, int VEC>
void adam_launch(hipStream_t st, const AdamScalars& s, const T* g, T* p, T* m, T* v, int64_t n) {
  const bool streaming = n * 4 * (int64_t)sizeof(T) > kOptCacheBytes;
  const int64_t n_vecs = n / VEC;
  if (n_vecs > 0) {
    const int64_t per = (int64_t)kOptBlock * kUnroll;
    const dim3 grid((uint32_t)((n_vecs + per - 1) / per));
    if (streaming) hipLaunchKernelGGL((adam_kernel<T, VEC, kUnroll, true>), grid, dim3(kOptBlock), 0, st, s, g, p, m, v, n_vecs);
    else hipLaunchKernelGGL((adam_kernel<T, VEC, kUnroll, false>), grid, dim3(kOptBlock), 0, st, s, g, p, m, v, n_vecs);
  }
  const int64_t done = n_vecs * VEC;
  if (VEC > 1 && done < n)
    hipLaunchKernelGGL((adam_kernel<T, 1, 1, false>), dim3(1), dim3(kOptBlock), 0, st, s, g + done, p + done, m + done,
                       v + done, n - done);
}

template <class T>
int adam_typed(hipStream_t st, double alpha, double beta1, double beta2, double eps, double pb1, double pb2,
               double ga, const void* g, void* p, void* m, void* v, int64_t n) {
  AdamScalars s;
  // scalars are cast to the datatype first (adam.clj:124-129), then widened
  s.alpha = (double)(T)alpha;
  s.beta1 = (double)(T)beta1;
  s.beta2 = (double)(T)beta2;
  s.eps = (double)(T)eps;
  s.ga = (double)(T)ga;
  s.one_minus_beta1 = 1.0 - s.beta1;
  s.one_minus_beta2 = 1.0 - s.beta2;
  s.one_minus_pb1 = 1.0 - (double)(T)pb1;
  s.one_minus_pb2 = 1.0 - (double)(T)pb2;
  const int vec = common_vec_width<T>(g, p, m, v);
  const T* gp = (const T*)g;
  T *pp = (T*)p, *mp = (T*)m, *vp = (T*)v;
  note_kernel(vec > 1 ? "adam_vec" : "adam_scalar");
  if (vec == 4) adam_launch<T, (sizeof(T) == 4 ? 4 : 1)>(st, s, gp, pp, mp, vp, n);
  else if (vec == 2) adam_launch<T, 2>(st, s, gp, pp, mp, vp, n);
  else adam_launch<T, 1>(st, s, gp, pp, mp, vp, n);
  return after_launch(st);
}

template <class T, int VEC>
void adadelta_launch(hipStream_t st, const AdadeltaScalars<T>& s, const T* g, T* p, T* a, T* d, int64_t n) {
  const bool streaming = n * 4 * (int64_t)sizeof(T) > kOptCacheBytes;
  const int64_t n_vecs = n / VEC;
  if (n_vecs > 0) {
    const int64_t per = (int64_t)kOptBlock * kUnroll;
    const dim3 grid((uint32_t)((n_vecs + per - 1) / per));
    if (streaming) hipLaunchKernelGGL((adadelta_kernel<T, VEC, kUnroll, true>), grid, dim3(kOptBlock), 0, st, s, g, p, a, d, n_vecs);
    else hipLaunchKernelGGL((adadelta_kernel<T, VEC, kUnroll, false>), grid, dim3(kOptBlock), 0, st, s, g, p, a, d, n_vecs);
  }
  const int64_t done = n_vecs * VEC;
  if (VEC > 1 && done < n)
    hipLaunchKernelGGL((adadelta_kernel<T, 1, 1, false>), dim3(1), dim3(kOptBlock), 0, st, s, g + done, p + done, a + done,
                       d + done, n - done);
}

template <class T>
int adadelta_typed(hipStream_t st, double decay, double eps, void* gacc, void* dacc, double ga, const void* g,
                   void* p, int64_t n) {
  AdadeltaScalars<T> s;
  s.ga = (T)ga;
  s.decay = (double)(T)decay;
  s.eps = (double)(T)eps;
  s.one_minus_decay = 1.0 - s.decay;
  const int vec = common_vec_width<T>(g, p, gacc, dacc);
  const T* gp = (const T*)g;
  T *pp = (T*)p, *ap = (T*)gacc, *dp = (T*)dacc;
  note_kernel(vec > 1 ? "adadelta_vec" : "adadelta_scalar");
  if (vec == 4) adadelta_launch<T, (sizeof(T) == 4 ? 4 : 1)>(st, s, gp, pp, ap, dp, n);
  else if (vec == 2) adadelta_launch<T, 2>(st, s, gp, pp, ap, dp, n);
  else adadelta_launch<T, 1>(st, s, gp, pp, ap, dp, n);
  return after_launch(st);
}

}  // namespace

extern "C" {

int ct_adam_step(void* stream, int dtype, double alpha, double beta1, double beta2, double epsilon,
                 double pow_beta1_t, double pow_beta2_t, double gradient_alpha, const void* gradient,
                 void* parameters, void* m, void* v, int64_t n) {
  CT_REQUIRE(n >= 0, "ct_adam_step: negative count");
  if (n == 0) return CT_OK;
  CT_REQUIRE(gradient && parameters && m && v, "ct_adam_step: null buffer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == CT_F32)
    return adam_typed<float>(st, alpha, beta1, beta2, epsilon, pow_beta1_t, pow_beta2_t, gradient_alpha, gradient,
                             parameters, m, v, n);
  if (dtype == CT_F64)
    return adam_typed<double>(st, alpha, beta1, beta2, epsilon, pow_beta1_t, pow_beta2_t, gradient_alpha, gradient,
                              parameters, m, v, n);
  return set_error(CT_ERR_INVALID, "ct_adam_step: datatype must be float or double");
}

int ct_adadelta_step(void* stream, int dtype, double decay, double epsilon, void* grad_sq_accum,
                     void* dx_sq_accum, double gradient_alpha, const void* gradient, void* parameters,
                     int64_t n) {
  CT_REQUIRE(n >= 0, "ct_adadelta_step: negative count");
  if (n == 0) return CT_OK;
  CT_REQUIRE(gradient && parameters && grad_sq_accum && dx_sq_accum, "ct_adadelta_step: null buffer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == CT_F32)
    return adadelta_typed<float>(st, decay, epsilon, grad_sq_accum, dx_sq_accum, gradient_alpha, gradient,
                                 parameters, n);
  if (dtype == CT_F64)
    return adadelta_typed<double>(st, decay, epsilon, grad_sq_accum, dx_sq_accum, gradient_alpha, gradient,
                                  parameters, n);
  return set_error(CT_ERR_INVALID, "ct_adadelta_step: datatype must be float or double");
}

}  // extern "C"
