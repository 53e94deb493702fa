// functors.h -- scalar operations of the tensor-math path with the value
// semantics of the reference's CPU backend.
//
// For float tensors the CPU backend widens every operand to double, performs
// the operation in double and rounds once at the store
// (src/cortex/compute/cpu/tensor_math.clj:211-223, 278-304, 464-466); integer
// tensors widen to long, wrap, and narrow by truncation.  The functors below
// do the same on the device, one rounding per JVM operation (the library is
// compiled with -ffp-contract=off so no multiply-add is fused).
//
// exp, tanh and logistic on float tensors with alpha == 1 are evaluated by the
// single-precision device routines (about 1 ulp, far inside the 2e-6 relative
// budget of a transcendental) because the double-precision routines would make
// these kernels compute-bound; tanh has a form of its own (tanh_f32, within 6e-7
// relative) because a transposing kernel has about 45 instruction slots per
// element at memory speed and the library routine's share of them made it the
// bound.  Every other float operation is bit-identical to the CPU backend.
//
// PLAIN functors are the float forms whose multipliers are +-1.  Then x * alpha
// is exact in float, and one correctly rounded float operation (+ - * / sqrt,
// floor, ceil, a comparison) equals the double operation rounded once to float
// (a double carries more than 2 * 24 + 2 bits), so the widening is skipped.
// Which form runs is decided on the host: a run-time flag inside the functor
// would put a branch, and both code paths, into every unrolled element of the
// kernels.
#pragma once

#include "common.h"

namespace cthip {

// ------------------------------------------------------------------ assign

template <class D, class S> struct AssignF {
  static constexpr int NIN = 1;
  static constexpr bool kLace = true;  // planar <-> interleaved images go through ew_lace_kernel
  using Out = D;
  using In0 = S;
  using In1 = D;
  using In2 = D;
  __device__ __forceinline__ D operator()(S s, D, D) const { return jvm_convert<D, S>(s); }
};

template <class T> struct ConstantF {
  static constexpr int NIN = 0;
  using Out = T;
  using In0 = T;
  using In1 = T;
  using In2 = T;
  T value;
  __device__ __forceinline__ T operator()(T, T, T) const { return value; }
};

// A multiplier of a byte or short tensor has been cast to T on the host.  Saying so again where it
// is used lets the compiler take the full-rate 24-bit multiply instead of the quarter-rate 32-bit one.
template <class T, class A> __device__ __forceinline__ A in_range_of(A a) {
  if constexpr (std::is_integral<T>::value && sizeof(T) <= 2) return (A)(T)a;
  else return a;
}

// ------------------------------------------------------------------ unary

// java.lang.Math.round: nearest long, ties toward +infinity, NaN -> 0.
__device__ __forceinline__ int64_t jvm_round(double v) {
  if (v != v) return 0;
  double r = floor(v);
  if (v - r >= 0.5) r += 1.0;
  return jvm_d2l(r);
}

// exp of a double argument to float accuracy (about 1 ulp of the float result): v * log2(e) is split
// in double into an integer n and a fraction in [-0.5, 0.5]; the hardware's exp2 takes the fraction
// as a float and ldexp applies n.  n is clamped to +-300, which keeps it a number for NaN and
// infinite arguments; those reach exp2 through the fraction and come out NaN, +infinity and 0.
__device__ __forceinline__ float exp_f32_of(double v) {
  const double a = v * 1.4426950408889634;
  const double n = __builtin_fmin(__builtin_fmax(__builtin_rint(a), -300.0), 300.0);
  return __builtin_ldexpf(__builtin_amdgcn_exp2f((float)(a - n)), (int)n);
}

__device__ __forceinline__ float tanh_f32(float x);

// tanh in double precision, for double and integer tensors (the library routine costs three times
// an exp and left these kernels at a third of the memory rate).  |x| >= 0.05: 1 - 2 / (exp(2|x|) + 1),
// whose subtraction magnifies the four or so roundings before it by 1 / (2|x|): within 5e-15 of the
// result.  Below: x - x^3/3 + 2x^5/15 - 17x^7/315 + 62x^9/2835 - 1382x^11/155925, truncated under
// 1e-18 of the result there.  Infinite arguments give +-1 (exp overflows to infinity and the quotient
// is 0), NaN stays NaN, the sign (of zero too) is the argument's.
__device__ __forceinline__ double tanh_f64(double x) {
  const double a = __builtin_fabs(x);
  if (a < 0.05) {
    const double s = x * x;
    return x * (1.0 + s * (-1.0 / 3.0 + s * (2.0 / 15.0 + s * (-17.0 / 315.0 + s * (62.0 / 2835.0 + s * (-1382.0 / 155925.0))))));
  }
  const double e = exp(2.0 * a);
  return __builtin_copysign(1.0 - 2.0 / (e + 1.0), x);
}

// perform-unary-op-impl (cpu/tensor_math.clj:211-223) on v = x * alpha.  Float tensors with a
// multiplier other than 1 take the transcendental ops through the single-precision forms too
// (the product itself is formed in double): inside the 2e-6 relative bar, and memory-bound where
// the double routines were not.
template <class T, int OP, class A> __device__ __forceinline__ T unary_value(A v) {
  if constexpr (std::is_same<T, float>::value && std::is_same<A, double>::value) {
    if constexpr (OP == CT_UOP_EXP) return exp_f32_of(v);
    else if constexpr (OP == CT_UOP_TANH) return tanh_f32((float)v);
    else if constexpr (OP == CT_UOP_LOGISTIC) return 1.0f / (1.0f + exp_f32_of(-v));
  }
  if constexpr (OP == CT_UOP_FLOOR) return jvm_cast<T>(floor((double)v));
  else if constexpr (OP == CT_UOP_CEIL) return jvm_cast<T>(ceil((double)v));
  else if constexpr (OP == CT_UOP_ROUND) return jvm_cast<T>(jvm_round((double)v));
  else if constexpr (OP == CT_UOP_NEGATE) return jvm_cast<T>(w_neg(v));
  else if constexpr (OP == CT_UOP_TANH) return jvm_cast<T>(tanh_f64((double)v));
  else if constexpr (OP == CT_UOP_LOGISTIC) return jvm_cast<T>(1.0 / (1.0 + exp((double)w_neg(v))));
  else if constexpr (OP == CT_UOP_EXP) return jvm_cast<T>(exp((double)v));
  else if constexpr (OP == CT_UOP_SQRT) return jvm_cast<T>(sqrt((double)v));
  else return jvm_cast<T>((double)v);
}

// tanh in single precision.  |x| >= 0.4: 1 - 2 / (exp(2|x|) + 1) with the hardware's exp2 and
// reciprocal (1 ulp each; the subtraction loses at most two bits there).  Below: the odd
// polynomial x + x^3 p(x^2), p fitted to (tanh(x)/x - 1)/x^2 on [0, 0.4] (6.4e-8 relative).
// A dense sweep of the argument range against the double routine stays within 6e-7 relative.
// Infinite arguments give +-1, NaN stays NaN, the sign (of zero too) is the argument's.
__device__ __forceinline__ float tanh_f32(float x) {
  const float a = __builtin_fabsf(x);
  const float e = __builtin_amdgcn_exp2f(a * 2.885390081777927f);  // exp(2a); inf for large a
  const float r = __builtin_amdgcn_rcpf(e + 1.0f);
  const float big = __builtin_fmaf(-2.0f, r, 1.0f);
  const float s = a * a;
  float p = 0.01873837038874626f;
  p = __builtin_fmaf(p, s, -0.05356000363826752f);
  p = __builtin_fmaf(p, s, 0.1333119422197342f);
  p = __builtin_fmaf(p, s, -0.33333298563957214f);
  const float small = __builtin_fmaf(a * s, p, a);
  return __builtin_copysignf(a < 0.4f ? small : big, x);
}

template <class T, int OP, bool PLAIN = false> struct UnaryF {
  static constexpr int NIN = 1;
  using Out = T;
  using In0 = T;
  using In1 = T;
  using In2 = T;
  using A = typename ew_acc_of<T>::type;
  A alpha;  // 1 when PLAIN
  __device__ __forceinline__ T operator()(T x, T, T) const {
    if constexpr (PLAIN) {
      static_assert(std::is_same<T, float>::value, "PLAIN is a float form");
      if constexpr (OP == CT_UOP_TANH) return tanh_f32(x);
      else if constexpr (OP == CT_UOP_EXP) return expf(x);
      else if constexpr (OP == CT_UOP_LOGISTIC) return 1.0f / (1.0f + expf(-x));
      else if constexpr (OP == CT_UOP_FLOOR) return floorf(x);
      else if constexpr (OP == CT_UOP_CEIL) return ceilf(x);
      else if constexpr (OP == CT_UOP_NEGATE) return -x;
      else if constexpr (OP == CT_UOP_SQRT) return sqrtf(x);
      else if constexpr (OP == CT_UOP_NOOP) return x;
      else return unary_value<T, OP, A>((A)x);
    } else {
      return unary_value<T, OP, A>(w_mul((A)x, in_range_of<T>(alpha)));
    }
  }
};

// ------------------------------------------------------------------ binary

__device__ __forceinline__ int32_t jvm_unchecked_int(int64_t v) { return (int32_t)(uint32_t)(uint64_t)v; }
__device__ __forceinline__ int32_t jvm_unchecked_int(int32_t v) { return v; }
__device__ __forceinline__ int32_t jvm_unchecked_int(double v) { return jvm_d2i(v); }

// perform-operation-impl (cpu/tensor_math.clj:278-304).  An integer division by zero, where the
// reference throws ArithmeticException, stores 0 and sets *div0 (when given).
template <class T, int OP, class A> __device__ __forceinline__ T binary_value(A x, A y, uint32_t* div0 = nullptr) {
  if constexpr (OP == CT_BOP_ADD) return jvm_cast<T>(w_add(x, y));
  else if constexpr (OP == CT_BOP_SUB) return jvm_cast<T>(w_sub(x, y));
  else if constexpr (OP == CT_BOP_MUL) return jvm_cast<T>(w_mul(x, y));
  else if constexpr (OP == CT_BOP_DIV) {
    if constexpr (std::is_same<A, double>::value) return jvm_cast<T>(x / y);
    else {
      if (y == 0 && div0) *div0 = 1u;
      return jvm_ratio_cast<T>(x, y);
    }
  }
  else if constexpr (OP == CT_BOP_MAX) return jvm_cast<T>(x > y ? x : y);
  else if constexpr (OP == CT_BOP_MIN) return jvm_cast<T>(x > y ? y : x);
  else if constexpr (OP == CT_BOP_BIT_AND) return jvm_cast<T>((int64_t)(jvm_unchecked_int(x) & jvm_unchecked_int(y)));
  else if constexpr (OP == CT_BOP_BIT_XOR) return jvm_cast<T>((int64_t)(jvm_unchecked_int(x) ^ jvm_unchecked_int(y)));
  else if constexpr (OP == CT_BOP_EQ) return jvm_cast<T>((int64_t)(x == y ? 1 : 0));
  else if constexpr (OP == CT_BOP_GT) return jvm_cast<T>((int64_t)(x > y ? 1 : 0));
  else if constexpr (OP == CT_BOP_GE) return jvm_cast<T>((int64_t)(x >= y ? 1 : 0));
  else if constexpr (OP == CT_BOP_LT) return jvm_cast<T>((int64_t)(x < y ? 1 : 0));
  else return jvm_cast<T>((int64_t)(x <= y ? 1 : 0));
}

// dest = op(x * xa, y * ya).  A scalar operand is passed as a constant input
// with alpha 1 (the caller has already folded its alpha, src/cortex/tensor.clj:680).
// PLAIN: float, xa and ya are +-1, and OP is one of binary_plain_op's.
constexpr bool binary_plain_op(int op) {
  return op == CT_BOP_ADD || op == CT_BOP_SUB || op == CT_BOP_MUL || op == CT_BOP_DIV || op == CT_BOP_MIN ||
         op == CT_BOP_MAX || op == CT_BOP_EQ || op == CT_BOP_GT || op == CT_BOP_GE || op == CT_BOP_LT || op == CT_BOP_LE;
}

template <class T, int OP, bool PLAIN = false> struct BinaryF {
  static constexpr int NIN = 2;
  using Out = T;
  using In0 = T;
  using In1 = T;
  using In2 = T;
  using A = typename ew_acc_of<T>::type;
  A xa, ya;
  uint32_t* div0 = nullptr;  // integer :/ only: the device's error word (see device_error_word)
  __device__ __forceinline__ T operator()(T x, T y, T) const {
    if constexpr (PLAIN) {
      static_assert(std::is_same<T, float>::value && binary_plain_op(OP), "PLAIN is a float form");
      const float fx = xa < 0 ? -x : x, fy = ya < 0 ? -y : y;
      if constexpr (OP == CT_BOP_ADD) return fx + fy;
      else if constexpr (OP == CT_BOP_SUB) return fx - fy;
      else if constexpr (OP == CT_BOP_MUL) return fx * fy;
      else if constexpr (OP == CT_BOP_DIV) return fx / fy;
      else if constexpr (OP == CT_BOP_MAX) return fx > fy ? fx : fy;
      else if constexpr (OP == CT_BOP_MIN) return fx > fy ? fy : fx;
      else if constexpr (OP == CT_BOP_EQ) return fx == fy ? 1.0f : 0.0f;
      else if constexpr (OP == CT_BOP_GT) return fx > fy ? 1.0f : 0.0f;
      else if constexpr (OP == CT_BOP_GE) return fx >= fy ? 1.0f : 0.0f;
      else if constexpr (OP == CT_BOP_LT) return fx < fy ? 1.0f : 0.0f;
      else return fx <= fy ? 1.0f : 0.0f;
    } else {
      return binary_value<T, OP, A>(w_mul((A)x, in_range_of<T>(xa)), w_mul((A)y, in_range_of<T>(ya)), div0);
    }
  }
};

template <class A> inline bool unit_magnitude(A v) { return v == (A)1 || v == (A)-1; }

// ------------------------------------------------------------------ ternary select

// Three tensors (cpu/tensor_math.clj:469-497): the comparison sees the
// unrounded products.  PLAIN: float with all three multipliers 1.
template <class T, bool PLAIN = false> struct SelectF {
  static constexpr int NIN = 3;
  using Out = T;
  using In0 = T;
  using In1 = T;
  using In2 = T;
  using A = typename ew_acc_of<T>::type;
  A xa, ya, za;
  __device__ __forceinline__ T operator()(T x, T y, T z) const {
    if constexpr (PLAIN) {
      return x >= (T)0 ? z : y;
    } else {
      const A vx = w_mul(xa, (A)x);
      return jvm_cast<T>(vx >= (A)0 ? w_mul(za, (A)z) : w_mul(ya, (A)y));
    }
  }
};

// One or two constants (cpu/tensor_math.clj:507-567): every argument is cast
// to the tensor datatype before the comparison; arg_idx routes the three slots
// (tensors first, then constants) to x, y, z.
template <class T> struct SelectRoutedF {
  static constexpr int NIN = 3;
  using Out = T;
  using In0 = T;
  using In1 = T;
  using In2 = T;
  using A = typename ew_acc_of<T>::type;
  A alpha[3];  // 1 for constant slots
  int8_t arg_idx[3];
  __device__ __forceinline__ T operator()(T s0, T s1, T s2) const {
    const T v0 = jvm_cast<T>(w_mul(alpha[0], (A)s0));
    const T v1 = jvm_cast<T>(w_mul(alpha[1], (A)s1));
    const T v2 = jvm_cast<T>(w_mul(alpha[2], (A)s2));
    auto pick = [&](int i) { return i == 0 ? v0 : (i == 1 ? v1 : v2); };
    const T x = pick(arg_idx[0]), y = pick(arg_idx[1]), z = pick(arg_idx[2]);
    return ((A)x >= (A)0) ? z : y;
  }
};

// The constant forms with the condition in a tensor, which is what callers write (a mask
// x >= 0 ? 1/p : 0, a clamp x >= 0 ? x : 0): the constants travel in the functor, so the call
// has one or two inputs and runs on the kernels of a unary or binary op, and nothing is routed
// per element.  Same value rules as SelectRoutedF.  PLAIN: float with every multiplier 1.
//   SelectCCF          x >= 0 ? cz : cy
//   SelectTCF<false>   x >= 0 ? cz : q      (q is the y argument)
//   SelectTCF<true>    x >= 0 ? q  : cy     (q is the z argument)
template <class T, bool PLAIN = false> struct SelectCCF {
  static constexpr int NIN = 1;
  using Out = T;
  using In0 = T;
  using In1 = T;
  using In2 = T;
  using A = typename ew_acc_of<T>::type;
  A xa;
  T cy, cz;
  __device__ __forceinline__ T operator()(T x, T, T) const {
    const T vx = PLAIN ? x : jvm_cast<T>(w_mul(xa, (A)x));
    return ((A)vx >= (A)0) ? cz : cy;
  }
};

template <class T, bool Q_IS_Z, bool PLAIN = false> struct SelectTCF {
  static constexpr int NIN = 2;
  using Out = T;
  using In0 = T;
  using In1 = T;
  using In2 = T;
  using A = typename ew_acc_of<T>::type;
  A xa, qa;
  T c;
  __device__ __forceinline__ T operator()(T x, T q, T) const {
    const T vx = PLAIN ? x : jvm_cast<T>(w_mul(xa, (A)x));
    const T vq = PLAIN ? q : jvm_cast<T>(w_mul(qa, (A)q));
    const bool pass = (A)vx >= (A)0;
    return Q_IS_Z ? (pass ? vq : c) : (pass ? c : vq);
  }
};

}  // namespace cthip
