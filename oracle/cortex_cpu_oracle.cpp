// cortex_cpu_oracle.cpp -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
//
// A CPU restatement of the cortex CPU tensor backend for the tensor-math hot
// path, written from the reference's source text (the reference is Clojure on
// the JVM and cannot be executed where this is built).  It exists to check the
// HIP library and to serve as the timed CPU baseline.  Only the tests, the
// smoke check and the benchmark's cpu_baseline leg may load it; the product
// library never does.
//
// What follows which reference file (paths under /root/reference):
//   address functions        src/cortex/compute/cpu/tensor_math.clj:33-134
//                            src/cortex/tensor/dimensions.clj:178-211, 226-353
//   casts                    src/cortex/compute/cpu/driver.clj:149-157 under
//                            *unchecked-math* (cpu/tensor_math.clj:28): Java
//                            primitive narrowing (JLS 5.1.3)
//   assign-constant!         cpu/tensor_math.clj:137-153
//   assign!                  cpu/tensor_math.clj:180-208
//   unary-op!/unary-accum!   cpu/tensor_math.clj:211-262
//   binary ops               cpu/tensor_math.clj:278-462
//   ternary select           cpu/tensor_math.clj:464-580
//   unary-reduce!            cpu/tensor_math.clj:582-663
//   activation-gradient!     cpu/tensor_math.clj:1318-1362
//   softmax (both forms)     cpu/tensor_math.clj:1037-1103
//   batch-normalize (6 forms) cpu/tensor_math.clj:731-1033, 1558-1638
//   convolution (3 methods)  cpu/tensor_math.clj:1118-1151, 1670-1792: unroll, gemm!,
//                            roll back
//   pooling (6 forms)        cpu/tensor_math.clj:1153-1284, 1800-1866 over the
//                            window walk of src/cortex/nn/impl.clj:8-96
//   gemm!, gemv!             cpu/tensor_math.clj:672-726, 1534-1556 and
//                            compute/math_util.clj:17-41 for the operand
//                            mapping; the product itself is netlib BLAS
//                            (com.github.fommil.netlib, not under
//                            /root/reference) whose published definition
//                            C = alpha op(A) op(B) + beta C is restated with a
//                            double accumulator
//   rand!                    cpu/tensor_math.clj:1867-1890 for the arithmetic
//                            around the draws; the generator itself is this
//                            build's (Philox4x32-10, Salmon et al. SC'11), pinned
//                            by the Random123 known-answer vectors -- the
//                            reference draws from SecureRandom / cuRAND and
//                            fixes only the distribution
//   local response           no CPU form in the reference: cuDNN's published cross-channel LRN,
//   normalization            called from cuda/tensor_math.clj:1277-1335
//   Adam                     src/cortex/optimize/adam.clj:68-102
//   Adadelta                 java/cortex/compute/optimize/AdadeltaOptimizer.java:29-64
//
// Parity pinning: every function here is checked by tests/test_oracle_*.py
// against the reference's stored vectors (src/cortex/verify/tensor.clj,
// src/cortex/compute/verify/optimize.clj, examples/optimise/test/...) and
// against closed forms / brute force.  CT_U8 has no reference counterpart
// (the reference's :byte is signed); it is pinned by closed form only.
//
// Arithmetic model.  Clojure has no float arithmetic: float operands widen to
// double, the operation runs in double, and the store rounds once.  Integer
// operands widen to long; under *unchecked-math* long arithmetic wraps and the
// narrowing casts truncate.  Each JVM operation rounds separately (no FMA), so
// this file is compiled with -ffp-contract=off.

#include <algorithm>
#include <cmath>
#ifdef _OPENMP
#include <omp.h>
#endif
#include <cstdint>
#include <cstring>
#include <limits>
#include <type_traits>

#include "../include/cortex_hip.h"

namespace {

thread_local char g_err[256] = "";
int fail(const char* msg) {
  std::strncpy(g_err, msg, sizeof(g_err) - 1);
  g_err[sizeof(g_err) - 1] = 0;
  return CT_ERR_INVALID;
}

// ---------------------------------------------------------------- JVM casts

inline int32_t j_d2i(double v) {  // JLS 5.1.3: NaN -> 0, saturating, toward zero
  if (v != v) return 0;
  if (v >= 2147483647.0) return INT32_MAX;
  if (v <= -2147483648.0) return INT32_MIN;
  return (int32_t)v;
}
inline int64_t j_d2l(double v) {
  if (v != v) return 0;
  if (v >= 9223372036854775808.0) return INT64_MAX;
  if (v <= -9223372036854775808.0) return INT64_MIN;
  return (int64_t)v;
}

// cast<T>(long) and cast<T>(double): datatype->cast-fn applied to the result of
// an integer or floating computation.
template <class T> inline T jcast(int64_t v) {
  if constexpr (std::is_floating_point<T>::value) return (T)v;  // round to nearest even
  else return (T)(uint64_t)v;                                   // truncate to the low bits
}
template <class T> inline T jcast(double v) {
  if constexpr (std::is_same<T, double>::value) return v;
  else if constexpr (std::is_same<T, float>::value) return (float)v;
  else if constexpr (std::is_same<T, int64_t>::value) return j_d2l(v);
  else return (T)(uint32_t)j_d2i(v);  // byte/short: through int, then truncate
}
// Element of type S converted to T (assign!).  float widens exactly to double,
// every integer type widens exactly to long.
template <class T, class S> inline T jconvert(S s) {
  if constexpr (std::is_floating_point<S>::value) return jcast<T>((double)s);
  else return jcast<T>((int64_t)s);
}

// Accumulator type of a tensor datatype: double for float/double, long otherwise.
template <class T> struct acc_of {
  using type = typename std::conditional<std::is_floating_point<T>::value, double, int64_t>::type;
};

inline int64_t wmul(int64_t a, int64_t b) { return (int64_t)((uint64_t)a * (uint64_t)b); }
inline int64_t wadd(int64_t a, int64_t b) { return (int64_t)((uint64_t)a + (uint64_t)b); }
inline int64_t wsub(int64_t a, int64_t b) { return (int64_t)((uint64_t)a - (uint64_t)b); }
inline int64_t wneg(int64_t a) { return (int64_t)(0 - (uint64_t)a); }
inline double wmul(double a, double b) { return a * b; }
inline double wadd(double a, double b) { return a + b; }
inline double wsub(double a, double b) { return a - b; }
inline double wneg(double a) { return -a; }

// java.lang.Math.round(double): nearest long, ties toward positive infinity.
inline int64_t j_round(double v) {
  if (v != v) return 0;
  double r = std::floor(v);
  if (v - r >= 0.5) r += 1.0;  // v - floor(v) is exact
  return j_d2l(r);
}
// java.lang.Math.max/min(double, double): NaN propagates, +0 > -0.
inline double j_max(double a, double b) {
  if (a != a) return a;
  if (b != b) return b;
  if (a == 0.0 && b == 0.0) return std::signbit(a) ? b : a;
  return a > b ? a : b;
}
inline double j_min(double a, double b) {
  if (a != a) return a;
  if (b != b) return b;
  if (a == 0.0 && b == 0.0) return std::signbit(a) ? a : b;
  return a < b ? a : b;
}
inline int64_t j_max(int64_t a, int64_t b) { return a > b ? a : b; }
inline int64_t j_min(int64_t a, int64_t b) { return a < b ? a : b; }

// ---------------------------------------------------------------- dimensions

struct Dims {  // one operand, slowest first
  int nd;
  int64_t shape[CT_MAX_DIMS];
  int64_t strides[CT_MAX_DIMS];
  const int32_t* index[CT_MAX_DIMS];
};

bool load_dims(const ct_dims* in, Dims* out) {
  if (!in || in->ndim < 1 || in->ndim > CT_MAX_DIMS) return false;
  out->nd = in->ndim;
  for (int i = 0; i < in->ndim; ++i) {
    if (in->shape[i] < 1) return false;
    out->shape[i] = in->shape[i];
    out->strides[i] = in->strides[i];
    out->index[i] = in->index[i];
  }
  return true;
}

int64_t ecount(const Dims& d) {  // dimensions.clj:131-134
  int64_t n = 1;
  for (int i = 0; i < d.nd; ++i) n *= d.shape[i];
  return n;
}
bool direct(const Dims& d) {  // dimensions.clj:61-63, 194-196
  for (int i = 0; i < d.nd; ++i)
    if (d.index[i]) return false;
  return true;
}
bool access_increasing(const Dims& d) {  // dimensions.clj:204-211
  if (!direct(d)) return false;
  for (int i = 0; i + 1 < d.nd; ++i)
    if (d.strides[i] < d.strides[i + 1]) return false;
  return true;
}
bool dense(const Dims& d) {  // dimensions.clj:178-191
  if (!direct(d)) return false;
  if (d.nd == 1) return d.strides[0] == 1;
  // drop size-1 dims, stable-sort by stride descending, compare the largest
  // stride with the product of the remaining shapes.
  int64_t shp[CT_MAX_DIMS], str[CT_MAX_DIMS];
  int k = 0;
  for (int i = 0; i < d.nd; ++i)
    if (d.shape[i] != 1) { shp[k] = d.shape[i]; str[k] = d.strides[i]; ++k; }
  if (k == 0) return false;  // (first []) is nil; (= nil 1) is false
  for (int i = 1; i < k; ++i)  // insertion sort, stable, descending stride
    for (int j = i; j > 0 && str[j - 1] < str[j]; --j) {
      std::swap(str[j - 1], str[j]);
      std::swap(shp[j - 1], shp[j]);
    }
  int64_t prod = 1;
  for (int i = 1; i < k; ++i) prod *= shp[i];
  return str[0] == prod;
}

// max-extend-strides (dimensions.clj:280-300): left-pad strides with
// stride*shape of the largest-stride dimension (first one on ties).
void padded(const Dims& d, int max_nd, int64_t* shape, int64_t* strides, const int32_t** index) {
  int mi = 0;
  for (int i = 1; i < d.nd; ++i)
    if (d.strides[i] > d.strides[mi]) mi = i;
  int64_t pad = d.strides[mi] * d.shape[mi];
  int off = max_nd - d.nd;
  for (int i = 0; i < off; ++i) { shape[i] = 1; strides[i] = pad; index[i] = nullptr; }
  for (int i = 0; i < d.nd; ++i) {
    shape[off + i] = d.shape[i];
    strides[off + i] = d.strides[i];
    index[off + i] = d.index[i];
  }
}

struct MaxShape { int nd; int64_t s[CT_MAX_DIMS]; };

// dimension-seq->max-shape (dimensions.clj:326-353)
MaxShape max_shape_of(const Dims* const* ops, int n_ops) {
  MaxShape m;
  m.nd = 0;
  for (int k = 0; k < n_ops; ++k)
    if (ops[k]->nd > m.nd) m.nd = ops[k]->nd;
  for (int i = 0; i < m.nd; ++i) m.s[i] = 0;
  for (int k = 0; k < n_ops; ++k) {
    int off = m.nd - ops[k]->nd;
    for (int i = 0; i < m.nd; ++i) {
      int64_t v = i < off ? 1 : ops[k]->shape[i - off];
      if (v > m.s[i]) m.s[i] = v;
    }
  }
  return m;
}

// get-elem-dims->address (cpu/tensor_math.clj:82-134): the four address
// objects of the CPU backend, selected exactly as the reference selects them.
struct Addr {
  enum Mode { IDENTITY, BCAST, REPEAT, GENERAL } mode;
  int64_t ec, amt;
  int nd;  // GENERAL: reversed (fastest first) data
  int64_t rshape[CT_MAX_DIMS], rstrides[CT_MAX_DIMS], rmax[CT_MAX_DIMS];
  const int32_t* rindex[CT_MAX_DIMS];

  inline int64_t operator()(int64_t e) const {
    switch (mode) {
      case IDENTITY: return e;                  // SimpleElemIdxToAddr :50-53
      case BCAST: return (e / amt) % ec;        // SimpleBcastAddr :56-60
      case REPEAT: return e % ec;               // SimpleRepeatAddr :63-66
      default: break;
    }
    // elem-idx->addr (dimensions.clj:226-252)
    int64_t off = 0, arg = e;
    for (int i = 0; i < nd; ++i) {
      int64_t c = arg % rshape[i];
      arg /= rmax[i];
      off += rstrides[i] * (rindex[i] ? (int64_t)rindex[i][c] : c);
    }
    return off;
  }
};

Addr make_addr(const Dims& d, const MaxShape& mx) {
  Addr a;
  std::memset(&a, 0, sizeof(a));
  const bool dn = dense(d), inc = access_increasing(d), dir = direct(d);
  const int64_t ec = ecount(d);
  bool same_shape = d.nd == mx.nd;
  for (int i = 0; same_shape && i < d.nd; ++i) same_shape = d.shape[i] == mx.s[i];
  if (dir && same_shape && dn && inc) { a.mode = Addr::IDENTITY; return a; }
  int64_t biggest = 0;
  for (int i = 0; i < d.nd; ++i) biggest = d.shape[i] > biggest ? d.shape[i] : biggest;
  if (dir && ec == biggest && dn && inc) {
    // first position in the left-padded shape whose size equals ec
    int off = mx.nd - d.nd, pos = -1;
    for (int i = 0; i < mx.nd && pos < 0; ++i) {
      int64_t v = i < off ? 1 : d.shape[i - off];
      if (v == ec) pos = i;
    }
    int64_t amt = 1;
    for (int i = pos + 1; i < mx.nd; ++i) amt *= mx.s[i];
    a.mode = Addr::BCAST; a.ec = ec; a.amt = amt;
    return a;
  }
  if (dir && dn && inc) {
    int lead = 0;  // drop leading 1s, compare with the tail of max-shape
    while (lead < d.nd && d.shape[lead] == 1) ++lead;
    int m = d.nd - lead;
    bool suffix = m <= mx.nd;
    for (int i = 0; suffix && i < m; ++i) suffix = d.shape[lead + i] == mx.s[mx.nd - m + i];
    if (suffix) { a.mode = Addr::REPEAT; a.ec = ec; return a; }
  }
  a.mode = Addr::GENERAL;
  a.nd = mx.nd;
  int64_t shp[CT_MAX_DIMS], str[CT_MAX_DIMS];
  const int32_t* idx[CT_MAX_DIMS];
  padded(d, mx.nd, shp, str, idx);
  for (int i = 0; i < mx.nd; ++i) {
    a.rshape[i] = shp[mx.nd - 1 - i];
    a.rstrides[i] = str[mx.nd - 1 - i];
    a.rindex[i] = idx[mx.nd - 1 - i];
    a.rmax[i] = mx.s[mx.nd - 1 - i];
  }
  return a;
}

MaxShape own_shape(const Dims& d) {
  MaxShape m;
  m.nd = d.nd;
  for (int i = 0; i < d.nd; ++i) m.s[i] = d.shape[i];
  return m;
}

// ---------------------------------------------------------------- scalar ops

// perform-unary-op-impl (cpu/tensor_math.clj:211-223); v = x * alpha in the
// accumulator type.
template <class T, class A> inline T unary_apply(int op, A v) {
  switch (op) {
    case CT_UOP_FLOOR: return jcast<T>(std::floor((double)v));
    case CT_UOP_CEIL: return jcast<T>(std::ceil((double)v));
    case CT_UOP_ROUND: return jcast<T>(j_round((double)v));
    case CT_UOP_NEGATE: return jcast<T>(wneg(v));
    case CT_UOP_TANH: return jcast<T>(std::tanh((double)v));
    case CT_UOP_LOGISTIC: return jcast<T>(1.0 / (1.0 + std::exp((double)wneg(v))));
    case CT_UOP_EXP: return jcast<T>(std::exp((double)v));
    case CT_UOP_SQRT: return jcast<T>(std::sqrt((double)v));
    default: return jcast<T>((double)v);  // :noop is (double x)
  }
}

// (dtype-cast (/ a b)) on integer operands.  Clojure's (/ long long) yields a
// Long when the division is exact and a Ratio otherwise.  The unchecked cast
// of a Long truncates to the low bits; Ratio.longValue truncates toward zero;
// Ratio.intValue (which the byte and short casts also go through) is
// (int)doubleValue, i.e. it saturates at the int range.
template <class T> inline T ratio_cast(int64_t n, int64_t d) {
  if (n == INT64_MIN && d == -1) return jcast<T>(n);
  const int64_t q = n / d;
  if (n % d == 0 || std::is_same<T, int64_t>::value) return jcast<T>(q);
  return jcast<T>((double)q);
}

inline int32_t unchecked_int(int64_t v) { return (int32_t)(uint32_t)(uint64_t)v; }
inline int32_t unchecked_int(double v) { return j_d2i(v); }

// perform-operation-impl (cpu/tensor_math.clj:278-304).  *div0 is raised when
// an integer division by zero occurs (the reference throws ArithmeticException).
template <class T, class A> inline T binary_apply(int op, A x, A y, bool* div0) {
  switch (op) {
    case CT_BOP_ADD: return jcast<T>(wadd(x, y));
    case CT_BOP_SUB: return jcast<T>(wsub(x, y));
    case CT_BOP_MUL: return jcast<T>(wmul(x, y));
    case CT_BOP_DIV:
      if constexpr (std::is_same<A, double>::value) {
        return jcast<T>(x / y);
      } else {  // boxed Ratio, then a truncating cast
        if (y == 0) { *div0 = true; return (T)0; }
        return ratio_cast<T>(x, y);
      }
    case CT_BOP_MAX: return jcast<T>(x > y ? x : y);
    case CT_BOP_MIN: return jcast<T>(x > y ? y : x);
    case CT_BOP_BIT_AND: return jcast<T>((int64_t)(unchecked_int(x) & unchecked_int(y)));
    case CT_BOP_BIT_XOR: return jcast<T>((int64_t)(unchecked_int(x) ^ unchecked_int(y)));
    case CT_BOP_EQ: return jcast<T>((int64_t)(x == y ? 1 : 0));
    case CT_BOP_GT: return jcast<T>((int64_t)(x > y ? 1 : 0));
    case CT_BOP_GE: return jcast<T>((int64_t)(x >= y ? 1 : 0));
    case CT_BOP_LT: return jcast<T>((int64_t)(x < y ? 1 : 0));
    default: return jcast<T>((int64_t)(x <= y ? 1 : 0));
  }
}

#define DISPATCH_DTYPE(dt, ...)                                      \
  switch (dt) {                                                      \
    case CT_I8: { using T = int8_t; __VA_ARGS__; } break;            \
    case CT_I16: { using T = int16_t; __VA_ARGS__; } break;          \
    case CT_I32: { using T = int32_t; __VA_ARGS__; } break;          \
    case CT_I64: { using T = int64_t; __VA_ARGS__; } break;          \
    case CT_F32: { using T = float; __VA_ARGS__; } break;            \
    case CT_F64: { using T = double; __VA_ARGS__; } break;           \
    case CT_U8: { using T = uint8_t; __VA_ARGS__; } break;           \
    default: return fail("unknown datatype");                        \
  }

// ---------------------------------------------------------------- op bodies

template <class T>
int assign_constant_t(T* d, const Dims& dd, double value, int64_t n) {
  const Addr ad = make_addr(dd, own_shape(dd));
  const T v = jcast<T>(value);
#pragma omp parallel for schedule(static)
  for (int64_t e = 0; e < n; ++e) d[ad(e)] = v;
  return 0;
}

template <class T, class S>
int assign_t(T* d, const Dims& dd, const S* s, const Dims& sd, int64_t n) {
  const Dims* ops[2] = {&dd, &sd};
  const MaxShape mx = max_shape_of(ops, 2);
  const Addr ad = make_addr(dd, mx), as = make_addr(sd, mx);
#pragma omp parallel for schedule(static)
  for (int64_t e = 0; e < n; ++e) d[ad(e)] = jconvert<T, S>(s[as(e)]);
  return 0;
}

template <class T>
int unary_t(T* d, const Dims& dd, const T* x, const Dims* xd, double alpha, int op, int64_t n) {
  using A = typename acc_of<T>::type;
  const A al = (A)jcast<T>(alpha);
  if (!xd) {  // unary-accum!: serial, in place
    const Addr ad = make_addr(dd, own_shape(dd));
    for (int64_t e = 0; e < n; ++e) {
      const int64_t i = ad(e);
      d[i] = unary_apply<T, A>(op, wmul((A)d[i], al));
    }
    return 0;
  }
  const Dims* ops[2] = {&dd, xd};
  const MaxShape mx = max_shape_of(ops, 2);
  const Addr ad = make_addr(dd, mx), ax = make_addr(*xd, mx);
#pragma omp parallel for schedule(static)
  for (int64_t e = 0; e < n; ++e) d[ad(e)] = unary_apply<T, A>(op, wmul((A)x[ax(e)], al));
  return 0;
}

// x == nullptr: accumulate into dest (serial).  y == nullptr: scalar operand.
template <class T>
int binary_t(T* d, const Dims& dd, const T* x, const Dims* xd, double x_alpha, const T* y,
             const Dims* yd, double y_alpha, double scalar, int64_t n, int op, bool reverse) {
  using A = typename acc_of<T>::type;
  const A xa = (A)jcast<T>(x_alpha);
  const A ya = (A)jcast<T>(y_alpha);
  const A sc = (A)jcast<T>(scalar);
  bool div0 = false;
  const Dims* ops[3];
  int n_ops = 0;
  ops[n_ops++] = &dd;
  if (xd) ops[n_ops++] = xd;
  if (yd) ops[n_ops++] = yd;
  // the accumulate-constant form takes its max-shape from dest alone
  const MaxShape mx = (n_ops == 1) ? own_shape(dd) : max_shape_of(ops, n_ops);
  const Addr ad = make_addr(dd, mx);
  Addr ax = ad, ay = ad;
  if (xd) ax = make_addr(*xd, mx);
  if (yd) ay = make_addr(*yd, mx);
  if (!x) {  // binary-accum! / binary-accum-constant!: c-for, increasing e
    for (int64_t e = 0; e < n; ++e) {
      const int64_t i = ad(e);
      const A lhs = wmul((A)d[i], xa);
      const A rhs = y ? wmul((A)y[ay(e)], ya) : sc;
      d[i] = reverse ? binary_apply<T, A>(op, rhs, lhs, &div0) : binary_apply<T, A>(op, lhs, rhs, &div0);
    }
  } else {
#pragma omp parallel for schedule(static) reduction(|| : div0)
    for (int64_t e = 0; e < n; ++e) {
      const A lhs = wmul((A)x[ax(e)], xa);
      const A rhs = y ? wmul((A)y[ay(e)], ya) : sc;
      d[ad(e)] = reverse ? binary_apply<T, A>(op, rhs, lhs, &div0) : binary_apply<T, A>(op, lhs, rhs, &div0);
    }
  }
  return div0 ? fail("Divide by zero") : 0;
}

// select-impl (cpu/tensor_math.clj:464-466)
template <class A> inline A select3(A x, A y, A z) { return (x >= (A)0) ? z : y; }

// Three tensors: the comparison sees the unrounded products
// (cpu/tensor_math.clj:469-497).  With constants every argument is cast to the
// datatype BEFORE the comparison (cpu/tensor_math.clj:530-537, 560-567).
template <class T>
int ternary_t(T* d, const Dims& dd, const T* const* t, const Dims* const* td, const double* alpha,
              int n_tensors, const double* constants, const int8_t* arg_idx, int64_t n) {
  using A = typename acc_of<T>::type;
  const Dims* ops[4];
  ops[0] = &dd;
  for (int k = 0; k < n_tensors; ++k) ops[k + 1] = td[k];
  const MaxShape mx = max_shape_of(ops, n_tensors + 1);
  const Addr ad = make_addr(dd, mx);
  Addr at[3];
  A al[3];
  for (int k = 0; k < n_tensors; ++k) { at[k] = make_addr(*td[k], mx); al[k] = (A)jcast<T>(alpha[k]); }
  if (n_tensors == 3) {
#pragma omp parallel for schedule(static)
    for (int64_t e = 0; e < n; ++e)
      d[ad(e)] = jcast<T>(select3<A>(wmul(al[0], (A)t[0][at[0](e)]), wmul(al[1], (A)t[1][at[1](e)]),
                                     wmul(al[2], (A)t[2][at[2](e)])));
    return 0;
  }
  T cst[3] = {0, 0, 0};  // constants arrive as boxed doubles and are cast to T
  for (int k = n_tensors; k < 3; ++k) cst[k] = jcast<T>(constants[k - n_tensors]);
#pragma omp parallel for schedule(static)
  for (int64_t e = 0; e < n; ++e) {
    T v[3];
    for (int k = 0; k < 3; ++k)
      v[k] = k < n_tensors ? jcast<T>(wmul(al[k], (A)t[k][at[k](e)])) : cst[k];
    d[ad(e)] = jcast<T>(select3<A>((A)v[arg_idx[0]], (A)v[arg_idx[1]], (A)v[arg_idx[2]]));
  }
  return 0;
}

// do-unary-reduce-op (cpu/tensor_math.clj:588-629): sequential, accumulator in
// the widened type, seeded with the first element.
template <class T>
int reduce_t(T* out, const Dims& od, double alpha, const T* in, const Dims& id, int op) {
  using A = typename acc_of<T>::type;
  const Addr ao = make_addr(od, own_shape(od)), ai = make_addr(id, own_shape(id));
  const A al = (A)jcast<T>(alpha);
  const int64_t par = ecount(od);
  const int64_t iter = ecount(id) / par;
  if (iter < 1) return fail("unary-reduce!: input smaller than output");
#pragma omp parallel for schedule(static)
  for (int64_t p = 0; p < par; ++p) {
    const int64_t start = p * iter, stop = start + iter;
    A acc = wmul(al, (A)in[ai(start)]);
    if (op == CT_ROP_MAGNITUDE || op == CT_ROP_MAGNITUDE_SQUARED) acc = wmul(acc, acc);
    for (int64_t i = start + 1; i < stop; ++i) {
      const A v = wmul(al, (A)in[ai(i)]);
      switch (op) {
        case CT_ROP_MAX: acc = j_max(acc, v); break;
        case CT_ROP_MIN: acc = j_min(acc, v); break;
        case CT_ROP_SUM:
        case CT_ROP_MEAN: acc = wadd(acc, v); break;
        default: acc = wadd(acc, wmul(v, v)); break;
      }
    }
    T r;
    if (op == CT_ROP_MEAN) {
      // (/ sum count): double division, or a Ratio truncated by the cast
      if constexpr (std::is_same<A, double>::value) r = jcast<T>(acc / (double)iter);
      else r = ratio_cast<T>(acc, iter);
    } else if (op == CT_ROP_MAGNITUDE) {
      r = jcast<T>(std::sqrt((double)acc));
    } else {
      r = jcast<T>(acc);
    }
    out[ao(p)] = r;
  }
  return 0;
}

// act-backward-impl (cpu/tensor_math.clj:1318-1362).  Float operands widen to
// double, the products run left to right in double, the store rounds once.
template <class T>
int activation_gradient_t(T* ig, const Dims& igd, const T* og, const Dims& ogd, const T* out, const Dims& od,
                          int op, int64_t n) {
  const Dims* ops[3] = {&igd, &ogd, &od};
  const MaxShape mx = max_shape_of(ops, 3);
  const Addr ia = make_addr(igd, mx), ga = make_addr(ogd, mx), oa = make_addr(od, mx);
#pragma omp parallel for schedule(static)
  for (int64_t e = 0; e < n; ++e) {
    const double o = (double)out[oa(e)], g = (double)og[ga(e)];
    double r;
    switch (op) {
      case CT_ACT_LOGISTIC: r = (o * (1.0 - o)) * g; break;
      case CT_ACT_TANH: r = (1.0 - o * o) * g; break;
      default: r = (o > 0.0 ? 1.0 : 0.0) * g; break;  // relu
    }
    ig[ia(e)] = (T)r;
  }
  return 0;
}

// softmax-impl (cpu/tensor_math.clj:1037-1088).  The loop that finds the row
// maximum reads element 0 through the input's address object and elements
// 1..k-1 of the INPUT buffer through the OUTPUT's address object (:1067-1072);
// that is restated as written.  The exponentials are stored rounded to T, their
// stored values are summed sequentially in double, the sum is rounded to T and
// every element is divided by it in T (ArrayView.diveq).
template <class T>
int softmax_t(T* out, const Dims& od, const T* in, const Dims& id) {
  const Dims* ops[2] = {&od, &id};
  const MaxShape mx = max_shape_of(ops, 2);
  if (mx.nd != 2 && mx.nd != 3) return fail("softmax implementation only supports shapes of 2 or 3 dimensions");
  const Addr oa = make_addr(od, mx), ia = make_addr(id, mx);
  const int64_t outer = mx.nd == 2 ? 1 : mx.s[0], par = mx.nd == 2 ? mx.s[0] : mx.s[1],
                k = mx.nd == 2 ? mx.s[1] : mx.s[2];
  for (int64_t o = 0; o < outer; ++o) {
#pragma omp parallel for schedule(static)
    for (int64_t p = 0; p < par; ++p) {
      const int64_t off = o * par * k + p * k;
      double mv = (double)in[ia(off)];
      for (int64_t i = 1; i < k; ++i) mv = j_max(mv, (double)in[oa(off + i)]);
      const T max_val = (T)mv;
      for (int64_t i = 0; i < k; ++i) out[oa(off + i)] = (T)std::exp((double)in[ia(off + i)] - (double)max_val);
      double sum = (double)out[oa(off)];
      for (int64_t i = 1; i < k; ++i) sum += (double)out[oa(off + i)];
      const T sum_val = (T)sum;
      for (int64_t i = 0; i < k; ++i) out[oa(off + i)] = out[oa(off + i)] / sum_val;
    }
  }
  return 0;
}

// dimensions/transpose with [0 2 1] (dimensions.clj:473-484)
inline bool transpose_021(const Dims& d, Dims* t) {
  if (d.nd != 3) return false;
  *t = d;
  std::swap(t->shape[1], t->shape[2]);
  std::swap(t->strides[1], t->strides[2]);
  std::swap(t->index[1], t->index[2]);
  return true;
}

// ---------------------------------------------------------------- batch normalization
// BNEltwiseOffsetter / BNSpatialOffsetter (cpu/tensor_math.clj:737-753): the
// "parallel" index selects the statistic (an element, or a channel), the other
// index walks the values that share it.  The eltwise form is the spatial form
// with one element per channel.
struct BnOffsetter {
  int64_t batch, channels, elements;
  int64_t parallel_count() const { return channels; }
  int64_t idx_count() const { return batch * elements; }
  int64_t operator()(int64_t c, int64_t i) const {
    return (i % elements) + c * elements + (i / elements) * (channels * elements);
  }
};

// sum-double-var (cpu/tensor_math.clj:805-817): a sequential double sum seeded
// with the first term.
template <class F> inline double sum_double_var(int64_t n, F term) {
  if (n == 0) return 0.0;
  double s = term((int64_t)0);
  for (int64_t i = 1; i < n; ++i) s = s + term(i);
  return s;
}

// batch-normalize-impl (cpu/tensor_math.clj:756-784).  inv-std-dev is rounded
// to T; the per-element arithmetic runs in double and the store rounds once.
template <class T>
void bn_apply_t(const BnOffsetter& o, T* out, const T* in, const T* means, const T* variances, const T* scale,
                const T* bias, double epsilon_) {
  const T epsilon = (T)epsilon_;
  const int64_t pc = o.parallel_count(), ic = o.idx_count();
#pragma omp parallel for schedule(static)
  for (int64_t c = 0; c < pc; ++c) {
    const T variance = variances[c];
    const T inv_std_dev = (T)std::sqrt(1.0 / ((double)variance + (double)epsilon));
    const T mean = means[c], sc = scale[c], shift = bias[c];
    for (int64_t i = 0; i < ic; ++i) {
      const int64_t off = o(c, i);
      const double x_hat = ((double)in[off] - (double)mean) * (double)inv_std_dev;
      out[off] = (T)(x_hat * (double)sc + (double)shift);
    }
  }
}

// batch-normalize-update-impl (cpu/tensor_math.clj:820-870).
template <class T>
void bn_update_t(const BnOffsetter& o, const T* in, T* batch_means, T* batch_variances, T* running_means,
                 T* running_variances, double average_factor) {
  const T ave_factor = (T)average_factor;
  const double ave_lerp = (double)(T)1.0 - (double)ave_factor;
  const int64_t pc = o.parallel_count(), ic = o.idx_count();
  const double count_val = std::max(1.0, (double)ic);
  const double running_count_val = std::max(1.0, count_val - 1.0);
#pragma omp parallel for schedule(static)
  for (int64_t c = 0; c < pc; ++c) {
    const T variance = running_variances[c], mean = running_means[c];
    const T new_mean = (T)(sum_double_var(ic, [&](int64_t i) { return (double)in[o(c, i)]; }) / count_val);
    const double new_var = sum_double_var(ic, [&](int64_t i) {
      const double mean_diff = (double)new_mean - (double)in[o(c, i)];
      return mean_diff * mean_diff;
    });
    batch_means[c] = new_mean;
    batch_variances[c] = (T)(new_var / count_val);
    running_means[c] = (T)((double)mean * ave_lerp + (double)new_mean * (double)ave_factor);
    running_variances[c] =
        (T)((double)variance * ave_lerp + (double)(T)(new_var / running_count_val) * (double)ave_factor);
  }
}

// batch-normalize-gradients-impl (cpu/tensor_math.clj:903-1001).  The scaled
// output gradient is parked, rounded to T, in the input-gradient buffer and
// read back from there (:956-960); `output` and `bias` are not read.
template <class T>
void bn_gradients_t(const BnOffsetter& o, T* input_gradient, T* scale_gradient, T* bias_gradient,
                    const T* output_gradient, const T* in, const T* means, const T* variances, const T* scale,
                    double epsilon_) {
  const T pow_factor = (T)(-3.0 / 2.0);
  const T epsilon = (T)epsilon_;
  const int64_t pc = o.parallel_count(), ic = o.idx_count();
#pragma omp parallel for schedule(static)
  for (int64_t c = 0; c < pc; ++c) {
    const T sc = scale[c];
    const double variance = (double)epsilon + (double)variances[c];
    const double inv_std_dev = 1.0 / std::sqrt(variance);
    const T mean = means[c];
    const T d_var = (T)(-0.5 * std::pow(variance, (double)pow_factor));
    bias_gradient[c] = (T)sum_double_var(ic, [&](int64_t i) { return (double)output_gradient[o(c, i)]; });
    scale_gradient[c] = (T)sum_double_var(ic, [&](int64_t i) {
      const int64_t off = o(c, i);
      return (double)output_gradient[off] * (((double)in[off] - (double)mean) * inv_std_dev);
    });
    for (int64_t i = 0; i < ic; ++i) {
      const int64_t off = o(c, i);
      input_gradient[off] = (T)((double)sc * (double)output_gradient[off]);
    }
    const T d_var_d_out = (T)sum_double_var(ic, [&](int64_t i) {
      const int64_t off = o(c, i);
      return ((double)input_gradient[off] * ((double)in[off] - (double)mean)) * (double)d_var;
    });
    const T d_mean_d_out = (T)(
        sum_double_var(ic, [&](int64_t i) { return (-(double)input_gradient[o(c, i)]) * inv_std_dev; }) +
        (double)d_var_d_out *
            (sum_double_var(ic, [&](int64_t i) { return -2.0 * ((double)in[o(c, i)] - (double)mean); }) /
             (double)ic));
    for (int64_t i = 0; i < ic; ++i) {
      const int64_t off = o(c, i);
      const double d_x_hat_d_out = (double)input_gradient[off];
      const double input_var = (double)in[off];
      const double one_over_index_count = 1.0 / (double)ic;
      const double sum_part_1 = d_x_hat_d_out * inv_std_dev;
      const double sum_part_2 = (((double)d_var_d_out * 2.0) * (input_var - (double)mean)) * one_over_index_count;
      const double sum_part_3 = (double)d_mean_d_out * one_over_index_count;
      input_gradient[off] = (T)((sum_part_1 + sum_part_2) + sum_part_3);
    }
  }
}

// ---------------------------------------------------------------- gemm!, gemv!
// gemm! through col->row-gemm (compute/math_util.clj:17-30) is the row-major
// product C[M, N] = alpha * op(A)[M, K] * op(B)[K, N] + beta * C with row pitches
// ("column strides" in the reference's column-major wording).  BLAS does not
// read C when beta is zero.
template <class T>
void gemm_t(T* c, int64_t ldc, bool ta, bool tb, double alpha, const T* a, int64_t M, int64_t K, int64_t lda,
            const T* b, int64_t N, int64_t ldb, double beta) {
  const T al = (T)alpha, be = (T)beta;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < M; ++i)
    for (int64_t j = 0; j < N; ++j) {
      double acc = 0.0;
      for (int64_t k = 0; k < K; ++k) {
        const double av = (double)(ta ? a[k * lda + i] : a[i * lda + k]);
        const double bv = (double)(tb ? b[j * ldb + k] : b[k * ldb + j]);
        acc += av * bv;
      }
      const double prev = be == (T)0 ? 0.0 : (double)be * (double)c[i * ldc + j];
      c[i * ldc + j] = (T)((double)al * acc + prev);
    }
}

// gemv! through col->row-gemv (compute/math_util.clj:33-41): y = alpha * op(A) x + beta * y for
// the stored row-major A[rows, cols].
template <class T>
void gemv_t(T* y, int64_t incy, bool ta, double alpha, const T* a, int64_t rows, int64_t cols, int64_t lda,
            const T* x, int64_t incx, double beta) {
  const T al = (T)alpha, be = (T)beta;
  const int64_t out_n = ta ? cols : rows, in_n = ta ? rows : cols;
  for (int64_t i = 0; i < out_n; ++i) {
    double acc = 0.0;
    for (int64_t k = 0; k < in_n; ++k) acc += (double)(ta ? a[k * lda + i] : a[i * lda + k]) * (double)x[k * incx];
    const double prev = be == (T)0 ? 0.0 : (double)be * (double)y[i * incy];
    y[i * incy] = (T)((double)al * acc + prev);
  }
}

// ---------------------------------------------------------------- rand!
// Philox4x32-10: ten rounds of two 32x32->64 multiplies, the key bumped by the
// Weyl constants between rounds.
inline void philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
  const uint64_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u;
  uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3], k0 = key[0], k1 = key[1];
  for (int r = 0; r < 10; ++r) {
    const uint64_t p0 = M0 * c0, p1 = M1 * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    c0 = n0; c1 = (uint32_t)p1; c2 = n2; c3 = (uint32_t)p0;
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

// cpu-adam-step-impl! (adam.clj:68-102).  The scalars are cast to the datatype
// first; the arithmetic then runs in double.
template <class T>
void adam_t(double alpha_, double beta1_, double beta2_, double eps_, double pb1_, double pb2_,
            double ga_, const T* g, T* p, T* m, T* v, int64_t n) {
  const double ga = (double)(T)ga_, alpha = (double)(T)alpha_, beta1 = (double)(T)beta1_,
               beta2 = (double)(T)beta2_, eps = (double)(T)eps_, pb1 = (double)(T)pb1_,
               pb2 = (double)(T)pb2_;
  const double one = 1.0, omb1 = one - beta1, omb2 = one - beta2;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    const double gv = ga * (double)g[i];
    const double pv = (double)p[i];
    const double lm = beta1 * (double)m[i] + omb1 * gv;
    const double lv = beta2 * (double)v[i] + (omb2 * gv) * gv;
    const double dx = alpha * (lm / ((one - pb1) * (std::sqrt(lv / (one - pb2)) + eps)));
    m[i] = (T)lm;
    v[i] = (T)lv;
    p[i] = (T)(pv - dx);
  }
}

// AdadeltaOptimizer.microStep (:29-37); single-threaded like the reference.
inline void adadelta_micro(double g, double decay, double eps, double ga_in, double dxa_in,
                           double* ga_out, double* dxa_out, double* dx_out) {
  const double ga = g * g * decay + ga_in * (1.0 - decay);
  const double rms_g = std::sqrt(ga + eps);
  const double rms_dx = std::sqrt(dxa_in + eps);
  const double dx = (-1.0 * rms_dx * g) / rms_g;
  *ga_out = ga;
  *dxa_out = dx * dx * decay + dxa_in * (1.0 - decay);
  *dx_out = dx;
}

// ------------------------------------------------------------------ pooling
// The window walk of src/cortex/nn/impl.clj:8-96 (convolution-outer-kernel with
// convolution-roll-unroll-inner-kernel) over one image, with the six bodies of
// cpu/tensor_math.clj:1153-1284.  Loops and their order are the reference's: the
// backward bodies scatter into the input gradient one tap at a time.

struct PoolGeom {
  int64_t channels, in_h, in_w, out_h, out_w;
  int64_t kw, kh, pad_x, pad_y, stride_x, stride_y;
};

// conv_addr (impl.clj:76-81) is passed to bodies that take six arguments.
template <class Body>
void pool_walk(const PoolGeom& g, Body body) {
  const int64_t min_x = -g.pad_x, min_y = -g.pad_y, max_x = g.in_w + g.pad_x, max_y = g.in_h + g.pad_y;
  for (int64_t chan = 0; chan < g.channels; ++chan) {
    const int64_t chan_in = chan * g.in_w * g.in_h, chan_out = chan * g.out_w * g.out_h;
    for (int64_t out_y = 0; out_y < g.out_h; ++out_y) {
      const int64_t rel_y = out_y * g.stride_y - g.pad_y;
      for (int64_t out_x = 0; out_x < g.out_w; ++out_x) {
        const int64_t rel_x = out_x * g.stride_x - g.pad_x;
        const int64_t over_x = std::max<int64_t>(0, rel_x + g.kw - g.in_w);
        const int64_t over_y = std::max<int64_t>(0, rel_y + g.kh - g.in_h);
        const int64_t under_x = std::min<int64_t>(rel_x, 0), under_y = std::min<int64_t>(rel_y, 0);
        const int64_t exc_w = std::max<int64_t>(0, g.kw - over_x + under_x);
        const int64_t exc_h = std::max<int64_t>(0, g.kh - over_y + under_y);
        const int64_t exc_count = exc_w * exc_h;
        const int64_t out_addr = out_y * g.out_w + out_x + chan_out;
        for (int64_t k_y = 0; k_y < g.kh; ++k_y)
          for (int64_t k_x = 0; k_x < g.kw; ++k_x) {
            const int64_t in_x = rel_x + k_x, in_y = rel_y + k_y;
            const bool input_valid = in_x >= 0 && in_x < g.in_w && in_y >= 0 && in_y < g.in_h;
            const bool loop_valid = in_x >= min_x && in_x < max_x && in_y >= min_y && in_y < max_y;
            if (loop_valid) body(in_y * g.in_w + in_x + chan_in, out_addr, k_y * g.kw + k_x, input_valid, exc_count);
          }
      }
    }
  }
}

template <class T>
void pool_forward_image(T* out, const T* in, const PoolGeom& g, int op) {
  const int64_t kernel_count = g.kw * g.kh;
  if (op == CT_POOL_MAX) {  // :1153-1172
    pool_walk(g, [&](int64_t ia, int64_t oa, int64_t k_idx, bool valid, int64_t) {
      const T v = valid ? in[ia] : (T)0.0;
      if (k_idx == 0 || v > out[oa]) out[oa] = v;
    });
  } else if (op == CT_POOL_AVG) {  // :1198-1219
    pool_walk(g, [&](int64_t ia, int64_t oa, int64_t k_idx, bool valid, int64_t) {
      const T v = valid ? in[ia] : (T)0.0;
      const T prev = k_idx == 0 ? (T)0 : out[oa];
      out[oa] = (T)((double)prev + (double)v / (double)kernel_count);
    });
  } else {  // :avg-exc-pad, :1243-1261 -- adds onto what the output holds
    pool_walk(g, [&](int64_t ia, int64_t oa, int64_t, bool valid, int64_t exc_count) {
      const T v = valid ? in[ia] : (T)0.0;
      out[oa] = (T)((double)out[oa] + (double)v / (double)exc_count);
    });
  }
}

template <class T>
void pool_backward_image(T* ig, const T* in, const T* out, const T* og, const PoolGeom& g, int op) {
  const int64_t kernel_count = g.kw * g.kh;
  if (op == CT_POOL_MAX) {  // :1175-1196
    pool_walk(g, [&](int64_t ia, int64_t oa, int64_t, bool valid, int64_t) {
      if (valid && in[ia] == out[oa]) ig[ia] = (T)((double)ig[ia] + (double)og[oa]);
    });
  } else if (op == CT_POOL_AVG) {  // :1221-1241
    pool_walk(g, [&](int64_t ia, int64_t oa, int64_t, bool valid, int64_t) {
      if (valid) ig[ia] = (T)((double)ig[ia] + (double)og[oa] / (double)kernel_count);
    });
  } else {  // :1263-1284
    pool_walk(g, [&](int64_t ia, int64_t oa, int64_t, bool valid, int64_t exc_count) {
      if (valid) ig[ia] = (T)((double)ig[ia] + (double)og[oa] / (double)exc_count);
    });
  }
}

bool pool_geom(const ct_pool_desc* d, int64_t batch, int64_t channels, int64_t in_h, int64_t in_w, int64_t out_h,
               int64_t out_w, PoolGeom* g) {
  if (!d || batch < 0 || channels < 0 || in_h < 0 || in_w < 0 || out_h < 0 || out_w < 0) return false;
  if (d->kernel_width < 1 || d->kernel_height < 1 || d->stride_x < 1 || d->stride_y < 1 || d->pad_x < 0 ||
      d->pad_y < 0)
    return false;
  if (d->pool_op != CT_POOL_MAX && d->pool_op != CT_POOL_AVG && d->pool_op != CT_POOL_AVG_EXC_PAD) return false;
  *g = PoolGeom{channels, in_h, in_w, out_h, out_w, d->kernel_width, d->kernel_height, d->pad_x, d->pad_y,
                d->stride_x, d->stride_y};
  return true;
}

// ------------------------------------------------------------------ convolution
// planar-input->convolution! and convolution->planar-output!
// (cpu/tensor_math.clj:1118-1151) over one image: the same window walk with
// output-conv-addr = (out_y * out_w + out_x) * (channels * kh * kw) + chan * kh * kw
// + k_y * kw + k_x (impl.clj:54-81).

template <class T>
void unroll_image(const T* in, T* conv, const PoolGeom& g) {
  const int64_t kk = g.kw * g.kh, n_cols = kk * g.channels;
  pool_walk(g, [&](int64_t ia, int64_t oa, int64_t k_idx, bool valid, int64_t) {
    const int64_t chan = oa / (g.out_w * g.out_h), offset = oa % (g.out_w * g.out_h);
    conv[offset * n_cols + chan * kk + k_idx] = valid ? in[ia] : (T)0.0;
  });
}

template <class T>
void roll_image(const T* conv, T* ig, const PoolGeom& g) {
  const int64_t kk = g.kw * g.kh, n_cols = kk * g.channels;
  pool_walk(g, [&](int64_t ia, int64_t oa, int64_t k_idx, bool valid, int64_t) {
    if (!valid) return;
    const int64_t chan = oa / (g.out_w * g.out_h), offset = oa % (g.out_w * g.out_h);
    ig[ia] = (T)((double)conv[offset * n_cols + chan * kk + k_idx] + (double)ig[ia]);
  });
}

bool conv_geom(const ct_conv_desc* d, int64_t batch, int64_t in_h, int64_t in_w, int64_t out_h, int64_t out_w,
               PoolGeom* g) {
  if (!d || batch < 0 || in_h < 0 || in_w < 0 || out_h < 0 || out_w < 0) return false;
  if (d->in_channels < 1 || d->out_channels < 1 || d->kernel_width < 1 || d->kernel_height < 1 ||
      d->stride_x < 1 || d->stride_y < 1 || d->pad_x < 0 || d->pad_y < 0)
    return false;
  *g = PoolGeom{d->in_channels, in_h, in_w, out_h, out_w, d->kernel_width, d->kernel_height, d->pad_x, d->pad_y,
                d->stride_x, d->stride_y};
  return true;
}

template <class T>
int convolution_t(int which, T* dest, double alpha, const T* other, const T* weights, T* workspace,
                  int64_t workspace_ecount, const ct_conv_desc* d, int64_t batch, const PoolGeom& g) {
  const int64_t n_rows = g.out_h * g.out_w, n_cols = g.kw * g.kh * g.channels, out_ch = d->out_channels;
  const int64_t in_img = g.channels * g.in_h * g.in_w, out_img = out_ch * n_rows, conv_img = n_rows * n_cols;
  if (workspace_ecount < batch * conv_img) return fail("convolution: workspace too small");
  if (which == 0) {  // forward (:1682-1714): dest = output, other = input
    for (int64_t b = 0; b < batch; ++b) {
      unroll_image(other + b * in_img, workspace + b * conv_img, g);
      gemm_t<T>(dest + b * out_img, n_rows, false, true, 1.0, weights, out_ch, n_cols, n_cols, workspace + b * conv_img,
                n_rows, n_cols, alpha);
    }
  } else if (which == 1) {  // backward-weights (:1716-1747): dest = weight gradient, other = output gradient
    for (int64_t b = 0; b < batch; ++b)
      gemm_t<T>(dest, n_cols, false, false, 1.0, other + b * out_img, out_ch, n_rows, n_rows, workspace + b * conv_img,
                n_cols, n_cols, b == 0 ? alpha : 1.0);
  } else {  // backward-data (:1749-1792): dest = input gradient, other = output gradient
    for (int64_t i = 0; i < batch * in_img; ++i) dest[i] = (T)0;
    for (int64_t b = 0; b < batch; ++b) {
      gemm_t<T>(workspace + b * conv_img, n_cols, true, false, 1.0, other + b * out_img, n_rows, out_ch, n_rows, weights,
                n_cols, n_cols, 0.0);
      roll_image(workspace + b * conv_img, dest + b * in_img, g);
    }
  }
  return 0;
}

}  // namespace

// ------------------------------------------------------------------ C entry points
// Same argument lists as the library's entry points in include/cortex_hip.h
// minus the stream; pointers are host pointers.

// ------------------------------------------------------------------ local response normalization
// lrn-forward! / lrn-backward! (tensor/math.clj:240-252; tensor.clj:1554-1616).  The reference has
// no CPU form: its only implementation hands the tensors to cuDNN's cross-channel LRN
// (cuda/tensor_math.clj:271-281, 1277-1335: cudnnLRNCrossChannelForward / Backward, mode
// CUDNN_LRN_CROSS_CHANNEL_DIM1, through org.bytedeco.javacpp-presets/cuda 8.0-1.2, project.clj:12),
// a closed library that is not under /root/reference.  What is restated here is that routine's
// published definition (cuDNN library guide, cudnnSetLRNDescriptor / cudnnLRNCrossChannelForward;
// the operator of Krizhevsky, Sutskever, Hinton 2012, section 3.3):
//   window(c) = [c - floor((n-1)/2), c + n - 1 - floor((n-1)/2)], clipped to the channels
//   s[c]      = k + (alpha / n) * sum over window(c) of x^2
//   y[c]      = x[c] * s[c]^-beta
//   dx[c]     = dy[c] * s[c]^-beta
//               - (2 alpha beta / n) * x[c] * sum over window(c) of dy[c'] y[c'] / s[c']
// evaluated in double and rounded once.  The backward sum runs over window(c) itself: for an even n,
// whose window is not centred, the exact derivative would run over the mirrored window, and the
// stored results for n = 2 below are those of the unmirrored one.  Tensors are [batch, channels, height, width] with any
// strides; a rank-3 tensor is one image (cuda/driver.clj:1094-1123 pads shapes to four entries).
// Pinned by the stored vectors of src/cortex/verify/tensor.clj:1088-1140 (n = 1, 2, 3 with
// k = alpha = beta = 1; they fix the window's placement in both directions and both formulas) and,
// for the other parameters, by central differences of the forward pass for odd n, where the
// backward pass is the exact derivative (tests/test_oracle_closed_forms.py).
struct LrnView {
  int64_t size[4], stride[4];
};

bool lrn_view(const Dims& d, LrnView* v) {
  if (d.nd < 3 || d.nd > 4 || !direct(d)) return false;
  for (int i = 0; i < 4; ++i) { v->size[i] = 1; v->stride[i] = 0; }
  for (int i = 0; i < d.nd; ++i) {
    v->size[i + 4 - d.nd] = d.shape[i];
    v->stride[i + 4 - d.nd] = d.strides[i];
  }
  return true;
}

bool lrn_same_shape(const LrnView& a, const LrnView& b) {
  for (int i = 0; i < 4; ++i)
    if (a.size[i] != b.size[i]) return false;
  return true;
}

inline int64_t lrn_at(const LrnView& v, int64_t b, int64_t c, int64_t y, int64_t x) {
  return b * v.stride[0] + c * v.stride[1] + y * v.stride[2] + x * v.stride[3];
}

template <class T>
double lrn_scale(const T* in, const LrnView& iv, int64_t b, int64_t c, int64_t y, int64_t x, int n, double k, double alpha) {
  const int64_t behind = (n - 1) / 2, ahead = n - 1 - behind;
  double sum = 0.0;
  for (int64_t w = std::max<int64_t>(0, c - behind); w <= std::min<int64_t>(iv.size[1] - 1, c + ahead); ++w) {
    const double v = (double)in[lrn_at(iv, b, w, y, x)];
    sum += v * v;
  }
  return k + (alpha / (double)n) * sum;
}

template <class T>
int lrn_forward_t(T* out, const LrnView& ov, const T* in, const LrnView& iv, int n, double k, double alpha, double beta) {
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t b = 0; b < iv.size[0]; ++b)
    for (int64_t c = 0; c < iv.size[1]; ++c)
      for (int64_t y = 0; y < iv.size[2]; ++y)
        for (int64_t x = 0; x < iv.size[3]; ++x) {
          const double s = lrn_scale(in, iv, b, c, y, x, n, k, alpha);
          out[lrn_at(ov, b, c, y, x)] = (T)((double)in[lrn_at(iv, b, c, y, x)] * std::pow(s, -beta));
        }
  return 0;
}

template <class T>
int lrn_backward_t(T* ig, const LrnView& gv, const T* out, const LrnView& ov, const T* in, const LrnView& iv, const T* og,
                   const LrnView& dv, int n, double k, double alpha, double beta) {
  const int64_t behind = (n - 1) / 2, ahead = n - 1 - behind;
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t b = 0; b < iv.size[0]; ++b)
    for (int64_t c = 0; c < iv.size[1]; ++c)
      for (int64_t y = 0; y < iv.size[2]; ++y)
        for (int64_t x = 0; x < iv.size[3]; ++x) {
          double cross = 0.0;
          for (int64_t w = std::max<int64_t>(0, c - behind); w <= std::min<int64_t>(iv.size[1] - 1, c + ahead); ++w)
            cross += (double)og[lrn_at(dv, b, w, y, x)] * (double)out[lrn_at(ov, b, w, y, x)] /
                     lrn_scale(in, iv, b, w, y, x, n, k, alpha);
          const double s = lrn_scale(in, iv, b, c, y, x, n, k, alpha);
          const double direct_term = (double)og[lrn_at(dv, b, c, y, x)] * std::pow(s, -beta);
          ig[lrn_at(gv, b, c, y, x)] =
              (T)(direct_term - (2.0 * alpha * beta / (double)n) * (double)in[lrn_at(iv, b, c, y, x)] * cross);
        }
  return 0;
}

bool lrn_params_ok(int n, double k, double alpha, double beta) {
  return n >= 1 && n <= 16 && k > 0.0 && std::isfinite(alpha) && std::isfinite(beta);
}

#define LOAD(name, src)        \
  Dims name;                   \
  if (!load_dims(src, &name)) return fail("bad dimensions: " #src)

extern "C" {

const char* co_last_error(void) { return g_err; }

int co_memset(void* buffer, int dtype, double value, int64_t n) {
  DISPATCH_DTYPE(dtype, { T* b = (T*)buffer; const T v = jcast<T>(value); for (int64_t i = 0; i < n; ++i) b[i] = v; });
  return 0;
}

int co_assign_constant(void* dest, const ct_dims* dest_dims, int dtype, double value, int64_t n) {
  LOAD(dd, dest_dims);
  DISPATCH_DTYPE(dtype, return assign_constant_t<T>((T*)dest, dd, value, n));
  return 0;
}

int co_assign(void* dest, const ct_dims* dest_dims, int dest_dtype, const void* src,
              const ct_dims* src_dims, int src_dtype, int64_t n) {
  LOAD(dd, dest_dims);
  LOAD(sd, src_dims);
#define INNER(S) DISPATCH_DTYPE(dest_dtype, return (assign_t<T, S>((T*)dest, dd, (const S*)src, sd, n)))
  switch (src_dtype) {
    case CT_I8: INNER(int8_t); break;
    case CT_I16: INNER(int16_t); break;
    case CT_I32: INNER(int32_t); break;
    case CT_I64: INNER(int64_t); break;
    case CT_F32: INNER(float); break;
    case CT_F64: INNER(double); break;
    case CT_U8: INNER(uint8_t); break;
    default: return fail("unknown source datatype");
  }
#undef INNER
  return 0;
}

int co_unary_accum(void* dest, const ct_dims* dest_dims, double alpha, int op, int dtype, int64_t n) {
  LOAD(dd, dest_dims);
  if (op < 0 || op > CT_UOP_NOOP) return fail("unknown unary op");
  DISPATCH_DTYPE(dtype, return unary_t<T>((T*)dest, dd, nullptr, nullptr, alpha, op, n));
  return 0;
}

int co_unary_op(void* dest, const ct_dims* dest_dims, const void* x, const ct_dims* x_dims,
                double alpha, int op, int dtype, int64_t n) {
  LOAD(dd, dest_dims);
  LOAD(xd, x_dims);
  if (op < 0 || op > CT_UOP_NOOP) return fail("unknown unary op");
  DISPATCH_DTYPE(dtype, return unary_t<T>((T*)dest, dd, (const T*)x, &xd, alpha, op, n));
  return 0;
}

int co_binary_accum_constant(void* dest, const ct_dims* dest_dims, double dest_alpha, double scalar,
                             int64_t n, int op, int reverse_operands, int dtype) {
  LOAD(dd, dest_dims);
  if (op < 0 || op > CT_BOP_LE) return fail("unknown binary op");
  DISPATCH_DTYPE(dtype, return binary_t<T>((T*)dest, dd, nullptr, nullptr, dest_alpha, nullptr, nullptr,
                                          0.0, scalar, n, op, reverse_operands != 0));
  return 0;
}

int co_binary_op_constant(void* dest, const ct_dims* dest_dims, const void* x, const ct_dims* x_dims,
                          double x_alpha, double scalar, int64_t n, int op, int reverse_operands,
                          int dtype) {
  LOAD(dd, dest_dims);
  LOAD(xd, x_dims);
  if (op < 0 || op > CT_BOP_LE) return fail("unknown binary op");
  DISPATCH_DTYPE(dtype, return binary_t<T>((T*)dest, dd, (const T*)x, &xd, x_alpha, nullptr, nullptr, 0.0,
                                          scalar, n, op, reverse_operands != 0));
  return 0;
}

int co_binary_op(void* dest, const ct_dims* dest_dims, const void* x, const ct_dims* x_dims,
                 double x_alpha, const void* y, const ct_dims* y_dims, double y_alpha, int64_t n,
                 int op, int dtype);

int co_binary_accum(void* dest, const ct_dims* dest_dims, double dest_alpha, const void* y,
                    const ct_dims* y_dims, double y_alpha, int64_t n, int op, int reverse_operands,
                    int dest_requires_cas, int dtype) {
  if (!dest_requires_cas) {  // cpu/tensor_math.clj:1451-1463: re-enter binary-op!
    return reverse_operands
               ? co_binary_op(dest, dest_dims, y, y_dims, y_alpha, dest, dest_dims, dest_alpha, n, op, dtype)
               : co_binary_op(dest, dest_dims, dest, dest_dims, dest_alpha, y, y_dims, y_alpha, n, op, dtype);
  }
  LOAD(dd, dest_dims);
  LOAD(yd, y_dims);
  if (op < 0 || op > CT_BOP_LE) return fail("unknown binary op");
  DISPATCH_DTYPE(dtype, return binary_t<T>((T*)dest, dd, nullptr, nullptr, dest_alpha, (const T*)y, &yd,
                                          y_alpha, 0.0, n, op, reverse_operands != 0));
  return 0;
}

int co_binary_op(void* dest, const ct_dims* dest_dims, const void* x, const ct_dims* x_dims,
                 double x_alpha, const void* y, const ct_dims* y_dims, double y_alpha, int64_t n,
                 int op, int dtype) {
  LOAD(dd, dest_dims);
  LOAD(xd, x_dims);
  LOAD(yd, y_dims);
  if (op < 0 || op > CT_BOP_LE) return fail("unknown binary op");
  DISPATCH_DTYPE(dtype, return binary_t<T>((T*)dest, dd, (const T*)x, &xd, x_alpha, (const T*)y, &yd,
                                          y_alpha, 0.0, n, op, false));
  return 0;
}

int co_ternary_op(void* dest, const ct_dims* dest_dims, const void* x, const ct_dims* x_dims,
                  double x_alpha, const void* y, const ct_dims* y_dims, double y_alpha, const void* z,
                  const ct_dims* z_dims, double z_alpha, int64_t n, int op, int dtype) {
  LOAD(dd, dest_dims);
  LOAD(xd, x_dims);
  LOAD(yd, y_dims);
  LOAD(zd, z_dims);
  if (op != CT_TOP_SELECT) return fail("unknown ternary op");
  const Dims* td[3] = {&xd, &yd, &zd};
  const double al[3] = {x_alpha, y_alpha, z_alpha};
  DISPATCH_DTYPE(dtype, {
    const T* t[3] = {(const T*)x, (const T*)y, (const T*)z};
    return ternary_t<T>((T*)dest, dd, t, td, al, 3, nullptr, nullptr, n);
  });
  return 0;
}

static bool valid_arg_idx(const int8_t* a) {
  if (!a) return false;
  int seen = 0;
  for (int k = 0; k < 3; ++k) {
    if (a[k] < 0 || a[k] > 2) return false;
    seen |= 1 << a[k];
  }
  return seen == 7;
}

int co_ternary_op_constant(void* dest, const ct_dims* dest_dims, const void* a, const ct_dims* a_dims,
                           double a_alpha, const void* b, const ct_dims* b_dims, double b_alpha,
                           double constant, int64_t n, int op, const int8_t arg_idx[3], int dtype) {
  LOAD(dd, dest_dims);
  LOAD(ad, a_dims);
  LOAD(bd, b_dims);
  if (op != CT_TOP_SELECT) return fail("unknown ternary op");
  if (!valid_arg_idx(arg_idx)) return fail("arg_idx must be a permutation of 0,1,2");
  const Dims* td[2] = {&ad, &bd};
  const double al[2] = {a_alpha, b_alpha};
  const double cs[1] = {constant};
  DISPATCH_DTYPE(dtype, {
    const T* t[2] = {(const T*)a, (const T*)b};
    return ternary_t<T>((T*)dest, dd, t, td, al, 2, cs, arg_idx, n);
  });
  return 0;
}

int co_ternary_op_constant_constant(void* dest, const ct_dims* dest_dims, const void* a,
                                    const ct_dims* a_dims, double a_alpha, double const_1,
                                    double const_2, int64_t n, int op, const int8_t arg_idx[3],
                                    int dtype) {
  LOAD(dd, dest_dims);
  LOAD(ad, a_dims);
  if (op != CT_TOP_SELECT) return fail("unknown ternary op");
  if (!valid_arg_idx(arg_idx)) return fail("arg_idx must be a permutation of 0,1,2");
  const Dims* td[1] = {&ad};
  const double al[1] = {a_alpha};
  const double cs[2] = {const_1, const_2};
  DISPATCH_DTYPE(dtype, {
    const T* t[1] = {(const T*)a};
    return ternary_t<T>((T*)dest, dd, t, td, al, 1, cs, arg_idx, n);
  });
  return 0;
}

int co_unary_reduce(void* output, const ct_dims* output_dims, double input_alpha, const void* input,
                    const ct_dims* input_dims, int op, int dtype) {
  LOAD(od, output_dims);
  LOAD(id, input_dims);
  if (op < 0 || op > CT_ROP_MAGNITUDE_SQUARED) return fail("unknown reduction op");
  DISPATCH_DTYPE(dtype, return reduce_t<T>((T*)output, od, input_alpha, (const T*)input, id, op));
  return 0;
}

int co_activation_gradient(void* input_gradient, const ct_dims* input_gradient_dims, const void* output_gradient,
                           const ct_dims* output_gradient_dims, const void* output, const ct_dims* output_dims,
                           int op, int64_t n, int dtype) {
  LOAD(igd, input_gradient_dims);
  LOAD(ogd, output_gradient_dims);
  LOAD(od, output_dims);
  if (op < CT_ACT_LOGISTIC || op > CT_ACT_RELU) return fail("Only :logistic :tanh and :relu are supported");
  if (dtype == CT_F32)
    return activation_gradient_t<float>((float*)input_gradient, igd, (const float*)output_gradient, ogd,
                                        (const float*)output, od, op, n);
  if (dtype == CT_F64)
    return activation_gradient_t<double>((double*)input_gradient, igd, (const double*)output_gradient, ogd,
                                         (const double*)output, od, op, n);
  return fail("activation-gradient! is only defined for float and double tensors");
}

int co_softmax_eltwise(void* output, const ct_dims* output_dims, const void* input, const ct_dims* input_dims,
                       int dtype) {
  LOAD(od, output_dims);
  LOAD(id, input_dims);
  if (dtype == CT_F32) return softmax_t<float>((float*)output, od, (const float*)input, id);
  if (dtype == CT_F64) return softmax_t<double>((double*)output, od, (const double*)input, id);
  return fail("softmax! is only defined for float and double tensors");
}

int co_softmax_spatial(void* output, const ct_dims* output_dims, const void* input, const ct_dims* input_dims,
                       int dtype) {
  LOAD(od, output_dims);
  LOAD(id, input_dims);
  Dims odt, idt;
  if (!transpose_021(od, &odt) || !transpose_021(id, &idt)) return fail("softmax-spatial! needs [batch channels elements]");
  if (dtype == CT_F32) return softmax_t<float>((float*)output, odt, (const float*)input, idt);
  if (dtype == CT_F64) return softmax_t<double>((double*)output, odt, (const double*)input, idt);
  return fail("softmax! is only defined for float and double tensors");
}

static bool bn_counts_ok(int64_t b, int64_t c, int64_t e) { return b >= 1 && c >= 1 && e >= 1; }

#define BN_FLOAT_DISPATCH(dtype, ...)                                               \
  if ((dtype) == CT_F32) { using T = float; __VA_ARGS__; }                          \
  else if ((dtype) == CT_F64) { using T = double; __VA_ARGS__; }                    \
  else return fail("batch-normalization is only defined for float and double tensors")

// batch-normalize-spatial! (cpu/tensor_math.clj:1566-1572); the eltwise form
// (:1558-1564) is the same with one element per channel.
int co_batch_normalize_spatial(void* output, const void* input, const void* means, const void* variances,
                               const void* scale, const void* bias, double epsilon, int64_t batch_count,
                               int64_t channel_count, int64_t element_count, int dtype) {
  if (!bn_counts_ok(batch_count, channel_count, element_count)) return fail("batch-normalize: counts must be positive");
  const BnOffsetter o{batch_count, channel_count, element_count};
  BN_FLOAT_DISPATCH(dtype, bn_apply_t<T>(o, (T*)output, (const T*)input, (const T*)means, (const T*)variances,
                                         (const T*)scale, (const T*)bias, epsilon));
  return 0;
}

int co_batch_normalize_eltwise(void* output, const void* input, const void* means, const void* variances,
                               const void* scale, const void* bias, double epsilon, int64_t batch_count,
                               int64_t element_count, int dtype) {
  return co_batch_normalize_spatial(output, input, means, variances, scale, bias, epsilon, batch_count,
                                    element_count, 1, dtype);
}

// batch-normalize-update-and-apply-spatial! (cpu/tensor_math.clj:1592-1608):
// the update, then the plain normalization with the batch statistics.
int co_batch_normalize_update_and_apply_spatial(void* output, const void* input, void* batch_means,
                                                void* batch_variances, void* running_means,
                                                void* running_variances, double average_factor, const void* scale,
                                                const void* bias, double epsilon, int64_t batch_count,
                                                int64_t channel_count, int64_t element_count, int dtype) {
  if (!bn_counts_ok(batch_count, channel_count, element_count)) return fail("batch-normalize: counts must be positive");
  const BnOffsetter o{batch_count, channel_count, element_count};
  BN_FLOAT_DISPATCH(dtype, {
    bn_update_t<T>(o, (const T*)input, (T*)batch_means, (T*)batch_variances, (T*)running_means,
                   (T*)running_variances, average_factor);
    bn_apply_t<T>(o, (T*)output, (const T*)input, (const T*)batch_means, (const T*)batch_variances,
                  (const T*)scale, (const T*)bias, epsilon);
  });
  return 0;
}

int co_batch_normalize_update_and_apply_eltwise(void* output, const void* input, void* batch_means,
                                                void* batch_variances, void* running_means,
                                                void* running_variances, double average_factor, const void* scale,
                                                const void* bias, double epsilon, int64_t batch_count,
                                                int64_t element_count, int dtype) {
  return co_batch_normalize_update_and_apply_spatial(output, input, batch_means, batch_variances, running_means,
                                                     running_variances, average_factor, scale, bias, epsilon,
                                                     batch_count, element_count, 1, dtype);
}

// batch-normalize-gradients-spatial! (cpu/tensor_math.clj:1624-1638)
int co_batch_normalize_gradients_spatial(void* input_gradient, void* scale_gradient, void* bias_gradient,
                                         const void* output_gradient, const void* output, const void* input,
                                         const void* batch_means, const void* batch_variances, const void* scale,
                                         const void* bias, double epsilon, int64_t batch_count,
                                         int64_t channel_count, int64_t element_count, int dtype) {
  (void)output;
  (void)bias;
  if (!bn_counts_ok(batch_count, channel_count, element_count)) return fail("batch-normalize: counts must be positive");
  const BnOffsetter o{batch_count, channel_count, element_count};
  BN_FLOAT_DISPATCH(dtype, bn_gradients_t<T>(o, (T*)input_gradient, (T*)scale_gradient, (T*)bias_gradient,
                                             (const T*)output_gradient, (const T*)input, (const T*)batch_means,
                                             (const T*)batch_variances, (const T*)scale, epsilon));
  return 0;
}

int co_batch_normalize_gradients_eltwise(void* input_gradient, void* scale_gradient, void* bias_gradient,
                                         const void* output_gradient, const void* output, const void* input,
                                         const void* batch_means, const void* batch_variances, const void* scale,
                                         const void* bias, double epsilon, int64_t batch_count,
                                         int64_t element_count, int dtype) {
  return co_batch_normalize_gradients_spatial(input_gradient, scale_gradient, bias_gradient, output_gradient, output,
                                              input, batch_means, batch_variances, scale, bias, epsilon, batch_count,
                                              element_count, 1, dtype);
}

int co_gemm(void* c, int64_t c_colstride, int trans_a, int trans_b, double alpha, const void* a, int64_t a_row_count,
            int64_t a_col_count, int64_t a_colstride, const void* b, int64_t b_col_count, int64_t b_colstride,
            double beta, int dtype) {
  if (dtype == CT_F32)
    gemm_t<float>((float*)c, c_colstride, trans_a != 0, trans_b != 0, alpha, (const float*)a, a_row_count, a_col_count,
                  a_colstride, (const float*)b, b_col_count, b_colstride, beta);
  else if (dtype == CT_F64)
    gemm_t<double>((double*)c, c_colstride, trans_a != 0, trans_b != 0, alpha, (const double*)a, a_row_count,
                   a_col_count, a_colstride, (const double*)b, b_col_count, b_colstride, beta);
  else
    return fail("gemm! is only defined for float and double tensors");
  return 0;
}

int co_gemv(void* c, int64_t inc_c, int trans_a, double alpha, const void* a, int64_t a_row_count,
            int64_t a_col_count, int64_t a_colstride, const void* x, int64_t inc_x, double beta, int dtype) {
  if (dtype == CT_F32)
    gemv_t<float>((float*)c, inc_c, trans_a != 0, alpha, (const float*)a, a_row_count, a_col_count, a_colstride,
                  (const float*)x, inc_x, beta);
  else if (dtype == CT_F64)
    gemv_t<double>((double*)c, inc_c, trans_a != 0, alpha, (const double*)a, a_row_count, a_col_count, a_colstride,
                   (const double*)x, inc_x, beta);
  else
    return fail("gemv! is only defined for float and double tensors");
  return 0;
}

// The library's rand!: value k of the stream (seed, offset) is word k % 4 of
// the Philox block with counter (k / 4, offset) and key seed.  The arithmetic
// around the draw follows cpu/tensor_math.clj:1873-1887: float parameters,
// double arithmetic, one rounding at the store.
int co_rand(void* dest, int64_t n, int dtype, int distribution, double a, double b, uint64_t seed,
            uint64_t offset) {
  if (dtype != CT_F32) return fail("Can only generate rands into floating point buffers");
  if (n < 0) return fail("negative count");
  float* d = (float*)dest;
  const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  const float inv24 = 5.9604644775390625e-08f, two_pi = 6.28318530717958647692f;
  double p0, p1;
  if (distribution == CT_DIST_FLAT) {
    const float minimum = (float)a, maximum = (float)b;
    if (!(minimum < maximum)) return fail("Minimum must be less than maximum");
    p0 = (double)minimum;
    p1 = (double)maximum - (double)minimum;
  } else if (distribution == CT_DIST_GAUSSIAN) {
    if (!((float)b >= 0.0f)) return fail("negative variance");
    p0 = (double)(float)a;
    p1 = std::sqrt((double)(float)b);
  } else {
    return fail("Unrecognized distribution");
  }
  for (int64_t i = 0; i * 4 < n; ++i) {
    const uint32_t ctr[4] = {(uint32_t)i, (uint32_t)((uint64_t)i >> 32), (uint32_t)offset, (uint32_t)(offset >> 32)};
    uint32_t r[4];
    float v[4];
    philox4x32_10(ctr, key, r);
    if (distribution == CT_DIST_FLAT) {
      for (int e = 0; e < 4; ++e) {
        const float u = (float)(r[e] >> 8) * inv24;
        v[e] = (float)(p0 + (double)u * p1);
      }
    } else {
      for (int h = 0; h < 2; ++h) {
        const float u1 = (float)((r[2 * h] >> 8) + 1u) * inv24;
        const float u2 = (float)(r[2 * h + 1] >> 8) * inv24;
        const float rad = std::sqrt(-2.0f * std::log(u1));
        const float ang = two_pi * u2;
        v[2 * h] = (float)(p1 * (double)(rad * std::cos(ang)) + p0);
        v[2 * h + 1] = (float)(p1 * (double)(rad * std::sin(ang)) + p0);
      }
    }
    for (int e = 0; e < 4 && i * 4 + e < n; ++e) d[i * 4 + e] = v[e];
  }
  return 0;
}

// pooling-forward! / pooling-backward! (cpu/tensor_math.clj:1800-1866): the
// images of the batch are independent (the reference maps them with pmap); the
// alphas are not read there and are not taken here.
int co_pooling_forward(void* output, double, const void* input, const ct_pool_desc* desc, int64_t batch_count,
                       int64_t channel_count, int64_t in_height, int64_t in_width, int64_t out_height,
                       int64_t out_width, int dtype) {
  PoolGeom g;
  if (!pool_geom(desc, batch_count, channel_count, in_height, in_width, out_height, out_width, &g))
    return fail("pooling: bad descriptor or counts");
  if (dtype != CT_F32 && dtype != CT_F64) return fail("Failed to find cpu pooling op");
  const int64_t in_img = channel_count * in_height * in_width, out_img = channel_count * out_height * out_width;
#pragma omp parallel for schedule(static)
  for (int64_t b = 0; b < batch_count; ++b) {
    if (dtype == CT_F32) pool_forward_image((float*)output + b * out_img, (const float*)input + b * in_img, g, desc->pool_op);
    else pool_forward_image((double*)output + b * out_img, (const double*)input + b * in_img, g, desc->pool_op);
  }
  return 0;
}

int co_pooling_backward(void* input_gradient, double, const void* input, const void* output,
                        const void* output_gradient, const ct_pool_desc* desc, int64_t batch_count,
                        int64_t channel_count, int64_t in_height, int64_t in_width, int64_t out_height,
                        int64_t out_width, int dtype) {
  PoolGeom g;
  if (!pool_geom(desc, batch_count, channel_count, in_height, in_width, out_height, out_width, &g))
    return fail("pooling: bad descriptor or counts");
  if (dtype != CT_F32 && dtype != CT_F64) return fail("Failed to find cpu pooling op");
  const int64_t in_img = channel_count * in_height * in_width, out_img = channel_count * out_height * out_width;
#pragma omp parallel for schedule(static)
  for (int64_t b = 0; b < batch_count; ++b) {
    if (dtype == CT_F32)
      pool_backward_image((float*)input_gradient + b * in_img, (const float*)input + b * in_img,
                          (const float*)output + b * out_img, (const float*)output_gradient + b * out_img, g,
                          desc->pool_op);
    else
      pool_backward_image((double*)input_gradient + b * in_img, (const double*)input + b * in_img,
                          (const double*)output + b * out_img, (const double*)output_gradient + b * out_img, g,
                          desc->pool_op);
  }
  return 0;
}

#define CONV_ENTRY(which, dest, alpha, other, weights)                                                                  \
  PoolGeom g;                                                                                                           \
  if (!conv_geom(desc, batch_count, in_height, in_width, out_height, out_width, &g))                                    \
    return fail("convolution: bad descriptor or counts");                                                              \
  if (dtype == CT_F32)                                                                                                  \
    return convolution_t<float>(which, (float*)dest, alpha, (const float*)other, (const float*)weights,                 \
                                (float*)workspace, workspace_ecount, desc, batch_count, g);                            \
  if (dtype == CT_F64)                                                                                                  \
    return convolution_t<double>(which, (double*)dest, alpha, (const double*)other, (const double*)weights,             \
                                 (double*)workspace, workspace_ecount, desc, batch_count, g);                          \
  return fail("convolution is only defined for float and double tensors")

int co_convolution_forward(void* output, double output_alpha, const void* input, const void* weights, void* workspace,
                           int64_t workspace_ecount, const ct_conv_desc* desc, int64_t batch_count, int64_t in_height,
                           int64_t in_width, int64_t out_height, int64_t out_width, int dtype) {
  CONV_ENTRY(0, output, output_alpha, input, weights);
}

int co_convolution_backward_weights(void* weight_gradient, double weight_gradient_alpha, const void* output_gradient,
                                    const void*, void* workspace, int64_t workspace_ecount, const ct_conv_desc* desc,
                                    int64_t batch_count, int64_t in_height, int64_t in_width, int64_t out_height,
                                    int64_t out_width, int dtype) {
  CONV_ENTRY(1, weight_gradient, weight_gradient_alpha, output_gradient, nullptr);
}

int co_convolution_backward_data(void* input_gradient, double, const void* output_gradient, const void* weights,
                                 void* workspace, int64_t workspace_ecount, const ct_conv_desc* desc,
                                 int64_t batch_count, int64_t in_height, int64_t in_width, int64_t out_height,
                                 int64_t out_width, int dtype) {
  CONV_ENTRY(2, input_gradient, 0.0, output_gradient, weights);
}

int co_lrn_forward(void* output, const ct_dims* output_dims, const void* input, const ct_dims* input_dims, int n, double k,
                   double alpha, double beta, int dtype) {
  LOAD(od, output_dims);
  LOAD(id, input_dims);
  LrnView ov, iv;
  if (!lrn_view(od, &ov) || !lrn_view(id, &iv)) return fail("lrn: tensor must be of rank 3 or 4 with direct dimensions");
  if (!lrn_same_shape(ov, iv)) return fail("lrn: Input and output shapes must match");
  if (!lrn_params_ok(n, k, alpha, beta)) return fail("lrn: bad descriptor");
  if (dtype == CT_F32) return lrn_forward_t<float>((float*)output, ov, (const float*)input, iv, n, k, alpha, beta);
  if (dtype == CT_F64) return lrn_forward_t<double>((double*)output, ov, (const double*)input, iv, n, k, alpha, beta);
  return fail("lrn-forward is only defined for float and double tensors");
}

int co_lrn_backward(void* input_gradient, const ct_dims* input_gradient_dims, const void* output, const ct_dims* output_dims,
                    const void* input, const ct_dims* input_dims, const void* output_gradient,
                    const ct_dims* output_gradient_dims, int n, double k, double alpha, double beta, int dtype) {
  LOAD(gd, input_gradient_dims);
  LOAD(od, output_dims);
  LOAD(id, input_dims);
  LOAD(dd, output_gradient_dims);
  LrnView gv, ov, iv, dv;
  if (!lrn_view(gd, &gv) || !lrn_view(od, &ov) || !lrn_view(id, &iv) || !lrn_view(dd, &dv))
    return fail("lrn: tensor must be of rank 3 or 4 with direct dimensions");
  if (!lrn_same_shape(gv, iv) || !lrn_same_shape(ov, iv) || !lrn_same_shape(dv, iv))
    return fail("lrn: Input and output shapes must match");
  if (!lrn_params_ok(n, k, alpha, beta)) return fail("lrn: bad descriptor");
  if (dtype == CT_F32)
    return lrn_backward_t<float>((float*)input_gradient, gv, (const float*)output, ov, (const float*)input, iv,
                                 (const float*)output_gradient, dv, n, k, alpha, beta);
  if (dtype == CT_F64)
    return lrn_backward_t<double>((double*)input_gradient, gv, (const double*)output, ov, (const double*)input, iv,
                                  (const double*)output_gradient, dv, n, k, alpha, beta);
  return fail("lrn-backward is only defined for float and double tensors");
}

// One Philox4x32-10 block, for the known-answer tests.
int co_philox4x32_10(const uint32_t* counter, const uint32_t* key, uint32_t* out) {
  philox4x32_10(counter, key, out);
  return 0;
}

int co_adam_step(int dtype, double alpha, double beta1, double beta2, double epsilon,
                 double pow_beta1_t, double pow_beta2_t, double gradient_alpha, const void* gradient,
                 void* parameters, void* m, void* v, int64_t n) {
  if (dtype == CT_F32)
    adam_t<float>(alpha, beta1, beta2, epsilon, pow_beta1_t, pow_beta2_t, gradient_alpha,
                  (const float*)gradient, (float*)parameters, (float*)m, (float*)v, n);
  else if (dtype == CT_F64)
    adam_t<double>(alpha, beta1, beta2, epsilon, pow_beta1_t, pow_beta2_t, gradient_alpha,
                   (const double*)gradient, (double*)parameters, (double*)m, (double*)v, n);
  else
    return fail("adam: datatype must be float or double");
  return 0;
}

// AdadeltaOptimizer.step_f / step_d (:39-64)
int co_adadelta_step(int dtype, double decay, double epsilon, void* grad_sq_accum, void* dx_sq_accum,
                     double gradient_alpha, const void* gradient, void* parameters, int64_t n) {
  if (dtype == CT_F32) {
    const float ga = (float)gradient_alpha, dc = (float)decay, ep = (float)epsilon;
    const float* g = (const float*)gradient;
    float *p = (float*)parameters, *gacc = (float*)grad_sq_accum, *dacc = (float*)dx_sq_accum;
    for (int64_t i = 0; i < n; ++i) {
      const double grad = (double)(float)(ga * g[i]);  // float product, then widened
      double a, b, dx;
      adadelta_micro(grad, (double)dc, (double)ep, (double)gacc[i], (double)dacc[i], &a, &b, &dx);
      gacc[i] = (float)a;
      dacc[i] = (float)b;
      p[i] = (float)(p[i] + (float)dx);  // float += float
    }
  } else if (dtype == CT_F64) {
    const double* g = (const double*)gradient;
    double *p = (double*)parameters, *gacc = (double*)grad_sq_accum, *dacc = (double*)dx_sq_accum;
    for (int64_t i = 0; i < n; ++i) {
      double a, b, dx;
      adadelta_micro(gradient_alpha * g[i], decay, epsilon, gacc[i], dacc[i], &a, &b, &dx);
      gacc[i] = a;
      dacc[i] = b;
      p[i] += dx;
    }
  } else {
    return fail("adadelta: datatype must be float or double");
  }
  return 0;
}

// Address of linear element e for an operand, given the other operands'
// dimensions: exposes get-elem-dims->address so the tests can brute-force it.
// all_dims[0..n_dims) are the operands that form the max-shape (pass only the
// operand itself for the single-operand ops); which selects the operand.
int co_elem_address(const ct_dims* const* all_dims, int n_dims, int which, int64_t e, int64_t* addr,
                    int* mode) {
  if (n_dims < 1 || n_dims > 4 || which < 0 || which >= n_dims) return fail("bad operand count");
  Dims d[4];
  const Dims* ops[4];
  for (int k = 0; k < n_dims; ++k) {
    if (!load_dims(all_dims[k], &d[k])) return fail("bad dimensions");
    ops[k] = &d[k];
  }
  const MaxShape mx = max_shape_of(ops, n_dims);
  const Addr a = make_addr(d[which], mx);
  *addr = a(e);
  if (mode) *mode = (int)a.mode;
  return 0;
}

int co_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

}  // extern "C"
