// ops_ternary.hip -- ternary-op!, ternary-op-constant!, ternary-op-constant-constant!
// (src/cortex/tensor/math.clj:75-102; src/cortex/compute/cpu/tensor_math.clj:464-580).
#include "elementwise.h"
#include "functors.h"

using namespace cthip;

namespace {
bool valid_arg_idx(const int8_t* a) {
  if (!a) return false;
  int seen = 0;
  for (int k = 0; k < 3; ++k) {
    if (a[k] < 0 || a[k] > 2) return false;
    seen |= 1 << a[k];
  }
  return seen == 7;
}

// slots 0..2: tensors first (with their alphas), then constants.
template <class T>
int routed_select(hipStream_t s, void* dest, const ct_dims* dd, const void* const* t, const ct_dims* const* td,
                  const double* alpha, int n_tensors, const double* constants, const int8_t* arg_idx, int64_t n) {
  using A = typename ew_acc_of<T>::type;
  SelectRoutedF<T> f;
  EwOperand ops[4];
  ops[0] = {dest, dd, (int)sizeof(T), 0};
  for (int k = 0; k < 3; ++k) {
    if (k < n_tensors) {
      f.alpha[k] = (A)jvm_cast<T>(alpha[k]);
      ops[k + 1] = {t[k], td[k], (int)sizeof(T), 0};
    } else {
      f.alpha[k] = (A)1;
      ops[k + 1] = {nullptr, nullptr, (int)sizeof(T), bits_of<T>(jvm_cast<T>(constants[k - n_tensors]))};
    }
    f.arg_idx[k] = arg_idx[k];
  }
  return launch_elementwise(s, f, ops, n);
}

// Role of slot k: which of x (0), y (1), z (2) it is routed to.
int role_of(const int8_t* arg_idx, int slot) {
  for (int r = 0; r < 3; ++r)
    if (arg_idx[r] == slot) return r;
  return -1;
}

// x in the tensor, both results constant.  Returns false when the routing is another one.
template <class T>
bool select_cc(hipStream_t s, void* dest, const ct_dims* dd, const void* a, const ct_dims* ad, double a_alpha,
               const double* constants, const int8_t* arg_idx, int64_t n, int* rc) {
  using A = typename ew_acc_of<T>::type;
  if (role_of(arg_idx, 0) != 0) return false;
  const T cy = jvm_cast<T>(constants[arg_idx[1] - 1]), cz = jvm_cast<T>(constants[arg_idx[2] - 1]);
  const A xa = (A)jvm_cast<T>(a_alpha);
  EwOperand ops[2] = {{dest, dd, (int)sizeof(T), 0}, {a, ad, (int)sizeof(T), 0}};
  if constexpr (std::is_same<T, float>::value) {
    if (xa == (A)1) {
      *rc = launch_elementwise(s, SelectCCF<T, true>{xa, cy, cz}, ops, n);
      return true;
    }
  }
  *rc = launch_elementwise(s, SelectCCF<T>{xa, cy, cz}, ops, n);
  return true;
}

// x in a tensor, one result in the other tensor, the other result constant.
template <class T>
bool select_tc(hipStream_t s, void* dest, const ct_dims* dd, const void* const* t, const ct_dims* const* td,
               const double* alpha, double constant, const int8_t* arg_idx, int64_t n, int* rc) {
  using A = typename ew_acc_of<T>::type;
  const int xs = arg_idx[0];  // the slot that holds x
  if (xs > 1 || role_of(arg_idx, 2) == 0) return false;
  const int qs = 1 - xs;      // the other tensor
  const bool q_is_z = role_of(arg_idx, qs) == 2;
  const A xa = (A)jvm_cast<T>(alpha[xs]), qa = (A)jvm_cast<T>(alpha[qs]);
  const T c = jvm_cast<T>(constant);
  EwOperand ops[3] = {{dest, dd, (int)sizeof(T), 0}, {t[xs], td[xs], (int)sizeof(T), 0}, {t[qs], td[qs], (int)sizeof(T), 0}};
  if constexpr (std::is_same<T, float>::value) {
    if (xa == (A)1 && qa == (A)1) {
      *rc = q_is_z ? launch_elementwise(s, SelectTCF<T, true, true>{xa, qa, c}, ops, n)
                   : launch_elementwise(s, SelectTCF<T, false, true>{xa, qa, c}, ops, n);
      return true;
    }
  }
  *rc = q_is_z ? launch_elementwise(s, SelectTCF<T, true>{xa, qa, c}, ops, n)
               : launch_elementwise(s, SelectTCF<T, false>{xa, qa, c}, ops, n);
  return true;
}
}  // namespace

extern "C" {

int ct_ternary_op(void* stream, void* dest, const ct_dims* dest_dims, const void* x, const ct_dims* x_dims,
                  double x_alpha, const void* y, const ct_dims* y_dims, double y_alpha, const void* z,
                  const ct_dims* z_dims, double z_alpha, int64_t n, int op, int dtype) {
  CT_REQUIRE(dest && x && y && z, "ct_ternary_op: null buffer");
  CT_REQUIRE(op == CT_TOP_SELECT, "unknown ternary operation %d", op);
  CT_DISPATCH_DTYPE(dtype, {
    using A = typename ew_acc_of<T>::type;
    const A xa = (A)jvm_cast<T>(x_alpha), ya = (A)jvm_cast<T>(y_alpha), za = (A)jvm_cast<T>(z_alpha);
    EwOperand ops[4] = {{dest, dest_dims, (int)sizeof(T), 0},
                        {x, x_dims, (int)sizeof(T), 0},
                        {y, y_dims, (int)sizeof(T), 0},
                        {z, z_dims, (int)sizeof(T), 0}};
    if constexpr (std::is_same<T, float>::value) {
      if (xa == (A)1 && ya == (A)1 && za == (A)1) {
        SelectF<T, true> f{xa, ya, za};
        return launch_elementwise(static_cast<hipStream_t>(stream), f, ops, n);
      }
    }
    SelectF<T> f{xa, ya, za};
    return launch_elementwise(static_cast<hipStream_t>(stream), f, ops, n);
  });
  return CT_OK;
}

int ct_ternary_op_constant(void* stream, void* dest, const ct_dims* dest_dims, const void* a,
                           const ct_dims* a_dims, double a_alpha, const void* b, const ct_dims* b_dims,
                           double b_alpha, double constant, int64_t n, int op, const int8_t arg_idx[3],
                           int dtype) {
  CT_REQUIRE(dest && a && b, "ct_ternary_op_constant: null buffer");
  CT_REQUIRE(op == CT_TOP_SELECT, "unknown ternary operation %d", op);
  CT_REQUIRE(valid_arg_idx(arg_idx), "arg_idx must be a permutation of 0,1,2");
  const void* t[2] = {a, b};
  const ct_dims* td[2] = {a_dims, b_dims};
  const double al[2] = {a_alpha, b_alpha};
  const double cs[1] = {constant};
  CT_DISPATCH_DTYPE(dtype, {
    int rc = CT_OK;
    if (select_tc<T>(static_cast<hipStream_t>(stream), dest, dest_dims, t, td, al, constant, arg_idx, n, &rc)) return rc;
    return routed_select<T>(static_cast<hipStream_t>(stream), dest, dest_dims, t, td, al, 2, cs, arg_idx, n);
  });
  return CT_OK;
}

int ct_ternary_op_constant_constant(void* stream, void* dest, const ct_dims* dest_dims, const void* a,
                                    const ct_dims* a_dims, double a_alpha, double const_1, double const_2,
                                    int64_t n, int op, const int8_t arg_idx[3], int dtype) {
  CT_REQUIRE(dest && a, "ct_ternary_op_constant_constant: null buffer");
  CT_REQUIRE(op == CT_TOP_SELECT, "unknown ternary operation %d", op);
  CT_REQUIRE(valid_arg_idx(arg_idx), "arg_idx must be a permutation of 0,1,2");
  const void* t[1] = {a};
  const ct_dims* td[1] = {a_dims};
  const double al[1] = {a_alpha};
  const double cs[2] = {const_1, const_2};
  CT_DISPATCH_DTYPE(dtype, {
    int rc = CT_OK;
    if (select_cc<T>(static_cast<hipStream_t>(stream), dest, dest_dims, a, a_dims, a_alpha, cs, arg_idx, n, &rc)) return rc;
    return routed_select<T>(static_cast<hipStream_t>(stream), dest, dest_dims, t, td, al, 1, cs, arg_idx, n);
  });
  return CT_OK;
}

}  // extern "C"
