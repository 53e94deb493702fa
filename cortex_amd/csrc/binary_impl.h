// binary_impl.h -- the per-datatype body of binary-op! and its constant / accumulate
// forms.  The thirteen operations of one datatype instantiate every kernel family,
// which makes this the longest compilation of the library; ops_binary_*.hip each
// instantiate it for some datatypes so that they compile side by side.
#pragma once
#include "elementwise.h"
#include "functors.h"
#include "ops.h"

namespace cthip {

template <class T> int binary_dispatch(hipStream_t s, const BinaryCall& c);

namespace binary_detail {
template <class T, int OP>
int binary_run(hipStream_t s, const BinaryCall& c) {
  using A = typename ew_acc_of<T>::type;
  // A scalar side has had its alpha folded in by the caller; its multiplier is 1.
  const A xa = c.x ? (A)jvm_cast<T>(c.x_alpha) : (A)1;
  const A ya = c.y ? (A)jvm_cast<T>(c.y_alpha) : (A)1;
  EwOperand ops[3] = {{c.dest, c.dest_dims, (int)sizeof(T), 0},
                      {c.x, c.x ? c.x_dims : nullptr, (int)sizeof(T), bits_of<T>(jvm_cast<T>(c.x_scalar))},
                      {c.y, c.y ? c.y_dims : nullptr, (int)sizeof(T), bits_of<T>(jvm_cast<T>(c.y_scalar))}};
  if constexpr (std::is_same<T, float>::value && binary_plain_op(OP)) {
    if (unit_magnitude(xa) && unit_magnitude(ya) && !c.serial) {
      BinaryF<T, OP, true> f{xa, ya};
      return launch_elementwise(s, f, ops, c.n);
    }
  }
  BinaryF<T, OP> f{xa, ya};
  if constexpr (OP == CT_BOP_DIV && !std::is_floating_point<T>::value) {
    if (int rc = device_error_word(&f.div0)) return rc;
    if (int rc = arm_device_error_word(s, f.div0)) return rc;
  }
  const int rc = c.serial ? launch_elementwise_serial(s, f, ops, c.n) : launch_elementwise(s, f, ops, c.n);
  if constexpr (OP == CT_BOP_DIV && !std::is_floating_point<T>::value) {
    if (rc == CT_OK) return check_device_errors("binary-op! :/");
  }
  return rc;
}

template <class T>
int dispatch(hipStream_t s, const BinaryCall& c) {
  switch (c.op) {
    case CT_BOP_ADD: return binary_run<T, CT_BOP_ADD>(s, c);
    case CT_BOP_SUB: return binary_run<T, CT_BOP_SUB>(s, c);
    case CT_BOP_MUL: return binary_run<T, CT_BOP_MUL>(s, c);
    case CT_BOP_DIV: return binary_run<T, CT_BOP_DIV>(s, c);
    case CT_BOP_MIN: return binary_run<T, CT_BOP_MIN>(s, c);
    case CT_BOP_MAX: return binary_run<T, CT_BOP_MAX>(s, c);
    case CT_BOP_BIT_AND: return binary_run<T, CT_BOP_BIT_AND>(s, c);
    case CT_BOP_BIT_XOR: return binary_run<T, CT_BOP_BIT_XOR>(s, c);
    case CT_BOP_EQ: return binary_run<T, CT_BOP_EQ>(s, c);
    case CT_BOP_GT: return binary_run<T, CT_BOP_GT>(s, c);
    case CT_BOP_GE: return binary_run<T, CT_BOP_GE>(s, c);
    case CT_BOP_LT: return binary_run<T, CT_BOP_LT>(s, c);
    case CT_BOP_LE: return binary_run<T, CT_BOP_LE>(s, c);
    default: return set_error(CT_ERR_INVALID, "unknown binary operation %d", c.op);
  }
}
}  // namespace binary_detail

template <class T> int binary_dispatch(hipStream_t s, const BinaryCall& c) { return binary_detail::dispatch<T>(s, c); }

}  // namespace cthip
