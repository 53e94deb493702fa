// ops_binary.hip -- binary-op!, binary-op-constant!, binary-accum-constant! and
// the non-aliasing half of binary-accum!
// (src/cortex/tensor/math.clj:36-73; src/cortex/compute/cpu/tensor_math.clj:278-462, 1439-1463).
#include "elementwise.h"
#include "functors.h"
#include "ops.h"

using namespace cthip;

namespace {
template <class T, int OP>
int binary_run(hipStream_t s, const BinaryCall& c) {
  using A = typename acc_of<T>::type;
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
  return c.serial ? launch_elementwise_serial(s, f, ops, c.n) : launch_elementwise(s, f, ops, c.n);
}

template <class T>
int binary_dispatch(hipStream_t s, const BinaryCall& c) {
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
}  // namespace

namespace cthip {
int run_binary(hipStream_t s, int dtype, const BinaryCall& c) {
  CT_DISPATCH_DTYPE(dtype, return binary_dispatch<T>(s, c));
  return CT_OK;
}
}  // namespace cthip

extern "C" {

int ct_binary_op(void* stream, void* dest, const ct_dims* dest_dims, const void* x, const ct_dims* x_dims,
                 double x_alpha, const void* y, const ct_dims* y_dims, double y_alpha, int64_t n, int op,
                 int dtype) {
  CT_REQUIRE(dest && x && y, "ct_binary_op: null buffer");
  BinaryCall c{dest, dest_dims, x, x_dims, x_alpha, 0.0, y, y_dims, y_alpha, 0.0, n, op};
  return run_binary(static_cast<hipStream_t>(stream), dtype, c);
}

int ct_binary_op_constant(void* stream, void* dest, const ct_dims* dest_dims, const void* x,
                          const ct_dims* x_dims, double x_alpha, double scalar, int64_t n, int op,
                          int reverse_operands, int dtype) {
  CT_REQUIRE(dest && x, "ct_binary_op_constant: null buffer");
  BinaryCall c = reverse_operands
                     ? BinaryCall{dest, dest_dims, nullptr, nullptr, 1.0, scalar, x, x_dims, x_alpha, 0.0, n, op}
                     : BinaryCall{dest, dest_dims, x, x_dims, x_alpha, 0.0, nullptr, nullptr, 1.0, scalar, n, op};
  return run_binary(static_cast<hipStream_t>(stream), dtype, c);
}

// dest is read and written by the same lane, so the plain kernels apply; an
// indirectly indexed destination keeps the reference's serial loop
// (cpu/tensor_math.clj:324).
int ct_binary_accum_constant(void* stream, void* dest, const ct_dims* dest_dims, double dest_alpha,
                             double scalar, int64_t n, int op, int reverse_operands, int dtype) {
  CT_REQUIRE(dest != nullptr, "ct_binary_accum_constant: null buffer");
  if (int rc = check_dims(dest_dims, "dest")) return rc;
  BinaryCall c = reverse_operands
                     ? BinaryCall{dest, dest_dims, nullptr, nullptr, 1.0, scalar, dest, dest_dims, dest_alpha, 0.0, n, op}
                     : BinaryCall{dest, dest_dims, dest, dest_dims, dest_alpha, 0.0, nullptr, nullptr, 1.0, scalar, n, op};
  c.serial = !dims_direct(*dest_dims);
  return run_binary(static_cast<hipStream_t>(stream), dtype, c);
}

}  // extern "C"
