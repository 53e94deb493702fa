// ops_binary.hip -- binary-op!, binary-op-constant!, binary-accum-constant! and
// the non-aliasing half of binary-accum!
// (src/cortex/tensor/math.clj:36-73; src/cortex/compute/cpu/tensor_math.clj:278-462, 1439-1463).
#include "elementwise.h"
#include "ops.h"

using namespace cthip;

namespace cthip {
// defined per datatype in ops_binary_f32.hip, _f64, _int_narrow and _int_wide
template <class T> int binary_dispatch(hipStream_t s, const BinaryCall& c);

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
