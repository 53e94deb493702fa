// ops_unary.hip -- unary-op! and unary-accum!
// (src/cortex/tensor/math.clj:27-35; src/cortex/compute/cpu/tensor_math.clj:211-262).
#include "elementwise.h"
#include "functors.h"

using namespace cthip;

namespace {
template <class T, int OP>
int unary_run(hipStream_t s, void* dest, const ct_dims* dd, const void* x, const ct_dims* xd, double alpha,
              int64_t n, bool serial) {
  using A = typename ew_acc_of<T>::type;
  const T a = jvm_cast<T>(alpha);
  EwOperand ops[2] = {{dest, dd, (int)sizeof(T), 0}, {x, xd, (int)sizeof(T), 0}};
  if constexpr (std::is_same<T, float>::value) {
    if (a == (T)1 && !serial) {
      UnaryF<T, OP, true> f{(A)1};
      return launch_elementwise(s, f, ops, n);
    }
  }
  UnaryF<T, OP> f{(A)a};
  return serial ? launch_elementwise_serial(s, f, ops, n) : launch_elementwise(s, f, ops, n);
}

template <class T>
int unary_dispatch(hipStream_t s, void* dest, const ct_dims* dd, const void* x, const ct_dims* xd, double alpha,
                   int op, int64_t n, bool serial) {
  switch (op) {
    case CT_UOP_FLOOR: return unary_run<T, CT_UOP_FLOOR>(s, dest, dd, x, xd, alpha, n, serial);
    case CT_UOP_CEIL: return unary_run<T, CT_UOP_CEIL>(s, dest, dd, x, xd, alpha, n, serial);
    case CT_UOP_ROUND: return unary_run<T, CT_UOP_ROUND>(s, dest, dd, x, xd, alpha, n, serial);
    case CT_UOP_NEGATE: return unary_run<T, CT_UOP_NEGATE>(s, dest, dd, x, xd, alpha, n, serial);
    case CT_UOP_TANH: return unary_run<T, CT_UOP_TANH>(s, dest, dd, x, xd, alpha, n, serial);
    case CT_UOP_LOGISTIC: return unary_run<T, CT_UOP_LOGISTIC>(s, dest, dd, x, xd, alpha, n, serial);
    case CT_UOP_EXP: return unary_run<T, CT_UOP_EXP>(s, dest, dd, x, xd, alpha, n, serial);
    case CT_UOP_SQRT: return unary_run<T, CT_UOP_SQRT>(s, dest, dd, x, xd, alpha, n, serial);
    case CT_UOP_NOOP: return unary_run<T, CT_UOP_NOOP>(s, dest, dd, x, xd, alpha, n, serial);
    default: return set_error(CT_ERR_INVALID, "unknown unary operation %d", op);
  }
}
}  // namespace

extern "C" {

int ct_unary_op(void* stream, void* dest, const ct_dims* dest_dims, const void* x, const ct_dims* x_dims,
                double alpha, int op, int dtype, int64_t n) {
  CT_REQUIRE(dest && x, "ct_unary_op: null buffer");
  CT_DISPATCH_DTYPE(dtype, return unary_dispatch<T>(static_cast<hipStream_t>(stream), dest, dest_dims, x, x_dims, alpha, op, n, false));
  return CT_OK;
}

// In place: every element is read and written by the same lane, so the
// elementwise kernels apply with dest as its own input.  An indirectly indexed
// destination may name one address several times; the reference's serial loop
// (cpu/tensor_math.clj:234) then applies the op repeatedly, which only the
// serial kernel reproduces.
int ct_unary_accum(void* stream, void* dest, const ct_dims* dest_dims, double alpha, int op, int dtype,
                   int64_t n) {
  CT_REQUIRE(dest != nullptr, "ct_unary_accum: null buffer");
  if (int rc = check_dims(dest_dims, "dest")) return rc;
  const bool serial = !dims_direct(*dest_dims);
  CT_DISPATCH_DTYPE(dtype, return unary_dispatch<T>(static_cast<hipStream_t>(stream), dest, dest_dims, dest, dest_dims, alpha, op, n, serial));
  return CT_OK;
}

}  // extern "C"
