// ops_assign.hip -- assign-constant! and the marshalling assign!
// (src/cortex/tensor/math.clj:14-26; src/cortex/compute/cpu/tensor_math.clj:137-208).
#include "elementwise.h"
#include "functors.h"

using namespace cthip;

namespace {
template <class D>
int assign_to(hipStream_t s, void* dest, const ct_dims* dd, const void* src, const ct_dims* sd, int src_dtype,
              int64_t n) {
#define CT_SRC_CASE(code, S)                                                                    \
  case code: {                                                                                  \
    AssignF<D, S> f;                                                                            \
    EwOperand ops[2] = {{dest, dd, (int)sizeof(D), 0}, {src, sd, (int)sizeof(S), 0}};           \
    return launch_elementwise(s, f, ops, n);                                                    \
  }
  switch (src_dtype) {
    CT_SRC_CASE(CT_I8, int8_t)
    CT_SRC_CASE(CT_I16, int16_t)
    CT_SRC_CASE(CT_I32, int32_t)
    CT_SRC_CASE(CT_I64, int64_t)
    CT_SRC_CASE(CT_F32, float)
    CT_SRC_CASE(CT_F64, double)
    CT_SRC_CASE(CT_U8, uint8_t)
    default: return set_error(CT_ERR_INVALID, "ct_assign: unknown source datatype %d", src_dtype);
  }
#undef CT_SRC_CASE
}
}  // namespace

extern "C" {

int ct_assign_constant(void* stream, void* dest, const ct_dims* dest_dims, int dtype, double value,
                       int64_t n) {
  CT_REQUIRE(dest != nullptr, "ct_assign_constant: null dest");
  CT_DISPATCH_DTYPE(dtype, {
    ConstantF<T> f{jvm_cast<T>(value)};
    EwOperand ops[1] = {{dest, dest_dims, (int)sizeof(T), 0}};
    return launch_elementwise(static_cast<hipStream_t>(stream), f, ops, n);
  });
  return CT_OK;
}

int ct_assign(void* stream, void* dest, const ct_dims* dest_dims, int dest_dtype, const void* src,
              const ct_dims* src_dims, int src_dtype, int64_t n) {
  CT_REQUIRE(dest && src, "ct_assign: null buffer");
  CT_DISPATCH_DTYPE(dest_dtype,
                    return assign_to<T>(static_cast<hipStream_t>(stream), dest, dest_dims, src, src_dims, src_dtype, n));
  return CT_OK;
}

}  // extern "C"
