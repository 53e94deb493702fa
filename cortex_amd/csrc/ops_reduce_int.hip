// ops_reduce_int.hip -- unary-reduce! for the byte tensors (see reduce_impl.h); the integer tensors are
// spread over three translation units so that they compile side by side.
#include "reduce_impl.h"

namespace cthip {
namespace reduce_detail {
template int reduce_dispatch<int8_t>(hipStream_t, const PartialStore&, void*, const ct_dims*, double, const void*, const ct_dims*, int);
}  // namespace reduce_detail
}  // namespace cthip
