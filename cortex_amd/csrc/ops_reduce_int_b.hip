// ops_reduce_int_b.hip -- unary-reduce! for the unsigned byte and long tensors (see reduce_impl.h); the integer tensors are
// spread over three translation units so that they compile side by side.
#include "reduce_impl.h"

namespace cthip {
namespace reduce_detail {
template int reduce_dispatch<uint8_t>(hipStream_t, const PartialStore&, void*, const ct_dims*, double, const void*, const ct_dims*, int);
template int reduce_dispatch<int64_t>(hipStream_t, const PartialStore&, void*, const ct_dims*, double, const void*, const ct_dims*, int);
}  // namespace reduce_detail
}  // namespace cthip
