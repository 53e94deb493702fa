// ops_reduce_int.hip -- unary-reduce! for the integer tensors (see reduce_impl.h).
#include "reduce_impl.h"

namespace cthip {
namespace reduce_detail {
template int reduce_dispatch<int8_t>(hipStream_t, const PartialStore&, void*, const ct_dims*, double, const void*, const ct_dims*, int);
template int reduce_dispatch<int16_t>(hipStream_t, const PartialStore&, void*, const ct_dims*, double, const void*, const ct_dims*, int);
template int reduce_dispatch<int32_t>(hipStream_t, const PartialStore&, void*, const ct_dims*, double, const void*, const ct_dims*, int);
template int reduce_dispatch<int64_t>(hipStream_t, const PartialStore&, void*, const ct_dims*, double, const void*, const ct_dims*, int);
template int reduce_dispatch<uint8_t>(hipStream_t, const PartialStore&, void*, const ct_dims*, double, const void*, const ct_dims*, int);
}  // namespace reduce_detail
}  // namespace cthip
