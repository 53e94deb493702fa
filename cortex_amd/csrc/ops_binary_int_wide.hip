// ops_binary_int_wide.hip -- binary-op! and its constant / accumulate forms for int32_t, int64_t (see binary_impl.h).
#include "binary_impl.h"

namespace cthip {
template int binary_dispatch<int32_t>(hipStream_t, const BinaryCall&);
template int binary_dispatch<int64_t>(hipStream_t, const BinaryCall&);
}  // namespace cthip
