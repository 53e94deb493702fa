// ops_binary_f32.hip -- binary-op! and its constant / accumulate forms for float (see binary_impl.h).
#include "binary_impl.h"

namespace cthip {
template int binary_dispatch<float>(hipStream_t, const BinaryCall&);
}  // namespace cthip
