// ops_binary_int_narrow.hip -- binary-op! and its constant / accumulate forms for int8_t, int16_t, uint8_t (see binary_impl.h).
#include "binary_impl.h"

namespace cthip {
template int binary_dispatch<int8_t>(hipStream_t, const BinaryCall&);
template int binary_dispatch<int16_t>(hipStream_t, const BinaryCall&);
template int binary_dispatch<uint8_t>(hipStream_t, const BinaryCall&);
}  // namespace cthip
