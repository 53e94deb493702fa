// ops_binary_f64.hip -- binary-op! and its constant / accumulate forms for double (see binary_impl.h).
#include "binary_impl.h"

namespace cthip {
template int binary_dispatch<double>(hipStream_t, const BinaryCall&);
}  // namespace cthip
