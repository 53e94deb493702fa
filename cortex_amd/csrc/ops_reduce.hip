// ops_reduce.hip -- unary-reduce! (src/cortex/tensor/math.clj:104-108;
// src/cortex/compute/cpu/tensor_math.clj:582-663): the entry points, and the kernels of float and double
// tensors (reduce_impl.h; the integer tensors are instantiated in ops_reduce_int*.hip).
#include "reduce_impl.h"

using namespace cthip;
using namespace cthip::reduce_detail;

namespace cthip {
namespace reduce_detail {
template int reduce_dispatch<float>(hipStream_t, const PartialStore&, void*, const ct_dims*, double, const void*, const ct_dims*, int);
template int reduce_dispatch<double>(hipStream_t, const PartialStore&, void*, const ct_dims*, double, const void*, const ct_dims*, int);
extern template int reduce_dispatch<int8_t>(hipStream_t, const PartialStore&, void*, const ct_dims*, double, const void*, const ct_dims*, int);
extern template int reduce_dispatch<int16_t>(hipStream_t, const PartialStore&, void*, const ct_dims*, double, const void*, const ct_dims*, int);
extern template int reduce_dispatch<int32_t>(hipStream_t, const PartialStore&, void*, const ct_dims*, double, const void*, const ct_dims*, int);
extern template int reduce_dispatch<int64_t>(hipStream_t, const PartialStore&, void*, const ct_dims*, double, const void*, const ct_dims*, int);
extern template int reduce_dispatch<uint8_t>(hipStream_t, const PartialStore&, void*, const ct_dims*, double, const void*, const ct_dims*, int);
}  // namespace reduce_detail
}  // namespace cthip

extern "C" int ct_unary_reduce(void* stream, void* output, const ct_dims* output_dims, double input_alpha,
                               const void* input, const ct_dims* input_dims, int op, int dtype) {
  CT_REQUIRE(output && input, "ct_unary_reduce: null buffer");
  if (int rc = check_dims(output_dims, "output")) return rc;
  if (int rc = check_dims(input_dims, "input")) return rc;
  const PartialStore ps{nullptr, 0, "ct_unary_reduce"};
  CT_DISPATCH_DTYPE(dtype, return reduce_dispatch<T>(static_cast<hipStream_t>(stream), ps, output, output_dims, input_alpha, input, input_dims, op));
  return CT_OK;
}

// output += reduction, with the addition formed as binary-op! :+ forms it.  The last pass of
// the staged binary-accum! :+ (ops_accum.hip).
int cthip::unary_reduce_accumulate(hipStream_t stream, void* output, const ct_dims* output_dims, double input_alpha,
                                   const void* input, const ct_dims* input_dims, int op, int dtype) {
  const PartialStore ps{nullptr, 0, "binary-accum!", true};
  CT_DISPATCH_DTYPE(dtype, return reduce_dispatch<T>(stream, ps, output, output_dims, input_alpha, input, input_dims, op));
  return CT_OK;
}

// ------------------------------------------------------------------ the entry point that allocates nothing
//
// Same kernels and the same plan as ct_unary_reduce, so the results are the
// same bits; the partial accumulators of a split reduction live in a fixed
// array in device memory instead of the stream's growing scratch block.  Every
// device the library runs on holds its own copy of the array, at its own
// address, until the process ends.  The array's name below is a host-side
// stand-in, not a device address: host code only ever uses the address that
// hipGetSymbolAddress returned for the current device.
//
// The partials are written in full by the first kernel of a call before the
// finishing kernel reads them, so nothing in the array has to start at zero.
// Calls on one device share the array: two calls that overlap in time on one
// device (different streams, or different host threads) race.

namespace {

constexpr size_t kFixedScratchBytes = size_t(2) << 20;
constexpr int kFixedScratchDevices = 64;

static __device__ __align__(256) unsigned char scratch[kFixedScratchBytes];

std::mutex g_fixed_mutex;
void* g_fixed_ptr[kFixedScratchDevices] = {};

// Device address of `scratch` on the current device, resolved once per device.
int fixed_scratch(void** out) {
  int dev = 0;
  CT_HIP(hipGetDevice(&dev));
  CT_REQUIRE(dev >= 0 && dev < kFixedScratchDevices, "ct_unary_reduce_noalloc: device %d outside 0..%d", dev,
             kFixedScratchDevices - 1);
  std::lock_guard<std::mutex> lock(g_fixed_mutex);
  if (!g_fixed_ptr[dev]) {
    void* ptr = nullptr;
    CT_HIP(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)));
    CT_REQUIRE(ptr != nullptr, "ct_unary_reduce_noalloc: the scratch array has no address on device %d", dev);
    g_fixed_ptr[dev] = ptr;
  }
  *out = g_fixed_ptr[dev];
  return CT_OK;
}

}  // namespace

extern "C" int ct_unary_reduce_noalloc(void* stream, void* output, const ct_dims* output_dims, double input_alpha,
                                       const void* input, const ct_dims* input_dims, int op, int dtype) {
  CT_REQUIRE(output && input, "ct_unary_reduce_noalloc: null buffer");
  if (int rc = check_dims(output_dims, "output")) return rc;
  if (int rc = check_dims(input_dims, "input")) return rc;
  void* ptr = nullptr;
  if (int rc = fixed_scratch(&ptr)) return rc;
  const PartialStore ps{ptr, kFixedScratchBytes, "ct_unary_reduce_noalloc"};
  CT_DISPATCH_DTYPE(dtype, return reduce_dispatch<T>(static_cast<hipStream_t>(stream), ps, output, output_dims, input_alpha, input, input_dims, op));
  return CT_OK;
}
