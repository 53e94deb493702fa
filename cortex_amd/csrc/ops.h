// ops.h -- internal call descriptors shared between translation units.
#pragma once

#include "common.h"

namespace cthip {

// dest = op(x * x_alpha, y * y_alpha).  A null x (or y) marks that side as the
// scalar x_scalar (y_scalar), whose alpha the caller has already folded in.
struct BinaryCall {
  void* dest;
  const ct_dims* dest_dims;
  const void* x;
  const ct_dims* x_dims;
  double x_alpha, x_scalar;
  const void* y;
  const ct_dims* y_dims;
  double y_alpha, y_scalar;
  int64_t n;
  int op;
  bool serial = false;  // apply the updates one by one in increasing e
};

int run_binary(hipStream_t s, int dtype, const BinaryCall& c);

// output += unary-reduce!(input * input_alpha): the reduction's kernels with the addition (both
// values widened, one rounding, as binary-op! :+ forms it) applied where they store their results.
int unary_reduce_accumulate(hipStream_t stream, void* output, const ct_dims* output_dims, double input_alpha,
                            const void* input, const ct_dims* input_dims, int op, int dtype);

}  // namespace cthip
