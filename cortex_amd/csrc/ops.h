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

// binary-accum! into a broadcast destination as chains of serial updates, one block per strip of
// neighbouring chains (ops_accum_stream.hip).  The caller has checked the shape: either the chains
// are unit-stride in y (`pitch` is y's stride of one step) or the steps are (`pitch` is y's stride
// between chains; a chain's steps are n_red / n_inner runs of n_inner contiguous elements,
// outer_stride apart); every stride of y and y itself sit on the 16-byte grid.
struct AccumStreamCall {
  void* dest;
  const void* y;
  int64_t n_red;
  int64_t pitch;
  int64_t u, d_ustride;           // chains along the strip axis and the destination's stride there
  bool steps_unit_stride;
  int64_t n_inner, outer_stride;  // steps unit-stride only
  int n_rest;                     // other kept axes
  int64_t rsize[CT_MAX_DIMS], rd_stride[CT_MAX_DIMS], ry_stride[CT_MAX_DIMS];
  double dest_alpha, y_alpha;
  bool reverse;
  int op, dtype;
  uint32_t* div0;                 // integer :/ only: the device's error word
};
int accum_stream(hipStream_t s, const AccumStreamCall& c);

}  // namespace cthip
