// plan.h -- host-side access-pattern analysis for the elementwise kernels.
//
// The reference evaluates every operand address per element through
// get-elem-dims->address (src/cortex/compute/cpu/tensor_math.clj:82-134), a
// loop of rem/quot per dimension (src/cortex/tensor/dimensions.clj:226-252).
// Here the same address function is analysed ONCE per call on the host:
// dimensions are left-padded to a common rank, size-1 dimensions dropped,
// dimensions re-ordered so the destination's fastest axis comes first, and
// adjacent dimensions merged when every operand's strides chain.  The result
// selects one of three kernel families:
//   VEC      every operand is unit-stride or broadcast along the innermost
//            axis: 128-bit coalesced loads/stores, address math per vector.
//            One of the first two outer axes of an operand may be addressed
//            through an index tensor (row gather / scatter).
//   TILE     the destination is unit-stride along axis A while some input is
//            unit-stride along another axis B (a transposed view): LDS tile.
//   GENERAL  anything else, including indirect (index tensor) dimensions and
//            non-commensurate shapes: the reference's address objects,
//            evaluated per element with precomputed multiply-shift division.
#pragma once

#include "common.h"

namespace cthip {

constexpr int kMaxOps = 4;  // destination + up to three tensor inputs

struct OperandIn {
  const void* ptr;       // device pointer; nullptr marks a scalar constant input
  const ct_dims* dims;   // nullptr for constants
  int elem_size;
};

// Canonical (merged) iteration space, fastest axis first.  stride 0 marks a
// broadcast axis of that operand.  index[k][d] != nullptr: operand k addresses
// axis d through an index tensor (coordinate c contributes index[c] * stride);
// such an axis is never merged with another and is never the innermost one.
struct Canon {
  int nd;
  int64_t size[CT_MAX_DIMS];
  int64_t stride[kMaxOps][CT_MAX_DIMS];
  const int32_t* index[kMaxOps][CT_MAX_DIMS];
  bool any_index;
};

// One operand of the GENERAL kernel: the four address objects of the CPU
// backend (cpu/tensor_math.clj:38-66).
struct GenOperand {
  int32_t mode;  // 0 identity, 1 (e / amt) % ec, 2 e % ec, 3 per-dimension
  int64_t ec, amt;
  int64_t shape[CT_MAX_DIMS];    // fastest first, padded with 1
  int64_t stride[CT_MAX_DIMS];
  const int32_t* index[CT_MAX_DIMS];
};

struct GenPlan {
  int nd;
  int64_t rmax[CT_MAX_DIMS];  // max-shape, fastest first
  GenOperand op[kMaxOps];
};

enum PlanKind { PK_VEC = 0, PK_TILE = 1, PK_GENERAL = 2 };

struct Plan {
  PlanKind kind;
  int n_ops;
  int64_t n;
  bool regular;   // pure broadcast structure, all direct, n == prod(max-shape)
  Canon canon;    // valid when regular
  int tile_b;     // TILE: canonical axis that is unit-stride for the transposed inputs
  bool via_lds[kMaxOps];  // TILE: which operands are read along axis B
  GenPlan gen;    // valid when kind == PK_GENERAL
};

// Host predicates of src/cortex/tensor/dimensions.clj.
bool dims_direct(const ct_dims& d);
bool dims_dense(const ct_dims& d);
bool dims_access_increasing(const ct_dims& d);
int64_t dims_ecount(const ct_dims& d);
// Validates rank and shape; returns 0 or sets the error.
int check_dims(const ct_dims* d, const char* what);

// Builds the plan for `n_ops` operands (ops[0] is the destination).  The
// max-shape is taken over the tensor operands given, so a call that passes the
// destination alone reproduces the single-operand methods of the reference
// (cpu/tensor_math.clj:144, 232, 321).
// With `reference_order` set the operands are never re-ordered or merged: the
// plan is PK_GENERAL over the reference's own address objects, so logical
// element e keeps the reference's meaning (needed when the order of the
// updates matters).
int build_plan(const OperandIn* ops, int n_ops, int64_t n, Plan* plan, bool reference_order = false);

// The reference's address object for one operand against an explicit
// max-shape (slowest first, `rank` entries): get-elem-dims->address
// (cpu/tensor_math.clj:82-134).  rmax receives the max-shape fastest first.
int reference_operand(const ct_dims* d, const int64_t* max_shape, int rank, GenOperand* out, int64_t* rmax);
// Same, with the operand's own shape as max-shape (the single-operand methods).
int reference_operand_own(const ct_dims* d, GenOperand* out, int64_t* rmax, int* rank);

}  // namespace cthip
