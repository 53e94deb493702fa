// elementwise.cpp -- turns a Plan into kernel argument blocks (host only).
#include "elementwise.h"

#include <algorithm>
#include <vector>

namespace cthip {

namespace {
constexpr int64_t kLim31 = int64_t(1) << 31;

// A call whose operands together exceed the 256 MiB last-level cache streams through the
// caches: its loads are marked non-temporal (level 1), and from about four times that size its
// stores too (level 2).  Below, plain accesses win: a copy of 242 MiB runs at 90 % of peak
// with plain loads and 83 % with non-temporal ones, one of 288 MiB at 77 % and 86 %; the
// transposing kernel and the widening conversions cross over at the same size.
uint32_t streaming_level(const Plan& plan, const EwOperand* ops) {
  int64_t bytes = 0;
  for (int k = 0; k < plan.n_ops; ++k)
    if (ops[k].ptr) bytes += plan.n * ops[k].elem_size;
  if (bytes >= (int64_t(1) << 30)) return 2;
  return bytes >= (int64_t(256) << 20) ? 1 : 0;
}
bool is_streaming(const Plan& plan, const EwOperand* ops) { return streaming_level(plan, ops) > 0; }

void common_vec(const Plan& plan, const EwOperand* ops, VecArgs* a) {
  const Canon& c = plan.canon;
  std::memset(a, 0, sizeof(*a));
  a->n_outer = c.nd - 1;
  a->streaming = streaming_level(plan, ops);
  for (int d = 0; d + 1 < c.nd; ++d) {
    if (d < 2) a->outer_fd01[d] = FastDiv((uint32_t)c.size[d + 1]);
    else a->outer_fd_hi[d - 2] = FastDiv((uint32_t)c.size[d + 1]);
  }
  for (int d = std::max(c.nd - 1, 0); d < 2; ++d) a->outer_fd01[d] = FastDiv(1);
  for (int k = 0; k < plan.n_ops; ++k) {
    a->ptr[k] = (char*)ops[k].ptr;
    a->cbits[k] = ops[k].cbits;
    if (!ops[k].ptr) a->const_mask |= 1u << k;
    else if (c.stride[k][0] == 1) a->unit_mask |= 1u << k;
    bool once = ops[k].ptr != nullptr;
    for (int d = 0; d < c.nd; ++d)
      if (c.stride[k][d] == 0 && c.size[d] > 1) once = false;
    if (once) a->nt_mask |= 1u << k;
    for (int d = 0; d + 1 < c.nd; ++d) {
      if (d < 2) a->outer_stride01[k][d] = c.stride[k][d + 1];
      else a->outer_stride_hi[k][d - 2] = c.stride[k][d + 1];
      if (d < 2 && c.any_index && c.index[k][d + 1]) {
        a->outer_index[k][d] = c.index[k][d + 1];
        a->indexed = 1;
        a->nt_mask &= ~(1u << k);
      }
    }
  }
}
}  // namespace

int prepare_vec(const Plan& plan, const EwOperand* ops, int vmax, VecArgs* main_args, int* main_vec,
                VecArgs* tail_args, bool* has_tail) {
  const Canon& c = plan.canon;
  const int64_t inner = c.size[0];
  int64_t rows = 1;
  for (int d = 1; d < c.nd; ++d) rows *= c.size[d];
  *has_tail = false;

  bool aligned = vmax > 1;
  for (int k = 0; aligned && k < plan.n_ops; ++k) {
    if (!ops[k].ptr || c.stride[k][0] != 1) continue;
    if (((uintptr_t)ops[k].ptr % (uintptr_t)(vmax * ops[k].elem_size)) != 0) aligned = false;
    for (int d = 1; aligned && d < c.nd; ++d)
      if (c.stride[k][d] % vmax != 0) aligned = false;
  }
  if (aligned && c.nd > 1 && inner % vmax != 0) aligned = false;
  if (aligned && c.nd == 1 && inner < vmax) aligned = false;

  common_vec(plan, ops, main_args);
  // The kernel decomposes a 32-bit vector index; a flat call is one row of up to
  // kVecLaunchMax vectors per launch (launch_vec walks longer ones in pieces).
  if (!aligned) {
    *main_vec = 1;
    main_args->inner_vecs = (uint32_t)std::min<int64_t>(inner, kVecLaunchMax);
    main_args->inner_fd = FastDiv(main_args->inner_vecs);
    main_args->total_vecs = (uint64_t)inner * (uint64_t)rows;
    CT_REQUIRE(c.nd == 1 || main_args->total_vecs < (uint64_t)kLim31, "tensor too large for 32-bit vector indexing");
    return CT_OK;
  }
  *main_vec = vmax;
  const int64_t inner_vecs = inner / vmax;
  main_args->inner_vecs = (uint32_t)std::min<int64_t>(inner_vecs, kVecLaunchMax);
  main_args->inner_fd = FastDiv(main_args->inner_vecs);
  main_args->total_vecs = (uint64_t)inner_vecs * (uint64_t)rows;
  CT_REQUIRE(c.nd == 1 || main_args->total_vecs < (uint64_t)kLim31, "tensor too large for 32-bit vector indexing");
  const int64_t tail = inner - inner_vecs * vmax;  // only possible when flat
  if (tail > 0) {
    *has_tail = true;
    common_vec(plan, ops, tail_args);
    for (int k = 0; k < plan.n_ops; ++k)
      if (ops[k].ptr && c.stride[k][0] == 1)
        tail_args->ptr[k] = (char*)ops[k].ptr + (inner_vecs * vmax) * ops[k].elem_size;
    tail_args->inner_vecs = (uint32_t)tail;
    tail_args->inner_fd = FastDiv((uint32_t)tail);
    tail_args->total_vecs = (uint64_t)tail;
  }
  return CT_OK;
}

int prepare_tile(const Plan& plan, const EwOperand* ops, int tile_a_edge, int tile_b_edge, bool wide_a, TileArgs* a,
                 size_t* lds_bytes, uint32_t* grid) {
  const Canon& c = plan.canon;
  const int b = plan.tile_b;
  std::memset(a, 0, sizeof(*a));
  a->sizeA = (uint32_t)c.size[0];
  a->sizeB = (uint32_t)c.size[b];
  a->tilesA = (a->sizeA + tile_a_edge - 1) / tile_a_edge;
  a->tilesB = (a->sizeB + tile_b_edge - 1) / tile_b_edge;
  // Super-tiles (see ew_tile_kernel): at most 64 x 2 tiles, 32 x 4 for the mirrored tile, evened
  // out so that the last super-tile along an axis is as full as the others.
  const uint32_t want_a = wide_a ? 32 : 64, want_b = wide_a ? 4 : 2;
  const uint32_t nsa = (a->tilesA + want_a - 1) / want_a, nsb = (a->tilesB + want_b - 1) / want_b;
  a->super_a = (a->tilesA + nsa - 1) / nsa;
  a->super_b = (a->tilesB + nsb - 1) / nsb;
  a->per_fd = FastDiv(a->super_a * a->super_b);
  a->sb_fd = FastDiv(a->super_b);
  a->nsb_fd = FastDiv(nsb);
  a->nst_fd = FastDiv(nsa * nsb);
  int64_t supers = (int64_t)nsa * nsb;
  int no = 0;
  for (int d = 1; d < c.nd; ++d) {
    if (d == b) continue;
    a->outer_fd[no] = FastDiv((uint32_t)c.size[d]);
    for (int k = 0; k < plan.n_ops; ++k) a->outer_stride[k][no] = c.stride[k][d];
    supers *= c.size[d];
    ++no;
  }
  a->n_outer = no;
  a->streaming = is_streaming(plan, ops) ? 1u : 0u;
  const int64_t blocks = (supers + kXcds - 1) / kXcds * kXcds * (int64_t)(a->super_a * a->super_b);
  CT_REQUIRE(supers < kLim31 && blocks < kLim31, "internal: tile grid too large");
  a->n_super = (uint32_t)supers;
  *grid = (uint32_t)blocks;
  size_t lds = 0;
  for (int k = 0; k < plan.n_ops; ++k) {
    a->ptr[k] = (char*)ops[k].ptr;
    a->cbits[k] = ops[k].cbits;
    a->strideA[k] = c.stride[k][0];
    a->strideB[k] = c.stride[k][b];
    if (!ops[k].ptr) a->const_mask |= 1u << k;
    if (plan.via_lds[k]) {
      a->lds_mask |= 1u << k;
      lds = std::max(lds, tile_slot_bytes((size_t)ops[k].elem_size, tile_a_edge, tile_b_edge));  // one tile, used in turn
    }
  }
  *lds_bytes = lds;
  return CT_OK;
}

// Cuts a call along its slowest axis of more than one element into pieces of at most `limit`
// elements: operands that span the axis get a shorter shape and a later start (in the index tensor
// when the axis is indexed), operands that broadcast along it stay as they are.  False when the
// call has another form (a count that is not the product of the largest shape, a commensurate
// operand).  When the trailing axes alone exceed the limit a piece is one coordinate of the axis,
// and the launcher cuts it again along the next axis.
bool split_leading(const EwOperand* ops, int n_ops, int64_t n, int64_t limit, std::vector<EwPiece>* pieces) {
  int rank = 0;
  for (int k = 0; k < n_ops; ++k)
    if (ops[k].ptr && ops[k].dims) rank = std::max(rank, ops[k].dims->ndim);
  if (rank == 0) return false;
  int64_t mx[CT_MAX_DIMS];
  for (int d = 0; d < rank; ++d) mx[d] = 1;
  for (int k = 0; k < n_ops; ++k) {
    if (!ops[k].ptr || !ops[k].dims) continue;
    const ct_dims& dm = *ops[k].dims;
    for (int i = 0; i < dm.ndim; ++i) mx[i + rank - dm.ndim] = std::max<int64_t>(mx[i + rank - dm.ndim], dm.shape[i]);
  }
  int lead = 0;
  while (lead < rank && mx[lead] == 1) ++lead;
  if (lead == rank) return false;
  int64_t rest = 1, total = 1;
  for (int d = lead + 1; d < rank; ++d) rest *= mx[d];
  for (int d = 0; d < rank; ++d) total *= mx[d];
  if (total != n) return false;
  const int64_t per = std::max<int64_t>(1, limit / rest);
  for (int64_t c0 = 0; c0 < mx[lead]; c0 += per) {
    const int64_t c1 = std::min(mx[lead], c0 + per);
    EwPiece piece;
    piece.n = (c1 - c0) * rest;
    for (int k = 0; k < n_ops; ++k) {
      piece.ptr[k] = ops[k].ptr;
      if (!ops[k].ptr || !ops[k].dims) { std::memset(&piece.dims[k], 0, sizeof(ct_dims)); continue; }
      piece.dims[k] = *ops[k].dims;
      const int di = lead - (rank - ops[k].dims->ndim);
      if (di < 0 || piece.dims[k].shape[di] == 1) {
        if (k == 0) return false;  // a destination that repeats along the axis is not cut here
        continue;
      }
      if (piece.dims[k].shape[di] != mx[lead]) return false;
      piece.dims[k].shape[di] = c1 - c0;
      if (piece.dims[k].index[di]) piece.dims[k].index[di] += c0;
      else piece.ptr[k] = static_cast<const char*>(ops[k].ptr) + c0 * piece.dims[k].strides[di] * ops[k].elem_size;
    }
    pieces->push_back(piece);
  }
  return true;
}

// Vectors that start anywhere (ew_vecu_kernel): rows of at least one vector whose starts or
// lengths keep them off the 16-byte grid.  False for small calls, indexed axes and rows shorter
// than a vector, which stay with one element per lane.
bool prepare_vecu(const Plan& plan, const EwOperand* ops, int vmax, VecArgs* a, uint32_t* inner_elems) {
  const Canon& c = plan.canon;
  if (c.any_index || vmax < 2 || plan.n < 4096) return false;
  const int64_t inner = c.size[0];
  if (inner < vmax || inner >= kLim31) return false;
  bool any_unit = false;
  for (int k = 0; k < plan.n_ops; ++k) any_unit = any_unit || (ops[k].ptr && c.stride[k][0] == 1);
  if (!any_unit) return false;
  int64_t rows = 1;
  for (int d = 1; d < c.nd; ++d) rows *= c.size[d];
  const int64_t inner_vecs = (inner + vmax - 1) / vmax;
  if (inner_vecs * rows >= kLim31) return false;
  common_vec(plan, ops, a);
  a->inner_vecs = (uint32_t)inner_vecs;
  a->inner_fd = FastDiv((uint32_t)inner_vecs);
  a->total_vecs = (uint64_t)(inner_vecs * rows);
  *inner_elems = (uint32_t)inner;
  return true;
}

// Rows that are no whole number of vectors, big operands dense over the whole call: see
// ew_ragged_kernel.  False when the call has another shape.
bool prepare_ragged(const Plan& plan, const EwOperand* ops, int vmax, RaggedArgs* a) {
  const Canon& c = plan.canon;
  if (c.any_index || c.nd < 2 || vmax < 2) return false;
  const int64_t inner = c.size[0];
  if (inner < vmax || inner % vmax == 0 || plan.n >= kLim31 || plan.n < 4096) return false;
  std::memset(a, 0, sizeof(*a));
  a->n = (uint32_t)plan.n;
  a->inner_fd = FastDiv((uint32_t)inner);
  a->n_outer = c.nd - 1;
  for (int d = 1; d < c.nd; ++d) a->outer_fd[d - 1] = FastDiv((uint32_t)c.size[d]);
  a->streaming = streaming_level(plan, ops) > 0 ? 1u : 0u;
  for (int k = 0; k < plan.n_ops; ++k) {
    a->ptr[k] = (char*)ops[k].ptr;
    a->cbits[k] = ops[k].cbits;
    if (!ops[k].ptr) {
      if (k == 0) return false;
      a->const_mask |= 1u << k;
      continue;
    }
    if (c.stride[k][0] == 1) {
      bool dense = true, periodic = true;
      int64_t expect = inner;
      for (int d = 1; d < c.nd; ++d) {
        if (c.stride[k][d] != expect) dense = false;
        if (c.stride[k][d] != 0) periodic = false;
        expect *= c.size[d];
      }
      if (dense) {
        if (((uintptr_t)ops[k].ptr % (uintptr_t)(vmax * ops[k].elem_size)) != 0) return false;
        a->dense_mask |= 1u << k;
      } else if (k == 0) {
        return false;
      } else if (!periodic) {
        a->pitched_mask |= 1u << k;
        for (int d = 1; d < c.nd; ++d) a->outer_stride[k][d - 1] = c.stride[k][d];
      }
    } else if (c.stride[k][0] == 0 && k != 0) {
      a->scalar_mask |= 1u << k;
      for (int d = 1; d < c.nd; ++d) a->outer_stride[k][d - 1] = c.stride[k][d];
    } else {
      return false;
    }
  }
  return (a->dense_mask & 1u) != 0;
}

// A dense destination [rows, w] from unit-stride rows of a pitch of at most 128 bytes that leaves at least
// a fifth of every pitch unused (otherwise reading each row where it lies moves about the same lines).
bool prepare_span(const Plan& plan, const EwOperand* ops, int vmax, SpanArgs* a) {
  const Canon& c = plan.canon;
  if (c.any_index || c.nd != 2 || plan.n_ops != 2 || !ops[0].ptr || !ops[1].ptr) return false;
  const int64_t w = c.size[0], rows = c.size[1], pitch = c.stride[1][1];
  if (c.stride[0][0] != 1 || c.stride[0][1] != w || c.stride[1][0] != 1) return false;
  if (w < 2 || pitch <= w || pitch * ops[1].elem_size > 128 || w * 5 > pitch * 4) return false;
  if (plan.n < (int64_t(1) << 20) || plan.n >= kLim31 || rows * pitch >= kLim31) return false;
  if (((uintptr_t)ops[0].ptr % 16) != 0 || ((uintptr_t)ops[1].ptr % 16) != 0) return false;
  // a block's rows: a multiple of 16 (so that its span and its share of the destination start on the 16-byte
  // grid whatever the element sizes) whose span fits the LDS budget
  int64_t per = kSpanLdsBytes / (pitch * ops[1].elem_size) / 16 * 16;
  if (per < 16) return false;
  if (per > 256) per = 256;
  (void)vmax;
  std::memset(a, 0, sizeof(*a));
  a->ptr[0] = (char*)ops[0].ptr;
  a->ptr[1] = (char*)ops[1].ptr;
  a->rows = (uint32_t)rows;
  a->w = (uint32_t)w;
  a->pitch = (uint32_t)pitch;
  a->w_fd = FastDiv((uint32_t)w);
  a->rows_per_block = (uint32_t)per;
  return true;
}

bool prepare_lace(const Plan& plan, const EwOperand* ops, int vmax, LaceArgs* a, int* n_short, int* ppt, uint32_t* grid) {
  const Canon& c = plan.canon;
  if (c.any_index || c.nd < 2 || c.stride[0][0] != 1) return false;
  // Axis 0 is the destination's unit-stride axis.  Either it is the long axis (planar destination) and
  // some other axis is the short one, or it is the short axis and the destination is laced along the
  // axis whose destination stride equals the short extent.
  int ls = -1, ll = -1;
  if (c.size[0] >= 2 && c.size[0] <= kLaceMaxShort) {
    for (int i = 1; i < c.nd && ll < 0; ++i)
      if (c.stride[0][i] == c.size[0]) ll = i;
    if (ll >= 0) ls = 0;
  }
  if (ls < 0) {
    // planar destination: the short axis is the one along which some input is unit-stride
    for (int k = 1; k < plan.n_ops && ls < 0; ++k) {
      if (!ops[k].ptr) continue;
      for (int i = 1; i < c.nd; ++i)
        if (c.stride[k][i] == 1 && c.size[i] >= 2 && c.size[i] <= kLaceMaxShort) { ls = i; break; }
    }
    ll = 0;
  }
  if (ls < 0 || ll < 0 || ls == ll) return false;
  const int64_t n_s = c.size[ls], n_l = c.size[ll];
  if (n_l < 16 || n_l >= kLim31) return false;
  std::memset(a, 0, sizeof(*a));
  bool any_laced = false, any_planar = false;
  for (int k = 0; k < plan.n_ops; ++k) {
    a->ptr[k] = (char*)ops[k].ptr;
    a->cbits[k] = ops[k].cbits;
    if (!ops[k].ptr) { a->const_mask |= 1u << k; continue; }
    if (c.stride[k][ls] == 1 && c.stride[k][ll] == n_s) {
      a->laced_mask |= 1u << k;
      any_laced = true;
    } else if (c.stride[k][ll] == 1 && c.stride[k][ls] > 0) {
      a->plane_stride[k] = c.stride[k][ls];
      any_planar = true;
    } else {
      return false;
    }
  }
  if (!any_laced || !any_planar) return false;
  a->streaming = streaming_level(plan, ops) > 0 ? 1u : 0u;
  int64_t rows = 1;
  int no = 0;
  for (int d = 0; d < c.nd; ++d) {
    if (d == ls || d == ll) continue;
    if (c.size[d] >= kLim31) return false;
    a->outer_fd[no] = FastDiv((uint32_t)c.size[d]);
    for (int k = 0; k < plan.n_ops; ++k) a->outer_stride[k][no] = c.stride[k][d];
    rows *= c.size[d];
    ++no;
  }
  a->n_outer = no;
  // full-width vectors need every piece a lane touches to start on a vector boundary
  bool vec = vmax > 1 && n_l % vmax == 0;
  for (int k = 0; vec && k < plan.n_ops; ++k) {
    if (!ops[k].ptr) continue;
    if (((uintptr_t)ops[k].ptr % (uintptr_t)(vmax * ops[k].elem_size)) != 0) vec = false;
    if (a->plane_stride[k] % vmax != 0) vec = false;
    for (int d = 0; vec && d < no; ++d)
      if (a->outer_stride[k][d] % vmax != 0) vec = false;
  }
  *ppt = vec ? vmax : 1;
  *n_short = (int)n_s;
  const int64_t per_block = (int64_t)kBlock * *ppt;
  const int64_t per_row = (n_l + per_block - 1) / per_block;
  if (per_row * rows >= kLim31) return false;
  a->n_long = (uint32_t)n_l;
  a->per_row_fd = FastDiv((uint32_t)per_row);
  *grid = (uint32_t)(per_row * rows);
  return true;
}

int prepare_gen(const Plan& plan, const EwOperand* ops, GenArgs* a, bool* use64, uint32_t* grid) {
  const GenPlan& g = plan.gen;
  std::memset(a, 0, sizeof(*a));
  a->n = plan.n;
  a->nd = g.nd;
  bool big = plan.n >= kLim31;
  for (int d = 0; d < CT_MAX_DIMS; ++d) {
    a->rmax[d] = g.rmax[d];
    if (g.rmax[d] >= kLim31) big = true;
  }
  for (int k = 0; k < plan.n_ops; ++k) {
    a->op[k] = g.op[k];
    a->ptr[k] = (char*)ops[k].ptr;
    a->cbits[k] = ops[k].cbits;
    if (g.op[k].mode == 3) a->need_coords = 1;
    if (g.op[k].ec >= kLim31 || g.op[k].amt >= kLim31) big = true;
    for (int d = 0; d < CT_MAX_DIMS; ++d)
      if (g.op[k].shape[d] >= kLim31) big = true;
  }
  for (int k = plan.n_ops; k < kMaxOps; ++k) a->op[k].mode = 4;
  if (!big)
    for (int d = 0; d < CT_MAX_DIMS; ++d) a->rmax_fd[d] = FastDiv((uint32_t)g.rmax[d]);
  *use64 = big;
  const int64_t blocks = (plan.n + kBlock - 1) / kBlock;
  *grid = (uint32_t)std::min<int64_t>(blocks, 16384);
  return CT_OK;
}

}  // namespace cthip
