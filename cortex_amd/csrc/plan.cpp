// plan.cpp -- see plan.h.
#include "plan.h"

#include <algorithm>

namespace cthip {

bool dims_direct(const ct_dims& d) {
  for (int i = 0; i < d.ndim; ++i)
    if (d.index[i]) return false;
  return true;
}

// src/cortex/tensor/dimensions.clj:204-211
bool dims_access_increasing(const ct_dims& d) {
  if (!dims_direct(d)) return false;
  for (int i = 0; i + 1 < d.ndim; ++i)
    if (d.strides[i] < d.strides[i + 1]) return false;
  return true;
}

// src/cortex/tensor/dimensions.clj:178-191
bool dims_dense(const ct_dims& d) {
  if (!dims_direct(d)) return false;
  if (d.ndim == 1) return d.strides[0] == 1;
  struct SS { int64_t shape, stride; } v[CT_MAX_DIMS];
  int k = 0;
  for (int i = 0; i < d.ndim; ++i)
    if (d.shape[i] != 1) v[k++] = {d.shape[i], d.strides[i]};
  if (k == 0) return false;
  std::stable_sort(v, v + k, [](const SS& a, const SS& b) { return a.stride > b.stride; });
  int64_t rest = 1;
  for (int i = 1; i < k; ++i) rest *= v[i].shape;
  return v[0].stride == rest;
}

int64_t dims_ecount(const ct_dims& d) {
  int64_t n = 1;
  for (int i = 0; i < d.ndim; ++i) n *= d.shape[i];
  return n;
}

int check_dims(const ct_dims* d, const char* what) {
  CT_REQUIRE(d != nullptr, "%s: dimensions are null", what);
  CT_REQUIRE(d->ndim >= 1 && d->ndim <= CT_MAX_DIMS, "%s: rank %d outside 1..%d", what, d->ndim, CT_MAX_DIMS);
  for (int i = 0; i < d->ndim; ++i)
    CT_REQUIRE(d->shape[i] >= 1, "%s: shape[%d] = %lld must be >= 1", what, i, (long long)d->shape[i]);
  return CT_OK;
}

namespace {

struct Padded {  // slowest first, rank = max rank
  int64_t shape[CT_MAX_DIMS], stride[CT_MAX_DIMS];
  const int32_t* index[CT_MAX_DIMS];
};

// max-extend-strides (dimensions.clj:280-300)
void pad_dims(const ct_dims& d, int rank, Padded* p) {
  int mi = 0;
  for (int i = 1; i < d.ndim; ++i)
    if (d.strides[i] > d.strides[mi]) mi = i;
  const int64_t pad = d.strides[mi] * d.shape[mi];
  const int off = rank - d.ndim;
  for (int i = 0; i < off; ++i) { p->shape[i] = 1; p->stride[i] = pad; p->index[i] = nullptr; }
  for (int i = 0; i < d.ndim; ++i) {
    p->shape[off + i] = d.shape[i];
    p->stride[off + i] = d.strides[i];
    p->index[off + i] = d.index[i];
  }
}

// The CPU backend's choice of address object (cpu/tensor_math.clj:82-134).
void reference_mode(const ct_dims& d, const Padded& p, const int64_t* mx, int rank, GenOperand* g) {
  const bool dn = dims_dense(d), inc = dims_access_increasing(d), dir = dims_direct(d);
  const int64_t ec = dims_ecount(d);
  g->ec = ec;
  g->amt = 1;
  for (int i = 0; i < CT_MAX_DIMS; ++i) { g->shape[i] = 1; g->stride[i] = 0; g->index[i] = nullptr; }
  for (int i = 0; i < rank; ++i) {
    g->shape[i] = p.shape[rank - 1 - i];
    g->stride[i] = p.stride[rank - 1 - i];
    g->index[i] = p.index[rank - 1 - i];
  }
  bool same = d.ndim == rank;
  for (int i = 0; same && i < rank; ++i) same = d.shape[i] == mx[i];
  if (dir && same && dn && inc) { g->mode = 0; return; }
  int64_t biggest = 0;
  for (int i = 0; i < d.ndim; ++i) biggest = std::max(biggest, d.shape[i]);
  if (dir && ec == biggest && dn && inc) {
    int pos = -1;
    for (int i = 0; i < rank && pos < 0; ++i)
      if (p.shape[i] == ec) pos = i;
    int64_t amt = 1;
    for (int i = pos + 1; i < rank; ++i) amt *= mx[i];
    g->mode = 1;
    g->amt = amt;
    return;
  }
  if (dir && dn && inc) {
    int lead = 0;
    while (lead < d.ndim && d.shape[lead] == 1) ++lead;
    const int m = d.ndim - lead;
    bool suffix = m <= rank;
    for (int i = 0; suffix && i < m; ++i) suffix = d.shape[lead + i] == mx[rank - m + i];
    if (suffix) { g->mode = 2; return; }
  }
  g->mode = 3;
}

}  // namespace

int reference_operand(const ct_dims* d, const int64_t* max_shape, int rank, GenOperand* out, int64_t* rmax) {
  if (int rc = check_dims(d, "operand")) return rc;
  CT_REQUIRE(d->ndim <= rank && rank <= CT_MAX_DIMS, "internal: rank mismatch");
  Padded p;
  pad_dims(*d, rank, &p);
  reference_mode(*d, p, max_shape, rank, out);
  for (int i = 0; i < CT_MAX_DIMS; ++i) rmax[i] = i < rank ? max_shape[rank - 1 - i] : 1;
  return CT_OK;
}

int reference_operand_own(const ct_dims* d, GenOperand* out, int64_t* rmax, int* rank) {
  if (int rc = check_dims(d, "operand")) return rc;
  *rank = d->ndim;
  return reference_operand(d, d->shape, d->ndim, out, rmax);
}

int build_plan(const OperandIn* ops, int n_ops, int64_t n, Plan* plan, bool reference_order) {
  CT_REQUIRE(n_ops >= 1 && n_ops <= kMaxOps, "internal: operand count %d", n_ops);
  CT_REQUIRE(n >= 0, "element count %lld is negative", (long long)n);
  plan->n_ops = n_ops;
  plan->n = n;
  plan->tile_b = -1;
  for (int k = 0; k < kMaxOps; ++k) plan->via_lds[k] = false;

  int rank = 0;
  for (int k = 0; k < n_ops; ++k) {
    if (!ops[k].dims) continue;
    if (int rc = check_dims(ops[k].dims, k == 0 ? "dest" : "operand")) return rc;
    CT_REQUIRE(ops[k].ptr != nullptr, "operand %d: null buffer", k);
    rank = std::max(rank, (int)ops[k].dims->ndim);
  }
  CT_REQUIRE(ops[0].dims != nullptr, "internal: destination must be a tensor");

  Padded pd[kMaxOps];
  int64_t mx[CT_MAX_DIMS];
  for (int i = 0; i < rank; ++i) mx[i] = 1;
  for (int k = 0; k < n_ops; ++k) {
    if (!ops[k].dims) continue;
    pad_dims(*ops[k].dims, rank, &pd[k]);
    for (int i = 0; i < rank; ++i) mx[i] = std::max(mx[i], pd[k].shape[i]);
  }

  // ---- regular: direct, pure (1-or-full) broadcasting, destination full, n covers the space once
  bool regular = !reference_order;
  int64_t total = 1;
  for (int i = 0; i < rank; ++i) total *= mx[i];
  if (total != n) regular = false;
  for (int k = 0; regular && k < n_ops; ++k) {
    if (!ops[k].dims) continue;
    for (int i = 0; regular && i < rank; ++i) {
      // an indexed axis stays regular only as a full axis of more than one entry (the vector
      // kernel's row gather / scatter); anything else goes to the reference's address objects
      if (pd[k].index[i] && (pd[k].shape[i] != mx[i] || mx[i] == 1)) regular = false;
      else if (pd[k].shape[i] != mx[i] && pd[k].shape[i] != 1) regular = false;
      else if (pd[k].shape[i] != 1 && pd[k].stride[i] < 0) regular = false;
      else if (k == 0 && pd[k].shape[i] != mx[i]) regular = false;
    }
  }
  plan->regular = regular;

  // `regular` may be withdrawn below (indexed axes that the vector kernel cannot take); the loop
  // runs once.
  while (regular) {
    Canon& c = plan->canon;
    c.nd = 0;
    c.any_index = false;
    for (int i = rank - 1; i >= 0; --i) {
      if (mx[i] == 1) continue;
      c.size[c.nd] = mx[i];
      for (int k = 0; k < n_ops; ++k) {
        c.stride[k][c.nd] = (!ops[k].dims || pd[k].shape[i] == 1) ? 0 : pd[k].stride[i];
        c.index[k][c.nd] = ops[k].dims ? pd[k].index[i] : nullptr;
        if (c.index[k][c.nd]) c.any_index = true;
      }
      ++c.nd;
    }
    if (c.nd == 0) {  // a single element
      c.nd = 1;
      c.size[0] = 1;
      for (int k = 0; k < n_ops; ++k) { c.stride[k][0] = ops[k].dims ? 1 : 0; c.index[k][0] = nullptr; }
    }
    // order axes by destination stride (stable insertion sort)
    for (int i = 1; i < c.nd; ++i)
      for (int j = i; j > 0 && c.stride[0][j - 1] > c.stride[0][j]; --j) {
        std::swap(c.size[j - 1], c.size[j]);
        for (int k = 0; k < n_ops; ++k) {
          std::swap(c.stride[k][j - 1], c.stride[k][j]);
          std::swap(c.index[k][j - 1], c.index[k][j]);
        }
      }
    // merge axis j into axis j-1 when every operand's strides chain (an indexed axis never merges)
    int w = 0;
    for (int j = 1; j < c.nd; ++j) {
      bool chain = true;
      for (int k = 0; chain && k < n_ops; ++k)
        chain = c.stride[k][j] == c.stride[k][w] * c.size[w] && !c.index[k][j] && !c.index[k][w];
      if (chain) {
        c.size[w] *= c.size[j];
      } else {
        ++w;
        c.size[w] = c.size[j];
        for (int k = 0; k < n_ops; ++k) { c.stride[k][w] = c.stride[k][j]; c.index[k][w] = c.index[k][j]; }
      }
    }
    c.nd = w + 1;
    // indexed axes must be among the first two outer axes, never the innermost
    bool index_ok = true;
    for (int k = 0; k < n_ops; ++k)
      for (int i = 0; i < c.nd; ++i)
        if (c.index[k][i] && (i == 0 || i > 2)) index_ok = false;
    if (!index_ok) { regular = false; plan->regular = false; break; }

    // ---- classify
    bool fits32 = n < (int64_t(1) << 31);
    for (int i = 0; i < c.nd; ++i)
      if (c.size[i] >= (int64_t(1) << 31)) fits32 = false;
    if (c.stride[0][0] == 1 && (fits32 || c.nd == 1)) {
      bool all_unit = true;
      for (int k = 1; k < n_ops; ++k)
        if (c.stride[k][0] != 0 && c.stride[k][0] != 1) all_unit = false;
      if (all_unit) { plan->kind = PK_VEC; return CT_OK; }
      if (fits32 && !c.any_index) {
        int b = -1;
        bool ok = true;
        for (int k = 1; ok && k < n_ops; ++k) {
          if (c.stride[k][0] == 0 || c.stride[k][0] == 1) continue;
          int kb = -1;
          for (int i = 1; i < c.nd; ++i)
            if (c.stride[k][i] == 1) { kb = i; break; }
          if (kb < 0 || (b >= 0 && kb != b)) ok = false;
          else { b = kb; plan->via_lds[k] = true; }
        }
        if (ok && b >= 0 && c.size[0] >= 16 && c.size[b] >= 16) {
          plan->kind = PK_TILE;
          plan->tile_b = b;
          return CT_OK;
        }
        for (int k = 0; k < kMaxOps; ++k) plan->via_lds[k] = false;
      }
    }
    if (c.any_index) { regular = false; plan->regular = false; break; }
    // regular but neither vectorisable nor tileable: per-element addressing
    // over the merged axes
    plan->kind = PK_GENERAL;
    GenPlan& g = plan->gen;
    g.nd = c.nd;
    for (int i = 0; i < CT_MAX_DIMS; ++i) g.rmax[i] = i < c.nd ? c.size[i] : 1;
    for (int k = 0; k < n_ops; ++k) {
      GenOperand& o = g.op[k];
      o.mode = ops[k].dims ? 3 : 4;
      o.ec = 1;
      o.amt = 1;
      for (int i = 0; i < CT_MAX_DIMS; ++i) {
        o.shape[i] = (i < c.nd && c.stride[k][i] != 0) ? c.size[i] : 1;
        o.stride[i] = i < c.nd ? c.stride[k][i] : 0;
        o.index[i] = nullptr;
      }
      // an axis of size 1 in the operand never contributes
    }
    return CT_OK;
  }

  // ---- irregular: the reference's own address objects, dimension by dimension
  plan->kind = PK_GENERAL;
  GenPlan& g = plan->gen;
  g.nd = rank;
  for (int i = 0; i < CT_MAX_DIMS; ++i) g.rmax[i] = i < rank ? mx[rank - 1 - i] : 1;
  for (int k = 0; k < n_ops; ++k) {
    if (!ops[k].dims) {
      GenOperand& o = g.op[k];
      o.mode = 4;
      o.ec = o.amt = 1;
      for (int i = 0; i < CT_MAX_DIMS; ++i) { o.shape[i] = 1; o.stride[i] = 0; o.index[i] = nullptr; }
      continue;
    }
    reference_mode(*ops[k].dims, pd[k], mx, rank, &g.op[k]);
  }
  return CT_OK;
}

}  // namespace cthip
