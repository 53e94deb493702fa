// ops_accum.hip -- binary-accum! (src/cortex/tensor/math.clj:53-65;
// src/cortex/compute/cpu/tensor_math.clj:386-420, 1439-1463).
//
//   dest[Ad(e)] = dest[Ad(e)]*dest_alpha op y[Ay(e)]*y_alpha     for e = 0 .. n-1
//
// Without dest_requires_cas every destination element is written once and the
// call is an ordinary in-place binary-op!.  With it, the destination is
// smaller than the operation (a broadcast target: "sum the rows into a
// vector", bias gradients) or indirectly indexed (scatter-add), so several e
// hit one address and the reference applies them serially in increasing e,
// rounding to the tensor datatype after every update.
//
// accum_owner_kernel reproduces exactly that for broadcast destinations:
// one lane owns one destination element and applies its updates in increasing
// e, so the result is bit-identical to the serial loop while all destination
// elements proceed in parallel.  For op :+ with dest_alpha 1 and enough updates
// per destination element (bias gradients: [k] <- [b,k], [C,1,1] <- [N,C,H,W])
// the call instead runs as sum reductions of y over the broadcast axes into a
// stream-owned temporary, innermost group of axes first, followed by one
// in-place add into the destination: every pass streams at the reduce kernels'
// rate.  Integer results are unchanged by that (sums wrap modulo 2^bits either
// way); float/double results are sums formed in double, closer to the exact sum
// than the reference's value-by-value accumulation (which the reference itself
// only checks to 1e-4, src/cortex/verify/tensor.clj:188-191).
//
// Indirectly indexed destinations (scatter-add of rows through a label tensor,
// src/cortex/loss/center.clj:92; src/cortex/verify/tensor.clj:1162-1174): two
// updates collide exactly when their coordinates along the indexed axis name
// the same index value and all other coordinates agree.  The positions of the
// index tensor are sorted by value, stably, so the positions of one value are
// adjacent and still in increasing order; then one lane per (value, element of
// the remaining axes) applies that destination element's updates in increasing
// position, which is increasing e: accum_grouped_kernel.  Bit-identical to the
// serial loop for every op.  Up to 8192 index entries are ranked by one small
// kernel; longer index tensors go through the vendor sort (rocPRIM's
// radix_sort_pairs, stable, the positions fed from a counting iterator).  Shapes outside that pattern (reduced axes next to an
// indexed one, an indexed y) keep the serial kernel.
#include <algorithm>

#include "elementwise.h"
#include "functors.h"
#include "ops.h"

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/iterator/counting_iterator.hpp>

using namespace cthip;

namespace {

struct OwnerArgs {
  void* dest;
  const void* y;
  int64_t n_dest;   // destination elements (owners)
  int64_t n_red;    // updates per destination element
  int32_t n_kept, n_redax;
  FastDiv ksize[CT_MAX_DIMS];   // kept axes, fastest first
  int64_t kd_stride[CT_MAX_DIMS], ky_stride[CT_MAX_DIMS];
  FastDiv rsize[CT_MAX_DIMS];   // reduced axes, fastest first
  int64_t ry_stride[CT_MAX_DIMS];
  int32_t reverse;
  // STAGED form: `reduced` holds, per destination element, the reduction of its updates
  // (unary-reduce! :max / :min of y * y_alpha), addressed through kt_stride per kept axis
  const void* reduced;
  int64_t kt_stride[CT_MAX_DIMS];
};

// STAGED (:max and :min with dest_alpha 1): the updates of every destination element have
// already been reduced, with java.lang.Math.max / min, into a.reduced.  Where that value is
// an ordinary non-zero number it is also what the serial chain of (x > y ? x : y) steps leaves
// (equal non-zero values are the same bits, so which of them a tie keeps does not show), and
// one step with it finishes the element; f_unit is f with the update's multiplier set to 1,
// since the reduction has applied it.  Where it is a NaN or a zero the chain's outcome depends
// on the order of the updates (a NaN restarts or freezes it, and +0 against -0 is a tie that
// the later or the earlier operand wins), and the lane walks the updates as the serial loop does.
template <class T, int OP, bool STAGED>
__global__ void __launch_bounds__(kBlock) accum_owner_kernel(const BinaryF<T, OP> f, const BinaryF<T, OP> f_unit,
                                                             const OwnerArgs a) {
  const int64_t t = (int64_t)blockIdx.x * kBlock + threadIdx.x;
  if (t >= a.n_dest) return;
  int64_t doff = 0, ybase = 0, toff = 0;
  uint32_t rem = (uint32_t)t;
  for (int d = 0; d < a.n_kept; ++d) {
    uint32_t q, r;
    a.ksize[d].divmod(rem, q, r);
    rem = q;
    doff += (int64_t)r * a.kd_stride[d];
    ybase += (int64_t)r * a.ky_stride[d];
    if constexpr (STAGED) toff += (int64_t)r * a.kt_stride[d];
  }
  T* dp = reinterpret_cast<T*>(a.dest) + doff;
  const T* yp = reinterpret_cast<const T*>(a.y) + ybase;
  T acc = *dp;
  if constexpr (STAGED) {
    const T red = reinterpret_cast<const T*>(a.reduced)[toff];
    bool ordinary = true;
    if constexpr (std::is_floating_point<T>::value) ordinary = red == red && red != (T)0;
    if (ordinary) {
      *dp = a.reverse ? f_unit(red, acc, acc) : f_unit(acc, red, red);
      return;
    }
  }
  uint32_t i = 0;
  if (a.n_redax == 1) {
    // one broadcast axis: fetch thirty-two updates ahead, apply them in order (the calls that reach
    // this kernel have short chains: a bias gradient of ten classes over a batch of 128 is four
    // trips to memory this way instead of sixteen)
    constexpr int UN = 32;
    const int64_t st = a.ry_stride[0];
    for (; i + UN <= (uint32_t)a.n_red; i += UN) {
      T yv[UN];
#pragma unroll
      for (int j = 0; j < UN; ++j) yv[j] = yp[(int64_t)(i + j) * st];
#pragma unroll
      for (int j = 0; j < UN; ++j) acc = a.reverse ? f(yv[j], acc, acc) : f(acc, yv[j], yv[j]);
    }
  }
  for (; i < (uint32_t)a.n_red; ++i) {
    int64_t yoff = 0;
    uint32_t rr = i;
    for (int d = 0; d < a.n_redax; ++d) {
      uint32_t q, r;
      a.rsize[d].divmod(rr, q, r);
      rr = q;
      yoff += (int64_t)r * a.ry_stride[d];
    }
    const T yv = yp[yoff];
    acc = a.reverse ? f(yv, acc, acc) : f(acc, yv, yv);
  }
  *dp = acc;
}

// Splits the joint iteration space into axes the destination keeps and axes it
// broadcasts over.  Fails (returns false) unless both operands are direct,
// every axis of either operand is 1 or the full size, and n covers the space.
bool owner_structure(const ct_dims& dd, const ct_dims& yd, int64_t n, OwnerArgs* a) {
  if (!dims_direct(dd) || !dims_direct(yd)) return false;
  const int rank = std::max(dd.ndim, yd.ndim);
  int64_t dshape[CT_MAX_DIMS], dstr[CT_MAX_DIMS], yshape[CT_MAX_DIMS], ystr[CT_MAX_DIMS], mx[CT_MAX_DIMS];
  for (int i = 0; i < rank; ++i) {
    const int di = i - (rank - dd.ndim), yi = i - (rank - yd.ndim);
    dshape[i] = di >= 0 ? dd.shape[di] : 1;
    dstr[i] = di >= 0 ? dd.strides[di] : 0;
    yshape[i] = yi >= 0 ? yd.shape[yi] : 1;
    ystr[i] = yi >= 0 ? yd.strides[yi] : 0;
    mx[i] = std::max(dshape[i], yshape[i]);
  }
  int64_t total = 1, n_dest = 1, n_red = 1;
  a->n_kept = a->n_redax = 0;
  for (int i = rank - 1; i >= 0; --i) {  // fastest first
    if (mx[i] >= (int64_t(1) << 31)) return false;
    total *= mx[i];
    if (mx[i] == 1) continue;
    if ((dshape[i] != 1 && dshape[i] != mx[i]) || (yshape[i] != 1 && yshape[i] != mx[i])) return false;
    const int64_t ys = yshape[i] == 1 ? 0 : ystr[i];
    if (dstr[i] < 0) return false;
    // a destination axis of stride 0 addresses like a broadcast one: every coordinate is one element
    if (dshape[i] == mx[i] && dstr[i] != 0) {
      a->ksize[a->n_kept] = FastDiv((uint32_t)mx[i]);
      a->kd_stride[a->n_kept] = dstr[i];
      a->ky_stride[a->n_kept] = ys;
      ++a->n_kept;
      n_dest *= mx[i];
    } else {
      a->rsize[a->n_redax] = FastDiv((uint32_t)mx[i]);
      a->ry_stride[a->n_redax] = ys;
      ++a->n_redax;
      n_red *= mx[i];
    }
  }
  if (total != n || n_dest >= (int64_t(1) << 31) || n_red >= (int64_t(1) << 31)) return false;
  if (a->n_redax == 0) { a->rsize[0] = FastDiv(1); a->ry_stride[0] = 0; a->n_redax = 1; }
  a->n_dest = n_dest;
  a->n_red = n_red;
  // two owners must never share an address: sorted by stride, each kept axis
  // has to step over everything the faster ones cover
  int order[CT_MAX_DIMS];
  for (int i = 0; i < a->n_kept; ++i) order[i] = i;
  std::sort(order, order + a->n_kept, [&](int l, int r) { return a->kd_stride[l] < a->kd_stride[r]; });
  int64_t span = 1;
  for (int i = 0; i < a->n_kept; ++i) {
    if (a->kd_stride[order[i]] < span) return false;
    span = a->kd_stride[order[i]] * ((int64_t)a->ksize[order[i]].d - 1) + span;
  }
  return true;
}

// Whether the streamed form (ops_accum_stream.hip) takes this call, and its description if so.
// It wants long chains (the owner kernel above is at its best with many short ones: a lane per
// chain is then enough lanes, and neighbouring lanes read neighbouring addresses), y on the
// 16-byte grid, and one of two arrangements: the chains unit-stride in y under one (merged)
// broadcast axis, or the steps unit-stride in y under at most one further broadcast axis.
constexpr int64_t kStreamMinSteps = 128;
constexpr int64_t kStreamMaxChains = int64_t(1) << 18;

template <class T> bool stream_structure(const OwnerArgs& a, AccumStreamCall* c) {
  constexpr int VEC = 16 / (int)sizeof(T);
  if (a.n_red < kStreamMinSteps || a.n_dest > kStreamMaxChains) return false;
  if (((uintptr_t)a.y % 16) != 0) return false;
  // broadcast axes, fastest first, neighbours that chain merged
  int64_t rs[CT_MAX_DIMS], rst[CT_MAX_DIMS];
  int nr = 0;
  for (int d = 0; d < a.n_redax; ++d) {
    const int64_t size = a.rsize[d].d, st = a.ry_stride[d];
    if (size == 1) continue;
    if (st < 0) return false;
    if (nr > 0 && st == rst[nr - 1] * rs[nr - 1]) rs[nr - 1] *= size;
    else { rs[nr] = size; rst[nr] = st; ++nr; }
  }
  if (nr == 0 || nr > 2) return false;
  std::memset(c, 0, sizeof(*c));
  c->dest = a.dest;
  c->y = a.y;
  c->n_red = a.n_red;
  int strip = -1;
  if (nr == 1 && rst[0] != 1) {
    // chains unit-stride
    for (int d = 0; d < a.n_kept; ++d)
      if (a.ky_stride[d] == 1) strip = d;
    if (strip < 0 || a.ksize[strip].d % VEC != 0 || rst[0] % VEC != 0) return false;
    c->steps_unit_stride = false;
    c->pitch = rst[0];
  } else {
    // steps unit-stride; the strip runs along the kept axis whose chains lie closest in y
    if (rst[0] != 1 || rs[0] % VEC != 0) return false;
    if (nr == 2 && rst[1] % VEC != 0) return false;
    for (int d = 0; d < a.n_kept; ++d)
      if (a.ky_stride[d] < 0) return false;
      else if (strip < 0 || a.ky_stride[d] < a.ky_stride[strip]) strip = d;
    if (strip >= 0 && a.ky_stride[strip] % VEC != 0) return false;
    c->steps_unit_stride = true;
    c->pitch = strip >= 0 ? a.ky_stride[strip] : 0;
    c->n_inner = rs[0];
    c->outer_stride = nr == 2 ? rst[1] : 0;
  }
  c->u = strip >= 0 ? (int64_t)a.ksize[strip].d : 1;
  c->d_ustride = strip >= 0 ? a.kd_stride[strip] : 0;
  for (int d = 0; d < a.n_kept; ++d) {
    if (d == strip) continue;
    if (a.ky_stride[d] < 0 || a.ky_stride[d] % VEC != 0) return false;
    c->rsize[c->n_rest] = a.ksize[d].d;
    c->rd_stride[c->n_rest] = a.kd_stride[d];
    c->ry_stride[c->n_rest] = a.ky_stride[d];
    ++c->n_rest;
  }
  return true;
}

// ------------------------------------------------------------------ indexed destinations

struct GroupedArgs {
  void* dest;
  const void* y;
  const int32_t* skey;   // index values, sorted
  const int32_t* perm;   // the position each sorted entry came from
  uint32_t n_index;      // entries of the index tensor
  uint32_t kept_vecs;    // vectors of the remaining axes per index entry
  uint32_t lane_vecs;    // lanes per index entry: kept_vecs, or half of it (rounded up) with two vectors per lane
  FastDiv lane_fd;       // lane_vecs
  int64_t d_gstride, y_gstride;  // strides of the indexed axis
  int32_t n_kept;
  FastDiv ksize[CT_MAX_DIMS];    // remaining axes, fastest first (axis 0 counted in vectors)
  int64_t kd_stride[CT_MAX_DIMS], ky_stride[CT_MAX_DIMS];
  int32_t reverse;
};

// rank[i] = number of entries that sort before entry i, where entries are ordered by
// (value bits, position): a stable counting rank, quadratic but one short launch.  Entry i is
// then stored at its rank.  (Any total order on the values will do: equal values must end up
// adjacent and in increasing position, nothing more.)  One wave per entry: its lanes walk the
// index tensor 64 entries at a time (coalesced; the tensor is a few KiB and stays cached),
// each lane counts the entries that precede i among those it sees, and the lanes' counts
// meet in a shuffle sum.
constexpr uint32_t kRankMaxEntries = 8192;
__global__ void __launch_bounds__(kBlock) index_rank_kernel(const int32_t* __restrict__ index, uint32_t n,
                                                            int32_t* __restrict__ skey, int32_t* __restrict__ perm) {
  const uint32_t lane = threadIdx.x & 63u;
  const uint32_t i = blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  if (i >= n) return;
  const int32_t mine = index[i];
  const uint64_t mine64 = ((uint64_t)(uint32_t)mine << 32) | i;
  uint32_t count = 0;
  uint32_t j = lane;
  for (; j + 3 * 64 < n; j += 4 * 64) {
    const int32_t v0 = index[j], v1 = index[j + 64], v2 = index[j + 128], v3 = index[j + 192];
    count += (((uint64_t)(uint32_t)v0 << 32) | j) < mine64 ? 1u : 0u;
    count += (((uint64_t)(uint32_t)v1 << 32) | (j + 64)) < mine64 ? 1u : 0u;
    count += (((uint64_t)(uint32_t)v2 << 32) | (j + 128)) < mine64 ? 1u : 0u;
    count += (((uint64_t)(uint32_t)v3 << 32) | (j + 192)) < mine64 ? 1u : 0u;
  }
  for (; j < n; j += 64) count += (((uint64_t)(uint32_t)index[j] << 32) | j) < mine64 ? 1u : 0u;
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) count += __shfl_xor(count, m, 64);
  if (lane == 0) {
    skey[count] = mine;
    perm[count] = (int32_t)i;
  }
}

// One lane per (sorted index entry, PER vectors of the remaining axes, lane_vecs apart).  A lane
// whose entry is not the first of its value leaves at once; the first walks the run of equal
// values, fetching kAhead updates before it applies them in order.  PER = 2 puts twice the bytes
// behind one look-up of the sorted entries.
template <class T, int OP, int VEC, int PER>
__global__ void __launch_bounds__(kBlock) accum_grouped_kernel(const BinaryF<T, OP> f, const GroupedArgs a) {
  using V = Vec<T, VEC>;
  const uint64_t t = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
  if (t >= (uint64_t)a.n_index * a.lane_vecs) return;
  uint32_t i, kv;
  if (a.lane_vecs >= 1u << 31 || t >= (uint64_t(1) << 32)) {
    i = (uint32_t)(t / a.lane_vecs);
    kv = (uint32_t)(t % a.lane_vecs);
  } else {
    a.lane_fd.divmod((uint32_t)t, i, kv);
  }
  // The first kAhead sorted entries and their positions are fetched before the run's extent
  // is known, so that a run of up to kAhead updates costs two dependent trips to memory
  // (entries, then updates) instead of three.
  constexpr int kAhead = 4;
  int32_t ks[kAhead], ps[kAhead];
#pragma unroll
  for (int u = 0; u < kAhead; ++u) {
    const uint32_t at = i + u < a.n_index ? i + u : a.n_index - 1;
    ks[u] = a.skey[at];
    ps[u] = a.perm[at];
  }
  const int32_t before = a.skey[i > 0 ? i - 1 : 0];
  const int32_t key = ks[0];
  if (i > 0 && before == key) return;
  V* dp[PER];
  const T* yb[PER];
  bool live[PER];
  V acc[PER];
#pragma unroll
  for (int h = 0; h < PER; ++h) {
    uint32_t rem = kv + (uint32_t)h * a.lane_vecs;
    live[h] = h == 0 || rem < a.kept_vecs;
    int64_t doff = (int64_t)key * a.d_gstride, yoff = 0;
    for (int d = 0; d < a.n_kept; ++d) {
      uint32_t q, r;
      a.ksize[d].divmod(rem, q, r);
      rem = q;
      const int64_t c = d == 0 ? (int64_t)r * VEC : (int64_t)r;
      doff += c * a.kd_stride[d];
      yoff += c * a.ky_stride[d];
    }
    dp[h] = reinterpret_cast<V*>(reinterpret_cast<T*>(a.dest) + doff);
    yb[h] = reinterpret_cast<const T*>(a.y) + yoff;
    if (live[h]) acc[h] = *dp[h];
  }
  const bool y_unit = a.ky_stride[0] == 1 || VEC == 1;
  const bool y_once = a.y_gstride != 0;  // every update is read by one lane only
  uint32_t j = i;
  for (;;) {
    V upd[kAhead][PER];
    int cnt = 0;
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      if (cnt == u && j + u < a.n_index && ks[u] == key) {
#pragma unroll
        for (int h = 0; h < PER; ++h) {
          if (!live[h]) continue;
          const T* yp = yb[h] + (int64_t)ps[u] * a.y_gstride;
          if (y_unit) {
            upd[u][h] = y_once ? nt_load(reinterpret_cast<const V*>(yp)) : *reinterpret_cast<const V*>(yp);
          } else {  // y broadcast along the vectorised axis
            const T yv = *yp;
#pragma unroll
            for (int e = 0; e < VEC; ++e) upd[u][h].v[e] = yv;
          }
        }
        cnt = u + 1;
      }
    }
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      if (u < cnt) {
#pragma unroll
        for (int h = 0; h < PER; ++h) {
          if (!live[h]) continue;
#pragma unroll
          for (int e = 0; e < VEC; ++e)
            acc[h].v[e] = a.reverse ? f(upd[u][h].v[e], acc[h].v[e], acc[h].v[e]) : f(acc[h].v[e], upd[u][h].v[e], upd[u][h].v[e]);
        }
      }
    }
    if (cnt < kAhead) break;
    j += kAhead;
#pragma unroll
    for (int u = 0; u < kAhead; ++u) {
      const uint32_t at = j + u < a.n_index ? j + u : a.n_index - 1;
      ks[u] = a.skey[at];
      ps[u] = a.perm[at];
    }
  }
#pragma unroll
  for (int h = 0; h < PER; ++h)
    if (live[h]) *dp[h] = acc[h];
}

// Recognises "one indexed axis in the destination, every other axis kept, y direct".
// Fills everything of GroupedArgs except the sorted index and the pointers; *index_out is the
// destination's index tensor, *vec_ok whether axis 0 may be walked in 16-byte vectors.
template <class T>
bool grouped_structure(const ct_dims& dd, const ct_dims& yd, const void* dest, const void* y, int64_t n, GroupedArgs* a,
                       const int32_t** index_out, bool* vec_ok) {
  if (!dims_direct(yd)) return false;
  const int rank = std::max(dd.ndim, yd.ndim);
  int gi = -1;
  struct Ax { int64_t size, ds, ys; } kept[CT_MAX_DIMS];
  int nk = 0;
  int64_t total = 1;
  for (int i = rank - 1; i >= 0; --i) {  // fastest first
    const int di = i - (rank - dd.ndim), yi = i - (rank - yd.ndim);
    const int64_t dshape = di >= 0 ? dd.shape[di] : 1, dstr = di >= 0 ? dd.strides[di] : 0;
    const int64_t yshape = yi >= 0 ? yd.shape[yi] : 1, ystr = yi >= 0 ? yd.strides[yi] : 0;
    const int32_t* idx = di >= 0 ? dd.index[di] : nullptr;
    const int64_t mx = std::max(dshape, yshape);
    if (mx >= (int64_t(1) << 31)) return false;
    total *= mx;
    if (idx) {
      if (gi >= 0 || dshape != mx || (yshape != 1 && yshape != mx)) return false;
      gi = i;
      a->n_index = (uint32_t)dshape;
      a->d_gstride = dstr;
      a->y_gstride = yshape == 1 ? 0 : ystr;
      *index_out = idx;
      continue;
    }
    if (mx == 1) continue;
    if (dshape != mx || dstr <= 0 || (yshape != 1 && yshape != mx)) return false;
    kept[nk++] = Ax{mx, dstr, yshape == 1 ? 0 : ystr};
  }
  if (gi < 0 || total != n) return false;
  // Kept axes must not overlap one another in the destination, and rows selected by different index
  // values must not share addresses either (different lanes own them): the kept axes that are finer
  // than the indexed axis have to fit inside one step of it.  A view whose rows overlap (a sliding
  // window, a non-positive row stride) keeps the serial kernel, which applies the updates one by one.
  // Kept axes coarser than the indexed axis are taken at their word: index values address the extent
  // of their own dimension, which lies inside one step of the next coarser axis in any dense layout.
  {
    if (a->d_gstride <= 0) return false;
    int order[CT_MAX_DIMS];
    for (int i = 0; i < nk; ++i) order[i] = i;
    std::sort(order, order + nk, [&](int l, int r) { return kept[l].ds < kept[r].ds; });
    int64_t span = 1;
    bool indexed_placed = false;
    for (int i = 0; i < nk; ++i) {
      if (!indexed_placed && kept[order[i]].ds >= a->d_gstride) {
        if (a->d_gstride < span) return false;
        indexed_placed = true;
      }
      if (kept[order[i]].ds < span) return false;
      span = kept[order[i]].ds * (kept[order[i]].size - 1) + span;
    }
    if (!indexed_placed && a->d_gstride < span) return false;
  }
  if (nk == 0) kept[nk++] = Ax{1, 1, 1};
  constexpr int VMAX = 16 / (int)sizeof(T);
  bool v = VMAX > 1 && kept[0].ds == 1 && (kept[0].ys == 1 || kept[0].ys == 0) && kept[0].size % VMAX == 0 &&
           a->d_gstride % VMAX == 0 && a->y_gstride % VMAX == 0 && ((uintptr_t)dest % 16) == 0 && ((uintptr_t)y % 16) == 0;
  for (int i = 1; v && i < nk; ++i) v = kept[i].ds % VMAX == 0 && kept[i].ys % VMAX == 0;
  *vec_ok = v;
  const int vec = v ? VMAX : 1;
  int64_t kv = 1;
  a->n_kept = nk;
  for (int i = 0; i < nk; ++i) {
    const int64_t sz = i == 0 ? kept[i].size / vec : kept[i].size;
    a->ksize[i] = FastDiv((uint32_t)sz);
    a->kd_stride[i] = kept[i].ds;
    a->ky_stride[i] = kept[i].ys;
    kv *= sz;
  }
  if (kv >= (int64_t(1) << 31)) return false;
  a->kept_vecs = (uint32_t)kv;
  a->lane_vecs = (uint32_t)kv;
  a->lane_fd = FastDiv((uint32_t)kv);
  return ((int64_t)a->n_index * kv + kBlock - 1) / kBlock < (int64_t(1) << 31);
}

// Sorts the index tensor's positions by value (stable) into the stream's scratch.
int sort_index(hipStream_t s, const int32_t* index, uint32_t n, const int32_t** skey, const int32_t** perm) {
  void* block = nullptr;
  if (n <= kRankMaxEntries) {
    if (int rc = stream_scratch(s, (size_t)n * 8, &block, kScratchAccumA)) return rc;
    int32_t* k = static_cast<int32_t*>(block);
    hipLaunchKernelGGL(index_rank_kernel, dim3((n + kBlock / 64 - 1) / (kBlock / 64)), dim3(kBlock), 0, s, index, n, k, k + n);
    *skey = k;
    *perm = k + n;
    return CT_OK;
  }
  // the positions come from a counting iterator, so no array of them has to be written first
  size_t temp_bytes = 0;
  const size_t arrays = ((size_t)n * 4 + 255) / 256 * 256;
  const rocprim::counting_iterator<int32_t> positions(0);
  CT_HIP(rocprim::radix_sort_pairs(nullptr, temp_bytes, index, (int32_t*)nullptr, positions, (int32_t*)nullptr, n, 0u, 32u, s));
  if (int rc = stream_scratch(s, 2 * arrays + temp_bytes, &block, kScratchAccumA)) return rc;
  char* base = static_cast<char*>(block);
  int32_t* k = reinterpret_cast<int32_t*>(base);
  int32_t* p = reinterpret_cast<int32_t*>(base + arrays);
  CT_HIP(rocprim::radix_sort_pairs(base + 2 * arrays, temp_bytes, index, k, positions, p, n, 0u, 32u, s));
  *skey = k;
  *perm = p;
  return CT_OK;
}

struct StageAxis {
  int64_t size, ystride, dstride;
  bool kept;
  int id;  // kept axes: position in OwnerArgs::ksize
};

constexpr int64_t kStagedMinUpdates = 64;     // per destination element
constexpr int64_t kStagedMinElements = 1024;   // of y
constexpr int64_t kStagedShortGroup = 64;      // a first pass over rows shorter than this is avoided

// Merges neighbouring kept axes of a pass (all but the last, reduced one) that chain in the input
// and in the output alike, so that the reduction sees [512, 49, 256] rather than [512, 7, 7, 256].
void merge_chained(ct_dims* id, ct_dims* od) {
  const int last = id->ndim - 1;
  int w = 0;
  for (int i = 0; i < last; ++i) {
    if (w > 0 && id->strides[w - 1] == id->strides[i] * id->shape[i] && od->strides[w - 1] == od->strides[i] * od->shape[i]) {
      id->shape[w - 1] *= id->shape[i];
      od->shape[w - 1] = id->shape[w - 1];
      id->strides[w - 1] = id->strides[i];
      od->strides[w - 1] = od->strides[i];
    } else {
      id->shape[w] = id->shape[i]; id->strides[w] = id->strides[i];
      od->shape[w] = od->shape[i]; od->strides[w] = od->strides[i];
      ++w;
    }
  }
  id->shape[w] = id->shape[last]; id->strides[w] = id->strides[last];
  od->shape[w] = od->shape[last]; od->strides[w] = od->strides[last];
  id->ndim = od->ndim = w + 1;
}

// Reduces y * y_alpha over the broadcast axes with unary-reduce! `rop`, innermost group of
// axes first, through the stream's two accumulate scratch blocks.  On success *result is the
// last temporary (one value per destination element) and ax[0..*nax) the kept axes, slowest
// first, with .ystride the temporary's stride.  *handled is false (and nothing ran) when y
// is itself broadcast along some axis.
int stage_reduce(hipStream_t s, const OwnerArgs& a, double y_alpha, int dtype, size_t elem_bytes, int rop,
                 bool* handled, const void** result, StageAxis* ax, int* nax_out, bool add_into_dest = false) {
  *handled = false;
  int nax = 0;
  for (int d = 0; d < a.n_kept; ++d) {
    if (a.ky_stride[d] <= 0) return CT_OK;
    ax[nax++] = StageAxis{(int64_t)a.ksize[d].d, a.ky_stride[d], a.kd_stride[d], true, d};
  }
  for (int d = 0; d < a.n_redax; ++d) {
    if (a.rsize[d].d == 1) continue;
    if (a.ry_stride[d] <= 0) return CT_OK;
    ax[nax++] = StageAxis{(int64_t)a.rsize[d].d, a.ry_stride[d], 0, false, -1};
  }
  if (nax > CT_MAX_DIMS) return CT_OK;
  std::sort(ax, ax + nax, [](const StageAxis& l, const StageAxis& r) { return l.ystride > r.ystride; });  // slowest first
  *handled = true;

  const void* cur = a.y;
  double alpha = y_alpha;
  int slot = kScratchAccumA;
  for (;;) {
    // innermost reduced axis, merged with the reduced axes that chain onto it
    int g = -1;
    for (int i = nax - 1; i >= 0; --i)
      if (!ax[i].kept) { g = i; break; }
    if (g < 0) break;
    int64_t gsize = ax[g].size;
    int64_t gstride = ax[g].ystride;
    bool taken[CT_MAX_DIMS] = {false};
    taken[g] = true;
    for (int i = g - 1; i >= 0; --i) {
      if (ax[i].kept) continue;
      if (ax[i].ystride != gstride * gsize) break;
      gsize *= ax[i].size;
      taken[i] = true;
    }
    // A short innermost group (the 49 pixels of a 7 x 7 image under a per-channel sum) makes a
    // poor first pass: rows of a few elements, seldom a whole number of vectors.  When a slower
    // broadcast axis is left (the batch), that one goes first instead: a reduction down the
    // columns of long contiguous rows, after which the short rows are a small tensor.
    if (gsize < kStagedShortGroup) {
      int outer = -1;
      for (int i = 0; i < nax; ++i)
        if (!ax[i].kept && !taken[i]) { outer = i; break; }
      if (outer >= 0) {
        for (int i = 0; i < nax; ++i) taken[i] = false;
        taken[outer] = true;
        gsize = ax[outer].size;
        gstride = ax[outer].ystride;
      }
    }
    ct_dims id, od;
    std::memset(&id, 0, sizeof(id));
    std::memset(&od, 0, sizeof(od));
    StageAxis rest[CT_MAX_DIMS];
    int nrest = 0;
    for (int i = 0; i < nax; ++i)
      if (!taken[i]) rest[nrest++] = ax[i];
    int64_t n_out = 1;
    for (int i = 0; i < nrest; ++i) n_out *= rest[i].size;
    int64_t mul = 1;
    for (int i = nrest - 1; i >= 0; --i) {
      id.shape[i] = od.shape[i] = rest[i].size;
      id.strides[i] = rest[i].ystride;
      od.strides[i] = mul;
      rest[i].ystride = mul;  // the layout of the temporary the next pass reads
      mul *= rest[i].size;
    }
    id.ndim = od.ndim = nrest + 1;
    id.shape[nrest] = gsize;
    id.strides[nrest] = gstride;
    od.shape[nrest] = 1;
    od.strides[nrest] = 1;
    bool last = add_into_dest;
    for (int i = 0; i < nrest; ++i) last = last && rest[i].kept;
    if (last) {
      // nothing is left to reduce after this pass: it adds straight into the destination (the
      // rest are the kept axes, addressed with the destination's strides), which saves the
      // temporary and the launch of the final add
      for (int i = 0; i < nrest; ++i) od.strides[i] = rest[i].dstride;
      merge_chained(&id, &od);
      if (int rc = unary_reduce_accumulate(s, a.dest, &od, alpha, cur, &id, rop, dtype)) return rc;
      *result = nullptr;
      *nax_out = nrest;
      return CT_OK;
    }
    void* tmp = nullptr;
    if (int rc = stream_scratch(s, (size_t)n_out * elem_bytes, &tmp, slot)) return rc;
    merge_chained(&id, &od);
    if (int rc = ct_unary_reduce((void*)s, tmp, &od, alpha, cur, &id, rop, dtype)) return rc;
    cur = tmp;
    alpha = 1.0;
    slot = slot == kScratchAccumA ? kScratchAccumB : kScratchAccumA;
    nax = nrest;
    for (int i = 0; i < nrest; ++i) ax[i] = rest[i];
  }
  *result = cur;
  *nax_out = nax;
  return CT_OK;
}

// dest += sum over the broadcast axes of y*y_alpha, as staged unary-reduce! :sum passes plus
// one in-place binary-op!.
int accum_sum_staged(hipStream_t s, const OwnerArgs& a, double y_alpha, int dtype, size_t elem_bytes, bool* handled) {
  StageAxis ax[CT_MAX_DIMS];
  int nax = 0;
  const void* cur = nullptr;
  if (int rc = stage_reduce(s, a, y_alpha, dtype, elem_bytes, CT_ROP_SUM, handled, &cur, ax, &nax, true)) return rc;
  if (!*handled) return CT_OK;
  if (!cur) {  // the last pass has added into the destination
    note_kernel("accum_staged_sum");
    return CT_OK;
  }
  ct_dims dd, td;
  std::memset(&dd, 0, sizeof(dd));
  std::memset(&td, 0, sizeof(td));
  if (nax == 0) {
    dd.ndim = td.ndim = 1;
    dd.shape[0] = td.shape[0] = 1;
    dd.strides[0] = td.strides[0] = 1;
  } else {
    dd.ndim = td.ndim = nax;
    for (int i = 0; i < nax; ++i) {
      dd.shape[i] = td.shape[i] = ax[i].size;
      dd.strides[i] = ax[i].dstride;
      td.strides[i] = ax[i].ystride;
    }
  }
  const BinaryCall c{a.dest, &dd, a.dest, &dd, 1.0, 0.0, cur, &td, 1.0, 0.0, a.n_dest, CT_BOP_ADD};
  const int rc = run_binary(s, dtype, c);
  note_kernel("accum_staged_sum");
  return rc;
}

template <class T, int OP>
int accum_run_with(hipStream_t s, BinaryF<T, OP> f, void* dest, const ct_dims* dd, double dest_alpha, const void* y,
                   const ct_dims* yd, double y_alpha, int64_t n, bool reverse, int dtype);

template <class T, int OP>
int accum_run(hipStream_t s, void* dest, const ct_dims* dd, double dest_alpha, const void* y, const ct_dims* yd,
              double y_alpha, int64_t n, bool reverse, int dtype) {
  using A = typename ew_acc_of<T>::type;
  BinaryF<T, OP> f;
  // f(first, second) = op(first * xa, second * ya)
  f.xa = reverse ? (A)jvm_cast<T>(y_alpha) : (A)jvm_cast<T>(dest_alpha);
  f.ya = reverse ? (A)jvm_cast<T>(dest_alpha) : (A)jvm_cast<T>(y_alpha);
  if constexpr (OP == CT_BOP_DIV && !std::is_floating_point<T>::value) {
    if (int rc = device_error_word(&f.div0)) return rc;
    if (int rc = arm_device_error_word(s, f.div0)) return rc;
    const int rc = accum_run_with(s, f, dest, dd, dest_alpha, y, yd, y_alpha, n, reverse, dtype);
    return rc == CT_OK ? check_device_errors("binary-accum! :/") : rc;
  } else {
    return accum_run_with(s, f, dest, dd, dest_alpha, y, yd, y_alpha, n, reverse, dtype);
  }
}

template <class T, int OP>
int accum_run_with(hipStream_t s, BinaryF<T, OP> f, void* dest, const ct_dims* dd, double dest_alpha, const void* y,
                   const ct_dims* yd, double y_alpha, int64_t n, bool reverse, int dtype) {
  using A = typename ew_acc_of<T>::type;
  OwnerArgs a;
  std::memset(&a, 0, sizeof(a));
  if (owner_structure(*dd, *yd, n, &a)) {
    a.dest = dest;
    a.y = y;
    a.reverse = reverse ? 1 : 0;
    if constexpr (OP == CT_BOP_ADD) {
      if (jvm_cast<T>(dest_alpha) == (T)1 && a.n_red >= kStagedMinUpdates && n >= kStagedMinElements) {
        bool handled = false;
        if (int rc = accum_sum_staged(s, a, y_alpha, dtype, sizeof(T), &handled)) return rc;
        if (handled) return CT_OK;
      }
    }
    if constexpr (OP == CT_BOP_MAX || OP == CT_BOP_MIN) {
      // max / min of the updates first, at the reduce kernels' rate, then one step per destination
      // element.  Floats: rounding to T is monotonic, so it commutes with max / min for any y_alpha.
      // Integers: the chain narrows to T after every step, which commutes only when nothing is
      // multiplied (y_alpha 1).
      const bool alpha_ok = std::is_floating_point<T>::value || jvm_cast<T>(y_alpha) == (T)1;
      if (jvm_cast<T>(dest_alpha) == (T)1 && alpha_ok && a.n_red >= kStagedMinUpdates && n >= kStagedMinElements) {
        StageAxis ax[CT_MAX_DIMS];
        int nax = 0;
        bool handled = false;
        const void* reduced = nullptr;
        const int rop = OP == CT_BOP_MAX ? CT_ROP_MAX : CT_ROP_MIN;
        if (int rc = stage_reduce(s, a, y_alpha, dtype, sizeof(T), rop, &handled, &reduced, ax, &nax)) return rc;
        if (handled) {
          a.reduced = reduced;
          for (int i = 0; i < nax; ++i) a.kt_stride[ax[i].id] = ax[i].ystride;
          BinaryF<T, OP> f_unit = f;
          if (reverse) f_unit.xa = (A)1; else f_unit.ya = (A)1;
          note_kernel("accum_staged_extreme");
          hipLaunchKernelGGL((accum_owner_kernel<T, OP, true>), dim3((uint32_t)((a.n_dest + kBlock - 1) / kBlock)),
                             dim3(kBlock), 0, s, f, f_unit, a);
          return after_launch(s);
        }
      }
    }
    {
      AccumStreamCall sc;
      if (stream_structure<T>(a, &sc)) {
        sc.dest_alpha = dest_alpha;
        sc.y_alpha = y_alpha;
        sc.reverse = reverse;
        sc.op = OP;
        sc.dtype = dtype;
        sc.div0 = f.div0;
        return accum_stream(s, sc);
      }
    }
    note_kernel("accum_owner");
    hipLaunchKernelGGL((accum_owner_kernel<T, OP, false>), dim3((uint32_t)((a.n_dest + kBlock - 1) / kBlock)), dim3(kBlock),
                       0, s, f, f, a);
    return after_launch(s);
  }
  GroupedArgs g;
  std::memset(&g, 0, sizeof(g));
  const int32_t* index = nullptr;
  bool vec_ok = false;
  if (grouped_structure<T>(*dd, *yd, dest, y, n, &g, &index, &vec_ok)) {
    if (int rc = sort_index(s, index, g.n_index, &g.skey, &g.perm)) return rc;
    g.dest = dest;
    g.y = y;
    g.reverse = reverse ? 1 : 0;
    constexpr int VMAX = 16 / (int)sizeof(T);
    // rows of at least a block of vectors: two vectors per lane, half a row apart (the accumulate
    // of 65536 rows of 4 KiB: 95 us with one vector per lane, 88 with two, 130 with four)
    constexpr int kPer = 2;
    const bool several = vec_ok && g.kept_vecs >= 256;
    if (several) {
      g.lane_vecs = (g.kept_vecs + kPer - 1) / kPer;
      g.lane_fd = FastDiv(g.lane_vecs);
    }
    const dim3 grid((uint32_t)(((int64_t)g.n_index * g.lane_vecs + kBlock - 1) / kBlock));
    note_kernel(vec_ok ? "accum_grouped_vec" : "accum_grouped");
    if (several) hipLaunchKernelGGL((accum_grouped_kernel<T, OP, VMAX, kPer>), grid, dim3(kBlock), 0, s, f, g);
    else if (vec_ok) hipLaunchKernelGGL((accum_grouped_kernel<T, OP, VMAX, 1>), grid, dim3(kBlock), 0, s, f, g);
    else hipLaunchKernelGGL((accum_grouped_kernel<T, OP, 1, 1>), grid, dim3(kBlock), 0, s, f, g);
    return after_launch(s);
  }
  EwOperand ops[3] = {{dest, dd, (int)sizeof(T), 0},
                      {reverse ? y : dest, reverse ? yd : dd, (int)sizeof(T), 0},
                      {reverse ? dest : y, reverse ? dd : yd, (int)sizeof(T), 0}};
  return launch_elementwise_serial(s, f, ops, n);
}

template <class T>
int accum_dispatch(hipStream_t s, void* dest, const ct_dims* dd, double da, const void* y, const ct_dims* yd, double ya,
                   int64_t n, int op, bool reverse, int dtype) {
#define CT_CASE(OP) case OP: return accum_run<T, OP>(s, dest, dd, da, y, yd, ya, n, reverse, dtype)
  switch (op) {
    CT_CASE(CT_BOP_ADD); CT_CASE(CT_BOP_SUB); CT_CASE(CT_BOP_MUL); CT_CASE(CT_BOP_DIV);
    CT_CASE(CT_BOP_MIN); CT_CASE(CT_BOP_MAX); CT_CASE(CT_BOP_BIT_AND); CT_CASE(CT_BOP_BIT_XOR);
    CT_CASE(CT_BOP_EQ); CT_CASE(CT_BOP_GT); CT_CASE(CT_BOP_GE); CT_CASE(CT_BOP_LT); CT_CASE(CT_BOP_LE);
    default: return set_error(CT_ERR_INVALID, "unknown binary operation %d", op);
  }
#undef CT_CASE
}

}  // namespace

extern "C" int ct_binary_accum(void* stream, void* dest, const ct_dims* dest_dims, double dest_alpha, const void* y,
                               const ct_dims* y_dims, double y_alpha, int64_t n, int op, int reverse_operands,
                               int dest_requires_cas, int dtype) {
  CT_REQUIRE(dest && y, "ct_binary_accum: null buffer");
  CT_REQUIRE(n >= 0, "ct_binary_accum: negative count");
  if (n == 0) return CT_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (!dest_requires_cas) {
    // every destination element is written once: an in-place binary-op!
    // (cpu/tensor_math.clj:1451-1463)
    BinaryCall c = reverse_operands
                       ? BinaryCall{dest, dest_dims, y, y_dims, y_alpha, 0.0, dest, dest_dims, dest_alpha, 0.0, n, op}
                       : BinaryCall{dest, dest_dims, dest, dest_dims, dest_alpha, 0.0, y, y_dims, y_alpha, 0.0, n, op};
    return run_binary(s, dtype, c);
  }
  if (int rc = check_dims(dest_dims, "dest")) return rc;
  if (int rc = check_dims(y_dims, "y")) return rc;
  CT_DISPATCH_DTYPE(dtype, return accum_dispatch<T>(s, dest, dest_dims, dest_alpha, y, y_dims, y_alpha, n, op, reverse_operands != 0, dtype));
  return CT_OK;
}
