// elementwise.h -- the three elementwise kernel families and their launcher.
//
// A functor F describes one scalar operation:
//   static constexpr int NIN;              number of inputs, 0..3
//   using Out, In0, In1, In2;              element types (unused inputs: any type)
//   __device__ Out operator()(In0, In1, In2) const;
// The launcher analyses the operands' dimensions (plan.h) and runs F through
//   ew_vec_kernel   128-bit coalesced accesses along the innermost axis;
//                   broadcast operands are read as wave-uniform scalars;
//                   address arithmetic is done once per vector, not per element
//   ew_tile_kernel  transposed inputs staged through a padded LDS tile so both
//                   the reads and the writes are coalesced
//   ew_gen_kernel   per-element addressing with the reference's address objects
#pragma once

#include <algorithm>
#include <vector>

#include "common.h"
#include "plan.h"

namespace cthip {

template <class T, int N> struct alignas(sizeof(T) * N) Vec { T v[N]; };

constexpr int kBlock = 256;
constexpr int64_t kVecLaunchMax = int64_t(1) << 30;  // vectors one launch of the vector kernel indexes

template <class T> __device__ __forceinline__ T const_from_bits(uint64_t bits) {
  T c;
  __builtin_memcpy(&c, &bits, sizeof(T));
  return c;
}
// Streaming (non-temporal) load of any 1/2/4/8/16-byte object: the data is
// used once, so it should not displace reusable lines from the caches.
template <int BYTES> struct raw_bits;
template <> struct raw_bits<1> { using type = uint8_t; };
template <> struct raw_bits<2> { using type = uint16_t; };
template <> struct raw_bits<4> { using type = uint32_t; };
template <> struct raw_bits<8> { using type = uint32_t __attribute__((ext_vector_type(2))); };
template <> struct raw_bits<16> { using type = uint32_t __attribute__((ext_vector_type(4))); };
template <class V> __device__ __forceinline__ V nt_load(const V* p) {
  using R = typename raw_bits<sizeof(V)>::type;
  const R r = __builtin_nontemporal_load(reinterpret_cast<const R*>(p));
  V v;
  __builtin_memcpy(&v, &r, sizeof(V));
  return v;
}

template <class V> __device__ __forceinline__ void nt_store(const V& v, V* p) {
  using R = typename raw_bits<sizeof(V)>::type;
  R r;
  __builtin_memcpy(&r, &v, sizeof(V));
  __builtin_nontemporal_store(r, reinterpret_cast<R*>(p));
}

template <class T> inline uint64_t bits_of(T c) {
  uint64_t b = 0;
  std::memcpy(&b, &c, sizeof(T));
  return b;
}

// ------------------------------------------------------------------ VEC

// The first block of members is everything a lane needs when the operands have
// at most two outer axes; the kernel fetches it in one batch (see ew_vec_kernel).
struct VecArgs {
  uint64_t total_vecs;
  FastDiv inner_fd;
  int32_t n_outer;
  FastDiv outer_fd01[2];  // an absent axis has size 1 (and stride 0)
  uint32_t unit_mask;     // bit k: operand k is unit-stride along the inner axis
  uint32_t const_mask;    // bit k: operand k is a scalar constant
  uint32_t nt_mask;       // bit k: operand k is read exactly once (no broadcast axis), so its loads may bypass the caches
  uint32_t streaming;     // 0: the call fits the caches; 1: non-temporal loads; 2: and non-temporal stores (see ew_vec_kernel)
  uint32_t grouped_blocks;  // see xcd_grouped_unit; set by the launcher
  char* ptr[kMaxOps];
  int64_t outer_stride01[kMaxOps][2];
  uint64_t cbits[kMaxOps];
  // outer axes beyond the second
  FastDiv outer_fd_hi[CT_MAX_DIMS - 3];
  int64_t outer_stride_hi[kMaxOps][CT_MAX_DIMS - 3];
  uint32_t inner_vecs;
  // Row gather / scatter: outer_index[k][d] != nullptr makes operand k take its offset along outer
  // axis d (one of the first two) as index[coordinate] * stride.  Read by the INDEXED kernels only.
  const int32_t* outer_index[kMaxOps][2];
  uint32_t indexed;  // some outer_index entry is set
};

// Kinds of an input operand of the vector kernel.
enum VecKind { VK_STREAM = 0,   // unit-stride, read exactly once: non-temporal vector load
               VK_CACHED = 1,   // unit-stride, re-read by other rows (a bias row): plain vector load
               VK_SCALAR = 2,   // one element broadcast along the inner axis (a per-row value)
               VK_CONST = 3 };  // a constant carried in the arguments
constexpr int vec_kinds(int k1, int k2 = 0, int k3 = 0) { return k1 | (k2 << 2) | (k3 << 4); }

// Operand k of one lane.  vp / sp are the lane's vector and scalar addresses.
// KIND < 0: the kind is read from the run-time masks.
template <class T, int VEC, int STREAM, int KIND>
__device__ __forceinline__ Vec<T, VEC> vec_load(uint32_t const_mask, uint32_t unit_mask, uint32_t nt_mask, uint64_t cbits,
                                                int k, const Vec<T, VEC>* vp, const T* sp) {
  Vec<T, VEC> r;
  const bool is_const = KIND < 0 ? ((const_mask >> k) & 1u) != 0 : KIND == VK_CONST;
  const bool is_unit = KIND < 0 ? ((unit_mask >> k) & 1u) != 0 : (KIND == VK_STREAM || KIND == VK_CACHED);
  const bool is_once = KIND < 0 ? ((nt_mask >> k) & 1u) != 0 : KIND == VK_STREAM;
  if (is_const) {
    const T c = const_from_bits<T>(cbits);
#pragma unroll
    for (int i = 0; i < VEC; ++i) r.v[i] = c;
  } else if (is_unit) {
    // a broadcast operand (a bias row, say) is re-read by every outer index and must stay cached
    if (STREAM >= 1 && is_once) r = nt_load(vp);
    else r = *vp;
  } else {
    const T c = *sp;
#pragma unroll
    for (int i = 0; i < VEC; ++i) r.v[i] = c;
  }
  return r;
}

// One 16-byte vector per lane.  On this part one vector per lane with many
// resident blocks sustains more bandwidth than several vectors per lane, and
// non-temporal loads add a few percent on streams larger than the caches.
// STREAM (0: plain accesses, 1: non-temporal loads, 2: non-temporal loads and
// stores) is a template parameter: a run-time choice between a plain and a
// non-temporal access to the same address is folded into one plain access by
// the compiler, which loses the hint.  Measured on an in-place add: below the
// last-level cache's size plain accesses win (92 % of peak at 256 MiB against
// 88 % with non-temporal loads and 83 % with non-temporal stores too); at 1 GiB
// non-temporal loads and stores together win (82 % against 73 %).
//
// A wave lives about as long as one trip to memory, so every scalar fetch of a
// kernel argument that sits between the wave's start and its first vector load
// costs bandwidth, and the compiler fetches an argument next to its first use,
// inside whatever branch that is.  The kernel therefore names every argument it
// needs in one empty asm statement at the top: they are fetched in one batch
// with one wait, and the code that follows only touches registers.  For the
// same reason there is no special case for flat operands: the host describes
// them as one row (absent outer axes have size 1 and stride 0).
//
// KINDS >= 0 fixes the operand kinds at compile time (vec_kinds): the common
// broadcast patterns then run without the operand-kind branches, which cost
// about 3 % of a copy's bandwidth.
//
// INDEXED: one of the first two outer axes of an operand may go through an
// index tensor (select rows by label, scatter rows back): the row's coordinate
// is replaced by index[coordinate] before it meets the stride.  For rows at
// least a block wide the look-up is one scalar load per wave.
template <class F, int VEC, int STREAM, int KINDS = -1, bool INDEXED = false, int PER = 1>
__global__ void __launch_bounds__(kBlock) ew_vec_kernel(const F f, const VecArgs a) {
  using Out = typename F::Out;
  using In0 = typename F::In0;
  using In1 = typename F::In1;
  using In2 = typename F::In2;
  constexpr int NIN = F::NIN;

  const uint64_t total = a.total_vecs;
  const FastDiv ifd = a.inner_fd, fd0 = a.outer_fd01[0], fd1 = a.outer_fd01[1];
  const int32_t n_outer = a.n_outer;
  const uint32_t unit_mask = a.unit_mask, const_mask = a.const_mask, nt_mask = a.nt_mask;
  const uint32_t grouped = a.grouped_blocks;
  char* const b0 = a.ptr[0];
  char* const b1 = a.ptr[NIN >= 1 ? 1 : 0];
  char* const b2 = a.ptr[NIN >= 2 ? 2 : 0];
  char* const b3 = a.ptr[NIN >= 3 ? 3 : 0];
  const int64_t s00 = a.outer_stride01[0][0], s01 = a.outer_stride01[0][1];
  const int64_t s10 = a.outer_stride01[NIN >= 1 ? 1 : 0][0], s11 = a.outer_stride01[NIN >= 1 ? 1 : 0][1];
  const int64_t s20 = a.outer_stride01[NIN >= 2 ? 2 : 0][0], s21 = a.outer_stride01[NIN >= 2 ? 2 : 0][1];
  const int64_t s30 = a.outer_stride01[NIN >= 3 ? 3 : 0][0], s31 = a.outer_stride01[NIN >= 3 ? 3 : 0][1];
  const uint64_t c1 = a.cbits[NIN >= 1 ? 1 : 0], c2 = a.cbits[NIN >= 2 ? 2 : 0], c3 = a.cbits[NIN >= 3 ? 3 : 0];
  asm volatile("" ::"s"(total), "s"(ifd.d), "s"(ifd.m), "s"(ifd.s), "s"(fd0.d), "s"(fd0.m), "s"(fd0.s), "s"(fd1.d),
               "s"(fd1.m), "s"(fd1.s), "s"(n_outer), "s"(unit_mask), "s"(const_mask), "s"(nt_mask), "s"(grouped), "s"(b0), "s"(b1),
               "s"(b2), "s"(b3), "s"(s00), "s"(s01), "s"(s10), "s"(s11), "s"(s20), "s"(s21), "s"(s30), "s"(s31),
               "s"(c1), "s"(c2), "s"(c3));

  // the block's first vector; a lane takes vector threadIdx.x of each of the block's PER runs of kBlock vectors
  const uint64_t v_block = (uint64_t)xcd_grouped_unit(blockIdx.x, grouped) * (uint64_t)(kBlock * PER);
  if (v_block + threadIdx.x >= total) return;
  // Offsets of the outer index `row` for every operand.  Called with a
  // wave-uniform row this is scalar arithmetic.
  auto outer_offsets = [&](uint32_t row, int64_t* off) {
    uint32_t q0, r0, q1, r1;
    fd0.divmod(row, q0, r0);
    fd1.divmod(q0, q1, r1);
    if constexpr (INDEXED) {
#pragma unroll
      for (int k = 0; k <= NIN; ++k) {
        const int32_t* i0 = a.outer_index[k][0];
        const int32_t* i1 = a.outer_index[k][1];
        const int64_t c0 = i0 ? (int64_t)i0[r0] : (int64_t)r0;
        const int64_t c1 = i1 ? (int64_t)i1[r1] : (int64_t)r1;
        off[k] = c0 * a.outer_stride01[k][0] + c1 * a.outer_stride01[k][1];
      }
#pragma unroll
      for (int k = NIN + 1; k < kMaxOps; ++k) off[k] = 0;
    } else {
      off[0] = (int64_t)r0 * s00 + (int64_t)r1 * s01;
      off[1] = (int64_t)r0 * s10 + (int64_t)r1 * s11;
      off[2] = (int64_t)r0 * s20 + (int64_t)r1 * s21;
      off[3] = (int64_t)r0 * s30 + (int64_t)r1 * s31;
    }
    if (n_outer > 2) {
      row = q1;
      for (int d = 2; d < n_outer; ++d) {
        uint32_t q, r;
        a.outer_fd_hi[d - 2].divmod(row, q, r);
        row = q;
#pragma unroll
        for (int k = 0; k <= NIN; ++k) off[k] += (int64_t)r * a.outer_stride_hi[k][d - 2];
      }
    }
  };
  struct Where { int64_t off[kMaxOps]; int64_t col; };
  auto locate = [&](uint64_t v_first, Where& w) {
    int64_t* const off = w.off;
    int64_t col;
    if (ifd.d >= (uint32_t)kBlock) {
      // Rows of at least a block's width: the block's 256 vectors lie in at most two
      // rows, whose offsets are computed once per wave on the scalar unit; a lane
      // only picks its row.
      uint32_t row_a, cv_a;
      ifd.divmod((uint32_t)v_first, row_a, cv_a);
      outer_offsets(row_a, off);
      uint32_t cv = cv_a + threadIdx.x;
      if (cv_a + (uint32_t)kBlock > ifd.d) {  // the block runs into the next row
        int64_t off_b[kMaxOps];
        outer_offsets(row_a + 1, off_b);
        const bool next = cv >= ifd.d;
        cv -= next ? ifd.d : 0u;
#pragma unroll
        for (int k = 0; k < kMaxOps; ++k) off[k] = next ? off_b[k] : off[k];
      }
      col = (int64_t)cv * VEC;
    } else {
      uint32_t row, cv;
      ifd.divmod((uint32_t)v_first + threadIdx.x, row, cv);
      col = (int64_t)cv * VEC;
      outer_offsets(row, off);
    }
    w.col = col;
  };
  char* const base[kMaxOps] = {b0, b1, b2, b3};
  const uint64_t cbits[kMaxOps] = {0, c1, c2, c3};
  Where w[PER];
  bool live[PER];
  Vec<In0, VEC> x0[PER];
  Vec<In1, VEC> x1[PER];
  Vec<In2, VEC> x2[PER];
  // every load of the lane's PER vectors is issued before its first store
#pragma unroll
  for (int h = 0; h < PER; ++h) {
    const uint64_t v_first = v_block + (uint64_t)h * kBlock;
    live[h] = h == 0 || v_first + threadIdx.x < total;
    if (!live[h]) continue;
    locate(v_first, w[h]);
    const int64_t* const off = w[h].off;
    const int64_t col = w[h].col;
    if constexpr (NIN >= 1) {
      const In0* sp = reinterpret_cast<const In0*>(base[1]) + off[1];
      x0[h] = vec_load<In0, VEC, STREAM, (KINDS < 0 ? -1 : (KINDS & 3))>(const_mask, unit_mask, nt_mask, cbits[1], 1, reinterpret_cast<const Vec<In0, VEC>*>(sp + col), sp);
    }
    if constexpr (NIN >= 2) {
      const In1* sp = reinterpret_cast<const In1*>(base[2]) + off[2];
      x1[h] = vec_load<In1, VEC, STREAM, (KINDS < 0 ? -1 : ((KINDS >> 2) & 3))>(const_mask, unit_mask, nt_mask, cbits[2], 2, reinterpret_cast<const Vec<In1, VEC>*>(sp + col), sp);
    }
    if constexpr (NIN >= 3) {
      const In2* sp = reinterpret_cast<const In2*>(base[3]) + off[3];
      x2[h] = vec_load<In2, VEC, STREAM, (KINDS < 0 ? -1 : ((KINDS >> 4) & 3))>(const_mask, unit_mask, nt_mask, cbits[3], 3, reinterpret_cast<const Vec<In2, VEC>*>(sp + col), sp);
    }
  }
#pragma unroll
  for (int h = 0; h < PER; ++h) {
    if (!live[h]) continue;
    Vec<Out, VEC> r;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      In0 p0{};
      In1 p1{};
      In2 p2{};
      if constexpr (NIN >= 1) p0 = x0[h].v[i];
      if constexpr (NIN >= 2) p1 = x1[h].v[i];
      if constexpr (NIN >= 3) p2 = x2[h].v[i];
      r.v[i] = f(p0, p1, p2);
    }
    Vec<Out, VEC>* dp = reinterpret_cast<Vec<Out, VEC>*>(reinterpret_cast<Out*>(base[0]) + w[h].off[0] + w[h].col);
    if constexpr (STREAM == 2) nt_store(r, dp);
    else *dp = r;
  }
}

// The contiguous case: every operand is a flat unit-stride array read (or
// written) exactly once.  No address decomposition and no operand kinds: a lane
// loads its vectors, applies F and stores.  The general vector kernel's
// scalar prologue and operand-kind branches cost it about 6 % of a plain copy's
// bandwidth, which this form gets back.
struct FlatArgs {
  uint64_t total_vecs;
  uint32_t grouped_blocks;  // see xcd_grouped_unit
  char* ptr[kMaxOps];
};

// PER > 1 (a conversion between element widths, where the narrow side moves only 16 / ratio
// bytes per lane and vector): a lane takes PER vectors, kBlock apart, and issues all of its
// loads before the first store.
template <class F, int VEC, int STREAM, int PER = 1>
__global__ void __launch_bounds__(kBlock) ew_flat_kernel(const F f, const FlatArgs a) {
  using Out = typename F::Out;
  using In0 = typename F::In0;
  using In1 = typename F::In1;
  using In2 = typename F::In2;
  constexpr int NIN = F::NIN;
  const uint64_t v0 = (uint64_t)xcd_grouped_unit(blockIdx.x, a.grouped_blocks) * (uint64_t)(kBlock * PER) + threadIdx.x;
  if (v0 >= a.total_vecs) return;
  Vec<In0, VEC> x0[PER];
  Vec<In1, VEC> x1[PER];
  Vec<In2, VEC> x2[PER];
#pragma unroll
  for (int h = 0; h < PER; ++h) {
    const uint64_t v = v0 + (uint64_t)h * kBlock;
    if (h > 0 && v >= a.total_vecs) break;
    if constexpr (NIN >= 1) {
      const Vec<In0, VEC>* p = reinterpret_cast<const Vec<In0, VEC>*>(a.ptr[1]) + v;
      if constexpr (STREAM >= 1) x0[h] = nt_load(p); else x0[h] = *p;
    }
    if constexpr (NIN >= 2) {
      const Vec<In1, VEC>* p = reinterpret_cast<const Vec<In1, VEC>*>(a.ptr[2]) + v;
      if constexpr (STREAM >= 1) x1[h] = nt_load(p); else x1[h] = *p;
    }
    if constexpr (NIN >= 3) {
      const Vec<In2, VEC>* p = reinterpret_cast<const Vec<In2, VEC>*>(a.ptr[3]) + v;
      if constexpr (STREAM >= 1) x2[h] = nt_load(p); else x2[h] = *p;
    }
  }
#pragma unroll
  for (int h = 0; h < PER; ++h) {
    const uint64_t v = v0 + (uint64_t)h * kBlock;
    if (h > 0 && v >= a.total_vecs) break;
    Vec<Out, VEC> r;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      In0 p0{};
      In1 p1{};
      In2 p2{};
      if constexpr (NIN >= 1) p0 = x0[h].v[i];
      if constexpr (NIN >= 2) p1 = x1[h].v[i];
      if constexpr (NIN >= 3) p2 = x2[h].v[i];
      r.v[i] = f(p0, p1, p2);
    }
    Vec<Out, VEC>* dp = reinterpret_cast<Vec<Out, VEC>*>(a.ptr[0]) + v;
    if constexpr (STREAM == 2) nt_store(r, dp);
    else *dp = r;
  }
}

// ------------------------------------------------------------------ UNALIGNED VECTORS
//
// Rows whose starts are not on the 16-byte grid (a [rows, 999] block of a pitch-1024 matrix
// copied to a contiguous one, a sub-buffer that starts at an odd element) or whose length is no
// whole number of vectors used to run one element per lane.  Global memory accesses only need
// the element's alignment, so a lane takes a vector that starts anywhere; the last lane of a row
// takes what is left of the row element by element.  a.inner_fd counts vectors per row, rounded up.
template <class T, int N> struct alignas(sizeof(T)) UVec { T v[N]; };
// A non-temporal store of such a vector: the same bytes, promised no more than the element's alignment.
template <int BYTES, int ALIGN> struct raw_unaligned {
  typedef typename raw_bits<BYTES>::type type __attribute__((aligned(ALIGN)));
};
template <class T, int N> __device__ __forceinline__ void nt_store(const UVec<T, N>& v, UVec<T, N>* p) {
  using R = typename raw_unaligned<(int)sizeof(UVec<T, N>), (int)sizeof(T)>::type;
  R r;
  __builtin_memcpy(&r, &v, sizeof(r));
  __builtin_nontemporal_store(r, reinterpret_cast<R*>(p));
}

template <class F, int VEC>
__global__ void __launch_bounds__(kBlock) ew_vecu_kernel(const F f, const VecArgs a, const uint32_t inner_elems) {
  using Out = typename F::Out;
  using In0 = typename F::In0;
  using In1 = typename F::In1;
  using In2 = typename F::In2;
  constexpr int NIN = F::NIN;
  const uint64_t v = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
  if (v >= a.total_vecs) return;
  uint32_t row, cv;
  a.inner_fd.divmod((uint32_t)v, row, cv);
  const uint32_t col = cv * (uint32_t)VEC;
  const uint32_t left = inner_elems - col;
  const bool whole = left >= (uint32_t)VEC;
  int64_t off[kMaxOps] = {0, 0, 0, 0};
  {
    uint32_t r = row;
    for (int d = 0; d < a.n_outer; ++d) {
      uint32_t q, c;
      (d < 2 ? a.outer_fd01[d] : a.outer_fd_hi[d - 2]).divmod(r, q, c);
      r = q;
#pragma unroll
      for (int k = 0; k <= NIN; ++k) off[k] += (int64_t)c * (d < 2 ? a.outer_stride01[k][d] : a.outer_stride_hi[k][d - 2]);
    }
  }
  auto fetch = [&](int k, auto* typed, auto& x) {
    using T = typename std::remove_cv<typename std::remove_pointer<decltype(typed)>::type>::type;
    if ((a.const_mask >> k) & 1u) {
      const T c = const_from_bits<T>(a.cbits[k]);
#pragma unroll
      for (int i = 0; i < VEC; ++i) x.v[i] = c;
      return;
    }
    const T* sp = reinterpret_cast<const T*>(a.ptr[k]) + off[k];
    if ((a.unit_mask >> k) & 1u) {
      if (whole) {
        const UVec<T, VEC> u = *reinterpret_cast<const UVec<T, VEC>*>(sp + col);
#pragma unroll
        for (int i = 0; i < VEC; ++i) x.v[i] = u.v[i];
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) x.v[i] = (uint32_t)i < left ? sp[col + i] : T{};
      }
    } else {
      const T c = *sp;
#pragma unroll
      for (int i = 0; i < VEC; ++i) x.v[i] = c;
    }
  };
  Vec<In0, VEC> x0;
  Vec<In1, VEC> x1;
  Vec<In2, VEC> x2;
  if constexpr (NIN >= 1) fetch(1, (const In0*)nullptr, x0);
  if constexpr (NIN >= 2) fetch(2, (const In1*)nullptr, x1);
  if constexpr (NIN >= 3) fetch(3, (const In2*)nullptr, x2);
  UVec<Out, VEC> r;
#pragma unroll
  for (int i = 0; i < VEC; ++i) {
    In0 p0{};
    In1 p1{};
    In2 p2{};
    if constexpr (NIN >= 1) p0 = x0.v[i];
    if constexpr (NIN >= 2) p1 = x1.v[i];
    if constexpr (NIN >= 3) p2 = x2.v[i];
    r.v[i] = f(p0, p1, p2);
  }
  // Stores that bypass the caches pay in a call too large for them whatever the alignment (a [65536,999]
  // block written into a pitch-1024 matrix: 69 -> 76 % of peak); loads that start off the grid do not.
  Out* dp = reinterpret_cast<Out*>(a.ptr[0]) + off[0] + col;
  if (whole) {
    if (a.streaming) {
      asm volatile("");  // keeps the two stores apart: merged into one, they lose the hint
      nt_store(r, reinterpret_cast<UVec<Out, VEC>*>(dp));
    } else {
      *reinterpret_cast<UVec<Out, VEC>*>(dp) = r;
    }
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i)
      if ((uint32_t)i < left) dp[i] = r.v[i];
  }
}

// ------------------------------------------------------------------ RAGGED ROWS
//
// Rows that are no whole number of vectors (49 pixels of a 7 x 7 image under a per-channel bias,
// ten classes under a per-row scale) used to run one element per lane.  When the big operands are
// dense over the whole call, their flat offset is the element number whatever the row length, and
// a lane can take an aligned 16-byte vector of them that may straddle the end of a row: at most
// one row boundary falls into a vector (rows are at least a vector long).  The small operands are
// fetched per element: a per-row value (constant along the row: any outer strides) for the row or
// the next one, a row vector (the same row for every outer index) at its column.  An input whose
// rows are unit-stride but lie a pitch apart (a [rows, 999] block of a pitch-1024 matrix copied
// out, ct/submatrix) is read per destination vector from where its row lies, so that the stores,
// which cost more than the loads when they straddle lines, stay aligned; in a call larger than the caches they bypass them (59 -> 80 % of peak).
struct RaggedArgs {
  uint32_t n;                 // elements; < 2^31
  FastDiv inner_fd;           // row length
  int32_t n_outer;
  FastDiv outer_fd[CT_MAX_DIMS - 1];
  uint32_t dense_mask;        // bit k: operand k is dense (offset = element number)
  uint32_t scalar_mask;       // bit k: one value per row
  uint32_t pitched_mask;      // bit k: unit-stride rows wherever the outer strides put them (a block of a wider matrix)
  uint32_t const_mask;        // bit k: a constant; every other input is a row vector
  uint32_t streaming;
  char* ptr[kMaxOps];
  uint64_t cbits[kMaxOps];
  int64_t outer_stride[kMaxOps][CT_MAX_DIMS - 1];
};

template <class F, int VEC, bool NT>
__global__ void __launch_bounds__(kBlock) ew_ragged_kernel(const F f, const RaggedArgs a) {
  using Out = typename F::Out;
  using In0 = typename F::In0;
  using In1 = typename F::In1;
  using In2 = typename F::In2;
  constexpr int NIN = F::NIN;
  const uint32_t e0 = (blockIdx.x * kBlock + threadIdx.x) * (uint32_t)VEC;
  if (e0 >= a.n) return;
  uint32_t row, col;
  a.inner_fd.divmod(e0, row, col);
  const uint32_t inner = a.inner_fd.d;
  const uint32_t in_row = inner - col;  // elements of the vector that belong to `row`
  const bool whole = e0 + VEC <= a.n;
  // offset of a per-row operand for a row
  auto row_offset = [&](int k, uint32_t r) {
    int64_t off = 0;
    for (int d = 0; d < a.n_outer; ++d) {
      uint32_t q, c;
      a.outer_fd[d].divmod(r, q, c);
      r = q;
      off += (int64_t)c * a.outer_stride[k][d];
    }
    return off;
  };
  auto fetch = [&](int k, auto* typed, auto& x) {
    using T = typename std::remove_cv<typename std::remove_pointer<decltype(typed)>::type>::type;
    const T* base = reinterpret_cast<const T*>(a.ptr[k]);
    if ((a.const_mask >> k) & 1u) {
      const T c = const_from_bits<T>(a.cbits[k]);
#pragma unroll
      for (int i = 0; i < VEC; ++i) x.v[i] = c;
    } else if ((a.dense_mask >> k) & 1u) {
      if (whole) {
        const Vec<T, VEC>* vp = reinterpret_cast<const Vec<T, VEC>*>(base + e0);
        if constexpr (NT) x = nt_load(vp); else x = *vp;
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i) x.v[i] = e0 + i < a.n ? base[e0 + i] : T{};
      }
    } else if ((a.pitched_mask >> k) & 1u) {
      // the destination's aligned vector is the tail of one row of this operand and, past the row's end,
      // the head of the next: a load that needs only the element's alignment when it stays inside the row
      const T* rp = base + row_offset(k, row) + col;
      if (in_row >= (uint32_t)VEC) {
        const UVec<T, VEC> u = *reinterpret_cast<const UVec<T, VEC>*>(rp);
#pragma unroll
        for (int i = 0; i < VEC; ++i) x.v[i] = u.v[i];
      } else {
        const T* np = e0 + in_row < a.n ? base + row_offset(k, row + 1) : rp;
#pragma unroll
        for (int i = 0; i < VEC; ++i) x.v[i] = (uint32_t)i < in_row ? rp[i] : (e0 + i < a.n ? np[(uint32_t)i - in_row] : T{});
      }
    } else if ((a.scalar_mask >> k) & 1u) {
      const T cur = base[row_offset(k, row)];
      T next = cur;
      if (in_row < (uint32_t)VEC && e0 + in_row < a.n) next = base[row_offset(k, row + 1)];
#pragma unroll
      for (int i = 0; i < VEC; ++i) x.v[i] = (uint32_t)i < in_row ? cur : next;
    } else {  // a row vector
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const uint32_t c = (uint32_t)i < in_row ? col + i : (uint32_t)i - in_row;
        x.v[i] = base[c];
      }
    }
  };
  Vec<In0, VEC> x0;
  Vec<In1, VEC> x1;
  Vec<In2, VEC> x2;
  if constexpr (NIN >= 1) fetch(1, (const In0*)nullptr, x0);
  if constexpr (NIN >= 2) fetch(2, (const In1*)nullptr, x1);
  if constexpr (NIN >= 3) fetch(3, (const In2*)nullptr, x2);
  Vec<Out, VEC> r;
#pragma unroll
  for (int i = 0; i < VEC; ++i) {
    In0 p0{};
    In1 p1{};
    In2 p2{};
    if constexpr (NIN >= 1) p0 = x0.v[i];
    if constexpr (NIN >= 2) p1 = x1.v[i];
    if constexpr (NIN >= 3) p2 = x2.v[i];
    r.v[i] = f(p0, p1, p2);
  }
  Out* dp = reinterpret_cast<Out*>(a.ptr[0]) + e0;
  if (whole) {
    if constexpr (NT) nt_store(r, reinterpret_cast<Vec<Out, VEC>*>(dp));
    else *reinterpret_cast<Vec<Out, VEC>*>(dp) = r;
  } else {
#pragma unroll
    for (int i = 0; i < VEC; ++i)
      if (e0 + i < a.n) dp[i] = r.v[i];
  }
}

// ------------------------------------------------------------------ SHORT PITCHED ROWS
//
// A dense [rows, w] destination taken from rows of a small pitch (ten values out of every sixteen:
// the first columns of a narrow matrix).  The memory system moves whole 64-byte lines whichever
// bytes are asked for, so a block takes the contiguous span of memory that holds its rows, padding
// included, with aligned 16-byte non-temporal loads, parks it in LDS and picks the values of its
// destination vectors from there; the stores are aligned and dense.  assign! (with conversion) only.
// (Per-vector loads from where the rows lie, as the ragged kernel does for longer rows, reach 52 % of
// peak on float [4M, 10] of pitch 16; the lines that have to move bound it at 77 %.)
struct SpanArgs {
  char* ptr[2];
  uint32_t rows;
  uint32_t w, pitch;
  FastDiv w_fd;
  uint32_t rows_per_block;
};

constexpr int kSpanLdsBytes = 16384;

template <class F, int VEC>
__global__ void __launch_bounds__(kBlock) ew_span_kernel(const F f, const SpanArgs a) {
  using Out = typename F::Out;
  using In = typename F::In0;
  constexpr int IV = 16 / (int)sizeof(In);
  __shared__ __align__(16) char smem[kSpanLdsBytes];
  In* tile = reinterpret_cast<In*>(smem);
  const uint32_t row0 = blockIdx.x * a.rows_per_block;
  const uint32_t n_rows = a.rows - row0 < a.rows_per_block ? a.rows - row0 : a.rows_per_block;
  const In* src = reinterpret_cast<const In*>(a.ptr[1]) + (int64_t)row0 * a.pitch;
  // the last row of the tensor ends with its last value: nothing behind it may be read
  const uint32_t span = (n_rows - 1) * a.pitch + a.w;
  const uint32_t span_vecs = span / IV;
  for (uint32_t v = threadIdx.x; v < span_vecs; v += kBlock)
    reinterpret_cast<Vec<In, IV>*>(tile)[v] = nt_load(reinterpret_cast<const Vec<In, IV>*>(src) + v);
  for (uint32_t e = span_vecs * IV + threadIdx.x; e < span; e += kBlock) tile[e] = src[e];
  __syncthreads();
  const uint32_t count = n_rows * a.w;
  Out* dst = reinterpret_cast<Out*>(a.ptr[0]) + (int64_t)row0 * a.w;
  for (uint32_t e0 = threadIdx.x * VEC; e0 < count; e0 += kBlock * VEC) {
    uint32_t r, c;
    a.w_fd.divmod(e0, r, c);
    Vec<Out, VEC> out;
#pragma unroll
    for (int i = 0; i < VEC; ++i) {
      out.v[i] = f(tile[r * a.pitch + c], typename F::In1{}, typename F::In2{});
      if (++c == a.w) { c = 0; ++r; }
    }
    if (e0 + VEC <= count) {
      *reinterpret_cast<Vec<Out, VEC>*>(dst + e0) = out;  // plain: stores that bypass the caches cost 3 points here
    } else {
#pragma unroll
      for (int i = 0; i < VEC; ++i)
        if (e0 + i < count) dst[e0 + i] = out.v[i];
    }
  }
}

// ------------------------------------------------------------------ TILE

struct TileArgs {
  uint32_t sizeA, sizeB, tilesA, tilesB;
  // Blocks are grouped into super-tiles of super_a x super_b tiles; see ew_tile_kernel.
  uint32_t super_a, super_b, n_super;
  FastDiv per_fd;      // tiles per super-tile (super_a * super_b)
  FastDiv sb_fd;       // super_b
  FastDiv nsb_fd;      // super-tiles along B
  FastDiv nst_fd;      // super-tiles per matrix (along A times along B)
  int32_t n_outer;
  FastDiv outer_fd[CT_MAX_DIMS - 2];
  char* ptr[kMaxOps];
  int64_t strideA[kMaxOps], strideB[kMaxOps];
  int64_t outer_stride[kMaxOps][CT_MAX_DIMS - 2];
  uint32_t lds_mask;    // bit k: operand k is unit-stride along B and goes through LDS
  uint32_t const_mask;
  uint32_t streaming;   // non-temporal loads and stores (see VecArgs)
  uint64_t cbits[kMaxOps];
};

// Largest element size among a functor's types (unused inputs alias Out).
template <class F> struct elem_sizes {
  static constexpr size_t m01 = sizeof(typename F::In0) > sizeof(typename F::In1) ? sizeof(typename F::In0) : sizeof(typename F::In1);
  static constexpr size_t m012 = m01 > sizeof(typename F::In2) ? m01 : sizeof(typename F::In2);
  static constexpr size_t max_in = m012;
  static constexpr size_t max_all = m012 > sizeof(typename F::Out) ? m012 : sizeof(typename F::Out);
};
// Tile shape: TA elements along A (the destination's unit-stride axis) by TB
// elements along B (the axis the transposed inputs are unit-stride along).
// The longer edge goes to the side with more streams.  Transposed inputs in the
// majority (or level with the directly readable streams, the destination
// included): 32 x 128, 512-byte source segments, which measured 83 % of peak on
// a transposing float copy against 76 % for 256-byte ones, while shrinking the
// written segments from 256 to 128 bytes cost about 1 %.  Directly readable
// streams in the majority (WIDE_A): the mirror image, so that they and the
// destination move in 512-byte segments.
// (A 64 x 128 tile for three transposed inputs, 256-byte written segments,
// measured the same 70 % of peak as 32 x 128.)
enum TileShape { TS_WIDE_B = 0, TS_WIDE_A = 1 };
template <class F, int SHAPE> struct tile_shape {
  static constexpr bool wide_elem = elem_sizes<F>::max_in > 4;
  static constexpr int ta = SHAPE == TS_WIDE_A ? (wide_elem ? 64 : 128) : 32;
  static constexpr int tb = SHAPE == TS_WIDE_A ? 32 : (wide_elem ? 64 : 128);
};
constexpr size_t tile_slot_bytes(size_t elem, int ta, int tb) { return ((elem * ta * (tb + 1)) + 15) & ~size_t(15); }

// Reads this lane's share of a TA x TB tile of an operand that is
// unit-stride along B: lane tx walks B (TB consecutive elements per source
// row), the block's ROWS lane rows walk A.  The pointer advances by a constant
// step.
template <class T, int TA, int TB, bool FULL, bool STREAM>
__device__ __forceinline__ void tile_read(T* v, const T* p, int64_t step, uint32_t a_left, bool b_ok, int ty) {
  constexpr int ROWS = kBlock / TB;
  constexpr int IT = TA / ROWS;
#pragma unroll
  for (int i = 0; i < IT; ++i) {
    if (FULL || (b_ok && (uint32_t)(ty + i * ROWS) < a_left)) {
      if constexpr (STREAM) v[i] = nt_load(p + (int64_t)i * step);
      else v[i] = p[(int64_t)i * step];
    } else {
      v[i] = T{};
    }
  }
}

// Reads this lane's share of the tile of an operand that needs no transposition:
// element i of the lane is (a = wx, b = wy + i * rows_w), the write-phase layout.
template <class T, int IT, bool FULL>
__device__ __forceinline__ void tile_read_direct(T* v, const T* q, int64_t step, bool a_ok, uint32_t b_left, int wy,
                                                 int rows_w) {
#pragma unroll
  for (int i = 0; i < IT; ++i) {
    if (FULL || (a_ok && (uint32_t)(wy + i * rows_w) < b_left)) v[i] = q[(int64_t)i * step];
    else v[i] = T{};
  }
}

// Transposes the lane values through the block's single LDS tile (rows padded
// to TB + 1 elements: conflict-free both ways).  On entry v[i] holds element
// (a = ty + i*ROWS_R, b = tx) with tx = t % TB; on exit element
// (a = wx, b = wy + i*ROWS_W) with wx = t % TA.
template <class T, int TA, int TB>
__device__ __forceinline__ void tile_transpose(T* v, char* smem, bool need_sync_before) {
  constexpr int ROWS_R = kBlock / TB, ROWS_W = kBlock / TA;
  constexpr int IT = TA / ROWS_R;
  static_assert(IT == TB / ROWS_W, "both phases move the same number of elements per lane");
  const int tx = threadIdx.x % TB, ty = threadIdx.x / TB;
  const int wx = threadIdx.x % TA, wy = threadIdx.x / TA;
  T* lds = reinterpret_cast<T*>(smem);
  if (need_sync_before) __syncthreads();
#pragma unroll
  for (int i = 0; i < IT; ++i) lds[(ty + i * ROWS_R) * (TB + 1) + tx] = v[i];
  __syncthreads();
#pragma unroll
  for (int i = 0; i < IT; ++i) v[i] = lds[wx * (TB + 1) + wy + i * ROWS_W];
}

template <class F, bool FULL, bool STREAM, int SHAPE>
__device__ __forceinline__ void tile_body(const F& f, const TileArgs& a, const int64_t* off, uint32_t a0, uint32_t b0,
                                          char* smem) {
  using Out = typename F::Out;
  using In0 = typename F::In0;
  using In1 = typename F::In1;
  using In2 = typename F::In2;
  constexpr int NIN = F::NIN;
  constexpr int TA = tile_shape<F, SHAPE>::ta, TB = tile_shape<F, SHAPE>::tb;
  constexpr int ROWS_R = kBlock / TB, ROWS_W = kBlock / TA;
  constexpr int IT = TA / ROWS_R;
  const int tx = threadIdx.x % TB, ty = threadIdx.x / TB;
  const int wx = threadIdx.x % TA, wy = threadIdx.x / TA;
  const uint32_t a_left = a.sizeA - a0, b_left = a.sizeB - b0;  // valid extent of this tile
  const bool t0 = NIN >= 1 && ((a.lds_mask >> 1) & 1u), t1 = NIN >= 2 && ((a.lds_mask >> 2) & 1u),
             t2 = NIN >= 3 && ((a.lds_mask >> 3) & 1u);

  // Addresses of the write phase, formed now: nothing after the LDS rounds needs a kernel argument again.
  const bool a_ok = (uint32_t)wx < a_left;
  Out* dp = reinterpret_cast<Out*>(a.ptr[0]) + off[0] + (int64_t)(a0 + wx) * a.strideA[0] + (int64_t)(b0 + wy) * a.strideB[0];
  const int64_t dstep = (int64_t)ROWS_W * a.strideB[0];
  const In0* q0 = nullptr;
  const In1* q1 = nullptr;
  const In2* q2 = nullptr;
  int64_t s0 = 0, s1 = 0, s2 = 0;
  In0 c0{};
  In1 c1{};
  In2 c2{};
  if constexpr (NIN >= 1) {
    if ((a.const_mask >> 1) & 1u) c0 = const_from_bits<In0>(a.cbits[1]);
    else if (!t0) { q0 = reinterpret_cast<const In0*>(a.ptr[1]) + off[1] + (int64_t)(a0 + wx) * a.strideA[1] + (int64_t)(b0 + wy) * a.strideB[1]; s0 = (int64_t)ROWS_W * a.strideB[1]; }
  }
  if constexpr (NIN >= 2) {
    if ((a.const_mask >> 2) & 1u) c1 = const_from_bits<In1>(a.cbits[2]);
    else if (!t1) { q1 = reinterpret_cast<const In1*>(a.ptr[2]) + off[2] + (int64_t)(a0 + wx) * a.strideA[2] + (int64_t)(b0 + wy) * a.strideB[2]; s1 = (int64_t)ROWS_W * a.strideB[2]; }
  }
  if constexpr (NIN >= 3) {
    if ((a.const_mask >> 3) & 1u) c2 = const_from_bits<In2>(a.cbits[3]);
    else if (!t2) { q2 = reinterpret_cast<const In2*>(a.ptr[3]) + off[3] + (int64_t)(a0 + wx) * a.strideA[3] + (int64_t)(b0 + wy) * a.strideB[3]; s2 = (int64_t)ROWS_W * a.strideB[3]; }
  }

  // phase 1: every load of every transposed operand is issued before the first LDS round
  In0 v0[IT];
  In1 v1[IT];
  In2 v2[IT];
  const bool b_ok = (uint32_t)tx < b_left;
  if constexpr (NIN >= 1)
    if (t0) tile_read<In0, TA, TB, FULL, STREAM>(v0, reinterpret_cast<const In0*>(a.ptr[1]) + off[1] + (int64_t)(a0 + ty) * a.strideA[1] + (b0 + tx),
                                     (int64_t)ROWS_R * a.strideA[1], a_left, b_ok, ty);
  if constexpr (NIN >= 2)
    if (t1) tile_read<In1, TA, TB, FULL, STREAM>(v1, reinterpret_cast<const In1*>(a.ptr[2]) + off[2] + (int64_t)(a0 + ty) * a.strideA[2] + (b0 + tx),
                                     (int64_t)ROWS_R * a.strideA[2], a_left, b_ok, ty);
  if constexpr (NIN >= 3)
    if (t2) tile_read<In2, TA, TB, FULL, STREAM>(v2, reinterpret_cast<const In2*>(a.ptr[3]) + off[3] + (int64_t)(a0 + ty) * a.strideA[3] + (b0 + tx),
                                     (int64_t)ROWS_R * a.strideA[3], a_left, b_ok, ty);
  // operands that are read along A directly (not through LDS) are fetched now as well, so
  // that their latency overlaps the transposed operands' instead of following the LDS rounds
  if constexpr (NIN >= 1)
    if (q0) tile_read_direct<In0, IT, FULL>(v0, q0, s0, a_ok, b_left, wy, ROWS_W);
  if constexpr (NIN >= 2)
    if (q1) tile_read_direct<In1, IT, FULL>(v1, q1, s1, a_ok, b_left, wy, ROWS_W);
  if constexpr (NIN >= 3)
    if (q2) tile_read_direct<In2, IT, FULL>(v2, q2, s2, a_ok, b_left, wy, ROWS_W);
  bool used = false;
  if constexpr (NIN >= 1) if (t0) { tile_transpose<In0, TA, TB>(v0, smem, used); used = true; }
  if constexpr (NIN >= 2) if (t1) { tile_transpose<In1, TA, TB>(v1, smem, used); used = true; }
  if constexpr (NIN >= 3) if (t2) { tile_transpose<In2, TA, TB>(v2, smem, used); used = true; }

  // phase 2: lane wx walks A (the destination's unit-stride axis), lane rows walk B
#pragma unroll
  for (int i = 0; i < IT; ++i) {
    const int row = wy + i * ROWS_W;
    if (FULL || (a_ok && (uint32_t)row < b_left)) {
      In0 p0 = c0;
      In1 p1 = c1;
      In2 p2 = c2;
      if constexpr (NIN >= 1) { if (t0 || q0) p0 = v0[i]; }
      if constexpr (NIN >= 2) { if (t1 || q1) p1 = v1[i]; }
      if constexpr (NIN >= 3) { if (t2 || q2) p2 = v2[i]; }
      // plain stores: element-wide non-temporal stores measured slower here
      dp[(int64_t)i * dstep] = f(p0, p1, p2);
    }
  }
}

// One block per TA x TB tile.  All transposed operands share one LDS tile,
// used in turn, so the LDS footprint (and with it the number of resident
// blocks) does not grow with the operand count.
template <class F, bool STREAM, int SHAPE>
__global__ void __launch_bounds__(kBlock) ew_tile_kernel(const F f, const TileArgs a) {
  constexpr int NIN = F::NIN;
  constexpr int TA = tile_shape<F, SHAPE>::ta, TB = tile_shape<F, SHAPE>::tb;
  extern __shared__ __align__(16) char smem[];

  // Every argument the block needs is named here so that the compiler fetches
  // them in one batch before the first branch (see ew_vec_kernel); the code
  // below reads the same values.
  {
    constexpr int K1 = NIN >= 1 ? 1 : 0, K2 = NIN >= 2 ? 2 : 0, K3 = NIN >= 3 ? 3 : 0;
    asm volatile("" ::"s"(a.sizeA), "s"(a.sizeB), "s"(a.tilesA), "s"(a.tilesB), "s"(a.super_a), "s"(a.super_b),
                 "s"(a.n_super), "s"(a.per_fd.d), "s"(a.per_fd.m), "s"(a.per_fd.s), "s"(a.sb_fd.d), "s"(a.sb_fd.m),
                 "s"(a.sb_fd.s), "s"(a.nsb_fd.d), "s"(a.nsb_fd.m), "s"(a.nsb_fd.s), "s"(a.nst_fd.d), "s"(a.nst_fd.m),
                 "s"(a.nst_fd.s), "s"(a.n_outer), "s"(a.lds_mask),
                 "s"(a.const_mask), "s"(a.ptr[0]), "s"(a.ptr[K1]), "s"(a.ptr[K2]), "s"(a.ptr[K3]), "s"(a.strideA[0]),
                 "s"(a.strideA[K1]), "s"(a.strideA[K2]), "s"(a.strideA[K3]), "s"(a.strideB[0]), "s"(a.strideB[K1]),
                 "s"(a.strideB[K2]), "s"(a.strideB[K3]), "s"(a.cbits[K1]), "s"(a.cbits[K2]), "s"(a.cbits[K3]));
  }

  // Block -> tile.  Consecutive block ids land on the eight XCDs in turn, each
  // with its own L2.  The tiles are grouped into super-tiles, long along A (about
  // 2048 elements: 8 KiB of every destination row) and short along B (256-512
  // bytes of every transposed source row), and every XCD works through whole
  // super-tiles: the 128-byte pieces that neighbouring tiles write to one
  // destination row, and the source segments they read, then pass through the
  // same L2 at about the same time.  Measured on transposed [8192,8192] float
  // views against plain row-major block order: :select with three transposed
  // inputs 69 % -> 79 % of peak, x^T + y^T 73 % -> 79 %, :exp 80 % -> 83 %; the
  // mirrored tile gains 5 points on x^T + y with 32 x 4 tiles per super-tile.
  // Dealing single rows of tiles to the XCDs instead loses 3 points.
  // The grid is padded to whole rounds of eight super-tiles; surplus blocks leave at once.
  uint32_t bid, ta, tb;
  {
    const uint32_t xcd = blockIdx.x % kXcds, k = blockIdx.x / kXcds;
    uint32_t round, w, st_in, sta, stb, ia, ib;
    a.per_fd.divmod(k, round, w);
    const uint32_t st = round * kXcds + xcd;
    if (st >= a.n_super) return;
    a.nst_fd.divmod(st, bid, st_in);
    a.nsb_fd.divmod(st_in, sta, stb);
    a.sb_fd.divmod(w, ia, ib);
    ta = sta * a.super_a + ia;
    tb = stb * a.super_b + ib;
    if (ta >= a.tilesA || tb >= a.tilesB) return;
  }
  int64_t off[kMaxOps] = {0, 0, 0, 0};
  for (int d = 0; d < a.n_outer; ++d) {
    uint32_t q, r;
    a.outer_fd[d].divmod(bid, q, r);
    bid = q;
#pragma unroll
    for (int k = 0; k <= NIN; ++k) off[k] += (int64_t)r * a.outer_stride[k][d];
  }
  const uint32_t a0 = ta * TA, b0 = tb * TB;
  if (a0 + TA <= a.sizeA && b0 + TB <= a.sizeB) tile_body<F, true, STREAM, SHAPE>(f, a, off, a0, b0, smem);
  else tile_body<F, false, STREAM, SHAPE>(f, a, off, a0, b0, smem);
}

// ------------------------------------------------------------------ LACE (planar <-> interleaved)

// A short axis S (2..4 entries: the channels of an image) and a long axis L (the pixels).  An
// operand is either PLANAR, unit-stride along L with any stride along S ([C,H,W]), or LACED,
// unit-stride along S with stride |S| along L ([H,W,C]); a call mixes the two (an image going
// from one layout to the other).  Neither the vector kernel (no common unit-stride axis) nor
// the tile kernel (an edge of 3) fits.
//
// A block takes kBlock * PPT consecutive positions of L with all of S.  In registers a lane
// holds its PPT positions plane by plane (S vectors of PPT elements).  A planar operand is
// read or written as exactly those vectors.  A laced operand's share of the block is one
// contiguous run of S * kBlock vectors: the lanes move it with fully coalesced vector accesses
// (lane i takes vectors i, i + kBlock, ...) and it changes layout on its way through LDS, kept
// there plane by plane: the laced side touches LDS element by element (position = flat / S,
// entry = flat % S, S a compile-time constant), the planar side vector by vector.
struct LaceArgs {
  uint32_t n_long;                 // |L|
  FastDiv per_row_fd;              // blocks per outer row: ceil(|L| / (kBlock * PPT))
  int32_t n_outer;
  FastDiv outer_fd[CT_MAX_DIMS - 2];
  char* ptr[kMaxOps];
  int64_t outer_stride[kMaxOps][CT_MAX_DIMS - 2];
  int64_t plane_stride[kMaxOps];   // planar operands: stride along S
  uint32_t laced_mask;             // bit k: operand k is laced
  uint32_t const_mask;
  uint32_t streaming;              // the call moves more than the caches hold: the stores bypass them
  uint64_t cbits[kMaxOps];
};

constexpr int kLaceMaxShort = 4;
constexpr int kLacePadBytes = 16;  // between the planes in LDS: shifts the banks, keeps vectors aligned

template <int S, int PPT> constexpr size_t lace_lds_bytes(size_t elem) { return S * (kBlock * PPT * elem + kLacePadBytes); }

// Reads one input of the block into registers, plane by plane: x[c].v[p] is entry c of the lane's position p.
template <class T, int S, int PPT>
__device__ __forceinline__ void lace_load(Vec<T, PPT>* x, const T* base, int64_t plane_stride, bool laced, uint32_t l_blk,
                                          uint32_t n_here, char* smem) {
  constexpr uint32_t kPlaneBytes = kBlock * PPT * sizeof(T) + kLacePadBytes;
  const uint32_t lp = threadIdx.x * PPT;
  const bool live = lp < n_here;
  if (!laced) {
    if (live) {
#pragma unroll
      for (int c = 0; c < S; ++c) x[c] = nt_load(reinterpret_cast<const Vec<T, PPT>*>(base + c * plane_stride + l_blk + lp));
    }
    return;
  }
  const Vec<T, PPT>* run = reinterpret_cast<const Vec<T, PPT>*>(base + (int64_t)l_blk * S);
  const uint32_t n_vecs = n_here * S / PPT;
  Vec<T, PPT> v[S];
#pragma unroll
  for (int j = 0; j < S; ++j)
    if (threadIdx.x + j * kBlock < n_vecs) v[j] = nt_load(run + threadIdx.x + j * kBlock);
#pragma unroll
  for (int j = 0; j < S; ++j) {
    const uint32_t vi = threadIdx.x + j * kBlock;
    if (vi < n_vecs) {
#pragma unroll
      for (int e = 0; e < PPT; ++e) {
        const uint32_t flat = vi * PPT + e;
        *reinterpret_cast<T*>(smem + (flat % S) * kPlaneBytes + (flat / S) * sizeof(T)) = v[j].v[e];
      }
    }
  }
  __syncthreads();
  if (live) {
#pragma unroll
    for (int c = 0; c < S; ++c) x[c] = *reinterpret_cast<const Vec<T, PPT>*>(smem + c * kPlaneBytes + lp * sizeof(T));
  }
  __syncthreads();  // the tile is free for the next operand
}

template <class F, int S, int PPT>
__global__ void __launch_bounds__(kBlock) ew_lace_kernel(const F f, const LaceArgs a) {
  using Out = typename F::Out;
  using In0 = typename F::In0;
  using In1 = typename F::In1;
  using In2 = typename F::In2;
  constexpr int NIN = F::NIN;
  __shared__ __align__(16) char smem[lace_lds_bytes<S, PPT>(elem_sizes<F>::max_all)];
  uint32_t row, lb;
  a.per_row_fd.divmod(blockIdx.x, row, lb);
  int64_t off[kMaxOps] = {0, 0, 0, 0};
  for (int d = 0; d < a.n_outer; ++d) {
    uint32_t q, r;
    a.outer_fd[d].divmod(row, q, r);
    row = q;
#pragma unroll
    for (int k = 0; k <= NIN; ++k) off[k] += (int64_t)r * a.outer_stride[k][d];
  }
  const uint32_t l_blk = lb * (uint32_t)(kBlock * PPT);
  const uint32_t left = a.n_long - l_blk;
  const uint32_t n_here = left < (uint32_t)(kBlock * PPT) ? left : (uint32_t)(kBlock * PPT);  // a multiple of PPT
  const uint32_t lp = threadIdx.x * PPT;
  const bool live = lp < n_here;

  Vec<In0, PPT> x0[S];
  Vec<In1, PPT> x1[S];
  Vec<In2, PPT> x2[S];
  const bool c0 = (a.const_mask >> 1) & 1u, c1 = (a.const_mask >> 2) & 1u, c2 = (a.const_mask >> 3) & 1u;
  if constexpr (NIN >= 1)
    if (!c0) lace_load<In0, S, PPT>(x0, reinterpret_cast<const In0*>(a.ptr[1]) + off[1], a.plane_stride[1], (a.laced_mask >> 1) & 1u, l_blk, n_here, smem);
  if constexpr (NIN >= 2)
    if (!c1) lace_load<In1, S, PPT>(x1, reinterpret_cast<const In1*>(a.ptr[2]) + off[2], a.plane_stride[2], (a.laced_mask >> 2) & 1u, l_blk, n_here, smem);
  if constexpr (NIN >= 3)
    if (!c2) lace_load<In2, S, PPT>(x2, reinterpret_cast<const In2*>(a.ptr[3]) + off[3], a.plane_stride[3], (a.laced_mask >> 3) & 1u, l_blk, n_here, smem);

  Vec<Out, PPT> o[S];
#pragma unroll
  for (int c = 0; c < S; ++c)
#pragma unroll
    for (int p = 0; p < PPT; ++p) {
      In0 p0{};
      In1 p1{};
      In2 p2{};
      if constexpr (NIN >= 1) p0 = c0 ? const_from_bits<In0>(a.cbits[1]) : x0[c].v[p];
      if constexpr (NIN >= 2) p1 = c1 ? const_from_bits<In1>(a.cbits[2]) : x1[c].v[p];
      if constexpr (NIN >= 3) p2 = c2 ? const_from_bits<In2>(a.cbits[3]) : x2[c].v[p];
      o[c].v[p] = f(p0, p1, p2);
    }

  Out* dbase = reinterpret_cast<Out*>(a.ptr[0]) + off[0];
  if (!(a.laced_mask & 1u)) {
    if (live) {
#pragma unroll
      for (int c = 0; c < S; ++c) {
        Vec<Out, PPT>* dp = reinterpret_cast<Vec<Out, PPT>*>(dbase + c * a.plane_stride[0] + l_blk + lp);
        if (a.streaming) {
          asm volatile("");  // keeps the two stores apart: merged into one, they lose the hint
          nt_store(o[c], dp);
        } else {
          *dp = o[c];
        }
      }
    }
    return;
  }
  constexpr uint32_t kPlaneBytes = kBlock * PPT * sizeof(Out) + kLacePadBytes;
  if (live) {
#pragma unroll
    for (int c = 0; c < S; ++c) *reinterpret_cast<Vec<Out, PPT>*>(smem + c * kPlaneBytes + lp * sizeof(Out)) = o[c];
  }
  __syncthreads();
  Vec<Out, PPT>* run = reinterpret_cast<Vec<Out, PPT>*>(dbase + (int64_t)l_blk * S);
  const uint32_t n_vecs = n_here * S / PPT;
#pragma unroll
  for (int j = 0; j < S; ++j) {
    const uint32_t vi = threadIdx.x + j * kBlock;
    if (vi < n_vecs) {
      Vec<Out, PPT> v;
#pragma unroll
      for (int e = 0; e < PPT; ++e) {
        const uint32_t flat = vi * PPT + e;
        v.v[e] = *reinterpret_cast<const Out*>(smem + (flat % S) * kPlaneBytes + (flat / S) * sizeof(Out));
      }
      if (a.streaming) {
        asm volatile("");
        nt_store(v, run + vi);
      } else {
        run[vi] = v;
      }
    }
  }
}

// ------------------------------------------------------------------ GENERAL

struct GenArgs {
  int64_t n;
  int32_t nd;
  int32_t need_coords;  // some operand is in per-dimension mode
  FastDiv rmax_fd[CT_MAX_DIMS];
  int64_t rmax[CT_MAX_DIMS];
  GenOperand op[kMaxOps];
  char* ptr[kMaxOps];
  uint64_t cbits[kMaxOps];
};

template <class I>
__device__ __forceinline__ int64_t gen_address(const GenArgs& a, int k, I e, const I* arg) {
  const GenOperand& o = a.op[k];
  switch (o.mode) {
    case 0: return (int64_t)e;
    case 1: return (int64_t)((e / (I)o.amt) % (I)o.ec);
    case 2: return (int64_t)(e % (I)o.ec);
    default: break;
  }
  int64_t off = 0;
  for (int d = 0; d < a.nd; ++d) {
    const int64_t s = o.shape[d];
    if (s == 1) {  // coordinate 0; an index tensor of one element still names the row
      if (o.index[d]) off += (int64_t)o.index[d][0] * o.stride[d];
      continue;
    }
    I c;
    if (s == a.rmax[d]) c = arg[d] - arg[d + 1] * (I)a.rmax[d];
    else c = arg[d] % (I)s;
    const int64_t ci = o.index[d] ? (int64_t)o.index[d][c] : (int64_t)c;
    off += ci * o.stride[d];
  }
  return off;
}

// Address of logical element e through one of the reference's address objects,
// with plain 64-bit division (used off the hot paths: reductions' fallback and
// the serial accumulate).
__device__ __forceinline__ int64_t ref_address(const GenOperand& o, int nd, const int64_t* rmax, int64_t e) {
  switch (o.mode) {
    case 0: return e;
    case 1: return (e / o.amt) % o.ec;
    case 2: return e % o.ec;
    default: break;
  }
  int64_t off = 0, arg = e;
  for (int d = 0; d < nd; ++d) {
    const int64_t c = arg % o.shape[d];
    arg /= rmax[d];
    off += (o.index[d] ? (int64_t)o.index[d][c] : c) * o.stride[d];
  }
  return off;
}

template <class F, class I>
__global__ void __launch_bounds__(kBlock) ew_gen_kernel(const F f, const GenArgs a) {
  using Out = typename F::Out;
  using In0 = typename F::In0;
  using In1 = typename F::In1;
  using In2 = typename F::In2;
  constexpr int NIN = F::NIN;
  const I n = (I)a.n;
  const I step = (I)gridDim.x * kBlock;
  for (I e = (I)blockIdx.x * kBlock + threadIdx.x; e < n; e += step) {
    I arg[CT_MAX_DIMS + 1];
    if (a.need_coords) {
      arg[0] = e;
      for (int d = 0; d < a.nd; ++d) {
        if constexpr (sizeof(I) == 4) arg[d + 1] = a.rmax_fd[d].div(arg[d]);
        else arg[d + 1] = arg[d] / (I)a.rmax[d];
      }
    }
    In0 p0{};
    In1 p1{};
    In2 p2{};
    if constexpr (NIN >= 1)
      p0 = (a.op[1].mode == 4) ? const_from_bits<In0>(a.cbits[1])
                               : reinterpret_cast<const In0*>(a.ptr[1])[gen_address<I>(a, 1, e, arg)];
    if constexpr (NIN >= 2)
      p1 = (a.op[2].mode == 4) ? const_from_bits<In1>(a.cbits[2])
                               : reinterpret_cast<const In1*>(a.ptr[2])[gen_address<I>(a, 2, e, arg)];
    if constexpr (NIN >= 3)
      p2 = (a.op[3].mode == 4) ? const_from_bits<In2>(a.cbits[3])
                               : reinterpret_cast<const In2*>(a.ptr[3])[gen_address<I>(a, 3, e, arg)];
    reinterpret_cast<Out*>(a.ptr[0])[gen_address<I>(a, 0, e, arg)] = f(p0, p1, p2);
  }
}

// One lane applies the updates for e = 0, 1, ... in order.  This is the
// reference's serial accumulate loop (cpu/tensor_math.clj:234, 324, 399) kept
// for the cases where several e hit one destination address in an order that
// cannot be recovered from the dimensions (indirectly indexed destinations).
template <class F>
__global__ void ew_serial_kernel(const F f, const GenArgs a) {
  using Out = typename F::Out;
  using In0 = typename F::In0;
  using In1 = typename F::In1;
  using In2 = typename F::In2;
  constexpr int NIN = F::NIN;
  if (blockIdx.x != 0 || threadIdx.x != 0) return;
  for (int64_t e = 0; e < a.n; ++e) {
    In0 p0{};
    In1 p1{};
    In2 p2{};
    if constexpr (NIN >= 1)
      p0 = (a.op[1].mode == 4) ? const_from_bits<In0>(a.cbits[1])
                               : reinterpret_cast<const In0*>(a.ptr[1])[ref_address(a.op[1], a.nd, a.rmax, e)];
    if constexpr (NIN >= 2)
      p1 = (a.op[2].mode == 4) ? const_from_bits<In1>(a.cbits[2])
                               : reinterpret_cast<const In1*>(a.ptr[2])[ref_address(a.op[2], a.nd, a.rmax, e)];
    if constexpr (NIN >= 3)
      p2 = (a.op[3].mode == 4) ? const_from_bits<In2>(a.cbits[3])
                               : reinterpret_cast<const In2*>(a.ptr[3])[ref_address(a.op[3], a.nd, a.rmax, e)];
    reinterpret_cast<Out*>(a.ptr[0])[ref_address(a.op[0], a.nd, a.rmax, e)] = f(p0, p1, p2);
  }
}

// ------------------------------------------------------------------ launcher

struct EwOperand {
  const void* ptr;      // nullptr: constant
  const ct_dims* dims;
  int elem_size;
  uint64_t cbits;       // constant value, already in the operand's element type
};

// A call of 2^31 elements or more is cut into pieces along its slowest axis (split_leading), each
// run on its own: the kernels index with 32 bits.
struct EwPiece {
  const void* ptr[kMaxOps];
  ct_dims dims[kMaxOps];
  int64_t n;
};
bool split_leading(const EwOperand* ops, int n_ops, int64_t n, int64_t limit, std::vector<EwPiece>* pieces);

int prepare_vec(const Plan& plan, const EwOperand* ops, int vmax, VecArgs* main_args, int* main_vec,
                VecArgs* tail_args, bool* has_tail);
int prepare_tile(const Plan& plan, const EwOperand* ops, int tile_a_edge, int tile_b_edge, bool wide_a, TileArgs* args,
                 size_t* lds_bytes,
                 uint32_t* grid);
int prepare_gen(const Plan& plan, const EwOperand* ops, GenArgs* args, bool* use64, uint32_t* grid);
// Recognises the planar <-> interleaved pattern in a regular plan that neither the vector nor the
// tile kernel took.  Returns false when it does not apply; otherwise fills the arguments, the
// short axis' extent (2..kLaceMaxShort) and the vector width (vmax or 1) and the grid.
bool prepare_lace(const Plan& plan, const EwOperand* ops, int vmax, LaceArgs* args, int* n_short, int* ppt, uint32_t* grid);
bool prepare_ragged(const Plan& plan, const EwOperand* ops, int vmax, RaggedArgs* args);
bool prepare_vecu(const Plan& plan, const EwOperand* ops, int vmax, VecArgs* args, uint32_t* inner_elems);
bool prepare_span(const Plan& plan, const EwOperand* ops, int vmax, SpanArgs* args);

// Functors that the lace kernel is built for declare `static constexpr bool kLace = true`.
template <class F, class = void> struct has_lace : std::false_type {};
template <class F> struct has_lace<F, std::enable_if_t<F::kLace>> : std::true_type {};

// Flat, every tensor operand unit-stride and no constants: the contiguous form.
// Vectors per lane of the flat kernel: 1 when every operand has the same element width.  A
// conversion moves only 16 / ratio bytes per lane and vector on its narrow side; a narrowing one
// (wide loads, narrow stores) takes ratio vectors per lane, at most 4, a widening one 2 from a
// ratio of 4 on.
template <class F> constexpr int flat_vectors_per_lane() {
  size_t mn = sizeof(typename F::Out), mx = sizeof(typename F::Out);
  if (F::NIN >= 1) { mn = sizeof(typename F::In0) < mn ? sizeof(typename F::In0) : mn; mx = sizeof(typename F::In0) > mx ? sizeof(typename F::In0) : mx; }
  if (F::NIN >= 2) { mn = sizeof(typename F::In1) < mn ? sizeof(typename F::In1) : mn; mx = sizeof(typename F::In1) > mx ? sizeof(typename F::In1) : mx; }
  if (F::NIN >= 3) { mn = sizeof(typename F::In2) < mn ? sizeof(typename F::In2) : mn; mx = sizeof(typename F::In2) > mx ? sizeof(typename F::In2) : mx; }
  const int ratio = (int)(mx / mn);
  if (sizeof(typename F::Out) < mx) return ratio > 4 ? 4 : (ratio < 1 ? 1 : ratio);  // narrowing
  return ratio >= 4 ? 2 : 1;  // widening: int -> double ran 3 % slower with two than with one
}

inline bool vec_is_flat(const VecArgs& a, int nin) {
  const uint32_t all = (2u << nin) - 1u;
  return a.n_outer == 0 && a.const_mask == 0 && (a.unit_mask & all) == all && !a.indexed;
}

template <class F, int VEC>
inline void launch_vec_once(hipStream_t s, const F& f, const VecArgs& args) {
  const dim3 grid((uint32_t)((args.total_vecs + kBlock - 1) / kBlock));
  VecArgs a = args;
  a.grouped_blocks = xcd_grouped_blocks(grid.x);
  if (VEC > 1 && vec_is_flat(a, F::NIN)) {
    FlatArgs fa;
    fa.total_vecs = a.total_vecs;
    fa.grouped_blocks = xcd_grouped_blocks(grid.x);
    for (int k = 0; k < kMaxOps; ++k) fa.ptr[k] = a.ptr[k];
    constexpr int kPer = flat_vectors_per_lane<F>();
    const dim3 fgrid((uint32_t)((args.total_vecs + kBlock * kPer - 1) / (kBlock * kPer)));
    fa.grouped_blocks = xcd_grouped_blocks(fgrid.x);
    if (a.streaming == 2) hipLaunchKernelGGL((ew_flat_kernel<F, VEC, 2, kPer>), fgrid, dim3(kBlock), 0, s, f, fa);
    else if (a.streaming) hipLaunchKernelGGL((ew_flat_kernel<F, VEC, 1, kPer>), fgrid, dim3(kBlock), 0, s, f, fa);
    else hipLaunchKernelGGL((ew_flat_kernel<F, VEC, 0, kPer>), fgrid, dim3(kBlock), 0, s, f, fa);
    return;
  }
  if (a.indexed) {
    // gathered rows are re-read wherever labels repeat and scattered rows are not written in
    // order: plain accesses, plain block order.  Four vectors per lane (from four rows when a row is
    // a block wide): a lane's look-ups and then its row loads are in flight together, which hides
    // the extra trip to memory that the look-up costs.  Gathering 65536 rows of 4 KiB: one vector
    // per lane 69 % of peak, two 73 %, four 79 %, eight 73 %.
    a.grouped_blocks = 0;
    constexpr int kPer = 4;
    const dim3 grid_per((uint32_t)((args.total_vecs + kBlock * kPer - 1) / (kBlock * kPer)));
    hipLaunchKernelGGL((ew_vec_kernel<F, VEC, 0, -1, true, kPer>), grid_per, dim3(kBlock), 0, s, f, a);
    return;
  }
  // The compile-time operand kinds are worth a few percent of memory bandwidth; integer tensors,
  // whose arithmetic sets their pace, keep the one general form (an eighth of the library's size
  // was specialisations of integer functors).
  if constexpr (VEC > 1 && std::is_floating_point<typename F::Out>::value) {
    // the operand kinds of this call, in vec_kinds' encoding
    int kinds = 0;
    for (int k = 1; k <= F::NIN; ++k) {
      const int kind = ((a.const_mask >> k) & 1u) ? VK_CONST
                       : ((a.unit_mask >> k) & 1u) ? (((a.nt_mask >> k) & 1u) ? VK_STREAM : VK_CACHED)
                                                   : VK_SCALAR;
      kinds |= kind << (2 * (k - 1));
      // A row that every row of the call re-reads (a bias) stays in the plain order in the largest
      // calls, where a die keeps meeting the same columns of it: regrouped, the bias add of a
      // [16384, 16384] matrix lost 6 points (74 % against 80 %); at [8192, 8192] the grouped order is
      // 4 points ahead (84 % against 80 %), below that the two are level.
      if (kind == VK_CACHED && a.streaming == 2) a.grouped_blocks = 0;
    }
#define CT_VEC_KINDS(K)                                                                                  \
  if (kinds == (K)) {                                                                                    \
    if (a.streaming == 2) hipLaunchKernelGGL((ew_vec_kernel<F, VEC, 2, (K)>), grid, dim3(kBlock), 0, s, f, a); \
    else if (a.streaming) hipLaunchKernelGGL((ew_vec_kernel<F, VEC, 1, (K)>), grid, dim3(kBlock), 0, s, f, a); \
    else hipLaunchKernelGGL((ew_vec_kernel<F, VEC, 0, (K)>), grid, dim3(kBlock), 0, s, f, a);            \
    return;                                                                                              \
  }
    if constexpr (F::NIN == 1) {
      CT_VEC_KINDS(vec_kinds(VK_STREAM))
    } else if constexpr (F::NIN == 2) {
      CT_VEC_KINDS(vec_kinds(VK_STREAM, VK_STREAM))
      CT_VEC_KINDS(vec_kinds(VK_STREAM, VK_CACHED))
      CT_VEC_KINDS(vec_kinds(VK_STREAM, VK_SCALAR))
      CT_VEC_KINDS(vec_kinds(VK_STREAM, VK_CONST))
      CT_VEC_KINDS(vec_kinds(VK_CONST, VK_STREAM))
    } else if constexpr (F::NIN == 3) {
      CT_VEC_KINDS(vec_kinds(VK_STREAM, VK_STREAM, VK_STREAM))
    }
#undef CT_VEC_KINDS
  }
  if (a.streaming) hipLaunchKernelGGL((ew_vec_kernel<F, VEC, 1>), grid, dim3(kBlock), 0, s, f, a);
  else hipLaunchKernelGGL((ew_vec_kernel<F, VEC, 0>), grid, dim3(kBlock), 0, s, f, a);
}

// A flat call longer than one launch's 32-bit vector index is walked in pieces.
template <class F, int VEC>
inline void launch_vec(hipStream_t s, const F& f, const VecArgs& a) {
  if (a.total_vecs == 0) return;
  if (a.n_outer > 0 || a.total_vecs <= (uint64_t)kVecLaunchMax) {
    launch_vec_once<F, VEC>(s, f, a);
    return;
  }
  const size_t elem[kMaxOps] = {sizeof(typename F::Out), sizeof(typename F::In0), sizeof(typename F::In1),
                                sizeof(typename F::In2)};
  for (uint64_t first = 0; first < a.total_vecs; first += (uint64_t)kVecLaunchMax) {
    VecArgs piece = a;
    piece.total_vecs = std::min<uint64_t>((uint64_t)kVecLaunchMax, a.total_vecs - first);
    for (int k = 0; k <= F::NIN; ++k)
      if (((a.unit_mask >> k) & 1u) && !((a.const_mask >> k) & 1u)) piece.ptr[k] = a.ptr[k] + first * VEC * elem[k];
    launch_vec_once<F, VEC>(s, f, piece);
  }
}

// ops[0] is the destination; ops[1..NIN] the inputs in functor order.
template <class F>
int launch_elementwise(hipStream_t s, const F& f, const EwOperand* ops, int64_t n) {
  constexpr int NIN = F::NIN;
  if (n == 0) return CT_OK;
  if (n >= (int64_t(1) << 31)) {
    // Beyond what a 32-bit index counts the fast kernels do not apply as they are (only the
    // per-element one has a 64-bit form, at a hundredth of the memory rate): the call is run as
    // pieces of at most 2^30 elements along its slowest axis, each on the kernel of its shape.
    std::vector<EwPiece> pieces;
    if (split_leading(ops, NIN + 1, n, int64_t(1) << 30, &pieces)) {
      for (const EwPiece& piece : pieces) {
        EwOperand sub[kMaxOps];
        for (int k = 0; k <= NIN; ++k) sub[k] = {piece.ptr[k], ops[k].dims ? &piece.dims[k] : nullptr, ops[k].elem_size, ops[k].cbits};
        if (int rc = launch_elementwise(s, f, sub, piece.n)) return rc;
      }
      return CT_OK;
    }
  }
  OperandIn in[kMaxOps];
  for (int k = 0; k <= NIN; ++k) in[k] = {ops[k].ptr, ops[k].dims, ops[k].elem_size};
  Plan plan;
  if (int rc = build_plan(in, NIN + 1, n, &plan)) return rc;

  constexpr int VMAX = 16 / (int)elem_sizes<F>::max_all;

  if (plan.kind == PK_VEC) {
    VecArgs main_args, tail_args;
    int vec = 1;
    bool has_tail = false;
    if (int rc = prepare_vec(plan, ops, VMAX, &main_args, &vec, &tail_args, &has_tail)) return rc;
    if constexpr (has_lace<F>::value && F::NIN == 1) {
      SpanArgs sa;
      if (prepare_span(plan, ops, VMAX, &sa)) {
        note_kernel("span");
        hipLaunchKernelGGL((ew_span_kernel<F, VMAX>), dim3((sa.rows + sa.rows_per_block - 1) / sa.rows_per_block), dim3(kBlock), 0, s, f, sa);
        return after_launch(s);
      }
    }
    if constexpr (VMAX > 1) {
      RaggedArgs ra;
      if (vec == 1 && prepare_ragged(plan, ops, VMAX, &ra)) {
        note_kernel("ragged");
        const dim3 grid((uint32_t)(((int64_t)ra.n + (int64_t)VMAX * kBlock - 1) / ((int64_t)VMAX * kBlock)));
        if (ra.streaming) hipLaunchKernelGGL((ew_ragged_kernel<F, VMAX, true>), grid, dim3(kBlock), 0, s, f, ra);
        else hipLaunchKernelGGL((ew_ragged_kernel<F, VMAX, false>), grid, dim3(kBlock), 0, s, f, ra);
        return after_launch(s);
      }
    }
    if constexpr (VMAX > 1) {
      VecArgs ua;
      uint32_t inner_elems = 0;
      if (vec == 1 && prepare_vecu(plan, ops, VMAX, &ua, &inner_elems)) {
        note_kernel("vecu");
        hipLaunchKernelGGL((ew_vecu_kernel<F, VMAX>), dim3((uint32_t)((ua.total_vecs + kBlock - 1) / kBlock)), dim3(kBlock), 0, s,
                           f, ua, inner_elems);
        return after_launch(s);
      }
    }
    if (vec == VMAX && VMAX > 1) {
      note_kernel("vec");
      launch_vec<F, VMAX>(s, f, main_args);
      if (has_tail) launch_vec<F, 1>(s, f, tail_args);
    } else {
      note_kernel("vec1");
      launch_vec<F, 1>(s, f, main_args);
    }
    return after_launch(s);
  }
  if (plan.kind == PK_TILE) {
    TileArgs ta;
    size_t lds = 0;
    uint32_t grid = 0;
    // streams read or written along A (the destination among them) against those read along B
    int along_a = 1, along_b = 0;
    for (int k = 1; k < plan.n_ops; ++k) {
      if (plan.via_lds[k]) ++along_b;
      else if (ops[k].ptr && plan.canon.stride[k][0] != 0) ++along_a;
    }
    // (a tie of two against two also runs better mirrored: 69 % against 65 %; one against one, a
    // transposing unary op, does not)
    const int shape = (F::NIN >= 2 && (along_a > along_b || (along_a == along_b && along_a >= 2))) ? TS_WIDE_A : TS_WIDE_B;
    const int tile_a = shape == TS_WIDE_A ? tile_shape<F, TS_WIDE_A>::ta : tile_shape<F, TS_WIDE_B>::ta;
    const int tile_b = shape == TS_WIDE_A ? tile_shape<F, TS_WIDE_A>::tb : tile_shape<F, TS_WIDE_B>::tb;
    if (int rc = prepare_tile(plan, ops, tile_a, tile_b, shape == TS_WIDE_A, &ta, &lds, &grid)) return rc;
    note_kernel(shape == TS_WIDE_A ? "tile_wide_a" : "tile");
#define CT_TILE_LAUNCH(SHAPE_)                                                                                    \
  do {                                                                                                            \
    if (ta.streaming) hipLaunchKernelGGL((ew_tile_kernel<F, true, SHAPE_>), dim3(grid), dim3(kBlock), lds, s, f, ta); \
    else hipLaunchKernelGGL((ew_tile_kernel<F, false, SHAPE_>), dim3(grid), dim3(kBlock), lds, s, f, ta);          \
  } while (0)
    if constexpr (F::NIN >= 2) {
      if (shape == TS_WIDE_A) { CT_TILE_LAUNCH(TS_WIDE_A); return after_launch(s); }
    }
    CT_TILE_LAUNCH(TS_WIDE_B);
#undef CT_TILE_LAUNCH
    return after_launch(s);
  }
  if constexpr (has_lace<F>::value) {
    LaceArgs la;
    int n_short = 0, ppt = 1;
    uint32_t lgrid = 0;
    if (plan.regular && prepare_lace(plan, ops, VMAX, &la, &n_short, &ppt, &lgrid)) {
      note_kernel(ppt > 1 ? "lace" : "lace1");
#define CT_LACE(S_)                                                                                          \
  case S_:                                                                                                   \
    if (ppt > 1) hipLaunchKernelGGL((ew_lace_kernel<F, S_, VMAX>), dim3(lgrid), dim3(kBlock), 0, s, f, la);  \
    else hipLaunchKernelGGL((ew_lace_kernel<F, S_, 1>), dim3(lgrid), dim3(kBlock), 0, s, f, la);             \
    break
      switch (n_short) {
        CT_LACE(2);
        CT_LACE(3);
        CT_LACE(4);
        default: return set_error(CT_ERR_INVALID, "internal: lace extent %d", n_short);
      }
#undef CT_LACE
      return after_launch(s);
    }
  }
  GenArgs ga;
  bool use64 = false;
  uint32_t grid = 0;
  if (int rc = prepare_gen(plan, ops, &ga, &use64, &grid)) return rc;
  note_kernel(use64 ? "general64" : "general");
  if (use64) hipLaunchKernelGGL((ew_gen_kernel<F, uint64_t>), dim3(grid), dim3(kBlock), 0, s, f, ga);
  else hipLaunchKernelGGL((ew_gen_kernel<F, uint32_t>), dim3(grid), dim3(kBlock), 0, s, f, ga);
  return after_launch(s);
}

// Serial, order-preserving execution of F (see ew_serial_kernel).
template <class F>
int launch_elementwise_serial(hipStream_t s, const F& f, const EwOperand* ops, int64_t n) {
  constexpr int NIN = F::NIN;
  if (n == 0) return CT_OK;
  OperandIn in[kMaxOps];
  for (int k = 0; k <= NIN; ++k) in[k] = {ops[k].ptr, ops[k].dims, ops[k].elem_size};
  Plan plan;
  if (int rc = build_plan(in, NIN + 1, n, &plan, true)) return rc;
  GenArgs ga;
  bool use64 = false;
  uint32_t grid = 0;
  if (int rc = prepare_gen(plan, ops, &ga, &use64, &grid)) return rc;
  note_kernel("serial");
  hipLaunchKernelGGL((ew_serial_kernel<F>), dim3(1), dim3(64), 0, s, f, ga);
  return after_launch(s);
}

}  // namespace cthip
