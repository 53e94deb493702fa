// ops_pool.hip -- pooling-forward! / pooling-backward!
// (src/cortex/tensor/math.clj:221-236) for packed [batch, channels, height, width]
// float and double buffers, with the values of the CPU backend
// (src/cortex/compute/cpu/tensor_math.clj:1153-1284, 1800-1866), whose window
// walk is src/cortex/nn/impl.clj:8-96:
//
//   for every output (y, x): rel = (y, x) * stride - pad; the taps (k_y, k_x) are
//   visited row by row; a tap beyond the PADDED input is skipped, a tap in the
//   padding reads 0, and every step rounds to the tensor's type.
//     max          tap 0 sets the value, a later tap replaces it when greater
//     avg          value = T(value + tap / (kw * kh)), starting from 0 at tap 0
//     avg-exc-pad  value = T(value + tap / (taps inside the input)), starting from
//                  what the output buffer holds
//
// The reference's backward bodies scatter: they walk the same windows and add
// into the input gradient one tap at a time, so an input under several windows
// receives their terms in increasing (y, x) order of the windows, on top of what
// the gradient buffer held.  Here every input element gathers its own terms in
// that order, which gives the same roundings with no atomics: one lane per
// input element, which reads the few (output, output gradient) pairs covering
// it out of the caches and the gradient and input once from memory.
//
// Both directions are streams of the large tensor (the input, or the input and
// its gradient) plus the smaller pooled one: HBM-bound.  A launch covers at most
// 2^31 - 1 elements of either tensor so that all index arithmetic is 32-bit with
// multiply-high divisions; the host walks larger batches in several launches.
//
// Kernel families, most specific first:
//   tile2    2 x 2 windows that tile the input exactly: no LDS, a lane takes two
//            neighbouring windows as 16-byte pieces of two input rows.
//   padded   forward, 2 x 2 and 3 x 3 windows that stay inside the padded input:
//            a block's rows are staged in an LDS tile that holds the zero padding
//            itself, so that the taps need no tests.
//   band     everything else that fits the LDS budget: a block takes a band of
//            destination rows of one plane (or several whole small planes); the
//            rows of the other tensor that the band touches are one contiguous
//            piece of memory, copied into LDS with aligned 16-byte loads, and the
//            windows are read from there, so that global memory sees only linear
//            streams.  The backward pass streams the gradient in 16-byte pieces.
//   direct   rows too long for the LDS budget: one lane per destination element
//            reads its windows from global memory.
//
// Division.  The averages divide every tap by an integer count d and round the
// quotient to double before the addition.  For float tensors and d <= 255 the
// quotient is computed as q = a * y, r = fma(-d, q, a), q' = fma(r, y, q) with
// y = RN(1 / d): r is exact (a has 24 significant bits, d * q at most 8 + 53, and
// the difference is below 2^9 ulp(q)), so a / d = q + r / d exactly and
// q + r * y differs from it by less than 2^-50 ulp(q); a / d cannot lie that close
// to a rounding boundary m of doubles without being m, because a - m * d is a
// multiple of ulp(q) / 2, and it cannot be m, because m * d has at least 54
// significant bits and a has 24.  So q' = RN(a / d), the value the JVM computes;
// zeros, infinities and NaN take q itself.  Doubles and larger windows divide.
#include <algorithm>

#include "common.h"

using namespace cthip;

namespace {

constexpr int kBlock = 256;

struct PoolArgs {
  const void* in;
  const void* out_values;  // backward: the forward result
  const void* out_grad;    // backward
  void* dest;              // forward: output; backward: input gradient
  uint32_t total;          // elements of dest this launch covers
  int32_t in_h, in_w, out_h, out_w;
  int32_t kw, kh, px, py, sx, sy;
  uint32_t in_plane, out_plane;
  uint32_t load_prev;      // forward: start from what the output holds
  FastDiv row_fd, plane_fd;  // of dest
  FastDiv sx_fd, sy_fd;      // backward
};

// Taps of the window at `rel` that lie inside the input (impl.clj:57-70).
__device__ __forceinline__ int32_t taps_inside(int32_t rel, int32_t k, int32_t extent) {
  const int32_t over = max(0, rel + k - extent), under = min(rel, 0);
  return max(0, k - over + under);
}

template <class T, int OP>
__global__ void __launch_bounds__(kBlock) pool_forward_kernel(const PoolArgs a) {
  const uint32_t e = blockIdx.x * kBlock + threadIdx.x;
  if (e >= a.total) return;
  uint32_t plane, r, oy, ox;
  a.plane_fd.divmod(e, plane, r);
  a.row_fd.divmod(r, oy, ox);
  const T* ip = reinterpret_cast<const T*>(a.in) + (int64_t)plane * a.in_plane;
  T* out = reinterpret_cast<T*>(a.dest);
  const int32_t rel_x = (int32_t)ox * a.sx - a.px, rel_y = (int32_t)oy * a.sy - a.py;
  T acc = (OP == CT_POOL_AVG_EXC_PAD || a.load_prev) ? out[e] : (T)0;
  double divisor = (double)(a.kw * a.kh);
  if (OP == CT_POOL_AVG_EXC_PAD)
    divisor = (double)(taps_inside(rel_x, a.kw, a.in_w) * taps_inside(rel_y, a.kh, a.in_h));
  for (int32_t ky = 0; ky < a.kh; ++ky) {
    const int32_t iy = rel_y + ky;
    if (iy >= a.in_h + a.py) break;  // iy >= -pad_y always holds
    const bool row_inside = iy >= 0 && iy < a.in_h;
    const T* row = ip + (int64_t)iy * a.in_w;
    for (int32_t kx = 0; kx < a.kw; ++kx) {
      const int32_t ix = rel_x + kx;
      if (ix >= a.in_w + a.px) break;
      const T v = (row_inside && ix >= 0 && ix < a.in_w) ? row[ix] : (T)0;
      const bool first = (ky | kx) == 0;
      if (OP == CT_POOL_MAX) {
        if (first || v > acc) acc = v;
      } else if (OP == CT_POOL_AVG) {
        acc = (T)((double)(first ? (T)0 : acc) + (double)v / divisor);
      } else {
        acc = (T)((double)acc + (double)v / divisor);
      }
    }
  }
  out[e] = acc;
}

template <class T, int OP>
__global__ void __launch_bounds__(kBlock) pool_backward_kernel(const PoolArgs a) {
  const uint32_t e = blockIdx.x * kBlock + threadIdx.x;
  if (e >= a.total) return;
  uint32_t plane, r, iy, ix;
  a.plane_fd.divmod(e, plane, r);
  a.row_fd.divmod(r, iy, ix);
  const T* ov = reinterpret_cast<const T*>(a.out_values) + (int64_t)plane * a.out_plane;
  const T* og = reinterpret_cast<const T*>(a.out_grad) + (int64_t)plane * a.out_plane;
  T* ig = reinterpret_cast<T*>(a.dest);
  // Windows o with o * stride - pad <= i < o * stride - pad + k.
  const int32_t ty = (int32_t)iy + a.py, tx = (int32_t)ix + a.px;
  const int32_t oy_hi = min(a.out_h - 1, (int32_t)a.sy_fd.div((uint32_t)ty));
  const int32_t ox_hi = min(a.out_w - 1, (int32_t)a.sx_fd.div((uint32_t)tx));
  const int32_t by = ty - a.kh + 1, bx = tx - a.kw + 1;
  const int32_t oy_lo = by <= 0 ? 0 : (int32_t)a.sy_fd.div((uint32_t)(by + a.sy - 1));
  const int32_t ox_lo = bx <= 0 ? 0 : (int32_t)a.sx_fd.div((uint32_t)(bx + a.sx - 1));
  T acc = ig[e];
  T v = (T)0;
  if (OP == CT_POOL_MAX) v = reinterpret_cast<const T*>(a.in)[e];
  const double kernel_count = (double)(a.kw * a.kh);
  for (int32_t oy = oy_lo; oy <= oy_hi; ++oy) {
    const int32_t exc_h = taps_inside(oy * a.sy - a.py, a.kh, a.in_h);
    for (int32_t ox = ox_lo; ox <= ox_hi; ++ox) {
      const int32_t oa = oy * a.out_w + ox;
      if (OP == CT_POOL_MAX) {
        if (v == ov[oa]) acc = acc + og[oa];
      } else if (OP == CT_POOL_AVG) {
        acc = (T)((double)acc + (double)og[oa] / kernel_count);
      } else {
        const double exc = (double)(taps_inside(ox * a.sx - a.px, a.kw, a.in_w) * exc_h);
        acc = (T)((double)acc + (double)og[oa] / exc);
      }
    }
  }
  ig[e] = acc;
}

// ------------------------------------------------------------------ band kernels

struct BandArgs {
  const void* in;
  const void* out_values;
  const void* out_grad;
  void* dest;
  int32_t in_h, in_w, out_h, out_w;
  int32_t kw, kh, px, py, sx, sy;
  uint32_t in_plane, out_plane;
  uint32_t planes;     // of this launch
  uint32_t pb;         // planes per block; above 1 a block takes whole planes
  uint32_t br;         // destination rows per band
  uint32_t bands;      // bands per plane
  uint32_t cap;        // LDS elements per staged array
  uint32_t load_prev;
  uint32_t fast_div;   // float tensor and kw * kh <= kRecipTable - 1
  double recip;        // RN(1 / (kw * kh))
  FastDiv bands_fd, dest_w_fd, dest_plane_fd, sx_fd, sy_fd;
};

constexpr int kRecipTable = 256;

struct alignas(16) Bytes16 { uint32_t w[4]; };

// Copies src[0, len) to tile[lead, lead + len), where lead is the distance of
// src from the 16-byte boundary below it, so that both sides of every full
// vector are aligned.  Returns lead.
template <class T>
__device__ __forceinline__ uint32_t stage_linear(T* tile, const T* src, uint32_t len) {
  constexpr uint32_t VEC = 16 / sizeof(T);
  const uint32_t lead = (uint32_t)((reinterpret_cast<uintptr_t>(src) / sizeof(T)) % VEC);
  const T* base = src - lead;
  const uint32_t end = lead + len;
  const uint32_t nvec = (end + VEC - 1) / VEC;
  for (uint32_t v = threadIdx.x; v < nvec; v += kBlock) {
    const uint32_t i0 = v * VEC;
    if (i0 >= lead && i0 + VEC <= end) {
      *reinterpret_cast<Bytes16*>(tile + i0) = *reinterpret_cast<const Bytes16*>(base + i0);
    } else {
#pragma unroll
      for (uint32_t e = 0; e < VEC; ++e)
        if (i0 + e >= lead && i0 + e < end) tile[i0 + e] = base[i0 + e];
    }
  }
  return lead;
}

// RN(a / d) for a float a and an integer 1 <= d <= 255 with y = RN(1 / d).
__device__ __forceinline__ double quotient_by_reciprocal(double a, double d, double y) {
  const double q = a * y;
  const double r = fma(-d, q, a);
  const double q2 = fma(r, y, q);
  // zeros (whose sign the correction would lose), infinities and NaN: q is the quotient
  constexpr int kZeroInfNan = 0x001 | 0x002 | 0x004 | 0x020 | 0x040 | 0x200;
  return __builtin_amdgcn_class(a, kZeroInfNan) ? q : q2;
}

template <class T>
__device__ __forceinline__ double tap_quotient(T v, double d, double y, bool fast) {
  if (sizeof(T) == 4 && fast) return quotient_by_reciprocal((double)v, d, y);
  return (double)v / d;
}

template <class T, int OP, int KW, int KH>
__global__ void __launch_bounds__(kBlock) pool_forward_band_kernel(const BandArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  T* tile = reinterpret_cast<T*>(smem);
  double* recips = reinterpret_cast<double*>(smem + (size_t)a.cap * sizeof(T));
  const int32_t kw = KW ? KW : a.kw, kh = KH ? KH : a.kh;
  uint32_t group, band;
  a.bands_fd.divmod(blockIdx.x, group, band);
  const uint32_t p0 = group * a.pb, np = min(a.pb, a.planes - p0);
  const int32_t oy0 = (int32_t)(band * a.br), rows = min((int32_t)a.br, a.out_h - oy0);
  int32_t iy_lo = 0, n_src_rows = a.in_h;
  if (a.pb == 1) {
    iy_lo = max(0, oy0 * a.sy - a.py);
    n_src_rows = max(0, min(a.in_h, (oy0 + rows - 1) * a.sy - a.py + kh) - iy_lo);
  }
  const uint32_t len = a.pb > 1 ? np * a.in_plane : (uint32_t)(n_src_rows * a.in_w);
  const T* src = reinterpret_cast<const T*>(a.in) + (int64_t)p0 * a.in_plane + (int64_t)iy_lo * a.in_w;
  const uint32_t lead = stage_linear(tile, src, len);
  if (OP == CT_POOL_AVG_EXC_PAD && a.fast_div)
    for (int32_t i = threadIdx.x; i <= kw * kh; i += kBlock) recips[i] = 1.0 / (double)i;
  __syncthreads();
  const uint32_t n_dest = np * (uint32_t)(rows * a.out_w);
  T* out = reinterpret_cast<T*>(a.dest) + (int64_t)p0 * a.out_plane + (int64_t)oy0 * a.out_w;
  const double kernel_count = (double)(kw * kh);
  for (uint32_t o = threadIdx.x; o < n_dest; o += kBlock) {
    uint32_t j = 0, rr = o, oyl, ox;
    if (a.pb > 1) a.dest_plane_fd.divmod(o, j, rr);
    a.dest_w_fd.divmod(rr, oyl, ox);
    const int32_t rel_x = (int32_t)ox * a.sx - a.px, rel_y = (oy0 + (int32_t)oyl) * a.sy - a.py;
    const int32_t plane_at = (int32_t)(lead + j * a.in_plane) - iy_lo * a.in_w;
    T acc = (OP == CT_POOL_AVG_EXC_PAD || a.load_prev) ? out[o] : (T)0;
    double divisor = kernel_count, y = a.recip;
    if (OP == CT_POOL_AVG_EXC_PAD) {
      const int32_t inside = taps_inside(rel_x, kw, a.in_w) * taps_inside(rel_y, kh, a.in_h);
      divisor = (double)inside;
      if (a.fast_div) y = recips[inside];
    }
    if constexpr (KW > 0) {
      // Fixed window: no branches.  Every tap is read (from LDS index 0 when it
      // lies outside the input) and takes part by selects.
      bool col_inside[KW], col_reached[KW];
#pragma unroll
      for (int32_t kx = 0; kx < KW; ++kx) {
        col_inside[kx] = (uint32_t)(rel_x + kx) < (uint32_t)a.in_w;
        col_reached[kx] = rel_x + kx < a.in_w + a.px;
      }
#pragma unroll
      for (int32_t ky = 0; ky < KH; ++ky) {
        const int32_t iy = rel_y + ky;
        const bool row_reached = iy < a.in_h + a.py;
        const bool row_inside = (uint32_t)iy < (uint32_t)a.in_h;
        const int32_t row_at = plane_at + iy * a.in_w + rel_x;
#pragma unroll
        for (int32_t kx = 0; kx < KW; ++kx) {
          const bool inside = row_inside && col_inside[kx];
          const bool reached = row_reached && col_reached[kx];
          const T read = tile[inside ? row_at + kx : 0];
          const T v = inside ? read : (T)0;
          const bool first = (ky | kx) == 0;
          T next;
          if (OP == CT_POOL_MAX) next = (first || v > acc) ? v : acc;
          else if (OP == CT_POOL_AVG) next = (T)((double)(first ? (T)0 : acc) + tap_quotient(v, divisor, y, a.fast_div));
          else next = (T)((double)acc + tap_quotient(v, divisor, y, a.fast_div));
          acc = reached ? next : acc;
        }
      }
    } else {
      for (int32_t ky = 0; ky < kh; ++ky) {
        const int32_t iy = rel_y + ky;
        if (iy >= a.in_h + a.py) break;
        const bool row_inside = iy >= 0 && iy < a.in_h;
        for (int32_t kx = 0; kx < kw; ++kx) {
          const int32_t ix = rel_x + kx;
          if (ix >= a.in_w + a.px) break;
          const T v = (row_inside && ix >= 0 && ix < a.in_w) ? tile[plane_at + iy * a.in_w + ix] : (T)0;
          const bool first = (ky | kx) == 0;
          if (OP == CT_POOL_MAX) {
            if (first || v > acc) acc = v;
          } else if (OP == CT_POOL_AVG) {
            acc = (T)((double)(first ? (T)0 : acc) + tap_quotient(v, divisor, y, a.fast_div));
          } else {
            acc = (T)((double)acc + tap_quotient(v, divisor, y, a.fast_div));
          }
        }
      }
    }
    out[o] = acc;
  }
}

// Forward pass over a zero-padded tile.  When no window reaches beyond the padded
// input, every tap is either an input element or padding that reads 0, so the
// tile is laid out with the padding in it and the taps need no tests at all:
// row r of the tile is input row iy_base + r as kPadCells zero cells, the row
// itself, and zero cells up to a pitch that is a multiple of four; rows above
// and below the input are zero, and four more zero cells follow the last row.
// The cells to the right of a row run on into the left padding of the next.
// Tap (k_y, k_x) of output (y, x) of the band is
// tile[(y * stride_y + k_y) * pitch + kPadCells - pad_x + x * stride_x + k_x].
// With rows that are whole 16-byte pieces of an aligned buffer, every piece
// loaded from memory is stored to LDS as one piece; otherwise cell by cell.
constexpr int32_t kPadCells = 4;
// LDS of a padded tile: a little more than the band kernels take, so that a
// 56 x 56 float plane with its padding (13.4 KiB) stays whole.
constexpr uint32_t kPaddedLdsBytes = 16 * 1024;

struct PaddedArgs {
  const void* in;
  void* dest;
  int32_t in_h, in_w, out_h, out_w;
  int32_t px, py, sx, sy;
  uint32_t in_plane, out_plane;
  uint32_t planes, pb, br, bands;
  uint32_t pitch;         // kPadCells + in_w rounded up to a multiple of four
  uint32_t tile_rows;     // whole planes: rows of a plane's tile
  uint32_t cap;
  uint32_t fast_div;
  double recip;
  FastDiv bands_fd, out_w_fd, out_plane_fd, in_w_fd, in_plane_fd;
};

template <class T, int OP, int KW, int KH>
__global__ void __launch_bounds__(kBlock) pool_forward_padded_kernel(const PaddedArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  T* tile = reinterpret_cast<T*>(smem);
  double* recips = reinterpret_cast<double*>(smem + (size_t)a.cap * sizeof(T));
  constexpr uint32_t VEC = 16 / sizeof(T);
  uint32_t group, band;
  a.bands_fd.divmod(blockIdx.x, group, band);
  const uint32_t p0 = group * a.pb, np = min(a.pb, a.planes - p0);
  const int32_t oy0 = (int32_t)(band * a.br), rows = min((int32_t)a.br, a.out_h - oy0);
  const int32_t iy_base = oy0 * a.sy - a.py;
  const uint32_t tile_rows = a.pb > 1 ? a.tile_rows : (uint32_t)((rows - 1) * a.sy + KH);
  // input rows [iy_lo, iy_hi) are staged; with whole planes, all of them
  const int32_t iy_lo = a.pb > 1 ? 0 : max(0, iy_base);
  const int32_t iy_hi = a.pb > 1 ? a.in_h : max(iy_lo, min(a.in_h, iy_base + (int32_t)tile_rows));
  const uint32_t top = (uint32_t)(iy_lo - iy_base);          // zero rows above the first staged one
  const uint32_t n_rows = (uint32_t)(iy_hi - iy_lo);
  const uint32_t plane_cells = tile_rows * a.pitch;
  const uint32_t gap = a.pitch - (uint32_t)a.in_w;            // cells between the end of a row and the next row's data

  // zeros: around every row, the rows outside the input, the cells after the last row
  for (uint32_t jr = threadIdx.x; jr < np * tile_rows; jr += kBlock) {
    T* row = tile + jr * a.pitch;
#pragma unroll
    for (int32_t c = 0; c < kPadCells; ++c) row[c] = (T)0;
    for (uint32_t c = kPadCells + (uint32_t)a.in_w; c < a.pitch; ++c) row[c] = (T)0;
  }
  if (threadIdx.x < kPadCells) tile[np * plane_cells + threadIdx.x] = (T)0;
  const uint32_t zero_rows = tile_rows - n_rows;               // `top` above, the rest below
  for (uint32_t j = 0; j < np; ++j)
    for (uint32_t z = 0; z < zero_rows; ++z) {
      const uint32_t r = z < top ? z : z + n_rows;
      for (uint32_t c = kPadCells + threadIdx.x; c < kPadCells + (uint32_t)a.in_w; c += kBlock)
        tile[j * plane_cells + r * a.pitch + c] = (T)0;
    }

  // the staged rows are one contiguous piece of memory
  const uint32_t len = a.pb > 1 ? np * a.in_plane : n_rows * (uint32_t)a.in_w;
  const T* src = reinterpret_cast<const T*>(a.in) + (int64_t)p0 * a.in_plane + (int64_t)iy_lo * a.in_w;
  const uint32_t lead = (uint32_t)((reinterpret_cast<uintptr_t>(src) / sizeof(T)) % VEC);
  if (lead == 0 && (uint32_t)a.in_w % VEC == 0) {
    for (uint32_t g0 = threadIdx.x * VEC; g0 < len; g0 += kBlock * VEC) {
      const Bytes16 raw = *reinterpret_cast<const Bytes16*>(src + g0);
      uint32_t j = 0, rr = g0, row, col;
      if (a.pb > 1) a.in_plane_fd.divmod(g0, j, rr);
      a.in_w_fd.divmod(rr, row, col);
      *reinterpret_cast<Bytes16*>(tile + j * plane_cells + (row + top) * a.pitch + kPadCells + col) = raw;
    }
  } else {
    const T* base = src - lead;
    const uint32_t end = lead + len;
    for (uint32_t v = threadIdx.x; v * VEC < end; v += kBlock) {
      const uint32_t i0 = v * VEC;
      T piece[VEC];
      if (i0 >= lead && i0 + VEC <= end) {
        const Bytes16 raw = *reinterpret_cast<const Bytes16*>(base + i0);
        __builtin_memcpy(piece, &raw, 16);
      } else {
#pragma unroll
        for (uint32_t e = 0; e < VEC; ++e) piece[e] = (i0 + e >= lead && i0 + e < end) ? base[i0 + e] : (T)0;
      }
      // element g of the piece of memory: plane j, row, column
      const uint32_t g0 = i0 >= lead ? i0 - lead : 0u;
      uint32_t j = 0, rr = g0, row, col;
      if (a.pb > 1) a.in_plane_fd.divmod(g0, j, rr);
      a.in_w_fd.divmod(rr, row, col);
      uint32_t at = j * plane_cells + (row + top) * a.pitch + kPadCells + col;
#pragma unroll
      for (uint32_t e = 0; e < VEC; ++e) {
        const uint32_t i = i0 + e;
        if (i >= lead && i < end) {
          tile[at] = piece[e];
          ++at;
          if (++col == (uint32_t)a.in_w) {
            col = 0;
            at += gap;
            if (a.pb > 1 && ++row == (uint32_t)a.in_h) { row = 0; at += (tile_rows - (uint32_t)a.in_h) * a.pitch; }
          }
        }
      }
    }
  }
  if (OP == CT_POOL_AVG_EXC_PAD && a.fast_div)
    for (int32_t i = threadIdx.x; i <= KW * KH; i += kBlock) recips[i] = 1.0 / (double)i;
  __syncthreads();

  const uint32_t n_dest = np * (uint32_t)(rows * a.out_w);
  T* out = reinterpret_cast<T*>(a.dest) + (int64_t)p0 * a.out_plane + (int64_t)oy0 * a.out_w;
  constexpr double kernel_count = (double)(KW * KH);
  const uint32_t first_tap = (uint32_t)(kPadCells - a.px);
  for (uint32_t o = threadIdx.x; o < n_dest; o += kBlock) {
    uint32_t j = 0, rr = o, oyl, ox;
    if (a.pb > 1) a.out_plane_fd.divmod(o, j, rr);
    a.out_w_fd.divmod(rr, oyl, ox);
    const T* window = tile + j * plane_cells + oyl * (uint32_t)a.sy * a.pitch + first_tap + ox * (uint32_t)a.sx;
    T acc = OP == CT_POOL_AVG_EXC_PAD ? out[o] : (T)0;
    double divisor = kernel_count, y = a.recip;
    if (OP == CT_POOL_AVG_EXC_PAD) {
      const int32_t inside = taps_inside((int32_t)ox * a.sx - a.px, KW, a.in_w) *
                             taps_inside((oy0 + (int32_t)oyl) * a.sy - a.py, KH, a.in_h);
      divisor = (double)inside;
      if (a.fast_div) y = recips[inside];
    }
#pragma unroll
    for (int32_t ky = 0; ky < KH; ++ky) {
#pragma unroll
      for (int32_t kx = 0; kx < KW; ++kx) {
        const T v = window[ky * a.pitch + kx];
        const bool first = (ky | kx) == 0;
        if (OP == CT_POOL_MAX) acc = (first || v > acc) ? v : acc;
        else if (OP == CT_POOL_AVG) acc = (T)((double)(first ? (T)0 : acc) + tap_quotient(v, divisor, y, a.fast_div));
        else acc = (T)((double)acc + tap_quotient(v, divisor, y, a.fast_div));
      }
    }
    out[o] = acc;
  }
}

template <class T, int OP, int KW, int KH>
__global__ void __launch_bounds__(kBlock) pool_backward_band_kernel(const BandArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  T* tile_v = reinterpret_cast<T*>(smem);
  T* tile_g = tile_v + a.cap;
  double* recips = reinterpret_cast<double*>(smem + (size_t)2 * a.cap * sizeof(T));
  const int32_t kw = KW ? KW : a.kw, kh = KH ? KH : a.kh;
  uint32_t group, band;
  a.bands_fd.divmod(blockIdx.x, group, band);
  const uint32_t p0 = group * a.pb, np = min(a.pb, a.planes - p0);
  const int32_t iy0 = (int32_t)(band * a.br), rows = min((int32_t)a.br, a.in_h - iy0);
  int32_t oy_first = 0, n_src_rows = a.out_h;
  if (a.pb == 1) {
    const int32_t t = iy0 + a.py - kh + 1;
    oy_first = t <= 0 ? 0 : min(a.out_h, (int32_t)a.sy_fd.div((uint32_t)(t + a.sy - 1)));
    const int32_t oy_end = min(a.out_h, (int32_t)a.sy_fd.div((uint32_t)(iy0 + rows - 1 + a.py)) + 1);
    n_src_rows = max(0, oy_end - oy_first);
  }
  const uint32_t len = a.pb > 1 ? np * a.out_plane : (uint32_t)(n_src_rows * a.out_w);
  const int64_t src_at = (int64_t)p0 * a.out_plane + (int64_t)oy_first * a.out_w;
  uint32_t lead_v = 0;
  if (OP == CT_POOL_MAX) lead_v = stage_linear(tile_v, reinterpret_cast<const T*>(a.out_values) + src_at, len);
  const uint32_t lead_g = stage_linear(tile_g, reinterpret_cast<const T*>(a.out_grad) + src_at, len);
  if (OP == CT_POOL_AVG_EXC_PAD && a.fast_div)
    for (int32_t i = threadIdx.x; i <= kw * kh; i += kBlock) recips[i] = 1.0 / (double)i;
  __syncthreads();
  const uint32_t n_dest = np * (uint32_t)(rows * a.in_w);
  const int64_t dest_at = (int64_t)p0 * a.in_plane + (int64_t)iy0 * a.in_w;
  T* ig = reinterpret_cast<T*>(a.dest) + dest_at;
  const T* in = reinterpret_cast<const T*>(a.in) + dest_at;
  const double kernel_count = (double)(kw * kh);
  // The input gradient at row iyl of the band, column ix of plane j of the block.
  auto gather = [&](uint32_t j, uint32_t iyl, uint32_t ix, T acc, T v) -> T {
    // Windows o with o * stride - pad <= i < o * stride - pad + k.
    const int32_t ty = iy0 + (int32_t)iyl + a.py, tx = (int32_t)ix + a.px;
    const int32_t oy_hi = min(a.out_h - 1, (int32_t)a.sy_fd.div((uint32_t)ty));
    const int32_t ox_hi = min(a.out_w - 1, (int32_t)a.sx_fd.div((uint32_t)tx));
    const int32_t by = ty - kh + 1, bx = tx - kw + 1;
    const int32_t oy_lo = by <= 0 ? 0 : (int32_t)a.sy_fd.div((uint32_t)(by + a.sy - 1));
    const int32_t ox_lo = bx <= 0 ? 0 : (int32_t)a.sx_fd.div((uint32_t)(bx + a.sx - 1));
    const int32_t plane_at = (int32_t)(j * a.out_plane) - oy_first * a.out_w;
    for (int32_t oy = oy_lo; oy <= oy_hi; ++oy) {
      const int32_t exc_h = taps_inside(oy * a.sy - a.py, kh, a.in_h);
      for (int32_t ox = ox_lo; ox <= ox_hi; ++ox) {
        const int32_t at = plane_at + oy * a.out_w + ox;
        const T g = tile_g[(int32_t)lead_g + at];
        if (OP == CT_POOL_MAX) {
          if (v == tile_v[(int32_t)lead_v + at]) acc = acc + g;
        } else if (OP == CT_POOL_AVG) {
          acc = (T)((double)acc + tap_quotient(g, kernel_count, a.recip, a.fast_div));
        } else {
          const int32_t inside = taps_inside(ox * a.sx - a.px, kw, a.in_w) * exc_h;
          acc = (T)((double)acc + tap_quotient(g, (double)inside, a.fast_div ? recips[inside] : 0.0, a.fast_div));
        }
      }
    }
    return acc;
  };
  // 16-byte pieces of the gradient (and of the input, for max) when the band
  // starts on a 16-byte boundary of both; the remainder one element at a time.
  constexpr uint32_t VEC = 16 / sizeof(T);
  struct alignas(16) Piece { T v[VEC]; };
  const bool pieces = reinterpret_cast<uintptr_t>(ig) % 16 == 0 &&
                      (OP != CT_POOL_MAX || reinterpret_cast<uintptr_t>(in) % 16 == 0);
  const uint32_t n_pieces = pieces ? n_dest / VEC : 0;
  for (uint32_t q = threadIdx.x; q < n_pieces; q += kBlock) {
    const uint32_t o = q * VEC;
    uint32_t j = 0, rr = o, iyl, ix;
    if (a.pb > 1) a.dest_plane_fd.divmod(o, j, rr);
    a.dest_w_fd.divmod(rr, iyl, ix);
    Piece acc = *reinterpret_cast<const Piece*>(ig + o);
    Piece vin;
    if (OP == CT_POOL_MAX) vin = *reinterpret_cast<const Piece*>(in + o);
#pragma unroll
    for (uint32_t e = 0; e < VEC; ++e) {
      acc.v[e] = gather(j, iyl, ix, acc.v[e], OP == CT_POOL_MAX ? vin.v[e] : (T)0);
      if (++ix == (uint32_t)a.in_w) {
        ix = 0;
        if (++iyl == (uint32_t)rows) { iyl = 0; ++j; }
      }
    }
    *reinterpret_cast<Piece*>(ig + o) = acc;
  }
  for (uint32_t o = n_pieces * VEC + threadIdx.x; o < n_dest; o += kBlock) {
    uint32_t j = 0, rr = o, iyl, ix;
    if (a.pb > 1) a.dest_plane_fd.divmod(o, j, rr);
    a.dest_w_fd.divmod(rr, iyl, ix);
    ig[o] = gather(j, iyl, ix, ig[o], OP == CT_POOL_MAX ? in[o] : (T)0);
  }
}

// ------------------------------------------------------------------ 2 x 2 windows that tile the input

// kernel 2 x 2, stride 2, no padding, in_h = 2 * out_h, in_w = 2 * out_w, in_w a
// multiple of 4: every input lies under exactly one window and global output
// row R reads input rows 2 R and 2 R + 1 whatever the plane, so a lane takes two
// neighbouring windows as 16-byte (float) pieces of the two rows.  No LDS, no
// plane arithmetic, every access a full aligned vector.  Blocks take the die-
// grouped order of the flat kernels (forward +4 points of the HBM peak, backward
// +1 to +3 measured); the band kernels, which wait at a barrier between their
// loads and their arithmetic, measured no gain from it and keep the plain order.
struct Tile2Args {
  const void* in;
  const void* out_values;
  const void* out_grad;
  void* dest;
  uint32_t total;  // pairs of windows in this launch
  uint32_t grouped_blocks;
  uint32_t in_w, out_w;
  FastDiv pairs_fd;  // pairs per output row
};

template <class T, int N>
struct alignas(N * sizeof(T) >= 16 ? 16 : N * sizeof(T)) Run { T v[N]; };

template <class T, int OP>
__device__ __forceinline__ T tile2_forward(T prev, T t0, T t1, T t2, T t3) {
  if (OP == CT_POOL_MAX) {
    T acc = t0;
    if (t1 > acc) acc = t1;
    if (t2 > acc) acc = t2;
    if (t3 > acc) acc = t3;
    return acc;
  }
  // a quarter is exact in double, so the multiplication is the division
  T acc = OP == CT_POOL_AVG ? (T)0 : prev;
  acc = (T)((double)acc + (double)t0 * 0.25);
  acc = (T)((double)acc + (double)t1 * 0.25);
  acc = (T)((double)acc + (double)t2 * 0.25);
  acc = (T)((double)acc + (double)t3 * 0.25);
  return acc;
}

template <class T, int OP>
__device__ __forceinline__ T tile2_backward(T grad_in, T x, T pooled, T grad_out) {
  if (OP == CT_POOL_MAX) return x == pooled ? grad_in + grad_out : grad_in;
  return (T)((double)grad_in + (double)grad_out * 0.25);
}

template <class T, int OP>
__global__ void __launch_bounds__(kBlock) pool_tile2_forward_kernel(const Tile2Args a) {
  const uint32_t idx = xcd_grouped_unit(blockIdx.x, a.grouped_blocks) * kBlock + threadIdx.x;
  if (idx >= a.total) return;
  uint32_t row, pair;
  a.pairs_fd.divmod(idx, row, pair);
  const T* top = reinterpret_cast<const T*>(a.in) + (int64_t)row * 2 * a.in_w + pair * 4;
  const Run<T, 4> r0 = *reinterpret_cast<const Run<T, 4>*>(top);
  const Run<T, 4> r1 = *reinterpret_cast<const Run<T, 4>*>(top + a.in_w);
  Run<T, 2>* out = reinterpret_cast<Run<T, 2>*>(reinterpret_cast<T*>(a.dest) + (int64_t)row * a.out_w + pair * 2);
  Run<T, 2> o;
  if (OP == CT_POOL_AVG_EXC_PAD) o = *out;
  o.v[0] = tile2_forward<T, OP>(o.v[0], r0.v[0], r0.v[1], r1.v[0], r1.v[1]);
  o.v[1] = tile2_forward<T, OP>(o.v[1], r0.v[2], r0.v[3], r1.v[2], r1.v[3]);
  *out = o;
}

template <class T, int OP>
__global__ void __launch_bounds__(kBlock) pool_tile2_backward_kernel(const Tile2Args a) {
  const uint32_t idx = xcd_grouped_unit(blockIdx.x, a.grouped_blocks) * kBlock + threadIdx.x;
  if (idx >= a.total) return;
  uint32_t row, pair;
  a.pairs_fd.divmod(idx, row, pair);
  const int64_t in_at = (int64_t)row * 2 * a.in_w + pair * 4, out_at = (int64_t)row * a.out_w + pair * 2;
  Run<T, 4>* g0 = reinterpret_cast<Run<T, 4>*>(reinterpret_cast<T*>(a.dest) + in_at);
  Run<T, 4>* g1 = reinterpret_cast<Run<T, 4>*>(reinterpret_cast<T*>(a.dest) + in_at + a.in_w);
  Run<T, 4> ig0 = *g0, ig1 = *g1, x0{}, x1{};
  Run<T, 2> pooled{};
  if (OP == CT_POOL_MAX) {
    x0 = *reinterpret_cast<const Run<T, 4>*>(reinterpret_cast<const T*>(a.in) + in_at);
    x1 = *reinterpret_cast<const Run<T, 4>*>(reinterpret_cast<const T*>(a.in) + in_at + a.in_w);
    pooled = *reinterpret_cast<const Run<T, 2>*>(reinterpret_cast<const T*>(a.out_values) + out_at);
  }
  const Run<T, 2> og = *reinterpret_cast<const Run<T, 2>*>(reinterpret_cast<const T*>(a.out_grad) + out_at);
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    ig0.v[c] = tile2_backward<T, OP>(ig0.v[c], x0.v[c], pooled.v[c / 2], og.v[c / 2]);
    ig1.v[c] = tile2_backward<T, OP>(ig1.v[c], x1.v[c], pooled.v[c / 2], og.v[c / 2]);
  }
  *g0 = ig0;
  *g1 = ig1;
}

struct PoolShape {
  int64_t planes, in_h, in_w, out_h, out_w;
};

int check_pool(const ct_pool_desc* d, int64_t batch_count, int64_t channel_count, int64_t in_height,
               int64_t in_width, int64_t out_height, int64_t out_width, int dtype, PoolShape* shape) {
  CT_REQUIRE(d != nullptr, "pooling: null descriptor");
  CT_REQUIRE(dtype == CT_F32 || dtype == CT_F64, "Failed to find pooling op for datatype %d", dtype);
  CT_REQUIRE(d->pool_op == CT_POOL_MAX || d->pool_op == CT_POOL_AVG || d->pool_op == CT_POOL_AVG_EXC_PAD,
             "Max pooling layers have three possible pool operations; got %d", d->pool_op);
  CT_REQUIRE(d->kernel_width >= 1 && d->kernel_height >= 1 && d->stride_x >= 1 && d->stride_y >= 1 &&
                 d->pad_x >= 0 && d->pad_y >= 0,
             "pooling: kernel and stride must be positive and padding non-negative");
  CT_REQUIRE(d->kernel_width <= 4096 && d->kernel_height <= 4096 && d->stride_x <= 4096 && d->stride_y <= 4096 &&
                 d->pad_x <= 4096 && d->pad_y <= 4096,
             "pooling: kernel, stride and padding above 4096 are not supported");
  CT_REQUIRE(batch_count >= 0 && channel_count >= 0 && in_height >= 0 && in_width >= 0 && out_height >= 0 &&
                 out_width >= 0,
             "pooling: negative count");
  const int64_t plane_limit = (int64_t(1) << 31) - 1;
  CT_REQUIRE(in_height <= 1 << 20 && in_width <= 1 << 20 && out_height <= 1 << 20 && out_width <= 1 << 20 &&
                 in_height * in_width <= plane_limit && out_height * out_width <= plane_limit,
             "pooling: an image plane exceeds the supported range");
  CT_REQUIRE(out_height * d->stride_y + d->kernel_height + d->pad_y <= plane_limit &&
                 out_width * d->stride_x + d->kernel_width + d->pad_x <= plane_limit,
             "pooling: window positions exceed the supported range");
  CT_REQUIRE(batch_count <= plane_limit && channel_count <= plane_limit &&
                 (channel_count == 0 || batch_count <= (int64_t(1) << 40) / channel_count),
             "pooling: batch_count * channel_count exceeds the supported range");
  *shape = PoolShape{batch_count * channel_count, in_height, in_width, out_height, out_width};
  return CT_OK;
}

// LDS given to the staged rows of a block.  The kernels are bound by latency and
// instruction issue, so the waves a compute unit holds matter more than the
// length of a band: measured on [64, 64, 224, 224] float, 3 x 3 stride 2, the
// forward max pass reads and writes at 53 / 57 / 52 / 41 / 34 % of the HBM peak
// with 8 / 12 / 20 / 32 / 48 KiB.
constexpr uint32_t kBandLdsBytes = 12 * 1024;
// Destination elements a block of whole small planes aims for.
constexpr uint32_t kBandDestTarget = 16 * kBlock;

struct BandPlan {
  bool usable;
  uint32_t pb, br, bands;
};

// Forward: `rows` destination rows read (rows - 1) * stride + k source rows.
// Backward: `rows` destination (input) rows are covered by at most
// (rows + k - 2) / stride + 2 source (output) rows.
BandPlan plan_bands(bool forward, uint32_t budget, int64_t src_plane, int64_t src_w, int64_t dest_plane,
                    int64_t dest_h, int64_t k, int64_t stride) {
  BandPlan p{false, 1, 1, 1};
  if (src_plane <= budget) {
    p.usable = true;
    const int64_t by_lds = budget / std::max<int64_t>(1, src_plane);
    const int64_t by_dest = std::max<int64_t>(1, kBandDestTarget / std::max<int64_t>(1, dest_plane));
    p.pb = (uint32_t)std::max<int64_t>(1, std::min(by_lds, by_dest));
    p.br = (uint32_t)dest_h;
    p.bands = 1;
    return p;
  }
  const int64_t src_rows = budget / std::max<int64_t>(1, src_w);
  int64_t rows;
  if (forward) rows = src_rows >= k ? (src_rows - k) / stride + 1 : 0;
  else rows = (src_rows - 2) * stride - k + 2;
  if (rows < 1) return p;
  rows = std::min(rows, dest_h);
  p.usable = true;
  p.bands = (uint32_t)((dest_h + rows - 1) / rows);
  p.br = (uint32_t)((dest_h + p.bands - 1) / p.bands);
  return p;
}

template <class T, int OP, int KW, int KH>
void launch_band(hipStream_t s, bool forward, dim3 grid, size_t lds, const BandArgs& a) {
  if (forward) hipLaunchKernelGGL((pool_forward_band_kernel<T, OP, KW, KH>), grid, dim3(kBlock), lds, s, a);
  else hipLaunchKernelGGL((pool_backward_band_kernel<T, OP, KW, KH>), grid, dim3(kBlock), lds, s, a);
}

template <class T, int OP>
void launch_band_window(hipStream_t s, bool forward, dim3 grid, size_t lds, const BandArgs& a) {
  if (a.kw == 2 && a.kh == 2) launch_band<T, OP, 2, 2>(s, forward, grid, lds, a);
  else if (a.kw == 3 && a.kh == 3) launch_band<T, OP, 3, 3>(s, forward, grid, lds, a);
  else launch_band<T, OP, 0, 0>(s, forward, grid, lds, a);
}

template <class T>
int pool_launch(hipStream_t s, bool forward, void* dest, const void* in, const void* out_values, const void* out_grad,
                const ct_pool_desc& d, const PoolShape& sh) {
  const int64_t in_plane = sh.in_h * sh.in_w, out_plane = sh.out_h * sh.out_w;
  const int64_t dest_plane = forward ? out_plane : in_plane;
  if (sh.planes == 0 || dest_plane == 0) return CT_OK;
  // The first tap lies inside the padded input unless the stride carries the
  // last window past it; then max and avg continue from what the output holds.
  const bool first_tap_inside = (sh.out_w - 1) * d.stride_x - d.pad_x < sh.in_w + d.pad_x &&
                                (sh.out_h - 1) * d.stride_y - d.pad_y < sh.in_h + d.pad_y;
  const int64_t limit = (int64_t(1) << 31) - 1;
  const int64_t planes_per_launch = std::max<int64_t>(1, limit / std::max<int64_t>(1, std::max(in_plane, out_plane)));

  auto aligned16 = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const bool tiles2 = d.kernel_width == 2 && d.kernel_height == 2 && d.stride_x == 2 && d.stride_y == 2 &&
                      d.pad_x == 0 && d.pad_y == 0 && sh.in_w == 2 * sh.out_w && sh.in_h == 2 * sh.out_h &&
                      sh.in_w % 4 == 0 && aligned16(dest) && aligned16(in) && aligned16(out_values) &&
                      aligned16(out_grad);
  if (tiles2) {
    Tile2Args a{};
    a.in_w = (uint32_t)sh.in_w; a.out_w = (uint32_t)sh.out_w;
    const int64_t pairs = sh.out_w / 2;
    a.pairs_fd = FastDiv((uint32_t)pairs);
    note_kernel(forward ? "pool_forward_tile2" : "pool_backward_tile2");
    for (int64_t p0 = 0; p0 < sh.planes; p0 += planes_per_launch) {
      const int64_t np = std::min(planes_per_launch, sh.planes - p0);
      a.total = (uint32_t)(np * sh.out_h * pairs);
      a.in = reinterpret_cast<const T*>(in) + p0 * in_plane;
      a.out_values = out_values ? reinterpret_cast<const T*>(out_values) + p0 * out_plane : nullptr;
      a.out_grad = out_grad ? reinterpret_cast<const T*>(out_grad) + p0 * out_plane : nullptr;
      a.dest = reinterpret_cast<T*>(dest) + p0 * dest_plane;
      const dim3 grid((a.total + kBlock - 1) / kBlock);
      a.grouped_blocks = xcd_grouped_blocks(grid.x);
#define CT_POOL(KERNEL)                                                                                       \
  switch (d.pool_op) {                                                                                        \
    case CT_POOL_MAX: hipLaunchKernelGGL((KERNEL<T, CT_POOL_MAX>), grid, dim3(kBlock), 0, s, a); break;       \
    case CT_POOL_AVG: hipLaunchKernelGGL((KERNEL<T, CT_POOL_AVG>), grid, dim3(kBlock), 0, s, a); break;       \
    default: hipLaunchKernelGGL((KERNEL<T, CT_POOL_AVG_EXC_PAD>), grid, dim3(kBlock), 0, s, a); break;        \
  }
      if (forward) { CT_POOL(pool_tile2_forward_kernel) } else { CT_POOL(pool_tile2_backward_kernel) }
#undef CT_POOL
    }
    return after_launch(s);
  }

  // Forward pass of a 2 x 2 or 3 x 3 window that never reaches beyond the padded input: zero-padded tile.
  const bool fixed_window = (d.kernel_width == 2 && d.kernel_height == 2) || (d.kernel_width == 3 && d.kernel_height == 3);
  const int64_t reach_x = (sh.out_w - 1) * d.stride_x - d.pad_x + d.kernel_width;
  const int64_t reach_y = (sh.out_h - 1) * d.stride_y - d.pad_y + d.kernel_height;
  if (forward && fixed_window && in_plane > 0 && d.pad_x <= kPadCells && reach_x <= sh.in_w + d.pad_x &&
      reach_y <= sh.in_h + d.pad_y) {
    const int64_t budget = kPaddedLdsBytes / (int64_t)sizeof(T);
    const int64_t pitch = (kPadCells + sh.in_w + 3) / 4 * 4;
    const int64_t plane_rows = d.pad_y + std::max<int64_t>(sh.in_h, reach_y);
    const int64_t plane_cells = plane_rows * pitch;
    PaddedArgs a{};
    bool usable = true;
    if (plane_cells + kPadCells <= budget) {
      const int64_t by_lds = (budget - kPadCells) / plane_cells;
      const int64_t by_dest = std::max<int64_t>(1, kBandDestTarget / out_plane);
      a.pb = (uint32_t)std::max<int64_t>(1, std::min(by_lds, by_dest));
      a.br = (uint32_t)sh.out_h;
      a.bands = 1;
    } else {
      const int64_t tile_rows = (budget - kPadCells) / pitch;
      int64_t rows = tile_rows >= d.kernel_height ? (tile_rows - d.kernel_height) / d.stride_y + 1 : 0;
      usable = rows >= 1;
      rows = std::min<int64_t>(std::max<int64_t>(rows, 1), sh.out_h);
      a.pb = 1;
      a.bands = (uint32_t)((sh.out_h + rows - 1) / rows);
      a.br = (uint32_t)((sh.out_h + a.bands - 1) / a.bands);
    }
    if (usable) {
      a.in_h = (int32_t)sh.in_h; a.in_w = (int32_t)sh.in_w; a.out_h = (int32_t)sh.out_h; a.out_w = (int32_t)sh.out_w;
      a.px = d.pad_x; a.py = d.pad_y; a.sx = d.stride_x; a.sy = d.stride_y;
      a.in_plane = (uint32_t)in_plane; a.out_plane = (uint32_t)out_plane;
      a.pitch = (uint32_t)pitch;
      a.tile_rows = (uint32_t)plane_rows;
      a.cap = ((uint32_t)budget + 8u) / 4u * 4u;
      const int64_t window = (int64_t)d.kernel_width * d.kernel_height;
      a.fast_div = sizeof(T) == 4 ? 1u : 0u;
      a.recip = 1.0 / (double)window;
      a.bands_fd = FastDiv(a.bands);
      a.out_w_fd = FastDiv((uint32_t)sh.out_w);
      a.out_plane_fd = FastDiv((uint32_t)out_plane);
      a.in_w_fd = FastDiv((uint32_t)sh.in_w);
      a.in_plane_fd = FastDiv((uint32_t)in_plane);
      const size_t lds = (size_t)a.cap * sizeof(T) + (size_t)kRecipTable * sizeof(double);
      note_kernel("pool_forward_padded");
      for (int64_t p0 = 0; p0 < sh.planes; p0 += planes_per_launch) {
        const int64_t np = std::min(planes_per_launch, sh.planes - p0);
        a.planes = (uint32_t)np;
        a.in = reinterpret_cast<const T*>(in) + p0 * in_plane;
        a.dest = reinterpret_cast<T*>(dest) + p0 * dest_plane;
        const int64_t groups = (np + a.pb - 1) / a.pb;
        const dim3 grid((uint32_t)(groups * a.bands));
#define CT_POOL(KW, KH)                                                                                                  \
  switch (d.pool_op) {                                                                                                   \
    case CT_POOL_MAX:                                                                                                    \
      hipLaunchKernelGGL((pool_forward_padded_kernel<T, CT_POOL_MAX, KW, KH>), grid, dim3(kBlock), lds, s, a); break;    \
    case CT_POOL_AVG:                                                                                                    \
      hipLaunchKernelGGL((pool_forward_padded_kernel<T, CT_POOL_AVG, KW, KH>), grid, dim3(kBlock), lds, s, a); break;    \
    default:                                                                                                             \
      hipLaunchKernelGGL((pool_forward_padded_kernel<T, CT_POOL_AVG_EXC_PAD, KW, KH>), grid, dim3(kBlock), lds, s, a);  \
  }
        if (d.kernel_width == 2) { CT_POOL(2, 2) } else { CT_POOL(3, 3) }
#undef CT_POOL
      }
      return after_launch(s);
    }
  }

  const uint32_t arrays = forward ? 1u : 2u;
  const uint32_t budget = kBandLdsBytes / (uint32_t)sizeof(T) / arrays;
  const BandPlan bp = forward ? plan_bands(true, budget, in_plane, sh.in_w, out_plane, sh.out_h, d.kernel_height,
                                           d.stride_y)
                              : plan_bands(false, budget, out_plane, sh.out_w, in_plane, sh.in_h, d.kernel_height,
                                           d.stride_y);
  if (bp.usable && (forward ? in_plane : out_plane) > 0) {
    BandArgs a{};
    a.in_h = (int32_t)sh.in_h; a.in_w = (int32_t)sh.in_w; a.out_h = (int32_t)sh.out_h; a.out_w = (int32_t)sh.out_w;
    a.kw = d.kernel_width; a.kh = d.kernel_height; a.px = d.pad_x; a.py = d.pad_y; a.sx = d.stride_x;
    a.sy = d.stride_y;
    a.in_plane = (uint32_t)in_plane; a.out_plane = (uint32_t)out_plane;
    a.pb = bp.pb; a.br = bp.br; a.bands = bp.bands;
    a.cap = (budget + 8u) / 4u * 4u;
    a.load_prev = first_tap_inside ? 0u : 1u;
    const int64_t window = (int64_t)d.kernel_width * d.kernel_height;
    a.fast_div = (sizeof(T) == 4 && window < kRecipTable) ? 1u : 0u;
    a.recip = 1.0 / (double)window;
    a.bands_fd = FastDiv(bp.bands);
    a.dest_w_fd = FastDiv((uint32_t)(forward ? sh.out_w : sh.in_w));
    a.dest_plane_fd = FastDiv((uint32_t)dest_plane);
    a.sx_fd = FastDiv((uint32_t)d.stride_x);
    a.sy_fd = FastDiv((uint32_t)d.stride_y);
    const size_t lds = (size_t)arrays * a.cap * sizeof(T) + (size_t)kRecipTable * sizeof(double);
    note_kernel(forward ? "pool_forward_band" : "pool_backward_band");
    for (int64_t p0 = 0; p0 < sh.planes; p0 += planes_per_launch) {
      const int64_t np = std::min(planes_per_launch, sh.planes - p0);
      a.planes = (uint32_t)np;
      a.in = reinterpret_cast<const T*>(in) + p0 * in_plane;
      a.out_values = out_values ? reinterpret_cast<const T*>(out_values) + p0 * out_plane : nullptr;
      a.out_grad = out_grad ? reinterpret_cast<const T*>(out_grad) + p0 * out_plane : nullptr;
      a.dest = reinterpret_cast<T*>(dest) + p0 * dest_plane;
      const int64_t groups = (np + bp.pb - 1) / bp.pb;
      const dim3 grid((uint32_t)(groups * bp.bands));
      switch (d.pool_op) {
        case CT_POOL_MAX: launch_band_window<T, CT_POOL_MAX>(s, forward, grid, lds, a); break;
        case CT_POOL_AVG: launch_band_window<T, CT_POOL_AVG>(s, forward, grid, lds, a); break;
        default: launch_band_window<T, CT_POOL_AVG_EXC_PAD>(s, forward, grid, lds, a); break;
      }
    }
    return after_launch(s);
  }

  PoolArgs a{};
  a.in_h = (int32_t)sh.in_h; a.in_w = (int32_t)sh.in_w; a.out_h = (int32_t)sh.out_h; a.out_w = (int32_t)sh.out_w;
  a.kw = d.kernel_width; a.kh = d.kernel_height; a.px = d.pad_x; a.py = d.pad_y; a.sx = d.stride_x; a.sy = d.stride_y;
  a.in_plane = (uint32_t)in_plane; a.out_plane = (uint32_t)out_plane;
  a.plane_fd = FastDiv((uint32_t)dest_plane);
  a.row_fd = FastDiv((uint32_t)(forward ? sh.out_w : sh.in_w));
  a.sx_fd = FastDiv((uint32_t)d.stride_x);
  a.sy_fd = FastDiv((uint32_t)d.stride_y);
  a.load_prev = first_tap_inside ? 0u : 1u;
  note_kernel(forward ? "pool_forward" : "pool_backward");
  for (int64_t p0 = 0; p0 < sh.planes; p0 += planes_per_launch) {
    const int64_t np = std::min(planes_per_launch, sh.planes - p0);
    a.total = (uint32_t)(np * dest_plane);
    a.in = in ? reinterpret_cast<const T*>(in) + p0 * in_plane : nullptr;
    a.out_values = out_values ? reinterpret_cast<const T*>(out_values) + p0 * out_plane : nullptr;
    a.out_grad = out_grad ? reinterpret_cast<const T*>(out_grad) + p0 * out_plane : nullptr;
    a.dest = reinterpret_cast<T*>(dest) + p0 * dest_plane;
    const dim3 grid((a.total + kBlock - 1) / kBlock);
#define CT_POOL(KERNEL)                                                                                       \
  switch (d.pool_op) {                                                                                        \
    case CT_POOL_MAX: hipLaunchKernelGGL((KERNEL<T, CT_POOL_MAX>), grid, dim3(kBlock), 0, s, a); break;       \
    case CT_POOL_AVG: hipLaunchKernelGGL((KERNEL<T, CT_POOL_AVG>), grid, dim3(kBlock), 0, s, a); break;       \
    default: hipLaunchKernelGGL((KERNEL<T, CT_POOL_AVG_EXC_PAD>), grid, dim3(kBlock), 0, s, a); break;        \
  }
    if (forward) { CT_POOL(pool_forward_kernel) } else { CT_POOL(pool_backward_kernel) }
#undef CT_POOL
  }
  return after_launch(s);
}

}  // namespace

extern "C" {

int ct_pooling_forward(void* stream, void* output, double /*output_alpha*/, const void* input,
                       const ct_pool_desc* desc, int64_t batch_count, int64_t channel_count, int64_t in_height,
                       int64_t in_width, int64_t out_height, int64_t out_width, int dtype) {
  PoolShape sh;
  if (int rc = check_pool(desc, batch_count, channel_count, in_height, in_width, out_height, out_width, dtype, &sh))
    return rc;
  if (sh.planes * sh.out_h * sh.out_w == 0) return CT_OK;
  CT_REQUIRE(output != nullptr && (input != nullptr || sh.in_h * sh.in_w == 0), "pooling-forward!: null buffer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == CT_F32) return pool_launch<float>(s, true, output, input, nullptr, nullptr, *desc, sh);
  return pool_launch<double>(s, true, output, input, nullptr, nullptr, *desc, sh);
}

int ct_pooling_backward(void* stream, void* input_gradient, double /*input_gradient_alpha*/, const void* input,
                        const void* output, const void* output_gradient, const ct_pool_desc* desc,
                        int64_t batch_count, int64_t channel_count, int64_t in_height, int64_t in_width,
                        int64_t out_height, int64_t out_width, int dtype) {
  PoolShape sh;
  if (int rc = check_pool(desc, batch_count, channel_count, in_height, in_width, out_height, out_width, dtype, &sh))
    return rc;
  if (sh.planes * sh.in_h * sh.in_w == 0 || sh.out_h * sh.out_w == 0) return CT_OK;
  CT_REQUIRE(input_gradient != nullptr && input != nullptr && output != nullptr && output_gradient != nullptr,
             "pooling-backward!: null buffer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == CT_F32) return pool_launch<float>(s, false, input_gradient, input, output, output_gradient, *desc, sh);
  return pool_launch<double>(s, false, input_gradient, input, output, output_gradient, *desc, sh);
}

}  // extern "C"
