// ops_batchnorm.hip -- the six batch-normalization methods of the TensorMath
// protocol (src/cortex/tensor/math.clj:124-174) after the CPU backend
// (src/cortex/compute/cpu/tensor_math.clj:731-1033, 1558-1638).
//
// All buffers are packed: values [batch, channels, elements], one statistic per
// channel; the eltwise forms are the spatial forms with one element per channel
// (BNEltwiseOffsetter and BNSpatialOffsetter, :737-753, give the same offsets).
//
// The CPU backend walks each channel several times (five sums in the gradient).
// Here every method is
//   statistics pass   all sums of a channel in one read of the operands, in
//                     double, as per-block partial sums in scratch memory
//   finishing pass    one wave per channel adds the partials in a fixed order
//                     and derives the channel's constants
//   apply pass        one flat, 128-bit vectorised elementwise pass
// so the operands are read twice and the result written once (the plain
// normalization with given statistics is the apply pass alone).  Per-element
// arithmetic follows the CPU backend operation by operation (double, one
// rounding at the store); only the order of the additions inside a sum differs
// (a tree instead of left to right), which moves a double sum by a few units in
// its last place.
//
// Variance: the CPU backend takes the mean first and then sums (mean - x)^2 in
// a second walk.  The statistics pass here accumulates d = x - K and d^2 for a
// pivot K (the channel's first value) and forms
//   sum (m - x)^2 = sum d^2 - 2 (m - K) sum d + n (m - K)^2
// with m the mean already rounded to the tensor type, as the reference uses it.
// With K inside the data's range the cancellation costs a few bits of a double.
#include <algorithm>

#include "elementwise.h"

using namespace cthip;

namespace {

enum { kBnNormalize = 0, kBnGradient = 1 };
constexpr int64_t kRowApplyBytes = int64_t(32) << 20;  // plain normalize: size from which the constants get a launch of their own
constexpr int kRowApplyMinVecs = 8;  // shortest row, in vectors, that the row kernel takes
constexpr int kRaggedApplyMinVecs = 64;  // the same for rows that are no whole number of vectors (measured: 49-element rows lose)
constexpr int kParamStride = 8;  // doubles per channel in the parameter table
// constants of a channel as the apply pass holds them:
//   normalize: mean, inv_std (rounded to T), scale, shift -- derived from the statistics vectors on the fly
//   gradient:  mean, inv_std (double), scale, d_var, 2 * d_var_d_out, d_mean_d_out / n, 1 / n -- the parameter table
constexpr int kUnroll = 4;

template <int MODE> struct bn_nacc { static constexpr int value = MODE == kBnGradient ? 5 : 2; };
template <int MODE> struct bn_nparam { static constexpr int value = MODE == kBnGradient ? 7 : 4; };

struct BnArgs {
  const void* x;    // input
  const void* og;   // output gradient (gradient mode)
  void* out;        // output, or input gradient
  double* params;   // [channels][kParamStride], gradient constants written by the finishing pass
  double* partials;
  const void* means;      // per channel, of the tensor type: the statistics in use
  const void* variances;
  const void* scale;
  const void* bias;
  double epsilon;
  int64_t B, C, E, W;        // W = C * E, the length of one batch row
  int64_t N;                 // B * C * E
  uint32_t S;                // row segments of the statistics pass
  uint32_t rows_per_seg;
  uint32_t nv;               // vectors per (batch, channel) row, row-style statistics
  uint32_t part_E;           // partial sums kept per channel and segment (1 row-style, E column-style)
  FastDiv nv_fd, s_fd, e_fd, c_fd;
  // apply pass
  int64_t first, count;      // element range of this launch
  uint32_t table_slots;      // channels held in the LDS table
  uint32_t table_full;       // the table holds every channel (indexed by channel) instead of a window of rows
  uint32_t apply_rows_per_seg;  // column-style apply: batch rows per block
  uint32_t row_holds_vectors;   // E and the launch's first element are multiples of the vector width
};

struct BnFinish {
  // normalize (update) mode
  void* batch_means; void* batch_variances; void* running_means; void* running_variances;
  double average_factor;
  // gradient mode
  void* scale_gradient; void* bias_gradient;
};

// ---------------------------------------------------------------- per-element sums

// Update: d = x - pivot; sums d and d*d.
template <class T> __device__ __forceinline__ void bn_accumulate_update(double* acc, T x, double pivot) {
  const double d = (double)x - pivot;
  acc[0] += d;
  acc[1] += d * d;
}

// The scaled output gradient as the CPU backend parks it in the input-gradient
// buffer (:956-960): scale * og evaluated in double and rounded to T.  For float
// that is the float product (the double product of two floats is exact).
template <class T> __device__ __forceinline__ double bn_d_x_hat(T scale, T og) {
  return (double)(T)(scale * og);
}

// Gradient: the five sums of batch-normalize-gradients-impl (cpu/tensor_math.clj:928-983)
// with their per-channel factors taken out of the sums:
//   acc0 = sum og                 bias gradient
//   acc1 = sum og * (x - mean)    scale gradient   = inv_std * acc1
//   acc2 = sum d_x_hat * (x-mean) d_var_d_out      = d_var * acc2
//   acc3 = sum d_x_hat            first term of d_mean_d_out = -inv_std * acc3
//   acc4 = sum (x - mean)         second term      = -2 * acc4
template <class T>
__device__ __forceinline__ void bn_accumulate_gradient(double* acc, T x, T g, double mean, T scale) {
  const double og = (double)g;
  const double xm = (double)x - mean;
  const double d_x_hat = bn_d_x_hat<T>(scale, g);
  acc[0] += og;
  acc[1] += og * xm;
  acc[2] += d_x_hat * xm;
  acc[3] += d_x_hat;
  acc[4] += xm;
}

// A vector of N elements that is only element-aligned: rows of a length that is
// not a multiple of the vector width start off the 16-byte grid.  The hardware
// takes multi-dword global loads at any dword address.
template <class T, int N> struct __attribute__((packed, aligned(sizeof(T)))) UVec { T v[N]; };

// Loads VEC elements from p.  ALIGNED: p is VEC-element aligned and all VEC exist.
// Otherwise `valid` elements exist (the row's tail vector is partial).
template <class T, int VEC, bool ALIGNED, bool NT>
__device__ __forceinline__ Vec<T, VEC> bn_load(const T* p, int valid) {
  Vec<T, VEC> r;
  if constexpr (ALIGNED) {
    if constexpr (NT) r = nt_load(reinterpret_cast<const Vec<T, VEC>*>(p));
    else r = *reinterpret_cast<const Vec<T, VEC>*>(p);
  } else {
    if (valid >= VEC) {
      const UVec<T, VEC> u = *reinterpret_cast<const UVec<T, VEC>*>(p);
#pragma unroll
      for (int e = 0; e < VEC; ++e) r.v[e] = u.v[e];
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) r.v[e] = e < valid ? p[e] : (T)0;
    }
  }
  return r;
}

template <int NACC>
__device__ __forceinline__ void bn_block_reduce_store(double* acc, double* dst, double* lds) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int k = 0; k < NACC; ++k) {
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) acc[k] += __shfl_xor(acc[k], s, 64);
  }
  if (lane == 0) {
#pragma unroll
    for (int k = 0; k < NACC; ++k) lds[wave * NACC + k] = acc[k];
  }
  __syncthreads();
  if (threadIdx.x < NACC) {
    double r = lds[threadIdx.x];
#pragma unroll
    for (int w = 1; w < kBlock / 64; ++w) r += lds[w * NACC + threadIdx.x];
    dst[threadIdx.x] = r;
  }
}

// ---------------------------------------------------------------- statistics, row style
// One block per (channel, segment of the batch).  The (batch, channel) rows of
// the segment are walked as one list of vectors, 256 lanes wide, kUnroll loads
// in flight per lane.
template <class T, int VEC, int MODE, bool ALIGNED, bool NT>
__global__ void __launch_bounds__(kBlock) bn_stats_row_kernel(const BnArgs a) {
  using V = Vec<T, VEC>;
  constexpr int NACC = bn_nacc<MODE>::value;
  __shared__ double lds[(kBlock / 64) * NACC];
  uint32_t c, s;
  a.s_fd.divmod(blockIdx.x, c, s);
  const int64_t b0 = (int64_t)s * a.rows_per_seg;
  const int64_t nb = b0 < a.B ? (a.B - b0 < (int64_t)a.rows_per_seg ? a.B - b0 : (int64_t)a.rows_per_seg) : 0;
  const uint32_t items = (uint32_t)nb * a.nv;
  const int64_t base = (b0 * a.C + c) * a.E;
  const T* x = reinterpret_cast<const T*>(a.x) + base;
  const T* og = reinterpret_cast<const T*>(a.og) + base;
  double p0;
  T scale = (T)0;
  if constexpr (MODE == kBnGradient) {
    p0 = (double)reinterpret_cast<const T*>(a.means)[c];
    scale = reinterpret_cast<const T*>(a.scale)[c];
  } else p0 = (double)reinterpret_cast<const T*>(a.x)[(int64_t)c * a.E];  // pivot: the channel's first value
  double acc[NACC];
#pragma unroll
  for (int k = 0; k < NACC; ++k) acc[k] = 0.0;
  for (uint32_t i0 = threadIdx.x; i0 < items; i0 += kBlock * kUnroll) {
    V xv[kUnroll], gv[kUnroll];
    int valid[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const uint32_t i = i0 + u * kBlock;
      valid[u] = 0;
      if (i < items) {
        uint32_t rr, vv;
        a.nv_fd.divmod(i, rr, vv);
        const int64_t off = (int64_t)rr * a.W + (int64_t)vv * VEC;
        const int64_t left = a.E - (int64_t)vv * VEC;  // elements of the row from this vector on
        valid[u] = ALIGNED || left >= VEC ? VEC : (int)left;
        xv[u] = bn_load<T, VEC, ALIGNED, NT>(x + off, valid[u]);
        if constexpr (MODE == kBnGradient) gv[u] = bn_load<T, VEC, ALIGNED, NT>(og + off, valid[u]);
      }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        if (e < valid[u]) {
          if constexpr (MODE == kBnGradient) bn_accumulate_gradient<T>(acc, xv[u].v[e], gv[u].v[e], p0, scale);
          else bn_accumulate_update<T>(acc, xv[u].v[e], p0);
        }
      }
    }
  }
  bn_block_reduce_store<NACC>(acc, a.partials + ((int64_t)s * a.C + c) * NACC, lds);
}

// ---------------------------------------------------------------- statistics, column style
// For few elements per channel (the eltwise form has one): the tensor is the
// matrix [batch, channels * elements]; a lane owns VEC neighbouring columns, the
// four waves of a block take every fourth row of the block's batch segment.
// Partial sums are kept per column.
template <class T, int VEC, int MODE>
__global__ void __launch_bounds__(kBlock) bn_stats_col_kernel(const BnArgs a) {
  using V = Vec<T, VEC>;
  constexpr int NACC = bn_nacc<MODE>::value;
  constexpr int WAVES = kBlock / 64;
  __shared__ double lds[(WAVES - 1) * 64 * VEC * NACC];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t j0 = ((int64_t)blockIdx.x * 64 + lane) * VEC;
  const bool live = j0 < a.W;
  const uint32_t s = blockIdx.y;
  const int64_t b0 = (int64_t)s * a.rows_per_seg;
  const int64_t nb = b0 < a.B ? (a.B - b0 < (int64_t)a.rows_per_seg ? a.B - b0 : (int64_t)a.rows_per_seg) : 0;
  double p0[VEC];
  T scale[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    p0[e] = 0.0;
    scale[e] = (T)0;
    if (live) {
      const uint32_t ch = a.e_fd.div((uint32_t)(j0 + e));
      if constexpr (MODE == kBnGradient) {
        p0[e] = (double)reinterpret_cast<const T*>(a.means)[ch];
        scale[e] = reinterpret_cast<const T*>(a.scale)[ch];
      } else {
        p0[e] = (double)reinterpret_cast<const T*>(a.x)[(int64_t)ch * a.E];
      }
    }
  }
  double acc[VEC][NACC];
#pragma unroll
  for (int e = 0; e < VEC; ++e)
#pragma unroll
    for (int k = 0; k < NACC; ++k) acc[e][k] = 0.0;
  const T* x = reinterpret_cast<const T*>(a.x) + b0 * a.W + j0;
  const T* og = reinterpret_cast<const T*>(a.og) + b0 * a.W + j0;
  if (live) {
    for (int64_t r0 = wave; r0 < nb; r0 += WAVES * kUnroll) {
      V xv[kUnroll], gv[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const int64_t r = r0 + u * WAVES;
        if (r < nb) {
          xv[u] = *reinterpret_cast<const V*>(x + r * a.W);
          if constexpr (MODE == kBnGradient) gv[u] = *reinterpret_cast<const V*>(og + r * a.W);
        }
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        if (r0 + u * WAVES < nb) {
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            if constexpr (MODE == kBnGradient)
              bn_accumulate_gradient<T>(acc[e], xv[u].v[e], gv[u].v[e], p0[e], scale[e]);
            else bn_accumulate_update<T>(acc[e], xv[u].v[e], p0[e]);
          }
        }
      }
    }
  }
  if (wave > 0) {
    double* mine = lds + ((wave - 1) * 64 + lane) * (VEC * NACC);
#pragma unroll
    for (int e = 0; e < VEC; ++e)
#pragma unroll
      for (int k = 0; k < NACC; ++k) mine[e * NACC + k] = acc[e][k];
  }
  __syncthreads();
  if (wave == 0 && live) {
#pragma unroll
    for (int w = 0; w < WAVES - 1; ++w) {
      const double* theirs = lds + (w * 64 + lane) * (VEC * NACC);
#pragma unroll
      for (int e = 0; e < VEC; ++e)
#pragma unroll
        for (int k = 0; k < NACC; ++k) acc[e][k] += theirs[e * NACC + k];
    }
    double* dst = a.partials + ((int64_t)s * a.W + j0) * NACC;
#pragma unroll
    for (int e = 0; e < VEC; ++e)
#pragma unroll
      for (int k = 0; k < NACC; ++k) dst[e * NACC + k] = acc[e][k];
  }
}

// ---------------------------------------------------------------- per-channel constants

// The constants of channel ch for the apply pass, NP doubles.  Normalize mode
// derives them from the statistics vectors (batch-normalize-impl, :766-777: the
// inverse standard deviation is rounded to T); gradient mode reads the table the
// finishing pass wrote.
// The load and the arithmetic are separate so that a caller can put other loads
// between them.
template <class T, int MODE>
__device__ __forceinline__ double bn_channel_constant_load(const BnArgs& a, uint32_t ch, int k) {
  if constexpr (MODE == kBnGradient) {
    return a.params[(int64_t)ch * kParamStride + k];
  } else {
    const void* src = k == 0 ? a.means : k == 1 ? a.variances : k == 2 ? a.scale : a.bias;
    return (double)reinterpret_cast<const T*>(src)[ch];
  }
}

template <class T, int MODE>
__device__ __forceinline__ double bn_channel_constant_finish(const BnArgs& a, double raw, int k) {
  if constexpr (MODE != kBnGradient) {
    if (k == 1) {
      const T eps = (T)a.epsilon;
      return (double)(T)sqrt(1.0 / (raw + (double)eps));
    }
  }
  return raw;
}

template <class T, int MODE>
__device__ __forceinline__ double bn_channel_constant(const BnArgs& a, uint32_t ch, int k) {
  return bn_channel_constant_finish<T, MODE>(a, bn_channel_constant_load<T, MODE>(a, ch, k), k);
}

// One wave per channel adds the channel's partial sums (segments, and columns in
// the column style) in a fixed order, then lane 0 finishes the channel.
template <class T, int MODE>
__global__ void __launch_bounds__(kBlock) bn_finish_kernel(const BnArgs a, const BnFinish f) {
  constexpr int NACC = bn_nacc<MODE>::value;
  const int lane = threadIdx.x & 63;
  const int64_t c = (int64_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  if (c >= a.C) return;
  double acc[NACC];
#pragma unroll
  for (int k = 0; k < NACC; ++k) acc[k] = 0.0;
  const uint32_t pe = a.part_E;
  const uint32_t n_part = a.S * pe;
  const int64_t seg_stride = a.C * (int64_t)pe;
  for (uint32_t i = lane; i < n_part; i += 64) {
    const uint32_t s = i / pe, e = i - s * pe;
    const double* p = a.partials + ((int64_t)s * seg_stride + c * pe + e) * NACC;
#pragma unroll
    for (int k = 0; k < NACC; ++k) acc[k] += p[k];
  }
#pragma unroll
  for (int k = 0; k < NACC; ++k) {
#pragma unroll
    for (int s = 32; s >= 1; s >>= 1) acc[k] += __shfl_xor(acc[k], s, 64);
  }
  if (lane != 0) return;
  double* pm = a.params + c * kParamStride;
  const int64_t count = a.B * a.E;
  if constexpr (MODE == kBnGradient) {
    // :922-983, with the factors put back
    const T eps = (T)a.epsilon;
    const T pow_factor = (T)(-3.0 / 2.0);
    const double variance = (double)eps + (double)reinterpret_cast<const T*>(a.variances)[c];
    const double inv_std = 1.0 / sqrt(variance);
    const double d_var = (double)(T)(-0.5 * pow(variance, (double)pow_factor));
    pm[0] = (double)reinterpret_cast<const T*>(a.means)[c];
    pm[1] = inv_std;
    pm[2] = (double)reinterpret_cast<const T*>(a.scale)[c];
    pm[3] = d_var;
    reinterpret_cast<T*>(f.bias_gradient)[c] = (T)acc[0];
    reinterpret_cast<T*>(f.scale_gradient)[c] = (T)(inv_std * acc[1]);
    const T d_var_d_out = (T)(d_var * acc[2]);
    const T d_mean_d_out = (T)((-inv_std) * acc[3] + (double)d_var_d_out * ((-2.0 * acc[4]) / (double)count));
    const double one_over_count = 1.0 / (double)count;
    pm[4] = (double)d_var_d_out * 2.0;
    pm[5] = (double)d_mean_d_out * one_over_count;
    pm[6] = one_over_count;
  } else {
    // batch-normalize-update-impl, :831-870
    const T ave_factor = (T)f.average_factor;
    const double ave_lerp = (double)(T)1.0 - (double)ave_factor;
    const double count_val = fmax(1.0, (double)count);
    const double running_count_val = fmax(1.0, count_val - 1.0);
    const double pivot = (double)reinterpret_cast<const T*>(a.x)[c * a.E];
    const T new_mean = (T)(pivot + acc[0] / count_val);
    const double delta = (double)new_mean - pivot;
    double new_var = (acc[1] - 2.0 * delta * acc[0]) + (double)count * delta * delta;
    new_var = new_var < 0.0 ? 0.0 : new_var;
    T* running_means = reinterpret_cast<T*>(f.running_means);
    T* running_variances = reinterpret_cast<T*>(f.running_variances);
    const T mean = running_means[c], variance = running_variances[c];
    const T batch_variance = (T)(new_var / count_val);
    reinterpret_cast<T*>(f.batch_means)[c] = new_mean;
    reinterpret_cast<T*>(f.batch_variances)[c] = batch_variance;
    // the apply pass's constants, as bn_channel_constant derives them from the stored statistics
    pm[0] = (double)new_mean;
    pm[1] = bn_channel_constant_finish<T, kBnNormalize>(a, (double)batch_variance, 1);
    pm[2] = (double)reinterpret_cast<const T*>(a.scale)[c];
    pm[3] = (double)reinterpret_cast<const T*>(a.bias)[c];
    running_means[c] = (T)((double)mean * ave_lerp + (double)new_mean * (double)ave_factor);
    running_variances[c] =
        (T)((double)variance * ave_lerp + (double)(T)(new_var / running_count_val) * (double)ave_factor);
  }
}

// ---------------------------------------------------------------- apply pass

// One output element from its channel's constants p (layout: see kParamStride).
template <class T, int MODE>
__device__ __forceinline__ T bn_apply_one(const double* p, T x, T g) {
  const double xm = (double)x - p[0];
  if constexpr (MODE == kBnGradient) {
    // cpu/tensor_math.clj:986-1001
    const double d_x_hat = bn_d_x_hat<T>((T)p[2], g);
    const double part1 = d_x_hat * p[1];
    const double part2 = (p[4] * xm) * p[6];
    return (T)((part1 + part2) + p[5]);
  } else {
    // cpu/tensor_math.clj:778-784
    return (T)((xm * p[1]) * p[2] + p[3]);
  }
}

// Column style, for few elements per channel: a lane keeps the constants of its
// VEC neighbouring columns of [batch, channels * elements] in registers and walks
// the rows of the block's batch segment.
template <class T, int VEC, int MODE>
__global__ void __launch_bounds__(kBlock) bn_apply_col_kernel(const BnArgs a) {
  using V = Vec<T, VEC>;
  constexpr int NP = bn_nparam<MODE>::value;
  const int64_t j0 = ((int64_t)blockIdx.x * kBlock + threadIdx.x) * VEC;
  if (j0 >= a.W) return;
  double p[VEC][NP];
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    const uint32_t ch = a.e_fd.div((uint32_t)(j0 + e));
#pragma unroll
    for (int k = 0; k < NP; ++k) p[e][k] = bn_channel_constant<T, MODE>(a, ch, k);
  }
  const int64_t b0 = (int64_t)blockIdx.y * a.apply_rows_per_seg;
  const int64_t nb = a.B - b0 < (int64_t)a.apply_rows_per_seg ? a.B - b0 : (int64_t)a.apply_rows_per_seg;
  const T* x = reinterpret_cast<const T*>(a.x) + b0 * a.W + j0;
  const T* og = reinterpret_cast<const T*>(a.og) + b0 * a.W + j0;
  T* out = reinterpret_cast<T*>(a.out) + b0 * a.W + j0;
  for (int64_t r0 = 0; r0 < nb; r0 += kUnroll) {
    V xv[kUnroll], gv[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      if (r0 + u < nb) {
        xv[u] = nt_load(reinterpret_cast<const V*>(x + (r0 + u) * a.W));
        if constexpr (MODE == kBnGradient) gv[u] = nt_load(reinterpret_cast<const V*>(og + (r0 + u) * a.W));
      }
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      if (r0 + u < nb) {
        V r;
#pragma unroll
        for (int e = 0; e < VEC; ++e) r.v[e] = bn_apply_one<T, MODE>(p[e], xv[u].v[e], MODE == kBnGradient ? gv[u].v[e] : (T)0);
        *reinterpret_cast<V*>(out + (r0 + u) * a.W) = r;
      }
    }
  }
}

// Flat over [first, first + count).  The constants of the channels a block can
// meet sit in an LDS table: either every channel, or the window of
// (batch, channel) rows the block's element range touches.
template <class T, int VEC, int MODE, int UNROLL>
__global__ void __launch_bounds__(kBlock) bn_apply_kernel(const BnArgs a) {
  using V = Vec<T, VEC>;
  constexpr int NP = bn_nparam<MODE>::value;
  extern __shared__ __align__(16) double table[];
  constexpr int64_t kSpan = (int64_t)kBlock * VEC * UNROLL;
  const int64_t blk_first = a.first + (int64_t)blockIdx.x * kSpan;
  const int64_t row_first = blk_first / a.E;                       // block-uniform
  const uint32_t ch_first = (uint32_t)(row_first % a.C);           // channel of that (batch, channel) row
  const uint32_t ch_base = a.table_full ? 0u : ch_first;           // channel held in table slot 0
  const int64_t end = a.first + a.count;
  const uint32_t rel0 = (uint32_t)(blk_first - row_first * a.E);  // < E
  const T* x = reinterpret_cast<const T*>(a.x);
  const T* og = reinterpret_cast<const T*>(a.og);
  T* out = reinterpret_cast<T*>(a.out);
  // Loads return in issue order: the first table entry's load goes out ahead of
  // the operands', so the table is complete while the operands are still in flight.
  const uint32_t n_table = a.table_slots * NP;
  const uint32_t slot_t = threadIdx.x / NP, k_t = threadIdx.x - slot_t * NP;
  double raw = 0.0;
  if (threadIdx.x < n_table) {
    uint32_t q, ch;
    a.c_fd.divmod(ch_base + slot_t, q, ch);
    raw = bn_channel_constant_load<T, MODE>(a, ch, (int)k_t);
  }
  V xv[UNROLL], gv[UNROLL];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const int64_t j = blk_first + ((int64_t)u * kBlock + threadIdx.x) * VEC;
    if (j < end) {
      xv[u] = nt_load(reinterpret_cast<const V*>(x + j));
      if constexpr (MODE == kBnGradient) gv[u] = nt_load(reinterpret_cast<const V*>(og + j));
    }
  }
  if (threadIdx.x < n_table) table[threadIdx.x] = bn_channel_constant_finish<T, MODE>(a, raw, (int)k_t);
  for (uint32_t i = threadIdx.x + kBlock; i < n_table; i += kBlock) {
    const uint32_t slot = i / NP, k = i - slot * NP;
    uint32_t q, ch;
    a.c_fd.divmod(ch_base + slot, q, ch);
    table[i] = bn_channel_constant<T, MODE>(a, ch, (int)k);
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const uint32_t jr = (u * kBlock + threadIdx.x) * VEC;
    const int64_t j = blk_first + jr;
    if (j < end) {
      V r;
      if (VEC > 1 && a.row_holds_vectors) {
        // a vector lies inside one (batch, channel) row: one table read serves its elements
        uint32_t slot = a.e_fd.div(rel0 + jr);
        if (a.table_full) {
          uint32_t q;
          a.c_fd.divmod(ch_first + slot, q, slot);
        }
        double p[NP];
#pragma unroll
        for (int k = 0; k < NP; ++k) p[k] = table[slot * NP + k];
#pragma unroll
        for (int e = 0; e < VEC; ++e) r.v[e] = bn_apply_one<T, MODE>(p, xv[u].v[e], MODE == kBnGradient ? gv[u].v[e] : (T)0);
      } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          uint32_t slot = a.e_fd.div(rel0 + jr + e);  // (batch, channel) rows past row_first
          if (a.table_full) {
            uint32_t q;
            a.c_fd.divmod(ch_first + slot, q, slot);
          }
          r.v[e] = bn_apply_one<T, MODE>(table + slot * NP, xv[u].v[e], MODE == kBnGradient ? gv[u].v[e] : (T)0);
        }
      }
      *reinterpret_cast<V*>(out + j) = r;
    }
  }
}

// The normalize constants of every channel into the parameter table, for the
// row kernel below when no finishing pass has written them.
template <class T>
__global__ void __launch_bounds__(kBlock) bn_constants_kernel(const BnArgs a) {
  const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
  const uint32_t ch = i >> 2, k = i & 3;
  if (ch >= a.C) return;
  a.params[(int64_t)ch * kParamStride + k] = bn_channel_constant<T, kBnNormalize>(a, ch, (int)k);
}

// One vector per lane, constants from the parameter table: no LDS table, no
// barrier, and waves as short as those of the plain elementwise kernels.  With
// rows of at least a block's width the block's 256 vectors lie in at most two
// (batch, channel) rows, so the constants are read with wave-uniform addresses
// and a lane only picks its row's set.
struct BnRowArgs {
  uint64_t total_vecs;
  uint32_t grouped_blocks;  // see xcd_grouped_unit
  FastDiv nv_fd, c_fd;   // vectors per row; channels
  const double* params;
  const void* x;
  const void* og;
  void* out;
};

template <class T, int VEC, int MODE, int STREAM, bool RAGGED = false>
__global__ void __launch_bounds__(kBlock) bn_apply_rows_kernel(const BnRowArgs a) {
  using V = Vec<T, VEC>;
  constexpr int NP = bn_nparam<MODE>::value;
  const uint64_t total = a.total_vecs;
  const FastDiv nfd = a.nv_fd, cfd = a.c_fd;
  const double* const params = a.params;
  const uint32_t grouped = a.grouped_blocks;
  const V* const x = reinterpret_cast<const V*>(a.x);
  const V* const og = reinterpret_cast<const V*>(MODE == kBnGradient ? a.og : a.x);
  V* const out = reinterpret_cast<V*>(a.out);
  asm volatile("" ::"s"(total), "s"(nfd.d), "s"(nfd.m), "s"(nfd.s), "s"(cfd.d), "s"(cfd.m), "s"(cfd.s), "s"(params),
               "s"(grouped), "s"(x), "s"(og), "s"(out));
  const uint64_t v_first = (uint64_t)xcd_grouped_unit(blockIdx.x, grouped) * (uint64_t)kBlock;
  const uint64_t v = v_first + threadIdx.x;
  if (v >= total) return;
  V xv, gv;
  if constexpr (STREAM >= 1) xv = nt_load(x + v); else xv = x[v];
  if constexpr (MODE == kBnGradient) {
    if constexpr (STREAM >= 1) gv = nt_load(og + v); else gv = og[v];
  }
  double p[NP];
  if constexpr (RAGGED) {
    // Rows of E >= VEC elements that are no whole number of vectors (nv_fd divides
    // by E here): a vector can end in the next row, whose constants the lane then
    // fetches as well.
    uint32_t row, rem, q, ch;
    nfd.divmod((uint32_t)v * VEC, row, rem);
    cfd.divmod(row, q, ch);
    const double* pl = params + (uint64_t)ch * kParamStride;
#pragma unroll
    for (int k = 0; k < NP; ++k) p[k] = pl[k];
    const uint32_t in_row = nfd.d - rem;  // elements of the vector that lie in `row`
    V r;
    if (in_row < (uint32_t)VEC) {
      const uint32_t ch_b = ch + 1 == cfd.d ? 0u : ch + 1;
      const double* pb = params + (uint64_t)ch_b * kParamStride;
      double p2[NP];
#pragma unroll
      for (int k = 0; k < NP; ++k) p2[k] = pb[k];
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        double pe[NP];
#pragma unroll
        for (int k = 0; k < NP; ++k) pe[k] = (uint32_t)e >= in_row ? p2[k] : p[k];
        r.v[e] = bn_apply_one<T, MODE>(pe, xv.v[e], MODE == kBnGradient ? gv.v[e] : (T)0);
      }
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) r.v[e] = bn_apply_one<T, MODE>(p, xv.v[e], MODE == kBnGradient ? gv.v[e] : (T)0);
    }
    if constexpr (STREAM == 2) nt_store(r, out + v);
    else out[v] = r;
    return;
  }
  if (nfd.d >= (uint32_t)kBlock) {
    uint32_t row_a, cv_a, q, ch_a;
    nfd.divmod((uint32_t)v_first, row_a, cv_a);
    cfd.divmod(row_a, q, ch_a);
    const double* pa = params + (uint64_t)ch_a * kParamStride;
#pragma unroll
    for (int k = 0; k < NP; ++k) p[k] = pa[k];
    if (cv_a + (uint32_t)kBlock > nfd.d) {  // the block runs into the next row
      const uint32_t ch_b = ch_a + 1 == cfd.d ? 0u : ch_a + 1;
      const double* pb = params + (uint64_t)ch_b * kParamStride;
      const bool next = cv_a + threadIdx.x >= nfd.d;
#pragma unroll
      for (int k = 0; k < NP; ++k) {
        const double other = pb[k];
        p[k] = next ? other : p[k];
      }
    }
  } else {
    // shorter rows: a lane finds its own row; its neighbours mostly read the same table entry
    uint32_t q, ch;
    cfd.divmod(nfd.div((uint32_t)v), q, ch);
    const double* pl = params + (uint64_t)ch * kParamStride;
#pragma unroll
    for (int k = 0; k < NP; ++k) p[k] = pl[k];
  }
  V r;
#pragma unroll
  for (int e = 0; e < VEC; ++e) r.v[e] = bn_apply_one<T, MODE>(p, xv.v[e], MODE == kBnGradient ? gv.v[e] : (T)0);
  if constexpr (STREAM == 2) nt_store(r, out + v);
  else out[v] = r;
}

// ---------------------------------------------------------------- host side

struct BnPlan {
  BnArgs a;
  bool col_style;   // few elements per channel: lanes own columns of [batch, channels * elements]
  bool vec_stats;
  bool nt_stats;    // the operands exceed the caches: the statistics pass reads them with non-temporal loads
  bool params_ready = false;  // the parameter table holds the apply pass's constants
  dim3 stats_grid;
  size_t scratch_bytes;
};

constexpr int64_t kRowStyleMinBytes = 128;           // (batch, channel) rows at least this long are walked row style
constexpr size_t kMaxPartialBytes = size_t(32) << 20;
// From this many bytes of operands on, loads are non-temporal: half the 256 MiB last-level cache.
// The update of a [64, C, 3136] float tensor: 103 MB runs 53 -> 50 us with plain loads, 206 MB
// 99 -> 116 us.
constexpr size_t kStreamingBytes = size_t(128) << 20;

template <class T, int MODE>
int bn_plan(hipStream_t s, int64_t B, int64_t C, int64_t E, const void* x, const void* og, void* out, bool need_stats,
            BnPlan* plan) {
  constexpr int NACC = bn_nacc<MODE>::value;
  constexpr int VMAX = 16 / (int)sizeof(T);
  CT_REQUIRE(B >= 1 && C >= 1 && E >= 1, "batch-normalize: batch, channel and element counts must be positive");
  CT_REQUIRE(B < (int64_t(1) << 31) && C < (int64_t(1) << 30) && E < (int64_t(1) << 30),
             "batch-normalize: a count exceeds the supported range");
  CT_REQUIRE((double)B * (double)C * (double)E < 5.0e11, "batch-normalize: tensor too large");
  BnArgs& a = plan->a;
  std::memset(&a, 0, sizeof(a));
  a.x = x; a.og = og; a.out = out;
  a.B = B; a.C = C; a.E = E; a.W = C * E; a.N = B * C * E;
  a.e_fd = FastDiv((uint32_t)E);
  a.c_fd = FastDiv((uint32_t)C);
  size_t partial_bytes = 0;
  plan->col_style = E * (int64_t)sizeof(T) < kRowStyleMinBytes;
  plan->vec_stats = false;
  plan->nt_stats = (double)a.N * sizeof(T) * (og ? 2 : 1) >= (double)kStreamingBytes;
  if (plan->col_style) CT_REQUIRE(a.W < (int64_t(1) << 31), "batch-normalize: channels * elements exceeds the supported range");
  if (need_stats) {
    const bool aligned = (uintptr_t)x % 16 == 0 && (og == nullptr || (uintptr_t)og % 16 == 0);
    if (plan->col_style) {
      plan->vec_stats = aligned && a.W % VMAX == 0;
      const int vec = plan->vec_stats ? VMAX : 1;
      const int64_t gx = (a.W + 64 * vec - 1) / (64 * vec);
      int64_t S = std::max<int64_t>(1, std::min<int64_t>((B + 15) / 16, (1024 + gx - 1) / gx));
      S = std::min<int64_t>(S, 65535);
      while (S > 1 && (size_t)S * a.W * NACC * sizeof(double) > kMaxPartialBytes) S = (S + 1) / 2;
      a.S = (uint32_t)S;
      a.rows_per_seg = (uint32_t)((B + S - 1) / S);
      a.part_E = (uint32_t)E;
      plan->stats_grid = dim3((uint32_t)gx, (uint32_t)S);
      partial_bytes = (size_t)S * a.W * NACC * sizeof(double);
    } else {
      // every row is walked in vectors; rows off the 16-byte grid take element-aligned loads and a partial last vector
      plan->vec_stats = aligned && E % VMAX == 0;
      a.nv = (uint32_t)((E + VMAX - 1) / VMAX);
      a.nv_fd = FastDiv(a.nv);
      // About 16384 blocks, each with at least half a round of its 1024 loads in flight
      // (measured 5-6 % faster on the whole call than 2048 longer-lived blocks; 65536 lost 40 %).
      int64_t S = std::max<int64_t>(1, std::min<int64_t>(B, (16384 + C - 1) / C));
      while (S > 1 && (B + S - 1) / S * (int64_t)a.nv < 512) S = (S + 1) / 2;
      // a block's list of vectors is indexed with 31 bits
      while ((B + S - 1) / S * (int64_t)a.nv >= (int64_t(1) << 31)) S *= 2;
      S = std::min(S, B);
      a.S = (uint32_t)S;
      a.rows_per_seg = (uint32_t)((B + S - 1) / S);
      CT_REQUIRE((int64_t)a.rows_per_seg * a.nv < (int64_t(1) << 31) && C * S < (int64_t(1) << 31),
                 "batch-normalize: tensor shape exceeds the supported range");
      a.s_fd = FastDiv(a.S);
      a.part_E = 1;
      plan->stats_grid = dim3((uint32_t)(C * S));
      partial_bytes = (size_t)S * C * NACC * sizeof(double);
    }
  }
  const size_t param_bytes = (size_t)C * kParamStride * sizeof(double);
  plan->scratch_bytes = param_bytes + partial_bytes;
  void* scratch = nullptr;
  if (int rc = stream_scratch(s, plan->scratch_bytes, &scratch)) return rc;
  a.params = reinterpret_cast<double*>(scratch);
  a.partials = reinterpret_cast<double*>(reinterpret_cast<char*>(scratch) + param_bytes);
  return CT_OK;
}

template <class T, int MODE>
void bn_launch_stats(hipStream_t s, const BnPlan& plan) {
  constexpr int VMAX = 16 / (int)sizeof(T);
  if (plan.col_style) {
    if (plan.vec_stats) hipLaunchKernelGGL((bn_stats_col_kernel<T, VMAX, MODE>), plan.stats_grid, dim3(kBlock), 0, s, plan.a);
    else hipLaunchKernelGGL((bn_stats_col_kernel<T, 1, MODE>), plan.stats_grid, dim3(kBlock), 0, s, plan.a);
  } else {
    if (plan.vec_stats && plan.nt_stats) hipLaunchKernelGGL((bn_stats_row_kernel<T, VMAX, MODE, true, true>), plan.stats_grid, dim3(kBlock), 0, s, plan.a);
    else if (plan.vec_stats) hipLaunchKernelGGL((bn_stats_row_kernel<T, VMAX, MODE, true, false>), plan.stats_grid, dim3(kBlock), 0, s, plan.a);
    else hipLaunchKernelGGL((bn_stats_row_kernel<T, VMAX, MODE, false, false>), plan.stats_grid, dim3(kBlock), 0, s, plan.a);
  }
}

constexpr size_t kMaxTableBytes = size_t(60) << 10;

template <class T, int VEC, int MODE, int UNROLL>
bool bn_try_apply_range(hipStream_t s, BnArgs a, int64_t first, int64_t count) {
  constexpr int NP = bn_nparam<MODE>::value;
  constexpr int64_t kSpan = (int64_t)kBlock * VEC * UNROLL;
  a.first = first;
  a.count = count;
  a.row_holds_vectors = (a.E % VEC == 0 && first % VEC == 0) ? 1u : 0u;
  const int64_t window = (kSpan + a.E - 1) / a.E + 1;  // (batch, channel) rows a block's range can touch
  a.table_full = window >= a.C ? 1u : 0u;
  a.table_slots = (uint32_t)(a.table_full ? a.C : window);
  const size_t lds = (size_t)a.table_slots * NP * sizeof(double);
  if (lds > kMaxTableBytes) return false;
  const dim3 grid((uint32_t)((count + kSpan - 1) / kSpan));
  hipLaunchKernelGGL((bn_apply_kernel<T, VEC, MODE, UNROLL>), grid, dim3(kBlock), lds, s, a);
  return true;
}

// Few elements per channel make the table of a wide block large: narrow the block then.
template <class T, int VEC, int MODE>
void bn_launch_apply_range(hipStream_t s, const BnArgs& a, int64_t first, int64_t count) {
  if (count <= 0) return;
  if (!bn_try_apply_range<T, VEC, MODE, kUnroll>(s, a, first, count)) bn_try_apply_range<T, VEC, MODE, 1>(s, a, first, count);
}

template <class T, int VEC, int MODE>
void bn_launch_apply_col(hipStream_t s, BnArgs a) {
  const int64_t gx = (a.W + (int64_t)kBlock * VEC - 1) / ((int64_t)kBlock * VEC);
  int64_t segs = std::max<int64_t>(1, std::min<int64_t>((a.B + 3) / 4, (2048 + gx - 1) / gx));
  segs = std::min<int64_t>(segs, 65535);
  a.apply_rows_per_seg = (uint32_t)((a.B + segs - 1) / segs);
  segs = (a.B + a.apply_rows_per_seg - 1) / a.apply_rows_per_seg;
  hipLaunchKernelGGL((bn_apply_col_kernel<T, VEC, MODE>), dim3((uint32_t)gx, (uint32_t)segs), dim3(kBlock), 0, s, a);
}

template <class T> bool bn_operands_aligned(const BnArgs& a) {
  return (uintptr_t)a.x % 16 == 0 && (uintptr_t)a.out % 16 == 0 && (a.og == nullptr || (uintptr_t)a.og % 16 == 0);
}

// The layouts bn_apply_rows_kernel takes (it also needs the constants in the parameter table).
template <class T> bool bn_rows_layout(const BnPlan& plan) {
  constexpr int VMAX = 16 / (int)sizeof(T);
  const BnArgs& a = plan.a;
  return !plan.col_style && bn_operands_aligned<T>(a) && VMAX > 1 &&
         a.E / VMAX >= (a.E % VMAX ? kRaggedApplyMinVecs : kRowApplyMinVecs) && a.N < (int64_t(1) << 32);
}

template <class T, int MODE>
void bn_launch_apply(hipStream_t s, const BnPlan& plan) {
  constexpr int VMAX = 16 / (int)sizeof(T);
  const BnArgs& a = plan.a;
  const bool aligned = bn_operands_aligned<T>(a);
  if (plan.col_style) {
    if (aligned && a.W % VMAX == 0) bn_launch_apply_col<T, VMAX, MODE>(s, a);
    else bn_launch_apply_col<T, 1, MODE>(s, a);
  } else if (plan.params_ready && bn_rows_layout<T>(plan)) {
    const bool ragged = a.E % VMAX != 0;
    BnRowArgs r;
    r.total_vecs = (uint64_t)(a.N / VMAX);
    r.nv_fd = FastDiv((uint32_t)(ragged ? a.E : a.E / VMAX));
    r.c_fd = FastDiv((uint32_t)a.C);
    r.params = a.params;
    r.x = a.x; r.og = a.og; r.out = a.out;
    const dim3 grid((uint32_t)((r.total_vecs + kBlock - 1) / kBlock));
    r.grouped_blocks = xcd_grouped_blocks(grid.x);
    const double bytes = (double)a.N * sizeof(T) * (MODE == kBnGradient ? 3 : 2);
    // the apply pass is an elementwise call: non-temporal loads from the last-level cache's size on
    const int level = bytes >= (double)(int64_t(1) << 30) ? 2 : bytes >= (double)(int64_t(256) << 20) ? 1 : 0;
    if (ragged) {
      if (level == 2) hipLaunchKernelGGL((bn_apply_rows_kernel<T, VMAX, MODE, 2, true>), grid, dim3(kBlock), 0, s, r);
      else if (level == 1) hipLaunchKernelGGL((bn_apply_rows_kernel<T, VMAX, MODE, 1, true>), grid, dim3(kBlock), 0, s, r);
      else hipLaunchKernelGGL((bn_apply_rows_kernel<T, VMAX, MODE, 0, true>), grid, dim3(kBlock), 0, s, r);
      // the elements past the last whole vector
      bn_launch_apply_range<T, 1, MODE>(s, a, a.N / VMAX * VMAX, a.N % VMAX);
    } else {
      if (level == 2) hipLaunchKernelGGL((bn_apply_rows_kernel<T, VMAX, MODE, 2>), grid, dim3(kBlock), 0, s, r);
      else if (level == 1) hipLaunchKernelGGL((bn_apply_rows_kernel<T, VMAX, MODE, 1>), grid, dim3(kBlock), 0, s, r);
      else hipLaunchKernelGGL((bn_apply_rows_kernel<T, VMAX, MODE, 0>), grid, dim3(kBlock), 0, s, r);
    }
  } else if (aligned && VMAX > 1) {
    const int64_t body = a.N / VMAX * VMAX;
    bn_launch_apply_range<T, VMAX, MODE>(s, a, 0, body);
    bn_launch_apply_range<T, 1, MODE>(s, a, body, a.N - body);
  } else {
    bn_launch_apply_range<T, 1, MODE>(s, a, 0, a.N);
  }
}

inline dim3 channel_grid(int64_t C, int per_block) { return dim3((uint32_t)((C + per_block - 1) / per_block)); }

// ---------------------------------------------------------------- one launch for small tensors
//
// The networks the reference trains itself move batches of 128 x 784 through these methods
// (src/cortex/verify/nn/train.clj:185-187): three launches cost three times what the arithmetic
// does.  When a channel has at most kSmallChannelValues values (batch x elements) a block keeps
// whole channels in registers: it reads its channels once, forms their statistics (the mean first,
// then the squared distances from the rounded mean, exactly the CPU backend's two walks, or the
// five sums of the gradients in one walk), finishes them as bn_finish_kernel does and applies them
// to the values it holds.  One read, one write, one launch.
//
// A block of 256 lanes takes CG neighbouring channels with TPC = 256 / CG lanes each; lane t owns
// channel t % CG and every TPC-th value of it.  CG is a power of two of at most 64, so the lanes
// of one channel inside a wave are a fixed distance apart and combine with shuffles; the four
// waves meet in LDS.
constexpr int64_t kSmallChannelValues = 4096;
constexpr int64_t kSmallTensorElements = int64_t(1) << 21;

struct BnSmallArgs {
  const void* x;
  const void* og;
  void* out;
  const void* means;      // gradient mode: the batch statistics
  const void* variances;
  const void* scale;
  const void* bias;
  double epsilon;
  int64_t C, E;
  uint32_t count;         // values per channel: batch x elements
  uint32_t cg, tpc, cg_shift;
  FastDiv e_fd;
  BnFinish f;
};

template <int NACC>
__device__ __forceinline__ void bn_small_combine(double (&acc)[NACC], double (*lds)[kBlock / 64][64], uint32_t cg_count,
                                                 int lane, int wave, int cg) {
#pragma unroll
  for (int k = 0; k < NACC; ++k)
    for (uint32_t m = 32; m >= cg_count; m >>= 1) acc[k] += __shfl_xor(acc[k], (int)m, 64);
  if ((uint32_t)lane < cg_count) {
#pragma unroll
    for (int k = 0; k < NACC; ++k) lds[k][wave][lane] = acc[k];
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < NACC; ++k) {
    double t = lds[k][0][cg];
#pragma unroll
    for (int w = 1; w < kBlock / 64; ++w) t += lds[k][w][cg];
    acc[k] = t;
  }
}

template <class T, int MODE, int R>
__global__ void __launch_bounds__(kBlock) bn_small_kernel(const BnSmallArgs a) {
  constexpr int NACC = bn_nacc<MODE>::value;
  __shared__ double lds[NACC][kBlock / 64][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int cg = (int)(threadIdx.x & (a.cg - 1));
  const uint32_t part = threadIdx.x >> a.cg_shift;
  const int64_t c = (int64_t)blockIdx.x * a.cg + cg;
  const bool live = c < a.C;
  const T* xp = reinterpret_cast<const T*>(a.x);
  const T* gp = reinterpret_cast<const T*>(a.og);
  T x[R], g[MODE == kBnGradient ? R : 1];
  int64_t off[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const uint32_t i = part + (uint32_t)r * a.tpc;
    uint32_t b, e;
    a.e_fd.divmod(i, b, e);
    off[r] = live && i < a.count ? ((int64_t)b * a.C + c) * a.E + e : -1;
    x[r] = (T)0;
    if (off[r] >= 0) {
      x[r] = xp[off[r]];
      if constexpr (MODE == kBnGradient) g[r] = gp[off[r]];
    }
  }
  double pm[kParamStride];
  const int64_t count = a.count;
  if constexpr (MODE == kBnGradient) {
    const double mean = live ? (double)reinterpret_cast<const T*>(a.means)[c] : 0.0;
    const T scale = live ? reinterpret_cast<const T*>(a.scale)[c] : (T)0;
    double acc[NACC] = {0.0, 0.0, 0.0, 0.0, 0.0};
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (off[r] >= 0) bn_accumulate_gradient<T>(acc, x[r], g[r], mean, scale);
    bn_small_combine<NACC>(acc, lds, a.cg, lane, wave, cg);
    if (!live) return;
    // as bn_finish_kernel (cpu/tensor_math.clj:922-983)
    const T eps = (T)a.epsilon;
    const T pow_factor = (T)(-3.0 / 2.0);
    const double variance = (double)eps + (double)reinterpret_cast<const T*>(a.variances)[c];
    const double inv_std = 1.0 / sqrt(variance);
    const double d_var = (double)(T)(-0.5 * pow(variance, (double)pow_factor));
    const T d_var_d_out = (T)(d_var * acc[2]);
    const T d_mean_d_out = (T)((-inv_std) * acc[3] + (double)d_var_d_out * ((-2.0 * acc[4]) / (double)count));
    const double one_over_count = 1.0 / (double)count;
    pm[0] = mean; pm[1] = inv_std; pm[2] = (double)scale; pm[3] = d_var;
    pm[4] = (double)d_var_d_out * 2.0;
    pm[5] = (double)d_mean_d_out * one_over_count;
    pm[6] = one_over_count;
    if (part == 0) {
      reinterpret_cast<T*>(a.f.bias_gradient)[c] = (T)acc[0];
      reinterpret_cast<T*>(a.f.scale_gradient)[c] = (T)(inv_std * acc[1]);
    }
  } else {
    // batch-normalize-update-impl (cpu/tensor_math.clj:831-870): the mean, then the squared distances from it
    double acc[NACC] = {0.0, 0.0};
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (off[r] >= 0) acc[0] += (double)x[r];
    bn_small_combine<NACC>(acc, lds, a.cg, lane, wave, cg);
    const double count_val = fmax(1.0, (double)count);
    const double running_count_val = fmax(1.0, count_val - 1.0);
    const T new_mean = (T)(acc[0] / count_val);
    double sq = 0.0;
#pragma unroll
    for (int r = 0; r < R; ++r)
      if (off[r] >= 0) {
        const double d = (double)new_mean - (double)x[r];
        sq += d * d;
      }
    __syncthreads();  // every lane has read the sums before the table is written again
    double acc2[NACC] = {sq, 0.0};
    bn_small_combine<NACC>(acc2, lds, a.cg, lane, wave, cg);
    if (!live) return;
    const double new_var = acc2[0];
    const T batch_variance = (T)(new_var / count_val);
    const T eps = (T)a.epsilon;
    pm[0] = (double)new_mean;
    pm[1] = (double)(T)sqrt(1.0 / ((double)batch_variance + (double)eps));
    pm[2] = (double)reinterpret_cast<const T*>(a.scale)[c];
    pm[3] = (double)reinterpret_cast<const T*>(a.bias)[c];
    if (part == 0) {
      const T ave_factor = (T)a.f.average_factor;
      const double ave_lerp = (double)(T)1.0 - (double)ave_factor;
      T* running_means = reinterpret_cast<T*>(a.f.running_means);
      T* running_variances = reinterpret_cast<T*>(a.f.running_variances);
      const T mean = running_means[c], variance = running_variances[c];
      reinterpret_cast<T*>(a.f.batch_means)[c] = new_mean;
      reinterpret_cast<T*>(a.f.batch_variances)[c] = batch_variance;
      running_means[c] = (T)((double)mean * ave_lerp + (double)new_mean * (double)ave_factor);
      running_variances[c] =
          (T)((double)variance * ave_lerp + (double)(T)(new_var / running_count_val) * (double)ave_factor);
    }
  }
  T* op = reinterpret_cast<T*>(a.out);
#pragma unroll
  for (int r = 0; r < R; ++r)
    if (off[r] >= 0) op[off[r]] = bn_apply_one<T, MODE>(pm, x[r], MODE == kBnGradient ? g[r] : (T)0);
}

// Launches the one-launch form when the tensor qualifies; *taken says whether it did.
template <class T, int MODE>
int bn_small(hipStream_t s, BnSmallArgs& a, int64_t B, int64_t C, int64_t E, bool* taken) {
  *taken = false;
  const int64_t count = B * E;
  if (count > kSmallChannelValues || count * C > kSmallTensorElements) return CT_OK;
  // lanes per channel: enough that a lane holds at most eight values, at least four (the waves
  // meet in LDS either way), at most the block
  int64_t tpc = 4;
  while (tpc < kBlock && tpc * 8 < count) tpc *= 2;
  const int64_t per_lane = (count + tpc - 1) / tpc;
  a.count = (uint32_t)count;
  a.tpc = (uint32_t)tpc;
  a.cg = (uint32_t)(kBlock / tpc);
  a.cg_shift = 0;
  while ((1u << a.cg_shift) < a.cg) ++a.cg_shift;
  a.C = C; a.E = E;
  a.e_fd = FastDiv((uint32_t)E);
  const dim3 grid((uint32_t)((C + a.cg - 1) / a.cg));
  if (per_lane <= 4) hipLaunchKernelGGL((bn_small_kernel<T, MODE, 4>), grid, dim3(kBlock), 0, s, a);
  else if (per_lane <= 8) hipLaunchKernelGGL((bn_small_kernel<T, MODE, 8>), grid, dim3(kBlock), 0, s, a);
  else hipLaunchKernelGGL((bn_small_kernel<T, MODE, 16>), grid, dim3(kBlock), 0, s, a);
  *taken = true;
  return CT_OK;
}

inline void bn_set_statistics(BnArgs* a, const void* means, const void* variances, const void* scale, const void* bias,
                              double epsilon) {
  a->means = means; a->variances = variances; a->scale = scale; a->bias = bias; a->epsilon = epsilon;
}

template <class T>
int bn_normalize(hipStream_t s, void* output, const void* input, const void* means, const void* variances,
                 const void* scale, const void* bias, double epsilon, int64_t B, int64_t C, int64_t E) {
  BnPlan plan;
  if (int rc = bn_plan<T, kBnNormalize>(s, B, C, E, input, nullptr, output, false, &plan)) return rc;
  bn_set_statistics(&plan.a, means, variances, scale, bias, epsilon);
  note_kernel(plan.col_style ? "bn_apply_col" : "bn_apply");
  // a launch of its own for the constants pays off once the tensor is large
  if (bn_rows_layout<T>(plan) && (double)plan.a.N * sizeof(T) >= (double)kRowApplyBytes) {
    hipLaunchKernelGGL((bn_constants_kernel<T>), dim3((uint32_t)((C * 4 + kBlock - 1) / kBlock)), dim3(kBlock), 0, s, plan.a);
    plan.params_ready = true;
  }
  bn_launch_apply<T, kBnNormalize>(s, plan);
  return after_launch(s);
}

template <class T>
int bn_update_and_apply(hipStream_t s, void* output, const void* input, void* batch_means, void* batch_variances,
                        void* running_means, void* running_variances, double average_factor, const void* scale,
                        const void* bias, double epsilon, int64_t B, int64_t C, int64_t E) {
  CT_REQUIRE(B >= 1 && C >= 1 && E >= 1, "batch-normalize: batch, channel and element counts must be positive");
  {
    BnSmallArgs sa;
    std::memset(&sa, 0, sizeof(sa));
    sa.x = input; sa.out = output; sa.scale = scale; sa.bias = bias; sa.epsilon = epsilon;
    sa.f.batch_means = batch_means; sa.f.batch_variances = batch_variances;
    sa.f.running_means = running_means; sa.f.running_variances = running_variances;
    sa.f.average_factor = average_factor;
    bool taken = false;
    if (int rc = bn_small<T, kBnNormalize>(s, sa, B, C, E, &taken)) return rc;
    if (taken) {
      note_kernel("bn_update_small");
      return after_launch(s);
    }
  }
  BnPlan plan;
  if (int rc = bn_plan<T, kBnNormalize>(s, B, C, E, input, nullptr, output, true, &plan)) return rc;
  // the apply pass normalizes with the batch statistics the finishing pass writes
  bn_set_statistics(&plan.a, batch_means, batch_variances, scale, bias, epsilon);
  note_kernel(plan.col_style ? "bn_update_col" : "bn_update_row");
  bn_launch_stats<T, kBnNormalize>(s, plan);
  BnFinish f;
  std::memset(&f, 0, sizeof(f));
  f.batch_means = batch_means; f.batch_variances = batch_variances;
  f.running_means = running_means; f.running_variances = running_variances;
  f.average_factor = average_factor;
  hipLaunchKernelGGL((bn_finish_kernel<T, kBnNormalize>), channel_grid(C, kBlock / 64), dim3(kBlock), 0, s, plan.a, f);
  plan.params_ready = true;
  bn_launch_apply<T, kBnNormalize>(s, plan);
  return after_launch(s);
}

template <class T>
int bn_gradients(hipStream_t s, void* input_gradient, void* scale_gradient, void* bias_gradient,
                 const void* output_gradient, const void* input, const void* batch_means, const void* batch_variances,
                 const void* scale, double epsilon, int64_t B, int64_t C, int64_t E) {
  CT_REQUIRE(B >= 1 && C >= 1 && E >= 1, "batch-normalize: batch, channel and element counts must be positive");
  {
    BnSmallArgs sa;
    std::memset(&sa, 0, sizeof(sa));
    sa.x = input; sa.og = output_gradient; sa.out = input_gradient;
    sa.means = batch_means; sa.variances = batch_variances; sa.scale = scale; sa.epsilon = epsilon;
    sa.f.scale_gradient = scale_gradient; sa.f.bias_gradient = bias_gradient;
    bool taken = false;
    if (int rc = bn_small<T, kBnGradient>(s, sa, B, C, E, &taken)) return rc;
    if (taken) {
      note_kernel("bn_gradients_small");
      return after_launch(s);
    }
  }
  BnPlan plan;
  if (int rc = bn_plan<T, kBnGradient>(s, B, C, E, input, output_gradient, input_gradient, true, &plan)) return rc;
  bn_set_statistics(&plan.a, batch_means, batch_variances, scale, nullptr, epsilon);
  note_kernel(plan.col_style ? "bn_gradients_col" : "bn_gradients_row");
  bn_launch_stats<T, kBnGradient>(s, plan);
  BnFinish f;
  std::memset(&f, 0, sizeof(f));
  f.scale_gradient = scale_gradient; f.bias_gradient = bias_gradient;
  hipLaunchKernelGGL((bn_finish_kernel<T, kBnGradient>), channel_grid(C, kBlock / 64), dim3(kBlock), 0, s, plan.a, f);
  plan.params_ready = true;
  bn_launch_apply<T, kBnGradient>(s, plan);
  return after_launch(s);
}

#define CT_BN_FLOAT(dtype, ...)                                                                               \
  do {                                                                                                        \
    if ((dtype) == CT_F32) { using T = float; return __VA_ARGS__; }                                           \
    if ((dtype) == CT_F64) { using T = double; return __VA_ARGS__; }                                          \
    return set_error(CT_ERR_INVALID, "batch-normalization is only defined for float and double tensors");     \
  } while (0)

}  // namespace

extern "C" {

int ct_batch_normalize_spatial(void* stream, void* output, const void* input, const void* means,
                               const void* variances, const void* scale, const void* bias, double epsilon,
                               int64_t batch_count, int64_t channel_count, int64_t element_count, int dtype) {
  CT_REQUIRE(output && input && means && variances && scale && bias, "batch-normalize!: null buffer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  CT_BN_FLOAT(dtype, bn_normalize<T>(s, output, input, means, variances, scale, bias, epsilon, batch_count,
                                     channel_count, element_count));
}

int ct_batch_normalize_eltwise(void* stream, void* output, const void* input, const void* means,
                               const void* variances, const void* scale, const void* bias, double epsilon,
                               int64_t batch_count, int64_t element_count, int dtype) {
  return ct_batch_normalize_spatial(stream, output, input, means, variances, scale, bias, epsilon, batch_count,
                                    element_count, 1, dtype);
}

int ct_batch_normalize_update_and_apply_spatial(void* stream, void* output, const void* input, void* batch_means,
                                                void* batch_variances, void* running_means,
                                                void* running_variances, double average_factor, const void* scale,
                                                const void* bias, double epsilon, int64_t batch_count,
                                                int64_t channel_count, int64_t element_count, int dtype) {
  CT_REQUIRE(output && input && batch_means && batch_variances && running_means && running_variances && scale && bias,
             "batch-normalize-update-and-apply!: null buffer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  CT_BN_FLOAT(dtype, bn_update_and_apply<T>(s, output, input, batch_means, batch_variances, running_means,
                                            running_variances, average_factor, scale, bias, epsilon, batch_count,
                                            channel_count, element_count));
}

int ct_batch_normalize_update_and_apply_eltwise(void* stream, void* output, const void* input, void* batch_means,
                                                void* batch_variances, void* running_means,
                                                void* running_variances, double average_factor, const void* scale,
                                                const void* bias, double epsilon, int64_t batch_count,
                                                int64_t element_count, int dtype) {
  return ct_batch_normalize_update_and_apply_spatial(stream, output, input, batch_means, batch_variances,
                                                     running_means, running_variances, average_factor, scale, bias,
                                                     epsilon, batch_count, element_count, 1, dtype);
}

int ct_batch_normalize_gradients_spatial(void* stream, void* input_gradient, void* scale_gradient,
                                         void* bias_gradient, const void* output_gradient, const void* output,
                                         const void* input, const void* batch_means, const void* batch_variances,
                                         const void* scale, const void* bias, double epsilon, int64_t batch_count,
                                         int64_t channel_count, int64_t element_count, int dtype) {
  (void)output;
  (void)bias;
  CT_REQUIRE(input_gradient && scale_gradient && bias_gradient && output_gradient && input && batch_means &&
                 batch_variances && scale,
             "batch-normalize-gradients!: null buffer");
  hipStream_t s = static_cast<hipStream_t>(stream);
  CT_BN_FLOAT(dtype, bn_gradients<T>(s, input_gradient, scale_gradient, bias_gradient, output_gradient, input,
                                     batch_means, batch_variances, scale, epsilon, batch_count, channel_count,
                                     element_count));
}

int ct_batch_normalize_gradients_eltwise(void* stream, void* input_gradient, void* scale_gradient,
                                         void* bias_gradient, const void* output_gradient, const void* output,
                                         const void* input, const void* batch_means, const void* batch_variances,
                                         const void* scale, const void* bias, double epsilon, int64_t batch_count,
                                         int64_t element_count, int dtype) {
  return ct_batch_normalize_gradients_spatial(stream, input_gradient, scale_gradient, bias_gradient, output_gradient,
                                              output, input, batch_means, batch_variances, scale, bias, epsilon,
                                              batch_count, element_count, 1, dtype);
}

}  // extern "C"
