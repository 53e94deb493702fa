// ops_lrn.hip -- lrn-forward! / lrn-backward! (src/cortex/tensor/math.clj:240-252;
// src/cortex/tensor.clj:1554-1616): local response normalization across the channels of
// [batch, channels, height, width] float and double tensors.  The reference has one
// implementation, cuDNN's cross-channel LRN (src/cortex/compute/cuda/tensor_math.clj:271-281,
// 1277-1335), whose published definition is what these kernels compute:
//
//   behind = (n - 1) / 2, ahead = n - 1 - behind, window(c) = [c - behind, c + ahead] inside [0, C)
//   s[c]  = k + (alpha / n) * sum over window(c) of x^2
//   y[c]  = x[c] * s[c]^-beta
//   dx[c] = dy[c] * s[c]^-beta - (2 alpha beta / n) * x[c] * sum over window(c) of dy y / s
//
// The backward sum runs over the same window as the forward one.  For an even n, whose window is
// not centred, the exact derivative would mirror it; the reference's stored results for n = 2
// (src/cortex/verify/tensor.clj:1105-1123) are those of the unmirrored window, so that is the
// definition here.
//
// Both directions are streams: 8 bytes per float element forward (read x, write y), 16 backward
// (read x, y, dy, write dx).  A block takes CH = 16 or 32 channels of 64 pixel vectors of one image
// and keeps the rows it needs in LDS: the CH + n - 1 rows of x around its channels (forward), or
// the CH + 2 (n - 1) rows of x and the CH + n - 1 rows of dy y / s (backward).  The x rows go from
// global memory straight into LDS (global_load_lds_dwordx4), all of a wave's rows issued at once;
// a lane's LDS accesses are 16 bytes wide and conflict-free
// (a wave reads one contiguous 1 KiB row), and the window sums are re-formed from their n terms
// for every channel: a running sum with subtraction would carry the error of large neighbours
// into small windows.  Double tensors compute in double throughout.  Float tensors compute in float
// on the hardware's exp2 / log2 / reciprocal units (about 20 instructions per element; the same
// arithmetic in double is 45 and bounds the kernel instead of memory), with a double path for
// the values where that would cost accuracy (see lrn_scales): results stay within 4e-6 of the
// double evaluation, relative to the terms that form them.
#include <atomic>

#include "elementwise.h"

namespace cthip {
namespace {

constexpr int kLrnMaxWindow = 16;  // cuDNN's CUDNN_LRN_MAX_N
constexpr int kLrnWaves = kBlock / 64;  // of the forward kernel

// Output channels per block.  Sixteen keep four to eight blocks on a compute unit, which hides the
// tiles' load-then-compute phases behind each other; the extra rows read around them (n - 1 of
// 16 + n - 1) come out of the caches.  Windows past 8 take 32.  Measured on float
// [64,256,56,56], n 5: forward 73 us with 16 channels against 77 with 32 and 99-106 with 64;
// backward, where LDS holds two tiles, 165 against 175 (eight waves per block; 194 / 217 with
// four, 183 / 202 with sixteen).
inline int lrn_channels_per_block(bool vec_ok, int n) { return vec_ok && n <= 8 ? 16 : 32; }

struct LrnOperand {
  const void* ptr;
  int64_t sb, sc, sh, sw;  // strides of batch, channel, row, column in elements
};

struct LrnArgs {
  LrnOperand x, y, dy, dx;  // forward: x -> y; backward: x, y, dy -> dx
  int32_t channels, window, behind, ahead;
  uint32_t pixels;          // height * width
  uint32_t pixel_vecs;      // vectors per image plane
  uint32_t p_tiles, c_chunks;
  FastDiv p_tiles_fd, c_chunks_fd, width_fd;
  double k, alpha_over_n, beta, cross_scale;  // cross_scale = 2 alpha beta / n
  float k_f, alpha_over_n_f, beta_f, cross_scale_f;
  int32_t beta_is_one;
};

// s^-beta for s > 0, for the lanes of float tensors that leave the hardware path (see lrn_scales):
// s = m 2^e with m in [1/2, 1); -beta (e + log2 m) is split into an integer and a fraction in
// [-1/2, 1/2] in double, and the hardware exp2 of the fraction is scaled by the integer.  The
// result stays a double: it may lie far outside the float range while its product with a large
// or small tensor value lies inside.
__device__ __forceinline__ double lrn_power_wide(double s, double beta, bool beta_is_one) {
  if (s > 1.7e308) return beta > 0.0 ? 0.0 : (beta < 0.0 ? s : 1.0);  // an infinite scale: pow(inf, -beta)
  int e;
  const float m = (float)frexp(s, &e);  // [1/2, 1)
  if (beta_is_one) return ldexp((double)__builtin_amdgcn_rcpf(m), -e);
  const double a = -beta * ((double)e + (double)__builtin_amdgcn_logf(m));
  const double whole = __builtin_rint(a);
  const float frac = (float)(a - whole);
  const double clipped = __builtin_fmin(__builtin_fmax(whole, -2000.0), 2000.0);
  return ldexp((double)__builtin_amdgcn_exp2f(frac), (int)clipped);
}

template <int VEC> __device__ __forceinline__ int64_t lrn_pixel_offset(const LrnOperand& t, const FastDiv& width_fd, uint32_t pv) {
  if constexpr (VEC > 1) {
    return (int64_t)pv * VEC;  // planes are contiguous on this path
  } else {
    uint32_t row, col;
    width_fd.divmod(pv, row, col);
    return (int64_t)row * t.sh + (int64_t)col * t.sw;
  }
}

// The scale s of one lane's vector at tile row `first` (the window is rows first .. first + n - 1
// of the x tile) and s^-beta.  Double tensors sum and take the power in double.  Float tensors sum
// the squares with float multiply-adds (no term cancels: n - 1 roundings at most) and take
// exp2(-beta log2 s) on the hardware units while |beta log2 s| <= 16, where the error of the
// product in the exponent stays under 1.5e-6 of the result.  Beyond that, and for sums past the
// float range, wide[e] is set to the scale recomputed in double (0 otherwise) and the caller forms
// its products with lrn_power_wide in double.
template <class T, int VEC>
__device__ __forceinline__ void lrn_scales(const LrnArgs& a, const Vec<T, VEC>* xt, int first, int lane, T* scale, T* power,
                                           double* wide) {
  using V = Vec<T, VEC>;
  if constexpr (std::is_same<T, double>::value) {
    double sum[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) sum[e] = 0.0;
    for (int w = 0; w < a.window; ++w) {
      const V t = xt[(first + w) * 64 + lane];
#pragma unroll
      for (int e = 0; e < VEC; ++e) sum[e] += t.v[e] * t.v[e];
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      scale[e] = a.k + a.alpha_over_n * sum[e];
      power[e] = a.beta_is_one ? 1.0 / scale[e] : pow(scale[e], -a.beta);
      wide[e] = 0.0;
    }
  } else {
    float sum[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) sum[e] = 0.0f;
    for (int w = 0; w < a.window; ++w) {
      const V t = xt[(first + w) * 64 + lane];
#pragma unroll
      for (int e = 0; e < VEC; ++e) sum[e] = __builtin_fmaf(t.v[e], t.v[e], sum[e]);
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      const float s = __builtin_fmaf(a.alpha_over_n_f, sum[e], a.k_f);
      const float exponent = -a.beta_f * __builtin_amdgcn_logf(s);
      scale[e] = s;
      power[e] = __builtin_amdgcn_exp2f(exponent);
      wide[e] = 0.0;
      if (!(s < 1e30f && __builtin_fabsf(exponent) <= 16.0f)) {
        double total = 0.0;
        for (int w = 0; w < a.window; ++w) {
          const double t = (double)xt[(first + w) * 64 + lane].v[e];
          total += t * t;
        }
        wide[e] = a.k + a.alpha_over_n * total;
      }
    }
  }
}

// Which (image, channel chunk, pixel tile) a block takes.  Consecutive block ids go round the
// eight dies, each with its own L2; the blocks of one die walk a contiguous eighth of the work,
// pixel tile fastest, then channel chunk, so that the chunks that read each other's border rows
// are resident on one die at the same time and those rows come out of its L2: HBM traffic falls
// from 1.12 (forward) and 1.23 (backward) times the algorithmic bytes to 1.00.  In time, against
// dealing consecutive units round the dies,
// float n 5: [128,96,27,27] forward 26 -> 21.5 us, backward 50 -> 43; [32,64,112,112] forward
// 35 -> 31, backward 76 -> 79; [64,256,56,56] 73.5 -> 76 and 146 -> 148.  (With the chunk running
// fastest instead, a die's loads are 1 KiB pieces a plane apart: 79 and 171 us on the last shape.)
__device__ __forceinline__ void lrn_block_place(const LrnArgs& a, uint32_t* image, uint32_t* chunk, uint32_t* tile) {
  const uint32_t per_die = gridDim.x / kXcds;
  uint32_t unit = blockIdx.x;
  if (unit < per_die * kXcds) unit = (unit % kXcds) * per_die + unit / kXcds;
  uint32_t q;
  a.p_tiles_fd.divmod(unit, q, *tile);
  a.c_chunks_fd.divmod(q, *image, *chunk);
}

// One row of a tile straight from global memory into LDS (gfx950's global_load_lds_dwordx4): the
// wave's 64 lanes bring 16 bytes each to consecutive places after `row`, with no register in
// between and no LDS store instruction.  `row` is the same for the whole wave; lanes that are
// switched off leave their places as they were.
template <class V> __device__ __forceinline__ void lrn_row_to_lds(const V* from, V* row) {
  static_assert(sizeof(V) == 16, "direct loads into LDS move 16 bytes per lane here");
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)from,
                                   (__attribute__((address_space(3))) void*)row, 16, 0, 0);
}

// A direct load into LDS is a vector-memory operation: it is counted by vmcnt, not by lgkmcnt, and
// the barrier waits for neither.  The rows one wave brings in are read by the other waves, so every
// wave waits for its own outstanding vector-memory loads before it reaches the barrier; only then
// does the barrier order those LDS writes before the other waves' reads.
__device__ __forceinline__ void lrn_wait_direct_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

template <class T, int VEC, int CH>
__global__ void __launch_bounds__(kBlock) lrn_forward_kernel(const LrnArgs a) {
  constexpr int kRows = (CH + kLrnMaxWindow - 1 + kLrnWaves - 1) / kLrnWaves;
  using V = Vec<T, VEC>;
  extern __shared__ __align__(16) char lrn_smem[];
  V* xt = reinterpret_cast<V*>(lrn_smem);  // [rows_x][64]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  uint32_t image, chunk, tile;
  lrn_block_place(a, &image, &chunk, &tile);
  const uint32_t pv = tile * 64 + lane;
  const bool live = pv < a.pixel_vecs;
  const int c0 = (int)chunk * CH;
  const int rows_x = CH + a.window - 1;
  const T* xp = reinterpret_cast<const T*>(a.x.ptr) + (int64_t)image * a.x.sb + lrn_pixel_offset<VEC>(a.x, a.width_fd, live ? pv : 0);
  if constexpr (VEC > 1) {
    V zero;
#pragma unroll
    for (int e = 0; e < VEC; ++e) zero.v[e] = (T)0;
    for (int j = wave; j < rows_x; j += kLrnWaves) {
      const int c = c0 - a.behind + j;
      if (c >= 0 && c < a.channels) {
        if (live) lrn_row_to_lds(reinterpret_cast<const V*>(xp + (int64_t)c * a.x.sc), xt + j * 64);
      } else {
        xt[j * 64 + lane] = zero;
      }
    }
  } else {
    V held[kRows];
#pragma unroll
    for (int q = 0; q < kRows; ++q) {
      const int j = wave + q * kLrnWaves;
      const int c = c0 - a.behind + j;
      held[q].v[0] = (T)0;
      if (j < rows_x && live && c >= 0 && c < a.channels) held[q] = *reinterpret_cast<const V*>(xp + (int64_t)c * a.x.sc);
    }
#pragma unroll
    for (int q = 0; q < kRows; ++q) {
      const int j = wave + q * kLrnWaves;
      if (j < rows_x) xt[j * 64 + lane] = held[q];
    }
  }
  if constexpr (VEC > 1) lrn_wait_direct_loads();
  __syncthreads();
  if (!live) return;
  T* yp = reinterpret_cast<T*>(const_cast<void*>(a.y.ptr)) + (int64_t)image * a.y.sb + lrn_pixel_offset<VEC>(a.y, a.width_fd, pv);
#pragma unroll
  for (int q = 0; q < CH / kLrnWaves; ++q) {
    const int i = wave + q * kLrnWaves;
    const int c = c0 + i;
    if (c >= a.channels) break;
    T scale[VEC], power[VEC];
    double wide[VEC];
    lrn_scales<T, VEC>(a, xt, i, lane, scale, power, wide);
    const V centre = xt[(i + a.behind) * 64 + lane];
    V out;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      out.v[e] = centre.v[e] * power[e];
      if (wide[e] != 0.0) out.v[e] = (T)((double)centre.v[e] * lrn_power_wide(wide[e], a.beta, a.beta_is_one != 0));
    }
    *reinterpret_cast<V*>(yp + (int64_t)c * a.y.sc) = out;
  }
}

template <class T, int VEC, int CH, int WAVES>
__global__ void __launch_bounds__(WAVES * 64) lrn_backward_kernel(const LrnArgs a) {
  constexpr int kRows = (CH + kLrnMaxWindow - 1 + WAVES - 1) / WAVES;
  constexpr int kXRows = (CH + 2 * (kLrnMaxWindow - 1) + WAVES - 1) / WAVES;
  using V = Vec<T, VEC>;
  using R = Vec<T, VEC>;  // dy y / s, kept in the tensor's type
  extern __shared__ __align__(16) char lrn_smem[];
  const int rows_x = CH + 2 * (a.window - 1);
  const int rows_r = CH + a.window - 1;
  V* xt = reinterpret_cast<V*>(lrn_smem);  // [rows_x][64], row j is channel c0 - 2 behind + j
  R* rt = reinterpret_cast<R*>(xt + rows_x * 64);  // [rows_r][64], row j is channel c0 - behind + j
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  uint32_t image, chunk, tile;
  lrn_block_place(a, &image, &chunk, &tile);
  const uint32_t pv = tile * 64 + lane;
  const bool live = pv < a.pixel_vecs;
  const int c0 = (int)chunk * CH;
  const uint32_t pv0 = live ? pv : 0;
  const T* xp = reinterpret_cast<const T*>(a.x.ptr) + (int64_t)image * a.x.sb + lrn_pixel_offset<VEC>(a.x, a.width_fd, pv0);
  const T* yp = reinterpret_cast<const T*>(a.y.ptr) + (int64_t)image * a.y.sb + lrn_pixel_offset<VEC>(a.y, a.width_fd, pv0);
  const T* gp = reinterpret_cast<const T*>(a.dy.ptr) + (int64_t)image * a.dy.sb + lrn_pixel_offset<VEC>(a.dy, a.width_fd, pv0);
  V yheld[kRows], gheld[kRows];
  if constexpr (VEC > 1) {
    V zero;
#pragma unroll
    for (int e = 0; e < VEC; ++e) zero.v[e] = (T)0;
    for (int j = wave; j < rows_x; j += WAVES) {
      const int c = c0 - 2 * a.behind + j;
      if (c >= 0 && c < a.channels) {
        if (live) lrn_row_to_lds(reinterpret_cast<const V*>(xp + (int64_t)c * a.x.sc), xt + j * 64);
      } else {
        xt[j * 64 + lane] = zero;
      }
    }
  }
  V xheld[VEC > 1 ? 1 : kXRows];
  if constexpr (VEC == 1) {
#pragma unroll
    for (int q = 0; q < kXRows; ++q) {
      const int j = wave + q * WAVES;
      const int c = c0 - 2 * a.behind + j;
      xheld[q].v[0] = (T)0;
      if (j < rows_x && live && c >= 0 && c < a.channels) xheld[q] = *reinterpret_cast<const V*>(xp + (int64_t)c * a.x.sc);
    }
  }
#pragma unroll
  for (int q = 0; q < kRows; ++q) {
    const int j = wave + q * WAVES;
    const int c = c0 - a.behind + j;
#pragma unroll
    for (int e = 0; e < VEC; ++e) { yheld[q].v[e] = (T)0; gheld[q].v[e] = (T)0; }
    if (j < rows_r && live && c >= 0 && c < a.channels) {
      yheld[q] = *reinterpret_cast<const V*>(yp + (int64_t)c * a.y.sc);
      gheld[q] = *reinterpret_cast<const V*>(gp + (int64_t)c * a.dy.sc);
    }
  }
  if constexpr (VEC == 1) {
#pragma unroll
    for (int q = 0; q < kXRows; ++q) {
      const int j = wave + q * WAVES;
      if (j < rows_x) xt[j * 64 + lane] = xheld[q];
    }
  }
  if constexpr (VEC > 1) lrn_wait_direct_loads();
  __syncthreads();
  // dy y / s of this wave's rows goes to LDS; dy s^-beta stays in gheld for the rows that are outputs
#pragma unroll
  for (int q = 0; q < kRows; ++q) {
    const int j = wave + q * WAVES;
    if (j >= rows_r) break;
    const int c = c0 - a.behind + j;
    R ratio;
#pragma unroll
    for (int e = 0; e < VEC; ++e) ratio.v[e] = (T)0;
    if (live && c >= 0 && c < a.channels) {
      T scale[VEC], power[VEC];
      double wide[VEC];
      lrn_scales<T, VEC>(a, xt, j, lane, scale, power, wide);
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const T g = gheld[q].v[e];
        if constexpr (std::is_same<T, double>::value) ratio.v[e] = g * yheld[q].v[e] / scale[e];
        else ratio.v[e] = g * yheld[q].v[e] * __builtin_amdgcn_rcpf(scale[e]);
        gheld[q].v[e] = g * power[e];
        if (wide[e] != 0.0) {
          ratio.v[e] = (T)((double)g * (double)yheld[q].v[e] / wide[e]);
          gheld[q].v[e] = (T)((double)g * lrn_power_wide(wide[e], a.beta, a.beta_is_one != 0));
        }
      }
    }
    rt[j * 64 + lane] = ratio;
  }
  __syncthreads();
  if (!live) return;
  T* dp = reinterpret_cast<T*>(const_cast<void*>(a.dx.ptr)) + (int64_t)image * a.dx.sb + lrn_pixel_offset<VEC>(a.dx, a.width_fd, pv);
#pragma unroll
  for (int q = 0; q < kRows; ++q) {
    const int j = wave + q * WAVES;
    if (j >= rows_r) break;
    const int i = j - a.behind;  // output row: channel c0 + i
    const int c = c0 + i;
    if (i < 0 || i >= CH || c >= a.channels) continue;
    T cross[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) cross[e] = (T)0;
    for (int w = 0; w < a.window; ++w) {
      const R t = rt[(i + w) * 64 + lane];
#pragma unroll
      for (int e = 0; e < VEC; ++e) cross[e] += t.v[e];
    }
    const V centre = xt[(i + 2 * a.behind) * 64 + lane];
    V out;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      if constexpr (std::is_same<T, double>::value) out.v[e] = gheld[q].v[e] - a.cross_scale * centre.v[e] * cross[e];
      else out.v[e] = gheld[q].v[e] - a.cross_scale_f * centre.v[e] * cross[e];
    }
    *reinterpret_cast<V*>(dp + (int64_t)c * a.dx.sc) = out;
  }
}

struct LrnShape {
  int64_t size[4];
};

// Pads the dimensions to [batch, channels, height, width] as cuda/driver.clj:1094-1108 does.
int lrn_operand(const ct_dims* d, const void* ptr, const char* what, LrnShape* shape, LrnOperand* op) {
  if (int rc = check_dims(d, what)) return rc;
  CT_REQUIRE(d->ndim >= 3, "tensor must be of at least rank 3 (%s has rank %d)", what, d->ndim);
  CT_REQUIRE(d->ndim <= 4, "lrn: at most 4 dimensions (%s has rank %d)", what, d->ndim);
  CT_REQUIRE(dims_direct(*d), "lrn: %s is indexed through a tensor; only direct dimensions are supported", what);
  int64_t size[4] = {1, 1, 1, 1}, stride[4] = {0, 0, 0, 0};
  for (int i = 0; i < d->ndim; ++i) {
    size[i + 4 - d->ndim] = d->shape[i];
    stride[i + 4 - d->ndim] = d->strides[i];
  }
  for (int i = 0; i < 4; ++i) shape->size[i] = size[i];
  op->ptr = ptr;
  op->sb = stride[0]; op->sc = stride[1]; op->sh = stride[2]; op->sw = stride[3];
  return CT_OK;
}

bool same_shape(const LrnShape& a, const LrnShape& b) {
  for (int i = 0; i < 4; ++i)
    if (a.size[i] != b.size[i]) return false;
  return true;
}

// True when the planes of t are contiguous and everything sits on the vector grid.
template <class T> bool lrn_vector_ok(const LrnOperand& t, const LrnShape& s, int vec) {
  const bool plane = (s.size[3] == 1 || t.sw == 1) && (s.size[2] == 1 || t.sh == s.size[3]);
  return plane && (s.size[2] * s.size[3]) % vec == 0 && (s.size[1] == 1 || t.sc % vec == 0) && (s.size[0] == 1 || t.sb % vec == 0) &&
         ((uintptr_t)t.ptr % (uintptr_t)(vec * sizeof(T))) == 0;
}

int lrn_fill(LrnArgs* a, const LrnShape& s, int n, double k, double alpha, double beta, int vec, int ch) {
  CT_REQUIRE(n >= 1 && n <= kLrnMaxWindow, "lrn: n = %d is outside [1, %d]", n, kLrnMaxWindow);
  CT_REQUIRE(k >= 1e-5, "lrn: k = %g is below 1e-5", k);  // cuDNN's CUDNN_LRN_MIN_K
  CT_REQUIRE(alpha == alpha && beta == beta && alpha - alpha == 0.0 && beta - beta == 0.0, "lrn: alpha and beta must be finite");
  const int64_t pixels = s.size[2] * s.size[3];
  CT_REQUIRE(s.size[1] < (int64_t(1) << 30) && pixels < (int64_t(1) << 31) && s.size[0] < (int64_t(1) << 31), "lrn: tensor too large");
  a->channels = (int32_t)s.size[1];
  a->window = n;
  a->behind = (n - 1) / 2;
  a->ahead = n - 1 - a->behind;
  a->pixels = (uint32_t)pixels;
  a->pixel_vecs = (uint32_t)(pixels / vec);
  a->p_tiles = (a->pixel_vecs + 63) / 64;
  a->c_chunks = (uint32_t)((s.size[1] + ch - 1) / ch);
  a->p_tiles_fd = FastDiv(a->p_tiles);
  a->c_chunks_fd = FastDiv(a->c_chunks);
  a->width_fd = FastDiv((uint32_t)s.size[3]);
  a->k = k;
  a->alpha_over_n = alpha / (double)n;
  a->beta = beta;
  a->cross_scale = 2.0 * alpha * beta / (double)n;
  a->beta_is_one = beta == 1.0 ? 1 : 0;
  a->k_f = (float)k;
  a->alpha_over_n_f = (float)a->alpha_over_n;
  a->beta_f = (float)beta;
  a->cross_scale_f = (float)a->cross_scale;
  const int64_t grid = (int64_t)a->p_tiles * a->c_chunks * s.size[0];
  CT_REQUIRE(grid < (int64_t(1) << 31), "lrn: tensor too large");
  return CT_OK;
}

// A launch may ask for more than 64 KiB of dynamic LDS only after the kernel's limit has been
// raised, once per kernel and device (the backward tiles of wide windows need up to 109 KiB).
constexpr size_t kLrnBackwardMaxLds = (size_t)(2 * 32 + 3 * (kLrnMaxWindow - 1)) * 64 * 16;
template <auto Kernel> int lrn_allow_lds(size_t bytes) {
  static std::atomic<uint64_t> raised{0};
  int dev = 0;
  CT_HIP(hipGetDevice(&dev));
  const uint64_t bit = uint64_t(1) << (dev & 63);
  if (raised.load(std::memory_order_acquire) & bit) return CT_OK;
  CT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(Kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
  raised.fetch_or(bit, std::memory_order_release);
  return CT_OK;
}

template <class T>
int lrn_forward_run(hipStream_t st, LrnArgs& a, const LrnShape& s, int n, double k, double alpha, double beta) {
  constexpr int VMAX = 16 / (int)sizeof(T);
  const bool vec_ok = lrn_vector_ok<T>(a.x, s, VMAX) && lrn_vector_ok<T>(a.y, s, VMAX);
  const int vec = vec_ok ? VMAX : 1;
  const int ch = lrn_channels_per_block(vec_ok, n);
  if (int rc = lrn_fill(&a, s, n, k, alpha, beta, vec, ch)) return rc;
  const dim3 grid((uint32_t)((int64_t)a.p_tiles * a.c_chunks * s.size[0]));
  const size_t lds = (size_t)(ch + n - 1) * 64 * vec * sizeof(T);  // at most 47 KiB
  note_kernel(vec_ok ? "lrn_forward_vec" : "lrn_forward");
  if (!vec_ok) hipLaunchKernelGGL((lrn_forward_kernel<T, 1, 32>), grid, dim3(kBlock), lds, st, a);
  else if (ch == 16) hipLaunchKernelGGL((lrn_forward_kernel<T, VMAX, 16>), grid, dim3(kBlock), lds, st, a);
  else hipLaunchKernelGGL((lrn_forward_kernel<T, VMAX, 32>), grid, dim3(kBlock), lds, st, a);
  return after_launch(st);
}

template <class T>
int lrn_backward_run(hipStream_t st, LrnArgs& a, const LrnShape& s, int n, double k, double alpha, double beta) {
  constexpr int VMAX = 16 / (int)sizeof(T);
  const bool vec_ok = lrn_vector_ok<T>(a.x, s, VMAX) && lrn_vector_ok<T>(a.y, s, VMAX) && lrn_vector_ok<T>(a.dy, s, VMAX) &&
                      lrn_vector_ok<T>(a.dx, s, VMAX);
  const int vec = vec_ok ? VMAX : 1;
  const int ch = lrn_channels_per_block(vec_ok, n);
  if (int rc = lrn_fill(&a, s, n, k, alpha, beta, vec, ch)) return rc;
  const dim3 grid((uint32_t)((int64_t)a.p_tiles * a.c_chunks * s.size[0]));
  const size_t lds = (size_t)(2 * ch + 3 * (n - 1)) * 64 * vec * sizeof(T);
  note_kernel(vec_ok ? "lrn_backward_vec" : "lrn_backward");
  if (!vec_ok) {
    hipLaunchKernelGGL((lrn_backward_kernel<T, 1, 32, 4>), grid, dim3(4 * 64), lds, st, a);
  } else if (ch == 16) {
    if (int rc = lrn_allow_lds<lrn_backward_kernel<T, VMAX, 16, 8>>(kLrnBackwardMaxLds)) return rc;
    hipLaunchKernelGGL((lrn_backward_kernel<T, VMAX, 16, 8>), grid, dim3(8 * 64), lds, st, a);
  } else {
    if (int rc = lrn_allow_lds<lrn_backward_kernel<T, VMAX, 32, 8>>(kLrnBackwardMaxLds)) return rc;
    hipLaunchKernelGGL((lrn_backward_kernel<T, VMAX, 32, 8>), grid, dim3(8 * 64), lds, st, a);
  }
  return after_launch(st);
}

}  // namespace
}  // namespace cthip

using namespace cthip;

extern "C" int ct_lrn_forward(void* stream, void* output, const ct_dims* output_dims, const void* input,
                              const ct_dims* input_dims, int n, double k, double alpha, double beta, int dtype) {
  CT_REQUIRE(output && input, "lrn-forward!: null buffer");
  CT_REQUIRE(output != input, "lrn-forward!: the output may not be the input (neighbouring channels read it)");
  LrnArgs a;
  std::memset(&a, 0, sizeof(a));
  LrnShape si, so;
  if (int rc = lrn_operand(input_dims, input, "input", &si, &a.x)) return rc;
  if (int rc = lrn_operand(output_dims, output, "output", &so, &a.y)) return rc;
  CT_REQUIRE(same_shape(si, so), "Input and output shapes must match");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == CT_F32) return lrn_forward_run<float>(st, a, si, n, k, alpha, beta);
  if (dtype == CT_F64) return lrn_forward_run<double>(st, a, si, n, k, alpha, beta);
  return set_error(CT_ERR_INVALID, "lrn-forward is only defined for float and double tensors");
}

extern "C" int ct_lrn_backward(void* stream, void* input_gradient, const ct_dims* input_gradient_dims, const void* output,
                               const ct_dims* output_dims, const void* input, const ct_dims* input_dims,
                               const void* output_gradient, const ct_dims* output_gradient_dims, int n, double k,
                               double alpha, double beta, int dtype) {
  CT_REQUIRE(input_gradient && output && input && output_gradient, "lrn-backward!: null buffer");
  CT_REQUIRE(input_gradient != output_gradient && input_gradient != output && input_gradient != input,
             "lrn-backward!: the input gradient may not be one of the tensors read (neighbouring channels read them)");
  LrnArgs a;
  std::memset(&a, 0, sizeof(a));
  LrnShape si, so, sg, sd;
  if (int rc = lrn_operand(input_dims, input, "input", &si, &a.x)) return rc;
  if (int rc = lrn_operand(output_dims, output, "output", &so, &a.y)) return rc;
  if (int rc = lrn_operand(output_gradient_dims, output_gradient, "output-gradient", &sg, &a.dy)) return rc;
  if (int rc = lrn_operand(input_gradient_dims, input_gradient, "input-gradient", &sd, &a.dx)) return rc;
  CT_REQUIRE(same_shape(si, so) && same_shape(si, sg) && same_shape(si, sd), "Input and output shapes must match");
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == CT_F32) return lrn_backward_run<float>(st, a, si, n, k, alpha, beta);
  if (dtype == CT_F64) return lrn_backward_run<double>(st, a, si, n, k, alpha, beta);
  return set_error(CT_ERR_INVALID, "lrn-backward is only defined for float and double tensors");
}
