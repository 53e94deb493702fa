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

template <class T>
int pool_launch(hipStream_t s, bool forward, void* dest, const void* in, const void* out_values, const void* out_grad,
                const ct_pool_desc& d, const PoolShape& sh) {
  const int64_t in_plane = sh.in_h * sh.in_w, out_plane = sh.out_h * sh.out_w;
  const int64_t dest_plane = forward ? out_plane : in_plane;
  if (sh.planes == 0 || dest_plane == 0) return CT_OK;
  PoolArgs a{};
  a.in_h = (int32_t)sh.in_h; a.in_w = (int32_t)sh.in_w; a.out_h = (int32_t)sh.out_h; a.out_w = (int32_t)sh.out_w;
  a.kw = d.kernel_width; a.kh = d.kernel_height; a.px = d.pad_x; a.py = d.pad_y; a.sx = d.stride_x; a.sy = d.stride_y;
  a.in_plane = (uint32_t)in_plane; a.out_plane = (uint32_t)out_plane;
  a.plane_fd = FastDiv((uint32_t)dest_plane);
  a.row_fd = FastDiv((uint32_t)(forward ? sh.out_w : sh.in_w));
  a.sx_fd = FastDiv((uint32_t)d.stride_x);
  a.sy_fd = FastDiv((uint32_t)d.stride_y);
  // The first tap lies inside the padded input unless the stride carries the
  // last window past it; then max and avg continue from what the output holds.
  const bool first_tap_inside = (sh.out_w - 1) * d.stride_x - d.pad_x < sh.in_w + d.pad_x &&
                                (sh.out_h - 1) * d.stride_y - d.pad_y < sh.in_h + d.pad_y;
  a.load_prev = first_tap_inside ? 0u : 1u;
  const int64_t limit = (int64_t(1) << 31) - 1;
  const int64_t planes_per_launch = std::max<int64_t>(1, limit / std::max<int64_t>(1, std::max(in_plane, out_plane)));
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
  note_kernel("pool_forward");
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
  note_kernel("pool_backward");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == CT_F32) return pool_launch<float>(s, false, input_gradient, input, output, output_gradient, *desc, sh);
  return pool_launch<double>(s, false, input_gradient, input, output, output_gradient, *desc, sh);
}

}  // extern "C"
