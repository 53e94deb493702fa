// ops_conv.hip -- convolution-forward!, convolution-backward-weights! and
// convolution-backward-data! (src/cortex/tensor/math.clj:185-220) with the
// decomposition of the reference's CPU backend
// (src/cortex/compute/cpu/tensor_math.clj:1118-1151, 1670-1792): the input is
// unrolled into the caller's workspace (window walk: src/cortex/nn/impl.clj:8-96)
// and each method is one gemm! per image around that matrix.
//
// Workspace layout.  The CPU backend stores an image's unrolled input as
// [position, in_channels * kh * kw]; here it is the transpose,
// [in_channels * kh * kw, position] with position = out_y * out_w + out_x.  The
// workspace is opaque to callers (they size it with choose-convolution-algorithms
// and only hand it back), the products merely swap their transposition flags,
// and with the positions innermost both data movements are linear on both sides:
// neighbouring lanes read neighbouring input elements and write neighbouring
// cells.  (With the CPU backend's layout the roll-back read 13 times its
// algorithmic bytes from HBM and ran at 7 % of the peak, the unroll at 20 %.)
//
//   unroll     one lane per 16 bytes of cells of one (channel, tap) row: reads a
//              run of input positions, writes one aligned piece.  HBM-bound on
//              the workspace it writes, kh * kw times the input.
//   roll back  the reference adds cell after cell into the input gradient while
//              it walks the windows; here every input element gathers the cells
//              that came from it, windows in increasing (row, column) order,
//              which is the order in which that walk reaches the element: the
//              same roundings, no atomics.  Reads the workspace once.
//   products   ONE strided-batched rocBLAS call per method (an image's product
//              alone leaves most of the device idle).  The weight gradient, which
//              the reference accumulates image after image into one matrix, is
//              formed as per-image products in the stream's scratch memory and
//              summed over the images in double by a small kernel.
#include <algorithm>

#include "common.h"

using namespace cthip;

namespace cthip {
int gemm_strided_batched(void* stream, void* c, int64_t c_colstride, int64_t c_stride, int trans_a, int trans_b,
                         double alpha, const void* a, int64_t a_row_count, int64_t a_col_count, int64_t a_colstride,
                         int64_t a_stride, const void* b, int64_t b_col_count, int64_t b_colstride, int64_t b_stride,
                         double beta, int64_t batch_count, int dtype);
}

namespace {

constexpr int kBlock = 256;

struct ConvArgs {
  const void* src;
  void* dest;
  uint32_t total;  // lanes' worth of work in this launch
  uint32_t grouped_blocks;
  int32_t in_h, in_w, out_h, out_w;
  int32_t kw, kh, px, py, sx, sy;
  uint32_t channels, n_cols, n_rows, in_plane;
  FastDiv cols_fd, kk_fd, kw_fd, out_w_fd, rows_fd;  // unroll: cell -> (image, position, channel, tap)
  FastDiv in_w_fd, in_plane_fd, image_fd, sx_fd, sy_fd;  // roll back: element -> (image, channel, row, column)
};

// workspace[image][channel * kh * kw + k_y * kw + k_x][position] = input tap or 0 in the padding
template <class T, int VEC>
__global__ void __launch_bounds__(kBlock) conv_unroll_kernel(const ConvArgs a) {
  // The kh * kw rows of one channel read the same input plane: in the die-grouped
  // block order they run on one die and share its L2 (HBM reads of the input for
  // [64, 64, 56, 56] float, 3 x 3: 3.7 times the input before, 1.2 times after).
  // A variant that gave every block one row of cells, to decode the row on the
  // scalar unit, left too many lanes idle at the row ends and was slower.
  const uint32_t lane = xcd_grouped_unit(blockIdx.x, a.grouped_blocks) * kBlock + threadIdx.x;
  if (lane >= a.total) return;
  const uint32_t cell0 = lane * VEC;
  uint32_t row_all, position, image, col, chan, tap, ky, kx, oy, ox;
  a.rows_fd.divmod(cell0, row_all, position);   // row_all = image * n_cols + col
  a.cols_fd.divmod(row_all, image, col);
  a.kk_fd.divmod(col, chan, tap);
  a.kw_fd.divmod(tap, ky, kx);
  a.out_w_fd.divmod(position, oy, ox);
  const T* in = reinterpret_cast<const T*>(a.src) + ((int64_t)image * a.channels + chan) * a.in_plane;
  struct alignas(sizeof(T) * VEC) Piece { T v[VEC]; } piece;
  int32_t iy = (int32_t)oy * a.sy - a.py + (int32_t)ky, ix = (int32_t)ox * a.sx - a.px + (int32_t)kx;
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    const bool inside = (uint32_t)iy < (uint32_t)a.in_h && (uint32_t)ix < (uint32_t)a.in_w;
    piece.v[e] = inside ? in[iy * a.in_w + ix] : (T)0;
    ix += a.sx;
    if (++ox == (uint32_t)a.out_w) {
      ox = 0;
      ix = (int32_t)kx - a.px;
      iy += a.sy;
    }
  }
  *reinterpret_cast<Piece*>(reinterpret_cast<T*>(a.dest) + (int64_t)cell0) = piece;
}

// The same for stride_x 1 and an output width that is a whole number of 16-byte pieces: the
// cells of a piece are consecutive input elements of one input row, fetched with ONE
// (unaligned) 16-byte load and then masked where they fall into the padding.  Only a run that
// would leave the channel's plane (first and last row) is read element by element.
template <class T>
__global__ void __launch_bounds__(kBlock) conv_unroll_unit_stride_kernel(const ConvArgs a) {
  constexpr int VEC = 16 / sizeof(T);
  const uint32_t lane = xcd_grouped_unit(blockIdx.x, a.grouped_blocks) * kBlock + threadIdx.x;
  if (lane >= a.total) return;
  const uint32_t cell0 = lane * VEC;
  uint32_t row_all, position, plane, tap, ky, kx, oy, ox;
  a.rows_fd.divmod(cell0, row_all, position);   // row_all = (image * channels + channel) * kh * kw + tap
  a.kk_fd.divmod(row_all, plane, tap);
  a.kw_fd.divmod(tap, ky, kx);
  a.out_w_fd.divmod(position, oy, ox);
  const T* in = reinterpret_cast<const T*>(a.src) + (int64_t)plane * a.in_plane;
  const int32_t iy = (int32_t)oy * a.sy - a.py + (int32_t)ky, ix = (int32_t)ox - a.px + (int32_t)kx;
  struct alignas(16) Piece { T v[VEC]; } piece;
#pragma unroll
  for (int e = 0; e < VEC; ++e) piece.v[e] = (T)0;
  if ((uint32_t)iy < (uint32_t)a.in_h) {
    const int32_t at = iy * a.in_w + ix;
    if (at >= 0 && at + VEC <= (int32_t)a.in_plane) {
      __builtin_memcpy(&piece, in + at, 16);
#pragma unroll
      for (int e = 0; e < VEC; ++e)
        if ((uint32_t)(ix + e) >= (uint32_t)a.in_w) piece.v[e] = (T)0;
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e)
        if ((uint32_t)(ix + e) < (uint32_t)a.in_w) piece.v[e] = in[at + e];
    }
  }
  *reinterpret_cast<Piece*>(reinterpret_cast<T*>(a.dest) + (int64_t)cell0) = piece;
}

// input_gradient[image][channel][y][x] = sum of the workspace cells unrolled from it
template <class T>
__global__ void __launch_bounds__(kBlock) conv_roll_kernel(const ConvArgs a) {
  const uint32_t e = blockIdx.x * kBlock + threadIdx.x;
  if (e >= a.total) return;
  uint32_t image, rest, chan, r, iy, ix;
  a.image_fd.divmod(e, image, rest);
  a.in_plane_fd.divmod(rest, chan, r);
  a.in_w_fd.divmod(r, iy, ix);
  const T* conv = reinterpret_cast<const T*>(a.src) +
                  ((int64_t)image * a.n_cols + (int64_t)chan * (uint32_t)(a.kw * a.kh)) * a.n_rows;
  // Windows o with o * stride - pad <= i < o * stride - pad + k.
  const int32_t ty = (int32_t)iy + a.py, tx = (int32_t)ix + a.px;
  const int32_t oy_hi = min(a.out_h - 1, (int32_t)a.sy_fd.div((uint32_t)ty));
  const int32_t ox_hi = min(a.out_w - 1, (int32_t)a.sx_fd.div((uint32_t)tx));
  const int32_t by = ty - a.kh + 1, bx = tx - a.kw + 1;
  const int32_t oy_lo = by <= 0 ? 0 : (int32_t)a.sy_fd.div((uint32_t)(by + a.sy - 1));
  const int32_t ox_lo = bx <= 0 ? 0 : (int32_t)a.sx_fd.div((uint32_t)(bx + a.sx - 1));
  T acc = (T)0;
  for (int32_t oy = oy_lo; oy <= oy_hi; ++oy) {
    const int32_t ky = ty - oy * a.sy;
    for (int32_t ox = ox_lo; ox <= ox_hi; ++ox) {
      const int32_t kx = tx - ox * a.sx;
      acc = acc + conv[(int64_t)(ky * a.kw + kx) * a.n_rows + oy * a.out_w + ox];
    }
  }
  reinterpret_cast<T*>(a.dest)[e] = acc;
}

// The same for stride 1 and a fixed window: window (y, x) holds input (i_y, i_x) at tap
// (i_y + pad - y, i_x + pad - x), so the taps taken in DEcreasing order are the windows in
// increasing order, and the cell of tap (k_y, k_x) lies a constant distance from the cell
// of tap (0, 0).  No loops, no divisions beyond the element's own decomposition.
template <class T, int KW, int KH>
__global__ void __launch_bounds__(kBlock) conv_roll_unit_stride_kernel(const ConvArgs a) {
  const uint32_t e = blockIdx.x * kBlock + threadIdx.x;
  if (e >= a.total) return;
  uint32_t image, rest, chan, r, iy, ix;
  a.image_fd.divmod(e, image, rest);
  a.in_plane_fd.divmod(rest, chan, r);
  a.in_w_fd.divmod(r, iy, ix);
  const int32_t ty = (int32_t)iy + a.py, tx = (int32_t)ix + a.px;
  const T* conv = reinterpret_cast<const T*>(a.src) +
                  ((int64_t)image * a.n_cols + (int64_t)chan * (KW * KH)) * a.n_rows + (ty * a.out_w + tx);
  T acc = (T)0;
#pragma unroll
  for (int32_t ky = KH - 1; ky >= 0; --ky) {
    const bool row_ok = (uint32_t)(ty - ky) < (uint32_t)a.out_h;
#pragma unroll
    for (int32_t kx = KW - 1; kx >= 0; --kx) {
      const bool ok = row_ok && (uint32_t)(tx - kx) < (uint32_t)a.out_w;
      const int64_t at = (int64_t)(ky * KW + kx) * a.n_rows - ky * a.out_w - kx;
      const T cell = ok ? conv[at] : (T)0;
      acc = ok ? acc + cell : acc;
    }
  }
  reinterpret_cast<T*>(a.dest)[e] = acc;
}

// The same, four (two for double) consecutive input elements of one row per lane: for a tap
// their cells are consecutive, one (unaligned) 16-byte load, masked where a window does not
// exist.  A run of cells that would leave the tap's row of the matrix is read cell by cell.
template <class T, int KW, int KH>
__global__ void __launch_bounds__(kBlock) conv_roll_unit_stride_pieces_kernel(const ConvArgs a) {
  constexpr int VEC = 16 / sizeof(T);
  const uint32_t lane = blockIdx.x * kBlock + threadIdx.x;
  if (lane >= a.total) return;
  const uint32_t e0 = lane * VEC;
  uint32_t image, rest, chan, r, iy, ix;
  a.image_fd.divmod(e0, image, rest);
  a.in_plane_fd.divmod(rest, chan, r);
  a.in_w_fd.divmod(r, iy, ix);
  const int32_t ty = (int32_t)iy + a.py, tx = (int32_t)ix + a.px;
  const T* conv = reinterpret_cast<const T*>(a.src) + ((int64_t)image * a.n_cols + (int64_t)chan * (KW * KH)) * a.n_rows;
  struct alignas(16) Piece { T v[VEC]; } acc;
#pragma unroll
  for (int e = 0; e < VEC; ++e) acc.v[e] = (T)0;
#pragma unroll
  for (int32_t ky = KH - 1; ky >= 0; --ky) {
    const int32_t oy = ty - ky;
    if ((uint32_t)oy >= (uint32_t)a.out_h) continue;
#pragma unroll
    for (int32_t kx = KW - 1; kx >= 0; --kx) {
      const int32_t ox = tx - kx;                       // of the first element; element e: ox + e
      const int32_t at = oy * a.out_w + ox;             // inside the tap's row of cells
      const T* cells = conv + (int64_t)(ky * KW + kx) * a.n_rows;
      Piece got;
      if (at >= 0 && at + VEC <= (int32_t)a.n_rows) {
        __builtin_memcpy(&got, cells + at, 16);
      } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) got.v[e] = (uint32_t)(ox + e) < (uint32_t)a.out_w ? cells[at + e] : (T)0;
      }
#pragma unroll
      for (int e = 0; e < VEC; ++e)
        if ((uint32_t)(ox + e) < (uint32_t)a.out_w) acc.v[e] = acc.v[e] + got.v[e];
    }
  }
  *reinterpret_cast<Piece*>(reinterpret_cast<T*>(a.dest) + e0) = acc;
}

struct ConvShape {
  int64_t batch, in_h, in_w, out_h, out_w, n_rows, n_cols, in_image, out_image, conv_image;
};

int check_conv(const ct_conv_desc* d, int64_t batch_count, int64_t in_height, int64_t in_width, int64_t out_height,
               int64_t out_width, int64_t workspace_ecount, int dtype, ConvShape* sh) {
  CT_REQUIRE(d != nullptr, "convolution: null descriptor");
  CT_REQUIRE(dtype == CT_F32 || dtype == CT_F64, "convolution is only defined for float and double tensors");
  CT_REQUIRE(d->in_channels >= 1 && d->out_channels >= 1 && d->kernel_width >= 1 && d->kernel_height >= 1 &&
                 d->stride_x >= 1 && d->stride_y >= 1 && d->pad_x >= 0 && d->pad_y >= 0,
             "convolution: channels, kernel and stride must be positive and padding non-negative");
  CT_REQUIRE(d->kernel_width <= 1024 && d->kernel_height <= 1024 && d->stride_x <= 1024 && d->stride_y <= 1024 &&
                 d->pad_x <= 1024 && d->pad_y <= 1024 && d->in_channels <= 1 << 20 && d->out_channels <= 1 << 20,
             "convolution: descriptor exceeds the supported range");
  CT_REQUIRE(batch_count >= 0 && in_height >= 0 && in_width >= 0 && out_height >= 0 && out_width >= 0,
             "convolution: negative count");
  CT_REQUIRE(in_height <= 1 << 20 && in_width <= 1 << 20 && out_height <= 1 << 20 && out_width <= 1 << 20 &&
                 batch_count <= 1 << 30,
             "convolution: counts exceed the supported range");
  if (out_height > 0 && out_width > 0)
    CT_REQUIRE((out_width - 1) * d->stride_x - d->pad_x + d->kernel_width <= in_width + d->pad_x &&
                   (out_height - 1) * d->stride_y - d->pad_y + d->kernel_height <= in_height + d->pad_y,
               "convolution: a window reaches beyond the padded input (output dimensions must follow the floor rule)");
  ConvShape s{};
  s.batch = batch_count; s.in_h = in_height; s.in_w = in_width; s.out_h = out_height; s.out_w = out_width;
  s.n_rows = out_height * out_width;
  s.n_cols = (int64_t)d->kernel_width * d->kernel_height * d->in_channels;
  s.in_image = (int64_t)d->in_channels * in_height * in_width;
  s.out_image = (int64_t)d->out_channels * s.n_rows;
  const int64_t limit = (int64_t(1) << 31) - 1;
  CT_REQUIRE(s.n_rows <= limit && s.n_cols <= limit, "convolution: one image exceeds the supported range");
  s.conv_image = s.n_rows * s.n_cols;
  CT_REQUIRE(s.in_image <= limit && s.out_image <= limit && s.conv_image <= limit && s.n_cols <= limit,
             "convolution: one image exceeds the supported range");
  CT_REQUIRE(workspace_ecount >= batch_count * s.conv_image,
             "convolution: workspace of %lld elements, %lld needed", (long long)workspace_ecount,
             (long long)(batch_count * s.conv_image));
  *sh = s;
  return CT_OK;
}

ConvArgs conv_args(const ct_conv_desc& d, const ConvShape& sh) {
  ConvArgs a{};
  a.in_h = (int32_t)sh.in_h; a.in_w = (int32_t)sh.in_w; a.out_h = (int32_t)sh.out_h; a.out_w = (int32_t)sh.out_w;
  a.kw = d.kernel_width; a.kh = d.kernel_height; a.px = d.pad_x; a.py = d.pad_y; a.sx = d.stride_x; a.sy = d.stride_y;
  a.channels = (uint32_t)d.in_channels;
  a.n_cols = (uint32_t)sh.n_cols; a.n_rows = (uint32_t)sh.n_rows;
  a.in_plane = (uint32_t)(sh.in_h * sh.in_w);
  a.cols_fd = FastDiv((uint32_t)std::max<int64_t>(1, sh.n_cols));
  a.kk_fd = FastDiv((uint32_t)(d.kernel_width * d.kernel_height));
  a.kw_fd = FastDiv((uint32_t)d.kernel_width);
  a.out_w_fd = FastDiv((uint32_t)std::max<int64_t>(1, sh.out_w));
  a.rows_fd = FastDiv((uint32_t)std::max<int64_t>(1, sh.n_rows));
  a.in_w_fd = FastDiv((uint32_t)std::max<int64_t>(1, sh.in_w));
  a.in_plane_fd = FastDiv(std::max<uint32_t>(1u, a.in_plane));
  a.image_fd = FastDiv((uint32_t)std::max<int64_t>(1, sh.in_image));
  a.sx_fd = FastDiv((uint32_t)d.stride_x);
  a.sy_fd = FastDiv((uint32_t)d.stride_y);
  return a;
}

// Images per launch so that a launch indexes fewer than 2^31 cells.
int64_t images_per_launch(int64_t per_image) {
  return std::max<int64_t>(1, ((int64_t(1) << 31) - 1) / std::max<int64_t>(1, per_image));
}

template <class T>
void unroll(hipStream_t s, const T* input, T* workspace, const ct_conv_desc& d, const ConvShape& sh) {
  if (sh.batch * sh.conv_image == 0) return;
  ConvArgs a = conv_args(d, sh);
  constexpr int VEC = 16 / sizeof(T);
  const bool pieces = sh.n_rows % VEC == 0 && reinterpret_cast<uintptr_t>(workspace) % 16 == 0;
  const int64_t step = images_per_launch(sh.conv_image);
  for (int64_t b0 = 0; b0 < sh.batch; b0 += step) {
    const int64_t nb = std::min(step, sh.batch - b0);
    a.src = input + b0 * sh.in_image;
    a.dest = workspace + b0 * sh.conv_image;
    const int64_t cells = nb * sh.conv_image;
    a.total = (uint32_t)(pieces ? cells / VEC : cells);
    const dim3 grid((a.total + kBlock - 1) / kBlock);
    a.grouped_blocks = xcd_grouped_blocks(grid.x);
    if (pieces && d.stride_x == 1 && sh.out_w % VEC == 0)
      hipLaunchKernelGGL((conv_unroll_unit_stride_kernel<T>), grid, dim3(kBlock), 0, s, a);
    else if (pieces) hipLaunchKernelGGL((conv_unroll_kernel<T, VEC>), grid, dim3(kBlock), 0, s, a);
    else hipLaunchKernelGGL((conv_unroll_kernel<T, 1>), grid, dim3(kBlock), 0, s, a);
  }
}

template <class T>
void roll_back(hipStream_t s, const T* workspace, T* input_gradient, const ct_conv_desc& d, const ConvShape& sh) {
  if (sh.batch * sh.in_image == 0) return;
  ConvArgs a = conv_args(d, sh);
  const int64_t step = std::min(images_per_launch(sh.in_image), images_per_launch(sh.conv_image));
  for (int64_t b0 = 0; b0 < sh.batch; b0 += step) {
    const int64_t nb = std::min(step, sh.batch - b0);
    a.src = workspace + b0 * sh.conv_image;
    a.dest = input_gradient + b0 * sh.in_image;
    a.total = (uint32_t)(nb * sh.in_image);
    const dim3 grid((a.total + kBlock - 1) / kBlock);
    const bool unit_stride = d.stride_x == 1 && d.stride_y == 1;
    constexpr int VEC = 16 / sizeof(T);
    const bool pieces = unit_stride && sh.in_w % VEC == 0 && reinterpret_cast<uintptr_t>(input_gradient) % 16 == 0 &&
                        d.kernel_width == d.kernel_height &&
                        (d.kernel_width == 1 || d.kernel_width == 3 || d.kernel_width == 5);
    if (pieces) {
      ConvArgs p = a;
      p.total = a.total / VEC;   // whole images: in_w, hence in_image, is a multiple of VEC
      const dim3 pgrid((p.total + kBlock - 1) / kBlock);
      if (d.kernel_width == 3)
        hipLaunchKernelGGL((conv_roll_unit_stride_pieces_kernel<T, 3, 3>), pgrid, dim3(kBlock), 0, s, p);
      else if (d.kernel_width == 5)
        hipLaunchKernelGGL((conv_roll_unit_stride_pieces_kernel<T, 5, 5>), pgrid, dim3(kBlock), 0, s, p);
      else
        hipLaunchKernelGGL((conv_roll_unit_stride_pieces_kernel<T, 1, 1>), pgrid, dim3(kBlock), 0, s, p);
    } else if (unit_stride && d.kernel_width == 3 && d.kernel_height == 3)
      hipLaunchKernelGGL((conv_roll_unit_stride_kernel<T, 3, 3>), grid, dim3(kBlock), 0, s, a);
    else if (unit_stride && d.kernel_width == 5 && d.kernel_height == 5)
      hipLaunchKernelGGL((conv_roll_unit_stride_kernel<T, 5, 5>), grid, dim3(kBlock), 0, s, a);
    else if (unit_stride && d.kernel_width == 1 && d.kernel_height == 1)
      hipLaunchKernelGGL((conv_roll_unit_stride_kernel<T, 1, 1>), grid, dim3(kBlock), 0, s, a);
    else
      hipLaunchKernelGGL((conv_roll_kernel<T>), grid, dim3(kBlock), 0, s, a);
  }
}

template <class T>
int forward_t(void* stream, T* output, double output_alpha, const T* input, const T* weights, T* workspace,
              const ct_conv_desc& d, const ConvShape& sh, int dtype) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  unroll(s, input, workspace, d, sh);
  if (int rc = after_launch(s)) return rc;
  // output[b] [out_channels, n_rows] = weights [out_channels, n_cols] x unrolled[b] [n_cols, n_rows]
  if (int rc = gemm_strided_batched(stream, output, sh.n_rows, sh.out_image, 0, 0, 1.0, weights, d.out_channels,
                                    sh.n_cols, sh.n_cols, 0, workspace, sh.n_rows, sh.n_rows, sh.conv_image,
                                    output_alpha, sh.batch, dtype))
    return rc;
  note_kernel("conv_unroll+gemm");
  return CT_OK;
}

// weight_gradient = T(alpha * weight_gradient + sum over the images of partial[image]), in double
template <class T>
__global__ void __launch_bounds__(kBlock) conv_sum_partials_kernel(T* weight_gradient, const T* partials, uint32_t n,
                                                                    uint32_t images, double alpha) {
  const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
  if (i >= n) return;
  double acc = alpha == 0.0 ? 0.0 : alpha * (double)weight_gradient[i];
  for (uint32_t b = 0; b < images; ++b) acc += (double)partials[(int64_t)b * n + i];
  weight_gradient[i] = (T)acc;
}

template <class T>
int backward_weights_t(void* stream, T* weight_gradient, double alpha, const T* output_gradient, T* workspace,
                       const ct_conv_desc& d, const ConvShape& sh, int dtype) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t n = (int64_t)d.out_channels * sh.n_cols;
  CT_REQUIRE(n <= (int64_t(1) << 31) - 1, "convolution: the weight matrix exceeds the supported range");
  // A product of few outputs over very many positions (a first layer: 64 x 27 outputs, 50176
  // positions) would occupy one workgroup per image: the positions are cut into pieces of about
  // kPositionsPerPiece, every piece a product of its own, and the sum takes the pieces too.
  constexpr int64_t kPositionsPerPiece = 4096;
  const int64_t pieces = std::max<int64_t>(1, std::min<int64_t>(64, sh.n_rows / kPositionsPerPiece));
  const int64_t piece_len = (sh.n_rows + pieces - 1) / pieces;
  // images per pass: partial products of at most 256 MiB
  const int64_t per_pass =
      std::max<int64_t>(1, std::min<int64_t>(sh.batch, (int64_t(256) << 20) / (pieces * n * (int64_t)sizeof(T))));
  void* scratch = nullptr;
  if (int rc = stream_scratch(s, (size_t)(per_pass * pieces * n) * sizeof(T), &scratch)) return rc;
  const T al = (T)alpha;
  for (int64_t b0 = 0; b0 < sh.batch; b0 += per_pass) {
    const int64_t nb = std::min(per_pass, sh.batch - b0);
    int64_t used = 0;
    for (int64_t p = 0; p < pieces; ++p) {
      const int64_t r0 = p * piece_len, len = std::min(piece_len, sh.n_rows - r0);
      if (len <= 0) break;
      // partial[p][b] [out_channels, n_cols] = output_gradient[b][:, r0 : r0 + len] x unrolled[b][:, r0 : r0 + len]^T
      if (int rc = gemm_strided_batched(stream, reinterpret_cast<T*>(scratch) + used * nb * n, sh.n_cols, n, 0, 1, 1.0,
                                        output_gradient + b0 * sh.out_image + r0, d.out_channels, len, sh.n_rows,
                                        sh.out_image, workspace + b0 * sh.conv_image + r0, sh.n_cols, sh.n_rows,
                                        sh.conv_image, 0.0, nb, dtype))
        return rc;
      ++used;
    }
    hipLaunchKernelGGL((conv_sum_partials_kernel<T>), dim3((uint32_t)((n + kBlock - 1) / kBlock)), dim3(kBlock), 0, s,
                       weight_gradient, reinterpret_cast<const T*>(scratch), (uint32_t)n, (uint32_t)(nb * used),
                       b0 == 0 ? (double)al : 1.0);
  }
  note_kernel("gemm+conv_sum_partials");
  return after_launch(s);
}

template <class T>
int backward_data_t(void* stream, T* input_gradient, const T* output_gradient, const T* weights, T* workspace,
                    const ct_conv_desc& d, const ConvShape& sh, int dtype) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  // unrolled[b] [n_cols, n_rows] = weights^T [n_cols, out_channels] x output_gradient[b] [out_channels, n_rows]
  if (sh.conv_image > 0)
    if (int rc = gemm_strided_batched(stream, workspace, sh.n_rows, sh.conv_image, 1, 0, 1.0, weights, sh.n_cols,
                                      d.out_channels, sh.n_cols, 0, output_gradient, sh.n_rows, sh.n_rows,
                                      sh.out_image, 0.0, sh.batch, dtype))
      return rc;
  roll_back(s, workspace, input_gradient, d, sh);
  note_kernel("gemm+conv_roll");
  return after_launch(s);
}

}  // namespace

extern "C" {

int ct_convolution_forward(void* stream, void* output, double output_alpha, const void* input, const void* weights,
                           void* workspace, int64_t workspace_ecount, const ct_conv_desc* desc, int64_t batch_count,
                           int64_t in_height, int64_t in_width, int64_t out_height, int64_t out_width, int dtype) {
  ConvShape sh;
  if (int rc = check_conv(desc, batch_count, in_height, in_width, out_height, out_width, workspace_ecount, dtype, &sh))
    return rc;
  if (sh.batch * sh.out_image == 0) return CT_OK;
  CT_REQUIRE(output && weights && workspace && (input || sh.in_image == 0), "convolution-forward!: null buffer");
  if (dtype == CT_F32)
    return forward_t<float>(stream, (float*)output, output_alpha, (const float*)input, (const float*)weights,
                            (float*)workspace, *desc, sh, dtype);
  return forward_t<double>(stream, (double*)output, output_alpha, (const double*)input, (const double*)weights,
                           (double*)workspace, *desc, sh, dtype);
}

int ct_convolution_backward_weights(void* stream, void* weight_gradient, double weight_gradient_alpha,
                                    const void* output_gradient, const void* /*input*/, void* workspace,
                                    int64_t workspace_ecount, const ct_conv_desc* desc, int64_t batch_count,
                                    int64_t in_height, int64_t in_width, int64_t out_height, int64_t out_width,
                                    int dtype) {
  ConvShape sh;
  if (int rc = check_conv(desc, batch_count, in_height, in_width, out_height, out_width, workspace_ecount, dtype, &sh))
    return rc;
  if (sh.batch * sh.conv_image == 0) return CT_OK;
  CT_REQUIRE(weight_gradient && output_gradient && workspace, "convolution-backward-weights!: null buffer");
  if (dtype == CT_F32)
    return backward_weights_t<float>(stream, (float*)weight_gradient, weight_gradient_alpha,
                                     (const float*)output_gradient, (float*)workspace, *desc, sh, dtype);
  return backward_weights_t<double>(stream, (double*)weight_gradient, weight_gradient_alpha,
                                    (const double*)output_gradient, (double*)workspace, *desc, sh, dtype);
}

int ct_convolution_backward_data(void* stream, void* input_gradient, double /*input_gradient_alpha*/,
                                 const void* output_gradient, const void* weights, void* workspace,
                                 int64_t workspace_ecount, const ct_conv_desc* desc, int64_t batch_count,
                                 int64_t in_height, int64_t in_width, int64_t out_height, int64_t out_width,
                                 int dtype) {
  ConvShape sh;
  if (int rc = check_conv(desc, batch_count, in_height, in_width, out_height, out_width, workspace_ecount, dtype, &sh))
    return rc;
  if (sh.batch * sh.in_image == 0) return CT_OK;
  CT_REQUIRE(input_gradient && (sh.conv_image == 0 || (output_gradient && weights && workspace)),
             "convolution-backward-data!: null buffer");
  if (dtype == CT_F32)
    return backward_data_t<float>(stream, (float*)input_gradient, (const float*)output_gradient,
                                  (const float*)weights, (float*)workspace, *desc, sh, dtype);
  return backward_data_t<double>(stream, (double*)input_gradient, (const double*)output_gradient,
                                 (const double*)weights, (double*)workspace, *desc, sh, dtype);
}

}  // extern "C"
