// ops_accum_stream.hip -- binary-accum! into a broadcast destination, any operation and any
// multipliers, at the rate the memory system and the serial chain allow
// (src/cortex/compute/cpu/tensor_math.clj:386-420; the reference's CUDA backend reaches the same
// destinations through compare-and-swap loops, resources/tensor_binary_accum.cu).
//
//   dest[Ad(e)] = dest[Ad(e)]*dest_alpha op y[Ay(e)]*y_alpha     for e = 0 .. n-1
//
// Every destination element is the end of a chain: its updates apply one after the other, in
// increasing e, and each step rounds to the tensor's datatype, so a chain cannot be cut or
// reordered without changing bits.  The chains are independent of one another.  With one lane
// per chain fetching its own updates (accum_owner_kernel) a destination of 4096 elements keeps 64
// waves busy on a chip that holds thousands, and each of them waits for its own loads.
//
// Here a block of sixteen waves owns a strip of neighbouring chains.  All of its waves stream the
// strip's updates into LDS, tile after tile, with 128-bit non-temporal loads that are issued
// kDepth tiles ahead of their use, so the block has 128 KiB in flight whatever the chains are
// doing; the first wave walks each tile in LDS, one lane per chain, in increasing e.  A tile is
// written to one of two LDS buffers while the previous one is walked from the other; one barrier
// per tile hands them over.  What a chain computes per step is what the per-element functor
// computes, so the result is bit-identical to the serial loop.
//
// Two arrangements of y cover the callers:
//   chains unit-stride    dest [k] <- y [b, k] (sum / product / ... of the rows into a vector):
//                         a tile is `rows x G chains`; a row of it is G neighbouring elements
//   steps unit-stride     dest [b, 1] <- y [b, k], dest [C, 1, 1] <- y [N, C, H, W]: a chain walks
//                         contiguous runs of y; a tile is `G chains x S steps`, each chain's
//                         share one contiguous run, kept in LDS chain by chain
// Anything else (rows off the 16-byte grid, several irregular broadcast axes) stays with
// accum_owner_kernel.
//
// The time of a call is bounded below by the longest chain: n_red dependent steps.  For float
// tensors with multipliers of +-1 a step of + - * is one instruction; with other multipliers, and
// for double arithmetic on float tensors, it is four (widen, multiply, operate, round).
#include <algorithm>

#include "elementwise.h"
#include "functors.h"
#include "ops.h"

using namespace cthip;

namespace {

constexpr int kStreamWaves = 16;
constexpr int kStreamBlock = kStreamWaves * 64;
constexpr int kDepth = 8;  // tiles a lane has in flight

struct StreamArgs {
  void* dest;
  const void* y;
  int64_t n_red;         // steps of a chain
  // chains unit-stride: y stride of one step.  steps unit-stride: y stride between chains
  int64_t pitch;
  uint32_t u;            // chains along the strip axis
  int64_t d_ustride;     // destination stride of that axis
  // steps unit-stride only: steps [0, n_inner) of a run are contiguous; n_red = n_inner * n_outer
  int64_t n_inner, outer_stride;
  uint32_t tiles_per_run;
  uint32_t n_strips;
  FastDiv strips_fd;
  int32_t n_rest;        // other kept axes, fastest first
  FastDiv rsize[CT_MAX_DIMS];
  int64_t rd_stride[CT_MAX_DIMS], ry_stride[CT_MAX_DIMS];
  int32_t reverse;
};

// The float operations whose correctly rounded single-precision result equals the double
// operation rounded once (53 >= 2 * 24 + 2), and the comparisons, which see the same values.
template <int OP> __device__ __forceinline__ float plain_apply(float x, float y) {
  if constexpr (OP == CT_BOP_ADD) return x + y;
  else if constexpr (OP == CT_BOP_SUB) return x - y;
  else if constexpr (OP == CT_BOP_MUL) return x * y;
  else if constexpr (OP == CT_BOP_DIV) return x / y;
  else if constexpr (OP == CT_BOP_MAX) return x > y ? x : y;
  else if constexpr (OP == CT_BOP_MIN) return x > y ? y : x;
  else if constexpr (OP == CT_BOP_EQ) return x == y ? 1.0f : 0.0f;
  else if constexpr (OP == CT_BOP_GT) return x > y ? 1.0f : 0.0f;
  else if constexpr (OP == CT_BOP_GE) return x >= y ? 1.0f : 0.0f;
  else if constexpr (OP == CT_BOP_LT) return x < y ? 1.0f : 0.0f;
  else return x <= y ? 1.0f : 0.0f;
}

// One step of a chain.  PLAIN: float tensors, dest_alpha 1, y_alpha +-1.  The y side of a step
// does not depend on the chain and is prepared ahead of it.
template <class T, int OP, bool PLAIN> struct ChainStep {
  using A = typename ew_acc_of<T>::type;
  using Y = typename std::conditional<PLAIN, T, A>::type;
  A da, ya;
  uint32_t* div0;
  __device__ __forceinline__ Y prepare(T y) const {
    if constexpr (PLAIN) return ya < 0 ? -y : y;
    else return w_mul((A)y, in_range_of<T>(ya));
  }
  template <bool REV> __device__ __forceinline__ T step(T acc, Y yv) const {
    if constexpr (PLAIN) {
      return REV ? plain_apply<OP>(yv, acc) : plain_apply<OP>(acc, yv);
    } else {
      const A av = w_mul((A)acc, in_range_of<T>(da));
      return REV ? binary_value<T, OP, A>(yv, av, div0) : binary_value<T, OP, A>(av, yv, div0);
    }
  }
};

// Walks `count` consecutive updates of one chain, `stride` elements apart in LDS.
template <class T, int OP, bool PLAIN, bool REV>
__device__ __forceinline__ T walk(const ChainStep<T, OP, PLAIN>& f, T acc, const T* p, int stride, int count) {
  constexpr int UN = 8;
  int s = 0;
  for (; s + UN <= count; s += UN) {
    typename ChainStep<T, OP, PLAIN>::Y yv[UN];
#pragma unroll
    for (int j = 0; j < UN; ++j) yv[j] = f.prepare(p[(s + j) * stride]);
#pragma unroll
    for (int j = 0; j < UN; ++j) acc = f.template step<REV>(acc, yv[j]);
  }
  for (; s < count; ++s) acc = f.template step<REV>(acc, f.prepare(p[s * stride]));
  return acc;
}

// BY_STEP false: chains unit-stride in y.  true: steps unit-stride in y.
template <class T, int OP, bool PLAIN, bool BY_STEP>
__global__ void __launch_bounds__(kStreamBlock) accum_stream_kernel(const StreamArgs a, const ChainStep<T, OP, PLAIN> f) {
  constexpr int VEC = 16 / (int)sizeof(T);
  using V = Vec<T, VEC>;
  // chains unit-stride: G chains side by side are one row of a tile, 128 bytes of y (64 chains
  // for bytes); a wave-load covers 64 / LPR rows.  steps unit-stride: a wave-load covers CPW
  // chains with a run of 64 / CPW vectors each, and a tile holds G = kStreamWaves * CPW chains.
  constexpr int G = BY_STEP ? 32 : (128 / (int)sizeof(T) < 64 ? 128 / (int)sizeof(T) : 64);
  constexpr int LPR = BY_STEP ? 64 / (G / kStreamWaves) : G / VEC;  // lanes per row (per chain's run)
  constexpr int RPW = 64 / LPR;                                     // rows (chains) per wave-load
  constexpr int RPR = kStreamWaves * RPW;                           // rows per tile (= G when BY_STEP)
  constexpr int RUN = LPR * VEC;                                    // BY_STEP: steps of a chain per tile
  constexpr int PITCH_V = LPR + 1;                                  // BY_STEP: vectors per chain in LDS (one of padding)
  constexpr int TILE_V = BY_STEP ? G * PITCH_V : kStreamBlock;
  __shared__ V lds[2][TILE_V];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  uint32_t rest, strip;
  a.strips_fd.divmod(blockIdx.x, rest, strip);
  int64_t dbase = 0, ybase = 0;
  for (int d = 0; d < a.n_rest; ++d) {
    uint32_t q, r;
    a.rsize[d].divmod(rest, q, r);
    rest = q;
    dbase += (int64_t)r * a.rd_stride[d];
    ybase += (int64_t)r * a.ry_stride[d];
  }
  const T* yp = reinterpret_cast<const T*>(a.y) + ybase;
  const int my_row = wave * RPW + lane / LPR, my_vcol = lane % LPR;
  uint32_t n_tiles;
  bool col_live;
  int64_t my_off;  // this lane's offset inside a tile's region of y
  if constexpr (BY_STEP) {
    n_tiles = a.tiles_per_run * (uint32_t)(a.n_red / a.n_inner);
    const uint32_t chain = strip * G + my_row;
    col_live = chain < a.u;
    my_off = (int64_t)chain * a.pitch + my_vcol * VEC;
  } else {
    n_tiles = (uint32_t)((a.n_red + RPR - 1) / RPR);
    const uint32_t col = strip * G + my_vcol * VEC;
    col_live = col < a.u;
    my_off = (int64_t)my_row * a.pitch + col;
  }
  // where tile t starts in y, and whether this lane's vector of it exists
  auto tile_load = [&](uint32_t t, V& x) {
    if constexpr (BY_STEP) {
      const uint32_t o = t / a.tiles_per_run, i = t - o * a.tiles_per_run;
      const int64_t s0 = (int64_t)i * RUN;
      if (col_live && s0 + my_vcol * VEC < a.n_inner) x = nt_load(reinterpret_cast<const V*>(yp + o * a.outer_stride + s0 + my_off));
    } else {
      const int64_t r0 = (int64_t)t * RPR;
      if (col_live && r0 + my_row < a.n_red) x = nt_load(reinterpret_cast<const V*>(yp + r0 * a.pitch + my_off));
    }
  };
  V x[kDepth];
#pragma unroll
  for (int j = 0; j < kDepth; ++j)
    if ((uint32_t)j < n_tiles) tile_load(j, x[j]);

  // the first wave's lanes own the chains
  const uint32_t my_chain = strip * G + lane;
  const bool chain_live = wave == 0 && lane < G && my_chain < a.u;
  T* dp = reinterpret_cast<T*>(a.dest) + dbase + (int64_t)my_chain * a.d_ustride;
  T acc = chain_live ? *dp : (T)0;

  for (uint32_t t = 0; t < n_tiles; ++t) {
    // hand this tile's vector to LDS and put the load of tile t + kDepth in its place; the
    // register that is copied is the oldest load, the only one this wave has to wait for
    V cur;
    const bool more = t + kDepth < n_tiles;
    switch (t % kDepth) {
#define CT_STAGE(J) case J: cur = x[J]; if (more) tile_load(t + kDepth, x[J]); break;
      CT_STAGE(0) CT_STAGE(1) CT_STAGE(2) CT_STAGE(3) CT_STAGE(4) CT_STAGE(5) CT_STAGE(6) CT_STAGE(7)
#undef CT_STAGE
    }
    static_assert(kDepth == 8, "the stages above are written out for a depth of 8");
    V* buf = lds[t & 1];
    if constexpr (BY_STEP) buf[my_row * PITCH_V + my_vcol] = cur;
    else buf[threadIdx.x] = cur;
    __syncthreads();
    if (chain_live) {
      const T* tile = reinterpret_cast<const T*>(buf);
      int count;
      const T* p;
      int stride;
      if constexpr (BY_STEP) {
        const uint32_t i = t % a.tiles_per_run;
        const int64_t left = a.n_inner - (int64_t)i * RUN;
        count = (int)(left < RUN ? left : RUN);
        p = tile + lane * (PITCH_V * VEC);
        stride = 1;
      } else {
        const int64_t left = a.n_red - (int64_t)t * RPR;
        count = (int)(left < RPR ? left : RPR);
        p = tile + lane;
        stride = G;
      }
      acc = a.reverse ? walk<T, OP, PLAIN, true>(f, acc, p, stride, count) : walk<T, OP, PLAIN, false>(f, acc, p, stride, count);
    }
  }
  if (chain_live) *dp = acc;
}

template <class T, int OP, bool PLAIN>
int stream_launch(hipStream_t s, const AccumStreamCall& c, const StreamArgs& a, uint32_t grid) {
  using A = typename ew_acc_of<T>::type;
  ChainStep<T, OP, PLAIN> f;
  f.da = (A)jvm_cast<T>(c.dest_alpha);
  f.ya = (A)jvm_cast<T>(c.y_alpha);
  f.div0 = c.div0;
  if (c.steps_unit_stride) {
    note_kernel(PLAIN ? "accum_stream_steps_plain" : "accum_stream_steps");
    hipLaunchKernelGGL((accum_stream_kernel<T, OP, PLAIN, true>), dim3(grid), dim3(kStreamBlock), 0, s, a, f);
  } else {
    note_kernel(PLAIN ? "accum_stream_plain" : "accum_stream");
    hipLaunchKernelGGL((accum_stream_kernel<T, OP, PLAIN, false>), dim3(grid), dim3(kStreamBlock), 0, s, a, f);
  }
  return after_launch(s);
}

template <class T, int OP>
int stream_run(hipStream_t s, const AccumStreamCall& c) {
  constexpr int VEC = 16 / (int)sizeof(T);
  StreamArgs a;
  std::memset(&a, 0, sizeof(a));
  a.dest = c.dest;
  a.y = c.y;
  a.n_red = c.n_red;
  a.pitch = c.pitch;
  a.u = (uint32_t)c.u;
  a.d_ustride = c.d_ustride;
  a.n_inner = c.n_inner;
  a.outer_stride = c.outer_stride;
  a.reverse = c.reverse ? 1 : 0;
  int g;
  if (c.steps_unit_stride) {
    g = 32;
    const int run = (64 / (g / kStreamWaves)) * VEC;
    a.tiles_per_run = (uint32_t)((c.n_inner + run - 1) / run);
  } else {
    g = std::min(128 / (int)sizeof(T), 64);
  }
  a.n_strips = (uint32_t)((c.u + g - 1) / g);
  a.strips_fd = FastDiv(a.n_strips);
  a.n_rest = c.n_rest;
  int64_t grid = a.n_strips;
  for (int d = 0; d < c.n_rest; ++d) {
    a.rsize[d] = FastDiv((uint32_t)c.rsize[d]);
    a.rd_stride[d] = c.rd_stride[d];
    a.ry_stride[d] = c.ry_stride[d];
    grid *= c.rsize[d];
  }
  CT_REQUIRE(grid < (int64_t(1) << 31), "binary-accum!: too many destination strips");
  if constexpr (std::is_same<T, float>::value && binary_plain_op(OP)) {
    const float da = jvm_cast<float>(c.dest_alpha), ya = jvm_cast<float>(c.y_alpha);
    if (da == 1.0f && (ya == 1.0f || ya == -1.0f)) return stream_launch<T, OP, true>(s, c, a, (uint32_t)grid);
  }
  return stream_launch<T, OP, false>(s, c, a, (uint32_t)grid);
}

template <class T>
int stream_dispatch(hipStream_t s, const AccumStreamCall& c) {
#define CT_CASE(OP) case OP: return stream_run<T, OP>(s, c)
  switch (c.op) {
    CT_CASE(CT_BOP_ADD); CT_CASE(CT_BOP_SUB); CT_CASE(CT_BOP_MUL); CT_CASE(CT_BOP_DIV);
    CT_CASE(CT_BOP_MIN); CT_CASE(CT_BOP_MAX); CT_CASE(CT_BOP_BIT_AND); CT_CASE(CT_BOP_BIT_XOR);
    CT_CASE(CT_BOP_EQ); CT_CASE(CT_BOP_GT); CT_CASE(CT_BOP_GE); CT_CASE(CT_BOP_LT); CT_CASE(CT_BOP_LE);
    default: return set_error(CT_ERR_INVALID, "unknown binary operation %d", c.op);
  }
#undef CT_CASE
}

}  // namespace

int cthip::accum_stream(hipStream_t s, const AccumStreamCall& c) {
  CT_DISPATCH_DTYPE(c.dtype, return stream_dispatch<T>(s, c));
  return CT_OK;
}
