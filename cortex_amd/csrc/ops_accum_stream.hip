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
// Here a block of sixteen waves owns a strip of neighbouring chains.  Fifteen of its waves stream
// the strip's updates into LDS, tile after tile, with 128-bit non-temporal loads that are issued
// kDepth tiles ahead of their use, so the block has 120 KiB in flight whatever the chains are
// doing; the first wave walks each tile in LDS, one lane per chain, in increasing e.  A tile is
// written to one of two LDS buffers while the previous one is walked from the other; one barrier
// per tile hands them over (every wave passes the same number of barriers).  What a chain computes per step is what the per-element functor
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
// The time of a call is bounded below by the longest chain: n_red dependent steps of about ten
// clocks per dependent instruction.  For float tensors with multipliers of +-1 a step of + - * is
// one instruction; with other multipliers it is four (widen, multiply, operate, round), three for
// + and - (the multiplication and the addition fuse exactly).
#include <algorithm>

#include "elementwise.h"
#include "functors.h"
#include "ops.h"

using namespace cthip;

namespace {

constexpr int kLoaderWaves = 15;                       // and one wave that walks the chains
constexpr int kStreamBlock = (kLoaderWaves + 1) * 64;
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

// One step of a chain.  PLAIN: float tensors, dest_alpha 1, y_alpha +1 (NEG false) or -1 (NEG true:
// the negation rides on the instruction's source modifier).  Otherwise the y side of a step, which
// does not depend on the chain, is prepared ahead of it.
template <class T, int OP, bool PLAIN, bool NEG> struct ChainStep {
  using A = typename ew_acc_of<T>::type;
  using Y = typename std::conditional<PLAIN, T, A>::type;
  A da, ya;
  uint32_t* div0;
  __device__ __forceinline__ Y prepare(T y) const {
    if constexpr (PLAIN) return NEG ? -y : y;
    else return w_mul((A)y, in_range_of<T>(ya));
  }
  template <bool REV> __device__ __forceinline__ T step(T acc, Y yv) const {
    if constexpr (PLAIN) {
      return REV ? plain_apply<OP>(yv, acc) : plain_apply<OP>(acc, yv);
    } else if constexpr (std::is_same<T, float>::value && (OP == CT_BOP_ADD || OP == CT_BOP_SUB)) {
      // acc * da is exact in double (24 x 24 bits), so one fused multiply-add rounds the same sum
      // once, as the separate multiplication and addition do: three dependent instructions, not four
      const double yd = OP == CT_BOP_ADD ? yv : (REV ? yv : -yv);
      const double ad = (OP == CT_BOP_SUB && REV) ? -da : da;
      return (float)__builtin_fma((double)acc, ad, yd);
    } else {
      const A av = w_mul((A)acc, in_range_of<T>(da));
      return REV ? binary_value<T, OP, A>(yv, av, div0) : binary_value<T, OP, A>(av, yv, div0);
    }
  }
};

// Walks `count` consecutive updates of one chain, which lie side by side in LDS from the 16-byte
// aligned `p` on.  A full tile (count == RUN, a whole number of groups of W vectors) is walked with
// two register sets that take turns: while one group is applied the next is on its way from LDS,
// and no register is ever copied.  The last tile of a run may be shorter and is walked plainly.
template <class F, class T, int W, int RUN, bool REV>
__device__ __forceinline__ T walk(const F& f, T acc, const T* p, int count) {
  constexpr int VEC = 16 / (int)sizeof(T);
  using V = Vec<T, VEC>;
  constexpr int GROUP = W * VEC, NG = RUN / GROUP;
  const V* vp = reinterpret_cast<const V*>(p);
  auto load = [&](V (&v)[W], int g) {
#pragma unroll
    for (int j = 0; j < W; ++j) v[j] = vp[g * W + j];
  };
  auto apply = [&](const V (&v)[W]) {
    typename F::Y yv[GROUP];
#pragma unroll
    for (int j = 0; j < W; ++j)
#pragma unroll
      for (int e = 0; e < VEC; ++e) yv[j * VEC + e] = f.prepare(v[j].v[e]);
#pragma unroll
    for (int i = 0; i < GROUP; ++i) acc = f.template step<REV>(acc, yv[i]);
  };
  V a[W], b[W];
  if (count == RUN) {
    load(a, 0);
    for (int g = 0; g + 2 <= NG; g += 2) {
      load(b, g + 1);
      apply(a);
      load(a, g + 2 < NG ? g + 2 : NG - 1);  // the last round reads a group again rather than branch
      apply(b);
    }
    if constexpr (NG % 2 == 1) apply(a);
    return acc;
  }
  const int groups = count / GROUP;
  for (int g = 0; g < groups; ++g) {
    load(a, g);
    apply(a);
  }
  for (int s = groups * GROUP; s < count; ++s) acc = f.template step<REV>(acc, f.prepare(p[s]));
  return acc;
}

// Geometry of a tile, shared by the kernel and its launcher.  BY_STEP false: chains unit-stride in
// y; G chains side by side are one row of a tile, 128 bytes of y (64 chains for bytes), and a
// wave-load covers 64 / LPR rows.  BY_STEP true: steps unit-stride in y; a wave-load covers two
// chains with a run of 32 vectors each.  In LDS a tile lies chain by chain, each chain's steps side
// by side and one vector of padding behind them, whichever way it lies in y: the walking lane reads
// its steps as 16-byte vectors.
template <class T, bool BY_STEP> struct StreamTile {
  static constexpr int VEC = 16 / (int)sizeof(T);
  static constexpr int G = BY_STEP ? 2 * kLoaderWaves : (128 / (int)sizeof(T) < 64 ? 128 / (int)sizeof(T) : 64);  // chains
  static constexpr int LPR = BY_STEP ? 32 : G / VEC;   // lanes per row of y (per chain's run)
  static constexpr int RPW = 64 / LPR;                 // rows (chains) per wave-load
  static constexpr int RUN = BY_STEP ? LPR * VEC : kLoaderWaves * RPW;  // steps of a chain per tile
  static constexpr int PITCH = RUN + VEC;              // elements per chain in LDS
  static constexpr int TILE_V = G * PITCH / VEC;
  static constexpr int WALK_VECS = (RUN / VEC) % 5 == 0 ? 5 : 4;  // vectors per group of the walk
  static_assert(RUN % (VEC * WALK_VECS) == 0, "a chain's share of a tile is a whole number of walk groups");
};

template <class T, int OP, bool PLAIN, bool NEG, bool BY_STEP>
__global__ void __launch_bounds__(kStreamBlock) accum_stream_kernel(const StreamArgs a, const ChainStep<T, OP, PLAIN, NEG> f) {
  using TL = StreamTile<T, BY_STEP>;
  constexpr int VEC = TL::VEC, G = TL::G, LPR = TL::LPR, RPW = TL::RPW, RUN = TL::RUN, PITCH = TL::PITCH;
  using V = Vec<T, VEC>;
  __shared__ V lds[2][TL::TILE_V];
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
  uint32_t n_tiles;
  if constexpr (BY_STEP) n_tiles = a.tiles_per_run * (uint32_t)(a.n_red / a.n_inner);
  else n_tiles = (uint32_t)((a.n_red + RUN - 1) / RUN);

  if (wave == 0) {
    // the walking wave: one lane per chain; it meets the loaders at one barrier per tile
    const uint32_t my_chain = strip * G + lane;
    const bool chain_live = lane < G && my_chain < a.u;
    T* dp = reinterpret_cast<T*>(a.dest) + dbase + (int64_t)my_chain * a.d_ustride;
    T acc = chain_live ? *dp : (T)0;
    for (uint32_t t = 0; t < n_tiles; ++t) {
      __syncthreads();
      if (chain_live) {
        int64_t left;
        if constexpr (BY_STEP) left = a.n_inner - (int64_t)(t % a.tiles_per_run) * RUN;
        else left = a.n_red - (int64_t)t * RUN;
        const int count = (int)(left < RUN ? left : RUN);
        const T* p = reinterpret_cast<const T*>(lds[t & 1]) + lane * PITCH;
        using F = ChainStep<T, OP, PLAIN, NEG>;
        acc = a.reverse ? walk<F, T, TL::WALK_VECS, RUN, true>(f, acc, p, count)
                        : walk<F, T, TL::WALK_VECS, RUN, false>(f, acc, p, count);
      }
    }
    if (chain_live) *dp = acc;
    return;
  }

  // the loading waves.  Every lane issues exactly one load per tile, whether its vector exists or
  // not (one that does not is fetched from a place that does, and never looked at): with a fixed
  // number of loads between the issue of a vector and its use the wave waits for that vector alone
  // and keeps the kDepth - 1 younger ones in flight.
  const T* yp = reinterpret_cast<const T*>(a.y) + ybase;
  const int my_row = (wave - 1) * RPW + lane / LPR, my_vcol = lane % LPR;
  int64_t my_off;  // this lane's offset inside a tile's region of y
  if constexpr (BY_STEP) {
    uint32_t chain = strip * G + my_row;
    if (chain >= a.u) chain = a.u - 1;
    my_off = (int64_t)chain * a.pitch;
  } else {
    uint32_t col = strip * G + my_vcol * VEC;
    if (col >= a.u) col = 0;
    my_off = col;
  }
  auto tile_load = [&](uint32_t t) -> V {
    if (t >= n_tiles) t = n_tiles - 1;
    if constexpr (BY_STEP) {
      const uint32_t o = t / a.tiles_per_run, i = t - o * a.tiles_per_run;
      int64_t s0 = (int64_t)i * RUN + my_vcol * VEC;
      if (s0 >= a.n_inner) s0 = 0;
      return nt_load(reinterpret_cast<const V*>(yp + o * a.outer_stride + s0 + my_off));
    } else {
      int64_t r = (int64_t)t * RUN + my_row;
      if (r >= a.n_red) r = a.n_red - 1;
      return nt_load(reinterpret_cast<const V*>(yp + r * a.pitch + my_off));
    }
  };
  auto tile_store = [&](uint32_t t, const V& x) {
    V* buf = lds[t & 1];
    if constexpr (BY_STEP) {
      buf[my_row * (PITCH / VEC) + my_vcol] = x;
    } else {
      // this lane holds one step of VEC neighbouring chains: one element into each chain's run
      T* tile = reinterpret_cast<T*>(buf);
#pragma unroll
      for (int e = 0; e < VEC; ++e) tile[(my_vcol * VEC + e) * PITCH + my_row] = x.v[e];
    }
  };
  V x[kDepth];
#pragma unroll
  for (int j = 0; j < kDepth; ++j) x[j] = tile_load(j);
  // whole rounds of kDepth tiles run without a branch between the loads, so that the number of
  // loads behind each vector is the same on every path; the last, partial round loads nothing more
  uint32_t t0 = 0;
  for (; t0 + kDepth <= n_tiles; t0 += kDepth) {
#pragma unroll
    for (int j = 0; j < kDepth; ++j) {
      tile_store(t0 + j, x[j]);
      x[j] = tile_load(t0 + j + kDepth);
      __syncthreads();
    }
  }
#pragma unroll
  for (int j = 0; j < kDepth; ++j) {
    if (t0 + j < n_tiles) {
      tile_store(t0 + j, x[j]);
      __syncthreads();
    }
  }
}

template <class T, int OP, bool PLAIN, bool NEG>
int stream_launch(hipStream_t s, const AccumStreamCall& c, const StreamArgs& a, uint32_t grid) {
  using A = typename ew_acc_of<T>::type;
  ChainStep<T, OP, PLAIN, NEG> f;
  f.da = (A)jvm_cast<T>(c.dest_alpha);
  f.ya = (A)jvm_cast<T>(c.y_alpha);
  f.div0 = c.div0;
  if (c.steps_unit_stride) {
    note_kernel(PLAIN ? "accum_stream_steps_plain" : "accum_stream_steps");
    hipLaunchKernelGGL((accum_stream_kernel<T, OP, PLAIN, NEG, true>), dim3(grid), dim3(kStreamBlock), 0, s, a, f);
  } else {
    note_kernel(PLAIN ? "accum_stream_plain" : "accum_stream");
    hipLaunchKernelGGL((accum_stream_kernel<T, OP, PLAIN, NEG, false>), dim3(grid), dim3(kStreamBlock), 0, s, a, f);
  }
  return after_launch(s);
}

template <class T, int OP>
int stream_run(hipStream_t s, const AccumStreamCall& c) {
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
    g = StreamTile<T, true>::G;
    constexpr int run = StreamTile<T, true>::RUN;
    a.tiles_per_run = (uint32_t)((c.n_inner + run - 1) / run);
  } else {
    g = StreamTile<T, false>::G;
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
    if (da == 1.0f && ya == 1.0f) return stream_launch<T, OP, true, false>(s, c, a, (uint32_t)grid);
    if (da == 1.0f && ya == -1.0f) return stream_launch<T, OP, true, true>(s, c, a, (uint32_t)grid);
  }
  return stream_launch<T, OP, false, false>(s, c, a, (uint32_t)grid);
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
