// ops_rand.hip -- rand! (src/cortex/tensor/math.clj:237): fills a dense float
// buffer with gaussian or flat random numbers.
//
// The reference's backends draw from stateful library generators
// (java.security.SecureRandom on the CPU, src/cortex/compute/cpu/tensor_math.clj:1867-1890;
// cuRAND on CUDA, src/cortex/compute/cuda/tensor_math.clj:1246-1274), so only the
// distribution is specified, not the values.  Here the generator is the
// counter-based Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy
// as 1, 2, 3", SC'11): value k of the stream (seed, offset) is word k % 4 of the
// Philox block with counter (k / 4, offset) and key seed.  The call is a pure
// function of (seed, offset, n), keeps no state on the device, and every lane
// writes one 16-byte vector.
//
//   flat      u = (word >> 8) * 2^-24 in [0, 1);  value = T(min + u * (max - min))
//             with min, max rounded to float first and the arithmetic in double,
//             as the CPU backend computes it (:1881-1887)
//   gaussian  Box-Muller on word pairs in float: u1 = ((w0 >> 8) + 1) * 2^-24 in
//             (0, 1], u2 = (w1 >> 8) * 2^-24, r = sqrt(-2 ln u1), a = 2 pi u2,
//             z = (r cos a, r sin a);  value = T(sqrt(variance) * z + mean) in
//             double (:1873-1880)
#include "elementwise.h"

using namespace cthip;

namespace {

struct Philox4 { uint32_t v[4]; };

__device__ __forceinline__ Philox4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                                                  uint32_t k1) {
  constexpr uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u, W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    // one 32 x 32 -> 64 multiplication per product instead of a high and a low one
    const uint64_t p0 = (uint64_t)M0 * c0, p1 = (uint64_t)M1 * c2;
    const uint32_t hi0 = (uint32_t)(p0 >> 32), lo0 = (uint32_t)p0;
    const uint32_t hi1 = (uint32_t)(p1 >> 32), lo1 = (uint32_t)p1;
    const uint32_t n0 = hi1 ^ c1 ^ k0, n2 = hi0 ^ c3 ^ k1;
    c0 = n0; c1 = lo1; c2 = n2; c3 = lo0;
    k0 += W0; k1 += W1;
  }
  return Philox4{{c0, c1, c2, c3}};
}

struct RandArgs {
  float* dest;
  int64_t n;
  uint32_t seed_lo, seed_hi, off_lo, off_hi;
  double p0, p1;  // flat: minimum, range; gaussian: mean, multiplier
};

constexpr float kInv24 = 5.9604644775390625e-08f;  // 2^-24
constexpr float kMinusTwoLn2 = -1.38629436111989061883f;  // -2 ln 2

template <int DIST>
__device__ __forceinline__ void rand_block(const RandArgs& a, uint64_t i, float* out) {
  const Philox4 r = philox4x32_10((uint32_t)i, (uint32_t)(i >> 32), a.off_lo, a.off_hi, a.seed_lo, a.seed_hi);
  if constexpr (DIST == CT_DIST_FLAT) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float u = (float)(r.v[e] >> 8) * kInv24;
      out[e] = (float)(a.p0 + (double)u * a.p1);
    }
  } else {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const float u1 = (float)((r.v[2 * h] >> 8) + 1u) * kInv24;
      const float u2 = (float)(r.v[2 * h + 1] >> 8) * kInv24;
      // the hardware's log2, and its sine and cosine of an angle given in turns: u2 is
      // the angle, no range reduction; each is good to about 1e-6 absolute here
      const float rad = __builtin_amdgcn_sqrtf(kMinusTwoLn2 * __log2f(u1));
      out[2 * h] = (float)(a.p1 * (double)(rad * __builtin_amdgcn_cosf(u2)) + a.p0);
      out[2 * h + 1] = (float)(a.p1 * (double)(rad * __builtin_amdgcn_sinf(u2)) + a.p0);
    }
  }
}

template <int DIST, bool ALIGNED>
__global__ void __launch_bounds__(kBlock) rand_kernel(const RandArgs a) {
  const uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
  const int64_t first = (int64_t)i * 4;
  if (first >= a.n) return;
  Vec<float, 4> v;
  rand_block<DIST>(a, i, v.v);
  if (ALIGNED && first + 4 <= a.n) {
    *reinterpret_cast<Vec<float, 4>*>(a.dest + first) = v;
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (first + e < a.n) a.dest[first + e] = v.v[e];
  }
}

}  // namespace

extern "C" {

int ct_rand(void* stream, void* dest, int64_t n, int dtype, int distribution, double a, double b, uint64_t seed,
            uint64_t offset) {
  CT_REQUIRE(dtype == CT_F32, "Can only generate rands into floating point buffers");
  CT_REQUIRE(n >= 0, "ct_rand: negative count");
  if (n == 0) return CT_OK;
  CT_REQUIRE(dest != nullptr, "ct_rand: null buffer");
  CT_REQUIRE(n < (int64_t(1) << 40), "ct_rand: count exceeds the supported range");
  RandArgs r;
  r.dest = reinterpret_cast<float*>(dest);
  r.n = n;
  r.seed_lo = (uint32_t)seed; r.seed_hi = (uint32_t)(seed >> 32);
  r.off_lo = (uint32_t)offset; r.off_hi = (uint32_t)(offset >> 32);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid((uint32_t)(((n + 3) / 4 + kBlock - 1) / kBlock));
  const bool aligned = (uintptr_t)dest % 16 == 0;
  if (distribution == CT_DIST_FLAT) {
    const float minimum = (float)a, maximum = (float)b;
    CT_REQUIRE(minimum < maximum, "Minimum must be less than maximum");
    r.p0 = (double)minimum;
    r.p1 = (double)maximum - (double)minimum;
    note_kernel("rand_flat");
    if (aligned) hipLaunchKernelGGL((rand_kernel<CT_DIST_FLAT, true>), grid, dim3(kBlock), 0, s, r);
    else hipLaunchKernelGGL((rand_kernel<CT_DIST_FLAT, false>), grid, dim3(kBlock), 0, s, r);
  } else if (distribution == CT_DIST_GAUSSIAN) {
    CT_REQUIRE((float)b >= 0.0f, "ct_rand: negative variance");
    r.p0 = (double)(float)a;
    r.p1 = sqrt((double)(float)b);
    note_kernel("rand_gaussian");
    if (aligned) hipLaunchKernelGGL((rand_kernel<CT_DIST_GAUSSIAN, true>), grid, dim3(kBlock), 0, s, r);
    else hipLaunchKernelGGL((rand_kernel<CT_DIST_GAUSSIAN, false>), grid, dim3(kBlock), 0, s, r);
  } else {
    return set_error(CT_ERR_INVALID, "Unrecognized distribution: %d", distribution);
  }
  return after_launch(s);
}

}  // extern "C"
