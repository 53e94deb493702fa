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

// The bernoulli dropout mask in one pass (src/cortex/compute/nn/layers.clj:170-195): the
// reference draws rand! flat over [p - 1, p) into a float buffer, assign!s it into the
// multiplier buffer (a conversion when the network runs in double) and turns it into the mask
// with ternary-op! :select, (x >= 0) ? 1 / p : 0.  One lane draws the same Philox block as
// rand_kernel, forms the same float, converts it as assign! does and selects: the stored
// values are those of the three calls, bit for bit.
template <class T, bool KEEP_RAND, bool ALIGNED>
__global__ void __launch_bounds__(kBlock) dropout_mask_kernel(const RandArgs a, T* mult, const T keep_value,
                                                              const T drop_value) {
  const uint64_t i = (uint64_t)blockIdx.x * kBlock + threadIdx.x;
  const int64_t first = (int64_t)i * 4;
  if (first >= a.n) return;
  Vec<float, 4> r;
  rand_block<CT_DIST_FLAT>(a, i, r.v);
  Vec<T, 4> m;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const T x = jvm_convert<T, float>(r.v[e]);          // assign!
    m.v[e] = ((double)x >= 0.0) ? keep_value : drop_value;  // select on x * 1.0
  }
  if (ALIGNED && first + 4 <= a.n) {
    if constexpr (KEEP_RAND) *reinterpret_cast<Vec<float, 4>*>(a.dest + first) = r;
    if constexpr (sizeof(T) == 4) {
      *reinterpret_cast<Vec<T, 4>*>(mult + first) = m;
    } else {
      *reinterpret_cast<Vec<T, 2>*>(mult + first) = Vec<T, 2>{{m.v[0], m.v[1]}};
      *reinterpret_cast<Vec<T, 2>*>(mult + first + 2) = Vec<T, 2>{{m.v[2], m.v[3]}};
    }
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (first + e < a.n) {
        if constexpr (KEEP_RAND) a.dest[first + e] = r.v[e];
        mult[first + e] = m.v[e];
      }
  }
}

template <class T>
int dropout_mask_run(hipStream_t s, RandArgs r, void* mult, double probability) {
  // the constants as the reference's front end hands them to the backend: already multiplied by
  // their alphas in double (src/cortex/tensor.clj:802-803), then cast to the tensor's datatype
  const T keep_value = jvm_cast<T>(1.0 * (1.0 / probability));
  const T drop_value = jvm_cast<T>(0.0 * 0.0);
  const bool keep_rand = r.dest != nullptr && (void*)r.dest != mult;
  const bool aligned = (uintptr_t)mult % 16 == 0 && (!keep_rand || (uintptr_t)r.dest % 16 == 0);
  const dim3 grid((uint32_t)(((r.n + 3) / 4 + kBlock - 1) / kBlock));
  T* m = reinterpret_cast<T*>(mult);
  note_kernel("dropout_mask");
#define CT_DROPOUT(KEEP, AL) hipLaunchKernelGGL((dropout_mask_kernel<T, KEEP, AL>), grid, dim3(kBlock), 0, s, r, m, keep_value, drop_value)
  if (keep_rand) { if (aligned) CT_DROPOUT(true, true); else CT_DROPOUT(true, false); }
  else { if (aligned) CT_DROPOUT(false, true); else CT_DROPOUT(false, false); }
#undef CT_DROPOUT
  return after_launch(s);
}

}  // namespace

extern "C" {

int ct_dropout_bernoulli_mask(void* stream, void* mult_buffer, int dtype, void* rand_buffer, int64_t n,
                              double probability, uint64_t seed, uint64_t offset) {
  CT_REQUIRE(dtype == CT_F32 || dtype == CT_F64, "ct_dropout_bernoulli_mask: datatype must be float or double");
  CT_REQUIRE(n >= 0, "ct_dropout_bernoulli_mask: negative count");
  if (n == 0) return CT_OK;
  CT_REQUIRE(mult_buffer != nullptr, "ct_dropout_bernoulli_mask: null buffer");
  CT_REQUIRE(n < (int64_t(1) << 40), "ct_dropout_bernoulli_mask: count exceeds the supported range");
  // the layer's distribution: maximum = (float probability), minimum = maximum - 1.0, then rand!'s own
  // rounding of both bounds to float (compute/nn/layers.clj:179-182; ct_rand)
  const double maximum_d = (double)(float)probability;
  const float minimum = (float)(maximum_d - 1.0), maximum = (float)maximum_d;
  CT_REQUIRE(minimum < maximum, "Minimum must be less than maximum");
  RandArgs r;
  r.dest = reinterpret_cast<float*>(rand_buffer);
  r.n = n;
  r.seed_lo = (uint32_t)seed; r.seed_hi = (uint32_t)(seed >> 32);
  r.off_lo = (uint32_t)offset; r.off_hi = (uint32_t)(offset >> 32);
  r.p0 = (double)minimum;
  r.p1 = (double)maximum - (double)minimum;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == CT_F32) return dropout_mask_run<float>(s, r, mult_buffer, probability);
  return dropout_mask_run<double>(s, r, mult_buffer, probability);
}

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
