// common.h -- shared host/device helpers of libcortex_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <type_traits>

#include "../../include/cortex_hip.h"

namespace cthip {

// ------------------------------------------------------------------ errors

// Thread-local message read back by ct_last_error().
char* err_buf();
const char** last_kernel_slot();
int set_error(int code, const char* fmt, ...);
bool debug_sync();

// Scratch memory owned by the library, one growing block per (device, stream,
// slot).  Kernels of one stream run in order, so consecutive calls may reuse a
// slot; a call that needs two live temporaries uses two slots.
enum ScratchSlot { kScratchReduce = 0, kScratchAccumA = 1, kScratchAccumB = 2, kScratchSlots = 3 };
int stream_scratch(hipStream_t s, size_t bytes, void** out, int slot = kScratchReduce);
void release_stream_scratch(hipStream_t s);

inline void note_kernel(const char* name) { *last_kernel_slot() = name; }

// A word of device memory per device that kernels set, with a plain store, when they meet a
// condition the reference's CPU backend would throw on (an integer division by zero).  It is
// allocated on the first call that may need it.  check_device_errors reads and clears it when
// debug-sync mode is on (the stream has been synchronised by then) and turns a set word into
// CT_ERR_INVALID; without debug-sync the word is never read and the call succeeds with 0
// stored where the division by zero happened.
int device_error_word(uint32_t** out);
int check_device_errors(const char* what);
// In debug-sync mode, clears the word on stream `s` ahead of a launch that may set it, so that
// what check_device_errors finds afterwards was set by that launch.
int arm_device_error_word(hipStream_t s, uint32_t* word);

#define CT_HIP(expr)                                                                          \
  do {                                                                                        \
    hipError_t e__ = (expr);                                                                  \
    if (e__ != hipSuccess)                                                                    \
      return ::cthip::set_error(CT_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(e__));  \
  } while (0)

#define CT_REQUIRE(cond, ...)                                              \
  do {                                                                     \
    if (!(cond)) return ::cthip::set_error(CT_ERR_INVALID, __VA_ARGS__);   \
  } while (0)

// Called after every kernel launch: surfaces launch errors and, in debug-sync
// mode, faults of the kernel itself.
inline int after_launch(hipStream_t s) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return set_error(CT_ERR_HIP, "kernel launch failed: %s", hipGetErrorString(e));
  if (debug_sync()) {
    e = hipStreamSynchronize(s);
    if (e != hipSuccess) return set_error(CT_ERR_HIP, "kernel failed: %s", hipGetErrorString(e));
  }
  return CT_OK;
}

// ------------------------------------------------------------------ datatypes

inline int dtype_size(int dt) {
  switch (dt) {
    case CT_I8: case CT_U8: return 1;
    case CT_I16: return 2;
    case CT_I32: case CT_F32: return 4;
    case CT_I64: case CT_F64: return 8;
    default: return 0;
  }
}

template <class T> struct acc_of {
  using type = typename std::conditional<std::is_floating_point<T>::value, double, int64_t>::type;
};

// The accumulator of the elementwise functors.  For byte and short tensors an int does what the
// reference's long does: every operand and multiplier has been cast to T first, so products of
// two fit in 32 bits exactly (what max, min, the comparisons and the division see), and sums,
// differences and products of those are truncated to T at the store, which gives the same bits
// from arithmetic modulo 2^32 as from arithmetic modulo 2^64.  (Reductions keep the long: a mean
// divides the untruncated sum.)
template <class T> struct ew_acc_of {
  using type = typename std::conditional<std::is_floating_point<T>::value, double,
                                         typename std::conditional<(sizeof(T) <= 2), int32_t, int64_t>::type>::type;
};

// Runs `body` with T bound to the C type of datatype `dt`.
#define CT_DISPATCH_DTYPE(dt, ...)                                              \
  switch (dt) {                                                                 \
    case CT_I8: { using T = int8_t; __VA_ARGS__; } break;                       \
    case CT_I16: { using T = int16_t; __VA_ARGS__; } break;                     \
    case CT_I32: { using T = int32_t; __VA_ARGS__; } break;                     \
    case CT_I64: { using T = int64_t; __VA_ARGS__; } break;                     \
    case CT_F32: { using T = float; __VA_ARGS__; } break;                       \
    case CT_F64: { using T = double; __VA_ARGS__; } break;                      \
    case CT_U8: { using T = uint8_t; __VA_ARGS__; } break;                      \
    default: return ::cthip::set_error(CT_ERR_INVALID, "unknown datatype %d", (int)(dt)); \
  }

// ------------------------------------------------------------------ JVM value semantics
// The CPU backend of the reference is JVM code compiled under *unchecked-math*
// (src/cortex/compute/cpu/tensor_math.clj:28): its casts are Java primitive
// conversions (src/cortex/compute/cpu/driver.clj:149-157).  These helpers give
// the same results on the device and on the host.

#define CT_HD __host__ __device__ __forceinline__

CT_HD int32_t jvm_d2i(double v) {  // NaN -> 0, saturates, rounds toward zero
  int32_t r = (int32_t)(v < 2147483647.0 ? (v > -2147483648.0 ? v : -2147483648.0) : 2147483647.0);
  return (v != v) ? 0 : r;
}
CT_HD int64_t jvm_d2l(double v) {
  const double hi = 9223372036854775808.0;
  if (v != v) return 0;
  if (v >= hi) return INT64_MAX;
  if (v <= -hi) return INT64_MIN;
  return (int64_t)v;
}

// Result of a long computation stored into T.
template <class T> CT_HD T jvm_cast(int64_t v) {
  if constexpr (std::is_floating_point<T>::value) return (T)v;
  else return (T)(uint64_t)v;
}
template <class T> CT_HD T jvm_cast(int32_t v) {
  if constexpr (std::is_floating_point<T>::value) return (T)v;
  else return (T)(uint32_t)v;
}
// Result of a double computation stored into T; byte and short go through int.
template <class T> CT_HD T jvm_cast(double v) {
  if constexpr (std::is_same<T, double>::value) return v;
  else if constexpr (std::is_same<T, float>::value) return (float)v;
  else if constexpr (std::is_same<T, int64_t>::value) return jvm_d2l(v);
  else return (T)(uint32_t)jvm_d2i(v);
}
template <class T, class S> CT_HD T jvm_convert(S s) {
  if constexpr (std::is_same<T, S>::value) return s;
  else if constexpr (std::is_floating_point<S>::value) return jvm_cast<T>((double)s);
  else return jvm_cast<T>((int64_t)s);
}

// Wrapping long arithmetic / plain double arithmetic under one name.
CT_HD int64_t w_mul(int64_t a, int64_t b) { return (int64_t)((uint64_t)a * (uint64_t)b); }
CT_HD int64_t w_add(int64_t a, int64_t b) { return (int64_t)((uint64_t)a + (uint64_t)b); }
CT_HD int64_t w_sub(int64_t a, int64_t b) { return (int64_t)((uint64_t)a - (uint64_t)b); }
CT_HD int64_t w_neg(int64_t a) { return (int64_t)(0ull - (uint64_t)a); }
CT_HD int32_t w_mul(int32_t a, int32_t b) { return (int32_t)((uint32_t)a * (uint32_t)b); }
CT_HD int32_t w_add(int32_t a, int32_t b) { return (int32_t)((uint32_t)a + (uint32_t)b); }
CT_HD int32_t w_sub(int32_t a, int32_t b) { return (int32_t)((uint32_t)a - (uint32_t)b); }
CT_HD int32_t w_neg(int32_t a) { return (int32_t)(0u - (uint32_t)a); }
CT_HD double w_mul(double a, double b) { return a * b; }
CT_HD double w_add(double a, double b) { return a + b; }
CT_HD double w_sub(double a, double b) { return a - b; }
CT_HD double w_neg(double a) { return -a; }

// Casting (/ a b) of two longs to T: exact quotients are Longs (truncating
// cast); inexact ones are Ratios whose intValue saturates and whose longValue
// truncates toward zero.  Division by zero yields 0 on the device (the
// reference throws ArithmeticException; a kernel cannot).
template <class T> CT_HD T jvm_ratio_cast(int64_t n, int64_t d) {
  if (d == 0) return (T)0;
  if ((int64_t)(int32_t)n == n && (int64_t)(int32_t)d == d) {
    // Both fit 32 bits (int tensors under multipliers of 1, small longs): a 32-bit division is a
    // fifth of the instructions of the 64-bit one (int [2^26] x / y: 37 -> 6x % of the memory rate).
    // -2^31 / -1 = 2^31 is an exact quotient and takes the truncating cast like any other.
    if (d == -1) return jvm_cast<T>(-n);
    const int32_t q = (int32_t)n / (int32_t)d;
    if (std::is_same<T, int64_t>::value || (int64_t)q * d == n) return jvm_cast<T>((int64_t)q);
    return jvm_cast<T>((double)q);
  }
  if (n == INT64_MIN && d == -1) return jvm_cast<T>(n);
  const int64_t q = n / d;
  if (std::is_same<T, int64_t>::value || q * d == n) return jvm_cast<T>(q);
  return jvm_cast<T>((double)q);
}

// The same for the int accumulator of byte and short tensors (|n|, |d| <= 2^30: no overflow case).
template <class T> CT_HD T jvm_ratio_cast(int32_t n, int32_t d) {
  if (d == 0) return (T)0;
  const int32_t q = n / d;
  if (q * d == n) return jvm_cast<T>(q);
  return jvm_cast<T>((double)q);
}

// ------------------------------------------------------------------ 32-bit division by an invariant

// q = n / d for 0 <= n < 2^31, 1 <= d < 2^31, with one multiply-high.
struct FastDiv {
  uint32_t d, m, s;
  FastDiv() : d(1), m(0), s(0) {}
  explicit FastDiv(uint32_t div) : d(div) {
    for (s = 0; s < 32; ++s)
      if ((1u << s) >= d) break;
    const uint64_t one = 1;
    m = (uint32_t)(((one << 32) * ((one << s) - d)) / d + 1);
  }
  __device__ __forceinline__ uint32_t div(uint32_t n) const { return (__umulhi(n, m) + n) >> s; }
  __device__ __forceinline__ void divmod(uint32_t n, uint32_t& q, uint32_t& r) const {
    q = div(n);
    r = n - q * d;
  }
};

// ------------------------------------------------------------------ block order across the dies

// Consecutive block ids are dealt round-robin to the eight dies (XCDs) of
// gfx950, each with its own L2.  A streaming kernel whose block b takes the b-th
// 4 KiB of a buffer therefore hands every die a comb of 4 KiB pieces 32 KiB
// apart.  Regrouped so that a die takes kXcdGroup consecutive pieces (512 KiB)
// at a time, about what its compute units hold in flight, bare streaming kernels
// measured, over 64 MiB ... 1 GiB per buffer: copy +1 to +3 points of the HBM
// peak, three reads and a write +2 to +4.5, a read-only stream +3 to +5, the
// optimizers' four reads and three writes in place +2 to +6; the library's own
// flat kernels, same range of sizes: copy +0.5 to +4, x + y +1 to +6.5, a
// three-input select -1 to +4.  Groups of 4 to 64 pieces gain as much at
// 256 MiB but lose up to 10 points at 1 GiB.  The reductions, softmax and rand!
// kernels gained nothing from the same regrouping (the double row reduction and
// rand! lost 5 points) and keep the plain order.
constexpr uint32_t kXcds = 8;
constexpr uint32_t kXcdGroup = 128;

// Host side: the leading blocks of a grid that are regrouped (whole spans of
// kXcds * kXcdGroup); the rest keep their own index.
inline uint32_t xcd_grouped_blocks(uint32_t grid) { return grid / (kXcds * kXcdGroup) * (kXcds * kXcdGroup); }

// Device side: the unit of work block b takes.  A bijection of [0, grid).
__device__ __forceinline__ uint32_t xcd_grouped_unit(uint32_t b, uint32_t grouped_blocks) {
  if (b >= grouped_blocks) return b;
  const uint32_t k = b / kXcds;
  return ((k / kXcdGroup) * kXcds + b % kXcds) * kXcdGroup + k % kXcdGroup;
}

}  // namespace cthip
