// driver.hip -- device, memory, stream and event entry points (the
// cortex.compute.driver protocols, src/cortex/compute/driver.clj:46-203) plus
// the library's error state.
#include <atomic>
#include <map>
#include <mutex>

#include "elementwise.h"
#include "functors.h"

namespace cthip {

namespace {
thread_local char g_err[512] = "";
thread_local const char* g_kernel = "";
std::atomic<int> g_debug_sync{0};
}  // namespace

char* err_buf() { return g_err; }
const char** last_kernel_slot() { return &g_kernel; }
bool debug_sync() { return g_debug_sync.load(std::memory_order_relaxed) != 0; }

namespace {
struct ScratchKey {
  int device;
  hipStream_t stream;
  int slot;
  bool operator<(const ScratchKey& o) const {
    if (device != o.device) return device < o.device;
    if (stream != o.stream) return stream < o.stream;
    return slot < o.slot;
  }
};
struct ScratchBlock { void* ptr; size_t bytes; };
std::mutex g_scratch_mutex;
std::map<ScratchKey, ScratchBlock> g_scratch;
}  // namespace

int stream_scratch(hipStream_t s, size_t bytes, void** out, int slot) {
  int dev = 0;
  CT_HIP(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  ScratchBlock& b = g_scratch[ScratchKey{dev, s, slot}];
  if (b.bytes < bytes) {
    if (b.ptr) {
      // earlier kernels of this stream may still be reading the old block
      CT_HIP(hipStreamSynchronize(s));
      CT_HIP(hipFree(b.ptr));
      b.ptr = nullptr;
      b.bytes = 0;
    }
    size_t want = bytes < (size_t(1) << 20) ? (size_t(1) << 20) : bytes;
    CT_HIP(hipMalloc(&b.ptr, want));
    b.bytes = want;
  }
  *out = b.ptr;
  return CT_OK;
}

void release_stream_scratch(hipStream_t s) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  for (int slot = 0; slot < kScratchSlots; ++slot) {
    auto it = g_scratch.find(ScratchKey{dev, s, slot});
    if (it == g_scratch.end()) continue;
    if (it->second.ptr) (void)hipFree(it->second.ptr);
    g_scratch.erase(it);
  }
}

namespace {
std::mutex g_error_word_mutex;
std::map<int, uint32_t*> g_error_word;
}  // namespace

int device_error_word(uint32_t** out) {
  int dev = 0;
  CT_HIP(hipGetDevice(&dev));
  std::lock_guard<std::mutex> lock(g_error_word_mutex);
  uint32_t*& w = g_error_word[dev];
  if (!w) {
    void* p = nullptr;
    CT_HIP(hipMalloc(&p, 256));
    hipError_t rc = hipMemset(p, 0, 256);
    if (rc != hipSuccess) {
      (void)hipFree(p);
      return set_error(CT_ERR_HIP, "hipMemset failed: %s", hipGetErrorString(rc));
    }
    w = static_cast<uint32_t*>(p);
  }
  *out = w;
  return CT_OK;
}

int arm_device_error_word(hipStream_t s, uint32_t* word) {
  if (debug_sync() && word) CT_HIP(hipMemsetAsync(word, 0, sizeof(uint32_t), s));
  return CT_OK;
}

int check_device_errors(const char* what) {
  if (!debug_sync()) return CT_OK;
  int dev = 0;
  CT_HIP(hipGetDevice(&dev));
  uint32_t* w = nullptr;
  {
    std::lock_guard<std::mutex> lock(g_error_word_mutex);
    auto it = g_error_word.find(dev);
    if (it == g_error_word.end()) return CT_OK;
    w = it->second;
  }
  uint32_t value = 0;
  CT_HIP(hipMemcpy(&value, w, sizeof(value), hipMemcpyDeviceToHost));
  if (value == 0) return CT_OK;
  CT_HIP(hipMemset(w, 0, sizeof(value)));
  return set_error(CT_ERR_INVALID, "%s: Divide by zero", what);
}

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

namespace {
// Lowest position whose entry lies outside [0, limit), kept with an unsigned minimum.
__global__ void __launch_bounds__(kBlock) index_check_kernel(const int32_t* index, uint32_t n, int64_t limit,
                                                             uint32_t* first_bad) {
  for (uint32_t i = blockIdx.x * kBlock + threadIdx.x; i < n; i += gridDim.x * kBlock) {
    const int64_t v = index[i];
    if (v < 0 || v >= limit) atomicMin(first_bad, i);
  }
}
}  // namespace

}  // namespace cthip

using namespace cthip;

extern "C" {

const char* ct_last_error(void) { return err_buf(); }
const char* ct_last_kernel(void) { return *last_kernel_slot(); }

int ct_set_debug_sync(int on) {
  g_debug_sync.store(on ? 1 : 0);
  return CT_OK;
}

int ct_device_count(int* n) {
  CT_REQUIRE(n != nullptr, "ct_device_count: null output");
  CT_HIP(hipGetDeviceCount(n));
  return CT_OK;
}

int ct_set_device(int device) {
  CT_HIP(hipSetDevice(device));
  return CT_OK;
}

int ct_get_device(int* device) {
  CT_REQUIRE(device != nullptr, "ct_get_device: null output");
  CT_HIP(hipGetDevice(device));
  return CT_OK;
}

int ct_memory_info(size_t* free_bytes, size_t* total_bytes) {
  CT_REQUIRE(free_bytes && total_bytes, "ct_memory_info: null output");
  CT_HIP(hipMemGetInfo(free_bytes, total_bytes));
  return CT_OK;
}

int ct_malloc(void** ptr, size_t bytes) {
  CT_REQUIRE(ptr != nullptr, "ct_malloc: null output");
  *ptr = nullptr;
  CT_HIP(hipMalloc(ptr, bytes ? bytes : 1));
  return CT_OK;
}

int ct_free(void* ptr) {
  if (ptr) CT_HIP(hipFree(ptr));
  return CT_OK;
}

int ct_host_alloc(void** ptr, size_t bytes) {
  CT_REQUIRE(ptr != nullptr, "ct_host_alloc: null output");
  *ptr = nullptr;
  CT_HIP(hipHostMalloc(ptr, bytes ? bytes : 1, hipHostMallocDefault));
  return CT_OK;
}

int ct_host_free(void* ptr) {
  if (ptr) CT_HIP(hipHostFree(ptr));
  return CT_OK;
}

int ct_stream_create(void** stream) {
  CT_REQUIRE(stream != nullptr, "ct_stream_create: null output");
  hipStream_t s = nullptr;
  CT_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  *stream = (void*)s;
  return CT_OK;
}

int ct_stream_destroy(void* stream) {
  if (stream) {
    CT_HIP(hipStreamSynchronize((hipStream_t)stream));
    release_stream_scratch((hipStream_t)stream);
    CT_HIP(hipStreamDestroy((hipStream_t)stream));
  }
  return CT_OK;
}

int ct_stream_reserve_scratch(void* stream, size_t partial_bytes, size_t accumulate_bytes) {
  void* unused = nullptr;
  if (partial_bytes)
    if (int rc = stream_scratch((hipStream_t)stream, partial_bytes, &unused, kScratchReduce)) return rc;
  if (accumulate_bytes) {
    if (int rc = stream_scratch((hipStream_t)stream, accumulate_bytes, &unused, kScratchAccumA)) return rc;
    if (int rc = stream_scratch((hipStream_t)stream, accumulate_bytes, &unused, kScratchAccumB)) return rc;
  }
  return CT_OK;
}

int ct_check_index_range(void* stream, const int32_t* index, int64_t n, int64_t limit) {
  if (n < 0 || n >= (int64_t(1) << 31)) return set_error(CT_ERR_INVALID, "ct_check_index_range: %lld entries", (long long)n);
  if (n == 0) return CT_OK;
  if (!index) return set_error(CT_ERR_INVALID, "ct_check_index_range: null index tensor");
  hipStream_t s = (hipStream_t)stream;
  uint32_t* word = nullptr;
  if (int rc = device_error_word(&word)) return rc;
  uint32_t* first_bad = word + 1;  // the word itself belongs to the divide-by-zero check
  static std::mutex one_check_at_a_time;  // concurrent checks on one device would share first_bad
  std::lock_guard<std::mutex> lock(one_check_at_a_time);
  CT_HIP(hipMemsetAsync(first_bad, 0xFF, sizeof(uint32_t), s));
  const uint32_t blocks = (uint32_t)std::min<int64_t>((n + kBlock - 1) / kBlock, 4096);
  hipLaunchKernelGGL(index_check_kernel, dim3(blocks), dim3(kBlock), 0, s, index, (uint32_t)n, limit, first_bad);
  CT_HIP(hipGetLastError());
  uint32_t at = 0;
  CT_HIP(hipMemcpyAsync(&at, first_bad, sizeof(at), hipMemcpyDeviceToHost, s));
  CT_HIP(hipStreamSynchronize(s));
  if (at == 0xFFFFFFFFu) return CT_OK;
  int32_t value = 0;
  CT_HIP(hipMemcpy(&value, index + at, sizeof(value), hipMemcpyDeviceToHost));
  return set_error(CT_ERR_INVALID, "Index out of range: entry %u of the index tensor is %d, outside [0, %lld)", at, value,
                   (long long)limit);
}

int ct_stream_sync(void* stream) {
  CT_HIP(hipStreamSynchronize((hipStream_t)stream));
  return CT_OK;
}

int ct_event_record(void** event, void* stream) {
  CT_REQUIRE(event != nullptr, "ct_event_record: null output");
  hipEvent_t e = nullptr;
  CT_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
  hipError_t rc = hipEventRecord(e, (hipStream_t)stream);
  if (rc != hipSuccess) {
    (void)hipEventDestroy(e);
    return set_error(CT_ERR_HIP, "hipEventRecord failed: %s", hipGetErrorString(rc));
  }
  *event = (void*)e;
  return CT_OK;
}

int ct_event_record_timed(void** event, void* stream) {
  CT_REQUIRE(event != nullptr, "ct_event_record_timed: null output");
  hipEvent_t e = nullptr;
  CT_HIP(hipEventCreate(&e));
  hipError_t rc = hipEventRecord(e, (hipStream_t)stream);
  if (rc != hipSuccess) {
    (void)hipEventDestroy(e);
    return set_error(CT_ERR_HIP, "hipEventRecord failed: %s", hipGetErrorString(rc));
  }
  *event = (void*)e;
  return CT_OK;
}

int ct_stream_wait_event(void* stream, void* event) {
  CT_REQUIRE(event != nullptr, "ct_stream_wait_event: null event");
  CT_HIP(hipStreamWaitEvent((hipStream_t)stream, (hipEvent_t)event, 0));
  return CT_OK;
}

int ct_event_sync(void* event) {
  CT_REQUIRE(event != nullptr, "ct_event_sync: null event");
  CT_HIP(hipEventSynchronize((hipEvent_t)event));
  return CT_OK;
}

int ct_event_destroy(void* event) {
  if (event) CT_HIP(hipEventDestroy((hipEvent_t)event));
  return CT_OK;
}

int ct_event_elapsed_ms(void* start_event, void* stop_event, float* ms) {
  CT_REQUIRE(start_event && stop_event && ms, "ct_event_elapsed_ms: null argument");
  CT_HIP(hipEventElapsedTime(ms, (hipEvent_t)start_event, (hipEvent_t)stop_event));
  return CT_OK;
}

int ct_memcpy_async(void* dst, const void* src, size_t bytes, int kind, void* stream) {
  if (bytes == 0) return CT_OK;
  CT_REQUIRE(dst && src, "ct_memcpy_async: null pointer");
  hipMemcpyKind k;
  switch (kind) {
    case CT_COPY_HOST_TO_DEVICE: k = hipMemcpyHostToDevice; break;
    case CT_COPY_DEVICE_TO_HOST: k = hipMemcpyDeviceToHost; break;
    case CT_COPY_DEVICE_TO_DEVICE: k = hipMemcpyDeviceToDevice; break;
    default: return set_error(CT_ERR_INVALID, "ct_memcpy_async: unknown copy kind %d", kind);
  }
  CT_HIP(hipMemcpyAsync(dst, src, bytes, k, (hipStream_t)stream));
  if (debug_sync()) CT_HIP(hipStreamSynchronize((hipStream_t)stream));
  return CT_OK;
}

// PStream memset (src/cortex/compute/cuda/driver.clj:1020-1032): a typed fill.
// It runs as a fill kernel for every value, zero included, so that it can be
// recorded into a captured graph.
int ct_memset(void* stream, void* buffer, int dtype, double value, int64_t n) {
  CT_REQUIRE(n >= 0, "ct_memset: negative count");
  if (n == 0) return CT_OK;
  CT_REQUIRE(buffer != nullptr, "ct_memset: null buffer");
  ct_dims d;
  std::memset(&d, 0, sizeof(d));
  d.ndim = 1;
  d.shape[0] = n;
  d.strides[0] = 1;
  CT_DISPATCH_DTYPE(dtype, {
    ConstantF<T> f{jvm_cast<T>(value)};
    EwOperand ops[1] = {{buffer, &d, (int)sizeof(T), 0}};
    return launch_elementwise(static_cast<hipStream_t>(stream), f, ops, n);
  });
  return CT_OK;
}

}  // extern "C"
