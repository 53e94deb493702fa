/*
 * cortex_hip.h -- C ABI of libcortex_hip.so, the gfx950 (MI355X) backend for
 * the cortex tensor-math driver.
 *
 * Every entry point replaces one method of the reference's compute-driver or
 * TensorMath protocols.  Paths cite /root/reference (originrose/cortex).
 * A JVM caller binds these through JNA; a Python caller through ctypes.
 *
 * Conventions
 *   - Every function returns 0 on success and a non-zero ct_status otherwise;
 *     ct_last_error() then returns a thread-local, human readable message.
 *     (The reference throws on every failed native call,
 *     src/cortex/compute/cuda/driver.clj:40-49.)
 *   - A stream is an opaque handle; NULL selects the device's default stream.
 *     Calls on one stream are ordered and asynchronous with respect to the
 *     host, as on the reference's CUDA backend.  One host thread issues calls
 *     on a given stream at a time: calls that take two launches keep their
 *     intermediate values in scratch memory owned by the stream, and calls
 *     from two threads on one stream could interleave between the launches.
 *     Different threads on different streams are independent.
 *   - Buffers are raw device pointers.  A sub-buffer is pointer arithmetic by
 *     the caller (src/cortex/compute/cuda/driver.clj:502-506).
 *   - Dimensions are given in ELEMENTS, slowest dimension first, exactly as the
 *     reference's {:shape :strides} maps (src/cortex/tensor/dimensions.clj:95-118).
 *   - Scalars (alphas, constants, optimizer hyper-parameters) cross as double
 *     and are cast to the tensor datatype inside the library with JVM
 *     primitive-conversion rules, mirroring drv/dtype-cast
 *     (src/cortex/compute/driver.clj:17-43) followed by the CPU backend's
 *     datatype->cast-fn (src/cortex/compute/cpu/driver.clj:149-157).
 *   - Operation codes reuse the reference's enums
 *     (resources/operations.h:27-45, 88-102; resources/tensor_unary_reduce.cu:9-20)
 *     so the keyword->int tables of src/cortex/compute/cuda/tensor_math.clj:54-92
 *     carry over unchanged.
 */
#ifndef CORTEX_HIP_H
#define CORTEX_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CT_MAX_DIMS 8

/* {:shape :strides} of one operand.  index[d] != NULL marks dimension d as
 * indirectly addressed: the element's coordinate c in [0, shape[d]) is looked
 * up as index[d][c] (a DEVICE pointer to int32) before it is multiplied by the
 * stride (src/cortex/tensor/dimensions.clj:7-9, 226-252). */
typedef struct ct_dims {
  int32_t ndim;
  int64_t shape[CT_MAX_DIMS];
  int64_t strides[CT_MAX_DIMS];
  const int32_t* index[CT_MAX_DIMS];
} ct_dims;

/* Datatypes.  The first six are the reference's, in its order
 * (src/cortex/compute/cuda/driver.clj:354-367; resources/datatypes.h:16-22).
 * CT_U8 has no counterpart there: the reference's :byte is signed. */
typedef enum ct_dtype {
  CT_I8 = 0, CT_I16 = 1, CT_I32 = 2, CT_I64 = 3, CT_F32 = 4, CT_F64 = 5, CT_U8 = 6
} ct_dtype;

/* resources/operations.h:88-102 */
typedef enum ct_unary_op_t {
  CT_UOP_FLOOR = 0, CT_UOP_CEIL = 1, CT_UOP_ROUND = 2, CT_UOP_NEGATE = 3, CT_UOP_TANH = 4,
  CT_UOP_LOGISTIC = 5, CT_UOP_EXP = 6, CT_UOP_SQRT = 7, CT_UOP_NOOP = 8
} ct_unary_op_t;

/* resources/operations.h:27-45 */
typedef enum ct_binary_op_t {
  CT_BOP_ADD = 0, CT_BOP_SUB = 1, CT_BOP_MUL = 2, CT_BOP_DIV = 3, CT_BOP_MIN = 4, CT_BOP_MAX = 5,
  CT_BOP_BIT_AND = 6, CT_BOP_BIT_XOR = 7, CT_BOP_EQ = 8, CT_BOP_GT = 9, CT_BOP_GE = 10,
  CT_BOP_LT = 11, CT_BOP_LE = 12
} ct_binary_op_t;

/* resources/operations.h:246-254: the only ternary op. */
typedef enum ct_ternary_op_t { CT_TOP_SELECT = 0 } ct_ternary_op_t;

/* resources/tensor_unary_reduce.cu:9-20 */
typedef enum ct_reduce_op_t {
  CT_ROP_MAX = 0, CT_ROP_MIN = 1, CT_ROP_SUM = 2, CT_ROP_MEAN = 3, CT_ROP_MAGNITUDE = 4,
  CT_ROP_MAGNITUDE_SQUARED = 5
} ct_reduce_op_t;

/* activation-gradient! operations (src/cortex/tensor.clj:1256-1284; the CUDA
 * backend maps the same three keywords in cuda/tensor_math.clj:179-185). */
typedef enum ct_activation_op_t {
  CT_ACT_LOGISTIC = 0, CT_ACT_TANH = 1, CT_ACT_RELU = 2
} ct_activation_op_t;

/* rand! distributions (src/cortex/tensor.clj:989-1017). */
typedef enum ct_distribution_t { CT_DIST_GAUSSIAN = 0, CT_DIST_FLAT = 1 } ct_distribution_t;

/* :pool-op of a pooling descriptor (src/cortex/tensor.clj:1495-1524). */
typedef enum ct_pool_op_t { CT_POOL_MAX = 0, CT_POOL_AVG = 1, CT_POOL_AVG_EXC_PAD = 2 } ct_pool_op_t;

/* The geometry of a pooling descriptor (src/cortex/tensor.clj:1499-1524): the
 * window, the zero padding on each side and the step between windows. */
typedef struct ct_pool_desc {
  int32_t kernel_width, kernel_height;
  int32_t pad_x, pad_y;
  int32_t stride_x, stride_y;
  int32_t pool_op; /* ct_pool_op_t */
} ct_pool_desc;

typedef enum ct_status {
  CT_OK = 0,
  CT_ERR_INVALID = 1,     /* bad argument: rank, dtype, op code, null pointer, shape rule */
  CT_ERR_HIP = 2,         /* a HIP runtime call failed; message carries hipGetErrorString */
  CT_ERR_UNSUPPORTED = 3  /* valid in the reference but not provided by this backend */
} ct_status;

typedef enum ct_copy_kind {
  CT_COPY_HOST_TO_DEVICE = 0, CT_COPY_DEVICE_TO_HOST = 1, CT_COPY_DEVICE_TO_DEVICE = 2
} ct_copy_kind;

/* ------------------------------------------------------------------ errors */

/* Message of the last failed call on the calling thread ("" if none).
 * Stands in for the exception text of cuda/driver.clj:40-49. */
const char* ct_last_error(void);

/* When on, every entry point synchronises its stream before returning so an
 * asynchronous fault surfaces at the call that caused it.  Mirrors
 * *cuda-library-debug-execution* (src/cortex/compute/cuda/driver.clj:88-93).
 * In this mode an integer division by zero inside binary-op! / binary-accum! :/
 * is reported by the call that met it: CT_ERR_INVALID, "Divide by zero", where the
 * reference's CPU backend throws ArithmeticException (cpu/tensor_math.clj:278-304).
 * With the mode off such a call succeeds and stores 0 for those elements. */
int ct_set_debug_sync(int on);

/* Name of the kernel family chosen by the most recent tensor call on this
 * thread ("vec", "tile", "general", ...).  Diagnostic only; no reference
 * counterpart. */
const char* ct_last_kernel(void);

/* ------------------------------------------------- driver / device (PDriver, PDevice) */

/* PDriver get-devices (src/cortex/compute/driver.clj:46-61;
 * cuda/driver.clj:725-762). */
int ct_device_count(int* n);
/* Select the calling thread's device; the reference re-selects on every call
 * because JVM threads migrate (cuda/driver.clj:63-85). */
int ct_set_device(int device);
int ct_get_device(int* device);
/* PDevice memory-info-impl (compute/driver.clj:74-84). */
int ct_memory_info(size_t* free_bytes, size_t* total_bytes);
/* PDevice allocate-device-buffer-impl (cuda/driver.clj:888-895). */
int ct_malloc(void** ptr, size_t bytes);
int ct_free(void* ptr);
/* PDriver allocate-host-buffer-impl: pinned host memory (cuda/driver.clj:849-887). */
int ct_host_alloc(void** ptr, size_t bytes);
int ct_host_free(void* ptr);

/* ------------------------------------------------- streams / events (PStream, PEvent) */

/* PDevice create-stream-impl (cuda/driver.clj:589-600). */
int ct_stream_create(void** stream);
int ct_stream_destroy(void* stream);
/* Grows the stream's scratch blocks ahead of time.  No reference counterpart.  Calls that take two
 * launches keep their intermediate values in scratch memory owned by the stream, which grows on
 * demand: a call that has to grow a block synchronises the stream, frees the old block and
 * allocates a new one.  A caller that wants no allocation and no synchronisation inside later
 * calls (a latency-critical loop, a stream about to be captured into a graph) reserves once:
 * partial_bytes for the partial results of split reductions, matrix-vector products, convolution
 * passes and batch-normalization statistics (reductions never need more than 16 MiB),
 * accumulate_bytes for each of the two blocks that accumulations into a broadcast or indexed
 * destination stage their temporaries through (at most the destination's size times the updates'
 * outermost extent; 12 bytes per index entry plus the sort's workspace for indexed rows).
 * Zero leaves a block as it is. */
int ct_stream_reserve_scratch(void* stream, size_t partial_bytes, size_t accumulate_bytes);

/* Checks that every entry of an index tensor (the :indexes of a dimension, src/cortex/tensor/
 * dimensions.clj:150-190) lies in [0, limit), limit being the extent of the dimension that the
 * entries select from.  The tensor calls themselves do not check: an entry outside the buffer
 * makes the JVM backend throw an array-bounds exception and makes a GPU kernel read or write
 * memory it does not own.  A descriptor carries no extent for an indexed dimension, so the caller
 * that builds the selection (which knows the extent) calls this when it wants the check, for
 * instance whenever ct_set_debug_sync is on.  Runs after the work already queued on the stream,
 * waits for the stream, and returns CT_ERR_INVALID "Index out of range: entry ..." naming the
 * first offending position; nothing is dereferenced through a bad entry.  n < 2^31. */
int ct_check_index_range(void* stream, const int32_t* index, int64_t n, int64_t limit);

/* Blocks the host until the stream drains: sync-stream
 * (compute/driver.clj:217-221). */
int ct_stream_sync(void* stream);
/* PStream create-event: creates an event and records it on the stream
 * (cuda/driver.clj:1033-1040). */
int ct_event_record(void** event, void* stream);
/* PStream sync-event: make `stream` wait for `event` (cuda/driver.clj:1041-1043). */
int ct_stream_wait_event(void* stream, void* event);
/* PEvent wait-for-event: block the host (cuda/driver.clj:1009-1018). */
int ct_event_sync(void* event);
int ct_event_destroy(void* event);
/* Milliseconds between two recorded events; used for timing. No reference counterpart. */
int ct_event_elapsed_ms(void* start_event, void* stop_event, float* ms);
/* Like ct_event_record but the event keeps timestamps (for ct_event_elapsed_ms). */
int ct_event_record_timed(void** event, void* stream);

/* PStream copy-host->device / copy-device->host / copy-device->device
 * (cuda/driver.clj:922-1019).  Offsets are applied by the caller.  Host
 * memory should come from ct_host_alloc for a truly asynchronous copy. */
int ct_memcpy_async(void* dst, const void* src, size_t bytes, int kind, void* stream);
/* PStream memset: buffer[i] = (dtype)value for i in [0, n)
 * (cuda/driver.clj:1020-1032; resources/memset.cu). */
int ct_memset(void* stream, void* buffer, int dtype, double value, int64_t n);

/* ------------------------------------------------- TensorMath (src/cortex/tensor/math.clj:11-104) */

/* assign-constant! (tensor/math.clj:14-15; cpu/tensor_math.clj:137-153):
 * dest[A(e)] = (dtype)value, e in [0, n). */
int ct_assign_constant(void* stream, void* dest, const ct_dims* dest_dims, int dtype,
                       double value, int64_t n);

/* assign! (tensor/math.clj:16-26; cpu/tensor_math.clj:180-208):
 * dest[Ad(e)] = (dest_dtype) src[As(e)], with JVM narrowing/widening rules. */
int ct_assign(void* stream, void* dest, const ct_dims* dest_dims, int dest_dtype,
              const void* src, const ct_dims* src_dims, int src_dtype, int64_t n);

/* unary-accum! (tensor/math.clj:27-30; cpu/tensor_math.clj:226-240):
 * dest = op(dest * alpha), in place. */
int ct_unary_accum(void* stream, void* dest, const ct_dims* dest_dims, double alpha, int op,
                   int dtype, int64_t n);

/* unary-op! (tensor/math.clj:31-35; cpu/tensor_math.clj:243-262):
 * dest = op(x * alpha). */
int ct_unary_op(void* stream, void* dest, const ct_dims* dest_dims, const void* x,
                const ct_dims* x_dims, double alpha, int op, int dtype, int64_t n);

/* binary-accum-constant! (tensor/math.clj:36-42; cpu/tensor_math.clj:314-344):
 * dest = dest*dest_alpha op scalar   (scalar op dest*dest_alpha when reverse_operands). */
int ct_binary_accum_constant(void* stream, void* dest, const ct_dims* dest_dims,
                             double dest_alpha, double scalar, int64_t n, int op,
                             int reverse_operands, int dtype);

/* binary-op-constant! (tensor/math.clj:44-51; cpu/tensor_math.clj:347-383):
 * dest = x*x_alpha op scalar   (scalar op x*x_alpha when reverse_operands). */
int ct_binary_op_constant(void* stream, void* dest, const ct_dims* dest_dims, const void* x,
                          const ct_dims* x_dims, double x_alpha, double scalar, int64_t n,
                          int op, int reverse_operands, int dtype);

/* binary-accum! (tensor/math.clj:53-65; cpu/tensor_math.clj:386-420, 1439-1463):
 * dest[Ad(e)] = dest[Ad(e)]*dest_alpha op y[Ay(e)]*y_alpha for e = 0..n-1.
 * With dest_requires_cas != 0 several e may hit one dest address (dest is a
 * broadcast target or indirectly indexed); the reference applies them serially
 * in increasing e. */
int ct_binary_accum(void* stream, void* dest, const ct_dims* dest_dims, double dest_alpha,
                    const void* y, const ct_dims* y_dims, double y_alpha, int64_t n, int op,
                    int reverse_operands, int dest_requires_cas, int dtype);

/* binary-op! (tensor/math.clj:67-73; cpu/tensor_math.clj:424-462):
 * dest = x*x_alpha op y*y_alpha. */
int ct_binary_op(void* stream, void* dest, const ct_dims* dest_dims, const void* x,
                 const ct_dims* x_dims, double x_alpha, const void* y, const ct_dims* y_dims,
                 double y_alpha, int64_t n, int op, int dtype);

/* ternary-op! (tensor/math.clj:75-82; cpu/tensor_math.clj:464-497):
 * select: dest = (x*xa >= 0) ? z*za : y*ya. */
int ct_ternary_op(void* stream, void* dest, const ct_dims* dest_dims, const void* x,
                  const ct_dims* x_dims, double x_alpha, const void* y, const ct_dims* y_dims,
                  double y_alpha, const void* z, const ct_dims* z_dims, double z_alpha,
                  int64_t n, int op, int dtype);

/* ternary-op-constant! (tensor/math.clj:84-92; cpu/tensor_math.clj:507-537).
 * a and b are the tensor arguments in x,y,z order, `constant` the remaining
 * one (already multiplied by its alpha, src/cortex/tensor.clj:802-803).
 * arg_idx[k] for k = x,y,z is the position (0 = a, 1 = b, 2 = constant) that
 * supplies that argument: cpu/tensor_math.clj:500-504 arg-order->indexes. */
int ct_ternary_op_constant(void* stream, void* dest, const ct_dims* dest_dims, const void* a,
                           const ct_dims* a_dims, double a_alpha, const void* b,
                           const ct_dims* b_dims, double b_alpha, double constant, int64_t n,
                           int op, const int8_t arg_idx[3], int dtype);

/* ternary-op-constant-constant! (tensor/math.clj:94-102; cpu/tensor_math.clj:540-567).
 * Positions: 0 = a, 1 = const_1, 2 = const_2. */
int ct_ternary_op_constant_constant(void* stream, void* dest, const ct_dims* dest_dims,
                                    const void* a, const ct_dims* a_dims, double a_alpha,
                                    double const_1, double const_2, int64_t n, int op,
                                    const int8_t arg_idx[3], int dtype);

/* unary-reduce! (tensor/math.clj:104-108; cpu/tensor_math.clj:582-663):
 * output [..., 1] <- reduce over the last axis of the input VIEW [..., k] of
 * op(input * input_alpha). */
int ct_unary_reduce(void* stream, void* output, const ct_dims* output_dims, double input_alpha,
                    const void* input, const ct_dims* input_dims, int op, int dtype);

/* The same reduction for callers that cannot allocate device memory while they
 * run: tight serving loops, harnesses that forbid hipMalloc, code that records
 * its calls into a graph.  No counterpart in the reference.  It runs ct_unary_reduce's
 * kernels with ct_unary_reduce's plan, so the results are the same bits, but
 * the partial accumulators of a split reduction (a column reduction through a
 * transposed view, a few very long rows) live in a fixed 2 MiB array that every
 * device the library runs on holds until the process ends, and the call makes
 * no hipMalloc / hipFree.  A reduction whose partial accumulators need more
 * than 2 MiB fails with CT_ERR_INVALID and launches nothing.  All calls on one
 * device share the array: calls that overlap in time on one device (two
 * streams, two host threads) race; calls on one stream are ordered and safe.
 * The first call on a device resolves the array's address.  A caller who
 * records the call into a HIP graph (hipStreamBeginCapture on the stream it
 * passes; replayed against the eager results in tests/test_gpu_graph_capture.py)
 * makes one call outside the capture first, which resolves the address, and
 * leaves debug-sync mode off (with ct_set_debug_sync(1) every call waits for
 * its stream, which a capture does not allow). */
int ct_unary_reduce_noalloc(void* stream, void* output, const ct_dims* output_dims,
                            double input_alpha, const void* input, const ct_dims* input_dims,
                            int op, int dtype);

/* ------------------------------------------------- neural-network tensor ops */

/* activation-gradient! (tensor/math.clj:176-181; cpu/tensor_math.clj:1318-1362):
 *   logistic  input_gradient = output * (1 - output) * output_gradient
 *   tanh      input_gradient = (1 - output * output) * output_gradient
 *   relu      input_gradient = (output > 0 ? 1 : 0) * output_gradient
 * each evaluated in double and rounded once.  dtype is CT_F32 or CT_F64. */
int ct_activation_gradient(void* stream, void* input_gradient, const ct_dims* input_gradient_dims,
                           const void* output_gradient, const ct_dims* output_gradient_dims,
                           const void* output, const ct_dims* output_dims, int op, int64_t n,
                           int dtype);

/* softmax-eltwise! (tensor/math.clj:183-185; cpu/tensor_math.clj:1037-1094):
 * dimensions are [rows, k] or [outer, rows, k]; every row becomes
 * exp(x - max(x)) / sum(exp(x - max(x))).  Direct dimensions only; dtype is
 * CT_F32 or CT_F64. */
int ct_softmax_eltwise(void* stream, void* output, const ct_dims* output_dims, const void* input,
                       const ct_dims* input_dims, int dtype);

/* softmax-spatial! (tensor/math.clj:187-189; cpu/tensor_math.clj:1097-1103):
 * dimensions are [batch, channels, elements]; the softmax runs across the
 * channels of every (batch, element) position. */
int ct_softmax_spatial(void* stream, void* output, const ct_dims* output_dims, const void* input,
                       const ct_dims* input_dims, int dtype);

/* gemm! (tensor/math.clj:106-116; cpu/tensor_math.clj:672-700, 1534-1545;
 * compute/math_util.clj:17-30): row-major
 *   C[a_row_count, b_col_count] = alpha * op(A) * op(B) + beta * C,
 * op(A) is [a_row_count, a_col_count], op(B) is [a_col_count, b_col_count]
 * (the counts are taken after the transposition, src/cortex/tensor.clj:920-951);
 * a column stride is the distance in elements between two stored rows.  Runs on
 * rocBLAS, loaded on first use.  dtype is CT_F32 or CT_F64. */
int ct_gemm(void* stream, void* c, int64_t c_colstride, int trans_a, int trans_b, double alpha,
            const void* a, int64_t a_row_count, int64_t a_col_count, int64_t a_colstride,
            const void* b, int64_t b_col_count, int64_t b_colstride, double beta, int dtype);

/* gemv! (tensor/math.clj:117-123; cpu/tensor_math.clj:701-726, 1547-1556;
 * compute/math_util.clj:33-41): c = alpha * op(A) * x + beta * c for the stored
 * row-major matrix A [a_row_count, a_col_count] (counts before the
 * transposition, src/cortex/tensor.clj:975-989) and vector increments in
 * elements.  The library's own kernels (the product is bound by memory, not by
 * the matrix cores); the sums run in double.  dtype is CT_F32 or CT_F64. */
int ct_gemv(void* stream, void* c, int64_t inc_c, int trans_a, double alpha, const void* a,
            int64_t a_row_count, int64_t a_col_count, int64_t a_colstride, const void* x,
            int64_t inc_x, double beta, int dtype);

/* rand! (tensor/math.clj:237; cpu/tensor_math.clj:1867-1890;
 * cuda/tensor_math.clj:1246-1274): fills n values of a dense float buffer.
 *   CT_DIST_GAUSSIAN  a = mean, b = variance
 *   CT_DIST_FLAT      a = minimum (included), b = maximum (excluded)
 * The reference draws from a stateful library generator, so only the
 * distribution is specified.  Here value k is a pure function of
 * (seed, offset, k) (Philox4x32-10, counter (k / 4, offset), key seed): the
 * caller keeps the generator state, e.g. one seed per stream and an offset it
 * increments per call.  dtype must be CT_F32, as in the reference
 * (src/cortex/tensor.clj:1020-1037). */
int ct_rand(void* stream, void* dest, int64_t n, int dtype, int distribution, double a, double b,
            uint64_t seed, uint64_t offset);

/* The bernoulli dropout mask of src/cortex/compute/nn/layers.clj:170-195 in one launch.  The
 * reference builds it from three tensor calls: rand! with the flat distribution over
 * [probability - 1, probability) into rand_buffer (float32), assign! into mult_buffer (the
 * network's datatype), ternary-op-constant-constant! :select turning every value x of
 * mult_buffer into (x >= 0) ? 1 / probability : 0.  This entry point stores what those three
 * calls store, bit for bit, for the same (seed, offset): mult_buffer receives the mask, and
 * rand_buffer, when it is neither NULL nor mult_buffer itself, the random draws.  dtype (of
 * mult_buffer) is CT_F32 or CT_F64.  A backend whose dropout layer may call it saves two
 * passes over the buffer; the three-call chain stays available and gives the same result. */
int ct_dropout_bernoulli_mask(void* stream, void* mult_buffer, int dtype, void* rand_buffer,
                              int64_t n, double probability, uint64_t seed, uint64_t offset);

/* Batch normalization.  Every buffer is packed: input and output hold
 * batch_count x channel_count x element_count values (the eltwise forms have
 * one element per channel: [batch_count, element_count] with a statistic per
 * element), the statistics / scale / bias vectors hold channel_count values.
 * dtype is CT_F32 or CT_F64.  The stream's scratch memory holds the partial
 * sums between the passes. */

/* batch-normalize-eltwise! / -spatial! (tensor/math.clj:124-137;
 * cpu/tensor_math.clj:756-802):
 *   output = (input - mean) * T(sqrt(1 / (variance + epsilon))) * scale + bias. */
int ct_batch_normalize_eltwise(void* stream, void* output, const void* input, const void* means,
                               const void* variances, const void* scale, const void* bias,
                               double epsilon, int64_t batch_count, int64_t element_count, int dtype);
int ct_batch_normalize_spatial(void* stream, void* output, const void* input, const void* means,
                               const void* variances, const void* scale, const void* bias,
                               double epsilon, int64_t batch_count, int64_t channel_count,
                               int64_t element_count, int dtype);

/* batch-normalize-update-and-apply-eltwise! / -spatial! (tensor/math.clj:138-156;
 * cpu/tensor_math.clj:820-900, 1574-1608): batch_means = mean over the batch,
 * batch_variances = population variance (divisor N),
 * running = running * (1 - average_factor) + batch * average_factor, where the
 * running variance takes the sample variance (divisor N - 1); then the
 * normalization above with the batch statistics. */
int ct_batch_normalize_update_and_apply_eltwise(void* stream, void* output, const void* input,
                                                void* batch_means, void* batch_variances,
                                                void* running_means, void* running_variances,
                                                double average_factor, const void* scale,
                                                const void* bias, double epsilon,
                                                int64_t batch_count, int64_t element_count, int dtype);
int ct_batch_normalize_update_and_apply_spatial(void* stream, void* output, const void* input,
                                                void* batch_means, void* batch_variances,
                                                void* running_means, void* running_variances,
                                                double average_factor, const void* scale,
                                                const void* bias, double epsilon,
                                                int64_t batch_count, int64_t channel_count,
                                                int64_t element_count, int dtype);

/* batch-normalize-gradients-eltwise! / -spatial! (tensor/math.clj:157-174;
 * cpu/tensor_math.clj:903-1033): input_gradient, scale_gradient and
 * bias_gradient are written; `output` and `bias` are accepted for signature
 * parity and not read (the CPU backend does not read them either).
 * input_gradient may alias output_gradient. */
int ct_batch_normalize_gradients_eltwise(void* stream, void* input_gradient, void* scale_gradient,
                                         void* bias_gradient, const void* output_gradient,
                                         const void* output, const void* input,
                                         const void* batch_means, const void* batch_variances,
                                         const void* scale, const void* bias, double epsilon,
                                         int64_t batch_count, int64_t element_count, int dtype);
int ct_batch_normalize_gradients_spatial(void* stream, void* input_gradient, void* scale_gradient,
                                         void* bias_gradient, const void* output_gradient,
                                         const void* output, const void* input,
                                         const void* batch_means, const void* batch_variances,
                                         const void* scale, const void* bias, double epsilon,
                                         int64_t batch_count, int64_t channel_count,
                                         int64_t element_count, int dtype);

/* The geometry of a convolution descriptor (src/cortex/tensor.clj:1320-1348). */
typedef struct ct_conv_desc {
  int32_t in_channels, out_channels;
  int32_t kernel_width, kernel_height;
  int32_t pad_x, pad_y;
  int32_t stride_x, stride_y;
} ct_conv_desc;

/* convolution-forward! / -backward-weights! / -backward-data!
 * (tensor/math.clj:185-220), decomposed as the CPU backend decomposes them
 * (cpu/tensor_math.clj:1118-1151, 1670-1792): the input is unrolled into the
 * caller's workspace (padding reads 0; stored here as [batch, in_channels *
 * kernel_height * kernel_width, out_height * out_width], the transpose of the
 * CPU backend's per-image matrix: the workspace is opaque to callers), and the
 * three methods are one gemm! per image around that matrix:
 *   forward           output[b] = weights x unrolled[b]^T + output_alpha * output[b]
 *   backward-weights  weight_gradient = sum over b of output_gradient[b] x unrolled[b],
 *                     on top of weight_gradient_alpha * weight_gradient; it reads the
 *                     workspace as the forward pass left it and not `input`
 *   backward-data     unrolled[b] = output_gradient[b]^T x weights, rolled back into
 *                     input_gradient by adding every cell to the input element it
 *                     came from, windows in increasing (row, column) order;
 *                     input_gradient is overwritten: the CPU backend replaces
 *                     input_gradient_alpha by 0.0 (:1766)
 * Buffers are packed: input [batch, in_channels, in_height, in_width], output
 * [batch, out_channels, out_height, out_width], weights [out_channels,
 * in_channels * kernel_height * kernel_width].  workspace_ecount must be at
 * least batch * out_height * out_width * in_channels * kernel_height *
 * kernel_width (choose-convolution-algorithms, :1670-1680).  Every window must
 * lie inside the padded input, as the floor rule for convolution output sizes
 * guarantees.  dtype is CT_F32 or CT_F64. */
int ct_convolution_forward(void* stream, void* output, double output_alpha, const void* input,
                           const void* weights, void* workspace, int64_t workspace_ecount,
                           const ct_conv_desc* desc, int64_t batch_count, int64_t in_height,
                           int64_t in_width, int64_t out_height, int64_t out_width, int dtype);
int ct_convolution_backward_weights(void* stream, void* weight_gradient,
                                    double weight_gradient_alpha, const void* output_gradient,
                                    const void* input, void* workspace, int64_t workspace_ecount,
                                    const ct_conv_desc* desc, int64_t batch_count,
                                    int64_t in_height, int64_t in_width, int64_t out_height,
                                    int64_t out_width, int dtype);
int ct_convolution_backward_data(void* stream, void* input_gradient, double input_gradient_alpha,
                                 const void* output_gradient, const void* weights, void* workspace,
                                 int64_t workspace_ecount, const ct_conv_desc* desc,
                                 int64_t batch_count, int64_t in_height, int64_t in_width,
                                 int64_t out_height, int64_t out_width, int dtype);

/* pooling-forward! / pooling-backward! (tensor/math.clj:221-236;
 * cpu/tensor_math.clj:1153-1284, 1800-1866; window walk src/cortex/nn/impl.clj:8-96).
 * Buffers are packed [batch_count, channel_count, height, width]; dtype is
 * CT_F32 or CT_F64.  The taps of a window are visited row by row, those beyond
 * the padded input are skipped, and padding reads as 0:
 *   max          the first tap, then every tap greater than the running value
 *                (padding takes part as 0, NaN only wins as the first tap)
 *   avg          sum of tap / (kernel_width * kernel_height), rounded to the
 *                tensor's type after every tap
 *   avg-exc-pad  tap / (taps of the window inside the input), added ONTO what
 *                `output` holds: the CPU backend never clears it
 * The backward pass adds into input_gradient (never cleared either): for max,
 * output_gradient of every window whose output equals this input; for the
 * averages, output_gradient / divisor of every window covering it; windows in
 * increasing (row, column) order.  output_alpha and input_gradient_alpha are
 * accepted for signature parity: the CPU backend does not read them. */
int ct_pooling_forward(void* stream, void* output, double output_alpha, const void* input,
                       const ct_pool_desc* desc, int64_t batch_count, int64_t channel_count,
                       int64_t in_height, int64_t in_width, int64_t out_height, int64_t out_width,
                       int dtype);
int ct_pooling_backward(void* stream, void* input_gradient, double input_gradient_alpha,
                        const void* input, const void* output, const void* output_gradient,
                        const ct_pool_desc* desc, int64_t batch_count, int64_t channel_count,
                        int64_t in_height, int64_t in_width, int64_t out_height, int64_t out_width,
                        int dtype);

/* lrn-forward! / lrn-backward! (tensor/math.clj:240-252; tensor.clj:1554-1616;
 * cuda/tensor_math.clj:1277-1335, where cuDNN's cross-channel LRN does the
 * work: the reference's CPU backend has no form of it).  Tensors are
 * [batch, channels, height, width] or one image [channels, height, width], of
 * equal shapes, each with its own strides; n, k, alpha and beta are the
 * fields of the reference's lrn-descriptor (1 <= n <= 16, k > 0).  With
 * behind = (n - 1) / 2 and window(c) = [c - behind, c + n - 1 - behind]
 * clipped to the channels:
 *   s[c]  = k + (alpha / n) * sum over window(c) of input^2
 *   output[c] = input[c] * s[c]^-beta
 *   input_gradient[c] = output_gradient[c] * s[c]^-beta
 *       - (2 alpha beta / n) * input[c]
 *         * sum over window(c) of output_gradient[c'] * output[c'] / s[c']
 * (the same window in both directions, as the stored results of
 * src/cortex/verify/tensor.clj:1105-1123 for n = 2 require).  The backward
 * pass keeps output_gradient * output / s of every channel in the tensor's
 * type before summing: for float tensors a quotient below 1e-45 counts as 0.
 * A channel's result needs its neighbours' operands, so neither call works in
 * place: output == input, or an input_gradient that is the same buffer as
 * output_gradient, output or input, is refused with CT_ERR_INVALID.
 * dtype is CT_F32 or CT_F64. */
int ct_lrn_forward(void* stream, void* output, const ct_dims* output_dims, const void* input,
                   const ct_dims* input_dims, int n, double k, double alpha, double beta, int dtype);
int ct_lrn_backward(void* stream, void* input_gradient, const ct_dims* input_gradient_dims,
                    const void* output, const ct_dims* output_dims, const void* input,
                    const ct_dims* input_dims, const void* output_gradient,
                    const ct_dims* output_gradient_dims, int n, double k, double alpha, double beta,
                    int dtype);

/* ------------------------------------------------- optimizers */

/* Adam step (src/cortex/optimize/adam.clj:68-102, 116-134; resources/adam.cu).
 * m and v already point at the parameter buffer's offset inside the flat
 * optimizer state.  dtype is CT_F32 or CT_F64. */
int ct_adam_step(void* stream, int dtype, double alpha, double beta1, double beta2,
                 double epsilon, double pow_beta1_t, double pow_beta2_t, double gradient_alpha,
                 const void* gradient, void* parameters, void* m, void* v, int64_t n);

/* Adadelta step (java/cortex/compute/optimize/AdadeltaOptimizer.java:29-64;
 * src/cortex/optimize/adadelta.clj:32-67; resources/adadelta.cu).
 * grad_sq_accum and dx_sq_accum already point at the parameter offset. */
int ct_adadelta_step(void* stream, int dtype, double decay, double epsilon, void* grad_sq_accum,
                     void* dx_sq_accum, double gradient_alpha, const void* gradient,
                     void* parameters, int64_t n);

#ifdef __cplusplus
}
#endif
#endif /* CORTEX_HIP_H */
