(ns cortex.compute.hip.tensor-math
  "cortex.tensor.math/TensorMath (src/cortex/tensor/math.clj:11-252) extended onto HipStream: one
  ct_* entry point of include/cortex_hip.h per protocol method.

  Parallels (extend-type CudaStream tm/TensorMath ...) in
  src/cortex/compute/cuda/tensor_math.clj:289-1341.  Where the CUDA backend explodes every operand
  into fifteen kernel arguments (dimensions->cuda, :34-51) this backend passes one ct_dims struct;
  where it looks up a fatbin function per datatype it passes a datatype code.  Scalars cross as
  double and are cast inside the library with drv/dtype-cast's rules.

  UNEXERCISED (no JVM in the build image); see cortex.compute.hip.ffi."
  (:require [cortex.tensor.math :as tm]
            [cortex.tensor :as ct]
            [cortex.tensor.dimensions :as ct-dims]
            [cortex.compute.driver :as drv]
            [cortex.compute.cpu.tensor-math :as cpu-tm]
            [cortex.compute.hip.ffi :as ffi :refer [call! dtype-code op-code bool->int]]
            [cortex.compute.hip.driver :as hip-drv :refer [->ptr]]
            [think.datatype.core :as dtype])
  (:import [cortex.compute.hip.driver HipStream]))

(set! *warn-on-reflection* true)

(defn- index-tensor->pointer
  "Device address of an index tensor's buffer; it must hold ints (cuda/tensor_math.clj:26-31)."
  [tensor]
  (let [buffer (ct/tensor->buffer tensor)]
    (when-not (= :int (dtype/get-datatype buffer))
      (throw (ex-info "Index buffers must be integer tensors" {:datatype (dtype/get-datatype buffer)})))
    (->ptr buffer)))

(defn- dims [dimensions] (ffi/dims->native dimensions index-tensor->pointer))

(defn- select-device! [stream]
  (call! "ct_set_device" (int (:index (:device stream)))))

(defn- arg-indexes [arg-order]
  (ffi/arg-indexes->native (cpu-tm/arg-order->indexes arg-order)))   ; cpu/tensor_math.clj:500-504

(extend-type HipStream
  tm/TensorMath

  ;; ------------------------------------------------------------ the hot path (tensor/math.clj:14-104)
  (assign-constant! [stream buffer dimensions value n-elems]
    (select-device! stream)
    (call! "ct_assign_constant" (:handle stream) (->ptr buffer) (dims dimensions) (dtype-code buffer)
           (double value) (long n-elems)))

  (assign! [stream dest dest-dims src src-dims n-elems]
    (select-device! stream)
    (call! "ct_assign" (:handle stream) (->ptr dest) (dims dest-dims) (dtype-code dest)
           (->ptr src) (dims src-dims) (dtype-code src) (long n-elems)))

  (unary-accum! [stream dest dest-dims alpha op n-elems]
    (select-device! stream)
    (call! "ct_unary_accum" (:handle stream) (->ptr dest) (dims dest-dims) (double alpha)
           (op-code ffi/unary-op->code op) (dtype-code dest) (long n-elems)))

  (unary-op! [stream dest dest-dims x x-dims alpha op n-elems]
    (select-device! stream)
    (call! "ct_unary_op" (:handle stream) (->ptr dest) (dims dest-dims) (->ptr x) (dims x-dims)
           (double alpha) (op-code ffi/unary-op->code op) (dtype-code dest) (long n-elems)))

  (binary-accum-constant! [stream dest dest-dims dest-alpha scalar n-elems operation reverse-operands?]
    (select-device! stream)
    (call! "ct_binary_accum_constant" (:handle stream) (->ptr dest) (dims dest-dims) (double dest-alpha)
           (double scalar) (long n-elems) (op-code ffi/binary-op->code operation)
           (bool->int reverse-operands?) (dtype-code dest)))

  (binary-op-constant! [stream dest dest-dims x x-dims x-alpha scalar n-elems operation reverse-operands?]
    (select-device! stream)
    (call! "ct_binary_op_constant" (:handle stream) (->ptr dest) (dims dest-dims) (->ptr x) (dims x-dims)
           (double x-alpha) (double scalar) (long n-elems) (op-code ffi/binary-op->code operation)
           (bool->int reverse-operands?) (dtype-code dest)))

  (binary-accum! [stream dest dest-dims dest-alpha y y-dims y-alpha n-elems operation
                  reverse-operands? dest-requires-cas?]
    (select-device! stream)
    (call! "ct_binary_accum" (:handle stream) (->ptr dest) (dims dest-dims) (double dest-alpha)
           (->ptr y) (dims y-dims) (double y-alpha) (long n-elems) (op-code ffi/binary-op->code operation)
           (bool->int reverse-operands?) (bool->int dest-requires-cas?) (dtype-code dest)))

  (binary-op! [stream dest dest-dims x x-dims x-alpha y y-dims y-alpha n-elems operation]
    (select-device! stream)
    (call! "ct_binary_op" (:handle stream) (->ptr dest) (dims dest-dims) (->ptr x) (dims x-dims) (double x-alpha)
           (->ptr y) (dims y-dims) (double y-alpha) (long n-elems) (op-code ffi/binary-op->code operation)
           (dtype-code dest)))

  (ternary-op! [stream dest dest-dims x x-dims x-alpha y y-dims y-alpha z z-dims z-alpha n-elems operation]
    (select-device! stream)
    (call! "ct_ternary_op" (:handle stream) (->ptr dest) (dims dest-dims) (->ptr x) (dims x-dims) (double x-alpha)
           (->ptr y) (dims y-dims) (double y-alpha) (->ptr z) (dims z-dims) (double z-alpha)
           (long n-elems) (op-code ffi/ternary-op->code operation) (dtype-code dest)))

  (ternary-op-constant! [stream dest dest-dims a a-dims a-alpha b b-dims b-alpha constant n-elems operation arg-order]
    (select-device! stream)
    (call! "ct_ternary_op_constant" (:handle stream) (->ptr dest) (dims dest-dims) (->ptr a) (dims a-dims)
           (double a-alpha) (->ptr b) (dims b-dims) (double b-alpha) (double constant) (long n-elems)
           (op-code ffi/ternary-op->code operation) (arg-indexes arg-order) (dtype-code dest)))

  (ternary-op-constant-constant! [stream dest dest-dims a a-dims a-alpha const-1 const-2 n-elems operation arg-order]
    (select-device! stream)
    (call! "ct_ternary_op_constant_constant" (:handle stream) (->ptr dest) (dims dest-dims) (->ptr a) (dims a-dims)
           (double a-alpha) (double const-1) (double const-2) (long n-elems)
           (op-code ffi/ternary-op->code operation) (arg-indexes arg-order) (dtype-code dest)))

  (unary-reduce! [stream output output-dims input-alpha input input-dims op]
    (select-device! stream)
    (call! "ct_unary_reduce" (:handle stream) (->ptr output) (dims output-dims) (double input-alpha)
           (->ptr input) (dims input-dims) (op-code ffi/reduce-op->code op) (dtype-code output)))

  ;; ------------------------------------------------------------ blas (tensor/math.clj:106-123)
  (gemm! [stream c c-colstride trans-a? trans-b? alpha a a-row-count a-col-count a-colstride
          b b-col-count b-colstride beta]
    (select-device! stream)
    (call! "ct_gemm" (:handle stream) (->ptr c) (long c-colstride) (bool->int trans-a?) (bool->int trans-b?)
           (double alpha) (->ptr a) (long a-row-count) (long a-col-count) (long a-colstride)
           (->ptr b) (long b-col-count) (long b-colstride) (double beta) (dtype-code c)))

  (gemv! [stream c inc-c trans-a? alpha a a-row-count a-col-count a-colstride x inc-x beta]
    (select-device! stream)
    (call! "ct_gemv" (:handle stream) (->ptr c) (long inc-c) (bool->int trans-a?) (double alpha) (->ptr a)
           (long a-row-count) (long a-col-count) (long a-colstride) (->ptr x) (long inc-x) (double beta)
           (dtype-code c)))

  ;; ------------------------------------------------------------ batch normalization (tensor/math.clj:124-174)
  (batch-normalize-eltwise! [stream output input means variances scale bias epsilon batch-count element-count]
    (select-device! stream)
    (call! "ct_batch_normalize_eltwise" (:handle stream) (->ptr output) (->ptr input) (->ptr means)
           (->ptr variances) (->ptr scale) (->ptr bias) (double epsilon) (long batch-count) (long element-count)
           (dtype-code output)))

  (batch-normalize-spatial! [stream output input means variances scale bias epsilon
                             batch-count channel-count element-count]
    (select-device! stream)
    (call! "ct_batch_normalize_spatial" (:handle stream) (->ptr output) (->ptr input) (->ptr means)
           (->ptr variances) (->ptr scale) (->ptr bias) (double epsilon) (long batch-count) (long channel-count)
           (long element-count) (dtype-code output)))

  (batch-normalize-update-and-apply-eltwise! [stream output input batch-means batch-variances
                                              running-means running-variances average-factor
                                              scale bias epsilon batch-count element-count]
    (select-device! stream)
    (call! "ct_batch_normalize_update_and_apply_eltwise" (:handle stream) (->ptr output) (->ptr input)
           (->ptr batch-means) (->ptr batch-variances) (->ptr running-means) (->ptr running-variances)
           (double average-factor) (->ptr scale) (->ptr bias) (double epsilon) (long batch-count)
           (long element-count) (dtype-code output)))

  (batch-normalize-update-and-apply-spatial! [stream output input batch-means batch-variances
                                              running-means running-variances average-factor
                                              scale bias epsilon batch-count channel-count element-count]
    (select-device! stream)
    (call! "ct_batch_normalize_update_and_apply_spatial" (:handle stream) (->ptr output) (->ptr input)
           (->ptr batch-means) (->ptr batch-variances) (->ptr running-means) (->ptr running-variances)
           (double average-factor) (->ptr scale) (->ptr bias) (double epsilon) (long batch-count)
           (long channel-count) (long element-count) (dtype-code output)))

  (batch-normalize-gradients-eltwise! [stream input-gradient scale-gradient bias-gradient output-gradient
                                       output input batch-means batch-variances scale bias epsilon
                                       batch-count element-count]
    (select-device! stream)
    (call! "ct_batch_normalize_gradients_eltwise" (:handle stream) (->ptr input-gradient) (->ptr scale-gradient)
           (->ptr bias-gradient) (->ptr output-gradient) (->ptr output) (->ptr input) (->ptr batch-means)
           (->ptr batch-variances) (->ptr scale) (->ptr bias) (double epsilon) (long batch-count)
           (long element-count) (dtype-code input-gradient)))

  (batch-normalize-gradients-spatial! [stream input-gradient scale-gradient bias-gradient output-gradient
                                       output input batch-means batch-variances scale bias epsilon
                                       batch-count channel-count element-count]
    (select-device! stream)
    (call! "ct_batch_normalize_gradients_spatial" (:handle stream) (->ptr input-gradient) (->ptr scale-gradient)
           (->ptr bias-gradient) (->ptr output-gradient) (->ptr output) (->ptr input) (->ptr batch-means)
           (->ptr batch-variances) (->ptr scale) (->ptr bias) (double epsilon) (long batch-count)
           (long channel-count) (long element-count) (dtype-code input-gradient)))

  ;; ------------------------------------------------------------ activation gradient, softmax (tensor/math.clj:176-189)
  (activation-gradient! [stream input-gradient input-grad-dim output-gradient output-grad-dim
                         output output-dim op element-count]
    (select-device! stream)
    (call! "ct_activation_gradient" (:handle stream) (->ptr input-gradient) (dims input-grad-dim)
           (->ptr output-gradient) (dims output-grad-dim) (->ptr output) (dims output-dim)
           (op-code ffi/activation-op->code op) (long element-count) (dtype-code input-gradient)))

  (softmax-eltwise! [stream output output-dims input input-dims]
    (select-device! stream)
    (call! "ct_softmax_eltwise" (:handle stream) (->ptr output) (dims output-dims) (->ptr input) (dims input-dims)
           (dtype-code output)))

  (softmax-spatial! [stream output output-dims input input-dims]
    (select-device! stream)
    (call! "ct_softmax_spatial" (:handle stream) (->ptr output) (dims output-dims) (->ptr input) (dims input-dims)
           (dtype-code output)))

  ;; ------------------------------------------------------------ convolution (tensor/math.clj:185-220)
  ;; the CPU backend's decomposition: no native descriptor object (cpu/tensor_math.clj:1665-1680)
  (convolution-descriptor [stream datatype out-channels in-channels kern-width kern-height
                           pad-x pad-y stride-x stride-y]
    {:datatype datatype :out-channels out-channels :in-channels in-channels
     :kernel-width kern-width :kernel-height kern-height
     :pad-x pad-x :pad-y pad-y :stride-x stride-x :stride-y stride-y})

  (choose-convolution-algorithms [stream conv-descriptor input-width input-height output-width output-height
                                  batch-size max-ideal-workspace-size use-defaults?]
    {:workspace-size (* (long (:kernel-width conv-descriptor)) (long (:kernel-height conv-descriptor))
                        (long (:in-channels conv-descriptor)) (long output-width) (long output-height)
                        (long batch-size))})

  (convolution-forward! [stream output output-dims output-alpha input input-dims weights weight-dims
                         workspace workspace-ecount conv-descriptor algorithms]
    (select-device! stream)
    (let [[batch _ in-height in-width] (:shape input-dims)
          [_ _ out-height out-width] (:shape output-dims)]
      (call! "ct_convolution_forward" (:handle stream) (->ptr output) (double output-alpha) (->ptr input)
             (->ptr weights) (->ptr workspace) (long workspace-ecount) (ffi/conv-desc->native conv-descriptor)
             (long batch) (long in-height) (long in-width) (long out-height) (long out-width)
             (dtype-code output))))

  (convolution-backward-weights! [stream weight-gradient weight-gradient-dims weight-gradient-alpha
                                  output-gradient output-gradient-dims input input-dims
                                  workspace workspace-ecount conv-descriptor algorithms]
    (select-device! stream)
    (let [[batch _ in-height in-width] (:shape input-dims)
          [_ _ out-height out-width] (:shape output-gradient-dims)]
      (call! "ct_convolution_backward_weights" (:handle stream) (->ptr weight-gradient)
             (double weight-gradient-alpha) (->ptr output-gradient) (->ptr input) (->ptr workspace)
             (long workspace-ecount) (ffi/conv-desc->native conv-descriptor)
             (long batch) (long in-height) (long in-width) (long out-height) (long out-width)
             (dtype-code weight-gradient))))

  (convolution-backward-data! [stream input-gradient input-gradient-dims input-gradient-alpha
                               output-gradient output-gradient-dims weights weights-dims
                               workspace workspace-ecount conv-descriptor algorithms]
    (select-device! stream)
    (let [[batch _ in-height in-width] (:shape input-gradient-dims)
          [_ _ out-height out-width] (:shape output-gradient-dims)]
      (call! "ct_convolution_backward_data" (:handle stream) (->ptr input-gradient)
             (double input-gradient-alpha) (->ptr output-gradient) (->ptr weights) (->ptr workspace)
             (long workspace-ecount) (ffi/conv-desc->native conv-descriptor)
             (long batch) (long in-height) (long in-width) (long out-height) (long out-width)
             (dtype-code input-gradient))))

  ;; ------------------------------------------------------------ pooling (tensor/math.clj:221-236)
  (pooling-descriptor [stream datatype kern-width kern-height pad-x pad-y stride-x stride-y pool-op dimension-op]
    {:datatype datatype :kernel-width kern-width :kernel-height kern-height :pad-x pad-x :pad-y pad-y
     :stride-x stride-x :stride-y stride-y :pool-op pool-op :dimension-op dimension-op})

  (pooling-forward! [stream output output-dims output-alpha input input-dims pool-descriptor]
    (select-device! stream)
    (let [[batch channels in-height in-width] (:shape input-dims)
          [_ _ out-height out-width] (:shape output-dims)]
      (call! "ct_pooling_forward" (:handle stream) (->ptr output) (double output-alpha) (->ptr input)
             (ffi/pool-desc->native pool-descriptor) (long batch) (long channels) (long in-height) (long in-width)
             (long out-height) (long out-width) (dtype-code output))))

  (pooling-backward! [stream input-grad input-grad-dims input-grad-alpha input input-dims
                      output output-dims output-grad output-grad-dims pool-descriptor]
    (select-device! stream)
    (let [[batch channels in-height in-width] (:shape input-dims)
          [_ _ out-height out-width] (:shape output-dims)]
      (call! "ct_pooling_backward" (:handle stream) (->ptr input-grad) (double input-grad-alpha) (->ptr input)
             (->ptr output) (->ptr output-grad) (ffi/pool-desc->native pool-descriptor)
             (long batch) (long channels) (long in-height) (long in-width) (long out-height) (long out-width)
             (dtype-code input-grad))))

  ;; ------------------------------------------------------------ rand! (tensor/math.clj:237)
  ;; The stream record keeps the state that the reference keeps inside cuRAND: a seed and the
  ;; number of calls so far, which becomes the Philox offset.
  (rand! [stream dest dest-dims distribution]
    (select-device! stream)
    (let [[kind a b] (case (:type distribution)
                       :gaussian [0 (:mean distribution) (:variance distribution)]
                       :flat [1 (:minimum distribution) (:maximum distribution)]
                       (throw (ex-info "Unrecognized distribution type" {:distribution distribution})))
          {:keys [seed calls]} (swap! (:rand-state stream) update :calls inc)]
      (call! "ct_rand" (:handle stream) (->ptr dest) (long (ct-dims/ecount dest-dims)) (dtype-code dest)
             (int kind) (double a) (double b) (long seed) (long calls))))

  ;; ------------------------------------------------------------ local response normalisation (tensor/math.clj:240-252)
  ;; cuDNN-only in the reference (src/cortex/tensor.clj:1554-1557; cuda/tensor_math.clj:1277-1335).
  ;; The descriptor is a plain map: the library keeps no native object for it.
  (lrn-descriptor [stream n k alpha beta]
    {:n (long n) :k (double k) :alpha (double alpha) :beta (double beta)})

  (lrn-forward! [stream output output-dims input input-dims lrn-descriptor]
    (select-device! stream)
    (let [{:keys [n k alpha beta]} lrn-descriptor]
      (call! "ct_lrn_forward" (:handle stream) (->ptr output) (dims output-dims) (->ptr input) (dims input-dims)
             (int n) (double k) (double alpha) (double beta) (dtype-code output))))

  (lrn-backward! [stream input-gradient input-grad-dims output output-dims input input-dims
                  output-gradient output-grad-dims lrn-descriptor]
    (select-device! stream)
    (let [{:keys [n k alpha beta]} lrn-descriptor]
      (call! "ct_lrn_backward" (:handle stream) (->ptr input-gradient) (dims input-grad-dims)
             (->ptr output) (dims output-dims) (->ptr input) (dims input-dims)
             (->ptr output-gradient) (dims output-grad-dims)
             (int n) (double k) (double alpha) (double beta) (dtype-code output)))))

;; ---------------------------------------------------------------- entry points beyond the protocol

(defn unary-reduce-noalloc!
  "unary-reduce! through ct_unary_reduce_noalloc: same kernels, same result, but no device
  allocation inside the call (partial accumulators in a fixed 2 MiB array per device).  For callers
  that record the stream into a graph or otherwise cannot allocate; a reduction needing more than
  2 MiB of partials throws."
  [stream output output-dims input-alpha input input-dims op]
  (select-device! stream)
  (call! "ct_unary_reduce_noalloc" (:handle stream) (->ptr output) (dims output-dims) (double input-alpha)
         (->ptr input) (dims input-dims) (op-code ffi/reduce-op->code op) (dtype-code output)))

(defn dropout-bernoulli-mask!
  "The three tensor calls of dropout-prepare-forward! (src/cortex/compute/nn/layers.clj:170-195:
  rand!, assign!, ternary-op! :select) as one launch with the same stored values.  `rand-buffer` may
  be nil or `mult-buffer` itself when the random draws need not be kept."
  [stream mult-buffer rand-buffer probability]
  (select-device! stream)
  (let [{:keys [seed calls]} (swap! (:rand-state stream) update :calls inc)]
    (call! "ct_dropout_bernoulli_mask" (:handle stream) (->ptr mult-buffer) (dtype-code mult-buffer)
           (when rand-buffer (->ptr rand-buffer)) (long (dtype/ecount mult-buffer)) (double probability)
           (long seed) (long calls))))

(defn last-kernel
  "Name of the kernel family the most recent tensor call on this thread ran (diagnostic)."
  ^String []
  (.invokeString (.getFunction ^com.sun.jna.NativeLibrary @ffi/lib "ct_last_kernel") (object-array 0) false))
