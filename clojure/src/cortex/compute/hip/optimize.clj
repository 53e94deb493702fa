(ns cortex.compute.hip.optimize
  "create-optimizer for the :hip backend: the fused Adam and Adadelta steps and SGD.

  Parallels (defmethod create-optimizer [:cuda :adam]) in src/cortex/optimize/adam.clj:173-179,
  [:cuda :adadelta] in src/cortex/optimize/adadelta.clj:92-113 and [:cuda :sgd] in
  src/cortex/optimize/sgd.clj:63-65.  The reference defines its methods inside those namespaces,
  next to private helpers; here each optimizer is a small record of its own that implements
  PGradientOptimizer with the same arithmetic around the native step:
    Adam      pow-beta_i-t *= beta_i per batch, in double (adam.clj:149-153); m and v are addressed at
              the parameter buffer's offset inside the flat optimizer state (adam.clj:132-133)
    Adadelta  both accumulators addressed at the parameter offset (AdadeltaOptimizer.java:42-43)
    SGD       four tensor calls (sgd.clj:16-40), so the :cuda method's body serves unchanged
  UNEXERCISED (no JVM in the build image)."
  (:require [cortex.optimize :refer [PGradientOptimizer create-optimizer]]
            [cortex.optimize.sgd]
            [cortex.compute.math :as math]
            [cortex.compute.driver :as drv]
            [cortex.compute.nn.backend :as compute-backend]
            [cortex.compute.hip.ffi :as ffi :refer [call!]]
            [cortex.compute.hip.driver :refer [->ptr]]
            [think.datatype.core :as dtype]))

(set! *warn-on-reflection* true)

(defn- ensure-datatype [datatype & arrays]
  (when-not (every? #(= datatype (dtype/get-datatype %)) arrays)
    (throw (ex-info "Buffer datatype mismatch"
                    {:expected-datatype datatype
                     :actual-datatypes (mapv dtype/get-datatype arrays)}))))

(defn- ->buffer
  "The device buffer behind a DeviceArray, `offset` elements in."
  ([array ^long offset]
   (drv/sub-buffer (math/device-buffer array) offset (- (long (dtype/ecount array)) offset)))
  ([array] (->buffer array 0)))

(defn- select-device! [stream]
  (call! "ct_set_device" (int (:index (:device stream)))))

(defrecord HipAdam [backend optimizer pow-beta1-t pow-beta2-t]
  PGradientOptimizer
  (batch-update [this optimizer-parameters]
    (let [{:keys [beta1 beta2]} optimizer]
      (-> this
          (update :pow-beta1-t #(* (double %) (double beta1)))
          (update :pow-beta2-t #(* (double %) (double beta2))))))
  (compute-parameters! [this {:keys [m v]} gradient-alpha offset gradient parameters]
    (let [{:keys [alpha beta1 beta2 epsilon]} optimizer
          datatype (dtype/get-datatype backend)
          stream (compute-backend/get-stream)]
      (ensure-datatype datatype gradient parameters m v)
      (select-device! stream)
      (call! "ct_adam_step" (:handle stream) (int (ffi/datatype->code datatype))
             (double alpha) (double beta1) (double beta2) (double epsilon)
             (double pow-beta1-t) (double pow-beta2-t) (double gradient-alpha)
             (->ptr (->buffer gradient)) (->ptr (->buffer parameters))
             (->ptr (->buffer m (long offset))) (->ptr (->buffer v (long offset)))
             (long (dtype/ecount gradient))))))

(defmethod create-optimizer [:hip :adam]
  [backend optimizer]
  (->HipAdam backend optimizer 1.0 1.0))

(defrecord HipAdadelta [backend optimizer]
  PGradientOptimizer
  (batch-update [this _] this)
  (compute-parameters! [this {:keys [grad-accum dx-accum]} gradient-alpha offset gradient parameters]
    (let [{:keys [decay epsilon]} optimizer
          datatype (dtype/get-datatype backend)
          stream (compute-backend/get-stream)]
      (ensure-datatype datatype gradient parameters grad-accum dx-accum)
      (select-device! stream)
      (call! "ct_adadelta_step" (:handle stream) (int (ffi/datatype->code datatype))
             (double decay) (double epsilon)
             (->ptr (->buffer grad-accum (long offset))) (->ptr (->buffer dx-accum (long offset)))
             (double gradient-alpha) (->ptr (->buffer gradient)) (->ptr (->buffer parameters))
             (long (dtype/ecount gradient))))))

(defmethod create-optimizer [:hip :adadelta]
  [backend optimizer]
  (->HipAdadelta backend optimizer))

;; SGD is composed from tensor calls only; the method registered for :cuda builds a record that holds
;; nothing backend-specific, so :hip reuses it.
(defmethod create-optimizer [:hip :sgd]
  [backend optimizer]
  ((get-method create-optimizer [:cuda :sgd]) backend optimizer))
