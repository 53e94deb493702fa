(ns cortex.compute.hip.backend
  "The :hip backend record: what cortex.nn.execute hands to the network (a device, a default
  stream, a datatype) plus the provider protocols the layers query.

  Parallels src/cortex/compute/cuda/backend.clj:33-72.  No cuDNN-style handles are needed: every
  layer in src/cortex/compute/nn/layers.clj is written against cortex.tensor, and the tensor calls
  land in cortex.compute.hip.tensor-math.  UNEXERCISED (no JVM in the build image)."
  (:require [cortex.compute.driver :as drv]
            [cortex.compute.hip.driver :as hip-drv]
            [cortex.compute.hip.tensor-math]      ; extends TensorMath onto HipStream
            [cortex.compute.hip.optimize]         ; create-optimizer [:hip ...]
            [think.datatype.base :as dtype-base]
            [think.resource.core :as resource]))

(set! *warn-on-reflection* true)

(defrecord HipBackend [type device stream datatype]
  resource/PResource
  (release-resource [backend]
    (drv/with-compute-device (get backend :device)
      (resource/release-resource-context (get backend :resource-context))))
  drv/PDeviceProvider
  (get-device [backend] (get backend :device))
  drv/PStreamProvider
  (get-stream [backend] (get backend :stream))
  drv/PDriverProvider
  (get-driver [backend] (drv/get-driver (drv/get-device backend)))
  dtype-base/PDatatype
  (get-datatype [backend] (get backend :datatype)))

(defn backend
  "Create a :hip backend.  Options as for the CPU and CUDA backends: :driver :device :stream :datatype."
  [& {:keys [driver device datatype stream]
      :or {datatype :float}}]
  (let [driver (or driver (hip-drv/driver))
        device (or device (drv/default-device driver))]
    ;; unsafe-with-compute-device: the backend must outlive this function, so its resources are
    ;; gathered into a context of their own that release-resource frees (cuda/backend.clj:58-72)
    (drv/unsafe-with-compute-device
     device
     (let [[backend res-ctx]
           (resource/return-resource-context
            (let [default-stream (or stream (drv/create-stream))]
              (->HipBackend :hip device default-stream datatype)))]
       (resource/track (assoc backend :resource-context res-ctx))))))
