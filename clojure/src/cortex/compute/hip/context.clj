(ns cortex.compute.hip.context
  "Backend selection.  cortex.nn.execute/compute-context (src/cortex/nn/execute.clj:37-67) knows two
  backends: it tries CUDA unless :backend :cpu was asked for and falls back to the CPU.  A :hip
  request is served by the function below, which returns the same {:backend-fn :datatype} map; the
  one-line edit in execute.clj is to consult it first:

      (defn compute-context [& {:keys [datatype backend] :or {datatype :float} :as args}]
        (if (= backend :hip)
          (do (require 'cortex.compute.hip.context)
              ((resolve 'cortex.compute.hip.context/compute-context) :datatype datatype))
          ...the existing body...))

  The namespace is resolved at run time, as execute.clj resolves the CUDA backend (:37-57), so a
  machine without the library or without JNA can still load cortex.  UNEXERCISED (no JVM in the
  build image)."
  (:require [cortex.compute.cpu.backend :as cpu]))

(defn- hip-backend-fn
  [datatype force-hip?]
  (fn []
    (try
      (require 'cortex.compute.hip.backend)
      ((resolve 'cortex.compute.hip.backend/backend) :datatype datatype)
      (catch Throwable e
        (if force-hip?
          (throw (ex-info "Unable to initialize the HIP back-end for GPU support." {:error e}))
          (do (println "HIP backend creation failed, reverting to CPU")
              (cpu/backend :datatype datatype)))))))

(defn compute-context
  "A compute context on the :hip backend.  :force? true (the default) throws when the backend cannot
  be created instead of falling back to the CPU."
  [& {:keys [datatype force?]
      :or {datatype :float force? true}}]
  {:backend-fn (hip-backend-fn datatype force?)
   :datatype datatype})
