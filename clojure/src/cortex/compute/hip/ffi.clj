(ns cortex.compute.hip.ffi
  "JNA binding of libcortex_hip.so (include/cortex_hip.h): library loading, status checking,
  and the marshalling of dimensions and descriptors into the C structs.

  Plays the part that the JavaCPP presets and `cuda-call` play for the CUDA backend
  (src/cortex/compute/cuda/driver.clj:40-103).  JNA is the one new dependency
  ([net.java.dev.jna/jna \"5.13.0\"] in project.clj); the library itself is plain C.

  UNEXERCISED: no JVM exists where this repository is built and tested.  The same entry points,
  in the same argument order, are driven through ctypes by cortex_amd/capi.py and
  cortex_amd/driver.py; tests/test_clojure_glue.py checks every ct_* call in these files
  against the header (name, argument count, and the machine type each coercion yields)."
  (:require [think.datatype.core :as dtype]
            [clojure.core.matrix :as m])
  (:import [com.sun.jna Function NativeLibrary Pointer Memory]
           [com.sun.jna.ptr PointerByReference IntByReference LongByReference FloatByReference]))

(set! *warn-on-reflection* true)

(def ^NativeLibrary lib
  "libcortex_hip.so, found on jna.library.path / LD_LIBRARY_PATH."
  (delay (NativeLibrary/getInstance "cortex_hip")))

(defn- native-fn ^Function [^String fn-name]
  (.getFunction ^NativeLibrary @lib fn-name))

(defn last-error ^String []
  (.invokeString (native-fn "ct_last_error") (object-array 0) false))

(defn call!
  "Invoke a ct_* entry point.  A non-zero status becomes an ex-info carrying ct_last_error, as
  every failed CUDA call becomes an exception in the reference (cuda/driver.clj:40-49)."
  [^String fn-name & args]
  (let [status (.invokeInt (native-fn fn-name) (object-array args))]
    (when-not (= 0 status)
      (throw (ex-info (last-error) {:function fn-name :status status})))
    nil))

;; ---------------------------------------------------------------- codes shared with the header

(def datatype->code
  "ct_dtype.  The first six in the reference's order (cuda/driver.clj:354-367); :ubyte is the
  unsigned-byte extension."
  {:byte 0 :short 1 :int 2 :long 3 :float 4 :double 5 :ubyte 6})

(def datatype->byte-size {:byte 1 :short 2 :int 4 :long 8 :float 4 :double 8 :ubyte 1})

(defn dtype-code [item] (int (datatype->code (dtype/get-datatype item))))

;; resources/operations.h:88-102 and cuda/tensor_math.clj:54-92
(def unary-op->code {:floor 0 :ceil 1 :round 2 :- 3 :tanh 4 :logistic 5 :exp 6 :sqrt 7 :noop 8})
(def binary-op->code {:+ 0 :- 1 :* 2 :/ 3 :min 4 :max 5 :bit-and 6 :bit-xor 7 :eq 8 :> 9 :>= 10 :< 11 :<= 12})
(def ternary-op->code {:select 0})
(def reduce-op->code {:max 0 :min 1 :sum 2 :mean 3 :magnitude 4 :magnitude-squared 5})
(def activation-op->code {:logistic 0 :tanh 1 :relu 2})
(def pool-op->code {:max 0 :avg 1 :avg-exc-pad 2})
(def copy-kind {:host->device 0 :device->host 1 :device->device 2})

(defn op-code [table op]
  (int (or (table op) (throw (ex-info "Unrecognized operation" {:operation op :known (keys table)})))))

(defn bool->int [flag] (int (if flag 1 0)))

;; ---------------------------------------------------------------- structs

(def ^:const ct-max-dims 8)
;; struct ct_dims { int32 ndim; (4 bytes padding) int64 shape[8]; int64 strides[8]; const int32* index[8]; }
(def ^:const dims-shape-offset 8)
(def ^:const dims-strides-offset 72)
(def ^:const dims-index-offset 136)
(def ^:const dims-byte-size 200)

(defn dims->native
  "A {:shape :strides} dimension map as a ct_dims struct.  A shape entry that is a tensor marks an
  indirectly addressed dimension (src/cortex/tensor/dimensions.clj:7-9): its length goes into
  shape[i] and the device address of its int32 buffer into index[i].  `tensor->pointer` resolves
  such an index tensor to a com.sun.jna.Pointer."
  ^Memory [{:keys [shape strides]} tensor->pointer]
  (when (> (count shape) ct-max-dims)
    (throw (ex-info "Rank exceeds the backend's maximum" {:shape shape :maximum ct-max-dims})))
  (let [mem (Memory. dims-byte-size)]
    (.clear mem)
    (.setInt mem 0 (int (count shape)))
    (doseq [[^long i entry] (map-indexed vector shape)]
      (if (number? entry)
        (.setLong mem (+ dims-shape-offset (* 8 i)) (long entry))
        (do (.setLong mem (+ dims-shape-offset (* 8 i)) (long (m/ecount entry)))
            (.setPointer mem (+ dims-index-offset (* 8 i)) (tensor->pointer entry)))))
    (doseq [[^long i stride] (map-indexed vector strides)]
      (.setLong mem (+ dims-strides-offset (* 8 i)) (long stride)))
    mem))

(defn pool-desc->native
  "ct_pool_desc: seven int32 fields (src/cortex/tensor.clj:1499-1524)."
  ^Memory [{:keys [kernel-width kernel-height pad-x pad-y stride-x stride-y pool-op]}]
  (doto (Memory. 28)
    (.setInt 0 (int kernel-width)) (.setInt 4 (int kernel-height))
    (.setInt 8 (int pad-x)) (.setInt 12 (int pad-y))
    (.setInt 16 (int stride-x)) (.setInt 20 (int stride-y))
    (.setInt 24 (op-code pool-op->code pool-op))))

(defn conv-desc->native
  "ct_conv_desc: eight int32 fields (src/cortex/tensor.clj:1320-1348)."
  ^Memory [{:keys [in-channels out-channels kernel-width kernel-height pad-x pad-y stride-x stride-y]}]
  (doto (Memory. 32)
    (.setInt 0 (int in-channels)) (.setInt 4 (int out-channels))
    (.setInt 8 (int kernel-width)) (.setInt 12 (int kernel-height))
    (.setInt 16 (int pad-x)) (.setInt 20 (int pad-y))
    (.setInt 24 (int stride-x)) (.setInt 28 (int stride-y))))

(defn arg-indexes->native
  "The int8[3] of ct_ternary_op_constant*: for x, y, z the position that supplies it."
  ^Memory [indexes]
  (let [mem (Memory. 3)]
    (doseq [[^long i v] (map-indexed vector indexes)]
      (.setByte mem i (byte v)))
    mem))
