(ns cortex.compute.hip.driver
  "The compute-driver protocols (src/cortex/compute/driver.clj:46-203) on libcortex_hip.so:
  driver, device, stream, device and host buffers, events.

  Parallels src/cortex/compute/cuda/driver.clj: DevicePointer (:489-510), the driver (:725-762),
  the device (:849-898), the stream (:1009-1045).  UNEXERCISED (no JVM in the build image); see
  cortex.compute.hip.ffi."
  (:require [cortex.compute.driver :as drv]
            [cortex.compute.hip.ffi :as ffi :refer [call!]]
            [think.datatype.core :as dtype]
            [think.datatype.base :as dtype-base]
            [think.resource.core :as resource]
            [clojure.core.matrix.protocols :as mp])
  (:import [com.sun.jna Pointer Memory]
           [com.sun.jna.ptr PointerByReference IntByReference LongByReference]))

(set! *warn-on-reflection* true)

(defn- byte-size ^long [datatype] (long (ffi/datatype->byte-size datatype)))

(defn- select-device!
  "JVM threads migrate between calls, so the device is selected again before every native call,
  as the CUDA backend does (cuda/driver.clj:63-85)."
  [device]
  (call! "ct_set_device" (int (:index device))))

;; ---------------------------------------------------------------- buffers

(declare ->HipBuffer)

(defrecord HipBuffer [^Pointer ptr ^long elem-count datatype device owner?]
  dtype-base/PDatatype
  (get-datatype [_] datatype)
  mp/PElementCount
  (element-count [_] elem-count)
  resource/PResource
  (release-resource [_]
    ;; a sub-buffer is an offset pointer into its parent and owns nothing (cuda/driver.clj:502-506)
    (when owner?
      (select-device! device)
      (call! "ct_free" ptr)))
  drv/PBuffer
  (sub-buffer-impl [_ offset length]
    (->HipBuffer (.share ptr (* (long offset) (byte-size datatype))) (long length) datatype device false))
  (alias? [_ rhs]
    (= (Pointer/nativeValue ptr) (Pointer/nativeValue ^Pointer (:ptr rhs))))
  (partially-alias? [_ rhs]
    (let [lhs-start (Pointer/nativeValue ptr)
          lhs-end (+ lhs-start (* elem-count (byte-size datatype)))
          rhs-start (Pointer/nativeValue ^Pointer (:ptr rhs))
          rhs-end (+ rhs-start (* (long (:elem-count rhs)) (byte-size (:datatype rhs))))]
      (and (< lhs-start rhs-end) (< rhs-start lhs-end)))))

(defn ->ptr
  "Device address of a buffer (or of anything math/device-buffer understands), optionally
  `offset` elements in."
  (^Pointer [buffer] (:ptr buffer))
  (^Pointer [buffer ^long offset]
   (.share ^Pointer (:ptr buffer) (* offset (byte-size (dtype/get-datatype buffer))))))

(defrecord HipHostBuffer [^Pointer ptr ^long elem-count datatype]
  ;; pinned host memory (ct_host_alloc); the dtype copy protocols see it through a direct
  ;; ByteBuffer view, as the CUDA backend exposes its page-locked pointers
  dtype-base/PDatatype
  (get-datatype [_] datatype)
  mp/PElementCount
  (element-count [_] elem-count)
  resource/PResource
  (release-resource [_] (call! "ct_host_free" ptr)))

(defn host-buffer->nio
  "A java.nio.ByteBuffer over the pinned allocation, for the datatype library's copy routines."
  [^HipHostBuffer buffer]
  (.getByteBuffer ^Pointer (:ptr buffer) 0 (* (long (:elem-count buffer)) (byte-size (:datatype buffer)))))

;; ---------------------------------------------------------------- events

(defrecord HipEvent [^Pointer handle]
  drv/PEvent
  (wait-for-event [_] (call! "ct_event_sync" handle))
  resource/PResource
  (release-resource [_] (call! "ct_event_destroy" handle)))

;; ---------------------------------------------------------------- stream

(defn- check-copy-extent
  "Copies past a buffer's extent are refused on the host (cuda/driver.clj:901-919)."
  [buffer ^long offset ^long elem-count]
  (when (> (+ offset elem-count) (long (dtype/ecount buffer)))
    (throw (ex-info "Copy out of range" {:buffer-ecount (dtype/ecount buffer) :offset offset :elem-count elem-count}))))

(defrecord HipStream [device ^Pointer handle rand-state]
  drv/PStream
  (copy-host->device [_ host-buffer host-offset device-buffer device-offset elem-count]
    (check-copy-extent host-buffer host-offset elem-count)
    (check-copy-extent device-buffer device-offset elem-count)
    (select-device! device)
    (call! "ct_memcpy_async" (->ptr device-buffer (long device-offset)) (->ptr host-buffer (long host-offset))
           (long (* (long elem-count) (byte-size (dtype/get-datatype device-buffer))))
           (int (ffi/copy-kind :host->device)) handle))
  (copy-device->host [_ device-buffer device-offset host-buffer host-offset elem-count]
    (check-copy-extent host-buffer host-offset elem-count)
    (check-copy-extent device-buffer device-offset elem-count)
    (select-device! device)
    (call! "ct_memcpy_async" (->ptr host-buffer (long host-offset)) (->ptr device-buffer (long device-offset))
           (long (* (long elem-count) (byte-size (dtype/get-datatype device-buffer))))
           (int (ffi/copy-kind :device->host)) handle))
  (copy-device->device [_ dev-a dev-a-off dev-b dev-b-off elem-count]
    (check-copy-extent dev-a dev-a-off elem-count)
    (check-copy-extent dev-b dev-b-off elem-count)
    (select-device! device)
    (call! "ct_memcpy_async" (->ptr dev-b (long dev-b-off)) (->ptr dev-a (long dev-a-off))
           (long (* (long elem-count) (byte-size (dtype/get-datatype dev-a))))
           (int (ffi/copy-kind :device->device)) handle))
  (memset [_ device-buffer device-offset elem-val elem-count]
    (select-device! device)
    (call! "ct_memset" handle (->ptr device-buffer (long device-offset)) (ffi/dtype-code device-buffer)
           (double elem-val) (long elem-count)))
  (create-event [_]
    (select-device! device)
    (let [event (PointerByReference.)]
      (call! "ct_event_record" event handle)
      (resource/track (->HipEvent (.getValue event)))))
  (sync-event [_ event]
    (select-device! device)
    (call! "ct_stream_wait_event" handle (:handle event)))
  drv/PDeviceProvider
  (get-device [_] device)
  drv/PDriverProvider
  (get-driver [_] (drv/get-driver device))
  resource/PResource
  (release-resource [_]
    (select-device! device)
    (call! "ct_stream_destroy" handle)))

;; ---------------------------------------------------------------- device and driver

(defrecord HipDevice [driver ^long index]
  drv/PDevice
  (memory-info-impl [this]
    (select-device! this)
    (let [free (LongByReference.) total (LongByReference.)]
      (call! "ct_memory_info" free total)
      {:free (.getValue free) :total (.getValue total)}))
  (create-stream-impl [this]
    (select-device! this)
    (let [stream (PointerByReference.)]
      (call! "ct_stream_create" stream)
      ;; rand! keeps its generator state here: a seed and a counter of calls (cortex.compute.hip.tensor-math)
      (resource/track (->HipStream this (.getValue stream) (atom {:seed (System/nanoTime) :calls 0})))))
  (allocate-device-buffer-impl [this elem-count elem-type]
    (select-device! this)
    (let [result (PointerByReference.)]
      (call! "ct_malloc" result (long (* (long elem-count) (byte-size elem-type))))
      (resource/track (->HipBuffer (.getValue result) (long elem-count) elem-type this true))))
  (allocate-rand-buffer-impl [this elem-count]
    ;; the generator has no parity requirement on the count; the buffer is a float buffer as in the reference
    (drv/allocate-device-buffer-impl this elem-count :float))
  drv/PDriverProvider
  (get-driver [_] driver)
  drv/PDeviceProvider
  (get-device [this] this))

(defrecord HipDriver []
  drv/PDriver
  (get-devices [this]
    (let [n (IntByReference.)]
      (call! "ct_device_count" n)
      (mapv #(->HipDevice this (long %)) (range (.getValue n)))))
  (allocate-host-buffer-impl [_ elem-count elem-type options]
    (let [result (PointerByReference.)]
      (call! "ct_host_alloc" result (long (* (long elem-count) (byte-size elem-type))))
      (resource/track (->HipHostBuffer (.getValue result) (long elem-count) elem-type))))
  drv/PDriverProvider
  (get-driver [this] this))

(defn driver [] (->HipDriver))

(defn debug-sync!
  "Synchronise after every native call so that an asynchronous fault (and an integer division by
  zero) is reported by the call that caused it: *cuda-library-debug-execution* (cuda/driver.clj:88-93)."
  [on?]
  (call! "ct_set_debug_sync" (ffi/bool->int on?)))

(defn sync-stream!
  "Block the host until the stream drains, without creating an event."
  [stream]
  (call! "ct_stream_sync" (:handle stream)))

(defn reserve-scratch!
  "Grow the stream's scratch blocks now, so that later calls neither allocate nor synchronise."
  [stream partial-bytes accumulate-bytes]
  (call! "ct_stream_reserve_scratch" (:handle stream) (long partial-bytes) (long accumulate-bytes)))

(defn check-index-range!
  "Throws unless every entry of the int index buffer lies in [0, limit). Synchronises the stream."
  [stream index-buffer n-entries limit]
  (call! "ct_check_index_range" (:handle stream) (->ptr index-buffer) (long n-entries) (long limit)))

(defn timed-event
  "An event that keeps a timestamp, for `elapsed-ms`."
  [stream]
  (let [event (PointerByReference.)]
    (call! "ct_event_record_timed" event (:handle stream))
    (resource/track (->HipEvent (.getValue event)))))

(defn elapsed-ms
  [start-event stop-event]
  (let [ms (com.sun.jna.ptr.FloatByReference.)]
    (call! "ct_event_elapsed_ms" (:handle start-event) (:handle stop-event) ms)
    (.getValue ms)))

(defn current-device-index []
  (let [index (IntByReference.)]
    (call! "ct_get_device" index)
    (.getValue index)))
