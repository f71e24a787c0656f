(in-package :cl-waffe2/backends.hip)

;; The device class.  It derives from AbstractTensor directly, NOT from LispTensor: LispTensor's
;; kernels `aref` the storage vector, which here is an opaque device handle.  The protocol
;; implemented is the one listed in source/vm/generic-tensor/tensor.lisp:146-210:
;; allocator, vref / (setf vref), tensor-finalizer, current-backend-state.

(defstruct (device-buffer (:constructor %make-device-buffer (pointer bytes)))
  "Storage of a HIPTensor: a device pointer from wf2hip_malloc and its size in bytes."
  (pointer (null-pointer) :type foreign-pointer)
  (bytes 0 :type fixnum))

(defun make-device-buffer (n-elements &key (zero t))
  (ensure-extension)
  (let ((bytes (* 4 n-elements)))
    (with-foreign-object (slot :pointer)
      (check (if zero
                 (wf2hip-malloc slot bytes)
                 (wf2hip-malloc-uninitialized slot bytes)))
      (let* ((pointer (mem-ref slot :pointer))
             (buffer (%make-device-buffer pointer bytes)))
        ;; ExistTensors created by the user are reclaimed by the GC; temporaries of a compiled
        ;; model go through tensor-finalizer (adjust-allocation!, source/vm/allocation.lisp:108).
        (trivial-garbage:finalize buffer (lambda () (wf2hip-free pointer)))
        buffer))))

(defclass HIPTensor (AbstractTensor) nil
  (:documentation "
## [AbstractTensor] HIPTensor

fp32 tensors resident in the HBM of an AMD MI355X; kernels come from libwaffe2-hip.so."))

(defmethod current-backend-state ((backend-name (eql 'HIPTensor)))
  (if *hip-extension-p*
      (with-foreign-pointer-as-string (buf 256)
        (wf2hip-device-info buf 256))
      "libwaffe2-hip.so: not available"))

(defmethod initialize-instance :before ((tensor HIPTensor) &rest initargs &key &allow-other-keys)
  ;; Same contract as LispTensor's allocator (source/backends/lisp/tensor.lisp:12-28):
  ;; only :exist tensors own storage; a given :vec is adopted; otherwise allocate
  ;; prod(shape) elements filled with :initial-element (default 0).
  (let ((shape (getf initargs :shape))
        (vec (getf initargs :vec))
        (facet (getf initargs :facet))
        (initial-element (getf initargs :initial-element)))
    (unless (member (or (getf initargs :dtype) :float) '(:float))
      (error "HIPTensor supports :float only, got ~a" (getf initargs :dtype)))
    (when (eql facet :exist)
      (if vec
          (setf (tensor-vec tensor) vec)
          (let* ((n (apply #'* shape))
                 (buffer (make-device-buffer n :zero t)))
            (when (and initial-element (not (zerop initial-element)))
              (check (wf2hip-fill-f32 (device-buffer-pointer buffer) n (coerce initial-element 'single-float))))
            (setf (tensor-vec tensor) buffer))))))

(defun tensor-device-pointer (tensor &optional (offset 0))
  "Device address of element OFFSET of TENSOR's storage (the analogue of incf-tensor-ptr,
source/backends/cpu/tensor.lisp:32-40)."
  (inc-pointer (device-buffer-pointer (tensor-vec tensor)) (* 4 offset)))

;; One element across PCIe.  Used by Mat->ScalarNode, tests and printing; never in a loop.
(defmethod vref ((tensor HIPTensor) index)
  (with-foreign-object (host :float)
    (check (wf2hip-memcpy-d2h host (tensor-device-pointer tensor index) 4))
    (mem-ref host :float)))

(defmethod (setf vref) (new-value (tensor HIPTensor) index)
  (with-foreign-object (host :float)
    (setf (mem-ref host :float) (coerce new-value 'single-float))
    (check (wf2hip-memcpy-h2d (tensor-device-pointer tensor index) host 4)))
  new-value)

(defmethod tensor-finalizer ((tensor HIPTensor))
  (let ((buffer (tensor-vec tensor)))
    (lambda ()
      (when (and buffer (not (null-pointer-p (device-buffer-pointer buffer))))
        (trivial-garbage:cancel-finalization buffer)
        (wf2hip-free (device-buffer-pointer buffer))
        (setf (device-buffer-pointer buffer) (null-pointer))))))

;; Bulk transfers.  The generic convert-tensor-facet path copies element by element through
;; vref (source/array-converter.lisp:154-197), which is unusable across PCIe; these methods move
;; the whole storage in one copy.
(defmethod cl-waffe2:convert-tensor-facet ((from HIPTensor) (to (eql 'simple-array)))
  (let* ((n (floor (device-buffer-bytes (tensor-vec from)) 4))
         (host (make-array n :element-type 'single-float)))
    (with-pointer-to-vector-data (p host)
      (check (wf2hip-memcpy-d2h p (tensor-device-pointer from) (* 4 n))))
    host))

(defun upload (array)
  "A fresh contiguous HIPTensor holding the contents of a (simple-array single-float)."
  (let* ((flat (make-array (array-total-size array) :element-type 'single-float :displaced-to array))
         (storage (coerce flat '(simple-array single-float (*))))
         (tensor (make-tensor (array-dimensions array) :dtype :float :device 'HIPTensor)))
    (with-pointer-to-vector-data (p storage)
      (check (wf2hip-memcpy-h2d (tensor-device-pointer tensor) p (* 4 (length storage)))))
    tensor))
