(in-package :cl-waffe2/backends.hip)

;; The device class.  It derives from AbstractTensor directly, NOT from LispTensor: LispTensor's
;; kernels `aref` the storage vector, which here is an opaque device handle.  The protocol
;; implemented is the one listed in source/vm/generic-tensor/tensor.lisp:146-210:
;; allocator, vref / (setf vref), tensor-finalizer, current-backend-state.

(defstruct (device-buffer (:constructor %make-device-buffer (pointer bytes)))
  "Storage of a HIPTensor: a device pointer from wf2hip_malloc and its size in bytes."
  (pointer (null-pointer) :type foreign-pointer)
  (bytes 0 :type fixnum))

(defun dtype-info (dtype)
  "(values CFFI-type bytes-per-element wf2hip_dtype-code) of a cl-waffe2 dtype keyword.  Every
node of the path runs on :float; the other dtypes have the arithmetic / move nodes (and :uint32
receives ArgMax-Node / ArgMin-Node results)."
  (ecase dtype
    (:float (values :float 4 0))
    (:double (values :double 8 1))
    (:int32 (values :int32 4 2))
    (:uint32 (values :uint32 4 3))
    (:int16 (values :int16 2 4))
    (:uint16 (values :uint16 2 5))
    (:int8 (values :int8 1 6))
    (:uint8 (values :uint8 1 7))))

(defun dtype-bytes (dtype) (nth-value 1 (dtype-info dtype)))

(defun make-device-buffer (n-elements &key (zero t) (dtype :float))
  (ensure-extension)
  (let ((bytes (* (dtype-bytes dtype) n-elements)))
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
    (dtype-info (or (getf initargs :dtype) :float)) ; signals on an unknown dtype
    (when (eql facet :exist)
      (if vec
          (setf (tensor-vec tensor) vec)
          (let* ((dtype (or (getf initargs :dtype) :float))
                 (n (apply #'* shape))
                 (buffer (make-device-buffer n :zero t :dtype dtype)))
            (when (and initial-element (not (zerop initial-element)))
              (if (eql dtype :float)
                  (check (wf2hip-fill-f32 (device-buffer-pointer buffer) n (coerce initial-element 'single-float)))
                  ;; the other dtypes: one element across PCIe into a buffer of its own, then a
                  ;; stride-0 move spreads it (source and destination must not be one buffer: the
                  ;; kernel reads the source while other lanes write the destination, and the
                  ;; library refuses overlapping runs)
                  (multiple-value-bind (ctype bytes code) (dtype-info dtype)
                    (let ((one (make-device-buffer 1 :zero nil :dtype dtype)))
                      (with-foreign-object (host ctype)
                        (setf (mem-ref host ctype) (coerce initial-element (dtype->lisp-type dtype)))
                        (check (wf2hip-memcpy-h2d (device-buffer-pointer one) host bytes)))
                      (check (wf2hip-binary-1d-typed code +move+ n (device-buffer-pointer buffer) 1
                                                     (device-buffer-pointer one) 0))))))
            (setf (tensor-vec tensor) buffer))))))

(defun tensor-device-pointer (tensor &optional (offset 0))
  "Device address of element OFFSET of TENSOR's storage (the analogue of incf-tensor-ptr,
source/backends/cpu/tensor.lisp:32-40)."
  (inc-pointer (device-buffer-pointer (tensor-vec tensor)) (* (dtype-bytes (dtype tensor)) offset)))

;; One element across PCIe.  Used by Mat->ScalarNode, tests and printing; never in a loop.
(defmethod vref ((tensor HIPTensor) index)
  (multiple-value-bind (ctype bytes) (dtype-info (dtype tensor))
    (with-foreign-object (host ctype)
      (check (wf2hip-memcpy-d2h host (tensor-device-pointer tensor index) bytes))
      (mem-ref host ctype))))

(defmethod (setf vref) (new-value (tensor HIPTensor) index)
  (multiple-value-bind (ctype bytes) (dtype-info (dtype tensor))
    (with-foreign-object (host ctype)
      (setf (mem-ref host ctype) (coerce new-value (dtype->lisp-type (dtype tensor))))
      (check (wf2hip-memcpy-h2d (tensor-device-pointer tensor index) host bytes))))
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
(defun dtype-lisp-type (dtype)
  "Element type of the host vector that mirrors a tensor of DTYPE (dtype->lisp-type,
source/vm/generic-tensor/dtype.lisp)."
  (ecase dtype
    (:float 'single-float) (:double 'double-float)
    (:int32 '(signed-byte 32)) (:uint32 '(unsigned-byte 32))
    (:int16 '(signed-byte 16)) (:uint16 '(unsigned-byte 16))
    (:int8 '(signed-byte 8)) (:uint8 '(unsigned-byte 8))))

(defmethod cl-waffe2:convert-tensor-facet ((from HIPTensor) (to (eql 'simple-array)))
  (let* ((size (dtype-bytes (dtype from)))
         (n (floor (device-buffer-bytes (tensor-vec from)) size))
         (host (make-array n :element-type (dtype-lisp-type (dtype from)))))
    (with-pointer-to-vector-data (p host)
      (check (wf2hip-memcpy-d2h p (tensor-device-pointer from) (* size n))))
    host))

(defun upload (array &key (dtype :float))
  "A fresh contiguous HIPTensor of DTYPE holding the contents of ARRAY, a specialised array whose
element type is DTYPE's host type (single-float for :float, (unsigned-byte 8) for :uint8 ...)."
  (let* ((type (dtype-lisp-type dtype))
         (flat (make-array (array-total-size array) :element-type type :displaced-to array))
         (storage (coerce flat `(simple-array ,type (*))))
         (tensor (make-tensor (array-dimensions array) :dtype dtype :device 'HIPTensor)))
    (with-pointer-to-vector-data (p storage)
      (check (wf2hip-memcpy-h2d (tensor-device-pointer tensor) p (* (dtype-bytes dtype) (length storage)))))
    tensor))

;; The other directions of convert-tensor-facet / device-as (source/array-converter.lisp:93-151).
;; As with CPUTensor, 'simple-array and 'array expose the whole storage vector in storage order;
;; views and permutations are properties of the tensor, not of its storage.
(defmethod cl-waffe2:convert-tensor-facet ((from HIPTensor) (to (eql 'array)))
  (make-array (cl-waffe2/vm.generic-tensor::original-shape from)
              :element-type (dtype-lisp-type (dtype from))
              :displaced-to (cl-waffe2:convert-tensor-facet from 'simple-array)
              :displaced-index-offset 0))

(defun host-tensor-from (tensor device)
  "A DEVICE (CPUTensor / LispTensor) tensor of TENSOR's original shape over a downloaded copy of
its storage."
  (let ((*using-backend* (list device)))
    (cl-waffe2/vm.generic-tensor::make-tensor-from-vec
     (cl-waffe2/vm.generic-tensor::original-shape tensor) (dtype tensor)
     (cl-waffe2:convert-tensor-facet tensor 'simple-array)
     :order (order tensor))))

(defmethod cl-waffe2:convert-tensor-facet ((from HIPTensor) (to (eql 'cl-waffe2/backends.cpu:CPUTensor)))
  (host-tensor-from from 'cl-waffe2/backends.cpu:CPUTensor))

(defmethod cl-waffe2:convert-tensor-facet ((from HIPTensor) (to (eql 'cl-waffe2/backends.lisp:LispTensor)))
  (host-tensor-from from 'cl-waffe2/backends.lisp:LispTensor))

(defmethod cl-waffe2:convert-tensor-facet ((from AbstractTensor) (to (eql 'HIPTensor)))
  "(device-as tensor 'HIPTensor): one bulk copy of the host tensor's storage vector."
  (if (typep from 'HIPTensor)
      from
      (let* ((storage (cl-waffe2:convert-tensor-facet from 'simple-array))
             (tensor (make-tensor (cl-waffe2/vm.generic-tensor::original-shape from)
                                  :dtype (dtype from) :order (order from) :device 'HIPTensor)))
        (with-pointer-to-vector-data (p storage)
          (check (wf2hip-memcpy-h2d (tensor-device-pointer tensor) p
                                    (* (dtype-bytes (dtype from)) (length storage)))))
        tensor)))
