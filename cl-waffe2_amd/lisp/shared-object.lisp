(in-package :cl-waffe2/backends.hip)

;; Same pattern as cl-waffe2-simd/shared-object.lisp:4-13: load the shared object that sits
;; next to the system, warn and return NIL when that fails.  Unlike CPUTensor there is no
;; lower device to fall back to for tensors that already live on the GPU, so every HIPTensor
;; operation signals an error while *hip-extension-p* is NIL.
;;
;; The library path can be overridden with
;;   (defparameter cl-user::*cl-waffe-config* '((:libwaffe2-hip "/path/to/libwaffe2-hip.so")))
;; following the :libblas convention of source/backends/cpu/package.lisp:51-56.

(defun default-library-pathname ()
  (or (and (boundp 'cl-user::*cl-waffe-config*)
           (second (assoc :libwaffe2-hip (symbol-value 'cl-user::*cl-waffe-config*))))
      (asdf:system-relative-pathname "cl-waffe2-hip" "../libwaffe2-hip.so")))

(defun try-loading-hip-extension (&key (pathname (default-library-pathname)) (device *hip-device*))
  (handler-case
      (progn
        (load-foreign-library pathname)
        (let ((code (foreign-funcall "wf2hip_init" :int device :int)))
          (unless (zerop code)
            (error "wf2hip_init(~a) = ~a: ~a" device code
                   (foreign-funcall "wf2hip_last_error" :string))))
        (setf *hip-extension-p* t))
    (error (c)
      (warn "cl-waffe2 HIP backend is not available: ~a~%Build it with `make -C cl-waffe2_amd/csrc` on a machine with ROCm and an MI355X." c)
      (setf *hip-extension-p* nil))))

(eval-when (:load-toplevel :execute)
  (try-loading-hip-extension))
