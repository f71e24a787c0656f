(in-package :cl-user)

(defpackage :cl-waffe2/backends.hip
  (:documentation "HIPTensor: cl-waffe2 tensors whose storage lives on an AMD MI355X and whose
kernels are the hand-written gfx950 kernels of libwaffe2-hip.so.")
  (:use :cl :cffi :cl-waffe2/vm.generic-tensor :cl-waffe2/vm.nodes :cl-waffe2/base-impl :cl-waffe2/vm)
  (:export
   #:HIPTensor
   #:*hip-extension-p*
   #:*hip-device*
   #:try-loading-hip-extension
   #:hip-synchronize
   #:with-sequential-reductions
   #:with-captured-graph
   #:hip-error
   #:!relu-hip #:!leaky-relu-hip #:!sigmoid-hip #:!gelu-hip #:!softmax-hip #:!layer-norm-hip
   #:!sum-hip #:!mean-hip #:!linear-hip #:!causal-softmax-hip #:!attention-hip
   #:softmax-cross-entropy-hip #:unfold-hip))

(in-package :cl-waffe2/backends.hip)

(defparameter *hip-extension-p* nil
  "T once libwaffe2-hip.so is loaded and wf2hip_init succeeded (cf. *simd-extension-p*,
source/backends/cpu/package.lisp:16).")

(defparameter *hip-device* 0 "HIP device ordinal passed to wf2hip_init.")
