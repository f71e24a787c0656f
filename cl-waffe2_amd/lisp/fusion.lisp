;;;; fusion.lisp -- the fused kernels of libwaffe2-hip.so behind cl-waffe2's own extension points.
;;;;
;;;; cl-waffe2 composes !relu, !sigmoid, !gelu, !leaky-relu and !softmax from the arithmetic /
;;;; math / compare nodes (source/nn/activation.lisp:11-159), one kernel and one temporary per
;;;; node.  The library holds each of them as one kernel; this file makes them reachable the way
;;;; the reference intends device-specific fusions to be added:
;;;;   * a define-op node per fused kernel (as Softmax-Cross-Entropy-Node, source/nn/criterion.lisp:90),
;;;;     forward = one library call, backward = the derivative composed from ordinary ! functions
;;;;     and evaluated with proceed, so it runs on the device through the nodes of kernels.lisp
;;;;     (a graph is compiled per backward call: the fused nodes pay off in inference and in
;;;;     forward-heavy training; a defmodel-as cache is the next step);
;;;;   * a define-bypass rule per function (source/vm/nodes/symbolic.lisp:118-131): with HIPTensor
;;;;     in *using-backend*, calls of cl-waffe2/nn:!relu & co. compiled after this file is loaded
;;;;     build the fused node instead ((setf *enable-symbolic-path* nil) switches that off).
;;;; The activation kernels round every step as the node recipe does (bit-identical results);
;;;; the softmax kernel subtracts the row maximum where the recipe subtracts the row mean, which
;;;; is the same function within the tolerance of the path (1e-5 relative).
;;;; Like the rest of this directory the file has not been run: no Common Lisp in the build image.

(in-package :cl-waffe2/backends.hip)

(defconstant +gelu+ 40) (defconstant +relu+ 41) (defconstant +sigmoid+ 42) (defconstant +leaky-relu+ 43)

(defun hip-float-tensor-p (x)
  (and (typep x 'HIPTensor) (eql (dtype x) :float)))

(defun call-composed (function &rest args)
  "The reference's own composition; through funcall so that the bypass does not apply again."
  (apply (symbol-function function) args))

;; ---- activations ---------------------------------------------------------------------------
(define-op (HIP-Activation-Node (self op p derivative)
            :slots ((op :initform 0 :accessor activation-op)
                    (p :initform 0.0 :accessor activation-parameter)
                    (derivative :initform nil :accessor activation-derivative))
            :save-for-backward-names (x)
            :where (X[~] OUT[~] -> OUT[~])
            :documentation "OUT <- f(X) as one kernel (WF2HIP_RELU / SIGMOID / LEAKY_RELU / GELU).
DERIVATIVE is a function of (x) returning df/dx built from ! functions."
            :forward ((self x out)
                      (with-setting-save4bw ((x x))
                        (run-unary (activation-op self) x out (activation-parameter self))))
            :backward ((self dout)
                       (with-reading-save4bw ((x x))
                         ;; the body of a define-op backward runs eagerly (it is the forward of the
                         ;; generated -backward node, source/vm/nodes/static-node.lisp:296-318), so
                         ;; the composed derivative is evaluated here with proceed
                         (values (proceed (!mul dout (funcall (activation-derivative self) x))) nil))))
  (setf (activation-op self) op
        (activation-parameter self) p
        (activation-derivative self) derivative))

(defun fused-activation (x op p derivative)
  (call (HIP-Activation-Node op p derivative)
        x
        (make-input (shape x) nil :dtype (dtype x) :order (order x))))

(defun !relu-hip (x)
  "(!relu x) as one kernel: x * (x > 0 ? 1 : 0)."
  (if (hip-float-tensor-p x)
      (fused-activation x +relu+ 0.0 #'(lambda (x) (A>scal x 0.0)))
      (call-composed 'cl-waffe2/nn:!relu x)))

(defun !leaky-relu-hip (x &key (negative-slope 0.01))
  "(!leaky-relu x :negative-slope s) as one kernel: x * (x >= 0 ? 1 : s)."
  (if (hip-float-tensor-p x)
      (fused-activation x +leaky-relu+ negative-slope
                        #'(lambda (x) (A>=scal x 0.0 :true-then 1.0 :false-then negative-slope)))
      (call-composed 'cl-waffe2/nn:!leaky-relu x :negative-slope negative-slope)))

(defun !sigmoid-hip (x)
  "(!sigmoid x) as one kernel; the derivative s (1 - s) recomputes s through the same node."
  (if (hip-float-tensor-p x)
      (fused-activation x +sigmoid+ 0.0
                        #'(lambda (x)
                            (let ((s (!sigmoid-hip x)))
                              (!mul s (!sub 1 s)))))
      (call-composed 'cl-waffe2/nn:!sigmoid x)))

(defun gelu-derivative (x)
  "d/dx of 0.5 x (1 + tanh u), u = c (x + a x^3): 0.5 (1 + t) + 0.5 x (1 - t^2) c (1 + 3 a x^2)."
  (let* ((c (coerce (sqrt (/ 2.0 pi)) 'single-float))
         (a 0.044715)
         (x2 (!mul x x))
         (u (!mul c (!add x (!mul a (!mul x2 x)))))
         (th (!tanh u))
         (du (!mul c (!add 1 (!mul (* 3 a) x2)))))
    (!add (!mul 0.5 (!add 1 th))
          (!mul (!mul 0.5 x) (!mul (!sub 1 (!mul th th)) du)))))

(defun !gelu-hip (x)
  "(!gelu x), the tanh form of source/nn/activation.lisp:45-66, as one kernel."
  (if (hip-float-tensor-p x)
      (fused-activation x +gelu+ 0.0 #'gelu-derivative)
      (call-composed 'cl-waffe2/nn:!gelu x)))

;; ---- row softmax ---------------------------------------------------------------------------
(define-op (HIP-Softmax-Node (self)
            :save-for-backward-names (y)
            :where (X[rows cols] OUT[rows cols] -> OUT[rows cols])
            :documentation "OUT <- softmax over the last axis of a contiguous matrix, one kernel
(wf2hip_softmax_rows_f32)."
            :forward ((self x out)
                      (ensure-extension)
                      (let ((rows (first (shape x))) (cols (second (shape x))))
                        (check (wf2hip-softmax-rows-f32 rows cols (tensor-device-pointer x) cols
                                                        (tensor-device-pointer out) cols)))
                      (with-setting-save4bw ((y out)) out))
            :backward ((self dout)
                       ;; dx = y * (dy - sum(dy * y) over the row)
                       (with-reading-save4bw ((y y))
                         (let ((dot (!sum (!mul dout y) :axis 1 :keepdims t)))
                           (values (proceed (!mul y (!sub dout dot))) nil))))))

(defun !softmax-hip (x &key (avoid-overflow t) (axis 1))
  "(!softmax x :axis 1) on a contiguous :float matrix as one kernel; anything else takes the
composed recipe."
  (if (and (hip-float-tensor-p x)
           (= (length (shape x)) 2)
           (eql axis 1)
           (every #'numberp (shape x)))
      (let ((x (->contiguous x)))
        (call (HIP-Softmax-Node) x (make-input (shape x) nil :dtype :float :order (order x))))
      (call-composed 'cl-waffe2/nn:!softmax x :avoid-overflow avoid-overflow :axis axis)))

;; ---- LayerNorm over the last axis ------------------------------------------------------------
(define-op (HIP-LayerNorm-Node (self eps)
            :slots ((eps :initform 1.0e-5 :accessor layernorm-eps))
            :where (X[rows cols] G[cols] B[cols] OUT[rows cols] -> OUT[rows cols])
            :documentation "OUT <- (x - mean) / sqrt(var + eps) * g + b per row, one kernel
(wf2hip_layernorm_rows_f32); forward only (use the composed LayerNorm when training)."
            :forward ((self x g b out)
                      (ensure-extension)
                      (check (wf2hip-layernorm-rows-f32 (first (shape x)) (second (shape x))
                                                        (tensor-device-pointer x)
                                                        (tensor-device-pointer g) (tensor-device-pointer b)
                                                        (coerce (layernorm-eps self) 'single-float)
                                                        (tensor-device-pointer out)))
                      out))
  (setf (layernorm-eps self) eps))

(defun !layer-norm-hip (x gamma beta &key (eps 1.0e-5))
  "LayerNorm of every row of the contiguous :float matrix X with scale GAMMA and shift BETA."
  (let ((x (->contiguous x)))
    (call (HIP-LayerNorm-Node eps) x gamma beta
          (make-input (shape x) nil :dtype :float :order (order x)))))

;; ---- bypass rules ----------------------------------------------------------------------------
(define-bypass HIPTensor cl-waffe2/nn:!relu !relu-hip)
(define-bypass HIPTensor cl-waffe2/nn:!leaky-relu !leaky-relu-hip)
(define-bypass HIPTensor cl-waffe2/nn:!sigmoid !sigmoid-hip)
(define-bypass HIPTensor cl-waffe2/nn:!gelu !gelu-hip)
(define-bypass HIPTensor cl-waffe2/nn:!softmax !softmax-hip)
