;;;; fusion.lisp -- the fused kernels of libwaffe2-hip.so behind cl-waffe2's own extension points.
;;;;
;;;; cl-waffe2 composes !relu, !sigmoid, !gelu, !leaky-relu and !softmax from the arithmetic /
;;;; math / compare nodes (source/nn/activation.lisp:11-159), one kernel and one temporary per
;;;; node.  The library holds each of them as one kernel; this file makes them reachable the way
;;;; the reference intends device-specific fusions to be added:
;;;;   * a define-op node per fused kernel (as Softmax-Cross-Entropy-Node, source/nn/criterion.lisp:90),
;;;;     forward = one library call; backward = one library call too where the library holds the
;;;;     gradient as a kernel (activations, softmax, causal softmax, LayerNorm, attention), otherwise the
;;;;     derivative composed from ordinary ! functions and evaluated with proceed, so it runs on
;;;;     the device through the nodes of kernels.lisp (a graph is compiled per such backward call;
;;;;     a defmodel-as cache is the next step);
;;;;   * a define-bypass rule per function (source/vm/nodes/symbolic.lisp:118-131): with HIPTensor
;;;;     in *using-backend*, calls of cl-waffe2/nn:!relu & co. compiled after this file is loaded
;;;;     build the fused node instead ((setf *enable-symbolic-path* nil) switches that off).
;;;; Also here, on the same two extension points: !sum / !mean as one node (HIP-Sum-Node, bypass rules),
;;;; LayerNorm with its backward, and the nodes behind the 1.06 ms block forward -- product + bias
;;;; (+ GELU) (+ residual) as one launch (HIP-Linear-Node, HIP-Linear-Residual-Node, !linear-hip),
;;;; causal softmax (HIP-Causal-Softmax-Node) and attention as one kernel (HIP-Attention-Node,
;;;; !attention-hip); the GPT-2 example's call sites they replace are named at each function.
;;;; The activation kernels round every step as the node recipe does (bit-identical results);
;;;; the softmax kernel subtracts the row maximum where the recipe subtracts the row mean, which
;;;; is the same function within the tolerance of the path (1e-5 relative).
;;;; Like the rest of this directory the file has not been run: no Common Lisp in the build image.

(in-package :cl-waffe2/backends.hip)

(defconstant +gelu+ 40) (defconstant +relu+ 41) (defconstant +sigmoid+ 42) (defconstant +leaky-relu+ 43)

(defparameter *compose-backward* nil
  "When true the fused nodes differentiate node for node (the compositions this file also holds)
instead of through the library's backward kernels.")

(defun hip-float-tensor-p (x)
  (and (typep x 'HIPTensor) (eql (dtype x) :float)))

(defun fresh-like (x)
  "An uninitialised-content-is-fine :float device tensor of X's shape (every element is written
by the kernel it is handed to)."
  (make-tensor (shape x) :dtype :float :order (order x) :device 'HIPTensor))

(defun eager-contiguous (x)
  "X as a contiguous tensor that starts at its storage, evaluated now: the row kernels take base
pointers.  Inside a backward body, which runs eagerly."
  (proceed (->contiguous x)))

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
Backward: dout f'(x) as one kernel as well (wf2hip_activation_backward_nd, on a copy of dout).
DERIVATIVE, a function of (x) returning df/dx built from ! functions, is the same gradient node
for node; it is what the kernel is checked against and what *compose-backward* selects."
            :forward ((self x out)
                      (with-setting-save4bw ((x x))
                        (run-unary (activation-op self) x out (activation-parameter self))))
            :backward ((self dout)
                       (with-reading-save4bw ((x x))
                         ;; the body of a define-op backward runs eagerly (it is the forward of the
                         ;; generated -backward node, source/vm/nodes/static-node.lisp:296-318)
                         (if *compose-backward*
                             (values (proceed (!mul dout (funcall (activation-derivative self) x))) nil)
                             (let ((dx (proceed (!copy dout))))
                               (ensure-extension)
                               (with-foreign-object (view '(:struct view2))
                                 (fill-view2 view dx x)
                                 (check (wf2hip-activation-backward-nd (activation-op self) view
                                                                       (tensor-device-pointer dx)
                                                                       (tensor-device-pointer x)
                                                                       (coerce (activation-parameter self) 'single-float))))
                               (values dx nil))))))
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
(defun softmax-gradient (y dout scale causal)
  "scale y (dout - sum_j dout y) over the last axis of the saved output Y in one kernel
(wf2hip_softmax_backward_rows_f32).  CAUSAL: rows of square matrices; dout is not read above
the diagonal and the gradient is 0 there."
  (ensure-extension)
  (let* ((dout (eager-contiguous dout))
         (dx (fresh-like y))
         (cols (car (last (shape y))))
         (rows (/ (apply #'* (shape y)) cols)))
    (check (wf2hip-softmax-backward-rows-f32 rows cols (tensor-device-pointer y) cols
                                             (tensor-device-pointer dout) cols
                                             (tensor-device-pointer dx) cols
                                             (coerce scale 'single-float) (if causal cols 0)))
    dx))

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
                         (if *compose-backward*
                             (let ((dot (!sum-hip (!mul dout y) :axis 1 :keepdims t)))
                               (values (proceed (!mul y (!sub dout dot))) nil))
                             (values (softmax-gradient y dout 1.0 nil) nil))))))

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

;; ---- softmax cross entropy --------------------------------------------------------------------
(defun softmax-cross-entropy-gradient (dout z label)
  "(dout (z - label)) / batch, the SubNode, MulNode and DivNode of sce-diff-static
(source/nn/criterion.lisp:82-88) in one kernel; batch is the second-to-last extent of Z."
  (ensure-extension)
  (let ((dout (eager-contiguous dout))
        (dx (fresh-like z)))
    (check (wf2hip-softmax-cross-entropy-backward-f32 (apply #'* (shape z)) (tensor-device-pointer dout) 0
                                                      (tensor-device-pointer z) (tensor-device-pointer label)
                                                      (coerce (car (last (shape z) 2)) 'single-float)
                                                      (tensor-device-pointer dx)))
    dx))

(define-op (HIP-Softmax-Cross-Entropy-Node (self delta)
            :slots ((delta :initform 1e-7 :accessor cross-entropy-delta))
            :save-for-backward-names (z label)
            :where (X[rows cols] Label[rows cols] Z[rows cols] OUT[rows cols] -> OUT[rows cols])
            :documentation "Softmax-Cross-Entropy-Node (source/nn/criterion.lisp:90-126) on contiguous
matrices as one kernel (wf2hip_softmax_cross_entropy_f32): Z <- softmax over the last axis of X, saved
for the backward as the reference saves it, OUT <- -1 (Labels log(Z + delta)).  Backward: one kernel
as well (wf2hip_softmax_cross_entropy_backward_f32)."
            :forward ((self x label z out)
                      (ensure-extension)
                      (check (wf2hip-softmax-cross-entropy-f32 (first (shape x)) (second (shape x))
                                                               (tensor-device-pointer x)
                                                               (tensor-device-pointer label)
                                                               (coerce (cross-entropy-delta self) 'single-float)
                                                               (tensor-device-pointer z)
                                                               (tensor-device-pointer out)))
                      (with-setting-save4bw ((z z) (label label)) out))
            :backward ((self dout)
                       (with-reading-save4bw ((z z) (label label))
                         (if *compose-backward*
                             (values (proceed (!div (!mul dout (!sub z label))
                                                    (make-tensor (car (last (shape z) 2)) :dtype :float)))
                                     nil nil nil)
                             (values (softmax-cross-entropy-gradient dout z label) nil nil nil)))))
  (setf (cross-entropy-delta self) delta))

(defun softmax-cross-entropy-hip (x labels &key (axis 1) (delta 1e-7) (avoid-overflow nil) (reduction t))
  "(softmax-cross-entropy x labels) on contiguous :float matrices with the classes on axis 1 as one
kernel; the reductions stay outside the node (source/nn/criterion.lisp:192-196).  Anything else takes
the reference's node."
  (if (and (hip-float-tensor-p x)
           (hip-float-tensor-p labels)
           (= (length (shape x)) 2)
           (equal (shape x) (shape labels))
           (eql axis 1)
           (every #'numberp (shape x)))
      (let* ((x (->contiguous x))
             (labels (->contiguous labels))
             (out (call (HIP-Softmax-Cross-Entropy-Node delta) x labels
                        (make-input (shape x) nil :dtype :float :order (order x))
                        (make-input (shape x) nil :dtype :float :order (order x)))))
        (case reduction
          (:sum (!sum-hip out))
          (:mean (!mean-hip out))
          (t out)))
      (call-composed 'cl-waffe2/nn:softmax-cross-entropy x labels :axis axis :delta delta
                                                              :avoid-overflow avoid-overflow :reduction reduction)))

;; ---- unfold ------------------------------------------------------------------------------------
(defun unfold-out-size (size pad kernel stride)
  "conv-out-size (source/nn/pool.lisp:10-17) with dilation 1."
  (1+ (floor (- (+ size (* 2 pad)) kernel) stride)))

(defun unfold-gradient (dout input-shape kernel-size stride padding)
  "The gradient of unfold with respect to its input as the reference's nodes derive it: the reshape and
the permutation undone (a copy into [N C k-h k-w h-out w-out]), Col2ImNode's kernel into the padded image,
the interior of the padding."
  (ensure-extension)
  (destructuring-bind (n c h w) input-shape
    (let* ((k-h (first kernel-size)) (k-w (second kernel-size))
           (s-h (first stride)) (s-w (second stride))
           (p-h (first padding)) (p-w (second padding))
           (h-out (unfold-out-size h p-h k-h s-h))
           (w-out (unfold-out-size w p-w k-w s-w))
           (hp (+ h (* 2 p-h) (mod h-out s-h)))
           (wp (+ w (* 2 p-w) (mod w-out s-w)))
           (col (eager-contiguous (!permute (!reshape dout n h-out w-out c k-h k-w) (torch-order 0 3 4 5 1 2))))
           (padded (make-tensor (list n c hp wp) :dtype :float :order (order dout) :device 'HIPTensor)))
      (check (wf2hip-col2im-f32 (tensor-device-pointer col) n c hp wp h-out w-out k-h k-w p-h p-w s-h s-w 1 1
                                (tensor-device-pointer padded)))
      (if (and (= hp h) (= wp w))
          padded
          (eager-contiguous (view padded t t (list p-h (+ p-h h)) (list p-w (+ p-w w))))))))

(define-op (HIP-Unfold-Node (self kernel-size stride padding)
            :slots ((kernel-size :initform nil :accessor unfold-kernel-size)
                    (stride :initform nil :accessor unfold-stride)
                    (padding :initform nil :accessor unfold-padding)
                    (input-shape :initform nil :accessor unfold-input-shape))
            :where (X[N C H W] OUT[rows cols] -> OUT[rows cols])
            :documentation "OUT[(N h-out w-out) (C k-h k-w)] <- unfold of the contiguous image X with dilation 1
(source/nn/im2col.lisp:51-95): the padding, Im2ColNode, the permutation and the reshape as one kernel
(wf2hip_unfold_f32), bit for bit the matrix the composition leaves.  Backward: the reference's own."
            :forward ((self x out)
                      (ensure-extension)
                      (setf (unfold-input-shape self) (copy-list (shape x)))
                      (destructuring-bind (n c h w) (shape x)
                        (check (wf2hip-unfold-f32 n c h w
                                                  (first (unfold-kernel-size self)) (second (unfold-kernel-size self))
                                                  (first (unfold-stride self)) (second (unfold-stride self))
                                                  (first (unfold-padding self)) (second (unfold-padding self))
                                                  (tensor-device-pointer x) (tensor-device-pointer out))))
                      out)
            :backward ((self dout)
                       (values (unfold-gradient dout (unfold-input-shape self) (unfold-kernel-size self)
                                                (unfold-stride self) (unfold-padding self))
                               nil)))
  (setf (unfold-kernel-size self) kernel-size
        (unfold-stride self) stride
        (unfold-padding self) padding))

(defun unfold-hip (input dilation kernel-size stride padding)
  "(unfold input dilation kernel-size stride padding) on a :float device image of static shape with
dilation 1 as one kernel; anything else takes the reference's composition."
  (if (and (hip-float-tensor-p input)
           (= (length (shape input)) 4)
           (every #'numberp (shape input))
           (equal dilation '(1 1))
           (every #'integerp (append kernel-size stride padding)))
      (destructuring-bind (n c h w) (shape input)
        (let ((h-out (unfold-out-size h (first padding) (first kernel-size) (first stride)))
              (w-out (unfold-out-size w (second padding) (second kernel-size) (second stride))))
          (call (HIP-Unfold-Node kernel-size stride padding)
                (->contiguous input)
                (make-input (list (* n h-out w-out) (* c (first kernel-size) (second kernel-size))) nil
                            :dtype :float :order (order input)))))
      (call-composed 'cl-waffe2/nn:unfold input dilation kernel-size stride padding)))

;; ---- LayerNorm over the last axis ------------------------------------------------------------
(defun layer-norm-gradients (x g dout eps)
  "Gradients of y = (x - u) / sqrt(s + eps) * g + b per row (source/nn/norms.lisp:72-82) from the
saved input: with xh = (x - u) rstd and dyh = dout g,
  dx = rstd (dyh - mean(dyh) - xh mean(dyh xh)),  dg = sum over rows of dout xh,  db = sum over rows of dout.
Composed from ! functions (!mean and !sum are one node each on the device)."
  (let* ((u    (!mean-hip x :axis -1 :keepdims t))
         (xc   (!sub x u))
         (s    (!mean-hip (!mul xc xc) :axis -1 :keepdims t))
         (rstd (!div 1 (!sqrt (!add (->contiguous s) eps))))
         (xh   (!mul xc rstd))
         (dyh  (!mul dout (!flexible g)))
         (m1   (!mean-hip dyh :axis -1 :keepdims t))
         (m2   (!mean-hip (!mul dyh xh) :axis -1 :keepdims t))
         (dx   (!mul rstd (!sub (!sub dyh m1) (!mul xh m2))))
         (dg   (!sum-hip (!mul dout xh) :axis 0))
         (db   (!sum-hip dout :axis 0)))
    (values dx dg db)))

(defun layer-norm-gradients-fused (x g dout eps)
  "The same three gradients from one row kernel and two small folds (wf2hip_layernorm_backward_f32;
rows beyond 8192 columns in pieces over several workgroups)."
  (ensure-extension)
  (let* ((dout (eager-contiguous dout))
         (rows (first (shape x)))
         (cols (second (shape x)))
         (dx (fresh-like x))
         (dg (fresh-like g))
         (db (fresh-like g)))
    (check (wf2hip-layernorm-backward-f32 rows cols (tensor-device-pointer x) (tensor-device-pointer g)
                                          (tensor-device-pointer dout) (coerce eps 'single-float)
                                          (tensor-device-pointer dx) (tensor-device-pointer dg)
                                          (tensor-device-pointer db)))
    (values dx dg db)))

(define-op (HIP-LayerNorm-Node (self eps)
            :slots ((eps :initform 1.0e-5 :accessor layernorm-eps))
            :save-for-backward-names (x g)
            :where (X[rows cols] G[cols] B[cols] OUT[rows cols] -> OUT[rows cols])
            :documentation "OUT <- (x - mean) / sqrt(var + eps) * g + b per row, one kernel
(wf2hip_layernorm_rows_f32).  Backward: the three gradients from the saved input by
wf2hip_layernorm_backward_f32 (layer-norm-gradients-fused), or composed from nodes
(layer-norm-gradients) under *compose-backward*."
            :forward ((self x g b out)
                      (ensure-extension)
                      (check (wf2hip-layernorm-rows-f32 (first (shape x)) (second (shape x))
                                                        (tensor-device-pointer x)
                                                        (tensor-device-pointer g) (tensor-device-pointer b)
                                                        (coerce (layernorm-eps self) 'single-float)
                                                        (tensor-device-pointer out)))
                      (with-setting-save4bw ((x x) (g g)) out))
            :backward ((self dout)
                       (with-reading-save4bw ((x x) (g g))
                         (if *compose-backward*
                             (multiple-value-bind (dx dg db) (layer-norm-gradients x g dout (layernorm-eps self))
                               (values (proceed dx)
                                       (proceed (!reshape dg (second (shape x))))
                                       (proceed (!reshape db (second (shape x))))
                                       nil))
                             (multiple-value-bind (dx dg db)
                                 (layer-norm-gradients-fused x g dout (layernorm-eps self))
                               (values dx dg db nil))))))
  (setf (layernorm-eps self) eps))

(defun !layer-norm-hip (x gamma beta &key (eps 1.0e-5))
  "LayerNorm over the last axis of the :float tensor X with scale GAMMA and shift BETA: what
LayerNorm-Revisit (examples/gpt-2/utils.lisp:114-127) and LayerNorm2D over one axis
(source/nn/norms.lisp:72-82) compose from ten nodes.  Leading axes are folded into rows."
  (let* ((cols (car (last (shape x))))
         (x2 (!reshape (->contiguous x) t cols))
         (y (call (HIP-LayerNorm-Node eps) x2 gamma beta
                  (make-input (shape x2) nil :dtype :float :order (order x)))))
    (apply #'!reshape y (shape x))))

;; ---- !sum / !mean as one node -------------------------------------------------------------------
(define-op (HIP-Sum-Node (self divisor)
            :slots ((divisor :initform 1.0 :accessor sum-divisor))
            :where (OUT[~] X[~] -> OUT[~])
            :documentation "OUT <- (sum of X over the axes on which OUT is viewed (:broadcast n)) / divisor,
overwriting OUT: one node for the A*=scal by 0, the A+=B into the broadcast view and the !div of
!sum / !mean (source/base-impl/reduction.lisp:5-136), with the bits of that composition
(wf2hip_sum_nd).  Backward: nothing flows to the overwritten OUT; X receives the gradient of the
broadcast view, which has X's shape, divided by the divisor."
            :forward ((self out x)
                      (ensure-extension)
                      (with-foreign-object (view '(:struct view2))
                        (fill-view2 view out x)
                        (check (wf2hip-sum-nd view (tensor-device-pointer out) (tensor-device-pointer x)
                                              (coerce (sum-divisor self) 'single-float))))
                      out)
            :backward ((self dout)
                       (values nil
                               (if (= (sum-divisor self) 1)
                                   dout
                                   (proceed (!div dout (sum-divisor self)))))))
  (setf (sum-divisor self) divisor))

(defun !sum-hip (tensor &key (axis t) (-> nil) (keepdims nil) (div-by nil))
  "(!sum tensor :axis .. :-> .. :keepdims ..) as one node on :float device tensors; same arguments as
cl-waffe2/base-impl:!sum, whose argument handling (source/base-impl/reduction.lisp:31-60) is
repeated here.  A DIV-BY that is not a number (the lazily multiplied scalar tensor !mean passes)
takes the composed route; !mean-hip passes the count as a number."
  (if (and (hip-float-tensor-p tensor)
           (or (null ->) (hip-float-tensor-p ->))
           (or (null div-by) (numberp div-by)))
      (let* ((shape (copy-list (shape tensor)))
             (dims (length shape))
             (view-args (make-list dims :initial-element t)))
        (flet ((reduce-axis (ax)
                 (let ((ax (if (< ax 0) (+ ax dims) ax)))
                   (setf (nth ax view-args) `(:broadcast ,(nth ax shape))
                         (nth ax shape) 1))))
          (typecase axis
            (fixnum (reduce-axis axis))
            (list (mapc #'reduce-axis axis))
            (t (dotimes (ax dims) (reduce-axis ax)))))
        (let ((out (or -> (make-input shape nil :dtype (dtype tensor) :order (order tensor)))))
          (assert (equal (shape out) shape) ()
                  "!sum: Assertion Failed because the given out's shape is ~a, but expected: ~a" (shape out) shape)
          (multiple-value-bind (out* reverser) (apply #'!view out view-args)
            (let ((result (call (HIP-Sum-Node (or div-by 1.0)) out* tensor)))
              (if keepdims
                  result
                  (apply #'!view result reverser))))))
      (call-composed 'cl-waffe2/base-impl:!sum tensor :axis axis :-> -> :keepdims keepdims :div-by div-by)))

(defun !mean-hip (tensor &key (axis t) (-> nil) (keepdims nil))
  "(!mean tensor ..) as one node: the element count is known from the shape when it is static."
  (if (and (hip-float-tensor-p tensor) (every #'numberp (shape tensor)))
      (let* ((dims (length (shape tensor)))
             (axes (typecase axis
                     (fixnum (list axis))
                     (list axis)
                     (t (loop for i below dims collect i))))
             (count (reduce #'* (mapcar #'(lambda (ax) (nth (if (< ax 0) (+ ax dims) ax) (shape tensor))) axes))))
        (!sum-hip tensor :axis axis :-> -> :keepdims keepdims :div-by (coerce count 'single-float)))
      (call-composed 'cl-waffe2/base-impl:!mean tensor :axis axis :-> -> :keepdims keepdims)))

;; ---- linear layers: product + bias (+ GELU) (+ residual) in the product's epilogue --------------
(defun fill-matmul-desc (desc rows n k activation bias residual)
  (macrolet ((field (name) `(foreign-slot-value desc '(:struct matmul-desc) ',name)))
    (setf (field trans-a) 0 (field trans-b) 0
          (field activation) (ecase activation ((nil :none) 0) (:gelu 1))
          (field causal) 0
          (field m) rows (field n) n (field k) k
          (field lda) k (field ldb) n (field ldc) n
          (field batch) 1 (field batch2) 1
          (field stride-a) 0 (field stride-a2) 0 (field stride-b) 0 (field stride-b2) 0
          (field stride-c) 0 (field stride-c2) 0
          (field bias) (if bias (tensor-device-pointer bias) (null-pointer))
          (field residual) (if residual (tensor-device-pointer residual) (null-pointer))
          (field ld-residual) n (field stride-residual) 0 (field stride-residual2) 0
          (field alpha) 1.0 (field reserved) 0))
  desc)

(defun run-linear (x w b residual out activation)
  "OUT[rows n] <- act(X[rows k] . W[k n] + B[n]) + RESIDUAL[rows n], one launch (wf2hip_matmul_fused)."
  (ensure-extension)
  (with-foreign-object (desc '(:struct matmul-desc))
    (fill-matmul-desc desc (first (shape x)) (second (shape w)) (second (shape x)) activation b residual)
    (check (wf2hip-matmul-fused desc (tensor-device-pointer x) (tensor-device-pointer w)
                                (tensor-device-pointer out))))
  out)

(defun linear-gradients (x w b dout activation)
  "dX = dZ W^T, dW = X^T dZ, dB = column sums of dZ, with dZ = dOUT for a plain layer and
dOUT gelu'(Z), Z = X W + B recomputed, for a GELU layer."
  (let* ((dz (cond ((not (eql activation :gelu)) dout)
                   (*compose-backward*
                    (!mul dout (gelu-derivative (!add (!matmul x w) (!flexible b)))))
                   (t
                    ;; Z through the product with the bias in its epilogue, dOUT gelu'(Z) in one kernel
                    (let ((z (run-linear x w b nil (fresh-like dout) nil))
                          (dz (proceed (!copy dout))))
                      (with-foreign-object (view '(:struct view2))
                        (fill-view2 view dz z)
                        (check (wf2hip-activation-backward-nd +gelu+ view (tensor-device-pointer dz)
                                                              (tensor-device-pointer z) 0.0)))
                      dz)))))
    (values (!matmul dz (!t w))
            (!matmul (!t x) dz)
            (!reshape (!sum-hip dz :axis 0) (second (shape w))))))

(define-op (HIP-Linear-Node (self activation)
            :slots ((activation :initform nil :accessor linear-activation))
            :save-for-backward-names (x w b)
            :where (X[rows k] W[k n] B[n] OUT[rows n] -> OUT[rows n])
            :documentation "OUT <- act(X . W + B): MatMulNode, the AddNode of the bias and the
activation (ACTIVATION nil or :gelu, the tanh form of source/nn/activation.lisp:45-66) as one
product with an epilogue."
            :forward ((self x w b out)
                      (with-setting-save4bw ((x x) (w w) (b b))
                        (run-linear x w b nil out (linear-activation self))))
            :backward ((self dout)
                       (with-reading-save4bw ((x x) (w w) (b b))
                         (multiple-value-bind (dx dw db) (linear-gradients x w b dout (linear-activation self))
                           (values (proceed dx) (proceed dw) (proceed db) nil)))))
  (setf (linear-activation self) activation))

(define-op (HIP-Linear-Residual-Node (self)
            :save-for-backward-names (x w)
            :where (X[rows k] W[k n] B[n] R[rows n] OUT[rows n] -> OUT[rows n])
            :documentation "OUT <- X . W + B + R: the projection that closes a residual branch
(examples/gpt-2/model.lisp:121-123,134-137) as one product."
            :forward ((self x w b r out)
                      (with-setting-save4bw ((x x) (w w))
                        (run-linear x w b r out nil)))
            :backward ((self dout)
                       (with-reading-save4bw ((x x) (w w))
                         (values (proceed (!matmul dout (!t w)))
                                 (proceed (!matmul (!t x) dout))
                                 (proceed (!reshape (!sum-hip dout :axis 0) (second (shape w))))
                                 dout
                                 nil)))))

(defun !linear-hip (x w b &key (activation nil) (residual nil))
  "act(X W + B) + RESIDUAL for X[~ k], W[k n], B[n] on :float device tensors: replaces
  (asnode #'!matmul w) (asnode #'!add (%transform b[i] -> [~ i])) [(asnode #'!gelu)] [(!add x ..)]
of examples/gpt-2/model.lisp:109-137 by one node.  Leading axes of X are folded into rows."
  (let* ((k (car (last (shape x))))
         (n (second (shape w)))
         (x2 (!reshape (->contiguous x) t k))
         (out (make-input (list (first (shape x2)) n) nil :dtype :float :order (order x)))
         (y (if residual
                (progn
                  (assert (null activation) () "!linear-hip: a residual closes a branch without activation")
                  (call (HIP-Linear-Residual-Node) x2 (->contiguous w) b
                        (!reshape (->contiguous residual) t n) out))
                (call (HIP-Linear-Node activation) x2 (->contiguous w) b out))))
    (apply #'!reshape y `(,@(butlast (shape x)) ,n))))

;; ---- causal softmax and attention -----------------------------------------------------------------
(define-op (HIP-Causal-Softmax-Node (self scale)
            :slots ((scale :initform 1.0 :accessor softmax-scale))
            :save-for-backward-names (y)
            :where (X[matrices seq seq2] OUT[matrices seq seq2] -> OUT[matrices seq seq2])
            :documentation "OUT[m, i, :] <- softmax over j <= i of scale X[m, i, j], 0 above the diagonal:
the MulNode by the scale, the AddNode of the mask and !softmax of causal attention as one kernel
(wf2hip_causal_softmax_f32) on contiguous square matrices."
            :forward ((self x out)
                      (ensure-extension)
                      (check (wf2hip-causal-softmax-f32 (first (shape x)) (second (shape x))
                                                        (tensor-device-pointer x) (tensor-device-pointer out)
                                                        (coerce (softmax-scale self) 'single-float)))
                      (with-setting-save4bw ((y out)) out))
            :backward ((self dout)
                       ;; dx = scale y (dy - sum_j dy y); y is 0 above the diagonal, so is dx
                       (with-reading-save4bw ((y y))
                         (if *compose-backward*
                             (let ((dot (!sum-hip (!mul dout y) :axis -1 :keepdims t)))
                               (values (proceed (!mul (softmax-scale self) (!mul y (!sub dout dot)))) nil))
                             (values (softmax-gradient y dout (softmax-scale self) t) nil)))))
  (setf (softmax-scale self) scale))

(defun !causal-softmax-hip (scores &key (scale 1.0))
  "Causal softmax of SCORES[~ seq seq] (any leading axes) times SCALE."
  (let* ((seq (car (last (shape scores))))
         (x (!reshape (->contiguous scores) t seq seq))
         (y (call (HIP-Causal-Softmax-Node scale) x
                  (make-input (shape x) nil :dtype :float :order (order scores)))))
    (apply #'!reshape y (shape scores))))

(defun fill-attention-desc (desc q k v out scale causal)
  (macrolet ((field (name) `(foreign-slot-value desc '(:struct attention-desc) ',name)))
    (destructuring-bind (batch heads seq head-dim) (shape q)
      (setf (field batch) batch (field heads) heads (field seq) seq (field head-dim) head-dim
            (field scale) (coerce scale 'single-float)
            (field causal) (if causal 1 0))
      (let ((offsets
              (loop for tensor in (list q k v out)
                    for slot in '(q-stride k-stride v-stride o-stride)
                    collect (multiple-value-bind (extents strides offset) (matrix-geometry tensor)
                              (declare (ignore extents))
                              (dotimes (axis 3)
                                (setf (mem-aref (foreign-slot-pointer desc '(:struct attention-desc) slot) :int64 axis)
                                      (nth axis strides)))
                              offset))))
        offsets))))

(define-op (HIP-Attention-Node (self scale causal)
            :slots ((scale :initform 1.0 :accessor attention-scale)
                    (causal :initform nil :accessor attention-causal))
            :save-for-backward-names (q k v o lse)
            :where (Q[batch heads seq dim] K[batch heads seq dim] V[batch heads seq dim] OUT[batch heads seq dim]
                    -> OUT[batch heads seq dim])
            :documentation "OUT <- softmax(scale Q K^T [+ causal mask]) V per (batch, head) in one kernel that
never forms the (seq, seq) score matrices (wf2hip_attention_forward_f32; heads up to 64 wide).  The operands
may be strided windows of a fused projection (last axis contiguous).  The forward also keeps, per query, the
base-2 logarithm of its row sum; with it the backward is one library call as well
(wf2hip_attention_backward_f32: D = sum dO O per query, dQ with queries resident, dK and dV with keys resident;
no (seq, seq) tensor either).  *compose-backward* selects the composition instead, with the probabilities
recomputed: dV = P^T dO, dP = dO V^T, dS = scale P (dP - sum_j dP P), dQ = dS K, dK = dS^T Q."
            :forward ((self q k v out)
                      (ensure-extension)
                      (let ((lse (make-tensor (butlast (shape q)) :dtype :float :order (order q) :device 'HIPTensor)))
                        (with-foreign-object (desc '(:struct attention-desc))
                          (destructuring-bind (oq ok ov oo)
                              (fill-attention-desc desc q k v out (attention-scale self) (attention-causal self))
                            (check (wf2hip-attention-forward-f32 desc
                                                                 (tensor-device-pointer q oq) (tensor-device-pointer k ok)
                                                                 (tensor-device-pointer v ov) (tensor-device-pointer out oo)
                                                                 (tensor-device-pointer lse)))))
                        (with-setting-save4bw ((q q) (k k) (v v) (o out) (lse lse)) out)))
            :backward ((self dout)
                       (with-reading-save4bw ((q q) (k k) (v v) (o o) (lse lse))
                         (let ((scale (attention-scale self)))
                           (if *compose-backward*
                               (let* ((s (!matmul q (!t k)))
                                      (p (if (attention-causal self)
                                             (!causal-softmax-hip s :scale scale)
                                             (!softmax-hip (!reshape (!mul scale s) t (car (last (shape s)))))))
                                      (p (apply #'!reshape p (shape s)))
                                      (dv (!matmul (!t p) dout))
                                      (dp (!matmul dout (!t v)))
                                      (ds (!mul scale (!mul p (!sub dp (!sum-hip (!mul dp p) :axis -1 :keepdims t)))))
                                      (dq (!matmul ds k))
                                      (dk (!matmul (!t ds) q)))
                                 (values (proceed dq) (proceed dk) (proceed dv) nil))
                               ;; the library addresses dO like O and dQ, dK, dV like Q, K, V: contiguous
                               ;; operands (copies of windows, 25 MB each at the block's shape) and fresh
                               ;; contiguous gradients share one set of strides
                               (let* ((q (eager-contiguous q)) (k (eager-contiguous k)) (v (eager-contiguous v))
                                      (o (eager-contiguous o)) (dout (eager-contiguous dout))
                                      (dq (fresh-like q)) (dk (fresh-like q)) (dv (fresh-like q)))
                                 (ensure-extension)
                                 (with-foreign-object (desc '(:struct attention-desc))
                                   (fill-attention-desc desc q k v o scale (attention-causal self))
                                   (check (wf2hip-attention-backward-f32
                                           desc (tensor-device-pointer q) (tensor-device-pointer k)
                                           (tensor-device-pointer v) (tensor-device-pointer o)
                                           (tensor-device-pointer dout) (tensor-device-pointer lse)
                                           (tensor-device-pointer dq) (tensor-device-pointer dk)
                                           (tensor-device-pointer dv))))
                                 (values dq dk dv nil)))))))
  (setf (attention-scale self) scale
        (attention-causal self) causal))

(defun !attention-hip (q k v &key (scale nil) (causal nil))
  "softmax(SCALE Q K^T) V for Q, K, V shaped (batch heads seq head-dim); SCALE defaults to
1 / sqrt(head-dim).  Replaces the !matmul / !div / !softmax / !matmul chain of SelfAttention
(examples/gpt-2/utils.lisp:222-243; the example divides by the sequence length and applies no mask:
pass :scale (/ 1.0 seq) for its numbers, :causal t for a decoder)."
  (let ((scale (or scale (/ 1.0 (sqrt (coerce (car (last (shape q))) 'single-float))))))
    (call (HIP-Attention-Node scale causal) q k v
          (make-input (shape q) nil :dtype :float :order (order q)))))

;; ---- bypass rules ----------------------------------------------------------------------------
(define-bypass HIPTensor cl-waffe2/nn:!relu !relu-hip)
(define-bypass HIPTensor cl-waffe2/nn:!leaky-relu !leaky-relu-hip)
(define-bypass HIPTensor cl-waffe2/nn:!sigmoid !sigmoid-hip)
(define-bypass HIPTensor cl-waffe2/nn:!gelu !gelu-hip)
(define-bypass HIPTensor cl-waffe2/nn:!softmax !softmax-hip)
(define-bypass HIPTensor cl-waffe2/nn:softmax-cross-entropy softmax-cross-entropy-hip)
(define-bypass HIPTensor cl-waffe2/nn:unfold unfold-hip)
(define-bypass HIPTensor cl-waffe2/base-impl:!sum !sum-hip)
(define-bypass HIPTensor cl-waffe2/base-impl:!mean !mean-hip)
