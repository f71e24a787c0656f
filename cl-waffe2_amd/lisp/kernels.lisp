(in-package :cl-waffe2/backends.hip)

;; define-impl-op registrations: closures that read the tensors' views at run time and make
;; ONE library call per node.  The CPU backend instead generates loops with call-with-view at
;; graph-construction time and compiles them per shape
;; (source/backends/cpu/arithmetic.lisp:32-144); ExptNode-CPUTensor already uses the run-time
;; form (source/backends/cpu/mathematics.lisp:55-76), which is the one followed here.

(defun float-or-double-p (dtype &rest more)
  "reject-p of the nodes the SIMD extension / BLAS serve for :float and :double only."
  (declare (ignore more))
  (not (member dtype '(:float :double))))

(defun only-float-p (dtype &rest more)
  "reject-p: everything but :float falls through to the next device in *using-backend*
(cf. supported-dtypes-are, source/vm/nodes/utils.lisp:71-93)."
  (declare (ignore more))
  (not (eql dtype :float)))

(defun fill-view2 (view a b)
  "Writes the iteration space shared by tensors A and B into the foreign struct VIEW: per axis
the visible extent and each tensor's effective stride (storage stride x view step, 0 when the
axis is (:broadcast n)), plus the start offsets (tensor-initial-offset + stride x range-nth 0).
These are exactly the numbers call-with-view computes per axis
(source/vm/generic-tensor/call-with-view.lisp:120-137,168-195)."
  (let ((rank (length (shape a))))
    (assert (<= 1 rank 8) () "HIPTensor kernels take rank 1..8 tensors, got ~a" rank)
    (setf (foreign-slot-value view '(:struct view2) 'rank) rank)
    (flet ((geometry (tensor stride-slot)
             (let ((offset (tensor-initial-offset tensor)))
               (loop for axis from 0
                     for extent in (shape tensor)
                     for stride in (tensor-stride tensor)
                     for subscript in (tensor-view tensor)
                     for range = (subscript-range subscript)
                     for first = (wf/iter:range-nth range 0)
                     do (setf (mem-aref (foreign-slot-pointer view '(:struct view2) 'shape) :int64 axis)
                              (cl-waffe2/vm:maybe-observe-axis extent))
                        (incf offset (* stride first))
                        (setf (mem-aref (foreign-slot-pointer view '(:struct view2) stride-slot) :int64 axis)
                              (if (subscript-broadcast subscript)
                                  0
                                  (* stride (- (wf/iter:range-nth range 1) first)))))
               offset)))
      (setf (foreign-slot-value view '(:struct view2) 'off-a) (geometry a 'stride-a)
            (foreign-slot-value view '(:struct view2) 'off-b) (geometry b 'stride-b)))
    view))

(defun run-binary (op x y)
  "X <- X op Y over both views in one call; :float through the kernels of the hot path, any
other dtype through the typed entry point (the CPU backend dispatches on dtype inside its impl
too, source/backends/cpu/arithmetic.lisp:65-123)."
  (ensure-extension)
  (unless (eql (dtype x) (dtype y))
    (error "HIPTensor: ~a and ~a operands in one node" (dtype x) (dtype y)))
  (with-foreign-object (view '(:struct view2))
    (fill-view2 view x y)
    (if (eql (dtype x) :float)
        (check (wf2hip-binary-nd op view (tensor-device-pointer x) (tensor-device-pointer y)))
        (check (wf2hip-binary-nd-typed (nth-value 2 (dtype-info (dtype x))) op view
                                       (tensor-device-pointer x) (tensor-device-pointer y)))))
  x)

(defun run-unary (op x out &optional (p 0.0))
  ":float through the kernels of the hot path, :double through the typed entry point (the SIMD
extension has both, source/backends/cpu/mathematics.lisp:8-76)."
  (ensure-extension)
  (with-foreign-object (view '(:struct view2))
    (fill-view2 view x out)
    (if (eql (dtype x) :float)
        (check (wf2hip-unary-nd op view (tensor-device-pointer x) (tensor-device-pointer out)
                                (coerce p 'single-float)))
        (check (wf2hip-unary-nd-typed (nth-value 2 (dtype-info (dtype x))) op view
                                      (tensor-device-pointer x) (tensor-device-pointer out)
                                      (coerce p 'double-float)))))
  out)

;; X <- X op Y, returns X (:where A[~] B[~] -> A[~], source/base-impl/arithmetic.lisp:57-103).
;; A stride-0 destination axis -- how !sum and !mean arrive (base-impl/reduction.lisp:5-79) --
;; is reduced in parallel by the library.
(macrolet ((define-arith (node op)
             `(define-impl-op (,node :device HIPTensor)
                              :forward ((self x y) (declare (ignore self)) (run-binary ,op x y)))))
  (define-arith AddNode +add+)
  (define-arith SubNode +sub+)
  (define-arith MulNode +mul+)
  (define-arith DivNode +div+))

;; X <- Y (source/base-impl/fundamental.lisp:9-43).  Without this impl every !copy on a device
;; tensor would fall through to CPUTensor's scopy on a device handle.
(define-impl-op (MoveTensorNode :device HIPTensor)
                :forward ((self x y)
                          (if (cl-waffe2/base-impl::movetensor-ignore-me self)
                              y
                              (run-binary +move+ x y))))

;; OUT <- f(X) (:where X[~] OUT[~] -> OUT[~], source/base-impl/mathematics.lisp:13-120)
(macrolet ((define-math (node op)
             `(define-impl-op (,node :device HIPTensor :reject-p #'float-or-double-p)
                              :forward ((self x out) (declare (ignore self)) (run-unary ,op x out)))))
  (define-math SinNode +sin+)
  (define-math CosNode +cos+)
  (define-math TanhNode +tanh+)
  (define-math LogENode +log+)
  (define-math ExpNode +exp+)
  (define-math SqrtNode +sqrt+)
  (define-math AbsNode +abs+)
  (define-math TanNode +tan+)
  (define-math ASinNode +asin+)
  (define-math ACosNode +acos+)
  (define-math ATanNode +atan+)
  (define-math SinHNode +sinh+)
  (define-math CosHNode +cosh+)
  (define-math Log2Node +log2+)
  (define-math Log10Node +log10+)
  (define-math Log1pNode +log1p+)
  ;; The CPU backend has no impl for these five and leaves them to LispTensor
  ;; (source/backends/lisp/mathematics.lisp:30), whose kernels aref the storage vector: with
  ;; HIPTensor first in *using-backend* they would be handed a device handle.  !abs's backward
  ;; multiplies by !sign (source/base-impl/mathematics.lisp:125-131).
  (define-math SignNode +sign+)
  (define-math SquareNode +square+)
  (define-math ASinHNode +asinh+)
  (define-math ACosHNode +acosh+)
  (define-math ATanHNode +atanh+))

;; OUT <- X^N with N a host ScalarTensor (source/base-impl/mathematics.lisp:267-303)
(define-impl-op (ExptNode :device HIPTensor :reject-p #'float-or-double-p)
                :forward ((self x out n)
                          (declare (ignore self))
                          (run-unary +pow+ x out (tensor-vec n))))

;; OUT <- (X cond scal) ? then : else and OUT <- (X cond Y) ? then : else
;; (source/base-impl/logical.lisp:12-62).  Like the CPU backend's SIMD path
;; (source/backends/cpu/logical.lisp:3-84) only the predicates < <= > >= = have a kernel; any
;; other condition is rejected so that the node falls through to the next device.
(defun condition->op (condition)
  (cond ((eql condition #'<) +lt+) ((eql condition #'<=) +le+) ((eql condition #'>) +gt+)
        ((eql condition #'>=) +ge+) ((eql condition #'=) +eq+)))

(defun where-reject-p (&rest args &key &allow-other-keys)
  "Where-Operation-Node carries its predicate and scalar in :compiler-info (logical.lisp:162-194)."
  (let ((info (car (last args))))
    (not (and (consp info) (condition->op (car info))))))

(defun compare-reject-p (&rest args)
  (not (condition->op (car args))))

(define-impl-op (Where-Operation-Node :device HIPTensor :reject-p #'where-reject-p)
                :forward ((self x out)
                          (ensure-extension)
                          (destructuring-bind (condition scal &rest more)
                              (cl-waffe2/base-impl::logical-compiler-info self)
                            (declare (ignore more))
                            (with-foreign-object (view '(:struct view2))
                              (fill-view2 view x out)
                              ;; every dtype, as the CPU impl (backends/cpu/logical.lisp:37-60)
                              (if (eql (dtype x) :float)
                                  (check (wf2hip-where-nd
                                          (condition->op condition) view
                                          (tensor-device-pointer x) (tensor-device-pointer out)
                                          (coerce scal 'single-float)
                                          (coerce (cl-waffe2/base-impl::logical-true-then self) 'single-float)
                                          (coerce (cl-waffe2/base-impl::logical-false-then self) 'single-float)))
                                  (check (wf2hip-where-nd-typed
                                          (nth-value 2 (dtype-info (dtype x))) (condition->op condition) view
                                          (tensor-device-pointer x) (tensor-device-pointer out)
                                          (coerce scal 'double-float)
                                          (coerce (cl-waffe2/base-impl::logical-true-then self) 'double-float)
                                          (coerce (cl-waffe2/base-impl::logical-false-then self) 'double-float))))))
                          out))

(defun fill-view3 (view x y out)
  "Like fill-view2 for three tensors: X and Y go through a view2 each paired with OUT."
  (with-foreign-objects ((xo '(:struct view2)) (yo '(:struct view2)))
    (fill-view2 xo x out)
    (fill-view2 yo y out)
    (setf (foreign-slot-value view '(:struct view3) 'rank) (foreign-slot-value xo '(:struct view2) 'rank))
    (dotimes (axis (length (shape out)))
      (flet ((copy-slot (to from-view from)
               (setf (mem-aref (foreign-slot-pointer view '(:struct view3) to) :int64 axis)
                     (mem-aref (foreign-slot-pointer from-view '(:struct view2) from) :int64 axis))))
        (copy-slot 'shape xo 'shape)
        (copy-slot 'stride-a xo 'stride-a)
        (copy-slot 'stride-b yo 'stride-a)
        (copy-slot 'stride-c xo 'stride-b)))
    (setf (foreign-slot-value view '(:struct view3) 'off-a) (foreign-slot-value xo '(:struct view2) 'off-a)
          (foreign-slot-value view '(:struct view3) 'off-b) (foreign-slot-value yo '(:struct view2) 'off-a)
          (foreign-slot-value view '(:struct view3) 'off-c) (foreign-slot-value xo '(:struct view2) 'off-b)))
  view)

(define-impl-op (Compare-Operation-Node :device HIPTensor :reject-p #'compare-reject-p)
                :forward ((self x y out)
                          (ensure-extension)
                          (with-foreign-object (view '(:struct view3))
                            (fill-view3 view x y out)
                            (if (eql (dtype x) :float)
                                (check (wf2hip-compare-nd
                                        (condition->op (cl-waffe2/base-impl::logical-condition self)) view
                                        (tensor-device-pointer x) (tensor-device-pointer y)
                                        (tensor-device-pointer out)
                                        (coerce (cl-waffe2/base-impl::logical-true-then self) 'single-float)
                                        (coerce (cl-waffe2/base-impl::logical-false-then self) 'single-float)))
                                (check (wf2hip-compare-nd-typed
                                        (nth-value 2 (dtype-info (dtype x)))
                                        (condition->op (cl-waffe2/base-impl::logical-condition self)) view
                                        (tensor-device-pointer x) (tensor-device-pointer y)
                                        (tensor-device-pointer out)
                                        (coerce (cl-waffe2/base-impl::logical-true-then self) 'double-float)
                                        (coerce (cl-waffe2/base-impl::logical-false-then self) 'double-float)))))
                          out))

;; A[~] OUT[out-size] -> OUT: largest / smallest value of every trailing run of A, or its index
;; (source/base-impl/matrix-ops.lisp:197-383).  !max / !argmax hand over A reshaped to
;; (kept... t) and OUT shaped (kept... 1); the outer axes go to the library as one view2 with the
;; last axis of A cut off, the run as (n, incx).  ArgMax / ArgMin write :uint32 into OUT, which is
;; therefore allocated by the device class as 4-byte elements like :float.
(defun run-select (op x out)
  (ensure-extension)
  (with-foreign-object (view '(:struct view2))
    (fill-view2 view x out)   ; shape slots come from X; only the outer axes are read below
    (let* ((rank (length (shape x)))
           (last-axis (1- rank))
           (n (mem-aref (foreign-slot-pointer view '(:struct view2) 'shape) :int64 last-axis))
           (incx (mem-aref (foreign-slot-pointer view '(:struct view2) 'stride-a) :int64 last-axis)))
      (if (= rank 1)
          (setf (mem-aref (foreign-slot-pointer view '(:struct view2) 'shape) :int64 0) 1
                (mem-aref (foreign-slot-pointer view '(:struct view2) 'stride-a) :int64 0) 0
                (mem-aref (foreign-slot-pointer view '(:struct view2) 'stride-b) :int64 0) 0)
          (setf (foreign-slot-value view '(:struct view2) 'rank) (1- rank)))
      (if (eql (dtype x) :float)
          (check (wf2hip-select-nd op view n incx (tensor-device-pointer x) (tensor-device-pointer out)))
          (check (wf2hip-select-nd-typed (nth-value 2 (dtype-info (dtype x))) op view n incx
                                         (tensor-device-pointer x) (tensor-device-pointer out))))))
  out)

;; The value nodes take every dtype (waffe2_<prefix>{max,min} on the CPU), the index nodes :float
;; and :double (BLAS i?max / i?min, source/backends/cpu/matrix-ops.lisp:254-266).
(macrolet ((define-select (node op reject)
             `(define-impl-op (,node :device HIPTensor :reject-p ,reject)
                              :forward ((self x out) (declare (ignore self)) (run-select ,op x out)))))
  (define-select MaxValue-Node +maxvalue+ #'(lambda (&rest args) (declare (ignore args)) nil))
  (define-select MinValue-Node +minvalue+ #'(lambda (&rest args) (declare (ignore args)) nil))
  (define-select ArgMax-Node +argmax+ #'float-or-double-p)
  (define-select ArgMin-Node +argmin+ #'float-or-double-p))

;; C[~ i k] = A[~ i j] . B[~ j k].  Same operand swap as expand-gemm-form-column
;; (source/backends/cpu/matrix-ops.lisp:12-112): a row-major product is the column-major
;; sgemm(transB, transA, n, m, k, 1, B, ldb, A, lda, 0, C, ldc).  Batch axes are walked on the
;; host exactly like call-with-view :at-least-dim 2 does, except that the innermost batch axis
;; goes to the library as one strided batch.
(defun matrix-geometry (tensor)
  (let* ((view (foreign-alloc '(:struct view2))))
    (unwind-protect
         (progn
           (fill-view2 view tensor tensor)
           (let* ((rank (length (shape tensor)))
                  (strides (loop for i below rank
                                 collect (mem-aref (foreign-slot-pointer view '(:struct view2) 'stride-a) :int64 i)))
                  (extents (loop for i below rank
                                 collect (mem-aref (foreign-slot-pointer view '(:struct view2) 'shape) :int64 i))))
             (assert (or (= 1 (nth (1- rank) extents)) (= 1 (nth (1- rank) strides))) ()
                     "MatMulNode-HIPTensor: operands must be contiguous along the last axis (use ->contiguous)")
             (values extents strides (foreign-slot-value view '(:struct view2) 'off-a))))
      (foreign-free view))))

(define-impl-op (MatMulNode :device HIPTensor :reject-p #'float-or-double-p)
                :forward ((self a b out)
                          (ensure-extension)
                          (let ((trans-a (trans-a? self))
                                (trans-b (trans-b? self))
                                (a (if (trans-a? self) (read-untransposed a) a))
                                (b (if (trans-b? self) (read-untransposed b) b)))
                            (multiple-value-bind (ea sa oa) (matrix-geometry a)
                              (multiple-value-bind (eb sb ob) (matrix-geometry b)
                                (multiple-value-bind (ec sc oc) (matrix-geometry out)
                                  (let* ((rank (length ec))
                                         (m (nth (- rank 2) ec))
                                         (n (nth (- rank 1) ec))
                                         (k (if trans-a (nth (- rank 2) ea) (nth (- rank 1) ea)))
                                         (lda (max 1 (nth (- rank 2) sa)))
                                         (ldb (max 1 (nth (- rank 2) sb)))
                                         (ldc (max 1 (nth (- rank 2) sc)))
                                         (batch-rank (- rank 2)))
                                    (labels ((launch (oa ob oc stride-a stride-b stride-c count)
                                               ;; sgemm_ or dgemm_ by dtype, like expand-gemm-form-column
                                               ;; (source/backends/cpu/matrix-ops.lisp:12-112)
                                               (if (eql (dtype out) :double)
                                                   (check (wf2hip-dgemm-strided-batched-2d
                                                           (char-code (if trans-b #\C #\N))
                                                           (char-code (if trans-a #\C #\N))
                                                           n m k 1.0d0
                                                           (tensor-device-pointer b ob) ldb stride-b 0
                                                           (tensor-device-pointer a oa) lda stride-a 0
                                                           0.0d0
                                                           (tensor-device-pointer out oc) ldc stride-c 0 count 1))
                                                   (check (wf2hip-sgemm-strided-batched
                                                           (char-code (if trans-b #\C #\N))
                                                           (char-code (if trans-a #\C #\N))
                                                           n m k 1.0
                                                           (tensor-device-pointer b ob) ldb stride-b
                                                           (tensor-device-pointer a oa) lda stride-a
                                                           0.0
                                                           (tensor-device-pointer out oc) ldc stride-c count))))
                                             (walk (axis oa ob oc)
                                               (cond
                                                 ((= batch-rank 0) (launch oa ob oc 0 0 0 1))
                                                 ((= axis (1- batch-rank))
                                                  (launch oa ob oc (nth axis sa) (nth axis sb) (nth axis sc)
                                                          (nth axis ec)))
                                                 (t
                                                  (dotimes (i (nth axis ec))
                                                    (walk (1+ axis)
                                                          (+ oa (* i (nth axis sa)))
                                                          (+ ob (* i (nth axis sb)))
                                                          (+ oc (* i (nth axis sc)))))))))
                                      (walk 0 oa ob oc))))))
                            out)))

;; Unfold / fold (source/base-impl/unfold.lisp; CPU forwards source/backends/cpu/im2col.lisp).
;; Same slots, same argument order as waffe2_im2col_s_column / waffe2_col2im_s_column.
(macrolet ((define-unfold (node fn first second)
             `(define-impl-op (,node :device HIPTensor :reject-p #'only-float-p)
                              :forward ((self ,first ,second)
                                        (ensure-extension)
                                        (let ((x ,(if (eq node 'Im2ColNode) first second))
                                              (col ,(if (eq node 'Im2ColNode) second first)))
                                          (setf (h-of self) (nth 2 (shape x))
                                                (w-of self) (nth 3 (shape x)))
                                          (with-slots (C h-out w-out k-h k-w padding-h padding-w
                                                       stride-h stride-w dilation-h dilation-w)
                                              self
                                            (check (,fn (tensor-device-pointer col)
                                                        (car (shape x)) C (h-of self) (w-of self)
                                                        h-out w-out k-h k-w padding-h padding-w
                                                        stride-h stride-w dilation-h dilation-w
                                                        (tensor-device-pointer x)))))
                                        ,second))))
  (define-unfold Im2ColNode wf2hip-im2col-f32 x col)
  (define-unfold Col2ImNode wf2hip-col2im-f32 col output-to))

;; Optimiser steps in one kernel.  step-optimize of SGD / Adam composes element-wise nodes
;; (source/optimizers/impls/sgd.lisp:18-34, adam.lisp:45-117); for a contiguous HIPTensor
;; parameter these :around methods run the same binary32 operations in the same order in one
;; pass instead (bit-identical result) and fall back to the node composition otherwise.
(defun contiguous-device-tensor-p (tensor)
  (and (typep tensor 'HIPTensor)
       (every #'(lambda (v) (eql (cl-waffe2/vm.generic-tensor::force-list v) t)) (tensor-view tensor))
       (zerop (tensor-initial-offset tensor))))

(defmethod cl-waffe2/optimizers:step-optimize :around ((optimizer cl-waffe2/optimizers:SGD))
  (let* ((param (cl-waffe2/optimizers:read-parameter optimizer))
         (grad (grad param)))
    (if (and *hip-extension-p* (contiguous-device-tensor-p param) (contiguous-device-tensor-p grad))
        (check (wf2hip-sgd-step-f32 (apply #'* (shape param))
                                    (tensor-device-pointer param) (tensor-device-pointer grad)
                                    (coerce (cl-waffe2/optimizers::sgd-lr optimizer) 'single-float)))
        (call-next-method))))

(defmethod cl-waffe2/optimizers:step-optimize :around ((optimizer cl-waffe2/optimizers:Adam))
  (let* ((param (cl-waffe2/optimizers:read-parameter optimizer))
         (grad (grad param))
         (m (cl-waffe2/optimizers::adam-m optimizer))
         (v (cl-waffe2/optimizers::adam-v optimizer)))
    (if (and *hip-extension-p* (every #'contiguous-device-tensor-p (list param grad m v)))
        (let ((lr-t (cl-waffe2/optimizers::adam-step-lr optimizer)))   ; also counts the step
          (check (wf2hip-adam-step-f32
                  (apply #'* (shape param))
                  (tensor-device-pointer param) (tensor-device-pointer grad)
                  (tensor-device-pointer m) (tensor-device-pointer v)
                  (- 1.0 (cl-waffe2/optimizers::beta1-of optimizer))
                  (- 1.0 (cl-waffe2/optimizers::beta2-of optimizer))
                  (coerce lr-t 'single-float)
                  (cl-waffe2/optimizers::eps-of optimizer))))
        (call-next-method))))

