(in-package :cl-waffe2/backends.hip)

;; CFFI bindings of include/waffe2_hip.h.  Counterpart of cl-waffe2-simd/api.lisp: where that
;; file declares `(defcfun "waffe2_sadd" :void (n :long) (x (:pointer :float)) (incx :long) ...)`
;; (api.lisp:63-82), the device library returns an int status that `check` turns into a Lisp
;; error, so that the VM's handler reports the failing instruction (source/vm/vm.lisp:230-256).

(define-condition hip-error (error)
  ((code :initarg :code :reader hip-error-code)
   (message :initarg :message :reader hip-error-message))
  (:report (lambda (c s)
             (format s "libwaffe2-hip: error ~a: ~a" (hip-error-code c) (hip-error-message c)))))

(defmacro check (form)
  "Evaluates a wf2hip_* call and signals HIP-ERROR unless it returned 0."
  (let ((code (gensym "CODE")))
    `(let ((,code ,form))
       (unless (zerop ,code)
         (error 'hip-error :code ,code :message (wf2hip-last-error)))
       ,code)))

(defun ensure-extension ()
  (unless *hip-extension-p*
    (error "HIPTensor: libwaffe2-hip.so is not loaded; there is no CPU fallback for device tensors.")))

(defcfun "wf2hip_last_error" :string)
(defcfun "wf2hip_malloc" :int (ptr :pointer) (bytes :size))
(defcfun "wf2hip_malloc_uninitialized" :int (ptr :pointer) (bytes :size))
(defcfun "wf2hip_free" :int (ptr :pointer))
(defcfun "wf2hip_memcpy_h2d" :int (dst :pointer) (src :pointer) (bytes :size))
(defcfun "wf2hip_memcpy_d2h" :int (dst :pointer) (src :pointer) (bytes :size))
(defcfun "wf2hip_memcpy_d2d" :int (dst :pointer) (src :pointer) (bytes :size))
(defcfun "wf2hip_fill_f32" :int (x :pointer) (n :size) (value :float))
(defcfun "wf2hip_sync" :int)
(defcfun "wf2hip_device_info" :int (buf :pointer) (len :size))
(defcfun "wf2hip_set_reduce_mode" :int (mode :int))
(defcfun "wf2hip_get_reduce_mode" :int)

;; struct wf2hip_view2
(defcstruct view2
  (rank :int32)
  (reserved :int32)
  (shape :int64 :count 8)
  (stride-a :int64 :count 8)
  (stride-b :int64 :count 8)
  (off-a :int64)
  (off-b :int64))

(defcfun "wf2hip_binary_nd" :int (op :int) (view (:pointer (:struct view2))) (a :pointer) (b :pointer))
(defcfun "wf2hip_unary_nd" :int (op :int) (view (:pointer (:struct view2))) (a :pointer) (b :pointer) (p :float))
(defcfun "wf2hip_sgemm_strided_batched" :int
  (transa :char) (transb :char) (m :long) (n :long) (k :long) (alpha :float)
  (a :pointer) (lda :long) (stride-a :long)
  (b :pointer) (ldb :long) (stride-b :long)
  (beta :float) (c :pointer) (ldc :long) (stride-c :long) (batch :long))
(defcfun "wf2hip_sum_nd" :int (view (:pointer (:struct view2))) (a :pointer) (b :pointer) (divisor :float))
(defcfun "wf2hip_softmax_rows_f32" :int (rows :long) (cols :long) (x :pointer) (ldx :long) (out :pointer) (ldo :long))
(defcfun "wf2hip_layernorm_rows_f32" :int (rows :long) (cols :long) (x :pointer) (g :pointer) (b :pointer) (eps :float) (out :pointer))
;; Softmax-Cross-Entropy-Node (source/nn/criterion.lisp:90-126): softmax and -labels log(z + delta) in one pass
(defcfun "wf2hip_softmax_cross_entropy_f32" :int (rows :long) (cols :long) (x :pointer) (labels :pointer) (delta :float)
  (z :pointer) (loss :pointer))
;; backward of the fused layers, one kernel each
(defcfun "wf2hip_softmax_backward_rows_f32" :int (rows :long) (cols :long) (y :pointer) (ldy :long) (dy :pointer) (lddy :long)
  (dx :pointer) (lddx :long) (scale :float) (causal-seq :long))
(defcfun "wf2hip_layernorm_backward_f32" :int (rows :long) (cols :long) (x :pointer) (g :pointer) (dy :pointer) (eps :float)
  (dx :pointer) (dg :pointer) (db :pointer))
(defcfun "wf2hip_activation_backward_nd" :int (op :int) (view :pointer) (dout :pointer) (x :pointer) (p :float))
;; sce-diff-static (source/nn/criterion.lisp:82-88) in one pass
(defcfun "wf2hip_softmax_cross_entropy_backward_f32" :int (n :long) (dy :pointer) (dy-is-scalar :int) (z :pointer)
  (labels :pointer) (batch :float) (dx :pointer))

;; struct wf2hip_view3 and the compare kernels (counterparts of waffe2_s{eq,lt,le,gt,ge}[_scal],
;; cl-waffe2-simd/api.lisp:143-209)
(defcstruct view3
  (rank :int32)
  (reserved :int32)
  (shape :int64 :count 8)
  (stride-a :int64 :count 8)
  (stride-b :int64 :count 8)
  (stride-c :int64 :count 8)
  (off-a :int64)
  (off-b :int64)
  (off-c :int64))
(defcfun "wf2hip_where_nd" :int
  (op :int) (view (:pointer (:struct view2))) (x :pointer) (out :pointer)
  (scal :float) (then-value :float) (else-value :float))
(defcfun "wf2hip_compare_nd" :int
  (op :int) (view (:pointer (:struct view3))) (x :pointer) (y :pointer) (out :pointer)
  (then-value :float) (else-value :float))
(defcfun "wf2hip_unary_nd_typed" :int
  (dtype :int) (op :int) (view (:pointer (:struct view2))) (x :pointer) (out :pointer) (p :double))
(defcfun "wf2hip_where_nd_typed" :int
  (dtype :int) (op :int) (view (:pointer (:struct view2))) (x :pointer) (out :pointer)
  (scal :double) (then-value :double) (else-value :double))
(defcfun "wf2hip_compare_nd_typed" :int
  (dtype :int) (op :int) (view (:pointer (:struct view3))) (x :pointer) (y :pointer) (out :pointer)
  (then-value :double) (else-value :double))
(defcfun "wf2hip_sinv" :int (n :long) (x :pointer) (incx :long))
;; :double and the integer dtypes (waffe2_d*, waffe2_{i32,...}*, cl-waffe2-simd/api.lisp:63-124):
;; one entry point per shape of call, the element type as a code (dtype-info in tensor.lisp)
(defcfun "wf2hip_binary_1d_typed" :int
  (dtype :int) (op :int) (n :long) (x :pointer) (incx :long) (y :pointer) (incy :long))
(defcfun "wf2hip_binary_nd_typed" :int
  (dtype :int) (op :int) (view (:pointer (:struct view2))) (a :pointer) (b :pointer))
(defcfun "wf2hip_inv_1d_typed" :int (dtype :int) (n :long) (x :pointer) (incx :long))
(defcfun "wf2hip_select_nd_typed" :int
  (dtype :int) (op :int) (outer (:pointer (:struct view2))) (n :long) (incx :long) (x :pointer) (out :pointer))
(defcfun "wf2hip_select_nd" :int
  (op :int) (outer (:pointer (:struct view2))) (n :long) (incx :long) (x :pointer) (out :pointer))
(defconstant +maxvalue+ 48) (defconstant +minvalue+ 49) (defconstant +argmax+ 50) (defconstant +argmin+ 51)
(defconstant +eq+ 0) (defconstant +lt+ 1) (defconstant +le+ 2) (defconstant +gt+ 3) (defconstant +ge+ 4)

;; Extensions without a BLAS / SIMD-extension counterpart.  cl-waffe2 reaches them through its own
;; extension points: a define-bypass rule (source/vm/nodes/symbolic.lisp:118-131) or a define-op node
;; like Softmax-Cross-Entropy-Node (source/nn/criterion.lisp:90).
(defcfun "wf2hip_sgemm_strided_batched_2d" :int
  (transa :char) (transb :char) (m :long) (n :long) (k :long) (alpha :float)
  (a :pointer) (lda :long) (stride-a :long) (stride-a2 :long)
  (b :pointer) (ldb :long) (stride-b :long) (stride-b2 :long)
  (beta :float) (c :pointer) (ldc :long) (stride-c :long) (stride-c2 :long) (batch :long) (batch2 :long))

(defcfun "wf2hip_dgemm_strided_batched_2d" :int
  (transa :char) (transb :char) (m :long) (n :long) (k :long) (alpha :double)
  (a :pointer) (lda :long) (stride-a :long) (stride-a2 :long)
  (b :pointer) (ldb :long) (stride-b :long) (stride-b2 :long)
  (beta :double) (c :pointer) (ldc :long) (stride-c :long) (stride-c2 :long) (batch :long) (batch2 :long))

;; struct wf2hip_matmul_desc
(defcstruct matmul-desc
  (trans-a :int32) (trans-b :int32) (activation :int32) (causal :int32)
  (m :int64) (n :int64) (k :int64)
  (lda :int64) (ldb :int64) (ldc :int64)
  (batch :int64) (batch2 :int64)
  (stride-a :int64) (stride-a2 :int64) (stride-b :int64) (stride-b2 :int64) (stride-c :int64) (stride-c2 :int64)
  (bias :pointer) (residual :pointer)
  (ld-residual :int64) (stride-residual :int64) (stride-residual2 :int64)
  (alpha :float) (reserved :int32))
(defcfun "wf2hip_matmul_fused" :int (desc (:pointer (:struct matmul-desc))) (a :pointer) (b :pointer) (c :pointer))

;; struct wf2hip_attention_desc
(defcstruct attention-desc
  (batch :int64) (heads :int64) (seq :int64) (head-dim :int64)
  (q-stride :int64 :count 3) (k-stride :int64 :count 3) (v-stride :int64 :count 3) (o-stride :int64 :count 3)
  (scale :float) (causal :int32))
(defcfun "wf2hip_attention_f32" :int
  (desc (:pointer (:struct attention-desc))) (q :pointer) (k :pointer) (v :pointer) (o :pointer))
(defcfun "wf2hip_attention_forward_f32" :int (desc :pointer) (q :pointer) (k :pointer) (v :pointer) (o :pointer) (lse :pointer))
(defcfun "wf2hip_attention_backward_f32" :int (desc :pointer) (q :pointer) (k :pointer) (v :pointer) (o :pointer)
  (dout :pointer) (lse :pointer) (dq :pointer) (dk :pointer) (dv :pointer))
(defcfun "wf2hip_causal_softmax_f32" :int (matrices :long) (seq :long) (x :pointer) (out :pointer) (scale :float))

(defcfun "wf2hip_im2col_f32" :int
  (col :pointer) (n :long) (c :long) (h :long) (w :long) (h-out :long) (w-out :long) (k-h :long) (k-w :long)
  (pad-h :long) (pad-w :long) (stride-h :long) (stride-w :long) (dilation-h :long) (dilation-w :long) (im :pointer))
(defcfun "wf2hip_col2im_f32" :int
  (col :pointer) (n :long) (c :long) (h :long) (w :long) (h-out :long) (w-out :long) (k-h :long) (k-w :long)
  (pad-h :long) (pad-w :long) (stride-h :long) (stride-w :long) (dilation-h :long) (dilation-w :long) (im :pointer))
;; unfold (source/nn/im2col.lisp:51-95) with dilation 1 as one kernel: padding, Im2ColNode, permutation and reshape
(defcfun "wf2hip_unfold_f32" :int (n :long) (c :long) (h :long) (w :long) (k-h :long) (k-w :long) (stride-h :long)
  (stride-w :long) (pad-h :long) (pad-w :long) (x :pointer) (out :pointer))
(defcfun "wf2hip_sgd_step_f32" :int (n :long) (param :pointer) (grad :pointer) (lr :float))
(defcfun "wf2hip_adam_step_f32" :int
  (n :long) (param :pointer) (grad :pointer) (m :pointer) (v :pointer)
  (one-minus-beta1 :float) (one-minus-beta2 :float) (lr-t :float) (eps :float))

;; HIP graphs: record the launches of one compiled forward, replay them with one call.
(defcfun "wf2hip_graph_begin" :int)
(defcfun "wf2hip_graph_end" :int (graph (:pointer :pointer)))
(defcfun "wf2hip_graph_launch" :int (graph :pointer))
(defcfun "wf2hip_graph_destroy" :int (graph :pointer))
(defcfun "wf2hip_pool_trim" :int)
(defcfun "wf2hip_pool_idle_bytes" :size)
(defcfun "wf2hip_pool_requests" :size)

(defmacro with-captured-graph ((graph) &body body)
  "Runs BODY once with every kernel launch recorded instead of executed and binds GRAPH to the
recorded graph handle (replay with (check (wf2hip-graph-launch graph)), release with
wf2hip-graph-destroy).  BODY must have run once eagerly before, so that its temporaries can be
served from the library's pool; transfers and vref are refused while recording."
  (let ((slot (gensym "SLOT")))
    `(cffi:with-foreign-object (,slot :pointer)
       (check (wf2hip-graph-begin))
       (unwind-protect (progn ,@body)
         (check (wf2hip-graph-end ,slot)))
       (let ((,graph (cffi:mem-ref ,slot :pointer)))
         ,graph))))

;; enum wf2hip_binary_op / wf2hip_unary_op
(defconstant +add+ 0) (defconstant +sub+ 1) (defconstant +mul+ 2) (defconstant +div+ 3) (defconstant +move+ 4)
(defconstant +sin+ 16) (defconstant +cos+ 17) (defconstant +tanh+ 18) (defconstant +log+ 19)
(defconstant +exp+ 20) (defconstant +sqrt+ 21) (defconstant +abs+ 22) (defconstant +pow+ 32)
(defconstant +tan+ 23) (defconstant +asin+ 24) (defconstant +acos+ 25) (defconstant +atan+ 26)
(defconstant +sinh+ 27) (defconstant +cosh+ 28) (defconstant +log2+ 29) (defconstant +log10+ 30) (defconstant +log1p+ 31)
(defconstant +sign+ 34) (defconstant +square+ 35) (defconstant +asinh+ 36) (defconstant +acosh+ 37) (defconstant +atanh+ 38)

(defun hip-synchronize ()
  "Blocks until every kernel enqueued so far has finished (needed around wall-clock timing such
as proceed-bench, source/base-impl/fundamental.lisp:706-777)."
  (ensure-extension)
  (check (wf2hip-sync)))

(defmacro with-sequential-reductions (&body body)
  "Runs BODY with AddNode-into-broadcast accumulations in the CPU backend's strictly sequential
fp32 order (bit parity with CPUTensor; slow)."
  (let ((old (gensym "OLD")))
    `(let ((,old (wf2hip-get-reduce-mode)))
       (check (wf2hip-set-reduce-mode 1))
       (unwind-protect (progn ,@body)
         (wf2hip-set-reduce-mode ,old)))))
