;;;; gpt2-example.lisp -- HIPTensor implementation of the one node the reference's GPT-2 example
;;;; defines for itself (examples/gpt-2/utils.lisp:68-110, GPT2PositionalEmbedding: LispTensor only,
;;;; through raw host pointers and waffe2_sadd), so that the example's model runs on the device from
;;;; the token ids to the logits.
;;;;
;;;; Not a component of cl-waffe2-hip.asd: it needs the package of the example.  Load it after both:
;;;;   (ql:quickload :cl-waffe2-hip) (load "examples/gpt-2/gpt-2.asd") (ql:quickload :gpt-2-example)
;;;;   (load ".../cl-waffe2_amd/lisp/gpt2-example.lisp")
;;;; With HIPTensor leading *using-backend* the example's remaining host-bound pieces are its
;;;; (with-devices (LispTensor) (!tanh ...)) inside !gelu-lisptanh -- use !gelu-hip or
;;;; (!linear-hip ... :activation :gelu) there -- and load-npy, whose tensors (hip:to-device ...) moves.
;;;; Like the rest of this directory the file has not been run: no Common Lisp in the build image.

(in-package :cl-waffe2/backends.hip)

(defcfun "wf2hip_embedding_add_f32" :int
  (rows :long) (seq :long) (dim :long) (ctx :pointer) (wte :pointer) (vocab :long) (wpe :pointer) (n-ctx :long)
  (out :pointer))

;; ctx[N sentence-length] wte[vocab-size embedding-size] wpe[n-ctx embedding-size]
;; ctx-out[N sentence-length embedding-size] -> ctx-out:  out <- wte[round(ctx)] + wpe[position].
;; The reference zeroes the first row of each sentence and adds the two table rows onto every
;; position of a freshly allocated (zero) output; the kernel writes the sum.
(define-impl-op (gpt-2-example::GPT2PositionalEmbedding :device HIPTensor)
                :forward ((self ctx wte wpe ctx-out)
                          (declare (ignore self))
                          (ensure-extension)
                          (assert (and (eql (dtype ctx) :float) (eql (dtype wte) :float) (eql (dtype wpe) :float)) ()
                                  "GPT2PositionalEmbedding-HIPTensor: :float tensors only")
                          (let ((n (first (shape ctx)))
                                (seq (second (shape ctx)))
                                (vocab (first (shape wte)))
                                (dim (second (shape wte))))
                            (check (wf2hip-embedding-add-f32 (* n seq) seq dim
                                                             (tensor-device-pointer ctx) (tensor-device-pointer wte) vocab
                                                             (tensor-device-pointer wpe) (first (shape wpe))
                                                             (tensor-device-pointer ctx-out))))
                          ctx-out))
