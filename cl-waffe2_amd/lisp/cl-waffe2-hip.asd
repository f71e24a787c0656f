;;;; cl-waffe2-hip.asd -- HIPTensor backend for cl-waffe2 on AMD MI355X (gfx950).
;;;;
;;;; Purely additive: loading this system defines a new device class and
;;;; registers define-impl-op implementations for the existing AbstractNodes
;;;; (source/vm/nodes/defnode.lisp:582-671).  Nothing in cl-waffe2 is modified.
;;;;
;;;;   (ql:quickload :cl-waffe2-hip)
;;;;   (cl-waffe2:with-devices (cl-waffe2/backends.hip:HIPTensor) ...)
(asdf:defsystem :cl-waffe2-hip
  :description "MI355X (gfx950) backend of cl-waffe2: HIPTensor + libwaffe2-hip.so"
  :license "MIT"
  :depends-on (:cl-waffe2 :cffi :trivial-garbage)
  :serial t
  :components ((:file "package")
               (:file "shared-object")
               (:file "api")
               (:file "tensor")
               (:file "kernels")
               (:file "fusion")))
