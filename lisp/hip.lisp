;;;; source/byoc/hip.lisp -- the `:HIP` backend for Caten, bound to libcaten_hip.so through CFFI.
;;;;
;;;; Drop this file next to source/byoc/metal.lisp, add "hip" to the :components of caten.byoc.asd
;;;; and run with BACKEND=HIP.  It fills the same slots the Metal backend fills
;;;; (source/byoc/metal.lisp:103-154,173-189,252-345): a Buffer class with the six buffer generics, a
;;;; Runtime class, a Renderer that turns blueprints into HIP source compiled once per graph with
;;;; hipRTC, and a caller lambda per Schedule-Item.  Everything below the `defcfun`s is the C ABI of
;;;; include/caten_hip.h.
;;;;
;;;; This image has no Common Lisp implementation, so this file has not been loaded by a Lisp here;
;;;; the same C ABI is exercised through the Python mirror in caten_amd/.

(defpackage :caten/byoc/hip
  (:use :cl :cffi :caten/runtime/buffer :caten/common.dtype :caten/runtime/runtime
        :caten/codegen/backend :caten/codegen/renderer :caten/air :caten/codegen/expr
        :caten/codegen/helpers :caten/codegen/shape-inference :caten/codegen/blueprint)
  (:import-from :caten/codegen/config #:define-auto-scheduler))

(in-package :caten/byoc/hip)

;;; ~~~ foreign library ~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~
(define-foreign-library libcaten-hip (t (:default "libcaten_hip")))
(defvar *loaded* nil)
(defun ensure-foreign-library ()
  (unless *loaded*
    (use-foreign-library libcaten-hip)
    (setf *loaded* t)))

(defcfun ("cthip_init" %init) :int (device :int))
(defcfun ("cthip_last_error" %last-error) :string)
(defcfun ("cthip_alloc" %alloc) :int (out :pointer) (bytes :size))
(defcfun ("cthip_free" %free) :int (p :pointer))
(defcfun ("cthip_h2d" %h2d) :int (dst :pointer) (src :pointer) (bytes :size))
(defcfun ("cthip_d2h" %d2h) :int (dst :pointer) (src :pointer) (bytes :size))
(defcfun ("cthip_d2d" %d2d) :int (dst :pointer) (src :pointer) (bytes :size))
(defcfun ("cthip_sync" %sync) :int)
(defcfun ("cthip_compile" %compile) :int (src :string) (arch :string) (code :pointer) (size :pointer) (log :pointer))
(defcfun ("cthip_release" %release) :void (p :pointer))
(defcfun ("cthip_module_load" %module-load) :int (module :pointer) (code :pointer))
(defcfun ("cthip_get_function" %get-function) :int (fn :pointer) (module :pointer) (name :string))
(defcfun ("cthip_launch" %launch) :int (fn :pointer) (grid :pointer) (block :pointer) (lds :uint) (args :pointer) (nargs :int))

(defmacro check (form)
  "Signals a Lisp error (=> runtime-error inside the VM, source/runtime/runtime.lisp:84-104) on a non-zero status."
  `(let ((status ,form))
     (unless (zerop status)
       (error "Caten[HIP]: ~a failed with status ~a: ~a" ',(car form) status (%last-error)))
     status))

;;; ~~~ Buffer / Runtime ~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~
(defclass HipBuffer (AbstractBuffer) nil)
(defclass HipRuntime (GraphRuntime) ((device :initform 0 :accessor hip-runtime-device)))

(defmethod initialize-instance :after ((runtime HipRuntime) &key)
  (ensure-foreign-library)
  (check (%init (hip-runtime-device runtime))))

(defun buffer-nbytes (buffer)
  (* (buffer-storage-size buffer) (dtype/size-of (buffer-dtype buffer))))

(defmethod open-buffer ((runtime HipRuntime) (buffer HipBuffer))
  ;; rank-0 buffers stay Lisp numbers, as in every other backend (metal.lisp:114-121);
  ;; cthip_alloc returns zeroed storage from a caching allocator
  (if (= 0 (buffer-nrank buffer))
      (setf (buffer-value buffer)
            (if (eql (buffer-dtype buffer) :bool) nil (coerce 0 (dtype->lisp (buffer-dtype buffer)))))
      (with-foreign-object (out :pointer)
        (check (%alloc out (buffer-nbytes buffer)))
        (setf (buffer-value buffer) (mem-ref out :pointer)))))

(defmethod close-buffer ((runtime HipRuntime) (buffer HipBuffer))
  (when (pointerp (buffer-value buffer))
    (check (%free (buffer-value buffer)))
    (setf (buffer-value buffer) nil)))

(defmethod transfer-from-array ((runtime HipRuntime) (buffer HipBuffer) array)
  ;; the array is pinned only for the duration of the call; cthip_h2d stages it
  (with-pointer-to-vector-data (src array)
    (check (%h2d (buffer-value buffer) src (buffer-nbytes buffer)))))

(defmethod transfer-into-array ((buffer HipBuffer))
  (when (numberp (buffer-value buffer))
    (return-from transfer-into-array (buffer-value buffer)))
  (let ((placeholder (make-array (buffer-storage-size buffer) :element-type (dtype->lisp (buffer-dtype buffer)))))
    (with-pointer-to-vector-data (dst placeholder)
      (check (%d2h dst (buffer-value buffer) (buffer-nbytes buffer)))) ; synchronises the stream
    placeholder))

(defmethod copy-buffer-value ((runtime HipRuntime) (buffer HipBuffer))
  (if (pointerp (buffer-value buffer))
      (with-foreign-object (out :pointer)
        (check (%alloc out (buffer-nbytes buffer)))
        (check (%d2d (mem-ref out :pointer) (buffer-value buffer) (buffer-nbytes buffer)))
        (mem-ref out :pointer))
      (buffer-value buffer)))

(defmethod bref ((buffer HipBuffer) idx)
  (let ((type (->cffi-dtype (buffer-dtype buffer))))
    (with-foreign-object (tmp type)
      (check (%d2h tmp (inc-pointer (buffer-value buffer) (* idx (dtype/size-of (buffer-dtype buffer))))
                   (dtype/size-of (buffer-dtype buffer))))
      (mem-ref tmp type))))

;;; ~~~ Renderer ~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~
(defclass Hip-Renderer (CStyle-Renderer) ((module :initform nil :accessor hip-renderer-module)))
(define-auto-scheduler (Hip-Auto-Scheduler ()) :n-global-loop 3)
(define-backend :hip HipBuffer HipRuntime Hip-Renderer Hip-Auto-Scheduler t)

(defun dtype->hiptype (dtype)
  (ecase dtype
    (:bool "bool") (:float64 "double") (:float32 "float")
    (:uint64 "unsigned long long") (:int64 "long long") (:uint32 "unsigned int") (:int32 "int")
    (:uint16 "unsigned short") (:int16 "short") (:uint8 "unsigned char") (:int8 "signed char")))

;; CStyle-Renderer has no :SPACE method (only the print-only Default-Renderer, renderer.lisp:233-236)
(defmethod %render-node ((renderer Hip-Renderer) (id (eql :SPACE)) node)
  (format nil "~a.~a"
          (ecase (getattr node :level) (:block "blockIdx") (:thread "threadIdx"))
          (ecase (getattr node :rank) (0 "x") (1 "y") (2 "z"))))

(defun header ()
  (format nil "~%#define _infinity __builtin_inff()~%#define _negative_infinity (-__builtin_inff())~%#define _nan __builtin_nanf(\"\")~%#define max(a, b) ((a) > (b) ? (a) : (b))~%#define min(a, b) ((a) < (b) ? (a) : (b))~%#define boolean bool~%"))

(defvar *indent*)
(defmethod %render-kernel ((renderer Hip-Renderer) si)
  ;; Signature: outputs, dynamic shapes by value, inputs (source/codegen/rewriting-rules.lisp:207-231)
  (let ((args (schedule-item-args si)))
    (with-output-to-string (out)
      (format out "extern \"C\" __global__ void ~(~a~)(" (getattr si :name))
      (format out "~{~a~^, ~}"
              (loop for item in args
                    collect (format nil "~a~a~a ~(~a~)"
                                    (if (eql (getattr item :type) :output) "" "const ")
                                    (dtype->hiptype (getattr item :dtype))
                                    (if (getattr item :pointer-p) "*" "")
                                    (car (node-writes item)))))
      (format out ") {~%")
      (let ((*indent* 2))
        (dolist (node (getattr si :blueprint))
          (render-bp node out)))
      (format out "}~%~%"))))

(defun render-bp (bp stream)
  ;; identical in structure to the Metal one (metal.lisp:190-237); loops marked :scope :global were
  ;; already rewritten by the auto-scheduler into :SPACE expressions plus a bounds :IF
  (flet ((indent () (make-string *indent* :initial-element #\space)))
    (ecase (node-type bp)
      (:FOR
       (format stream "~afor(int ~(~a~)=~a;~a;~(~a~)+=~a) {~%" (indent) (getattr bp :idx)
               (render-expr 'Hip-Renderer (getattr bp :upfrom)) (render-expr 'Hip-Renderer (getattr bp :below))
               (getattr bp :idx) (render-expr 'Hip-Renderer (getattr bp :by)))
       (incf *indent* 2))
      (:ENDFOR (decf *indent* 2) (format stream "~a}~%" (indent)))
      (:IF (format stream "~aif(~a){~%" (indent) (render-expr 'Hip-Renderer (getattr bp :condition))) (incf *indent* 2))
      (:ENDIF (decf *indent* 2) (format stream "~a}~%" (indent)))
      (:EXPR
       (let ((pre-iterations (getattr bp :iterations)))
         (format stream "~a~a~a = ~a;~%" (indent)
                 (if (car (getattr bp :declare-type))
                     (format nil "~a " (dtype->hiptype (buffer-dtype (car (relay-writes (read-type-relay bp))))))
                     "")
                 (render-list
                  (map 'list #'(lambda (x y z) (render-aref-from-space x y z pre-iterations))
                       (node-writes bp) (relay-writes (read-type-relay bp)) (relay-write-iters (read-type-relay bp))))
                 (render-expr 'Hip-Renderer (getattr bp :EXPR) :index-space pre-iterations))))
      (:DEFINE-GLOBAL))))

(defun render-aref-from-space (name b is iterations)
  ;; index = sum_d stride_d * (from_d + by_d * gid_d)  (source/byoc/clang.lisp:82-97)
  (if (and is (not (= -1 (buffer-nrank b))) (> (length (iteration-space-shape is)) 0) (> (length iterations) 0))
      (format nil "~(~a~)[~(~a~)]" name
              (render-expr 'Hip-Renderer
                           (apply #'expr-add
                                  (map 'list
                                       #'(lambda (view stride i)
                                           (if view
                                               (expr-mul stride (expr-add (expr-const (car view) :int64) (expr-mul (expr-const (third view) :int64) i)))
                                               (expr-mul stride i)))
                                       (iteration-space-views is) (iteration-space-strides is) iterations))))
      (format nil "~(~a~)" name)))

;;; ~~~ Program / launch ~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~
(defclass Hip-Program ()
  ((name :initarg :name :accessor hp-name)
   (fxn :initarg :fxn :accessor hp-fxn)
   (grid-size :initarg :grid-size :accessor hp-grid-size)
   (argtypes :initarg :argtypes :accessor hp-argtypes)
   (uploads :initform (make-hash-table :test #'eq) :accessor hp-uploads)))

(defmethod runtime-invoke-jit-kernel ((runtime HipRuntime) kernel-info node args)
  (apply (caten/codegen/jit:compiled-kernel-caller kernel-info) runtime node args))

(defun device-pointer-of (hp runtime buf)
  "Weights loaded from GGUF are LispBuffers whatever BACKEND is (external/gguf/tensor-info.lisp:104-120)
and enter through :Allocate :from untouched (source/runtime/runtime.lisp:228-243): upload once, cache."
  (cond
    ((typep buf 'HipBuffer) (buffer-value buf))
    ((and (buffer-p buf) (arrayp (buffer-value buf)))
     (or (gethash buf (hp-uploads hp))
         (let ((dev (make-buffer (buffer-shape buf) (buffer-stride buf) (buffer-dtype buf) (buffer-views buf) :device 'HipBuffer)))
           (open-buffer runtime dev)
           (transfer-from-array runtime dev (buffer-value buf))
           (setf (gethash buf (hp-uploads hp)) (buffer-value dev)))))
    (t (error "Caten[HIP]: ~a is neither a device buffer nor a host array" buf))))

(defmethod invoke ((hp Hip-Program) runtime node &rest buffers)
  (assert (= (length buffers) (length (hp-argtypes hp))) ()
          "HIP: the number of arguments does not match the kernel ~a" (hp-name hp))
  (let* ((n (length buffers))
         (params (map 'list #'cons (node-reads node) buffers)))
    (with-foreign-objects ((argv :pointer n) (slots :uint64 n) (grid :uint 3) (block :uint 3))
      (loop for buf in buffers
            for argtyp in (hp-argtypes hp)
            for nth upfrom 0
            for slot = (mem-aptr slots :uint64 nth) do
              (if (and (buffer-p buf) (> (buffer-nrank buf) 0))
                  (setf (mem-ref slot :pointer) (device-pointer-of hp runtime buf))
                  ;; rank-0: by value with its declared dtype (coerce-dtyped-buffer already cast it)
                  (setf (mem-ref slot (->cffi-dtype argtyp))
                        (if (buffer-p buf) (buffer-value buf) buf)))
              (setf (mem-aref argv :pointer nth) slot))
      (loop for g in (hp-grid-size hp) for i upfrom 0 do
        (setf (mem-aref grid :uint i) (exprgrid-global-size-int g params)
              (mem-aref block :uint i) (exprgrid-local-size-int g)))
      (check (%launch (hp-fxn hp) grid block 0 argv n)))))
;; [Note] rank-0 *outputs* are declared as pointers by schedule-item-write-define-global; CLANG boxes the
;; Lisp number and writes it back (clang.lisp:166-185).  On HIP such a scalar needs a 1-element device
;; cell and a cthip_d2h after the launch; add it to `invoke` when a graph produces one.

(defun make-hip-caller (hp) `(lambda (runtime node &rest args) (apply #'invoke ,hp runtime node args)))

(defmethod %compile-kernel ((renderer Hip-Renderer) items dir)
  (declare (ignore dir))
  (ensure-foreign-library)
  (let ((code (apply #'concatenate 'string
                     (append (list (header))
                             (loop for item in items
                                   if (getattr item :rendered-object) collect (getattr item :rendered-object))))))
    (when (>= (ctx:getenv :JIT_DEBUG) 3) (format t "[Final Code]:~%~a~%" code))
    (with-foreign-objects ((blob :pointer) (size :size) (log :pointer) (module :pointer) (fn :pointer))
      (unless (zerop (%compile code "gfx950" blob size log))
        (error "Caten[HIP]: Failed to compile the kernels:~%~a~%Compiled with hipRTC --offload-arch=gfx950 -O3"
               (if (null-pointer-p (mem-ref log :pointer)) (%last-error) (foreign-string-to-lisp (mem-ref log :pointer)))))
      (check (%module-load module (mem-ref blob :pointer)))
      (%release (mem-ref blob :pointer))
      (setf (hip-renderer-module renderer) (mem-ref module :pointer))
      (loop for item in items
            if (getattr item :rendered-object) do
              (check (%get-function fn (mem-ref module :pointer) (string-downcase (princ-to-string (getattr item :name)))))
              (setf (getattr item :compiled-object)
                    (make-hip-caller
                     (make-instance 'Hip-Program :name (getattr item :name) :fxn (mem-ref fn :pointer)
                                                 :argtypes (map 'list #'(lambda (x) (getattr x :dtype)) (schedule-item-args item))
                                                 :grid-size (blueprint-gather-grids (getattr item :blueprint) :max-dimension 3))))))
    nil))
