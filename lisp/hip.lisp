;;;; source/byoc/hip.lisp -- the `:HIP` backend for Caten, bound to libcaten_hip.so through CFFI.
;;;;
;;;; Drop this file next to source/byoc/metal.lisp, add "hip" to the :components of caten.byoc.asd
;;;; and run with BACKEND=HIP.  It fills the same slots the Metal backend fills
;;;; (source/byoc/metal.lisp:103-154,173-189,252-345): a Buffer class with the six buffer generics, a
;;;; Runtime class, a Renderer that turns blueprints into HIP source compiled once per graph with
;;;; hipRTC, and a caller lambda per Schedule-Item.  Everything below the `defcfun`s is the C ABI of
;;;; include/caten_hip.h.
;;;;
;;;; The renderer protocol is implemented by PRINTING: %render-kernel prints the Schedule-Item's blueprint as an
;;;; s-expression (the grammar is in the header of caten_amd/csrc/render.hip) and hands it to
;;;; cthip_program_create, which returns HIP source with gfx950-aware work distribution and, for the matmul /
;;;; Linear / one-hot Embedding / ArgMax / softmax / LayerNorm / RMSNorm row shapes, a route to a hand-written
;;;; kernel; `invoke` is cthip_program_launch.  Nothing about work distribution lives on this side.
;;;;
;;;; This image has no Common Lisp implementation, so this file has not been loaded by a Lisp here;
;;;; the same C ABI, including the s-expression text, is exercised through the Python mirror in caten_amd/.

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
(defcfun ("cthip_render_header" %render-header) :string)
(defcfun ("cthip_program_create" %program-create) :int (program :pointer) (blueprint :string))
(defcfun ("cthip_program_destroy" %program-destroy) :int (program :pointer))
(defcfun ("cthip_program_source" %program-source) :string (program :pointer))
(defcfun ("cthip_program_bind" %program-bind) :int (program :pointer) (module :pointer))
(defcfun ("cthip_program_launch" %program-launch) :int (program :pointer) (args :pointer) (nargs :int))
(defcfun ("cthip_program_last_route" %program-last-route) :string (program :pointer))
(defcfun ("cthip_wmat_create" %wmat-create) :int (wmat :pointer) (type :int) (raw :pointer) (rows :int64) (cols :int64))
(defcfun ("cthip_wmat_destroy" %wmat-destroy) :int (wmat :pointer))
(defcfun ("cthip_wmat_fold_layernorm" %wmat-fold-layernorm) :int (wmat :pointer) (gamma :pointer) (beta :pointer) (bias :pointer))
(defcfun ("cthip_linear" %linear) :int (y :pointer) (wmat :pointer) (x :pointer) (m :int) (bias :pointer)
  (residual :pointer) (act :int) (prologue :int) (norm-g :pointer) (norm-b :pointer) (eps :float))

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

;; What a rank > 0 HipBuffer keeps in its `value` slot is not the raw device pointer but a BLOCK: the pointer plus a
;; flag that the storage is still allocated.  copy-buffer (source/runtime/buffer.lisp:60-68) copies slots, so a :View's
;; buffer, every other copy and the buffer that opened the storage all hold the SAME block object.  Device storage has
;; to go back to the allocator exactly once and must never be touched afterwards -- the caching allocator hands a freed
;; address to the next open-buffer -- so: the first close-buffer through any of them frees the block and marks it dead;
;; later closes (free-runtime closes every buffer of the variable table, runtime.lisp:76-81) find it dead and do
;; nothing; and a stale view of a closed pool signals an error instead of reading or freeing somebody else's memory.
(defstruct (hip-block (:constructor make-hip-block (pointer))) pointer (alive t))

(defun device-pointer (buffer)
  "The device address of a rank > 0 HipBuffer whose storage is still open."
  (let ((blk (buffer-value buffer)))
    (unless (hip-block-p blk)
      (error "Caten[HIP]: ~a holds no device storage (open-buffer it first)" buffer))
    (unless (hip-block-alive blk)
      (error "Caten[HIP]: the storage of ~a has been closed" buffer))
    (hip-block-pointer blk)))

(defmethod open-buffer ((runtime HipRuntime) (buffer HipBuffer))
  ;; rank-0 buffers stay Lisp numbers, as in every other backend (metal.lisp:114-121);
  ;; cthip_alloc returns zeroed storage from a caching allocator
  (if (= 0 (buffer-nrank buffer))
      (setf (buffer-value buffer)
            (if (eql (buffer-dtype buffer) :bool) nil (coerce 0 (dtype->lisp (buffer-dtype buffer)))))
      (with-foreign-object (out :pointer)
        (check (%alloc out (buffer-nbytes buffer)))
        (setf (buffer-value buffer) (make-hip-block (mem-ref out :pointer))))))

(defmethod close-buffer ((runtime HipRuntime) (buffer HipBuffer))
  (let ((blk (buffer-value buffer)))
    (when (hip-block-p blk)
      (when (hip-block-alive blk)
        (setf (hip-block-alive blk) nil) ; every buffer sharing the block sees it closed from here on
        (check (%free (hip-block-pointer blk))))
      (setf (buffer-value buffer) nil))))

(defmethod transfer-from-array ((runtime HipRuntime) (buffer HipBuffer) array)
  ;; the array is pinned only for the duration of the call; cthip_h2d stages it
  (with-pointer-to-vector-data (src array)
    (check (%h2d (device-pointer buffer) src (buffer-nbytes buffer)))))

(defmethod transfer-into-array ((buffer HipBuffer))
  (unless (hip-block-p (buffer-value buffer)) ; rank 0: the Lisp number / boolean itself
    (return-from transfer-into-array (buffer-value buffer)))
  (let ((placeholder (make-array (buffer-storage-size buffer) :element-type (dtype->lisp (buffer-dtype buffer)))))
    (with-pointer-to-vector-data (dst placeholder)
      (check (%d2h dst (device-pointer buffer) (buffer-nbytes buffer)))) ; synchronises the stream
    placeholder))

(defmethod copy-buffer-value ((runtime HipRuntime) (buffer HipBuffer))
  ;; new storage with the same bytes: a block of its own, owned by whichever buffer the caller stores it in
  (if (hip-block-p (buffer-value buffer))
      (with-foreign-object (out :pointer)
        (check (%alloc out (buffer-nbytes buffer)))
        (check (%d2d (mem-ref out :pointer) (device-pointer buffer) (buffer-nbytes buffer)))
        (make-hip-block (mem-ref out :pointer)))
      (buffer-value buffer)))

(defmethod bref ((buffer HipBuffer) idx)
  (let ((type (->cffi-dtype (buffer-dtype buffer))))
    (with-foreign-object (tmp type)
      (check (%d2h tmp (inc-pointer (device-pointer buffer) (* idx (dtype/size-of (buffer-dtype buffer))))
                   (dtype/size-of (buffer-dtype buffer))))
      (mem-ref tmp type))))

;;; ~~~ Renderer ~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~
(defclass Hip-Renderer (CStyle-Renderer) ((module :initform nil :accessor hip-renderer-module)))
(define-auto-scheduler (Hip-Auto-Scheduler ()) :n-global-loop 3)
(define-backend :hip HipBuffer HipRuntime Hip-Renderer Hip-Auto-Scheduler t)

;; Expressions are printed by a renderer of their own, through the same render-expr / render-node walk every
;; renderer uses (source/codegen/renderer.lisp:115-133): each %render-node method returns the s-expression text
;; of its node.  The catch-all covers the arithmetic instruction set uniformly -- (ADD a b), (MAX a b), (SIN a),
;; (WMMA c a b), (WHERE c a b) ... -- the methods below are the nodes whose reads are not their operands.
(defclass Sexp-Renderer (Renderer) nil)

(defmethod %render-const ((renderer Sexp-Renderer) obj)
  (cond
    ((and (numberp obj) (eql (float-type-of obj) :inf)) "inf")
    ((and (numberp obj) (eql (float-type-of obj) :-inf)) "-inf")
    ((and (numberp obj) (eql (float-type-of obj) :nan)) "nan")
    ((eql obj t) "t")
    ((null obj) "nil")
    (t (let ((*read-default-float-format* 'single-float)) (format nil "~(~a~)" obj)))))

(defmethod %render-node ((renderer Sexp-Renderer) id node)
  (format nil "(~(~a~)~{ ~a~})" (node-type node) (map 'list #'(lambda (x) (render-node renderer x)) (node-reads node))))
(defmethod %render-node ((renderer Sexp-Renderer) (id (eql :LOAD)) node)
  (%render-const renderer (getattr node :value)))
(defmethod %render-node ((renderer Sexp-Renderer) (id (eql :Allocate)) node) "0")
(defmethod %render-node ((renderer Sexp-Renderer) (id (eql :MOVE)) node) (render-node renderer (second (node-reads node))))
(defmethod %render-node ((renderer Sexp-Renderer) (id (eql :STORE)) node) (render-node renderer (second (node-reads node))))
(defmethod %render-node ((renderer Sexp-Renderer) (id (eql :CAST)) node)
  (format nil "(cast ~(~a~) ~a)" (getattr node :dtype) (render-node renderer (second (node-reads node)))))
(macrolet ((def (id)
             `(defmethod %render-node ((renderer Sexp-Renderer) (id (eql ,id)) node)
                ;; the first read is the output's placeholder (renderer.lisp:381-388)
                (format nil "(~(~a~) ~a ~a)" ,id (render-node renderer (nth 1 (node-reads node))) (render-node renderer (nth 2 (node-reads node)))))))
  (def :!=)
  (def :<))
(defmethod %render-node ((renderer Sexp-Renderer) (id (eql :SPACE)) node)
  (format nil "(space ~(~a~) ~a)" (getattr node :level) (getattr node :rank)))
(defmethod %render-node ((renderer Sexp-Renderer) (id (eql :INDEX-COMPONENTS)) node)
  ;; flattened to the linear index of the element being computed, as every renderer does (renderer.lisp:194-221)
  (render-expr 'Sexp-Renderer (expr-index-components renderer node (renderer-index-space renderer))))
(defmethod %render-node ((renderer Sexp-Renderer) (id (eql :Aref)) node)
  ;; (aref ID INDEX) with the flat index sum_d stride_d * (from_d + by_d * gid_d) (clang.lisp:82-97); a scalar is (aref ID)
  (let ((index (render-aref-index renderer node)))
    (if index
        (format nil "(aref ~(~a~) ~a)" (getattr node :storage-id) index)
        (format nil "(aref ~(~a~))" (getattr node :storage-id)))))

(defun sexp (expr &optional index-space) (render-expr 'Sexp-Renderer expr :index-space index-space))

(defun write-sexp (name b is iterations)
  "The destination of an :EXPR as CLANG's print-aref addresses it (clang.lisp:84-101)."
  (if (and is (not (= -1 (buffer-nrank b))) (> (length (iteration-space-shape is)) 0) (> (length iterations) 0))
      (format nil "(aref ~(~a~) ~a)" name
              (sexp (apply #'expr-add
                           (map 'list
                                #'(lambda (view stride i)
                                    (if view
                                        (expr-mul stride (expr-add (expr-const (car view) :int64) (expr-mul (expr-const (third view) :int64) i)))
                                        (expr-mul stride i)))
                                (iteration-space-views is) (iteration-space-strides is) iterations))))
      (format nil "(aref ~(~a~))" name)))

(defun bp-sexp (bp out)
  (ecase (node-type bp)
    (:DEFINE-GLOBAL
     (format out "  (define-global ~(~a~) ~(~a~) ~a ~(~a~) ~a)~%" (car (node-writes bp)) (getattr bp :dtype)
             (if (getattr bp :pointer-p) "t" "nil") (getattr bp :type) (getattr bp :nrank)))
    (:FOR
     (format out "  (for ~(~a~) ~a ~a ~a ~(~a~))~%" (getattr bp :idx) (sexp (getattr bp :upfrom)) (sexp (getattr bp :below))
             (sexp (getattr bp :by)) (or (getattr bp :scope) :local)))
    (:ENDFOR (format out "  (endfor ~(~a~))~%" (getattr bp :idx)))
    (:IF (format out "  (if ~a)~%" (sexp (getattr bp :condition))))
    (:ENDIF (format out "  (endif)~%"))
    (:EXPR
     (let ((iterations (getattr bp :iterations))
           (type (read-type-relay bp)))
       (format out "  (expr (~{~a~^ ~}) ~a :dtype ~(~a~)~a~a~a)~%"
               (map 'list #'(lambda (x y z) (write-sexp x y z iterations)) (node-writes bp) (relay-writes type) (relay-write-iters type))
               (sexp (getattr bp :EXPR) iterations)
               (buffer-dtype (car (relay-writes type)))
               (if (car (getattr bp :declare-type)) " :declare t" "")
               (if (getattr bp :reduction :allow-undefined t) " :reduction t" "")
               ;; an index the GLOBAL directive bound to blockIdx / threadIdx brings the launch size of its axis
               ;; (source/codegen/auto-scheduler/directive.lisp:94-117; Metal gathers them with blueprint-gather-grids)
               (let ((meta (getattr bp :meta :allow-undefined t)))
                 (if (typep meta 'ExprGrid)
                     (format nil " :grid (~a ~a ~a)" (exprgrid-rank meta) (sexp (exprgrid-global-size meta)) (sexp (exprgrid-local-size meta)))
                     "")))))))

(defclass Hip-Program ()
  ((name :initarg :name :accessor hp-name)
   (handle :initarg :handle :accessor hp-handle :documentation "cthip_program_create's object")
   (args :initarg :args :accessor hp-args :documentation "the item's DEFINE-GLOBAL nodes, in argument order")
   (uploads :initform (make-hash-table :test #'eq) :accessor hp-uploads)))

(defvar *programs* (make-hash-table :test #'equal) "kernel name -> Hip-Program, from %render-kernel to %compile-kernel")

(defmethod %render-kernel ((renderer Hip-Renderer) si)
  (ensure-foreign-library)
  (let ((text (with-output-to-string (out)
                (format out "(item ~(~a~)~%" (getattr si :name))
                (dolist (bp (getattr si :blueprint)) (bp-sexp bp out))
                (format out ")~%"))))
    (with-foreign-object (program :pointer)
      (unless (zerop (%program-create program text))
        (error "Caten[HIP]: cannot render ~a: ~a~%~a" (getattr si :name) (%last-error) text))
      (setf (gethash (string-downcase (princ-to-string (getattr si :name))) *programs*)
            (make-instance 'Hip-Program :name (getattr si :name) :handle (mem-ref program :pointer)
                                        :args (schedule-item-args si)))
      (%program-source (mem-ref program :pointer)))))

;;; ~~~ launch ~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~
(defmethod runtime-invoke-jit-kernel ((runtime HipRuntime) kernel-info node args)
  (apply (caten/codegen/jit:compiled-kernel-caller kernel-info) runtime node args))

(defun device-pointer-of (hp runtime buf)
  "Weights loaded from GGUF are LispBuffers whatever BACKEND is (external/gguf/tensor-info.lisp:104-120)
and enter through :Allocate :from untouched (source/runtime/runtime.lisp:228-243): upload once, cache."
  (cond
    ((typep buf 'HipBuffer) (device-pointer buf))
    ((and (buffer-p buf) (arrayp (buffer-value buf)))
     (or (gethash buf (hp-uploads hp))
         (let ((dev (make-buffer (buffer-shape buf) (buffer-stride buf) (buffer-dtype buf) (buffer-views buf) :device 'HipBuffer)))
           (open-buffer runtime dev)
           (transfer-from-array runtime dev (buffer-value buf))
           (setf (gethash buf (hp-uploads hp)) (device-pointer dev)))))
    (t (error "Caten[HIP]: ~a is neither a device buffer nor a host array" buf))))

(defmethod invoke ((hp Hip-Program) runtime node &rest buffers)
  (declare (ignore node))
  (assert (= (length buffers) (length (hp-args hp))) ()
          "HIP: the number of arguments does not match the kernel ~a" (hp-name hp))
  (let ((n (length buffers))
        (cells nil)) ; (buffer cell dtype): rank-0 values passed by pointer
    (with-foreign-objects ((argv :pointer n) (slots :uint64 n))
      (unwind-protect
           (progn
             (loop for buf in buffers
                   for arg in (hp-args hp)
                   for dtype = (getattr arg :dtype)
                   for nth upfrom 0
                   for slot = (mem-aptr slots :uint64 nth) do
                     (cond
                       ((and (buffer-p buf) (> (buffer-nrank buf) 0))
                        (setf (mem-ref slot :pointer) (device-pointer-of hp runtime buf)))
                       ((getattr arg :pointer-p)
                        ;; A rank-0 value declared as a pointer (every output is, rewriting-rules.lisp:207-231).  CLANG
                        ;; boxes the number in a one-element foreign object and stores the result back after the
                        ;; call (clang.lisp:166-185); here the box is an 8-byte device cell.
                        (with-foreign-objects ((cell :pointer) (host :uint64))
                          (check (%alloc cell 8))
                          (setf (mem-ref host (->cffi-dtype dtype)) (if (buffer-p buf) (buffer-value buf) buf))
                          (check (%h2d (mem-ref cell :pointer) host (dtype/size-of dtype)))
                          (push (list buf (mem-ref cell :pointer) dtype) cells)
                          (setf (mem-ref slot :pointer) (mem-ref cell :pointer))))
                       (t
                        ;; rank-0 by value with its declared dtype (coerce-dtyped-buffer already cast it, runner.lisp:25)
                        (setf (mem-ref slot (->cffi-dtype dtype)) (if (buffer-p buf) (buffer-value buf) buf))))
                     (setf (mem-aref argv :pointer nth) slot))
             (check (%program-launch (hp-handle hp) argv n))
             (loop for (buf cell dtype) in cells
                   when (buffer-p buf) do
                     (with-foreign-object (host :uint64)
                       (check (%d2h host cell (dtype/size-of dtype))) ; synchronises, as the CLANG call does
                       (setf (buffer-value buf) (mem-ref host (->cffi-dtype dtype))))))
        (loop for (nil cell nil) in cells do (%free cell))))))

(defun make-hip-caller (hp) `(lambda (runtime node &rest args) (apply #'invoke ,hp runtime node args)))

(defmethod %compile-kernel ((renderer Hip-Renderer) items dir)
  (declare (ignore dir))
  (ensure-foreign-library)
  (let ((code (apply #'concatenate 'string
                     (append (list (%render-header))
                             (loop for item in items
                                   if (getattr item :rendered-object) collect (getattr item :rendered-object))))))
    (when (>= (ctx:getenv :JIT_DEBUG) 3) (format t "[Final Code]:~%~a~%" code))
    (with-foreign-objects ((blob :pointer) (size :size) (log :pointer) (module :pointer))
      (unless (zerop (%compile code "gfx950" blob size log))
        (error "Caten[HIP]: Failed to compile the kernels:~%~a~%Compiled with hipRTC --offload-arch=gfx950 -O3"
               (if (null-pointer-p (mem-ref log :pointer)) (%last-error) (foreign-string-to-lisp (mem-ref log :pointer)))))
      (check (%module-load module (mem-ref blob :pointer)))
      (%release (mem-ref blob :pointer))
      (setf (hip-renderer-module renderer) (mem-ref module :pointer))
      (loop for item in items
            if (getattr item :rendered-object) do
              (let ((hp (gethash (string-downcase (princ-to-string (getattr item :name))) *programs*)))
                (assert hp () "Caten[HIP]: ~a was not rendered by this backend" (getattr item :name))
                (check (%program-bind (hp-handle hp) (mem-ref module :pointer)))
                (setf (getattr item :compiled-object) (make-hip-caller hp)))))
    nil))

;;; ~~~ the dequant-in-register Linear as a custom op ~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~~
;; Caten's second extension mechanism (source/runtime/runtime.lisp:118): a node that is not JITAble is isolated by
;; the scheduler as a VM instruction (source/codegen/scheduler.lisp:99-102,573-576) and realised by a method on
;; the runtime class; the precedent is the test-only Custom/LazyApply (source/test-suite/test-activations.lisp:4-14).
;; :QLinear is  y = act(prologue(x) @ W^T + bias) + residual  on a weight kept PACKED (GGUF Q8_0 / Q4_0 / F16 / F32
;; blocks), i.e. what external/gguf/dequantize.lisp + nn/linear.lisp compute without the fp32 copy of W.
(defparameter +ggml-type-ids+ '(:f32 0 :f16 1 :q4_0 2 :q8_0 8))          ; external/gguf/tensor-info.lisp:3-31
(defparameter +acts+ '(:none 0 :relu 1 :gelu 2 :silu 3 :sigmoid 4 :tanh 5))
(defparameter +prologues+ '(:none 0 :layernorm 1 :rmsnorm 2 :swiglu 3))

(defnode (:HIP :QLinear) ()
         "y[m, out] = act(prologue(x[m, in]) @ W^T + bias) + residual.  reads: y, packed weight handle, x, then the
optional bias, residual, norm-g, norm-b in that order (absent ones are left out from the end)."
         :slots ((act :type keyword) (prologue :type keyword) (eps :type single-float)
                 (has-bias :type boolean) (has-residual :type boolean) (has-norm :type boolean)))

(defclass PackedWeight ()
  ((handle :initarg :handle :accessor packed-weight-handle)
   (rows :initarg :rows :reader packed-weight-rows)
   (cols :initarg :cols :reader packed-weight-cols))
  (:documentation "A GGUF tensor uploaded as it sits in the file and re-laid into quant / scale planes (cthip_wmat_create)."))

(defun make-packed-weight (runtime ggml-type raw-bytes rows cols)
  "raw-bytes: (simple-array (unsigned-byte 8)) holding the tensor's GGUF blocks (what tensor-info->tensor reads,
external/gguf/tensor-info.lisp:104-120, before it would dequantise them)."
  (declare (ignore runtime))
  (with-foreign-objects ((dev :pointer) (wmat :pointer))
    (check (%alloc dev (length raw-bytes)))
    (with-pointer-to-vector-data (src raw-bytes)
      (check (%h2d (mem-ref dev :pointer) src (length raw-bytes))))
    (check (%wmat-create wmat (getf +ggml-type-ids+ ggml-type) (mem-ref dev :pointer) rows cols))
    (check (%free (mem-ref dev :pointer))) ; the planes are a copy; stream order keeps the block alive until they are written
    (make-instance 'PackedWeight :handle (mem-ref wmat :pointer) :rows rows :cols cols)))

(defun fold-layernorm (weight gamma beta &optional bias)
  "A LayerNorm in front of this Linear is carried through the product from now on (cthip_wmat_fold_layernorm): later
:QLinear nodes with prologue :layernorm and these same gamma / beta / bias buffers need the row statistics only in
their epilogue."
  (check (%wmat-fold-layernorm (packed-weight-handle weight) (device-pointer gamma) (device-pointer beta)
                               (if bias (device-pointer bias) (null-pointer)))))

(defmethod realize-node ((id (eql :QLinear)) (runtime HipRuntime) node args)
  (let* ((y (first args))
         (w (second args))
         (x (third args))
         (rest (cdddr args))
         (bias (when (getattr node :has-bias) (pop rest)))
         (residual (when (getattr node :has-residual) (pop rest)))
         (norm-g (when (getattr node :has-norm) (pop rest)))
         (norm-b (when (and (getattr node :has-norm) rest) (pop rest)))
         (m (/ (buffer-storage-size x) (* (packed-weight-cols (buffer-value w))
                                          (if (eql (getattr node :prologue) :swiglu) 2 1)))))
    (flet ((ptr (b) (if b (device-pointer b) (null-pointer))))
      (check (%linear (device-pointer y) (packed-weight-handle (buffer-value w)) (device-pointer x) m
                      (ptr bias) (ptr residual) (getf +acts+ (getattr node :act)) (getf +prologues+ (getattr node :prologue))
                      (ptr norm-g) (ptr norm-b) (getattr node :eps))))
    y))

;; The graph-level function: a Func whose lower emits the node (source/api/tensor.lisp; cf. Custom/LazyApply).
(defclass QLinearFunc (caten/api:Func)
  ((act :initarg :act :initform :none) (prologue :initarg :prologue :initform :none) (eps :initarg :eps :initform 1e-5)
   (has-bias :initarg :has-bias :initform nil) (has-residual :initarg :has-residual :initform nil)
   (has-norm :initarg :has-norm :initform nil)))
(defmethod caten/api:forward ((op QLinearFunc) &rest inputs)
  ;; inputs: y (the output placeholder, (m out)), the weight holder, x, ...
  (caten/api:make-tensor (caten/api:shape (first inputs)) :dtype (caten/api:dtype-of (first inputs)) :order (caten/api:order (first inputs))))
(defmethod caten/api:backward ((op QLinearFunc) &optional prev-grad) (declare (ignore prev-grad)) nil)
(defmethod caten/api:lower ((op QLinearFunc) &rest inputs)
  (with-slots (act prologue eps has-bias has-residual has-norm) op
    (caten/air:with-context
      (_ (caten/air:make-node :HIP :QLinear (list (gensym "QLINEAR")) inputs
                              :act act :prologue prologue :eps eps
                              :has-bias has-bias :has-residual has-residual :has-norm has-norm)))))

(defun !qlinear (y weight x &key bias residual norm-g norm-b (act :none) (prologue :none) (eps 1e-5))
  "act(prologue(x) @ W^T + bias) + residual with W a PackedWeight wrapped in a rank-0 tensor; y receives the result."
  (apply #'caten/api:forward
         (make-instance 'QLinearFunc :act act :prologue prologue :eps eps
                                     :has-bias (and bias t) :has-residual (and residual t) :has-norm (and norm-g t))
         (remove nil (list y weight x bias residual norm-g norm-b))))
