; (apply #'!matmul (multiple-value-list (!chunk (make-tensor `(2 64 64)) 2))): the batched four-loop nest whose
; reduction the reference's own test renders as
;   (val_2+(val_4[(((4096*a)+(64*b))+d)]*val_4[(((4096*(1+a))+c)+(64*d))]))
; (source/test-suite/test-scheduler.lisp:117-138): both operands are chunks of ONE buffer, the second one starts
; 4096 elements in.  Index expressions verbatim; loop indices named as that test names them; symbols and keywords
; in upper case, floats with exponent markers, as a Lisp printer may leave them.
(ITEM FUSED_MATMUL_CHUNK
  (DEFINE-GLOBAL VAL_5 FLOAT32 T OUTPUT 3)
  (DEFINE-GLOBAL VAL_4 FLOAT32 T INPUT 3)
  (FOR A 0 (< A 1) 1 LOCAL)
  (FOR B 0 (< B 64) 1 LOCAL)
  (FOR C 0 (< C 64) 1 LOCAL)
  (EXPR ((AREF VAL_2)) 0.0f0 :DTYPE FLOAT32 :DECLARE T)
  (FOR D 0 (< D 64) 1 LOCAL)
  (EXPR ((AREF VAL_2)) (ADD VAL_2 (MUL (AREF VAL_4 (ADD (ADD (MUL 4096 A) (MUL 64 B)) D)) (AREF VAL_4 (ADD (ADD (MUL 4096 (ADD 1 A)) C) (MUL 64 D))))) :DTYPE FLOAT32 :REDUCTION T)
  (ENDFOR D)
  (EXPR ((AREF VAL_5 (ADD (ADD (MUL 4096 A) (MUL 64 B)) C))) VAL_2 :DTYPE FLOAT32)
  (ENDFOR C)
  (ENDFOR B)
  (ENDFOR A))
