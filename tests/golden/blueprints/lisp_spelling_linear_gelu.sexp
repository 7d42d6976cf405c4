; c_fc of FeedForward fused with its bias and GeLU :tanh (external/llm/layers.lisp:53-59, nn/activations.lisp:202-215;
; "matmul -> gelu -> matmul = 2 kernels", source/test-suite/test-scheduler.lisp:140-163), constants as single floats
; (0.7978846, 0.044715) and 1/ln 2 as a double with a d0 marker, operands of the commutative nodes in another order
; than the Python mirror prints them.
(ITEM FUSED_LINEAR_GELU
  (DEFINE-GLOBAL VAL_8 FLOAT32 T OUTPUT 3)
  (DEFINE-GLOBAL S INT64 NIL SHAPE 0)
  (DEFINE-GLOBAL VAL_0 FLOAT32 T INPUT 3)
  (DEFINE-GLOBAL VAL_1 FLOAT32 T INPUT 2)
  (DEFINE-GLOBAL VAL_2 FLOAT32 T INPUT 1)
  (FOR _GID0 0 (< _GID0 S) 1 LOCAL)
  (FOR _GID1 0 (< _GID1 3072) 1 LOCAL)
  (EXPR ((AREF VAL_3)) 0.0 :DTYPE FLOAT32 :DECLARE T)
  (FOR _GID2 0 (< _GID2 768) 1 LOCAL)
  (EXPR ((AREF VAL_3)) (ADD (MUL (AREF VAL_0 (ADD (MUL 768 _GID0) _GID2)) (AREF VAL_1 (ADD (MUL 768 _GID1) _GID2))) VAL_3) :DTYPE FLOAT32 :REDUCTION T)
  (ENDFOR _GID2)
  (EXPR ((AREF VAL_8 (ADD (MUL 3072 _GID0) _GID1))) (MUL (ADD 1.0 (ADD (MUL 2.0 (RECIP (ADD (EXP2 (MUL (MUL (MUL (ADD (MUL (MUL (MUL (ADD (AREF VAL_2 _GID1) VAL_3) (ADD (AREF VAL_2 _GID1) VAL_3)) (ADD (AREF VAL_2 _GID1) VAL_3)) 0.044715) (ADD (AREF VAL_2 _GID1) VAL_3)) 0.7978846) 2.0) -1.4426950408889634d0)) 1.0))) -1.0)) (MUL (ADD (AREF VAL_2 _GID1) VAL_3) 0.5)) :DTYPE FLOAT32)
  (ENDFOR _GID1)
  (ENDFOR _GID0))
