(item fused_triu_mask
  (define-global val_mask float32 t output 4)
  (define-global s int64 nil shape 0)
  (define-global n int64 nil shape 0)
  (for _gid0 0 (< _gid0 s) 1 local)
  (for _gid1 0 (< _gid1 (add n s)) 1 local)
  (expr ((aref val_mask (add (mul (add n s) _gid0) _gid1))) (where (not (< (add _gid1 (neg (add 1 n))) _gid0)) -inf 0.0) :dtype float32)
  (endfor _gid1)
  (endfor _gid0))
