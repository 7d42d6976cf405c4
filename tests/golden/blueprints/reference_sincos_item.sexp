(item fused_sin_sin_add_load_load6914144
  (define-global val_6 float32 t output 0)
  (expr ((aref val_6 0)) (sin (sin (add 1.0 1.5707964))) :dtype float32))
