"""Timings of the single fused items on one MI355X (`python -m caten_amd.bench_items`):
the benchmark configurations `!relu(!matmul A B)` at 1024^3 fp32 and the row ops (LayerNorm -> softmax and
GELU(tanh) over fp32 (64,1024,768)), each against the roofline that bounds it.  HIP events on the
library's stream; inputs resident on the device."""
from __future__ import annotations

import ctypes as C
import json

import numpy as np

from . import _lib
from .ops import DeviceArray


def _time(lib, fn, reps=50, warm=5):
    for _ in range(warm):
        fn()
    _lib.check(lib.cthip_sync())
    _lib.check(lib.cthip_timer_start())
    for _ in range(reps):
        fn()
    ms = C.c_float()
    _lib.check(lib.cthip_timer_stop(C.byref(ms)))
    return ms.value * 1e3 / reps  # us


def main():
    lib = _lib.init(0)
    rng = np.random.default_rng(0)
    out = []
    # ---- config 1 ----
    n = 1024
    A = DeviceArray.from_numpy(rng.uniform(-1, 1, (n, n)).astype(np.float32))
    B = DeviceArray.from_numpy(rng.uniform(-1, 1, (n, n)).astype(np.float32))
    Cm = DeviceArray((n, n), np.float32)
    for prec, name, peak in ((0, "fp32 MFMA", 157.3), (3, "bf16 MFMA, operands split in 3 terms (6 MFMAs per product), fp32 acc", 2500.0),
                             (2, "bf16 MFMA, operands split in 2 terms (3 MFMAs per product), fp32 acc", 2500.0),
                             (1, "bf16 MFMA / fp32 acc", 2500.0)):
        us = _time(lib, lambda: _lib.check(lib.cthip_matmul(Cm.ptr, A.ptr, B.ptr, n, n, n, _lib.ACT_RELU, prec)))
        tf = 2.0 * n ** 3 / (us * 1e-6) / 1e12
        out.append({"item": f"relu(matmul) 1024^3 {name}", "us": us, "achieved": tf, "unit": "TFLOP/s", "peak": peak,
                    "frac": tf / peak})
    # ---- config 2 ----
    rows, d = 64 * 1024, 768
    x = DeviceArray.from_numpy(rng.normal(0, 1, (rows, d)).astype(np.float32))
    y = DeviceArray((rows, d), np.float32)
    g = DeviceArray.from_numpy(rng.normal(1, 0.02, d).astype(np.float32))
    b = DeviceArray.from_numpy(rng.normal(0, 0.02, d).astype(np.float32))
    nbytes = 2.0 * rows * d * 4
    items = [
        ("LayerNorm->softmax fused (64,1024,768)", lambda: _lib.check(lib.cthip_layernorm_softmax(y.ptr, x.ptr, g.ptr, b.ptr, 1e-5, rows, d))),
        ("GELU(tanh) (64,1024,768)", lambda: _lib.check(lib.cthip_unary(_lib.ACT_GELU, y.ptr, x.ptr, rows * d))),
        ("LayerNorm (64,1024,768)", lambda: _lib.check(lib.cthip_layernorm(y.ptr, x.ptr, g.ptr, b.ptr, 1e-5, rows, d))),
        ("softmax (64,1024,768)", lambda: _lib.check(lib.cthip_softmax(y.ptr, x.ptr, rows, d))),
    ]
    # the same softmax as a RENDERED kernel: blueprint -> HIP source (one wavefront per row) -> hipRTC
    from . import blueprints
    from .renderer import HipRenderer
    from .buffer import HipBuffer

    it = blueprints.softmax_rows()  # dynamic shape: rows and n are arguments
    its = blueprints.softmax_rows("fused_softmax_static", rows, d)  # static shape: the bounds are literals
    rr = HipRenderer()
    rr.render_kernel(it)
    rr.render_kernel(its)
    rr.compile_kernel([it, its])
    # buffers over the same device arrays the hand-written items use
    bx = HipBuffer(shape=[rows, d], stride=[d, 1], dtype="float32", nrank=2, value=x.ptr)
    by = HipBuffer(shape=[rows, d], stride=[d, 1], dtype="float32", nrank=2, value=y.ptr)
    items.append(("softmax (64,1024,768), RENDERED from its blueprint, dynamic shape", lambda: it["compiled_object"](None, by, rows, d, bx)))
    items.append(("softmax (64,1024,768), RENDERED from its blueprint, static shape", lambda: its["compiled_object"](None, by, bx)))
    for name, fn in items:
        us = _time(lib, fn)
        gbs = nbytes / (us * 1e-6) / 1e9
        out.append({"item": name, "us": us, "achieved": gbs, "unit": "GB/s", "peak": 8000.0, "frac": gbs / 8000.0,
                    "bytes": nbytes})
    for o in out:
        print(json.dumps(o))


if __name__ == "__main__":
    main()
