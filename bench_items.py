#!/usr/bin/env python3
"""Timings of the single fused items on one MI355X (`python bench_items.py`):
the benchmark configurations `!relu(!matmul A B)` at 1024^3 fp32 and the row ops (LayerNorm -> softmax and
GELU(tanh) over fp32 (64,1024,768)), each against the roofline that bounds it; the row ops also against a
device-to-device copy of the same array, the streaming rate this box actually reaches.  HIP events on the
library's stream; inputs resident on the device.  Every timed item's output is checked on sampled rows against an
fp64 NumPy evaluation of the same formula before its figure is printed."""
from __future__ import annotations

import ctypes as C
import json

import numpy as np

import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

from caten_amd import _lib  # noqa: E402
from caten_amd.ops import DeviceArray  # noqa: E402


def _check(name, got, want, rtol=1e-3, atol=1e-4):
    bad = np.abs(got.astype(np.float64) - want) > atol + rtol * np.abs(want)
    if bad.any():
        raise SystemExit(f"bench_items: {name}: {int(bad.sum())} of {bad.size} sampled values are off "
                         f"(max abs err {np.abs(got - want).max():.3e}); no figure is reported for a wrong result")



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


def measure(rendered_items: bool = True):
    """Every figure as a dict.  `rendered_items` False leaves out the blueprint-rendered variants of the row ops (and
    their hipRTC compilation) and times the hand-written items only."""
    lib = _lib.init(0)
    rng = np.random.default_rng(0)
    out = []
    # ---- config 1 ----
    n = 1024
    Ah = rng.uniform(-1, 1, (n, n)).astype(np.float32)
    Bh = rng.uniform(-1, 1, (n, n)).astype(np.float32)
    A, B = DeviceArray.from_numpy(Ah), DeviceArray.from_numpy(Bh)
    Cm = DeviceArray((n, n), np.float32)
    sample = rng.choice(n, 32, replace=False)
    want_c = np.maximum(Ah[sample].astype(np.float64) @ Bh.astype(np.float64), 0.0)
    for prec, name, peak in ((0, "fp32 MFMA", 157.3), (3, "bf16 MFMA, operands split in 3 terms (6 MFMAs per product), fp32 acc", 2500.0),
                             (2, "bf16 MFMA, operands split in 2 terms (3 MFMAs per product), fp32 acc", 2500.0),
                             (1, "bf16 MFMA / fp32 acc", 2500.0)):
        us = _time(lib, lambda: _lib.check(lib.cthip_matmul(Cm.ptr, A.ptr, B.ptr, n, n, n, _lib.ACT_RELU, prec)))
        tf = 2.0 * n ** 3 / (us * 1e-6) / 1e12
        got_c = Cm.numpy()[sample]
        if prec == 1:
            # operands rounded to bf16: 2^-9 per operand over 1024 random-sign products is not an element-wise 1e-2
            # band around outputs near zero; the check is the error of the sampled rows as a whole
            rel = np.linalg.norm(got_c - want_c) / np.linalg.norm(want_c)
            if not rel < 1e-2:
                raise SystemExit(f"bench_items: relu(matmul) {name}: relative error {rel:.3e} of the sampled rows")
        else:
            _check(f"relu(matmul) {name}", got_c, want_c, 1e-3, 1e-3 if prec == 2 else 1e-4)  # two terms lose 2^-16 of each product
        out.append({"item": f"relu(matmul) 1024^3 {name}", "us": us, "achieved": tf, "unit": "TFLOP/s", "peak": peak,
                    "frac": tf / peak})
    # ---- config 2 ----
    rows, d = 64 * 1024, 768
    xh = rng.standard_normal((rows, d), dtype=np.float32)
    gh, bh = rng.normal(1, 0.02, d).astype(np.float32), rng.normal(0, 0.02, d).astype(np.float32)
    x = DeviceArray.from_numpy(xh)
    y = DeviceArray((rows, d), np.float32)
    g = DeviceArray.from_numpy(gh)
    b = DeviceArray.from_numpy(bh)
    nbytes = 2.0 * rows * d * 4
    rs = rng.choice(rows, 64, replace=False)
    xs = xh[rs].astype(np.float64)
    ln = (xs - xs.mean(-1, keepdims=True)) / np.sqrt(xs.var(-1, keepdims=True) + 1e-5) * gh + bh

    def softmax64(v):
        e = np.exp(v - v.max(-1, keepdims=True))
        return e / e.sum(-1, keepdims=True)
    want = {"LayerNorm->softmax": softmax64(ln), "LayerNorm (": ln, "softmax (": softmax64(xs),
            "GELU": 0.5 * xs * (1 + np.tanh(np.sqrt(2 / np.pi) * (xs + 0.044715 * xs ** 3)))}
    items = [
        ("LayerNorm->softmax fused (64,1024,768)", lambda: _lib.check(lib.cthip_layernorm_softmax(y.ptr, x.ptr, g.ptr, b.ptr, 1e-5, rows, d))),
        ("GELU(tanh) (64,1024,768)", lambda: _lib.check(lib.cthip_unary(_lib.ACT_GELU, y.ptr, x.ptr, rows * d))),
        ("LayerNorm (64,1024,768)", lambda: _lib.check(lib.cthip_layernorm(y.ptr, x.ptr, g.ptr, b.ptr, 1e-5, rows, d))),
        ("softmax (64,1024,768)", lambda: _lib.check(lib.cthip_softmax(y.ptr, x.ptr, rows, d))),
    ]
    # the streaming ceiling of this box: a device-to-device copy of the same array (the same bytes read and written)
    copy_us = _time(lib, lambda: _lib.check(lib.cthip_d2d(y.ptr, x.ptr, rows * d * 4)))
    if not np.array_equal(y.numpy()[rs], xh[rs]):
        raise SystemExit("bench_items: the device-to-device copy did not copy")
    copy_gbs = nbytes / (copy_us * 1e-6) / 1e9
    out.append({"item": "device-to-device copy (64,1024,768): the measured streaming ceiling", "us": copy_us, "achieved": copy_gbs,
                "unit": "GB/s", "peak": 8000.0, "frac": copy_gbs / 8000.0, "bytes": nbytes})
    if rendered_items:
        # the same softmax as a RENDERED kernel: blueprint -> HIP source (one wavefront per row) -> hipRTC
        from caten_amd import blueprints
        from caten_amd.renderer import HipRenderer
        from caten_amd.buffer import HipBuffer

        it = blueprints.softmax_rows()  # dynamic shape: rows and n are arguments
        its = blueprints.softmax_rows("fused_softmax_static", rows, d)  # static shape: the bounds are literals
        rr = HipRenderer()
        rr.render_kernel(it)
        rr.render_kernel(its)
        rr.compile_kernel([it, its])
        # buffers over the same device arrays the hand-written items use
        bx = HipBuffer(shape=[rows, d], stride=[d, 1], dtype="float32", nrank=2, value=x.ptr)
        by = HipBuffer(shape=[rows, d], stride=[d, 1], dtype="float32", nrank=2, value=y.ptr)
        items.append(("softmax (64,1024,768), its blueprint through the program interface (routed to the row kernel), dynamic shape",
                      lambda: it["compiled_object"](None, by, rows, d, bx)))

        def rendered(item, *args):
            def run():
                _lib.check(lib.cthip_set_option(b"render_routes", 0))
                try:
                    item["compiled_object"](None, *args)
                finally:
                    _lib.check(lib.cthip_set_option(b"render_routes", 1))
            return run
        items.append(("softmax (64,1024,768), RENDERED from its blueprint, dynamic shape", rendered(it, by, rows, d, bx)))
        items.append(("softmax (64,1024,768), RENDERED from its blueprint, static shape", rendered(its, by, bx)))
        # GELU(tanh) as a RENDERED element-wise kernel (there is no route for it: this is what an item of that shape runs)
        ig = blueprints.gelu_tanh()
        igs = blueprints.gelu_tanh("fused_gelu_static", rows, d)
        rr.render_kernel(ig)
        rr.render_kernel(igs)
        rr.compile_kernel([ig, igs])
        items.append(("GELU(tanh) (64,1024,768), RENDERED from its blueprint, dynamic shape", lambda: ig["compiled_object"](None, by, rows, d, bx)))
        items.append(("GELU(tanh) (64,1024,768), RENDERED from its blueprint, static shape", lambda: igs["compiled_object"](None, by, bx)))
        # LayerNorm -> softmax as ONE rendered item (five loops over the row)
        bg = HipBuffer(shape=[d], stride=[1], dtype="float32", nrank=1, value=g.ptr)
        bb = HipBuffer(shape=[d], stride=[1], dtype="float32", nrank=1, value=b.ptr)
        il = blueprints.layernorm_softmax_rows()
        ils = blueprints.layernorm_softmax_rows("fused_layernorm_softmax_static", 1e-5, rows, d)
        rr.render_kernel(il)
        rr.render_kernel(ils)
        rr.compile_kernel([il, ils])
        items.append(("LayerNorm->softmax (64,1024,768), RENDERED from its blueprint, dynamic shape",
                      lambda: il["compiled_object"](None, by, rows, d, bx, bg, bb)))
        items.append(("LayerNorm->softmax (64,1024,768), RENDERED from its blueprint, static shape",
                      lambda: ils["compiled_object"](None, by, bx, bg, bb)))
    for name, fn in items:
        us = _time(lib, fn)
        key = [k for k in want if name.startswith(k)]
        _check(name, y.numpy()[rs], want[key[0]] if key else want["softmax ("], 1e-3, 1e-5)
        gbs = nbytes / (us * 1e-6) / 1e9
        out.append({"item": name, "us": us, "achieved": gbs, "unit": "GB/s", "peak": 8000.0, "frac": gbs / 8000.0,
                    "frac_of_copy": gbs / copy_gbs, "bytes": nbytes})
    for a in (A, B, Cm, x, y, g, b):
        a.free()
    return out


def main():
    for o in measure():
        print(json.dumps(o))


if __name__ == "__main__":
    main()
