"""NumPy-in / NumPy-out front-ends of the hand-written fused items.

Each function uploads its operands, calls the C ABI (include/caten_hip.h) and
downloads the result; they exist so that tests and examples read like the
reference's own (`(proceed (!softmax x))` ...).  The hot path itself (the decoder
session, `caten_amd.llm`) keeps everything resident on the device.
"""
from __future__ import annotations

import ctypes as C
from typing import Optional

import numpy as np

from . import _lib
from .quant import packed_nbytes


class DeviceArray:
    """A flat device allocation from the caching allocator holding a NumPy-typed array."""

    def __init__(self, shape, dtype=np.float32):
        self.shape = tuple(int(s) for s in np.atleast_1d(shape)) if not isinstance(shape, tuple) else shape
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape)) * self.dtype.itemsize
        p = C.c_void_p()
        _lib.check(_lib.init().cthip_alloc(C.byref(p), self.nbytes))
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, a) -> "DeviceArray":
        a = np.ascontiguousarray(a)
        d = cls(a.shape, a.dtype)
        if a.nbytes:
            _lib.check(_lib.load().cthip_h2d(d.ptr, a.ctypes.data, a.nbytes))
        return d

    def numpy(self) -> np.ndarray:
        out = np.empty(self.shape, self.dtype)
        _lib.check(_lib.load().cthip_d2h(out.ctypes.data if out.nbytes else None, self.ptr, out.nbytes))
        return out

    def free(self):
        if self.ptr:
            _lib.check(_lib.load().cthip_free(self.ptr))
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def _dev(a, dtype=np.float32) -> Optional[DeviceArray]:
    return None if a is None else DeviceArray.from_numpy(np.asarray(a, dtype=dtype))


def _p(d: Optional[DeviceArray]):
    return None if d is None else d.ptr


def dequantize(kind: str, raw, n: int) -> np.ndarray:
    """caten/gguf:dequantize (external/gguf/dequantize.lisp:14-53) on the device."""
    raw = np.ascontiguousarray(np.asarray(raw).view(np.uint8).ravel())
    d_raw = DeviceArray.from_numpy(raw)
    out = DeviceArray((n,), np.float32)
    _lib.check(_lib.load().cthip_dequant(_lib.GGML_TYPE[kind], d_raw.ptr, n, out.ptr))
    return out.numpy()


class WeightMatrix:
    """A Linear weight (rows=out, cols=in) kept packed in HBM (cthip_wmat_*)."""

    def __init__(self, kind: str, raw, rows: int, cols: int):
        raw = np.ascontiguousarray(np.asarray(raw).view(np.uint8).ravel())
        want = packed_nbytes(kind, rows * cols)
        if raw.size != want:
            raise ValueError(f"WeightMatrix: {raw.size} bytes given, a {kind} ({rows},{cols}) matrix has {want}")
        self.kind, self.rows, self.cols = kind, rows, cols
        d_raw = DeviceArray.from_numpy(raw)
        h = C.c_void_p()
        _lib.check(_lib.init().cthip_wmat_create(C.byref(h), _lib.GGML_TYPE[kind], d_raw.ptr, rows, cols))
        self.handle = h
        d_raw.free()

    @property
    def nbytes(self) -> int:
        return int(_lib.load().cthip_wmat_nbytes(self.handle))

    def dequantize(self) -> np.ndarray:
        out = DeviceArray((self.rows, self.cols), np.float32)
        _lib.check(_lib.load().cthip_wmat_dequant(self.handle, out.ptr))
        return out.numpy()

    def fold_layernorm(self, gamma, beta, bias=None) -> None:
        """cthip_wmat_fold_layernorm: keeps device copies of gamma / beta / bias (the fold is keyed on their
        addresses) and prepares LayerNorm(gamma, beta) in front of this Linear to go through the product."""
        self._fold = (_dev(np.ascontiguousarray(gamma, np.float32)), _dev(np.ascontiguousarray(beta, np.float32)),
                      _dev(None if bias is None else np.ascontiguousarray(bias, np.float32)))
        dg, db, dbias = self._fold
        _lib.check(_lib.load().cthip_wmat_fold_layernorm(self.handle, dg.ptr, db.ptr, _p(dbias)))

    def linear_folded(self, x, act=None, eps: float = 1e-5) -> np.ndarray:
        """act(LayerNorm(x) @ W^T + bias) with the vectors given to fold_layernorm (fewer than 8 input rows)."""
        dg, db, dbias = self._fold
        x = np.ascontiguousarray(x, np.float32)
        m = x.size // self.cols
        dx = _dev(x)
        y = DeviceArray(x.shape[:-1] + (self.rows,), np.float32)
        _lib.check(_lib.load().cthip_linear(y.ptr, self.handle, dx.ptr, m, _p(dbias), None, _ACT[act],
                                            _PRO["layernorm"], dg.ptr, db.ptr, eps))
        return y.numpy()

    def free(self):
        if self.handle:
            _lib.load().cthip_wmat_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


_ACT = {None: _lib.ACT_NONE, "relu": _lib.ACT_RELU, "gelu": _lib.ACT_GELU, "silu": _lib.ACT_SILU,
        "sigmoid": _lib.ACT_SIGMOID, "tanh": _lib.ACT_TANH}
_PRO = {None: _lib.PRO_NONE, "layernorm": _lib.PRO_LAYERNORM, "rmsnorm": _lib.PRO_RMSNORM, "swiglu": _lib.PRO_SWIGLU}


def linear(x, w: WeightMatrix, bias=None, residual=None, act=None, prologue=None, norm_g=None, norm_b=None,
           eps: float = 1e-5) -> np.ndarray:
    """Linear with fused neighbours: act(prologue(x) @ W^T + bias) + residual (source/nn/linear.lisp:3-17)."""
    x = np.ascontiguousarray(x, np.float32)
    in_cols = 2 * w.cols if prologue == "swiglu" else w.cols
    if x.shape[-1] != in_cols:
        raise ValueError(f"linear: x has {x.shape[-1]} features, expected {in_cols}")
    m = x.size // in_cols
    dx, db, dr = _dev(x), _dev(bias), _dev(residual)
    dg, dbt = _dev(norm_g), _dev(norm_b)
    y = DeviceArray(x.shape[:-1] + (w.rows,), np.float32)
    _lib.check(_lib.load().cthip_linear(y.ptr, w.handle, dx.ptr, m, _p(db), _p(dr), _ACT[act], _PRO[prologue],
                                        _p(dg), _p(dbt), eps))
    return y.numpy()


def matmul(A, B, relu: bool = False, precision: str = "bf16x6") -> np.ndarray:
    """!matmul (+ fused !relu) (api/high-level-ops.lisp:76-99).

    precision: "fp32" = fp32 MFMA operands; "bf16x6" (default) = operands split in three bf16 terms,
    fp32-grade; "bf16x3" = two terms (2^-16 per product); "bf16" = operands rounded to bf16."""
    A, B = np.ascontiguousarray(A, np.float32), np.ascontiguousarray(B, np.float32)
    M, K = A.shape
    K2, N = B.shape
    if K != K2:
        raise ValueError("matmul: inner dimensions differ")
    dA, dB, dC = _dev(A), _dev(B), DeviceArray((M, N), np.float32)
    _lib.check(_lib.load().cthip_matmul(dC.ptr, dA.ptr, dB.ptr, M, N, K, _lib.ACT_RELU if relu else _lib.ACT_NONE,
                                        {"fp32": 0, "bf16": 1, "bf16x3": 2, "bf16x6": 3}[precision]))
    return dC.numpy()


def _rowop(fn_name, x, *vecs, eps=None):
    x = np.ascontiguousarray(x, np.float32)
    n = x.shape[-1] if x.ndim else 0
    rows = x.size // n if n else 0
    dx, dy = _dev(x), DeviceArray(x.shape, np.float32)
    dv = [_dev(v) for v in vecs]
    fn = getattr(_lib.load(), fn_name)
    args = [dy.ptr, dx.ptr] + [_p(v) for v in dv] + ([eps] if eps is not None else []) + [rows, n]
    _lib.check(fn(*args))
    return dy.numpy()


def softmax(x):
    return _rowop("cthip_softmax", x)


def layernorm(x, gamma=None, beta=None, eps=1e-5):
    return _rowop("cthip_layernorm", x, gamma, beta, eps=eps)


def rmsnorm(x, w=None, eps=1e-5):
    return _rowop("cthip_rmsnorm", x, w, eps=eps)


def layernorm_softmax(x, gamma=None, beta=None, eps=1e-5):
    return _rowop("cthip_layernorm_softmax", x, gamma, beta, eps=eps)


def unary(kind: str, x):
    x = np.ascontiguousarray(x, np.float32)
    dx, dy = _dev(x), DeviceArray(x.shape, np.float32)
    _lib.check(_lib.load().cthip_unary(_ACT[kind], dy.ptr, dx.ptr, x.size))
    return dy.numpy()


def relu(x):
    return unary("relu", x)


def gelu(x):
    return unary("gelu", x)


def silu(x):
    return unary("silu", x)


def sigmoid(x):
    return unary("sigmoid", x)


def tanh(x):
    return unary("tanh", x)


def embedding(W, idx):
    W = np.ascontiguousarray(W, np.float32)
    idx = np.ascontiguousarray(idx, np.float32)
    V, D = W.shape
    dW, di, out = _dev(W), _dev(idx), DeviceArray(idx.shape + (D,), np.float32)
    _lib.check(_lib.load().cthip_embedding(out.ptr, dW.ptr, di.ptr, idx.size, V, D))
    return out.numpy()


def argmax(x):
    x = np.ascontiguousarray(x, np.float32)
    n = x.shape[-1]
    rows = x.size // n
    dx, out = _dev(x), DeviceArray(x.shape[:-1] if x.ndim > 1 else (1,), np.int64)
    _lib.check(_lib.load().cthip_argmax(out.ptr, dx.ptr, rows, n))
    r = out.numpy()
    return r if x.ndim > 1 else int(r[0])


def rope(x, base=10000.0, start_pos=0):
    x = np.ascontiguousarray(x, np.float32)
    B, S, H, Dh = x.shape
    dx, out = _dev(x), DeviceArray(x.shape, np.float32)
    _lib.check(_lib.load().cthip_rope(out.ptr, dx.ptr, B, S, H, Dh, base, start_pos))
    return out.numpy()


def sdpa_cached(q, k_cache, v_cache, start_pos: int):
    """q (S,H,Dh) at positions start_pos.., caches (max_len,Hkv,Dh) -> (S,H,Dh), causal."""
    q = np.ascontiguousarray(q, np.float32)
    S, H, Dh = q.shape
    Hkv = k_cache.shape[1]
    dq, dk, dv = _dev(q), _dev(k_cache), _dev(v_cache)
    out = DeviceArray(q.shape, np.float32)
    _lib.check(_lib.load().cthip_sdpa_cached(out.ptr, dq.ptr, dk.ptr, dv.ptr, S, start_pos, H, Hkv, Dh))
    return out.numpy()
