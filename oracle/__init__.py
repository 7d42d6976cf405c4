"""CPU oracle for the Caten decode path -- TEST INFRASTRUCTURE ONLY.

ctypes front-end of ``caten_oracle.c`` (a plain-C, single-thread restatement of
what Caten's ``BACKEND=CLANG`` path computes; every C function cites the
reference lines it follows).  Only ``tests/``, ``__graft_entry__.smoke()`` and
the ``cpu_baseline`` leg of ``bench.py`` may import this package; the product
(``caten_amd``) never does.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libcaten_oracle.so")
_lib = None

_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_u8p = np.ctypeslib.ndpointer(dtype=np.uint8, flags="C_CONTIGUOUS")


def build(force: bool = False) -> str:
    """Compile the oracle with gcc -O3 (what the reference's CLANG backend uses,
    source/byoc/clang.lisp:217)."""
    src = os.path.join(_HERE, "caten_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["gcc", "-O3", "-shared", "-fPIC", "-o", _SO, src, "-lm"])
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = C.CDLL(_SO)
        L = _lib
        L.orc_f16_to_f32.restype = C.c_float
        L.orc_f16_to_f32.argtypes = [C.c_uint16]
        L.orc_f32_to_f16.restype = C.c_uint16
        L.orc_f32_to_f16.argtypes = [C.c_float]
        L.orc_argmax.restype = C.c_int64
        L.orc_gpt2_forward.restype = C.c_int64
        L.orc_llama_forward.restype = C.c_int64
    return _lib


def _f(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _ptr(a):
    return a.ctypes.data_as(C.c_void_p)


# ---------------------------------------------------------------- codecs
def f16_to_f32(bits) -> np.ndarray:
    bits = np.asarray(bits, dtype=np.uint16).ravel()
    out = np.empty(bits.size, np.float32)
    lib().orc_dequant_f16(_ptr(np.ascontiguousarray(bits.view(np.uint8))), C.c_int64(bits.size), _ptr(out))
    return out


def f32_to_f16_bits(x) -> np.ndarray:
    x = _f(x).ravel()
    L = lib()
    return np.array([L.orc_f32_to_f16(float(v)) for v in x], dtype=np.uint16)


def dequant(kind: str, raw, n: int) -> np.ndarray:
    raw = np.ascontiguousarray(np.frombuffer(raw, dtype=np.uint8) if not isinstance(raw, np.ndarray) else raw.view(np.uint8).ravel())
    out = np.empty(n, np.float32)
    fn = {"q8_0": lib().orc_dequant_q8_0, "q4_0": lib().orc_dequant_q4_0,
          "f16": lib().orc_dequant_f16, "f32": lib().orc_dequant_f32}[kind]
    fn(_ptr(raw), C.c_int64(n), _ptr(out))
    return out


def quantize(kind: str, w) -> np.ndarray:
    w = _f(w).ravel()
    assert w.size % 32 == 0
    bpb = {"q8_0": 34, "q4_0": 18}[kind]
    out = np.empty(w.size // 32 * bpb, np.uint8)
    fn = {"q8_0": lib().orc_quantize_q8_0, "q4_0": lib().orc_quantize_q4_0}[kind]
    fn(_ptr(w), C.c_int64(w.size), _ptr(out))
    return out


# ---------------------------------------------------------------- fused items
def matmul(A, B, relu=False):
    A, B = _f(A), _f(B)
    M, K = A.shape
    K2, N = B.shape
    assert K == K2
    out = np.empty((M, N), np.float32)
    lib().orc_matmul(_ptr(A), _ptr(B), _ptr(out), M, N, K, int(relu))
    return out


def linear(x, W, b=None):
    x, W = _f(x), _f(W)
    M, K = x.reshape(-1, x.shape[-1]).shape
    N = W.shape[0]
    assert W.shape[1] == K
    out = np.empty((M, N), np.float32)
    bb = _f(b) if b is not None else None
    lib().orc_linear(_ptr(x), _ptr(W), _ptr(bb) if bb is not None else None, _ptr(out), M, K, N)
    return out.reshape(x.shape[:-1] + (N,))


def _unary(name):
    def fn(x):
        x = _f(x)
        out = np.empty_like(x)
        getattr(lib(), name)(_ptr(x), _ptr(out), C.c_int64(x.size))
        return out
    fn.__name__ = name
    return fn


relu = _unary("orc_relu")
sigmoid = _unary("orc_sigmoid")
tanh = _unary("orc_tanh")
gelu_tanh = _unary("orc_gelu_tanh")
silu = _unary("orc_silu")


def softmax(x):
    x = _f(x)
    out = np.empty_like(x)
    n = x.shape[-1]
    lib().orc_softmax(_ptr(x), _ptr(out), C.c_int64(x.size // n), n)
    return out


def layernorm(x, gamma=None, beta=None, eps=1e-5):
    x = _f(x)
    out = np.empty_like(x)
    n = x.shape[-1]
    g = _f(gamma) if gamma is not None else None
    b = _f(beta) if beta is not None else None
    lib().orc_layernorm(_ptr(x), _ptr(g) if g is not None else None, _ptr(b) if b is not None else None,
                        C.c_double(eps), _ptr(out), C.c_int64(x.size // n), n)
    return out


def rmsnorm(x, w=None, eps=1e-5):
    x = _f(x)
    out = np.empty_like(x)
    n = x.shape[-1]
    ww = _f(w) if w is not None else None
    lib().orc_rmsnorm(_ptr(x), _ptr(ww) if ww is not None else None, C.c_double(eps), _ptr(out),
                      C.c_int64(x.size // n), n)
    return out


def rope(x, base=10000.0, start_pos=0):
    x = _f(x)
    B, S, H, Dh = x.shape
    out = np.empty_like(x)
    lib().orc_rope(_ptr(x), _ptr(out), B, S, H, Dh, C.c_double(base), start_pos)
    return out


def embedding_onehot(W, idx):
    W = _f(W)
    idx = _f(idx)
    V, D = W.shape
    out = np.empty(idx.shape + (D,), np.float32)
    lib().orc_embedding_onehot(_ptr(W), _ptr(idx), _ptr(out), idx.size, V, D)
    return out


def argmax(x) -> int:
    x = _f(x).ravel()
    return int(lib().orc_argmax(_ptr(x), x.size))


def triu_neginf(rows, cols, k):
    out = np.empty((rows, cols), np.float32)
    lib().orc_triu_neginf(_ptr(out), rows, cols, k)
    return out


def triu(x, k=0):
    x = _f(x)
    out = np.empty_like(x)
    r, c = x.shape[-2:]
    for a, o in zip(x.reshape(-1, r, c), out.reshape(-1, r, c)):
        lib().orc_triu(_ptr(a), _ptr(o), r, c, k)
    return out


def tril(x, k=0):
    x = _f(x)
    out = np.empty_like(x)
    r, c = x.shape[-2:]
    for a, o in zip(x.reshape(-1, r, c), out.reshape(-1, r, c)):
        lib().orc_tril(_ptr(a), _ptr(o), r, c, k)
    return out


def sdpa(q, k, v, mask=None):
    """q (S,H,Dh); k, v (T,Hkv,Dh) in KV-cache layout; mask (S,T) or None -> (S,H,Dh)."""
    q, k, v = _f(q), _f(k), _f(v)
    S, H, Dh = q.shape
    T, Hkv, _ = k.shape
    out = np.empty_like(q)
    scr = np.empty(S * T, np.float32)
    mk = _f(mask) if mask is not None else None
    lib().orc_sdpa(_ptr(q), _ptr(k), _ptr(v), _ptr(mk) if mk is not None else None, _ptr(out),
                   S, T, H, Hkv, Dh, _ptr(scr))
    return out


# ---------------------------------------------------------------- decoders
class _GPT2Struct(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("n_layers", "dim", "n_heads", "vocab", "max_seq", "ffn")] + \
               [("eps", C.c_double)] + \
               [(n, C.c_void_p) for n in ("wte", "wpe", "lnf_g", "lnf_b", "lm_head",
                                          "ln1_g", "ln1_b", "attn_w", "attn_b", "proj_w", "proj_b",
                                          "ln2_g", "ln2_b", "fc_w", "fc_b", "fc2_w", "fc2_b",
                                          "k_cache", "v_cache")]


class _LlamaStruct(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("n_layers", "dim", "n_heads", "n_kv_heads", "vocab", "max_seq", "ffn")] + \
               [("eps", C.c_double), ("rope_base", C.c_double)] + \
               [(n, C.c_void_p) for n in ("tok_emb", "norm_w", "lm_head", "attn_norm", "ffn_norm",
                                          "wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down",
                                          "k_cache", "v_cache")]


def _ptr_array(arrs):
    a = (C.c_void_p * len(arrs))(*[x.ctypes.data for x in arrs])
    return a


class GPT2:
    """Oracle GPT-2-shaped decoder.  ``weights`` is a dict of fp32 arrays:
    wte, wpe, lnf_g, lnf_b, lm_head and per-layer lists ln1_g, ln1_b, attn_w,
    attn_b, proj_w, proj_b, ln2_g, ln2_b, fc_w, fc_b, fc2_w, fc2_b."""

    PER_LAYER = ("ln1_g", "ln1_b", "attn_w", "attn_b", "proj_w", "proj_b",
                 "ln2_g", "ln2_b", "fc_w", "fc_b", "fc2_w", "fc2_b")

    def __init__(self, cfg: dict, weights: dict):
        self.cfg = dict(cfg)
        L, D = cfg["n_layers"], cfg["dim"]
        self.w = {}
        for k in ("wte", "wpe", "lnf_g", "lnf_b", "lm_head"):
            self.w[k] = _f(weights[k])
        for k in self.PER_LAYER:
            self.w[k] = [_f(a) for a in weights[k]]
        self.k_cache = [np.zeros((cfg["max_seq"], D), np.float32) for _ in range(L)]
        self.v_cache = [np.zeros((cfg["max_seq"], D), np.float32) for _ in range(L)]
        s = _GPT2Struct()
        s.n_layers, s.dim, s.n_heads, s.vocab, s.max_seq, s.ffn = (
            L, D, cfg["n_heads"], cfg["vocab"], cfg["max_seq"], cfg["ffn"])
        s.eps = cfg.get("eps", 1e-5)
        self._keep = []
        for k in ("wte", "wpe", "lnf_g", "lnf_b", "lm_head"):
            setattr(s, k, self.w[k].ctypes.data)
        for k in self.PER_LAYER:
            pa = _ptr_array(self.w[k])
            self._keep.append(pa)
            setattr(s, k, C.cast(pa, C.c_void_p))
        for k, arrs in (("k_cache", self.k_cache), ("v_cache", self.v_cache)):
            pa = _ptr_array(arrs)
            self._keep.append(pa)
            setattr(s, k, C.cast(pa, C.c_void_p))
        self._s = s

    def forward(self, tokens, n: int, onehot: bool = False, all_logits: bool = False):
        """One compiled-graph `forward` (apps/gpt2/gpt2.lisp:104): returns (token, last-row logits)."""
        t = _f(tokens).ravel()
        logits = np.empty(self.cfg["vocab"], np.float32)
        tok = lib().orc_gpt2_forward(C.byref(self._s), _ptr(t), t.size, n, _ptr(logits),
                                     int(onehot), int(all_logits))
        return int(tok), logits

    def generate(self, prompt, max_length: int, onehot: bool = False, all_logits: bool = False,
                 keep_logits: bool = False):
        """gpt2-generate (apps/gpt2/gpt2.lisp:97-113): max_length forwards, the first over the
        whole prompt.  Returns the generated tokens (and per-step logits if asked)."""
        tokens = [int(t) for t in prompt]
        start = 0
        out, logs = [], []
        for _ in range(max_length):
            tok, lg = self.forward(tokens[start:], start, onehot, all_logits)
            start = len(tokens)
            tokens.append(tok)
            out.append(tok)
            if keep_logits:
                logs.append(lg)
        return (out, logs) if keep_logits else out


class Llama:
    PER_LAYER = ("attn_norm", "ffn_norm", "wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down")

    def __init__(self, cfg: dict, weights: dict):
        self.cfg = dict(cfg)
        L, D = cfg["n_layers"], cfg["dim"]
        kd = D // cfg["n_heads"] * cfg["n_kv_heads"]
        self.w = {}
        for k in ("tok_emb", "norm_w", "lm_head"):
            self.w[k] = _f(weights[k])
        for k in self.PER_LAYER:
            self.w[k] = [_f(a) for a in weights[k]]
        self.k_cache = [np.zeros((cfg["max_seq"], kd), np.float32) for _ in range(L)]
        self.v_cache = [np.zeros((cfg["max_seq"], kd), np.float32) for _ in range(L)]
        s = _LlamaStruct()
        s.n_layers, s.dim, s.n_heads, s.n_kv_heads, s.vocab, s.max_seq, s.ffn = (
            L, D, cfg["n_heads"], cfg["n_kv_heads"], cfg["vocab"], cfg["max_seq"], cfg["ffn"])
        s.eps = cfg.get("eps", 1e-5)
        s.rope_base = cfg.get("rope_base", 10000.0)
        self._keep = []
        for k in ("tok_emb", "norm_w", "lm_head"):
            setattr(s, k, self.w[k].ctypes.data)
        for k in self.PER_LAYER:
            pa = _ptr_array(self.w[k])
            self._keep.append(pa)
            setattr(s, k, C.cast(pa, C.c_void_p))
        for k, arrs in (("k_cache", self.k_cache), ("v_cache", self.v_cache)):
            pa = _ptr_array(arrs)
            self._keep.append(pa)
            setattr(s, k, C.cast(pa, C.c_void_p))
        self._s = s

    def forward(self, tokens, n: int):
        t = _f(tokens).ravel()
        logits = np.empty(self.cfg["vocab"], np.float32)
        tok = lib().orc_llama_forward(C.byref(self._s), _ptr(t), t.size, n, _ptr(logits))
        return int(tok), logits

    def generate(self, prompt, max_length: int, keep_logits: bool = False):
        tokens = [int(t) for t in prompt]
        start = 0
        out, logs = [], []
        for _ in range(max_length):
            tok, lg = self.forward(tokens[start:], start)
            start = len(tokens)
            tokens.append(tok)
            out.append(tok)
            if keep_logits:
                logs.append(lg)
        return (out, logs) if keep_logits else out
