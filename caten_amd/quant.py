"""GGUF block quantisers for synthetic weights (host side, NumPy).

The reference only *reads* quantised files (external/gguf/dequantize.lisp:40-53),
so the quantiser is this build's choice; it follows ggml's reference row
quantisers (Q8_0: d = absmax/127, q = round(w/d); Q4_0: d = signed-absmax/-8,
q = min(15, trunc(w/d + 8.5))) and writes ggml's on-disk block layout:
Q8_0 = fp16 d + 32 x int8 (34 bytes), Q4_0 = fp16 d + 16 nibble-pair bytes (18 bytes).
"""
from __future__ import annotations

import numpy as np

BLOCK = 32
BYTES_PER_BLOCK = {"q8_0": 34, "q4_0": 18}
# ggml type ids (external/gguf/tensor-info.lisp:3-31)
GGML_TYPE_ID = {"f32": 0, "f16": 1, "q4_0": 2, "q8_0": 8}


def _round_half_away(x):
    return np.sign(x) * np.floor(np.abs(x) + np.float32(0.5))


def quantize_q8_0(w: np.ndarray) -> np.ndarray:
    w = np.ascontiguousarray(w, np.float32).reshape(-1, BLOCK)
    amax = np.abs(w).max(axis=1)
    d = (amax / np.float32(127.0)).astype(np.float32)
    with np.errstate(divide="ignore"):
        inv = np.where(d != 0, np.float32(1.0) / d, np.float32(0.0)).astype(np.float32)
    q = _round_half_away((w * inv[:, None]).astype(np.float32)).astype(np.int8)
    out = np.empty((w.shape[0], 34), np.uint8)
    out[:, :2] = d.astype(np.float16).view(np.uint8).reshape(-1, 2)
    out[:, 2:] = q.view(np.uint8)
    return out.reshape(-1)


def quantize_q4_0(w: np.ndarray) -> np.ndarray:
    w = np.ascontiguousarray(w, np.float32).reshape(-1, BLOCK)
    am = np.argmax(np.abs(w), axis=1)  # first occurrence, as ggml's strict `<` scan keeps
    mx = w[np.arange(w.shape[0]), am]
    d = (mx / np.float32(-8.0)).astype(np.float32)
    with np.errstate(divide="ignore"):
        inv = np.where(d != 0, np.float32(1.0) / d, np.float32(0.0)).astype(np.float32)
    x = (w * inv[:, None]).astype(np.float32) + np.float32(8.5)
    xi = np.minimum(x.astype(np.int8), 15).astype(np.uint8)
    out = np.empty((w.shape[0], 18), np.uint8)
    out[:, :2] = d.astype(np.float16).view(np.uint8).reshape(-1, 2)
    out[:, 2:] = xi[:, :16] | (xi[:, 16:] << 4)
    return out.reshape(-1)


def quantize(kind: str, w: np.ndarray) -> np.ndarray:
    return {"q8_0": quantize_q8_0, "q4_0": quantize_q4_0}[kind](w)


def packed_nbytes(kind: str, n_elements: int) -> int:
    if kind == "f32":
        return 4 * n_elements
    if kind == "f16":
        return 2 * n_elements
    return (n_elements + BLOCK - 1) // BLOCK * BYTES_PER_BLOCK[kind]
