"""GGUF files: reader front-end (the C++ reader of libcaten_hip.so) and a minimal writer.

Reader mirrors `load-gguf` / `gguf-metadata-get` / Tensor-Info of external/gguf
(gguf-file.lisp:26-27,93-104; tensor-info.lisp:43-60).  The writer exists because the reference has
none (its tests use the Python `gguf` package, external/test-gguf.lisp:3-30); it emits GGUF v3 with
`general.alignment`-aligned tensor data.
"""
from __future__ import annotations

import ctypes as C
import struct
from typing import Dict, List, Tuple

import numpy as np

from . import _lib
from .quant import GGML_TYPE_ID, packed_nbytes

_KIND_OF = {v: k for k, v in GGML_TYPE_ID.items()}
# gguf metadata value types (metadata.lisp:3-17)
_T_U8, _T_I8, _T_U16, _T_I16, _T_U32, _T_I32, _T_F32, _T_BOOL, _T_STR, _T_ARR, _T_U64, _T_I64, _T_F64 = range(13)


class TensorInfo:
    def __init__(self, name, kind, type_id, dims, abs_offset, nbytes):
        self.name, self.kind, self.type_id = name, kind, type_id
        self.dims = dims                      # as stored: innermost first
        self.shape = tuple(reversed(dims))    # row-major shape (tensor-info.lisp:104-120)
        self.abs_offset, self.nbytes = abs_offset, nbytes


class GGUF:
    """(load-gguf pathname)"""

    def __init__(self, path: str):
        self.lib = _lib.load()
        self.h = C.c_void_p()
        _lib.check(self.lib.cthip_gguf_open(C.byref(self.h), str(path).encode()))
        self.version = self.lib.cthip_gguf_version(self.h)
        self.alignment = self.lib.cthip_gguf_alignment(self.h)
        self.tensor_info: List[TensorInfo] = []
        name, typ, nd, dims = C.c_char_p(), C.c_int(), C.c_int(), (C.c_int64 * 4)()
        off, nb = C.c_int64(), C.c_int64()
        for i in range(self.lib.cthip_gguf_tensor_count(self.h)):
            _lib.check(self.lib.cthip_gguf_tensor_info(self.h, i, C.byref(name), C.byref(typ), C.byref(nd), dims,
                                                        C.byref(off), C.byref(nb)))
            self.tensor_info.append(TensorInfo(name.value.decode(), _KIND_OF.get(typ.value), typ.value,
                                               [int(dims[d]) for d in range(nd.value)], off.value, nb.value))

    @property
    def metadata_kv_count(self) -> int:
        return int(self.lib.cthip_gguf_metadata_count(self.h))

    def metadata_get(self, key: str):
        """(gguf-metadata-get gguf key): the value, or None."""
        i = self.lib.cthip_gguf_find_metadata(self.h, key.encode())
        if i < 0:
            return None
        k, typ, et, cnt = C.c_char_p(), C.c_int(), C.c_int(), C.c_int64()
        _lib.check(self.lib.cthip_gguf_metadata_info(self.h, i, C.byref(k), C.byref(typ), C.byref(et), C.byref(cnt)))

        def string(j):
            p, n = C.c_void_p(), C.c_int64()
            _lib.check(self.lib.cthip_gguf_metadata_string(self.h, i, j, C.byref(p), C.byref(n)))
            return C.string_at(p.value, n.value).decode("utf-8", "replace")

        if typ.value == _T_STR:
            return string(0)
        if typ.value == _T_ARR:
            if et.value == _T_STR:
                return [string(j) for j in range(cnt.value)]
            raise NotImplementedError("numeric metadata arrays are not exposed")
        v = C.c_double()
        _lib.check(self.lib.cthip_gguf_metadata_number(self.h, i, C.byref(v)))
        if typ.value == _T_BOOL:
            return bool(v.value)
        return v.value if typ.value in (_T_F32, _T_F64) else int(v.value)

    def tensor_bytes(self, name: str) -> np.ndarray:
        """The tensor's raw bytes as they sit in the file (a copy)."""
        i = self.lib.cthip_gguf_find_tensor(self.h, name.encode())
        if i < 0:
            raise KeyError(name)
        t = self.tensor_info[i]
        p = self.lib.cthip_gguf_tensor_data(self.h, i)
        return np.frombuffer(C.string_at(p, t.nbytes), dtype=np.uint8).copy()

    def load_into(self, model) -> int:
        """gguf->state-dict + remap-key + load-state-dict for a `caten_amd.llm.Transformer`."""
        n = C.c_int()
        arch = _lib.ARCH_GPT2 if model.arch == "gpt2" else _lib.ARCH_LLAMA
        _lib.check(self.lib.cthip_decoder_load_gguf(model.handle, self.h, arch, C.byref(n)))
        missing = self.lib.cthip_decoder_missing(model.handle)
        if missing:
            raise _lib.HipError(-5, f"load-state-dict: {missing} tensors of the model are missing from the file")
        return n.value

    def close(self):
        if self.h:
            self.lib.cthip_gguf_close(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def _s(b: str) -> bytes:
    e = b.encode()
    return struct.pack("<Q", len(e)) + e


def _value(v) -> bytes:
    if isinstance(v, bool):
        return struct.pack("<IB", _T_BOOL, int(v))
    if isinstance(v, int):
        return struct.pack("<II", _T_U32, v) if 0 <= v < 2 ** 32 else struct.pack("<Iq", _T_I64, v)
    if isinstance(v, float):
        return struct.pack("<If", _T_F32, v)
    if isinstance(v, str):
        return struct.pack("<I", _T_STR) + _s(v)
    if isinstance(v, (list, tuple)) and all(isinstance(x, str) for x in v):
        return struct.pack("<IIQ", _T_ARR, _T_STR, len(v)) + b"".join(_s(x) for x in v)
    raise TypeError(f"unsupported metadata value {v!r}")


def write_gguf(path: str, metadata: Dict[str, object], tensors: List[Tuple[str, str, Tuple[int, ...], np.ndarray]],
               alignment: int = 32) -> None:
    """Writes GGUF v3.  tensors: (name, kind, row-major shape, raw bytes in ggml block layout)."""
    meta = dict(metadata)
    meta.setdefault("general.alignment", alignment)
    out = [b"GGUF", struct.pack("<IQQ", 3, len(tensors), len(meta))]
    for k, v in meta.items():
        out.append(_s(k) + _value(v))
    rel, blobs = 0, []
    for name, kind, shape, raw in tensors:
        raw = np.ascontiguousarray(raw).view(np.uint8).ravel()
        n = int(np.prod(shape))
        if raw.size != packed_nbytes(kind, n):
            raise ValueError(f"{name}: {raw.size} bytes for a {kind} tensor of {n} elements")
        dims = list(reversed(shape))  # stored innermost first
        out.append(_s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims) +
                   struct.pack("<IQ", GGML_TYPE_ID[kind], rel))
        blobs.append((rel, raw))
        rel += (raw.size + alignment - 1) // alignment * alignment
    head = b"".join(out)
    pad = (alignment - len(head) % alignment) % alignment
    with open(path, "wb") as f:
        f.write(head + b"\0" * pad)
        base = f.tell()
        for r, raw in blobs:
            f.seek(base + r)
            f.write(raw.tobytes())
        f.truncate(base + rel)


# GGUF tensor names of a GPT-2 file (the left column of *remap-key*, apps/gpt2/gpt2.lisp:52-70)
def gpt2_gguf_tensors(weights: dict, linear_kind: str = "f32"):
    from .llm import Tensor
    out = []

    def add(name, a, kind="f32"):
        t = Tensor.from_f32(a, kind)
        out.append((name, kind, a.shape, t.raw))

    add("token_embd.weight", weights["wte"]); add("position_embd.weight", weights["wpe"])
    add("output_norm.weight", weights["lnf_g"]); add("output_norm.bias", weights["lnf_b"])
    add("output.weight", weights["lm_head"], linear_kind)
    names = {"ln1_g": "attn_norm.weight", "ln1_b": "attn_norm.bias", "attn_w": "attn_qkv.weight", "attn_b": "attn_qkv.bias",
             "proj_w": "attn_output.weight", "proj_b": "attn_output.bias", "ln2_g": "ffn_norm.weight", "ln2_b": "ffn_norm.bias",
             "fc_w": "ffn_up.weight", "fc_b": "ffn_up.bias", "fc2_w": "ffn_down.weight", "fc2_b": "ffn_down.bias"}
    for src, dst in names.items():
        for l, a in enumerate(weights[src]):
            add(f"blk.{l}.{dst}", a, linear_kind if src.endswith("_w") else "f32")
    return out
