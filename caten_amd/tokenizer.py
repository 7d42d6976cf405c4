"""caten/llm's tokenizer interface (external/llm/tokenizers.lisp, external/llm/bpe.lisp) over the C ABI.

`Tokenizer.encode(text) -> list[int]`, `Tokenizer.decode(ids) -> str`; `make_bpe_tokenizer(tokens, merges)`
takes the two strings the reference's constructor takes (bpe.lisp:14-38); `gguf_bpe_tokenizer(gguf)` builds
them from a GGUF file's `tokenizer.ggml.tokens` / `tokenizer.ggml.merges` metadata
(external/gguf/gguf-file.lisp:118-153).
"""
from __future__ import annotations

import ctypes as C

from . import _lib


class Tokenizer:
    """encode / decode protocol (tokenizers.lisp:3-13)."""

    def encode(self, text: str) -> list:
        raise NotImplementedError

    def decode(self, ids) -> str:
        raise NotImplementedError


class BPETokenizer(Tokenizer):
    def __init__(self, tokens: str, merges: str):
        t, m = tokens.encode("utf-8"), merges.encode("utf-8")
        h = C.c_void_p()
        _lib.check(_lib.load().cthip_bpe_create(C.byref(h), t, len(t), m, len(m)))
        self.handle = h

    @property
    def vocab_size(self) -> int:
        return _lib.load().cthip_bpe_vocab_size(self.handle)

    def encode(self, text: str) -> list:
        if not isinstance(text, str):
            raise TypeError("encode: text must be a string")  # check-type text string (bpe.lisp:87)
        raw = text.encode("utf-8")
        lib = _lib.load()
        n = C.c_size_t()
        _lib.check(lib.cthip_bpe_encode(self.handle, raw, len(raw), None, 0, C.byref(n)))
        ids = (C.c_int * max(n.value, 1))()
        _lib.check(lib.cthip_bpe_encode(self.handle, raw, len(raw), ids, n.value, C.byref(n)))
        return list(ids[:n.value])

    def decode(self, ids) -> str:
        ids = [int(i) for i in ids]
        arr = (C.c_int * max(len(ids), 1))(*ids)
        lib = _lib.load()
        n = C.c_size_t()
        _lib.check(lib.cthip_bpe_decode(self.handle, arr, len(ids), None, 0, C.byref(n)))
        buf = C.create_string_buffer(max(n.value, 1))
        _lib.check(lib.cthip_bpe_decode(self.handle, arr, len(ids), buf, n.value, C.byref(n)))
        return buf.raw[:n.value].decode("utf-8", "replace")

    def close(self):
        if self.handle:
            _lib.load().cthip_bpe_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def make_bpe_tokenizer(tokens: str, merges: str) -> BPETokenizer:
    """(make-bpe-tokenizer tokens merges), bpe.lisp:14-38."""
    return BPETokenizer(tokens, merges)


def gguf_bpe_tokenizer(gguf, metadata_tokens="tokenizer.ggml.tokens", metadata_merges="tokenizer.ggml.merges") -> BPETokenizer:
    """(gguf->bpe-tokenizer gguf): token i of the metadata array gets id i, merge j rank j."""
    tokens, merges = gguf.metadata_get(metadata_tokens), gguf.metadata_get(metadata_merges)
    if tokens is None or merges is None:
        raise KeyError(f"the gguf file has no tokenizer metadata ({metadata_tokens}, {metadata_merges})")
    # the constructor drops the first piece / first line of its two strings
    return BPETokenizer(" " + " ".join(tokens), "\n" + "\n".join(merges))
