"""Decoder front-end: mirrors `make-gpt2` / `gpt2-generate` (apps/gpt2/gpt2.lisp:82-113)
and the Transformer it compiles (external/llm/layers.lisp:73-90) on top of the
device-resident decoder session of libcaten_hip.so.

    model = make_gpt2(cfg, state_dict)           # state dict: reference keys -> (kind, raw GGUF bytes, shape)
    tok = model.forward(x=[...], s=len, n=start) # one compiled-graph `forward`
    toks = gpt2_generate(model, prompt_ids, max_length=100)
"""
from __future__ import annotations

import ctypes as C
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from . import _lib
from .quant import quantize, packed_nbytes

# *remap-key* (apps/gpt2/gpt2.lisp:52-70): GGUF tensor names -> Caten state-dict keys
GPT2_REMAP = [
    ("blk.", "h."), ("token_embd.weight", "wte.weight"), ("position_embd.weight", "wpe.weight"),
    (".attn_norm.weight", ".ln_1.affine"), (".attn_norm.bias", ".ln_1.bias"),
    (".attn_qkv.weight", ".attn.c_attn.weight"), (".attn_qkv.bias", ".attn.c_attn.bias"),
    (".ffn_down.weight", ".mlp.c_proj.weight"), (".ffn_down.bias", ".mlp.c_proj.bias"),
    (".ffn_norm.weight", ".ln_2.affine"), (".ffn_norm.bias", ".ln_2.bias"),
    (".ffn_up.weight", ".mlp.c_fc.weight"), (".ffn_up.bias", ".mlp.c_fc.bias"),
    (".attn_output.weight", ".attn.c_proj.weight"), (".attn_output.bias", ".attn.c_proj.bias"),
    ("output.weight", "lm_head.weight"), ("output_norm.bias", "ln_f.bias"), ("output_norm.weight", "ln_f.affine"),
]


def remap_key(key: str) -> str:
    for before, after in GPT2_REMAP:
        key = key.replace(before, after)
    return key


class Tensor:
    """One state-dict entry as it sits in a GGUF file: type, raw bytes, (rows, cols)."""

    def __init__(self, kind: str, raw: np.ndarray, rows: int, cols: int):
        self.kind, self.rows, self.cols = kind, int(rows), int(cols)
        self.raw = np.ascontiguousarray(np.asarray(raw).view(np.uint8).ravel())
        want = packed_nbytes(kind, self.rows * self.cols)
        if self.raw.size != want:
            raise ValueError(f"Tensor: {self.raw.size} bytes for a {kind} ({rows},{cols}) tensor, expected {want}")

    @classmethod
    def from_f32(cls, a: np.ndarray, kind: str = "f32") -> "Tensor":
        a = np.ascontiguousarray(a, np.float32)
        rows, cols = (a.shape if a.ndim == 2 else (1, a.size))
        if kind == "f32":
            return cls(kind, a.view(np.uint8), rows, cols)
        if kind == "f16":
            return cls(kind, a.astype(np.float16).view(np.uint8), rows, cols)
        return cls(kind, quantize(kind, a), rows, cols)


def gpt2_state_dict(weights: dict, linear_kind: str = "f32") -> Dict[str, Tensor]:
    """Synthetic weights (caten_amd.synth.gpt2_weights) -> state dict under the reference's keys.
    Linear weights are stored as `linear_kind`; embeddings, LayerNorm and biases stay fp32."""
    sd = {"wte.weight": Tensor.from_f32(weights["wte"]), "wpe.weight": Tensor.from_f32(weights["wpe"]),
          "ln_f.affine": Tensor.from_f32(weights["lnf_g"]), "ln_f.bias": Tensor.from_f32(weights["lnf_b"]),
          "lm_head.weight": Tensor.from_f32(weights["lm_head"], linear_kind)}
    names = {"ln1_g": "ln_1.affine", "ln1_b": "ln_1.bias", "attn_w": "attn.c_attn.weight", "attn_b": "attn.c_attn.bias",
             "proj_w": "attn.c_proj.weight", "proj_b": "attn.c_proj.bias", "ln2_g": "ln_2.affine", "ln2_b": "ln_2.bias",
             "fc_w": "mlp.c_fc.weight", "fc_b": "mlp.c_fc.bias", "fc2_w": "mlp.c_proj.weight", "fc2_b": "mlp.c_proj.bias"}
    for src, dst in names.items():
        for l, a in enumerate(weights[src]):
            sd[f"h.{l}.{dst}"] = Tensor.from_f32(a, linear_kind if src.endswith("_w") else "f32")
    return sd


def llama_state_dict(weights: dict, linear_kind: str = "f32", threads: int = 1) -> Dict[str, Tensor]:
    """`threads` > 1 quantises the tensors on a thread pool (NumPy releases the interpreter lock inside its loops)."""
    names = {"attn_norm": "attention_norm.weight", "ffn_norm": "ffn_norm.weight", "wq": "attention.wq.weight",
             "wk": "attention.wk.weight", "wv": "attention.wv.weight", "wo": "attention.wo.weight",
             "w_gate": "feed_forward.w1.weight", "w_down": "feed_forward.w2.weight", "w_up": "feed_forward.w3.weight"}
    jobs = [("tok_embeddings.weight", weights["tok_emb"], "f32"), ("norm.weight", weights["norm_w"], "f32"),
            ("output.weight", weights["lm_head"], linear_kind)]
    for src, dst in names.items():
        for l, a in enumerate(weights[src]):
            jobs.append((f"layers.{l}.{dst}", a, linear_kind if src.startswith("w") else "f32"))
    if threads > 1:
        from concurrent.futures import ThreadPoolExecutor
        with ThreadPoolExecutor(threads) as pool:
            tensors = list(pool.map(lambda j: Tensor.from_f32(j[1], j[2]), jobs))
    else:
        tensors = [Tensor.from_f32(a, kind) for _, a, kind in jobs]
    return {key: t for (key, _, _), t in zip(jobs, tensors)}


class Transformer:
    """The compiled Transformer graph: `forward(x, s, n)` as apps/gpt2/gpt2.lisp:104 calls it."""

    def __init__(self, cfg: dict, arch: str = "gpt2", device: int = 0):
        self.cfg = dict(cfg)
        self.arch = arch
        self.lib = _lib.init(device)
        c = _lib.DecoderConfig()
        c.arch = _lib.ARCH_GPT2 if arch == "gpt2" else _lib.ARCH_LLAMA
        c.n_layers, c.dim, c.n_heads = cfg["n_layers"], cfg["dim"], cfg["n_heads"]
        c.n_kv_heads = cfg.get("n_kv_heads", cfg["n_heads"])
        c.ffn, c.vocab, c.max_seq = cfg["ffn"], cfg["vocab"], cfg["max_seq"]
        c.eps = cfg.get("eps", 1e-5)
        c.rope_base = cfg.get("rope_base", 10000.0)
        self.handle = C.c_void_p()
        _lib.check(self.lib.cthip_decoder_create(C.byref(self.handle), C.byref(c)))

    def load_state_dict(self, sd: Dict[str, Tensor]) -> "Transformer":
        """load-state-dict (source/api/module.lisp:290-320)"""
        for key, t in sd.items():
            _lib.check(self.lib.cthip_decoder_load(self.handle, key.encode(), _lib.GGML_TYPE[t.kind], t.raw.ctypes.data,
                                                   t.rows, t.cols))
        missing = self.lib.cthip_decoder_missing(self.handle)
        if missing:
            raise _lib.HipError(-5, f"load-state-dict: {missing} tensors of the model are missing from the state dict")
        return self

    def forward(self, x: Sequence[float], s: Optional[int] = None, n: int = 0, return_logits: bool = False):
        """(forward model `(x . tokens) `(s . len) `(n . start-pos)) -> greedy token of the last position."""
        toks = np.ascontiguousarray(x, np.float32).ravel()
        s = toks.size if s is None else s
        if s != toks.size:
            raise ValueError(f"forward: s = {s} but x holds {toks.size} tokens")
        tok = C.c_int64()
        logits = np.empty(self.cfg["vocab"], np.float32) if return_logits else None
        _lib.check(self.lib.cthip_decoder_forward(self.handle, toks.ctypes.data, s, n, C.byref(tok),
                                                  logits.ctypes.data if return_logits else None))
        return (int(tok.value), logits) if return_logits else int(tok.value)

    def generate_until(self, max_steps: int, eos_token: int) -> List[int]:
        """Greedy tokens from the device-resident loop until `eos_token` has been produced (it is the last element)
        or `max_steps` tokens exist; the stop condition is evaluated on the device."""
        out = np.empty(max(max_steps, 1), np.int64)
        n = C.c_int()
        _lib.check(self.lib.cthip_decoder_generate_until(self.handle, max_steps, int(eos_token), out.ctypes.data, C.byref(n)))
        return [int(t) for t in out[:n.value]]

    def generate_on_device(self, steps: int) -> List[int]:
        """Continues greedily for `steps` tokens without returning to the host in between."""
        out = np.empty(max(steps, 1), np.int64)
        _lib.check(self.lib.cthip_decoder_generate(self.handle, steps, out.ctypes.data))
        return [int(t) for t in out[:steps]]

    @property
    def position(self) -> int:
        return int(self.lib.cthip_decoder_position(self.handle))

    def step_bytes(self, t: int) -> int:
        return int(self.lib.cthip_decoder_step_bytes(self.handle, t))

    def peek(self, what: str) -> np.ndarray:
        p, n = C.c_void_p(), C.c_int64()
        _lib.check(self.lib.cthip_decoder_peek(self.handle, what.encode(), C.byref(p), C.byref(n)))
        out = np.empty(n.value, np.float32)
        _lib.check(self.lib.cthip_d2h(out.ctypes.data, p.value, out.nbytes))
        return out

    def close(self):
        if self.handle:
            self.lib.cthip_decoder_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def make_gpt2(cfg: dict, state_dict: Dict[str, Tensor], device: int = 0) -> Transformer:
    """make-gpt2 (apps/gpt2/gpt2.lisp:82-93) minus the download: build the Transformer, load the state dict."""
    return Transformer(cfg, "gpt2", device).load_state_dict(state_dict)


def make_llama(cfg: dict, state_dict: Dict[str, Tensor], device: int = 0) -> Transformer:
    return Transformer(cfg, "llama", device).load_state_dict(state_dict)


def gpt2_generate(model: Transformer, prompt: Sequence[int], max_length: int = 100, on_device: bool = True,
                  keep_logits: bool = False):
    """gpt2-generate (apps/gpt2/gpt2.lisp:97-113): `max_length` forwards, the first over the whole
    prompt (prefill), each of the rest over the one new token.  With on_device the single-token
    forwards run back to back on the GPU and their tokens are read once at the end; otherwise every
    step returns its token to the host, as the reference's loop does."""
    tokens = [int(t) for t in prompt]
    out: List[int] = []
    logs = []
    if max_length <= 0:
        return (out, logs) if keep_logits else out
    if on_device and not keep_logits:
        tok = model.forward([float(t) for t in tokens], len(tokens), 0)
        out.append(tok)
        out.extend(model.generate_on_device(max_length - 1))
        return out
    start = 0
    for _ in range(max_length):
        chunk = tokens[start:]
        r = model.forward([float(t) for t in chunk], len(chunk), start, return_logits=keep_logits)
        tok = r[0] if keep_logits else r
        if keep_logits:
            logs.append(r[1])
        start = len(tokens)
        tokens.append(tok)
        out.append(tok)
    return (out, logs) if keep_logits else out


def gpt2_generate_text(model: Transformer, tokenizer, text: str, max_length: int = 100, on_device: bool = True,
                       expected: Optional[str] = None) -> str:
    """gpt2-generate with its string interface (apps/gpt2/gpt2.lisp:97-113): encode the input, run `max_length`
    greedy forwards, decode prompt + generated tokens; `expected` asserts the decoded text as the reference's
    keyword does."""
    if not isinstance(text, str):
        raise TypeError("gpt2_generate_text: input must be a string")
    prompt = tokenizer.encode(text)
    if not prompt:
        raise ValueError("gpt2_generate_text: the input encodes to no tokens")
    decoded = tokenizer.decode(prompt + gpt2_generate(model, prompt, max_length, on_device=on_device))
    if expected is not None and decoded != expected:
        raise AssertionError(f"Expected output: {expected}, but got: {decoded}")
    return decoded
