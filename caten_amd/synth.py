"""Synthetic, seeded weights and prompts of the shapes the decode path is measured on.

Caten's own RNG (threefry2x32 built from graph ops, source/api/initializers.lisp:55-99)
has no golden stream, so inputs are generated here with NumPy ``default_rng(seed)``
and fed to both the HIP path and the CPU oracle.
"""
from __future__ import annotations

import numpy as np

# apps/gpt2/gpt2.lisp:36-44 parameter table (+ the tiny shapes the tests use)
GPT2_CONFIGS = {
    "gpt2": dict(n_layers=12, n_heads=12, dim=768, ffn=3072, vocab=50257, max_seq=1024, eps=1e-5),
    "gpt2-medium": dict(n_layers=24, n_heads=16, dim=1024, ffn=4096, vocab=50257, max_seq=1024, eps=1e-5),
    "gpt2-large": dict(n_layers=36, n_heads=20, dim=1280, ffn=5120, vocab=50257, max_seq=1024, eps=1e-5),
    "gpt2-xl": dict(n_layers=48, n_heads=25, dim=1600, ffn=6400, vocab=50257, max_seq=1024, eps=1e-5),
    "gpt2-tiny": dict(n_layers=2, n_heads=4, dim=256, ffn=1024, vocab=1000, max_seq=64, eps=1e-5),
    "gpt2-mini": dict(n_layers=3, n_heads=12, dim=768, ffn=3072, vocab=5003, max_seq=128, eps=1e-5),
}

LLAMA_CONFIGS = {
    "llama-1.1b": dict(n_layers=22, n_heads=32, n_kv_heads=4, dim=2048, ffn=5632, vocab=32000,
                       max_seq=2048, eps=1e-5, rope_base=10000.0),
    "llama-tiny": dict(n_layers=2, n_heads=8, n_kv_heads=2, dim=512, ffn=1024, vocab=1000,
                       max_seq=64, eps=1e-5, rope_base=10000.0),
}


def gpt2_weights(cfg: dict, seed: int = 0) -> dict:
    """Random-init fp32 weights ~N(0,0.02); LayerNorm gamma~N(1,0.02), beta~N(0,0.02)."""
    rng = np.random.default_rng(seed)
    D, F, V, L = cfg["dim"], cfg["ffn"], cfg["vocab"], cfg["n_layers"]

    def n(*shape, mean=0.0):
        return (mean + 0.02 * rng.standard_normal(shape, dtype=np.float32)).astype(np.float32)

    w = dict(wte=n(V, D), wpe=n(cfg["max_seq"], D), lnf_g=n(D, mean=1.0), lnf_b=n(D), lm_head=n(V, D))
    for k in ("ln1_g", "ln1_b", "attn_w", "attn_b", "proj_w", "proj_b",
              "ln2_g", "ln2_b", "fc_w", "fc_b", "fc2_w", "fc2_b"):
        w[k] = []
    for _ in range(L):
        w["ln1_g"].append(n(D, mean=1.0)); w["ln1_b"].append(n(D))
        w["attn_w"].append(n(3 * D, D)); w["attn_b"].append(n(3 * D))
        w["proj_w"].append(n(D, D)); w["proj_b"].append(n(D))
        w["ln2_g"].append(n(D, mean=1.0)); w["ln2_b"].append(n(D))
        w["fc_w"].append(n(F, D)); w["fc_b"].append(n(F))
        w["fc2_w"].append(n(D, F)); w["fc2_b"].append(n(D))
    return w


GPT2_LINEAR_KEYS = ("attn_w", "proj_w", "fc_w", "fc2_w")  # + "lm_head"
LLAMA_LINEAR_KEYS = ("wq", "wk", "wv", "wo", "w_gate", "w_up", "w_down")  # + "lm_head"


def llama_weights(cfg: dict, seed: int = 0, threads: int = 1) -> dict:
    """Random-init fp32 weights ~N(0,0.02), norm weights ~N(1,0.02).  `threads` > 1 draws every tensor from a
    generator of its own (seeded by (seed, tensor number)) on a thread pool: other values than the serial stream
    gives, the same distribution, and a 1.1 B-parameter model in seconds instead of a minute."""
    D, F, V, L = cfg["dim"], cfg["ffn"], cfg["vocab"], cfg["n_layers"]
    KD = D // cfg["n_heads"] * cfg["n_kv_heads"]
    if threads > 1:
        from concurrent.futures import ThreadPoolExecutor
        per_layer = {"attn_norm": ((D,), 1.0), "ffn_norm": ((D,), 1.0), "wq": ((D, D), 0.0), "wk": ((KD, D), 0.0),
                     "wv": ((KD, D), 0.0), "wo": ((D, D), 0.0), "w_gate": ((F, D), 0.0), "w_up": ((F, D), 0.0),
                     "w_down": ((D, F), 0.0)}
        jobs = [("tok_emb", None, (V, D), 0.0), ("norm_w", None, (D,), 1.0), ("lm_head", None, (V, D), 0.0)]
        jobs += [(k, l, sh, mean) for l in range(L) for k, (sh, mean) in per_layer.items()]

        def draw(i):
            _, _, shape, mean = jobs[i]
            a = np.random.default_rng([seed, i]).standard_normal(shape, dtype=np.float32)
            a *= np.float32(0.02)
            if mean:
                a += np.float32(mean)
            return a
        with ThreadPoolExecutor(threads) as pool:
            arrs = list(pool.map(draw, range(len(jobs))))
        w = {k: [None] * L for k in per_layer}
        for (k, l, _, _), a in zip(jobs, arrs):
            if l is None:
                w[k] = a
            else:
                w[k][l] = a
        return w
    rng = np.random.default_rng(seed)

    def n(*shape, mean=0.0):
        return (mean + 0.02 * rng.standard_normal(shape, dtype=np.float32)).astype(np.float32)

    w = dict(tok_emb=n(V, D), norm_w=n(D, mean=1.0), lm_head=n(V, D))
    for k in ("attn_norm", "ffn_norm") + LLAMA_LINEAR_KEYS:
        w[k] = []
    for _ in range(L):
        w["attn_norm"].append(n(D, mean=1.0)); w["ffn_norm"].append(n(D, mean=1.0))
        w["wq"].append(n(D, D)); w["wk"].append(n(KD, D)); w["wv"].append(n(KD, D)); w["wo"].append(n(D, D))
        w["w_gate"].append(n(F, D)); w["w_up"].append(n(F, D)); w["w_down"].append(n(D, F))
    return w


def prompt(vocab: int, length: int = 16, seed: int = 0) -> list:
    rng = np.random.default_rng(seed + 1000)
    return [int(t) for t in rng.integers(0, vocab, size=length)]
