#!/usr/bin/env python3
"""Prefill timing on one MI355X (`python bench_prefill.py`): a 512-token prompt through the
GPT-2-small shaped Q8_0 model as one batch (the prefill leg of the GPT-2 Q8_0 benchmark configuration; `--model llama-1.1b
--kind q4_0 --tokens 128` is the Llama-1.1B Q4_0 configuration's): MFMA GEMMs over the
rows with the weights dequantised while staged.  Reports the wall time of `forward` (synchronous) and
the linear-layer FLOP rate against the MFMA peak of the operand type.  The logits of every operand format are checked
against the fp32-operand run (fp32-grade formats: rtol 1e-3 / atol 1e-4 per logit; bf16: 5e-2 of the vector's norm) and the greedy token must agree
before a figure is printed."""
from __future__ import annotations

import json
import time

import numpy as np

import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

from caten_amd import _lib, llm, synth  # noqa: E402


def measure(model="gpt2", kind="q8_0", s=512, modes=(0, 3, 2, 1), weights=None, reps=5):
    """one dict per operand format in `modes` (the first one is the reference the others' logits are checked against)"""
    llama = model in synth.LLAMA_CONFIGS
    cfg = synth.LLAMA_CONFIGS[model] if llama else synth.GPT2_CONFIGS[model]
    w = weights if weights is not None else (synth.llama_weights(cfg, seed=0) if llama else synth.gpt2_weights(cfg, seed=0))
    prompt = [float(t) for t in synth.prompt(cfg["vocab"], s, seed=0)]
    lib = _lib.init(0)
    m = llm.make_llama(cfg, llm.llama_state_dict(w, kind)) if llama else llm.make_gpt2(cfg, llm.gpt2_state_dict(w, kind))
    D, F, L, V = cfg["dim"], cfg["ffn"], cfg["n_layers"], cfg["vocab"]
    if llama:
        KD = D // cfg["n_heads"] * cfg["n_kv_heads"]
        lin_flop = 2.0 * s * L * (D * (D + 2 * KD) + D * D + 3 * D * F) + 2.0 * V * D
    else:
        lin_flop = 2.0 * s * L * (3 * D * D + D * D + 2 * D * F) + 2.0 * V * D  # lm_head on the last row only
    att_flop = 2.0 * 2.0 * L * cfg["n_heads"] * (D // cfg["n_heads"]) * s * (s + 1) / 2
    names = {0: "fp32", 3: "3-term split bf16 (6 MFMAs per product)", 2: "2-term split bf16 (3 MFMAs per product)", 1: "bf16"}
    ref_tok = ref_logits = None
    peaks = {0: 157.3, 3: 2500.0, 2: 2500.0, 1: 2500.0}
    out = []
    for mode in modes:
        peak = peaks[mode]
        _lib.check(lib.cthip_set_option(b"gemm_precision", mode))
        tok, logits = m.forward(prompt, s, 0, return_logits=True)
        if ref_logits is None:
            ref_tok, ref_logits = tok, logits.astype(np.float64)
        else:
            if mode == 1:
                # operands rounded to bf16 through every layer: checked as a whole (relative error of the logits vector)
                rel = np.linalg.norm(logits - ref_logits) / np.linalg.norm(ref_logits)
                bad = np.array([not rel < 5e-2])
            else:
                bad = np.abs(logits - ref_logits) > 1e-4 + 1e-3 * np.abs(ref_logits)
            if bad.any() or (tok != ref_tok and mode != 1):
                raise SystemExit(f"bench_prefill: {names[mode]}: {int(bad.sum())} logits differ from the fp32-operand run "
                                 f"(token {tok} vs {ref_tok}); no figure is reported for a wrong result")
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            m.forward(prompt, s, 0)
            ts.append(time.perf_counter() - t0)
        t = min(ts)
        out.append({"item": f"prefill {s} tokens {model} {kind} ({names[mode]} MFMA operands)", "gemm_precision": mode,
                    "ms": t * 1e3, "tokens_per_s": s / t, "linear_TFLOPs": lin_flop / t / 1e12,
                    "peak_TFLOPs": peak, "frac": lin_flop / t / 1e12 / peak,
                    "linear_GFLOP": lin_flop / 1e9, "attention_GFLOP": att_flop / 1e9})
    _lib.check(lib.cthip_set_option(b"gemm_precision", 2))
    m.close()
    return out


def main(model="gpt2", kind="q8_0", s=512):
    for o in measure(model, kind, s):
        print(json.dumps(o))


if __name__ == "__main__":
    import argparse
    ap = argparse.ArgumentParser()
    ap.add_argument("--model", default="gpt2")
    ap.add_argument("--kind", default="q8_0")
    ap.add_argument("--tokens", type=int, default=512)
    a = ap.parse_args()
    main(a.model, a.kind, a.tokens)
