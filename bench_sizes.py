#!/usr/bin/env python3
"""Batch-1 greedy decode across model sizes on one MI355X: what fraction of the HBM roofline the same kernels
reach as the bytes per step grow from 0.13 GB (GPT-2 small, the headline workload, bound by launch and memory
round-trip latencies) to tens of GB (a 70B-parameter shape in Q4_0, which one GPU's 288 GB holds).

Shapes: the reference's GPT-2 table (apps/gpt2/gpt2.lisp:36-44) with Q8_0 weights and Llama-shaped models
(external/llm/layers.lisp; TinyLlama-1.1B and the public Llama-2 shapes) with Q4_0 weights (--llama-kind q8_0 / f16
for the other formats).  Weights are synthetic: ONE layer is drawn and quantised on the host and loaded into every
layer of the session, so the host work stays small while every layer has its own copy in HBM (a step reads every
byte of every copy).  One JSON line per model:
  {"model", "kind", "weights_GB", "us_per_step", "tokens_per_s", "bytes_per_step", "GBps", "frac", "launches_per_layer"}
`frac` = algorithmic bytes per step (cthip_decoder_step_bytes) / time / 8 TB/s.

  python bench_sizes.py [--models gpt2,gpt2-xl,llama-7b,...] [--steps 64] [--prompt 16] [--option NAME=VALUE]
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import sys
import time

import numpy as np

HBM_PEAK_GBS = 8000.0

LLAMA_SHAPES = {
    "llama-1.1b": dict(n_layers=22, n_heads=32, n_kv_heads=4, dim=2048, ffn=5632, vocab=32000),
    "llama-7b": dict(n_layers=32, n_heads=32, n_kv_heads=32, dim=4096, ffn=11008, vocab=32000),
    "llama-13b": dict(n_layers=40, n_heads=40, n_kv_heads=40, dim=5120, ffn=13824, vocab=32000),
    "llama-70b": dict(n_layers=80, n_heads=64, n_kv_heads=8, dim=8192, ffn=28672, vocab=32000),
}
DEFAULT = "gpt2,gpt2-medium,gpt2-large,gpt2-xl,llama-1.1b,llama-7b,llama-13b,llama-70b"


def shared_layer_state_dict(name: str, kind: str, max_seq: int):
    """(cfg, arch, state dict) with one drawn layer under every layer's keys"""
    from caten_amd import llm, synth
    if name in synth.GPT2_CONFIGS:
        cfg = dict(synth.GPT2_CONFIGS[name], max_seq=max_seq)
        one = llm.gpt2_state_dict(synth.gpt2_weights(dict(cfg, n_layers=1), seed=0), kind)
        prefix, arch = "h.", "gpt2"
    else:
        cfg = dict(LLAMA_SHAPES[name], max_seq=max_seq, eps=1e-5, rope_base=10000.0)
        one = llm.llama_state_dict(synth.llama_weights(dict(cfg, n_layers=1), seed=0, threads=8), kind, threads=8)
        prefix, arch = "layers.", "llama"
    sd = {}
    for key, t in one.items():
        if key.startswith(prefix + "0."):
            for l in range(cfg["n_layers"]):
                sd[prefix + str(l) + key[len(prefix) + 1:]] = t
        else:
            sd[key] = t
    return cfg, arch, sd


def run(name: str, kind: str, steps: int, plen: int, max_seq: int) -> dict:
    from caten_amd import _lib, llm, synth
    lib = _lib.init()
    t0 = time.perf_counter()
    cfg, arch, sd = shared_layer_state_dict(name, kind, max_seq)
    weights_bytes = sum(t.raw.size for key, t in sd.items() if t.kind == kind and t.rows > 1)
    print(f"# {name}: weights drawn in {time.perf_counter() - t0:.1f} s, {weights_bytes / 1e9:.2f} GB of {kind} Linears", file=sys.stderr, flush=True)
    t0 = time.perf_counter()
    model = (llm.make_gpt2 if arch == "gpt2" else llm.make_llama)(cfg, sd)
    print(f"# {name}: loaded in {time.perf_counter() - t0:.1f} s", file=sys.stderr, flush=True)
    prompt = synth.prompt(cfg["vocab"], plen, seed=1)
    model.forward([float(t) for t in prompt], len(prompt), 0)
    model.generate_on_device(8)  # picks kernels, captures the step graphs
    best = None
    for _ in range(3):
        model.forward([float(t) for t in prompt], len(prompt), 0)
        model.generate_on_device(8)
        pos0 = model.position
        out = np.empty(steps, np.int64)
        _lib.check(lib.cthip_sync())
        _lib.check(lib.cthip_timer_start())
        _lib.check(lib.cthip_decoder_generate(model.handle, steps, out.ctypes.data))
        ms = C.c_float()
        _lib.check(lib.cthip_timer_stop(C.byref(ms)))
        us = ms.value * 1e3 / steps
        best = us if best is None else min(best, us)
    step_bytes = float(np.mean([model.step_bytes(t + 1) for t in range(pos0, pos0 + steps)]))
    launches = int(lib.cthip_decoder_layer_launches(model.handle))
    model.close()
    gbs = step_bytes / (best * 1e-6) / 1e9
    return {"model": name, "kind": kind, "weights_GB": round(weights_bytes / 1e9, 3), "us_per_step": round(best, 1),
            "tokens_per_s": round(1e6 / best, 1), "bytes_per_step": int(step_bytes), "GBps": round(gbs, 1),
            "frac": round(gbs / HBM_PEAK_GBS, 4), "launches_per_layer": launches,
            "positions": f"{pos0}..{pos0 + steps - 1}"}


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--models", default=DEFAULT)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--prompt", type=int, default=16)
    ap.add_argument("--max-seq", type=int, default=256)
    ap.add_argument("--gpt2-kind", default="q8_0")
    ap.add_argument("--llama-kind", default="q4_0")
    ap.add_argument("--option", action="append", default=[], metavar="NAME=VALUE",
                    help="cthip_set_option before the sessions are created (decoder_graph=0: steps launched one by one)")
    args = ap.parse_args()
    from caten_amd import _lib, synth
    for kv in args.option:
        name, value = kv.split("=")
        _lib.check(_lib.init().cthip_set_option(name.encode(), int(value)))
    for name in args.models.split(","):
        if name not in synth.GPT2_CONFIGS and name not in LLAMA_SHAPES:
            raise SystemExit(f"bench_sizes: unknown model {name}")
        kind = args.gpt2_kind if name in synth.GPT2_CONFIGS else args.llama_kind
        print(json.dumps(run(name, kind, args.steps, args.prompt, args.max_seq)), flush=True)


if __name__ == "__main__":
    main()
