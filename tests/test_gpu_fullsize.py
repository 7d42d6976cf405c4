"""GPU parity at the sizes the benchmark figures are quoted on (the five configurations of the decode path), through
the C ABI.  Where the CPU oracle would need minutes, it checks sampled rows and the domain's size-independent
properties cover the rest; whole decoders at full width are checked against the independent fp64 PyTorch decoders
of tests/test_oracle_decoders.py (library routines only) on the dequantised weights.

Bars: token ids bit-exact; logits and activations within rtol 1e-3 / atol 1e-4.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-3, 1e-4


def close(a, b, rtol=RTOL, atol=ATOL):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    bad = np.abs(a - b) > atol + rtol * np.abs(b)
    assert not bad.any(), f"{bad.sum()} of {bad.size} differ; max abs err {np.abs(a - b).max():.3e}"


def _dequantised(oracle, weights, keys, kind):
    if kind == "f32":
        return weights
    from caten_amd.llm import Tensor
    out = dict(weights)
    for k in keys:
        if isinstance(weights[k], list):
            out[k] = [oracle.dequant(kind, Tensor.from_f32(a, kind).raw, a.size).reshape(a.shape) for a in weights[k]]
        else:
            a = weights[k]
            out[k] = oracle.dequant(kind, Tensor.from_f32(a, kind).raw, a.size).reshape(a.shape)
    return out


def test_row_ops_at_64x1024x768(oracle):
    """Configuration 2 at its real size: LayerNorm (eps 1e-5, gamma ~ N(1, 0.02), beta ~ N(0, 0.02)) -> softmax over
    the last axis, and GELU(tanh), on x ~ N(0, 1) of shape (64, 1024, 768).  Oracle on sampled rows; on every row:
    softmax rows sum to 1 and are non-negative, LayerNorm -> softmax does not see a constant added to its input,
    gelu(x) - gelu(-x) = x."""
    print("case: row ops (64,1024,768)", flush=True)
    from caten_amd import ops
    rng = np.random.default_rng(0)
    rows, d = 64 * 1024, 768
    x = rng.standard_normal((rows, d), dtype=np.float32)
    g = (1 + 0.02 * rng.standard_normal(d)).astype(np.float32)
    b = (0.02 * rng.standard_normal(d)).astype(np.float32)
    y = ops.layernorm_softmax(x, g, b, 1e-5)
    pick = rng.choice(rows, 96, replace=False)
    close(y[pick], oracle.softmax(oracle.layernorm(x[pick], g, b, 1e-5)))
    assert np.all(y >= 0) and np.allclose(y.sum(-1, dtype=np.float64), 1.0, atol=1e-5)
    y2 = ops.layernorm_softmax(x + np.float32(3.0), g, b, 1e-5)
    assert np.max(np.abs(y2 - y)) < 1e-5
    ln = ops.layernorm(x, g, b, 1e-5)
    close(ln[pick], oracle.layernorm(x[pick], g, b, 1e-5))
    # LayerNorm's output has the statistics its definition fixes: ((y - beta) / gamma) has mean 0 and variance 1 - eps-ish
    z = (ln.astype(np.float64) - b) / g
    assert np.max(np.abs(z.mean(-1))) < 1e-5 and np.max(np.abs(z.var(-1) - 1.0)) < 1e-3
    ge = ops.unary("gelu", x)
    close(ge[pick], oracle.gelu_tanh(x[pick]))
    gneg = ops.unary("gelu", -x)
    assert np.max(np.abs(ge.astype(np.float64) - gneg - x)) < 1e-5


def test_gpt2_small_fp32_full_size_matches_oracle(oracle):
    """Configuration 3 at its real size: GPT-2 small shape, fp32 weights, 16-token prompt, greedy decode against the
    CPU oracle (identical tokens, logits inside the band); then the 100-token decode of the configuration: the
    device-resident loop and the host-driven loop give the same tokens."""
    print("case: gpt2 small f32 full size", flush=True)
    from caten_amd import synth, llm
    cfg = synth.GPT2_CONFIGS["gpt2"]
    w = synth.gpt2_weights(cfg, seed=0)
    prompt = synth.prompt(cfg["vocab"], 16, seed=0)
    steps = 4
    ref = oracle.GPT2(cfg, w)
    want_tokens, want_logits = ref.generate(prompt, steps, onehot=False, keep_logits=True)
    sd = llm.gpt2_state_dict(w, "f32")
    model = llm.make_gpt2(cfg, sd)
    got_tokens, got_logits = llm.gpt2_generate(model, prompt, steps, on_device=False, keep_logits=True)
    assert got_tokens == want_tokens
    for g, r in zip(got_logits, want_logits):
        close(g, r)
    model.close()
    model = llm.make_gpt2(cfg, sd)
    long_run = llm.gpt2_generate(model, prompt, 100, on_device=True)
    assert long_run[:steps] == want_tokens
    # depth: the cache now holds 115 rows written by the device-resident loop.  One more forward, of the 100th token at
    # position 115: its logits against the independent fp64 decoder run over the whole 116-token history.
    import torch
    from tests.test_oracle_decoders import torch_gpt2_logits
    tok, late = model.forward([float(long_run[-1])], 1, len(prompt) + 99, return_logits=True)
    with torch.no_grad():
        ref = torch_gpt2_logits(cfg, w, list(prompt) + long_run)[-1].numpy()
    close(late, ref)
    assert tok == int(np.argmax(ref))
    model.close()
    model = llm.make_gpt2(cfg, sd)
    assert llm.gpt2_generate(model, prompt, 100, on_device=False) == long_run
    model.close()


def test_gpt2_small_q8_0_prefill_512_matches_fp64_decoder(oracle):
    """Configuration 4's prefill at its real size: 512 tokens through GPT-2 small Q8_0 as one batch (MFMA GEMMs on
    the packed weights, MFMA attention): last-row logits and greedy token against the independent fp64 decoder on
    the dequantised weights, cache rows against the oracle's Linear on sampled positions of layer 0, and the decode
    that continues from that cache against the fp64 decoder's next tokens."""
    print("case: gpt2 small q8_0 prefill 512", flush=True)
    import torch
    from caten_amd import synth, llm
    from tests.test_oracle_decoders import torch_gpt2_logits
    cfg = synth.GPT2_CONFIGS["gpt2"]
    w = synth.gpt2_weights(cfg, seed=0)
    wd = _dequantised(oracle, w, synth.GPT2_LINEAR_KEYS + ("lm_head",), "q8_0")
    prompt = synth.prompt(cfg["vocab"], 512, seed=0)
    model = llm.make_gpt2(cfg, llm.gpt2_state_dict(w, "q8_0"))
    tok, logits = model.forward([float(t) for t in prompt], 512, 0, return_logits=True)
    with torch.no_grad():
        ref = torch_gpt2_logits(cfg, wd, prompt)[-1].numpy()
    assert tok == int(np.argmax(ref))
    close(logits, ref)
    # layer-0 K / V rows of sampled positions: k, v = c_attn(LayerNorm(wte[id] + wpe[pos]))
    D = cfg["dim"]
    kc, vc = model.peek("k_cache.0"), model.peek("v_cache.0")
    for pos in (0, 1, 255, 511):
        x0 = wd["wte"][prompt[pos]] + wd["wpe"][pos]
        qkv = oracle.linear(oracle.layernorm(x0[None], wd["ln1_g"][0], wd["ln1_b"][0], cfg["eps"])[0], wd["attn_w"][0], wd["attn_b"][0])
        close(kc[pos * D:(pos + 1) * D], qkv[D:2 * D])
        close(vc[pos * D:(pos + 1) * D], qkv[2 * D:])
    # two more tokens from that cache: what the fp64 decoder continues with
    nxt = model.generate_on_device(2)
    toks = list(prompt) + [tok]
    for t in nxt:
        with torch.no_grad():
            want = int(torch.argmax(torch_gpt2_logits(cfg, wd, toks)[-1]))
        assert t == want
        toks.append(t)
    # depth: the logits of the forward at position 514 (512 prompt rows from the batch, two from the decode step)
    tok3, late = model.forward([float(toks[-1])], 1, len(toks) - 1, return_logits=True)
    with torch.no_grad():
        ref = torch_gpt2_logits(cfg, wd, toks)[-1].numpy()
    close(late, ref)
    assert tok3 == int(np.argmax(ref))
    model.close()


def test_llama_1b_q4_0_full_size(oracle):
    """Configuration 5 at its real size (22 layers, d 2048, 32 query / 4 KV heads, SwiGLU 5632, vocab 32000, Q4_0):
    a 128-token prompt as one batch -- last-row logits and greedy token against the independent fp64 decoder on the
    dequantised weights -- then 128 greedy tokens: the device-resident loop and the host-driven loop agree, and the
    first of them are the fp64 decoder's."""
    print("case: llama 1.1b q4_0 full size", flush=True)
    import torch
    from caten_amd import synth, llm
    from tests.test_oracle_decoders import torch_llama_logits
    cfg = synth.LLAMA_CONFIGS["llama-1.1b"]
    w = synth.llama_weights(cfg, seed=0)
    sd = llm.llama_state_dict(w, "q4_0")
    wd = _dequantised(oracle, w, synth.LLAMA_LINEAR_KEYS + ("lm_head",), "q4_0")
    del w
    prompt = synth.prompt(cfg["vocab"], 128, seed=0)
    model = llm.make_llama(cfg, sd)
    tok, logits = model.forward([float(t) for t in prompt], 128, 0, return_logits=True)
    with torch.no_grad():
        ref = torch_llama_logits(cfg, wd, prompt)[-1].numpy()
    assert tok == int(np.argmax(ref))
    close(logits, ref)
    on_device = [tok] + model.generate_on_device(127)
    # depth: the cache holds 255 rows, 127 of them written by the device-resident loop.  The forward of the 128th token
    # at position 255: its logits against the independent fp64 decoder over the whole 256-token history.
    tok_late, late = model.forward([float(on_device[-1])], 1, 255, return_logits=True)
    model.close()
    toks = list(prompt)
    for t in on_device[:2]:
        with torch.no_grad():
            want = int(torch.argmax(torch_llama_logits(cfg, wd, toks)[-1]))
        assert t == want
        toks.append(t)
    with torch.no_grad():
        ref = torch_llama_logits(cfg, wd, list(prompt) + on_device)[-1].numpy()
    close(late, ref)
    assert tok_late == int(np.argmax(ref))
    del wd
    model = llm.make_llama(cfg, sd)
    assert llm.gpt2_generate(model, prompt, 128, on_device=False) == on_device
    model.close()
