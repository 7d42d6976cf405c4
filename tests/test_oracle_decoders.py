"""Pins the oracle's whole-decoder functions against independent fp64 PyTorch decoders built
only from library routines (F.layer_norm, F.embedding, F.scaled_dot_product_attention, F.gelu,
F.silu, torch.argmax) -- nothing here shares code with oracle/caten_oracle.c."""
import numpy as np
import torch
import torch.nn.functional as F


def _t(a):
    return torch.from_numpy(np.ascontiguousarray(a)).double()


def torch_gpt2_logits(cfg, w, tokens):
    """Full (uncached) forward over `tokens`; returns the logits of every position."""
    D, H = cfg["dim"], cfg["n_heads"]
    ids = torch.tensor(tokens, dtype=torch.long)
    S = ids.numel()
    x = F.embedding(ids, _t(w["wte"])) + _t(w["wpe"])[:S]
    for l in range(cfg["n_layers"]):
        h = F.layer_norm(x, (D,), _t(w["ln1_g"][l]), _t(w["ln1_b"][l]), cfg["eps"])
        qkv = F.linear(h, _t(w["attn_w"][l]), _t(w["attn_b"][l]))
        q, k, v = (t.reshape(S, H, D // H).transpose(0, 1) for t in qkv.split(D, dim=-1))
        a = F.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(0, 1).reshape(S, D)
        x = x + F.linear(a, _t(w["proj_w"][l]), _t(w["proj_b"][l]))
        h = F.layer_norm(x, (D,), _t(w["ln2_g"][l]), _t(w["ln2_b"][l]), cfg["eps"])
        h = F.gelu(F.linear(h, _t(w["fc_w"][l]), _t(w["fc_b"][l])), approximate="tanh")
        x = x + F.linear(h, _t(w["fc2_w"][l]), _t(w["fc2_b"][l]))
    x = F.layer_norm(x, (D,), _t(w["lnf_g"]), _t(w["lnf_b"]), cfg["eps"])
    return F.linear(x, _t(w["lm_head"]))


def _rope(x, base, start=0):  # x (S, H, Dh), interleaved pairs
    S, H, Dh = x.shape
    theta = 1.0 / (base ** (torch.arange(0, Dh, 2).double() / Dh))
    ang = torch.arange(start, start + S).double()[:, None] * theta[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    x0, x1 = x[..., 0::2], x[..., 1::2]
    return torch.stack([x0 * c - x1 * s, x0 * s + x1 * c], dim=-1).flatten(-2)


def torch_llama_logits(cfg, w, tokens):
    D, H, Hkv = cfg["dim"], cfg["n_heads"], cfg["n_kv_heads"]
    Dh = D // H
    ids = torch.tensor(tokens, dtype=torch.long)
    S = ids.numel()

    def rms(x, wt):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + cfg["eps"]) * _t(wt)

    x = F.embedding(ids, _t(w["tok_emb"]))
    for l in range(cfg["n_layers"]):
        h = rms(x, w["attn_norm"][l])
        q = _rope(F.linear(h, _t(w["wq"][l])).reshape(S, H, Dh), cfg["rope_base"])
        k = _rope(F.linear(h, _t(w["wk"][l])).reshape(S, Hkv, Dh), cfg["rope_base"])
        v = F.linear(h, _t(w["wv"][l])).reshape(S, Hkv, Dh)
        k, v = (t.repeat_interleave(H // Hkv, dim=1) for t in (k, v))
        a = F.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True)
        x = x + F.linear(a.transpose(0, 1).reshape(S, D), _t(w["wo"][l]))
        h = rms(x, w["ffn_norm"][l])
        x = x + F.linear(F.silu(F.linear(h, _t(w["w_gate"][l]))) * F.linear(h, _t(w["w_up"][l])), _t(w["w_down"][l]))
    return F.linear(rms(x, w["norm_w"]), _t(w["lm_head"]))


def _greedy(logits_fn, cfg, w, prompt, steps):
    toks = list(prompt)
    out, logs = [], []
    for _ in range(steps):
        lg = logits_fn(cfg, w, toks)[-1]
        t = int(torch.argmax(lg))
        toks.append(t)
        out.append(t)
        logs.append(lg.numpy())
    return out, logs


def test_gpt2_oracle_vs_torch_fp64(oracle):
    from caten_amd import synth
    cfg = synth.GPT2_CONFIGS["gpt2-tiny"]
    w = synth.gpt2_weights(cfg, seed=5)
    prompt = synth.prompt(cfg["vocab"], 7, seed=5)
    want_t, want_l = _greedy(torch_gpt2_logits, cfg, w, prompt, 6)
    m = oracle.GPT2(cfg, w)
    got_t, got_l = m.generate(prompt, 6, onehot=True, all_logits=True, keep_logits=True)
    assert got_t == want_t
    for g, r in zip(got_l, want_l):
        assert np.max(np.abs(g - r)) < 1e-4
    # the row-copy embedding and last-row-only lm_head shortcuts give the same values
    m2 = oracle.GPT2(cfg, w)
    t2, l2 = m2.generate(prompt, 6, onehot=False, all_logits=False, keep_logits=True)
    assert t2 == got_t and all(np.array_equal(a, b) for a, b in zip(l2, got_l))
    # a prompt pushed through one forward (prefill) equals feeding it token by token
    m3 = oracle.GPT2(cfg, w)
    for i, t in enumerate(prompt):
        tok, lg = m3.forward([t], i)
    assert tok == got_t[0] and np.max(np.abs(lg - got_l[0])) < 1e-5
    # KV cache rows hold k and v of every fed position (layers.lisp:30-31)
    assert np.any(m.k_cache[0][len(prompt) + 4] != 0) and np.all(m.k_cache[0][len(prompt) + 5:] == 0)


def test_llama_oracle_vs_torch_fp64(oracle):
    from caten_amd import synth
    cfg = synth.LLAMA_CONFIGS["llama-tiny"]
    w = synth.llama_weights(cfg, seed=6)
    prompt = synth.prompt(cfg["vocab"], 6, seed=6)
    want_t, want_l = _greedy(torch_llama_logits, cfg, w, prompt, 5)
    m = oracle.Llama(cfg, w)
    got_t, got_l = m.generate(prompt, 5, keep_logits=True)
    assert got_t == want_t
    for g, r in zip(got_l, want_l):
        assert np.max(np.abs(g - r)) < 2e-4
