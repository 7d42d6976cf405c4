"""The KV cache as GGUF-Q8_0 rows (option "kv_cache" 1).  The reference's cache is dense fp32
(external/llm/layers.lisp:19-33) and it has no quantised cache to compare with, so the bars are: the stored planes are
bit-exactly what ggml's Q8_0 row quantiser (the oracle's, pinned against the reference's block layout in
tests/test_oracle_pins.py) makes of the fp32 rows; attention over the planes equals the oracle's attention over their
dequantised values inside the fp32 band; and a whole decoder with such a cache stays within rtol 2e-2 / atol 2e-2 of
the same decoder with the fp32 cache -- the band of 8-bit keys and values."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _planes(oracle, rows):
    """(quant plane int8 [n][KD], scale plane fp16 bits [n][KD/32]) the oracle's quantiser makes of fp32 rows"""
    n, kd = rows.shape
    raw = oracle.quantize("q8_0", rows).reshape(n, kd // 32, 34)
    return raw[:, :, 2:].reshape(n, kd).view(np.int8), raw[:, :, :2].copy().view(np.uint16).reshape(n, kd // 32)


@pytest.mark.parametrize("H,Hkv,Dh", [(4, 4, 64), (8, 2, 64), (4, 2, 32), (2, 1, 128)])
def test_append_and_attention_over_q8_0_rows(oracle, H, Hkv, Dh):
    print(f"case: q8_0 cache rows H {H} Hkv {Hkv} Dh {Dh}", flush=True)
    from caten_amd import _lib
    from caten_amd.ops import DeviceArray
    lib = _lib.init()
    KD, L = Hkv * Dh, 600
    rng = np.random.default_rng(H * 7 + Dh)
    k = rng.standard_normal((L, KD)).astype(np.float32) * rng.uniform(0.01, 3.0, (L, 1)).astype(np.float32)
    v = rng.standard_normal((L, KD)).astype(np.float32)
    k[5, :32] = 0.0  # a block of zeros: scale 0
    k[7, 3] = 1e4    # a large value among small ones
    planes = {}
    for name, a in (("k", k), ("v", v)):
        dq, dd = DeviceArray((L, KD), np.int8), DeviceArray((L, KD // 32), np.uint16)
        src = DeviceArray.from_numpy(a)
        # appended in pieces, as a session does: a prompt, then row by row, then another batch
        for row0, s in ((0, 17), (17, 1), (18, 1), (19, L - 19)):
            _lib.check(lib.cthip_kv_append_q8(dq.ptr, dd.ptr, src.ptr + 4 * row0 * KD, s, row0, KD))
        want_q, want_d = _planes(oracle, a)
        assert np.array_equal(dq.numpy(), want_q) and np.array_equal(dd.numpy(), want_d), name
        planes[name] = (dq, dd)
    kd_f = oracle.dequant("q8_0", oracle.quantize("q8_0", k), k.size).reshape(L, Hkv, Dh)
    vd_f = oracle.dequant("q8_0", oracle.quantize("q8_0", v), v.size).reshape(L, Hkv, Dh)
    out = DeviceArray((H, Dh), np.float32)
    for T in (1, 2, 63, 64, 65, 255, 256, 257, 600):
        q = rng.standard_normal((1, H, Dh)).astype(np.float32)
        dq_ = DeviceArray.from_numpy(q)
        _lib.check(lib.cthip_sdpa_cached_q8(out.ptr, dq_.ptr, planes["k"][0].ptr, planes["k"][1].ptr, planes["v"][0].ptr,
                                            planes["v"][1].ptr, T, H, Hkv, Dh))
        want = oracle.sdpa(q, kd_f[:T], vd_f[:T])[0]
        got = out.numpy()
        assert np.allclose(got, want, rtol=1e-3, atol=1e-4), (T, float(np.max(np.abs(got - want))))


@pytest.mark.parametrize("arch,plen", [("gpt2", 3), ("gpt2", 12), ("llama", 3), ("llama", 12)])
def test_decoder_with_a_q8_0_cache_stays_in_the_band_of_the_fp32_cache(oracle, arch, plen):
    """A short prompt goes row by row through the decode step, a longer one as one batch; both then decode.  Layer 0's
    cache rows depend on the tokens only, so its planes must be the quantised fp32 rows of the other session bit for bit."""
    print(f"case: decoder with q8_0 cache {arch} prompt {plen}", flush=True)
    from caten_amd import _lib, synth, llm
    lib = _lib.init()
    if arch == "gpt2":
        cfg = synth.GPT2_CONFIGS["gpt2-tiny"]
        sd = llm.gpt2_state_dict(synth.gpt2_weights(cfg, seed=21), "q8_0")
        make = llm.make_gpt2
    else:
        cfg = synth.LLAMA_CONFIGS["llama-tiny"]
        sd = llm.llama_state_dict(synth.llama_weights(cfg, seed=21), "q4_0")
        make = llm.make_llama
    prompt = synth.prompt(cfg["vocab"], plen, seed=21)
    kd = cfg["dim"] // cfg["n_heads"] * cfg.get("n_kv_heads", cfg["n_heads"])
    steps = 12
    runs = {}
    try:
        for mode in (0, 1):
            _lib.check(lib.cthip_set_option(b"kv_cache", mode))
            _lib.check(lib.cthip_set_option(b"decode_fused", 0))  # the fp32 session with the same arithmetic per Linear
            m = make(cfg, sd)
            toks, logs = llm.gpt2_generate(m, prompt, steps, on_device=False, keep_logits=True)
            n_rows = plen + steps - 1
            k0 = m.peek("k_cache.0").reshape(cfg["max_seq"], kd)[:n_rows].copy()
            launches = lib.cthip_decoder_layer_launches(m.handle)
            extra = None
            if mode == 1:
                extra = (m.peek("k_cache_q8.0").view(np.int8).reshape(cfg["max_seq"], kd)[:n_rows].copy(),
                         m.peek("k_cache_d.0").view(np.uint16).reshape(cfg["max_seq"], kd // 32)[:n_rows].copy())
                per_row = (kd + kd // 32 * 2) * 2 * cfg["n_layers"]
                assert m.step_bytes(11) - m.step_bytes(10) == per_row  # what a step reads grows by the rows' packed size
            # the device-resident loop on the same kind of session gives the same tokens
            m.close()
            m = make(cfg, sd)
            assert llm.gpt2_generate(m, prompt, steps, on_device=True) == toks
            m.close()
            runs[mode] = (toks, logs, k0, extra, launches)
    finally:
        _lib.check(lib.cthip_set_option(b"kv_cache", 0))
        _lib.check(lib.cthip_set_option(b"decode_fused", 1))
    (t0, l0, k0, _, n0), (t1, l1, k1, (q1, d1), n1) = runs[0], runs[1]
    assert n0 == 5 and n1 == (7 if arch == "gpt2" else 9)
    # 8-bit keys and values may turn a near-tie of the greedy choice; from there on the two sessions see other tokens.
    # Everything is compared over the steps that had the same history (at least the prompt and half of the decode).
    same = 0
    while same < steps and t0[same] == t1[same]:
        same += 1
    print("tokens", t0, t1, "agree for", same, flush=True)
    assert same >= steps // 2, (t0, t1)
    for a, b in zip(l0[:same + 1], l1[:same + 1]):
        assert np.allclose(b, a, rtol=2e-2, atol=2e-2), float(np.max(np.abs(a - b)))
    if same < steps:  # the step that chose differently did so on a near-tie of the fp32 session's logits
        a = l0[same]
        assert abs(a[t0[same]] - a[t1[same]]) < 2e-2 * (1.0 + abs(a[t0[same]]))
    rows = min(plen + same, k0.shape[0])  # cache rows written from identical inputs
    want_q, want_d = _planes(oracle, k0[:rows])
    assert np.array_equal(q1[:rows], want_q) and np.array_equal(d1[:rows], want_d)
    assert np.array_equal(k1[:rows], oracle.dequant("q8_0", oracle.quantize("q8_0", k0[:rows]), rows * kd).reshape(rows, kd))
    assert not np.array_equal(l0[same if same < steps else -1], l1[same if same < steps else -1])  # the cache IS quantised


def test_three_launch_layer_is_what_supported_shapes_run():
    """the load-time checks the three-launch layer depends on (XCD ids 0..7; atomics of different workgroups of an XCD
    meeting in its L2) pass on this device, for both layer families"""
    from caten_amd import _lib, synth, llm
    lib = _lib.init()
    cfg = synth.GPT2_CONFIGS["gpt2-mini"]
    m = llm.make_gpt2(cfg, llm.gpt2_state_dict(synth.gpt2_weights(cfg, seed=1), "q8_0"))
    assert lib.cthip_decoder_layer_launches(m.handle) == 3
    m.close()
    cfg = dict(synth.LLAMA_CONFIGS["llama-1.1b"], n_layers=1, max_seq=64, vocab=500)
    m = llm.make_llama(cfg, llm.llama_state_dict(synth.llama_weights(cfg, seed=1), "q4_0"))
    assert lib.cthip_decoder_layer_launches(m.handle) == 3
    m.close()
