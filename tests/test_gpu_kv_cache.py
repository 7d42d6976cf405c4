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
    assert n0 == 5 and n1 == 5  # (the Q8_0 session's attention launch rotates, quantises and appends the new row itself)
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


@pytest.mark.parametrize("H,Hkv,Dh", [(4, 4, 64), (8, 2, 64), (4, 2, 32), (2, 1, 128)])
def test_append_and_attention_over_paged_rows(oracle, H, Hkv, Dh):
    """The cache in pages (option "kv_cache" 2; the reference allocates max_len rows at once, layers.lisp:25-26): rows
    appended through the page table come back from it, and one query row over the pages gives, bit for bit, what
    cthip_sdpa_cached gives over the same rows laid out densely -- and the oracle's attention inside rtol 1e-3 /
    atol 1e-4."""
    print(f"case: paged cache rows H {H} Hkv {Hkv} Dh {Dh}", flush=True)
    import ctypes as C
    from caten_amd import _lib
    from caten_amd.ops import DeviceArray
    lib = _lib.init()
    P = lib.cthip_kv_page_rows()
    assert P == 64
    KD, L = Hkv * Dh, 600
    npages = (L + P - 1) // P
    rng = np.random.default_rng(H * 11 + Dh)
    k = rng.standard_normal((L, KD)).astype(np.float32)
    v = rng.standard_normal((L, KD)).astype(np.float32)
    # pages in scrambled order, as an allocator hands them out
    order = rng.permutation(npages)
    kpool, vpool = DeviceArray((npages, P, KD), np.float32), DeviceArray((npages, P, KD), np.float32)
    ktab = np.array([kpool.ptr + 4 * int(order[p]) * P * KD for p in range(npages)], np.uint64)
    vtab = np.array([vpool.ptr + 4 * int(order[p]) * P * KD for p in range(npages)], np.uint64)
    dkt, dvt = DeviceArray.from_numpy(ktab), DeviceArray.from_numpy(vtab)
    dk, dv = DeviceArray.from_numpy(k), DeviceArray.from_numpy(v)
    for row0, s in ((0, 17), (17, 1), (18, 1), (19, 45), (64, 1), (65, L - 65)):  # pieces that end on, and cross, page edges
        _lib.check(lib.cthip_kv_append_paged(dkt.ptr, dvt.ptr, dk.ptr + 4 * row0 * KD, dv.ptr + 4 * row0 * KD, s, row0, KD))
    got_k = kpool.numpy()[order].reshape(npages * P, KD)[:L]
    got_v = vpool.numpy()[order].reshape(npages * P, KD)[:L]
    assert np.array_equal(got_k, k) and np.array_equal(got_v, v)
    out, ref = DeviceArray((H, Dh), np.float32), DeviceArray((H, Dh), np.float32)
    for T in (1, 2, 63, 64, 65, 255, 256, 257, 600):
        q = rng.standard_normal((1, H, Dh)).astype(np.float32)
        dq_ = DeviceArray.from_numpy(q)
        _lib.check(lib.cthip_sdpa_cached_paged(out.ptr, dq_.ptr, dkt.ptr, dvt.ptr, T, H, Hkv, Dh))
        _lib.check(lib.cthip_sdpa_cached(ref.ptr, dq_.ptr, dk.ptr, dv.ptr, 1, T - 1, H, Hkv, Dh))
        got = out.numpy()
        assert np.array_equal(got, ref.numpy()), T
        want = oracle.sdpa(q, k[:T].reshape(T, Hkv, Dh), v[:T].reshape(T, Hkv, Dh))[0]
        assert np.allclose(got, want, rtol=1e-3, atol=1e-4), (T, float(np.max(np.abs(got - want))))


@pytest.mark.parametrize("arch,plen", [("gpt2", 3), ("gpt2", 70), ("llama", 3), ("llama", 70), ("gpt2", 600), ("llama", 600)])
def test_decoder_with_a_paged_cache_equals_the_dense_cache(arch, plen):
    """A session whose cache lives in pages against one with the dense cache, both with one launch per Linear: a prompt
    fed row by row or as one batch that crosses a page edge, then decode steps across another edge.  Same tokens; for
    either shape the same logits and cache rows bit for bit (the arithmetic is the same, the rotation of q and the new
    key inside the attention launch included).  The prompts of 600 reach contexts whose keys
    several workgroups per head share, in both sessions.  The paged session holds the rows it has reached, not
    max_seq rows."""
    print(f"case: decoder with paged cache {arch} prompt {plen}", flush=True)
    import ctypes as C
    from caten_amd import _lib, synth, llm
    lib = _lib.init()
    if arch == "gpt2":
        cfg = dict(synth.GPT2_CONFIGS["gpt2-tiny"], max_seq=1024)
        sd = llm.gpt2_state_dict(synth.gpt2_weights(cfg, seed=23), "q8_0")
        make = llm.make_gpt2
    else:
        cfg = dict(synth.LLAMA_CONFIGS["llama-tiny"], max_seq=1024)
        sd = llm.llama_state_dict(synth.llama_weights(cfg, seed=23), "q4_0")
        make = llm.make_llama
    prompt = synth.prompt(cfg["vocab"], plen, seed=23)
    kd = cfg["dim"] // cfg["n_heads"] * cfg.get("n_kv_heads", cfg["n_heads"])
    steps = 70
    runs = {}
    live = C.c_size_t()
    try:
        _lib.check(lib.cthip_set_option(b"decode_fused", 0))
        for mode in (0, 2):
            _lib.check(lib.cthip_set_option(b"kv_cache", mode))
            _lib.check(lib.cthip_cache_stats(C.byref(live), None, None))
            before = live.value
            m = make(cfg, sd)
            toks, logs = llm.gpt2_generate(m, prompt, steps, on_device=False, keep_logits=True)
            _lib.check(lib.cthip_cache_stats(C.byref(live), None, None))
            held = live.value - before
            n_rows = plen + steps - 1
            k0 = m.peek("k_cache.0").reshape(cfg["max_seq"], kd).copy()
            vl = m.peek(f"v_cache.{cfg['n_layers'] - 1}").reshape(cfg["max_seq"], kd).copy()
            launches = lib.cthip_decoder_layer_launches(m.handle)
            m.close()
            m = make(cfg, sd)
            assert llm.gpt2_generate(m, prompt, steps, on_device=True) == toks  # the device-resident loop, pages opened ahead
            m.close()
            runs[mode] = (toks, logs, k0, vl, launches, held, n_rows)
    finally:
        _lib.check(lib.cthip_set_option(b"kv_cache", 0))
        _lib.check(lib.cthip_set_option(b"decode_fused", 1))
    (t0, l0, k0, v0, n0, held0, n_rows), (t2, l2, k2, v2, n2, held2, _) = runs[0], runs[2]
    assert t0 == t2
    assert n0 == 5 and n2 == 5  # (the paged session's attention launch rotates and appends the new row itself)
    # the same arithmetic in the same order, rotation included: logits and cache rows bit for bit
    assert all(np.array_equal(a, b) for a, b in zip(l0, l2))
    assert np.array_equal(k0, k2) and np.array_equal(v0, v2)
    assert not k2[n_rows:].any()  # rows never reached read as zeros, as the dense cache holds them
    # the dense session holds max_seq rows per layer, the paged one three pages (139 or 72 rows reached)
    dense_rows = 2 * cfg["n_layers"] * cfg["max_seq"] * kd * 4
    if n_rows <= 256:
        assert held0 - held2 > dense_rows // 2, (held0, held2, dense_rows)
    else:
        assert held0 > held2, (held0, held2)


@pytest.mark.parametrize("name,wtype,plen", [("gpt2-tiny", "q8_0", 3), ("gpt2-tiny", "q4_0", 20), ("gpt2-mini", "q8_0", 5),
                                              ("gpt2-mini", "q8_0", 505)])
def test_three_launch_layer_over_a_q8_0_cache(oracle, name, wtype, plen):
    """GPT-2 shapes keep three launches per layer over Q8_0 cache rows: the attention launch quantises the step's new
    row itself.  Bars: layer 0's planes are the oracle's quantisation of the rows the fp32-cache session of the same
    three-launch layer wrote, bit for bit (decoded rows and batched prompt rows alike); logits inside the 8-bit band of
    the five-launch Q8_0 session; two runs bit-identical; the device-resident loop gives the same tokens.  The long
    prompt makes the decode steps cross the 512 keys one pass of the launch covers."""
    print(f"case: three-launch layer over q8_0 cache {name} {wtype} prompt {plen}", flush=True)
    from caten_amd import _lib, synth, llm
    lib = _lib.init()
    cfg = dict(synth.GPT2_CONFIGS[name], n_layers=2)
    if plen > 100:
        cfg["max_seq"] = 640
    sd = llm.gpt2_state_dict(synth.gpt2_weights(cfg, seed=31), wtype)
    prompt = synth.prompt(cfg["vocab"], plen, seed=31)
    kd, steps = cfg["dim"], 14
    n_rows = plen + steps - 1
    runs = []
    try:
        for kv, fused in ((1, 1), (1, 0), (0, 1), (1, 1)):
            _lib.check(lib.cthip_set_option(b"kv_cache", kv))
            _lib.check(lib.cthip_set_option(b"decode_fused", fused))
            m = llm.make_gpt2(cfg, sd)
            toks, logs = llm.gpt2_generate(m, prompt, steps, on_device=False, keep_logits=True)
            launches = lib.cthip_decoder_layer_launches(m.handle)
            rows = [m.peek(f"{n}.0").reshape(cfg["max_seq"], kd)[:n_rows].copy() for n in ("k_cache", "v_cache")]
            planes = None
            if kv:
                planes = [(m.peek(f"{n}_cache_q8.0").view(np.int8).reshape(cfg["max_seq"], kd)[:n_rows].copy(),
                           m.peek(f"{n}_cache_d.0").view(np.uint16).reshape(cfg["max_seq"], kd // 32)[:n_rows].copy())
                          for n in ("k", "v")]
            m.close()
            if kv and fused:
                m = llm.make_gpt2(cfg, sd)
                assert llm.gpt2_generate(m, prompt, steps, on_device=True) == toks
                m.close()
            runs.append((toks, logs, launches, rows, planes))
    finally:
        _lib.check(lib.cthip_set_option(b"kv_cache", 0))
        _lib.check(lib.cthip_set_option(b"decode_fused", 1))
    a, b, f, a2 = runs
    assert (a[2], b[2], f[2]) == (3, 5, 3)
    assert a[0] == a2[0] and all(np.array_equal(x, y) for x, y in zip(a[1], a2[1]))
    for (q, d), (q2, d2) in zip(a[4], a2[4]):
        assert np.array_equal(q, q2) and np.array_equal(d, d2)

    def agree(t0, t1):
        n = 0
        while n < steps and t0[n] == t1[n]:
            n += 1
        return n

    # against the five-launch session over the same kind of cache: a near-tie may turn the greedy choice
    same = agree(a[0], b[0])
    print("tokens", a[0], b[0], "agree for", same, flush=True)
    assert same >= steps // 2
    for x, y in zip(a[1][:same + 1], b[1][:same + 1]):
        assert np.allclose(x, y, rtol=2e-2, atol=2e-2), float(np.max(np.abs(x - y)))
    # against the fp32 cache of the same three launches: layer 0's rows depend on the tokens only
    same = agree(a[0], f[0])
    assert same >= steps // 2
    rows = min(plen + same, n_rows)
    for (q, d), r in zip(a[4], f[3]):
        want_q, want_d = _planes(oracle, r[:rows])
        assert np.array_equal(q[:rows], want_q) and np.array_equal(d[:rows], want_d)
    for x, y in zip(a[1][:same + 1], f[1][:same + 1]):
        assert np.allclose(x, y, rtol=2e-2, atol=2e-2), float(np.max(np.abs(x - y)))
    assert not np.array_equal(a[1][-1], f[1][-1])  # the cache IS quantised
