"""GPU parity of the decode path end to end: Transformer.forward / gpt2-generate through the
C ABI against the CPU oracle on the same seeded weights and prompt.

Bars: token ids bit-exact; last-position logits within rtol 1e-3 / atol 1e-4 of the oracle,
which runs on the dequantised fp32 weights (the reference's only mode, dequantize.lisp:3-5).
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
    """What the reference would compute with: every Linear weight quantised then dequantised."""
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


@pytest.mark.parametrize("name,kind", [("gpt2-tiny", "f32"), ("gpt2-tiny", "q8_0"), ("gpt2-tiny", "q4_0"),
                                       ("gpt2-tiny", "f16"), ("gpt2-mini", "q8_0"), ("gpt2-mini", "q4_0")])
def test_gpt2_generate_matches_oracle(oracle, name, kind):
    print(f"case: gpt2 decode {name} {kind}", flush=True)
    from caten_amd import synth, llm
    cfg = synth.GPT2_CONFIGS[name]
    w = synth.gpt2_weights(cfg, seed=0)
    prompt = synth.prompt(cfg["vocab"], 16, seed=0)
    steps = 12
    ref = oracle.GPT2(cfg, _dequantised(oracle, w, synth.GPT2_LINEAR_KEYS + ("lm_head",), kind))
    want_tokens, want_logits = ref.generate(prompt, steps, onehot=(name == "gpt2-tiny"), keep_logits=True)

    model = llm.make_gpt2(cfg, llm.gpt2_state_dict(w, kind))
    assert model.lib.cthip_decoder_layer_launches(model.handle) == 3  # every weight format runs the three-launch layer
    got_tokens, got_logits = llm.gpt2_generate(model, prompt, steps, on_device=False, keep_logits=True)
    assert got_tokens == want_tokens
    for g, r in zip(got_logits, want_logits):
        close(g, r)
    # the KV cache rows written so far equal the oracle's
    T = len(prompt) + steps - 1
    for l in (0, cfg["n_layers"] - 1):
        close(model.peek(f"k_cache.{l}")[:T * cfg["dim"]], ref.k_cache[l].ravel()[:T * cfg["dim"]])
        close(model.peek(f"v_cache.{l}")[:T * cfg["dim"]], ref.v_cache[l].ravel()[:T * cfg["dim"]])
    model.close()

    # the device-resident loop yields the same tokens as the host-driven one
    model = llm.make_gpt2(cfg, llm.gpt2_state_dict(w, kind))
    assert llm.gpt2_generate(model, prompt, steps, on_device=True) == want_tokens
    assert model.position == len(prompt) + steps - 1
    model.close()


def test_gpt2_long_context_attention(oracle):
    """Positions past 512: the attention kernel walks the cache in several passes."""
    print("case: gpt2 decode to position 600", flush=True)
    from caten_amd import synth, llm
    cfg = dict(synth.GPT2_CONFIGS["gpt2-tiny"], max_seq=640)
    w = synth.gpt2_weights(cfg, seed=6)
    prompt = synth.prompt(cfg["vocab"], 250, seed=6)
    steps = 350
    ref = oracle.GPT2(cfg, _dequantised(oracle, w, synth.GPT2_LINEAR_KEYS + ("lm_head",), "q8_0"))
    want = ref.generate(prompt, steps)
    model = llm.make_gpt2(cfg, llm.gpt2_state_dict(w, "q8_0"))
    assert llm.gpt2_generate(model, prompt, steps, on_device=True) == want
    T = len(prompt) + steps - 1
    close(model.peek("k_cache.1")[:T * cfg["dim"]], ref.k_cache[1].ravel()[:T * cfg["dim"]])
    model.close()


@pytest.mark.parametrize("kind", ["q4_0", "q8_0"])
@pytest.mark.parametrize("dim,heads,ffn,plen", [(1024, 16, 2048, 5), (1280, 20, 5120, 5), (1600, 25, 6400, 12)])
def test_gpt2_wide_model_folded_layernorm(oracle, kind, dim, heads, ffn, plen):
    """The widths of GPT-2 medium / large / xl (apps/gpt2/gpt2.lisp:36-48), two layers each: from 1024 features on
    the 4-bit decode GEMVs stage the input per workgroup, with the folded LayerNorm's statistics computed there;
    1280 and 1600 features leave lanes of the row groups without a chunk; the 12-token prompt goes through the
    batched prefill."""
    print(f"case: gpt2 d{dim} {kind} prompt {plen}", flush=True)
    from caten_amd import synth, llm
    cfg = dict(n_layers=2, n_heads=heads, dim=dim, ffn=ffn, vocab=700, max_seq=48, eps=1e-5)
    w = synth.gpt2_weights(cfg, seed=8)
    prompt = synth.prompt(cfg["vocab"], plen, seed=8)
    ref = oracle.GPT2(cfg, _dequantised(oracle, w, synth.GPT2_LINEAR_KEYS + ("lm_head",), kind))
    want_tokens, want_logits = ref.generate(prompt, 8, keep_logits=True)
    model = llm.make_gpt2(cfg, llm.gpt2_state_dict(w, kind))
    got_tokens, got_logits = llm.gpt2_generate(model, prompt, 8, on_device=False, keep_logits=True)
    assert got_tokens == want_tokens
    for g, r in zip(got_logits, want_logits):
        close(g, r)
    model.close()


@pytest.mark.parametrize("arch", ["gpt2", "llama"])
def test_streamed_weights_decode_identical(arch):
    """A session whose kernels request the weights non-temporally (the policy for models past the Infinity Cache,
    forced here on a small one) generates the same tokens and bit-identical logits as the default session."""
    print(f"case: streamed weights {arch}", flush=True)
    from caten_amd import _lib, synth, llm
    lib = _lib.load()
    if arch == "gpt2":
        cfg = synth.GPT2_CONFIGS["gpt2-tiny"]
        sd = llm.gpt2_state_dict(synth.gpt2_weights(cfg, seed=5), "q8_0")
        make, gen = llm.make_gpt2, llm.gpt2_generate
    else:
        cfg = synth.LLAMA_CONFIGS["llama-tiny"]
        sd = llm.llama_state_dict(synth.llama_weights(cfg, seed=5), "q4_0")
        make, gen = llm.make_llama, llm.gpt2_generate  # the loop is the same for both architectures
    prompt = synth.prompt(cfg["vocab"], 6, seed=5)
    runs = []
    try:
        for mode in (0, 1):
            _lib.check(lib.cthip_set_option(b"gemv_stream_weights", mode))
            model = make(cfg, sd)
            runs.append(gen(model, prompt, 10, on_device=False, keep_logits=True))
            model.close()
    finally:
        _lib.check(lib.cthip_set_option(b"gemv_stream_weights", -1))
    assert runs[0][0] == runs[1][0]
    for a, b in zip(runs[0][1], runs[1][1]):
        assert np.array_equal(a, b)


@pytest.mark.parametrize("name,plen,kind", [("gpt2-tiny", 5, "q8_0"), ("gpt2-mini", 40, "q8_0"), ("gpt2-tiny", 5, "f32"),
                                            ("gpt2-mini", 40, "f32"), ("gpt2-tiny", 5, "f16"), ("gpt2-mini", 40, "f16"),
                                            ("gpt2-tiny", 5, "q4_0"), ("gpt2-mini", 40, "q4_0")])
def test_three_launch_layer_equals_five_launch_layer(name, plen, kind):
    """The decode layer as three launches (attention + its projection, and the whole MLP, one launch each, partial
    vectors added up by the consumer) and as five launches (one per Linear) are the same function: identical greedy
    tokens, logits inside the fp32 band, and -- the per-XCD accumulators being integers -- bit-identical logits
    from one run of the three-launch layer to the next."""
    print(f"case: three-launch vs five-launch layer {name} {kind}", flush=True)
    from caten_amd import _lib, synth, llm
    lib = _lib.load()
    cfg = synth.GPT2_CONFIGS[name]
    sd = llm.gpt2_state_dict(synth.gpt2_weights(cfg, seed=11), kind)
    prompt = synth.prompt(cfg["vocab"], plen, seed=11)
    runs = []
    try:
        for mode in (1, 0, 1):
            _lib.check(lib.cthip_set_option(b"decode_fused", mode))
            model = llm.make_gpt2(cfg, sd)
            runs.append(llm.gpt2_generate(model, prompt, 20, on_device=False, keep_logits=True))
            model.close()
    finally:
        _lib.check(lib.cthip_set_option(b"decode_fused", 1))
    assert runs[0][0] == runs[1][0] == runs[2][0]
    for a, b, c in zip(*[r[1] for r in runs]):
        close(a, b)
        assert np.array_equal(a, c)


@pytest.mark.parametrize("kind", ["q4_0", "q8_0", "f16", "f32"])
def test_llama_swiglu_in_the_epilogue_of_the_gate_up_launch(oracle, kind):
    """A model whose gate|up launch holds (gate, up) row pairs applies SwiGLU in that launch's epilogue, and the down
    projection stages one vector instead of two.  8192 rows of gate and up in turn: on the wide-row kernel (option
    gemv_wide 2 sends every launch it supports there) a wavefront streams the two rows together; on the
    register-resident kernels the pair sits in neighbouring lane groups (Q8_0 / Q4_0 at this width) or, with one row
    per wavefront (fp16 / fp32 at this width), in neighbouring slots of the wavefront's ring.  Same tokens as the
    CPU decoder either way; logits inside the fp32 band of it and of each other."""
    print(f"case: SwiGLU in the epilogue of the wide-row gate|up launch, {kind}", flush=True)
    from caten_amd import _lib, synth, llm
    lib = _lib.load()
    cfg = dict(synth.LLAMA_CONFIGS["llama-tiny"], ffn=4096, max_seq=64)
    w = synth.llama_weights(cfg, seed=31)
    sd = llm.llama_state_dict(w, kind)
    prompt = synth.prompt(cfg["vocab"], 9, seed=31)
    runs = []
    try:
        for wide in (2, 1):
            _lib.check(lib.cthip_set_option(b"gemv_wide", wide))
            model = llm.make_llama(cfg, sd)
            runs.append(llm.gpt2_generate(model, prompt, 12, on_device=False, keep_logits=True))
            model.close()
            model = llm.make_llama(cfg, sd)
            assert llm.gpt2_generate(model, prompt, 12, on_device=True) == runs[-1][0]
            model.close()
    finally:
        _lib.check(lib.cthip_set_option(b"gemv_wide", 1))
    assert runs[0][0] == runs[1][0]
    for a, b in zip(runs[0][1], runs[1][1]):
        close(a, b)
    ref = oracle.Llama(cfg, _dequantised(oracle, w, synth.LLAMA_LINEAR_KEYS + ("lm_head",), kind))
    want_tokens, want_logits = ref.generate(prompt, 12, keep_logits=True)
    assert runs[0][0] == want_tokens
    for g, r in zip(runs[0][1], want_logits):
        close(g, r)


@pytest.mark.parametrize("arch,plen,kv", [("gpt2", 40, 0), ("gpt2", 700, 0), ("llama", 40, 0), ("llama", 600, 0), ("gpt2", 40, 1),
                                          ("gpt2", 700, 1)])
def test_three_launch_layer_with_the_attention_as_a_launch_of_its_own(arch, plen, kv):
    """Long contexts of the three-launch layers (option attn_long_from, a position): from there on the attention is a
    launch of its own in which several workgroups share a head's keys, and the projection launch takes its outputs
    instead of repeating the attention in every workgroup of the head -- four launches per layer.  Same greedy tokens
    as three launches throughout (attn_long_from 0) and logits inside the fp32 band (the keys are added in another
    order); two runs bit-identical; the threshold crossed in the middle of a generation (prompt 40, from position 64)
    and far behind it (prompts of 600 / 700); the host-driven loop and the device-resident loop (graphs of one and of
    eight steps, picked per launch by the position the host knows); over fp32 cache rows and, for the GPT-2 shape, over
    Q8_0 rows (kv 1: the attention launch also quantises and appends the step's row)."""
    print(f"case: three-launch layer, attention as its own launch from position 64, {arch} prompt {plen} kv_cache {kv}", flush=True)
    from caten_amd import _lib, synth, llm
    lib = _lib.load()
    if arch == "gpt2":
        cfg = dict(synth.GPT2_CONFIGS["gpt2-mini"], max_seq=1024)
        sd = llm.gpt2_state_dict(synth.gpt2_weights(cfg, seed=29), "q8_0")
        make = llm.make_gpt2
    else:
        cfg = dict(synth.LLAMA_CONFIGS["llama-1.1b"], n_layers=2, max_seq=1024, vocab=2000)
        sd = llm.llama_state_dict(synth.llama_weights(cfg, seed=29), "q4_0")
        make = llm.make_llama
    prompt = synth.prompt(cfg["vocab"], plen, seed=29)
    steps = 72  # (over Q8_0 rows the threshold is half as far again: position 96)
    runs = []
    try:
        _lib.check(lib.cthip_set_option(b"kv_cache", kv))
        for long_from in (64, 0, 64):
            _lib.check(lib.cthip_set_option(b"attn_long_from", long_from))
            model = make(cfg, sd)
            assert lib.cthip_decoder_layer_launches(model.handle) == 3  # (what the session runs at short contexts)
            runs.append(llm.gpt2_generate(model, prompt, steps, on_device=False, keep_logits=True))
            model.close()
            if long_from:
                model = make(cfg, sd)
                assert llm.gpt2_generate(model, prompt, steps, on_device=True) == runs[-1][0]
                model.close()
    finally:
        _lib.check(lib.cthip_set_option(b"attn_long_from", 896))
        _lib.check(lib.cthip_set_option(b"kv_cache", 0))
    assert runs[0][0] == runs[1][0] == runs[2][0]
    for a, b, c in zip(*[r[1] for r in runs]):
        close(a, b)
        assert np.array_equal(a, c)
    # (the other launch sequence did run: where a head's keys are cut into several ranges the low bits differ; a
    # context of one tile is one range, added up in the order of the three-launch layer)
    if plen >= 600:
        assert any(not np.array_equal(a, b) for a, b in zip(runs[0][1][-8:], runs[1][1][-8:]))


@pytest.mark.parametrize("plen", [3, 40])
def test_three_launch_grouped_query_layer_equals_five_launch_layer(plen):
    """The same for RMSNorm / RoPE / grouped-query / SwiGLU layers with Q4_0 weights at the width the three-launch
    layer is built for (d 2048, 32 query / 4 key-value heads, SwiGLU 5632; 2 layers, small vocabulary): both column
    Linears add into per-XCD integer accumulators.  Identical greedy tokens and cache rows inside the fp32 band
    against the five-launch layer, bit-identical logits between two runs."""
    print(f"case: three-launch vs five-launch grouped-query layer, prompt {plen}", flush=True)
    from caten_amd import _lib, synth, llm
    lib = _lib.load()
    cfg = dict(synth.LLAMA_CONFIGS["llama-1.1b"], n_layers=2, max_seq=96, vocab=2000)
    sd = llm.llama_state_dict(synth.llama_weights(cfg, seed=13), "q4_0")
    prompt = synth.prompt(cfg["vocab"], plen, seed=13)
    kd = cfg["dim"] // cfg["n_heads"] * cfg["n_kv_heads"]
    runs, caches = [], []
    try:
        for mode in (1, 0, 1):
            _lib.check(lib.cthip_set_option(b"decode_fused", mode))
            model = llm.make_llama(cfg, sd)
            runs.append(llm.gpt2_generate(model, prompt, 20, on_device=False, keep_logits=True))
            caches.append([model.peek(f"{n}.{l}")[:(plen + 19) * kd] for n in ("k_cache", "v_cache") for l in (0, 1)])
            model.close()
    finally:
        _lib.check(lib.cthip_set_option(b"decode_fused", 1))
    assert runs[0][0] == runs[1][0] == runs[2][0]
    for a, b, c in zip(*[r[1] for r in runs]):
        close(a, b)
        assert np.array_equal(a, c)
    for a, b, c in zip(*caches):
        close(a, b)
        assert np.array_equal(a, c)
    # the device-resident loop (graphs of several steps) gives the host-driven loop's tokens
    model = llm.make_llama(cfg, sd)
    assert llm.gpt2_generate(model, prompt, 20, on_device=True) == runs[0][0]
    model.close()


def test_gpt2_prompt_lengths_and_restart(oracle):
    from caten_amd import synth, llm
    cfg = synth.GPT2_CONFIGS["gpt2-tiny"]
    w = synth.gpt2_weights(cfg, seed=3)
    model = llm.make_gpt2(cfg, llm.gpt2_state_dict(w, "q8_0"))
    wd = _dequantised(oracle, w, synth.GPT2_LINEAR_KEYS + ("lm_head",), "q8_0")
    for plen in (1, 2, 33):
        prompt = synth.prompt(cfg["vocab"], plen, seed=plen)
        ref = oracle.GPT2(cfg, wd)
        want = ref.generate(prompt, 5)
        # a fresh forward at n = 0 restarts the sequence: stale cache rows are overwritten or masked
        assert llm.gpt2_generate(model, prompt, 5, on_device=True) == want
    # fills the cache exactly to max_seq, then refuses to go past it
    prompt = synth.prompt(cfg["vocab"], 4, seed=9)
    ref = oracle.GPT2(cfg, wd)
    n = cfg["max_seq"] - 4 + 1
    assert llm.gpt2_generate(model, prompt, n, on_device=True) == ref.generate(prompt, n)
    from caten_amd import HipError
    with pytest.raises(HipError):
        model.generate_on_device(1)
    with pytest.raises(HipError):
        model.forward([1.0], 1, cfg["max_seq"])
    with pytest.raises(HipError):
        model.forward([], 0, 0)
    model.close()


def test_decoder_state_errors():
    from caten_amd import synth, llm, HipError
    cfg = synth.GPT2_CONFIGS["gpt2-tiny"]
    m = llm.Transformer(cfg, "gpt2")
    with pytest.raises(HipError):
        m.forward([1.0], 1, 0)  # no weights loaded
    with pytest.raises(HipError):
        m.load_state_dict({"no.such.tensor": llm.Tensor.from_f32(np.zeros((1, 4), np.float32))})
    with pytest.raises(HipError):
        m.generate_on_device(1)  # nothing primed
    m.close()


@pytest.mark.parametrize("kind", ["q4_0", "q8_0", "f32"])
def test_llama_generate_matches_oracle(oracle, kind):
    print(f"case: llama decode {kind}", flush=True)
    from caten_amd import synth, llm
    cfg = synth.LLAMA_CONFIGS["llama-tiny"]
    w = synth.llama_weights(cfg, seed=0)
    prompt = synth.prompt(cfg["vocab"], 9, seed=1)
    steps = 10
    ref = oracle.Llama(cfg, _dequantised(oracle, w, synth.LLAMA_LINEAR_KEYS + ("lm_head",), kind))
    want_tokens, want_logits = ref.generate(prompt, steps, keep_logits=True)
    model = llm.make_llama(cfg, llm.llama_state_dict(w, kind))
    got_tokens, got_logits = llm.gpt2_generate(model, prompt, steps, on_device=False, keep_logits=True)
    assert got_tokens == want_tokens
    for g, r in zip(got_logits, want_logits):
        close(g, r)
    # rotated keys and values appended by the decode step's attention launch equal the oracle's cache rows
    kd = cfg["dim"] // cfg["n_heads"] * cfg["n_kv_heads"]
    T = len(prompt) + steps - 1
    for l in (0, cfg["n_layers"] - 1):
        close(model.peek(f"k_cache.{l}")[:T * kd], ref.k_cache[l].ravel()[:T * kd])
        close(model.peek(f"v_cache.{l}")[:T * kd], ref.v_cache[l].ravel()[:T * kd])
    model.close()
    model = llm.make_llama(cfg, llm.llama_state_dict(w, kind))
    assert llm.gpt2_generate(model, prompt, steps, on_device=True) == want_tokens
    # a prompt shorter than the batch threshold goes row by row through the decode step, from position 0
    short = synth.prompt(cfg["vocab"], 3, seed=2)
    ref2 = oracle.Llama(cfg, _dequantised(oracle, w, synth.LLAMA_LINEAR_KEYS + ("lm_head",), kind))
    assert llm.gpt2_generate(model, short, 6, on_device=True) == ref2.generate(short, 6)
    model.close()


def test_prefill_batch_equals_token_by_token(oracle):
    """A prompt pushed through one forward as a batch (MFMA GEMMs) and the same prompt fed row by row
    through the decode step are the same function: identical greedy tokens, logits and cache rows
    within the fp32 band; with bf16 MFMA operands within the 1e-2 band."""
    from caten_amd import synth, llm, _lib
    cfg = synth.GPT2_CONFIGS["gpt2-mini"]
    w = synth.gpt2_weights(cfg, seed=2)
    prompt = synth.prompt(cfg["vocab"], 100, seed=2)
    sd = llm.gpt2_state_dict(w, "q8_0")
    x = [float(t) for t in prompt]
    m1 = llm.make_gpt2(cfg, sd)
    tok1, lg1 = m1.forward(x, len(x), 0, return_logits=True)
    lib = _lib.load()
    _lib.check(lib.cthip_set_option(b"prefill_gemm", 0))
    try:
        m2 = llm.make_gpt2(cfg, sd)
        tok2, lg2 = m2.forward(x, len(x), 0, return_logits=True)
    finally:
        _lib.check(lib.cthip_set_option(b"prefill_gemm", 1))
    assert tok1 == tok2
    close(lg1, lg2)
    close(m1.peek("k_cache.2")[:100 * cfg["dim"]], m2.peek("k_cache.2")[:100 * cfg["dim"]])
    close(m1.peek("v_cache.2")[:100 * cfg["dim"]], m2.peek("v_cache.2")[:100 * cfg["dim"]])
    # continuing from either cache gives the same tokens
    assert m1.generate_on_device(6) == m2.generate_on_device(6)
    # prefill appended to an existing sequence (n > 0)
    more = [float(t) for t in synth.prompt(cfg["vocab"], 9, seed=4)]
    ta, la = m1.forward(more, 9, m1.position, return_logits=True)
    _lib.check(lib.cthip_set_option(b"prefill_gemm", 0))
    try:
        tb, lb = m2.forward(more, 9, m2.position, return_logits=True)
    finally:
        _lib.check(lib.cthip_set_option(b"prefill_gemm", 1))
    assert ta == tb
    close(la, lb)
    m1.close()
    # bf16 MFMA operands
    _lib.check(_lib.load().cthip_set_option(b"gemm_bf16", 1))
    try:
        m3 = llm.make_gpt2(cfg, sd)
        tok3, lg3 = m3.forward(x, len(x), 0, return_logits=True)
    finally:
        _lib.check(_lib.load().cthip_set_option(b"gemm_bf16", 0))
    close(lg3, lg2, 1e-2, 1e-2)
    m2.close()
    m3.close()


def test_gpt2_small_q8_0_full_size_matches_oracle(oracle):
    """The GPT-2-small Q8_0 benchmark configuration at its real size (12 layers, d 768, vocab 50257, Q8_0): a 16-token prompt and
    greedy decode against the CPU oracle on the dequantised weights -- identical tokens, logits inside
    rtol 1e-3 / atol 1e-4.  (The oracle needs ~0.1 s per token, so a handful of steps.)"""
    print("case: gpt2 small q8_0 full size", flush=True)
    from caten_amd import synth, llm
    cfg = synth.GPT2_CONFIGS["gpt2"]
    w = synth.gpt2_weights(cfg, seed=0)
    prompt = synth.prompt(cfg["vocab"], 16, seed=0)
    steps = 6
    ref = oracle.GPT2(cfg, _dequantised(oracle, w, synth.GPT2_LINEAR_KEYS + ("lm_head",), "q8_0"))
    want_tokens, want_logits = ref.generate(prompt, steps, onehot=False, keep_logits=True)
    model = llm.make_gpt2(cfg, llm.gpt2_state_dict(w, "q8_0"))
    got_tokens, got_logits = llm.gpt2_generate(model, prompt, steps, on_device=False, keep_logits=True)
    assert got_tokens == want_tokens
    for g, r in zip(got_logits, want_logits):
        close(g, r)
    assert model.step_bytes(17) == 131252784 + 4 * (12 * (2 * 768 * 2 + 2304 + 768 + 3072 + 768) + 2 * 768) \
        + 2 * 768 * 4 + 2 * 12 * 17 * 768 * 4 + 2 * 12 * 768 * 4
    model.close()
    # size-independent property at the full size: the device-resident loop reproduces the host-driven one
    model = llm.make_gpt2(cfg, llm.gpt2_state_dict(w, "q8_0"))
    long_run = llm.gpt2_generate(model, prompt, 40, on_device=True)
    assert long_run[:steps] == want_tokens
    model2 = llm.make_gpt2(cfg, llm.gpt2_state_dict(w, "q8_0"))
    assert llm.gpt2_generate(model2, prompt, 40, on_device=False) == long_run
    model.close()
    model2.close()


def test_llama_1b_width_q4_0_matches_oracle(oracle):
    """The Llama-1.1B Q4_0 benchmark configuration's layer shape at its real width (d 2048, 32 query / 4 KV heads, SwiGLU 5632, vocab 32000,
    Q4_0) with 2 of the 22 layers so the CPU oracle finishes in seconds: a 12-token prompt (batched prefill)
    and greedy decode -- identical tokens, logits inside rtol 1e-3 / atol 1e-4, cache rows equal."""
    print("case: llama 1.1b width q4_0, 2 layers", flush=True)
    from caten_amd import synth, llm
    cfg = dict(synth.LLAMA_CONFIGS["llama-1.1b"], n_layers=2, max_seq=64)
    w = synth.llama_weights(cfg, seed=2)
    prompt = synth.prompt(cfg["vocab"], 12, seed=2)
    steps = 5
    ref = oracle.Llama(cfg, _dequantised(oracle, w, synth.LLAMA_LINEAR_KEYS + ("lm_head",), "q4_0"))
    want_tokens, want_logits = ref.generate(prompt, steps, keep_logits=True)
    model = llm.make_llama(cfg, llm.llama_state_dict(w, "q4_0"))
    got_tokens, got_logits = llm.gpt2_generate(model, prompt, steps, on_device=False, keep_logits=True)
    assert got_tokens == want_tokens
    for g, r in zip(got_logits, want_logits):
        close(g, r)
    kd = cfg["dim"] // cfg["n_heads"] * cfg["n_kv_heads"]
    T = len(prompt) + steps - 1
    close(model.peek("k_cache.1")[:T * kd], ref.k_cache[1].ravel()[:T * kd])
    model.close()


@pytest.mark.parametrize("name", ["gpt2-tiny", "gpt2-mini"])
def test_generate_until_stops_on_the_device(name):
    """The device-resident loop with a stop condition: the step that produces the end token is the last one that
    changes anything (token, position, history), however many steps were already queued behind it; what comes out
    is the unconditional loop's sequence cut after that token, and generation can go on from there."""
    print(f"case: generate_until {name}", flush=True)
    from caten_amd import synth, llm, HipError
    cfg = synth.GPT2_CONFIGS[name]
    sd = llm.gpt2_state_dict(synth.gpt2_weights(cfg, seed=4), "q8_0")
    prompt = synth.prompt(cfg["vocab"], 9, seed=4)
    model = llm.make_gpt2(cfg, sd)
    first = model.forward([float(t) for t in prompt], len(prompt), 0)
    free = model.generate_on_device(40)
    model.close()
    # an end token that first appears somewhere in the middle (and one that appears at the very first step)
    for k in (0, 5, 17, 30):
        eos = free[k]
        k = free.index(eos)
        model = llm.make_gpt2(cfg, sd)
        assert model.forward([float(t) for t in prompt], len(prompt), 0) == first
        got = model.generate_until(40, eos)
        assert got == free[:k + 1]
        assert model.position == len(prompt) + k + 1
        # the loop state is where the end token left it: going on reproduces the unconditional sequence
        assert model.generate_on_device(3) == free[k + 1:k + 4]
        model.close()
    # a token that never comes: all max_steps tokens
    model = llm.make_gpt2(cfg, sd)
    model.forward([float(t) for t in prompt], len(prompt), 0)
    never = next(t for t in range(cfg["vocab"]) if t not in free)
    assert model.generate_until(40, never) == free
    with pytest.raises(HipError):
        model.generate_until(5, cfg["vocab"])
    model.close()


@pytest.mark.parametrize("kv", [0, 1, 2])
@pytest.mark.parametrize("arch,heads,kv_heads,dim,plen", [("llama", 8, 2, 512, 700), ("llama", 4, 4, 512, 1300), ("gpt2", 4, 4, 256, 900),
                                                          ("llama", 8, 8, 256, 130)])
def test_decode_attention_with_the_keys_of_a_head_shared_by_workgroups(arch, heads, kv_heads, dim, plen, kv):
    """One launch per Linear, long contexts: the decode attention cuts a head's keys into ranges of whole tiles, one
    workgroup each, and the workgroup that draws the last ticket adds the ranges up (option attn_split, on by
    default).  Same tokens as one workgroup per head, logits inside the fp32 band (the sums are taken in another
    order), two runs bit-identical (the ranges are added in a fixed order whichever workgroup finishes last);
    head_dim 64, 128 and 32, grouped-query and plain heads, with the rotation and the append inside the launch and
    without, contexts of one range and of many; over fp32 cache rows (kv 0) and over Q8_0 rows (kv 1: the launch
    also quantises the new row, and the planes of layer 0 have the same bits either way) and over fp32 pages (kv 2: the
    launch also rotates the new row and stores it into its page)."""
    print(f"case: split decode attention {arch} heads {heads}/{kv_heads} dim {dim} prompt {plen} kv_cache {kv}", flush=True)
    from caten_amd import _lib, synth, llm
    lib = _lib.load()
    if arch == "gpt2":
        cfg = dict(synth.GPT2_CONFIGS["gpt2-tiny"], n_heads=heads, dim=dim, ffn=4 * dim, max_seq=1536)
        sd = llm.gpt2_state_dict(synth.gpt2_weights(cfg, seed=17), "q8_0")
        make = llm.make_gpt2
    else:
        cfg = dict(synth.LLAMA_CONFIGS["llama-tiny"], n_heads=heads, n_kv_heads=kv_heads, dim=dim, ffn=2 * dim, max_seq=1536)
        sd = llm.llama_state_dict(synth.llama_weights(cfg, seed=17), "q8_0")
        make = llm.make_llama
    prompt = synth.prompt(cfg["vocab"], plen, seed=17)
    runs, planes = [], []
    try:
        _lib.check(lib.cthip_set_option(b"decode_fused", 0))
        _lib.check(lib.cthip_set_option(b"kv_cache", kv))
        for split in (1, 0, 1, 3):  # (3: exactly three key ranges per head)
            _lib.check(lib.cthip_set_option(b"attn_split", split))
            model = make(cfg, sd)
            runs.append(llm.gpt2_generate(model, prompt, 24, on_device=False, keep_logits=True))
            if kv == 1:
                planes.append(tuple(model.peek(n).view(np.uint8).copy() for n in ("k_cache_q8.0", "k_cache_d.0", "v_cache_q8.0", "v_cache_d.0")))
            if split == 1:
                m2 = make(cfg, sd)
                assert llm.gpt2_generate(m2, prompt, 24, on_device=True) == runs[-1][0]  # inside the step graphs too
                m2.close()
            model.close()
    finally:
        _lib.check(lib.cthip_set_option(b"decode_fused", 1))
        _lib.check(lib.cthip_set_option(b"attn_split", 1))
        _lib.check(lib.cthip_set_option(b"kv_cache", 0))
    assert runs[0][0] == runs[1][0] == runs[2][0] == runs[3][0]
    for a, b, c, d in zip(*[r[1] for r in runs]):
        close(a, b)
        close(a, d)
        assert np.array_equal(a, c)
    for x, y in zip(planes[:1] * 3, planes[1:]):
        assert all(np.array_equal(p, q) for p, q in zip(x, y))
