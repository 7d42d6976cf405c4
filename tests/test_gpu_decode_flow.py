"""All layers of a decode step as ONE launch of role-specialised workgroups that hand their results over through
tagged device memory (option "decode_flow", csrc/decode_flow.hip) against the three-launch layer: the same function of
one GPT-2 block (external/llm/layers.lisp:35-71).  Bars: identical greedy tokens, logits inside the fp32 band
(rtol 1e-4 / atol 1e-4: the two paths add the same products in another order), bit-identical logits from one run to
the next (every sum has a fixed order), the device-resident loop equal to the host loop, and an in-kernel timeline
whose stamps are ordered the way the data flows."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _runs(name, plen, steps, modes):
    from caten_amd import _lib, synth, llm
    lib = _lib.init()
    cfg = synth.GPT2_CONFIGS[name]
    sd = llm.gpt2_state_dict(synth.gpt2_weights(cfg, seed=11), "q8_0")
    prompt = synth.prompt(cfg["vocab"], plen, seed=11)
    out = []
    try:
        for mode in modes:
            _lib.check(lib.cthip_set_option(b"decode_flow", mode))
            m = llm.make_gpt2(cfg, sd)
            launches = lib.cthip_decoder_layer_launches(m.handle)
            toks, logs = llm.gpt2_generate(m, prompt, steps, on_device=False, keep_logits=True)
            m.close()
            m = llm.make_gpt2(cfg, sd)
            dev = llm.gpt2_generate(m, prompt, steps, on_device=True)
            m.close()
            out.append((launches, toks, logs, dev))
    finally:
        _lib.check(lib.cthip_set_option(b"decode_flow", 0))
    return out


@pytest.mark.parametrize("name,plen", [("gpt2-tiny", 5), ("gpt2-mini", 40), ("gpt2-mini", 3)])
def test_one_launch_step_equals_three_launch_layer(name, plen):
    print(f"case: one-launch decode step {name} prompt {plen}", flush=True)
    (n0, t0, l0, d0), (n1, t1, l1, d1), (n2, t2, l2, d2) = _runs(name, plen, 20, (0, 1, 1))
    assert (n0, n1, n2) == (3, 1, 1)
    assert t0 == t1 == t2 == d0 == d1 == d2
    for a, b, c in zip(l0, l1, l2):
        assert np.allclose(b, a, rtol=1e-4, atol=1e-4), float(np.max(np.abs(a - b)))
        assert np.array_equal(b, c)


def test_one_launch_step_is_refused_where_it_has_no_kernel():
    """other widths, weight formats and the Q8_0 cache keep the three launches per layer"""
    from caten_amd import _lib, synth, llm
    lib = _lib.init()
    cfg = synth.GPT2_CONFIGS["gpt2-tiny"]
    try:
        _lib.check(lib.cthip_set_option(b"decode_flow", 1))
        m = llm.make_gpt2(cfg, llm.gpt2_state_dict(synth.gpt2_weights(cfg, seed=1), "f16"))
        assert lib.cthip_decoder_layer_launches(m.handle) == 3
        m.close()
        _lib.check(lib.cthip_set_option(b"kv_cache", 1))
        m = llm.make_gpt2(cfg, llm.gpt2_state_dict(synth.gpt2_weights(cfg, seed=1), "q8_0"))
        assert lib.cthip_decoder_layer_launches(m.handle) == 3  # the three-launch layer over Q8_0 rows, not the one launch
        m.close()
        assert lib.cthip_set_option(b"decode_flow", 3) != 0
    finally:
        _lib.check(lib.cthip_set_option(b"kv_cache", 0))
        _lib.check(lib.cthip_set_option(b"decode_flow", 0))


def test_timeline_of_a_traced_step():
    """option value 2 keeps four clock stamps per workgroup and layer (100 MHz): start of the wait, input complete,
    middle, output stored.  Printed per layer for GPT-2 small; the order of the stamps is what is asserted."""
    print("case: one-launch decode step, timeline, gpt2", flush=True)
    from caten_amd import _lib, synth, llm
    lib = _lib.init()
    cfg = synth.GPT2_CONFIGS["gpt2"]
    sd = llm.gpt2_state_dict(synth.gpt2_weights(cfg, seed=11), "q8_0")
    prompt = synth.prompt(cfg["vocab"], 16, seed=11)
    try:
        _lib.check(lib.cthip_set_option(b"decode_flow", 2))
        m = llm.make_gpt2(cfg, sd)
        llm.gpt2_generate(m, prompt, 40, on_device=True)
        tr = m.peek("flow_trace").view(np.int64)
        m.close()
    finally:
        _lib.check(lib.cthip_set_option(b"decode_flow", 0))
    D, H, F, NL = cfg["dim"], cfg["n_heads"], cfg["ffn"], cfg["n_layers"]
    counts = [("Q", 3 * D // 32), ("A", H), ("P", D // 32), ("M", F // 32), ("R", 32)]
    tr = tr.reshape(sum(n for _, n in counts), NL, 4).astype(np.float64)
    tr = (tr - tr[:, 0, 0].min()) / 100.0  # microseconds
    roles, at = {}, 0
    for k, n in counts:
        roles[k] = tr[at:at + n]
        at += n
    print("layer role: input complete (first..last workgroup) | middle (last) | output stored (first..last)  [us]")
    for layer in range(NL):
        for k, v in roles.items():
            mid = "   -   " if k == "R" else f"{v[:, layer, 2].max():7.2f}"
            print(f"{layer:2d} {k}: {v[:, layer, 1].min():7.2f}..{v[:, layer, 1].max():7.2f} | {mid} | "
                  f"{v[:, layer, 3].min():7.2f}..{v[:, layer, 3].max():7.2f}")
    done = roles["R"][:, :, 3].max(axis=0)
    print("per layer:", np.round(np.diff(done), 2), "us; all layers:", round(float(done[-1]), 1), "us", flush=True)
    order = ["Q", "A", "P", "M", "R"]
    for layer in range(NL):
        for k in order:
            assert (roles[k][:, layer, 3] > roles[k][:, layer, 1]).all()
        for up, down in zip(order, order[1:]):  # a role's input needs every workgroup of the role before it
            assert roles[down][:, layer, 1].min() > roles[up][:, layer, 1].max(), (layer, up, down)
        if layer:
            assert roles["Q"][:, layer, 1].min() > roles["R"][:, layer - 1, 1].max()
    assert 3.0 < float(np.diff(done).mean()) < 60.0
