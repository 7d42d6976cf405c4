"""GGUF reader (C++ in libcaten_hip.so) -- host-side tests need no GPU; the decoder-load test does.

The reference tests its reader by writing arange(64) as f32/f16/q8_0 with the Python `gguf` package
and comparing dequantised values (external/test-gguf.lisp:3-75).  That package is absent here, so the
files are written by caten_amd.gguf.write_gguf (GGUF v3 per the layout external/gguf/gguf-file.lisp
parses) and the values are checked with the pinned oracle codecs."""
import os
import struct

import numpy as np
import pytest


@pytest.fixture()
def tmp_gguf(tmp_path):
    return str(tmp_path / "dummy.gguf")


@pytest.mark.parametrize("kind", ["f32", "f16", "q8_0", "q4_0"])
def test_dummy_gguf_arange64(oracle, tmp_gguf, kind):
    from caten_amd import gguf
    from caten_amd.llm import Tensor
    data = np.arange(64, dtype=np.float32)
    t = Tensor.from_f32(data, kind)
    gguf.write_gguf(tmp_gguf, {"general.architecture": "test_arch"}, [("tensor", kind, (64,), t.raw)])
    g = gguf.GGUF(tmp_gguf)
    assert g.version == 3 and len(g.tensor_info) == 1 and g.metadata_get("general.architecture") == "test_arch"
    info = g.tensor_info[0]
    assert info.name == "tensor" and info.kind == kind and info.shape == (64,) and info.abs_offset % 32 == 0
    raw = g.tensor_bytes("tensor")
    got = oracle.dequant(kind, raw, 64)
    if kind in ("f32", "f16"):
        assert np.array_equal(got, data)
    else:
        step = {"q8_0": 63 / 127, "q4_0": 63 / 8}[kind]
        assert np.all(np.abs(got - data) <= step * 0.51 + 1e-3)
    g.close()


def test_reader_layout_metadata_and_alignment(tmp_gguf):
    from caten_amd import gguf
    rng = np.random.default_rng(0)
    a = rng.normal(size=(3, 32)).astype(np.float32)
    b = rng.normal(size=(5,)).astype(np.float32)
    c = rng.normal(size=(2, 4, 8)).astype(np.float32)
    meta = {"general.architecture": "gpt2", "gpt2.block_count": 12, "gpt2.attention.layer_norm_epsilon": 1e-5,
            "flag": True, "big": -5, "tokenizer.ggml.tokens": ["!", "\"", "Ġthe", "日本"]}
    for align in (32, 64, 256):
        gguf.write_gguf(tmp_gguf, meta, [("a", "f32", a.shape, a), ("b", "f32", b.shape, b), ("c", "f32", c.shape, c)], align)
        g = gguf.GGUF(tmp_gguf)
        assert g.alignment == align and g.metadata_kv_count == len(meta) + 1
        assert g.metadata_get("gpt2.block_count") == 12 and g.metadata_get("flag") is True and g.metadata_get("big") == -5
        assert abs(g.metadata_get("gpt2.attention.layer_norm_epsilon") - 1e-5) < 1e-12
        assert g.metadata_get("tokenizer.ggml.tokens") == ["!", "\"", "Ġthe", "日本"]
        assert g.metadata_get("missing") is None
        for name, arr in (("a", a), ("b", b), ("c", c)):
            assert np.array_equal(g.tensor_bytes(name).view(np.float32).reshape(arr.shape), arr)
        infos = {t.name: t for t in g.tensor_info}
        assert infos["c"].dims == [8, 4, 2] and infos["c"].shape == (2, 4, 8)  # stored innermost first
        assert all(t.abs_offset % align == 0 for t in g.tensor_info)
        with pytest.raises(KeyError):
            g.tensor_bytes("nope")
        g.close()


def test_reader_rejects_malformed_files(tmp_gguf, tmp_path):
    from caten_amd import gguf, HipError
    with pytest.raises(HipError):
        gguf.GGUF(str(tmp_path / "does_not_exist.gguf"))
    open(tmp_gguf, "wb").write(b"GGML" + b"\0" * 64)
    with pytest.raises(HipError) as e:
        gguf.GGUF(tmp_gguf)
    assert "GGUF" in str(e.value)
    open(tmp_gguf, "wb").write(b"GGUF" + struct.pack("<IQQ", 1, 0, 0) + b"\0" * 32)
    with pytest.raises(HipError):
        gguf.GGUF(tmp_gguf)  # version 1
    a = np.zeros((4, 32), np.float32)
    gguf.write_gguf(tmp_gguf, {"k": "v"}, [("a", "f32", a.shape, a)])
    blob = open(tmp_gguf, "rb").read()
    open(tmp_gguf, "wb").write(blob[:-100])
    with pytest.raises(HipError) as e:
        gguf.GGUF(tmp_gguf)  # tensor data truncated
    assert "past the end" in str(e.value)
    open(tmp_gguf, "wb").write(blob[:40])
    with pytest.raises(HipError):
        gguf.GGUF(tmp_gguf)  # metadata truncated
    def one_tensor(dims, ggml_type, offset):
        name = b"t"
        info = struct.pack("<Q", len(name)) + name + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        return b"GGUF" + struct.pack("<IQQ", 3, 1, 0) + info + struct.pack("<IQ", ggml_type, offset) + b"\0" * 64
    for dims, off in [((1 << 62, 8), 0), ((1 << 63,), 0), ((1 << 40,), 0), ((8,), (1 << 64) - 16), ((8,), 1 << 20)]:
        open(tmp_gguf, "wb").write(one_tensor(dims, 0, off))
        with pytest.raises(HipError):
            gguf.GGUF(tmp_gguf)  # element counts / offsets that overflow or leave the file
    open(tmp_gguf, "wb").write(one_tensor((8,), 0, 0))
    g = gguf.GGUF(tmp_gguf)
    assert g.tensor_info[0].shape == (8,)
    g.close()
    open(tmp_gguf, "wb").write(b"GGUF" + struct.pack("<IQQ", 3, 0, 0))
    g = gguf.GGUF(tmp_gguf)  # empty but valid
    assert len(g.tensor_info) == 0 and g.metadata_kv_count == 0


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["q8_0", "f32"])
def test_decoder_from_gguf_file(oracle, tmp_gguf, kind):
    """make-gpt2's path: GGUF file -> remapped state dict -> Transformer -> greedy tokens."""
    from caten_amd import gguf, llm, synth
    from tests.test_gpu_decoder import _dequantised
    cfg = synth.GPT2_CONFIGS["gpt2-tiny"]
    w = synth.gpt2_weights(cfg, seed=7)
    gguf.write_gguf(tmp_gguf, {"general.architecture": "gpt2", "gpt2.block_count": cfg["n_layers"]},
                    gguf.gpt2_gguf_tensors(w, kind))
    g = gguf.GGUF(tmp_gguf)
    model = llm.Transformer(cfg, "gpt2")
    assert g.load_into(model) == 5 + 12 * cfg["n_layers"]
    prompt = synth.prompt(cfg["vocab"], 9, seed=7)
    got = llm.gpt2_generate(model, prompt, 8, on_device=True)
    ref = oracle.GPT2(cfg, _dequantised(oracle, w, synth.GPT2_LINEAR_KEYS + ("lm_head",), kind))
    assert got == ref.generate(prompt, 8)
    # the file's Q8_0 bytes dequantise on the device to the reference's values, bit for bit
    from caten_amd import ops
    raw = g.tensor_bytes("blk.0.ffn_up.weight")
    n = cfg["ffn"] * cfg["dim"]
    assert np.array_equal(ops.dequantize(kind, raw, n).view(np.uint32), oracle.dequant(kind, raw, n).view(np.uint32))
    model.close()
    g.close()
    # a file that lacks tensors of the model is refused
    gguf.write_gguf(tmp_gguf, {}, gguf.gpt2_gguf_tensors(w, kind)[:10])
    g = gguf.GGUF(tmp_gguf)
    with pytest.raises(llm._lib.HipError):
        g.load_into(llm.Transformer(cfg, "gpt2"))
