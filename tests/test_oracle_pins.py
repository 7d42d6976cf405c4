"""Pins the CPU oracle before anything is compared against it.

Every check here is independent of the oracle's own formulas: PyTorch library
routines at the tolerances the reference's test-suite uses, the literal golden
values held in the reference's tests (tests/golden/reference_literals.json),
NumPy's IEEE half conversion, and closed forms.
"""
import json
import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_literals.json")))


def close(a, b, atol, rtol):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return np.all(np.abs(a - b) <= atol + rtol * np.abs(b))


# ------------------------------------------------------------ codecs (Q1/Q2/Q3)
def test_f16_decode_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    got = oracle.f16_to_f32(bits)
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f16_encode_roundtrip_and_rounding(oracle):
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.normal(0, 1, 4000), rng.normal(0, 1e-5, 2000), rng.normal(0, 3e4, 2000),
                        [0.0, -0.0, 65504.0, 65519.0, 1e-8, 5.96e-8, 2.98e-8, 2.9802322387695312e-08]]).astype(np.float32)
    got = oracle.f32_to_f16_bits(x)
    want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)


def test_q8_0_dequant_exhaustive_scale_times_q(oracle):
    # every fp16 scale x every int8 value: out must be the exact single-float product
    scales = np.arange(65536, dtype=np.uint16)
    scales = scales[np.isfinite(scales.view(np.float16))]
    rng = np.random.default_rng(1)
    nb = scales.size * 8
    q = np.tile(np.arange(-128, 128, dtype=np.int8), nb * 32 // 256)
    sc = np.repeat(scales, 8)
    raw = np.empty((nb, 34), np.uint8)
    raw[:, 0:2] = sc.view(np.uint8).reshape(-1, 2)
    raw[:, 2:] = q.view(np.uint8).reshape(nb, 32)
    got = oracle.dequant("q8_0", raw, nb * 32).reshape(nb, 32)
    want = sc.view(np.float16).astype(np.float32)[:, None] * q.reshape(nb, 32).astype(np.float32)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_q8_0_reference_fixture_arange64(oracle):
    # The reference's own dequant test quantises arange(64) with ggml's quantiser and
    # compares at atol 1e-5 (external/test-gguf.lisp:3-59).  Restated with closed forms:
    # scale = fp16(absmax/127), q = round(x/d) -> |deq - x| <= d/2 and deq = q*d exactly.
    x = np.arange(64, dtype=np.float32)
    raw = oracle.quantize("q8_0", x)
    assert raw.size == 68
    d0 = raw[0:2].view(np.float16)[0]
    d1 = raw[34:36].view(np.float16)[0]
    assert d0 == np.float16(31 / 127) and d1 == np.float16(63 / 127)
    deq = oracle.dequant("q8_0", raw, 64)
    # q is chosen with the single-float d, the value is rebuilt with the fp16-rounded d
    assert np.all(np.abs(deq[:32] - x[:32]) <= float(d0) / 2 + 127 * abs(float(d0) - 31 / 127) + 1e-6)
    assert np.all(np.abs(deq[32:] - x[32:]) <= float(d1) / 2 + 127 * abs(float(d1) - 63 / 127) + 1e-6)
    assert np.all(np.abs(deq - x) <= 1e-5 + 0.5)  # and nowhere near a whole step off
    assert deq[31] == np.float32(127) * np.float32(d0) and deq[63] == np.float32(127) * np.float32(d1)
    # short last block (dequantize.lisp:48: elements-in-block = min 32 (size - idx))
    deq_short = oracle.dequant("q8_0", raw, 40)
    assert np.array_equal(deq_short, deq[:40])


def test_f16_f32_dequant_arange64(oracle):
    x = np.arange(64, dtype=np.float32)
    assert np.array_equal(oracle.dequant("f16", x.astype(np.float16).view(np.uint8), 64), x)
    assert np.array_equal(oracle.dequant("f32", x.view(np.uint8), 64), x)


def test_q4_0_layout_closed_form(oracle):
    # ggml block_q4_0: d then 16 bytes; low nibbles are elements 0..15, high nibbles 16..31
    raw = np.zeros(18, np.uint8)
    raw[0:2] = np.array([np.float16(0.5)]).view(np.uint8)
    raw[2:] = np.arange(16, dtype=np.uint8) | ((15 - np.arange(16, dtype=np.uint8)) << 4)
    deq = oracle.dequant("q4_0", raw, 32)
    want = np.concatenate([(np.arange(16) - 8) * 0.5, ((15 - np.arange(16)) - 8) * 0.5]).astype(np.float32)
    assert np.array_equal(deq, want)
    # exhaustive nibble x a sweep of scales
    sc = np.array([1.0, -1.0, 0.1, 6.1e-5, 5.96e-8, 1024.0], dtype=np.float16)
    for s in sc:
        raw[0:2] = np.array([s]).view(np.uint8)
        raw[2:] = np.arange(16, dtype=np.uint8) * 17
        deq = oracle.dequant("q4_0", raw, 32)
        want = np.tile((np.arange(16) - 8).astype(np.float32) * np.float32(s), 2)
        assert np.array_equal(deq, want)


def test_q4_0_quantiser_roundtrip_bound(oracle):
    rng = np.random.default_rng(2)
    w = rng.normal(0, 0.02, 32 * 64).astype(np.float32)
    raw = oracle.quantize("q4_0", w)
    deq = oracle.dequant("q4_0", raw, w.size)
    d = np.abs(raw.reshape(-1, 18)[:, :2].copy().view(np.float16).astype(np.float32))
    err = np.abs(deq - w).reshape(-1, 32)
    assert np.all(err <= d * 1.01 + 1e-7)  # one step (the +8 end is clamped to 15)
    # the extreme element maps to nibble 0, i.e. -8*d
    am = np.argmax(np.abs(w.reshape(-1, 32)), axis=1)
    assert np.allclose(deq.reshape(-1, 32)[np.arange(64), am], w.reshape(-1, 32)[np.arange(64), am], rtol=2e-3)


# ------------------------------------------------------------ golden literals
def test_embedding_golden(oracle):
    W = (0.1 * np.arange(100, dtype=np.float32)).reshape(10, 10)  # linspace (10 10) 0.1 0.0
    for idx, key in ((1.0, "embedding_row_idx1"), (2.0, "embedding_row_idx2")):
        out = oracle.embedding_onehot(W, np.full((2, 10), idx, np.float32))
        want = np.tile(np.array(GOLD[key], np.float32), (2, 10, 1))
        assert np.all(np.abs(out - want) <= GOLD["embedding_tol"])
    rng = np.random.default_rng(3)
    W = rng.normal(size=(37, 12)).astype(np.float32)
    idx = rng.integers(0, 37, size=(3, 5))
    assert np.array_equal(oracle.embedding_onehot(W, idx.astype(np.float32)), W[idx])


def test_argmax_golden_and_ties(oracle):
    x = np.arange(10, dtype=np.float32)  # linspace (1 10) 1 0
    assert oracle.argmax(x) == GOLD["argmax_linspace_1_10"]
    rng = np.random.default_rng(4)
    for _ in range(50):
        x = rng.integers(0, 4, size=rng.integers(1, 40)).astype(np.float32)  # many ties
        assert oracle.argmax(x) == int(np.argmax(x)) == int(torch.argmax(torch.from_numpy(x)))
    x = rng.normal(size=50257).astype(np.float32)
    assert oracle.argmax(x) == int(np.argmax(x))


def test_tri_golden(oracle):
    ones = np.ones((10, 10), np.float32)
    assert np.array_equal(oracle.tril(ones), np.tril(ones))
    assert np.array_equal(oracle.triu(ones), np.triu(ones))
    assert np.array_equal(oracle.triu(np.ones((5, 5, 5), np.float32)), np.triu(np.ones((5, 5, 5), np.float32)))
    # the causal mask of Transformer (layers.lisp:83) against the reference test's torch spelling
    # (test-llm.lisp:159,209): triu(full(-inf), diagonal=1+n)
    for s, n in ((1, 0), (1, 7), (5, 0), (4, 3)):
        want = torch.triu(torch.full((s, n + s), float("-inf")), diagonal=1 + n).numpy()
        assert np.array_equal(oracle.triu_neginf(s, n + s, 1 + n), want)


def test_squared_gemm_golden(oracle):
    for ans, x, y, n in GOLD["squared_gemm"]:
        out = oracle.matmul(np.full((n, n), x, np.float32), np.full((n, n), y, np.float32))
        assert np.all(out == ans)


# ------------------------------------------------------------ library routines
def test_matmul_vs_torch(oracle):
    rng = np.random.default_rng(5)
    for (m, k, n) in ((3, 64, 5), (64, 64, 64), (17, 33, 9), (128, 96, 32)):
        A = rng.uniform(-1, 1, (m, k)).astype(np.float32)
        B = rng.uniform(-1, 1, (k, n)).astype(np.float32)
        want = torch.matmul(torch.from_numpy(A).double(), torch.from_numpy(B).double()).numpy()
        assert close(oracle.matmul(A, B), want, 1e-5, 1e-5)  # test-gemm.lisp:3-22
        assert np.array_equal(oracle.matmul(A, B, relu=True), np.maximum(oracle.matmul(A, B), 0))
    # a transposed operand would fail this: non-square, asymmetric
    A = np.arange(6, dtype=np.float32).reshape(2, 3)
    B = np.arange(12, dtype=np.float32).reshape(3, 4)
    assert np.array_equal(oracle.matmul(A, B), A @ B)


def test_linear_vs_torch(oracle):
    rng = np.random.default_rng(6)
    x = rng.normal(size=(2, 7, 48)).astype(np.float32)
    W = rng.normal(size=(20, 48)).astype(np.float32)
    b = rng.normal(size=20).astype(np.float32)
    want = F.linear(torch.from_numpy(x).double(), torch.from_numpy(W).double(), torch.from_numpy(b).double()).numpy()
    assert close(oracle.linear(x, W, b), want, 1e-5, 1e-5)
    want = F.linear(torch.from_numpy(x).double(), torch.from_numpy(W).double()).numpy()
    assert close(oracle.linear(x, W), want, 1e-5, 1e-5)


def test_softmax_vs_torch(oracle):
    rng = np.random.default_rng(7)
    x = rng.normal(size=(128, 128)).astype(np.float32)
    assert close(oracle.softmax(x), F.softmax(torch.from_numpy(x), -1).numpy(), 1e-5, 1e-6)  # test-llm.lisp:64-80
    x = rng.normal(10, 100, size=(512, 512)).astype(np.float32)
    y = oracle.softmax(x)
    assert close(y, F.softmax(torch.from_numpy(x).double(), -1).numpy(), 1e-5, 1e-5)  # test-activations.lisp:60-73
    assert np.allclose(y.sum(-1), 1.0, atol=1e-5)
    assert np.allclose(oracle.softmax(x + 3.0), y, atol=1e-5)


def test_layernorm_rmsnorm_vs_torch(oracle):
    rng = np.random.default_rng(8)
    x = rng.normal(size=(30, 40)).astype(np.float32)
    want = F.layer_norm(torch.from_numpy(x), (40,), eps=1e-5).numpy()
    assert close(oracle.layernorm(x), want, 1e-5, 1e-2)  # test-normalization.lisp:18-33
    g = rng.normal(1, 0.02, 40).astype(np.float32)
    b = rng.normal(0, 0.02, 40).astype(np.float32)
    want = F.layer_norm(torch.from_numpy(x).double(), (40,), torch.from_numpy(g).double(), torch.from_numpy(b).double(), 1e-5).numpy()
    assert close(oracle.layernorm(x, g, b), want, 2e-6, 1e-5)
    # an unbiased variance (N-1) would fail this
    x2 = np.array([[1.0, 2.0, 3.0, 6.0]], np.float32)
    var = ((x2 - 3.0) ** 2).mean()
    assert np.allclose(oracle.layernorm(x2, eps=0.0), (x2 - 3.0) / math.sqrt(var), atol=1e-6)
    # RMSNorm, torchtune formula (test-normalization.lisp:7-16,57-63)
    w = rng.normal(1, 0.02, 40).astype(np.float32)
    xt = torch.from_numpy(x).double()
    want = (xt * torch.rsqrt(xt.pow(2).mean(-1, keepdim=True) + 1e-5) * torch.from_numpy(w).double()).numpy()
    assert close(oracle.rmsnorm(x, w), want, 1e-5, 1e-6)


def test_activations_vs_torch(oracle):
    x = np.linspace(-8, 8, 4001).astype(np.float32)
    xt = torch.from_numpy(x).double()
    assert close(oracle.gelu_tanh(x), F.gelu(xt, approximate="tanh").numpy(), 1e-6, 1e-6)
    assert close(oracle.silu(x), F.silu(xt).numpy(), 1e-6, 1e-6)
    assert close(oracle.sigmoid(x), torch.sigmoid(xt).numpy(), 1e-6, 1e-6)
    assert close(oracle.tanh(x), torch.tanh(xt).numpy(), 1e-6, 1e-6)
    assert np.array_equal(oracle.relu(x), np.maximum(x, 0))


def _torch_rope(x, base=10000.0, start=0):
    # torchtune interleaved formula, as spelled in the reference's test (test-rope.lisp:38-56)
    dim = x.shape[-1]
    theta = 1.0 / (base ** (torch.arange(0, dim, 2).double() / dim))
    seq_len = x.size(1)
    seq_idx = torch.arange(start, start + seq_len).double()
    idx_theta = torch.einsum("i,j->ij", seq_idx, theta)
    cache = torch.stack([torch.cos(idx_theta), torch.sin(idx_theta)], dim=-1)
    xs = x.double().reshape(*x.shape[:-1], -1, 2)
    rc = cache.view(1, seq_len, 1, xs.size(-2), 2)
    out = torch.stack([xs[..., 0] * rc[..., 0] - xs[..., 1] * rc[..., 1],
                       xs[..., 1] * rc[..., 0] + xs[..., 0] * rc[..., 1]], dim=-1)
    return out.flatten(-2)


def test_rope_vs_torchtune(oracle):
    torch.manual_seed(0)
    x = torch.rand(1, 10, 10, 10)
    assert close(oracle.rope(x.numpy()), _torch_rope(x).numpy(), 1e-5, 5e-4)  # test-rope.lisp:58-66
    x = torch.randn(2, 6, 4, 64)
    assert close(oracle.rope(x.numpy(), start_pos=37), _torch_rope(x, start=37).numpy(), 2e-5, 5e-4)
    # rotating position p alone equals row p of a full rotation
    full = oracle.rope(x.numpy()[:, :, :, :], start_pos=0)
    one = oracle.rope(x.numpy()[:, 3:4], start_pos=3)
    assert np.array_equal(one, full[:, 3:4])


def test_sdpa_vs_torch(oracle):
    rng = np.random.default_rng(9)
    S, T, H, Dh = 5, 9, 4, 16
    q = rng.normal(size=(S, H, Dh)).astype(np.float32)
    k = rng.normal(size=(T, H, Dh)).astype(np.float32)
    v = rng.normal(size=(T, H, Dh)).astype(np.float32)
    mask = oracle.triu_neginf(S, T, 1 + (T - S))
    qt, kt, vt = (torch.from_numpy(a).double().transpose(0, 1) for a in (q, k, v))
    want = F.scaled_dot_product_attention(qt, kt, vt, attn_mask=torch.from_numpy(mask).double()).transpose(0, 1).numpy()
    assert close(oracle.sdpa(q, k, v, mask), want, 1e-5, 1e-5)
    # GQA: 4 query heads over 2 kv heads == repeat_interleave of kv heads
    k2, v2 = k[:, :2], v[:, :2]
    want = oracle.sdpa(q, np.repeat(k2, 2, axis=1), np.repeat(v2, 2, axis=1), mask)
    assert np.array_equal(oracle.sdpa(q, np.ascontiguousarray(k2), np.ascontiguousarray(v2), mask), want)
