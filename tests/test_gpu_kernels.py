"""GPU parity: every hand-written fused item, called through the C ABI, against the CPU oracle.

Bars: bit-exact for dequantised weight values and indices/argmax;
rtol 1e-3 / atol 1e-4 for fp32 arithmetic.
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


@pytest.fixture(scope="module")
def ops():
    from caten_amd import _lib, ops as o
    _lib.init(0)
    return o


def _bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


# ------------------------------------------------------------------ codecs
@pytest.mark.parametrize("n", [32, 64, 40, 1, 31, 33, 32 * 1000 + 7, 768 * 2304])
def test_dequant_q8_0_bit_exact(ops, oracle, n):
    print(f"case: q8_0 dequant n={n}", flush=True)
    rng = np.random.default_rng(n)
    nb = (n + 31) // 32
    raw = rng.integers(0, 256, size=nb * 34, dtype=np.uint8)
    sc = rng.normal(0, 0.01, nb).astype(np.float16)
    raw.reshape(nb, 34)[:, :2] = sc.view(np.uint8).reshape(nb, 2)
    got = ops.dequantize("q8_0", raw, n)
    want = oracle.dequant("q8_0", raw, n)
    assert np.array_equal(_bits(got), _bits(want))


def test_dequant_q8_0_all_scales(ops, oracle):
    # every finite fp16 scale (incl. denormals) x int8 values
    scales = np.arange(65536, dtype=np.uint16)
    scales = scales[np.isfinite(scales.view(np.float16))]
    nb = scales.size
    raw = np.empty((nb, 34), np.uint8)
    raw[:, :2] = scales.view(np.uint8).reshape(nb, 2)
    q = (np.arange(nb * 32) * 7 % 256).astype(np.uint8)
    raw[:, 2:] = q.reshape(nb, 32)
    got = ops.dequantize("q8_0", raw, nb * 32)
    want = oracle.dequant("q8_0", raw, nb * 32)
    assert np.array_equal(_bits(got), _bits(want))


@pytest.mark.parametrize("n", [32, 64, 32 * 999])
def test_dequant_q4_0_bit_exact(ops, oracle, n):
    rng = np.random.default_rng(n)
    nb = n // 32
    raw = rng.integers(0, 256, size=nb * 18, dtype=np.uint8)
    raw.reshape(nb, 18)[:, :2] = rng.normal(0, 0.01, nb).astype(np.float16).view(np.uint8).reshape(nb, 2)
    assert np.array_equal(_bits(ops.dequantize("q4_0", raw, n)), _bits(oracle.dequant("q4_0", raw, n)))


def test_dequant_q4_0_rejects_ragged(ops):
    from caten_amd import HipError
    with pytest.raises(HipError):
        ops.dequantize("q4_0", np.zeros(36, np.uint8), 40)


def test_host_pointers_are_refused_not_dereferenced(ops):
    """The codecs take device pointers; pageable host memory is rejected on the host side, before any launch."""
    import ctypes as C
    from caten_amd import _lib, HipError
    lib = _lib.load()
    raw = np.zeros(34 * 8, np.uint8)
    out = ops.DeviceArray((256,), np.float32)
    with pytest.raises(HipError, match="device pointer"):
        _lib.check(lib.cthip_dequant(_lib.Q8_0, raw.ctypes.data, 256, out.ptr))
    h = C.c_void_p()
    with pytest.raises(HipError, match="device pointer"):
        _lib.check(lib.cthip_wmat_create(C.byref(h), _lib.Q8_0, raw.ctypes.data, 8, 32))


def test_dequant_f16_f32(ops, oracle):
    bits = np.arange(65536, dtype=np.uint16)
    got = ops.dequantize("f16", bits.view(np.uint8), 65536)
    want = oracle.dequant("f16", bits.view(np.uint8), 65536)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan) and np.array_equal(_bits(got[~nan]), _bits(want[~nan]))
    x = np.random.default_rng(0).normal(size=1001).astype(np.float32)
    assert np.array_equal(_bits(ops.dequantize("f32", x.view(np.uint8), 1001)), _bits(x))


@pytest.mark.parametrize("kind", ["q8_0", "q4_0", "f16", "f32"])
def test_weight_matrix_planes_keep_values(ops, oracle, kind):
    from caten_amd.llm import Tensor
    rng = np.random.default_rng(11)
    w = rng.normal(0, 0.02, (37, 256)).astype(np.float32)
    t = Tensor.from_f32(w, kind)
    wm = ops.WeightMatrix(kind, t.raw, 37, 256)
    assert wm.nbytes == t.raw.size
    got = wm.dequantize()
    want = oracle.dequant(kind, t.raw, w.size).reshape(37, 256)
    assert np.array_equal(_bits(got), _bits(want))


def test_quantisers_match_oracle(oracle):
    from caten_amd import quant
    rng = np.random.default_rng(12)
    w = rng.normal(0, 0.02, 32 * 500).astype(np.float32)
    w[:32] = 0.0  # an all-zero block
    for kind in ("q8_0", "q4_0"):
        assert np.array_equal(quant.quantize(kind, w), oracle.quantize(kind, w))


# ------------------------------------------------------------------ Linear / GEMV
SHAPES = [(768, 768), (2304, 768), (3072, 768), (768, 3072), (5003, 768), (1000, 256), (64, 2048), (96, 5632),
          (33, 96), (17, 1024), (50257, 768)]


@pytest.mark.parametrize("kind", ["q8_0", "q4_0", "f32", "f16"])
@pytest.mark.parametrize("rows,cols", SHAPES)
def test_gemv_plain(ops, oracle, kind, rows, cols):
    print(f"case: gemv {kind} ({rows},{cols})", flush=True)
    from caten_amd.llm import Tensor
    rng = np.random.default_rng(rows * 7 + cols)
    w = rng.normal(0, 0.02, (rows, cols)).astype(np.float32)
    x = rng.normal(0, 1, cols).astype(np.float32)
    t = Tensor.from_f32(w, kind)
    wd = oracle.dequant(kind, t.raw, w.size).reshape(rows, cols)
    wm = ops.WeightMatrix(kind, t.raw, rows, cols)
    close(ops.linear(x, wm), oracle.linear(x, wd))


@pytest.mark.parametrize("kind,cols", [("f32", 10), ("f32", 1023), ("f16", 12), ("f16", 770)])
@pytest.mark.parametrize("m", [1, 5])
def test_gemv_rows_that_are_not_whole_chunks(ops, oracle, kind, cols, m):
    """fp32 / fp16 weight rows whose width is no multiple of four / eight elements: rows start at any element and the
    last columns count (every column gets a weight that a dropped tail or a wrong row stride would miss)."""
    print(f"case: gemv {kind} cols {cols} m {m}", flush=True)
    from caten_amd.llm import Tensor
    rows = 37
    rng = np.random.default_rng(cols * 3 + m)
    w = rng.normal(0, 0.5, (rows, cols)).astype(np.float32)
    w[:, -1] += 3.0
    x = rng.normal(0, 1, (m, cols)).astype(np.float32)
    b = rng.normal(0, 1, rows).astype(np.float32)
    t = Tensor.from_f32(w, kind)
    wd = oracle.dequant(kind, t.raw, w.size).reshape(rows, cols)
    wm = ops.WeightMatrix(kind, t.raw, rows, cols)
    got = ops.linear(x, wm, bias=b, act="relu")
    close(got, oracle.relu(oracle.linear(x, wd, b)))
    ref = np.maximum(x.astype(np.float64) @ wd.astype(np.float64).T + b, 0.0)
    close(got, ref)


@pytest.mark.parametrize("kind", ["q8_0", "q4_0", "f32"])
def test_gemv_fused_neighbours(ops, oracle, kind):
    from caten_amd.llm import Tensor
    rng = np.random.default_rng(21)
    rows, cols = 3072, 768
    w = rng.normal(0, 0.02, (rows, cols)).astype(np.float32)
    x = rng.normal(0.3, 2, cols).astype(np.float32)
    b = rng.normal(0, 0.02, rows).astype(np.float32)
    r = rng.normal(0, 1, rows).astype(np.float32)
    g = rng.normal(1, 0.02, cols).astype(np.float32)
    be = rng.normal(0, 0.02, cols).astype(np.float32)
    t = Tensor.from_f32(w, kind)
    wd = oracle.dequant(kind, t.raw, w.size).reshape(rows, cols)
    wm = ops.WeightMatrix(kind, t.raw, rows, cols)
    # LayerNorm -> Linear + bias -> GELU (items 9+10 of a decode step)
    want = oracle.gelu_tanh(oracle.linear(oracle.layernorm(x, g, be), wd, b))
    close(ops.linear(x, wm, bias=b, act="gelu", prologue="layernorm", norm_g=g, norm_b=be), want)
    # Linear + bias + residual
    close(ops.linear(x, wm, bias=b, residual=r), oracle.linear(x, wd, b) + r)
    # RMSNorm -> Linear, ReLU
    close(ops.linear(x, wm, act="relu", prologue="rmsnorm", norm_g=g), oracle.relu(oracle.linear(oracle.rmsnorm(x, g), wd)))
    # SwiGLU prologue: silu(gate) * up
    xx = rng.normal(0, 1, 2 * cols).astype(np.float32)
    want = oracle.linear(oracle.silu(xx[:cols]) * xx[cols:], wd)
    close(ops.linear(xx, wm, prologue="swiglu"), want)


@pytest.mark.parametrize("kind", ["q4_0", "q8_0"])
def test_gemv_wide_input_with_norms(ops, oracle, kind):
    """2048 input features: 4-bit launches stage the input (and the folded RMSNorm's gamma * x and statistics)
    in LDS once per workgroup."""
    from caten_amd.llm import Tensor
    rng = np.random.default_rng(24)
    cols = 2048
    for rows in (200, 2560):
        w = rng.normal(0, 0.02, (rows, cols)).astype(np.float32)
        x = rng.normal(0.2, 1.5, cols).astype(np.float32)
        g = rng.normal(1, 0.05, cols).astype(np.float32)
        be = rng.normal(0, 0.05, cols).astype(np.float32)
        t = Tensor.from_f32(w, kind)
        wd = oracle.dequant(kind, t.raw, w.size).reshape(rows, cols)
        wm = ops.WeightMatrix(kind, t.raw, rows, cols)
        close(ops.linear(x, wm, prologue="rmsnorm", norm_g=g), oracle.linear(oracle.rmsnorm(x, g), wd))
        close(ops.linear(x, wm, prologue="layernorm", norm_g=g, norm_b=be), oracle.linear(oracle.layernorm(x, g, be), wd))
        close(ops.linear(x, wm), oracle.linear(x, wd))


@pytest.mark.parametrize("kind", ["q4_0", "q8_0", "f16", "f32"])
def test_gemv_streamed_weights_give_the_same_bits(ops, kind):
    """The non-temporal request of the weights (what models past the Infinity Cache get) changes the cache policy
    of the loads and nothing else: outputs are bit-identical to the cached-weights kernels, on a one-tile-per-
    wavefront launch and on a looping one, with and without a staged input."""
    from caten_amd import _lib
    from caten_amd.llm import Tensor
    rng = np.random.default_rng(27)
    lib = _lib.load()
    for rows, cols in ((300, 768), (9000, 768), (2560, 2048)):
        w = rng.normal(0, 0.02, (rows, cols)).astype(np.float32)
        x = rng.normal(0.1, 1.0, cols).astype(np.float32)
        g = rng.normal(1, 0.05, cols).astype(np.float32)
        wm = ops.WeightMatrix(kind, Tensor.from_f32(w, kind).raw, rows, cols)
        outs = {}
        try:
            for mode in (0, 1):
                _lib.check(lib.cthip_set_option(b"gemv_stream_weights", mode))
                outs[mode] = (ops.linear(x, wm), ops.linear(x, wm, prologue="rmsnorm", norm_g=g))
        finally:
            _lib.check(lib.cthip_set_option(b"gemv_stream_weights", -1))
        for a, b in zip(outs[0], outs[1]):
            assert np.array_equal(a, b)
    with pytest.raises(_lib.HipError):
        _lib.check(lib.cthip_set_option(b"gemv_stream_weights", 2))


@pytest.mark.parametrize("kind", ["q8_0", "q4_0", "f32", "f16"])
def test_layernorm_folded_through_the_product(ops, oracle, kind):
    """cthip_wmat_fold_layernorm: LayerNorm carried through the product (S = W.gamma, C = W.beta + bias) gives the
    Linear of the normalised input, on one-tile-per-wavefront launches, on looping ones (which normalise the staged
    vector themselves when no per-row operand is left) and with several input rows; a call with other vectors
    keeps normalising first."""
    from caten_amd.llm import Tensor
    rng = np.random.default_rng(31)
    for rows, cols, with_bias in ((2304, 768, True), (9000, 768, False), (9000, 768, True), (1500, 2048, True)):
        w = rng.normal(0, 0.02, (rows, cols)).astype(np.float32)
        g = rng.normal(1, 0.05, cols).astype(np.float32)
        b = rng.normal(0, 0.05, cols).astype(np.float32)
        bias = rng.normal(0, 0.1, rows).astype(np.float32) if with_bias else None
        t = Tensor.from_f32(w, kind)
        wd = oracle.dequant(kind, t.raw, w.size).reshape(rows, cols)
        wm = ops.WeightMatrix(kind, t.raw, rows, cols)
        wm.fold_layernorm(g, b, bias)
        for m in (1, 3):
            x = rng.normal(0.3, 1.5, (m, cols)).astype(np.float32)
            want = oracle.linear(oracle.layernorm(x, g, b), wd, bias)
            close(wm.linear_folded(x), want, rtol=2e-3, atol=2e-4)
            close(ops.linear(x, wm, bias=bias, prologue="layernorm", norm_g=g, norm_b=b), want, rtol=2e-3, atol=2e-4)
        wm.free()


@pytest.mark.parametrize("kind", ["q8_0", "q4_0"])
def test_looping_launches_with_long_staged_inputs(ops, oracle, kind):
    """Looping launches whose staged input is longer than what a thread requests ahead of the weights (4096 floats):
    the rest of the vector is staged by a loop behind the first tile; a LayerNorm that is not folded and has a bias
    beside it is applied by the workgroup before the stream starts.  RMSNorm, SwiGLU and plain inputs, with and
    without residual."""
    from caten_amd.llm import Tensor
    rng = np.random.default_rng(33)
    rows, cols = 5000, 6144
    w = rng.normal(0, 0.02, (rows, cols)).astype(np.float32)
    t = Tensor.from_f32(w, kind)
    wd = oracle.dequant(kind, t.raw, w.size).reshape(rows, cols)
    wm = ops.WeightMatrix(kind, t.raw, rows, cols)
    x = rng.normal(0.2, 1.0, cols).astype(np.float32)
    g = rng.normal(1, 0.05, cols).astype(np.float32)
    b = rng.normal(0, 0.05, cols).astype(np.float32)
    bias = rng.normal(0, 0.1, rows).astype(np.float32)
    res = rng.normal(0, 1, rows).astype(np.float32)
    tol = dict(rtol=2e-3, atol=3e-4)
    close(ops.linear(x, wm, prologue="rmsnorm", norm_g=g), oracle.linear(oracle.rmsnorm(x, g), wd), **tol)
    close(ops.linear(x, wm, residual=res, prologue="rmsnorm", norm_g=g), oracle.linear(oracle.rmsnorm(x, g), wd) + res, **tol)
    close(ops.linear(x, wm, bias=bias, prologue="layernorm", norm_g=g, norm_b=b),
          oracle.linear(oracle.layernorm(x, g, b), wd, bias), **tol)
    close(ops.linear(x, wm, prologue="layernorm", norm_g=g, norm_b=b), oracle.linear(oracle.layernorm(x, g, b), wd), **tol)
    close(ops.linear(x, wm, bias=bias, residual=res), oracle.linear(x, wd, bias) + res, **tol)
    xu = rng.normal(0, 1, 2 * cols).astype(np.float32)
    gate, up = xu[:cols].astype(np.float64), xu[cols:].astype(np.float64)
    sw = (gate / (1 + np.exp(-gate)) * up).astype(np.float32)
    close(ops.linear(xu, wm, residual=res, prologue="swiglu"), oracle.linear(sw, wd) + res, **tol)
    wm.free()


def test_gemv_fallback_shapes_with_prologue(ops, oracle):
    from caten_amd.llm import Tensor
    rng = np.random.default_rng(22)
    rows, cols = 45, 9984  # no register-resident variant covers 9984 columns of q8_0
    w = rng.normal(0, 0.02, (rows, cols)).astype(np.float32)
    x = rng.normal(0, 1, cols).astype(np.float32)
    g = rng.normal(1, 0.02, cols).astype(np.float32)
    t = Tensor.from_f32(w, "q8_0")
    wd = oracle.dequant("q8_0", t.raw, w.size).reshape(rows, cols)
    wm = ops.WeightMatrix("q8_0", t.raw, rows, cols)
    close(ops.linear(x, wm, prologue="layernorm", norm_g=g), oracle.linear(oracle.layernorm(x, g), wd))


@pytest.mark.parametrize("wide", [0, 1])
@pytest.mark.parametrize("kind,rows,cols,m", [("q4_0", 4096, 11008, 1), ("q8_0", 1000, 11008, 1), ("q4_0", 515, 28672, 1),
                                              ("f32", 300, 12288, 1), ("f16", 300, 6400, 1), ("q8_0", 300, 8224, 3)])
def test_gemv_rows_wider_than_any_variant(ops, oracle, kind, rows, cols, m, wide):
    """FFN down-projections of 7B-class models and up (11008, 13824, 28672 input features) are wider than what a
    lane group keeps in registers.  Quantised rows that LDS holds take the wide-row kernel (option gemv_wide 1, the
    default); otherwise (gemv_wide 0, fp32 / fp16 rows) the launcher cuts the columns into equal slices, slice 0
    carries bias and residual, the others add to it.  Every column gets a weight that a wrong chunk index, slice
    offset or row pitch would miss; SwiGLU reads `up` behind the whole gate half."""
    print(f"case: wide gemv {kind} ({rows},{cols}) m {m} gemv_wide {wide}", flush=True)
    from caten_amd import _lib
    _lib.check(_lib.load().cthip_set_option(b"gemv_wide", wide))
    try:
        _wide_rows_case(ops, oracle, kind, rows, cols, m)
    finally:
        _lib.check(_lib.load().cthip_set_option(b"gemv_wide", 1))


def _wide_rows_case(ops, oracle, kind, rows, cols, m):
    from caten_amd.llm import Tensor
    rng = np.random.default_rng(rows + cols)
    w = rng.normal(0, 0.02, (rows, cols)).astype(np.float32)
    w[:, ::97] += 0.05  # columns that stand out, spread over every slice
    x = rng.normal(0.1, 1, (m, cols)).astype(np.float32)
    b = rng.normal(0, 0.02, rows).astype(np.float32)
    r = rng.normal(0, 1, (m, rows)).astype(np.float32)
    t = Tensor.from_f32(w, kind)
    wd = oracle.dequant(kind, t.raw, w.size).reshape(rows, cols)
    wm = ops.WeightMatrix(kind, t.raw, rows, cols)
    tol = dict(rtol=2e-4, atol=2e-4)
    xs, rs = (x[0], r[0]) if m == 1 else (x, r)
    close(ops.linear(xs, wm), oracle.linear(xs, wd), **tol)
    close(ops.linear(xs, wm, bias=b, residual=rs), oracle.linear(xs, wd, b) + rs, **tol)
    xu = rng.normal(0, 1, (m, 2 * cols)).astype(np.float32)
    sw = (oracle.silu(xu[:, :cols]) * xu[:, cols:]).astype(np.float32)
    xus, sws = (xu[0], sw[0]) if m == 1 else (xu, sw)
    close(ops.linear(xus, wm, residual=rs, prologue="swiglu"), oracle.linear(sws, wd) + rs, **tol)
    # what needs the whole row at once still goes through the wave-per-row kernel
    g = rng.normal(1, 0.02, cols).astype(np.float32)
    close(ops.linear(xs, wm, act="relu", prologue="rmsnorm", norm_g=g), oracle.relu(oracle.linear(oracle.rmsnorm(xs, g), wd)), **tol)
    wm.free()


@pytest.mark.parametrize("kind", ["q4_0", "q8_0", "f16", "f32"])
def test_gemv_wide_row_kernel_on_every_launch_it_supports(ops, oracle, kind):
    """option gemv_wide 2 sends every single-row Linear without a LayerNorm or a fused argmax through the
    wide-row kernel: widths of one partial round, whole and partial tiles of 1..4 rounds, fewer rows than wavefronts
    and many more, several input rows, every prologue and epilogue it carries."""
    from caten_amd import _lib
    from caten_amd.llm import Tensor
    lib = _lib.load()
    tol = dict(rtol=2e-4, atol=2e-4)
    _lib.check(lib.cthip_set_option(b"gemv_wide", 2))
    try:
        for rows, cols, m in [(5, 64, 1), (70, 96, 2), (1000, 2048, 1), (777, 2080, 3), (2304, 768, 1), (640, 4096, 1),
                              (5000, 5504, 1), (300, 6144, 1), (9, 8192, 7), (16500, 1024, 1)]:
            print(f"case: wide-row kernel {kind} ({rows},{cols}) m {m}", flush=True)
            rng = np.random.default_rng(rows * 3 + cols)
            w = rng.normal(0, 0.02, (rows, cols)).astype(np.float32)
            w[:, ::61] += 0.05
            x = rng.normal(0.1, 1, (m, cols)).astype(np.float32)
            x[:, 32:64] = 0.0      # a chunk of zeros
            x[:, 5] = 30.0         # a large input among small ones
            b = rng.normal(0, 0.02, rows).astype(np.float32)
            r = rng.normal(0, 1, (m, rows)).astype(np.float32)
            g = rng.normal(1, 0.02, cols).astype(np.float32)
            t = Tensor.from_f32(w, kind)
            wd = oracle.dequant(kind, t.raw, w.size).reshape(rows, cols)
            wm = ops.WeightMatrix(kind, t.raw, rows, cols)
            xs, rs = (x[0], r[0]) if m == 1 else (x, r)
            close(ops.linear(xs, wm), oracle.linear(xs, wd), **tol)
            close(ops.linear(xs, wm, bias=b, residual=rs, act="gelu"), oracle.gelu_tanh(oracle.linear(xs, wd, b)) + rs, **tol)
            close(ops.linear(xs, wm, residual=rs, prologue="rmsnorm", norm_g=g), oracle.linear(oracle.rmsnorm(xs, g), wd) + rs, **tol)
            close(ops.linear(xs, wm, bias=b, prologue="rmsnorm"), oracle.linear(oracle.rmsnorm(xs), wd, b), **tol)
            xu = rng.normal(0, 1, (m, 2 * cols)).astype(np.float32)
            sw = (oracle.silu(xu[:, :cols]) * xu[:, cols:]).astype(np.float32)
            xus, sws = (xu[0], sw[0]) if m == 1 else (xu, sw)
            close(ops.linear(xus, wm, bias=b, prologue="swiglu"), oracle.linear(sws, wd, b), **tol)
            # a LayerNorm in front keeps the register-resident kernels
            close(ops.linear(xs, wm, prologue="layernorm", norm_g=g), oracle.linear(oracle.layernorm(xs, g), wd), **tol)
            wm.free()
    finally:
        _lib.check(lib.cthip_set_option(b"gemv_wide", 1))


def test_linear_batched_rows(ops, oracle):
    from caten_amd.llm import Tensor
    rng = np.random.default_rng(23)
    rows, cols, m = 300, 768, 5
    w = rng.normal(0, 0.02, (rows, cols)).astype(np.float32)
    x = rng.normal(0, 1, (m, cols)).astype(np.float32)
    b = rng.normal(0, 0.02, rows).astype(np.float32)
    t = Tensor.from_f32(w, "q8_0")
    wd = oracle.dequant("q8_0", t.raw, w.size).reshape(rows, cols)
    wm = ops.WeightMatrix("q8_0", t.raw, rows, cols)
    close(ops.linear(x, wm, bias=b), oracle.linear(x, wd, b))
    assert ops.linear(np.zeros((0, cols), np.float32), wm).shape == (0, rows)


def test_linear_argument_errors(ops):
    from caten_amd import HipError
    with pytest.raises(ValueError):
        ops.WeightMatrix("q8_0", np.zeros(10, np.uint8), 4, 32)  # wrong byte count
    with pytest.raises(HipError):
        ops.WeightMatrix("q8_0", np.zeros(68, np.uint8), 3, 16)  # quantised rows need cols % 32 == 0
    wm = ops.WeightMatrix("f32", np.zeros(4 * 64, np.uint8), 2, 32)
    with pytest.raises(ValueError):
        ops.linear(np.zeros(31, np.float32), wm)


# ------------------------------------------------------------------ row ops
@pytest.mark.parametrize("shape", [(128, 128), (64, 768), (7, 40), (3, 2048), (2, 5000), (5, 1), (300, 36)])
def test_rowops(ops, oracle, shape):
    print(f"case: rowops {shape}", flush=True)
    rng = np.random.default_rng(shape[0] + shape[1])
    x = rng.normal(0, 1, shape).astype(np.float32)
    g = rng.normal(1, 0.02, shape[-1]).astype(np.float32)
    b = rng.normal(0, 0.02, shape[-1]).astype(np.float32)
    close(ops.softmax(x), oracle.softmax(x), 1e-5, 1e-6)
    if shape[-1] > 1:
        close(ops.layernorm(x, g, b), oracle.layernorm(x, g, b), 1e-4, 1e-5)
        close(ops.layernorm(x), oracle.layernorm(x), 1e-4, 1e-5)
        close(ops.layernorm_softmax(x, g, b), oracle.softmax(oracle.layernorm(x, g, b)), 1e-4, 1e-6)
    close(ops.rmsnorm(x, g), oracle.rmsnorm(x, g), 1e-4, 1e-5)


def test_softmax_fuzz_large_values(ops, oracle):
    rng = np.random.default_rng(31)
    x = rng.normal(10, 100, (512, 512)).astype(np.float32)  # test-activations.lisp:60-73
    y = ops.softmax(x)
    close(y, oracle.softmax(x), 1e-5, 1e-5)
    assert np.allclose(y.sum(-1), 1.0, atol=1e-5)


def test_rowops_empty(ops):
    assert ops.softmax(np.zeros((0, 8), np.float32)).shape == (0, 8)
    assert ops.layernorm(np.zeros((0, 8), np.float32)).shape == (0, 8)


def test_unary(ops, oracle):
    x = np.linspace(-9, 9, 100003).astype(np.float32)
    assert np.array_equal(ops.relu(x), oracle.relu(x))
    close(ops.gelu(x), oracle.gelu_tanh(x), 1e-5, 1e-6)
    close(ops.silu(x), oracle.silu(x), 1e-5, 1e-6)
    close(ops.sigmoid(x), oracle.sigmoid(x), 1e-5, 1e-6)
    close(ops.tanh(x), oracle.tanh(x), 1e-5, 1e-6)
    assert ops.gelu(np.zeros(0, np.float32)).shape == (0,)


@pytest.mark.parametrize("n", [1, 1023, 1024, 1025, 5000])
def test_unary_on_pointers_that_are_not_16_byte_aligned(ops, oracle, n):
    """Arrays that start 4 bytes into an allocation take the element-wise form of the kernel (whole blocks of 1024
    and a tail) instead of the 128-bit one."""
    from caten_amd import _lib
    from caten_amd.ops import DeviceArray
    print(f"case: unaligned unary n={n}", flush=True)
    x = np.linspace(-4, 4, n + 1).astype(np.float32)
    dx, dy = DeviceArray.from_numpy(x), DeviceArray((n + 1,), np.float32)
    _lib.check(_lib.load().cthip_unary(_lib.ACT_GELU, dy.ptr + 4, dx.ptr + 4, n))
    got = dy.numpy()
    assert got[0] == 0.0  # the element in front of the output stays as allocated
    close(got[1:], oracle.gelu_tanh(x[1:]), 1e-5, 1e-6)


def test_embedding_and_argmax(ops, oracle):
    rng = np.random.default_rng(41)
    W = rng.normal(size=(523, 48)).astype(np.float32)
    idx = rng.integers(0, 523, (3, 7)).astype(np.float32)
    assert np.array_equal(ops.embedding(W, idx), oracle.embedding_onehot(W, idx))
    # an index that equals no vocabulary row selects nothing in the one-hot sum
    odd = np.array([1.0, 522.0, 523.0, -1.0, 2.5], np.float32)
    assert np.array_equal(ops.embedding(W, odd), oracle.embedding_onehot(W, odd))
    for n in (1, 10, 63, 64, 65, 1024, 50257):
        x = rng.integers(0, 5, n).astype(np.float32)  # many ties -> lowest index
        assert ops.argmax(x) == oracle.argmax(x)
    x = rng.normal(size=(9, 50257)).astype(np.float32)
    assert np.array_equal(ops.argmax(x), np.array([oracle.argmax(r) for r in x]))
    # few long rows are reduced in 64 parts per row, then settled: ties across parts, the maximum in the last, short
    # part, rows of -inf and of NaN, and the sizes either side of where that path starts
    for n in (8191, 8192, 8193, 50257, 50304):
        x = rng.integers(0, 3, (3, n)).astype(np.float32)
        x[1, :] = 0.0
        x[1, n - 1] = 7.0
        x[2, :] = -np.inf
        assert np.array_equal(ops.argmax(x), np.array([oracle.argmax(r) for r in x])), n
        assert ops.argmax(np.full(n, np.nan, np.float32)) == 0
    x = rng.normal(size=(17, 9000)).astype(np.float32)  # more rows than that path takes
    assert np.array_equal(ops.argmax(x), np.array([oracle.argmax(r) for r in x]))
    assert ops.argmax(np.arange(10, dtype=np.float32)) == 9  # test-ops.lisp:107-114


def test_rope(ops, oracle):
    rng = np.random.default_rng(51)
    x = rng.uniform(0, 1, (1, 10, 10, 10)).astype(np.float32)
    close(ops.rope(x), oracle.rope(x), 5e-4, 1e-5)  # test-rope.lisp:58-66
    x = rng.normal(size=(2, 6, 4, 64)).astype(np.float32)
    close(ops.rope(x, start_pos=900), oracle.rope(x, start_pos=900), 1e-3, 1e-4)


@pytest.mark.parametrize("S,start,H,Hkv,Dh", [(1, 0, 4, 4, 64), (1, 37, 12, 12, 64), (5, 3, 8, 2, 64),
                                             (1, 700, 4, 1, 128), (3, 0, 2, 2, 32),
                                             # prompt-sized row counts: groups of rows share their K / V tiles
                                             (16, 0, 4, 4, 64), (37, 5, 8, 2, 64), (130, 0, 2, 2, 64), (21, 200, 2, 1, 128),
                                             (19, 3, 2, 2, 32), (512, 0, 2, 2, 64),
                                             # 32 rows and more: the matrix-core kernel (ragged last group, GQA, other head sizes)
                                             (32, 0, 2, 2, 64), (33, 7, 4, 2, 64), (70, 100, 2, 1, 128), (45, 2, 2, 2, 32),
                                             # several tiles per wavefront, tiles whose keys some rows do not see
                                             # (start not a multiple of 32)
                                             (300, 21, 4, 2, 64), (200, 150, 2, 1, 128), (1100, 0, 1, 1, 32),
                                             (40, 2100, 2, 1, 64)])
def test_sdpa_cached(ops, oracle, S, start, H, Hkv, Dh):
    print(f"case: sdpa_cached S={S} start={start} H={H}/{Hkv} Dh={Dh}", flush=True)
    rng = np.random.default_rng(S + start)
    T = start + S
    maxlen = T + 5
    q = rng.normal(size=(S, H, Dh)).astype(np.float32)
    k = rng.normal(size=(maxlen, Hkv, Dh)).astype(np.float32)
    v = rng.normal(size=(maxlen, Hkv, Dh)).astype(np.float32)
    mask = oracle.triu_neginf(S, T, 1 + start)
    want = oracle.sdpa(q, np.ascontiguousarray(k[:T]), np.ascontiguousarray(v[:T]), mask)
    close(ops.sdpa_cached(q, k, v, start), want, 1e-4, 1e-5)
    if S >= 32:  # the matrix-core kernel with fp32 operands instead of two bf16 terms per operand
        from caten_amd import _lib
        lib = _lib.load()
        _lib.check(lib.cthip_set_option(b"gemm_precision", 0))
        try:
            close(ops.sdpa_cached(q, k, v, start), want, 1e-4, 1e-5)
        finally:
            _lib.check(lib.cthip_set_option(b"gemm_precision", 2))


# ------------------------------------------------------------------ matmul (MFMA)
@pytest.mark.parametrize("M,N,K", [(256, 256, 256), (64, 64, 32), (3, 5, 7), (65, 33, 17), (100, 768, 1024), (1, 64, 64),
                                   (128, 128, 64), (64, 128, 160), (70, 64, 128), (64, 192, 96),  # 2, 5, 4, 3 K-steps of 32
                                   (100, 70, 2000), (33, 65, 1030), (64, 64, 4096)])  # the last three split K
def test_matmul_relu_vs_oracle(ops, oracle, M, N, K):
    print(f"case: matmul {M}x{N}x{K}", flush=True)
    rng = np.random.default_rng(M * 31 + N * 7 + K)
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    for precision in ("fp32", "bf16x6"):  # both hold the fp32 bar
        close(ops.matmul(A, B, relu=True, precision=precision), oracle.matmul(A, B, relu=True))
        close(ops.matmul(A, B, precision=precision), oracle.matmul(A, B))
    # two bf16 terms per operand: 2^-16 of a product is lost, sqrt(K) of them add up
    close(ops.matmul(A, B, relu=True, precision="bf16x3"), oracle.matmul(A, B, relu=True), 1e-3, 2e-5 * np.sqrt(K))
    close(ops.matmul(A, B, relu=True, precision="bf16"), oracle.matmul(A, B, relu=True), 1e-2, 1e-2 * np.sqrt(K))


def test_matmul_1024_cubed(ops):
    # the 1024^3 benchmark configuration: A, B ~ U(-1,1) fp32 (1024,1024); fp64 NumPy is the tie-breaker at this size
    rng = np.random.default_rng(0)
    A = rng.uniform(-1, 1, (1024, 1024)).astype(np.float32)
    B = rng.uniform(-1, 1, (1024, 1024)).astype(np.float32)
    want = np.maximum(A.astype(np.float64) @ B.astype(np.float64), 0)
    close(ops.matmul(A, B, relu=True, precision="fp32"), want)
    got = ops.matmul(A, B, relu=True, precision="bf16x6")
    close(got, want)
    assert np.max(np.abs(got - want)) < 1e-4  # three bf16 terms carry all 24 bits; what is left is fp32 accumulation
    assert np.max(np.abs(ops.matmul(A, B, relu=True, precision="bf16x3") - want)) < 6e-4
    got = ops.matmul(A, B, relu=True, precision="bf16")
    assert np.max(np.abs(got - want)) < 1e-2 * np.sqrt(1024) and np.all(got >= 0)
    # all-ones closed form (test-runtime.lisp:241-252): every entry is K
    for precision in ("fp32", "bf16x6", "bf16x3", "bf16"):
        assert np.all(ops.matmul(np.ones((64, 96), np.float32), np.ones((96, 32), np.float32), precision=precision) == 96)


def test_matmul_degenerate(ops):
    assert ops.matmul(np.zeros((0, 8), np.float32), np.zeros((8, 4), np.float32)).shape == (0, 4)
    assert np.all(ops.matmul(np.zeros((3, 0), np.float32), np.zeros((0, 4), np.float32)) == 0)


@pytest.mark.parametrize("kind", ["q8_0", "q4_0"])
@pytest.mark.parametrize("rows,cols,m", [(4100, 256, 130), (333, 160, 70), (200, 4160, 40), (70, 12352, 9)])
def test_linear_many_rows_quantised(ops, oracle, kind, rows, cols, m):
    """Several input rows on the quantised MFMA path (integer plane times the block scales) against the product
    with the dequantised weights: ragged tile edges in both directions; a row width whose scale rows are not
    16-byte aligned; reductions longer than one scale tile (2048) with a partial last tile and a partial last
    period of steps; a reduction long enough to be split over several workgroups per tile."""
    from caten_amd import _lib
    from caten_amd.llm import Tensor
    rng = np.random.default_rng(62)
    w = rng.normal(0, 0.02, (rows, cols)).astype(np.float32)
    x = rng.normal(0, 1, (m, cols)).astype(np.float32)
    b = rng.normal(0, 0.02, rows).astype(np.float32)
    t = Tensor.from_f32(w, kind)
    wd = oracle.dequant(kind, t.raw, w.size).reshape(rows, cols)
    wm = ops.WeightMatrix(kind, t.raw, rows, cols)
    want = oracle.linear(x, wd, b)
    lib = _lib.load()
    try:
        for mode in (2, 3, 0):
            _lib.check(lib.cthip_set_option(b"gemm_precision", mode))
            close(ops.linear(x, wm, bias=b), want)
        _lib.check(lib.cthip_set_option(b"gemm_precision", 1))
        close(ops.linear(x, wm, bias=b), want, 1e-2, 1e-2)
    finally:
        _lib.check(lib.cthip_set_option(b"gemm_precision", 2))


@pytest.mark.parametrize("kind", ["f16", "f32"])
@pytest.mark.parametrize("cols", [100, 203, 1000])
def test_linear_many_rows_odd_width(ops, oracle, kind, cols):
    """Unquantised weight rows whose width is no multiple of 16 (4, 8): several input rows must not read across
    the end of a weight row, in any precision mode."""
    from caten_amd import _lib
    from caten_amd.llm import Tensor
    rng = np.random.default_rng(63)
    rows, m = 77, 70
    w = rng.normal(0, 0.05, (rows, cols)).astype(np.float32)
    x = rng.normal(0, 1, (m, cols)).astype(np.float32)
    t = Tensor.from_f32(w, kind)
    wd = oracle.dequant(kind, t.raw, w.size).reshape(rows, cols)
    wm = ops.WeightMatrix(kind, t.raw, rows, cols)
    want = oracle.linear(x, wd, None)
    lib = _lib.load()
    try:
        for mode in (0, 1, 2, 3):
            _lib.check(lib.cthip_set_option(b"gemm_precision", mode))
            if mode == 1 and cols % 16 == 0:
                close(ops.linear(x, wm), want, 1e-2, 1e-2)
            else:
                close(ops.linear(x, wm), want)
    finally:
        _lib.check(lib.cthip_set_option(b"gemm_precision", 2))


@pytest.mark.parametrize("kind", ["q8_0", "q4_0", "f16", "f32"])
def test_linear_prefill_rows_mfma(ops, oracle, kind):
    # m >= 8 input rows take the MFMA tile path with the weights dequantised while staged
    from caten_amd import _lib
    from caten_amd.llm import Tensor
    rng = np.random.default_rng(61)
    rows, cols, m = 300, 768, 37
    w = rng.normal(0, 0.02, (rows, cols)).astype(np.float32)
    x = rng.normal(0, 1, (m, cols)).astype(np.float32)
    b = rng.normal(0, 0.02, rows).astype(np.float32)
    r = rng.normal(0, 1, (m, rows)).astype(np.float32)
    g = rng.normal(1, 0.02, cols).astype(np.float32)
    be = rng.normal(0, 0.02, cols).astype(np.float32)
    t = Tensor.from_f32(w, kind)
    wd = oracle.dequant(kind, t.raw, w.size).reshape(rows, cols)
    wm = ops.WeightMatrix(kind, t.raw, rows, cols)
    want = oracle.gelu_tanh(oracle.linear(oracle.layernorm(x, g, be), wd, b))
    lib = _lib.load()
    try:
        for mode in (2, 3, 0):  # split bf16 operands (two terms = the default, three terms), fp32 operands
            _lib.check(lib.cthip_set_option(b"gemm_precision", mode))
            close(ops.linear(x, wm, bias=b, residual=r), oracle.linear(x, wd, b) + r)
            close(ops.linear(x, wm, bias=b, act="gelu", prologue="layernorm", norm_g=g, norm_b=be), want)
        _lib.check(lib.cthip_set_option(b"gemm_bf16", 1))
        close(ops.linear(x, wm, bias=b, residual=r), oracle.linear(x, wd, b) + r, 1e-2, 1e-2)
    finally:
        _lib.check(lib.cthip_set_option(b"gemm_bf16", 0))
    with pytest.raises(_lib.HipError):
        _lib.check(lib.cthip_set_option(b"gemm_precision", 4))
    with pytest.raises(_lib.HipError):
        _lib.check(_lib.load().cthip_set_option(b"no_such_option", 1))
