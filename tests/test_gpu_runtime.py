"""GPU checks of the backend boundary itself: buffers, the VM (Allocate / View / JIT_KERNEL), the
renderer's kernels launched through hipRTC + cthip_launch, the caching allocator."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def rt():
    import caten_amd as ca
    return ca.HipRuntime()


def test_buffer_protocol(rt):
    from caten_amd.buffer import (HipBuffer, make_buffer, open_buffer, close_buffer, transfer_from_array,
                                  transfer_into_array, copy_buffer_value, bref, buffer_ref)
    b = make_buffer([3, 4], [4, 1], "float32", device=HipBuffer)
    open_buffer(rt, b)
    assert np.all(transfer_into_array(b) == 0)  # open-buffer zero-fills (buffer.lisp:78-79)
    a = np.arange(12, dtype=np.float32)
    transfer_from_array(rt, b, a)
    assert np.array_equal(transfer_into_array(b), a)
    assert bref(b, 7) == 7.0 and buffer_ref(b, 2, 1) == 9.0
    c = b.copy()
    c.value = copy_buffer_value(rt, b)
    transfer_from_array(rt, b, np.zeros(12, np.float32))
    assert np.array_equal(transfer_into_array(c), a)  # a real copy, not an alias
    close_buffer(rt, b)
    close_buffer(rt, b)  # idempotent
    close_buffer(rt, c)
    s = make_buffer([], [], "int64", device=HipBuffer)
    open_buffer(rt, s)
    assert s.value == 0 and transfer_into_array(s) == 0  # rank 0 stays a host number
    for dt in ("int64", "int32", "uint8", "float64", "bool", "float16"):
        d = make_buffer([5], [1], dt, device=HipBuffer)
        open_buffer(rt, d)
        v = (np.arange(5) % 2).astype(d.dtype if dt != "bool" else np.bool_)
        transfer_from_array(rt, d, v)
        assert np.array_equal(transfer_into_array(d), v)
        close_buffer(rt, d)
    with pytest.raises(ValueError):
        d = make_buffer([5], [1], "float32", device=HipBuffer)
        open_buffer(rt, d)
        transfer_from_array(rt, d, np.zeros(4, np.float32))


def test_caching_allocator_reuses_blocks(rt):
    from caten_amd import _lib
    lib = _lib.load()
    live0, cached0, allocs0 = C.c_size_t(), C.c_size_t(), C.c_size_t()
    p = C.c_void_p()
    _lib.check(lib.cthip_alloc(C.byref(p), 100000))
    first = p.value
    _lib.check(lib.cthip_free(p))
    lib.cthip_cache_stats(C.byref(live0), C.byref(cached0), C.byref(allocs0))
    for _ in range(50):  # the per-step reallocation pattern of `s`/`n`-shaped buffers (runtime.lisp:248-259)
        _lib.check(lib.cthip_alloc(C.byref(p), 99000))
        assert p.value == first  # same size class -> same block, no driver call
        out = np.empty(8, np.uint8)
        _lib.check(lib.cthip_d2h(out.ctypes.data, p.value, 8))
        assert np.all(out == 0)  # and zeroed again
        _lib.check(lib.cthip_memset(p.value, 0xAB, 99000))
        _lib.check(lib.cthip_free(p))
    live1, cached1, allocs1 = C.c_size_t(), C.c_size_t(), C.c_size_t()
    lib.cthip_cache_stats(C.byref(live1), C.byref(cached1), C.byref(allocs1))
    assert allocs1.value == allocs0.value and live1.value == live0.value
    assert lib.cthip_free(12345) != 0  # not a block of this allocator
    _lib.check(lib.cthip_alloc(C.byref(p), 0))
    assert p.value
    _lib.check(lib.cthip_free(p))


def _relu_matmul_graph(ca, M, N, K, native=True):
    """The VM graph `jit` would hand the runtime for (caten (!relu (!matmul a b))) with symbolic sizes."""
    from tests.test_host import _matmul_item
    r = ca.HipRenderer()
    item = _matmul_item()
    r.render_kernel(item)
    r.compile_kernel([item])
    info = ca.CompiledKernel(name="fused_relu_matmul", caller=item["compiled_object"], code=r.code, out_positions=(0,))
    graph = [
        ca.Node("Allocate", ["a"], [], {"from": "a_in"}),
        ca.Node("Allocate", ["b"], [], {"from": "b_in"}),
        ca.Node("Allocate", ["out"], ["m", "n", "n", 1], {"nrank": 2, "dtype": "float32"}),
        ca.Node("JIT_KERNEL", ["out2"], ["out", "m", "n", "kk", "a", "b"],
                {"kernel_info": info, "dtypes": ["float32", "int64", "int64", "int64", "float32", "float32"]}),
    ]
    return ca.HipRuntime(graph, fw_outputs=["out2"], renderer=r, native=native)


@pytest.mark.parametrize("native", [True, False])
def test_vm_runs_a_rendered_kernel_with_dynamic_shapes(oracle, native):
    """native: the node list is walked inside the library (one call per forward); else node by node on the host"""
    import caten_amd as ca
    from caten_amd.buffer import AbstractBuffer, make_buffer, transfer_into_array
    vm = _relu_matmul_graph(ca, 0, 0, 0, native=native)
    rng = np.random.default_rng(0)
    pools = []
    for (M, N, K) in ((33, 20, 17), (33, 20, 17), (64, 64, 64), (5, 300, 9)):
        A = rng.uniform(-1, 1, (M, K)).astype(np.float32)
        B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
        # weights/inputs arrive as HOST buffers and are uploaded on first sight
        ha = make_buffer([M, K], [K, 1], "float32", value=A.ravel())
        hb = make_buffer([K, N], [N, 1], "float32", value=B.ravel())
        out = vm.forward(("a_in", ha), ("b_in", hb), ("m", M), ("n", N), ("kk", K))
        got = transfer_into_array(out).reshape(M, N)
        want = oracle.matmul(A, B, relu=True)
        assert np.max(np.abs(got - want)) < 1e-4
        assert (vm._walk is not None) == native
        pools.append(out.value if native else vm.graph[2].attrs["pool"].value)
        assert out.value == pools[-1]
    assert pools[0] == pools[1]  # equal shape -> the :Allocate pool is reused (runtime.lisp:248-252)
    vm.free()


def test_vm_view_and_errors():
    import caten_amd as ca
    from caten_amd.buffer import make_buffer, HipBuffer, open_buffer, transfer_from_array, buffer_ref
    from caten_amd.runtime import RuntimeError_
    rt = ca.HipRuntime([ca.Node("View", ["v"], ["x", 2, 3, 1, 0, 3, 3, 1, 1, 4, 1], {"nrank": 2, "broadcast": [False, False]})],
                       fw_outputs=["v"])
    x = make_buffer([3, 4], [4, 1], "float32", device=HipBuffer)
    open_buffer(rt, x)
    transfer_from_array(rt, x, np.arange(12, dtype=np.float32))
    v = rt.forward(("x", x))
    assert v.shape == [2, 3] and v.value == x.value  # a view moves no data (runtime.lisp:261-284)
    assert buffer_ref(v, 0, 0) == 4.0 and buffer_ref(v, 1, 2) == 10.0  # rows from 1, by 1
    # free-runtime with the buffer and its view both in the variable table: the block goes back once
    import ctypes as C
    lib = ca._lib.load()
    live0, live1 = C.c_size_t(), C.c_size_t()
    ca._lib.check(lib.cthip_cache_stats(C.byref(live0), None, None))
    rt.free()
    ca._lib.check(lib.cthip_cache_stats(C.byref(live1), None, None))
    assert live0.value - live1.value == 256 and v.value is None and x.value is None
    rt.free()
    # a wrong argument count surfaces as a runtime-error carrying the pc (cf. metal.lisp:289)
    vm = _relu_matmul_graph(ca, 0, 0, 0)
    vm.graph[3].reads = ["out", "m", "n", "a", "b"]
    vm.graph[3].attrs["dtypes"] = ["float32", "int64", "int64", "float32", "float32"]
    ha = make_buffer([2, 2], [2, 1], "float32", value=np.zeros(4, np.float32))
    with pytest.raises(RuntimeError_) as e:
        vm.forward(("a_in", ha), ("b_in", ha), ("m", 2), ("n", 2), ("kk", 2))
    assert "instruction 3" in str(e.value)
    vm.free()


def test_rendered_rowwise_kernels_match_oracle(oracle):
    """Softmax as Caten lowers it (one kernel, three loops over the row; test-activations.lisp:60-73),
    authored as a blueprint and run through render -> hipRTC -> launch."""
    import caten_amd as ca
    from caten_amd.buffer import make_buffer, HipBuffer, open_buffer, transfer_from_array, transfer_into_array
    A = lambda id_, idx: {"op": "AREF", "id": id_, "index": idx}  # noqa: E731
    add = lambda *a: {"op": "ADD", "args": list(a)}  # noqa: E731
    mul = lambda *a: {"op": "MUL", "args": list(a)}  # noqa: E731
    lt = lambda a, b: {"op": "<", "args": [a, b]}  # noqa: E731
    idx = add(mul("n", "_gid0"), "_gid1")
    ex = {"op": "EXP2", "args": [mul(add(A("val_x", idx), {"op": "NEG", "args": ["m"]}), 1.442695)]}
    item = {"name": "fused_softmax", "blueprint": [
        {"type": "DEFINE-GLOBAL", "id": "val_y", "dtype": "float32", "pointer_p": True, "arg_type": "output", "nrank": 2},
        {"type": "DEFINE-GLOBAL", "id": "rows", "dtype": "int64", "pointer_p": False, "arg_type": "shape", "nrank": 0},
        {"type": "DEFINE-GLOBAL", "id": "n", "dtype": "int64", "pointer_p": False, "arg_type": "shape", "nrank": 0},
        {"type": "DEFINE-GLOBAL", "id": "val_x", "dtype": "float32", "pointer_p": True, "arg_type": "input", "nrank": 2},
        {"type": "FOR", "idx": "_gid0", "upfrom": 0, "below": lt("_gid0", "rows"), "by": 1},
        {"type": "EXPR", "writes": [A("m", None)], "expr": float("-inf"), "declare_type": True, "dtype": "float32"},
        {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": lt("_gid1", "n"), "by": 1},
        {"type": "EXPR", "writes": [A("m", None)], "expr": {"op": "MAX", "args": ["m", A("val_x", idx)]}, "dtype": "float32", "reduction": True},
        {"type": "ENDFOR", "idx": "_gid1"},
        {"type": "EXPR", "writes": [A("s", None)], "expr": 0.0, "declare_type": True, "dtype": "float32"},
        {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": lt("_gid1", "n"), "by": 1},
        {"type": "EXPR", "writes": [A("s", None)], "expr": add("s", ex), "dtype": "float32", "reduction": True},
        {"type": "ENDFOR", "idx": "_gid1"},
        {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": lt("_gid1", "n"), "by": 1},
        {"type": "EXPR", "writes": [A("val_y", idx)], "expr": mul(ex, {"op": "RECIP", "args": ["s"]}), "dtype": "float32"},
        {"type": "ENDFOR", "idx": "_gid1"},
        {"type": "ENDFOR", "idx": "_gid0"},
    ]}
    rt = ca.HipRuntime()
    r = ca.HipRenderer()
    src = r.render_kernel(item)
    # rows became wavefronts: the three row loops are strided by the 64 lanes, the two reductions end in a butterfly;
    # rows of at most 256 ... 2048 elements take copies of the body with 4 ... 32 counted passes, each behind a pass
    # that loads the row's elements of the input into registers once (the three loops then read those)
    assert src.count("for (int") == 27 and src.count("+=64") == 3 and "blockIdx.x" in src and "(n) <= 2048" in src
    assert src.count("_h0[_gid1_i] = val_x[((n*_gid0)+_gid1)];") == 6 and src.count("val_x[") == 6 + 3
    assert "m = ct_wave_max_f(m);" in src and "s = ct_wave_add_f(s);" in src
    r.compile_kernel([item])
    rows, n = 300, 77
    x = np.random.default_rng(1).normal(0, 3, (rows, n)).astype(np.float32)
    bx = make_buffer([rows, n], [n, 1], "float32", device=HipBuffer)
    by = make_buffer([rows, n], [n, 1], "float32", device=HipBuffer)
    open_buffer(rt, bx)
    open_buffer(rt, by)
    transfer_from_array(rt, bx, x)
    item["compiled_object"](None, by, rows, n, bx)
    got = transfer_into_array(by).reshape(rows, n)
    want = oracle.softmax(x)
    assert np.max(np.abs(got - want)) < 1e-6

    # LayerNorm as Caten lowers it (one kernel; normalization.lisp:39-58, test-scheduler.lisp:37-45): mean, then
    # biased variance of the centred row, then the affine output; scalar statements sit between the loops and
    # a per-row result (the mean) is also stored, which only one lane of the row's wavefront may do
    sub = lambda a, b: add(a, {"op": "NEG", "args": [b]})  # noqa: E731
    xi = A("val_x", idx)
    ln = {"name": "fused_layernorm", "blueprint": [
        {"type": "DEFINE-GLOBAL", "id": "val_y", "dtype": "float32", "pointer_p": True, "arg_type": "output", "nrank": 2},
        {"type": "DEFINE-GLOBAL", "id": "val_mean", "dtype": "float32", "pointer_p": True, "arg_type": "output", "nrank": 1},
        {"type": "DEFINE-GLOBAL", "id": "rows", "dtype": "int64", "pointer_p": False, "arg_type": "shape", "nrank": 0},
        {"type": "DEFINE-GLOBAL", "id": "n", "dtype": "int64", "pointer_p": False, "arg_type": "shape", "nrank": 0},
        {"type": "DEFINE-GLOBAL", "id": "val_x", "dtype": "float32", "pointer_p": True, "arg_type": "input", "nrank": 2},
        {"type": "DEFINE-GLOBAL", "id": "val_g", "dtype": "float32", "pointer_p": True, "arg_type": "input", "nrank": 1},
        {"type": "DEFINE-GLOBAL", "id": "val_b", "dtype": "float32", "pointer_p": True, "arg_type": "input", "nrank": 1},
        {"type": "FOR", "idx": "_gid0", "upfrom": 0, "below": lt("_gid0", "rows"), "by": 1},
        {"type": "EXPR", "writes": [A("s", None)], "expr": 0.0, "declare_type": True, "dtype": "float32"},
        {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": lt("_gid1", "n"), "by": 1},
        {"type": "EXPR", "writes": [A("s", None)], "expr": add("s", xi), "dtype": "float32", "reduction": True},
        {"type": "ENDFOR", "idx": "_gid1"},
        {"type": "EXPR", "writes": [A("u", None)], "declare_type": True, "dtype": "float32",
         "expr": mul("s", {"op": "RECIP", "args": [{"op": "CAST", "dtype": "float32", "args": ["n"]}]})},
        {"type": "EXPR", "writes": [A("val_mean", "_gid0")], "expr": "u", "dtype": "float32"},
        {"type": "EXPR", "writes": [A("q", None)], "expr": 0.0, "declare_type": True, "dtype": "float32"},
        {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": lt("_gid1", "n"), "by": 1},
        {"type": "EXPR", "writes": [A("q", None)], "expr": add("q", mul(sub(xi, "u"), sub(xi, "u"))), "dtype": "float32",
         "reduction": True},
        {"type": "ENDFOR", "idx": "_gid1"},
        {"type": "EXPR", "writes": [A("r", None)], "declare_type": True, "dtype": "float32",
         "expr": {"op": "RECIP", "args": [{"op": "SQRT", "args": [add(mul("q", {"op": "RECIP", "args": [
             {"op": "CAST", "dtype": "float32", "args": ["n"]}]}), 1e-5)]}]}},
        {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": lt("_gid1", "n"), "by": 1},
        {"type": "EXPR", "writes": [A("val_y", idx)], "dtype": "float32",
         "expr": add(mul(mul(sub(xi, "u"), "r"), A("val_g", "_gid1")), A("val_b", "_gid1"))},
        {"type": "ENDFOR", "idx": "_gid1"},
        {"type": "ENDFOR", "idx": "_gid0"},
    ]}
    # a row sum whose accumulator does NOT start at the operation's identity: lane partials would each carry the
    # offset, so the row must stay in one thread
    off = {"name": "offset_rowsum", "blueprint": [
        {"type": "DEFINE-GLOBAL", "id": "val_o", "dtype": "float32", "pointer_p": True, "arg_type": "output", "nrank": 1},
        {"type": "DEFINE-GLOBAL", "id": "rows", "dtype": "int64", "pointer_p": False, "arg_type": "shape", "nrank": 0},
        {"type": "DEFINE-GLOBAL", "id": "n", "dtype": "int64", "pointer_p": False, "arg_type": "shape", "nrank": 0},
        {"type": "DEFINE-GLOBAL", "id": "val_x", "dtype": "float32", "pointer_p": True, "arg_type": "input", "nrank": 2},
        {"type": "FOR", "idx": "_gid0", "upfrom": 0, "below": lt("_gid0", "rows"), "by": 1},
        {"type": "EXPR", "writes": [A("s", None)], "expr": 2.5, "declare_type": True, "dtype": "float32"},
        {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": lt("_gid1", "n"), "by": 1},
        {"type": "EXPR", "writes": [A("s", None)], "expr": add("s", xi), "dtype": "float32", "reduction": True},
        {"type": "ENDFOR", "idx": "_gid1"},
        {"type": "EXPR", "writes": [A("val_o", "_gid0")], "expr": "s", "dtype": "float32"},
        {"type": "ENDFOR", "idx": "_gid0"},
    ]}
    r2 = ca.HipRenderer()
    src_ln, src_off = r2.render_kernel(ln), r2.render_kernel(off)
    assert src_ln.count("+=64") == 3 and src_ln.count("if (_lane == 0) { val_mean[_gid0] = u; }") == 7
    assert "_lane" not in src_off and "+=64" not in src_off
    r2.compile_kernel([ln, off])
    for rows, n in ((300, 77), (5, 768), (64, 1)):
        x = np.random.default_rng(rows).normal(0.5, 3, (rows, n)).astype(np.float32)
        g = np.random.default_rng(2).normal(1, 0.1, n).astype(np.float32)
        b = np.random.default_rng(3).normal(0, 0.1, n).astype(np.float32)
        bufs = {}
        for name, shape, arr in (("x", [rows, n], x), ("g", [n], g), ("b", [n], b), ("y", [rows, n], None),
                                 ("mean", [rows], None), ("o", [rows], None)):
            strides = [n, 1] if len(shape) == 2 else [1]
            bufs[name] = make_buffer(shape, strides, "float32", device=HipBuffer)
            open_buffer(rt, bufs[name])
            if arr is not None:
                transfer_from_array(rt, bufs[name], arr)
        ln["compiled_object"](None, bufs["y"], bufs["mean"], rows, n, bufs["x"], bufs["g"], bufs["b"])
        off["compiled_object"](None, bufs["o"], rows, n, bufs["x"])
        got = transfer_into_array(bufs["y"]).reshape(rows, n)
        want = oracle.layernorm(x, g, b)
        assert np.max(np.abs(got - want)) < 2e-5
        assert np.allclose(transfer_into_array(bufs["mean"]), x.mean(axis=1), rtol=1e-5, atol=1e-5)
        assert np.allclose(transfer_into_array(bufs["o"]), 2.5 + x.sum(axis=1, dtype=np.float64), rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize("n", [768, 700, 64, 5])
def test_rendered_softmax_static_shape(oracle, n):
    """A static-shape row reduction is rendered as counted, unrolled loops: a lane owns four consecutive elements per
    pass when the row is whole quads, at least one per lane (the compiler merges them into 128-bit accesses), one
    element per pass otherwise; ragged rows get a guard.  The result must equal the dynamic-shape kernel's, i.e.
    the oracle's softmax."""
    import caten_amd as ca
    from caten_amd import blueprints
    from caten_amd.buffer import HipBuffer, make_buffer, open_buffer, transfer_from_array, transfer_into_array
    rows = 130
    item = blueprints.softmax_rows("fused_softmax_static", rows, n)
    rt = ca.HipRuntime()
    r = ca.HipRenderer()
    src = r.render_kernel(item)
    if n % 4 == 0 and n // 4 >= 64:
        quads = n // 4
        trips = (quads + 63) // 64
        # three loops over the row, behind one of the same shape that loads the row into registers
        assert src.count("#pragma unroll") == 8 and src.count(f"_gid1_i<{trips};") == 4 and src.count("_gid1_k<4;") == 4
        assert (f"_gid1_q=_lane+64*_gid1_i<{quads};" in src) == (quads % 64 != 0)
        assert src.count("_h0[_gid1_i][_gid1_k] = val_x[") == 1 and src.count("val_x[") == 1
    else:
        trips = (n + 63) // 64
        assert src.count("#pragma unroll") == 4 and src.count(f"_gid1_i<{trips};") == 4
        assert (f"if (_gid1<{n})" in src) == (n % 64 != 0)
        assert src.count("_h0[_gid1_i] = val_x[") == 1 and src.count("val_x[") == 1
    r.compile_kernel([item])
    x = np.random.default_rng(n).normal(0, 3, (rows, n)).astype(np.float32)
    bx = make_buffer([rows, n], [n, 1], "float32", device=HipBuffer)
    by = make_buffer([rows, n], [n, 1], "float32", device=HipBuffer)
    open_buffer(rt, bx)
    open_buffer(rt, by)
    transfer_from_array(rt, bx, x)
    item["compiled_object"](None, by, bx)
    got = transfer_into_array(by).reshape(rows, n)
    # the reference's own softmax tolerance (test-llm.lisp:64-80): the lanes add a 5000-element row in another order
    assert np.allclose(got, oracle.softmax(x), atol=1e-5, rtol=1e-6)


def test_rendered_argmax_with_index_components(oracle):
    """ArgMax as Caten lowers it (high-level-ops.lisp:314-343): the row maximum, then the maximum over the row of
    where(x == max, (N - 1) - index, 0) with the index from :INDEX-COMPONENTS, and N - that - 1 cast to int64 --
    the lowest index among ties.  Rendered, compiled, run; checked against the oracle's argmax."""
    import caten_amd as ca
    from caten_amd.buffer import HipBuffer, make_buffer, open_buffer, transfer_from_array, transfer_into_array
    A = lambda id_, idx: {"op": "AREF", "id": id_, "index": idx}  # noqa: E731
    add = lambda *a: {"op": "ADD", "args": list(a)}  # noqa: E731
    mul = lambda *a: {"op": "MUL", "args": list(a)}  # noqa: E731
    lt = lambda a, b: {"op": "<", "args": [a, b]}  # noqa: E731
    neg = lambda a: {"op": "NEG", "args": [a]}  # noqa: E731
    rows, n = 37, 500
    idx = add(mul(n, "_gid0"), "_gid1")
    # the column index of the element: the row axis has stride 0 in this index space
    col = {"op": "CAST", "dtype": "float32",
           "args": [None, {"op": "INDEX-COMPONENTS", "shape": [rows, n], "strides": [0, 1], "iterations": ["_gid0", "_gid1"]}]}
    eq = {"op": "NOT", "args": [{"op": "!=", "args": [None, A("val_x", idx), "m"]}]}
    item = {"name": "fused_argmax", "blueprint": [
        {"type": "DEFINE-GLOBAL", "id": "val_out", "dtype": "int64", "pointer_p": True, "arg_type": "output", "nrank": 1},
        {"type": "DEFINE-GLOBAL", "id": "val_x", "dtype": "float32", "pointer_p": True, "arg_type": "input", "nrank": 2},
        {"type": "FOR", "idx": "_gid0", "upfrom": 0, "below": lt("_gid0", rows), "by": 1},
        {"type": "EXPR", "writes": [A("m", None)], "expr": float("-inf"), "declare_type": True, "dtype": "float32"},
        {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": lt("_gid1", n), "by": 1},
        {"type": "EXPR", "writes": [A("m", None)], "expr": {"op": "MAX", "args": ["m", A("val_x", idx)]}, "dtype": "float32", "reduction": True},
        {"type": "ENDFOR", "idx": "_gid1"},
        {"type": "EXPR", "writes": [A("best", None)], "expr": 0.0, "declare_type": True, "dtype": "float32"},
        {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": lt("_gid1", n), "by": 1},
        {"type": "EXPR", "writes": [A("best", None)], "dtype": "float32", "reduction": True,
         "expr": {"op": "MAX", "args": ["best", {"op": "WHERE", "args": [eq, add(float(n - 1), neg(col)), 0.0]}]}},
        {"type": "ENDFOR", "idx": "_gid1"},
        {"type": "EXPR", "writes": [A("val_out", "_gid0")], "dtype": "int64",
         "expr": {"op": "CAST", "dtype": "int64", "args": [None, add(add(float(n), neg("best")), -1.0)]}},
        {"type": "ENDFOR", "idx": "_gid0"},
    ]}
    rt = ca.HipRuntime()
    r = ca.HipRenderer()
    src = r.render_kernel(item)
    assert "(1*_gid1)" in src and "ct_wave_max_f(best)" in src  # index components; both reductions one wavefront per row
    r.compile_kernel([item])
    rng = np.random.default_rng(3)
    x = rng.integers(-5, 6, (rows, n)).astype(np.float32)  # many ties: the lowest index must win
    bx = make_buffer([rows, n], [n, 1], "float32", device=HipBuffer)
    bo = make_buffer([rows], [1], "int64", device=HipBuffer)
    open_buffer(rt, bx)
    open_buffer(rt, bo)
    transfer_from_array(rt, bx, x)
    item["compiled_object"](None, bo, bx)
    got = transfer_into_array(bo).reshape(rows)
    assert np.array_equal(got, np.argmax(x, axis=1))
    assert np.array_equal(got, np.asarray([oracle.argmax(row) for row in x]).reshape(rows))


# ------------------------------------------------------------------ programs routed to the hand-written kernels
def _run_item(ca, item, arg_values):
    """render -> compile -> call one Schedule-Item the way realize-node :JIT_KERNEL does; arg_values in DEFINE-GLOBAL
    order, arrays become device buffers.  Returns (outputs as arrays, the program)."""
    from caten_amd.buffer import make_buffer, HipBuffer, open_buffer, transfer_from_array, transfer_into_array, close_buffer
    rt = ca.HipRuntime()
    r = ca.HipRenderer()
    r.render_kernel(item)
    r.compile_kernel([item])
    prog = item["compiled_object"]
    args, bufs = [], []
    globs = [n for n in item["blueprint"] if n["type"] == "DEFINE-GLOBAL"]
    for g, v in zip(globs, arg_values):
        if isinstance(v, np.ndarray):
            shape = list(v.shape)
            stride = [int(np.prod(shape[k + 1:])) for k in range(len(shape))]
            b = make_buffer(shape, stride, g["dtype"], device=HipBuffer)
            open_buffer(rt, b)
            transfer_from_array(rt, b, v.ravel())
            bufs.append(b)
            args.append(b)
        else:
            args.append(v)
    prog(None, *args)
    outs = [transfer_into_array(b).reshape(b.shape) for g, b in zip(globs, args) if g["arg_type"] == "output" and hasattr(b, "shape") and b.nrank > 0]
    for b in bufs:
        close_buffer(rt, b)
    return outs, prog


def test_matmul_item_runs_the_mfma_gemm(oracle):
    """The 1024^3 matmul configuration through the plug-in path: the blueprint of (caten (!relu (!matmul a b))) at 1024^3 is
    recognised and the launch goes to the MFMA GEMM, not to the rendered thread-per-output kernel; the result is
    the oracle's (rtol 1e-3 / atol 1e-4); with routes switched off the rendered kernel gives the same."""
    import caten_amd as ca
    from caten_amd import blueprints as bp, _lib
    rng = np.random.default_rng(0)
    M = N = K = 1024
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    out0 = np.zeros((M, N), np.float32)
    print("case: routed matmul 1024^3", flush=True)
    (got,), prog = _run_item(ca, bp.matmul(relu=True), [out0, M, N, K, A, B])
    assert prog.last_route == "cthip_matmul"
    want = np.maximum(A.astype(np.float64) @ B.astype(np.float64), 0.0)
    assert np.all(np.abs(got - want) <= 1e-4 + 1e-3 * np.abs(want))
    sub = oracle.matmul(A[:16], B, relu=True)  # the oracle's serial fp32 accumulation on a few rows
    assert np.all(np.abs(got[:16] - sub) <= 1e-4 + 1e-3 * np.abs(sub))
    # the rendered kernel (routes off) on a smaller case, same function
    lib = _lib.load()
    _lib.check(lib.cthip_set_option(b"render_routes", 0))
    try:
        (g2,), prog2 = _run_item(ca, bp.matmul(relu=True), [np.zeros((70, 50), np.float32), 70, 50, 33, A[:70, :33].copy(), B[:33, :50].copy()])
        assert prog2.last_route == "rendered"
    finally:
        _lib.check(lib.cthip_set_option(b"render_routes", 1))
    (g3,), prog3 = _run_item(ca, bp.matmul(relu=True), [np.zeros((70, 50), np.float32), 70, 50, 33, A[:70, :33].copy(), B[:33, :50].copy()])
    assert prog3.last_route == "cthip_matmul"
    assert np.all(np.abs(g2 - g3) <= 1e-4 + 1e-3 * np.abs(g3))


@pytest.mark.parametrize("M", [1, 5, 64, 130])
def test_linear_item_through_a_transposed_view(oracle, M):
    """x @ W^T + b with W (out, in) read through a transposed view (nn/linear.lisp:3-17), ReLU fused
    (test-scheduler.lisp:140-163): fewer than eight rows go to the single-row kernels, more to the GEMM."""
    import caten_amd as ca
    from caten_amd import blueprints as bp
    print(f"case: routed linear m={M}", flush=True)
    rng = np.random.default_rng(M)
    N, K = 300, 768
    X = rng.normal(0, 1, (M, K)).astype(np.float32)
    W = rng.normal(0, 0.05, (N, K)).astype(np.float32)
    b = rng.normal(0, 1, N).astype(np.float32)
    (got,), prog = _run_item(ca, bp.matmul(bias=True, relu=True, transposed_b=True), [np.zeros((M, N), np.float32), M, N, K, X, W, b])
    assert prog.last_route == "cthip_linear"
    want = oracle.relu(oracle.linear(X, W, b))
    assert np.all(np.abs(got - want) <= 1e-4 + 1e-3 * np.abs(want))


def test_matmul_item_with_another_layout_falls_back_to_its_rendered_kernel(oracle):
    """The route is checked against the actual index arithmetic at every launch: an A that is read with a row
    stride of 2*k (every other row of a taller matrix) is not what the GEMM takes, so the rendered kernel runs."""
    import caten_amd as ca
    from caten_amd import blueprints as bp
    item = bp.matmul()
    red = item["blueprint"][-5]["expr"]["args"][1]["args"][0]  # the aref of val_a
    red["index"] = {"op": "ADD", "args": [{"op": "MUL", "args": [{"op": "MUL", "args": [2, "kk"]}, "_gid0"]}, "_gid2"]}
    rng = np.random.default_rng(3)
    M, N, K = 20, 30, 40
    A2 = rng.uniform(-1, 1, (2 * M, K)).astype(np.float32)
    B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    (got,), prog = _run_item(ca, item, [np.zeros((M, N), np.float32), M, N, K, A2, B])
    assert item["route"] == "matmul" and prog.last_route == "rendered"
    assert np.allclose(got, oracle.matmul(A2[::2].copy(), B), rtol=1e-3, atol=1e-4)


def test_embedding_item_becomes_a_gather(oracle):
    """The one-hot masked sum over the vocabulary (nn/embedding.lisp:13-25) is launched as a row gather; ids that
    equal no row (out of range, fractional) select nothing, as in the sum."""
    import caten_amd as ca
    from caten_amd import blueprints as bp
    rng = np.random.default_rng(5)
    V, D = 5003, 96
    W = rng.normal(0, 1, (V, D)).astype(np.float32)
    idx = np.array([0, 17, 5002, 4, 4, 5003, -1, 2.5, 1234], np.float32)
    (got,), prog = _run_item(ca, bp.embedding_onehot(), [np.zeros((idx.size, D), np.float32), idx.size, D, V, idx, W])
    assert prog.last_route == "cthip_embedding"
    assert np.array_equal(got, oracle.embedding_onehot(W, idx))


def test_argmax_item(oracle):
    """ArgMaxNode (high-level-ops.lisp:314-325) routed to the argmax kernel: lowest index among ties, int64 result;
    the rendered two-reduction kernel agrees."""
    import caten_amd as ca
    from caten_amd import blueprints as bp, _lib
    rng = np.random.default_rng(9)
    R, N = 7, 50257
    x = rng.normal(0, 1, (R, N)).astype(np.float32)
    x[1, 777] = x[1, 40000] = 9.0   # a tie: the lower index wins
    x[2, 0] = 11.0
    x[3, N - 1] = 11.0
    (got,), prog = _run_item(ca, bp.argmax_rows(), [np.zeros(R, np.int64), R, N, x])
    assert prog.last_route == "cthip_argmax"
    want = np.array([int(oracle.argmax(row)) for row in x], np.int64)
    assert np.array_equal(got, want) and got[1] == 777 and got[2] == 0 and got[3] == N - 1
    lib = _lib.load()
    _lib.check(lib.cthip_set_option(b"render_routes", 0))
    try:
        (g2,), prog2 = _run_item(ca, bp.argmax_rows(), [np.zeros(R, np.int64), R, N, x])
    finally:
        _lib.check(lib.cthip_set_option(b"render_routes", 1))
    assert prog2.last_route == "rendered" and np.array_equal(g2, want)


def test_softmax_item_with_dynamic_shape(oracle):
    import caten_amd as ca
    from caten_amd import blueprints as bp
    rng = np.random.default_rng(2)
    x = (10 + 100 * rng.normal(0, 1, (300, 777))).astype(np.float32)
    (got,), prog = _run_item(ca, bp.softmax_rows(), [np.zeros_like(x), 300, 777, x])
    assert prog.last_route == "cthip_softmax"
    want = oracle.softmax(x)
    assert np.allclose(got, want, rtol=1e-5, atol=1e-5) and np.allclose(got.sum(-1), 1.0, atol=1e-5)


@pytest.mark.parametrize("static", [False, True])
def test_layernorm_and_rmsnorm_items_are_routed(oracle, static):
    """LayerNorm / RMSNorm rows lowered as one kernel each (nn/normalization.lisp:39-58,78-92) go to the row
    kernels; eps is read off the item.  The same items with routing switched off run their rendered kernels, and
    an item that also stores the row mean is not a LayerNorm the row kernel can stand in for."""
    import copy
    import caten_amd as ca
    from caten_amd import blueprints as bp, _lib
    rows, n = 37, 768
    rng = np.random.default_rng(9)
    x = rng.normal(0.5, 3, (rows, n)).astype(np.float32)
    g = rng.normal(1, 0.1, n).astype(np.float32)
    b = rng.normal(0, 0.1, n).astype(np.float32)
    shape = dict(rows=rows, n=n) if static else {}
    dyn = [] if static else [rows, n]
    y0 = np.zeros_like(x)
    cases = [
        (bp.layernorm_rows(eps=1e-5, **shape), [y0, *dyn, x, g, b], "cthip_layernorm", oracle.layernorm(x, g, b, eps=1e-5)),
        (bp.layernorm_rows(affine=False, eps=1e-3, **shape), [y0, *dyn, x], "cthip_layernorm",
         oracle.layernorm(x, np.ones(n, np.float32), np.zeros(n, np.float32), eps=1e-3)),
        (bp.rmsnorm_rows(eps=1e-6, **shape), [y0, *dyn, x, g], "cthip_rmsnorm", oracle.rmsnorm(x, g, eps=1e-6)),
        (bp.rmsnorm_rows(weight=False, eps=1e-5, **shape), [y0, *dyn, x], "cthip_rmsnorm",
         oracle.rmsnorm(x, np.ones(n, np.float32), eps=1e-5)),
    ]
    lib = _lib.load()
    for item, args, route, want in cases:
        (got,), prog = _run_item(ca, copy.deepcopy(item), args)
        assert prog.last_route == route, (item["name"], prog.last_route)
        assert np.max(np.abs(got - want)) < 2e-5
        _lib.check(lib.cthip_set_option(b"render_routes", 0))
        try:
            (got2,), prog2 = _run_item(ca, copy.deepcopy(item), args)
        finally:
            _lib.check(lib.cthip_set_option(b"render_routes", 1))
        assert prog2.last_route == "rendered" and np.max(np.abs(got2 - want)) < 2e-5
    # variations that are not the norm: the mean is also stored / the variance is not of the centred row
    ln = bp.layernorm_rows(**shape)
    k = next(i for i, nd in enumerate(ln["blueprint"]) if nd.get("writes") and nd["writes"][0]["id"] == "q")
    ln["blueprint"].insert(k, {"type": "EXPR", "writes": [{"op": "AREF", "id": "val_y", "index": "_gid0"}], "expr": "u", "dtype": "float32"})
    r = ca.HipRenderer()
    r.render_kernel(ln)
    r.compile_kernel([ln])
    assert ln["route"] == "rendered"
    bad = bp.layernorm_rows(**shape)
    for nd in bad["blueprint"]:
        if nd.get("reduction") and nd["writes"][0]["id"] == "q":
            xi = nd["expr"]["args"][1]["args"][0]["args"][0]
            nd["expr"] = {"op": "ADD", "args": ["q", {"op": "MUL", "args": [xi, xi]}]}  # sum of x^2, not of (x - u)^2
    r.render_kernel(bad)
    r.compile_kernel([bad])
    assert bad["route"] == "rendered"


def test_rank0_output_passed_by_pointer_is_written_back():
    """A rank-0 OUTPUT is declared as a pointer (rewriting-rules.lisp:207-231); CLANG boxes the Lisp number in a
    one-element foreign object and stores the result back into the buffer (clang.lisp:166-185).  Here the box is a
    device cell: the kernel writes it, the caller reads it back into the buffer's value."""
    import caten_amd as ca
    from caten_amd import blueprints as bp
    from caten_amd.buffer import make_buffer, HipBuffer, open_buffer, transfer_from_array, close_buffer
    A = lambda id_, idx: {"op": "AREF", "id": id_, "index": idx}  # noqa: E731
    item = {"name": "sum_all", "blueprint": [
        bp._glob("val_s", "output", 0) | {"pointer_p": True}, bp._glob("n", "shape", 0, "int64"), bp._glob("val_x", "input", 1),
        {"type": "EXPR", "writes": [A("acc", None)], "expr": 0.0, "declare_type": True, "dtype": "float32"},
        {"type": "FOR", "idx": "_gid0", "upfrom": 0, "below": bp._lt("_gid0", "n"), "by": 1},
        {"type": "EXPR", "writes": [A("acc", None)], "expr": {"op": "ADD", "args": ["acc", A("val_x", "_gid0")]}, "dtype": "float32", "reduction": True},
        {"type": "ENDFOR", "idx": "_gid0"},
        {"type": "EXPR", "writes": [A("val_s", 0)], "expr": {"op": "ADD", "args": ["acc", A("val_s", 0)]}, "dtype": "float32"},
    ]}
    rt = ca.HipRuntime()
    r = ca.HipRenderer()
    r.render_kernel(item)
    r.compile_kernel([item])
    x = make_buffer([100], [1], "float32", device=HipBuffer)
    open_buffer(rt, x)
    transfer_from_array(rt, x, np.arange(100, dtype=np.float32))
    s = make_buffer([], [], "float32", value=0.5, device=HipBuffer)
    item["compiled_object"](None, s, 100, x)
    assert s.value == 4950.5  # the incoming value went in, the result came back
    close_buffer(rt, x)


@pytest.mark.parametrize("rows,n", [(1, 1), (37, 1000), (256, 64)])
def test_item_with_an_explicit_grid_launches_on_that_grid(rows, n):
    """An item the auto-scheduler marked GLOBAL (directive.lisp:94-117): indices are blockIdx * local + threadIdx with
    a bounds IF, the launch takes ceil(size / local) blocks from the ExprGrid expressions (2-D here)."""
    import caten_amd as ca
    from caten_amd import blueprints as bp
    print(f"case: explicit grid {rows}x{n}", flush=True)
    rng = np.random.default_rng(rows)
    x = rng.standard_normal((rows, n)).astype(np.float32)
    y = rng.standard_normal((rows, n)).astype(np.float32)
    (got,), prog = _run_item(ca, bp.add_global_2d(), [np.full((rows, n), np.nan, np.float32), rows, n, x, y])
    assert prog.last_route == "rendered"
    assert np.array_equal(got, x + y)


def test_conv2d_and_maxpool_items(oracle):
    """relu(conv2d + bias) (nn/conv.lisp) and 2x2 max-pool (nn/pool.lisp) as their static loop nests: output
    positions across threads, window reductions serial in the thread; against NumPy in fp64."""
    import caten_amd as ca
    from caten_amd import blueprints as bp
    print("case: conv2d / maxpool items", flush=True)
    rng = np.random.default_rng(0)
    N, Cc, H, W, K, R, S = 3, 5, 17, 19, 7, 3, 4
    x = rng.standard_normal((N, Cc, H, W)).astype(np.float32)
    w = (0.2 * rng.standard_normal((K, Cc, R, S))).astype(np.float32)
    b = rng.standard_normal(K).astype(np.float32)
    OH, OW = H - R + 1, W - S + 1
    (got,), _ = _run_item(ca, bp.conv2d_relu(N, Cc, H, W, K, R, S), [np.zeros((N, K, OH, OW), np.float32), x, w, b])
    win = np.lib.stride_tricks.sliding_window_view(x.astype(np.float64), (R, S), axis=(2, 3))  # N C OH OW R S
    want = np.maximum(np.einsum("nchwrs,kcrs->nkhw", win, w.astype(np.float64)) + b[None, :, None, None], 0.0)
    assert np.all(np.abs(got - want) <= 1e-4 + 1e-3 * np.abs(want))
    H2, W2 = 16, 18
    xp = rng.standard_normal((N, Cc, H2, W2)).astype(np.float32)
    (gp,), _ = _run_item(ca, bp.maxpool2x2(N, Cc, H2, W2), [np.zeros((N, Cc, H2 // 2, W2 // 2), np.float32), xp])
    assert np.array_equal(gp, xp.reshape(N, Cc, H2 // 2, 2, W2 // 2, 2).max(axis=(3, 5)))


@pytest.mark.parametrize("m,n", [(1, 5), (130, 300), (1000, 64)])
def test_backward_item_with_a_first_axis_reduction(m, n):
    """The backward of relu(x W^T + b) with respect to the pre-activation and the bias: dz = dy * (y > 0) and
    db = dz.sum(axis 0) in one item; the batch loop is the reduction, taken by the lanes of a wavefront."""
    import caten_amd as ca
    from caten_amd import blueprints as bp
    print(f"case: relu/bias backward {m}x{n}", flush=True)
    rng = np.random.default_rng(m)
    y = np.maximum(rng.standard_normal((m, n)), 0).astype(np.float32)
    dy = rng.standard_normal((m, n)).astype(np.float32)
    (dz, db), _ = _run_item(ca, bp.linear_relu_backward(), [np.zeros((m, n), np.float32), np.zeros(n, np.float32), m, n, dy, y])
    want = np.where(y > 0, dy, 0).astype(np.float32)
    assert np.array_equal(dz, want)
    assert np.allclose(db, want.astype(np.float64).sum(0), rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("rows,n", [(300, 77), (4, 256), (4, 257), (7, 512), (7, 513), (6, 768), (6, 769), (9, 1024), (9, 1025),
                                     (3, 1536), (3, 1537), (5, 2048), (3, 2049), (2, 5000), (64, 1)])
def test_rendered_softmax_dynamic_rows_short_and_long(oracle, rows, n):
    """The softmax blueprint RENDERED (routes switched off) with a row length known only at launch: rows of at most
    256 ... 2048 elements run a copy of the body whose row loops are 4 ... 32 counted passes with clamped,
    unconditional reads and guarded effects (the row is read once), longer rows the lane-strided loops; all against
    the oracle, on both sides of every boundary."""
    import caten_amd as ca
    from caten_amd import _lib, blueprints as bp
    print(f"case: rendered dynamic softmax {rows}x{n}", flush=True)
    lib = _lib.load()
    x = np.random.default_rng(n).normal(0, 3, (rows, n)).astype(np.float32)
    _lib.check(lib.cthip_set_option(b"render_routes", 0))
    try:
        (got,), prog = _run_item(ca, bp.softmax_rows(), [np.zeros((rows, n), np.float32), rows, n, x])
        assert prog.last_route == "rendered"
    finally:
        _lib.check(lib.cthip_set_option(b"render_routes", 1))
    # the reference's own softmax tolerance (test-llm.lisp:64-80): the lanes add a 5000-element row in another order
    assert np.allclose(got, oracle.softmax(x), atol=1e-5, rtol=1e-6)


@pytest.mark.parametrize("rows,n", [(5, 77), (3, 256), (4, 300), (2, 2048), (2, 2100)])
def test_rendered_dynamic_rows_with_an_update_in_place_and_two_inputs(rows, n):
    """Two loops over a row of run-time length: s = sum_j x[j] * g[j], then y[j] = y[j] + s * x[j].  The counted
    passes hold x and g in registers (loaded once), and the second loop's store reads the array it writes, so it
    has to stay guarded: a pass beyond the row must not add to the row's last element a second time."""
    import caten_amd as ca
    from caten_amd import _lib
    print(f"case: rendered dynamic update in place {rows}x{n}", flush=True)
    A = lambda id_, idx: {"op": "AREF", "id": id_, "index": idx}  # noqa: E731
    add = lambda *a: {"op": "ADD", "args": list(a)}  # noqa: E731
    mul = lambda *a: {"op": "MUL", "args": list(a)}  # noqa: E731
    lt = lambda a, b: {"op": "<", "args": [a, b]}  # noqa: E731
    idx = add(mul("n", "_gid0"), "_gid1")
    item = {"name": "fused_axpy_rows", "blueprint": [
        {"type": "DEFINE-GLOBAL", "id": "val_y", "dtype": "float32", "pointer_p": True, "arg_type": "output", "nrank": 2},
        {"type": "DEFINE-GLOBAL", "id": "rows", "dtype": "int64", "pointer_p": False, "arg_type": "shape", "nrank": 0},
        {"type": "DEFINE-GLOBAL", "id": "n", "dtype": "int64", "pointer_p": False, "arg_type": "shape", "nrank": 0},
        {"type": "DEFINE-GLOBAL", "id": "val_x", "dtype": "float32", "pointer_p": True, "arg_type": "input", "nrank": 2},
        {"type": "DEFINE-GLOBAL", "id": "val_g", "dtype": "float32", "pointer_p": True, "arg_type": "input", "nrank": 1},
        {"type": "FOR", "idx": "_gid0", "upfrom": 0, "below": lt("_gid0", "rows"), "by": 1},
        {"type": "EXPR", "writes": [A("s", None)], "expr": 0.0, "declare_type": True, "dtype": "float32"},
        {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": lt("_gid1", "n"), "by": 1},
        {"type": "EXPR", "writes": [A("s", None)], "expr": add("s", mul(A("val_x", idx), A("val_g", "_gid1"))), "dtype": "float32",
         "reduction": True},
        {"type": "ENDFOR", "idx": "_gid1"},
        {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": lt("_gid1", "n"), "by": 1},
        {"type": "EXPR", "writes": [A("val_y", idx)], "expr": add(A("val_y", idx), mul("s", A("val_x", idx))), "dtype": "float32"},
        {"type": "ENDFOR", "idx": "_gid1"},
        {"type": "ENDFOR", "idx": "_gid0"},
    ]}
    src = ca.HipRenderer().render_kernel(item)
    # both inputs held, the output (read and written) not; its store keeps the guard in the counted passes
    assert src.count("_h0[_gid1_i] = val_x[") == 6 and src.count("_h1[_gid1_i] = val_g[") == 6
    assert src.count("if (_gid1_ok) { val_y[") == 6
    rng = np.random.default_rng(n)
    x = rng.normal(0, 1, (rows, n)).astype(np.float32)
    g = rng.normal(0, 1, n).astype(np.float32)
    y0 = rng.normal(0, 1, (rows, n)).astype(np.float32)
    lib = _lib.load()
    _lib.check(lib.cthip_set_option(b"render_routes", 0))
    try:
        (got,), prog = _run_item(ca, item, [y0.copy(), rows, n, x, g])
        assert prog.last_route == "rendered"
    finally:
        _lib.check(lib.cthip_set_option(b"render_routes", 1))
    s = (x.astype(np.float64) * g).sum(-1, keepdims=True)
    want = y0 + s * x
    assert np.allclose(got, want, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("rows,n", [(1, 1), (5, 77), (3, 1024), (4, 256), (41, 25), (130, 300), (1, 1025)])
@pytest.mark.parametrize("static", [False, True])
def test_rendered_elementwise_items_four_elements_per_thread(rows, n, static):
    """Element-wise items (no loop inside the parallel ones): a thread takes four elements 256 apart, whole blocks of
    1024 without a test and the last one with; operands whose index is the row-major position are addressed by the
    flat position, others (a bias along the row, a transposed read) through the indices taken apart.
    y[i][j] = x[i][j] * 2 + b[j] + xt[j][i]."""
    import caten_amd as ca
    from caten_amd import _lib
    print(f"case: rendered element-wise {rows}x{n} static={static}", flush=True)
    A = lambda id_, idx: {"op": "AREF", "id": id_, "index": idx}  # noqa: E731
    add = lambda *a: {"op": "ADD", "args": list(a)}  # noqa: E731
    mul = lambda *a: {"op": "MUL", "args": list(a)}  # noqa: E731
    lt = lambda a, b: {"op": "<", "args": [a, b]}  # noqa: E731
    R, N = (rows, n) if static else ("rows", "n")
    idx = add(mul(N, "_gid0"), "_gid1")
    idx_t = add(mul(R, "_gid1"), "_gid0")
    glob = lambda id_, ty, nr: {"type": "DEFINE-GLOBAL", "id": id_, "dtype": "float32", "pointer_p": True, "arg_type": ty, "nrank": nr}  # noqa: E731
    shape = [] if static else [
        {"type": "DEFINE-GLOBAL", "id": "rows", "dtype": "int64", "pointer_p": False, "arg_type": "shape", "nrank": 0},
        {"type": "DEFINE-GLOBAL", "id": "n", "dtype": "int64", "pointer_p": False, "arg_type": "shape", "nrank": 0}]
    item = {"name": "fused_affine_ew", "blueprint": [glob("val_y", "output", 2)] + shape + [
        glob("val_x", "input", 2), glob("val_b", "input", 1), glob("val_xt", "input", 2),
        {"type": "FOR", "idx": "_gid0", "upfrom": 0, "below": lt("_gid0", R), "by": 1},
        {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": lt("_gid1", N), "by": 1},
        {"type": "EXPR", "writes": [A("val_y", idx)], "expr": add(mul(A("val_x", idx), 2.0), A("val_b", "_gid1"), A("val_xt", idx_t)), "dtype": "float32"},
        {"type": "ENDFOR", "idx": "_gid1"},
        {"type": "ENDFOR", "idx": "_gid0"},
    ]}
    src = ca.HipRenderer().render_kernel(item)
    assert "val_x[_t]" in src and "val_y[_t] =" in src
    if rows > 1 and n > 1:  # (a 1 x n or n x 1 array read transposed IS read in row-major order)
        assert "val_b[_gid1]" in src and "val_xt[_t]" not in src
    assert "_e < 4" in src and "blockIdx.x * 1024" in src
    rng = np.random.default_rng(rows * 1000 + n)
    x = rng.normal(0, 1, (rows, n)).astype(np.float32)
    bias = rng.normal(0, 1, n).astype(np.float32)
    xt = rng.normal(0, 1, (n, rows)).astype(np.float32)
    lib = _lib.load()
    _lib.check(lib.cthip_set_option(b"render_routes", 0))
    try:
        args = [np.zeros((rows, n), np.float32)] + ([] if static else [rows, n]) + [x, bias, xt]
        (got,), prog = _run_item(ca, item, args)
        assert prog.last_route == "rendered"
    finally:
        _lib.check(lib.cthip_set_option(b"render_routes", 1))
    assert np.array_equal(got, (x * np.float32(2.0) + bias) + xt.T)


@pytest.mark.parametrize("ntok,d", [(5, 8), (300, 64), (17, 1000)])
def test_rendered_gather_keeps_its_indexed_read_behind_the_index(ntok, d):
    """An element-wise item whose read goes through a temporary of the body (row = (int) idx[i]; y[i][j] = W[row][j]):
    the reads hoisted in front of the statements are only those whose index is made of loop indices and shape
    arguments; W[row * d + j] has to stay where `row` is known."""
    import caten_amd as ca
    from caten_amd import _lib
    print(f"case: rendered gather {ntok}x{d}", flush=True)
    A = lambda id_, idx: {"op": "AREF", "id": id_, "index": idx}  # noqa: E731
    add = lambda *a: {"op": "ADD", "args": list(a)}  # noqa: E731
    mul = lambda *a: {"op": "MUL", "args": list(a)}  # noqa: E731
    lt = lambda a, b: {"op": "<", "args": [a, b]}  # noqa: E731
    glob = lambda id_, ty, nr, dt="float32": {"type": "DEFINE-GLOBAL", "id": id_, "dtype": dt, "pointer_p": nr > 0, "arg_type": ty, "nrank": nr}  # noqa: E731
    item = {"name": "fused_gather", "blueprint": [
        glob("val_y", "output", 2), glob("ntok", "shape", 0, "int64"), glob("d", "shape", 0, "int64"),
        glob("val_w", "input", 2), glob("val_i", "input", 1),
        {"type": "FOR", "idx": "_gid0", "upfrom": 0, "below": lt("_gid0", "ntok"), "by": 1},
        {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": lt("_gid1", "d"), "by": 1},
        {"type": "EXPR", "writes": [A("row", None)], "expr": {"op": "CAST", "dtype": "int64", "args": [A("val_i", "_gid0")]},
         "declare_type": True, "dtype": "int64"},
        {"type": "EXPR", "writes": [A("val_y", add(mul("d", "_gid0"), "_gid1"))], "expr": A("val_w", add(mul("d", "row"), "_gid1")), "dtype": "float32"},
        {"type": "ENDFOR", "idx": "_gid1"},
        {"type": "ENDFOR", "idx": "_gid0"},
    ]}
    src = ca.HipRenderer().render_kernel(item)
    assert "_e < 4" in src and "_h0[_e] = val_i[_gid0];" in src  # the index array is read ahead ...
    assert "] = val_w[" not in src.replace("val_y[_t] = val_w[", "") and "val_y[_t] = val_w[((d*row)+_gid1)];" in src  # ... the table is not
    rng = np.random.default_rng(ntok)
    vocab = 37
    w = rng.normal(0, 1, (vocab, d)).astype(np.float32)
    idx = rng.integers(0, vocab, ntok).astype(np.float32)
    lib = _lib.load()
    _lib.check(lib.cthip_set_option(b"render_routes", 0))
    try:
        (got,), prog = _run_item(ca, item, [np.zeros((ntok, d), np.float32), ntok, d, w, idx])
        assert prog.last_route == "rendered"
    finally:
        _lib.check(lib.cthip_set_option(b"render_routes", 1))
    assert np.array_equal(got, w[idx.astype(np.int64)])


@pytest.mark.parametrize("rows,n", [(3, 70), (5, 256), (2, 700)])
@pytest.mark.parametrize("static", [False, True])
def test_rendered_row_with_a_guarded_neighbour_read(rows, n, static):
    """s = sum_j x[j]; y[j] = s + (0 < j ? x[j - 1] : 0).  The read of the left neighbour is only valid where the
    `where` selects it (for j = 0 it lies in front of the row, for row 0 in front of the array): it has to stay
    inside the conditional, while x[j] itself is held in registers."""
    import caten_amd as ca
    from caten_amd import _lib
    print(f"case: rendered guarded neighbour {rows}x{n} static={static}", flush=True)
    A = lambda id_, idx: {"op": "AREF", "id": id_, "index": idx}  # noqa: E731
    add = lambda *a: {"op": "ADD", "args": list(a)}  # noqa: E731
    mul = lambda *a: {"op": "MUL", "args": list(a)}  # noqa: E731
    lt = lambda a, b: {"op": "<", "args": [a, b]}  # noqa: E731
    R, N = (rows, n) if static else ("rows", "n")
    idx = add(mul(N, "_gid0"), "_gid1")
    left = {"op": "WHERE", "args": [lt(0, "_gid1"), A("val_x", add(idx, -1)), 0.0]}
    glob = lambda id_, ty, nr, dt="float32": {"type": "DEFINE-GLOBAL", "id": id_, "dtype": dt, "pointer_p": nr > 0, "arg_type": ty, "nrank": nr}  # noqa: E731
    shape = [] if static else [glob("rows", "shape", 0, "int64"), glob("n", "shape", 0, "int64")]
    loop = {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": lt("_gid1", N), "by": 1}
    item = {"name": "fused_left_neighbour", "blueprint": [glob("val_y", "output", 2)] + shape + [
        glob("val_x", "input", 2),
        {"type": "FOR", "idx": "_gid0", "upfrom": 0, "below": lt("_gid0", R), "by": 1},
        {"type": "EXPR", "writes": [A("s", None)], "expr": 0.0, "declare_type": True, "dtype": "float32"},
        dict(loop),
        {"type": "EXPR", "writes": [A("s", None)], "expr": add("s", A("val_x", idx)), "dtype": "float32", "reduction": True},
        {"type": "ENDFOR", "idx": "_gid1"},
        dict(loop),
        {"type": "EXPR", "writes": [A("val_y", idx)], "expr": add("s", left), "dtype": "float32"},
        {"type": "ENDFOR", "idx": "_gid1"},
        {"type": "ENDFOR", "idx": "_gid0"},
    ]}
    src = ca.HipRenderer().render_kernel(item)
    assert "] = val_x[((" in src  # the row itself is held ...
    assert "+-1)]" in src and "] = val_x[(((" not in src  # ... its left neighbour is read where the `where` selects it
    rng = np.random.default_rng(n)
    x = rng.normal(0, 1, (rows, n)).astype(np.float32)
    lib = _lib.load()
    _lib.check(lib.cthip_set_option(b"render_routes", 0))
    try:
        args = [np.zeros((rows, n), np.float32)] + ([] if static else [rows, n]) + [x]
        (got,), prog = _run_item(ca, item, args)
        assert prog.last_route == "rendered"
    finally:
        _lib.check(lib.cthip_set_option(b"render_routes", 1))
    leftv = np.concatenate([np.zeros((rows, 1), np.float32), x[:, :-1]], axis=1)
    want = x.astype(np.float64).sum(-1, keepdims=True) + leftv
    assert np.allclose(got, want, rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize("rows,n,static", [(7, 768, True), (7, 768, False), (5, 77, True), (5, 77, False), (3, 1000, False), (2, 2500, False)])
def test_rendered_layernorm_softmax_in_one_item(oracle, rows, n, static):
    """LayerNorm -> softmax fused into one Schedule-Item (five loops over the row, three input arrays held in registers)
    against the oracle's LayerNorm followed by its softmax."""
    import caten_amd as ca
    from caten_amd import blueprints as bp
    print(f"case: rendered layernorm->softmax {rows}x{n} static={static}", flush=True)
    rng = np.random.default_rng(n + rows)
    x = rng.normal(0, 2, (rows, n)).astype(np.float32)
    g = rng.normal(1, 0.1, n).astype(np.float32)
    b = rng.normal(0, 0.1, n).astype(np.float32)
    item = bp.layernorm_softmax_rows("ln_sm", 1e-5, rows if static else None, n if static else None)
    args = [np.zeros((rows, n), np.float32)] + ([] if static else [rows, n]) + [x, g, b]
    (got,), prog = _run_item(ca, item, args)
    assert prog.last_route == "rendered"  # no hand-written kernel is recognised for the pair
    want = oracle.softmax(oracle.layernorm(x, g, b, 1e-5))
    assert np.allclose(got, want, atol=1e-5, rtol=1e-4)
