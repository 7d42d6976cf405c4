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


def _relu_matmul_graph(ca, M, N, K):
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
    return ca.HipRuntime(graph, fw_outputs=["out2"], renderer=r)


def test_vm_runs_a_rendered_kernel_with_dynamic_shapes(oracle):
    import caten_amd as ca
    from caten_amd.buffer import AbstractBuffer, make_buffer, transfer_into_array
    vm = _relu_matmul_graph(ca, 0, 0, 0)
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
        pools.append(vm.graph[2].attrs["pool"].value)
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
    # rows became wavefronts: the three row loops are strided by the 64 lanes, the two reductions end in a butterfly
    assert src.count("for (int") == 3 and src.count("+=64") == 3 and "blockIdx.x" in src
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
    assert src_ln.count("+=64") == 3 and "if (_lane == 0) { val_mean[_gid0] = u; }" in src_ln
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
    """A static-shape row reduction is rendered as counted, unrolled lane-strided loops (ragged rows get a guard on
    the element index); the result must equal the dynamic-shape kernel's, i.e. the oracle's softmax."""
    import caten_amd as ca
    from caten_amd import blueprints
    from caten_amd.buffer import HipBuffer, make_buffer, open_buffer, transfer_from_array, transfer_into_array
    rows = 130
    item = blueprints.softmax_rows("fused_softmax_static", rows, n)
    rt = ca.HipRuntime()
    r = ca.HipRenderer()
    src = r.render_kernel(item)
    trips = (n + 63) // 64
    assert src.count("#pragma unroll") == 3 and src.count(f"_gid1_i<{trips};") == 3
    assert (f"if (_gid1<{n})" in src) == (n % 64 != 0)
    r.compile_kernel([item])
    x = np.random.default_rng(n).normal(0, 3, (rows, n)).astype(np.float32)
    bx = make_buffer([rows, n], [n, 1], "float32", device=HipBuffer)
    by = make_buffer([rows, n], [n, 1], "float32", device=HipBuffer)
    open_buffer(rt, bx)
    open_buffer(rt, by)
    transfer_from_array(rt, bx, x)
    item["compiled_object"](None, by, bx)
    got = transfer_into_array(by).reshape(rows, n)
    assert np.max(np.abs(got - oracle.softmax(x))) < 1e-6


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
