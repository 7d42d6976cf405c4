"""CPU-side checks: the C-ABI library loads and exports every declared symbol, the host
mirror of Caten's backend interface behaves like the reference's, hipRTC compiles rendered
kernels for gfx950 without a device.  No compute is launched here."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    from caten_amd import _lib
    header = open(os.path.join(ROOT, "include", "caten_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(cthip_[a-z0-9_]+)\s*\(", header))
    assert declared, "no declarations found"
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} is declared in caten_hip.h but not exported"
    assert declared == set(_lib.PROTOTYPES), declared ^ set(_lib.PROTOTYPES)
    _lib.load()


def test_calls_fail_loudly_without_init():
    from caten_amd import _lib
    lib = _lib.load()
    if _lib.is_initialised():
        pytest.skip("a device is initialised in this process")
    p = ctypes.c_void_p()
    assert lib.cthip_alloc(ctypes.byref(p), 16) == -1
    assert b"cthip_init" in lib.cthip_last_error()
    assert lib.cthip_softmax(None, None, 1, 4) == -1
    # the walk of a node list and the paged cache entry points need a device too
    assert lib.cthip_vm_create(ctypes.byref(p), 4) == -1
    assert lib.cthip_vm_run(None) == -1
    assert lib.cthip_kv_append_paged(None, None, None, None, 0, 0, 64) == -1
    assert lib.cthip_kv_page_rows() == 64  # a constant of the layout: no device needed
    assert lib.cthip_vm_launches(None) == -1 and lib.cthip_vm_destroy(None) == 0


def test_backend_registry():
    import caten_amd as ca
    assert ca.get_backend_buffer("HIP") is ca.HipBuffer
    assert ca.get_backend_runtime(":hip") is ca.HipRuntime
    assert ca.get_backend_renderer("hip") is ca.HipRenderer
    assert ca.jit_mode_p("HIP") is True
    with pytest.raises(KeyError):
        ca.get_backend_buffer("CUDA")  # byoc/cuda.lisp is an empty stub in the reference too


def test_buffer_storage_size_and_views():
    from caten_amd.buffer import make_buffer, buffer_storage_size, HipBuffer
    b = make_buffer([3, 4], [4, 1], "float32", device=HipBuffer)
    assert buffer_storage_size(b) == 12 and b.nrank == 2
    b = make_buffer([3, 4], [0, 1], "float32", [(0, 3, 1, True), None])
    assert buffer_storage_size(b) == 4  # broadcast axis counts once (buffer.lisp:70-76)
    with pytest.raises(ValueError):
        make_buffer([3, True], [1, 1], "float32")
    with pytest.raises(ValueError):
        make_buffer([3], [1, 1], "float32")


class _StubLib:
    """Stands in for the C ABI's allocator and copies: hands out fake addresses, records every free and upload."""

    def __init__(self):
        self.next = 0x1000
        self.live = set()
        self.freed = []
        self.uploads = {}

    def cthip_alloc(self, out, nbytes):
        p = self.next
        self.next += 0x1000
        self.live.add(p)
        out._obj.value = p
        return 0

    def cthip_free(self, p):
        assert p in self.live, f"freeing {p:#x}, which is not a live block (double free or stale pointer)"
        self.live.discard(p)
        self.freed.append(p)
        return 0

    def cthip_h2d(self, dst, src, nbytes):
        self.uploads[dst] = bytes((ctypes.c_char * nbytes).from_address(src))
        return 0


@pytest.fixture
def stub_lib(monkeypatch):
    from caten_amd import _lib
    stub = _StubLib()
    monkeypatch.setattr(_lib, "load", lambda: stub)
    monkeypatch.setattr(_lib, "init", lambda device=0: stub)
    monkeypatch.setattr(_lib, "check", lambda status: None if status == 0 else (_ for _ in ()).throw(AssertionError(status)))
    return stub


def _view_node(nrank, shape, stride, broadcast=None):
    from caten_amd.runtime import Node
    reads = ["base"] + list(shape) + [0] * nrank + list(shape) + [1] * nrank + list(stride)
    return Node("View", ["v"], reads, {"nrank": nrank, "broadcast": broadcast or [False] * nrank})


def test_views_do_not_own_storage(stub_lib):
    """A :View shares its base's storage (copy-buffer, buffer.lisp:60-68): free-runtime releases every block once,
    and a view of a pool that a dynamic shape closed holds no pointer a later owner could lose."""
    from caten_amd.runtime import GraphRuntime, Node
    from caten_amd.buffer import HipBuffer

    class RT(GraphRuntime):
        buffer_type = HipBuffer

    alloc = Node("Allocate", ["base"], ["n", 4, 4, 1], {"nrank": 2, "dtype": "float32"})
    rt = RT([alloc, _view_node(2, ["n", 4], [4, 1])], ["v"])
    v = rt.forward(("n", 3))
    base = rt.getvar("base")
    assert v.value == base.value and not v.owns_storage and base.owns_storage
    first = base.value
    # the dynamic shape changes: the pool is closed and re-opened; the old view points nowhere
    v2 = rt.forward(("n", 5))
    assert stub_lib.freed == [first]
    assert v.value is None
    assert v2.value == rt.getvar("base").value != first
    rt.free()  # the base and its view are both in the variable table: one block, one free
    assert len(stub_lib.freed) == 2 and not stub_lib.live
    rt.free()  # idempotent
    assert len(stub_lib.freed) == 2


def test_view_casts_a_scalar_to_an_array(stub_lib):
    """realize-node :View on a buffer holding a number with nrank > 0 opens storage and fills it with the number,
    sized by the non-broadcast axes (runtime.lisp:274-283)."""
    from caten_amd.runtime import GraphRuntime
    from caten_amd.buffer import HipBuffer, make_buffer

    class RT(GraphRuntime):
        buffer_type = HipBuffer

    scalar = make_buffer([], [], "float32", value=2.5, device=HipBuffer)
    rt = RT([_view_node(2, [3, 4], [0, 1], broadcast=[True, False])], ["v"], {"base": scalar})
    v = rt.forward()
    assert v.nrank == 2 and isinstance(v.value, int) and v.owns_storage
    assert np.frombuffer(stub_lib.uploads[v.value], np.float32).tolist() == [2.5] * 4
    assert scalar.value == 2.5
    rt.free()
    assert not stub_lib.live


def test_remap_key():
    from caten_amd.llm import remap_key
    assert remap_key("blk.3.attn_qkv.weight") == "h.3.attn.c_attn.weight"
    assert remap_key("blk.11.ffn_down.bias") == "h.11.mlp.c_proj.bias"
    assert remap_key("token_embd.weight") == "wte.weight"
    assert remap_key("output_norm.weight") == "ln_f.affine"
    assert remap_key("output.weight") == "lm_head.weight"


def _matmul_item(name="fused_relu_matmul"):
    """The blueprint of (caten (!relu (!matmul a b))) with symbolic m n k, as the reference lowers it
    (test-scheduler.lisp:126-135): out[n*i+j] = max(sum_k a[k_*i+k]*b[j+n*k], 0)."""
    A = lambda id_, idx: {"op": "AREF", "id": id_, "index": idx}  # noqa: E731
    add = lambda *a: {"op": "ADD", "args": list(a)}  # noqa: E731
    mul = lambda *a: {"op": "MUL", "args": list(a)}  # noqa: E731
    lt = lambda a, b: {"op": "<", "args": [a, b]}  # noqa: E731
    return {"name": name, "blueprint": [
        {"type": "DEFINE-GLOBAL", "id": "val_out", "dtype": "float32", "pointer_p": True, "arg_type": "output", "nrank": 2},
        {"type": "DEFINE-GLOBAL", "id": "m", "dtype": "int64", "pointer_p": False, "arg_type": "shape", "nrank": 0},
        {"type": "DEFINE-GLOBAL", "id": "n", "dtype": "int64", "pointer_p": False, "arg_type": "shape", "nrank": 0},
        {"type": "DEFINE-GLOBAL", "id": "kk", "dtype": "int64", "pointer_p": False, "arg_type": "shape", "nrank": 0},
        {"type": "DEFINE-GLOBAL", "id": "val_a", "dtype": "float32", "pointer_p": True, "arg_type": "input", "nrank": 2},
        {"type": "DEFINE-GLOBAL", "id": "val_b", "dtype": "float32", "pointer_p": True, "arg_type": "input", "nrank": 2},
        {"type": "FOR", "idx": "_gid0", "upfrom": 0, "below": lt("_gid0", "m"), "by": 1},
        {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": lt("_gid1", "n"), "by": 1},
        {"type": "EXPR", "writes": [A("acc", None)], "expr": 0.0, "declare_type": True, "dtype": "float32"},
        {"type": "FOR", "idx": "_gid2", "upfrom": 0, "below": lt("_gid2", "kk"), "by": 1},
        {"type": "EXPR", "writes": [A("acc", None)], "dtype": "float32", "reduction": True,
         "expr": add("acc", mul(A("val_a", add(mul("kk", "_gid0"), "_gid2")), A("val_b", add("_gid1", mul("n", "_gid2")))))},
        {"type": "ENDFOR", "idx": "_gid2"},
        {"type": "EXPR", "writes": [A("val_out", add(mul("n", "_gid0"), "_gid1"))], "dtype": "float32",
         "expr": {"op": "MAX", "args": ["acc", 0.0]}},
        {"type": "ENDFOR", "idx": "_gid1"},
        {"type": "ENDFOR", "idx": "_gid0"},
    ]}


def test_renderer_emits_and_hiprtc_compiles_for_gfx950():
    from caten_amd import HipRenderer
    r = HipRenderer()
    item = _matmul_item()
    src = r.render_kernel(item)
    assert 'extern "C" __global__' in src and "fused_relu_matmul(" in src
    # argument order: outputs, dynamic shapes (by value), inputs (rewriting-rules.lisp:207-231)
    sig = src.split("(", 1)[1].split(")")[0] if False else src[src.index("fused_relu_matmul(")::].split("{")[0]
    assert sig.index("val_out") < sig.index("const long long m") < sig.index("val_a") < sig.index("val_b")
    assert "const float* __restrict__ val_a" in sig
    # the two output loops became the thread grid, the reduction loop stayed serial
    assert src.count("for (int") == 1 and "_gid2" in src and "blockIdx.x" in src
    assert "ct_max(acc, 0.0f)" in src
    r.compile_kernel([item])
    assert r.code_object[:4] == b"\x7fELF"


def test_programs_recognise_the_shapes_hand_written_kernels_cover():
    """cthip_program_create: the matmul nest (test-scheduler.lisp:126-135) with its epilogues, Linear's transposed
    read, the one-hot Embedding (nn/embedding.lisp:13-25), ArgMaxNode (high-level-ops.lisp:314-325) and softmax rows
    get a route next to their rendered source; anything else is rendered only."""
    from caten_amd import HipRenderer, blueprints as bp
    r = HipRenderer()
    cases = [(bp.matmul(), "matmul"), (bp.matmul(relu=True), "matmul"), (bp.matmul(bias=True, relu=True, transposed_b=True), "matmul"),
             (_matmul_item(), "matmul"), (bp.embedding_onehot(), "embedding"), (bp.argmax_rows(), "argmax"),
             (bp.softmax_rows(), "softmax"), (bp.softmax_rows(rows=8, n=40), "softmax"),
             # LayerNorm / RMSNorm rows (nn/normalization.lisp:39-58,78-92), recognised by the VALUE of their scalar
             # statements and element expressions: with and without affine parameters, static and dynamic shape
             (bp.layernorm_rows(), "layernorm"), (bp.layernorm_rows(affine=False, eps=1e-3), "layernorm"),
             (bp.layernorm_rows(rows=8, n=40), "layernorm"), (bp.rmsnorm_rows(), "rmsnorm"),
             (bp.rmsnorm_rows(weight=False, rows=4, n=96, eps=1e-6), "rmsnorm")]
    for item, want in cases:
        src = r.render_kernel(item)
        assert item["route"] == want, (item["name"], item["route"])
        assert 'extern "C" __global__' in src  # the rendered kernel is always there to fall back on
    # a GELU epilogue is not one of the epilogues the GEMM applies: rendered
    gelu = bp.matmul()
    gelu["blueprint"][-3]["expr"] = {"op": "MUL", "args": ["acc", {"op": "RECIP", "args": [{"op": "ADD", "args": [1.0, {"op": "EXP2", "args": ["acc"]}]}]}]}
    r.render_kernel(gelu)
    assert gelu["route"] == "rendered"
    # the reduction multiplies by something that is not an array element: rendered
    odd = bp.matmul()
    odd["blueprint"][-5]["expr"]["args"][1]["args"][1] = "m"
    r.render_kernel(odd)
    assert odd["route"] == "rendered"
    # a "LayerNorm" whose variance is the mean of x^2 (not of the centred row), one whose output forgets the mean,
    # and an RMSNorm that adds a bias: not what the row kernels compute, so rendered
    ln = bp.layernorm_rows()
    for nd in ln["blueprint"]:
        if nd.get("reduction") and nd["writes"][0]["id"] == "q":
            xi = nd["expr"]["args"][1]["args"][0]["args"][0]
            nd["expr"] = {"op": "ADD", "args": ["q", {"op": "MUL", "args": [xi, xi]}]}
    r.render_kernel(ln)
    assert ln["route"] == "rendered"
    ln2 = bp.layernorm_rows(affine=False)
    st = next(nd for nd in ln2["blueprint"] if nd.get("writes") and nd["writes"][0]["id"] == "val_y")
    st["expr"] = {"op": "MUL", "args": [st["expr"]["args"][0]["args"][0], "r"]}  # x * r instead of (x - u) * r
    r.render_kernel(ln2)
    assert ln2["route"] == "rendered"
    rms = bp.rmsnorm_rows()
    st = next(nd for nd in rms["blueprint"] if nd.get("writes") and nd["writes"][0]["id"] == "val_y")
    st["expr"] = {"op": "ADD", "args": [st["expr"], 1.0]}
    r.render_kernel(rms)
    assert rms["route"] == "rendered"


def test_row_with_a_running_sum_stays_in_one_thread():
    """s += x[i]; y[i] = s inside one loop is a scan, not a reduction: splitting the loop over the lanes of a
    wavefront would store every lane's partial, so such a row keeps one thread (no lane-strided loop)."""
    from caten_amd import HipRenderer, blueprints as bp
    A = lambda id_, idx: {"op": "AREF", "id": id_, "index": idx}  # noqa: E731
    add = lambda *a: {"op": "ADD", "args": list(a)}  # noqa: E731
    mul = lambda *a: {"op": "MUL", "args": list(a)}  # noqa: E731
    idx = add(mul("n", "_gid0"), "_gid1")
    for order in (0, 1):
        red = {"type": "EXPR", "writes": [A("s", None)], "expr": add("s", A("val_x", idx)), "dtype": "float32", "reduction": True}
        store = {"type": "EXPR", "writes": [A("val_y", idx)], "expr": "s", "dtype": "float32"}
        item = {"name": "running_sum", "blueprint": [
            bp._glob("val_y", "output", 2), bp._glob("rows", "shape", 0, "int64"), bp._glob("n", "shape", 0, "int64"),
            bp._glob("val_x", "input", 2),
            {"type": "FOR", "idx": "_gid0", "upfrom": 0, "below": bp._lt("_gid0", "rows"), "by": 1},
            {"type": "EXPR", "writes": [A("s", None)], "expr": 0.0, "declare_type": True, "dtype": "float32"},
            {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": bp._lt("_gid1", "n"), "by": 1},
            *([red, store] if order == 0 else [store, red]),
            {"type": "ENDFOR", "idx": "_gid1"},
            {"type": "ENDFOR", "idx": "_gid0"},
        ]}
        src = HipRenderer().render_kernel(item)
        assert "+=64" not in src and "ct_wave_" not in src and "_lane" not in src
    # the plain reduction next to it does get a wavefront per row
    src = HipRenderer().render_kernel(bp.softmax_rows())
    assert "+=64" in src and "ct_wave_max_f" in src and "ct_wave_add_f" in src


def test_program_text_errors_are_reported():
    from caten_amd import _lib, HipError
    lib = _lib.load()
    p = ctypes.c_void_p()
    for text, what in [(b"(item k (for i 0", b"unbalanced"), (b"(item k (frobnicate 1))", b"unknown blueprint node"),
                       (b"(item k (for i 0 (< i 4) 1))", b"unbalanced for"), (b"(kernel k)", b"expected (item"),
                       (b"(item k (define-global a float33 t input 1))", b"unknown dtype")]:
        assert lib.cthip_program_create(ctypes.byref(p), text) != 0
        assert what in lib.cthip_last_error(), lib.cthip_last_error()
    # an instruction the renderer has no spelling for
    assert lib.cthip_program_create(ctypes.byref(p), b"(item k (expr (y) (frob x) :dtype float32))") == _lib.E_UNSUPPORTED
    assert b"no %render-node method for :frob" in lib.cthip_last_error()
    # Lisp float syntax and keywords are read: 1.0d0, 1.0f0, :dtype, upper case
    assert lib.cthip_program_create(ctypes.byref(p), b"(ITEM K (EXPR ((AREF Y 0)) (ADD 1.5d0 2.0f0 1.0e-5) :DTYPE :FLOAT32))") == 0
    assert b"y[0] = (1.5f+2.0f+0.00001f);" in lib.cthip_program_source(p)
    lib.cthip_program_destroy(p)


def test_renderer_reports_compile_errors():
    from caten_amd import HipRenderer, HipError
    r = HipRenderer()
    bad = {"name": "broken", "blueprint": [], "rendered_object": 'extern "C" __global__ void broken() { this is not C; }\n'}
    with pytest.raises(HipError) as e:
        r.compile_kernel([bad])
    assert "error" in str(e.value).lower() and "hipRTC" in str(e.value)


def test_renderer_spellings():
    from caten_amd import HipRenderer
    r = HipRenderer()
    assert r.render_expr({"op": "RECIP", "args": ["x"]}) == "(1.0f/(x))"
    assert r.render_expr({"op": "EXP2", "args": [{"op": "MUL", "args": ["x", 1.442695]}]}) == "exp2f((x*1.442695f))"
    assert r.render_expr(float("-inf")) == "_negative_infinity"
    assert r.render_expr({"op": "WHERE", "args": [{"op": "<", "args": ["a", "b"]}, "a", "b"]}) == "((a<b) ? a : b)"
    assert r.render_expr({"op": "CAST", "dtype": "int64", "args": ["x"]}) == "((long long)x)"
    assert r.render_expr({"op": "SPACE", "level": "block", "rank": 0}) == "blockIdx.x"
    # clang.lisp:82-97: index = sum stride*(from + by*gid); broadcast axes drop out
    aref = {"op": "AREF", "id": "V", "space": {"strides": [12, 1, 0], "views": [None, (2, 9, 3, False), (0, 4, 1, True)],
                                                "iterations": ["i", "j", "k"]}}
    assert r.render_expr(aref) == "v[((12*i)+(1*(2+(3*j))))]"
    # renderer.lisp:194-221: the index of the element being computed; size-1 axes contribute nothing
    ic = {"op": "INDEX-COMPONENTS", "shape": [4, 1, "n"], "strides": ["n", "n", 1], "iterations": ["_gid0", "_gid1", "_gid2"]}
    assert r.render_expr(ic) == "((n*_gid0)+(1*_gid2))"
    assert r.render_expr({"op": "INDEX-COMPONENTS", "shape": [1], "strides": [1], "iterations": ["_gid0"]}) == "0"
    with pytest.raises(NotImplementedError):
        r.render_expr({"op": "NOPE", "args": []})


def test_runtime_vm_semantics_on_host_scalars():
    """The parts of GraphRuntime that need no device: variables, pc, error wrapping, arity checks."""
    from caten_amd.runtime import GraphRuntime, Node, RuntimeError_, coerce_dtyped_buffer
    from caten_amd.buffer import make_buffer
    rt = GraphRuntime([Node("Pause/Backward", ["out"], ["a"])], fw_outputs=["out"])
    assert rt.forward(("a", 3)) == 3
    rt = GraphRuntime([Node("NoSuchOp", ["out"], ["a"])], fw_outputs=["out"])
    with pytest.raises(RuntimeError_) as e:
        rt.forward(("a", 1))
    assert "instruction 0" in str(e.value) and "NoSuchOp" in str(e.value)
    with pytest.raises(RuntimeError_):
        GraphRuntime([Node("Pause/Backward", ["o"], ["undefined_var"])]).forward()
    s = make_buffer([], [], "int64")
    s.value = 7
    assert coerce_dtyped_buffer(s, "float32") == 7.0 and coerce_dtyped_buffer(3.9, "int64") == 3


def test_explicit_grid_item_keeps_its_own_indexing():
    """An item whose indices are bound from blockIdx / threadIdx (ExprGrid) gets no second work distribution from the
    renderer, and the text of its grid sizes is carried into the program."""
    from caten_amd import HipRenderer, blueprints as bp
    it = bp.add_global_2d(local=(16, 8))
    src = HipRenderer().render_kernel(it)
    assert "_total" not in src and "__launch_bounds__(1024)" in src
    assert "((blockIdx.y*8)+threadIdx.y)" in src and "((blockIdx.x*16)+threadIdx.x)" in src
    assert "if ((_gid1<n))" in src


def test_conv_pool_and_backward_items_render():
    from caten_amd import HipRenderer, blueprints as bp
    r = HipRenderer()
    conv = r.render_kernel(bp.conv2d_relu(2, 3, 8, 8, 4, 3, 3))
    assert "(long long)(2)*(long long)(4)*(long long)(6)*(long long)(6)" in conv and conv.count("for (int") == 3
    pool = r.render_kernel(bp.maxpool2x2(2, 3, 8, 8))
    assert "_negative_infinity" in pool and "ct_max(m," in pool
    bwd = r.render_kernel(bp.linear_relu_backward())
    assert "ct_wave_add_f(acc)" in bwd and "_gid1+=64" in bwd


def test_elementwise_and_row_items_hold_their_reads_in_registers():
    """What the renderer does for memory parallelism, checked on the emitted source and compiled for gfx950:
    element-wise items take four elements per thread with the reads issued first and flat operands addressed by
    the flat position; row items load the row's input elements once, in front of the first loop over the row."""
    from caten_amd import HipRenderer, blueprints as bp
    r = HipRenderer()
    g = bp.gelu_tanh()
    src = r.render_kernel(g)
    assert src.count("_e < 4") == 8  # (32-bit, 64-bit) x (whole block, last block) x (reads, statements)
    assert "_h0[_e] = val_x[_t];" in src and "val_y[_t] = " in src and "val_x[((n*_gid0)+_gid1)]" not in src
    assert "blockIdx.x * 1024 + 1024 <= _total" in src
    gs = bp.gelu_tanh("fused_gelu_static", 64, 768)
    src = r.render_kernel(gs)
    assert "_h0[_e] = val_x[_t];" in src and "% (unsigned)(768)" in src  # a static bound is divided by the compiler
    ln = bp.layernorm_rows("ln_static", True, 1e-5, 64, 768)
    src = r.render_kernel(ln)
    # three arrays held as [passes][4] quads; the three loops over the row read no global memory but the store
    for k, name in enumerate(("val_x", "val_g", "val_b")):
        assert src.count(f"_h{k}[_gid1_i][_gid1_k] = {name}[") == 1 and src.count(f"{name}[") == 1
    sd = bp.softmax_rows()
    src = r.render_kernel(sd)
    assert src.count("_h0[_gid1_i] = val_x[((n*_gid0)+_gid1)];") == 6 and src.count("if (_gid1_ok)") == 0
    assert src.count("m = _gid1_ok ? _w : m;") == 6 and src.count("s = _gid1_ok ? _w : s;") == 6
    r.compile_kernel([g, gs, ln, sd])
    assert r.code_object[:4] == b"\x7fELF"


# ---------------------------------------------------------------------------------------------------------------
# The Schedule-Items of a GPT-2 `forward` (tests/golden/blueprints/): interchange text pinned as fixtures
GOLDEN_BP = os.path.join(ROOT, "tests", "golden", "blueprints")
GPT2_ITEM_ROUTES = {
    "embed_tokens": "embedding", "embed_positions": "embedding", "mask": "rendered", "layernorm": "layernorm",
    "c_attn": "matmul", "assign_k": "rendered", "assign_v": "rendered", "scores": "matmul", "softmax": "softmax",
    "values": "matmul", "merge_heads": "rendered", "attn_proj": "matmul", "c_fc": "matmul", "mlp_proj": "matmul",
    "lm_head": "matmul", "argmax": "argmax"}


def _create(text: bytes):
    from caten_amd import _lib
    lib = _lib.load()
    prog = ctypes.c_void_p()
    rc = lib.cthip_program_create(ctypes.byref(prog), text)
    assert rc == 0, lib.cthip_last_error().decode()
    route, src = lib.cthip_program_route(prog).decode(), lib.cthip_program_source(prog).decode()
    lib.cthip_program_destroy(prog)
    return route, src


def test_gpt2_step_items_print_as_their_golden_text_and_route():
    """every distinct item of the decode step (external/llm/layers.lisp:3-90): the printer's text is the committed
    fixture, the library reads it, and each Linear / attention / norm / embedding / argmax item has a hand-written
    kernel behind it"""
    from caten_amd import blueprints as bp, synth
    from caten_amd.renderer import item_sexp
    items = bp.gpt2_step_items(synth.GPT2_CONFIGS["gpt2"])
    assert set(items) == set(GPT2_ITEM_ROUTES)
    for key, item in items.items():
        with open(os.path.join(GOLDEN_BP, f"gpt2_{key}.sexp")) as f:
            golden = f.read()
        assert item_sexp(item) == golden, f"{key}: the printed blueprint differs from tests/golden/blueprints/gpt2_{key}.sexp"
        route, src = _create(golden.encode())
        assert route == GPT2_ITEM_ROUTES[key], (key, route)
        assert 'extern "C" __global__' in src


def test_rope_and_swiglu_items_print_as_their_golden_text():
    """RoPE with its tables computed in place (nn/positional-encoding.lisp:23-48) and silu(gate) * up
    (nn/activations.lisp:180-189): element-wise items, rendered"""
    from caten_amd import blueprints as bp
    from caten_amd.renderer import item_sexp
    for fname, item in (("rope_32x64", bp.rope_rows(32, 64)), ("swiglu_5632", bp.swiglu_rows(5632))):
        with open(os.path.join(GOLDEN_BP, fname + ".sexp")) as f:
            golden = f.read()
        assert item_sexp(item) == golden, fname
        route, src = _create(golden.encode())
        assert route == "rendered" and 'extern "C" __global__' in src


def test_blueprints_in_a_lisp_printers_spelling_are_read_the_same():
    """upper-case symbols, exponent markers (0.0f0, 1.0e-5, ...d0), single-float folded constants (1/768 =
    0.0013020834, 3e-8 off), commutative operands in another order; and the one rendered matmul the reference's own
    tests hold, with its index expressions verbatim (source/test-suite/test-scheduler.lisp:117-138)"""
    for name, want in (("lisp_spelling_layernorm", "layernorm"), ("lisp_spelling_linear_gelu", "matmul"),
                       ("reference_chunk_matmul", "matmul")):
        with open(os.path.join(GOLDEN_BP, name + ".sexp"), "rb") as f:
            route, _ = _create(f.read())
        assert route == want, (name, route)


def test_the_references_own_rendered_item_renders_to_the_same_statement():
    """the one Schedule-Item whose blueprint AND rendered C the reference prints side by side
    (docs/end-to-end-example.lisp:225-250): `val_6[0] = sin(sin((1.0+1.5707964)));` -- the HIP text is that statement
    with single-precision spellings"""
    with open(os.path.join(GOLDEN_BP, "reference_sincos_item.sexp"), "rb") as f:
        route, src = _create(f.read())
    assert route == "rendered"
    body = [ln.strip() for ln in src.splitlines() if ln.strip().startswith("val_6[0]")]
    assert body == ["val_6[0] = sinf(sinf((1.0f+1.5707964f)));"], src
    assert "fused_sin_sin_add_load_load6914144(float* val_6)" in src  # the reference's signature, verbatim


def test_near_misses_of_the_decode_step_items_stay_rendered():
    from caten_amd import HipRenderer, blueprints as bp
    import copy
    r = HipRenderer()

    def route(item):
        r.render_kernel(item)
        return item["route"]
    A = lambda id_, idx: {"op": "AREF", "id": id_, "index": idx}  # noqa: E731
    # Linear + GELU with another constant inside the tanh: not the kernels' GELU
    it = bp.gpt2_linear(32, 16, bias=True, gelu=True)
    text = repr(it).replace("0.7978845608", "0.81")
    assert route(eval(text, {"inf": float("inf")})) == "rendered"
    assert route(bp.gpt2_linear(32, 16, bias=True, gelu=True)) == "matmul"
    # an epilogue that squares the accumulator, one that reads three more arrays, one that reads the output
    sq = bp.gpt2_linear(32, 16, bias=False)
    sq["blueprint"][-3]["expr"] = {"op": "MUL", "args": ["acc", "acc"]}
    assert route(sq) == "rendered"
    three = bp.gpt2_linear(32, 16, bias=True, residual=True)
    three["blueprint"].insert(1, {"type": "DEFINE-GLOBAL", "id": "val_z", "dtype": "float32", "pointer_p": True, "arg_type": "input", "nrank": 1})
    three["blueprint"][-3]["expr"] = {"op": "ADD", "args": [three["blueprint"][-3]["expr"], A("val_z", "_gid1")]}
    assert route(three) == "rendered"
    own = bp.gpt2_linear(32, 16, bias=False)
    own["blueprint"][-3]["expr"] = {"op": "ADD", "args": ["acc", A("val_y", {"op": "ADD", "args": [{"op": "MUL", "args": [32, "_gid0"]}, "_gid1"]})]}
    assert route(own) == "rendered"
    # the bias added AFTER the GELU is still a matmul item (the router decides at launch which kernel can apply it)
    post = bp.gpt2_linear(32, 16, bias=False, gelu=True)
    post["blueprint"].insert(4, {"type": "DEFINE-GLOBAL", "id": "val_b", "dtype": "float32", "pointer_p": True, "arg_type": "input", "nrank": 1})
    post["blueprint"][-3]["expr"] = {"op": "ADD", "args": [post["blueprint"][-3]["expr"], A("val_b", "_gid1")]}
    assert route(post) == "matmul"
    # softmax whose second loop reads the row shifted by one element; LayerNorm whose store loop does
    sm = bp.gpt2_softmax_rows(4)
    shifted = copy.deepcopy(sm)
    red = [n for n in shifted["blueprint"] if n.get("reduction") and n["writes"][0]["id"] == "e"][0]
    aref = red["expr"]["args"][1]["args"][0]["args"][0]["args"][0]
    assert aref["op"] == "AREF"
    aref["index"] = {"op": "ADD", "args": [aref["index"], 1]}
    assert route(sm) == "softmax" and route(shifted) == "rendered"
    ln = bp.gpt2_layernorm(64)
    shifted = copy.deepcopy(ln)
    st = shifted["blueprint"][-3]
    assert st["writes"][0]["id"] == "val_y"
    centred = st["expr"]["args"][0]["args"][0]["args"][0]  # (x - u): the blueprint shares one aref object between its loops
    xa = centred["args"][0]
    assert xa["op"] == "AREF" and xa["id"] == "val_x"
    st["expr"]["args"][0]["args"][0]["args"][0] = {"op": "ADD", "args": [A("val_x", {"op": "ADD", "args": [xa["index"], 1]}), centred["args"][1]]}
    assert route(ln) == "layernorm" and route(shifted) == "rendered"
    # the position embedding compared with something that also depends on the column: not a row gather
    pe = bp.gpt2_embed_positions_add(64, 32)
    bad = eval(repr(pe).replace("{'op': 'ADD', 'args': ['n', '_gid0']}", "{'op': 'ADD', 'args': ['n', '_gid1']}"), {"inf": float("inf")})
    assert route(pe) == "embedding" and route(bad) == "rendered"
