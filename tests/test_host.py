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
