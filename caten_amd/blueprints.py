"""Blueprints of row-wise Schedule-Items in the dict interchange format of renderer.py, shaped the way Caten
lowers them (one kernel, several loops over the row: source/test-suite/test-scheduler.lisp:37-45,
test-activations.lisp:60-73).  Used by the item benchmark to time RENDERED kernels next to the hand-written ones."""
from __future__ import annotations


def _A(id_, idx):
    return {"op": "AREF", "id": id_, "index": idx}


def _add(*a):
    return {"op": "ADD", "args": list(a)}


def _mul(*a):
    return {"op": "MUL", "args": list(a)}


def _lt(a, b):
    return {"op": "<", "args": [a, b]}


def _glob(id_, arg_type, nrank, dtype="float32"):
    return {"type": "DEFINE-GLOBAL", "id": id_, "dtype": dtype, "pointer_p": nrank > 0, "arg_type": arg_type, "nrank": nrank}


def softmax_rows(name: str = "fused_softmax", rows: int | None = None, n: int | None = None) -> dict:
    """softmax over the last axis of (rows, n): max, sum of exp2((x - max) * 1/ln2), normalise
    (nn/activations.lisp:59-62,107-119).  With `rows` and `n` given the shape is static, as for a tensor made
    with a fixed shape: the bounds are literals and the arguments are val_y, val_x; otherwise they are the
    dynamic-shape arguments val_y, rows, n, val_x."""
    static = rows is not None and n is not None
    R, N = (rows, n) if static else ("rows", "n")
    idx = _add(_mul(N, "_gid0"), "_gid1")
    ex = {"op": "EXP2", "args": [_mul(_add(_A("val_x", idx), {"op": "NEG", "args": ["m"]}), 1.442695)]}
    loop = {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": _lt("_gid1", N), "by": 1}
    end = {"type": "ENDFOR", "idx": "_gid1"}
    shapes = [] if static else [_glob("rows", "shape", 0, "int64"), _glob("n", "shape", 0, "int64")]
    return {"name": name, "blueprint": [
        _glob("val_y", "output", 2), *shapes, _glob("val_x", "input", 2),
        {"type": "FOR", "idx": "_gid0", "upfrom": 0, "below": _lt("_gid0", R), "by": 1},
        {"type": "EXPR", "writes": [_A("m", None)], "expr": float("-inf"), "declare_type": True, "dtype": "float32"},
        dict(loop),
        {"type": "EXPR", "writes": [_A("m", None)], "expr": {"op": "MAX", "args": ["m", _A("val_x", idx)]}, "dtype": "float32", "reduction": True},
        dict(end),
        {"type": "EXPR", "writes": [_A("s", None)], "expr": 0.0, "declare_type": True, "dtype": "float32"},
        dict(loop),
        {"type": "EXPR", "writes": [_A("s", None)], "expr": _add("s", ex), "dtype": "float32", "reduction": True},
        dict(end),
        dict(loop),
        {"type": "EXPR", "writes": [_A("val_y", idx)], "expr": _mul(ex, {"op": "RECIP", "args": ["s"]}), "dtype": "float32"},
        dict(end),
        {"type": "ENDFOR", "idx": "_gid0"},
    ]}
