"""Blueprints of row-wise and element-wise Schedule-Items in the dict interchange format of renderer.py, shaped the way Caten
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


def _neg(a):
    return {"op": "NEG", "args": [a]}


def gelu_tanh(name: str = "fused_gelu", rows: int | None = None, n: int | None = None) -> dict:
    """GELU(tanh) of every element of (rows, n), decomposed the way the reference does (nn/activations.lisp:202-215,
    3-7; api/high-level-ops.lisp:112-117): 0.5 x (1 + tanh(u)) with u = sqrt(2/pi) (x + 0.044715 x^3),
    tanh(u) = 2 sigmoid(2u) - 1, sigmoid(z) = recip(1 + exp2(z * -1/ln2)).  Static or dynamic shape as for
    softmax_rows."""
    static = rows is not None and n is not None
    R, N = (rows, n) if static else ("rows", "n")
    idx = _add(_mul(N, "_gid0"), "_gid1")
    x = _A("val_x", idx)
    u = _mul(0.7978845608, _add(x, _mul(0.044715, _mul(x, _mul(x, x)))))
    sig = {"op": "RECIP", "args": [_add(1.0, {"op": "EXP2", "args": [_mul(_mul(2.0, u), -1.4426950408889634)]})]}
    shapes = [] if static else [_glob("rows", "shape", 0, "int64"), _glob("n", "shape", 0, "int64")]
    return {"name": name, "blueprint": [
        _glob("val_y", "output", 2), *shapes, _glob("val_x", "input", 2),
        {"type": "FOR", "idx": "_gid0", "upfrom": 0, "below": _lt("_gid0", R), "by": 1},
        {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": _lt("_gid1", N), "by": 1},
        {"type": "EXPR", "writes": [_A("val_y", idx)], "expr": _mul(_mul(0.5, x), _add(1.0, _add(_mul(2.0, sig), -1.0))), "dtype": "float32"},
        {"type": "ENDFOR", "idx": "_gid1"},
        {"type": "ENDFOR", "idx": "_gid0"},
    ]}


def _rstd(q, N, eps):
    """1 / sqrt(q / n + eps), the division spelled recip(cast(n)) as the simplifier leaves it"""
    n = {"op": "CAST", "dtype": "float32", "args": [N]} if isinstance(N, str) else float(N)
    return {"op": "RECIP", "args": [{"op": "SQRT", "args": [_add(_mul(q, {"op": "RECIP", "args": [n]}), eps)]}]}


def layernorm_rows(name: str = "fused_layernorm", affine: bool = True, eps: float = 1e-5, rows: int | None = None,
                   n: int | None = None) -> dict:
    """LayerNorm over the last axis of (rows, n) as one kernel (nn/normalization.lisp:39-58): the mean, the biased
    variance of the centred row, then (x - mean) * rstd [* gamma + beta].  Arguments: val_y, [rows, n,] val_x
    [, val_g, val_b]."""
    static = rows is not None and n is not None
    R, N = (rows, n) if static else ("rows", "n")
    idx = _add(_mul(N, "_gid0"), "_gid1")
    xi = _A("val_x", idx)
    nf = {"op": "CAST", "dtype": "float32", "args": [N]} if not static else float(N)
    loop = {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": _lt("_gid1", N), "by": 1}
    end = {"type": "ENDFOR", "idx": "_gid1"}
    shapes = [] if static else [_glob("rows", "shape", 0, "int64"), _glob("n", "shape", 0, "int64")]
    params = [_glob("val_g", "input", 1), _glob("val_b", "input", 1)] if affine else []
    centred = _add(xi, _neg("u"))
    y = _mul(centred, "r")
    if affine:
        y = _add(_mul(y, _A("val_g", "_gid1")), _A("val_b", "_gid1"))
    return {"name": name, "blueprint": [
        _glob("val_y", "output", 2), *shapes, _glob("val_x", "input", 2), *params,
        {"type": "FOR", "idx": "_gid0", "upfrom": 0, "below": _lt("_gid0", R), "by": 1},
        {"type": "EXPR", "writes": [_A("s", None)], "expr": 0.0, "declare_type": True, "dtype": "float32"},
        dict(loop),
        {"type": "EXPR", "writes": [_A("s", None)], "expr": _add("s", xi), "dtype": "float32", "reduction": True},
        dict(end),
        {"type": "EXPR", "writes": [_A("u", None)], "expr": _mul("s", {"op": "RECIP", "args": [nf]}), "declare_type": True, "dtype": "float32"},
        {"type": "EXPR", "writes": [_A("q", None)], "expr": 0.0, "declare_type": True, "dtype": "float32"},
        dict(loop),
        {"type": "EXPR", "writes": [_A("q", None)], "expr": _add("q", _mul(centred, centred)), "dtype": "float32", "reduction": True},
        dict(end),
        {"type": "EXPR", "writes": [_A("r", None)], "expr": _rstd("q", N, eps), "declare_type": True, "dtype": "float32"},
        dict(loop),
        {"type": "EXPR", "writes": [_A("val_y", idx)], "expr": y, "dtype": "float32"},
        dict(end),
        {"type": "ENDFOR", "idx": "_gid0"},
    ]}


def layernorm_softmax_rows(name: str = "fused_layernorm_softmax", eps: float = 1e-5, rows: int | None = None,
                           n: int | None = None) -> dict:
    """softmax(LayerNorm(x) * gamma + beta) over the last axis of (rows, n) as ONE kernel with five loops over the
    row: mean, biased variance, maximum of the normalised row, sum of exp2, normalise (nn/normalization.lisp:39-58
    followed by nn/activations.lisp:59-62,107-119 in one Schedule-Item).  Arguments: val_y, [rows, n,] val_x, val_g,
    val_b."""
    static = rows is not None and n is not None
    R, N = (rows, n) if static else ("rows", "n")
    idx = _add(_mul(N, "_gid0"), "_gid1")
    xi = _A("val_x", idx)
    nf = {"op": "CAST", "dtype": "float32", "args": [N]} if not static else float(N)
    loop = {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": _lt("_gid1", N), "by": 1}
    end = {"type": "ENDFOR", "idx": "_gid1"}
    shapes = [] if static else [_glob("rows", "shape", 0, "int64"), _glob("n", "shape", 0, "int64")]
    centred = _add(xi, _neg("u"))
    ln = _add(_mul(_mul(centred, "r"), _A("val_g", "_gid1")), _A("val_b", "_gid1"))
    ex = {"op": "EXP2", "args": [_mul(_add(ln, _neg("m")), 1.442695)]}
    red = lambda name, expr: {"type": "EXPR", "writes": [_A(name, None)], "expr": expr, "dtype": "float32", "reduction": True}  # noqa: E731
    decl = lambda name, expr: {"type": "EXPR", "writes": [_A(name, None)], "expr": expr, "declare_type": True, "dtype": "float32"}  # noqa: E731
    return {"name": name, "blueprint": [
        _glob("val_y", "output", 2), *shapes, _glob("val_x", "input", 2), _glob("val_g", "input", 1), _glob("val_b", "input", 1),
        {"type": "FOR", "idx": "_gid0", "upfrom": 0, "below": _lt("_gid0", R), "by": 1},
        decl("s", 0.0), dict(loop), red("s", _add("s", xi)), dict(end),
        decl("u", _mul("s", {"op": "RECIP", "args": [nf]})),
        decl("q", 0.0), dict(loop), red("q", _add("q", _mul(centred, centred))), dict(end),
        decl("r", _rstd("q", N, eps)),
        decl("m", float("-inf")), dict(loop), red("m", {"op": "MAX", "args": ["m", ln]}), dict(end),
        decl("e", 0.0), dict(loop), red("e", _add("e", ex)), dict(end),
        dict(loop),
        {"type": "EXPR", "writes": [_A("val_y", idx)], "expr": _mul(ex, {"op": "RECIP", "args": ["e"]}), "dtype": "float32"},
        dict(end),
        {"type": "ENDFOR", "idx": "_gid0"},
    ]}


def rmsnorm_rows(name: str = "fused_rmsnorm", weight: bool = True, eps: float = 1e-5, rows: int | None = None,
                 n: int | None = None) -> dict:
    """RMSNorm over the last axis of (rows, n) (nn/normalization.lisp:78-92): x / sqrt(mean(x^2) + eps) [* w].
    Arguments: val_y, [rows, n,] val_x [, val_w]."""
    static = rows is not None and n is not None
    R, N = (rows, n) if static else ("rows", "n")
    idx = _add(_mul(N, "_gid0"), "_gid1")
    xi = _A("val_x", idx)
    loop = {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": _lt("_gid1", N), "by": 1}
    end = {"type": "ENDFOR", "idx": "_gid1"}
    shapes = [] if static else [_glob("rows", "shape", 0, "int64"), _glob("n", "shape", 0, "int64")]
    y = _mul(xi, "r")
    if weight:
        y = _mul(_A("val_w", "_gid1"), y)
    return {"name": name, "blueprint": [
        _glob("val_y", "output", 2), *shapes, _glob("val_x", "input", 2), *([_glob("val_w", "input", 1)] if weight else []),
        {"type": "FOR", "idx": "_gid0", "upfrom": 0, "below": _lt("_gid0", R), "by": 1},
        {"type": "EXPR", "writes": [_A("q", None)], "expr": 0.0, "declare_type": True, "dtype": "float32"},
        dict(loop),
        {"type": "EXPR", "writes": [_A("q", None)], "expr": _add(_mul(xi, xi), "q"), "dtype": "float32", "reduction": True},
        dict(end),
        {"type": "EXPR", "writes": [_A("r", None)], "expr": _rstd("q", N, eps), "declare_type": True, "dtype": "float32"},
        dict(loop),
        {"type": "EXPR", "writes": [_A("val_y", idx)], "expr": y, "dtype": "float32"},
        dict(end),
        {"type": "ENDFOR", "idx": "_gid0"},
    ]}


def matmul(name: str = "fused_matmul", relu: bool = False, bias: bool = False, transposed_b: bool = False) -> dict:
    """(caten (!matmul a b)) with symbolic m n k as the reference lowers it (test-scheduler.lisp:126-135):
    out[n*i+j] = epilogue(sum_k a[kk*i+k] * b[..]); `transposed_b`: b is (n, kk) read through a transposed view,
    i.e. Linear's x @ W^T (nn/linear.lisp:3-17); `bias`: + bias[j]; `relu`: max(., 0) (test-scheduler.lisp:140-163).
    Arguments: val_out, m, n, kk, val_a, val_b [, val_bias]."""
    b_idx = _add(_mul("kk", "_gid1"), "_gid2") if transposed_b else _add("_gid1", _mul("n", "_gid2"))
    e = "acc"
    if bias:
        e = _add("acc", _A("val_bias", "_gid1"))
    if relu:
        e = {"op": "MAX", "args": [e, 0.0]}
    return {"name": name, "blueprint": [
        _glob("val_out", "output", 2), _glob("m", "shape", 0, "int64"), _glob("n", "shape", 0, "int64"),
        _glob("kk", "shape", 0, "int64"), _glob("val_a", "input", 2), _glob("val_b", "input", 2),
        *([_glob("val_bias", "input", 1)] if bias else []),
        {"type": "FOR", "idx": "_gid0", "upfrom": 0, "below": _lt("_gid0", "m"), "by": 1},
        {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": _lt("_gid1", "n"), "by": 1},
        {"type": "EXPR", "writes": [_A("acc", None)], "expr": 0.0, "declare_type": True, "dtype": "float32"},
        {"type": "FOR", "idx": "_gid2", "upfrom": 0, "below": _lt("_gid2", "kk"), "by": 1},
        {"type": "EXPR", "writes": [_A("acc", None)], "dtype": "float32", "reduction": True,
         "expr": _add("acc", _mul(_A("val_a", _add(_mul("kk", "_gid0"), "_gid2")), _A("val_b", b_idx)))},
        {"type": "ENDFOR", "idx": "_gid2"},
        {"type": "EXPR", "writes": [_A("val_out", _add(_mul("n", "_gid0"), "_gid1"))], "dtype": "float32", "expr": e},
        {"type": "ENDFOR", "idx": "_gid1"},
        {"type": "ENDFOR", "idx": "_gid0"},
    ]}


def embedding_onehot(name: str = "fused_embedding") -> dict:
    """Embedding as the reference computes it (nn/embedding.lisp:13-25): out[t, d] = sum_v where(v == idx[t], W[v, d], 0),
    the vocabulary index compared as a float (index-components cast to the table's dtype), `==` spelled not(!=).
    Arguments: val_out, t, d, v, val_idx, val_w."""
    eq = {"op": "NOT", "args": [{"op": "!=", "args": [{"op": "CAST", "dtype": "float32", "args": ["_gid2"]}, _A("val_idx", "_gid0")]}]}
    return {"name": name, "blueprint": [
        _glob("val_out", "output", 2), _glob("t", "shape", 0, "int64"), _glob("d", "shape", 0, "int64"),
        _glob("v", "shape", 0, "int64"), _glob("val_idx", "input", 1), _glob("val_w", "input", 2),
        {"type": "FOR", "idx": "_gid0", "upfrom": 0, "below": _lt("_gid0", "t"), "by": 1},
        {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": _lt("_gid1", "d"), "by": 1},
        {"type": "EXPR", "writes": [_A("acc", None)], "expr": 0.0, "declare_type": True, "dtype": "float32"},
        {"type": "FOR", "idx": "_gid2", "upfrom": 0, "below": _lt("_gid2", "v"), "by": 1},
        {"type": "EXPR", "writes": [_A("acc", None)], "dtype": "float32", "reduction": True,
         "expr": _add("acc", {"op": "WHERE", "args": [eq, _A("val_w", _add(_mul("d", "_gid2"), "_gid1")), 0.0]})},
        {"type": "ENDFOR", "idx": "_gid2"},
        {"type": "EXPR", "writes": [_A("val_out", _add(_mul("d", "_gid0"), "_gid1"))], "dtype": "float32", "expr": "acc"},
        {"type": "ENDFOR", "idx": "_gid1"},
        {"type": "ENDFOR", "idx": "_gid0"},
    ]}


def argmax_rows(name: str = "fused_argmax") -> dict:
    """ArgMaxNode over the last axis (api/high-level-ops.lisp:314-325): m = max(x); g = max(where(x == m, (n-1) - i, 0));
    out = cast_int64(n - g - 1) -- the lowest index among ties.  Arguments: val_out (int64), rows, n, val_x."""
    x = _A("val_x", _add(_mul("n", "_gid0"), "_gid1"))
    eq = {"op": "NOT", "args": [{"op": "!=", "args": [x, "m"]}]}
    rev = {"op": "CAST", "dtype": "float32", "args": [_add(_add("n", {"op": "NEG", "args": [1]}), _mul("_gid1", -1))]}
    loop = {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": _lt("_gid1", "n"), "by": 1}
    end = {"type": "ENDFOR", "idx": "_gid1"}
    return {"name": name, "blueprint": [
        _glob("val_out", "output", 1, "int64"), _glob("rows", "shape", 0, "int64"), _glob("n", "shape", 0, "int64"),
        _glob("val_x", "input", 2),
        {"type": "FOR", "idx": "_gid0", "upfrom": 0, "below": _lt("_gid0", "rows"), "by": 1},
        {"type": "EXPR", "writes": [_A("m", None)], "expr": float("-inf"), "declare_type": True, "dtype": "float32"},
        dict(loop),
        {"type": "EXPR", "writes": [_A("m", None)], "expr": {"op": "MAX", "args": ["m", x]}, "dtype": "float32", "reduction": True},
        dict(end),
        {"type": "EXPR", "writes": [_A("g", None)], "expr": 0.0, "declare_type": True, "dtype": "float32"},
        dict(loop),
        {"type": "EXPR", "writes": [_A("g", None)], "dtype": "float32", "reduction": True,
         "expr": {"op": "MAX", "args": ["g", {"op": "WHERE", "args": [eq, rev, 0.0]}]}},
        dict(end),
        {"type": "EXPR", "writes": [_A("val_out", "_gid0")], "dtype": "int64",
         "expr": {"op": "CAST", "dtype": "int64", "args": [_add(_add("n", {"op": "NEG", "args": ["g"]}), {"op": "NEG", "args": [1]})]}},
        {"type": "ENDFOR", "idx": "_gid0"},
    ]}


def _sub(a, b):
    return _add(a, {"op": "NEG", "args": [b]})


def add_global_2d(name: str = "fused_add_global", local=(16, 8)) -> dict:
    """z = x + y over (rows, n) after the auto-scheduler's GLOBAL directive (directive.lisp:94-117): each loop has
    become `idx = blockIdx.d * local + threadIdx.d` (an EXPR carrying its ExprGrid) and a bounds IF; the grid size is
    spelled the way astfor-mutate-global spells it.  Arguments: val_z, rows, n, val_x, val_y."""
    def bind(idx, rank, upper, loc):
        size = {"op": "CAST", "dtype": "float32", "args": [upper]}
        gs = {"op": "CAST", "dtype": "int64",
              "args": [_add(_mul(size, {"op": "RECIP", "args": [float(loc)]}), (loc - 1) / float(loc))]}  # ceil(size / local)
        sp = lambda lv: {"op": "SPACE", "level": lv, "rank": rank}  # noqa: E731
        return {"type": "EXPR", "writes": [_A(idx, None)], "declare_type": True, "dtype": "int64",
                "expr": _add(_mul(sp("block"), loc), sp("thread")), "grid": {"rank": rank, "global": gs, "local": loc}}
    idx = _add(_mul("n", "_gid0"), "_gid1")
    return {"name": name, "blueprint": [
        _glob("val_z", "output", 2), _glob("rows", "shape", 0, "int64"), _glob("n", "shape", 0, "int64"),
        _glob("val_x", "input", 2), _glob("val_y", "input", 2),
        bind("_gid0", 1, "rows", local[1]),
        {"type": "IF", "condition": _lt("_gid0", "rows")},
        bind("_gid1", 0, "n", local[0]),
        {"type": "IF", "condition": _lt("_gid1", "n")},
        {"type": "EXPR", "writes": [_A("val_z", idx)], "expr": _add(_A("val_x", idx), _A("val_y", idx)), "dtype": "float32"},
        {"type": "ENDIF"},
        {"type": "ENDIF"},
    ]}


def conv2d_relu(N, C, H, W, K, R, S, name: str = "fused_conv2d") -> dict:
    """relu(conv2d(x, w) + b), NCHW, stride 1, no padding, static shapes: the seven-loop nest the reference lowers a
    ConvND to (nn/conv.lisp: im2col-free windowed views, one reduction nest over c, r, s).  Arguments: val_y, val_x, val_w, val_b."""
    OH, OW = H - R + 1, W - S + 1
    loops = [("_gid0", N), ("_gid1", K), ("_gid2", OH), ("_gid3", OW)]
    red = [("_gid4", C), ("_gid5", R), ("_gid6", S)]
    xi = _add(_mul(C * H * W, "_gid0"), _mul(H * W, "_gid4"), _mul(W, _add("_gid2", "_gid5")), _add("_gid3", "_gid6"))
    wi = _add(_mul(C * R * S, "_gid1"), _mul(R * S, "_gid4"), _mul(S, "_gid5"), "_gid6")
    yi = _add(_mul(K * OH * OW, "_gid0"), _mul(OH * OW, "_gid1"), _mul(OW, "_gid2"), "_gid3")
    bp = [_glob("val_y", "output", 4), _glob("val_x", "input", 4), _glob("val_w", "input", 4), _glob("val_b", "input", 1)]
    bp += [{"type": "FOR", "idx": i, "upfrom": 0, "below": _lt(i, n), "by": 1} for i, n in loops]
    bp.append({"type": "EXPR", "writes": [_A("acc", None)], "expr": 0.0, "declare_type": True, "dtype": "float32"})
    bp += [{"type": "FOR", "idx": i, "upfrom": 0, "below": _lt(i, n), "by": 1} for i, n in red]
    bp.append({"type": "EXPR", "writes": [_A("acc", None)], "dtype": "float32", "reduction": True,
               "expr": _add("acc", _mul(_A("val_x", xi), _A("val_w", wi)))})
    bp += [{"type": "ENDFOR", "idx": i} for i, _ in reversed(red)]
    bp.append({"type": "EXPR", "writes": [_A("val_y", yi)], "dtype": "float32",
               "expr": {"op": "MAX", "args": [_add("acc", _A("val_b", "_gid1")), 0.0]}})
    bp += [{"type": "ENDFOR", "idx": i} for i, _ in reversed(loops)]
    return {"name": name, "blueprint": bp}


def maxpool2x2(N, C, H, W, name: str = "fused_maxpool") -> dict:
    """MaxPool 2x2 stride 2 over NCHW (nn/pool.lisp): max-reduction over the window.  Arguments: val_y, val_x."""
    OH, OW = H // 2, W // 2
    loops = [("_gid0", N * C), ("_gid1", OH), ("_gid2", OW)]
    xi = _add(_mul(H * W, "_gid0"), _mul(W, _add(_mul(2, "_gid1"), "_gid3")), _add(_mul(2, "_gid2"), "_gid4"))
    yi = _add(_mul(OH * OW, "_gid0"), _mul(OW, "_gid1"), "_gid2")
    bp = [_glob("val_y", "output", 4), _glob("val_x", "input", 4)]
    bp += [{"type": "FOR", "idx": i, "upfrom": 0, "below": _lt(i, n), "by": 1} for i, n in loops]
    bp.append({"type": "EXPR", "writes": [_A("m", None)], "expr": float("-inf"), "declare_type": True, "dtype": "float32"})
    bp += [{"type": "FOR", "idx": i, "upfrom": 0, "below": _lt(i, 2), "by": 1} for i in ("_gid3", "_gid4")]
    bp.append({"type": "EXPR", "writes": [_A("m", None)], "dtype": "float32", "reduction": True, "expr": {"op": "MAX", "args": ["m", _A("val_x", xi)]}})
    bp += [{"type": "ENDFOR", "idx": i} for i in ("_gid4", "_gid3")]
    bp.append({"type": "EXPR", "writes": [_A("val_y", yi)], "dtype": "float32", "expr": "m"})
    bp += [{"type": "ENDFOR", "idx": i} for i, _ in reversed(loops)]
    return {"name": name, "blueprint": bp}


def linear_relu_backward(name: str = "fused_relu_bias_backward") -> dict:
    """A backward item of y = relu(x @ W^T + b): dz = dy * (y > 0) written back, and db[j] = sum_i dz[i, j] -- a
    reduction over the FIRST axis, so the parallel loop is the feature axis and the batch loop stays serial inside a
    thread.  Arguments: val_dz, val_db, m, n, val_dy, val_y."""
    idx = _add(_mul("n", "_gid1"), "_gid0")
    gate = {"op": "WHERE", "args": [_lt(0.0, _A("val_y", idx)), _A("val_dy", idx), 0.0]}
    return {"name": name, "blueprint": [
        _glob("val_dz", "output", 2), _glob("val_db", "output", 1), _glob("m", "shape", 0, "int64"), _glob("n", "shape", 0, "int64"),
        _glob("val_dy", "input", 2), _glob("val_y", "input", 2),
        {"type": "FOR", "idx": "_gid0", "upfrom": 0, "below": _lt("_gid0", "n"), "by": 1},
        {"type": "EXPR", "writes": [_A("acc", None)], "expr": 0.0, "declare_type": True, "dtype": "float32"},
        {"type": "FOR", "idx": "_gid1", "upfrom": 0, "below": _lt("_gid1", "m"), "by": 1},
        {"type": "EXPR", "writes": [_A("val_dz", idx)], "expr": gate, "dtype": "float32"},
        {"type": "EXPR", "writes": [_A("acc", None)], "expr": _add("acc", gate), "dtype": "float32", "reduction": True},
        {"type": "ENDFOR", "idx": "_gid1"},
        {"type": "EXPR", "writes": [_A("val_db", "_gid0")], "expr": "acc", "dtype": "float32"},
        {"type": "ENDFOR", "idx": "_gid0"},
    ]}


# ---------------------------------------------------------------------------------------------------------------
# The Schedule-Items of one `forward` of the GPT-2 graph of apps/gpt2/gpt2.lisp:95 -- (caten (forward model (make-tensor
# `(1 s) :from 'x) (iconst 'n))) over the Transformer of external/llm/layers.lisp:73-90 -- with the sequence length `s`
# and the start position `n` symbolic and every model dimension static, the way that call compiles them.  The
# partition into items follows the reference's kernel-count tests (source/test-suite/test-scheduler.lisp:28-45,140-163,
# source/test-suite/external/test-llm.lisp:303-328, source/test-suite/test-iseq-lowerer.lisp:3-7): one kernel per
# Embedding, LayerNorm and softmax; a Linear fuses with the element-wise work behind it (bias, GELU, the residual
# add); attention is c_attn, scores (+ scale + mask), softmax, P.V, the head-merging copy and c_proj.  Argument order:
# outputs, then the dynamic shapes in use, then inputs (source/codegen/rewriting-rules.lisp:207-231).
def _shape(*names):
    return [_glob(n, "shape", 0, "int64") for n in names]


def _for(idx, below):
    return {"type": "FOR", "idx": idx, "upfrom": 0, "below": _lt(idx, below), "by": 1}


def _end(idx):
    return {"type": "ENDFOR", "idx": idx}


def _decl(name, value):
    return {"type": "EXPR", "writes": [_A(name, None)], "expr": value, "declare_type": True, "dtype": "float32"}


def _red(name, expr):
    return {"type": "EXPR", "writes": [_A(name, None)], "expr": expr, "dtype": "float32", "reduction": True}


def _store(id_, idx, expr, dtype="float32"):
    return {"type": "EXPR", "writes": [_A(id_, idx)], "expr": expr, "dtype": dtype}


def _eq(a, b):
    """`==` as the reference spells it: not(a != b) (source/api/function.lisp)"""
    return {"op": "NOT", "args": [{"op": "!=", "args": [a, b]}]}


def _f32(e):
    return {"op": "CAST", "dtype": "float32", "args": [e]}


def gpt2_embed_tokens(vocab: int, dim: int, name: str = "fused_embedding_wte") -> dict:
    """wte(tokens) (nn/embedding.lisp:13-25): out[t, d] = sum_v where(v == tok[t], W[v, d], 0).
    Arguments: val_emb, s, val_tok, val_wte."""
    return {"name": name, "blueprint": [
        _glob("val_emb", "output", 2), *_shape("s"), _glob("val_tok", "input", 2), _glob("val_wte", "input", 2),
        _for("_gid0", "s"), _for("_gid1", dim), _decl("acc", 0.0), _for("_gid2", vocab),
        _red("acc", _add("acc", {"op": "WHERE", "args": [_eq(_f32("_gid2"), _A("val_tok", "_gid0")),
                                                         _A("val_wte", _add(_mul(dim, "_gid2"), "_gid1")), 0.0]})),
        _end("_gid2"), _store("val_emb", _add(_mul(dim, "_gid0"), "_gid1"), "acc"), _end("_gid1"), _end("_gid0"),
    ]}


def gpt2_embed_positions_add(max_pos: int, dim: int, name: str = "fused_embedding_wpe_add") -> dict:
    """hi = token-emb + wpe(cast(start-pos + index-components)) (layers.lisp:80-82): the one-hot sum over the position
    table compared with n + t, the token embedding added in the store.  Arguments: val_hi, s, n, val_emb, val_wpe."""
    return {"name": name, "blueprint": [
        _glob("val_hi", "output", 2), *_shape("s", "n"), _glob("val_emb", "input", 2), _glob("val_wpe", "input", 2),
        _for("_gid0", "s"), _for("_gid1", dim), _decl("acc", 0.0), _for("_gid2", max_pos),
        _red("acc", _add("acc", {"op": "WHERE", "args": [_eq(_f32("_gid2"), _f32(_add("n", "_gid0"))),
                                                         _A("val_wpe", _add(_mul(dim, "_gid2"), "_gid1")), 0.0]})),
        _end("_gid2"),
        _store("val_hi", _add(_mul(dim, "_gid0"), "_gid1"), _add(_A("val_emb", _add(_mul(dim, "_gid0"), "_gid1")), "acc")),
        _end("_gid1"), _end("_gid0"),
    ]}


def gpt2_causal_mask(name: str = "fused_triu_mask") -> dict:
    """mask = triu(full((1 1 s n+s), -inf), diagonal = 1 + n) (layers.lisp:83; TriuNode, api/high-level-ops.lisp:278-291:
    where(i <= j - k, x, 0), `<=` spelled not(j - k < i)).  Arguments: val_mask, s, n."""
    t = _add("n", "s")
    keep = {"op": "NOT", "args": [_lt(_add("_gid1", _neg(_add(1, "n"))), "_gid0")]}
    return {"name": name, "blueprint": [
        _glob("val_mask", "output", 4), *_shape("s", "n"),
        _for("_gid0", "s"), _for("_gid1", t),
        _store("val_mask", _add(_mul(t, "_gid0"), "_gid1"), {"op": "WHERE", "args": [keep, float("-inf"), 0.0]}),
        _end("_gid1"), _end("_gid0"),
    ]}


def gpt2_layernorm(dim: int, eps: float = 1e-5, name: str = "fused_layernorm") -> dict:
    """LayerNorm over rows of a static width (nn/normalization.lisp:39-58), 1 / n folded to a single-float constant as
    the simplifier leaves it for a static shape.  Arguments: val_y, s, val_x, val_g, val_b."""
    import numpy as np
    inv = float(np.float32(1.0) / np.float32(dim))
    idx = _add(_mul(dim, "_gid0"), "_gid1")
    xi = _A("val_x", idx)
    centred = _add(xi, _neg("u"))
    rstd = {"op": "RECIP", "args": [{"op": "SQRT", "args": [_add(_mul("q", inv), eps)]}]}
    return {"name": name, "blueprint": [
        _glob("val_y", "output", 3), *_shape("s"), _glob("val_x", "input", 3), _glob("val_g", "input", 1), _glob("val_b", "input", 1),
        _for("_gid0", "s"),
        _decl("sm", 0.0), _for("_gid1", dim), _red("sm", _add("sm", xi)), _end("_gid1"),
        _decl("u", _mul("sm", inv)),
        _decl("q", 0.0), _for("_gid1", dim), _red("q", _add("q", _mul(centred, centred))), _end("_gid1"),
        _decl("r", rstd),
        _for("_gid1", dim),
        _store("val_y", idx, _add(_mul(_mul(centred, "r"), _A("val_g", "_gid1")), _A("val_b", "_gid1"))),
        _end("_gid1"), _end("_gid0"),
    ]}


def _gelu_of(x):
    """GeLU :tanh decomposed as the reference does (nn/activations.lisp:202-215; tanh and sigmoid through exp2)"""
    u = _mul(0.7978845608, _add(x, _mul(0.044715, _mul(x, _mul(x, x)))))
    sig = {"op": "RECIP", "args": [_add(1.0, {"op": "EXP2", "args": [_mul(_mul(2.0, u), -1.4426950408889634)]})]}
    return _mul(_mul(0.5, x), _add(1.0, _add(_mul(2.0, sig), -1.0)))


def gpt2_linear(n_out: int, n_in: int, bias: bool = True, gelu: bool = False, residual: bool = False,
                name: str = "fused_linear") -> dict:
    """Linear over s rows (nn/linear.lisp:3-17: x @ W^T through a transposed view of W (n_out, n_in)) fused with what
    follows it: + bias[j], GELU (c_fc, layers.lisp:53-59), + residual[t, j] (the !add of TransformerBlock, layers.lisp:69-71).
    Arguments: val_y, s, val_x, val_w [, val_b] [, val_r]."""
    e = "acc"
    if bias:
        e = _add("acc", _A("val_b", "_gid1"))
    if gelu:
        e = _gelu_of(e)
    if residual:
        e = _add(_A("val_r", _add(_mul(n_out, "_gid0"), "_gid1")), e)
    return {"name": name, "blueprint": [
        _glob("val_y", "output", 3), *_shape("s"), _glob("val_x", "input", 3), _glob("val_w", "input", 2),
        *([_glob("val_b", "input", 1)] if bias else []), *([_glob("val_r", "input", 3)] if residual else []),
        _for("_gid0", "s"), _for("_gid1", n_out), _decl("acc", 0.0), _for("_gid2", n_in),
        _red("acc", _add("acc", _mul(_A("val_x", _add(_mul(n_in, "_gid0"), "_gid2")), _A("val_w", _add(_mul(n_in, "_gid1"), "_gid2"))))),
        _end("_gid2"), _store("val_y", _add(_mul(n_out, "_gid0"), "_gid1"), e), _end("_gid1"), _end("_gid0"),
    ]}


def gpt2_cache_assign(dim: int, part: int, name: str = "fused_assign_cache") -> dict:
    """!assign of the new key (part 1) / value (part 2) rows into the cache view [n, n+s) (merge-kv-cache,
    layers.lisp:19-33): cache[(n + t), c] = qkv[t, part * dim + c]; heads and head-dim are contiguous on both sides and
    collapse into one loop.  The cache is written in place.  Arguments: val_cache, s, n, val_qkv."""
    return {"name": name, "blueprint": [
        _glob("val_cache", "output", 4), *_shape("s", "n"), _glob("val_qkv", "input", 3),
        _for("_gid0", "s"), _for("_gid1", dim),
        _store("val_cache", _add(_mul(dim, _add("n", "_gid0")), "_gid1"), _A("val_qkv", _add(_mul(3 * dim, "_gid0"), _add(part * dim, "_gid1")))),
        _end("_gid1"), _end("_gid0"),
    ]}


def gpt2_attention_scores(n_heads: int, head_dim: int, name: str = "fused_attention_scores") -> dict:
    """scores = q . k^T / sqrt(head-dim) + mask (scaled-dot-product-attention, layers.lisp:3-5) over the cache view
    [0, n+s): q is read out of the fused qkv rows, k out of the (max_len, heads, head_dim) cache, both through their
    transposed views; the division is a multiplication by the folded constant.  Batched nest of four loops as in
    source/test-suite/test-scheduler.lisp:126-138.  Arguments: val_sc, s, n, val_qkv, val_k, val_mask."""
    dim = n_heads * head_dim
    t = _add("n", "s")
    return {"name": name, "blueprint": [
        _glob("val_sc", "output", 4), *_shape("s", "n"), _glob("val_qkv", "input", 3), _glob("val_k", "input", 4), _glob("val_mask", "input", 4),
        _for("_gid0", n_heads), _for("_gid1", "s"), _for("_gid2", t), _decl("acc", 0.0), _for("_gid3", head_dim),
        _red("acc", _add("acc", _mul(_A("val_qkv", _add(_add(_mul(3 * dim, "_gid1"), _mul(head_dim, "_gid0")), "_gid3")),
                                     _A("val_k", _add(_add(_mul(dim, "_gid2"), _mul(head_dim, "_gid0")), "_gid3"))))),
        _end("_gid3"),
        _store("val_sc", _add(_add(_mul(_mul("s", t), "_gid0"), _mul(t, "_gid1")), "_gid2"),
               _add(_mul("acc", float(1.0 / head_dim ** 0.5)), _A("val_mask", _add(_mul(t, "_gid1"), "_gid2")))),
        _end("_gid2"), _end("_gid1"), _end("_gid0"),
    ]}


def gpt2_softmax_rows(n_heads: int, name: str = "fused_softmax") -> dict:
    """softmax over the last axis of (1, heads, s, n+s): heads and rows collapse into one loop of heads * s rows of
    n + s (nn/activations.lisp:59-62,107-119).  Arguments: val_y, s, n, val_x."""
    t = _add("n", "s")
    idx = _add(_mul(t, "_gid0"), "_gid1")
    ex = {"op": "EXP2", "args": [_mul(_add(_A("val_x", idx), _neg("m")), 1.4426950408889634)]}
    return {"name": name, "blueprint": [
        _glob("val_y", "output", 4), *_shape("s", "n"), _glob("val_x", "input", 4),
        _for("_gid0", _mul(n_heads, "s")),
        _decl("m", float("-inf")), _for("_gid1", t), _red("m", {"op": "MAX", "args": ["m", _A("val_x", idx)]}), _end("_gid1"),
        _decl("e", 0.0), _for("_gid1", t), _red("e", _add("e", ex)), _end("_gid1"),
        _for("_gid1", t), _store("val_y", idx, _mul(ex, {"op": "RECIP", "args": ["e"]})), _end("_gid1"),
        _end("_gid0"),
    ]}


def gpt2_attention_values(n_heads: int, head_dim: int, name: str = "fused_attention_values") -> dict:
    """out = probs . v over the cache view [0, n+s) (layers.lisp:3-5): v read in place out of the (max_len, heads,
    head_dim) cache.  Arguments: val_o, s, n, val_p, val_v."""
    dim = n_heads * head_dim
    t = _add("n", "s")
    return {"name": name, "blueprint": [
        _glob("val_o", "output", 4), *_shape("s", "n"), _glob("val_p", "input", 4), _glob("val_v", "input", 4),
        _for("_gid0", n_heads), _for("_gid1", "s"), _for("_gid2", head_dim), _decl("acc", 0.0), _for("_gid3", t),
        _red("acc", _add("acc", _mul(_A("val_p", _add(_add(_mul(_mul("s", t), "_gid0"), _mul(t, "_gid1")), "_gid3")),
                                     _A("val_v", _add(_add(_mul(dim, "_gid3"), _mul(head_dim, "_gid0")), "_gid2"))))),
        _end("_gid3"),
        _store("val_o", _add(_add(_mul(_mul(head_dim, "s"), "_gid0"), _mul(head_dim, "_gid1")), "_gid2"), "acc"),
        _end("_gid2"), _end("_gid1"), _end("_gid0"),
    ]}


def gpt2_merge_heads(n_heads: int, head_dim: int, name: str = "fused_merge_heads") -> dict:
    """(!reshape (!permute attn-output 0 2 1 3) ...) (layers.lisp:46-49): the contiguous copy that puts the heads of a
    row side by side.  Arguments: val_y, s, val_o."""
    dim = n_heads * head_dim
    return {"name": name, "blueprint": [
        _glob("val_y", "output", 3), *_shape("s"), _glob("val_o", "input", 4),
        _for("_gid0", "s"), _for("_gid1", n_heads), _for("_gid2", head_dim),
        _store("val_y", _add(_add(_mul(dim, "_gid0"), _mul(head_dim, "_gid1")), "_gid2"),
               _A("val_o", _add(_add(_mul(_mul(head_dim, "s"), "_gid1"), _mul(head_dim, "_gid0")), "_gid2"))),
        _end("_gid2"), _end("_gid1"), _end("_gid0"),
    ]}


def gpt2_argmax_last(vocab: int, name: str = "fused_argmax_last") -> dict:
    """(!argmax (!view logits t -1 t)) (layers.lisp:90; ArgMaxNode, api/high-level-ops.lisp:314-325) over the LAST row of
    the (1, s, vocab) logits: the view shows up as the offset vocab * (s - 1).  Arguments: val_out (int64), s, val_x."""
    x = _A("val_x", _add(_mul(vocab, _add("s", -1)), _add(_mul(vocab, "_gid0"), "_gid1")))
    rev = _f32(_add(_add(vocab, _neg(1)), _mul("_gid1", -1)))
    return {"name": name, "blueprint": [
        _glob("val_out", "output", 2, "int64"), *_shape("s"), _glob("val_x", "input", 3),
        _for("_gid0", 1),
        _decl("m", float("-inf")), _for("_gid1", vocab), _red("m", {"op": "MAX", "args": ["m", x]}), _end("_gid1"),
        _decl("g", 0.0), _for("_gid1", vocab),
        _red("g", {"op": "MAX", "args": ["g", {"op": "WHERE", "args": [_eq(x, "m"), rev, 0.0]}]}), _end("_gid1"),
        _store("val_out", "_gid0", {"op": "CAST", "dtype": "int64", "args": [_add(_add(vocab, _neg("g")), _neg(1))]}, "int64"),
        _end("_gid0"),
    ]}


def gpt2_step_items(cfg: dict) -> dict:
    """Every distinct Schedule-Item of one GPT-2 `forward` for the shape `cfg` (the schedule cache gives the twelve
    layers one set of kernels, source/codegen/jit.lisp:361-372)."""
    D, H, F, V, L = cfg["dim"], cfg["n_heads"], cfg["ffn"], cfg["vocab"], cfg["max_seq"]
    Dh = D // H
    return {
        "embed_tokens": gpt2_embed_tokens(V, D),
        "embed_positions": gpt2_embed_positions_add(L, D),
        "mask": gpt2_causal_mask(),
        "layernorm": gpt2_layernorm(D, cfg.get("eps", 1e-5)),
        "c_attn": gpt2_linear(3 * D, D, bias=True, name="fused_linear_c_attn"),
        "assign_k": gpt2_cache_assign(D, 1, name="fused_assign_k"),
        "assign_v": gpt2_cache_assign(D, 2, name="fused_assign_v"),
        "scores": gpt2_attention_scores(H, Dh),
        "softmax": gpt2_softmax_rows(H),
        "values": gpt2_attention_values(H, Dh),
        "merge_heads": gpt2_merge_heads(H, Dh),
        "attn_proj": gpt2_linear(D, D, bias=True, residual=True, name="fused_linear_attn_proj"),
        "c_fc": gpt2_linear(F, D, bias=True, gelu=True, name="fused_linear_c_fc_gelu"),
        "mlp_proj": gpt2_linear(D, F, bias=True, residual=True, name="fused_linear_mlp_proj"),
        "lm_head": gpt2_linear(V, D, bias=False, name="fused_linear_lm_head"),
        "argmax": gpt2_argmax_last(V),
    }


# ---------------------------------------------------------------------------------------------------------------
# Items of RoPE / SwiGLU blocks (nn/positional-encoding.lisp:3-64, nn/activations.lisp:180-189).  The reference has no
# model that uses them in a decoder (its Transformer is GPT-2 shaped), so only the element-wise items exist here;
# both run as rendered kernels.
def rope_rows(n_heads: int, head_dim: int, base: float = 10000.0, name: str = "fused_rope") -> dict:
    """`(!rope x dim)` over (1, s, heads, head_dim) with the tables computed in place, as the module builds them
    (positional-encoding.lisp:23-48): theta_i = exp(-(2i / head_dim) * log(base)) with exp(x) = exp2(x / ln 2) and
    log(x) = log2(x) * ln 2 (api/function.lisp:432-448), cos(a) = sin(a + pi/2) (api/high-level-ops.lisp:119-122);
    the two rotated halves are written into the even / odd elements of the output (the `!concatenate` of two
    strided views).  Positions are 0..s-1: the module takes no start position.  Arguments: val_y, s, val_x."""
    import math
    half = head_dim // 2
    i_f = _f32("_gid2")
    log_base = _mul({"op": "LOG2", "args": [float(base)]}, 0.6931471805599453)
    theta = {"op": "EXP2", "args": [_mul(_neg(_mul(_mul(_mul(2.0, i_f), {"op": "RECIP", "args": [float(head_dim)]}), log_base)), 1.4426950408889634)]}
    ang = _mul(_f32("_gid0"), theta)
    sin = {"op": "SIN", "args": [ang]}
    cos = {"op": "SIN", "args": [_add(ang, math.pi / 2)]}
    row = _add(_mul(n_heads * head_dim, "_gid0"), _mul(head_dim, "_gid1"))
    e0, e1 = _add(row, _mul(2, "_gid2")), _add(row, _add(_mul(2, "_gid2"), 1))
    x0, x1 = _A("val_x", e0), _A("val_x", e1)
    return {"name": name, "blueprint": [
        _glob("val_y", "output", 4), *_shape("s"), _glob("val_x", "input", 4),
        _for("_gid0", "s"), _for("_gid1", n_heads), _for("_gid2", half),
        _store("val_y", e0, _add(_mul(x0, cos), _neg(_mul(x1, sin)))),
        _store("val_y", e1, _add(_mul(x0, sin), _mul(x1, cos))),
        _end("_gid2"), _end("_gid1"), _end("_gid0"),
    ]}


def swiglu_rows(width: int, name: str = "fused_swiglu") -> dict:
    """silu(gate) * up over (s, width) (SiLU, nn/activations.lisp:180-189: x * sigmoid(x), sigmoid through exp2).
    Arguments: val_y, s, val_g, val_u."""
    idx = _add(_mul(width, "_gid0"), "_gid1")
    g = _A("val_g", idx)
    sig = {"op": "RECIP", "args": [_add(1.0, {"op": "EXP2", "args": [_mul(g, -1.4426950408889634)]})]}
    return {"name": name, "blueprint": [
        _glob("val_y", "output", 2), *_shape("s"), _glob("val_g", "input", 2), _glob("val_u", "input", 2),
        _for("_gid0", "s"), _for("_gid1", width),
        _store("val_y", idx, _mul(_mul(g, sig), _A("val_u", idx))),
        _end("_gid1"), _end("_gid0"),
    ]}
