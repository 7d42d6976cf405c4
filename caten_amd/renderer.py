"""Hip-Renderer: Render-IR blueprints -> HIP source -> launchable kernels.

Mirrors the renderer protocol of source/codegen/renderer.lisp:30-34
(`%render-kernel`, `%compile-kernel`, `%render-node`) as Caten's Metal backend
implements it (source/byoc/metal.lisp:152-250,326-345), for every Schedule-Item
that is not matched to a hand-written kernel.

Interchange format (plain dicts, so a blueprint can be authored or exported
without a Lisp image).  A Schedule-Item is ``{"name": str, "blueprint": [node...]}``
with the Render-IR node types of renderer.lisp:36-92 / aasm/attrs.lisp:298-318:

  {"type": "DEFINE-GLOBAL", "id", "dtype", "pointer_p", "arg_type": "output"|"shape"|"input", "nrank"}
  {"type": "FOR", "idx", "upfrom": expr, "below": expr, "by": expr, "scope": "local"|"global"}
  {"type": "ENDFOR", "idx"}            {"type": "IF", "condition": expr}      {"type": "ENDIF"}
  {"type": "EXPR", "writes": [aref], "expr": expr, "declare_type": bool, "dtype": str, "reduction": bool}

  expr := number | "symbol" | aref | {"op": OP, "args": [expr...]}            (OP = aasm instruction set)
        | {"op": "CAST", "dtype": str, "args": [expr]} | {"op": "CONST", "value": v, "dtype": str}
        | {"op": "SPACE", "level": "block"|"thread", "rank": 0|1|2}
  aref := {"op": "AREF", "id": str, "index": expr|None}
        | {"op": "AREF", "id": str, "space": {"strides": [expr], "views": [(from,to,by,bcast)|None], "iterations": [expr]}}

`below` is the loop condition, e.g. {"op": "<", "args": ["_gid0", "n"]} as the reference renders it
(clang.lisp:58-73).  An aref with a `space` gets the reference's index
sum_d stride_d * (from_d + by_d * gid_d) (clang.lisp:82-97).

Work distribution (the reference leaves every loop serial at OPTIMIZE=1, so its
Metal kernels run in one thread, metal.lisp:341-345): the outermost perfectly
nested loops whose index appears in every global write below them are
data-parallel; they are flattened into one global thread id, innermost loop
fastest so that consecutive lanes touch consecutive addresses, and launched as
256-thread workgroups with a bounds guard.  Reduction loops stay serial inside a
thread.  Loops already marked ``scope: global`` are always mapped to threads.

Row reductions (softmax, LayerNorm, RMSNorm, sums over the last axis: a parallel prefix whose body is a
sequence of scalar statements and loops over one more axis, some of them reductions into scalars that start
at their operation's identity) get one WAVEFRONT per row instead of one thread: the 64 lanes stride the inner
axis together, so consecutive lanes read consecutive addresses, every lane keeps a partial, and the partials
meet in a `__shfl_xor` butterfly after the loop; statements between the loops run redundantly in all lanes
and only lane 0 performs their global writes.

Spelling follows the CStyle renderer (renderer.lisp:314-411) with two deliberate
differences for fp32 kernels: literals carry an `f` suffix and the libm calls are
the float ones, so arithmetic stays in fp32 registers instead of promoting to
double; results differ from the CLANG backend by a few ulp at most.
"""
from __future__ import annotations

import ctypes as C
import math
from typing import Any, Dict, List, Optional

import numpy as np

from . import _lib
from .buffer import AbstractBuffer, DTYPES

CDTYPE = {  # ->cdtype (source/codegen/helpers.lisp:101-113)
    "bool": "bool", "float64": "double", "float32": "float", "float16": "_Float16",
    "uint64": "unsigned long long", "int64": "long long", "uint32": "unsigned int", "int32": "int",
    "uint16": "unsigned short", "int16": "short", "uint8": "unsigned char", "int8": "signed char",
}
CTYPES = {
    "bool": C.c_bool, "float64": C.c_double, "float32": C.c_float, "uint64": C.c_uint64, "int64": C.c_int64,
    "uint32": C.c_uint32, "int32": C.c_int32, "uint16": C.c_uint16, "int16": C.c_int16,
    "uint8": C.c_uint8, "int8": C.c_int8,
}

HEADER = """
#define _infinity __builtin_inff()
#define _negative_infinity (-__builtin_inff())
#define _nan __builtin_nanf("")
#define ct_max(a, b) ((a) > (b) ? (a) : (b))
#define ct_min(a, b) ((a) < (b) ? (a) : (b))
// reductions over the 64 lanes of a wavefront (every lane gets the result)
#define CT_WAVE_REDUCE(name, T, OP)                                        \\
  static __device__ __forceinline__ T name(T v) {                          \\
    for (int o = 32; o > 0; o >>= 1) { T w = __shfl_xor(v, o, 64); v = OP; } \\
    return v;                                                              \\
  }
CT_WAVE_REDUCE(ct_wave_add_f, float, v + w)
CT_WAVE_REDUCE(ct_wave_max_f, float, ct_max(v, w))
CT_WAVE_REDUCE(ct_wave_min_f, float, ct_min(v, w))
CT_WAVE_REDUCE(ct_wave_mul_f, float, v * w)
"""

BLOCK = 256


class Renderer:
    """Renderer protocol (renderer.lisp:30-34)."""

    def render_kernel(self, item: dict) -> str:
        raise NotImplementedError

    def compile_kernel(self, items: List[dict]) -> None:
        raise NotImplementedError


class HipRenderer(Renderer):
    def __init__(self, arch: str = "gfx950"):
        self.arch = arch
        self.module = None
        self.code = ""

    # ------------------------------------------------------------ expressions
    def render_const(self, v, dtype: Optional[str] = None) -> str:
        """%render-const (renderer.lisp:319-329)"""
        if isinstance(v, bool):
            return "true" if v else "false"
        if isinstance(v, float) or (dtype or "").startswith("float"):
            v = float(v)
            if math.isinf(v):
                return "_infinity" if v > 0 else "_negative_infinity"
            if math.isnan(v):
                return "_nan"
            if dtype == "float64":
                return f"{v:.17g}" if ("e" in f"{v:.17g}" or "." in f"{v:.17g}") else f"{v:.17g}.0"
            s = np.format_float_positional(np.float32(v), unique=True)
            if s.endswith("."):
                s += "0"
            return s + "f"
        return str(int(v))

    def render_expr(self, e, fdtype: str = "float32") -> str:
        """render-expr / %render-node dispatch (renderer.lisp:331-411)"""
        if isinstance(e, bool):
            return "true" if e else "false"
        if isinstance(e, (int, np.integer)):
            return str(int(e))
        if isinstance(e, float):
            return self.render_const(e, fdtype)
        if isinstance(e, str):
            return e.lower()
        op = e["op"].upper()
        a = e.get("args", [])
        r = lambda x: self.render_expr(x, fdtype)  # noqa: E731
        f64 = fdtype == "float64"
        if op == "CONST":
            return self.render_const(e["value"], e.get("dtype", fdtype))
        if op == "AREF":
            return self.render_aref(e, fdtype)
        if op == "SPACE":  # metal.lisp:173-176 -> blockIdx / threadIdx
            return f"{'blockIdx' if e['level'] == 'block' else 'threadIdx'}.{'xyz'[e['rank']]}"
        if op in ("ADD", "MUL", "MOD", "IDIV", "AND", "OR", "XOR"):
            sym = {"ADD": "+", "MUL": "*", "MOD": "%", "IDIV": "/", "AND": " & ", "OR": " | ", "XOR": " ^ "}[op]
            return "(" + sym.join(r(x) for x in a) + ")"
        if op == "WMMA":
            return f"({r(a[0])}+{r(a[1])}*{r(a[2])})"
        if op == "MAX":
            return f"ct_max({r(a[0])}, {r(a[1])})"
        if op == "NEG":
            return f"(-{r(a[0])})"
        if op == "NOT":
            return f"(!{r(a[0])})"
        if op in ("SIN", "LOG2", "EXP2", "SQRT"):
            return f"{op.lower()}{'' if f64 else 'f'}({r(a[0])})"
        if op == "RECIP":
            if e.get("dtype", fdtype).startswith("float"):
                return f"({'1.0' if f64 else '1.0f'}/({r(a[0])}))"
            return f"(1/({r(a[0])}))"
        if op in ("!=", "<"):
            x, y = a[-2], a[-1]
            return f"({r(x)}{op}{r(y)})"
        if op in ("MOVE", "STORE"):
            return r(a[-1])
        if op == "CAST":
            return f"(({CDTYPE[e['dtype']]}){r(a[-1])})"
        if op == "WHERE":
            return f"({r(a[0])} ? {r(a[1])} : {r(a[2])})"
        if op == "INDEX-COMPONENTS":
            # expr-index-components (renderer.lisp:194-221): the linear index of the element being computed,
            # sum of stride * gid over the axes of the iteration space; an axis of size 1 contributes 0
            terms = [{"op": "MUL", "args": [st, it]} for sz, st, it in zip(e["shape"], e["strides"], e["iterations"])
                     if not (isinstance(sz, (int, np.integer)) and int(sz) == 1)]
            if not terms:
                return "0"
            return self.render_expr(terms[0] if len(terms) == 1 else {"op": "ADD", "args": terms}, "int64")
        raise NotImplementedError(f"Hip-Renderer: no %render-node method for :{op}")

    def render_aref(self, e: dict, fdtype: str = "float32") -> str:
        """render-aref (renderer.lisp:134-192; index form of clang.lisp:82-97)"""
        name = e["id"].lower()
        if "space" in e and e["space"] is not None:
            sp = e["space"]
            terms = []
            for stride, view, it in zip(sp["strides"], sp.get("views") or [None] * len(sp["strides"]), sp["iterations"]):
                if view is not None:
                    frm, _to, by = view[0], view[1], view[2]
                    if len(view) > 3 and view[3]:
                        continue  # broadcast axis: stride 0
                    terms.append({"op": "MUL", "args": [stride, {"op": "ADD", "args": [frm, {"op": "MUL", "args": [by, it]}]}]})
                else:
                    terms.append({"op": "MUL", "args": [stride, it]})
            if not terms:
                return f"{name}[0]"
            return f"{name}[{self.render_expr({'op': 'ADD', 'args': terms}, 'int64')}]"
        idx = e.get("index")
        if idx is None:
            return name
        return f"{name}[{self.render_expr(idx, 'int64')}]"

    # ------------------------------------------------------------ kernels
    @staticmethod
    def _args(item: dict) -> List[dict]:
        return [n for n in item["blueprint"] if n["type"] == "DEFINE-GLOBAL"]

    @staticmethod
    def _uses(e, sym: str) -> bool:
        if isinstance(e, str):
            return e.lower() == sym.lower()
        if isinstance(e, dict):
            if e.get("op") == "AREF" and e.get("index") is None and "space" not in e and e["id"].lower() == sym.lower():
                return True  # a scalar named by an aref
            if any(HipRenderer._uses(x, sym) for x in e.get("args", [])):
                return True
            if e.get("index") is not None and HipRenderer._uses(e["index"], sym):
                return True
            sp = e.get("space")
            if sp and any(HipRenderer._uses(x, sym) for x in sp["iterations"]):
                return True
            if e.get("op") == "INDEX-COMPONENTS":
                return any(HipRenderer._uses(x, sym) for x in list(e["iterations"]) + list(e["strides"]))
        return False

    def _parallel_prefix(self, body: List[dict]) -> int:
        """How many leading FOR nodes of `body` (a perfect nest) are data-parallel."""
        depth = 0
        i = 0
        while i < len(body) and body[i]["type"] == "FOR":
            f = body[i]
            # find the matching ENDFOR; the nest is perfect when it is the last node
            lvl, j = 0, i
            while True:
                t = body[j]["type"]
                if t == "FOR":
                    lvl += 1
                elif t == "ENDFOR":
                    lvl -= 1
                    if lvl == 0:
                        break
                j += 1
            if j != len(body) - 1 - depth:
                break
            inner = body[i + 1:j]
            ok = True
            if f.get("scope") != "global":
                for n in inner:
                    if n["type"] != "EXPR":
                        continue
                    for w in n["writes"]:
                        local = n.get("declare_type") or w.get("index") is None and "space" not in w
                        if w["id"].lower() in self._locals:
                            local = True
                        if not local and not self._uses(w, f["idx"]):
                            ok = False
                if not (self._is_zero(f["upfrom"]) and self._upper_bound(f) is not None):
                    ok = False
            if not ok:
                break
            depth += 1
            i += 1
        return depth

    _IDENTITY = {"ADD": ("add", 0.0), "MAX": ("max", float("-inf")), "MIN": ("min", float("inf")), "MUL": ("mul", 1.0)}

    @staticmethod
    def _const_value(e):
        if isinstance(e, (int, float, np.integer, np.floating)) and not isinstance(e, bool):
            return float(e)
        if isinstance(e, dict) and e.get("op") == "CONST" and isinstance(e.get("value"), (int, float)):
            return float(e["value"])
        if isinstance(e, dict) and e.get("op") == "NEG" and len(e.get("args", [])) == 1:
            v = HipRenderer._const_value(e["args"][0])
            return None if v is None else -v
        return None

    def _wave_reductions(self, body: List[dict]):
        """If `body` (what is left inside the parallel prefix) is a row-reduction pattern, returns
        {position of an ENDFOR: [(scalar, op)...]} = the scalars to combine across lanes after that loop;
        otherwise None (the row then stays in one thread)."""
        depth, init, found = 0, {}, {}
        loop_red: List = []
        for pos, n in enumerate(body):
            t = n["type"]
            if t == "FOR":
                depth += 1
                by = n.get("by", 1)
                if depth > 1 or n.get("scope") == "global" or not (isinstance(by, (int, np.integer)) and int(by) == 1):
                    return None
                loop_red = []
            elif t == "ENDFOR":
                depth -= 1
                if loop_red:
                    found[pos] = loop_red
                loop_red = []
            elif t in ("IF", "ENDIF"):
                return None
            elif t == "EXPR":
                if len(n["writes"]) != 1:
                    return None
                w = n["writes"][0]
                scalar = w.get("index") is None and "space" not in w
                name = w["id"].lower()
                if depth == 0:
                    if scalar:
                        init[name] = self._const_value(n["expr"])  # None: not a constant
                    continue
                if not n.get("reduction"):
                    if scalar:
                        return None  # a loop-carried scalar that is not a reduction cannot be split over lanes
                    continue
                if n.get("dtype", "float32") != "float32":
                    return None  # the lane butterflies are fp32
                e = n["expr"]
                if not (scalar and isinstance(e, dict) and e.get("op", "").upper() in self._IDENTITY and len(e.get("args", [])) == 2):
                    return None
                op, ident = self._IDENTITY[e["op"].upper()]
                args = e["args"]
                selfref = [isinstance(x, str) and x.lower() == name or isinstance(x, dict) and x.get("op") == "AREF"
                           and x["id"].lower() == name and x.get("index") is None and "space" not in x for x in args]
                if sum(selfref) != 1 or self._uses(args[1 - selfref.index(True)], name):
                    return None
                # lane partials combine when each starts at the identity; max / min are idempotent, so there any
                # start value that all lanes share (a scalar set before the loop) will do
                if init.get(name) != ident and not (op in ("max", "min") and name in init):
                    return None
                loop_red.append((name, op))
        return found or None

    @staticmethod
    def _is_zero(e) -> bool:
        return isinstance(e, (int, np.integer)) and int(e) == 0 or (isinstance(e, dict) and e.get("op") == "CONST" and e["value"] == 0)

    @staticmethod
    def _upper_bound(f: dict):
        """`below` is the condition (idx < N); returns N when it has that shape and by == 1."""
        b = f["below"]
        by = f.get("by", 1)
        if not (isinstance(by, (int, np.integer)) and int(by) == 1):
            return None
        if isinstance(b, dict) and b.get("op") == "<":
            x, y = b["args"][-2], b["args"][-1]
            if isinstance(x, str) and x.lower() == f["idx"].lower():
                return y
        return None

    def render_kernel(self, item: dict) -> str:
        """%render-kernel: one `extern "C" __global__` per Schedule-Item; argument order is the
        DEFINE-GLOBAL order (outputs, dynamic shapes, inputs; rewriting-rules.lisp:207-231)."""
        args = self._args(item)
        body = [n for n in item["blueprint"] if n["type"] != "DEFINE-GLOBAL"]
        self._locals = {w["id"].lower() for n in body if n["type"] == "EXPR" and n.get("declare_type")
                        for w in n["writes"]}
        params = []
        for a in args:
            ct = CDTYPE[a["dtype"]]
            if a["pointer_p"]:
                const = "const " if a["arg_type"] == "input" else ""
                restrict = " __restrict__" if a["arg_type"] == "input" else ""
                params.append(f"{const}{ct}*{restrict} {a['id'].lower()}")
            else:
                params.append(f"const {ct} {a['id'].lower()}")
        out = [f'extern "C" __global__ void __launch_bounds__({BLOCK}) {item["name"].lower()}({", ".join(params)}) {{']
        npar = self._parallel_prefix(body)
        grid_bounds = []
        indent = 2
        pad = lambda: " " * indent  # noqa: E731
        wave_red = self._wave_reductions(body[npar:len(body) - npar]) if npar else None
        item["_rows_per_block"] = BLOCK
        if npar:
            loops = body[:npar]
            bounds = [self._upper_bound(f) for f in loops]
            grid_bounds = bounds
            total = "*".join(f"(long long)({self.render_expr(b, 'int64')})" for b in bounds)
            out.append(f"{pad()}const long long _total = {total};")
            if wave_red is not None:
                item["_rows_per_block"] = BLOCK // 64
                out.append(f"{pad()}long long _t = ((long long)blockIdx.x * {BLOCK} + threadIdx.x) >> 6;  // one wavefront per row")
                out.append(f"{pad()}const int _lane = threadIdx.x & 63;")
            else:
                out.append(f"{pad()}long long _t = (long long)blockIdx.x * {BLOCK} + threadIdx.x;")
            out.append(f"{pad()}if (_t >= _total) return;")
            for f, b in zip(reversed(loops), reversed(bounds)):  # innermost loop varies fastest
                bs = self.render_expr(b, "int64")
                out.append(f"{pad()}const int {f['idx'].lower()} = (int)(_t % (long long)({bs})); _t /= (long long)({bs});")
            body = body[npar:len(body) - npar]
        depth = 0
        closers: List[str] = []  # what ends each open loop
        for pos, n in enumerate(body):
            t = n["type"]
            if t == "FOR":
                if wave_red is not None:  # the lanes of the row's wavefront stride this axis together
                    lo, hi = self._const_value(n["upfrom"]), self._const_value(self._upper_bound(n))
                    idx = n["idx"].lower()
                    if lo is not None and hi is not None and float(lo).is_integer() and float(hi).is_integer() \
                            and 0 < (int(hi) - int(lo) + 63) // 64 <= 32:
                        # a static row of at most 32 elements per lane: a counted loop, unrolled, so that the loops
                        # over the same row share their loads (inputs are __restrict__) and the row is read once
                        lo, hi = int(lo), int(hi)
                        out.append(f"{pad()}#pragma unroll")
                        out.append(f"{pad()}for (int {idx}_i=0; {idx}_i<{(hi - lo + 63) // 64}; {idx}_i++) {{ "
                                   f"const int {idx}={lo}+_lane+64*{idx}_i;" + (f" if ({idx}<{hi}) {{" if (hi - lo) % 64 else ""))
                        closers.append("}}" if (hi - lo) % 64 else "}")
                    else:
                        out.append(f"{pad()}for (int {idx}=({self.render_expr(n['upfrom'], 'int64')})+_lane; "
                                   f"{self.render_expr(n['below'], 'int64')}; {idx}+=64) {{")
                        closers.append("}")
                else:
                    out.append(f"{pad()}for (int {n['idx'].lower()}={self.render_expr(n['upfrom'], 'int64')}; "
                               f"{self.render_expr(n['below'], 'int64')}; {n['idx'].lower()}+={self.render_expr(n.get('by', 1), 'int64')}) {{")
                    closers.append("}")
                indent += 2
                depth += 1
            elif t == "ENDFOR":
                indent -= 2
                depth -= 1
                out.append(f"{pad()}{closers.pop()}")
                if wave_red is not None:
                    for var, op in wave_red.get(pos, []):
                        out.append(f"{pad()}{var} = ct_wave_{op}_f({var});")
            elif t == "IF":
                out.append(f"{pad()}if ({self.render_expr(n['condition'], 'int64')}) {{")
                indent += 2
            elif t == "ENDIF":
                indent -= 2
                out.append(f"{pad()}}}")
            elif t == "EXPR":
                dt = n.get("dtype", "float32")
                lhs = ", ".join(self.render_aref(w, dt) for w in n["writes"])
                decl = f"{CDTYPE[dt]} " if n.get("declare_type") else ""
                stmt = f"{decl}{lhs} = {self.render_expr(n['expr'], dt)};"
                if wave_red is not None and depth == 0 and not n.get("declare_type") and \
                        any(w["id"].lower() not in self._locals for w in n["writes"]):
                    stmt = f"if (_lane == 0) {{ {stmt} }}"  # every lane holds the value; one of them stores it
                out.append(f"{pad()}{stmt}")
            else:
                raise NotImplementedError(f"Hip-Renderer: unknown blueprint node :{t}")
        out.append("}")
        item["_grid_bounds"] = grid_bounds
        item["rendered_object"] = "\n".join(out) + "\n"
        return item["rendered_object"]

    def compile_kernel(self, items: List[dict]) -> None:
        """%compile-kernel (renderer.lisp:33; metal.lisp:326-345): concatenate header + every
        rendered-object, compile ONCE, then give each item its caller as `compiled_object`."""
        code = HEADER + "".join(it["rendered_object"] for it in items if it.get("rendered_object"))
        self.code = code
        lib = _lib.load()
        blob, n, log = C.c_void_p(), C.c_size_t(), C.c_void_p()
        rc = lib.cthip_compile(code.encode(), self.arch.encode(), C.byref(blob), C.byref(n), C.byref(log))
        if rc != 0:
            text = C.cast(log, C.c_char_p).value.decode("utf-8", "replace") if log.value else ""
            if log.value:
                lib.cthip_release(log)
            raise _lib.HipError(rc, f"Caten[HIP]: Failed to compile the kernels:\n{text}\n\n"
                                    f"Compiled with hipRTC --offload-arch={self.arch} -O3")
        self.code_object = C.string_at(blob.value, n.value)
        lib.cthip_release(blob)
        if not _lib.is_initialised():
            # no device in this process: the code object exists, callers are bound at first use
            for it in items:
                if it.get("rendered_object"):
                    it["compiled_object"] = None
            return
        mod = C.c_void_p()
        _lib.check(lib.cthip_module_load(C.byref(mod), self.code_object))
        self.module = mod
        for it in items:
            if not it.get("rendered_object"):
                continue
            fn = C.c_void_p()
            _lib.check(lib.cthip_get_function(C.byref(fn), mod, it["name"].lower().encode()))
            it["compiled_object"] = HipProgram(it["name"].lower(), fn, self._args(it), it["_grid_bounds"], self,
                                               it.get("_rows_per_block", BLOCK))


class HipProgram:
    """Metal-Program's role (metal.lisp:252-322): holds the function handle, the argument
    dtypes and the grid expression; calling it marshals Caten's argument list and launches."""

    def __init__(self, name: str, fn, defglobals: List[dict], grid_bounds: list, renderer: HipRenderer,
                 rows_per_block: int = BLOCK):
        self.name, self.fn, self.defglobals, self.grid_bounds, self.renderer = name, fn, defglobals, grid_bounds, renderer
        self.rows_per_block = rows_per_block  # parallel iterations one 256-thread workgroup covers

    def _eval(self, e, env: Dict[str, Any]) -> int:
        if isinstance(e, (int, np.integer)):
            return int(e)
        if isinstance(e, str):
            return int(env[e.lower()])
        op = e["op"].upper()
        a = [self._eval(x, env) for x in e.get("args", [])]
        if op == "CONST":
            return int(e["value"])
        if op == "ADD":
            return sum(a)
        if op == "MUL":
            return int(np.prod(a))
        if op == "IDIV":
            return a[0] // a[1]
        if op == "MOD":
            return a[0] % a[1]
        if op == "NEG":
            return -a[0]
        if op == "MAX":
            return max(a)
        raise NotImplementedError(f"grid expression op {op}")

    def __call__(self, node, *args):
        if len(args) != len(self.defglobals):
            raise AssertionError(f"HIP: {self.name} takes {len(self.defglobals)} arguments, got {len(args)}")
        env, boxed = {}, []
        for a, g in zip(args, self.defglobals):
            if g["pointer_p"]:
                if isinstance(a, AbstractBuffer) and a.nrank > 0:
                    if not isinstance(a.value, int):
                        raise TypeError(f"HIP: please transfer the buffer {g['id']} to the device first")
                    boxed.append(C.c_void_p(a.value))
                else:
                    raise TypeError(f"HIP: argument {g['id']} must be a device buffer")
            else:
                v = a.value if isinstance(a, AbstractBuffer) else a
                env[g["id"].lower()] = v
                boxed.append(CTYPES[g["dtype"]](v))
        total = 1
        for b in self.grid_bounds:
            total *= max(self._eval(b, env), 0)
        per = self.rows_per_block
        grid = (C.c_uint * 3)((total + per - 1) // per if self.grid_bounds else 1, 1, 1)
        block = (C.c_uint * 3)(BLOCK if self.grid_bounds else 1, 1, 1)
        argv = (C.c_void_p * len(boxed))(*[C.cast(C.pointer(b), C.c_void_p) for b in boxed])
        _lib.check(_lib.load().cthip_launch(self.fn, grid, block, 0, argv, len(boxed)))
