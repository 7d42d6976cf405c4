"""Hip-Renderer: Render-IR blueprints -> programs (HIP source + route to a hand-written kernel) -> launches.

Mirrors the renderer protocol of source/codegen/renderer.lisp:30-34 (`%render-kernel`, `%compile-kernel`) as Caten's
Metal backend implements it (source/byoc/metal.lisp:152-250,326-345).  The rendering itself -- work distribution for
gfx950, spelling of the instruction set, recognition of the matmul / Linear / Embedding / ArgMax / softmax shapes and
their routing to the hand-written kernels -- lives behind the C ABI (cthip_program_*, caten_amd/csrc/render.hip), so
that a Lisp Hip-Renderer and this mirror produce the same kernels; what is left here is what the Lisp side has to do
as well: print the blueprint as an s-expression, concatenate the sources, compile once, bind, marshal arguments.

Blueprints are authored as plain dicts (so a fixture needs no Lisp image).  A Schedule-Item is
``{"name": str, "blueprint": [node...]}`` with the Render-IR node types of renderer.lisp:36-92 / aasm/attrs.lisp:298-318:

  {"type": "DEFINE-GLOBAL", "id", "dtype", "pointer_p", "arg_type": "output"|"shape"|"input", "nrank"}
  {"type": "FOR", "idx", "upfrom": expr, "below": expr, "by": expr, "scope": "local"|"global"}
  {"type": "ENDFOR", "idx"}            {"type": "IF", "condition": expr}      {"type": "ENDIF"}
  {"type": "EXPR", "writes": [aref], "expr": expr, "declare_type": bool, "dtype": str, "reduction": bool,
   "grid": {"rank": 0|1|2, "global": expr, "local": expr}}     (grid: only on the statement that binds an index to
                                                                 blockIdx / threadIdx, its ExprGrid, directive.lisp:94-117)

  expr := number | "symbol" | aref | {"op": OP, "args": [expr...]}            (OP = aasm instruction set)
        | {"op": "CAST", "dtype": str, "args": [expr]} | {"op": "CONST", "value": v, "dtype": str}
        | {"op": "SPACE", "level": "block"|"thread", "rank": 0|1|2}
        | {"op": "INDEX-COMPONENTS", "shape": [...], "strides": [...], "iterations": [...]}
  aref := {"op": "AREF", "id": str, "index": expr|None}
        | {"op": "AREF", "id": str, "space": {"strides": [expr], "views": [(from,to,by,bcast)|None], "iterations": [expr]}}

`below` is the loop condition, e.g. {"op": "<", "args": ["_gid0", "n"]} as the reference renders it
(clang.lisp:58-73).  An aref with a `space` is flattened here to the reference's index
sum_d stride_d * (from_d + by_d * gid_d) (clang.lisp:82-97), and INDEX-COMPONENTS to the linear index of
renderer.lisp:194-221, exactly as the Lisp side does with `render-aref` / `expr-index-components` before printing.
"""
from __future__ import annotations

import ctypes as C
import math
from typing import List, Optional

import numpy as np

from . import _lib
from .buffer import AbstractBuffer

CTYPES = {
    "bool": C.c_bool, "float64": C.c_double, "float32": C.c_float, "uint64": C.c_uint64, "int64": C.c_int64,
    "uint32": C.c_uint32, "int32": C.c_int32, "uint16": C.c_uint16, "int16": C.c_int16,
    "uint8": C.c_uint8, "int8": C.c_int8,
}


# ------------------------------------------------------------------ dict blueprint -> s-expression text
def _num(v) -> str:
    if isinstance(v, bool):
        return "t" if v else "nil"
    if isinstance(v, (int, np.integer)):
        return str(int(v))
    v = float(v)
    if math.isinf(v):
        return "inf" if v > 0 else "-inf"
    if math.isnan(v):
        return "nan"
    return repr(v)


def flatten_space(sp: dict):
    """iteration-space-expr-aref: sum_d stride_d * (from_d + by_d * gid_d); broadcast axes drop out."""
    terms = []
    for stride, view, it in zip(sp["strides"], sp.get("views") or [None] * len(sp["strides"]), sp["iterations"]):
        if view is not None:
            if len(view) > 3 and view[3]:
                continue
            terms.append({"op": "MUL", "args": [stride, {"op": "ADD", "args": [view[0], {"op": "MUL", "args": [view[2], it]}]}]})
        else:
            terms.append({"op": "MUL", "args": [stride, it]})
    if not terms:
        return 0
    return {"op": "ADD", "args": terms}


def flatten_index_components(e: dict):
    """expr-index-components (renderer.lisp:194-221): sum of stride * gid; an axis of size 1 contributes 0."""
    terms = [{"op": "MUL", "args": [st, it]} for sz, st, it in zip(e["shape"], e["strides"], e["iterations"])
             if not (isinstance(sz, (int, np.integer)) and int(sz) == 1)]
    if not terms:
        return 0
    return terms[0] if len(terms) == 1 else {"op": "ADD", "args": terms}


def sexp(e) -> str:
    """One expression of the dict interchange as s-expression text."""
    if e is None:  # the placeholder read of :!= / :< / :CAST (their first read is the output, renderer.lisp:381-388)
        return "nil"
    if isinstance(e, (bool, int, float, np.integer, np.floating)):
        return _num(e)
    if isinstance(e, str):
        return e.lower()
    op = e["op"].upper()
    if op == "AREF":
        if e.get("space") is not None:
            return f"(aref {e['id'].lower()} {sexp(flatten_space(e['space']))})"
        if e.get("index") is None:
            return f"(aref {e['id'].lower()})"
        return f"(aref {e['id'].lower()} {sexp(e['index'])})"
    if op == "CONST":
        return f"(const {_num(e['value'])} {e.get('dtype', 'float32')})" if "dtype" in e else f"(const {_num(e['value'])})"
    if op == "CAST":
        return f"(cast {e['dtype']} {sexp(e['args'][-1])})"
    if op == "SPACE":
        return f"(space {e['level']} {int(e['rank'])})"
    if op == "INDEX-COMPONENTS":
        return sexp(flatten_index_components(e))
    return "(" + " ".join([op.lower()] + [sexp(a) for a in e.get("args", [])]) + ")"


def item_from_sexp(text: str) -> dict:
    """A Schedule-Item that already IS interchange text (what a Lisp process prints, a golden fixture): the text is
    handed to the library as it is; only the argument list is read off it here, for marshalling."""
    import re
    body = "\n".join(ln for ln in text.splitlines() if not ln.lstrip().startswith(";"))
    m = re.search(r"\(\s*item\s+([^\s()]+)", body, re.I)
    if not m:
        raise ValueError("item_from_sexp: expected (item NAME node...)")
    globs = [{"type": "DEFINE-GLOBAL", "id": g[0].lower(), "dtype": g[1].lower(), "pointer_p": g[2].lower() == "t",
              "arg_type": g[3].lower(), "nrank": int(g[4])}
             for g in re.findall(r"\(\s*define-global\s+(\S+)\s+(\S+)\s+(\S+)\s+(\S+)\s+(\d+)\s*\)", body, re.I)]
    return {"name": m.group(1).lower(), "blueprint": globs, "sexp": text}


def item_sexp(item: dict) -> str:
    """A Schedule-Item as the text cthip_program_create reads."""
    if item.get("sexp") is not None:
        return item["sexp"]
    out = [f"(item {item['name'].lower()}"]
    for n in item["blueprint"]:
        t = n["type"]
        if t == "DEFINE-GLOBAL":
            out.append(f"  (define-global {n['id'].lower()} {n['dtype']} {'t' if n['pointer_p'] else 'nil'} "
                       f"{n['arg_type']} {int(n['nrank'])})")
        elif t == "FOR":
            out.append(f"  (for {n['idx'].lower()} {sexp(n['upfrom'])} {sexp(n['below'])} {sexp(n.get('by', 1))} "
                       f"{n.get('scope', 'local')})")
        elif t == "ENDFOR":
            out.append(f"  (endfor {n.get('idx', '').lower()})")
        elif t == "IF":
            out.append(f"  (if {sexp(n['condition'])})")
        elif t == "ENDIF":
            out.append("  (endif)")
        elif t == "EXPR":
            flags = f" :dtype {n.get('dtype', 'float32')}"
            if n.get("declare_type"):
                flags += " :declare t"
            if n.get("reduction"):
                flags += " :reduction t"
            if n.get("grid") is not None:  # ExprGrid of an index bound to blockIdx / threadIdx (directive.lisp:94-117)
                g = n["grid"]
                flags += f" :grid ({int(g['rank'])} {sexp(g['global'])} {sexp(g['local'])})"
            out.append(f"  (expr ({' '.join(sexp(w) for w in n['writes'])}) {sexp(n['expr'])}{flags})")
        else:
            out.append(f"  ({t.lower()})")  # the library reports the unknown node type
    return "\n".join(out) + ")\n"


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

    def render_expr(self, e, fdtype: str = "float32") -> str:
        """render-expr (renderer.lisp:331-411) of one expression, through a one-statement item."""
        probe = {"name": "probe", "blueprint": [
            {"type": "EXPR", "writes": [{"op": "AREF", "id": "_probe", "index": None}], "expr": e, "dtype": fdtype}]}
        src = self._create(probe, keep=False)
        line = [ln for ln in src.splitlines() if ln.strip().startswith("_probe = ")][0].strip()
        return line[len("_probe = "):-1]

    @staticmethod
    def _args(item: dict) -> List[dict]:
        return [n for n in item["blueprint"] if n["type"] == "DEFINE-GLOBAL"]

    def _create(self, item: dict, keep: bool = True) -> str:
        lib = _lib.load()
        prog = C.c_void_p()
        rc = lib.cthip_program_create(C.byref(prog), item_sexp(item).encode())
        if rc != 0:
            msg = lib.cthip_last_error().decode("utf-8", "replace")
            if rc == _lib.E_UNSUPPORTED:
                raise NotImplementedError(msg)
            raise _lib.HipError(rc, msg)
        src = lib.cthip_program_source(prog).decode()
        if keep:
            old = item.get("_program")
            if old is not None:
                lib.cthip_program_destroy(old)
            item["_program"] = prog
            item["route"] = lib.cthip_program_route(prog).decode()
        else:
            lib.cthip_program_destroy(prog)
        return src

    def render_kernel(self, item: dict) -> str:
        """%render-kernel: one `extern "C" __global__` per Schedule-Item; argument order is the
        DEFINE-GLOBAL order (outputs, dynamic shapes, inputs; rewriting-rules.lisp:207-231)."""
        item["rendered_object"] = self._create(item)
        return item["rendered_object"]

    def compile_kernel(self, items: List[dict]) -> None:
        """%compile-kernel (renderer.lisp:33; metal.lisp:326-345): concatenate header + every
        rendered-object, compile ONCE, then give each item its caller as `compiled_object`."""
        lib = _lib.load()
        code = lib.cthip_render_header().decode() + "".join(it["rendered_object"] for it in items if it.get("rendered_object"))
        self.code = code
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
            if it.get("_program") is None:  # a source that did not come from render_kernel
                raise _lib.HipError(-1, f"Caten[HIP]: {it['name']} has a rendered object but no program")
            _lib.check(lib.cthip_program_bind(it["_program"], mod))
            it["compiled_object"] = HipProgram(it["name"].lower(), it["_program"], self._args(it), self)


class HipProgram:
    """Metal-Program's role (metal.lisp:252-322): holds the program handle and the argument dtypes; calling it
    marshals Caten's argument list (coerce-dtyped-buffer has already cast the scalars, runner.lisp:25) and
    launches.  A rank-0 OUTPUT is declared as a pointer (rewriting-rules.lisp:207-231): like the CLANG backend
    (clang.lisp:166-185) the number is boxed -- here in an 8-byte device cell -- and written back after the call."""

    def __init__(self, name: str, program, defglobals: List[dict], renderer: HipRenderer):
        self.name, self.program, self.defglobals, self.renderer = name, program, defglobals, renderer
        # the argument block is built once: one ctypes cell per DEFINE-GLOBAL (a pointer or a by-value scalar of the
        # declared dtype) and the array of their addresses cthip_program_launch takes; a call only stores values
        self._cells = [C.c_void_p() if g["pointer_p"] else CTYPES[g["dtype"]]() for g in defglobals]
        self._argv = (C.c_void_p * len(self._cells))(*[C.addressof(c) for c in self._cells])
        self._pointer = [bool(g["pointer_p"]) for g in defglobals]
        self._launch = _lib.load().cthip_program_launch

    @property
    def last_route(self) -> str:
        return _lib.load().cthip_program_last_route(self.program).decode()

    def __call__(self, node, *args):
        if len(args) != len(self._cells):
            raise AssertionError(f"HIP: {self.name} takes {len(self.defglobals)} arguments, got {len(args)}")
        boxed = None
        for k, a in enumerate(args):
            if self._pointer[k]:
                if isinstance(a, AbstractBuffer) and a.nrank > 0:
                    v = a.value
                    if not isinstance(v, int):
                        raise TypeError(f"HIP: please transfer the buffer {self.defglobals[k]['id']} to the device first")
                    self._cells[k].value = v
                elif isinstance(a, (AbstractBuffer, bool, int, float, np.number)):
                    # a rank-0 value passed by pointer: a one-element device cell holding the number
                    boxed = self._box(k, a, boxed)
                else:
                    raise TypeError(f"HIP: argument {self.defglobals[k]['id']} must be a device buffer")
            else:
                self._cells[k].value = a.value if isinstance(a, AbstractBuffer) else a
        if boxed is None:
            rc = self._launch(self.program, self._argv, len(self._cells))
            if rc != 0:
                _lib.check(rc)
            return
        lib = _lib.load()
        try:
            _lib.check(self._launch(self.program, self._argv, len(self._cells)))
            for cell, host, a in boxed:  # write the scalars back (synchronises, as the CLANG call does)
                _lib.check(lib.cthip_d2h(C.byref(host), cell, C.sizeof(host)))
                if isinstance(a, AbstractBuffer):
                    a.value = host.value
        finally:
            for cell, _h, _a in boxed:
                lib.cthip_free(cell)

    def _box(self, k, a, boxed):
        lib = _lib.load()
        v = a.value if isinstance(a, AbstractBuffer) else a
        host = CTYPES[self.defglobals[k]["dtype"]](v)
        cell = C.c_void_p()
        _lib.check(lib.cthip_alloc(C.byref(cell), 8))
        _lib.check(lib.cthip_h2d(cell, C.byref(host), C.sizeof(host)))
        self._cells[k].value = cell.value
        boxed = boxed or []
        boxed.append((cell, host, a))
        return boxed
