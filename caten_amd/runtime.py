"""HipRuntime: the VM half of the `:HIP` backend.

Mirrors Caten's GraphRuntime (source/runtime/runtime.lisp:39-145,228-284) and the
JIT_KERNEL node (source/codegen/jit.lisp:92-143, source/codegen/runner.lisp:20-32):
a program counter walks a flat node list; `:Allocate` opens (or reuses) buffers,
`:View` re-describes storage without moving data, `:JIT_KERNEL` launches one
compiled kernel and returns the arguments at its out-positions.  Custom,
non-rendered ops (the hand-written fused kernels) are ordinary node types with a
`realize_node` method, the extension mechanism of source/runtime/runtime.lisp:118.

The graph is handed over as plain data (see `Node`): in a Lisp process the same
walk is driven by Caten itself and only the C ABI below it is shared.
"""
from __future__ import annotations

import ctypes as C
import os
import time
import weakref
from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional, Sequence

import numpy as np

from . import _lib
from .backend import define_backend
from .buffer import (AbstractBuffer, DTYPES, HipBuffer, close_buffer, make_buffer, open_buffer,
                     transfer_from_array, transfer_into_array)


@dataclass
class Node:
    """caten/air Node: type, writes, reads and an attribute plist."""
    type: str
    writes: List[str]
    reads: List[Any]
    attrs: Dict[str, Any] = field(default_factory=dict)


class RuntimeError_(RuntimeError):
    """runtime-error (runtime.lisp:84-104): carries the pc and a disassembly."""

    def __init__(self, runtime: "GraphRuntime", cond: BaseException):
        lines = []
        for i, n in enumerate(runtime.graph):
            lines.append(f"{'*' if i == runtime.pc else ' '}{i} | {n.type} {n.writes} <- {n.reads}")
        super().__init__(f"Runtime-Error: Encountered the runtime error at instruction {runtime.pc}.\n"
                         f"condition:\n  {cond}\ndisassemble:\n" + "\n".join(lines))
        self.cond = cond


@dataclass
class CompiledKernel:
    """Compiled-Kernel (jit.lisp:92-103)."""
    name: str
    caller: Callable
    device: str = "HIP"
    code: str = ""
    out_positions: Sequence[int] = (0,)
    flops: Optional[int] = None


def coerce_dtyped_buffer(arg, dtype: str):
    """coerce-dtyped-buffer (source/codegen/helpers.lisp:118-125): rank-0 buffers are
    passed by value, cast to the declared dtype."""
    if isinstance(arg, AbstractBuffer):
        if arg.nrank == 0:
            return DTYPES[dtype](arg.value).item()
        return arg
    return DTYPES[dtype](arg).item()


class GraphRuntime:
    buffer_type = AbstractBuffer

    def __init__(self, graph: List[Node], fw_outputs: Sequence[str] = (), variables: Optional[dict] = None,
                 renderer=None):
        self.graph = list(graph)
        self.fw_outputs = list(fw_outputs)
        self.variables: Dict[Any, Any] = dict(variables or {})
        self.renderer = renderer
        self.pc = 0
        self.profile = os.environ.get("PROFILE", "0") == "1"
        self.times = {"kernel": 0.0, "vm": 0.0, "allocate": 0.0}
        self._casts: List[AbstractBuffer] = []  # storage opened by :View nodes that cast a scalar to an array
        self._methods: Dict[str, Callable] = {}  # node type -> its realize-node method

    # runtime-setvar / runtime-getvar (runtime.lisp:66-74)
    def setvar(self, var, value):
        if not (isinstance(value, (int, float, bool, np.number, AbstractBuffer))):
            raise TypeError(f"Runtime: the value {value!r} is not one of AbstractBuffer, number, boolean")
        self.variables[var] = value

    def getvar(self, var):
        if var not in self.variables:
            raise KeyError(f"Runtime: the variable {var} is not defined in the graph.")
        return self.variables[var]

    def step(self) -> bool:
        """runtime-step (runtime.lisp:106-132)"""
        node = self.graph[self.pc]
        t1 = time.perf_counter() if self.profile else 0.0
        variables = self.variables
        try:
            args = [a if type(a) is int or type(a) is float else (variables[a] if a in variables else self.getvar(a))
                    for a in node.reads]
            out = self.realize_node(node, args)
        except Exception as e:  # wrapped like handler-bind ... runtime-error
            raise RuntimeError_(self, e) from e
        if self.profile and node.type != "JIT_KERNEL":
            self.times["allocate" if node.type == "Allocate" else "vm"] += time.perf_counter() - t1
        writes = node.writes
        if len(writes) == 1 and not isinstance(out, tuple):
            self.setvar(writes[0], out)
        else:
            if not isinstance(out, tuple):
                out = (out,)
            if writes and len(out) != len(writes):
                raise RuntimeError_(self, AssertionError("Runtime: the number of outputs does not match the number of writes."))
            for place, value in zip(writes, out):
                self.setvar(place, value)
        self.pc += 1
        return True

    def forward(self, *params):
        """runtime-forward after runtime-set-params (api/iseq.lisp:481-529): params are
        (symbol, buffer-or-number) pairs; returns the fw-outputs."""
        for k, v in params:
            self.setvar(k, v)
        self.pc = 0
        while self.pc < len(self.graph):
            self.step()
        outs = tuple(self.getvar(o) for o in self.fw_outputs)
        return outs[0] if len(outs) == 1 else outs

    def free(self):
        """free-runtime (runtime.lisp:76-81)"""
        # views and copies are closed like the rest but own nothing: every block goes back exactly once
        for v in self.variables.values():
            if isinstance(v, AbstractBuffer):
                close_buffer(self, v)
        for b in self._casts:
            close_buffer(self, b)
        self._casts.clear()
        for n in self.graph:
            pool = n.attrs.get("pool")
            if isinstance(pool, AbstractBuffer):
                close_buffer(self, pool)
                n.attrs["pool"] = None

    # ---- realize-node ----
    def realize_node(self, node: Node, args):
        fn = self._methods.get(node.type)
        if fn is None:
            fn = getattr(self, "realize_" + node.type.lower().replace("/", "_").replace("-", "_"), None)
            if fn is None:
                raise NotImplementedError(f"realize-node: no method for node type :{node.type} on {type(self).__name__}")
            self._methods[node.type] = fn
        return fn(node, args)

    def _num(self, x):
        return x.value if isinstance(x, AbstractBuffer) else x

    def realize_allocate(self, node: Node, args):
        """realize-node :Allocate incl. the :from case and pool reuse (runtime.lisp:228-259).
        args = shape numbers then stride numbers (nrank each)."""
        frm = node.attrs.get("from")
        if frm is not None:
            val = self.getvar(frm) if not isinstance(frm, AbstractBuffer) else frm
            if not isinstance(val, AbstractBuffer):
                raise TypeError(f"The :from attribute in the {node.type} node should be a buffer or a symbol.")
            return self.adopt(val)
        nrank = node.attrs["nrank"]
        shape = [int(self._num(a)) for a in args[:nrank]]
        stride = [int(self._num(a)) for a in args[nrank:2 * nrank]]
        pool = node.attrs.get("pool")
        if isinstance(pool, AbstractBuffer) and shape:
            if shape == list(pool.shape):
                return pool
            close_buffer(self, pool)
        buf = make_buffer(shape, stride, node.attrs["dtype"], None, device=self.buffer_type)
        open_buffer(self, buf)
        node.attrs["pool"] = buf
        return buf

    def adopt(self, buf: AbstractBuffer) -> AbstractBuffer:
        return buf

    def realize_view(self, node: Node, args):
        """realize-node :View (runtime.lisp:261-284): args = buffer, shape, from, to, by, stride (nrank each)."""
        nrank = node.attrs["nrank"]
        base = args[0]
        rest = [self._num(a) for a in args[1:]]
        shape, v1, v2, v3, stride = (rest[i * nrank:(i + 1) * nrank] for i in range(5))
        bc = node.attrs.get("broadcast", [False] * nrank)
        buf = base.copy()
        initial = buf.value
        scalar_to_tensor = nrank > 0 and isinstance(initial, (bool, int, float, np.number)) and base.nrank == 0
        buf.shape, buf.stride = [int(s) for s in shape], [int(s) for s in stride]
        buf.views = [(int(a), int(b), int(c), bool(d)) for a, b, c, d in zip(v1, v2, v3, bc)]
        buf.nrank = nrank
        if scalar_to_tensor:
            # casting a scalar to an array: storage of its own, every element the scalar (runtime.lisp:274-283)
            open_buffer(self, buf)
            n = int(np.prod([1 if b else int(s) for b, s in zip(bc, shape)])) if nrank else 1
            transfer_from_array(self, buf, np.full(n, initial, DTYPES[buf.dtype]))
            self._casts.append(buf)
        return buf

    def realize_jit_kernel(self, node: Node, args):
        """realize-node :JIT_KERNEL (runner.lisp:23-32)"""
        info: CompiledKernel = node.attrs["kernel_info"]
        args = [coerce_dtyped_buffer(a, dt) for a, dt in zip(args, node.attrs["dtypes"])]
        t1 = time.perf_counter()
        self.invoke_jit_kernel(info, node, args)
        if self.profile:
            _lib.check(_lib.load().cthip_sync())  # PROFILE assumes synchronous kernels (runner.lisp:27)
            dt = time.perf_counter() - t1
            self.times["kernel"] += dt
            print(f"{self.pc} |  KERNEL  | {dt:.6f}s | {info.device}[{info.name}]")
        outs = tuple(args[i] for i in info.out_positions)
        return outs if len(outs) != 1 else outs[0]

    def invoke_jit_kernel(self, info: CompiledKernel, node: Node, args):
        """runtime-invoke-jit-kernel (runner.lisp:20-21; Metal passes the node too, metal.lisp:285-286)"""
        info.caller(node, *args)

    # scalar arithmetic of the VM (runtime.lisp:396-449): dynamic shapes and strides are computed by :Add / :Mul /
    # :Neg / :Idiv / :Mod / :Max / :Load nodes over rank-0 values; arrays go through JIT kernels on this backend
    def _scalar_op(self, node: Node, args, fn):
        vals = [self._num(a) for a in args]
        if any(isinstance(a, AbstractBuffer) and a.nrank > 0 for a in args):
            raise NotImplementedError(f"realize-node :{node.type} over arrays is not a VM operation on this backend "
                                      f"(it is part of a JIT kernel)")
        out = fn(*vals)
        first = args[0]
        if isinstance(first, AbstractBuffer):
            b = first.copy()
            b.value = out
            return b
        return out

    def realize_add(self, node: Node, args):
        return self._scalar_op(node, args, lambda *v: sum(v[1:], v[0]))

    def realize_mul(self, node: Node, args):
        def mul(*v):
            out = v[0]
            for x in v[1:]:
                out = out * x
            return out
        return self._scalar_op(node, args, mul)

    def realize_neg(self, node: Node, args):
        return self._scalar_op(node, args, lambda x: -x)

    def realize_idiv(self, node: Node, args):
        return self._scalar_op(node, args, lambda a, b: a // b)

    def realize_mod(self, node: Node, args):
        return self._scalar_op(node, args, lambda a, b: a % b)

    def realize_max(self, node: Node, args):
        return self._scalar_op(node, args, max)

    def realize_load(self, node: Node, args):
        """:Load (runtime.lisp:396-405) of a rank-0 target: the node's :value, a number or a variable name"""
        val = node.attrs["value"]
        val = self._num(self.getvar(val)) if isinstance(val, str) else val
        return self._scalar_op(node, args, lambda _t: val)

    def realize_pause_backward(self, node: Node, args):
        return tuple(args) if len(args) != 1 else args[0]


class HipRuntime(GraphRuntime):
    """GraphRuntime whose buffers live in HBM; opens the device on creation
    (cf. MetalRuntime's initialize-instance :after, source/byoc/metal.lisp:106-112)."""
    buffer_type = HipBuffer

    def __init__(self, graph=(), fw_outputs=(), variables=None, renderer=None, device: int = 0, native: bool = True):
        super().__init__(list(graph), fw_outputs, variables, renderer)
        self.lib = _lib.init(device)
        self._uploaded: Dict[int, HipBuffer] = {}
        # native: hand the node list to the library at the first forward and walk it there (NativeWalk); lists
        # with node kinds that walk does not know, and PROFILE=1 runs, are walked here
        self.native = native
        self._walk: Optional[NativeWalk] = None

    def forward(self, *params):
        if self.native and not self.profile and self._walk is None:
            try:
                self._walk = NativeWalk(self)
            except Exception:
                # a list the library does not walk -- or a malformed one, which the walk here reports at its node,
                # wrapped like the reference's runtime-error
                self.native = False
        if self._walk is not None:
            try:
                return self._walk.forward(params)
            except _lib.HipError as e:
                raise RuntimeError_(self, e) from e
        return super().forward(*params)

    def getvar(self, var):
        # after a forward walked by the library the variable table lives there
        if self._walk is not None and var in self._walk.slots:
            try:
                return self._walk._output(var)
            except KeyError:
                pass
        return super().getvar(var)

    def adopt(self, buf: AbstractBuffer) -> AbstractBuffer:
        """Weights loaded from GGUF are host buffers whatever the backend
        (external/gguf/tensor-info.lisp:104-120) and enter through `:Allocate :from`
        untouched (runtime.lisp:228-243): upload once and cache the device copy."""
        if isinstance(buf, HipBuffer) or buf.nrank == 0:
            return buf
        key = id(buf)
        if key not in self._uploaded:
            dev = make_buffer(buf.shape, buf.stride, buf.dtype, buf.views, device=HipBuffer)
            open_buffer(self, dev)
            transfer_from_array(self, dev, np.asarray(buf.value))
            self._uploaded[key] = dev
            # the device copy lives exactly as long as the host buffer it mirrors (an id may be
            # reused once that object is collected)
            weakref.finalize(buf, self._drop_upload, key)
        return self._uploaded[key]

    def _drop_upload(self, key):
        dev = self._uploaded.pop(key, None)
        if dev is not None:
            close_buffer(self, dev)

    def sync(self):
        _lib.check(self.lib.cthip_sync())

    def free(self):
        if self._walk is not None:
            self._walk.close()
            self._walk = None
        super().free()
        for b in self._uploaded.values():
            close_buffer(self, b)
        self._uploaded.clear()


class NativeWalk:
    """The node list of a HipRuntime handed to the library once, so that a forward is one call (cthip_vm_run) instead
    of one host step per node: the walk of runtime-forward (runtime.lisp:106-145) over `:Allocate`, the scalar nodes
    and `:JIT_KERNEL`.  Raises NotImplementedError for a list that holds anything else (views, custom ops, kernels
    with boxed rank-0 outputs); the runtime then keeps walking it here."""

    SCALAR_OPS = {"Add": 0, "Mul": 1, "Neg": 2, "Idiv": 3, "Mod": 4, "Max": 5}
    DTYPE_CODES = {"bool": 1, "float64": 2, "float32": 3, "uint64": 4, "int64": 5, "uint32": 6, "int32": 7,
                   "uint16": 8, "int16": 9, "uint8": 10, "int8": 11}

    def __init__(self, rt: "HipRuntime"):
        from .renderer import HipProgram
        self.rt, self.lib = rt, rt.lib
        self.slots: Dict[Any, int] = {}
        self.inputs: Dict[Any, int] = {}        # symbol bound by forward(...) -> slot of the `:Allocate :from` that reads it
        self.meta: Dict[int, tuple] = {}        # slot -> (dtype, shape operands) of the :Allocate that opened it
        for n in rt.graph:
            for name in list(n.writes) + [r for r in n.reads if isinstance(r, str)]:
                self.slots.setdefault(name, len(self.slots))
            frm = n.attrs.get("from") if n.type == "Allocate" else None
            if isinstance(frm, str):
                self.slots.setdefault(frm, len(self.slots))
        self.vm = C.c_void_p()
        _lib.check(self.lib.cthip_vm_create(C.byref(self.vm), max(1, len(self.slots))))
        self._holders: Dict[int, HipBuffer] = {}
        try:
            for n in rt.graph:
                self._add(n, HipProgram)
        except Exception:
            self.close()
            raise

    def _operands(self, reads):
        k = (C.c_int * len(reads))()
        iv = (C.c_longlong * len(reads))()
        fv = (C.c_double * len(reads))()
        for j, r in enumerate(reads):
            if isinstance(r, str):
                k[j], iv[j] = 2, self.slots[r]
            elif isinstance(r, (bool, int, np.integer)):
                k[j], iv[j] = 0, int(r)
            elif isinstance(r, (float, np.floating)):
                k[j], fv[j] = 1, float(r)
            else:
                raise NotImplementedError(f"native walk: operand {r!r}")
        return k, iv, fv

    def _add(self, n: Node, HipProgram):
        lib = self.lib
        if n.type == "Allocate":
            out = self.slots[n.writes[0]]
            frm = n.attrs.get("from")
            if frm is not None:
                if isinstance(frm, AbstractBuffer):  # a parameter: uploaded once, bound for good
                    dev = self.rt.adopt(frm)
                    if dev.nrank == 0:
                        raise NotImplementedError("native walk: a rank-0 parameter")
                    _lib.check(lib.cthip_vm_set_buffer(self.vm, out, dev.value))
                else:
                    self.inputs[frm] = out
                return
            nrank = n.attrs["nrank"]
            if nrank == 0:
                raise NotImplementedError("native walk: a rank-0 :Allocate")
            k, iv, _ = self._operands(n.reads[:nrank])
            _lib.check(lib.cthip_vm_add_allocate(self.vm, out, np.dtype(DTYPES[n.attrs["dtype"]]).itemsize, nrank, k, iv))
            self.meta[out] = (n.attrs["dtype"], list(n.reads[:nrank]))
        elif n.type in self.SCALAR_OPS:
            k, iv, fv = self._operands(n.reads)
            _lib.check(lib.cthip_vm_add_scalar(self.vm, self.SCALAR_OPS[n.type], self.slots[n.writes[0]], len(n.reads), k, iv, fv))
        elif n.type == "JIT_KERNEL":
            info: CompiledKernel = n.attrs["kernel_info"]
            prog = info.caller
            if not isinstance(prog, HipProgram):
                raise NotImplementedError("native walk: a kernel whose caller is not a HipProgram")
            codes = (C.c_int * len(n.reads))()
            for j, (g, r) in enumerate(zip(prog.defglobals, n.reads)):
                if g["pointer_p"]:
                    if not isinstance(r, str):
                        raise NotImplementedError("native walk: a number passed by pointer")
                    codes[j] = 0
                else:
                    codes[j] = self.DTYPE_CODES[g["dtype"]]
            if len(prog.defglobals) != len(n.reads):
                raise AssertionError(f"HIP: {prog.name} takes {len(prog.defglobals)} arguments, got {len(n.reads)}")
            k, iv, fv = self._operands(n.reads)
            pos = (C.c_int * len(info.out_positions))(*info.out_positions)
            outs = (C.c_int * len(n.writes))(*[self.slots[w] for w in n.writes])
            if len(info.out_positions) != len(n.writes):
                raise AssertionError("Runtime: the number of outputs does not match the number of writes.")
            _lib.check(lib.cthip_vm_add_kernel(self.vm, prog.program, len(n.reads), k, iv, fv, codes, len(n.writes), pos, outs))
            for w, p_ in zip(n.writes, info.out_positions):  # the written name is the same storage as the argument
                src = n.reads[p_]
                if isinstance(src, str) and self.slots[src] in self.meta:
                    self.meta[self.slots[w]] = self.meta[self.slots[src]]
        else:
            raise NotImplementedError(f"native walk: node type :{n.type}")

    def forward(self, params):
        lib, rt = self.lib, self.rt
        for name, v in params:
            rt.setvar(name, v)
            slot = self.inputs.get(name, self.slots.get(name))
            if slot is None:
                continue
            if isinstance(v, AbstractBuffer) and v.nrank > 0:
                _lib.check(lib.cthip_vm_set_buffer(self.vm, slot, rt.adopt(v).value))
                continue
            x = v.value if isinstance(v, AbstractBuffer) else v
            if isinstance(x, (bool, int, np.integer)):
                _lib.check(lib.cthip_vm_set_int(self.vm, slot, int(x)))
            else:
                _lib.check(lib.cthip_vm_set_float(self.vm, slot, float(x)))
        rc = lib.cthip_vm_run(self.vm)
        if rc != 0:
            _lib.check(rc)
        outs = tuple(self._output(o) for o in rt.fw_outputs)
        for name, b in zip(rt.fw_outputs, outs):
            rt.variables[name] = b
        return outs[0] if len(outs) == 1 else outs

    def _value(self, slot):
        kind, iv, fv, ptr = C.c_int(), C.c_longlong(), C.c_double(), C.c_void_p()
        _lib.check(self.lib.cthip_vm_get(self.vm, slot, C.byref(kind), C.byref(iv), C.byref(fv), C.byref(ptr)))
        return kind.value, iv.value, fv.value, ptr.value

    def _output(self, name):
        slot = self.slots[name]
        kind, iv, fv, ptr = self._value(slot)
        if kind == 1:
            return iv
        if kind == 2:
            return fv
        if kind != 3 or slot not in self.meta:
            raise KeyError(f"Runtime: the variable {name} is not defined in the graph.")
        dtype, shape_ops = self.meta[slot]
        shape = [int(self._value(self.slots[s])[1]) if isinstance(s, str) else int(s) for s in shape_ops]
        stride, acc = [], 1
        for s in reversed(shape):
            stride.append(acc)
            acc *= s
        # the storage belongs to the walk's pool: the holder is never closed here, the result is a copy of it
        holder = self._holders.get(slot)
        if holder is None or holder.value != ptr or holder.shape != shape:
            holder = make_buffer(shape, list(reversed(stride)), dtype, None, value=ptr, device=HipBuffer)
            self._holders[slot] = holder
        return holder.copy()

    @property
    def launches(self) -> int:
        return int(self.lib.cthip_vm_launches(self.vm))

    def close(self):
        if self.vm:
            self.lib.cthip_vm_destroy(self.vm)
            self.vm = C.c_void_p()
        for h in self._holders.values():
            h._value = None
        self._holders.clear()


class HipAutoScheduler:
    """define-auto-scheduler (Hip-Auto-Scheduler ()) :n-global-loop 3 (cf. metal.lisp:153).
    Work distribution is chosen by the renderer per kernel pattern, not by ISL marks."""
    n_global_loop = 3
    tile_sizes = (2, 4, 8, 16, 32)


def _register():
    from .renderer import HipRenderer
    define_backend("HIP", HipBuffer, HipRuntime, HipRenderer, HipAutoScheduler, True)


_register()
