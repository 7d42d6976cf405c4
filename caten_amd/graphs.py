"""The node list of one compiled GPT-2 `forward`, as the VM of the `:HIP` backend walks it.

In a Lisp process this list is what `caten` + `jit` leave in the GraphRuntime (source/codegen/jit.lisp:513-530): `:Allocate`
nodes for every intermediate (dynamic shapes computed by scalar nodes of the VM, source/runtime/runtime.lisp:396-449),
parameters entering through `:Allocate :from`, and one `:JIT_KERNEL` per Schedule-Item, launched one after another by
`runtime-forward` (source/runtime/runtime.lisp:106-145) each time `gpt2-generate` asks for a token
(apps/gpt2/gpt2.lisp:97-113).  No Lisp implementation exists where this package is tested, so the list is assembled
here from the Transformer definition (external/llm/layers.lisp:8-90) with the blueprints of `blueprints.gpt2_step_items`;
everything below the list -- renderer, router, kernels, buffers -- is what a Caten process would drive as well.

The KV cache is an ordinary `:Allocate` of `(1, max_len, heads, head_dim)` (`linspace ... 0 0`, layers.lisp:25-26): its
shape never changes, so the pool hands the same zero-initialised storage back on every call and the rows written by
`!assign` persist from one `forward` to the next, which is how the reference keeps its cache.
"""
from __future__ import annotations

from typing import Dict, List

import numpy as np

from . import _lib, blueprints
from .buffer import make_buffer
from .renderer import HipRenderer
from .runtime import CompiledKernel, HipRuntime, Node


def _row_major(shape):
    st, acc = [], 1
    for s in reversed(shape):
        st.append(acc)
        acc *= int(s)
    return list(reversed(st))


class GPT2Graph:
    """make-gpt2's compiled model (apps/gpt2/gpt2.lisp:82-95) behind `forward(x, s, n)`."""

    def __init__(self, cfg: dict, weights: dict, device: int = 0, native: bool = True):
        self.cfg = dict(cfg)
        D, H, F, V, L, NL = cfg["dim"], cfg["n_heads"], cfg["ffn"], cfg["vocab"], cfg["max_seq"], cfg["n_layers"]
        Dh = D // H
        _lib.init(device)  # the callers are bound to the loaded module when the kernels are compiled
        self.items = blueprints.gpt2_step_items(cfg)
        self.renderer = HipRenderer()
        for it in self.items.values():
            self.renderer.render_kernel(it)
        self.renderer.compile_kernel(list(self.items.values()))
        g: List[Node] = []
        params: Dict[str, object] = {}

        def param(name, arr):
            a = np.ascontiguousarray(arr, np.float32)
            params[name] = make_buffer(list(a.shape), _row_major(list(a.shape)), "float32", value=a.ravel())
            g.append(Node("Allocate", [name], [], {"nrank": a.ndim, "dtype": "float32", "from": params[name]}))
            return name

        def scalar(out, op, a, b):
            g.append(Node(op, [out], [a, b], {}))
            return out

        def alloc(name, shape, dtype="float32"):
            # shape entries: numbers or names of scalars in the variable table; row-major strides by scalar nodes
            strides = [1] * len(shape)
            for i in range(len(shape) - 2, -1, -1):
                nxt, ext = strides[i + 1], shape[i + 1]
                if isinstance(nxt, int) and isinstance(ext, int):
                    strides[i] = nxt * ext
                elif nxt == 1:
                    strides[i] = ext
                else:
                    strides[i] = scalar(f"{name}_st{i}", "Mul", nxt, ext)
            g.append(Node("Allocate", [name], list(shape) + strides, {"nrank": len(shape), "dtype": dtype}))
            return name

        def kernel(item_key, writes, reads):
            it = self.items[item_key]
            dts = [n["dtype"] for n in it["blueprint"] if n["type"] == "DEFINE-GLOBAL"]
            nout = sum(1 for n in it["blueprint"] if n["type"] == "DEFINE-GLOBAL" and n["arg_type"] == "output")
            info = CompiledKernel(it["name"], it["compiled_object"], out_positions=tuple(range(nout)))
            g.append(Node("JIT_KERNEL", list(writes), list(reads), {"kernel_info": info, "dtypes": dts}))

        g.append(Node("Allocate", ["tok"], [], {"nrank": 2, "dtype": "float32", "from": "x"}))
        scalar("t", "Add", "n", "s")  # cached + new positions
        wte, wpe = param("wte", weights["wte"]), param("wpe", weights["wpe"])
        kernel("embed_tokens", ["emb"], [alloc("emb", ["s", D]), "s", "tok", wte])
        kernel("embed_positions", ["h0"], [alloc("h0", ["s", D]), "s", "n", "emb", wpe])
        kernel("mask", ["mask"], [alloc("mask", ["s", "t"]), "s", "n"])
        hi = "h0"
        for l in range(NL):
            p = lambda k: param(f"l{l}_{k}", weights[k][l])  # noqa: E731
            a = lambda nm, shape: alloc(f"l{l}_{nm}", shape)  # noqa: E731
            kernel("layernorm", [f"l{l}_ln1"], [a("ln1", ["s", D]), "s", hi, p("ln1_g"), p("ln1_b")])
            kernel("c_attn", [f"l{l}_qkv"], [a("qkv", ["s", 3 * D]), "s", f"l{l}_ln1", p("attn_w"), p("attn_b")])
            kc, vc = a("kc", [L, H, Dh]), a("vc", [L, H, Dh])
            kernel("assign_k", [kc], [kc, "s", "n", f"l{l}_qkv"])
            kernel("assign_v", [vc], [vc, "s", "n", f"l{l}_qkv"])
            kernel("scores", [f"l{l}_sc"], [a("sc", [H, "s", "t"]), "s", "n", f"l{l}_qkv", kc, "mask"])
            kernel("softmax", [f"l{l}_pr"], [a("pr", [H, "s", "t"]), "s", "n", f"l{l}_sc"])
            kernel("values", [f"l{l}_ao"], [a("ao", [H, "s", Dh]), "s", "n", f"l{l}_pr", vc])
            kernel("merge_heads", [f"l{l}_am"], [a("am", ["s", D]), "s", f"l{l}_ao"])
            kernel("attn_proj", [f"l{l}_h1"], [a("h1", ["s", D]), "s", f"l{l}_am", p("proj_w"), p("proj_b"), hi])
            kernel("layernorm", [f"l{l}_ln2"], [a("ln2", ["s", D]), "s", f"l{l}_h1", p("ln2_g"), p("ln2_b")])
            kernel("c_fc", [f"l{l}_fc"], [a("fc", ["s", F]), "s", f"l{l}_ln2", p("fc_w"), p("fc_b")])
            kernel("mlp_proj", [f"l{l}_h2"], [a("h2", ["s", D]), "s", f"l{l}_fc", p("fc2_w"), p("fc2_b"), f"l{l}_h1"])
            hi = f"l{l}_h2"
        kernel("layernorm", ["lnf"], [alloc("lnf", ["s", D]), "s", hi, param("lnf_g", weights["lnf_g"]), param("lnf_b", weights["lnf_b"])])
        kernel("lm_head", ["logits"], [alloc("logits", ["s", V]), "s", "lnf", param("lm_head", weights["lm_head"])])
        kernel("argmax", ["out"], [alloc("out", [1, 1], "int64"), "s", "logits"])
        self.params = params
        self.vm = HipRuntime(g, fw_outputs=["out"], renderer=self.renderer, device=device, native=native)
        self.n_kernels = sum(1 for n in g if n.type == "JIT_KERNEL")

    def forward(self, tokens, n: int):
        """(forward model `(x . tokens) `(s . len) `(n . start-pos)) (gpt2.lisp:104): the (1, 1) int64 buffer."""
        x = np.asarray(tokens, np.float32).ravel()  # ->input makes floats of the ids (gpt2.lisp:95)
        hx = make_buffer([1, x.size], [x.size, 1], "float32", value=x)
        return self.vm.forward(("x", hx), ("s", int(x.size)), ("n", int(n)))

    def routes(self) -> Dict[str, str]:
        """what each item's last launch ran: a hand-written kernel's entry point, or "rendered" """
        return {k: it["compiled_object"].last_route for k, it in self.items.items()}

    def generate(self, prompt, max_length: int) -> list:
        """gpt2-generate's loop (gpt2.lisp:97-113): the first forward takes the whole prompt, each token comes back to
        the host (8-byte D2H) and goes in again."""
        from .buffer import transfer_into_array
        tokens = [int(t) for t in prompt]
        start, out = 0, []
        for _ in range(max_length):
            o = self.forward(tokens[start:], start)
            tok = int(np.asarray(transfer_into_array(o)).ravel()[0])
            start = len(tokens)
            tokens.append(tok)
            out.append(tok)
        return out

    def close(self):
        self.vm.free()
