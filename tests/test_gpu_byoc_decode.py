"""One GPT-2 `forward` after another through the plug-in path: the node list of the compiled graph (Allocate / scalar
nodes / one JIT_KERNEL per Schedule-Item) walked by the VM, every item created from its blueprint text by
cthip_program_create and launched through cthip_program_launch -- what `BACKEND=HIP` gives a Caten user who calls
gpt2-generate (apps/gpt2/gpt2.lisp:97-113).  Tokens must be the CPU oracle's, and every Linear and attention item must
have run a hand-written kernel."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

HAND_WRITTEN = {"embed_tokens": "cthip_embedding", "embed_positions": "cthip_embedding", "layernorm": "cthip_layernorm",
                "c_attn": "cthip_linear", "scores": "cthip_bmm", "softmax": "cthip_softmax", "values": "cthip_bmm",
                "attn_proj": "cthip_linear", "c_fc": "cthip_linear", "mlp_proj": "cthip_linear", "lm_head": "cthip_linear",
                "argmax": "cthip_argmax"}
RENDERED = ("mask", "assign_k", "assign_v", "merge_heads")  # element-wise generators and copies


def _run(oracle, name, prompt_len, steps, seed=0, native=True):
    from caten_amd import synth, graphs
    cfg = synth.GPT2_CONFIGS[name]
    w = synth.gpt2_weights(cfg, seed=seed)
    prompt = synth.prompt(cfg["vocab"], prompt_len, seed=seed)
    model = graphs.GPT2Graph(cfg, w, native=native)
    from caten_amd.buffer import transfer_into_array
    try:
        got = model.generate(prompt, steps)
        # native: the node list is walked by the library, one call per forward; else node by node on the host
        assert (model.vm._walk is not None) == native
        if native:
            assert model.vm._walk.launches == steps * model.n_kernels
        routes = model.routes()
        n_kernels = model.n_kernels
        logits = np.asarray(transfer_into_array(model.vm.getvar("logits"))).reshape(-1, cfg["vocab"])[-1]
    finally:
        model.close()
    want, logs = oracle.GPT2(cfg, w).generate(prompt, steps, keep_logits=True)
    # the last forward's logits inside the north star's band (fp32: rtol 1e-3 / atol 1e-4)
    assert np.allclose(logits, logs[-1], rtol=1e-3, atol=1e-4), float(np.max(np.abs(logits - logs[-1])))
    return got, want, routes, n_kernels, cfg


@pytest.mark.parametrize("native", [True, False])
def test_gpt2_tiny_forward_through_the_vm_matches_oracle(oracle, native):
    got, want, routes, n_kernels, cfg = _run(oracle, "gpt2-tiny", 8, 12, native=native)
    assert got == want, f"plug-in path {got} vs oracle {want}"
    assert n_kernels == 6 + 12 * cfg["n_layers"]  # embeddings, mask, ln_f, lm_head, argmax + 12 items per block
    for k, entry in HAND_WRITTEN.items():
        assert routes[k] == entry, (k, routes[k])
    for k in RENDERED:
        assert routes[k] == "rendered", (k, routes[k])


@pytest.mark.parametrize("native", [True, False])
def test_gpt2_tiny_single_token_prompt_and_ragged_lengths(oracle, native):
    # s = 1 from the first call on (every Linear a single-row launch), then a 5-token prompt (fewer than 8 rows)
    for plen in (1, 5):
        got, want, routes, _, _ = _run(oracle, "gpt2-tiny", plen, 9, seed=plen, native=native)
        assert got == want, (plen, got, want)


def test_gpt2_small_forward_through_the_vm_matches_oracle(oracle):
    """GPT-2-small shape, fp32 weights (what gguf->state-dict hands a Caten graph whatever the file's type): a 16-token
    prompt (the Linears take the MFMA path, the attention items the batched kernel with 16 rows) and 8 decode steps."""
    got, want, routes, n_kernels, cfg = _run(oracle, "gpt2", 16, 9)
    assert got == want, f"plug-in path {got} vs oracle {want}"
    assert n_kernels == 6 + 12 * 12
    for k, entry in HAND_WRITTEN.items():
        assert routes[k] == entry, (k, routes[k])


def test_items_run_rendered_when_routes_are_off_and_agree(oracle):
    """option render_routes 0: the same graph on rendered kernels only -- the router changes which kernel runs, not
    what the item computes."""
    import caten_amd as ca
    lib = ca._lib.init()
    ca._lib.check(lib.cthip_set_option(b"render_routes", 0))
    try:
        got, want, routes, _, _ = _run(oracle, "gpt2-tiny", 4, 6, seed=3)
    finally:
        ca._lib.check(lib.cthip_set_option(b"render_routes", 1))
    assert got == want
    assert set(routes.values()) == {"rendered"}


def _run_items(items):
    """render + compile + bind a list of item dicts; returns their callers"""
    import caten_amd as ca
    ca._lib.init()
    r = ca.HipRenderer()
    for it in items:
        r.render_kernel(it)
    r.compile_kernel(items)
    return [it["compiled_object"] for it in items]


def _dev(a, dtype="float32"):
    from caten_amd.buffer import make_buffer, HipBuffer, open_buffer, transfer_from_array
    a = np.ascontiguousarray(a)
    st, acc = [], 1
    for s in reversed(a.shape):
        st.append(acc)
        acc *= s
    b = make_buffer(list(a.shape), list(reversed(st)), dtype, device=HipBuffer)
    open_buffer(None, b)
    transfer_from_array(None, b, a.ravel())
    return b


def _host(b, shape):
    from caten_amd.buffer import transfer_into_array
    return np.asarray(transfer_into_array(b)).reshape(shape)


@pytest.mark.parametrize("H,Dh", [(4, 64), (3, 32), (2, 6)])
def test_attention_items_over_the_cache_view(H, Dh):
    """scores = q . k^T * scale + mask, softmax, out = probs . v as three items (external/llm/layers.lisp:3-5), q out of
    the fused qkv rows and k / v in place out of the (max_len, heads, head_dim) cache, for one row and for prompts, at
    several start positions; against NumPy in double.  head_dim 6 fits neither layout of the batched kernel (not a
    multiple of four): those launches run the rendered kernels, with the same result."""
    from caten_amd import blueprints as bp
    from caten_amd.buffer import close_buffer
    D, L = H * Dh, 64
    items = [bp.gpt2_causal_mask(), bp.gpt2_attention_scores(H, Dh), bp.gpt2_softmax_rows(H), bp.gpt2_attention_values(H, Dh),
             bp.gpt2_merge_heads(H, Dh)]
    mask_k, sc_k, sm_k, pv_k, mh_k = _run_items(items)
    rng = np.random.default_rng(H * 100 + Dh)
    for s, n in ((1, 0), (1, 37), (3, 5), (16, 0), (16, 40), (7, 1)):
        t = n + s
        qkv = rng.standard_normal((s, 3 * D)).astype(np.float32)
        kc = np.zeros((L, H, Dh), np.float32)
        vc = np.zeros((L, H, Dh), np.float32)
        kc[:t] = rng.standard_normal((t, H, Dh)).astype(np.float32)
        vc[:t] = rng.standard_normal((t, H, Dh)).astype(np.float32)
        d_qkv, d_k, d_v = _dev(qkv), _dev(kc), _dev(vc)
        d_mask, d_sc, d_pr = _dev(np.zeros((s, t), np.float32)), _dev(np.zeros((H, s, t), np.float32)), _dev(np.zeros((H, s, t), np.float32))
        d_o, d_m = _dev(np.zeros((H, s, Dh), np.float32)), _dev(np.zeros((s, D), np.float32))
        mask_k(None, d_mask, s, n)
        sc_k(None, d_sc, s, n, d_qkv, d_k, d_mask)
        sm_k(None, d_pr, s, n, d_sc)
        pv_k(None, d_o, s, n, d_pr, d_v)
        mh_k(None, d_m, s, d_o)
        q = qkv[:, :D].reshape(s, H, Dh).astype(np.float64)
        mask = np.where(np.arange(t)[None, :] - np.arange(s)[:, None] >= 1 + n, -np.inf, 0.0)
        assert np.array_equal(_host(d_mask, (s, t)), mask.astype(np.float32))
        sc = np.einsum("shd,thd->hst", q, kc[:t].astype(np.float64)) / np.sqrt(Dh) + mask[None]
        got_sc = _host(d_sc, (H, s, t))
        fin = np.isfinite(sc)
        assert np.array_equal(np.isneginf(got_sc), ~fin)
        assert np.allclose(got_sc[fin], sc[fin], rtol=1e-5, atol=1e-5)
        e = np.exp(sc - sc.max(-1, keepdims=True))
        pr = e / e.sum(-1, keepdims=True)
        assert np.allclose(_host(d_pr, (H, s, t)), pr, rtol=1e-5, atol=1e-6)
        o = np.einsum("hst,thd->shd", pr, vc[:t].astype(np.float64)).reshape(s, D)
        assert np.allclose(_host(d_m, (s, D)), o, rtol=1e-4, atol=1e-5)
        want_route = "cthip_bmm" if Dh % 4 == 0 else "rendered"
        assert sc_k.last_route == want_route and pv_k.last_route == want_route, (sc_k.last_route, pv_k.last_route)
        assert sm_k.last_route == "cthip_softmax"
        for b in (d_qkv, d_k, d_v, d_mask, d_sc, d_pr, d_o, d_m):
            close_buffer(None, b)


def test_the_references_rendered_chunk_matmul_runs_on_the_mfma_gemm():
    """the fixture with the index expressions of source/test-suite/test-scheduler.lisp:117-138, verbatim: the two
    halves of one (2, 64, 64) buffer multiplied; the second operand starts 4096 elements in"""
    import os
    from caten_amd.renderer import item_from_sexp
    from caten_amd.buffer import close_buffer
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    with open(os.path.join(root, "tests", "golden", "blueprints", "reference_chunk_matmul.sexp")) as f:
        item = item_from_sexp(f.read())
    (k,) = _run_items([item])
    rng = np.random.default_rng(5)
    x = rng.uniform(-1, 1, (2, 64, 64)).astype(np.float32)
    d_x, d_y = _dev(x), _dev(np.zeros((1, 64, 64), np.float32))
    k(None, d_y, d_x)
    want = x[0].astype(np.float64) @ x[1].astype(np.float64)
    assert np.allclose(_host(d_y, (64, 64)), want, rtol=1e-4, atol=1e-4)
    assert k.last_route == "cthip_matmul"
    close_buffer(None, d_x)
    close_buffer(None, d_y)


def test_linear_items_with_their_epilogues_vs_oracle(oracle):
    """c_fc + bias + GELU and c_proj + bias + residual as items (layers.lisp:53-71), one row, a few rows and a prompt's
    rows: the single-row kernels and the MFMA GEMM behind cthip_program_launch, against the oracle's Linear"""
    from caten_amd import blueprints as bp
    from caten_amd.buffer import close_buffer
    N, K = 384, 256
    fc, proj = bp.gpt2_linear(N, K, bias=True, gelu=True, name="fused_fc"), bp.gpt2_linear(N, K, bias=True, residual=True, name="fused_proj")
    k_fc, k_proj = _run_items([fc, proj])
    rng = np.random.default_rng(9)
    W = (0.05 * rng.standard_normal((N, K))).astype(np.float32)
    b = (0.05 * rng.standard_normal(N)).astype(np.float32)
    d_w, d_b = _dev(W), _dev(b)
    for s in (1, 3, 8, 33):
        x = rng.standard_normal((s, K)).astype(np.float32)
        r = rng.standard_normal((s, N)).astype(np.float32)
        d_x, d_r, d_y = _dev(x), _dev(r), _dev(np.zeros((s, N), np.float32))
        k_fc(None, d_y, s, d_x, d_w, d_b)
        want = oracle.gelu_tanh(oracle.linear(x, W, b))
        assert np.allclose(_host(d_y, (s, N)), want, rtol=1e-3, atol=1e-4)
        assert k_fc.last_route == "cthip_linear"
        k_proj(None, d_y, s, d_x, d_w, d_b, d_r)
        want = oracle.linear(x, W, b) + r
        assert np.allclose(_host(d_y, (s, N)), want, rtol=1e-3, atol=1e-4)
        assert k_proj.last_route == "cthip_linear"
        for q in (d_x, d_r, d_y):
            close_buffer(None, q)
    close_buffer(None, d_w)
    close_buffer(None, d_b)


def test_rope_and_swiglu_items_vs_oracle(oracle):
    """the element-wise items of RoPE / SwiGLU blocks as rendered kernels: `(!rope x dim)` at the reference's own bar
    (atol 1e-5 rtol 5e-4, source/test-suite/nn/test-rope.lisp:38-66) against the oracle (pinned by the torchtune
    formula), silu(gate) * up at 1e-6 (test-activations.lisp:153-162)"""
    from caten_amd import blueprints as bp
    from caten_amd.buffer import close_buffer
    H, Dh, F = 8, 64, 1536
    k_rope, k_glu = _run_items([bp.rope_rows(H, Dh), bp.swiglu_rows(F)])
    rng = np.random.default_rng(12)
    for s in (1, 10, 77):
        x = rng.standard_normal((1, s, H, Dh)).astype(np.float32)
        d_x, d_y = _dev(x), _dev(np.zeros_like(x))
        k_rope(None, d_y, s, d_x)
        assert np.allclose(_host(d_y, x.shape), oracle.rope(x, 10000.0, 0), rtol=5e-4, atol=1e-5)
        gate, up = rng.standard_normal((s, F)).astype(np.float32) * 3, rng.standard_normal((s, F)).astype(np.float32)
        d_g, d_u, d_o = _dev(gate), _dev(up), _dev(np.zeros_like(up))
        k_glu(None, d_o, s, d_g, d_u)
        assert np.allclose(_host(d_o, up.shape), oracle.silu(gate) * up, rtol=1e-6, atol=1e-6)
        assert k_rope.last_route == "rendered" and k_glu.last_route == "rendered"
        for b in (d_x, d_y, d_g, d_u, d_o):
            close_buffer(None, b)


def test_the_librarys_walk_of_scalar_nodes_equals_the_hosts():
    """:Add :Mul :Neg :Idiv :Mod :Max over numbers (runtime.lisp:396-449): the walk inside the library gives what the
    host's walk gives, also for negative operands of the integer division and for mixed integers and floats"""
    from caten_amd.runtime import HipRuntime, Node
    g = [Node("Add", ["a"], ["n", "s", 3]), Node("Mul", ["b"], ["a", "s", 2]), Node("Neg", ["c"], ["b"]),
         Node("Idiv", ["d"], ["c", 7]), Node("Mod", ["e"], ["c", 7]), Node("Max", ["f"], ["d", "e", -100]),
         Node("Mod", ["g"], ["a", -5]), Node("Idiv", ["h"], ["a", -5]), Node("Mul", ["i"], ["a", 0.5]),
         Node("Idiv", ["j"], ["i", 2]), Node("Mod", ["k"], ["c", 2.5])]
    outs = [n.writes[0] for n in g]
    for n, s in ((0, 1), (5, 3), (17, 16), (1023, 1)):
        res = []
        for native in (True, False):
            rt = HipRuntime(g, fw_outputs=outs, native=native)
            res.append(rt.forward(("n", n), ("s", s)))
            assert (rt._walk is not None) == native
            rt.free()
        assert res[0] == res[1], (n, s, res)
        assert all(type(a) is type(b) for a, b in zip(*res)), res


def test_a_list_with_other_node_kinds_stays_with_the_hosts_walk():
    """a :View is not one of the three node kinds the library walks: the runtime keeps the list and walks it itself"""
    from caten_amd.runtime import HipRuntime, Node
    from caten_amd.buffer import transfer_into_array
    g = [Node("Allocate", ["x"], [4, 6, 6, 1], {"nrank": 2, "dtype": "float32"}),
         Node("View", ["v"], ["x", 2, 6, 0, 0, 2, 6, 1, 1, 6, 1], {"nrank": 2, "broadcast": [False, False]})]
    rt = HipRuntime(g, fw_outputs=["v"])
    v = rt.forward()
    assert rt._walk is None and rt.native is False
    assert v.shape == [2, 6] and np.array_equal(transfer_into_array(v), np.zeros(12, np.float32))
    rt.free()


def test_pools_of_the_librarys_walk_keep_and_clear_storage_like_the_hosts():
    """a buffer whose shape is unchanged comes back with its contents (the KV cache lives on that); one whose shape
    changed is zero-filled again, whether its storage was kept or not (runtime.lisp:248-259)"""
    from caten_amd import blueprints, renderer
    from caten_amd.runtime import HipRuntime, Node, CompiledKernel
    from caten_amd.buffer import transfer_into_array
    # y[i] = y[i] + 1 over n elements: what is read is what the pool handed out
    item = {"name": "fused_increment", "blueprint": [
        {"type": "DEFINE-GLOBAL", "id": "y", "dtype": "float32", "pointer_p": True, "arg_type": "output", "nrank": 1},
        {"type": "DEFINE-GLOBAL", "id": "n", "dtype": "int64", "pointer_p": False, "arg_type": "shape", "nrank": 0},
        {"type": "FOR", "idx": "_gid0", "upfrom": 0, "below": {"op": "<", "args": ["_gid0", "n"]}, "by": 1, "scope": "local"},
        {"type": "EXPR", "writes": [{"op": "AREF", "id": "y", "index": "_gid0"}],
         "expr": {"op": "ADD", "args": [{"op": "AREF", "id": "y", "index": "_gid0"}, 1.0]}, "dtype": "float32"},
        {"type": "ENDFOR", "idx": "_gid0"}]}
    r = renderer.HipRenderer()
    r.render_kernel(item)
    r.compile_kernel([item])
    info = CompiledKernel(item["name"], item["compiled_object"], out_positions=(0,))
    for native in (True, False):
        g = [Node("Allocate", ["y"], ["n", 1], {"nrank": 1, "dtype": "float32"}),
             Node("JIT_KERNEL", ["y"], ["y", "n"], {"kernel_info": info, "dtypes": ["float32", "int64"]})]
        rt = HipRuntime(g, fw_outputs=["y"], renderer=r, native=native)
        seen = []
        for n in (8, 8, 8, 5, 12, 12, 300, 8):
            seen.append((n, np.asarray(transfer_into_array(rt.forward(("n", n)))).tolist()))
        rt.free()
        want, cur, last = [], 0, None
        for n in (8, 8, 8, 5, 12, 12, 300, 8):
            cur = cur + 1 if n == last else 1
            last = n
            want.append((n, [float(cur)] * n))
        assert seen == want, (native, seen)


def test_the_librarys_walk_reports_what_the_hosts_walk_reports():
    """a forward that leaves a shape variable unset stops at the node that needs it, wrapped as the reference's
    runtime-error (runtime.lisp:84-104) whichever side walks the list; the entry points refuse malformed nodes"""
    import ctypes as C
    from caten_amd import _lib
    from caten_amd.runtime import HipRuntime, Node, RuntimeError_
    g = [Node("Add", ["t"], ["n", "s"]), Node("Allocate", ["y"], ["t", 1], {"nrank": 1, "dtype": "float32"})]
    for native in (True, False):
        rt = HipRuntime(g, fw_outputs=["y"], native=native)
        with pytest.raises(RuntimeError_) as e:
            rt.forward(("n", 3))  # s is never bound
        assert "Runtime-Error" in str(e.value)
        if native:
            assert "vm: node 0" in str(e.value)
        y = rt.forward(("n", 3), ("s", 2))  # the runtime is usable afterwards
        assert y.shape == [5]
        rt.free()
    lib = _lib.init()
    vm = C.c_void_p()
    _lib.check(lib.cthip_vm_create(C.byref(vm), 4))
    kinds, iv, fv = (C.c_int * 2)(2, 0), (C.c_longlong * 2)(1, 7), (C.c_double * 2)()
    assert lib.cthip_vm_add_scalar(vm, 9, 0, 2, kinds, iv, fv) == _lib.E_BAD_ARG          # no such operation
    assert lib.cthip_vm_add_scalar(vm, 2, 0, 2, kinds, iv, fv) == _lib.E_BAD_ARG          # :Neg of two operands
    bad = (C.c_longlong * 2)(99, 7)
    assert lib.cthip_vm_add_scalar(vm, 0, 0, 2, kinds, bad, fv) == _lib.E_BAD_ARG         # a slot that does not exist
    assert lib.cthip_vm_add_allocate(vm, 1, 4, 9, kinds, iv) == _lib.E_BAD_ARG            # rank 9
    assert lib.cthip_vm_set_buffer(vm, 0, None) == _lib.E_BAD_ARG
    _lib.check(lib.cthip_vm_add_scalar(vm, 3, 0, 2, kinds, (C.c_longlong * 2)(1, 0), fv))  # slot 1 // 0
    _lib.check(lib.cthip_vm_set_int(vm, 1, 5))
    assert lib.cthip_vm_run(vm) == _lib.E_STATE and b"division by zero" in lib.cthip_last_error()
    _lib.check(lib.cthip_vm_destroy(vm))
