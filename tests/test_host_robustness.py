"""Text and files from outside must never take the host process down: the blueprint reader (s-expressions a Lisp host
prints), the GGUF reader and the BPE tokenizer are driven with seeded mutations of valid inputs through the C ABI, in
a child process, and the child has to end normally -- refusing an input is fine, crashing on it is not.  No device.

Found this way and fixed: a double past the float range among an item's constants (the shortest-decimal printer read
past its buffer), lists nested a hundred thousand deep (every pass recurses over the tree: the reader now bounds the
depth), a loop whose step is zero (accepted and rendered into a kernel that would never end)."""
import ctypes
import glob
import os
import random
import struct
import subprocess
import sys
import tempfile

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _mutate(rng, b: bytes) -> bytes:
    b = bytearray(b)
    for _ in range(rng.randint(1, 4)):
        if not b:
            break
        k, i = rng.randint(0, 7), rng.randrange(len(b))
        if k == 0:
            del b[i:]
        elif k == 1:
            b[i] = rng.randrange(256)
        elif k == 2:
            del b[i:i + rng.randint(1, 8)]
        elif k == 3:
            b[i:i] = rng.choice([b"(", b")", b" ", b"-1", b"99999999999999999999", b"nil", b":", b"\"", b"1e999", b"1.5d300",
                                 b"(for", b"(aref x", b" 0 ", b"-0.0"])
        elif k == 4:
            j = rng.randrange(len(b))
            b[i:i] = b[j:j + rng.randint(1, 40)]
        elif k == 5:
            b[i] = ord(rng.choice("()"))
        elif k == 6:
            j = min(len(b), i + rng.randint(1, 30))
            b[i:j] = b[i:j][::-1]
        else:
            b[i:i] = bytes(rng.randrange(256) for _ in range(rng.randint(1, 6)))
    return bytes(b)


def _child_blueprints(seed: int, n: int) -> None:
    from caten_amd import _lib
    lib = _lib.load()
    rng = random.Random(seed)
    texts = [open(f, "rb").read() for f in sorted(glob.glob(os.path.join(ROOT, "tests", "golden", "blueprints", "*.sexp")))]
    deep = [b"(" * 200000,
            b"(item k (expr ((aref y 0)) " + b"(add 1 " * 100000 + b"1" + b")" * 100000 + b" :dtype float32))",
            b"(item k (expr ((aref y 0)) (add 1.0 0.69314718055994d53) :dtype float32))",
            b"(item k (define-global y float32 t output 1) (for i 0 (< i 4) 0 local) (expr ((aref y i)) 1.0 :dtype float32) (endfor i))",
            b"(item " + b"k" * 1000000 + b")", b"", b"()", b"(item)", b"(item k (expr (y) 1 :dtype))", b"(item k (expr ((aref)) (aref) :dtype float32))"]
    accepted = 0
    for it in range(n + len(deep)):
        t = deep[it - n] if it >= n else _mutate(rng, rng.choice(texts)).replace(b"\0", b" ")
        p = ctypes.c_void_p()
        if lib.cthip_program_create(ctypes.byref(p), t) == 0:
            accepted += 1
            lib.cthip_program_route(p)
            lib.cthip_program_source(p)
            lib.cthip_program_destroy(p)
        else:
            assert lib.cthip_last_error()
    # the four texts that must be refused: too deep (twice), a loop that does not advance, nothing at all
    for t in (deep[0], deep[1], deep[3], deep[5]):
        p = ctypes.c_void_p()
        assert lib.cthip_program_create(ctypes.byref(p), t) != 0
    print(f"blueprints: {accepted} of {n + len(deep)} accepted", flush=True)


def _child_gguf(seed: int, n: int) -> None:
    import numpy as np
    from caten_amd import gguf
    rng = random.Random(seed)
    path = os.path.join(tempfile.mkdtemp(), "a.gguf")
    a = np.arange(4 * 32, dtype=np.float32).reshape(4, 32)
    gguf.write_gguf(path, {"general.name": "x", "n": 3, "f": 1.5, "toks": ["a", "bc"], "flag": True},
                    [("a", "f32", a.shape, a), ("b", "f32", (32,), a[0])])
    blob = open(path, "rb").read()
    head = len(blob) - a.nbytes - a[0].nbytes - 64  # header, metadata and tensor infos: where a flipped count hurts
    accepted = 0
    for it in range(n):
        b = bytearray(blob)
        for _ in range(rng.randint(1, 3)):
            if len(b) < 9:
                break
            k, i = rng.randint(0, 3), rng.randrange(min(max(head, 8), len(b) - 8))
            if k == 0:
                b[i] = rng.randrange(256)
            elif k == 1:
                b[i:i + 8] = struct.pack("<Q", rng.choice([0, 1, 2**31, 2**32 - 1, 2**62, 2**63, 2**64 - 1, rng.randrange(2**64)]))
            elif k == 2:
                del b[rng.randrange(len(b)):]
            else:
                b[i:i + 4] = struct.pack("<I", rng.choice([0, 1, 12, 13, 255, 2**31, 2**32 - 1]))
        open(path, "wb").write(bytes(b))
        try:
            g = gguf.GGUF(path)
        except Exception:
            continue
        accepted += 1
        for t in g.tensor_info:
            try:
                g.tensor_bytes(t.name)
            except Exception:
                pass
        try:
            dict(g.metadata)
        except Exception:
            pass
        g.close()
    print(f"gguf: {accepted} of {n} accepted", flush=True)


def _child_bpe(seed: int, n: int) -> None:
    from caten_amd import _lib, tokenizer
    rng = random.Random(seed)
    d = os.path.join(ROOT, "tests", "golden", "gpt2_tokenizer")
    tokens = open(os.path.join(d, "tokens.txt"), encoding="utf-8").read()
    merges = open(os.path.join(d, "merges.txt"), encoding="utf-8").read()
    tk = tokenizer.make_bpe_tokenizer(tokens, merges)
    alphabet = [chr(c) for c in list(range(32, 127)) + [10, 9, 0xe9, 0x4e2d, 0x1f600, 0x300, 0xa0, 0x2028, 0xfffd, 0x10ffff, 0xd7ff]]
    for it in range(n):
        s = "".join(rng.choice(alphabet) for _ in range(rng.randint(0, 80)))
        assert tk.decode(tk.encode(s)) == s  # byte-level BPE gives every string back
        if it % 5 == 0:
            try:
                tk.decode([rng.randrange(-5, 60000) for _ in range(5)])
            except Exception:
                pass
    lib = _lib.load()
    tb, mb = tokens.encode(), merges.encode()
    for it in range(12):  # vocabularies and merge tables with damage in them
        t2 = _mutate(rng, tb[:200000]) if it % 2 else tb
        m2 = _mutate(rng, mb[:100000])
        h = ctypes.c_void_p()
        if lib.cthip_bpe_create(ctypes.byref(h), t2, len(t2), m2, len(m2)) == 0:
            ids, nn = (ctypes.c_int * 256)(), ctypes.c_size_t()
            txt = "hello wörld 中 123".encode()
            lib.cthip_bpe_encode(h, txt, len(txt), ids, 256, ctypes.byref(nn))
            lib.cthip_bpe_destroy(h)
    print("bpe: ok", flush=True)


def _run_child(what: str, seed: int, n: int) -> str:
    env = dict(os.environ, PYTHONPATH=ROOT + os.pathsep + os.environ.get("PYTHONPATH", ""))
    r = subprocess.run([sys.executable, os.path.abspath(__file__), what, str(seed), str(n)], capture_output=True, text=True,
                       timeout=600, env=env)
    assert r.returncode == 0, f"{what} seed {seed}: the child ended with {r.returncode}\n{r.stdout[-2000:]}\n{r.stderr[-2000:]}"
    return r.stdout


def test_blueprint_reader_survives_mutated_items():
    for seed in (1, 3):  # (seed 3 is the one that first met the out-of-range double)
        assert "blueprints:" in _run_child("blueprints", seed, 4000)


def test_gguf_reader_survives_mutated_files():
    assert "gguf:" in _run_child("gguf", 1, 4000)


def test_bpe_tokenizer_survives_any_text_and_damaged_tables():
    assert "bpe: ok" in _run_child("bpe", 1, 1500)


if __name__ == "__main__":
    {"blueprints": _child_blueprints, "gguf": _child_gguf, "bpe": _child_bpe}[sys.argv[1]](int(sys.argv[2]), int(sys.argv[3]))
