"""Writes tests/golden/blueprints/gpt2_*.sexp (and rope_32x64.sexp, swiglu_5632.sexp): the interchange text of every Schedule-Item of one GPT-2-small `forward`
(caten_amd.blueprints.gpt2_step_items), exactly what the Python mirror's printer hands cthip_program_create.  The
fixtures pin that text: tests/test_host.py fails when the printer, the blueprints or the library's reading of them drift.
Run from the repository root:  python tests/golden/make_blueprints.py"""
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from caten_amd import blueprints, synth  # noqa: E402
from caten_amd.renderer import item_sexp  # noqa: E402

if __name__ == "__main__":
    out = os.path.join(ROOT, "tests", "golden", "blueprints")
    os.makedirs(out, exist_ok=True)
    for key, item in blueprints.gpt2_step_items(synth.GPT2_CONFIGS["gpt2"]).items():
        with open(os.path.join(out, f"gpt2_{key}.sexp"), "w") as f:
            f.write(item_sexp(item))
        print("wrote", key)
    # the element-wise items of RoPE / SwiGLU blocks (Llama-1.1B shape: 32 heads of 64, FFN 5632)
    for fname, item in (("rope_32x64", blueprints.rope_rows(32, 64)), ("swiglu_5632", blueprints.swiglu_rows(5632))):
        with open(os.path.join(out, fname + ".sexp"), "w") as f:
            f.write(item_sexp(item))
        print("wrote", fname)
