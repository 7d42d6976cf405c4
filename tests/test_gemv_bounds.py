"""Every single-row Linear launch the library can plan, walked lane by lane on the CPU: no access outside its
operand, no null operand dereferenced, the looping kernels only ever launched with the 256 threads they are compiled
for (tests/host/gemv_bounds.cpp; the plan is the library's own, caten_amd/csrc/gemv_plan.h)."""
import os
import subprocess
import tempfile

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_gemv_launch_plans_stay_inside_their_operands():
    exe = os.path.join(tempfile.mkdtemp(), "gemv_bounds")
    subprocess.check_call(["g++", "-O2", "-std=c++17", "-o", exe, os.path.join(ROOT, "tests", "host", "gemv_bounds.cpp")])
    r = subprocess.run([exe], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-4000:]
    last = r.stdout.strip().splitlines()[-1]
    assert last.endswith(" 0 violations") and "launches" in last
    assert int(last.split()[2]) > 10000  # launches walked


def test_column_slices_of_wide_rows_stay_inside_their_operands():
    """rows wider than any register-resident variant (the FFN down-projections of the 7B, 13B and 70B Llama shapes,
    a wide fp32 / fp16 row, a Q8_0 row one block past the widest variant) go as column slices with a row pitch and
    pointer offsets: the same walk over what launch_gemv queues for them"""
    exe = os.path.join(tempfile.mkdtemp(), "gemv_bounds")
    subprocess.check_call(["g++", "-O2", "-std=c++17", "-o", exe, os.path.join(ROOT, "tests", "host", "gemv_bounds.cpp")])
    shapes = "2 4096 11008 8 1000 11008 2 640 13824 2 515 28672 0 300 12288 1 300 6400 8 300 8224"
    r = subprocess.run([exe, "shape"] + shapes.split(), capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-4000:]
    last = r.stdout.strip().splitlines()[-1]
    assert last.endswith(" 0 violations") and int(last.split()[2]) >= 7 * 2 * 4 * 2 * 2
