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
