"""The single-workgroup dispatch kernel (csrc/dispatch.hip::dispatch_small_kernel) run on the CPU in
lock step: its source text is spliced into a small C++ harness (tests/emulation/) that gives every
lane an OS thread and implements the wave intrinsics with barriers, with bounds checks on every
global array.  Checks the results against a stable sort, and catches what a GPU run would turn into
a memory fault: an index out of bounds (abort) or a shuffle/ballot that only some lanes of a wave
reach (deadlock, caught by the time limit)."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_small_dispatch_kernel_in_lock_step_on_the_cpu(tmp_path):
    src = open(os.path.join(ROOT, "train-large-model-from-scratch_amd", "csrc", "dispatch.hip")).read()
    a = src.index("__global__ __launch_bounds__(SMALL_WAVES* MOE_WAVE) void dispatch_small_kernel(")
    b = src.index("// ---- row movers", a)
    kern = src[a:b]
    kern = kern.replace("__global__ __launch_bounds__(SMALL_WAVES* MOE_WAVE) void", "void")
    kern = kern.replace("extern __shared__ int sm[];", "int* sm = g_lds;")
    kern = kern.replace("const int32_t* __restrict__ ids", "Checked<const int32_t> ids")
    for name in ("counts", "offs", "pos_to_row", "row_to_pos"):
        kern = kern.replace("int32_t* __restrict__ " + name, "Checked<int32_t> " + name)
    kern = kern.replace("int32_t* __restrict__ bad_total", "int32_t* bad_total")
    kern = re.sub(r"#pragma unroll\n", "", kern)
    harness = open(os.path.join(ROOT, "tests", "emulation", "dispatch_small_emu.cpp")).read()
    assert "// KERNEL_SOURCE" in harness
    cpp = tmp_path / "emu.cpp"
    cpp.write_text(harness.replace("// KERNEL_SOURCE", kern))
    exe = tmp_path / "emu"
    subprocess.run(["g++", "-std=c++20", "-O1", "-pthread", str(cpp), "-o", str(exe)], check=True)
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=240)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.count(" ok") == 6 and "MISMATCH" not in r.stdout, r.stdout
