"""CPU: the register allocator of the fused point-wise kernels (kernels/eltwise_params.h, fused_allocate), checked
on the host: tests/native/fused_alloc_check.cpp builds 20000 random programs in single-assignment form, evaluates
them as written and through the physical registers, phase by phase with the per-element phases repeated, and
compares every output."""
import os
import subprocess
import tempfile

from conftest import ROOT


def test_allocated_programs_compute_what_the_single_assignment_form_computes():
    src = os.path.join(ROOT, "tests", "native", "fused_alloc_check.cpp")
    inc = os.path.join(ROOT, "graph-compiler_amd", "csrc")
    with tempfile.TemporaryDirectory() as d:
        exe = os.path.join(d, "fused_alloc_check")
        subprocess.run(["g++", "-std=c++17", "-O1", "-I", inc, "-o", exe, src], check=True)
        out = subprocess.run([exe], check=True, capture_output=True, text=True).stdout.split()
    assert out[0] == "ok" and int(out[1]) > 10000
    assert int(out[3]) <= 15  # gcmi::FUSED_MAX_PHYS
