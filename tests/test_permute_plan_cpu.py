"""Host logic of tnn_rocm_permute on the CPU: the launcher (normal form, choice between 16-byte / 4-byte row copies,
the tiled transpose and the generic gather) is compiled from the text of tnn_amd/csrc/elementwise.hip with g++, its
kernel launches run as bounds-checked host loops, and ~17 000 random cases are compared with a plain index loop.
A wrong stride or tile bound shows up here as an out-of-bounds count instead of as a GPU memory fault."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HARNESS = os.path.join(ROOT, "tests", "cpu_harness")


def _between(text, a, b):
    i = text.index(a)
    return text[i:text.index(b, i)]


def test_permute_launcher_indexing_stays_in_bounds(tmp_path):
    src = open(os.path.join(ROOT, "tnn_amd", "csrc", "elementwise.hip")).read()
    structs = _between(src, "struct PermDesc {", "template <typename T>\n__global__ void __launch_bounds__(kBlock) permute_kernel")
    tdesc = _between(src, "struct TransDesc {", "template <typename T>\n__global__ void __launch_bounds__(kBlock) permute_transpose_kernel")
    launcher = _between(src, "int tnn_rocm_permute(void *stream", "int tnn_rocm_gather(void *stream")
    parts = [open(os.path.join(HARNESS, n)).read() for n in
             ("permute_plan_prelude.inc", "permute_plan_kernels.inc", "permute_plan_main.inc")]
    cc = tmp_path / "permute_plan_check.cc"
    cc.write_text(parts[0] + structs + tdesc + parts[1] + launcher + parts[2])
    exe = tmp_path / "permute_plan_check"
    subprocess.check_call(["g++", "-O1", "-std=c++17", "-w", "-o", str(exe), str(cc)])
    out = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout[-2000:]
    last = out.stdout.strip().splitlines()[-1].split()  # "cases N bad B paths P"
    assert int(last[1]) > 10000 and int(last[3]) == 0
    assert int(last[5]) == 15, "every path (16-byte, 4-byte, element-wise, transpose) must have been taken"
