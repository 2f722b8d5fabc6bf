"""Compile the gfx950 kernels + C ABI into tnn_amd/lib/libtnn_rocm.so (hipcc cross-compiles
without a GPU).  Run as `python -m tnn_amd.build`."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libtnn_rocm.so")

HIP_SOURCES = ["runtime.hip", "elementwise.hip", "rowwise.hip", "gemm.hip", "attention.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    # hipcc contracts a*b+c into an FMA by default; the int8 epilogues and quantisers must round the
    # product and the +-0.5 add separately (as the CPU paths do), so contraction is off everywhere
    # and kernels spell fmaf() where a fused multiply-add is wanted.
    "-ffp-contract=off",
    # packed fp32 instructions are kept off on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result", "-Wno-unknown-attributes",
]


def build_kernels(verbose=True):
    os.makedirs(LIB_DIR, exist_ok=True)
    objs = []
    procs = []
    for src in HIP_SOURCES:
        obj = os.path.join(LIB_DIR, src.replace(".hip", ".o"))
        cmd = ["hipcc"] + HIPCC_FLAGS + ["-I", os.path.join(ROOT, "include"), "-I", CSRC,
                                         "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if out.strip() and verbose:
            print(out)
        if p.returncode != 0:
            failed = True
            print("FAILED: %s" % src, file=sys.stderr)
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB_PATH


if __name__ == "__main__":
    build_kernels()
