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
    # per-kernel register / scratch figures as remarks; build_kernels() lists the kernels that spill
    "-Rpass-analysis=kernel-resource-usage",
]


def spilled_kernels(compiler_output):
    """[(kernel symbol, spilled VGPRs)] from the kernel-resource-usage remarks of one compilation."""
    out, name = [], None
    for line in compiler_output.splitlines():
        if "remark:" not in line:
            continue
        text = line.split("remark:", 1)[1].strip()
        if text.startswith("Function Name:"):
            name = text.split(":", 1)[1].split("[")[0].strip()
        elif text.startswith("VGPRs Spill:") and name:
            n = int(text.split(":", 1)[1].split("[")[0])
            if n > 0:
                out.append((name, n))
    return out


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
        for kernel, n in spilled_kernels(out):
            print("note: %s: %s spills %d VGPRs" % (src, kernel, n), file=sys.stderr)
        keep, skip = [], 0
        for l in out.splitlines():  # drop the remarks (and the two source lines clang prints under each)
            if "kernel-resource-usage" in l:
                skip = 2
            elif skip and (l.lstrip().startswith("|") or "|" in l[:12]):
                skip -= 1
            elif "packed-fp32-ops" not in l:
                keep.append(l)
        out = "\n".join(keep)
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


def build_simd_probe(verbose=True):
    """Compile csrc/probe_simd.hip (a stand-alone micro-benchmark of one SIMD: matrix pipe, vector ALU and LDS reads
    sharing its time) into tnn_amd/lib/probe_simd.  On demand only (`python -m tnn_amd.bench_ops --simd-probe`):
    nothing in the library uses it and build_kernels() does not compile it."""
    os.makedirs(LIB_DIR, exist_ok=True)
    exe = os.path.join(LIB_DIR, "probe_simd")
    cmd = ["hipcc", "--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off", "-Wno-unused-result", "-Xclang",
           "-target-feature", "-Xclang", "-packed-fp32-ops", "-I", CSRC, os.path.join(CSRC, "probe_simd.hip"), "-o", exe]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return exe


if __name__ == "__main__":
    build_kernels()
