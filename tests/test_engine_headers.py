"""The DEVICE_ROCM backend sources against the engine's real headers.

tnn_amd/host/*.cc build in two ways: against this repository's restatement of the engine's plug-in contract
(tnn_host.h, the default) and, with -DTNN_ROCM_ENGINE_TREE, against the engine's own headers plus
rocm_engine_additions.h.  This test runs the second form through `g++ -fsyntax-only` with the reference tree's
include/ and source/ on the include path, in the C++ standard the engine builds with (C++11) and in the one this
repository uses, and expects no diagnostics of severity error.  It is what keeps `RocmDevice : AbstractDevice`,
`RocmContext : Context`, `Rocm*LayerAcc : AbstractLayerAcc`, `RocmNetwork : DefaultNetwork`, the optimizer passes
and every registration static honest against core/abstract_device.h, context.h, abstract_layer_acc.h,
default_network.h, optimizer/net_optimizer_manager.h and utils/blob_converter_internal.h.

Skipped where the reference tree is absent."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST = os.path.join(ROOT, "tnn_amd", "host")
REF = os.environ.get("TNN_REFERENCE_TREE", "/root/reference")
BACKEND_SOURCES = ["rocm_device.cc", "rocm_network.cc", "rocm_layer_accs.cc", "rocm_fused.cc", "rocm_fused_layers.cc"]

pytestmark = pytest.mark.skipif(not os.path.isdir(os.path.join(REF, "source", "tnn", "core")),
                                reason="reference tree not present")


@pytest.mark.parametrize("std", ["c++11", "c++14"])
@pytest.mark.parametrize("src", BACKEND_SOURCES)
def test_backend_source_compiles_against_engine_headers(src, std):
    cmd = ["g++", "-std=" + std, "-fsyntax-only", "-DTNN_ROCM_ENGINE_TREE", "-I" + os.path.join(REF, "include"),
           "-I" + os.path.join(REF, "source"), "-I" + os.path.join(ROOT, "include"), "-I" + HOST,
           os.path.join(HOST, src)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    errors = [l for l in r.stderr.splitlines() if " error" in l]
    assert r.returncode == 0 and not errors, "\n".join(errors[:20]) or r.stderr[-2000:]


CLANG = "/opt/rocm/llvm/bin/clang++"


@pytest.mark.skipif(not os.path.exists(CLANG), reason="no clang in this image")
@pytest.mark.parametrize("src", BACKEND_SOURCES)
def test_backend_source_compiles_with_clang_against_engine_headers(src):
    """a second compiler: clang rejects what g++ lets through, e.g. a constant of an engine enum whose value lies outside
    the enum's range of values (LayerType ends at 1001, so a constant of 0x7001 is not a constant expression)"""
    cmd = [CLANG, "-std=c++11", "-fsyntax-only", "-DTNN_ROCM_ENGINE_TREE", "-I" + os.path.join(REF, "include"),
           "-I" + os.path.join(REF, "source"), "-I" + os.path.join(ROOT, "include"), "-I" + HOST, os.path.join(HOST, src)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    errors = [l for l in r.stderr.splitlines() if " error" in l]
    assert r.returncode == 0 and not errors, "\n".join(errors[:20]) or r.stderr[-2000:]


@pytest.mark.parametrize("src", BACKEND_SOURCES)
def test_backend_source_compiles_in_a_profiler_build_of_the_engine(src):
    """-DTNN_PROFILE (the engine's TNN_PROFILER_ENABLE option, CMakeLists.txt:74-76) adds StartProfile / FinishProfile /
    AddProfilingData to Context and the networks; the backend's per-layer timing (RocmNetwork::ProfiledForward) only
    exists in that form"""
    cmd = ["g++", "-std=c++11", "-fsyntax-only", "-DTNN_ROCM_ENGINE_TREE", "-DTNN_PROFILE", "-I" + os.path.join(REF, "include"),
           "-I" + os.path.join(REF, "source"), "-I" + os.path.join(ROOT, "include"), "-I" + HOST, os.path.join(HOST, src)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    errors = [l for l in r.stderr.splitlines() if " error" in l]
    assert r.returncode == 0 and not errors, "\n".join(errors[:20]) or r.stderr[-2000:]


def test_backend_sources_do_not_include_the_restated_contract_in_engine_form():
    """in the engine form nothing of tnn_host.h may be reachable: the only headers of this repository the backend
    pulls in are its own rocm_*.h and the C ABI"""
    cmd = ["g++", "-std=c++11", "-DTNN_ROCM_ENGINE_TREE", "-I" + os.path.join(REF, "include"),
           "-I" + os.path.join(REF, "source"), "-I" + os.path.join(ROOT, "include"), "-I" + HOST, "-MM"]
    for src in BACKEND_SOURCES:
        deps = subprocess.run(cmd + [os.path.join(HOST, src)], capture_output=True, text=True, check=True).stdout
        mine = sorted({os.path.basename(t) for t in deps.replace("\\\n", " ").split() if t.startswith(ROOT)})
        assert "tnn_host.h" not in mine, (src, mine)
        assert set(mine) <= {src, "rocm_device.h", "rocm_network.h", "rocm_engine_additions.h", "tnn_rocm.h"}, (src, mine)
