"""The reference's own layer unit-test grids (tests/layer_grid.py) on DEVICE_ROCM inside the reference engine: every case
runs on the engine's DEVICE_NAIVE and on DEVICE_ROCM (fp16 blobs as the harness's PRECISION_AUTO gives them, fp32 blobs,
bf16 where the reference test lists it, int8 blobs for the quantised layers) and is judged by the harness's own
comparison rules.  One pytest case per op; each prints how many cases ran and passed."""
import os
import time

import numpy as np
import pytest

import layer_grid
import ref_driver
from test_gpu_engine import engine, say

pytestmark = pytest.mark.gpu

DEVICE = {"fp16": "ROCM", "fp32": "ROCM:fp32", "bf16": "ROCM:bf16"}
STRIDE = int(os.environ.get("TNN_LAYER_GRID_STRIDE", "1"))     # run every n-th case of each grid
MAX_ELEMS = layer_grid.MAX_ELEMS                               # larger blobs are left out (counted, see the summary)


def _session(graph, device, inputs, int8):
    s = ref_driver.RefSession(graph, device)
    for name, arr in inputs.items():
        s.set_input(name, arr)
    s.forward()
    dt = s.output_data_type("output0")
    out = s.output_as("output0", np.int8 if dt == layer_grid.DT_INT8 else (np.int32 if dt == layer_grid.DT_INT32 else np.float32))
    s.close()
    return out, dt


@pytest.mark.parametrize("op", sorted(layer_grid.GRIDS))
def test_reference_layer_grid(op):
    engine()
    rng = np.random.default_rng(102)
    ran = passed = too_large = 0
    failures = []
    t0 = time.time()
    for i, case in enumerate(layer_grid.GRIDS[op](rng)):
        if i % STRIDE:
            continue
        if case.inputs is None:
            too_large += 1
            continue
        try:
            ref, _ = _session(case.graph, "NAIVE", case.inputs, case.int8)
        except RuntimeError as e:
            failures.append("%s: DEVICE_NAIVE: %s" % (case.ident, e))
            ran += 1
            continue
        for precision in case.precisions:
            ran += 1
            try:
                got, dt = _session(case.graph, DEVICE[precision], case.inputs, case.int8)
                why = layer_grid.compare(ref, got, dt)
            except RuntimeError as e:
                why = str(e)
            if why is None:
                passed += 1
            else:
                failures.append("%s [%s]: %s" % (case.ident, precision, why))
    say("layer grid %-22s %5d run, %5d passed, %4d failed, %3d above %d elements left out, %.1f s"
        % (op, ran, passed, len(failures), too_large, MAX_ELEMS, time.time() - t0))
    for f in failures[:12]:
        say("    " + f)
    assert ran > 0 and not failures, "%d of %d cases failed, first: %s" % (len(failures), ran, failures[:3])
