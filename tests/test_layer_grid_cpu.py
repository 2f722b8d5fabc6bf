"""CPU checks of the restated layer unit-test grids (tests/layer_grid.py): every grid has the number of cases the
reference's INSTANTIATE_TEST_SUITE_P yields after its own skip rules, the comparison rules behave as
test/test_utils.cc:104-172 on hand-made pairs, and a sample of every grid is accepted by the reference engine itself
(DEVICE_NAIVE against DEVICE_X86 where the reference has an x86 acc), so the model files say what the unit tests build."""
import numpy as np
import pytest

import layer_grid
import ref_driver

# cases per grid, counted by hand from the Values(...) lists and skip rules of the cited test files
EXPECTED = {"MatMul": 78, "InnerProduct": 512, "QuantizedInnerProduct": 160, "GELU": 96, "Tanh": 24, "Permute": 7296,
            "Add": 2880, "Sub": 2880, "Mul": 2880, "Div": 2880, "QuantizedAdd": 216, "LayerNorm": 240, "Reformat": 96}


@pytest.mark.parametrize("op", sorted(EXPECTED))
def test_grid_sizes(op):
    n = sum(1 for _ in layer_grid.GRIDS[op](np.random.default_rng(0)))
    assert n == EXPECTED[op], (op, n)


def test_comparison_rules():
    a = np.array([1.0, 2.0, 0.0], np.float32)
    assert layer_grid.compare(a, a.copy(), layer_grid.DT_FLOAT) is None
    assert layer_grid.compare(a, a + np.float32(5e-5), layer_grid.DT_FLOAT) is None          # below the absolute floor
    assert layer_grid.compare(a, a * np.float32(1.015), layer_grid.DT_FLOAT) is None         # 0.75 % of |a| + |b|
    big = np.linspace(-1, 1, 1000).astype(np.float32)
    off = big.copy()
    off[10] += 0.1
    assert layer_grid.compare(big, off, layer_grid.DT_HALF) is None                         # cosine similarity saves it
    assert layer_grid.compare(big, -big, layer_grid.DT_HALF) is not None
    q = np.array([1, -128, 127], np.int8)
    assert layer_grid.compare(q, np.array([2, -127, 126], np.int8), layer_grid.DT_INT8) is None
    assert layer_grid.compare(q, np.array([3, -128, 127], np.int8), layer_grid.DT_INT8) is not None
    assert layer_grid.compare(a, a.reshape(1, 3), layer_grid.DT_FLOAT) is not None           # dims differ


@pytest.mark.skipif(not ref_driver.available(), reason="oracle/_ref (the reference engine) was not built")
@pytest.mark.parametrize("op", ["MatMul", "InnerProduct", "QuantizedInnerProduct", "Softmax", "LayerNorm", "GELU", "Permute",
                                "Add", "Div", "QuantizedAdd", "Reformat", "Reshape", "Squeeze", "Unsqueeze"])
def test_sampled_cases_run_on_the_reference_engine(op):
    rng = np.random.default_rng(7)
    ran = 0
    for i, case in enumerate(layer_grid.GRIDS[op](rng)):
        if i % (97 if op != "Reformat" else 19) or case.inputs is None:
            continue
        outs = []
        for device in ("NAIVE", "X86"):
            s = ref_driver.RefSession(case.graph, device)
            for name, arr in case.inputs.items():
                s.set_input(name, arr)
            s.forward()
            dt = s.output_data_type("output0")
            outs.append(s.output_as("output0", np.int8 if dt == layer_grid.DT_INT8 else np.float32))
            s.close()
        why = layer_grid.compare(outs[0], outs[1], dt)
        assert why is None, (case.ident, why)
        ran += 1
    assert ran > 0
