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
                                "Add", "Cast", "Div", "QuantizedAdd", "Reformat", "Reshape", "Squeeze", "Unsqueeze"])
def test_sampled_cases_run_on_the_reference_engine(op):
    rng = np.random.default_rng(7)
    ran = 0
    for i, case in enumerate(layer_grid.GRIDS[op](rng)):
        if i % ({"Reformat": 19, "Cast": 1}.get(op, 97)) or case.inputs is None:
            continue
        outs = []
        for device in ("NAIVE", "X86"):
            s = ref_driver.RefSession(case.graph, device)
            for name, arr in case.inputs.items():
                s.set_input(name, arr)
            s.forward()
            dt = s.output_data_type("output0")
            outs.append(s.output_as("output0", np.int8 if dt == layer_grid.DT_INT8 else
                                    (np.int32 if dt == layer_grid.DT_INT32 else np.float32)))
            s.close()
        why = layer_grid.compare(outs[0], outs[1], dt)
        assert why is None, (case.ident, why)
        ran += 1
    assert ran > 0


@pytest.mark.skipif(not ref_driver.available(), reason="oracle/_ref (the reference engine) was not built")
def test_gather_grid_on_the_reference_engine_is_numpy_take():
    """The Gather grid is this repository's own (the reference has no unit test for the layer): on DEVICE_NAIVE every
    case equals numpy's take with the negative indices wrapped (cpu_gather_layer_acc.cc:74-77; the reference's x86 acc
    refuses negative indices, x86_gather_layer_acc.cc:66-70, so it is not the second device here)."""
    rng = np.random.default_rng(7)
    ran = 0
    for i, case in enumerate(layer_grid.GRIDS["Gather"](rng)):
        if i % 3:
            continue
        s = ref_driver.RefSession(case.graph, "NAIVE")
        for name, arr in case.inputs.items():
            s.set_input(name, arr)
        s.forward()
        dt = s.output_data_type("output0")
        out = s.output_as("output0", np.int32 if dt == layer_grid.DT_INT32 else np.float32)
        s.close()
        data, idx, axis = case.expect
        assert np.array_equal(out, np.take(data, idx, axis=axis)), case.ident
        ran += 1
    assert ran > 20
