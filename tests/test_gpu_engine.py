"""The DEVICE_ROCM backend inside the reference engine itself.

oracle/_ref/libtnn_rocm_engine.so is this repository's backend sources compiled against the reference's headers and
linked against the reference engine built from its own sources (oracle/Makefile.ref).  Loading it registers the device,
its layer accs, the optimizer passes, the blob converter and the network implementation with that engine, and the
engine's own TNN / Instance / DefaultNetwork / BlobManager then run a model on DEVICE_ROCM: SetInputMat, Forward,
GetOutputMat through the reference's code, side by side with its DEVICE_NAIVE path in the same process."""
import ctypes
import os

import numpy as np
import pytest

import ref_driver
from tnn_amd import tnnmodel
from tnn_amd.encoder import EncoderConfig, make_inputs, make_weights

pytestmark = pytest.mark.gpu

PLUGIN = os.path.join(ref_driver.ROOT, "oracle", "_ref", "libtnn_rocm_engine.so")
_plugin = None


def say(msg):
    print("[case] " + msg, flush=True)


def rel_err(a, b):
    return float(np.abs(a.astype(np.float64) - b.astype(np.float64)).max() / max(np.abs(b).max(), 1e-30))


def engine():
    global _plugin
    if not (ref_driver.available() and os.path.exists(PLUGIN)):
        pytest.skip("oracle/_ref (the reference engine and the backend linked against it) was not built")
    ref_driver.lib()
    if _plugin is None:
        _plugin = ctypes.CDLL(PLUGIN)
    return ref_driver


def run(graph, device, inputs, out_name, forwards=1):
    s = ref_driver.RefSession(graph, device)
    for name, arr in inputs.items():
        s.set_input(name, arr)
    outs = []
    for _ in range(forwards):
        s.forward()
        outs.append(s.output(out_name))
    s.close()
    return outs


def test_encoder_on_device_rocm_inside_the_reference_engine():
    """Two BERT-base-width encoder layers with embeddings and a padding mask: the reference engine's DEVICE_NAIVE result
    against the same engine running DEVICE_ROCM in fp32 blobs (bar 2e-3) and in fp16 blobs with the fused kernels (bar
    1e-2); five forwards each, so the recorded-graph replay of the backend's network runs under the engine as well; and
    against this repository's own host running the same backend sources."""
    engine()
    from tnn_amd import host
    say("reference engine: DEVICE_NAIVE vs DEVICE_ROCM (fp32, fp16), 2-layer encoder B3 S64")
    cfg = EncoderConfig.bert_base(2)
    w = make_weights(cfg, seed=41, bias_std=0.02)
    B, S = 3, 64
    ids, seg, lens, mask = make_inputs(cfg, B, S, 20, S, seed=42)
    graph = tnnmodel.encoder_graph(cfg, w, B, S)
    inputs = {"input_ids": ids.astype(np.int32), "token_type_ids": seg.astype(np.int32),
              "attention_bias": mask.reshape(B, 1, 1, S).astype(np.float32)}
    naive = run(graph, "NAIVE", inputs, "last_hidden")[0]
    say("  DEVICE_NAIVE done")
    for device, bar in (("ROCM:fp32", 2e-3), ("ROCM", 1e-2)):
        outs = run(graph, device, inputs, "last_hidden", forwards=5)
        errs = [rel_err(o, naive) for o in outs]
        say("  %s vs DEVICE_NAIVE over five forwards: %s" % (device, " ".join("%.3g" % e for e in errs)))
        assert max(errs) <= bar
        assert all(np.array_equal(o, outs[0]) for o in outs[1:])   # eager, recorded and replayed forwards agree exactly
        precision = "fp32" if device.endswith("fp32") else "fp16"
        inst = host.RocmInstance.from_graph(graph, precision)
        for name, arr in inputs.items():
            inst.set_input(name, arr)
        inst.forward()
        own = inst.output("last_hidden")
        inst.close()
        e = rel_err(outs[0], own)
        say("  %s vs this repository's host (%s): %.3g" % (device, precision, e))
        assert e <= (1e-6 if precision == "fp32" else 2e-3)


def test_single_attention_layer_on_device_rocm_inside_the_reference_engine():
    """BASELINE configuration 1 (one self-attention layer, fp32, S128 H768 h12, the un-fused op sequence of the
    reference's own CPU-runnable case) through the reference engine on DEVICE_NAIVE and on DEVICE_ROCM."""
    engine()
    say("reference engine: configuration 1 on DEVICE_NAIVE vs DEVICE_ROCM fp32")
    cfg = EncoderConfig(1, 768, 12, 3072)
    lw = make_weights(cfg, seed=43, with_embeddings=False)["layers"][0]
    graph = tnnmodel.attention_layer_graph(lw, 128, 768, 12)
    x = np.random.default_rng(44).standard_normal((128, 768)).astype(np.float32)
    naive = run(graph, "NAIVE", {"x": x}, "y")[0]
    rocm = run(graph, "ROCM:fp32", {"x": x}, "y", forwards=4)
    errs = [rel_err(o, naive) for o in rocm]
    say("  rel err over four forwards: %s" % " ".join("%.3g" % e for e in errs))
    assert max(errs) <= 2e-3


def test_int8_encoder_on_device_rocm_inside_the_reference_engine(monkeypatch):
    """A two-layer encoder with int8 projections (QuantizedInnerProduct layers and blob scales in the model, no Reformat
    layers: the backend's own insertion pass writes them, the engine's serves its CPU devices only), calibrated on this
    repository's fp32 forward.  Inside the reference engine DEVICE_ROCM gives, value for value, what this repository's
    host gives with the same backend sources - with the explicit Reformat chain and with the fused int8 layers - and
    stays close to the engine's own DEVICE_NAIVE run of the same quantised model."""
    engine()
    from tnn_amd import host, quant
    say("reference engine: int8 encoder on DEVICE_NAIVE vs DEVICE_ROCM")
    cfg = EncoderConfig.bert_base(2)
    w = make_weights(cfg, seed=51)
    B, S = 2, 64
    ids, seg, lens, mask = make_inputs(cfg, B, S, 24, S, seed=52)
    inputs = {"input_ids": ids.astype(np.int32), "token_type_ids": seg.astype(np.int32),
              "attention_bias": mask.reshape(B, 1, 1, S).astype(np.float32)}
    names = quant.calibration_outputs(cfg)
    inst = host.RocmInstance.from_graph(tnnmodel.encoder_graph(cfg, w, B, S, extra_outputs=names), "fp32")
    for k, v in inputs.items():
        inst.set_input(k, v)
    inst.forward()
    scales = {n: quant.activation_scale(inst.output(n, max_elems=1 << 24)) for n in names}
    inst.close()
    graph = quant.int8_encoder_graph(cfg, w, scales, B, S)
    naive = run(graph, "NAIVE", inputs, "last_hidden")[0]
    x86 = run(graph, "X86", inputs, "last_hidden")[0]    # the quantiser forms this backend follows (reciprocal multiply)
    say("  DEVICE_NAIVE and DEVICE_X86 done; they differ by %.3g" % rel_err(x86, naive))
    for fuse in ("0", "1"):
        monkeypatch.setenv("TNN_ROCM_FUSE_INT8", fuse)
        for device, precision in (("ROCM:fp32", "fp32"), ("ROCM", "fp16")):
            outs = run(graph, device, inputs, "last_hidden", forwards=4)
            assert all(np.array_equal(o, outs[0]) for o in outs[1:])
            inst = host.RocmInstance.from_graph(graph, precision)
            for k, v in inputs.items():
                inst.set_input(k, v)
            inst.forward()
            own = inst.output("last_hidden")
            inst.close()
            e_own, e_naive, e_x86 = rel_err(outs[0], own), rel_err(outs[0], naive), rel_err(outs[0], x86)
            say("  fused=%s %s: vs this repository's host %.3g, vs DEVICE_NAIVE %.3g, vs DEVICE_X86 %.3g"
                % (fuse, device, e_own, e_naive, e_x86))
            assert e_own == 0.0
            # a quantised network amplifies last-ulp differences of its float layers into single int8 steps, so the
            # engines' two CPU devices differ from each other by about as much as the GPU differs from either
            # (observed on MI355X: 1.5e-2 .. 3.5e-2 against either CPU device, while DEVICE_NAIVE and DEVICE_X86 differ
            # from each other by 2e-2 .. 3e-2; the per-projection int8 outputs are bit-exact in test_gpu_golden.py)
            assert e_naive <= 5e-2 and e_x86 <= 5e-2


def test_benchmark_model_inside_the_reference_engine():
    """The benchmark's own model (12-layer BERT-base, batch 8, seq 384, seeds of bench.py) run by the reference engine on
    DEVICE_ROCM: the same values as this repository's host gives, and the reference benchmark tool's loop
    (SetInputMat x3 + Forward + GetOutputMat, 5 warm-up + 20 timed) timed on both, printed side by side."""
    engine()
    from tnn_amd import host
    say("reference engine: the benchmark model on DEVICE_ROCM")
    cfg = EncoderConfig.bert_base(12)
    w = make_weights(cfg, seed=20240601)
    B, S = 8, 384
    ids, seg, lens, mask = make_inputs(cfg, B, S, 200, S, seed=20240602)
    graph = tnnmodel.encoder_graph(cfg, w, B, S)
    inputs = {"input_ids": ids.astype(np.int32), "token_type_ids": seg.astype(np.int32),
              "attention_bias": mask.reshape(B, 1, 1, S).astype(np.float32)}
    s = ref_driver.RefSession(graph, "ROCM")
    for name, arr in inputs.items():
        s.set_input(name, arr)
    for _ in range(4):
        s.forward()
    in_engine = s.output("last_hidden")
    mn, avg, mx = s.time_loop(5, 20, "last_hidden")
    fwd = s.time_forward(5, 50)
    s.close()
    inst = host.RocmInstance.from_graph(graph, "fp16")
    for name, arr in inputs.items():
        inst.set_input(name, arr)
    for _ in range(4):
        inst.forward()
    own = inst.output("last_hidden")
    omn, oavg, omx = inst.time_loop(5, 20, "last_hidden")
    inst.close()
    say("  in the reference engine: Forward %.3f ms; tool loop min/avg/max %.3f / %.3f / %.3f ms" % (fwd * 1e3, mn * 1e3, avg * 1e3, mx * 1e3))
    say("  this repository's host:  tool loop min/avg/max %.3f / %.3f / %.3f ms" % (omn * 1e3, oavg * 1e3, omx * 1e3))
    assert np.isfinite(in_engine).all() and rel_err(in_engine, own) == 0.0
    assert fwd < 5e-3   # milliseconds, not the seconds of a CPU path: the fused kernels and the graph replay ran


PROFILE_CHILD = r"""
import ctypes, os, sys
import numpy as np
root = sys.argv[1]
sys.path.insert(0, root)
from tnn_amd import tnnmodel
from tnn_amd.encoder import EncoderConfig, make_inputs, make_weights
prof = os.path.join(root, "oracle", "_ref", "prof")
drv = ctypes.CDLL(os.path.join(prof, "libtnn_ref_driver.so"))
ctypes.CDLL(os.path.join(prof, "libtnn_rocm_engine.so"))
drv.tnn_ref_create.restype = ctypes.c_void_p
cfg = EncoderConfig.bert_base(2)
w = make_weights(cfg, seed=61, bias_std=0.02)
B, S = 2, 64
ids, seg, lens, mask = make_inputs(cfg, B, S, 20, S, seed=62)
g = tnnmodel.encoder_graph(cfg, w, B, S)
proto, model = g.proto().encode(), g.model()
err = ctypes.create_string_buffer(512)
h = drv.tnn_ref_create(proto, ctypes.c_size_t(len(proto)), model, ctypes.c_size_t(len(model)), b"ROCM", 0, err, ctypes.c_size_t(512))
assert h, err.value
h = ctypes.c_void_p(h)
for name, arr, code in (("input_ids", ids.astype(np.int32), 1), ("token_type_ids", seg.astype(np.int32), 1),
                        ("attention_bias", mask.reshape(B, 1, 1, S).astype(np.float32), 0)):
    a = np.ascontiguousarray(arr)
    dims = (ctypes.c_int * a.ndim)(*a.shape)
    assert drv.tnn_ref_set_input(h, name.encode(), a.ctypes.data_as(ctypes.c_void_p), code, dims, a.ndim) == 0
for _ in range(4):          # beyond the third forward the network replays a recorded graph ...
    assert drv.tnn_ref_forward(h) == 0
buf = ctypes.create_string_buffer(1 << 16)
assert drv.tnn_ref_profile(h, 3, buf, ctypes.c_size_t(1 << 16)) == 0      # ... and profiling must still see layers
print(buf.value.decode())
assert drv.tnn_ref_forward(h) == 0
"""


def test_profiler_build_of_the_engine_reports_every_layer():
    """A profiler build of the reference engine (-DTNN_PROFILE, oracle/_ref/prof) with the backend linked into it:
    between Instance::StartProfile and FinishProfile the backend times every layer with an event pair and the engine
    prints its per-layer table (core/profile.cc:111-201).  Run in a process of its own (the two builds of the engine
    cannot share one)."""
    import subprocess
    import sys
    from tnn_amd import host
    prof = os.path.join(ref_driver.ROOT, "oracle", "_ref", "prof")
    if not os.path.exists(os.path.join(prof, "libtnn_rocm_engine.so")):
        pytest.skip("oracle/_ref/prof (the profiler build of the reference engine) was not built")
    say("reference engine, profiler build: per-layer table on DEVICE_ROCM")
    r = subprocess.run([sys.executable, "-c", PROFILE_CHILD, ref_driver.ROOT], capture_output=True, text=True, timeout=300)
    say("  child exit %d" % r.returncode)
    assert r.returncode == 0, r.stderr[-3000:]
    table = r.stdout
    print(table[-3000:], flush=True)
    # the layers of the rewritten graph, as this repository's host plans the same model
    cfg = EncoderConfig.bert_base(2)
    w = make_weights(cfg, seed=61, bias_std=0.02)
    plan = host.plan(tnnmodel.encoder_graph(cfg, w, 2, 64), precision="fp16")
    for layer in plan:
        assert layer["name"] in table, layer["name"]
    for type_str in ("RocmFusedAttention", "RocmFusedLinear", "RocmFusedEmbedding", "LayerNorm"):
        assert type_str in table, type_str


def test_model_input_shared_by_quantised_and_float_layers():
    """A model input that a quantised layer and a float layer both read (the head-of-graph Reformat case of
    net_optimizer_insert_int8_reformat.cc:84-131): DEVICE_ROCM in the reference engine against its DEVICE_X86, whose
    quantiser forms the backend follows, value for value in fp32 blobs."""
    engine()
    from test_host_plan import _input_read_by_both_kinds
    say("reference engine: model input read by quantised and float layers")
    g = _input_read_by_both_kinds()
    x = (np.random.default_rng(3).standard_normal((64, 128)) * 0.8).astype(np.float32)
    x86 = run(g, "X86", {"x": x}, "z")[0]
    rocm = run(g, "ROCM:fp32", {"x": x}, "z", forwards=4)
    assert all(np.array_equal(o, rocm[0]) for o in rocm[1:])
    d = np.abs(rocm[0] - x86)
    say("  max |d| vs DEVICE_X86 %.3g (one int8 step of the output scale is 0.05)" % d.max())
    assert d.max() <= 1e-6


def test_blob_memory_brought_by_the_caller():
    """SHARE_MEMORY_MODE_SET_FROM_EXTERNAL (include/tnn/core/common.h, instance.cc GetForwardMemorySize /
    SetForwardMemory, blob_manager.cc): the engine allocates no blob memory, reports the size, and the caller hands over
    device memory; blobs are then base + bytes_offset into it.  Same result as the engine-allocated run, also after the
    memory is exchanged for another buffer between forwards (the recorded graph names the old addresses and must not be
    replayed)."""
    engine()
    import torch
    say("reference engine: DEVICE_ROCM with blob memory brought by the caller")
    cfg = EncoderConfig.bert_base(2)
    w = make_weights(cfg, seed=43, bias_std=0.02)
    B, S = 2, 64
    ids, seg, lens, mask = make_inputs(cfg, B, S, 20, S, seed=44)
    graph = tnnmodel.encoder_graph(cfg, w, B, S)
    inputs = {"input_ids": ids.astype(np.int32), "token_type_ids": seg.astype(np.int32),
              "attention_bias": mask.reshape(B, 1, 1, S).astype(np.float32)}
    for device in ("ROCM:fp32", "ROCM"):
        plain = run(graph, device, inputs, "last_hidden")[0]
        s = ref_driver.RefSession(graph, device + "+extmem")
        size = s.forward_memory_size()
        say("  %s: forward memory %d bytes" % (device, size))
        assert size > 0
        first = torch.full((size + 256,), 0x5a, dtype=torch.uint8, device="cuda")
        second = torch.full((size + 256,), 0xa5, dtype=torch.uint8, device="cuda")
        outs = []
        for buf, forwards in ((first, 4), (second, 4), (first, 1)):
            base = (buf.data_ptr() + 255) // 256 * 256
            s.set_forward_memory(base)
            for name, arr in inputs.items():
                s.set_input(name, arr)
            for _ in range(forwards):
                s.forward()
                outs.append(s.output("last_hidden"))
        s.close()
        assert all(np.array_equal(o, plain) for o in outs), device


def test_instance_reshape_inside_the_reference_engine():
    """Instance::Reshape of the reference engine itself (instance.cc:48-128, default_network.cc:456-500) on DEVICE_ROCM: an
    instance created for shapes up to B4 S96 walks through several (B, S), among them a sequence length that is no
    multiple of 8 and shapes seen before; at each shape, on each of three forwards, the result is that of the engine's
    DEVICE_NAIVE reshaped the same way (fp32 blobs 2e-3, fp16 blobs 1e-2)."""
    engine()
    say("reference engine: Instance::Reshape on DEVICE_ROCM next to DEVICE_NAIVE")
    cfg = EncoderConfig(2, 256, 4, 512)
    S_MAX = 96
    w = make_weights(cfg, seed=61, bias_std=0.05)
    w["pos_emb"] = w["pos_emb"][:S_MAX]
    # positions looked up by a third Gather: the constant-rows form names S_MAX rows, which the engine's own Add cannot
    # broadcast against a shorter sequence
    graph = tnnmodel.encoder_graph(cfg, w, 4, S_MAX, dynamic=True, position_ids=True)

    def shapes(B, S):
        return {"input_ids": [B, S], "token_type_ids": [B, S], "position_ids": [B, S], "attention_bias": [B, 1, 1, S]}

    sessions = {d: ref_driver.RefSession(graph, d, min_shapes=shapes(1, 8), max_shapes=shapes(4, S_MAX))
                for d in ("NAIVE", "ROCM:fp32", "ROCM")}
    for step, (B, S) in enumerate([(4, 96), (2, 40), (3, 24), (2, 36), (4, 96), (1, 8), (2, 40)]):
        ids, seg, lens, mask = make_inputs(cfg, B, S, max(S // 3, 1), S, seed=200 + step)
        outs = {}
        for d, s in sessions.items():
            s.reshape(shapes(B, S))
            s.set_input("input_ids", ids.astype(np.int32))
            s.set_input("token_type_ids", seg.astype(np.int32))
            s.set_input("position_ids", np.tile(np.arange(S, dtype=np.int32), (B, 1)))
            s.set_input("attention_bias", mask.reshape(B, 1, 1, S).astype(np.float32))
            res = []
            for _ in range(1 if d == "NAIVE" else 3):
                s.forward()
                res.append(s.output("last_hidden"))
            assert res[0].shape == (B, S, cfg.hidden), (d, res[0].shape)
            assert all(np.array_equal(r, res[0]) for r in res[1:]), d
            outs[d] = res[0]
        e32, e16 = rel_err(outs["ROCM:fp32"], outs["NAIVE"]), rel_err(outs["ROCM"], outs["NAIVE"])
        say("  B=%d S=%d: fp32 blobs %.3g, fp16 blobs %.3g" % (B, S, e32, e16))
        assert e32 <= 2e-3 and e16 <= 1e-2
    for s in sessions.values():
        s.close()


def test_sessions_inside_the_reference_engine_leave_no_memory_behind():
    """TNN::Init + CreateInst + Forward x4 + the instance's and the interpreter's destruction, in the reference engine on
    DEVICE_ROCM, twenty times over: the device memory in use (read from the driver) and the resident host memory stay
    where they were after the first four rounds"""
    engine()
    torch = pytest.importorskip("torch")
    say("reference engine: create / forward / destroy cycles on DEVICE_ROCM, memory in use")
    cfg = EncoderConfig(2, 256, 4, 512)
    w = make_weights(cfg, seed=11, bias_std=0.02)
    B, S = 2, 64
    ids, seg, lens, mask = make_inputs(cfg, B, S, 20, S, seed=12)
    graph = tnnmodel.encoder_graph(cfg, w, B, S)

    def resident():
        with open("/proc/self/statm") as f:
            return int(f.read().split()[1]) * 4096

    def in_use():
        free, total = torch.cuda.mem_get_info()
        return total - free

    def cycle(device):
        s = ref_driver.RefSession(graph, device)
        s.set_input("input_ids", ids.astype(np.int32))
        s.set_input("token_type_ids", seg.astype(np.int32))
        s.set_input("attention_bias", mask.reshape(B, 1, 1, S).astype(np.float32))
        for _ in range(4):
            s.forward()
        s.output("last_hidden")
        s.close()

    for device in ("ROCM", "ROCM:fp32"):
        for _ in range(4):
            cycle(device)
        dev0, host0 = in_use(), resident()
        for _ in range(16):
            cycle(device)
        dev1, host1 = in_use(), resident()
        say("  %s: device in use %.1f -> %.1f MiB, host resident %.1f -> %.1f MiB over 16 cycles"
            % (device, dev0 / 2**20, dev1 / 2**20, host0 / 2**20, host1 / 2**20))
        assert dev1 - dev0 <= 2 << 20, (device, dev0, dev1)
        assert host1 - host0 <= 4 << 20, (device, host0, host1)


def test_blob_converter_grid_inside_the_reference_engine():
    """The reference's BlobConverterTest (test/unit_test/blob_converter_test.cc) for the Mat type of this path: the same
    fp32 NCHW Mat through ConvertFromMat and ConvertToMat with per-channel scale and bias, by a BlobConverter on a
    DEVICE_NAIVE blob and by one on a DEVICE_ROCM blob of the same dims, over the test's grid of batch, channel, size,
    scale and bias (96 cases); the test's bar is 0.01, fp32 blobs meet it with no difference at all."""
    engine()
    from test_gpu_host import converter_grid
    say("reference engine: blob converter grid, DEVICE_ROCM next to DEVICE_NAIVE")
    rng = np.random.default_rng(10)
    worst16 = 0.0
    for batch, channel, size, scale, bias in converter_grid():
        g = tnnmodel.Graph()
        g.add_input("x", [batch, channel, size, size])
        g.add_layer("GELU", "act", ["x"], ["y"])
        g.add_output("y")
        x = rng.random((batch, channel, size, size), dtype=np.float32)
        sc = [scale * (c + 1) for c in range(channel)]
        bi = [bias * (c + 1) for c in range(channel)]
        outs = {}
        for device in ("NAIVE", "ROCM:fp32", "ROCM"):
            s = ref_driver.RefSession(g, device)
            outs[device] = s.input_blob_round_trip("x", x, sc, bi)
            s.close()
        case = (batch, channel, size, scale, bias)
        assert np.array_equal(outs["ROCM:fp32"], outs["NAIVE"]), case
        d16 = np.abs(outs["ROCM"] - outs["NAIVE"])
        assert np.all(d16 <= 1e-3 + 1e-3 * np.abs(outs["NAIVE"])), case     # one half rounding of the blob, then * scale
        worst16 = max(worst16, float(d16.max()))
    say("  fp32 blobs identical to DEVICE_NAIVE; half blobs differ by at most %.3g" % worst16)


def test_device_mats_inside_the_reference_engine():
    """Instance::SetInputMat / GetOutputMat of the reference engine with Mats in DEVICE_ROCM memory (the engine allocates the
    output Mat through RocmDevice::Allocate(mat type, dims)): same bits as with host Mats; and the converter grid with
    device Mats against DEVICE_NAIVE."""
    engine()
    torch = pytest.importorskip("torch")
    from test_gpu_host import converter_grid, _device_to_numpy
    say("reference engine: Mats in device memory")
    cfg = EncoderConfig(2, 256, 4, 512)
    w = make_weights(cfg, seed=83, bias_std=0.05)
    B, S = 2, 40
    w["pos_emb"] = w["pos_emb"][:S]
    ids, seg, lens, mask = make_inputs(cfg, B, S, 9, S, seed=84)
    graph = tnnmodel.encoder_graph(cfg, w, B, S)
    for device in ("ROCM:fp32", "ROCM"):
        s = ref_driver.RefSession(graph, device)
        s.set_input("input_ids", ids.astype(np.int32))
        s.set_input("token_type_ids", seg.astype(np.int32))
        s.set_input("attention_bias", mask.reshape(B, 1, 1, S).astype(np.float32))
        s.forward()
        want = s.output("last_hidden")
        s.set_input("input_ids", np.zeros((B, S), np.int32))
        s.forward()
        d_ids = torch.from_numpy(ids.astype(np.int32)).cuda()
        d_seg = torch.from_numpy(seg.astype(np.int32)).cuda()
        d_mask = torch.from_numpy(mask.reshape(B, 1, 1, S).astype(np.float32)).cuda()
        torch.cuda.synchronize()
        s.set_input_device("input_ids", d_ids.data_ptr(), True, [B, S])
        s.set_input_device("token_type_ids", d_seg.data_ptr(), True, [B, S])
        s.set_input_device("attention_bias", d_mask.data_ptr(), False, [B, 1, 1, S])
        s.forward()
        ptr, shape = s.output_device("last_hidden")
        got = _device_to_numpy(ptr, shape, np.float32)
        assert shape == list(want.shape) and np.array_equal(got, want), device
        s.close()
    rng = np.random.default_rng(11)
    for batch, channel, size, scale, bias in converter_grid():
        g = tnnmodel.Graph()
        g.add_input("x", [batch, channel, size, size])
        g.add_layer("GELU", "act", ["x"], ["y"])
        g.add_output("y")
        x = rng.random((batch, channel, size, size), dtype=np.float32)
        sc = [scale * (c + 1) for c in range(channel)]
        bi = [bias * (c + 1) for c in range(channel)]
        s = ref_driver.RefSession(g, "NAIVE")
        want = s.input_blob_round_trip("x", x, sc, bi)
        s.close()
        s = ref_driver.RefSession(g, "ROCM:fp32")
        d_in = torch.from_numpy(x).cuda()
        d_out = torch.full_like(d_in, -7.0)
        torch.cuda.synchronize()
        s.input_blob_round_trip("x", None, sc, bi, device_ptrs=(d_in.data_ptr(), d_out.data_ptr()))
        torch.cuda.synchronize()
        s.close()
        assert np.array_equal(d_out.cpu().numpy(), want), (batch, channel, size, scale, bias)


def test_mat_utils_copy_inside_the_reference_engine():
    """the reference's own MatUtils::Copy finds DEVICE_ROCM's Mat converter (REGISTER_MAT_CONVERTER) and the device's
    Allocate(mat type, dims): host -> DEVICE_ROCM -> DEVICE_ROCM -> host returns the values"""
    engine()
    say("reference engine: MatUtils::Copy through DEVICE_ROCM")
    rng = np.random.default_rng(5)
    for shape in ((1, 1, 1, 1), (2, 3, 7, 5), (4, 1, 96, 256)):   # the engine's check wants the four image dims
        a = rng.standard_normal(shape).astype(np.float32)
        assert np.array_equal(ref_driver.mat_copy_round_trip("ROCM", a), a), shape


def test_weight_only_int8_model_inside_the_reference_engine():
    """A dynamic-range quantised model (int8 MatMul weights and embedding tables + fp32 scales) in the reference engine:
    its own dequantisation pass runs ahead of the ROCm passes (both at priority P1, ordered by name), so DEVICE_ROCM
    still runs the fused layers and agrees with DEVICE_NAIVE on the same file."""
    engine()
    say("reference engine: weight-only int8 model, DEVICE_ROCM next to DEVICE_NAIVE")
    cfg = EncoderConfig(2, 256, 4, 512)
    w = make_weights(cfg, seed=93, bias_std=0.05)
    B, S = 2, 40
    w["pos_emb"] = w["pos_emb"][:S]
    ids, seg, lens, mask = make_inputs(cfg, B, S, 9, S, seed=94)
    graph = tnnmodel.encoder_graph(cfg, w, B, S)
    graph.weight_only_int8()
    inputs = {"input_ids": ids.astype(np.int32), "token_type_ids": seg.astype(np.int32),
              "attention_bias": mask.reshape(B, 1, 1, S).astype(np.float32)}
    want = run(graph, "NAIVE", inputs, "last_hidden")[0]
    got32 = run(graph, "ROCM:fp32", inputs, "last_hidden", forwards=2)
    got16 = run(graph, "ROCM", inputs, "last_hidden", forwards=4)
    assert all(np.array_equal(g, got32[0]) for g in got32) and all(np.array_equal(g, got16[0]) for g in got16)
    e32, e16 = rel_err(got32[0], want), rel_err(got16[0], want)
    say("  fp32 blobs %.3g, fp16 blobs (fused) %.3g" % (e32, e16))
    assert e32 <= 2e-3 and e16 <= 1e-2
    # and against the float model: the quantisation itself costs something, the device adds nothing to it
    plain = run(tnnmodel.encoder_graph(cfg, w, B, S), "NAIVE", inputs, "last_hidden")[0]
    assert 1e-4 < rel_err(want, plain) < 0.2


def test_half_precision_weight_file_inside_the_reference_engine():
    """a model file with half-precision weight records in the reference engine: DEVICE_NAIVE widens them layer by layer,
    DEVICE_ROCM ahead of its rewrites; the two agree as they do on the fp32 file, and DEVICE_ROCM gives on the half file
    exactly what it gives on the fp32 file of the same values"""
    engine()
    say("reference engine: half-precision weight file, DEVICE_ROCM next to DEVICE_NAIVE")
    cfg = EncoderConfig(2, 256, 4, 512)
    w = make_weights(cfg, seed=99, bias_std=0.05)
    B, S = 2, 40
    w["pos_emb"] = w["pos_emb"][:S]

    def r16(a):
        return a.astype(np.float16).astype(np.float32)
    w = {k: ([{n: r16(a) for n, a in lw.items()} for lw in v] if k == "layers" else r16(v)) for k, v in w.items()}
    ids, seg, lens, mask = make_inputs(cfg, B, S, 9, S, seed=100)
    inputs = {"input_ids": ids.astype(np.int32), "token_type_ids": seg.astype(np.int32),
              "attention_bias": mask.reshape(B, 1, 1, S).astype(np.float32)}
    plain = tnnmodel.encoder_graph(cfg, w, B, S)
    half = tnnmodel.encoder_graph(cfg, w, B, S)
    half.half_weights(tables=False, constants=False)   # what the engine's CPU devices widen: layer resources
    want = run(half, "NAIVE", inputs, "last_hidden")[0]
    assert np.array_equal(want, run(plain, "NAIVE", inputs, "last_hidden")[0])
    for device, bar in (("ROCM:fp32", 2e-3), ("ROCM", 1e-2)):
        got = run(half, device, inputs, "last_hidden", forwards=2)[0]
        assert np.array_equal(got, run(plain, device, inputs, "last_hidden")[0]), device
        e = rel_err(got, want)
        say("  %s: %.3g" % (device, e))
        assert e <= bar


def test_first_version_of_the_file_format_inside_the_reference_engine():
    """the same attention block written in the first version of the file format (no rank or type on the input lines, no
    dims in the weight records), read by the reference's own parser: DEVICE_ROCM agrees with DEVICE_NAIVE and gives the
    bits it gives on the current format"""
    engine()
    say("reference engine: first version of the file format")
    cfg = EncoderConfig(1, 256, 4, 512)
    lw = make_weights(cfg, seed=5, bias_std=0.05)["layers"][0]
    B, S, H = 2, 40, 256
    x = np.random.default_rng(6).standard_normal((B * S, H)).astype(np.float32)
    mask = np.zeros((B, 1, 1, S), np.float32)
    mask[1, 0, 0, 25:] = -10000.0
    inputs = {"hidden": x, "attention_bias": mask}
    current = tnnmodel.attention_block_graph(lw, B, S, H, 4, proj="inner_product")
    with tnnmodel.legacy_format():
        old = tnnmodel.attention_block_graph(lw, B, S, H, 4, proj="inner_product")
        got = {d: run(old, d, inputs, "y")[0] for d in ("NAIVE", "ROCM:fp32", "ROCM")}
    for d in ("ROCM:fp32", "ROCM"):
        assert np.array_equal(got[d], run(current, d, inputs, "y")[0]), d
    e32, e16 = rel_err(got["ROCM:fp32"], got["NAIVE"]), rel_err(got["ROCM"], got["NAIVE"])
    say("  fp32 blobs %.3g, fp16 blobs %.3g" % (e32, e16))
    assert e32 <= 2e-3 and e16 <= 1e-2
