"""Full-depth parity: the benchmark's own models at their real number of layers.

The short encoder cases elsewhere stop after 2-3 layers; here the 12-layer model that bench.py times (same seeds,
same shapes, whole-forward graph replay on), the 24-layer BERT-large of config 5 and the 12-layer int8 model of config 4
run at full depth.  Sequences are independent, so the CPU checker evaluates ONE sequence of the batch (the shortest:
the most padding) through every layer.  The bar is the one written for fp16: max |d| / max |ref| <= 1e-2; next to it an
element-wise |d| <= atol + rtol * |ref| check, so that a small element that is badly wrong cannot hide behind the
largest one."""
import numpy as np
import pytest

import encoder_ref
import orc
from test_gpu_ops import rel_err, say, FP16_TOL
from test_gpu_host import r16w, _mods

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

# outputs are LayerNorm results (unit variance, |values| up to ~5); fp16 keeps 11 bits, one rounding is 5e-4 relative
ATOL, RTOL = 1.5e-2, 1e-2


def mixed_violations(got, ref, atol=ATOL, rtol=RTOL):
    d = np.abs(np.asarray(got, np.float64) - ref)
    return int((d > atol + rtol * np.abs(ref)).sum()), float(d.max()), float(np.sqrt((d ** 2).mean()))


def _progress(capsys, text):
    """a line past pytest's capture: these tests spend minutes in the CPU checker and in building gigabyte model files,
    and a run that prints nothing for that long looks hung from outside"""
    if capsys is None:
        print(text, flush=True)
        return
    with capsys.disabled():
        print(text, flush=True)


def _run_full_depth(cfg, w, B, S, lo, hi, seed, precision="fp16", capsys=None):
    host, tnnmodel, _, _, make_inputs = _mods()
    ids, seg, lens, mask = make_inputs(cfg, B, S, lo, hi, seed=seed)
    _progress(capsys, "[depth] writing the model files (%d layers, hidden %d)" % (cfg.layers, cfg.hidden))
    graph = tnnmodel.encoder_graph(cfg, w, B, S)
    _progress(capsys, "[depth] creating the instance")
    inst = host.RocmInstance.from_graph(graph, precision)
    _progress(capsys, "[depth] forward x4")
    inst.set_input("input_ids", ids)
    inst.set_input("token_type_ids", seg)
    inst.set_input("attention_bias", mask.reshape(B, 1, 1, S))
    outs = []
    for _ in range(4):  # eager, eager, the recording pass, a graph replay
        inst.forward()
        outs.append(inst.output("last_hidden", max_elems=1 << 26).reshape(B, S, cfg.hidden))
    inst.close()
    for o in outs[1:]:
        assert np.array_equal(o, outs[0]), "eager / recorded / replayed forwards differ"
    return ids, seg, lens, mask, outs[-1]


def _check_one_sequence(cfg, w, ids, seg, lens, mask, got, S, what, capsys):
    b = int(np.argmin(lens))
    w16 = r16w(w)
    ref = encoder_ref.embed(w16, ids[b:b + 1], seg[b:b + 1], cfg.eps)
    for li, lw in enumerate(w16["layers"]):  # the checker takes seconds per layer: show progress past pytest's capture
        ref = encoder_ref.encoder_layer(ref, lw, 1, S, cfg.heads, mask[b:b + 1], cfg.eps)
        _progress(capsys, "[checker] %s: layer %d of %d" % (what, li + 1, cfg.layers))
    g = got[b].reshape(S, cfg.hidden)
    err = rel_err(g, ref)
    bad, dmax, rms = mixed_violations(g, ref)
    say("  %s: sequence %d (valid %d of %d), %d layers: max rel err %.3g, max |d| %.3g, rms |d| %.3g, "
        "elements outside atol %.3g + rtol %.3g: %d of %d" % (what, b, lens[b], S, cfg.layers, err, dmax, rms, ATOL, RTOL,
                                                                bad, ref.size))
    assert np.isfinite(got).all()
    assert err <= FP16_TOL
    assert bad == 0
    # padded query rows are still produced, as the reference produces them, and must match too (checked above: all S
    # rows of the sequence were compared); valid rows of a LayerNorm(gamma=1, beta=0) output have zero mean
    assert np.abs(g[:lens[b]].mean(-1)).max() < 5e-3


@pytest.mark.timeout(300)
def test_bench_model_12_layers_against_checker(capsys):
    """Exactly the model bench.py times: 12-layer BERT-base, fp16, B8 S384, weights seed 20240601, inputs seed 20240602,
    lengths U[200,384]."""
    _, _, EncoderConfig, make_weights, _ = _mods()
    say("depth: bench.py's model, 12 layers B8 S384 fp16")
    cfg = EncoderConfig.bert_base(12)
    w = make_weights(cfg, seed=20240601)
    ids, seg, lens, mask, got = _run_full_depth(cfg, w, 8, 384, 200, 384, 20240602, capsys=capsys)
    _check_one_sequence(cfg, w, ids, seg, lens, mask, got, 384, "config 2", capsys)


@pytest.mark.timeout(600)
def test_bert_large_24_layers_against_checker(capsys):
    """Config 5 at full depth: 24-layer BERT-large, fp16, B16 S512, lengths U[384,512]."""
    _, _, EncoderConfig, make_weights, _ = _mods()
    say("depth: config 5, 24 layers B16 S512 fp16")
    cfg = EncoderConfig.bert_large(24)
    _progress(capsys, "[depth] drawing the weights of 24 BERT-large layers")
    w = make_weights(cfg, seed=20240605)
    ids, seg, lens, mask, got = _run_full_depth(cfg, w, 16, 512, 384, 512, 20240606, capsys=capsys)
    _check_one_sequence(cfg, w, ids, seg, lens, mask, got, 512, "config 5", capsys)


@pytest.mark.timeout(600)
def test_int8_model_12_layers_properties(monkeypatch, capsys):
    """Config 4 at full depth (12 layers, B16 S256, hidden 768, FFN 3072): calibrated on this backend's fp32 forward,
    run quantised.  Every projection of the first and of the last layer reproduces its own int8 output bit-exactly from
    its own input blob (checker on a 192-row slice; the int32 accumulators behind them are pinned by an integer matmul
    in the checker's own tests), the folded graph agrees with the explicit Reformat chain, and the quantised network
    stays close to the float one."""
    host, tnnmodel, EncoderConfig, make_weights, make_inputs = _mods()
    import golden_util
    from tnn_amd import quant
    say("depth: config 4, 12 layers B16 S256 int8")
    cfg = EncoderConfig.bert_base(12)
    w = make_weights(cfg, seed=20240604)
    B, S = 16, 256
    ids, seg, lens, mask = make_inputs(cfg, B, S, 100, 256, seed=42)
    inputs = {"input_ids": ids, "token_type_ids": seg, "attention_bias": mask.reshape(B, 1, 1, S)}
    names = quant.calibration_outputs(cfg)
    _progress(capsys, "[depth] calibration forward in fp32")
    inst = host.RocmInstance.from_graph(tnnmodel.encoder_graph(cfg, w, B, S, extra_outputs=names), "fp32")
    for k, v in inputs.items():
        inst.set_input(k, v)
    inst.forward()
    scales = {n: quant.activation_scale(inst.output(n, max_elems=1 << 26)) for n in names}
    float_out = inst.output("last_hidden", max_elems=1 << 26)
    inst.close()
    last = cfg.layers - 1
    check = ["x0"] + ["l%d_%s" % (li, b) for li in (0, last) for b in quant.CALIBRATION_BLOBS] + ["l%d_x2" % (last - 1)]
    runs = {}
    for fuse, extra in (("0", check), ("1", [])):
        monkeypatch.setenv("TNN_ROCM_FUSE_INT8", fuse)
        _progress(capsys, "[depth] quantised model, TNN_ROCM_FUSE_INT8=" + fuse)
        inst = host.RocmInstance.from_graph(quant.int8_encoder_graph(cfg, w, scales, B, S, extra_outputs=extra), "fp16")
        for k, v in inputs.items():
            inst.set_input(k, v)
        inst.forward()
        runs[fuse] = inst.output("last_hidden", max_elems=1 << 26)
        if fuse == "0":
            blobs = {n: inst.output(n, max_elems=1 << 26) for n in extra}
        inst.close()
    _progress(capsys, "[depth] checker: twelve projections on 192 rows")
    n = golden_util.check_projections_bit_exact(cfg, w, scales, blobs, B * S, orc.quantize_x86, layers=(0, last), rows=192)
    assert n == 12
    e_fused, e_float = rel_err(runs["1"], runs["0"]), rel_err(runs["1"], float_out)
    say("  folded vs explicit chain %.3g ; quantised vs float network %.3g" % (e_fused, e_float))
    assert e_fused <= 5e-2 and e_float <= 1.5e-1
    valid = (np.arange(S)[None, :] < lens[:, None])
    assert np.isfinite(runs["1"]).all() and np.abs(runs["1"].reshape(B, S, -1)[valid].mean(-1)).max() < 5e-3
