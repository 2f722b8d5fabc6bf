"""The attention rewrite against graphs its authors did not write: every spelling of the attention core the matcher
claims to accept, and every look-alike it must leave decomposed, runs through Instance::Forward on DEVICE_ROCM in fp16
and is compared with the same op sequence evaluated by the CPU checker.  A silent mis-fusion (a softmax over the wrong
axis, a per-query mask treated as a per-key one) shows here as a wrong result; a refused graph that no longer
initialises shows as an error."""
import numpy as np
import pytest

import orc
from test_gpu_ops import rel_err, say, FP16_TOL
from test_host_plan import ACCEPTED_SPELLINGS, REFUSED_SPELLINGS

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def _r16(a):
    return a.astype(np.float16).astype(np.float32)


def reference(lw, x, mask, B, S, H, heads, scale="mul", mask_first=False, proj="matmul", rank3=False, softmax_axis=None,
              tap_scores=False, **_):
    """the graph of tnnmodel.attention_block_graph, op by op, on the CPU checker (fp32 on fp16-rounded weights)"""
    d = H // heads
    x2 = x.reshape(B * S, H)
    lin = lambda t, w, b: orc.inner_product(t, _r16(lw[w]), lw[b])
    q, k, v = (lin(x2, "w" + n, "b" + n) for n in "qkv")
    if rank3:
        q, k, v = (t.reshape(S, heads, d) for t in (q, k, v))
        qh, kt, vh = orc.permute(q, (1, 0, 2)), orc.permute(k, (1, 2, 0)), orc.permute(v, (1, 0, 2))
    else:
        q, k, v = (t.reshape(B, S, heads, d) for t in (q, k, v))
        qh, kt, vh = orc.permute(q, (0, 2, 1, 3)), orc.permute(k, (0, 2, 3, 1)), orc.permute(v, (0, 2, 1, 3))
    if scale in ("q", "qk"):
        f = np.array([d ** -0.5 if scale == "q" else d ** -0.25], np.float32)
        qh = orc.binary("mul", qh, f)
        if scale == "qk":
            kt = orc.binary("mul", kt, f)
    s = orc.matmul(qh, kt)
    if scale == "mul":
        s = orc.binary("mul", s, np.array([1.0 / np.sqrt(d)], np.float32))
    elif scale == "div":
        s = orc.binary("div", s, np.array([np.sqrt(d)], np.float32))
    if mask is not None:
        s = orc.binary("add", mask, s) if mask_first else orc.binary("add", s, mask)
    rank = 3 if rank3 else 4
    p = orc.softmax(s, (rank - 1) if softmax_axis is None else softmax_axis)
    c = orc.matmul(p, vh)
    c = orc.permute(c, (1, 0, 2) if rank3 else (0, 2, 1, 3)).reshape(B * S, H)
    y = lin(c, "wo", "bo")
    return y if (rank3 or proj == "inner_product") else y.reshape(B, S, H)   # the head-merging Reshape's dims


def _run(name, spelling, fused):
    from tnn_amd import host, tnnmodel
    from tnn_amd.encoder import EncoderConfig, make_weights
    sp = dict(spelling)
    B, S, H, heads = sp.pop("B", 3), 72, 256, sp.pop("heads", 4)
    say("spelling %s: %s" % (name, spelling))
    cfg = EncoderConfig(1, H, heads, 2 * H)
    lw = make_weights(cfg, seed=3, bias_std=0.02)["layers"][0]
    g = tnnmodel.attention_block_graph(lw, B, S, H, heads, **sp)
    rng = np.random.default_rng(17)
    flat = sp.get("proj") == "inner_product"
    x = _r16(rng.standard_normal((B * S, H) if flat else (B, S, H)).astype(np.float32))
    kind = sp.get("mask", "b11s")
    mask = None
    if kind is not None:
        shape = {"b11s": (B, 1, 1, S), "111s": (1, 1, 1, S), "b1ss": (B, 1, S, S), "11s": (1, 1, S), "1ss": (1, S, S)}[kind]
        mask = np.zeros(shape, np.float32)
        if kind in ("b1ss", "1ss"):          # causal: a different key set for every query
            mask[...] = np.triu(np.full((S, S), -10000.0, np.float32), 1)
        else:                                # padding: the tail of every sequence
            for b in range(shape[0]):
                mask[b, ..., S - 5 - 11 * b:] = -10000.0
    inst = host.RocmInstance.from_graph(g, "fp16")
    types = [t for t, _ in inst.layers()]
    assert ("RocmFusedAttention" in types) == fused, types
    if not fused:
        assert types.count("Softmax") == 1 and types.count("MatMul") == 2
    inst.set_input("hidden", x)
    if mask is not None:
        inst.set_input("attention_bias", mask)
    inst.forward()
    got = inst.output("y")
    inst.close()
    ref = reference(lw, x, mask, B, S, H, heads, **{k: v for k, v in sp.items() if k != "mask"})
    err = rel_err(got, ref)
    say("  fused %s, max rel err %.3g" % (fused, err))
    assert got.shape == ref.shape and err <= FP16_TOL, (name, err)


@pytest.mark.parametrize("name", sorted(ACCEPTED_SPELLINGS))
def test_accepted_spelling_matches_the_checker(name):
    _run(name, ACCEPTED_SPELLINGS[name], True)


@pytest.mark.parametrize("name", sorted(REFUSED_SPELLINGS))
def test_refused_lookalike_runs_decomposed_and_matches_the_checker(name):
    _run(name, REFUSED_SPELLINGS[name], False)
