"""Loads the committed fixtures of tests/golden/ (written by tests/golden/make_vectors.py from the reference engine's
own DEVICE_NAIVE / DEVICE_X86 runs) and rebuilds the graphs they belong to."""
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return dict(np.load(os.path.join(GOLDEN, name), allow_pickle=False))


def tiny_encoder():
    """-> (cfg, weights, B, S, fixture dict) of tiny_encoder.npz"""
    from tnn_amd.encoder import EncoderConfig
    f = load("tiny_encoder.npz")
    cfg = EncoderConfig(1, 64, 1, 128, vocab=50, max_pos=32)
    w = {k[2:]: v for k, v in f.items() if k.startswith("w_")}
    w["layers"] = [{k[3:]: v for k, v in f.items() if k.startswith("l0_") and k not in ("l0_probs", "l0_x1")}]
    B, S = f["ids"].shape
    return cfg, w, B, S, f


def config1_inputs():
    """Regenerates the seeded config-1 inputs and checks their digests against the fixture (so a change of the
    generator cannot silently turn the comparison into a different problem)."""
    from tnn_amd.encoder import EncoderConfig, make_weights
    f = load("config1_attention_naive.npz")
    cfg = EncoderConfig(1, 768, 12, 3072)
    lw = make_weights(cfg, seed=1, with_embeddings=False)["layers"][0]
    x = np.random.default_rng(2).standard_normal((128, 768)).astype(np.float32)
    assert float(x.astype(np.float64).sum()) == float(f["x_sum"])
    assert float(np.abs(x).astype(np.float64).sum()) == float(f["x_abs_sum"])
    assert float(lw["wq"].astype(np.float64).sum()) == float(f["wq_sum"])
    assert float(lw["wo"].astype(np.float64).sum()) == float(f["wo_sum"])
    return lw, x, f
