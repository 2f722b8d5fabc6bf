"""Per-blob check of a DEVICE_ROCM instance, and the per-layer profile report.

Role of the engine's tools/model_check (reference tools/model_check/model_checker.cc:658-728: run the model on the device
under test and on the reference device, compare every layer's output blobs, print which layers are out of tolerance) and
of its TNN_PROFILE report (source/tnn/core/profile.cc:111-201).  Two reference sides:
  * `reference=` blob values computed on the CPU by the caller (the engine's DEVICE_NAIVE side of the comparison: the
    test-suite passes the CPU checker's evaluation of the same graph, blob by blob) - check_against();
  * without one, the un-fused fp32 graph on this device (every layer one kernel, every layer output kept) - check(),
    which is what the command line runs, since the shipped package carries no CPU path.
Each row also carries the engine's own pass rule (model_checker.cc:739-752: an element fails when
|d| / (|a| + |b|) > 0.005 and |d| > 1e-3).

    python -m tnn_amd.model_check --layers 2 --batch 2 --seq 128 --precision fp16 [--profile]
"""
import argparse
import copy
import sys

import numpy as np

from . import host


def _with_outputs(graph, outputs):
    g = copy.copy(graph)
    seen, out = set(), []
    for name in list(graph.outputs) + list(outputs):
        if name not in seen:
            seen.add(name)
            out.append(name)
    g.outputs = out
    return g


def _run(inst, inputs):
    for name, arr in inputs.items():
        inst.set_input(name, arr)
    inst.forward()


def check(graph, inputs, precision="fp16", rel_tol=None):
    """Returns (rows, same_layers): rows = [{blob, layer, type, max_abs, rel, cosine, ok}] for every output blob of the
    optimised graph in `precision`; same_layers tells whether keeping those blobs as model outputs left the optimised
    graph unchanged (it should: only blobs that survive the fusion pass are kept)."""
    if rel_tol is None:
        rel_tol = {"fp32": 1e-4, "fp16": 1e-2, "bf16": 4e-2}[precision]
    prod = host.RocmInstance.from_graph(graph, precision)
    prod_types = [t for t, _ in prod.layers()]
    io = prod.layer_io()
    prod.close()
    produced, elems = {}, {}
    for t, layer in zip(prod_types, io):
        for blob, dims in zip(layer["outputs"], layer["output_dims"]):
            produced[blob] = (layer["name"], t)
            elems[blob]    = int(np.prod(dims, dtype=np.int64)) if dims else 1
    all_layer_outputs = [o for (_, _, _, outs, _) in graph.layers for o in outs]
    survivors = [b for b in produced if b in set(all_layer_outputs)]

    chk = host.RocmInstance.from_graph(_with_outputs(graph, survivors), precision)
    same_layers = [t for t, _ in chk.layers()] == prod_types
    ref = host.RocmInstance.from_graph(_with_outputs(graph, all_layer_outputs), "fp32")
    _run(chk, inputs)
    _run(ref, inputs)
    rows = []
    for blob in survivors:
        a = chk.output(blob, max_elems=elems[blob]).astype(np.float64).ravel()
        b = ref.output(blob, max_elems=elems[blob]).astype(np.float64).ravel()
        if a.shape != b.shape:
            rows.append({"blob": blob, "layer": produced[blob][0], "type": produced[blob][1], "max_abs": float("nan"),
                         "rel": float("nan"), "cosine": float("nan"), "ok": False})
            continue
        d = np.abs(a - b)
        scale = np.abs(b).max()
        na, nb = np.linalg.norm(a), np.linalg.norm(b)
        rel = float(d.max() / scale) if scale > 0 else float(d.max())
        rows.append({"blob": blob, "layer": produced[blob][0], "type": produced[blob][1], "max_abs": float(d.max()),
                     "rel": rel, "cosine": float(a @ b / (na * nb)) if na > 0 and nb > 0 else 1.0, "ok": rel <= rel_tol})
    chk.close()
    ref.close()
    return rows, same_layers


def _row(blob, layer, type_str, a, b, rel_tol):
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    if a.shape != b.shape:
        return {"blob": blob, "layer": layer, "type": type_str, "max_abs": float("nan"), "rel": float("nan"),
                "cosine": float("nan"), "engine_rule_failures": -1, "ok": False}
    d = np.abs(a - b)
    scale = np.abs(b).max()
    na, nb = np.linalg.norm(a), np.linalg.norm(b)
    rel = float(d.max() / scale) if scale > 0 else float(d.max())
    with np.errstate(divide="ignore", invalid="ignore"):
        engine_fail = int(((d / (np.abs(a) + np.abs(b)) > 0.005) & (d > 1e-3)).sum())
    return {"blob": blob, "layer": layer, "type": type_str, "max_abs": float(d.max()), "rel": rel,
            "cosine": float(a @ b / (na * nb)) if na > 0 and nb > 0 else 1.0, "engine_rule_failures": engine_fail,
            "ok": rel <= rel_tol}


def check_against(graph, inputs, reference, precision="fp16", rel_tol=None):
    """Device versus CPU, blob by blob (the comparison of model_checker.cc:658-728).  `reference` maps blob names of
    `graph` to their values as the CPU evaluates the graph; every blob that survives the optimiser passes in
    `precision` and has a reference value is kept as a model output of the device instance and compared.
    Returns (rows, same_layers, skipped): skipped = surviving blobs without a reference value."""
    if rel_tol is None:
        rel_tol = {"fp32": 1e-4, "fp16": 1e-2, "bf16": 4e-2}[precision]
    prod = host.RocmInstance.from_graph(graph, precision)
    prod_types = [t for t, _ in prod.layers()]
    io = prod.layer_io()
    prod.close()
    produced, elems = {}, {}
    for t, layer in zip(prod_types, io):
        for blob, dims in zip(layer["outputs"], layer["output_dims"]):
            produced[blob] = (layer["name"], t)
            elems[blob]    = int(np.prod(dims, dtype=np.int64)) if dims else 1
    graph_blobs = {o for (_, _, _, outs, _) in graph.layers for o in outs}
    survivors = [b for b in produced if b in graph_blobs]
    compared = [b for b in survivors if b in reference]
    skipped = [b for b in survivors if b not in reference]
    chk = host.RocmInstance.from_graph(_with_outputs(graph, compared), precision)
    same_layers = [t for t, _ in chk.layers()] == prod_types
    _run(chk, inputs)
    rows = [_row(b, produced[b][0], produced[b][1], chk.output(b, max_elems=elems[b]), reference[b], rel_tol)
            for b in compared]
    chk.close()
    return rows, same_layers, skipped


def report(rows):
    head = "%-28s %-20s %-40s %12s %12s %10s %8s  %s" % ("blob", "Op Type", "layer", "max |diff|", "rel", "cosine",
                                                        "rule", "")
    lines = [head, "-" * len(head)]
    for r in rows:
        rule = r.get("engine_rule_failures")
        lines.append("%-28s %-20s %-40s %12.4g %12.4g %10.6f %8s  %s" % (
            r["blob"][:28], r["type"][:20], r["layer"][:40], r["max_abs"], r["rel"], r["cosine"],
            "-" if rule is None else str(rule), "" if r["ok"] else "OUT OF TOLERANCE"))
    bad = sum(not r["ok"] for r in rows)
    lines.append("%d blobs compared, %d out of tolerance" % (len(rows), bad))
    return "\n".join(lines)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--layers", type=int, default=2)
    ap.add_argument("--batch", type=int, default=2)
    ap.add_argument("--seq", type=int, default=128)
    ap.add_argument("--hidden", type=int, default=768)
    ap.add_argument("--heads", type=int, default=12)
    ap.add_argument("--ffn", type=int, default=3072)
    ap.add_argument("--precision", default="fp16", choices=["fp32", "fp16", "bf16"])
    ap.add_argument("--profile", action="store_true", help="also print the per-layer profile report")
    args = ap.parse_args(argv)
    from . import tnnmodel
    from .encoder import EncoderConfig, make_weights, make_inputs
    host.load()
    cfg = EncoderConfig(args.layers, args.hidden, args.heads, args.ffn)
    w = make_weights(cfg, seed=1, bias_std=0.02)
    ids, seg, lens, mask = make_inputs(cfg, args.batch, args.seq, max(1, args.seq // 2), args.seq, seed=2)
    graph = tnnmodel.encoder_graph(cfg, w, args.batch, args.seq)
    inputs = {"input_ids": ids, "token_type_ids": seg, "attention_bias": mask.reshape(args.batch, 1, 1, args.seq)}
    rows, same = check(graph, inputs, args.precision)
    print(report(rows))
    if not same:
        print("note: keeping the checked blobs as model outputs changed the optimised graph")
    if args.profile:
        inst = host.RocmInstance.from_graph(graph, args.precision)
        for name, arr in inputs.items():
            inst.set_input(name, arr)
        for _ in range(3):
            inst.forward()
        print(inst.profile_table(10))
        inst.close()
    return 0 if all(r["ok"] for r in rows) else 1


if __name__ == "__main__":
    sys.exit(main())
