"""Achieved HBM bandwidth of the memory-bound kernels of the encoder path, each against the MI355X peak (8 TB/s).

    python -m tnn_amd.bench_ops [--launches 20] [--only layernorm,softmax] [--json]

Every kernel is timed at two sizes:

  encoder   the shape it has inside a BERT-base forward at batch 8, sequence 384 (3072 token rows; hidden 768,
            FFN 3072, 96 x 384 x 384 scores): a few MB, served by the caches and bounded by launch latency
  stream    the same row shape over 196608 rows: inputs + outputs are at least 0.6 GB, more than twice the 256 MB
            memory-side cache, so the rate is what HBM delivers

Bytes are the algorithmic ones: every input and every output once.  A case is `launches` launches captured into one
graph (so the gaps between launches are the device's, not Python's) and replayed between two events on the launch
stream; the best of five replays counts.  All launches go through the C entry points of libtnn_rocm.so (tnn_amd.ops
passes raw device pointers); there is no other implementation behind them."""
import argparse
import json
import os
import sys

import torch

from . import capi, ops

PEAK_GBS = 8000.0
ROWS_ENC = 3072
H, F, HEADS, S = 768, 3072, 12, 384


def _time_us(fn, launches):
    fn()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for _ in range(launches):
            fn()
    g.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best = float("inf")
    for _ in range(5):
        e0.record()
        g.replay()
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1) * 1e3 / launches)
    del g
    return best


def _randn(shape, dtype):
    # filled in slices: a 1 GiB fp32 staging tensor for a half-precision operand is not needed
    t = torch.empty(shape, dtype=dtype, device="cuda")
    flat = t.view(-1)
    step = 1 << 26
    for i in range(0, flat.numel(), step):
        n = min(step, flat.numel() - i)
        flat[i:i + n] = torch.randn(n, device="cuda", dtype=torch.float32).to(dtype)
    return t


def _randi8(shape):
    return torch.randint(-127, 128, shape, dtype=torch.int8, device="cuda")


def cases(rows):
    """(name, bytes, callable) for `rows` token rows; softmax and permute scale their leading dimension instead"""
    f16, f32 = torch.float16, torch.float32
    out = []
    gamma, beta = torch.ones(H, device="cuda"), torch.zeros(H, device="cuda")

    # yardstick: what a plain device-to-device copy of the same footprint reaches on this box
    src = _randn((rows, F), f16)
    dst = torch.empty_like(src)
    out.append(("device copy (yardstick) [T,3072] f16", 2 * src.numel() * 2,
                lambda: capi.call("tnn_rocm_memcpy_d2d", dst.data_ptr(), src.data_ptr(), src.numel() * 2,
                                  torch.cuda.current_stream().cuda_stream)))

    for dtype, tag in ((f16, "f16"), (f32, "f32")):
        es = 2 if dtype == f16 else 4
        x, r = _randn((rows, H), dtype), _randn((rows, H), dtype)
        out.append(("layernorm %s [T,768]" % tag, 2 * rows * H * es, lambda x=x: ops.layernorm(x, gamma, beta, 1e-12)))
        out.append(("layernorm+residual %s [T,768]" % tag, 3 * rows * H * es,
                    lambda x=x, r=r: ops.layernorm(x, gamma, beta, 1e-12, residual=r)))
        if dtype == f16:
            out.append(("layernorm+residual f16 -> f16 + int8 [T,768]", rows * H * (3 * es + 1),
                        lambda x=x, r=r: ops.layernorm(x, gamma, beta, 1e-12, residual=r, q_inv_scale=20.0)))
        out.append(("add %s [T,768] + [T,768]" % tag, 3 * rows * H * es, lambda x=x, r=r: ops.binary("add", x, r)))
        b = _randn((H,), dtype)
        out.append(("add %s [T,768] + [768] (bias)" % tag, 2 * rows * H * es, lambda x=x, b=b: ops.binary("add", x, b)))
        hbuf = _randn((rows, F), dtype)
        out.append(("gelu %s [T,3072]" % tag, 2 * rows * F * es, lambda hbuf=hbuf: ops.gelu(hbuf)))
        if dtype == f32:
            out.append(("cast f32 -> f16 [T,3072]", rows * F * 6, lambda hbuf=hbuf: ops.cast(hbuf, f16)))
        else:
            out.append(("quantize f16 -> int8 [T,3072]", rows * F * 3, lambda hbuf=hbuf: ops.quantize(hbuf, 20.0)))

    q = _randi8((rows, F))
    q2 = _randi8((rows, F))
    out.append(("dequantize int8 -> f16 [T,3072]", rows * F * 3, lambda: ops.dequantize(q, 0.05, f16)))
    out.append(("add int8 [T,3072]", rows * F * 3, lambda: ops.add_i8(q, 0.05, q2, 0.04, 12.0)))
    out.append(("gelu int8 (table) [T,3072]", rows * F * 2, lambda: ops.gelu_i8(q, 0.05, 20.0)))

    # scores of the un-fused fp32 attention core: [B*h, S, S], softmax over the last axis
    bh = max(1, rows * 96 // ROWS_ENC)
    sc = _randn((bh, S, S), f32)
    out.append(("softmax f32 [B*h,384,384] last axis", 2 * bh * S * S * 4, lambda: ops.softmax(sc, -1)))
    # head split / merge of the un-fused path: [S,h,d] -> [h,S,d] per sequence, here [B,S,h,d] -> [B,h,S,d]
    nb = max(1, rows // S)
    px = _randn((nb, S, HEADS, 64), f32)
    out.append(("permute f32 [B,S,h,d] -> [B,h,S,d]", 2 * px.numel() * 4, lambda: ops.permute(px, (0, 2, 1, 3))))
    out.append(("permute f32 [B,S,h,d] -> [B,h,d,S] (K^T)", 2 * px.numel() * 4, lambda: ops.permute(px, (0, 2, 3, 1))))

    # embedding front end: word rows gathered (2 B/elem in, 2 B/elem out), position and type tables stay in cache
    word, typ, pos = _randn((30522, H), f16), _randn((2, H), f16), _randn((512, H), f16)
    ids = torch.randint(0, 30522, (rows // S if rows >= S else 1, S), dtype=torch.int32, device="cuda")
    tt = torch.zeros_like(ids)
    out.append(("embedding (2 gathers + position + LayerNorm) f16", 2 * ids.numel() * H * 2 + ids.numel() * 8,
                lambda: ops.embed_layernorm(ids, tt, word, typ, pos, gamma, beta, 1e-12)))
    out.append(("gather f16 rows of [30522,768]", 2 * ids.numel() * H * 2 + ids.numel() * 4,
                lambda: ops.gather(word, ids.view(-1), 0)))
    return out


def run(launches, only=None, sizes=("encoder", "stream"), report=None):
    capi.load()
    assert torch.cuda.is_available(), "needs a GPU"
    results = []
    for size in sizes:
        # stream: 0.6 GB of traffic for the smallest case (fp16 LayerNorm: 2 x rows x 768 x 2 B), 2.4 GB tensors at most
        rows = ROWS_ENC if size == "encoder" else 192 * 1024
        n = launches if size == "encoder" else max(3, launches // 4)
        for name, nbytes, fn in cases(rows):
            if only and not any(o in name for o in only):
                continue
            us = _time_us(fn, n)
            gbs = nbytes / us / 1e3
            results.append({"kernel": name, "size": size, "rows": rows, "bytes": nbytes, "us_per_launch": round(us, 2),
                            "GB_per_s": round(gbs, 1), "frac_of_hbm_peak": round(gbs / PEAK_GBS, 4)})
            if report:
                report(results[-1])
        torch.cuda.empty_cache()
    return results


def mall_probe(launches=20):
    """Does the memory-side cache (256 MB, shared by the eight XCDs) serve the panel re-reads of the projection GEMMs?
    No counter visible from the GPU separates its hits from HBM accesses, so this times each GEMM of the batch-8 /
    seq-384 encoder twice with an event pair around the single launch: once with its operands as a previous launch
    left them (resident in that cache, like the activations a layer has just written), once right after a 1 GiB device
    copy that evicts them (every first touch then goes to HBM).  A spinning kernel in front of both keeps the queue
    filled, so the host's launch latency is in neither figure.  The difference is what HBM-side re-reads cost."""
    capi.load()
    T, H, F = ROWS_ENC, 768, 3072
    f16 = torch.float16
    shapes = {"qkv (M3072 N2304 K768)": (T, 3 * H, H), "out (M3072 N768 K768)": (T, H, H),
              "ffn1 (M3072 N3072 K768)": (T, F, H), "ffn2 (M3072 N768 K3072)": (T, H, F)}
    big_a = torch.empty(1 << 28, dtype=torch.float32, device="cuda")
    big_b = torch.empty(1 << 28, dtype=torch.float32, device="cuda")
    rows = []
    for name, (M, N, K) in shapes.items():
        a, w = _randn((M, K), f16), _randn((N, K), f16) * 0.02
        bias = torch.zeros(N, device="cuda")
        res = _randn((M, N), f16)
        out = torch.empty(M, N, dtype=f16, device="cuda")
        fn = lambda: ops.gemm(a, w, True, bias=bias, residual=res, out=out)
        for _ in range(3):
            fn()
        t = {}
        for mode in ("resident", "evicted"):
            tot = 0.0
            for _ in range(launches):
                if mode == "evicted":
                    big_b.copy_(big_a)
                torch.cuda._sleep(400000)  # ~0.2 ms without memory traffic: the launches below are queued behind it
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                fn()
                e1.record()
                torch.cuda.synchronize()
                tot += e0.elapsed_time(e1)
            t[mode] = tot / launches * 1e3
        rows.append({"gemm": name, "us_resident": round(t["resident"], 2), "us_evicted": round(t["evicted"], 2),
                     "operand_MiB": round((M * K + N * K + 2 * M * N) * 2 / 2**20, 1)})
    return rows


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--mall-probe", action="store_true", help="projection GEMMs with resident / evicted operands")
    ap.add_argument("--simd-probe", action="store_true",
                    help="build (if missing) and run the stand-alone SIMD micro-benchmark csrc/probe_simd.hip")
    ap.add_argument("--build-only", action="store_true", help="with --simd-probe: compile it, do not run it")
    ap.add_argument("--launches", type=int, default=20)
    ap.add_argument("--only", default="")
    ap.add_argument("--sizes", default="encoder,stream")
    ap.add_argument("--json", action="store_true")
    a = ap.parse_args()
    if a.simd_probe:
        import subprocess
        from tnn_amd import build
        exe = os.path.join(build.LIB_DIR, "probe_simd")
        if a.build_only or not os.path.exists(exe):
            build.build_simd_probe()
        if not a.build_only:
            sys.exit(subprocess.call([exe]))
        return
    if a.mall_probe:
        for r in mall_probe(a.launches):
            print(json.dumps(r) if a.json else "%-28s operands %6.1f MiB   resident %7.2f us   evicted %7.2f us" % (
                r["gemm"], r["operand_MiB"], r["us_resident"], r["us_evicted"]), flush=True)
        return
    def line(r):
        if a.json:
            print(json.dumps(r), flush=True)
        else:
            print("%-52s %-8s %12.1f %10.2f %10.1f %7.1f%%" % (r["kernel"], r["size"], r["bytes"] / 2**20,
                                                              r["us_per_launch"], r["GB_per_s"],
                                                              100 * r["frac_of_hbm_peak"]), flush=True)

    if not a.json:
        print("%-52s %-8s %12s %10s %10s %8s" % ("kernel", "size", "MiB", "us", "GB/s", "of peak"), flush=True)
    run(a.launches, [s for s in a.only.split(",") if s], tuple(a.sizes.split(",")), report=line)


if __name__ == "__main__":
    main()
