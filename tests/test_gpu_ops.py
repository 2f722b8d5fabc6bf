"""GPU parity tests: every C-ABI entry point against the CPU checker on the same seeded inputs.

Tolerances (stated per assertion):
  fp32  : max|d| / max|ref| <= 2e-3   (most ops are asserted far tighter)
  fp16  : max|d| / max|ref| <= 1e-2, reference computed in fp32 on the fp16-rounded inputs
  int8 / int32 / index work: bit-exact
"""
import sys

import numpy as np
import pytest

import golden_util
import orc

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

FP32_TOL = 2e-3      # the bar stated for fp32 against the reference's CPU paths
FP32_ASSERT = 5e-5   # what the fp32 cases assert: true-fp32 MFMA products, fp32 accumulation (observed <= 1e-5)
FP16_TOL = 1e-2
BF16_TOL = 4e-2


def say(msg):
    print("[case] " + msg, flush=True)
    sys.stdout.flush()


def ops():
    from tnn_amd import ops as o
    return o


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    return t if dtype is None else t.to(dtype)


def host(t):
    torch.cuda.synchronize()
    return t.float().cpu().numpy() if t.dtype in (torch.float16, torch.bfloat16) else t.cpu().numpy()


def rel_err(got, ref):
    ref = np.asarray(ref, np.float64)
    got = np.asarray(got, np.float64)
    return float(np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-30))


def r16(a):
    """round to fp16 and back: the values an fp16 kernel actually sees"""
    return np.asarray(a, np.float32).astype(np.float16).astype(np.float32)


# ---------------------------------------------------------------------------------------------
def test_library_loads_on_gpu():
    from tnn_amd import capi
    import ctypes as C
    n = C.c_int(0)
    capi.call("tnn_rocm_device_count", C.byref(n))
    assert n.value >= 1
    buf = C.create_string_buffer(256)
    capi.call("tnn_rocm_device_name", 0, buf, 256)
    say("device: " + buf.value.decode())
    assert b"gfx950" in buf.value


@pytest.mark.parametrize("n", [1, 7, 4096, 128 * 3072 + 3])
def test_gelu_fp32(n):
    say("gelu fp32 n=%d" % n)
    rng = np.random.default_rng(n)
    x = (rng.standard_normal(n) * 3).astype(np.float32)
    x[:1] = -2.281006575  # the point where the tanh form is visibly wrong
    got = host(ops().gelu(dev(x)))
    ref = orc.gelu(x)
    # the device evaluates the reference's expression (fp32 products, double erf, one rounding to fp32): the only room
    # left is a last-bit difference between two double erf routines surviving that rounding
    assert (got != ref).mean() <= 1e-5 and rel_err(got, ref) <= 2e-7
    # special values
    sp = np.array([0.0, -0.0, np.inf, -40.0, 40.0], np.float32)
    got = host(ops().gelu(dev(sp)))
    assert got[0] == 0 and got[1] == 0 and got[2] == np.inf and got[3] == 0 and got[4] == 40.0


def test_tanh():
    say("tanh")
    x = np.concatenate([np.linspace(-12, 12, 4001), [0.0, 1e-8, -1e-8, 50.0, -50.0]]).astype(np.float32)
    ref = np.tanh(x.astype(np.float64))
    got = host(ops().tanh(dev(x)))
    assert np.max(np.abs(got - ref)) <= 3e-7
    got16 = host(ops().tanh(dev(x, torch.float16)))
    ref16 = np.tanh(x.astype(np.float16).astype(np.float64))
    assert np.max(np.abs(got16 - ref16)) <= 1e-3


def test_gelu_fp16():
    say("gelu fp16")
    rng = np.random.default_rng(1)
    x = r16(rng.standard_normal(10001) * 3)
    got = host(ops().gelu(dev(x, torch.float16)))
    assert rel_err(got, orc.gelu(x)) <= 1e-3  # one fp16 rounding of the result
    sp = np.array([0.0, np.inf, 40.0, -40.0, 65504.0, -65504.0], np.float32)
    got = host(ops().gelu(dev(sp, torch.float16)))
    assert got.tolist() == [0.0, np.inf, 40.0, 0.0, 65504.0, 0.0]
    # a NaN stays a NaN (an overflow upstream must not turn into zeros), in every float type and in the GEMM epilogue
    for td in (torch.float32, torch.float16, torch.bfloat16):
        got = host(ops().gelu(dev(np.array([np.nan, 1.0, -np.inf], np.float32), td)))
        assert np.isnan(got[0]) and abs(got[1] - 0.8413) < 5e-3 and np.isnan(got[2]), (td, got)
    a = torch.zeros(64, 64, dtype=torch.float16, device="cuda")
    a[3, 5] = float("nan")
    w = torch.eye(64, dtype=torch.float16, device="cuda")
    y = host(ops().gemm(a, w, True, bias=torch.zeros(64, device="cuda"), gelu=True))
    assert np.isnan(y[3]).any() and not np.isnan(np.delete(y, 3, axis=0)).any()


@pytest.mark.parametrize("rows,cols", [(1, 8), (5, 768), (33, 1024), (7, 100), (3, 5000), (4096, 768)])
def test_layernorm_fp32(rows, cols):
    say("layernorm fp32 %dx%d" % (rows, cols))
    rng = np.random.default_rng(rows * 131 + cols)
    x = (rng.standard_normal((rows, cols)) * 2 + 0.5).astype(np.float32)
    g = rng.standard_normal(cols).astype(np.float32)
    b = rng.standard_normal(cols).astype(np.float32)
    for eps in (1e-5, 1e-12):
        got = host(ops().layernorm(dev(x), dev(g), dev(b), eps))
        ref = orc.layernorm(x, g, b, eps)
        assert rel_err(got, ref) <= 2e-6, (rows, cols, eps)


def test_layernorm_large_mean_fp32():
    # a large common offset makes E[x^2]-E[x]^2 cancel; the double-precision statistics must cope
    say("layernorm fp32 large mean")
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((16, 768)) + 100.0).astype(np.float32)
    g = np.ones(768, np.float32)
    b = np.zeros(768, np.float32)
    got = host(ops().layernorm(dev(x), dev(g), dev(b), 1e-5))
    assert rel_err(got, orc.layernorm(x, g, b, 1e-5)) <= 1e-4


def test_layernorm_residual_and_quant():
    say("layernorm fp32 residual + fused quantise")
    rng = np.random.default_rng(6)
    x = rng.standard_normal((64, 768)).astype(np.float32)
    r = rng.standard_normal((64, 768)).astype(np.float32)
    g = rng.standard_normal(768).astype(np.float32)
    b = rng.standard_normal(768).astype(np.float32)
    scale = np.float32(0.031)
    inv = np.float32(1.0 / np.float64(scale))
    y, q = ops().layernorm(dev(x), dev(g), dev(b), 1e-5, residual=dev(r), q_inv_scale=float(inv))
    ref = orc.layernorm(orc.binary("add", x, r), g, b, 1e-5)
    y = host(y)
    assert rel_err(y, ref) <= 2e-6
    # the quantised copy must be exactly the quantisation of the y the kernel stored
    assert np.array_equal(host(q), orc.quantize_x86(y, scale))


def test_layernorm_fp16():
    say("layernorm fp16")
    rng = np.random.default_rng(7)
    x = r16(rng.standard_normal((384, 768)))
    r = r16(rng.standard_normal((384, 768)))
    g = np.ones(768, np.float32)
    b = np.zeros(768, np.float32)
    got = host(ops().layernorm(dev(x, torch.float16), dev(g), dev(b), 1e-12, residual=dev(r, torch.float16)))
    ref = orc.layernorm(x + r, g, b, 1e-12)
    assert rel_err(got, ref) <= 2e-3
    # gamma=1, beta=0: rows have mean 0 and variance 1
    assert abs(got.mean(-1)).max() < 2e-3 and abs(got.var(-1) - 1).max() < 5e-3


def test_layernorm_rejects_empty():
    from tnn_amd import capi
    o = ops()
    x = torch.zeros(4, device="cuda")
    with pytest.raises(capi.TnnRocmError):
        capi.call("tnn_rocm_layernorm", None, 0, x.data_ptr(), None, x.data_ptr(), x.data_ptr(), x.data_ptr(), 0, 4,
                  1e-5, None, 0.0)
    assert o is not None


@pytest.mark.parametrize("shape,axis", [((4, 16), -1), ((3, 5, 7), 1), ((2, 12, 33, 33), -1), ((2, 3, 4, 5, 6), 2),
                                        ((8, 512), 1), ((3, 2000), 1), ((6, 1, 9), 0)])
def test_softmax_fp32(shape, axis):
    say("softmax fp32 %s axis=%d" % (shape, axis))
    rng = np.random.default_rng(sum(shape) + axis)
    x = (rng.standard_normal(shape) * 4).astype(np.float32)
    got = host(ops().softmax(dev(x), axis))
    ref = orc.softmax(x, axis)
    # the reference adds the exponentials sequentially in fp32; a tree sum differs by a few ulp
    assert rel_err(got, ref) <= 1e-5
    assert np.abs(got.sum(axis) - 1).max() <= 1e-5


def test_softmax_masked_columns_are_exact_zero():
    say("softmax -inf columns")
    rng = np.random.default_rng(3)
    x = rng.standard_normal((8, 64)).astype(np.float32)
    x[:, 40:] = -np.inf
    got = host(ops().softmax(dev(x), -1))
    assert np.all(got[:, 40:] == 0)
    assert rel_err(got, orc.softmax(x, -1)) <= 1e-6


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
@pytest.mark.parametrize("sa,sb", [((4, 8, 16), (16,)), ((4, 8, 16), (4, 8, 16)), ((4, 8, 16), (1,)),
                                   ((2, 12, 33, 33), (2, 1, 1, 33)), ((5, 1, 7), (1, 6, 7)), ((3, 4), (4, 3, 4)),
                                   ((1024, 768), (768,))])
def test_binary_fp32(op, sa, sb):
    say("binary %s %s %s" % (op, sa, sb))
    rng = np.random.default_rng(len(sa) * 7 + len(sb))
    a = rng.standard_normal(sa).astype(np.float32)
    b = (rng.standard_normal(sb) + 3).astype(np.float32)
    got = host(ops().binary(op, dev(a), dev(b)))
    ref = orc.binary(op, a, b)
    assert got.shape == ref.shape
    assert np.array_equal(got, ref)  # single IEEE operations: bit-exact


def test_binary_fp16():
    say("binary fp16 add bias")
    rng = np.random.default_rng(9)
    a = r16(rng.standard_normal((96, 768)))
    b = r16(rng.standard_normal(768))
    got = host(ops().binary("add", dev(a, torch.float16), dev(b, torch.float16)))
    assert np.array_equal(got, r16(a + b))


@pytest.mark.parametrize("shape,order", [((128, 12, 64), (1, 0, 2)), ((128, 12, 64), (1, 2, 0)),
                                         ((2, 16, 12, 64), (0, 2, 1, 3)), ((3, 4, 5, 6, 7), (4, 0, 3, 1, 2)),
                                         ((9,), (0,))])
def test_permute(shape, order):
    say("permute %s %s" % (shape, order))
    rng = np.random.default_rng(len(shape))
    x = rng.standard_normal(shape).astype(np.float32)
    got = host(ops().permute(dev(x), order))
    ref = orc.permute(x, order)
    assert np.array_equal(got, ref) and np.array_equal(ref, np.transpose(x, order))
    x8 = rng.integers(-128, 128, shape, dtype=np.int8)
    assert np.array_equal(host(ops().permute(dev(x8), order)), np.transpose(x8, order))
    x16 = x.astype(np.float16)
    assert np.array_equal(ops().permute(dev(x16), order).cpu().numpy(), np.transpose(x16, order))


def test_gather_embedding():
    say("gather")
    rng = np.random.default_rng(11)
    table = rng.standard_normal((30522, 96)).astype(np.float32)
    idx = rng.integers(0, 30522, (4, 37)).astype(np.int32)
    idx[0, 0] = -1  # wraps to the last row
    got, flag = ops().gather(dev(table), dev(idx), 0)
    ref, rc = orc.gather(table, idx, 0)
    assert rc == 0 and int(flag.item()) == 0
    assert np.array_equal(host(got), ref)
    # out-of-range index: reference reports an error; the kernel raises its flag
    idx[1, 1] = 30522
    got, flag = ops().gather(dev(table), dev(idx), 0)
    assert orc.gather(table, idx, 0)[1] != 0 and int(flag.item()) == 1
    # odd slice size (3 bytes) and a batch axis
    t8 = rng.integers(-128, 128, (3, 50, 3), dtype=np.int8)
    i2 = rng.integers(0, 50, (11,)).astype(np.int32)
    got, flag = ops().gather(dev(t8), dev(i2), 1)
    assert np.array_equal(host(got), orc.gather(t8, i2, 1)[0])


def test_cast_roundtrip():
    say("cast")
    rng = np.random.default_rng(12)
    x = (rng.standard_normal(100003) * 100).astype(np.float32)
    h = ops().cast(dev(x), torch.float16)
    assert np.array_equal(h.cpu().numpy(), x.astype(np.float16))
    assert np.array_equal(host(ops().cast(h, torch.float32)), x.astype(np.float16).astype(np.float32))
    bf = ops().cast(dev(x), torch.bfloat16)
    assert torch.equal(bf.cpu(), torch.from_numpy(x).to(torch.bfloat16))


def test_cast_int32():
    # cpu_cast_layer_acc.cc:41-53: static_cast both ways
    say("cast int32 <-> float types")
    rng = np.random.default_rng(13)
    i = rng.integers(-70000, 70000, 10007).astype(np.int32)
    i[:4] = [0, 1, -1, 30521]
    assert np.array_equal(host(ops().cast(dev(i), torch.float32)), i.astype(np.float32))
    assert torch.equal(ops().cast(dev(i), torch.float16).cpu(), torch.from_numpy(i).to(torch.float16))
    assert torch.equal(ops().cast(dev(i), torch.bfloat16).cpu(), torch.from_numpy(i).to(torch.bfloat16))
    f = (rng.standard_normal(10007) * 1000).astype(np.float32)
    f[:6] = [0.0, 0.99, -0.99, 1.5, -1.5, 2.0]
    assert np.array_equal(ops().cast(dev(f), torch.int32).cpu().numpy(), f.astype(np.int32))   # truncation
    h = torch.from_numpy(f).to(torch.float16)
    assert np.array_equal(ops().cast(h.cuda(), torch.int32).cpu().numpy(), h.float().numpy().astype(np.int32))


# ---- int8 boundary ops: bit-exact ---------------------------------------------------------------
def _half_integer_grid(scale):
    """values whose scaled image sits on and next to every .5 boundary of the int8 range"""
    k = np.arange(-130, 131, dtype=np.float64) + 0.5
    base = (k * np.float64(scale)).astype(np.float32)
    out = [base]
    for _ in range(3):
        out.append(np.nextafter(out[-1], np.float32(np.inf)))
    lo = base
    for _ in range(3):
        lo = np.nextafter(lo, np.float32(-np.inf))
        out.append(lo)
    return np.concatenate(out).astype(np.float32)


@pytest.mark.parametrize("scale", [0.05, 0.0123, 1.0, 3.7e-3])
def test_quantize_bit_exact(scale):
    say("quantize scale=%g" % scale)
    rng = np.random.default_rng(13)
    scale = np.float32(scale)
    inv = np.float32(1.0 / np.float64(scale))
    x = np.concatenate([_half_integer_grid(scale), (rng.standard_normal(200001) * 40 * scale).astype(np.float32),
                        np.array([0.0, -0.0, 1e30, -1e30], np.float32)])
    got = host(ops().quantize(dev(x), float(inv)))
    assert np.array_equal(got, orc.quantize_x86(x, scale))
    # values no sane activation holds, pinned so that a change shows: infinities saturate, a NaN becomes -128 (what the
    # reference's x86 quantiser makes of it: INT_MIN out of the truncating conversion, then the saturating pack)
    got = host(ops().quantize(dev(np.array([np.inf, -np.inf, np.nan], np.float32)), float(inv)))
    assert got.tolist() == [127, -128, -128]


def test_dequantize_and_add_i8_bit_exact():
    say("dequantize / add_i8")
    rng = np.random.default_rng(14)
    q = rng.integers(-128, 128, 100001, dtype=np.int8)
    assert np.array_equal(host(ops().dequantize(dev(q), 0.0371)), orc.dequantize(q, np.float32(0.0371)))
    a = rng.integers(-128, 128, 100001, dtype=np.int8)
    sa, sb, so = np.float32(0.021), np.float32(0.047), np.float32(0.052)
    inv = np.float32(1.0 / np.float64(so))
    got = host(ops().add_i8(dev(a), float(sa), dev(q), float(sb), float(inv)))
    assert np.array_equal(got, orc.add_int8_x86(a, sa, q, sb, so))


@pytest.mark.parametrize("dims", [(2, 10, 9, 9), (1, 32, 19, 19), (3, 4, 16), (5, 7)])
def test_quantize_and_dequantize_with_one_scale_per_channel(dims):
    """Blob scales with one entry per channel (axis 1), as the reference's int8 unit tests generate them and its Reformat
    kernels take them (x86_compute_int8.cc:1193-1318): every channel's slice equals the per-tensor routine of the
    checker with that channel's scale, bit for bit."""
    say("per-channel quantize / dequantize %s" % (dims,))
    rng = np.random.default_rng(sum(dims))
    C = dims[1]
    scales = rng.uniform(0.01, 1.0, size=C).astype(np.float32)
    inv = (1.0 / scales.astype(np.float64)).astype(np.float32)
    x = (rng.standard_normal(dims) * 20).astype(np.float32) * scales.reshape((1, C) + (1,) * (len(dims) - 2))
    x.reshape(-1)[:: 7] = (np.round(x.reshape(-1)[:: 7] / 0.5) * 0.5).astype(np.float32)
    q = host(ops().quantize_per_channel(dev(x), dev(inv)))
    back = host(ops().dequantize_per_channel(dev(q), dev(scales)))
    for c in range(C):
        sl = (slice(None), c)
        assert np.array_equal(q[sl], orc.quantize_x86(np.ascontiguousarray(x[sl]).reshape(-1), scales[c]).reshape(q[sl].shape)), c
        assert np.array_equal(back[sl], orc.dequantize(np.ascontiguousarray(q[sl]).reshape(-1), scales[c]).reshape(q[sl].shape)), c
    h = ops().dequantize_per_channel(dev(q), dev(scales), torch.float16).cpu().numpy()
    assert np.array_equal(h, back.astype(np.float16))


@pytest.mark.parametrize("n,offset", [(15, 0), (16, 0), (4099, 0), (4099, 1), (100000, 3)])
@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_dequantize_and_add_i8_tails_and_unaligned_buffers(n, offset, dtype):
    """sixteen values per lane when the buffers are 16-byte aligned, one per lane otherwise and for the tail: the
    same values either way (offset = elements by which the int8 buffers start off a 16-byte boundary)"""
    say("dequantize / add_i8 n=%d offset=%d %s" % (n, offset, dtype))
    rng = np.random.default_rng(n + offset)
    q = rng.integers(-128, 128, n, dtype=np.int8)
    a = rng.integers(-128, 128, n, dtype=np.int8)
    qd = dev(np.concatenate([np.zeros(offset, np.int8), q]))[offset:]
    ad = dev(np.concatenate([np.zeros(offset, np.int8), a]))[offset:]
    tdt = torch.float32 if dtype == "f32" else torch.float16
    ref = orc.dequantize(q, np.float32(0.0371))
    got = ops().dequantize(qd, 0.0371, tdt).cpu().numpy()
    assert np.array_equal(got, ref if dtype == "f32" else ref.astype(np.float16))
    sa, sb, so = np.float32(0.021), np.float32(0.047), np.float32(0.052)
    inv = np.float32(1.0 / np.float64(so))
    got = host(ops().add_i8(ad, float(sa), qd, float(sb), float(inv)))
    assert np.array_equal(got, orc.add_int8_x86(a, sa, q, sb, so))


@pytest.mark.parametrize("dims", [(1, 256, 256, 1), (1, 12, 4096, 1), (3, 772, 5), (2, 768), (7, 3)])
def test_add_i8_tie_heavy_scales_follow_the_compiled_x86_forms(dims):
    """Equal input scales and an output scale of twice that put every odd a+b on a half-integer, where the two
    contracted forms of the reference's x86 build (vector body / scalar tail channels) and the un-contracted sum all
    round differently for thousands of pairs."""
    say("add_i8 tie-heavy dims=%s" % (dims,))
    sa, sb, so = (np.float32(v) for v in golden_util.INT8_ADD_SCALES[1])
    n = int(np.prod(dims))
    idx = np.arange(n) % 65536
    a = ((idx // 256) - 128).astype(np.int8).reshape(dims)
    b = ((idx % 256) - 128).astype(np.int8).reshape(dims)
    inv = np.float32(1.0 / np.float64(so))
    got = host(ops().add_i8(dev(a), float(sa), dev(b), float(sb), float(inv)))
    assert np.array_equal(got, orc.add_int8_x86(a, sa, b, sb, so))
    if dims == (1, 256, 256, 1):  # the committed result of the reference's own DEVICE_X86 run
        assert np.array_equal(got, golden_util.load("int8_add.npz")["y1_x86"])


@pytest.mark.parametrize("shape,order,offset", [
    ((2, 130, 3, 70), (0, 2, 3, 1), 0),      # transpose, ragged 64 x 64 tiles, two batch axes
    ((5, 64, 96), (0, 2, 1), 0),             # plain batched transpose
    ((3, 4, 5, 6, 7, 8), (5, 0, 4, 1, 3, 2), 0),  # rank 6, three batch axes after merging
    ((4, 100, 12, 64), (0, 2, 1, 3), 0),     # head split: rows of 64 values copied in 16-byte units
    ((4, 100, 12, 64), (0, 2, 1, 3), 1),     # the same from a buffer that is not 16-byte aligned
    ((7, 9, 6), (1, 0, 2), 0),               # innermost run of 6 values: 4-byte units at most
    ((1, 33, 1, 65), (3, 1, 0, 2), 1),       # extent-1 axes dropped: a 2-D transpose, unaligned
    ((2, 3, 4, 5), (0, 1, 2, 3), 0),         # identity: one merged axis
    ((6, 1, 50), (2, 1, 0), 0)])
def test_permute_normal_form_paths(shape, order, offset):
    say("permute paths %s %s offset=%d" % (shape, order, offset))
    rng = np.random.default_rng(sum(shape) + offset)
    n = int(np.prod(shape))
    for np_dt in (np.float32, np.float16, np.int8):
        x = (rng.standard_normal(n) * 50).astype(np_dt)
        buf = dev(np.concatenate([np.zeros(offset, np_dt), x]))
        xd = buf[offset:].view(*shape)
        got = ops().permute(xd, order).cpu().numpy()
        assert np.array_equal(got, np.transpose(x.reshape(shape), order)), np_dt


def test_gelu_i8_matches_three_layer_chain():
    say("gelu_i8")
    q = np.arange(-128, 128, dtype=np.int8)
    q = np.tile(q, 64)
    s_in, s_out = np.float32(0.043), np.float32(0.019)
    inv = np.float32(1.0 / np.float64(s_out))
    got = host(ops().gelu_i8(dev(q), float(s_in), float(inv)))
    ref = orc.quantize_x86(orc.gelu(orc.dequantize(q, s_in)), s_out)
    assert np.array_equal(got, ref)  # the table is built with the C library's double erf, as the CPU chain
    for s_in, s_out in ((0.0005, 0.0003), (0.11, 0.07), (1.7, 0.9), (0.031, 0.25)):
        s_in, s_out = np.float32(s_in), np.float32(s_out)
        inv = np.float32(1.0 / np.float64(s_out))
        got = host(ops().gelu_i8(dev(q), float(s_in), float(inv)))
        assert np.array_equal(got, orc.quantize_x86(orc.gelu(orc.dequantize(q, s_in)), s_out)), (s_in, s_out)


# ---- GEMM ------------------------------------------------------------------------------------------
GEMM_SHAPES = [(1, 1, 1), (3, 4, 9), (8, 21, 10), (11, 50, 19), (33, 65, 130), (128, 768, 768), (130, 96, 264),
               (256, 3072, 768), (64, 768, 3072), (200, 2304, 768)]


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
@pytest.mark.parametrize("b_is_nk", [True, False])
def test_gemm_fp32(M, N, K, b_is_nk):
    say("gemm fp32 M=%d N=%d K=%d nk=%s" % (M, N, K, b_is_nk))
    rng = np.random.default_rng(M * 7 + N * 3 + K)
    a = rng.standard_normal((M, K)).astype(np.float32)
    w = (rng.standard_normal((N, K)) * 0.05).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    if b_is_nk:
        got = host(ops().gemm(dev(a), dev(w), True, bias=dev(bias)))
        ref = orc.inner_product(a, w, bias)           # NaiveFC
    else:
        wt = np.ascontiguousarray(w.T)
        got = host(ops().gemm(dev(a), dev(wt), False))
        ref = orc.matmul(a, wt)                       # double-accumulated MatMul
    assert rel_err(got, ref) <= 1e-5  # far inside the 2e-3 fp32 bar


def test_gemm_identity_and_onehot():
    # closed forms that catch a transposed operand or a wrong index
    say("gemm identity / one-hot")
    rng = np.random.default_rng(21)
    a = rng.standard_normal((70, 96)).astype(np.float32)
    eye = np.eye(96, dtype=np.float32)
    assert np.array_equal(host(ops().gemm(dev(a), dev(eye), True)), a)
    assert np.array_equal(host(ops().gemm(dev(a), dev(eye), False)), a)
    w = np.zeros((5, 96), np.float32)
    for n, k in enumerate([3, 95, 0, 17, 64]):
        w[n, k] = 2.0
    assert np.array_equal(host(ops().gemm(dev(a), dev(w), True)), 2 * a[:, [3, 95, 0, 17, 64]])
    assert np.array_equal(host(ops().gemm(dev(a), dev(np.ascontiguousarray(w.T)), False)),
                          2 * a[:, [3, 95, 0, 17, 64]])


@pytest.mark.parametrize("ba,bb", [(12, 12), (12, 1), (1, 12), (6, 3)])
def test_gemm_batched_broadcast_fp32(ba, bb):
    say("gemm batched ba=%d bb=%d" % (ba, bb))
    rng = np.random.default_rng(ba * 13 + bb)
    a = rng.standard_normal((ba, 40, 64)).astype(np.float32)
    b = rng.standard_normal((bb, 64, 48)).astype(np.float32)
    got = host(ops().gemm(dev(a), dev(b), False))
    assert rel_err(got, orc.matmul(a, b)) <= 1e-5


@pytest.mark.parametrize("M,N,K", [(128, 768, 768), (384, 2304, 768), (200, 3072, 768), (96, 768, 3072),
                                   (17, 40, 24), (5, 7, 9)])
@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_gemm_half_epilogues(M, N, K, dtype):
    say("gemm %s M=%d N=%d K=%d" % (dtype, M, N, K))
    td = torch.float16 if dtype == "f16" else torch.bfloat16
    rng = np.random.default_rng(M + N + K)
    a = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(td)
    w = torch.from_numpy((rng.standard_normal((N, K)) * 0.02).astype(np.float32)).to(td)
    res = torch.from_numpy(rng.standard_normal((M, N)).astype(np.float32)).to(td)
    bias = (rng.standard_normal(N) * 0.1).astype(np.float32)
    af, wf, rf = a.float().numpy(), w.float().numpy(), res.float().numpy()
    tol = FP16_TOL if dtype == "f16" else 2e-2  # bf16 keeps 8 mantissa bits
    got = host(ops().gemm(a.cuda(), w.cuda(), True, bias=dev(bias)))
    assert rel_err(got, orc.inner_product(af, wf, bias)) <= tol
    got = host(ops().gemm(a.cuda(), w.cuda(), True, bias=dev(bias), gelu=True))
    assert rel_err(got, orc.gelu(orc.inner_product(af, wf, bias))) <= tol
    got = host(ops().gemm(a.cuda(), w.cuda(), True, bias=dev(bias), residual=res.cuda()))
    assert rel_err(got, orc.inner_product(af, wf, bias) + rf) <= tol


TILE_CODES = [112211, 222221, 224211, 332221, 331182,   # slabs staged through registers
              2112211, 2222221, 3332221, 3331182]       # slabs loaded global -> LDS directly (2 / 3 stages)


@pytest.mark.parametrize("code", TILE_CODES)
def test_gemm_every_tile_configuration(code):
    """Each tuning configuration of the tiled kernel, forced for a ragged shape (M and N are no tile multiples, K spans
    several slabs): fp16 with the fused epilogues against the checker, int8 bit-exact."""
    from tnn_amd import capi
    lib = capi.load()
    say("tile configuration %d" % code)
    M, N, K = 333, 520, 1536
    rng = np.random.default_rng(code)
    a = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).half()
    w = torch.from_numpy((rng.standard_normal((N, K)) * 0.02).astype(np.float32)).half()
    res = torch.from_numpy(rng.standard_normal((M, N)).astype(np.float32)).half()
    bias = (rng.standard_normal(N) * 0.1).astype(np.float32)
    af, wf, rf = a.float().numpy(), w.float().numpy(), res.float().numpy()
    a8 = rng.integers(-128, 128, (M, K), dtype=np.int8)
    w8 = rng.integers(-127, 128, (N, K), dtype=np.int8)
    b8 = rng.integers(-20000, 20000, N).astype(np.int32)
    scale = orc.fc_int8_scale((rng.uniform(0.5, 1.5, N) * 1e-3).astype(np.float32), np.float32(0.37), N)
    ref_q, ref_acc = orc.fc_int8(a8, w8, b8, scale)
    lib.tnn_rocm_debug_set_gemm_config(code)
    try:
        got = host(ops().gemm(a.cuda(), w.cuda(), True, bias=dev(bias), gelu=True))
        assert rel_err(got, orc.gelu(orc.inner_product(af, wf, bias))) <= FP16_TOL
        got = host(ops().gemm(a.cuda(), w.cuda(), True, bias=dev(bias), residual=res.cuda()))
        assert rel_err(got, orc.inner_product(af, wf, bias) + rf) <= FP16_TOL
        q, acc, _ = ops().gemm_i8(dev(a8), dev(w8), dev(b8), dev(scale), want_acc=True)
        assert np.array_equal(host(acc), ref_acc)
        assert np.array_equal(host(q), ref_q)
    finally:
        lib.tnn_rocm_debug_set_gemm_config(0)


# ---- int8 GEMM: bit-exact accumulators and outputs -----------------------------------------------
@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (2, 4, 9), (2, 16, 19), (7, 32, 16), (128, 3072, 768), (128, 768, 3072),
                                   (300, 768, 768), (65, 100, 200)])
def test_gemm_i8_bit_exact(M, N, K):
    say("gemm_i8 M=%d N=%d K=%d" % (M, N, K))
    rng = np.random.default_rng(M * 5 + N + K)
    a = rng.integers(-128, 128, (M, K), dtype=np.int8)   # full int8 range, not the unit tests' [-8,8)
    w = rng.integers(-127, 128, (N, K), dtype=np.int8)
    bias = rng.integers(-20000, 20000, N).astype(np.int32)
    w_scale = (rng.uniform(0.5, 1.5, N) * 1e-3).astype(np.float32)
    scale = orc.fc_int8_scale(w_scale, np.float32(0.37), N)
    # make sure real rounding happens: typical |acc*scale| ~ tens
    q, acc, outf = ops().gemm_i8(dev(a), dev(w), dev(bias), dev(scale), want_acc=True, dequant_scale=0.37)
    ref_q, ref_acc = orc.fc_int8(a, w, bias, scale)
    assert np.array_equal(host(acc), ref_acc)
    assert np.array_equal(ref_acc, a.astype(np.int64) @ w.astype(np.int64).T + bias)  # pins the checker itself
    assert np.array_equal(host(q), ref_q)
    assert np.array_equal(host(outf), orc.dequantize(ref_q, np.float32(0.37)))


def test_gemm_i8_large_accumulators():
    # |acc| > 2^24: (float)acc rounds before the scale multiply on every path
    say("gemm_i8 saturating inputs")
    M, N, K = 64, 64, 3072
    a = np.full((M, K), 127, np.int8)
    w = np.full((N, K), 127, np.int8)
    w[1::2] = -127
    scale = np.full(N, 2.0e-6, np.float32)
    q, acc, _ = ops().gemm_i8(dev(a), dev(w), None, dev(scale), want_acc=True)
    ref_q, ref_acc = orc.fc_int8(a, w, None, scale)
    assert np.array_equal(host(acc), ref_acc) and abs(int(ref_acc[0, 0])) > 2 ** 24
    assert np.array_equal(host(q), ref_q)


@pytest.mark.parametrize("M,N,K,dtype", [(200, 768, 768, "f32"), (256, 768, 3072, "f32"), (384, 3072, 768, "f16"),
                                         (3072, 768, 3072, "f16")])
def test_gemm_i8_dequant_residual_matches_the_three_layer_chain(M, N, K, dtype):
    """QuantizedInnerProduct -> Reformat(int8->float) -> Add(residual) in one launch: the int8 value is the checker's,
    the float result is q*s + r with the product and the sum rounded separately in fp32 (then once to fp16)."""
    say("gemm_i8_dequant_residual M=%d N=%d K=%d %s" % (M, N, K, dtype))
    rng = np.random.default_rng(M + N + K)
    a = rng.integers(-128, 128, (M, K), dtype=np.int8)
    w = rng.integers(-127, 128, (N, K), dtype=np.int8)
    bias = rng.integers(-20000, 20000, N).astype(np.int32)
    w_scale = (rng.uniform(0.5, 1.5, N) * (2e-3 * 768 / K)).astype(np.float32)
    s_out = np.float32(0.41)
    scale = orc.fc_int8_scale(w_scale, s_out, N)
    tdt = torch.float32 if dtype == "f32" else torch.float16
    res = rng.standard_normal((M, N)).astype(np.float32)
    if dtype == "f16":
        res = r16(res)
    ref_q, _ = orc.fc_int8(a, w, bias, scale)
    assert np.abs(ref_q).max() > 60  # the int8 range is used
    deq = orc.dequantize(ref_q, s_out)
    for r in (None, res):
        got = host(ops().gemm_i8_dequant_residual(dev(a), dev(w), dev(bias), dev(scale), float(s_out),
                                                  None if r is None else dev(r, tdt), tdt))
        want = deq if r is None else (deq + r).astype(np.float32)
        if dtype == "f16":
            want = want.astype(np.float16).astype(np.float32)
        assert np.array_equal(got, want)


@pytest.mark.parametrize("B,S,heads,K", [(2, 64, 2, 128), (3, 40, 12, 768), (8, 384, 12, 768)])
def test_gemm_i8_qkv_split_bit_exact(B, S, heads, K):
    """Three quantised projections + their dequantising Reformat layers in one GEMM, written as Q|K rows and V^T."""
    say("gemm_i8_qkv_split B=%d S=%d heads=%d K=%d" % (B, S, heads, K))
    rng = np.random.default_rng(B * 7 + S + heads)
    H, T = heads * 64, B * S
    x = rng.integers(-128, 128, (T, K), dtype=np.int8)
    w = rng.integers(-127, 128, (3 * H, K), dtype=np.int8)
    bias = rng.integers(-20000, 20000, 3 * H).astype(np.int32)
    w_scale = (rng.uniform(0.5, 1.5, 3 * H) * (2e-3 * 768 / K)).astype(np.float32)
    s_out = np.array([0.41, 0.37, 0.29], np.float32)  # output blob scales of the q, k, v projections
    scale = np.concatenate([orc.fc_int8_scale(w_scale[i * H:(i + 1) * H], s_out[i], H) for i in range(3)])
    dequant = np.repeat(s_out, H).astype(np.float32)
    qk, vt = ops().gemm_i8_qkv_split(dev(x), dev(w), dev(bias), dev(scale), dev(dequant), B, S, heads)
    ref_q, _ = orc.fc_int8(x, w, bias, scale)
    ref = (ref_q.astype(np.float32) * dequant[None, :]).astype(np.float16).astype(np.float32)
    assert np.array_equal(host(qk), ref[:, :2 * H])
    v_ref = ref[:, 2 * H:].reshape(B, S, heads, 64).transpose(0, 2, 3, 1)
    assert np.array_equal(host(vt), v_ref)


def test_embed_layernorm_matches_the_five_layer_chain():
    """Gather(word) + Add(position constant) + Gather(type) + Add + LayerNorm in one launch.  fp32: the checker's
    embedding front end (same order of the two additions, double-precision statistics); fp16: within the fp16 bar;
    an index outside the table raises the error flag like the Gather kernel."""
    import encoder_ref
    say("embed_layernorm")
    rng = np.random.default_rng(11)
    B, S, H, V = 3, 40, 768, 500
    w = {"word_emb": rng.standard_normal((V, H)).astype(np.float32) * 0.05,
         "type_emb": rng.standard_normal((2, H)).astype(np.float32) * 0.05,
         "pos_emb": rng.standard_normal((64, H)).astype(np.float32) * 0.05,
         "emb_ln_g": (1 + 0.1 * rng.standard_normal(H)).astype(np.float32),
         "emb_ln_b": (0.1 * rng.standard_normal(H)).astype(np.float32)}
    ids = rng.integers(0, V, (B, S)).astype(np.int32)
    ids[0, 0] = -1  # negative indices wrap (cpu_gather_layer_acc.cc)
    seg = rng.integers(0, 2, (B, S)).astype(np.int32)
    ids_ref = np.where(ids < 0, ids + V, ids)
    ref = encoder_ref.embed({**w, "pos_emb": w["pos_emb"]}, ids_ref, seg, 1e-12)
    for tdt, tol in ((torch.float32, 2e-6), (torch.float16, FP16_TOL)):
        y, flag = ops().embed_layernorm(dev(ids), dev(seg), dev(w["word_emb"], tdt), dev(w["type_emb"], tdt),
                                        dev(w["pos_emb"][:S], tdt), dev(w["emb_ln_g"]), dev(w["emb_ln_b"]), 1e-12)
        assert int(flag.item()) == 0
        assert rel_err(host(y), ref) <= tol
    # positions looked up through ids of their own (third Gather): the natural order reproduces the result above,
    # other ids pick other rows; one row of ids [1,S] is shared by the batch; an id outside the table raises the flag
    pos = np.tile(np.arange(S, dtype=np.int32), (B, 1))
    y1, flag = ops().embed_layernorm(dev(ids), dev(seg), dev(w["word_emb"]), dev(w["type_emb"]), dev(w["pos_emb"]),
                                     dev(w["emb_ln_g"]), dev(w["emb_ln_b"]), 1e-12, pos_ids=dev(pos))
    assert int(flag.item()) == 0 and rel_err(host(y1), ref) <= 2e-6
    y1b, _ = ops().embed_layernorm(dev(ids), dev(seg), dev(w["word_emb"]), dev(w["type_emb"]), dev(w["pos_emb"]),
                                   dev(w["emb_ln_g"]), dev(w["emb_ln_b"]), 1e-12, pos_ids=dev(pos[:1]))
    assert np.array_equal(host(y1b), host(y1))
    pos2 = rng.integers(0, w["pos_emb"].shape[0], (B, S)).astype(np.int32)
    pos2[0, 1] = -1
    y2, flag = ops().embed_layernorm(dev(ids), dev(seg), dev(w["word_emb"]), dev(w["type_emb"]), dev(w["pos_emb"]),
                                     dev(w["emb_ln_g"]), dev(w["emb_ln_b"]), 1e-12, pos_ids=dev(pos2))
    H_ = w["word_emb"].shape[1]
    tok = orc.binary("add", orc.binary("add", orc.gather(w["word_emb"], ids_ref.reshape(-1))[0],
                                       orc.gather(w["pos_emb"], pos2.reshape(-1))[0]),
                     orc.gather(w["type_emb"], seg.reshape(-1))[0])
    ref2 = orc.layernorm(tok.reshape(B * S, H_), w["emb_ln_g"], w["emb_ln_b"], 1e-12)
    assert int(flag.item()) == 0 and rel_err(host(y2), ref2) <= 2e-6
    pos2[1, 2] = w["pos_emb"].shape[0]
    _, flag = ops().embed_layernorm(dev(ids), dev(seg), dev(w["word_emb"]), dev(w["type_emb"]), dev(w["pos_emb"]),
                                    dev(w["emb_ln_g"]), dev(w["emb_ln_b"]), 1e-12, pos_ids=dev(pos2))
    assert int(flag.item()) == 1
    bad = ids.copy()
    bad[1, 3] = V
    _, flag = ops().embed_layernorm(dev(bad), dev(seg), dev(w["word_emb"]), dev(w["type_emb"]), dev(w["pos_emb"][:S]),
                                    dev(w["emb_ln_g"]), dev(w["emb_ln_b"]), 1e-12)
    assert int(flag.item()) == 1


# ---- fused attention ------------------------------------------------------------------------------
def _attn_case(B, h, S, lens, seed, dtype=torch.float16, with_mask=False):
    rng = np.random.default_rng(seed)
    q = torch.from_numpy(rng.standard_normal((B, h, S, 64)).astype(np.float32)).to(dtype)
    k = torch.from_numpy(rng.standard_normal((B, h, S, 64)).astype(np.float32)).to(dtype)
    v = torch.from_numpy(rng.standard_normal((B, h, S, 64)).astype(np.float32)).to(dtype)
    mask = None
    if lens is not None:
        mask = np.zeros((B, S), np.float32)
        for b, l in enumerate(lens):
            mask[b, l:] = -np.inf
    o = ops()
    kv = None if lens is None else dev(np.asarray(lens, np.int32))
    add_mask = None
    if with_mask:  # TNN-style additive padding mask (0 / -10000) given as data
        add_mask = np.where(np.isinf(mask), np.float32(-10000.0), np.float32(0)) if mask is not None else None
    got = host(o.attention(q.cuda(), k.cuda(), v.cuda(), 0.125, mask=None if add_mask is None else dev(add_mask),
                           kv_len=kv))
    ref = orc.attention_core(q.float().numpy(), k.float().numpy(), v.float().numpy(), 0.125,
                             add_mask if with_mask else mask)
    return got, ref


@pytest.mark.parametrize("B,h,S", [(1, 1, 32), (1, 12, 128), (2, 3, 200), (2, 2, 384), (1, 2, 65), (1, 1, 1)])
def test_attention_fp16_full(B, h, S):
    say("attention fp16 B=%d h=%d S=%d" % (B, h, S))
    got, ref = _attn_case(B, h, S, None, seed=S)
    assert rel_err(got, ref) <= FP16_TOL


def test_attention_fp16_varlen():
    say("attention fp16 variable lengths")
    lens = [16, 512, 100, 257, 64, 1, 333, 480]
    got, ref = _attn_case(8, 2, 512, lens, seed=99)
    assert rel_err(got, ref) <= FP16_TOL
    # the same padding expressed the TNN way: additive -10000 mask + kv_len hint
    got2, ref2 = _attn_case(8, 2, 512, lens, seed=99, with_mask=True)
    assert rel_err(got2, ref2) <= FP16_TOL
    # tiles without a mask take a shorter path (one fused multiply-add per score): equal up to an fp16 rounding
    assert rel_err(got2, got) <= 1e-3


def test_attention_config3_full_shape_slices():
    """Benchmark config 3 at full size (B32, 12 heads x 64, S512, valid lengths U[16,512], padding masked to -inf,
    Q/K/V ~ N(0,1)): the device result of a handful of (batch, head) pairs -- the shortest, the longest and a few
    others -- against the checker in fp32 on the fp16-rounded inputs; (batch, head) pairs are independent."""
    say("attention fp16 config 3 full shape")
    rng = np.random.default_rng(20240603)
    B, h, S = 32, 12, 512
    lens = rng.integers(16, 513, B).astype(np.int32)
    q, k, v = (torch.from_numpy(rng.standard_normal((B, h, S, 64)).astype(np.float32)).half() for _ in range(3))
    got = host(ops().attention(q.cuda(), k.cuda(), v.cuda(), 0.125, kv_len=dev(lens)))
    assert np.isfinite(got).all()
    picks = [(int(np.argmin(lens)), 0), (int(np.argmax(lens)), 11), (3, 5), (17, 7), (31, 2)]
    worst = 0.0
    for b, hh in picks:
        mask = np.zeros((1, S), np.float32)
        mask[0, lens[b]:] = -np.inf
        sl = lambda t: t[b:b + 1, hh:hh + 1].float().numpy()
        ref = orc.attention_core(sl(q), sl(k), sl(v), 0.125, mask)
        worst = max(worst, rel_err(got[b:b + 1, hh:hh + 1], ref))
    say("  worst of %d slices: max rel err %.3g (lengths %d..%d)" % (len(picks), worst, lens.min(), lens.max()))
    assert worst <= FP16_TOL


def test_attention_fp16_128row_blocks():
    # enough (batch, head, query-block) work that the launcher picks the 4-wave / 128-row variant
    say("attention fp16 4-wave variant")
    rng = np.random.default_rng(7)
    lens = rng.integers(16, 513, 8).tolist()
    got, ref = _attn_case(8, 16, 512, lens, seed=123)
    assert rel_err(got, ref) <= FP16_TOL


def test_attention_bf16():
    say("attention bf16")
    got, ref = _attn_case(2, 4, 192, [192, 77], seed=5, dtype=torch.bfloat16)
    assert rel_err(got, ref) <= 3e-2


def test_attention_packed_qkv_layout():
    say("attention packed [T,3H]")
    B, S, h = 2, 96, 12
    H = h * 64
    rng = np.random.default_rng(31)
    qkv = torch.from_numpy(rng.standard_normal((B * S, 3 * H)).astype(np.float32)).half()
    lens = np.array([96, 50], np.int32)
    out = host(ops().attention_packed(qkv.cuda(), B, S, h, 0.125, kv_len=dev(lens)))
    x = qkv.float().numpy().reshape(B, S, 3, h, 64)
    q, k, v = (np.ascontiguousarray(x[:, :, i].transpose(0, 2, 1, 3)) for i in range(3))
    mask = np.zeros((B, S), np.float32)
    mask[1, 50:] = -np.inf
    ref = orc.attention_core(q, k, v, 0.125, mask).transpose(0, 2, 1, 3).reshape(B * S, H)
    assert rel_err(out, ref) <= FP16_TOL


def test_qkv_split_and_attention_vt():
    say("qkv_split GEMM + attention with transposed V")
    B, S, h = 3, 200, 12
    H = h * 64
    rng = np.random.default_rng(41)
    x = torch.from_numpy(rng.standard_normal((B * S, H)).astype(np.float32)).half()
    w = torch.from_numpy((rng.standard_normal((3 * H, H)) * 0.05).astype(np.float32)).half()
    bias = (rng.standard_normal(3 * H) * 0.1).astype(np.float32)
    qk, vt = ops().qkv_split(x.cuda(), w.cuda(), dev(bias), B, S, h)
    ref = orc.inner_product(x.float().numpy(), w.float().numpy(), bias)
    got_qk = host(qk)
    got_v = host(vt).transpose(0, 3, 1, 2).reshape(B * S, H)   # [B,h,64,S] -> [B*S, H]
    assert rel_err(got_qk, ref[:, :2 * H]) <= FP16_TOL
    assert rel_err(got_v, ref[:, 2 * H:]) <= FP16_TOL
    # the transposed copy is exactly the fp16 rounding the row-major epilogue would store
    plain = host(ops().gemm(x.cuda(), w.cuda(), True, bias=dev(bias)))
    assert np.array_equal(got_qk, plain[:, :2 * H]) and np.array_equal(got_v, plain[:, 2 * H:])
    lens = np.array([200, 37, 128], np.int32)
    out = host(ops().attention_qk_vt(qk, vt, B, S, h, 0.125, kv_len=dev(lens)))
    # same inputs through the kernel that transposes V itself: the two feed the keys of a tile into the P.V MFMAs in
    # a different order, so they agree to fp32 accumulation order (one fp16 ulp after the final rounding)
    qkv = torch.from_numpy(plain.astype(np.float16))
    out2 = host(ops().attention_packed(qkv.cuda(), B, S, h, 0.125, kv_len=dev(lens)))
    assert rel_err(out, out2) <= 1e-3
    # and the register-staged form of the same V^T kernel
    from tnn_amd import capi
    capi.load().tnn_rocm_debug_set_attention_dma(0)
    try:
        out3 = host(ops().attention_qk_vt(qk, vt, B, S, h, 0.125, kv_len=dev(lens)))
    finally:
        capi.load().tnn_rocm_debug_set_attention_dma(1)
    assert rel_err(out, out3) <= 1e-3
    xq = plain.reshape(B, S, 3, h, 64)
    q, k, v = (np.ascontiguousarray(xq[:, :, i].transpose(0, 2, 1, 3)) for i in range(3))
    mask = np.zeros((B, S), np.float32)
    for b_, l in enumerate(lens):
        mask[b_, l:] = -np.inf
    ref_o = orc.attention_core(q, k, v, 0.125, mask).transpose(0, 2, 1, 3).reshape(B * S, H)
    assert rel_err(out, ref_o) <= FP16_TOL


@pytest.mark.parametrize("B,S,h,dtype", [(3, 208, 12, "f16"), (2, 80, 4, "f16"), (8, 384, 12, "f16"), (32, 512, 12, "f16"),
                                         (3, 208, 12, "bf16"), (32, 512, 12, "bf16")])
def test_vt_in_accumulator_key_order(B, S, h, dtype):
    """V^T key order 1 (inside every 16 keys the blocks k4-7 and k8-11 exchanged): the three QKV-split projections write
    exactly the natural-order tensor with its keys permuted, and the attention kernels -- the two- and the four-wave form,
    the direct-to-LDS and the register-staged one, plain lengths and an additive mask -- give on the permuted tensor
    what they give on the natural one (the keys of a 16-group meet the P.V MFMA in another order: fp32 accumulation
    order, one fp16 ulp) and what the checker gives."""
    say("V^T in accumulator key order B%d S%d h%d %s" % (B, S, h, dtype))
    from tnn_amd import capi
    o = ops()
    td = torch.float16 if dtype == "f16" else torch.bfloat16
    tol = FP16_TOL if dtype == "f16" else BF16_TOL
    H = h * 64
    rng = np.random.default_rng(B * S)
    x = torch.from_numpy(rng.standard_normal((B * S, H)).astype(np.float32)).to(td).cuda()
    w = torch.from_numpy((rng.standard_normal((3 * H, H)) * 0.05).astype(np.float32)).to(td).cuda()
    bias = dev((rng.standard_normal(3 * H) * 0.1).astype(np.float32))
    qk0, vt0 = o.qkv_split(x, w, bias, B, S, h)
    qk1, vt1 = o.qkv_split(x, w, bias, B, S, h, vt_key_order=1)
    assert torch.equal(qk0, qk1) and torch.equal(vt1, o.permute_keys(vt0)) and not torch.equal(vt1, vt0)
    if H % 128 == 0:   # the LayerNorm-folding form (its weights need no meaning here: same launch, two key orders)
        cs, eps = w.float().sum(1).contiguous(), 1e-12
        a0 = o.qkv_split_ln(x, w, bias, cs, eps, B, S, h)
        a1 = o.qkv_split_ln(x, w, bias, cs, eps, B, S, h, vt_key_order=1)
        assert torch.equal(a0[0], a1[0]) and torch.equal(a1[1], o.permute_keys(a0[1]))
    x8 = torch.randint(-128, 128, (B * S, H), dtype=torch.int8, device="cuda")
    w8 = torch.randint(-127, 128, (3 * H, H), dtype=torch.int8, device="cuda")
    sc = (torch.rand(3 * H, device="cuda") * 2e-4 + 1e-4).float()
    dq = torch.full((3 * H,), 0.05, device="cuda")
    i0 = o.gemm_i8_qkv_split(x8, w8, None, sc, dq, B, S, h, dtype=td)
    i1 = o.gemm_i8_qkv_split(x8, w8, None, sc, dq, B, S, h, dtype=td, vt_key_order=1)
    assert torch.equal(i0[0], i1[0]) and torch.equal(i1[1], o.permute_keys(i0[1]))
    lens = rng.integers(1, S + 1, B).astype(np.int32)
    lens[0] = S
    mask = np.zeros((B, S), np.float32)
    for b_, l in enumerate(lens):
        mask[b_, l:] = -10000.0
    mask[0, 3] = -0.75                                   # a visible key with a bias: that row takes the biased tile form
    plain = host(o.gemm(x, w, True, bias=bias)).reshape(B, S, 3, h, 64)
    q, k, v = (np.ascontiguousarray(plain[:, :, i].transpose(0, 2, 1, 3)) for i in range(3))
    for use_mask in (False, True):
        kw = dict(mask=dev(mask), kv_len=o.mask_to_kv_len(dev(mask), flagged=True)) if use_mask else dict(kv_len=dev(lens))
        ref_mask = mask if use_mask else np.where(np.arange(S)[None, :] < lens[:, None], 0.0, -np.inf).astype(np.float32)
        ref = orc.attention_core(q, k, v, 0.125, ref_mask).transpose(0, 2, 1, 3).reshape(B * S, H)
        for dma in (1, 0):
            capi.load().tnn_rocm_debug_set_attention_dma(dma)
            try:
                nat = host(o.attention_qk_vt(qk0, vt0, B, S, h, 0.125, **kw))
                per = host(o.attention_qk_vt(qk1, vt1, B, S, h, 0.125, vt_key_order=1, **kw))
            finally:
                capi.load().tnn_rocm_debug_set_attention_dma(1)
            assert rel_err(per, nat) <= (1e-3 if dtype == "f16" else 8e-3), (use_mask, dma)
            assert rel_err(per, ref) <= tol, (use_mask, dma)
    # the quantised second output rides along unchanged
    out, out_q = o.attention_qk_vt(qk1, vt1, B, S, h, 0.125, kv_len=dev(lens), q8_inv_scale=np.float32(40.0), vt_key_order=1)
    assert np.array_equal(host(out_q), host(o.quantize(out, np.float32(40.0))))
    with pytest.raises(capi.TnnRocmError):
        o.attention_qk_vt(qk1[: B * 8], vt1[:, :, :, :8].contiguous(), B, 8, h, 0.125, vt_key_order=1)   # S % 16 != 0


def test_mask_prepare_any_float_type():
    """One launch turns an additive mask of any float type into the flagged key counts and, for a half-precision
    mask, its fp32 copy: the same counts and flags as the fp32 kernel gives on the widened mask, row by row -- plain
    padding rows (flagged), rows with a non-zero value on a visible key, holes, a row that masks everything (all keys
    stay visible), a row that masks nothing."""
    say("mask_prepare")
    rng = np.random.default_rng(5)
    B, S = 9, 200
    m = np.zeros((B, S), np.float32)
    m[0, 150:] = -10000.0                      # plain padding
    m[1, 31:] = -10000.0
    m[2, 100:] = -10000.0
    m[2, 17] = -0.5                            # a visible key with a bias: not plain
    m[3, 120:] = -10000.0
    m[3, 40:60] = -10000.0                     # a hole: not plain
    m[4, :] = -10000.0                         # everything masked: every key stays
    m[5, 199:] = -10000.0
    m[6, 1:] = -10000.0                        # a single key
    m[7, :] = rng.standard_normal(S) * 0.1     # a bias everywhere, nothing masked
    for dtype in (torch.float32, torch.float16, torch.bfloat16):
        md = dev(m).to(dtype)
        kv, f32 = ops().mask_prepare(md)
        wide = md.float()
        want = ops().mask_to_kv_len(wide, flagged=True)
        assert torch.equal(kv, want), (dtype, host(kv), host(want))
        assert torch.equal(f32, wide)
        got = host(kv)
        plain = (got & (1 << 30)) != 0
        assert list(plain) == [True, True, False, False, False, True, True, False, True], (dtype, plain)
        assert list(got & ~(1 << 30)) == [150, 31, 100, 120, 200, 199, 1, 200, 200]


def test_store_through_switch_changes_no_result():
    """GEMM, attention and LayerNorm results leave the kernels through device-scope stores by default and through
    ordinary write-back stores with the switch off: the same bits either way, in every epilogue form."""
    say("store-through switch")
    from tnn_amd import capi
    lib, o = capi.load(), ops()
    rng = np.random.default_rng(77)
    B, S, h = 2, 136, 4
    H, T = h * 64, 2 * 136
    x = dev((rng.standard_normal((T, H)) * 0.5).astype(np.float32)).half()
    w = dev((rng.standard_normal((3 * H, H)) * 0.05).astype(np.float32)).half()
    b3 = dev((rng.standard_normal(3 * H) * 0.1).astype(np.float32))
    x32, w32 = x.float(), w.float()
    a8 = dev(rng.integers(-128, 128, (T, H)).astype(np.int8))
    w8 = dev(rng.integers(-127, 128, (3 * H, H)).astype(np.int8))
    bi = dev(rng.integers(-500, 500, 3 * H).astype(np.int32))
    sc = dev((rng.random(3 * H) * 1e-3 + 1e-4).astype(np.float32))
    dq = dev((rng.random(3 * H) * 0.05 + 0.01).astype(np.float32))
    g, be = dev(rng.standard_normal(H).astype(np.float32)), dev(rng.standard_normal(H).astype(np.float32))
    lens = dev(np.array([136, 51], np.int32))
    res = x.clone()

    def run():
        out = []
        out.append(o.gemm(x, w, True, bias=b3, gelu=True))
        out.append(o.gemm(x, w[:H], True, bias=b3[:H], residual=res))
        out.append(o.gemm(x32, w32, True, bias=b3))
        qk, vt = o.qkv_split(x, w, b3, B, S, h)
        out += [qk, vt]
        ctx, ctx_q = o.attention_qk_vt(qk, vt, B, S, h, 0.125, kv_len=lens, q8_inv_scale=20.0)
        out += [ctx, ctx_q]
        out.append(o.attention_packed(torch.cat([qk, vt.permute(0, 3, 1, 2).reshape(T, H)], 1).contiguous(), B, S, h,
                                      0.125, kv_len=lens))
        q, acc, outf = o.gemm_i8(a8, w8, bi, sc, want_acc=True, dequant_scale=0.03, dequant_dtype=torch.float16)
        out += [q, acc, outf]
        out.append(o.gemm_i8_dequant_residual(a8, w8[:H], bi[:H], sc[:H], 0.03, residual=res, dtype=torch.float16))
        out += list(o.gemm_i8_qkv_split(a8, w8, bi, sc, dq, B, S, h))
        y, yq = o.layernorm(x, g, be, 1e-5, residual=res, q_inv_scale=8.0)
        out += [y, yq]
        torch.cuda.synchronize()
        return out

    try:
        assert lib.tnn_rocm_debug_set_store_through(0) == 0
        back = run()
    finally:
        assert lib.tnn_rocm_debug_set_store_through(1) == 0
    through = run()
    assert len(back) == len(through)
    for i, (a, b) in enumerate(zip(back, through)):
        assert torch.equal(a, b), "result %d differs between the two store forms" % i
    # and the default form against the checker, on the plain GEMM
    ref = orc.inner_product(x.float().cpu().numpy(), w.float().cpu().numpy()[:H], host(b3)[:H]) + host(res)
    assert rel_err(host(through[1]), ref) <= FP16_TOL


@pytest.mark.parametrize("S,order", [(328, 0), (336, 1)])
@pytest.mark.parametrize("dtype,tol", [("f16", FP16_TOL), ("bf16", 3e-2)])
def test_attention_vt_scores_that_outgrow_the_running_reference(dtype, tol, S, order):
    """The V^T kernel keeps a running reference for the exponentials that only moves when a score outgrows it by a
    margin.  Keys whose scores jump by far more than that margin from one 64-key tile to the next (both upwards and
    downwards), a ragged last tile, a length-1 and a length-0 sequence, without and with an additive mask given as
    data, against the checker."""
    say("attention V^T kernel, score jumps across key tiles, %s, S %d, key order %d" % (dtype, S, order))
    tdt = torch.float16 if dtype == "f16" else torch.bfloat16
    B, h = 5, 2
    H = h * 64
    rng = np.random.default_rng(77)
    q = rng.standard_normal((B, h, S, 64)).astype(np.float32) * 2
    k = rng.standard_normal((B, h, S, 64)).astype(np.float32)
    v = rng.standard_normal((B, h, S, 64)).astype(np.float32)
    gain = np.ones((B, S), np.float32) * 0.2
    gain[0, 128:] = 4.0                      # up by ~30 in the exp2 domain after two tiles
    gain[1, :128] = 4.0                      # down after two tiles
    # one outlier key per tile, growing: in the second 32 keys of tiles 1 and 2 (the kernel then gives the tile up
    # between its halves), in the first 32 keys of the later ones
    gain[2] = 0.2 + 6.0 * (np.arange(S) % 64 == np.where(np.arange(S) // 64 < 3, 63, 5)) * (np.arange(S) // 64) / 5
    gain[3] = np.linspace(0.1, 5.0, S)
    k *= gain[:, None, :, None]
    q, k, v = (torch.from_numpy(t).to(tdt) for t in (q, k, v))
    lens = np.array([S, S, 300, 1, 0], np.int32)
    qk = torch.cat([q.permute(0, 2, 1, 3).reshape(B * S, H), k.permute(0, 2, 1, 3).reshape(B * S, H)], 1).contiguous()
    vt = v.permute(0, 1, 3, 2).contiguous()
    if order:
        vt = ops().permute_keys(vt)
    mask = np.zeros((B, S), np.float32)
    for b_, l in enumerate(lens):
        mask[b_, l:] = -np.inf
    qf, kf, vf = (t.float().numpy() for t in (q, k, v))
    ref = orc.attention_core(qf[:4], kf[:4], vf[:4], 0.125, mask[:4]).transpose(0, 2, 1, 3).reshape(4 * S, H)
    out = host(ops().attention_qk_vt(qk.cuda(), vt.cuda(), B, S, h, 0.125, kv_len=dev(lens), vt_key_order=order))
    assert np.isfinite(out).all()
    err = rel_err(out[:4 * S], ref)
    say("  lengths only: max rel err %.3g" % err)
    assert err <= tol
    assert np.all(out[4 * S:] == 0)          # no visible key: the row is written as zeros
    # additive mask as data (a bias on some visible keys too), keys past the length still cut by kv_len
    add = (rng.standard_normal((B, S)) * 3).astype(np.float32)
    ref2 = orc.attention_core(qf[:4], kf[:4], vf[:4], 0.125, (mask + add)[:4]).transpose(0, 2, 1, 3).reshape(4 * S, H)
    out2 = host(ops().attention_qk_vt(qk.cuda(), vt.cuda(), B, S, h, 0.125, mask=dev(add), kv_len=dev(lens), vt_key_order=order))
    err2 = rel_err(out2[:4 * S], ref2)
    say("  with additive mask: max rel err %.3g" % err2)
    assert err2 <= tol


def test_attention_vt_precision_on_very_peaked_softmax():
    """What the pre-scaled Q of the V^T kernel costs, pinned so that a change shows.  Projection weights six times the
    usual width give scores whose scaled magnitude reaches ~70 (every softmax row is one-hot but for near ties): the
    direct-to-LDS form, which multiplies Q by scale * log2(e) in fp16 ahead of the score product, stays within 3e-2 of
    the checker there, the register-staged form, which scales the fp32 scores, within 2e-3; at the usual width both are
    inside 2e-3."""
    say("attention V^T kernel, very peaked softmax")
    from tnn_amd import capi
    o = ops()
    B, S, h = 1, 192, 12
    H = h * 64
    for wstd, bar_dma, bar_staged in ((0.3, 3e-2, 2e-3), (0.05, 2e-3, 2e-3)):
        rng = np.random.default_rng(53)
        x = torch.from_numpy(rng.standard_normal((B * S, H)).astype(np.float32)).half().cuda()
        w = torch.from_numpy((rng.standard_normal((3 * H, H)) * wstd).astype(np.float32)).half().cuda()
        bias = dev((rng.standard_normal(3 * H) * 0.1).astype(np.float32))
        plain = host(o.gemm(x, w, True, bias=bias)).reshape(B, S, 3, h, 64)
        q, k, v = (np.ascontiguousarray(plain[:, :, i].transpose(0, 2, 1, 3)) for i in range(3))
        ref = orc.attention_core(q, k, v, 0.125, np.zeros((B, S), np.float32)).transpose(0, 2, 1, 3).reshape(B * S, H)
        qk, vt = o.qkv_split(x, w, bias, B, S, h, vt_key_order=1)
        errs = {}
        for dma in (1, 0):
            capi.load().tnn_rocm_debug_set_attention_dma(dma)
            try:
                errs[dma] = rel_err(host(o.attention_qk_vt(qk, vt, B, S, h, 0.125, vt_key_order=1)), ref)
            finally:
                capi.load().tnn_rocm_debug_set_attention_dma(1)
        say("  weight width %.2f: direct-to-LDS form %.3g, register-staged form %.3g" % (wstd, errs[1], errs[0]))
        assert errs[1] <= bar_dma and errs[0] <= bar_staged


def test_attention_padding_only_sequence_matches_the_reference_softmax():
    """A sequence whose mask is -10000 on every key: the reference computes softmax(scores - 10000) V = softmax(scores) V
    (in fp32 the shifted scores are quantised to 2^-10, which the fp16 bar absorbs); the kernel must do the same,
    not write zeros."""
    say("attention: padding-only sequence")
    rng = np.random.default_rng(77)
    B, S, h, d = 3, 136, 2, 64
    H = h * d
    q, k, v = (r16(rng.standard_normal((B, h, S, d))) for _ in range(3))
    mask = np.zeros((B, S), np.float32)
    mask[0, 100:] = -10000.0
    mask[1, :] = -10000.0
    mask[2, 17:] = -10000.0
    ref = orc.attention_core(q, k, v, 0.125, mask).transpose(0, 2, 1, 3).reshape(B * S, H)
    qt, kt, vt_ = (torch.from_numpy(t).half() for t in (q, k, v))
    qk = torch.cat([qt.permute(0, 2, 1, 3).reshape(B * S, H), kt.permute(0, 2, 1, 3).reshape(B * S, H)], 1).contiguous()
    vt = vt_.permute(0, 1, 3, 2).contiguous()
    lens = ops().mask_to_kv_len(dev(mask), flagged=True)
    out = host(ops().attention_qk_vt(qk.cuda(), vt.cuda(), B, S, h, 0.125, mask=dev(mask), kv_len=lens))
    assert np.abs(out[S:2 * S]).max() > 0.01
    assert rel_err(out, ref) <= FP16_TOL
    assert rel_err(out[S:2 * S], ref[S:2 * S]) <= FP16_TOL


def test_mask_to_kv_len():
    say("mask_to_kv_len")
    m = np.zeros((5, 300), np.float32)
    lens = [300, 1, 64, 65, 299]
    for b, l in enumerate(lens):
        m[b, l:] = -10000.0
    got = host(ops().mask_to_kv_len(dev(m)))
    assert got.tolist() == lens
    # a padding-only row keeps all its keys: the constant -10000 cancels in the reference's softmax
    m0 = m.copy()
    m0[1, :] = -10000.0
    assert host(ops().mask_to_kv_len(dev(m0))).tolist() == [300, 300, 64, 65, 299]
    assert host(ops().mask_to_kv_len(dev(m0), flagged=True)).tolist()[1] == 300  # not flagged: its bias is not zero
    # flagged form: bit 30 marks rows whose visible part is exactly zero; a row with any other visible value is not marked
    m[2, 5] = -0.5
    got = host(ops().mask_to_kv_len(dev(m), flagged=True))
    assert [int(v) & ~(1 << 30) for v in got] == lens
    assert [bool(int(v) >> 30 & 1) for v in got] == [True, True, False, True, True]
    # attention with flagged lengths + mask equals attention with the mask alone (general additive values kept)
    B, S, h = 5, 300, 2
    S8 = 304
    mm = np.full((B, S8), -10000.0, np.float32)
    mm[:, :S] = m
    g = torch.Generator().manual_seed(3)
    qk = torch.randn(B * S8, 2 * h * 64, generator=g).half().cuda()
    vt = torch.randn(B, h, 64, S8, generator=g).half().cuda()
    a1 = ops().attention_qk_vt(qk, vt, B, S8, h, 0.125, mask=dev(mm))
    a2 = ops().attention_qk_vt(qk, vt, B, S8, h, 0.125, mask=dev(mm), kv_len=ops().mask_to_kv_len(dev(mm), flagged=True))
    assert rel_err(host(a2), host(a1)) <= 1e-3


def test_mask_cut_is_relative_to_the_row_maximum():
    """The key count cuts trailing keys whose additive value lies far below the row's best key, not below a fixed
    number: a row whose visible keys carry -999 and -1001 keeps both groups (their weights differ by exp(-2), not by
    exp(-1000)), a row shifted by -5000 as a whole is cut where its padding starts, and one mask row can serve every
    sequence.  The attention result with those counts equals the checker's softmax(scores + mask)."""
    say("mask cut relative to the row maximum")
    B, S, h = 4, 128, 2
    H = h * 64
    m = np.zeros((B, S), np.float32)
    m[0, :50], m[0, 50:100], m[0, 100:] = -999.0, -1001.0, -20000.0
    m[1, :70], m[1, 70:] = -5000.0, -15000.0            # a constant on the whole row: cut at 70, not "nothing visible"
    m[2, :30], m[2, 30:] = 4000.0, 0.0                  # the zeros are the masked ones here
    m[3, 90:] = -10000.0
    kv = host(ops().mask_to_kv_len(dev(m), flagged=True))
    assert [int(v) & ~(1 << 30) for v in kv] == [100, 70, 30, 90]
    assert [bool(int(v) >> 30 & 1) for v in kv] == [False, False, False, True]
    rng = np.random.default_rng(8)
    q, k, v = (rng.standard_normal((B, h, S, 64)).astype(np.float16).astype(np.float32) for _ in range(3))
    ref = orc.attention_core(q, k, v, 0.125, m).transpose(0, 2, 1, 3).reshape(B * S, H)
    qt, kt, vt_ = (torch.from_numpy(t).half() for t in (q, k, v))
    qk = torch.cat([qt.permute(0, 2, 1, 3).reshape(B * S, H), kt.permute(0, 2, 1, 3).reshape(B * S, H)], 1).contiguous()
    vt = vt_.permute(0, 1, 3, 2).contiguous()
    out = host(ops().attention_qk_vt(qk.cuda(), vt.cuda(), B, S, h, 0.125, mask=dev(m), kv_len=dev(kv.astype(np.int32))))
    assert rel_err(out, ref) <= FP16_TOL
    # one row for all sequences, any float type: dense fp32 copy + the same count for every sequence
    for dtype in (torch.float32, torch.float16):
        row = dev(m[3]).to(dtype)
        kv1, f32 = ops().mask_prepare_broadcast(row, 5)
        assert host(kv1).tolist() == [90 | (1 << 30)] * 5
        assert torch.equal(f32, row.float()[None, :].expand(5, S))


def test_attention_rejects_bad_args():
    from tnn_amd import capi
    q = torch.zeros(1, 1, 8, 32, dtype=torch.float16, device="cuda")
    with pytest.raises(capi.TnnRocmError):
        ops().attention(q, q, q, 1.0)  # head_dim 32 is not implemented


# ---- LayerNorm folded into the projections around it ----------------------------------------------
def _fold_ln_weights(w, bias, gamma, beta, td):
    """W' = gamma (.) W rounded to the compute type, its row sums, and bias + W beta"""
    wf = torch.from_numpy((w * gamma[None, :]).astype(np.float32)).to(td)
    colsum = wf.double().sum(1).float().numpy()
    b2 = (bias.astype(np.float64) + w.astype(np.float64) @ beta.astype(np.float64)).astype(np.float32)
    return wf, colsum, b2


@pytest.mark.parametrize("M,dtype", [(300, "f16"), (3072, "f16"), (200, "bf16")])
def test_gemm_layernorm_folded_into_projection(M, dtype):
    """FFN1 and the QKV projection on LayerNorm(t), given the raw t and the folded weights, against the checker's
    LayerNorm -> InnerProduct (-> GELU); the LayerNorm output the kernels also leave for other readers against the
    checker's LayerNorm; non-trivial mean (the folded form subtracts mean * colsum from the accumulators)."""
    say("LayerNorm folded into a projection M=%d %s" % (M, dtype))
    td = torch.float16 if dtype == "f16" else torch.bfloat16
    tol = FP16_TOL if dtype == "f16" else 4e-2
    H, F, heads, eps = 768, 3072, 12, 1e-5
    B, S = (M // 100, 104) if M % 100 == 0 else (M // 384, 384)
    M = B * S
    rng = np.random.default_rng(M)
    r32 = lambda *s: rng.standard_normal(s).astype(np.float32)
    rnd = lambda a: torch.from_numpy(a).to(td).float().numpy()
    t = rnd(r32(M, H) * 1.7 + 0.8 + r32(M, 1))          # row means up to a few sigma
    res = rnd(r32(M, F))
    w1, wqkv = r32(F, H) * 0.05, r32(3 * H, H) * 0.05
    b1, bqkv = r32(F) * 0.1, r32(3 * H) * 0.1
    g, be = 1 + 0.2 * r32(H), 0.3 * r32(H) + 0.5
    D = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(td).cuda()
    o = ops()
    y_ref = orc.layernorm(t, g, be, eps)
    w1f, cs1, b1f = _fold_ln_weights(w1, b1, g, be, td)
    h, y = o.gemm_ln(D(t), w1f.cuda(), dev(b1f), dev(cs1), eps, gamma=dev(g), beta=dev(be), gelu=True, want_y=True)
    assert rel_err(host(y), y_ref) <= tol
    assert rel_err(host(h), orc.gelu(orc.inner_product(y_ref, rnd(w1), b1))) <= tol
    h2 = o.gemm_ln(D(t), w1f.cuda(), dev(b1f), dev(cs1), eps, residual=D(res))
    assert rel_err(host(h2), orc.inner_product(y_ref, rnd(w1), b1) + res) <= tol
    wqf, csq, bqf = _fold_ln_weights(wqkv, bqkv, g, be, td)
    qk, vt, y2 = o.qkv_split_ln(D(t), wqf.cuda(), dev(bqf), dev(csq), eps, B, S, heads, gamma=dev(g), beta=dev(be),
                                want_y=True)
    ref = orc.inner_product(y_ref, rnd(wqkv), bqkv)
    assert rel_err(host(y2), y_ref) <= tol
    assert rel_err(host(qk), ref[:, :2 * H]) <= tol
    vref = ref[:, 2 * H:].reshape(B, S, heads, 64).transpose(0, 2, 3, 1)
    assert rel_err(host(vt), vref) <= tol
    # the rows' {rstd, mean} handed on instead of the LayerNorm output: the statistics themselves, unchanged results,
    # and a projection that rebuilds LayerNorm(t) from them as its residual (the out-projection / FFN2 form)
    mean = t.astype(np.float64).mean(1)
    rstd = 1.0 / np.sqrt(t.astype(np.float64).var(1) + eps)
    h3, st1 = o.gemm_ln(D(t), w1f.cuda(), dev(b1f), dev(cs1), eps, gelu=True, want_stats=True)
    qk3, vt3, st2 = o.qkv_split_ln(D(t), wqf.cuda(), dev(bqf), dev(csq), eps, B, S, heads, want_stats=True)
    assert torch.equal(h3, h) and torch.equal(qk3, qk) and torch.equal(vt3, vt) and torch.equal(st1, st2)
    assert np.abs(host(st1)[:, 0] / rstd - 1).max() <= 1e-5 and np.abs(host(st1)[:, 1] - mean).max() <= 1e-5
    x2, w2, b2 = rnd(r32(M, F) * 0.5), r32(H, F) * 0.03, r32(H) * 0.1
    ref2 = orc.inner_product(x2, rnd(w2), b2) + y_ref
    got2 = o.gemm_residual_ln(D(x2), D(w2), D(t), st1, dev(g), dev(be), bias=dev(b2))
    assert rel_err(host(got2), ref2) <= tol
    via_y = o.gemm(D(x2), D(w2), True, bias=dev(b2), residual=y)   # the same sum with the stored LayerNorm output
    assert rel_err(host(got2), host(via_y)) <= tol
    xo, wo = rnd(r32(M, H) * 0.5), r32(H, H) * 0.05               # K = 768: the 64x64-tile shape
    got3 = o.gemm_residual_ln(D(xo), D(wo), D(t), st1, dev(g), dev(be), bias=dev(b2), gelu=True)
    assert rel_err(host(got3), orc.gelu(orc.inner_product(xo, rnd(wo), b2)) + y_ref) <= tol
    # the same projections also leaving the row sums of what they stored, per tile column; a folding GEMM that is handed
    # those sums gives the results and statistics of one that takes them from its own operand
    for xx, ww, plain in ((x2, w2, got2), (xo, wo, None)):
        c, (sums, blocks) = o.gemm_residual_ln(D(xx), D(ww), D(t), st1, dev(g), dev(be), bias=dev(b2), want_row_sums=True)
        if plain is not None:
            assert torch.equal(c, plain)
        assert 1 <= blocks <= o.MAX_ROW_SUM_BLOCKS and H % blocks == 0
        cf = c.float().cpu().numpy().astype(np.float64)
        per = cf.reshape(M, blocks, H // blocks)
        got_s = host(sums)[:blocks]                               # [blocks, M, 2]
        assert np.abs(got_s[:, :, 0].T - per.sum(2)).max() <= 1e-3 * max(1.0, np.abs(per.sum(2)).max())
        assert np.abs(got_s[:, :, 1].T / (per ** 2).sum(2) - 1).max() <= 1e-5
        assert not host(sums)[blocks:].any()                      # nothing written past the blocks reported
        own_h, own_st = o.gemm_ln(c, w1f.cuda(), dev(b1f), dev(cs1), eps, gelu=True, want_stats=True)
        fed_h, fed_st = o.gemm_ln(c, w1f.cuda(), dev(b1f), dev(cs1), eps, gelu=True, want_stats=True, row_sums=(sums, blocks))
        assert np.abs(host(fed_st)[:, 0] / host(own_st)[:, 0] - 1).max() <= 1e-5
        assert np.abs(host(fed_st)[:, 1] - host(own_st)[:, 1]).max() <= 1e-5
        assert rel_err(host(fed_h), host(own_h)) <= 2e-3
        assert rel_err(host(fed_h), orc.gelu(orc.inner_product(orc.layernorm(cf.astype(np.float32), g, be, eps), rnd(w1), b1))) <= tol
        own_q = o.qkv_split_ln(c, wqf.cuda(), dev(bqf), dev(csq), eps, B, S, heads, want_stats=True)
        fed_q = o.qkv_split_ln(c, wqf.cuda(), dev(bqf), dev(csq), eps, B, S, heads, want_stats=True, row_sums=(sums, blocks))
        assert rel_err(host(fed_q[0]), host(own_q[0])) <= 2e-3 and rel_err(host(fed_q[1]), host(own_q[1])) <= 2e-3
        assert np.abs(host(fed_q[2])[:, 0] / host(own_q[2])[:, 0] - 1).max() <= 1e-5


@pytest.mark.parametrize("blocks", [4, 12, 16, 24])
@pytest.mark.parametrize("offset_rows", [False, True])
def test_folding_gemm_fed_row_sums_against_own_statistics(blocks, offset_rows):
    """A LayerNorm-folding GEMM that is handed its rows' sums per block of columns (made here on the host, so the block
    count is free: up to twelve blocks the kernels request them late, above that the shapes that share a CU request them
    ahead of their first slabs) against the same GEMM taking the statistics from its own operand: FFN1-shaped
    (192x192 tiles) and QKV-shaped (128x128 tiles) at M = 3072.  offset_rows: every row sits at 20 +- 0.1, where
    E[x^2] - mean^2 loses most of its digits in fp32 block sums and must still not go negative."""
    say("folding GEMM, fed row sums, %d blocks%s" % (blocks, ", offset rows" if offset_rows else ""))
    o = ops()
    rng = np.random.default_rng(100 + blocks)
    M, H, F, B, S, heads = 3072, 768, 3072, 8, 384, 12
    eps = 1e-12
    t = rng.standard_normal((M, H)).astype(np.float32)
    if offset_rows:
        t = (20.0 + 0.1 * t).astype(np.float32)
    t16 = torch.from_numpy(t).half()
    tf = t16.float().numpy().astype(np.float64)
    per = tf.reshape(M, blocks, H // blocks)
    sums = np.zeros((o.MAX_ROW_SUM_BLOCKS, M, 2), np.float32)
    sums[:blocks, :, 0] = per.sum(2).T
    sums[:blocks, :, 1] = (per ** 2).sum(2).T
    g, be = (1 + 0.1 * rng.standard_normal(H)).astype(np.float32), (0.1 * rng.standard_normal(H)).astype(np.float32)
    w1, b1 = (rng.standard_normal((F, H)) * 0.03).astype(np.float32), (rng.standard_normal(F) * 0.1).astype(np.float32)
    wq, bq = (rng.standard_normal((3 * H, H)) * 0.03).astype(np.float32), (rng.standard_normal(3 * H) * 0.1).astype(np.float32)
    w1f, cs1, b1f = _fold_ln_weights(w1, b1, g, be, torch.float16)
    wqf, csq, bqf = _fold_ln_weights(wq, bq, g, be, torch.float16)
    c, dsums = t16.cuda(), dev(sums)
    own_h, own_st = o.gemm_ln(c, w1f.cuda(), dev(b1f), dev(cs1), eps, gelu=True, want_stats=True)
    fed_h, fed_st = o.gemm_ln(c, w1f.cuda(), dev(b1f), dev(cs1), eps, gelu=True, want_stats=True, row_sums=(dsums, blocks))
    own_q = o.qkv_split_ln(c, wqf.cuda(), dev(bqf), dev(csq), eps, B, S, heads, want_stats=True)
    fed_q = o.qkv_split_ln(c, wqf.cuda(), dev(bqf), dev(csq), eps, B, S, heads, want_stats=True, row_sums=(dsums, blocks))
    mean = tf.mean(1)
    rstd = 1.0 / np.sqrt(tf.var(1) + eps)
    # with rows at 20 +- 0.1 the variance is 1e-2 out of E[x^2] = 400: fp32 sums of squares leave it ~3 digits
    rtol = 3e-3 if offset_rows else 1e-5
    for st in (fed_st, fed_q[2]):
        st = host(st)
        assert np.isfinite(st).all()
        assert np.abs(st[:, 0] / rstd - 1).max() <= rtol and np.abs(st[:, 1] - mean).max() <= 1e-5 * max(1.0, np.abs(mean).max())
    if not offset_rows:
        assert np.abs(host(fed_st)[:, 0] / host(own_st)[:, 0] - 1).max() <= 1e-5
        assert rel_err(host(fed_h), host(own_h)) <= 2e-3
        assert rel_err(host(fed_q[0]), host(own_q[0])) <= 2e-3 and rel_err(host(fed_q[1]), host(own_q[1])) <= 2e-3
    else:
        assert np.isfinite(host(fed_h)).all() and np.isfinite(host(fed_q[0])).all()
        ref = orc.gelu(orc.inner_product(orc.layernorm(tf.astype(np.float32), g, be, eps), w1f.float().numpy() / g[None, :], b1))
        assert rel_err(host(fed_h), ref) <= 3e-2     # three digits of rstd, then a 768-term product


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_attention_quantised_second_output_bit_exact(dtype):
    """The int8 tensor the attention kernel can write next to its output equals the checker's x86 quantiser applied to
    that output (the Reformat layer it replaces), bit for bit; the float output is unchanged by asking for it."""
    say("attention with a quantised second output, " + dtype)
    td = torch.float16 if dtype == "f16" else torch.bfloat16
    B, S, heads, H = 3, 200, 12, 768
    g = torch.Generator().manual_seed(5)
    qk = torch.randn(B * S, 2 * H, generator=g).to(td).cuda()
    vt = torch.randn(B, heads, 64, S, generator=g).to(td).cuda()
    lens = torch.tensor([200, 77, 130], dtype=torch.int32).cuda()
    scale = np.float32(0.0173)
    inv = np.float32(1.0 / scale)
    plain = ops().attention_qk_vt(qk, vt, B, S, heads, 0.125, kv_len=lens)
    out, out_q = ops().attention_qk_vt(qk, vt, B, S, heads, 0.125, kv_len=lens, q8_inv_scale=inv)
    assert torch.equal(plain, out)
    ref_q = orc.quantize_x86(out.float().cpu().numpy(), scale)
    assert np.array_equal(host(out_q), ref_q)
    assert np.array_equal(host(out_q), host(ops().quantize(out, inv)))
    assert np.abs(host(out_q).astype(int)).max() >= 30  # the scale makes real use of the int8 range


@pytest.mark.parametrize("M,N,K", [(300, 3072, 768), (65, 100, 200), (4096, 3072, 768)])
def test_gemm_i8_with_gelu_table_bit_exact(M, N, K):
    """QuantizedInnerProduct -> int8 GELU as one launch (the 256-entry table applied in the GEMM epilogue) equals the two
    launches, and the checker's chain, bit for bit."""
    say("gemm_i8 + GELU table M=%d N=%d K=%d" % (M, N, K))
    rng = np.random.default_rng(M + N)
    a = rng.integers(-128, 128, (M, K), dtype=np.int8)
    w = rng.integers(-127, 128, (N, K), dtype=np.int8)
    bias = rng.integers(-20000, 20000, N).astype(np.int32)
    s_mid, s_out = np.float32(0.031), np.float32(0.027)
    scale = orc.fc_int8_scale((rng.uniform(0.5, 1.5, N) * 1e-5).astype(np.float32), s_mid, N)
    inv_out = np.float32(1.0 / s_out)
    o = ops()
    iota = torch.arange(-128, 128, dtype=torch.int16).to(torch.int8).cuda()
    lut = o.gelu_i8(iota, s_mid, inv_out)
    fused = host(o.gemm_i8_lut(dev(a), dev(w), dev(bias), dev(scale), lut))
    q, _, _ = o.gemm_i8(dev(a), dev(w), dev(bias), dev(scale))
    two = host(o.gelu_i8(q, s_mid, inv_out))
    assert np.array_equal(fused, two)
    ref_q, _ = orc.fc_int8(a, w, bias, scale)
    ref = orc.quantize_x86(orc.gelu(orc.dequantize(ref_q, s_mid)), s_out)
    assert np.array_equal(fused, ref)
    assert len(np.unique(host(q))) > 100                    # the requantised values span the int8 range
