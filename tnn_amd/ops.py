"""Thin tensor-level wrappers over the C ABI.

torch is used only as plumbing: it owns device memory and the stream.  Every function passes raw
device pointers into libtnn_rocm.so; there is no torch implementation behind any of them.
"""
import torch

from . import capi
from .capi import F32, F16, I8, I32, BF16, EPI_BIAS, EPI_GELU, EPI_RESIDUAL, EPI_NONE  # noqa: F401

_DT = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16, torch.int8: I8, torch.int32: I32}


def dt(t):
    return _DT[t.dtype]


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _p(t):
    return None if t is None else t.data_ptr()


def _chk(*ts):
    for t in ts:
        if t is not None:
            assert t.is_cuda and t.is_contiguous(), "device-resident contiguous tensors only"


def gemm(a, b, b_is_nk=True, bias=None, gelu=False, residual=None, out=None):
    """a: [batch?, M, K]; b: [N, K] (b_is_nk) or [K, N]; optional leading batch dims broadcast by modulo."""
    _chk(a, b, bias, residual, out)
    M, K = a.shape[-2], a.shape[-1]
    N = b.shape[-2] if b_is_nk else b.shape[-1]
    assert (b.shape[-1] if b_is_nk else b.shape[-2]) == K
    batch_a = a.numel() // (M * K) if M * K else 1
    batch_b = b.numel() // (N * K) if N * K else 1
    batch = max(batch_a, batch_b)
    if out is None:
        lead = a.shape[:-2] if batch_a >= batch_b else b.shape[:-2]
        out = torch.empty(*lead, M, N, dtype=a.dtype, device=a.device)
    epi = (EPI_BIAS if bias is not None else 0) | (EPI_GELU if gelu else 0) | (EPI_RESIDUAL if residual is not None else 0)
    capi.call("tnn_rocm_gemm", _stream(), dt(a), 1 if b_is_nk else 0, _p(a), _p(b), _p(out), M, N, K,
              K, K if b_is_nk else N, N, batch, batch_a, batch_b, epi, _p(bias), _p(residual), N)
    return out


def gemm_i8(a, w, bias, scale, want_acc=False, want_q=True, dequant_scale=None, dequant_dtype=torch.float32):
    _chk(a, w, bias, scale)
    M, K = a.shape
    N = w.shape[0]
    q = torch.empty(M, N, dtype=torch.int8, device=a.device) if want_q else None
    acc = torch.empty(M, N, dtype=torch.int32, device=a.device) if want_acc else None
    outf = torch.empty(M, N, dtype=dequant_dtype, device=a.device) if dequant_scale is not None else None
    capi.call("tnn_rocm_gemm_i8", _stream(), _p(a), _p(w), _p(bias), _p(scale), _p(q), _p(acc), M, N, K, K, K, N,
              _p(outf), _DT[dequant_dtype], float(dequant_scale or 0.0))
    return q, acc, outf


def gemm_i8_lut(a, w, bias, scale, lut, out=None):
    """int8 out = lut[requantise(a w^T + bias) + 128]; lut: 256 int8 values on the device"""
    _chk(a, w, bias, scale, lut)
    M, K = a.shape
    N = w.shape[0]
    q = out if out is not None else torch.empty(M, N, dtype=torch.int8, device=a.device)
    capi.call("tnn_rocm_gemm_i8_lut", _stream(), _p(a), _p(w), _p(bias), _p(scale), _p(q), M, N, K, K, K, N, _p(lut))
    return q


def gemm_i8_dequant_residual(a, w, bias, scale, dequant_scale, residual=None, dtype=torch.float32):
    """float out = requantise(a w^T + bias) * dequant_scale (+ residual); a [M,K] int8, w [N,K] int8"""
    _chk(a, w, bias, scale, residual)
    M, K = a.shape
    N = w.shape[0]
    out = torch.empty(M, N, dtype=dtype, device=a.device)
    capi.call("tnn_rocm_gemm_i8_dequant_residual", _stream(), _p(a), _p(w), _p(bias), _p(scale), M, N, K, K, K, _p(out),
              _DT[dtype], N, float(dequant_scale), _p(residual))
    return out


def gemm_i8_qkv_split(x, wqkv, bias, scale, dequant, B, S, heads, dtype=torch.float16, vt_key_order=0):
    """x [B*S,K] int8, wqkv [3H,K] int8 -> (qk [B*S,2H], vt [B,heads,64,S]) dequantised"""
    _chk(x, wqkv, bias, scale, dequant)
    H = heads * 64
    qk = torch.empty(B * S, 2 * H, dtype=dtype, device=x.device)
    vt = torch.empty(B, heads, 64, S, dtype=dtype, device=x.device)
    capi.call("tnn_rocm_gemm_i8_qkv_split", _stream(), _DT[dtype], _p(x), _p(wqkv), _p(bias), _p(scale), _p(dequant),
              _p(qk), _p(vt), B, S, heads, x.shape[1], int(vt_key_order))
    return qk, vt


def attention(q, k, v, scale, mask=None, kv_len=None, out=None):
    """q, k, v: [B, h, S, d] contiguous."""
    _chk(q, k, v, mask, kv_len)
    B, h, S, d = q.shape
    if out is None:
        out = torch.empty_like(q)
    capi.call("tnn_rocm_attention", _stream(), dt(q), _p(q), _p(k), _p(v), _p(out), B, h, S, d,
              h * S * d, S * d, d, h * S * d, S * d, d, h * S * d, S * d, d, float(scale), _p(mask), _p(kv_len))
    return out


def attention_packed(qkv, B, S, heads, scale, mask=None, kv_len=None, out=None):
    """qkv: [B*S, 3*H] (Q | K | V column blocks, heads contiguous inside each); out: [B*S, H]."""
    _chk(qkv, mask, kv_len, out)
    H = qkv.shape[1] // 3
    d = H // heads
    if out is None:
        out = torch.empty(B * S, H, dtype=qkv.dtype, device=qkv.device)
    es = qkv.element_size()
    base = qkv.data_ptr()
    capi.call("tnn_rocm_attention", _stream(), dt(qkv), base, base + H * es, base + 2 * H * es, _p(out), B, heads, S, d,
              S * 3 * H, d, 3 * H, S * 3 * H, d, 3 * H, S * H, d, H, float(scale), _p(mask), _p(kv_len))
    return out


def qkv_split(x, wqkv, bqkv, B, S, heads, vt_key_order=0):
    """x [B*S, K], wqkv [3H, K] -> (qk [B*S, 2H], vt [B, heads, 64, S]); vt_key_order 1: the keys of vt in the order
    the attention kernel's accumulators hold them (see permute_keys)"""
    _chk(x, wqkv, bqkv)
    H = heads * 64
    qk = torch.empty(B * S, 2 * H, dtype=x.dtype, device=x.device)
    vt = torch.empty(B, heads, 64, S, dtype=x.dtype, device=x.device)
    capi.call("tnn_rocm_gemm_qkv_split", _stream(), dt(x), _p(x), _p(wqkv), _p(bqkv), _p(qk), _p(vt), B, S, heads,
              x.shape[1], int(vt_key_order))
    return qk, vt


MAX_ROW_SUM_BLOCKS = 24   # TNN_ROCM_MAX_ROW_SUM_BLOCKS


def gemm_ln(t, w_folded, bias_folded, colsum, eps, gamma=None, beta=None, gelu=False, residual=None, want_y=False,
            want_stats=False, row_sums=None):
    """C = act(LayerNorm(t) W^T + b) (+ residual) from the raw t and the folded weights; optionally also LayerNorm(t)
    and / or the rows' {rstd, mean} ([M, 2] fp32); returns C, then y, then the statistics, as asked for.
    row_sums = (buffer, blocks) as returned by gemm_residual_ln(want_row_sums=True) for the launch that wrote t."""
    _chk(t, w_folded, bias_folded, colsum, gamma, beta, residual)
    M, K = t.shape
    N = w_folded.shape[0]
    c = torch.empty(M, N, dtype=t.dtype, device=t.device)
    y = torch.empty_like(t) if want_y else None
    st = torch.empty(M, 2, dtype=torch.float32, device=t.device) if want_stats else None
    flags = (2 if gelu else 0) | (4 if residual is not None else 0)
    sums, blocks = row_sums if row_sums is not None else (None, 0)
    capi.call("tnn_rocm_gemm_ln", _stream(), dt(t), _p(t), _p(w_folded), _p(bias_folded), _p(colsum), _p(gamma), _p(beta),
              float(eps), _p(c), _p(y), _p(st), _p(sums), blocks, M, N, K, flags, _p(residual))
    out = (c,) + ((y,) if want_y else ()) + ((st,) if want_stats else ())
    return out if len(out) > 1 else c


def qkv_split_ln(t, wqkv_folded, bqkv_folded, colsum, eps, B, S, heads, gamma=None, beta=None, want_y=False,
                 want_stats=False, row_sums=None, vt_key_order=0):
    """qkv_split on LayerNorm(t) given as the raw t and the folded weights; optionally also LayerNorm(t) and / or the
    rows' {rstd, mean}; row_sums as for gemm_ln"""
    _chk(t, wqkv_folded, bqkv_folded, colsum, gamma, beta)
    H = heads * 64
    qk = torch.empty(B * S, 2 * H, dtype=t.dtype, device=t.device)
    vt = torch.empty(B, heads, 64, S, dtype=t.dtype, device=t.device)
    y = torch.empty_like(t) if want_y else None
    st = torch.empty(B * S, 2, dtype=torch.float32, device=t.device) if want_stats else None
    sums, blocks = row_sums if row_sums is not None else (None, 0)
    capi.call("tnn_rocm_gemm_qkv_split_ln", _stream(), dt(t), _p(t), _p(wqkv_folded), _p(bqkv_folded), _p(colsum), _p(gamma),
              _p(beta), float(eps), _p(qk), _p(vt), _p(y), _p(st), _p(sums), blocks, B, S, heads, t.shape[1], int(vt_key_order))
    return (qk, vt) + ((y,) if want_y else ()) + ((st,) if want_stats else ())


def gemm_residual_ln(x, w, t, row_stats, gamma, beta, bias=None, gelu=False, out=None, want_row_sums=False,
                     row_sums_out=None):
    """C = act(x W^T + b) + LayerNorm(t), the LayerNorm rebuilt from t and its rows' {rstd, mean}; with want_row_sums
    also (buffer, blocks): the sums / sums of squares of C's rows per tile column, for gemm_ln / qkv_split_ln on C"""
    import ctypes
    _chk(x, w, t, row_stats, gamma, beta, bias, out)
    M, K = x.shape
    N = w.shape[0]
    if out is None:
        out = torch.empty(M, N, dtype=x.dtype, device=x.device)
    flags = (1 if bias is not None else 0) | (2 if gelu else 0)
    sums, blocks = None, ctypes.c_int(0)
    if want_row_sums:
        sums = row_sums_out if row_sums_out is not None else torch.zeros(MAX_ROW_SUM_BLOCKS, M, 2, dtype=torch.float32,
                                                                       device=x.device)
    capi.call("tnn_rocm_gemm_residual_ln", _stream(), dt(x), _p(x), _p(w), _p(bias), _p(out), _p(t), _p(row_stats), _p(gamma),
              _p(beta), M, N, K, flags, _p(sums), ctypes.addressof(blocks) if want_row_sums else None)
    return (out, (sums, blocks.value)) if want_row_sums else out


def permute_keys(vt):
    """vt [..., S] with S % 16 == 0 -> the same tensor with, inside every group of 16 keys, the blocks k4-7 and k8-11
    exchanged: V^T key order 1 of the C ABI"""
    S = vt.shape[-1]
    idx = torch.arange(S, device=vt.device)
    src = (idx & ~12) | ((idx & 4) << 1) | ((idx & 8) >> 1)
    return vt.index_select(-1, src).contiguous()


def attention_qk_vt(qk, vt, B, S, heads, scale, mask=None, kv_len=None, out=None, q8_inv_scale=None, vt_key_order=0):
    """qk [B*S, 2H] (Q | K), vt [B, heads, 64, S]; out [B*S, H]; with q8_inv_scale also the int8 quantisation of out"""
    _chk(qk, vt, mask, kv_len, out)
    H = heads * 64
    if out is None:
        out = torch.empty(B * S, H, dtype=qk.dtype, device=qk.device)
    es = qk.element_size()
    base = qk.data_ptr()
    if q8_inv_scale is not None or vt_key_order:
        out_q = torch.empty(B * S, H, dtype=torch.int8, device=qk.device) if q8_inv_scale is not None else None
        capi.call("tnn_rocm_attention_vt_q8", _stream(), dt(qk), base, base + H * es, _p(vt), _p(out), _p(out_q),
                  float(q8_inv_scale or 0.0), B, heads, S, 64, S * 2 * H, 64, 2 * H, S * 2 * H, 64, 2 * H, heads * 64 * S,
                  64 * S, S, S * H, 64, H, float(scale), _p(mask), _p(kv_len), int(vt_key_order))
        return (out, out_q) if q8_inv_scale is not None else out
    capi.call("tnn_rocm_attention_vt", _stream(), dt(qk), base, base + H * es, _p(vt), _p(out), B, heads, S, 64,
              S * 2 * H, 64, 2 * H, S * 2 * H, 64, 2 * H, heads * 64 * S, 64 * S, S, S * H, 64, H, float(scale),
              _p(mask), _p(kv_len))
    return out


def mask_to_kv_len(mask, threshold=-1000.0, flagged=False):
    """flagged: bit 30 of an entry marks a mask row that is exactly 0 on every visible key"""
    _chk(mask)
    B, S = mask.shape
    out = torch.empty(B, dtype=torch.int32, device=mask.device)
    capi.call("tnn_rocm_mask_to_kv_len_flagged" if flagged else "tnn_rocm_mask_to_kv_len", _stream(), _p(mask), _p(out), B,
              S, float(threshold))
    return out


def mask_prepare(mask, threshold=-1000.0):
    """flagged kv_len of a mask [B,S] of any float type and, for a half-precision mask, its fp32 copy: (kv_len, mask_f32)"""
    _chk(mask)
    B, S = mask.shape
    out = torch.empty(B, dtype=torch.int32, device=mask.device)
    f32 = mask if mask.dtype == torch.float32 else torch.empty(B, S, dtype=torch.float32, device=mask.device)
    capi.call("tnn_rocm_mask_prepare", _stream(), dt(mask), _p(mask), None if mask.dtype == torch.float32 else _p(f32), _p(out),
              B, S, float(threshold))
    return out, f32


def mask_prepare_broadcast(mask_row, B, threshold=-1000.0):
    """one mask row [S] of any float type serving B sequences: (flagged kv_len [B], dense fp32 mask [B,S])"""
    _chk(mask_row)
    S = mask_row.shape[-1]
    out = torch.empty(B, dtype=torch.int32, device=mask_row.device)
    f32 = torch.empty(B, S, dtype=torch.float32, device=mask_row.device)
    capi.call("tnn_rocm_mask_prepare_strided", _stream(), dt(mask_row), _p(mask_row), 0, _p(f32), _p(out), B, S, float(threshold))
    return out, f32


def softmax(x, axis=-1):
    _chk(x)
    axis = axis % x.dim()
    outer = 1
    for s in x.shape[:axis]:
        outer *= s
    inner = 1
    for s in x.shape[axis + 1:]:
        inner *= s
    y = torch.empty_like(x)
    capi.call("tnn_rocm_softmax", _stream(), dt(x), _p(x), _p(y), outer, x.shape[axis], inner)
    return y


def layernorm(x, gamma, beta, eps, residual=None, q_inv_scale=None):
    _chk(x, gamma, beta, residual)
    cols = gamma.numel()
    rows = x.numel() // cols
    y = torch.empty_like(x)
    q = torch.empty(x.shape, dtype=torch.int8, device=x.device) if q_inv_scale is not None else None
    capi.call("tnn_rocm_layernorm", _stream(), dt(x), _p(x), _p(residual), _p(gamma), _p(beta), _p(y), rows, cols,
              float(eps), _p(q), float(q_inv_scale or 0.0))
    return (y, q) if q is not None else y


def embed_layernorm(ids, type_ids, word_table, type_table, pos_table, gamma, beta, eps, pos_ids=None):
    """ids/type_ids int32 [B,S] -> LayerNorm(word[ids] + pos[s] + type[type_ids]) as [B*S, H]; with pos_ids (int32,
    [B,S] or [1,S]) the position rows are pos[pos_ids] instead"""
    _chk(ids, type_ids, word_table, type_table, pos_table, gamma, beta, pos_ids)
    rows, H = ids.numel(), word_table.shape[1]
    y = torch.empty(rows, H, dtype=word_table.dtype, device=word_table.device)
    flag = torch.zeros(1, dtype=torch.int32, device=word_table.device)
    if pos_ids is not None:
        capi.call("tnn_rocm_embed_layernorm_pos", _stream(), dt(word_table), _p(ids), _p(type_ids), _p(pos_ids),
                  pos_ids.numel(), _p(word_table), word_table.shape[0], _p(type_table), type_table.shape[0], _p(pos_table),
                  pos_table.shape[0], _p(gamma), _p(beta), float(eps), _p(y), rows, H, _p(flag))
        return y, flag
    capi.call("tnn_rocm_embed_layernorm", _stream(), dt(word_table), _p(ids), _p(type_ids), _p(word_table),
              word_table.shape[0], _p(type_table), type_table.shape[0], _p(pos_table), pos_table.shape[0], _p(gamma),
              _p(beta), float(eps), _p(y), rows, H, _p(flag))
    return y, flag


def gelu(x):
    _chk(x)
    y = torch.empty_like(x)
    capi.call("tnn_rocm_gelu", _stream(), dt(x), _p(x), _p(y), x.numel())
    return y


def tanh(x):
    _chk(x)
    y = torch.empty_like(x)
    capi.call("tnn_rocm_tanh", _stream(), dt(x), _p(x), _p(y), x.numel())
    return y


def binary(op, a, b, out_shape=None):
    _chk(a, b)
    if out_shape is None:
        out_shape = torch.broadcast_shapes(a.shape, b.shape)
    out = torch.empty(*out_shape, dtype=a.dtype, device=a.device)
    capi.call("tnn_rocm_binary", _stream(), dt(a), {"add": 0, "sub": 1, "mul": 2, "div": 3}[op], _p(a),
              capi.int_array(a.shape), a.dim(), _p(b), capi.int_array(b.shape), b.dim(), _p(out),
              capi.int_array(out_shape), len(out_shape))
    return out


def permute(x, order):
    _chk(x)
    out = torch.empty(*[x.shape[o] for o in order], dtype=x.dtype, device=x.device)
    capi.call("tnn_rocm_permute", _stream(), x.element_size(), _p(x), _p(out), capi.int_array(x.shape),
              capi.int_array(order), x.dim())
    return out


def gather(data, indices, axis=0):
    _chk(data, indices)
    batch = 1
    for s in data.shape[:axis]:
        batch *= s
    slices = data.shape[axis]
    slice_elems = 1
    for s in data.shape[axis + 1:]:
        slice_elems *= s
    out = torch.empty(*data.shape[:axis], *indices.shape, *data.shape[axis + 1:], dtype=data.dtype, device=data.device)
    flag = torch.zeros(1, dtype=torch.int32, device=data.device)
    capi.call("tnn_rocm_gather", _stream(), _p(data), _p(indices), _p(out), batch, slices,
              slice_elems * data.element_size(), indices.numel(), _p(flag))
    return out, flag


def cast(x, dtype):
    _chk(x)
    y = torch.empty(x.shape, dtype=dtype, device=x.device)
    capi.call("tnn_rocm_cast", _stream(), dt(x), _p(x), _DT[dtype], _p(y), x.numel())
    return y


def quantize(x, inv_scale):
    _chk(x)
    q = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    capi.call("tnn_rocm_quantize", _stream(), dt(x), _p(x), float(inv_scale), _p(q), x.numel())
    return q


def dequantize(q, scale, dtype=torch.float32):
    _chk(q)
    x = torch.empty(q.shape, dtype=dtype, device=q.device)
    capi.call("tnn_rocm_dequantize", _stream(), _p(q), float(scale), _DT[dtype], _p(x), q.numel())
    return x


def _channel_layout(t):
    channels = t.shape[1] if t.dim() >= 2 else 1
    inner = 1
    for d in t.shape[2:]:
        inner *= d
    return channels, inner


def quantize_per_channel(x, inv_scales):
    """x in the blob's own dims (axis 1 = channels); inv_scales: fp32 device tensor of x.shape[1] reciprocal scales"""
    _chk(x, inv_scales)
    q = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    channels, inner = _channel_layout(x)
    capi.call("tnn_rocm_quantize_per_channel", _stream(), dt(x), _p(x), _p(inv_scales), _p(q), x.numel(), channels, inner)
    return q


def dequantize_per_channel(q, scales, dtype=torch.float32):
    _chk(q, scales)
    x = torch.empty(q.shape, dtype=dtype, device=q.device)
    channels, inner = _channel_layout(q)
    capi.call("tnn_rocm_dequantize_per_channel", _stream(), _p(q), _p(scales), _DT[dtype], _p(x), q.numel(), channels, inner)
    return x


def add_i8(a, sa, b, sb, inv_so):
    """a, b in the blob's own dims: axis 1 is the channel axis the reference's loop walks."""
    _chk(a, b)
    y = torch.empty_like(a)
    channels = a.shape[1] if a.dim() >= 2 else 1
    inner = 1
    for d in a.shape[2:]:
        inner *= d
    capi.call("tnn_rocm_add_i8", _stream(), _p(a), float(sa), _p(b), float(sb), float(inv_so), _p(y), a.numel(),
              int(channels), max(int(inner), 1))
    return y


def gelu_i8(q, in_scale, out_inv_scale):
    _chk(q)
    y = torch.empty_like(q)
    capi.call("tnn_rocm_gelu_i8", _stream(), _p(q), float(in_scale), float(out_inv_scale), _p(y), q.numel())
    return y
