"""Independent numpy statement of the int8 arithmetic, used to pin the C oracle.

Deliberately written in a different shape from oracle/ncnn_int8_oracle.c (vectorised im2col +
int64 matmul, float64-based rounding, array-at-a-time float32 epilogues) so that an indexing,
sign or ordering mistake in either one shows up as a disagreement.
"""
import numpy as np

F = np.float32


def float2int8(v):
    v64 = np.asarray(v, dtype=np.float32).astype(np.float64)
    r = np.sign(v64) * np.floor(np.abs(v64) + 0.5)  # exact in binary64 for binary32 inputs
    return np.clip(r, -127, 127).astype(np.int8)


def activation(f, act_type, params=(0.0, 0.0)):
    f = np.asarray(f, dtype=np.float32)
    if act_type == 1:
        return np.maximum(f, F(0))
    if act_type == 2:
        return np.where(f > 0, f, f * F(params[0])).astype(np.float32)
    if act_type == 3:
        return np.minimum(np.maximum(f, F(params[0])), F(params[1]))
    if act_type == 6:
        a, b = F(params[0]), F(params[1])
        lower = F(-b / a)
        upper = F(F(1) / a) + lower
        mid = f * (f * a + b)
        return np.where(f < lower, F(0), np.where(f > upper, f, mid)).astype(np.float32)
    assert act_type == 0
    return f


def resolve_pads(w, h, kw, kh, dw, dh, sw, sh, pads):
    l, r, t, b = pads
    kew, keh = dw * (kw - 1) + 1, dh * (kh - 1) + 1
    if l > 0 or r > 0 or t > 0 or b > 0:
        return t, b, l, r
    if (l, r, t, b) in ((-233,) * 4, (-234,) * 4):
        wpad = kew + (w - 1) // sw * sw - w
        hpad = keh + (h - 1) // sh * sh - h
        if wpad > 0 or hpad > 0:
            if l == -233:
                return hpad // 2, hpad - hpad // 2, wpad // 2, wpad - wpad // 2
            return hpad - hpad // 2, hpad // 2, wpad - wpad // 2, wpad // 2
    return 0, 0, 0, 0


def im2col(xq, kw, kh, dw, dh, sw, sh, pads4, pad_byte=0):
    """xq int8 [c][h][w] -> int64 [c][kh][kw][oh][ow]."""
    t, b, l, r = pads4
    xp = np.pad(xq.astype(np.int64), ((0, 0), (t, b), (l, r)), constant_values=int(pad_byte))
    c, H, W = xp.shape
    oh = (H - (dh * (kh - 1) + 1)) // sh + 1
    ow = (W - (dw * (kw - 1) + 1)) // sw + 1
    cols = np.empty((c, kh, kw, oh, ow), np.int64)
    for ky in range(kh):
        for kx in range(kw):
            cols[:, ky, kx] = xp[:, ky * dh: ky * dh + (oh - 1) * sh + 1: sh, kx * dw: kx * dw + (ow - 1) * sw + 1: sw]
    return cols


def conv_family(x, weight, bias, w_scales, in_scales, top_scales, num_output, kernel, dilation=(1, 1), stride=(1, 1),
                pads=(0, 0, 0, 0), pad_value=0.0, group=1, term=1, act=0, act_params=(0.0, 0.0), scale_by_group=False):
    """Returns (out, acc).  Scales index: conv -> weight scale per output channel, activation scales [0];
    depthwise/group -> everything per group."""
    c, h, w = x.shape
    kw, kh = kernel
    cg, og = c // group, num_output // group
    in_scales = np.asarray(in_scales, np.float32).reshape(-1)
    w_scales = np.asarray(w_scales, np.float32).reshape(-1)
    if x.dtype == np.int8:
        xq = x
    else:
        per_ch = np.repeat(in_scales, cg) if scale_by_group else np.full(c, in_scales[0], np.float32)
        xq = float2int8(x.astype(np.float32) * per_ch[:, None, None])
    pads4 = resolve_pads(w, h, kw, kh, dilation[0], dilation[1], stride[0], stride[1], pads)
    cols = im2col(xq, kw, kh, dilation[0], dilation[1], stride[0], stride[1], pads4, np.int8(np.float32(pad_value)))
    oh, ow = cols.shape[-2:]
    wt = np.asarray(weight, np.int8).astype(np.int64).reshape(group, og, cg, kh, kw)
    colsg = cols.reshape(group, cg, kh, kw, oh, ow)
    acc = np.einsum("gpqyx,gqyxhw->gphw", wt, colsg).reshape(num_output, oh, ow)
    assert np.abs(acc).max(initial=0) < 2 ** 31
    p = np.arange(num_output)
    wsi = p // og if scale_by_group else p
    asi = p // og if scale_by_group else np.zeros(num_output, np.int64)
    prod = in_scales[asi] * w_scales[wsi]  # float32 * float32
    with np.errstate(divide="ignore"):
        scale_in = np.where(w_scales[wsi] == 0, F(0), F(1) / prod).astype(np.float32)
    f = acc.astype(np.float32) * scale_in[:, None, None]
    if bias is not None:
        f = f + np.asarray(bias, np.float32)[:, None, None]
    f = activation(f, act, act_params)
    if term > 100:
        ts = np.asarray(top_scales, np.float32).reshape(-1)[asi]
        return float2int8(f * ts[:, None, None]), acc.astype(np.int32)
    return f.astype(np.float32), acc.astype(np.int32)


def innerproduct(x, weight, bias, w_scales, in_scale, act=0, act_params=(0.0, 0.0)):
    xq = x if x.dtype == np.int8 else float2int8(x.astype(np.float32) * F(in_scale))
    acc = xq.astype(np.int64) @ np.asarray(weight, np.int8).astype(np.int64).T
    w_scales = np.asarray(w_scales, np.float32)
    with np.errstate(divide="ignore"):
        scale_in = np.where(w_scales == 0, F(0), F(1) / (F(in_scale) * w_scales)).astype(np.float32)
    f = acc.astype(np.float32) * scale_in[None, :]
    if bias is not None:
        f = f + np.asarray(bias, np.float32)[None, :]
    return activation(f, act, act_params).astype(np.float32), acc.astype(np.int32)


def gemm_quantize_rows(a):
    a = np.asarray(a, np.float32)
    absmax = np.abs(a).max(axis=1)
    with np.errstate(divide="ignore"):
        s = np.where(absmax == 0, F(1), F(127) / absmax).astype(np.float32)
    return float2int8(a * s[:, None]), s


def gemm_acc_exact(aq, bq):
    """int8 x int8 accumulators through a float64 BLAS matmul: every partial sum is an integer below 127*127*K < 2^53,
    so no rounding happens whatever the summation order (fast enough for the 4096-cube benchmark size)."""
    assert aq.shape[1] * 127 * 127 < 2 ** 53
    return (aq.astype(np.float64) @ bq.astype(np.float64).T).astype(np.int64)


def gemm_int8(aq, bq, a_scales, b_scales, c=None, bt=-1, alpha=1.0, beta=1.0, transpose=False, acc=None):
    if acc is None:
        acc = aq.astype(np.int64) @ bq.astype(np.int64).T
    m, n = acc.shape
    a_scales = np.asarray(a_scales, np.float32)
    b_scales = np.asarray(b_scales, np.float32).reshape(-1)
    if b_scales.size == 1:
        descale = (F(1) / (a_scales[:, None] * b_scales[:1][None, :])).astype(np.float32)
        f = acc.astype(np.float32) * descale
    else:  # per-column generalisation: (acc * 1/sA_i) * 1/sB_j
        f = (acc.astype(np.float32) * (F(1) / a_scales)[:, None]).astype(np.float32) * (F(1) / b_scales)[None, :]
    if c is not None and bt >= 0:
        c = np.asarray(c, np.float32)
        cv = {0: lambda: c.reshape(-1)[0], 1: lambda: c.reshape(m, 1), 2: lambda: c.reshape(m, 1),
              3: lambda: c.reshape(m, n), 4: lambda: c.reshape(1, n)}[bt]()
        f = f + cv * F(beta)
    f = (f * F(alpha)).astype(np.float32)
    return (f.T.copy() if transpose else f), acc.astype(np.int32)


def blockquant_unpack_all(packed, k, bits):
    """uint8 [n][ceil(k*bits/8)] -> int [n][k] (LSB-first bit stream, two's complement fields)."""
    bitsarr = np.unpackbits(packed, axis=1, bitorder="little")[:, : k * bits].reshape(packed.shape[0], k, bits)
    vals = (bitsarr.astype(np.int64) << np.arange(bits)).sum(axis=2)
    return np.where(vals >= (1 << (bits - 1)), vals - (1 << bits), vals)


def blockquant_gemm_f64(a, packed, scales, bits, block, in_scales=None, c=None, bt=-1, alpha=1.0, beta=1.0):
    """float64 value of the block-quant gemm and the magnitude floor sum |a*w| used for tolerances."""
    a = np.asarray(a, np.float32)
    m, k = a.shape
    q = blockquant_unpack_all(packed, k, bits)
    descale = (F(1) / np.asarray(scales, np.float32)).astype(np.float32)
    wdq = (q.astype(np.float32) * np.repeat(descale, block, axis=1)[:, :k]).astype(np.float32)  # q*descale in f32
    av = a if in_scales is None else (a * np.asarray(in_scales, np.float32)[None, :]).astype(np.float32)
    val = av.astype(np.float64) @ wdq.astype(np.float64).T
    floor = np.abs(av).astype(np.float64) @ np.abs(wdq).astype(np.float64).T
    n = packed.shape[0]
    if c is not None and bt >= 0:
        c = np.asarray(c, np.float64)
        cv = {0: lambda: c.reshape(-1)[0], 1: lambda: c.reshape(m, 1), 2: lambda: c.reshape(m, 1),
              3: lambda: c.reshape(m, n), 4: lambda: c.reshape(1, n)}[bt]()
        val = val + cv * float(np.float32(beta))
        floor = floor + np.abs(cv * float(np.float32(beta)))
    return val * float(np.float32(alpha)), floor * abs(float(np.float32(alpha)))


def blockquant_dequantise(packed, scales, k, bits, block):
    """The fp32 weight values q * (1/scale) the block-quantised layers multiply with, [n][k]."""
    q = blockquant_unpack_all(packed, k, bits)
    descale = (F(1) / np.asarray(scales, np.float32)).astype(np.float32)
    return (q.astype(np.float32) * np.repeat(descale, block, axis=1)[:, :k]).astype(np.float32)


def mha_f64(q, k, v, weights, embed_dim, num_heads, scale, bits, block, mask=None, cached_k=None, cached_v=None, self_attention=True):
    """float64 softmax(q k^T * scale + mask) v with dequantised weights; the textbook formulation, batch-free.
    weights: 4 x (packed, scales, in_scales or None, bias).  Returns (out [src][qdim], k [embed][dst], v [embed][dst])."""
    def proj(x, w):
        packed, scales, ins, bias = w
        x = np.asarray(x, np.float64)
        wd = blockquant_dequantise(packed, scales, x.shape[1], bits, block).astype(np.float64)
        if ins is not None:
            x = x * np.asarray(ins, np.float64)[None, :]
        return x @ wd.T + np.asarray(bias, np.float64)[None, :]

    qa = proj(q, weights[0]) * float(np.float32(scale))
    past = 0 if cached_k is None else cached_k.shape[1]
    if past > 0 and not self_attention:
        ka, va = np.asarray(cached_k, np.float64).T, np.asarray(cached_v, np.float64).T
    else:
        ka, va = proj(k, weights[1]), proj(v, weights[2])
        if past > 0:
            ka = np.concatenate([np.asarray(cached_k, np.float64).T, ka])
            va = np.concatenate([np.asarray(cached_v, np.float64).T, va])
    hd = embed_dim // num_heads
    ctx = np.empty((qa.shape[0], embed_dim))
    for h in range(num_heads):
        sl = slice(h * hd, (h + 1) * hd)
        s = qa[:, sl] @ ka[:, sl].T
        if mask is not None:
            s = s + np.asarray(mask if mask.ndim == 2 else mask[h], np.float64)
        s = np.exp(s - s.max(axis=1, keepdims=True))
        s = s / s.sum(axis=1, keepdims=True)
        ctx[:, sl] = s @ va[:, sl]
    return proj(ctx, weights[3]), ka.T, va.T
