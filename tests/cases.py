"""Seeded synthetic inputs shaped like the benchmark configurations (reduced sizes where noted)."""
import numpy as np

F = np.float32


def conv_case(seed, c, h, w, outc, kernel, group=1, term=1, bias=True, int8_in=False, by_group=False, batch=1,
              w_sigma=0.05, x_range=(-1.0, 1.0)):
    """Weights N(0, w_sigma) quantised per output channel (or per group) with 127/absmax, input scale
    127/absmax(x), bias U(-0.1, 0.1): the single-layer configuration of the benchmark."""
    rng = np.random.default_rng(seed)
    kw, kh = kernel
    cg = c // group
    x = rng.uniform(x_range[0], x_range[1], (batch, c, h, w)).astype(F)
    wf = rng.normal(0, w_sigma, (outc, cg, kh, kw)).astype(F)
    if by_group:
        og = outc // group
        absmax = np.abs(wf.reshape(group, -1)).max(axis=1)
        w_scales = (F(127) / absmax).astype(F)
        wq = np.clip(np.round(wf.reshape(group, -1).astype(np.float64) * w_scales[:, None].astype(np.float64)), -127, 127)
        # the oracle's own quantiser is the authority; this is only input synthesis
        from oracle import oracle
        wq = oracle.quantize_weights(wf.reshape(group, og * cg * kh * kw), w_scales).reshape(outc, cg, kh, kw)
        n_as = group
    else:
        absmax = np.abs(wf.reshape(outc, -1)).max(axis=1)
        w_scales = (F(127) / absmax).astype(F)
        from oracle import oracle
        wq = oracle.quantize_weights(wf.reshape(outc, -1), w_scales).reshape(outc, cg, kh, kw)
        n_as = 1
    in_scales = np.full(n_as, F(127) / np.abs(x).max(), F)
    b = rng.uniform(-0.1, 0.1, outc).astype(F) if bias else None
    top_scales = None
    if term > 100:
        top_scales = np.full(n_as, F(127) / F(rng.uniform(2.0, 6.0)), F)
    if int8_in:
        from oracle import oracle
        x = oracle.quantize(x.reshape(batch * c, h * w), in_scales[:1]).reshape(batch, c, h, w)
    return x, wq, b, w_scales, in_scales, top_scales


def gemm_case(seed, m, n, k, per_col=False):
    from ncnn_amd import synth
    return synth.gemm_operands(seed, m, n, k, per_col)


def blockquant_case(seed, m, n, k, bits=8, block=64, half_exact=True):
    """bits == 8 comes from the benchmark's own generator and is cross-checked here against the packer that
    ncnn's test defines (restated in the oracle)."""
    from ncnn_amd import synth
    from oracle import oracle
    assert bits == 8
    a, packed, scales = synth.blockquant8_operands(seed, m, n, k, block, half_exact)
    return a, packed, scales


def mha_case(seed, embed_dim, num_heads, qdim, kdim, vdim, src, cur, bits, block, in_scales=False, past=0, self_attention=True, mask=None):
    """Inputs and block-quantised weights of one MultiHeadAttention call (src/layer/multiheadattention.cpp:119-200 for
    the weight order and shapes).  mask: None, "2d" or "3d" (additive, some entries -1e30 = masked out)."""
    from oracle import oracle
    rng = np.random.default_rng(seed)
    dims = [(embed_dim, qdim), (embed_dim, kdim), (embed_dim, vdim), (qdim, embed_dim)]
    weights = []
    for rows, k in dims:
        w = rng.normal(0, 1.0 / np.sqrt(k), (rows, k)).astype(np.float32)
        packed, scales = oracle.blockquant_pack(w, bits, block)
        ins = rng.uniform(0.5, 1.5, k).astype(np.float32) if in_scales else None
        weights.append((packed, scales, ins, rng.uniform(-0.1, 0.1, rows).astype(np.float32)))
    q = rng.normal(0, 1, (src, qdim)).astype(np.float32)
    k = q if (self_attention and kdim == qdim and cur == src) else rng.normal(0, 1, (cur, kdim)).astype(np.float32)
    v = k if vdim == kdim else rng.normal(0, 1, (cur, vdim)).astype(np.float32)
    ck = cv = None
    if past:
        ck = rng.normal(0, 1, (embed_dim, past)).astype(np.float32)
        cv = rng.normal(0, 1, (embed_dim, past)).astype(np.float32)
    dst = (past + cur if self_attention else past) if past else cur
    m = None
    if mask:
        shape = (src, dst) if mask == "2d" else (num_heads, src, dst)
        m = rng.normal(0, 1, shape).astype(np.float32)
        drop = rng.random(shape) < 0.25
        drop[..., 0] = False  # every row keeps one key
        m[drop] = np.float32(-1e30)
    return dict(q=q, k=k, v=v, weights=weights, embed_dim=embed_dim, num_heads=num_heads, scale=np.float32(1.0 / np.sqrt(embed_dim // num_heads)),
                bits=bits, block=block, mask=m, cached_k=ck, cached_v=cv, self_attention=self_attention)


MHA_CASES = [
    # seed, embed, heads, qdim, kdim, vdim, src, cur, bits, block, in_scales, past, self, mask
    (1, 64, 4, 64, 64, 64, 9, 9, 8, 64, False, 0, True, None),
    (2, 96, 3, 80, 72, 40, 7, 11, 4, 32, True, 0, True, "2d"),
    (3, 128, 8, 128, 128, 128, 5, 5, 6, 128, False, 0, True, "3d"),
    (4, 64, 2, 64, 64, 64, 1, 1, 8, 64, False, 13, True, None),    # one decode step appended to a cache
    (5, 64, 2, 48, 56, 56, 3, 4, 8, 32, True, 10, False, "2d"),    # cross attention on cached keys / values
    (6, 64, 4, 64, 64, 64, 40, 40, 8, 64, False, 0, True, None),   # 32 rows and more: the projections take the tiled kernel with its workspace
    (7, 128, 8, 128, 128, 128, 33, 33, 4, 32, True, 0, True, "2d"),
    (8, 64, 2, 64, 64, 64, 1, 1, 8, 64, False, 300, True, None),   # decode steps on a long cache: the few-query attention kernels
    (9, 96, 4, 96, 96, 96, 3, 3, 8, 32, False, 401, True, "2d"),
]
