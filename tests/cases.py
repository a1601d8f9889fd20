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
