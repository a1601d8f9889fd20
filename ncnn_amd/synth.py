"""Seeded synthetic operands of the benchmark configurations (numpy only, no checker code involved)."""
import numpy as np

F = np.float32


def _round_half_away(v):
    v = np.asarray(v, np.float64)
    return np.sign(v) * np.floor(np.abs(v) + 0.5)


def gemm_operands(seed, m, n, k, per_col=False):
    """A fp32 N(0,1); constant B fp32 N(0,0.02) quantised to int8 with 127/absmax per column of the
    product (= per row of B[N][K]) or per tensor; fp32 bias [N]."""
    rng = np.random.default_rng(seed)
    a = rng.standard_normal((m, k), dtype=F)
    b = (rng.standard_normal((n, k), dtype=F) * F(0.02)).astype(F)
    if per_col:
        sb = (F(127) / np.abs(b).max(axis=1)).astype(F)
        bq = np.clip(_round_half_away(b * sb[:, None]), -127, 127).astype(np.int8)
    else:
        sb = np.array([F(127) / np.abs(b).max()], F)
        bq = np.clip(_round_half_away(b * sb[0]), -127, 127).astype(np.int8)
    bias = rng.standard_normal(n, dtype=F)
    return a, bq, sb, bias


def blockquant8_operands(seed, m, n, k, block=64, half_exact=True):
    """Activations N(0,1) (rounded to fp16-representable values by default), weights N(0,0.02) quantised to
    int8 in blocks of `block` along K; scales are stored the way the .bin holds them (127/absmax, fp32)."""
    rng = np.random.default_rng(seed)
    a = rng.standard_normal((m, k), dtype=F)
    if half_exact:
        a = a.astype(np.float16).astype(F)
    w = (rng.standard_normal((n, k), dtype=F) * F(0.02)).astype(F)
    nblk = (k + block - 1) // block
    pad = nblk * block - k
    wp = np.pad(w, ((0, 0), (0, pad))).reshape(n, nblk, block)
    absmax = np.abs(wp).max(axis=2)
    with np.errstate(divide="ignore"):
        scales = np.where(absmax == 0, F(1), F(127) / absmax).astype(F)
    q = np.clip(_round_half_away((wp * scales[:, :, None]).astype(F)), -127, 127).astype(np.int8)
    packed = q.reshape(n, nblk * block)[:, :k].copy().view(np.uint8)
    return a, packed, scales


def blockquant_weights(w, bits, block):
    """fp32 [n][k] -> (packed uint8 [n][ceil(k*bits/8)], scales fp32 [n][ceil(k/block)]) in the .bin layout of the
    block-quantised layers: scale = qmax/absmax per block (1 for an all-zero block), q = clamp(round_half_away(w*scale)),
    fields of `bits` bits, two's complement, LSB first along K (src/layer/gemm.cpp:318-336; the packer of
    tests/test_gemm_block_quant.cpp:80-129)."""
    w = np.asarray(w, F)
    n, k = w.shape
    qmax = (1 << (bits - 1)) - 1
    nblk = (k + block - 1) // block
    wp = np.pad(w, ((0, 0), (0, nblk * block - k))).reshape(n, nblk, block)
    absmax = np.abs(wp).max(axis=2)
    with np.errstate(divide="ignore"):
        scales = np.where(absmax == 0, F(1), F(qmax) / absmax).astype(F)
    q = np.clip(_round_half_away((wp * scales[:, :, None]).astype(F)), -qmax, qmax).astype(np.int64).reshape(n, nblk * block)[:, :k]
    if bits == 8:
        return q.astype(np.int8).view(np.uint8).copy(), scales
    fields = (q & ((1 << bits) - 1)).astype(np.uint8)
    stream = ((fields[:, :, None] >> np.arange(bits, dtype=np.uint8)) & 1).reshape(n, k * bits)
    return np.packbits(stream, axis=1, bitorder="little"), scales


def blockquant_operands(seed, m, n, k, bits=8, block=64, half_exact=True):
    """Activations N(0,1) (fp16-representable by default) and N(0,0.02) weights block-quantised to `bits` bits."""
    if bits == 8:
        return blockquant8_operands(seed, m, n, k, block, half_exact)
    rng = np.random.default_rng(seed)
    a = rng.standard_normal((m, k), dtype=F)
    if half_exact:
        a = a.astype(np.float16).astype(F)
    packed, scales = blockquant_weights((rng.standard_normal((n, k), dtype=F) * F(0.02)).astype(F), bits, block)
    return a, packed, scales
