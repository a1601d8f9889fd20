"""MultiHeadAttention with block-quantised weights at seeded random arrangements, through load_param / load_model /
extract in both execution modes, against the oracle (src/layer/multiheadattention.cpp:186-560 with the block-quantised
projections of src/layer/gemm.cpp:339-483): heads and head sizes, q / k / v widths, query and key counts, self and cross
attention, shared / per-head / no mask, a cache of 1 to 500 positions in and out, every weight layout.  Tolerances as in
the listed cases of test_gpu_net.py (2e-5 of the largest output, 1e-5 for the caches)."""
import os

import numpy as np
import pytest

import test_gpu_net as listed

pytestmark = pytest.mark.gpu
COUNT = int(os.environ.get("NCNN_RANDOM_LAYERS", "60"))  # NCNN_RANDOM_LAYERS=<count> widens the walk


def _pick(rng, options):
    return options[int(rng.integers(len(options)))]


@pytest.mark.parametrize("resident", [False, True], ids=["host-blobs", "device-resident"])
@pytest.mark.parametrize("seed", range(COUNT))
def test_random_multiheadattention_layer_matches_oracle(seed, resident):
    rng = np.random.default_rng(17000 + seed)
    heads, head_dim = _pick(rng, [1, 2, 3, 4, 8]), _pick(rng, [8, 16, 24, 32, 64])
    embed = heads * head_dim
    # the layer tells self attention from cross attention by its blobs: one blob is q = k = v; else k (and v, when its width
    # differs from k's) come as blobs of their own
    self_att = rng.random() < 0.55
    qdim = 8 * int(rng.integers(2, 18))
    kdim = qdim if self_att else 8 * int(rng.integers(2, 18))
    vdim = kdim if (self_att or rng.random() < 0.5) else 8 * int(rng.integers(2, 18))
    src = _pick(rng, [1, 1, 2, 3, 5, 9, 17, 33, 40, 50])
    cur = src if self_att else int(rng.integers(1, 51))
    if not self_att and kdim == qdim and cur == src:
        cur += 1  # (the case builder would hand q over as k)
    bits, block = _pick(rng, [8, 8, 4, 6]), _pick(rng, [64, 64, 32, 128])
    past = _pick(rng, [0, 0, 0, int(rng.integers(1, 41)), int(rng.integers(100, 501))])
    mask = _pick(rng, [None, None, "2d", "3d"])
    spec = (1000 + seed, embed, heads, qdim, kdim, vdim, src, cur, bits, block, bool(rng.integers(2)), past, self_att, mask)
    print("[case] random multi-head attention", seed, "resident" if resident else "host", spec, flush=True)
    listed.test_multiheadattention_layer_block_quant(spec, resident)
