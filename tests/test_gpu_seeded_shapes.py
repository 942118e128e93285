"""Seeded draws of shapes, activation-row counts and format mixes: GEMV within 1e-5 (relative L2, against the oracle's
double-precision sums) and dequantize bit-exact, through the C ABI.  The draws reach combinations the hand-picked
cases of the other files do not list (rows below the tile height, widths of 1 to 100 blocks, two to six formats per
tensor in any proportion, every uniform format at 1 to 17 activation rows)."""
import numpy as np
import pytest
import torch

import innova_amd as ia
import oracle as O
from gpu_util import gaussian_weights, rel_l2, to_orc_blocks

pytestmark = pytest.mark.gpu
TOL = 1e-5
ROWS = [1, 2, 3, 5, 8, 16, 17, 100, 257, 1000, 2049, 4100]
WIDTHS = [1, 2, 3, 5, 8, 16, 17, 24, 43, 56, 100]


def check(payload, blocks, rows, cols, X, tag):
    with ia.DeviceWeights.from_blocks(payload, blocks, rows, cols) as dw:
        got = dw.gemv(torch.from_numpy(X).cuda()).cpu().numpy()
        deq = dw.dequant().cpu().numpy()
    ob = to_orc_blocks(blocks)
    want = O.block_gemm(payload, ob, rows, cols, X, wide=True)
    assert rel_l2(got, want) <= TOL, tag
    assert np.array_equal(deq.view(np.uint32), O.dequant_blocks(payload, ob).view(np.uint32)), tag


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_seeded_format_mixes(seed):
    rng = np.random.default_rng(seed)
    for it in range(30):
        nf = int(rng.integers(2, 7))
        ids = rng.choice(15, size=nf, replace=False).astype(np.uint8)
        rows, cols, M = int(rng.choice(ROWS)), 256 * int(rng.choice(WIDTHS)), int(rng.choice([1, 1, 1, 2, 3, 4, 5, 7]))
        if rows * cols > 6e6:
            rows = max(1, int(6e6 // cols))
        fm = rng.choice(ids, size=rows * cols // 256, p=rng.dirichlet(np.ones(nf)))
        if fm.min() == fm.max():
            fm[0] = ids[0] if fm[0] != ids[0] else ids[1]
        payload, blocks = ia.block_codec.quantize_tensor(gaussian_weights(rows * cols, 2000 * seed + it, outlier_every=13), fm)
        X = rng.standard_normal((M, cols)).astype(np.float32)
        check(payload, blocks, rows, cols, X, (seed, it, list(ids), rows, cols, M))


@pytest.mark.parametrize("seed", [21, 22])
def test_seeded_uniform_formats(seed):
    rng = np.random.default_rng(seed)
    for it in range(30):
        fmt = ia.Format(it % 15)
        rows, cols, M = int(rng.choice(ROWS)), 256 * int(rng.choice(WIDTHS)), int(rng.choice([1, 1, 2, 3, 4, 5, 7, 9, 16, 17]))
        if rows * cols > 6e6:
            rows = max(1, int(6e6 // cols))
        payload, blocks = ia.block_codec.quantize_tensor(gaussian_weights(rows * cols, 3000 * seed + it, outlier_every=13), fmt)
        X = rng.standard_normal((M, cols)).astype(np.float32)
        check(payload, blocks, rows, cols, X, (seed, fmt.name, rows, cols, M))
