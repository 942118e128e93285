"""Prefill GEMM through the C ABI (oilhip_gemm_bf16): bf16 activations, OIL4 weights
dequantized to bf16 in LDS, MFMA with FP32 accumulation.

Tolerance (north star): relative L2 error <= 2e-3 against the FP32/double oracle
(double-precision dot of the bit-exact decoded weights with the same bf16 inputs)."""
import numpy as np
import pytest
import torch

import innova_amd as ia
import oracle as O
from gpu_util import gaussian_weights, rel_l2, to_orc_blocks

pytestmark = pytest.mark.gpu
TOL = 2e-3


def run(rows, cols, M, seed, sample_rows=None):
    w = gaussian_weights(rows * cols, seed, outlier_every=29)
    payload, blocks = ia.block_codec.quantize_tensor(w, ia.Format.OIL4)
    xb = torch.randn(M, cols, generator=torch.Generator().manual_seed(seed)).to(torch.bfloat16)
    with ia.DeviceWeights.from_blocks(payload, blocks, rows, cols) as dw:
        y = dw.gemm_bf16(xb.cuda()).cpu().numpy()
    X = xb.to(torch.float32).numpy()
    ob = to_orc_blocks(blocks)
    if sample_rows is None:
        want = O.block_gemm(payload, ob, rows, cols, X, wide=True)
        return rel_l2(y, want), y, want
    sel = np.unique(np.concatenate([np.arange(0, rows, max(1, rows // sample_rows)), np.arange(rows - 4, rows)]))
    bpr = cols // 256
    want = O.block_gemm(payload, ob.reshape(rows, bpr)[sel].reshape(-1), sel.size, cols, X, wide=True)
    return rel_l2(y[:, sel], want), y, want


@pytest.mark.parametrize("rows,cols,M", [(128, 256, 128), (256, 512, 64), (130, 768, 33), (1, 256, 1),
                                          (384, 1024, 300), (512, 2048, 512), (77, 256, 257)])
def test_small_shapes(rows, cols, M):
    err, y, want = run(rows, cols, M, seed=rows + cols + M)
    assert y.shape == (M, rows)
    assert err <= TOL


def test_layout_is_not_transposed():
    """Distinct M, N, K and a single hot activation column / weight row pin the index maps."""
    rows, cols, M = 96, 512, 40
    w = np.zeros(rows * cols, dtype=np.float32)
    w[5 * cols + 300] = 1.0                      # W[5][300]
    w[17 * cols + 64] = -2.0                     # W[17][64] (first weight after a slot)
    payload, blocks = ia.block_codec.quantize_tensor(w, ia.Format.OIL4)
    x = torch.zeros(M, cols, dtype=torch.bfloat16)
    x[3, 300] = 1.0
    x[9, 64] = 0.5
    with ia.DeviceWeights.from_blocks(payload, blocks, rows, cols) as dw:
        y = dw.gemm_bf16(x.cuda()).cpu().numpy()
        deq = dw.dequant().cpu().numpy().reshape(rows, cols)
    want = x.to(torch.float32).numpy().astype(np.float64) @ deq.astype(np.float64).T
    assert rel_l2(y, want) <= TOL
    assert abs(y[3, 5]) > 0 and abs(y[9, 17]) > 0 and np.count_nonzero(np.abs(y) > 1e-12) <= 2 * 96


@pytest.mark.parametrize("rows,cols", [(4096, 4096), (11008, 4096)])
@pytest.mark.parametrize("M", [512, 2048])
def test_config_shapes(rows, cols, M):
    err, y, _ = run(rows, cols, M, seed=M + rows, sample_rows=96)
    assert err <= TOL
    assert np.all(np.isfinite(y))


def test_rejects_non_oil4():
    w = gaussian_weights(256 * 4, 1)
    payload, blocks = ia.block_codec.quantize_tensor(w, ia.Format.OIL8)
    with ia.DeviceWeights.from_blocks(payload, blocks, 4, 256) as dw:
        with pytest.raises(ia.OilHipError):
            dw.gemm_bf16(torch.zeros(2, 256, dtype=torch.bfloat16, device="cuda"))
