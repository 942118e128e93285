"""Decode-step pieces around the quantized matmuls (Qwen35Engine::rmsnorm / mlp_step / embedding lookup) on the
device against the CPU oracle; closed forms in double precision pin the oracle's two formulas here as well."""
import numpy as np
import pytest
import torch

import innova_amd as ia
import oracle as O
from gpu_util import gaussian_weights, rel_l2, to_orc_blocks
from innova_amd import layers

pytestmark = pytest.mark.gpu
TOL = 1e-5


def test_rmsnorm():
    rng = np.random.default_rng(0)
    for rows, n in [(1, 4096), (3, 1000), (2, 7), (2, 16384), (1, 20480), (2, 4100)]:
        x = rng.standard_normal((rows, n)).astype(np.float32)
        w = (rng.standard_normal(n) * 0.1).astype(np.float32)
        got = layers.rmsnorm(torch.from_numpy(x).cuda(), torch.from_numpy(w).cuda()).cpu().numpy()
        want = O.rmsnorm(x, w)
        x64 = x.astype(np.float64)
        closed = x64 / np.sqrt((x64 ** 2).mean(1, keepdims=True) + 1e-6) * (1.0 + w.astype(np.float64))
        assert rel_l2(want, closed) <= 1e-6          # the oracle is the textbook formula
        assert rel_l2(got, closed) <= 1e-6
        assert np.abs(got - want).max() <= 4e-6 * np.abs(want).max()


def block_formats(fmt, nblocks, seed):
    """A Format for a uniform tensor, or a tuple of format ids drawn per block (a tensor whose rows mix formats)."""
    if not isinstance(fmt, tuple):
        return fmt
    return np.random.default_rng(seed).choice(np.array(fmt, dtype=np.uint8), size=nblocks)


# OIL4 and window-stream tensors (mixed rows, other uniform formats) fuse the input transforms into one-row launches;
# OIL8 and several activation rows take the separate kernels
@pytest.mark.parametrize("M,D,F,fmt", [(1, 512, 768, ia.Format.OIL4), (1, 4096, 11008, ia.Format.OIL4),
                                        (3, 512, 768, ia.Format.OIL4), (1, 256, 512, ia.Format.OIL8),
                                        (1, 1024, 2816, (0, 1)), (1, 512, 768, ia.Format.SPARK_Q0),
                                        (2, 512, 768, (0, 1, 3))])
def test_mlp_step(M, D, F, fmt):
    rng = np.random.default_rng(D + F + M)
    mats = {}
    for name, (r, c) in (("gate", (F, D)), ("up", (F, D)), ("down", (D, F))):
        w = gaussian_weights(r * c, seed=len(name) + D) * np.float32(50.0 / np.sqrt(c))
        mats[name] = (r, c) + ia.block_codec.quantize_tensor(w, block_formats(fmt, r * c // 256, len(name)))
    x = rng.standard_normal((M, D)).astype(np.float32)
    dev = {k: ia.DeviceWeights.from_blocks(v[2], v[3], v[0], v[1]) for k, v in mats.items()}
    gu = ia.DeviceWeights.stack_rows([dev["gate"], dev["up"]])
    assert (gu.rows, gu.cols) == (2 * F, D)
    assert gu.info()["payload_bytes"] == dev["gate"].info()["payload_bytes"] + dev["up"].info()["payload_bytes"]
    got = layers.mlp_step(gu, dev["down"], torch.from_numpy(x).cuda()).cpu().numpy()
    # oracle: the reference's steps with the matmuls in double precision
    g = O.block_gemm(mats["gate"][2], to_orc_blocks(mats["gate"][3]), F, D, x, wide=True)
    u = O.block_gemm(mats["up"][2], to_orc_blocks(mats["up"][3]), F, D, x, wide=True)
    h = O.swiglu(g.astype(np.float32), u.astype(np.float32))
    g64 = g.astype(np.float64)
    assert rel_l2(h, g64 / (1.0 + np.exp(-g64)) * u) <= 1e-6      # siluf(g) * u in closed form
    want = O.block_gemm(mats["down"][2], to_orc_blocks(mats["down"][3]), D, F, h, wide=True)
    assert rel_l2(got, want) <= TOL
    # the stacked tensor alone is the two GEMVs side by side
    y2 = gu.gemv(torch.from_numpy(x).cuda()).cpu().numpy()
    assert rel_l2(y2[:, :F], g) <= TOL and rel_l2(y2[:, F:], u) <= TOL
    for d in list(dev.values()) + [gu]:
        d.close()


@pytest.mark.parametrize("M,rows,cols,fmt", [(1, 768, 512, ia.Format.OIL4), (1, 12288, 4096, ia.Format.OIL4),
                                              (1, 300, 11008, ia.Format.OIL4), (3, 768, 512, ia.Format.OIL4),
                                              (1, 256, 512, ia.Format.OIL8), (1, 1000, 4096, (0, 1)),
                                              (1, 300, 2816, (0, 1, 3, 10)), (1, 5000, 1024, ia.Format.OIL2_GRP),
                                              (2, 300, 1024, (0, 1))])
def test_gemv_rmsnorm(M, rows, cols, fmt):
    """W . rmsnorm(x): one launch for one row of an OIL4 or window-stream tensor, norm kernel + GEMV otherwise; both
    against the oracle's two steps."""
    rng = np.random.default_rng(rows + cols + M)
    payload, blocks = ia.block_codec.quantize_tensor(gaussian_weights(rows * cols, seed=rows),
                                                     block_formats(fmt, rows * cols // 256, rows))
    x = (rng.standard_normal((M, cols)) * 3.0).astype(np.float32)
    nw = (rng.standard_normal(cols) * 0.2).astype(np.float32)
    dw = ia.DeviceWeights.from_blocks(payload, blocks, rows, cols)
    got = layers.gemv_rmsnorm(dw, torch.from_numpy(x).cuda(), torch.from_numpy(nw).cuda()).cpu().numpy()
    want = O.block_gemm(payload, to_orc_blocks(blocks), rows, cols, O.rmsnorm(x, nw), wide=True)
    assert rel_l2(got, want) <= TOL
    dw.close()


@pytest.mark.parametrize("fmt", [ia.Format.OIL4, (0, 1)])
def test_mlp_step_with_norm(fmt):
    M, D, F = 1, 1024, 2816
    rng = np.random.default_rng(9)
    mats = {}
    for name, (r, c) in (("gate", (F, D)), ("up", (F, D)), ("down", (D, F))):
        w = gaussian_weights(r * c, seed=len(name) + D) * np.float32(50.0 / np.sqrt(c))
        mats[name] = (r, c) + ia.block_codec.quantize_tensor(w, block_formats(fmt, r * c // 256, len(name)))
    x = (rng.standard_normal((M, D)) * 2.0).astype(np.float32)
    nw = (rng.standard_normal(D) * 0.2).astype(np.float32)
    dev = {k: ia.DeviceWeights.from_blocks(v[2], v[3], v[0], v[1]) for k, v in mats.items()}
    gu = ia.DeviceWeights.stack_rows([dev["gate"], dev["up"]])
    for m_rows in (1, 2):
        xm = np.repeat(x, m_rows, axis=0) * np.arange(1, m_rows + 1, dtype=np.float32)[:, None]
        got = layers.mlp_step(gu, dev["down"], torch.from_numpy(xm).cuda(), norm_w=torch.from_numpy(nw).cuda()).cpu().numpy()
        xn = O.rmsnorm(xm, nw)
        g = O.block_gemm(mats["gate"][2], to_orc_blocks(mats["gate"][3]), F, D, xn, wide=True)
        u = O.block_gemm(mats["up"][2], to_orc_blocks(mats["up"][3]), F, D, xn, wide=True)
        h = O.swiglu(g.astype(np.float32), u.astype(np.float32))
        want = O.block_gemm(mats["down"][2], to_orc_blocks(mats["down"][3]), D, F, h, wide=True)
        assert rel_l2(got, want) <= TOL
    for d in list(dev.values()) + [gu]:
        d.close()


def test_embed_rows():
    vocab, cols = 40, 1024
    w = gaussian_weights(vocab * cols, 5)
    fmts = (np.arange(vocab * cols // 256) % 15).astype(np.uint8)
    payload, blocks = ia.block_codec.quantize_tensor(w, fmts)
    dense = O.dequant_blocks(payload, to_orc_blocks(blocks)).reshape(vocab, cols)
    ids = np.array([3, 0, 39, 3, -1, 40], np.int32)
    with ia.DeviceWeights.from_blocks(payload, blocks, vocab, cols) as dw:
        got = layers.embed_rows(dw, torch.from_numpy(ids).cuda()).cpu().numpy()
    for k, i in enumerate(ids):
        want = dense[i] if 0 <= i < vocab else np.zeros(cols, np.float32)
        assert np.array_equal(got[k].view(np.uint32), want.view(np.uint32)), k


def test_stack_rows_rejects_mismatched_parts():
    a = ia.DeviceWeights.quantize(gaussian_weights(4 * 512, 1), ia.Format.OIL4, 4, 512)
    b = ia.DeviceWeights.quantize(gaussian_weights(4 * 256, 2), ia.Format.OIL4, 4, 256)
    with pytest.raises(ia.OilHipError):
        ia.DeviceWeights.stack_rows([a, b])


def test_stack_rows_of_mixed_and_different_formats():
    """Parts that mix formats, or differ in format, stack into one mixed tensor: GEMV and dequantization of the
    stack equal those of the parts one after the other."""
    rng = np.random.default_rng(12)
    cols, parts, ys, dq = 1024, [], [], []
    X = rng.standard_normal((2, cols)).astype(np.float32)
    for i, (rows, fm) in enumerate([(9, (0, 1)), (5, (3,)), (14, (0, 1, 10))]):
        w = gaussian_weights(rows * cols, 40 + i)
        fmts = rng.choice(np.array(fm, dtype=np.uint8), size=rows * cols // 256)
        payload, blocks = ia.block_codec.quantize_tensor(w, fmts)
        parts.append(ia.DeviceWeights.from_blocks(payload, blocks, rows, cols))
        ys.append(O.block_gemm(payload, to_orc_blocks(blocks), rows, cols, X, wide=True))
        dq.append(O.dequant_blocks(payload, to_orc_blocks(blocks)))
    with ia.DeviceWeights.stack_rows(parts) as st:
        info = st.info()
        assert info["rows"] == 28 and info["uniform_fmt"] == -1
        # stored as window streams: block bytes plus tags and window headers, never less than the payload
        assert info["payload_bytes"] <= info["stored_bytes"] <= 2 * info["payload_bytes"] + 4096
        assert info["descriptor_bytes"] == 16 * info["nblocks"]
        got = st.gemv(torch.from_numpy(X).cuda()).cpu().numpy()
        deq = st.dequant().cpu().numpy()
    assert rel_l2(got, np.concatenate(ys, axis=1)) <= 1e-5
    assert np.array_equal(deq.view(np.uint32), np.concatenate(dq).view(np.uint32))
    for p in parts:
        p.close()
