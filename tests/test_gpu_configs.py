"""The benchmark configurations at their full sizes, HIP path against the CPU oracle.

* the 1.50-bpw layer stack: seven Llama-7B-shaped matrices, weights N(0, 0.02) with 1 % of the blocks scaled x8,
  formats from FormatPlanner(1.50) after score_importance (src/format_planner.cpp:12-37, 133-315), decode GEMV at M = 1,
  alone, stacked (q/k/v, gate/up) and through the fused RMSNorm / SwiGLU launches;
* the mixture-of-experts step: 8 OIL4 experts 4096 <-> 14336, 64 tokens, top-2 with an uneven load
  (moe_dispatch_batched, src/moe_variants.cpp:767-827);
* the output head: OIL4 at 248,320 x 4096 (M = 1) and 131,072 x 4096 (M = 16)
  (src/adapters/tools/qwen35_engine.cpp:624-627).

Bars: dequantized weights bit for bit, FP32 outputs within relative L2 1e-5 of the oracle's double-precision sums.
Where the oracle would take minutes it runs on a row sample and linearity covers the rest of the rows."""
import numpy as np
import pytest
import torch

import innova_amd as ia
import oracle as O
from gpu_util import rel_l2, to_orc_blocks
from innova_amd import layers, moe
from innova_amd.format_planner import FormatPlanner

pytestmark = pytest.mark.gpu
TOL = 1e-5

STACK = [("q", 4096, 4096), ("k", 4096, 4096), ("v", 4096, 4096), ("o", 4096, 4096),
         ("gate", 11008, 4096), ("up", 11008, 4096), ("down", 4096, 11008)]


def planned_matrix(name, rows, cols):
    """N(0, 0.02) weights, 1 % of the blocks x8, routed by the planner at 1.50 bpw, quantized by the host codec."""
    seed = 9000 + sum(map(ord, name))
    rng = np.random.default_rng(seed)
    w = rng.standard_normal(rows * cols, dtype=np.float32) * np.float32(0.02)
    nb = rows * cols // 256
    hot = rng.choice(nb, nb // 100, replace=False)
    w.reshape(nb, 256)[hot] *= np.float32(8.0)
    pl = FormatPlanner(1.50)
    pl.score_importance(w)
    plan = pl.allocate(nb)
    payload, blocks = ia.block_codec.quantize_tensor(w, plan.formats)
    return plan, payload, blocks


def sample_rows(rows, step=64, tail=8):
    return np.unique(np.concatenate([np.arange(0, rows, step), np.arange(rows - tail, rows)]))


def oracle_rows(payload, blocks, rows, cols, sel, X):
    ob = to_orc_blocks(blocks).reshape(rows, cols // 256)[sel].reshape(-1)
    return O.block_gemm(payload, ob, sel.size, cols, X, wide=True)


@pytest.fixture(scope="module")
def stack():
    return {name: (rows, cols) + planned_matrix(name, rows, cols) for name, rows, cols in STACK}


@pytest.mark.parametrize("name", [n for n, _, _ in STACK])
def test_planner_stack_matrix(stack, name):
    rows, cols, plan, payload, blocks = stack[name]
    nb = rows * cols // 256
    # the planner's answer at 1.50: the more important half SPARK_Q0, the rest OIL1 (src/format_planner.cpp:89-92, 281-304)
    counts = np.bincount(plan.formats, minlength=15)
    assert counts[int(ia.Format.SPARK_Q0)] + counts[int(ia.Format.OIL1)] == nb
    assert abs(int(counts[int(ia.Format.SPARK_Q0)]) - nb // 2) <= 1
    rng = np.random.default_rng(rows + cols)
    X = rng.standard_normal((1, cols)).astype(np.float32)
    X2 = rng.standard_normal((1, cols)).astype(np.float32)
    with ia.DeviceWeights.from_blocks(payload, blocks, rows, cols) as dw:
        xd, xd2 = torch.from_numpy(X).cuda(), torch.from_numpy(X2).cuda()
        y = dw.gemv(xd).cpu().numpy()
        y2 = dw.gemv(xd2).cpu().numpy()
        ysum = dw.gemv(xd + xd2).cpu().numpy()
        ygen = dw.gemv(xd, general=True).cpu().numpy()
        deq = dw.dequant().cpu().numpy().reshape(nb, 256)
    sel = sample_rows(rows)
    assert rel_l2(y[:, sel], oracle_rows(payload, blocks, rows, cols, sel, X)) <= TOL
    assert rel_l2(ysum, y + y2) <= TOL                      # every row, through linearity
    assert rel_l2(y, ygen) <= TOL                           # ... and against the per-weight kernel
    # dequantized weights, bit for bit, on a sampled block set (every 509th block and the last ones)
    bsel = np.unique(np.concatenate([np.arange(0, nb, 509), np.arange(nb - 16, nb)]))
    want = O.dequant_blocks(payload, to_orc_blocks(blocks)[bsel]).reshape(bsel.size, 256)
    assert np.array_equal(deq[bsel].view(np.uint32), want.view(np.uint32))


def test_planner_stack_stacked_and_fused(stack):
    """q/k/v and gate/up stacked into one tensor each, and the layer as the decode step runs it: RMSNorm inside the
    q/k/v and gate/up launches, SwiGLU inside the down projection's."""
    D, F = 4096, 11008
    rng = np.random.default_rng(77)
    x = rng.standard_normal((1, D)).astype(np.float32)
    wn = (rng.standard_normal(D) * 0.1).astype(np.float32)
    dws = {n: ia.DeviceWeights.from_blocks(stack[n][3], stack[n][4], stack[n][0], stack[n][1]) for n in stack}
    qkv = ia.DeviceWeights.stack_rows([dws["q"], dws["k"], dws["v"]])
    gu = ia.DeviceWeights.stack_rows([dws["gate"], dws["up"]])
    xd, wd = torch.from_numpy(x).cuda(), torch.from_numpy(wn).cuda()
    try:
        y_qkv = qkv.gemv(xd).cpu().numpy()
        parts = np.concatenate([dws[n].gemv(xd).cpu().numpy() for n in ("q", "k", "v")], axis=1)
        assert rel_l2(y_qkv, parts) <= TOL
        # stacked rows against the oracle, row sample per part
        for i, n in enumerate(("q", "k", "v")):
            sel = sample_rows(4096, 128)
            want = oracle_rows(stack[n][3], stack[n][4], 4096, D, sel, x)
            assert rel_l2(y_qkv[:, i * 4096 + sel], want) <= TOL
        y_gu = gu.gemv(xd).cpu().numpy()
        for i, n in enumerate(("gate", "up")):
            sel = sample_rows(F, 128)
            want = oracle_rows(stack[n][3], stack[n][4], F, D, sel, x)
            assert rel_l2(y_gu[:, i * F + sel], want) <= TOL
        # fused norm + q/k/v
        xn = O.rmsnorm(x, wn)
        y_nqkv = layers.gemv_rmsnorm(qkv, xd, wd).cpu().numpy()
        sel = sample_rows(4096, 128)
        want = oracle_rows(stack["k"][3], stack["k"][4], 4096, D, sel, xn)
        assert rel_l2(y_nqkv[:, 4096 + sel], want) <= TOL
        assert rel_l2(y_nqkv, qkv.gemv(torch.from_numpy(xn).cuda()).cpu().numpy()) <= TOL
        # fused MLP step: norm + gate/up, SwiGLU + down; the oracle needs every gate/up row for one down row, so the
        # hidden vector comes from the oracle's double-precision GEMV over all rows of gate and up
        y_mlp = layers.mlp_step(gu, dws["down"], xd, norm_w=wd).cpu().numpy()
        g = O.block_gemm(stack["gate"][3], to_orc_blocks(stack["gate"][4]), F, D, xn, wide=True)
        u = O.block_gemm(stack["up"][3], to_orc_blocks(stack["up"][4]), F, D, xn, wide=True)
        h = O.swiglu(g, u)
        sel = sample_rows(D, 32)
        want = oracle_rows(stack["down"][3], stack["down"][4], D, F, sel, h)
        assert rel_l2(y_mlp[:, sel], want) <= TOL
    finally:
        for d in list(dws.values()) + [qkv, gu]:
            d.close()


def test_moe_step_full_size():
    """8 OIL4 experts with d_model 4096 and d_ff 14336, 64 tokens, top-2, uneven loads.  One expert is quantized and the
    other seven are its rows rotated (distinct matrices, same statistics); the oracle runs the whole dispatch in double
    precision on the decoded matrices."""
    D, F, E, T, K = 4096, 14336, 8, 64, 2
    rng = np.random.default_rng(2026)
    base = []
    for r, c in ((F, D), (F, D), (D, F)):
        w = rng.standard_normal(r * c, dtype=np.float32) * np.float32(0.02)
        payload, blocks = ia.block_codec.quantize_tensor(w, ia.Format.OIL4)
        dense = O.dequant_blocks(payload, to_orc_blocks(blocks)).reshape(r, c)
        base.append((r, c, payload, blocks, dense))
        del w
    experts, dense = [], ([], [], [])
    for e in range(E):
        dev = []
        for j, (r, c, payload, blocks, dm) in enumerate(base):
            shift = (e * 37) % r                                   # rows rotated by `shift`: whole blocks move
            rb = (c // 256) * 128
            pay = np.roll(payload.reshape(r, rb), shift, axis=0).reshape(-1)
            dev.append(ia.DeviceWeights.from_blocks(pay, blocks, r, c))
            dense[j].append(np.roll(dm, shift, axis=0))
        experts.append(moe.ExpertFFN(*dev))
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[:, 0] += 1.0
    _, idx, wgt = moe.softmax_with_topk(logits, K)
    _, oidx, owgt = O.softmax_topk(logits, K)
    assert np.array_equal(idx, oidx) and np.array_equal(wgt.view(np.uint32), owgt.view(np.uint32))
    hist = np.bincount(idx.ravel(), minlength=E)
    assert hist.max() > 32 and hist.min() >= 1 and hist.sum() == T * K     # one expert beyond a 32-token pass, none idle
    wgt[5, 1] = 0.0                                                        # a dropped pair
    x = rng.standard_normal((T, D)).astype(np.float32)
    try:
        out, z, dropped = moe.moe_dispatch_batched(torch.from_numpy(x).cuda(), experts, idx, wgt)
        out2, _, _ = moe.moe_dispatch_batched(torch.from_numpy(x).cuda(), experts, idx, wgt, want_z_loss=False)
    finally:
        for ex in experts:
            for d in (ex.gate_proj, ex.up_proj, ex.down_proj):
                d.close()
    want, zw, dw = O.moe_dispatch(x, dense[0], dense[1], dense[2], idx, wgt, wide=True)
    assert rel_l2(out.cpu().numpy(), want) <= TOL
    assert np.array_equal(out.cpu().numpy().view(np.uint32), out2.cpu().numpy().view(np.uint32))   # the same bits from run to run
    assert dropped == dw == 1
    # the reference adds the 5e5 squared contributions in one FP32 chain (fmaf), the device in double: the chain's own
    # rounding is what separates the two
    assert abs(z - zw) <= 1e-3 * zw


def random_oil4_payload(rows, cols, seed):
    """Valid OIL4 blocks straight from random bytes: every code value occurs, scales are finite FP16 values around 0.02."""
    rng = np.random.default_rng(seed)
    nb = rows * cols // 256
    payload = rng.integers(0, 256, nb * 128, dtype=np.uint8)
    scale = (0.005 + 0.045 * rng.random(nb)).astype(np.float16).view(np.uint16)
    payload[0::128] = (scale & 0xFF).astype(np.uint8)
    payload[1::128] = (scale >> 8).astype(np.uint8)
    blocks = np.zeros(nb, dtype=ia._lib.BLOCK_DTYPE)
    blocks["idx_off"] = np.arange(nb, dtype=np.uint64) * 128
    blocks["cb_off"] = blocks["idx_off"]
    blocks["idx_bytes"], blocks["nw"], blocks["fmt"] = 128, 256, int(ia.Format.OIL4)
    return payload, blocks


@pytest.mark.parametrize("rows,M", [(248320, 1), (131072, 16)])
def test_output_head_shapes(rows, M):
    cols = 4096
    payload, blocks = random_oil4_payload(rows, cols, seed=rows)
    rng = np.random.default_rng(M)
    X = rng.standard_normal((M, cols)).astype(np.float32)
    X2 = rng.standard_normal((M, cols)).astype(np.float32)
    with ia.DeviceWeights.from_blocks(payload, blocks, rows, cols) as dw:
        xd, xd2 = torch.from_numpy(X).cuda(), torch.from_numpy(X2).cuda()
        y = dw.gemv(xd).cpu().numpy()
        ysum = dw.gemv(xd + xd2).cpu().numpy()
        y2 = dw.gemv(xd2).cpu().numpy()
        yb = dw.gemv(xd).cpu().numpy()
    sel = np.unique(np.concatenate([np.arange(0, rows, 997), np.arange(16), np.arange(rows - 16, rows)]))
    assert rel_l2(y[:, sel], oracle_rows(payload, blocks, rows, cols, sel, X)) <= TOL
    assert rel_l2(ysum, y + y2) <= TOL
    assert np.array_equal(y.view(np.uint32), yb.view(np.uint32))            # identical bits from one launch to the next
