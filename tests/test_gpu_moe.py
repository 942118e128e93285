"""moe_dispatch_batched on the device over quantized experts, against the compiled reference's
output for the same inputs (tests/golden/moe.npz) and the CPU oracle in double precision.
Tolerance: relative L2 <= 1e-5 (FP32 accumulation in a different order than the reference's chain)."""
import importlib.util
import os

import numpy as np
import pytest
import torch

import innova_amd as ia
import oracle as O
from innova_amd import moe

pytestmark = pytest.mark.gpu
TOL = 1e-5
HERE = os.path.dirname(os.path.abspath(__file__))
_spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(HERE, "golden", "make_fixtures.py"))
MF = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(MF)


def rel(a, b):
    return float(np.linalg.norm(a.astype(np.float64) - b.astype(np.float64)) / np.linalg.norm(b.astype(np.float64)))


def upload(packs, D, F):
    ex = []
    for (gp, up, dp) in packs:
        ex.append(moe.ExpertFFN(ia.DeviceWeights.from_blocks(np.asarray(gp[0]), ia_blocks(gp[1]), F, D),
                                ia.DeviceWeights.from_blocks(np.asarray(up[0]), ia_blocks(up[1]), F, D),
                                ia.DeviceWeights.from_blocks(np.asarray(dp[0]), ia_blocks(dp[1]), D, F)))
    return ex


def ia_blocks(ob):
    b = np.zeros(ob.size, ia._lib.BLOCK_DTYPE)
    for k in ("cb_off", "idx_off", "cb_bytes", "idx_bytes", "nw", "fmt"):
        b[k] = ob[k]
    return b


def test_dispatch_matches_reference_fixture():
    gold = np.load(os.path.join(HERE, "golden", "moe.npz"))
    sh = MF.MOE_SHAPE
    packs, _ = MF.moe_experts(11, sh["E"], sh["D"], sh["F"])
    ex = upload(packs, sh["D"], sh["F"])
    out, z, dropped = moe.moe_dispatch_batched(torch.from_numpy(gold["disp_x"]).cuda(), ex, gold["disp_idx"], gold["disp_w"])
    want = gold["disp_out"].view(np.float32)
    assert rel(out.cpu().numpy(), want) <= TOL
    assert dropped == 1
    assert abs(z - float(gold["disp_z"][0])) <= 1e-4 * float(gold["disp_z"][0])


@pytest.mark.parametrize("T,E,K,D,F,fmts", [(24, 4, 2, 512, 768, (3, 3, 3)),        # OIL4 experts: fast kernel, 1..many tokens each
                                             (40, 2, 2, 256, 512, (3, 3, 3)),        # > 16 tokens per expert: several passes
                                             (12, 8, 2, 256, 512, (3, 3, 3)),        # a few tokens per expert: passes of 8 only
                                             (50, 6, 2, 256, 512, (3, 3, 3)),        # passes of 32, 16 and 8 side by side in one launch
                                             (30, 20, 2, 256, 12288, (3, 3, 3)),     # twenty batches: two grouped launches per side over one workspace; rows cut in three
                                             (9, 3, 1, 256, 512, (4, 10, 1))])       # OIL8 / OIL4_GRP / SPARK_Q0: general kernel
def test_dispatch_against_oracle(T, E, K, D, F, fmts):
    packs, dense = MF.moe_experts(5 + T, E, D, F, fmts)
    ex = upload(packs, D, F)
    rng = np.random.default_rng(T)
    x = rng.standard_normal((T, D)).astype(np.float32)
    _, idx, w = moe.softmax_with_topk(rng.standard_normal((T, E)).astype(np.float32) * 2, K)
    out, z, dropped = moe.moe_dispatch_batched(torch.from_numpy(x).cuda(), ex, idx, w)
    g, u, d = ([e[j] for e in dense] for j in range(3))
    want, zw, dw = O.moe_dispatch(x, g, u, d, idx, w, wide=True)
    assert rel(out.cpu().numpy(), want) <= TOL
    assert dropped == dw == 0
    assert abs(z - zw) <= 1e-4 * zw


def test_step_with_caller_workspace_is_captured_and_replays_bit_for_bit():
    """With the caller's workspace and without the z-loss a step only queues launches: captured into a graph, every
    replay returns the bits of the eager step (passes of 32, 16 and 8 tokens; rows cut along K with ordered sums)."""
    T, E, K, D, F = 44, 3, 2, 512, 12288                                  # d_ff 12288: the down projection's rows are cut in three
    packs, dense = MF.moe_experts(91, E, D, F, (3, 3, 3))
    ex = upload(packs, D, F)
    rng = np.random.default_rng(92)
    xh = rng.standard_normal((T, D)).astype(np.float32)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    logits[:, 0] += 1.5
    _, idx, w = moe.softmax_with_topk(logits, K)
    hist = np.bincount(idx.ravel(), minlength=E)
    assert hist.max() > 32 and hist.min() >= 1
    x = torch.from_numpy(xh).cuda()
    ws, out = moe.moe_workspace(x, ex, K), torch.zeros(T, D, device="cuda")
    st = torch.cuda.Stream()
    with torch.cuda.stream(st):
        moe.moe_dispatch_batched(x, ex, idx, w, want_z_loss=False, workspace=ws, out=out)
        st.synchronize()
        eager = out.clone()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=st):
            moe.moe_dispatch_batched(x, ex, idx, w, want_z_loss=False, workspace=ws, out=out)
        for _ in range(3):
            out.zero_()
            g.replay()
            st.synchronize()
            assert torch.equal(out, eager)
    gd, ud, dd = ([e[j] for e in dense] for j in range(3))
    want, _, _ = O.moe_dispatch(xh, gd, ud, dd, idx, w, wide=True)
    assert rel(eager.cpu().numpy(), want) <= TOL


def test_bad_arguments():
    packs, _ = MF.moe_experts(1, 2, 256, 512)
    ex = upload(packs, 256, 512)
    x = torch.zeros(4, 256, device="cuda")
    idx = np.zeros((4, 1), np.int64)
    w = np.ones((4, 1), np.float32)
    bad = [moe.ExpertFFN(ex[0].gate_proj, ex[0].down_proj, ex[0].down_proj), ex[1]]     # up has the wrong shape
    with pytest.raises(ia.OilHipError):
        moe.moe_dispatch_batched(x, bad, idx, w)
