"""Mixture-of-experts routing (host) and the oracle's dispatch against fixtures written from the
compiled reference (tests/golden/moe.npz)."""
import importlib.util
import os

import numpy as np
import pytest

import oracle as O
from innova_amd import moe

HERE = os.path.dirname(os.path.abspath(__file__))
_spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(HERE, "golden", "make_fixtures.py"))
MF = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(MF)


@pytest.fixture(scope="module")
def gold():
    return np.load(os.path.join(HERE, "golden", "moe.npz"))


@pytest.mark.parametrize("who", ["oracle", "library"])
def test_routing_matches_reference(gold, who):
    rng = np.random.default_rng(1)
    po = io = 0
    for T, E, k in MF.MOE_ROUTE_CASES:
        for kind in range(3):
            lg = MF.moe_route_logits(T, E, kind, rng)
            p, i, w = O.softmax_topk(lg, k) if who == "oracle" else moe.softmax_with_topk(lg, k)
            assert np.array_equal(p.view(np.uint32).ravel(), gold["route_probs"][po:po + T * E]), (T, E, k, kind)
            assert np.array_equal(i.ravel(), gold["route_idx"][io:io + T * k]), (T, E, k, kind)
            assert np.array_equal(w.view(np.uint32).ravel(), gold["route_w"][io:io + T * k])
            po += T * E
            io += T * k
    assert po == gold["route_probs"].size


def test_routing_closed_forms():
    lg = np.random.default_rng(3).standard_normal((50, 8)).astype(np.float32)
    p, i, w = moe.softmax_with_topk(lg, 2)
    assert np.allclose(p.sum(1), 1.0, atol=1e-6)
    order = np.argsort(-p, axis=1, kind="stable")[:, :2]          # distinct probabilities: plain top-2
    assert np.array_equal(i, order)
    assert np.array_equal(w, np.take_along_axis(p, i, 1))          # raw probabilities, no renormalisation
    with pytest.raises(Exception):
        moe.softmax_with_topk(lg, 9)


def test_oracle_dispatch_matches_reference(gold):
    sh = MF.MOE_SHAPE
    _, dense = MF.moe_experts(11, sh["E"], sh["D"], sh["F"])
    g, u, d = ([e[j] for e in dense] for j in range(3))
    out, z, dr = O.moe_dispatch(gold["disp_x"], g, u, d, gold["disp_idx"], gold["disp_w"])
    assert np.array_equal(out.view(np.uint32), gold["disp_out"])
    assert np.float32(z) == gold["disp_z"][0] and dr == gold["disp_dropped"][0] == 1
    # brute force: y_t = sum_k w * down(silu(gate x) * up x) per token, in double
    x = gold["disp_x"].astype(np.float64)
    want = np.zeros_like(x)
    for t in range(sh["T"]):
        for e in range(sh["E"]):
            n = int((gold["disp_idx"][t] == e).sum())
            if n == 0:
                continue
            wgt = float(gold["disp_w"][t][list(gold["disp_idx"][t]).index(e)])
            if wgt <= 0:
                continue
            gg = g[e].astype(np.float64) @ x[t]
            h = gg / (1.0 + np.exp(-gg)) * (u[e].astype(np.float64) @ x[t])
            want[t] += n * wgt * (d[e].astype(np.float64) @ h)
    assert np.linalg.norm(out - want) / np.linalg.norm(want) < 1e-5
    wide, _, _ = O.moe_dispatch(gold["disp_x"], g, u, d, gold["disp_idx"], gold["disp_w"], wide=True)
    assert np.linalg.norm(wide - want) / np.linalg.norm(want) < 1e-6
