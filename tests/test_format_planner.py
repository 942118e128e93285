"""Format routing (host planner) against fixtures written from the compiled reference
(tests/golden/planner.npz): registry tables, FormatPlanner::allocate, score_importance.
The reference's own planner test (tests/test_format.cpp:112-159) is restated at the end."""
import importlib.util
import os

import numpy as np
import pytest

from innova_amd import Format, format_bpw
from innova_amd.format_planner import MIXES, FormatPlanner

HERE = os.path.dirname(os.path.abspath(__file__))
_spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(HERE, "golden", "make_fixtures.py"))
MF = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(MF)


@pytest.fixture(scope="module")
def gold():
    return np.load(os.path.join(HERE, "golden", "planner.npz"))


def test_registry_tables(gold):
    singles = [(str(n), float(b), int(t[0])) for n, k, b, t in zip(gold["reg_name"], gold["reg_kind"], gold["reg_bpw"], gold["reg_tiers"]) if k == 0]
    assert len(singles) == 15
    for name, bpw, fmt in singles:
        assert Format[name] == fmt
        assert np.float32(format_bpw(fmt)) == np.float32(bpw)
    mixes = {str(n): (b, t[:nt], r[:nt]) for n, k, b, t, r, nt in zip(gold["reg_name"], gold["reg_kind"], gold["reg_bpw"], gold["reg_tiers"], gold["reg_ratios"], gold["reg_ntiers"]) if k > 0}
    assert set(mixes) == set(MIXES)
    for name, (tiers, ratios, bpw) in MIXES.items():
        b, t, r = mixes[name]
        assert np.float32(bpw) == b
        assert [int(f) for f in tiers] == list(t)
        assert np.array_equal(np.array(ratios, np.float32), r)


def test_allocate_matches_reference(gold):
    rng = np.random.default_rng(5)
    meta, fm = gold["plan_meta"], gold["plan_fmts"]
    off = i = 0
    for target in MF.PLAN_TARGETS:
        for nb in MF.PLAN_BLOCKS:
            for kind in range(4):
                scores = MF.plan_scores(kind, nb, rng)
                pl = FormatPlanner(target)
                pl._scores = scores
                plan = pl.allocate(nb)
                row = meta[i]
                assert (row[1], row[2]) == (nb, kind)
                assert np.array_equal(plan.formats, fm[off:off + nb]), (target, nb, kind)
                assert plan.uses_mix == bool(row[3])
                assert list(plan.counts.values()) == list(row[4:11])
                if nb:
                    assert np.float32(plan.achieved_bpw) == gold["plan_achieved"][i]
                    assert np.float32(FormatPlanner.estimate_bpw(plan)) == gold["plan_estimated"][i]
                off += nb
                i += 1
    assert i == len(meta) and off == len(fm)


def test_score_importance_matches_reference(gold):
    meta, out = gold["score_meta"], gold["score_out"]
    w_all, a_all = gold["score_w"], gold["score_a"]
    woff = ooff = 0
    seen = {}
    for n, bs, mode in meta:
        key = (int(n), int(bs))
        if key not in seen:
            seen[key] = woff
            woff += n
        w, a = w_all[seen[key]:seen[key] + n], a_all[seen[key]:seen[key] + n]
        nb = (n + bs - 1) // bs
        pl = FormatPlanner()
        if mode == 2:
            pl.score_importance_fisher(w, a, int(bs))
        else:
            pl.score_importance(w, a if mode else None, int(bs))
        assert pl.importance_scores().tobytes() == out[ooff:ooff + nb].tobytes(), (n, bs, mode)
        ooff += nb
    assert ooff == len(out)


def test_reference_planner_invariants():
    plan = FormatPlanner(1.5).plan_for_model(1000000)
    assert plan.formats.size == 3906 and plan.achieved_bpw > 0 and plan.target_bpw > 0
    assert FormatPlanner.estimate_bpw(plan) > 0
    for bpw in (1.5, 2.0, 2.3, 3.0, 3.5, 4.0, 4.5, 5.0, 6.0, 7.0, 8.0):
        plan = FormatPlanner(bpw).plan_for_model(1000000)
        assert plan.formats.size > 0
        assert abs(FormatPlanner.estimate_bpw(plan) - bpw) < 1.0


def test_important_blocks_get_the_precise_formats():
    # config "1.50 bpw stack": half SPARK_Q0, half OIL1, SPARK_Q0 on the important half
    # ... 1.5 is itself a single (SPARK_Q0), so use 1.25: 25% SPARK_Q0 + 75% OIL1
    w = np.random.default_rng(0).standard_normal(64 * 256).astype(np.float32)
    w[: 16 * 256] *= 10
    pl = FormatPlanner(1.25)
    pl.score_importance(w)
    plan = pl.allocate(64)
    assert not plan.uses_mix
    assert (plan.formats[:16] == Format.SPARK_Q0).all() and (plan.formats[16:] == Format.OIL1).all()
