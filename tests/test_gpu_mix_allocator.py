"""FormatRegistry::allocate_mix_blocks on the device path (candidate errors measured by a HIP
kernel) against the plans the compiled reference produced (tests/golden/planner.npz)."""
import importlib.util
import os

import numpy as np
import pytest

from innova_amd.format_planner import allocate_mix_blocks

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
_spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(HERE, "golden", "make_fixtures.py"))
MF = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(MF)


def test_mix_plans_match_reference():
    gold = np.load(os.path.join(HERE, "golden", "planner.npz"))
    off = 0
    for k, (name, seed, n, bs, rows, cols) in enumerate(MF.MIX_CASES):
        w = MF.mix_tensor(seed, n)
        nb = int(gold["mix_nb"][k])
        fm, st, ln = allocate_mix_blocks(name, w, bs, (rows, cols) if rows else None)
        assert fm.size == nb, name
        assert np.array_equal(st, gold["mix_starts"][off:off + nb])
        assert np.array_equal(ln, gold["mix_lens"][off:off + nb])
        assert np.array_equal(fm, gold["mix_fmts"][off:off + nb]), (name, int((fm != gold["mix_fmts"][off:off + nb]).sum()))
        off += nb
