"""Tensors taken from an .oil file straight to the device: decode is bit-exact with what the
reference's OILReader::read_tensor produced for the same file, and the matmul runs off the
uploaded records."""
import importlib.util
import os

import numpy as np
import pytest
import torch

import innova_amd as ia
import oracle as O

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
_spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(HERE, "golden", "make_fixtures.py"))
MF = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(MF)
PATH = os.path.join(HERE, "golden", "mixed.oil")


def test_read_tensor_bit_exact():
    gold = np.load(os.path.join(HERE, "golden", "container.npz"))
    with ia.OILReader(PATH) as r:
        for k, t in enumerate(MF.container_tensors()):
            got = r.read_tensor(t[0])
            assert got.size == t[1].size
            assert np.array_equal(got.view(np.uint32), gold[f"decoded{k}"]), t[0]
        assert r.read_tensor("missing") is None


def test_gemv_from_file_records():
    name, data, fmts, starts, lens = MF.container_tensors()[0]       # 32 x 256, one format per row
    gold = np.load(os.path.join(HERE, "golden", "container.npz"))
    W = gold["decoded0"].view(np.float32).reshape(32, 256).astype(np.float64)
    x = np.random.default_rng(3).standard_normal((3, 256)).astype(np.float32)
    with ia.OILReader(PATH) as r, r.upload_tensor(name, 32, 256) as w:
        assert w.info()["uniform_fmt"] == -1
        y = w.gemv(torch.from_numpy(x).cuda()).cpu().numpy().astype(np.float64)
    ref = x.astype(np.float64) @ W.T
    assert np.linalg.norm(y - ref) / np.linalg.norm(ref) <= 1e-5      # FP32 accumulate vs double dot
