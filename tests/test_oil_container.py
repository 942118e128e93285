"""The .oil container against a file the reference's OILWriter wrote (tests/golden/mixed.oil):
parsing, block access, truncated/garbled files, and our writer reproducing the file byte for byte."""
import importlib.util
import os

import numpy as np
import pytest

import innova_amd as ia
from innova_amd import _lib, block_codec

HERE = os.path.dirname(os.path.abspath(__file__))
_spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(HERE, "golden", "make_fixtures.py"))
MF = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(MF)
PATH = os.path.join(HERE, "golden", "mixed.oil")


def quantize_segments(data, fmts, starts, lens):
    """(payload, blocks) with one block per (start, len) segment."""
    pay, blocks = [], np.zeros(len(fmts), _lib.BLOCK_DTYPE)
    off = 0
    for b, (f, s, n) in enumerate(zip(fmts, starts, lens)):
        idx, cb = block_codec.quantize_block_all(int(f), data[s:s + n])
        blocks[b] = (off, off + cb.size, cb.size, idx.size, n, int(f), (0, 0, 0))
        pay += [cb, idx]
        off += cb.size + idx.size
    return np.concatenate(pay), blocks


def test_reader_parses_reference_file():
    ts = MF.container_tensors()
    gold = np.load(os.path.join(HERE, "golden", "container.npz"))
    with ia.OILReader(PATH) as r:
        assert r.valid()
        assert (r.version, r.flags) == (MF.CONTAINER_VERSION, MF.CONTAINER_FLAGS)
        assert r.read_config() == MF.CONTAINER_CONFIG
        assert r.num_blocks() == gold["meta"][0] == sum(len(t[2]) for t in ts)
        assert r.tensor_names() == [t[0] for t in ts]
        assert r.tensor_blocks(ts[2][0]) == (gold["meta"][2], gold["meta"][3])
        assert r.tensor_blocks("missing") is None
        bid = 0
        for name, data, fmts, starts, lens in ts:
            assert [int(f) for f in r.tensor_formats(name)] == list(fmts)
            for f, s, n in zip(fmts, starts, lens):
                bd = r.read_block(bid)
                idx, cb = block_codec.quantize_block_all(int(f), data[s:s + n])
                assert bd.format == f and bd.num_weights == n
                assert bd.indices.tobytes() == idx.tobytes() and bd.codebook.tobytes() == cb.tobytes()
                bid += 1
        with pytest.raises(ia.OilHipError):
            r.read_block(bid)


def test_writer_reproduces_reference_file(tmp_path):
    ts = MF.container_tensors()
    out = tmp_path / "ours.oil"
    ia.write_oil(out, [(name, *quantize_segments(d, f, s, n)) for name, d, f, s, n in ts],
                 version=MF.CONTAINER_VERSION, flags=MF.CONTAINER_FLAGS, config=MF.CONTAINER_CONFIG)
    assert out.read_bytes() == open(PATH, "rb").read()


def test_flat_tensor_roundtrip_through_file(tmp_path):
    w = np.random.default_rng(1).standard_normal(8 * 512).astype(np.float32)
    payload, blocks = block_codec.quantize_tensor(w, ia.Format.OIL4)
    ia.write_oil(tmp_path / "t.oil", [("w", payload, blocks), ("w2", payload, blocks)])
    with ia.OILReader(tmp_path / "t.oil") as r:
        assert r.tensor_names() == ["w", "w2"] and r.num_blocks() == 32 and r.read_config() == b""
        assert r.tensor_blocks("w2") == (16, 16)
        assert r.read_block(17).indices.tobytes() == payload[blocks[1]["idx_off"]:][:128].tobytes()


def test_bad_files_are_rejected_or_clipped():
    raw = open(PATH, "rb").read()
    assert not ia.OILReader(b"OIL").valid()
    assert not ia.OILReader(b"XIL1" + raw[4:]).valid()
    assert not ia.OILReader(raw[:40]).valid()               # cut inside the format table
    assert not ia.OILReader("/nonexistent/file.oil").valid()
    r = ia.OILReader(raw[:-100])                            # cut inside the last records: they drop out of the index
    assert r.valid() and r.num_blocks() == 100
    r.read_block(90)
    with pytest.raises(ia.OilHipError):
        r.read_block(99)
    with pytest.raises(ia.OilHipError):
        ia.OILReader(b"OIL").read_config()
