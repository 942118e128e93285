"""The CPU oracle's OIL4 KV cache (OIL4KVCache, src/kv_cache_oil4.cpp; CodebookOIL4 half conversions,
src/codebook.cpp:16-64) against the vectors the compiled reference wrote (tests/golden/kv.npz), against the
compiled reference where it is built, and against what the definitions fix by themselves."""
import importlib.util
import os

import numpy as np
import pytest

import oracle as O

HERE = os.path.dirname(__file__)
_spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(HERE, "golden", "make_fixtures.py"))
MF = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(MF)
KV = np.load(os.path.join(HERE, "golden", "kv.npz"))


def test_half_to_float_all_codes():
    got = O.kv_half_to_float(np.arange(65536, dtype=np.uint16)).view(np.uint32)
    assert np.array_equal(got, KV["h2f"])
    # normal halves, zeros and infinities are the IEEE values; subnormals are not (the reference's own decode)
    h = np.arange(65536, dtype=np.uint16)
    ieee = h.view(np.float16).astype(np.float32).view(np.uint32)
    normal = ((h >> 10) & 0x1F != 0) & ((h >> 10) & 0x1F != 31) | (h & 0x7FFF == 0) | (h & 0x7FFF == 0x7C00)
    assert np.array_equal(got[normal], ieee[normal])


def test_float_to_half_truncates():
    bits = MF.kv_f2h_inputs()
    got = O.kv_float_to_half(bits.view(np.float32))
    assert np.array_equal(got, KV["f2h"])
    # in the normal half range the encoder drops the low 13 mantissa bits: never above the input in magnitude,
    # within one half ulp step of numpy's round-to-nearest
    f = bits.view(np.float32)
    sel = (np.abs(f) >= 2.0 ** -14) & (np.abs(f) < 65504)
    back = got[sel].view(np.float16).astype(np.float32)
    assert np.all(np.abs(back) <= np.abs(f[sel]))
    rn = f[sel].astype(np.float16).view(np.uint16).astype(np.int64)
    assert np.all(np.abs(rn - got[sel].astype(np.int64)) <= 1)


def test_quantize_block_fixture():
    for j in range(84):
        cb, codes = O.kv_quantize_block(MF.kv_block_inputs(j))
        assert np.array_equal(cb, KV[f"qcb{j}"]), j
        assert np.array_equal(codes, KV[f"qcodes{j}"]), j


def test_quantize_block_properties():
    rng = np.random.default_rng(5)
    for n in (2, 17, 64, 128):
        x = rng.standard_normal(n).astype(np.float32)
        cb, codes = O.kv_quantize_block(x)
        cen = cb.view(np.float16).astype(np.float32)
        # ascending centroids inside the data range; codes name a nearest centroid up to FP16 truncation of the table
        assert np.all(np.diff(cen) >= 0) and cen[0] >= x.min() - 1e-3 and cen[-1] <= x.max() + 1e-3
        d = np.abs(x[:, None] - cen[None, :])
        assert np.all(d[np.arange(n), codes] <= d.min(1) + 2e-3 * np.abs(x).max())
    # a constant chunk: every code 8, every centroid the value itself (truncated)
    x = np.full(64, 0.3, np.float32)
    cb, codes = O.kv_quantize_block(x)
    assert np.all(codes == 8) and np.all(cb == O.kv_float_to_half(x[:1])[0])
    # sixteen distinct values are their own centroids: the round trip is exact up to the FP16 truncation
    x = (np.arange(16, dtype=np.float32) - 8) * 0.25
    cb, codes = O.kv_quantize_block(np.repeat(x, 4))
    assert np.array_equal(cb.view(np.float16).astype(np.float32)[codes], np.repeat(x, 4))


@pytest.mark.parametrize("i", range(len(MF.KV_CASES)))
def test_cache_fixture(i):
    ms, h, d, block, lens = MF.KV_CASES[i]
    k, v = MF.kv_inputs(i)
    c = O.KVCache(ms, h, d, block)
    at = 0
    for s in lens:
        c.append(k[at:at + s], v[at:at + s])
        at += s
    tot = sum(lens)
    for r, (st, en) in enumerate([(0, tot), (1, tot - 1), (0, tot + 5)]):
        ko, vo = c.get_range(st, en)
        assert np.array_equal(ko.view(np.uint32), KV[f"k{i}_{r}"]) and np.array_equal(vo.view(np.uint32), KV[f"v{i}_{r}"])
        sb, cl = (int(x) for x in KV[f"meta{i}_{r}"])
        assert cl == c.pos and sb == 2 * c.k_idx.size + 2 * (c.k_cb.size + c.v_cb.size)


def test_cache_is_flat_nibbles_for_even_tokens():
    """With an even number of values per token every chunk starts on a byte: element e of the cache is nibble e & 1
    of byte e / 2 and reads the centroids of block e / block -- the layout the device path relies on."""
    rng = np.random.default_rng(11)
    c = O.KVCache(16, 2, 24, 32)
    k = rng.standard_normal((9, 48)).astype(np.float32)
    c.append(k[:4], k[:4])
    c.append(k[4:], k[4:])
    ko, _ = c.get_range(0, 9)
    e = np.arange(9 * 48)
    code = (c.k_idx[e // 2] >> (4 * (e & 1))) & 15
    want = O.kv_half_to_float(c.k_cb[(e // 32) * 16 + code])
    assert np.array_equal(ko.ravel().view(np.uint32), want.view(np.uint32))


@pytest.mark.skipif(O.ref(True) is None, reason="compiled reference not built here")
def test_against_compiled_reference():
    rng = np.random.default_rng(21)
    R = O.ref(True)
    for t in range(300):
        n = int(rng.choice(MF.KV_BLOCK_SIZES))
        x = (rng.standard_normal(n) * 10.0 ** rng.integers(-6, 4)).astype(np.float32)
        a, b = O.kv_quantize_block(x), O.kv_quantize_block(x, fn=R.ref_kv_quantize_block)
        assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
    for t in range(20):
        h, d = int(rng.integers(1, 5)), int(rng.choice([7, 16, 24, 64]))
        block = int(rng.choice([32, 64, 128, 50]))
        lens = [int(x) for x in rng.integers(1, 5, size=rng.integers(1, 5))]
        tot = sum(lens)
        ms = tot + int(rng.integers(-2, 3))            # also appends that run past max_seq_len
        if ms < 1:
            ms = 1
        k = rng.standard_normal((tot, h * d)).astype(np.float32)
        v = rng.standard_normal((tot, h * d)).astype(np.float32)
        end = min(tot, ms)
        rk, rv, _, _ = O.ref_kv_run(ms, h, d, block, k, v, lens, 0, end)
        c = O.KVCache(ms, h, d, block)
        at = 0
        for s in lens:
            c.append(k[at:at + s], v[at:at + s])
            at += s
        ok, ov = c.get_range(0, end)
        assert np.array_equal(rk.view(np.uint32), ok.view(np.uint32)) and np.array_equal(rv.view(np.uint32), ov.view(np.uint32))
