"""The device OIL4 KV cache (oilhip_kv_*, through the C ABI) against the vectors the compiled reference wrote
(tests/golden/kv.npz) and the CPU oracle: codes, centroids and decoded values bit for bit."""
import importlib.util
import os

import numpy as np
import pytest
import torch

import innova_amd as ia
import oracle as O

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(__file__)
_spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(HERE, "golden", "make_fixtures.py"))
MF = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(MF)
KV = np.load(os.path.join(HERE, "golden", "kv.npz"))


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def as_ref_shape(x, heads, dim):
    return dev(x).reshape(1, heads, -1, dim)       # the reference's shape over [seq][heads * dim] memory


def test_half_decode_all_codes():
    cb = dev(np.arange(65536, dtype=np.uint16).view(np.int16).reshape(4096, 16))
    codes = dev(np.tile(np.arange(16, dtype=np.uint8), (4096, 1)))
    got = ia.OIL4KVCache.dequantize_block_oil4(codes, cb).cpu().numpy().ravel().view(np.uint32)
    assert np.array_equal(got, KV["h2f"])


def test_quantize_blocks_fixture_and_oracle():
    for j in range(84):
        x = MF.kv_block_inputs(j)
        if x.size > 128:
            with pytest.raises(ia.OilHipError):
                ia.OIL4KVCache.quantize_block_oil4(dev(x[None, :]))
            continue
        codes, cb = ia.OIL4KVCache.quantize_block_oil4(dev(x[None, :]))
        assert np.array_equal(codes.cpu().numpy()[0], KV[f"qcodes{j}"]), j
        assert np.array_equal(cb.cpu().numpy()[0].view(np.uint16), KV[f"qcb{j}"]), j
    rng = np.random.default_rng(3)
    for n in (2, 31, 32, 64, 65, 96, 127, 128):
        x = (rng.standard_normal((300, n)) * 10.0 ** rng.integers(-6, 4, size=(300, 1))).astype(np.float32)
        x[5] = 0.0                                 # constant rows, signed zeros, ties
        x[6] = -0.0
        x[7, ::2] = -0.0
        x[7, 1::2] = 0.0
        x[8] = np.round(x[8])
        x[9] = 1.5
        codes, cb = ia.OIL4KVCache.quantize_block_oil4(dev(x))
        codes, cb = codes.cpu().numpy(), cb.cpu().numpy().view(np.uint16)
        for b in range(300):
            wcb, wcodes = O.kv_quantize_block(x[b])
            assert np.array_equal(cb[b], wcb) and np.array_equal(codes[b], wcodes), (n, b)
        back = ia.OIL4KVCache.dequantize_block_oil4(dev(codes), dev(cb.view(np.int16))).cpu().numpy()
        want = O.kv_half_to_float(cb[0])[codes[0]]
        assert np.array_equal(back[0].view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("i", range(len(MF.KV_CASES)))
def test_cache_fixture(i):
    ms, h, d, block, lens = MF.KV_CASES[i]
    k, v = MF.kv_inputs(i)
    c = ia.OIL4KVCache(2, ms, h, d, block)
    o = O.KVCache(ms, h, d, block)
    at = 0
    for s in lens:
        c.append(1, as_ref_shape(k[at:at + s], h, d), as_ref_shape(v[at:at + s], h, d))
        c.append(0, as_ref_shape(v[at:at + s], h, d), as_ref_shape(k[at:at + s], h, d))   # layers are independent
        c.append(5, as_ref_shape(k[at:at + s], h, d), as_ref_shape(v[at:at + s], h, d))   # no such layer: ignored
        o.append(k[at:at + s], v[at:at + s])
        at += s
    tot = sum(lens)
    for r, (st, en) in enumerate([(0, tot), (1, tot - 1), (0, tot + 5)]):
        gk, gv = c.get_range(1, st, en)
        assert tuple(gk.shape) == (1, h, KV[f"k{i}_{r}"].shape[0], d)
        assert np.array_equal(gk.cpu().numpy().reshape(-1, h * d).view(np.uint32), KV[f"k{i}_{r}"])
        assert np.array_equal(gv.cpu().numpy().reshape(-1, h * d).view(np.uint32), KV[f"v{i}_{r}"])
        sb, cl = (int(x) for x in KV[f"meta{i}_{r}"])
        assert c.context_len() == cl and c.size_bytes() == 2 * sb      # the fixture's cache has one layer, this one two
    for got, want in zip(c.state(1), (o.k_idx, o.v_idx, o.k_cb, o.v_cb)):
        assert np.array_equal(got, want)
    assert c.get_range(1, 2, 2)[0].numel() == 0 and c.get_range(7, 0, 3)[0].numel() == 0
    assert c.block_size() == (block if block in (32, 64, 128) else 64)
    assert c.compression_ratio() == pytest.approx(tot * h * d * 8 / c.size_bytes())


@pytest.mark.parametrize("heads,dim,block,prefill,steps", [(8, 128, 64, 96, 5), (2, 64, 128, 33, 3), (4, 80, 32, 40, 4),
                                                          (1, 6, 64, 50, 7), (3, 50, 64, 21, 6),
                                                          (3, 11, 64, 19, 5), (5, 7, 32, 30, 4), (1, 129, 128, 9, 3)])   # odd token sizes: chunks share bytes
def test_prefill_then_decode_against_oracle(heads, dim, block, prefill, steps):
    rng = np.random.default_rng(heads * 1000 + dim)
    ms = prefill + steps + 2
    tot = prefill + steps + 4                      # the last appends run past max_seq_len: dropped, still counted
    k = rng.standard_normal((tot, heads * dim)).astype(np.float32)
    v = (rng.standard_normal((tot, heads * dim)) * np.linspace(0.01, 30, heads * dim)).astype(np.float32)
    c = ia.OIL4KVCache(1, ms, heads, dim, block)
    o = O.KVCache(ms, heads, dim, block)
    lens = [prefill] + [1] * steps + [4]
    at = 0
    for s in lens:
        c.append(0, as_ref_shape(k[at:at + s], heads, dim), as_ref_shape(v[at:at + s], heads, dim))
        o.append(k[at:at + s], v[at:at + s])
        at += s
        if at <= ms:
            gk, gv = c.get_all(0)
            wk, wv = o.get_range(0, at)
            assert np.array_equal(gk.cpu().numpy().reshape(-1, heads * dim).view(np.uint32), wk.view(np.uint32))
            assert np.array_equal(gv.cpu().numpy().reshape(-1, heads * dim).view(np.uint32), wv.view(np.uint32))
    assert c.context_len() == tot                  # as the reference counts
    for got, want in zip(c.state(0), (o.k_idx, o.v_idx, o.k_cb, o.v_cb)):
        assert np.array_equal(got, want)
    gk, _ = c.get_all(0)
    assert gk.shape[2] == ms                       # only tokens that were stored come back
    # quantization error: sixteen levels over a chunk keep every value within an eighth of the data range
    # (tokens that are whole blocks only: a block shared by several tokens keeps the K centroids of the token that
    # opened it, src/kv_cache_oil4.cpp:256-261, and the later tokens decode through those)
    if (heads * dim) % block == 0:
        err = np.abs(gk.cpu().numpy().reshape(-1, heads * dim) - k[:ms])
        assert err.max() <= (k.max() - k.min()) / 8
    c.clear()
    assert c.context_len() == 0 and c.get_all(0)[0].numel() == 0 and not any(a.any() for a in c.state(0))
    c.resize(4)
    c.append(0, as_ref_shape(k[:3], heads, dim), as_ref_shape(v[:3], heads, dim))
    o2 = O.KVCache(4, heads, dim, block)
    o2.append(k[:3], v[:3])
    assert np.array_equal(c.get_all(0)[0].cpu().numpy().reshape(-1, heads * dim).view(np.uint32), o2.get_range(0, 3)[0].view(np.uint32))


def test_full_size_layer():
    """A Llama-7B layer (32 heads x 128) with a 2048-token prefill: sampled chunks against the oracle's quantizer,
    ranges against slices of the whole, decoded values against the stored centroids."""
    heads, dim, block, n = 32, 128, 64, 2048
    pt = heads * dim
    g = torch.Generator(device="cuda").manual_seed(7)
    k = torch.randn((1, heads, n, dim), generator=g, device="cuda")
    v = torch.randn((1, heads, n, dim), generator=g, device="cuda") * 4
    c = ia.OIL4KVCache(1, n + 8, heads, dim, block)
    c.append(0, k, v)
    for t in range(4):
        c.append(0, k.reshape(n, pt)[t:t + 1].reshape(1, heads, 1, dim).contiguous(), v.reshape(n, pt)[t:t + 1].reshape(1, heads, 1, dim).contiguous())
    ak, av = c.get_all(0)
    assert ak.shape[2] == n + 4
    pk, pv = c.get_range(0, 100, 1500)
    assert torch.equal(pk.reshape(-1, pt), ak.reshape(-1, pt)[100:1500]) and torch.equal(pv.reshape(-1, pt), av.reshape(-1, pt)[100:1500])
    assert torch.equal(ak.reshape(-1, pt)[n:n + 4], ak.reshape(-1, pt)[:4])       # the same token quantizes the same way
    ki, vi, kc, vc = c.state(0)
    kh, akh = k.reshape(n, pt).cpu().numpy(), ak.reshape(-1, pt).cpu().numpy()
    rng = np.random.default_rng(1)
    for t, b in zip(rng.integers(0, n, 200), rng.integers(0, pt // block, 200)):
        wcb, wcodes = O.kv_quantize_block(kh[t, b * block:(b + 1) * block])
        blk = t * (pt // block) + b
        assert np.array_equal(kc[blk * 16:(blk + 1) * 16], wcb)
        e = blk * block + np.arange(block)
        assert np.array_equal((ki[e // 2] >> (4 * (e & 1))) & 15, wcodes)
        assert np.array_equal(akh[t, b * block:(b + 1) * block].view(np.uint32), O.kv_half_to_float(wcb)[wcodes].view(np.uint32))


def test_argument_errors():
    with pytest.raises(ia.OilHipError):
        ia.OIL4KVCache(1, -8, 3, 5, 64)
    c = ia.OIL4KVCache(1, 8, 2, 8, 64)
    with pytest.raises(ia.OilHipError):
        c.get_range(0, -1, 3)
    with pytest.raises(ia.OilHipError):
        c.get_range(-1, 0, 3)
    assert c.get_all(0)[0].numel() == 0
