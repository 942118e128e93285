"""The CPU oracle's block codec against the reference's golden vectors
(tests/golden/codec.npz, written by the compiled reference), against the
compiled reference itself where it is built, and against the invariants the
reference's own codec test asserts (tests/test_block_codec.cpp)."""
import math
import os

import numpy as np
import pytest

import oracle as O

G = np.load(os.path.join(os.path.dirname(__file__), "golden", "codec.npz"))
NCASE = G["fmt"].size
FULL_BYTES = {  # payload bytes of a full 256-weight block, per format
    "OIL1": 16, "SPARK_Q0": 48, "OIL2": 64, "OIL4": 128, "OIL8": 256, "OIL16": 512, "OIL32": 1024,
    "OIL1_GRP": 32, "SPARK_Q0_GRP": 48, "OIL2_GRP": 80, "OIL4_GRP": 144, "OIL8_GRP": 272,
    "OIL16_GRP": 512, "SPARK_SPARSE": 64, "SPARK_SPARSE_GRP": 64}


def _case(i):
    fmt, n = int(G["fmt"][i]), int(G["n"][i])
    w = G["w_bits"][G["w_off"][i]: G["w_off"][i] + n].view(np.float32)
    idx = G["idx"][G["idx_off"][i]: G["idx_off"][i] + G["idx_len"][i]]
    cb = G["cb"][G["cb_off"][i]: G["cb_off"][i] + G["cb_len"][i]]
    dec = G["dec_bits"][G["dec_off"][i]: G["dec_off"][i] + n]
    return fmt, n, w, idx, cb, dec


def test_golden_encode_bytes_identical():
    for i in range(NCASE):
        fmt, n, w, idx, cb, _ = _case(i)
        oi, oc = O.quantize_block(fmt, w)
        assert np.array_equal(oi, idx), G["tags"][i]
        assert np.array_equal(oc, cb), G["tags"][i]


def test_golden_decode_bits_identical():
    for i in range(NCASE):
        fmt, n, _, idx, cb, dec = _case(i)
        out = O.dequantize_block(fmt, idx, cb, n)
        assert np.array_equal(out.view(np.uint32), dec), G["tags"][i]


def test_half_conversions_golden():
    hs = np.arange(65536, dtype=np.uint16)
    out = O.dequantize_block(O.FORMATS["OIL16"], hs.view(np.uint8), np.zeros(0, np.uint8), 65536)
    assert np.array_equal(out.view(np.uint32), G["f16_to_f32_bits"])
    f = G["f32_in_bits"].view(np.float32)
    h = np.concatenate([O.quantize_block(O.FORMATS["OIL16"], f[s:s + 4096])[0]
                        for s in range(0, f.size, 4096)]).view(np.uint16)
    assert np.array_equal(h, G["f32_to_f16"])


def test_half_conversions_against_numpy():
    # finite, non-NaN halves widen exactly as IEEE says (numpy as the library routine)
    hs = np.arange(65536, dtype=np.uint16)
    L = O.lib()
    mine = np.array([L.orc_f16_to_f32(int(h)) for h in hs[::7]], dtype=np.float32)
    ref = hs[::7].view(np.float16).astype(np.float32)
    ok = ~np.isnan(ref)
    assert np.array_equal(mine[ok].view(np.uint32), ref[ok].view(np.uint32))
    # narrowing: RNE for everything numpy keeps finite and >= 2^-24; the reference flushes
    # below 2^-24 (numpy would round 2^-25..2^-24 up) and maps NaN to infinity
    rng = np.random.default_rng(0)
    v = (rng.standard_normal(20000) * 10.0 ** rng.integers(-7, 5, 20000)).astype(np.float32)
    v = v[np.abs(v) >= 2.0 ** -24]
    mine = np.array([L.orc_f32_to_f16(float(x)) for x in v], dtype=np.uint16)
    with np.errstate(over="ignore"):
        assert np.array_equal(mine, v.astype(np.float16).view(np.uint16))
    assert L.orc_f32_to_f16(float(np.float32(2.0 ** -25 * 1.5))) == 0
    assert L.orc_f32_to_f16(float("nan")) == 0x7C00


def test_full_block_payload_sizes():
    w = O.xorshift_fill(256, 42)
    for name, nbytes in FULL_BYTES.items():
        idx, cb = O.quantize_block(O.FORMATS[name], w)
        assert idx.size + cb.size == nbytes, name
        assert O.max_payload_bytes(O.FORMATS[name], 256) == nbytes
        if name == "OIL1":
            assert idx.size == 0 and cb.size == 16


def test_budget_contract_tails():
    # stored bytes <= ceil((bpw*n + 8)/8)  (tests/test_block_codec.cpp:57-62,176-190)
    for n in [1, 7, 15, 16, 17, 20, 21, 25, 26, 31, 32, 33, 39, 40, 63, 100, 128, 200, 255, 256, 512]:
        w = O.xorshift_fill(n, 1000 + n)
        for fmt in range(15):
            idx, cb = O.quantize_block(fmt, w)
            budget = math.ceil((O.lib().orc_format_bpw(fmt) * n + 8.0) / 8.0)
            assert idx.size + cb.size <= budget, (fmt, n)
            assert idx.size + cb.size <= O.max_payload_bytes(fmt, n)


def test_zero_block_decodes_to_zero_with_reference_signs():
    w = np.zeros(256, dtype=np.float32)
    for fmt in range(15):
        idx, cb = O.quantize_block(fmt, w)
        out = O.dequantize_block(fmt, idx, cb, 256)
        assert np.all(out == 0.0), fmt
    # level * 0 keeps the level's sign: ties pick the lower (negative) level for OIL2/OIL4
    for name, neg in (("OIL4", True), ("OIL2", True), ("OIL8", False)):
        idx, cb = O.quantize_block(O.FORMATS[name], w)
        out = O.dequantize_block(O.FORMATS[name], idx, cb, 256)
        slots = {"OIL4": 4, "OIL2": 8, "OIL8": 2}[name]
        is_slot = np.array([((i + 1) * slots) // 256 != (i * slots) // 256 for i in range(256)])
        assert np.all(np.signbit(out[~is_slot]) == neg), name
        assert not np.any(np.signbit(out[is_slot]))


def test_sign_preservation_and_sparse_nonzero():
    for n in [1, 7, 15, 16, 17, 20, 21, 25, 26, 31, 32, 33, 39, 40, 63, 100, 128, 200, 255]:
        w = O.xorshift_fill(n, 1000 + n)
        for name in ("SPARK_Q0", "SPARK_Q0_GRP", "OIL1_GRP"):
            idx, cb = O.quantize_block(O.FORMATS[name], w)
            out = O.dequantize_block(O.FORMATS[name], idx, cb, n)
            keep = np.ones(n, dtype=bool)
            if name == "OIL1_GRP" and n >= 32:
                keep = np.array([((i + 1) * 16) // n == (i * 16) // n for i in range(n)])
            assert np.array_equal((w >= 0)[keep], (out >= 0)[keep]), (name, n)
        if n >= 32:
            for name in ("SPARK_SPARSE", "SPARK_SPARSE_GRP"):
                idx, cb = O.quantize_block(O.FORMATS[name], w)
                assert np.count_nonzero(O.dequantize_block(O.FORMATS[name], idx, cb, n)) > 0


def test_oil32_bitwise_and_oil16_roundtrip():
    rng = np.random.default_rng(5)
    w = rng.standard_normal(256).astype(np.float32)
    idx, cb = O.quantize_block(O.FORMATS["OIL32"], w)
    assert np.array_equal(O.dequantize_block(O.FORMATS["OIL32"], idx, cb, 256).view(np.uint32), w.view(np.uint32))
    idx, cb = O.quantize_block(O.FORMATS["OIL16"], w)
    assert np.array_equal(O.dequantize_block(O.FORMATS["OIL16"], idx, cb, 256), w.astype(np.float16).astype(np.float32))


def test_closed_form_positions():
    """Independent statement of the stream layout: OIL4 weight i sits at nibble
    4 + i - i//64, slots at 63,127,191,255 decode to +0; OIL8 byte 2 + i - i//128;
    OIL2 field 8 + i - i//32; SPARK_Q0 sub-block s starts at bit 48*s."""
    rng = np.random.default_rng(9)
    lv4 = np.array([-2.7178, -2.0522, -1.5995, -1.2392, -0.9275, -0.6508, -0.3976, -0.1260,
                    0.1260, 0.3976, 0.6508, 0.9275, 1.2392, 1.5995, 2.0522, 2.7178], dtype=np.float32)
    lv2 = np.array([-1.5104, -0.4528, 0.4528, 1.5104], dtype=np.float32)
    pay = rng.integers(0, 256, 256, dtype=np.uint8).astype(np.uint8)
    pay[0:2] = np.array([0.0137], dtype=np.float16).view(np.uint8)
    scale = np.float32(np.array([0.0137], dtype=np.float16)[0])
    # OIL4
    out = O.dequantize_block(O.FORMATS["OIL4"], pay[:128], np.zeros(0, np.uint8), 256)
    nib = np.stack([pay[:128] & 15, pay[:128] >> 4], axis=1).reshape(-1)
    for i in range(256):
        exp = np.float32(0.0) if i % 64 == 63 else lv4[nib[4 + i - i // 64]] * scale
        assert out[i].view(np.uint32) == np.float32(exp).view(np.uint32)
    # OIL8
    out = O.dequantize_block(O.FORMATS["OIL8"], pay, np.zeros(0, np.uint8), 256)
    for i in range(256):
        if i % 128 == 127:
            exp = np.float32(0.0)
        else:
            q = np.float32(pay[2 + i - i // 128])
            exp = (np.float32(-8.0) + (np.float32(16.0) * q) / np.float32(255.0)) * scale
        assert out[i].view(np.uint32) == np.float32(exp).view(np.uint32)
    # OIL2
    out = O.dequantize_block(O.FORMATS["OIL2"], pay[:64], np.zeros(0, np.uint8), 256)
    f2 = np.stack([(pay[:64] >> s) & 3 for s in (0, 2, 4, 6)], axis=1).reshape(-1)
    for i in range(256):
        exp = np.float32(0.0) if i % 32 == 31 else lv2[f2[8 + i - i // 32]] * scale
        assert out[i].view(np.uint32) == np.float32(exp).view(np.uint32)
    # SPARK_Q0
    p = pay[:48].copy()
    for s in range(8):
        p[6 * s: 6 * s + 2] = np.array([0.01 * (s + 1)], dtype=np.float16).view(np.uint8)
    out = O.dequantize_block(O.FORMATS["SPARK_Q0"], p, np.zeros(0, np.uint8), 256)
    bits = np.unpackbits(p, bitorder="little")
    for i in range(256):
        s = i // 32
        sc = np.float32(np.array([0.01 * (s + 1)], dtype=np.float16)[0])
        exp = sc if bits[48 * s + 16 + i % 32] else -sc
        assert out[i] == exp
    # OIL4_GRP: group g at bit g*(32+64*4); fused level*scale+zp
    p = pay[:144].copy()
    for g in range(4):
        p[36 * g: 36 * g + 4] = np.array([0.003 * (g - 1.5), 0.02 + 0.001 * g], dtype=np.float16).view(np.uint8)
    out = O.dequantize_block(O.FORMATS["OIL4_GRP"], p, np.zeros(0, np.uint8), 256)
    for i in range(256):
        g, j = divmod(i, 64)
        zp, sc = p[36 * g: 36 * g + 4].view(np.float16).astype(np.float64)
        byte = p[36 * g + 4 + j // 2]
        q = (byte >> 4) if j & 1 else (byte & 15)
        exp = np.float32(np.float64(lv4[q]) * sc + zp)      # one rounding == fmaf
        assert out[i].view(np.uint32) == exp.view(np.uint32)


def test_truncated_payloads_read_as_zero_padded():
    w = O.xorshift_fill(256, 99)
    for fmt in range(15):
        idx, cb = O.quantize_block(fmt, w)
        for cut in range(0, min(idx.size, 8) + 1):
            a = O.dequantize_block(fmt, idx[:cut], cb, 256)
            if fmt in (O.FORMATS["OIL32"], O.FORMATS["OIL16"], O.FORMATS["OIL16_GRP"],
                       O.FORMATS["SPARK_SPARSE"], O.FORMATS["SPARK_SPARSE_GRP"]):
                assert np.all(np.isfinite(a))
                continue
            padded = np.zeros(idx.size, dtype=np.uint8)
            padded[:cut] = idx[:cut]
            b = O.dequantize_block(fmt, padded, cb, 256)
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (fmt, cut)


def test_quantize_tensor_layout_and_roundtrip():
    rng = np.random.default_rng(3)
    w = (rng.standard_normal(256 * 11 + 100) * 0.02).astype(np.float32)
    fmts = np.array([i % 15 for i in range(12)], dtype=np.uint8)
    payload, blocks = O.quantize_tensor(w, fmts, align=16)
    assert blocks["nw"].tolist() == [256] * 11 + [100]
    dec = O.dequant_blocks(payload, blocks)
    at = 0
    for b in range(12):
        n = int(blocks["nw"][b])
        idx, cb = O.quantize_block(int(fmts[b]), w[at: at + n])
        d = blocks[b]
        assert d["cb_off"] % 16 == 0
        assert np.array_equal(payload[d["cb_off"]: d["cb_off"] + d["cb_bytes"]], cb)
        assert np.array_equal(payload[d["idx_off"]: d["idx_off"] + d["idx_bytes"]], idx)
        assert np.array_equal(dec[at: at + n].view(np.uint32),
                              O.dequantize_block(int(fmts[b]), idx, cb, n).view(np.uint32))
        at += n


@pytest.mark.skipif(O.ref() is None, reason="compiled reference not built in this environment")
def test_against_compiled_reference_random_blocks():
    rng = np.random.default_rng(17)
    for fmt in range(15):
        for n in (256, 255, 129, 64, 33, 31, 9, 7, 3):
            for k in range(3):
                w = (rng.standard_normal(n) * (0.02 if k else 1.0)).astype(np.float32)
                if k == 2:
                    w = np.round(w * 100).astype(np.float32)       # ties
                a, b = O.quantize_block(fmt, w), O.ref_quantize_block(fmt, w)
                assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1]), (fmt, n, k)
                g = rng.integers(0, 256, max(1, a[0].size), dtype=np.uint8).astype(np.uint8)
                gc = rng.integers(0, 256, a[1].size, dtype=np.uint8).astype(np.uint8)
                for cut in (g.size, g.size // 2):
                    x = O.dequantize_block(fmt, g[:cut], gc, n)
                    y = O.ref_dequantize_block(fmt, g[:cut], gc, n)
                    assert np.array_equal(x.view(np.uint32), y.view(np.uint32)), (fmt, n, k, cut)
