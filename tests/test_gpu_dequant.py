"""GPU dequantize (oilhip_dequant_f32 through the C ABI) is bit-exact with the
reference decode: against the golden vectors written by the compiled reference
and against the CPU oracle on fresh tensors, all 15 formats, full, ragged and
truncated blocks."""
import os

import numpy as np
import pytest

import innova_amd as ia
import oracle as O
from gpu_util import gaussian_weights, to_orc_blocks

pytestmark = pytest.mark.gpu
G = np.load(os.path.join(os.path.dirname(__file__), "golden", "codec.npz"))


def test_probe_reports_gfx950():
    p = ia.probe()
    assert p["gfx"] == 950 and p["compute_units"] > 0 and p["hbm_bytes"] > (64 << 30)


def test_golden_blocks_bit_exact():
    """Every golden case in one upload: one block per case, its own format and length."""
    n_case = G["fmt"].size
    blocks = np.zeros(n_case, dtype=ia._lib.BLOCK_DTYPE)
    cb_base = G["idx"].size
    payload = np.concatenate([G["idx"], G["cb"], np.zeros(16, np.uint8)])
    blocks["fmt"], blocks["nw"] = G["fmt"], G["n"]
    blocks["idx_off"], blocks["idx_bytes"] = G["idx_off"], G["idx_len"]
    blocks["cb_off"], blocks["cb_bytes"] = G["cb_off"] + cb_base, G["cb_len"]
    total = int(G["n"].sum())
    with ia.DeviceWeights.from_blocks(payload, blocks, 1, total) as dw:
        got = dw.dequant().cpu().numpy().view(np.uint32)
    want = G["dec_bits"]
    bad = np.nonzero(got != want)[0]
    if bad.size:
        case = int(np.searchsorted(G["dec_off"], bad[0], side="right") - 1)
        raise AssertionError(f"{bad.size} mismatching weights, first in case {G['tags'][case]}")


@pytest.mark.parametrize("fmt", list(ia.Format))
def test_fresh_tensor_bit_exact(fmt):
    w = gaussian_weights(256 * 301 + 100, seed=100 + int(fmt), outlier_every=17)   # ragged last block
    w[256 * 5: 256 * 6] = 0.0                                                     # an all-zero block
    w[256 * 9: 256 * 10] *= np.float32(1e-6)                                      # FP16 scale underflow
    payload, blocks = ia.block_codec.quantize_tensor(w, fmt)
    with ia.DeviceWeights.from_blocks(payload, blocks, 1, w.size) as dw:
        got = dw.dequant().cpu().numpy()
    want = O.dequant_blocks(payload, to_orc_blocks(blocks))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_mixed_formats_and_record_framing():
    rng = np.random.default_rng(5)
    nb = 600
    w = gaussian_weights(256 * nb, seed=6, outlier_every=11)
    fmts = rng.integers(0, 15, nb).astype(np.uint8)
    payload, blocks = ia.block_codec.quantize_tensor(w, fmts)
    want = O.dequant_blocks(payload, to_orc_blocks(blocks))
    with ia.DeviceWeights.from_blocks(payload, blocks, nb, 256) as dw:
        assert dw.info()["uniform_fmt"] == -1
        assert dw.info()["payload_bytes"] == int(blocks["cb_bytes"].sum() + blocks["idx_bytes"].sum())
        got = dw.dequant().cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # the same blocks as on-disk records [nw][cb_bytes][cb][idx_bytes][idx]
    rec = bytearray()
    for b in blocks:
        rec += np.uint32(b["nw"]).tobytes() + np.uint32(b["cb_bytes"]).tobytes()
        rec += payload[b["cb_off"]: b["cb_off"] + b["cb_bytes"]].tobytes()
        rec += np.uint32(b["idx_bytes"]).tobytes()
        rec += payload[b["idx_off"]: b["idx_off"] + b["idx_bytes"]].tobytes()
    with ia.DeviceWeights.from_records(np.frombuffer(bytes(rec), dtype=np.uint8), fmts, nb, 256) as dw:
        got2 = dw.dequant().cpu().numpy()
    assert np.array_equal(got2.view(np.uint32), want.view(np.uint32))


def test_truncated_and_garbage_payloads_match_reference_rules():
    rng = np.random.default_rng(8)
    for fmt in ia.Format:
        for n in (256, 100, 31, 7):
            idx, cb = ia.block_codec.quantize_block_all(fmt, gaussian_weights(n, 9, 1.0))
            garbage = rng.integers(0, 256, max(1, idx.size), dtype=np.uint8).astype(np.uint8)
            gcb = rng.integers(0, 256, cb.size, dtype=np.uint8).astype(np.uint8)
            for cut in (garbage.size, garbage.size // 2, 1):
                got = ia.block_codec.dequantize_block_all(fmt, garbage[:cut], gcb, n)
                want = O.dequantize_block(int(fmt), garbage[:cut], gcb, n)
                assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (fmt, n, cut)


@pytest.mark.parametrize("fmt,nbytes", [(ia.Format.OIL4, 128), (ia.Format.OIL8, 256), (ia.Format.OIL2, 64),
                                        (ia.Format.OIL1, 16), (ia.Format.SPARK_Q0, 48), (ia.Format.OIL16, 512),
                                        (ia.Format.OIL32, 1024), (ia.Format.OIL1_GRP, 32), (ia.Format.SPARK_Q0_GRP, 48),
                                        (ia.Format.OIL2_GRP, 80), (ia.Format.OIL4_GRP, 144), (ia.Format.OIL8_GRP, 272),
                                        (ia.Format.OIL16_GRP, 512), (ia.Format.SPARK_SPARSE, 64),
                                        (ia.Format.SPARK_SPARSE_GRP, 64)])
def test_uniform_full_blocks_random_payload_bit_exact(fmt, nbytes):
    """Tensors of full blocks of one fixed-size format take the wavefront-per-block kernels: random payload bytes (every
    code, scales and zero points including subnormals, infinities and NaNs, zero scales) against the oracle, and
    quantized data against it as well."""
    rng = np.random.default_rng(int(fmt) + 40)
    nb = 3001
    payload = rng.integers(0, 256, nb * nbytes, dtype=np.uint8).astype(np.uint8)
    blocks = np.zeros(nb, dtype=ia._lib.BLOCK_DTYPE)
    blocks["cb_off"] = np.arange(nb, dtype=np.uint64) * nbytes
    if fmt == ia.Format.OIL1:                      # the run means live in the codebook channel
        blocks["cb_bytes"], blocks["idx_off"], blocks["idx_bytes"] = nbytes, blocks["cb_off"] + nbytes, 0
    else:
        blocks["idx_off"], blocks["idx_bytes"] = blocks["cb_off"], nbytes
    blocks["nw"], blocks["fmt"] = 256, int(fmt)
    with ia.DeviceWeights.from_blocks(payload, blocks, nb, 256) as dw:
        assert dw.info()["uniform_fmt"] == int(fmt)
        got = dw.dequant().cpu().numpy()
    want = O.dequant_blocks(payload, to_orc_blocks(blocks))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    w = gaussian_weights(256 * 777, seed=3 + int(fmt), outlier_every=19)
    payload, blocks = ia.block_codec.quantize_tensor(w, fmt)
    with ia.DeviceWeights.from_blocks(payload, blocks, 777, 256) as dw:
        got = dw.dequant().cpu().numpy()
    assert np.array_equal(got.view(np.uint32), O.dequant_blocks(payload, to_orc_blocks(blocks)).view(np.uint32))


def test_full_size_tensor_oil4_bit_exact():
    """The 4096 x 11008 OIL4 matrix of the decode benchmark, checked whole."""
    rows, cols = 11008, 4096
    w = gaussian_weights(rows * cols, seed=1)
    payload, blocks = ia.block_codec.quantize_tensor(w, ia.Format.OIL4)
    assert payload.size == 22544384
    with ia.DeviceWeights.from_blocks(payload, blocks, rows, cols) as dw:
        got = dw.dequant().cpu().numpy()
    want = O.dequant_blocks(payload, to_orc_blocks(blocks))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_bad_arguments_raise():
    blocks = np.zeros(1, dtype=ia._lib.BLOCK_DTYPE)
    blocks[0]["nw"], blocks[0]["fmt"], blocks[0]["idx_bytes"] = 256, 3, 128
    with pytest.raises(ia.OilHipError):
        ia.DeviceWeights.from_blocks(np.zeros(64, np.uint8), blocks, 1, 256)      # payload too short
    blocks[0]["idx_bytes"] = 64
    blocks[0]["fmt"] = 99
    with pytest.raises(ia.OilHipError):
        ia.DeviceWeights.from_blocks(np.zeros(64, np.uint8), blocks, 1, 256)      # unknown format
    blocks[0]["fmt"] = 3
    with pytest.raises(ia.OilHipError):
        ia.DeviceWeights.from_blocks(np.zeros(64, np.uint8), blocks, 2, 256)      # rows*cols mismatch
