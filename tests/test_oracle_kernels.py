"""The CPU oracle's matmul restatements against the golden vectors written by the
compiled reference (tests/golden/block_gemv.npz, flat.npz), against the
compiled reference where built, and against brute force / library reductions."""
import os

import numpy as np
import pytest

import oracle as O

HERE = os.path.dirname(__file__)
GV = np.load(os.path.join(HERE, "golden", "block_gemv.npz"))
FL = np.load(os.path.join(HERE, "golden", "flat.npz"))


def rel_l2(a, b):
    a = np.asarray(a, dtype=np.float64).ravel()
    b = np.asarray(b, dtype=np.float64).ravel()
    d = np.linalg.norm(b)
    return float(np.linalg.norm(a - b) / d) if d > 0 else float(np.linalg.norm(a - b))


def golden_matrix(name):
    """Rebuild (payload, blocks) from the reference payloads stored per block."""
    rows, cols, B = (int(v) for v in GV["shape"])
    il, cl = GV[f"{name}/idx_len"], GV[f"{name}/cb_len"]
    idx, cb = GV[f"{name}/idx"], GV[f"{name}/cb"]
    nb = il.size
    blocks = np.zeros(nb, dtype=O.BLOCK_DTYPE)
    parts, off, io, co = [], 0, 0, 0
    for b in range(nb):
        off = (off + 15) // 16 * 16
        pad = off - sum(p.size for p in parts)
        if pad:
            parts.append(np.zeros(pad, np.uint8))
        blocks[b]["cb_off"] = off
        blocks[b]["idx_off"] = off + cl[b]
        blocks[b]["cb_bytes"] = cl[b]
        blocks[b]["idx_bytes"] = il[b]
        blocks[b]["nw"] = 256
        blocks[b]["fmt"] = O.FORMATS[name]
        parts.append(cb[co: co + cl[b]]); parts.append(idx[io: io + il[b]])
        off += int(cl[b]) + int(il[b]); io += int(il[b]); co += int(cl[b])
    payload = np.concatenate(parts) if parts else np.zeros(0, np.uint8)
    return payload, blocks, rows, cols, B


@pytest.mark.parametrize("name", list(O.FORMATS))
def test_block_gemm_golden(name):
    payload, blocks, rows, cols, B = golden_matrix(name)
    X = GV["x_bits"].view(np.float32).reshape(B, cols)
    want = GV[f"{name}/y_bits"].view(np.float32).reshape(B, rows)
    wide = O.block_gemm(payload, blocks, rows, cols, X, wide=True)
    assert np.array_equal(wide.view(np.uint32), want.view(np.uint32))
    f32 = O.block_gemm(payload, blocks, rows, cols, X, wide=False)
    assert rel_l2(f32, want) < 2e-6
    # the oracle's own encoder reproduces the reference payloads from the same weights
    mine, myblocks = O.quantize_tensor(GV["w_bits"].view(np.float32), O.FORMATS[name], align=16)
    assert np.array_equal(mine, payload) and np.array_equal(myblocks, blocks)


def test_block_gemm_brute_force_mixed_and_threads():
    rng = np.random.default_rng(1)
    rows, cols, B = 10, 512, 2
    w = (rng.standard_normal(rows * cols) * 0.02).astype(np.float32)
    fmts = rng.integers(0, 15, rows * cols // 256).astype(np.uint8)
    payload, blocks = O.quantize_tensor(w, fmts)
    X = rng.standard_normal((B, cols)).astype(np.float32)
    Wd = O.dequant_blocks(payload, blocks).reshape(rows, cols).astype(np.float64)
    want = (X.astype(np.float64) @ Wd.T)
    for th in (1, 3, 0):
        got = O.block_gemm(payload, blocks, rows, cols, X, wide=True, threads=th)
        assert np.allclose(got, want, rtol=1e-6, atol=1e-9)
        got32 = O.block_gemm(payload, blocks, rows, cols, X, wide=False, threads=th)
        assert rel_l2(got32, want) < 2e-6
    # transposing X or W would show here: rows != cols, B > 1
    assert got.shape == (B, rows)


def test_flat_golden():
    M, N, K = (int(v) for v in FL["oil8/mnk"])
    y = O.oil8_gemm(FL["oil8/idx"], FL["oil8/cb_bits"].view(np.float32), FL["oil8/act_bits"].view(np.float32), M, N, K, order=1)
    assert np.array_equal(y.ravel().view(np.uint32), FL["oil8/y_bits"])
    M, N, K = (int(v) for v in FL["oil4/mnk"])
    y = O.oil4_gemm(FL["oil4/packed"], FL["oil4/cb16"], FL["oil4/act_bits"].view(np.float32), M, N, K, order=1)
    assert np.array_equal(y.ravel().view(np.uint32), FL["oil4/y_bits"])
    Mg, Kg = (int(v) for v in FL["prod/mk"])
    x = FL["prod/x_bits"].view(np.float32)
    assert np.array_equal(O.gemv_spark(FL["prod/w_spark"], 0.37, x, Mg, Kg, 2).view(np.uint32), FL["prod/y_spark_bits"])
    assert np.array_equal(O.gemv_oil4(FL["prod/w_oil4"], FL["oil4/cb16"], 0.37, x, Mg, Kg, 2).view(np.uint32), FL["prod/y_oil4_bits"])
    assert np.array_equal(O.gemv_oil8(FL["prod/w_oil8"], FL["oil8/cb_bits"].view(np.float32), 0.37, x, Mg, Kg, 2).view(np.uint32), FL["prod/y_oil8_bits"])
    Me, Ne, Ke = (int(v) for v in FL["eng/mnk"])
    for bits in (8, 4, 2):
        c = O.engine_quant_gemm(bits, FL["eng/A_bits"].view(np.float32), FL["eng/b"],
                                FL[f"eng/cb{bits}_bits"].view(np.float32), Me, Ne, Ke)
        assert np.array_equal(c.ravel().view(np.uint32), FL[f"eng/c{bits}_bits"])


def test_flat_reduce_to_library_matmul():
    rng = np.random.default_rng(2)
    M, N, K = 4, 9, 64
    # OIL8 with an identity-like codebook is an ordinary X . W^T
    idx = rng.integers(0, 256, N * K, dtype=np.uint8).astype(np.uint8)
    cb = np.arange(256, dtype=np.float32)
    act = rng.standard_normal((M, K)).astype(np.float32)
    want = act.astype(np.float64) @ idx.reshape(N, K).astype(np.float64).T
    for order in (0, 1, 2):
        assert np.allclose(O.oil8_gemm(idx, cb, act, M, N, K, order), want, rtol=1e-5, atol=1e-3)
    # OIL4: weights per (m, n) pair, activations per n, low nibble first
    packed = rng.integers(0, 256, M * N * K // 2, dtype=np.uint8).astype(np.uint8)
    cb16 = np.arange(16, dtype=np.float16).view(np.uint16)
    act4 = rng.standard_normal((N, K)).astype(np.float32)
    nib = np.stack([packed & 15, packed >> 4], axis=1).reshape(M, N, K).astype(np.float64)
    want = np.einsum("mnk,nk->mn", nib, act4.astype(np.float64))
    for order in (0, 1, 2):
        assert np.allclose(O.oil4_gemm(packed, cb16, act4, M, N, K, order), want, rtol=1e-5, atol=1e-3)
    # production: y = scale * W x ; SPARK code 0 -> -1, 1 -> 0, 2/3 -> +1
    Mg, Kg = 5, 50
    x = rng.standard_normal(Kg).astype(np.float32)
    ws = rng.integers(0, 256, Mg * ((Kg + 3) // 4), dtype=np.uint8).astype(np.uint8)
    codes = np.stack([(ws >> s) & 3 for s in (0, 2, 4, 6)], axis=1).reshape(Mg, -1)[:, :Kg]
    tern = np.where(codes == 0, -1.0, np.where(codes == 1, 0.0, 1.0))
    assert np.allclose(O.gemv_spark(ws, 0.5, x, Mg, Kg, 1), 0.5 * (tern @ x.astype(np.float64)), rtol=1e-6)
    # engine [K][N] layout: C = A . B with B[k][n] = cb[code(k*N+n)], zero rows of A skipped
    Me, Ne, Ke = 3, 8, 12
    A = rng.standard_normal((Me, Ke)).astype(np.float32)
    A[0, 3] = 0
    b = rng.integers(0, 256, Ke * Ne, dtype=np.uint8).astype(np.uint8)
    cb4 = rng.standard_normal(16).astype(np.float32)
    codes4 = np.stack([b & 15, b >> 4], axis=1).reshape(-1)[: Ke * Ne].reshape(Ke, Ne)
    want = A.astype(np.float64) @ cb4[codes4].astype(np.float64)
    assert np.allclose(O.engine_quant_gemm(4, A, b, cb4, Me, Ne, Ke, True), want, rtol=1e-6, atol=1e-7)


@pytest.mark.skipif(O.ref() is None, reason="compiled reference not built in this environment")
def test_flat_against_compiled_reference():
    import ctypes as C
    R = O.ref(True)
    f32p, u8p, u16p = C.POINTER(C.c_float), C.POINTER(C.c_uint8), C.POINTER(C.c_uint16)
    rng = np.random.default_rng(4)
    for (M, N, K) in [(1, 7, 256), (3, 5, 100), (2, 4, 37)]:
        idx = rng.integers(0, 256, N * K, dtype=np.uint8).astype(np.uint8)
        cb = rng.standard_normal(256).astype(np.float32)
        act = rng.standard_normal(M * K).astype(np.float32)
        out = np.zeros(M * N, np.float32)
        R.ref_oil8_gemm(idx.ctypes.data_as(u8p), cb.ctypes.data_as(f32p), act.ctypes.data_as(f32p),
                        out.ctypes.data_as(f32p), M, N, K)
        assert np.array_equal(out, O.oil8_gemm(idx, cb, act, M, N, K, 1).ravel())
        pk = rng.integers(0, 256, M * N * K // 2 + 8, dtype=np.uint8).astype(np.uint8)
        cb16 = rng.standard_normal(16).astype(np.float16).view(np.uint16)
        act4 = rng.standard_normal(N * K).astype(np.float32)
        out = np.zeros(M * N, np.float32)
        R.ref_oil4_gemm(pk.ctypes.data_as(u8p), cb16.ctypes.data_as(u16p), act4.ctypes.data_as(f32p),
                        out.ctypes.data_as(f32p), M, N, K)
        assert np.array_equal(out, O.oil4_gemm(pk, cb16, act4, M, N, K, 1).ravel())


@pytest.mark.parametrize("kind", [1, 3, 16, 32])
def test_engine_dense_gemm_matches_reference(kind):
    """Oil1 / Spark / OIL16 / OIL32 engine quant_gemm: oracle bit-equal to the compiled reference's output."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(os.path.dirname(__file__), "golden", "make_fixtures.py"))
    MF = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(MF)
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "engines.npz"))
    sh = MF.ENGINE_DENSE
    A, B, scales = MF.engine_dense_inputs(kind)
    got = O.engine_dense_gemm(kind, A, B, sh["M"], sh["N"], sh["K"], scales, sh["block"])
    assert np.array_equal(got.view(np.uint32), gold[f"c{kind}"])
    # brute force in double on the decoded operand
    flat = np.arange(sh["K"] * sh["N"])
    if kind == 1:
        dense = B[flat // 32]
    elif kind == 32:
        dense = B
    elif kind == 16:
        dense = B.view(np.float16).astype(np.float32)
    else:
        code = (B[flat // 4] >> ((flat % 4) * 2)) & 3
        dense = np.where(code == 2, 1.0, np.where(code == 0, -1.0, 0.0)) * scales[flat // sh["block"]]
    want = A.astype(np.float64) @ np.asarray(dense, np.float64).reshape(sh["K"], sh["N"])
    assert np.linalg.norm(got - want) / np.linalg.norm(want) < 1e-5


# ------------------------------------------------------------------ SPARK lookup kernels (tl1_gemm / tl2_gemm)
TL = np.load(os.path.join(HERE, "golden", "tl.npz"))


@pytest.mark.parametrize("i", range(len(TL["cases"])))
def test_tl_gemm_matches_golden(i):
    """Outputs of the compiled reference's tl1_gemm / tl2_gemm (src/kernel_tl.cpp:32-90,124-184), bit for bit."""
    kind, M, N, K = (int(v) for v in TL["cases"][i])
    got = O.tl_gemm(kind, TL[f"w{i}"], TL[f"a{i}"], M, N, K)
    assert np.array_equal(got.view(np.uint32), TL[f"out{i}"])


@pytest.mark.parametrize("kind", [1, 2])
def test_tl_gemm_is_an_integer_matrix_product(kind):
    """With activations small enough that no pair sum leaves int8, both kernels are an integer matrix product of the
    int8 activations with the ternary weights, divided by the row's scale."""
    rng = np.random.default_rng(77 + kind)
    M, N, K = 5, 4, 48
    rb = O.tl_row_bytes(kind, K)
    w = rng.integers(0, 256, size=M * N * rb, dtype=np.uint8)
    a = rng.uniform(-0.45, 0.45, size=(N, K)).astype(np.float32)
    a[:, 0], a[:, 1] = 1.0, 0.0                                # the row maximum beside a zero: every other |code| < 64
    codes = (w.reshape(M * N, rb)[:, :, None] >> (2 * np.arange(4))[None, None, :]) & 3
    tern = np.where(codes == 0, -1, np.where(codes == 1, 0, 1)).reshape(M * N, rb * 4)[:, :K].reshape(M, N, K)
    scale = np.float32(127.0) / np.abs(a).max(axis=1).astype(np.float32)
    v = (a * scale[:, None]).astype(np.float32)
    q = (np.sign(v) * np.floor(np.abs(v) + np.float32(0.5))).astype(np.int64)      # round half away from zero
    want = (np.einsum("mnk,nk->mn", tern, q).astype(np.float32) / scale[None, :]).astype(np.float32)
    got = O.tl_gemm(kind, w, a, M, N, K)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_tl1_pair_sums_saturate():
    """Two full-scale activations under two +1 weights: 127 + 127 is stored as 127 (the table entry is an int8)."""
    a = np.array([[1.0, 1.0, -1.0, -1.0]], dtype=np.float32)
    w = np.array([0b10101010], dtype=np.uint8)                  # four +1 weights
    assert O.tl_gemm(1, w, a, 1, 1, 4)[0, 0] == np.float32((127 - 128) / 127.0)
    assert O.tl_gemm(2, np.array([0b10101010, 0, 0], np.uint8), np.array([[1.0, 1.0, -1.0]], np.float32), 1, 1, 3)[0, 0] == np.float32(1.0)


def test_tl_gemm_matches_compiled_reference():
    R = O.ref()
    if R is None:
        pytest.skip("compiled reference not built")
    rng = np.random.default_rng(99)
    for kind in (1, 2):
        for _ in range(6):
            M, N = int(rng.integers(1, 6)), int(rng.integers(1, 6))
            K = int(rng.integers(1, 400)) if kind == 1 else 3 * int(rng.integers(1, 130))
            w = rng.integers(0, 256, size=M * N * O.tl_row_bytes(kind, K), dtype=np.uint8)
            a = (rng.standard_normal((N, K)) * 10.0 ** rng.integers(-4, 3)).astype(np.float32)
            got = O.tl_gemm(kind, w, a, M, N, K)
            ref = O.tl_gemm(kind, w, a, M, N, K, fn=R.ref_tl_gemm)
            assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), (kind, M, N, K)
