"""Flat-codebook entry points through the C ABI (oilhip_flat_*, oilhip_prod_gemv_*,
oilhip_engine_quant_gemm) against the golden vectors of the compiled reference
and against the CPU oracle.  Tolerance: relative L2 <= 1e-5 against the
double-precision result (the reference's own summation order differs between
its scalar and AVX2 builds by about that much)."""
import os

import numpy as np
import pytest

import innova_amd as ia
import oracle as O
from gpu_util import rel_l2

pytestmark = pytest.mark.gpu
TOL = 1e-5
FL = np.load(os.path.join(os.path.dirname(__file__), "golden", "flat.npz"))


def test_golden_oil8_oil4_gemm():
    M, N, K = (int(v) for v in FL["oil8/mnk"])
    got = ia.kernel.oil8_gemm(FL["oil8/idx"], FL["oil8/cb_bits"].view(np.float32), FL["oil8/act_bits"].view(np.float32), M, N, K)
    assert rel_l2(got, FL["oil8/y_bits"].view(np.float32)) <= TOL
    M, N, K = (int(v) for v in FL["oil4/mnk"])
    got = ia.kernel.oil4_gemm(FL["oil4/packed"], FL["oil4/cb16"], FL["oil4/act_bits"].view(np.float32), M, N, K)
    assert rel_l2(got, FL["oil4/y_bits"].view(np.float32)) <= TOL


def test_golden_production_gemv():
    Mg, Kg = (int(v) for v in FL["prod/mk"])
    x = FL["prod/x_bits"].view(np.float32)
    cb16, cb8 = FL["oil4/cb16"], FL["oil8/cb_bits"].view(np.float32)
    assert rel_l2(ia.kernel.gemv_spark_tiled(FL["prod/w_spark"], 0.37, x, Mg, Kg), FL["prod/y_spark_bits"].view(np.float32)) <= TOL
    assert rel_l2(ia.kernel.gemv_oil4_tiled(FL["prod/w_oil4"], cb16, 0.37, x, Mg, Kg), FL["prod/y_oil4_bits"].view(np.float32)) <= TOL
    assert rel_l2(ia.kernel.gemv_oil8_tiled(FL["prod/w_oil8"], cb8, 0.37, x, Mg, Kg), FL["prod/y_oil8_bits"].view(np.float32)) <= TOL


def test_golden_engine_quant_gemm():
    Me, Ne, Ke = (int(v) for v in FL["eng/mnk"])
    A = FL["eng/A_bits"].view(np.float32)
    for bits in (8, 4, 2):
        got = ia.kernel.engine_quant_gemm(bits, A, FL["eng/b"], FL[f"eng/cb{bits}_bits"].view(np.float32), Me, Ne, Ke)
        # same k-order FMA chain as the reference loop: bit-identical
        assert np.array_equal(got.ravel().view(np.uint32), FL[f"eng/c{bits}_bits"])


# K a multiple of 16 and M <= 4 take the register-resident kernel (one and several slabs per row, several chunks per
# wavefront, a partial last column set); the rest the plain one
@pytest.mark.parametrize("M,N,K", [(1, 4096, 4096), (4, 300, 1000), (3, 17, 37), (2, 5, 1), (1, 1000, 11008), (2, 77, 2304),
                                   (4, 300, 1024), (3, 50, 4096), (1, 40000, 512), (1, 9, 16), (1, 5000, 48), (5, 64, 1024)])
def test_oil8_gemm_against_oracle(M, N, K):
    rng = np.random.default_rng(M * 1000 + N + K)
    idx = rng.integers(0, 256, N * K, dtype=np.uint8).astype(np.uint8)
    cb = (rng.standard_normal(256) * 0.02).astype(np.float32)
    act = rng.standard_normal(M * K).astype(np.float32)
    got = ia.kernel.oil8_gemm(idx, cb, act, M, N, K)
    assert rel_l2(got, O.oil8_gemm(idx, cb, act, M, N, K, order=2)) <= TOL
    assert rel_l2(O.oil8_gemm(idx, cb, act, M, N, K, order=1), O.oil8_gemm(idx, cb, act, M, N, K, order=2)) <= TOL


@pytest.mark.parametrize("M,N,K", [(1, 512, 4096), (3, 40, 301), (2, 9, 33)])
def test_oil4_gemm_against_oracle(M, N, K):
    rng = np.random.default_rng(M * 77 + N + K)
    packed = rng.integers(0, 256, (M * N * K + 1) // 2 + 8, dtype=np.uint8).astype(np.uint8)
    cb16 = (rng.standard_normal(16) * 0.5).astype(np.float16).view(np.uint16).copy()
    cb16[2] = 0x0003                 # FP16 subnormal entry
    act = rng.standard_normal(N * K).astype(np.float32)
    got = ia.kernel.oil4_gemm(packed, cb16, act, M, N, K)
    assert rel_l2(got, O.oil4_gemm(packed, cb16, act, M, N, K, order=2)) <= TOL


@pytest.mark.parametrize("M,K,batch", [(1000, 4096, 1), (50, 333, 5), (7, 2, 3), (4096, 11008, 1), (300, 256, 2), (40000, 512, 1),
                                       (77, 2304, 2)])
def test_production_gemv_batch_against_oracle(M, K, batch):
    rng = np.random.default_rng(M + K + batch)
    X = rng.standard_normal((batch, K)).astype(np.float32)
    cb16 = (rng.standard_normal(16)).astype(np.float16).view(np.uint16)
    cb8 = rng.standard_normal(256).astype(np.float32)
    ws = rng.integers(0, 256, M * ((K + 3) // 4), dtype=np.uint8).astype(np.uint8)
    w4 = rng.integers(0, 256, M * ((K + 1) // 2), dtype=np.uint8).astype(np.uint8)
    w8 = rng.integers(0, 256, M * K, dtype=np.uint8).astype(np.uint8)
    ys = ia.kernel.gemv_spark_batch(ws, 1.7, X, M, batch, K)
    y4 = ia.kernel.gemv_oil4_batch(w4, cb16, 1.7, X, M, batch, K)
    y8 = ia.kernel.gemv_oil8_batch(w8, cb8, 1.7, X, M, batch, K)
    assert ys.shape == (batch, M)
    for n in range(batch):                      # Y + n*M holds activation row n (kernel_production.cpp:345-364)
        assert rel_l2(ys[n], O.gemv_spark(ws, 1.7, X[n], M, K, 1)) <= TOL
        assert rel_l2(y4[n], O.gemv_oil4(w4, cb16, 1.7, X[n], M, K, 1)) <= TOL
        assert rel_l2(y8[n], O.gemv_oil8(w8, cb8, 1.7, X[n], M, K, 1)) <= TOL


@pytest.mark.parametrize("bits", [8, 4, 2])
def test_engine_quant_gemm_against_oracle(bits):
    rng = np.random.default_rng(bits)
    M, N, K = 5, 1000, 300
    A = rng.standard_normal((M, K)).astype(np.float32)
    A[:, ::9] = 0.0                               # zero activations are skipped by the reference loop
    b = rng.integers(0, 256, (K * N * bits + 7) // 8, dtype=np.uint8).astype(np.uint8)
    cb = rng.standard_normal(1 << bits).astype(np.float32)
    got = ia.kernel.engine_quant_gemm(bits, A, b, cb, M, N, K)
    want = O.engine_quant_gemm(bits, A, b, cb, M, N, K)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_empty_and_bad_arguments():
    assert ia.kernel.oil8_gemm(np.zeros(0, np.uint8), np.zeros(256, np.float32), np.zeros(0, np.float32), 0, 0, 4).shape == (0, 0)
    with pytest.raises(ia.OilHipError):
        ia.kernel.engine_quant_gemm(3, np.zeros(4, np.float32), np.zeros(4, np.uint8), np.zeros(8, np.float32), 1, 1, 4)


@pytest.mark.parametrize("kind", [1, 3, 16, 32])
def test_engine_dense_gemm_bit_exact(kind):
    """Oil1 / Spark / OIL16 / OIL32 engine quant_gemm on the device: same k order and fused multiply-add as the
    reference build, so the compiled reference's output is reproduced bit for bit."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(os.path.dirname(__file__), "golden", "make_fixtures.py"))
    MF = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(MF)
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "engines.npz"))
    sh = MF.ENGINE_DENSE
    A, B, scales = MF.engine_dense_inputs(kind)
    got = ia.kernel.engine_dense_gemm(kind, A, B, sh["M"], sh["N"], sh["K"], scales=scales, block_size=sh["block"])
    assert np.array_equal(np.asarray(got).view(np.uint32), gold[f"c{kind}"])
    with pytest.raises(ia.OilHipError):
        ia.kernel.engine_dense_gemm(5, A, B, 1, 1, 1)


def test_engine_dequant_bit_exact():
    """dequant_tensor (packed codes) and dequantize_per_block against the compiled reference's outputs."""
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(os.path.dirname(__file__), "golden", "make_fixtures.py"))
    MF = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(MF)
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "engines.npz"))
    for bits in (8, 4, 2):
        idx, n = MF.engine_dequant_inputs(bits)
        got = ia.kernel.engine_dequant(bits, idx, gold[f"cb{bits}"].view(np.float32), n)
        assert np.array_equal(np.asarray(got).view(np.uint32), gold[f"dq{bits}"]), bits
    for bits in (8, 4):
        idx, scales, n, block = MF.engine_block_inputs(bits)
        got = ia.kernel.engine_dequant(bits, idx, gold[f"cb{bits}"].view(np.float32), n, scales=scales, block_size=block)
        assert np.array_equal(np.asarray(got).view(np.uint32), gold[f"pb{bits}"]), bits
    with pytest.raises(ia.OilHipError):
        ia.kernel.engine_dequant(2, np.zeros(4, np.uint8), np.zeros(4, np.float32), 4, scales=np.zeros(1, np.float32), block_size=4)
