"""SPARK lookup kernels (oilhip_tl_gemm), the profiling hooks (oilhip_profile_gemv) and the dense FP32 operations of
the backend object (oilhip_dense_*) through the C ABI.  The lookup kernels are integer work: bit-identical to the
compiled reference's outputs (tests/golden/tl.npz) and to the CPU oracle.  The dense operations are floating point:
relative L2 <= 1e-5 (gemm, gemv: FP32 sums in another order than the reference's k loop) and <= 1e-6 (norms, softmax,
activations: same formula, sums in double on both sides) against NumPy in double precision."""
import ctypes as C
import os

import numpy as np
import pytest

import innova_amd as ia
import oracle as O
from innova_amd import _lib
from gpu_util import rel_l2

pytestmark = pytest.mark.gpu
TL = np.load(os.path.join(os.path.dirname(__file__), "golden", "tl.npz"))


@pytest.mark.parametrize("i", range(len(TL["cases"])))
def test_tl_gemm_golden(i):
    kind, M, N, K = (int(v) for v in TL["cases"][i])
    fn = ia.kernel.tl1_gemm if kind == 1 else ia.kernel.tl2_gemm
    got = fn(TL[f"w{i}"], TL[f"a{i}"], M, N, K)
    assert np.array_equal(got.ravel().view(np.uint32), TL[f"out{i}"].ravel())


@pytest.mark.parametrize("kind,M,N,K", [(1, 64, 48, 4096), (2, 64, 48, 4092), (1, 1, 2000, 31), (2, 300, 1, 768)])
def test_tl_gemm_oracle(kind, M, N, K):
    rng = np.random.default_rng(K + kind)
    w = rng.integers(0, 256, size=M * N * O.tl_row_bytes(kind, K), dtype=np.uint8)
    a = (rng.standard_normal((N, K)) * 10.0 ** rng.integers(-3, 3, size=(N, 1))).astype(np.float32)
    fn = ia.kernel.tl1_gemm if kind == 1 else ia.kernel.tl2_gemm
    got = fn(w, a, M, N, K)
    assert np.array_equal(got.view(np.uint32), O.tl_gemm(kind, w, a, M, N, K).view(np.uint32))


def test_tl_gemm_rejects_what_the_reference_leaves_undefined():
    w = np.zeros(64, np.uint8)
    a = np.ones((1, 16), np.float32)
    with pytest.raises(_lib.OilHipError):
        ia.kernel.tl2_gemm(w, a, 1, 1, 16)          # a triple would straddle the end of the activation row
    with pytest.raises(_lib.OilHipError):
        ia.kernel._tl(3, w, a, 1, 1, 15)


def test_profile_gemv_fills_kernel_perf():
    rng = np.random.default_rng(3)
    M, K = 2048, 4096
    x = rng.standard_normal(K).astype(np.float32)
    cb16 = rng.standard_normal(16).astype(np.float16).view(np.uint16)
    cb8 = rng.standard_normal(256).astype(np.float32)
    w4 = rng.integers(0, 256, M * K // 2, dtype=np.uint8)
    w8 = rng.integers(0, 256, M * K, dtype=np.uint8)
    ws = rng.integers(0, 256, M * K // 4, dtype=np.uint8)
    for perf, y, want, read in (
            ia.kernel._profile(4, w4, cb16, np.uint16, 0.5, x, M, K, 20) + (O.gemv_oil4(w4, cb16, 0.5, x, M, K, 1), M * K // 2 + M * K * 4),
            ia.kernel._profile(8, w8, cb8, np.float32, 0.5, x, M, K, 20) + (O.gemv_oil8(w8, cb8, 0.5, x, M, K, 1), M * K + M * 1024),
            ia.kernel._profile(0, ws, None, None, 0.5, x, M, K, 20) + (O.gemv_spark(ws, 0.5, x, M, K, 1), M * K * 2)):
        assert perf.bytes_read == read and perf.bytes_written == M * 4          # src/kernel_production.cpp:445-446,462-463,479-480
        assert perf.cycles > 0 and 1.0 < perf.gflops < 1e6
        assert rel_l2(y.cpu().numpy(), want) <= 1e-5                            # y holds the GEMV's result afterwards
    p = ia.kernel.profile_gemv_oil4(w4, cb16, 0.5, x, M, K)
    assert isinstance(p, ia.kernel.KernelPerf) and p.gflops > 0


def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a, np.float32)).cuda()


def test_dense_gemm_gemv():
    import torch
    L = _lib.lib()
    rng = np.random.default_rng(11)
    for (M, N, K, alpha, beta) in [(67, 130, 45, 0.75, -0.5), (1, 1, 1, 1.0, 0.0), (256, 64, 512, 1.0, 1.0), (5, 200, 0, 2.0, 0.5)]:
        A, B, Cm = rng.standard_normal((M, K)), rng.standard_normal((K, N)), rng.standard_normal((M, N))
        dA, dB, dC = _dev(A), _dev(B), _dev(Cm)
        _lib.check(L.oilhip_dense_gemm_f32(alpha, dA.data_ptr(), dB.data_ptr(), beta, dC.data_ptr(), M, N, K, _lib.current_stream()))
        want = alpha * (A.astype(np.float32).astype(np.float64) @ B.astype(np.float32).astype(np.float64)) + beta * Cm.astype(np.float32)
        assert rel_l2(dC.cpu().numpy(), want) <= 1e-5, (M, N, K)
    # beta == 0 must not read C (NaN in the output buffer stays out of the result)
    dC = torch.full((8, 8), float("nan"), device="cuda")
    dA, dB = _dev(np.eye(8)), _dev(np.eye(8))
    _lib.check(L.oilhip_dense_gemm_f32(1.0, dA.data_ptr(), dB.data_ptr(), 0.0, dC.data_ptr(), 8, 8, 8, _lib.current_stream()))
    assert np.array_equal(dC.cpu().numpy(), np.eye(8, dtype=np.float32))
    for (M, N) in [(129, 300), (1, 7), (1000, 64)]:
        A, x, y = rng.standard_normal((M, N)), rng.standard_normal(N), rng.standard_normal(M)
        dA, dx, dy = _dev(A), _dev(x), _dev(y)
        _lib.check(L.oilhip_dense_gemv_f32(2.0, dA.data_ptr(), dx.data_ptr(), 0.25, dy.data_ptr(), M, N, _lib.current_stream()))
        want = 2.0 * (A.astype(np.float32).astype(np.float64) @ x.astype(np.float32).astype(np.float64)) + 0.25 * y.astype(np.float32)
        assert rel_l2(dy.cpu().numpy(), want) <= 1e-5


def test_dense_norms_softmax_and_maps():
    import torch
    from scipy.special import erf
    L = _lib.lib()
    rng = np.random.default_rng(12)
    x = (rng.standard_normal((9, 515)) * 2.0 + 0.3).astype(np.float32)
    g, b = rng.standard_normal(515).astype(np.float32), rng.standard_normal(515).astype(np.float32)
    dx, dg, db = _dev(x), _dev(g), _dev(b)
    dy = torch.empty_like(dx)
    x64 = x.astype(np.float64)
    _lib.check(L.oilhip_dense_norm_f32(0, dx.data_ptr(), dg.data_ptr(), db.data_ptr(), 1e-5, dy.data_ptr(), 9, 515, _lib.current_stream()))
    mu, var = x64.mean(1, keepdims=True), x64.var(1, keepdims=True)
    assert rel_l2(dy.cpu().numpy(), (x64 - mu) / np.sqrt(var + np.float32(1e-5)) * g + b) <= 1e-6
    _lib.check(L.oilhip_dense_norm_f32(1, dx.data_ptr(), dg.data_ptr(), None, 1e-6, dy.data_ptr(), 9, 515, _lib.current_stream()))
    assert rel_l2(dy.cpu().numpy(), x64 / np.sqrt((x64 ** 2).mean(1, keepdims=True) + np.float32(1e-6)) * g) <= 1e-6
    t = (rng.standard_normal((5, 33, 7)) * 3.0).astype(np.float32)
    dt = _dev(t)
    do = torch.empty_like(dt)
    for axis in (0, 1, 2):
        outer = int(np.prod(t.shape[:axis], dtype=np.int64))
        inner = int(np.prod(t.shape[axis + 1:], dtype=np.int64))
        _lib.check(L.oilhip_dense_softmax_f32(dt.data_ptr(), do.data_ptr(), outer, t.shape[axis], inner, _lib.current_stream()))
        e = np.exp(t.astype(np.float64) - t.max(axis=axis, keepdims=True))
        assert rel_l2(do.cpu().numpy(), e / e.sum(axis=axis, keepdims=True)) <= 1e-6, axis
    n = 100003
    a, c = (rng.standard_normal(n) * 2.0).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    da, dc = _dev(a), _dev(c)
    dz = torch.empty_like(da)
    a64 = a.astype(np.float64)
    cases = {0: np.maximum(a, 0), 1: 0.5 * a64 * (1.0 + erf(a64 * 0.7071067811865475)), 2: a64 / (1.0 + np.exp(-a64)),
             3: a + c, 4: a * c, 5: np.float32(-1.5) * a, 6: np.full(n, -1.5, np.float32)}
    for op, want in cases.items():
        _lib.check(L.oilhip_dense_map_f32(op, da.data_ptr(), dc.data_ptr(), -1.5, dz.data_ptr(), n, _lib.current_stream()))
        got = dz.cpu().numpy()
        if op in (0, 3, 4, 5, 6):
            assert np.array_equal(got, want.astype(np.float32)), op
        else:
            assert rel_l2(got, want) <= 1e-6, op
    with pytest.raises(_lib.OilHipError):
        _lib.check(L.oilhip_dense_map_f32(9, da.data_ptr(), dc.data_ptr(), 0.0, dz.data_ptr(), n, _lib.current_stream()))


def test_backend_object_mirrors_the_dispatch():
    """probe -> select -> create -> operate, as a caller of backend.h:98-139 would."""
    B = ia.backend
    hw = B.probe_hardware()
    assert hw["has_hip_gfx950"] and hw["vram_total"] > 64 << 30
    cfg = B.select_optimal_backend(hw, 14 << 30)
    assert cfg["type"] == B.BackendType.GPU_HIP_GFX950 and cfg["device_name"] == "hip-gfx950"
    assert B.select_optimal_backend(hw, 1 << 50)["type"] is None
    be = B.create(cfg)
    assert be.name() == "hip-gfx950" and be.is_available() and 0 < be.memory_free() <= be.memory_total()
    rng = np.random.default_rng(5)
    A, Bm = rng.standard_normal((33, 70)).astype(np.float32), rng.standard_normal((70, 21)).astype(np.float32)
    assert rel_l2(be.gemm(1.0, A, Bm), A.astype(np.float64) @ Bm) <= 1e-5
    x = rng.standard_normal(70).astype(np.float32)
    assert rel_l2(be.gemv(0.5, A, x), 0.5 * (A.astype(np.float64) @ x)) <= 1e-5
    assert np.array_equal(be.add(A, A), A + A) and np.array_equal(be.relu(A), np.maximum(A, 0))
    s = be.softmax(A, -1)
    assert np.allclose(s.sum(-1), 1.0, atol=1e-6)
    with pytest.raises(_lib.OilHipError):
        be.gemm(1.0, A, A)
    be.synchronize()
