"""Host mirror of the reference's flat-codebook kernel entry points
(include/oil/kernel.h:24-32, include/oil/kernel_production.h:25-52,
include/oil/oil_engines.h quant_gemm).  Arguments may be numpy arrays (uploaded
per call, as the reference's host-pointer signatures imply) or cuda tensors
(used in place); results come back in the same kind."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib


def _dev(a, np_dtype):
    import torch
    if isinstance(a, torch.Tensor):
        assert a.is_cuda and a.is_contiguous()
        return a, True
    t = torch.from_numpy(np.ascontiguousarray(a, dtype=np_dtype).reshape(-1).view(
        np.int16 if np_dtype == np.uint16 else np_dtype)).cuda()
    return t, False


def _ret(out, on_device):
    return out if on_device else out.cpu().numpy()


def oil8_gemm(indices, codebook, activations, M: int, N: int, K: int):
    """out[m*N+n] = sum_k codebook[indices[n*K+k]] * activations[m*K+k]  (kernel.h:24-26)."""
    import torch
    i, d1 = _dev(indices, np.uint8)
    c, _ = _dev(codebook, np.float32)
    a, d2 = _dev(activations, np.float32)
    out = torch.empty((M, N), dtype=torch.float32, device="cuda")
    _lib.check(_lib.lib().oilhip_flat_oil8_gemm(i.data_ptr(), c.data_ptr(), a.data_ptr(), out.data_ptr(),
                                                M, N, K, _lib.current_stream()))
    return _ret(out, d1 and d2)


def oil4_gemm(packed_indices, codebook, activations, M: int, N: int, K: int):
    """out[m*N+n] = sum_k f16(codebook[nib((m*N+n)*K+k)]) * activations[n*K+k]  (kernel.h:30-32)."""
    import torch
    i, d1 = _dev(packed_indices, np.uint8)
    c, _ = _dev(codebook, np.uint16)
    a, d2 = _dev(activations, np.float32)
    out = torch.empty((M, N), dtype=torch.float32, device="cuda")
    _lib.check(_lib.lib().oilhip_flat_oil4_gemm(i.data_ptr(), c.data_ptr(), a.data_ptr(), out.data_ptr(),
                                                M, N, K, _lib.current_stream()))
    return _ret(out, d1 and d2)


def _prod(fn, w, cb, cb_dtype, scale, X, M, N, K):
    import torch
    wd, d1 = _dev(w, np.uint8)
    xd, d2 = _dev(X, np.float32)
    Y = torch.empty((N, M), dtype=torch.float32, device="cuda")
    if cb is None:
        _lib.check(fn(wd.data_ptr(), float(scale), xd.data_ptr(), Y.data_ptr(), M, K, N, _lib.current_stream()))
    else:
        cd, _ = _dev(cb, cb_dtype)
        _lib.check(fn(wd.data_ptr(), cd.data_ptr(), float(scale), xd.data_ptr(), Y.data_ptr(), M, K, N,
                      _lib.current_stream()))
    return _ret(Y, d1 and d2)


def gemv_spark_batch(packed_w, scale, X, M: int, N: int, K: int):
    """Y[n*M+m] = scale * sum_k tern(W[m][k]) * X[n*K+k]  (kernel_production.h:40-42)."""
    return _prod(_lib.lib().oilhip_prod_gemv_spark, packed_w, None, None, scale, X, M, N, K)


def gemv_oil4_batch(packed_indices, codebook, scale, X, M: int, N: int, K: int):
    return _prod(_lib.lib().oilhip_prod_gemv_oil4, packed_indices, codebook, np.uint16, scale, X, M, N, K)


def gemv_oil8_batch(indices, codebook, scale, X, M: int, N: int, K: int):
    return _prod(_lib.lib().oilhip_prod_gemv_oil8, indices, codebook, np.float32, scale, X, M, N, K)


def gemv_spark_tiled(packed_w, scale, x, M: int, K: int, tile_m: int = 32):
    """y = scale * (W @ x)  (kernel_production.h:25-27); tile_m is a CPU cache hint, unused here."""
    return gemv_spark_batch(packed_w, scale, x, M, 1, K).reshape(-1)


def gemv_oil4_tiled(packed_indices, codebook, scale, x, M: int, K: int, tile_m: int = 32):
    return gemv_oil4_batch(packed_indices, codebook, scale, x, M, 1, K).reshape(-1)


def gemv_oil8_tiled(indices, codebook, scale, x, M: int, K: int, tile_m: int = 32):
    return gemv_oil8_batch(indices, codebook, scale, x, M, 1, K).reshape(-1)


def engine_quant_gemm(bits: int, a, b_idx, codebook, M: int, N: int, K: int):
    """C[m*N+n] = sum_k A[m*K+k] * codebook[code(k*N+n)]: OIL{8,4,2}Engine::quant_gemm
    (include/oil/oil_engines.h:49,78,151)."""
    import torch
    ad, d1 = _dev(a, np.float32)
    bd, d2 = _dev(b_idx, np.uint8)
    cd, _ = _dev(codebook, np.float32)
    if cd.numel() < (1 << bits):
        raise _lib.OilHipError("engine_quant_gemm: codebook has fewer than 2^bits entries")
    out = torch.empty((M, N), dtype=torch.float32, device="cuda")
    _lib.check(_lib.lib().oilhip_engine_quant_gemm(bits, ad.data_ptr(), bd.data_ptr(), cd.data_ptr(), out.data_ptr(),
                                                   M, N, K, _lib.current_stream()))
    return _ret(out, d1 and d2)


def engine_dense_gemm(kind: int, a, b, M: int, N: int, K: int, scales=None, block_size: int = 128):
    """quant_gemm of the engines whose B operand is not a codebook index (include/oil/oil_engines.h:103,123,167):
    kind 1 Oil1Engine (b: float32, one value per 32 flat positions), 3 SparkEngine (b: uint8 2-bit codes,
    scales: float32 per block_size flat positions), 16 OIL16Engine (b: uint16 FP16 bits), 32 OIL32Engine (b: float32)."""
    import torch
    bdt = {1: np.float32, 3: np.uint8, 16: np.uint16, 32: np.float32}.get(kind)
    if bdt is None:
        raise _lib.OilHipError("engine_dense_gemm: kind must be 1, 3, 16 or 32")
    ad, d1 = _dev(a, np.float32)
    if bdt is np.uint16 and not hasattr(b, "is_cuda"):
        b = np.ascontiguousarray(b, np.uint16).view(np.int16)
        bd, d2 = torch.from_numpy(b).cuda(), True
    else:
        bd, d2 = _dev(b, bdt)
    sd = None
    if kind == 3:
        if scales is None:
            raise _lib.OilHipError("engine_dense_gemm: the SPARK engine needs scales")
        sd, _ = _dev(scales, np.float32)
    out = torch.empty((M, N), dtype=torch.float32, device="cuda")
    _lib.check(_lib.lib().oilhip_engine_dense_gemm(kind, ad.data_ptr(), bd.data_ptr(), sd.data_ptr() if sd is not None else None,
                                                   int(block_size), out.data_ptr(), M, N, K, _lib.current_stream()))
    return _ret(out, d1 and d2)


def engine_dequant(bits: int, indices, codebook, n: int, scales=None, block_size: int = 0):
    """OIL{8,4,2}Engine::dequant_tensor (packed codes; scales None) or OIL8/OIL4Engine::dequantize_per_block
    (one index byte per weight; OIL8: one scale per block, OIL4: {center, half_range} per block)."""
    import torch
    i, d1 = _dev(indices, np.uint8)
    c, _ = _dev(codebook, np.float32)
    sd = None
    if scales is not None:
        sd, _ = _dev(scales, np.float32)
    out = torch.empty(n, dtype=torch.float32, device="cuda")
    _lib.check(_lib.lib().oilhip_engine_dequant(bits, i.data_ptr(), c.data_ptr(), n, sd.data_ptr() if sd is not None else None,
                                                int(block_size), out.data_ptr(), _lib.current_stream()))
    return _ret(out, d1)


def _tl(kind, weights, activations, M, N, K):
    import torch
    w, d1 = _dev(weights, np.uint8)
    a, d2 = _dev(activations, np.float32)
    out = torch.empty((M, N), dtype=torch.float32, device="cuda")
    _lib.check(_lib.lib().oilhip_tl_gemm(kind, w.data_ptr(), a.data_ptr(), out.data_ptr(), M, N, K, _lib.current_stream()))
    return _ret(out, d1 and d2)


def tl1_gemm(weights, activations, M: int, N: int, K: int):
    """SPARK lookup kernel, pairs (kernel.h:11-12, src/kernel_tl.cpp:32-90): one packed row of K ternary codes per
    (m, n), activations [N][K] quantized per row to int8; every pair sum is clamped to int8 before it is added."""
    return _tl(1, weights, activations, M, N, K)


def tl2_gemm(weights, activations, M: int, N: int, K: int):
    """SPARK lookup kernel, triples (kernel.h:17-18, src/kernel_tl.cpp:124-184); K must be a multiple of 3."""
    return _tl(2, weights, activations, M, N, K)


class KernelPerf:
    """include/oil/kernel_production.h:68-73.  `cycles` counts shader clocks at the device's current frequency
    (the reference counts CPU timestamp ticks); the byte formulas are the reference's own
    (src/kernel_production.cpp:433-485)."""

    def __init__(self, cycles=0, bytes_read=0, bytes_written=0, gflops=0.0):
        self.cycles, self.bytes_read, self.bytes_written, self.gflops = cycles, bytes_read, bytes_written, gflops

    def __repr__(self):
        return (f"KernelPerf(cycles={self.cycles}, bytes_read={self.bytes_read}, "
                f"bytes_written={self.bytes_written}, gflops={self.gflops:.3f})")


class _Perf(C.Structure):            # oilhip_kernel_perf_t
    _fields_ = [("cycles", C.c_uint64), ("bytes_read", C.c_uint64), ("bytes_written", C.c_uint64), ("gflops", C.c_double)]


def _profile(kind, w, cb, cb_dtype, scale, x, M, K, repeats):
    import torch
    wd, _ = _dev(w, np.uint8)
    xd, _ = _dev(x, np.float32)
    cd = _dev(cb, cb_dtype)[0] if cb is not None else None
    y = torch.empty(M, dtype=torch.float32, device="cuda")
    p = _Perf()
    _lib.check(_lib.lib().oilhip_profile_gemv(kind, wd.data_ptr(), cd.data_ptr() if cd is not None else None, float(scale),
                                              xd.data_ptr(), y.data_ptr(), M, K, int(repeats), C.addressof(p),
                                              _lib.current_stream()))
    return KernelPerf(p.cycles, p.bytes_read, p.bytes_written, p.gflops), y


def profile_gemv_spark(packed_w, scale, x, M: int, K: int, repeats: int = 100):
    """kernel_production.h:75-76: `repeats` launches of gemv_spark_tiled between two events."""
    return _profile(0, packed_w, None, None, scale, x, M, K, repeats)[0]


def profile_gemv_oil4(packed_indices, codebook, scale, x, M: int, K: int, repeats: int = 100):
    """kernel_production.h:78-79."""
    return _profile(4, packed_indices, codebook, np.uint16, scale, x, M, K, repeats)[0]


def profile_gemv_oil8(indices, codebook, scale, x, M: int, K: int, repeats: int = 100):
    """kernel_production.h:81-82."""
    return _profile(8, indices, codebook, np.float32, scale, x, M, K, repeats)[0]
