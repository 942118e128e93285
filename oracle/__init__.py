"""ctypes front end of the CPU oracle (liboiloracle.so) and, when built, of the
compiled reference (oracle/_ref/liboilref*.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
cpu_baseline leg of bench.py.  The product package never imports this module.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

FORMATS = {
    "OIL1": 0, "SPARK_Q0": 1, "OIL2": 2, "OIL4": 3, "OIL8": 4, "OIL16": 5, "OIL32": 6,
    "OIL1_GRP": 7, "SPARK_Q0_GRP": 8, "OIL2_GRP": 9, "OIL4_GRP": 10, "OIL8_GRP": 11,
    "OIL16_GRP": 12, "SPARK_SPARSE": 13, "SPARK_SPARSE_GRP": 14,
}
FORMAT_NAMES = {v: k for k, v in FORMATS.items()}

# orc_block_t
BLOCK_DTYPE = np.dtype(
    [("cb_off", "<u8"), ("idx_off", "<u8"), ("cb_bytes", "<u4"), ("idx_bytes", "<u4"),
     ("nw", "<u4"), ("fmt", "u1"), ("pad", "u1", (3,))], align=True)
assert BLOCK_DTYPE.itemsize == 32

_u8p = C.POINTER(C.c_uint8)
_f32p = C.POINTER(C.c_float)
_u16p = C.POINTER(C.c_uint16)


def _p(a, t):
    return a.ctypes.data_as(t)


def build(ref: bool = False) -> None:
    """Compile the oracle (and the compiled reference when asked and present)."""
    subprocess.run(["make", "-C", _HERE, "liboiloracle.so"], check=True, capture_output=True)
    if ref and os.path.isdir("/root/reference/src"):
        subprocess.run(["make", "-C", _HERE, "ref"], check=True, capture_output=True)


_lib = None


def lib():
    global _lib
    if _lib is None:
        path = os.path.join(_HERE, "liboiloracle.so")
        if not os.path.exists(path):
            build()
        L = C.CDLL(path)
        L.orc_f32_to_f16.restype = C.c_uint16
        L.orc_f32_to_f16.argtypes = [C.c_float]
        L.orc_f16_to_f32.restype = C.c_float
        L.orc_f16_to_f32.argtypes = [C.c_uint16]
        L.orc_flat_fp16_to_float.restype = C.c_float
        L.orc_flat_fp16_to_float.argtypes = [C.c_uint16]
        L.orc_format_bpw.restype = C.c_float
        L.orc_format_bpw.argtypes = [C.c_int]
        L.orc_max_payload_bytes.restype = C.c_size_t
        L.orc_max_payload_bytes.argtypes = [C.c_int, C.c_int]
        L.orc_quantize_block.restype = C.c_int
        L.orc_quantize_block.argtypes = [C.c_int, _f32p, C.c_int, _u8p, C.c_size_t,
                                         C.POINTER(C.c_size_t), _u8p, C.c_size_t,
                                         C.POINTER(C.c_size_t)]
        L.orc_dequantize_block.restype = None
        L.orc_dequantize_block.argtypes = [C.c_int, _u8p, C.c_size_t, _u8p, C.c_size_t,
                                           C.c_uint32, _f32p]
        L.orc_quantize_tensor.restype = C.c_uint64
        L.orc_quantize_tensor.argtypes = [_u8p, C.c_uint32, _f32p, C.c_uint64, C.c_uint32,
                                          _u8p, C.c_uint64, C.c_void_p, C.c_int]
        L.orc_dequant_blocks.restype = None
        L.orc_dequant_blocks.argtypes = [_u8p, C.c_void_p, C.c_uint32, _f32p]
        for name in ("orc_block_gemm_f32", "orc_block_gemm_f64"):
            f = getattr(L, name)
            f.restype = None
            f.argtypes = [_u8p, C.c_void_p, C.c_uint32, C.c_uint32, _f32p, _f32p, C.c_int, C.c_int]
        L.orc_oil8_gemm.restype = None
        L.orc_oil8_gemm.argtypes = [_u8p, _f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int]
        L.orc_oil4_gemm.restype = None
        L.orc_oil4_gemm.argtypes = [_u8p, _u16p, _f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int]
        L.orc_gemv_spark.restype = None
        L.orc_gemv_spark.argtypes = [_u8p, C.c_float, _f32p, _f32p, C.c_int, C.c_int, C.c_int]
        L.orc_gemv_oil4.restype = None
        L.orc_gemv_oil4.argtypes = [_u8p, _u16p, C.c_float, _f32p, _f32p, C.c_int, C.c_int, C.c_int]
        L.orc_gemv_oil8.restype = None
        L.orc_gemv_oil8.argtypes = [_u8p, _f32p, C.c_float, _f32p, _f32p, C.c_int, C.c_int, C.c_int]
        L.orc_engine_quant_gemm.restype = None
        L.orc_engine_quant_gemm.argtypes = [C.c_int, _f32p, _u8p, _f32p, _f32p,
                                            C.c_int64, C.c_int64, C.c_int64, C.c_int]
        L.orc_tl_gemm.restype = None
        L.orc_tl_gemm.argtypes = [C.c_int, _u8p, _f32p, _f32p, C.c_int, C.c_int, C.c_int]
        _lib = L
    return _lib


_ref = {}


def ref(simd: bool = True):
    """The compiled reference, or None where it has not been built."""
    key = "liboilref.so" if simd else "liboilref_scalar.so"
    if key not in _ref:
        path = os.path.join(_HERE, "_ref", key)
        if not os.path.exists(path):
            _ref[key] = None
        else:
            R = C.CDLL(path)
            R.ref_quantize_block.restype = C.c_int
            R.ref_quantize_block.argtypes = lib().orc_quantize_block.argtypes
            R.ref_dequantize_block.restype = None
            R.ref_dequantize_block.argtypes = lib().orc_dequantize_block.argtypes
            R.ref_format_bpw.restype = C.c_float
            R.ref_format_bpw.argtypes = [C.c_int]
            R.ref_oil8_gemm.restype = None
            R.ref_oil8_gemm.argtypes = [_u8p, _f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int]
            R.ref_oil4_gemm.restype = None
            R.ref_oil4_gemm.argtypes = [_u8p, _u16p, _f32p, _f32p, C.c_int, C.c_int, C.c_int]
            R.ref_gemv_spark.restype = None
            R.ref_gemv_spark.argtypes = [_u8p, C.c_float, _f32p, _f32p, C.c_int, C.c_int]
            R.ref_gemv_oil4.restype = None
            R.ref_gemv_oil4.argtypes = [_u8p, _u16p, C.c_float, _f32p, _f32p, C.c_int, C.c_int]
            R.ref_gemv_oil8.restype = None
            R.ref_gemv_oil8.argtypes = [_u8p, _f32p, C.c_float, _f32p, _f32p, C.c_int, C.c_int]
            R.ref_engine_codebook.restype = C.c_int
            R.ref_engine_codebook.argtypes = [C.c_int, _f32p]
            R.ref_engine_quant_gemm.restype = None
            R.ref_engine_quant_gemm.argtypes = [C.c_int, _f32p, _u8p, _f32p,
                                                C.c_int64, C.c_int64, C.c_int64]
            R.ref_tl_gemm.restype = None
            R.ref_tl_gemm.argtypes = [C.c_int, _u8p, C.c_size_t, _f32p, _f32p, C.c_int, C.c_int, C.c_int]
            _ref[key] = R
    return _ref[key]


# --------------------------------------------------------------------------- codec
def _quantize_block(fn, fmt: int, w: np.ndarray):
    w = np.ascontiguousarray(w, dtype=np.float32)
    n = w.size
    idx = np.zeros(max(16, 4 * n + 64), dtype=np.uint8)
    cb = np.zeros(max(16, 2 * ((n + 31) // 32) + 16), dtype=np.uint8)
    il, cl = C.c_size_t(0), C.c_size_t(0)
    ok = fn(fmt, _p(w, _f32p), n, _p(idx, _u8p), idx.size, C.byref(il),
            _p(cb, _u8p), cb.size, C.byref(cl))
    if ok != 1:
        raise RuntimeError(f"quantize_block failed for fmt={fmt} n={n} (rc={ok})")
    return idx[: il.value].copy(), cb[: cl.value].copy()


def quantize_block(fmt: int, w: np.ndarray):
    """-> (index bytes, codebook bytes) of one block."""
    return _quantize_block(lib().orc_quantize_block, fmt, w)


def ref_quantize_block(fmt: int, w: np.ndarray, simd: bool = True):
    return _quantize_block(ref(simd).ref_quantize_block, fmt, w)


def _dequantize_block(fn, fmt, idx, cb, nw, prefill=None):
    idx = np.ascontiguousarray(idx, dtype=np.uint8)
    cb = np.ascontiguousarray(cb, dtype=np.uint8)
    out = np.full(nw, np.nan if prefill is None else prefill, dtype=np.float32)
    # numpy gives a valid pointer even for empty arrays
    fn(fmt, _p(idx, _u8p), idx.size, _p(cb, _u8p), cb.size, nw, _p(out, _f32p))
    return out


def dequantize_block(fmt: int, idx, cb, nw: int) -> np.ndarray:
    return _dequantize_block(lib().orc_dequantize_block, fmt, idx, cb, nw)


def ref_dequantize_block(fmt: int, idx, cb, nw: int, simd: bool = True) -> np.ndarray:
    return _dequantize_block(ref(simd).ref_dequantize_block, fmt, idx, cb, nw)


def max_payload_bytes(fmt: int, n: int) -> int:
    return int(lib().orc_max_payload_bytes(fmt, n))


def quantize_tensor(w: np.ndarray, fmts, align: int = 16, threads: int = 0):
    """Quantize a flat weight array block by block.

    fmts: one format id, or an array of one id per 256-block.
    -> (payload uint8[total], blocks BLOCK_DTYPE[nblocks])
    """
    w = np.ascontiguousarray(w, dtype=np.float32).reshape(-1)
    nblocks = (w.size + 255) // 256
    if np.isscalar(fmts):
        fmts = np.full(nblocks, int(fmts), dtype=np.uint8)
    fmts = np.ascontiguousarray(fmts, dtype=np.uint8)
    assert fmts.size == nblocks
    L = lib()
    cap = L.orc_quantize_tensor(_p(fmts, _u8p), nblocks, _p(w, _f32p), w.size, align,
                                None, 0, None, threads)
    if cap == 0:
        raise RuntimeError("orc_quantize_tensor: bad arguments")
    payload = np.zeros(cap, dtype=np.uint8)
    blocks = np.zeros(nblocks, dtype=BLOCK_DTYPE)
    total = L.orc_quantize_tensor(_p(fmts, _u8p), nblocks, _p(w, _f32p), w.size, align,
                                  _p(payload, _u8p), cap, blocks.ctypes.data, threads)
    if total == 0:
        raise RuntimeError("orc_quantize_tensor failed")
    return payload[:total].copy(), blocks


def dequant_blocks(payload: np.ndarray, blocks: np.ndarray) -> np.ndarray:
    payload = np.ascontiguousarray(payload, dtype=np.uint8)
    blocks = np.ascontiguousarray(blocks)
    out = np.full(int(blocks["nw"].astype(np.int64).sum()), np.nan, dtype=np.float32)
    lib().orc_dequant_blocks(_p(payload, _u8p), blocks.ctypes.data, blocks.size, _p(out, _f32p))
    return out


def block_gemm(payload, blocks, rows: int, cols: int, X: np.ndarray, wide: bool = True,
               threads: int = 0) -> np.ndarray:
    """Y[B][rows] = X[B][cols] . W^T from block payloads.  wide=True: double
    accumulation (the tolerance yardstick); wide=False: the reference's FP32 order."""
    payload = np.ascontiguousarray(payload, dtype=np.uint8)
    blocks = np.ascontiguousarray(blocks)
    X = np.ascontiguousarray(X, dtype=np.float32).reshape(-1, cols)
    B = X.shape[0]
    assert cols % 256 == 0 and blocks.size == rows * (cols // 256)
    Y = np.zeros((B, rows), dtype=np.float32)
    fn = lib().orc_block_gemm_f64 if wide else lib().orc_block_gemm_f32
    fn(_p(payload, _u8p), blocks.ctypes.data, rows, cols, _p(X, _f32p), _p(Y, _f32p), B, threads)
    return Y


# ------------------------------------------------------------------- flat kernels
def oil8_gemm(idx, cb, act, M, N, K, order=0):
    idx = np.ascontiguousarray(idx, dtype=np.uint8)
    cb = np.ascontiguousarray(cb, dtype=np.float32)
    act = np.ascontiguousarray(act, dtype=np.float32)
    out = np.zeros(M * N, dtype=np.float32)
    lib().orc_oil8_gemm(_p(idx, _u8p), _p(cb, _f32p), _p(act, _f32p), _p(out, _f32p), M, N, K, order)
    return out.reshape(M, N)


def oil4_gemm(packed, cb16, act, M, N, K, order=0):
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    cb16 = np.ascontiguousarray(cb16, dtype=np.uint16)
    act = np.ascontiguousarray(act, dtype=np.float32)
    out = np.zeros(M * N, dtype=np.float32)
    lib().orc_oil4_gemm(_p(packed, _u8p), _p(cb16, _u16p), _p(act, _f32p), _p(out, _f32p), M, N, K, order)
    return out.reshape(M, N)


def gemv_spark(w, scale, x, M, K, mode=0):
    w = np.ascontiguousarray(w, dtype=np.uint8)
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.zeros(M, dtype=np.float32)
    lib().orc_gemv_spark(_p(w, _u8p), scale, _p(x, _f32p), _p(y, _f32p), M, K, int(mode))
    return y


def gemv_oil4(w, cb16, scale, x, M, K, mode=0):
    w = np.ascontiguousarray(w, dtype=np.uint8)
    cb16 = np.ascontiguousarray(cb16, dtype=np.uint16)
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.zeros(M, dtype=np.float32)
    lib().orc_gemv_oil4(_p(w, _u8p), _p(cb16, _u16p), scale, _p(x, _f32p), _p(y, _f32p), M, K, int(mode))
    return y


def gemv_oil8(w, cb, scale, x, M, K, mode=0):
    w = np.ascontiguousarray(w, dtype=np.uint8)
    cb = np.ascontiguousarray(cb, dtype=np.float32)
    x = np.ascontiguousarray(x, dtype=np.float32)
    y = np.zeros(M, dtype=np.float32)
    lib().orc_gemv_oil8(_p(w, _u8p), _p(cb, _f32p), scale, _p(x, _f32p), _p(y, _f32p), M, K, int(mode))
    return y


def engine_quant_gemm(bits, A, b_idx, cb, M, N, K, as_double=False):
    A = np.ascontiguousarray(A, dtype=np.float32)
    b_idx = np.ascontiguousarray(b_idx, dtype=np.uint8)
    cb = np.ascontiguousarray(cb, dtype=np.float32)
    out = np.zeros(M * N, dtype=np.float32)
    lib().orc_engine_quant_gemm(bits, _p(A, _f32p), _p(b_idx, _u8p), _p(cb, _f32p), _p(out, _f32p),
                                M, N, K, int(as_double))
    return out.reshape(M, N)


def tl_row_bytes(kind: int, K: int) -> int:
    return (K + 3) // 4 if kind == 1 else ((K + 11) // 12) * 3


def tl_gemm(kind, w, a, M, N, K, fn=None):
    """tl1_gemm (kind 1) / tl2_gemm (kind 2); fn = ref().ref_tl_gemm runs the compiled reference instead."""
    w = np.ascontiguousarray(w, dtype=np.uint8)
    a = np.ascontiguousarray(a, dtype=np.float32)
    assert w.size >= M * N * tl_row_bytes(kind, K) and a.size == N * K
    out = np.zeros(M * N, dtype=np.float32)
    if fn is None:
        lib().orc_tl_gemm(kind, _p(w, _u8p), _p(a, _f32p), _p(out, _f32p), M, N, K)
    else:
        fn(kind, _p(w, _u8p), w.size, _p(a, _f32p), _p(out, _f32p), M, N, K)
    return out.reshape(M, N)


# --------------------------------------------------------------- test generators
def xorshift_fill(n: int, seed: int) -> np.ndarray:
    """The reference codec test's deterministic generator
    (tests/test_block_codec.cpp:49-55): uniform in [-1, 1]."""
    state = (seed * 2654435761 + 12345) & 0xFFFFFFFF
    out = np.empty(n, dtype=np.float32)
    f = np.float32
    for i in range(n):
        state ^= (state << 13) & 0xFFFFFFFF
        state ^= state >> 17
        state ^= (state << 5) & 0xFFFFFFFF
        out[i] = (f(state & 0xFFFF) / f(65535.0) - f(0.5)) * f(2.0)
    return out


# ---------------------------------------------------------------- mixture of experts
def softmax_topk(logits: np.ndarray, k: int, fn=None):
    """orc_softmax_topk -> (probs, indices, weights)."""
    lg = np.ascontiguousarray(logits, np.float32)
    T, E = lg.shape
    probs = np.zeros((T, E), np.float32)
    idx = np.zeros((T, k), np.int64)
    w = np.zeros((T, k), np.float32)
    (fn or lib().orc_softmax_topk)(C.c_void_p(lg.ctypes.data), C.c_int64(T), C.c_int64(E), C.c_int64(k),
                                   C.c_void_p(probs.ctypes.data), C.c_void_p(idx.ctypes.data), C.c_void_p(w.ctypes.data))
    return probs, idx, w


def moe_dispatch(x, gate, up, down, indices, weights, wide: bool = False, fn=None):
    """orc_moe_dispatch over decoded expert matrices (lists of [F][D], [F][D], [D][F] float32 arrays).
    -> (out [T][D], z_loss, dropped).  fn: a compiled-reference entry point with the same leading arguments."""
    x = np.ascontiguousarray(x, np.float32)
    T, D = x.shape
    E, F = len(gate), gate[0].shape[0]
    idx = np.ascontiguousarray(indices, np.int64)
    w = np.ascontiguousarray(weights, np.float32)
    K = idx.shape[1]
    keep = [[np.ascontiguousarray(m, np.float32) for m in lst] for lst in (gate, up, down)]
    ptrs = [(C.c_void_p * E)(*[m.ctypes.data for m in lst]) for lst in keep]
    out = np.zeros((T, D), np.float32)
    z, dr = C.c_float(0), C.c_int64(0)
    args = [C.c_void_p(x.ctypes.data), ptrs[0], ptrs[1], ptrs[2], C.c_void_p(idx.ctypes.data), C.c_void_p(w.ctypes.data),
            C.c_int64(T), C.c_int64(K), C.c_int64(E), C.c_int64(D), C.c_int64(F), C.c_void_p(out.ctypes.data),
            C.byref(z), C.byref(dr)]
    if fn is None:
        lib().orc_moe_dispatch(*args, C.c_int(1 if wide else 0))
    else:
        fn(*args)
    return out, z.value, dr.value


def ref_moe():
    """The compiled reference's routing/dispatch library, or None where it has not been built."""
    path = os.path.join(_HERE, "_ref", "liboilref_moe.so")
    return C.CDLL(path) if os.path.exists(path) else None


def engine_dense_gemm(kind: int, A, B, M: int, N: int, K: int, scales=None, block: int = 128, fn=None):
    """orc_engine_dense_gemm, or with fn = the compiled reference's ref_engine_dense_gemm."""
    A = np.ascontiguousarray(A, np.float32)
    B = np.ascontiguousarray(B)
    sc = np.ascontiguousarray(scales, np.float32) if scales is not None else np.zeros(1, np.float32)
    out = np.zeros((M, N), np.float32)
    if fn is None:
        lib().orc_engine_dense_gemm(C.c_int(kind), C.c_void_p(A.ctypes.data), C.c_void_p(B.ctypes.data), C.c_void_p(sc.ctypes.data),
                                    C.c_int64(block), C.c_void_p(out.ctypes.data), C.c_int64(M), C.c_int64(N), C.c_int64(K))
    else:
        fn(C.c_int(kind), C.c_void_p(A.ctypes.data), C.c_void_p(B.ctypes.data), C.c_size_t(B.nbytes), C.c_void_p(sc.ctypes.data),
           C.c_int64(sc.size), C.c_int64(block), C.c_void_p(out.ctypes.data), C.c_int64(M), C.c_int64(N), C.c_int64(K))
    return out


# ---------------------------------------------------------------- decode-step pieces
def rmsnorm(x, w) -> np.ndarray:
    x = np.ascontiguousarray(x, np.float32)
    w = np.ascontiguousarray(w, np.float32)
    out = np.zeros_like(x)
    for r in range(x.reshape(-1, w.size).shape[0]):
        xr = np.ascontiguousarray(x.reshape(-1, w.size)[r])
        o = np.zeros(w.size, np.float32)
        lib().orc_rmsnorm(C.c_void_p(xr.ctypes.data), C.c_void_p(w.ctypes.data), C.c_int(w.size), C.c_void_p(o.ctypes.data))
        out.reshape(-1, w.size)[r] = o
    return out


def swiglu(g, u) -> np.ndarray:
    g = np.ascontiguousarray(g, np.float32)
    u = np.ascontiguousarray(u, np.float32)
    h = np.zeros_like(g)
    lib().orc_swiglu(C.c_void_p(g.ctypes.data), C.c_void_p(u.ctypes.data), C.c_int64(g.size), C.c_void_p(h.ctypes.data))
    return h


# ---------------------------------------------------------------- OIL4 KV cache (src/kv_cache_oil4.cpp)
def _vp(a):
    return C.c_void_p(a.ctypes.data)


def kv_half_to_float(h: np.ndarray) -> np.ndarray:
    """CodebookOIL4::half_to_float over an array of uint16 (src/codebook.cpp:36-64).  Runs through orc_kv_get_range so
    that the floats come back through memory (a ctypes float return would quiet signalling NaNs)."""
    hh = np.asarray(h, np.uint16).ravel()
    nb = (hh.size + 15) // 16
    cb = np.zeros(nb * 16, np.uint16)
    cb[:hh.size] = hh
    idx = np.tile(np.array([0x10, 0x32, 0x54, 0x76, 0x98, 0xBA, 0xDC, 0xFE] * 2, np.uint8), nb)   # codes 0..15 twice per block of 32
    out = np.zeros((nb, 32), np.float32)
    if nb:
        lib().orc_kv_get_range(_vp(idx), _vp(cb), C.c_int64(idx.size), C.c_int64(32), C.c_int64(32), C.c_int64(0),
                               C.c_int64(nb), _vp(out))
    return out[:, :16].ravel()[:hh.size].reshape(np.shape(h)).copy()


def kv_float_to_half(f: np.ndarray) -> np.ndarray:
    """CodebookOIL4::float_to_half over an array of float32 (src/codebook.cpp:16-34)."""
    L = lib()
    L.orc_kv_float_to_half.restype = C.c_uint16
    L.orc_kv_float_to_half.argtypes = [C.c_float]
    return np.array([L.orc_kv_float_to_half(float(x)) for x in np.asarray(f, np.float32).ravel()],
                    np.uint16).reshape(np.shape(f))


def kv_quantize_block(src: np.ndarray, fn=None):
    """OIL4KVCache::quantize_block_oil4 (src/kv_cache_oil4.cpp:75-163): (codebook uint16[16], codes uint8[n])."""
    src = np.ascontiguousarray(src, np.float32)
    cb = np.zeros(16, np.uint16)
    codes = np.zeros(max(src.size, 1), np.uint8)
    (fn or lib().orc_kv_quantize_block)(_vp(src), C.c_int64(src.size), _vp(cb), _vp(codes))
    return cb, codes[:src.size]


class KVCache:
    """OIL4KVCache (include/oil/kv_cache_oil4.h:26-83) for one layer, state in numpy arrays."""

    def __init__(self, max_seq_len, num_heads, head_dim, block_size=64):
        self.max_seq, self.per_token = int(max_seq_len), int(num_heads * head_dim)
        self.block = block_size if block_size in (32, 64, 128) else 64
        total = self.max_seq * self.per_token
        self.idx_bytes = (total + 1) // 2
        nblocks = (total + self.block - 1) // self.block
        self.k_idx = np.zeros(self.idx_bytes, np.uint8)
        self.v_idx = np.zeros(self.idx_bytes, np.uint8)
        self.k_cb = np.zeros(nblocks * 16, np.uint16)
        self.v_cb = np.zeros(nblocks * 16, np.uint16)
        self.pos = 0

    def append(self, k, v):
        k = np.ascontiguousarray(k, np.float32).reshape(-1, self.per_token)
        v = np.ascontiguousarray(v, np.float32).reshape(-1, self.per_token)
        lib().orc_kv_append(_vp(self.k_idx), _vp(self.v_idx), _vp(self.k_cb), _vp(self.v_cb), C.c_int64(self.idx_bytes),
                            C.c_int64(self.max_seq), C.c_int64(self.per_token), C.c_int64(self.block),
                            C.c_int64(self.pos), _vp(k), _vp(v), C.c_int64(k.shape[0]))
        self.pos += k.shape[0]

    def get_range(self, start, end):
        n = min(end, self.pos) - start
        if end - start <= 0 or n <= 0:
            return np.zeros((0, self.per_token), np.float32), np.zeros((0, self.per_token), np.float32)
        out = []
        for idx, cb in ((self.k_idx, self.k_cb), (self.v_idx, self.v_cb)):
            o = np.zeros((n, self.per_token), np.float32)
            lib().orc_kv_get_range(_vp(idx), _vp(cb), C.c_int64(self.idx_bytes), C.c_int64(self.per_token),
                                   C.c_int64(self.block), C.c_int64(start), C.c_int64(n), _vp(o))
            out.append(o)
        return out[0], out[1]


def ref_kv_run(max_seq, heads, dim, block, k, v, seq_lens, start, end):
    """The compiled reference's OIL4KVCache: the appends, then get_range -> (k, v, size_bytes, context_len)."""
    R = ref(True)
    k = np.ascontiguousarray(k, np.float32)
    v = np.ascontiguousarray(v, np.float32)
    pt = heads * dim
    tot = int(sum(seq_lens))
    ko = np.zeros((max(tot, 1), pt), np.float32)
    vo = np.zeros_like(ko)
    sl = np.array(seq_lens, np.int64)
    sb, cl = C.c_uint64(), C.c_int()
    R.ref_kv_run.restype = C.c_int64
    n = R.ref_kv_run(C.c_int(1), C.c_int64(max_seq), C.c_int64(heads), C.c_int64(dim), C.c_int64(block), C.c_int(0),
                     _vp(k), _vp(v), _vp(sl), C.c_int(len(seq_lens)), C.c_int64(start), C.c_int64(end), _vp(ko), _vp(vo),
                     C.byref(sb), C.byref(cl))
    return ko[:n].copy(), vo[:n].copy(), sb.value, cl.value
