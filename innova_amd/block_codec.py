"""Host mirror of the reference block codec interface (include/oil/block_codec.h).

quantize_block_all / quantize_tensor run on the host like the reference's
quantizer; dequantize_block_all runs on the GPU (one-block upload: meant for
checks and tools; tensors go through DeviceWeights.dequant)."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from .formats import Format, format_bpw


def payload_bound(fmt, n: int) -> int:
    return int(_lib.lib().oilhip_payload_bound(int(fmt), int(n)))


def quantize_block_all(fmt, w) -> tuple[np.ndarray, np.ndarray]:
    """-> (indices, codebook) byte arrays of one block (block_codec.h:55-56)."""
    w = np.ascontiguousarray(w, dtype=np.float32).reshape(-1)
    if w.size <= 0:
        raise _lib.OilHipError("quantize_block_all: empty block")
    n = w.size
    idx = np.zeros(max(16, payload_bound(fmt, n)), dtype=np.uint8)
    cb = np.zeros(max(16, 2 * ((n + 31) // 32)), dtype=np.uint8)
    il, cl = C.c_size_t(0), C.c_size_t(0)
    _lib.check(_lib.lib().oilhip_quantize_block(int(fmt), w.ctypes.data, n, idx.ctypes.data, idx.size, C.byref(il),
                                                cb.ctypes.data, cb.size, C.byref(cl)))
    return idx[: il.value].copy(), cb[: cl.value].copy()


def quantize_tensor(w, fmts, threads: int = 0) -> tuple[np.ndarray, np.ndarray]:
    """Per-256-block quantize of a flat tensor (FormatRegistry::quantize,
    src/format_registry.cpp:158-197).  fmts: one format or one per block.
    -> (payload uint8[], blocks BLOCK_DTYPE[])"""
    w = np.ascontiguousarray(w, dtype=np.float32).reshape(-1)
    nblocks = (w.size + 255) // 256
    if np.isscalar(fmts) or isinstance(fmts, Format):
        fmts = np.full(nblocks, int(fmts), dtype=np.uint8)
    fmts = np.ascontiguousarray(fmts, dtype=np.uint8)
    if fmts.size != nblocks:
        raise _lib.OilHipError("quantize_tensor: need one format per 256-weight block")
    L = _lib.lib()
    total = C.c_uint64(0)
    _lib.check(L.oilhip_quantize_tensor(fmts.ctypes.data, nblocks, w.ctypes.data, w.size, None, 0, None,
                                        C.byref(total), threads))
    payload = np.zeros(total.value, dtype=np.uint8)
    blocks = np.zeros(nblocks, dtype=_lib.BLOCK_DTYPE)
    _lib.check(L.oilhip_quantize_tensor(fmts.ctypes.data, nblocks, w.ctypes.data, w.size, payload.ctypes.data,
                                        payload.size, blocks.ctypes.data, C.byref(total), threads))
    return payload[: total.value], blocks


def dequantize_block_all(fmt, indices, codebook, nw: int) -> np.ndarray:
    """Decode one block payload on the GPU (block_codec.h:60-63)."""
    from .weights import DeviceWeights
    indices = np.ascontiguousarray(indices, dtype=np.uint8).reshape(-1)
    codebook = np.ascontiguousarray(codebook, dtype=np.uint8).reshape(-1)
    if nw == 0:
        return np.zeros(0, dtype=np.float32)
    payload = np.concatenate([codebook, indices, np.zeros(1, np.uint8)])
    blocks = np.zeros(1, dtype=_lib.BLOCK_DTYPE)
    blocks[0]["cb_off"], blocks[0]["cb_bytes"] = 0, codebook.size
    blocks[0]["idx_off"], blocks[0]["idx_bytes"] = codebook.size, indices.size
    blocks[0]["nw"], blocks[0]["fmt"] = nw, int(fmt)
    with DeviceWeights.from_blocks(payload, blocks, 1, nw) as dw:
        return dw.dequant().cpu().numpy()


def block_actual_bpw(nw: int, idx_bytes: int, cb_bytes: int) -> float:
    return 0.0 if nw == 0 else (idx_bytes + cb_bytes) * 8.0 / nw


def block_claimed_bytes(fmt, n: int) -> int:
    import math
    return int(math.ceil(np.float32(format_bpw(fmt)) * np.float32(n) / np.float32(8.0)))
