"""Host mirror of oil::OIL4KVCache (include/oil/kv_cache_oil4.h:26-83, src/kv_cache_oil4.cpp): the cache lives in HBM,
append quantizes on the device with the reference's Lloyd-Max, get_range decodes to FP32 cuda tensors."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib


class OIL4KVCache:
    """Same methods and meaning as the reference class.  k / v of append: float32 cuda tensors shaped [1, heads, seq, dim]
    like the reference's, whose memory the reference reads as [seq][heads * dim] (:213, :223-229); get_range returns
    tensors of the reference's shape [1, heads, len, dim] over memory in that same [len][heads * dim] order."""

    OIL4_CODEBOOK_SIZE = 16

    def __init__(self, num_layers, max_seq_len, num_heads, head_dim, block_size=64):
        self._h = C.c_void_p()
        _lib.check(_lib.lib().oilhip_kv_create(num_layers, max_seq_len, num_heads, head_dim, block_size, C.byref(self._h)))
        self._layers, self._max_seq, self._heads, self._dim = num_layers, max_seq_len, num_heads, head_dim

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            try:
                _lib.lib().oilhip_kv_destroy(h)
            except Exception:
                pass

    # ---- the reference's accessors
    def max_seq_len(self): return self._max_seq
    def num_layers(self): return self._layers
    def num_heads(self): return self._heads
    def head_dim(self): return self._dim

    def _info(self):
        ctx, blk, sb, fb = C.c_int(), C.c_int64(), C.c_uint64(), C.c_uint64()
        _lib.check(_lib.lib().oilhip_kv_info(self._h, C.byref(ctx), C.byref(blk), C.byref(sb), C.byref(fb)))
        return ctx.value, blk.value, sb.value, fb.value

    def context_len(self): return self._info()[0]
    def block_size(self): return self._info()[1]
    def size_bytes(self): return self._info()[2]
    def size_bytes_fp32_equivalent(self): return self._info()[3]

    def compression_ratio(self):
        _, _, sb, fb = self._info()
        return 0.0 if sb == 0 else fb / sb

    # ---- core operations
    def append(self, layer, k, v):
        import torch
        for t in (k, v):
            assert t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() and t.dim() == 4
        seq = k.shape[2]
        assert k.numel() == v.numel() == seq * self._heads * self._dim
        _lib.check(_lib.lib().oilhip_kv_append(self._h, layer, k.data_ptr(), v.data_ptr(), seq, _lib.current_stream()))

    def get_range(self, layer, start, end):
        import torch
        n = max(0, min(end, self._max_seq) - start)
        k = torch.empty((1, self._heads, n, self._dim), dtype=torch.float32, device="cuda")
        v = torch.empty_like(k)
        got = C.c_int64()
        _lib.check(_lib.lib().oilhip_kv_get_range(self._h, layer, start, end, k.data_ptr(), v.data_ptr(), C.byref(got),
                                                  _lib.current_stream()))
        if got.value != n:                      # end past the tokens held: the reference returns the shorter tensors
            k = k.reshape(-1)[: got.value * self._heads * self._dim].reshape(1, self._heads, got.value, self._dim)
            v = v.reshape(-1)[: got.value * self._heads * self._dim].reshape(1, self._heads, got.value, self._dim)
        return k, v

    def get_all(self, layer):
        return self.get_range(layer, 0, self._max_seq)      # end is clipped to the tokens the layer holds (:365)

    def clear(self):
        _lib.check(_lib.lib().oilhip_kv_clear(self._h, _lib.current_stream()))

    def resize(self, new_max_seq_len):
        _lib.check(_lib.lib().oilhip_kv_resize(self._h, new_max_seq_len))
        self._max_seq = new_max_seq_len

    def state(self, layer):
        """Host copies (k_idx, v_idx, k_cb, v_cb) of a layer's arrays."""
        total = self._max_seq * self._heads * self._dim
        blk = self.block_size()
        ki, vi = np.zeros((total + 1) // 2, np.uint8), np.zeros((total + 1) // 2, np.uint8)
        kc, vc = np.zeros((total + blk - 1) // blk * 16, np.uint16), np.zeros((total + blk - 1) // blk * 16, np.uint16)
        _lib.check(_lib.lib().oilhip_kv_state(self._h, layer, ki.ctypes.data, vi.ctypes.data, kc.ctypes.data, vc.ctypes.data))
        return ki, vi, kc, vc

    # ---- the reference's static pair
    @staticmethod
    def quantize_block_oil4(src):
        """src: float32 cuda tensor [nblocks][n] (n <= 128) -> (codes uint8 [nblocks][n], codebooks int16-viewed uint16 [nblocks][16])."""
        import torch
        assert src.is_cuda and src.dtype == torch.float32 and src.is_contiguous() and src.dim() == 2
        nb, n = src.shape
        codes = torch.empty((nb, n), dtype=torch.uint8, device=src.device)
        cb = torch.empty((nb, 16), dtype=torch.int16, device=src.device)
        _lib.check(_lib.lib().oilhip_kv_quantize_blocks(src.data_ptr(), n, nb, codes.data_ptr(), cb.data_ptr(), _lib.current_stream()))
        return codes, cb

    @staticmethod
    def dequantize_block_oil4(codes, cb):
        import torch
        assert codes.is_cuda and codes.dtype == torch.uint8 and codes.is_contiguous() and cb.is_cuda and cb.dtype == torch.int16
        nb, n = codes.shape
        out = torch.empty((nb, n), dtype=torch.float32, device=codes.device)
        _lib.check(_lib.lib().oilhip_kv_dequantize_blocks(codes.data_ptr(), cb.data_ptr(), out.data_ptr(), n, nb, _lib.current_stream()))
        return out
