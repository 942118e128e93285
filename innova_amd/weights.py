"""A quantized tensor resident in HBM (the oilhip_weights handle)."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib


class DeviceWeights:
    """rows x cols weights as .oil blocks in HBM, uploaded once.

    Stands in for the reference's (OILReader, Th{start,count,fmt,rows,cols}) pair
    (include/oil/qwen35_engine.h:29): gemv()/gemm_bf16() are Qwen35Engine::gemm
    (src/adapters/tools/qwen35_engine.cpp:47-85) for decode and prefill."""

    def __init__(self, handle: int, rows: int, cols: int):
        self._h = handle
        self.rows, self.cols = rows, cols

    # ---- construction -------------------------------------------------------
    @classmethod
    def from_blocks(cls, payload, blocks, rows: int, cols: int) -> "DeviceWeights":
        payload = np.ascontiguousarray(payload, dtype=np.uint8)
        blocks = np.ascontiguousarray(blocks, dtype=_lib.BLOCK_DTYPE)
        h = C.c_void_p(0)
        _lib.check(_lib.lib().oilhip_weights_create(payload.ctypes.data, payload.size, blocks.ctypes.data,
                                                    blocks.size, rows, cols, C.byref(h)))
        return cls(h.value, rows, cols)

    @classmethod
    def from_records(cls, records, fmts, rows: int, cols: int) -> "DeviceWeights":
        """records: the .oil file's block records [nw][cb_bytes][cb][idx_bytes][idx] end to end."""
        records = np.ascontiguousarray(records, dtype=np.uint8)
        fmts = np.ascontiguousarray(fmts, dtype=np.uint8)
        h = C.c_void_p(0)
        _lib.check(_lib.lib().oilhip_weights_create_from_records(records.ctypes.data, records.size, fmts.ctypes.data,
                                                                 fmts.size, rows, cols, C.byref(h)))
        return cls(h.value, rows, cols)

    @classmethod
    def quantize(cls, w, fmts, rows: int, cols: int) -> "DeviceWeights":
        from .block_codec import quantize_tensor
        payload, blocks = quantize_tensor(w, fmts)
        return cls.from_blocks(payload, blocks, rows, cols)

    @classmethod
    def stack_rows(cls, parts) -> "DeviceWeights":
        """Tensors of one format, width and regular block layout as one tensor of their rows (device copy);
        gate + up or q + k + v then run as a single launch."""
        arr = (C.c_void_p * len(parts))(*[p.handle for p in parts])
        h = C.c_void_p(0)
        _lib.check(_lib.lib().oilhip_weights_stack_rows(arr, len(parts), C.byref(h)))
        return cls(h.value, sum(p.rows for p in parts), parts[0].cols)

    # ---- lifetime -------------------------------------------------------------
    def close(self) -> None:
        if self._h:
            _lib.lib().oilhip_weights_destroy(self._h)
            self._h = 0

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def handle(self) -> int:
        if not self._h:
            raise _lib.OilHipError("DeviceWeights used after close()")
        return self._h

    def info(self) -> dict:
        rows, cols, pb = C.c_uint64(0), C.c_uint64(0), C.c_uint64(0)
        nb, uf = C.c_uint32(0), C.c_int(0)
        _lib.check(_lib.lib().oilhip_weights_info(self.handle, C.byref(rows), C.byref(cols), C.byref(nb),
                                                  C.byref(pb), C.byref(uf)))
        stored, desc = C.c_uint64(0), C.c_uint64(0)
        _lib.check(_lib.lib().oilhip_weights_device_bytes(self.handle, C.byref(stored), C.byref(desc)))
        return {"rows": rows.value, "cols": cols.value, "nblocks": nb.value, "payload_bytes": pb.value,
                "uniform_fmt": uf.value, "stored_bytes": stored.value, "descriptor_bytes": desc.value}

    # ---- compute ----------------------------------------------------------------
    def dequant(self, out=None):
        """All blocks decoded back to back -> float32 cuda tensor [rows*cols]."""
        import torch
        if out is None:
            out = torch.empty(self.rows * self.cols, dtype=torch.float32, device="cuda")
        assert out.is_cuda and out.dtype == torch.float32 and out.is_contiguous() and out.numel() >= self.rows * self.cols
        _lib.check(_lib.lib().oilhip_dequant_f32(self.handle, out.data_ptr(), _lib.current_stream()))
        return out

    def _xy(self, x, dtype, out):
        import torch
        assert x.is_cuda and x.dtype == dtype and x.is_contiguous()
        x2 = x.reshape(-1, self.cols)
        M = x2.shape[0]
        if out is None:
            out = torch.empty((M, self.rows), dtype=torch.float32, device=x.device)
        assert out.is_cuda and out.dtype == torch.float32 and out.is_contiguous() and out.numel() == M * self.rows
        return x2, M, out

    def gemv(self, x, out=None, general: bool = False, noalloc: bool = False):
        """Y[M][rows] = X[M][cols] . W^T, FP32 (decode path).  general=True forces the
        all-format kernel (used by tests to cross-check the specialised kernels); noalloc=True takes the entry
        point that allocates no device memory (uniform OIL4 only, scratch in a fixed device array)."""
        import torch
        x2, M, out = self._xy(x, torch.float32, out)
        L = _lib.lib()
        fn = L.oilhip_gemv_f32_general if general else L.oilhip_gemv_oil4_f32_noalloc if noalloc else L.oilhip_gemv_f32
        _lib.check(fn(self.handle, x2.data_ptr(), out.data_ptr(), M, _lib.current_stream()))
        return out

    def gemm_bf16(self, x, out=None):
        """Y[M][rows] = X[M][cols] . W^T with bf16 operands on MFMA, FP32 accumulate (prefill path)."""
        import torch
        x2, M, out = self._xy(x, torch.bfloat16, out)
        _lib.check(_lib.lib().oilhip_gemm_bf16(self.handle, x2.data_ptr(), out.data_ptr(), M, _lib.current_stream()))
        return out

    def gemm_f32(self, x, out=None):
        """The prefill GEMM for FP32 activations (the reference's own gemm() arguments, qwen35_engine.cpp:47-85):
        X is rounded once to bf16 inside the kernel's pre-pass; bf16 tolerance (rel-L2 <= 2e-3)."""
        import torch
        x2, M, out = self._xy(x, torch.float32, out)
        _lib.check(_lib.lib().oilhip_gemm_f32(self.handle, x2.data_ptr(), out.data_ptr(), M, _lib.current_stream()))
        return out
