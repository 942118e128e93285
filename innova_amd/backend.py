"""Host mirror of the reference's backend dispatch for the gfx950 device (include/oil/backend.h:9-139):
BackendType / backend_name, probe_hardware, select_optimal_backend and a ComputeBackend-shaped object whose dense FP32
operations run as HIP kernels (oilhip_dense_*).  Operands are numpy arrays (uploaded per call, as every backend of
the reference works on host tensors) or contiguous cuda tensors (used in place); there is no CPU fallback."""
from __future__ import annotations

import enum
import os

import numpy as np

from . import _lib


class BackendType(enum.IntEnum):
    """include/oil/backend.h:9-20, plus the value the gfx950 patch appends."""
    CPU_SCALAR = 0
    CPU_AVX2 = 1
    CPU_AVX512 = 2
    CPU_NEON = 3
    GPU_CUDA = 4
    GPU_DIRECTX = 5
    GPU_VULKAN = 6
    IGPU_SHARED = 7
    RAM_SWAP = 8
    DISTRIBUTED = 9
    GPU_HIP_GFX950 = 10


def backend_name(t: BackendType) -> str:
    return BackendType(t).name


def is_hip_gfx950_available() -> bool:
    try:
        return _lib.probe()["gfx"] == 950
    except _lib.OilHipError:
        return False


def probe_hardware() -> dict:
    """The fields of HardwareProfile (backend.h:102-119) this path decides on."""
    hw = {"has_hip_gfx950": False, "vram_total": 0, "vram_free": 0, "cpu_threads": os.cpu_count() or 0}
    if is_hip_gfx950_available():
        import torch
        free, total = torch.cuda.mem_get_info()
        hw.update(has_hip_gfx950=True, vram_total=int(total), vram_free=int(free))
    return hw


def select_optimal_backend(hw: dict, model_size_bytes: int = 0) -> dict:
    """The rule the patch puts in front of select_optimal_backend (src/backend.cpp:732-786): the device when the model
    fits in 80 % of its free memory.  Anything else is the reference's own business (None here)."""
    if hw.get("has_hip_gfx950") and hw.get("vram_total", 0) > 0:
        if model_size_bytes == 0 or model_size_bytes <= int(hw["vram_free"] * 0.8):
            return {"type": BackendType.GPU_HIP_GFX950, "device_name": "hip-gfx950", "memory_fraction": 0.9}
    return {"type": None, "device_name": "", "memory_fraction": 0.0}


def _dev(a):
    import torch
    if isinstance(a, torch.Tensor):
        assert a.is_cuda and a.is_contiguous() and a.dtype == torch.float32
        return a
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()


def _back(t, like):
    import torch
    return t if isinstance(like, torch.Tensor) else t.cpu().numpy()


class Gfx950Backend:
    """ComputeBackend (backend.h:49-80) on the device.  Methods return their result instead of filling an output
    tensor; argument order and meaning are the reference's (CPU bodies: src/math.cpp:50-283)."""

    def type(self):
        return BackendType.GPU_HIP_GFX950

    def name(self):
        return "hip-gfx950"

    def is_available(self):
        return is_hip_gfx950_available()

    def memory_free(self):
        import torch
        return int(torch.cuda.mem_get_info()[0])

    def memory_total(self):
        import torch
        return int(torch.cuda.mem_get_info()[1])

    def synchronize(self):
        import torch
        torch.cuda.synchronize()

    def gemm(self, alpha, A, B, beta=0.0, C=None):
        import torch
        a, b = _dev(A), _dev(B)
        if a.dim() != 2 or b.dim() != 2 or a.shape[1] != b.shape[0]:
            raise _lib.OilHipError("gemm A cols != B rows")
        M, K, N = a.shape[0], a.shape[1], b.shape[1]
        c = _dev(C).clone() if C is not None else torch.zeros((M, N), dtype=torch.float32, device="cuda")
        if tuple(c.shape) != (M, N):
            raise _lib.OilHipError("gemm C shape mismatch")
        _lib.check(_lib.lib().oilhip_dense_gemm_f32(float(alpha), a.data_ptr(), b.data_ptr(), float(beta if C is not None else 0.0),
                                                    c.data_ptr(), M, N, K, _lib.current_stream()))
        return _back(c, A)

    def gemv(self, alpha, A, x, beta=0.0, y=None):
        import torch
        a, v = _dev(A), _dev(x)
        if a.dim() != 2 or v.numel() != a.shape[1]:
            raise _lib.OilHipError("gemv x size != A cols")
        out = _dev(y).clone() if y is not None else torch.zeros(a.shape[0], dtype=torch.float32, device="cuda")
        if out.numel() != a.shape[0]:
            raise _lib.OilHipError("gemv y size != A rows")
        _lib.check(_lib.lib().oilhip_dense_gemv_f32(float(alpha), a.data_ptr(), v.data_ptr(), float(beta if y is not None else 0.0),
                                                    out.data_ptr(), a.shape[0], a.shape[1], _lib.current_stream()))
        return _back(out, A)

    def softmax(self, x, axis=-1):
        import torch
        t = _dev(x)
        axis = axis + t.dim() if axis < 0 else axis
        if not 0 <= axis < t.dim():
            raise _lib.OilHipError("softmax axis out of range")
        outer = int(np.prod(t.shape[:axis], dtype=np.int64))
        inner = int(np.prod(t.shape[axis + 1:], dtype=np.int64))
        out = torch.empty_like(t)
        _lib.check(_lib.lib().oilhip_dense_softmax_f32(t.data_ptr(), out.data_ptr(), outer, t.shape[axis], inner, _lib.current_stream()))
        return _back(out, x)

    def _norm(self, kind, x, gamma, beta, eps):
        import torch
        t, g = _dev(x), _dev(gamma)
        n = t.shape[-1]
        if g.numel() != n:
            raise _lib.OilHipError("norm gamma dim mismatch")
        b = _dev(beta) if beta is not None else None
        if b is not None and b.numel() != n:
            raise _lib.OilHipError("layer_norm beta dim mismatch")
        out = torch.empty_like(t)
        _lib.check(_lib.lib().oilhip_dense_norm_f32(kind, t.data_ptr(), g.data_ptr(), b.data_ptr() if b is not None else None,
                                                    float(eps), out.data_ptr(), t.numel() // n if n else 0, n, _lib.current_stream()))
        return _back(out, x)

    def layer_norm(self, x, gamma, beta, eps):
        return self._norm(0, x, gamma, beta, eps)

    def rms_norm(self, x, gamma, eps):
        return self._norm(1, x, gamma, None, eps)

    def _map(self, op, a, b=None, s=0.0):
        import torch
        ta = _dev(a)
        tb = _dev(b) if b is not None else None
        if tb is not None and tb.numel() != ta.numel():
            raise _lib.OilHipError("elementwise shape mismatch")
        out = torch.empty_like(ta)
        _lib.check(_lib.lib().oilhip_dense_map_f32(op, ta.data_ptr(), tb.data_ptr() if tb is not None else None, float(s),
                                                   out.data_ptr(), ta.numel(), _lib.current_stream()))
        return _back(out, a)

    def relu(self, x):
        return self._map(0, x)

    def gelu(self, x):
        return self._map(1, x)

    def silu(self, x):
        return self._map(2, x)

    def add(self, a, b):
        return self._map(3, a, b)

    def mul(self, a, b):
        return self._map(4, a, b)

    def scale(self, s, x):
        return self._map(5, x, None, s)


def create(cfg: dict):
    """ComputeBackend::create (backend.h:79) for the one type this package provides."""
    if cfg.get("type") != BackendType.GPU_HIP_GFX950:
        raise _lib.OilHipError("only BackendType.GPU_HIP_GFX950 is provided here")
    if not is_hip_gfx950_available():
        raise _lib.OilHipError("no usable gfx950 device")
    return Gfx950Backend()
