"""Host mirror of the decode-step pieces of Qwen35Engine around the quantized matmuls
(src/adapters/tools/qwen35_engine.cpp: rmsnorm :39-44, mlp_step :611-621, embedding lookup :756-760)."""
from __future__ import annotations

from . import _lib
from .weights import DeviceWeights


def rmsnorm(x, w, out=None):
    """out = x * r * (1 + w), r = 1 / sqrt(mean(x^2) + 1e-6), per row of a float32 cuda tensor [..., n]."""
    import torch
    assert x.is_cuda and w.is_cuda and x.dtype == torch.float32 and w.dtype == torch.float32 and x.is_contiguous()
    n = w.numel()
    rows = x.numel() // n
    if out is None:
        out = torch.empty_like(x)
    _lib.check(_lib.lib().oilhip_rmsnorm_f32(x.data_ptr(), w.data_ptr(), n, rows, out.data_ptr(), _lib.current_stream()))
    return out


def gemv_rmsnorm(w: DeviceWeights, x, norm_w, out=None):
    """y = W . rmsnorm(x; norm_w): the norm in front of a projection, formed inside the GEMV for one OIL4 row."""
    import torch
    assert x.is_cuda and x.dtype == torch.float32 and x.is_contiguous() and norm_w.is_cuda and norm_w.dtype == torch.float32
    x2 = x.reshape(-1, w.cols)
    M = x2.shape[0]
    if out is None:
        out = torch.empty((M, w.rows), dtype=torch.float32, device=x.device)
    xn = torch.empty_like(x2)
    _lib.check(_lib.lib().oilhip_gemv_rmsnorm_f32(w.handle, x2.data_ptr(), norm_w.data_ptr(), out.data_ptr(), M, xn.data_ptr(),
                                                  _lib.current_stream()))
    torch.cuda.current_stream().synchronize()      # xn is released when this returns
    return out


def mlp_step(gate_up: DeviceWeights, down: DeviceWeights, x, out=None, norm_w=None):
    """y = down(siluf(gate x') * up x'), x' = rmsnorm(x; norm_w) or x; gate_up = the gate and up projections stacked
    (DeviceWeights.stack_rows)."""
    import torch
    assert x.is_cuda and x.dtype == torch.float32 and x.is_contiguous()
    x2 = x.reshape(-1, gate_up.cols)
    M, F = x2.shape[0], down.cols
    if out is None:
        out = torch.empty((M, down.rows), dtype=torch.float32, device=x.device)
    scratch = torch.empty((3 * F + gate_up.cols) * M, dtype=torch.float32, device=x.device)
    _lib.check(_lib.lib().oilhip_mlp_step_f32(gate_up.handle, down.handle, x2.data_ptr(),
                                              norm_w.data_ptr() if norm_w is not None else None, out.data_ptr(), M,
                                              scratch.data_ptr(), _lib.current_stream()))
    torch.cuda.current_stream().synchronize()      # scratch is released when this returns
    return out


def embed_rows(w: DeviceWeights, ids, out=None):
    """Rows ids[i] of a quantized [vocab][cols] tensor decoded to float32 [n][cols]; ids: int32 cuda tensor."""
    import torch
    assert ids.is_cuda and ids.dtype == torch.int32 and ids.is_contiguous()
    n = ids.numel()
    if out is None:
        out = torch.empty((n, w.cols), dtype=torch.float32, device=ids.device)
    _lib.check(_lib.lib().oilhip_embed_rows_f32(w.handle, ids.data_ptr(), n, out.data_ptr(), _lib.current_stream()))
    return out
