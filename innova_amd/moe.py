"""Host mirror of the reference's mixture-of-experts routing and batched dispatch
(include/oil/moe_variants.h:693-706) over experts held as quantized device tensors."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from .weights import DeviceWeights


def softmax_with_topk(logits, k: int):
    """-> (probs [T][E] float32, indices [T][k] int64, weights [T][k] float32), all numpy
    (src/moe_variants.cpp:97-134: weights are the raw probabilities of the k largest)."""
    lg = np.ascontiguousarray(logits, np.float32)
    T, E = lg.shape
    probs = np.zeros((T, E), np.float32)
    idx = np.zeros((T, k), np.int64)
    w = np.zeros((T, k), np.float32)
    _lib.check(_lib.lib().oilhip_moe_route(lg.ctypes.data, T, E, k, probs.ctypes.data, idx.ctypes.data, w.ctypes.data))
    return probs, idx, w


class ExpertFFN:
    """gate/up: [F][D] tensors, down: [D][F] (ExpertFFN, include/oil/moe_variants.h:126-135, SiLU)."""

    def __init__(self, gate: DeviceWeights, up: DeviceWeights, down: DeviceWeights):
        self.gate_proj, self.up_proj, self.down_proj = gate, up, down


def moe_workspace(x, experts, K: int):
    """A device buffer of the size one step over x needs (oilhip_moe_workspace_bytes): a caller that passes it to
    moe_dispatch_batched owns it across steps, and the call then neither allocates nor waits for the stream."""
    import torch
    T, D = x.shape
    nbytes = _lib.lib().oilhip_moe_workspace_bytes(T, K, D, experts[0].gate_proj.rows)
    return torch.empty(nbytes, dtype=torch.uint8, device=x.device)


def moe_dispatch_batched(x, experts, indices, weights, want_z_loss: bool = True, workspace=None, out=None):
    """x: float32 cuda tensor [T][D]; experts: list of ExpertFFN; indices/weights: [T][K] host arrays.
    -> (out cuda tensor [T][D], z_loss or None, dropped)   (src/moe_variants.cpp:767-827)
    With `workspace` (moe_workspace) and without the z-loss the call only queues launches on the current stream: it
    can be captured into a graph, and the caller keeps workspace and out alive until the work is done."""
    import torch
    assert x.is_cuda and x.dtype == torch.float32 and x.is_contiguous() and x.dim() == 2
    T, D = x.shape
    idx = np.ascontiguousarray(indices, np.int64)
    w = np.ascontiguousarray(weights, np.float32)
    assert idx.shape == w.shape and idx.shape[0] == T
    K = idx.shape[1]
    E = len(experts)
    F = experts[0].gate_proj.rows
    arr = lambda ts: (C.c_void_p * E)(*[t.handle for t in ts])  # noqa: E731
    g, u, d = arr([e.gate_proj for e in experts]), arr([e.up_proj for e in experts]), arr([e.down_proj for e in experts])
    L = _lib.lib()
    nbytes = L.oilhip_moe_workspace_bytes(T, K, D, F)
    own_ws = workspace is None
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device) if own_ws else workspace
    assert ws.is_cuda and ws.dtype == torch.uint8 and ws.numel() >= nbytes
    if out is None:
        out = torch.empty((T, D), dtype=torch.float32, device=x.device)
    assert out.is_cuda and out.dtype == torch.float32 and out.is_contiguous() and tuple(out.shape) == (T, D)
    z, dropped = C.c_float(0), C.c_int64(0)
    _lib.check(L.oilhip_moe_forward(g, u, d, E, x.data_ptr(), idx.ctypes.data, w.ctypes.data, T, K, out.data_ptr(),
                                    ws.data_ptr(), nbytes, C.byref(z) if want_z_loss else None, C.byref(dropped),
                                    _lib.current_stream()))
    if own_ws:
        torch.cuda.current_stream().synchronize()   # ws is released when this returns
    return out, (z.value if want_z_loss else None), dropped.value
