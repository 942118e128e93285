"""Host mirror of the reference's format routing: FormatPlanner (include/oil/format_planner.h:44-78)
and the adaptive mix allocator FormatRegistry::allocate_mix_blocks (include/oil/format_registry.h:151-154).

The planner is host arithmetic (liboilhip's C++ host code); the mix allocator measures every
candidate encoding's reconstruction error on the GPU."""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field

import numpy as np

from . import _lib
from .formats import Format, format_bpw

# registry mixes with their member formats in tier order and claimed bits per weight
# (src/format_registry.cpp:42-101)
MIXES = {
    "OIL8+OIL2_1_99": ((Format.OIL8, Format.OIL2), (0.01, 0.99), 2.06),
    "OIL8+OIL4_5_95": ((Format.OIL8, Format.OIL4), (0.05, 0.95), 4.20),
    "OIL4+OIL2_10_90": ((Format.OIL4, Format.OIL2), (0.10, 0.90), 2.20),
    "OIL8+OIL2_10_90": ((Format.OIL8, Format.OIL2), (0.10, 0.90), 2.60),
    "SPARK+OIL8_5_95": ((Format.SPARK_Q0, Format.OIL8), (0.05, 0.95), 7.675),
    "OIL16+OIL4_1_99": ((Format.OIL16, Format.OIL4), (0.01, 0.99), 4.12),
    "OIL16+OIL8_5_95": ((Format.OIL16, Format.OIL8), (0.05, 0.95), 8.40),
    "OIL32+OIL8_1_99": ((Format.OIL32, Format.OIL8), (0.01, 0.99), 8.24),
    "SPARK_MIX_Q0": ((Format.OIL8_GRP, Format.OIL4_GRP, Format.OIL2_GRP, Format.OIL1_GRP), (0.01, 0.02, 0.52, 0.45), 1.925),
    "QUAD_OIL2_OIL4_OIL8_OIL16": ((Format.OIL16, Format.OIL8, Format.OIL4, Format.OIL2), (0.01, 0.05, 0.24, 0.70), 2.92),
    "QUAD_OIL4_OIL8_OIL16_OIL32": ((Format.OIL32, Format.OIL16, Format.OIL8, Format.OIL4), (0.01, 0.05, 0.24, 0.70), 5.84),
    "QUAD_SPARK_Q1": ((Format.OIL32, Format.OIL8_GRP, Format.OIL2_GRP, Format.OIL1_GRP), (0.01, 0.01, 0.46, 0.52), 2.075),
}


@dataclass
class FormatPlan:
    """include/oil/format_planner.h:20-36 (blocks flattened to one format id per block)."""
    target_bpw: float
    achieved_bpw: float
    formats: np.ndarray            # uint8[num_blocks], Format ids
    uses_mix: bool
    counts: dict = field(default_factory=dict)   # num_oil32_blocks ... num_oil1_blocks


class FormatPlanner:
    def __init__(self, target_bpw: float = 1.50):
        self.target_bpw = float(target_bpw)
        self._scores = np.zeros(0, np.float32)

    def _score(self, weights, aux, block_size, fisher):
        w = np.ascontiguousarray(weights, np.float32).reshape(-1)
        a = None if aux is None else np.ascontiguousarray(aux, np.float32).reshape(-1)
        if a is not None and a.size != w.size:
            raise _lib.OilHipError("score_importance: weights and activations differ in size")
        nb = (w.size + block_size - 1) // block_size
        s = np.zeros(nb, np.float32)
        _lib.check(_lib.lib().oilhip_score_importance(w.ctypes.data, None if a is None else a.ctypes.data, w.size,
                                                      int(block_size), int(fisher), s.ctypes.data, nb))
        self._scores = s

    def score_importance(self, weights, calibration_activations=None, block_size: int = 256, fisher: bool = False):
        self._score(weights, calibration_activations, block_size, fisher)

    def score_importance_fisher(self, weights, gradients, block_size: int = 256):
        self._score(weights, gradients, block_size, True)

    def importance_scores(self) -> np.ndarray:
        return self._scores

    def allocate(self, num_weight_blocks: int, weights_per_block: int = 256) -> FormatPlan:
        nb = int(num_weight_blocks)
        fmts = np.zeros(max(nb, 1), np.uint8)
        ach, mix = C.c_float(0), C.c_int(0)
        cnt = np.zeros(7, np.int32)
        s = self._scores
        _lib.check(_lib.lib().oilhip_plan_formats(self.target_bpw, s.ctypes.data if s.size else None, s.size, nb,
                                                  fmts.ctypes.data, C.byref(ach), C.byref(mix), cnt.ctypes.data))
        names = ["num_oil32_blocks", "num_oil16_blocks", "num_oil8_blocks", "num_oil4_blocks", "num_oil2_blocks",
                 "num_spark_blocks", "num_oil1_blocks"]
        return FormatPlan(self.target_bpw, float(ach.value), fmts[:nb].copy(), bool(mix.value),
                          dict(zip(names, (int(c) for c in cnt))))

    def plan_for_model(self, num_weights: int) -> FormatPlan:
        return self.allocate(int(num_weights) // 256, 256)

    @staticmethod
    def plan_for_target(target_bpw: float, num_blocks: int, weights_per_block: int = 256) -> FormatPlan:
        return FormatPlanner(target_bpw).allocate(num_blocks, weights_per_block)

    @staticmethod
    def estimate_bpw(plan: FormatPlan) -> float:
        if plan.formats.size == 0:
            return 0.0
        total = np.float32(0)
        for f in plan.formats:
            total = np.float32(total + np.float32(format_bpw(int(f))))
        return float(total / np.float32(plan.formats.size))


def allocate_mix_blocks(mix, data, block_size: int = 256, shape=None):
    """-> (formats uint8[nb], block_starts int64[nb], block_lens int64[nb]).  mix: a registry
    name or (member formats, effective_bpw)."""
    if isinstance(mix, str):
        if mix not in MIXES:
            raise _lib.OilHipError(f"unknown mix {mix!r}")
        tiers, _, bpw = MIXES[mix]
    else:
        tiers, bpw = mix
    t = np.array([int(f) for f in tiers], np.uint8)
    d = np.ascontiguousarray(data, np.float32).reshape(-1)
    rows, cols = (int(shape[0]), int(shape[1])) if shape is not None and len(shape) >= 2 else (0, 0)
    nb = C.c_int64(0)
    L = _lib.lib()
    _lib.check(L.oilhip_mix_allocate(t.ctypes.data, t.size, bpw, d.ctypes.data, d.size, int(block_size), rows, cols,
                                     None, None, None, 0, C.byref(nb)))
    fm = np.zeros(nb.value, np.uint8)
    st = np.zeros(nb.value, np.int64)
    ln = np.zeros(nb.value, np.int64)
    _lib.check(L.oilhip_mix_allocate(t.ctypes.data, t.size, bpw, d.ctypes.data, d.size, int(block_size), rows, cols,
                                     fm.ctypes.data, st.ctypes.data, ln.ctypes.data, nb.value, C.byref(nb)))
    return fm, st, ln
