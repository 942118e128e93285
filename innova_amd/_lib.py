"""ctypes binding of liboilhip.so.  There is no fallback: if the library has not
been built the import of a kernel entry point fails loudly."""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "liboilhip.so")

u8p = C.POINTER(C.c_uint8)
f32p = C.POINTER(C.c_float)
vp = C.c_void_p

# oilhip_block_t
BLOCK_DTYPE = np.dtype(
    [("cb_off", "<u8"), ("idx_off", "<u8"), ("cb_bytes", "<u4"), ("idx_bytes", "<u4"),
     ("nw", "<u4"), ("fmt", "u1"), ("reserved", "u1", (3,))], align=True)
assert BLOCK_DTYPE.itemsize == 32


class OilHipError(RuntimeError):
    """A liboilhip call failed (the counterpart of oil::Error, include/oil/types.h:184-190)."""


_lib = None

_SIGNATURES = {
    "oilhip_last_error": (C.c_char_p, []),
    "oilhip_probe": (C.c_int, [C.POINTER(C.c_int), C.POINTER(C.c_uint64), C.POINTER(C.c_int), C.c_char_p, C.c_size_t]),
    "oilhip_payload_bound": (C.c_size_t, [C.c_int, C.c_int]),
    "oilhip_quantize_block": (C.c_int, [C.c_int, vp, C.c_int, vp, C.c_size_t, C.POINTER(C.c_size_t),
                                        vp, C.c_size_t, C.POINTER(C.c_size_t)]),
    "oilhip_quantize_tensor": (C.c_int, [vp, C.c_uint32, vp, C.c_uint64, vp, C.c_uint64, vp,
                                         C.POINTER(C.c_uint64), C.c_int]),
    "oilhip_score_importance": (C.c_int, [vp, vp, C.c_int64, C.c_int, C.c_int, vp, C.c_int64]),
    "oilhip_plan_formats": (C.c_int, [C.c_float, vp, C.c_int64, C.c_int, vp, C.POINTER(C.c_float), C.POINTER(C.c_int), vp]),
    "oilhip_mix_allocate": (C.c_int, [vp, C.c_int, C.c_float, vp, C.c_int64, C.c_int, C.c_int64, C.c_int64, vp, vp, vp,
                                      C.c_int64, C.POINTER(C.c_int64)]),
    "oilhip_weights_create": (C.c_int, [vp, C.c_uint64, vp, C.c_uint32, C.c_uint64, C.c_uint64, C.POINTER(vp)]),
    "oilhip_weights_create_from_records": (C.c_int, [vp, C.c_uint64, vp, C.c_uint32, C.c_uint64, C.c_uint64, C.POINTER(vp)]),
    "oilhip_weights_destroy": (C.c_int, [vp]),
    "oilhip_weights_device_bytes": (C.c_int, [vp, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "oilhip_weights_info": (C.c_int, [vp, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64), C.POINTER(C.c_uint32),
                                      C.POINTER(C.c_uint64), C.POINTER(C.c_int)]),
    "oilhip_file_open": (C.c_int, [C.c_char_p, C.POINTER(vp)]),
    "oilhip_file_open_memory": (C.c_int, [vp, C.c_uint64, C.POINTER(vp)]),
    "oilhip_file_close": (C.c_int, [vp]),
    "oilhip_file_info": (C.c_int, [vp] + [C.POINTER(C.c_uint32)] * 5),
    "oilhip_file_config": (C.c_int, [vp, vp, C.c_uint32]),
    "oilhip_file_tensor": (C.c_int, [vp, C.c_uint32, C.c_char_p, C.c_size_t, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32),
                                     C.POINTER(C.c_uint64)]),
    "oilhip_file_find_tensor": (C.c_int, [vp, C.c_char_p, C.POINTER(C.c_uint32)]),
    "oilhip_file_block": (C.c_int, [vp, C.c_uint32, C.POINTER(C.c_uint8), C.POINTER(C.c_uint32), C.POINTER(u8p),
                                    C.POINTER(C.c_uint32), C.POINTER(u8p), C.POINTER(C.c_uint32)]),
    "oilhip_file_upload_tensor": (C.c_int, [vp, C.c_uint32, C.c_uint64, C.c_uint64, C.POINTER(vp)]),
    "oilhip_file_write": (C.c_int, [C.c_char_p, C.c_uint32, C.c_uint32, vp, C.c_uint32, C.c_uint32, C.POINTER(C.c_char_p), vp,
                                    vp, vp, C.c_uint32]),
    "oilhip_engine_dequant": (C.c_int, [C.c_int, vp, vp, C.c_int64, vp, C.c_int64, vp, vp]),
    "oilhip_engine_dense_gemm": (C.c_int, [C.c_int, vp, vp, vp, C.c_int64, vp, C.c_int64, C.c_int64, C.c_int64, vp]),
    "oilhip_weights_stack_rows": (C.c_int, [vp, C.c_int, C.POINTER(vp)]),
    "oilhip_rmsnorm_f32": (C.c_int, [vp, vp, C.c_int, C.c_int, vp, vp]),
    "oilhip_gemv_rmsnorm_f32": (C.c_int, [vp, vp, vp, vp, C.c_int, vp, vp]),
    "oilhip_mlp_step_f32": (C.c_int, [vp, vp, vp, vp, vp, C.c_int, vp, vp]),
    "oilhip_embed_rows_f32": (C.c_int, [vp, vp, C.c_int, vp, vp]),
    "oilhip_moe_route": (C.c_int, [vp, C.c_int64, C.c_int64, C.c_int64, vp, vp, vp]),
    "oilhip_moe_workspace_bytes": (C.c_size_t, [C.c_int64, C.c_int64, C.c_int64, C.c_int64]),
    "oilhip_moe_forward": (C.c_int, [vp, vp, vp, C.c_int, vp, vp, vp, C.c_int64, C.c_int64, vp, vp, C.c_size_t,
                                     C.POINTER(C.c_float), C.POINTER(C.c_int64), vp]),
    "oilhip_dequant_f32": (C.c_int, [vp, vp, vp]),
    "oilhip_gemv_f32": (C.c_int, [vp, vp, vp, C.c_int, vp]),
    "oilhip_gemv_f32_general": (C.c_int, [vp, vp, vp, C.c_int, vp]),
    "oilhip_gemv_oil4_f32_noalloc": (C.c_int, [vp, vp, vp, C.c_int, vp]),
    "oilhip_set_ordered_sums": (C.c_int, [C.c_int]),
    "oilhip_gemm_bf16": (C.c_int, [vp, vp, vp, C.c_int, vp]),
    "oilhip_gemm_f32": (C.c_int, [vp, vp, vp, C.c_int, vp]),
    "oilhip_release_stream_scratch": (C.c_int, [vp]),
    "oilhip_profile_gemv": (C.c_int, [C.c_int, vp, vp, C.c_float, vp, vp, C.c_int, C.c_int, C.c_int, vp, vp]),
    "oilhip_tl_gemm": (C.c_int, [C.c_int, vp, vp, vp, C.c_int, C.c_int, C.c_int, vp]),
    "oilhip_dense_gemm_f32": (C.c_int, [C.c_float, vp, vp, C.c_float, vp, C.c_int64, C.c_int64, C.c_int64, vp]),
    "oilhip_dense_gemv_f32": (C.c_int, [C.c_float, vp, vp, C.c_float, vp, C.c_int64, C.c_int64, vp]),
    "oilhip_dense_norm_f32": (C.c_int, [C.c_int, vp, vp, vp, C.c_float, vp, C.c_int64, C.c_int64, vp]),
    "oilhip_dense_softmax_f32": (C.c_int, [vp, vp, C.c_int64, C.c_int64, C.c_int64, vp]),
    "oilhip_dense_map_f32": (C.c_int, [C.c_int, vp, vp, C.c_float, vp, C.c_int64, vp]),
    "oilhip_flat_oil8_gemm": (C.c_int, [vp, vp, vp, vp, C.c_int, C.c_int, C.c_int, vp]),
    "oilhip_flat_oil4_gemm": (C.c_int, [vp, vp, vp, vp, C.c_int, C.c_int, C.c_int, vp]),
    "oilhip_prod_gemv_spark": (C.c_int, [vp, C.c_float, vp, vp, C.c_int, C.c_int, C.c_int, vp]),
    "oilhip_prod_gemv_oil4": (C.c_int, [vp, vp, C.c_float, vp, vp, C.c_int, C.c_int, C.c_int, vp]),
    "oilhip_prod_gemv_oil8": (C.c_int, [vp, vp, C.c_float, vp, vp, C.c_int, C.c_int, C.c_int, vp]),
    "oilhip_engine_quant_gemm": (C.c_int, [C.c_int, vp, vp, vp, vp, C.c_int64, C.c_int64, C.c_int64, vp]),
    "oilhip_kv_create": (C.c_int, [C.c_int, C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.POINTER(vp)]),
    "oilhip_kv_destroy": (C.c_int, [vp]),
    "oilhip_kv_append": (C.c_int, [vp, C.c_int, vp, vp, C.c_int64, vp]),
    "oilhip_kv_get_range": (C.c_int, [vp, C.c_int, C.c_int64, C.c_int64, vp, vp, C.POINTER(C.c_int64), vp]),
    "oilhip_kv_info": (C.c_int, [vp, C.POINTER(C.c_int), C.POINTER(C.c_int64), C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]),
    "oilhip_kv_clear": (C.c_int, [vp, vp]),
    "oilhip_kv_resize": (C.c_int, [vp, C.c_int64]),
    "oilhip_kv_state": (C.c_int, [vp, C.c_int, vp, vp, vp, vp]),
    "oilhip_kv_quantize_blocks": (C.c_int, [vp, C.c_int64, C.c_int64, vp, vp, vp]),
    "oilhip_kv_dequantize_blocks": (C.c_int, [vp, vp, vp, C.c_int64, C.c_int64, vp]),
}


def lib():
    """The loaded library.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise OilHipError(
                f"{LIB_PATH} is missing: build it first (make -C innova_amd/csrc, or "
                "python -c 'import __graft_entry__ as g; g.build()'); there is no CPU fallback")
        try:                          # torch ships its own HIP runtime: it has to be the one both of us use, so it
            import torch  # noqa: F401  # is loaded first (the other order leaves torch without a visible GPU)
        except ImportError:
            pass
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def exported_symbols():
    return list(_SIGNATURES)


def check(rc: int) -> None:
    if rc != 0:
        raise OilHipError(f"liboilhip error {rc}: {lib().oilhip_last_error().decode(errors='replace')}")


def probe() -> dict:
    """Runtime probe of the device path (cf. detect_cpu_isa / probe_hardware)."""
    gfx, hbm, cus = C.c_int(0), C.c_uint64(0), C.c_int(0)
    name = C.create_string_buffer(256)
    check(lib().oilhip_probe(C.byref(gfx), C.byref(hbm), C.byref(cus), name, 256))
    return {"gfx": gfx.value, "hbm_bytes": hbm.value, "compute_units": cus.value, "name": name.value.decode()}


def current_stream() -> int:
    import torch
    return torch.cuda.current_stream().cuda_stream
