"""innova_amd -- MI355X (gfx950) implementation of the OIL quantized-weight matmul
path: .oil block dequantization fused with GEMV (decode) and GEMM (prefill).

All compute goes through liboilhip.so (hand-written HIP behind a C ABI,
include/oilhip.h); importing works without a GPU, calling a kernel does not.
"""
from .formats import Format, format_bpw, FULL_BLOCK_BYTES, WIRE_BLOCK  # noqa: F401
from ._lib import OilHipError, lib, probe  # noqa: F401
from . import backend, block_codec, format_planner, kernel, layers, moe  # noqa: F401
from .kv_cache import OIL4KVCache  # noqa: F401
from .weights import DeviceWeights  # noqa: F401
from .oil_format import OILReader, write_oil  # noqa: F401

__all__ = ["Format", "format_bpw", "FULL_BLOCK_BYTES", "WIRE_BLOCK", "OilHipError", "lib", "probe",
           "backend", "block_codec", "format_planner", "kernel", "layers", "moe", "DeviceWeights", "OILReader", "write_oil"]
