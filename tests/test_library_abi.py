"""CPU-side checks of the product: the C-ABI library loads and exports every
symbol include/oilhip.h declares, and the host quantizer is byte-identical with
the oracle and the golden vectors (no GPU needed, no compute calls)."""
import ctypes
import os
import re

import numpy as np

import innova_amd as ia
import oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
G = np.load(os.path.join(ROOT, "tests", "golden", "codec.npz"))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "oilhip.h")).read()
    declared = set(re.findall(r"\b(oilhip_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 18
    L = ctypes.CDLL(ia._lib.LIB_PATH)
    for name in sorted(declared):
        assert hasattr(L, name), f"{name} is declared in oilhip.h but not exported"
    assert declared <= set(ia._lib.exported_symbols()) | {"oilhip_last_error"}


def test_block_struct_layout_matches_header():
    assert ia._lib.BLOCK_DTYPE.itemsize == 32
    assert [ia._lib.BLOCK_DTYPE.fields[k][1] for k in ("cb_off", "idx_off", "cb_bytes", "idx_bytes", "nw", "fmt")] == [0, 8, 16, 20, 24, 28]


def test_format_enum_values():
    # tests/test_format.cpp:183-186 pins these
    assert ia.Format.OIL1 == 0 and ia.Format.SPARK_Q0 == 1 and ia.Format.OIL4 == 3 and ia.Format.SPARK_SPARSE_GRP == 14
    for f in ia.Format:
        assert ia.format_bpw(f) == O.lib().orc_format_bpw(int(f))


def test_host_quantizer_matches_golden_payloads():
    for i in range(G["fmt"].size):
        fmt, n = int(G["fmt"][i]), int(G["n"][i])
        w = G["w_bits"][G["w_off"][i]: G["w_off"][i] + n].view(np.float32)
        idx, cb = ia.block_codec.quantize_block_all(fmt, w)
        assert np.array_equal(idx, G["idx"][G["idx_off"][i]: G["idx_off"][i] + G["idx_len"][i]]), G["tags"][i]
        assert np.array_equal(cb, G["cb"][G["cb_off"][i]: G["cb_off"][i] + G["cb_len"][i]]), G["tags"][i]


def test_host_quantizer_matches_oracle_tensor():
    rng = np.random.default_rng(0)
    w = (rng.standard_normal(256 * 64 + 77) * 0.02).astype(np.float32)
    w[512:768] = 0
    fmts = rng.integers(0, 15, 65).astype(np.uint8)
    p1, b1 = ia.block_codec.quantize_tensor(w, fmts)
    p2, b2 = O.quantize_tensor(w, fmts)
    assert np.array_equal(p1, p2)
    for k in ("cb_off", "idx_off", "cb_bytes", "idx_bytes", "nw", "fmt"):
        assert np.array_equal(b1[k], b2[k])
    for f in ia.Format:
        assert ia.block_codec.payload_bound(f, 256) == ia.FULL_BLOCK_BYTES[f] == O.max_payload_bytes(int(f), 256)


def test_host_quantizer_rejects_bad_arguments():
    import pytest
    with pytest.raises(ia.OilHipError):
        ia.block_codec.quantize_block_all(99, np.zeros(4, np.float32))
    with pytest.raises(ia.OilHipError):
        ia.block_codec.quantize_tensor(np.zeros(512, np.float32), np.zeros(3, np.uint8))


def test_entry_points_reject_bad_arguments_before_touching_the_device():
    """Argument checks come first in every entry point: these calls fail with OILHIP_E_ARG on a machine without a GPU
    (nothing is launched) and the thread-local message says why."""
    import ctypes as C

    from innova_amd import _lib
    L = _lib.lib()
    one = C.c_float(0.0)
    p = C.addressof(one)

    def refused(rc, needle):
        assert rc != 0
        assert needle in L.oilhip_last_error().decode()

    refused(L.oilhip_tl_gemm(3, p, p, p, 1, 1, 3, None), "kind")
    refused(L.oilhip_tl_gemm(2, p, p, p, 1, 1, 16, None), "multiple of 3")
    refused(L.oilhip_tl_gemm(1, None, p, p, 1, 1, 4, None), "null")
    refused(L.oilhip_dense_map_f32(9, p, p, 0.0, p, 4, None), "operation")
    refused(L.oilhip_dense_map_f32(3, p, None, 0.0, p, 4, None), "null")
    refused(L.oilhip_dense_norm_f32(2, p, p, p, 1e-5, p, 1, 4, None), "kind")
    refused(L.oilhip_dense_gemm_f32(1.0, p, p, 0.0, p, -1, 1, 1, None), "negative")
    refused(L.oilhip_dense_gemv_f32(1.0, None, p, 0.0, p, 2, 2, None), "null")
    refused(L.oilhip_dense_softmax_f32(None, p, 1, 4, 1, None), "null")
    refused(L.oilhip_profile_gemv(4, p, p, 1.0, p, p, 4, 16, 10, None, None), "null result")
    perf = (C.c_uint64 * 4)()
    refused(L.oilhip_profile_gemv(5, p, p, 1.0, p, p, 4, 16, 10, C.addressof(perf), None), "kind")
    # empty problems are not errors and launch nothing
    assert L.oilhip_tl_gemm(1, p, p, p, 0, 4, 8, None) == 0
    assert L.oilhip_dense_map_f32(0, p, None, 0.0, p, 0, None) == 0
    assert L.oilhip_dense_gemm_f32(1.0, p, p, 0.0, p, 0, 5, 5, None) == 0
