"""The read-only streaming probe (innova_amd/csrc/liboilhip_probe.so) is a measurement tool beside the product: the
product library and its header do not know it, and it refuses bad arguments before touching the device."""
import ctypes
import os
import re

import innova_amd as ia

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PATH = os.path.join(ROOT, "innova_amd", "csrc", "liboilhip_probe.so")


def test_probe_is_not_part_of_the_product_abi():
    header = open(os.path.join(ROOT, "include", "oilhip.h")).read()
    assert "probe_read" not in header and "read_probe" not in header
    assert not any("read_probe" in s or "oilprobe" in s for s in ia._lib.exported_symbols())


def test_probe_refuses_bad_arguments():
    assert os.path.exists(PATH), "liboilhip_probe.so is not built (make -C innova_amd/csrc)"
    L = ctypes.CDLL(PATH)
    L.oilprobe_read.restype = ctypes.c_int
    L.oilprobe_read.argtypes = [ctypes.c_void_p, ctypes.c_uint64] + [ctypes.c_int] * 5 + [ctypes.c_void_p, ctypes.c_void_p]
    L.oilprobe_last_error.restype = ctypes.c_char_p
    buf = ctypes.create_string_buffer(64)
    p = (ctypes.addressof(buf) + 15) & ~15

    def refused(rc, word):
        assert rc != 0 and re.search(word, L.oilprobe_last_error().decode()), L.oilprobe_last_error()

    refused(L.oilprobe_read(None, 4096, 4, 0, 0, 256, 512, p, None), "null")
    refused(L.oilprobe_read(p, 4096, 3, 0, 0, 256, 512, p, None), "in flight")
    refused(L.oilprobe_read(p, 4096, 4, 0, 0, 256, 100, p, None), "threads")
    refused(L.oilprobe_read(p, 4096, 4, 0, 3, 256, 512, p, None), "pattern")
    refused(L.oilprobe_read(p, 1 << 20, 4, 0, 2, 256, 256, p, None), "pattern 2")      # needs 512 threads
    refused(L.oilprobe_read(p, 1 << 20, 4, 0, 2, 256, 512, p, None), "pattern 2")      # less than 32 KB per workgroup
