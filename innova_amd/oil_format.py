"""Host mirror of the .oil container classes (include/oil/oil_format.h:14-108): OILReader over
liboilhip's mapped-file index, and a writer with OILWriter's section order."""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import numpy as np

from . import _lib
from .formats import Format
from .weights import DeviceWeights


@dataclass
class BlockData:
    """include/oil/oil_format.h:35-40"""
    format: Format
    codebook: np.ndarray
    indices: np.ndarray
    num_weights: int


class OILReader:
    def __init__(self, source):
        """source: a path, or the file's bytes."""
        self._f = C.c_void_p(0)
        L = _lib.lib()
        if isinstance(source, (bytes, bytearray, memoryview, np.ndarray)):
            buf = np.frombuffer(bytes(source), np.uint8) if not isinstance(source, np.ndarray) else np.ascontiguousarray(source, np.uint8)
            rc = L.oilhip_file_open_memory(buf.ctypes.data, buf.size, C.byref(self._f))
        else:
            rc = L.oilhip_file_open(str(source).encode(), C.byref(self._f))
        self.error = None if rc == 0 else L.oilhip_last_error().decode(errors="replace")
        self.version = self.flags = self.config_size = 0
        self._nblocks = self._ntensors = 0
        self._tensors = []
        if rc == 0:
            v, fl, cs, nb, nt = (C.c_uint32(0) for _ in range(5))
            _lib.check(L.oilhip_file_info(self._f, C.byref(v), C.byref(fl), C.byref(cs), C.byref(nb), C.byref(nt)))
            self.version, self.flags, self.config_size = v.value, fl.value, cs.value
            self._nblocks, self._ntensors = nb.value, nt.value
            for i in range(nt.value):
                name = C.create_string_buffer(65536 + 1)
                st, cnt, nw = C.c_uint32(0), C.c_uint32(0), C.c_uint64(0)
                _lib.check(L.oilhip_file_tensor(self._f, i, name, len(name), C.byref(st), C.byref(cnt), C.byref(nw)))
                self._tensors.append((name.value.decode(errors="replace"), st.value, cnt.value, nw.value))

    def valid(self) -> bool:
        return bool(self._f.value)

    def _need(self):
        if not self._f.value:
            raise _lib.OilHipError(f"OILReader is not valid: {self.error}")

    def close(self):
        if self._f.value:
            _lib.lib().oilhip_file_close(self._f)
            self._f = C.c_void_p(0)

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def read_config(self) -> bytes:
        self._need()
        buf = np.zeros(max(self.config_size, 1), np.uint8)
        _lib.check(_lib.lib().oilhip_file_config(self._f, buf.ctypes.data, buf.size))
        return buf[: self.config_size].tobytes()

    def num_blocks(self) -> int:
        return self._nblocks

    def tensor_names(self) -> list:
        return [t[0] for t in self._tensors]

    def _find(self, name):
        for i, t in enumerate(self._tensors):
            if t[0] == name:
                return i, t
        return None, None

    def tensor_blocks(self, name):
        """-> (start, count) or None"""
        _, t = self._find(name)
        return None if t is None else (t[1], t[2])

    def read_block(self, block_id: int) -> BlockData:
        self._need()
        fmt, nw, cbn, ixn = C.c_uint8(0), C.c_uint32(0), C.c_uint32(0), C.c_uint32(0)
        cb, ix = C.POINTER(C.c_uint8)(), C.POINTER(C.c_uint8)()
        _lib.check(_lib.lib().oilhip_file_block(self._f, int(block_id), C.byref(fmt), C.byref(nw), C.byref(cb),
                                                C.byref(cbn), C.byref(ix), C.byref(ixn)))
        grab = lambda p, n: np.ctypeslib.as_array(p, shape=(n,)).copy() if n else np.zeros(0, np.uint8)  # noqa: E731
        return BlockData(Format(fmt.value), grab(cb, cbn.value), grab(ix, ixn.value), nw.value)

    def tensor_formats(self, name) -> list:
        t = self.tensor_blocks(name)
        if t is None:
            return []
        return [self.read_block(t[0] + b).format for b in range(t[1]) if t[0] + b < self._nblocks]

    def upload_tensor(self, name, rows: int = 0, cols: int = 0) -> DeviceWeights:
        """The tensor's block records into HBM (rows = cols = 0: a 1 x numel tensor)."""
        self._need()
        i, t = self._find(name)
        if t is None:
            raise _lib.OilHipError(f"no tensor named {name!r}")
        h = C.c_void_p(0)
        _lib.check(_lib.lib().oilhip_file_upload_tensor(self._f, i, rows, cols, C.byref(h)))
        if rows == 0 and cols == 0:
            rows, cols = 1, t[3]
        return DeviceWeights(h.value, rows, cols)

    def read_tensor(self, name):
        """Decoded float32 weights (numpy, flat), dequantized on the GPU; None if absent or empty
        (the reference returns an empty Tensor, src/oil_format.cpp:445-483)."""
        _, t = self._find(name)
        if t is None or t[3] == 0:
            return None
        with self.upload_tensor(name) as w:
            return w.dequant().cpu().numpy()


def write_oil(path, tensors, version: int = 1, flags: int = 0, config: bytes = b"") -> None:
    """tensors: [(name, payload uint8[], blocks BLOCK_DTYPE[])] as quantize_tensor returns them.
    Section order and record framing of OILWriter (src/oil_format.cpp:196-279)."""
    names = [t[0].encode() for t in tensors]
    counts = np.array([len(t[2]) for t in tensors], np.uint32)
    pays, blks, base = [], [], 0
    for _, payload, blocks in tensors:
        payload = np.ascontiguousarray(payload, np.uint8)
        b = np.array(blocks, dtype=_lib.BLOCK_DTYPE, copy=True)
        b["cb_off"] += base
        b["idx_off"] += base
        pays.append(payload)
        blks.append(b)
        base += payload.size
    payload = np.concatenate(pays) if pays else np.zeros(0, np.uint8)
    blocks = np.concatenate(blks) if blks else np.zeros(0, _lib.BLOCK_DTYPE)
    arr = (C.c_char_p * max(len(names), 1))(*names)
    cfg = np.frombuffer(config, np.uint8) if config else np.zeros(1, np.uint8)
    _lib.check(_lib.lib().oilhip_file_write(str(path).encode(), version, flags, cfg.ctypes.data if config else None,
                                            len(config), len(names), arr, counts.ctypes.data,
                                            payload.ctypes.data if payload.size else None,
                                            blocks.ctypes.data if blocks.size else None, blocks.size))
