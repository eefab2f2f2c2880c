"""Reader of built tier packs ("SBRPACK1") for the iu8 linears: ctypes binding of the
`saber_iu8_pack_*` functions of include/saber_iu8.h (the counterpart of
crates/saber-mem/src/pack/reader.rs `PackReader`). Host memory only; nothing here touches a GPU."""
import ctypes as C

import numpy as np

from . import iu8


class Header(C.Structure):
    _fields_ = [("format_version", C.c_uint32), ("record_count", C.c_uint32), ("tp_size", C.c_uint32), ("rank", C.c_uint32),
                ("chunk_bytes", C.c_uint32), ("data_off", C.c_uint64), ("file_bytes", C.c_uint64),
                ("build_unix_seconds", C.c_uint64), ("plan_hash", C.c_uint8 * 32), ("tier_id", C.c_uint8 * 32)]


class Record(C.Structure):
    _fields_ = [("name", C.c_char * 128), ("rank", C.c_uint32), ("layout_id", C.c_uint32), ("flags", C.c_uint32),
                ("dtype", C.c_uint16), ("ndim", C.c_uint8), ("shard_kind", C.c_uint8), ("data_off", C.c_uint64),
                ("length", C.c_uint64), ("shape", C.c_uint64 * 8), ("sha256", C.c_uint8 * 32)]


class LinearInfo(C.Structure):
    _fields_ = [("wkind", C.c_int), ("n", C.c_uint32), ("k", C.c_uint32), ("w_record", C.c_uint32), ("s_record", C.c_uint32),
                ("w_bytes", C.c_uint64), ("shard_kind", C.c_uint8)]


def _lib():
    L = iu8.lib()
    if not getattr(L, "_pack_bound", False):
        L.saber_iu8_pack_open.argtypes = [C.c_char_p, C.c_char_p, C.POINTER(C.c_void_p)]
        L.saber_iu8_pack_close.argtypes = [C.c_void_p]
        L.saber_iu8_pack_close.restype = None
        L.saber_iu8_pack_info.argtypes = [C.c_void_p, C.POINTER(Header)]
        L.saber_iu8_pack_record_at.argtypes = [C.c_void_p, C.c_uint32, C.POINTER(Record)]
        L.saber_iu8_pack_find.argtypes = [C.c_void_p, C.c_char_p]
        L.saber_iu8_pack_read.argtypes = [C.c_void_p, C.c_uint32, C.c_void_p, C.c_uint64]
        L.saber_iu8_pack_linear.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(LinearInfo)]
        L.saber_iu8_pack_load_linear.argtypes = [C.c_void_p, C.c_char_p, C.c_void_p, C.c_uint64, C.c_void_p, C.c_uint64]
        L._pack_bound = True
    return L


class Pack:
    """An opened, structurally validated pack. `expected_plan_hash` (32 bytes) refuses a pack built
    for another plan (PackReader::open_expecting)."""

    def __init__(self, path, expected_plan_hash=None):
        self._h = C.c_void_p()
        if expected_plan_hash is not None and len(expected_plan_hash) != 32:
            raise ValueError("a plan hash is 32 bytes")
        iu8._check(_lib().saber_iu8_pack_open(str(path).encode(), expected_plan_hash, C.byref(self._h)))

    def close(self):
        if self._h:
            _lib().saber_iu8_pack_close(self._h)
            self._h = C.c_void_p()

    __del__ = close

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    @property
    def header(self):
        h = Header()
        iu8._check(_lib().saber_iu8_pack_info(self._h, C.byref(h)))
        return h

    def record(self, index):
        r = Record()
        iu8._check(_lib().saber_iu8_pack_record_at(self._h, index, C.byref(r)))
        return r

    def find(self, name):
        return _lib().saber_iu8_pack_find(self._h, name.encode())

    def read(self, index):
        r = self.record(index)
        out = np.empty(r.length, np.uint8)
        iu8._check(_lib().saber_iu8_pack_read(self._h, index, out.ctypes.data_as(C.c_void_p), out.nbytes))
        return out

    def linear(self, op):
        li = LinearInfo()
        iu8._check(_lib().saber_iu8_pack_linear(self._h, op.encode(), C.byref(li)))
        return li

    def load_linear(self, op):
        """-> (wkind, n, k, codes in the gfx950 fragment order (uint8), row scales (float32))."""
        li = self.linear(op)
        w = np.empty(li.w_bytes, np.uint8)
        ws = np.empty(li.n, np.float32)
        iu8._check(_lib().saber_iu8_pack_load_linear(self._h, op.encode(), w.ctypes.data_as(C.c_void_p), w.nbytes,
                                                     ws.ctypes.data_as(C.c_void_p), li.n))
        return li.wkind, li.n, li.k, w, ws
