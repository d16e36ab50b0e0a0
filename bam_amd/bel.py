"""Graph file pair <prefix>.col / <prefix>.dst as the reference's graph benchmarks read it
(benchmarks/bfs/main.cu:1238-1284): ctypes wrapper over the host library's reader and writer (include/bel.h)."""
import ctypes
import os

import numpy as np

from . import _lib

HEADER_BYTES = 16
_U64P = ctypes.POINTER(ctypes.c_uint64)


def _h():
    L = _lib.load_host()
    if not getattr(L, "_bel_ready", False):
        L.bel_info.restype = ctypes.c_int
        L.bel_info.argtypes = [ctypes.c_char_p, _U64P, _U64P]
        L.bel_read_offsets.restype = ctypes.c_int
        L.bel_read_offsets.argtypes = [ctypes.c_char_p, ctypes.c_void_p, ctypes.c_uint64]
        L.bel_read_edges.restype = ctypes.c_int
        L.bel_read_edges.argtypes = [ctypes.c_char_p, ctypes.c_uint64, ctypes.c_uint64, ctypes.c_void_p]
        L.bel_write.restype = ctypes.c_int
        L.bel_write.argtypes = [ctypes.c_char_p, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p, ctypes.c_uint64]
        L._bel_ready = True
    return L


def _chk(rc, what):
    if rc:
        raise OSError(rc, f"{what}: {os.strerror(rc)}")


def info(prefix):
    """(V + 1, E) from the two headers"""
    n, e = ctypes.c_uint64(0), ctypes.c_uint64(0)
    _chk(_h().bel_info(os.fsencode(prefix), ctypes.byref(n), ctypes.byref(e)), f"bel_info({prefix})")
    return n.value, e.value


def read_offsets(prefix):
    n, _ = info(prefix)
    out = np.empty(n, dtype=np.uint64)
    _chk(_h().bel_read_offsets(os.fsencode(prefix), out.ctypes.data, n), f"bel_read_offsets({prefix})")
    return out


def read_edges(prefix, first=0, count=None):
    if count is None:
        count = info(prefix)[1] - first
    out = np.empty(count, dtype=np.uint64)
    _chk(_h().bel_read_edges(os.fsencode(prefix), first, count, out.ctypes.data), f"bel_read_edges({prefix})")
    return out


def write(prefix, offsets, edges):
    offsets = np.ascontiguousarray(offsets, dtype=np.uint64)
    edges = np.ascontiguousarray(edges, dtype=np.uint64)
    _chk(_h().bel_write(os.fsencode(prefix), offsets.ctypes.data, len(offsets), edges.ctypes.data, len(edges)), f"bel_write({prefix})")
