"""ctypes bindings of the C-ABI (include/bam_amd.h)."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None
_HOST = None

c_u64, c_u32, c_int, c_vp = ctypes.c_uint64, ctypes.c_uint32, ctypes.c_int, ctypes.c_void_p
P = ctypes.POINTER


class LibraryMissing(RuntimeError):
    pass


# name -> (restype, argtypes); every symbol include/bam_amd.h declares
SIGNATURES = {
    "bam_last_error": (ctypes.c_char_p, []),
    "bam_device_count": (c_int, [P(c_int)]),
    "bam_target_create": (c_int, [P(c_vp), ctypes.c_char_p, c_u64, c_u32, c_int, c_u64, c_u32, c_u32, c_u32, c_u32, c_u32, c_u32]),
    "bam_target_destroy": (None, [c_vp]),
    "bam_target_stats": (c_int, [c_vp, P(c_u64), c_int]),
    "bam_target_backing": (c_vp, [c_vp]),
    "bam_ctrl_create": (c_int, [P(c_vp), ctypes.c_char_p, c_u32, c_u32, c_u64, c_u64, c_u32, c_u32]),
    "bam_ctrl_destroy": (None, [c_vp]),
    "bam_ctrl_info": (c_int, [c_vp, P(c_u64), c_int]),
    "bam_ctrl_queue_state": (c_int, [c_vp, c_u32, P(c_u64), P(c_u32), c_u32]),
    "bam_target_queue_state": (c_int, [c_vp, c_u32, P(c_u64)]),
    "bam_ctrl_aborted": (c_int, [c_vp, c_int]),
    "bam_page_cache_create": (c_int, [P(c_vp), c_u64, c_u64, c_u32, c_vp, c_u64]),
    "bam_page_cache_create_multi": (c_int, [P(c_vp), c_u64, c_u64, c_u32, P(c_vp), c_u32, c_u64]),
    "bam_page_cache_destroy": (None, [c_vp]),
    "bam_page_cache_info": (c_int, [c_vp, P(c_u64)]),
    "bam_page_cache_export_dmabuf": (c_int, [c_vp, P(c_int), P(c_u64)]),
    "bam_page_cache_flush": (c_int, [c_vp]),
    "bam_page_cache_profile": (c_int, [c_vp, P(c_u64), c_int]),
    "bam_range_create": (c_int, [P(c_vp), c_u64, c_u64, c_u64, c_u64, c_u64, c_u64, c_vp, c_u32, c_int]),
    "bam_range_destroy": (None, [c_vp]),
    "bam_array_create": (c_int, [P(c_vp), c_u64, c_u64, P(c_vp), c_u32, c_u32]),
    "bam_array_destroy": (None, [c_vp]),
    "bam_array_stats": (c_int, [c_vp, P(c_u64), c_int]),
    "bam_array_read": (c_int, [c_vp, c_u64, c_vp, c_u64, c_u64, c_u32, c_vp, c_vp]),
    "bam_array_read_shaped": (c_int, [c_vp, c_u64, c_vp, c_int, c_u32, c_u32, c_vp, c_vp]),
    "bam_array_write": (c_int, [c_vp, c_u64, c_vp, c_u64, c_vp, c_u32, c_vp]),
    "bam_array_update": (c_int, [c_vp, c_int, c_u64, c_vp, c_vp, c_vp, c_u32, c_vp]),
    "bam_sqe_image": (c_int, [ctypes.c_uint16, ctypes.c_uint8, c_u32, c_u64, c_u64, c_u64, ctypes.c_uint16, c_int, c_u32, P(c_u32), c_vp, c_vp]),
    "bam_cache_stream": (c_int, [c_vp, c_u64, c_u64, c_vp, c_int, c_vp, c_vp]),
    "bam_block_io": (c_int, [c_vp, c_vp, c_u64, c_u32, c_vp, c_int, c_int, c_u32, c_vp]),
    "bam_warp_memcpy": (c_int, [c_vp, c_vp, c_u64, c_u64, c_vp]),
    "bam_unheld_window_cases": (c_int, [c_vp, c_u64, P(c_u32)]),
    "bam_block_checksum": (c_int, [c_vp, c_u64, c_u32, c_vp, c_vp]),
    "bam_bfs": (c_int, [c_vp, c_vp, c_u64, c_u64, c_vp, c_u32, P(c_u32), c_vp]),
    "bam_cc": (c_int, [c_vp, c_vp, c_u64, c_vp, c_u32, P(c_u32), c_vp]),
    "bam_bfs_shaped": (c_int, [c_vp, c_vp, c_u64, c_u64, c_vp, c_int, c_u32, c_u32, P(c_u32), c_vp]),
    "bam_cc_shaped": (c_int, [c_vp, c_vp, c_u64, c_vp, c_int, c_u32, c_u32, P(c_u32), c_vp]),
    "bam_array_set_graph": (c_int, [c_vp, c_vp, c_u64, c_vp]),
    "bam_array_gather": (c_int, [c_vp, c_u64, c_vp, c_u64, c_u32, c_vp, c_vp]),
    "bam_array_read_via": (c_int, [c_vp, c_int, c_u64, c_vp, c_u64, c_u32, c_vp, c_vp]),
    "bam_block_io_async": (c_int, [c_vp, c_vp, c_u64, c_u32, c_u32, c_vp, c_u32, c_vp]),
    "bam_store_write_file": (c_int, [c_vp, c_vp, ctypes.c_char_p, c_u64, c_u64, c_u64, P(c_u64)]),
    "bam_store_read_file": (c_int, [c_vp, c_vp, ctypes.c_char_p, c_u64, c_u64]),
    "bam_bfs_by_page": (c_int, [c_vp, c_vp, c_u64, c_u64, c_vp, P(c_u32), c_vp]),
    "bam_cc_by_page": (c_int, [c_vp, c_vp, c_u64, c_vp, P(c_u32), c_vp]),
    "bam_vectoradd": (c_int, [c_vp, c_vp, c_vp, c_u64, c_vp]),
    "bam_reduce": (c_int, [c_vp, c_u64, c_u32, c_vp, c_vp]),
    "bam_scan": (c_int, [c_vp, c_u64, c_u32, c_vp, c_vp]),
    "bam_scan_noalloc": (c_int, [c_vp, c_u64, c_u32, c_vp, c_vp]),
    "bam_pagerank": (c_int, [c_vp, c_vp, c_u64, ctypes.c_float, ctypes.c_float, c_u32, c_int, c_vp, P(c_u32), c_vp]),
    "bam_range32_create": (c_int, [P(c_vp), c_u64, c_u64, c_u64, c_u64, c_u64, c_u64, c_vp, c_u32, c_int]),
    "bam_range32_destroy": (None, [c_vp]),
    "bam_array32_create": (c_int, [P(c_vp), c_u64, c_u64, P(c_vp), c_u32, c_u32]),
    "bam_array32_destroy": (None, [c_vp]),
    "bam_array32_stats": (c_int, [c_vp, P(c_u64)]),
    "bam_array32_read": (c_int, [c_vp, c_u64, c_vp, c_u64, c_u32, c_vp, c_vp]),
    "bam_sssp": (c_int, [c_vp, c_vp, c_vp, c_u64, c_u64, c_vp, P(c_u32), c_vp]),
    "bam_sssp_float": (c_int, [c_vp, c_vp, c_vp, c_u64, c_u64, c_vp, P(c_u32), c_vp]),
    "bam_bfs_frontier": (c_int, [c_vp, c_vp, c_u64, c_u64, c_vp, P(c_u32), c_vp]),
    "bam_gen_words": (c_int, [c_u64, c_u64, c_u64, c_vp, c_vp]),
    "bam_gen_mod": (c_int, [c_u64, c_u64, c_u64, c_u64, c_u64, c_vp, c_vp]),
    "bam_gen_rmat": (c_int, [c_u64, c_u32, c_u64, c_u64, c_vp, c_vp, c_vp]),
    "bam_gen_uniform": (c_int, [c_u64, c_u64, c_u64, c_u64, c_vp, c_vp, c_vp]),
    "bam_copy_kernel": (c_int, [c_vp, c_vp, c_u64, P(ctypes.c_float), c_vp]),
    "bam_read_kernel": (c_int, [c_vp, c_u64, P(ctypes.c_float), c_vp]),
    "bam_atomic_pairs_kernel": (c_int, [c_vp, c_vp, c_u64, c_int, P(ctypes.c_float), c_vp]),
    "bam_xcd_relay": (c_int, [c_vp, c_u64, c_u32, c_u32, c_u32, c_u32, c_u32, P(c_u64), c_vp]),
    "bam_hit_path_parts": (c_int, [c_vp, c_int, c_int, c_u64, c_u64, c_vp, c_vp]),
    "bam_gather_kernel": (c_int, [c_vp, c_vp, c_u64, P(ctypes.c_float), c_vp]),
    "bam_host_read_ceiling": (c_int, [c_u64, c_u32, P(ctypes.c_float)]),
    "bam_event_create": (c_int, [P(c_vp)]),
    "bam_event_record": (c_int, [c_vp, c_vp]),
    "bam_event_elapsed_ms": (c_int, [c_vp, c_vp, P(ctypes.c_float)]),
    "bam_event_destroy": (None, [c_vp]),
    "bam_target_ceiling_iops": (ctypes.c_double, [c_u64, c_u32, c_int, c_u32, c_u32, c_u32, c_u64, c_u32]),
}


def lib_path():
    """The built library; BAM_AMD_LIB names another build of it (the one with the phase timers, `make prof`)."""
    return os.environ.get("BAM_AMD_LIB") or os.path.join(_HERE, "libbam_amd.so")


def host_lib_path():
    return os.path.join(_HERE, "libbam_host.so")


def load():
    """The full library (device path + C-ABI).  Raises LibraryMissing when it has not been built."""
    global _LIB
    if _LIB is not None:
        return _LIB
    path = lib_path()
    if not os.path.exists(path):
        raise LibraryMissing(f"{path} is not built: run `make -C bam_amd/csrc` (needs hipcc); there is no CPU fallback")
    L = ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)
    for name, (res, args) in SIGNATURES.items():
        f = getattr(L, name)
        f.restype = res
        f.argtypes = args
    _LIB = L
    return L


def load_host():
    """Host-only library (software NVMe target + NVMe host layer); needs no GPU."""
    global _HOST
    if _HOST is None:
        path = host_lib_path()
        if not os.path.exists(path):
            raise LibraryMissing(f"{path} is not built: run `make -C bam_amd/csrc host`")
        _HOST = ctypes.CDLL(path)
    return _HOST
