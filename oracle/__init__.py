"""CPU oracle for the storage-access path.  TEST INFRASTRUCTURE ONLY.

Only tests/, the smoke check and the benchmark's CPU-baseline leg may import
this package; the shipped library never does.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

u64 = ctypes.c_uint64
u32 = ctypes.c_uint32
_p64 = np.ctypeslib.ndpointer(dtype=np.uint64, flags="C_CONTIGUOUS")
_p32 = np.ctypeslib.ndpointer(dtype=np.uint32, flags="C_CONTIGUOUS")
_pf32 = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_pf64 = np.ctypeslib.ndpointer(dtype=np.float64, flags="C_CONTIGUOUS")


def build(force=False):
    """Compile the C oracle in place (gcc, seconds)."""
    so = os.path.join(_HERE, "libbam_oracle.so")
    if force and os.path.exists(so):
        os.remove(so)
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    return so


def lib():
    global _LIB
    if _LIB is not None:
        return _LIB
    so = os.path.join(_HERE, "libbam_oracle.so")
    if not os.path.exists(so):
        build()
    L = ctypes.CDLL(so)
    sig = {
        "bo_splitmix64": (u64, [u64, u64]),
        "bo_fill_store": (None, [u64, u64, u64, _p64]),
        "bo_store_sum": (u64, [u64, u64, u64, u64]),
        "bo_gather_indices": (None, [u64, u64, u64, u64, _p64]),
        "bo_gather_sum": (u64, [u64, u64, u64, u64, u64]),
        "bo_block_lbas": (None, [u64, u64, u64, u64, u32, u32, _p64]),
        "bo_block_checksum": (u64, [u64, u64, u32, u32]),
        "bo_rmat_edges": (None, [u64, u32, u64, u64, _p64, _p64]),
        "bo_uniform_edges": (None, [u64, u64, u64, u64, _p64, _p64]),
        "bo_build_csr": (u64, [u64, u64, _p64, _p64, _p64, _p64]),
        "bo_bfs_sources": (None, [u64, u64, _p64, u32, _p64]),
        "bo_bfs_levels": (u32, [u64, _p64, _p64, u64, _p32]),
        "bo_bfs_levels_sweep": (u32, [u64, _p64, _p64, u64, _p32]),
        "bo_cc_labels": (u64, [u64, _p64, _p64, _p64]),
        "bo_cc_labels_sweep": (u64, [u64, _p64, _p64, _p64, ctypes.POINTER(u32)]),
        "bo_bfs_edges_scanned": (u64, [u64, _p64, _p32]),
        "bo_edge_weights": (None, [u64, u64, u64, _p32]),
        "bo_sssp_costs": (None, [u64, _p64, _p64, _p32, u64, _p32]),
        "bo_sssp_costs_sweep": (u32, [u64, _p64, _p64, _p32, u64, _p32]),
        "bo_sssp_costs_float": (None, [u64, _p64, _p64, _pf32, u64, _pf32]),
        "bo_sssp_costs_float_sweep": (u32, [u64, _p64, _p64, _pf32, u64, _pf32]),
        "bo_reduce_blocks": (None, [_p64, u64, u32, _p64]),
        "bo_scan": (None, [_p64, u64, _p64]),
        "bo_pagerank": (u32, [u64, _p64, _p64, ctypes.c_float, ctypes.c_float, u32, _pf32]),
        "bo_pagerank_limit": (None, [u64, _p64, _p64, ctypes.c_double, u32, _pf64]),
        "bo_cmd_rw": (None, [_p32, ctypes.c_uint16, ctypes.c_uint8, u32, u64, u64, u64, ctypes.c_uint16]),
    }
    for name, (res, args) in sig.items():
        f = getattr(L, name)
        f.restype = res
        f.argtypes = args
    _LIB = L
    return L


# ---- convenience wrappers -------------------------------------------------

def store(seed, first, n):
    out = np.empty(n, dtype=np.uint64)
    lib().bo_fill_store(seed, first, n, out)
    return out


def gather_indices(seed, first_k, n, n_elems):
    out = np.empty(n, dtype=np.uint64)
    lib().bo_gather_indices(seed, first_k, n, n_elems, out)
    return out


def block_lbas(seed, first_k, n, ns_bytes, req_bytes, lba_bytes):
    out = np.empty(n, dtype=np.uint64)
    lib().bo_block_lbas(seed, first_k, n, ns_bytes, req_bytes, lba_bytes, out)
    return out


def rmat_csr(seed, scale, edge_factor=16):
    n_v, n_p = 1 << scale, edge_factor << scale
    u = np.empty(n_p, dtype=np.uint64)
    v = np.empty(n_p, dtype=np.uint64)
    lib().bo_rmat_edges(seed, scale, 0, n_p, u, v)
    return _csr(n_v, u, v)


def uniform_csr(seed, n_vertices, n_pairs):
    u = np.empty(n_pairs, dtype=np.uint64)
    v = np.empty(n_pairs, dtype=np.uint64)
    lib().bo_uniform_edges(seed, n_vertices, 0, n_pairs, u, v)
    return _csr(n_vertices, u, v)


def _csr(n_v, u, v):
    off = np.empty(n_v + 1, dtype=np.uint64)
    nb = np.empty(max(2 * len(u), 1), dtype=np.uint64)
    e = lib().bo_build_csr(n_v, len(u), u, v, off, nb)
    return off, nb[:e].copy()


def csr_from_pairs(n_vertices, u, v):
    """symmetrized, sorted, deduplicated CSR of the pairs (u[k], v[k]), self loops dropped"""
    return _csr(n_vertices, np.ascontiguousarray(u, dtype=np.uint64), np.ascontiguousarray(v, dtype=np.uint64))


def bfs_sources(seed, offsets, n_src=8):
    out = np.empty(n_src, dtype=np.uint64)
    lib().bo_bfs_sources(seed, len(offsets) - 1, offsets, n_src, out)
    return out


def bfs_levels(offsets, neigh, src, sweep=False):
    lv = np.empty(len(offsets) - 1, dtype=np.uint32)
    nb = neigh if len(neigh) else np.zeros(1, dtype=np.uint64)
    f = lib().bo_bfs_levels_sweep if sweep else lib().bo_bfs_levels
    iters = f(len(offsets) - 1, offsets, nb, int(src), lv)
    return lv, iters


def cc_labels(offsets, neigh, sweep=False):
    lb = np.empty(len(offsets) - 1, dtype=np.uint64)
    nb = neigh if len(neigh) else np.zeros(1, dtype=np.uint64)
    if sweep:
        it = u32(0)
        comps = lib().bo_cc_labels_sweep(len(offsets) - 1, offsets, nb, lb, ctypes.byref(it))
        return lb, comps, it.value
    comps = lib().bo_cc_labels(len(offsets) - 1, offsets, nb, lb)
    return lb, comps


def edge_weights(seed, n, first=0):
    out = np.empty(max(n, 1), dtype=np.uint32)
    lib().bo_edge_weights(seed, first, n, out)
    return out[:n]


def sssp_costs(offsets, neigh, weights, src, sweep=False):
    costs = np.empty(len(offsets) - 1, dtype=np.uint32)
    nb = neigh if len(neigh) else np.zeros(1, dtype=np.uint64)
    w = weights if len(weights) else np.zeros(1, dtype=np.uint32)
    if sweep:
        rounds = lib().bo_sssp_costs_sweep(len(offsets) - 1, offsets, nb, w, int(src), costs)
        return costs, rounds
    lib().bo_sssp_costs(len(offsets) - 1, offsets, nb, w, int(src), costs)
    return costs


def sssp_costs_float(offsets, neigh, weights, src, sweep=False):
    """single-precision costs (unreached = 1e9) for float32 weights >= 0"""
    costs = np.empty(len(offsets) - 1, dtype=np.float32)
    nb = neigh if len(neigh) else np.zeros(1, dtype=np.uint64)
    w = np.ascontiguousarray(weights, dtype=np.float32) if len(weights) else np.zeros(1, dtype=np.float32)
    if sweep:
        rounds = lib().bo_sssp_costs_float_sweep(len(offsets) - 1, offsets, nb, w, int(src), costs)
        return costs, rounds
    lib().bo_sssp_costs_float(len(offsets) - 1, offsets, nb, w, int(src), costs)
    return costs


def reduce_blocks(a, block):
    a = np.ascontiguousarray(a, dtype=np.uint64)
    per = 2 * block
    out = np.empty(max((len(a) + per - 1) // per, 1), dtype=np.uint64)
    lib().bo_reduce_blocks(a if len(a) else np.zeros(1, dtype=np.uint64), len(a), block, out)
    return out[:(len(a) + per - 1) // per]


def scan(a):
    a = np.ascontiguousarray(a, dtype=np.uint64)
    out = np.empty(len(a) + 1, dtype=np.uint64)
    lib().bo_scan(a if len(a) else np.zeros(1, dtype=np.uint64), len(a), out)
    return out


def pagerank(offsets, neigh, alpha=0.85, tolerance=0.001, max_iterations=100):
    value = np.empty(len(offsets) - 1, dtype=np.float32)
    nb = neigh if len(neigh) else np.zeros(1, dtype=np.uint64)
    it = lib().bo_pagerank(len(offsets) - 1, offsets, nb, alpha, tolerance, max_iterations, value)
    return value, it


def pagerank_limit(offsets, neigh, alpha=0.85, sweeps=300):
    x = np.empty(len(offsets) - 1, dtype=np.float64)
    nb = neigh if len(neigh) else np.zeros(1, dtype=np.uint64)
    lib().bo_pagerank_limit(len(offsets) - 1, offsets, nb, alpha, sweeps, x)
    return x


# ---- CPU restatement of the page-cache + queue protocol (cpu_path.c) -------
_CPU = None


def cpu_lib():
    global _CPU
    if _CPU is not None:
        return _CPU
    so = os.path.join(_HERE, "libbam_cpu_path.so")
    if not os.path.exists(so):
        build()
    L = ctypes.CDLL(so)
    vp = ctypes.c_void_p
    L.bo_cpu_path_create.restype = vp
    L.bo_cpu_path_create.argtypes = [u64, u32, u64, vp, u32, u32, u32, u64, u64, u64, u64]
    L.bo_cpu_path_destroy.argtypes = [vp]
    L.bo_cpu_path_stats.argtypes = [vp, ctypes.POINTER(u64), ctypes.c_int]
    L.bo_cpu_path_check.restype = ctypes.c_int
    L.bo_cpu_path_check.argtypes = [vp]
    L.bo_cpu_array_sum.restype = u64
    L.bo_cpu_array_sum.argtypes = [vp, u32, u64, vp, u64]
    L.bo_cpu_block_reads.restype = u64
    L.bo_cpu_block_reads.argtypes = [vp, u32, u64, _p64, u32, vp]
    L.bo_cpu_bfs.restype = u32
    L.bo_cpu_bfs.argtypes = [vp, u32, _p64, u64, u64, _p32]
    L.bo_cpu_cc.restype = u32
    L.bo_cpu_cc.argtypes = [vp, u32, _p64, u64, _p64]
    _CPU = L
    return L


class CpuPath:
    """The reference's path restated on CPU threads, over the software NVMe target.

    backing: None for a procedural namespace (word w = splitmix64(seed, w)), or a
    C-contiguous numpy array that is the namespace content (kept alive here).
    """

    def __init__(self, ns_bytes, n_elems, page_size=4096, cache_pages=1024, lba_bytes=512, seed=42, backing=None,
                 n_io_threads=2, n_queues=4, queue_depth=64, disk_offset_bytes=0):
        self.L = cpu_lib()
        self._backing = backing
        bp = backing.ctypes.data if backing is not None else None
        self.h = self.L.bo_cpu_path_create(ns_bytes, lba_bytes, seed, bp, n_io_threads, n_queues, queue_depth,
                                           page_size, cache_pages, n_elems, disk_offset_bytes)
        if not self.h:
            raise RuntimeError("bo_cpu_path_create failed")

    def array_sum(self, n_reqs, idx=None, stride=1, n_threads=4):
        p = idx.ctypes.data if idx is not None else None
        return self.L.bo_cpu_array_sum(self.h, n_threads, n_reqs, p, stride)

    def block_reads(self, lbas, req_bytes, n_threads=4):
        cs = np.empty(len(lbas), dtype=np.uint64)
        self.L.bo_cpu_block_reads(self.h, n_threads, len(lbas), lbas, req_bytes, cs.ctypes.data)
        return cs

    def bfs(self, offsets, src, n_threads=4):
        lv = np.empty(len(offsets), dtype=np.uint32)      # one spare slot: the current level is parked there
        it = self.L.bo_cpu_bfs(self.h, n_threads, offsets, len(offsets) - 1, int(src), lv)
        return lv[:-1].copy(), it

    def cc(self, offsets, n_threads=4):
        lb = np.empty(len(offsets) - 1, dtype=np.uint64)
        it = self.L.bo_cpu_cc(self.h, n_threads, offsets, len(offsets) - 1, lb)
        return lb, it

    def stats(self, reset=True):
        out = (u64 * 4)()
        self.L.bo_cpu_path_stats(self.h, out, int(reset))
        return dict(zip(("read_io_cnt", "access_cnt", "miss_cnt", "hit_cnt"), list(out)))

    def check(self):
        """0 when the quiescent-state invariants hold."""
        return self.L.bo_cpu_path_check(self.h)

    def close(self):
        if self.h:
            self.L.bo_cpu_path_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
