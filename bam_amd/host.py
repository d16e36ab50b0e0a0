"""Host-side mirror of the reference's host objects over the C-ABI.

Controller / PageCache / Range / Array correspond to Controller
(include/ctrl.h:39-78), page_cache_t (include/page_cache.h:631-887),
range_t<uint64_t> (:964-1030) and array_t<uint64_t> (:1718-1774) of the
reference, with the same constructor arguments in the same order.  Device
buffers are torch tensors on the handle's device; 64-bit unsigned data travels
as int64 tensors (same bits).
"""
import ctypes
import errno
import os

import torch

from . import _lib

c_u64, c_u32, c_vp = ctypes.c_uint64, ctypes.c_uint32, ctypes.c_void_p
MASK64 = (1 << 64) - 1


class BamError(RuntimeError):
    pass


# a target must outlive the controllers attached to it: controllers tear their queues down through it
_TARGETS = {}


def _chk(status, what):
    if status != 0:
        msg = _lib.load().bam_last_error()
        raise BamError(f"{what}: {msg.decode() if msg else 'error'} (status {status})")


def _ptr(t):
    if t is None:
        return None
    if not t.is_cuda or not t.is_contiguous():
        raise BamError("expected a contiguous tensor in device memory")
    return c_vp(t.data_ptr())


def _stream():
    return c_vp(torch.cuda.current_stream().cuda_stream)


class Target:
    """Software NVMe target published under `path` (stands where /dev/libnvmN does in the reference)."""

    def __init__(self, path, ns_bytes, lba_bytes=512, backing=False, seed=42, n_io_threads=4,
                 max_queue_entries=1024, max_io_queues=128, completion_order=0, fail_every=0, drop_every=0):
        self.L = _lib.load()
        self.h = c_vp()
        self.path = path
        _chk(self.L.bam_target_create(ctypes.byref(self.h), path.encode(), ns_bytes, lba_bytes, int(backing), seed,
                                      n_io_threads, max_queue_entries, max_io_queues, completion_order, fail_every, drop_every),
             "bam_target_create")
        _TARGETS[path] = self

    def stats(self, reset=False):
        out = (c_u64 * 12)()
        _chk(self.L.bam_target_stats(self.h, out, int(reset)), "bam_target_stats")
        keys = ("admin_cmds", "io_cmds", "read_cmds", "write_cmds", "bytes_read", "bytes_written", "error_cpls",
                "sq_doorbells", "cq_full_stalls", "dropped", "sqe_retries", "stale_doorbells")
        return dict(zip(keys, list(out)))

    def close(self):
        if self.h:
            _TARGETS.pop(self.path, None)
            self.L.bam_target_destroy(self.h)
            self.h = c_vp()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Controller:
    def __init__(self, path, ns_id=1, device=0, queue_depth=1024, n_queues=128, stage_bytes=4096, spin_limit=10_000_000):
        self.L = _lib.load()
        self.h = c_vp()
        self.device = device
        self._target = _TARGETS.get(path)
        _chk(self.L.bam_ctrl_create(ctypes.byref(self.h), path.encode(), ns_id, device, queue_depth, n_queues, stage_bytes, spin_limit),
             "bam_ctrl_create")

    def info(self, reset=False):
        out = (c_u64 * 6)()
        _chk(self.L.bam_ctrl_info(self.h, out, int(reset)), "bam_ctrl_info")
        keys = ("n_qps", "queue_depth", "blk_size", "ns_blocks", "ssd_accesses", "error_completions")
        return dict(zip(keys, list(out)))

    def aborted(self, clear=False):
        return bool(self.L.bam_ctrl_aborted(self.h, int(clear)))

    def close(self):
        if self.h:
            self.L.bam_ctrl_destroy(self.h)
            self.h = c_vp()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class PageCache:
    def __init__(self, page_size, n_pages, device, ctrl, max_range=64):
        self.L = _lib.load()
        self.h = c_vp()
        self.ctrls = list(ctrl) if isinstance(ctrl, (list, tuple)) else [ctrl]
        self.ctrl = self.ctrls[0]
        self.device = device
        if len(self.ctrls) == 1:
            _chk(self.L.bam_page_cache_create(ctypes.byref(self.h), page_size, n_pages, device, self.ctrl.h, max_range), "bam_page_cache_create")
        else:
            arr = (c_vp * len(self.ctrls))(*[c.h for c in self.ctrls])
            _chk(self.L.bam_page_cache_create_multi(ctypes.byref(self.h), page_size, n_pages, device, arr, len(self.ctrls), max_range),
                 "bam_page_cache_create_multi")

    def info(self):
        out = (c_u64 * 5)()
        _chk(self.L.bam_page_cache_info(self.h, out), "bam_page_cache_info")
        return dict(zip(("n_pages", "page_size", "wave_batch", "staged", "direct_share"), list(out)))

    def flush(self):
        _chk(self.L.bam_page_cache_flush(self.h), "bam_page_cache_flush")

    def export_dmabuf(self):
        """(fd, bytes) of a dma-buf descriptor over the cache's slots, or None where device memory cannot be exported."""
        fd, n = ctypes.c_int(-1), c_u64(0)
        rc = self.L.bam_page_cache_export_dmabuf(self.h, ctypes.byref(fd), ctypes.byref(n))
        if rc == errno.ENOTSUP:
            return None
        _chk(rc, "bam_page_cache_export_dmabuf")
        return fd.value, n.value

    def profile(self, reset=True):
        """Miss-path phase timers (only a library built with -DBAM_PROFILE fills them)."""
        out = (c_u64 * 32)()
        _chk(self.L.bam_page_cache_profile(self.h, out, int(reset)), "bam_page_cache_profile")
        keys = ("batches", "commands", "t_cid", "t_submit", "t_wait", "t_copy", "t_find_slot", "find_slot_calls", "find_slot_lanes",
                "t_sq_ticket", "t_sq_write", "t_sq_cover", "sq_cover_trips", "sq_sweeps", "sq_swept", "sq_doorbells",
                "cq_wait_trips", "cq_drains", "cq_drained", "t_cq_drain", "cq_empty_looks", "t_cq_notice",
                "n_ld_dev", "t_ld_dev", "n_sqe_store", "t_sqe_store", "t_doorbell", "n_ld_cqe", "t_ld_cqe", "t_pull", "n_pull")
        return dict(zip(keys, list(out)))

    def block_io(self, n_reqs, req_bytes, lbas=None, write=False, queue_policy=1, block_size=64):
        """One thread per NVMe command into cache slot tid (benchmarks/block/main.cu:99-200)."""
        _chk(self.L.bam_block_io(self.ctrl.h, self.h, n_reqs, req_bytes, _ptr(lbas), int(write), queue_policy, block_size, _stream()),
             "bam_block_io")

    def block_io_async(self, n_threads, depth, req_bytes, lbas, block_size=64):
        """`depth` commands in flight per thread (benchmarks/iodepth-block/main.cu:97-140)."""
        _chk(self.L.bam_block_io_async(self.ctrl.h, self.h, n_threads, depth, req_bytes, _ptr(lbas), block_size, _stream()), "bam_block_io_async")

    def write_file(self, path, file_offset=0, store_offset=0, n_bytes=0):
        """file -> store through the cache slots (benchmarks/readwrite, write mode); returns the bytes written."""
        done = c_u64(0)
        _chk(self.L.bam_store_write_file(self.ctrl.h, self.h, os.fsencode(path), file_offset, store_offset, n_bytes, ctypes.byref(done)),
             "bam_store_write_file")
        return done.value

    def read_file(self, path, store_offset, n_bytes):
        """store -> a new file (benchmarks/readwrite, read mode)"""
        _chk(self.L.bam_store_read_file(self.ctrl.h, self.h, os.fsencode(path), store_offset, n_bytes), "bam_store_read_file")

    def block_checksums(self, n_slots, req_bytes):
        out = torch.empty(n_slots, dtype=torch.int64, device=f"cuda:{self.device}")
        _chk(self.L.bam_block_checksum(self.h, n_slots, req_bytes, _ptr(out), _stream()), "bam_block_checksum")
        return out

    def close(self):
        if self.h:
            self.L.bam_page_cache_destroy(self.h)
            self.h = c_vp()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Range:
    REPLICATE, STRIPE = 0, 1

    def __init__(self, index_start, count, page_start, page_count, page_start_offset, page_size, cache, device, dist=0):
        self.L = _lib.load()
        self.h = c_vp()
        self.cache = cache
        _chk(self.L.bam_range_create(ctypes.byref(self.h), index_start, count, page_start, page_count, page_start_offset,
                                     page_size, cache.h, device, dist), "bam_range_create")

    def close(self):
        if self.h:
            self.L.bam_range_destroy(self.h)
            self.h = c_vp()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Array:
    def __init__(self, n_elems, disk_start_offset, ranges, device):
        self.L = _lib.load()
        self.h = c_vp()
        self.ranges = list(ranges)
        self.device = device
        arr = (c_vp * len(ranges))(*[r.h for r in ranges])
        _chk(self.L.bam_array_create(ctypes.byref(self.h), n_elems, disk_start_offset, arr, len(ranges), device), "bam_array_create")

    def _sum_buf(self):
        return torch.zeros(1, dtype=torch.int64, device=f"cuda:{self.device}")

    def read_async(self, n_reqs, d_sum, assignment=None, stride=1, reqs_per_thread=1, block_size=64):
        _chk(self.L.bam_array_read(self.h, n_reqs, _ptr(assignment), stride, reqs_per_thread, block_size, _ptr(d_sum), _stream()),
             "bam_array_read")

    def read(self, n_reqs, assignment=None, stride=1, reqs_per_thread=1, block_size=64):
        """Sum (mod 2^64) of the elements read: thread t reads assignment[t] (or t * stride)."""
        s = self._sum_buf()
        self.read_async(n_reqs, s, assignment, stride, reqs_per_thread, block_size)
        return int(s.item()) & MASK64

    ONE_PER_THREAD, FOUR_PER_THREAD, TWO_LAUNCHES = 1, 2, 3

    def read_shaped_async(self, n_reqs, d_sum, assignment, shape, reads_per_lane=4, block_size=64):
        _chk(self.L.bam_array_read_shaped(self.h, n_reqs, _ptr(assignment), shape, reads_per_lane, block_size, _ptr(d_sum), _stream()),
             "bam_array_read_shaped")

    def read_shaped(self, n_reqs, assignment, shape, reads_per_lane=4, block_size=64):
        """The scattered reads of read() with the launch shape named: ONE_PER_THREAD (the reference's kernel as it is),
        FOUR_PER_THREAD, or TWO_LAUNCHES with 1, 2, 4 or 8 reads per lane in the first."""
        s = self._sum_buf()
        self.read_shaped_async(n_reqs, s, assignment, shape, reads_per_lane, block_size)
        return int(s.item()) & MASK64

    def set_graph(self, offsets=None):
        """Prepare (or with None drop) what the graph entry points need for the CSR whose neighbour ids this array holds;
        later calls with the same offsets tensor allocate nothing."""
        _chk(self.L.bam_array_set_graph(self.h, _ptr(offsets), (offsets.numel() - 1) if offsets is not None else 0, _stream()), "bam_array_set_graph")
        self._graph_offsets = offsets               # keeps the tensor alive while the plan names its address

    def gather(self, n_reqs, assignment=None, stride=1, block_size=64):
        """The elements themselves: out[t] = element assignment[t] (or t * stride), an int64 tensor of bit patterns."""
        out = torch.empty(n_reqs, dtype=torch.int64, device=f"cuda:{self.device}")
        _chk(self.L.bam_array_gather(self.h, n_reqs, _ptr(assignment), stride, block_size, _ptr(out), _stream()), "bam_array_gather")
        return out

    def xcd_relay(self, seed, page_bytes, n_pages, rounds, n_waves=64, spin_limit=0):
        """Pages loaded by a wave on one compute-unit cluster and read by waves on the others (bam_xcd_relay)."""
        out = (c_u64 * 4)()
        _chk(self.L.bam_xcd_relay(self.h, seed, page_bytes, n_pages, rounds, n_waves, spin_limit, out, _stream()), "bam_xcd_relay")
        return dict(zip(("mismatches", "waits_given_up", "cluster_mask", "reads_checked"), list(out)))

    def read_via(self, api, n_reqs, assignment=None, span=1, block_size=64):
        """The read pattern through another access route of array_d_t (1 get_raw, 2 acquire_page_, 3 acquire_page,
        4 bam_ptr, 5 wave memcpy of up to `span` elements per request); sum of what was read."""
        s = self._sum_buf()
        _chk(self.L.bam_array_read_via(self.h, api, n_reqs, _ptr(assignment), span, block_size, _ptr(s), _stream()), "bam_array_read_via")
        return int(s.item()) & MASK64

    def write(self, n_reqs, values, assignment=None, stride=1, block_size=64):
        _chk(self.L.bam_array_write(self.h, n_reqs, _ptr(assignment), stride, _ptr(values), block_size, _stream()), "bam_array_write")

    def unheld_window_cases(self, page):
        """bam_unheld_window_cases: what the second look of the pointer that holds no reference says, case by case."""
        out = (c_u32 * 7)()
        _chk(self.L.bam_unheld_window_cases(self.h, page, out), "bam_unheld_window_cases")
        return list(out)

    def stream_async(self, n_waves, n_pages_per_wave, d_sum, assignment=None, mode=2):
        _chk(self.L.bam_cache_stream(self.h, n_waves, n_pages_per_wave, _ptr(assignment), mode, _ptr(d_sum), _stream()), "bam_cache_stream")

    def stream(self, n_waves, n_pages_per_wave, assignment=None, mode=2):
        s = self._sum_buf()
        self.stream_async(n_waves, n_pages_per_wave, s, assignment, mode)
        return int(s.item()) & MASK64

    def bfs(self, offsets, src, coarse=1, by_page=False, frontier=False):
        """Levels (uint32 bit patterns in an int32 tensor) and launch count; by_page: the edge-page kernel; frontier: the
        kernel that walks a queue of the level's vertices."""
        n_v = offsets.numel() - 1
        labels = torch.empty(n_v, dtype=torch.int32, device=offsets.device)
        it = c_u32(0)
        if frontier:
            _chk(self.L.bam_bfs_frontier(self.h, _ptr(offsets), n_v, int(src), _ptr(labels), ctypes.byref(it), _stream()), "bam_bfs_frontier")
        elif by_page:
            _chk(self.L.bam_bfs_by_page(self.h, _ptr(offsets), n_v, int(src), _ptr(labels), ctypes.byref(it), _stream()), "bam_bfs_by_page")
        else:
            _chk(self.L.bam_bfs(self.h, _ptr(offsets), n_v, int(src), _ptr(labels), coarse, ctypes.byref(it), _stream()), "bam_bfs")
        return labels, it.value

    def bfs_shaped(self, offsets, src, shape, coarse=1, stride=1):
        """BFS with the vertices shared out as the reference's hash (0), hash + coarse (1), sixteen lanes per vertex (2) or
        chunk (3) kernels do; levels and launch count."""
        n_v = offsets.numel() - 1
        labels = torch.empty(n_v, dtype=torch.int32, device=offsets.device)
        it = c_u32(0)
        _chk(self.L.bam_bfs_shaped(self.h, _ptr(offsets), n_v, int(src), _ptr(labels), shape, coarse, stride, ctypes.byref(it), _stream()), "bam_bfs_shaped")
        return labels, it.value

    def cc_shaped(self, offsets, shape, coarse=1, stride=1):
        n_v = offsets.numel() - 1
        labels = torch.empty(n_v, dtype=torch.int64, device=offsets.device)
        it = c_u32(0)
        _chk(self.L.bam_cc_shaped(self.h, _ptr(offsets), n_v, _ptr(labels), shape, coarse, stride, ctypes.byref(it), _stream()), "bam_cc_shaped")
        return labels, it.value

    def cc(self, offsets, coarse=1, by_page=False):
        n_v = offsets.numel() - 1
        labels = torch.empty(n_v, dtype=torch.int64, device=offsets.device)
        it = c_u32(0)
        if by_page:
            _chk(self.L.bam_cc_by_page(self.h, _ptr(offsets), n_v, _ptr(labels), ctypes.byref(it), _stream()), "bam_cc_by_page")
        else:
            _chk(self.L.bam_cc(self.h, _ptr(offsets), n_v, _ptr(labels), coarse, ctypes.byref(it), _stream()), "bam_cc")
        return labels, it.value

    def reduce(self, n_elems, block_size=64):
        """Per-workgroup sums of 2 * block_size consecutive elements (benchmarks/reduction); int64 tensor of bit patterns."""
        n_blocks = (n_elems + 2 * block_size - 1) // (2 * block_size)
        out = torch.zeros(n_blocks, dtype=torch.int64, device=f"cuda:{self.device}")
        _chk(self.L.bam_reduce(self.h, n_elems, block_size, _ptr(out), _stream()), "bam_reduce")
        return out

    def scan(self, n_elems, block_size=64):
        """n_elems + 1 running sums, the first 0 and the last the total (benchmarks/scan); int64 tensor of bit patterns."""
        out = torch.empty(n_elems + 1, dtype=torch.int64, device=f"cuda:{self.device}")
        _chk(self.L.bam_scan(self.h, n_elems, block_size, _ptr(out), _stream()), "bam_scan")
        return out

    def scan_noalloc(self, n_elems, out, block_size=64):
        """bam_scan into `out` (n_elems + 1 words) without any allocation by the library; does not synchronise."""
        _chk(self.L.bam_scan_noalloc(self.h, n_elems, block_size, _ptr(out), _stream()), "bam_scan_noalloc")

    def update(self, api, assignment, values, block_size=64):
        """element assignment[t] += values[t] through AtomicAdd (api 0), an atomic on bam_ptr::memref (1) or ptr[i] += v (2);
        returns what each element held before (int64 tensor of bit patterns)."""
        n = assignment.numel()
        old = torch.zeros(n, dtype=torch.int64, device=f"cuda:{self.device}")
        _chk(self.L.bam_array_update(self.h, api, n, _ptr(assignment), _ptr(values), _ptr(old), block_size, _stream()), "bam_array_update")
        return old

    def pagerank(self, offsets, alpha=0.85, tolerance=0.001, max_iterations=100, by_page=False):
        """PageRank values (float32) by residual pushes over the CSR whose neighbour ids this array holds, and the sweeps taken."""
        n_v = offsets.numel() - 1
        value = torch.empty(n_v, dtype=torch.float32, device=offsets.device)
        it = c_u32(0)
        _chk(self.L.bam_pagerank(self.h, _ptr(offsets), n_v, alpha, tolerance, max_iterations, int(by_page), _ptr(value),
                                 ctypes.byref(it), _stream()), "bam_pagerank")
        return value, it.value

    def stats(self, reset=True):
        out = (c_u64 * 4)()
        _chk(self.L.bam_array_stats(self.h, out, int(reset)), "bam_array_stats")
        return dict(zip(("read_io_cnt", "access_cnt", "miss_cnt", "hit_cnt"), list(out)))

    def close(self):
        if self.h:
            self.L.bam_array_destroy(self.h)
            self.h = c_vp()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Range32:
    """range_t<uint32_t>: same arguments as Range"""

    def __init__(self, index_start, count, page_start, page_count, page_start_offset, page_size, cache, device, dist=0):
        self.L = _lib.load()
        self.h = c_vp()
        self.cache = cache
        _chk(self.L.bam_range32_create(ctypes.byref(self.h), index_start, count, page_start, page_count, page_start_offset,
                                       page_size, cache.h, device, dist), "bam_range32_create")

    def close(self):
        if self.h:
            self.L.bam_range32_destroy(self.h)
            self.h = c_vp()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Array32:
    """array_t<uint32_t>"""

    def __init__(self, n_elems, disk_start_offset, ranges, device):
        self.L = _lib.load()
        self.h = c_vp()
        self.ranges = list(ranges)
        self.device = device
        arr = (c_vp * len(ranges))(*[r.h for r in ranges])
        _chk(self.L.bam_array32_create(ctypes.byref(self.h), n_elems, disk_start_offset, arr, len(ranges), device), "bam_array32_create")

    def read(self, n_reqs, assignment=None, stride=1, block_size=64):
        s = torch.zeros(1, dtype=torch.int64, device=f"cuda:{self.device}")
        _chk(self.L.bam_array32_read(self.h, n_reqs, _ptr(assignment), stride, block_size, _ptr(s), _stream()), "bam_array32_read")
        return int(s.item()) & MASK64

    def stats(self):
        out = (c_u64 * 4)()
        _chk(self.L.bam_array32_stats(self.h, out), "bam_array32_stats")
        return dict(zip(("read_io_cnt", "access_cnt", "miss_cnt", "hit_cnt"), list(out)))

    def close(self):
        if self.h:
            self.L.bam_array32_destroy(self.h)
            self.h = c_vp()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def vectoradd(a, b, c, n_elems):
    """c[i] = a[i] + b[i] through the cache (benchmarks/vectoradd)"""
    _chk(a.L.bam_vectoradd(a.h, b.h, c.h, n_elems, _stream()), "bam_vectoradd")


def sssp(edges, weights, offsets, src):
    """Costs (uint32 bit patterns in an int32 tensor) of the cheapest paths from src, and the number of rounds."""
    n_v = offsets.numel() - 1
    costs = torch.empty(n_v, dtype=torch.int32, device=offsets.device)
    it = c_u32(0)
    _chk(edges.L.bam_sssp(edges.h, weights.h, _ptr(offsets), n_v, int(src), _ptr(costs), ctypes.byref(it), _stream()), "bam_sssp")
    return costs, it.value


def sssp_float(edges, weights, offsets, src):
    """The same with single-precision weights (their bit patterns in the 32-bit array): float32 costs, 1e9 = unreached."""
    n_v = offsets.numel() - 1
    costs = torch.empty(n_v, dtype=torch.float32, device=offsets.device)
    it = c_u32(0)
    _chk(edges.L.bam_sssp_float(edges.h, weights.h, _ptr(offsets), n_v, int(src), _ptr(costs), ctypes.byref(it), _stream()), "bam_sssp_float")
    return costs, it.value


def make_array(ctrl, n_elems, page_size, cache_pages, device=0, disk_offset_bytes=0, max_range=64):
    """page cache + one range + array over n_elems u64 stored from byte disk_offset_bytes (page aligned)."""
    pc = PageCache(page_size, cache_pages, device, ctrl, max_range)
    n_pages = (n_elems * 8 + page_size - 1) // page_size
    r = Range(0, n_elems, disk_offset_bytes // page_size, n_pages, 0, page_size, pc, device)
    a = Array(n_elems, disk_offset_bytes, [r], device)
    return pc, r, a
