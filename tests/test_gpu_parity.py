"""GPU parity: the gfx950 path, called through the C-ABI, against the CPU oracle.  Bit-exact everywhere (integer work)."""
import ctypes
import json
import os

import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu

G = os.path.join(os.path.dirname(__file__), "golden")
SEED = 42
LIMIT_US = 20_000_000      # bound of every device-side wait in these tests


@pytest.fixture(scope="module")
def bam():
    import torch
    import bam_amd
    if not torch.cuda.is_available():
        pytest.fail("gpu tests need a GPU")
    bam_amd.load()          # raises when the HIP library is missing: there is no fallback
    return bam_amd


_n = [0]


def _path():
    _n[0] += 1
    return "/dev/libnvm-t%d" % _n[0]


class Rig:
    """target + controller (+ array) with teardown in the right order"""

    def __init__(self, bam, ns_bytes, lba=512, backing=False, seed=SEED, n_queues=8, depth=256, io_threads=4, order=0,
                 fail_every=0, drop_every=0, stage_bytes=4096, limit=LIMIT_US):
        self.bam = bam
        self.path = _path()
        self.t = bam.Target(self.path, ns_bytes, lba, backing=backing, seed=seed, n_io_threads=io_threads,
                            completion_order=order, fail_every=fail_every, drop_every=drop_every)
        self.c = bam.Controller(self.path, 1, 0, queue_depth=depth, n_queues=n_queues, stage_bytes=stage_bytes, spin_limit=limit)
        self.objs = []

    def array(self, n_elems, page_size, cache_pages, disk_offset=0):
        from bam_amd.host import make_array
        pc, r, a = make_array(self.c, n_elems, page_size, cache_pages, 0, disk_offset)
        self.objs.append((a, r, pc))
        return a

    def backing(self, n_words):
        p = self.t.L.bam_target_backing(self.t.h)
        return np.ctypeslib.as_array(ctypes.cast(p, ctypes.POINTER(ctypes.c_uint64)), shape=(n_words,))

    def close(self):
        for a, r, pc in self.objs:
            a.close(); r.close(); pc.close()
        self.c.close(); self.t.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def _dev(x):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x).view(np.int64)).cuda()


def _u64(t):
    return t.cpu().numpy().view(np.uint64)


# ---------------------------------------------------------------- generators

def test_device_generators_match_oracle(bam):
    from bam_amd import gen
    assert np.array_equal(_u64(gen.words(SEED, 1000, 5000)), oracle.store(SEED, 1000, 5000))
    assert np.array_equal(_u64(gen.gather_indices(SEED, 4096, 1 << 20, first=7)), oracle.gather_indices(SEED, 7, 4096, 1 << 20))
    assert np.array_equal(_u64(gen.block_lbas(SEED, 1000, 64 << 30, 4096, 512)), oracle.block_lbas(SEED, 0, 1000, 64 << 30, 4096, 512))
    for scale in (6, 12):
        u, v = gen.rmat_pairs(SEED, scale, 0, 16 << scale)
        ru = np.empty(16 << scale, dtype=np.uint64); rv = np.empty(16 << scale, dtype=np.uint64)
        oracle.lib().bo_rmat_edges(SEED, scale, 0, 16 << scale, ru, rv)
        assert np.array_equal(_u64(u), ru) and np.array_equal(_u64(v), rv)
        off, nb = gen.rmat_csr(SEED, scale)
        roff, rnb = oracle.rmat_csr(SEED, scale)
        assert np.array_equal(_u64(off), roff) and np.array_equal(_u64(nb), rnb)
    off, nb = gen.uniform_csr(SEED, 5000, 9000)
    roff, rnb = oracle.uniform_csr(SEED, 5000, 9000)
    assert np.array_equal(_u64(off), roff) and np.array_equal(_u64(nb), rnb)


# ---------------------------------------------------------------- array

def test_config1_reduction_on_gpu(bam):
    """2^24 u64, 128 MiB store, 4 KiB pages, 64 MiB cache, stride-8 reads: the reference's plumbing case"""
    with open(os.path.join(G, "splitmix64.json")) as f:
        g = json.load(f)
    for seed in (0, 42):
        with Rig(bam, 128 << 20, seed=seed, n_queues=32, depth=1024) as r:
            a = r.array(1 << 24, 4096, 16384)
            s = a.read(1 << 21, stride=8, block_size=64)
            st = a.stats()
            assert s == int(g["cfg1_stride8_sum_2p21"][str(seed)], 16)
            assert st["access_cnt"] == 1 << 21 and st["hit_cnt"] + st["miss_cnt"] == 1 << 21
            assert 32768 <= st["read_io_cnt"] < 32768 + 8192
            assert not r.c.aborted() and r.c.info()["error_completions"] == 0
            assert r.t.stats()["read_cmds"] == st["read_io_cnt"]


def test_counter_invariants_without_eviction(bam):
    """read I/Os = distinct pages first touched; accesses = lane accesses; second pass all hits (reference logs)"""
    n = 1 << 20
    with Rig(bam, 16 << 20) as r:
        a = r.array(n, 4096, 4096)
        assert a.read(n, block_size=64) == oracle.lib().bo_store_sum(SEED, 0, 1, n)
        st = a.stats()
        assert st["read_io_cnt"] == n // 512 and st["access_cnt"] == n and st["hit_cnt"] + st["miss_cnt"] == n
        assert a.read(n, block_size=256) == oracle.lib().bo_store_sum(SEED, 0, 1, n)
        st = a.stats()
        assert st == {"read_io_cnt": 0, "access_cnt": n, "miss_cnt": 0, "hit_cnt": n}
        assert r.c.info(reset=True)["ssd_accesses"] == n // 512


@pytest.mark.parametrize("cache_pages,n_queues,depth,block", [(64, 4, 64, 64), (1024, 2, 16, 256), (4096, 16, 1024, 128)])
def test_random_gather_with_eviction(bam, cache_pages, n_queues, depth, block):
    from bam_amd import gen
    n_elems, n = 1 << 22, 1 << 18          # 8192 pages of data
    with Rig(bam, 64 << 20, n_queues=n_queues, depth=depth) as r:
        a = r.array(n_elems, 4096, cache_pages)
        idx = gen.gather_indices(SEED, n, n_elems)
        for _ in range(2):
            assert a.read(n, idx, block_size=block) == oracle.lib().bo_gather_sum(SEED, SEED, 0, n, n_elems)
            st = a.stats()
            assert st["access_cnt"] == n and st["hit_cnt"] + st["miss_cnt"] == n and st["read_io_cnt"] > 0
        assert a.read(n // 2, idx, reqs_per_thread=2, block_size=block) == (2 * oracle.lib().bo_gather_sum(SEED, SEED, 0, n // 2, n_elems)) % 2**64
        assert not r.c.aborted()


@pytest.mark.parametrize("cache_pages,n_queues,depth", [(8, 4, 64), (300, 8, 256), (8192, 16, 1024)])
def test_launch_shapes_of_the_gather_agree(bam, cache_pages, n_queues, depth):
    """The scattered gather in every launch shape (one request per thread as the reference has it, four per thread, and in
    two launches with 1 to 8 reads per lane in the first), a ragged request count, caches from a few pages to one that
    holds everything: same sum, every request counted once, and hits + misses = accesses, whatever the shape; on the cache
    that holds everything the second round is all hits and does no I/O."""
    from bam_amd import gen
    n_elems, n = 1 << 22, (1 << 17) + 37          # 8192 pages of data
    want = oracle.lib().bo_gather_sum(SEED, SEED, 0, n, n_elems)
    with Rig(bam, 64 << 20, n_queues=n_queues, depth=depth) as r:
        a = r.array(n_elems, 4096, cache_pages)
        idx = gen.gather_indices(SEED, n, n_elems)
        shapes = [(a.ONE_PER_THREAD, 1), (a.FOUR_PER_THREAD, 4)] + [(a.TWO_LAUNCHES, k) for k in (1, 2, 4, 8)]
        for rnd in range(2):
            for shape, lanes in shapes:
                for block in (64, 256):
                    assert a.read_shaped(n, idx, shape, lanes, block_size=block) == want, (shape, lanes, block)
                    st = a.stats()
                    assert st["access_cnt"] == n and st["hit_cnt"] + st["miss_cnt"] == n, (shape, lanes, st)
                    if cache_pages == 8192 and rnd == 1:
                        assert st["read_io_cnt"] == 0 and st["hit_cnt"] == n
                    if cache_pages == 8:
                        assert st["read_io_cnt"] > 0
        assert a.read(n, idx, block_size=64) == want                  # what bam_array_read picks for a launch of this size
        assert a.stats()["access_cnt"] == n
        assert not r.c.aborted() and r.c.info()["error_completions"] == 0


@pytest.mark.parametrize("cache_pages,n_queues,depth,block", [(64, 4, 64, 64), (1024, 2, 16, 256), (4096, 16, 1024, 128)])
def test_every_element_of_a_gather_and_of_an_update_under_eviction(bam, cache_pages, n_queues, depth, block):
    """Element by element instead of a sum: 2^18 random reads through a cache that holds a fraction of the data, on queues so
    shallow that a wave's misses go through them in rounds, and on deep ones.  Then the same requests as atomic adds of zero
    (every page dirty, so every eviction is a write-back followed by a read into the same slot), the reads again, and adds
    to distinct elements that must show up in a gather and, after a flush, in the store."""
    n_elems, n = 1 << 22, 1 << 18
    rng = np.random.default_rng(SEED)
    with Rig(bam, n_elems * 8, backing=True, n_queues=n_queues, depth=depth) as r:
        store = r.backing(n_elems)
        store[:] = oracle.store(SEED, 0, n_elems)
        model = store.copy()
        a = r.array(n_elems, 4096, cache_pages)
        idx = rng.integers(0, n_elems, n).astype(np.uint64)
        d_idx, want = _dev(idx), model[idx.astype(np.int64)]
        assert np.array_equal(_u64(a.gather(n, d_idx, block_size=block)), want)
        assert np.array_equal(_u64(a.update(0, d_idx, _dev(np.zeros(n, dtype=np.uint64)), block_size=block)), want)
        assert np.array_equal(_u64(a.gather(n, d_idx, block_size=block)), want)
        didx = rng.permutation(n_elems)[:n].astype(np.uint64)
        vals = rng.integers(1, 1 << 63, n).astype(np.uint64)
        assert np.array_equal(_u64(a.update(0, _dev(didx), _dev(vals), block_size=block)), model[didx.astype(np.int64)])
        model[didx.astype(np.int64)] += vals
        assert np.array_equal(_u64(a.gather(n, _dev(didx), block_size=block)), model[didx.astype(np.int64)])
        assert np.array_equal(_u64(a.gather(n, d_idx, block_size=block)), model[idx.astype(np.int64)])
        r.objs[0][2].flush()
        assert np.array_equal(r.backing(n_elems), model)
        assert not r.c.aborted() and r.c.info()["error_completions"] == 0 and r.t.stats()["write_cmds"] > 0


@pytest.mark.parametrize("fast", ["1", "0"])
def test_reads_with_and_without_a_reference_give_the_same_elements(bam, fast, monkeypatch):
    """BAM_FAST_READS=0 takes out the read of a resident page that holds no reference (two looks at the page's descriptor
    around the load instead): every read then counts itself in and out, as in the reference.  The elements of a gather
    under eviction (a cache of 256 pages under 2^18 random reads, so every slot changes hands a thousand times while other
    waves read), the sum of the same launch as bam_array_read shapes it and the number of accesses are the same either way."""
    monkeypatch.setenv("BAM_FAST_READS", fast)
    n_elems, n = 1 << 22, 1 << 18
    rng = np.random.default_rng(SEED + 1)
    with Rig(bam, n_elems * 8, backing=True, n_queues=4, depth=64) as r:
        store = r.backing(n_elems)
        store[:] = oracle.store(SEED, 0, n_elems)
        a = r.array(n_elems, 4096, 256)
        idx = rng.integers(0, n_elems, n).astype(np.uint64)
        d_idx, want = _dev(idx), store[idx.astype(np.int64)]
        for _ in range(2):
            assert np.array_equal(_u64(a.gather(n, d_idx, block_size=64)), want)
        a.stats()
        assert a.read(n, d_idx, block_size=256) == int(np.sum(want, dtype=np.uint64))
        assert a.stats()["access_cnt"] == n
        assert not r.c.aborted() and r.c.info()["error_completions"] == 0


@pytest.mark.parametrize("stage_bytes,cache_pages", [(4096, 5), (0, 5), (4096, 16)])
def test_pages_loaded_on_one_cluster_are_read_on_the_others(bam, stage_bytes, cache_pages):
    """The device has eight clusters of compute units with an L2 each.  A page that a wave on one cluster brings into the
    cache (pulled from a staging page, or placed by the controller when there is no staging) must be what waves on the
    other clusters read a moment later, in a slot that held another page a few rounds before (their L2 may remember it).
    bam_xcd_relay hands 600 pages round a ring of 64 waves through a cache of a few slots and compares every element read."""
    n_pages = 600
    with Rig(bam, 64 << 20, n_queues=4, depth=64, stage_bytes=stage_bytes) as r:
        a = r.array(n_pages * 512, 4096, cache_pages)
        res = a.xcd_relay(SEED, 4096, n_pages, rounds=n_pages, n_waves=64, spin_limit=1 << 18)
        assert bin(res["cluster_mask"]).count("1") >= 2, "the waves ran on one cluster only: nothing was tested"
        assert res["waits_given_up"] == 0
        assert res["mismatches"] == 0 and res["reads_checked"] >= n_pages * 63 * 2
        st = a.stats()
        assert st["read_io_cnt"] >= n_pages and not r.c.aborted()


def test_ragged_and_empty_and_last_element(bam):
    n_elems = (1 << 16) + 37                 # last page partly used
    with Rig(bam, 1 << 20) as r:
        a = r.array(n_elems, 4096, 32)
        assert a.read(0) == 0
        assert a.read(1) == oracle.lib().bo_splitmix64(SEED, 0)
        assert a.read(77) == oracle.lib().bo_store_sum(SEED, 0, 1, 77)          # one and a bit waves
        idx = np.array([n_elems - 1, 0, n_elems - 1, 511, 512, n_elems - 37], dtype=np.uint64)
        assert a.read(len(idx), _dev(idx)) == int(np.sum(oracle.store(SEED, 0, n_elems)[idx.astype(np.int64)], dtype=np.uint64))
        st = a.stats()
        assert st["access_cnt"] == 0 + 1 + 77 + 6


def test_memory_backed_store_disk_offset_and_small_pages(bam):
    data = (np.arange(1 << 18, dtype=np.uint64) * np.uint64(0x9E3779B97F4A7C15)) ^ np.uint64(0xABCDEF)
    with Rig(bam, data.nbytes, backing=True) as r:
        r.backing(len(data))[:] = data
        off_elems = 4096
        a = r.array(len(data) - off_elems, 512, 256, disk_offset=off_elems * 8)     # 512-byte lines as in the reference's Optane runs
        idx = oracle.gather_indices(7, 0, 1 << 16, len(data) - off_elems)
        assert a.read(len(idx), _dev(idx), block_size=64) == int(np.sum(data[idx.astype(np.int64) + off_elems], dtype=np.uint64))
        st = a.stats()
        assert st["access_cnt"] == len(idx) and st["read_io_cnt"] > 256
        assert r.t.stats()["bytes_read"] == st["read_io_cnt"] * 512


def test_large_pages_through_bigger_staging(bam):
    with Rig(bam, 32 << 20, stage_bytes=8192) as r:
        a = r.array(1 << 20, 8192, 64)
        assert a.read(1 << 18, stride=3) == oracle.lib().bo_store_sum(SEED, 0, 3, 1 << 18)
        assert r.t.stats()["bytes_read"] == a.stats()["read_io_cnt"] * 8192


def test_array_of_several_ranges(bam):
    """three ranges of one array, placed apart on the store, the third starting in the middle of a page (range_t's
    page_start / page_start_offset, include/page_cache.h:984-1030 of the reference)"""
    from bam_amd import gen
    per = 1 << 16
    with Rig(bam, 16 << 20, n_queues=8, depth=256) as r:
        pc = bam.PageCache(4096, 256, 0, r.c)
        layout = [(0, 0), (1000, 0), (300, 1024)]                    # (first page on the store, byte offset of the first element in it)
        ranges = [bam.Range(k * per, (k + 1) * per, ps, (per * 8 + pso + 4095) // 4096, pso, 4096, pc, 0) for k, (ps, pso) in enumerate(layout)]
        a = bam.Array(3 * per, 0, ranges, 0)
        store = oracle.store(SEED, 0, 2 << 20)
        flat = np.concatenate([store[ps * 512 + pso // 8: ps * 512 + pso // 8 + per] for ps, pso in layout])
        assert a.read(3 * per) == int(np.sum(flat, dtype=np.uint64))
        idx = gen.gather_indices(SEED, 1 << 17, 3 * per)
        assert a.read(1 << 17, idx, block_size=256) == int(np.sum(flat[_u64(idx)], dtype=np.uint64))
        # bam_ptr crosses ranges too (every lane keeps the page it points into: few enough threads for the slots there are)
        assert a.read_via(4, 64, idx) == int(np.sum(flat[_u64(idx)[:64]], dtype=np.uint64))
        seams = np.concatenate([np.arange(k * per - 1024, k * per + 1024, dtype=np.uint64) for k in (1, 2)])
        assert a.read_via(4, len(seams), _dev(seams)) == int(np.sum(flat[seams], dtype=np.uint64))
        st = a.stats()
        assert st["access_cnt"] == 3 * per + (1 << 17) + 64 + len(seams) and not r.c.aborted()
        a.close()
        for x in ranges:
            x.close()
        pc.close()


@pytest.mark.parametrize("dist", [0, 1])
def test_two_controllers_behind_one_cache(bam, dist):
    """REPLICATE: the same data on both, reads spread over them; STRIPE: page p on controller p % 2 at page p / 2
    (get_backing_page_ / get_backing_ctrl_, include/page_cache.h:556-582 of the reference)"""
    from bam_amd import gen
    n_elems, n = 1 << 20, 1 << 17
    seeds = (SEED, SEED) if dist == 0 else (11, 22)
    paths = [_path(), _path()]
    ts = [bam.Target(p, 16 << 20, 512, seed=sd, n_io_threads=2) for p, sd in zip(paths, seeds)]
    cs = [bam.Controller(p, 1, 0, queue_depth=256, n_queues=4, spin_limit=LIMIT_US) for p in paths]
    try:
        pc = bam.PageCache(4096, 256, 0, cs)
        rg = bam.Range(0, n_elems, 0, n_elems // 512, 0, 4096, pc, 0, dist=dist)
        a = bam.Array(n_elems, 0, [rg], 0)
        if dist == 0:
            flat = oracle.store(SEED, 0, n_elems)
        else:
            pages = [oracle.store(sd, 0, n_elems // 2).reshape(-1, 512) for sd in seeds]
            flat = np.empty((n_elems // 512, 512), dtype=np.uint64)
            flat[0::2] = pages[0]
            flat[1::2] = pages[1]
            flat = flat.reshape(-1)
        idx = gen.gather_indices(SEED, n, n_elems)
        for _ in range(2):
            assert a.read(n, idx, block_size=128) == int(np.sum(flat[_u64(idx)], dtype=np.uint64))
        assert a.read(n_elems, block_size=256) == int(np.sum(flat, dtype=np.uint64))
        reads = [t.stats()["read_cmds"] for t in ts]
        assert min(reads) > 0.3 * max(reads) and sum(reads) == a.stats()["read_io_cnt"]
        assert not cs[0].aborted() and not cs[1].aborted()
        a.close(); rg.close(); pc.close()
    finally:
        for c in cs:
            c.close()
        for t in ts:
            t.close()


def test_direct_placement_without_staging(bam):
    """stage_bytes = 0: PRPs name the cache slots themselves and the controller writes the payload into device memory"""
    from bam_amd import gen
    n_elems, n = 1 << 22, 1 << 18
    with Rig(bam, 32 << 20, n_queues=8, depth=256, stage_bytes=0, backing=True) as r:
        a = r.array(n_elems, 4096, 1024)
        assert r.objs[0][2].info()["staged"] == 0
        for rep in range(2):
            idx = gen.gather_indices(SEED, n, n_elems, first=rep * n)
            assert a.read(n, idx, block_size=128) == oracle.lib().bo_gather_sum(SEED, SEED, rep * n, n, n_elems)
        # the write path the other way: dirty pages are read by the controller out of device memory
        vals = np.arange(1 << 16, dtype=np.uint64) * np.uint64(7) + np.uint64(3)
        a.write(1 << 16, _dev(vals), block_size=64)
        r.objs[0][2].flush()
        assert np.array_equal(r.backing(1 << 16), vals)
        assert a.stats()["read_io_cnt"] > 0 and not r.c.aborted()


@pytest.mark.parametrize("page,stage", [(16384, 0), (65536, 0), (16384, 4096)])
def test_pages_above_two_controller_pages_use_prp_lists(bam, page, stage):
    """cache pages of 4 and 16 controller pages: PRP1 + a PRP list per slot (include/page_cache.h:826-867 of the
    reference), placed directly; with staging pages configured they are too small for such a page and are bypassed"""
    from bam_amd import gen
    n_elems, n = 1 << 22, 1 << 16
    with Rig(bam, 32 << 20, n_queues=8, depth=256, stage_bytes=stage, backing=True) as r:
        a = r.array(n_elems, page, 40)
        idx = gen.gather_indices(SEED, n, n_elems)
        assert a.read(n, idx, block_size=128) == oracle.lib().bo_gather_sum(SEED, SEED, 0, n, n_elems)
        assert a.read(1 << 18, stride=16) == oracle.lib().bo_store_sum(SEED, 0, 16, 1 << 18)
        st = a.stats()
        assert r.t.stats()["bytes_read"] == r.c.info()["ssd_accesses"] * page and st["read_io_cnt"] > 40 and not r.c.aborted()
        vals = np.arange(1 << 15, dtype=np.uint64) * np.uint64(5) + np.uint64(9)
        a.write(1 << 15, _dev(vals), block_size=64)               # dirty large pages go back the same way
        r.objs[0][2].flush()
        assert np.array_equal(r.backing(1 << 15), vals) and not r.c.aborted()


def test_cache_slots_exported_as_a_dma_buf(bam):
    """The GPU side of putting a real NVMe device behind the cache: the slots' device memory as a dma-buf descriptor that
    a driver can import and map for the device's DMA.  Where the runtime exports it, the descriptor is a real one, as
    large as the slots; where it cannot, the call says so (ENOTSUP) and nothing else changes."""
    import os
    import stat
    with Rig(bam, 64 << 20) as r:
        a = r.array(1 << 20, 4096, 256)
        pc = r.objs[0][2]
        got = pc.export_dmabuf()
        if got is None:
            pytest.skip("this runtime does not export device memory")
        fd, n = got
        try:
            assert fd >= 0 and n == 256 * 4096
            st = os.fstat(fd)
            assert not stat.S_ISREG(st.st_mode) and not stat.S_ISDIR(st.st_mode)
            assert st.st_size in (0, n) or st.st_size >= n
        finally:
            os.close(fd)
        assert a.read(1 << 16, stride=16) == oracle.lib().bo_store_sum(SEED, 0, 16, 1 << 16)      # the cache works as before


# ---------------------------------------------------------------- cache / pattern streaming

@pytest.mark.parametrize("mode", [0, 1, 2, 3, 4, 5, 6])
def test_page_streaming_modes(bam, mode):
    n_pages = 4096
    with Rig(bam, 64 << 20) as r:
        a = r.array(n_pages * 512, 4096, n_pages)
        ref = oracle.lib().bo_store_sum(SEED, 0, 1, n_pages * 512)
        assert a.stream(n_pages // 2, 2, mode=mode) == ref          # cold: every page read once
        st = a.stats()
        # every page comes in once.  Per-element operator[] in one launch (mode 5): the wave's first access to a page misses,
        # its seven others hit; bam_ptr in one launch (6) and the page-wise kernel (2) take each page once per wave, as a miss;
        # modes 3 and 4, and the second launch of modes 0 and 1, ask for the pages of a wave's run as one batch before they read
        # (not counted as accesses), so their own accesses all find their page
        assert st["read_io_cnt"] == n_pages
        assert st["hit_cnt"] == {0: n_pages * 512, 1: n_pages * 64, 2: 0, 3: n_pages * 64, 4: n_pages * 512, 5: n_pages * 448, 6: 0}[mode]
        # accesses: one per element with operator[], one per lane per page with bam_ptr, one per page when pages are taken in batches
        assert st["access_cnt"] == {0: n_pages * 512, 1: n_pages * 64, 2: n_pages, 3: n_pages * 64, 4: n_pages * 512, 5: n_pages * 512, 6: n_pages * 64}[mode]
        assert a.stream(n_pages // 2, 2, mode=mode) == ref          # hot: no I/O at all
        st = a.stats()
        assert st["read_io_cnt"] == 0 and st["miss_cnt"] == 0
        # permuted page assignment, smaller cache than data
    with Rig(bam, 64 << 20) as r:
        a = r.array(n_pages * 512, 4096, 512)
        perm = np.random.default_rng(3).permutation(n_pages).astype(np.uint64)
        assert a.stream(n_pages, 1, _dev(perm), mode=mode) == ref
        assert not r.c.aborted()


def test_second_look_of_the_pointer_that_holds_no_reference(bam):
    """bam_ptr<T, true> opens its window on a look at the page's descriptor and what was read counts once still() finds the
    descriptor as it was.  Changed under the window, one way at a time: other readers' references and the dirty bit do
    not matter; busy, not valid, another slot, or the same slot after one more load of the page, and the window falls
    (a mask with a bit too few in it would let one of them through)."""
    with Rig(bam, 8 << 20) as r:
        a = r.array(1 << 18, 4096, 64)
        assert a.read(1 << 15, stride=1) == oracle.lib().bo_store_sum(SEED, 0, 1, 1 << 15)      # pages 0..63 are resident now
        assert a.unheld_window_cases(5) == [1, 1, 1, 2, 2, 2, 2]
        assert a.unheld_window_cases(63) == [1, 1, 1, 2, 2, 2, 2]
        assert a.unheld_window_cases(200) == [4] * 7                                              # never loaded: no window at all
        assert a.read(1 << 15, stride=1) == oracle.lib().bo_store_sum(SEED, 0, 1, 1 << 15) and a.stats()["read_io_cnt"] == 64
        assert not r.c.aborted()


def test_streaming_what_is_resident_while_another_stream_evicts(bam):
    """Two arrays behind one cache, each driven from a stream of its own.  One is streamed element by element (modes 0 and
    1: first a launch that reads what is resident without holding it, every page confirmed by a second look at its
    descriptor, then a launch for the rest) while random reads of the other, four times the cache, take its pages away
    under it: a page that goes between the two looks must be left to the second launch, and a page that goes and comes
    back must not be read half old, half new.  Every sum of both arrays is exact, launch after launch."""
    import torch
    page, nx_pages, ny_pages, cache_pages, n = 4096, 2048, 8192, 1024, 1 << 17
    nx, ny = nx_pages * 512, ny_pages * 512
    with Rig(bam, (nx + ny) * 8, n_queues=16, depth=256) as r:
        pc = bam.PageCache(page, cache_pages, 0, r.c)
        rx = bam.Range(0, nx, 0, nx_pages, 0, page, pc, 0)
        ry = bam.Range(0, ny, nx_pages, ny_pages, 0, page, pc, 0)
        ax, ay = bam.Array(nx, 0, [rx], 0), bam.Array(ny, nx_pages * page, [ry], 0)
        want_x = oracle.lib().bo_store_sum(SEED, 0, 1, nx)
        words_y = oracle.store(SEED, nx, ny)
        rng = np.random.default_rng(SEED + 5)
        reps = 8
        idx = [rng.integers(0, ny, n).astype(np.uint64) for _ in range(reps)]
        d_idx = [_dev(i) for i in idx]
        sums_x = [torch.zeros(1, dtype=torch.int64, device="cuda:0") for _ in range(reps)]
        sums_y = [torch.zeros(1, dtype=torch.int64, device="cuda:0") for _ in range(reps)]
        sx, sy = torch.cuda.Stream(), torch.cuda.Stream()
        torch.cuda.synchronize()
        for k in range(reps):
            with torch.cuda.stream(sx):
                ax.stream_async(nx_pages // 16, 16, sums_x[k], mode=k % 2)
            with torch.cuda.stream(sy):
                ay.read_async(n, sums_y[k], d_idx[k], block_size=256)
        torch.cuda.synchronize()
        for k in range(reps):
            assert int(sums_x[k].item()) & (2**64 - 1) == want_x, "streamed array, launch %d" % k
            assert int(sums_y[k].item()) & (2**64 - 1) == int(np.sum(words_y[idx[k].astype(np.int64)], dtype=np.uint64)), "gathered array, launch %d" % k
        # one access per element through operator[] (mode 0), one per lane and page through bam_ptr (mode 1): a page that was
        # given up on in the first launch is counted in the second and nowhere else
        assert ax.stats()["access_cnt"] == reps // 2 * (nx + nx_pages * 64) and ay.stats()["access_cnt"] == reps * n
        assert r.t.stats()["read_cmds"] > reps * nx_pages // 2 and not r.c.aborted() and r.c.info()["error_completions"] == 0
        ax.close(); ay.close(); rx.close(); ry.close(); pc.close()


@pytest.mark.parametrize("mode", [0, 1, 3, 4, 5, 6])
@pytest.mark.parametrize("page", [512, 4096, 16384])
def test_element_streaming_over_other_page_sizes_and_a_ragged_last_page(bam, mode, page):
    """The per-element streaming kernels where a lane reads one element of a page (512 B), eight (4 KiB) or thirty-two
    (16 KiB), and over an array that ends inside its last page: the lanes past the end read nothing, and bam_ptr's
    side-by-side reads (covers/peek) give way to operator[] per element on the page the array ends in."""
    epp, n_pages = page // 8, 1024
    n_elems = n_pages * epp - epp // 4
    with Rig(bam, 64 << 20) as r:
        a = r.array(n_elems, page, n_pages)
        ref = oracle.lib().bo_store_sum(SEED, 0, 1, n_elems)
        assert a.stream(n_pages // 4, 4, mode=mode) == ref          # cold
        assert a.stats()["read_io_cnt"] == n_pages
        assert a.stream(n_pages // 4, 4, mode=mode) == ref          # resident
        assert a.stats()["read_io_cnt"] == 0 and not r.c.aborted()
    with Rig(bam, 64 << 20) as r:
        a = r.array(n_elems, page, 96)                              # a tenth of the data fits
        assert a.stream(n_pages // 4, 4, mode=mode) == ref and not r.c.aborted()


# ---------------------------------------------------------------- the other access routes of array_d_t

@pytest.mark.parametrize("api", [1, 2, 3, 4, 6, 7])
def test_access_routes_give_the_same_sums(bam, api):
    """get_raw/release_raw, get_page_gid + acquire_page_, acquire_page/release_page, bam_ptr, bam_ptr_tlb and bafs_ptr read what operator[] reads"""
    from bam_amd import gen
    n_elems, n = 1 << 22, 4096                  # 8192 pages of data; 64 waves hold at most 4096 pages at a time
    with Rig(bam, 32 << 20, n_queues=8, depth=256) as r:
        a = r.array(n_elems, 4096, 6000)
        for rep in range(3):                    # 3 x 4096 random pages through 6000 slots: later passes evict
            idx = gen.gather_indices(SEED, n, n_elems, first=rep * n)
            assert a.read_via(api, n, idx) == oracle.lib().bo_gather_sum(SEED, SEED, rep * n, n, n_elems)
        st = a.stats()
        assert st["access_cnt"] == 3 * n * (2 if api == 7 else 1) and st["read_io_cnt"] > 6000 and not r.c.aborted()      # route 7 dereferences twice
        assert a.read_via(api, 1000, None, span=517) == int(np.sum(oracle.store(SEED, 0, n_elems)[:1000 * 517:517], dtype=np.uint64))
        # neighbouring elements: the lanes of a wave share pages (and, through a tlb, entries)
        assert a.read_via(api, 50000, None, span=3, block_size=256) == int(np.sum(oracle.store(SEED, 0, n_elems)[:150000:3], dtype=np.uint64))


def test_wave_memcpy_out_of_the_cache(bam):
    """array_d_t::memcpy: a wave copies up to `span` elements from its index on, clipped to the page and the array"""
    from bam_amd import gen
    n_elems, n, span = 1 << 18, 2048, 96
    with Rig(bam, 2 << 20) as r:
        a = r.array(n_elems, 4096, 64)
        idx = gen.gather_indices(SEED, n, n_elems)
        store = oracle.store(SEED, 0, n_elems)
        want = 0
        for i in _u64(idx).tolist():
            cnt = min(span, 512 - i % 512, n_elems - i)
            want = (want + int(np.sum(store[i:i + cnt], dtype=np.uint64))) % 2**64
        assert a.read_via(5, n, idx, span=span) == want
        assert not r.c.aborted()


# ---------------------------------------------------------------- raw block

@pytest.mark.parametrize("req,lba,order,raw_share", [(4096, 512, 0, None), (4096, 512, 0, "3"), (4096, 512, 0, "8"), (512, 512, 2, None), (4096, 4096, 1, None)])
def test_block_reads_payload_checksums(bam, req, lba, order, raw_share, monkeypatch):
    """raw reads into slots the caller names; by default all of them staged, with BAM_DIRECT_SHARE_RAW three of eight
    batches or all of them placed by the target"""
    from bam_amd import gen
    if raw_share is not None:
        monkeypatch.setenv("BAM_DIRECT_SHARE_RAW", raw_share)
    n, ns = 1 << 16, 64 << 30
    with Rig(bam, ns, lba=lba, n_queues=16, depth=256, order=order) as r:
        pc = bam.PageCache(4096, n, 0, r.c)
        lbas = gen.block_lbas(SEED, n, ns, req, lba)
        for policy in (0, 1):
            pc.block_io(n, req, lbas, queue_policy=policy)
            cs = _u64(pc.block_checksums(n, req))
            ref = np.array([oracle.lib().bo_block_checksum(SEED, int(x), lba, req) for x in _u64(lbas)], dtype=np.uint64)
            assert np.array_equal(cs, ref)
        pc.block_io(1000, req, None)            # sequential LBAs, ragged last wave
        cs = _u64(pc.block_checksums(1000, req))
        ref = np.array([oracle.lib().bo_block_checksum(SEED, k * req // lba, lba, req) for k in range(1000)], dtype=np.uint64)
        assert np.array_equal(cs, ref)
        ts = r.t.stats()
        assert ts["read_cmds"] == 2 * n + 1000 and ts["error_cpls"] == 0 and ts["sq_doorbells"] < ts["read_cmds"]
        assert not r.c.aborted()
        pc.close()


@pytest.mark.parametrize("n_queues,depth,order", [(4, 16, 0), (8, 16, 2), (7, 64, 1), (128, 1024, 0), (7, 16, 0), (2, 16, 1), (1, 4, 0)])
def test_block_io_through_the_per_thread_queue_operations(bam, n_queues, depth, order):
    """Every thread builds and runs its own command with get_cid, nvm_cmd_*, sq_enqueue, cq_poll, cq_dequeue and put_cid,
    as the reference's read_data is written, thread t on queue pair t mod n_qps: the lanes of a wave are on different
    queue pairs, sixteen of them per queue of sixteen slots (the whole queue per wave), eight (half of it), nine or
    ten where 64 does not divide (consecutive waves then meet the queues in rotated orders), thirty-two or all sixty-four
    on queues of sixteen and of four slots (more lanes than slots), the last wave ragged; completions in order, reversed
    and shuffled.  Payload checksums
    against the oracle, then a write of the same slots further on and a read back, and the ids come back every time (the
    launches repeat on the same queues)."""
    from bam_amd import gen
    n, ns, req, lba = 5000 + 37, 1 << 30, 4096, 512
    with Rig(bam, ns, lba=lba, n_queues=n_queues, depth=depth, order=order, backing=True) as r:
        pc = bam.PageCache(4096, n, 0, r.c)
        for rep in range(3):
            lbas = gen.block_lbas(SEED + rep, n, ns // 2, req, lba)
            pc.block_io(n, req, lbas, queue_policy=2, block_size=256 if rep else 64)
            cs = _u64(pc.block_checksums(n, req))
            assert not r.c.aborted(), (rep, r.t.stats())
            ref = np.array([oracle.lib().bo_block_checksum(SEED, int(x), lba, req) for x in _u64(lbas)], dtype=np.uint64)
            assert np.array_equal(cs, ref), (rep, int((cs != ref).sum()), r.t.stats())
        # the slots as they are now, written to distinct blocks in the upper half of the namespace and read back
        before = cs.copy()
        up = _dev(np.arange(n, dtype=np.uint64) * np.uint64(req // lba) + np.uint64(ns // 2 // lba))
        pc.block_io(n, req, up, write=True, queue_policy=2)
        pc.block_io(n, req, None, queue_policy=2)                     # something else into the slots in between
        assert not np.array_equal(_u64(pc.block_checksums(n, req)), before)
        pc.block_io(n, req, up, queue_policy=2)
        assert np.array_equal(_u64(pc.block_checksums(n, req)), before)
        ts = r.t.stats()
        assert ts["read_cmds"] == 5 * n and ts["write_cmds"] == n and ts["error_cpls"] == 0 and not r.c.aborted()
        pc.close()


@pytest.mark.parametrize("lanes", [(1 << 64) - 1, (1 << 37) - 1, 0xAAAAAAAAAAAAAAAA, 1 << 63, 0x8000000100000001])
def test_warp_memcpy_with_any_set_of_lanes(bam, lanes):
    """util.h's warp_memcpy: a count of elements, shared out over whichever lanes are active; nothing is written past it"""
    import torch
    for n in (0, 1, 63, 64, 1000, 4097):
        src = torch.arange(1, n + 9, dtype=torch.int64, device="cuda") * 0x9E3779B97F4A7C15
        dst = torch.full((n + 8,), -1, dtype=torch.int64, device="cuda")
        assert bam._lib.load().bam_warp_memcpy(ctypes.c_void_p(dst.data_ptr()), ctypes.c_void_p(src.data_ptr()), n, lanes, None) == 0
        torch.cuda.synchronize()
        assert torch.equal(dst[:n], src[:n]) and bool((dst[n:] == -1).all())


@pytest.mark.parametrize("req", [4096, 512])
def test_block_reads_at_full_size_every_checksum(bam, req):
    """The raw-read configuration at its full shape: 2^22 reads on 128 queue pairs of 1024 entries, every payload checked.
    What a block must hold comes from the device generator of the store's words (pinned to the oracle by the generator
    tests) through a running sum over the namespace: checksum(block) = S[w0 + words] - S[w0]; a sample is also checked
    against the oracle's own checksum."""
    import torch
    from bam_amd import gen
    n, ns, lba = 1 << 22, 2 << 30, 512
    with Rig(bam, ns, lba=lba, n_queues=128, depth=1024, io_threads=12) as r:
        pc = bam.PageCache(4096, n, 0, r.c)
        lbas = gen.block_lbas(SEED, n, ns, req, lba)
        pc.block_io(n, req, lbas)
        cs = pc.block_checksums(n, req)
        words = gen.words(SEED, 0, ns // 8)
        run = torch.cumsum(words, 0)                       # wraps mod 2^64 like the checksum does
        del words
        w0 = lbas * (lba // 8)
        want = run[w0 + (req // 8 - 1)] - torch.where(w0 > 0, run[torch.clamp(w0 - 1, min=0)], torch.zeros_like(w0))
        assert bool(torch.equal(cs, want))
        host_cs, host_lba = _u64(cs), _u64(lbas)
        for k in np.random.default_rng(SEED).integers(0, n, 2048):
            assert int(host_cs[k]) == oracle.lib().bo_block_checksum(SEED, int(host_lba[k]), lba, req)
        ts = r.t.stats()
        assert ts["read_cmds"] == n and ts["error_cpls"] == 0 and ts["bytes_read"] == n * req and not r.c.aborted()
        pc.close()


@pytest.mark.parametrize("depth,n_threads", [(1, 4096), (2, 2048), (4, 1024)])
def test_block_reads_with_several_commands_in_flight_per_thread(bam, depth, n_threads):
    """access_data_async / poll_async: every payload arrives, ids come back (the launch can be repeated)"""
    from bam_amd import gen
    ns, req, lba = 1 << 30, 4096, 512
    with Rig(bam, ns, n_queues=16, depth=256) as r:             # 4 blocks of 64 command ids per queue pair
        n = n_threads * depth
        pc = bam.PageCache(4096, n, 0, r.c)
        for rep in range(3):
            lbas = gen.block_lbas(SEED + rep, n, ns, req, lba)
            pc.block_io_async(n_threads, depth, req, lbas)
            cs = _u64(pc.block_checksums(n, req))
            ref = np.array([oracle.lib().bo_block_checksum(SEED, int(x), lba, req) for x in _u64(lbas)], dtype=np.uint64)
            assert np.array_equal(cs, ref)
        assert r.t.stats()["read_cmds"] == 3 * n and not r.c.aborted()
        with pytest.raises(Exception):
            pc.block_io_async(n_threads * 2, depth * 2 if depth < 8 else 8, req, lbas)      # would not fit the command ids
        pc.close()


def test_block_write_then_read_back(bam):
    n = 4096
    with Rig(bam, 64 << 20, backing=True) as r:
        pc = bam.PageCache(4096, n, 0, r.c)
        pc.block_io(n, 4096, None)                                   # slots <- LBAs 0..
        before = _u64(pc.block_checksums(n, 4096)).copy()
        shifted = _dev(np.arange(n, dtype=np.uint64) * np.uint64(8) + np.uint64(8 * n))
        pc.block_io(n, 4096, shifted, write=True)                    # same payload to LBAs further on
        store = r.backing((64 << 20) // 8)
        assert np.array_equal(store[n * 512: 2 * n * 512], oracle.store(SEED, 0, n * 512))
        pc.block_io(n, 4096, shifted)
        assert np.array_equal(_u64(pc.block_checksums(n, 4096)), before)
        assert r.t.stats()["write_cmds"] == n
        pc.close()


# ---------------------------------------------------------------- write path through the cache

def test_array_write_eviction_write_back_and_flush(bam):
    n_elems = 1 << 16
    with Rig(bam, n_elems * 8, backing=True) as r:
        a = r.array(n_elems, 4096, 16)                               # 128 pages of data, 16 cached: dirty pages get evicted
        vals = np.arange(n_elems, dtype=np.uint64) * np.uint64(3) + np.uint64(1)
        a.write(n_elems, _dev(vals), block_size=64)
        r.objs[0][2].flush()
        assert np.array_equal(r.backing(n_elems), vals)
        assert a.read(n_elems) == int(np.sum(vals, dtype=np.uint64))
        assert r.t.stats()["write_cmds"] >= 128 and not r.c.aborted()


@pytest.mark.parametrize("cache_pages,direct_share", [(24, None), (96, None), (96, "8"), (96, "0")])
def test_random_writes_and_reads_against_a_model_of_the_store(bam, cache_pages, direct_share, monkeypatch):
    """rounds of scattered writes (distinct elements per round, many per page) and scattered reads through a cache far
    smaller than the data: dirty pages are evicted, written back and read again all the time; a numpy array plays the
    store.  Reads of a round see the writes of all rounds before it, whatever the cache did with the pages in between."""
    if direct_share is not None:
        monkeypatch.setenv("BAM_DIRECT_SHARE", direct_share)
    n_elems = 1 << 19                                                # 1024 pages of data
    rng = np.random.default_rng(SEED + cache_pages)
    with Rig(bam, n_elems * 8, backing=True, n_queues=16, depth=256) as r:
        model = r.backing(n_elems).copy()
        a = r.array(n_elems, 4096, cache_pages)
        for rnd in range(6):
            widx = rng.permutation(n_elems)[:1 << 15].astype(np.uint64)
            wval = (widx * np.uint64(0x9E3779B97F4A7C15) + np.uint64(rnd + 1)).astype(np.uint64)
            a.write(len(widx), _dev(wval), assignment=_dev(widx), block_size=64)
            model[widx] = wval
            ridx = rng.integers(0, n_elems, 1 << 16).astype(np.uint64)
            assert a.read(len(ridx), _dev(ridx), block_size=256) == int(np.sum(model[ridx], dtype=np.uint64)), "round %d" % rnd
        r.objs[0][2].flush()
        assert np.array_equal(r.backing(n_elems), model)
        assert a.read(n_elems) == int(np.sum(model, dtype=np.uint64))
        assert r.t.stats()["write_cmds"] > 0 and not r.c.aborted()


def test_vectoradd_three_arrays_write_back(bam):
    """C = A + B with all three arrays behind one cache (three ranges): the results reach the store with the flush.
    Every lane keeps a page of each array while it works, so the cache has to hold what the waves in flight can pin:
    here all 768 pages."""
    n = 1 << 17                                                  # 256 pages per array
    pages = n // 512
    with Rig(bam, 3 * n * 8, backing=True, n_queues=8, depth=256) as r:
        store = r.backing(3 * n)
        a_h = oracle.store(SEED, 0, n)
        b_h = oracle.store(SEED + 1, 0, n)
        store[:n] = a_h
        store[n:2 * n] = b_h
        store[2 * n:] = 0
        pc = bam.PageCache(4096, 800, 0, r.c)
        rs = [bam.Range(0, n, k * pages, pages, 0, 4096, pc, 0) for k in range(3)]
        arrs = [bam.Array(n, k * n * 8, [rs[k]], 0) for k in range(3)]
        bam.vectoradd(arrs[0], arrs[1], arrs[2], n)
        pc.flush()
        assert np.array_equal(store[2 * n:], a_h + b_h)
        assert np.array_equal(store[:n], a_h) and np.array_equal(store[n:2 * n], b_h)      # inputs untouched
        assert r.t.stats()["write_cmds"] >= pages and not r.c.aborted()
        assert arrs[2].read(n) == int(np.sum(a_h + b_h, dtype=np.uint64))
        for x in arrs + rs:
            x.close()
        pc.close()


@pytest.mark.parametrize("n,block,cache_pages", [(1, 64, 8), (1000, 64, 8), (1 << 16, 256, 32), ((1 << 18) + 77, 1024, 128), (1 << 18, 512, 1024)])
def test_reduction_and_scan_through_bam_ptr(bam, n, block, cache_pages):
    """benchmarks/reduction and benchmarks/scan: per-workgroup sums, and running sums with the total last; unsigned 64-bit
    arithmetic, so bit-exact whatever the order of the adds"""
    pad = (-n) % 512
    with Rig(bam, (n + pad) * 8, backing=True, n_queues=8, depth=256) as r:
        vals = oracle.store(SEED, 11, n)
        r.backing(n + pad)[:n] = vals
        a = r.array(n, 4096, cache_pages)
        assert np.array_equal(_u64(a.reduce(n, block)), oracle.reduce_blocks(vals, block))
        if cache_pages >= (n + pad) // 512:
            # the read-ahead of these kernels touches pages before their readers come: every page still comes in once
            assert a.stats(reset=False)["read_io_cnt"] == (n + pad) // 512
        assert np.array_equal(_u64(a.scan(n, block)), oracle.scan(vals))
        # a prefix of the array only: the tail must not leak in
        m = n - n // 3
        assert np.array_equal(_u64(a.scan(m, block)), oracle.scan(vals[:m]))
        assert int(_u64(a.reduce(m, block)).sum(dtype=np.uint64)) == int(oracle.scan(vals[:m])[-1])
        assert a.stats()["access_cnt"] > 0 and not r.c.aborted()


@pytest.mark.parametrize("direct_share", ["8", "3", "0"])
def test_program_written_against_the_cpp_surface(bam, direct_share):
    """bam_amd/examples/array_sum: an ordinary HIP program that includes page_cache.h and ctrl.h, builds the host objects
    itself and launches its own kernels (operator[] and bam_ptr), as a benchmark of the reference does.  4096 waves, each
    reading one page, share 256 cache slots: a slot is evicted and refilled within microseconds of its last read, which
    is what once let a payload load that was still in flight when its reference was dropped return the next page's data
    (most readily with payload placed directly by the target, hence the three placements)."""
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bam_amd", "examples", "array_sum")
    assert os.path.exists(exe), "bam_amd/examples/array_sum is built by make -C bam_amd/csrc"
    n_elems, cache_pages, stride = 1 << 21, 256, 8                       # 4096 pages of data behind 256 cached pages
    want = oracle.lib().bo_store_sum(SEED, 0, stride, n_elems // stride)
    env = dict(os.environ, BAM_DIRECT_SHARE=direct_share)
    for _ in range(3):
        r = subprocess.run([exe, str(n_elems), str(cache_pages), str(stride), str(SEED)], capture_output=True, text=True, timeout=110, env=env)
        assert r.returncode == 0, r.stdout + r.stderr
        out = dict(line.split(None, 1) for line in r.stdout.splitlines() if line.startswith(("sum_by", "aborted")))
        assert int(out["sum_by_index"], 16) == want and int(out["sum_by_ptr"], 16) == want and out["aborted"].strip() == "0"


# ---------------------------------------------------------------- graphs

def _graph_rig(bam, nb, cache_pages, **kw):
    pad = (-len(nb)) % 512
    r = Rig(bam, (len(nb) + pad) * 8, backing=True, **kw)
    r.backing(len(nb) + pad)[:len(nb)] = nb
    return r, r.array(max(len(nb), 1), 4096, cache_pages)


def test_reference_sample_graph(bam):
    with open(os.path.join(G, "sample_graph.json")) as f:
        g = json.load(f)
    off = np.array(g["offsets"], dtype=np.uint64)
    nb = np.array(g["edges"], dtype=np.uint64)
    r, a = _graph_rig(bam, nb, 64)
    with r:
        for by_page in (False, True):
            for src, exp in g["bfs"].items():
                lv, it = a.bfs(_dev(off), int(src), by_page=by_page)
                assert lv.cpu().numpy().view(np.uint32).tolist() == exp["levels"] and it == exp["iterations"]
            lb, it = a.cc(_dev(off), by_page=by_page)
            assert _u64(lb).tolist() == g["cc"]["labels"]


@pytest.mark.parametrize("scale,cache_pages,coarse", [(10, 4096, 1), (14, 512, 128), (16, 8192, 8)])
def test_bfs_levels_rmat(bam, scale, cache_pages, coarse):
    off, nb = oracle.rmat_csr(SEED, scale)
    r, a = _graph_rig(bam, nb, cache_pages, n_queues=16, depth=256)
    with r:
        doff = _dev(off)
        for src in oracle.bfs_sources(SEED, off, 4):
            lv, it = a.bfs(doff, int(src), coarse=coarse)
            ref, rit = oracle.bfs_levels(off, nb, int(src))
            assert np.array_equal(lv.cpu().numpy().view(np.uint32), ref) and it == rit
        assert not r.c.aborted()


@pytest.mark.parametrize("n_v,n_p,cache_pages,coarse", [(1 << 12, 3000, 256, 1), (1 << 16, 1 << 18, 512, 512), (1 << 14, 1 << 17, 4096, 4)])
def test_cc_labels_uniform(bam, n_v, n_p, cache_pages, coarse):
    off, nb = oracle.uniform_csr(SEED, n_v, n_p)
    r, a = _graph_rig(bam, nb, cache_pages, n_queues=16, depth=256)
    with r:
        lb, it = a.cc(_dev(off), coarse=coarse)
        ref, comps = oracle.cc_labels(off, nb)
        assert np.array_equal(_u64(lb), ref)
        assert len(np.unique(_u64(lb))) == comps and it >= 1
        assert not r.c.aborted()


@pytest.mark.parametrize("scale,cache_pages", [(10, 4096), (14, 2), (14, 64), (16, 8192), (17, 700)])
def test_bfs_levels_rmat_by_edge_page(bam, scale, cache_pages):
    """the edge-page kernel gives the same levels and launch counts; caches from two pages up (what a wave holds is sized from it)"""
    off, nb = oracle.rmat_csr(SEED, scale)
    r, a = _graph_rig(bam, nb, cache_pages, n_queues=16, depth=256)
    with r:
        doff = _dev(off)
        for src in oracle.bfs_sources(SEED, off, 3):
            lv, it = a.bfs(doff, int(src), by_page=True)
            ref, rit = oracle.bfs_levels(off, nb, int(src))
            assert np.array_equal(lv.cpu().numpy().view(np.uint32), ref) and it == rit
        st = a.stats()
        assert st["read_io_cnt"] > 0 and not r.c.aborted()


@pytest.mark.parametrize("by_page", [False, True])
def test_cc_labels_of_a_graph_with_millions_of_components(bam, by_page):
    """2^24 vertices and 0.6 x 2^24 random pairs: below the threshold where a giant component takes over, so the answer is
    millions of labels, not one.  Against the union-find oracle, through a cache that holds a quarter of the edge list."""
    n_v = 1 << 24
    off, nb = oracle.uniform_csr(SEED, n_v, int(0.6 * n_v))
    r, a = _graph_rig(bam, nb, len(nb) // 512 // 4, n_queues=128, depth=1024, io_threads=12)
    with r:
        lb, it = a.cc(_dev(off), coarse=64, by_page=by_page)
        ref, comps = oracle.cc_labels(off, nb)
        got = _u64(lb)
        assert np.array_equal(got, ref)
        assert comps > 1 << 22 and len(np.unique(got)) == comps and it >= 2
        assert a.stats()["read_io_cnt"] > 0 and not r.c.aborted()


def test_graph_plan_gives_the_same_answers_and_is_dropped_when_the_graph_changes(bam):
    """bam_array_set_graph prepares the per-graph tables once; every graph entry point must answer as it does without it, call
    after call, and a call that names other offsets (here: a copy at another address) must not use the plan"""
    off, nb = oracle.rmat_csr(SEED, 14)
    r, a = _graph_rig(bam, nb, 300, n_queues=16, depth=256)
    with r:
        doff, doff2 = _dev(off), _dev(off.copy())
        srcs = [int(x) for x in oracle.bfs_sources(SEED, off, 3)]
        want_cc, comps = oracle.cc_labels(off, nb)
        for planned in (False, True, True):
            if planned:
                a.set_graph(doff)
            for use in (doff, doff2):
                for src in srcs:
                    ref, rit = oracle.bfs_levels(off, nb, src)
                    for kw in ({"coarse": 64}, {"by_page": True}, {"frontier": True}):
                        lv, it = a.bfs(use, src, **kw)
                        assert np.array_equal(lv.cpu().numpy().view(np.uint32), ref) and it == rit, (planned, kw)
                for kw in ({"coarse": 8}, {"by_page": True}):
                    lb, it = a.cc(use, **kw)
                    assert np.array_equal(_u64(lb), want_cc)
        pr_plan, it_plan = a.pagerank(doff)
        a.set_graph(None)
        pr_none, it_none = a.pagerank(doff)
        assert abs(it_plan - it_none) <= 3 and np.allclose(pr_plan.cpu().numpy(), pr_none.cpu().numpy(), rtol=2e-2)    # pushes land in any order: both within the tolerance of the fixed point
        assert not r.c.aborted()


@pytest.mark.parametrize("shape,coarse,stride", [(0, 1, 1), (0, 1, 7), (0, 1, 128), (1, 4, 3), (1, 16, 1), (2, 1, 1), (2, 1, 5), (3, 1, 1)])
def test_bfs_and_cc_with_the_vertices_shared_out_as_the_reference_variants_do(bam, shape, coarse, stride):
    """hash (0), hash + coarse (1), sixteen lanes per vertex (2) and chunk (3) assignment of vertices to waves: the same levels,
    launch counts and labels as the oracle, whatever the stride"""
    off, nb = oracle.rmat_csr(SEED, 13)
    r, a = _graph_rig(bam, nb, 2048, n_queues=16, depth=256)
    with r:
        doff = _dev(off)
        for src in oracle.bfs_sources(SEED, off, 2):
            lv, it = a.bfs_shaped(doff, int(src), shape, coarse=coarse, stride=stride)
            ref, rit = oracle.bfs_levels(off, nb, int(src))
            assert np.array_equal(lv.cpu().numpy().view(np.uint32), ref) and it == rit
        assert not r.c.aborted()
    off, nb = oracle.uniform_csr(SEED, 1 << 13, 1 << 13)
    r, a = _graph_rig(bam, nb, 2048, n_queues=16, depth=256)
    with r:
        lb, it = a.cc_shaped(_dev(off), shape, coarse=coarse, stride=stride)
        ref, comps = oracle.cc_labels(off, nb)
        assert np.array_equal(_u64(lb), ref) and len(np.unique(_u64(lb))) == comps
        assert a.stats()["read_io_cnt"] > 0 and not r.c.aborted()


@pytest.mark.parametrize("n_v,n_p,cache_pages", [(1 << 12, 3000, 256), (1 << 16, 1 << 18, 6), (1 << 14, 1 << 17, 4096)])
def test_cc_labels_uniform_by_edge_page(bam, n_v, n_p, cache_pages):
    off, nb = oracle.uniform_csr(SEED, n_v, n_p)
    r, a = _graph_rig(bam, nb, cache_pages, n_queues=16, depth=256)
    with r:
        lb, it = a.cc(_dev(off), by_page=True)
        ref, comps = oracle.cc_labels(off, nb)
        assert np.array_equal(_u64(lb), ref)
        assert len(np.unique(_u64(lb))) == comps and it >= 1
        assert not r.c.aborted()


@pytest.mark.parametrize("cache_pages,coarse", [(24, 1), (256, 4), (4096, 64), (4096, 200)])
def test_hub_lists_are_cut_into_pieces(bam, cache_pages, coarse):
    """two hubs with lists of 9000 and 4096 entries (18 and 8 pages) on top of a sparse random graph: the per-vertex
    kernels walk such lists in pieces, a wave each; levels and labels must not notice.  The hubs sit in
    different components until an edge of the random part joins them."""
    n_v = 20000
    pu = np.empty(6000, dtype=np.uint64); pv = np.empty(6000, dtype=np.uint64)
    oracle.lib().bo_uniform_edges(SEED, n_v, 0, 6000, pu, pv)
    hub_a = np.full(9000, 7, dtype=np.uint64); leaves_a = np.arange(100, 9100, dtype=np.uint64)
    hub_b = np.full(4096, 15000, dtype=np.uint64); leaves_b = np.arange(9100, 9100 + 4096, dtype=np.uint64)
    off, nb = oracle.csr_from_pairs(n_v, np.concatenate([pu, hub_a, hub_b]), np.concatenate([pv, leaves_a, leaves_b]))
    deg = np.diff(off.astype(np.int64))
    assert deg[7] >= 9000 and deg[15000] >= 4096
    r, a = _graph_rig(bam, nb, cache_pages, n_queues=8, depth=256)
    with r:
        doff = _dev(off)
        for src in (7, 15000, 100, int(oracle.bfs_sources(SEED, off, 1)[0])):
            lv, it = a.bfs(doff, src, coarse=coarse)
            want, want_it = oracle.bfs_levels(off, nb, src)
            assert np.array_equal(lv.cpu().numpy().view(np.uint32), want) and it == want_it
            lv, it = a.bfs(doff, src, frontier=True)
            assert np.array_equal(lv.cpu().numpy().view(np.uint32), want) and it == want_it
        lb, _ = a.cc(doff, coarse=coarse)
        assert np.array_equal(_u64(lb), oracle.cc_labels(off, nb)[0])
        # PageRank pushes over the same lists (tolerance as in test_pagerank_values)
        x = oracle.pagerank_limit(off, nb, 0.85)
        v, it = a.pagerank(doff, 0.85, 1e-3, 1000)
        v = v.cpu().numpy().astype(np.float64)
        assert 1 < it < 1000 and np.all(v <= x * (1 + 1e-5)) and np.all(v >= x * (1 - 1e-3 / 0.15 - 1e-5))
        assert not r.c.aborted()


@pytest.mark.parametrize("empty_every", [0, 4, 2])
def test_lists_that_all_cross_a_page_boundary(bam, empty_every):
    """every list has 600 entries (a page holds 512), so each one ends on another page than it starts on, and every
    `empty_every`-th vertex has none: the read-ahead of a group asks for the last pages on the lanes that have no first
    page to ask for, and for the rest in a second batch (none empty: all in the second batch; every second one empty:
    all in the first).  Neighbours are the next 600 vertices, so the levels step through the graph."""
    n_v, d = 4096, 600
    deg = np.full(n_v, d, dtype=np.uint64)
    if empty_every:
        deg[empty_every - 1::empty_every] = 0
    off = np.concatenate([[0], np.cumsum(deg)]).astype(np.uint64)
    owner = np.repeat(np.arange(n_v, dtype=np.uint64), deg.astype(np.int64))
    nb = (owner + 1 + (np.arange(len(owner), dtype=np.uint64) - off[owner])) % np.uint64(n_v)
    r, a = _graph_rig(bam, nb, 256, n_queues=8, depth=256)
    with r:
        doff = _dev(off)
        for src in (0, 1000, 4092):
            want, want_it = oracle.bfs_levels(off, nb, src)
            assert want_it >= 6
            for kw in (dict(coarse=1), dict(coarse=64), dict(frontier=True)):
                lv, it = a.bfs(doff, src, **kw)
                assert np.array_equal(lv.cpu().numpy().view(np.uint32), want) and it == want_it
        assert a.stats()["read_io_cnt"] > len(nb) // 512 and not r.c.aborted()


@pytest.mark.parametrize("scale,cache_pages", [(10, 2048), (13, 160)])
def test_sssp_costs_two_arrays_in_one_cache(bam, scale, cache_pages):
    """neighbour ids (64-bit) and weights (32-bit) as two arrays behind one page cache; costs against Dijkstra"""
    off, nb = oracle.rmat_csr(SEED, scale)
    w = oracle.edge_weights(SEED, len(nb))
    e_pages = (len(nb) * 8 + 4095) // 4096
    w_pages = (len(w) * 4 + 4095) // 4096
    with Rig(bam, (e_pages + w_pages + 1) * 4096, backing=True, n_queues=8, depth=256) as r:
        store = r.backing((e_pages + w_pages + 1) * 512)
        store[:len(nb)] = nb
        store[e_pages * 512:].view(np.uint32)[:len(w)] = w
        pc = bam.PageCache(4096, cache_pages, 0, r.c)
        re_ = bam.Range(0, len(nb), 0, e_pages, 0, 4096, pc, 0)
        rw = bam.Range32(0, len(w), e_pages, w_pages, 0, 4096, pc, 0)
        edges = bam.Array(len(nb), 0, [re_], 0)
        weights = bam.Array32(len(w), e_pages * 4096, [rw], 0)
        # the 32-bit array by itself first
        assert weights.read(len(w)) == int(np.sum(w, dtype=np.uint64))
        assert weights.read(1000, stride=7, block_size=128) == int(np.sum(w[:7000:7], dtype=np.uint64))
        ws = weights.stats()
        assert ws["access_cnt"] == len(w) + 1000 and ws["read_io_cnt"] >= w_pages
        doff = _dev(off)
        for src in oracle.bfs_sources(SEED, off, 3):
            costs, rounds = bam.sssp(edges, weights, doff, int(src))
            assert np.array_equal(costs.cpu().numpy().view(np.uint32), oracle.sssp_costs(off, nb, w, int(src))) and rounds >= 2
        assert edges.stats()["read_io_cnt"] > 0 and weights.stats()["access_cnt"] > 0 and not r.c.aborted()
        edges.close(); weights.close(); re_.close(); rw.close(); pc.close()


@pytest.mark.parametrize("scale,cache_pages", [(10, 2048), (13, 160)])
def test_sssp_float_costs(bam, scale, cache_pages):
    """benchmarks/sssp_float: single-precision weights whose sums round; costs must equal the serial Dijkstra in single
    precision to the bit (adding a weight keeps the order of two costs, so the order of relaxation does not matter)"""
    off, nb = oracle.rmat_csr(SEED, scale)
    w = oracle.edge_weights(SEED, len(nb)).astype(np.float32) * np.float32(0.37) + np.float32(1e-3)
    e_pages = (len(nb) * 8 + 4095) // 4096
    w_pages = (len(w) * 4 + 4095) // 4096
    with Rig(bam, (e_pages + w_pages + 1) * 4096, backing=True, n_queues=8, depth=256) as r:
        store = r.backing((e_pages + w_pages + 1) * 512)
        store[:len(nb)] = nb
        store[e_pages * 512:].view(np.float32)[:len(w)] = w
        pc = bam.PageCache(4096, cache_pages, 0, r.c)
        re_ = bam.Range(0, len(nb), 0, e_pages, 0, 4096, pc, 0)
        rw = bam.Range32(0, len(w), e_pages, w_pages, 0, 4096, pc, 0)
        edges = bam.Array(len(nb), 0, [re_], 0)
        weights = bam.Array32(len(w), e_pages * 4096, [rw], 0)
        doff = _dev(off)
        for src in oracle.bfs_sources(SEED, off, 3):
            costs, rounds = bam.sssp_float(edges, weights, doff, int(src))
            want = oracle.sssp_costs_float(off, nb, w, int(src))
            assert np.array_equal(costs.cpu().numpy().view(np.uint32), want.view(np.uint32)) and rounds >= 2
            assert np.any(want == np.float32(1e9)) or scale > 10        # unreached vertices are part of the case where there are any
        assert edges.stats()["read_io_cnt"] > 0 and weights.stats()["access_cnt"] > 0 and not r.c.aborted()
        edges.close(); weights.close(); re_.close(); rw.close(); pc.close()


@pytest.mark.parametrize("scale,cache_pages", [(10, 4096), (14, 24), (16, 8192), (17, 700)])
@pytest.mark.parametrize("sort", ["1", "0"])
def test_bfs_levels_rmat_by_queue_of_vertices(bam, scale, cache_pages, sort, monkeypatch):
    """the kernel that walks a queue of the level's vertices: same levels, same launch count, whether the queue is
    sorted between levels (the default) or walked in the order of discovery"""
    monkeypatch.setenv("BAM_FRONTIER_SORT", sort)
    off, nb = oracle.rmat_csr(SEED, scale)
    r, a = _graph_rig(bam, nb, cache_pages, n_queues=16, depth=256)
    with r:
        doff = _dev(off)
        for src in list(oracle.bfs_sources(SEED, off, 3)) + [int(np.flatnonzero(np.diff(off) == 0)[0])]:
            lv, it = a.bfs(doff, int(src), frontier=True)
            ref, rit = oracle.bfs_levels(off, nb, int(src))
            assert np.array_equal(lv.cpu().numpy().view(np.uint32), ref) and it == rit
        assert a.stats()["read_io_cnt"] > 0 and not r.c.aborted()


@pytest.mark.parametrize("scale,cache_pages,tol", [(10, 2048, 1e-3), (13, 96, 1e-3), (14, 512, 1e-4)])
@pytest.mark.parametrize("by_page", [False, True])
def test_pagerank_values(bam, scale, cache_pages, tol, by_page):
    """benchmarks/pagerank, single precision with atomic float adds in no fixed order (as in the reference), so no two
    runs need agree bit for bit.  Tolerance, stated: with x the exact solution (double-precision limit of the pushes),
    every value must satisfy x (1 - tol / (1 - alpha)) - 1e-5 x <= value <= x + 1e-5 x (what is left unpushed is at most
    `tol` per vertex; 1e-5 x covers float rounding of a few hundred adds), and therefore lies within
    x tol / (1 - alpha) + 2e-5 x of the oracle's serial run of the same algorithm."""
    alpha = 0.85
    off, nb = oracle.rmat_csr(SEED, scale)
    x = oracle.pagerank_limit(off, nb, alpha)
    want, want_it = oracle.pagerank(off, nb, alpha, tol, 1000)
    r, a = _graph_rig(bam, nb, cache_pages, n_queues=16, depth=256)
    with r:
        v, it = a.pagerank(_dev(off), alpha, tol, 1000, by_page=by_page)
        v = v.cpu().numpy().astype(np.float64)
        assert 1 < it < 1000 and abs(it - want_it) <= 3
        assert np.all(v <= x * (1 + 1e-5)) and np.all(v >= x * (1 - tol / (1 - alpha) - 1e-5))
        assert np.all(np.abs(v - want) <= x * (tol / (1 - alpha) + 2e-5))
        deg = np.diff(off.astype(np.int64))
        assert np.all(v[deg == 0] == np.float32(1) - np.float32(alpha))
        # a capped run stops at the cap
        v1, it1 = a.pagerank(_dev(off), alpha, tol, 1, by_page=by_page)
        w1, _ = oracle.pagerank(off, nb, alpha, tol, 1)
        assert it1 == 1 and np.allclose(v1.cpu().numpy(), w1, rtol=1e-5)
        assert a.stats()["read_io_cnt"] > 0 and not r.c.aborted()


# ---------------------------------------------------------------- dataset placement (readwrite) and graph files

def test_graph_file_to_store_then_traverse(bam, tmp_path):
    """.bel pair on disk -> payload of .dst written to the store at a page-aligned offset through the cache slots ->
    BFS and CC over an array that starts at that offset -> the store read back into a file"""
    from bam_amd import bel
    off, nb = oracle.rmat_csr(SEED, 12)
    prefix = str(tmp_path / "rmat12.bel")
    bel.write(prefix, off, nb)
    n_off, n_e = bel.info(prefix)
    assert n_off == len(off) and n_e == len(nb)
    loffset = 3 << 20                                           # --loffset of the reference's graph benchmarks
    ns_bytes = 16 << 20
    with Rig(bam, ns_bytes, backing=True, n_queues=8, depth=256) as r:
        store = r.backing(ns_bytes // 8)
        store[:] = 0x5a5a5a5a5a5a5a5a
        loader = bam.PageCache(4096, 100, 0, r.c)              # smaller than the file: several passes, ragged last page
        assert loader.write_file(prefix + ".dst", file_offset=bel.HEADER_BYTES, store_offset=loffset) == n_e * 8
        first = loffset // 8
        assert np.array_equal(store[first:first + n_e], nb)
        pad = (-n_e) % 512
        assert not store[first + n_e:first + n_e + pad].any() and store[first + n_e + pad] == 0x5a5a5a5a5a5a5a5a and store[first - 1] == 0x5a5a5a5a5a5a5a5a
        back = str(tmp_path / "back.bin")
        loader.read_file(back, loffset, n_e * 8)
        assert np.array_equal(np.fromfile(back, dtype=np.uint64), nb)
        with pytest.raises(Exception):
            loader.write_file(prefix + ".dst", file_offset=16, store_offset=loffset + 512)      # not page aligned
        with pytest.raises(Exception):
            loader.write_file(prefix + ".dst", file_offset=16, store_offset=ns_bytes - 4096)    # past the end
        loader.close()
        a = r.array(n_e, 4096, 64, disk_offset=loffset)
        doff = _dev(bel.read_offsets(prefix))
        for by_page in (False, True):
            for src in oracle.bfs_sources(SEED, off, 2):
                lv, it = a.bfs(doff, int(src), coarse=2, by_page=by_page)
                ref, rit = oracle.bfs_levels(off, nb, int(src))
                assert np.array_equal(lv.cpu().numpy().view(np.uint32), ref) and it == rit
            lb, _ = a.cc(doff, coarse=2, by_page=by_page)
            assert np.array_equal(_u64(lb), oracle.cc_labels(off, nb)[0])
        assert r.t.stats()["write_cmds"] == (n_e * 8 + 4095) // 4096 and not r.c.aborted()



# ---------------------------------------------------------------- read-modify-write routes

def _check_add_chains(x0, idx, vals, olds, final):
    """Every element that received adds v_1..v_k (in whatever order the device applied them) must show that order in what
    the adds returned: sorted by (old - x0), the returned values are x0, x0 + v_a, x0 + v_a + v_b, ... and the element
    ends at x0 + sum(v).  The steps between consecutive returned values (and from the last one to the final value) are
    therefore a permutation of the values added."""
    order = np.argsort(idx, kind="stable")
    idx_s, vals_s, olds_s = idx[order], vals[order], olds[order]
    starts = np.flatnonzero(np.r_[True, idx_s[1:] != idx_s[:-1]])
    ends = np.r_[starts[1:], len(idx_s)]
    for a, b in zip(starts, ends):
        e = int(idx_s[a])
        d = np.sort((olds_s[a:b] - x0[e]).astype(np.uint64))           # mod 2^64
        steps = np.diff(np.r_[d, (final[e] - x0[e]).astype(np.uint64)])
        assert d[0] == 0, "element %d: no add saw the initial value" % e
        assert np.array_equal(np.sort(steps), np.sort(vals_s[a:b])), "element %d: returned values do not chain" % e


@pytest.mark.parametrize("api,cache_pages,block", [(0, 24, 64), (0, 300, 256), (1, 4096, 64)])
def test_atomic_add_on_scattered_and_colliding_elements(bam, api, cache_pages, block):
    """array_d_t::AtomicAdd (reference include/page_cache.h:1647) and atomics on the address bam_ptr::memref hands out (:467):
    several launches of adds to elements drawn from a small hot set (many lanes of a launch on one element) and from all
    over the array, through a cache smaller than what is touched, so dirty pages are evicted, written back and read again
    between the adds.  A numpy array plays the store; the values returned must chain (see above)."""
    n_elems, n = 1 << 23, 2048                                       # 16384 pages of data; 2048 adds per launch
    rng = np.random.default_rng(SEED + api)
    with Rig(bam, n_elems * 8, backing=True, n_queues=8, depth=256) as r:
        x0 = r.backing(n_elems).copy()
        model = x0.copy()
        a = r.array(n_elems, 4096, cache_pages)
        hot = rng.integers(0, n_elems, 64).astype(np.uint64)
        all_idx, all_val, all_old = [], [], []
        for launch in range(5):
            idx = np.where(rng.random(n) < 0.5, hot[rng.integers(0, len(hot), n)], rng.integers(0, n_elems, n).astype(np.uint64)).astype(np.uint64)
            vals = rng.integers(1, 1 << 20, n).astype(np.uint64)
            old = _u64(a.update(api, _dev(idx), _dev(vals), block_size=block))
            np.add.at(model, idx.astype(np.int64), vals)
            all_idx.append(idx); all_val.append(vals); all_old.append(old)
        r.objs[0][2].flush()
        final = r.backing(n_elems)
        assert np.array_equal(final, model)
        _check_add_chains(x0, np.concatenate(all_idx), np.concatenate(all_val), np.concatenate(all_old), final)
        idx = np.concatenate(all_idx)
        assert a.read(len(idx), _dev(idx), block_size=64) == int(np.sum(model[idx.astype(np.int64)], dtype=np.uint64))
        ts = r.t.stats()
        assert ts["write_cmds"] > 0 and not r.c.aborted() and r.c.info()["error_completions"] == 0


def test_add_assign_through_a_bam_ptr_lvalue(bam):
    """ptr[i] += v on a non-const bam_ptr (reference include/page_cache.h:478: operator[] as an lvalue marks the page
    dirty): distinct elements per launch, several launches over the same elements, a cache smaller than what they touch"""
    n_elems, n = 1 << 23, 2048
    rng = np.random.default_rng(SEED)
    with Rig(bam, n_elems * 8, backing=True, n_queues=8, depth=256) as r:
        model = r.backing(n_elems).copy()
        a = r.array(n_elems, 4096, 4096)
        for launch in range(6):
            idx = rng.permutation(n_elems)[:n].astype(np.uint64)
            if launch % 2:
                idx[: n // 2] = prev[: n // 2]                         # half of them again: read back what the last launch wrote
                idx = np.unique(idx)
            vals = rng.integers(0, 1 << 63, len(idx)).astype(np.uint64)
            old = _u64(a.update(2, _dev(idx), _dev(vals), block_size=64))
            assert np.array_equal(old, model[idx.astype(np.int64)]), "launch %d" % launch
            model[idx.astype(np.int64)] += vals
            prev = idx
        r.objs[0][2].flush()
        assert np.array_equal(r.backing(n_elems), model)
        assert r.t.stats()["write_cmds"] > 0 and not r.c.aborted()


def _seal_value(dw, ticket):
    """nvm_cmd_seal_value restated: a multiplicative hash over the dwords of the entry except CDW3, keyed by the ticket"""
    M = 0xFFFFFFFF
    h = (ticket * 0x9E3779B1 + 0x7F4A7C15) & M
    for i in range(16):
        if i == 3:
            continue
        h = ((h ^ int(dw[i])) * 0x85EBCA6B) & M
        h ^= h >> 13
    return h | 1


@pytest.mark.parametrize("opcode", [0x02, 0x01])
def test_submission_entries_built_on_the_device_match_the_nvme_layout(bam, opcode):
    """the product's encoders (include/nvm_cmd.h; reference include/nvm_cmd.h:54-88), compiled for the host and for gfx950,
    against the oracle's independent encoder and the NVMe byte layout; then sealed, against a restatement of the seal"""
    import torch
    L = bam.load()
    cid, nsid, prp1, prp2, lba, nblk, ticket = 0xBE00, 1, 0x1122334455667000, 0xAABBCCDD00112000, 0x0123456789ABCD00, 8, 0xFFFFFFF0
    for seal in (0, 1):
        host = (ctypes.c_uint32 * 16)()
        dev = torch.zeros(64 * 16, dtype=torch.int32, device="cuda")
        assert L.bam_sqe_image(cid, opcode, nsid, prp1, prp2, lba, nblk, seal, ticket, host, ctypes.c_void_p(dev.data_ptr()), None) == 0
        torch.cuda.synchronize()
        d = dev.cpu().numpy().view(np.uint32).reshape(64, 16)
        for lane in range(64):
            want = np.zeros(16, dtype=np.uint32)
            oracle.lib().bo_cmd_rw(want, cid + lane, opcode, nsid, prp1, prp2, lba + lane, nblk)
            if seal:
                want[2] = (ticket + lane) & 0xFFFFFFFF               # the ticket wraps within the wave
                want[3] = _seal_value(want, int(want[2]))
            assert np.array_equal(d[lane], want), "lane %d seal %d" % (lane, seal)
        assert np.array_equal(np.frombuffer(host, dtype=np.uint32), d[0])
        if not seal:
            b = d[0].tobytes()
            assert b[0] == opcode and b[1] == 0 and b[2:4] == bytes([0x00, 0xBE]) and b[4:8] == (1).to_bytes(4, "little")
            assert b[8:24] == bytes(16) and b[24:32] == prp1.to_bytes(8, "little") and b[32:40] == prp2.to_bytes(8, "little")
            assert b[40:48] == lba.to_bytes(8, "little") and b[48:50] == (7).to_bytes(2, "little") and b[50:64] == bytes(14)


# ---------------------------------------------------------------- queue policies: ring placement, unsealed entries

@pytest.mark.parametrize("place", ["host", "device"])
@pytest.mark.parametrize("order,depth", [(0, 256), (2, 16), (1, 64)])
def test_completion_ring_placement(bam, place, order, depth, monkeypatch):
    """completion rings in host-pinned memory or in device memory (written by the controller across the interconnect):
    in-order, shuffled and reversed completions, queues so shallow that the completion ring fills up"""
    from bam_amd import gen
    monkeypatch.setenv("BAM_CQ_PLACE", place)
    n_elems, n = 1 << 22, 1 << 18
    with Rig(bam, 64 << 20, n_queues=4, depth=depth, order=order) as r:
        a = r.array(n_elems, 4096, 1024)
        idx = gen.gather_indices(SEED, n, n_elems)
        assert a.read(n, idx, block_size=128) == oracle.lib().bo_gather_sum(SEED, SEED, 0, n, n_elems)
        st, ts = a.stats(), r.t.stats()
        assert st["access_cnt"] == n and st["read_io_cnt"] == ts["read_cmds"] > 0
        assert not r.c.aborted() and r.c.info()["error_completions"] == 0 and ts["error_cpls"] == 0
    ns = 1 << 30
    with Rig(bam, ns, n_queues=2, depth=depth, order=order) as r:                 # raw block reads, far more commands than ring entries
        nb = 1 << 14
        pc = bam.PageCache(4096, nb, 0, r.c)
        lbas = gen.block_lbas(SEED, nb, ns, 4096, 512)
        pc.block_io(nb, 4096, lbas)
        ref = np.array([oracle.lib().bo_block_checksum(SEED, int(x), 512, 4096) for x in _u64(lbas)], dtype=np.uint64)
        assert np.array_equal(_u64(pc.block_checksums(nb, 4096)), ref) and not r.c.aborted()
        pc.close()


@pytest.mark.parametrize("seal,flush", [("0", "2"), ("0", "1"), ("1", "0"), ("1", "2")])
def test_submission_entries_sealed_and_unsealed(bam, seal, flush, monkeypatch):
    """Submission queues as the NVMe specification has them (no seal in the entries, what a real controller needs; the
    default), with each of the two ways a submitter has of knowing that its entry arrived before a doorbell covers it
    (2 read the entry back, 1 system-scope release), and sealed (the target verifies a ticket and a checksum in the entry
    and reads it again if they do not hold, so the submitter need not know: the wave's store counter alone, 0, will do;
    on an unsealed queue 0 is not offered, the controller turns it into 2).  Checksum, no error completions, no wait
    given up; the target's counters say what it saw."""
    from bam_amd import gen
    monkeypatch.setenv("BAM_SQ_SEAL", seal)
    monkeypatch.setenv("BAM_SQ_FLUSH", flush)
    n_elems, n = 1 << 24, 1 << 20
    with Rig(bam, n_elems * 8, n_queues=32, depth=256, io_threads=8) as r:
        a = r.array(n_elems, 4096, 8192)
        for rep in range(3):
            idx = gen.gather_indices(SEED + rep, n, n_elems)
            assert a.read(n, idx, block_size=256) == oracle.lib().bo_gather_sum(SEED, SEED + rep, 0, n, n_elems)
        ts = r.t.stats()
        print("seal %s, flush %s: %d commands, %d doorbells, %d stale doorbells, %d entry retries" % (seal, flush, ts["read_cmds"], ts["sq_doorbells"], ts["stale_doorbells"], ts["sqe_retries"]))
        if seal == "0":
            assert ts["sqe_retries"] == 0                                 # nothing is verified on an unsealed queue
        assert not r.c.aborted() and r.c.info()["error_completions"] == 0 and ts["error_cpls"] == 0

# ---------------------------------------------------------------- failure handling

def test_lost_completion_ends_the_kernel_with_the_abort_flag(bam):
    """the target swallows one command in 500; the waits are bounded, so the launch returns and says so"""
    with Rig(bam, 16 << 20, drop_every=500, limit=300_000) as r:
        a = r.array(1 << 20, 4096, 4096)
        a.read(1 << 18, block_size=64)
        assert r.c.aborted() and r.t.stats()["dropped"] >= 1
        assert r.c.aborted(clear=True) and not r.c.aborted()


@pytest.mark.parametrize("api", [1, 2, 3, 4, 5, 6, 7])
def test_lost_completion_through_every_access_route(bam, api):
    """the same through get_raw, acquire_page_, acquire_page, bam_ptr, the wave memcpy, bam_ptr_tlb and bafs_ptr: a route
    whose wait was given up hands out no address (NULL, an empty window, T()), its kernel reads nothing through it and
    ends, and the flag is up"""
    with Rig(bam, 16 << 20, drop_every=200, limit=300_000) as r:
        a = r.array(1 << 20, 4096, 4096)
        if api == 5:
            a.read_via(5, 1 << 11, span=512, block_size=64)
        else:
            a.read_via(api, 1 << 17, span=8, block_size=64)
        assert r.c.aborted() and r.t.stats()["dropped"] >= 1


@pytest.mark.parametrize("kernel", [dict(coarse=4), dict(frontier=True), dict(by_page=True)])
def test_lost_completion_during_a_graph_traversal(bam, kernel):
    """the same while edge lists are being read, where what is read is used as an index: the sweep ends, the flag says
    that the levels are not to be used, and neighbour ids that never arrived stay inside the label array (a read
    through bam_ptr gives 0 after a wait that was given up; a page declared valid without its payload holds what the
    slot or the staging page held before, which is other neighbour ids, so the padding behind the last list is zeroed
    here as a loader would)"""
    off, nb = oracle.rmat_csr(SEED, 13)
    pad = (-len(nb)) % 512
    with Rig(bam, (len(nb) + pad) * 8, backing=True, n_queues=8, depth=256, drop_every=300, limit=300_000) as r:
        store = r.backing(len(nb) + pad)
        store[:len(nb)] = nb
        store[len(nb):] = 0
        a = r.array(len(nb), 4096, 64)
        lv, it = a.bfs(_dev(off), int(oracle.bfs_sources(SEED, off, 1)[0]), **kernel)
        assert r.c.aborted() and r.t.stats()["dropped"] >= 1 and it >= 1
        lv = lv.cpu().numpy().view(np.uint32)
        assert np.all((lv == 0xFFFFFFFF) | (lv <= it))


def test_error_completions_are_counted(bam):
    """one command in 100 completes with an error status: its page is not shown as valid with whatever the slot held,
    the read is issued again, and the sum comes out right"""
    n = 1 << 18
    with Rig(bam, 16 << 20, fail_every=100) as r:
        a = r.array(1 << 20, 4096, 4096)
        assert a.read(n, block_size=64) == oracle.lib().bo_store_sum(SEED, 0, 1, n)
        assert not r.c.aborted()
        ts = r.t.stats()
        assert r.c.info()["error_completions"] == ts["error_cpls"] > 0
        assert a.stats()["read_io_cnt"] == ts["read_cmds"] + ts["error_cpls"] == n // 512 + ts["error_cpls"]


# ---------------------------------------------------------------- full size (config 2)

def test_config2_full_size_gather(bam):
    """2^28 u64 behind a 1 GiB cache, 2^26 uniform reads, one thread per read: checksum against the closed form"""
    from bam_amd import gen
    n_elems, n = 1 << 28, 1 << 26
    with Rig(bam, n_elems * 8, n_queues=128, depth=1024, io_threads=12) as r:
        a = r.array(n_elems, 4096, 1 << 18)
        idx = gen.gather_indices(SEED, n, n_elems)
        assert a.read(n, idx, block_size=256) == oracle.lib().bo_gather_sum(SEED, SEED, 0, n, n_elems)
        st = a.stats()
        assert st["access_cnt"] == n and st["hit_cnt"] + st["miss_cnt"] == n
        # a page can be fetched at most once per distinct wave-level miss: between #distinct pages and #misses
        assert (1 << 18) < st["read_io_cnt"] <= st["miss_cnt"]
        assert not r.c.aborted() and r.c.info()["error_completions"] == 0
