"""CPU restatement of the reference's page cache + queue protocol, against closed forms and invariants."""
import json
import os

import numpy as np
import pytest

import oracle

G = os.path.join(os.path.dirname(__file__), "golden")
SEED = 42


def test_config1_reduction_matches_closed_form():
    """2^24 u64 in a 128 MiB store, 4 KiB pages, 64 MiB cache, stride-8 reads summed mod 2^64 (the CPU reference run)."""
    with open(os.path.join(G, "splitmix64.json")) as f:
        g = json.load(f)
    for seed in (0, 42):
        p = oracle.CpuPath(128 << 20, 1 << 24, 4096, 16384, seed=seed, n_io_threads=2, n_queues=4, queue_depth=256)
        s = p.array_sum(1 << 21, stride=8, n_threads=4)
        st = p.stats()
        assert s == int(g["cfg1_stride8_sum_2p21"][str(seed)], 16)
        # every page is touched by 64 consecutive reads; the cache holds half of the pages
        assert st["access_cnt"] == 1 << 21
        assert st["read_io_cnt"] >= 32768 and st["read_io_cnt"] < 32768 + 4096
        assert st["hit_cnt"] + st["miss_cnt"] == st["access_cnt"]
        assert p.check() == 0
        p.close()


def test_counter_invariants_without_eviction():
    """read I/Os = distinct pages first touched, accesses = lane accesses (reference logs, width independent)."""
    p = oracle.CpuPath(16 << 20, 1 << 20, 4096, 4096, n_queues=2, queue_depth=16)
    n = 1 << 18
    s = p.array_sum(n, stride=1, n_threads=4)
    st = p.stats()
    assert s == oracle.lib().bo_store_sum(SEED, 0, 1, n)
    assert st["read_io_cnt"] == n // 512 and st["access_cnt"] == n
    s = p.array_sum(n, stride=1, n_threads=3)           # second pass: all hits
    st = p.stats()
    assert s == oracle.lib().bo_store_sum(SEED, 0, 1, n)
    assert st["read_io_cnt"] == 0 and st["hit_cnt"] == n and st["miss_cnt"] == 0
    assert p.check() == 0
    p.close()


@pytest.mark.parametrize("cache_pages,queue_depth,n_threads", [(2, 2, 4), (4, 4, 8), (3, 8, 5), (64, 2, 6)])
def test_tiny_caches_and_queues_random_gather(cache_pages, queue_depth, n_threads):
    """brute force on tiny resources: heavy eviction, full queues, wrap-around of every ring many times over"""
    n_elems = 1 << 14
    p = oracle.CpuPath(1 << 20, n_elems, 4096, cache_pages, n_queues=2, queue_depth=queue_depth, n_io_threads=1)
    idx = oracle.gather_indices(SEED, 0, 6000, n_elems)
    s = p.array_sum(len(idx), idx, n_threads=n_threads)
    assert s == oracle.lib().bo_gather_sum(SEED, SEED, 0, len(idx), n_elems)
    st = p.stats()
    assert st["access_cnt"] == len(idx) and st["hit_cnt"] + st["miss_cnt"] == len(idx)
    assert p.check() == 0
    p.close()


def test_memory_backed_store_and_disk_offset():
    data = np.arange(1 << 16, dtype=np.uint64) * np.uint64(2654435761)
    p = oracle.CpuPath(data.nbytes, (1 << 16) - 1024, 4096, 8, backing=data, disk_offset_bytes=8192, n_queues=1, queue_depth=8)
    idx = oracle.gather_indices(7, 0, 3000, (1 << 16) - 1024)
    s = p.array_sum(len(idx), idx, n_threads=4)
    assert s == int(np.sum(data[idx.astype(np.int64) + 1024], dtype=np.uint64))
    p.close()


@pytest.mark.parametrize("req_bytes,lba", [(4096, 512), (512, 512), (4096, 4096)])
def test_block_reads_checksums(req_bytes, lba):
    p = oracle.CpuPath(1 << 30, 8, 4096, 2, lba_bytes=lba, n_queues=3, queue_depth=32)
    lbas = oracle.block_lbas(SEED, 0, 2000, 1 << 30, req_bytes, lba)
    cs = p.block_reads(lbas, req_bytes, n_threads=6)
    ref = np.array([oracle.lib().bo_block_checksum(SEED, int(x), lba, req_bytes) for x in lbas], dtype=np.uint64)
    assert np.array_equal(cs, ref)
    p.close()


def test_bfs_and_cc_through_the_cache():
    off, nb = oracle.rmat_csr(SEED, 10)
    pad = (-len(nb)) % 512
    store = np.concatenate([nb, np.zeros(pad, dtype=np.uint64)])
    p = oracle.CpuPath(store.nbytes, len(nb), 4096, 16, backing=store, n_queues=2, queue_depth=16)
    for src in oracle.bfs_sources(SEED, off, 3):
        lv, it = p.bfs(off, src, n_threads=4)
        ref, rit = oracle.bfs_levels(off, nb, src)
        assert np.array_equal(lv, ref) and it == rit
    lb, it = p.cc(off, n_threads=4)
    ref, comps = oracle.cc_labels(off, nb)
    assert np.array_equal(lb, ref)
    assert p.check() == 0
    p.close()


def test_sample_graph_through_the_cache():
    with open(os.path.join(G, "sample_graph.json")) as f:
        g = json.load(f)
    off = np.array(g["offsets"], dtype=np.uint64)
    nb = np.array(g["edges"] + [0] * (512 - len(g["edges"])), dtype=np.uint64)
    p = oracle.CpuPath(nb.nbytes, len(g["edges"]), 4096, 2, backing=nb, n_queues=1, queue_depth=4)
    for src, exp in g["bfs"].items():
        lv, it = p.bfs(off, int(src), n_threads=3)
        assert lv.tolist() == exp["levels"] and it == exp["iterations"]
    lb, _ = p.cc(off, n_threads=3)
    assert lb.tolist() == g["cc"]["labels"]
    p.close()
