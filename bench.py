#!/usr/bin/env python3
"""Benchmark of the GPU-side storage-access path on one MI355X.

A step is one launch of the random-gather array benchmark: 2^26 element reads,
one thread per read (the reference's kernel as it is), at uniform-random indices
into a 2^28-element u64 array (2 GiB store) behind a 1 GiB page cache with 4 KiB
pages, the store being the software NVMe target.  The index tensors are generated
and resident in HBM before the timed region.  `value` is 4 KiB read I/Os per
second over the timed steps.  On the same JSON line:

  two_launches  the same steps the way bam_array_read runs a launch of this size by
                default: a first launch reads what is resident, a second the rest
  roofline      the hit-path streaming kernel of the reference's shape (a wave per
                run of pages, every element through bam_ptr) over the resident 1 GiB
                cache (HBM bound), timed with HIP events on its stream; the
                page-wise kernel alongside
  cpu_baseline  the CPU restatement of the reference path (oracle/cpu_path.c)
                on a bounded sample of the same workload, on the host cores
  store         what the backing store can do: the target's service rate with
                plain host clients and the rate at which payload crosses the
                interconnect to the GPU, both measured in this run; the
                ceiling is the slower of the two
  block         raw block benchmark (2^22 reads, 128 queue pairs x 1024)
  bfs           RMAT-24 BFS through the page cache (with --bfs-scale): the edge-page kernel and the reference-shaped one
  cc            connected components of a 2^26-vertex uniform graph, 16 GiB of edges behind an 8 GiB cache (with --cc-logv)

Everything is checked against the closed-form oracle while it is measured.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

SEED = 42
N_ELEMS = 1 << 28
CACHE_PAGES = 1 << 18
PAGE = 4096
N_READS = 1 << 26
HBM_PEAK_GBS = 8000.0
PCIE_GEN5_X16_GBPS = 64.0       # what the link between host memory and the GPU carries one way, before protocol overhead
STREAM_PAGES_PER_WAVE = 16      # pages per wave of the streaming kernels (one acquire batch of the page-wise one)
# HBM bytes one launch of a streaming kernel moves over the 1 GiB cache, from the profiler's FETCH_SIZE and WRITE_SIZE
# counters scaled by what they read for a plain 1 GiB copy; figures, commands and date in the files named.  They hold for
# this workload and the tree state the profile was taken on, which is why the source is printed beside them.
HIT_TRAFFIC = {
    "bam_ptr": {"bytes": 1078487040, "source": "profiles/k_cache_stream_hit_path_1GiB_cache.md"},
    "page_wise": {"bytes": 1079590912, "source": "profiles/k_cache_stream_hit_path_1GiB_cache.md"},
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def splitmix_block_sums(torch, seed, first_word, n_words):
    """sum over k < n_words of splitmix64(seed, first_word + k) (mod 2^64) for a tensor of first words, in int64 tensor
    arithmetic: word i of the procedural store is mix64(seed + (i + 1) * 0x9E3779B97F4A7C15) with the published finalizer"""
    def s64(x):
        x &= (1 << 64) - 1
        return x - (1 << 64) if x >> 63 else x
    gamma, c1, c2 = s64(0x9E3779B97F4A7C15), s64(0xBF58476D1CE4E5B9), s64(0x94D049BB133111EB)
    def lsr(z, k):
        return (z >> k) & ((1 << (64 - k)) - 1)
    acc = torch.zeros_like(first_word)
    for k in range(n_words):
        z = (first_word + (k + 1)) * gamma + s64(seed)
        z = (z ^ lsr(z, 30)) * c1
        z = (z ^ lsr(z, 27)) * c2
        acc += z ^ lsr(z, 31)
    return acc


def usable_cores():
    """the cores this process may use: what the scheduler allows it, capped by the share the environment names (a GPU box
    exports the share of its one GPU as OMP_NUM_THREADS while os.cpu_count() shows the whole machine)"""
    try:
        n = len(os.sched_getaffinity(0))
    except AttributeError:
        n = os.cpu_count() or 1
    share = os.environ.get("OMP_NUM_THREADS", "")
    if share.isdigit() and int(share) > 0:
        n = min(n, int(share))
    return max(n, 2)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--io-threads", type=int, default=12, help="service threads of the software NVMe target")
    ap.add_argument("--queues", type=int, default=128)
    ap.add_argument("--depth", type=int, default=1024)
    ap.add_argument("--block", type=int, default=256, help="threads per block of the gather kernel")
    ap.add_argument("--cpu-reads", type=int, default=1 << 26, help="size of the CPU-baseline sample (element reads)")
    ap.add_argument("--cpu-threads", type=int, default=0, help="threads of the CPU legs, lanes and target together (0 = every core this process may use)")
    ap.add_argument("--bfs-scale", type=int, default=24, help="RMAT scale of the BFS leg (0 = skip)")
    ap.add_argument("--bfs-sources", type=int, default=8)
    ap.add_argument("--cc-logv", type=int, default=26, help="log2 of the vertex count of the connected-components leg (0 = skip)")
    ap.add_argument("--skip-cpu", action="store_true")
    ap.add_argument("--skip-block", action="store_true")
    ap.add_argument("--probe", action="store_true",
                    help="the kernels the counter passes of the profiler look at, once each, and nothing else: the element gather at "
                         "100 %% hits, the plain gather, the atomic pairs, the gather through the LDS translation table, the timed steps")
    ap.add_argument("--probe-batches", type=str, default="",
                    help="comma-separated K: 65536 waves whose 64 lanes read K distinct pages of a cold 4 GiB cache, one launch per K, "
                         "batches per second and I/Os per second (with BAM_AMD_LIB naming the build with the phase timers, those too); nothing else")
    ap.add_argument("--pages-per-wave", type=int, default=STREAM_PAGES_PER_WAVE, help="pages a wave of the streaming kernels reads (a power of two up to 16)")
    ap.add_argument("--only-hit", action="store_true",
                    help="hit-path leg and a plain 1 GiB copy only (short; what the counter passes of the profiler are run on)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path runs on one GPU; --gpus %d is not supported (a GPU box here has one GPU, "
                 "and the path has no collective step to scale)" % args.gpus)

    import numpy as np
    import torch
    import bam_amd
    from bam_amd import gen, _lib
    from bam_amd.host import make_array
    import oracle

    L = _lib.load()                     # raises if the HIP library is missing: nothing here falls back to the CPU
    O = oracle.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def event():
        e = ctypes.c_void_p()
        assert L.bam_event_create(ctypes.byref(e)) == 0
        return e

    def elapsed_ms(a, b):
        ms = ctypes.c_float(0)
        assert L.bam_event_elapsed_ms(a, b, ctypes.byref(ms)) == 0
        return ms.value

    # ------------------------------------------------------------------ small batches (a mode of its own)
    if args.probe_batches:
        # 65536 waves; the 64 lanes of a wave read K distinct pages of a cold 4 GiB cache over a 4 GiB procedural store
        # (K = 1: the whole wave wants one page, K = 64: every lane its own), one thread per read, one launch per K
        n_el, waves = 1 << 29, 1 << 16
        target = bam_amd.Target("/dev/libnvm0", n_el * 8, 512, backing=False, seed=SEED, n_io_threads=args.io_threads)
        ctrl = bam_amd.Controller("/dev/libnvm0", 1, 0, queue_depth=args.depth, n_queues=args.queues, spin_limit=60_000_000)
        rows = []
        for K in [int(x) for x in args.probe_batches.split(",")]:
            pc, rng, arr = make_array(ctrl, n_el, PAGE, 1 << 20)
            waves = min(1 << 16, n_el // 512 // K)          # every wave its own K pages of the store
            tid = torch.arange(waves * 64, dtype=torch.int64, device=dev)
            idx_k = ((tid // 64) * K + (tid % 64) % K) * 512 + (tid % 64)
            s_k = torch.zeros(1, dtype=torch.int64, device=dev)
            arr.stats(); pc.profile()
            a, b = event(), event()
            L.bam_event_record(a, stream)
            arr.read_shaped_async(waves * 64, s_k, idx_k, arr.ONE_PER_THREAD, 1, block_size=64)
            L.bam_event_record(b, stream)
            ms = elapsed_ms(a, b)
            st, pr = arr.stats(), pc.profile()
            assert st["read_io_cnt"] == waves * K
            row = {"K": K, "waves": waves, "ms": ms, "read_ios": st["read_io_cnt"], "M_batches_per_s": waves / ms / 1e3, "MIOPS": st["read_io_cnt"] / ms / 1e3}
            if pr["batches"]:
                nb_ = pr["batches"]
                row["per_batch_us"] = {k: pr[k] / nb_ / 100 for k in ("t_cid", "t_submit", "t_wait", "t_copy")}
                row["commands_per_batch"] = pr["commands"] / nb_
            rows.append(row)
            log("[bench] K=%d: %s" % (K, row))
            assert not ctrl.aborted()
            arr.close(); rng.close(); pc.close()
        print(json.dumps({"probe_batches": rows}), flush=True)
        ctrl.close(); target.close()
        return

    # ------------------------------------------------------------------ set-up
    t0 = time.time()
    target = bam_amd.Target("/dev/libnvm0", N_ELEMS * 8, 512, backing=False, seed=SEED, n_io_threads=args.io_threads)
    ctrl = bam_amd.Controller("/dev/libnvm0", 1, 0, queue_depth=args.depth, n_queues=args.queues, spin_limit=60_000_000)
    pc, rng, arr = make_array(ctrl, N_ELEMS, PAGE, CACHE_PAGES)
    n_steps = args.warmup + args.steps
    idx = [gen.gather_indices(SEED, N_READS, N_ELEMS, first=s * N_READS) for s in range(n_steps)]
    sums = [torch.zeros(1, dtype=torch.int64, device=dev) for _ in range(n_steps)]
    torch.cuda.synchronize()
    log("[bench] set-up %.1fs: %s %s" % (time.time() - t0, ctrl.info(), pc.info()))

    # ------------------------------------------------------------------ hit path (roofline): stream the resident cache
    ppw = args.pages_per_wave
    assert ppw in (1, 2, 4, 8, 16)
    arr.stream(CACHE_PAGES // ppw, ppw, mode=2)             # cold pass fills the cache with pages 0 .. CACHE_PAGES-1
    arr.stats()
    ref_stream = O.bo_store_sum(SEED, 0, 1, 1 << 24)
    hit_reps = 20
    s_hit = torch.zeros(1, dtype=torch.int64, device=dev)
    # mode 1: the reference's kernel (a wave per run of pages, every element through bam_ptr), as bam_cache_stream runs it on an
    # array of one range: the kernel that reads what is resident, then the one for what it noted (here: nothing).  Both launches
    # are inside the events.  6: the same loop as one launch of the kernel that can miss; 0: operator[] per element; 2: page-wise
    kinds = ((1, "bam_ptr"), (2, "page_wise"), (6, "bam_ptr_one_launch"), (0, "element_operator"))
    for mode, name in kinds:
        assert arr.stream((1 << 24) // 512 // 4, 4, mode=mode) == ref_stream, "hit-path checksum mismatch (%s)" % name
        arr.stream_async(CACHE_PAGES // ppw, ppw, s_hit, mode=mode)
    torch.cuda.synchronize()
    hit = {}
    for mode, name in kinds:
        a, b = event(), event()
        L.bam_event_record(a, stream)
        for _ in range(hit_reps):
            arr.stream_async(CACHE_PAGES // ppw, ppw, s_hit, mode=mode)
        L.bam_event_record(b, stream)
        ms = elapsed_ms(a, b) / hit_reps
        hit[name] = {"ms_per_launch": ms, "GBps": CACHE_PAGES * PAGE / ms / 1e6}
    st = arr.stats()
    assert st["read_io_cnt"] == 0 and st["miss_cnt"] == 0, "hit-path pass did I/O"
    roofline = {"bound": "hbm", "kernel": "k_cache_stream<1> (a wave per run of pages, every element through bam_ptr: benchmarks/cache/main.cu:44-114), "
                                          "with the launch that follows it for pages that are not resident (none here) inside the timed region",
                "achieved": hit["bam_ptr"]["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": hit["bam_ptr"]["GBps"] / HBM_PEAK_GBS, "traffic": HIT_TRAFFIC["bam_ptr"]["bytes"], "traffic_source": HIT_TRAFFIC["bam_ptr"]["source"],
                "bytes_per_launch": CACHE_PAGES * PAGE, "ms_per_launch": hit["bam_ptr"]["ms_per_launch"], "pages_per_wave": ppw,
                "page_wise_kernel": {"kernel": "k_cache_stream_pages (one acquire per 16 pages, streamed loads; no counterpart in the reference)",
                                     "achieved": hit["page_wise"]["GBps"], "frac": hit["page_wise"]["GBps"] / HBM_PEAK_GBS,
                                     "ms_per_launch": hit["page_wise"]["ms_per_launch"],
                                     "traffic": HIT_TRAFFIC["page_wise"]["bytes"], "traffic_source": HIT_TRAFFIC["page_wise"]["source"]},
                "bam_ptr_one_launch_GBps": hit["bam_ptr_one_launch"]["GBps"], "element_operator_GBps": hit["element_operator"]["GBps"]}
    # what the memory system gives a plain kernel that only reads (no cache protocol): the practical ceiling under `peak`
    probe = torch.empty(1 << 27, dtype=torch.int64, device=dev).fill_(1)
    ms_c = ctypes.c_float(0)
    best = 1e9
    for _ in range(5):
        assert L.bam_read_kernel(ctypes.c_void_p(probe.data_ptr()), ctypes.c_uint64(1 << 30), ctypes.byref(ms_c), stream) == 0
        best = min(best, ms_c.value)
    roofline["plain_read_kernel_GBps"] = (1 << 30) / best / 1e6
    log("[bench] hit path: %s" % hit)
    if args.only_hit:
        # the hit path taken apart: what taking references (none / per page / sixteen at a time) and keeping the payload in the L2
        # or not cost, against the plain reader above
        parts = {}
        for refs, rname in ((0, "no_reference"), (1, "reference_per_page"), (2, "references_16_at_a_time")):
            for nt, nname in ((0, "kept"), (1, "not_kept")):
                args_ = (arr.h, refs, nt, ctypes.c_uint64(CACHE_PAGES // ppw), ctypes.c_uint64(ppw), ctypes.c_void_p(s_hit.data_ptr()), stream)
                s_hit.zero_()
                assert L.bam_hit_path_parts(*args_) == 0
                torch.cuda.synchronize()
                assert int(s_hit.item()) & (2**64 - 1) == O.bo_store_sum(SEED, 0, 1, CACHE_PAGES * 512), "hit-path parts checksum mismatch"
                a, b = event(), event()
                L.bam_event_record(a, stream)
                for _ in range(hit_reps):
                    L.bam_hit_path_parts(*args_)
                L.bam_event_record(b, stream)
                parts["%s_%s_GBps" % (rname, nname)] = CACHE_PAGES * PAGE / (elapsed_ms(a, b) / hit_reps) / 1e6
        roofline["hit_path_parts"] = parts
        # a plain device copy of known size in the same process: the scale of the profiler's traffic counters
        src = torch.empty(1 << 27, dtype=torch.int64, device=dev).fill_(1)
        dst = torch.empty_like(src)
        ms_c = ctypes.c_float(0)
        for _ in range(3):
            assert L.bam_copy_kernel(ctypes.c_void_p(src.data_ptr()), ctypes.c_void_p(dst.data_ptr()), ctypes.c_uint64(1 << 30), ctypes.byref(ms_c), stream) == 0
        roofline["copy_1GiB_ms"] = ms_c.value
        roofline["copy_GBps_read_plus_write"] = 2 * (1 << 30) / ms_c.value / 1e6
        print(json.dumps({"roofline": roofline}), flush=True)
        arr.close(); rng.close(); pc.close(); ctrl.close(); target.close()
        return

    # 100 %-hit element gather (indices restricted to the resident half)
    idx_hit = gen.gather_indices(SEED, N_READS, CACHE_PAGES * 512)
    arr.read_async(N_READS, s_hit.zero_(), idx_hit, block_size=args.block)
    torch.cuda.synchronize()
    a, b = event(), event()
    L.bam_event_record(a, stream)
    arr.read_async(N_READS, s_hit.zero_(), idx_hit, block_size=args.block)
    L.bam_event_record(b, stream)
    ms = elapsed_ms(a, b)
    assert int(s_hit.item()) & (2**64 - 1) == O.bo_gather_sum(SEED, SEED, 0, N_READS, CACHE_PAGES * 512), "hit gather checksum mismatch"
    gather_hit = {"reads_per_s": N_READS / ms * 1e3, "GBps_of_u64": N_READS * 8 / ms / 1e6, "ms": ms,
                  "kernel": "k_array_read_n<8> (what bam_array_read launches for a launch of this size: eight reads per lane), with the launch that follows it for "
                            "requests whose page is not resident (none here) inside the timed region"}
    for shape, key in ((arr.ONE_PER_THREAD, "one_read_per_thread_reads_per_s"), (arr.FOUR_PER_THREAD, "four_per_thread_one_launch_reads_per_s")):
        arr.read_shaped_async(N_READS, s_hit.zero_(), idx_hit, shape, 4, block_size=args.block)
        a, b = event(), event()
        L.bam_event_record(a, stream)
        arr.read_shaped_async(N_READS, s_hit.zero_(), idx_hit, shape, 4, block_size=args.block)
        L.bam_event_record(b, stream)
        gather_hit[key] = N_READS / elapsed_ms(a, b) * 1e3
        assert int(s_hit.item()) & (2**64 - 1) == O.bo_gather_sum(SEED, SEED, 0, N_READS, CACHE_PAGES * 512), "hit gather checksum mismatch"
    for _ in range(2):      # the same index pattern as a plain gather from a flat 1 GiB array, no cache protocol
        assert L.bam_gather_kernel(ctypes.c_void_p(probe.data_ptr()), ctypes.c_void_p(idx_hit.data_ptr()), ctypes.c_uint64(N_READS), ctypes.byref(ms_c), stream) == 0
    gather_hit["plain_gather_reads_per_s"] = N_READS / ms_c.value * 1e3
    gather_hit["frac_of_plain_gather"] = gather_hit["reads_per_s"] / gather_hit["plain_gather_reads_per_s"]
    # a random 8-byte read costs a 128-byte line from HBM whatever the load's cache policy (FETCH_SIZE: 136 bytes per read with
    # the 8-byte index, profiles/k_array_read_counters_hits_and_random_gather.md), so the roofline of any gather is
    # 8 TB/s / 128 B = 62.5 G reads/s, and in bytes moved the gather through the cache runs at this fraction of the HBM peak
    gather_hit["hbm_bytes_per_read"] = 136
    gather_hit["hbm_GBps_by_traffic"] = gather_hit["reads_per_s"] * 136 / 1e9
    gather_hit["frac_of_hbm_peak_by_traffic"] = gather_hit["hbm_GBps_by_traffic"] / HBM_PEAK_GBS
    gather_hit["plain_gather_frac_of_hbm_peak_by_traffic"] = gather_hit["plain_gather_reads_per_s"] * 136 / 1e9 / HBM_PEAK_GBS
    # what the counted hit path pays: a take-and-drop pair of atomics per read on words scattered like the page descriptors
    table = torch.zeros(CACHE_PAGES, dtype=torch.int64, device=dev)
    pages_hit = idx_hit // 512
    for returns, key in ((1, "atomic_pairs_per_s"), (0, "atomic_pairs_unread_per_s")):
        for _ in range(2):
            assert L.bam_atomic_pairs_kernel(ctypes.c_void_p(table.data_ptr()), ctypes.c_void_p(pages_hit.data_ptr()), ctypes.c_uint64(N_READS), returns, ctypes.byref(ms_c), stream) == 0
        gather_hit[key] = N_READS / ms_c.value * 1e3
    assert int(table.abs().sum().item()) == 0
    del table, pages_hit
    del probe
    if args.probe:
        # the same reads through bam_ptr_tlb over a translation table in LDS (what the LDS counters are for)
        n_tlb = N_READS // 8
        for _ in range(2):
            a, b = event(), event()
            L.bam_event_record(a, stream)
            s_tlb = arr.read_via(6, n_tlb, idx_hit[:n_tlb], block_size=args.block)
            L.bam_event_record(b, stream)
        assert s_tlb == O.bo_gather_sum(SEED, SEED, 0, n_tlb, CACHE_PAGES * 512), "tlb gather checksum mismatch"
        gather_hit["tlb_route_reads_per_s"] = n_tlb / elapsed_ms(a, b) * 1e3
    arr.stats()
    del idx_hit
    log("[bench] hit gather: %s" % gather_hit)

    # ------------------------------------------------------------------ timed steps (configuration 2): one thread per read
    def run_steps(shape, lanes):
        for s_ in range(args.warmup):
            arr.read_shaped_async(N_READS, sums[s_].zero_(), idx[s_], shape, lanes, block_size=args.block)
        torch.cuda.synchronize()
        arr.stats(); target.stats(reset=True)
        a, b = event(), event()
        t_wall = time.time()
        L.bam_event_record(a, stream)
        for s_ in range(args.warmup, n_steps):
            arr.read_shaped_async(N_READS, sums[s_].zero_(), idx[s_], shape, lanes, block_size=args.block)
        L.bam_event_record(b, stream)
        torch.cuda.synchronize()
        t_wall = time.time() - t_wall
        ms_total = elapsed_ms(a, b)
        st = arr.stats()
        ts = target.stats()
        ok = not ctrl.aborted() and ctrl.info()["error_completions"] == 0
        for s_ in range(n_steps):
            want = O.bo_gather_sum(SEED, SEED, s_ * N_READS, N_READS, N_ELEMS)
            ok = ok and (int(sums[s_].item()) & (2**64 - 1)) == want
        assert ok, "configuration-2 checksum mismatch or aborted wait"
        assert st["access_cnt"] == args.steps * N_READS and st["read_io_cnt"] == ts["read_cmds"]
        return {"ms_per_step": ms_total / max(args.steps, 1), "iops": st["read_io_cnt"] / ms_total * 1e3, "reads_per_s": args.steps * N_READS / ms_total * 1e3,
                "hit_rate": st["hit_cnt"] / max(st["access_cnt"], 1), "read_ios_per_step": st["read_io_cnt"] / max(args.steps, 1),
                "doorbells": ts["sq_doorbells"], "sqe_retries": ts["sqe_retries"], "wall_s": t_wall, "ms_total": ms_total}

    one = run_steps(arr.ONE_PER_THREAD, 1)
    iops, ms_per_step, ms_total, cfg2_hit_rate = one["iops"], one["ms_per_step"], one["ms_total"], one["hit_rate"]
    log("[bench] cfg2, one thread per read: %s" % one)
    # the same steps as bam_array_read runs a launch of this size by default: what is resident is read by a kernel that cannot
    # miss, the rest 64 requests to a wave by one that can; the first launch leaves the second only requests whose page it did
    # not find, and the pages those bring in are the ones the rest of the step asks for
    two = run_steps(arr.TWO_LAUNCHES, 8)
    log("[bench] cfg2, two launches: %s" % two)
    del idx, sums
    if args.probe:
        print(json.dumps({"probe": {"hit_gather": gather_hit, "cfg2_ms_per_step": ms_per_step, "cfg2_iops": iops, "cfg2_hit_rate": cfg2_hit_rate,
                                    "two_launches": two}}), flush=True)
        arr.close(); rng.close(); pc.close(); ctrl.close(); target.close()
        return

    # ------------------------------------------------------------------ what the store can do
    ms_c = ctypes.c_float(0)
    assert L.bam_host_read_ceiling(8 << 30, 4096, ctypes.byref(ms_c)) == 0
    link_gbps = (8 << 30) / ms_c.value / 1e6
    n_clients = max(2, min(8, (os.cpu_count() or 8) // 2))
    # the target's own service rate with plain host clients on the host cores: short runs are noisy (the clients share
    # the cores with the service threads), so the median of five
    runs = sorted(L.bam_target_ceiling_iops(64 << 30, 512, 0, args.io_threads, n_clients, 256, 400000, 4096) for _ in range(5))
    target_iops = runs[2]
    # every page the store delivers crosses the interconnect towards the GPU, pulled by the GPU from a staging page or
    # pushed by the target into the cache slot: the store's ceiling as the GPU sees it is the slower of the target's own
    # service rate and the rate at which payload gets across, measured here as a bulk pull of host memory in 4 KiB pieces
    link_iops = link_gbps * 1e9 / PAGE
    ceiling = min(target_iops, link_iops)
    store = {"target_service_iops": target_iops, "target_service_runs": runs, "target_clients": n_clients,
             "interconnect_pull_GBps": link_gbps, "interconnect_pull_iops_4k": link_iops,
             "ceiling_iops_4k": ceiling, "ceiling_is": "interconnect" if link_iops < target_iops else "target", "cfg2_frac_of_ceiling": iops / ceiling, "direct_share_of_8": pc.info().get("direct_share", None),
             # the outer bound: what a PCIe Gen5 x16 link carries one way; a 4 KiB read moves its payload, a 64-byte entry and a 16-byte completion
             "pcie_gen5_x16_GBps": PCIE_GEN5_X16_GBPS, "pcie_gen5_x16_iops_4k": PCIE_GEN5_X16_GBPS * 1e9 / (PAGE + 64 + 16),
             "cfg2_GBps_on_the_link": iops * (PAGE + 64 + 16) / 1e9, "cfg2_frac_of_pcie_gen5_x16": iops * (PAGE + 64 + 16) / 1e9 / PCIE_GEN5_X16_GBPS}
    cores = args.cpu_threads if args.cpu_threads > 0 else usable_cores()
    cpu_target_threads = max(2, cores // 4)
    cpu_lanes = max(1, cores - cpu_target_threads)
    log("[bench] store: %s" % store)

    # ------------------------------------------------------------------ raw block benchmark (configuration 3)
    block = None
    if not args.skip_block:
        arr.close(); rng.close(); pc.close(); ctrl.close(); target.close()
        target = bam_amd.Target("/dev/libnvm0", 64 << 30, 512, backing=False, seed=SEED, n_io_threads=args.io_threads)
        ctrl = bam_amd.Controller("/dev/libnvm0", 1, 0, queue_depth=1024, n_queues=128, spin_limit=60_000_000)
        n_blk = 1 << 22
        pcb = bam_amd.PageCache(PAGE, n_blk, 0, ctrl)
        block = {}
        for req in (4096, 512):
            lbas = gen.block_lbas(SEED, n_blk, 64 << 30, req, 512)
            pcb.block_io(n_blk, req, lbas, block_size=64)           # warm-up launch
            torch.cuda.synchronize()
            a, b = event(), event()
            L.bam_event_record(a, stream)
            pcb.block_io(n_blk, req, lbas, block_size=64)
            L.bam_event_record(b, stream)
            ms = elapsed_ms(a, b)
            cs_d = pcb.block_checksums(n_blk, req)
            # every payload: the sums of the store's words, restated with tensor arithmetic (SplitMix64 as published); and a
            # sample against the oracle's C routine
            good = bool(torch.equal(cs_d, splitmix_block_sums(torch, SEED, lbas * (512 // 8), req // 8)))
            cs = cs_d.cpu().numpy().view(np.uint64)
            sample = np.random.default_rng(1).integers(0, n_blk, 4096)
            lb = lbas.cpu().numpy().view(np.uint64)
            good = good and all(int(cs[k]) == O.bo_block_checksum(SEED, int(lb[k]), 512, req) for k in sample)
            assert good and not ctrl.aborted(), "raw block payload checksum mismatch"
            block["read_%dB" % req] = {"iops": n_blk / ms * 1e3, "GBps": n_blk * req / ms / 1e6, "ms": ms}
        block["frac_of_ceiling_4k"] = block["read_4096B"]["iops"] / ceiling
        block["frac_of_ceiling"] = block["frac_of_ceiling_4k"]
        block["frac_of_pcie_gen5_x16_4k"] = block["read_4096B"]["iops"] * (PAGE + 64 + 16) / 1e9 / PCIE_GEN5_X16_GBPS
        log("[bench] block: %s" % block)
        pcb.close()

    # ------------------------------------------------------------------ BFS on RMAT (configuration 4)
    bfs = None
    if args.bfs_scale:
        t0 = time.time()
        if ctrl is not None:
            ctrl.close(); target.close()
        off, nb = gen.rmat_csr(SEED, args.bfs_scale)
        n_e = nb.numel()
        ns_bytes = (n_e * 8 + PAGE - 1) // PAGE * PAGE
        target = bam_amd.Target("/dev/libnvm0", ns_bytes, 512, backing=True, seed=SEED, n_io_threads=args.io_threads)
        dst = (ctypes.c_char * (n_e * 8)).from_address(target.L.bam_target_backing(target.h))
        nb_h = nb.cpu().numpy()
        ctypes.memmove(dst, nb_h.ctypes.data, n_e * 8)
        ctrl = bam_amd.Controller("/dev/libnvm0", 1, 0, queue_depth=1024, n_queues=128, spin_limit=60_000_000)
        cache_pages = max(1 << 14, (n_e * 8 // PAGE) // 4)              # 25 % of the edge array
        pcg, rg, ag = make_array(ctrl, n_e, PAGE, cache_pages)
        off_h = off.cpu().numpy().view(np.uint64)
        srcs = oracle.bfs_sources(SEED, off_h, args.bfs_sources)
        del nb
        log("[bench] bfs graph: V=2^%d E=%d cache_pages=%d (%.1fs to build)" % (args.bfs_scale, n_e, cache_pages, time.time() - t0))
        nb_u = nb_h.view(np.uint64)
        ag.set_graph(off)              # the per-graph preparation, outside the timed calls as in the reference's host code
        # the serial oracle on every source: the first alone (timed: the CPU figure), the others side by side on the host's cores
        from concurrent.futures import ThreadPoolExecutor
        t1 = time.time()
        refs = [oracle.bfs_levels(off_h, nb_u, int(srcs[0]))]
        cpu_bfs_s = time.time() - t1
        cpu_bfs_edges = O.bo_bfs_edges_scanned(len(off_h) - 1, off_h, refs[0][0])
        with ThreadPoolExecutor(max(1, min(8, len(srcs) - 1))) as ex:
            refs += list(ex.map(lambda x: oracle.bfs_levels(off_h, nb_u, int(x)), srcs[1:]))
        log("[bench] bfs oracle: %d sources, %.1fs" % (len(refs), time.time() - t1))
        legs = {}
        # the edge-page kernel on every source; the reference-shaped kernel (a wave per vertex, bam_ptr per element) on the first two
        # (64 vertices per wave: consecutive vertices share pages, so the more vertices a wave has, the more distinct pages are asked for at a time)
        # and the kernel that walks a queue of the level's vertices, sorted between levels
        for name, by_page, n_src, coarse in (("by_page", True, len(srcs), 1), ("per_vertex_bam_ptr", False, min(4, len(srcs)), 64),
                                             ("queue_of_vertices", False, min(4, len(srcs)), 0)):
            tot_ms, tot_edges, levels_ok, iters = 0.0, 0, True, []
            ag.stats()
            for k, src in enumerate(srcs[:n_src]):
                a, b = event(), event()
                L.bam_event_record(a, stream)
                lv, it = ag.bfs(off, int(src), frontier=True) if not coarse else ag.bfs(off, int(src), coarse=coarse, by_page=by_page)
                L.bam_event_record(b, stream)
                ms = elapsed_ms(a, b)
                lv_h = lv.cpu().numpy().view(np.uint32)
                levels_ok = levels_ok and np.array_equal(lv_h, refs[k][0]) and it == refs[k][1]      # every source of every kernel, full size
                tot_edges += O.bo_bfs_edges_scanned(len(off_h) - 1, off_h, lv_h)
                tot_ms += ms
                iters.append(it)
            assert levels_ok and not ctrl.aborted(), "BFS levels differ from the oracle (%s)" % name
            st = ag.stats()
            legs[name] = {"sources": n_src, "coarse": coarse, "GTEPS": tot_edges / tot_ms / 1e6, "ms_per_source": tot_ms / n_src, "iterations": iters,
                          "read_ios": st["read_io_cnt"], "MIOPS": st["read_io_cnt"] / tot_ms / 1e3,
                          "frac_of_ceiling": st["read_io_cnt"] / tot_ms * 1e3 / ceiling,
                          "hit_rate": st["hit_cnt"] / max(st["access_cnt"], 1)}
            log("[bench] bfs %s: %s" % (name, legs[name]))
        bfs = {"scale": args.bfs_scale, "edges": n_e, "cache_pages": cache_pages, "GTEPS": legs["by_page"]["GTEPS"]}
        bfs.update(legs)
        # CPU figure: the oracle's uncached in-RAM serial BFS on one core, same graph, first source
        bfs["cpu_serial_GTEPS"] = cpu_bfs_edges / cpu_bfs_s / 1e9
        bfs["frac_of_ceiling"] = bfs["by_page"]["frac_of_ceiling"]
        ag.close(); rg.close(); pcg.close(); ctrl.close(); target.close()
        if not args.skip_cpu:
            # the reference's path on the host cores (oracle/cpu_path.c: its bam_ptr, page cache and queues restated per thread,
            # against the same software target): the same graph, the same cache share, the first source; levels checked
            pad = (-n_e) % (PAGE // 8)
            store_h = nb_u if pad == 0 else np.concatenate([nb_u, np.zeros(pad, dtype=np.uint64)])
            cp = oracle.CpuPath(store_h.size * 8, n_e, PAGE, cache_pages, seed=SEED, backing=store_h, n_io_threads=cpu_target_threads, n_queues=cpu_lanes, queue_depth=1024)
            t1 = time.time()
            lv_c, it_c = cp.bfs(off_h, int(srcs[0]), n_threads=cpu_lanes)
            dt = time.time() - t1
            cst = cp.stats()
            assert np.array_equal(lv_c, refs[0][0]) and cp.check() == 0, "CPU-path BFS levels differ from the oracle"
            cp.close()
            bfs["cpu_path"] = {"GTEPS": cpu_bfs_edges / dt / 1e9, "seconds": dt, "scale": args.bfs_scale, "sources": 1, "cores": cores,
                               "lane_threads": cpu_lanes, "target_threads": cpu_target_threads, "read_ios": cst["read_io_cnt"], "MIOPS": cst["read_io_cnt"] / dt / 1e6,
                               "kind": "port", "sample": "the first source of the %d, whole graph, cache a quarter of the edge array" % len(srcs)}
            del store_h
        log("[bench] bfs: %s" % bfs)
        del off, nb_h, nb_u, off_h, lv, lv_h, refs
        target = ctrl = None

    # ------------------------------------------------------------------ CC on a uniform random graph (configuration 5)
    cc = None
    if args.cc_logv:
        t0 = time.time()
        if ctrl is not None:
            ctrl.close(); target.close()
        n_v = 1 << args.cc_logv
        off, nb = gen.uniform_csr(SEED, n_v, 16 * n_v)
        n_e = nb.numel()
        ns_bytes = (n_e * 8 + PAGE - 1) // PAGE * PAGE
        target = bam_amd.Target("/dev/libnvm0", ns_bytes, 512, backing=True, seed=SEED, n_io_threads=args.io_threads)
        store_words = torch.frombuffer((ctypes.c_char * (n_e * 8)).from_address(target.L.bam_target_backing(target.h)), dtype=torch.int64)
        store_words.copy_(nb)                                           # device -> the target's host memory
        torch.cuda.synchronize()
        ctrl = bam_amd.Controller("/dev/libnvm0", 1, 0, queue_depth=1024, n_queues=128, spin_limit=60_000_000)
        cache_pages = 1 << 21 if args.cc_logv == 26 else max(1 << 14, ns_bytes // PAGE // 2)        # 8 GiB at full size
        pcc, rc_, ac = make_array(ctrl, n_e, PAGE, cache_pages)
        log("[bench] cc graph: V=2^%d E=%d (%.1f GiB) cache_pages=%d (%.1fs to build)" % (args.cc_logv, n_e, n_e * 8 / 2**30, cache_pages, time.time() - t0))
        ac.set_graph(off)
        a, b = event(), event()
        L.bam_event_record(a, stream)
        lb, it = ac.cc(off, by_page=True)
        L.bam_event_record(b, stream)
        ms = elapsed_ms(a, b)
        st = ac.stats()
        # full-size parity: the labels are the unique fixed point of min-label propagation with label[v] <= v; the same
        # fixed point computed independently with torch gathers and scatter-min over the in-HBM copy of the graph
        src = torch.repeat_interleave(torch.arange(n_v, device=dev), off[1:] - off[:-1])
        ref = torch.arange(n_v, device=dev)
        while True:
            new = ref.clone()
            new.scatter_reduce_(0, nb, ref[src], "amin")
            if torch.equal(new, ref):
                break
            ref = new
        assert torch.equal(ref, lb) and not ctrl.aborted(), "CC labels differ from the fixed point"
        # the reference's per-vertex kernel (edge lists through bam_ptr) on the same graph, starting on what the sweeps above left in the cache
        a2, b2 = event(), event()
        L.bam_event_record(a2, stream)
        lb2, it2 = ac.cc(off, coarse=64)
        L.bam_event_record(b2, stream)
        ms2 = elapsed_ms(a2, b2)
        st2 = ac.stats()
        assert torch.equal(ref, lb2) and not ctrl.aborted(), "CC labels of the per-vertex kernel differ from the fixed point"
        by_page = {"ms": ms, "iterations": it, "GTEPS": it * n_e / ms / 1e6, "read_ios": st["read_io_cnt"], "MIOPS": st["read_io_cnt"] / ms / 1e3,
                   "frac_of_ceiling": st["read_io_cnt"] / ms * 1e3 / ceiling}
        per_vertex = {"coarse": 64, "ms": ms2, "iterations": it2, "GTEPS": it2 * n_e / ms2 / 1e6, "read_ios": st2["read_io_cnt"], "MIOPS": st2["read_io_cnt"] / ms2 / 1e3,
                      "frac_of_ceiling": st2["read_io_cnt"] / ms2 * 1e3 / ceiling}
        # the headline of the leg is the faster of the two kernels; both are reported (the per-vertex one starts on what the
        # by-page one left in the cache)
        lead, lead_name = (by_page, "by_page") if ms <= ms2 else (per_vertex, "per_vertex_bam_ptr")
        cc = {"log2_vertices": args.cc_logv, "edges": n_e, "cache_pages": cache_pages, "ms": lead["ms"], "iterations": lead["iterations"],
              "GTEPS": lead["GTEPS"], "read_ios": lead["read_ios"], "MIOPS": lead["MIOPS"], "frac_of_ceiling": lead["frac_of_ceiling"],
              "components": int(torch.unique(lb).numel()), "kernel": lead_name, "by_page": by_page, "per_vertex_bam_ptr": per_vertex}
        del src, ref, new, nb, off, lb, lb2, store_words
        ac.close(); rc_.close(); pcc.close(); ctrl.close(); target.close()
        target = ctrl = None
        if not args.skip_cpu:
            # the reference's path on the host cores, on a bounded graph of the same kind (2^24 vertices, edge factor 16, half of
            # the edge array cached as at full size): labels against union-find
            logv_c = min(args.cc_logv, 24)
            off_c, nb_c = gen.uniform_csr(SEED, 1 << logv_c, 16 << logv_c)
            off_ch, nb_ch = off_c.cpu().numpy().view(np.uint64), nb_c.cpu().numpy().view(np.uint64)
            del off_c, nb_c
            n_ec = nb_ch.size
            pad = (-n_ec) % (PAGE // 8)
            store_h = nb_ch if pad == 0 else np.concatenate([nb_ch, np.zeros(pad, dtype=np.uint64)])
            cp = oracle.CpuPath(store_h.size * 8, n_ec, PAGE, max(64, store_h.size * 8 // PAGE // 2), seed=SEED, backing=store_h,
                                n_io_threads=cpu_target_threads, n_queues=cpu_lanes, queue_depth=1024)
            t1 = time.time()
            lb_c, it_c = cp.cc(off_ch, n_threads=cpu_lanes)
            dt = time.time() - t1
            cst = cp.stats()
            assert np.array_equal(lb_c, oracle.cc_labels(off_ch, nb_ch)[0]) and cp.check() == 0, "CPU-path CC labels differ from the oracle"
            cp.close()
            cc["cpu_path"] = {"GTEPS": it_c * n_ec / dt / 1e9, "seconds": dt, "log2_vertices": logv_c, "edges": int(n_ec), "iterations": it_c, "cores": cores,
                              "lane_threads": cpu_lanes, "target_threads": cpu_target_threads, "read_ios": cst["read_io_cnt"], "MIOPS": cst["read_io_cnt"] / dt / 1e6,
                              "kind": "port", "sample": "a graph of 2^%d vertices of the same kind, half of its edge array cached" % logv_c}
            del store_h, off_ch, nb_ch, lb_c
        log("[bench] cc: %s" % cc)

    if ctrl is not None:
        ctrl.close(); target.close()

    # ------------------------------------------------------------------ CPU baseline (the reference path restated on host cores)
    cpu = None
    if not args.skip_cpu:
        n_s = args.cpu_reads
        cp = oracle.CpuPath(N_ELEMS * 8, N_ELEMS, PAGE, CACHE_PAGES, seed=SEED, n_io_threads=cpu_target_threads, n_queues=cpu_lanes, queue_depth=1024)
        idx_h = oracle.gather_indices(SEED, 0, n_s, N_ELEMS)
        t1 = time.time()
        s = cp.array_sum(n_s, idx_h, n_threads=cpu_lanes)
        dt = time.time() - t1
        cst = cp.stats()
        assert s == O.bo_gather_sum(SEED, SEED, 0, n_s, N_ELEMS) and cp.check() == 0, "CPU baseline checksum mismatch"
        cp.close()
        cpu = {"value": cst["read_io_cnt"] / dt, "unit": "IOPS", "cores": cores, "kind": "port",
               "lane_threads": cpu_lanes, "target_threads": cpu_target_threads, "cores_online": os.cpu_count(),
               "sample": "the first %d of the element reads of the timed steps (one step is 2^26), cold cache, on the %d cores this process may use: "
                         "%d lane threads + %d target threads; %.1f s" % (n_s, cores, cpu_lanes, cpu_target_threads, dt),
               "reads_per_s": n_s / dt, "bfs_cpu_path_GTEPS": (bfs or {}).get("cpu_path", {}).get("GTEPS"), "cc_cpu_path_GTEPS": (cc or {}).get("cpu_path", {}).get("GTEPS")}
        log("[bench] cpu baseline: %s" % cpu)

    out = {
        "metric": "4KiB read IOPS (random gather through the page cache); cache-hit GB/s and BFS GTEPS alongside",
        "value": iops, "unit": "IOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u64", "data": "synthetic",
        "config": {"workload": "random gather array bench: 2^28 u64 (2 GiB store), 4 KiB pages, 1 GiB page cache, 2^26 uniform-random reads per launch, one thread per read, "
                               "one launch (the reference's kernel as it is, benchmarks/array/main.cu:43-65; BAM_READ_ONE_PER_THREAD)",
                   "store": "software NVMe target, procedural namespace, %d service threads, %d queue pairs x %d" % (args.io_threads, args.queues, args.depth),
                   "seed": SEED, "block_size": args.block},
        "reads_per_s": args.steps * N_READS / ms_total * 1e3,
        "hit_rate": cfg2_hit_rate,
        "one_read_per_thread": {"ms": ms_per_step, "iops": iops, "hit_rate": cfg2_hit_rate, "read_ios_per_step": one["read_ios_per_step"]},
        # the same steps the way bam_array_read runs a launch of this size when left to choose: far fewer reads from the store
        # for the same 2^26 element reads, so a step is over sooner and the store is not kept at its rate for as long
        "two_launches": {"ms_per_step": two["ms_per_step"], "iops": two["iops"], "reads_per_s": two["reads_per_s"], "hit_rate": two["hit_rate"],
                         "read_ios_per_step": two["read_ios_per_step"], "frac_of_ceiling": two["iops"] / ceiling,
                         "speedup_per_step": ms_per_step / two["ms_per_step"]},
        "roofline": roofline,
        # the kernel that `value` times is bound by the store, not by HBM: its own entry, priced against what gets across the
        # interconnect in 4 KiB pieces (measured in this run by bam_host_read_ceiling) or the target's service rate if lower
        "roofline_miss_path": {"bound": "store", "kernel": "k_array_read (the timed steps)", "achieved": iops, "peak": ceiling, "unit": "IOPS",
                               "frac": iops / ceiling, "peak_is": store["ceiling_is"], "bytes_per_unit": PAGE,
                               "achieved_GBps": iops * PAGE / 1e9, "peak_GBps": ceiling * PAGE / 1e9,
                               "pcie_gen5_x16_GBps": PCIE_GEN5_X16_GBPS, "bytes_on_the_link_per_unit": PAGE + 64 + 16,
                               "frac_of_pcie_gen5_x16": store["cfg2_frac_of_pcie_gen5_x16"]},
        "cpu_baseline": cpu, "store": store, "hit_gather": gather_hit, "block": block, "bfs": bfs, "cc": cc,
    }
    print(json.dumps(out), flush=True)
    # nothing of this process outlives the line above: every target, controller and CPU-path handle has been closed (their
    # service threads joined), the thread pool of the serial BFS oracle was a context manager
    import threading
    log("[bench] done; python threads alive: %d, native threads of the process: %d"
        % (threading.active_count(), len(os.listdir("/proc/self/task"))))


if __name__ == "__main__":
    main()
