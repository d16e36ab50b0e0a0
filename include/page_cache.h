/*
 * Software page cache in GPU memory in front of NVMe-resident arrays:
 * page_cache_t / range_t<T> / array_t<T> on the host, page_cache_d_t /
 * range_d_t<T> / array_d_t<T> / bam_ptr<T> on the device.
 *
 * Same surface and same page state machine as include/page_cache.h of the
 * reference: state word layout :57-70, data_page_t :96-102, bam_ptr :414-485,
 * cache_page_t :487-493, page_cache_d_t :501-550, backing-page mapping
 * :556-582, __flush :584-629, page_cache_t :631-887, range_d_t :891-962 and
 * its members :1035-1224 (acquire_page :1122-1224), range_t :964-1030,
 * array_d_t :1229-1716 (coalesce_page :1330-1366, seq_read :1541-1574),
 * array_t :1718-1774, find_slot :1786-1927, read_data/write_data/access_data
 * :1930-2132.
 *
 * What is different, and why:
 *   - A gfx950 wave is 64 lanes in lock step.  The reference lets the one
 *     "master" thread of each group of same-page requests run the whole miss
 *     path alone; in lock step that would serialise up to 64 I/Os per wave.
 *     Here all masters of a wave move through the state machine together:
 *     their state atomics are one vector instruction, their victim searches
 *     run side by side, and their NVMe reads are submitted as one batch (one
 *     ticket grab, one doorbell) and awaited together.
 *   - The reference orders payload DMA against the completion with a second
 *     dummy read serialised on a global lock (enqueue_second :1961-2007).
 *     Here the completion is read with a system-scope acquire and the page is
 *     published with an agent-scope release; extra_reads stays 0.
 *   - Statistics counters are sharded by compute unit instead of four global
 *     words that every access of every wave would hit.
 *   - Descriptors are dense (8-byte data_page_t, 16-byte cache_page_t).
 */
#ifndef __PAGE_CACHE_H__
#define __PAGE_CACHE_H__

#include <cmath>
#include <cstdint>
#include <cstring>
#include <iostream>
#include <vector>
#include <simt/atomic>
#include "bam_wave.h"
#include "buffer.h"
#include "ctrl.h"
#include "nvm_cmd.h"
#include "nvm_parallel_queue.h"
#include "nvm_types.h"
#include "nvm_util.h"
#include "util.h"

#define FREE 2

enum data_dist_t { REPLICATE = 0, STRIPE = 1 };

#define ALL_CTRLS 0xffffffffffffffffULL

/* page state word: bit 31 VALID, bit 30 BUSY, bit 29 DIRTY, bits 28:0 reference count */
#define INVALID 0x00000000U
#define VALID   0x80000000U
#define BUSY    0x40000000U
#define DIRTY   0x20000000U
#define CNT_SHIFT (29ULL)
#define CNT_MASK 0x1fffffffU
#define DISABLE_BUSY_ENABLE_VALID 0xc0000000U
#define DISABLE_BUSY_MASK 0xbfffffffU
#define NV_NB 0x00U
#define NV_B  0x01U
#define V_NB  0x02U
#define V_B   0x03U

/*
 * data_page_t::offset: the cache slot in the low BAM_SLOT_BITS bits, above them a count of how many times the page has
 * been loaded (mod 32).  Readers that take no reference (bam_read_unpinned) look at the descriptor before and after
 * their load and need the second look to tell them that the page has not left the slot and come back in between.
 */
#define BAM_SLOT_BITS 27u
#define BAM_SLOT_MASK ((1u << BAM_SLOT_BITS) - 1u)

/* batches smaller than this are never placed directly: the controller pushes a page into device memory in several
 * microseconds, which a wave with a few commands waits for in full, while what it pulls itself is there in two */
#ifndef BAM_DIRECT_MIN_BATCH
#define BAM_DIRECT_MIN_BATCH 24u
#endif

#define BAM_TOKEN_SLOTS 4096u
#define BAM_STAT_SHARDS 4096

struct page_cache_t;
struct page_cache_d_t;
template <typename T> struct range_t;
template <typename T> struct array_d_t;
template <typename T> struct range_d_t;

/* one per backing page */
typedef struct __attribute__((aligned(8))) { uint32_t state; uint32_t offset; } data_page_t;   /* read as one 64-bit word on the hit path */
typedef data_page_t* pages_t;
__forceinline__ __device__ void bam_release_refs(data_page_t* dp, const uint32_t count, const bool wrote);

/*
 * One per cache slot: which page the slot holds and who may change that, in one word, so that taking the slot's lock
 * tells the taker in the same round trip what the slot holds.  Bits 63:62 are the reference's page_take_lock (FREE = 2,
 * LOCKED = 1, UNLOCKED = 0; 3 = locked by the one who found it free), bits 61:0 its page_translation.
 */
typedef struct { uint64_t page_translation; } cache_page_t;
#define BAM_TAKE_SHIFT 62
#define BAM_TRANSLATION_MASK ((1ull << BAM_TAKE_SHIFT) - 1ull)

/* statistics of one range, one shard per group of compute units */
typedef struct { unsigned long long access_cnt, miss_cnt, hit_cnt, read_io_cnt, pad[4]; } bam_stat_shard_t;

template <typename T>
struct returned_cache_page_t {
    T* addr;
    uint32_t size;
    uint32_t offset;
    __host__ __device__ T operator[](size_t i) const { return i < size ? addr[i] : 0; }
    __host__ __device__ T& operator[](size_t i) { return i < size ? addr[i] : addr[0]; }
};

struct page_cache_d_t {
    uint8_t* base_addr;
    uint64_t page_size;
    uint64_t page_size_minus_1;
    uint64_t page_size_log;
    uint64_t n_pages;
    uint64_t n_pages_minus_1;
    cache_page_t* cache_pages;
    uint32_t* page_ticket;
    uint64_t* prp1;                  /* [n_pages] bus address of each slot (direct transfers) */
    uint32_t direct_share;           /* with staging available: of every 8 read batches of the cache's miss path, this many go direct all the same */
    uint32_t direct_limit_ahead;     /* the same bound for batches of waves that only fetch ahead of others (range_view::read_ahead): nobody copies for them */
    uint32_t direct_limit;           /* not 0: instead of that share, a read batch of the miss path goes direct while fewer than this many directly placed commands are in flight on the whole cache (*direct_gauge) */
    uint32_t* direct_gauge;
    uint32_t direct_share_raw;       /* the same for reads through read_data / access_data (raw block I/O into slots the caller names) */
    uint64_t* prp2;                  /* [n_pages] second page or PRP list when page_size > controller page */
    uint64_t ctrl_page_size;
    uint64_t range_cap;
    pages_t* ranges;
    uint64_t n_ranges;
    uint64_t n_ranges_bits;
    uint64_t n_ranges_mask;
    uint64_t* ranges_page_starts;
    data_dist_t* ranges_dists;
    simt::atomic<uint64_t, simt::thread_scope_device>* ctrl_counter;
    simt::atomic<uint64_t, simt::thread_scope_device>* extra_reads;   /* stays 0: no fence reads are issued */
    Controller** d_ctrls;
    uint64_t n_ctrls;
    bool prps;
    uint64_t n_blocks_per_page;
    uint32_t wave_batch;             /* distinct pages one wave loads side by side (64: a whole wave) */
    uint32_t fast_reads;             /* element reads (seq_read, operator[]) of resident pages take no reference: bam_read_unpinned */
    uint32_t* miss_tokens;           /* number of waves inside the miss path right now */
    uint32_t miss_waves;             /* at most this many at a time per compute unit (0 = no limit) */
    unsigned long long* prof;        /* [32] phase timers in 100 MHz ticks (the first controller's), filled only by builds with BAM_PROFILE */
    bam_guard_t* guard;
    uint32_t spin_limit;

    __forceinline__ __device__ cache_page_t* get_cache_page(const uint32_t page) const { return &cache_pages[page]; }
    __forceinline__ __device__ uint32_t find_slot(uint64_t address, uint64_t range_id, const uint32_t queue_);
    __forceinline__ __device__ bool spin_giveup(bam::spin_t& s) const { return bam::spin_giveup(guard, spin_limit, s); }
};

__device__ void read_data(page_cache_d_t* pc, QueuePair* qp, const uint64_t starting_lba, const uint64_t n_blocks, const unsigned long long pc_entry);
__device__ void write_data(page_cache_d_t* pc, QueuePair* qp, const uint64_t starting_lba, const uint64_t n_blocks, const unsigned long long pc_entry);

/* page of a range -> (controller, page on that controller): include/page_cache.h:556-582 of the reference */
__forceinline__ __host__ __device__
uint64_t get_backing_page_(const uint64_t page_start, const size_t page_offset, const uint64_t n_ctrls, const data_dist_t dist)
{
    return dist == STRIPE ? page_start + page_offset / n_ctrls : page_start + page_offset;
}
__forceinline__ __host__ __device__
uint64_t get_backing_ctrl_(const size_t page_offset, const uint64_t n_ctrls, const data_dist_t dist)
{
    return dist == STRIPE ? page_offset % n_ctrls : ALL_CTRLS;
}

/* ------------------------------------------------------------------ */
/* NVMe I/O glue                                                      */
/* ------------------------------------------------------------------ */
namespace bam {

/*
 * Move each active lane's payload (dst/src/bytes differ per lane) with the
 * whole group: one lane's payload at a time, 16 bytes per lane per access.
 * All loads of a 4 KiB page are issued before its stores so that one page
 * costs one trip over the interconnect, not four.  The lanes that move are the
 * largest power of two within the group, so that every access of the group
 * covers one aligned piece of 16 x 2^k bytes: a group of, say, 27 lanes would
 * otherwise read 432-byte pieces whose ends split lines, which costs extra
 * requests on the interconnect (measured: 16 movers out of 27 lanes carry 6 %
 * more pages per second than all 27).
 */
__device__ __forceinline__ void copy_pages(uint8_t* dst, const uint8_t* src, uint32_t bytes, uint64_t act, uint32_t n, uint32_t rank)
{
    const uint32_t movers = 1u << (31 - __builtin_clz(n));
    for (uint64_t m = act; m; m &= m - 1) {
        const uint32_t j = first_lane(m);
        const u32x4_t* s = (const u32x4_t*)bcast((uint64_t)src, j);
        u32x4_t* d = (u32x4_t*)bcast((uint64_t)dst, j);
        const uint32_t nb = bcast(bytes, j) / 16;
        if (rank >= movers) continue;
        /* system scope both ways (ld16_sys / st16_sys): nothing stale is read, and what is written is in memory when the
         * wave's store counter says so */
        uint32_t i = rank;
        for (; i + 3 * movers < nb; i += 4 * movers) {
            u32x4_t x0, x1, x2, x3;
            ld16x4_sys(s + i, s + i + movers, s + i + 2 * movers, s + i + 3 * movers, x0, x1, x2, x3);
            st16_sys(d + i, x0); st16_sys(d + i + movers, x1); st16_sys(d + i + 2 * movers, x2); st16_sys(d + i + 3 * movers, x3);
        }
        for (; i < nb; i += movers) { const u32x4_t x = ld16_sys(s + i); st16_sys(d + i, x); }
    }
    /* the compiler does not count stores issued from asm, and drops the counter wait of a later fence when it knows of
     * nothing outstanding: wait here, so that what follows (publishing the page, releasing the staging slot) is ordered
     * after the payload by the hardware and not by luck */
    wait_stores();
}
/*
 * Permission to pull staged payload from host memory, taken by the wave (all active lanes call, one lane acts) before
 * it loads from a staging page and given back when the loads are in: see Controller::pull_limit.  The holder waits for
 * nothing but its own loads, so the permission always comes back; a wait that is given up goes ahead without one.
 */
__device__ __forceinline__ uint32_t* pull_begin(QueuePair* qp)
{
    const uint32_t limit = qp->pull_limit;
    if (!limit) return nullptr;
    /* two words per cluster: [0] turns taken, [1] turns finished; the n-th to ask goes ahead once n - finished < limit,
     * so the waves are served in the order they asked and a turn that ends is taken up within one look of the next in line */
    uint32_t* word = qp->pull_tokens + xcc_id() * 16u;
    if (lane() == first_lane(active_mask())) {
        const uint32_t turn = __hip_atomic_fetch_add(word, 1u, __ATOMIC_RELAXED, BAM_AGENT);
        spin_t sp;
        for (uint32_t looks = 1; (int32_t)(turn - ld_relaxed(word + 1)) >= (int32_t)limit; looks++) {
            __builtin_amdgcn_s_sleep(4);
            /* the abort flag and the clock once in a while (spin_giveup looks at them every 256th call) */
            if ((looks & 255u) == 0) { sp.n = 255u; sp.slp = 1; if (spin_giveup(&qp->cq, sp)) break; }
        }
    }
    return word;
}
__device__ __forceinline__ void pull_end(uint32_t* word)
{
    if (!word) return;
    fence_meta();                    /* the loads from host memory have come back */
    if (lane() == first_lane(active_mask())) __hip_atomic_fetch_add(word + 1, 1u, __ATOMIC_RELAXED, BAM_AGENT);
}

/*
 * Run `body` for the active lanes in rounds of at most `max_n` lanes at a time (in rank order).  A group of lanes
 * larger than half a queue is taken through the queue in such rounds, each a whole transfer: a round that held its
 * slots while the next waited for slots would wait for itself.
 */
template <typename F>
__device__ __forceinline__ void for_each_chunk(const uint32_t max_n, F&& body)
{
    const uint64_t act = active_mask();
    const uint32_t n = popc(act), rank = rank_in(act), step = max_n ? max_n : 1u;
    for (uint32_t base = 0; base < n; base += step)
        if (rank >= base && rank - base < step) body();
}

/*
 * The same with helpers: called by all active lanes, of which those with `mine` have payload to move; the others
 * lend their load slots.  A wave that loads one page for all of its lanes (a bam_ptr walking an edge list) moves it
 * in one trip of 64 lanes instead of sixty-four trips of one.
 */
__device__ __forceinline__ void copy_pages_helped(uint8_t* dst, const uint8_t* src, uint32_t bytes, bool mine)
{
    const uint64_t owners = ballot(mine);
    if (!owners) return;
    const uint64_t all = active_mask();
    copy_pages(dst, src, mine ? bytes : 0u, owners, popc(all), rank_in(all));
}

/*
 * One command per active lane on queue pair `qp` (wave-uniform), first half:
 * allocate ids, build the entries and submit them as one batch.  `pc_entry`
 * is the cache slot the data belongs to.  Returns the lane's command id;
 * `stage` is its staging page (NULL when the controller addresses the slot
 * itself) and `pos` the submission-queue slot its entry went to.
 */
__device__ __forceinline__ uint32_t io_submit_group(page_cache_d_t* pc, QueuePair* qp, uint64_t lba, uint32_t n_blocks, uint64_t pc_entry, uint8_t opcode,
                                                    uint8_t*& stage, uint32_t& pos, const uint32_t direct_share, uint32_t& gauged)
{
    const uint64_t act = active_mask();
    const uint32_t n = popc(act), rank = rank_in(act);
    const uint32_t bytes = n_blocks << qp->block_size_log;
    /* payload on its way out was written with plain stores, maybe by other compute units (which made it visible
     * when they dropped their references): nothing stale may be read when it is copied to a staging page, and
     * what this wave wrote itself must have reached memory before the controller fetches it */
    if (opcode == NVM_IO_WRITE) __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "");
#ifdef BAM_PROFILE
    const uint64_t pt0 = wall_clock64();
#endif
    /* placement by load: count this batch among the directly placed commands in flight, and see how many there were */
    uint32_t gauge_before = 0;
    const uint32_t gauged_kind = gauged;        /* 0: not counted (the caller has no end to report), 1: a batch somebody waits for, 2: read-ahead */
    gauged = gauged && direct_share && pc->direct_limit && pc->prp1 && qp->stage && opcode == NVM_IO_READ && bytes >= 2048 && bytes <= qp->stage_stride && n >= BAM_DIRECT_MIN_BATCH ? n : 0u;
    if (gauged && lane() == first_lane(act)) gauge_before = __hip_atomic_fetch_add(pc->direct_gauge, n, __ATOMIC_RELAXED, BAM_AGENT);
    /* the command's id is the submission slot it goes to, taken until read_end / io_group / poll_async gives it back */
    const uint32_t ticket = sq_reserve_group(&qp->sq);
    if (gauged) gauge_before = bcast(gauge_before, first_lane(act));
    const uint32_t cid = ticket & qp->sq.qs_minus_1;
#ifdef BAM_PROFILE
    const uint64_t pt1 = wall_clock64();
#endif
    uint64_t prp1, prp2 = 0;
    stage = nullptr;
    /*
     * Staged or direct.  Staged payload is pulled by the GPU (reads of host memory), direct payload is pushed by the
     * controller (writes into device memory): the two use opposite directions of the interconnect, so sending a
     * share of the read batches each way carries more than either alone.  Small reads stay staged: pushed in
     * pieces of a few hundred bytes they cost the controller more than they save.  Transfers larger than a staging
     * page (cache pages above two controller pages) always go direct, through their PRP lists.  The share differs
     * by caller: the cache's miss path has the waves busy with the page states as well and gains from handing three
     * batches of eight to the controller (12.3 against 11.4 M reads/s), raw block reads do best all staged (12.8
     * against 11.7 M).
     */
    bool direct = pc->prp1 && (bytes > qp->stage_stride ||
                               (opcode == NVM_IO_READ && bytes >= 2048 && n >= BAM_DIRECT_MIN_BATCH && ((ticket >> 6) & 7u) < direct_share));
    if (gauged) {
        /* the count was taken before the wait for the slots, so it cost no round trip of its own */
        direct = gauge_before < (gauged_kind == 2u ? pc->direct_limit_ahead : pc->direct_limit);
        if (!direct) {
            if (lane() == first_lane(act)) __hip_atomic_fetch_sub(pc->direct_gauge, n, __ATOMIC_RELAXED, BAM_AGENT);
            gauged = 0;
        }
    }
    const bool staged = qp->stage && !direct;
    if (staged) {
        stage = qp->stage + (size_t)cid * qp->stage_stride;
        prp1 = qp->stage_ioaddr + (uint64_t)cid * qp->stage_stride;
        if (bytes > qp->pageSize) prp2 = prp1 + qp->pageSize;         /* staging pages are contiguous: second controller page */
        if (opcode == NVM_IO_WRITE) {
            copy_pages(stage, pc->base_addr + pc_entry * pc->page_size, bytes, act, n, rank);
            fence_meta();                    /* written through to host memory: there before the command goes out */
        }
    } else {
        prp1 = pc->prp1[pc_entry];
        if (pc->prps) prp2 = pc->prp2[pc_entry];
    }
    nvm_cmd_t cmd;
#pragma unroll
    for (int i = 0; i < 16; i++) cmd.dword[i] = 0;
    nvm_cmd_header(&cmd, (uint16_t)cid, opcode, qp->nvmNamespace);
    nvm_cmd_data_ptr(&cmd, prp1, prp2);
    nvm_cmd_rw_blks(&cmd, lba, (uint16_t)n_blocks);
    sq_submit_group(&qp->sq, &cmd, ticket);
    pos = cid;
#ifdef BAM_PROFILE
    if (pc->prof && rank == 0) {
        const uint64_t pt2 = wall_clock64();
        atomicAdd(&pc->prof[0], 1ull); atomicAdd(&pc->prof[1], (unsigned long long)n);
        atomicAdd(&pc->prof[2], pt1 - pt0); atomicAdd(&pc->prof[3], pt2 - pt1);
    }
#endif
    return cid;
}

/* the completions of a batch that io_submit_group counted as directly placed (`gauged` commands) are in */
__device__ __forceinline__ void direct_done(page_cache_d_t* pc, const uint32_t gauged)
{
    if (gauged && lane() == first_lane(active_mask())) __hip_atomic_fetch_sub(pc->direct_gauge, gauged, __ATOMIC_RELAXED, BAM_AGENT);
}

/* the whole of one batch: submit, wait for all completions, move staged payload, recycle ids; true for the lanes whose
 * transfer happened (completed, without an error status) */
__device__ __forceinline__ bool io_group(page_cache_d_t* pc, QueuePair* qp, uint64_t lba, uint32_t n_blocks, uint64_t pc_entry, uint8_t opcode,
                                         const uint32_t direct_share)
{
    const uint64_t act = active_mask();
    uint8_t* stage;
    uint32_t pos;
    uint32_t gauged = 1;
    const uint32_t cid = io_submit_group(pc, qp, lba, n_blocks, pc_entry, opcode, stage, pos, direct_share, gauged);
#ifdef BAM_PROFILE
    const uint64_t pt2 = wall_clock64();
#endif
    const bool ok = cq_wait_group(&qp->cq, &qp->sq, cid);
    direct_done(pc, gauged);
#ifdef BAM_PROFILE
    const uint64_t pt3 = wall_clock64();
#endif
    /* a read that failed leaves its destination alone: the staging page holds what the last command of this id brought */
    if (ballot(stage && opcode == NVM_IO_READ && ok)) {
        uint32_t* pull = pull_begin(qp);
        copy_pages(pc->base_addr + pc_entry * pc->page_size, stage, stage && opcode == NVM_IO_READ && ok ? n_blocks << qp->block_size_log : 0u, act, popc(act), rank_in(act));
        pull_end(pull);
    }
    sq_release_group(&qp->sq, cid);
#ifdef BAM_PROFILE
    if (pc->prof && lane() == first_lane(act)) { atomicAdd(&pc->prof[4], pt3 - pt2); atomicAdd(&pc->prof[5], wall_clock64() - pt3); }
#endif
    return ok;
}

} // namespace bam

inline __device__ void access_data(page_cache_d_t* pc, QueuePair* qp, const uint64_t starting_lba, const uint64_t n_blocks, const unsigned long long pc_entry, const uint8_t opcode)
{
    bam::for_each_group((uint64_t)qp, (uint64_t)pc, [&](uint64_t q, uint64_t c) {
        bam::for_each_chunk(((QueuePair*)q)->sq.qs >> 1, [&]() {
            bam::io_group((page_cache_d_t*)c, (QueuePair*)q, starting_lba, (uint32_t)n_blocks, pc_entry, opcode, ((page_cache_d_t*)c)->direct_share_raw);
        });
    });
}

/*
 * read_data in two halves: submitted and completed, payload still in `stage` (NULL: already in the slot) | ids handed
 * back.  The split exists so that between the halves every lane of the wave can help move the payload.  It is only
 * taken when the calling lanes form one group (one queue pair, one cache): a wave that holds the command ids of one
 * queue while it waits for ids of another could end up waiting for a wave that does the same the other way round, so
 * with several groups each one runs its whole transfer before the next starts, and `held` comes back false.
 */
inline __device__ void read_begin(page_cache_d_t* pc, QueuePair* qp, const uint64_t starting_lba, const uint64_t n_blocks, const unsigned long long pc_entry,
                                  uint32_t& cid, uint8_t*& stage, bool& held, bool& ok, const bool ahead = false)
{
    const uint64_t all = bam::active_mask();
    bool one_group = bam::ballot(qp == (QueuePair*)bam::first((uint64_t)qp) && pc == (page_cache_d_t*)bam::first((uint64_t)pc)) == all;
    /* and one that the queue takes in one go: more commands than half its slots go through it in rounds */
    if (one_group && bam::popc(all) > (((QueuePair*)bam::first((uint64_t)qp))->sq.qs >> 1)) one_group = false;
    held = one_group;
    stage = nullptr;
    cid = 0;
    ok = false;
    if (!one_group) {
        bam::for_each_group((uint64_t)qp, (uint64_t)pc, [&](uint64_t q, uint64_t c) {
            bam::for_each_chunk(((QueuePair*)q)->sq.qs >> 1, [&]() {
                ok = bam::io_group((page_cache_d_t*)c, (QueuePair*)q, starting_lba, (uint32_t)n_blocks, pc_entry, NVM_IO_READ, ((page_cache_d_t*)c)->direct_share);
            });
        });
        return;
    }
    QueuePair* cur = (QueuePair*)bam::first((uint64_t)qp);
    page_cache_d_t* cpc = (page_cache_d_t*)bam::first((uint64_t)pc);
    uint32_t pos;
    uint32_t gauged = ahead ? 2u : 1u;
    cid = bam::io_submit_group(cpc, cur, starting_lba, (uint32_t)n_blocks, pc_entry, NVM_IO_READ, stage, pos, cpc->direct_share, gauged);
#ifdef BAM_PROFILE
    const uint64_t pt2 = wall_clock64();
#endif
    ok = bam::cq_wait_group(&cur->cq, &cur->sq, cid);
    bam::direct_done(cpc, gauged);
#ifdef BAM_PROFILE
    if (cpc->prof && bam::lane() == bam::first_lane(all)) atomicAdd(&cpc->prof[4], wall_clock64() - pt2);
#endif
}
/* for the lanes of a read_begin that came back with `held`: one queue pair */
inline __device__ void read_end(QueuePair* qp, const uint32_t cid)
{
    bam::sq_release_group(&((QueuePair*)bam::first((uint64_t)qp))->sq, cid);
}

inline __device__ void read_data(page_cache_d_t* pc, QueuePair* qp, const uint64_t starting_lba, const uint64_t n_blocks, const unsigned long long pc_entry)
{
    access_data(pc, qp, starting_lba, n_blocks, pc_entry, NVM_IO_READ);
}

inline __device__ void write_data(page_cache_d_t* pc, QueuePair* qp, const uint64_t starting_lba, const uint64_t n_blocks, const unsigned long long pc_entry)
{
    access_data(pc, qp, starting_lba, n_blocks, pc_entry, NVM_IO_WRITE);
}

/*
 * The two halves of access_data as separate calls (include/page_cache.h:1930-1959 of the reference): submit now,
 * collect later, so that a thread can keep several commands in flight.  A staged read leaves its destination with
 * the queue pair under its command id; poll_async moves the payload once the completion is in.  The threads of a
 * wave that submit together may poll together or one by one.
 */
inline __device__ void access_data_async(page_cache_d_t* pc, QueuePair* qp, const uint64_t starting_lba, const uint64_t n_blocks, const unsigned long long pc_entry,
                                         const uint8_t opcode, uint16_t* cid, uint16_t* sq_pos)
{
    bam::for_each_group((uint64_t)qp, (uint64_t)pc, [&](uint64_t q, uint64_t c) {
        QueuePair* cur = (QueuePair*)q;
        page_cache_d_t* cpc = (page_cache_d_t*)c;
        uint8_t* stage;
        uint32_t pos;
        uint32_t gauged = 0;                 /* not counted: the completion is collected elsewhere, so this path keeps to the fixed share */
        const uint32_t id = bam::io_submit_group(cpc, cur, starting_lba, (uint32_t)n_blocks, pc_entry, opcode, stage, pos, cpc->direct_share_raw, gauged);
        /* written for every command of a queue pair that has staging pages, staged or not: the id may have been used
         * by a staged read before, and poll_async must not find that command's destination */
        if (cur->stage) {
            cur->async_dst[id] = stage && opcode == NVM_IO_READ ? (uint64_t)(cpc->base_addr + pc_entry * cpc->page_size) : 0;
            cur->async_len[id] = (uint32_t)n_blocks << cur->block_size_log;
        }
        *cid = (uint16_t)id;
        *sq_pos = (uint16_t)pos;
    });
}

inline __device__ void poll_async(QueuePair* qp, uint16_t cid, uint16_t sq_pos)
{
    (void)sq_pos;
    bam::for_each_group((uint64_t)qp, [&](uint64_t q) {
        QueuePair* cur = (QueuePair*)q;
        const uint64_t act = bam::active_mask();
        const bool ok = bam::cq_wait_group(&cur->cq, &cur->sq, cid);
        uint8_t* dst = nullptr;
        uint32_t len = 0;
        if (cur->stage && ok) { dst = (uint8_t*)cur->async_dst[cid]; len = cur->async_len[cid]; }
        if (bam::ballot(dst != nullptr)) {
            uint32_t* pull = bam::pull_begin(cur);
            bam::copy_pages(dst, cur->stage + (size_t)cid * cur->stage_stride, dst ? len : 0, act, bam::popc(act), bam::rank_in(act));
            bam::pull_end(pull);
        }
        bam::sq_release_group(&cur->sq, cid);
    });
}

/* ------------------------------------------------------------------ */
/* eviction                                                           */
/* ------------------------------------------------------------------ */

#define BAM_NO_SLOT 0xffffffffu
#define BAM_FIND_SLOT_TRIES 64

/*
 * Find a cache slot for page `address` of range `range_id`: a global
 * round-robin hand (page_ticket); a slot is taken if it is free, or if its
 * current page has no references and is not busy, in which case that page is
 * invalidated (and written back first when dirty).  Called by all lanes of a
 * wave that need a slot; they advance side by side and take one ticket grab
 * per trip for the whole group.  A lane gives up after BAM_FIND_SLOT_TRIES
 * slots and returns BAM_NO_SLOT: its caller then lets the lanes that did get
 * a slot finish their loads before trying again, so that waves never wait for
 * slots while sitting on slots other waves wait for.
 */
__forceinline__ __device__
uint32_t page_cache_d_t::find_slot(uint64_t address, uint64_t range_id, const uint32_t queue_)
{
    using namespace bam;
    const uint64_t global_address = (address << n_ranges_bits) | range_id;
    uint32_t page = BAM_NO_SLOT;
    bool looking = true;
    for (uint32_t tries = 0;; tries++) {
        const uint64_t need = ballot(looking);
        if (!need) break;
        if (looking) {
            /* three round trips when the first slot will do: the hand, the slot's lock (which brings what the slot
             * holds), the victim's state */
            const uint32_t ld = first_lane(need);
            uint32_t base = 0;
            if (lane() == ld) base = __hip_atomic_fetch_add(page_ticket, popc(need), __ATOMIC_RELAXED, BAM_AGENT);
            base = bcast(base, ld);
            const uint32_t p = (uint32_t)((base + rank_in(need)) % n_pages);
            cache_page_t* cp = &cache_pages[p];
            const uint64_t w = __hip_atomic_fetch_or(&cp->page_translation, (uint64_t)LOCKED << BAM_TAKE_SHIFT, __ATOMIC_RELAXED, BAM_AGENT);
            const uint32_t v = (uint32_t)(w >> BAM_TAKE_SHIFT);
            if (v == FREE) {
                /* this lane holds it (the word reads FREE | LOCKED to everybody else until the store below) */
                page = p; looking = false;
            } else if (v == UNLOCKED) {
                const uint64_t prev = w & BAM_TRANSLATION_MASK;
                const uint64_t prev_range = prev & n_ranges_mask, prev_page = prev >> n_ranges_bits;
                data_page_t* victim = &ranges[prev_range][prev_page];
                /* BUSY first, questions later: a page that turns out to be in use has it taken off again (its users see a
                 * page that is busy for a moment and look again) */
                const uint32_t o = __hip_atomic_fetch_or(&victim->state, BUSY, __ATOMIC_RELAXED, BAM_AGENT);
                if ((o & BUSY) == 0) {
                    if ((o & CNT_MASK) == 0) {
                        if (o & DIRTY) {
                            const data_dist_t dist = ranges_dists[prev_range];
                            const uint64_t index = get_backing_page_(ranges_page_starts[prev_range], prev_page, n_ctrls, dist);
                            uint64_t c = get_backing_ctrl_(prev_page, n_ctrls, dist);
                            const uint64_t c_end = c == ALL_CTRLS ? n_ctrls : c + 1;
                            for (c = c == ALL_CTRLS ? 0 : c; c < c_end; c++) {
                                Controller* ctl = d_ctrls[c];
                                write_data(this, ctl->d_qps + (queue_ % ctl->n_qps), index * n_blocks_per_page, n_blocks_per_page, p);
                            }
                            fence_meta();
                        }
                        /* -> INVALID; references taken meanwhile stay counted and their owners reload */
                        __hip_atomic_fetch_and(&victim->state, CNT_MASK, __ATOMIC_RELAXED, BAM_AGENT);
                        page = p; looking = false;
                    } else {
                        __hip_atomic_fetch_and(&victim->state, DISABLE_BUSY_MASK, __ATOMIC_RELAXED, BAM_AGENT);
                    }
                }
                /* taken: the new translation goes in with the lock coming off; not taken: the old one stays */
                if (looking) st_relaxed(&cp->page_translation, prev);
            }
            /* (v == LOCKED or FREE | LOCKED: somebody else has it, and the fetch-or changed nothing) */
            if (page == p) st_relaxed(&cp->page_translation, global_address);
            if (looking && tries + 1 >= BAM_FIND_SLOT_TRIES) looking = false;
        }
    }
    return page;
}

/* ------------------------------------------------------------------ */
/* ranges                                                             */
/* ------------------------------------------------------------------ */

template <typename T>
struct range_d_t {
    uint64_t index_start;
    uint64_t count;
    uint64_t range_id;
    uint64_t page_start_offset;
    uint64_t page_size;
    uint64_t page_start;
    uint64_t page_count;
    size_t n_elems_per_page;
    data_dist_t dist;
    uint8_t* src;

    /* totals, filled in by the host when statistics are read back */
    unsigned long long access_cnt, miss_cnt, hit_cnt, read_io_cnt;
    bam_stat_shard_t* stats;         /* [BAM_STAT_SHARDS] live counters */

    pages_t pages;
    page_cache_d_t cache;

    __forceinline__ __device__ uint64_t get_backing_page(const size_t page_offset) const { return get_backing_page_(page_start, page_offset, cache.n_ctrls, dist); }
    __forceinline__ __device__ uint64_t get_backing_ctrl(const size_t page_offset) const { return get_backing_ctrl_(page_offset, cache.n_ctrls, dist); }
    __forceinline__ __device__ uint64_t get_sector_size() const { return page_size; }
    __forceinline__ __device__ uint64_t get_page(const size_t i) const { return ((i - index_start) * sizeof(T) + page_start_offset) >> cache.page_size_log; }
    __forceinline__ __device__ uint64_t get_subindex(const size_t i) const { return ((i - index_start) * sizeof(T) + page_start_offset) & cache.page_size_minus_1; }
    __forceinline__ __device__ uint64_t get_global_address(const size_t page) const { return (page << cache.n_ranges_bits) | range_id; }
    __forceinline__ __device__ void release_page(const size_t pg, const uint32_t count, const bool wrote) const { bam_release_refs(&pages[pg], count, wrote); }
    __forceinline__ __device__ void release_page(const size_t pg) const { release_page(pg, 1, true); }
    __forceinline__ __device__ void release_page(const size_t pg, const uint32_t count) const { release_page(pg, count, true); }
    __forceinline__ __device__ cache_page_t* get_cache_page(const size_t pg) const { return cache.get_cache_page(pages[pg].offset & BAM_SLOT_MASK); }
    __forceinline__ __device__ uint64_t get_cache_page_addr(const uint32_t page_trans) const { return (uint64_t)(cache.base_addr + (uint64_t)page_trans * cache.page_size); }
    __forceinline__ __device__ void mark_page_dirty(const size_t index) { __hip_atomic_fetch_or(&pages[index].state, DIRTY, __ATOMIC_RELAXED, BAM_AGENT); }
    __forceinline__ __device__ uint64_t acquire_page(const size_t pg, const uint32_t count, const bool write, const uint32_t ctrl, const uint32_t queue);
    /* spread by workgroup so that no counter word is shared by more than a few waves at a time */
    __forceinline__ __device__ bam_stat_shard_t* shard() const { return stats + (((blockIdx.x + blockIdx.y * gridDim.x) * 0x9E3779B1u) >> 20) % BAM_STAT_SHARDS; }
    __forceinline__ __device__ bool slow_step(const size_t pg, const bool write, const uint32_t queue, uint64_t& sv, uint32_t& slot, bool& was_hit, bool& progressed, const bool take_part = true,
                                              const bool may_load = true, bool* wants_load = nullptr, const bool ahead = false);
};

/*
 * Drop `count` references of a page.  A reader only has to have its loads of
 * the page returned before the count drops (a wait on the wave's own memory
 * counters); only a writer must also make its stores visible to the other
 * compute units before an evictor may write the page back, which costs an L2
 * write-back.  The wait is spelt out: a release fence at workgroup scope
 * compiles to a wait for LDS and scalar operations only (within a workgroup
 * vector memory is ordered by the hardware), so a payload load could still be
 * in flight when the count reached zero, and with a cache so small that a slot
 * is evicted and refilled within that load's latency it returned the next
 * page's data.
 */
__forceinline__ __device__ void bam_release_refs(data_page_t* dp, const uint32_t count, const bool wrote)
{
    if (bam::ballot(wrote)) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
    else bam::fence_meta();
    __hip_atomic_fetch_add(&dp->state, 0u - count, __ATOMIC_RELAXED, BAM_AGENT);
}

/*
 * Take `count` references on a page with one 64-bit fetch-add on
 * {state, offset}.  True on a hit (VALID, not BUSY): `slot` is the cache slot,
 * learnt from the same round trip.  On false the references are taken all the
 * same and `sv` holds the word as it was; acquire_page_slow carries on from it.
 * Relaxed on purpose: payload is read past the vector L1 (bam::ld_payload), so
 * no cache invalidation is needed on a page visit.
 */
__forceinline__ __device__ bool bam_try_hit(data_page_t* dp, const uint32_t count, const bool write, uint64_t& sv, uint32_t& slot)
{
    sv = __hip_atomic_fetch_add((uint64_t*)dp, (uint64_t)count, __ATOMIC_RELAXED, BAM_AGENT);
    const uint32_t s = (uint32_t)sv;
    if ((s >> (CNT_SHIFT + 1)) != V_NB) return false;
    if (write && (s & DIRTY) == 0) __hip_atomic_fetch_or(&dp->state, DIRTY, __ATOMIC_RELAXED, BAM_AGENT);
    slot = (uint32_t)(sv >> 32) & BAM_SLOT_MASK;
    return true;
}

/*
 * Read one element of a resident page without taking a reference: look at the descriptor, load the element, and once it
 * has arrived look at the descriptor again.  If both looks show the page valid, not busy, in the same slot and loaded
 * the same number of times, the slot held the page for the whole of the load: an evictor sets BUSY before it touches
 * anything, and a page that comes back carries a new load count.  False if the page is not resident or the looks
 * differ; the caller then goes the counted way (bam_try_hit).  This takes both read-modify-write operations out of a
 * hit: scattered over the descriptor table, the device does some ten thousand million such pairs per second, and five
 * times as many plain loads.  Reads only: a writer needs the page to stay until it has marked it dirty.
 */
template <typename T>
__forceinline__ __device__ bool bam_read_unpinned(const data_page_t* dp, const uint8_t* base_addr, const uint32_t page_size_log, const uint64_t in_page, T& out)
{
    const uint64_t s1 = __hip_atomic_load((const uint64_t*)dp, __ATOMIC_RELAXED, BAM_AGENT);
    const bool resident = ((uint32_t)s1 >> (CNT_SHIFT + 1)) == V_NB;
    if (resident) out = bam::ld_payload((const T*)(base_addr + ((uint64_t)((uint32_t)(s1 >> 32) & BAM_SLOT_MASK) << page_size_log) + in_page));
    bam::fence_meta();                               /* the element is here before the second look goes out */
    const uint64_t s2 = __hip_atomic_load((const uint64_t*)dp, __ATOMIC_RELAXED, BAM_AGENT);
    return resident && ((s1 ^ s2) & 0xFFFFFFFFC0000000ull) == 0;
}

namespace bam {
/*
 * Add v (below 2^BITS) of every active lane to a counter with one atomic per
 * distinct counter word: the lane values are summed with BITS ballots
 * (bit-sliced population count), which works for any set of active lanes.
 */
template <int BITS = 7>
__device__ __forceinline__ void stat_add(unsigned long long* ctr, uint32_t v)
{
    for_each_group((uint64_t)ctr, [&](uint64_t a0) {
        unsigned long long total = 0;
        if constexpr (BITS > 8) {
            /* any width: as many trips as the largest value of the group has bits (a view that lived through sixteen
             * page changes makes five, not thirty-two) */
            uint32_t rest = v;
#pragma unroll 1
            for (uint32_t b = 0; ballot(rest != 0); b++, rest >>= 1) total += (unsigned long long)popc(ballot(rest & 1u)) << b;
        } else {
#pragma unroll
            for (uint32_t b = 0; b < BITS; b++) total += (unsigned long long)popc(ballot((v >> b) & 1u)) << b;
        }
        if (lane() == first_lane(active_mask()) && total)
            __hip_atomic_fetch_add((unsigned long long*)a0, total, __ATOMIC_RELAXED, BAM_AGENT);
    });
}
} // namespace bam

/*
 * One pass of the page state machine past the hit test: the caller holds its
 * references (bam_try_hit) and `sv` is the state word it last saw.  True once
 * the page is valid, with its cache slot in `slot`.  Callable by any subset of
 * a wave's lanes, each for a different page: the lanes look at their pages
 * together, and those that have to load one do their victim search and their
 * NVMe reads as one batch.  `progressed` tells whether this pass loaded a page.
 *
 *   VALID, not BUSY     : hit (somebody else loaded it while we waited)
 *   not VALID, not BUSY : whoever sets BUSY first loads the page, then flips BUSY->VALID
 *   BUSY                : somebody else is loading or evicting; look again later
 *
 * Callers use a resolved page and drop its references before they make the
 * next pass for the lanes still waiting: a lane that sat on a resident page
 * while its siblings look for slots could pin the last evictable slot.
 */
template <typename T>
__forceinline__ __device__
bool range_d_t<T>::slow_step(const size_t pg, const bool write, const uint32_t queue, uint64_t& sv, uint32_t& slot, bool& was_hit, bool& progressed, const bool take_part,
                             const bool may_load, bool* wants_load, const bool ahead)
{
    using namespace bam;
    data_page_t* dp = &pages[pg];
    bool load_me = false, resolved = false;
    const uint32_t s = (uint32_t)sv, st = s >> (CNT_SHIFT + 1);
    progressed = false;
    if (!take_part) {
        /* here only to help move payload */
    } else if (st == V_NB) {
        if (write && (s & DIRTY) == 0) __hip_atomic_fetch_or(&dp->state, DIRTY, __ATOMIC_RELAXED, BAM_AGENT);
        slot = (uint32_t)(sv >> 32) & BAM_SLOT_MASK;
        was_hit = true;
        resolved = true;
    } else if (st == NV_NB) {
        if (!may_load) {
            *wants_load = true;                 /* the caller has to be admitted to the miss path first */
        } else {
            const uint32_t o = __hip_atomic_fetch_or(&dp->state, BUSY, __ATOMIC_RELAXED, BAM_AGENT);
            if ((o & BUSY) == 0) {
                if ((o >> (CNT_SHIFT + 1)) == NV_NB) load_me = true;
                else __hip_atomic_fetch_and(&dp->state, DISABLE_BUSY_MASK, __ATOMIC_RELAXED, BAM_AGENT);  /* became valid meanwhile */
            }
        }
    }
    uint32_t found = BAM_NO_SLOT, cid = 0;
    uint8_t* stage = nullptr;
    QueuePair* qp = nullptr;
    bool held = false, io_ok = false;
    if (load_me) {
#ifdef BAM_PROFILE
        const uint64_t pf0 = wall_clock64();
#endif
        found = cache.find_slot(pg, range_id, queue);
#ifdef BAM_PROFILE
        if (cache.prof && bam::lane() == bam::first_lane(bam::active_mask())) { atomicAdd(&cache.prof[6], wall_clock64() - pf0); atomicAdd(&cache.prof[7], 1ull); atomicAdd(&cache.prof[8], (unsigned long long)bam::popc(bam::active_mask())); }
#endif
        if (found == BAM_NO_SLOT) {
            /* no evictable slot right now: hand the page back; a later pass tries again */
            __hip_atomic_fetch_and(&dp->state, DISABLE_BUSY_MASK, __ATOMIC_RELAXED, BAM_AGENT);
            load_me = false;
        } else {
            uint64_t c = get_backing_ctrl(pg);
            if (c == ALL_CTRLS) c = cache.n_ctrls == 1 ? 0 : cache.ctrl_counter->fetch_add(1, simt::memory_order_relaxed) % cache.n_ctrls;
            Controller* ctl = cache.d_ctrls[c];
            stat_add((unsigned long long*)&ctl->access_counter, 1);
            stat_add(&shard()->read_io_cnt, 1);
            qp = ctl->d_qps + (queue % ctl->n_qps);
            read_begin(&cache, qp, get_backing_page(pg) * cache.n_blocks_per_page, cache.n_blocks_per_page, found, cid, stage, held, io_ok, ahead);
        }
    }
    /* staged payload is moved by every lane that came in, whether it loaded a page itself or not */
#ifdef BAM_PROFILE
    const uint64_t pc0 = wall_clock64();
#endif
    if (bam::ballot(load_me && io_ok && stage != nullptr)) {
        /* all lanes that came in are here: the queue pair of any lane that has payload to move will do for the permission */
        QueuePair* pq = (QueuePair*)bam::bcast((uint64_t)qp, bam::first_lane(bam::ballot(load_me && io_ok && stage != nullptr)));
        uint32_t* pull = bam::pull_begin(pq);
        [[maybe_unused]] const uint64_t pp0 = BAM_PROF_NOW();
        copy_pages_helped(cache.base_addr + (uint64_t)found * cache.page_size, stage, (uint32_t)cache.page_size, load_me && io_ok && stage != nullptr);
#ifdef BAM_PROFILE
        {
            const uint64_t pp1 = BAM_PROF_NOW(), pulled = bam::popc(bam::ballot(load_me && io_ok && stage != nullptr));
            if (cache.prof && bam::lane() == bam::first_lane(bam::active_mask())) { atomicAdd(&cache.prof[29], pp1 - pp0); atomicAdd(&cache.prof[30], (unsigned long long)pulled); }
        }
#endif
        bam::pull_end(pull);
    }
#ifdef BAM_PROFILE
    if (cache.prof && bam::ballot(load_me) && bam::lane() == bam::first_lane(bam::active_mask())) atomicAdd(&cache.prof[5], wall_clock64() - pc0);
#endif
    if (load_me) {
        if (held) read_end(qp, cid);
        if (!io_ok) {
            /*
             * The read did not happen (error completion) or nobody knows whether it did (the wait was given up): the
             * page must not show as valid with whatever the slot or the staging page held before.  The slot goes back
             * to the free ones and the page stays invalid; the caller's next pass finds it so and tries again, or, after
             * a wait that was given up, finds the abort flag.  While this lane holds BUSY nobody else takes the slot
             * (an evictor that lands on it finds its page busy and moves on), so its lock is free within a few steps.
             */
            cache_page_t* cp = &cache.cache_pages[found];
            bam::spin_t lk;
            bool locked = false;
            while (!locked) {
                locked = (__hip_atomic_fetch_or(&cp->page_translation, (uint64_t)LOCKED << BAM_TAKE_SHIFT, __ATOMIC_RELAXED, BAM_AGENT) >> BAM_TAKE_SHIFT) == UNLOCKED;
                if (!locked && cache.spin_giveup(lk)) break;
            }
            if (locked) st_relaxed(&cp->page_translation, (uint64_t)FREE << BAM_TAKE_SHIFT);
            fence_meta();
            __hip_atomic_fetch_and(&dp->state, DISABLE_BUSY_MASK, __ATOMIC_RELAXED, BAM_AGENT);
        } else {
            /* the slot, and one more load of this page on the count above it (this lane owns the descriptor while BUSY is set) */
            st_relaxed(&dp->offset, found | (((ld_relaxed(&dp->offset) >> BAM_SLOT_BITS) + 1u) << BAM_SLOT_BITS));
            if (write) __hip_atomic_fetch_or(&dp->state, DIRTY, __ATOMIC_RELAXED, BAM_AGENT);
        }
    }
    /* payload this wave (helpers included) moved in went through to memory (copy_pages): once the wave's store counter
     * is down it is there for every compute unit; payload the controller placed is in memory already */
    if (bam::ballot(load_me && io_ok)) fence_meta();
    if (load_me && io_ok) {
        /* BUSY -> 0 and VALID -> 1 in one step; publishes the payload and the offset */
        __hip_atomic_fetch_xor(&dp->state, DISABLE_BUSY_ENABLE_VALID, __ATOMIC_RELAXED, BAM_AGENT);
        slot = found;
        was_hit = false;
        resolved = true;
        progressed = true;
    }
    if (take_part && !resolved) sv = __hip_atomic_load((uint64_t*)dp, __ATOMIC_RELAXED, BAM_AGENT);
    return resolved;
}

/*
 * slow_step as a function of its own, values in and values out.  It holds everything that is heavy in registers
 * (victim search, command submission, completion handling, payload copy); kept out of line, the callers' path for
 * resident pages stays lean, and what has to be saved around the call is saved on the miss path only.
 */
struct bam_pass_t { uint64_t sv; uint32_t slot; uint32_t flags; };
#define BAM_PASS_RESOLVED   1u
#define BAM_PASS_HIT        2u
#define BAM_PASS_PROGRESSED 4u
#define BAM_PASS_WANTS      8u
#define BAM_PASS_WRITE      16u     /* in: */
#define BAM_PASS_TAKE_PART  32u
#define BAM_PASS_MAY_LOAD   64u
#define BAM_PASS_AHEAD      128u    /* the caller fetches for others (placement: page_cache_d_t::direct_limit_ahead) */
template <typename T>
__forceinline__ __device__ bam_pass_t bam_slow_pass_inline(range_d_t<T>* r, const uint64_t pg, const uint32_t queue, uint64_t sv, uint32_t slot, const uint32_t in)
{
    bool hit = false, progressed = false, wants = false;
    const bool resolved = r->slow_step(pg, (in & BAM_PASS_WRITE) != 0, queue, sv, slot, hit, progressed, (in & BAM_PASS_TAKE_PART) != 0,
                                       (in & BAM_PASS_MAY_LOAD) != 0, &wants, (in & BAM_PASS_AHEAD) != 0);
    bam_pass_t out;
    out.sv = sv;
    out.slot = slot;
    out.flags = (resolved ? BAM_PASS_RESOLVED : 0u) | (hit ? BAM_PASS_HIT : 0u) | (progressed ? BAM_PASS_PROGRESSED : 0u) | (wants ? BAM_PASS_WANTS : 0u);
    return out;
}
template <typename T>
__attribute__((noinline)) __device__ bam_pass_t bam_slow_pass_call(range_d_t<T>* r, const uint64_t pg, const uint32_t queue, uint64_t sv, uint32_t slot, const uint32_t in)
{
    return bam_slow_pass_inline(r, pg, queue, sv, slot, in);
}
/* OUTLINE: as a call (measured best for kernels that are mostly misses: one thread per random element) or expanded in
 * place (best where the caller is mostly hits and would otherwise carry the callee's register budget) */
template <bool OUTLINE, typename T>
__forceinline__ __device__ bam_pass_t bam_slow_pass(range_d_t<T>* r, const uint64_t pg, const uint32_t queue, uint64_t sv, uint32_t slot, const uint32_t in)
{
    if constexpr (OUTLINE) return bam_slow_pass_call(r, pg, queue, sv, slot, in);
    else return bam_slow_pass_inline(r, pg, queue, sv, slot, in);
}

/* the reference's entry point: references + slot, and the access is accounted in the range's counters; BAM_NO_SLOT
 * (with the references taken all the same) when the wait for the page was given up */
template <typename T>
__forceinline__ __device__
uint64_t range_d_t<T>::acquire_page(const size_t pg, const uint32_t count, const bool write, const uint32_t ctrl_, const uint32_t queue)
{
    (void)ctrl_;
    uint64_t sv;
    uint32_t slot = 0;
    bool hit = bam_try_hit(&pages[pg], count, write, sv, slot);
    if (!hit) {
        /* every lane keeps its references until all are in: callers of this entry point hold pages anyway */
        bool resolved = false;
        bam::spin_t sp;
        for (;;) {
            /* resolved lanes go in too: they help move payload */
            const bam_pass_t ps = bam_slow_pass<false>(this, pg, queue, sv, slot, (write ? BAM_PASS_WRITE : 0u) | (resolved ? 0u : BAM_PASS_TAKE_PART) | BAM_PASS_MAY_LOAD);
            const bool progressed = (ps.flags & BAM_PASS_PROGRESSED) != 0;
            if (!resolved) { sv = ps.sv; slot = ps.slot; hit = (ps.flags & BAM_PASS_HIT) != 0; resolved = (ps.flags & BAM_PASS_RESOLVED) != 0; }
            if (!bam::ballot(!resolved)) break;
            if (!bam::ballot(progressed) && cache.spin_giveup(sp)) { if (!resolved) slot = BAM_NO_SLOT; break; }
        }
    }
    bam_stat_shard_t* sh = shard();
    bam::stat_add(&sh->access_cnt, count);
    bam::stat_add(&sh->hit_cnt, hit ? count : 0);
    return slot;
}

/* ------------------------------------------------------------------ */
/* arrays                                                             */
/* ------------------------------------------------------------------ */

namespace bam {
/*
 * What the device path needs to know about a range, read once and kept in
 * registers: a kernel that walks an array re-derives page numbers and
 * addresses from these instead of re-reading the descriptors from memory
 * around every atomic.
 */
template <typename T>
struct range_view {
    range_d_t<T>* r = nullptr;       /* full descriptor, for the miss path */
    data_page_t* pages;
    uint8_t* base_addr;
    uint64_t index_start, index_end, pso;
    uint32_t page_size_log, page_size;
    uint32_t n_access = 0, n_hit = 0;   /* this lane's accesses since the last flush_stats() */
    bool read_ahead = false;            /* set by waves that fetch for others: their batches may be placed directly up to the higher bound */

    __forceinline__ __device__ void load(range_d_t<T>* r_)
    {
        flush_stats();
        r = r_;
        fill();
    }
    /*
     * The descriptor read (again).  Also called at the end of the miss path: what is read again there need not be
     * kept in registers over the passes of that path, which is a call, and a value that lives across a call costs
     * the caller a register the callee must not touch, of which there are few.  The path for resident pages, which
     * has no call, then has the registers of a kernel with four waves per SIMD instead of three.
     */
    __forceinline__ __device__ void fill()
    {
        range_d_t<T>* const r_ = r;
        pages = r_->pages;
        base_addr = r_->cache.base_addr;
        index_start = r_->index_start;
        index_end = r_->count;
        pso = r_->page_start_offset;
        page_size_log = (uint32_t)r_->cache.page_size_log;
        page_size = (uint32_t)r_->cache.page_size;
    }
    __forceinline__ __device__ bool holds(const size_t i) const { return r && i >= index_start && i < index_end; }
    __forceinline__ __device__ uint64_t byte_of(const size_t i) const { return (i - index_start) * sizeof(T) + pso; }
    __forceinline__ __device__ uint64_t page_of(const size_t i) const { return byte_of(i) >> page_size_log; }
    __forceinline__ __device__ uint8_t* slot_addr(const uint32_t slot) const { return base_addr + ((uint64_t)slot << page_size_log); }
    /* element window [start, end) covered by `page`, clipped to the range */
    __forceinline__ __device__ void window(const uint64_t page, size_t& start, size_t& end) const
    {
        const uint64_t first_byte = page << page_size_log;
        start = index_start + (first_byte <= pso ? 0 : (first_byte - pso + sizeof(T) - 1) / sizeof(T));
        end = index_start + (first_byte + page_size - pso) / sizeof(T);
        if (end > index_end) end = index_end;
    }
    /*
     * One access per active lane, hit or miss as its group's master found the
     * page.  Counted in registers; flush_stats() adds the lanes' totals to the
     * range's counters with one atomic per counter per wave.  Misses are not
     * counted separately: every access is either one or the other.
     */
    __forceinline__ __device__ void account(const bool hit) { n_access++; n_hit += hit ? 1u : 0u; }

    /* WIDE: the lanes may hold more than one access each (a view that lived through many acquires) */
    template <bool WIDE = true>
    __forceinline__ __device__ void flush_stats() { flush_stats_bits<WIDE ? 32 : 1>(); }
    /* every lane holds fewer than 2^BITS accesses */
    template <int BITS>
    __forceinline__ __device__ void flush_stats_bits()
    {
        if (!r) return;
        bam_stat_shard_t* const shard = r->shard();      /* looked up here, once in a view's life, rather than carried along */
        stat_add<BITS>(&shard->access_cnt, n_access);
        stat_add<BITS>(&shard->hit_cnt, n_hit);
        n_access = n_hit = 0;
    }

    /*
     * Wave-level request coalescing + acquire.  Lanes that want the same page
     * form a group; the lowest lane of each group (its master) takes the
     * group's references with one atomic.  Groups whose page is resident are
     * served first: `on_hit(slot)` runs for their lanes and, if it returns
     * true, their references are dropped right away.  Only then do the
     * masters of the remaining groups go through the miss path together, so a
     * wave that waits for I/O holds no reference on anything but the pages it
     * is loading.  `on_miss(slot)` runs for those lanes once their page is in.
     */
    template <bool OUTLINE = false, typename FH, typename FM>
    __forceinline__ __device__ void acquire(const uint64_t page, const bool write, FH&& on_hit, FM&& on_miss)
    {
        acquire_<OUTLINE, false>(page, write, on_hit, on_miss, true);
    }
    /*
     * The same for callers of which only some lanes want a page (`take`): the others come along to help.  A wave that
     * touches two or three pages ahead of its work would otherwise have each staged page moved by the two or three
     * lanes that asked, sixty-four round trips over the interconnect per page instead of one.
     */
    template <bool OUTLINE = false, typename FH, typename FM>
    __forceinline__ __device__ void acquire_helped(const uint64_t page, const bool take, const bool write, FH&& on_hit, FM&& on_miss)
    {
        acquire_<OUTLINE, true>(page, write, on_hit, on_miss, take);
    }
    template <bool OUTLINE, bool HELPERS, typename FH, typename FM>
    __forceinline__ __device__ void acquire_(const uint64_t page_, const bool write, FH&& on_hit, FM&& on_miss, const bool take)
    {
        const uint32_t me = lane();
        /* helpers form a group of their own on a page number no range has; they take nothing */
        const uint64_t page = HELPERS && !take ? ~0ull : page_;
        /* lanes with the same page of the same range have the same descriptor, and only they */
        data_page_t* dp = pages + page;
        const uint64_t eq_mask = match_any(HELPERS && !take ? 0ull : (uint64_t)dp);
        const uint32_t master = first_lane(eq_mask), count = popc(eq_mask);
        const bool dirty = (ballot(write) & eq_mask) != 0;
        uint64_t sv = 0, pack = 0;
        uint32_t slot = 0;
        if (master == me && (!HELPERS || take)) { const bool h = bam_try_hit(dp, count, dirty, sv, slot); pack = (uint64_t)slot | ((uint64_t)h << 63); }
        pack = shfl(pack, master);
        if (__builtin_expect((pack >> 63) != 0, 1)) {          /* resident: the path to keep lean; register spills, if any, belong in the other branch */
            account(true);
            const bool drop = on_hit((uint32_t)pack);
            /* the lanes of a group may answer differently (one keeps the page, another only touched it) */
            const uint32_t n_drop = popc(ballot(drop) & eq_mask);
            if (n_drop && master == me) bam_release_refs(dp, n_drop, dirty);
        } else {
            /* miss path: pass after pass; groups whose page came in are served and release before the next pass */
            const uint32_t queue = wave_slot_hash();
            const uint32_t leader = first_lane(active_mask());
            bool done = HELPERS && !take;
            spin_t sp;
            /*
             * Admission: only so many waves per compute unit load pages at a time.  Every wave that has I/O in
             * flight polls queues and command words; with all resident waves doing that at once the polling itself
             * takes the memory system and the interconnect away from the waves that are moving payload, and
             * throughput drops.  A wave asks for admission when one of its pages is there to be loaded, and steps
             * out again whenever it finds itself only waiting for pages that other waves are loading.  One counter
             * per compute unit, 64 bytes apart: waiting waves poll their own unit's word.
             */
            page_cache_d_t* cache = (page_cache_d_t*)first((uint64_t)&r->cache);
            const uint32_t limit = cache->miss_waves;
            uint32_t* tokens = cache->miss_tokens + (cu_id() & (BAM_TOKEN_SLOTS - 1)) * 16;
            bool admitted = limit == 0;
            if (!HELPERS || ballot(!done))          /* helpers alone: nobody missed, nothing to help with */
            for (;;) {
                /* every lane of the miss branch goes in: the masters that still wait for their page take part, the rest help move payload */
                const bool part = !done && master == me;
                const bam_pass_t ps = bam_slow_pass<OUTLINE>(r, page, queue, sv, slot,
                                                    (dirty ? BAM_PASS_WRITE : 0u) | (part ? BAM_PASS_TAKE_PART : 0u) | (admitted ? BAM_PASS_MAY_LOAD : 0u) |
                                                    (read_ahead ? BAM_PASS_AHEAD : 0u));
                const bool progressed = (ps.flags & BAM_PASS_PROGRESSED) != 0, wants = (ps.flags & BAM_PASS_WANTS) != 0;
                if (part) {
                    sv = ps.sv;
                    pack = (uint64_t)ps.slot | ((uint64_t)((ps.flags & BAM_PASS_HIT) != 0) << 63) | ((uint64_t)((ps.flags & BAM_PASS_RESOLVED) != 0) << 62);
                }
                if (!done) {
                    pack = shfl(pack, master);
                    if ((pack >> 62) & 1) {
                        account((pack >> 63) != 0);
                        const bool drop = on_miss((uint32_t)pack);
                        const uint32_t n_drop = popc(ballot(drop) & eq_mask);
                        if (n_drop && master == me) bam_release_refs(dp, n_drop, dirty);
                        done = true;
                    }
                }
                if (!ballot(!done)) break;
                if (!admitted && ballot(wants)) {
                    const bool holder = !done && master == me;                 /* lanes that hold their group's references */
                    uint32_t ok = 0;
                    if (me == leader) {
                        if (__hip_atomic_fetch_add(tokens, 1u, __ATOMIC_RELAXED, BAM_AGENT) < limit) ok = 1;
                        else __hip_atomic_fetch_add(tokens, 0u - 1u, __ATOMIC_RELAXED, BAM_AGENT);
                    }
                    if (!bcast(ok, leader)) {
                        /*
                         * Queue up without references: a page that somebody else brings in meanwhile must stay
                         * evictable, or the waves that wait here could pin every slot the admitted ones need.
                         */
                        if (holder) __hip_atomic_fetch_add(&dp->state, 0u - count, __ATOMIC_RELAXED, BAM_AGENT);
                        if (me == leader) {
                            for (uint32_t i = 1;; i++) {
                                if (ld_relaxed(tokens) < limit) {
                                    if (__hip_atomic_fetch_add(tokens, 1u, __ATOMIC_RELAXED, BAM_AGENT) < limit) { ok = 1; break; }
                                    __hip_atomic_fetch_add(tokens, 0u - 1u, __ATOMIC_RELAXED, BAM_AGENT);
                                }
                                __builtin_amdgcn_s_sleep(127);
                                __builtin_amdgcn_s_sleep(127);
                                __builtin_amdgcn_s_sleep(127);
                                __builtin_amdgcn_s_sleep(127);
                                /* no clock of its own: the waves inside time their waits, this one only watches for their outcome */
                                if ((i & 15u) == 0 && cache->guard && ld_relaxed_sys(&cache->guard->abort)) break;
                            }
                        }
                        if (holder) bam_try_hit(dp, count, dirty, sv, slot);   /* the next pass reads the outcome from sv */
                    }
                    admitted = bcast(ok, leader) != 0;
                    if (!admitted) break;                                      /* only an abort ends the wait without admission */
                    continue;
                }
                if (ballot(progressed)) sp = spin_t();
                else {
                    /* only waiting for pages other waves are loading: make room for a wave that has something to load */
                    if (limit && admitted) {
                        if (me == leader) __hip_atomic_fetch_add(tokens, 0u - 1u, __ATOMIC_RELAXED, BAM_AGENT);
                        admitted = false;
                    }
                    if (cache->spin_giveup(sp)) break;
                }
            }
            if (limit && admitted && me == leader) __hip_atomic_fetch_add(tokens, 0u - 1u, __ATOMIC_RELAXED, BAM_AGENT);
            fill();
        }
    }

    /* drop the reference each active lane holds on `page` (one atomic per group of lanes on the same page) */
    __forceinline__ __device__ void release(const uint64_t page, const bool wrote) const
    {
        const uint64_t eq_mask = match_any((uint64_t)(pages + page));
        const bool any_wrote = (ballot(wrote) & eq_mask) != 0;
        if (first_lane(eq_mask) == lane()) bam_release_refs(pages + page, popc(eq_mask), any_wrote);
    }
};
} // namespace bam

template <typename T>
struct array_d_t {
    uint64_t n_elems;
    uint64_t start_offset;
    uint64_t n_ranges;
    uint8_t* src;
    range_d_t<T>* d_ranges;

    __forceinline__ __device__ int64_t find_range(const size_t i) const
    {
        for (int64_t k = 0; k < (int64_t)n_ranges; k++)
            if (d_ranges[k].index_start <= i && d_ranges[k].count > i) return k;
        return -1;
    }

    /* the view of the range holding element i; false if no range does */
    __forceinline__ __device__ bool view_of(const size_t i, bam::range_view<T>& v) const
    {
        const int64_t r = find_range(i);
        if (r == -1) return false;
        v.load(d_ranges + r);
        return true;
    }

    /*
     * The reference's coalescing entry point (include/page_cache.h:1330-1366):
     * eq_mask/master/count describe the caller's group of same-page lanes,
     * base_master is the cache slot; the group's references stay taken.
     */
    __forceinline__ __device__ void coalesce_page(const uint32_t lane, const uint64_t mask, const int64_t r, const uint64_t page, const uint64_t gaddr, const bool write,
                                                  uint64_t& eq_mask, int& master, uint32_t& count, uint64_t& base_master) const
    {
        (void)mask; (void)lane; (void)gaddr;
        bam::range_view<T> v;
        v.load(d_ranges + r);
        eq_mask = bam::match_any(page, (uint64_t)v.r);
        master = (int)bam::first_lane(eq_mask);
        count = bam::popc(eq_mask);
        uint32_t slot = BAM_NO_SLOT;
        auto keep = [&](uint32_t s_) { slot = s_; return false; };
        v.acquire(page, write, keep, keep);
        v.template flush_stats<false>();
        base_master = slot;                     /* BAM_NO_SLOT if the wait for the page was given up */
    }

    /* run fn(address of element i in the cache) with the page referenced, for every active lane */
    template <typename F>
    __forceinline__ __device__ void with_element(const size_t i, const bool write, F&& fn) const
    {
        bam::range_view<T> v;
        if (!view_of(i, v)) return;
        const uint64_t byte = v.byte_of(i);
        auto use = [&](uint32_t slot) { fn((T*)(v.slot_addr(slot) + (byte & (v.page_size - 1)))); return true; };
        v.template acquire<true>(byte >> v.page_size_log, write, use, use);
        v.template flush_stats<false>();
    }

    __forceinline__ __device__ T seq_read(const size_t i) const
    {
        T ret = T();
        bam::range_view<T> v;
        if (!view_of(i, v)) return ret;
        const uint64_t byte = v.byte_of(i);
        /* resident pages are read without a reference (each lane for itself: lanes on one page load the same descriptor
         * word, which costs the memory system one access); what is left goes the counted way, coalesced */
        bool got = false;
        if (v.r->cache.fast_reads) {
            got = bam_read_unpinned(v.pages + (byte >> v.page_size_log), v.base_addr, v.page_size_log, byte & (v.page_size - 1), ret);
            if (got) v.account(true);
        }
        if (!got) {
            auto use = [&](uint32_t slot) { ret = bam::ld_payload((T*)(v.slot_addr(slot) + (byte & (v.page_size - 1)))); return true; };
            v.template acquire<true>(byte >> v.page_size_log, false, use, use);
        }
        v.template flush_stats<false>();
        return ret;
    }

    /*
     * N reads per lane, the looks and loads of the unpinned route issued side by side: a read of a resident page is three
     * dependent trips to memory (descriptor, element, descriptor again), and a lane that does them for one element at a
     * time has one request in flight; N elements share the three waits.  out[j] for the j with want[j]; what is not
     * resident goes the counted way one element after the other.  Same results and counters as N calls of seq_read.
     */
    template <int N>
    __forceinline__ __device__ void seq_read_n(const size_t (&idx)[N], const bool (&want)[N], T (&out)[N]) const
    {
        bam::range_view<T> v;
        if (n_ranges == 1) v.load(d_ranges);
        seq_read_n(idx, want, out, v);
        v.template flush_stats_bits<(N < 8 ? 3 : 4)>();
    }
    /*
     * The same with the caller's view of the array's one range (`v.r` null: the array has several, and every read goes
     * the counted way): a kernel that makes many such calls reads the range's descriptor once, and its lanes count their
     * accesses in the view until the caller flushes it (range_view::flush_stats).
     */
    template <int N>
    __forceinline__ __device__ void seq_read_n(const size_t (&idx)[N], const bool (&want)[N], T (&out)[N], bam::range_view<T>& v) const
    {
        static_assert(N >= 1 && N <= 15, "the counters of the plain form are flushed with three or four ballots");
        bool got[N];
        seq_read_n_resident(idx, want, out, got, v);
#pragma unroll
        for (int j = 0; j < N; j++)
            if (want[j] && !got[j]) out[j] = seq_read_call(idx[j]);
    }
    /*
     * The half of seq_read_n that cannot miss: out[j] and got[j] = true for the elements that were read from resident
     * pages (and counted as hits in the view); got[j] = false for the others, which nothing was done for.  No call, no
     * atomic, no store: a kernel made of this alone (the first of two launches, the second reading what this one could
     * not) needs a fraction of the registers of one that can miss.  The view is that of the array's one range.
     */
    template <int N, bool SCATTERED = false>
    __forceinline__ __device__ void seq_read_n_resident(const size_t (&idx)[N], const bool (&want)[N], T (&out)[N], bool (&got)[N], bam::range_view<T>& v) const
    {
        const bool one = v.r != nullptr;
#pragma unroll
        for (int j = 0; j < N; j++) { got[j] = false; out[j] = T(); }
        if constexpr (SCATTERED && sizeof(T) == 8 && (N == 1 || N == 2 || N == 4 || N == 8)) {
            /* elements anywhere in the array (a gather): no two are expected on one page, so every element has its own looks,
             * and every lane makes every load (one with nothing to read looks at the first page's descriptor and loads the
             * cache's first word): three rounds of N loads with nothing but arithmetic between them */
            if (one && v.r->cache.fast_reads) {
                const data_page_t* dp[N];
                const uint64_t* p[N];
                uint64_t s1[N], x[N];
                uint32_t in_page[N];
                bool res[N];
#pragma unroll
                for (int j = 0; j < N; j++) {
                    res[j] = want[j] && idx[j] - v.index_start < v.index_end - v.index_start;
                    const uint64_t byte = res[j] ? v.byte_of(idx[j]) : 0;
                    dp[j] = v.pages + (byte >> v.page_size_log);
                    in_page[j] = (uint32_t)byte & (v.page_size - 1);
                }
#pragma unroll
                for (int j = 0; j < N; j++) s1[j] = __hip_atomic_load((const uint64_t*)dp[j], __ATOMIC_RELAXED, BAM_AGENT);
#pragma unroll
                for (int j = 0; j < N; j++) asm volatile("" : "+v"(s1[j]));
#pragma unroll
                for (int j = 0; j < N; j++) {
                    res[j] = res[j] & (((uint32_t)s1[j] >> (CNT_SHIFT + 1)) == V_NB);
                    p[j] = (const uint64_t*)(v.base_addr + (res[j] ? ((uint64_t)((uint32_t)(s1[j] >> 32) & BAM_SLOT_MASK) << v.page_size_log) + in_page[j] : 0));
                }
                bam::ld_payload_nt(p, x);               /* with its wait: the elements are here before the second looks go out */
                uint64_t s2[N];
#pragma unroll
                for (int j = 0; j < N; j++) s2[j] = __hip_atomic_load((const uint64_t*)dp[j], __ATOMIC_RELAXED, BAM_AGENT);
                /* all N looks are out before the first is used (left to itself the compiler moves each look into the branch
                 * that uses it, one wait per look) */
#pragma unroll
                for (int j = 0; j < N; j++) asm volatile("" : "+v"(s2[j]));
#pragma unroll
                for (int j = 0; j < N; j++) {
                    got[j] = res[j] & (((s1[j] ^ s2[j]) & 0xFFFFFFFFC0000000ull) == 0);
                    out[j] = got[j] ? *(T*)&x[j] : T();
                    v.n_access += got[j] ? 1u : 0u;
                    v.n_hit += got[j] ? 1u : 0u;
                }
            }
            return;
        }
        if (one && v.r->cache.fast_reads) {
            uint64_t s1[N], byte[N];
            bool res[N], again[N];
            /* an element on the page of the one before it (a lane that reads along an array) shares that one's two
             * looks at the descriptor: what holds for the page holds for both */
#pragma unroll
            for (int j = 0; j < N; j++) {
                res[j] = want[j] && v.index_start <= idx[j] && v.index_end > idx[j];
                byte[j] = res[j] ? v.byte_of(idx[j]) : 0;
                again[j] = j > 0 && res[j] && res[j - 1] && (byte[j] >> v.page_size_log) == (byte[j - 1] >> v.page_size_log);
                s1[j] = 0;
                if (again[j]) s1[j] = s1[j - 1];
                else if (res[j]) s1[j] = __hip_atomic_load((const uint64_t*)(v.pages + (byte[j] >> v.page_size_log)), __ATOMIC_RELAXED, BAM_AGENT);
            }
#pragma unroll
            for (int j = 0; j < N; j++) res[j] = res[j] && ((uint32_t)s1[j] >> (CNT_SHIFT + 1)) == V_NB;
            if constexpr (sizeof(T) == 8 && (N == 1 || N == 2 || N == 4 || N == 8)) {
                /* scattered 8-byte elements: loaded as not to be kept, all behind one wait (lanes with nothing to read load
                 * the cache's first word and drop it) */
                const uint64_t* p[N];
                uint64_t x[N];
#pragma unroll
                for (int j = 0; j < N; j++)
                    p[j] = (const uint64_t*)(v.base_addr + (res[j] ? ((uint64_t)((uint32_t)(s1[j] >> 32) & BAM_SLOT_MASK) << v.page_size_log) + (byte[j] & (v.page_size - 1)) : 0));
                bam::ld_payload_nt(p, x);               /* with its wait: the elements are here before the second looks go out */
#pragma unroll
                for (int j = 0; j < N; j++) if (res[j]) out[j] = *(T*)&x[j];
            } else {
#pragma unroll
                for (int j = 0; j < N; j++)
                    if (res[j]) out[j] = bam::ld_payload((const T*)(v.base_addr + ((uint64_t)((uint32_t)(s1[j] >> 32) & BAM_SLOT_MASK) << v.page_size_log) + (byte[j] & (v.page_size - 1))));
                bam::fence_meta();                       /* the elements are here before the second looks go out */
            }
            uint64_t s2 = 0;                            /* the second look of the element before, for one that shares it */
#pragma unroll
            for (int j = 0; j < N; j++) {
                if (!again[j]) {
                    s2 = ~s1[j];
                    if (res[j]) s2 = __hip_atomic_load((const uint64_t*)(v.pages + (byte[j] >> v.page_size_log)), __ATOMIC_RELAXED, BAM_AGENT);
                }
                got[j] = res[j] && ((s1[j] ^ s2) & 0xFFFFFFFFC0000000ull) == 0;
                if (got[j]) v.account(true);
            }
        }
    }
    /* seq_read as a call: the N places above where an element goes the counted way would otherwise each carry the whole
     * of that path, and its registers with it */
    __attribute__((noinline)) __device__ T seq_read_call(const size_t i) const { return seq_read(i); }

    __forceinline__ __device__ void seq_write(const size_t i, const T val) const
    {
        with_element(i, true, [&](T* p) { *p = val; });
    }

    __forceinline__ __device__ T AtomicAdd(const size_t i, const T val) const
    {
        T old = T();
        with_element(i, true, [&](T* p) { old = atomicAdd(p, val); });
        return old;
    }

    __forceinline__ __device__ T operator[](size_t i) const { return seq_read(i); }
    __forceinline__ __device__ void operator()(size_t i, T val) const { seq_write(i, val); }

    /*
     * Reference the page holding element i and keep it referenced: returns the
     * address of the first element of the window [start, end) the page covers,
     * the page descriptor and the range index.  Pair with release_page.
     */
    __forceinline__ __device__ void* acquire_page(const size_t i, data_page_t*& page_, size_t& start, size_t& end, int64_t& r) const
    {
        r = find_range(i);
        page_ = nullptr;
        if (r == -1) return nullptr;
        bam::range_view<T> v;
        v.load(d_ranges + r);
        const uint64_t page = v.page_of(i);
        uint32_t slot = BAM_NO_SLOT;
        auto keep = [&](uint32_t s_) { slot = s_; return false; };
        v.acquire(page, false, keep, keep);
        v.template flush_stats<false>();
        page_ = v.pages + page;
        v.window(page, start, end);
        if (slot == BAM_NO_SLOT) { start = end = 0; return nullptr; }        /* wait given up; the references stay counted: release_page as usual */
        return (void*)(v.slot_addr(slot) + (v.byte_of(start) & (v.page_size - 1)));
    }

    __forceinline__ __device__ void release_page(data_page_t* page_, const int64_t r, const size_t i, const bool wrote = true) const
    {
        (void)page_;
        if (r == -1) return;
        bam::range_view<T> v;
        v.load(d_ranges + r);
        v.release(v.page_of(i), wrote);
    }

    /* range, page within the range and global page address of element i (reference :1240-1253); r_ = NULL if no range holds i */
    __forceinline__ __device__ void get_page_gid(const uint64_t i, range_d_t<T>*& r_, size_t& pg, size_t& gid) const
    {
        const int64_t r = find_range(i);
        r_ = nullptr;
        if (r == -1) return;
        r_ = d_ranges + r;
        pg = r_->get_page(i);
        gid = r_->get_global_address(pg);
    }

    /*
     * Per-thread acquire of `page` of range `r_`, no coalescing across lanes (reference :1443-1468): one reference
     * per calling lane.  Returns the address of the page's payload, its descriptor in `page_` and the element
     * window [start, end) it covers.  The reference indexes the descriptor table by the cache slot here
     * (`&r_->pages[base_master]`); this returns the descriptor of the page, which is what its callers release.
     */
    __forceinline__ __device__ void* acquire_page_(const size_t i, data_page_t*& page_, size_t& start, size_t& end, range_d_t<T>* r_, const size_t page) const
    {
        (void)i;
        page_ = nullptr;
        if (!r_) return nullptr;
        const uint32_t slot = (uint32_t)r_->acquire_page(page, 1, false, 0, bam::wave_slot_hash());
        page_ = &r_->pages[page];
        bam::range_view<T> v;
        v.load(r_);
        v.window(page, start, end);
        if (slot == BAM_NO_SLOT) { start = end = 0; return nullptr; }        /* the reference is held all the same: release_page as usual */
        return (void*)(v.slot_addr(slot) + (v.byte_of(start) & (v.page_size - 1)));
    }

    /*
     * The page holding element i, handed out raw (reference :1370-1403): address of the page's payload, its size
     * in elements and the position of element i in it.  The references of the lanes that ask for the same page
     * are taken with one atomic and stay taken until release_raw(i) is called by the same lanes.
     */
    __forceinline__ __device__ returned_cache_page_t<T> get_raw(const size_t i) const
    {
        returned_cache_page_t<T> ret;
        ret.addr = nullptr; ret.size = 0; ret.offset = 0;
        bam::range_view<T> v;
        if (!view_of(i, v)) return ret;
        const uint64_t byte = v.byte_of(i);
        uint32_t slot = BAM_NO_SLOT;
        auto keep = [&](uint32_t s_) { slot = s_; return false; };
        v.acquire(byte >> v.page_size_log, false, keep, keep);
        v.template flush_stats<false>();
        if (slot == BAM_NO_SLOT) return ret;         /* wait given up: addr NULL, size 0; release_raw as usual */
        ret.addr = (T*)v.slot_addr(slot);
        ret.size = v.page_size / sizeof(T);
        ret.offset = (uint32_t)((byte & (v.page_size - 1)) / sizeof(T));
        return ret;
    }

    __forceinline__ __device__ void release_raw(const size_t i) const
    {
        bam::range_view<T> v;
        if (!view_of(i, v)) return;
        v.release(v.page_of(i), false);
    }

    /*
     * Wave-cooperative copy out of the cache: the active lanes, all called with the same i, copy `count` elements
     * starting at element i to `dest`, clipped to the end of the page that holds i.  (The reference's version,
     * :1256-1316, ignores `count` and always copies the first 512 bytes of the page.)
     */
    __forceinline__ __device__ void memcpy(const uint64_t i, const uint64_t count, T* dest) const
    {
        bam::range_view<T> v;
        if (!view_of(i, v)) return;
        const uint64_t byte = v.byte_of(i);
        const uint64_t page = byte >> v.page_size_log;
        size_t start, end;
        v.window(page, start, end);
        const uint64_t n = i + count < end ? count : end - i;
        const uint64_t act = bam::active_mask();
        const uint32_t lanes = bam::popc(act), rank = bam::rank_in(act);
        auto copy = [&](uint32_t slot) {
            const T* src = (const T*)(v.slot_addr(slot) + (byte & (v.page_size - 1)));
            for (uint64_t k = rank; k < n; k += lanes) dest[k] = bam::ld_payload(src + k);
            return true;
        };
        v.acquire(page, false, copy, copy);
        v.template flush_stats<false>();
    }
};

template <typename T, bool DEFER = false> struct bam_ptr;

/*
 * What bam_ptr::operator[] hands out on a non-const pointer: converts to T for
 * a read and marks the page dirty only when assigned through.  (The reference
 * returns T& there and marks the page dirty on every window change, reads
 * included, include/page_cache.h:476-483, which turns every eviction of a
 * read-only workload into a write-back.)
 */
template <typename T>
struct bam_ref {
    bam_ptr<T, false>* p;
    size_t i;
    __forceinline__ __host__ __device__ operator T() const { return p->read(i); }
    __forceinline__ __host__ __device__ bam_ref& operator=(T v) { p->write(i, v); return *this; }
    __forceinline__ __host__ __device__ bam_ref& operator=(const bam_ref& o) { p->write(i, (T)o); return *this; }
    __forceinline__ __host__ __device__ bam_ref& operator+=(T v) { p->write(i, p->read(i) + v); return *this; }
    __forceinline__ __host__ __device__ bam_ref& operator-=(T v) { p->write(i, p->read(i) - v); return *this; }
};

/*
 * Per-thread window onto an array: keeps the page of the last access
 * referenced, so that a run of accesses to one page costs one acquire and one
 * release.  Same contract as the reference's bam_ptr (include/page_cache.h:414-485).
 * A thread holds one page referenced for as long as the window stays on it, so
 * the cache must have more pages than the threads of the resident waves can
 * hold at once (the reference has the same requirement).  The range
 * descriptor is read once and kept in registers for as long as the accesses
 * stay inside that range.
 *
 * DEFER (no counterpart in the reference): a pointer for the first of two launches.  It reads what is resident; when
 * the page of an access is not, the access yields T(), `missed` is set and nothing is loaded: the kernel notes the work
 * for the second launch, which uses a plain bam_ptr.  Reads only, and it holds no reference: the window is opened on a
 * look at the page's descriptor (valid, not busy: slot and load count noted), and what was read through it counts only
 * once still() has looked again and found the same, as for every read of a resident page that takes no reference
 * (bam_read_unpinned).  A reference is two read-modify-writes of the descriptor per page, and those are performed at
 * the memory, not in a cache: taking them out is worth a fifth of the rate of a wave that streams through pages.
 */
template <typename T, bool DEFER>
struct bam_ptr {
    data_page_t* page = nullptr;
    array_d_t<T>* array = nullptr;
    size_t start = 0;
    size_t end = 0;
    int64_t range_id = -1;
    T* addr = nullptr;
    bool dirty = false;
    bool missed = false;             /* DEFER: an access since the flag was last cleared found its page not resident (any more) */
    uint64_t seen = 0;               /* DEFER: the descriptor as it was when the window was opened */
    data_page_t* ahead = nullptr;    /* DEFER: the descriptor after the window's, looked at when the window was opened, */
    uint64_t ahead_sv = 0;           /* and what was seen there: a walk along an array finds its next look already made */
#if defined(__HIP_DEVICE_COMPILE__)
    bam::range_view<T> view;
#endif

    __forceinline__ __host__ __device__ bam_ptr(array_d_t<T>* a) { init(a); }
    __forceinline__ __host__ __device__ ~bam_ptr()
    {
        fini();
#if defined(__HIP_DEVICE_COMPILE__)
        view.flush_stats();
#endif
    }
    __forceinline__ __host__ __device__ void init(array_d_t<T>* a)
    {
        array = a;
#if defined(__HIP_DEVICE_COMPILE__)
        /* a deferring pointer is for arrays of one range: its descriptor is read here, once */
        if constexpr (DEFER) { range_id = 0; view.load(a->d_ranges); }
#endif
    }

    __forceinline__ __host__ __device__ void fini(void)
    {
#if defined(__HIP_DEVICE_COMPILE__)
        if constexpr (!DEFER) { if (page) view.release((uint64_t)(page - view.pages), dirty); }
        page = nullptr;
#endif
    }

    /* move the window to the page of element i (the reference's update_page, include/page_cache.h:447); NULL when there is no
     * such page to be had: no range holds i, the wait for the page was given up, or, DEFER, the page is not resident */
    __forceinline__ __host__ __device__ T* update_page(const size_t i)
    {
#if defined(__HIP_DEVICE_COMPILE__)
        if constexpr (DEFER) {
            if (!view.holds(i)) { page = nullptr; start = end = 0; addr = nullptr; return nullptr; }       /* past the array's one range */
            return move_window(i);
        }
#endif
        return update_page_general(i);
    }

    __forceinline__ __host__ __device__ T* update_page_general(const size_t i)
    {
#if defined(__HIP_DEVICE_COMPILE__)
        fini();
        start = end = 0;
        addr = nullptr;
        dirty = false;
        if (!view.holds(i)) {
            range_id = array->find_range(i);
            if (range_id == -1) { view.r = nullptr; return nullptr; }
            view.load(array->d_ranges + range_id);
        }
        const uint64_t pg = view.page_of(i);
        uint32_t slot = BAM_NO_SLOT;
        auto keep = [&](uint32_t s_) { slot = s_; return false; };
        view.template acquire<true>(pg, false, keep, keep);
        page = view.pages + pg;                 /* the references of the group stay counted either way */
        if (slot == BAM_NO_SLOT) return nullptr;        /* the wait was given up (the controller is marked aborted): no window */
        view.window(pg, start, end);
        addr = (T*)(view.slot_addr(slot) + (view.byte_of(start) & (view.page_size - 1)));
#endif
        return addr;
    }

#if defined(__HIP_DEVICE_COMPILE__)
    /*
     * DEFER: the window moves to the page of element i, which the range at hand holds: one look at the page's descriptor.
     * Where the lanes of the wave all go to the same page (a wave that walks pages together) the window and the address
     * of its first element are worked out once per wave, over the scalar unit, instead of once per lane.
     */
    __forceinline__ __device__ T* move_window(const size_t i)
    {
        using namespace bam;
        const uint64_t pg = view.page_of(i);
        const uint64_t upg = first(pg);
        const bool together = ballot(pg != upg) == 0;
        data_page_t* const dp = view.pages + (together ? upg : pg);
        uint64_t sv = ahead_sv;
        if (ahead != dp) sv = __hip_atomic_load((const uint64_t*)dp, __ATOMIC_RELAXED, BAM_AGENT);
        ahead = nullptr;
        if (((uint32_t)sv >> (CNT_SHIFT + 1)) == V_NB) {
            view.account(true);
            page = dp;
            seen = sv;
            if (together) {
                size_t s_, e_;
                view.window(upg, s_, e_);
                start = s_; end = e_;
                addr = (T*)(view.slot_addr((uint32_t)(sv >> 32) & BAM_SLOT_MASK) + (view.byte_of(s_) & (view.page_size - 1)));
            } else {
                view.window(pg, start, end);
                addr = (T*)(view.slot_addr((uint32_t)(sv >> 32) & BAM_SLOT_MASK) + (view.byte_of(start) & (view.page_size - 1)));
            }
            /* the look at the next page goes out now, beside this page's reads, and is not used before the next move: a
             * page then costs a walking wave its reads and the look that confirms them, not a third trip between them */
            if (end < view.index_end) {
                ahead = dp + 1;
                ahead_sv = __hip_atomic_load((const uint64_t*)(dp + 1), __ATOMIC_RELAXED, BAM_AGENT);
            }
            return addr;
        }
        page = nullptr;
        start = end = 0;
        addr = nullptr;
        missed = true;
        return nullptr;
    }
#endif

    /*
     * DEFER: whether what was read through the window since it was opened stands: the page is still valid, not busy, in
     * the same slot and loaded the same number of times (the reads have come back: callers ask after using them).  If
     * not, `missed` is set and the window is closed, as if the page had not been resident in the first place.
     */
    __forceinline__ __host__ __device__ bool still()
    {
#if defined(__HIP_DEVICE_COMPILE__)
        if (!page) return true;
        const uint64_t now = __hip_atomic_load((const uint64_t*)page, __ATOMIC_RELAXED, BAM_AGENT);
        if (((seen ^ now) & 0xFFFFFFFFC0000000ull) == 0) return true;
        page = nullptr;
        start = end = 0;
        addr = nullptr;
        missed = true;
        return false;
#else
        return true;
#endif
    }

    /* after a wait that was given up the value is T(): callers that use what they read as an index (the neighbour
     * ids of a graph) stay inside their arrays until the host sees the abort */
    __forceinline__ __host__ __device__ T read(const size_t i)
    {
#if defined(__HIP_DEVICE_COMPILE__)
        if constexpr (DEFER) {
            if (i < start || i >= end) { if (!update_page(i)) return T(); }
            return bam::ld_payload(addr + (i - start));
        }
#endif
        if (i < start || i >= end) { if (!update_page(i)) return T(); }
#if defined(__HIP_DEVICE_COMPILE__)
        return bam::ld_payload(addr + (i - start));
#else
        return addr[i - start];
#endif
    }

    /* the accesses this pointer has counted and not yet handed to the range's counters, read and put back: a kernel that
     * leaves a piece of work to a later launch takes back what it counted for it */
    __forceinline__ __host__ __device__ void counted(uint32_t& n_access, uint32_t& n_hit) const
    {
#if defined(__HIP_DEVICE_COMPILE__)
        n_access = view.n_access; n_hit = view.n_hit;
#else
        n_access = n_hit = 0;
#endif
    }
    __forceinline__ __host__ __device__ void set_counted(const uint32_t n_access, const uint32_t n_hit)
    {
#if defined(__HIP_DEVICE_COMPILE__)
        view.n_access = n_access; view.n_hit = n_hit;
#else
        (void)n_access; (void)n_hit;
#endif
    }

    /* whether elements a and b (a <= b), and so all between them, lie in the page this pointer holds now */
    __forceinline__ __host__ __device__ bool covers(const size_t a, const size_t b) const { return a >= start && b < end; }
    /* element i of the page held now, for callers that have asked covers() about it: no window test, so a lane's reads
     * of one page go out side by side instead of one behind the test of the one before */
    __forceinline__ __host__ __device__ T peek(const size_t i) const
    {
#if defined(__HIP_DEVICE_COMPILE__)
        return bam::ld_payload(addr + (i - start));
#else
        return addr[i - start];
#endif
    }

    /* N elements i, i + stride, ... of the page held now (the caller has asked covers() about the first and the last),
     * side by side; 8-byte elements are loaded as not to be kept (bam::ld_payload_nt) */
    template <int N>
    __forceinline__ __host__ __device__ void peek_n(const size_t i, const size_t stride, T (&out)[N]) const
    {
#if defined(__HIP_DEVICE_COMPILE__)
        if constexpr (sizeof(T) == 8 && N == 8) {
            if (stride == BAM_WAVE_SIZE) {              /* a wave's share of a page side by side: one address, eight offsets */
                uint64_t x[8];
                bam::ld_payload_stream8((const uint64_t*)(addr + (i - start)), x);
#pragma unroll
                for (int u = 0; u < N; u++) out[u] = *(T*)&x[u];
                return;
            }
        }
        if constexpr (sizeof(T) == 8 && (N == 1 || N == 2 || N == 4 || N == 7 || N == 8)) {
            const uint64_t* p[N];
            uint64_t x[N];
#pragma unroll
            for (int u = 0; u < N; u++) p[u] = (const uint64_t*)(addr + (i - start) + (size_t)u * stride);
            bam::ld_payload_nt(p, x);
#pragma unroll
            for (int u = 0; u < N; u++) out[u] = *(T*)&x[u];
        } else {
#pragma unroll
            for (int u = 0; u < N; u++) out[u] = bam::ld_payload(addr + (i - start) + (size_t)u * stride);
        }
#else
        for (int u = 0; u < N; u++) out[u] = addr[i - start + (size_t)u * stride];
#endif
    }

    __forceinline__ __host__ __device__ void mark_dirty()
    {
#if defined(__HIP_DEVICE_COMPILE__)
        if (!dirty) { __hip_atomic_fetch_or(&page->state, DIRTY, __ATOMIC_RELAXED, BAM_AGENT); dirty = true; }
#endif
    }

    __forceinline__ __host__ __device__ void write(const size_t i, const T v)
    {
        static_assert(!DEFER, "a deferring bam_ptr only reads");
        if (i < start || i >= end) { if (!update_page(i)) return; }
        mark_dirty();
        addr[i - start] = v;
    }

    __forceinline__ __host__ __device__ T operator[](const size_t i) const { return const_cast<bam_ptr*>(this)->read(i); }
    __forceinline__ __host__ __device__ auto operator[](const size_t i)
    {
        if constexpr (DEFER) return read(i);
        else return bam_ref<T>{this, i};
    }

    /* address of element i for the caller to read or write: counts as a write.  NULL when no range holds i or the wait
     * for the page was given up (the reference returns an address computed from a null window there) */
    __forceinline__ __host__ __device__ T* memref(size_t i)
    {
        static_assert(!DEFER, "a deferring bam_ptr only reads");
        if (i < start || i >= end) { if (!update_page(i)) return nullptr; }
        mark_dirty();
        return addr + (i - start);
    }
};

/* ------------------------------------------------------------------ */
/* translation table in front of the cache                            */
/* ------------------------------------------------------------------ */
/*
 * tlb / bam_ptr_tlb (include/page_cache.h:127-411 of the reference): a small direct-mapped table, shared by the
 * threads of a workgroup (in LDS) or of a launch (in device memory), that keeps one reference on each page it
 * names; threads that find their page in the table pay a count on the entry instead of an atomic on the page state.
 *
 * entry.state: bit 31 = entry locked, bits 29:0 = threads using the entry right now.
 *
 * The reference lets a thread wait on an entry that other threads are using for a different page.  In a wave the
 * users may be lanes of the waiting lane's own wave, which cannot move while it waits; such a lane takes its page
 * straight from the cache instead (`direct`), and so does a lane that finds the entry locked by a lane of its own
 * wave that is in the middle of I/O.
 */
#define THREAD_ 0
#define SHARED_ 1
#define GLOBAL_ 2
#define TLB_LOCK_  0x80000000u
#define TLB_COUNT_ 0x3fffffffu

struct tlb_entry {
    uint64_t global_id;
    uint32_t state;
    uint32_t slot;
    data_page_t* page;

    __forceinline__ __host__ __device__ void init() { global_id = 0; state = 0; slot = 0; page = nullptr; }
    /* drop the reference the entry itself holds on its page */
    __forceinline__ __device__ void release()
    {
        if (page) { bam_release_refs(page, 1, false); page = nullptr; }
    }
    __forceinline__ __device__ void release(const uint32_t count) { __hip_atomic_fetch_add(&state, 0u - count, __ATOMIC_RELEASE, BAM_AGENT); }
};

template <typename T, size_t n = 32, simt::thread_scope _scope = simt::thread_scope_device, size_t loc = GLOBAL_>
struct tlb {
    tlb_entry entries[n ? n : 1];
    array_d_t<T>* array;

    /* by all threads of the workgroup (or by one thread with the others waiting), before first use */
    __forceinline__ __device__ void init(array_d_t<T>* a)
    {
        const size_t tid = threadIdx.x + blockDim.x * (threadIdx.y + blockDim.y * threadIdx.z);
        const size_t bs = (size_t)blockDim.x * blockDim.y * blockDim.z;
        if (tid == 0) array = a;
        for (size_t k = tid; k < n; k += bs) entries[k].init();
    }
    /* after the last use: the references the entries hold go back */
    __forceinline__ __device__ void fini()
    {
        const size_t tid = threadIdx.x + blockDim.x * (threadIdx.y + blockDim.y * threadIdx.z);
        const size_t bs = (size_t)blockDim.x * blockDim.y * blockDim.z;
        for (size_t k = tid; k < n; k += bs) entries[k].release();
    }

    /*
     * Address of the first element of the page `page_` of `range` (global id `gid`), the window it covers in
     * [start, end), and in `direct` whether the table was bypassed; pair with release(gid, direct, range, page_).
     */
    __forceinline__ __device__ T* acquire(const size_t i, const size_t gid, size_t& start, size_t& end, range_d_t<T>* range, const size_t page_, bool& direct)
    {
        using namespace bam;
        (void)i;
        tlb_entry* entry = entries + (n ? gid % n : 0);
        const uint64_t eq_mask = match_any((uint64_t)gid, (uint64_t)this);
        const uint32_t master = first_lane(eq_mask), count = popc(eq_mask);
        uint64_t pack = 0;                       /* slot | direct << 32 */
        if (lane() == master) {
            bool settled = false, go_direct = n == 0;
            uint32_t slot = 0;
            /* the masters of a wave come round this loop together; whoever holds an entry's lock finishes
             * within the trip, so nobody spins on a lock held by a lane that cannot run */
            for (uint32_t tries = 0; !settled && !go_direct; tries++) {
                const uint32_t st = __hip_atomic_fetch_or(&entry->state, TLB_LOCK_, __ATOMIC_ACQUIRE, BAM_AGENT);
                if ((st & TLB_LOCK_) == 0) {
                    /* the lock goes, and the users come, with one add: users that leave meanwhile (tlb_entry::release,
                     * an add of its own) are not written over */
                    if (entry->page != nullptr && entry->global_id == gid) {
                        slot = entry->slot;
                        __hip_atomic_fetch_add(&entry->state, count - TLB_LOCK_, __ATOMIC_RELEASE, BAM_AGENT);
                        settled = true;
                    } else if (entry->page == nullptr || (st & TLB_COUNT_) == 0) {
                        entry->release();
                        slot = (uint32_t)range->acquire_page(page_, 1, false, 0, wave_slot_hash());
                        if (slot == BAM_NO_SLOT) {
                            /* the wait for the page was given up: the entry stays empty */
                            range->release_page(page_, 1, false);
                            __hip_atomic_fetch_add(&entry->state, 0u - TLB_LOCK_, __ATOMIC_RELEASE, BAM_AGENT);
                            go_direct = true;
                        } else {
                            entry->page = &range->pages[page_];
                            entry->slot = slot;
                            entry->global_id = gid;
                            __hip_atomic_fetch_add(&entry->state, count - TLB_LOCK_, __ATOMIC_RELEASE, BAM_AGENT);
                            settled = true;
                        }
                    } else {
                        __hip_atomic_fetch_add(&entry->state, 0u - TLB_LOCK_, __ATOMIC_RELEASE, BAM_AGENT);     /* in use for another page */
                        go_direct = true;
                    }
                } else if (tries >= 8) go_direct = true;
            }
            if (go_direct) slot = (uint32_t)range->acquire_page(page_, count, false, 0, wave_slot_hash());
            pack = (uint64_t)slot | ((uint64_t)go_direct << 32);
        }
        pack = shfl(pack, master);
        direct = (pack >> 32) != 0;
        range_view<T> v;
        v.load(range);
        v.window(page_, start, end);
        if ((uint32_t)pack == BAM_NO_SLOT) { start = end = 0; return nullptr; }      /* wait given up (direct, references counted): release as usual */
        return (T*)(v.slot_addr((uint32_t)pack) + (v.byte_of(start) & (v.page_size - 1)));
    }

    __forceinline__ __device__ void release(const size_t gid, const bool direct, range_d_t<T>* range, const size_t page_)
    {
        using namespace bam;
        const uint64_t eq_mask = match_any((uint64_t)gid, (uint64_t)this ^ (direct ? 1ull : 0ull));
        if (lane() != first_lane(eq_mask)) return;
        if (direct) range->release_page(page_, popc(eq_mask), false);
        else entries[n ? gid % n : 0].release(popc(eq_mask));
    }
};

template <typename T, size_t n = 32, simt::thread_scope _scope = simt::thread_scope_device, size_t loc = GLOBAL_>
struct bam_ptr_tlb {
    tlb<T, n, _scope, loc>* tlb_ = nullptr;
    array_d_t<T>* array = nullptr;
    range_d_t<T>* range = nullptr;
    size_t page = 0;
    size_t start = 0;
    size_t end = 0;
    size_t gid = 0;
    T* addr = nullptr;
    bool direct = false;

    __forceinline__ __device__ bam_ptr_tlb(array_d_t<T>* a, tlb<T, n, _scope, loc>* t) { init(a, t); }
    __forceinline__ __device__ ~bam_ptr_tlb() { fini(); }
    __forceinline__ __device__ void init(array_d_t<T>* a, tlb<T, n, _scope, loc>* t) { array = a; tlb_ = t; }

    bool held = false;               /* a reference (on the table's entry or on the page) is out */

    __forceinline__ __device__ void fini(void)
    {
        if (held) {
            tlb_->release(gid, direct, range, page);
            held = false;
            addr = nullptr;
            start = end = 0;
        }
    }

    __forceinline__ __device__ void update_page(const size_t i)
    {
        fini();
        array->get_page_gid(i, range, page, gid);
        if (range) { addr = tlb_->acquire(i, gid, start, end, range, page, direct); held = true; }
    }

    /* T() when no range holds i or the wait for the page was given up */
    __forceinline__ __device__ T operator[](const size_t i) const
    {
        bam_ptr_tlb* self = const_cast<bam_ptr_tlb*>(this);
        if (i < start || i >= end) self->update_page(i);
        if (!self->addr || i < self->start || i >= self->end) return T();
        return bam::ld_payload(self->addr + (i - start));
    }

    /* address of element i for the caller to write through: the page is marked dirty; NULL when no range holds i or
     * the wait for the page was given up */
    __forceinline__ __device__ T* memref(const size_t i)
    {
        if (i < start || i >= end) update_page(i);
        if (!addr || i < start || i >= end) return nullptr;
        range->mark_page_dirty(page);
        return addr + (i - start);
    }
};

/* ------------------------------------------------------------------ */
/* host side                                                          */
/* ------------------------------------------------------------------ */

/* one thread per cache slot: write dirty pages back (page_cache_t::flush_cache) */
static __global__ void __flush(page_cache_d_t* pc)
{
    const uint64_t page = threadIdx.x + (uint64_t)blockIdx.x * blockDim.x;
    if (page >= pc->n_pages) return;
    const uint64_t w = bam::ld_relaxed(&pc->cache_pages[page].page_translation);
    if ((w >> BAM_TAKE_SHIFT) & FREE) return;
    const uint64_t g = w & BAM_TRANSLATION_MASK;
    const uint64_t range = g & pc->n_ranges_mask, addr = g >> pc->n_ranges_bits;
    data_page_t* dp = &pc->ranges[range][addr];
    const uint32_t s = bam::ld_relaxed(&dp->state);
    if ((s & DIRTY) == 0 || (s & VALID) == 0 || (bam::ld_relaxed(&dp->offset) & BAM_SLOT_MASK) != page) return;
    const data_dist_t dist = pc->ranges_dists[range];
    const uint64_t index = get_backing_page_(pc->ranges_page_starts[range], addr, pc->n_ctrls, dist);
    uint64_t c = get_backing_ctrl_(addr, pc->n_ctrls, dist);
    const uint64_t c_end = c == ALL_CTRLS ? pc->n_ctrls : c + 1;
    const uint32_t smid = get_smid();
    for (c = c == ALL_CTRLS ? 0 : c; c < c_end; c++) {
        Controller* ctl = pc->d_ctrls[c];
        write_data(pc, ctl->d_qps + (smid % ctl->n_qps), index * pc->n_blocks_per_page, pc->n_blocks_per_page, page);
    }
    __hip_atomic_fetch_and(&dp->state, ~DIRTY, __ATOMIC_RELEASE, BAM_AGENT);
}

struct page_cache_t {
    page_cache_d_t pdt;
    pages_t* h_ranges;
    uint64_t* h_ranges_page_starts;
    data_dist_t* h_ranges_dists;
    page_cache_d_t* d_pc_ptr;

    DmaPtr pages_dma;
    DmaPtr prp_list_dma;
    BufferPtr pages_buf;
    BufferPtr prp1_buf, prp2_buf;
    BufferPtr cache_pages_buf;
    BufferPtr ranges_buf;
    BufferPtr pc_buff;
    BufferPtr d_ctrls_buff;
    BufferPtr ranges_page_starts_buf;
    BufferPtr ranges_dists_buf;
    BufferPtr page_ticket_buf;
    BufferPtr direct_gauge_buf;
    BufferPtr ctrl_counter_buf;
    BufferPtr extra_reads_buf;
    BufferPtr tokens_buf;

    uint64_t reset_stats()
    {
        uint64_t v = 0;
        hip_err_chk(hipMemcpy(&v, pdt.extra_reads, sizeof(uint64_t), hipMemcpyDeviceToHost));
        hip_err_chk(hipMemset(pdt.extra_reads, 0, sizeof(uint64_t)));
        return v;
    }
    void print_reset_stats(void) { (void)reset_stats(); }

    void flush_cache()
    {
        const size_t threads = 64;
        const size_t n_blocks = (pdt.n_pages + threads - 1) / threads;
        hipLaunchKernelGGL(__flush, dim3((uint32_t)n_blocks), dim3((uint32_t)threads), 0, 0, d_pc_ptr);
        hip_err_chk(hipGetLastError());
    }

    template <typename T>
    void add_range(range_t<T>* range)
    {
        if (pdt.n_ranges >= pdt.range_cap) throw error(string("page_cache_t: too many ranges"));
        range->rdt.range_id = pdt.n_ranges++;
        h_ranges[range->rdt.range_id] = range->rdt.pages;
        h_ranges_page_starts[range->rdt.range_id] = range->rdt.page_start;
        h_ranges_dists[range->rdt.range_id] = range->rdt.dist;
        hip_err_chk(hipMemcpy(pdt.ranges_page_starts, h_ranges_page_starts, pdt.n_ranges * sizeof(uint64_t), hipMemcpyHostToDevice));
        hip_err_chk(hipMemcpy(pdt.ranges, h_ranges, pdt.n_ranges * sizeof(pages_t), hipMemcpyHostToDevice));
        hip_err_chk(hipMemcpy(pdt.ranges_dists, h_ranges_dists, pdt.n_ranges * sizeof(data_dist_t), hipMemcpyHostToDevice));
        hip_err_chk(hipMemcpy(d_pc_ptr, &pdt, sizeof(page_cache_d_t), hipMemcpyHostToDevice));
    }

    page_cache_t(const uint64_t ps, const uint64_t np, const uint32_t hipDevice, const Controller& ctrl, const uint64_t max_range, const std::vector<Controller*>& ctrls)
    {
        if (np == 0 || ps < ctrl.ns.lba_data_size || (ps & (ps - 1)) || max_range == 0 || (max_range & (max_range - 1)) || ctrls.empty())
            throw error(string("page_cache_t: Can't have such page size or number of pages"));
        memset(&pdt, 0, sizeof(pdt));
        hip_err_chk(hipSetDevice(hipDevice));
        ctrl_counter_buf = createBuffer(sizeof(uint64_t), hipDevice);
        extra_reads_buf = createBuffer(sizeof(uint64_t), hipDevice);
        pdt.ctrl_counter = (simt::atomic<uint64_t, simt::thread_scope_device>*)ctrl_counter_buf.get();
        pdt.extra_reads = (simt::atomic<uint64_t, simt::thread_scope_device>*)extra_reads_buf.get();
        pdt.page_size = ps;
        pdt.page_size_minus_1 = ps - 1;
        pdt.page_size_log = (uint64_t)__builtin_ctzll(ps);
        pdt.n_pages = np;
        pdt.n_pages_minus_1 = np - 1;
        pdt.ctrl_page_size = ctrl.ctrl->page_size;
        pdt.n_ctrls = ctrls.size();
        d_ctrls_buff = createBuffer(pdt.n_ctrls * sizeof(Controller*), hipDevice);
        pdt.d_ctrls = (Controller**)d_ctrls_buff.get();
        pdt.n_blocks_per_page = ps / ctrl.blk_size;
        for (size_t k = 0; k < pdt.n_ctrls; k++)
            hip_err_chk(hipMemcpy(pdt.d_ctrls + k, &ctrls[k]->d_ctrl_ptr, sizeof(Controller*), hipMemcpyHostToDevice));
        pdt.guard = ctrl.guard;
        pdt.spin_limit = ctrl.guard ? ctrl.guard->spin_limit : 0;

        pdt.range_cap = max_range;
        pdt.n_ranges = 0;
        pdt.n_ranges_bits = max_range == 1 ? 1 : (uint64_t)__builtin_ctzll(max_range);
        pdt.n_ranges_mask = max_range - 1;
        ranges_buf = createBuffer(max_range * sizeof(pages_t), hipDevice);
        pdt.ranges = (pages_t*)ranges_buf.get();
        h_ranges = new pages_t[max_range]();
        h_ranges_page_starts = new uint64_t[max_range]();
        h_ranges_dists = new data_dist_t[max_range]();
        ranges_page_starts_buf = createBuffer(max_range * sizeof(uint64_t), hipDevice);
        pdt.ranges_page_starts = (uint64_t*)ranges_page_starts_buf.get();
        ranges_dists_buf = createBuffer(max_range * sizeof(data_dist_t), hipDevice);
        pdt.ranges_dists = (data_dist_t*)ranges_dists_buf.get();

        cache_pages_buf = createBuffer(np * sizeof(cache_page_t), hipDevice);
        pdt.cache_pages = (cache_page_t*)cache_pages_buf.get();
        {
            std::vector<cache_page_t> tps(np);
            for (size_t i = 0; i < np; i++) tps[i].page_translation = (uint64_t)FREE << BAM_TAKE_SHIFT;
            hip_err_chk(hipMemcpy(pdt.cache_pages, tps.data(), np * sizeof(cache_page_t), hipMemcpyHostToDevice));
        }
        page_ticket_buf = createBuffer(sizeof(uint32_t), hipDevice);
        pdt.page_ticket = (uint32_t*)page_ticket_buf.get();

        if (np > BAM_SLOT_MASK) throw error(string("page_cache_t: more cache pages than a page descriptor can name"));
        pdt.wave_batch = BAM_WAVE_SIZE;
        pdt.fast_reads = 1;
        if (const char* e = getenv("BAM_FAST_READS")) pdt.fast_reads = atoi(e) != 0;
        tokens_buf = createBuffer(BAM_TOKEN_SLOTS * 64, hipDevice);
        pdt.miss_tokens = (uint32_t*)tokens_buf.get();
        pdt.miss_waves = 0;
        if (const char* e = getenv("BAM_MISS_WAVES")) pdt.miss_waves = (uint32_t)atoi(e);
        pdt.prof = ctrl.prof;

        const bool staged = ctrl.n_qps && ctrl.h_qps[0]->stage != nullptr;
        const uint64_t cache_size = ps * np;
        pdt.direct_share = 3;        /* measured best on the random-gather workload: 12.1M 4 KiB reads/s against 11.4M all staged, 10.4M all direct */
        if (const char* e = getenv("BAM_DIRECT_SHARE")) pdt.direct_share = (uint32_t)atoi(e);
        /* 1024 measured: the random gather 13.2 M reads of 4 KiB per second (13.4 M at 64, 13.3 M all staged, 12.8 M at 8192,
         * 11.9 M at 32768), connected components of 2^26 vertices 0.50 s (0.59 at 8192), the per-vertex traversal of a
         * 2^24-vertex graph 4.5 thousand million edges per second (4.35 at 512 and at 8192) */
        pdt.direct_limit = 1024;
        /* waves that only fetch have nobody to copy staged pages for them: 8192, the cold streaming modes read every page
         * once at 12.6 M pages per second (with 1024: a fifth of the pages twice) */
        pdt.direct_limit_ahead = 8192;
        if (const char* e = getenv("BAM_DIRECT_LIMIT_AHEAD")) pdt.direct_limit_ahead = (uint32_t)atoi(e);
        if (const char* e = getenv("BAM_DIRECT_LIMIT")) pdt.direct_limit = (uint32_t)atoi(e);
        direct_gauge_buf = createBuffer(64, hipDevice);
        pdt.direct_gauge = (uint32_t*)direct_gauge_buf.get();
        hip_err_chk(hipMemset(pdt.direct_gauge, 0, 64));
        pdt.direct_share_raw = 0;    /* raw 4 KiB block reads: 12.8 M/s all staged, 11.7 M with three of eight direct, 10.4 M all direct */
        if (const char* e = getenv("BAM_DIRECT_SHARE_RAW")) pdt.direct_share_raw = (uint32_t)atoi(e);
        if (!staged) pdt.direct_share = pdt.direct_share_raw = 0;
        if (staged && ps > ctrl.h_qps[0]->stage_stride) pdt.direct_share = pdt.direct_share_raw = 8;      /* pages that do not fit a staging page: all direct */
        if (staged && pdt.direct_share == 0) {
            /* the controller never addresses the cache: plain device memory, no PRP tables */
            pages_buf = createBuffer(cache_size, hipDevice);
            pdt.base_addr = (uint8_t*)pages_buf.get();
            pdt.prps = false;
        } else {
            pages_dma = createDma(ctrl.ctrl, NVM_PAGE_ALIGN(cache_size, 1UL << 16), hipDevice, BAM_DMA_DEVICE);
            pdt.base_addr = (uint8_t*)pages_dma->vaddr;
            const uint64_t cps = ctrl.ctrl->page_size;
            std::vector<uint64_t> t1(np), t2(np);
            prp1_buf = createBuffer(np * sizeof(uint64_t), hipDevice);
            pdt.prp1 = (uint64_t*)prp1_buf.get();
            if (ps <= cps) {
                /* several cache pages share one controller page */
                for (size_t i = 0; i < np; i++) t1[i] = pages_dma->ioaddrs[i * ps / cps] + (i * ps) % cps;
                pdt.prps = false;
            } else {
                prp2_buf = createBuffer(np * sizeof(uint64_t), hipDevice);
                pdt.prp2 = (uint64_t*)prp2_buf.get();
                const uint64_t per = ps / cps;
                if (per == 2) {
                    for (size_t i = 0; i < np; i++) { t1[i] = pages_dma->ioaddrs[i * 2]; t2[i] = pages_dma->ioaddrs[i * 2 + 1]; }
                } else {
                    /* one PRP-list page per slot */
                    if (per - 1 > cps / sizeof(uint64_t)) throw error(string("page_cache_t: page size needs chained PRP lists"));
                    prp_list_dma = createDma(ctrl.ctrl, NVM_PAGE_ALIGN(cps * np, 1UL << 16));
                    uint64_t* lists = (uint64_t*)prp_list_dma->vaddr;
                    for (size_t i = 0; i < np; i++) {
                        t1[i] = pages_dma->ioaddrs[i * per];
                        t2[i] = prp_list_dma->ioaddrs[i];
                        for (size_t j = 0; j + 1 < per; j++) lists[i * (cps / sizeof(uint64_t)) + j] = pages_dma->ioaddrs[i * per + j + 1];
                    }
                }
                hip_err_chk(hipMemcpy(pdt.prp2, t2.data(), np * sizeof(uint64_t), hipMemcpyHostToDevice));
                pdt.prps = true;
            }
            hip_err_chk(hipMemcpy(pdt.prp1, t1.data(), np * sizeof(uint64_t), hipMemcpyHostToDevice));
        }

        pc_buff = createBuffer(sizeof(page_cache_d_t), hipDevice);
        d_pc_ptr = (page_cache_d_t*)pc_buff.get();
        hip_err_chk(hipMemcpy(d_pc_ptr, &pdt, sizeof(page_cache_d_t), hipMemcpyHostToDevice));
    }

    page_cache_t(const page_cache_t&) = delete;
    page_cache_t& operator=(const page_cache_t&) = delete;

    ~page_cache_t()
    {
        delete[] h_ranges;
        delete[] h_ranges_page_starts;
        delete[] h_ranges_dists;
    }
};

template <typename T>
struct range_t {
    range_d_t<T> rdt;
    range_d_t<T>* d_range_ptr;
    page_cache_d_t* cache;
    BufferPtr pages_buff;
    BufferPtr stats_buff;
    BufferPtr range_buff;

    /* is: first element index, count: one past the last element index, ps: first backing page, pc: number of pages,
     * pso: byte offset of element `is` inside the first page, p_size: page size, c_h: the cache, dist: placement over controllers */
    range_t(uint64_t is, uint64_t count, uint64_t ps, uint64_t pc, uint64_t pso, uint64_t p_size, page_cache_t* c_h, uint32_t hipDevice, data_dist_t dist = REPLICATE)
    {
        (void)p_size;
        memset(&rdt, 0, sizeof(rdt));
        rdt.index_start = is;
        rdt.count = count;
        rdt.page_start = ps;
        rdt.page_count = pc;
        rdt.page_size = c_h->pdt.page_size;
        rdt.page_start_offset = pso;
        rdt.dist = dist;
        rdt.n_elems_per_page = rdt.page_size / sizeof(T);
        cache = (page_cache_d_t*)c_h->d_pc_ptr;
        pages_buff = createBuffer(pc * sizeof(data_page_t), hipDevice);      /* zero = INVALID, no references */
        rdt.pages = (pages_t)pages_buff.get();
        stats_buff = createBuffer(BAM_STAT_SHARDS * sizeof(bam_stat_shard_t), hipDevice);
        rdt.stats = (bam_stat_shard_t*)stats_buff.get();
        range_buff = createBuffer(sizeof(range_d_t<T>), hipDevice);
        d_range_ptr = (range_d_t<T>*)range_buff.get();
        c_h->add_range(this);
        rdt.cache = c_h->pdt;
        hip_err_chk(hipMemcpy((void*)d_range_ptr, (const void*)&rdt, sizeof(range_d_t<T>), hipMemcpyHostToDevice));
    }
    range_t(const range_t&) = delete;
    range_t& operator=(const range_t&) = delete;
};

struct bam_array_counters { unsigned long long read_io_cnt, access_cnt, miss_cnt, hit_cnt; };

template <typename T>
struct array_t {
    array_d_t<T> adt;
    array_d_t<T>* d_array_ptr;
    BufferPtr d_array_buff;
    BufferPtr d_d_ranges_buff;
    std::vector<range_d_t<T>> h_ranges;

    /* sum the shards of every range, zero them, return the totals of all ranges */
    bam_array_counters reset_stats(std::vector<bam_array_counters>* per_range = nullptr)
    {
        bam_array_counters tot = {0, 0, 0, 0};
        std::vector<bam_stat_shard_t> sh(BAM_STAT_SHARDS);
        for (size_t i = 0; i < adt.n_ranges; i++) {
            hip_err_chk(hipMemcpy(sh.data(), h_ranges[i].stats, sh.size() * sizeof(bam_stat_shard_t), hipMemcpyDeviceToHost));
            hip_err_chk(hipMemset(h_ranges[i].stats, 0, sh.size() * sizeof(bam_stat_shard_t)));
            bam_array_counters r = {0, 0, 0, 0};
            for (auto& s : sh) { r.read_io_cnt += s.read_io_cnt; r.access_cnt += s.access_cnt; r.hit_cnt += s.hit_cnt; }
            r.miss_cnt = r.access_cnt - r.hit_cnt;      /* every access is a hit or a miss; only hits are counted on the device */
            if (per_range) per_range->push_back(r);
            tot.read_io_cnt += r.read_io_cnt; tot.access_cnt += r.access_cnt; tot.miss_cnt += r.miss_cnt; tot.hit_cnt += r.hit_cnt;
        }
        return tot;
    }

    void print_reset_stats(void)
    {
        std::vector<bam_array_counters> rs;
        reset_stats(&rs);
        for (size_t i = 0; i < rs.size(); i++) {
            std::cout << std::dec << "#READ IOs: " << rs[i].read_io_cnt
                      << "\t#Accesses:" << rs[i].access_cnt
                      << "\t#Misses:" << rs[i].miss_cnt
                      << "\tMiss Rate:" << ((float)rs[i].miss_cnt / rs[i].access_cnt)
                      << "\t#Hits: " << rs[i].hit_cnt
                      << "\tHit Rate:" << ((float)rs[i].hit_cnt / rs[i].access_cnt)
                      << "\tCLSize:" << h_ranges[i].page_size << std::endl;
            std::cout << "*********************************" << std::endl;
        }
    }

    array_t(const uint64_t num_elems, const uint64_t disk_start_offset, const std::vector<range_t<T>*>& ranges, uint32_t hipDevice)
    {
        memset(&adt, 0, sizeof(adt));
        adt.n_elems = num_elems;
        adt.start_offset = disk_start_offset;
        adt.n_ranges = ranges.size();
        d_array_buff = createBuffer(sizeof(array_d_t<T>), hipDevice);
        d_array_ptr = (array_d_t<T>*)d_array_buff.get();
        d_d_ranges_buff = createBuffer(adt.n_ranges * sizeof(range_d_t<T>), hipDevice);
        adt.d_ranges = (range_d_t<T>*)d_d_ranges_buff.get();
        for (size_t k = 0; k < adt.n_ranges; k++) {
            h_ranges.push_back(ranges[k]->rdt);
            hip_err_chk(hipMemcpy((void*)(adt.d_ranges + k), (const void*)ranges[k]->d_range_ptr, sizeof(range_d_t<T>), hipMemcpyDeviceToDevice));
        }
        hip_err_chk(hipMemcpy((void*)d_array_ptr, (const void*)&adt, sizeof(array_d_t<T>), hipMemcpyHostToDevice));
    }
    array_t(const array_t&) = delete;
    array_t& operator=(const array_t&) = delete;
};

#endif /* __PAGE_CACHE_H__ */
