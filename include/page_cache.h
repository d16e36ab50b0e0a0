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

#define BAM_STAT_SHARDS 64

struct page_cache_t;
struct page_cache_d_t;
template <typename T> struct range_t;
template <typename T> struct array_d_t;
template <typename T> struct range_d_t;

/* one per backing page */
typedef struct { uint32_t state; uint32_t offset; } data_page_t;
typedef data_page_t* pages_t;

/* one per cache slot */
typedef struct { uint32_t page_take_lock; uint32_t pad; uint64_t page_translation; } cache_page_t;

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
    uint64_t* prp1;                  /* [n_pages] bus address of each slot (direct transfers only) */
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
    uint32_t wave_batch;             /* distinct pages one wave may hold referenced while it loads (1..64) */
    bam_guard_t* guard;
    uint32_t spin_limit;

    __forceinline__ __device__ cache_page_t* get_cache_page(const uint32_t page) const { return &cache_pages[page]; }
    __forceinline__ __device__ uint32_t find_slot(uint64_t address, uint64_t range_id, const uint32_t queue_);
    __forceinline__ __device__ bool spin_giveup(bam::spin_t& s) const
    {
        bam::backoff(s.slp);
        s.n++;
        if (!guard) return false;
        if ((s.n & 127u) == 0 && bam::ld_relaxed_sys(&guard->abort)) return true;
        if (spin_limit && s.n > spin_limit) { bam::st_relaxed_sys(&guard->abort, 1u); return true; }
        return false;
    }
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
 * One command per active lane on queue pair `qp` (wave-uniform): allocate ids,
 * build and submit the entries as one batch, wait for all completions, move
 * staged payload, recycle ids.  `pc_entry` is the cache slot the data belongs to.
 */
__device__ __forceinline__ void io_group(page_cache_d_t* pc, QueuePair* qp, uint64_t lba, uint32_t n_blocks, uint64_t pc_entry, uint8_t opcode)
{
    const uint32_t bytes = n_blocks << qp->block_size_log;
    uint8_t* slot_addr = pc->base_addr + pc_entry * pc->page_size;
    bool pending = true;
    spin_t sp;
    for (;;) {
        /* lanes that get a command id run their command to completion; the others try again afterwards */
        uint32_t cid = 0;
        const bool ready = pending && try_get_cid_group(&qp->sq, cid);
        if (ready) {
            const uint64_t act = active_mask();
            const uint32_t n = popc(act), rank = rank_in(act);
            uint64_t prp1, prp2 = 0;
            uint8_t* stage = nullptr;
            if (qp->stage) {
                stage = qp->stage + (size_t)cid * qp->stage_stride;
                prp1 = qp->stage_ioaddr + (uint64_t)cid * qp->stage_stride;
                if (opcode == NVM_IO_WRITE) {
                    /* payload to staging, one lane's page at a time, 16 bytes per lane per trip */
                    for (uint64_t m = act; m; m &= m - 1) {
                        const uint32_t j = first_lane(m);
                        uint4* d = (uint4*)bcast((uint64_t)stage, j);
                        const uint4* s = (const uint4*)bcast((uint64_t)slot_addr, j);
                        const uint32_t nb = bcast(bytes, j) / 16;
                        for (uint32_t i = rank; i < nb; i += n) d[i] = s[i];
                    }
                    fence_release_sys();
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
            sq_enqueue_group(&qp->sq, &cmd);
            cq_wait_group(&qp->cq, &qp->sq, cid);
            if (stage && opcode == NVM_IO_READ) {
                for (uint64_t m = act; m; m &= m - 1) {
                    const uint32_t j = first_lane(m);
                    const uint4* s = (const uint4*)bcast((uint64_t)stage, j);
                    uint4* d = (uint4*)bcast((uint64_t)slot_addr, j);
                    const uint32_t nb = bcast(bytes, j) / 16;
                    for (uint32_t i = rank; i < nb; i += n) d[i] = s[i];
                }
            }
            st_release(&qp->sq.cid[cid].val, (uint32_t)UNLOCKED);
            pending = false;
        }
        if (!ballot(pending)) break;
        if (!ballot(ready) && spin_giveup(&qp->sq, sp)) break;
    }
}

} // namespace bam

inline __device__ void access_data(page_cache_d_t* pc, QueuePair* qp, const uint64_t starting_lba, const uint64_t n_blocks, const unsigned long long pc_entry, const uint8_t opcode)
{
    for (bool done = false; !done;) {
        QueuePair* cur = (QueuePair*)bam::first((uint64_t)qp);
        page_cache_d_t* cpc = (page_cache_d_t*)bam::first((uint64_t)pc);
        if (cur == qp && cpc == pc) { bam::io_group(cpc, cur, starting_lba, (uint32_t)n_blocks, pc_entry, opcode); done = true; }
    }
}

inline __device__ void read_data(page_cache_d_t* pc, QueuePair* qp, const uint64_t starting_lba, const uint64_t n_blocks, const unsigned long long pc_entry)
{
    access_data(pc, qp, starting_lba, n_blocks, pc_entry, NVM_IO_READ);
}

inline __device__ void write_data(page_cache_d_t* pc, QueuePair* qp, const uint64_t starting_lba, const uint64_t n_blocks, const unsigned long long pc_entry)
{
    access_data(pc, qp, starting_lba, n_blocks, pc_entry, NVM_IO_WRITE);
}

/* ------------------------------------------------------------------ */
/* eviction                                                           */
/* ------------------------------------------------------------------ */

/*
 * Find a cache slot for page `address` of range `range_id`: a global
 * round-robin hand (page_ticket); a slot is taken if it is free, or if its
 * current page has no references and is not busy, in which case that page is
 * invalidated (and written back first when dirty).  Called by all lanes of a
 * wave that need a slot; they advance side by side and take one ticket grab
 * per trip for the whole group.
 */
__forceinline__ __device__
uint32_t page_cache_d_t::find_slot(uint64_t address, uint64_t range_id, const uint32_t queue_)
{
    using namespace bam;
    const uint64_t global_address = (address << n_ranges_bits) | range_id;
    uint32_t page = 0;
    bool found = false;
    spin_t sp;
    for (;;) {
        const uint64_t need = ballot(!found);
        if (!need) break;
        if (!found) {
            const uint32_t ld = first_lane(need);
            uint32_t base = 0;
            if (lane() == ld) base = __hip_atomic_fetch_add(page_ticket, popc(need), __ATOMIC_RELAXED, BAM_AGENT);
            base = bcast(base, ld);
            const uint32_t p = (uint32_t)((base + rank_in(need)) % n_pages);
            cache_page_t* cp = &cache_pages[p];
            uint32_t v = ld_relaxed(&cp->page_take_lock);
            if (v == FREE) {
                if (__hip_atomic_compare_exchange_strong(&cp->page_take_lock, &v, (uint32_t)LOCKED, __ATOMIC_ACQUIRE, __ATOMIC_RELAXED, BAM_AGENT)) {
                    cp->page_translation = global_address;
                    st_release(&cp->page_take_lock, (uint32_t)UNLOCKED);
                    page = p; found = true;
                }
            } else if (v == UNLOCKED) {
                if (__hip_atomic_compare_exchange_strong(&cp->page_take_lock, &v, (uint32_t)LOCKED, __ATOMIC_ACQUIRE, __ATOMIC_RELAXED, BAM_AGENT)) {
                    const uint64_t prev = cp->page_translation;
                    const uint64_t prev_range = prev & n_ranges_mask, prev_page = prev >> n_ranges_bits;
                    data_page_t* victim = &ranges[prev_range][prev_page];
                    const uint32_t e = ld_relaxed(&victim->state);
                    if ((e & CNT_MASK) == 0 && (e & BUSY) == 0) {
                        const uint32_t o = __hip_atomic_fetch_or(&victim->state, BUSY, __ATOMIC_ACQUIRE, BAM_AGENT);
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
                                }
                                /* -> INVALID; references taken meanwhile stay counted and their owners reload */
                                __hip_atomic_fetch_and(&victim->state, CNT_MASK, __ATOMIC_RELEASE, BAM_AGENT);
                                cp->page_translation = global_address;
                                page = p; found = true;
                            } else {
                                __hip_atomic_fetch_and(&victim->state, DISABLE_BUSY_MASK, __ATOMIC_RELEASE, BAM_AGENT);
                            }
                        }
                    }
                    st_release(&cp->page_take_lock, (uint32_t)UNLOCKED);
                }
            }
        }
        if (ballot(!found) && (++sp.n & 1023u) == 0 && spin_giveup(sp)) break;
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
    __forceinline__ __device__ void release_page(const size_t pg) const { __hip_atomic_fetch_add(&pages[pg].state, (uint32_t)-1, __ATOMIC_RELEASE, BAM_AGENT); }
    __forceinline__ __device__ void release_page(const size_t pg, const uint32_t count) const { __hip_atomic_fetch_add(&pages[pg].state, 0u - count, __ATOMIC_RELEASE, BAM_AGENT); }
    __forceinline__ __device__ cache_page_t* get_cache_page(const size_t pg) const { return cache.get_cache_page(pages[pg].offset); }
    __forceinline__ __device__ uint64_t get_cache_page_addr(const uint32_t page_trans) const { return (uint64_t)(cache.base_addr + (uint64_t)page_trans * cache.page_size); }
    __forceinline__ __device__ void mark_page_dirty(const size_t index) { __hip_atomic_fetch_or(&pages[index].state, DIRTY, __ATOMIC_RELAXED, BAM_AGENT); }
    __forceinline__ __device__ uint64_t acquire_page(const size_t pg, const uint32_t count, const bool write, const uint32_t ctrl, const uint32_t queue);
    __forceinline__ __device__ bam_stat_shard_t* shard() const { return stats + (bam::cu_id() & (BAM_STAT_SHARDS - 1)); }
};

namespace bam {
/* add to a counter; when every active lane names the same word the address is made
 * wave-uniform so that the compiler folds the wave's adds into one atomic */
__device__ __forceinline__ void stat_add(unsigned long long* ctr, uint32_t v)
{
    const uint64_t a0 = first((uint64_t)ctr);
    if (!ballot((uint64_t)ctr != a0)) __hip_atomic_fetch_add((unsigned long long*)a0, (unsigned long long)v, __ATOMIC_RELAXED, BAM_AGENT);
    else __hip_atomic_fetch_add(ctr, (unsigned long long)v, __ATOMIC_RELAXED, BAM_AGENT);
}
} // namespace bam

/*
 * The page state machine.  Takes `count` references on page `pg` and returns
 * the cache slot that holds it, loading it first if needed.  Callable by any
 * subset of a wave's lanes, each for a different page: the lanes step through
 * the states together, and those that have to load a page do their victim
 * search and their NVMe reads as one batch.
 *
 *   VALID, not BUSY : hit
 *   not VALID, not BUSY : whoever sets BUSY first loads the page, then flips BUSY->VALID
 *   BUSY : somebody else is loading or evicting; wait and look again
 */
template <typename T>
__forceinline__ __device__
uint64_t range_d_t<T>::acquire_page(const size_t pg, const uint32_t count, const bool write, const uint32_t ctrl_, const uint32_t queue)
{
    using namespace bam;
    (void)ctrl_;
    data_page_t* dp = &pages[pg];
    bam_stat_shard_t* sh = shard();
    stat_add(&sh->access_cnt, count);
    uint32_t s = __hip_atomic_fetch_add(&dp->state, count, __ATOMIC_ACQUIRE, BAM_AGENT);
    uint32_t slot = 0;
    bool resolved = false;
    spin_t sp;
    for (;;) {
        bool load_me = false;
        if (!resolved) {
            const uint32_t st = s >> (CNT_SHIFT + 1);
            if (st == V_NB) {
                if (write && (s & DIRTY) == 0) __hip_atomic_fetch_or(&dp->state, DIRTY, __ATOMIC_RELAXED, BAM_AGENT);
                slot = ld_relaxed(&dp->offset);
                stat_add(&sh->hit_cnt, count);
                resolved = true;
            } else if (st == NV_NB) {
                const uint32_t o = __hip_atomic_fetch_or(&dp->state, BUSY, __ATOMIC_ACQUIRE, BAM_AGENT);
                if ((o & BUSY) == 0) {
                    if ((o >> (CNT_SHIFT + 1)) == NV_NB) load_me = true;
                    else __hip_atomic_fetch_and(&dp->state, DISABLE_BUSY_MASK, __ATOMIC_RELEASE, BAM_AGENT);  /* became valid meanwhile */
                }
            }
        }
        const uint64_t loaders = ballot(load_me);
        if (load_me) {
            slot = cache.find_slot(pg, range_id, queue);
            uint64_t c = get_backing_ctrl(pg);
            if (c == ALL_CTRLS) c = cache.n_ctrls == 1 ? 0 : cache.ctrl_counter->fetch_add(1, simt::memory_order_relaxed) % cache.n_ctrls;
            Controller* ctl = cache.d_ctrls[c];
            stat_add((unsigned long long*)&ctl->access_counter, 1);
            stat_add(&sh->read_io_cnt, 1);
            read_data(&cache, ctl->d_qps + (queue % ctl->n_qps), get_backing_page(pg) * cache.n_blocks_per_page, cache.n_blocks_per_page, slot);
            st_relaxed(&dp->offset, slot);
            stat_add(&sh->miss_cnt, count);
            if (write) __hip_atomic_fetch_or(&dp->state, DIRTY, __ATOMIC_RELAXED, BAM_AGENT);
            /* BUSY -> 0 and VALID -> 1 in one step; publishes the payload and the offset */
            __hip_atomic_fetch_xor(&dp->state, DISABLE_BUSY_ENABLE_VALID, __ATOMIC_RELEASE, BAM_AGENT);
            resolved = true;
        }
        if (!ballot(!resolved)) break;
        if (!loaders && cache.spin_giveup(sp)) break;
        if (!resolved) s = ld_acquire(&dp->state);
    }
    return slot;
}

/* ------------------------------------------------------------------ */
/* arrays                                                             */
/* ------------------------------------------------------------------ */

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

    /*
     * Wave-level request coalescing: lanes that want the same page of the same
     * array form a group; the lowest lane of each group ("master") takes the
     * group's references in one go.  eq_mask/master/count describe the caller's
     * group, base_master is the cache slot.
     */
    __forceinline__ __device__ void coalesce_page(const uint32_t lane, const uint64_t mask, const int64_t r, const uint64_t page, const uint64_t gaddr, const bool write,
                                                  uint64_t& eq_mask, int& master, uint32_t& count, uint64_t& base_master) const
    {
        (void)mask;
        range_d_t<T>* r_ = d_ranges + r;
        const uint32_t queue = get_smid();        /* reduced modulo the controller's queue count at the point of use */
        eq_mask = bam::match_any(gaddr, (uint64_t)this);
        master = (int)bam::first_lane(eq_mask);
        count = bam::popc(eq_mask);
        const bool dirty = (bam::ballot(write) & eq_mask) != 0;
        uint64_t base = 0;
        if (master == (int)lane) base = r_->acquire_page(page, count, dirty, 0, queue);
        base_master = bam::shfl(base, (uint32_t)master);
    }

    /*
     * Run `fn(address of element i in the cache)` with the page referenced, for
     * every active lane, holding at most cache.wave_batch distinct pages of
     * this wave referenced at any time.
     */
    template <typename F>
    __forceinline__ __device__ void with_element(const size_t i, const bool write, F&& fn) const
    {
        const int64_t r = find_range(i);
        if (r == -1) return;
        range_d_t<T>* r_ = d_ranges + r;
        const uint32_t lane = lane_id();
        const uint64_t page = r_->get_page(i), subindex = r_->get_subindex(i), gaddr = r_->get_global_address(page);
        const uint64_t eq_mask = bam::match_any(gaddr, (uint64_t)this);
        const uint32_t master = bam::first_lane(eq_mask), count = bam::popc(eq_mask);
        const bool dirty = (bam::ballot(write) & eq_mask) != 0;
        const uint64_t masters = bam::ballot(master == lane);
        const uint32_t n_masters = bam::popc(masters), my_group = bam::popc(masters & bam::lanes_below(master));
        const uint32_t batch = bam::first(r_->cache.wave_batch);
        const uint32_t queue = get_smid();
        for (uint32_t g0 = 0; g0 < n_masters; g0 += batch) {
            if (my_group >= g0 && my_group < g0 + batch) {
                uint64_t base = 0;
                if (master == lane) base = r_->acquire_page(page, count, dirty, 0, queue);
                base = bam::shfl(base, master);
                fn((T*)(r_->get_cache_page_addr((uint32_t)base) + subindex));
                /* every lane of the group has used the page before the master drops the references */
                __builtin_amdgcn_wave_barrier();
                if (master == lane) r_->release_page(page, count);
            }
        }
    }

    __forceinline__ __device__ T seq_read(const size_t i) const
    {
        T ret = T();
        with_element(i, false, [&](T* p) { ret = *p; });
        return ret;
    }

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
     * address of the page in the cache, the element window [start, end) it
     * covers, the page descriptor and the range index.  Pair with release_page.
     */
    __forceinline__ __device__ void* acquire_page(const size_t i, data_page_t*& page_, size_t& start, size_t& end, int64_t& r) const
    {
        const uint32_t lane = lane_id();
        r = find_range(i);
        page_ = nullptr;
        if (r == -1) return nullptr;
        range_d_t<T>* r_ = d_ranges + r;
        uint64_t eq_mask, base_master;
        int master;
        uint32_t count;
        const uint64_t page = r_->get_page(i);
        coalesce_page(lane, bam::active_mask(), r, page, r_->get_global_address(page), false, eq_mask, master, count, base_master);
        page_ = &r_->pages[page];
        /* first element of the page; a page may start before the range when page_start_offset != 0 */
        const uint64_t first_byte = (page << r_->cache.page_size_log);
        const uint64_t first_elem = first_byte <= r_->page_start_offset ? 0 : (first_byte - r_->page_start_offset) / sizeof(T);
        start = r_->index_start + first_elem;
        end = r_->index_start + ((first_byte + r_->cache.page_size - r_->page_start_offset) / sizeof(T));
        return (void*)(r_->get_cache_page_addr((uint32_t)base_master) + r_->get_subindex(start));
    }

    __forceinline__ __device__ void release_page(data_page_t* page_, const int64_t r, const size_t i) const
    {
        (void)page_;
        if (r == -1) return;
        range_d_t<T>* r_ = d_ranges + r;
        const uint64_t page = r_->get_page(i);
        const uint64_t eq_mask = bam::match_any(r_->get_global_address(page), (uint64_t)this);
        if (bam::first_lane(eq_mask) == lane_id()) r_->release_page(page, bam::popc(eq_mask));
    }
};

template <typename T> struct bam_ptr;

/*
 * What bam_ptr::operator[] hands out on a non-const pointer: converts to T for
 * a read and marks the page dirty only when assigned through.  (The reference
 * returns T& there and marks the page dirty on every window change, reads
 * included, include/page_cache.h:476-483, which turns every eviction of a
 * read-only workload into a write-back.)
 */
template <typename T>
struct bam_ref {
    bam_ptr<T>* p;
    size_t i;
    __forceinline__ __host__ __device__ operator T() const { return p->read(i); }
    __forceinline__ __host__ __device__ bam_ref& operator=(T v) { p->write(i, v); return *this; }
    __forceinline__ __host__ __device__ bam_ref& operator=(const bam_ref& o) { p->write(i, (T)o); return *this; }
    __forceinline__ __host__ __device__ bam_ref& operator+=(T v) { p->write(i, p->read(i) + v); return *this; }
};

/*
 * Per-thread window onto an array: keeps the page of the last access
 * referenced, so that a run of accesses to one page costs one acquire and one
 * release.  Same contract as the reference's bam_ptr (include/page_cache.h:414-485).
 * A thread holds one page referenced for as long as the window stays on it, so
 * the cache must have more pages than the threads of the resident waves can
 * hold at once (the reference has the same requirement).
 */
template <typename T>
struct bam_ptr {
    data_page_t* page = nullptr;
    array_d_t<T>* array = nullptr;
    size_t start = 0;
    size_t end = 0;
    int64_t range_id = -1;
    T* addr = nullptr;
    bool dirty = false;

    __forceinline__ __host__ __device__ bam_ptr(array_d_t<T>* a) { init(a); }
    __forceinline__ __host__ __device__ ~bam_ptr() { fini(); }
    __forceinline__ __host__ __device__ void init(array_d_t<T>* a) { array = a; }

    __forceinline__ __host__ __device__ void fini(void)
    {
#if defined(__HIP_DEVICE_COMPILE__)
        if (page) {
            array->release_page(page, range_id, start);
            page = nullptr;
        }
#endif
    }

    __forceinline__ __host__ __device__ T* update_page(const size_t i)
    {
#if defined(__HIP_DEVICE_COMPILE__)
        fini();
        addr = (T*)array->acquire_page(i, page, start, end, range_id);
        dirty = false;
#endif
        return addr;
    }

    __forceinline__ __host__ __device__ T read(const size_t i)
    {
        if (i < start || i >= end) update_page(i);
        return addr[i - start];
    }

    __forceinline__ __host__ __device__ void mark_dirty()
    {
#if defined(__HIP_DEVICE_COMPILE__)
        if (!dirty) { __hip_atomic_fetch_or(&page->state, DIRTY, __ATOMIC_RELAXED, BAM_AGENT); dirty = true; }
#endif
    }

    __forceinline__ __host__ __device__ void write(const size_t i, const T v)
    {
        if (i < start || i >= end) update_page(i);
        mark_dirty();
        addr[i - start] = v;
    }

    __forceinline__ __host__ __device__ T operator[](const size_t i) const { return const_cast<bam_ptr*>(this)->read(i); }
    __forceinline__ __host__ __device__ bam_ref<T> operator[](const size_t i) { return bam_ref<T>{this, i}; }

    /* address of element i for the caller to read or write: counts as a write */
    __forceinline__ __host__ __device__ T* memref(size_t i)
    {
        if (i < start || i >= end) update_page(i);
        mark_dirty();
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
    if (bam::ld_relaxed(&pc->cache_pages[page].page_take_lock) == FREE) return;
    const uint64_t g = pc->cache_pages[page].page_translation;
    const uint64_t range = g & pc->n_ranges_mask, addr = g >> pc->n_ranges_bits;
    data_page_t* dp = &pc->ranges[range][addr];
    const uint32_t s = bam::ld_relaxed(&dp->state);
    if ((s & DIRTY) == 0 || (s & VALID) == 0 || bam::ld_relaxed(&dp->offset) != page) return;
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
    BufferPtr ctrl_counter_buf;
    BufferPtr extra_reads_buf;

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
            for (size_t i = 0; i < np; i++) { tps[i].page_take_lock = FREE; tps[i].pad = 0; tps[i].page_translation = 0; }
            hip_err_chk(hipMemcpy(pdt.cache_pages, tps.data(), np * sizeof(cache_page_t), hipMemcpyHostToDevice));
        }
        page_ticket_buf = createBuffer(sizeof(uint32_t), hipDevice);
        pdt.page_ticket = (uint32_t*)page_ticket_buf.get();

        /* how many pages a wave may pin while loading: leave at least half of the cache evictable */
        hipDeviceProp_t prop;
        hip_err_chk(hipGetDeviceProperties(&prop, hipDevice));
        const uint64_t max_waves = (uint64_t)prop.multiProcessorCount * prop.maxThreadsPerMultiProcessor / BAM_WAVE_SIZE;
        uint64_t batch = np / (2 * (max_waves ? max_waves : 1));
        pdt.wave_batch = (uint32_t)(batch < 1 ? 1 : batch > BAM_WAVE_SIZE ? BAM_WAVE_SIZE : batch);
        if (const char* e = getenv("BAM_WAVE_BATCH")) { int v = atoi(e); if (v >= 1 && v <= BAM_WAVE_SIZE) pdt.wave_batch = (uint32_t)v; }

        const bool staged = ctrl.n_qps && ctrl.h_qps[0]->stage != nullptr;
        const uint64_t cache_size = ps * np;
        if (staged) {
            /* the controller never addresses the cache: plain device memory, no PRP tables */
            if (ps > ctrl.h_qps[0]->stage_stride) throw error(string("page_cache_t: page size exceeds the staging window of the queue pairs"));
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
            for (auto& s : sh) { r.read_io_cnt += s.read_io_cnt; r.access_cnt += s.access_cnt; r.miss_cnt += s.miss_cnt; r.hit_cnt += s.hit_cnt; }
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
