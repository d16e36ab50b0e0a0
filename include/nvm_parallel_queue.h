/*
 * Concurrent NVMe submission/completion protocol for gfx950 wavefronts.
 *
 * Same job and same entry points as include/nvm_parallel_queue.h of the
 * reference (get_cid :35-52, put_cid :54-57, move_tail :59-80, move_head_cq
 * :82-123, sq_enqueue :167-330, cq_poll :378-422, cq_dequeue :424-535), and
 * the same wire behaviour towards the controller: ticketed SQ slots, one tail
 * doorbell per contiguous run of written entries, SQ slots recycled from the
 * SQHD field of completions, one CQ-head doorbell per run of consumed entries.
 *
 * The execution model is different.  A gfx950 wave runs its 64 lanes in lock
 * step, so a lane must never spin on something a masked-off sibling produces.
 * Every operation here is therefore done by the whole group of active lanes
 * that target the same queue:
 *   - one in_ticket fetch_add(n) per group reserves n consecutive SQ slots;
 *   - lanes write their own 64-byte entries and set tail_mark; the group's
 *     leader try-locks tail_lock and the group sweeps up to 64 marks per load;
 *   - completions are not searched for per thread.  Whichever group holds
 *     head_lock drains the CQ 64 entries per load and flags each completed
 *     command in the cid table (cid[c] = LOCKED|DONE); waiters poll their own
 *     word.  The drainer frees SQ slots from SQHD and rings the CQ doorbell
 *     once per sweep.
 * All waits are bounded (bam_guard_t).
 */
#ifndef __NVM_PARALLEL_QUEUE_H_
#define __NVM_PARALLEL_QUEUE_H_

#include "bam_wave.h"
#include "nvm_cmd.h"
#include "nvm_types.h"
#include "nvm_util.h"

#define LOCKED   1
#define UNLOCKED 0
#define BAM_CID_DONE 2u
#define BAM_CID_ERR  4u          /* completed with a non-zero status: the transfer did not happen */

namespace bam {

struct spin_t { uint32_t n = 0, slp = 1; uint64_t t0 = 0; };

/* phase timers: compiled in with -DBAM_PROFILE only */
#ifdef BAM_PROFILE
/* the clock, read once everything the wave has in flight has come back (the clock is a scalar read that the hardware
 * would otherwise let overtake vector memory operations it does not depend on) */
__device__ __forceinline__ uint64_t prof_clock()
{
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    const uint64_t t = wall_clock64();
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    return t;
}
#define BAM_PROF_NOW() bam::prof_clock()
#define BAM_PROF_ADD(q, i, v) do { if ((q)->prof) atomicAdd(&(q)->prof[i], (unsigned long long)(v)); } while (0)
#else
#define BAM_PROF_NOW() 0ull
#define BAM_PROF_ADD(q, i, v) do { } while (0)
#endif

/*
 * One back-off step of a wait loop; true = give up.  Every 256 steps the loop
 * looks at the shared abort flag and at the wall clock (100 MHz constant
 * counter): a wait that has lasted longer than `limit_us` microseconds raises
 * the abort flag itself.  limit_us = 0 waits for ever.
 */
__device__ __forceinline__ bool spin_giveup(bam_guard_t* g, uint32_t limit_us, spin_t& s)
{
    backoff(s.slp);
    if ((++s.n & 255u) != 0 || !g) return false;
    if (ld_relaxed_sys(&g->abort)) return true;
    if (!limit_us) return false;
    const uint64_t now = wall_clock64();
    if (!s.t0) { s.t0 = now; return false; }
    if (now - s.t0 > (uint64_t)limit_us * 100u) { st_relaxed_sys(&g->abort, 1u); return true; }
    return false;
}
__device__ __forceinline__ bool spin_giveup(const nvm_queue_t* q, spin_t& s) { return spin_giveup(q->guard, q->spin_limit, s); }

/* lanes of `act` with rank below `run` where run = length of the leading all-true prefix of `ok` in rank order */
__device__ __forceinline__ uint32_t leading_run(uint64_t act, uint64_t ok)
{
    uint64_t miss = act & ~ok;
    return miss ? popc(act & lanes_below(first_lane(miss))) : popc(act);
}

/* ---- command ids ---- */
/*
 * Command ids are handed out to a group of lanes as one block of 64 (ids
 * 64*b .. 64*b+63): one atomic per wave instead of one per command, and a
 * wave never sits on a few ids while it waits for more, which would leave two
 * waves that share a queue each holding part of what the other needs.
 * Blocks are ticket locks: the n-th wave to ask gets block n mod n_blocks and
 * waits for that block's turn counter to reach n div n_blocks, so waves are
 * served in arrival order and none starves.  Returns the lane's id (block
 * base + rank of the lane in the group); the caller holds nothing else it
 * would have to give up while this waits.
 */
__device__ __forceinline__ uint32_t get_cid_group(nvm_queue_t* sq)
{
    const uint64_t act = active_mask();
    const uint32_t leader = first_lane(act);
    const uint32_t n_blocks = (sq->cid_mask + 1u) >> 6;          /* power of two */
    uint32_t base = 0;
    if (lane() == leader) {
        const uint32_t t = __hip_atomic_fetch_add(&sq->cid_ticket, 1u, __ATOMIC_RELAXED, BAM_AGENT);
        const uint32_t b = t & (n_blocks - 1), shift = (uint32_t)__builtin_ctz(n_blocks);
        const uint32_t turn_mask = 0xffffffffu >> shift;
        spin_t sp;
        /* polled with plain loads: an acquire per look would invalidate this compute unit's cache every time */
        while (((ld_relaxed(&sq->pos_locks[b].val) - (t >> shift)) & turn_mask) != 0)
            if (spin_giveup(sq, sp)) break;
        fence_meta();
        st_relaxed(&sq->head_mark[b].val, popc(act));       /* ids of this block still out */
        base = b << 6;
    }
    base = bcast(base, leader);
    const uint32_t id = base + rank_in(act);
    st_relaxed(&sq->cid[id].val, (uint32_t)LOCKED);
    return id;
}

/*
 * Give command ids back.  The lanes that took a block together may return
 * their ids in one call or in several (the asynchronous entry points are
 * called thread by thread); the block's turn moves on when its last id is in.
 */
__device__ __forceinline__ void put_cid_group(nvm_queue_t* sq, uint32_t id)
{
    st_relaxed(&sq->cid[id].val, (uint32_t)UNLOCKED);
    fence_meta();                    /* whatever the lanes did with their ids and staging pages is over */
    for_each_group((uint64_t)(id >> 6), [&](uint64_t b) {
        const uint64_t grp = active_mask();
        if (lane() == first_lane(grp)) {
            const uint32_t k = popc(grp);
            if (__hip_atomic_fetch_add(&sq->head_mark[b].val, 0u - k, __ATOMIC_RELAXED, BAM_AGENT) == k)
                __hip_atomic_fetch_add(&sq->pos_locks[b].val, 1u, __ATOMIC_RELAXED, BAM_AGENT);   /* next turn */
        }
    });
}

__device__ __forceinline__ void cq_drain_group(nvm_queue_t* cq, nvm_queue_t* sq, uint64_t act);

/*
 * Drain the completion queue if nobody else is doing so; true if this group
 * did.  The ring may live on the far side of the interconnect, and every
 * waiting wave comes through here, so an idle ring must cost next to nothing:
 * the holder of head_lock first reads the one entry at the head (a single
 * small read), and only when that entry is new does the group read a window
 * of 64; after an empty look a ring in host memory is left alone for
 * cq->idle_ticks (two microseconds; the time is kept in the otherwise unused
 * `tail` word of the CQ descriptor).  A ring in device memory has no such
 * pause: a look at it stays on the device.
 */
__device__ __forceinline__ bool try_drain_group(nvm_queue_t* cq, nvm_queue_t* sq)
{
    const uint64_t act = active_mask();
    const uint32_t leader = first_lane(act);
    uint32_t got = 0;
    if (lane() == leader) {
        /* the word holds the time of the next look (low 32 bits of the clock): wait only while that lies within
         * the next idle_ticks, so that a stale or never-written value can never hold anybody up */
        const uint32_t idle = cq->idle_ticks;
        const uint32_t ahead = idle ? ld_relaxed(&cq->tail) - (uint32_t)wall_clock64() : 0u;
        if (ahead - 1u >= idle && ld_relaxed(&cq->head_lock) == UNLOCKED &&
            __hip_atomic_exchange(&cq->head_lock, (uint32_t)LOCKED, __ATOMIC_RELAXED, BAM_AGENT) == UNLOCKED) {
            fence_meta();
            const uint32_t h = ld_relaxed(&cq->head);
            [[maybe_unused]] const uint64_t po5 = BAM_PROF_NOW();
            const uint32_t dw3 = ld_relaxed_sys(&((nvm_cpl_t*)cq->vaddr)[h & cq->qs_minus_1].dword[3]);
            BAM_PROF_ADD(cq, 27, 1); BAM_PROF_ADD(cq, 28, BAM_PROF_NOW() - po5);
            if (((dw3 >> 16) & 1u) == ((~(h >> cq->qs_log2)) & 1u)) got = 1;
            else {
                if (idle) st_relaxed(&cq->tail, (uint32_t)wall_clock64() + idle);      /* nothing new: leave the ring alone for a while */
                st_publish(&cq->head_lock, (uint32_t)UNLOCKED);
                BAM_PROF_ADD(cq, 20, 1);
            }
        }
    }
    got = bcast(got, leader);
    if (got) {
        [[maybe_unused]] const uint64_t pd0 = BAM_PROF_NOW();
        cq_drain_group(cq, sq, act);
        if (lane() == leader) { st_publish(&cq->head_lock, (uint32_t)UNLOCKED); BAM_PROF_ADD(cq, 17, 1); BAM_PROF_ADD(cq, 19, BAM_PROF_NOW() - pd0); }
    }
    return got != 0;
}

/*
 * Submit one command per active lane to `sq` (wave-uniform).  Returns the
 * slot the lane's entry went to.  On return every entry is covered by a
 * doorbell write.
 */
__device__ __forceinline__ uint32_t sq_enqueue_group(nvm_queue_t* sq, nvm_cmd_t* cmd)
{
    const uint64_t act = active_mask();
    const uint32_t n = popc(act), rank = rank_in(act), leader = first_lane(act);
    const uint32_t mask = sq->qs_minus_1;
    uint32_t t0 = 0;
    [[maybe_unused]] const uint64_t pq0 = BAM_PROF_NOW();
    [[maybe_unused]] uint64_t pq2 = 0;
    [[maybe_unused]] uint32_t p_trips = 0;
    if (lane() == leader) t0 = __hip_atomic_fetch_add(&sq->in_ticket, n, __ATOMIC_RELAXED, BAM_AGENT);
    t0 = bcast(t0, leader);
    [[maybe_unused]] const uint64_t pq1 = BAM_PROF_NOW();
    const uint32_t ticket = t0 + rank, pos = ticket & mask;
    if (sq->sealed) nvm_cmd_seal(cmd, ticket);
    bool written = false;
    spin_t sp;
    for (;;) {
#ifdef BAM_PROFILE
        const uint64_t po0 = BAM_PROF_NOW();
        const uint32_t slot_word = ld_relaxed(&sq->tickets[pos].val);
        const uint64_t po1 = BAM_PROF_NOW();
        if (lane() == leader && !written) { BAM_PROF_ADD(sq, 22, 1); BAM_PROF_ADD(sq, 23, po1 - po0); }
#else
        const uint32_t slot_word = ld_relaxed(&sq->tickets[pos].val);
#endif
        if (!written && nvm_sq_slot_free(slot_word, ticket, sq->qs_log2)) {
            fence_meta();
            [[maybe_unused]] const uint64_t po2 = BAM_PROF_NOW();
            /* written through to the ring, which may be host memory the L2 would otherwise hold on to */
            uint64_t* dst = (uint64_t*)(((nvm_cmd_t*)sq->vaddr) + pos);
            const uint64_t* src = (const uint64_t*)cmd->dword;
#pragma unroll
            for (int i = 0; i < 8; i++) __hip_atomic_store(dst + i, src[i], __ATOMIC_RELAXED, BAM_SYSTEM);
            /*
             * The entry must be in the ring before its mark can be swept into a doorbell.  A sealed queue leaves that
             * to the controller (it takes an entry only once the seal verifies).  An unsealed one (a controller that
             * follows the NVMe specification to the letter) has to know: the wait on the wave's own store counters
             * says that the stores have been handed on, not that they have arrived, and the doorbell, written later by
             * another wave, may travel another way.  Reading the entry back does say so: the reply to a read does not
             * pass writes posted before it.
             */
#ifdef BAM_PROFILE
            { const uint64_t po3 = BAM_PROF_NOW(); if (lane() == leader) { BAM_PROF_ADD(sq, 24, 1); BAM_PROF_ADD(sq, 25, po3 - po2); } }
#endif
            if (!sq->sealed) {
                if (sq->flush == 1u) fence_release_sys();
                else if (sq->flush == 2u) {
                    fence_meta();
                    const uint64_t back = __hip_atomic_load(dst + 7, __ATOMIC_RELAXED, BAM_SYSTEM);
                    asm volatile("" :: "v"(back));
                }
            }
            st_publish(&sq->tail_mark[pos].val, 1u);
            written = true;
        }
        if (!pq2 && !ballot(!written)) pq2 = BAM_PROF_NOW();
        p_trips++;
        const uint32_t tl = ld_relaxed(&sq->tail);
        const bool covered = written && (int32_t)(tl - ticket) > 0;
        if (!ballot(!covered)) break;
        bool progressed = false;
        if (ballot(written && !covered)) {
            /* try to become the tail mover for this queue */
            uint32_t got = 0;
            if (lane() == leader)
                got = ld_relaxed(&sq->tail_lock) == UNLOCKED &&
                      __hip_atomic_exchange(&sq->tail_lock, (uint32_t)LOCKED, __ATOMIC_RELAXED, BAM_AGENT) == UNLOCKED;
            got = bcast(got, leader);
            if (got) {
                fence_meta();
                const uint32_t cur = ld_relaxed(&sq->tail);
                /* never let tail + 1 == head (mod qs): at most qs - 1 entries outstanding */
                const uint32_t room = ld_relaxed(&sq->head) + sq->qs - 1u - cur;
                uint32_t total = 0;
                for (;;) {
                    const uint32_t k = total + rank;
                    const bool m = k < room && ld_relaxed(&sq->tail_mark[(cur + k) & mask].val) == 1u;
                    const uint32_t run = leading_run(act, ballot(m));
                    if (rank < run) st_relaxed(&sq->tail_mark[(cur + k) & mask].val, 0u);
                    total += run;
                    if (run < n) break;
                }
                fence_meta();                /* the marks read and cleared above: before the doorbell and the unlock */
                if (lane() == leader) {
                    if (total) {
                        [[maybe_unused]] const uint64_t po4 = BAM_PROF_NOW();
                        st_relaxed_sys(sq->db, (cur + total) & mask);     /* one doorbell for the whole run */
                        BAM_PROF_ADD(sq, 26, BAM_PROF_NOW() - po4);
                        st_relaxed(&sq->tail, cur + total);
                        BAM_PROF_ADD(sq, 15, 1); BAM_PROF_ADD(sq, 14, total);
                    }
                    st_publish(&sq->tail_lock, (uint32_t)UNLOCKED);
                    BAM_PROF_ADD(sq, 13, 1);
                }
                progressed = total != 0;
            }
        }
        if (!progressed) {
            /* a full SQ only empties when completions are consumed: do that here too, or a
             * group larger than the queue would wait on itself */
            try_drain_group((nvm_queue_t*)sq->pair, sq);
            if (spin_giveup(sq, sp)) break;
        }
    }
#ifdef BAM_PROFILE
    if (lane() == leader) {
        const uint64_t pq3 = BAM_PROF_NOW();
        if (!pq2) pq2 = pq3;
        BAM_PROF_ADD(sq, 9, pq1 - pq0); BAM_PROF_ADD(sq, 10, pq2 - pq1); BAM_PROF_ADD(sq, 11, pq3 - pq2); BAM_PROF_ADD(sq, 12, p_trips);
    }
#endif
    return pos;
}

/*
 * Drain the completion queue: caller's group holds cq->head_lock.  Flags every
 * completed command in sq->cid[], frees the SQ slots the controller has
 * consumed (SQHD of the newest completion) and rings the CQ head doorbell once.
 */
__device__ __forceinline__ void cq_drain_group(nvm_queue_t* cq, nvm_queue_t* sq, uint64_t act)
{
    const uint32_t n = popc(act), rank = rank_in(act), leader = first_lane(act);
    const uint32_t mask = cq->qs_minus_1;
    const uint32_t h = ld_relaxed(&cq->head);
    nvm_cpl_t* ring = (nvm_cpl_t*)cq->vaddr;
    uint32_t moved = 0, sqhd = 0;
    for (;;) {
        const uint32_t idx = h + moved + rank, loc = idx & mask;
        const uint32_t phase = (~(idx >> cq->qs_log2)) & 1u;          /* first lap carries phase 1 */
        /* SQHD and the phase tag in one access: the controller may write an entry in pieces of eight bytes */
        const uint64_t dw23 = __hip_atomic_load((uint64_t*)&ring[loc].dword[2], __ATOMIC_RELAXED, BAM_SYSTEM);
        const uint32_t dw3 = (uint32_t)(dw23 >> 32);
        fence_meta();
        const bool valid = ((dw3 >> 16) & 1u) == phase && moved + rank < mask;
        const uint32_t run = leading_run(act, ballot(valid));
        if (rank < run) {
            const bool err = (dw3 >> 17) != 0;
            if (err) __hip_atomic_fetch_add(&cq->n_errors, 1u, __ATOMIC_RELAXED, BAM_AGENT);
            st_relaxed(&sq->cid[dw3 & sq->cid_mask].val, (uint32_t)LOCKED | BAM_CID_DONE | (err ? BAM_CID_ERR : 0u));
        }
        if (run) {
            /* lane holding the newest entry of the run */
            const uint64_t holder = ballot(rank == run - 1);
            sqhd = bcast((uint32_t)dw23 & 0xffffu, first_lane(holder));
        }
        moved += run;
        if (run < n) break;
    }
    if (moved) {
        const uint32_t smask = sq->qs_minus_1;
        const uint32_t sh = ld_relaxed(&sq->head);
        const uint32_t freed = (sqhd - sh) & smask;
        fence_meta();
        for (uint32_t i = rank; i < freed; i += n)
            __hip_atomic_fetch_add(&sq->tickets[(sh + i) & smask].val, 2u, __ATOMIC_RELAXED, BAM_AGENT);
        if (lane() == leader) {
            if (freed) st_relaxed(&sq->head, sh + freed);
            st_relaxed_sys(cq->db, (h + moved) & mask);                /* one doorbell for the whole run */
            st_relaxed(&cq->head, h + moved);
            BAM_PROF_ADD(cq, 18, moved);
        }
    }
}

/*
 * Wait until the command `cid` of every active lane has completed on (sq, cq) (wave-uniform).  True for the lanes
 * whose command completed without an error status; false where the transfer did not happen (error completion) or
 * nobody knows (the wait was given up).
 */
__device__ __forceinline__ bool cq_wait_group(nvm_queue_t* cq, nvm_queue_t* sq, uint32_t cid)
{
    spin_t sp;
    uint32_t w;
    [[maybe_unused]] uint32_t p_trips = 0;
    for (;;) {
        w = ld_relaxed(&sq->cid[cid].val);
        if (!ballot((w & BAM_CID_DONE) == 0)) break;
        p_trips++;
        try_drain_group(cq, sq);
        if (spin_giveup(cq, sp)) break;
    }
    if (lane() == first_lane(active_mask())) BAM_PROF_ADD(cq, 16, p_trips);
    /* what the controller wrote before posting the completion is visible from here on */
    fence_acquire_sys();
    return (w & (BAM_CID_DONE | BAM_CID_ERR)) == BAM_CID_DONE;
}

} // namespace bam

/* ---- per-thread entry points with the reference's names ---- */

inline __device__ uint16_t get_cid(nvm_queue_t* sq)
{
    uint32_t id = 0;
    bam::for_each_group((uint64_t)sq, [&](uint64_t q) { id = bam::get_cid_group((nvm_queue_t*)q); });
    return (uint16_t)id;
}

/* to be called by the same lanes that called get_cid together, all at once or in parts */
inline __device__ void put_cid(nvm_queue_t* sq, uint16_t id)
{
    bam::for_each_group((uint64_t)sq, [&](uint64_t q) { bam::put_cid_group((nvm_queue_t*)q, id); });
}

/* returns the SQ slot used */
inline __device__ uint16_t sq_enqueue(nvm_queue_t* sq, nvm_cmd_t* cmd)
{
    uint32_t pos = 0;
    bam::for_each_group((uint64_t)sq, [&](uint64_t q) { pos = bam::sq_enqueue_group((nvm_queue_t*)q, cmd); });
    return (uint16_t)pos;
}

/*
 * Wait for the completion of command `search_cid` submitted on the SQ paired
 * with `cq` (cq->pair).  The reference scans the ring and hands back the entry's position
 * for cq_dequeue; here the drainer has already consumed the entry, so the
 * out-parameters (which the reference dereferences even when NULL,
 * nvm_parallel_queue.h:406-407) are optional and receive the current head.
 */
inline __device__ uint32_t cq_poll(nvm_queue_t* cq, uint16_t search_cid, uint32_t* loc_ = nullptr, uint32_t* cq_head = nullptr)
{
    bam::for_each_group((uint64_t)cq, [&](uint64_t q) { bam::cq_wait_group((nvm_queue_t*)q, (nvm_queue_t*)((nvm_queue_t*)q)->pair, search_cid); });
    uint32_t h = bam::ld_relaxed(&cq->head);
    if (loc_) *loc_ = h;
    if (cq_head) *cq_head = h;
    return h & cq->qs_minus_1;
}

/* Completions are consumed by the drainer inside cq_poll; nothing is left to do per entry. */
inline __device__ void cq_dequeue(nvm_queue_t* cq, uint16_t pos, nvm_queue_t* sq, uint32_t loc_ = 0, uint32_t cur_head_ = 0)
{
    (void)cq; (void)pos; (void)sq; (void)loc_; (void)cur_head_;
}

#endif /* __NVM_PARALLEL_QUEUE_H_ */
