/*
 * Concurrent NVMe submission/completion protocol for gfx950 wavefronts.
 *
 * Same job and same entry points as include/nvm_parallel_queue.h of the
 * reference (get_cid :35-52, put_cid :54-57, move_tail :59-80, move_head_cq
 * :82-123, sq_enqueue :167-330, cq_poll :378-422, cq_dequeue :424-535), and
 * the same wire behaviour towards the controller: ticketed SQ slots, one tail
 * doorbell per contiguous run of written entries, one CQ-head doorbell per run
 * of consumed entries.
 *
 * The execution model is different.  A gfx950 wave runs its 64 lanes in lock
 * step, so a lane must never spin on something a masked-off sibling produces.
 * Every operation here is therefore done by the whole group of active lanes
 * that target the same queue.  And every step that has to wait for memory
 * costs the wave a round trip of a microsecond or several (the payload that
 * other waves of the compute unit pull from host memory comes back through
 * the same in-order return path), so the protocol is laid out to need few of
 * them, one after the other:
 *   - one in_ticket fetch_add(n) per group reserves n consecutive SQ slots; a
 *     command's id IS its slot, and the slot stays taken until the command's
 *     owner has finished with the completion and the staged payload, so there
 *     is no separate allocator of command ids (1 round trip, and 1 to see the
 *     slot free);
 *   - lanes write their own 64-byte entries and mark their slots with the
 *     lap number; the lock of the tail holds the tail itself, so whoever takes
 *     it (1 round trip) knows where to sweep from, reads up to 64 marks at a
 *     time (1), rings one doorbell for the run and lets go without waiting;
 *   - completions are not searched for per thread.  The lock of the CQ head
 *     holds the head; whoever takes it reads 64 entries at a time and flags
 *     each completed command in the cid table (cid[c] = LOCKED|DONE); waiters
 *     poll their own word.  One CQ doorbell per drain.
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

/* ---- lock words that carry the position they guard ---- */
/*
 * tail_lock of an SQ and head_lock of a CQ: bit 0 = held, bits 31:1 = the tail / head (free running, 31 bits).  Taking
 * the lock with a fetch-or hands the taker the position in the same round trip, and letting go is one store of the new
 * position.
 */
#define BAM_POS_MASK 0x7fffffffu
__device__ __forceinline__ bool pos_before(uint32_t ticket, uint32_t pos31)          /* ticket < pos, both mod 2^31 */
{
    const uint32_t d = (pos31 - ticket) & BAM_POS_MASK;
    return d != 0 && d < 0x40000000u;
}
/* what a slot's mark reads once its entry for the lap of `idx` (free-running index, any width above 31 bits ignored) is written */
__device__ __forceinline__ uint32_t lap_mark(uint32_t idx, uint32_t qs_log2) { return ((idx & BAM_POS_MASK) >> qs_log2) + 1u; }

__device__ __forceinline__ void cq_drain_group(nvm_queue_t* cq, nvm_queue_t* sq, uint64_t act, uint32_t h);

/*
 * Drain the completion queue if nobody else is doing so; true if this group
 * did.  Every waiting wave comes through here, so a look must cost next to
 * nothing: one fetch-or for lock and head, one read of the entry at the head
 * (by every lane: the window of 64 that a drain starts with).  A ring in host
 * memory is left alone for cq->idle_ticks after an empty look (two
 * microseconds; the time is kept in the otherwise unused `tail` word of the
 * CQ descriptor): a look at it crosses the interconnect.  A ring in device
 * memory has no such pause.
 */
__device__ __forceinline__ bool try_drain_group(nvm_queue_t* cq, nvm_queue_t* sq)
{
    const uint64_t act = active_mask();
    const uint32_t leader = first_lane(act);
    uint32_t got = 0, h = 0;
    if (lane() == leader) {
        /* the word holds the time of the next look (low 32 bits of the clock): wait only while that lies within
         * the next idle_ticks, so that a stale or never-written value can never hold anybody up */
        const uint32_t idle = cq->idle_ticks;
        const uint32_t ahead = idle ? ld_relaxed(&cq->tail) - (uint32_t)wall_clock64() : 0u;
        if (ahead - 1u >= idle) {
            const uint32_t old = __hip_atomic_fetch_or(&cq->head_lock, 1u, __ATOMIC_RELAXED, BAM_AGENT);
            if ((old & 1u) == 0) { got = 1; h = old >> 1; }
        }
    }
    got = bcast(got, leader);
    if (!got) return false;
    h = bcast(h, leader);
    [[maybe_unused]] const uint64_t pd0 = BAM_PROF_NOW();
    cq_drain_group(cq, sq, act, h);
    if (lane() == leader) { BAM_PROF_ADD(cq, 17, 1); BAM_PROF_ADD(cq, 19, BAM_PROF_NOW() - pd0); }
    return true;
}

/*
 * Drain the completion queue from head `h`: the caller's group holds cq->head_lock and lets go of it here.  Flags
 * every completed command in sq->cid[], notes how far the controller has read the SQ (SQHD of the newest completion;
 * the tail sweep keeps the tail one entry short of it) and rings the CQ head doorbell once.
 */
__device__ __forceinline__ void cq_drain_group(nvm_queue_t* cq, nvm_queue_t* sq, uint64_t act, uint32_t h)
{
    const uint32_t n = popc(act), rank = rank_in(act), leader = first_lane(act);
    const uint32_t mask = cq->qs_minus_1;
    nvm_cpl_t* ring = (nvm_cpl_t*)cq->vaddr;
    uint32_t moved = 0, sqhd = 0;
    for (;;) {
        const uint32_t idx = (h + moved + rank) & BAM_POS_MASK, loc = idx & mask;
        const uint32_t phase = (~(idx >> cq->qs_log2)) & 1u;          /* first lap carries phase 1 */
        /* SQHD and the phase tag in one access: the controller may write an entry in pieces of eight bytes */
        const uint64_t dw23 = __hip_atomic_load((uint64_t*)&ring[loc].dword[2], __ATOMIC_RELAXED, BAM_SYSTEM);
        const uint32_t dw3 = (uint32_t)(dw23 >> 32);
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
    if (lane() == leader) {
        if (moved) {
            /* how far the controller has read the submission ring, free running: the newest SQHD is at most one lap ahead of the last */
            const uint32_t sh = ld_relaxed(&sq->head);
            st_relaxed(&sq->head, sh + ((sqhd - sh) & sq->qs_minus_1));
            st_relaxed_sys(cq->db, (h + moved) & mask);                /* one doorbell for the whole run */
            st_relaxed(&cq->head, h + moved);
            st_relaxed(&cq->in_ticket, 0u);
            /* The controller looks at this doorbell only when the ring is full as far as it knows, and then it must
             * find the newest value: the store has been handed on before the next drainer can write another.  (Handed
             * on is not arrived: see the empty look below.) */
            fence_meta();
            BAM_PROF_ADD(cq, 18, moved);
        } else {
            if (cq->idle_ticks) st_relaxed(&cq->tail, (uint32_t)wall_clock64() + cq->idle_ticks);      /* nothing new: leave the ring alone for a while */
            /* Two doorbell writes of two waves may still arrive in the wrong order, and the controller, finding the
             * older value last, would wait with a full ring for a doorbell that nobody owes it.  Waves that keep
             * finding the ring empty therefore write the head again now and then (the in_ticket word, unused on a CQ,
             * counts the empty looks since the last drain). */
            const uint32_t looks = ld_relaxed(&cq->in_ticket) + 1u;
            st_relaxed(&cq->in_ticket, looks);
            if ((looks & 63u) == 0) st_relaxed_sys(cq->db, h & mask);
            BAM_PROF_ADD(cq, 20, 1);
        }
        /* the entries have been read (their values were used above): the next drainer may have the ring */
        st_relaxed(&cq->head_lock, ((h + moved) & BAM_POS_MASK) << 1);
    }
}

/* ---- submission ---- */
/*
 * Reserve one SQ slot per active lane on `sq` (wave-uniform) and wait until each is free.  Returns the lane's ticket;
 * its slot, which is also its command id, is ticket & (qs - 1).  A slot is free again when the owner of the command
 * that had it before has given it back (sq_release_group), so at most qs commands of a queue are out at a time and a
 * command id never names two of them.
 */
__device__ __forceinline__ uint32_t sq_reserve_group(nvm_queue_t* sq)
{
    const uint64_t act = active_mask();
    const uint32_t n = popc(act), rank = rank_in(act), leader = first_lane(act);
    uint32_t t0 = 0;
    [[maybe_unused]] const uint64_t pq0 = BAM_PROF_NOW();
    if (lane() == leader) t0 = __hip_atomic_fetch_add(&sq->in_ticket, n, __ATOMIC_RELAXED, BAM_AGENT);
    t0 = bcast(t0, leader);
    [[maybe_unused]] const uint64_t pq1 = BAM_PROF_NOW();
    const uint32_t ticket = t0 + rank, pos = ticket & sq->qs_minus_1;
    spin_t sp;
    for (;;) {
        const bool is_free = nvm_sq_slot_free(ld_relaxed(&sq->tickets[pos].val), ticket, sq->qs_log2);
        if (!ballot(!is_free)) break;
        /* the slots come back when completions are consumed: do that here too, or a group larger than what is
         * left of the queue would wait on itself */
        try_drain_group((nvm_queue_t*)sq->pair, sq);
        if (spin_giveup(sq, sp)) break;
    }
    st_relaxed(&sq->cid[pos].val, (uint32_t)LOCKED);
    if (lane() == leader) { BAM_PROF_ADD(sq, 9, pq1 - pq0); BAM_PROF_ADD(sq, 10, BAM_PROF_NOW() - pq1); }
    return ticket;
}

/* Give the slots (command ids) of the active lanes back: what the lanes did with their completions and staging pages is over. */
__device__ __forceinline__ void sq_release_group(nvm_queue_t* sq, uint32_t pos)
{
    fence_meta();
    __hip_atomic_fetch_add(&sq->tickets[pos].val, 2u, __ATOMIC_RELAXED, BAM_AGENT);
}

/*
 * Write the entry of every active lane into its reserved slot of `sq` (wave-uniform) and see to it that a doorbell
 * covers it.  `cmd` carries the slot as its command id.
 */
__device__ __forceinline__ void sq_submit_group(nvm_queue_t* sq, nvm_cmd_t* cmd, const uint32_t ticket)
{
    const uint64_t act = active_mask();
    const uint32_t n = popc(act), rank = rank_in(act), leader = first_lane(act);
    const uint32_t mask = sq->qs_minus_1, pos = ticket & mask;
    const uint32_t t0 = bcast(ticket, leader);
    [[maybe_unused]] const uint64_t pq2 = BAM_PROF_NOW();
    if (sq->sealed) nvm_cmd_seal(cmd, ticket);
    /* written through to the ring, which may be host memory the L2 would otherwise hold on to */
    uint64_t* dst = (uint64_t*)(((nvm_cmd_t*)sq->vaddr) + pos);
    /* four stores of sixteen bytes, not eight of eight: an entry in host memory leaves the GPU as one write per store,
     * and the rate at which single-command batches go out doubled with half as many (2.5 to 5 M per second) */
    {
        const uint32_t* w = cmd->dword;
#pragma unroll
        for (int i = 0; i < 4; i++) { u32x4_t v = {w[4 * i], w[4 * i + 1], w[4 * i + 2], w[4 * i + 3]}; st16_sys((uint8_t*)dst + 16 * i, v); }
    }
    /*
     * The entry must be in the ring before a doorbell that covers it reaches the controller.  A sealed queue leaves
     * that to the controller (it takes an entry only once the seal verifies, doorbell or no doorbell).  An unsealed
     * one (a controller that follows the NVMe specification to the letter) has to know: a wait on the wave's own store
     * counters says that the stores have been handed on, not that they have arrived, and the doorbell, written later by
     * another wave, may travel another way.  Reading the entry back does say so: the reply to a read does not pass
     * writes posted before it.
     */
    if (!sq->sealed) {
        if (sq->flush == 1u) fence_release_sys();
        else if (sq->flush == 2u) {
            fence_meta();
            const uint64_t back = __hip_atomic_load(dst + 7, __ATOMIC_RELAXED, BAM_SYSTEM);
            asm volatile("" :: "v"(back));
        }
        fence_meta();
    }
    st_relaxed(&sq->tail_mark[pos].val, lap_mark(ticket, sq->qs_log2));
    [[maybe_unused]] const uint64_t pq3 = BAM_PROF_NOW();
    [[maybe_unused]] uint32_t p_trips = 0;
    /* cover: sweep the marks from the tail on, or wait for whoever is doing that to get past this group's entries */
    bool covered = false;
    spin_t sp;
    for (;;) {
        p_trips++;
        uint32_t got = 0, cur = 0;
        if (lane() == leader) {
            const uint32_t old = __hip_atomic_fetch_or(&sq->tail_lock, 1u, __ATOMIC_RELAXED, BAM_AGENT);
            got = (old & 1u) == 0;
            cur = old >> 1;
        }
        got = bcast(got, leader);
        cur = bcast(cur, leader);
        bool progressed = false;
        if (got) {
            /* never let tail + 1 == head (mod qs): at most qs - 1 entries between what the controller has read and the tail */
            const uint32_t room = ((ld_relaxed(&sq->head) & BAM_POS_MASK) + sq->qs - 1u - cur) & BAM_POS_MASK;
            uint32_t total = 0;
            for (;;) {
                const uint32_t k = total + rank, idx = (cur + k) & BAM_POS_MASK;
                /* this group's own entries are written (above), whatever their marks read by now */
                const bool own = ((idx - t0) & BAM_POS_MASK) < n;
                const bool m = k < room && (own || ld_relaxed(&sq->tail_mark[idx & mask].val) == lap_mark(idx, sq->qs_log2));
                const uint32_t run = leading_run(act, ballot(m));
                total += run;
                if (run < n) break;
            }
            const uint32_t new_tail = (cur + total) & BAM_POS_MASK;
            if (lane() == leader) {
                if (total) {
                    st_relaxed_sys(sq->db, new_tail & mask);     /* one doorbell for the whole run */
                    /* unsealed: the doorbell is there before the next one can leave */
                    if (!sq->sealed && sq->flush) { fence_meta(); const uint32_t back = ld_relaxed_sys(sq->db); asm volatile("" :: "v"(back)); fence_meta(); }
                    st_relaxed(&sq->tail, new_tail);
                    BAM_PROF_ADD(sq, 15, 1); BAM_PROF_ADD(sq, 14, total);
                }
                st_relaxed(&sq->tail_lock, new_tail << 1);
                BAM_PROF_ADD(sq, 13, 1);
            }
            covered = pos_before(ticket, new_tail);
            progressed = total != 0;
        } else
            covered = pos_before(ticket, cur);
        /* A sealed queue's controller takes entries by their seals, announced or not: the doorbell is a courtesy, rung
         * by whoever finds the lock free, and nobody waits for it.  (Waiting would even be wrong: the controller may
         * have read a whole lap of entries between two completions that report how far it has read, which looks like
         * no progress at all, and the tail would stay one entry short of a head that never seems to move.) */
        if (sq->sealed) break;
        if (!ballot(!covered)) break;
        if (!progressed) {
            /* somebody else is sweeping, or the queue is full: watch the tail with plain loads until this group is
             * covered or the lock is free again; a full SQ only empties when completions are consumed */
            const uint32_t w = bcast(ld_relaxed(&sq->tail_lock), leader);
            covered = pos_before(ticket, w >> 1);
            if (!ballot(!covered)) break;
            if (w & 1u) { if (spin_giveup(sq, sp)) break; }
            else if (!got) continue;
            else { try_drain_group((nvm_queue_t*)sq->pair, sq); if (spin_giveup(sq, sp)) break; }
        }
    }
#ifdef BAM_PROFILE
    if (lane() == leader) { BAM_PROF_ADD(sq, 11, BAM_PROF_NOW() - pq3); BAM_PROF_ADD(sq, 25, pq3 - pq2); BAM_PROF_ADD(sq, 24, 1); BAM_PROF_ADD(sq, 12, p_trips); }
#endif
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
    /* What the controller wrote before posting the completion is in memory: staged payload in host memory, which
     * copy_pages reads at system scope, or payload placed in a cache slot, which its readers load past the caches that
     * could remember the slot's last tenant (bam::ld_payload).  No cache has to be invalidated for either. */
    fence_meta();
    return (w & (BAM_CID_DONE | BAM_CID_ERR)) == BAM_CID_DONE;
}

} // namespace bam

/* ---- per-thread entry points with the reference's names ---- */

/*
 * The reference's threads each take a command id, build an entry around it, enqueue it, poll for its completion and hand
 * the id back (get_cid, sq_enqueue, cq_poll, cq_dequeue, put_cid; include/page_cache.h:2009-2054 strings them together),
 * and a thread that waits in one of these steps does not keep its neighbours from going through theirs.  The lanes of a
 * wave move together: a wave whose lanes are on several queues, holding slots of one queue (reserved, their entries not
 * yet written) while it waits for slots or for a covering doorbell on another, can wait for a wave that does the same the
 * other way round; with seven queues, where consecutive waves meet the queues in rotated orders, that happens within
 * milliseconds.  So a wave never holds anything of one queue while it waits on another: sq_enqueue does the whole of a
 * command's life for one queue's lanes at a time (slot, entry, doorbell, completion, slot handed back), in rounds of half
 * a queue where the lanes are more than that, and the calls around it have nothing left to wait for.  For the caller the
 * sequence is the reference's: after cq_poll the transfer of the entry it enqueued has happened.  The id get_cid hands
 * out is a token; the id the controller sees is the slot sq_enqueue writes the entry to, which it puts into the entry.
 * Threads that want several commands in flight use access_data_async / poll_async.
 */
inline __device__ uint16_t get_cid(nvm_queue_t* sq)
{
    (void)sq;
    return (uint16_t)bam::lane();
}

/* nothing is held after sq_enqueue */
inline __device__ void put_cid(nvm_queue_t* sq, uint16_t id)
{
    (void)sq; (void)id;
}

/* submits the entry and waits for its completion; returns the SQ slot used, which is the command id the controller saw.
 * Bit 15 of the entry's dword 12 upward and the other fields are the caller's; only the id in dword 0 is replaced. */
inline __device__ uint16_t sq_enqueue(nvm_queue_t* sq, nvm_cmd_t* cmd)
{
    uint32_t id = 0;
    bam::for_each_group((uint64_t)sq, [&](uint64_t q) {
        nvm_queue_t* s = (nvm_queue_t*)q;
        const uint64_t act = bam::active_mask();
        const uint32_t n = bam::popc(act), rank = bam::rank_in(act), step = s->qs >> 1 ? s->qs >> 1 : 1u;
        for (uint32_t base = 0; base < n; base += step)
            if (rank >= base && rank - base < step) {
                const uint32_t ticket = bam::sq_reserve_group(s);
                id = ticket & s->qs_minus_1;
                cmd->dword[0] = (cmd->dword[0] & 0xffffu) | (id << 16);
                bam::sq_submit_group(s, cmd, ticket);
                bam::cq_wait_group((nvm_queue_t*)s->pair, s, id);
                bam::sq_release_group(s, id);
            }
    });
    return (uint16_t)id;
}

/*
 * The completion of the command was waited for in sq_enqueue.  The reference scans the ring here and hands back the
 * entry's position for cq_dequeue; the out-parameters (which the reference dereferences even when NULL,
 * nvm_parallel_queue.h:406-407) are optional and receive the current head.
 */
inline __device__ uint32_t cq_poll(nvm_queue_t* cq, uint16_t search_cid, uint32_t* loc_ = nullptr, uint32_t* cq_head = nullptr)
{
    (void)search_cid;
    uint32_t h = bam::ld_relaxed(&cq->head_lock) >> 1;
    if (loc_) *loc_ = h;
    if (cq_head) *cq_head = h;
    return h & cq->qs_minus_1;
}

/* Completions are consumed by whoever drains the ring; nothing is left to do per entry. */
inline __device__ void cq_dequeue(nvm_queue_t* cq, uint16_t pos, nvm_queue_t* sq, uint32_t loc_ = 0, uint32_t cur_head_ = 0)
{
    (void)cq; (void)pos; (void)sq; (void)loc_; (void)cur_head_;
}

#endif /* __NVM_PARALLEL_QUEUE_H_ */
