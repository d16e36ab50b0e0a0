/*
 * gfx950 wavefront-64 primitives used by the device path.
 *
 * Stands where the reference uses CUDA warp intrinsics and inline PTX:
 * lane_id / warp_id / get_smid (include/nvm_util.h:276-295), __activemask,
 * __match_any_sync, __shfl_sync, __any_sync, __syncwarp and __nanosleep call
 * sites throughout include/page_cache.h and include/nvm_parallel_queue.h.
 * Masks are 64 bits wide; gfx950 has no match-any instruction, so grouping
 * lanes by key is a readfirstlane/ballot loop (one trip per distinct key).
 *
 * Memory operations on shared words go through __hip_atomic_* with an explicit
 * scope: agent for state shared between waves, system for anything the NVMe
 * controller (a device, or host threads of the software target) reads or writes.
 */
#ifndef __BAM_WAVE_H__
#define __BAM_WAVE_H__
#include <hip/hip_runtime.h>
#include <stdint.h>

#define BAM_WAVE_SIZE 64

namespace bam {

__device__ __forceinline__ uint32_t lane() { return __lane_id(); }
__device__ __forceinline__ uint64_t ballot(bool p) { return __builtin_amdgcn_ballot_w64(p); }
/*
 * The lanes executing right now, read from the execution mask itself.  A ballot of `true` says the same, but the
 * compiler may move such a ballot out of a branch it sits in (it has no operands that tie it there), and the mask
 * of the enclosing region is not the mask of the branch: inside "for each distinct queue of the wave: if (mine) {...}"
 * that hands the group of one queue the lanes of all of them.
 */
__device__ __forceinline__ uint64_t active_mask()
{
    uint64_t m;
    asm volatile("s_mov_b64 %0, exec" : "=s"(m));
    return m;
}
__device__ __forceinline__ uint32_t popc(uint64_t m) { return (uint32_t)__builtin_popcountll(m); }
__device__ __forceinline__ uint32_t first_lane(uint64_t m) { return (uint32_t)__builtin_ctzll(m); }
__device__ __forceinline__ uint64_t lanes_below(uint32_t l) { return (1ull << l) - 1ull; }
/* position of this lane among the set lanes of m */
__device__ __forceinline__ uint32_t rank_in(uint64_t m) { return popc(m & lanes_below(lane())); }

/* value held by lane `src` (wave-uniform src) */
__device__ __forceinline__ uint32_t bcast(uint32_t v, uint32_t src) { return (uint32_t)__builtin_amdgcn_readlane((int)v, (int)src); }
__device__ __forceinline__ uint64_t bcast(uint64_t v, uint32_t src)
{
    return ((uint64_t)bcast((uint32_t)(v >> 32), src) << 32) | bcast((uint32_t)v, src);
}
/* value held by the first active lane */
__device__ __forceinline__ uint32_t first(uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); }
__device__ __forceinline__ uint64_t first(uint64_t v)
{
    return ((uint64_t)first((uint32_t)(v >> 32)) << 32) | first((uint32_t)v);
}
/* value held by lane `src`, src differing per lane (ds_bpermute) */
__device__ __forceinline__ uint32_t shfl(uint32_t v, uint32_t src) { return (uint32_t)__builtin_amdgcn_ds_bpermute((int)(src << 2), (int)v); }
__device__ __forceinline__ uint64_t shfl(uint64_t v, uint32_t src)
{
    return ((uint64_t)shfl((uint32_t)(v >> 32), src) << 32) | shfl((uint32_t)v, src);
}

/*
 * Group the active lanes by a 64-bit key: returns the mask of active lanes
 * holding the same key as the caller.  One loop trip per distinct key.
 */
__device__ __forceinline__ uint64_t match_any(uint64_t key)
{
    uint64_t mine = 0;
    bool done = false;
    while (!done) {
        uint64_t k = first(key);            /* key of the first lane still looping */
        bool eq = key == k;
        uint64_t grp = ballot(eq);
        if (eq) { mine = grp; done = true; }
    }
    return mine;
}
__device__ __forceinline__ uint64_t match_any(uint64_t key_a, uint64_t key_b)
{
    uint64_t mine = 0;
    bool done = false;
    while (!done) {
        uint64_t a = first(key_a), b = first(key_b);
        bool eq = key_a == a && key_b == b;
        uint64_t grp = ballot(eq);
        if (eq) { mine = grp; done = true; }
    }
    return mine;
}

/*
 * Run `body` once for each distinct key among the active lanes, with exactly the lanes that hold that key active.
 *
 * The loop is driven by a wave-uniform set of lanes still to be served, so every lane makes every trip and the
 * branch around the body is the only place where the lanes part.  (Written the obvious way, "pick the first lane's
 * key; the lanes that match do the work and leave the loop", the work sits right before a lane's loop exit, and the
 * compiler is free to move it behind the loop, where all lanes are back together: group operations in the body,
 * ballots, lane counts, elections of a leader, would then see the lanes of every key at once.)
 */
template <typename F>
__device__ __forceinline__ void for_each_group(const uint64_t key_a, const uint64_t key_b, F&& body)
{
    uint64_t todo = active_mask();
    while (todo) {
        const uint32_t l = first_lane(todo);
        const uint64_t a = bcast(key_a, l), b = bcast(key_b, l);
        const bool mine = key_a == a && key_b == b;
        const uint64_t grp = ballot(mine);
        if (mine) body(a, b);
        todo &= ~grp;
    }
}
template <typename F>
__device__ __forceinline__ void for_each_group(const uint64_t key, F&& body)
{
    for_each_group(key, 0, [&](uint64_t a, uint64_t) { body(a); });
}
/* compute-unit identity across the whole device: XCC, shader engine and CU bits */
__device__ __forceinline__ uint32_t cu_id() { return __smid(); }

/* which of the device's clusters of compute units (XCDs) this wave runs on */
__device__ __forceinline__ uint32_t xcc_id() { return __builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20) & 7u; }

/*
 * A number that differs between the waves resident on the device at one time
 * and is spread evenly: hash of the hardware wave slot (XCC, SE, CU, SIMD,
 * wave).  Used to pick an I/O queue per wave: the CU number alone (what the
 * reference uses, smid % n_qps) has gaps and repeats across the eight XCDs,
 * which would leave most queues idle and a few overrun.
 */
__device__ __forceinline__ uint32_t wave_slot_hash()
{
    const uint32_t hw = __builtin_amdgcn_s_getreg((31 << 11) | (0 << 6) | 4);          /* HW_ID, all 32 bits */
    const uint32_t xcc = __builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20);          /* XCC_ID[3:0] */
    uint32_t h = (hw & 0xffffu) | (xcc << 16);
    h *= 0x9E3779B1u;
    return h ^ (h >> 15);
}

/*
 * Back-off of a wait loop: sleep n * 64 clocks, n doubling from 1 up to 127
 * (about 4 us).  Waits here are for I/O that takes tens of microseconds or
 * more, and thousands of waves may be waiting at once: polling faster than
 * that only takes memory bandwidth away from the waves that are moving data.
 */
__device__ __forceinline__ void backoff(uint32_t& n)
{
    switch (n) {
    case 1: __builtin_amdgcn_s_sleep(1); break;
    case 2: __builtin_amdgcn_s_sleep(2); break;
    case 4: __builtin_amdgcn_s_sleep(4); break;
    case 8: __builtin_amdgcn_s_sleep(8); break;
    case 16: __builtin_amdgcn_s_sleep(16); break;
    case 32: __builtin_amdgcn_s_sleep(32); break;
    case 64: __builtin_amdgcn_s_sleep(64); break;
    default: __builtin_amdgcn_s_sleep(127); break;
    }
    if (n < 128) n <<= 1;
}

/* ---- scoped atomics on plain words ---- */
#define BAM_AGENT  __HIP_MEMORY_SCOPE_AGENT
#define BAM_SYSTEM __HIP_MEMORY_SCOPE_SYSTEM

template <typename T> __device__ __forceinline__ T ld_relaxed(const T* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, BAM_AGENT); }
template <typename T> __device__ __forceinline__ T ld_acquire(const T* p) { return __hip_atomic_load(p, __ATOMIC_ACQUIRE, BAM_AGENT); }
template <typename T> __device__ __forceinline__ T ld_relaxed_sys(const volatile T* p) { return __hip_atomic_load((const T*)p, __ATOMIC_RELAXED, BAM_SYSTEM); }
template <typename T> __device__ __forceinline__ T ld_acquire_sys(const volatile T* p) { return __hip_atomic_load((const T*)p, __ATOMIC_ACQUIRE, BAM_SYSTEM); }
template <typename T> __device__ __forceinline__ void st_relaxed(T* p, T v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, BAM_AGENT); }
template <typename T> __device__ __forceinline__ void st_release(T* p, T v) { __hip_atomic_store(p, v, __ATOMIC_RELEASE, BAM_AGENT); }
template <typename T> __device__ __forceinline__ void st_relaxed_sys(volatile T* p, T v) { __hip_atomic_store((T*)p, v, __ATOMIC_RELAXED, BAM_SYSTEM); }
template <typename T> __device__ __forceinline__ void st_release_sys(volatile T* p, T v) { __hip_atomic_store((T*)p, v, __ATOMIC_RELEASE, BAM_SYSTEM); }

/*
 * Load of page-cache payload.  A cache slot is refilled by other compute units
 * over the life of a kernel, so payload must never be served from this compute
 * unit's vector L1: an agent-scope load goes to L2, which the hardware keeps
 * coherent for device memory.  This is what lets the hit path take its page
 * reference with a relaxed atomic instead of an acquire (an acquire at agent
 * scope invalidates caches on every page visit).
 */
/*
 * Eight 64-bit words of payload, 512 bytes apart (a lane's share of a 4 KiB page that a wave reads side by side), for
 * readers that stream through pages once: loaded past the vector L1 like ld_payload (sc1), and marked as not to be kept
 * (nt), which spares the L2 the allocation and carries a seventh more bytes per second from HBM than the same loads
 * without the mark (7.2 against 6.4 TB/s for a plain reader of 1 GiB).  The compiler has no such load of its own, and
 * does not count what an asm statement leaves in flight: the loads and the wait for them are one statement.
 */
__device__ __forceinline__ void ld_payload_stream8(const uint64_t* p, uint64_t (&x)[8])
{
    asm volatile("global_load_dwordx2 %0, %8, off sc1 nt\n\t"
                 "global_load_dwordx2 %1, %8, off offset:512 sc1 nt\n\t"
                 "global_load_dwordx2 %2, %8, off offset:1024 sc1 nt\n\t"
                 "global_load_dwordx2 %3, %8, off offset:1536 sc1 nt\n\t"
                 "global_load_dwordx2 %4, %8, off offset:2048 sc1 nt\n\t"
                 "global_load_dwordx2 %5, %8, off offset:2560 sc1 nt\n\t"
                 "global_load_dwordx2 %6, %8, off offset:3072 sc1 nt\n\t"
                 "global_load_dwordx2 %7, %8, off offset:3584 sc1 nt\n\t"
                 "s_waitcnt vmcnt(0)"
                 : "=&v"(x[0]), "=&v"(x[1]), "=&v"(x[2]), "=&v"(x[3]), "=&v"(x[4]), "=&v"(x[5]), "=&v"(x[6]), "=&v"(x[7])
                 : "v"(p)
                 : "memory");
}

/* the same for two pages at a time: sixteen loads in flight per lane before the wait */
__device__ __forceinline__ void ld_payload_stream16(const uint64_t* p, const uint64_t* q, uint64_t (&x)[16])
{
    asm volatile("global_load_dwordx2 %0, %16, off sc1 nt\n\t"
                 "global_load_dwordx2 %1, %16, off offset:512 sc1 nt\n\t"
                 "global_load_dwordx2 %2, %16, off offset:1024 sc1 nt\n\t"
                 "global_load_dwordx2 %3, %16, off offset:1536 sc1 nt\n\t"
                 "global_load_dwordx2 %4, %16, off offset:2048 sc1 nt\n\t"
                 "global_load_dwordx2 %5, %16, off offset:2560 sc1 nt\n\t"
                 "global_load_dwordx2 %6, %16, off offset:3072 sc1 nt\n\t"
                 "global_load_dwordx2 %7, %16, off offset:3584 sc1 nt\n\t"
                 "global_load_dwordx2 %8, %17, off sc1 nt\n\t"
                 "global_load_dwordx2 %9, %17, off offset:512 sc1 nt\n\t"
                 "global_load_dwordx2 %10, %17, off offset:1024 sc1 nt\n\t"
                 "global_load_dwordx2 %11, %17, off offset:1536 sc1 nt\n\t"
                 "global_load_dwordx2 %12, %17, off offset:2048 sc1 nt\n\t"
                 "global_load_dwordx2 %13, %17, off offset:2560 sc1 nt\n\t"
                 "global_load_dwordx2 %14, %17, off offset:3072 sc1 nt\n\t"
                 "global_load_dwordx2 %15, %17, off offset:3584 sc1 nt\n\t"
                 "s_waitcnt vmcnt(0)"
                 : "=&v"(x[0]), "=&v"(x[1]), "=&v"(x[2]), "=&v"(x[3]), "=&v"(x[4]), "=&v"(x[5]), "=&v"(x[6]), "=&v"(x[7]),
                   "=&v"(x[8]), "=&v"(x[9]), "=&v"(x[10]), "=&v"(x[11]), "=&v"(x[12]), "=&v"(x[13]), "=&v"(x[14]), "=&v"(x[15])
                 : "v"(p), "v"(q)
                 : "memory");
}

/*
 * N 64-bit words of payload at N addresses of the lane's own (scattered reads, or a lane's elements of one page), all in
 * flight behind one wait: past the vector L1 and marked as not to be kept, like the streaming loads above.  Payload that
 * is read once should not push the page descriptors out of the L2: with the mark the element gather's looks at the
 * descriptors keep hitting, and it runs at 43 instead of 38 thousand million reads a second.  Every address must be
 * readable (a lane with nothing to read passes any address inside the cache).
 */
template <int N>
__device__ __forceinline__ void ld_payload_nt(const uint64_t* const (&p)[N], uint64_t (&x)[N])
{
    static_assert(N == 1 || N == 2 || N == 4 || N == 7 || N == 8, "1, 2, 4, 7 or 8 words");
    if constexpr (N == 1)
        asm volatile("global_load_dwordx2 %0, %1, off sc1 nt\n\ts_waitcnt vmcnt(0)" : "=&v"(x[0]) : "v"(p[0]) : "memory");
    else if constexpr (N == 2)
        asm volatile("global_load_dwordx2 %0, %2, off sc1 nt\n\tglobal_load_dwordx2 %1, %3, off sc1 nt\n\ts_waitcnt vmcnt(0)"
                     : "=&v"(x[0]), "=&v"(x[1]) : "v"(p[0]), "v"(p[1]) : "memory");
    else if constexpr (N == 4)
        asm volatile("global_load_dwordx2 %0, %4, off sc1 nt\n\tglobal_load_dwordx2 %1, %5, off sc1 nt\n\t"
                     "global_load_dwordx2 %2, %6, off sc1 nt\n\tglobal_load_dwordx2 %3, %7, off sc1 nt\n\ts_waitcnt vmcnt(0)"
                     : "=&v"(x[0]), "=&v"(x[1]), "=&v"(x[2]), "=&v"(x[3]) : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]) : "memory");
    else if constexpr (N == 7)
        asm volatile("global_load_dwordx2 %0, %7, off sc1 nt\n\tglobal_load_dwordx2 %1, %8, off sc1 nt\n\t"
                     "global_load_dwordx2 %2, %9, off sc1 nt\n\tglobal_load_dwordx2 %3, %10, off sc1 nt\n\t"
                     "global_load_dwordx2 %4, %11, off sc1 nt\n\tglobal_load_dwordx2 %5, %12, off sc1 nt\n\t"
                     "global_load_dwordx2 %6, %13, off sc1 nt\n\ts_waitcnt vmcnt(0)"
                     : "=&v"(x[0]), "=&v"(x[1]), "=&v"(x[2]), "=&v"(x[3]), "=&v"(x[4]), "=&v"(x[5]), "=&v"(x[6])
                     : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]), "v"(p[6]) : "memory");
    else
        asm volatile("global_load_dwordx2 %0, %8, off sc1 nt\n\tglobal_load_dwordx2 %1, %9, off sc1 nt\n\t"
                     "global_load_dwordx2 %2, %10, off sc1 nt\n\tglobal_load_dwordx2 %3, %11, off sc1 nt\n\t"
                     "global_load_dwordx2 %4, %12, off sc1 nt\n\tglobal_load_dwordx2 %5, %13, off sc1 nt\n\t"
                     "global_load_dwordx2 %6, %14, off sc1 nt\n\tglobal_load_dwordx2 %7, %15, off sc1 nt\n\ts_waitcnt vmcnt(0)"
                     : "=&v"(x[0]), "=&v"(x[1]), "=&v"(x[2]), "=&v"(x[3]), "=&v"(x[4]), "=&v"(x[5]), "=&v"(x[6]), "=&v"(x[7])
                     : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3]), "v"(p[4]), "v"(p[5]), "v"(p[6]), "v"(p[7]) : "memory");
}

/*
 * Sixteen bytes per lane at system scope, for moving payload between a staging page in host memory and a cache slot.
 * The load is never served from a cache that remembers the staging page's last tenant, so nobody has to invalidate
 * caches after a completion; the store goes through to memory, so the wave that moved a page in can publish it after
 * a wait on its own store counter instead of a write-back of the whole L2.  Those two cache-wide operations, once per
 * batch of commands, were what the miss path as a whole queued behind.  The compiler has no 16-byte access with a
 * scope, hence the asm; what an asm load leaves in flight the compiler does not count, so the wait is spelt out and
 * tied to the registers it is for.
 */
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
/* The load and the wait for it are one statement: between two statements the compiler may copy or spill a register it
 * believes written, and one whose load is still on its way would be copied as it was before. */
__device__ __forceinline__ u32x4_t ld16_sys(const void* p)
{
    u32x4_t v;
    asm volatile("global_load_dwordx4 %0, %1, off sc0 sc1\n\ts_waitcnt vmcnt(0)" : "=&v"(v) : "v"(p) : "memory");
    return v;
}
/* four of them in flight behind one wait */
__device__ __forceinline__ void ld16x4_sys(const void* p0, const void* p1, const void* p2, const void* p3, u32x4_t& a, u32x4_t& b, u32x4_t& c, u32x4_t& d)
{
    asm volatile("global_load_dwordx4 %0, %4, off sc0 sc1\n\t"
                 "global_load_dwordx4 %1, %5, off sc0 sc1\n\t"
                 "global_load_dwordx4 %2, %6, off sc0 sc1\n\t"
                 "global_load_dwordx4 %3, %7, off sc0 sc1\n\t"
                 "s_waitcnt vmcnt(0)"
                 : "=&v"(a), "=&v"(b), "=&v"(c), "=&v"(d)
                 : "v"(p0), "v"(p1), "v"(p2), "v"(p3)
                 : "memory");
}
/* The two idle cycles after the store are part of it: a store of more than 8 bytes reads its data registers over the
 * cycles that follow its issue, and a vector instruction that writes one of them in that window changes what is stored.
 * The compiler keeps that distance for stores it emits itself, not for one inside an asm statement. */
__device__ __forceinline__ void st16_sys(void* p, const u32x4_t v)
{
    asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1\n\ts_nop 1" :: "v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void wait_stores() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

template <typename T> __device__ __forceinline__ T ld_payload(const T* p)
{
    if constexpr (sizeof(T) == 8) { uint64_t v = __hip_atomic_load((const uint64_t*)p, __ATOMIC_RELAXED, BAM_AGENT); return *(T*)&v; }
    else if constexpr (sizeof(T) == 4) { uint32_t v = __hip_atomic_load((const uint32_t*)p, __ATOMIC_RELAXED, BAM_AGENT); return *(T*)&v; }
    else if constexpr (sizeof(T) == 2) { uint16_t v = __hip_atomic_load((const uint16_t*)p, __ATOMIC_RELAXED, BAM_AGENT); return *(T*)&v; }
    else if constexpr (sizeof(T) == 1) { uint8_t v = __hip_atomic_load((const uint8_t*)p, __ATOMIC_RELAXED, BAM_AGENT); return *(T*)&v; }
    else if constexpr (sizeof(T) == 16) {
        uint64_t v[2];
        v[0] = __hip_atomic_load((const uint64_t*)p, __ATOMIC_RELAXED, BAM_AGENT);
        v[1] = __hip_atomic_load((const uint64_t*)p + 1, __ATOMIC_RELAXED, BAM_AGENT);
        return *(T*)v;
    } else { __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent"); return *p; }
}

/*
 * Ordering among words that are only ever touched with agent-scope atomics (the bookkeeping of the queues and of
 * the cache: tickets, marks, locks, page states) and stores to uncached host memory (submission entries,
 * doorbells).  Such accesses are performed at the device's point of coherence whatever the caches hold, so a
 * hand-over needs one thing only: the wave's earlier accesses have completed before its later ones are issued.
 * That is a wait on the wave's own memory counters.  A release or acquire at agent scope does the same wait and
 * also writes back or invalidates the caches of the whole compute-unit cluster, which only payload moved with
 * plain loads and stores needs; at several such operations per command, and with the L2 full of other waves'
 * dirty lines, those write-backs were most of the latency of a single command.
 */
__device__ __forceinline__ void fence_meta() { asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory"); }
template <typename T> __device__ __forceinline__ void st_publish(T* p, T v) { fence_meta(); __hip_atomic_store(p, v, __ATOMIC_RELAXED, BAM_AGENT); }

__device__ __forceinline__ void fence_release_sys() { __builtin_amdgcn_fence(__ATOMIC_RELEASE, ""); }
__device__ __forceinline__ void fence_acquire_sys() { __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, ""); }
__device__ __forceinline__ void fence_acquire_agent() { __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent"); }
__device__ __forceinline__ void fence_acq_rel_agent() { __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "agent"); }

} // namespace bam

/* names the reference's kernels use */
__device__ __forceinline__ uint32_t lane_id() { return bam::lane(); }
__device__ __forceinline__ uint32_t get_smid() { return bam::cu_id(); }
__device__ __forceinline__ uint32_t warp_id() { return (threadIdx.x + threadIdx.y * blockDim.x) / BAM_WAVE_SIZE; }

#endif /* __BAM_WAVE_H__ */
