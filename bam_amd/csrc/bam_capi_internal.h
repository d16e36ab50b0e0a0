// Shared by the translation units of the C-ABI library (bam_capi.hip, bam_graph.hip, bam_apps.hip): error plumbing, the
// handle types behind the opaque pointers of include/bam_amd.h, and the device helpers the kernels of every unit use.
#ifndef __BAM_CAPI_INTERNAL_H__
#define __BAM_CAPI_INTERNAL_H__
#include "bam_amd.h"

#include <memory>
#include <hip/hip_runtime.h>
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>
#include <algorithm>
#include <cerrno>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "ctrl.h"
#include "event.h"
#include "nvmt.h"
#include "page_cache.h"
#include "bafs_ptr.h"

// ---------------------------------------------------------------------------
// error plumbing
// ---------------------------------------------------------------------------
std::string& bam_err();            /* message of the last failure on the calling thread (defined in bam_capi.hip) */
#define g_err bam_err()

#define BAM_API_BEGIN try {
#define BAM_API_END                                                        \
    return 0;                                                              \
    } catch (const std::exception& e) { g_err = e.what(); return EIO; }    \
      catch (...) { g_err = "unknown error"; return EIO; }

static inline int fail(int code, const char* msg) { g_err = msg; return code; }
static inline int fail(int code, const std::string& msg) { g_err = msg; return code; }

struct bam_target {
    nvmt_t* t = nullptr;
    void* bar = nullptr;
    void* backing = nullptr;
    size_t backing_bytes = 0;
    nvmt_config_t cfg{};
};
struct bam_ctrl { Controller* c; };
struct bam_page_cache { page_cache_t* pc; Controller* ctrl; };      /* ctrl: the first controller of the cache */
struct bam_range { range_t<uint64_t>* r; };
#define BAM_SUM_PARTIALS 4096
struct bam_array {
    array_t<uint64_t>* a;
    BufferPtr partials, progress;       /* progress: the word the computing workgroups of vectoradd, reduction and scan count themselves off in */
    std::shared_ptr<void> graph;        /* what bam_array_set_graph prepared (bam_graph.hip) */
    /* the entry points that read in two launches: what the first launch leaves for the second (grown on demand, kept),
     * and the count of workgroups of the second that have finished (zero between launches) */
    BufferPtr notes, finished;
    size_t notes_bytes = 0;
    uint32_t calls = 0;
    void* notes_for(size_t bytes)
    {
        if (bytes > notes_bytes) { notes = createBuffer(bytes, 0); notes_bytes = bytes; }
        if (!finished) finished = createBuffer(512, 0);      /* [0 .. 64] the count of workgroups done, [96] the call that left work for its second launch */
        return notes.get();
    }
    uint32_t next_call() { if (++calls == 0) calls = 1; return calls; }      /* never 0: the word starts out as that */
};
struct bam_range32 { range_t<uint32_t>* r; };
struct bam_array32 { array_t<uint32_t>* a; BufferPtr partials; };      /* partials: [BAM_SUM_PARTIALS] checksum shards, zero between launches */

// ---------------------------------------------------------------------------
// device helpers
// ---------------------------------------------------------------------------
namespace {

__device__ __forceinline__ uint64_t mix64(uint64_t z)
{
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
__device__ __forceinline__ uint64_t splitmix64(uint64_t seed, uint64_t i) { return mix64(seed + (i + 1) * 0x9E3779B97F4A7C15ull); }

/* sum over the 64 lanes of a wave (all lanes active); result valid in every lane */
__device__ __forceinline__ uint64_t wave_sum(uint64_t v)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += bam::shfl(v, bam::lane() ^ o);
    return v;
}

/*
 * Add the wave's values into the launch's checksum.  A single word would take one atomic per wave of the
 * whole grid, all serialised on one address (about 12 ns each: a million waves cost more than the reads they
 * sum), so the sum is kept in BAM_SUM_PARTIALS shards picked by workgroup and folded by k_fold_partials.
 */
__device__ __forceinline__ void block_accumulate(unsigned long long* partials, uint64_t v)
{
    v = wave_sum(v);
    if (bam::lane() == 0 && v) atomicAdd(&partials[(blockIdx.x * 0x9E3779B1u) >> 20], (unsigned long long)v);
}

/* a page that is not resident as far as one look at its state tells: what the read-ahead asks for (a page that is resident is
 * left alone, which spares its state word two atomics per touch; if it goes before it is read, it is read on demand) */
template <typename T>
__device__ __forceinline__ bool page_absent(const bam::range_view<T>& view, const uint64_t page)
{
    return (bam::ld_relaxed(&view.pages[page].state) & VALID) == 0;
}

/*
 * Read-ahead for kernels in which consecutive threads read consecutive elements (one element or two per thread, as in
 * benchmarks/vectoradd, reduction and scan).  Left to themselves such kernels ask the store for one page per wave
 * and trip, and the store path takes about a million such batches per second whatever their size: 1 GiB comes in
 * at 5 GB/s.  Here the wave that reads the first element of a window of W pages (W = a 64th of the cache, at most
 * 64) touches the W pages that lie up to 32 windows further on, one page per lane, taken and dropped again: they come
 * in as one batch of W commands, before the waves that read them are started (workgroups start in order, and the
 * device holds a few thousand waves, that is up to a thousand pages, at a time).  The first windows are touched by
 * their own first waves.  `first` is the index of the wave's first element (wave-uniform), `wave_span` the elements
 * from one wave's first to the next one's (more than 64 where the threads read with a stride).
 */
template <typename T>
__device__ __forceinline__ void touch_ahead(array_d_t<T>* da, const uint64_t first, const uint64_t n_read, const uint64_t wave_span = BAM_WAVE_SIZE,
                                            const uint32_t which = 0)
{
    if (da->n_ranges != 1) return;
    const uint64_t n_elems = n_read < da->n_elems ? n_read : da->n_elems;         /* nothing is touched that the array does not hold */
    const page_cache_d_t& cache = da->d_ranges[0].cache;
    const uint64_t w_pages = cache.n_pages >> 6 > BAM_WAVE_SIZE ? BAM_WAVE_SIZE : cache.n_pages >> 6;
    if (w_pages < 2) return;
    const uint64_t epp = cache.page_size / sizeof(T), w_elems = w_pages * epp;
    /* the wave that does it is the `which`-th of those that begin in the window (`wave_span` elements per wave): a kernel
     * that walks several arrays gives each array's windows to a different wave, and their batches are in flight together */
    if ((first % w_elems) / wave_span != which) return;
    /* how far ahead: beyond what the waves in flight cover (a few thousand waves at one page per four to eight waves), within an
     * eighth of the cache (a kernel may walk several arrays behind one cache at a time) */
    uint64_t dist = (cache.n_pages / 8) / w_pages;
    dist = (dist > 32 ? 32 : dist < 1 ? 1 : dist) * w_elems;
    bam::range_view<T> view;
    view.load(da->d_ranges);
    auto touch = [](uint32_t) { return true; };
    const uint64_t mine = first - first % w_elems + bam::lane() * epp;
    if (first < dist) {
        const uint64_t page = view.page_of(mine < n_elems ? mine : first);
        const bool take = bam::lane() < w_pages && mine < n_elems && page_absent(view, page);
        if (bam::ballot(take)) view.acquire_helped(page, take, false, touch, touch);
    }
    const uint64_t ahead = mine + dist;
    if (first + dist < n_elems) {
        const uint64_t page = view.page_of(ahead < n_elems ? ahead : first);
        const bool take = bam::lane() < w_pages && ahead < n_elems && page_absent(view, page);
        if (bam::ballot(take)) view.acquire_helped(page, take, false, touch, touch);
    }
    view.n_access = view.n_hit = 0;
}

/*
 * Waves that only fetch.  The read-ahead above is done by waves that also compute, so what is on its way from the store is
 * bounded by the windows the running waves happen to begin in (a few hundred pages).  A launch of these kernels therefore
 * starts with a few workgroups whose waves do nothing else: wave k of them walks windows k, k + n_waves, ... of the
 * arrays, takes the pages of a window that are not resident as one batch of commands per array (one page per lane), drops
 * them again and goes on, so that n_waves batches are on their way at any time whatever the computing waves do.  They stay
 * at most `lead_elems` elements ahead of the computing workgroups, which count themselves off in *done as they finish
 * (elems_per_done elements each); a fetch wave that waits longer than the spin limit for that count to move gives up,
 * and the computing waves read on demand as they would without it.  Nothing waits for a fetch wave.
 */
struct fetch_plan {
    unsigned long long* done;       /* NULL: no fetch waves in this launch */
    uint32_t blocks;                /* workgroups at the front of the grid that fetch */
    uint32_t spin_limit;
    uint64_t lead_elems, elems_per_done;
};

template <typename T, int N>
__device__ __forceinline__ void fetch_role(array_d_t<T>* const (&arrays)[N], const uint64_t n_elems, const fetch_plan& fp)
{
    for (int a = 0; a < N; a++) if (arrays[a]->n_ranges != 1) return;
    const page_cache_d_t& cache = arrays[0]->d_ranges[0].cache;
    const uint64_t w_pages = cache.n_pages >> 6 > BAM_WAVE_SIZE ? BAM_WAVE_SIZE : cache.n_pages >> 6;
    if (w_pages < 2) return;
    const uint64_t epp = cache.page_size / sizeof(T), w_elems = w_pages * epp;
    const uint64_t waves_per_block = blockDim.x / BAM_WAVE_SIZE;
    const uint64_t wave = (uint64_t)blockIdx.x * waves_per_block + threadIdx.x / BAM_WAVE_SIZE, n_waves = (uint64_t)fp.blocks * waves_per_block;
    const uint64_t n_windows = (n_elems + w_elems - 1) / w_elems;
    auto touch = [](uint32_t) { return true; };
    for (uint64_t w = wave; w < n_windows; w += n_waves) {
        const uint64_t first = w * w_elems;
        uint32_t spins = 0;
        while (first > __hip_atomic_load(fp.done, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) * fp.elems_per_done + fp.lead_elems) {
            if (++spins >= fp.spin_limit) return;
            __builtin_amdgcn_s_sleep(64);
        }
        const uint64_t mine = first + bam::lane() * epp;
#pragma unroll
        for (int a = 0; a < N; a++) {
            bam::range_view<T> view;
            view.load(arrays[a]->d_ranges);
            view.read_ahead = true;
            const uint64_t n_a = n_elems < arrays[a]->n_elems ? n_elems : arrays[a]->n_elems;
            const uint64_t page = view.page_of(mine < n_a ? mine : 0);
            const bool take = bam::lane() < w_pages && mine < n_a && page_absent(view, page);
            if (bam::ballot(take)) view.acquire_helped(page, take, false, touch, touch);
            view.n_access = view.n_hit = 0;
        }
    }
}

/* fetch waves for a launch whose computing workgroups cover `elems_per_block` consecutive elements each: up to 512 waves
 * (32768 pages on their way; measured on 1 GiB read from the store: 32 waves 18 GB/s, 64 waves 29, 256 waves 34-42, 512 waves
 * 37-44, none 9-11), fewer where a quarter of the cache is less than that; BAM_FETCH_WAVES in the environment overrides the
 * number (0: none); `done` is cleared on the stream */
inline fetch_plan make_fetch_plan(bam_array_t* a, int n_arrays, uint32_t block_size, uint64_t elems_per_block, hipStream_t st)
{
    fetch_plan fp{nullptr, 0, 1u << 18, 0, elems_per_block};
    if (a->a->adt.n_ranges != 1) return fp;
    const page_cache_d_t& cache = a->a->h_ranges[0].cache;
    const uint64_t w_pages = cache.n_pages >> 6 > BAM_WAVE_SIZE ? BAM_WAVE_SIZE : cache.n_pages >> 6;
    if (w_pages < 2) return fp;
    const uint64_t budget_pages = cache.n_pages / 4 / n_arrays;               /* what may lie fetched and unread, per array */
    uint64_t waves = budget_pages / w_pages / 2;                              /* half of it on its way, half waiting to be read */
    uint64_t most = 512;
    if (const char* e = getenv("BAM_FETCH_WAVES")) most = (uint64_t)atoll(e);
    if (waves > most) waves = most;
    if (waves < 1) return fp;
    const uint32_t waves_per_block = block_size / BAM_WAVE_SIZE;
    fp.blocks = (uint32_t)((waves + waves_per_block - 1) / waves_per_block);
    fp.lead_elems = budget_pages * (cache.page_size / sizeof(uint64_t));
    if (!a->progress) a->progress = createBuffer(64, 0);
    fp.done = (unsigned long long*)a->progress.get();
    hip_err_chk(hipMemsetAsync(fp.done, 0, sizeof(unsigned long long), st));
    return fp;
}

inline uint32_t blocks_for(uint64_t n, uint32_t bs) { return (uint32_t)((n + bs - 1) / bs); }

} // namespace
#endif /* __BAM_CAPI_INTERNAL_H__ */
