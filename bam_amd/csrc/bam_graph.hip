// Graph kernels of the C-ABI library: BFS (per vertex, over queues of vertices, by edge page), connected components,
// PageRank and SSSP over CSR graphs whose neighbour ids (and weights) are read through the page cache.  Kernel shapes
// follow the reference's benchmark kernels (cited per kernel); lane arithmetic is for 64-wide waves.
#include "bam_capi_internal.h"

namespace {

/* the per-vertex kernels (the group walk below) are held to the registers of this many waves per SIMD: left alone the
 * compiler takes what a workgroup of two waves may have, all 512, and one wave per SIMD is what runs */
#ifndef BAM_GRAPH_WAVES
#define BAM_GRAPH_WAVES 2
#endif
#define BAM_GRAPH_KERNEL_WAVES __attribute__((amdgpu_waves_per_eu(BAM_GRAPH_WAVES)))

// ---- BFS: wave per `coarse` vertices, edges through bam_ptr (benchmarks/bfs/main.cu:658-689) ----
#define MYINFINITY 0xFFFFFFFFu
/*
 * Read-ahead for a wave that walks one vertex's edge list through bam_ptr.  Left to itself the walk meets the
 * pages of the list one after the other and pays one full trip to the store for each; the list of a hub of a
 * power-law graph covers hundreds of pages, and the one wave that has it then decides how long the whole level
 * takes.  Whenever the walk is about to enter pages it has not asked for yet, the lanes touch the next pages of
 * the list (one each, taken and dropped again): those that are not resident are loaded as one batch of commands,
 * and the walk that follows finds them there.  Nothing is held, so a page that is evicted again before the walk
 * gets to it is simply read once more; results do not depend on it.  Arrays of one range only, and the reach
 * scales with the cache (a 64th of its pages, at most one page per lane).
 */
template <typename T>
struct list_read_ahead {
    bam::range_view<T> view;
    uint64_t asked_to = 0, last_page = 0;
    uint32_t reach = 0;
    bool long_list = false;
    __device__ __forceinline__ void init(array_d_t<T>* da)
    {
        if (da->n_ranges != 1) return;
        view.load(da->d_ranges);
        /* what is touched ahead may be placed directly up to the higher of the cache's two bounds: measured on the per-vertex
         * BFS (RMAT-24) 4.55 GTEPS with at most 1024 directly placed commands in flight, 4.7 with 4096 to 8192, 4.46 with 16384 */
        view.read_ahead = true;
        const uint64_t r = da->d_ranges[0].cache.n_pages >> 6;
        reach = r > BAM_WAVE_SIZE ? BAM_WAVE_SIZE : (uint32_t)r;
    }
    /* every lane's elements [es, ee) (empty for lanes without any) are about to be read: touch the first and the last page
     * of each run, so that what is not resident comes in as one batch or two, not one trip to the store per run */
    __device__ __forceinline__ void group(const uint64_t es, const uint64_t ee)
    {
        if (reach < 2) return;
        const bool want = ee > es;
        if (!bam::ballot(want)) return;
        auto touch = [](uint32_t) { return true; };
        const uint64_t pf = want ? view.page_of(es) : 0, pl = want ? view.page_of(ee - 1) : 0;
        /* all lanes go in: those without a page of their own help move what the others load */
        const bool take_f = want && page_absent(view, pf), take_l = want && pl != pf && page_absent(view, pl);
        /* the last pages go along with the first ones as far as there are lanes without a first page to ask for (the k-th such
         * lane takes the last page of the k-th lane that has one): one batch of commands instead of two, of which the second
         * would be small (few lists cross a page boundary) */
        const uint64_t need_l = bam::ballot(take_l), idle = ~bam::ballot(take_f);
        const uint32_t k = bam::popc(idle & bam::lanes_below(bam::lane()));
        const bool adopt = !take_f && k < bam::popc(need_l);
        uint64_t m = need_l;
        if (adopt) for (uint32_t i = 0; i < k; i++) m &= m - 1;
        const uint64_t adopted = bam::shfl(pl, adopt ? bam::first_lane(m) : 0u);
        const bool take_1 = take_f || adopt;
        if (bam::ballot(take_1)) view.template acquire_helped<true>(take_f ? pf : adopted, take_1, false, touch, touch);
        /* last pages nobody had a lane for */
        const bool take_2 = take_l && bam::popc(need_l & bam::lanes_below(bam::lane())) >= bam::popc(idle);
        if (bam::ballot(take_2)) view.template acquire_helped<true>(pl, take_2, false, touch, touch);
        view.n_access = view.n_hit = 0;
    }
    /*
     * The lists of the items [first, last) lie in the array in the order of the items (consecutive vertices, or a sorted
     * queue of them): touch every page that holds
     * entries of a list that is about to be walked (item(v, v) says which; lists that go to the queue of long ones are
     * left out), `reach` pages at a time with one page per lane, so that what is not resident comes in as few, large
     * batches of commands.  The store path moves several times more pages per second in batches of sixteen than in
     * batches of two or three, which is what touching the lists of 64 vertices at a time gives on a graph with a few
     * dozen edges per vertex.  False if the span is too wide for that (the caller then touches list by list).
     */
    template <typename Item>
    __device__ __forceinline__ bool span(const uint64_t* vertexList, const uint64_t first, const uint64_t last, const uint64_t heavy_from, Item item,
                                         bool& nothing)
    {
        nothing = false;
        if (reach < 2) return false;
        uint64_t v_first = 0, v_last = 0;
        item(first, v_first); item(last - 1, v_last);
        const uint64_t e0 = vertexList[v_first], e1 = vertexList[v_last + 1];
        if (e1 <= e0) { nothing = true; return true; }
        const uint64_t p0 = view.page_of(e0), p1 = view.page_of(e1 - 1);
        if (p1 - p0 >= 4ull * reach) return false;
        auto touch = [](uint32_t) { return true; };
        const uint32_t lane = bam::lane();
        uint64_t seen = 0;
        for (uint64_t c = p0; c <= p1; c += reach) {
            uint64_t m = 0;
            for (uint64_t b = first; b < last; b += BAM_WAVE_SIZE) {
                uint64_t v = 0;
                if (b + lane < last && item(b + lane, v)) {
                    const uint64_t es = vertexList[v], ee = vertexList[v + 1];
                    if (ee > es && ee - es < heavy_from) {
                        const uint64_t pf = view.page_of(es), pl = view.page_of(ee - 1);
                        const uint64_t f = pf > c ? pf - c : 0, l = pl < c + reach - 1 ? pl - c : reach - 1;
                        if (pl >= c && f <= l) m |= (~0ull >> (63 - l)) & (~0ull << f);
                    }
                }
            }
#pragma unroll
            for (uint32_t o = BAM_WAVE_SIZE / 2; o; o >>= 1) m |= bam::shfl(m, lane ^ o);
            const bool take = ((m >> lane) & 1) != 0 && page_absent(view, c + lane);
            if (bam::ballot(take)) view.template acquire_helped<true>(c + lane, take, false, touch, touch);
            seen |= m;
        }
        view.n_access = view.n_hit = 0;
        nothing = seen == 0;            /* no list to walk in [first, last): the caller need not look again */
        return true;
    }
    /* wave-uniform: the list is elements [start, end); its first `asked` pages have been touched already */
    __device__ __forceinline__ void begin(const uint64_t start, const uint64_t end, const uint32_t asked = 0)
    {
        long_list = false;
        if (reach < 2 || end <= start) return;
        last_page = view.page_of(end - 1);
        long_list = last_page > view.page_of(start);
        asked_to = asked ? view.page_of(start) + asked : 0;
    }
    /* lane l brings page (l mod 16) of a run of elements [start, end) of its own (four runs per wave, `want` says whether
     * the lane's run is to be read at all): one batch of commands for what is not resident of the first sixteen pages of
     * each.  False if the cache is too small for a wave to ask for that much at a time. */
    __device__ __forceinline__ bool quads(const uint64_t start, const uint64_t end, const bool want)
    {
        if (reach < BAM_WAVE_SIZE) return false;
        auto touch = [](uint32_t) { return true; };
        const uint64_t page = want ? view.page_of(start) + (bam::lane() & 15u) : 0;
        const bool take = want && end > start && page <= view.page_of(end - 1) && page_absent(view, page);
        if (bam::ballot(take)) view.template acquire_helped<true>(page, take, false, touch, touch);
        view.n_access = view.n_hit = 0;
        return true;
    }
    /* wave-uniform: the walk is about to read from element `at` on */
    __device__ __forceinline__ void step(const uint64_t at)
    {
        if (!long_list) return;
        const uint64_t pg = view.page_of(at);
        if (pg < asked_to) return;
        const uint64_t p = pg + bam::lane();
        auto touch = [](uint32_t) { return true; };
        const bool take = bam::lane() < reach && p <= last_page && page_absent(view, p);
        if (bam::ballot(take)) view.template acquire_helped<true>(p, take, false, touch, touch);
        asked_to = pg + reach;
        view.n_access = view.n_hit = 0;         /* not accesses of the kernel's own: kept out of the counters */
    }
};

/*
 * Every lane brings a run of elements [es, ee) (possibly empty, each shorter than 2^20) and the vertex `src` the run
 * belongs to; the wave visits all elements of all runs, 64 per step, consecutive lanes taking consecutive elements
 * across the ends of the runs.  With lists of a dozen edges, walking one list per step leaves most lanes idle and
 * pays the whole chain of dependent loads (offsets, payload, label) once per vertex; packed, it is paid once per 64
 * edges.  A lane finds the run its element belongs to by binary search in the running sums of the run lengths
 * (six shuffles).  `read(i)` fetches element i, `visit(src, value, i)` consumes it.
 */
template <typename Read, typename Visit>
__device__ __forceinline__ void walk_packed(const uint64_t es, const uint64_t ee, const uint64_t src, Read read, Visit visit)
{
    const uint32_t lane = bam::lane();
    const uint32_t len = (uint32_t)(ee - es);
    uint32_t incl = len;
#pragma unroll
    for (uint32_t o = 1; o < BAM_WAVE_SIZE; o <<= 1) {
        const uint32_t u = bam::shfl(incl, lane >= o ? lane - o : lane);
        if (lane >= o) incl += u;
    }
    const uint32_t total = bam::shfl(incl, BAM_WAVE_SIZE - 1), excl = incl - len;
    for (uint32_t base = 0; base < total; base += BAM_WAVE_SIZE) {
        const uint32_t k = base + lane;
        uint32_t j = 0;                                          /* number of runs that end at or before k */
#pragma unroll
        for (uint32_t step = BAM_WAVE_SIZE / 2; step; step >>= 1)
            if (bam::shfl(incl, j + step - 1) <= k) j += step;
        j &= BAM_WAVE_SIZE - 1;                                  /* lanes past the end: any valid lane, they do not visit */
        const uint64_t i = bam::shfl(es, j) + (k - bam::shfl(excl, j));
        const uint64_t s = bam::shfl(src, j);
        if (k < total) visit(s, read(i), i);
    }
}

/*
 * The traversal of the reference's coarsened per-vertex kernels (bfs/main.cu:658-689, cc/main.cu:123-144): the
 * vertices are handed out in groups of `coarse`, and the edge list of every active vertex is read through bam_ptr.
 * What differs, for the store's and the memory system's sake:
 *  - the launch has as many waves as the device holds at a time, and a wave takes the next piece of work when it is
 *    done with its last one (one atomic each).  One group per wave of a large grid leaves most of the device idle
 *    here: groups differ in length by orders of magnitude, and workgroups are started in order;
 *  - the flags and offsets of 64 vertices are read at a time, one vertex per lane, and the lists of those vertices
 *    are walked packed (walk_packed): 64 edges per step whichever vertices they belong to;
 *  - before the walk the pages that hold the lists of the group's active vertices are touched (list_read_ahead::span),
 *    so that what is not resident comes in as one batch of commands, not one trip to the store per vertex;
 *  - lists of BAM_HEAVY_EDGES entries and more are walked in pieces, by a wave each (below).
 */
/*
 * A list of BAM_HEAVY_EDGES entries or more is not walked with its group: it is cut into pieces of BAM_PIECE_EDGES
 * entries, each walked by a wave of its own.  The hubs of a power-law graph have lists of hundreds of pages; walked
 * by one wave, a single hub takes longer than all other vertices of its level together.  Which lists are long does
 * not change from sweep to sweep, so the pieces are listed once per call (k_heavy_pieces) and every sweep hands them
 * out before the groups, longest work first: a piece whose vertex is not active costs its wave one look at the flag.
 */
#define BAM_HEAVY_EDGES 1024u
/* entries per piece: 16 pages of 4 KiB, which the wave that walks the piece asks for as one batch of commands.  Pieces
 * of the threshold's size reach the store as batches of two or three commands, and the store path moves far fewer
 * pages per second in such batches than in batches of sixteen */
#define BAM_PIECE_EDGES 8192u
#define BAM_PIECE_BUNDLE 4u             /* pieces handed to a wave at a time: sixteen lanes look after the sixteen pages of each */
static_assert(BAM_PIECE_BUNDLE * 16u == BAM_WAVE_SIZE && BAM_PIECE_EDGES * 8u == 16u * 4096u, "a bundle's pages are shared out one per lane");
struct heavy_piece_t { uint64_t v, first, last; };      /* entries [first, last) of the list of vertex v */

__global__ void k_heavy_pieces(const uint64_t* vertexList, const uint64_t vertex_count, heavy_piece_t* pieces, unsigned long long* count)
{
    const uint64_t v = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (v >= vertex_count) return;
    const uint64_t start = vertexList[v], end = vertexList[v + 1];
    if (end - start < BAM_HEAVY_EDGES) return;
    const uint64_t n = (end - start + BAM_PIECE_EDGES - 1) / BAM_PIECE_EDGES;
    const unsigned long long at = atomicAdd(count, (unsigned long long)n);
    for (uint64_t k = 0; k < n; k++) {
        const uint64_t f = start + k * BAM_PIECE_EDGES;
        pieces[at + k] = heavy_piece_t{v, f, f + BAM_PIECE_EDGES < end ? f + BAM_PIECE_EDGES : end};
    }
}

/*
 * Reads with the page referenced for the one read only.  bam_ptr keeps every lane's page referenced until the lane
 * moves on: fine where the lanes of a wave read side by side, but 64 lanes that walk lists scattered over the edge
 * array would pin up to 64 pages per wave, and a cache with fewer free slots than that stops for good (lanes that
 * have their page wait for those that cannot get one).  Lanes on the same page still share one pair of atomics.
 */
template <typename T>
struct touch_reader {
    array_d_t<T>* da = nullptr;
    bam::range_view<T> view;
    bool one_range = false, fast = false;
    __device__ __forceinline__ void init(array_d_t<T>* a)
    {
        da = a;
        one_range = a->n_ranges == 1;
        if (one_range) { view.load(a->d_ranges); fast = a->d_ranges[0].cache.fast_reads != 0; }
    }
    __device__ __forceinline__ T read(const uint64_t i)
    {
        if (!one_range) return da->seq_read(i);
        T ret = T();                                    /* stays T() if the wait is given up */
        const uint64_t byte = view.byte_of(i);
        /* resident pages without a reference at all, as array_d_t::seq_read does */
        if (fast && bam_read_unpinned(view.pages + (byte >> view.page_size_log), view.base_addr, view.page_size_log, byte & (view.page_size - 1), ret)) {
            view.account(true);
            return ret;
        }
        auto use = [&](uint32_t slot) { ret = bam::ld_payload((T*)(view.slot_addr(slot) + (byte & (view.page_size - 1)))); return true; };
        view.template acquire<true>(byte >> view.page_size_log, false, use, use);
        return ret;
    }
    __device__ __forceinline__ void fini() { if (one_range) view.flush_stats(); }
};

/*
 * One sweep: the pieces of the long lists whose vertex is active(v), then `n_items` work items in groups of `coarse`,
 * each of which names a vertex and says whether it is to be walked: item(i, v).  visit(src, value, i) for every entry.
 * HOLD: the items are the vertices themselves (item i is vertex i, lists side by side), read through bam_ptr;
 * otherwise the items' lists lie anywhere, and they are read page by page without holding any.
 */
#define BAM_WORK_RUN 8
template <bool HOLD, typename Item, typename Active, typename Visit>
__device__ __forceinline__ void walk_item_groups(array_d_t<uint64_t>* da, const uint64_t* vertexList, const uint64_t n_items, const uint64_t coarse,
                                                 const heavy_piece_t* heavy, const uint64_t n_heavy, unsigned long long* next_work,
                                                 const bool backwards, Item item, Active active, Visit visit,
                                                 list_read_ahead<uint32_t>* with = nullptr, const bool in_order = HOLD)
{
    const uint64_t laneIdx = threadIdx.x % BAM_WAVE_SIZE;
    const uint64_t n_groups = (n_items + coarse - 1) / coarse;
    const uint64_t n_bundles = (n_heavy + BAM_PIECE_BUNDLE - 1) / BAM_PIECE_BUNDLE;
    bam_ptr<uint64_t> ptr(da);
    touch_reader<uint64_t> touch;
    if (!HOLD) touch.init(da);
    list_read_ahead<uint64_t> ahead;
    bool ready = false;
    /* A wave whose last group had nothing to walk takes BAM_WORK_RUN turns at the counter in one: every wave of the device
     * adds to the same word, which takes the device about 12 ns a time, and a sweep with nothing to walk is made of little
     * else (0.6 ms for 2^24 vertices one group per turn, 0.35 ms this way, 0.2 ms with runs of four for everybody).  A wave that
     * found work goes back to single turns: on a dense level, runs of neighbouring groups per wave cost 7 % (fewer waves
     * share a page at a time). */
    bool idle = false;
    for (unsigned long long w0 = 0, left = 0;;) {
        if (!left) {
            left = idle ? BAM_WORK_RUN : 1;
            if (laneIdx == 0) w0 = atomicAdd(next_work, left);
            w0 = bam::bcast((uint64_t)w0, 0);
        }
        const unsigned long long w = w0++;
        left--;
        /* every other sweep runs from the far end of both lists of work: what the last sweep left in the cache is what
         * this one asks for first */
        const uint64_t wb = backwards ? n_bundles - 1 - w : w;
        if (w < n_bundles) {
            /* pieces of long lists, BAM_PIECE_BUNDLE per turn at the counter (every turn costs one atomic on one word, and on
             * a sweep with little to do those atomics are what the sweep takes): all lanes side by side through bam_ptr,
             * read ahead over the piece */
            /* what the active pieces of the bundle need comes in as one batch: a piece by itself asks for six pages on
             * average on a power-law graph, where most long lists are just over the threshold */
            bool asked = false;
            {
                const uint64_t k = wb * BAM_PIECE_BUNDLE + laneIdx / 16;
                heavy_piece_t mine = {0, 0, 0};
                bool want = false;
                if (k < n_heavy) { mine = heavy[k]; want = active(mine.v); }
                if (bam::ballot(want)) {
                    if (!ready) { ahead.init(da); ready = true; }
                    asked = ahead.quads(mine.first, mine.last, want);
                    if (with) with->quads(mine.first, mine.last, want);
                }
            }
            for (uint64_t k = wb * BAM_PIECE_BUNDLE; k < (wb + 1) * BAM_PIECE_BUNDLE && k < n_heavy; k++) {
                const heavy_piece_t pc = heavy[k];
                if (!active(pc.v)) continue;
                if (!ready) { ahead.init(da); ready = true; }
                ahead.begin(pc.first, pc.last, asked ? 16u : 0u);
                if (with) with->begin(pc.first, pc.last, asked ? 16u : 0u);
                for (uint64_t i = (pc.first & 0xFFFFFFFFFFFFFFF0ull) + laneIdx; i < pc.last; i += BAM_WAVE_SIZE) {
                    ahead.step(i - laneIdx > pc.first ? i - laneIdx : pc.first);
                    if (with) with->step(i - laneIdx > pc.first ? i - laneIdx : pc.first);
                    if (i >= pc.first) visit(pc.v, ptr.read(i), i);
                }
            }
            continue;
        }
        if (w - n_bundles >= n_groups) break;
        const uint64_t g = backwards ? n_groups - 1 - (w - n_bundles) : w - n_bundles;
        const uint64_t first = g * coarse;
        bool touched = false, nothing = false;
        if (in_order) {
            if (!ready) { ahead.init(da); ready = true; }
            touched = ahead.span(vertexList, first, first + coarse < n_items ? first + coarse : n_items, BAM_HEAVY_EDGES, item, nothing);
            if (with && touched && !nothing) { bool none; with->span(vertexList, first, first + coarse < n_items ? first + coarse : n_items, BAM_HEAVY_EDGES, item, none); }
            idle = nothing;
            if (nothing) continue;
        }
        for (uint64_t b = 0; b < coarse; b += BAM_WAVE_SIZE) {
            const uint64_t at_item = first + b + laneIdx;
            uint64_t mine = 0;
            const bool act = b + laneIdx < coarse && at_item < n_items && item(at_item, mine);
            if (!bam::ballot(act)) continue;
            if (!ready) { ahead.init(da); ready = true; }
            uint64_t es = 0, ee = 0;
            if (act) { es = vertexList[mine]; ee = vertexList[mine + 1]; }
            if (ee - es >= BAM_HEAVY_EDGES) ee = es;            /* walked in pieces */
            if (!touched) {
                /* a group whose lists cover too many pages for one look: the same for the 64 vertices at hand */
                bool block_touched = false;
                if (in_order) {
                    const uint64_t last = first + coarse < n_items ? first + coarse : n_items;
                    bool none;
                    block_touched = ahead.span(vertexList, first + b, first + b + BAM_WAVE_SIZE < last ? first + b + BAM_WAVE_SIZE : last, BAM_HEAVY_EDGES, item, none);
                    if (with && block_touched) with->span(vertexList, first + b, first + b + BAM_WAVE_SIZE < last ? first + b + BAM_WAVE_SIZE : last, BAM_HEAVY_EDGES, item, none);
                }
                if (!block_touched) { ahead.group(es, ee); if (with) with->group(es, ee); }
            }
            walk_packed(es, ee, mine, [&](uint64_t i) { if constexpr (HOLD) return ptr.read(i); else return touch.read(i); }, visit);
        }
    }
    if (!HOLD) touch.fini();
}

/* the items are the vertices themselves, walked where active(v) */
template <typename Active, typename Visit>
__device__ __forceinline__ void walk_vertex_groups(array_d_t<uint64_t>* da, const uint64_t* vertexList, const uint64_t vertex_count, const uint64_t coarse,
                                                   const heavy_piece_t* heavy, const uint64_t n_heavy, unsigned long long* next_work, const bool backwards,
                                                   Active active, Visit visit, list_read_ahead<uint32_t>* with = nullptr)
{
    walk_item_groups<true>(da, vertexList, vertex_count, coarse, heavy, n_heavy, next_work, backwards,
                           [&](uint64_t i, uint64_t& v) { v = i; return active(i); }, active, visit, with);
}

__global__ __launch_bounds__(128) BAM_GRAPH_KERNEL_WAVES void k_bfs_coalesce_coarse_ptr_pc(array_d_t<uint64_t>* da, uint32_t* label, const uint32_t level, const uint64_t vertex_count,
                                                                   const uint64_t* vertexList, uint64_t* changed, uint64_t coarse,
                                                                   const heavy_piece_t* heavy, uint64_t n_heavy, unsigned long long* next_work)
{
    bool any = false;
    walk_vertex_groups(da, vertexList, vertex_count, coarse, heavy, n_heavy, next_work, (level & 1u) != 0,
                       [&](uint64_t v) { return label[v] == level; },
                       [&](uint64_t, uint64_t next, uint64_t) { if (label[next] == MYINFINITY) { label[next] = level + 1; any = true; } });
    if (any) *changed = 1;
}

// ---- the reference's other ways of sharing the vertices out (benchmarks/bfs/main.cu:733-760 hash, :810-850 hash + coarse,
// :852-905 sixteen lanes per vertex, :961-1000 chunks; benchmarks/cc has the same set) ----
/*
 * The same relaxation as the kernels above, the vertices shared out as these variants of the reference do, with none of
 * the machinery around the group walk (no touching ahead, no pieces of long lists): a unit of lanes walks a vertex's
 * list through bam_ptr, and which vertex unit u takes is
 *   SHAPE 0  unit = wave:       v = u / nep + (u % nep) * stride, nep = (V + stride) / stride          (hash)
 *   SHAPE 1  unit = wave:       the `coarse` vertices c * coarse + j of c = u / nep + (u % nep) * stride,
 *                               nep = (V + stride * coarse) / (stride * coarse)                          (hash, coarse)
 *   SHAPE 2  unit = 16 lanes:   v as for SHAPE 0 (four vertices per wave side by side; the reference's page-cache
 *                               version of this kernel has an empty loop body, its in-memory twin has the relaxation)
 *   SHAPE 3  unit = wave:       the eight vertices 8 u .. 8 u + 7 one after the other                   (chunk)
 * The units of a launch are walked by a bounded number of waves (`n_units` are shared out round robin), so that the
 * pages the waves hold fit the cache.
 */
#define BAM_SHAPE_CHUNK 8
template <int SHAPE, typename Active, typename Visit>
__device__ __forceinline__ void walk_shaped(array_d_t<uint64_t>* da, const uint64_t* vertexList, const uint64_t n, const uint64_t coarse, const uint64_t stride,
                                            const uint64_t n_units, Active active, Visit visit)
{
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x, n_threads = (uint64_t)gridDim.x * blockDim.x;
    bam_ptr<uint64_t> ptr(da);
    const uint64_t width = SHAPE == 2 ? 16 : BAM_WAVE_SIZE;
    const uint64_t l = tid % width;
    auto walk = [&](const uint64_t v) {
        const uint64_t start = vertexList[v], end = vertexList[v + 1];
        for (uint64_t i = (start & 0xFFFFFFFFFFFFFFF0ull) + l; i < end; i += width)
            if (i >= start) visit(v, ptr.read(i), i);
    };
    for (uint64_t u = tid / width; u < n_units; u += n_threads / width) {
        if (SHAPE == 3) {
            for (uint64_t v = u * BAM_SHAPE_CHUNK; v < (u + 1) * BAM_SHAPE_CHUNK && v < n; v++)
                if (active(v)) walk(v);
        } else if (SHAPE == 1) {
            const uint64_t nep = (n + stride * coarse) / (stride * coarse);
            const uint64_t c = u / nep + (u % nep) * stride;
            for (uint64_t j = 0; j < coarse; j++) {
                const uint64_t v = c * coarse + j;
                if (v < n && active(v)) walk(v);
            }
        } else {
            const uint64_t nep = (n + stride) / stride;
            const uint64_t v = u / nep + (u % nep) * stride;
            if (v < n && active(v)) walk(v);
        }
    }
}

template <int SHAPE>
__global__ __launch_bounds__(128) void k_bfs_shaped(array_d_t<uint64_t>* da, uint32_t* label, const uint32_t level, const uint64_t vertex_count, const uint64_t* vertexList,
                                                    uint64_t* changed, uint64_t coarse, uint64_t stride, uint64_t n_units)
{
    bool any = false;
    walk_shaped<SHAPE>(da, vertexList, vertex_count, coarse, stride, n_units,
                       [&](uint64_t v) { return label[v] == level; },
                       [&](uint64_t, uint64_t next, uint64_t) { if (label[next] == MYINFINITY) { label[next] = level + 1; any = true; } });
    if (any) *changed = 1;
}

// ---- BFS over a queue of the level's vertices (benchmarks/bfs/main.cu:409-451 kernel_frontier_coalesce_ptr_pc) ----
/* a vertex found for the first time (the exchange on its label decides who found it) goes to the next level's queue;
 * the lanes of a wave that found one at the same step take their places in it with one atomic */
__device__ __forceinline__ void bfs_frontier_visit(uint32_t* label, const uint32_t level, uint32_t* next_frontier, unsigned long long* next_size, const uint64_t next)
{
    if (label[next] != MYINFINITY) return;
    if (atomicExch(label + next, level + 1) != MYINFINITY) return;
    const uint64_t mask = bam::active_mask();
    const uint32_t leader = bam::first_lane(mask);
    unsigned long long pos = 0;
    if (bam::lane() == leader) pos = atomicAdd(next_size, (unsigned long long)bam::popc(mask));
    pos = bam::bcast((uint64_t)pos, leader);
    next_frontier[pos + bam::rank_in(mask)] = (uint32_t)next;
}

__global__ __launch_bounds__(128) BAM_GRAPH_KERNEL_WAVES void k_bfs_frontier_coalesce_ptr_pc(array_d_t<uint64_t>* da, uint32_t* label, const uint32_t level, const uint64_t* vertexList,
                                                                     const uint32_t* curr_frontier, const uint64_t curr_size, uint32_t* next_frontier,
                                                                     unsigned long long* next_size, uint64_t group,
                                                                     const heavy_piece_t* heavy, uint64_t n_heavy, unsigned long long* next_work, bool sorted)
{
    walk_item_groups<false>(da, vertexList, curr_size, group, heavy, n_heavy, next_work, false,
                            [&](uint64_t i, uint64_t& v) { v = curr_frontier[i]; return true; },
                            [&](uint64_t v) { return label[v] == level; },
                            [&](uint64_t, uint64_t next, uint64_t) { bfs_frontier_visit(label, level, next_frontier, next_size, next); },
                            nullptr, sorted);
}

/*
 * The queue of a level put in the order of its vertices.  A vertex enters a queue once, so the entries are distinct, and
 * sorting distinct numbers below V is marking them in a map of V bits and reading the map front to back: four small
 * kernels (mark; count the marks of every 4096 vertices, a wave each; running sums of those counts by one workgroup;
 * write the vertices out, a wave per 4096 again, and clear the map), a few microseconds a level for 2^24 vertices,
 * and no library.
 */
__global__ void k_queue_mark(const uint32_t* __restrict__ queue, const uint64_t n, unsigned long long* bits)
{
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) { const uint32_t v = queue[i]; atomicOr(&bits[v >> 6], 1ull << (v & 63u)); }
}
__global__ void k_bits_count(const unsigned long long* __restrict__ bits, const uint64_t n_words, uint32_t* totals)
{
    const uint64_t wave = ((uint64_t)blockIdx.x * blockDim.x + threadIdx.x) / BAM_WAVE_SIZE, at = wave * BAM_WAVE_SIZE + bam::lane();
    const uint64_t c = wave_sum((uint64_t)bam::popc(at < n_words ? bits[at] : 0ull));
    if (bam::lane() == 0 && wave * BAM_WAVE_SIZE < n_words) totals[wave] = (uint32_t)c;
}
/* totals[k] <- totals[0] + ... + totals[k - 1]; one workgroup of 1024 threads, a run of entries per thread */
__global__ void k_totals_scan(uint32_t* totals, const uint64_t n)
{
    __shared__ uint32_t sums[1024];
    const uint64_t per = (n + blockDim.x - 1) / blockDim.x, a = threadIdx.x * per, b = a + per < n ? a + per : n;
    uint32_t mine = 0;
    for (uint64_t k = a; k < b; k++) mine += totals[k];
    sums[threadIdx.x] = mine;
    __syncthreads();
    for (uint32_t o = 1; o < blockDim.x; o <<= 1) {
        const uint32_t add = threadIdx.x >= o ? sums[threadIdx.x - o] : 0;
        __syncthreads();
        sums[threadIdx.x] += add;
        __syncthreads();
    }
    uint32_t run = sums[threadIdx.x] - mine;
    for (uint64_t k = a; k < b; k++) { const uint32_t t = totals[k]; totals[k] = run; run += t; }
}
__global__ void k_bits_emit(unsigned long long* bits, const uint64_t n_words, const uint32_t* __restrict__ first_of_wave, uint32_t* out)
{
    const uint64_t wave = ((uint64_t)blockIdx.x * blockDim.x + threadIdx.x) / BAM_WAVE_SIZE, at = wave * BAM_WAVE_SIZE + bam::lane();
    if (wave * BAM_WAVE_SIZE >= n_words) return;
    unsigned long long w = at < n_words ? bits[at] : 0ull;
    if (w) bits[at] = 0;
    const uint32_t c = bam::popc(w);
    uint32_t incl = c;
#pragma unroll
    for (uint32_t o = 1; o < BAM_WAVE_SIZE; o <<= 1) {
        const uint32_t u = bam::shfl(incl, bam::lane() >= o ? bam::lane() - o : bam::lane());
        if (bam::lane() >= o) incl += u;
    }
    uint32_t pos = first_of_wave[wave] + incl - c;
    for (; w; w &= w - 1) out[pos++] = (uint32_t)(at * 64 + (uint64_t)__builtin_ctzll(w));
}

// ---- CC: min-label propagation (benchmarks/cc/main.cu:123-144, 595-617) ----
__device__ __forceinline__ void cc_compute(uint64_t cid, unsigned long long* comp, uint64_t next, bool* next_visit, bool* changed)
{
    const unsigned long long comp_src = comp[cid], comp_next = comp[next];
    if (comp_next == comp_src) return;
    uint64_t next_target;
    unsigned long long comp_target;
    if (comp_src < comp_next) { next_target = next; comp_target = comp_src; }
    else { next_target = cid; comp_target = comp_next; }
    atomicMin(&comp[next_target], comp_target);
    next_visit[next_target] = true;
    *changed = true;
}

__global__ __launch_bounds__(128) BAM_GRAPH_KERNEL_WAVES void k_cc_coalesce_coarse_ptr_pc(array_d_t<uint64_t>* da, bool* curr_visit, bool* next_visit, uint64_t vertex_count,
                                                                  const uint64_t* vertexList, unsigned long long* comp, bool* changed, uint64_t coarse,
                                                                  const heavy_piece_t* heavy, uint64_t n_heavy, unsigned long long* next_work, uint32_t sweep)
{
    walk_vertex_groups(da, vertexList, vertex_count, coarse, heavy, n_heavy, next_work, (sweep & 1u) != 0,
                       [&](uint64_t v) { return curr_visit[v]; },
                       [&](uint64_t v, uint64_t next, uint64_t) { cc_compute(v, comp, next, next_visit, changed); });
}

template <int SHAPE>
__global__ __launch_bounds__(128) void k_cc_shaped(array_d_t<uint64_t>* da, bool* curr_visit, bool* next_visit, uint64_t vertex_count, const uint64_t* vertexList,
                                                   unsigned long long* comp, bool* changed, uint64_t coarse, uint64_t stride, uint64_t n_units)
{
    walk_shaped<SHAPE>(da, vertexList, vertex_count, coarse, stride, n_units,
                       [&](uint64_t v) { return curr_visit[v]; },
                       [&](uint64_t v, uint64_t next, uint64_t) { cc_compute(v, comp, next, next_visit, changed); });
}

// ---- BFS / CC by edge page (benchmarks/bfs/main.cu:1074-1140 kernel_optimized_ptr_pc, first-vertex table :122-181) ----
/*
 * first[p], p = 0 .. n_pages: the vertex whose edge list holds edge p * epp (the last vertex with
 * offsets[v] <= p * epp); first[n_pages] = V - 1.  The vertices with edges on page p are first[p] .. first[p + 1].
 */
__global__ void k_page_first_vertex(const uint64_t* offsets, uint64_t n_vertices, uint64_t epp, uint64_t n_pages, uint64_t* first)
{
    const uint64_t p = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (p > n_pages) return;
    const uint64_t e = p * epp;
    uint64_t lo = 0, hi = n_vertices + 1;            /* first index with offsets[idx] > e */
    while (lo < hi) {
        const uint64_t mid = (lo + hi) >> 1;
        if (offsets[mid] > e) hi = mid; else lo = mid + 1;
    }
    uint64_t v = lo ? lo - 1 : 0;
    if (v >= n_vertices) v = n_vertices - 1;
    first[p] = v;
}

/*
 * One wave, `ppw` consecutive pages of the edge array per trip (lane l looks after page l of the trip), trips
 * handed out wave by wave along the array.  A page is wanted when one of its vertices is active; the wanted pages
 * of a trip are taken with one acquire, so their misses go to the store as one batch of commands, and the whole
 * wave then walks the active vertices of each page, 64 edges at a time, before the references are dropped.
 * A wave holds at most `ppw` pages at a time; the launch keeps waves x ppw under half the cache.
 */
template <typename Active, typename Visit>
__device__ __forceinline__ void graph_by_page(array_d_t<uint64_t>* da, const uint64_t* offsets, const uint64_t* first, const uint64_t n_edges,
                                              const uint32_t ppw, const bool backwards, Active active, Visit visit)
{
    const uint32_t lane = bam::lane();
    const uint64_t wave = ((uint64_t)blockIdx.x * blockDim.x + threadIdx.x) / BAM_WAVE_SIZE;
    const uint64_t n_waves = (uint64_t)gridDim.x * blockDim.x / BAM_WAVE_SIZE;
    bam::range_view<uint64_t> view;
    view.load(da->d_ranges);
    const uint32_t epp = view.page_size / 8;
    const uint64_t n_pages = (n_edges + epp - 1) / epp;
    const uint64_t pso_pages = view.pso >> view.page_size_log;
    const uint64_t n_trips = (n_pages + ppw - 1) / ppw;
    for (uint64_t t = wave; t < n_trips; t += n_waves) {
        /* every other sweep runs from the far end: what the last sweep left in the cache is what this one asks for first */
        const uint64_t p0 = (backwards ? n_trips - 1 - t : t) * ppw;
        const uint64_t p = p0 + lane;
        /* which pages of the trip hold entries of an active vertex: the lanes go over the trip's vertices side by side
         * (their flags and offsets are consecutive in memory) and mark the pages each active list covers */
        const uint64_t p_end = p0 + ppw < n_pages ? p0 + ppw : n_pages;
        const uint64_t trip_start = p0 * epp, trip_end = p_end * epp < n_edges ? p_end * epp : n_edges;
        uint64_t marks = 0;
        for (uint64_t vbase = first[p0], v_last = first[p_end]; vbase <= v_last; vbase += BAM_WAVE_SIZE) {
            const uint64_t v = vbase + lane;
            if (v <= v_last && active(v)) {
                uint64_t es = offsets[v], ee = offsets[v + 1];
                if (es < trip_start) es = trip_start;
                if (ee > trip_end) ee = trip_end;
                if (ee > es) marks |= (~0ull >> (63 - (ee - 1 - trip_start) / epp)) & (~0ull << ((es - trip_start) / epp));
            }
        }
#pragma unroll
        for (uint32_t o = BAM_WAVE_SIZE / 2; o; o >>= 1) marks |= bam::shfl(marks, lane ^ o);
        const bool want = ((marks >> lane) & 1) != 0;
        uint64_t va = 0, vb = 0;
        if (want) { va = first[p]; vb = first[p + 1]; }
        uint32_t slot = BAM_NO_SLOT;
        if (bam::ballot(want)) {
            /* the lanes without a page of their own come along and help move what the others load */
            auto keep = [&](uint32_t s_) { slot = s_; return false; };
            view.acquire_helped(p + pso_pages, want, false, keep, keep);
        }
        /* a page whose wait was given up (the controller is marked aborted) has no slot and is not walked */
        for (uint64_t m = bam::ballot(want && slot != BAM_NO_SLOT); m; m &= m - 1) {
            const uint32_t j = bam::first_lane(m);
            const uint64_t va_j = bam::bcast(va, j), vb_j = bam::bcast(vb, j);
            const uint64_t ps = (p0 + j) * epp, pe = ps + epp < n_edges ? ps + epp : n_edges;
            const uint64_t* payload = (const uint64_t*)view.slot_addr(bam::bcast(slot, j));
            for (uint64_t vbase = va_j; vbase <= vb_j; vbase += BAM_WAVE_SIZE) {
                const uint64_t v = vbase + lane;
                uint64_t es = 0, ee = 0;
                if (v <= vb_j && active(v)) {
                    es = offsets[v]; ee = offsets[v + 1];
                    if (es < ps) es = ps;
                    if (ee > pe) ee = pe;
                }
                if (ee < es) ee = es;
                walk_packed(es, ee, v, [&](uint64_t i) { return bam::ld_payload(payload + (i - ps)); }, visit);
            }
        }
        if (want) view.release(p + pso_pages, false);
    }
    view.flush_stats();
}

__global__ __launch_bounds__(64) void k_bfs_by_page(array_d_t<uint64_t>* da, uint32_t* label, const uint32_t level, const uint64_t* offsets,
                                                     const uint64_t* first, uint64_t n_edges, uint32_t ppw, uint64_t* changed)
{
    bool any = false;
    graph_by_page(da, offsets, first, n_edges, ppw, (level & 1u) != 0,
                  [&](uint64_t v) { return label[v] == level; },
                  [&](uint64_t, uint64_t next, uint64_t) { if (label[next] == MYINFINITY) { label[next] = level + 1; any = true; } });
    if (any) *changed = 1;
}

__global__ __launch_bounds__(64) void k_cc_by_page(array_d_t<uint64_t>* da, bool* curr_visit, bool* next_visit, const uint64_t* offsets,
                                                    const uint64_t* first, uint64_t n_edges, uint32_t ppw, uint32_t sweep, unsigned long long* comp, bool* changed)
{
    graph_by_page(da, offsets, first, n_edges, ppw, (sweep & 1u) != 0,
                  [&](uint64_t v) { return curr_visit[v]; },
                  [&](uint64_t src, uint64_t next, uint64_t) { cc_compute(src, comp, next, next_visit, changed); });
}

// ---- PageRank by residual pushes (benchmarks/pagerank/main.cu:107-115 initialize, :252-273 kernel_coalesce_pc, :412-421 update) ----
__global__ void k_pr_initialize(bool* label, float* delta, float* residual, float* value, const uint64_t vertex_count, const uint64_t* vertexList, float alpha)
{
    const uint64_t tid = (uint64_t)blockDim.x * blockIdx.x + threadIdx.x;
    if (tid < vertex_count) {
        value[tid] = 1.0f - alpha;
        delta[tid] = (1.0f - alpha) * alpha / (vertexList[tid + 1] - vertexList[tid]);
        residual[tid] = 0.0f;
        label[tid] = true;
    }
}

/* every neighbour of a flagged vertex receives the vertex's delta: the group walk of the per-vertex graph kernels; the flags
 * are cleared by the host loop after the sweep */
__global__ __launch_bounds__(128) BAM_GRAPH_KERNEL_WAVES void k_pr_coalesce_pc(array_d_t<uint64_t>* da, const bool* label, const float* delta, float* residual,
                                                        const uint64_t vertex_count, const uint64_t* vertexList, uint64_t group,
                                                        const heavy_piece_t* heavy, uint64_t n_heavy, unsigned long long* next_work, uint32_t sweep)
{
    walk_vertex_groups(da, vertexList, vertex_count, group, heavy, n_heavy, next_work, (sweep & 1u) != 0,
                       [&](uint64_t v) { return label[v]; },
                       [&](uint64_t src, uint64_t next, uint64_t) { unsafeAtomicAdd(&residual[next], delta[src]); });
}

/* the same pushes taken page by page of the edge array; the flags are cleared by the host loop after the sweep */
__global__ __launch_bounds__(64) void k_pr_by_page(array_d_t<uint64_t>* da, const bool* label, const float* delta, float* residual, const uint64_t* offsets,
                                                    const uint64_t* first, uint64_t n_edges, uint32_t ppw, uint32_t sweep)
{
    graph_by_page(da, offsets, first, n_edges, ppw, (sweep & 1u) != 0,
                  [&](uint64_t v) { return label[v]; },
                  [&](uint64_t src, uint64_t next, uint64_t) { unsafeAtomicAdd(&residual[next], delta[src]); });
}

__global__ void k_pr_update(bool* label, float* delta, float* residual, float* value, const uint64_t vertex_count, const uint64_t* vertexList,
                            float tolerance, float alpha, bool* changed)
{
    const uint64_t tid = (uint64_t)blockDim.x * blockIdx.x + threadIdx.x;
    if (tid < vertex_count && residual[tid] > tolerance) {
        value[tid] += residual[tid];
        delta[tid] = residual[tid] * alpha / (vertexList[tid + 1] - vertexList[tid]);
        residual[tid] = 0.0f;
        label[tid] = true;
        *changed = true;
    }
}

// ---- SSSP (benchmarks/sssp/main.cu:174-201 kernel_coalesce_pc, :282-292 update): 32-bit costs, weights in their own array ----
/* relaxation of the edges of the flagged vertices with the cost each has at the time (any cost a vertex holds is the cost of a
 * path to it); the group walk of the per-vertex graph kernels, the weight of entry i read through a bam_ptr of its own */
template <bool FLOAT>
__device__ __forceinline__ void sssp_relax(uint32_t* newCostList, const bam_ptr<uint32_t>& weights, uint64_t src, uint64_t next, uint64_t i)
{
    const uint32_t have = __hip_atomic_load(&newCostList[src], __ATOMIC_RELAXED, BAM_AGENT), w = weights[i];
    /* single-precision costs (benchmarks/sssp_float/main.cu:69, 91-106, 194-217) travel as their bit patterns: for floats that
     * are not negative the order of the patterns is the order of the values, so the minimum is the integer one */
    const uint32_t cost = FLOAT ? __float_as_uint(__uint_as_float(have) + __uint_as_float(w)) : have + w;
    if (__hip_atomic_load(&newCostList[next], __ATOMIC_RELAXED, BAM_AGENT) > cost) atomicMin(&newCostList[next], cost);
}

template <bool FLOAT>
__global__ __launch_bounds__(128) BAM_GRAPH_KERNEL_WAVES void k_sssp_coalesce_pc(array_d_t<uint64_t>* de, array_d_t<uint32_t>* dw, const bool* label, uint32_t* newCostList,
                                                          const uint64_t vertex_count, const uint64_t* vertexList, uint64_t group,
                                                          const heavy_piece_t* heavy, uint64_t n_heavy, unsigned long long* next_work, uint32_t sweep)
{
    bam_ptr<uint32_t> wptr(dw);
    /* entry i of the weight array belongs to entry i of the edge array: what is touched ahead for the one is touched for the other */
    list_read_ahead<uint32_t> wahead;
    wahead.init(dw);
    walk_vertex_groups(de, vertexList, vertex_count, group, heavy, n_heavy, next_work, (sweep & 1u) != 0,
                       [&](uint64_t v) { return label[v]; },
                       [&](uint64_t src, uint64_t next, uint64_t i) { sssp_relax<FLOAT>(newCostList, wptr, src, next, i); }, &wahead);
}

__global__ void k_sssp_update(bool* label, uint32_t* costList, const uint32_t* newCostList, const uint64_t vertex_count, bool* changed)
{
    const uint64_t tid = (uint64_t)blockDim.x * blockIdx.x + threadIdx.x;
    if (tid < vertex_count && newCostList[tid] < costList[tid]) {
        costList[tid] = newCostList[tid];
        label[tid] = true;
        *changed = true;
    }
}

__global__ void k_iota(unsigned long long* p, uint64_t n)
{
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = i;
}

} // namespace

extern "C" {

namespace {
/* launch shape of the by-page graph kernels: pages per wave trip and number of waves, so that what the waves hold
 * at any time stays under half of the cache */
struct by_page_plan { uint64_t n_edges = 0, n_pages = 0; uint32_t epp = 0, ppw = 0, blocks = 0; BufferPtr first; };

/* the end of a level: the device's `changed` word goes to the host through pinned memory, and it and the counter the next
 * sweep takes its work from start the next level at zero.  One small launch instead of two copies and a fill. */
__global__ void k_level_end(uint64_t* changed, unsigned long long* next_work, volatile uint64_t* host_flag)
{
    *host_flag = *changed;
    *changed = 0;
    *next_work = 0;
}

/*
 * What the graph entry points need besides the graph, made once per graph (bam_array_set_graph) or, without that, once per
 * call: the pieces of the long edge lists (a list of d >= BAM_HEAVY_EDGES entries makes at most d / BAM_PIECE_EDGES + 1 <=
 * 2 d / BAM_HEAVY_EDGES pieces), the counter that hands out the work of a sweep, the `changed` word and its pinned copy,
 * the first-vertex table of the by-page kernels, and the per-vertex buffers of the algorithms, which come when first asked for.
 */
struct graph_plan {
    const uint64_t* offsets = nullptr;
    uint64_t n_vertices = 0, n_edges = 0;
    BufferPtr buf, words, host_words;
    heavy_piece_t* pieces = nullptr;
    unsigned long long* count = nullptr;     /* [0] number of pieces, [1] next piece of work of the sweep */
    uint64_t* changed = nullptr;             /* device */
    volatile uint64_t* host_flag = nullptr;  /* pinned host memory */
    uint64_t n_pieces = 0;
    uint64_t group = 512;                    /* vertices handed to a wave at a time */
    uint64_t resident = 0;                   /* waves a sweep runs */
    by_page_plan bp;
    bool bp_built = false;
    BufferPtr bytes_a, bytes_b, floats_a, floats_b, words_a;      /* per-vertex buffers: flags, PageRank's delta and residual, SSSP's new costs */
    BufferPtr queue_a, queue_b, queue_bits, queue_totals;         /* bam_bfs_frontier: the two queues, the bit map that puts a queue in order and its counts per 4096 vertices */

    int build(bam_array_t* edges, const uint64_t* d_offsets, uint64_t nv, uint64_t other_cache_pages, hipStream_t st)
    {
        offsets = d_offsets; n_vertices = nv; n_edges = edges->a->adt.n_elems;
        const uint64_t cap = 2 * (n_edges / BAM_HEAVY_EDGES) + 1;
        buf = createBuffer(cap * sizeof(heavy_piece_t), 0);
        words = createBuffer(64, 0);
        host_words = createHostBuffer(64);
        pieces = (heavy_piece_t*)buf.get();
        count = (unsigned long long*)words.get();
        changed = (uint64_t*)words.get() + 2;
        host_flag = (volatile uint64_t*)host_words.get();
        int dev = 0, cus = 0;
        hip_err_chk(hipGetDevice(&dev));
        hip_err_chk(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
        resident = (uint64_t)cus * 16;
        /* every lane of a running wave may hold a page of its own (its bam_ptr keeps the last one it read): more waves
         * than the cache has pages for would wait for slots that only they can give back */
        uint64_t cache_pages = edges->a->adt.n_ranges ? edges->a->h_ranges[0].cache.n_pages : 0;
        if (other_cache_pages && other_cache_pages < cache_pages) cache_pages = other_cache_pages;
        if (cache_pages && resident > cache_pages / BAM_WAVE_SIZE) resident = cache_pages / BAM_WAVE_SIZE;
        if (resident < 2) resident = 2;
        hip_err_chk(hipMemsetAsync(words.get(), 0, 64, st));
        hipLaunchKernelGGL(k_heavy_pieces, dim3(blocks_for(n_vertices, 256)), dim3(256), 0, st, d_offsets, n_vertices, pieces, count);
        hip_err_chk(hipGetLastError());
        unsigned long long n = 0;
        hip_err_chk(hipMemcpyAsync(&n, count, sizeof(n), hipMemcpyDeviceToHost, st));
        hip_err_chk(hipStreamSynchronize(st));
        n_pieces = n;
        return 0;
    }
    /* workgroups of two waves for a sweep over `n_items` items in groups of `grp` */
    uint32_t blocks(uint64_t n_items, uint64_t grp) const
    {
        const uint64_t units = (n_pieces + BAM_PIECE_BUNDLE - 1) / BAM_PIECE_BUNDLE + (n_items + grp - 1) / grp;
        return (uint32_t)(((units < resident ? units : resident) + 1) / 2);
    }
    unsigned long long* next_work() const { return count + 1; }
    /* between sweeps `changed` and the work counter are zero; true if the sweep just queued on `st` changed anything */
    bool level_end(hipStream_t st)
    {
        hipLaunchKernelGGL(k_level_end, dim3(1), dim3(1), 0, st, changed, count + 1, host_flag);
        hip_err_chk(hipGetLastError());
        hip_err_chk(hipStreamSynchronize(st));
        return *host_flag != 0;
    }
    int by_page(bam_array_t* edges, hipStream_t st);
    static void* sized(BufferPtr& b, uint64_t bytes) { if (!b) b = createBuffer(bytes ? bytes : 8, 0); return b.get(); }
};

int graph_plan::by_page(bam_array_t* edges, hipStream_t st)
{
    if (bp_built) return 0;
    by_page_plan& pl = bp;
    array_t<uint64_t>* a = edges->a;
    if (a->adt.n_ranges != 1) return fail(EINVAL, "by-page graph kernels take an array of one range");
    const range_d_t<uint64_t>& r = a->h_ranges[0];
    if (r.index_start != 0 || r.page_start_offset % r.cache.page_size) return fail(EINVAL, "by-page graph kernels need a range that starts on a page boundary");
    pl.n_edges = a->adt.n_elems;
    pl.epp = (uint32_t)(r.cache.page_size / 8);
    pl.n_pages = (pl.n_edges + pl.epp - 1) / pl.epp;
    const uint64_t budget = r.cache.n_pages / 2;               /* pages all waves together may hold */
    if (!budget) return fail(EINVAL, "by-page graph kernels need a cache of at least two pages");
    int dev = 0, cus = 0;
    hip_err_chk(hipGetDevice(&dev));
    hip_err_chk(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const uint64_t max_waves = (uint64_t)cus * 8;              /* eight waves per compute unit */
    uint64_t ppw = budget / max_waves;
    if (ppw > BAM_WAVE_SIZE) ppw = BAM_WAVE_SIZE;
    if (ppw < 1) ppw = 1;
    uint64_t waves = budget / ppw;
    if (waves > max_waves) waves = max_waves;
    const uint64_t trips = (pl.n_pages + ppw - 1) / ppw;
    if (waves > trips) waves = trips;
    pl.ppw = (uint32_t)ppw;
    pl.blocks = (uint32_t)waves;                               /* one wave per workgroup */
    pl.first = createBuffer((pl.n_pages + 1) * sizeof(uint64_t), dev);
    hipLaunchKernelGGL(k_page_first_vertex, dim3(blocks_for(pl.n_pages + 1, 256)), dim3(256), 0, st, offsets, n_vertices, (uint64_t)pl.epp, pl.n_pages,
                       (uint64_t*)pl.first.get());
    hip_err_chk(hipGetLastError());
    bp_built = true;
    return 0;
}

/* the plan bam_array_set_graph made for this graph, or one made now in `local` that lives for the call */
graph_plan* plan_for(bam_array_t* edges, const uint64_t* d_offsets, uint64_t n_vertices, uint64_t other_cache_pages, hipStream_t st, std::unique_ptr<graph_plan>& local)
{
    graph_plan* p = (graph_plan*)edges->graph.get();
    if (p && p->offsets == d_offsets && p->n_vertices == n_vertices && p->n_edges == edges->a->adt.n_elems && !other_cache_pages) return p;
    local.reset(new graph_plan());
    local->build(edges, d_offsets, n_vertices, other_cache_pages, st);
    return local.get();
}
} // namespace

int bam_array_set_graph(bam_array_t* edges, const uint64_t* d_offsets, uint64_t n_vertices, void* stream)
{
    if (!edges) return fail(EINVAL, "bam_array_set_graph: null argument");
    if (!d_offsets) { edges->graph.reset(); return 0; }
    if (!n_vertices) return fail(EINVAL, "bam_array_set_graph: empty graph");
    BAM_API_BEGIN
    hipStream_t st = (hipStream_t)stream;
    std::shared_ptr<graph_plan> p(new graph_plan());
    p->build(edges, d_offsets, n_vertices, 0, st);
    if (edges->a->adt.n_ranges == 1) {
        const range_d_t<uint64_t>& r = edges->a->h_ranges[0];
        if (r.index_start == 0 && r.page_start_offset % r.cache.page_size == 0 && r.cache.n_pages >= 2) p->by_page(edges, st);
    }
    /* the per-vertex buffers the sweeps use, so that no later call has to allocate */
    graph_plan::sized(p->bytes_a, n_vertices); graph_plan::sized(p->bytes_b, n_vertices);
    graph_plan::sized(p->floats_a, n_vertices * sizeof(float)); graph_plan::sized(p->floats_b, n_vertices * sizeof(float));
    if (n_vertices <= 0xFFFFFFFFull) {
        /* bam_bfs_frontier's queues and what puts them in order */
        const uint64_t n_words = (n_vertices + 63) / 64;
        graph_plan::sized(p->queue_a, n_vertices * sizeof(uint32_t)); graph_plan::sized(p->queue_b, n_vertices * sizeof(uint32_t));
        graph_plan::sized(p->queue_bits, n_words * sizeof(unsigned long long));
        graph_plan::sized(p->queue_totals, (n_words + BAM_WAVE_SIZE - 1) / BAM_WAVE_SIZE * sizeof(uint32_t));
    }
    hip_err_chk(hipStreamSynchronize(st));
    edges->graph = p;
    BAM_API_END
}

int bam_bfs(bam_array_t* edges, const uint64_t* d_offsets, uint64_t n_vertices, uint64_t src, uint32_t* d_labels,
            uint32_t coarse, uint32_t* iterations, void* stream)
{
    if (!edges || !d_offsets || !d_labels) return fail(EINVAL, "bam_bfs: null argument");
    if (src >= n_vertices || !coarse) return fail(EINVAL, "bam_bfs: source out of range or coarse = 0");
    BAM_API_BEGIN
    hipStream_t st = (hipStream_t)stream;
    std::unique_ptr<graph_plan> local;
    graph_plan* pl = plan_for(edges, d_offsets, n_vertices, 0, st, local);
    /* a group's lists are asked for as one batch of commands: a few hundred vertices make that batch large enough for the
     * store path, and keep the one word all waves take their work from out of the way */
    const uint64_t group = coarse > 512 ? coarse : 512;
    hip_err_chk(hipMemsetAsync(d_labels, 0xFF, n_vertices * sizeof(uint32_t), st));
    hip_err_chk(hipMemsetAsync(d_labels + src, 0, sizeof(uint32_t), st));
    const uint32_t threads = 128;
    uint32_t level = 0, iter = 0;
    bool changed;
    do {
        hipLaunchKernelGGL(k_bfs_coalesce_coarse_ptr_pc, dim3(pl->blocks(n_vertices, group)), dim3(threads), 0, st,
                           edges->a->d_array_ptr, d_labels, level, n_vertices, d_offsets, pl->changed, group, pl->pieces, pl->n_pieces, pl->next_work());
        hip_err_chk(hipGetLastError());
        iter++; level++;
        changed = pl->level_end(st);
    } while (changed);
    if (iterations) *iterations = iter;
    BAM_API_END
}

namespace {
/* units of a shaped launch and the waves that walk them (see walk_shaped): at most one wave per eight pages of the cache */
struct shaped_launch { uint64_t n_units; uint32_t blocks; };
shaped_launch shape_of(int shape, uint64_t n_vertices, uint64_t coarse, uint64_t stride, uint64_t cache_pages)
{
    shaped_launch sl{};
    if (shape == 3) sl.n_units = (n_vertices + BAM_SHAPE_CHUNK - 1) / BAM_SHAPE_CHUNK;
    else if (shape == 1) sl.n_units = ((n_vertices + stride * coarse) / (stride * coarse)) * stride;
    else sl.n_units = ((n_vertices + stride) / stride) * stride;
    const uint64_t per_wave = shape == 2 ? 4 : 1;
    uint64_t waves = (sl.n_units + per_wave - 1) / per_wave;
    int dev = 0, cus = 0;
    hip_err_chk(hipGetDevice(&dev));
    hip_err_chk(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    if (waves > (uint64_t)cus * 16) waves = (uint64_t)cus * 16;
    if (cache_pages && waves > cache_pages / 8) waves = cache_pages / 8;
    if (waves < 2) waves = 2;
    sl.blocks = (uint32_t)((waves + 1) / 2);            /* workgroups of two waves */
    return sl;
}
} // namespace

int bam_bfs_shaped(bam_array_t* edges, const uint64_t* d_offsets, uint64_t n_vertices, uint64_t src, uint32_t* d_labels,
                   int shape, uint32_t coarse, uint32_t stride, uint32_t* iterations, void* stream)
{
    if (!edges || !d_offsets || !d_labels) return fail(EINVAL, "bam_bfs_shaped: null argument");
    if (src >= n_vertices || shape < 0 || shape > 3 || !coarse || !stride) return fail(EINVAL, "bam_bfs_shaped: source out of range, shape not 0..3, or coarse / stride = 0");
    BAM_API_BEGIN
    hipStream_t st = (hipStream_t)stream;
    std::unique_ptr<graph_plan> local;
    graph_plan* pl = plan_for(edges, d_offsets, n_vertices, 0, st, local);
    const shaped_launch sl = shape_of(shape, n_vertices, coarse, stride, edges->a->adt.n_ranges ? edges->a->h_ranges[0].cache.n_pages : 0);
    hip_err_chk(hipMemsetAsync(d_labels, 0xFF, n_vertices * sizeof(uint32_t), st));
    hip_err_chk(hipMemsetAsync(d_labels + src, 0, sizeof(uint32_t), st));
    uint32_t level = 0, iter = 0;
    bool changed;
    do {
        const dim3 grid(sl.blocks), block(128);
        array_d_t<uint64_t>* d = edges->a->d_array_ptr;
        switch (shape) {
        case 0: hipLaunchKernelGGL(k_bfs_shaped<0>, grid, block, 0, st, d, d_labels, level, n_vertices, d_offsets, pl->changed, (uint64_t)coarse, (uint64_t)stride, sl.n_units); break;
        case 1: hipLaunchKernelGGL(k_bfs_shaped<1>, grid, block, 0, st, d, d_labels, level, n_vertices, d_offsets, pl->changed, (uint64_t)coarse, (uint64_t)stride, sl.n_units); break;
        case 2: hipLaunchKernelGGL(k_bfs_shaped<2>, grid, block, 0, st, d, d_labels, level, n_vertices, d_offsets, pl->changed, (uint64_t)coarse, (uint64_t)stride, sl.n_units); break;
        default: hipLaunchKernelGGL(k_bfs_shaped<3>, grid, block, 0, st, d, d_labels, level, n_vertices, d_offsets, pl->changed, (uint64_t)coarse, (uint64_t)stride, sl.n_units); break;
        }
        hip_err_chk(hipGetLastError());
        iter++; level++;
        changed = pl->level_end(st);
    } while (changed);
    if (iterations) *iterations = iter;
    BAM_API_END
}

int bam_cc_shaped(bam_array_t* edges, const uint64_t* d_offsets, uint64_t n_vertices, uint64_t* d_labels,
                  int shape, uint32_t coarse, uint32_t stride, uint32_t* iterations, void* stream)
{
    if (!edges || !d_offsets || !d_labels) return fail(EINVAL, "bam_cc_shaped: null argument");
    if (!n_vertices || shape < 0 || shape > 3 || !coarse || !stride) return fail(EINVAL, "bam_cc_shaped: empty graph, shape not 0..3, or coarse / stride = 0");
    BAM_API_BEGIN
    hipStream_t st = (hipStream_t)stream;
    std::unique_ptr<graph_plan> local;
    graph_plan* pl = plan_for(edges, d_offsets, n_vertices, 0, st, local);
    const shaped_launch sl = shape_of(shape, n_vertices, coarse, stride, edges->a->adt.n_ranges ? edges->a->h_ranges[0].cache.n_pages : 0);
    bool* curr = (bool*)graph_plan::sized(pl->bytes_a, n_vertices);
    bool* next = (bool*)graph_plan::sized(pl->bytes_b, n_vertices);
    hipLaunchKernelGGL(k_iota, dim3(blocks_for(n_vertices, 256)), dim3(256), 0, st, (unsigned long long*)d_labels, n_vertices);
    hip_err_chk(hipMemsetAsync(curr, 0x01, n_vertices, st));
    hip_err_chk(hipMemsetAsync(next, 0x00, n_vertices, st));
    uint32_t iter = 0;
    bool changed;
    do {
        const dim3 grid(sl.blocks), block(128);
        array_d_t<uint64_t>* d = edges->a->d_array_ptr;
        unsigned long long* comp = (unsigned long long*)d_labels;
        bool* ch = (bool*)pl->changed;
        switch (shape) {
        case 0: hipLaunchKernelGGL(k_cc_shaped<0>, grid, block, 0, st, d, curr, next, n_vertices, d_offsets, comp, ch, (uint64_t)coarse, (uint64_t)stride, sl.n_units); break;
        case 1: hipLaunchKernelGGL(k_cc_shaped<1>, grid, block, 0, st, d, curr, next, n_vertices, d_offsets, comp, ch, (uint64_t)coarse, (uint64_t)stride, sl.n_units); break;
        case 2: hipLaunchKernelGGL(k_cc_shaped<2>, grid, block, 0, st, d, curr, next, n_vertices, d_offsets, comp, ch, (uint64_t)coarse, (uint64_t)stride, sl.n_units); break;
        default: hipLaunchKernelGGL(k_cc_shaped<3>, grid, block, 0, st, d, curr, next, n_vertices, d_offsets, comp, ch, (uint64_t)coarse, (uint64_t)stride, sl.n_units); break;
        }
        hip_err_chk(hipGetLastError());
        hip_err_chk(hipMemsetAsync(curr, 0x00, n_vertices, st));
        bool* t = curr; curr = next; next = t;
        iter++;
        changed = pl->level_end(st);
    } while (changed);
    if (iterations) *iterations = iter;
    BAM_API_END
}

int bam_bfs_frontier(bam_array_t* edges, const uint64_t* d_offsets, uint64_t n_vertices, uint64_t src, uint32_t* d_labels,
                     uint32_t* iterations, void* stream)
{
    if (!edges || !d_offsets || !d_labels) return fail(EINVAL, "bam_bfs_frontier: null argument");
    if (src >= n_vertices) return fail(EINVAL, "bam_bfs_frontier: source out of range");
    if (n_vertices > 0xFFFFFFFFull) return fail(EINVAL, "bam_bfs_frontier: the queues hold 32-bit vertex numbers");
    BAM_API_BEGIN
    hipStream_t st = (hipStream_t)stream;
    std::unique_ptr<graph_plan> local;
    graph_plan* pl = plan_for(edges, d_offsets, n_vertices, 0, st, local);
    /* two queues of at most every vertex once (benchmarks/bfs/main.cu:1489-1492); the size of the next one is the reference's `changed`.
     * They, and what puts a queue in order, belong to the plan: with bam_array_set_graph nothing is allocated here */
    uint32_t* curr = (uint32_t*)graph_plan::sized(pl->queue_a, n_vertices * sizeof(uint32_t));
    uint32_t* next = (uint32_t*)graph_plan::sized(pl->queue_b, n_vertices * sizeof(uint32_t));
    const uint64_t n_words = (n_vertices + 63) / 64, n_bit_waves = (n_words + BAM_WAVE_SIZE - 1) / BAM_WAVE_SIZE;
    unsigned long long* bits = (unsigned long long*)graph_plan::sized(pl->queue_bits, n_words * sizeof(unsigned long long));      /* zero between levels */
    uint32_t* totals = (uint32_t*)graph_plan::sized(pl->queue_totals, n_bit_waves * sizeof(uint32_t));
    unsigned long long* next_size = (unsigned long long*)pl->changed;
    const uint32_t src32 = (uint32_t)src;
    hip_err_chk(hipMemsetAsync(d_labels, 0xFF, n_vertices * sizeof(uint32_t), st));
    hip_err_chk(hipMemsetAsync(d_labels + src, 0, sizeof(uint32_t), st));
    hip_err_chk(hipMemcpyAsync(curr, &src32, sizeof(uint32_t), hipMemcpyHostToDevice, st));
    const uint32_t threads = 128;
    uint64_t group = BAM_WAVE_SIZE;                 /* queue entries handed to a wave at a time: one per lane, more of a sorted queue */
    bool sorted = true;                             /* the first queue holds the source alone */
    uint32_t level = 0, iter = 0;
    unsigned long long active = 1;
    const char* e = getenv("BAM_FRONTIER_SORT");
    const bool sort_queue = !e || atoi(e) != 0;
    do {
        hipLaunchKernelGGL(k_bfs_frontier_coalesce_ptr_pc, dim3(pl->blocks(active, group)), dim3(threads), 0, st, edges->a->d_array_ptr, d_labels, level,
                           d_offsets, curr, (uint64_t)active, next, next_size, group, pl->pieces, pl->n_pieces, pl->next_work(), sorted);
        hip_err_chk(hipGetLastError());
        iter++; level++;
        pl->level_end(st);
        active = *pl->host_flag;
        sorted = sort_queue;
        group = sorted ? pl->group : BAM_WAVE_SIZE;
        if (sorted && active > 1) {
            /* the queue comes out in the order of discovery; in the order of the vertices the level reads the edge array
             * front to back (neighbouring lists share pages, a page is not evicted between two of its lists, and the pages
             * under the lists of a group of entries can be asked for together as in the sweep over all vertices).  The
             * ordered queue goes into the buffer the level just walked, so the two do not change places. */
            hipLaunchKernelGGL(k_queue_mark, dim3(blocks_for(active, 256)), dim3(256), 0, st, next, (uint64_t)active, bits);
            hipLaunchKernelGGL(k_bits_count, dim3(blocks_for(n_bit_waves * BAM_WAVE_SIZE, 256)), dim3(256), 0, st, bits, n_words, totals);
            hipLaunchKernelGGL(k_totals_scan, dim3(1), dim3(1024), 0, st, totals, n_bit_waves);
            hipLaunchKernelGGL(k_bits_emit, dim3(blocks_for(n_bit_waves * BAM_WAVE_SIZE, 256)), dim3(256), 0, st, bits, n_words, totals, curr);
            hip_err_chk(hipGetLastError());
        } else
            std::swap(curr, next);
    } while (active);
    if (iterations) *iterations = iter;
    BAM_API_END
}

int bam_cc(bam_array_t* edges, const uint64_t* d_offsets, uint64_t n_vertices, uint64_t* d_labels,
           uint32_t coarse, uint32_t* iterations, void* stream)
{
    if (!edges || !d_offsets || !d_labels) return fail(EINVAL, "bam_cc: null argument");
    if (!coarse || !n_vertices) return fail(EINVAL, "bam_cc: empty graph or coarse = 0");
    BAM_API_BEGIN
    hipStream_t st = (hipStream_t)stream;
    std::unique_ptr<graph_plan> local;
    graph_plan* pl = plan_for(edges, d_offsets, n_vertices, 0, st, local);
    const uint64_t group = coarse > 512 ? coarse : 512;
    bool* curr = (bool*)graph_plan::sized(pl->bytes_a, n_vertices);
    bool* next = (bool*)graph_plan::sized(pl->bytes_b, n_vertices);
    hipLaunchKernelGGL(k_iota, dim3(blocks_for(n_vertices, 256)), dim3(256), 0, st, (unsigned long long*)d_labels, n_vertices);
    hip_err_chk(hipMemsetAsync(curr, 0x01, n_vertices, st));
    hip_err_chk(hipMemsetAsync(next, 0x00, n_vertices, st));
    const uint32_t threads = 128;
    uint32_t iter = 0;
    bool changed;
    do {
        hipLaunchKernelGGL(k_cc_coalesce_coarse_ptr_pc, dim3(pl->blocks(n_vertices, group)), dim3(threads), 0, st, edges->a->d_array_ptr, curr, next,
                           n_vertices, d_offsets, (unsigned long long*)d_labels, (bool*)pl->changed, group, pl->pieces, pl->n_pieces, pl->next_work(), iter);
        hip_err_chk(hipGetLastError());
        hip_err_chk(hipMemsetAsync(curr, 0x00, n_vertices, st));
        bool* t = curr; curr = next; next = t;
        iter++;
        changed = pl->level_end(st);
    } while (changed);
    if (iterations) *iterations = iter;
    BAM_API_END
}

int bam_bfs_by_page(bam_array_t* edges, const uint64_t* d_offsets, uint64_t n_vertices, uint64_t src, uint32_t* d_labels,
                    uint32_t* iterations, void* stream)
{
    if (!edges || !d_offsets || !d_labels) return fail(EINVAL, "bam_bfs_by_page: null argument");
    if (src >= n_vertices) return fail(EINVAL, "bam_bfs_by_page: source out of range");
    BAM_API_BEGIN
    hipStream_t st = (hipStream_t)stream;
    std::unique_ptr<graph_plan> local;
    graph_plan* pl = plan_for(edges, d_offsets, n_vertices, 0, st, local);
    if (int rc = pl->by_page(edges, st)) return rc;
    hip_err_chk(hipMemsetAsync(d_labels, 0xFF, n_vertices * sizeof(uint32_t), st));
    hip_err_chk(hipMemsetAsync(d_labels + src, 0, sizeof(uint32_t), st));
    uint32_t level = 0, iter = 0;
    bool changed;
    do {
        if (pl->bp.n_pages)
            hipLaunchKernelGGL(k_bfs_by_page, dim3(pl->bp.blocks), dim3(BAM_WAVE_SIZE), 0, st, edges->a->d_array_ptr, d_labels, level, d_offsets,
                               (const uint64_t*)pl->bp.first.get(), pl->bp.n_edges, pl->bp.ppw, pl->changed);
        hip_err_chk(hipGetLastError());
        iter++; level++;
        changed = pl->level_end(st);
    } while (changed);
    if (iterations) *iterations = iter;
    BAM_API_END
}

int bam_cc_by_page(bam_array_t* edges, const uint64_t* d_offsets, uint64_t n_vertices, uint64_t* d_labels, uint32_t* iterations, void* stream)
{
    if (!edges || !d_offsets || !d_labels) return fail(EINVAL, "bam_cc_by_page: null argument");
    if (!n_vertices) return fail(EINVAL, "bam_cc_by_page: empty graph");
    BAM_API_BEGIN
    hipStream_t st = (hipStream_t)stream;
    std::unique_ptr<graph_plan> local;
    graph_plan* pl = plan_for(edges, d_offsets, n_vertices, 0, st, local);
    if (int rc = pl->by_page(edges, st)) return rc;
    bool* curr = (bool*)graph_plan::sized(pl->bytes_a, n_vertices);
    bool* next = (bool*)graph_plan::sized(pl->bytes_b, n_vertices);
    hipLaunchKernelGGL(k_iota, dim3(blocks_for(n_vertices, 256)), dim3(256), 0, st, (unsigned long long*)d_labels, n_vertices);
    hip_err_chk(hipMemsetAsync(curr, 0x01, n_vertices, st));
    hip_err_chk(hipMemsetAsync(next, 0x00, n_vertices, st));
    uint32_t iter = 0;
    bool changed;
    do {
        if (pl->bp.n_pages)
            hipLaunchKernelGGL(k_cc_by_page, dim3(pl->bp.blocks), dim3(BAM_WAVE_SIZE), 0, st, edges->a->d_array_ptr, curr, next, d_offsets,
                               (const uint64_t*)pl->bp.first.get(), pl->bp.n_edges, pl->bp.ppw, iter, (unsigned long long*)d_labels, (bool*)pl->changed);
        hip_err_chk(hipGetLastError());
        hip_err_chk(hipMemsetAsync(curr, 0x00, n_vertices, st));
        bool* t = curr; curr = next; next = t;
        iter++;
        changed = pl->level_end(st);
    } while (changed);
    if (iterations) *iterations = iter;
    BAM_API_END
}

int bam_pagerank(bam_array_t* edges, const uint64_t* d_offsets, uint64_t n_vertices, float alpha, float tolerance, uint32_t max_iterations,
                 int by_page, float* d_value, uint32_t* iterations, void* stream)
{
    if (!edges || !d_offsets || !d_value) return fail(EINVAL, "bam_pagerank: null argument");
    if (iterations) *iterations = 0;
    if (!n_vertices) return 0;
    BAM_API_BEGIN
    hipStream_t st = (hipStream_t)stream;
    std::unique_ptr<graph_plan> local;
    graph_plan* pl = plan_for(edges, d_offsets, n_vertices, 0, st, local);
    if (by_page)
        if (int rc = pl->by_page(edges, st)) return rc;
    float* delta_d = (float*)graph_plan::sized(pl->floats_a, n_vertices * sizeof(float));
    float* residual_d = (float*)graph_plan::sized(pl->floats_b, n_vertices * sizeof(float));
    bool* label_d = (bool*)graph_plan::sized(pl->bytes_a, n_vertices);
    const uint32_t upd_blocks = blocks_for(n_vertices, 256);
    hipLaunchKernelGGL(k_pr_initialize, dim3(upd_blocks), dim3(256), 0, st, label_d, delta_d, residual_d, d_value, n_vertices, d_offsets, alpha);
    uint32_t iter = 0;
    bool changed;
    do {
        if (by_page) {
            if (pl->bp.n_pages)
                hipLaunchKernelGGL(k_pr_by_page, dim3(pl->bp.blocks), dim3(BAM_WAVE_SIZE), 0, st, edges->a->d_array_ptr, label_d, delta_d, residual_d, d_offsets,
                                   (const uint64_t*)pl->bp.first.get(), pl->bp.n_edges, pl->bp.ppw, iter);
        } else
            hipLaunchKernelGGL(k_pr_coalesce_pc, dim3(pl->blocks(n_vertices, pl->group)), dim3(128), 0, st, edges->a->d_array_ptr, label_d, delta_d, residual_d,
                               n_vertices, d_offsets, pl->group, pl->pieces, pl->n_pieces, pl->next_work(), iter);
        hip_err_chk(hipMemsetAsync(label_d, 0, n_vertices, st));
        iter++;
        hipLaunchKernelGGL(k_pr_update, dim3(upd_blocks), dim3(256), 0, st, label_d, delta_d, residual_d, d_value, n_vertices, d_offsets, tolerance, alpha, (bool*)pl->changed);
        hip_err_chk(hipGetLastError());
        changed = pl->level_end(st);
    } while (changed && iter < max_iterations);
    if (iterations) *iterations = iter;
    BAM_API_END
}

namespace {
/* the loop of benchmarks/sssp/main.cu:663-725 (and of sssp_float, :624-700): relax from the flagged vertices, adopt what got
 * cheaper, flag it, until nothing does.  FLOAT: costs and weights are single-precision values, unreached = 1e9 (sssp_float :529) */
void sssp_run(const bool FLOAT, bam_array_t* edges, bam_array32_t* weights, const uint64_t* d_offsets, uint64_t n_vertices, uint64_t src, uint32_t* d_costs,
              uint32_t* iterations, hipStream_t st)
{
    /* a lane holds a page of the weights beside its page of the edges: the waves a sweep runs must fit the smaller cache too */
    const uint64_t weight_pages = weights->a->adt.n_ranges ? weights->a->h_ranges[0].cache.n_pages : 0;
    std::unique_ptr<graph_plan> local;
    graph_plan* pl = plan_for(edges, d_offsets, n_vertices, weight_pages ? weight_pages : 1, st, local);
    uint32_t* new_d = (uint32_t*)graph_plan::sized(pl->words_a, n_vertices * sizeof(uint32_t));
    bool* label_d = (bool*)graph_plan::sized(pl->bytes_a, n_vertices);
    const uint32_t zero = 0;                    /* the pattern of 0.0f as well */
    const bool one = true;
    const float far = 1000000000.0f;
    uint32_t unreached = 0xFFFFFFFFu;
    if (FLOAT) memcpy(&unreached, &far, sizeof(unreached));
    hip_err_chk(hipMemsetD32Async((hipDeviceptr_t)d_costs, (int)unreached, n_vertices, st));
    hip_err_chk(hipMemsetD32Async((hipDeviceptr_t)new_d, (int)unreached, n_vertices, st));
    hip_err_chk(hipMemsetAsync(label_d, 0, n_vertices, st));
    hip_err_chk(hipMemcpyAsync(label_d + src, &one, sizeof(bool), hipMemcpyHostToDevice, st));
    hip_err_chk(hipMemcpyAsync(d_costs + src, &zero, sizeof(uint32_t), hipMemcpyHostToDevice, st));
    hip_err_chk(hipMemcpyAsync(new_d + src, &zero, sizeof(uint32_t), hipMemcpyHostToDevice, st));
    const uint32_t threads = 128;
    uint32_t iter = 0;
    bool changed;
    do {
        hipLaunchKernelGGL(FLOAT ? k_sssp_coalesce_pc<true> : k_sssp_coalesce_pc<false>, dim3(pl->blocks(n_vertices, pl->group)), dim3(threads), 0, st,
                           edges->a->d_array_ptr, weights->a->d_array_ptr, label_d, new_d, n_vertices, d_offsets, pl->group, pl->pieces, pl->n_pieces, pl->next_work(), iter);
        hip_err_chk(hipMemsetAsync(label_d, 0, n_vertices, st));
        hipLaunchKernelGGL(k_sssp_update, dim3(blocks_for(n_vertices, 256)), dim3(256), 0, st, label_d, d_costs, new_d, n_vertices, (bool*)pl->changed);
        hip_err_chk(hipGetLastError());
        iter++;
        changed = pl->level_end(st);
    } while (changed);
    if (iterations) *iterations = iter;
}
} // namespace

int bam_sssp(bam_array_t* edges, bam_array32_t* weights, const uint64_t* d_offsets, uint64_t n_vertices, uint64_t src, uint32_t* d_costs,
             uint32_t* iterations, void* stream)
{
    if (!edges || !weights || !d_offsets || !d_costs) return fail(EINVAL, "bam_sssp: null argument");
    if (src >= n_vertices) return fail(EINVAL, "bam_sssp: source out of range");
    if (edges->a->adt.n_elems != weights->a->adt.n_elems) return fail(EINVAL, "bam_sssp: one weight per edge");
    BAM_API_BEGIN
    sssp_run(false, edges, weights, d_offsets, n_vertices, src, d_costs, iterations, (hipStream_t)stream);
    BAM_API_END
}

int bam_sssp_float(bam_array_t* edges, bam_array32_t* weights, const uint64_t* d_offsets, uint64_t n_vertices, uint64_t src, float* d_costs,
                   uint32_t* iterations, void* stream)
{
    if (!edges || !weights || !d_offsets || !d_costs) return fail(EINVAL, "bam_sssp_float: null argument");
    if (src >= n_vertices) return fail(EINVAL, "bam_sssp_float: source out of range");
    if (edges->a->adt.n_elems != weights->a->adt.n_elems) return fail(EINVAL, "bam_sssp_float: one weight per edge");
    BAM_API_BEGIN
    sssp_run(true, edges, weights, d_offsets, n_vertices, src, (uint32_t*)d_costs, iterations, (hipStream_t)stream);
    BAM_API_END
}

} // extern "C"
