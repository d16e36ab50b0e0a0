// C-ABI of the GPU-side storage-access path: handle management over the C++
// host objects (ctrl.h, page_cache.h) and the gfx950 kernels of the array, cache,
// pattern and block benchmarks.  Kernel shapes follow the reference's benchmark
// kernels (cited per kernel); lane arithmetic is for 64-wide waves.  The graph
// kernels are in bam_graph.hip, vectoradd / reduction / scan in bam_apps.hip.
#include "bam_capi_internal.h"

std::string& bam_err()
{
    static thread_local std::string err;
    return err;
}

namespace {

/* one block of 1024 threads: *sum += all shards; shards are left zero for the next launch */
__global__ void k_fold_partials(unsigned long long* partials, unsigned long long* sum)
{
    uint64_t v = 0;
    for (uint32_t i = threadIdx.x; i < BAM_SUM_PARTIALS; i += blockDim.x) { v += partials[i]; partials[i] = 0; }
    v = wave_sum(v);
    if (bam::lane() == 0 && v) atomicAdd(sum, (unsigned long long)v);
}

/*
 * The launch's checksum folded by the last workgroup of a kernel to finish, instead of by a launch of its own.  Called by
 * all threads of every workgroup after their block_accumulate.  The partial sums are only ever touched with atomics at
 * device scope, and a wave's additions have been performed when its memory counter says so (bam::fence_meta), so the
 * workgroup that draws the last number finds them all.  The workgroups count themselves off in two steps (64 words, one per
 * residue of the workgroup number, and one word for the residues that are complete): a single word would take one atomic
 * per workgroup of the grid, all on one address.  finished[0 .. 64] are zero between launches.
 */
#define BAM_FINISHED_WORDS 65u
__device__ __forceinline__ void fold_by_last_block(unsigned long long* partials, unsigned long long* sum, uint32_t* finished)
{
    __shared__ uint32_t last;
    bam::fence_meta();
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t is_last = 0;
        const uint32_t r = blockIdx.x & 63u, with_r = (gridDim.x - r + 63u) / 64u, residues = gridDim.x < 64u ? gridDim.x : 64u;
        if (__hip_atomic_fetch_add(finished + 1 + r, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1 == with_r) {
            __hip_atomic_store(finished + 1 + r, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            bam::fence_meta();
            if (__hip_atomic_fetch_add(finished, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1 == residues) {
                __hip_atomic_store(finished, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                is_last = 1;
            }
        }
        last = is_last;
    }
    __syncthreads();
    if (!last) return;
    uint64_t v = 0;
    for (uint32_t i = threadIdx.x; i < BAM_SUM_PARTIALS; i += blockDim.x) {
        const unsigned long long x = __hip_atomic_load(partials + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (x) { v += x; __hip_atomic_store(partials + i, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
    }
    v = wave_sum(v);
    if (bam::lane() == 0 && v) atomicAdd(sum, (unsigned long long)v);
}
/* the word through which the first of two launches tells the second whether it left anything: the number of the call when it
 * did (the host counts the calls per array), so that nobody has to clear it */
#define BAM_LEFT_WORD 96u
/* by a whole wave that left something; the word is written only while it does not say so yet (thousands of waves storing to
 * one address take the device 12 ns a time, one after the other) */
__device__ __forceinline__ void note_work_left(uint32_t* finished, const uint32_t call)
{
    if (bam::lane() == bam::first_lane(bam::active_mask()) && __hip_atomic_load(finished + BAM_LEFT_WORD, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != call)
        __hip_atomic_store(finished + BAM_LEFT_WORD, call, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---- array benchmark (benchmarks/array/main.cu:43-65), with a checksum ----
__global__ void k_array_read(array_d_t<uint64_t>* dr, uint64_t n_reqs, const uint64_t* assignment, uint64_t stride, uint64_t reqs_per_thread, unsigned long long* sum)
{
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint64_t v = 0;
    /* thread t reads element t * stride: where a wave covers only a few pages (less than 32 KiB) they are touched ahead in
     * windows, or every wave would ask the store for its one page or its few by itself */
    const uint64_t first_tid = tid - threadIdx.x % BAM_WAVE_SIZE;
    if (!assignment && stride && first_tid < n_reqs && BAM_WAVE_SIZE * stride * sizeof(uint64_t) < 32768)
        touch_ahead(dr, first_tid * stride, (n_reqs - 1) * stride + 1, BAM_WAVE_SIZE * stride);
    if (tid < n_reqs) {
        const uint64_t idx = assignment ? assignment[tid] : tid * stride;
        for (uint64_t i = 0; i < reqs_per_thread; i++) v += (*dr)[idx];
    }
    block_accumulate(sum, v);
}

/* the same sum for a launch of scattered requests, BAM_READS_PER_LANE of them per thread a quarter of the launch apart
 * (request t + j * threads for j = 0 .. 3), read side by side (array_d_t::seq_read_n): what the lanes of a wave ask for
 * together is as scattered as with one request per thread, and each lane keeps four requests in flight instead of one */
#define BAM_READS_PER_LANE 4
__global__ void k_array_read_n_whole(array_d_t<uint64_t>* dr, uint64_t n_reqs, const uint64_t* __restrict__ assignment, uint64_t threads, unsigned long long* sum)
{
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t idx[BAM_READS_PER_LANE];
    bool want[BAM_READS_PER_LANE];
    uint64_t out[BAM_READS_PER_LANE];
#pragma unroll
    for (int j = 0; j < BAM_READS_PER_LANE; j++) {
        const uint64_t t = tid + (uint64_t)j * threads;
        want[j] = tid < threads && t < n_reqs;
        idx[j] = want[j] ? assignment[t] : 0;
    }
    dr->seq_read_n(idx, want, out);
    uint64_t v = 0;
#pragma unroll
    for (int j = 0; j < BAM_READS_PER_LANE; j++) v += want[j] ? out[j] : 0;
    block_accumulate(sum, v);
}

/*
 * A launch of scattered requests in two launches (arrays of one range).  The first, this kernel: thread t takes requests
 * t, t + threads, ... (N at a time for `rounds` rounds, `threads` a multiple of 64) and reads those whose page is resident, without a reference
 * (array_d_t::seq_read_n_resident); bit t of missed[] says whether request t is left for the second launch
 * (k_array_read_deferred).  No call, no atomic but the checksum's and the counters', no stack: a kernel that can miss
 * carries the registers of the miss path (four waves per SIMD) and its frame in scratch memory through every read.  The
 * last workgroup folds the checksum of what was read; the second launch adds what it reads.
 */
template <int N>
__global__ __launch_bounds__(256) void k_array_read_n(array_d_t<uint64_t>* dr, uint64_t n_reqs, const uint64_t* __restrict__ assignment, uint64_t threads, uint32_t rounds,
                                                      unsigned long long* partials, uint64_t* missed, unsigned long long* sum, uint32_t* finished, uint32_t call)
{
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    bam::range_view<uint64_t> view;
    view.load(dr->d_ranges);
    uint64_t v = 0, any_left = 0;
    /* thread t takes requests t + k * threads, k = 0 .. N * rounds - 1, N at a time: what a wave, a workgroup and the launch
     * do once (the range's descriptor, the counters, the checksum) is shared by more reads the more rounds there are */
    /* the indices of a round are asked for a round ahead: a read is four trips to memory one after the other (index,
     * descriptor, element, descriptor again), and this takes the first out of the chain (44 against 41 thousand million reads
     * a second with eight reads per lane).  Every lane loads (one without a request the first index): N loads side by side,
     * no branch around any.  Read once: not to be kept in the L2 the descriptors live in */
    size_t ahead[N];
#pragma unroll
    for (int j = 0; j < N; j++) {
        const uint64_t t = tid + (uint64_t)j * threads;
        ahead[j] = __builtin_nontemporal_load(assignment + (tid < threads && t < n_reqs ? t : 0));
    }
    for (uint32_t r = 0; r < rounds; r++) {
        size_t idx[N];
        bool want[N], got[N];
        uint64_t out[N];
#pragma unroll
        for (int j = 0; j < N; j++) {
            const uint64_t t = tid + (uint64_t)(r * N + j) * threads;
            want[j] = tid < threads && t < n_reqs;
            idx[j] = ahead[j];
        }
        if (r + 1 < rounds) {
#pragma unroll
            for (int j = 0; j < N; j++) {
                const uint64_t t = tid + (uint64_t)((r + 1) * N + j) * threads;
                ahead[j] = __builtin_nontemporal_load(assignment + (tid < threads && t < n_reqs ? t : 0));
            }
        }
        dr->template seq_read_n_resident<N, true>(idx, want, out, got, view);
        /* the N words of notes of the round with one store: lane j writes the j-th */
        uint64_t mine = 0;
#pragma unroll
        for (int j = 0; j < N; j++) {
            v += got[j] ? out[j] : 0;
            const uint64_t m = bam::ballot(want[j] & !got[j]);
            if (bam::lane() == (uint32_t)j) mine = m;
            any_left |= m;
        }
        if (bam::lane() < (uint32_t)N && tid - bam::lane() < threads)
            missed[(tid - bam::lane() + (uint64_t)(r * N + bam::lane()) * threads) / BAM_WAVE_SIZE] = mine;
    }
    view.flush_stats();
    if (any_left) note_work_left(finished, call);
    block_accumulate(partials, v);
    fold_by_last_block(partials, sum, finished);
}

/*
 * The second launch: the requests the first one left, one per lane through array_d_t::operator[], which has the miss
 * path.  A wave takes `words` words of missed[] at a time (1 to 16, a power of two: lane l looks after `words` bits),
 * lines the requests noted there up in LDS and reads them 64 at a time: whatever the share of misses, the batches of
 * commands that go to the store are whole waves' worth.  The last workgroup to finish adds the checksum of these reads
 * to the first launch's.  When the first launch left nothing (it says so in a word of its own) this one ends at once.
 */
#define BAM_DEFER_MAX_WORDS 16u
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4))) void k_array_read_deferred(array_d_t<uint64_t>* dr, uint64_t n_reqs, const uint64_t* __restrict__ assignment, const uint64_t* missed,
                                                             uint64_t n_words, uint32_t words, unsigned long long* partials, unsigned long long* sum, uint32_t* finished, uint32_t call)
{
    __shared__ uint16_t ids[256 / BAM_WAVE_SIZE][BAM_DEFER_MAX_WORDS * BAM_WAVE_SIZE];
    if (__hip_atomic_load(finished + BAM_LEFT_WORD, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != call) return;      /* nothing was left */
    const uint32_t lane = bam::lane(), w_in_block = threadIdx.x / BAM_WAVE_SIZE;
    const uint64_t gwave = ((uint64_t)blockIdx.x * blockDim.x + threadIdx.x) / BAM_WAVE_SIZE, n_gwaves = (uint64_t)gridDim.x * blockDim.x / BAM_WAVE_SIZE;
    const uint64_t n_chunks = (n_words + words - 1) / words;
    uint64_t v = 0;
    bool any = false;
    for (uint64_t c = gwave; c < n_chunks; c += n_gwaves) {
        /* lane l: bits [l * words, (l + 1) * words) of the chunk's 64 * words */
        const uint32_t bit0 = lane * words;
        const uint64_t word = c * words + bit0 / 64;
        const uint32_t seg = word < n_words ? (uint32_t)((missed[word] >> (bit0 % 64)) & ((1u << words) - 1u)) : 0u;
        uint32_t incl = bam::popc((uint64_t)seg);
        const uint32_t mine = incl;
#pragma unroll
        for (uint32_t o = 1; o < BAM_WAVE_SIZE; o <<= 1) {
            const uint32_t u = bam::shfl(incl, lane >= o ? lane - o : lane);
            if (lane >= o) incl += u;
        }
        const uint32_t total = bam::bcast(incl, BAM_WAVE_SIZE - 1);
        if (!total) continue;
        any = true;
        uint32_t at = incl - mine;
        for (uint32_t m = seg; m; m &= m - 1) ids[w_in_block][at++] = (uint16_t)(bit0 + (uint32_t)__builtin_ctz(m));
        /* written and read by the lanes of one wave, which runs its LDS operations in order */
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        for (uint32_t b = 0; b < total; b += BAM_WAVE_SIZE) {
            if (b + lane < total) {
                const uint64_t t = c * words * BAM_WAVE_SIZE + ids[w_in_block][b + lane];
                if (t < n_reqs) v += (*dr)[assignment[t]];
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }
    if (bam::ballot(any)) block_accumulate(partials, v);
    fold_by_last_block(partials, sum, finished);
}

/* thread t hands out the element it read instead of adding it to a sum */
__global__ void k_array_gather(array_d_t<uint64_t>* dr, uint64_t n_reqs, const uint64_t* assignment, uint64_t stride, uint64_t* out)
{
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (tid < n_reqs) out[tid] = (*dr)[assignment ? assignment[tid] : tid * stride];
}

/*
 * The same read pattern through the other access routes of array_d_t:
 *   1  get_raw / release_raw            (the raw page handed out, lanes on one page share the references)
 *   2  get_page_gid + acquire_page_ + release_page   (per-thread, no coalescing)
 *   3  acquire_page / release_page      (coalesced, page kept while in use)
 *   4  bam_ptr                          (per-thread cached page)
 *   5  memcpy                           (wave-cooperative copy of up to `span` elements starting at the wave's index;
 *                                        one request per wave, the copied elements are summed)
 *   6  bam_ptr_tlb over a 64-entry tlb in LDS, shared by the workgroup
 *   7  bafs_ptr                         (pointer arithmetic + dereference)
 */
template <int API>
__global__ void k_array_read_via(array_d_t<uint64_t>* dr, uint64_t n_reqs, const uint64_t* assignment, uint64_t span, uint64_t* scratch, unsigned long long* sum)
{
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint64_t v = 0;
    if (API == 5) {
        const uint64_t wave = tid / BAM_WAVE_SIZE;
        if (wave < n_reqs) {
            const uint64_t idx = assignment ? assignment[wave] : wave * span;
            uint64_t* dst = scratch + wave * span;
            for (uint64_t k = bam::lane(); k < span; k += BAM_WAVE_SIZE) dst[k] = 0;
            dr->memcpy(idx, span, dst);
            for (uint64_t k = bam::lane(); k < span; k += BAM_WAVE_SIZE) v += dst[k];
        }
    } else if (API == 6) {
        typedef tlb<uint64_t, 64, simt::thread_scope_device, SHARED_> tlb_t;
        __shared__ tlb_t table;
        table.init(dr);
        __syncthreads();
        if (tid < n_reqs) {
            const uint64_t idx = assignment ? assignment[tid] : tid * span;
            bam_ptr_tlb<uint64_t, 64, simt::thread_scope_device, SHARED_> ptr(dr, &table);
            const bam_ptr_tlb<uint64_t, 64, simt::thread_scope_device, SHARED_>& cptr = ptr;
            v = cptr[idx];
            ptr.fini();
        }
        __syncthreads();
        table.fini();
    } else if (tid < n_reqs) {
        const uint64_t idx = assignment ? assignment[tid] : tid * span;
        if (API == 7) {
            bafs_ptr<uint64_t> p(dr, 0);
            bafs_ptr<uint64_t> q = p + idx;
            v = *q;
            if (q[0] != v || !(q - idx == p)) v = 0;
        } else if (API == 1) {
            returned_cache_page_t<uint64_t> pg = dr->get_raw(idx);
            if (pg.addr) v = bam::ld_payload(pg.addr + pg.offset);      /* no address after a wait that was given up */
            dr->release_raw(idx);
        } else if (API == 2) {
            range_d_t<uint64_t>* r;
            size_t page, gid, start, end;
            data_page_t* dp;
            dr->get_page_gid(idx, r, page, gid);
            const uint64_t* base = (const uint64_t*)dr->acquire_page_(idx, dp, start, end, r, page);
            if (base && idx >= start && idx < end && gid == r->get_global_address(page)) v = bam::ld_payload(base + (idx - start));
            if (r) r->release_page(page, 1, false);
        } else if (API == 3) {
            size_t start, end;
            data_page_t* dp;
            int64_t r;
            const uint64_t* base = (const uint64_t*)dr->acquire_page(idx, dp, start, end, r);
            if (base) v = bam::ld_payload(base + (idx - start));
            dr->release_page(dp, r, idx, false);
        } else {
            bam_ptr<uint64_t> ptr(dr);
            const bam_ptr<uint64_t>& cptr = ptr;
            v = cptr[idx];
        }
    }
    block_accumulate(sum, v);
}

__global__ void k_array_write(array_d_t<uint64_t>* dr, uint64_t n_reqs, const uint64_t* assignment, uint64_t stride, const uint64_t* values)
{
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (tid < n_reqs) (*dr)(assignment ? assignment[tid] : tid * stride, values[tid]);
}

/*
 * Read-modify-write through the three routes the reference offers for it (include/page_cache.h:1647 AtomicAdd, :467 memref,
 * :478 non-const operator[] used as an lvalue): element assignment[t] += values[t], old[t] = what the element held before.
 *   0  array_d_t::AtomicAdd                      (any indices, colliding ones included)
 *   1  atomicAdd on the address bam_ptr::memref hands out   (any indices)
 *   2  ptr[i] += v through a non-const bam_ptr   (a plain read and write: the indices of one launch must differ)
 */
template <int API>
__global__ void k_array_update(array_d_t<uint64_t>* dr, uint64_t n_reqs, const uint64_t* assignment, const uint64_t* values, uint64_t* old)
{
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (tid >= n_reqs) return;
    const uint64_t idx = assignment[tid], val = values[tid];
    uint64_t before = 0;
    if (API == 0) before = dr->AtomicAdd(idx, val);
    else {
        bam_ptr<uint64_t> ptr(dr);
        if (API == 1) {
            unsigned long long* p = (unsigned long long*)ptr.memref(idx);
            if (p) before = atomicAdd(p, (unsigned long long)val);
        } else {
            before = ptr[idx];
            ptr[idx] += val;
        }
    }
    if (old) old[tid] = before;
}

/* lane l encodes the submission entry of command (cid + l) for block (lba + l) the way the miss path does (nvm_cmd_header,
 * nvm_cmd_data_ptr, nvm_cmd_rw_blks, and nvm_cmd_seal with ticket + l on top when asked): 64 entries of 16 dwords */
__global__ void k_sqe_image(uint16_t cid, uint8_t opcode, uint32_t nsid, uint64_t prp1, uint64_t prp2, uint64_t lba, uint16_t n_blocks, int seal, uint32_t ticket,
                            uint32_t* out)
{
    const uint32_t l = bam::lane();
    nvm_cmd_t cmd;
#pragma unroll
    for (int i = 0; i < 16; i++) cmd.dword[i] = 0;
    nvm_cmd_header(&cmd, (uint16_t)(cid + l), opcode, nsid);
    nvm_cmd_data_ptr(&cmd, prp1, prp2);
    nvm_cmd_rw_blks(&cmd, lba + l, n_blocks);
    if (seal) nvm_cmd_seal(&cmd, ticket + l);
    for (int i = 0; i < 16; i++) out[l * 16 + i] = cmd.dword[i];
}

/* the pages [first, first + n) of a range (n <= 64), one per lane: those that are not resident are taken and dropped again as
 * one batch.  A function of its own: the view of the range it works on lives in registers only while it runs. */
__device__ __attribute__((noinline)) void stream_touch(range_d_t<uint64_t>* r, const uint64_t first, const uint64_t n)
{
    bam::range_view<uint64_t> view;
    view.load(r);
    auto touch = [](uint32_t) { return true; };
    const uint64_t lane = bam::lane(), epp = r->n_elems_per_page;
    const uint64_t page = view.page_of((first + (lane < n ? lane : 0)) * epp);
    const bool take = lane < n && page_absent(view, page);
    if (bam::ballot(take)) view.template acquire_helped<true>(page, take, false, touch, touch);
    view.n_access = view.n_hit = 0;
}

// ---- cache / pattern benchmark (benchmarks/cache/main.cu:44-114): a wave streams whole pages ----
/* the fetch waves of the streaming modes for data that is not resident: the runs of the streaming waves laid end to end,
 * 64 pages per batch (lane l of batch b looks after page (64 b + l) % n_pages_per_wave of streaming wave (64 b + l) /
 * n_pages_per_wave), never further ahead of the waves that have finished than `lead_elems` pages */
__device__ __forceinline__ void stream_fetch_role(array_d_t<uint64_t>* dr, const uint64_t n_waves, const uint64_t ppw, const uint64_t* assignment, const fetch_plan& fp)
{
    if (dr->n_ranges != 1) return;
    bam::range_view<uint64_t> view;
    view.load(dr->d_ranges);
    view.read_ahead = true;
    const uint64_t epp = dr->d_ranges->n_elems_per_page;
    const uint64_t fwave = ((uint64_t)blockIdx.x * blockDim.x + threadIdx.x) / BAM_WAVE_SIZE, n_fwaves = (uint64_t)fp.blocks * blockDim.x / BAM_WAVE_SIZE;
    const uint64_t total = n_waves * ppw, n_batches = (total + BAM_WAVE_SIZE - 1) / BAM_WAVE_SIZE;
    auto touch = [](uint32_t) { return true; };
    for (uint64_t b = fwave; b < n_batches; b += n_fwaves) {
        const uint64_t first_wave = b * BAM_WAVE_SIZE / ppw;
        uint32_t spins = 0;
        while (first_wave * ppw > __hip_atomic_load(fp.done, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) * ppw + fp.lead_elems) {
            if (++spins >= fp.spin_limit) return;
            __builtin_amdgcn_s_sleep(64);
        }
        const uint64_t at = b * BAM_WAVE_SIZE + bam::lane();
        const uint64_t cw = at < total ? at / ppw : 0;
        const uint64_t elem = ((assignment ? assignment[cw] : cw * ppw) + at % ppw) * epp;
        const bool in = at < total && elem < dr->n_elems;
        const uint64_t page = view.page_of(in ? elem : 0);
        const bool take = in && page_absent(view, page);
        if (bam::ballot(take)) view.acquire_helped(page, take, false, touch, touch);
        view.n_access = view.n_hit = 0;
    }
}

/*
 * One page of a streaming wave, every element read once and added up: lane l reads elements l, l + 64, ... of the page
 * whose first element is `first`.  ELEM: through array_d_t::operator[] per element (the eight elements a lane reads of a
 * page side by side, array_d_t::seq_read_n); otherwise through bam_ptr per element.  DEFER: the page is read only if it is
 * resident; true (for the whole wave) if it was not, and then nothing of it is counted, neither in `v` nor in the views.
 */
template <bool ELEM, bool DEFER, typename PTR>
__device__ __forceinline__ bool stream_page(array_d_t<uint64_t>* dr, PTR& ptr, bam::range_view<uint64_t>& elem_view, const uint64_t first, const uint64_t epp,
                                            const uint32_t lane, uint64_t& v)
{
    const uint64_t start_idx = first + lane;
    uint64_t sum = 0;
    bool miss = false;
    [[maybe_unused]] uint32_t na = 0, nh = 0;
    if constexpr (DEFER) { if (ELEM) { na = elem_view.n_access; nh = elem_view.n_hit; } else ptr.counted(na, nh); }
    if constexpr (ELEM) {
        for (uint64_t j = 0; j < epp; j += 8 * BAM_WAVE_SIZE) {
            size_t at[8];
            bool want[8];
            uint64_t x[8];
#pragma unroll
            for (int u = 0; u < 8; u++) { at[u] = start_idx + j + u * BAM_WAVE_SIZE; want[u] = j + u * BAM_WAVE_SIZE + lane < epp; }
            if constexpr (DEFER) {
                bool got[8];
                dr->seq_read_n_resident(at, want, x, got, elem_view);
#pragma unroll
                for (int u = 0; u < 8; u++) miss = miss || (want[u] && !got[u]);
            } else
                dr->seq_read_n(at, want, x, elem_view);
#pragma unroll
            for (int u = 0; u < 8; u++) sum += want[u] ? x[u] : 0;
        }
    } else {
        /* The page changes in one place, update_page for the lane's first element of the stretch; when the lane's other
         * elements lie in the window that opens, as they do unless a range ends inside the page, all eight are asked for
         * side by side: the window test of an element needs nothing that an earlier load brings. */
        for (uint64_t j = 0; j < epp; j += 8 * BAM_WAVE_SIZE) {
            const uint64_t i0 = start_idx + j;
            const uint32_t n_here = (uint32_t)((epp - j + BAM_WAVE_SIZE - 1) / BAM_WAVE_SIZE < 8 ? (epp - j + BAM_WAVE_SIZE - 1) / BAM_WAVE_SIZE : 8);
            const uint64_t i_last = i0 + (uint64_t)(n_here - 1) * BAM_WAVE_SIZE;
            if (!ptr.covers(i0, i_last)) ptr.update_page(i0);
            if constexpr (DEFER) { if (bam::ballot(ptr.missed)) break; }
            uint64_t acc = 0;
            if (ptr.covers(i0, i_last)) {
                uint64_t x[8];
                if (n_here == 8) ptr.template peek_n<8>(i0, BAM_WAVE_SIZE, x);
                else {
#pragma unroll
                    for (int u = 0; u < 8; u++) x[u] = (uint32_t)u < n_here ? (uint64_t)ptr.peek(i0 + (uint64_t)u * BAM_WAVE_SIZE) : 0;
                }
                acc = ((x[0] + x[1]) + (x[2] + x[3])) + ((x[4] + x[5]) + (x[6] + x[7]));
            } else {
#pragma unroll 1
                for (uint32_t u = 0; u < n_here; u++) acc += (uint64_t)ptr[i0 + (uint64_t)u * BAM_WAVE_SIZE];
            }
            sum += acc;
        }
        /* a pointer that holds no reference: what it read of the page counts if the page is still what it was */
        if constexpr (DEFER) { ptr.still(); miss = ptr.missed; ptr.missed = false; }
    }
    if constexpr (DEFER) {
        if (bam::ballot(miss)) {
            if (ELEM) { elem_view.n_access = na; elem_view.n_hit = nh; } else ptr.set_counted(na, nh);
            return true;
        }
    }
    v += sum;
    return false;
}

template <int MODE>
__device__ __forceinline__ void cache_stream_body(array_d_t<uint64_t>* dr, uint64_t n_waves, uint64_t n_pages_per_wave, const uint64_t* assignment, unsigned long long* sum,
                                                  const fetch_plan fp = fetch_plan{nullptr, 0, 0, 0, 0})
{
    if (MODE >= 3 && fp.done && blockIdx.x < fp.blocks) {
        stream_fetch_role(dr, n_waves, n_pages_per_wave, assignment, fp);
        return;
    }
    const uint64_t tid = (uint64_t)(blockIdx.x - (MODE >= 3 && fp.done ? fp.blocks : 0u)) * blockDim.x + threadIdx.x;
    /* the same for all lanes of a wave, and said so: what follows from it (first page, loop counts) then lives in scalar registers */
    const uint64_t wave = bam::first(tid / BAM_WAVE_SIZE), lane = tid % BAM_WAVE_SIZE;
    uint64_t v = 0;
    if (wave < n_waves) {
        range_d_t<uint64_t>* r0 = dr->d_ranges;
        const uint64_t epp = bam::first(r0->n_elems_per_page);
        const uint64_t start_page = bam::first(assignment ? assignment[wave] : wave * n_pages_per_wave);
        if (MODE == 2) {
            /*
             * Descriptor read once.  Pages are taken sixteen at a time: lane l of the wave asks for page l of the
             * batch, so the sixteen reference counts go out as one vector atomic; then the whole wave streams the
             * sixteen pages, eight 8-byte loads in flight per lane, and the sixteen references are dropped together.
             */
            bam::range_view<uint64_t> view;
            view.load(r0);
            const uint32_t n8 = view.page_size / 8;
            uint64_t a0 = 0, a1 = 0;
            for (uint64_t p0 = 0; p0 < n_pages_per_wave; p0 += 16) {
                const uint32_t nb = (uint32_t)(n_pages_per_wave - p0 < 16 ? n_pages_per_wave - p0 : 16);
                uint32_t slot = BAM_NO_SLOT;
                const uint64_t page = view.page_of((start_page + p0 + (lane < nb ? lane : 0)) * epp);
                if (lane < nb) {
                    auto keep = [&](uint32_t s_) { slot = s_; return false; };
                    view.acquire<true>(page, false, keep, keep);
                }
                /* a page whose wait was given up (the controller is marked aborted) has no slot: nothing of the batch is read */
                const bool all_in = bam::ballot(lane < nb && slot == BAM_NO_SLOT) == 0;
                uint32_t k = all_in ? 0 : nb;
                if (n8 == 8 * BAM_WAVE_SIZE)            /* 4 KiB pages: two at a time */
                    for (; k + 1 < nb; k += 2) {
                        uint64_t x[16];
                        bam::ld_payload_stream16((const uint64_t*)view.slot_addr(bam::bcast(slot, k)) + lane,
                                                 (const uint64_t*)view.slot_addr(bam::bcast(slot, k + 1)) + lane, x);
                        a0 += ((x[0] + x[2]) + (x[4] + x[6])) + ((x[8] + x[10]) + (x[12] + x[14]));
                        a1 += ((x[1] + x[3]) + (x[5] + x[7])) + ((x[9] + x[11]) + (x[13] + x[15]));
                    }
                for (; k < nb; k++) {
                    const uint64_t* base = (const uint64_t*)view.slot_addr(bam::bcast(slot, k));
                    for (uint32_t i = (uint32_t)lane; i < n8; i += 8 * BAM_WAVE_SIZE) {
                        uint64_t x[8];
                        if (i + 7 * BAM_WAVE_SIZE < n8) bam::ld_payload_stream8(base + i, x);
                        else {
#pragma unroll
                            for (int j = 0; j < 8; j++) x[j] = i + j * BAM_WAVE_SIZE < n8 ? bam::ld_payload(base + i + j * BAM_WAVE_SIZE) : 0;
                        }
                        a0 += x[0] + x[2] + x[4] + x[6];
                        a1 += x[1] + x[3] + x[5] + x[7];
                    }
                }
                if (lane < nb) view.release(page, false);
            }
            v += a0 + a1;
            view.flush_stats();
        } else {
            bam_ptr<uint64_t> ptr(dr);
            bam::range_view<uint64_t> elem_view;            /* modes 0 and 4: the descriptor read once, the accesses counted here */
            if ((MODE == 0 || MODE == 4) && dr->n_ranges == 1) elem_view.load(r0);
            /* a wave reads its pages one after the other: those of the next stretch that are not resident are touched
             * together, one page per lane, so that a cold run asks the store for a batch per stretch and not for a page
             * per trip (1.5 M pages/s otherwise); on a resident cache this costs one look at a state word per page */
            /* (modes 3 and 4: the helper needs more registers than the kernels themselves, which costs them a third of the
             * waves they run with on a resident cache, hence modes 0 and 1 without) */
            const uint32_t reach = MODE < 3 || dr->n_ranges != 1 ? 1 : (uint32_t)(r0->cache.n_pages >> 6 > BAM_WAVE_SIZE ? BAM_WAVE_SIZE : r0->cache.n_pages >> 6);
            for (uint64_t p = 0; p < n_pages_per_wave; p++) {
                if (MODE >= 3 && reach >= 2 && p % reach == 0) stream_touch(r0, start_page + p, n_pages_per_wave - p < reach ? n_pages_per_wave - p : reach);
                /* the lane number worked out afresh at every page (two instructions): held in a register across the
                 * loop it is the value the compiler parks in scratch memory, and a reload with its wait costs more */
                uint32_t lane_now;
                asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane_now));
                stream_page<MODE == 0 || MODE == 4, false>(dr, ptr, elem_view, (start_page + p) * epp, epp, lane_now, v);
            }
            elem_view.flush_stats();
        }
        if (MODE >= 3 && fp.done && lane == 0) __hip_atomic_fetch_add(fp.done, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    block_accumulate(sum, v);
}

/* one kernel per mode; the page-wise one has a name of its own because it is the one the hit-path roofline is quoted on */
/* mode 1 is held to the registers of four waves per SIMD (128; left alone the compiler takes 130): it fits, without a
 * spill, since the lane number is worked out per page rather than kept */
template <int MODE>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(MODE == 1 ? 4 : 1))) void k_cache_stream_whole(array_d_t<uint64_t>* dr, uint64_t n_waves, uint64_t n_pages_per_wave, const uint64_t* assignment, unsigned long long* sum)
{
    cache_stream_body<MODE>(dr, n_waves, n_pages_per_wave, assignment, sum);
}
/* modes 3 and 4 with fetch waves at the front of the grid */
template <int MODE>
__global__ __launch_bounds__(256) void k_cache_stream_fetched(array_d_t<uint64_t>* dr, uint64_t n_waves, uint64_t n_pages_per_wave, const uint64_t* assignment, unsigned long long* sum,
                                                             const fetch_plan fp)
{
    cache_stream_body<MODE>(dr, n_waves, n_pages_per_wave, assignment, sum, fp);
}
__global__ __launch_bounds__(256) void k_cache_stream_pages(array_d_t<uint64_t>* dr, uint64_t n_waves, uint64_t n_pages_per_wave, const uint64_t* assignment, unsigned long long* sum)
{
    cache_stream_body<2>(dr, n_waves, n_pages_per_wave, assignment, sum);
}

/*
 * Modes 0 and 1 in two launches (arrays of one range).  The first, this kernel, is the reference's kernel
 * (benchmarks/cache/main.cu:44-114: a wave per run of pages, every element through bam_ptr or operator[]) with pointers
 * that do not load: a page that is not resident is noted in deferred[wave * n_pages_per_wave + p] and left to the second
 * launch (k_cache_stream_deferred), which has the miss path.  A kernel that can miss carries the registers and the stack of
 * the miss path through every page visit (four waves per SIMD, a frame in scratch memory); this one has neither.
 */
template <int MODE>
__global__ __launch_bounds__(256) void k_cache_stream(array_d_t<uint64_t>* dr, uint64_t n_waves, uint64_t n_pages_per_wave, const uint64_t* assignment, unsigned long long* partials,
                                                      uint8_t* deferred, unsigned long long* sum, uint32_t* finished, uint32_t call)
{
    static_assert(MODE == 0 || MODE == 1, "the page-wise mode and the fetching modes are kernels of their own");
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint64_t wave = bam::first(tid / BAM_WAVE_SIZE);
    const uint32_t lane = bam::lane();
    uint64_t v = 0;
    if (wave < n_waves) {
        range_d_t<uint64_t>* r0 = dr->d_ranges;
        const uint64_t epp = bam::first(r0->n_elems_per_page);
        const uint64_t start_page = bam::first(assignment ? assignment[wave] : wave * n_pages_per_wave);
        bam_ptr<uint64_t, true> ptr(dr);
        bam::range_view<uint64_t> elem_view;
        if (MODE == 0) elem_view.load(r0);
        uint64_t later = 0;                 /* bit p % 64: page p is left to the second launch (the same in every lane) */
        for (uint64_t p = 0; p < n_pages_per_wave; p++) {
            if (stream_page<MODE == 0, true>(dr, ptr, elem_view, (start_page + p) * epp, epp, lane, v)) later |= 1ull << (p & 63u);
            if ((p & 63u) == 63u || p + 1 == n_pages_per_wave) {
                /* the notes of up to 64 pages with one store, a byte per lane */
                const uint64_t first = p & ~63ull;
                if (first + lane <= p) deferred[wave * n_pages_per_wave + first + lane] = (uint8_t)((later >> lane) & 1u);
                if (later) note_work_left(finished, call);
                later = 0;
            }
        }
        elem_view.flush_stats();
    }
    block_accumulate(partials, v);
    fold_by_last_block(partials, sum, finished);
}

/*
 * The second launch: the pages the first one noted, read by waves that can load them.  A wave looks at 64 notes at a
 * time; the pages it finds noted and not resident it asks for as one batch (one page per lane, taken and dropped again,
 * as many at a time as a 64th of the cache allows), then it reads them one after the other as the one-launch kernel
 * would.  On a resident cache the first launch noted nothing, says so, and this one ends at once.  The last workgroup
 * to finish adds the checksum of what was read here to the first launch's.
 */
template <int MODE>
__global__ __launch_bounds__(256) void k_cache_stream_deferred(array_d_t<uint64_t>* dr, uint64_t n_waves, uint64_t n_pages_per_wave, const uint64_t* assignment,
                                                               unsigned long long* partials, const uint8_t* deferred, unsigned long long* sum, uint32_t* finished, uint32_t call)
{
    if (__hip_atomic_load(finished + BAM_LEFT_WORD, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != call) return;      /* nothing was noted */
    const uint64_t gwave = ((uint64_t)blockIdx.x * blockDim.x + threadIdx.x) / BAM_WAVE_SIZE, n_gwaves = (uint64_t)gridDim.x * blockDim.x / BAM_WAVE_SIZE;
    const uint64_t total = n_waves * n_pages_per_wave, n_chunks = (total + BAM_WAVE_SIZE - 1) / BAM_WAVE_SIZE;
    uint64_t v = 0;
    bool any = false;
    for (uint64_t c = gwave; c < n_chunks; c += n_gwaves) {
        const uint64_t q = c * BAM_WAVE_SIZE + bam::lane();
        const bool noted = q < total && deferred[q] != 0;
        const uint64_t m = bam::ballot(noted);
        if (!m) continue;
        any = true;
        range_d_t<uint64_t>* r0 = dr->d_ranges;
        const uint64_t epp = bam::first(r0->n_elems_per_page);
        const uint64_t cw = noted ? q / n_pages_per_wave : 0;
        const uint64_t page = noted ? (assignment ? assignment[cw] : cw * n_pages_per_wave) + q % n_pages_per_wave : 0;
        {
            bam::range_view<uint64_t> view;
            view.load(r0);
            const uint32_t reach = (uint32_t)(r0->cache.n_pages >> 6 > BAM_WAVE_SIZE ? BAM_WAVE_SIZE : r0->cache.n_pages >> 6);
            auto touch = [](uint32_t) { return true; };
            const bool in = noted && page * epp < dr->n_elems;
            const uint64_t pg = view.page_of(in ? page * epp : 0);
            const bool absent = in && page_absent(view, pg);
            if (reach >= 2)
                for (uint32_t b = 0; b < BAM_WAVE_SIZE; b += reach) {
                    const bool take = absent && bam::lane() >= b && bam::lane() < b + reach;
                    if (bam::ballot(take)) view.template acquire_helped<true>(pg, take, false, touch, touch);
                }
            view.n_access = view.n_hit = 0;
        }
        bam_ptr<uint64_t> ptr(dr);
        bam::range_view<uint64_t> elem_view;
        if (MODE == 0) elem_view.load(r0);
        for (uint64_t mm = m; mm; mm &= mm - 1) {
            const uint64_t first = bam::bcast(page, bam::first_lane(mm)) * epp;
            stream_page<MODE == 0, false>(dr, ptr, elem_view, first, epp, bam::lane(), v);
        }
        elem_view.flush_stats();
    }
    if (bam::ballot(any)) block_accumulate(partials, v);
    fold_by_last_block(partials, sum, finished);
}

// ---- raw block benchmark (benchmarks/block/main.cu:99-200) ----
__global__ void k_block_io(Controller** ctrls, page_cache_d_t* pc, uint32_t req_size, uint64_t n_reqs, const uint64_t* lbas, int write, int queue_policy)
{
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint64_t act = bam::active_mask();
    const uint32_t leader = bam::first_lane(act);
    uint32_t ctrl = 0, queue = 0;
    if (bam::lane() == leader) {
        ctrl = pc->n_ctrls == 1 ? 0 : (uint32_t)(pc->ctrl_counter->fetch_add(1, simt::memory_order_relaxed) % pc->n_ctrls);
        queue = queue_policy == 0 ? get_smid() % ctrls[ctrl]->n_qps
                                  : (uint32_t)(ctrls[ctrl]->queue_counter.fetch_add(1, simt::memory_order_relaxed) % ctrls[ctrl]->n_qps);
    }
    ctrl = bam::bcast(ctrl, leader);
    queue = bam::bcast(queue, leader);
    if (tid < n_reqs) {
        QueuePair* qp = ctrls[ctrl]->d_qps + queue;
        const uint64_t start_block = lbas ? lbas[tid] : (tid * req_size) >> qp->block_size_log;
        const uint64_t n_blocks = req_size >> qp->block_size_log;
        if (write) write_data(pc, qp, start_block, n_blocks, tid);
        else read_data(pc, qp, start_block, n_blocks, tid);
    }
}

/*
 * One command per thread, put together by the thread itself from the per-thread queue operations, as the reference's
 * read_data does it (include/page_cache.h:2009-2054: get_cid, the entry, sq_enqueue, cq_poll, cq_dequeue, put_cid), the
 * controller addressing cache slot t directly.  Thread t uses queue pair t mod n_qps, so the lanes of a wave are on as many
 * different queue pairs as there are; the calls take the lanes of one queue at a time.
 */
__global__ void k_block_io_per_thread(Controller** ctrls, page_cache_d_t* pc, uint32_t req_size, uint64_t n_reqs, const uint64_t* lbas, int write)
{
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (tid >= n_reqs) return;
    Controller* c = ctrls[0];
    QueuePair* qp = c->d_qps + tid % c->n_qps;
    const uint64_t start_block = lbas ? lbas[tid] : (tid * req_size) >> qp->block_size_log;
    const uint64_t n_blocks = req_size >> qp->block_size_log;
    if (write) __builtin_amdgcn_fence(__ATOMIC_RELEASE, "");      /* what the slot holds has reached memory before the controller fetches it */
    nvm_cmd_t cmd;
#pragma unroll
    for (int i = 0; i < 16; i++) cmd.dword[i] = 0;
    const uint16_t cid = get_cid(&qp->sq);
    nvm_cmd_header(&cmd, cid, write ? NVM_IO_WRITE : NVM_IO_READ, qp->nvmNamespace);
    nvm_cmd_data_ptr(&cmd, pc->prp1[tid], pc->prps ? pc->prp2[tid] : 0);
    nvm_cmd_rw_blks(&cmd, start_block, (uint16_t)n_blocks);
    const uint16_t sq_pos = sq_enqueue(&qp->sq, &cmd);
    (void)sq_pos;
    uint32_t head = 0, head_ = 0;
    const uint32_t cq_pos = cq_poll(&qp->cq, cid, &head, &head_);
    cq_dequeue(&qp->cq, (uint16_t)cq_pos, &qp->sq, head, head_);
    put_cid(&qp->sq, cid);
}

/* one wave, the lanes named in `lanes` active: util.h's warp_memcpy of n words */
__global__ void k_warp_memcpy(uint64_t* dst, const uint64_t* src, uint64_t n, uint64_t lanes)
{
    if ((lanes >> bam::lane()) & 1) warp_memcpy(dst, src, (size_t)n);
}

/*
 * The second look of a pointer that holds no reference, case by case: one wave opens a window on a resident page through
 * bam_ptr<T, true>, the page's descriptor is changed under it in one way (by the same wave: nobody else uses the cache
 * meanwhile), still() is asked, and the descriptor is put back.  out[c] = 1 if still() found the window standing.
 * Cases: 0 nothing changed, 1 other readers' references (the count in the state word), 2 the dirty bit, 3 busy, 4 not
 * valid, 5 another slot, 6 the same slot loaded once more.  Only the first three may stand.
 */
__global__ void k_unheld_window_cases(array_d_t<uint64_t>* dr, uint64_t page, uint32_t* out)
{
    uint64_t* const word = (uint64_t*)(dr->d_ranges[0].pages + page);
    const uint64_t epp = dr->d_ranges[0].n_elems_per_page;
    for (uint32_t c = 0; c < 7; c++) {
        bam_ptr<uint64_t, true> ptr(dr);
        const uint64_t x = ptr[page * epp + bam::lane()];
        const bool opened = !ptr.missed;
        const uint64_t was = __hip_atomic_load(word, __ATOMIC_RELAXED, BAM_AGENT);
        uint64_t now = was;
        switch (c) {
        case 1: now = was + 5; break;
        case 2: now = was | (uint64_t)DIRTY; break;
        case 3: now = was | (uint64_t)BUSY; break;
        case 4: now = was & ~(uint64_t)VALID; break;
        case 5: now = was ^ (1ull << 32); break;
        case 6: now = was + (1ull << (32 + BAM_SLOT_BITS)); break;
        default: break;
        }
        if (bam::lane() == 0) { __hip_atomic_store(word, now, __ATOMIC_RELAXED, BAM_AGENT); bam::fence_meta(); }
        const bool stands = ptr.still();
        if (bam::lane() == 0) { __hip_atomic_store(word, was, __ATOMIC_RELAXED, BAM_AGENT); bam::fence_meta(); }
        const uint64_t all = bam::ballot(stands), none = bam::ballot(!stands);
        /* every lane says the same; a window that fell must have set `missed`, one that stands must not */
        if (bam::lane() == 0) out[c] = (opened && none == 0 && !ptr.missed ? 1u : 0u) | (opened && all == 0 && ptr.missed ? 2u : 0u) | (x == 0 && !opened ? 4u : 0u);
    }
}

/*
 * Raw block reads with several commands in flight per thread (benchmarks/iodepth-block/main.cu:97-140): thread t
 * submits its `depth` commands with access_data_async (command k of thread t reads LBA lbas[t * depth + k] into slot
 * t * depth + k), then collects them with poll_async.  Wave w uses queue pair w mod n_qps.
 */
template <int DEPTH>
__global__ void k_block_io_async(Controller** ctrls, page_cache_d_t* pc, uint32_t req_size, uint64_t n_threads, const uint64_t* lbas)
{
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (tid >= n_threads) return;
    QueuePair* qp = ctrls[0]->d_qps + (tid / BAM_WAVE_SIZE) % ctrls[0]->n_qps;
    const uint64_t n_blocks = req_size >> qp->block_size_log;
    uint16_t cids[DEPTH], poss[DEPTH];
#pragma unroll
    for (int k = 0; k < DEPTH; k++) access_data_async(pc, qp, lbas[tid * DEPTH + k], n_blocks, tid * DEPTH + k, NVM_IO_READ, cids + k, poss + k);
#pragma unroll
    for (int k = 0; k < DEPTH; k++) poll_async(qp, cids[k], poss[k]);
}

// ---- readwrite benchmark (benchmarks/readwrite/main.cu:73-116): cache slots <-> consecutive pages of the store ----
__global__ void k_sequential_access(Controller** ctrls, page_cache_d_t* pc, uint32_t req_size, uint64_t n_slots, uint64_t store_byte, int write)
{
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint64_t n_threads = (uint64_t)gridDim.x * blockDim.x;
    QueuePair* qp = ctrls[0]->d_qps + (tid / BAM_WAVE_SIZE) % ctrls[0]->n_qps;
    const uint64_t n_blocks = req_size >> qp->block_size_log;
    for (uint64_t t = tid; t < n_slots; t += n_threads) {
        const uint64_t start_block = (store_byte + t * req_size) >> qp->block_size_log;
        if (write) write_data(pc, qp, start_block, n_blocks, t);
        else read_data(pc, qp, start_block, n_blocks, t);
    }
}

__global__ void k_block_checksum(page_cache_d_t* pc, uint64_t n_slots, uint32_t req_bytes, uint64_t* out)
{
    /* one wave per slot */
    const uint64_t wave = ((uint64_t)blockIdx.x * blockDim.x + threadIdx.x) / BAM_WAVE_SIZE;
    uint64_t v = 0;
    if (wave < n_slots) {
        const uint64_t* p = (const uint64_t*)(pc->base_addr + wave * pc->page_size);
        for (uint32_t i = bam::lane(); i < req_bytes / 8; i += BAM_WAVE_SIZE) v += p[i];
    }
    v = wave_sum(v);
    if (wave < n_slots && bam::lane() == 0) out[wave] = v;
}

/* one thread per request over an array of 32-bit elements: sum of the values read */
__global__ void k_array32_read(array_d_t<uint32_t>* dr, uint64_t n_reqs, const uint64_t* assignment, uint64_t stride, unsigned long long* sum)
{
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint64_t v = 0;
    if (tid < n_reqs) v = (*dr)[assignment ? assignment[tid] : tid * stride];
    block_accumulate(sum, v);
}

// ---- synthetic inputs ----
__global__ void k_gen_words(uint64_t seed, uint64_t first, uint64_t n, uint64_t* out)
{
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = splitmix64(seed, first + i);
}
__global__ void k_gen_mod(uint64_t seed, uint64_t first, uint64_t n, uint64_t modulus, uint64_t scale, uint64_t* out)
{
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = (splitmix64(seed, first + i) % modulus) * scale;
}
/* RMAT a=.57 b=.19 c=.19 d=.05 as 32-bit thresholds floor(p * 2^32); one quadrant draw per level from splitmix64(seed, edge * scale + level) */
__global__ void k_gen_rmat(uint64_t seed, uint32_t scale, uint64_t first, uint64_t n, uint64_t* u, uint64_t* v)
{
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const uint32_t T1 = 2448131358u, T2 = T1 + 816043786u, T3 = T2 + 816043786u;
    const uint64_t e = first + i;
    uint64_t uu = 0, vv = 0;
    for (uint32_t l = 0; l < scale; l++) {
        const uint32_t x = (uint32_t)(splitmix64(seed, e * scale + l) >> 32);
        const uint32_t q = x < T1 ? 0 : x < T2 ? 1 : x < T3 ? 2 : 3;
        uu = (uu << 1) | (q >> 1);
        vv = (vv << 1) | (q & 1);
    }
    u[i] = uu; v[i] = vv;
}
__global__ void k_gen_uniform(uint64_t seed, uint64_t n_vertices, uint64_t first, uint64_t n, uint64_t* u, uint64_t* v)
{
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const uint64_t p = first + i;
    u[i] = splitmix64(seed, 2 * p) % n_vertices;
    v[i] = splitmix64(seed, 2 * p + 1) % n_vertices;
}

// ---- measurement helpers ----
__global__ void k_copy16(const uint4* __restrict__ src, uint4* __restrict__ dst, uint64_t n16)
{
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (uint64_t)gridDim.x * blockDim.x) dst[i] = src[i];
}
/* plain streaming read of device memory with the loads of the hit path (a wave reads 4 KiB pieces side by side, eight 8-byte
 * words per lane, past the vector L1 and marked as not to be kept) and nothing else: what the memory system gives such a
 * reader, the practical ceiling over the hit-path figure */
__global__ __launch_bounds__(256) void k_read_stream(const uint64_t* __restrict__ src, uint64_t n8, unsigned long long* partials)
{
    uint64_t a = 0;
    const uint64_t wave = ((uint64_t)blockIdx.x * blockDim.x + threadIdx.x) / BAM_WAVE_SIZE, lane = threadIdx.x % BAM_WAVE_SIZE;
    const uint64_t n_waves = (uint64_t)gridDim.x * blockDim.x / BAM_WAVE_SIZE;
    const uint64_t per_wave = (n8 / n_waves) & ~511ull;             /* whole 4 KiB pieces; the rest goes to the last wave */
    const uint64_t* p = src + wave * per_wave;
    const uint64_t mine = wave + 1 == n_waves ? n8 - wave * per_wave : per_wave;
    uint64_t i = 0;
    for (; i + 512 <= mine; i += 512) {
        uint64_t x[8];
        bam::ld_payload_stream8(p + i + lane, x);
        a += ((x[0] + x[1]) + (x[2] + x[3])) + ((x[4] + x[5]) + (x[6] + x[7]));
    }
    for (i += lane; i < mine; i += BAM_WAVE_SIZE) a += p[i];
    block_accumulate(partials, a);
}
/*
 * The hit path of the streaming kernels taken apart, for measurement: a wave reads a run of resident pages of the cache,
 * 4 KiB each, and what it does around the payload loads is chosen.  REFS 0: the page's descriptor is read for the slot and
 * no reference is taken (only safe while nothing is evicted: a measurement, not an access route); 1: a reference per page,
 * taken before the page is read and dropped after (what bam_ptr does); 2: the references of sixteen pages taken with one
 * vector atomic and dropped with one (what the page-wise kernel does).  NT: the payload loads marked as not to be kept.
 * The differences between the six and the plain reader (k_read_stream) are what each part of the protocol costs.
 */
template <int REFS, bool NT>
__global__ __launch_bounds__(256) void k_hit_path_parts(array_d_t<uint64_t>* dr, uint64_t n_waves, uint64_t ppw, unsigned long long* partials)
{
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint64_t wave = bam::first(tid / BAM_WAVE_SIZE);
    const uint32_t lane = bam::lane();
    uint64_t v = 0;
    if (wave < n_waves) {
        bam::range_view<uint64_t> view;
        view.load(dr->d_ranges);
        const uint64_t start_page = wave * ppw;
        auto read_page = [&](const uint32_t slot) {
            const uint64_t* base = (const uint64_t*)view.slot_addr(slot) + lane;
            uint64_t x[8];
            if (NT) bam::ld_payload_stream8(base, x);
            else {
#pragma unroll
                for (int j = 0; j < 8; j++) x[j] = bam::ld_payload(base + j * BAM_WAVE_SIZE);
            }
            v += ((x[0] + x[1]) + (x[2] + x[3])) + ((x[4] + x[5]) + (x[6] + x[7]));
        };
        if (REFS == 2) {
            for (uint64_t p0 = 0; p0 < ppw; p0 += 16) {
                const uint32_t nb = (uint32_t)(ppw - p0 < 16 ? ppw - p0 : 16);
                data_page_t* dp = view.pages + start_page + p0 + (lane < nb ? lane : 0);
                uint64_t sv = 0;
                if (lane < nb) sv = __hip_atomic_fetch_add((uint64_t*)dp, 1ull, __ATOMIC_RELAXED, BAM_AGENT);
                const uint32_t slot = (uint32_t)(sv >> 32) & BAM_SLOT_MASK;
                for (uint32_t k = 0; k < nb; k++) read_page(bam::bcast(slot, k));
                bam::fence_meta();
                if (lane < nb) __hip_atomic_fetch_add(&dp->state, 0u - 1u, __ATOMIC_RELAXED, BAM_AGENT);
            }
        } else {
            for (uint64_t p = 0; p < ppw; p++) {
                data_page_t* dp = view.pages + start_page + p;
                uint64_t sv = 0;
                if (REFS == 0) sv = __hip_atomic_load((uint64_t*)dp, __ATOMIC_RELAXED, BAM_AGENT);
                else if (lane == 0) sv = __hip_atomic_fetch_add((uint64_t*)dp, (uint64_t)BAM_WAVE_SIZE, __ATOMIC_RELAXED, BAM_AGENT);
                sv = bam::bcast(sv, 0);
                read_page((uint32_t)(sv >> 32) & BAM_SLOT_MASK);
                if (REFS == 1) { bam::fence_meta(); if (lane == 0) __hip_atomic_fetch_add(&dp->state, 0u - (uint32_t)BAM_WAVE_SIZE, __ATOMIC_RELAXED, BAM_AGENT); }
            }
        }
    }
    block_accumulate(partials, v);
}
/* plain random gather of 8-byte words from device memory: the ceiling of that access pattern without any cache protocol */
__global__ void k_gather8(const uint64_t* __restrict__ src, const uint64_t* __restrict__ idx, uint64_t n, unsigned long long* partials)
{
    const uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    block_accumulate(partials, t < n ? src[idx[t]] : 0);
}
/* what a hit of the counted path costs the memory system: per request one 64-bit add that returns the old word and, once it
 * is back, one add on the same word whose result nobody reads (take a reference, drop it), on words scattered by idx[] */
template <int RETURNS>
__global__ void k_atomic_pairs(unsigned long long* table, const uint64_t* __restrict__ idx, uint64_t n, unsigned long long* partials)
{
    const uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    unsigned long long v = 0;
    if (t < n) {
        unsigned long long* w = table + idx[t];
        if (RETURNS) v = __hip_atomic_fetch_add(w, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        else __hip_atomic_fetch_add(w, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (v != ~0ull) __hip_atomic_fetch_add(w, ~0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    block_accumulate(partials, v);
}

/*
 * Pages handed from one compute-unit cluster to the others.  The grid is one wave per workgroup, which the dispatcher
 * deals out over the clusters in turn.  In round r the wave r % waves touches page r (a miss: the page is read into a
 * slot that another page left a few rounds ago) and raises flag[r]; every other wave waits for the flag with a bounded
 * spin, then reads elements of the page through array_d_t::operator[] and compares them with what the procedural store
 * holds; the next round starts when all have reported.  out[0] elements that differed, out[1] waits given up,
 * out[2] bit mask of the clusters that took part, out[3] reads checked.
 */
__global__ void k_xcd_relay(array_d_t<uint64_t>* dr, uint64_t seed, uint32_t n_pages, uint32_t rounds, uint32_t elems_per_page, uint32_t spin_limit,
                            uint32_t* flag, uint32_t* done, unsigned long long* out)
{
    const uint32_t me = blockIdx.x, waves = gridDim.x, l = bam::lane();
    if (l == 0) atomicOr(&out[2], 1ull << bam::xcc_id());
    unsigned long long bad = 0, late = 0, checked = 0;
    for (uint32_t r = 0; r < rounds; r++) {
        const uint64_t first = (uint64_t)(r % n_pages) * elems_per_page;
        if (me == r % waves) {
            /* the wave before last round's readers are through: their reads of the slot's last tenant are over */
            if (r) {
                uint32_t spins = 0;
                while (__hip_atomic_load(&done[r - 1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < waves - 1 && ++spins < spin_limit) __builtin_amdgcn_s_sleep(8);
                late += spins >= spin_limit;
            }
            const uint64_t v = (*dr)[first + l];
            bad += v != splitmix64(seed, first + l);
            checked++;
            bam::fence_meta();
            if (l == 0) __hip_atomic_store(&flag[r], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        } else {
            uint32_t spins = 0;
            while (__hip_atomic_load(&flag[r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0 && ++spins < spin_limit) __builtin_amdgcn_s_sleep(8);
            late += spins >= spin_limit;
            for (uint32_t k = l; k < elems_per_page; k += 4 * BAM_WAVE_SIZE) {
                const uint64_t v = (*dr)[first + k];
                bad += v != splitmix64(seed, first + k);
                checked++;
            }
            bam::fence_meta();
            if (l == 0) __hip_atomic_fetch_add(&done[r], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    atomicAdd(&out[0], bad); atomicAdd(&out[3], checked);
    if (l == 0) atomicAdd(&out[1], late);
}

/* every wave pulls whole chunks of host-pinned memory into device memory, 16 bytes per lane per load */
__global__ void k_host_pull(const uint4* __restrict__ host, uint4* __restrict__ dev, uint64_t n_chunks, uint32_t chunk16, uint64_t host_chunks)
{
    const uint64_t wave = ((uint64_t)blockIdx.x * blockDim.x + threadIdx.x) / BAM_WAVE_SIZE;
    const uint64_t n_waves = (uint64_t)gridDim.x * blockDim.x / BAM_WAVE_SIZE;
    for (uint64_t c = wave; c < n_chunks; c += n_waves) {
        const uint4* s = host + (c % host_chunks) * chunk16;
        uint4* d = dev + (c % host_chunks) * chunk16;
        for (uint32_t i = bam::lane(); i < chunk16; i += BAM_WAVE_SIZE) d[i] = s[i];
    }
}

void fill_backing(uint64_t seed, uint64_t* p, uint64_t n_words)
{
    unsigned nt = std::thread::hardware_concurrency();
    if (nt < 1) nt = 1;
    if (nt > 16) nt = 16;
    std::vector<std::thread> th;
    const uint64_t per = (n_words + nt - 1) / nt;
    for (unsigned t = 0; t < nt; t++) {
        const uint64_t a = t * per, b = a + per < n_words ? a + per : n_words;
        if (a < b) th.emplace_back([=]() { nvmt_fill_words(seed, a, b - a, p + a); });
    }
    for (auto& x : th) x.join();
}

} // namespace

// ---------------------------------------------------------------------------
// C entry points
// ---------------------------------------------------------------------------
extern "C" {

const char* bam_last_error(void) { return g_err.c_str(); }

int bam_device_count(int* count)
{
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (count) *count = e == hipSuccess ? n : 0;
    return e == hipSuccess ? 0 : fail(ENODEV, hipGetErrorString(e));
}

int bam_target_create(bam_target_t** out, const char* path, uint64_t ns_bytes, uint32_t lba_bytes, int backing, uint64_t seed,
                      uint32_t n_io_threads, uint32_t max_queue_entries, uint32_t max_io_queues, uint32_t completion_order,
                      uint32_t fail_every, uint32_t drop_every)
{
    if (!out || !path) return fail(EINVAL, "bam_target_create: null argument");
    *out = nullptr;
    BAM_API_BEGIN
    bam_target* bt = new bam_target();
    nvmt_config_t& c = bt->cfg;
    c.ns_bytes = ns_bytes; c.lba_bytes = lba_bytes; c.seed = seed; c.n_io_threads = n_io_threads;
    c.max_queue_entries = max_queue_entries; c.max_io_queues = max_io_queues; c.dstrd = 4;     /* one doorbell per 64-byte line */
    c.order = completion_order; c.fail_every = fail_every; c.drop_every = drop_every;
    if (backing) {
        if (posix_memalign(&bt->backing, 4096, ns_bytes)) { delete bt; return fail(ENOMEM, "bam_target_create: backing store allocation failed"); }
        bt->backing_bytes = ns_bytes;
        fill_backing(seed, (uint64_t*)bt->backing, ns_bytes / 8);
        c.backing = bt->backing;
    }
    const size_t bar_size = nvmt_bar_size(&c);
    hip_err_chk(hipHostMalloc(&bt->bar, bar_size, hipHostMallocMapped));
    memset(bt->bar, 0, bar_size);
    bt->t = nvmt_create(&c, bt->bar);
    if (!bt->t) { (void)hipHostFree(bt->bar); free(bt->backing); delete bt; return fail(EINVAL, "bam_target_create: invalid target configuration"); }
    int err = nvmt_publish(path, bt->t);
    if (err) { nvmt_destroy(bt->t); (void)hipHostFree(bt->bar); free(bt->backing); delete bt; return fail(err, "bam_target_create: path already published"); }
    *out = bt;
    BAM_API_END
}

void bam_target_destroy(bam_target_t* t)
{
    if (!t) return;
    nvmt_destroy(t->t);
    (void)hipHostFree(t->bar);
    free(t->backing);
    delete t;
}

int bam_target_stats(bam_target_t* t, uint64_t* out, int reset)
{
    if (!t || !out) return fail(EINVAL, "bam_target_stats: null argument");
    nvmt_stats_t s;
    nvmt_stats(t->t, &s);
    const uint64_t v[12] = {s.admin_cmds, s.io_cmds, s.read_cmds, s.write_cmds, s.bytes_read, s.bytes_written, s.error_cpls, s.sq_doorbells, s.cq_full_stalls, s.dropped, s.sqe_retries, s.stale_doorbells};
    memcpy(out, v, sizeof(v));
    if (reset) nvmt_reset_stats(t->t);
    return 0;
}

void* bam_target_backing(bam_target_t* t) { return t ? t->backing : nullptr; }

int bam_ctrl_create(bam_ctrl_t** out, const char* path, uint32_t ns_id, uint32_t device, uint64_t queue_depth, uint64_t n_queues,
                    uint32_t stage_bytes, uint32_t spin_limit)
{
    if (!out || !path) return fail(EINVAL, "bam_ctrl_create: null argument");
    *out = nullptr;
    BAM_API_BEGIN
    Controller* c = new Controller(path, ns_id, device, queue_depth, n_queues, stage_bytes, spin_limit);
    *out = new bam_ctrl{c};
    BAM_API_END
}

void bam_ctrl_destroy(bam_ctrl_t* c)
{
    if (!c) return;
    delete c->c;
    delete c;
}

int bam_ctrl_info(bam_ctrl_t* c, uint64_t* out, int reset)
{
    if (!c || !out) return fail(EINVAL, "bam_ctrl_info: null argument");
    BAM_API_BEGIN
    out[0] = c->c->n_qps;
    out[1] = c->c->n_qps ? c->c->h_qps[0]->sq.qs : 0;
    out[2] = c->c->blk_size;
    out[3] = c->c->ns.size;
    if (reset) out[4] = c->c->reset_stats();
    else hip_err_chk(hipMemcpy(&out[4], c->c->d_ctrl_ptr, sizeof(uint64_t), hipMemcpyDeviceToHost));
    out[5] = c->c->completion_errors();
    BAM_API_END
}

int bam_ctrl_queue_state(bam_ctrl_t* c, uint32_t qp, uint64_t* out16, uint32_t* slots, uint32_t n_slots)
{
    if (!c || !out16) return fail(EINVAL, "bam_ctrl_queue_state: null argument");
    if (qp >= c->c->n_qps) return fail(EINVAL, "bam_ctrl_queue_state: no such queue pair");
    BAM_API_BEGIN
    nvm_queue_t sq, cq;
    hip_err_chk(hipMemcpy(&sq, &c->c->d_qps[qp].sq, sizeof(sq), hipMemcpyDeviceToHost));
    hip_err_chk(hipMemcpy(&cq, &c->c->d_qps[qp].cq, sizeof(cq), hipMemcpyDeviceToHost));
    out16[0] = sq.qs; out16[1] = sq.in_ticket; out16[2] = sq.tail_lock >> 1; out16[3] = sq.tail_lock & 1u; out16[4] = sq.head;
    out16[5] = cq.head_lock >> 1; out16[6] = cq.head_lock & 1u; out16[7] = cq.n_errors;
    for (uint32_t k = 0; k < 8; k++) out16[8 + k] = 0;
    if (slots && n_slots) {
        const uint32_t n = n_slots < sq.qs ? n_slots : sq.qs;
        std::vector<uint32_t> a(sq.qs), b(sq.qs), d(sq.qs);
        hip_err_chk(hipMemcpy(a.data(), sq.tickets, sq.qs * 4, hipMemcpyDeviceToHost));
        hip_err_chk(hipMemcpy(b.data(), sq.tail_mark, sq.qs * 4, hipMemcpyDeviceToHost));
        hip_err_chk(hipMemcpy(d.data(), sq.cid, sq.qs * 4, hipMemcpyDeviceToHost));
        for (uint32_t i = 0; i < n; i++) { slots[3 * i] = a[i]; slots[3 * i + 1] = b[i]; slots[3 * i + 2] = d[i]; }
    }
    BAM_API_END
}

int bam_target_queue_state(bam_target_t* t, uint32_t qid, uint64_t* out8)
{
    if (!t || !out8) return fail(EINVAL, "bam_target_queue_state: null argument");
    const int rc = nvmt_queue_state(t->t, (uint16_t)qid, out8);
    return rc ? fail(rc, "bam_target_queue_state: no such queue") : 0;
}

int bam_ctrl_aborted(bam_ctrl_t* c, int clear)
{
    if (!c) return 0;
    int a = c->c->aborted();
    if (clear) c->c->clear_abort();
    return a;
}

int bam_page_cache_create(bam_page_cache_t** out, uint64_t page_size, uint64_t n_pages, uint32_t device, bam_ctrl_t* ctrl, uint64_t max_range)
{
    if (!out || !ctrl) return fail(EINVAL, "bam_page_cache_create: null argument");
    *out = nullptr;
    BAM_API_BEGIN
    std::vector<Controller*> ctrls{ctrl->c};
    page_cache_t* pc = new page_cache_t(page_size, n_pages, device, *ctrl->c, max_range, ctrls);
    *out = new bam_page_cache{pc, ctrl->c};
    BAM_API_END
}

int bam_page_cache_create_multi(bam_page_cache_t** out, uint64_t page_size, uint64_t n_pages, uint32_t device, bam_ctrl_t** ctrls, uint32_t n_ctrls,
                                uint64_t max_range)
{
    if (!out || !ctrls || !n_ctrls) return fail(EINVAL, "bam_page_cache_create_multi: null argument");
    *out = nullptr;
    std::vector<Controller*> cs;
    for (uint32_t i = 0; i < n_ctrls; i++) {
        if (!ctrls[i]) return fail(EINVAL, "bam_page_cache_create_multi: null controller");
        cs.push_back(ctrls[i]->c);
    }
    BAM_API_BEGIN
    page_cache_t* pc = new page_cache_t(page_size, n_pages, device, *cs[0], max_range, cs);
    *out = new bam_page_cache{pc, cs[0]};
    BAM_API_END
}

void bam_page_cache_destroy(bam_page_cache_t* pc)
{
    if (!pc) return;
    delete pc->pc;
    delete pc;
}

int bam_page_cache_info(bam_page_cache_t* pc, uint64_t* out)
{
    if (!pc || !out) return fail(EINVAL, "bam_page_cache_info: null argument");
    out[0] = pc->pc->pdt.n_pages;
    out[1] = pc->pc->pdt.page_size;
    out[2] = pc->pc->pdt.wave_batch;
    out[3] = pc->ctrl->n_qps && pc->ctrl->h_qps[0]->stage != nullptr;
    out[4] = pc->pc->pdt.direct_share;
    return 0;
}

int bam_page_cache_export_dmabuf(bam_page_cache_t* pc, int* fd, uint64_t* bytes)
{
    if (!pc || !fd || !bytes) return fail(EINVAL, "bam_page_cache_export_dmabuf: null argument");
    *fd = -1;
    /* whole host pages: the allocation behind the slots is at least that large (allocations are made in larger pieces) */
    const uint64_t want = (pc->pc->pdt.n_pages * pc->pc->pdt.page_size + 4095ull) & ~4095ull;
    int out = -1;
    const hipError_t e = hipMemGetHandleForAddressRange(&out, (hipDeviceptr_t)pc->pc->pdt.base_addr, want, hipMemRangeHandleTypeDmaBufFd, 0);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return fail(ENOTSUP, std::string("bam_page_cache_export_dmabuf: ") + hipGetErrorString(e));
    }
    *fd = out;
    *bytes = want;
    return 0;
}

int bam_page_cache_profile(bam_page_cache_t* pc, uint64_t* out32, int reset)
{
    if (!pc || !out32) return fail(EINVAL, "bam_page_cache_profile: null argument");
    BAM_API_BEGIN
    hip_err_chk(hipDeviceSynchronize());
    hip_err_chk(hipMemcpy(out32, pc->pc->pdt.prof, 32 * sizeof(uint64_t), hipMemcpyDeviceToHost));
    if (reset) hip_err_chk(hipMemset(pc->pc->pdt.prof, 0, 32 * sizeof(uint64_t)));
    BAM_API_END
}

int bam_page_cache_flush(bam_page_cache_t* pc)
{
    if (!pc) return fail(EINVAL, "bam_page_cache_flush: null argument");
    BAM_API_BEGIN
    pc->pc->flush_cache();
    hip_err_chk(hipDeviceSynchronize());
    BAM_API_END
}

int bam_range_create(bam_range_t** out, uint64_t index_start, uint64_t count, uint64_t page_start, uint64_t page_count,
                     uint64_t page_start_offset, uint64_t page_size, bam_page_cache_t* pc, uint32_t device, int dist)
{
    if (!out || !pc) return fail(EINVAL, "bam_range_create: null argument");
    *out = nullptr;
    if (dist != REPLICATE && dist != STRIPE) return fail(EINVAL, "bam_range_create: unknown distribution");
    if (page_size != pc->pc->pdt.page_size) return fail(EINVAL, "bam_range_create: page size differs from the cache's");
    if (page_start_offset >= page_size || count <= index_start || page_count == 0) return fail(EINVAL, "bam_range_create: empty or misaligned range");
    if (((count - index_start) * sizeof(uint64_t) + page_start_offset + page_size - 1) / page_size > page_count)
        return fail(EINVAL, "bam_range_create: page_count does not cover the elements");
    BAM_API_BEGIN
    *out = new bam_range{new range_t<uint64_t>(index_start, count, page_start, page_count, page_start_offset, page_size, pc->pc, device, (data_dist_t)dist)};
    BAM_API_END
}

void bam_range_destroy(bam_range_t* r)
{
    if (!r) return;
    delete r->r;
    delete r;
}

int bam_array_create(bam_array_t** out, uint64_t n_elems, uint64_t disk_start_offset, bam_range_t** ranges, uint32_t n_ranges, uint32_t device)
{
    if (!out || !ranges || !n_ranges) return fail(EINVAL, "bam_array_create: null argument");
    *out = nullptr;
    BAM_API_BEGIN
    std::vector<range_t<uint64_t>*> rs;
    for (uint32_t i = 0; i < n_ranges; i++) rs.push_back(ranges[i]->r);
    *out = new bam_array{new array_t<uint64_t>(n_elems, disk_start_offset, rs, device), createBuffer(BAM_SUM_PARTIALS * sizeof(uint64_t), device)};
    BAM_API_END
}

void bam_array_destroy(bam_array_t* a)
{
    if (!a) return;
    delete a->a;
    delete a;
}

int bam_array_stats(bam_array_t* a, uint64_t* out, int reset)
{
    if (!a || !out) return fail(EINVAL, "bam_array_stats: null argument");
    BAM_API_BEGIN
    hip_err_chk(hipDeviceSynchronize());
    if (!reset) {
        /* read without clearing: read-and-reset, then put the totals back into shard 0 */
        std::vector<bam_array_counters> per;
        a->a->reset_stats(&per);
        for (size_t i = 0; i < per.size(); i++) {
            bam_stat_shard_t s0 = {per[i].access_cnt, 0, per[i].hit_cnt, per[i].read_io_cnt, {0, 0, 0, 0}};
            hip_err_chk(hipMemcpy(a->a->h_ranges[i].stats, &s0, sizeof(s0), hipMemcpyHostToDevice));
        }
        out[0] = out[1] = out[2] = out[3] = 0;
        for (auto& p : per) { out[0] += p.read_io_cnt; out[1] += p.access_cnt; out[2] += p.miss_cnt; out[3] += p.hit_cnt; }
    } else {
        bam_array_counters t = a->a->reset_stats();
        out[0] = t.read_io_cnt; out[1] = t.access_cnt; out[2] = t.miss_cnt; out[3] = t.hit_cnt;
    }
    BAM_API_END
}

/* whether the entry points that have a two-launch form may use it on this array: one range, reads of resident pages
 * without a reference switched on (the first launch reads that way) */
static bool two_launches_ok(bam_array_t* a)
{
    return a->a->adt.n_ranges == 1 && a->a->h_ranges[0].cache.fast_reads != 0;
}

int bam_array_read_shaped(bam_array_t* a, uint64_t n_reqs, const uint64_t* d_assignment, int shape, uint32_t reads_per_lane, uint32_t block_size,
                          uint64_t* d_sum, void* stream)
{
    if (!a || !d_sum || !d_assignment) return fail(EINVAL, "bam_array_read_shaped: null argument");
    if (!block_size || block_size % BAM_WAVE_SIZE || block_size > 1024) return fail(EINVAL, "bam_array_read_shaped: block size must be a multiple of 64, at most 1024");
    if (shape < BAM_READ_ONE_PER_THREAD || shape > BAM_READ_TWO_LAUNCHES) return fail(EINVAL, "bam_array_read_shaped: unknown shape");
    if (shape == BAM_READ_TWO_LAUNCHES && reads_per_lane != 1 && reads_per_lane != 2 && reads_per_lane != 4 && reads_per_lane != 8)
        return fail(EINVAL, "bam_array_read_shaped: 1, 2, 4 or 8 reads per lane");
    if (shape == BAM_READ_TWO_LAUNCHES && !two_launches_ok(a)) return fail(EINVAL, "bam_array_read_shaped: two launches need an array of one range and BAM_FAST_READS on");
    if (!n_reqs) return 0;
    BAM_API_BEGIN
    hipStream_t st = (hipStream_t)stream;
    array_d_t<uint64_t>* d = a->a->d_array_ptr;
    unsigned long long* part = (unsigned long long*)a->partials.get();
    if (shape == BAM_READ_ONE_PER_THREAD) {
        hipLaunchKernelGGL(k_array_read, dim3(blocks_for(n_reqs, block_size)), dim3(block_size), 0, st, d, n_reqs, d_assignment, (uint64_t)1, (uint64_t)1, part);
        hipLaunchKernelGGL(k_fold_partials, dim3(1), dim3(1024), 0, st, part, (unsigned long long*)d_sum);
    } else if (shape == BAM_READ_FOUR_PER_THREAD) {
        const uint64_t threads = (n_reqs + BAM_READS_PER_LANE - 1) / BAM_READS_PER_LANE;
        hipLaunchKernelGGL(k_array_read_n_whole, dim3(blocks_for(threads, block_size)), dim3(block_size), 0, st, d, n_reqs, d_assignment, threads, part);
        hipLaunchKernelGGL(k_fold_partials, dim3(1), dim3(1024), 0, st, part, (unsigned long long*)d_sum);
    } else {
        const uint32_t N = reads_per_lane;
        /* rounds of N reads per thread: as many as leave sixteen thousand workgroups, several times what the device holds at a time
         * (a launch of about as many workgroups as the device holds ends with most of the device idle) */
        uint32_t rounds = 1;
        while (rounds < 32 && n_reqs / ((uint64_t)N * rounds * 2 * 256) >= 16384) rounds *= 2;
        const uint64_t per_thread = (uint64_t)N * rounds;
        const uint64_t threads = ((n_reqs + per_thread - 1) / per_thread + BAM_WAVE_SIZE - 1) / BAM_WAVE_SIZE * BAM_WAVE_SIZE;
        const uint64_t n_words = threads / BAM_WAVE_SIZE * per_thread;
        uint64_t* missed = (uint64_t*)a->notes_for(n_words * sizeof(uint64_t));
        const dim3 grid(blocks_for(threads, 256)), block(256);
        unsigned long long* sum = (unsigned long long*)d_sum;
        uint32_t* fin = (uint32_t*)a->finished.get();
        const uint32_t call = a->next_call();
        switch (N) {
        case 1: hipLaunchKernelGGL(k_array_read_n<1>, grid, block, 0, st, d, n_reqs, d_assignment, threads, rounds, part, missed, sum, fin, call); break;
        case 2: hipLaunchKernelGGL(k_array_read_n<2>, grid, block, 0, st, d, n_reqs, d_assignment, threads, rounds, part, missed, sum, fin, call); break;
        case 4: hipLaunchKernelGGL(k_array_read_n<4>, grid, block, 0, st, d, n_reqs, d_assignment, threads, rounds, part, missed, sum, fin, call); break;
        default: hipLaunchKernelGGL(k_array_read_n<8>, grid, block, 0, st, d, n_reqs, d_assignment, threads, rounds, part, missed, sum, fin, call); break;
        }
        /* the second launch: as many words per wave as leave some eight thousand waves' worth of chunks */
        uint32_t words = 1;
        while (words < BAM_DEFER_MAX_WORDS && n_words / (words * 2) >= 8192) words *= 2;
        const uint64_t n_chunks = (n_words + words - 1) / words;
        const uint64_t waves = n_chunks < 16384 ? n_chunks : 16384;
        hipLaunchKernelGGL(k_array_read_deferred, dim3(blocks_for(waves * BAM_WAVE_SIZE, 256)), dim3(256), 0, st, d, n_reqs, d_assignment, missed, n_words, words,
                           part, sum, fin, call);
    }
    hip_err_chk(hipGetLastError());
    BAM_API_END
}

int bam_array_read(bam_array_t* a, uint64_t n_reqs, const uint64_t* d_assignment, uint64_t stride, uint64_t reqs_per_thread,
                   uint32_t block_size, uint64_t* d_sum, void* stream)
{
    if (!a || !d_sum) return fail(EINVAL, "bam_array_read: null argument");
    if (!block_size || block_size % BAM_WAVE_SIZE || block_size > 1024) return fail(EINVAL, "bam_array_read: block size must be a multiple of 64, at most 1024");
    if (!n_reqs) return 0;
    /* a large launch of scattered requests, one read each: in two launches where the array allows it, else four requests per
     * thread (results and counters are the same) */
    if (d_assignment && reqs_per_thread == 1 && n_reqs >= (1ull << 16)) {
        static const int shape_env = getenv("BAM_READ_SHAPE") ? atoi(getenv("BAM_READ_SHAPE")) : 0;
        /* eight reads per lane in the first launch: 44 thousand million reads a second on resident data against 39 with four
         * (what bounds the kernel is how many requests a compute unit's L1 keeps in flight, and for how long each) */
        static const int lanes_env = getenv("BAM_READS_PER_LANE") ? atoi(getenv("BAM_READS_PER_LANE")) : 8;
        int shape = two_launches_ok(a) ? BAM_READ_TWO_LAUNCHES : BAM_READ_FOUR_PER_THREAD;
        if (shape_env >= BAM_READ_ONE_PER_THREAD && shape_env <= BAM_READ_TWO_LAUNCHES && (shape_env != BAM_READ_TWO_LAUNCHES || two_launches_ok(a))) shape = shape_env;
        return bam_array_read_shaped(a, n_reqs, d_assignment, shape, (uint32_t)lanes_env, block_size, d_sum, stream);
    }
    BAM_API_BEGIN
    hipLaunchKernelGGL(k_array_read, dim3(blocks_for(n_reqs, block_size)), dim3(block_size), 0, (hipStream_t)stream,
                       a->a->d_array_ptr, n_reqs, d_assignment, stride, reqs_per_thread, (unsigned long long*)a->partials.get());
    hipLaunchKernelGGL(k_fold_partials, dim3(1), dim3(1024), 0, (hipStream_t)stream, (unsigned long long*)a->partials.get(), (unsigned long long*)d_sum);
    hip_err_chk(hipGetLastError());
    BAM_API_END
}

int bam_array_gather(bam_array_t* a, uint64_t n_reqs, const uint64_t* d_assignment, uint64_t stride, uint32_t block_size, uint64_t* d_out, void* stream)
{
    if (!a || !d_out) return fail(EINVAL, "bam_array_gather: null argument");
    if (!block_size || block_size % BAM_WAVE_SIZE || block_size > 1024) return fail(EINVAL, "bam_array_gather: block size must be a multiple of 64, at most 1024");
    if (!n_reqs) return 0;
    BAM_API_BEGIN
    hipLaunchKernelGGL(k_array_gather, dim3(blocks_for(n_reqs, block_size)), dim3(block_size), 0, (hipStream_t)stream,
                       a->a->d_array_ptr, n_reqs, d_assignment, stride, d_out);
    hip_err_chk(hipGetLastError());
    BAM_API_END
}

int bam_array_read_via(bam_array_t* a, int api, uint64_t n_reqs, const uint64_t* d_assignment, uint64_t span, uint32_t block_size,
                       uint64_t* d_sum, void* stream)
{
    if (!a || !d_sum) return fail(EINVAL, "bam_array_read_via: null argument");
    if (api < 1 || api > 7) return fail(EINVAL, "bam_array_read_via: api must be 1..7");
    if (!block_size || block_size % BAM_WAVE_SIZE || block_size > 1024) return fail(EINVAL, "bam_array_read_via: block size must be a multiple of 64, at most 1024");
    if (!span) return fail(EINVAL, "bam_array_read_via: span must be at least 1");
    if (!n_reqs) return 0;
    BAM_API_BEGIN
    hipStream_t st = (hipStream_t)stream;
    array_d_t<uint64_t>* d = a->a->d_array_ptr;
    unsigned long long* s = (unsigned long long*)a->partials.get();
    const dim3 grid(blocks_for(api == 5 ? n_reqs * BAM_WAVE_SIZE : n_reqs, block_size)), block(block_size);
    BufferPtr scratch;
    if (api == 5) scratch = createBuffer(n_reqs * span * sizeof(uint64_t), 0);
    uint64_t* sc = (uint64_t*)scratch.get();
    switch (api) {
    case 1: hipLaunchKernelGGL(k_array_read_via<1>, grid, block, 0, st, d, n_reqs, d_assignment, span, sc, s); break;
    case 2: hipLaunchKernelGGL(k_array_read_via<2>, grid, block, 0, st, d, n_reqs, d_assignment, span, sc, s); break;
    case 3: hipLaunchKernelGGL(k_array_read_via<3>, grid, block, 0, st, d, n_reqs, d_assignment, span, sc, s); break;
    case 4: hipLaunchKernelGGL(k_array_read_via<4>, grid, block, 0, st, d, n_reqs, d_assignment, span, sc, s); break;
    case 5: hipLaunchKernelGGL(k_array_read_via<5>, grid, block, 0, st, d, n_reqs, d_assignment, span, sc, s); break;
    case 6: hipLaunchKernelGGL(k_array_read_via<6>, grid, block, 0, st, d, n_reqs, d_assignment, span, sc, s); break;
    default: hipLaunchKernelGGL(k_array_read_via<7>, grid, block, 0, st, d, n_reqs, d_assignment, span, sc, s); break;
    }
    hipLaunchKernelGGL(k_fold_partials, dim3(1), dim3(1024), 0, st, s, (unsigned long long*)d_sum);
    hip_err_chk(hipGetLastError());
    if (api == 5) hip_err_chk(hipStreamSynchronize(st));       /* the scratch buffer goes away with this call */
    BAM_API_END
}

int bam_array_write(bam_array_t* a, uint64_t n_reqs, const uint64_t* d_assignment, uint64_t stride, const uint64_t* d_values,
                    uint32_t block_size, void* stream)
{
    if (!a || !d_values) return fail(EINVAL, "bam_array_write: null argument");
    if (!block_size || block_size % BAM_WAVE_SIZE || block_size > 1024) return fail(EINVAL, "bam_array_write: block size must be a multiple of 64, at most 1024");
    if (!n_reqs) return 0;
    BAM_API_BEGIN
    hipLaunchKernelGGL(k_array_write, dim3(blocks_for(n_reqs, block_size)), dim3(block_size), 0, (hipStream_t)stream,
                       a->a->d_array_ptr, n_reqs, d_assignment, stride, d_values);
    hip_err_chk(hipGetLastError());
    BAM_API_END
}

int bam_array_update(bam_array_t* a, int api, uint64_t n_reqs, const uint64_t* d_assignment, const uint64_t* d_values, uint64_t* d_old,
                     uint32_t block_size, void* stream)
{
    if (!a || !d_assignment || !d_values) return fail(EINVAL, "bam_array_update: null argument");
    if (api < 0 || api > 2) return fail(EINVAL, "bam_array_update: api must be 0, 1 or 2");
    if (!block_size || block_size % BAM_WAVE_SIZE || block_size > 1024) return fail(EINVAL, "bam_array_update: block size must be a multiple of 64, at most 1024");
    if (!n_reqs) return 0;
    BAM_API_BEGIN
    const dim3 grid(blocks_for(n_reqs, block_size)), block(block_size);
    hipStream_t st = (hipStream_t)stream;
    array_d_t<uint64_t>* d = a->a->d_array_ptr;
    if (api == 0) hipLaunchKernelGGL(k_array_update<0>, grid, block, 0, st, d, n_reqs, d_assignment, d_values, d_old);
    else if (api == 1) hipLaunchKernelGGL(k_array_update<1>, grid, block, 0, st, d, n_reqs, d_assignment, d_values, d_old);
    else hipLaunchKernelGGL(k_array_update<2>, grid, block, 0, st, d, n_reqs, d_assignment, d_values, d_old);
    hip_err_chk(hipGetLastError());
    BAM_API_END
}

int bam_sqe_image(uint16_t cid, uint8_t opcode, uint32_t nsid, uint64_t prp1, uint64_t prp2, uint64_t lba, uint16_t n_blocks, int seal, uint32_t ticket,
                  uint32_t* host_out16, uint32_t* d_out64x16, void* stream)
{
    if (!host_out16 && !d_out64x16) return fail(EINVAL, "bam_sqe_image: null argument");
    BAM_API_BEGIN
    if (host_out16) {
        nvm_cmd_t cmd;
        memset(&cmd, 0, sizeof(cmd));
        nvm_cmd_header(&cmd, cid, opcode, nsid);
        nvm_cmd_data_ptr(&cmd, prp1, prp2);
        nvm_cmd_rw_blks(&cmd, lba, n_blocks);
        if (seal) nvm_cmd_seal(&cmd, ticket);
        memcpy(host_out16, cmd.dword, sizeof(cmd.dword));
    }
    if (d_out64x16) {
        hipLaunchKernelGGL(k_sqe_image, dim3(1), dim3(BAM_WAVE_SIZE), 0, (hipStream_t)stream, cid, opcode, nsid, prp1, prp2, lba, n_blocks, seal, ticket, d_out64x16);
        hip_err_chk(hipGetLastError());
    }
    BAM_API_END
}

int bam_cache_stream(bam_array_t* a, uint64_t n_waves, uint64_t n_pages_per_wave, const uint64_t* d_assignment, int mode,
                     uint64_t* d_sum, void* stream)
{
    if (!a || !d_sum) return fail(EINVAL, "bam_cache_stream: null argument");
    if (mode < 0 || mode > 6) return fail(EINVAL, "bam_cache_stream: mode must be 0 to 6");
    if (!n_waves || !n_pages_per_wave) return 0;
    BAM_API_BEGIN
    const uint32_t bs = 256;
    const dim3 grid(blocks_for(n_waves * BAM_WAVE_SIZE, bs)), block(bs);
    array_d_t<uint64_t>* d = a->a->d_array_ptr;
    unsigned long long* s = (unsigned long long*)a->partials.get();
    if (mode <= 1 && two_launches_ok(a)) {
        /* the kernel that reads what is resident, then the one that reads what it noted (and folds the checksum) */
        const uint64_t total = n_waves * n_pages_per_wave;
        uint8_t* notes = (uint8_t*)a->notes_for(total);
        unsigned long long* sum = (unsigned long long*)d_sum;
        uint32_t* fin = (uint32_t*)a->finished.get();
        const uint32_t call = a->next_call();
        if (mode == 0) hipLaunchKernelGGL(k_cache_stream<0>, grid, block, 0, (hipStream_t)stream, d, n_waves, n_pages_per_wave, d_assignment, s, notes, sum, fin, call);
        else hipLaunchKernelGGL(k_cache_stream<1>, grid, block, 0, (hipStream_t)stream, d, n_waves, n_pages_per_wave, d_assignment, s, notes, sum, fin, call);
        const uint64_t n_chunks = (total + BAM_WAVE_SIZE - 1) / BAM_WAVE_SIZE;
        const dim3 grid2(blocks_for((n_chunks < 1024 ? n_chunks : 1024) * BAM_WAVE_SIZE, bs));      /* a thousand waves with 64 pages each keep the store busy; when nothing was noted the fewer the better */
        if (mode == 0) hipLaunchKernelGGL(k_cache_stream_deferred<0>, grid2, block, 0, (hipStream_t)stream, d, n_waves, n_pages_per_wave, d_assignment, s, notes, sum, fin, call);
        else hipLaunchKernelGGL(k_cache_stream_deferred<1>, grid2, block, 0, (hipStream_t)stream, d, n_waves, n_pages_per_wave, d_assignment, s, notes, sum, fin, call);
        hip_err_chk(hipGetLastError());
        return 0;
    }
    if (mode == 0 || mode == 5) hipLaunchKernelGGL(k_cache_stream_whole<0>, grid, block, 0, (hipStream_t)stream, d, n_waves, n_pages_per_wave, d_assignment, s);
    else if (mode == 1 || mode == 6) hipLaunchKernelGGL(k_cache_stream_whole<1>, grid, block, 0, (hipStream_t)stream, d, n_waves, n_pages_per_wave, d_assignment, s);
    else if (mode >= 3) {
        /* the lead is counted in pages here: one finished streaming wave stands for its n_pages_per_wave pages */
        fetch_plan fp = make_fetch_plan(a, 1, bs, 1, (hipStream_t)stream);
        fp.lead_elems /= a->a->h_ranges[0].cache.page_size / sizeof(uint64_t);
        const dim3 grid_f(grid.x + fp.blocks);
        if (mode == 3) hipLaunchKernelGGL(k_cache_stream_fetched<3>, grid_f, block, 0, (hipStream_t)stream, d, n_waves, n_pages_per_wave, d_assignment, s, fp);
        else hipLaunchKernelGGL(k_cache_stream_fetched<4>, grid_f, block, 0, (hipStream_t)stream, d, n_waves, n_pages_per_wave, d_assignment, s, fp);
    }
    else hipLaunchKernelGGL(k_cache_stream_pages, grid, block, 0, (hipStream_t)stream, d, n_waves, n_pages_per_wave, d_assignment, s);
    hipLaunchKernelGGL(k_fold_partials, dim3(1), dim3(1024), 0, (hipStream_t)stream, s, (unsigned long long*)d_sum);
    hip_err_chk(hipGetLastError());
    BAM_API_END
}

int bam_block_io(bam_ctrl_t* c, bam_page_cache_t* pc, uint64_t n_reqs, uint32_t req_bytes, const uint64_t* d_lbas, int write,
                 int queue_policy, uint32_t block_size, void* stream)
{
    if (!c || !pc) return fail(EINVAL, "bam_block_io: null argument");
    if (!block_size || block_size % BAM_WAVE_SIZE || block_size > 1024) return fail(EINVAL, "bam_block_io: block size must be a multiple of 64, at most 1024");
    if (n_reqs > pc->pc->pdt.n_pages) return fail(EINVAL, "bam_block_io: needs one cache page per request");
    if (!req_bytes || req_bytes % c->c->blk_size || req_bytes > pc->pc->pdt.page_size) return fail(EINVAL, "bam_block_io: request size must be a multiple of the block size and fit a page");
    if (queue_policy < 0 || queue_policy > 2) return fail(EINVAL, "bam_block_io: queue policy must be 0, 1 or 2");
    if (!n_reqs) return 0;
    BAM_API_BEGIN
    if (queue_policy == 2) {
        if (!pc->pc->pdt.prp1) return fail(EINVAL, "bam_block_io: the per-thread route addresses the cache slots directly, and this cache has no bus addresses for them");
        hipLaunchKernelGGL(k_block_io_per_thread, dim3(blocks_for(n_reqs, block_size)), dim3(block_size), 0, (hipStream_t)stream,
                           pc->pc->pdt.d_ctrls, pc->pc->d_pc_ptr, req_bytes, n_reqs, d_lbas, write);
    } else
        hipLaunchKernelGGL(k_block_io, dim3(blocks_for(n_reqs, block_size)), dim3(block_size), 0, (hipStream_t)stream,
                           pc->pc->pdt.d_ctrls, pc->pc->d_pc_ptr, req_bytes, n_reqs, d_lbas, write, queue_policy);
    hip_err_chk(hipGetLastError());
    BAM_API_END
}

int bam_warp_memcpy(uint64_t* d_dst, const uint64_t* d_src, uint64_t n_words, uint64_t lanes, void* stream)
{
    if (!d_dst || !d_src || !lanes) return fail(EINVAL, "bam_warp_memcpy: null argument or no lane");
    BAM_API_BEGIN
    hipLaunchKernelGGL(k_warp_memcpy, dim3(1), dim3(BAM_WAVE_SIZE), 0, (hipStream_t)stream, d_dst, d_src, n_words, lanes);
    hip_err_chk(hipGetLastError());
    BAM_API_END
}

int bam_unheld_window_cases(bam_array_t* a, uint64_t page, uint32_t* host_out7)
{
    if (!a || !host_out7) return fail(EINVAL, "bam_unheld_window_cases: null argument");
    if (a->a->adt.n_ranges != 1 || page >= a->a->h_ranges[0].page_count) return fail(EINVAL, "bam_unheld_window_cases: an array of one range and a page of it");
    BAM_API_BEGIN
    BufferPtr out = createBuffer(7 * sizeof(uint32_t), 0);
    hip_err_chk(hipMemset(out.get(), 0, 7 * sizeof(uint32_t)));
    hipLaunchKernelGGL(k_unheld_window_cases, dim3(1), dim3(BAM_WAVE_SIZE), 0, 0, a->a->d_array_ptr, page, (uint32_t*)out.get());
    hip_err_chk(hipGetLastError());
    hip_err_chk(hipDeviceSynchronize());
    hip_err_chk(hipMemcpy(host_out7, out.get(), 7 * sizeof(uint32_t), hipMemcpyDeviceToHost));
    BAM_API_END
}

int bam_block_io_async(bam_ctrl_t* c, bam_page_cache_t* pc, uint64_t n_threads, uint32_t depth, uint32_t req_bytes, const uint64_t* d_lbas,
                       uint32_t block_size, void* stream)
{
    if (!c || !pc || !d_lbas) return fail(EINVAL, "bam_block_io_async: null argument");
    if (!block_size || block_size % BAM_WAVE_SIZE || block_size > 1024) return fail(EINVAL, "bam_block_io_async: block size must be a multiple of 64, at most 1024");
    if (depth != 1 && depth != 2 && depth != 4 && depth != 8) return fail(EINVAL, "bam_block_io_async: depth must be 1, 2, 4 or 8");
    if (n_threads * depth > pc->pc->pdt.n_pages) return fail(EINVAL, "bam_block_io_async: needs one cache page per command");
    if (!req_bytes || req_bytes % c->c->blk_size || req_bytes > pc->pc->pdt.page_size) return fail(EINVAL, "bam_block_io_async: request size must be a multiple of the block size and fit a page");
    /* a wave holds `depth` blocks of command ids of its queue pair until it has polled: all waves that can be in
     * flight on one queue pair together must fit its blocks, or they would wait for each other's */
    const uint64_t n_waves = (n_threads + BAM_WAVE_SIZE - 1) / BAM_WAVE_SIZE;
    const uint64_t blocks_per_qp = (c->c->h_qps[0]->sq.cid_mask + 1u) / 64;
    if ((n_waves + c->c->n_qps - 1) / c->c->n_qps * depth > blocks_per_qp)
        return fail(EINVAL, "bam_block_io_async: more commands in flight per queue pair than it has command ids (waves per queue pair x depth x 64)");
    if (!n_threads) return 0;
    BAM_API_BEGIN
    const dim3 grid(blocks_for(n_threads, block_size)), block(block_size);
    hipStream_t st = (hipStream_t)stream;
    Controller** dc = pc->pc->pdt.d_ctrls;
    page_cache_d_t* dp = pc->pc->d_pc_ptr;
    switch (depth) {
    case 1: hipLaunchKernelGGL(k_block_io_async<1>, grid, block, 0, st, dc, dp, req_bytes, n_threads, d_lbas); break;
    case 2: hipLaunchKernelGGL(k_block_io_async<2>, grid, block, 0, st, dc, dp, req_bytes, n_threads, d_lbas); break;
    case 4: hipLaunchKernelGGL(k_block_io_async<4>, grid, block, 0, st, dc, dp, req_bytes, n_threads, d_lbas); break;
    default: hipLaunchKernelGGL(k_block_io_async<8>, grid, block, 0, st, dc, dp, req_bytes, n_threads, d_lbas); break;
    }
    hip_err_chk(hipGetLastError());
    BAM_API_END
}

namespace {
/* a file mapped read-only, or created and mapped for writing */
struct mapped_file {
    int fd = -1;
    uint8_t* p = nullptr;
    size_t size = 0;
    int open_ro(const char* path)
    {
        fd = ::open(path, O_RDONLY);
        if (fd < 0) return errno;
        struct stat sb;
        if (fstat(fd, &sb)) return errno;
        size = (size_t)sb.st_size;
        if (size) { void* m = mmap(nullptr, size, PROT_READ, MAP_PRIVATE, fd, 0); if (m == MAP_FAILED) return errno; p = (uint8_t*)m; }
        return 0;
    }
    int create_rw(const char* path, size_t bytes)
    {
        fd = ::open(path, O_RDWR | O_CREAT | O_TRUNC, 0644);
        if (fd < 0) return errno;
        if (ftruncate(fd, (off_t)bytes)) return errno;
        size = bytes;
        if (size) { void* m = mmap(nullptr, size, PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0); if (m == MAP_FAILED) return errno; p = (uint8_t*)m; }
        return 0;
    }
    ~mapped_file() { if (p) munmap(p, size); if (fd >= 0) ::close(fd); }
};

int check_store_span(bam_ctrl_t* c, bam_page_cache_t* pc, uint64_t store_offset, uint64_t n_bytes, const char* who)
{
    const uint64_t ps = pc->pc->pdt.page_size;
    if (store_offset % ps) return fail(EINVAL, std::string(who) + ": the store offset must be a multiple of the page size");
    const uint64_t ns_bytes = (uint64_t)c->c->ns.size * c->c->blk_size;
    const uint64_t padded = (n_bytes + ps - 1) / ps * ps;
    if (store_offset > ns_bytes || padded > ns_bytes - store_offset) return fail(ERANGE, std::string(who) + ": past the end of the namespace");
    return 0;
}
} // namespace

int bam_store_write_file(bam_ctrl_t* c, bam_page_cache_t* pc, const char* path, uint64_t file_offset, uint64_t store_offset, uint64_t n_bytes,
                         uint64_t* bytes_done)
{
    if (!c || !pc || !path) return fail(EINVAL, "bam_store_write_file: null argument");
    BAM_API_BEGIN
    mapped_file in;
    if (int rc = in.open_ro(path)) return fail(rc, std::string("bam_store_write_file: ") + path + ": " + strerror(rc));
    if (file_offset > in.size) return fail(ERANGE, "bam_store_write_file: offset past the end of the file");
    if (!n_bytes) n_bytes = in.size - file_offset;
    if (n_bytes > in.size - file_offset) return fail(ERANGE, "bam_store_write_file: more bytes than the file holds");
    if (int rc = check_store_span(c, pc, store_offset, n_bytes, "bam_store_write_file")) return rc;
    const uint64_t ps = pc->pc->pdt.page_size, cache_bytes = ps * pc->pc->pdt.n_pages;
    uint64_t done = 0;
    while (done < n_bytes) {
        const uint64_t chunk = std::min(cache_bytes, n_bytes - done);
        const uint64_t n_slots = (chunk + ps - 1) / ps;
        hip_err_chk(hipMemcpy(pc->pc->pdt.base_addr, in.p + file_offset + done, chunk, hipMemcpyHostToDevice));
        if (chunk % ps) hip_err_chk(hipMemset(pc->pc->pdt.base_addr + chunk, 0, n_slots * ps - chunk));      /* the tail of the last page */
        hipLaunchKernelGGL(k_sequential_access, dim3(blocks_for(std::min<uint64_t>(n_slots, 1u << 18), 64)), dim3(64), 0, 0,
                           pc->pc->pdt.d_ctrls, pc->pc->d_pc_ptr, (uint32_t)ps, n_slots, store_offset + done, 1);
        hip_err_chk(hipGetLastError());
        hip_err_chk(hipDeviceSynchronize());
        if (c->c->aborted()) return fail(EIO, "bam_store_write_file: a device-side wait gave up");
        done += chunk;
    }
    if (bytes_done) *bytes_done = done;
    BAM_API_END
}

int bam_store_read_file(bam_ctrl_t* c, bam_page_cache_t* pc, const char* path, uint64_t store_offset, uint64_t n_bytes)
{
    if (!c || !pc || !path || !n_bytes) return fail(EINVAL, "bam_store_read_file: null argument or nothing to read");
    BAM_API_BEGIN
    if (int rc = check_store_span(c, pc, store_offset, n_bytes, "bam_store_read_file")) return rc;
    mapped_file out;
    if (int rc = out.create_rw(path, n_bytes)) return fail(rc, std::string("bam_store_read_file: ") + path + ": " + strerror(rc));
    const uint64_t ps = pc->pc->pdt.page_size, cache_bytes = ps * pc->pc->pdt.n_pages;
    uint64_t done = 0;
    while (done < n_bytes) {
        const uint64_t chunk = std::min(cache_bytes, n_bytes - done);
        const uint64_t n_slots = (chunk + ps - 1) / ps;
        hipLaunchKernelGGL(k_sequential_access, dim3(blocks_for(std::min<uint64_t>(n_slots, 1u << 18), 64)), dim3(64), 0, 0,
                           pc->pc->pdt.d_ctrls, pc->pc->d_pc_ptr, (uint32_t)ps, n_slots, store_offset + done, 0);
        hip_err_chk(hipGetLastError());
        hip_err_chk(hipDeviceSynchronize());
        if (c->c->aborted()) return fail(EIO, "bam_store_read_file: a device-side wait gave up");
        hip_err_chk(hipMemcpy(out.p + done, pc->pc->pdt.base_addr, chunk, hipMemcpyDeviceToHost));
        done += chunk;
    }
    if (msync(out.p, out.size, MS_SYNC)) return fail(errno, "bam_store_read_file: msync failed");
    BAM_API_END
}

int bam_block_checksum(bam_page_cache_t* pc, uint64_t n_slots, uint32_t req_bytes, uint64_t* d_out, void* stream)
{
    if (!pc || !d_out) return fail(EINVAL, "bam_block_checksum: null argument");
    if (n_slots > pc->pc->pdt.n_pages || req_bytes > pc->pc->pdt.page_size || req_bytes % 8) return fail(EINVAL, "bam_block_checksum: out of range");
    if (!n_slots) return 0;
    BAM_API_BEGIN
    hipLaunchKernelGGL(k_block_checksum, dim3(blocks_for(n_slots * BAM_WAVE_SIZE, 256)), dim3(256), 0, (hipStream_t)stream,
                       pc->pc->d_pc_ptr, n_slots, req_bytes, d_out);
    hip_err_chk(hipGetLastError());
    BAM_API_END
}

// ---- arrays of 32-bit elements and SSSP ----
int bam_range32_create(bam_range32_t** out, uint64_t index_start, uint64_t count, uint64_t page_start, uint64_t page_count,
                       uint64_t page_start_offset, uint64_t page_size, bam_page_cache_t* pc, uint32_t device, int dist)
{
    if (!out || !pc) return fail(EINVAL, "bam_range32_create: null argument");
    *out = nullptr;
    if (dist != REPLICATE && dist != STRIPE) return fail(EINVAL, "bam_range32_create: unknown distribution");
    if (page_size != pc->pc->pdt.page_size) return fail(EINVAL, "bam_range32_create: page size differs from the cache's");
    if (page_start_offset >= page_size || page_start_offset % sizeof(uint32_t) || count <= index_start || page_count == 0)
        return fail(EINVAL, "bam_range32_create: empty or misaligned range");
    if (((count - index_start) * sizeof(uint32_t) + page_start_offset + page_size - 1) / page_size > page_count)
        return fail(EINVAL, "bam_range32_create: page_count does not cover the elements");
    BAM_API_BEGIN
    *out = new bam_range32{new range_t<uint32_t>(index_start, count, page_start, page_count, page_start_offset, page_size, pc->pc, device, (data_dist_t)dist)};
    BAM_API_END
}

void bam_range32_destroy(bam_range32_t* r)
{
    if (!r) return;
    delete r->r;
    delete r;
}

int bam_array32_create(bam_array32_t** out, uint64_t n_elems, uint64_t disk_start_offset, bam_range32_t** ranges, uint32_t n_ranges, uint32_t device)
{
    if (!out || !ranges || !n_ranges) return fail(EINVAL, "bam_array32_create: null argument");
    *out = nullptr;
    BAM_API_BEGIN
    std::vector<range_t<uint32_t>*> rs;
    for (uint32_t i = 0; i < n_ranges; i++) rs.push_back(ranges[i]->r);
    *out = new bam_array32{new array_t<uint32_t>(n_elems, disk_start_offset, rs, device), createBuffer(BAM_SUM_PARTIALS * sizeof(uint64_t), device)};
    BAM_API_END
}

void bam_array32_destroy(bam_array32_t* a)
{
    if (!a) return;
    delete a->a;
    delete a;
}

int bam_array32_stats(bam_array32_t* a, uint64_t* out)
{
    if (!a || !out) return fail(EINVAL, "bam_array32_stats: null argument");
    BAM_API_BEGIN
    hip_err_chk(hipDeviceSynchronize());
    bam_array_counters t = a->a->reset_stats();
    out[0] = t.read_io_cnt; out[1] = t.access_cnt; out[2] = t.miss_cnt; out[3] = t.hit_cnt;
    BAM_API_END
}

int bam_array32_read(bam_array32_t* a, uint64_t n_reqs, const uint64_t* d_assignment, uint64_t stride, uint32_t block_size, uint64_t* d_sum, void* stream)
{
    if (!a || !d_sum) return fail(EINVAL, "bam_array32_read: null argument");
    if (!block_size || block_size % BAM_WAVE_SIZE || block_size > 1024) return fail(EINVAL, "bam_array32_read: block size must be a multiple of 64, at most 1024");
    if (!n_reqs) return 0;
    BAM_API_BEGIN
    hipLaunchKernelGGL(k_array32_read, dim3(blocks_for(n_reqs, block_size)), dim3(block_size), 0, (hipStream_t)stream,
                       a->a->d_array_ptr, n_reqs, d_assignment, stride, (unsigned long long*)a->partials.get());
    hipLaunchKernelGGL(k_fold_partials, dim3(1), dim3(1024), 0, (hipStream_t)stream, (unsigned long long*)a->partials.get(), (unsigned long long*)d_sum);
    hip_err_chk(hipGetLastError());
    BAM_API_END
}

int bam_gen_words(uint64_t seed, uint64_t first, uint64_t n, uint64_t* d_out, void* stream)
{
    if (!d_out) return fail(EINVAL, "bam_gen_words: null argument");
    if (!n) return 0;
    BAM_API_BEGIN
    hipLaunchKernelGGL(k_gen_words, dim3(blocks_for(n, 256)), dim3(256), 0, (hipStream_t)stream, seed, first, n, d_out);
    hip_err_chk(hipGetLastError());
    BAM_API_END
}

int bam_gen_mod(uint64_t seed, uint64_t first, uint64_t n, uint64_t modulus, uint64_t scale, uint64_t* d_out, void* stream)
{
    if (!d_out || !modulus) return fail(EINVAL, "bam_gen_mod: null argument or zero modulus");
    if (!n) return 0;
    BAM_API_BEGIN
    hipLaunchKernelGGL(k_gen_mod, dim3(blocks_for(n, 256)), dim3(256), 0, (hipStream_t)stream, seed, first, n, modulus, scale, d_out);
    hip_err_chk(hipGetLastError());
    BAM_API_END
}

int bam_gen_rmat(uint64_t seed, uint32_t scale, uint64_t first_edge, uint64_t n, uint64_t* d_u, uint64_t* d_v, void* stream)
{
    if (!d_u || !d_v || !scale || scale > 40) return fail(EINVAL, "bam_gen_rmat: bad argument");
    if (!n) return 0;
    BAM_API_BEGIN
    hipLaunchKernelGGL(k_gen_rmat, dim3(blocks_for(n, 256)), dim3(256), 0, (hipStream_t)stream, seed, scale, first_edge, n, d_u, d_v);
    hip_err_chk(hipGetLastError());
    BAM_API_END
}

int bam_gen_uniform(uint64_t seed, uint64_t n_vertices, uint64_t first_pair, uint64_t n, uint64_t* d_u, uint64_t* d_v, void* stream)
{
    if (!d_u || !d_v || !n_vertices) return fail(EINVAL, "bam_gen_uniform: bad argument");
    if (!n) return 0;
    BAM_API_BEGIN
    hipLaunchKernelGGL(k_gen_uniform, dim3(blocks_for(n, 256)), dim3(256), 0, (hipStream_t)stream, seed, n_vertices, first_pair, n, d_u, d_v);
    hip_err_chk(hipGetLastError());
    BAM_API_END
}

int bam_copy_kernel(const void* d_src, void* d_dst, uint64_t n_bytes, float* ms, void* stream)
{
    if (!d_src || !d_dst || n_bytes % 16) return fail(EINVAL, "bam_copy_kernel: bad argument");
    BAM_API_BEGIN
    hipStream_t st = (hipStream_t)stream;
    Event a(st);
    hipLaunchKernelGGL(k_copy16, dim3(256 * 16), dim3(256), 0, st, (const uint4*)d_src, (uint4*)d_dst, n_bytes / 16);
    hip_err_chk(hipGetLastError());
    Event b(st);
    if (ms) *ms = (float)((b - a) / 1e3);
    BAM_API_END
}

int bam_read_kernel(const void* d_src, uint64_t n_bytes, float* ms, void* stream)
{
    if (!d_src || n_bytes % 16) return fail(EINVAL, "bam_read_kernel: bad argument");
    BAM_API_BEGIN
    hipStream_t st = (hipStream_t)stream;
    BufferPtr partials = createBuffer(BAM_SUM_PARTIALS * sizeof(unsigned long long), 0);
    Event a(st);
    /* 16 KiB per wave at 1 GiB: many short waves carry more than few long ones here */
    hipLaunchKernelGGL(k_read_stream, dim3(256 * 64), dim3(256), 0, st, (const uint64_t*)d_src, n_bytes / 8, (unsigned long long*)partials.get());
    hip_err_chk(hipGetLastError());
    Event b(st);
    if (ms) *ms = (float)((b - a) / 1e3);
    BAM_API_END
}

int bam_hit_path_parts(bam_array_t* a, int refs, int not_kept, uint64_t n_waves, uint64_t n_pages_per_wave, uint64_t* d_sum, void* stream)
{
    if (!a || !d_sum || refs < 0 || refs > 2) return fail(EINVAL, "bam_hit_path_parts: bad argument");
    if (a->a->adt.n_ranges != 1 || a->a->h_ranges[0].cache.page_size != 4096) return fail(EINVAL, "bam_hit_path_parts: one range of 4 KiB pages");
    if (n_waves * n_pages_per_wave > a->a->h_ranges[0].page_count) return fail(EINVAL, "bam_hit_path_parts: more pages than the range has");
    if (!n_waves || !n_pages_per_wave) return 0;
    BAM_API_BEGIN
    hipStream_t st = (hipStream_t)stream;
    array_d_t<uint64_t>* d = a->a->d_array_ptr;
    unsigned long long* s = (unsigned long long*)a->partials.get();
    const dim3 grid(blocks_for(n_waves * BAM_WAVE_SIZE, 256)), block(256);
    switch (refs * 2 + (not_kept ? 1 : 0)) {
    case 0: hipLaunchKernelGGL((k_hit_path_parts<0, false>), grid, block, 0, st, d, n_waves, n_pages_per_wave, s); break;
    case 1: hipLaunchKernelGGL((k_hit_path_parts<0, true>), grid, block, 0, st, d, n_waves, n_pages_per_wave, s); break;
    case 2: hipLaunchKernelGGL((k_hit_path_parts<1, false>), grid, block, 0, st, d, n_waves, n_pages_per_wave, s); break;
    case 3: hipLaunchKernelGGL((k_hit_path_parts<1, true>), grid, block, 0, st, d, n_waves, n_pages_per_wave, s); break;
    case 4: hipLaunchKernelGGL((k_hit_path_parts<2, false>), grid, block, 0, st, d, n_waves, n_pages_per_wave, s); break;
    default: hipLaunchKernelGGL((k_hit_path_parts<2, true>), grid, block, 0, st, d, n_waves, n_pages_per_wave, s); break;
    }
    hipLaunchKernelGGL(k_fold_partials, dim3(1), dim3(1024), 0, st, s, (unsigned long long*)d_sum);
    hip_err_chk(hipGetLastError());
    BAM_API_END
}

int bam_gather_kernel(const uint64_t* d_src, const uint64_t* d_idx, uint64_t n, float* ms, void* stream)
{
    if (!d_src || !d_idx || !n) return fail(EINVAL, "bam_gather_kernel: bad argument");
    BAM_API_BEGIN
    hipStream_t st = (hipStream_t)stream;
    BufferPtr partials = createBuffer(BAM_SUM_PARTIALS * sizeof(unsigned long long), 0);
    Event a(st);
    hipLaunchKernelGGL(k_gather8, dim3(blocks_for(n, 256)), dim3(256), 0, st, d_src, d_idx, n, (unsigned long long*)partials.get());
    hip_err_chk(hipGetLastError());
    Event b(st);
    if (ms) *ms = (float)((b - a) / 1e3);
    BAM_API_END
}

int bam_atomic_pairs_kernel(uint64_t* d_table, const uint64_t* d_idx, uint64_t n, int returns, float* ms, void* stream)
{
    if (!d_table || !d_idx || !n) return fail(EINVAL, "bam_atomic_pairs_kernel: bad argument");
    BAM_API_BEGIN
    hipStream_t st = (hipStream_t)stream;
    BufferPtr partials = createBuffer(BAM_SUM_PARTIALS * sizeof(unsigned long long), 0);
    Event a(st);
    if (returns) hipLaunchKernelGGL(k_atomic_pairs<1>, dim3(blocks_for(n, 256)), dim3(256), 0, st, (unsigned long long*)d_table, d_idx, n, (unsigned long long*)partials.get());
    else hipLaunchKernelGGL(k_atomic_pairs<0>, dim3(blocks_for(n, 256)), dim3(256), 0, st, (unsigned long long*)d_table, d_idx, n, (unsigned long long*)partials.get());
    hip_err_chk(hipGetLastError());
    Event b(st);
    if (ms) *ms = (float)((b - a) / 1e3);
    BAM_API_END
}

int bam_xcd_relay(bam_array_t* a, uint64_t seed, uint32_t page_bytes, uint32_t n_pages, uint32_t rounds, uint32_t n_waves, uint32_t spin_limit, uint64_t* out4, void* stream)
{
    if (!a || !out4 || page_bytes < 512 || !n_pages || !rounds || n_waves < 2 || n_waves > 256) return fail(EINVAL, "bam_xcd_relay: bad argument (2 to 256 waves)");
    BAM_API_BEGIN
    hipStream_t st = (hipStream_t)stream;
    /* every wave must be running while the others wait for it: 256 workgroups of one wave fit the device many times over */
    BufferPtr words = createBuffer((2ull * rounds) * sizeof(uint32_t) + 4 * sizeof(unsigned long long), 0);
    hip_err_chk(hipMemsetAsync(words.get(), 0, (2ull * rounds) * sizeof(uint32_t) + 4 * sizeof(unsigned long long), st));
    unsigned long long* out = (unsigned long long*)words.get();
    uint32_t* flag = (uint32_t*)(out + 4);
    const uint32_t per_page = page_bytes / (uint32_t)sizeof(uint64_t);
    hipLaunchKernelGGL(k_xcd_relay, dim3(n_waves), dim3(BAM_WAVE_SIZE), 0, st, a->a->d_array_ptr, seed, n_pages, rounds, per_page, spin_limit ? spin_limit : 1u << 22, flag, flag + rounds, out);
    hip_err_chk(hipGetLastError());
    hip_err_chk(hipMemcpyAsync(out4, out, 4 * sizeof(uint64_t), hipMemcpyDeviceToHost, st));
    hip_err_chk(hipStreamSynchronize(st));
    BAM_API_END
}

int bam_host_read_ceiling(uint64_t n_bytes, uint32_t chunk_bytes, float* ms)
{
    if (!n_bytes || !chunk_bytes || chunk_bytes % 1024) return fail(EINVAL, "bam_host_read_ceiling: chunk must be a multiple of 1024 bytes");
    BAM_API_BEGIN
    const uint64_t window = n_bytes < (256ull << 20) ? n_bytes : (256ull << 20);
    const uint64_t host_chunks = window / chunk_bytes;
    if (!host_chunks) return fail(EINVAL, "bam_host_read_ceiling: less than one chunk");
    BufferPtr host = createHostBuffer(window), dev = createBuffer(window, 0);
    const uint64_t n_chunks = n_bytes / chunk_bytes;
    for (int rep = 0; rep < 2; rep++) {           /* first pass warms mappings */
        Event a(0);
        hipLaunchKernelGGL(k_host_pull, dim3(256 * 8), dim3(256), 0, 0, (const uint4*)host.get(), (uint4*)dev.get(), n_chunks, chunk_bytes / 16, host_chunks);
        hip_err_chk(hipGetLastError());
        Event b(0);
        if (ms) *ms = (float)((b - a) / 1e3);
    }
    BAM_API_END
}

int bam_event_create(void** ev)
{
    if (!ev) return fail(EINVAL, "bam_event_create: null argument");
    BAM_API_BEGIN
    hipEvent_t e;
    hip_err_chk(hipEventCreate(&e));
    *ev = (void*)e;
    BAM_API_END
}

int bam_event_record(void* ev, void* stream)
{
    BAM_API_BEGIN
    hip_err_chk(hipEventRecord((hipEvent_t)ev, (hipStream_t)stream));
    BAM_API_END
}

int bam_event_elapsed_ms(void* start, void* stop, float* ms)
{
    if (!ms) return fail(EINVAL, "bam_event_elapsed_ms: null argument");
    BAM_API_BEGIN
    hip_err_chk(hipEventSynchronize((hipEvent_t)stop));
    hip_err_chk(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    BAM_API_END
}

void bam_event_destroy(void* ev)
{
    if (ev) (void)hipEventDestroy((hipEvent_t)ev);
}

double bam_target_ceiling_iops(uint64_t ns_bytes, uint32_t lba_bytes, int backing, uint32_t n_io_threads, uint32_t n_clients,
                               uint32_t depth, uint64_t n_cmds, uint32_t req_bytes)
{
    nvmt_config_t c{};
    c.ns_bytes = ns_bytes; c.lba_bytes = lba_bytes; c.seed = 42; c.n_io_threads = n_io_threads;
    c.max_queue_entries = 1024; c.max_io_queues = 128; c.dstrd = 4;
    void* mem = nullptr;
    if (backing) {
        if (posix_memalign(&mem, 4096, ns_bytes)) return -1.0;
        fill_backing(42, (uint64_t*)mem, ns_bytes / 8);
        c.backing = mem;
    }
    double r = nvmt_selftest_iops(&c, n_clients, depth, n_cmds, req_bytes);
    free(mem);
    return r;
}

} // extern "C"
