// C-ABI of the GPU-side storage-access path: handle management over the C++
// host objects (ctrl.h, page_cache.h) and the gfx950 kernels that drive them.
// Kernel shapes follow the reference's benchmark kernels (cited per kernel);
// lane arithmetic is for 64-wide waves.
#include "bam_amd.h"

#include <hip/hip_runtime.h>
#include <hipcub/hipcub.hpp>
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
static thread_local std::string g_err;

#define BAM_API_BEGIN try {
#define BAM_API_END                                                        \
    return 0;                                                              \
    } catch (const std::exception& e) { g_err = e.what(); return EIO; }    \
      catch (...) { g_err = "unknown error"; return EIO; }

static int fail(int code, const char* msg) { g_err = msg; return code; }
static int fail(int code, const std::string& msg) { g_err = msg; return code; }

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
struct bam_array { array_t<uint64_t>* a; BufferPtr partials; };
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

/* one block of 1024 threads: *sum += all shards; shards are left zero for the next launch */
__global__ void k_fold_partials(unsigned long long* partials, unsigned long long* sum)
{
    uint64_t v = 0;
    for (uint32_t i = threadIdx.x; i < BAM_SUM_PARTIALS; i += blockDim.x) { v += partials[i]; partials[i] = 0; }
    v = wave_sum(v);
    if (bam::lane() == 0 && v) atomicAdd(sum, (unsigned long long)v);
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
            v = bam::ld_payload(pg.addr + pg.offset);
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
template <int MODE>
__device__ __forceinline__ void cache_stream_body(array_d_t<uint64_t>* dr, uint64_t n_waves, uint64_t n_pages_per_wave, const uint64_t* assignment, unsigned long long* sum)
{
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint64_t wave = tid / BAM_WAVE_SIZE, lane = tid % BAM_WAVE_SIZE;
    uint64_t v = 0;
    if (wave < n_waves) {
        range_d_t<uint64_t>* r0 = dr->d_ranges;
        const uint64_t epp = r0->n_elems_per_page;
        const uint64_t start_page = assignment ? assignment[wave] : wave * n_pages_per_wave;
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
            /* a wave reads its pages one after the other: those of the next stretch that are not resident are touched
             * together, one page per lane, so that a cold run asks the store for a batch per stretch and not for a page
             * per trip (1.5 M pages/s otherwise); on a resident cache this costs one look at a state word per page */
            /* (modes 3 and 4: the helper needs more registers than the kernels themselves, which costs them a third of the
             * waves they run with on a resident cache, hence modes 0 and 1 without) */
            const uint32_t reach = MODE < 3 || dr->n_ranges != 1 ? 0 : (uint32_t)(r0->cache.n_pages >> 6 > BAM_WAVE_SIZE ? BAM_WAVE_SIZE : r0->cache.n_pages >> 6);
            for (uint64_t p = 0; p < n_pages_per_wave; p++) {
                if (MODE >= 3 && reach >= 2 && p % reach == 0) stream_touch(r0, start_page + p, n_pages_per_wave - p < reach ? n_pages_per_wave - p : reach);
                const uint64_t start_idx = (start_page + p) * epp + lane;
                if (MODE == 0 || MODE == 4) {
                    for (uint64_t j = 0; j < epp; j += BAM_WAVE_SIZE) v += (*dr)[start_idx + j];
                } else {
                    /* eight elements asked for before the first is used: the window test of an element needs nothing that
                     * an earlier load brings, so the loads of a page are in flight together */
                    for (uint64_t j = 0; j < epp; j += 8 * BAM_WAVE_SIZE) {
                        uint64_t x[8];
#pragma unroll
                        for (int u = 0; u < 8; u++) x[u] = j + u * BAM_WAVE_SIZE < epp ? (uint64_t)ptr[start_idx + j + u * BAM_WAVE_SIZE] : 0;
                        v += ((x[0] + x[1]) + (x[2] + x[3])) + ((x[4] + x[5]) + (x[6] + x[7]));
                    }
                }
            }
        }
    }
    block_accumulate(sum, v);
}

/* one kernel per mode; the page-wise one has a name of its own because it is the one the hit-path roofline is quoted on */
template <int MODE>
__global__ __launch_bounds__(256) void k_cache_stream(array_d_t<uint64_t>* dr, uint64_t n_waves, uint64_t n_pages_per_wave, const uint64_t* assignment, unsigned long long* sum)
{
    cache_stream_body<MODE>(dr, n_waves, n_pages_per_wave, assignment, sum);
}
__global__ __launch_bounds__(256) void k_cache_stream_pages(array_d_t<uint64_t>* dr, uint64_t n_waves, uint64_t n_pages_per_wave, const uint64_t* assignment, unsigned long long* sum)
{
    cache_stream_body<2>(dr, n_waves, n_pages_per_wave, assignment, sum);
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
        if (bam::ballot(take_1)) view.acquire_helped(take_f ? pf : adopted, take_1, false, touch, touch);
        /* last pages nobody had a lane for */
        const bool take_2 = take_l && bam::popc(need_l & bam::lanes_below(bam::lane())) >= bam::popc(idle);
        if (bam::ballot(take_2)) view.acquire_helped(pl, take_2, false, touch, touch);
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
            if (bam::ballot(take)) view.acquire_helped(c + lane, take, false, touch, touch);
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
        if (bam::ballot(take)) view.acquire_helped(page, take, false, touch, touch);
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
        if (bam::ballot(take)) view.acquire_helped(p, take, false, touch, touch);
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
    for (;;) {
        unsigned long long w = 0;
        if (laneIdx == 0) w = atomicAdd(next_work, 1ull);
        w = bam::bcast((uint64_t)w, 0);
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

__global__ __launch_bounds__(128) void k_bfs_coalesce_coarse_ptr_pc(array_d_t<uint64_t>* da, uint32_t* label, const uint32_t level, const uint64_t vertex_count,
                                                                   const uint64_t* vertexList, uint64_t* changed, uint64_t coarse,
                                                                   const heavy_piece_t* heavy, uint64_t n_heavy, unsigned long long* next_work)
{
    bool any = false;
    walk_vertex_groups(da, vertexList, vertex_count, coarse, heavy, n_heavy, next_work, (level & 1u) != 0,
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

__global__ __launch_bounds__(128) void k_bfs_frontier_coalesce_ptr_pc(array_d_t<uint64_t>* da, uint32_t* label, const uint32_t level, const uint64_t* vertexList,
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

__global__ __launch_bounds__(128) void k_cc_coalesce_coarse_ptr_pc(array_d_t<uint64_t>* da, bool* curr_visit, bool* next_visit, uint64_t vertex_count,
                                                                  const uint64_t* vertexList, unsigned long long* comp, bool* changed, uint64_t coarse,
                                                                  const heavy_piece_t* heavy, uint64_t n_heavy, unsigned long long* next_work, uint32_t sweep)
{
    walk_vertex_groups(da, vertexList, vertex_count, coarse, heavy, n_heavy, next_work, (sweep & 1u) != 0,
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

// ---- vectoradd (benchmarks/vectoradd/main.cu:102-117 kernel_baseline_ptr_pc): C[i] = A[i] + B[i], all three behind the cache ----
__global__ __launch_bounds__(64) void k_vectoradd_ptr_pc(array_d_t<uint64_t>* da, array_d_t<uint64_t>* db, uint64_t n_elems, array_d_t<uint64_t>* dc)
{
    const uint64_t tid = (uint64_t)blockDim.x * blockIdx.x + threadIdx.x;
    bam_ptr<uint64_t> Aptr(da);
    bam_ptr<uint64_t> Bptr(db);
    bam_ptr<uint64_t> Cptr(dc);
    const bam_ptr<uint64_t>& A = Aptr;
    const bam_ptr<uint64_t>& B = Bptr;
    const uint64_t first = tid - threadIdx.x % BAM_WAVE_SIZE;
    if (first < n_elems) {
        touch_ahead(da, first, n_elems, BAM_WAVE_SIZE, 0);
        touch_ahead(db, first, n_elems, BAM_WAVE_SIZE, 1);
        touch_ahead(dc, first, n_elems, BAM_WAVE_SIZE, 2);
    }
    if (tid < n_elems) Cptr[tid] = A[tid] + B[tid];
}

// ---- reduction (benchmarks/reduction/main.cu:166-195 kernel_reduce_baseline_ptr_pc): output[b] = sum of the 2 x blockDim elements of block b ----
__global__ void k_reduce_ptr_pc(array_d_t<uint64_t>* da, unsigned long long* output, uint64_t len)
{
    __shared__ uint64_t wave_total[1024 / BAM_WAVE_SIZE];
    const uint64_t tid = threadIdx.x, start = 2ull * blockDim.x * blockIdx.x;
    uint64_t v = 0;
    {
        bam_ptr<uint64_t> in_ptr(da);
        const bam_ptr<uint64_t>& input = in_ptr;
        /* a workgroup reads 2 x blockDim consecutive elements: its waves' first elements */
        const uint64_t first = start + tid - tid % BAM_WAVE_SIZE;
        if (first < len) touch_ahead(da, first, len);
        if (first + blockDim.x < len) touch_ahead(da, first + blockDim.x, len);
        if (start + tid < len) v = input[start + tid];
        if (blockDim.x + start + tid < len) v += input[blockDim.x + start + tid];
    }
    v = wave_sum(v);
    if (bam::lane() == 0) wave_total[tid / BAM_WAVE_SIZE] = v;
    __syncthreads();
    if (tid < BAM_WAVE_SIZE) {
        v = wave_sum(tid < blockDim.x / BAM_WAVE_SIZE ? wave_total[tid] : 0);
        if (tid == 0) output[blockIdx.x] = v;
    }
}

// ---- scan (benchmarks/scan/main.cu:147-190 kernel_scan_baseline_ptr_pc, :89-100 finalsum) ----
/* inclusive sums over the 64 lanes of a wave (all lanes active) */
__device__ __forceinline__ uint64_t wave_inclusive_sum(uint64_t v)
{
    const uint32_t lane = bam::lane();
#pragma unroll
    for (uint32_t o = 1; o < BAM_WAVE_SIZE; o <<= 1) {
        const uint64_t u = bam::shfl(v, lane >= o ? lane - o : lane);
        if (lane >= o) v += u;
    }
    return v;
}

/*
 * Block b scans its 2 x blockDim elements: output[i] = sum of the block's elements up to and including i,
 * intermediate[b] = the block's total.  The elements are read as the reference reads them (thread t takes t and
 * t + blockDim, so a wave reads consecutive elements through one page reference); the scan itself runs over wave
 * shuffles on pairs of neighbours rather than the two tree passes over shared memory.
 */
__global__ void k_scan_ptr_pc(array_d_t<uint64_t>* da, unsigned long long* output, unsigned long long* intermediate, uint64_t len)
{
    extern __shared__ uint64_t scan_mem[];                      /* 2 x blockDim elements, then one total per wave */
    const uint32_t B = blockDim.x, t = threadIdx.x;
    uint64_t* wave_total = scan_mem + 2 * B;
    const uint64_t idx = 2ull * blockIdx.x * B + t;
    {
        bam_ptr<uint64_t> in_ptr(da);
        const bam_ptr<uint64_t>& ptr = in_ptr;
        const uint64_t first = idx - t % BAM_WAVE_SIZE;
        if (first < len) touch_ahead(da, first, len);
        if (first + B < len) touch_ahead(da, first + B, len);
        scan_mem[t] = idx < len ? ptr[idx] : 0;
        scan_mem[t + B] = idx + B < len ? ptr[idx + B] : 0;
    }
    __syncthreads();
    const uint64_t a = scan_mem[2 * t], b = a + scan_mem[2 * t + 1];
    const uint64_t s = wave_inclusive_sum(b);
    if (bam::lane() == BAM_WAVE_SIZE - 1) wave_total[t / BAM_WAVE_SIZE] = s;
    __syncthreads();
    uint64_t before = s - b;
    for (uint32_t w = 0; w < t / BAM_WAVE_SIZE; w++) before += wave_total[w];
    scan_mem[2 * t] = before + a;
    scan_mem[2 * t + 1] = before + b;
    __syncthreads();
    if (idx < len) output[idx] = scan_mem[t];
    if (idx + B < len) output[idx + B] = scan_mem[t + B];
    if (intermediate && t == B - 1) intermediate[blockIdx.x] = before + b;
}

/* one block: v[i] = v[0] + ... + v[i] in place (the reference calls cub::DeviceScan::InclusiveSum here, scan/main.cu:416-418) */
__global__ void k_scan_block_totals(unsigned long long* v, uint64_t n)
{
    __shared__ uint64_t wave_total[1024 / BAM_WAVE_SIZE];
    __shared__ uint64_t carry_s;
    const uint32_t t = threadIdx.x;
    if (t == 0) carry_s = 0;
    __syncthreads();
    for (uint64_t base = 0; base < n; base += blockDim.x) {
        const uint64_t x = base + t < n ? v[base + t] : 0;
        const uint64_t s = wave_inclusive_sum(x);
        if (bam::lane() == BAM_WAVE_SIZE - 1) wave_total[t / BAM_WAVE_SIZE] = s;
        __syncthreads();
        uint64_t r = carry_s + s;
        for (uint32_t w = 0; w < t / BAM_WAVE_SIZE; w++) r += wave_total[w];
        if (base + t < n) v[base + t] = r;
        __syncthreads();
        if (t == blockDim.x - 1) carry_s = r;
        __syncthreads();
    }
}

__global__ void k_scan_finalsum(const unsigned long long* scanned_totals, unsigned long long* output, uint64_t len)
{
    if (blockIdx.x == 0) return;
    const uint64_t B = blockDim.x, idx = 2ull * blockIdx.x * B + threadIdx.x;
    const uint64_t add = scanned_totals[blockIdx.x - 1];
    if (idx < len) output[idx] += add;
    if (idx + B < len) output[idx + B] += add;
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
__global__ __launch_bounds__(128) void k_pr_coalesce_pc(array_d_t<uint64_t>* da, const bool* label, const float* delta, float* residual,
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
__global__ __launch_bounds__(128) void k_sssp_coalesce_pc(array_d_t<uint64_t>* de, array_d_t<uint32_t>* dw, const bool* label, uint32_t* newCostList,
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

/* one thread per request over an array of 32-bit elements: sum of the values read */
__global__ void k_array32_read(array_d_t<uint32_t>* dr, uint64_t n_reqs, const uint64_t* assignment, uint64_t stride, unsigned long long* sum)
{
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    uint64_t v = 0;
    if (tid < n_reqs) v = (*dr)[assignment ? assignment[tid] : tid * stride];
    block_accumulate(sum, v);
}

__global__ void k_iota(unsigned long long* p, uint64_t n)
{
    const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = i;
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
/* plain random gather of 8-byte words from device memory: the ceiling of that access pattern without any cache protocol */
__global__ void k_gather8(const uint64_t* __restrict__ src, const uint64_t* __restrict__ idx, uint64_t n, unsigned long long* partials)
{
    const uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    block_accumulate(partials, t < n ? src[idx[t]] : 0);
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

inline uint32_t blocks_for(uint64_t n, uint32_t bs) { return (uint32_t)((n + bs - 1) / bs); }

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

int bam_array_read(bam_array_t* a, uint64_t n_reqs, const uint64_t* d_assignment, uint64_t stride, uint64_t reqs_per_thread,
                   uint32_t block_size, uint64_t* d_sum, void* stream)
{
    if (!a || !d_sum) return fail(EINVAL, "bam_array_read: null argument");
    if (!block_size || block_size % BAM_WAVE_SIZE || block_size > 1024) return fail(EINVAL, "bam_array_read: block size must be a multiple of 64, at most 1024");
    if (!n_reqs) return 0;
    BAM_API_BEGIN
    hipLaunchKernelGGL(k_array_read, dim3(blocks_for(n_reqs, block_size)), dim3(block_size), 0, (hipStream_t)stream,
                       a->a->d_array_ptr, n_reqs, d_assignment, stride, reqs_per_thread, (unsigned long long*)a->partials.get());
    hipLaunchKernelGGL(k_fold_partials, dim3(1), dim3(1024), 0, (hipStream_t)stream, (unsigned long long*)a->partials.get(), (unsigned long long*)d_sum);
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
    if (mode < 0 || mode > 4) return fail(EINVAL, "bam_cache_stream: mode must be 0 to 4");
    if (!n_waves || !n_pages_per_wave) return 0;
    BAM_API_BEGIN
    const uint32_t bs = 256;
    const dim3 grid(blocks_for(n_waves * BAM_WAVE_SIZE, bs)), block(bs);
    array_d_t<uint64_t>* d = a->a->d_array_ptr;
    unsigned long long* s = (unsigned long long*)a->partials.get();
    if (mode == 0) hipLaunchKernelGGL(k_cache_stream<0>, grid, block, 0, (hipStream_t)stream, d, n_waves, n_pages_per_wave, d_assignment, s);
    else if (mode == 1) hipLaunchKernelGGL(k_cache_stream<1>, grid, block, 0, (hipStream_t)stream, d, n_waves, n_pages_per_wave, d_assignment, s);
    else if (mode == 3) hipLaunchKernelGGL(k_cache_stream<3>, grid, block, 0, (hipStream_t)stream, d, n_waves, n_pages_per_wave, d_assignment, s);
    else if (mode == 4) hipLaunchKernelGGL(k_cache_stream<4>, grid, block, 0, (hipStream_t)stream, d, n_waves, n_pages_per_wave, d_assignment, s);
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
    if (!n_reqs) return 0;
    BAM_API_BEGIN
    hipLaunchKernelGGL(k_block_io, dim3(blocks_for(n_reqs, block_size)), dim3(block_size), 0, (hipStream_t)stream,
                       pc->pc->pdt.d_ctrls, pc->pc->d_pc_ptr, req_bytes, n_reqs, d_lbas, write, queue_policy);
    hip_err_chk(hipGetLastError());
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

namespace {
/* the pieces of the long edge lists of a graph, listed once per call, and the counter that hands out the work of a sweep:
 * a list of d >= BAM_HEAVY_EDGES entries makes at most d / BAM_PIECE_EDGES + 1 <= 2 d / BAM_HEAVY_EDGES pieces */
struct sweep_work {
    BufferPtr buf, cnt;
    heavy_piece_t* pieces;
    unsigned long long* count;       /* [0] number of pieces, [1] next piece of work of the sweep */
    uint64_t n_pieces = 0;
    uint64_t group;                  /* vertices handed to a wave at a time */
    uint64_t resident;               /* waves the device holds at a time */
    sweep_work(uint64_t n_edges, uint64_t n_vertices, uint32_t coarse, const uint64_t* d_offsets, hipStream_t st)
    {
        const uint64_t cap = 2 * (n_edges / BAM_HEAVY_EDGES) + 1;
        buf = createBuffer(cap * sizeof(heavy_piece_t), 0);
        cnt = createBuffer(2 * sizeof(unsigned long long), 0);
        pieces = (heavy_piece_t*)buf.get();
        count = (unsigned long long*)cnt.get();
        /* a group's lists are asked for as one batch of commands: a few hundred vertices make that batch large enough for the
         * store path, and keep the one word all waves take their work from out of the way */
        group = coarse > 512 ? coarse : 512;
        int dev = 0, cus = 0;
        hip_err_chk(hipGetDevice(&dev));
        hip_err_chk(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
        resident = (uint64_t)cus * 16;
        hip_err_chk(hipMemsetAsync(count, 0, 2 * sizeof(unsigned long long), st));
        hipLaunchKernelGGL(k_heavy_pieces, dim3(blocks_for(n_vertices, 256)), dim3(256), 0, st, d_offsets, n_vertices, pieces, count);
        hip_err_chk(hipGetLastError());
        unsigned long long n = 0;
        hip_err_chk(hipMemcpyAsync(&n, count, sizeof(n), hipMemcpyDeviceToHost, st));
        hip_err_chk(hipStreamSynchronize(st));
        n_pieces = n;
    }
    /* workgroups of two waves for a sweep over `n_items` items in groups of `grp` */
    uint32_t blocks(uint64_t n_items, uint64_t grp) const
    {
        const uint64_t units = (n_pieces + BAM_PIECE_BUNDLE - 1) / BAM_PIECE_BUNDLE + (n_items + grp - 1) / grp;
        return (uint32_t)(((units < resident ? units : resident) + 1) / 2);
    }
    void reset(hipStream_t st) { hip_err_chk(hipMemsetAsync(count + 1, 0, sizeof(unsigned long long), st)); }
};
} // namespace

int bam_bfs(bam_array_t* edges, const uint64_t* d_offsets, uint64_t n_vertices, uint64_t src, uint32_t* d_labels,
            uint32_t coarse, uint32_t* iterations, void* stream)
{
    if (!edges || !d_offsets || !d_labels) return fail(EINVAL, "bam_bfs: null argument");
    if (src >= n_vertices || !coarse) return fail(EINVAL, "bam_bfs: source out of range or coarse = 0");
    BAM_API_BEGIN
    hipStream_t st = (hipStream_t)stream;
    BufferPtr changed_buf = createBuffer(sizeof(uint64_t), 0);
    uint64_t* changed_d = (uint64_t*)changed_buf.get();
    const uint32_t zero = 0;
    hip_err_chk(hipMemsetAsync(d_labels, 0xFF, n_vertices * sizeof(uint32_t), st));
    hip_err_chk(hipMemcpyAsync(d_labels + src, &zero, sizeof(uint32_t), hipMemcpyHostToDevice, st));
    const uint32_t threads = 128;
    sweep_work work(edges->a->adt.n_elems, n_vertices, coarse, d_offsets, st);
    uint32_t level = 0, iter = 0;
    uint64_t changed_h;
    do {
        changed_h = 0;
        hip_err_chk(hipMemcpyAsync(changed_d, &changed_h, sizeof(uint64_t), hipMemcpyHostToDevice, st));
        work.reset(st);
        hipLaunchKernelGGL(k_bfs_coalesce_coarse_ptr_pc, dim3(work.blocks(n_vertices, work.group)), dim3(threads), 0, st,
                           edges->a->d_array_ptr, d_labels, level, n_vertices, d_offsets, changed_d, work.group, work.pieces, work.n_pieces, work.count + 1);
        hip_err_chk(hipGetLastError());
        iter++; level++;
        hip_err_chk(hipMemcpyAsync(&changed_h, changed_d, sizeof(uint64_t), hipMemcpyDeviceToHost, st));
        hip_err_chk(hipStreamSynchronize(st));
    } while (changed_h);
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
    /* two queues of at most every vertex once (benchmarks/bfs/main.cu:1489-1492); the size of the next one is the reference's `changed` */
    BufferPtr queue_a = createBuffer(n_vertices * sizeof(uint32_t), 0), queue_b = createBuffer(n_vertices * sizeof(uint32_t), 0);
    BufferPtr size_buf = createBuffer(sizeof(unsigned long long), 0);
    uint32_t* curr = (uint32_t*)queue_a.get();
    uint32_t* next = (uint32_t*)queue_b.get();
    unsigned long long* next_size = (unsigned long long*)size_buf.get();
    const uint32_t zero = 0, src32 = (uint32_t)src;
    hip_err_chk(hipMemsetAsync(d_labels, 0xFF, n_vertices * sizeof(uint32_t), st));
    hip_err_chk(hipMemcpyAsync(d_labels + src, &zero, sizeof(uint32_t), hipMemcpyHostToDevice, st));
    hip_err_chk(hipMemcpyAsync(curr, &src32, sizeof(uint32_t), hipMemcpyHostToDevice, st));
    const uint32_t threads = 128;
    uint64_t group = BAM_WAVE_SIZE;                 /* queue entries handed to a wave at a time: one per lane, more of a sorted queue */
    bool sorted = true;                             /* the first queue holds the source alone */
    sweep_work work(edges->a->adt.n_elems, n_vertices, 1, d_offsets, st);
    uint32_t level = 0, iter = 0;
    unsigned long long active = 1;
    const char* e = getenv("BAM_FRONTIER_SORT");
    const bool sort_queue = !e || atoi(e) != 0;
    int vertex_bits = 1;
    while (vertex_bits < 32 && (1ull << vertex_bits) < n_vertices) vertex_bits++;
    size_t sort_bytes = 0;
    if (sort_queue) hip_err_chk(hipcub::DeviceRadixSort::SortKeys(nullptr, sort_bytes, curr, next, (int)std::min<uint64_t>(n_vertices, 0x7FFFFFFFull), 0, vertex_bits, st));
    BufferPtr sort_tmp = createBuffer(sort_bytes ? sort_bytes : 8, 0);
    do {
        hip_err_chk(hipMemsetAsync(next_size, 0, sizeof(unsigned long long), st));
        work.reset(st);
        hipLaunchKernelGGL(k_bfs_frontier_coalesce_ptr_pc, dim3(work.blocks(active, group)), dim3(threads), 0, st, edges->a->d_array_ptr, d_labels, level,
                           d_offsets, curr, (uint64_t)active, next, next_size, group, work.pieces, work.n_pieces, work.count + 1, sorted);
        hip_err_chk(hipGetLastError());
        iter++; level++;
        hip_err_chk(hipMemcpyAsync(&active, next_size, sizeof(unsigned long long), hipMemcpyDeviceToHost, st));
        hip_err_chk(hipStreamSynchronize(st));
        sorted = sort_queue && active <= 0x7FFFFFFFull;
        group = sorted ? work.group : BAM_WAVE_SIZE;
        if (sorted && active > 1) {
            /* the queue comes out in the order of discovery; sorted by vertex, the level reads the edge array front to back
             * (neighbouring lists share pages, a page is not evicted between two of its lists, and the pages under the
             * lists of a group of entries can be asked for together as in the sweep over all vertices).  The sorted queue
             * goes into the buffer the level just walked, so the two do not change places. */
            size_t need = sort_bytes;
            hip_err_chk(hipcub::DeviceRadixSort::SortKeys(sort_tmp.get(), need, next, curr, (int)active, 0, vertex_bits, st));
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
    BufferPtr visit_a = createBuffer(n_vertices, 0), visit_b = createBuffer(n_vertices, 0), changed_buf = createBuffer(sizeof(uint64_t), 0);
    bool* curr = (bool*)visit_a.get();
    bool* next = (bool*)visit_b.get();
    bool* changed_d = (bool*)changed_buf.get();
    hipLaunchKernelGGL(k_iota, dim3(blocks_for(n_vertices, 256)), dim3(256), 0, st, (unsigned long long*)d_labels, n_vertices);
    hip_err_chk(hipMemsetAsync(curr, 0x01, n_vertices, st));
    hip_err_chk(hipMemsetAsync(next, 0x00, n_vertices, st));
    const uint32_t threads = 128;
    sweep_work work(edges->a->adt.n_elems, n_vertices, coarse, d_offsets, st);
    uint32_t iter = 0;
    bool changed_h;
    do {
        changed_h = false;
        hip_err_chk(hipMemcpyAsync(changed_d, &changed_h, sizeof(bool), hipMemcpyHostToDevice, st));
        work.reset(st);
        hipLaunchKernelGGL(k_cc_coalesce_coarse_ptr_pc, dim3(work.blocks(n_vertices, work.group)), dim3(threads), 0, st, edges->a->d_array_ptr, curr, next,
                           n_vertices, d_offsets, (unsigned long long*)d_labels, changed_d, work.group, work.pieces, work.n_pieces, work.count + 1, iter);
        hip_err_chk(hipGetLastError());
        hip_err_chk(hipMemsetAsync(curr, 0x00, n_vertices, st));
        bool* t = curr; curr = next; next = t;
        iter++;
        hip_err_chk(hipMemcpyAsync(&changed_h, changed_d, sizeof(bool), hipMemcpyDeviceToHost, st));
        hip_err_chk(hipStreamSynchronize(st));
    } while (changed_h);
    if (iterations) *iterations = iter;
    BAM_API_END
}

namespace {
/* launch shape of the by-page graph kernels: pages per wave trip and number of waves, so that what the waves hold
 * at any time stays under half of the cache */
struct by_page_plan { uint64_t n_edges, n_pages; uint32_t epp, ppw, blocks; BufferPtr first; };

int plan_by_page(bam_array_t* edges, const uint64_t* d_offsets, uint64_t n_vertices, hipStream_t st, by_page_plan& pl)
{
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
    hipLaunchKernelGGL(k_page_first_vertex, dim3(blocks_for(pl.n_pages + 1, 256)), dim3(256), 0, st, d_offsets, n_vertices, (uint64_t)pl.epp, pl.n_pages,
                       (uint64_t*)pl.first.get());
    hip_err_chk(hipGetLastError());
    return 0;
}
} // namespace

int bam_bfs_by_page(bam_array_t* edges, const uint64_t* d_offsets, uint64_t n_vertices, uint64_t src, uint32_t* d_labels,
                    uint32_t* iterations, void* stream)
{
    if (!edges || !d_offsets || !d_labels) return fail(EINVAL, "bam_bfs_by_page: null argument");
    if (src >= n_vertices) return fail(EINVAL, "bam_bfs_by_page: source out of range");
    BAM_API_BEGIN
    hipStream_t st = (hipStream_t)stream;
    by_page_plan pl;
    if (int rc = plan_by_page(edges, d_offsets, n_vertices, st, pl)) return rc;
    BufferPtr changed_buf = createBuffer(sizeof(uint64_t), 0);
    uint64_t* changed_d = (uint64_t*)changed_buf.get();
    const uint32_t zero = 0;
    hip_err_chk(hipMemsetAsync(d_labels, 0xFF, n_vertices * sizeof(uint32_t), st));
    hip_err_chk(hipMemcpyAsync(d_labels + src, &zero, sizeof(uint32_t), hipMemcpyHostToDevice, st));
    uint32_t level = 0, iter = 0;
    uint64_t changed_h;
    do {
        changed_h = 0;
        hip_err_chk(hipMemcpyAsync(changed_d, &changed_h, sizeof(uint64_t), hipMemcpyHostToDevice, st));
        if (pl.n_pages)
            hipLaunchKernelGGL(k_bfs_by_page, dim3(pl.blocks), dim3(BAM_WAVE_SIZE), 0, st, edges->a->d_array_ptr, d_labels, level, d_offsets,
                               (const uint64_t*)pl.first.get(), pl.n_edges, pl.ppw, changed_d);
        hip_err_chk(hipGetLastError());
        iter++; level++;
        hip_err_chk(hipMemcpyAsync(&changed_h, changed_d, sizeof(uint64_t), hipMemcpyDeviceToHost, st));
        hip_err_chk(hipStreamSynchronize(st));
    } while (changed_h);
    if (iterations) *iterations = iter;
    BAM_API_END
}

int bam_cc_by_page(bam_array_t* edges, const uint64_t* d_offsets, uint64_t n_vertices, uint64_t* d_labels, uint32_t* iterations, void* stream)
{
    if (!edges || !d_offsets || !d_labels) return fail(EINVAL, "bam_cc_by_page: null argument");
    if (!n_vertices) return fail(EINVAL, "bam_cc_by_page: empty graph");
    BAM_API_BEGIN
    hipStream_t st = (hipStream_t)stream;
    by_page_plan pl;
    if (int rc = plan_by_page(edges, d_offsets, n_vertices, st, pl)) return rc;
    BufferPtr visit_a = createBuffer(n_vertices, 0), visit_b = createBuffer(n_vertices, 0), changed_buf = createBuffer(sizeof(uint64_t), 0);
    bool* curr = (bool*)visit_a.get();
    bool* next = (bool*)visit_b.get();
    bool* changed_d = (bool*)changed_buf.get();
    hipLaunchKernelGGL(k_iota, dim3(blocks_for(n_vertices, 256)), dim3(256), 0, st, (unsigned long long*)d_labels, n_vertices);
    hip_err_chk(hipMemsetAsync(curr, 0x01, n_vertices, st));
    hip_err_chk(hipMemsetAsync(next, 0x00, n_vertices, st));
    uint32_t iter = 0;
    bool changed_h;
    do {
        changed_h = false;
        hip_err_chk(hipMemcpyAsync(changed_d, &changed_h, sizeof(bool), hipMemcpyHostToDevice, st));
        if (pl.n_pages)
            hipLaunchKernelGGL(k_cc_by_page, dim3(pl.blocks), dim3(BAM_WAVE_SIZE), 0, st, edges->a->d_array_ptr, curr, next, d_offsets,
                               (const uint64_t*)pl.first.get(), pl.n_edges, pl.ppw, iter, (unsigned long long*)d_labels, changed_d);
        hip_err_chk(hipGetLastError());
        hip_err_chk(hipMemsetAsync(curr, 0x00, n_vertices, st));
        bool* t = curr; curr = next; next = t;
        iter++;
        hip_err_chk(hipMemcpyAsync(&changed_h, changed_d, sizeof(bool), hipMemcpyDeviceToHost, st));
        hip_err_chk(hipStreamSynchronize(st));
    } while (changed_h);
    if (iterations) *iterations = iter;
    BAM_API_END
}

int bam_vectoradd(bam_array_t* a, bam_array_t* b, bam_array_t* c, uint64_t n_elems, void* stream)
{
    if (!a || !b || !c) return fail(EINVAL, "bam_vectoradd: null argument");
    if (n_elems > a->a->adt.n_elems || n_elems > b->a->adt.n_elems || n_elems > c->a->adt.n_elems) return fail(EINVAL, "bam_vectoradd: more elements than the arrays hold");
    if (!n_elems) return 0;
    BAM_API_BEGIN
    hipLaunchKernelGGL(k_vectoradd_ptr_pc, dim3(blocks_for(n_elems, 64)), dim3(64), 0, (hipStream_t)stream,
                       a->a->d_array_ptr, b->a->d_array_ptr, n_elems, c->a->d_array_ptr);
    hip_err_chk(hipGetLastError());
    BAM_API_END
}

int bam_reduce(bam_array_t* a, uint64_t n_elems, uint32_t block_size, uint64_t* d_partials, void* stream)
{
    if (!a || !d_partials) return fail(EINVAL, "bam_reduce: null argument");
    if (!block_size || block_size % BAM_WAVE_SIZE || block_size > 1024) return fail(EINVAL, "bam_reduce: block size must be a multiple of 64, at most 1024");
    if (n_elems > a->a->adt.n_elems) return fail(EINVAL, "bam_reduce: more elements than the array holds");
    if (!n_elems) return 0;
    BAM_API_BEGIN
    hipLaunchKernelGGL(k_reduce_ptr_pc, dim3(blocks_for(n_elems, 2ull * block_size)), dim3(block_size), 0, (hipStream_t)stream,
                       a->a->d_array_ptr, (unsigned long long*)d_partials, n_elems);
    hip_err_chk(hipGetLastError());
    BAM_API_END
}

int bam_scan(bam_array_t* a, uint64_t n_elems, uint32_t block_size, uint64_t* d_result, void* stream)
{
    if (!a || !d_result) return fail(EINVAL, "bam_scan: null argument");
    if (!block_size || block_size % BAM_WAVE_SIZE || block_size > 1024) return fail(EINVAL, "bam_scan: block size must be a multiple of 64, at most 1024");
    if (n_elems > a->a->adt.n_elems) return fail(EINVAL, "bam_scan: more elements than the array holds");
    BAM_API_BEGIN
    hipStream_t st = (hipStream_t)stream;
    hip_err_chk(hipMemsetAsync(d_result, 0, sizeof(uint64_t), st));
    if (n_elems) {
        const uint64_t n_blocks = blocks_for(n_elems, 2ull * block_size);
        BufferPtr totals = createBuffer(n_blocks * sizeof(uint64_t), 0);
        unsigned long long* out = (unsigned long long*)d_result + 1;
        const size_t lds = (2 * block_size + 1024 / BAM_WAVE_SIZE) * sizeof(uint64_t);
        hipLaunchKernelGGL(k_scan_ptr_pc, dim3(n_blocks), dim3(block_size), lds, st, a->a->d_array_ptr, out, (unsigned long long*)totals.get(), n_elems);
        hipLaunchKernelGGL(k_scan_block_totals, dim3(1), dim3(1024), 0, st, (unsigned long long*)totals.get(), n_blocks);
        hipLaunchKernelGGL(k_scan_finalsum, dim3(n_blocks), dim3(block_size), 0, st, (const unsigned long long*)totals.get(), out, n_elems);
        hip_err_chk(hipGetLastError());
        hip_err_chk(hipStreamSynchronize(st));         /* `totals` is released on return */
    }
    BAM_API_END
}

} // extern "C"

/*
 * bam_scan for callers that cannot allocate (code under stream capture, serving loops, harnesses that forbid it): the block
 * totals, which bam_scan keeps in a buffer it allocates and frees per call, live in a file-scope device array of fixed size.
 * Every device the library runs on holds its own copy of the array at its own address until the process ends; the address is
 * looked up once per device (the array's name means nothing to the host) and handed to the kernels like any other buffer.
 */
/* BAM_SCAN_NOALLOC_MAX_BLOCKS (bam_amd.h): 65536 block totals, 512 KiB */
#define BAM_SCAN_NOALLOC_MAX_DEVICES 64
static __device__ __align__(256) unsigned long long scratch[BAM_SCAN_NOALLOC_MAX_BLOCKS];

namespace {
std::mutex g_scratch_mu;
unsigned long long* g_scratch_ptr[BAM_SCAN_NOALLOC_MAX_DEVICES];      /* per device: where its copy of `scratch` lives */

/* the current device's copy of the array; NULL (and the error recorded) if it cannot be found */
unsigned long long* scan_scratch_of_current_device()
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= BAM_SCAN_NOALLOC_MAX_DEVICES) { g_err = "bam_scan_noalloc: no current device"; return nullptr; }
    std::lock_guard<std::mutex> g(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) { g_err = std::string("bam_scan_noalloc: hipGetSymbolAddress: ") + hipGetErrorString(e); return nullptr; }
        g_scratch_ptr[dev] = (unsigned long long*)p;
    }
    return g_scratch_ptr[dev];
}

__global__ void k_store_zero64(unsigned long long* p) { *p = 0; }
} // namespace

extern "C" {

int bam_scan_noalloc(bam_array_t* a, uint64_t n_elems, uint32_t block_size, uint64_t* d_result, void* stream)
{
    if (!a || !d_result) return fail(EINVAL, "bam_scan_noalloc: null argument");
    if (!block_size || block_size % BAM_WAVE_SIZE || block_size > 1024) return fail(EINVAL, "bam_scan_noalloc: block size must be a multiple of 64, at most 1024");
    if (n_elems > a->a->adt.n_elems) return fail(EINVAL, "bam_scan_noalloc: more elements than the array holds");
    const uint64_t n_blocks = (n_elems + 2ull * block_size - 1) / (2ull * block_size);
    if (n_blocks > BAM_SCAN_NOALLOC_MAX_BLOCKS)
        return fail(E2BIG, "bam_scan_noalloc: " + std::to_string(n_elems) + " elements in blocks of " + std::to_string(2ull * block_size) + " need " + std::to_string(n_blocks) +
                           " block totals, the fixed scratch array holds " + std::to_string(BAM_SCAN_NOALLOC_MAX_BLOCKS) + " (use bam_scan, or a larger block size)");
    unsigned long long* totals = scan_scratch_of_current_device();
    if (!totals) return EIO;
    hipStream_t st = (hipStream_t)stream;
    unsigned long long* out = (unsigned long long*)d_result + 1;
    /* no memset node: a fill kernel clears the first word (a caller may be capturing this stream) */
    hipLaunchKernelGGL(k_store_zero64, dim3(1), dim3(1), 0, st, (unsigned long long*)d_result);
    if (n_elems) {
        /* totals[0 .. n_blocks) are written by the first kernel before the second reads them; what an earlier, longer call
         * left behind them is never read, so nothing has to be cleared */
        const size_t lds = (2 * block_size + 1024 / BAM_WAVE_SIZE) * sizeof(uint64_t);
        hipLaunchKernelGGL(k_scan_ptr_pc, dim3((uint32_t)n_blocks), dim3(block_size), lds, st, a->a->d_array_ptr, out, totals, n_elems);
        hipLaunchKernelGGL(k_scan_block_totals, dim3(1), dim3(1024), 0, st, totals, n_blocks);
        hipLaunchKernelGGL(k_scan_finalsum, dim3((uint32_t)n_blocks), dim3(block_size), 0, st, (const unsigned long long*)totals, out, n_elems);
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(EIO, std::string("bam_scan_noalloc: ") + hipGetErrorString(e));
    return 0;
}

int bam_pagerank(bam_array_t* edges, const uint64_t* d_offsets, uint64_t n_vertices, float alpha, float tolerance, uint32_t max_iterations,
                 int by_page, float* d_value, uint32_t* iterations, void* stream)
{
    if (!edges || !d_offsets || !d_value) return fail(EINVAL, "bam_pagerank: null argument");
    if (iterations) *iterations = 0;
    if (!n_vertices) return 0;
    BAM_API_BEGIN
    hipStream_t st = (hipStream_t)stream;
    BufferPtr delta = createBuffer(n_vertices * sizeof(float), 0), residual = createBuffer(n_vertices * sizeof(float), 0),
              label = createBuffer(n_vertices, 0), changed_buf = createBuffer(sizeof(uint64_t), 0);
    float* delta_d = (float*)delta.get();
    float* residual_d = (float*)residual.get();
    bool* label_d = (bool*)label.get();
    bool* changed_d = (bool*)changed_buf.get();
    by_page_plan pl{};
    if (by_page)
        if (int rc = plan_by_page(edges, d_offsets, n_vertices, st, pl)) return rc;
    const uint32_t upd_blocks = blocks_for(n_vertices, 256);
    sweep_work work(edges->a->adt.n_elems, n_vertices, 1, d_offsets, st);
    hipLaunchKernelGGL(k_pr_initialize, dim3(upd_blocks), dim3(256), 0, st, label_d, delta_d, residual_d, d_value, n_vertices, d_offsets, alpha);
    uint32_t iter = 0;
    bool changed_h;
    do {
        changed_h = false;
        hip_err_chk(hipMemcpyAsync(changed_d, &changed_h, sizeof(bool), hipMemcpyHostToDevice, st));
        if (by_page) {
            if (pl.n_pages)
                hipLaunchKernelGGL(k_pr_by_page, dim3(pl.blocks), dim3(BAM_WAVE_SIZE), 0, st, edges->a->d_array_ptr, label_d, delta_d, residual_d, d_offsets,
                                   (const uint64_t*)pl.first.get(), pl.n_edges, pl.ppw, iter);
            hip_err_chk(hipMemsetAsync(label_d, 0, n_vertices, st));
        } else {
            work.reset(st);
            hipLaunchKernelGGL(k_pr_coalesce_pc, dim3(work.blocks(n_vertices, work.group)), dim3(128), 0, st, edges->a->d_array_ptr, label_d, delta_d, residual_d,
                               n_vertices, d_offsets, work.group, work.pieces, work.n_pieces, work.count + 1, iter);
            hip_err_chk(hipMemsetAsync(label_d, 0, n_vertices, st));
        }
        iter++;
        hipLaunchKernelGGL(k_pr_update, dim3(upd_blocks), dim3(256), 0, st, label_d, delta_d, residual_d, d_value, n_vertices, d_offsets, tolerance, alpha, changed_d);
        hip_err_chk(hipGetLastError());
        hip_err_chk(hipMemcpyAsync(&changed_h, changed_d, sizeof(bool), hipMemcpyDeviceToHost, st));
        hip_err_chk(hipStreamSynchronize(st));
    } while (changed_h && iter < max_iterations);
    if (iterations) *iterations = iter;
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

namespace {
/* the loop of benchmarks/sssp/main.cu:663-725 (and of sssp_float, :624-700): relax from the flagged vertices, adopt what got
 * cheaper, flag it, until nothing does.  FLOAT: costs and weights are single-precision values, unreached = 1e9 (sssp_float :529) */
void sssp_run(const bool FLOAT, bam_array_t* edges, bam_array32_t* weights, const uint64_t* d_offsets, uint64_t n_vertices, uint64_t src, uint32_t* d_costs,
              uint32_t* iterations, hipStream_t st)
{
    BufferPtr new_cost = createBuffer(n_vertices * sizeof(uint32_t), 0), label = createBuffer(n_vertices, 0), changed_buf = createBuffer(sizeof(uint64_t), 0);
    uint32_t* new_d = (uint32_t*)new_cost.get();
    bool* label_d = (bool*)label.get();
    bool* changed_d = (bool*)changed_buf.get();
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
    sweep_work work(edges->a->adt.n_elems, n_vertices, 1, d_offsets, st);
    uint32_t iter = 0;
    bool changed_h;
    do {
        changed_h = false;
        hip_err_chk(hipMemcpyAsync(changed_d, &changed_h, sizeof(bool), hipMemcpyHostToDevice, st));
        work.reset(st);
        hipLaunchKernelGGL(FLOAT ? k_sssp_coalesce_pc<true> : k_sssp_coalesce_pc<false>, dim3(work.blocks(n_vertices, work.group)), dim3(threads), 0, st,
                           edges->a->d_array_ptr, weights->a->d_array_ptr, label_d, new_d, n_vertices, d_offsets, work.group, work.pieces, work.n_pieces, work.count + 1, iter);
        hip_err_chk(hipMemsetAsync(label_d, 0, n_vertices, st));
        hipLaunchKernelGGL(k_sssp_update, dim3(blocks_for(n_vertices, 256)), dim3(256), 0, st, label_d, d_costs, new_d, n_vertices, changed_d);
        hip_err_chk(hipGetLastError());
        iter++;
        hip_err_chk(hipMemcpyAsync(&changed_h, changed_d, sizeof(bool), hipMemcpyDeviceToHost, st));
        hip_err_chk(hipStreamSynchronize(st));
    } while (changed_h);
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
