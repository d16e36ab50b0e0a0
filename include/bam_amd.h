/*
 * C-ABI of the GPU-side storage-access path (libbam_amd.so).
 *
 * Plain pointers and sizes only.  Handles are opaque; they wrap the C++ host
 * objects of ctrl.h / page_cache.h, which mirror the reference's.  Every entry
 * point returns 0 on success or a non-zero errno-style code; bam_last_error()
 * gives the message of the last failure on the calling thread.  Device
 * pointers (d_*) must be valid on the device the handle was created for.
 * Kernels are launched on the given stream (0 = the null stream) and the
 * calls that return results through host pointers synchronise that stream.
 */
#ifndef __BAM_AMD_H__
#define __BAM_AMD_H__
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

typedef struct bam_target bam_target_t;       /* software NVMe target + its register window and backing store */
typedef struct bam_ctrl bam_ctrl_t;           /* Controller */
typedef struct bam_page_cache bam_page_cache_t;
typedef struct bam_range bam_range_t;         /* range_t<uint64_t> */
typedef struct bam_array bam_array_t;         /* array_t<uint64_t> */
typedef struct bam_range32 bam_range32_t;     /* range_t<uint32_t> */
typedef struct bam_array32 bam_array32_t;     /* array_t<uint32_t> */

const char* bam_last_error(void);
/* 1 when the library was built with the gfx950 device path and a HIP device is present */
int bam_device_count(int* count);

/* ---- backing store ----
 * Stands where the reference opens /dev/libnvmN (benchmarks/array/main.cu:39-40,
 * include/ctrl.h:148-163): creates a software NVMe target and publishes it under
 * `path`.  backing = 0: procedural namespace (word w = splitmix64(seed, w));
 * backing = 1: memory-backed namespace in host-pinned memory, initialised to
 * the same words so that both read identically until written. */
int bam_target_create(bam_target_t** out, const char* path, uint64_t ns_bytes, uint32_t lba_bytes, int backing, uint64_t seed,
                      uint32_t n_io_threads, uint32_t max_queue_entries, uint32_t max_io_queues, uint32_t completion_order,
                      uint32_t fail_every, uint32_t drop_every);
void bam_target_destroy(bam_target_t* t);
/* out[12]: admin_cmds, io_cmds, read_cmds, write_cmds, bytes_read, bytes_written, error_cpls, sq_doorbells, cq_full_stalls, dropped,
 *          sqe_retries, stale_doorbells */
int bam_target_stats(bam_target_t* t, uint64_t* out, int reset);
/* host pointer to the memory-backed namespace (NULL for procedural) */
void* bam_target_backing(bam_target_t* t);

/* ---- Controller (include/ctrl.h:148-199 of the reference) ----
 * stage_bytes: size of the per-command staging page (0 = PRPs address device memory directly, needs CPU-visible VRAM);
 * spin_limit: bound of every device-side wait loop, in microseconds (0 = unbounded). */
int bam_ctrl_create(bam_ctrl_t** out, const char* path, uint32_t ns_id, uint32_t device, uint64_t queue_depth, uint64_t n_queues,
                    uint32_t stage_bytes, uint32_t spin_limit);
void bam_ctrl_destroy(bam_ctrl_t* c);
/* out[6]: n_qps, queue depth, block size, namespace blocks, #SSDAccesses since last reset, error completions */
int bam_ctrl_info(bam_ctrl_t* c, uint64_t* out, int reset);
/* Where queue pair `qp` (0-based) stands, for diagnosis after a run that was given up; call with the device idle.
 * out16[0..7]: queue depth, slot tickets handed out, SQ tail, SQ tail lock held, how far the controller has read the SQ
 * (from completions), CQ head, CQ head lock held, error completions; [8..15] reserved.  slots (may be NULL): for each of
 * the first n_slots slots three words: its free/lap counter, its written-for-lap mark, its command word (1 in flight,
 * 3 completed, 7 completed with an error status). */
int bam_ctrl_queue_state(bam_ctrl_t* c, uint32_t qp, uint64_t* out16, uint32_t* slots, uint32_t n_slots);
/* the software target's side of I/O queue `qid` (1-based, as created): out8 = SQ head, commands fetched, SQ tail doorbell,
 * sealed, CQ tail, CQ head as last seen, CQ head doorbell, CQ phase */
int bam_target_queue_state(bam_target_t* t, uint32_t qid, uint64_t* out8);
/* 1 if a device-side wait gave up (lost completion / spin limit); clear = reset the flag */
int bam_ctrl_aborted(bam_ctrl_t* c, int clear);

/* ---- page_cache_t / range_t<uint64_t> / array_t<uint64_t> (include/page_cache.h:697-875, 984-1030, 1754-1772) ---- */
int bam_page_cache_create(bam_page_cache_t** out, uint64_t page_size, uint64_t n_pages, uint32_t device, bam_ctrl_t* ctrl, uint64_t max_range);
/* one cache in front of several controllers (the `ctrls` vector of page_cache_t, include/page_cache.h:697-705): ranges
 * created with dist = 1 (STRIPE) put page p on controller p % n at page p / n, ranges with dist = 0 (REPLICATE) expect
 * the same data on every controller and spread their reads over them (:556-582) */
int bam_page_cache_create_multi(bam_page_cache_t** out, uint64_t page_size, uint64_t n_pages, uint32_t device, bam_ctrl_t** ctrls, uint32_t n_ctrls,
                                uint64_t max_range);
void bam_page_cache_destroy(bam_page_cache_t* pc);
/* out[5]: n_pages, page_size, wave_batch, staged(0/1), of every 8 read batches how many bypass the staging pages */
int bam_page_cache_info(bam_page_cache_t* pc, uint64_t* out);
/* The cache's payload memory as a dma-buf descriptor (reference: module/map.c:307-399, where the kernel module pins the
 * GPU pages of the cache with nvidia_p2p_get_pages and hands the controller their bus addresses).  This is the GPU side
 * of the same step for a real NVMe device here: the descriptor names the device memory [base, base + *bytes) of the
 * cache's slots, and whoever drives the device (a kernel driver, VFIO / iommufd) imports it, maps it for the device's
 * DMA and supplies the bus addresses to nvm_dma_map_device.  The caller owns *fd and closes it.  ENOTSUP where the
 * runtime or the machine cannot export device memory. */
int bam_page_cache_export_dmabuf(bam_page_cache_t* pc, int* fd, uint64_t* bytes);
int bam_page_cache_flush(bam_page_cache_t* pc);
/* phase timers of the miss path (100 MHz ticks, summed over the batches of the cache's first controller), non-zero only in
 * a library built with -DBAM_PROFILE (make prof); out32[0..8]: I/O batches, commands, ticks waiting for command ids,
 * submitting, waiting for completions, moving payload, ticks in the victim search, victim searches, lanes searching;
 * [9..15] inside the submission: ticks for the slot tickets, until the entries are written and marked, until they are
 * covered by a doorbell, trips of that wait, tail sweeps done, entries swept, doorbells; [16..21] inside the wait for
 * completions: trips, ring drains done by the waiting wave, entries drained, ticks draining, looks at an empty ring,
 * ticks between the last drain that flagged this wave's commands and the wave noticing */
int bam_page_cache_profile(bam_page_cache_t* pc, uint64_t* out32, int reset);
int bam_range_create(bam_range_t** out, uint64_t index_start, uint64_t count, uint64_t page_start, uint64_t page_count,
                     uint64_t page_start_offset, uint64_t page_size, bam_page_cache_t* pc, uint32_t device, int dist);
void bam_range_destroy(bam_range_t* r);
int bam_array_create(bam_array_t** out, uint64_t n_elems, uint64_t disk_start_offset, bam_range_t** ranges, uint32_t n_ranges, uint32_t device);
void bam_array_destroy(bam_array_t* a);
/* array_t::print_reset_stats (include/page_cache.h:1731-1752) as numbers; out[4]: read_io_cnt, access_cnt, miss_cnt, hit_cnt */
int bam_array_stats(bam_array_t* a, uint64_t* out, int reset);

/* ---- array benchmark kernels (benchmarks/array/main.cu:43-65) ----
 * One thread per request: thread t reads element d_assignment[t] (or t * stride when d_assignment is NULL)
 * reqs_per_thread times through array_d_t::operator[] and the launch adds every value read into *d_sum
 * (mod 2^64).  The reference discards the values; the checksum is what makes the result checkable.  A launch of 2^16 or
 * more scattered requests read once each runs with a quarter of the threads, thread t taking requests t, t + n/4, t + 2n/4
 * and t + 3n/4 side by side (array_d_t::seq_read_n): the same reads, sum and counters, four of them in flight per lane. */
int bam_array_read(bam_array_t* a, uint64_t n_reqs, const uint64_t* d_assignment, uint64_t stride, uint64_t reqs_per_thread,
                   uint32_t block_size, uint64_t* d_sum, void* stream);
/* The same scattered requests (thread t reads element d_assignment[t] once; sum into *d_sum) with the launch shape named,
 * whatever the size of the launch; sums and counters of accesses do not depend on the shape.
 *   BAM_READ_ONE_PER_THREAD   the reference's kernel as it is: one thread per request, one launch (benchmarks/array/main.cu:43-65)
 *   BAM_READ_FOUR_PER_THREAD  a quarter of the threads, four requests per thread side by side, one launch
 *   BAM_READ_TWO_LAUNCHES     a first launch reads what is resident, reads_per_lane (1, 2, 4, 8) requests per thread, with a
 *                             kernel that cannot miss (no call, no stack, a fraction of the registers) and notes the rest;
 *                             a second launch reads the rest, one request per lane and 64 per wave whatever the share of
 *                             misses was.  Arrays of one range only (EINVAL otherwise).
 * bam_array_read picks BAM_READ_TWO_LAUNCHES with eight reads per lane for launches of 2^16 requests and more where the array
 * allows it (BAM_READ_FOUR_PER_THREAD where not) and BAM_READ_ONE_PER_THREAD below that. */
#define BAM_READ_ONE_PER_THREAD  1
#define BAM_READ_FOUR_PER_THREAD 2
#define BAM_READ_TWO_LAUNCHES    3
int bam_array_read_shaped(bam_array_t* a, uint64_t n_reqs, const uint64_t* d_assignment, int shape, uint32_t reads_per_lane, uint32_t block_size,
                          uint64_t* d_sum, void* stream);
/* the same requests with the values handed out: d_out[t] = element d_assignment[t] (or t * stride); what a kernel of the
 * reference's benchmark would hold in its register after array_d_t::operator[] (benchmarks/array/main.cu:57) */
int bam_array_gather(bam_array_t* a, uint64_t n_reqs, const uint64_t* d_assignment, uint64_t stride, uint32_t block_size, uint64_t* d_out, void* stream);
/* The read pattern of bam_array_read (one thread per request, element d_assignment[t] or t * span) through the other
 * access routes of array_d_t (include/page_cache.h:1240-1716, 414-485): api 1 get_raw/release_raw, 2 get_page_gid +
 * acquire_page_ + release_page, 3 acquire_page/release_page, 4 bam_ptr, 5 memcpy (one request per wave: up to `span`
 * elements starting at the wave's index, clipped to the page, are copied out and summed), 6 bam_ptr_tlb over a tlb in
 * LDS shared by the workgroup (:127-411), 7 bafs_ptr (include/bafs_ptr.h:17-132). */
int bam_array_read_via(bam_array_t* a, int api, uint64_t n_reqs, const uint64_t* d_assignment, uint64_t span, uint32_t block_size,
                       uint64_t* d_sum, void* stream);
/* same request pattern through array_d_t::operator() (seq_write): element <- d_values[t] */
int bam_array_write(bam_array_t* a, uint64_t n_reqs, const uint64_t* d_assignment, uint64_t stride, const uint64_t* d_values,
                    uint32_t block_size, void* stream);

/* read-modify-write through the three routes the reference's kernels have for it: element d_assignment[t] += d_values[t],
 * d_old[t] (may be NULL) = what the element held before.  api 0: array_d_t::AtomicAdd (include/page_cache.h:1647), api 1:
 * an atomic add on the address bam_ptr::memref returns (:467), api 2: ptr[i] += v on a non-const bam_ptr (:478; a plain read
 * and write, so the indices of one launch must be distinct).  The pages touched are dirty afterwards and reach the store
 * on eviction or bam_page_cache_flush. */
int bam_array_update(bam_array_t* a, int api, uint64_t n_reqs, const uint64_t* d_assignment, const uint64_t* d_values, uint64_t* d_old,
                     uint32_t block_size, void* stream);
/* The submission entry the device path builds for one read or write (nvm_cmd_header / nvm_cmd_data_ptr / nvm_cmd_rw_blks,
 * include/nvm_cmd.h:54-88 of the reference; with seal != 0 also nvm_cmd_seal for slot ticket `ticket`): host_out16 (may be
 * NULL) receives the 16 dwords as the host compiler encodes them, d_out64x16 (device memory, may be NULL) 64 entries
 * encoded by the 64 lanes of one wave, lane l for command id cid + l, block lba + l and ticket + l. */
int bam_sqe_image(uint16_t cid, uint8_t opcode, uint32_t nsid, uint64_t prp1, uint64_t prp2, uint64_t lba, uint16_t n_blocks, int seal, uint32_t ticket,
                  uint32_t* host_out16, uint32_t* d_out64x16, void* stream);

/* ---- cache / pattern benchmark kernels (benchmarks/cache/main.cu:44-114, benchmarks/pattern/main.cu:105-170) ----
 * One wave per run of n_pages_per_wave whole pages starting at page d_assignment[w] (or w * n_pages_per_wave),
 * every element read once and summed into *d_sum.  mode 0: array_d_t::operator[] per element,
 * mode 1: bam_ptr per element (the reference's kernel, 64-wide), mode 2: one acquire per page and
 * streamed 8-byte loads; modes 3 and 4: modes 1 and 0 for data that is not
 * resident: a few workgroups at the front of the launch only fetch (they walk the runs of the streaming waves in order,
 * 64 pages per batch of commands, at most a quarter of the cache ahead of the waves that have finished), and a streaming
 * wave that gets ahead of them touches the missing pages of its run itself, up to 64 at a time (12 M instead of 2.5 M
 * pages per second on a cold cache).
 * Modes 0 and 1 on an array of one range run as two launches: the reference's kernel with pointers that read what is
 * resident and note the pages that are not (a kernel without the miss path: no call, no stack, twice the waves; it holds
 * no reference on a page, it looks at the page's descriptor before and after reading it, and a page whose two looks
 * differ is noted like one that was not there), then a kernel that has the miss path over the pages noted, 64 at a time,
 * which also folds the checksum.  Same sum, same number
 * of accesses counted; pages that the second launch loads are asked for as batches before they are read, so their
 * accesses count as hits.  Modes 5 and 6 are modes 0 and 1 as one launch of the kernel that can miss (what arrays of
 * several ranges get under modes 0 and 1). */
int bam_cache_stream(bam_array_t* a, uint64_t n_waves, uint64_t n_pages_per_wave, const uint64_t* d_assignment, int mode,
                     uint64_t* d_sum, void* stream);

/* ---- raw block benchmark kernels (benchmarks/block/main.cu:99-200) ----
 * One thread per command: thread t transfers req_bytes between LBA d_lbas[t] (or t * req_bytes / lba_size when
 * NULL) and cache slot t with read_data / write_data; no cache lookup.  Needs n_pages >= n_reqs.
 * queue_policy 0: queue = compute unit % n_qps (sequential kernel), 1: round-robin counter (random kernel);
 * 2: every thread puts its command together itself from the per-thread queue operations, the way the reference's
 * read_data is written (include/page_cache.h:2009-2054: get_cid, nvm_cmd_*, sq_enqueue, cq_poll, cq_dequeue, put_cid;
 * include/nvm_parallel_queue.h:35-57, 167-330, 378-535), thread t on queue pair t mod n_qps, the controller addressing
 * slot t itself (EINVAL for a cache whose slots have no bus addresses). */
int bam_block_io(bam_ctrl_t* c, bam_page_cache_t* pc, uint64_t n_reqs, uint32_t req_bytes, const uint64_t* d_lbas, int write,
                 int queue_policy, uint32_t block_size, void* stream);
/* raw block reads with `depth` (1, 2, 4, 8) commands in flight per thread through access_data_async / poll_async
 * (benchmarks/iodepth-block/main.cu:97-140): command k of thread t reads LBA d_lbas[t * depth + k] into slot
 * t * depth + k; wave w uses queue pair w mod n_qps.  The waves of one launch that share a queue pair must fit its
 * command ids (waves per queue pair x depth x 64 <= queue depth), checked here. */
int bam_block_io_async(bam_ctrl_t* c, bam_page_cache_t* pc, uint64_t n_threads, uint32_t depth, uint32_t req_bytes, const uint64_t* d_lbas,
                       uint32_t block_size, void* stream);
/* ---- readwrite benchmark (benchmarks/readwrite/main.cu:73-116, host loops :283-316 and :317-391) ----
 * Copy n_bytes (0 = to the end) of the file from file_offset on to the store from byte store_offset on (a multiple of
 * the page size), one pass of the cache at a time: file -> cache slots -> one NVMe write per slot.  This is how a
 * dataset, e.g. the payload of a graph's .dst file (file_offset 16, see bel.h), is placed on the store.  The tail of
 * the last page is zero-filled.  read_file is the inverse: store -> cache slots -> a new file of n_bytes. */
int bam_store_write_file(bam_ctrl_t* c, bam_page_cache_t* pc, const char* path, uint64_t file_offset, uint64_t store_offset, uint64_t n_bytes,
                         uint64_t* bytes_done);
int bam_store_read_file(bam_ctrl_t* c, bam_page_cache_t* pc, const char* path, uint64_t store_offset, uint64_t n_bytes);
/* util.h's warp_memcpy (reference include/util.h:102-117) run by one wave with the lanes named in the bit mask `lanes`
 * active: n_words 64-bit words from d_src to d_dst */
int bam_warp_memcpy(uint64_t* d_dst, const uint64_t* d_src, uint64_t n_words, uint64_t lanes, void* stream);
/* The second look of bam_ptr<T, true> (the pointer of the first streaming launch, which holds no reference) case by case
 * on a resident page of an array of one range, with nothing else using the cache: host_out7[c] is 1 if the window stood
 * and 2 if it fell after the page's descriptor was changed under it in way c: 0 not at all, 1 other readers' references,
 * 2 the dirty bit, 3 busy, 4 not valid, 5 another slot, 6 the same slot loaded once more (4 if the page was not resident
 * to begin with).  A test helper; no counterpart in the reference. */
int bam_unheld_window_cases(bam_array_t* a, uint64_t page, uint32_t* host_out7);
/* sum of the 64-bit words of the first req_bytes of slots 0..n-1, one sum per slot */
int bam_block_checksum(bam_page_cache_t* pc, uint64_t n_slots, uint32_t req_bytes, uint64_t* d_out, void* stream);

/* ---- what the graph entry points prepare per graph (the host code around the reference's loops, benchmarks/bfs/main.cu:
 * 1330-1560, allocates and fills its per-graph arrays once before the timed loop over sources) ----
 * Lists the pieces of the long edge lists of the CSR (d_offsets[V+1], device memory), builds the first-vertex table of the
 * by-page kernels when the array qualifies for them, and allocates the per-vertex flag and value buffers, the sweep counter
 * and the word through which a level tells the host whether anything changed.  Calls of bam_bfs, bam_bfs_frontier, bam_cc,
 * bam_bfs_by_page, bam_cc_by_page and bam_pagerank on `edges` with the same d_offsets and n_vertices then use it and
 * allocate nothing themselves; any other call prepares the same for itself and drops it
 * at its end.  The offsets must not change while the plan is set, and calls that use it must not overlap (they share its
 * counters and buffers).  d_offsets = NULL drops the plan; so does bam_array_destroy.
 * The waves a sweep runs are limited to one per 64 pages of the cache, since every lane of a wave may hold a page. */
int bam_array_set_graph(bam_array_t* edges, const uint64_t* d_offsets, uint64_t n_vertices, void* stream);
/* ---- BFS (benchmarks/bfs/main.cu:658-689 kernel_coalesce_coarse_ptr_pc, host loop :1557-1566, 1577-1736) ----
 * Level-synchronous BFS from src: d_offsets[V+1] in device memory, neighbour ids read through the array,
 * d_labels[V] receives the level of every vertex (0xFFFFFFFF = unreachable).  *iterations = levels swept.
 * The vertices are handed out in groups of max(coarse, 512) to as many waves as the device holds.  A wave first
 * touches the pages that hold the lists of its group's active vertices (what is not resident comes in as one batch of
 * commands), then reads the lists of 64 vertices at a time through bam_ptr, 64 entries per step across list ends.
 * Lists of 1024 entries and more are walked in pieces of 8192 entries by a wave each; the pieces are listed once per
 * call and handed out in every sweep before the groups, four per turn, their pages asked for as one batch (the same
 * for bam_cc, bam_sssp and bam_pagerank without by_page). */
int bam_bfs(bam_array_t* edges, const uint64_t* d_offsets, uint64_t n_vertices, uint64_t src, uint32_t* d_labels,
            uint32_t coarse, uint32_t* iterations, void* stream);
/* ---- the reference's other launch shapes of BFS and CC (benchmarks/bfs/main.cu:733-760 kernel_coalesce_hash_ptr_pc,
 * :810-850 kernel_coalesce_hash_coarse_ptr_pc, :852-905 kernel_coalesce_hash_half(_ptr_pc), :961-1000 kernel_coalesce_chunk_pc;
 * benchmarks/cc/main.cu has the same set) ----
 * The same levels and labels as bam_bfs / bam_cc, the vertices shared out as those variants do: shape 0 a wave per vertex,
 * wave u taking vertex u / nep + (u % nep) * stride with nep = (V + stride) / stride; shape 1 the same over runs of `coarse`
 * vertices; shape 2 sixteen lanes per vertex (four vertices per wave side by side), strided like shape 0; shape 3 a wave
 * per chunk of eight consecutive vertices.  stride = 1 is the plain order.  These are the reference's kernels as they
 * are, without read-ahead or splitting of long lists: for comparison and for programs that ask for them by name, not for
 * speed (bam_bfs, bam_bfs_by_page). */
int bam_bfs_shaped(bam_array_t* edges, const uint64_t* d_offsets, uint64_t n_vertices, uint64_t src, uint32_t* d_labels,
                   int shape, uint32_t coarse, uint32_t stride, uint32_t* iterations, void* stream);
int bam_cc_shaped(bam_array_t* edges, const uint64_t* d_offsets, uint64_t n_vertices, uint64_t* d_labels,
                  int shape, uint32_t coarse, uint32_t stride, uint32_t* iterations, void* stream);
/* ---- BFS over queues of vertices (benchmarks/bfs/main.cu:409-451 kernel_frontier_coalesce_ptr_pc, queues :1489-1492,
 * host loop :1561-1563, 1702-1711) ----
 * Instead of sweeping all labels, every level walks the queue of the vertices found by the level before and fills the
 * next one: a vertex enters it when the exchange on its label finds it unreached, the lanes of a wave that found one
 * at the same step take their places with one atomic.  Otherwise the walk of bam_bfs (lists packed 64 entries per
 * step, long lists in pieces).  Same levels and the same *iterations as bam_bfs; no result depends on the order of a
 * queue, which is that of discovery when a level ends.  Between levels the queue is put in the order of its vertices (they
 * are distinct: marked in a bit map and read back front to back), so that a level reads the edge array front to back and a wave can take 512 entries at a time and ask
 * for the pages under their lists as one batch, as bam_bfs does for 512 vertices; environment BAM_FRONTIER_SORT=0
 * leaves the queue as it comes (64 entries per wave at a time, first and last page of each list asked for).
 * n_vertices <= 2^32 - 1 (32-bit queue entries). */
int bam_bfs_frontier(bam_array_t* edges, const uint64_t* d_offsets, uint64_t n_vertices, uint64_t src, uint32_t* d_labels,
                     uint32_t* iterations, void* stream);
/* ---- CC (benchmarks/cc/main.cu:123-144 cc_compute, :595-617 kernel, host loop :1410-1425, 1515-1521) ----
 * Min-label propagation; d_labels[V] receives the smallest vertex id of each vertex's component. */
int bam_cc(bam_array_t* edges, const uint64_t* d_offsets, uint64_t n_vertices, uint64_t* d_labels,
           uint32_t coarse, uint32_t* iterations, void* stream);

/* ---- the same two traversals, laid out along the edge array instead of along the vertices ----
 * The reference's page-tiled variant (benchmarks/bfs/main.cu:1074-1140 kernel_optimized_ptr_pc, with the table of the
 * first vertex of every page built by kernel_first_vertex_step1/2, :122-181; the same in benchmarks/cc): one warp per
 * page of the edge array, which it walks vertex by vertex.  Here a wave takes a run of up to 64 consecutive pages,
 * acquires those that hold edges of active vertices with one call (their misses reach the store as one batch of
 * commands) and relaxes those vertices' edges from the resident pages; the table is built by binary search.
 * Same inputs, same outputs as bam_bfs / bam_cc (levels and labels are unique, so they are bit-identical).
 * The array must consist of one range that starts on a page boundary. */
int bam_bfs_by_page(bam_array_t* edges, const uint64_t* d_offsets, uint64_t n_vertices, uint64_t src, uint32_t* d_labels,
                    uint32_t* iterations, void* stream);
int bam_cc_by_page(bam_array_t* edges, const uint64_t* d_offsets, uint64_t n_vertices, uint64_t* d_labels, uint32_t* iterations, void* stream);

/* ---- vectoradd (benchmarks/vectoradd/main.cu:102-117 kernel_baseline_ptr_pc) ----
 * c[i] = a[i] + b[i] for i < n_elems, one thread per element, all three arrays read and written through bam_ptr; the
 * results reach the store when their pages are evicted or the cache is flushed (bam_page_cache_flush).
 * In this kernel, in bam_reduce, bam_scan and in bam_array_read without an assignment, consecutive threads read
 * consecutive (or evenly spaced) elements: the first wave of every window of up to 64 pages touches a window further
 * on, one page per lane, so that the store is asked for pages in batches of a window and not one page per wave
 * (arrays of one range; off for caches under 128 pages).  Results and counters of accesses are not affected. */
int bam_vectoradd(bam_array_t* a, bam_array_t* b, bam_array_t* c, uint64_t n_elems, void* stream);

/* ---- reduction (benchmarks/reduction/main.cu:166-195 kernel_reduce_baseline_ptr_pc, launch :476) ----
 * Workgroup b of block_size threads sums elements [2 b block_size, 2 (b + 1) block_size) of the array, read through
 * bam_ptr, into d_partials[b]; ceil(n_elems / (2 block_size)) partial sums, which the caller adds up as the reference's
 * main() does (:507-511).  The reference's "optimized" variant (:198-237) overwrites one shared buffer from every warp of
 * a block and is not reproduced. */
int bam_reduce(bam_array_t* a, uint64_t n_elems, uint32_t block_size, uint64_t* d_partials, void* stream);

/* ---- scan (benchmarks/scan/main.cu:147-190 kernel_scan_baseline_ptr_pc, :89-100 finalsum, host :413-420) ----
 * d_result[0] = 0, d_result[i + 1] = a[0] + ... + a[i] (mod 2^64) for i < n_elems: n_elems + 1 words, the total last,
 * as the reference lays its result out (:370-373, 405).  Per-block scans of 2 block_size elements read through bam_ptr,
 * a scan of the block totals, and the pass that adds them back. */
int bam_scan(bam_array_t* a, uint64_t n_elems, uint32_t block_size, uint64_t* d_result, void* stream);

/* ---- bam_scan without allocation ----
 * No counterpart in the reference.  For callers that cannot allocate device memory: code under stream capture, tight
 * serving loops, harnesses that forbid it.  Same arguments and same result as bam_scan; the block totals, which bam_scan
 * keeps in a buffer it allocates and frees per call, live in a device array of fixed size inside the library (512 KiB,
 * held by every device the library runs on until the process ends), so n_elems may need at most
 * BAM_SCAN_NOALLOC_MAX_BLOCKS blocks of 2 * block_size elements (E2BIG beyond that, nothing launched).  Calls no
 * hipMalloc / hipFree and does not synchronise; the first call on a device looks the array's address up (make that call
 * outside a capture).  All calls on one device share the array: calls that overlap on a device race. */
#define BAM_SCAN_NOALLOC_MAX_BLOCKS 65536u
int bam_scan_noalloc(bam_array_t* a, uint64_t n_elems, uint32_t block_size, uint64_t* d_result, void* stream);

/* ---- PageRank (benchmarks/pagerank/main.cu: initialize :107-115, kernel_coalesce_pc :252-273, update :412-421,
 * host loop :704-768; the reference runs alpha = 0.85, tolerance = 0.001, at most 100 iterations, :476-477) ----
 * Residual pushes in single precision: every flagged vertex adds its delta to the residual of each neighbour (atomic
 * float adds, neighbour ids through the cache), then every vertex whose residual exceeds `tolerance` moves it into its
 * value and is flagged with delta = residual * alpha / degree.  d_value[V] receives the values; *iterations = sweeps.
 * by_page = 0: vertex by vertex as the reference (the group walk of bam_bfs); 1: along the pages of the edge array as
 * bam_bfs_by_page.
 * The order of the float adds is not fixed (neither is it in the reference), so values agree between runs only to
 * rounding, and a residual that lands within rounding of `tolerance` may be moved one sweep earlier or later;
 * whatever the order, on return 0 <= x - value <= x * tolerance / (1 - alpha) up to rounding, x the exact solution of
 * x = (1 - alpha) + alpha * sum over in-neighbours u of x_u / degree(u). */
int bam_pagerank(bam_array_t* edges, const uint64_t* d_offsets, uint64_t n_vertices, float alpha, float tolerance, uint32_t max_iterations,
                 int by_page, float* d_value, uint32_t* iterations, void* stream);

/* ---- arrays of 32-bit elements (the weight arrays of the reference's weighted-graph benchmarks are array_t<WeightT>,
 * WeightT = uint32_t, benchmarks/sssp/main.cu:69, 640-661) ----
 * Same arguments as the 64-bit handles; ranges of both element sizes may share one page cache. */
int bam_range32_create(bam_range32_t** out, uint64_t index_start, uint64_t count, uint64_t page_start, uint64_t page_count,
                       uint64_t page_start_offset, uint64_t page_size, bam_page_cache_t* pc, uint32_t device, int dist);
void bam_range32_destroy(bam_range32_t* r);
int bam_array32_create(bam_array32_t** out, uint64_t n_elems, uint64_t disk_start_offset, bam_range32_t** ranges, uint32_t n_ranges, uint32_t device);
void bam_array32_destroy(bam_array32_t* a);
/* out[4]: read_io_cnt, access_cnt, miss_cnt, hit_cnt since the last call */
int bam_array32_stats(bam_array32_t* a, uint64_t* out);
/* thread t reads element d_assignment[t] (or t * stride); the values read are summed into *d_sum */
int bam_array32_read(bam_array32_t* a, uint64_t n_reqs, const uint64_t* d_assignment, uint64_t stride, uint32_t block_size, uint64_t* d_sum, void* stream);

/* ---- SSSP (benchmarks/sssp/main.cu:174-201 kernel_coalesce_pc, :282-292 update, host loop :663-725) ----
 * Rounds of relax + update from src until nothing changes: neighbour ids through `edges`, one 32-bit weight per CSR
 * entry through `weights`; d_costs[V] receives the cost of the cheapest path to every vertex (0xFFFFFFFF =
 * unreachable).  *iterations = rounds. */
int bam_sssp(bam_array_t* edges, bam_array32_t* weights, const uint64_t* d_offsets, uint64_t n_vertices, uint64_t src, uint32_t* d_costs,
             uint32_t* iterations, void* stream);
/* ---- SSSP with single-precision weights (benchmarks/sssp_float/main.cu: WeightT = float :69, AtomicMin :91-106,
 * kernel_coalesce_pc :194-217, update :302-312, unreached = 1e9 :529) ----
 * The elements of `weights` are the bit patterns of floats, which must not be negative (nor NaN); d_costs[V] receives
 * the least cost, each path's weights added in single precision from the source on (1e9 = unreached, and a path is
 * only taken while its cost stays below that).  Costs that are not negative order as their bit patterns, so the
 * minimum is the integer atomic on the pattern.  Adding a weight keeps the order of two costs, so the result does not
 * depend on the order of relaxation: bit-exact against a serial Dijkstra in single precision. */
int bam_sssp_float(bam_array_t* edges, bam_array32_t* weights, const uint64_t* d_offsets, uint64_t n_vertices, uint64_t src, float* d_costs,
                   uint32_t* iterations, void* stream);

/* ---- synthetic inputs on the device (no counterpart in the reference, which reads dataset files) ---- */
int bam_gen_words(uint64_t seed, uint64_t first, uint64_t n, uint64_t* d_out, void* stream);                 /* out[k] = splitmix64(seed, first + k) */
int bam_gen_mod(uint64_t seed, uint64_t first, uint64_t n, uint64_t modulus, uint64_t scale, uint64_t* d_out, void* stream); /* (splitmix64(seed, first+k) % modulus) * scale */
int bam_gen_rmat(uint64_t seed, uint32_t scale, uint64_t first_edge, uint64_t n, uint64_t* d_u, uint64_t* d_v, void* stream);
int bam_gen_uniform(uint64_t seed, uint64_t n_vertices, uint64_t first_pair, uint64_t n, uint64_t* d_u, uint64_t* d_v, void* stream);

/* ---- measurement helpers ----
 * plain device copy of n bytes (calibration of traffic counters), and a bulk read of host-pinned memory by the
 * GPU (the interconnect ceiling of staged transfers); both return elapsed milliseconds measured with HIP events. */
int bam_copy_kernel(const void* d_src, void* d_dst, uint64_t n_bytes, float* ms, void* stream);
int bam_host_read_ceiling(uint64_t n_bytes, uint32_t chunk_bytes, float* ms);
/* what the memory system gives plain kernels with the access patterns of the hit path, no cache protocol: a streaming
 * read of n bytes, and a gather of n 8-byte words at d_idx[] from d_src; elapsed milliseconds */
int bam_read_kernel(const void* d_src, uint64_t n_bytes, float* ms, void* stream);
int bam_gather_kernel(const uint64_t* d_src, const uint64_t* d_idx, uint64_t n, float* ms, void* stream);
/* The hit path of the streaming kernels taken apart (measurement only): n_waves waves read runs of n_pages_per_wave pages of
 * the array's one range, which must all be resident and must stay so (nothing may evict meanwhile), and add every word into
 * *d_sum.  refs 0: the descriptor is read for the slot, no reference taken; 1: a reference per page, taken before and dropped
 * after, as bam_ptr does; 2: the references of sixteen pages per vector atomic, as the page-wise kernel does.  not_kept:
 * payload loads marked as not to be kept in the L2.  Against bam_read_kernel (no protocol at all) the six say what each part
 * costs.  4 KiB pages. */
int bam_hit_path_parts(bam_array_t* a, int refs, int not_kept, uint64_t n_waves, uint64_t n_pages_per_wave, uint64_t* d_sum, void* stream);
/* the atomics of a hit that takes and drops a reference, without the cache around them: per request an add on the 8-byte
 * word d_table[d_idx[t]] and, once it is back, the opposite add on the same word (the table ends as it began).
 * returns != 0: the first add hands back the old word, as bam_try_hit needs it; 0: neither result is read. */
int bam_atomic_pairs_kernel(uint64_t* d_table, const uint64_t* d_idx, uint64_t n, int returns, float* ms, void* stream);
/* Pages handed between the compute-unit clusters of the device (each has an L2 of its own): n_waves workgroups of one wave,
 * dealt out over the clusters by the dispatcher; in round r wave r % n_waves reads page r % n_pages (of page_bytes, the
 * cache's page size) of a procedural store with seed `seed` into the cache (choose the cache smaller than n_pages, so every round re-uses a slot), the others wait
 * for it (bounded by spin_limit looks, 0 = 2^22) and then compare elements of that page, read through operator[], with the
 * store's words.  out4 (host): elements that differed, waits given up, bit mask of the clusters that ran waves, reads
 * compared.  No counterpart in the reference, whose GPUs have one L2. */
int bam_xcd_relay(bam_array_t* a, uint64_t seed, uint32_t page_bytes, uint32_t n_pages, uint32_t rounds, uint32_t n_waves, uint32_t spin_limit, uint64_t* out4, void* stream);
/* time a callback-free region: record/elapsed on the stream the kernels above were launched on */
int bam_event_create(void** ev);
int bam_event_record(void* ev, void* stream);
int bam_event_elapsed_ms(void* start, void* stop, float* ms);
void bam_event_destroy(void* ev);
/* protocol ceiling of the target with plain host clients (nvmt_selftest_iops) */
double bam_target_ceiling_iops(uint64_t ns_bytes, uint32_t lba_bytes, int backing, uint32_t n_io_threads, uint32_t n_clients,
                               uint32_t depth, uint64_t n_cmds, uint32_t req_bytes);

#ifdef __cplusplus
}
#endif
#endif /* __BAM_AMD_H__ */
