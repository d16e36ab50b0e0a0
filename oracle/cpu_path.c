/*
 * CPU restatement of the reference's GPU-side storage-access path.
 * TEST INFRASTRUCTURE ONLY (checker and CPU baseline); the shipped library
 * never links or calls this file.
 *
 * One software lane per POSIX thread, C11 atomics where the reference uses
 * simt::atomic (semantics of that un-vendored template: parity unpinned, ISO
 * C++11 atomics assumed).  Restated from the reference, function by function:
 *   get_cid / put_cid          include/nvm_parallel_queue.h:35-57
 *   move_tail                  :59-80   (without the stray head_lock increment at :78)
 *   move_head_cq               :82-123
 *   sq_enqueue                 :167-330
 *   cq_poll                    :378-422
 *   cq_dequeue                 :424-535
 *   read_data                  include/page_cache.h:2009-2054 (without enqueue_second :1961-2007,
 *                              a PCIe visibility work-around with no effect on results)
 *   acquire_page / release     include/page_cache.h:1122-1224, 1091-1094
 *   find_slot                  include/page_cache.h:1786-1927 (read-only ranges: no dirty write-back)
 *   seq_read                   include/page_cache.h:1541-1574 with a one-lane "warp" (count = 1)
 *   bam_ptr                    include/page_cache.h:414-485
 *   BFS / CC loops             benchmarks/bfs/main.cu:658-689,1577-1736; benchmarks/cc/main.cu:123-144,595-617
 * It drives the same software NVMe target as the GPU path, through the same
 * NVMe host API (controller bring-up, admin queue, queue creation).
 *
 * Pinned by: closed-form sums (bam_oracle.c), the counter invariants of the
 * reference's logs (read I/Os = distinct pages first touched when nothing is
 * evicted; accesses = number of lane accesses), textbook BFS/CC.
 */
#define _GNU_SOURCE
#include <errno.h>
#include <pthread.h>
#include <sched.h>
#include <stdatomic.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "nvm_admin.h"
#include "nvm_aq.h"
#include "nvm_cmd.h"
#include "nvm_ctrl.h"
#include "nvm_dma.h"
#include "nvm_types.h"
#include "nvmt.h"

#define LOCKED 1u
#define UNLOCKED 0u
#define FREE 2u
#define VALID 0x80000000u
#define BUSY 0x40000000u
#define DIRTY 0x20000000u
#define CNT_MASK 0x1fffffffu
#define NV_NB 0u
#define V_NB 2u
#define N_CIDS 65536u

typedef struct { _Atomic uint32_t val; uint8_t pad[28]; } padded_t;   /* include/nvm_types.h:94-98 */

typedef struct {
    _Atomic uint32_t head_lock; uint8_t p0[28];
    _Atomic uint32_t tail_lock; uint8_t p1[28];
    _Atomic uint32_t head;      uint8_t p2[28];
    _Atomic uint32_t tail;      uint8_t p3[28];
    _Atomic uint32_t in_ticket; uint8_t p4[28];
    _Atomic uint32_t cid_ticket; uint8_t p5[28];
    padded_t *tickets, *head_mark, *tail_mark, *cid, *pos_locks;
    uint32_t qs, qs_minus_1, qs_log2;
    volatile uint32_t* db;
    volatile void* vaddr;
} queue_t;

typedef struct { queue_t sq, cq; nvm_queue_t nsq, ncq; nvm_dma_t *sq_mem, *cq_mem; uint32_t block_size_log, nsid; } qpair_t;

typedef struct { _Atomic uint32_t state; uint32_t offset; uint8_t pad[24]; } data_page_t;         /* include/page_cache.h:96-102 */
typedef struct { _Atomic uint32_t page_take_lock; uint64_t page_translation; uint8_t pad[16]; } cache_page_t;  /* :487-493 */

typedef struct bo_cpu_path {
    nvmt_config_t cfg;
    nvmt_t* target;
    void* bar;
    nvm_ctrl_t* ctrl;
    nvm_dma_t* aq_mem;
    nvm_aq_ref aq;
    uint32_t n_qps;
    qpair_t* qps;
    /* page cache */
    uint64_t page_size, page_size_log, n_pages, n_blocks_per_page, n_data_pages;
    uint8_t* base_addr;
    cache_page_t* cache_pages;
    _Atomic uint32_t page_ticket;
    data_page_t* pages;
    uint64_t page_start;
    _Atomic uint64_t access_cnt, miss_cnt, hit_cnt, read_io_cnt;
} bo_cpu_path_t;

static inline void relax(unsigned* ns)
{
    /* stands for __nanosleep(ns), ns doubling up to 256 */
    for (unsigned i = 0; i < *ns / 8; i++) __builtin_ia32_pause();
    if (*ns < 256) *ns *= 2; else sched_yield();
}

/* ---- queue protocol ---- */
static uint16_t get_cid(queue_t* sq)
{
    uint32_t id, old;
    do {
        id = atomic_fetch_add_explicit(&sq->cid_ticket, 1, memory_order_relaxed) & (N_CIDS - 1);
        old = atomic_fetch_or_explicit(&sq->cid[id].val, LOCKED, memory_order_acquire);
    } while (old == LOCKED);
    return (uint16_t)id;
}

static void put_cid(queue_t* sq, uint16_t id) { atomic_store_explicit(&sq->cid[id].val, UNLOCKED, memory_order_release); }

static uint32_t move_tail(queue_t* q, uint32_t cur_tail)
{
    uint32_t count = 0;
    int pass = 1;
    while (pass) {
        pass = ((cur_tail + count + 1) & q->qs_minus_1) != (atomic_load_explicit(&q->head, memory_order_relaxed) & q->qs_minus_1);
        if (pass) {
            pass = atomic_exchange_explicit(&q->tail_mark[(cur_tail + count) & q->qs_minus_1].val, UNLOCKED, memory_order_relaxed) == LOCKED;
            if (pass) count++;
        }
    }
    return count;
}

static uint32_t move_head_cq(queue_t* q, uint32_t cur_head, queue_t* sq)
{
    uint32_t count = 0;
    int pass = 1;
    while (pass) {
        uint32_t loc = (cur_head + count++) & q->qs_minus_1;
        pass = atomic_exchange_explicit(&q->head_mark[loc].val, UNLOCKED, memory_order_relaxed) == LOCKED;
    }
    count -= 1;
    if (count) {
        uint32_t last = (cur_head + (count - 1)) & q->qs_minus_1;
        uint32_t new_sq_head = ((volatile nvm_cpl_t*)q->vaddr)[last].dword[2] & 0xffffu;
        uint32_t n = 0, loc = atomic_load_explicit(&sq->head, memory_order_relaxed) & sq->qs_minus_1;
        for (; loc != new_sq_head; n++, loc = (loc + 1) & sq->qs_minus_1)
            atomic_fetch_add_explicit(&sq->tickets[loc].val, 1, memory_order_relaxed);
        if (n) atomic_fetch_add_explicit(&sq->head, n, memory_order_acq_rel);
    }
    return count;
}

static uint16_t sq_enqueue(queue_t* sq, const nvm_cmd_t* cmd)
{
    uint32_t ticket = atomic_fetch_add_explicit(&sq->in_ticket, 1, memory_order_relaxed);
    uint32_t pos = ticket & sq->qs_minus_1;
    uint32_t id = (ticket >> sq->qs_log2) * 2;
    unsigned ns = 8;
    while (atomic_load_explicit(&sq->tickets[pos].val, memory_order_acquire) != id) relax(&ns);
    memcpy((void*)(((nvm_cmd_t*)sq->vaddr) + pos), cmd, sizeof(nvm_cmd_t));
    atomic_store_explicit(&sq->tail_mark[pos].val, LOCKED, memory_order_release);
    ns = 8;
    while (atomic_load_explicit(&sq->tail_mark[pos].val, memory_order_relaxed) == LOCKED) {
        if (atomic_load_explicit(&sq->tail_lock, memory_order_relaxed) != LOCKED &&
            atomic_fetch_or_explicit(&sq->tail_lock, LOCKED, memory_order_acquire) != LOCKED) {
            uint32_t cur_tail = atomic_load_explicit(&sq->tail, memory_order_relaxed);
            uint32_t moved = move_tail(sq, cur_tail);
            if (moved) {
                __atomic_store_n((uint32_t*)sq->db, (cur_tail + moved) & sq->qs_minus_1, __ATOMIC_RELEASE);
                atomic_store_explicit(&sq->tail, cur_tail + moved, memory_order_release);
            }
            atomic_store_explicit(&sq->tail_lock, UNLOCKED, memory_order_release);
        }
        if (atomic_load_explicit(&sq->tail_mark[pos].val, memory_order_relaxed) == LOCKED) relax(&ns);
    }
    atomic_fetch_add_explicit(&sq->tickets[pos].val, 1, memory_order_acq_rel);
    return (uint16_t)pos;
}

static uint32_t cq_poll(queue_t* cq, uint16_t search_cid, uint32_t* loc_, uint32_t* cq_head)
{
    unsigned ns = 8;
    for (;;) {
        uint32_t head = atomic_load_explicit(&cq->head, memory_order_relaxed);
        for (uint32_t i = 0; i < cq->qs_minus_1; i++) {
            uint32_t cur = head + i;
            uint32_t search_phase = (~(cur >> cq->qs_log2)) & 1u;
            uint32_t loc = cur & cq->qs_minus_1;
            uint32_t e = __atomic_load_n((uint32_t*)&((volatile nvm_cpl_t*)cq->vaddr)[loc].dword[3], __ATOMIC_ACQUIRE);
            uint32_t phase = (e >> 16) & 1u;
            if ((e & 0xffffu) == search_cid && phase == search_phase) { *cq_head = head; *loc_ = cur; return loc; }
            if (phase != search_phase) break;
        }
        relax(&ns);
    }
}

static void cq_dequeue(queue_t* cq, uint16_t pos, queue_t* sq, uint32_t loc_, uint32_t cur_head_)
{
    unsigned ns = 8;
    atomic_fetch_add_explicit(&cq->tail, 1, memory_order_acq_rel);
    while (atomic_fetch_or_explicit(&cq->pos_locks[pos].val, 1, memory_order_acquire) != 0) relax(&ns);
    atomic_store_explicit(&cq->head_mark[pos].val, LOCKED, memory_order_release);
    ns = 8;
    while (atomic_load_explicit(&cq->head_mark[pos].val, memory_order_relaxed) == LOCKED) {
        if (atomic_fetch_or_explicit(&cq->head_lock, LOCKED, memory_order_acquire) != LOCKED) {
            uint32_t cur_head = atomic_load_explicit(&cq->head, memory_order_relaxed);
            uint32_t moved = move_head_cq(cq, cur_head, sq);
            if (moved) {
                __atomic_store_n((uint32_t*)cq->db, (cur_head + moved) & cq->qs_minus_1, __ATOMIC_RELEASE);
                atomic_store_explicit(&cq->head, cur_head + moved, memory_order_release);
            }
            atomic_store_explicit(&cq->head_lock, UNLOCKED, memory_order_release);
        }
        if (atomic_load_explicit(&cq->head_mark[pos].val, memory_order_relaxed) == LOCKED) relax(&ns);
    }
    /* wait until the head has passed this entry, so a next-lap completion in the slot is not marked early */
    ns = 8;
    for (;;) {
        uint32_t new_head = atomic_load_explicit(&cq->head, memory_order_relaxed);
        if (new_head > cur_head_) { if (loc_ >= cur_head_ && loc_ < new_head) break; }
        else if (new_head < cur_head_) { if (loc_ >= cur_head_ || loc_ < new_head) break; }
        relax(&ns);
    }
    atomic_store_explicit(&cq->pos_locks[pos].val, 0, memory_order_release);
}

/* one NVMe read of n_blocks at starting_lba into dst (include/page_cache.h:2009-2054) */
static void read_data(qpair_t* qp, uint64_t starting_lba, uint64_t n_blocks, void* dst)
{
    nvm_cmd_t cmd;
    memset(&cmd, 0, sizeof(cmd));
    uint16_t cid = get_cid(&qp->sq);
    nvm_cmd_header(&cmd, cid, NVM_IO_READ, qp->nsid);
    nvm_cmd_data_ptr(&cmd, (uint64_t)(uintptr_t)dst, 0);
    nvm_cmd_rw_blks(&cmd, starting_lba, (uint16_t)n_blocks);
    sq_enqueue(&qp->sq, &cmd);
    uint32_t head, head_;
    uint32_t cq_pos = cq_poll(&qp->cq, cid, &head, &head_);
    cq_dequeue(&qp->cq, (uint16_t)cq_pos, &qp->sq, head, head_);
    put_cid(&qp->sq, cid);
}

/* ---- page cache ---- */
static uint32_t find_slot(bo_cpu_path_t* p, uint64_t address)
{
    for (;;) {
        uint32_t page = atomic_fetch_add_explicit(&p->page_ticket, 1, memory_order_relaxed) % p->n_pages;
        cache_page_t* cp = &p->cache_pages[page];
        uint32_t v = atomic_load_explicit(&cp->page_take_lock, memory_order_relaxed);
        if (v == FREE) {
            if (atomic_compare_exchange_strong_explicit(&cp->page_take_lock, &v, LOCKED, memory_order_acquire, memory_order_relaxed)) {
                cp->page_translation = address;
                atomic_store_explicit(&cp->page_take_lock, UNLOCKED, memory_order_release);
                return page;
            }
        } else if (v == UNLOCKED) {
            if (atomic_compare_exchange_strong_explicit(&cp->page_take_lock, &v, LOCKED, memory_order_acquire, memory_order_relaxed)) {
                int ok = 0;
                data_page_t* victim = &p->pages[cp->page_translation];
                uint32_t e = atomic_load_explicit(&victim->state, memory_order_relaxed);
                if ((e & CNT_MASK) == 0 && (e & BUSY) == 0) {
                    uint32_t o = atomic_fetch_or_explicit(&victim->state, BUSY, memory_order_acquire);
                    if ((o & BUSY) == 0) {
                        if ((o & CNT_MASK) == 0) {
                            atomic_fetch_and_explicit(&victim->state, CNT_MASK, memory_order_release);
                            cp->page_translation = address;
                            ok = 1;
                        } else atomic_fetch_and_explicit(&victim->state, ~BUSY, memory_order_release);
                    }
                }
                atomic_store_explicit(&cp->page_take_lock, UNLOCKED, memory_order_release);
                if (ok) return page;
            }
        }
    }
}

static uint32_t acquire_page(bo_cpu_path_t* p, uint64_t pg, uint32_t count, uint32_t queue)
{
    data_page_t* dp = &p->pages[pg];
    unsigned ns = 8;
    atomic_fetch_add_explicit(&p->access_cnt, count, memory_order_relaxed);
    uint32_t s = atomic_fetch_add_explicit(&dp->state, count, memory_order_acquire);
    for (;;) {
        uint32_t st = (s >> 30) & 3u;
        if (st == NV_NB) {
            uint32_t o = atomic_fetch_or_explicit(&dp->state, BUSY, memory_order_acquire);
            if ((o & BUSY) == 0) {
                if (((o >> 30) & 3u) == NV_NB) {
                    uint32_t slot = find_slot(p, pg);
                    atomic_fetch_add_explicit(&p->read_io_cnt, 1, memory_order_relaxed);
                    read_data(&p->qps[queue % p->n_qps], (p->page_start + pg) * p->n_blocks_per_page, p->n_blocks_per_page,
                              p->base_addr + (uint64_t)slot * p->page_size);
                    dp->offset = slot;
                    atomic_fetch_add_explicit(&p->miss_cnt, count, memory_order_relaxed);
                    atomic_fetch_xor_explicit(&dp->state, VALID | BUSY, memory_order_release);
                    return slot;
                }
                atomic_fetch_and_explicit(&dp->state, ~BUSY, memory_order_release);
            }
        } else if (st == V_NB) {
            atomic_fetch_add_explicit(&p->hit_cnt, count, memory_order_relaxed);
            return dp->offset;
        }
        relax(&ns);
        s = atomic_load_explicit(&dp->state, memory_order_acquire);
    }
}

static inline void release_page(bo_cpu_path_t* p, uint64_t pg, uint32_t count)
{
    atomic_fetch_sub_explicit(&p->pages[pg].state, count, memory_order_release);
}

static inline uint64_t seq_read(bo_cpu_path_t* p, uint64_t i, uint32_t queue)
{
    uint64_t pg = (i * 8) >> p->page_size_log, sub = (i * 8) & (p->page_size - 1);
    uint32_t slot = acquire_page(p, pg, 1, queue);
    uint64_t v = *(volatile uint64_t*)(p->base_addr + (uint64_t)slot * p->page_size + sub);
    release_page(p, pg, 1);
    return v;
}

/* bam_ptr: keeps the page of the last access referenced */
typedef struct { bo_cpu_path_t* p; uint64_t start, end, pg; const uint64_t* addr; int held; uint32_t queue; } cpu_bam_ptr_t;

static inline uint64_t ptr_read(cpu_bam_ptr_t* b, uint64_t i)
{
    if (i < b->start || i >= b->end) {
        if (b->held) release_page(b->p, b->pg, 1);
        uint64_t epp = b->p->page_size / 8;
        b->pg = i / epp;
        uint32_t slot = acquire_page(b->p, b->pg, 1, b->queue);
        b->addr = (const uint64_t*)(b->p->base_addr + (uint64_t)slot * b->p->page_size);
        b->start = b->pg * epp; b->end = b->start + epp; b->held = 1;
    }
    return ((volatile const uint64_t*)b->addr)[i - b->start];
}

static inline void ptr_fini(cpu_bam_ptr_t* b) { if (b->held) { release_page(b->p, b->pg, 1); b->held = 0; } }

/* ---- set-up ---- */
static void* zalloc(size_t n) { void* m = NULL; if (posix_memalign(&m, 4096, n ? n : 1)) return NULL; memset(m, 0, n); return m; }

static int queue_init(queue_t* q, const nvm_queue_t* nq, int is_sq)
{
    memset(q, 0, sizeof(*q));
    q->qs = nq->qs; q->qs_minus_1 = nq->qs - 1; q->qs_log2 = nq->qs_log2; q->db = nq->db; q->vaddr = nq->vaddr;
    if (is_sq) {
        q->tickets = zalloc(q->qs * sizeof(padded_t));
        q->tail_mark = zalloc(q->qs * sizeof(padded_t));
        q->cid = zalloc(N_CIDS * sizeof(padded_t));
        return q->tickets && q->tail_mark && q->cid ? 0 : ENOMEM;
    }
    q->head_mark = zalloc(q->qs * sizeof(padded_t));
    q->pos_locks = zalloc(q->qs * sizeof(padded_t));
    return q->head_mark && q->pos_locks ? 0 : ENOMEM;
}

void bo_cpu_path_destroy(bo_cpu_path_t* p);

bo_cpu_path_t* bo_cpu_path_create(uint64_t ns_bytes, uint32_t lba_bytes, uint64_t seed, void* backing, uint32_t n_io_threads,
                                  uint32_t n_queues, uint32_t queue_depth, uint64_t page_size, uint64_t cache_pages,
                                  uint64_t n_elems, uint64_t disk_offset_bytes)
{
    bo_cpu_path_t* p = calloc(1, sizeof(*p));
    if (!p) return NULL;
    p->cfg.ns_bytes = ns_bytes; p->cfg.lba_bytes = lba_bytes; p->cfg.seed = seed; p->cfg.backing = backing;
    p->cfg.n_io_threads = n_io_threads; p->cfg.max_queue_entries = 1024; p->cfg.max_io_queues = 128; p->cfg.dstrd = 4;
    p->bar = zalloc(nvmt_bar_size(&p->cfg));
    p->target = p->bar ? nvmt_create(&p->cfg, p->bar) : NULL;
    uint16_t ncq = (uint16_t)n_queues, nsq = (uint16_t)n_queues;
    int ok = p->target &&
             nvm_raw_ctrl_init(&p->ctrl, nvmt_bar(p->target), nvmt_bar_size(&p->cfg)) == 0 &&
             nvm_dma_create(&p->aq_mem, p->ctrl, 3 * p->ctrl->page_size) == 0 &&
             nvm_aq_create(&p->aq, p->ctrl, p->aq_mem) == 0 &&
             nvm_admin_request_num_queues(p->aq, &ncq, &nsq) == 0;
    p->qps = ok ? calloc(n_queues, sizeof(qpair_t)) : NULL;
    for (uint32_t i = 0; ok && p->qps && i < n_queues; i++) {
        qpair_t* q = &p->qps[i];
        ok = nvm_dma_create(&q->cq_mem, p->ctrl, queue_depth * sizeof(nvm_cpl_t)) == 0 &&
             nvm_dma_create(&q->sq_mem, p->ctrl, queue_depth * sizeof(nvm_cmd_t)) == 0 &&
             nvm_admin_cq_create(p->aq, &q->ncq, (uint16_t)(i + 1), q->cq_mem, 0, queue_depth, 0) == 0 &&
             nvm_admin_sq_create(p->aq, &q->nsq, &q->ncq, (uint16_t)(i + 1), q->sq_mem, 0, queue_depth, 0) == 0 &&
             queue_init(&q->sq, &q->nsq, 1) == 0 && queue_init(&q->cq, &q->ncq, 0) == 0;
        q->block_size_log = (uint32_t)__builtin_ctz(lba_bytes); q->nsid = 1;
        if (ok) p->n_qps = i + 1;
    }
    p->page_size = page_size; p->page_size_log = (uint64_t)__builtin_ctzll(page_size);
    p->n_pages = cache_pages; p->n_blocks_per_page = page_size / lba_bytes;
    p->n_data_pages = (n_elems * 8 + page_size - 1) / page_size;
    p->page_start = disk_offset_bytes / page_size;
    p->base_addr = zalloc(page_size * cache_pages);
    p->cache_pages = zalloc(cache_pages * sizeof(cache_page_t));
    p->pages = zalloc(p->n_data_pages * sizeof(data_page_t));
    if (!ok || !p->qps || !p->base_addr || !p->cache_pages || !p->pages) { bo_cpu_path_destroy(p); return NULL; }
    for (uint64_t i = 0; i < cache_pages; i++) atomic_store(&p->cache_pages[i].page_take_lock, FREE);
    return p;
}

void bo_cpu_path_destroy(bo_cpu_path_t* p)
{
    if (!p) return;
    for (uint32_t i = 0; p->qps && i < p->n_qps; i++) {
        qpair_t* q = &p->qps[i];
        if (q->nsq.db) nvm_admin_sq_delete(p->aq, &q->nsq, &q->ncq);
        if (q->ncq.db) nvm_admin_cq_delete(p->aq, &q->ncq);
        nvm_dma_unmap(q->sq_mem); nvm_dma_unmap(q->cq_mem);
        free(q->sq.tickets); free(q->sq.tail_mark); free(q->sq.cid); free(q->cq.head_mark); free(q->cq.pos_locks);
    }
    free(p->qps);
    nvm_aq_destroy(p->aq);
    nvm_dma_unmap(p->aq_mem);
    nvm_ctrl_free(p->ctrl);
    nvmt_destroy(p->target);
    free(p->bar); free(p->base_addr); free(p->cache_pages); free(p->pages);
    free(p);
}

void bo_cpu_path_stats(bo_cpu_path_t* p, uint64_t out[4], int reset)
{
    out[0] = atomic_load(&p->read_io_cnt); out[1] = atomic_load(&p->access_cnt);
    out[2] = atomic_load(&p->miss_cnt); out[3] = atomic_load(&p->hit_cnt);
    if (reset) { atomic_store(&p->read_io_cnt, 0); atomic_store(&p->access_cnt, 0); atomic_store(&p->miss_cnt, 0); atomic_store(&p->hit_cnt, 0); }
}

/* invariants of the page state machine at quiescence: every state is INVALID or VALID with no references,
 * every valid page's slot translates back to it, no two valid pages share a slot.  0 = all hold. */
int bo_cpu_path_check(bo_cpu_path_t* p)
{
    uint8_t* used = calloc(p->n_pages, 1);
    int bad = 0;
    for (uint64_t g = 0; g < p->n_data_pages; g++) {
        uint32_t s = atomic_load(&p->pages[g].state);
        if (s & (CNT_MASK | BUSY)) bad |= 1;
        if (s & VALID) {
            uint32_t o = p->pages[g].offset;
            if (o >= p->n_pages || p->cache_pages[o].page_translation != g) bad |= 2;
            else if (used[o]++) bad |= 4;
        }
    }
    for (uint32_t i = 0; i < p->n_qps; i++) {
        queue_t* sq = &p->qps[i].sq;
        if (atomic_load(&sq->tail) - atomic_load(&sq->head) > sq->qs - 1) bad |= 8;
        for (uint32_t c = 0; c < N_CIDS; c++) if (atomic_load(&sq->cid[c].val)) { bad |= 16; break; }
    }
    free(used);
    return bad;
}

/* ---- workloads ---- */
typedef struct {
    bo_cpu_path_t* p; uint32_t tid, n_threads;
    uint64_t n_reqs; const uint64_t* idx; uint64_t stride; uint64_t sum;
    /* block */
    uint32_t req_bytes; uint64_t* checksums; uint8_t* scratch;
    /* graphs */
    const uint64_t* offsets; uint64_t n_vertices; uint32_t* levels; uint64_t* comp; uint8_t *curr, *next;
    uint32_t level; _Atomic int* changed; pthread_barrier_t* bar; int* stop;
} work_t;

static void* array_worker(void* arg)
{
    work_t* w = arg;
    uint64_t s = 0;
    /* thread t takes requests t, t + T, t + 2T, ... (the way consecutive GPU threads take consecutive requests) */
    for (uint64_t k = w->tid; k < w->n_reqs; k += w->n_threads)
        s += seq_read(w->p, w->idx ? w->idx[k] : k * w->stride, w->tid);
    w->sum = s;
    return NULL;
}

static uint64_t run_threads(work_t* proto, uint32_t n_threads, void* (*fn)(void*))
{
    pthread_t* th = calloc(n_threads, sizeof(*th));
    work_t* w = calloc(n_threads, sizeof(*w));
    uint64_t sum = 0;
    for (uint32_t t = 0; t < n_threads; t++) { w[t] = *proto; w[t].tid = t; w[t].n_threads = n_threads; pthread_create(&th[t], NULL, fn, &w[t]); }
    for (uint32_t t = 0; t < n_threads; t++) { pthread_join(th[t], NULL); sum += w[t].sum; }
    free(th); free(w);
    return sum;
}

/* array benchmark: n_reqs element reads through seq_read, sum mod 2^64 */
uint64_t bo_cpu_array_sum(bo_cpu_path_t* p, uint32_t n_threads, uint64_t n_reqs, const uint64_t* idx, uint64_t stride)
{
    work_t w; memset(&w, 0, sizeof(w));
    w.p = p; w.n_reqs = n_reqs; w.idx = idx; w.stride = stride;
    return run_threads(&w, n_threads, array_worker);
}

static void* block_worker(void* arg)
{
    work_t* w = arg;
    qpair_t* qp = &w->p->qps[w->tid % w->p->n_qps];
    uint8_t* buf = zalloc(4096);
    for (uint64_t k = w->tid; k < w->n_reqs; k += w->n_threads) {
        read_data(qp, w->idx[k], w->req_bytes >> qp->block_size_log, buf);
        uint64_t s = 0;
        for (uint32_t i = 0; i < w->req_bytes / 8; i++) s += ((uint64_t*)buf)[i];
        if (w->checksums) w->checksums[k] = s;
        w->sum += s;
    }
    free(buf);
    return NULL;
}

/* raw block benchmark: one command per request, no cache; per-request payload checksums */
uint64_t bo_cpu_block_reads(bo_cpu_path_t* p, uint32_t n_threads, uint64_t n_reqs, const uint64_t* lbas, uint32_t req_bytes, uint64_t* checksums)
{
    work_t w; memset(&w, 0, sizeof(w));
    w.p = p; w.n_reqs = n_reqs; w.idx = lbas; w.req_bytes = req_bytes; w.checksums = checksums;
    return run_threads(&w, n_threads, block_worker);
}

static void* bfs_worker(void* arg)
{
    work_t* w = arg;
    cpu_bam_ptr_t ptr = { w->p, 0, 0, 0, NULL, 0, w->tid };
    for (;;) {
        pthread_barrier_wait(w->bar);
        if (*w->stop) break;
        uint32_t level = *(volatile uint32_t*)&((work_t*)w)->levels[w->n_vertices];   /* current level is parked past the end */
        for (uint64_t v = w->tid; v < w->n_vertices; v += w->n_threads) {
            if (__atomic_load_n(&w->levels[v], __ATOMIC_RELAXED) != level) continue;
            for (uint64_t i = w->offsets[v]; i < w->offsets[v + 1]; i++) {
                uint64_t next = ptr_read(&ptr, i);
                if (__atomic_load_n(&w->levels[next], __ATOMIC_RELAXED) == 0xFFFFFFFFu) {
                    __atomic_store_n(&w->levels[next], level + 1, __ATOMIC_RELAXED);
                    atomic_store(w->changed, 1);
                }
            }
        }
        ptr_fini(&ptr);
        pthread_barrier_wait(w->bar);
    }
    return NULL;
}

/* level-synchronous BFS, edges through the cache; levels must have n_vertices + 1 entries; returns launches */
uint32_t bo_cpu_bfs(bo_cpu_path_t* p, uint32_t n_threads, const uint64_t* offsets, uint64_t n_vertices, uint64_t src, uint32_t* levels)
{
    pthread_barrier_t bar;
    _Atomic int changed = 0;
    int stop = 0;
    pthread_barrier_init(&bar, NULL, n_threads + 1);
    memset(levels, 0xFF, n_vertices * sizeof(uint32_t));
    levels[src] = 0;
    pthread_t* th = calloc(n_threads, sizeof(*th));
    work_t* w = calloc(n_threads, sizeof(*w));
    for (uint32_t t = 0; t < n_threads; t++) {
        w[t].p = p; w[t].tid = t; w[t].n_threads = n_threads; w[t].offsets = offsets; w[t].n_vertices = n_vertices;
        w[t].levels = levels; w[t].changed = &changed; w[t].bar = &bar; w[t].stop = &stop;
        pthread_create(&th[t], NULL, bfs_worker, &w[t]);
    }
    uint32_t level = 0, iter = 0;
    int again;
    do {
        atomic_store(&changed, 0);
        levels[n_vertices] = level;
        pthread_barrier_wait(&bar);     /* launch */
        pthread_barrier_wait(&bar);     /* done */
        iter++; level++;
        again = atomic_load(&changed);
    } while (again);
    stop = 1;
    pthread_barrier_wait(&bar);
    for (uint32_t t = 0; t < n_threads; t++) pthread_join(th[t], NULL);
    pthread_barrier_destroy(&bar);
    free(th); free(w);
    return iter;
}

static void* cc_worker(void* arg)
{
    work_t* w = arg;
    cpu_bam_ptr_t ptr = { w->p, 0, 0, 0, NULL, 0, w->tid };
    for (;;) {
        pthread_barrier_wait(w->bar);
        if (*w->stop) break;
        uint8_t* curr = *(uint8_t* volatile*)&w->curr;
        uint8_t* next_v = *(uint8_t* volatile*)&w->next;
        for (uint64_t v = w->tid; v < w->n_vertices; v += w->n_threads) {
            if (!curr[v]) continue;
            for (uint64_t i = w->offsets[v]; i < w->offsets[v + 1]; i++) {
                uint64_t next = ptr_read(&ptr, i);
                uint64_t cs = __atomic_load_n(&w->comp[v], __ATOMIC_RELAXED), cn = __atomic_load_n(&w->comp[next], __ATOMIC_RELAXED);
                if (cs == cn) continue;
                uint64_t tgt = cs < cn ? next : v, val = cs < cn ? cs : cn;
                uint64_t cur = __atomic_load_n(&w->comp[tgt], __ATOMIC_RELAXED);       /* atomicMin */
                while (val < cur && !__atomic_compare_exchange_n(&w->comp[tgt], &cur, val, 1, __ATOMIC_RELAXED, __ATOMIC_RELAXED)) {}
                __atomic_store_n(&next_v[tgt], 1, __ATOMIC_RELAXED);
                atomic_store(w->changed, 1);
            }
        }
        ptr_fini(&ptr);
        pthread_barrier_wait(w->bar);
    }
    return NULL;
}

/* min-label propagation, edges through the cache; returns iterations */
uint32_t bo_cpu_cc(bo_cpu_path_t* p, uint32_t n_threads, const uint64_t* offsets, uint64_t n_vertices, uint64_t* comp)
{
    pthread_barrier_t bar;
    _Atomic int changed = 0;
    int stop = 0;
    uint8_t* a = malloc(n_vertices), *b = calloc(n_vertices, 1);
    memset(a, 1, n_vertices);
    for (uint64_t v = 0; v < n_vertices; v++) comp[v] = v;
    pthread_barrier_init(&bar, NULL, n_threads + 1);
    pthread_t* th = calloc(n_threads, sizeof(*th));
    work_t* w = calloc(n_threads, sizeof(*w));
    for (uint32_t t = 0; t < n_threads; t++) {
        w[t].p = p; w[t].tid = t; w[t].n_threads = n_threads; w[t].offsets = offsets; w[t].n_vertices = n_vertices;
        w[t].comp = comp; w[t].curr = a; w[t].next = b; w[t].changed = &changed; w[t].bar = &bar; w[t].stop = &stop;
        pthread_create(&th[t], NULL, cc_worker, &w[t]);
    }
    uint32_t iter = 0;
    int again;
    do {
        atomic_store(&changed, 0);
        pthread_barrier_wait(&bar);
        pthread_barrier_wait(&bar);
        memset(a, 0, n_vertices);
        uint8_t* t = a; a = b; b = t;
        for (uint32_t k = 0; k < n_threads; k++) { w[k].curr = a; w[k].next = b; }
        iter++;
        again = atomic_load(&changed);
    } while (again);
    stop = 1;
    pthread_barrier_wait(&bar);
    for (uint32_t t = 0; t < n_threads; t++) pthread_join(th[t], NULL);
    pthread_barrier_destroy(&bar);
    free(th); free(w); free(a); free(b);
    return iter;
}
