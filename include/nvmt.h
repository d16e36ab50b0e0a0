/*
 * Software NVMe target: a controller model served by host threads.
 *
 * It exposes a register window (CAP/CC/CSTS/AQA/ASQ/ACQ + doorbells, the BAR0
 * layout of src/regs.h:9-47 of the reference) in memory supplied by the caller,
 * runs the admin command set that the reference's Controller/QueuePair bring-up
 * issues (include/ctrl.h:94-123,179, include/queue.h:181-203, src/admin.cpp:20-64)
 * and serves READ/WRITE/FLUSH on I/O queues with the exact SQ/CQ protocol a
 * device would: SQEs are fetched from queue memory after a tail-doorbell
 * write, completions carry CID, phase tag and SQHD, the CQ-full rule is
 * honoured through the CQ head doorbell.  It has no counterpart in the
 * reference, which only runs against real SSDs; it stands where the SSD does.
 *
 * A bus address is a host virtual address the service threads can dereference.
 * The namespace is either memory-backed or procedural: 64-bit word w of the
 * namespace reads as splitmix64(seed, w), so a 64 GiB namespace costs no RAM.
 */
#ifndef __NVMT_H__
#define __NVMT_H__
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

typedef struct nvmt nvmt_t;

enum nvmt_order { NVMT_ORDER_FIFO = 0, NVMT_ORDER_REVERSE = 1, NVMT_ORDER_SHUFFLE = 2 };

typedef struct
{
    uint64_t ns_bytes;          /* namespace size in bytes */
    uint32_t lba_bytes;         /* 512 or 4096 */
    void*    backing;           /* memory-backed namespace (ns_bytes long), or NULL for procedural */
    uint64_t seed;              /* procedural content seed */
    uint32_t n_io_threads;      /* service threads for I/O queues (>= 1) */
    uint32_t max_queue_entries; /* MQES + 1, power of two, <= 65536 */
    uint32_t max_io_queues;     /* queue pairs the controller grants (<= 1023) */
    uint32_t dstrd;             /* doorbell stride exponent: stride = 4 << dstrd bytes */
    uint32_t order;             /* completion order within a fetched batch (enum nvmt_order) */
    uint32_t fail_every;        /* > 0: every n-th I/O command completes with status Data Transfer Error */
    uint32_t drop_every;        /* > 0: every n-th I/O command is never completed (lost-completion test) */
    uint32_t never_ready;       /* != 0: CSTS.RDY never follows CC.EN (controller-timeout test) */
    uint32_t timeout_500ms;     /* CAP.TO in 500 ms units (0 -> 2) */
} nvmt_config_t;

typedef struct
{
    uint64_t admin_cmds;
    uint64_t io_cmds;
    uint64_t read_cmds;
    uint64_t write_cmds;
    uint64_t bytes_read;
    uint64_t bytes_written;
    uint64_t error_cpls;        /* completions posted with a non-zero status */
    uint64_t sq_doorbells;      /* distinct tail values observed */
    uint64_t cq_full_stalls;    /* times a completion had to wait for CQ space */
    uint64_t dropped;           /* commands swallowed by drop_every */
    uint64_t sqe_retries;       /* sealed SQ: entries found stale or incomplete when first looked at */
    uint64_t stale_doorbells;   /* doorbell values that pointed behind what had already been seen */
} nvmt_stats_t;

/* bytes of register window needed for this configuration (>= 0x2000) */
size_t   nvmt_bar_size(const nvmt_config_t* cfg);
/* bar_mem: zeroed memory of nvmt_bar_size() bytes, 4 KiB aligned, readable and
 * writable by both the service threads and whoever rings doorbells */
nvmt_t*  nvmt_create(const nvmt_config_t* cfg, void* bar_mem);
void     nvmt_destroy(nvmt_t* t);
volatile void* nvmt_bar(nvmt_t* t);
void     nvmt_stats(nvmt_t* t, nvmt_stats_t* out);
void     nvmt_reset_stats(nvmt_t* t);
/*
 * Name registry, so that code written against the reference's
 * Controller(const char* path, ...) constructor (include/ctrl.h:148) can name a
 * target the way it names /dev/libnvm0.  publish returns 0 or EEXIST/EINVAL;
 * lookup returns NULL for unknown names; destroy unpublishes.
 */
int      nvmt_publish(const char* path, nvmt_t* t);
nvmt_t*  nvmt_lookup(const char* path);
const nvmt_config_t* nvmt_config(nvmt_t* t);
/* where the target stands on I/O queue pair `qid` (read without stopping the service threads: for diagnosis after a
 * run that was given up).  out8: SQ head, commands fetched so far, SQ tail doorbell, sealed, CQ tail, CQ head as last
 * seen, CQ head doorbell, CQ phase.  0, EINVAL or ENOENT (no such queue). */
int      nvmt_queue_state(nvmt_t* t, uint16_t qid, uint64_t* out8);
/* procedural content: fills out[0..n) with words first_word.. of a namespace with this seed */
void     nvmt_fill_words(uint64_t seed, uint64_t first_word, uint64_t n, uint64_t* out);
/*
 * Protocol ceiling: drive queue pair(s) already created on this target from
 * `n_clients` plain host threads (no page cache, no GPU), each issuing
 * `n_cmds` reads of `req_bytes` at pseudo-random LBAs into `dst` buffers it
 * owns, keeping up to `depth` in flight.  Returns commands per second.
 */
double   nvmt_selftest_iops(const nvmt_config_t* cfg, uint32_t n_clients, uint32_t depth, uint64_t n_cmds, uint32_t req_bytes);

#ifdef __cplusplus
}
#endif
#endif
