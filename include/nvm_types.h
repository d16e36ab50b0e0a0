/*
 * Handle and wire types of the NVMe layer (C, shared by host code, the
 * software NVMe target and the gfx950 device code).
 *
 * Replaces include/nvm_types.h of the reference (nvm_ctrl_t :24-32, nvm_dma_t
 * :70-78, nvm_queue_t :123-165, nvm_cpl_t :185-188, nvm_cmd_t :196-199,
 * nvm_ctrl_info :209-227, nvm_ns_info :236-244).  Field names are kept; the
 * device-side words are plain uint32_t that device code updates with
 * __hip_atomic_* at an explicit scope instead of simt::atomic members, and
 * the per-slot arrays are dense uint32_t (no 32-byte padding).
 */
#ifndef __NVM_TYPES_H__
#define __NVM_TYPES_H__
#include <stddef.h>
#include <stdint.h>

#ifndef __HIPCC__
#ifndef __host__
#define __host__
#endif
#ifndef __device__
#define __device__
#endif
#endif

/* NVM controller handle: allocated and released by the API. */
typedef struct
{
    size_t                  page_size;      /* Memory page size used by the controller (MPS) */
    uint8_t                 dstrd;          /* Doorbell stride (encoded) */
    uint64_t                timeout;        /* Controller timeout in milliseconds (TO) */
    uint32_t                max_qs;         /* Maximum queue entries supported (MQES + 1) */
    size_t                  mm_size;        /* Size of the register window */
    volatile void*          mm_ptr;         /* Register window (BAR0 of a device, or the software target's) */
} nvm_ctrl_t;

struct nvm_admin_reference;
typedef struct nvm_admin_reference* nvm_aq_ref;

/* DMA mapping descriptor: allocated and released by the API. */
typedef struct
{
    void*                   vaddr;          /* Virtual address of the region (may be NULL) */
    int8_t                  local;
    int8_t                  contiguous;
    size_t                  page_size;      /* Controller page size (MPS) */
    size_t                  n_ioaddrs;      /* Number of MPS-sized pages */
    uint64_t                ioaddrs[];      /* Bus address of every page */
} nvm_dma_t;

/*
 * Bounded waits of the device path.  Every spin loop gives up once it has
 * waited spin_limit microseconds (0 = never) or as soon as `abort` is
 * non-zero, and sets `abort` when it does, so that a lost completion ends the
 * kernel instead of hanging the GPU.  Lives in host-pinned memory; the host reads it after the
 * kernel to tell whether results are valid.
 */
typedef struct bam_guard
{
    uint32_t abort;
    uint32_t spin_limit;
} bam_guard_t;

/* One word of per-slot queue state. */
typedef struct { uint32_t val; } padded_struct;

/*
 * Queue descriptor, used for both SQs and CQs.  The six hot words sit on
 * separate 64-byte lines: they are hit by device-scope atomics from every
 * wave that uses the queue.
 */
typedef struct
{
    uint32_t head_lock;  uint8_t pad0[60];  /* CQ: bit 0 = held by the wave draining completions, bits 31:1 = head (free running) */
    uint32_t tail_lock;  uint8_t pad1[60];  /* SQ: bit 0 = held by the wave sweeping tail marks, bits 31:1 = tail (free running) */
    uint32_t head;       uint8_t pad2[60];  /* free-running */
    uint32_t tail;       uint8_t pad3[60];  /* free-running */
    uint32_t in_ticket;  uint8_t pad4[60];  /* SQ: next slot ticket */
    uint32_t cid_ticket;                    /* SQ: next command-id probe */
    uint32_t n_errors;   uint8_t pad5[56];  /* CQ: completions seen with a non-zero status */

    padded_struct*          tickets;        /* SQ [qs]: 2 * lap = free for the ticket of that lap (its owner adds 2 when done with the command) */
    padded_struct*          head_mark;      /* SQ [qs]: a spare word per slot (the reference marks consumed CQ entries in an array of this name) */
    padded_struct*          tail_mark;      /* SQ [qs]: lap + 1 of the entry last written to the slot, read by the tail sweep */
    padded_struct*          cid;            /* SQ [qs]: per command id (= slot), 1 in flight, 3 in flight + completed, 7 completed with an error status */
    padded_struct*          pos_locks;      /* unused (the reference's per-slot CQ locks) */
    uint32_t                cid_mask;       /* qs - 1 */
    uint32_t                sealed;         /* SQ: entries carry a sequence number and checksum (nvm_cmd_seal) */
    uint32_t                flush;          /* SQ, unsealed: how a written entry is known to have reached the ring before its mark is set
                                               (0 nothing beyond the wave's own store counters, 1 system-scope release, 2 read the entry back) */
    uint32_t                idle_ticks;     /* CQ: 100 MHz ticks an empty ring is left alone after a look (0: ring in device memory, a look costs nothing) */
    unsigned long long*     prof;           /* device path: [32] phase timers, filled only by builds with BAM_PROFILE (may be NULL) */
    struct bam_guard*       guard;          /* device path: bounded-wait control (may be NULL) */
    uint32_t                spin_limit;     /* device path: copy of guard->spin_limit */
    void*                   pair;           /* device path: the CQ of an SQ / the SQ of a CQ (device address) */
    uint32_t                qs_minus_1;
    uint32_t                qs_log2;
    uint16_t                no;             /* Queue number (unique per SQ/CQ pair) */
    uint16_t                es;             /* Entry size */
    uint32_t                qs;             /* Number of entries */
    int8_t                  phase;          /* Host-side single-thread ops: current phase tag */
    int8_t                  local;
    uint32_t                last;           /* Host-side single-thread ops: last doorbell value */
    volatile uint32_t*      db;             /* Doorbell register (write only) */
    volatile void*          vaddr;          /* Queue memory */
    uint64_t                ioaddr;         /* Bus address of queue memory */
} nvm_queue_t;

/*
 * Is SQ slot `ticket & (qs - 1)` free for the submitter holding `ticket`?  tickets[slot] counts 2 per lap (the
 * drainer adds 2 when the controller has consumed the slot's entry), the lap of a ticket is ticket >> qs_log2.
 * The 32-bit ticket counter wraps after 2^(32 - qs_log2) laps while the slot word keeps counting to twice that,
 * so the two are compared modulo the lap range.
 */
__host__ __device__ static inline
int nvm_sq_slot_free(uint32_t slot_word, uint32_t ticket, uint32_t qs_log2)
{
    const uint32_t want = (ticket >> qs_log2) * 2u;
    const uint32_t lap_mask = (uint32_t)((2ull << (32u - qs_log2)) - 1ull);
    return ((slot_word - want) & lap_mask) == 0;
}

typedef struct __attribute__((aligned(32)))
{
    volatile void*          vaddr;
    int16_t                 local;
    size_t                  page_size;
    uint64_t                ioaddr;
} nvm_prp_list_t;

/* Completion queue entry (16 bytes) */
typedef struct __attribute__((aligned(16)))
{
    volatile uint32_t       dword[4];
} nvm_cpl_t;

/* Submission queue entry (64 bytes) */
typedef struct __attribute__((aligned(64)))
{
    uint32_t                dword[16];
} nvm_cmd_t;

struct nvm_ctrl_info
{
    uint32_t                nvme_version;
    size_t                  page_size;
    size_t                  db_stride;
    uint64_t                timeout;
    int                     contiguous;
    uint16_t                max_entries;
    uint8_t                 pci_vendor[4];
    char                    serial_no[20];
    char                    model_no[40];
    char                    firmware[8];
    size_t                  max_data_size;
    size_t                  max_data_pages;
    size_t                  cq_entry_size;
    size_t                  sq_entry_size;
    size_t                  max_out_cmds;
    size_t                  max_n_ns;
};

struct nvm_ns_info
{
    uint32_t                ns_id;
    size_t                  size;           /* NSZE, logical blocks */
    size_t                  capacity;       /* NCAP */
    size_t                  utilization;    /* NUSE */
    size_t                  lba_data_size;  /* bytes per logical block */
    size_t                  metadata_size;
};

#endif /* __NVM_TYPES_H__ */
