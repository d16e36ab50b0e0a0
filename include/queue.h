/*
 * I/O queue pair as the device sees it, plus the host code that creates it.
 * Replaces include/queue.h of the reference (QueuePair :27-49, queue sizing
 * :95-107, init_gpu_specific_struct :58-85, admin creation :181-203).
 *
 * Differences that follow from the wave-cooperative engine: per-slot state is
 * dense 32-bit words, the command-id table has as many entries as the queue
 * (ids index a staging window, see below) instead of 65536 and is handed out
 * to waves in blocks of 64 ids, and the head_mark array is gone.
 *
 * Staged transfers.  When the controller cannot address device memory (the
 * software target on a machine without CPU-visible VRAM) every queue pair owns
 * a window of controller-visible staging pages, one per command id; commands
 * carry the staging page as PRP1 and the submitting lanes move the payload
 * between staging and device memory themselves.
 */
#ifndef __BAM_QUEUE_H__
#define __BAM_QUEUE_H__
#include <algorithm>
#include <cstdint>
#include <stdexcept>
#include <string>
#include "buffer.h"
#include "nvm_admin.h"
#include "nvm_aq.h"
#include "nvm_error.h"
#include "nvm_types.h"
#include "util.h"

#define BAM_CQ_IDLE_TICKS_DEFAULT 200u       /* 2 us at 100 MHz: an empty completion ring in host memory is left alone that long after a look */

struct QueuePair
{
    uint32_t            pageSize;
    uint32_t            block_size;
    uint32_t            block_size_log;
    uint32_t            block_size_minus_1;
    uint32_t            nvmNamespace;
    nvm_queue_t         sq;
    nvm_queue_t         cq;
    uint16_t            qp_id;
    uint8_t*            stage;          /* staging window (NULL: PRPs address device memory directly) */
    uint64_t            stage_ioaddr;
    uint32_t            stage_stride;   /* bytes per command id */
    uint32_t*           pull_tokens;    /* [8 x 16] waves pulling staged payload from host memory right now, one word per compute-unit cluster, 64 bytes apart */
    uint32_t            pull_limit;     /* at most this many per cluster at a time (0 = no limit) */
    uint64_t*           async_dst;      /* [n_cids] staged asynchronous reads: destination address, 0 = none */
    uint32_t*           async_len;      /* [n_cids] and length in bytes */

    /* host-side owners; a raw pointer keeps the struct trivially copyable to the device */
    struct Owners {
        DmaPtr sq_mem, cq_mem, stage_mem;
        BufferPtr sq_tickets, sq_tail_mark, sq_cid, sq_cid_blocks, sq_cid_left, async_dst, async_len;
    };
    Owners*             own;
    nvm_aq_ref          aq;

    QueuePair(const nvm_ctrl_t* ctrl, const uint32_t hipDevice, const struct nvm_ns_info ns, const struct nvm_ctrl_info info,
              nvm_aq_ref& aq_ref, const uint16_t qp_id, const uint64_t queueDepth,
              bam_guard_t* guard = nullptr, uint32_t stage_bytes = 4096, bam_dma_place ring_place = BAM_DMA_HOST,
              bam_dma_place cq_place = BAM_DMA_HOST, int seal = 1, uint32_t flush = 2, unsigned long long* prof = nullptr,
              uint32_t* pull_tokens_ = nullptr, uint32_t pull_limit_ = 0)
    {
        own = new Owners();
        aq = aq_ref;
        /* depth: what was asked for, capped by MQES + 1 and rounded down to a power of two */
        uint64_t depth = std::min<uint64_t>(queueDepth, (uint64_t)info.max_entries + 1);
        uint32_t qs = 2;
        while ((uint64_t)qs * 2 <= depth) qs *= 2;

        own->sq_mem = createDma(ctrl, NVM_PAGE_ALIGN(qs * sizeof(nvm_cmd_t), 1UL << 16), hipDevice, ring_place);
        /* the completion ring may sit in device memory: the controller then posts completions across the interconnect
         * (16-byte writes behind the payload) and the waves look for them in local memory, which costs them nothing
         * and keeps those looks out of the way of the payload they pull from host memory */
        own->cq_mem = createDma(ctrl, NVM_PAGE_ALIGN(qs * sizeof(nvm_cpl_t), 1UL << 16), hipDevice, cq_place);

        pageSize = info.page_size;
        block_size = ns.lba_data_size;
        block_size_minus_1 = ns.lba_data_size - 1;
        block_size_log = (uint32_t)__builtin_ctzl(ns.lba_data_size);
        nvmNamespace = ns.ns_id;
        this->qp_id = qp_id;

        int status = nvm_admin_cq_create(aq_ref, &cq, qp_id, own->cq_mem.get(), 0, qs);
        if (!nvm_ok(status)) { delete own; throw std::runtime_error(std::string("Failed to create completion queue: ") + nvm_strerror(status)); }
        status = nvm_admin_sq_create(aq_ref, &sq, &cq, qp_id, own->sq_mem.get(), 0, qs);
        if (!nvm_ok(status)) { nvm_admin_cq_delete(aq_ref, &cq); delete own; throw std::runtime_error(std::string("Failed to create submission queue: ") + nvm_strerror(status)); }

        /* the ring is filled by the GPU across the interconnect and fetched by the controller from the other side:
         * have entries sealed so that one that has not fully arrived is never taken (see nvm_cmd_seal) */
        status = seal ? nvm_admin_sq_set_sealed(aq_ref, &sq) : 0;
        /* a controller that does not know the vendor command (a real device) answers with an NVMe status: the queue
         * then runs unsealed, as the NVMe specification has it; anything else is a failed admin round trip */
        if (!nvm_ok(status) && status > 0) { nvm_admin_sq_delete(aq_ref, &sq, &cq); nvm_admin_cq_delete(aq_ref, &cq); delete own; throw std::runtime_error(std::string("Failed to seal submission queue: ") + nvm_strerror(status)); }
        /* unsealed: a submitter makes sure its entry is in the ring before the entry can be covered by a doorbell */
        sq.flush = flush;
        cq.idle_ticks = cq_place == BAM_DMA_HOST ? BAM_CQ_IDLE_TICKS_DEFAULT : 0;

        /* device-side protocol state */
        const uint32_t n_cids = qs;                     /* a command's id is the submission slot it goes to */
        own->sq_tickets = createBuffer(qs * sizeof(padded_struct), hipDevice);
        own->sq_tail_mark = createBuffer(qs * sizeof(padded_struct), hipDevice);
        own->sq_cid = createBuffer(n_cids * sizeof(padded_struct), hipDevice);
        sq.tickets = (padded_struct*)own->sq_tickets.get();
        sq.tail_mark = (padded_struct*)own->sq_tail_mark.get();
        sq.cid = (padded_struct*)own->sq_cid.get();
        sq.cid_mask = n_cids - 1;
        own->sq_cid_blocks = createBuffer(sizeof(padded_struct), hipDevice);
        sq.pos_locks = (padded_struct*)own->sq_cid_blocks.get();        /* unused */
        own->sq_cid_left = createBuffer(qs * sizeof(padded_struct), hipDevice);
        sq.head_mark = (padded_struct*)own->sq_cid_left.get();         /* a spare word per slot */
        cq.cid = sq.cid;
        cq.cid_mask = sq.cid_mask;
        sq.prof = cq.prof = prof;
        sq.guard = cq.guard = guard;
        sq.spin_limit = cq.spin_limit = guard ? guard->spin_limit : 0;

        stage = nullptr; stage_ioaddr = 0; stage_stride = 0; async_dst = nullptr; async_len = nullptr;
        pull_tokens = pull_tokens_; pull_limit = pull_tokens_ ? pull_limit_ : 0;
        if (stage_bytes > 2 * ctrl->page_size || (stage_bytes & (stage_bytes - 1)))
            throw std::runtime_error("QueuePair: the staging page must be a power of two of at most two controller pages (PRP1 + PRP2)");
        if (stage_bytes) {
            own->stage_mem = createDma(ctrl, (size_t)n_cids * stage_bytes);
            stage = (uint8_t*)own->stage_mem->vaddr;
            stage_ioaddr = own->stage_mem->ioaddrs[0];
            stage_stride = stage_bytes;
            /* where the payload of a read submitted with access_data_async goes once poll_async has seen it complete */
            own->async_dst = createBuffer(n_cids * sizeof(uint64_t), hipDevice);
            own->async_len = createBuffer(n_cids * sizeof(uint32_t), hipDevice);
            async_dst = (uint64_t*)own->async_dst.get();
            async_len = (uint32_t*)own->async_len.get();
        }
    }

    /* the device copy lives at d_self: let each queue find its partner there */
    void bind_device(QueuePair* d_self)
    {
        sq.pair = &d_self->cq;
        cq.pair = &d_self->sq;
    }

    QueuePair(const QueuePair&) = delete;
    QueuePair& operator=(const QueuePair&) = delete;

    ~QueuePair()
    {
        if (sq.db) nvm_admin_sq_delete(aq, &sq, &cq);
        if (cq.db) nvm_admin_cq_delete(aq, &cq);
        delete own;
    }
};
#endif
