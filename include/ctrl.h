/*
 * Controller: brings an NVMe controller up and creates its I/O queue pairs.
 * Replaces include/ctrl.h of the reference (struct :39-78, initializeController
 * :94-123, constructor :148-199, reserveQueues :223-242, print_reset_stats
 * :86-92).  Kernels take Controller** and read n_qps, d_qps, queue_counter,
 * access_counter, blk_size(_log) exactly as there.
 *
 * `path` names a software NVMe target published with nvmt_publish(); the
 * reference opens /dev/libnvmN of its kernel module at this point.
 */
#ifndef __BAM_CTRL_H__
#define __BAM_CTRL_H__
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <iostream>
#include <stdexcept>
#include <string>
#include <simt/atomic>
#include "buffer.h"
#include "nvm_admin.h"
#include "nvm_aq.h"
#include "nvm_ctrl.h"
#include "nvm_error.h"
#include "nvm_types.h"
#include "nvmt.h"
#include "queue.h"

#define MAX_QUEUES 1024

using error = std::runtime_error;
using std::string;

struct Controller
{
    simt::atomic<uint64_t, simt::thread_scope_device> access_counter;
    nvm_ctrl_t*             ctrl;
    nvm_aq_ref              aq_ref;
    struct nvm_ctrl_info    info;
    struct nvm_ns_info      ns;
    uint16_t                n_sqs;
    uint16_t                n_cqs;
    uint16_t                n_qps;
    uint32_t                deviceId;
    QueuePair**             h_qps;
    QueuePair*              d_qps;
    simt::atomic<uint64_t, simt::thread_scope_device> queue_counter;
    uint32_t                page_size;
    uint32_t                blk_size;
    uint32_t                blk_size_log;
    bam_guard_t*            guard;          /* host-pinned; shared by every queue of this controller */
    bam_dma_place           cq_place;       /* completion rings in host-pinned or in device memory */
    int                     sq_seal;        /* submission entries sealed (nvm_cmd_seal) */
    uint32_t                sq_flush;       /* unsealed queues: nvm_queue_t::flush */
    uint32_t                pull_limit;     /* waves per compute-unit cluster that pull staged payload at a time (0 = no limit) */
    void*                   d_ctrl_ptr;

    unsigned long long*     prof;           /* [32] phase timers of the miss path in device memory (100 MHz ticks; builds with BAM_PROFILE fill them) */

    struct Owners { DmaPtr aq_mem; BufferPtr d_ctrl_buff, guard_buff, prof_buff, pull_buff; };
    Owners*                 own;

    Controller(const char* path, uint32_t nvmNamespace, uint32_t hipDevice, uint64_t queueDepth, uint64_t numQueues,
               uint32_t stage_bytes = 4096, uint32_t spin_limit = 10000000)
        : ctrl(nullptr), aq_ref(nullptr), deviceId(hipDevice)
    {
        nvmt_t* target = nvmt_lookup(path);
        if (!target) throw error(string("Failed to open descriptor: no software NVMe target published as ") + (path ? path : "(null)"));
        bringup(nvmt_bar(target), nvmt_bar_size(nvmt_config(target)), nvmNamespace, queueDepth, numQueues, stage_bytes, spin_limit);
    }

    /* register window supplied directly (a target the caller owns, or a mapped BAR0) */
    Controller(volatile void* mm_ptr, size_t mm_size, uint32_t nvmNamespace, uint32_t hipDevice, uint64_t queueDepth, uint64_t numQueues,
               uint32_t stage_bytes = 4096, uint32_t spin_limit = 10000000)
        : ctrl(nullptr), aq_ref(nullptr), deviceId(hipDevice)
    {
        bringup(mm_ptr, mm_size, nvmNamespace, queueDepth, numQueues, stage_bytes, spin_limit);
    }

    Controller(const Controller&) = delete;
    Controller& operator=(const Controller&) = delete;

    void reserveQueues() { reserveQueues(n_sqs, n_cqs); }
    void reserveQueues(uint16_t numSubmissionQueues) { reserveQueues(numSubmissionQueues, n_cqs); }
    void reserveQueues(uint16_t numSubs, uint16_t numCpls)
    {
        int status = nvm_admin_request_num_queues(aq_ref, &numCpls, &numSubs);
        if (!nvm_ok(status)) throw error(string("Failed to reserve queues: ") + nvm_strerror(status));
        n_sqs = numSubs;
        n_cqs = numCpls;
    }

    /* number of read commands issued through the page cache since the last call */
    uint64_t reset_stats()
    {
        uint64_t v = 0;
        hip_err_chk(hipMemcpy(&v, d_ctrl_ptr, sizeof(uint64_t), hipMemcpyDeviceToHost));
        hip_err_chk(hipMemset(d_ctrl_ptr, 0, sizeof(uint64_t)));
        return v;
    }

    void print_reset_stats(void)
    {
        uint64_t v = reset_stats();
        std::cout << "------------------------------------" << std::endl;
        std::cout << std::dec << "#SSDAccesses:\t" << v << std::endl;
    }

    /* completions that carried an error status, summed over the queues */
    uint64_t completion_errors() const
    {
        uint64_t total = 0;
        for (size_t i = 0; i < n_qps; i++) {
            uint32_t e = 0;
            hip_err_chk(hipMemcpy(&e, &d_qps[i].cq.n_errors, sizeof(e), hipMemcpyDeviceToHost));
            total += e;
        }
        return total;
    }

    bool aborted() const { return __atomic_load_n(&guard->abort, __ATOMIC_ACQUIRE) != 0; }
    void clear_abort() { __atomic_store_n(&guard->abort, 0u, __ATOMIC_RELEASE); }

    ~Controller()
    {
        for (size_t i = 0; h_qps && i < n_qps; i++) delete h_qps[i];
        free(h_qps);
        if (d_qps) (void)hipFree(d_qps);
        nvm_aq_destroy(aq_ref);
        nvm_ctrl_free(ctrl);
        delete own;
    }

private:
    void bringup(volatile void* mm_ptr, size_t mm_size, uint32_t ns_id, uint64_t queueDepth, uint64_t numQueues, uint32_t stage_bytes, uint32_t spin_limit)
    {
        own = new Owners();
        h_qps = nullptr; d_qps = nullptr; n_qps = 0; d_ctrl_ptr = nullptr;
        access_counter = 0; queue_counter = 0;
        hip_err_chk(hipSetDevice(deviceId));
        int status = nvm_raw_ctrl_init(&ctrl, mm_ptr, mm_size);
        if (!nvm_ok(status)) throw error(string("Failed to get controller reference: ") + nvm_strerror(status));

        own->aq_mem = createDma(ctrl, ctrl->page_size * 3);
        status = nvm_aq_create(&aq_ref, ctrl, own->aq_mem.get());
        if (!nvm_ok(status)) throw error(string("Failed to reset controller: ") + nvm_strerror(status));
        status = nvm_admin_ctrl_info(aq_ref, &info, NVM_DMA_OFFSET(own->aq_mem, 2), own->aq_mem->ioaddrs[0] + 2 * ctrl->page_size);
        if (!nvm_ok(status)) throw error(nvm_strerror(status));
        status = nvm_admin_ns_info(aq_ref, &ns, ns_id, NVM_DMA_OFFSET(own->aq_mem, 2), own->aq_mem->ioaddrs[0] + 2 * ctrl->page_size);
        if (!nvm_ok(status)) throw error(nvm_strerror(status));
        status = nvm_admin_get_num_queues(aq_ref, &n_cqs, &n_sqs);
        if (!nvm_ok(status)) throw error(nvm_strerror(status));

        page_size = ctrl->page_size;
        blk_size = ns.lba_data_size;
        blk_size_log = (uint32_t)__builtin_ctz(blk_size);
        reserveQueues(MAX_QUEUES, MAX_QUEUES);
        n_qps = std::min(n_sqs, n_cqs);
        n_qps = std::min(n_qps, (uint16_t)numQueues);

        own->guard_buff = createHostBuffer(sizeof(bam_guard_t));
        guard = (bam_guard_t*)own->guard_buff.get();
        guard->abort = 0;
        guard->spin_limit = spin_limit;

        own->prof_buff = createBuffer(32 * sizeof(unsigned long long), deviceId);
        prof = (unsigned long long*)own->prof_buff.get();
        h_qps = (QueuePair**)calloc(n_qps, sizeof(QueuePair*));
        hip_err_chk(hipMalloc((void**)&d_qps, sizeof(QueuePair) * n_qps));
        /* runtime policy of the queue pairs: where the completion rings live, whether submission entries are sealed, and
         * what an unsealed queue does to know its entries have arrived (see QueuePair and nvm_parallel_queue.h) */
        cq_place = BAM_DMA_DEVICE; sq_seal = 0; sq_flush = 2;
        if (const char* e = getenv("BAM_CQ_PLACE")) cq_place = (e[0] == 'd' || e[0] == '1') ? BAM_DMA_DEVICE : BAM_DMA_HOST;
        if (const char* e = getenv("BAM_SQ_SEAL")) sq_seal = atoi(e) != 0;
        if (const char* e = getenv("BAM_SQ_FLUSH")) sq_flush = (uint32_t)atoi(e);
        /* an unsealed queue's controller goes by the doorbell alone, so the submitter has to know that its entry arrived
         * before a doorbell can cover it: 0 (the wave's store counter only: handed on, not arrived) is for sealed queues,
         * whose controller checks each entry; asked for on an unsealed queue it becomes the read-back */
        if (!sq_seal && sq_flush == 0) sq_flush = 2;
        /* staged payload is pulled from host memory by the waves themselves, and a compute unit returns the loads of
         * all its waves in order: while one wave waits for host memory, every other load of that unit waits with it.
         * With more pulls in flight than the interconnect needs to stay busy, each waits longer and so does everybody
         * else; the number of waves pulling at a time is therefore bounded (per cluster of compute units). */
        pull_limit = 0;
        if (const char* e = getenv("BAM_PULL_LIMIT")) pull_limit = (uint32_t)atoi(e);
        own->pull_buff = createBuffer(8 * 64, deviceId);
        for (size_t i = 0; i < n_qps; i++) {
            h_qps[i] = new QueuePair(ctrl, deviceId, ns, info, aq_ref, (uint16_t)(i + 1), queueDepth, guard, stage_bytes, BAM_DMA_HOST, cq_place, sq_seal, sq_flush, prof,
                                     (uint32_t*)own->pull_buff.get(), pull_limit);
            h_qps[i]->bind_device(d_qps + i);
            hip_err_chk(hipMemcpy((void*)(d_qps + i), (const void*)h_qps[i], sizeof(QueuePair), hipMemcpyHostToDevice));
        }
        own->d_ctrl_buff = createBuffer(sizeof(Controller), deviceId);
        d_ctrl_ptr = own->d_ctrl_buff.get();
        hip_err_chk(hipMemcpy(d_ctrl_ptr, (const void*)this, sizeof(Controller), hipMemcpyHostToDevice));
    }
};
#endif
