// Protocol-ceiling measurement for the software NVMe target: plain host
// threads drive queue pairs through the public NVMe host API with no page
// cache and no GPU in the way.  Each client owns one queue pair and keeps up
// to `depth` reads in flight, so the figure is what the target's service
// threads can sustain for this request size.
#include "nvmt.h"
#include "nvm_admin.h"
#include "nvm_aq.h"
#include "nvm_cmd.h"
#include "nvm_ctrl.h"
#include "nvm_dma.h"
#include "nvm_queue.h"

#include <atomic>
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <thread>
#include <vector>

namespace {

struct Client {
    nvm_queue_t sq, cq;
    nvm_dma_t *sq_mem = nullptr, *cq_mem = nullptr;
    uint8_t* dst = nullptr;
    uint64_t done = 0, bad = 0;
};

inline uint64_t mix64(uint64_t z)
{
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

void run_client(Client* c, uint32_t id, const nvmt_config_t* cfg, uint32_t depth, uint64_t n_cmds, uint32_t req_bytes)
{
    const uint64_t units = cfg->ns_bytes / req_bytes;
    const uint32_t blocks = req_bytes / cfg->lba_bytes;
    uint64_t issued = 0, rng = mix64(id + 1);
    uint32_t inflight = 0;
    while (c->done < n_cmds) {
        bool rang = false;
        while (inflight < depth && issued < n_cmds) {
            nvm_cmd_t* e = nvm_sq_enqueue(&c->sq);
            if (!e) break;
            rng = mix64(rng + 0x9E3779B97F4A7C15ull);
            uint32_t slot = (uint32_t)(issued % depth);
            nvm_cmd_t cmd;
            memset(&cmd, 0, sizeof(cmd));
            nvm_cmd_header(&cmd, (uint16_t)slot, NVM_IO_READ, 1);
            nvm_cmd_data_ptr(&cmd, (uint64_t)(uintptr_t)(c->dst + (size_t)slot * req_bytes), 0);
            nvm_cmd_rw_blks(&cmd, (rng % units) * blocks, (uint16_t)blocks);
            *e = cmd;
            issued++; inflight++; rang = true;
        }
        if (rang) nvm_sq_submit(&c->sq);
        nvm_cpl_t* cpl;
        bool got = false;
        while ((cpl = nvm_cq_dequeue(&c->cq)) != nullptr) {
            if (cpl->dword[3] >> 17) c->bad++;
            nvm_sq_update(&c->sq);
            c->done++; inflight--; got = true;
        }
        if (got) nvm_cq_update(&c->cq);
    }
}

} // namespace

extern "C" double nvmt_selftest_iops(const nvmt_config_t* cfg, uint32_t n_clients, uint32_t depth, uint64_t n_cmds, uint32_t req_bytes)
{
    if (!cfg || !n_clients || !depth || !n_cmds || req_bytes % cfg->lba_bytes || req_bytes > 4096 || n_clients > cfg->max_io_queues) return -1.0;
    uint32_t qs = 2;
    while (qs < depth + 1) qs <<= 1;
    if (qs > cfg->max_queue_entries) return -1.0;

    void* bar = nullptr;
    if (posix_memalign(&bar, 4096, nvmt_bar_size(cfg))) return -1.0;
    memset(bar, 0, nvmt_bar_size(cfg));
    nvmt_t* t = nvmt_create(cfg, bar);
    if (!t) { free(bar); return -1.0; }

    double result = -1.0;
    nvm_ctrl_t* ctrl = nullptr;
    nvm_dma_t* aq_mem = nullptr;
    nvm_aq_ref aq = nullptr;
    std::vector<Client> clients(n_clients);
    uint16_t ncq = (uint16_t)n_clients, nsq = (uint16_t)n_clients;
    bool ok = nvm_raw_ctrl_init(&ctrl, nvmt_bar(t), nvmt_bar_size(cfg)) == 0 &&
              nvm_dma_create(&aq_mem, ctrl, 3 * ctrl->page_size) == 0 &&
              nvm_aq_create(&aq, ctrl, aq_mem) == 0 &&
              nvm_admin_request_num_queues(aq, &ncq, &nsq) == 0 && ncq >= n_clients && nsq >= n_clients;
    for (uint32_t i = 0; ok && i < n_clients; i++) {
        Client& c = clients[i];
        ok = nvm_dma_create(&c.cq_mem, ctrl, qs * sizeof(nvm_cpl_t)) == 0 &&
             nvm_dma_create(&c.sq_mem, ctrl, qs * sizeof(nvm_cmd_t)) == 0 &&
             nvm_admin_cq_create(aq, &c.cq, (uint16_t)(i + 1), c.cq_mem, 0, qs) == 0 &&
             nvm_admin_sq_create(aq, &c.sq, &c.cq, (uint16_t)(i + 1), c.sq_mem, 0, qs) == 0 &&
             posix_memalign((void**)&c.dst, 4096, (size_t)depth * 4096) == 0;
    }
    if (ok) {
        std::vector<std::thread> th;
        auto t0 = std::chrono::steady_clock::now();
        for (uint32_t i = 0; i < n_clients; i++) th.emplace_back(run_client, &clients[i], i, cfg, depth, n_cmds, req_bytes);
        for (auto& x : th) x.join();
        double s = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
        uint64_t bad = 0;
        for (auto& c : clients) bad += c.bad;
        result = bad ? -2.0 : (double)n_cmds * n_clients / s;
    }
    for (auto& c : clients) {
        if (c.sq.db && aq) nvm_admin_sq_delete(aq, &c.sq, &c.cq);
        if (c.cq.db && aq) nvm_admin_cq_delete(aq, &c.cq);
        nvm_dma_unmap(c.sq_mem); nvm_dma_unmap(c.cq_mem); free(c.dst);
    }
    nvm_aq_destroy(aq);
    nvm_dma_unmap(aq_mem);
    nvm_ctrl_free(ctrl);
    nvmt_destroy(t);
    free(bar);
    return result;
}
