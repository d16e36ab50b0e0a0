// Host-side checks of the NVMe layer and the software NVMe target (no GPU): bring-up, admin commands,
// error paths, PRP handling, completion ordering, CQ back-pressure.  Prints "ok <name>" per check; exit 0 = all passed.
#include <cerrno>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <ctime>
#include <vector>
#include <fcntl.h>
#include <unistd.h>
#include <time.h>
#include "nvm_admin.h"
#include "nvm_aq.h"
#include "nvm_cmd.h"
#include "nvm_ctrl.h"
#include "nvm_dma.h"
#include "nvm_error.h"
#include "nvm_queue.h"
#include "nvmt.h"

static int failures = 0;
#define CHECK(name, cond) do { if (cond) printf("ok %s\n", name); else { printf("FAIL %s (%s:%d)\n", name, __FILE__, __LINE__); failures++; } } while (0)

static uint64_t mix64(uint64_t z) { z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull; z = (z ^ (z >> 27)) * 0x94D049BB133111EBull; return z ^ (z >> 31); }
static uint64_t word(uint64_t seed, uint64_t w) { return mix64(seed + (w + 1) * 0x9E3779B97F4A7C15ull); }

struct Rig {
    nvmt_config_t cfg{};
    void* bar = nullptr;
    nvmt_t* t = nullptr;
    nvm_ctrl_t* ctrl = nullptr;
    nvm_dma_t* aq_mem = nullptr;
    nvm_aq_ref aq = nullptr;
    Rig(uint32_t order = 0, uint32_t fail_every = 0, void* backing = nullptr, uint64_t ns = 1ull << 30)
    {
        cfg.ns_bytes = ns; cfg.lba_bytes = 512; cfg.seed = 42; cfg.n_io_threads = 2; cfg.max_queue_entries = 1024;
        cfg.max_io_queues = 16; cfg.dstrd = 4; cfg.order = order; cfg.fail_every = fail_every; cfg.backing = backing;
        posix_memalign(&bar, 4096, nvmt_bar_size(&cfg));
        memset(bar, 0, nvmt_bar_size(&cfg));
        t = nvmt_create(&cfg, bar);
        nvm_raw_ctrl_init(&ctrl, nvmt_bar(t), nvmt_bar_size(&cfg));
        nvm_dma_create(&aq_mem, ctrl, 3 * ctrl->page_size);
        nvm_aq_create(&aq, ctrl, aq_mem);
    }
    ~Rig() { nvm_aq_destroy(aq); nvm_dma_unmap(aq_mem); nvm_ctrl_free(ctrl); nvmt_destroy(t); free(bar); }
};

struct Qp {
    nvm_queue_t sq, cq;
    nvm_dma_t *sqm = nullptr, *cqm = nullptr;
    int status = 0;
    Qp(Rig& r, uint16_t id, uint32_t qs)
    {
        nvm_dma_create(&cqm, r.ctrl, qs * sizeof(nvm_cpl_t));
        nvm_dma_create(&sqm, r.ctrl, qs * sizeof(nvm_cmd_t));
        status = nvm_admin_cq_create(r.aq, &cq, id, cqm, 0, qs);
        if (!status) status = nvm_admin_sq_create(r.aq, &sq, &cq, id, sqm, 0, qs);
    }
    void submit(uint16_t cid, uint8_t op, uint64_t prp1, uint64_t prp2, uint64_t lba, uint16_t nblk)
    {
        nvm_cmd_t* e = nvm_sq_enqueue(&sq);
        nvm_cmd_t c; memset(&c, 0, sizeof(c));
        nvm_cmd_header(&c, cid, op, 1); nvm_cmd_data_ptr(&c, prp1, prp2); nvm_cmd_rw_blks(&c, lba, nblk);
        *e = c;
    }
    nvm_cpl_t wait()
    {
        nvm_cpl_t* c = nvm_cq_dequeue_block(&cq, 2000);
        nvm_cpl_t out; memset((void*)&out, 0xff, sizeof(out));
        if (c) { for (int i = 0; i < 4; i++) out.dword[i] = c->dword[i]; nvm_sq_update(&sq); nvm_cq_update(&cq); }
        return out;
    }
};

int main()
{
    // ---- controller handle ----
    {
        nvm_ctrl_t* c = nullptr;
        alignas(4096) static uint8_t fake[0x2000];
        CHECK("ctrl_init_small_window", nvm_raw_ctrl_init(&c, fake, 0x1000) == EINVAL && !c);
        uint64_t cap = 1023ull | (1ull << 16) | (2ull << 24) | (4ull << 48) | (4ull << 52);   // MPSMIN = 64 KiB > host page
        memcpy(fake, &cap, 8);
        CHECK("ctrl_init_page_size_out_of_range", nvm_raw_ctrl_init(&c, fake, sizeof(fake)) == ERANGE);
        nvm_queue_t q;
        nvm_ctrl_t dummy{}; dummy.mm_ptr = fake;
        CHECK("queue_clear_rejects_qs_1", nvm_queue_clear(&q, &dummy, true, 1, 1, true, fake, 0) == EINVAL);
        CHECK("queue_clear_rejects_non_pow2", nvm_queue_clear(&q, &dummy, true, 1, 48, true, fake, 0) == EINVAL);
        CHECK("queue_clear_rejects_null_vaddr", nvm_queue_clear(&q, &dummy, true, 1, 16, true, nullptr, 0) == EINVAL);
    }
    // ---- controller that never becomes ready: admin queue creation times out ----
    {
        nvmt_config_t cfg{}; cfg.ns_bytes = 1 << 20; cfg.lba_bytes = 512; cfg.n_io_threads = 1; cfg.max_queue_entries = 64;
        cfg.max_io_queues = 2; cfg.never_ready = 1; cfg.timeout_500ms = 1;
        void* bar; posix_memalign(&bar, 4096, nvmt_bar_size(&cfg)); memset(bar, 0, nvmt_bar_size(&cfg));
        nvmt_t* t = nvmt_create(&cfg, bar);
        nvm_ctrl_t* c = nullptr; nvm_dma_t* m = nullptr; nvm_aq_ref aq = nullptr;
        nvm_raw_ctrl_init(&c, nvmt_bar(t), nvmt_bar_size(&cfg));
        nvm_dma_create(&m, c, 3 * c->page_size);
        CHECK("ctrl_timeout_value", c->timeout == 500);
        CHECK("aq_create_times_out", nvm_aq_create(&aq, c, m) == ETIME && !aq);
        nvm_dma_unmap(m); nvm_ctrl_free(c); nvmt_destroy(t); free(bar);
        CHECK("invalid_target_config", nvmt_create(&cfg, nullptr) == nullptr);
    }
    // ---- identify, features, queue creation errors ----
    {
        Rig r;
        CHECK("bringup", r.aq != nullptr && r.ctrl->page_size == 4096 && r.ctrl->max_qs == 1024 && r.ctrl->dstrd == 4);
        nvm_ctrl_info ci; nvm_ns_info ni;
        int s = nvm_admin_ctrl_info(r.aq, &ci, NVM_DMA_OFFSET(r.aq_mem, 2), r.aq_mem->ioaddrs[2]);
        CHECK("identify_ctrl", s == 0 && ci.sq_entry_size == 64 && ci.cq_entry_size == 16 && ci.max_entries == 1023 && ci.max_n_ns == 1 && ci.contiguous == 1 && ci.db_stride == 64);
        s = nvm_admin_ns_info(r.aq, &ni, 1, NVM_DMA_OFFSET(r.aq_mem, 2), r.aq_mem->ioaddrs[2]);
        CHECK("identify_ns", s == 0 && ni.lba_data_size == 512 && ni.size == (1ull << 30) / 512);
        s = nvm_admin_ns_info(r.aq, &ni, 7, NVM_DMA_OFFSET(r.aq_mem, 2), r.aq_mem->ioaddrs[2]);
        CHECK("identify_bad_ns_is_nvme_status", s < 0 && NVM_ERR_UNPACK_SC(s) == 0x02);
        uint16_t ncq = 1024, nsq = 1024;
        s = nvm_admin_request_num_queues(r.aq, &ncq, &nsq);
        CHECK("num_queues_granted", s == 0 && ncq == 16 && nsq == 16);
        nvm_queue_t q; nvm_dma_t* m; nvm_dma_create(&m, r.ctrl, 64 * 1024);
        CHECK("cq_create_id0_einval", nvm_admin_cq_create(r.aq, &q, 0, m, 0, 16) == EINVAL);
        s = nvm_admin_cq_create(r.aq, &q, 17, m, 0, 16);
        CHECK("cq_create_id_beyond_granted", s < 0 && NVM_ERR_UNPACK_SCT(s) == 1 && NVM_ERR_UNPACK_SC(s) == 0x01);
        s = nvm_admin_cq_create(r.aq, &q, 1, m, 0, 2048);
        CHECK("cq_create_too_deep", s < 0 && NVM_ERR_UNPACK_SCT(s) == 1 && NVM_ERR_UNPACK_SC(s) == 0x02);
        nvm_queue_t cq_fake; memset(&cq_fake, 0, sizeof(cq_fake)); cq_fake.no = 5;
        s = nvm_admin_sq_create(r.aq, &q, &cq_fake, 1, m, 0, 16);
        CHECK("sq_create_without_cq", s < 0 && NVM_ERR_UNPACK_SCT(s) == 1 && NVM_ERR_UNPACK_SC(s) == 0x00);
        Qp a(r, 1, 16);
        CHECK("qp_create", a.status == 0);
        nvm_queue_t dup;
        s = nvm_admin_cq_create(r.aq, &dup, 1, m, 0, 16);
        CHECK("cq_create_duplicate", s < 0 && NVM_ERR_UNPACK_SC(s) == 0x01);
        s = nvm_admin_cq_delete(r.aq, &a.cq);
        CHECK("cq_delete_with_live_sq_refused", s < 0);
        CHECK("sq_then_cq_delete", nvm_admin_sq_delete(r.aq, &a.sq, &a.cq) == 0 && nvm_admin_cq_delete(r.aq, &a.cq) == 0);
        CHECK("strerror_texts", !strcmp(nvm_strerror(0), "Success") && !strcmp(nvm_strerror(-0x102), "Invalid queue size") &&
                                !strcmp(nvm_strerror(-0x80), "LBA out of range") && !strcmp(nvm_strerror(ETIME), strerror(ETIME)));
        nvm_dma_unmap(m);
    }
    // ---- DMA descriptors ----
    {
        Rig r;
        uint64_t addrs[2] = {0x100000, 0x300000};
        nvm_dma_t* m = nullptr;
        int s = nvm_dma_map(&m, r.ctrl, nullptr, 8192, 2, addrs);
        CHECK("dma_map_splits_host_pages", s == 0 && m->n_ioaddrs == 4 && m->ioaddrs[1] == 0x101000 && m->ioaddrs[2] == 0x300000 && !m->contiguous);
        nvm_dma_t* m2 = nullptr;
        CHECK("dma_remap", nvm_dma_remap(&m2, m) == 0 && m2->n_ioaddrs == 4 && m2->ioaddrs[3] == 0x301000);
        CHECK("ctrl_from_dma", nvm_ctrl_from_dma(m) == r.ctrl && nvm_ctrl_from_aq_ref(r.aq) == r.ctrl);
        nvm_dma_unmap(m); nvm_dma_unmap(m2);
        uint64_t bad = 0x100800;
        CHECK("dma_map_unaligned", nvm_dma_map(&m, r.ctrl, nullptr, 4096, 1, &bad) == EINVAL);
        CHECK("dma_map_null", nvm_dma_map(&m, r.ctrl, nullptr, 4096, 0, addrs) == EINVAL);
    }
    // ---- I/O: content, PRP1 offset + PRP2, PRP list, errors ----
    {
        Rig r;
        Qp q(r, 1, 64);
        uint8_t* buf; posix_memalign((void**)&buf, 4096, 1 << 16);
        q.submit(9, NVM_IO_READ, (uint64_t)buf, 0, 24, 8); nvm_sq_submit(&q.sq);
        nvm_cpl_t c = q.wait();
        bool ok = (c.dword[3] & 0xffff) == 9 && (c.dword[3] >> 17) == 0 && (c.dword[2] >> 16) == 1 && (c.dword[2] & 0xffff) == 1;
        for (int k = 0; k < 512; k++) ok &= ((uint64_t*)buf)[k] == word(42, 24 * 64 + k);
        CHECK("read_4k_content_cid_sqid_sqhd", ok);
        // 8 KiB starting 512 bytes into a page: PRP1 covers 3584 bytes, PRP2 is a list (two more pages)
        uint64_t* list; posix_memalign((void**)&list, 4096, 4096);
        list[0] = (uint64_t)(buf + 8192); list[1] = (uint64_t)(buf + 16384);
        memset(buf, 0, 1 << 16);
        q.submit(10, NVM_IO_READ, (uint64_t)(buf + 512), (uint64_t)list, 0, 16); nvm_sq_submit(&q.sq);
        c = q.wait();
        ok = (c.dword[3] >> 17) == 0;
        for (int k = 0; k < 448; k++) ok &= ((uint64_t*)(buf + 512))[k] == word(42, k);
        for (int k = 0; k < 512; k++) ok &= ((uint64_t*)(buf + 8192))[k] == word(42, 448 + k);
        for (int k = 0; k < 64; k++) ok &= ((uint64_t*)(buf + 16384))[k] == word(42, 960 + k);
        CHECK("read_prp1_offset_and_prp_list", ok);
        // 8 KiB page aligned: PRP2 is the second page itself
        q.submit(11, NVM_IO_READ, (uint64_t)buf, (uint64_t)(buf + 20480), 8, 16); nvm_sq_submit(&q.sq);
        c = q.wait();
        ok = (c.dword[3] >> 17) == 0 && ((uint64_t*)buf)[0] == word(42, 512) && ((uint64_t*)(buf + 20480))[511] == word(42, 512 + 1023);
        CHECK("read_prp2_second_page", ok);
        q.submit(12, NVM_IO_READ, (uint64_t)buf, 0, (1ull << 30) / 512 - 4, 8); nvm_sq_submit(&q.sq);
        c = q.wait();
        CHECK("read_past_end_lba_out_of_range", (c.dword[3] >> 17) == 0x80);
        q.submit(13, NVM_IO_WRITE, (uint64_t)buf, 0, 0, 8); nvm_sq_submit(&q.sq);
        c = q.wait();
        CHECK("write_to_procedural_namespace_refused", (c.dword[3] >> 17) == 0x82);
        q.submit(14, 0x7f, (uint64_t)buf, 0, 0, 8); nvm_sq_submit(&q.sq);
        c = q.wait();
        CHECK("invalid_opcode", (c.dword[3] >> 17) == 0x01);
        q.submit(15, NVM_IO_FLUSH, 0, 0, 0, 1); nvm_sq_submit(&q.sq);
        c = q.wait();
        CHECK("flush_ok", (c.dword[3] >> 17) == 0 && (c.dword[3] & 0xffff) == 15);
        nvmt_stats_t st; nvmt_stats(r.t, &st);
        CHECK("target_stats", st.io_cmds == 7 && st.read_cmds == 3 && st.error_cpls == 3 && st.bytes_read == 4096 + 8192 + 8192);
        free(buf); free(list);
    }
    // ---- memory-backed namespace: write then read back ----
    {
        std::vector<uint64_t> store(1 << 17, 0);
        Rig r(0, 0, store.data(), store.size() * 8);
        Qp q(r, 1, 16);
        uint64_t* buf; posix_memalign((void**)&buf, 4096, 8192);
        for (int k = 0; k < 512; k++) buf[k] = 1000 + k;
        q.submit(1, NVM_IO_WRITE, (uint64_t)buf, 0, 40, 8); nvm_sq_submit(&q.sq);
        nvm_cpl_t c = q.wait();
        q.submit(2, NVM_IO_READ, (uint64_t)(buf + 512), 0, 40, 8); nvm_sq_submit(&q.sq);
        nvm_cpl_t c2 = q.wait();
        CHECK("write_read_back", (c.dword[3] >> 17) == 0 && (c2.dword[3] >> 17) == 0 && !memcmp(buf, buf + 512, 4096) && store[40 * 64 + 5] == 1005);
        free(buf);
    }
    // ---- completions out of order: matched by CID; phase tag flips per lap; SQHD advances ----
    for (uint32_t order : {1u, 2u}) {
        Rig r(order);
        Qp q(r, 1, 8);
        uint8_t* buf; posix_memalign((void**)&buf, 4096, 8 * 4096);
        bool ok = true;
        uint32_t total = 0;
        for (int lap = 0; lap < 6; lap++) {
            for (uint16_t i = 0; i < 7; i++) q.submit((uint16_t)(lap * 16 + i), NVM_IO_READ, (uint64_t)(buf + i * 4096), 0, (lap * 7 + i) * 8, 8);
            nvm_sq_submit(&q.sq);
            uint32_t seen = 0;
            for (int i = 0; i < 7; i++) {
                nvm_cpl_t c = q.wait();
                uint16_t cid = c.dword[3] & 0xffff;
                ok &= (c.dword[3] >> 17) == 0 && cid / 16 == lap && cid % 16 < 7 && !(seen & (1u << (cid % 16)));
                seen |= 1u << (cid % 16);
                ok &= ((uint64_t*)(buf + (cid % 16) * 4096))[3] == word(42, (uint64_t)(lap * 7 + cid % 16) * 512 + 3);
                total++;
            }
            ok &= seen == 0x7f && (q.sq.head & 7) == (q.sq.tail & 7);
        }
        CHECK(order == 1 ? "reverse_completion_order" : "shuffled_completion_order", ok && total == 42);
        free(buf);
    }
    // ---- injected failures surface as NVMe status and in the counters ----
    {
        Rig r(0, 3);
        Qp q(r, 1, 16);
        uint8_t* buf; posix_memalign((void**)&buf, 4096, 4096);
        int errs = 0;
        for (int i = 0; i < 9; i++) { q.submit((uint16_t)i, NVM_IO_READ, (uint64_t)buf, 0, 0, 8); nvm_sq_submit(&q.sq); if ((q.wait().dword[3] >> 17) == 0x04) errs++; }
        nvmt_stats_t st; nvmt_stats(r.t, &st);
        CHECK("fail_every_third", errs == 3 && st.error_cpls == 3);
        free(buf);
    }
    // ---- CQ back-pressure: the target must not overwrite unconsumed entries ----
    {
        Rig r;
        Qp q(r, 1, 4);       // CQ of 4 holds 3 unacknowledged completions
        nvm_queue_t sq2; nvm_dma_t* m; nvm_dma_create(&m, r.ctrl, 4096);
        // a second, deeper SQ on the same CQ is not needed: submit 3, leave them, submit 3 more after freeing SQ slots by hand
        uint8_t* buf; posix_memalign((void**)&buf, 4096, 4096);
        for (uint16_t i = 0; i < 3; i++) q.submit(i, NVM_IO_READ, (uint64_t)buf, 0, 0, 8);
        nvm_sq_submit(&q.sq);
        struct timespec ts = {0, 50 * 1000 * 1000}; nanosleep(&ts, nullptr);
        q.sq.head += 3;       // the controller has fetched them (three completions are waiting in the CQ)
        for (uint16_t i = 3; i < 6; i++) q.submit(i, NVM_IO_READ, (uint64_t)buf, 0, 0, 8);
        nvm_sq_submit(&q.sq);
        nanosleep(&ts, nullptr);
        nvmt_stats_t st; nvmt_stats(r.t, &st);
        bool stalled = st.cq_full_stalls >= 1;
        bool ok = true;
        for (int i = 0; i < 6; i++) { nvm_cpl_t* c = nvm_cq_dequeue_block(&q.cq, 2000); ok &= c && (c->dword[3] & 0xffff) == i; nvm_cq_update(&q.cq); }
        CHECK("cq_full_back_pressure", stalled && ok);
        (void)sq2; nvm_dma_unmap(m); free(buf);
    }
    // ---- registry ----
    {
        Rig r;
        CHECK("publish_lookup", nvmt_publish("/dev/libnvm-test", r.t) == 0 && nvmt_lookup("/dev/libnvm-test") == r.t &&
                                nvmt_publish("/dev/libnvm-test", r.t) == EEXIST && nvmt_lookup("/dev/nope") == nullptr);
    }
    CHECK("unpublished_on_destroy", nvmt_lookup("/dev/libnvm-test") == nullptr);
    // ---- protocol ceiling helper runs and counts ----
    {
        nvmt_config_t cfg{}; cfg.ns_bytes = 1 << 26; cfg.lba_bytes = 512; cfg.seed = 1; cfg.n_io_threads = 1; cfg.max_queue_entries = 256; cfg.max_io_queues = 4;
        double iops = nvmt_selftest_iops(&cfg, 2, 32, 20000, 4096);
        CHECK("selftest_iops_positive", iops > 1000.0);
        CHECK("selftest_rejects_bad_args", nvmt_selftest_iops(&cfg, 0, 32, 10, 4096) < 0 && nvmt_selftest_iops(&cfg, 1, 1024, 10, 4096) < 0);
    }
    // ---- nvm_ctrl_init(fd): maps the register window behind a descriptor (reference include/nvm_ctrl.h:36) ----
    {
        nvm_ctrl_t* c = nullptr;
        CHECK("ctrl_init_fd_bad_descriptor", nvm_ctrl_init(&c, -1) == EBADF && !c);
        char path[] = "/tmp/bam_bar0_XXXXXX";
        int fd = mkstemp(path);
        std::vector<uint8_t> img(NVM_CTRL_MEM_MINSIZE, 0);
        // CAP: MQES = 255, TO = 3 (1500 ms), DSTRD = 2, MPSMIN = 0 (4 KiB), MPSMAX = 4
        uint64_t cap = 255ull | (3ull << 24) | (2ull << 32) | (0ull << 48) | (4ull << 52);
        memcpy(img.data(), &cap, 8);
        bool wrote = write(fd, img.data(), img.size()) == (ssize_t)img.size();
        int s = nvm_ctrl_init(&c, fd);
        CHECK("ctrl_init_fd_maps_and_reads_cap", wrote && s == 0 && c && c->max_qs == 256 && c->timeout == 1500 && c->dstrd == 2 && c->page_size == 4096 && c->mm_size == NVM_CTRL_MEM_MINSIZE);
        if (c) { *(volatile uint32_t*)((volatile char*)c->mm_ptr + 0x14) = 0x00460001u; }
        uint32_t cc = 0;
        bool through = c && pread(fd, &cc, 4, 0x14) == 4 && cc == 0x00460001u;       // a shared mapping: register writes reach the file
        CHECK("ctrl_init_fd_mapping_is_shared", through);
        nvm_ctrl_free(c);
        close(fd); unlink(path);
        // a regular file shorter than the register window (or empty): an error code, not a bus error at the first register read
        for (size_t short_size : {(size_t)0, (size_t)64, (size_t)NVM_CTRL_MEM_MINSIZE - 1}) {
            char spath[] = "/tmp/bam_bar0s_XXXXXX";
            int sfd = mkstemp(spath);
            bool sized = ftruncate(sfd, (off_t)short_size) == 0;
            c = nullptr;
            int e = nvm_ctrl_init(&c, sfd);
            CHECK("ctrl_init_fd_short_file", sized && e == ENODEV && !c);
            close(sfd); unlink(spath);
        }
        int pfd[2];
        if (pipe(pfd) == 0) {
            c = nullptr;
            int e = nvm_ctrl_init(&c, pfd[0]);
            CHECK("ctrl_init_fd_unmappable", e != 0 && e > 0 && !c);
            close(pfd[0]); close(pfd[1]);
        }
    }
    // ---- SQ slot laps across the wrap of the 32-bit ticket counter ----
    {
        bool ok = true;
        for (uint32_t qs_log2 : {1u, 4u, 10u, 16u}) {
            const uint32_t qs = 1u << qs_log2;
            uint32_t word = 0;                                    // the slot word of slot 5 % qs, freed once per lap
            const uint32_t pos = 5u % qs;
            // walk the laps up to and across the wrap of the ticket counter: start a few laps before 2^32
            const uint64_t laps_total = 1ull << (32 - qs_log2);
            const uint64_t first_lap = laps_total - 3;
            word = (uint32_t)(first_lap * 2);                     // freed first_lap times so far
            for (uint64_t lap = first_lap; lap < laps_total + 4; lap++) {
                const uint32_t ticket = (uint32_t)(lap * qs + pos);   // wraps with the counter
                ok &= nvm_sq_slot_free(word, ticket, qs_log2) == 1;                       // my lap: free
                ok &= nvm_sq_slot_free(word, ticket + qs, qs_log2) == 0;                  // the next lap's holder must wait
                ok &= nvm_sq_slot_free(word - 2, ticket, qs_log2) == 0;                   // not yet freed for my lap
                word += 2;                                                                // the drainer frees the slot
            }
        }
        CHECK("sq_slot_laps_across_ticket_wrap", ok);
    }
    // ---- submission entry image against the NVMe layout, byte for byte (reference include/nvm_cmd.h:54-88) ----
    {
        nvm_cmd_t c; memset(&c, 0, sizeof(c));
        nvm_cmd_header(&c, 0xBEEF, NVM_IO_READ, 1);
        nvm_cmd_data_ptr(&c, 0x1122334455667000ull, 0xAABBCCDD00112000ull);
        nvm_cmd_rw_blks(&c, 0x0123456789ABCDEFull, 8);
        const uint8_t want[64] = {
            0x02, 0x00, 0xEF, 0xBE,  0x01, 0x00, 0x00, 0x00,                               // opcode, FUSE/PSDT, CID | NSID
            0, 0, 0, 0, 0, 0, 0, 0,  0, 0, 0, 0, 0, 0, 0, 0,                               // CDW2-3, MPTR
            0x00, 0x70, 0x66, 0x55, 0x44, 0x33, 0x22, 0x11,                                // PRP1
            0x00, 0x20, 0x11, 0x00, 0xDD, 0xCC, 0xBB, 0xAA,                                // PRP2
            0xEF, 0xCD, 0xAB, 0x89, 0x67, 0x45, 0x23, 0x01,                                // SLBA
            0x07, 0x00, 0x00, 0x00,  0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0 };                 // NLB (zero based), CDW13-15
        CHECK("sqe_read_image_matches_spec_bytes", memcmp(c.dword, want, 64) == 0);
        nvm_cmd_t w; memset(&w, 0xff, sizeof(w));               // the encoders must not depend on what the entry held, except DW12's upper half
        for (int i = 0; i < 16; i++) w.dword[i] = 0;
        nvm_cmd_header(&w, 0x0001, NVM_IO_WRITE, 0xffffffffu);
        nvm_cmd_data_ptr(&w, 0x1000, 0);
        nvm_cmd_rw_blks(&w, 0, 1);
        const uint8_t* wb = (const uint8_t*)w.dword;
        CHECK("sqe_write_image", wb[0] == 0x01 && wb[2] == 0x01 && wb[3] == 0x00 && w.dword[1] == 0xffffffffu && w.dword[6] == 0x1000 && w.dword[12] == 0);
        // the seal only touches CDW2 and CDW3, verifies, and breaks on any change of the entry or of the ticket
        nvm_cmd_t sld = c;
        nvm_cmd_seal(&sld, 0x12345678u);
        bool only23 = true;
        for (int i = 0; i < 16; i++) if (i != 2 && i != 3) only23 &= sld.dword[i] == c.dword[i];
        bool breaks = nvm_cmd_seal_ok(&sld, 0x12345678u) && !nvm_cmd_seal_ok(&sld, 0x12345679u) && !nvm_cmd_seal_ok(&c, 0);
        for (int i = 0; i < 16 && breaks; i++)
            for (int b = 0; b < 32; b += 7) { nvm_cmd_t x = sld; x.dword[i] ^= 1u << b; breaks &= !nvm_cmd_seal_ok(&x, 0x12345678u); }
        CHECK("sqe_seal_touches_cdw2_cdw3_only_and_verifies", only23 && sld.dword[2] == 0x12345678u && breaks);
    }
    printf("%s (%d failures)\n", failures ? "FAILED" : "PASSED", failures);
    return failures ? 1 : 0;
}
