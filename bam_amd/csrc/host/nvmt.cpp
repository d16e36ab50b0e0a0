// Software NVMe target: controller model served by host threads (see nvmt.h).
// Register layout follows the NVMe 1.x specification (the same offsets the
// reference lists in src/regs.h:9-47); admin command fields follow the
// specification sections the reference encodes in src/admin.cpp:20-64.
#include "nvmt.h"
#include "nvm_cmd.h"
#include "nvm_types.h"

#if defined(__x86_64__)
#include <immintrin.h>
#endif
#include <atomic>
#include <cerrno>
#include <chrono>
#include <map>
#include <string>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <thread>
#include <vector>

namespace {

constexpr uint32_t REG_CAP = 0x00, REG_VER = 0x08, REG_CC = 0x14, REG_CSTS = 0x1c,
                   REG_AQA = 0x24, REG_ASQ = 0x28, REG_ACQ = 0x30, REG_DBS = 0x1000;

// status = (SCT << 8 | SC); goes into CQE DW3[31:17]
constexpr uint16_t ST_OK = 0x000, ST_INVALID_OPCODE = 0x001, ST_INVALID_FIELD = 0x002,
                   ST_DATA_XFER_ERROR = 0x004, ST_LBA_RANGE = 0x080, ST_WRITE_RO = 0x082,
                   ST_CQ_INVALID = 0x100, ST_QID_INVALID = 0x101, ST_QSIZE_INVALID = 0x102;

inline uint64_t mix64(uint64_t z)
{
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

inline void cpu_relax()
{
#if defined(__x86_64__)
    __builtin_ia32_pause();
#endif
}

template <typename T> inline T ld(const volatile void* p) { return __atomic_load_n((const T*)p, __ATOMIC_ACQUIRE); }
template <typename T> inline void st(volatile void* p, T v) { __atomic_store_n((T*)p, v, __ATOMIC_RELEASE); }

struct Cq {
    bool valid = false;
    uint32_t qs = 0, tail = 0, phase = 1;
    uint32_t head_seen = 0;        // newest plausible value of the head doorbell
    nvm_cpl_t* mem = nullptr;
    volatile uint32_t* head_db = nullptr;
};

struct Sq {
    bool valid = false;
    uint16_t id = 0, cqid = 0;
    uint32_t qs = 0, head = 0, last_tail = 0;
    bool sealed = false;           // entries carry sequence number + checksum (nvm_cmd_seal)
    uint32_t fetched = 0;          // commands fetched so far = sequence number expected next
    bool retry_counted = false;
    nvm_cmd_t* mem = nullptr;
    volatile uint32_t* tail_db = nullptr;
};

// Counters are kept per service thread (relaxed atomics on a private cache line: uncontended) and summed on read.
struct alignas(128) Stats {
    std::atomic<uint64_t> admin_cmds{0}, io_cmds{0}, read_cmds{0}, write_cmds{0}, bytes_read{0},
        bytes_written{0}, error_cpls{0}, sq_doorbells{0}, cq_full_stalls{0}, dropped{0}, sqe_retries{0}, stale_doorbells{0};
    void bump(std::atomic<uint64_t>& c, uint64_t v = 1) { c.store(c.load(std::memory_order_relaxed) + v, std::memory_order_relaxed); }
    void clear() { for (auto* c : {&admin_cmds, &io_cmds, &read_cmds, &write_cmds, &bytes_read, &bytes_written, &error_cpls, &sq_doorbells, &cq_full_stalls, &dropped, &sqe_retries, &stale_doorbells}) c->store(0, std::memory_order_relaxed); }
};

struct IoThread {
    Stats stats;
    std::thread th;
    std::mutex mu;                 // guards `sqs` (held by the service loop for one pass)
    std::vector<uint16_t> sqs;     // SQ ids served by this thread
    uint64_t rng = 0x9E3779B97F4A7C15ull;
};



} // namespace

struct nvmt {
    nvmt_config_t cfg;
    uint8_t* bar = nullptr;
    size_t bar_size = 0;
    uint32_t db_stride = 4;
    std::atomic<bool> stop{false};
    bool enabled = false;
    uint32_t mps = 4096;
    uint16_t granted_sqs = 0, granted_cqs = 0;
    Sq asq; Cq acq;
    std::vector<Sq> sqs;           // index = qid
    std::vector<Cq> cqs;
    std::vector<IoThread*> io;
    std::thread ctrl_thread;
    std::atomic<uint64_t> cmd_seq{0};
    std::atomic<int> trace_errors{0};      // NVMT_TRACE_ERRORS=n: print the first n failing I/O commands to stderr
    Stats stats;

    volatile uint32_t* sq_db(uint32_t y) { return (volatile uint32_t*)(bar + REG_DBS + (2 * y) * db_stride); }
    volatile uint32_t* cq_db(uint32_t y) { return (volatile uint32_t*)(bar + REG_DBS + (2 * y + 1) * db_stride); }
};

namespace {

// Walk the PRP entries of a command: fn(bus_addr, length) for every contiguous piece.
template <typename F>
bool for_each_prp(const nvmt* t, const nvm_cmd_t& c, uint64_t bytes, F&& fn)
{
    const uint64_t P = t->mps;
    uint64_t prp1 = ((uint64_t)c.dword[7] << 32) | c.dword[6];
    uint64_t prp2 = ((uint64_t)c.dword[9] << 32) | c.dword[8];
    if (!prp1) return false;
    uint64_t first = P - (prp1 & (P - 1));
    if (first > bytes) first = bytes;
    fn(prp1, first);
    uint64_t left = bytes - first;
    if (!left) return true;
    if (!prp2) return false;
    if (left <= P) { fn(prp2, left); return true; }
    // PRP2 addresses a list of page pointers; the last entry of a list page chains to the next one
    uint64_t lp = prp2 & ~7ull;
    while (left) {
        uint64_t e = ld<uint64_t>((const void*)lp);
        if ((lp & (P - 1)) == P - 8 && left > P) { lp = e & ~7ull; continue; }
        uint64_t n = left < P ? left : P;
        if (!e) return false;
        fn(e, n);
        left -= n; lp += 8;
    }
    return true;
}

// words w0.. of a procedural namespace.  The loop has independent iterations and 64-bit multiplies, so it
// vectorises; it is built three times and the widest variant the CPU supports is picked once.
#define BAM_GEN_WORDS_BODY                                              \
    const uint64_t s0 = seed + (w0 + 1) * 0x9E3779B97F4A7C15ull;        \
    for (uint64_t k = 0; k < n; k++) {                                  \
        uint64_t z = s0 + k * 0x9E3779B97F4A7C15ull;                    \
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;                    \
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;                    \
        out[k] = z ^ (z >> 31);                                         \
    }
#if defined(__x86_64__)
__attribute__((target("avx512f,avx512dq,avx512vl"), optimize("O3")))
void gen_words_avx512(uint64_t seed, uint64_t w0, uint64_t n, uint64_t* __restrict__ out) { BAM_GEN_WORDS_BODY }
__attribute__((target("avx2"), optimize("O3")))
void gen_words_avx2(uint64_t seed, uint64_t w0, uint64_t n, uint64_t* __restrict__ out) { BAM_GEN_WORDS_BODY }
#endif
void gen_words_base(uint64_t seed, uint64_t w0, uint64_t n, uint64_t* __restrict__ out) { BAM_GEN_WORDS_BODY }

// Copy to a DMA destination with streaming stores: the destination is read next by the device over the
// interconnect, never by this core, so it should neither be read for ownership nor stay in this core's cache.
#if defined(__x86_64__)
__attribute__((target("avx2")))
void copy_out_avx2(void* dst, const void* src, size_t n)
{
    if (((uintptr_t)dst | (uintptr_t)src | n) & 31) { memcpy(dst, src, n); return; }
    const __m256i* s = (const __m256i*)src;
    __m256i* d = (__m256i*)dst;
    for (size_t i = 0; i < n / 32; i++) _mm256_stream_si256(d + i, _mm256_load_si256(s + i));
}
#endif
void copy_out_base(void* dst, const void* src, size_t n) { memcpy(dst, src, n); }
typedef void (*copy_out_fn)(void*, const void*, size_t);
copy_out_fn pick_copy_out()
{
#if defined(__x86_64__)
    __builtin_cpu_init();
    if (__builtin_cpu_supports("avx2") && !getenv("NVMT_NO_STREAMING_STORES")) return copy_out_avx2;
#endif
    return copy_out_base;
}
const copy_out_fn copy_out = pick_copy_out();
inline void copy_out_fence()
{
#if defined(__x86_64__)
    _mm_sfence();
#endif
}

typedef void (*gen_words_fn)(uint64_t, uint64_t, uint64_t, uint64_t*);
gen_words_fn pick_gen_words()
{
#if defined(__x86_64__)
    __builtin_cpu_init();
    if (__builtin_cpu_supports("avx512dq") && __builtin_cpu_supports("avx512vl")) return gen_words_avx512;
    if (__builtin_cpu_supports("avx2")) return gen_words_avx2;
#endif
    return gen_words_base;
}
const gen_words_fn gen_words = pick_gen_words();

uint16_t do_rw(nvmt* t, Stats& st_, const nvm_cmd_t& c, bool write)
{
    const uint32_t lba = t->cfg.lba_bytes;
    uint64_t slba = ((uint64_t)c.dword[11] << 32) | c.dword[10];
    uint64_t nlb = (c.dword[12] & 0xffffu) + 1;
    uint64_t bytes = nlb * lba, off = slba * lba;
    if (off + bytes > t->cfg.ns_bytes || off + bytes < off) return ST_LBA_RANGE;
    if (c.dword[1] != 1) return ST_INVALID_FIELD;
    if (write && !t->cfg.backing) return ST_WRITE_RO;
    uint64_t done = 0;
    alignas(64) uint64_t tmp[512];      /* sizeof(tmp) is the generation chunk */
    bool ok = for_each_prp(t, c, bytes, [&](uint64_t addr, uint64_t len) {
        uint8_t* p = (uint8_t*)addr;
        if (write) {
            memcpy((uint8_t*)t->cfg.backing + off + done, p, len);
        } else if (t->cfg.backing) {
            copy_out(p, (const uint8_t*)t->cfg.backing + off + done, len);
        } else {
            // procedural content, generated in cache then copied out (pieces are multiples of 8 bytes)
            for (uint64_t k = 0; k < len; k += sizeof(tmp)) {
                uint64_t n = len - k < sizeof(tmp) ? len - k : sizeof(tmp);
                gen_words(t->cfg.seed, (off + done + k) / 8, n / 8, tmp);
                copy_out(p + k, tmp, n);
            }
        }
        done += len;
    });
    if (!ok) return ST_INVALID_FIELD;
    /* streaming stores are weakly ordered: the caller drains them (copy_out_fence) before it posts completions */
    if (write) { st_.bump(st_.write_cmds); st_.bump(st_.bytes_written, bytes); }
    else       { st_.bump(st_.read_cmds);  st_.bump(st_.bytes_read, bytes); }
    return ST_OK;
}

// Post one completion; waits while the CQ is full (head doorbell not advanced).
bool post_cpl(nvmt* t, Stats& st_, Cq& cq, uint16_t sqid, uint16_t sqhd, uint16_t cid, uint16_t status, uint32_t dw0)
{
    // tail is an index in [0, qs); admin queues need not be powers of two
    const uint32_t next = cq.tail + 1 == cq.qs ? 0 : cq.tail + 1;
    bool stalled = false;
    // the head doorbell is written by the consumer, so reading it is a cache miss every time it has moved: it is
    // looked at only when the ring is full as far as this side knows
    while (next == cq.head_seen) {
        // the consumer can only have acknowledged entries that were posted: a doorbell value outside
        // [head_seen, tail] is an old one that arrived late, and is ignored
        const uint32_t hd = ld<uint32_t>(cq.head_db) % cq.qs;
        const uint32_t adv = (hd + cq.qs - cq.head_seen) % cq.qs, outstanding = (cq.tail + cq.qs - cq.head_seen) % cq.qs;
        if (adv <= outstanding) cq.head_seen = hd;
        else st_.bump(st_.stale_doorbells);
        if (next != cq.head_seen) break;
        if (!stalled) { st_.bump(st_.cq_full_stalls); stalled = true; }
        if (t->stop.load(std::memory_order_relaxed)) return false;
        cpu_relax();
    }
    nvm_cpl_t* e = cq.mem + cq.tail;
    const uint32_t dw2 = (uint32_t)sqhd | ((uint32_t)sqid << 16);
    const uint32_t dw3 = (uint32_t)cid | (cq.phase << 16) | ((uint32_t)status << 17);
#if defined(__x86_64__)
    // The whole entry as one aligned 16-byte store.  The ring may be device memory reached through a write-combining
    // window, where separate stores to one entry can leave in pieces and in any order; a 16-byte store leaves in one
    // piece or in aligned halves, and SQHD shares its half with the phase tag, which is what the consumer reads together.
    std::atomic_thread_fence(std::memory_order_release);
    _mm_store_si128((__m128i*)e, _mm_set_epi32((int)dw3, (int)dw2, 0, (int)dw0));
#else
    e->dword[0] = dw0;
    e->dword[1] = 0;
    e->dword[2] = dw2;
    // DW3 carries the phase tag: it must become visible last
    st<uint32_t>(&e->dword[3], dw3);
#endif
    cq.tail = next;
    if (next == 0) cq.phase ^= 1;
    if (status) st_.bump(st_.error_cpls);
    return true;
}

void serve_sq(nvmt* t, IoThread* me, Sq& sq)
{
    Cq& cq = t->cqs[sq.cqid];
    const uint32_t mask = sq.qs - 1;
    Stats& st_ = me->stats;
    // A sealed queue is read by its seals: the entry at the head is looked at whether a doorbell has announced it or
    // not (the line stays in this core's cache until the submitter writes it, so a look at an idle queue costs next to
    // nothing), and entries are taken for as long as sequence number and checksum match.  Doorbells and entries are
    // not ordered on their way here, and neither are two doorbells: the last doorbell of a burst may be an old one,
    // and a queue read by its doorbell would then sit on entries nobody announces again.  The doorbell register is
    // still read for the counters.  An unsealed queue is read by its doorbell, as the NVMe specification has it.
    uint32_t tail = sq.sealed ? sq.last_tail : ld<uint32_t>(sq.tail_db) & mask;
    if (!sq.sealed && tail != sq.last_tail) { st_.bump(st_.sq_doorbells); sq.last_tail = tail; }
    for (;;) {
        nvm_cmd_t batch[64];
        uint32_t n;
        if (sq.sealed) {
            uint32_t got = 0;
            for (; got < 64; got++) {
                batch[got] = sq.mem[(sq.head + got) & mask];
                std::atomic_thread_fence(std::memory_order_acquire);
                if (!nvm_cmd_seal_ok(&batch[got], sq.fetched + got)) break;
            }
            if (got < 64) {
                // an entry that a doorbell covers but that does not verify yet has been overtaken by its doorbell
                tail = ld<uint32_t>(sq.tail_db) & mask;
                if (tail != sq.last_tail) { st_.bump(st_.sq_doorbells); sq.last_tail = tail; }
                const uint32_t announced = (tail - sq.head) & mask;
                if (announced > got && announced <= sq.qs / 2 && !sq.retry_counted) {
                    st_.bump(st_.sqe_retries); sq.retry_counted = true;
                    if (getenv("NVMT_DEBUG_SEAL")) {
                        const nvm_cmd_t& e = batch[got];
                        fprintf(stderr, "[nvmt %p] sq %u slot %u: want ticket %u, entry dw0 %08x dw2 %08x dw3 %08x (seal %08x) slba %u head %u tail %u\n", (void*)t, sq.id,
                                (sq.head + got) & mask, sq.fetched + got, e.dword[0], e.dword[2], e.dword[3], nvm_cmd_seal_value(&e, sq.fetched + got), e.dword[10], sq.head, tail);
                    }
                }
            }
            if (!got) return;
            sq.retry_counted = false;
            n = got;
            sq.fetched += n;
        } else {
            n = (tail - sq.head) & mask;
            if (!n) return;
            if (n > 64) n = 64;
            for (uint32_t i = 0; i < n; i++) batch[i] = sq.mem[(sq.head + i) & mask];
        }
        sq.head = (sq.head + n) & mask;
        uint32_t order[64];
        for (uint32_t i = 0; i < n; i++) order[i] = t->cfg.order == NVMT_ORDER_REVERSE ? n - 1 - i : i;
        if (t->cfg.order == NVMT_ORDER_SHUFFLE)
            for (uint32_t i = n; i > 1; i--) {
                me->rng = mix64(me->rng + 0x9E3779B97F4A7C15ull);
                uint32_t j = (uint32_t)(me->rng % i), x = order[i - 1];
                order[i - 1] = order[j]; order[j] = x;
            }
        // all commands of the batch first, then one drain of the streaming stores, then their completions
        uint16_t statuses[64];
        bool dropped[64];
        for (uint32_t k = 0; k < n; k++) {
            const nvm_cmd_t& c = batch[order[k]];
            uint8_t op = c.dword[0] & 0xff;
            uint16_t status;
            const bool inject = t->cfg.drop_every || t->cfg.fail_every;
            const uint64_t seq = inject ? ++t->cmd_seq : 0;       // a shared counter only when fault injection needs one
            st_.bump(st_.io_cmds);
            dropped[k] = false;
            statuses[k] = ST_OK;
            if (t->cfg.drop_every && seq % t->cfg.drop_every == 0) { st_.bump(st_.dropped); dropped[k] = true; continue; }
            if (t->cfg.fail_every && seq % t->cfg.fail_every == 0) status = ST_DATA_XFER_ERROR;
            else if (op == NVM_IO_READ) status = do_rw(t, st_, c, false);
            else if (op == NVM_IO_WRITE) status = do_rw(t, st_, c, true);
            else if (op == NVM_IO_FLUSH) status = ST_OK;
            else status = ST_INVALID_OPCODE;
            if (status && t->trace_errors.load(std::memory_order_relaxed) > 0 && t->trace_errors.fetch_sub(1) > 0)
                fprintf(stderr, "[nvmt] sq %u status %#x: dw0 %08x nsid %u prp1 %08x%08x prp2 %08x%08x slba %08x%08x dw12 %08x (sq head %u)\n",
                        sq.id, status, c.dword[0], c.dword[1], c.dword[7], c.dword[6], c.dword[9], c.dword[8], c.dword[11], c.dword[10], c.dword[12], sq.head);
            statuses[k] = status;
        }
        copy_out_fence();
        for (uint32_t k = 0; k < n; k++) {
            if (dropped[k]) continue;
            const uint16_t cid = batch[order[k]].dword[0] >> 16;
            if (!post_cpl(t, st_, cq, sq.id, (uint16_t)sq.head, cid, statuses[k], 0)) return;
        }
        copy_out_fence();       // completions written through a write-combining window (a ring in device memory) leave now

    }
}

void io_loop(nvmt* t, IoThread* me)
{
    uint32_t idle = 0;
    const bool dbg = getenv("NVMT_DEBUG_LOOP") != nullptr;
    uint64_t d_sweeps = 0, d_busy_sweeps = 0, d_visits = 0, d_cmds = 0, d_busy_ns = 0, d_max_sweep_ns = 0, d_t_first = 0, d_t_last = 0;
    while (!t->stop.load(std::memory_order_relaxed)) {
        bool any = false;
        {
            std::lock_guard<std::mutex> g(me->mu);
            const auto s0 = dbg ? std::chrono::steady_clock::now() : std::chrono::steady_clock::time_point();
            for (uint16_t id : me->sqs) {
                Sq& sq = t->sqs[id];
                if (!sq.valid) continue;
                uint32_t before = sq.head;
                serve_sq(t, me, sq);
                any |= before != sq.head;
                if (dbg && before != sq.head) { d_visits++; d_cmds += (sq.head - before) & (sq.qs - 1); }
            }
            if (dbg) {
                const uint64_t ns = (uint64_t)std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::steady_clock::now() - s0).count();
                d_sweeps++;
                if (any) {
                    d_busy_sweeps++;
                    d_busy_ns += ns;
                    if (ns > d_max_sweep_ns) d_max_sweep_ns = ns;
                    const uint64_t now = (uint64_t)std::chrono::duration_cast<std::chrono::nanoseconds>(s0.time_since_epoch()).count();
                    if (!d_t_first) d_t_first = now;
                    d_t_last = now + ns;
                }
            }
            if (me->sqs.empty()) idle = 1u << 20;
        }
        if (any) idle = 0;
        else if (++idle > 4096) std::this_thread::sleep_for(std::chrono::microseconds(idle > (1u << 19) ? 200 : 20));
        else cpu_relax();
    }
    if (dbg && d_cmds)
        fprintf(stderr, "[nvmt loop] queues %zu: busy sweeps %llu of %llu, busy time %.1f ms over a span of %.1f ms, max sweep %.1f us, visits with work %llu, cmds %llu (%.2f per visit, %.2f us per cmd)\n",
                me->sqs.size(), (unsigned long long)d_busy_sweeps, (unsigned long long)d_sweeps, d_busy_ns / 1e6, (d_t_last - d_t_first) / 1e6, d_max_sweep_ns / 1e3,
                (unsigned long long)d_visits, (unsigned long long)d_cmds, (double)d_cmds / d_visits, d_busy_ns / 1e3 / d_cmds);
}

// ---- admin side ----
void identify(nvmt* t, const nvm_cmd_t& c, uint16_t& status)
{
    uint64_t prp1 = ((uint64_t)c.dword[7] << 32) | c.dword[6];
    uint8_t* d = (uint8_t*)prp1;
    uint32_t cns = c.dword[10] & 0xff;
    if (!d) { status = ST_INVALID_FIELD; return; }
    memset(d, 0, 4096);
    if (cns == 1) {
        d[0] = 0x02; d[1] = 0x10; d[2] = 0x02; d[3] = 0x10;            // VID / SSVID
        memcpy(d + 4, "SWTARGET0001        ", 20);                     // SN
        memcpy(d + 24, "bam-amd software NVMe target            ", 40); // MN
        memcpy(d + 64, "1.0     ", 8);                                 // FR
        d[77] = 8;                                                     // MDTS: 2^8 pages
        d[512] = 0x66; d[513] = 0x44;                                  // SQES 64 B, CQES 16 B
        uint16_t maxcmd = (uint16_t)(t->cfg.max_queue_entries - 1);
        memcpy(d + 514, &maxcmd, 2);
        uint32_t nn = 1; memcpy(d + 516, &nn, 4);
    } else if (cns == 0) {
        if (c.dword[1] != 1) { status = ST_INVALID_FIELD; return; }
        uint64_t blocks = t->cfg.ns_bytes / t->cfg.lba_bytes;
        memcpy(d + 0, &blocks, 8); memcpy(d + 8, &blocks, 8); memcpy(d + 16, &blocks, 8);
        d[25] = 0; d[26] = 0;                                          // NLBAF = 0, FLBAS = format 0
        uint32_t lbaf = (uint32_t)__builtin_ctz(t->cfg.lba_bytes) << 16;
        memcpy(d + 128, &lbaf, 4);
    } else status = ST_INVALID_FIELD;
}

void assign_sq(nvmt* t, uint16_t id, bool add)
{
    IoThread* th = t->io[t->sqs[id].cqid % t->io.size()];
    std::lock_guard<std::mutex> g(th->mu);
    if (add) th->sqs.push_back(id);
    else for (size_t i = 0; i < th->sqs.size(); i++) if (th->sqs[i] == id) { th->sqs.erase(th->sqs.begin() + i); break; }
}

void admin_cmd(nvmt* t, const nvm_cmd_t& c)
{
    uint8_t op = c.dword[0] & 0xff;
    uint16_t cid = c.dword[0] >> 16, status = ST_OK;
    uint32_t dw0 = 0;
    uint64_t prp1 = ((uint64_t)c.dword[7] << 32) | c.dword[6];
    uint16_t qid = c.dword[10] & 0xffff;
    uint32_t qs = (c.dword[10] >> 16) + 1;
    t->stats.bump(t->stats.admin_cmds);
    switch (op) {
    case NVM_ADMIN_IDENTIFY: identify(t, c, status); break;
    case NVM_ADMIN_SET_FEATURES:
    case NVM_ADMIN_GET_FEATURES:
        if ((c.dword[10] & 0xff) != 0x07) { status = ST_INVALID_FIELD; break; }
        if (op == NVM_ADMIN_SET_FEATURES) {
            uint32_t nsq = (c.dword[11] & 0xffff) + 1, ncq = (c.dword[11] >> 16) + 1;
            t->granted_sqs = (uint16_t)(nsq < t->cfg.max_io_queues ? nsq : t->cfg.max_io_queues);
            t->granted_cqs = (uint16_t)(ncq < t->cfg.max_io_queues ? ncq : t->cfg.max_io_queues);
        }
        dw0 = ((uint32_t)(t->granted_cqs - 1) << 16) | (uint32_t)(t->granted_sqs - 1);
        break;
    case NVM_ADMIN_CREATE_CQ:
        if (qid == 0 || qid > t->cfg.max_io_queues || t->cqs[qid].valid) { status = ST_QID_INVALID; break; }
        if (qs < 2 || qs > t->cfg.max_queue_entries || (qs & (qs - 1))) { status = ST_QSIZE_INVALID; break; }
        if (!prp1 || !(c.dword[11] & 1)) { status = ST_INVALID_FIELD; break; }
        {
            Cq& q = t->cqs[qid];
            q.qs = qs; q.tail = 0; q.phase = 1; q.head_seen = 0; q.mem = (nvm_cpl_t*)prp1; q.head_db = t->cq_db(qid);
            st<uint32_t>(q.head_db, 0);
            q.valid = true;
        }
        break;
    case NVM_ADMIN_CREATE_SQ: {
        uint16_t cqid = c.dword[11] >> 16;
        if (qid == 0 || qid > t->cfg.max_io_queues || t->sqs[qid].valid) { status = ST_QID_INVALID; break; }
        if (cqid == 0 || cqid > t->cfg.max_io_queues || !t->cqs[cqid].valid) { status = ST_CQ_INVALID; break; }
        if (qs < 2 || qs > t->cfg.max_queue_entries || (qs & (qs - 1))) { status = ST_QSIZE_INVALID; break; }
        if (!prp1 || !(c.dword[11] & 1)) { status = ST_INVALID_FIELD; break; }
        Sq& q = t->sqs[qid];
        q.id = qid; q.cqid = cqid; q.qs = qs; q.head = 0; q.last_tail = 0; q.sealed = false; q.fetched = 0; q.retry_counted = false; q.mem = (nvm_cmd_t*)prp1; q.tail_db = t->sq_db(qid);
        st<uint32_t>(q.tail_db, 0);
        q.valid = true;
        assign_sq(t, qid, true);
        break;
    }
    case NVM_ADMIN_DELETE_SQ:
        if (qid == 0 || qid > t->cfg.max_io_queues || !t->sqs[qid].valid) { status = ST_QID_INVALID; break; }
        assign_sq(t, qid, false);
        t->sqs[qid].valid = false;
        break;
    case NVM_ADMIN_DELETE_CQ: {
        if (qid == 0 || qid > t->cfg.max_io_queues || !t->cqs[qid].valid) { status = ST_QID_INVALID; break; }
        bool used = false;
        for (auto& s : t->sqs) used |= s.valid && s.cqid == qid;
        if (used) { status = ST_INVALID_FIELD; break; }   // SQs must be deleted first
        t->cqs[qid].valid = false;
        break;
    }
    case NVM_ADMIN_GET_LOG_PAGE: {
        uint32_t numd = ((c.dword[10] >> 16) & 0xfff) + 1;
        if (!prp1) { status = ST_INVALID_FIELD; break; }
        memset((void*)prp1, 0, (size_t)numd * 4);
        break;
    }
    case NVM_ADMIN_ABORT: break;
    case NVM_ADMIN_VS_SEAL_SQ:
        if (qid == 0 || qid > t->cfg.max_io_queues || !t->sqs[qid].valid) { status = ST_QID_INVALID; break; }
        {
            IoThread* th = t->io[t->sqs[qid].cqid % t->io.size()];
            std::lock_guard<std::mutex> g(th->mu);
            t->sqs[qid].sealed = true;
        }
        break;
    default: status = ST_INVALID_OPCODE;
    }
    post_cpl(t, t->stats, t->acq, 0, (uint16_t)t->asq.head, cid, status, dw0);
}

void teardown_io(nvmt* t)
{
    for (IoThread* th : t->io) { std::lock_guard<std::mutex> g(th->mu); th->sqs.clear(); }
    for (auto& s : t->sqs) s.valid = false;
    for (auto& c : t->cqs) c.valid = false;
}

void ctrl_loop(nvmt* t)
{
    uint32_t idle = 0;
    while (!t->stop.load(std::memory_order_relaxed)) {
        uint32_t cc = ld<uint32_t>(t->bar + REG_CC);
        bool en = cc & 1;
        if (en && !t->enabled) {
            uint32_t aqa = ld<uint32_t>(t->bar + REG_AQA);
            t->mps = 1u << (12 + ((cc >> 7) & 0xf));
            t->asq = Sq(); t->acq = Cq();
            t->asq.qs = (aqa & 0xfff) + 1; t->asq.mem = (nvm_cmd_t*)ld<uint64_t>(t->bar + REG_ASQ); t->asq.tail_db = t->sq_db(0);
            t->acq.qs = ((aqa >> 16) & 0xfff) + 1; t->acq.mem = (nvm_cpl_t*)ld<uint64_t>(t->bar + REG_ACQ); t->acq.head_db = t->cq_db(0);
            st<uint32_t>(t->asq.tail_db, 0); st<uint32_t>(t->acq.head_db, 0);
            t->asq.valid = t->acq.valid = t->asq.mem && t->acq.mem;
            t->granted_sqs = t->granted_cqs = (uint16_t)t->cfg.max_io_queues;
            t->enabled = true;
            if (!t->cfg.never_ready) st<uint32_t>(t->bar + REG_CSTS, 1);
        } else if (!en && t->enabled) {
            teardown_io(t);
            t->asq.valid = t->acq.valid = false;
            t->enabled = false;
            st<uint32_t>(t->bar + REG_CSTS, 0);
        }
        bool any = false;
        if (t->enabled && t->asq.valid) {
            // admin queues need not be powers of two: index arithmetic by modulo
            uint32_t tail = ld<uint32_t>(t->asq.tail_db) % t->asq.qs;
            while (t->asq.head != tail) {
                nvm_cmd_t c = t->asq.mem[t->asq.head];
                t->asq.head = (t->asq.head + 1) % t->asq.qs;
                admin_cmd(t, c);
                any = true;
            }
        }
        if (any) idle = 0;
        else if (++idle > 2000) std::this_thread::sleep_for(std::chrono::microseconds(50));
        else cpu_relax();
    }
}

} // namespace

static std::mutex g_registry_mu;
static std::map<std::string, nvmt*> g_registry;

extern "C" {

int nvmt_publish(const char* path, nvmt_t* t)
{
    if (!path || !*path || !t) return EINVAL;
    std::lock_guard<std::mutex> g(g_registry_mu);
    if (g_registry.count(path)) return EEXIST;
    g_registry[path] = t;
    return 0;
}

nvmt_t* nvmt_lookup(const char* path)
{
    if (!path) return nullptr;
    std::lock_guard<std::mutex> g(g_registry_mu);
    auto it = g_registry.find(path);
    return it == g_registry.end() ? nullptr : it->second;
}

const nvmt_config_t* nvmt_config(nvmt_t* t) { return &t->cfg; }

size_t nvmt_bar_size(const nvmt_config_t* cfg)
{
    size_t n = REG_DBS + (size_t)2 * (cfg->max_io_queues + 1) * (4u << cfg->dstrd);
    if (n < 0x2000) n = 0x2000;
    return (n + 4095) & ~(size_t)4095;
}

nvmt_t* nvmt_create(const nvmt_config_t* cfg, void* bar_mem)
{
    if (!cfg || !bar_mem || ((uintptr_t)bar_mem & 4095)) return nullptr;
    if (cfg->lba_bytes != 512 && cfg->lba_bytes != 4096) return nullptr;
    if (!cfg->n_io_threads || cfg->max_io_queues < 1 || cfg->max_io_queues > 1023 || cfg->dstrd > 8) return nullptr;
    uint32_t mq = cfg->max_queue_entries;
    if (mq < 2 || mq > 65536 || (mq & (mq - 1)) || cfg->ns_bytes % cfg->lba_bytes) return nullptr;

    nvmt* t = new nvmt();
    t->cfg = *cfg;
    t->bar = (uint8_t*)bar_mem;
    t->bar_size = nvmt_bar_size(cfg);
    t->db_stride = 4u << cfg->dstrd;
    if (const char* e = getenv("NVMT_TRACE_ERRORS")) t->trace_errors = atoi(e);
    t->sqs.resize(cfg->max_io_queues + 1);
    t->cqs.resize(cfg->max_io_queues + 1);
    memset(t->bar, 0, t->bar_size);
    uint64_t to = cfg->timeout_500ms ? cfg->timeout_500ms : 2;
    uint64_t cap = (uint64_t)(mq - 1) | (1ull << 16) | (to << 24) | ((uint64_t)cfg->dstrd << 32) |
                   (1ull << 37) | (0ull << 48) | (4ull << 52);   // CQR, CSS = NVM, MPSMIN 4 KiB, MPSMAX 64 KiB
    st<uint64_t>(t->bar + REG_CAP, cap);
    st<uint32_t>(t->bar + REG_VER, 0x00010400);
    for (uint32_t i = 0; i < cfg->n_io_threads; i++) {
        IoThread* th = new IoThread();
        th->rng ^= mix64(i + 1);
        t->io.push_back(th);
    }
    for (IoThread* th : t->io) th->th = std::thread(io_loop, t, th);
    t->ctrl_thread = std::thread(ctrl_loop, t);
    return t;
}

void nvmt_destroy(nvmt_t* t)
{
    if (!t) return;
    {
        std::lock_guard<std::mutex> g(g_registry_mu);
        for (auto it = g_registry.begin(); it != g_registry.end();)
            it = it->second == t ? g_registry.erase(it) : std::next(it);
    }
    t->stop = true;
    t->ctrl_thread.join();
    for (IoThread* th : t->io) { th->th.join(); delete th; }
    delete t;
}

volatile void* nvmt_bar(nvmt_t* t) { return t->bar; }

void nvmt_stats(nvmt_t* t, nvmt_stats_t* o)
{
    memset(o, 0, sizeof(*o));
    auto add = [&](const Stats& s) {
        o->admin_cmds += s.admin_cmds; o->io_cmds += s.io_cmds; o->read_cmds += s.read_cmds; o->write_cmds += s.write_cmds;
        o->bytes_read += s.bytes_read; o->bytes_written += s.bytes_written; o->error_cpls += s.error_cpls;
        o->sq_doorbells += s.sq_doorbells; o->cq_full_stalls += s.cq_full_stalls; o->dropped += s.dropped;
        o->sqe_retries += s.sqe_retries; o->stale_doorbells += s.stale_doorbells;
    };
    add(t->stats);
    for (IoThread* th : t->io) add(th->stats);
}

void nvmt_reset_stats(nvmt_t* t)
{
    t->stats.clear();
    for (IoThread* th : t->io) th->stats.clear();
}

void nvmt_fill_words(uint64_t seed, uint64_t first_word, uint64_t n, uint64_t* out) { gen_words(seed, first_word, n, out); }

int nvmt_queue_state(nvmt_t* t, uint16_t qid, uint64_t* out8)
{
    if (!t || !out8 || qid == 0 || qid >= t->sqs.size()) return EINVAL;
    const Sq& sq = t->sqs[qid];
    if (!sq.valid) return ENOENT;
    const Cq& cq = t->cqs[sq.cqid];
    out8[0] = sq.head; out8[1] = sq.fetched; out8[2] = ld<uint32_t>(sq.tail_db); out8[3] = sq.sealed;
    out8[4] = cq.tail; out8[5] = cq.head_seen; out8[6] = ld<uint32_t>(cq.head_db); out8[7] = cq.phase;
    return 0;
}

} // extern "C"
