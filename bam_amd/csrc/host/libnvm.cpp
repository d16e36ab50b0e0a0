// Host side of the NVMe layer: controller handle, admin queue pair, admin
// commands, DMA descriptors, status text.  Written against the NVMe 1.x
// specification; the entry points and their error behaviour are those of the
// reference's libnvm (src/ctrl.cpp:147-271 controller init/reset,
// src/rpc.cpp:299-494 admin RPC, src/admin.cpp:20-470 admin commands,
// src/dma.cpp:192-394 descriptors, src/queue.cpp:12-66 queue helpers,
// src/error.cpp:163-181 nvm_strerror).
#include "nvm_admin.h"
#include "nvm_aq.h"
#include "nvm_cmd.h"
#include "nvm_ctrl.h"
#include "nvm_dma.h"
#include "nvm_error.h"
#include "nvm_queue.h"
#include "nvm_types.h"
#include "nvm_util.h"

#include <cerrno>
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <thread>
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

namespace {

using clk = std::chrono::steady_clock;

struct CtrlBox {
    nvm_ctrl_t handle;      // first member: the public handle is the box address
    std::mutex mu;
    int refs = 1;
    void* mapped = nullptr;     // register window this layer mapped itself (nvm_ctrl_init): unmapped with the last reference
    size_t mapped_size = 0;
};

struct DmaBox {
    CtrlBox* ctrl;
    void* owned;            // memory allocated by nvm_dma_create (freed on unmap)
    nvm_dma_t map;          // flexible tail: must stay last
};

inline CtrlBox* box_of(const nvm_ctrl_t* c) { return (CtrlBox*)(void*)c; }
inline DmaBox* box_of(const nvm_dma_t* d) { return (DmaBox*)((char*)d - offsetof(DmaBox, map)); }

void ctrl_get(CtrlBox* b) { std::lock_guard<std::mutex> g(b->mu); b->refs++; }
void ctrl_put(CtrlBox* b)
{
    bool last;
    { std::lock_guard<std::mutex> g(b->mu); last = --b->refs == 0; }
    if (last) {
        if (b->mapped) munmap(b->mapped, b->mapped_size);
        delete b;
    }
}

inline uint32_t rd32(volatile void* base, uint32_t off) { return __atomic_load_n((uint32_t*)((char*)base + off), __ATOMIC_ACQUIRE); }
inline uint64_t rd64(volatile void* base, uint32_t off) { return __atomic_load_n((uint64_t*)((char*)base + off), __ATOMIC_ACQUIRE); }
inline void wr32(volatile void* base, uint32_t off, uint32_t v) { __atomic_store_n((uint32_t*)((char*)base + off), v, __ATOMIC_RELEASE); }
inline void wr64(volatile void* base, uint32_t off, uint64_t v) { __atomic_store_n((uint64_t*)((char*)base + off), v, __ATOMIC_RELEASE); }

int wait_ready(const nvm_ctrl_t* c, uint32_t want)
{
    auto deadline = clk::now() + std::chrono::milliseconds(c->timeout);
    while ((rd32(c->mm_ptr, 0x1c) & 1) != want) {
        if (clk::now() > deadline) return ETIME;
        std::this_thread::sleep_for(std::chrono::microseconds(50));
    }
    return 0;
}

} // namespace

struct nvm_admin_reference {
    CtrlBox* ctrl;
    std::mutex lock;
    nvm_queue_t acq, asq;
    uint16_t next_cid = 0;
};

extern "C" {

// ---- controller ----
int nvm_raw_ctrl_init(nvm_ctrl_t** ctrl, volatile void* mm_ptr, size_t mm_size)
{
    if (!ctrl) return EINVAL;
    *ctrl = nullptr;
    if (!mm_ptr || mm_size < NVM_CTRL_MEM_MINSIZE) return EINVAL;
    uint64_t cap = rd64(mm_ptr, 0x00);
    size_t host_page = (size_t)sysconf(_SC_PAGESIZE);
    size_t min_page = (size_t)1 << (12 + _RB(cap, 51, 48)), max_page = (size_t)1 << (12 + _RB(cap, 55, 52));
    if (host_page < min_page || host_page > max_page) return ERANGE;
    CtrlBox* b = new CtrlBox();
    b->handle.page_size = host_page;
    b->handle.dstrd = (uint8_t)_RB(cap, 35, 32);
    b->handle.timeout = _RB(cap, 31, 24) * 500;
    b->handle.max_qs = (uint32_t)_RB(cap, 15, 0) + 1;
    b->handle.mm_size = mm_size;
    b->handle.mm_ptr = mm_ptr;
    *ctrl = &b->handle;
    return 0;
}

// The reference maps BAR0 of the device behind `fd` (a /dev/libnvmN node of its kernel module, or a sysfs resource
// file) and reads the handle from it (src/ctrl.cpp:147-199, src/linux/device.cpp:137-160).  The same here for any
// descriptor that can be mapped shared and read-write: errno of the failing call otherwise (EBADF, ENODEV, EACCES ...).
int nvm_ctrl_init(nvm_ctrl_t** ctrl, int fd)
{
    if (!ctrl) return EINVAL;
    *ctrl = nullptr;
    if (fcntl(fd, F_GETFL) == -1) return errno;
    /* a regular file shorter than the window maps all the same, and the first register read behind its end would be a
     * bus error instead of an error code */
    struct stat sb;
    if (fstat(fd, &sb) == -1) return errno;
    if (S_ISREG(sb.st_mode) && (uint64_t)sb.st_size < NVM_CTRL_MEM_MINSIZE) return ENODEV;
    void* mm = mmap(nullptr, NVM_CTRL_MEM_MINSIZE, PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
    if (mm == MAP_FAILED) return errno ? errno : ENODEV;
    int err = nvm_raw_ctrl_init(ctrl, mm, NVM_CTRL_MEM_MINSIZE);
    if (err) { munmap(mm, NVM_CTRL_MEM_MINSIZE); return err; }
    box_of(*ctrl)->mapped = mm;
    box_of(*ctrl)->mapped_size = NVM_CTRL_MEM_MINSIZE;
    return 0;
}

void nvm_ctrl_free(nvm_ctrl_t* ctrl)
{
    if (ctrl) ctrl_put(box_of(ctrl));
}

int nvm_raw_ctrl_reset(const nvm_ctrl_t* c, uint64_t acq_ioaddr, uint64_t asq_ioaddr)
{
    if (!c) return EINVAL;
    uint32_t cc = rd32(c->mm_ptr, 0x14);
    wr32(c->mm_ptr, 0x14, cc & ~1u);
    int err = wait_ready(c, 0);
    if (err) return err;
    uint32_t acq_entries = (uint32_t)(c->page_size / sizeof(nvm_cpl_t)), asq_entries = (uint32_t)(c->page_size / sizeof(nvm_cmd_t));
    wr32(c->mm_ptr, 0x24, (uint32_t)(_WB(acq_entries - 1, 27, 16) | _WB(asq_entries - 1, 11, 0)));
    wr64(c->mm_ptr, 0x28, asq_ioaddr);
    wr64(c->mm_ptr, 0x30, acq_ioaddr);
    uint32_t mps = (uint32_t)__builtin_ctzl(c->page_size) - 12;
    wr32(c->mm_ptr, 0x14, (uint32_t)(_WB(4, 23, 20) | _WB(6, 19, 16) | _WB(mps, 10, 7) | _WB(0, 3, 1) | 1u));
    return wait_ready(c, 1);
}

// ---- queue descriptors ----
int nvm_queue_clear(nvm_queue_t* q, const nvm_ctrl_t* ctrl, bool cq, uint16_t no, uint32_t qs, bool local, volatile void* vaddr, uint64_t ioaddr)
{
    if (!q || !ctrl || qs < 2 || (qs & (qs - 1)) || qs > 65536 || !vaddr) return EINVAL;
    memset(q, 0, sizeof(*q));
    q->no = no;
    q->qs = qs;
    q->qs_minus_1 = qs - 1;
    q->qs_log2 = (uint32_t)__builtin_ctz(qs);
    q->es = cq ? sizeof(nvm_cpl_t) : sizeof(nvm_cmd_t);
    q->phase = 1;
    q->local = local;
    q->vaddr = vaddr;
    q->ioaddr = ioaddr;
    q->db = (volatile uint32_t*)((volatile unsigned char*)ctrl->mm_ptr + 0x1000 + (size_t)(2 * no + (cq ? 1 : 0)) * (4u << ctrl->dstrd));
    return 0;
}

void nvm_queue_reset(nvm_queue_t* q)
{
    q->head = q->tail = q->last = 0;
    q->head_lock = q->tail_lock = q->in_ticket = q->cid_ticket = 0;
    q->phase = 1;
}

nvm_cpl_t* nvm_cq_dequeue_block(nvm_queue_t* cq, uint64_t timeout)
{
    auto deadline = clk::now() + std::chrono::milliseconds(timeout);
    for (uint32_t spins = 0;; spins++) {
        nvm_cpl_t* c = nvm_cq_dequeue(cq);
        if (c) return c;
        if (clk::now() > deadline) return nullptr;
        if (spins > 200) std::this_thread::sleep_for(std::chrono::microseconds(20));
    }
}

// ---- admin queue pair ----
int nvm_aq_create(nvm_aq_ref* ref, const nvm_ctrl_t* ctrl, const nvm_dma_t* win)
{
    if (!ref) return EINVAL;
    *ref = nullptr;
    if (!ctrl || !win || !win->vaddr || win->n_ioaddrs < 2 || win->page_size != ctrl->page_size) return EINVAL;
    memset(win->vaddr, 0, 2 * win->page_size);
    nvm_admin_reference* r = new nvm_admin_reference();
    r->ctrl = box_of(ctrl);
    nvm_queue_clear(&r->acq, ctrl, true, 0, (uint32_t)(ctrl->page_size / sizeof(nvm_cpl_t)), true, NVM_DMA_OFFSET(win, 0), win->ioaddrs[0]);
    nvm_queue_clear(&r->asq, ctrl, false, 0, (uint32_t)(ctrl->page_size / sizeof(nvm_cmd_t)), true, NVM_DMA_OFFSET(win, 1), win->ioaddrs[1]);
    int err = nvm_raw_ctrl_reset(ctrl, r->acq.ioaddr, r->asq.ioaddr);
    if (err) { delete r; return err; }
    ctrl_get(r->ctrl);
    *ref = r;
    return 0;
}

void nvm_aq_destroy(nvm_aq_ref ref)
{
    if (!ref) return;
    ctrl_put(ref->ctrl);
    delete ref;
}

void nvm_rpc_unbind(nvm_aq_ref ref) { nvm_aq_destroy(ref); }

const nvm_ctrl_t* nvm_ctrl_from_aq_ref(nvm_aq_ref ref) { return ref ? &ref->ctrl->handle : nullptr; }

int nvm_raw_rpc(nvm_aq_ref ref, nvm_cmd_t* cmd, nvm_cpl_t* cpl)
{
    if (!ref || !cmd || !cpl) return EINVAL;
    std::lock_guard<std::mutex> g(ref->lock);
    nvm_cmd_t* slot = nvm_sq_enqueue(&ref->asq);
    if (!slot) return EAGAIN;
    uint16_t cid = ref->next_cid++;
    cmd->dword[0] = (cmd->dword[0] & 0xffffu) | ((uint32_t)cid << 16);
    memcpy(slot, cmd, sizeof(nvm_cmd_t));
    nvm_sq_submit(&ref->asq);
    nvm_cpl_t* c = nvm_cq_dequeue_block(&ref->acq, ref->ctrl->handle.timeout);
    if (!c) return ETIME;
    nvm_sq_update(&ref->asq);
    for (int i = 0; i < 4; i++) cpl->dword[i] = c->dword[i];
    nvm_cq_update(&ref->acq);
    if ((cpl->dword[3] & 0xffffu) != cid) return EBADMSG;
    return NVM_ERR_PACK(cpl, 0);
}

// ---- admin commands ----
static void admin_cmd(nvm_cmd_t* c, uint8_t opcode, uint32_t nsid)
{
    memset(c, 0, sizeof(*c));
    nvm_cmd_header(c, 0, opcode, nsid);
}

int nvm_admin_ctrl_info(nvm_aq_ref ref, struct nvm_ctrl_info* info, void* buffer, uint64_t ioaddr)
{
    if (!ref || !info || !buffer || !ioaddr) return EINVAL;
    const nvm_ctrl_t* ctrl = &ref->ctrl->handle;
    nvm_cmd_t cmd; nvm_cpl_t cpl;
    memset(info, 0, sizeof(*info));
    memset(buffer, 0, 4096);
    admin_cmd(&cmd, NVM_ADMIN_IDENTIFY, 0);
    nvm_cmd_data_ptr(&cmd, ioaddr, 0);
    cmd.dword[10] = 1;      // CNS: identify controller
    int err = nvm_raw_rpc(ref, &cmd, &cpl);
    if (err) return err;
    const unsigned char* b = (const unsigned char*)buffer;
    uint64_t cap = rd64(ctrl->mm_ptr, 0x00);
    info->nvme_version = rd32(ctrl->mm_ptr, 0x08);
    info->page_size = ctrl->page_size;
    info->db_stride = (size_t)4 << ctrl->dstrd;
    info->timeout = ctrl->timeout;
    info->contiguous = (int)_RB(cap, 16, 16);
    info->max_entries = (uint16_t)(ctrl->max_qs - 1);
    memcpy(info->pci_vendor, b, 4);
    memcpy(info->serial_no, b + 4, 20);
    memcpy(info->model_no, b + 24, 40);
    memcpy(info->firmware, b + 64, 8);
    info->max_data_pages = b[77] ? (size_t)1 << b[77] : 0;
    info->max_data_size = info->max_data_pages * ((size_t)1 << (12 + _RB(cap, 51, 48)));
    info->sq_entry_size = (size_t)1 << (b[512] & 0xf);
    info->cq_entry_size = (size_t)1 << (b[513] & 0xf);
    uint16_t maxcmd; memcpy(&maxcmd, b + 514, 2);
    uint32_t nn; memcpy(&nn, b + 516, 4);
    info->max_out_cmds = maxcmd;
    info->max_n_ns = nn;
    return 0;
}

int nvm_admin_ns_info(nvm_aq_ref ref, struct nvm_ns_info* info, uint32_t ns_id, void* buffer, uint64_t ioaddr)
{
    if (!ref || !info || !buffer || !ioaddr) return EINVAL;
    nvm_cmd_t cmd; nvm_cpl_t cpl;
    memset(info, 0, sizeof(*info));
    memset(buffer, 0, 4096);
    admin_cmd(&cmd, NVM_ADMIN_IDENTIFY, ns_id);
    nvm_cmd_data_ptr(&cmd, ioaddr, 0);
    cmd.dword[10] = 0;      // CNS: identify namespace
    int err = nvm_raw_rpc(ref, &cmd, &cpl);
    if (err) return err;
    const unsigned char* b = (const unsigned char*)buffer;
    uint64_t v;
    info->ns_id = ns_id;
    memcpy(&v, b + 0, 8);  info->size = v;
    memcpy(&v, b + 8, 8);  info->capacity = v;
    memcpy(&v, b + 16, 8); info->utilization = v;
    uint32_t lbaf; memcpy(&lbaf, b + 128 + 4 * (b[26] & 0xf), 4);
    info->lba_data_size = (size_t)1 << _RB(lbaf, 23, 16);
    info->metadata_size = _RB(lbaf, 15, 0);
    return 0;
}

static int num_queues(nvm_aq_ref ref, uint8_t opcode, uint16_t* n_cqs, uint16_t* n_sqs)
{
    nvm_cmd_t cmd; nvm_cpl_t cpl;
    admin_cmd(&cmd, opcode, 0);
    cmd.dword[10] = 0x07;   // feature: number of queues
    if (opcode == NVM_ADMIN_SET_FEATURES) cmd.dword[11] = ((uint32_t)(*n_cqs - 1) << 16) | (uint32_t)(*n_sqs - 1);
    int err = nvm_raw_rpc(ref, &cmd, &cpl);
    if (err) return err;
    *n_sqs = (uint16_t)((cpl.dword[0] & 0xffff) + 1);
    *n_cqs = (uint16_t)((cpl.dword[0] >> 16) + 1);
    return 0;
}

int nvm_admin_set_num_queues(nvm_aq_ref ref, uint16_t n_cqs, uint16_t n_sqs)
{
    if (!ref || !n_cqs || !n_sqs) return EINVAL;
    return num_queues(ref, NVM_ADMIN_SET_FEATURES, &n_cqs, &n_sqs);
}

int nvm_admin_get_num_queues(nvm_aq_ref ref, uint16_t* n_cqs, uint16_t* n_sqs)
{
    if (!ref || !n_cqs || !n_sqs) return EINVAL;
    return num_queues(ref, NVM_ADMIN_GET_FEATURES, n_cqs, n_sqs);
}

int nvm_admin_request_num_queues(nvm_aq_ref ref, uint16_t* n_cqs, uint16_t* n_sqs)
{
    if (!ref || !n_cqs || !n_sqs || !*n_cqs || !*n_sqs) return EINVAL;
    return num_queues(ref, NVM_ADMIN_SET_FEATURES, n_cqs, n_sqs);
}

static int create_queue(nvm_aq_ref ref, nvm_queue_t* q, bool is_cq, uint16_t id, uint16_t cqid, const nvm_dma_t* dma, size_t page_offset, size_t qs, bool need_prp)
{
    if (!ref || !q || id == 0 || !dma || qs < 2 || qs > 65536 || need_prp) return EINVAL;
    if (!dma->vaddr || page_offset >= dma->n_ioaddrs) return EINVAL;
    size_t es = is_cq ? sizeof(nvm_cpl_t) : sizeof(nvm_cmd_t);
    size_t pages = NVM_PAGE_ALIGN(qs * es, dma->page_size) / dma->page_size;
    if (page_offset + pages > dma->n_ioaddrs) return EINVAL;
    if (pages > 1 && !dma->contiguous) return EINVAL;     // queue memory must be physically contiguous (CQR)
    const nvm_ctrl_t* ctrl = &ref->ctrl->handle;
    int err = nvm_queue_clear(q, ctrl, is_cq, id, (uint32_t)qs, dma->local, NVM_DMA_OFFSET(dma, page_offset), dma->ioaddrs[page_offset]);
    if (err) return err;
    nvm_cmd_t cmd; nvm_cpl_t cpl;
    admin_cmd(&cmd, is_cq ? NVM_ADMIN_CREATE_CQ : NVM_ADMIN_CREATE_SQ, 0);
    nvm_cmd_data_ptr(&cmd, q->ioaddr, 0);
    cmd.dword[10] = ((uint32_t)(qs - 1) << 16) | id;
    cmd.dword[11] = is_cq ? 0x1u : (((uint32_t)cqid << 16) | 0x1u);   // PC = 1; CQ: interrupts disabled
    return nvm_raw_rpc(ref, &cmd, &cpl);
}

static int delete_queue(nvm_aq_ref ref, nvm_queue_t* q, bool is_cq)
{
    if (!ref || !q || q->no == 0) return EINVAL;
    nvm_cmd_t cmd; nvm_cpl_t cpl;
    admin_cmd(&cmd, is_cq ? NVM_ADMIN_DELETE_CQ : NVM_ADMIN_DELETE_SQ, 0);
    cmd.dword[10] = q->no;
    int err = nvm_raw_rpc(ref, &cmd, &cpl);
    if (!err) q->db = nullptr;
    return err;
}

int nvm_admin_get_log_page(nvm_aq_ref ref, uint32_t ns_id, void* ptr, uint64_t ioaddr, uint8_t log_id, uint64_t log_offset)
{
    if (!ref || !ptr || !ioaddr || (log_offset & 3)) return EINVAL;
    nvm_cmd_t cmd; nvm_cpl_t cpl;
    admin_cmd(&cmd, NVM_ADMIN_GET_LOG_PAGE, ns_id);
    nvm_cmd_data_ptr(&cmd, ioaddr, 0);
    cmd.dword[10] = ((uint32_t)(1024 - 1) << 16) | log_id;    // one 4 KiB page of dwords
    cmd.dword[12] = (uint32_t)log_offset;
    cmd.dword[13] = (uint32_t)(log_offset >> 32);
    return nvm_raw_rpc(ref, &cmd, &cpl);
}

// ---- DMA descriptors ----
int nvm_dma_map(nvm_dma_t** map, const nvm_ctrl_t* ctrl, void* vaddr, size_t page_size, size_t n_pages, const uint64_t* page_addrs)
{
    if (!map) return EINVAL;
    *map = nullptr;
    if (!ctrl || !page_size || !n_pages || !page_addrs) return EINVAL;
    size_t cps = ctrl->page_size;
    if (page_size % cps && cps % page_size) return EINVAL;
    size_t n_io = n_pages * page_size / cps;
    if (!n_io) return EINVAL;
    DmaBox* b = (DmaBox*)calloc(1, sizeof(DmaBox) + n_io * sizeof(uint64_t));
    if (!b) return ENOMEM;
    b->ctrl = box_of(ctrl);
    b->map.vaddr = vaddr;
    b->map.local = 1;
    b->map.page_size = cps;
    b->map.n_ioaddrs = n_io;
    bool contiguous = true;
    for (size_t i = 0; i < n_io; i++) {
        size_t byte = i * cps;
        uint64_t a = page_addrs[byte / page_size] + byte % page_size;
        if (a & (cps - 1)) { free(b); return EINVAL; }
        b->map.ioaddrs[i] = a;
        contiguous &= i == 0 || a == b->map.ioaddrs[i - 1] + cps;
    }
    b->map.contiguous = contiguous;
    ctrl_get(b->ctrl);
    *map = &b->map;
    return 0;
}

static int map_identity(nvm_dma_t** map, const nvm_ctrl_t* ctrl, void* vaddr, size_t size)
{
    if (!map) return EINVAL;
    *map = nullptr;
    if (!ctrl || !vaddr || !size || ((uintptr_t)vaddr & (ctrl->page_size - 1))) return EINVAL;
    // one "page" covering the whole region: bus address = virtual address
    size_t span = NVM_PAGE_ALIGN(size, ctrl->page_size);
    uint64_t a = (uint64_t)(uintptr_t)vaddr;
    return nvm_dma_map(map, ctrl, vaddr, span, 1, &a);
}

int nvm_dma_map_host(nvm_dma_t** map, const nvm_ctrl_t* ctrl, void* vaddr, size_t size) { return map_identity(map, ctrl, vaddr, size); }
int nvm_dma_map_device(nvm_dma_t** map, const nvm_ctrl_t* ctrl, void* devptr, size_t size) { return map_identity(map, ctrl, devptr, size); }

int nvm_dma_create(nvm_dma_t** map, const nvm_ctrl_t* ctrl, size_t size)
{
    if (!map) return EINVAL;
    *map = nullptr;
    if (!ctrl || !size) return EINVAL;
    size_t span = NVM_PAGE_ALIGN(size, ctrl->page_size);
    void* mem = nullptr;
    if (posix_memalign(&mem, ctrl->page_size, span)) return ENOMEM;
    memset(mem, 0, span);
    int err = map_identity(map, ctrl, mem, span);
    if (err) { free(mem); return err; }
    box_of(*map)->owned = mem;
    return 0;
}

int nvm_dma_remap(nvm_dma_t** new_map, const nvm_dma_t* other)
{
    if (!new_map) return EINVAL;
    *new_map = nullptr;
    if (!other) return EINVAL;
    return nvm_dma_map(new_map, &box_of(other)->ctrl->handle, other->vaddr, other->page_size, other->n_ioaddrs, other->ioaddrs);
}

void nvm_dma_unmap(nvm_dma_t* map)
{
    if (!map) return;
    DmaBox* b = box_of(map);
    ctrl_put(b->ctrl);
    free(b->owned);
    free(b);
}

const nvm_ctrl_t* nvm_ctrl_from_dma(const nvm_dma_t* dma) { return dma ? &box_of(dma)->ctrl->handle : nullptr; }

// ---- status text ----
const char* nvm_strerror(int status)
{
    if (status >= 0) return status ? strerror(status) : "Success";
    int sct = NVM_ERR_UNPACK_SCT(status), sc = NVM_ERR_UNPACK_SC(status);
    if (sct == 0) switch (sc) {
        case 0x00: return "Success";
        case 0x01: return "Invalid command opcode";
        case 0x02: return "Invalid field in command";
        case 0x03: return "Command ID conflict";
        case 0x04: return "Data transfer error";
        case 0x06: return "Internal error";
        case 0x07: return "Command abort requested";
        case 0x0b: return "Invalid namespace or format";
        case 0x80: return "LBA out of range";
        case 0x81: return "Capacity exceeded";
        case 0x82: return "Attempted write to read-only range";
        default:   return "Unknown generic command status";
    }
    if (sct == 1) switch (sc) {
        case 0x00: return "Completion queue invalid";
        case 0x01: return "Invalid queue identifier";
        case 0x02: return "Invalid queue size";
        case 0x03: return "Abort command limit exceeded";
        case 0x08: return "Invalid interrupt vector";
        case 0x09: return "Invalid log page";
        case 0x0c: return "Invalid queue deletion";
        default:   return "Unknown command specific status";
    }
    if (sct == 2) return "Media or data integrity error";
    return "Unknown status code type";
}

} // extern "C"

extern "C" {
int nvm_admin_cq_create(nvm_aq_ref ref, nvm_queue_t* cq, uint16_t id, const nvm_dma_t* dma, size_t page_offset, size_t qs, bool need_prp)
{
    return create_queue(ref, cq, true, id, 0, dma, page_offset, qs, need_prp);
}

int nvm_admin_sq_create(nvm_aq_ref ref, nvm_queue_t* sq, const nvm_queue_t* cq, uint16_t id, const nvm_dma_t* dma, size_t page_offset, size_t qs, bool need_prp)
{
    if (!cq) return EINVAL;
    return create_queue(ref, sq, false, id, cq->no, dma, page_offset, qs, need_prp);
}

int nvm_admin_sq_set_sealed(nvm_aq_ref ref, nvm_queue_t* sq)
{
    if (!ref || !sq || sq->no == 0) return EINVAL;
    nvm_cmd_t cmd; nvm_cpl_t cpl;
    admin_cmd(&cmd, 0, 0);
    cmd.dword[0] = NVM_ADMIN_VS_SEAL_SQ;        /* full 8-bit opcode: nvm_cmd_header keeps only the low seven bits */
    cmd.dword[10] = sq->no;
    int err = nvm_raw_rpc(ref, &cmd, &cpl);
    if (!err) sq->sealed = 1;
    return err;
}

int nvm_admin_cq_delete(nvm_aq_ref ref, nvm_queue_t* cq) { return delete_queue(ref, cq, true); }
int nvm_admin_sq_delete(nvm_aq_ref ref, nvm_queue_t* sq, const nvm_queue_t* cq) { (void)cq; return delete_queue(ref, sq, false); }
} // extern "C"
