/*
 * NVMe command opcodes and SQE encoders.
 * Replaces include/nvm_cmd.h of the reference: opcode enums :25-47,
 * nvm_cmd_header :54-58, nvm_cmd_data_ptr :66-74, nvm_cmd_rw_blks :82-87,
 * nvm_prp_list :106-140.  Layout is the NVMe 1.x submission entry.
 */
#ifndef __NVM_COMMAND_H__
#define __NVM_COMMAND_H__
#include <stdint.h>
#include "nvm_types.h"
#include "nvm_util.h"

#define NVM_CMD_NS_ALL                  0xffffffff
#define NVM_CMD_OPCODE(gen, fun, data)  ((uint8_t)(_WB((gen), 7, 7) | _WB((fun), 6, 2) | _WB((data), 1, 0)))

enum nvm_io_command_set
{
    NVM_IO_FLUSH            = 0x00,
    NVM_IO_WRITE            = 0x01,
    NVM_IO_READ             = 0x02,
    NVM_IO_WRITE_ZEROES     = 0x08
};

enum nvm_admin_command_set
{
    NVM_ADMIN_DELETE_SQ     = 0x00,
    NVM_ADMIN_CREATE_SQ     = 0x01,
    NVM_ADMIN_GET_LOG_PAGE  = 0x02,
    NVM_ADMIN_DELETE_CQ     = 0x04,
    NVM_ADMIN_CREATE_CQ     = 0x05,
    NVM_ADMIN_IDENTIFY      = 0x06,
    NVM_ADMIN_ABORT         = 0x08,
    NVM_ADMIN_SET_FEATURES  = 0x09,
    NVM_ADMIN_GET_FEATURES  = 0x0A,
    NVM_ADMIN_VS_SEAL_SQ    = 0xC1      /* vendor specific: CDW10[15:0] = SQ id whose entries are sealed from now on */
};

/* DW0 (opcode, FUSE = PSDT = 0, CID) and DW1 (NSID) */
__host__ __device__ static inline
void nvm_cmd_header(nvm_cmd_t* cmd, uint16_t cid, uint8_t opcode, uint32_t ns_id)
{
    cmd->dword[0] = ((uint32_t)cid << 16) | (uint32_t)(opcode & 0x7f);
    cmd->dword[1] = ns_id;
}

/* DPTR as two PRP entries (DW6-9); clears PSDT/FUSE */
__host__ __device__ static inline
void nvm_cmd_data_ptr(nvm_cmd_t* cmd, uint64_t prp1, uint64_t prp2)
{
    cmd->dword[0] &= ~((0x03u << 14) | (0x03u << 8));
    cmd->dword[6] = (uint32_t)prp1;
    cmd->dword[7] = (uint32_t)(prp1 >> 32);
    cmd->dword[8] = (uint32_t)prp2;
    cmd->dword[9] = (uint32_t)(prp2 >> 32);
}

/* SLBA (DW10-11) and zero-based NLB (DW12[15:0]) */
__host__ __device__ static inline
void nvm_cmd_rw_blks(nvm_cmd_t* cmd, uint64_t start_lba, uint16_t n_blks)
{
    cmd->dword[10] = (uint32_t)start_lba;
    cmd->dword[11] = (uint32_t)(start_lba >> 32);
    cmd->dword[12] = (cmd->dword[12] & 0xffff0000u) | ((uint32_t)(n_blks - 1) & 0xffffu);
}

/*
 * Sealed submission entries (extension; no counterpart in the reference).
 *
 * A queue whose entries are written by one agent and fetched by another over
 * an interconnect that may reorder posted writes (a GPU filling a ring in host
 * memory for the software target) cannot rely on "entry first, doorbell
 * second" arriving in that order.  On a sealed SQ the writer stores the
 * entry's absolute sequence number (its slot ticket) in CDW2 and a checksum of
 * the other fifteen dwords, keyed by that number, in CDW3 (both reserved in
 * NVM read/write/flush commands); the fetching side takes an entry only when
 * both match, so an entry that is stale, torn or not yet complete is simply
 * looked at again later.
 */
__host__ __device__ static inline
uint32_t nvm_cmd_seal_value(const nvm_cmd_t* cmd, uint32_t ticket)
{
    uint32_t h = ticket * 0x9E3779B1u + 0x7F4A7C15u;
    for (int i = 0; i < 16; i++) {
        if (i == 3) continue;
        h = (h ^ cmd->dword[i]) * 0x85EBCA6Bu;
        h ^= h >> 13;
    }
    return h | 1u;
}

__host__ __device__ static inline
void nvm_cmd_seal(nvm_cmd_t* cmd, uint32_t ticket)
{
    cmd->dword[2] = ticket;
    cmd->dword[3] = nvm_cmd_seal_value(cmd, ticket);
}

__host__ __device__ static inline
int nvm_cmd_seal_ok(const nvm_cmd_t* cmd, uint32_t ticket)
{
    return cmd->dword[2] == ticket && cmd->dword[3] == nvm_cmd_seal_value(cmd, ticket);
}

/*
 * Fill one PRP-list page with the bus addresses of `n_pages` data pages.  When
 * more pages remain than the list holds, the last entry is left for chaining.
 * Returns the number of entries written.
 */
__host__ __device__ static inline
size_t nvm_prp_list(const nvm_prp_list_t* list, size_t n_pages, const uint64_t* ioaddrs)
{
    size_t cap = list->page_size / sizeof(uint64_t);
    size_t n = n_pages <= cap ? n_pages : cap - 1;
    volatile uint64_t* e = (volatile uint64_t*)list->vaddr;
    for (size_t i = 0; i < n; i++) e[i] = ioaddrs[i];
    return n;
}

#endif /* __NVM_COMMAND_H__ */
