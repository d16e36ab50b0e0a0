/*
 * Bit-field, register and descriptor helper macros.
 * Replaces the macro part of include/nvm_util.h of the reference (:21-26 masks,
 * :88-100 _RB/_WB/_REG, :106-170 page/block/DMA helpers, :200-230 CQE accessors).
 * The SIMT identity helpers (lane_id, get_smid, :276-295) are wave64 versions
 * and live in bam_wave.h.
 */
#ifndef __NVM_UTIL_H__
#define __NVM_UTIL_H__
#include <stddef.h>
#include <stdint.h>
#include "nvm_types.h"

#define _NVM_MASK(num_bits)        ((1ULL << (num_bits)) - 1)
#define _NVM_MASK_PART(hi, lo)     (_NVM_MASK((hi) + 1) - _NVM_MASK(lo))

/* read bits hi..lo of v / place v into bits hi..lo */
#define _RB(v, hi, lo)             (((v) & _NVM_MASK_PART((hi), (lo))) >> (lo))
#define _WB(v, hi, lo)             (((uint64_t)(v) << (lo)) & _NVM_MASK_PART((hi), (lo)))
#define _REG(p, offs, bits)        ((volatile uint##bits##_t*)(((volatile unsigned char*)((volatile void*)(p))) + (offs)))

#define NVM_PAGE_ALIGN(size, page_size)   (((size) + (page_size) - 1) & ~((uint64_t)(page_size) - 1))
#define NVM_ADDR_MASK(addr, page_size)    ((addr) & ~((uint64_t)(page_size) - 1))
#define NVM_PAGE_TO_BLOCK(page_size, block_size, pageno)   (((page_size) * (pageno)) / (block_size))
#define NVM_BLOCK_TO_PAGE(page_size, block_size, blockno)  (((block_size) * (blockno)) / (page_size))
#define NVM_CQ_PAGES(dma, n)       (NVM_PAGE_ALIGN((n) * sizeof(nvm_cpl_t), (dma)->page_size) / (dma)->page_size)
#define NVM_SQ_PAGES(dma, n)       (NVM_PAGE_ALIGN((n) * sizeof(nvm_cmd_t), (dma)->page_size) / (dma)->page_size)

/* pointer to page number `pageno` of a DMA region */
#define NVM_DMA_OFFSET(dma_ptr, pageno)   ((void*)(((unsigned char*)(dma_ptr)->vaddr) + (dma_ptr)->page_size * (pageno)))

/* CQE field accessors (NVMe completion entry: DW2 = SQHD | SQID<<16, DW3 = CID | P<<16 | status<<17) */
#define NVM_CPL_CID(cpl)           _REG(cpl, 12, 16)
#define NVM_CPL_SQHD(cpl)          _REG(cpl,  8, 16)
#define NVM_CPL_SQID(cpl)          _REG(cpl, 10, 16)
#define NVM_CPL_STATUS(cpl)        _REG(cpl, 14, 16)

#endif /* __NVM_UTIL_H__ */
