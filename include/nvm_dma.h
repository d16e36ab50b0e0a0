/*
 * DMA mapping descriptors.  Replaces include/nvm_dma.h of the reference
 * (nvm_dma_map :35-40, nvm_dma_remap :48, nvm_dma_unmap :58,
 * nvm_dma_map_host :69, nvm_dma_map_device :85, nvm_dma_create :147).
 * Without an IOMMU-programming kernel module a "bus address" is whatever the
 * controller can dereference: for the software target that is a host virtual
 * address, so map_host/map_device use identity addresses.
 */
#ifndef __NVM_DMA_H__
#define __NVM_DMA_H__
#include <stddef.h>
#include <stdint.h>
#include "nvm_types.h"
#ifdef __cplusplus
extern "C" {
#endif
int  nvm_dma_map(nvm_dma_t** map, const nvm_ctrl_t* ctrl, void* vaddr, size_t page_size, size_t n_pages, const uint64_t* page_addrs);
int  nvm_dma_remap(nvm_dma_t** new_map, const nvm_dma_t* other_map);
void nvm_dma_unmap(nvm_dma_t* map);
/* identity mapping of host memory the controller can reach */
int  nvm_dma_map_host(nvm_dma_t** map, const nvm_ctrl_t* ctrl, void* vaddr, size_t size);
/* identity mapping of device memory through its host-visible alias `devptr` */
int  nvm_dma_map_device(nvm_dma_t** map, const nvm_ctrl_t* ctrl, void* devptr, size_t size);
/* allocate page-aligned host memory and map it; freed by nvm_dma_unmap */
int  nvm_dma_create(nvm_dma_t** map, const nvm_ctrl_t* ctrl, size_t size);
const nvm_ctrl_t* nvm_ctrl_from_dma(const nvm_dma_t* dma);
#ifdef __cplusplus
}
#endif
#endif
