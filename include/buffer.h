/*
 * Owning handles for device buffers and controller-visible (DMA) memory.
 * Replaces include/buffer.h of the reference (createDma host :149-180 and
 * device :183-260 variants, createBuffer :95-146, DmaPtr/BufferPtr :31-36).
 *
 * The reference pins GPU pages for the SSD through its kernel module.  Here a
 * DMA region is memory that both the GPU and the controller can address:
 *   - host-pinned memory (hipHostMalloc: fine-grained, mapped into the GPU at
 *     the same address), always available; or
 *   - device memory through its host-visible large-BAR alias, when the caller
 *     asks for it (BAM_DMA_DEVICE) and the platform exposes VRAM to the CPU.
 * Either way the bus address handed to the controller is the virtual address.
 */
#ifndef __BAM_BUFFER_H__
#define __BAM_BUFFER_H__
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include "nvm_dma.h"
#include "nvm_error.h"
#include "nvm_types.h"
#include "nvm_util.h"
#include "util.h"

typedef std::shared_ptr<nvm_dma_t> DmaPtr;
typedef std::shared_ptr<void> BufferPtr;

enum bam_dma_place { BAM_DMA_HOST = 0, BAM_DMA_DEVICE = 1 };

/* zero-filled device buffer */
inline BufferPtr createBuffer(size_t size, int hipDevice)
{
    void* p = nullptr;
    hip_err_chk(hipSetDevice(hipDevice));
    hip_err_chk(hipMalloc(&p, size ? size : 1));
    hip_err_chk(hipMemset(p, 0, size ? size : 1));
    return BufferPtr(p, [](void* q) { (void)hipFree(q); });
}

/* zero-filled host-pinned buffer the GPU can address */
inline BufferPtr createHostBuffer(size_t size)
{
    void* p = nullptr;
    hip_err_chk(hipHostMalloc(&p, size ? size : 1, hipHostMallocMapped));
    memset(p, 0, size ? size : 1);
    return BufferPtr(p, [](void* q) { (void)hipHostFree(q); });
}

/* DMA region of `size` bytes (rounded up to controller pages), zero-filled */
inline DmaPtr createDma(const nvm_ctrl_t* ctrl, size_t size, int hipDevice = -1, bam_dma_place place = BAM_DMA_HOST)
{
    size = NVM_PAGE_ALIGN(size, ctrl->page_size);
    void* mem = nullptr;
    nvm_dma_t* dma = nullptr;
    int status;
    if (place == BAM_DMA_DEVICE) {
        hip_err_chk(hipSetDevice(hipDevice));
        hip_err_chk(hipMalloc(&mem, size));
        hip_err_chk(hipMemset(mem, 0, size));
        hip_err_chk(hipDeviceSynchronize());
        status = nvm_dma_map_device(&dma, ctrl, mem, size);
    } else {
        hip_err_chk(hipHostMalloc(&mem, size, hipHostMallocMapped));
        memset(mem, 0, size);
        status = nvm_dma_map_host(&dma, ctrl, mem, size);
    }
    if (!nvm_ok(status)) {
        if (place == BAM_DMA_DEVICE) (void)hipFree(mem); else (void)hipHostFree(mem);
        throw std::runtime_error(std::string("Failed to map DMA memory: ") + nvm_strerror(status));
    }
    return DmaPtr(dma, [mem, place](nvm_dma_t* d) {
        nvm_dma_unmap(d);
        if (place == BAM_DMA_DEVICE) (void)hipFree(mem); else (void)hipHostFree(mem);
    });
}
#endif
