/*
 * Controller handle.  Replaces include/nvm_ctrl.h of the reference
 * (nvm_ctrl_init :36, nvm_raw_ctrl_init :53, nvm_ctrl_free :60,
 * nvm_raw_ctrl_reset :76).  The register window comes from the software NVMe
 * target (nvmt.h), from a caller that has mapped a real BAR0, or from a
 * descriptor that nvm_ctrl_init maps itself.
 */
#ifndef __NVM_CTRL_H__
#define __NVM_CTRL_H__
#include <stddef.h>
#include <stdint.h>
#include "nvm_types.h"

#define NVM_CTRL_MEM_MINSIZE 0x2000

#ifdef __cplusplus
extern "C" {
#endif
/* Map the first NVM_CTRL_MEM_MINSIZE bytes behind `fd` shared and read-write (BAR0 of a device node or sysfs resource
 * file) and build a handle from the registers found there; the mapping goes with the handle's last reference.  0 or
 * errno (EBADF not a descriptor, ENODEV/EACCES it cannot be mapped, EINVAL/ERANGE as nvm_raw_ctrl_init). */
int nvm_ctrl_init(nvm_ctrl_t** ctrl, int fd);
/* Read CAP from a mapped register window and build a handle.  0 or errno
 * (EINVAL window too small, ERANGE host page size outside MPSMIN..MPSMAX). */
int nvm_raw_ctrl_init(nvm_ctrl_t** ctrl, volatile void* mm_ptr, size_t mm_size);
/* Drop one reference; the handle is freed with the last one. */
void nvm_ctrl_free(nvm_ctrl_t* ctrl);
/* CC.EN 1->0, wait RDY=0, program AQA/ACQ/ASQ, CC.EN=1, wait RDY=1.  ETIME on controller timeout. */
int nvm_raw_ctrl_reset(const nvm_ctrl_t* ctrl, uint64_t acq_ioaddr, uint64_t asq_ioaddr);
#ifdef __cplusplus
}
#endif
#endif
