/*
 * Status packing: 0 = ok, > 0 = errno, < 0 = -(SCT << 8 | SC) of an NVMe completion.
 * Replaces include/nvm_error.h of the reference (:17-59 macros, :67 nvm_strerror).
 */
#ifndef __NVM_ERROR_H__
#define __NVM_ERROR_H__
#include <stdint.h>
#include "nvm_types.h"
#include "nvm_util.h"

#define NVM_ERR_SCT(cpl)            ((uint8_t)_RB(*NVM_CPL_STATUS(cpl), 11, 9))
#define NVM_ERR_SC(cpl)             ((uint8_t)_RB(*NVM_CPL_STATUS(cpl), 8, 1))
#define NVM_ERR_DNR(cpl)            (!!_RB(*NVM_CPL_STATUS(cpl), 15, 15))
#define NVM_ERR_MORE(cpl)           (!!_RB(*NVM_CPL_STATUS(cpl), 14, 14))
#define NVM_ERR_STATUS(cpl)         ((int)((cpl) != NULL ? -((NVM_ERR_SCT(cpl) << 8) | NVM_ERR_SC(cpl)) : 0))
#define NVM_ERR_OK(cpl)             (!NVM_ERR_SCT(cpl) && !NVM_ERR_SC(cpl))
#define NVM_ERR_PACK(cpl, err)      ((int)((err) != 0 ? (err) : NVM_ERR_STATUS(cpl)))
#define NVM_ERR_UNPACK_ERRNO(status) (((status) > 0) ? (status) : 0)
#define NVM_ERR_UNPACK_SCT(status)   (((status) < 0) ? (((-(status)) >> 8) & 0xff) : 0)
#define NVM_ERR_UNPACK_SC(status)    (((status) < 0) ? ((-(status)) & 0xff) : 0)
#define nvm_ok(status)              (!(status))

#ifdef __cplusplus
extern "C" {
#endif
/* strerror() for positive values, NVMe status text for negative ones */
const char* nvm_strerror(int status);
#ifdef __cplusplus
}
#endif
#endif /* __NVM_ERROR_H__ */
