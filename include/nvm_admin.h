/*
 * Admin commands.  Replaces include/nvm_admin.h of the reference
 * (ctrl_info :18-21, ns_info :28-32, set/get/request_num_queues :39-51,
 * cq_create :63-69, cq_delete :76, sq_create :89-96, sq_delete :104-106,
 * get_log_page :112-117).  All return 0, an errno, or a packed NVMe status.
 */
#ifndef __NVM_ADMIN_H__
#define __NVM_ADMIN_H__
#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>
#include "nvm_types.h"
#ifdef __cplusplus
#define NVM_DEFAULT(x) = x
extern "C" {
#else
#define NVM_DEFAULT(x)
#endif
int nvm_admin_ctrl_info(nvm_aq_ref ref, struct nvm_ctrl_info* info, void* buffer, uint64_t ioaddr);
int nvm_admin_ns_info(nvm_aq_ref ref, struct nvm_ns_info* info, uint32_t ns_id, void* buffer, uint64_t ioaddr);
int nvm_admin_set_num_queues(nvm_aq_ref ref, uint16_t n_cqs, uint16_t n_sqs);
int nvm_admin_get_num_queues(nvm_aq_ref ref, uint16_t* n_cqs, uint16_t* n_sqs);
int nvm_admin_request_num_queues(nvm_aq_ref ref, uint16_t* n_cqs, uint16_t* n_sqs);
int nvm_admin_cq_create(nvm_aq_ref ref, nvm_queue_t* cq, uint16_t id, const nvm_dma_t* dma, size_t page_offset, size_t qs, bool need_prp NVM_DEFAULT(false));
int nvm_admin_cq_delete(nvm_aq_ref ref, nvm_queue_t* cq);
int nvm_admin_sq_create(nvm_aq_ref ref, nvm_queue_t* sq, const nvm_queue_t* cq, uint16_t id, const nvm_dma_t* dma, size_t page_offset, size_t qs, bool need_prp NVM_DEFAULT(false));
int nvm_admin_sq_delete(nvm_aq_ref ref, nvm_queue_t* sq, const nvm_queue_t* cq);
/* extension: from now on the controller only takes entries of `sq` that pass nvm_cmd_seal_ok (software target only) */
int nvm_admin_sq_set_sealed(nvm_aq_ref ref, nvm_queue_t* sq);
int nvm_admin_get_log_page(nvm_aq_ref ref, uint32_t ns_id, void* ptr, uint64_t ioaddr, uint8_t log_id, uint64_t log_offset);
#ifdef __cplusplus
}
#endif
#endif
