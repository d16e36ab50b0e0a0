/*
 * Admin queue pair.  Replaces include/nvm_aq.h (nvm_aq_create :23-25,
 * nvm_aq_destroy :38) and include/nvm_rpc.h (nvm_raw_rpc :53,
 * nvm_rpc_unbind :33) of the reference.
 */
#ifndef __NVM_AQ_H__
#define __NVM_AQ_H__
#include "nvm_types.h"
#ifdef __cplusplus
extern "C" {
#endif
/* Reset the controller with admin queues placed in pages 0 (ACQ) and 1 (ASQ) of dma_window. */
int  nvm_aq_create(nvm_aq_ref* ref, const nvm_ctrl_t* ctrl, const nvm_dma_t* dma_window);
void nvm_aq_destroy(nvm_aq_ref ref);
/* Execute one admin command and wait for its completion (serialized per reference).
 * 0, errno (ETIME on controller timeout) or packed NVMe status. */
int  nvm_raw_rpc(nvm_aq_ref ref, nvm_cmd_t* cmd, nvm_cpl_t* cpl);
void nvm_rpc_unbind(nvm_aq_ref ref);
const nvm_ctrl_t* nvm_ctrl_from_aq_ref(nvm_aq_ref ref);
#ifdef __cplusplus
}
#endif
#endif
