/*
 * Single-threaded host-side queue operations (admin path, host test clients).
 * Replaces include/nvm_queue.h of the reference (nvm_queue_clear :30-37,
 * nvm_queue_reset :50, nvm_sq_enqueue :64-90, nvm_cq_poll :156-176,
 * nvm_cq_dequeue :189-209, nvm_cq_dequeue_block :220, nvm_sq_submit :233-250,
 * nvm_sq_update :260-269, nvm_cq_update :279-291).  The concurrent device-side
 * protocol is in nvm_parallel_queue.h.
 */
#ifndef __NVM_QUEUE_H__
#define __NVM_QUEUE_H__
#include <stdbool.h>
#include <stdint.h>
#include "nvm_types.h"
#include "nvm_util.h"
#ifdef __cplusplus
extern "C" {
#endif
/* EINVAL if qs < 2 or not a power of two, or vaddr == NULL */
int  nvm_queue_clear(nvm_queue_t* q, const nvm_ctrl_t* ctrl, bool cq, uint16_t no, uint32_t qs, bool local, volatile void* vaddr, uint64_t ioaddr);
void nvm_queue_reset(nvm_queue_t* q);
/* block up to timeout ms for the next completion; NULL on timeout */
nvm_cpl_t* nvm_cq_dequeue_block(nvm_queue_t* cq, uint64_t timeout);
#ifdef __cplusplus
}
#endif

/* next free SQ slot or NULL when the queue is full (tail + 1 == head) */
static inline nvm_cmd_t* nvm_sq_enqueue(nvm_queue_t* sq)
{
    if (((sq->tail + 1) & sq->qs_minus_1) == (sq->head & sq->qs_minus_1)) return NULL;
    nvm_cmd_t* c = ((nvm_cmd_t*)sq->vaddr) + (sq->tail & sq->qs_minus_1);
    sq->tail++;
    return c;
}

/* completion at the head if its phase tag is current, else NULL */
static inline nvm_cpl_t* nvm_cq_poll(const nvm_queue_t* cq)
{
    nvm_cpl_t* c = ((nvm_cpl_t*)cq->vaddr) + (cq->head & cq->qs_minus_1);
    uint32_t dw3 = __atomic_load_n((const uint32_t*)&c->dword[3], __ATOMIC_ACQUIRE);
    return (((dw3 >> 16) & 1u) == (uint32_t)(cq->phase & 1)) ? c : NULL;
}

static inline nvm_cpl_t* nvm_cq_dequeue(nvm_queue_t* cq)
{
    nvm_cpl_t* c = nvm_cq_poll(cq);
    if (c) {
        cq->head++;
        if ((cq->head & cq->qs_minus_1) == 0) cq->phase = !cq->phase;
    }
    return c;
}

/* ring the SQ tail doorbell if the tail moved */
static inline void nvm_sq_submit(nvm_queue_t* sq)
{
    uint32_t t = sq->tail & sq->qs_minus_1;
    if (sq->last != t) {
        __atomic_store_n((uint32_t*)sq->db, t, __ATOMIC_RELEASE);
        sq->last = t;
    }
}

/* one more submission entry has been consumed by the controller */
static inline void nvm_sq_update(nvm_queue_t* sq)
{
    sq->head++;
}

/* ring the CQ head doorbell if the head moved */
static inline void nvm_cq_update(nvm_queue_t* cq)
{
    uint32_t h = cq->head & cq->qs_minus_1;
    if (cq->last != h) {
        __atomic_store_n((uint32_t*)cq->db, h, __ATOMIC_RELEASE);
        cq->last = h;
    }
}
#endif
