/*
 * Stream timer.  Replaces include/event.h of the reference (Event :13-51):
 * a HIP event recorded on a stream; operator- gives microseconds.
 */
#ifndef __BAM_EVENT_H__
#define __BAM_EVENT_H__
#include <hip/hip_runtime.h>
#include "util.h"

struct Event
{
    hipEvent_t event;

    Event(hipStream_t stream = 0)
    {
        hip_err_chk(hipEventCreate(&event));
        hip_err_chk(hipEventRecord(event, stream));
    }
    Event(const Event&) = delete;
    Event& operator=(const Event&) = delete;
    ~Event() { (void)hipEventDestroy(event); }

    void record(hipStream_t stream = 0) { hip_err_chk(hipEventRecord(event, stream)); }

    /* microseconds from `other` to this event */
    double operator-(const Event& other) const
    {
        float ms = 0.0f;
        hip_err_chk(hipEventSynchronize(event));
        hip_err_chk(hipEventElapsedTime(&ms, other.event, event));
        return (double)ms * 1e3;
    }
};
#endif
