/*
 * Small host/device helpers.  Replaces include/util.h of the reference
 * (cuda_err_chk :18-35, hexdump :52-96, warp_memcpy :102-117, CEIL :45) with
 * HIP equivalents; warp_memcpy shares the elements out over the active lanes
 * of a 64-wide wave.
 */
#ifndef __BAM_UTIL_H__
#define __BAM_UTIL_H__
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
#include <stdexcept>
#include <string>
#include "bam_wave.h"

#define hip_err_chk(ans) { bam_hip_assert((ans), __FILE__, __LINE__); }
#define cuda_err_chk(ans) hip_err_chk(ans)

inline void bam_hip_assert(hipError_t code, const char* file, int line)
{
    if (code != hipSuccess)
        throw std::runtime_error(std::string("HIP error: ") + hipGetErrorString(code) + " at " + file + ":" + std::to_string(line));
}

#ifndef CEIL
#define CEIL(X, Y, Z) (((X) + (Y) - 1) >> (Z))
#endif

/* cooperative copy by the active lanes, all called with the same arguments: `num` elements of type T (a count, not
 * bytes, as in the reference), the k-th active lane taking elements k, k + n, ... of n active lanes */
template <typename T>
__device__ __forceinline__ void warp_memcpy(T* dest, const T* src, size_t num)
{
    const uint64_t act = bam::active_mask();
    const uint32_t n = bam::popc(act), rank = bam::rank_in(act);
    for (size_t i = rank; i < num; i += n) dest[i] = src[i];
}

inline __host__ void hexdump(const void* data, size_t size)
{
    const unsigned char* p = (const unsigned char*)data;
    for (size_t i = 0; i < size; i += 16) {
        printf("%08zx ", i);
        for (size_t j = i; j < i + 16 && j < size; j++) printf(" %02x", p[j]);
        printf("\n");
    }
}
#endif
