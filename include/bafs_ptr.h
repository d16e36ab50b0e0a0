/*
 * bafs_ptr<T>: a pointer-like handle on an array_t<T> (include/bafs_ptr.h:17-132 of the reference): element
 * access through the page cache with pointer arithmetic on an element offset.  Every dereference is one
 * array_d_t access (operator[] / operator()); for runs of neighbouring elements bam_ptr is the cheaper tool.
 */
#ifndef __BAFS_PTR_H__
#define __BAFS_PTR_H__
#include <cstdint>
#include "page_cache.h"

template <typename T>
class bafs_ptr {
    array_t<T>* h_pData;
    array_d_t<T>* pData;
    uint64_t start_idx;

public:
    __host__ void print_stats() const { if (h_pData) h_pData->print_reset_stats(); }

    __host__ __device__ bafs_ptr() : h_pData(nullptr), pData(nullptr), start_idx(0) {}
    __host__ __device__ bafs_ptr(array_d_t<T>* const pValue, const uint64_t start_off) : h_pData(nullptr), pData(pValue), start_idx(start_off) {}
    __host__ bafs_ptr(array_t<T>* const pValue) : h_pData(pValue), pData(pValue->d_array_ptr), start_idx(0) {}
    __host__ bafs_ptr(array_t<T>* const pValue, const uint64_t start_off) : h_pData(pValue), pData(pValue->d_array_ptr), start_idx(start_off) {}
    bafs_ptr(const bafs_ptr&) = default;
    bafs_ptr& operator=(const bafs_ptr&) = default;

    __device__ T operator*() const { return (*pData)[start_idx]; }
    __device__ T operator[](const uint64_t i) const { return (*pData)[start_idx + i]; }
    /* store: p(i, v) writes v to element i of the array (not offset by the pointer, as in the reference) */
    __device__ void operator()(const uint64_t i, const T val) const { (*pData)(i, val); }

    __host__ __device__ bafs_ptr operator+(const uint64_t i) const { bafs_ptr r(*this); r.start_idx += i; return r; }
    __host__ __device__ bafs_ptr operator-(const uint64_t i) const { bafs_ptr r(*this); r.start_idx -= i; return r; }
    __host__ __device__ bafs_ptr operator++(int) { bafs_ptr c(*this); start_idx += 1; return c; }
    __host__ __device__ bafs_ptr& operator++() { start_idx += 1; return *this; }
    __host__ __device__ bafs_ptr operator--(int) { bafs_ptr c(*this); start_idx -= 1; return c; }
    __host__ __device__ bafs_ptr& operator--() { start_idx -= 1; return *this; }
    __host__ __device__ uint64_t offset() const { return start_idx; }

    /* wave-cooperative copy of `count` elements from element src_idx on (clipped to its page) to dest */
    __device__ void memcpy_to_array_aligned(const uint64_t src_idx, const uint64_t count, T* dest) const { pData->memcpy(src_idx, count, dest); }

    friend __host__ __device__ bool operator==(const bafs_ptr& l, const bafs_ptr& r) { return l.pData == r.pData && l.start_idx == r.start_idx && l.h_pData == r.h_pData; }
    friend __host__ __device__ bool operator!=(const bafs_ptr& l, const bafs_ptr& r) { return !(l == r); }
};
#endif /* __BAFS_PTR_H__ */
