/*
 * A benchmark written against the C++ surface the reference's benchmarks use (Controller, page_cache_t, range_t,
 * array_t on the host; array_d_t, bam_ptr in the kernels; compare benchmarks/array/main.cu:100-330), built as an
 * ordinary HIP program against include/ and libbam_amd.so.  It reads a strided run of a 64-bit array twice, once
 * through array_d_t::operator[] and once through a bam_ptr, and prints both sums with the cache's counters:
 *
 *     array_sum <elements> <cache pages> <stride> <seed>
 *
 * The store is the software NVMe target with its procedural namespace (word w holds splitmix64(seed, w)), so the
 * sums can be checked against the closed form by whoever runs it (tests/test_gpu_parity.py does).
 */
#include <bam_amd.h>
#include <ctrl.h>
#include <page_cache.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

__global__ void sum_by_index(array_d_t<uint64_t>* a, uint64_t n_reads, uint64_t stride, unsigned long long* sum)
{
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (tid < n_reads) atomicAdd(sum, (unsigned long long)(*a)[tid * stride]);
}

__global__ void sum_by_ptr(array_d_t<uint64_t>* a, uint64_t n_reads, uint64_t stride, unsigned long long* sum)
{
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    bam_ptr<uint64_t> p(a);
    const bam_ptr<uint64_t>& in = p;
    if (tid < n_reads) atomicAdd(sum, (unsigned long long)in[tid * stride]);
}

int main(int argc, char** argv)
{
    const uint64_t n_elems = argc > 1 ? strtoull(argv[1], nullptr, 0) : 1ull << 22;
    const uint64_t cache_pages = argc > 2 ? strtoull(argv[2], nullptr, 0) : 1024;
    const uint64_t stride = argc > 3 ? strtoull(argv[3], nullptr, 0) : 8;
    const uint64_t seed = argc > 4 ? strtoull(argv[4], nullptr, 0) : 42;
    const uint64_t page_size = 4096, n_pages = (n_elems * 8 + page_size - 1) / page_size, n_reads = n_elems / stride;
    int status = 1;

    bam_target_t* target = nullptr;
    if (bam_target_create(&target, "/dev/libnvm0", n_pages * page_size, 512, 0, seed, 4, 1024, 32, 0, 0, 0)) {
        fprintf(stderr, "target: %s\n", bam_last_error());
        return 1;
    }
    try {
        hip_err_chk(hipSetDevice(0));
        Controller ctrl("/dev/libnvm0", 1, 0, 1024, 32);
        std::vector<Controller*> ctrls{&ctrl};
        page_cache_t cache(page_size, cache_pages, 0, ctrl, 64, ctrls);
        range_t<uint64_t> range(0, n_elems, 0, n_pages, 0, page_size, &cache, 0);
        std::vector<range_t<uint64_t>*> ranges{&range};
        array_t<uint64_t> array(n_elems, 0, ranges, 0);

        unsigned long long* d_sums = nullptr;
        hip_err_chk(hipMalloc((void**)&d_sums, 2 * sizeof(unsigned long long)));
        hip_err_chk(hipMemset(d_sums, 0, 2 * sizeof(unsigned long long)));
        const uint32_t threads = 64, blocks = (uint32_t)((n_reads + threads - 1) / threads);
        hipLaunchKernelGGL(sum_by_index, dim3(blocks), dim3(threads), 0, 0, array.d_array_ptr, n_reads, stride, d_sums);
        hipLaunchKernelGGL(sum_by_ptr, dim3(blocks), dim3(threads), 0, 0, array.d_array_ptr, n_reads, stride, d_sums + 1);
        hip_err_chk(hipDeviceSynchronize());
        unsigned long long sums[2];
        hip_err_chk(hipMemcpy(sums, d_sums, sizeof(sums), hipMemcpyDeviceToHost));
        printf("sum_by_index %llx\nsum_by_ptr %llx\n", sums[0], sums[1]);
        array.print_reset_stats();
        printf("aborted %d\n", ctrl.aborted() ? 1 : 0);
        status = ctrl.aborted() ? 2 : 0;
        (void)hipFree(d_sums);
    } catch (const std::exception& e) {
        fprintf(stderr, "error: %s\n", e.what());
    }
    bam_target_destroy(target);
    return status;
}
