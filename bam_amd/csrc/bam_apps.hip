// vectoradd, reduction and scan of the C-ABI library (benchmarks/vectoradd, reduction, scan of the reference): kernels
// in which consecutive threads read consecutive elements through bam_ptr, and the scan that allocates nothing.
#include "bam_capi_internal.h"

namespace {

// ---- vectoradd (benchmarks/vectoradd/main.cu:102-117 kernel_baseline_ptr_pc): C[i] = A[i] + B[i], all three behind the cache ----
__global__ __launch_bounds__(64) void k_vectoradd_ptr_pc(array_d_t<uint64_t>* da, array_d_t<uint64_t>* db, uint64_t n_elems, array_d_t<uint64_t>* dc, const fetch_plan fp)
{
    if (fp.done && blockIdx.x < fp.blocks) {
        array_d_t<uint64_t>* const arrays[3] = {da, db, dc};
        fetch_role(arrays, n_elems, fp);
        return;
    }
    const uint64_t bid = blockIdx.x - (fp.done ? fp.blocks : 0u);
    const uint64_t tid = (uint64_t)blockDim.x * bid + threadIdx.x;
    bam_ptr<uint64_t> Aptr(da);
    bam_ptr<uint64_t> Bptr(db);
    bam_ptr<uint64_t> Cptr(dc);
    const bam_ptr<uint64_t>& A = Aptr;
    const bam_ptr<uint64_t>& B = Bptr;
    const uint64_t first = tid - threadIdx.x % BAM_WAVE_SIZE;
    if (first < n_elems) {
        touch_ahead(da, first, n_elems, BAM_WAVE_SIZE, 0);
        touch_ahead(db, first, n_elems, BAM_WAVE_SIZE, 1);
        touch_ahead(dc, first, n_elems, BAM_WAVE_SIZE, 2);
    }
    if (tid < n_elems) Cptr[tid] = A[tid] + B[tid];
    if (fp.done && threadIdx.x == 0) __hip_atomic_fetch_add(fp.done, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ---- reduction (benchmarks/reduction/main.cu:166-195 kernel_reduce_baseline_ptr_pc): output[b] = sum of the 2 x blockDim elements of block b ----
__global__ void k_reduce_ptr_pc(array_d_t<uint64_t>* da, unsigned long long* output, uint64_t len, const fetch_plan fp)
{
    __shared__ uint64_t wave_total[1024 / BAM_WAVE_SIZE];
    if (fp.done && blockIdx.x < fp.blocks) {
        array_d_t<uint64_t>* const arrays[1] = {da};
        fetch_role(arrays, len, fp);
        return;
    }
    const uint64_t bid = blockIdx.x - (fp.done ? fp.blocks : 0u);
    const uint64_t tid = threadIdx.x, start = 2ull * blockDim.x * bid;
    uint64_t v = 0;
    {
        bam_ptr<uint64_t> in_ptr(da);
        const bam_ptr<uint64_t>& input = in_ptr;
        /* a workgroup reads 2 x blockDim consecutive elements: its waves' first elements */
        const uint64_t first = start + tid - tid % BAM_WAVE_SIZE;
        if (first < len) touch_ahead(da, first, len);
        if (first + blockDim.x < len) touch_ahead(da, first + blockDim.x, len);
        if (start + tid < len) v = input[start + tid];
        if (blockDim.x + start + tid < len) v += input[blockDim.x + start + tid];
    }
    v = wave_sum(v);
    if (bam::lane() == 0) wave_total[tid / BAM_WAVE_SIZE] = v;
    __syncthreads();
    if (tid < BAM_WAVE_SIZE) {
        v = wave_sum(tid < blockDim.x / BAM_WAVE_SIZE ? wave_total[tid] : 0);
        if (tid == 0) output[bid] = v;
        if (fp.done && tid == 0) __hip_atomic_fetch_add(fp.done, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// ---- scan (benchmarks/scan/main.cu:147-190 kernel_scan_baseline_ptr_pc, :89-100 finalsum) ----
/* inclusive sums over the 64 lanes of a wave (all lanes active) */
__device__ __forceinline__ uint64_t wave_inclusive_sum(uint64_t v)
{
    const uint32_t lane = bam::lane();
#pragma unroll
    for (uint32_t o = 1; o < BAM_WAVE_SIZE; o <<= 1) {
        const uint64_t u = bam::shfl(v, lane >= o ? lane - o : lane);
        if (lane >= o) v += u;
    }
    return v;
}

/*
 * Block b scans its 2 x blockDim elements: output[i] = sum of the block's elements up to and including i,
 * intermediate[b] = the block's total.  The elements are read as the reference reads them (thread t takes t and
 * t + blockDim, so a wave reads consecutive elements through one page reference); the scan itself runs over wave
 * shuffles on pairs of neighbours rather than the two tree passes over shared memory.
 */
__global__ void k_scan_ptr_pc(array_d_t<uint64_t>* da, unsigned long long* output, unsigned long long* intermediate, uint64_t len, const fetch_plan fp)
{
    extern __shared__ uint64_t scan_mem[];                      /* 2 x blockDim elements, then one total per wave */
    if (fp.done && blockIdx.x < fp.blocks) {
        array_d_t<uint64_t>* const arrays[1] = {da};
        fetch_role(arrays, len, fp);
        return;
    }
    const uint32_t bid = blockIdx.x - (fp.done ? fp.blocks : 0u);
    const uint32_t B = blockDim.x, t = threadIdx.x;
    uint64_t* wave_total = scan_mem + 2 * B;
    const uint64_t idx = 2ull * bid * B + t;
    {
        bam_ptr<uint64_t> in_ptr(da);
        const bam_ptr<uint64_t>& ptr = in_ptr;
        const uint64_t first = idx - t % BAM_WAVE_SIZE;
        if (first < len) touch_ahead(da, first, len);
        if (first + B < len) touch_ahead(da, first + B, len);
        scan_mem[t] = idx < len ? ptr[idx] : 0;
        scan_mem[t + B] = idx + B < len ? ptr[idx + B] : 0;
    }
    __syncthreads();
    const uint64_t a = scan_mem[2 * t], b = a + scan_mem[2 * t + 1];
    const uint64_t s = wave_inclusive_sum(b);
    if (bam::lane() == BAM_WAVE_SIZE - 1) wave_total[t / BAM_WAVE_SIZE] = s;
    __syncthreads();
    uint64_t before = s - b;
    for (uint32_t w = 0; w < t / BAM_WAVE_SIZE; w++) before += wave_total[w];
    scan_mem[2 * t] = before + a;
    scan_mem[2 * t + 1] = before + b;
    __syncthreads();
    if (idx < len) output[idx] = scan_mem[t];
    if (idx + B < len) output[idx + B] = scan_mem[t + B];
    if (intermediate && t == B - 1) intermediate[bid] = before + b;
    if (fp.done && t == 0) __hip_atomic_fetch_add(fp.done, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

/* one block: v[i] = v[0] + ... + v[i] in place (the reference calls cub::DeviceScan::InclusiveSum here, scan/main.cu:416-418) */
__global__ void k_scan_block_totals(unsigned long long* v, uint64_t n)
{
    __shared__ uint64_t wave_total[1024 / BAM_WAVE_SIZE];
    __shared__ uint64_t carry_s;
    const uint32_t t = threadIdx.x;
    if (t == 0) carry_s = 0;
    __syncthreads();
    for (uint64_t base = 0; base < n; base += blockDim.x) {
        const uint64_t x = base + t < n ? v[base + t] : 0;
        const uint64_t s = wave_inclusive_sum(x);
        if (bam::lane() == BAM_WAVE_SIZE - 1) wave_total[t / BAM_WAVE_SIZE] = s;
        __syncthreads();
        uint64_t r = carry_s + s;
        for (uint32_t w = 0; w < t / BAM_WAVE_SIZE; w++) r += wave_total[w];
        if (base + t < n) v[base + t] = r;
        __syncthreads();
        if (t == blockDim.x - 1) carry_s = r;
        __syncthreads();
    }
}

__global__ void k_scan_finalsum(const unsigned long long* scanned_totals, unsigned long long* output, uint64_t len)
{
    if (blockIdx.x == 0) return;
    const uint64_t B = blockDim.x, idx = 2ull * blockIdx.x * B + threadIdx.x;
    const uint64_t add = scanned_totals[blockIdx.x - 1];
    if (idx < len) output[idx] += add;
    if (idx + B < len) output[idx + B] += add;
}

} // namespace

extern "C" {

int bam_vectoradd(bam_array_t* a, bam_array_t* b, bam_array_t* c, uint64_t n_elems, void* stream)
{
    if (!a || !b || !c) return fail(EINVAL, "bam_vectoradd: null argument");
    if (n_elems > a->a->adt.n_elems || n_elems > b->a->adt.n_elems || n_elems > c->a->adt.n_elems) return fail(EINVAL, "bam_vectoradd: more elements than the arrays hold");
    if (!n_elems) return 0;
    BAM_API_BEGIN
    const fetch_plan fp = make_fetch_plan(a, 3, 64, 64, (hipStream_t)stream);
    hipLaunchKernelGGL(k_vectoradd_ptr_pc, dim3(blocks_for(n_elems, 64) + fp.blocks), dim3(64), 0, (hipStream_t)stream,
                       a->a->d_array_ptr, b->a->d_array_ptr, n_elems, c->a->d_array_ptr, fp);
    hip_err_chk(hipGetLastError());
    BAM_API_END
}

int bam_reduce(bam_array_t* a, uint64_t n_elems, uint32_t block_size, uint64_t* d_partials, void* stream)
{
    if (!a || !d_partials) return fail(EINVAL, "bam_reduce: null argument");
    if (!block_size || block_size % BAM_WAVE_SIZE || block_size > 1024) return fail(EINVAL, "bam_reduce: block size must be a multiple of 64, at most 1024");
    if (n_elems > a->a->adt.n_elems) return fail(EINVAL, "bam_reduce: more elements than the array holds");
    if (!n_elems) return 0;
    BAM_API_BEGIN
    const fetch_plan fp = make_fetch_plan(a, 1, block_size, 2ull * block_size, (hipStream_t)stream);
    hipLaunchKernelGGL(k_reduce_ptr_pc, dim3(blocks_for(n_elems, 2ull * block_size) + fp.blocks), dim3(block_size), 0, (hipStream_t)stream,
                       a->a->d_array_ptr, (unsigned long long*)d_partials, n_elems, fp);
    hip_err_chk(hipGetLastError());
    BAM_API_END
}

int bam_scan(bam_array_t* a, uint64_t n_elems, uint32_t block_size, uint64_t* d_result, void* stream)
{
    if (!a || !d_result) return fail(EINVAL, "bam_scan: null argument");
    if (!block_size || block_size % BAM_WAVE_SIZE || block_size > 1024) return fail(EINVAL, "bam_scan: block size must be a multiple of 64, at most 1024");
    if (n_elems > a->a->adt.n_elems) return fail(EINVAL, "bam_scan: more elements than the array holds");
    BAM_API_BEGIN
    hipStream_t st = (hipStream_t)stream;
    hip_err_chk(hipMemsetAsync(d_result, 0, sizeof(uint64_t), st));
    if (n_elems) {
        const uint64_t n_blocks = blocks_for(n_elems, 2ull * block_size);
        BufferPtr totals = createBuffer(n_blocks * sizeof(uint64_t), 0);
        unsigned long long* out = (unsigned long long*)d_result + 1;
        const size_t lds = (2 * block_size + 1024 / BAM_WAVE_SIZE) * sizeof(uint64_t);
        const fetch_plan fp = make_fetch_plan(a, 1, block_size, 2ull * block_size, st);
        hipLaunchKernelGGL(k_scan_ptr_pc, dim3(n_blocks + fp.blocks), dim3(block_size), lds, st, a->a->d_array_ptr, out, (unsigned long long*)totals.get(), n_elems, fp);
        hipLaunchKernelGGL(k_scan_block_totals, dim3(1), dim3(1024), 0, st, (unsigned long long*)totals.get(), n_blocks);
        hipLaunchKernelGGL(k_scan_finalsum, dim3(n_blocks), dim3(block_size), 0, st, (const unsigned long long*)totals.get(), out, n_elems);
        hip_err_chk(hipGetLastError());
        hip_err_chk(hipStreamSynchronize(st));         /* `totals` is released on return */
    }
    BAM_API_END
}

} // extern "C"

/*
 * bam_scan for callers that cannot allocate (code under stream capture, serving loops, harnesses that forbid it): the block
 * totals, which bam_scan keeps in a buffer it allocates and frees per call, live in a file-scope device array of fixed size.
 * Every device the library runs on holds its own copy of the array at its own address until the process ends; the address is
 * looked up once per device (the array's name means nothing to the host) and handed to the kernels like any other buffer.
 */
/* BAM_SCAN_NOALLOC_MAX_BLOCKS (bam_amd.h): 65536 block totals, 512 KiB */
#define BAM_SCAN_NOALLOC_MAX_DEVICES 64
static __device__ __align__(256) unsigned long long scratch[BAM_SCAN_NOALLOC_MAX_BLOCKS];

namespace {
std::mutex g_scratch_mu;
unsigned long long* g_scratch_ptr[BAM_SCAN_NOALLOC_MAX_DEVICES];      /* per device: where its copy of `scratch` lives */

/* the current device's copy of the array; NULL (and the error recorded) if it cannot be found */
unsigned long long* scan_scratch_of_current_device()
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= BAM_SCAN_NOALLOC_MAX_DEVICES) { g_err = "bam_scan_noalloc: no current device"; return nullptr; }
    std::lock_guard<std::mutex> g(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) { g_err = std::string("bam_scan_noalloc: hipGetSymbolAddress: ") + hipGetErrorString(e); return nullptr; }
        g_scratch_ptr[dev] = (unsigned long long*)p;
    }
    return g_scratch_ptr[dev];
}

__global__ void k_store_zero64(unsigned long long* p) { *p = 0; }
} // namespace

extern "C" {

int bam_scan_noalloc(bam_array_t* a, uint64_t n_elems, uint32_t block_size, uint64_t* d_result, void* stream)
{
    if (!a || !d_result) return fail(EINVAL, "bam_scan_noalloc: null argument");
    if (!block_size || block_size % BAM_WAVE_SIZE || block_size > 1024) return fail(EINVAL, "bam_scan_noalloc: block size must be a multiple of 64, at most 1024");
    if (n_elems > a->a->adt.n_elems) return fail(EINVAL, "bam_scan_noalloc: more elements than the array holds");
    const uint64_t n_blocks = (n_elems + 2ull * block_size - 1) / (2ull * block_size);
    if (n_blocks > BAM_SCAN_NOALLOC_MAX_BLOCKS)
        return fail(E2BIG, "bam_scan_noalloc: " + std::to_string(n_elems) + " elements in blocks of " + std::to_string(2ull * block_size) + " need " + std::to_string(n_blocks) +
                           " block totals, the fixed scratch array holds " + std::to_string(BAM_SCAN_NOALLOC_MAX_BLOCKS) + " (use bam_scan, or a larger block size)");
    unsigned long long* totals = scan_scratch_of_current_device();
    if (!totals) return EIO;
    hipStream_t st = (hipStream_t)stream;
    unsigned long long* out = (unsigned long long*)d_result + 1;
    /* no memset node: a fill kernel clears the first word (a caller may be capturing this stream) */
    hipLaunchKernelGGL(k_store_zero64, dim3(1), dim3(1), 0, st, (unsigned long long*)d_result);
    if (n_elems) {
        /* totals[0 .. n_blocks) are written by the first kernel before the second reads them; what an earlier, longer call
         * left behind them is never read, so nothing has to be cleared */
        const size_t lds = (2 * block_size + 1024 / BAM_WAVE_SIZE) * sizeof(uint64_t);
        /* no fetch waves here: their counter would have to be allocated and cleared */
        const fetch_plan none{nullptr, 0, 0, 0, 0};
        hipLaunchKernelGGL(k_scan_ptr_pc, dim3((uint32_t)n_blocks), dim3(block_size), lds, st, a->a->d_array_ptr, out, totals, n_elems, none);
        hipLaunchKernelGGL(k_scan_block_totals, dim3(1), dim3(1024), 0, st, totals, n_blocks);
        hipLaunchKernelGGL(k_scan_finalsum, dim3((uint32_t)n_blocks), dim3(block_size), 0, st, (const unsigned long long*)totals, out, n_elems);
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(EIO, std::string("bam_scan_noalloc: ") + hipGetErrorString(e));
    return 0;
}

} // extern "C"
