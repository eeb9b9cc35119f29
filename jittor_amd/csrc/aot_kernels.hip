// Ahead-of-time kernels that need no run-time specialisation: device copy and
// fill.  The copy kernel doubles as the calibration kernel for HBM counters
// (a launch that moves a known number of bytes).
#include "common.h"

namespace mjt {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void mjt_copy_kernel(u32x4* __restrict__ dst, const u32x4* __restrict__ src, size_t n16) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    size_t stride = (size_t)gridDim.x * 256;
    for (; i < n16; i += stride) {
        u32x4 v = __builtin_nontemporal_load(src + i);
        __builtin_nontemporal_store(v, dst + i);
    }
}

__global__ __launch_bounds__(256) void mjt_copy_tail_kernel(unsigned char* __restrict__ dst,
                                                            const unsigned char* __restrict__ src, size_t n) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = src[i];
}

__global__ __launch_bounds__(256) void mjt_fill_u32_kernel(uint32_t* __restrict__ dst, uint32_t v, size_t n) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    size_t stride = (size_t)gridDim.x * 256;
    for (; i < n; i += stride) dst[i] = v;
}

template <class T>
__global__ __launch_bounds__(256) void mjt_fill_pattern_kernel(T* __restrict__ dst, T v, size_t n) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    size_t stride = (size_t)gridDim.x * 256;
    for (; i < n; i += stride) dst[i] = v;
}

// Fills n elements of elem_size bytes with the low bytes of `pattern`
// (identity values of the scatter op).
void launch_fill_pattern(void* dst, uint64_t pattern, int elem_size, size_t n) {
    Context& c = ctx();
    if (c.dry_run || n == 0) return;
    size_t blocks = (n + 256 * 8 - 1) / (256 * 8);
    if (blocks > (size_t)1 << 20) blocks = (size_t)1 << 20;
    set_last_kernel("mjt_fill_pattern_kernel");
    switch (elem_size) {
        case 1: hipLaunchKernelGGL(mjt_fill_pattern_kernel<uint8_t>, dim3((unsigned)blocks), dim3(256), 0, c.stream, (uint8_t*)dst, (uint8_t)pattern, n); break;
        case 2: hipLaunchKernelGGL(mjt_fill_pattern_kernel<uint16_t>, dim3((unsigned)blocks), dim3(256), 0, c.stream, (uint16_t*)dst, (uint16_t)pattern, n); break;
        case 4: hipLaunchKernelGGL(mjt_fill_pattern_kernel<uint32_t>, dim3((unsigned)blocks), dim3(256), 0, c.stream, (uint32_t*)dst, (uint32_t)pattern, n); break;
        case 8: hipLaunchKernelGGL(mjt_fill_pattern_kernel<uint64_t>, dim3((unsigned)blocks), dim3(256), 0, c.stream, (uint64_t*)dst, (uint64_t)pattern, n); break;
        default: MJT_FAIL(MJT_ERR_INVALID, "fill: element size " << elem_size);
    }
    HIP_CHECK(hipGetLastError());
}

void launch_copy(void* dst, const void* src, size_t bytes) {
    Context& c = ctx();
    if (c.dry_run) return;
    bool aligned = ((uintptr_t)dst % 16 == 0) && ((uintptr_t)src % 16 == 0);
    size_t n16 = aligned ? bytes / 16 : 0;
    if (n16) {
        size_t per_block = 256 * 4;   // four 16-byte vectors per lane
        size_t blocks = (n16 + per_block - 1) / per_block;
        if (blocks > (size_t)1 << 30) blocks = (size_t)1 << 30;
        set_last_kernel("mjt_copy_kernel");
        hipLaunchKernelGGL(mjt_copy_kernel, dim3((unsigned)blocks), dim3(256), 0, c.stream, (u32x4*)dst, (const u32x4*)src, n16);
    }
    size_t done = n16 * 16;
    if (done < bytes) {
        size_t n = bytes - done;
        hipLaunchKernelGGL(mjt_copy_tail_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, c.stream,
                           (unsigned char*)dst + done, (const unsigned char*)src + done, n);
    }
    HIP_CHECK(hipGetLastError());
}

void launch_fill_u32(void* dst, uint32_t pattern, size_t n_words) {
    Context& c = ctx();
    if (c.dry_run) return;
    size_t blocks = (n_words + 256 * 8 - 1) / (256 * 8);
    if (blocks > (size_t)1 << 20) blocks = (size_t)1 << 20;
    set_last_kernel("mjt_fill_u32_kernel");
    hipLaunchKernelGGL(mjt_fill_u32_kernel, dim3((unsigned)blocks), dim3(256), 0, c.stream, (uint32_t*)dst, pattern, n_words);
    HIP_CHECK(hipGetLastError());
}

}  // namespace mjt
