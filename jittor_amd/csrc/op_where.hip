// mjt_where_count / mjt_where: the positions of the non-zero elements of a tensor, as one int32 index tensor per
// axis, in row-major order (reference: python/jittor/src/ops/where_op.cc:20-60 and its kernels :62-230; what
// boolean-mask slicing, x[mask] and x[mask] = v, is built from).  The result's length depends on the data: the
// caller first asks for the count (one pass + a synchronous 8-byte copy, as the reference's executor fixes the
// uncertain shape after the op ran), allocates, then asks for the positions.
//
// Three kernels, no global atomics, deterministic order: (1) every workgroup counts the non-zeros of its 4096 elements;
// (2) one workgroup turns the counts into offsets (exclusive scan) and the total; (3) every workgroup ranks its own
// non-zeros (ballots inside a wave, wave totals through LDS) behind its offset and writes their coordinates.
#include "common.h"

namespace mjt {

namespace {
constexpr int kBlock = 256, kPer = 16, kTile = kBlock * kPer;      // elements per workgroup

// element i of a tensor of `esz`-byte elements is non-zero; floats: -0.0 is zero, NaN is not
template <int ESZ, bool FLT> __device__ __forceinline__ bool nonzero(const void* p, size_t i) {
    if constexpr (ESZ == 1) return ((const unsigned char*)p)[i] != 0;
    else if constexpr (ESZ == 2) return (((const unsigned short*)p)[i] & (FLT ? 0x7fffu : 0xffffu)) != 0;
    else if constexpr (ESZ == 4) return (((const unsigned*)p)[i] & (FLT ? 0x7fffffffu : 0xffffffffu)) != 0;
    else return (((const unsigned long long*)p)[i] & (FLT ? 0x7fffffffffffffffull : ~0ull)) != 0;
}

// Element t * kBlock + tid of the tile (t = 0..kPer-1): consecutive lanes read consecutive elements.  Returns the
// thread's flags as a bit mask.
template <int ESZ, bool FLT> __device__ __forceinline__ unsigned flags_of(const void* p, size_t n, size_t tile0) {
    unsigned m = 0;
#pragma unroll
    for (int t = 0; t < kPer; t++) {
        const size_t i = tile0 + (size_t)t * kBlock + threadIdx.x;
        if (i < n && nonzero<ESZ, FLT>(p, i)) m |= 1u << t;
    }
    return m;
}

template <int ESZ, bool FLT>
__global__ __launch_bounds__(kBlock) void where_count_kernel(const void* __restrict__ p, size_t n, unsigned* __restrict__ counts) {
    __shared__ unsigned total;
    if (threadIdx.x == 0) total = 0;
    __syncthreads();
    const unsigned m = flags_of<ESZ, FLT>(p, n, (size_t)blockIdx.x * kTile);
    unsigned c = (unsigned)__popc(m);
    for (int off = 32; off > 0; off >>= 1) c += __shfl_down(c, off, 64);
    if ((threadIdx.x & 63) == 0 && c) atomicAdd(&total, c);        // LDS, four adds
    __syncthreads();
    if (threadIdx.x == 0) counts[blockIdx.x] = total;
}

// offsets[b] = sum of counts[0..b); offsets[nblocks] = the total (64-bit: a tensor may hold more than 2^32 elements)
__global__ __launch_bounds__(1024) void where_scan_kernel(const unsigned* __restrict__ counts, unsigned long long* __restrict__ offsets,
                                                          size_t nblocks) {
    __shared__ unsigned long long wsum[16];
    __shared__ unsigned long long carry;
    if (threadIdx.x == 0) carry = 0;
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (size_t b0 = 0; b0 < nblocks; b0 += 1024) {
        const size_t b = b0 + threadIdx.x;
        unsigned long long v = b < nblocks ? counts[b] : 0, incl = v;
        for (int off = 1; off < 64; off <<= 1) {
            const unsigned long long o = __shfl_up(incl, off, 64);
            if (lane >= off) incl += o;
        }
        if (lane == 63) wsum[wave] = incl;
        __syncthreads();
        unsigned long long base = carry;
        for (int w = 0; w < wave; w++) base += wsum[w];
        if (b < nblocks) offsets[b] = base + incl - v;
        __syncthreads();
        if (threadIdx.x == 1023) carry = base + incl;
        __syncthreads();
    }
    if (threadIdx.x == 0) offsets[nblocks] = carry;
}

struct WhereOuts {
    int* out[MJT_MAX_DIM];
    long long stride[MJT_MAX_DIM];      // row-major strides of the condition tensor, in elements
    long long shape[MJT_MAX_DIM];
    int ndim;
};

template <int ESZ, bool FLT>
__global__ __launch_bounds__(kBlock) void where_write_kernel(const void* __restrict__ p, size_t n,
                                                             const unsigned long long* __restrict__ offsets, WhereOuts o,
                                                             unsigned long long limit) {
    __shared__ unsigned wave_total[kPer][kBlock / 64];
    const size_t tile0 = (size_t)blockIdx.x * kTile;
    const unsigned m = flags_of<ESZ, FLT>(p, n, tile0);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // row-major order inside the tile: step t (all lanes of wave 0, then wave 1, ...), then step t + 1
    unsigned before[kPer];               // non-zeros of this wave's lower lanes in step t
#pragma unroll
    for (int t = 0; t < kPer; t++) {
        const unsigned long long b = __ballot((m >> t) & 1u);
        before[t] = (unsigned)__popcll(b & ((1ull << lane) - 1ull));
        if (lane == 0) wave_total[t][wave] = (unsigned)__popcll(b);
    }
    __syncthreads();
    unsigned long long pos = offsets[blockIdx.x];
#pragma unroll
    for (int t = 0; t < kPer; t++) {
        unsigned mine = before[t];
        for (int w = 0; w < wave; w++) mine += wave_total[t][w];
        unsigned step_total = 0;
        for (int w = 0; w < kBlock / 64; w++) step_total += wave_total[t][w];
        if ((m >> t) & 1u) {
            const unsigned long long at = pos + mine;
            if (at < limit) {                        // never beyond what the caller allocated
                size_t i = tile0 + (size_t)t * kBlock + threadIdx.x;
                for (int d = 0; d < o.ndim; d++) {
                    const long long c = (long long)(i / (size_t)o.stride[d]);
                    i -= (size_t)c * (size_t)o.stride[d];
                    o.out[d][at] = (int)c;
                }
            }
        }
        pos += step_total;
    }
}

template <int ESZ, bool FLT> void launch_count(hipStream_t st, const void* p, size_t n, unsigned* counts, size_t nblocks) {
    hipLaunchKernelGGL((where_count_kernel<ESZ, FLT>), dim3((unsigned)nblocks), dim3(kBlock), 0, st, p, n, counts);
}
template <int ESZ, bool FLT>
void launch_write(hipStream_t st, const void* p, size_t n, const unsigned long long* offsets, const WhereOuts& o, unsigned long long limit,
                  size_t nblocks) {
    hipLaunchKernelGGL((where_write_kernel<ESZ, FLT>), dim3((unsigned)nblocks), dim3(kBlock), 0, st, p, n, offsets, o, limit);
}

bool is_float_dtype(int dt) { return dt == MJT_FLOAT16 || dt == MJT_FLOAT32 || dt == MJT_FLOAT64 || dt == MJT_BFLOAT16; }

// counts, then offsets, in the scratch arena; returns the device address of the offsets (nblocks + 1 words of 8 bytes)
unsigned long long* count_and_scan(const mjt_tensor* cond, size_t n, size_t nblocks) {
    Context& c = ctx();
    const size_t off_bytes = (nblocks + 1) * 8;
    char* base = (char*)scratch(off_bytes + nblocks * 4 + 64);
    unsigned long long* offsets = (unsigned long long*)base;
    unsigned* counts = (unsigned*)(base + off_bytes);
    const int esz = dtype_size(cond->dtype);
    const bool flt = is_float_dtype(cond->dtype);
#define MJT_WHERE_DISPATCH(FN, ...)                                                                       \
    switch (esz * 2 + (flt ? 1 : 0)) {                                                                    \
        case 2: FN<1, false>(__VA_ARGS__); break;                                                         \
        case 4: FN<2, false>(__VA_ARGS__); break;                                                         \
        case 5: FN<2, true>(__VA_ARGS__); break;                                                          \
        case 8: FN<4, false>(__VA_ARGS__); break;                                                         \
        case 9: FN<4, true>(__VA_ARGS__); break;                                                          \
        case 16: FN<8, false>(__VA_ARGS__); break;                                                        \
        case 17: FN<8, true>(__VA_ARGS__); break;                                                         \
        default: MJT_FAIL(MJT_ERR_UNSUPPORTED, "where: dtype " << mjt_dtype_name(cond->dtype));           \
    }
    MJT_WHERE_DISPATCH(launch_count, c.stream, cond->ptr, n, counts, nblocks)
    HIP_CHECK(hipGetLastError());
    hipLaunchKernelGGL(where_scan_kernel, dim3(1), dim3(1024), 0, c.stream, (const unsigned*)counts, offsets, nblocks);
    HIP_CHECK(hipGetLastError());
    return offsets;
}
}  // namespace

void where_count_impl(const mjt_tensor* cond, int64_t* count) {
    require_init();
    check_tensor(cond, "where cond");
    MJT_CHECK(count, "where: null count");
    const size_t n = (size_t)numel(cond);
    *count = 0;
    Context& c = ctx();
    if (n == 0 || c.dry_run) return;
    const size_t nblocks = (n + kTile - 1) / kTile;
    MJT_CHECK(nblocks < (size_t(1) << 31), "where: tensor too large");
    unsigned long long* offsets = count_and_scan(cond, n, nblocks);
    set_last_kernel("mjt_where_count");
    unsigned long long total = 0;
    HIP_CHECK(hipMemcpyAsync(&total, offsets + nblocks, 8, hipMemcpyDeviceToHost, c.stream));
    HIP_CHECK(hipStreamSynchronize(c.stream));
    *count = (int64_t)total;
}

void where_impl(const mjt_tensor* cond, int64_t count, const mjt_tensor* outs) {
    require_init();
    check_tensor(cond, "where cond");
    MJT_CHECK(count >= 0, "where: negative count");
    MJT_CHECK(cond->ndim >= 1 && outs, "where: cond needs a rank of at least 1 and one output per axis");
    WhereOuts o;
    memset(&o, 0, sizeof(o));
    o.ndim = cond->ndim;
    long long stride = 1;
    for (int d = cond->ndim - 1; d >= 0; d--) {
        o.stride[d] = stride;
        o.shape[d] = cond->shape[d];
        stride *= cond->shape[d];
        MJT_CHECK(cond->shape[d] < (int64_t(1) << 31), "where: an axis of 2^31 or more elements does not fit int32 indexes");
    }
    for (int d = 0; d < cond->ndim; d++) {
        check_tensor(&outs[d], "where out");
        MJT_CHECK(outs[d].dtype == MJT_INT32 && outs[d].ndim == 1 && outs[d].shape[0] == count,
                  "where: output " << d << " must be int32 [" << count << "], got " << mjt_dtype_name(outs[d].dtype) << " " << shape_str(&outs[d]));
        o.out[d] = (int*)outs[d].ptr;
    }
    const size_t n = (size_t)numel(cond);
    Context& c = ctx();
    if (n == 0 || count == 0 || c.dry_run) return;
    const size_t nblocks = (n + kTile - 1) / kTile;
    MJT_CHECK(nblocks < (size_t(1) << 31), "where: tensor too large");
    unsigned long long* offsets = count_and_scan(cond, n, nblocks);
    const int esz = dtype_size(cond->dtype);
    const bool flt = is_float_dtype(cond->dtype);
    MJT_WHERE_DISPATCH(launch_write, c.stream, cond->ptr, n, (const unsigned long long*)offsets, o, (unsigned long long)count, nblocks)
    HIP_CHECK(hipGetLastError());
    set_last_kernel("mjt_where");
}

}  // namespace mjt

extern "C" int mjt_where_count(const mjt_tensor* cond, int64_t* count) {
    return mjt::guarded([&] { mjt::where_count_impl(cond, count); });
}

extern "C" int mjt_where(const mjt_tensor* cond, int64_t count, const mjt_tensor* outs) {
    return mjt::guarded([&] { mjt::where_impl(cond, count, outs); });
}
