// One-axis scatter  x[idx[i]] = OP(x[idx[i]], y[i])  for i in [0, n), idx a
// 1-d integer tensor (the pattern jt.histc and jt.scatter produce,
// reference: python/jittor/misc.py:2233; semantics
// python/jittor/src/ops/reindex_reduce_op.cc:93-131).
//
// Supplied by the host: TX (element type), TE (index type), WBINS (bins
// privatised in LDS, power of two), NTHREADS, MODE (0 add, 1 maximum,
// 2 minimum), IDENT_BITS (bit pattern of the identity).
//
// Hot bins serialise global atomics, so each workgroup keeps a private copy
// of a window of WBINS consecutive bins [lo, lo+WBINS) in LDS, applies every
// update that falls into the window with LDS atomics, and flushes the touched
// entries to x with one global atomic each when its share of the input is
// done.  Updates outside the window go straight to global atomics.  `lo` is
// read from device memory: a sampling pass picks the window that holds the
// most updates.  x must hold the identity before this kernel runs.

struct Params { void* a[8]; };   // 8-byte words; typed as pointers so loads/stores use the global address space
// a[0] x, a[1] y, a[2] idx, a[3] n, a[4] bins, a[5] &lo (int), a[6] elements per workgroup

#if MODE == 0
#define LDS_UPDATE(addr, v) atomicAdd((addr), (v))
#define GLB_UPDATE(addr, v) mjt_atomic_add<TX>((addr), (v))
#elif MODE == 1
#define LDS_UPDATE(addr, v) mjt_lds_max((addr), (v))
#define GLB_UPDATE(addr, v) mjt_atomic_maximum<TX>((addr), (v))
#else
#define LDS_UPDATE(addr, v) mjt_lds_min((addr), (v))
#define GLB_UPDATE(addr, v) mjt_atomic_minimum<TX>((addr), (v))
#endif

__device__ __forceinline__ void mjt_lds_max(float* a, float v) {
    if (v != v) return;
    unsigned b = __float_as_uint(v);
    if (b >> 31) atomicMin((unsigned*)a, b); else atomicMax((int*)a, (int)b);
}
__device__ __forceinline__ void mjt_lds_min(float* a, float v) {
    if (v != v) return;
    unsigned b = __float_as_uint(v);
    if (b >> 31) atomicMax((unsigned*)a, b); else atomicMin((int*)a, (int)b);
}
__device__ __forceinline__ void mjt_lds_max(int* a, int v) { atomicMax(a, v); }
__device__ __forceinline__ void mjt_lds_min(int* a, int v) { atomicMin(a, v); }
__device__ __forceinline__ void mjt_lds_max(unsigned* a, unsigned v) { atomicMax(a, v); }
__device__ __forceinline__ void mjt_lds_min(unsigned* a, unsigned v) { atomicMin(a, v); }

extern "C" __global__ __launch_bounds__(NTHREADS) void ENTRY(Params p) {
    TX* __restrict__ xp = (TX*)p.a[0];
    const TX* __restrict__ yp = (const TX*)p.a[1];
    const TE* __restrict__ ip = (const TE*)p.a[2];
    const long long n = (long long)(unsigned long long)p.a[3];
    const long long bins = (long long)(unsigned long long)p.a[4];
    const long long lo = *(const int*)p.a[5];
    const long long per = (long long)(unsigned long long)p.a[6];
    __shared__ TX win[WBINS];
    TX ident;
    {
        unsigned ib = IDENT_BITS;
        __builtin_memcpy(&ident, &ib, 4);
    }
    for (int t = threadIdx.x; t < WBINS; t += NTHREADS) win[t] = ident;
    __syncthreads();
    const long long begin = (long long)blockIdx.x * per;
    const long long end = begin + per < n ? begin + per : n;
    // per is a multiple of 4*NTHREADS and the bases are 16-byte aligned: full vectors first
    long long i = begin + (long long)threadIdx.x * 4;
    for (; i + 3 < end; i += (long long)NTHREADS * 4) {
        mjt_pack<TX, 4> v;
        mjt_pack<TE, 4> id;
        mjt_load_nt(v, yp + i);
        mjt_load_nt(id, ip + i);
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const long long b = (long long)id.v[k];
            if (b < 0 || b >= bins) continue;               // overflow: skipped
            const unsigned long long w = (unsigned long long)(b - lo);
            if (w < (unsigned long long)WBINS) { LDS_UPDATE(&win[w], v.v[k]); }
            else { GLB_UPDATE(xp + b, v.v[k]); }
        }
    }
    for (; i < end; i++) {                                   // ragged tail of the last workgroup
        const long long b = (long long)ip[i];
        if (b < 0 || b >= bins) continue;
        const unsigned long long w = (unsigned long long)(b - lo);
        if (w < (unsigned long long)WBINS) { LDS_UPDATE(&win[w], yp[i]); }
        else { GLB_UPDATE(xp + b, yp[i]); }
    }
    __syncthreads();
    for (int t = threadIdx.x; t < WBINS; t += NTHREADS) {
        const TX v = win[t];
        unsigned vb;
        __builtin_memcpy(&vb, &v, 4);
        const long long b = lo + t;
        if (vb != IDENT_BITS && b < bins) { GLB_UPDATE(xp + b, v); }
    }
}

// Sampling pass: a strided sample of the indices votes for windows of WBINS
// bins; the start of the fullest window is written to *lo.
extern "C" __global__ __launch_bounds__(1024) void ENTRY_SAMPLE(Params p) {
    const TE* __restrict__ ip = (const TE*)p.a[2];
    const long long n = (long long)(unsigned long long)p.a[3];
    const long long bins = (long long)(unsigned long long)p.a[4];
    int* lo = (int*)p.a[5];
    __shared__ int votes[1024];
    __shared__ int best_votes, best_tile;
    const long long tiles = (bins + WBINS - 1) / WBINS;
    const long long group = (tiles + 1023) / 1024;          // windows per counter when there are more than 1024
    votes[threadIdx.x] = 0;
    if (threadIdx.x == 0) { best_votes = -1; best_tile = 0; }
    __syncthreads();
    const long long samples = n < 16384 ? n : 16384;
    const long long stride = n / samples;
    for (long long s = threadIdx.x; s < samples; s += 1024) {
        const long long b = (long long)ip[s * stride];
        if (b >= 0 && b < bins) atomicAdd(&votes[(b / WBINS) / group], 1);
    }
    __syncthreads();
    atomicMax(&best_votes, votes[threadIdx.x]);
    __syncthreads();
    if (votes[threadIdx.x] == best_votes) atomicMax(&best_tile, (int)threadIdx.x);
    __syncthreads();
    if (threadIdx.x == 0) {
        long long start = (long long)best_tile * group * WBINS;
        if (start + WBINS > bins) start = bins > WBINS ? bins - WBINS : 0;
        *lo = (int)start;
    }
}
