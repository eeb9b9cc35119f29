// Sliding-window gather: y[b.., oh, ow, kh, kw] = x[b.., oh*SH+kh*DH+CH, ow*SW+kw*DW+CW]
// with the overflow value outside x.  This is the affine special case of the
// gather op (reference: python/jittor/src/ops/reindex_op.cc:111-139) that
// im2col-style reindexes produce.
//
// Geometry is baked in by the host (the reference's compile_shapes option does
// the same, opt/pass/compile_shapes_pass.cc): H, W, OH, OW, KH, KW, SH, SW, DH,
// DW, CH, CW, TH (output rows per workgroup), LH x LW (LDS tile), ESZ-byte
// elements moved as raw bits (TB), VEC elements per store.
//
// A workgroup owns TPW consecutive tiles of one plane, a tile being TH output rows.  Per tile it stages the
// input rows they touch in LDS (out-of-range cells hold the overflow value, so no bounds test is left in the
// inner loop), then writes its part of y, which is one contiguous run of TH*OW*KH*KW elements, as 16-byte
// vectors: lane l owns vectors l, l+WTHREADS, ... of that run and finds (row, ow, kh, kw) of each element by
// constant division.  The input of the next tile is loaded into registers before the current tile is stored and
// written to the other LDS buffer after: the read latency hides behind the stores.  Loads and stores are
// unconditional instructions with clamped addresses or masked lanes, and the store loop has a constant trip
// count: memory operations of a wave complete in order, and the wait for the prefetched input may leave exactly
// the stores issued after it outstanding only if their number is known.

// cache policy of the stores of y: non-temporal and system scope (sc0 sc1 nt).  y is written once and not read here; on
// MI355X these stores stream 3 - 5 % faster than plain non-temporal ones (a fill of 231 MB: 6.9 against 6.6 TB/s; this
// kernel at 32 x 64 x 56 x 56, 3 x 3: 44.8 against 45.5 us) and plain stores are slower still (49 us).
#define ST_AUX 19
struct Params { void* a[4]; };   // 8-byte words; typed as pointers so loads/stores use the global address space   // x, y, overflow bits, number of planes

// Element and vector moves through buffer descriptors: an offset past the end of the descriptor's range reads
// zeros and drops a store, which is how lanes without work stay out of the way without a branch.
typedef unsigned mjt_wu32x2 __attribute__((ext_vector_type(2)));
typedef unsigned mjt_wu32x4 __attribute__((ext_vector_type(4)));
template <int BYTES> struct mjt_win_io;
template <> struct mjt_win_io<2> {
    typedef unsigned short raw;
    static __device__ __forceinline__ raw load(__amdgpu_buffer_rsrc_t r, unsigned off) { return __builtin_amdgcn_raw_buffer_load_b16(r, (int)off, 0, 0); }
    static __device__ __forceinline__ void store(raw v, __amdgpu_buffer_rsrc_t r, unsigned off) { __builtin_amdgcn_raw_buffer_store_b16(v, r, (int)off, 0, ST_AUX); }
};
template <> struct mjt_win_io<4> {
    typedef unsigned raw;
    static __device__ __forceinline__ raw load(__amdgpu_buffer_rsrc_t r, unsigned off) { return __builtin_amdgcn_raw_buffer_load_b32(r, (int)off, 0, 0); }
    static __device__ __forceinline__ void store(raw v, __amdgpu_buffer_rsrc_t r, unsigned off) { __builtin_amdgcn_raw_buffer_store_b32(v, r, (int)off, 0, ST_AUX); }
};
template <> struct mjt_win_io<8> {
    typedef mjt_wu32x2 raw;
    static __device__ __forceinline__ raw load(__amdgpu_buffer_rsrc_t r, unsigned off) { return __builtin_amdgcn_raw_buffer_load_b64(r, (int)off, 0, 0); }
    static __device__ __forceinline__ void store(raw v, __amdgpu_buffer_rsrc_t r, unsigned off) { __builtin_amdgcn_raw_buffer_store_b64(v, r, (int)off, 0, ST_AUX); }
};
template <> struct mjt_win_io<16> {
    typedef mjt_wu32x4 raw;
    static __device__ __forceinline__ void store(raw v, __amdgpu_buffer_rsrc_t r, unsigned off) { __builtin_amdgcn_raw_buffer_store_b128(v, r, (int)off, 0, ST_AUX); }
};
__device__ __forceinline__ TB mjt_win_load(__amdgpu_buffer_rsrc_t r, unsigned off) {
    return __builtin_bit_cast(TB, mjt_win_io<sizeof(TB)>::load(r, off));
}
__device__ __forceinline__ void mjt_win_store(__amdgpu_buffer_rsrc_t r, unsigned off, const mjt_pack<TB, VEC>& v) {
    typedef mjt_win_io<sizeof(TB) * VEC> io;
    io::store(__builtin_bit_cast(typename io::raw, v), r, off);
}

extern "C" __global__ __launch_bounds__(WTHREADS) void ENTRY(Params p) {
    const TB* __restrict__ xp = (const TB*)p.a[0];
    TB* __restrict__ yp = (TB*)p.a[1];
    const TB ov = (TB)(unsigned long long)p.a[2];
    __shared__ TB tile[2][LH * LW];
    constexpr int TILES = (OH + TH - 1) / TH;
    constexpr int PARTS = (TILES + TPW - 1) / TPW;          // workgroups per plane
    const unsigned plane = blockIdx.x / PARTS;
    const int first = (int)(blockIdx.x % PARTS) * TPW;
    const int last = first + TPW < TILES ? first + TPW : TILES;
    constexpr int KK = KH * KW;
    constexpr int ROWLEN = OW * KK;
    constexpr unsigned OUTSIDE = 0x80000000u;               // beyond every plane (the host keeps planes below 2 GB)
    const __amdgpu_buffer_rsrc_t xr =
        __builtin_amdgcn_make_buffer_rsrc((void*)(xp + (size_t)plane * (H * W)), 0, (int)(H * W * sizeof(TB)), 0x00020000);
    const __amdgpu_buffer_rsrc_t yr =
        __builtin_amdgcn_make_buffer_rsrc((void*)(yp + (size_t)plane * OH * ROWLEN), 0, (int)(OH * ROWLEN * sizeof(TB)), 0x00020000);
    constexpr int NLOAD = (LH * LW + WTHREADS - 1) / WTHREADS;
    TB pre[NLOAD];
    // whether element i of this lane's share of tile t lies inside the input, and its byte offset there
    auto cell = [&](int t, int i, unsigned& off) -> bool {
        const int e = threadIdx.x + i * WTHREADS;
        const int lr = e / LW, lc = e - lr * LW;
        const int ih = t * TH * SH + CH + lr, iw = CW + lc;
        off = (unsigned)((ih * W + iw) * sizeof(TB));
        return e < LH * LW && ih >= 0 && ih < H && iw >= 0 && iw < W;
    };
    auto fetch = [&](int t) {                               // issues the loads; nothing here looks at a loaded value
#pragma unroll
        for (int i = 0; i < NLOAD; i++) {
            unsigned off;
            const bool inside = cell(t, i, off);
            pre[i] = mjt_win_load(xr, inside ? off : OUTSIDE);
        }
    };
    auto commit = [&](int t, int buf) {
#pragma unroll
        for (int i = 0; i < NLOAD; i++) {
            unsigned off;
            const bool inside = cell(t, i, off);
            if (threadIdx.x + i * WTHREADS < LH * LW) tile[buf][threadIdx.x + i * WTHREADS] = inside ? pre[i] : ov;
        }
    };
    constexpr int NV = (TH * ROWLEN / VEC + WTHREADS - 1) / WTHREADS;    // vectors per lane of a full tile
    fetch(first);
    commit(first, first & 1);
    __syncthreads();
#pragma unroll 1
    for (int t = first; t < last; t++) {
        if (t + 1 < last) fetch(t + 1);                     // (uniform)
        const int oh0 = t * TH;
        const int rows = (OH - oh0) < TH ? (OH - oh0) : TH;
        const int nvec = rows * ROWLEN / VEC;
        const unsigned run0 = (unsigned)(oh0 * ROWLEN * sizeof(TB));
        const TB* __restrict__ cur = tile[t & 1];
#pragma unroll
        for (int j = 0; j < NV; j++) {
            const int q = threadIdx.x + j * WTHREADS;
            const int qc = q < nvec ? q : 0;                // lanes past the end recompute vector 0 and store nowhere
            const int t0 = qc * VEC;
            int r = t0 / ROWLEN;
            int rem = t0 - r * ROWLEN;
            int ow = rem / KK;
            int kk = rem - ow * KK;
            int kh = kk / KW;
            int kw = kk - kh * KW;
            mjt_pack<TB, VEC> out;
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                out.v[k] = cur[(r * SH + kh * DH) * LW + ow * SW + kw * DW];
                // advance to the next element of the run
                kw++;
                if (kw == KW) { kw = 0; kh++; }
                if (kh == KH) { kh = 0; ow++; }
                if (ow == OW) { ow = 0; r++; }
            }
            mjt_win_store(yr, q < nvec ? run0 + (unsigned)(t0 * sizeof(TB)) : OUTSIDE, out);
        }
        if (t + 1 < last) {
            commit(t + 1, (t + 1) & 1);
            // LDS traffic only: a full fence would also wait for the stores of this tile to be acknowledged
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" : : : "memory");
        }
    }
}
