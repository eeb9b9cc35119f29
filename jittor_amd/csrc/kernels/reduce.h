// Axis-set reduction kernels (reference semantics:
// python/jittor/src/ops/reduce_op.cc:374-399 -- identity, then
// y[kept] = OP(y[kept], x[kept, reduced]) with the accumulator in Ty).
//
// Specialised at run time through these macros:
//   TX, TY          element types of x and y
//   TACC            accumulator type: TY, or float when TY is a 16-bit float type (the sum is
//                   rounded to TY once, at the store)
//   index_t         int or long long
//   NK, NR          number of merged kept / reduced axes (each 0..5, NR >= 1)
//   VEC             elements per vector load
//   G               lanes that cooperate on one output (row kernel), power of 2 <= 64
//   SPLIT           1: several workgroup rows share one output and write partials
//   COMBINE(a, x)   first-level update, a is TACC, x is TX
//   MERGE(a, b)     update between two partial results, both TACC
//   INIT            identity, TACC
//   ROW             1: innermost merged axis is reduced; 0: it is kept
//   UNR             independent loads per lane and step (row kernel)
//   MJT_LD          mjt_load or mjt_load_nt (streaming input)
//   NPRO, MJT_PRO_SCALARS, MJT_RD(dst, off)
//                   element-wise prologue (a fused group whose only consumer is
//                   this reduce, python/jittor/src/executor.cc:555): NPRO extra
//                   parameter words, by-value scalars, and the statement that
//                   fills the pack `dst` with the elements at offset `off` --
//                   one vector load per prologue input, then the op chain.
//                   MJT_PRO_PER_OUTPUT loads the prologue inputs that are broadcast
//                   along exactly the reduced axes (one value per output: the
//                   mean in a variance, the maximum in a softmax) once, at output
//                   index `o`.  Without a prologue MJT_RD is a plain load from x.
//
// The host merges adjacent axes of equal kind, so kept and reduced axes
// alternate.  Row kernel: G lanes stride over the contiguous reduced run with
// VEC-wide loads and finish with a cross-lane xor-shuffle tree, no LDS.
// Column kernel: each lane owns VEC adjacent outputs and walks the reduced
// coordinates; lanes of a wave read one contiguous run per step.
// When SPLIT is set the partials go to a scratch buffer and a second launch of
// the same kernel family folds them (two-pass grid reduce).

#ifndef NPRO
#define NPRO 0
#define MJT_PRO_SCALARS
#define MJT_PRO_PER_OUTPUT
#define MJT_RD(dst, off) MJT_LD(dst, xp + (off))
#endif
struct Params { void* a[8 + 6 * 5 + NPRO]; };   // 8-byte words; typed as pointers so loads/stores use the global address space
// a[0] x, a[1] y or partials, a[2] O (outputs), a[3] S (splits), a[4] rcount (double bits),
// a[5] work items per split, a[6] total work items,
// a[8+0*5..]  kshape   a[8+1*5..] kstride (in x)   a[8+2*5..] kdiv
// a[8+3*5..]  rshape   a[8+4*5..] rstride (in x)   a[8+5*5..] rdiv
// a[38..]     prologue inputs (pointers) and scalars

#if USE64
#define MJT_DIVQ(n, k, tab) ((n) / (index_t)(unsigned long long)p.a[8 + ((tab)-2) * 5 + (k)])
#else
#define MJT_DIVQ(n, k, tab) ((index_t)mjt_div((unsigned)(n), mjt_unpack_divmod((unsigned long long)p.a[8 + (tab) * 5 + (k)], 0)))
#endif

template <class T> __device__ __forceinline__ T mjt_shfl_xor_any(T v, int off) {
    if constexpr (sizeof(T) == 8) {
        long long t;
        __builtin_memcpy(&t, &v, 8);
        t = __shfl_xor(t, off, 64);
        __builtin_memcpy(&v, &t, 8);
        return v;
    } else {
        int t = 0;
        __builtin_memcpy(&t, &v, sizeof(T));
        t = __shfl_xor(t, off, 64);
        __builtin_memcpy(&v, &t, sizeof(T));
        return v;
    }
}

__device__ __forceinline__ index_t mjt_kept_offset(const Params& p, index_t o) {
    index_t off = 0;
#pragma unroll
    for (int k = NK - 1; k >= 0; k--) {
        index_t shape = (index_t)(unsigned long long)p.a[8 + 0 * 5 + k];
        index_t q = (k == 0) ? 0 : MJT_DIVQ(o, k, 2);
        index_t c = (k == 0) ? o : o - q * shape;
        off += c * (index_t)(unsigned long long)p.a[8 + 1 * 5 + k];
        o = q;
    }
    return off;
}

// offset of reduced coordinate `r` counted over the first `nd` reduced axes
template <int ND> __device__ __forceinline__ index_t mjt_red_offset(const Params& p, index_t r) {
    index_t off = 0;
#pragma unroll
    for (int k = ND - 1; k >= 0; k--) {
        index_t shape = (index_t)(unsigned long long)p.a[8 + 3 * 5 + k];
        index_t q = (k == 0) ? 0 : MJT_DIVQ(r, k, 5);
        index_t c = (k == 0) ? r : r - q * shape;
        off += c * (index_t)(unsigned long long)p.a[8 + 4 * 5 + k];
        r = q;
    }
    return off;
}

#if ROW
// G lanes share one output: up to a wave (shuffles only), or 128 .. 1024 lanes (whole waves; their results meet in
// LDS).  Wide groups are for long rows streamed from memory: a lane then has one batch of UNR loads instead of
// several, and the memory system serves many lanes with few loads each faster than few lanes with many
// (a plain read of 134 MB: 64 lanes x 16 loads per workgroup 21.6 us, 128 x 8 20.4 us).
#define BLK (G > 256 ? G : 256)
extern "C" __global__ __launch_bounds__(BLK) void ENTRY(Params p) {
    const TX* __restrict__ xp = (const TX*)p.a[0];
    TY* __restrict__ yp = (TY*)p.a[1];
    const index_t O = (index_t)(unsigned long long)p.a[2];
    const index_t S = (index_t)(unsigned long long)p.a[3];
    const TACC rcount = (TACC)__longlong_as_double((long long)(unsigned long long)p.a[4]);
    (void)rcount;
    (void)xp;
    MJT_PRO_SCALARS
    const unsigned lane = threadIdx.x % G;
    const index_t o = (index_t)blockIdx.x * (BLK / G) + threadIdx.x / G;
    const index_t s = blockIdx.y;
    TACC acc[VEC];
#pragma unroll
    for (int k = 0; k < VEC; k++) acc[k] = INIT;
    if (o < O) {
        MJT_PRO_PER_OUTPUT
        const index_t kbase = mjt_kept_offset(p, o);
        const index_t L = (index_t)(unsigned long long)p.a[8 + 3 * 5 + (NR - 1)];
        const index_t nL = (L + (G * VEC) - 1) / (G * VEC);
        const index_t per = (index_t)(unsigned long long)p.a[5];
        const index_t total = (index_t)(unsigned long long)p.a[6];
        index_t it = s * per;
        index_t it_end = it + per < total ? it + per : total;
        index_t ro = (NR == 1) ? 0 : it / nL;
        index_t lc = (NR == 1) ? it : it - ro * nL;
        while (it < it_end) {
            const index_t row = kbase + ((NR == 1) ? 0 : mjt_red_offset<(NR > 1 ? NR - 1 : 1)>(p, ro));
            index_t lc_end = nL - lc < it_end - it ? nL : lc + (it_end - it);
            it += lc_end - lc;
            // full steps: every lane in range, UNR independent loads in flight
            const index_t nfull = L / (G * VEC);
            for (; lc + UNR <= lc_end && lc + UNR <= nfull; lc += UNR) {
                mjt_pack<TX, VEC> v[UNR];
#pragma unroll
                for (int u = 0; u < UNR; u++) MJT_RD(v[u], row + ((lc + u) * G + lane) * VEC);
#pragma unroll
                for (int u = 0; u < UNR; u++)
#pragma unroll
                    for (int k = 0; k < VEC; k++) acc[k] = (TACC)(COMBINE(acc[k], v[u].v[k]));
            }
            for (; lc < lc_end; lc++) {
                index_t l = (lc * G + lane) * VEC;
                if (l < L) {
                    mjt_pack<TX, VEC> v;
                    MJT_RD(v, row + l);
#pragma unroll
                    for (int k = 0; k < VEC; k++) acc[k] = (TACC)(COMBINE(acc[k], v.v[k]));
                }
            }
            lc = 0;
            ro++;
        }
    }
    TACC r = acc[0];
#pragma unroll
    for (int k = 1; k < VEC; k++) r = (TACC)(MERGE(r, acc[k]));
#pragma unroll
    for (int off = (G < 64 ? G : 64) / 2; off > 0; off >>= 1) {
        TACC other = mjt_shfl_xor_any(r, off);
        r = (TACC)(MERGE(r, other));
    }
#if G > 64
    __shared__ TACC part[BLK / 64];
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = r;
    __syncthreads();
    if (lane == 0) {
#pragma unroll
        for (int j = 1; j < G / 64; j++) r = (TACC)(MERGE(r, part[(threadIdx.x >> 6) + j]));
    }
#endif
    if (lane == 0 && o < O) yp[SPLIT ? o * S + s : o] = (TY)r;
}
#else
extern "C" __global__ __launch_bounds__(256) void ENTRY(Params p) {
    const TX* __restrict__ xp = (const TX*)p.a[0];
    TY* __restrict__ yp = (TY*)p.a[1];
    const index_t O = (index_t)(unsigned long long)p.a[2];
    const TACC rcount = (TACC)__longlong_as_double((long long)(unsigned long long)p.a[4]);
    (void)rcount;
    (void)xp;
    MJT_PRO_SCALARS
    // G lanes across the outputs (a power of two up to 256, or 1 for 256): with fewer than 256 vectors of outputs the
    // rest of the workgroup takes other slices of the rows instead of idling
    constexpr int TXL = G > 1 ? G : 256;
    const index_t o = ((index_t)blockIdx.x * TXL + threadIdx.x % TXL) * VEC;
    const index_t s = (index_t)blockIdx.y * (256 / TXL) + threadIdx.x / TXL;
    if (o >= O || (SPLIT && s >= (index_t)(unsigned long long)p.a[3])) return;
    MJT_PRO_PER_OUTPUT
    const index_t kbase = mjt_kept_offset(p, o);
    const index_t per = (index_t)(unsigned long long)p.a[5];
    const index_t total = (index_t)(unsigned long long)p.a[6];
    index_t r = s * per;
    const index_t r_end = r + per < total ? r + per : total;
    TACC acc[VEC];
#pragma unroll
    for (int k = 0; k < VEC; k++) acc[k] = INIT;
#pragma unroll 4
    for (; r < r_end; r++) {
        index_t roff = (NR == 1) ? r * (index_t)(unsigned long long)p.a[8 + 4 * 5] : mjt_red_offset<NR>(p, r);
        mjt_pack<TX, VEC> v;
        MJT_RD(v, kbase + roff);
#pragma unroll
        for (int k = 0; k < VEC; k++) acc[k] = (TACC)(COMBINE(acc[k], v.v[k]));
    }
#if SPLIT && SPLIT_T
    // many slices: partial sums go out as [O, S], the layout the row kernel folds (S contiguous per output): a fold that
    // walked S rows of an [S, O] array with one lane per output would be one long chain of dependent loads
    const index_t S = (index_t)(unsigned long long)p.a[3];
#pragma unroll
    for (int k = 0; k < VEC; k++) yp[(o + k) * S + s] = (TY)acc[k];
#else
    mjt_pack<TY, VEC> out;                      // [O], or with a few slices [S, O], folded by this kernel
#pragma unroll
    for (int k = 0; k < VEC; k++) out.v[k] = (TY)acc[k];
    mjt_store(yp + (SPLIT ? s * O : 0) + o, out);
#endif
}
#endif
