// Generic gather / scatter kernels for arbitrary index expressions
// (reference: python/jittor/src/ops/reindex_op.cc:111-139 and
// python/jittor/src/ops/reindex_reduce_op.cc:93-131).
//
// Constants and fragments supplied by the host:
//   TX, index_t, VEC, NPARAM, SCATTER (0 gather, 1 scatter), LDIM, FLAT_VEC and SAFE_LOAD (gather only)
//   MJT_RX_SETUP    shapes, strides and extras pointers under the names the
//                   index language uses (xshapeK, yshapeK, xstrideK, ystrideK,
//                   XDIM, YDIM, eKp, eKstrideJ)
//   MJT_RX_DECODE   loop coordinates i0..i{LDIM-1} of flat element e; the
//                   innermost one is named ilast_ (the lane's first element)
//   MJT_RX_LASTVAR  name of the innermost coordinate (iN)
//   MJT_RX_INDEX    per element: xid0.., flat xid, bool ov_
//   ATOMIC_UPDATE(addr, v)   scatter only
//   SC_PROLOGUE, MJT_SC_SCALARS, MJT_SC_VALUE   scatter with an element-wise prologue: by-value scalars, and the
//                   statements that compute the scattered value `val_` of element e_ (coordinates i0..) from the
//                   group's inputs
//
// The loop runs over y: the output of a gather, the input of a scatter.  Each
// lane owns VEC adjacent elements of y's innermost axis so that y moves as
// one vector per lane; the x side is accessed element by element.

struct Params { void* a[NPARAM]; };   // 8-byte words; typed as pointers so loads/stores use the global address space

#if REDUCE_TAIL
// Gather fused with the reduce that consumes it (the reference fuses a reindex with its consumer: it is a
// broadcast-type op, executor.cc:555; the pooling group of python/jittor/pool.py:200-208): the loop space y is never
// written.  A lane owns OV adjacent outputs: for each it walks the elements of y's last axes that fold into it, gathers
// them and combines them in TACC, in the order of the flat tail offset.  Extra constants: TZ, TACC, COMBINE(a, x), INIT;
// a[1] is z, a[2] its element count, P_RTAIL / P_RCOUNT the parameter words of the tail length and of 1 / tail length
// (mean); MJT_RX_DECODE_KEPT gives the kept coordinates of output o_, MJT_RX_DECODE_TAIL the folded ones of tail
// offset r (extents as literals).  RTAIL_C > 0: the tail length, known when the kernel is built -- the walk is
// unrolled, out-of-range elements load x[0] and are replaced afterwards, so that the loads of all OV * RTAIL_C
// elements are in flight together (x is not empty then); TAIL_IN is the extent of the innermost folded axis (a window's
// row), loaded as one vector when a wave finds all its rows in range and adjacent in x.  RTAIL_C == 0: a loop of the
// length given at launch.
extern "C" __global__ __launch_bounds__(256) void ENTRY(Params p) {
    const TX* __restrict__ xp = (const TX*)p.a[0];
    TZ* __restrict__ zp = (TZ*)p.a[1];
    const TX ovalue_ = (TX)__longlong_as_double((long long)(unsigned long long)p.a[3]);
    const index_t nout = (index_t)(unsigned long long)p.a[2];
    const index_t rtail = (index_t)(unsigned long long)p.a[P_RTAIL];
    const TACC rcount = (TACC)__longlong_as_double((long long)(unsigned long long)p.a[P_RCOUNT]);
    (void)rcount;
    (void)rtail;
    MJT_RX_SETUP
    const index_t o0 = ((index_t)blockIdx.x * 256 + threadIdx.x) * OV;
    if (o0 >= nout) return;
#if RTAIL_C
    TX got[OV][RTAIL_C];
    bool out_[OV][RTAIL_C];
    index_t at_[OV][RTAIL_C];
    bool runs_ = TAIL_IN > 1;              // every row of the window (TAIL_IN elements, the innermost folded axis) in range and adjacent in x
#pragma unroll
    for (int k = 0; k < OV; k++) {
        const index_t o_ = o0 + k < nout ? o0 + k : nout - 1;
        MJT_RX_DECODE_KEPT
#pragma unroll
        for (int r = 0; r < RTAIL_C; r++) {
            MJT_RX_DECODE_TAIL
            MJT_RX_INDEX
            out_[k][r] = ov_;
            at_[k][r] = ov_ ? (index_t)0 : xid;
            runs_ = runs_ & !ov_ & (at_[k][r] == at_[k][r - r % TAIL_IN] + r % TAIL_IN);
        }
    }
    // decided for the wave as a whole, so that it walks one of the two branches
    if (TAIL_IN > 1 && __builtin_amdgcn_ballot_w64(!runs_) == 0) {
        struct __attribute__((packed, aligned(sizeof(TX)))) mjt_run { TX v[TAIL_IN]; };
#pragma unroll
        for (int k = 0; k < OV; k++)
#pragma unroll
            for (int r = 0; r < RTAIL_C; r += TAIL_IN) {
                index_t first_ = at_[k][r];
                asm volatile("" : "+v"(first_));       // keeps the compiler from folding this branch into the element-wise one
                const mjt_run row_ = *(const mjt_run*)(xp + first_);
#pragma unroll
                for (int s = 0; s < TAIL_IN; s++) got[k][r + s] = row_.v[s];
            }
    } else {
#pragma unroll
        for (int k = 0; k < OV; k++)
#pragma unroll
            for (int r = 0; r < RTAIL_C; r++) got[k][r] = xp[at_[k][r]];
    }
#pragma unroll
    for (int k = 0; k < OV; k++) {
        TACC acc = INIT;
#pragma unroll
        for (int r = 0; r < RTAIL_C; r++) {
            const TX v = out_[k][r] ? ovalue_ : got[k][r];
            acc = (TACC)(COMBINE(acc, v));
        }
        if (o0 + k < nout) zp[o0 + k] = (TZ)acc;
    }
#else
    const index_t o_ = o0;
    MJT_RX_DECODE_KEPT
    TACC acc = INIT;
    for (index_t r = 0; r < rtail; r++) {
        MJT_RX_DECODE_TAIL
        MJT_RX_INDEX
        const TX v = ov_ ? ovalue_ : xp[xid];
        acc = (TACC)(COMBINE(acc, v));
    }
    zp[o_] = (TZ)acc;
#endif
}
#else
extern "C" __global__ __launch_bounds__(256) void ENTRY(Params p) {
#if SCATTER
    TX* __restrict__ xp = (TX*)p.a[0];
    const TX* __restrict__ yp = (const TX*)p.a[1];
#else
    const TX* __restrict__ xp = (const TX*)p.a[0];
    TX* __restrict__ yp = (TX*)p.a[1];
    const TX ovalue_ = (TX)__longlong_as_double((long long)(unsigned long long)p.a[3]);
#endif
    const index_t nvec = (index_t)(unsigned long long)p.a[2];
    MJT_RX_SETUP
    const index_t j = (index_t)blockIdx.x * 256 + threadIdx.x;
    if (j >= nvec) return;
#if !SCATTER && SAFE_LOAD && (FLAT_VEC || VEC > 1)
    // A gather of a non-empty x with several elements per lane.  FLAT_VEC: the innermost extent does not divide into full
    // vectors while y as a whole does -- the lane's VEC elements are adjacent in y's memory and may lie in two rows, so
    // each one is decoded by itself; otherwise they share a row and differ in the innermost coordinate only.  When all
    // of them are in range and adjacent in x as well (the inside of a padded, cropped or shifted row) they arrive as one
    // load (a flipped row, descending addresses, gains nothing from the same: 45.9 us either way for [64,512,1024]);
    // when the even and the odd ones are each adjacent (two sources woven column by column, or every source element
    // taken twice) they arrive as two loads of half a vector; otherwise out-of-range elements load x[0] and are
    // replaced afterwards, which keeps the VEC loads in flight together.
    const index_t ebase_ = j * VEC;
    mjt_pack<TX, VEC> yv;
    bool out_[VEC];
    index_t at_[VEC];
    bool run_ = true;                      // all in range and adjacent in x: one load of the whole vector
    bool twin_ = VEC >= 4;                 // all in range, the even and the odd ones each adjacent in x: two loads of half a vector
#if !FLAT_VEC
    const index_t e = ebase_;
    MJT_RX_DECODE
#endif
#pragma unroll
    for (int k = 0; k < VEC; k++) {
#if FLAT_VEC
        const index_t e = ebase_ + k;
        MJT_RX_DECODE
        const index_t MJT_RX_LASTVAR = ilast_;
#else
        const index_t MJT_RX_LASTVAR = ilast_ + k;
#endif
        MJT_RX_INDEX
        out_[k] = ov_;
        at_[k] = ov_ ? (index_t)0 : xid;
        run_ = run_ & !ov_ & (at_[k] == at_[0] + k);
        twin_ = twin_ & !ov_ & (k < 2 || at_[k] == at_[k - 2] + 1);
    }
    // decided for the wave as a whole: with both kinds of lanes in a wave it would walk both branches (rows of 66
    // elements: nearly every wave has a lane at a row's end)
    if (__builtin_amdgcn_ballot_w64(!run_) == 0) {
        // x + at_[0] is aligned for one element only
        struct __attribute__((packed, aligned(sizeof(TX)))) mjt_run { TX v[VEC]; };
        index_t first_ = at_[0];
        asm volatile("" : "+v"(first_));       // keeps the compiler from folding this branch into the element-wise one
        const mjt_run got_ = *(const mjt_run*)(xp + first_);
#pragma unroll
        for (int k = 0; k < VEC; k++) yv.v[k] = got_.v[k];
    } else if (VEC >= 4 && __builtin_amdgcn_ballot_w64(!twin_) == 0) {
        // two runs woven into each other (columns interleaved from two sources, every source element taken twice)
        struct __attribute__((packed, aligned(sizeof(TX)))) mjt_half_run { TX v[VEC / 2 > 0 ? VEC / 2 : 1]; };
        index_t even_ = at_[0], odd_ = at_[1];
        asm volatile("" : "+v"(even_), "+v"(odd_));
        const mjt_half_run a_ = *(const mjt_half_run*)(xp + even_);
        const mjt_half_run b_ = *(const mjt_half_run*)(xp + odd_);
#pragma unroll
        for (int k = 0; k < VEC; k++) yv.v[k] = (k & 1) ? b_.v[k / 2] : a_.v[k / 2];
    } else {
#pragma unroll
        for (int k = 0; k < VEC; k++) yv.v[k] = xp[at_[k]];
#pragma unroll
        for (int k = 0; k < VEC; k++)
            if (out_[k]) yv.v[k] = ovalue_;
    }
    mjt_store(yp + ebase_, yv);
    return;
#else
    const index_t e = j * VEC;
    MJT_RX_DECODE
    mjt_pack<TX, VEC> yv;
#if SCATTER && SC_PROLOGUE
    MJT_SC_SCALARS
    (void)yp;
#elif SCATTER
    mjt_load(yv, yp + e);
#endif
#pragma unroll
    for (int k = 0; k < VEC; k++) {
        const index_t MJT_RX_LASTVAR = ilast_ + k;
        MJT_RX_INDEX
#if SCATTER && SC_PROLOGUE
        // the scattered value is computed here from the group's inputs (MJT_SC_VALUE leaves it in val_): only for
        // elements that land somewhere, so a gathered input is always read inside its tensor
        if (!ov_) {
            const index_t e_ = e + k;
            (void)e_;
            MJT_SC_VALUE
            ATOMIC_UPDATE(xp + xid, val_);
        }
#elif SCATTER
        if (!ov_) { ATOMIC_UPDATE(xp + xid, yv.v[k]); }
#else
#if SAFE_LOAD
        // x is not empty: an out-of-range element loads x[0] and is replaced, so no branch separates the lane's loads
        const TX got_ = xp[ov_ ? (index_t)0 : xid];
        yv.v[k] = ov_ ? ovalue_ : got_;
#else
        if (ov_) yv.v[k] = ovalue_; else yv.v[k] = xp[xid];
#endif
#endif
    }
#if !SCATTER
    mjt_store(yp + e, yv);
#endif
#endif
}
#endif
