// Scatter through a window pattern, turned into a gather
// (reference: python/jittor/src/ops/reindex_reduce_op.cc:93-131; the gradient of pooling, python/jittor/pool.py:200-208).
//
// x[b.., oh*SH + kh*DH + CH, ow*SW + kw*DW + CW] op= y[b.., oh, ow, kh, kw]: with windows that overlap, neighbouring
// elements of y meet in the same element of x and atomic updates queue up behind each other.  Every element of x knows
// which windows reach it, so one lane per element of x folds them itself: no atomics, no identity fill, one coalesced
// store.  Row h is reached from output row oh through tap kh when oh*SH + kh*DH + CH == h; the candidates are the NCH
// output rows at and below (h - CH) / SH (NCH = (KH-1)*DH / SH + 1), likewise for columns.
//
// Constants and fragments supplied by the host:
//   TX, TACC, index_t, VEC, NPARAM, NB (batch axes), KH, KW, SH, SW, DH, DW, CH, CW, NCH, NCW
//   MJT_RX_SETUP    xshapeK, yshapeK and strides (the names the index language uses)
//   MJT_WS_BATCH    coordinates i0 .. i{NB-1} of plane number plane_
//   I_OH, I_OW, I_KH, I_KW   the names of the four window coordinates (i{NB} .. i{NB+3})
//   INIT, COMBINE(a, v)
//   SC_PROLOGUE, MJT_SC_SCALARS, MJT_SC_VALUE   as in the generic scatter kernel: the scattered value `val_` of element e_
//                   of y, computed from the group's inputs (a gathered input is read at xid, which is this lane's element)
//
// A candidate that does not exist is computed at clamped coordinates and dropped afterwards, so that no branch separates
// the loads of a lane.

struct Params { void* a[NPARAM]; };

extern "C" __global__ __launch_bounds__(256) void ENTRY(Params p) {
    TX* __restrict__ xp = (TX*)p.a[0];
    const TX* __restrict__ yp = (const TX*)p.a[1];
    (void)yp;
    const index_t nx = (index_t)(unsigned long long)p.a[2];
    MJT_RX_SETUP
#if SC_PROLOGUE
    MJT_SC_SCALARS
#endif
    // a lane owns VEC adjacent elements of a row of x (W is a multiple of VEC) and stores them as one vector
    const index_t xbase_ = ((index_t)blockIdx.x * 256 + threadIdx.x) * VEC;
    if (xbase_ >= nx) return;
    const index_t H_ = xshape_h, W_ = xshape_w, OH_ = yshape_oh, OW_ = yshape_ow;
    const index_t w0_ = xbase_ % W_;
    const index_t t_ = xbase_ / W_;
    const index_t h_ = t_ % H_;
    const index_t plane_ = t_ / H_;
    MJT_WS_BATCH
    const index_t th_ = h_ - (CH);
    const index_t oh_hi = th_ >= 0 ? th_ / SH : (index_t)-1;
    mjt_pack<TX, VEC> out_;
#pragma unroll
    for (int k = 0; k < VEC; k++) {
        const index_t xid = xbase_ + k;
        const index_t tw_ = w0_ + k - (CW);
        const index_t ow_hi = tw_ >= 0 ? tw_ / SW : (index_t)-1;
        TACC acc = INIT;
#pragma unroll
        for (int a = 0; a < NCH; a++) {
            const index_t oh_c = oh_hi - a;
            const index_t rh_ = th_ - oh_c * SH;                   // kh * DH, if this candidate exists
            const bool ok_h = oh_c >= 0 && oh_c < OH_ && rh_ % DH == 0 && rh_ / DH < KH;
            const index_t I_OH = ok_h ? oh_c : (index_t)0;
            const index_t I_KH = ok_h ? rh_ / DH : (index_t)0;
#pragma unroll
            for (int b = 0; b < NCW; b++) {
                const index_t ow_c = ow_hi - b;
                const index_t rw_ = tw_ - ow_c * SW;
                const bool ok_w = ow_c >= 0 && ow_c < OW_ && rw_ % DW == 0 && rw_ / DW < KW;
                const index_t I_OW = ok_w ? ow_c : (index_t)0;
                const index_t I_KW = ok_w ? rw_ / DW : (index_t)0;
                const index_t e_ = (((plane_ * OH_ + I_OH) * OW_ + I_OW) * KH + I_KH) * KW + I_KW;
#if SC_PROLOGUE
                MJT_SC_VALUE
#else
                const TX val_ = yp[e_];
#endif
                const TACC next_ = (TACC)(COMBINE(acc, val_));
                acc = ok_h && ok_w ? next_ : acc;
            }
        }
        out_.v[k] = (TX)acc;
    }
    mjt_store(xp + xbase_, out_);
}
