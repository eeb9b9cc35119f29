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
// One workgroup owns TH output rows of one plane.  It stages the input rows
// they touch in LDS once (out-of-range cells hold the overflow value, so no
// bounds test is left in the inner loop), then writes its part of y, which is
// one contiguous run of TH*OW*KH*KW elements, as 16-byte vectors: lane l owns
// vectors l, l+256, ... of that run and finds (row, ow, kh, kw) of each
// element by constant division.

struct Params { void* a[4]; };   // 8-byte words; typed as pointers so loads/stores use the global address space   // x, y, overflow bits, number of planes

extern "C" __global__ __launch_bounds__(WTHREADS) void ENTRY(Params p) {
    const TB* __restrict__ xp = (const TB*)p.a[0];
    TB* __restrict__ yp = (TB*)p.a[1];
    const TB ov = (TB)(unsigned long long)p.a[2];
    __shared__ TB tile[LH * LW];
    constexpr int TILES = (OH + TH - 1) / TH;
    const unsigned plane = blockIdx.x / TILES;
    const int oh0 = (int)(blockIdx.x % TILES) * TH;
    const int rows = (OH - oh0) < TH ? (OH - oh0) : TH;
    const int ih0 = oh0 * SH + CH;          // input row of LDS row 0
    const TB* __restrict__ xplane = xp + (size_t)plane * (H * W);
    for (int t = threadIdx.x; t < LH * LW; t += WTHREADS) {
        const int lr = t / LW, lc = t - lr * LW;
        const int ih = ih0 + lr, iw = CW + lc;
        TB v = ov;
        if (ih >= 0 && ih < H && iw >= 0 && iw < W) v = xplane[ih * W + iw];
        tile[t] = v;
    }
    __syncthreads();
    constexpr int KK = KH * KW;
    constexpr int ROWLEN = OW * KK;
    const int nvec = rows * ROWLEN / VEC;
    TB* __restrict__ yrun = yp + ((size_t)plane * OH + oh0) * ROWLEN;
    for (int q = threadIdx.x; q < nvec; q += WTHREADS) {
        const int t0 = q * VEC;
        int r = t0 / ROWLEN;
        int rem = t0 - r * ROWLEN;
        int ow = rem / KK;
        int kk = rem - ow * KK;
        int kh = kk / KW;
        int kw = kk - kh * KW;
        mjt_pack<TB, VEC> out;
#pragma unroll
        for (int k = 0; k < VEC; k++) {
            out.v[k] = tile[(r * SH + kh * DH) * LW + ow * SW + kw * DW];
            // advance to the next element of the run
            kw++;
            if (kw == KW) { kw = 0; kh++; }
            if (kh == KH) { kh = 0; ow++; }
            if (ow == OW) { ow = 0; r++; }
        }
        mjt_store_nt(yrun + t0, out);
    }
}
