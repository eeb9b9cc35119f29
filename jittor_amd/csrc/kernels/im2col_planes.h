// Shifted input planes, taps outermost: y[g, c, kh, kw, i, oh, ow] = x[g*NB + i, c, oh*SH + kh*DH + CH, ow*SW + kw*DW + CW]
// with the overflow value outside x -- the column matrices [(c, kh, kw), pixels] of a convolution, per image (NB = 1),
// for the whole batch (one group) or per chunk of NB images laid side by side.  Like the sliding-window gather it is
// an affine special case of the gather op (reference: python/jittor/src/ops/reindex_op.cc:111-139); there the taps are
// the innermost axes of y, here the pixels are, so every (c, tap) owns one contiguous run of NB * OH * OW elements.
//
// Baked in by the host: H, W, OH, OW, KH, KW, SH, SW, DH, DW, CH, CW, NB, LH x LW (a padded plane in LDS), TB (an
// element as raw bits), VEC (elements per store: the runs start on vector boundaries), THREADS.
//
// A workgroup owns one (g, c): it stages the NB planes of channel c in LDS, cells outside x holding the overflow value
// (so that no bounds test is left in the store loop), then writes the KH*KW runs, which follow one another in y, as
// vectors: a lane finds (tap, image, oh, ow) of a vector's first element by constant division and steps from there.
struct Params { void* a[4]; };   // x, y, overflow bits, channels

extern "C" __global__ __launch_bounds__(THREADS) void ENTRY(Params p) {
    const TB* __restrict__ xp = (const TB*)p.a[0];
    TB* __restrict__ yp = (TB*)p.a[1];
    const TB ov = (TB)(unsigned long long)p.a[2];
    const unsigned C = (unsigned)(unsigned long long)p.a[3];
    __shared__ TB planes[NB * LH * LW];
    constexpr int KK = KH * KW, P = OH * OW, RUN = NB * P;
    const unsigned g = blockIdx.x / C, c = blockIdx.x - g * C;
    for (int e = threadIdx.x; e < NB * LH * LW; e += THREADS) {
        const int i = e / (LH * LW), cell = e - i * (LH * LW);
        const int lr = cell / LW, lc = cell - lr * LW;
        const int ih = lr + CH, iw = lc + CW;
        const bool inside = ih >= 0 && ih < H && iw >= 0 && iw < W;
        const size_t plane = ((size_t)g * NB + i) * C + c;
        planes[e] = inside ? xp[plane * (H * W) + ih * W + iw] : ov;
    }
    __syncthreads();
    TB* __restrict__ out = yp + (size_t)blockIdx.x * ((size_t)KK * RUN);
    constexpr int VPR = RUN / VEC;                            // vectors per run
    for (int q = threadIdx.x; q < KK * VPR; q += THREADS) {
        const int kk = q / VPR, e0 = (q - kk * VPR) * VEC;
        const int kh = kk / KW, kw = kk - kh * KW;
        int i = e0 / P;
        const int px = e0 - i * P;
        int oh = px / OW, ow = px - oh * OW;
        mjt_pack<TB, VEC> v;
#pragma unroll
        for (int k = 0; k < VEC; k++) {
            v.v[k] = planes[i * (LH * LW) + (oh * SH + kh * DH) * LW + ow * SW + kw * DW];
            ow++;
            if (ow == OW) { ow = 0; oh++; }
            if (oh == OH) { oh = 0; i++; }
        }
        mjt_store(out + (size_t)kk * RUN + e0, v);             // (plain stores: the product that follows reads y from the caches)
    }
}
