// Permutation of axes through LDS tiles: y[i0, .., i(n-1)] = x[i_perm[0], .., i_perm[n-1]], the special case of the
// gather op (reference: python/jittor/src/ops/reindex_op.cc:111-139) whose index expressions are the output
// coordinates in another order (transpose, permute).  The generic kernel gives every output element a lane, which
// reads x with the stride of whatever axis became innermost: one cache line per lane.  Here a workgroup moves a
// TILE x TILE piece spanned by x's innermost axis (axis A of the tile, extent LA) and by the x axis that becomes y's
// innermost one (axis B, extent LB): it reads rows along A (contiguous in x), keeps them in LDS, and writes rows
// along B (contiguous in y).  All other axes only select the piece.
//
// Baked in by the host (adjacent axes that stay adjacent are merged first): TB (element as raw bits), ND, LA, LB,
// XSTR_B (stride of axis B in x), YSTR_A (stride of axis A in y), NOTH other axes with extents OEXT[], x strides
// OXS[], y strides OYS[].
struct Params { void* a[4]; };   // x, y

#define TILE 64
extern "C" __global__ __launch_bounds__(256) void ENTRY(Params p) {
    const TB* __restrict__ xp = (const TB*)p.a[0];
    TB* __restrict__ yp = (TB*)p.a[1];
    __shared__ TB tile[TILE][TILE + (sizeof(TB) >= 4 ? 1 : 2)];      // odd word stride: columns spread over the banks
    constexpr long long TA = (LA + TILE - 1) / TILE, TBN = (LB + TILE - 1) / TILE;
    long long rest = blockIdx.x;
    const int ta = (int)(rest % TA);
    rest /= TA;
    const int tb = (int)(rest % TBN);
    rest /= TBN;
    long long xbase = 0, ybase = 0;
#if NOTH > 0
    constexpr long long oext[NOTH] = {OEXT}, oxs[NOTH] = {OXS}, oys[NOTH] = {OYS};
#pragma unroll
    for (int d = NOTH - 1; d >= 0; d--) {
        const long long c = rest % oext[d];
        rest /= oext[d];
        xbase += c * oxs[d];
        ybase += c * oys[d];
    }
#endif
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const long long a0 = (long long)ta * TILE, b0 = (long long)tb * TILE;
    // rows along A: element (b0 + r, a0 + tx) of x
    TB v[TILE / 4];
#pragma unroll
    for (int k = 0; k < TILE / 4; k++) {
        const int r = ty + 4 * k;
        const bool in = b0 + r < LB && a0 + tx < LA;
        v[k] = in ? xp[xbase + (b0 + r) * (long long)XSTR_B + a0 + tx] : (TB)0;
    }
#pragma unroll
    for (int k = 0; k < TILE / 4; k++) tile[ty + 4 * k][tx] = v[k];
    __syncthreads();
    // rows along B: element (a0 + r, b0 + tx) of y
#pragma unroll
    for (int k = 0; k < TILE / 4; k++) {
        const int r = ty + 4 * k;
        if (a0 + r < LA && b0 + tx < LB) yp[ybase + (a0 + r) * (long long)YSTR_A + b0 + tx] = tile[tx][r];
    }
}
