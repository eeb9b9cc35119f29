// CPU restatement of the reference's JIT kernel templates for the five
// benchmark configurations.  TEST INFRASTRUCTURE ONLY: used by tests, the smoke
// check and the cpu_baseline leg of the bench; never by the product path.
//
// Each function is the loop nest the reference's template expands to for that
// configuration (citations are relative to python/jittor/src/ of the reference
// tree), with the element-wise formulas of type/common_op_type.cc:82-152.  The
// reference compiles such kernels with g++ -std=c++14 -Ofast -march=native
// -fopenmp (python/jittor/compiler.py:1029-1032,1069-1074,1165-1170); this file
// is built with the same flags except -march=x86-64-v3 (the build machine and
// the machine it runs on differ).  `threads` = 1 is the reference's default
// (loop option parallel = 0, opt/pass/loop_to_func_pass.cc:17-21); threads > 1
// is its compile_options={"parallel":1} mode: OpenMP over the outermost
// independent loop.
//
// Pin status: every function here is checked against oracle.py (itself pinned
// by closed forms and the reference's known-answer vectors) in
// tests/test_oracle_kernels.py.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <omp.h>

typedef int index_t;   // op.cc:158-192: int32 unless a Var has >= 2^31 elements

extern "C" {

// ops/reduce_op.cc:374-399 with Tx=Ty=float32, OP=add, DIM=2, REDUCE=0b10
void ork_reduce_sum_axis1(const float* __restrict__ xp, float* __restrict__ yp, index_t xshape0, index_t xshape1,
                          int threads) {
    index_t ystride0 = 1, xstride1 = 1, xstride0 = xshape1;
#pragma omp parallel for num_threads(threads) if (threads > 1)
    for (index_t xi0 = 0; xi0 < xshape0; xi0++) yp[xi0 * ystride0] = float(0);
#pragma omp parallel for num_threads(threads) if (threads > 1)
    for (index_t xi0 = 0; xi0 < xshape0; xi0++)
        for (index_t xi1 = 0; xi1 < xshape1; xi1++) {
            index_t yid = xi0 * ystride0;
            index_t xid = xi0 * xstride0 + xi1 * xstride1;
            yp[yid] = ((yp[yid]) + (xp[xid]));
        }
}

// ops/reindex_op.cc:111-139 with XDIM=4, YDIM=6,
// INDEX = i0, i1, i2+i4-1, i3+i5-1, OVERFLOW=0
void ork_reindex_im2col3x3(const float* __restrict__ xp, float* __restrict__ yp, index_t N, index_t C, index_t H,
                           index_t W, int threads) {
    const index_t yshape0 = N, yshape1 = C, yshape2 = H, yshape3 = W, yshape4 = 3, yshape5 = 3;
    const index_t ystride5 = 1, ystride4 = 3, ystride3 = 9, ystride2 = 9 * W, ystride1 = 9 * W * H,
                  ystride0 = 9 * W * H * C;
    const index_t xshape0 = N, xshape1 = C, xshape2 = H, xshape3 = W;
    const index_t xstride3 = 1, xstride2 = W, xstride1 = W * H, xstride0 = W * H * C;
#pragma omp parallel for num_threads(threads) if (threads > 1)
    for (index_t i0 = 0; i0 < yshape0; i0++)
        for (index_t i1 = 0; i1 < yshape1; i1++)
            for (index_t i2 = 0; i2 < yshape2; i2++)
                for (index_t i3 = 0; i3 < yshape3; i3++)
                    for (index_t i4 = 0; i4 < yshape4; i4++)
                        for (index_t i5 = 0; i5 < yshape5; i5++) {
                            index_t yid = i0 * ystride0 + i1 * ystride1 + i2 * ystride2 + i3 * ystride3 + i4 * ystride4 +
                                          i5 * ystride5;
                            index_t xid0 = i0, xid1 = i1, xid2 = i2 + i4 - 1, xid3 = i3 + i5 - 1;
                            index_t xid = xid0 * xstride0 + xid1 * xstride1 + xid2 * xstride2 + xid3 * xstride3;
                            bool check_overflow = 0 || xid0 < 0 || xid0 >= xshape0 || xid1 < 0 || xid1 >= xshape1 ||
                                                  xid2 < 0 || xid2 >= xshape2 || xid3 < 0 || xid3 >= xshape3;
                            yp[yid] = check_overflow ? float(0) : xp[xid];
                        }
}

// ops/reindex_reduce_op.cc:93-131 with YDIM=1, XDIM=1, INDEX0=@e0(i0),
// Te0=int32; op 0 = add, 1 = maximum.  The update loop carries a dependence
// through x, so the reference runs it on one thread in either mode.
void ork_scatter_1d(const float* __restrict__ yp, const int* __restrict__ extras0p, float* __restrict__ xp,
                    index_t yshape0, index_t xshape0, int op) {
    for (index_t i0 = 0; i0 < xshape0; i0++)
        xp[i0] = op == 0 ? float(0) : std::numeric_limits<float>::lowest();
    for (index_t i0 = 0; i0 < yshape0; i0++) {
        index_t yid = i0;
        index_t xid0 = extras0p[i0 * 1];
        index_t xid = xid0;
        bool check_overflow = 0 || xid0 < 0 || xid0 >= xshape0;
        if (!check_overflow) {
            if (op == 0) xp[xid] = ((xp[xid]) + (yp[yid]));
            else xp[xid] = std::max(float(xp[xid]), float(yp[yid]));
        }
    }
}

// Fused group of python/jittor/nn.py:182-183 relu + exp, sigmoid, multiply:
//   t = x*scale + bias; r = (t > 0) ? t : 0; out = exp(-r) * sigmoid(x)
// one loop nest, intermediates as scalars (opt/pass/remove_intermediate_pass.cc:26-47);
// broadcasts index with masks 0b101 and 0b011 (ops/broadcast_to_op.cc:177-194).
void ork_fused_chain(const float* __restrict__ xp, const float* __restrict__ scalep, const float* __restrict__ biasp,
                     float* __restrict__ zp, index_t s0, index_t s1, index_t s2, int threads) {
#pragma omp parallel for num_threads(threads) if (threads > 1)
    for (index_t i0 = 0; i0 < s0; i0++)
        for (index_t i1 = 0; i1 < s1; i1++)
            for (index_t i2 = 0; i2 < s2; i2++) {
                index_t id = (i0 * s1 + i1) * s2 + i2;
                float x = xp[id];
                float t = ((((x) * (scalep[i1]))) + (biasp[i2]));
                bool c = ((t) > (float(0)));
                float r = c ? t : float(0);
                float e = std::exp((float)((-(r))));
                float sg = ((float)(1.0f / (1.0f + std::exp(std::min(float(-(x)), float(30))))));
                zp[id] = ((e) * (sg));
            }
}

// The meta-op convolution group of python/jittor/nn.py:1251-1262 for bfloat16
// inputs: reindex + broadcast + multiply + reduce.add over (c, kh, kw), float
// products and a float32 accumulator (opt/kernel_ir.cc:958-968,
// ops/reduce_op.cc:259-266), bfloat16 <-> float by bit shifts
// (type/fp16_compute.h:235-252).  x [N,C,H,W], w [K,C,R,S] as uint16 bit
// patterns, y [N,K,OH,OW] float32.
static inline float bf16_to_float(uint16_t b) {
    uint32_t u = ((uint32_t)b) << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

void ork_conv_meta_bf16(const uint16_t* __restrict__ xp, const uint16_t* __restrict__ wp, float* __restrict__ yp,
                        index_t N, index_t C, index_t H, index_t W, index_t K, index_t R, index_t S, index_t stride,
                        index_t pad, index_t dil, int threads) {
    const index_t OH = (H + pad * 2 - R * dil + dil - 1) / stride + 1;
    const index_t OW = (W + pad * 2 - S * dil + dil - 1) / stride + 1;
#pragma omp parallel for collapse(2) num_threads(threads) if (threads > 1)
    for (index_t i0 = 0; i0 < N; i0++)
        for (index_t i1 = 0; i1 < K; i1++)
            for (index_t i3 = 0; i3 < OH; i3++)
                for (index_t i4 = 0; i4 < OW; i4++) {
                    float acc = float(0);
                    for (index_t i2 = 0; i2 < C; i2++)
                        for (index_t i5 = 0; i5 < R; i5++)
                            for (index_t i6 = 0; i6 < S; i6++) {
                                index_t xid2 = i3 * stride - pad + i5 * dil;
                                index_t xid3 = i4 * stride - pad + i6 * dil;
                                bool check_overflow = xid2 < 0 || xid2 >= H || xid3 < 0 || xid3 >= W;
                                float xv = check_overflow ? float(0) : bf16_to_float(xp[((i0 * C + i2) * H + xid2) * W + xid3]);
                                float wv = bf16_to_float(wp[((i1 * C + i2) * R + i5) * S + i6]);
                                acc = ((acc) + (((xv) * (wv))));
                            }
                    yp[((i0 * K + i1) * OH + i3) * OW + i4] = acc;
                }
}

int ork_max_threads(void) { return omp_get_max_threads(); }

}  // extern "C"
