// Meta-op convolution on MFMA: the fused group
//   reindex(x) * broadcast(w) summed over (c, kh, kw)
// (reference: python/jittor/nn.py:1251-1262; recognised by
// python/jittor/src/opt/tuner/conv_tuner.cc:218-411) as an implicit GEMM
//   Y[n][ko][p] = sum_{kh,kw,c} Wp[kh,kw][ko][c] * X[n][c][oh*SH-PH+kh*DH][ow*SW-PW+kw*DW]
// with bfloat16 operands, exact products and float32 accumulation
// (opt/kernel_ir.cc:958-968, ops/reduce_op.cc:259-266).  Taps outside the image
// contribute 0 (overflow value 0 times w).
//
// All geometry is baked in by the host: C_, H_, W_, K_, R_, S_, OH_, OW_, SH, SW,
// PH, PW, DH, DW, TRW (output rows per wave), NT (16-pixel tiles per wave),
// LROWS x LCOLS (input tile held in LDS), ITEMS_PER_WAVE, Y_BF16.
//
// Mapping.  v_mfma_f32_16x16x32_bf16 computes D[16 ko][16 px] += A[16 ko][32 c] *
// B[32 c][16 px].  A workgroup of 4 waves owns 128 output channels x (2*TRW
// output rows) of one image; wave (wko, wpx) owns 64 channels x TRW rows =
// 4 x NT accumulator tiles.  Channels are consumed 64 at a time:
//   * the input rows the tile touches are staged through LDS as
//     [row][col][64 c] (channel innermost) so that a B fragment is one 16-byte
//     LDS read per lane; the NCHW -> channel-innermost transpose happens in the
//     LDS write (lane = channel, so the 2-byte writes of a wave fill whole
//     128-byte rows and the 16-byte chunk index is XOR-swizzled with the column
//     to keep fragment reads conflict-free);
//   * A fragments come straight from the re-packed weights
//     Wp[tap][c/64][k-step][ko][32 c] (1 KB contiguous per fragment, L2 resident);
//   * the A fragments of the next step are loaded while the MFMAs of the
//     current step run; two workgroups per CU overlap one's staging with the
//     other's MFMAs.
// Halo cells (padding, rows outside the image) are zeroed once: they are the
// same for every channel block.

typedef __bf16 mjt_bf16x8 __attribute__((ext_vector_type(8)));
typedef float mjt_f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned short mjt_u16x8 __attribute__((ext_vector_type(8)));

struct Params { void* a[4]; };   // 8-byte words; typed as pointers so loads/stores use the global address space   // x, packed w, y, number of images

#define CB 64
#define KO_WG 128
#define MT 4
#define TR (2 * TRW)
#define TILES_R ((OH_ + TR - 1) / TR)
#define NCB (C_ / CB)
#define GROUPS (W_ / 8)
#define ITEMS (LROWS * GROUPS)

__device__ __forceinline__ int mjt_lds_off(int pos, int chunk) {
    // element offset (in bf16) of 16-byte chunk `chunk` (0..7) of position `pos`
    return pos * CB + ((chunk ^ (pos & 7)) << 3);
}

extern "C" __global__ __launch_bounds__(256, 2) void ENTRY(Params p) {
    const unsigned short* __restrict__ xp = (const unsigned short*)p.a[0];
    const unsigned short* __restrict__ wp = (const unsigned short*)p.a[1];
    const int n_img = (int)(unsigned long long)p.a[3];
    __shared__ __attribute__((aligned(16))) unsigned short xs[LROWS * LCOLS * CB];

    // tile id: the two channel halves of one pixel tile are 8 workgroups apart,
    // so they land on the same XCD (workgroups go round-robin over 8 XCDs) and
    // share the input rows in that XCD's L2
    const int id = blockIdx.x;
    const int xcd = id & 7, j = id >> 3;
    const int khalf = j % (K_ / KO_WG);
    const int ptile = (j / (K_ / KO_WG)) * 8 + xcd;
    if (ptile >= n_img * TILES_R) return;
    const int n = ptile / TILES_R;
    const int r0 = (ptile % TILES_R) * TR;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wpx = wave & 1, wko = wave >> 1;
    const int ko_base = khalf * KO_WG + wko * 64;
    const int l16 = lane & 15, lg = lane >> 4;

    // zero the whole tile once (halo cells stay zero)
    for (int t = tid; t < LROWS * LCOLS * CB / 8; t += 256) ((mjt_u16x8*)xs)[t] = (mjt_u16x8)(0);

    // per-lane pixel of each of the NT tiles
    int bpos[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) {
        int q = t * 16 + l16;
        int r = q / OW_, col = q - r * OW_;
        if (q >= TRW * OW_) { r = 0; col = 0; }
        bpos[t] = ((wpx * TRW + r) * SH) * LCOLS + col * SW;
    }

    mjt_f32x4 acc[MT][NT];
#pragma unroll
    for (int m = 0; m < MT; m++)
#pragma unroll
        for (int t = 0; t < NT; t++) acc[m][t] = (mjt_f32x4)(0.0f);

    // staging: item = (tile row, group of 8 columns); a wave moves 64 channels of an item
    const int ir0 = r0 * SH - PH;
    auto stage_in = [&](int cb) {
        mjt_u16x8 stage[ITEMS_PER_WAVE];
#pragma unroll
        for (int it = 0; it < ITEMS_PER_WAVE; it++) {
            const int item = it * 4 + wave;
            const int lr = item / GROUPS, g = item - lr * GROUPS;
            const int ir = ir0 + lr;
            mjt_u16x8 v = (mjt_u16x8)(0);
            if (item < ITEMS && ir >= 0 && ir < H_)
                v = *(const mjt_u16x8*)(xp + (((size_t)n * C_ + cb * CB + lane) * H_ + ir) * W_ + g * 8);
            stage[it] = v;
        }
        __syncthreads();              // zero fill / the previous channel block's reads are done
#pragma unroll
        for (int it = 0; it < ITEMS_PER_WAVE; it++) {
            const int item = it * 4 + wave;
            const int lr = item / GROUPS, g = item - lr * GROUPS;
            const int ir = ir0 + lr;
            if (item < ITEMS && ir >= 0 && ir < H_) {
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const int pos = lr * LCOLS + PW + g * 8 + e;
                    xs[mjt_lds_off(pos, lane >> 3) + (lane & 7)] = stage[it][e];
                }
            }
        }
        __syncthreads();
    };

    // A fragments: Wp[step][ko][32 c], step = (tap * NCB + cb) * 2 + ks; 16 rows x 64 B per fragment
    const unsigned short* __restrict__ wlane = wp + (size_t)(ko_base + l16) * 32 + lg * 8;
    auto load_a = [&](mjt_bf16x8 (&a)[MT], int cb, int s) {
        const int tap = s >> 1, ks = s & 1;
        const unsigned short* f = wlane + (size_t)((tap * NCB + cb) * 2 + ks) * (K_ * 32);
#pragma unroll
        for (int m = 0; m < MT; m++) a[m] = *(const mjt_bf16x8*)(f + m * 16 * 32);
    };
    auto compute = [&](const mjt_bf16x8 (&a)[MT], int s) {
        const int tap = s >> 1, ks = s & 1;
        const int kh = tap / S_, kw = tap - kh * S_;
        const int tap_pos = kh * DH * LCOLS + kw * DW;
        mjt_bf16x8 b[NT];
#pragma unroll
        for (int t = 0; t < NT; t++) b[t] = *(const mjt_bf16x8*)(xs + mjt_lds_off(bpos[t] + tap_pos, ks * 4 + lg));
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int m = 0; m < MT; m++)
                acc[m][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[m], b[t], acc[m][t], 0, 0, 0);
    };

    // the weights of step s+1 are in flight while the MFMAs of step s run
    mjt_bf16x8 a0[MT], a1[MT];
    load_a(a0, 0, 0);
    for (int cb = 0; cb < NCB; cb++) {
        stage_in(cb);
#pragma unroll 1
        for (int s = 0; s < 2 * R_ * S_; s += 2) {
            load_a(a1, cb, s + 1);
            compute(a0, s);
            if (s + 2 < 2 * R_ * S_) load_a(a0, cb, s + 2);
            else if (cb + 1 < NCB) load_a(a0, cb + 1, 0);
            compute(a1, s + 1);
        }
    }

    // epilogue: lane holds D[ko = 4*(lane/16)+i][px = lane%16] of each tile
#pragma unroll
    for (int t = 0; t < NT; t++) {
        const int q = t * 16 + l16;
        const int r = q / OW_, col = q - r * OW_;
        const int orow = r0 + wpx * TRW + r;
        if (q < TRW * OW_ && orow < OH_) {
#pragma unroll
            for (int m = 0; m < MT; m++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int ko = ko_base + m * 16 + lg * 4 + i;
                    const size_t o = (((size_t)n * K_ + ko) * OH_ + orow) * OW_ + col;
#if Y_BF16
                    ((unsigned short*)p.a[2])[o] = (unsigned short)(__float_as_uint(acc[m][t][i]) >> 16);
#else
                    ((float*)p.a[2])[o] = acc[m][t][i];
#endif
                }
        }
    }
}

// Weight re-pack: w[ko][c][kh][kw] -> Wp[tap][c/64][k-step][ko][32 c]
extern "C" __global__ __launch_bounds__(256) void ENTRY_PACK(Params p) {
    const unsigned short* __restrict__ w = (const unsigned short*)p.a[0];
    unsigned short* __restrict__ wp = (unsigned short*)p.a[1];
    const int total = K_ * C_ * R_ * S_;
    for (int o = blockIdx.x * 256 + threadIdx.x; o < total; o += gridDim.x * 256) {
        int c32 = o & 31;
        int rest = o >> 5;
        int ko = rest % K_; rest /= K_;
        int ks = rest & 1; rest >>= 1;
        int cb = rest % NCB;
        int tap = rest / NCB;
        int c = cb * CB + ks * 32 + c32;
        wp[o] = w[((size_t)ko * C_ + c) * (R_ * S_) + tap];
    }
}
