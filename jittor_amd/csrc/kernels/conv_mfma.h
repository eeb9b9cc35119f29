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
// PH, PW, DH, DW, WKO (groups of 64 output channels per workgroup), WPX (row
// groups per workgroup), TRW / NT / LROWS (output rows per wave, 16-pixel tiles per
// wave and input rows in LDS of a full tile), RPW (output rows a workgroup owns),
// NFULL full tiles followed, when TAIL_TRW > 0, by one shorter tile (TAIL_TRW,
// TAIL_NT, TAIL_LROWS), LCOLS, ITEMS_PER_WAVE, Y_BF16.
//
// Mapping.  v_mfma_f32_16x16x32_bf16 computes D[16 ko][16 px] += A[16 ko][32 c] *
// B[32 c][16 px].  A workgroup of WPX*WKO waves owns 64*WKO output channels x RPW
// consecutive output rows of one image and walks them tile by tile (WPX*TRW rows
// each), so that the number of workgroups can match the number of compute units
// whatever the row count, and the stores of one tile and the loads of the next
// overlap the MFMAs.  Within a tile wave (wko, wpx) owns 64 channels x TRW rows =
// 4 x NT accumulator tiles.  Channels are consumed 64 at a time:
//   * the input rows the tile touches are staged through LDS as
//     [row][col][64 c] (channel innermost) so that a B fragment is one 16-byte
//     LDS read per lane.  The NCHW -> channel-innermost transpose happens in the
//     LDS write: a lane loads 8 columns of one channel, swaps halves with its
//     neighbour lane so that it owns two channels x four columns, packs the two
//     channels of a column into one dword, and the dwords of a wave fill whole
//     128-byte rows; positions are padded to 144 bytes, which makes the address
//     of a fragment linear in the tap.  The tile is double buffered across
//     channel blocks and across tiles: the loads of the next block are issued
//     before the MFMAs of the current one and written to the other buffer after
//     them (one barrier per channel block);
//   * A fragments come straight from the re-packed weights
//     Wp[tap][c/64][k-step][ko][32 c] (1 KB contiguous per fragment, L2
//     resident) and are loaded one step before the MFMAs that use them.
// Padding columns are zeroed once; rows outside the image are written as zeros.

typedef __bf16 mjt_bf16x8 __attribute__((ext_vector_type(8)));
typedef float mjt_f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned mjt_u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned mjt_u32x4v __attribute__((ext_vector_type(4)));

struct Params { void* a[4]; };   // x, packed w, y, number of images (typed as pointers: global address space)

#define CB 64
#define KO_WG (64 * WKO)
#define NWAVES (WPX * WKO)
#define NTHR (64 * NWAVES)
#define MT 4
#define TR (WPX * TRW)
#define SPLITS ((OH_ + RPW - 1) / RPW)      // row ranges per image
#define NCB (C_ / CB)
#define GROUPS (W_ / 8)                 // groups of 8 columns
#define TILE_ELEMS (LROWS * LCOLS * PSTRIDE)

// LDS tile: position (row, col) holds its 64 channels in 128 bytes followed by 16 bytes of padding.
// With a 144-byte stride, 8 neighbouring positions read by 8 lanes (one 16-byte chunk each) fall on 8
// different groups of 4 banks, so fragment reads are conflict-free, and the address of a fragment is
// linear in the tap: it folds into the immediate offset of the LDS read.
#define PSTRIDE 72
__device__ __forceinline__ int mjt_lds_off(int pos, int chunk) {
    // element offset (in bf16) of 16-byte chunk `chunk` (0..7) of position `pos`
    return pos * PSTRIDE + (chunk << 3);
}

template <int V> struct mjt_ic { static constexpr int v = V; };

extern "C" __global__ __launch_bounds__(NTHR) void ENTRY(Params p) {
    const unsigned short* __restrict__ xp = (const unsigned short*)p.a[0];
    const unsigned short* __restrict__ wp = (const unsigned short*)p.a[1];
    const int n_img = (int)(unsigned long long)p.a[3];
    __shared__ __attribute__((aligned(16))) unsigned short xs[2][TILE_ELEMS];

    // range id: the channel groups of one row range are 8 workgroups apart, so
    // they land on the same XCD (workgroups go round-robin over 8 XCDs) and
    // share the input rows in that XCD's L2
    const int id = blockIdx.x;
    const int xcd = id & 7, j = id >> 3;
    const int kpart = j % (K_ / KO_WG);
    const int range = (j / (K_ / KO_WG)) * 8 + xcd;
    if (range >= n_img * SPLITS) return;
    const int n = range / SPLITS;
    const int row_begin = (range % SPLITS) * RPW;
    const int row_end = row_begin + RPW < OH_ ? row_begin + RPW : OH_;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: what depends on it alone stays scalar
    const int wpx = wave % WPX, wko = wave / WPX;
    const int ko_base = kpart * KO_WG + wko * 64;
    const int l16 = lane & 15, lg = lane >> 4;

    // zero both buffers once (padding columns stay zero)
    for (int t = tid; t < 2 * TILE_ELEMS / 8; t += NTHR) ((mjt_u32x4v*)&xs[0][0])[t] = (mjt_u32x4v)(0u);

    // staging: item = (tile row, group of 8 columns); a wave moves the 64 channels of an item, lane l
    // loading 16 bytes (8 columns) of channel l -- one scattered load per lane is what the address unit
    // is charged for, so it should be as wide as possible.  Adjacent lanes (channels 2k, 2k+1) then swap
    // halves so that each owns 4 columns of both channels, and write one dword (channel pair) per column.
    const int odd = lane & 1;
    mjt_u32x4v stage[ITEMS_PER_WAVE];
    const unsigned x_lane_off = (unsigned)lane * (H_ * W_ * 2);   // byte offset of the lane's channel
    auto fetch = [&](int r0, int lrows, int cb) {            // input rows of the tile whose first output row is r0
        const int ir0 = r0 * SH - PH;
#pragma unroll
        for (int it = 0; it < ITEMS_PER_WAVE; it++) {
            const int item = it * NWAVES + wave;
            const int lr = item / GROUPS, g = item - lr * GROUPS;
            const int ir = ir0 + lr;
            mjt_u32x4v v = (mjt_u32x4v)(0u);
            if (lr < lrows && ir >= 0 && ir < H_) {
                const char* base = (const char*)(xp + (((size_t)n * C_ + cb * CB) * H_ + ir) * W_ + g * 8);   // uniform
                v = *(const mjt_u32x4v*)(base + x_lane_off);
            }
            stage[it] = v;
        }
    };
    const int commit_lane_off = (odd * 4 * PSTRIDE + (lane & ~1)) >> 1;   // in dwords: 4 columns on for odd lanes, channel pair
    auto commit = [&](int lrows, int buf) {
#pragma unroll
        for (int it = 0; it < ITEMS_PER_WAVE; it++) {
            const int item = it * NWAVES + wave;
            const int lr = item / GROUPS, g = item - lr * GROUPS;
            // even lane keeps its columns 0..3 and receives columns 0..3 of the odd lane; the odd lane
            // keeps columns 4..7 and receives columns 4..7 of the even lane
            const unsigned give0 = odd ? stage[it][0] : stage[it][2];
            const unsigned give1 = odd ? stage[it][1] : stage[it][3];
            const unsigned got0 = (unsigned)__shfl_xor((int)give0, 1, 64);
            const unsigned got1 = (unsigned)__shfl_xor((int)give1, 1, 64);
            const unsigned mine0 = odd ? stage[it][2] : stage[it][0];
            const unsigned mine1 = odd ? stage[it][3] : stage[it][1];
            const unsigned lo0 = odd ? got0 : mine0, hi0 = odd ? mine0 : got0;   // lo = even channel, hi = odd channel
            const unsigned lo1 = odd ? got1 : mine1, hi1 = odd ? mine1 : got1;
            if (lr < lrows) {                                // rows outside the image carry zeros
                // uniform part of the address (row, column group, buffer) + the lane's part (column half, channel pair)
                unsigned* dst = (unsigned*)&xs[buf][0] + ((lr * LCOLS + PW + g * 8) * PSTRIDE >> 1) + commit_lane_off;
                dst[0 * (PSTRIDE >> 1)] = (lo0 & 0xffffu) | (hi0 << 16);
                dst[1 * (PSTRIDE >> 1)] = (lo0 >> 16) | (hi0 & 0xffff0000u);
                dst[2 * (PSTRIDE >> 1)] = (lo1 & 0xffffu) | (hi1 << 16);
                dst[3 * (PSTRIDE >> 1)] = (lo1 >> 16) | (hi1 & 0xffff0000u);
            }
        }
    };

    // A fragments: Wp[step][ko][32 c], step = (tap * NCB + cb) * 2 + ks; 16 rows x 64 B per fragment
    const unsigned a_lane_off = (unsigned)(((wko * 64 + l16) * 32 + lg * 8) * 2);   // bytes
    auto load_a = [&](mjt_bf16x8 (&a)[MT], int cb, int s) {
        const int tap = s >> 1, ks = s & 1;
        const char* f = (const char*)(wp + (size_t)((tap * NCB + cb) * 2 + ks) * (K_ * 32) + (size_t)kpart * KO_WG * 32);   // uniform
#pragma unroll
        for (int m = 0; m < MT; m++) a[m] = *(const mjt_bf16x8*)(f + a_lane_off + m * 16 * 32 * 2);
    };

    constexpr int STEPS = 2 * R_ * S_;            // steps per channel block (even)
    mjt_bf16x8 ring[2][MT];                       // weights of the next step are in flight during a step
    int buf = 0;                                  // LDS buffer that holds the current channel block

    // One tile: TRW_ output rows per wave starting at r0, NT_ accumulator tiles per wave, LR_ input rows
    // in LDS.  On entry its first channel block is in xs[buf] and its first A fragments are in ring[0];
    // when another tile follows (next_lrows > 0) its first block and fragments are prepared the same way.
    auto run_tile = [&](auto trw_c, auto nt_c, auto lr_c, const int r0, const int next_r0, const int next_lrows) {
        constexpr int TRW_ = decltype(trw_c)::v, NT_ = decltype(nt_c)::v, LR_ = decltype(lr_c)::v;
        // per-lane pixel of each of the NT_ tiles
        unsigned baddr[NT_];                                 // byte address in a buffer of the fragment at tap (0,0), k-step 0
#pragma unroll
        for (int t = 0; t < NT_; t++) {
            int q = t * 16 + l16;
            int r = q / OW_, col = q - r * OW_;
            if (q >= TRW_ * OW_) { r = 0; col = 0; }
            baddr[t] = (unsigned)mjt_lds_off(((wpx * TRW_ + r) * SH) * LCOLS + col * SW, lg) * 2;
        }
        mjt_f32x4 acc[MT][NT_];
#pragma unroll
        for (int m = 0; m < MT; m++)
#pragma unroll
            for (int t = 0; t < NT_; t++) acc[m][t] = (mjt_f32x4)(0.0f);

        auto compute = [&](const mjt_bf16x8 (&a)[MT], int s, int b_) {
            const int tap = s >> 1, ks = s & 1;
            const int kh = tap / S_, kw = tap - kh * S_;
            const char* tile = (const char*)&xs[b_][0] + mjt_lds_off(kh * DH * LCOLS + kw * DW, ks * 4) * 2;   // uniform
            mjt_bf16x8 b[NT_];
#pragma unroll
            for (int t = 0; t < NT_; t++) b[t] = *(const mjt_bf16x8*)(tile + baddr[t]);
#pragma unroll
            for (int t = 0; t < NT_; t++)
#pragma unroll
                for (int m = 0; m < MT; m++)
                    acc[m][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[m], b[t], acc[m][t], 0, 0, 0);
        };

        // two steps per iteration (the ring has two slots); the tap is a run-time value
#pragma unroll 1
        for (int g0 = 0; g0 < NCB * STEPS; g0 += 2) {
#pragma unroll
            for (int u = 0; u < 2; u++) {
                const int g = g0 + u;
                const int cb = g / STEPS, st = g - cb * STEPS;
                const bool more = cb + 1 < NCB;
                if (st == 0) {                                   // in flight during this block's MFMAs
                    if (more) fetch(r0, LR_, cb + 1);
                    else if (next_lrows) fetch(next_r0, next_lrows, 0);
                }
                if (g + 1 < NCB * STEPS) load_a(ring[u ^ 1], (g + 1) / STEPS, (g + 1) % STEPS);
                else if (next_lrows) load_a(ring[u ^ 1], 0, 0);
                compute(ring[u], st, buf);
                if (st == STEPS - 1 && (more || next_lrows)) {
                    commit(more ? LR_ : next_lrows, buf ^ 1);    // the other buffer: nobody reads it now
                    __syncthreads();
                    buf ^= 1;
                }
            }
        }

        // epilogue: lane holds D[ko = 4*(lane/16)+i][px = lane%16] of each tile
#pragma unroll
        for (int t = 0; t < NT_; t++) {
            const int q = t * 16 + l16;
            const int r = q / OW_, col = q - r * OW_;
            const int orow = r0 + wpx * TRW_ + r;
            if (q < TRW_ * OW_ && orow < row_end) {
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
    };

    // tiles of this workgroup: full tiles while they start inside the row range, then the short one
    int nfull = (row_end - row_begin + TR - 1) / TR;
    if (nfull > NFULL) nfull = NFULL;
    const bool tail = TAIL_TRW > 0 && row_begin + NFULL * TR < row_end;
    const int first_lrows = nfull ? LROWS : TAIL_LROWS;

    load_a(ring[0], 0, 0);
    fetch(row_begin, first_lrows, 0);
    __syncthreads();                              // zero fill done
    commit(first_lrows, 0);
    __syncthreads();
    for (int s = 0; s < nfull; s++) {
        const int r0 = row_begin + s * TR;
        const int next_lrows = s + 1 < nfull ? LROWS : tail ? TAIL_LROWS : 0;
        run_tile(mjt_ic<TRW>(), mjt_ic<NT>(), mjt_ic<LROWS>(), r0, r0 + TR, next_lrows);
    }
#if TAIL_TRW > 0
    if (tail) run_tile(mjt_ic<TAIL_TRW>(), mjt_ic<TAIL_NT>(), mjt_ic<TAIL_LROWS>(), row_begin + NFULL * TR, 0, 0);
#endif
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
