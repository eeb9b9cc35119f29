// Meta-op convolution on MFMA: the fused group
//   reindex(x) * broadcast(w) summed over (c, kh, kw)
// (reference: python/jittor/nn.py:1251-1262; recognised by
// python/jittor/src/opt/tuner/conv_tuner.cc:218-411) as an implicit GEMM
//   Y[n][ko][p] = sum_{kh,kw,c} Wp[kh,kw][ko][c] * X[n][c][oh*SH-PH+kh*DH][ow*SW-PW+kw*DW]
// with bfloat16 (or float16) operands, exact products and float32 accumulation
// (opt/kernel_ir.cc:958-968, ops/reduce_op.cc:259-266).  Taps outside the image
// contribute 0 (overflow value 0 times w).
//
// All geometry is baked in by the host: C_, H_, W_, K_, R_, S_, OH_, OW_, SH, SW,
// PH, PW, DH, DW, WKO (groups of 64 output channels per workgroup), WPX (row
// groups per workgroup), TRW / NT / LROWS (output rows per wave, 16-pixel tiles per
// wave and input rows in LDS of a full tile), RPW (output rows a workgroup owns),
// NFULL full tiles followed, when TAIL_TRW > 0, by one shorter tile (TAIL_TRW,
// TAIL_NT, TAIL_LROWS), LCOLS, ITEMS_PER_WAVE, Y_BF16 (16-bit output in the operand type), IN_F16.
//
// Mapping.  v_mfma_f32_16x16x32_bf16 computes D[16 ko][16 px] += A[16 ko][32 c] *
// B[32 c][16 px].  A workgroup of WPX*WKO waves owns 64*WKO output channels x RPW
// consecutive output rows of one image and walks them tile by tile (WPX*TRW rows
// each), so that the number of workgroups can match the number of compute units
// whatever the row count, and the stores of one tile and the loads of the next
// overlap the MFMAs.  Within a tile wave (wko, wpx) owns 64 channels x TRW rows =
// 4 x NT accumulator tiles.  Channels are consumed 64 at a time:
//   * the input rows the tile touches are staged through LDS as 8 planes
//     [8 c][row][col][8 c] (one per group of 8 channels, channels innermost) so
//     that a B fragment is one 16-byte LDS read per lane.  The NCHW ->
//     channel-innermost transpose happens on the way: a lane loads 8 columns of
//     one channel, the 8 lanes of a column group exchange among themselves until
//     each owns one column for the 8 channels, and writes 16 bytes: a wave fills
//     a linear 1 KB run of a plane.  The address of a fragment is linear in the
//     tap and the k-step.  The tile is double buffered across channel blocks and
//     across tiles: the loads of the next block are issued before the MFMAs of
//     the current one and written to the other buffer after them (one barrier
//     per channel block);
//   * A fragments come straight from the re-packed weights
//     Wp[tap][c/64][k-step][ko/16][lane][8 c] (1 KB per fragment in lane order, L2
//     resident) and are loaded one step before the MFMAs that use them.
// Padding columns are zeroed once; rows outside the image are written as zeros.

// operands: bfloat16, or with IN_F16 float16 (same kernel: only the MFMA and the narrowing of a 16-bit result differ)
#if IN_F16
typedef _Float16 mjt_bf16x8 __attribute__((ext_vector_type(8)));
#define MJT_MFMA __builtin_amdgcn_mfma_f32_16x16x32_f16
// float16 <- float rounds to nearest even (type/fp16_compute.h:147-198)
__device__ __forceinline__ unsigned mjt_narrow2(float lo, float hi) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    h2 v;
    v[0] = (_Float16)lo;
    v[1] = (_Float16)hi;
    return __builtin_bit_cast(unsigned, v);
}
#else
typedef __bf16 mjt_bf16x8 __attribute__((ext_vector_type(8)));
#define MJT_MFMA __builtin_amdgcn_mfma_f32_16x16x32_bf16
// bfloat16 <- float keeps the upper 16 bits (type/fp16_compute.h:238-241)
__device__ __forceinline__ unsigned mjt_narrow2(float lo, float hi) {
    return (__float_as_uint(lo) >> 16) | (__float_as_uint(hi) & 0xffff0000u);
}
#endif
typedef float mjt_f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned mjt_u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned mjt_u32x4v __attribute__((ext_vector_type(4)));

struct Params { void* a[4]; };   // x, packed w, y, number of images (typed as pointers: global address space)

#define CB 64
#define KO_WG (16 * MT * WKO)
#define NWAVES (WPX * WKO)
#define NTHR (64 * NWAVES)
#define TR (WPX * TRW)
#define SPLITS ((OH_ + RPW - 1) / RPW)      // row ranges per image
#define NCB (C_ / CB)
#define GROUPS ((W_ + 7) / 8)           // groups of 8 columns; the last one may reach past the row: what it reads there is never written
#define SEGS ((GROUPS + 7) / 8)         // segments of 64 columns
#define TILE_ELEMS (LROWS * LCOLS * 64)

// LDS tile: 8 planes, one per group of 8 channels, each [row][col][8 c] (16 bytes per position).  The 16 lanes
// that read a fragment together (16 neighbouring pixels, one channel group) then touch one 256-byte run, which
// the LDS serves at its full rate (a position stride of 64 bytes or more halves it, whatever the banks), the
// address of a fragment stays linear in the tap (it folds into the immediate offset of the read), and the
// transposed tile is written as linear 1 KB runs.
#define PLANE_ELEMS (LROWS * LCOLS * 8)
__device__ __forceinline__ int mjt_lds_off(int pos, int chunk) {
    // element offset (in bf16) of 16-byte chunk `chunk` (0..7) of position `pos`
    return chunk * PLANE_ELEMS + (pos << 3);
}

template <int V> struct mjt_ic { static constexpr int v = V; };
template <int I, int N, class F> __device__ __forceinline__ void mjt_static_for(F&& f) {
    if constexpr (I < N) {
        f(mjt_ic<I>());
        mjt_static_for<I + 1, N>(f);
    }
}
// byte offset inside the LDS tile of step s = (tap, k-step): row/column shift of the tap, 4 planes per k-step
__device__ constexpr int mjt_frag_off(int s) {
    return ((((s >> 1) / S_) * DH * LCOLS + ((s >> 1) % S_) * DW) * 8 + (s & 1) * 4 * PLANE_ELEMS) * 2;
}
// value of lane ^ 1, ^ 2, ^ 4 through data-parallel-primitive moves (quad permutes; ^ 4 is a mirror
// of each group of 8 lanes followed by a reversal inside each quad)
__device__ __forceinline__ unsigned mjt_xor1(unsigned v) { return (unsigned)__builtin_amdgcn_mov_dpp((int)v, 0xB1, 0xf, 0xf, true); }
__device__ __forceinline__ unsigned mjt_xor2(unsigned v) { return (unsigned)__builtin_amdgcn_mov_dpp((int)v, 0x4E, 0xf, 0xf, true); }
__device__ __forceinline__ float mjt_xor1f(float v) { return __uint_as_float(mjt_xor1(__float_as_uint(v))); }
__device__ __forceinline__ float mjt_xor2f(float v) { return __uint_as_float(mjt_xor2(__float_as_uint(v))); }
__device__ __forceinline__ unsigned mjt_xor4(unsigned v) {
    return (unsigned)__builtin_amdgcn_mov_dpp(__builtin_amdgcn_mov_dpp((int)v, 0x141, 0xf, 0xf, true), 0x1B, 0xf, 0xf, true);
}
template <int OFF> __device__ __forceinline__ void mjt_ds_read(mjt_u32x4v& dst, unsigned addr) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF) : "memory");
}
// wait until at most N LDS operations issued after the one that fills x are outstanding (LDS returns in order)
template <int N> __device__ __forceinline__ void mjt_lds_wait(mjt_u32x4v& x) {
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(x) : "n"(N));
}

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
    const int ko_base = kpart * KO_WG + wko * (16 * MT);
    const int l16 = lane & 15, lg = lane >> 4;
    const unsigned xs_base = (unsigned)(unsigned long long)(__attribute__((address_space(3))) unsigned short*)&xs[0][0];

    // zero both buffers once (padding columns stay zero)
    for (int t = tid; t < 2 * TILE_ELEMS / 8; t += NTHR) ((mjt_u32x4v*)&xs[0][0])[t] = (mjt_u32x4v)(0u);

    // Staging.  An item is (tile row, segment of 64 columns, 8 channels); a wave moves one item per
    // load: lane (g = lane / 8, r = lane % 8) loads the 16 bytes of columns 8g..8g+7 of channel r, so
    // that a wave touches 8 cache lines per load instead of 64 (the address unit handles one line per
    // cycle).  The 8 lanes of a column group then transpose their 8 channels x 8 columns among
    // themselves with three butterfly exchanges (lane ^ 4, ^ 2, ^ 1; data-parallel-primitive moves,
    // no LDS), after which lane r owns column 8g + r for the 8 channels in order: one 16-byte LDS
    // write, at a lane stride of one position.
    const int sg = lane >> 3, sr = lane & 7;
    const bool b2 = lane & 4, b1 = lane & 2, b0 = lane & 1;
    // byte selectors of v_perm_b32 (bytes 0-3 = second operand, 4-7 = first operand):
    //   sel_t  what the lane gives away: the high halves of two dwords (even lane) or the low halves (odd lane)
    //   sel_a  even lane: own low half | received low half << 16;  odd lane: received low half | own high half << 16
    //   sel_b  even lane: own low half | received high half << 16; odd lane: received high half | own high half << 16
    const unsigned sel_t = b0 ? 0x05040100u : 0x07060302u;
    const unsigned sel_a = b0 ? 0x03020504u : 0x05040100u;
    const unsigned sel_b = b0 ? 0x03020706u : 0x07060100u;
    mjt_u32x4v stage[ITEMS_PER_WAVE];
    // buffer descriptors (base, size in bytes): addresses are a scalar offset plus a 32-bit lane offset,
    // so no per-item 64-bit address lives in vector registers
    const __amdgpu_buffer_rsrc_t x_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void*)(xp + (size_t)n * C_ * H_ * W_), 0, C_ * H_ * W_ * 2, 0x00020000);
    const unsigned x_lane_off = (unsigned)sr * (H_ * W_ * 2);
    auto item_of = [&](int it, int& lr, int& seg, int& cg) {
        const int item = wave * ITEMS_PER_WAVE + it;
        cg = item & 7;
        const int rest = item >> 3;
        lr = rest / SEGS;
        seg = rest - lr * SEGS;
    };
    // The loads are unconditional (rows outside the image and idle lanes read a clamped address and
    // are zeroed or skipped when written): a load under a branch would make every later wait for a
    // weight fragment wait for all staging loads as well.
    auto fetch = [&](int r0, int lrows, int cb) {            // input rows of the tile whose first output row is r0
        const int ir0 = r0 * SH - PH;
#pragma unroll
        for (int it = 0; it < ITEMS_PER_WAVE; it++) {
            int lr, seg, cg;
            item_of(it, lr, seg, cg);
            int ir = ir0 + (lr < lrows ? lr : lrows - 1);
            ir = ir < 0 ? 0 : ir >= H_ ? H_ - 1 : ir;
            const int soff = (((cb * CB + cg * 8) * H_ + ir) * W_) * 2;     // uniform: channel group and row inside the image
            int grp = seg * 8 + sg;
            grp = grp < GROUPS ? grp : GROUPS - 1;
            stage[it] = __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, (int)(x_lane_off + (unsigned)grp * 16), soff, 0);
        }
    };
    auto commit = [&](int r0, int lrows, int buf) {
        const int ir0 = r0 * SH - PH;
#pragma unroll
        for (int it = 0; it < ITEMS_PER_WAVE; it++) {
            int lr, seg, cg;
            item_of(it, lr, seg, cg);
            mjt_u32x4v d = stage[it];                        // d[k] = columns 2k (low half), 2k+1 (high half) of channel r
            if (ir0 + lr < 0 || ir0 + lr >= H_) d = (mjt_u32x4v)(0u);   // uniform: a row outside the image
            // lane ^ 4: keep one half of the columns, get the same half from the channel 4 away
            const unsigned g0 = mjt_xor4(b2 ? d[0] : d[2]), g1 = mjt_xor4(b2 ? d[1] : d[3]);
            const unsigned a0 = b2 ? g0 : d[0], a1 = b2 ? g1 : d[1];      // channel r & 3:       column pairs 0, 1 of the half
            const unsigned a2 = b2 ? d[2] : g0, a3 = b2 ? d[3] : g1;      // channel (r & 3) + 4
            // lane ^ 2: keep one column pair, get it from the channel 2 away
            const unsigned h0 = mjt_xor2(b1 ? a0 : a1), h1 = mjt_xor2(b1 ? a2 : a3);
            const unsigned c0 = b1 ? h0 : a0, c1 = b1 ? a1 : h0;          // channels q, q+2 (q = r & 1), one column pair
            const unsigned c2 = b1 ? h1 : a2, c3 = b1 ? a3 : h1;          // channels q+4, q+6
            // lane ^ 1: keep one column, get it from the neighbouring channels (two 16-bit values per
            // move; byte permutes with per-lane selectors keep this free of branches)
            const unsigned s0 = mjt_xor1(__builtin_amdgcn_perm(c1, c0, sel_t)), s1 = mjt_xor1(__builtin_amdgcn_perm(c3, c2, sel_t));
            mjt_u32x4v f;                                    // channels (0,1) (2,3) (4,5) (6,7) of column 8g + r
            f[0] = __builtin_amdgcn_perm(s0, c0, sel_a);
            f[1] = __builtin_amdgcn_perm(s0, c1, sel_b);
            f[2] = __builtin_amdgcn_perm(s1, c2, sel_a);
            f[3] = __builtin_amdgcn_perm(s1, c3, sel_b);
            if (lr < lrows && seg * 64 + lane < W_) {        // rows outside the image carry zeros; columns past the row end are not the row's
                unsigned short* dst = &xs[buf][0] + mjt_lds_off(lr * LCOLS + PW + seg * 64 + lane, cg);
                *(mjt_u32x4v*)dst = f;
            }
        }
    };

    // A fragments: Wp[step][ko / 16][lane][8 c], step = (tap * NCB + cb) * 2 + ks: a fragment is 1 KB in lane order
    // (lane = lg * 16 + l16 holds channels lg*8.. of row l16), so that a wave's load is one linear run of 8 cache
    // lines; in [ko][32 c] order the 16 lanes the address unit takes together would touch 8 lines each time
    const unsigned a_lane_off = (unsigned)(wko * MT * 1024 + lane * 16);   // bytes
    const __amdgpu_buffer_rsrc_t w_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void*)(wp + (size_t)kpart * KO_WG * 32), 0, (R_ * S_ * C_ * K_ - kpart * KO_WG * 32) * 2, 0x00020000);
    auto load_a = [&](mjt_bf16x8 (&a)[MT], int cb, int s) {
        const int tap = s >> 1, ks = s & 1;
        const int soff = ((tap * NCB + cb) * 2 + ks) * (K_ * 32 * 2);   // uniform
#pragma unroll
        for (int m = 0; m < MT; m++)
            a[m] = __builtin_bit_cast(mjt_bf16x8, __builtin_amdgcn_raw_buffer_load_b128(w_rsrc, (int)a_lane_off + (m & 3) * 1024, soff + (m >> 2) * 4096, 0));
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
        unsigned baddr[NT_];                                 // LDS byte address of the fragment at tap (0,0), k-step 0, in the current buffer
#pragma unroll
        for (int t = 0; t < NT_; t++) {
            int q = t * 16 + l16;
            int r = q / OW_, col = q - r * OW_;
            if (q >= TRW_ * OW_) { r = 0; col = 0; }
            baddr[t] = xs_base + (unsigned)(buf * TILE_ELEMS * 2) + (unsigned)mjt_lds_off(((wpx * TRW_ + r) * SH) * LCOLS + col * SW, lg) * 2;
        }
        mjt_f32x4 acc[MT][NT_];
#pragma unroll
        for (int m = 0; m < MT; m++)
#pragma unroll
            for (int t = 0; t < NT_; t++) acc[m][t] = (mjt_f32x4)(0.0f);

        // Main loop.  Per channel block the STEPS x NT_ B fragments form one stream; fragment f is
        // requested BQ_DIST fragments before the four MFMAs that use it (a ring of BQ_DIST + 1
        // registers), so the LDS latency hides behind 4 * BQ_DIST MFMAs of this wave.  The reads and
        // the waits for them are written out so that this order is what runs: tap and k-step are
        // compile-time here and fold into the offset field of the read.
        constexpr int NF = STEPS * NT_;
        mjt_u32x4v bq[BQ_DIST + 1];
#pragma unroll 1
        for (int cb = 0; cb < NCB; cb++) {
            const bool more = cb + 1 < NCB;
            mjt_static_for<0, BQ_DIST>([&](auto fc) {
                constexpr int f = decltype(fc)::v;
                mjt_ds_read<mjt_frag_off(f / NT_)>(bq[f % (BQ_DIST + 1)], baddr[f % NT_]);
            });
            mjt_static_for<0, STEPS>([&](auto sc) {
                constexpr int st = decltype(sc)::v;
                if (st + 1 < STEPS) load_a(ring[(st + 1) & 1], cb, st + 1);
                else if (more) load_a(ring[0], cb + 1, 0);
                else if (next_lrows) load_a(ring[0], 0, 0);
                if (st == 0) {                                   // in flight during this block's MFMAs; after the weight loads,
                    if (more) fetch(r0, LR_, cb + 1);            // so that the wait for those does not include these
                    else if (next_lrows) fetch(next_r0, next_lrows, 0);
                }
                mjt_static_for<0, NT_>([&](auto tc) {
                    constexpr int t = decltype(tc)::v;
                    constexpr int f = st * NT_ + t;
                    if constexpr (f + BQ_DIST < NF)
                        mjt_ds_read<mjt_frag_off((f + BQ_DIST) / NT_)>(bq[(f + BQ_DIST) % (BQ_DIST + 1)], baddr[(f + BQ_DIST) % NT_]);
                    mjt_lds_wait<(NF - 1 - f < BQ_DIST ? NF - 1 - f : BQ_DIST)>(bq[f % (BQ_DIST + 1)]);
                    const mjt_bf16x8 b = __builtin_bit_cast(mjt_bf16x8, bq[f % (BQ_DIST + 1)]);
#pragma unroll
                    for (int m = 0; m < MT; m++)
                        acc[m][t] = MJT_MFMA(ring[st & 1][m], b, acc[m][t], 0, 0, 0);
                });
            });
            if (more || next_lrows) {
                commit(more ? r0 : next_r0, more ? LR_ : next_lrows, buf ^ 1);        // the other buffer: nobody reads it now
                __syncthreads();
                buf ^= 1;
#pragma unroll
                for (int t = 0; t < NT_; t++) baddr[t] += buf ? (unsigned)(TILE_ELEMS * 2) : (unsigned)(-(TILE_ELEMS * 2));
            }
        }

        // epilogue: lane holds D[ko = 4*(lane/16)+i][px = lane%16] of each tile
#if OW_ % 4 == 0
        // The four lanes of a quad (4 pixels x 4 channels) transpose among themselves, after which lane j
        // of the quad owns channel 4*(lane/16)+j for the quad's 4 consecutive pixels: one 16-byte (or
        // 8-byte bfloat16) store instead of four scattered 4-byte stores.  Four pixels never straddle
        // an output row because OW is a multiple of 4.
        const int qj = lane & 3;
#pragma unroll
        for (int t = 0; t < NT_; t++) {
            const int q0 = t * 16 + (l16 & ~3);
            const int r = q0 / OW_, col = q0 - r * OW_;
            const int orow = r0 + wpx * TRW_ + r;
            const bool ok = q0 < TRW_ * OW_ && orow < row_end;
#pragma unroll
            for (int m = 0; m < MT; m++) {
                const mjt_f32x4 v = acc[m][t];
                // lane ^ 1: rows (0,1) and (2,3) trade pixels
                const float g0 = mjt_xor1f(b0 ? v[0] : v[1]), g1 = mjt_xor1f(b0 ? v[2] : v[3]);
                const float a0 = b0 ? g0 : v[0], a1 = b0 ? v[1] : g0;     // row (j & 1):     pixel pair of this lane pair
                const float a2 = b0 ? g1 : v[2], a3 = b0 ? v[3] : g1;     // row (j & 1) + 2
                // lane ^ 2: row pairs trade pixel pairs
                const float h0 = mjt_xor2f(b1 ? a0 : a2), h1 = mjt_xor2f(b1 ? a1 : a3);
                mjt_f32x4 y4;                                             // row j, pixels 0..3 of the quad
                y4[0] = b1 ? h0 : a0;
                y4[1] = b1 ? h1 : a1;
                y4[2] = b1 ? a2 : h0;
                y4[3] = b1 ? a3 : h1;
                if (ok) {
                    const int ko = ko_base + m * 16 + lg * 4 + qj;
                    const size_t o = (((size_t)n * K_ + ko) * OH_ + orow) * OW_ + col;
#if Y_BF16
                    mjt_u32x2 pk;
                    pk[0] = mjt_narrow2(y4[0], y4[1]);
                    pk[1] = mjt_narrow2(y4[2], y4[3]);
                    *(mjt_u32x2*)((unsigned short*)p.a[2] + o) = pk;
#else
                    *(mjt_f32x4*)((float*)p.a[2] + o) = y4;
#endif
                }
            }
        }
#else
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
                        ((unsigned short*)p.a[2])[o] = (unsigned short)mjt_narrow2(acc[m][t][i], 0.0f);
#else
                        ((float*)p.a[2])[o] = acc[m][t][i];
#endif
                    }
            }
        }
#endif
    };

    // tiles of this workgroup: full tiles while they start inside the row range, then the short one
    int nfull = (row_end - row_begin + TR - 1) / TR;
    if (nfull > NFULL) nfull = NFULL;
    const bool tail = TAIL_TRW > 0 && row_begin + NFULL * TR < row_end;
    const int first_lrows = nfull ? LROWS : TAIL_LROWS;

    load_a(ring[0], 0, 0);
    fetch(row_begin, first_lrows, 0);
    __syncthreads();                              // zero fill done
    commit(row_begin, first_lrows, 0);
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

// Weight re-pack: w[ko][c][kh][kw] -> Wp[tap][c/64][k-step][ko/16][lg][l16][8 c] (c = 32 k-step + 8 lg + ..)
extern "C" __global__ __launch_bounds__(256) void ENTRY_PACK(Params p) {
    const unsigned short* __restrict__ w = (const unsigned short*)p.a[0];
    unsigned short* __restrict__ wp = (unsigned short*)p.a[1];
    const int total = K_ * C_ * R_ * S_;
    for (int o = blockIdx.x * 256 + threadIdx.x; o < total; o += gridDim.x * 256) {
        int c8 = o & 7, l16 = (o >> 3) & 15, lg = (o >> 7) & 3;
        int rest = o >> 9;
        int ko = (rest % (K_ / 16)) * 16 + l16; rest /= K_ / 16;
        int c32 = lg * 8 + c8;
        int ks = rest & 1; rest >>= 1;
        int cb = rest % NCB;
        int tap = rest / NCB;
        int c = cb * CB + ks * 32 + c32;
        wp[o] = w[((size_t)ko * C_ + c) * (R_ * S_) + tap];
    }
}
