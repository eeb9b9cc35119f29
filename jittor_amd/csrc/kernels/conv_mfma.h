// Meta-op convolution on MFMA: the fused group
//   reindex(x) * broadcast(w) summed over (c, kh, kw)
// (reference: python/jittor/nn.py:1251-1262; recognised by
// python/jittor/src/opt/tuner/conv_tuner.cc:218-411) as an implicit GEMM
//   Y[n][ko][p] = sum_{kh,kw,c} Wp[kh,kw][ko][c] * X[n][c][oh*SH-PH+kh*DH][ow*SW-PW+kw*DW]
// with bfloat16 (or float16) operands, exact products and float32 accumulation
// (opt/kernel_ir.cc:958-968, ops/reduce_op.cc:259-266).  Taps outside the image
// contribute 0 (overflow value 0 times w).
//
// All geometry is baked in by the host: C_, H_, W_, K_ (input and output channels of the convolution: of one group when
// it is grouped; XC_ and YK_ are then the channel counts of the whole x and y, and blockIdx.y is the group),
// R_, S_, OH_, OW_, SH, SW,
// PH, PW, DH, DW, WKO (groups of 16*MT output channels per workgroup), WPX (row
// groups per workgroup), TRW / NT / LROWS (output rows per wave, 16-pixel tiles per
// wave and input rows in LDS of a full tile), RPW (output rows a workgroup owns),
// NFULL full tiles followed, when TAIL_TRW > 0, by one shorter tile (TAIL_TRW,
// TAIL_NT, TAIL_LROWS), LCOLS, CB (channels per block: 32 or 64), NS (slabs in the
// weight ring), STAGE_DEPTH, WPS (waves per SIMD the register budget is for),
// Y_BF16 (16-bit output in the operand type), IN_F16.
//
// Mapping.  v_mfma_f32_16x16x32_bf16 computes D[16 px][16 ko] += A[16 px][32 c] *
// B[32 c][16 ko]: the input fragment is the first operand, so that a lane ends up with
// four consecutive pixels of one channel, which it stores as they are.  A workgroup of WPX*WKO waves owns 16*MT*WKO output channels x RPW
// consecutive output rows of one image and walks them tile by tile (WPX*TRW rows
// each), so that the number of workgroups can match the number of compute units
// whatever the row count.  Within a tile wave (wko, wpx) owns 16*MT channels x TRW
// rows = MT x NT accumulator tiles.  Channels are consumed CB at a time, a block
// being CB/32 steps per tap; both operands of a step come from LDS:
//   * the input rows the tile touches are staged through LDS as CB/8 planes
//     [row][col][8 c] (one per group of 8 channels, channels innermost) so
//     that a B fragment is one 16-byte LDS read per lane.  The NCHW ->
//     channel-innermost transpose happens on the way: a lane loads 8 columns of
//     one channel, the 8 lanes of a column group exchange among themselves until
//     each owns one column for the 8 channels, and writes 16 bytes: a wave fills
//     a linear 1 KB run of a plane.  The address of a fragment is linear in the
//     tap and the k-step.  The tile is double buffered across channel blocks and
//     across tiles: the rows of the next block are asked for during the first
//     steps of a block and written to the other buffer a few steps later;
//   * the weights are re-packed as Wp[tap][c/32][ko/16][lane][8 c] (1 KB per A
//     fragment in lane order, L2 resident).  The fragments of one step for the
//     workgroup's channels, a slab, are contiguous there; slabs are copied
//     straight into a ring in LDS several steps ahead of their use (no registers
//     on the way), and every wave reads its MT fragments from the ring.
// One barrier per step hands over the slab that has landed and frees the oldest.
// Padding columns are zeroed once; rows outside the image are written as zeros.

// operands: bfloat16, or with IN_F16 float16 (same kernel: only the MFMA and the narrowing of a 16-bit result differ)
#if IN_F16
typedef _Float16 mjt_bf16x8 __attribute__((ext_vector_type(8)));
#define MJT_MFMA __builtin_amdgcn_mfma_f32_16x16x32_f16
#define MJT_MFMA_ASM "v_mfma_f32_16x16x32_f16"
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
#define MJT_MFMA_ASM "v_mfma_f32_16x16x32_bf16"
// bfloat16 <- float keeps the upper 16 bits (type/fp16_compute.h:238-241)
__device__ __forceinline__ unsigned mjt_narrow2(float lo, float hi) {
    return (__float_as_uint(lo) >> 16) | (__float_as_uint(hi) & 0xffff0000u);
}
#endif
typedef float mjt_f32x4 __attribute__((ext_vector_type(4)));
typedef float mjt_f32x2 __attribute__((ext_vector_type(2)));
typedef unsigned mjt_u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned mjt_u32x4v __attribute__((ext_vector_type(4)));

struct Params { void* a[4]; };   // x, packed w, y, number of images (typed as pointers: global address space)

// ABL (0 in production): timing-only ablations, results are wrong with any bit set.  1 no output stores, 2 no input
// rows (neither loaded nor written to LDS), 4 (only together with 1 and 2) no weight slabs copied, no fragment reads
// from LDS and no barrier per step: 7 leaves the MFMAs alone, 16 no MFMAs: leaves the data movement alone.  The host
// admits 0, 1, 2, 3, 7, 16 and 17 only.
#ifndef ABL
#define ABL 0
#endif

#define KSTEPS (CB / 32)                    // MFMA k-steps per tap in a channel block of CB (32 or 64) channels
#define KO_WG (16 * MT * WKO)
#define NWAVES (WPX * WKO)
#define NTHR (64 * NWAVES)
#define TR (WPX * TRW)
#define SPLITS ((OH_ + RPW - 1) / RPW)      // row ranges per image
#define NCB (C_ / CB)
#define GROUPS ((W_ + 7) / 8)           // groups of 8 columns; the last one may reach past the row: what it reads there is never written
// An item of the staging is what one load instruction of a wave brings: 8 channels x 8 groups of 8 columns.  Rows of more than
// 32 columns take SEGS items of 64 columns each; narrower rows share an item, RPI of them with GP2 groups each, since on a
// 14-column map an item of one row would use a quarter of its lanes and cost the same instructions.
#define GP2 (GROUPS <= 1 ? 1 : GROUPS <= 2 ? 2 : GROUPS <= 4 ? 4 : 8)       // groups that a row takes in an item
#define RPI (8 / GP2)                                                        // rows per item
#define SEGS (RPI > 1 ? 1 : (GROUPS + 7) / 8)                                // segments of 64 columns
#define ROWITEMS ((LROWS + RPI - 1) / RPI)                                   // items along the rows of a full tile
#define TILE_ELEMS (LROWS * LCOLS * CB)

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
    return ((((s / KSTEPS) / S_) * DH * LCOLS + ((s / KSTEPS) % S_) * DW) * 8 + (s % KSTEPS) * 4 * PLANE_ELEMS) * 2;
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
// The MFMAs of the main loop are spelled out like its LDS reads and waits: between those the compiler would
// otherwise move them freely (it sees no latency in the reads), and the order below is the schedule.  The
// compiler takes a spelled-out MFMA for finished the moment it is issued and keeps none of the cycles the
// hardware wants between an MFMA and an instruction that touches its registers.  The accumulators therefore live
// in the accumulation registers for the whole loop, where nothing but these MFMAs touches them (the loop has no
// use for them, and no copies are made to feed an MFMA); before and after the loop they are tied to points
// behind explicit idle cycles.
__device__ __forceinline__ void mjt_mfma(mjt_f32x4& c, const mjt_u32x4v& a, const mjt_u32x4v& b) {
#if ABL & 16
    asm volatile("" : "+a"(c) : "v"(a), "v"(b));
#else
    asm volatile(MJT_MFMA_ASM " %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
#endif
}
__device__ __forceinline__ void mjt_keep(const mjt_u32x4v& x) { asm volatile("" : : "v"(x)); }     // x is in its registers up to here
__device__ __forceinline__ void mjt_pin(mjt_f32x4& x) { asm volatile("" : "+a"(x)); }             // what reads x later comes after this point
template <int OFF> __device__ __forceinline__ void mjt_ds_read(mjt_u32x4v& dst, unsigned addr) {
#if ABL & 4
    asm volatile("" : "+v"(dst) : "v"(addr));
#else
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF) : "memory");
#endif
}
// wait until at most N LDS operations issued after the one that fills x are outstanding (LDS returns in order)
template <int N> __device__ __forceinline__ void mjt_lds_wait(mjt_u32x4v& x) {
    asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(x) : "n"(N < 15 ? N : 15));   // the counter has four bits
}

extern "C" __global__ __launch_bounds__(NTHR) __attribute__((amdgpu_waves_per_eu(WPS, WPS))) void ENTRY(Params p) {
    // blockIdx.y = group of a grouped convolution (0 otherwise): its channels of x, its weights, its channels of y
    const unsigned short* __restrict__ xp = (const unsigned short*)p.a[0] + (size_t)blockIdx.y * (C_ * H_ * W_);
    const unsigned short* __restrict__ wp = (const unsigned short*)p.a[1] + (size_t)blockIdx.y * (K_ * C_ * R_ * S_);
    const int y_k0 = blockIdx.y * K_;
    const int n_img = (int)(unsigned long long)p.a[3];
    __shared__ __attribute__((aligned(16))) unsigned short xs[2][TILE_ELEMS];
    __shared__ __attribute__((aligned(16))) unsigned short as_ring[NS * KO_WG * 32 + 512];   // ring of weight slabs and a spare KB, see below

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
    // Every wave moves its share of the input rows of a block and of every weight slab.  Vector memory
    // operations of a wave complete in order: the ring is deep enough that the wait for a slab, which also waits
    // for every older load, never asks for an input row earlier than the row is needed itself.
    constexpr int ITEMS = ROWITEMS * SEGS * (CB / 8);                    // of a full tile
    constexpr int IPW = (ITEMS + NWAVES - 1) / NWAVES;            // items of one wave per channel block
    // A wave asks for item k of its share at the start of step fetch_step(k) and writes it to LDS at the end
    // of step fetch_step(k) + SD - 1: SD steps for the row to arrive from HBM, SG items per step, SQ registers.
    constexpr int STEPS = KSTEPS * R_ * S_;       // steps per channel block
    // When the steps of a block are too few for that (more than SGMAX items per step), the items of a step go in
    // rounds of at most SGMAX instead, each written as soon as it has arrived, the last one at the end of the step.
    constexpr int SGMAX = 8;
    // Rows on their way occupy registers the compiler knows nothing about (it takes a spelled-out load for finished when it
    // is issued): were it to run out of registers and move one of them aside, it would move what the load has not written
    // yet.  So their number stays inside what the loop leaves free of the 128 registers of a wave (B fragments and their
    // addresses: 5 per accumulator tile; A fragments, descriptors, selectors and addresses: 44), by way of a shorter flight.
    constexpr int SQMAX = (84 - 5 * NT) / 4;
    constexpr int SD1 = STEPS < STAGE_DEPTH ? STEPS : STAGE_DEPTH;
    constexpr auto sg_of = [](int sd) { return (IPW + (STEPS - sd + 1) - 1) / (STEPS - sd + 1); };
    constexpr auto sq_of = [=](int sd) { return sg_of(sd) * sd < IPW ? sg_of(sd) * sd : IPW; };
    constexpr auto fits = [=](int sd) { return sg_of(sd) <= SGMAX && sq_of(sd) <= SQMAX; };
    constexpr int SD0 = fits(SD1) ? SD1 : SD1 > 2 && fits(SD1 - 1) ? SD1 - 1 : SD1 > 3 && fits(SD1 - 2) ? SD1 - 2 : 0;
    constexpr bool BULK = SD0 == 0;
    constexpr int SD = BULK ? 1 : SD0;
    constexpr int SG = sg_of(SD);
    constexpr int RPS = BULK ? (SG + SGMAX - 1) / SGMAX : 1;      // rounds per step
    constexpr int RS = (SG + RPS - 1) / RPS;                      // items per round
    constexpr int SQ = BULK ? RS : SG * SD < IPW ? SG * SD : IPW;
    mjt_u32x4v stage[SQ];
    // buffer descriptors (base, size in bytes): addresses are a scalar offset plus a 32-bit lane offset,
    // so no per-item 64-bit address lives in vector registers
    const __amdgpu_buffer_rsrc_t x_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void*)(xp + (size_t)n * XC_ * H_ * W_), 0, C_ * H_ * W_ * 2, 0x00020000);
    const unsigned x_lane_off = (unsigned)sr * (H_ * W_ * 2);
    const unsigned as_spare = (unsigned)(unsigned long long)(__attribute__((address_space(3))) unsigned short*)&as_ring[0] + NS * KO_WG * 64;
    auto item_of = [&](int item, int& lr, int& seg, int& cg) {
        cg = item % (CB / 8);
        const int rest = item / (CB / 8);
        lr = rest / SEGS;
        seg = rest - lr * SEGS;
        lr *= RPI;                                           // the item's first row
    };
    // the lane's row inside an item and its group of 8 columns inside the row
    const int row_in_item = RPI > 1 ? sg / GP2 : 0, grp_in_row = RPI > 1 ? sg % GP2 : sg;
    // The loads are unconditional instructions (rows outside the image and idle lanes read a clamped address and
    // are zeroed or skipped when written; a wave whose role this is not reads beyond the descriptor's range, which
    // costs no memory traffic): around a load under a branch the compiler no longer knows how many loads are under
    // way and makes every later wait a wait for all of them.
    auto fetch_item = [&](bool live, int r0, int lrows, int cb, int item) -> mjt_u32x4v {   // of the tile whose first output row is r0
        const int ir0 = r0 * SH - PH;
        int lr, seg, cg;
        item_of(item, lr, seg, cg);
        if constexpr (RPI > 1) {                             // the row differs between lanes
            lr += row_in_item;
            int ir = ir0 + (lr < lrows ? lr : lrows - 1);
            ir = ir < 0 ? 0 : ir >= H_ ? H_ - 1 : ir;
            const int soff = __builtin_amdgcn_readfirstlane(((cb * CB + cg * 8) * H_ * W_) * 2);      // uniform: the channel group
            const int grp = grp_in_row < GROUPS ? grp_in_row : GROUPS - 1;
            return __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, (int)((live ? x_lane_off : 0x80000000u) + (unsigned)(ir * W_ * 2 + grp * 16)), soff, 0);
        } else {
            int ir = ir0 + (lr < lrows ? lr : lrows - 1);
            ir = ir < 0 ? 0 : ir >= H_ ? H_ - 1 : ir;
            const int soff = __builtin_amdgcn_readfirstlane((((cb * CB + cg * 8) * H_ + ir) * W_) * 2);     // uniform: channel group and row inside the image
            int grp = seg * 8 + sg;
            grp = grp < GROUPS ? grp : GROUPS - 1;
            return __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, (int)((live ? x_lane_off : 0x80000000u) + (unsigned)grp * 16), soff, 0);
        }
    };
    // Writing an item to LDS, in four stages that work in place on its four registers (the main loop spreads them
    // between its MFMAs): three exchanges, then the write.
    // The same load spelled out, for the main loop: every vector memory operation there is, and so the number of them
    // issued between two points is known and the waits can name exactly the loads that may still be under way.
    mjt_u32x4v x_desc;
    {
        const unsigned long long base = (unsigned long long)(xp + (size_t)n * XC_ * H_ * W_);
        x_desc[0] = __builtin_amdgcn_readfirstlane((unsigned)base);
        x_desc[1] = __builtin_amdgcn_readfirstlane((unsigned)(base >> 32) & 0xffffu);
        x_desc[2] = C_ * H_ * W_ * 2;
        x_desc[3] = 0x00020000;
    }
    auto fetch_item_fixed = [&](mjt_u32x4v& dst, bool live, int r0, int lrows, int cb, int item) {
        const int ir0 = r0 * SH - PH;
        int lr, seg, cg;
        item_of(item, lr, seg, cg);
        int soff;
        unsigned voff;
        if constexpr (RPI > 1) {
            lr += row_in_item;
            int ir = ir0 + (lr < lrows ? lr : lrows - 1);
            ir = ir < 0 ? 0 : ir >= H_ ? H_ - 1 : ir;
            soff = __builtin_amdgcn_readfirstlane(((cb * CB + cg * 8) * H_ * W_) * 2);
            const int grp = grp_in_row < GROUPS ? grp_in_row : GROUPS - 1;
            voff = (live ? x_lane_off : 0x80000000u) + (unsigned)(ir * W_ * 2 + grp * 16);
        } else {
            int ir = ir0 + (lr < lrows ? lr : lrows - 1);
            ir = ir < 0 ? 0 : ir >= H_ ? H_ - 1 : ir;
            soff = __builtin_amdgcn_readfirstlane((((cb * CB + cg * 8) * H_ + ir) * W_) * 2);
            int grp = seg * 8 + sg;
            grp = grp < GROUPS ? grp : GROUPS - 1;
            voff = (live ? x_lane_off : 0x80000000u) + (unsigned)grp * 16;
        }
        asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=v"(dst) : "v"(voff), "s"(x_desc), "s"(soff) : "memory");
    };
    auto commit_stage = [&](auto sc, bool live, mjt_u32x4v& d, int r0, int lrows, int buf, int item, int limit) {
        constexpr int stg = decltype(sc)::v;
        // (the item number is made opaque here: what follows from it is worked out in place, with scalar instructions,
        // instead of once per item in front of the loop, where every item's address would hold a register for good)
        item = __builtin_amdgcn_readfirstlane(item);         // (it is the same in every lane)
        asm volatile("" : "+s"(item));
        int lr, seg, cg;
        item_of(item, lr, seg, cg);
        if constexpr (stg == 0) {
            // d[k] = columns 2k (low half), 2k+1 (high half) of channel r
            const int ir0 = r0 * SH - PH;
            if constexpr (RPI > 1) {                         // per lane: the rows of an item
                const bool outside = ir0 + lr + row_in_item < 0 || ir0 + lr + row_in_item >= H_;
                d[0] = outside ? 0u : d[0]; d[1] = outside ? 0u : d[1]; d[2] = outside ? 0u : d[2]; d[3] = outside ? 0u : d[3];
            } else {
                if (ir0 + lr < 0 || ir0 + lr >= H_) d = (mjt_u32x4v)(0u);   // uniform: a row outside the image
            }
            // lane ^ 4: keep one half of the columns, get the same half from the channel 4 away
            const unsigned g0 = mjt_xor4(b2 ? d[0] : d[2]), g1 = mjt_xor4(b2 ? d[1] : d[3]);
            const unsigned a0 = b2 ? g0 : d[0], a1 = b2 ? g1 : d[1];      // channel r & 3:       column pairs 0, 1 of the half
            const unsigned a2 = b2 ? d[2] : g0, a3 = b2 ? d[3] : g1;      // channel (r & 3) + 4
            d[0] = a0; d[1] = a1; d[2] = a2; d[3] = a3;
        } else if constexpr (stg == 1) {
            // lane ^ 2: keep one column pair, get it from the channel 2 away
            const unsigned h0 = mjt_xor2(b1 ? d[0] : d[1]), h1 = mjt_xor2(b1 ? d[2] : d[3]);
            const unsigned c0 = b1 ? h0 : d[0], c1 = b1 ? d[1] : h0;      // channels q, q+2 (q = r & 1), one column pair
            const unsigned c2 = b1 ? h1 : d[2], c3 = b1 ? d[3] : h1;      // channels q+4, q+6
            d[0] = c0; d[1] = c1; d[2] = c2; d[3] = c3;
        } else if constexpr (stg == 2) {
            // lane ^ 1: keep one column, get it from the neighbouring channels (two 16-bit values per
            // move; byte permutes with per-lane selectors keep this free of branches)
            const unsigned s0 = mjt_xor1(__builtin_amdgcn_perm(d[1], d[0], sel_t)), s1 = mjt_xor1(__builtin_amdgcn_perm(d[3], d[2], sel_t));
            mjt_u32x4v f;                                    // channels (0,1) (2,3) (4,5) (6,7) of column 8g + r
            f[0] = __builtin_amdgcn_perm(s0, d[0], sel_a);
            f[1] = __builtin_amdgcn_perm(s0, d[1], sel_b);
            f[2] = __builtin_amdgcn_perm(s1, d[2], sel_a);
            f[3] = __builtin_amdgcn_perm(s1, d[3], sel_b);
            d = f;
        } else {
            // rows outside the image carry zeros; columns past the row end are not the row's; what is not to be written
            // goes to the spare piece of LDS.  The write is spelled out: a compiler-made LDS access after the copies
            // into the slab ring would wait for all of those first.
            // (after the exchanges the lane holds column 8 * group + lane % 8 of its row)
            const int lrow = lr + row_in_item, col = RPI > 1 ? grp_in_row * 8 + sr : seg * 64 + lane;
            const bool wr = live && item < limit && lrow < lrows && col < W_;
            const unsigned dst = wr ? xs_base + (unsigned)(buf * TILE_ELEMS + mjt_lds_off(lrow * LCOLS + PW + col, cg)) * 2
                                    : as_spare + (unsigned)lane * 16;
            asm volatile("ds_write_b128 %0, %1" : : "v"(dst), "v"(d) : "memory");
        }
    };
    auto commit_item = [&](bool live, mjt_u32x4v d, int r0, int lrows, int buf, int item, int limit) {
        mjt_static_for<0, 4>([&](auto sc) { commit_stage(sc, live, d, r0, lrows, buf, item, limit); });
    };

    // A fragments: Wp[step][ko / 16][lane][8 c], step = (tap * NCB + cb) * KSTEPS + ks: a fragment is 1 KB in lane order
    // (lane = lg * 16 + l16 holds channels lg*8.. of row l16).  The fragments of one step for the workgroup's
    // output channels (a slab: KO_WG / 16 KB, contiguous in Wp) go through a ring of NS slabs in LDS: while step g
    // runs the waves copy slab g + NS - 1 straight from memory into LDS (no registers); every wave reads its own
    // MT fragments from the ring two passes ahead of the MFMAs.  One barrier per step hands a landed slab over and
    // frees the oldest one.
    constexpr int SLAB = KO_WG * 64;              // bytes
    constexpr int FPL = (KO_WG / 16) / NWAVES;    // fragments a wave moves per slab
    const unsigned as_base = (unsigned)(unsigned long long)(__attribute__((address_space(3))) unsigned short*)&as_ring[0];
    const unsigned a_rd_base = as_base + (unsigned)(wko * MT * 1024 + lane * 16);
    const __amdgpu_buffer_rsrc_t w_rsrc =
        __builtin_amdgcn_make_buffer_rsrc((void*)(wp + (size_t)kpart * KO_WG * 32), 0, (R_ * S_ * C_ * K_ - kpart * KO_WG * 32) * 2, 0x00020000);
    auto slab_load = [&](int cb, int st, int slot) {          // all arguments uniform
        const int tap = st / KSTEPS, ks = st % KSTEPS;
        const int soff = ((tap * NCB + cb) * KSTEPS + ks) * (K_ * 64) + wave * (FPL * 1024);
        __attribute__((address_space(3))) unsigned short* dst =
            (__attribute__((address_space(3))) unsigned short*)&as_ring[0] + (slot * SLAB + wave * (FPL * 1024)) / 2;
        const unsigned voff = (unsigned)lane * 16;
        if (ABL & 4) return;
        mjt_static_for<0, FPL>([&](auto fc) {
            constexpr int f = decltype(fc)::v;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(w_rsrc, (__attribute__((address_space(3))) void*)(dst + (f >> 2) * 2048), 16, (int)voff,
                                                     soff + (f >> 2) * 4096, (f & 3) * 1024, 0);
        });
    };
    // (channel block, step) k steps after (cb, st); the sequence wraps after the last block: every tile uses the same weights
    auto slab_ahead = [&](int cb, int st, int k, int& cb2, int& st2) {
        st2 = st + k;
        cb2 = cb;
        while (st2 >= STEPS) {
            st2 -= STEPS;
            cb2 = cb2 + 1 < NCB ? cb2 + 1 : 0;
        }
    };
    // End of step g: slab g + 2 has landed (the next step reads its first fragments).  What was asked for later may
    // still be under way: the loads of the last NS - 3 steps, slabs and input rows alike (all of them are spelled out
    // in the loop, so their number is known).
    auto step_sync = [&](auto nc) {                  // nc: loads issued in the last NS - 3 steps, this one included
        asm volatile("s_waitcnt vmcnt(%0)" : : "n"(decltype(nc)::v < 63 ? decltype(nc)::v : 63) : "memory");
        if (!(ABL & 4)) asm volatile("s_barrier" : : : "memory");
    };

    int buf = 0;                                  // LDS buffer that holds the current channel block
    int g = 0;                                    // steps done so far, modulo NS: slab of the current step is in slot g

    // One tile: TRW_ output rows per wave starting at r0, NT_ accumulator tiles per wave, LR_ input rows
    // in LDS.  On entry its first channel block is in xs[buf], its first A fragments are in ring[0] and the
    // slabs of its first three steps are in the ring or under way; when another tile follows
    // (next_lrows > 0) its first block is prepared the same way.
    auto run_tile = [&](auto trw_c, auto nt_c, auto lr_c, const int r0, const int row_lim, const int next_r0, const int next_lrows) {
        constexpr int TRW_ = decltype(trw_c)::v, NT_ = decltype(nt_c)::v, LR_ = decltype(lr_c)::v;
        // per-lane pixel of each of the NT_ tiles
        unsigned baddr[NT_];                                 // LDS byte address of the fragment at tap (0,0), k-step 0, in the current buffer
        // (from a copy of the lane number made here: worked out per tile, the addresses of the full and of the short tile do
        // not both hold registers for the whole kernel)
        int lane_t = lane;
        asm volatile("" : "+v"(lane_t));
#pragma unroll
        for (int t = 0; t < NT_; t++) {
            int q = t * 16 + (lane_t & 15);
            int r = q / OW_, col = q - r * OW_;
            if (q >= TRW_ * OW_) { r = 0; col = 0; }
            baddr[t] = xs_base + (unsigned)(buf * TILE_ELEMS * 2) + (unsigned)mjt_lds_off(((wpx * TRW_ + r) * SH) * LCOLS + col * SW, lane_t >> 4) * 2;
        }
        mjt_f32x4 acc[MT][NT_];
#pragma unroll
        for (int m = 0; m < MT; m++)
#pragma unroll
            for (int t = 0; t < NT_; t++) acc[m][t] = (mjt_f32x4)(0.0f);
        // the zeros are written here, not next to the first MFMA that reads them: between a plain write of a register
        // and a spelled-out MFMA that reads it the compiler leaves none of the cycles the hardware asks for
        mjt_static_for<0, MT * NT_>([&](auto ic) { mjt_pin(acc[decltype(ic)::v / NT_][decltype(ic)::v % NT_]); });
        asm volatile("s_nop 7" : : : "memory");

        // Main loop.  A step multiplies MT A fragments with NT_ B fragments.  It runs fragment by fragment of A
        // (MT passes of NT_ MFMAs on independent accumulators): the A fragment of the next pass is read during a
        // pass, and in the last pass each B register is refilled with the next step's fragment right after
        // its last use, so that every LDS read has at least a pass of MFMAs to arrive.  The reads and the
        // waits for them are written out so that this order is what runs (tap and k-step are compile-time here
        // and fold into the offset field of the read).  LDS operations of a wave complete in order; a wait names
        // how many of those issued later may still be under way.
        constexpr auto writes_in = [](int st) {                  // input rows written to LDS at the end of step st
            int n = 0;
            for (int k = 0; k < IPW; k++) n += (k / SG + SD - 1 == st) ? 1 : 0;
            return n;
        };
        // input-row loads a wave issues in step s of a block (s may run past the block's ends: every block has the same schedule)
        constexpr auto loads_in = [](int s) {
            const int st = ((s % STEPS) + STEPS) % STEPS;
            int n = 0;
            for (int k = 0; k < IPW; k++) n += (k / SG == st) ? 1 : 0;
            return n;
        };
        constexpr auto loads_between = [=](int s0, int s1) {      // in steps s0 .. s1 - 1
            int n = 0;
            for (int s = s0; s < s1; s++) n += loads_in(s);
            return n;
        };
        // item i of round r of step st, or -1
        constexpr auto bulk_item = [](int st, int r, int i) {
            const int k = st * SG + r * RS + i;
            return (r * RS + i < SG && k < IPW) ? k : -1;
        };
        mjt_u32x4v bfr[NT_];
        mjt_u32x4v afr[3];                                   // A fragments of this pass and the next two
        constexpr int PASSES = STEPS * MT;
#pragma unroll 1
        for (int cb = 0; cb < NCB; cb++) {
            const bool more = cb + 1 < NCB;
            const bool feed = (more || next_lrows) && !(ABL & 2);   // somebody needs another block of input rows
            const int f_r0 = more ? r0 : next_r0, f_lrows = more ? LR_ : next_lrows, f_cb = more ? cb + 1 : 0;
            const int my_first = wave * IPW, my_limit = (wave + 1) * IPW < ITEMS ? (wave + 1) * IPW : ITEMS;
            // nothing is under way here
            mjt_ds_read<0>(afr[0], a_rd_base + (unsigned)((g % NS) * SLAB));
            mjt_ds_read<1024>(afr[1], a_rd_base + (unsigned)((g % NS) * SLAB));
            mjt_static_for<0, NT_>([&](auto tc) { mjt_ds_read<mjt_frag_off(0)>(bfr[decltype(tc)::v], baddr[decltype(tc)::v]); });
            mjt_static_for<0, STEPS>([&](auto sc) {
                constexpr int st = decltype(sc)::v;
                // what a step does besides its MFMAs goes between them, where it costs no MFMA time: the loads right after
                // the first one, the stages of writing input rows to LDS after MFMA number stage_at(0..3) of the step
                auto issue_loads = [&]() {
                    if constexpr (!BULK) {
                        mjt_static_for<0, IPW>([&](auto kc) {
                            constexpr int k = decltype(kc)::v;
                            if constexpr (k / SG == st) fetch_item_fixed(stage[k % SQ], feed, f_r0, f_lrows, f_cb, my_first + k);
                        });
                    } else {
                        mjt_static_for<0, RPS>([&](auto rc) {
                            constexpr int r = decltype(rc)::v;
                            mjt_static_for<0, RS>([&](auto ic) {
                                constexpr int k = bulk_item(st, r, decltype(ic)::v);
                                if constexpr (k >= 0) stage[decltype(ic)::v] = fetch_item(feed, f_r0, f_lrows, f_cb, my_first + k);
                            });
                            if constexpr (r + 1 < RPS)
                                mjt_static_for<0, RS>([&](auto ic) {
                                    constexpr int k = bulk_item(st, r, decltype(ic)::v);
                                    if constexpr (k >= 0) commit_item(feed, stage[decltype(ic)::v], f_r0, f_lrows, buf ^ 1, my_first + k, my_limit);
                                });
                        });
                    }
                    int cb3, st3;
                    slab_ahead(cb, st, NS - 1, cb3, st3);
                    slab_load(cb3, st3, (g + st + NS - 1) % NS);
                };
                constexpr auto stage_at = [](int sg) { return NT_ + (sg * (MT - 2) * NT_) / 4; };
                auto commit_stages = [&](auto ic) {          // ic: MFMAs of this step issued so far
                    constexpr int i = decltype(ic)::v;
                    mjt_static_for<0, 4>([&](auto sc) {
                        if constexpr (stage_at(decltype(sc)::v) == i) {
                            if constexpr (!BULK) {
                                mjt_static_for<0, IPW>([&](auto kc) {
                                    constexpr int k = decltype(kc)::v;
                                    if constexpr (k / SG + SD - 1 == st) {
                                        // loads issued after that of item k: the rest of its step (input rows come first in a step, then
                                        // the slab), then SD - 1 whole steps
                                        if constexpr (decltype(sc)::v == 0) {
                                            constexpr int after = (loads_in(k / SG) - 1 - k % SG) + FPL + (SD - 1) * FPL + loads_between(k / SG + 1, k / SG + SD);
                                            asm volatile("s_waitcnt vmcnt(%1)" : "+v"(stage[k % SQ]) : "n"(after < 63 ? after : 63));
                                        }
                                        commit_stage(sc, feed, stage[k % SQ], f_r0, f_lrows, buf ^ 1, my_first + k, my_limit);   // the other buffer: nobody reads it now
                                    }
                                });
                            } else {
                                mjt_static_for<0, RS>([&](auto jc) {
                                    constexpr int k = bulk_item(st, RPS - 1, decltype(jc)::v);
                                    if constexpr (k >= 0) commit_stage(sc, feed, stage[decltype(jc)::v], f_r0, f_lrows, buf ^ 1, my_first + k, my_limit);
                                });
                            }
                        }
                    });
                };
                const unsigned a_cur = a_rd_base + (unsigned)(((g + st) % NS) * SLAB);
                const unsigned a_nxt = a_rd_base + (unsigned)(((g + st + 1) % NS) * SLAB);
                mjt_static_for<0, MT>([&](auto mc) {
                    constexpr int m = decltype(mc)::v;
                    constexpr int P = st * MT + m;                           // pass number in the block; its fragment sits in afr[P % 3]
                    if constexpr (P + 2 < PASSES) {                          // the fragment two passes ahead: of this step or the next
                        if constexpr (m + 2 < MT) mjt_ds_read<(m + 2) * 1024>(afr[(P + 2) % 3], a_cur);
                        else mjt_ds_read<(m + 2 - MT) * 1024>(afr[(P + 2) % 3], a_nxt);
                    }
                    mjt_static_for<0, NT_>([&](auto tc) {
                        constexpr int t = decltype(tc)::v;
                        // the rows written in this step are written before its last pass: no LDS write follows the B reads
                        // B fragment t was asked for before the reads of the rest of its step and of the A fragment two passes
                        // ahead (the A fragment of this pass is older than all of those); behind an A fragment come those of
                        // the next two passes
                        if constexpr (m == 0) mjt_lds_wait<(BULK ? 0 : NT_ - 1 - t + (P + 2 < PASSES ? 1 : 0))>(bfr[t]);
                        else if constexpr (t == 0) mjt_lds_wait<(P + 1 < PASSES ? 1 : 0) + (P + 2 < PASSES ? 1 : 0)>(afr[P % 3]);
                        mjt_mfma(acc[m][t], bfr[t], afr[P % 3]);
                        if constexpr (m + 1 == MT && st + 1 < STEPS) mjt_ds_read<mjt_frag_off(st + 1)>(bfr[t], baddr[t]);
                        if constexpr (m == 0 && t == 0) issue_loads();
                        commit_stages(mjt_ic<m * NT_ + t + 1>());
                    });
                });
                if (st + 1 == STEPS) asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");   // the rows written for the next block
                step_sync(mjt_ic<(BULK ? 0 : (NS - 3) * FPL + loads_between(st - (NS - 4), st + 1))>());
            });
            g = (g + STEPS) % NS;
            if (feed) {
                buf ^= 1;
#pragma unroll
                for (int t = 0; t < NT_; t++) baddr[t] += buf ? (unsigned)(TILE_ELEMS * 2) : (unsigned)(-(TILE_ELEMS * 2));
            }
        }

        // epilogue: lane holds D[px = 4*(lane/16)+i][ko = lane%16] of each tile
        // The compiler takes a spelled-out MFMA for finished the moment it is issued.  Give the last ones the
        // time to read their operands and write their results, and tie the registers to a point behind that:
        // the operands stay allocated up to here, and nothing reads an accumulator before.
        asm volatile("s_nop 15\n\ts_nop 15" : : : "memory");
        mjt_keep(afr[0]);
        mjt_keep(afr[1]);
        mjt_keep(afr[2]);
        mjt_static_for<0, NT_>([&](auto tc) { mjt_keep(bfr[decltype(tc)::v]); });
        mjt_static_for<0, MT * NT_>([&](auto ic) { mjt_pin(acc[decltype(ic)::v / NT_][decltype(ic)::v % NT_]); });
        // (the lane's coordinates are taken from a copy of the lane number made here: what is worked out from it cannot
        // be moved in front of the loop, where it would sit in registers the loop needs)
        int lane_e = lane;
        asm volatile("" : "+v"(lane_e));
        const int l16_e = lane_e & 15, lg_e = lane_e >> 4;
#pragma unroll
        for (int t = 0; t < NT_; t++) {
#if OW_ % 4 == 0
            // 16 bytes (8 as a 16-bit type) per lane: four pixels never straddle an output row because OW is a multiple
            // of 4.  The four 16-lane rows of a register make up the 64 bytes of a pixel tile, for 16 channels.
            // (Regrouping registers so that an instruction writes 256-byte runs of 4 channels, by quad transposes
            // or row swaps, was no faster.)
            const int q0 = t * 16 + lg_e * 4;
            const int r = q0 / OW_, col = q0 - r * OW_;
            const int orow = r0 + wpx * TRW_ + r;
            if (q0 < TRW_ * OW_ && orow < row_lim && !(ABL & 1)) {
#pragma unroll
                for (int m = 0; m < MT; m++) {
                    const mjt_f32x4 v = acc[m][t];
                    const size_t o = (((size_t)n * YK_ + y_k0 + ko_base + m * 16 + l16_e) * OH_ + orow) * OW_ + col;
#if Y_BF16
                    mjt_u32x2 pk;
                    pk[0] = mjt_narrow2(v[0], v[1]);
                    pk[1] = mjt_narrow2(v[2], v[3]);
                    *(mjt_u32x2*)((unsigned short*)p.a[2] + o) = pk;
#else
                    *(mjt_f32x4*)((float*)p.a[2] + o) = v;
#endif
                }
            }
#elif OW_ % 2 == 0
            // an even width: pairs of pixels never straddle an output row (widths of 14: half the stores of single pixels)
#pragma unroll
            for (int i = 0; i < 4; i += 2) {
                const int q = t * 16 + lg_e * 4 + i;
                const int r = q / OW_, col = q - r * OW_;
                const int orow = r0 + wpx * TRW_ + r;
                if (q < TRW_ * OW_ && orow < row_lim && !(ABL & 1)) {
#pragma unroll
                    for (int m = 0; m < MT; m++) {
                        const size_t o = (((size_t)n * YK_ + y_k0 + ko_base + m * 16 + l16_e) * OH_ + orow) * OW_ + col;
#if Y_BF16
                        *(unsigned*)((unsigned short*)p.a[2] + o) = mjt_narrow2(acc[m][t][i], acc[m][t][i + 1]);
#else
                        mjt_f32x2 pr;
                        pr[0] = acc[m][t][i];
                        pr[1] = acc[m][t][i + 1];
                        *(mjt_f32x2*)((float*)p.a[2] + o) = pr;
#endif
                    }
                }
            }
#else
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int q = t * 16 + lg_e * 4 + i;
                const int r = q / OW_, col = q - r * OW_;
                const int orow = r0 + wpx * TRW_ + r;
                if (q < TRW_ * OW_ && orow < row_lim && !(ABL & 1)) {
#pragma unroll
                    for (int m = 0; m < MT; m++) {
                        const size_t o = (((size_t)n * YK_ + y_k0 + ko_base + m * 16 + l16_e) * OH_ + orow) * OW_ + col;
#if Y_BF16
                        ((unsigned short*)p.a[2])[o] = (unsigned short)mjt_narrow2(acc[m][t][i], 0.0f);
#else
                        ((float*)p.a[2])[o] = acc[m][t][i];
#endif
                    }
                }
            }
#endif
        }
    };
    // tiles of this workgroup: full tiles while they start inside the row range, then the short one
    int nfull = (row_end - row_begin + TR - 1) / TR;
    if (nfull > NFULL) nfull = NFULL;
    const bool tail = TAIL_TRW > 0 && row_begin + NFULL * TR < row_end;
    const int first_lrows = nfull ? LROWS : TAIL_LROWS;
    const int ntiles = nfull + (tail ? 1 : 0);

    // the slabs of the first NS - 1 steps and the first block of input rows (every wave takes a share)
    mjt_static_for<0, NS - 1>([&](auto kc) {
        int cb0, st0;
        slab_ahead(0, 0, decltype(kc)::v, cb0, st0);
        slab_load(cb0, st0, decltype(kc)::v);
    });
    __syncthreads();                              // zero fill done
    {
        constexpr int PQ0 = (ITEMS + NWAVES - 1) / NWAVES;     // no accumulators yet: registers to spare
        constexpr int PQ = PQ0 < 16 ? PQ0 : 16;
        mjt_u32x4v pre[PQ];
#pragma unroll 1
        for (int first = wave * PQ; first < ITEMS; first += NWAVES * PQ) {
#pragma unroll
            for (int k = 0; k < PQ; k++) pre[k] = fetch_item(true, row_begin, first_lrows, 0, first + k);
#pragma unroll
            for (int k = 0; k < PQ; k++) commit_item(true, pre[k], row_begin, first_lrows, 0, first + k, ITEMS);
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");   // the slabs
    __syncthreads();
#pragma unroll 1
    for (int i = 0; i < ntiles; i++) {
        const int next_lrows = i + 1 >= ntiles ? 0 : i + 1 == nfull ? TAIL_LROWS : LROWS;
        const int r0 = row_begin + i * TR;
#if TAIL_TRW > 0
        if (i == nfull) {
            run_tile(mjt_ic<TAIL_TRW>(), mjt_ic<TAIL_NT>(), mjt_ic<TAIL_LROWS>(), r0, row_end, 0, 0);
            continue;
        }
#endif
        run_tile(mjt_ic<TRW>(), mjt_ic<NT>(), mjt_ic<LROWS>(), r0, row_end, r0 + TR, next_lrows);
    }
    asm volatile("s_waitcnt vmcnt(0)" : : : "memory");   // slabs asked for past the last step
}

// Weight re-pack: w[ko][c][kh][kw] -> Wp[tap][c/CB][k-step][ko/16][lg][l16][8 c] (c = CB block + 32 k-step + 8 lg + ..)
extern "C" __global__ __launch_bounds__(256) void ENTRY_PACK(Params p) {
    const int total = K_ * C_ * R_ * S_;                      // of one group: blockIdx.y
    const unsigned short* __restrict__ w = (const unsigned short*)p.a[0] + (size_t)blockIdx.y * total;
    unsigned short* __restrict__ wp = (unsigned short*)p.a[1] + (size_t)blockIdx.y * total;
    for (int o = blockIdx.x * 256 + threadIdx.x; o < total; o += gridDim.x * 256) {
        int c8 = o & 7, l16 = (o >> 3) & 15, lg = (o >> 7) & 3;
        int rest = o >> 9;
        int ko = (rest % (K_ / 16)) * 16 + l16; rest /= K_ / 16;
        int c32 = lg * 8 + c8;
        int ks = rest % KSTEPS; rest /= KSTEPS;
        int cb = rest % NCB;
        int tap = rest / NCB;
        int c = cb * CB + ks * 32 + c32;
        wp[o] = w[((size_t)ko * C_ + c) * (R_ * S_) + tap];
    }
}
