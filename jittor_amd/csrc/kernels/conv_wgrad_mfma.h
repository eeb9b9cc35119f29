// Weight gradient of the meta-op convolution on MFMA: the group
//   reduce.add over (n, oh, ow) of  reindex(x) * broadcast(dy)
// that jt.grad builds for the weights (python/jittor/nn.py:1251-1262 differentiated by
// ops/reduce_op.cc:339-362, ops/broadcast_to_op.cc:112-117; recognised by
// opt/tuner/conv_tuner.cc:375-397 and relayed there to a backward-w library call):
//   dW[k][c][r][s] = sum_{n,oh,ow} dy[n][k][oh][ow] * x[n][c][oh*SH-PH+r*DH][ow-PW+s*DW]
// for bfloat16 (or, with IN_F16, float16) operands with exact products and float32 accumulation; taps outside the image
// contribute 0.  Horizontal stride 1 only (consecutive output columns read consecutive input
// columns), everything else is baked in by the host: C_, H_, W_, K_, R_, S_, OH_, OW_, SH, PH, PW, DH,
// DW, KG (groups of 64 output channels per workgroup: 1, 2 or 4; the 8 waves of a workgroup are KG
// channel groups x 8 / KG tiles of 16 input channels).
//
// Mapping.  The contraction runs over pixels, and in NCHW both operands have the pixels of a row
// contiguous, so no transposes are needed: v_mfma_f32_16x16x32_bf16 computes
// D[16 k][16 c] += A[16 k][32 px] * B[32 px][16 c] with lane (l16, lg) of A holding
// dy[k = l16][8 pixels lg*8..], of B holding x[c = l16][the same 8 pixels, shifted by the tap].
// A step is one chunk of 32 output columns of one output row of one image: 4 fragments of dy,
// R_*S_ of x, 4*R_*S_ MFMAs per wave.  In that lane order neighbouring lanes read different rows
// (a cache line per lane), so a fragment is fetched in row order instead -- lane i takes 16 bytes of
// row i / 4, piece i % 4, four neighbouring lanes one 64-byte run -- by a load that writes straight
// into a 1 KB slot of LDS (no registers), and read back from there in fragment order.  The slots of
// a step are shared: the waves of one channel group read the same dy fragments, the waves of one
// channel tile the same x fragments, so each is fetched once per workgroup (the loads are dealt
// out to the 8 waves) and a barrier per step separates filling from reading.  A fragment of x whose column shift is odd starts in the middle of a dword: it
// comes as the four dwords above its first element plus the dword below, shifted down by 16 bits
// (every load is dword-aligned).  Columns outside the image (and the columns of a last, partial
// chunk) are cleared with lane masks; rows and images outside read zeros through the
// range check of the buffer loads (the whole offset travels in the lane offset, which is what the
// hardware checks).  While the MFMAs of a step run, the loads of the next step fill a second set
// of slots (when two sets fit into LDS; otherwise the same set, after a second barrier).
//
// A workgroup owns 64*KG output channels x 16*8/KG input channels x all taps, over the output rows
// [slice*rps, slice*rps+rps) of the batch (row n*OH + oh: a slice may be a part of an image or span
// several): the partial sums of the slices go to partial[slice][k][c][r][s] (float32) and are added
// up by a reduce launch.

#if IN_F16
typedef _Float16 mjt_bf16x8 __attribute__((ext_vector_type(8)));
#define MJT_MFMA __builtin_amdgcn_mfma_f32_16x16x32_f16
#else
typedef __bf16 mjt_bf16x8 __attribute__((ext_vector_type(8)));
#define MJT_MFMA __builtin_amdgcn_mfma_f32_16x16x32_bf16
#endif
typedef float mjt_f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned mjt_u32x4v __attribute__((ext_vector_type(4)));

struct Params { void* a[6]; };   // x, dy, partial, number of images, images per slice (typed as pointers: 8-byte words)

// ABL (0 in production): timing-only ablations, results are wrong with any bit set.  1: the loads of dy fetch nothing
// (offsets beyond the buffer: zeros, no memory traffic), 2: likewise the loads of x, 4: no MFMAs, 8: no fragment reads
// from LDS, 16: no loads issued at all, 32: the partial sums are not stored.
#ifndef ABL
#define ABL 0
#endif
#define TAPS (R_ * S_)
#define NCHUNK ((OW_ + 31) / 32)
#define CTW (8 / KG)
#define INVALID 0x80000000u      // added to an offset: beyond every buffer, the load returns zeros

template <int V> struct mjt_ic { static constexpr int v = V; };
template <int I, int N, class F> __device__ __forceinline__ void mjt_static_for(F&& f) {
    if constexpr (I < N) {
        f(mjt_ic<I>());
        mjt_static_for<I + 1, N>(f);
    }
}
__device__ constexpr int mjt_col_shift(int s) { return s * DW - PW; }      // input column - output column of tap column s
// does chunk ch with tap column s reach outside the row (of dy or of x)?
__device__ constexpr bool mjt_edge(int ch, int s) {
    return ch * 32 + mjt_col_shift(s) < 0 || ch * 32 + 31 + mjt_col_shift(s) >= W_ || ch * 32 + 31 >= OW_;
}

typedef unsigned mjt_u32x2 __attribute__((ext_vector_type(2)));
template <int OFF> __device__ __forceinline__ void mjt_ds_read128(mjt_u32x4v& dst, unsigned addr) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF) : "memory");
}
__device__ __forceinline__ void mjt_no_mfma(mjt_f32x4& c, const mjt_u32x4v& a, const mjt_u32x4v& b) { asm volatile("" : "+v"(c) : "v"(a), "v"(b)); }
__device__ __forceinline__ void mjt_pin_acc(mjt_f32x4& x) { asm volatile("" : "+v"(x)); }
__device__ __forceinline__ void mjt_ds_read32(unsigned& dst, unsigned addr) { asm volatile("ds_read_b32 %0, %1" : "=v"(dst) : "v"(addr) : "memory"); }
__device__ __forceinline__ void mjt_ds_read64(mjt_u32x2& dst, unsigned addr) { asm volatile("ds_read_b64 %0, %1" : "=v"(dst) : "v"(addr) : "memory"); }
// wait until at most N LDS operations issued after the one that fills x are outstanding (the counter has four bits)
template <int N> __device__ __forceinline__ void mjt_lds_wait(mjt_u32x4v& x) { asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(x) : "n"(N < 15 ? N : 15)); }
template <int N> __device__ __forceinline__ void mjt_lds_wait1(unsigned& x) { asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(x) : "n"(N < 15 ? N : 15)); }
template <int N> __device__ __forceinline__ void mjt_lds_wait2(mjt_u32x2& x) { asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(x) : "n"(N < 15 ? N : 15)); }

extern "C" __global__ __launch_bounds__(512) void ENTRY(Params p) {
    const int n_img = (int)(unsigned long long)p.a[3];
    const int rps = (int)(unsigned long long)p.a[4];                    // output rows (of all images, in order) per slice
    float* __restrict__ partial = (float*)p.a[2];

    // the last block of input channels may reach beyond C_ (a multiple of 16): its tiles there read zeros and write nothing
    constexpr int KBLOCKS = K_ / (64 * KG), CBLOCKS = (C_ + 16 * CTW - 1) / (16 * CTW);
    // the workgroups of one slice read the same dy: they are 8 apart, so that they land on the same XCD
    // (workgroups go round-robin over the 8 XCDs) and share it through that XCD's L2
    const int id = blockIdx.x;
    const int xcd = id & 7, j = id >> 3;
    const int kblock = j % KBLOCKS;
    const int cblock = (j / KBLOCKS) % CBLOCKS;
    const int slice = (j / (KBLOCKS * CBLOCKS)) * 8 + xcd;
    const int n_rows = n_img * OH_;
    if (slice * rps >= n_rows) return;                      // the grid is padded to a multiple of 8 slices
    const int row_begin = slice * rps;
    const int row_end = row_begin + rps < n_rows ? row_begin + rps : n_rows;
    const int img_begin = row_begin / OH_, oh_begin = row_begin - img_begin * OH_;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kg = wave % KG, ct = wave / KG;
    const int k0 = (kblock * KG + kg) * 64, c0 = (cblock * CTW + ct) * 16;
    const int l16 = lane & 15, lg = lane >> 4;

    // Which of a lane's 8 elements lie inside the image, per (chunk, tap column): 16 bits per element pair.  Only the
    // combinations that touch an edge of the row are ever applied (the first chunk with a negative shift, the last
    // chunk), the others are never materialised.
    mjt_u32x4v masks[NCHUNK * S_];
    mjt_static_for<0, NCHUNK * S_>([&](auto ic) {
        constexpr int idx = decltype(ic)::v, ch = idx / S_, s = idx % S_;
        if constexpr (mjt_edge(ch, s)) {
            constexpr int off = mjt_col_shift(s);
#pragma unroll
            for (int j = 0; j < 4; j++) {
                unsigned v = 0;
#pragma unroll
                for (int h = 0; h < 2; h++) {
                    const int ow = ch * 32 + lg * 8 + 2 * j + h, iw = ow + off;
                    if (ow < OW_ && iw >= 0 && iw < W_) v |= h ? 0xffff0000u : 0x0000ffffu;
                }
                masks[idx][j] = v;
            }
        }
    });

    // An output width that is no multiple of 8: the last piece of dy that a row has ends in the next row's first columns.
    // The fragments of x are zero there (the masks above), but a product with zero is only zero for finite values, so the
    // lane group that holds that piece clears what lies beyond the row in dy as well.
    constexpr bool DY_TAIL = OW_ % 8 != 0;
    mjt_u32x4v dy_mask = (mjt_u32x4v)(0xffffffffu);
    if constexpr (DY_TAIL) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            unsigned v = 0;
#pragma unroll
            for (int h = 0; h < 2; h++)
                if ((NCHUNK - 1) * 32 + lg * 8 + 2 * j + h < OW_) v |= h ? 0xffff0000u : 0x0000ffffu;
            dy_mask[j] = v;
        }
    }

    // buffer descriptors over the whole tensors; every offset is a lane offset, so the range check sees all of it
    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(p.a[0], 0, n_img * (C_ * H_ * W_ * 2), 0x00020000);
    const __amdgpu_buffer_rsrc_t y_rsrc = __builtin_amdgcn_make_buffer_rsrc(p.a[1], 0, n_img * (K_ * OH_ * OW_ * 2), 0x00020000);
    // fetch order: lane i takes row i / 4 of the fragment (an output or input channel), piece i % 4 (8 columns)
    const int frow = lane >> 2, fpiece = lane & 3;
    const unsigned a_lane = (unsigned)((frow * OH_ * OW_ + fpiece * 8) * 2);
    const unsigned b_lane = (unsigned)((frow * H_ * W_ + fpiece * 8) * 2);
    // Staging area of a step, shared by the workgroup: 4 KG fragments of dy (its KG channel groups; 1 KB each, lane i of
    // the fetch at byte 16 i) and, for each of its CTW channel tiles and each tap row, the 32 columns of the chunk of that
    // input row (1 KB, same order) plus the 4 columns after and the 2 before (16 B per channel: dwords right0, right1,
    // left, unused), from which the fragments of all tap columns are cut.
    // Four areas when they fit (the loads of a step are then requested three steps ahead: memory latency under load is
    // longer than a step), else three, two, one.  A unit, what lies between two hand-over barriers, is one chunk.
    constexpr int NA = 4 * KG, NB = CTW * R_;
#ifndef WG_UNIT2
#define WG_UNIT2 1
#endif
    // WHOLE_ROW: a unit holds every chunk of its row (rows of at most 32 / 64 outputs).  What lies left of its first and
    // right of its last chunk is outside the image and cleared by the edge masks whatever is read there, and the columns
    // between two chunks of the unit are in the neighbouring chunk's piece: no edge dwords are loaded at all.
    constexpr bool WHOLE_ROW = NCHUNK <= 2 && (NCHUNK == 1 || (NCHUNK == 2 && WG_UNIT2 && 3 * 2 * (NA * 1024 + NB * 1024) <= 150 * 1024)) &&
                               NCHUNK * 32 >= W_;
    constexpr int AREA_B = NA * 1024, AREA_X = AREA_B + NB * 1024, AREA = AREA_X + (WHOLE_ROW ? 0 : NB * 256);
    // two chunks per unit (half the barriers, and the MFMAs of a unit then last as long as its loads and reads) when three
    // such units fit and a row splits into pairs of chunks; their fragments are all in registers at once
    constexpr int UNIT = WG_UNIT2 && NCHUNK % 2 == 0 && 3 * 2 * AREA <= 150 * 1024 ? 2 : 1;
    constexpr int UAREA = UNIT * AREA;
    constexpr int NBUF = 4 * UAREA <= 150 * 1024 ? 4 : 3 * UAREA <= 150 * 1024 ? 3 : 2 * UAREA <= 150 * 1024 ? 2 : 1;
    // With three or more areas the two waves of a SIMD (wave w and w + 4) work in opposite phases: while one reads the
    // fragments of a unit from LDS, the other runs the MFMAs of the unit before.  With every wave in the same phase a
    // step was the sum of the two: all eight waves read (about 100 KB per chunk, LDS-bound), then all eight multiply.
    constexpr bool SPLIT = NBUF >= 3;
    __shared__ __attribute__((aligned(16))) unsigned char stage[NBUF * UAREA];
    typedef __attribute__((address_space(3))) void* mjt_lds_ptr;
    // fragment order: lane (l16, lg) wants row l16, piece lg
    const int rd = (l16 * 4 + lg) * 16;
    const unsigned stage_base = (unsigned)(unsigned long long)(__attribute__((address_space(3))) unsigned char*)&stage[0];

    mjt_f32x4 acc[4][TAPS];
#pragma unroll
    for (int m = 0; m < 4; m++)
#pragma unroll
        for (int t = 0; t < TAPS; t++) acc[m][t] = (mjt_f32x4)(0.0f);

    // The loads of one step, dealt to the waves (item it to wave it % 8): NA fragments of dy, NB row chunks of x, NB
    // sets of edge dwords.  Bit 31 set in an offset puts it beyond every buffer (the tensors are smaller than 2 GB): the
    // load delivers zeros.
    // edge dwords: lane i fetches for channel i / 4 one of the two dwords right of the chunk (i % 4 = 0, 1) or the dword
    // left of it (i % 4 = 2); 16 B per channel: right0, right1, left, unused
    const unsigned e_lane = (unsigned)(frow * H_ * W_ * 2) + (fpiece == 2 ? (unsigned)-4 : (unsigned)(64 + 4 * fpiece));
    // Which loads a wave issues is fixed: fragment q * 8 + wave of dy, row chunk q * 8 + wave of x, edge set
    // q * 8 + (wave + 6) % 8; what depends on that alone is worked out here, so that a unit's loads are a few scalar
    // additions and one branch per slot (with the items dealt round-robin over one combined list the loads of a unit were
    // 200 instructions with 30 branches, a fifth of the kernel's time).
    constexpr int QA = (NA + 7) / 8, QB = (NB + 7) / 8;
    // the fewest loads any wave issues per unit: the wait for a unit's loads names that many per unit still under way
    // (a wave that issues more waits for a few loads of a later unit as well)
    constexpr auto min_per_unit = []() {
        int best = 1 << 30;
        for (int w = 0; w < 8; w++) {
            int n = 0;
            for (int q = 0; q < (NA + 7) / 8; q++) n += q * 8 + w < NA ? 1 : 0;
            for (int q = 0; q < (NB + 7) / 8; q++) n += (q * 8 + w < NB ? 1 : 0) + (q * 8 + ((w + 6) & 7) < NB ? 1 : 0);
            best = n < best ? n : best;
        }
        return best;
    };
    constexpr int MINPER = min_per_unit();
    // loads of the later units that may still be under way when a unit's own have to have landed
    constexpr int LOADS_AHEAD = UNIT * MINPER * (NBUF - 2) < 63 ? (NBUF >= 2 ? UNIT * MINPER * (NBUF - 2) : 0) : 63;
    bool a_on[QA], b_on[QB], e_on[QB], b_cok[QB], e_cok[QB];
    unsigned a_off[QA], b_off[QB], e_off[QB];                            // byte offset inside the image's dy / x
    int a_dst[QA], b_dst[QB], e_dst[QB], b_dih[QB], e_dih[QB];
#pragma unroll
    for (int q = 0; q < QA; q++) {
        const int it = q * 8 + wave;
        a_on[q] = it < NA;
        a_off[q] = (unsigned)(((kblock * KG + it / 4) * 64 + (it & 3) * 16) * (OH_ * OW_ * 2));
        a_dst[q] = it * 1024;
    }
#pragma unroll
    for (int q = 0; q < QB; q++) {
        const int j = q * 8 + wave, je = q * 8 + ((wave + 6) & 7);
        const int tile = j / R_, r = j - tile * R_, tile_e = je / R_, r_e = je - tile_e * R_;
        const int cc = (cblock * CTW + tile) * 16, cc_e = (cblock * CTW + tile_e) * 16;
        b_on[q] = j < NB;
        e_on[q] = je < NB && !WHOLE_ROW;
        b_cok[q] = cc < C_;
        e_cok[q] = cc_e < C_;
        b_dih[q] = r * DH;
        e_dih[q] = r_e * DH;
        b_off[q] = (unsigned)((cc * H_ + r * DH) * (W_ * 2));
        e_off[q] = (unsigned)((cc_e * H_ + r_e * DH) * (W_ * 2));
        b_dst[q] = AREA_B + j * 1024;
        e_dst[q] = AREA_X + je * 256;
    }
    int per_unit = 0;                                                    // loads this wave issues per unit
#pragma unroll
    for (int q = 0; q < QA; q++) per_unit += a_on[q] ? 1 : 0;
#pragma unroll
    for (int q = 0; q < QB; q++) per_unit += (b_on[q] ? 1 : 0) + (e_on[q] ? 1 : 0);
    auto fetch = [&](unsigned char* area, int img, int oh, int ch) -> int {
        if (ABL & 16) return 0;
        const bool img_ok = img * OH_ + oh < row_end;
        const int ih0 = oh * SH - PH;
        // of the unit: (image, row 0 of the taps, chunk) inside dy and x, bytes (unsigned arithmetic: a row above the image
        // wraps and is never used)
        const unsigned dy_unit = ((unsigned)img * (unsigned)(K_ * OH_ * OW_) + (unsigned)(oh * OW_ + ch * 32)) * 2u;
        const unsigned x_unit = ((unsigned)img * (unsigned)(C_ * H_ * W_) + (unsigned)(ih0 * W_ + ch * 32)) * 2u;
        const unsigned a_flag = (img_ok && !(ABL & 1) ? 0u : INVALID) | (ch * 32 + fpiece * 8 < OW_ ? 0u : INVALID);
        mjt_static_for<0, QA>([&](auto qc) {
            constexpr int q = decltype(qc)::v;
            if (a_on[q])
                __builtin_amdgcn_raw_ptr_buffer_load_lds(y_rsrc, (mjt_lds_ptr)(area + a_dst[q]), 16, (int)((a_lane + dy_unit + a_off[q]) | a_flag), 0, 0, 0);
        });
        mjt_static_for<0, QB>([&](auto qc) {
            constexpr int q = decltype(qc)::v;
            if (b_on[q]) {
                const int ih = ih0 + b_dih[q];
                const bool ok = img_ok && ih >= 0 && ih < H_ && b_cok[q] && !(ABL & 2);
                __builtin_amdgcn_raw_ptr_buffer_load_lds(x_rsrc, (mjt_lds_ptr)(area + b_dst[q]), 16,
                                                         (int)((b_lane + x_unit + b_off[q]) | (ok ? 0u : INVALID)), 0, 0, 0);
            }
            if (e_on[q]) {
                const int ih = ih0 + e_dih[q];
                const bool ok = img_ok && ih >= 0 && ih < H_ && e_cok[q] && !(ABL & 2);
                // at the very start of the tensor the left dword lies in front of it: its offset wraps, out of range, zeros
                const unsigned flag = (ok ? 0u : INVALID) | (fpiece == 3 ? INVALID : 0u);
                __builtin_amdgcn_raw_ptr_buffer_load_lds(x_rsrc, (mjt_lds_ptr)(area + e_dst[q]), 4, (int)((e_lane + x_unit + e_off[q]) | flag), 0, 0, 0);
            }
        });
        return per_unit;
    };
    // wait until at most n of this wave's loads are outstanding (they complete in order)
    auto wait_loads = [&](int n) {
        switch (n) {
        case 1: asm volatile("s_waitcnt vmcnt(1)" ::: "memory"); break;
        case 2: asm volatile("s_waitcnt vmcnt(2)" ::: "memory"); break;
        case 3: asm volatile("s_waitcnt vmcnt(3)" ::: "memory"); break;
        case 4: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
        case 5: asm volatile("s_waitcnt vmcnt(5)" ::: "memory"); break;
        case 6: asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); break;
        case 7: asm volatile("s_waitcnt vmcnt(7)" ::: "memory"); break;
        case 8: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
        case 9: asm volatile("s_waitcnt vmcnt(9)" ::: "memory"); break;
        case 10: asm volatile("s_waitcnt vmcnt(10)" ::: "memory"); break;
        case 11: asm volatile("s_waitcnt vmcnt(11)" ::: "memory"); break;
        case 12: asm volatile("s_waitcnt vmcnt(12)" ::: "memory"); break;
        case 13: asm volatile("s_waitcnt vmcnt(13)" ::: "memory"); break;
        case 14: asm volatile("s_waitcnt vmcnt(14)" ::: "memory"); break;
        default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
        }
    };

    // the loads of a unit: its chunks ch0 .. ch0 + UNIT - 1 of row (img, oh), one area each
    auto fetch_unit = [&](unsigned char* uarea, int img, int oh, int ch0) -> int {
        int issued = 0;
#pragma unroll
        for (int u = 0; u < UNIT; u++) issued += fetch(uarea + u * AREA, img, oh, ch0 + u);
        return issued;
    };
    // The fragments of a chunk: per tap row the lane's columns 8 lg .. 8 lg + 7, the two columns before them and the four
    // after them; four fragments of dy.  (Zero at first: the second wave group multiplies what it read a unit earlier.)
    mjt_u32x4v afrag[UNIT][4], bd[UNIT][R_];
    unsigned bp[UNIT][R_];
    mjt_u32x2 bn[UNIT][R_];
#pragma unroll
    for (int u = 0; u < UNIT; u++) {
#pragma unroll
        for (int m = 0; m < 4; m++) afrag[u][m] = (mjt_u32x4v)(0u);
#pragma unroll
        for (int r = 0; r < R_; r++) { bd[u][r] = (mjt_u32x4v)(0u); bp[u][r] = 0u; bn[u][r] = (mjt_u32x2)(0u); }
    }
    int cur = 0, newest = 0;                                             // newest: loads of this wave's latest request
    // All reads of a chunk are issued at once, in the order of their use, and spelled out (the compiler sees no latency in
    // an LDS read and would otherwise issue them one by one between the MFMAs, each with a full wait).  LDS addresses
    // (bytes): the fragments of dy, the lane's piece of each tap row of x, and its neighbours: the previous / next piece
    // of the row, or the edge dwords (pieces of the rows of a tile are 1 KB apart per tap row, their edge dwords 256 B).
    auto read_frags = [&](auto uc) {
        constexpr int U = decltype(uc)::v;                               // chunk of the unit
        if (ABL & 8) return;
        const unsigned area_at = stage_base + (unsigned)(cur * UAREA + U * AREA);
        const unsigned my_a = area_at + (unsigned)(kg * 4096 + rd);
        const unsigned my_b = area_at + (unsigned)(AREA_B + ct * (R_ * 1024) + rd);
        unsigned prev0, next0, prev_step, next_step;
        if constexpr (WHOLE_ROW) {
            // the last dword of the piece before / the first two of the piece after: in this chunk, or (for the first and
            // the last lane group) in the same row of the chunk before / after; at the ends of the row anything (masked)
            prev0 = lg > 0 ? my_b - 4 : U > 0 ? my_b - AREA + 3 * 16 + 12 : my_b;
            next0 = lg < 3 ? my_b + 16 : U + 1 < UNIT ? my_b + AREA - 3 * 16 : my_b;
            prev_step = next_step = 1024;
        } else {
            const unsigned my_x = area_at + (unsigned)(AREA_X + ct * (R_ * 256) + l16 * 16);
            prev0 = lg > 0 ? my_b - 4 : my_x + 8;
            next0 = lg < 3 ? my_b + 16 : my_x;
            prev_step = lg > 0 ? 1024 : 256;
            next_step = lg < 3 ? 1024 : 256;
        }
        mjt_static_for<0, 4>([&](auto mc) { mjt_ds_read128<decltype(mc)::v * 1024>(afrag[U][decltype(mc)::v], my_a); });
        mjt_static_for<0, R_>([&](auto rc) {
            constexpr int r = decltype(rc)::v;
            mjt_ds_read128<r * 1024>(bd[U][r], my_b);
            mjt_ds_read32(bp[U][r], prev0 + r * prev_step);
            mjt_ds_read64(bn[U][r], next0 + r * next_step);
        });
    };
    const int grp = wave >> 2;                                           // waves w and w + 4 share a SIMD
    // The MFMAs of chunk CH on the fragments in registers.  LDS operations of a wave complete in order: the wait in front
    // of a tap row names the reads of the later rows (the waits also tie the MFMAs to a place behind the reads).
    auto mfmas = [&](auto ch_c, auto uc) {
        constexpr int CH = decltype(ch_c)::v, U = decltype(uc)::v;
        constexpr int AFTER = (UNIT - 1 - U) * (4 + 3 * R_);             // reads of the unit's later chunks
        mjt_static_for<0, TAPS>([&](auto tc) {
            constexpr int t = decltype(tc)::v;
            constexpr int r = t / S_, s = t % S_;
            constexpr int off = mjt_col_shift(s);                        // -2 .. 4: the host admits nothing else
            if constexpr (s == 0) {                                      // the reads of this tap row (and, in front of them, of dy) have arrived
                constexpr int later = 3 * (R_ - 1 - r) + AFTER;
                if constexpr (r == 0) mjt_static_for<0, 4>([&](auto mc) { mjt_lds_wait<later + 3>(afrag[U][decltype(mc)::v]); });
                if constexpr (r == 0 && DY_TAIL && CH == NCHUNK - 1) mjt_static_for<0, 4>([&](auto mc) { afrag[U][decltype(mc)::v] &= dy_mask; });
                mjt_lds_wait<later + 2>(bd[U][r]);
                mjt_lds_wait1<later + 1>(bp[U][r]);
                mjt_lds_wait2<later>(bn[U][r]);
            }
            // the seven dwords around the lane's columns: elements 8 lg - 2 .. 8 lg + 11
            const unsigned w[7] = {bp[U][r], bd[U][r][0], bd[U][r][1], bd[U][r][2], bd[U][r][3], bn[U][r][0], bn[U][r][1]};
            constexpr int first = (off + 2) >> 1;                        // dword of element 8 lg + off
            mjt_u32x4v v;
            if constexpr (off & 1) {
#pragma unroll
                for (int j = 0; j < 4; j++) v[j] = __builtin_amdgcn_alignbit(w[first + j + 1], w[first + j], 16);
            } else {
#pragma unroll
                for (int j = 0; j < 4; j++) v[j] = w[first + j];
            }
            if constexpr (mjt_edge(CH, s)) v &= masks[CH * S_ + s];
#pragma unroll
            for (int m = 0; m < 4; m++) {
#if ABL & 4
                mjt_no_mfma(acc[m][t], afrag[U][m], v);
#else
                acc[m][t] = MJT_MFMA(__builtin_bit_cast(mjt_bf16x8, afrag[U][m]), __builtin_bit_cast(mjt_bf16x8, v), acc[m][t], 0, 0, 0);
#endif
            }
        });
    };
    // the MFMAs issued so far stay in front of this point
    auto pin_acc = [&]() {
        mjt_static_for<0, 4 * TAPS>([&](auto ic) { mjt_pin_acc(acc[decltype(ic)::v / TAPS][decltype(ic)::v % TAPS]); });
    };
    // One unit (chunk CH): its data is in area `cur` once every wave's loads have
    // arrived; the loads of the unit NBUF - 1 ahead (nimg, noh, nch) go into the area that was read last (with a single
    // area: into the same, after everybody has read it).
    auto unit = [&](auto ch_c, const int nimg, const int noh, const int nch) {
        if constexpr (SPLIT) {
            // Every wave runs: barrier P, loads of the unit NBUF - 1 ahead, LDS reads of this unit, barrier Q, MFMAs.  The
            // second group enters one barrier late (and the first leaves one barrier late), so one group's P meets the
            // other's Q: while a wave reads, the other wave of its SIMD multiplies.  A wave waits for its loads of the
            // *next* unit before Q: whichever barrier the other group is at when it passes, those loads have landed
            // before anybody reads them, and everybody has read the area of the unit before this one when a wave passes P.
            asm volatile("s_barrier" ::: "memory");
            newest = fetch_unit(stage + (cur == 0 ? NBUF - 1 : cur - 1) * UAREA, nimg, noh, nch);
            mjt_static_for<0, UNIT>([&](auto uc) { read_frags(uc); });
            asm volatile("s_waitcnt lgkmcnt(0)\n\ts_waitcnt vmcnt(%0)\n\ts_barrier" : : "n"(LOADS_AHEAD) : "memory");
            mjt_static_for<0, UNIT>([&](auto uc) { mfmas(mjt_ic<decltype(ch_c)::v + decltype(uc)::v>(), uc); });
            pin_acc();
        } else {
            wait_loads(0);                                               // this wave's loads for this unit have arrived
            __syncthreads();                                             // ... everybody's; and the area read last is free
            if constexpr (NBUF >= 2) newest = fetch_unit(stage + (cur == 0 ? NBUF - 1 : cur - 1) * UAREA, nimg, noh, nch);
            read_frags(mjt_ic<0>());
            if constexpr (NBUF == 1) {
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");       // read by this wave
                __syncthreads();                                         // ... by everybody: the area may be refilled
                fetch(stage, nimg, noh, nch);
            }
            mfmas(ch_c, mjt_ic<0>());
        }
        if constexpr (NBUF >= 2) cur = cur + 1 == NBUF ? 0 : cur + 1;
    };

    // units in order: images of the slice, rows, chunks; (img, oh, ch) advanced by `ahead` units
    constexpr int AHEAD = NBUF == 1 ? 1 : NBUF - 1;
    auto advance = [&](int& img, int& oh, int& ch, int ahead) {
        ch += ahead * UNIT;
        while (ch >= NCHUNK) {
            ch -= NCHUNK;
            if (++oh >= OH_) { oh = 0; img++; }
        }
    };
    mjt_static_for<0, AHEAD>([&](auto ac) {
        int i1 = img_begin, o1 = oh_begin, c1 = 0;
        advance(i1, o1, c1, decltype(ac)::v);
        newest = fetch_unit(stage + decltype(ac)::v * UAREA, i1, o1, c1);
    });
    if constexpr (SPLIT) {
        // this wave's loads of the first unit have landed; the second group runs half a unit behind
        asm volatile("s_waitcnt vmcnt(%0)" : : "n"(LOADS_AHEAD) : "memory");
        if (grp == 1) asm volatile("s_barrier" ::: "memory");
    }
    {
        int img = img_begin, oh = oh_begin;
#pragma unroll 1
        for (int row = row_begin; row < row_end; row++) {
            mjt_static_for<0, NCHUNK / UNIT>([&](auto cc) {
                constexpr int ch0 = decltype(cc)::v * UNIT;
                int ni = img, no = oh, nc = ch0;
                advance(ni, no, nc, AHEAD);                              // beyond the slice: read as zeros
                unit(mjt_ic<ch0>(), ni, no, nc);
            });
            if (++oh >= OH_) { oh = 0; img++; }
        }
    }
    if constexpr (SPLIT)
        if (grp == 0) asm volatile("s_barrier" ::: "memory");            // the second group's last barrier
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                     // nothing may arrive in LDS after the wave has ended

    // lane holds D[k = 4*lg + i][c = l16] of each (channel tile m, tap): the taps of one (k, c) are neighbours in
    // partial[slice][k][c][tap], and the 16 lanes of a row hold 16 neighbouring c, so a row writes one contiguous run of
    // 16 * TAPS floats, each lane its TAPS of them (with one store per element the stores were a fifth of the kernel)
    typedef float mjt_f4u __attribute__((ext_vector_type(4), aligned(4)));
    typedef float mjt_f2u __attribute__((ext_vector_type(2), aligned(4)));
    const size_t KC = (size_t)K_ * C_;
    if (c0 >= C_ || (ABL & 32)) return;
#pragma unroll
    for (int m = 0; m < 4; m++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const size_t k = (size_t)(k0 + m * 16 + lg * 4 + i);
            float* const dst = partial + ((size_t)slice * KC + k * C_ + (size_t)(c0 + l16)) * TAPS;
            mjt_static_for<0, TAPS / 4>([&](auto qc) {
                constexpr int t0 = decltype(qc)::v * 4;
                mjt_f4u v;
                v[0] = acc[m][t0][i]; v[1] = acc[m][t0 + 1][i]; v[2] = acc[m][t0 + 2][i]; v[3] = acc[m][t0 + 3][i];
                *(mjt_f4u*)(dst + t0) = v;
            });
            constexpr int T4 = TAPS / 4 * 4;
            if constexpr (TAPS - T4 >= 2) {
                mjt_f2u v;
                v[0] = acc[m][T4][i]; v[1] = acc[m][T4 + 1][i];
                *(mjt_f2u*)(dst + T4) = v;
            }
            if constexpr ((TAPS - T4) & 1) dst[TAPS - 1] = acc[m][TAPS - 1][i];
        }
}
