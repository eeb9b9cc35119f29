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
    // Three areas when they fit (the loads of a step are then requested two steps ahead: memory latency under
    // load is longer than one step), else two, else one.
    constexpr int NA = 4 * KG, NB = CTW * R_;
    constexpr int AREA_B = NA * 1024, AREA_X = AREA_B + NB * 1024, AREA = AREA_X + NB * 256;
    // A unit is what lies between two barriers: a whole row of chunks when three units of that size fit, else a chunk.
    constexpr int UNIT = NCHUNK <= 2 && 3 * NCHUNK * AREA <= 150 * 1024 ? NCHUNK : 1;
    constexpr int UAREA = UNIT * AREA;
    constexpr int NBUF = 3 * UAREA <= 150 * 1024 ? 3 : 2 * UAREA <= 150 * 1024 ? 2 : 1;
    __shared__ __attribute__((aligned(16))) unsigned char stage[NBUF * UAREA];
    typedef __attribute__((address_space(3))) void* mjt_lds_ptr;
    // fragment order: lane (l16, lg) wants row l16, piece lg
    const int rd = (l16 * 4 + lg) * 16;

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
    auto fetch = [&](unsigned char* area, int img, int oh, int ch) -> int {
        int issued = 0;                                                  // by this wave
        const bool img_ok = img * OH_ + oh < row_end;
#pragma unroll
        for (int it0 = 0; it0 < NA + 2 * NB; it0 += 8) {
            const int it = it0 + wave;
            if (it < NA) {
                const int kk = (kblock * KG + it / 4) * 64 + (it & 3) * 16;
                const unsigned base = img_ok ? (unsigned)((((img * K_ + kk) * OH_ + oh) * OW_ + ch * 32) * 2) : 0u;
                const unsigned flag = (img_ok ? 0u : INVALID) | (ch * 32 + fpiece * 8 < OW_ ? 0u : INVALID);
                __builtin_amdgcn_raw_ptr_buffer_load_lds(y_rsrc, (mjt_lds_ptr)(area + it * 1024), 16, (int)((a_lane + base) | flag), 0, 0, 0);
                issued++;
            } else if (it < NA + 2 * NB) {
                const bool edge = it >= NA + NB;
                const int j = it - NA - (edge ? NB : 0);
                const int tile = j / R_, r = j - tile * R_;
                const int ih = oh * SH - PH + r * DH;
                const int cc = (cblock * CTW + tile) * 16;
                const bool ok = img_ok && ih >= 0 && ih < H_ && cc < C_;
                const unsigned base = ok ? (unsigned)((((img * C_ + cc) * H_ + ih) * W_ + ch * 32) * 2) : 0u;
                if (!edge) {
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(x_rsrc, (mjt_lds_ptr)(area + AREA_B + j * 1024), 16,
                                                             (int)((b_lane + base) | (ok ? 0u : INVALID)), 0, 0, 0);
                } else {
                    // at the very start of the tensor the left dword lies in front of it: its offset wraps, out of range, zeros
                    const unsigned flag = (ok ? 0u : INVALID) | (fpiece == 3 ? INVALID : 0u);
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(x_rsrc, (mjt_lds_ptr)(area + AREA_X + j * 256), 4, (int)((e_lane + base) | flag), 0, 0, 0);
                }
                issued++;
            }
        }
        return issued;
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
    // One unit: its fragments are in unit area `cur` once every wave's loads have arrived; request those of the unit
    // NBUF - 1 ahead (nimg, noh, nch) into the area that was read last (with a single area: into the same, after
    // everybody has read it), run the MFMAs chunk by chunk.
    int cur = 0, newest = 0;                                             // newest: loads of this wave's latest request
    auto unit = [&](auto ch_c, const int nimg, const int noh, const int nch) {
        constexpr int CH0 = decltype(ch_c)::v;
        unsigned char* const uarea = stage + cur * UAREA;
        wait_loads(NBUF == 3 ? newest : 0);                              // this wave's loads for this unit have arrived
        __syncthreads();                                                 // ... everybody's; and the area read last is free
        if constexpr (NBUF >= 2) newest = fetch_unit(stage + (cur == 0 ? NBUF - 1 : cur - 1) * UAREA, nimg, noh, nch);
        mjt_static_for<0, UNIT>([&](auto uc) {
        constexpr int CH = CH0 + decltype(uc)::v;
        unsigned char* const area = uarea + decltype(uc)::v * AREA;
        mjt_u32x4v afrag[4], bd[R_];                                     // per tap row: columns 8 lg .. 8 lg + 7 of the chunk
        unsigned bp[R_];                                                 // ... the two columns before them
        unsigned long long bn[R_];                                       // ... the four after them
        const unsigned char* const my_a = area + kg * 4096 + rd;
        const unsigned char* const my_b = area + AREA_B + ct * (R_ * 1024);
        const unsigned char* const my_x = area + AREA_X + ct * (R_ * 256);
        // a lane's neighbours are in the previous / next piece of the row, or among the edge dwords (pieces of the rows of
        // a tile are 1 KB apart per tap row, their edge dwords 256 B)
        const unsigned char* const prev0 = lg > 0 ? my_b + rd - 4 : my_x + l16 * 16 + 8;
        const unsigned char* const next0 = lg < 3 ? my_b + rd + 16 : my_x + l16 * 16;
        const int prev_step = lg > 0 ? 1024 : 256, next_step = lg < 3 ? 1024 : 256;
#pragma unroll
        for (int m = 0; m < 4; m++) afrag[m] = *(const mjt_u32x4v*)(my_a + m * 1024);
        mjt_static_for<0, R_>([&](auto rc) {
            constexpr int r = decltype(rc)::v;
            bd[r] = *(const mjt_u32x4v*)(my_b + r * 1024 + rd);
            bp[r] = *(const unsigned*)(prev0 + r * prev_step);
            bn[r] = *(const unsigned long long*)(next0 + r * next_step);
        });
        if constexpr (NBUF == 1) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");           // read by this wave
            __syncthreads();                                             // ... by everybody: the area may be refilled
            fetch(area, nimg, noh, nch);
        }
        mjt_static_for<0, TAPS>([&](auto tc) {
            constexpr int t = decltype(tc)::v;
            constexpr int r = t / S_, s = t % S_;
            constexpr int off = mjt_col_shift(s);                        // -2 .. 4: the host admits nothing else
            // the seven dwords around the lane's columns: elements 8 lg - 2 .. 8 lg + 11
            const unsigned w[7] = {bp[r], bd[r][0], bd[r][1], bd[r][2], bd[r][3], (unsigned)bn[r], (unsigned)(bn[r] >> 32)};
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
            const mjt_bf16x8 b = __builtin_bit_cast(mjt_bf16x8, v);
#pragma unroll
            for (int m = 0; m < 4; m++)
                acc[m][t] = MJT_MFMA(__builtin_bit_cast(mjt_bf16x8, afrag[m]), b, acc[m][t], 0, 0, 0);
        });
        });
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
    fetch_unit(stage, img_begin, oh_begin, 0);
    if constexpr (NBUF == 3) {
        int i1 = img_begin, o1 = oh_begin, c1 = 0;
        advance(i1, o1, c1, 1);
        newest = fetch_unit(stage + UAREA, i1, o1, c1);
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
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                     // nothing may arrive in LDS after the wave has ended

    // lane holds D[k = 4*lg + i][c = l16] of each (channel tile m, tap)
    const size_t KC = (size_t)K_ * C_;
    if (c0 >= C_) return;
#pragma unroll
    for (int m = 0; m < 4; m++)
#pragma unroll
        for (int t = 0; t < TAPS; t++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const size_t k = (size_t)(k0 + m * 16 + lg * 4 + i);
                partial[((size_t)slice * KC + k * C_ + (size_t)(c0 + l16)) * TAPS + t] = acc[m][t][i];
            }
}
