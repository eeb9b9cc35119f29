// Weight gradient of the meta-op convolution on MFMA: the group
//   reduce.add over (n, oh, ow) of  reindex(x) * broadcast(dy)
// that jt.grad builds for the weights (python/jittor/nn.py:1251-1262 differentiated by
// ops/reduce_op.cc:339-362, ops/broadcast_to_op.cc:112-117; recognised by
// opt/tuner/conv_tuner.cc:375-397 and relayed there to a backward-w library call):
//   dW[k][c][r][s] = sum_{n,oh,ow} dy[n][k][oh][ow] * x[n][c][oh*SH-PH+r*DH][ow-PW+s*DW]
// for bfloat16 operands with exact products and float32 accumulation; taps outside the image
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
// into a wave-private 1 KB slot of LDS (no registers, no barrier), and read back from there in
// fragment order.  A fragment of x whose column shift is odd starts in the middle of a dword: it
// comes as the four dwords above its first element plus the dword below, shifted down by 16 bits
// (every load is dword-aligned).  Columns outside the image (and the columns of a last, partial
// chunk) are cleared with lane masks kept in LDS; rows and images outside read zeros through the
// range check of the buffer loads (the whole offset travels in the lane offset, which is what the
// hardware checks).  While the MFMAs of a step run, the loads of the next step fill the slots the
// step's fragments were just read from.
//
// A workgroup owns 64*KG output channels x 16*8/KG input channels x all taps, over the images
// [slice*ips, slice*ips+ips): the partial sums of the slices go to partial[slice][k][c][r][s]
// (float32) and are added up by a reduce launch.

typedef __bf16 mjt_bf16x8 __attribute__((ext_vector_type(8)));
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

extern "C" __global__ __launch_bounds__(512) void ENTRY(Params p) {
    const int n_img = (int)(unsigned long long)p.a[3];
    const int ips = (int)(unsigned long long)p.a[4];
    float* __restrict__ partial = (float*)p.a[2];
    __shared__ mjt_u32x4v masks[NCHUNK * S_][64];

    constexpr int KBLOCKS = K_ / (64 * KG), CBLOCKS = C_ / (16 * CTW);
    // the workgroups of one slice read the same dy: they are 8 apart, so that they land on the same XCD
    // (workgroups go round-robin over the 8 XCDs) and share it through that XCD's L2
    const int id = blockIdx.x;
    const int xcd = id & 7, j = id >> 3;
    const int kblock = j % KBLOCKS;
    const int cblock = (j / KBLOCKS) % CBLOCKS;
    const int slice = (j / (KBLOCKS * CBLOCKS)) * 8 + xcd;
    if (slice * ips >= n_img) return;                       // the grid is padded to a multiple of 8 slices
    const int img_begin = slice * ips;
    const int img_end = img_begin + ips < n_img ? img_begin + ips : n_img;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kg = wave % KG, ct = wave / KG;
    const int k0 = (kblock * KG + kg) * 64, c0 = (cblock * CTW + ct) * 16;
    const int l16 = lane & 15, lg = lane >> 4;

    // which of a lane's 8 elements lie inside the image, per (chunk, tap column): 16 bits per element pair
    for (int idx = wave; idx < NCHUNK * S_; idx += 8) {
        const int ch = idx / S_, s = idx - ch * S_;
        const int off = s * DW - PW;
        mjt_u32x4v m;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            unsigned v = 0;
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int ow = ch * 32 + lg * 8 + 2 * j + h, iw = ow + off;
                if (ow < OW_ && iw >= 0 && iw < W_) v |= h ? 0xffff0000u : 0x0000ffffu;
            }
            m[j] = v;
        }
        masks[idx][lane] = m;
    }
    __syncthreads();

    // buffer descriptors over the whole tensors; every offset is a lane offset, so the range check sees all of it
    const __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc(p.a[0], 0, n_img * (C_ * H_ * W_ * 2), 0x00020000);
    const __amdgpu_buffer_rsrc_t y_rsrc = __builtin_amdgcn_make_buffer_rsrc(p.a[1], 0, n_img * (K_ * OH_ * OW_ * 2), 0x00020000);
    // fetch order: lane i takes row i / 4 of the fragment (an output or input channel), piece i % 4 (8 columns)
    const int frow = lane >> 2, fpiece = lane & 3;
    const unsigned a_lane = (unsigned)((frow * OH_ * OW_ + fpiece * 8) * 2);
    const unsigned b_lane = (unsigned)((frow * H_ * W_ + fpiece * 8) * 2);
    // a wave's slots: 4 fragments of dy, TAPS of x (1 KB each, lane i at byte 16 i), TAPS dwords-below (256 B each)
    constexpr int SLOT_B = 4 * 1024, SLOT_X = SLOT_B + TAPS * 1024, WAVE_LDS = SLOT_X + TAPS * 256;
    __shared__ __attribute__((aligned(16))) unsigned char stage[8 * WAVE_LDS];
    typedef __attribute__((address_space(3))) void* mjt_lds_ptr;
    unsigned char* const mine = stage + wave * WAVE_LDS;
    // fragment order: lane (l16, lg) wants row l16, piece lg
    const int rd = (l16 * 4 + lg) * 16;

    mjt_f32x4 acc[4][TAPS];
#pragma unroll
    for (int m = 0; m < 4; m++)
#pragma unroll
        for (int t = 0; t < TAPS; t++) acc[m][t] = (mjt_f32x4)(0.0f);

    // bit 31 set in an offset puts it beyond every buffer (the tensors are smaller than 2 GB): the load delivers zeros
    auto fetch = [&](int img, int oh, int ch) {
        {
            const bool ok = img < img_end && oh < OH_;
            const unsigned base = ok ? (unsigned)((((img * K_ + k0) * OH_ + oh) * OW_ + ch * 32) * 2) : 0u;
            const unsigned flag = (ok ? 0u : INVALID) | (ch * 32 + fpiece * 8 < OW_ ? 0u : INVALID);
#pragma unroll
            for (int m = 0; m < 4; m++)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(y_rsrc, (mjt_lds_ptr)(mine + m * 1024), 16,
                                                         (int)((a_lane + base + (unsigned)(m * 16 * OH_ * OW_ * 2)) | flag), 0, 0, 0);
        }
        mjt_static_for<0, R_>([&](auto rc) {
            constexpr int r = decltype(rc)::v;
            const int ih = oh * SH - PH + r * DH;
            const bool ok = img < img_end && oh < OH_ && ih >= 0 && ih < H_;
            const unsigned base = ok ? (unsigned)((((img * C_ + c0) * H_ + ih) * W_ + ch * 32) * 2) : 0u;
            const unsigned flag = ok ? 0u : INVALID;
            mjt_static_for<0, S_>([&](auto sc) {
                constexpr int s = decltype(sc)::v;
                constexpr int off = mjt_col_shift(s);                    // >= -1: the host admits no wider left padding
                constexpr int t = r * S_ + s;
                if constexpr (off & 1) {
                    // elements off+1 .. off+8 as four dwords, and the dword below them (elements off-1, off); at the very
                    // start of the tensor that dword lies in front of it: its offset wraps, out of range, zeros
                    const unsigned o = b_lane + base + (unsigned)((off + 1) * 2);
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(x_rsrc, (mjt_lds_ptr)(mine + SLOT_B + t * 1024), 16, (int)(o | flag), 0, 0, 0);
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(x_rsrc, (mjt_lds_ptr)(mine + SLOT_X + t * 256), 4, (int)((o - 4u) | flag), 0, 0, 0);
                } else {
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(x_rsrc, (mjt_lds_ptr)(mine + SLOT_B + t * 1024), 16,
                                                             (int)((b_lane + base + (unsigned)(off * 2)) | flag), 0, 0, 0);
                }
            });
        });
    };

    // One step: read the fragments of (img, oh, CH) that the loads have put into the slots, request those of the
    // next step into the same slots, and run the MFMAs.
    auto step = [&](auto ch_c, const int nimg, const int noh, const int nch) {
        constexpr int CH = decltype(ch_c)::v;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                 // the slots are filled
        mjt_u32x4v afrag[4], bq[TAPS];
        unsigned bx[TAPS];
#pragma unroll
        for (int m = 0; m < 4; m++) afrag[m] = *(const mjt_u32x4v*)(mine + m * 1024 + rd);
        mjt_static_for<0, TAPS>([&](auto tc) {
            constexpr int t = decltype(tc)::v;
            bq[t] = *(const mjt_u32x4v*)(mine + SLOT_B + t * 1024 + rd);
            if constexpr (mjt_col_shift(t % S_) & 1) bx[t] = *(const unsigned*)(mine + SLOT_X + t * 256 + (rd >> 2));
        });
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");               // ... and read: they may be overwritten
        fetch(nimg, noh, nch);
        mjt_static_for<0, TAPS>([&](auto tc) {
            constexpr int t = decltype(tc)::v;
            constexpr int s = t % S_;
            mjt_u32x4v v = bq[t];
            if constexpr (mjt_col_shift(s) & 1) {                        // (below, d0, d1, d2, d3) shifted down by one element
                const mjt_u32x4v d = v;
                v[0] = __builtin_amdgcn_alignbit(d[0], bx[t], 16);
                v[1] = __builtin_amdgcn_alignbit(d[1], d[0], 16);
                v[2] = __builtin_amdgcn_alignbit(d[2], d[1], 16);
                v[3] = __builtin_amdgcn_alignbit(d[3], d[2], 16);
            }
            v &= masks[CH * S_ + s][lane];
            const mjt_bf16x8 b = __builtin_bit_cast(mjt_bf16x8, v);
#pragma unroll
            for (int m = 0; m < 4; m++)
                acc[m][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(mjt_bf16x8, afrag[m]), b, acc[m][t], 0, 0, 0);
        });
    };

    // steps in order: images of the slice, rows, chunks
    fetch(img_begin, 0, 0);
    for (int img = img_begin; img < img_end; img++) {
#pragma unroll 1
        for (int oh = 0; oh < OH_; oh++) {
            const bool wrap = oh + 1 >= OH_;
            const int after_img = wrap ? img + 1 : img, after_oh = wrap ? 0 : oh + 1;
            mjt_static_for<0, NCHUNK>([&](auto cc) {
                constexpr int ch = decltype(cc)::v;
                constexpr bool last = ch + 1 == NCHUNK;
                step(cc, last ? after_img : img, last ? after_oh : oh, last ? 0 : ch + 1);
            });
        }
    }

    // lane holds D[k = 4*lg + i][c = l16] of each (channel tile m, tap)
    const size_t KC = (size_t)K_ * C_;
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
