// Matrix product on MFMA:  C[b][M][N] = sum_k A'[b][M][K] * B'[b][K][N]
// (reference: the broadcast * broadcast -> reduce.add pattern that
// python/jittor/src/opt/tuner/matmul_tuner.cc:16-104 relays to a library GEMM,
// python/jittor/extern/cuda/cublas/ops/cublas_matmul_op.cc:27-126; batched form
// cublas_batched_matmul_op.cc:63-85).  Row-major operands; A' is a, or a
// transposed when A_KCONT == 0 (memory [K][M]); B' is b, or b transposed when
// B_KCONT == 1 (memory [N][K]).  bfloat16 / float16 operands with exact products
// and float32 accumulation, or float32 throughout.
//
// Supplied by the host: IN (0 bfloat16, 1 float16, 2 float32), OUT (0 bfloat16 by
// truncation, 1 float16 rounded to nearest even, 2 float32), MI, NI (32x32 accumulator
// tiles per wave along m and n), A_KCONT, B_KCONT (the operand's memory has k innermost).
//
// Mapping.  A workgroup of four waves (2 x 2) owns a TM x TN = 64 MI x 64 NI tile of C and
// walks K in stages of KS elements (eight 16-byte chunks per row: 64 for 16-bit operands,
// 32 for float32).  Both operand tiles of a stage sit in LDS with k innermost,
// [row][8 chunks + one chunk of padding] (144 bytes per row: 16-byte fragment reads of
// 16 neighbouring rows then do not meet in a bank), which is the order an MFMA operand
// wants: lane (row = lane % 32, half = lane / 32) of v_mfma_f32_32x32x16 reads the 8
// consecutive k of its row and half with one ds_read_b128.  An operand whose memory has k
// innermost is copied as it is (a lane moves 16 bytes; 8 lanes read one 128-byte line).
// The other kind (m or n innermost) is transposed on the way in registers: 8 lanes load
// 16 bytes of 8 consecutive k rows, exchange among themselves with three butterfly steps
// (4 lanes and two steps for float32) until each owns one column for the 8 (4) k, and
// write 16 bytes.  The loads of the next stage are in flight during the MFMAs of the
// current one and are written to the other LDS buffer after them: one barrier per stage.
// float32 uses v_mfma_f32_32x32x2: a lane's 16-byte read holds 4 k of its row, which feed
// four MFMAs (lanes 32..63 read the next chunk, so that an MFMA sums k and k + 4 of a
// chunk pair; any pairing is right as long as both operands use the same one).
//
// CONV = 1 makes the kernel an implicit-GEMM convolution, the meta-op group of
// python/jittor/nn.py:1251-1262 that opt/tuner/conv_tuner.cc:233-240,365-373 relays for every float type:
// A = the weights [K_][C_*R_*S_] (rows padded to 16 bytes by the host), B'[k = (c, r, s)][j = (image, oh, ow)] =
// x[image][c][oh*SH-PH+r*DH][ow*SW-PW+s*DW] (0 outside the image) is never written to memory -- the B tile of a
// stage is gathered from x element by element on its way to LDS (a float32 MFMA runs at a sixteenth of the 16-bit
// rate, so the gather's address arithmetic hides behind it; with 16-bit operands the gather is what bounds the
// kernel, which then serves the shapes the MFMA convolution kernel does not take) -- and C[k][j] is stored as
// y[image][k][oh][ow].
// Geometry comes as C_, H_, W_, K_, R_, S_, OH_, OW_, SH, SW, PH, PW, DH, DW; N = images * OH_ * OW_.
//
// Rows of A' and columns of B' beyond M and N are read from the last valid row (their
// results are not stored); k beyond K is zeroed in both operands.  Leading dimensions are
// multiples of 16 bytes and the operand pointers 16-byte aligned (the host sends
// everything else to the plain kernel below).

#if IN == 2
typedef float TIN;
#define EPC 4                    // elements per 16-byte chunk
#else
typedef unsigned short TIN;
#define EPC 8
#endif
#define KC 8                     // chunks per row and stage
#define KS (KC * EPC)            // k per stage
#define TM (64 * MI)
#define TN (64 * NI)
#define ROWB 144                 // bytes per LDS row: 8 chunks + 1 of padding
#define NTHR 256
#ifndef CONV
#define CONV 0
#endif
#ifndef NBUF
#define NBUF 2                   // staging buffers: 2, or 1 for a product of a single stage (K <= KS)
#endif

typedef float mjt_f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned mjt_u32x4v __attribute__((ext_vector_type(4)));
#if IN == 0
typedef __bf16 mjt_h8 __attribute__((ext_vector_type(8)));
#define MJT_MFMA16(a, b, c) __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0)
#elif IN == 1
typedef _Float16 mjt_h8 __attribute__((ext_vector_type(8)));
#define MJT_MFMA16(a, b, c) __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0)
#endif

template <int V> struct mjt_ic { static constexpr int v = V; };
struct Params { void* a[12]; };
// a[0] A  a[1] B  a[2] C  a[3] M  a[4] N  a[5] K  a[6] lda  a[7] ldb  a[8] ldc (elements)
// a[9] batch stride of A  a[10] of B  a[11] of C (elements)

__device__ __forceinline__ unsigned mjt_dpp_xor1(unsigned v) { return (unsigned)__builtin_amdgcn_mov_dpp((int)v, 0xB1, 0xf, 0xf, true); }
__device__ __forceinline__ unsigned mjt_dpp_xor2(unsigned v) { return (unsigned)__builtin_amdgcn_mov_dpp((int)v, 0x4E, 0xf, 0xf, true); }
__device__ __forceinline__ unsigned mjt_dpp_xor4(unsigned v) {   // mirror of each group of 8 lanes, then a reversal inside each quad
    return (unsigned)__builtin_amdgcn_mov_dpp(__builtin_amdgcn_mov_dpp((int)v, 0x141, 0xf, 0xf, true), 0x1B, 0xf, 0xf, true);
}

// 8 lanes hold 8 rows (k) x 8 columns of 16-bit values, lane r = row r with d[j] = columns 2j, 2j+1.
// Returns column r for the 8 rows: d'[j] = rows 2j, 2j+1.
__device__ __forceinline__ mjt_u32x4v mjt_transpose8x8_b16(mjt_u32x4v d, int lane) {
    const bool b2 = lane & 4, b1 = lane & 2, b0 = lane & 1;
    const unsigned sel_t = b0 ? 0x05040100u : 0x07060302u;
    const unsigned sel_a = b0 ? 0x03020504u : 0x05040100u;
    const unsigned sel_b = b0 ? 0x03020706u : 0x07060100u;
    const unsigned g0 = mjt_dpp_xor4(b2 ? d[0] : d[2]), g1 = mjt_dpp_xor4(b2 ? d[1] : d[3]);
    const unsigned a0 = b2 ? g0 : d[0], a1 = b2 ? g1 : d[1];
    const unsigned a2 = b2 ? d[2] : g0, a3 = b2 ? d[3] : g1;
    const unsigned h0 = mjt_dpp_xor2(b1 ? a0 : a1), h1 = mjt_dpp_xor2(b1 ? a2 : a3);
    const unsigned c0 = b1 ? h0 : a0, c1 = b1 ? a1 : h0;
    const unsigned c2 = b1 ? h1 : a2, c3 = b1 ? a3 : h1;
    const unsigned s0 = mjt_dpp_xor1(__builtin_amdgcn_perm(c1, c0, sel_t)), s1 = mjt_dpp_xor1(__builtin_amdgcn_perm(c3, c2, sel_t));
    mjt_u32x4v f;
    f[0] = __builtin_amdgcn_perm(s0, c0, sel_a);
    f[1] = __builtin_amdgcn_perm(s0, c1, sel_b);
    f[2] = __builtin_amdgcn_perm(s1, c2, sel_a);
    f[3] = __builtin_amdgcn_perm(s1, c3, sel_b);
    return f;
}
// 4 lanes hold 4 rows x 4 columns of 32-bit values, lane r = row r.  Returns column r for the 4 rows.
__device__ __forceinline__ mjt_u32x4v mjt_transpose4x4_b32(mjt_u32x4v v, int lane) {
    const bool b1 = lane & 2, b0 = lane & 1;
    const unsigned g0 = mjt_dpp_xor1(b0 ? v[0] : v[1]), g1 = mjt_dpp_xor1(b0 ? v[2] : v[3]);
    const unsigned a0 = b0 ? g0 : v[0], a1 = b0 ? v[1] : g0;
    const unsigned a2 = b0 ? g1 : v[2], a3 = b0 ? v[3] : g1;
    const unsigned h0 = mjt_dpp_xor2(b1 ? a0 : a2), h1 = mjt_dpp_xor2(b1 ? a1 : a3);
    mjt_u32x4v y;
    y[0] = b1 ? h0 : a0;
    y[1] = b1 ? h1 : a1;
    y[2] = b1 ? a2 : h0;
    y[3] = b1 ? a3 : h1;
    return y;
}

// Fragment reads and the waits for them are written out, so that the order below is what runs: the compiler
// would otherwise move every read next to its first use and wait for it there.
template <int OFF> __device__ __forceinline__ void mjt_ds_read(mjt_u32x4v& dst, unsigned addr) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF) : "memory");
}
// wait until at most N LDS operations are outstanding (LDS returns in order); names the registers that are
// ready then, so that no use of them is scheduled in front of the wait
template <int N, int CNT> __device__ __forceinline__ void mjt_frag_wait(mjt_u32x4v (&f)[CNT]) {
    if constexpr (CNT == 1) asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(f[0]) : "n"(N));
    else if constexpr (CNT == 2) asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(f[0]), "+v"(f[1]) : "n"(N));
    else asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(f[0]), "+v"(f[1]), "+v"(f[2]), "+v"(f[3]) : "n"(N));
}
template <int I, int N, class F> __device__ __forceinline__ void mjt_static_for(F&& f) {
    if constexpr (I < N) {
        f(mjt_ic<I>());
        mjt_static_for<I + 1, N>(f);
    }
}

// One operand tile of a stage on its way from memory to LDS.  ROWS = tile rows (m or n), KCONT = memory has k
// innermost.  p = first element of the operand (of this batch), ld = leading dimension in elements, r0 = first
// tile row, rmax = rows of the operand, k0 = first k of the stage, K = total k.
// fetch() only issues the loads (unconditional: nothing in it looks at a loaded value, so no wait is needed
// before the MFMAs that follow); commit() zeroes what lies beyond K, transposes and writes to LDS.
template <int ROWS, bool KCONT> struct mjt_stager {
    static constexpr int PER = ROWS * KC / NTHR;          // 16-byte moves per thread
    mjt_u32x4v reg[PER];

    __device__ __forceinline__ void fetch(const TIN* __restrict__ p, long long ld, int r0, int rmax, int k0, int K, int tid) {
#pragma unroll
        for (int i = 0; i < PER; i++) {
            if constexpr (KCONT) {
                // chunk c = tid + i * NTHR: row c / KC, k-chunk c % KC (8 consecutive lanes read one 128-byte line)
                const int c = tid + i * NTHR;
                int row = r0 + c / KC;
                row = row < rmax ? row : rmax - 1;
                const int k = k0 + (c % KC) * EPC;
                const int kk = k < K ? k : 0;             // a chunk past the end reads chunk 0 and is zeroed in commit
                reg[i] = *(const mjt_u32x4v*)(p + (long long)row * ld + kk);
            } else {
                // blocks of EPC k-rows x EPC columns: EPC lanes each load 16 bytes (EPC columns) of one k-row.
                // Block b = tid / EPC + i * (NTHR / EPC): column group b % (ROWS / EPC), k-chunk b / (ROWS / EPC);
                // the blocks of a wave are neighbouring column groups, so a k-row's loads of a wave are contiguous.
                const int b = tid / EPC + i * (NTHR / EPC);
                const int cg = b % (ROWS / EPC), kc = b / (ROWS / EPC);
                int col = r0 + cg * EPC;
                col = col < rmax ? col : ((rmax - 1) / EPC) * EPC;      // a group outside the operand reads the last one (ld is a multiple of EPC: a group never leaves its row)
                const int k = k0 + kc * EPC + tid % EPC;
                const int kk = k < K ? k : 0;
                reg[i] = *(const mjt_u32x4v*)(p + (long long)kk * ld + col);
            }
        }
    }
    // TAIL: the stage reaches beyond K
    template <bool TAIL> __device__ __forceinline__ void commit_as(unsigned char* lds, int k0, int K, int tid) const {
#pragma unroll
        for (int i = 0; i < PER; i++) {
            mjt_u32x4v v = reg[i];
            int row, kc;
            if constexpr (KCONT) {
                const int c = tid + i * NTHR;
                row = c / KC;
                kc = c % KC;
                if constexpr (TAIL) {
                    const int valid = K - (k0 + kc * EPC);    // elements of this chunk that exist
#if IN == 2
#pragma unroll
                    for (int e = 0; e < 4; e++) v[e] = e < valid ? v[e] : 0u;
#else
#pragma unroll
                    for (int e = 0; e < 4; e++) v[e] = 2 * e + 1 < valid ? v[e] : 2 * e < valid ? (v[e] & 0xffffu) : 0u;
#endif
                }
            } else {
                const int b = tid / EPC + i * (NTHR / EPC);
                row = (b % (ROWS / EPC)) * EPC + tid % EPC;
                kc = b / (ROWS / EPC);
                if constexpr (TAIL) {
                    if (k0 + kc * EPC + tid % EPC >= K) v = (mjt_u32x4v)(0u);
                }
#if IN == 2
                v = mjt_transpose4x4_b32(v, tid);
#else
                v = mjt_transpose8x8_b16(v, tid);
#endif
            }
            *(mjt_u32x4v*)(lds + row * ROWB + kc * 16) = v;
        }
    }
    __device__ __forceinline__ void commit(unsigned char* lds, int k0, int K, int tid) const {
        if (k0 + KS > K) commit_as<true>(lds, k0, K, tid);    // uniform
        else commit_as<false>(lds, k0, K, tid);
    }
};

#if CONV
// The B tile of a stage of the implicit-GEMM convolution.  Same blocks as mjt_stager<TN, false>: EPC lanes hold EPC
// k-rows x EPC columns (4 x 4 float32 values, 8 x 8 16-bit ones), lane tid % EPC the k-row.  What depends on a column
// alone (its image and pixel) is worked out once per workgroup (mjt_conv_cols): base = element offset of
// x[image][0][oh*SH-PH][ow*SW-PW], hw = that row and column, both biased by 0x4000, in one word (0 for a column past
// N: every tap of it then fails the range check).
struct mjt_conv_cols {
    static constexpr int PER = TN * KC / NTHR;
    int base[PER][EPC];
    unsigned hw[PER][EPC];
    // (compile-time loop indices throughout: with run-time ones the compiler keeps these arrays in scratch memory
    // once the loops are too long for it to unroll them itself)
    __device__ __forceinline__ void init(int n0, int N, int tid) {
        mjt_static_for<0, PER * EPC>([&](auto ic) {
            constexpr int i = decltype(ic)::v / EPC, e = decltype(ic)::v % EPC;
            const int b = tid / EPC + i * (NTHR / EPC);
            const int j = n0 + (b % (TN / EPC)) * EPC + e;
            const int img = j / (OH_ * OW_), px = j - img * (OH_ * OW_);
            const int oh = px / OW_, ow = px - oh * OW_;
            const int ih = oh * SH - PH, iw = ow * SW - PW;
            base[i][e] = j < N ? (img * C_ * H_ + ih) * W_ + iw : 0;
            hw[i][e] = j < N ? ((unsigned)(ih + 0x4000) << 16) | (unsigned)(iw + 0x4000) : 0u;
        });
    }
};
struct mjt_conv_stager {
    static constexpr int PER = TN * KC / NTHR;
    static constexpr int RS = R_ * S_, CRS = C_ * R_ * S_;
    mjt_u32x4v reg[PER];

    __device__ __forceinline__ void fetch(const TIN* __restrict__ x, const mjt_conv_cols& cols, int k0, int tid) {
        mjt_static_for<0, PER>([&](auto ic) {
            constexpr int i = decltype(ic)::v;
            const int b = tid / EPC + i * (NTHR / EPC);
            const int k = k0 + (b / (TN / EPC)) * EPC + tid % EPC;
            const bool kvalid = k < CRS;
            const int kk = kvalid ? k : 0;
            const int c = kk / RS, rs = kk - c * RS;
            const int r = rs / S_, t = rs - r * S_;
            const int koff = (c * H_ + r * DH) * W_ + t * DW;
            const unsigned dhw = ((unsigned)(r * DH) << 16) | (unsigned)(t * DW);
            unsigned v[EPC];
            mjt_static_for<0, EPC>([&](auto ec) {
                constexpr int e = decltype(ec)::v;
                const unsigned q = cols.hw[i][e] + dhw;
                const bool ok = kvalid && (q >> 16) - 0x4000u < (unsigned)H_ && (q & 0xffffu) - 0x4000u < (unsigned)W_;
                // an unconditional load from a valid address, zeroed afterwards: a load under a condition is a branch per
                // element
#if IN == 2
                const unsigned ld = __float_as_uint(x[ok ? cols.base[i][e] + koff : 0]);
#else
                const unsigned ld = x[ok ? cols.base[i][e] + koff : 0];
#endif
                v[e] = ok ? ld : 0u;
            });
#if IN == 2
            reg[i][0] = v[0]; reg[i][1] = v[1]; reg[i][2] = v[2]; reg[i][3] = v[3];
#else
            reg[i][0] = v[0] | (v[1] << 16); reg[i][1] = v[2] | (v[3] << 16); reg[i][2] = v[4] | (v[5] << 16); reg[i][3] = v[6] | (v[7] << 16);
#endif
        });
    }
    __device__ __forceinline__ void commit(unsigned char* lds, int tid) const {
        mjt_static_for<0, PER>([&](auto ic) {
            constexpr int i = decltype(ic)::v;
            const int b = tid / EPC + i * (NTHR / EPC);
            const int row = (b % (TN / EPC)) * EPC + tid % EPC, kc = b / (TN / EPC);
#if IN == 2
            *(mjt_u32x4v*)(lds + row * ROWB + kc * 16) = mjt_transpose4x4_b32(reg[i], tid);
#else
            *(mjt_u32x4v*)(lds + row * ROWB + kc * 16) = mjt_transpose8x8_b16(reg[i], tid);
#endif
        });
    }
};
#endif

extern "C" __global__ __launch_bounds__(NTHR) void ENTRY(Params p) {
    const int M = (int)(long long)p.a[3], N = (int)(long long)p.a[4], K = (int)(long long)p.a[5];
    const long long lda = (long long)p.a[6], ldb = (long long)p.a[7], ldc = (long long)p.a[8];
    const TIN* __restrict__ A = (const TIN*)p.a[0] + (long long)blockIdx.y * (long long)p.a[9];
    const TIN* __restrict__ B = (const TIN*)p.a[1] + (long long)blockIdx.y * (long long)p.a[10];
    // NBUF 1: the host promises K <= KS, a single stage -- one staging buffer, so twice as many workgroups fit a compute unit
    __shared__ __attribute__((aligned(16))) unsigned char lds[NBUF][(TM + TN) * ROWB];

    // Tile order: panels of 4 tile rows, inside a panel column by column.  Workgroups go round-robin over the
    // 8 XCDs, so workgroup id takes tile (id % 8) * per_xcd + id / 8: every XCD works on a compact run of
    // tiles and finds the operand rows and columns it shares in its own L2.
    const int tiles_m = (M + TM - 1) / TM, tiles_n = (N + TN - 1) / TN;
    const int tiles = tiles_m * tiles_n;
    int L = blockIdx.x;
    {
        const int per_xcd = (tiles + 7) / 8;
        L = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
        if (L >= tiles || (blockIdx.x >> 3) >= per_xcd) return;
    }
    int tm, tn;
    {
        const int panel = L / (4 * tiles_n);
        const int rows_here = tiles_m - panel * 4 < 4 ? tiles_m - panel * 4 : 4;
        const int within = L - panel * 4 * tiles_n;
        tn = within / rows_here;
        tm = panel * 4 + within - tn * rows_here;
    }
    const int m0 = tm * TM, n0 = tn * TN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    // The operand tiles of a stage are asked for NSET stages ahead: one stage of 16-bit MFMAs on tiles up to 128 x 128
    // is shorter than a trip to memory, so those keep two stages in registers (2048^3 bfloat16: 31.7 -> 30.6 us; tiles
    // of 64 x 64: 40.8 -> 38.6 us).  Larger tiles have no registers to spare, and float32 stages are long enough (two
    // sets: 153 -> 159 us for 2048^3).
    constexpr int NSET = (NBUF > 1 && MI * NI <= 4 && IN != 2 && !CONV) ? 2 : 1;
    const int nstages = NBUF == 1 ? 1 : (K + KS - 1) / KS;
    mjt_stager<TM, A_KCONT> sa[NSET];
    const int arows = M, brows = N;
#if CONV
    mjt_conv_cols cols;
    cols.init(n0, N, tid);
    mjt_conv_stager sb[NSET];
#else
    mjt_stager<TN, B_KCONT> sb[NSET];
#endif
    auto fetch = [&](auto setc, int stage) {
        constexpr int SET = decltype(setc)::v;
        sa[SET].fetch(A, lda, m0, arows, stage * KS, K, tid);
#if CONV
        sb[SET].fetch(B, cols, stage * KS, tid);
#else
        sb[SET].fetch(B, ldb, n0, brows, stage * KS, K, tid);
#endif
    };
    auto commit = [&](auto setc, int stage) {
        constexpr int SET = decltype(setc)::v;
        unsigned char* buf = &lds[stage & (NBUF - 1)][0];
        sa[SET].commit(buf, stage * KS, K, tid);
#if CONV
        sb[SET].commit(buf + TM * ROWB, tid);
#else
        sb[SET].commit(buf + TM * ROWB, stage * KS, K, tid);
#endif
    };
    mjt_static_for<0, NSET>([&](auto tc) {
        if (decltype(tc)::v < nstages) fetch(tc, decltype(tc)::v);
    });

    mjt_f32x16 acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NI; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    commit(mjt_ic<0>(), 0);
    __syncthreads();

    // fragment addresses of this lane: row lane % 32 of its wave's tile rows, chunk lane / 32
    const int frow = lane & 31, fhalf = lane >> 5;
    // stage s: its tiles sit in LDS buffer s % NBUF; the registers of set s % NSET are free (committed before the
    // stage began) and take stage s + NSET; at the end stage s + 1 goes from set (s + 1) % NSET to the other buffer
    auto run_stage = [&](auto parc, const int s) {
        constexpr int PAR = decltype(parc)::v;
        const unsigned char* la = &lds[s & (NBUF - 1)][0] + (wm * 32 * MI + frow) * ROWB + fhalf * 16;
        const unsigned char* lb = &lds[s & (NBUF - 1)][TM * ROWB] + (wn * 32 * NI + frow) * ROWB + fhalf * 16;
        if (s + NSET < nstages) fetch(parc, s + NSET);
        // a pair of chunks per step; the fragments of the next step are requested before the MFMAs of this one
        mjt_u32x4v fa[2][MI], fb[2][NI];
        const unsigned la_addr = (unsigned)(unsigned long long)(__attribute__((address_space(3))) const unsigned char*)la;
        const unsigned lb_addr = (unsigned)(unsigned long long)(__attribute__((address_space(3))) const unsigned char*)lb;
        auto request = [&](auto ksc, auto setc) {
            constexpr int KSX = decltype(ksc)::v, SET = decltype(setc)::v;
            mjt_static_for<0, MI>([&](auto ic) { mjt_ds_read<decltype(ic)::v * 32 * ROWB + KSX * 32>(fa[SET][decltype(ic)::v], la_addr); });
            mjt_static_for<0, NI>([&](auto jc) { mjt_ds_read<decltype(jc)::v * 32 * ROWB + KSX * 32>(fb[SET][decltype(jc)::v], lb_addr); });
        };
        request(mjt_ic<0>(), mjt_ic<0>());
        mjt_static_for<0, KC / 2>([&](auto ksc) {
            constexpr int ks = decltype(ksc)::v, cur = ks & 1, nxt = cur ^ 1;
            constexpr bool more = ks + 1 < KC / 2;
            if constexpr (more) request(mjt_ic<ks + 1>(), mjt_ic<nxt>());
            mjt_frag_wait<(more ? MI + NI : 0), MI>(fa[cur]);
            mjt_frag_wait<(more ? MI + NI : 0), NI>(fb[cur]);
#if IN == 2
#pragma unroll
            for (int e = 0; e < 4; e++)
#pragma unroll
                for (int i = 0; i < MI; i++)
#pragma unroll
                    for (int j = 0; j < NI; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(fa[cur][i][e]), __uint_as_float(fb[cur][j][e]), acc[i][j], 0, 0, 0);
#else
#pragma unroll
            for (int i = 0; i < MI; i++)
#pragma unroll
                for (int j = 0; j < NI; j++)
                    acc[i][j] = MJT_MFMA16(__builtin_bit_cast(mjt_h8, fa[cur][i]), __builtin_bit_cast(mjt_h8, fb[cur][j]), acc[i][j]);
#endif
        });
        if (s + 1 < nstages) {
            commit(mjt_ic<(PAR + 1) % NSET>(), s + 1);           // the other buffer: nobody reads it now
            __syncthreads();
        }
    };
    for (int s0 = 0; s0 < nstages; s0 += NSET)
        mjt_static_for<0, NSET>([&](auto parc) {
            if (s0 + decltype(parc)::v < nstages) run_stage(parc, s0 + decltype(parc)::v);
        });

    // D of a 32x32 tile: lane holds column lane % 32, rows 8 * (e / 4) + 4 * (lane / 32) + e % 4
#if OUT == 2
    float* __restrict__ C = (float*)p.a[2] + (long long)blockIdx.y * (long long)p.a[11];
#else
    unsigned short* __restrict__ C = (unsigned short*)p.a[2] + (long long)blockIdx.y * (long long)p.a[11];
#endif
#pragma unroll
    for (int i = 0; i < MI; i++)
#pragma unroll
        for (int j = 0; j < NI; j++) {
            const int col = n0 + wn * 32 * NI + j * 32 + (lane & 31);
#if CONV
            const int img = col / (OH_ * OW_), px = col - img * (OH_ * OW_);      // y[img][row][px]
#endif
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int row = m0 + wm * 32 * MI + i * 32 + 8 * (e / 4) + 4 * (lane >> 5) + (e & 3);
                if (row < M && col < N) {
                    const float v = acc[i][j][e];
#if CONV
                    const long long at = ((long long)img * K_ + row) * (OH_ * OW_) + px;
#else
                    const long long at = (long long)row * ldc + col;
#endif
#if OUT == 2
                    C[at] = v;
#elif OUT == 0
                    C[at] = (unsigned short)(__float_as_uint(v) >> 16);     // truncation (type/fp16_compute.h:238-241)
#else
                    const _Float16 h = (_Float16)v;                        // nearest even (type/fp16_compute.h:147-198)
                    C[at] = __builtin_bit_cast(unsigned short, h);
#endif
                }
            }
        }
}
