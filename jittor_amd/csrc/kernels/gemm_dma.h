// Matrix product on MFMA for 16-bit operands, operands copied from memory straight into LDS:
//   C[b][M][N] = sum_k A'[b][M][K] * B'[b][K][N]
// (reference: the broadcast * broadcast -> reduce.add pattern that
// python/jittor/src/opt/tuner/matmul_tuner.cc:16-104 relays to a library GEMM,
// python/jittor/extern/cuda/cublas/ops/cublas_matmul_op.cc:27-126; a x b^T is the forward product of a linear
// layer, python/jittor/nn.py:628-643).  Row-major operands; A' is a, or a transposed when A_KCONT == 0 (memory
// [K][M]); B' is b, or b transposed when B_KCONT == 1 (memory [N][K]).  bfloat16 / float16 operands with exact
// products and float32 accumulation.
//
// Supplied by the host: IN (0 bfloat16, 1 float16), OUT (0 bfloat16 by truncation, 1 float16 rounded to
// nearest even, 2 float32), A_KCONT, B_KCONT (the operand's memory has k innermost).  K is a multiple of 64, leading
// dimensions are multiples of 16 bytes and the operand pointers 16-byte aligned (the host sends everything else to the
// general kernel).
//
// Mapping.  A workgroup of four waves (2 x 2, one wave per SIMD) owns a 256 x 256 tile of C; a wave owns
// 128 x 128 of it as 4 x 4 accumulator tiles of v_mfma_f32_32x32x16, 256 accumulation registers.  K is walked in
// stages of 64 (whole 128-byte lines of both operands): the 256 x 64 pieces of both operands (64 KB) alternate
// between two buffers in LDS.  Nothing on that way passes through registers: a wave copies 1 KB per instruction
// straight from memory into LDS (lane i lands at byte 16 i of that KB), a stage ahead of its use.  For an operand
// with k innermost that is 8 rows x 128 bytes: a row of a stage is eight 16-byte chunks, chunk c of row r sits at
// position c ^ (r / 2 % 8), which the copying lane arranges by choosing what it fetches; the 16 lanes that read a
// fragment together (16 neighbouring rows, one chunk) then touch 16 different bank groups, and lane (row =
// lane % 32, half = lane / 32) reads the 8 consecutive k of its row and half with one 16-byte LDS read.  An operand
// with m or n innermost stays as it lies in memory, [64 k][256 columns], and the fragment is made by two transposing
// LDS reads (ds_read_b64_tr_b16: the 16 lanes of a group present 16 8-byte pieces, four k-rows x 16 columns, and
// each receives one column's four k); its 32-byte units are permuted within a row by the k-row so that the four
// rows of a read fall into different banks.  The fragments of the next k-step are read while the 16 MFMAs of a
// k-step run.  One barrier per stage, before its last k-step, hands over the next stage, which has landed by then,
// and frees the buffer of the current one, whose last fragments are in registers.  Rows beyond M and N of an operand
// with k innermost are read from the last valid row, columns beyond them of the other kind from whatever follows in
// memory (zero past the operand's end); their results are not stored.
//
// The MFMAs are spelled out, like the LDS reads and the waits, so that the order below is the schedule; the
// accumulators live in the accumulation registers, which nothing but these MFMAs touches inside the loop (the
// compiler takes a spelled-out MFMA for finished the moment it is issued).

typedef float mjt_f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned mjt_u32x4v __attribute__((ext_vector_type(4)));
#if IN == 0
#define MJT_MFMA_ASM "v_mfma_f32_32x32x16_bf16"
#else
#define MJT_MFMA_ASM "v_mfma_f32_32x32x16_f16"
#endif
#ifndef TILE
#define TILE 256
#endif
#ifndef NBUF
#define NBUF 2
#endif
#define TM TILE
#define TN TILE
#define KS 64
#define STAGE_BYTES ((TM + TN) * 128)
#define NTHR 256
#define FR (TILE / 64)          // 32 x 32 accumulator tiles per wave along each axis
#define NM (FR * FR)            // MFMAs of a k-step
#define WT (TILE / 2)           // rows and columns of C per wave
#define CPW (TILE / 32)         // 1 KB copies per wave, operand and stage
#define ROWB (TILE * 2)         // bytes of a k-row of an operand staged with m or n innermost
#define RPI (1024 / ROWB)       // k-rows of such an operand per copy
#define PPR (ROWB / 16)         // 16-byte pieces of such a k-row
#define PFD (TILE == 256 ? 1 : 2)                   // how many k-steps ahead the fragments are read
#define NSETS (PFD == 1 ? 2 : 4)                    // fragment sets

template <int V> struct mjt_ic { static constexpr int v = V; };
template <int I, int N, class F> __device__ __forceinline__ void mjt_static_for(F&& f) {
    if constexpr (I < N) {
        f(mjt_ic<I>());
        mjt_static_for<I + 1, N>(f);
    }
}
typedef unsigned mjt_u32x2 __attribute__((ext_vector_type(2)));
// a 16-byte read delivered as two halves (so that fragments have one representation whichever read fills them)
template <int OFF> __device__ __forceinline__ void mjt_ds_read_pair(mjt_u32x2& lo, mjt_u32x2& hi, unsigned addr) {
    mjt_u32x4v v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF) : "memory");
    lo[0] = v[0]; lo[1] = v[1]; hi[0] = v[2]; hi[1] = v[3];
}
// transposing read: the lane receives four 16-bit values, one from each of four lanes' 8-byte pieces
template <int OFF> __device__ __forceinline__ void mjt_ds_read_tr(mjt_u32x2& dst, unsigned addr) {
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF) : "memory");
}
__device__ __forceinline__ void mjt_mfma2(mjt_f32x16& c, const mjt_u32x2& alo, const mjt_u32x2& ahi, const mjt_u32x2& blo, const mjt_u32x2& bhi) {
    mjt_u32x4v a, b;
    a[0] = alo[0]; a[1] = alo[1]; a[2] = ahi[0]; a[3] = ahi[1];
    b[0] = blo[0]; b[1] = blo[1]; b[2] = bhi[0]; b[3] = bhi[1];
    asm volatile(MJT_MFMA_ASM " %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mjt_keep2(const mjt_u32x2& x) { asm volatile("" : : "v"(x)); }     // x is in its registers up to here
__device__ __forceinline__ void mjt_pin(mjt_f32x16& x) { asm volatile("" : "+a"(x)); }            // what reads x later comes after this point

struct Params { void* a[12]; };

#ifndef WPE
#define WPE 1                   // workgroups (of one wave per SIMD) a compute unit is meant to hold
#endif
extern "C" __global__ __launch_bounds__(NTHR) __attribute__((amdgpu_waves_per_eu(1, WPE))) void ENTRY(Params p) {
    const int M = (int)(long long)p.a[3], N = (int)(long long)p.a[4], K = (int)(long long)p.a[5];
    const long long lda = (long long)p.a[6], ldb = (long long)p.a[7], ldc = (long long)p.a[8];
    const unsigned short* __restrict__ A = (const unsigned short*)p.a[0] + (long long)blockIdx.y * (long long)p.a[9];
    const unsigned short* __restrict__ B = (const unsigned short*)p.a[1] + (long long)blockIdx.y * (long long)p.a[10];
    __shared__ __attribute__((aligned(16))) unsigned char lds[NBUF * STAGE_BYTES];

    // Tile order: panels of 4 tile rows, inside a panel column by column.  Workgroups go round-robin over the
    // 8 XCDs, so workgroup id takes tile (id % 8) * per_xcd + id / 8: every XCD works on a compact run of
    // tiles and finds the operand rows and columns it shares in its own L2.
    const int tiles_m = (M + TM - 1) / TM, tiles_n = (N + TN - 1) / TN;
    const int tiles = tiles_m * tiles_n;
    int L;
    {
        const int per_xcd = (tiles + 7) / 8;
        L = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
        if (L >= tiles || (int)(blockIdx.x >> 3) >= per_xcd) return;
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
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int nstages = K / KS;

    // Copies.  A stage is 64 instructions of 1 KB (32 per operand); wave w issues number 8w .. 8w+7 of each operand.
    // An operand with k innermost is staged [256 rows][64 k]: lane i of instruction j fills row 8 j + i / 8, position
    // i % 8, with chunk (i % 8) ^ (row / 2 % 8); its descriptor starts at the tile's first row, the lane offset is its
    // row (clamped to the matrix) times the leading dimension plus its chunk, and a stage adds 128 bytes through the
    // scalar offset.  An operand with m (or n) innermost is staged as it lies in memory, [64 k][256 columns], 512-byte
    // rows of sixteen 32-byte units: lane i of instruction j fills k-row 2 j + i / 32, 16-byte piece i % 32, and unit u of
    // k-row r sits at position u ^ (r % 4).  Its descriptor starts at the tile's first column and ends with the operand,
    // so whatever lies past the matrix reads as zero; a stage adds 64 rows through the scalar offset.
    const int last_a = M - 1 - m0, last_b = N - 1 - n0;             // last valid row of the tile
    unsigned voff_a[CPW], voff_b[CPW];
#pragma unroll
    for (int q = 0; q < CPW; q++) {
        const int row = (wave * CPW + q) * 8 + (lane >> 3);
        const unsigned chunk = (unsigned)((lane & 7) ^ ((row >> 1) & 7));
        const int krow = (wave * CPW + q) * RPI + lane / PPR;
        const int pl = lane % PPR;
        const unsigned piece = (unsigned)((((pl >> 1) ^ (krow & 3)) << 1) | (pl & 1));                  // 16-byte piece of the k-row in memory
#if A_KCONT
        voff_a[q] = (unsigned)(row < last_a ? row : last_a) * (unsigned)(lda * 2) + chunk * 16;
#else
        voff_a[q] = (unsigned)krow * (unsigned)(lda * 2) + piece * 16;
#endif
#if B_KCONT
        voff_b[q] = (unsigned)(row < last_b ? row : last_b) * (unsigned)(ldb * 2) + chunk * 16;
#else
        voff_b[q] = (unsigned)krow * (unsigned)(ldb * 2) + piece * 16;
#endif
    }
#if A_KCONT
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)(A + (long long)m0 * lda), 0, 0x7fffffff, 0x00020000);
    const int a_step = KS * 2;
#else
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)(A + m0), 0, (int)(((long long)(K - 1) * lda + (M - m0)) * 2), 0x00020000);
    const int a_step = (int)(KS * lda * 2);
#endif
#if B_KCONT
    const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)(B + (long long)n0 * ldb), 0, 0x7fffffff, 0x00020000);
    const int b_step = KS * 2;
#else
    const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)(B + n0), 0, (int)(((long long)(K - 1) * ldb + (N - n0)) * 2), 0x00020000);
    const int b_step = (int)(KS * ldb * 2);
#endif
    // instruction q (0 .. 15: eight of A, eight of B) of this wave's share of stage s; s and slot uniform
    auto copy_one = [&](auto qc, int s, int slot) {
        constexpr int q = decltype(qc)::v;
        const int st = s < nstages ? s : nstages - 1;               // past the end: a stage nobody reads
        __attribute__((address_space(3))) unsigned char* dst =
            (__attribute__((address_space(3))) unsigned char*)&lds[0] + slot * STAGE_BYTES + wave * (CPW * 1024);
        // (an immediate offset would move the place in memory along with the place in LDS)
        if constexpr (q < CPW)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, (__attribute__((address_space(3))) void*)(dst + q * 1024), 16, (int)voff_a[q], st * a_step, 0, 0);
        else
            __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, (__attribute__((address_space(3))) void*)(dst + TM * 128 + (q - CPW) * 1024), 16, (int)voff_b[q - CPW], st * b_step, 0, 0);
    };
    auto copy_stage = [&](int s, int slot) { mjt_static_for<0, 2 * CPW>([&](auto qc) { copy_one(qc, s, slot); }); };

    // Fragments.  Lane (row = lane % 32, half = lane / 32) of v_mfma_f32_32x32x16 wants the 8 consecutive k of its row
    // and half.  From a [rows][64 k] tile that is one 16-byte read: row lane % 32 of each 32-row block of the wave's
    // rows, chunk 2 * k-step + half at position chunk ^ (row / 2 % 8), i.e. the position of k-step 0 with the k-step's
    // bits flipped.  From a [64 k][256 columns] tile it is two transposing reads of four k each: the 16 lanes of a group
    // point at four k-rows x four 8-byte pieces (lane i at k-row i / 4, piece i % 4 of the group's 16 columns) and
    // receive column i of the group for those four k.
    const int frow = lane & 31;
    const unsigned pos0 = (unsigned)((lane >> 5) ^ ((frow >> 1) & 7));
    const unsigned lds_base = (unsigned)(unsigned long long)(__attribute__((address_space(3))) unsigned char*)&lds[0];
    const int ti = lane & 15, tg = (lane >> 4) & 1, tk = lane >> 5;
#if A_KCONT
    const unsigned a_lane = lds_base + (unsigned)((wm * WT + frow) * 128);
#else
    unsigned a_tr[FR];
#pragma unroll
    for (int f = 0; f < FR; f++) a_tr[f] = lds_base + (unsigned)((tk * 8 + (ti >> 2)) * ROWB + (((wm * (WT / 16) + 2 * f + tg) ^ (ti >> 2)) * 32) + (ti & 3) * 8);
#endif
#if B_KCONT
    const unsigned b_lane = lds_base + (unsigned)(TM * 128 + (wn * WT + frow) * 128);
#else
    unsigned b_tr[FR];
#pragma unroll
    for (int f = 0; f < FR; f++) b_tr[f] = lds_base + (unsigned)(TM * 128 + (tk * 8 + (ti >> 2)) * ROWB + (((wn * (WT / 16) + 2 * f + tg) ^ (ti >> 2)) * 32) + (ti & 3) * 8);
#endif
    mjt_u32x2 falo[NSETS][FR], fahi[NSETS][FR], fblo[NSETS][FR], fbhi[NSETS][FR];       // a fragment's four registers in two halves
    constexpr int A_READS = A_KCONT ? FR : 2 * FR, B_READS = B_KCONT ? FR : 2 * FR, READS = A_READS + B_READS;
    // read number r (0 .. READS-1) of the fragments of k-step kstep (compile-time) of the stage in slot, into set SET
    auto request_one = [&](auto setc, auto rc, int slot, auto kc) {
        constexpr int SET = decltype(setc)::v, r = decltype(rc)::v, kstep = decltype(kc)::v;
        const unsigned soff = (unsigned)(slot * STAGE_BYTES);
        if constexpr (r < A_READS) {
#if A_KCONT
            mjt_ds_read_pair<r * 4096>(falo[SET][r], fahi[SET][r], a_lane + soff + ((pos0 ^ (unsigned)(kstep * 2)) * 16));
#else
            if constexpr (r % 2 == 0) mjt_ds_read_tr<(kstep * 16) * ROWB>(falo[SET][r / 2], a_tr[r / 2] + soff);
            else mjt_ds_read_tr<(kstep * 16 + 4) * ROWB>(fahi[SET][r / 2], a_tr[r / 2] + soff);
#endif
        } else {
            constexpr int rb = r - A_READS;
#if B_KCONT
            mjt_ds_read_pair<rb * 4096>(fblo[SET][rb], fbhi[SET][rb], b_lane + soff + ((pos0 ^ (unsigned)(kstep * 2)) * 16));
#else
            if constexpr (rb % 2 == 0) mjt_ds_read_tr<(kstep * 16) * ROWB>(fblo[SET][rb / 2], b_tr[rb / 2] + soff);
            else mjt_ds_read_tr<(kstep * 16 + 4) * ROWB>(fbhi[SET][rb / 2], b_tr[rb / 2] + soff);
#endif
        }
    };

    mjt_f32x16 acc[FR][FR];
#pragma unroll
    for (int i = 0; i < FR; i++)
#pragma unroll
        for (int j = 0; j < FR; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;
    // the zeros are written here, not next to the first MFMA that reads them
    mjt_static_for<0, NM>([&](auto ic) { mjt_pin(acc[decltype(ic)::v / FR][decltype(ic)::v % FR]); });
    asm volatile("s_nop 7" : : : "memory");

    // A k-step: NM MFMAs on the fragments of set SET.  What else the wave has to issue goes between them, behind the
    // MFMAs, where it costs no MFMA time (the wave is alone on its SIMD): the reads of the fragments of the k-step PFD
    // steps ahead into that step's set and, in the last PFD k-steps of a stage, the copies of the stage NBUF stages ahead
    // (COPY0 .. COPY0 + COPYN - 1 of the wave's 2 CPW).  With 256 x 256 tiles a k-step is 16 MFMAs and hides the reads of
    // the next one (PFD 1, two sets); the 4 MFMAs of a 128 x 128 tile's k-step do not, so there the reads run two k-steps
    // ahead (PFD 2, a set per k-step of a stage) and a k-step waits for all but the latest READS of them.
    auto kstep = [&](auto setc, auto rdsetc, int rd_slot, auto rd_kstep, auto copy0c, auto copync, int cp_stage, int cp_slot) {
        constexpr int SET = decltype(setc)::v, RDSET = decltype(rdsetc)::v;
        constexpr int COPY0 = decltype(copy0c)::v, COPYN = decltype(copync)::v;
        constexpr int RPM = (READS + NM - 1) / NM, CPM = (COPYN + NM - 1) / NM;       // reads and copies behind one MFMA
        mjt_static_for<0, NM>([&](auto ic) {
            constexpr int i = decltype(ic)::v;
            mjt_mfma2(acc[i / FR][i % FR], falo[SET][i / FR], fahi[SET][i / FR], fblo[SET][i % FR], fbhi[SET][i % FR]);
            mjt_static_for<0, RPM>([&](auto jc) {
                constexpr int r = i * RPM + decltype(jc)::v;
                if constexpr (r < READS) request_one(mjt_ic<RDSET>(), mjt_ic<r>(), rd_slot, rd_kstep);
            });
            mjt_static_for<0, CPM>([&](auto jc) {
                constexpr int q = i * CPM + decltype(jc)::v;
                if constexpr (q < COPYN) copy_one(mjt_ic<COPY0 + q>(), cp_stage, cp_slot);
            });
        });
    };
    // the first NBUF stages are asked for; stage 0 must have landed before the loop (a wave's copies land in order)
    mjt_static_for<0, NBUF>([&](auto sc) { copy_stage(decltype(sc)::v, decltype(sc)::v); });
    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" : : "n"((NBUF - 1) * 2 * CPW) : "memory");
    mjt_static_for<0, PFD>([&](auto kc) {
        mjt_static_for<0, READS>([&](auto rc) { request_one(kc, rc, 0, kc); });
    });

#pragma unroll 1
    for (int s = 0; s < nstages; s++) {
        const int slot = s & (NBUF - 1), next_slot = (s + 1) & (NBUF - 1);
        mjt_static_for<0, 4>([&](auto jc) {
            constexpr int j = decltype(jc)::v, ahead = j + PFD;                 // this k-step, and the one whose fragments it asks for
            constexpr int COPYN = j >= 4 - PFD ? 2 * CPW / PFD : 0, COPY0 = j >= 4 - PFD ? (j - (4 - PFD)) * COPYN : 0;
            // Before the first k-step that reads the next stage (PFD steps before the stage's end): every fragment of
            // this stage is in registers, so nobody reads its buffer any more once every wave is here, and the copies of
            // the next stage, asked for NBUF - 1 stages ago, have landed.
            if constexpr (j == 4 - PFD)
                asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" : : "n"((NBUF - 2) * 2 * CPW) : "memory");
            else
                asm volatile("s_waitcnt lgkmcnt(%0)" : : "n"((PFD - 1) * READS) : "memory");
            kstep(mjt_ic<j % NSETS>(), mjt_ic<ahead % NSETS>(), ahead < 4 ? slot : next_slot, mjt_ic<ahead % 4>(), mjt_ic<COPY0>(), mjt_ic<COPYN>(),
                  s + NBUF, slot);
        });
    }
    // The last MFMAs need time to read their operands and write their results; tie the registers to a point behind that.
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15" : : : "memory");
    mjt_static_for<0, NSETS * FR>([&](auto ic) {
        constexpr int st = decltype(ic)::v / FR, f = decltype(ic)::v % FR;
        mjt_keep2(falo[st][f]); mjt_keep2(fahi[st][f]); mjt_keep2(fblo[st][f]); mjt_keep2(fbhi[st][f]);
    });
    mjt_static_for<0, NM>([&](auto ic) { mjt_pin(acc[decltype(ic)::v / FR][decltype(ic)::v % FR]); });

    // D of a 32x32 tile: lane holds column lane % 32, rows 8 * (e / 4) + 4 * (lane / 32) + e % 4
#if OUT == 2
    float* __restrict__ C = (float*)p.a[2] + (long long)blockIdx.y * (long long)p.a[11];
#else
    unsigned short* __restrict__ C = (unsigned short*)p.a[2] + (long long)blockIdx.y * (long long)p.a[11];
#endif
#pragma unroll
    for (int i = 0; i < FR; i++)
#pragma unroll
        for (int j = 0; j < FR; j++) {
            const int col = n0 + wn * WT + j * 32 + (lane & 31);
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int row = m0 + wm * WT + i * 32 + 8 * (e / 4) + 4 * (lane >> 5) + (e & 3);
                if (row < M && col < N) {
                    const float v = acc[i][j][e];
#if OUT == 2
                    C[(long long)row * ldc + col] = v;
#elif OUT == 0
                    C[(long long)row * ldc + col] = (unsigned short)(__float_as_uint(v) >> 16);     // truncation (type/fp16_compute.h:238-241)
#else
                    const _Float16 h = (_Float16)v;                                                  // nearest even (type/fp16_compute.h:147-198)
                    C[(long long)row * ldc + col] = __builtin_bit_cast(unsigned short, h);
#endif
                }
            }
        }
}
