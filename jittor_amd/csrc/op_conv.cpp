// mjt_conv2d_meta: host side of the meta-op convolution (the group
// python/jittor/nn.py:1251-1262 builds; parameters as solved by
// python/jittor/src/opt/tuner/conv_tuner.cc:312-356).
#include "common.h"
#include <array>
#include <mutex>
#include <unordered_map>

namespace mjt {

namespace {
std::mutex g_mu;
std::unordered_map<std::string, JitKernel*> g_kernels;
JitKernel* cached(const std::string& key) {
    std::lock_guard<std::mutex> lock(g_mu);
    auto it = g_kernels.find(key);
    return it == g_kernels.end() ? nullptr : it->second;
}
void remember(const std::string& key, JitKernel* k) {
    std::lock_guard<std::mutex> lock(g_mu);
    g_kernels.emplace(key, k);
}
void* g_wpack = nullptr;
size_t g_wpack_bytes = 0;
void* g_wgrad_part = nullptr;      // per-slice partial weight gradients (its own buffer: the reduce that folds them uses the arena)
size_t g_wgrad_bytes = 0;
// column matrices of a chunk of images; float32 copy of a bfloat16 result; for the input gradient: rearranged weights,
// and dy spread out with zeros or the results of the stride phases
// [4]: weights with rows padded to 16 bytes for the product; [5]: the product of a whole batch, channels outermost
void* g_conv_scratch[6] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
size_t g_conv_scratch_bytes[6] = {0, 0, 0, 0, 0, 0};

void forget() {
    std::lock_guard<std::mutex> lock(g_mu);
    for (auto& kv : g_kernels)
        if (kv.first.size() > 5 && kv.first.compare(kv.first.size() - 5, 5, "|pack") == 0) delete kv.second;   // shares its module with the main kernel
    g_kernels.clear();                                  // the kernels themselves belong to the run-time compiler's cache
    if (!ctx().dry_run) {
        if (g_wpack) (void)hipFree(g_wpack);
        if (g_wgrad_part) (void)hipFree(g_wgrad_part);
        for (void* b : g_conv_scratch)
            if (b) (void)hipFree(b);
    }
    g_wpack = g_wgrad_part = nullptr;
    g_wpack_bytes = g_wgrad_bytes = 0;
    for (int i = 0; i < 6; i++) {
        g_conv_scratch[i] = nullptr;
        g_conv_scratch_bytes[i] = 0;
    }
}
const bool g_registered = (at_shutdown(&forget), true);

// One of the two growing buffers of the GEMM path.
void* conv_scratch(int which, size_t bytes) {
    Context& c = ctx();
    if (c.dry_run) return (void*)(uintptr_t)0x1000;
    if (bytes > g_conv_scratch_bytes[which]) {
        if (g_conv_scratch[which]) {
            HIP_CHECK(hipStreamSynchronize(c.stream));
            HIP_CHECK(hipFree(g_conv_scratch[which]));
            g_conv_scratch[which] = nullptr;
            g_conv_scratch_bytes[which] = 0;
        }
        HIP_CHECK(hipMalloc(&g_conv_scratch[which], bytes));
        g_conv_scratch_bytes[which] = bytes;
    }
    return g_conv_scratch[which];
}
}  // namespace

void matmul_impl(const mjt_tensor* a, const mjt_tensor* b, const mjt_tensor* c, int trans_a, int trans_b, bool share_a);
bool matmul_available();
void gemm_launch(int in_dtype, int out_dtype, const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K,
                 int64_t lda, int64_t ldb, int64_t ldc, int64_t sa, int64_t sb, int64_t sc, int64_t batch, bool a_kcont,
                 bool b_kcont, int tile_m = 0, int tile_n = 0, bool allow_direct = true);

// free_extent: y's rows and columns are taken as they are instead of checked against the extents that stride, padding and
// taps give (output (oh, ow) reads x around (oh*sh - ph, ow*sw - pw) whatever oh and ow; outside the image x is 0): what the
// stride phases of an input gradient need, whose zero margins differ between the two ends of an axis.
// packed / pack_mode: 0 the call packs the weights itself (into the library's buffer) and runs; 1 it only packs them
// into `packed`; 2 it runs on weights packed by an earlier call of mode 1 for the same shapes and parameters.  Modes 1
// and 2 exist for the MFMA kernel only and fail with MJT_ERR_UNSUPPORTED for a convolution that takes another route.
void conv_impl(const mjt_tensor* x, const mjt_tensor* w, const mjt_tensor* y, const mjt_conv_params* p, int64_t G, bool free_extent = false,
               int pack_mode = 0, void* packed = nullptr) {
    require_init();
    check_tensor(x, "conv x");
    check_tensor(w, "conv w");
    check_tensor(y, "conv y");
    MJT_CHECK(p, "conv: null parameters");
    MJT_CHECK(x->ndim == 4 && w->ndim == 4 && y->ndim == 4, "conv: x, w and y must have rank 4");
    MJT_CHECK(x->dtype == w->dtype && (x->dtype == MJT_BFLOAT16 || x->dtype == MJT_FLOAT16 || x->dtype == MJT_FLOAT32),
              "conv: x and w must both be bfloat16, float16 or float32");
    MJT_CHECK(y->dtype == MJT_FLOAT32 || y->dtype == x->dtype, "conv: y must be float32 or the input dtype");
    MJT_CHECK(G >= 1, "conv: groups must be >= 1, got " << G);
    // C is the number of channels one output channel sees: all of x's, or those of its group
    const int64_t N = x->shape[0], C = w->shape[1], H = x->shape[2], W = x->shape[3];
    const int64_t K = w->shape[0], R = w->shape[2], S = w->shape[3];
    MJT_CHECK(x->shape[1] == C * G, "conv: weight channels " << C << " x " << G << " group(s) != input channels " << x->shape[1]);
    MJT_CHECK(K % G == 0, "conv: " << K << " output channels do not divide into " << G << " groups");
    MJT_CHECK(p->stride_h >= 1 && p->stride_w >= 1 && p->dil_h >= 1 && p->dil_w >= 1 && p->pad_h >= 0 && p->pad_w >= 0,
              "conv: bad stride / padding / dilation");
    const int64_t OH = free_extent ? y->shape[2] : (H + 2 * p->pad_h - p->dil_h * (R - 1) - 1) / p->stride_h + 1;
    const int64_t OW = free_extent ? y->shape[3] : (W + 2 * p->pad_w - p->dil_w * (S - 1) - 1) / p->stride_w + 1;
    MJT_CHECK(OH >= 1 && OW >= 1, "conv: empty output");
    MJT_CHECK(y->shape[0] == N && y->shape[1] == K && y->shape[2] == OH && y->shape[3] == OW,
              "conv: y shape " << shape_str(y) << " != [" << N << "," << K << "," << OH << "," << OW << "]");
    if (N == 0 || K == 0) return;
    MJT_CHECK(numel(x) < (int64_t(1) << 40) && numel(y) < (int64_t(1) << 40), "conv: too large");
    Context& c = ctx();

    std::ostringstream geo;
    geo << "#define C_ " << C << "\n#define H_ " << H << "\n#define W_ " << W << "\n#define K_ " << K << "\n#define R_ " << R
        << "\n#define S_ " << S << "\n#define OH_ " << OH << "\n#define OW_ " << OW << "\n#define SH " << p->stride_h
        << "\n#define SW " << p->stride_w << "\n#define PH " << p->pad_h << "\n#define PW " << p->pad_w << "\n#define DH "
        << p->dil_h << "\n#define DW " << p->dil_w << "\n";

    // ---- MFMA path ----------------------------------------------------------------
    const int64_t WPX = 2;                                  // pixel halves per workgroup (1: one wave per SIMD with 224-pixel wave tiles, 224-227 us on the 3x3 256-channel 56x56 layer against 215)
    const int64_t max_px = WPX == 1 ? 224 : 112;            // pixels per wave: 16 per accumulator tile
    const int64_t WPS = max_px == 224 ? 1 : 2;              // waves per SIMD the register budget is set for
    // output channels per wave: 16 per accumulator-tile row; per workgroup: up to 256
    const int64_t Kg = K / G;                                // output channels of one group: the K of the MFMA kernel
    // accumulator-tile rows (of 16 output channels) per wave: 4; 2 for groups of 64 or 128 output channels, which then have four
    // waves share an input tile instead of two (64 x 64 x 56 x 56 3x3 -> 64: 42.9 -> 31.7 us; 64 x 256 x 56 x 56 -> 64:
    // 124 -> 86; 64 x 64 x 28 x 28 -> 64: 20.8 -> 14.3)
    // (groups of 128: eight waves of 32 channels instead of four of 64: 64 x 128 x 28 x 28 3x3 -> 128: 25.4 -> 24.6 us,
    // with 8 images 23.0 -> 18.4)
    int64_t MT = Kg == 32 || Kg == 64 || Kg == 128 ? 2 : 4;
    auto widest = [&]() {                                   // groups of output channels per workgroup: up to 256 channels, eight waves
        const int64_t v = Kg % 256 == 0 ? 256 / (16 * MT) : Kg % 128 == 0 ? 128 / (16 * MT) : Kg % 64 == 0 ? 64 / (16 * MT) : 32 / (16 * MT);
        return v > 4 ? int64_t(4) : v;
    };
    int64_t WKO = widest();
    // LDS: two buffers of input rows (one block of CB channels each), a ring of NS weight slabs (64 bytes per output
    // channel of the workgroup each) and a spare KB that takes the writes of idle lanes.  Blocks of 32 channels
    // leave room for a deeper ring, which is what hides the latency of the slabs; the ring needs three slabs at least.
    const int64_t lds_total = 160 * 1024;
    const int64_t CBLK = 32;
    const int64_t slab0 = 64 * 16 * MT * WKO, spare0 = 1024;
    const int64_t tile_limit = (lds_total - 4 * slab0 - spare0) / 2;         // leaves room for four slabs of the widest workgroup
    int64_t TRW = OW <= max_px ? max_px / OW : 0;
    if (TRW > OH) TRW = OH;
    while (TRW > 1 && WPX * TRW > OH && (OH % (WPX * TRW)) != 0 && (WPX * (TRW - 1)) >= OH) TRW--;
    auto lds_rows = [&](int64_t trw) { return (WPX * trw - 1) * p->stride_h + (R - 1) * p->dil_h + 1; };
    const int64_t LCOLS = (OW - 1) * p->stride_w + (S - 1) * p->dil_w + 1 > W + 2 * p->pad_w
                              ? (OW - 1) * p->stride_w + (S - 1) * p->dil_w + 1
                              : W + 2 * p->pad_w;
    while (TRW > 1 && lds_rows(TRW) * LCOLS * CBLK * 2 > tile_limit) TRW--;
    const int64_t NT = TRW ? (TRW * OW + 15) / 16 : 0;
    const int64_t LROWS = lds_rows(TRW);
    {
        // fewer output channels per workgroup while the grid would leave compute units idle (small maps, small batches):
        // the same input tile is then staged by more workgroups, which the L2 absorbs
        const int64_t cus0 = c.dry_run || c.prop.multiProcessorCount <= 0 ? 256 : c.prop.multiProcessorCount;
        const int64_t tile_rows = WPX * (TRW > 0 ? TRW : 1);
        const int64_t min_ranges = N * ((OH + tile_rows - 1) / tile_rows);
        // (down to 128 channels per workgroup, four waves, never to workgroups of two waves: 64 x 256 x 14 x 14 3x3 -> 256 on 128
        // workgroups of four waves 48 us, on 256 of two waves 61, on 64 of eight 65; with 8 images 48 against 58)
        const int64_t before = WKO;
        while (WKO > 2 && 2 * min_ranges * (Kg / (16 * MT * WKO)) <= cus0) WKO /= 2;
        // such a small grid with more channels: wave tiles of 32 channels as well, so that twice as many workgroups of four
        // waves share the work (64 x 256 x 14 x 14 3x3 -> 256: 48 -> 39 us; 64 x 256 x 14 x 14 3x3 stride 2 -> 512: 42 -> 37)
        if (WKO < before && MT == 4) {
            MT = 2;
            WKO = widest();
            while (WKO > 2 && 2 * min_ranges * (Kg / (16 * MT * WKO)) <= cus0) WKO /= 2;
        }
    }
    const bool half = x->dtype == MJT_FLOAT16;
    // Small maps with long sums that the MFMA kernel below does not take (7 x 7 and 13 x 13 maps: odd widths): one
    // product for the whole batch, y'[K][N * P] = w [K][C*R*S] x cols [C*R*S][N * P], on column matrices with the images
    // side by side, then y' -> y [N][K][P] by one permutation.  The gather of the implicit GEMM is paid once per 64 or
    // 128 output channels, the column matrices once (us, bf16, gather / per-image column matrices / this:
    // 64 x 512 x 7 x 7 3x3 -> 512: 126 / 85 / 60; 64 x 256 x 13 x 13 3x3 -> 384: 76 / 103 / 69; 1x1 on 7 x 7 maps,
    // gather / this: 2048 -> 512: 60 / 35; 1024 -> 1024: 38 / 29; 512 -> 2048: 38 / 31; on 14 x 14: 1024 -> 512: 63 / 51;
    // 512 -> 512: 36 / 36; 1024 -> 256: 36 / 41; short sums, few output channels and larger maps stay with the gather:
    // 64 x 48 x 28 x 28 3x3 -> 96: 35 / 69 / 62; with fewer than 64 tiles of 128 x 128 the per-image matrices win:
    // 32 x 512 x 7 x 7 3x3 -> 512: 70 against 79; where the MFMA kernel applies it wins: 64 x 256 x 14 x 14 3x3 -> 256:
    // 61 against 71).  MJT_CONV_FLAT=1 sends every eligible shape this way, =0 none.
    const int64_t esz0 = dtype_size(x->dtype), NP0 = N * OH * OW, CRS0 = C * R * S;
    const bool flat_ok = G == 1 && pack_mode == 0 && esz0 == 2 && !getenv("MJT_NO_FASTPATH") && !getenv("MJT_CONV_NO_GEMM") && matmul_available() &&
                         (NP0 * esz0) % 16 == 0 && (uintptr_t)x->ptr % 16 == 0 && (uintptr_t)y->ptr % 16 == 0 && NP0 < (int64_t(1) << 31) &&
                         CRS0 * NP0 * esz0 <= (int64_t(1) << 30) && CRS0 * esz0 >= 128 && (double)N * K * OH * OW * CRS0 >= (double)(1 << 22);
    const char* flat_env = getenv("MJT_CONV_FLAT");
    const bool flat_forced = flat_ok && flat_env && atoi(flat_env) != 0;
    const bool flat = flat_forced || (flat_ok && !flat_env && OH * OW <= 256 && ((K + 127) / 128) * ((NP0 + 127) / 128) >= 64 &&
                                      ((K >= 512 && CRS0 >= 512) || (K >= 256 && CRS0 >= 2048)));
    // (a grouped convolution is one launch per group on the group's channels: worth it from 32 x 64 channels per group)
    const bool mfma_ok = !flat_forced && (x->dtype == MJT_BFLOAT16 || half) && !getenv("MJT_NO_FASTPATH") && !getenv("MJT_CONV_NO_MFMA") && C % CBLK == 0 && (Kg % 64 == 0 || Kg == 32) && G <= 64 &&
                         W % 2 == 0 && TRW >= 1 && NT <= max_px / 16 && LROWS * LCOLS * CBLK * 2 <= tile_limit &&
                         // tap shift + k-step plane offset of a fragment read must fit the 16-bit offset field
                         ((R - 1) * p->dil_h * LCOLS + (S - 1) * p->dil_w) * 16 + (CBLK == 64 ? 4 * LROWS * LCOLS * 16 : 0) < 65536 &&
                         (uintptr_t)x->ptr % 16 == 0 && (uintptr_t)y->ptr % 16 == 0 && R * S <= 49 &&
                         // byte offsets inside one image and inside the weights are 32-bit in the kernel
                         C * G * H * W * 2 < (int64_t(1) << 31) && K * OH * OW * 4 < (int64_t(1) << 31) && numel(w) * 2 < (int64_t(1) << 31) &&
                         // a 1x1 convolution of stride 1 is a matrix product per image: when the rows of a plane are 16-byte
                         // multiples the product kernel below reads x as it lies and is as fast or faster for every shape
                         // measured (64 x 512 x 28 x 28 -> 128 channels: 22 us against 42; 64 x 256 x 56 x 56 -> 64: 31 against
                         // 73; 64 x 1024 x 16 x 16 -> 2048: 82 against 387; closest 64 x 512 x 28 x 28 -> 512: 74 against 74),
                         // this kernel walking one-step channel blocks.  With other plane sizes the product kernel gathers x
                         // (its CONV mode), which wins with more than 64 output channels and enough 128 x 64 tiles for the chip
                         // (64 x 512 x 14 x 14 -> 512: 36 against 61; 64 x 1024 x 14 x 14 -> 512: 63 against 100; -> 256: 37
                         // against 142) and with many more input than output channels and few output channels or a small map
                         !(R * S == 1 && G == 1 && p->stride_h == 1 && p->stride_w == 1 && matmul_available() && !getenv("MJT_CONV_NO_GEMM") &&
                           ((p->pad_h == 0 && p->pad_w == 0 && OH == H && OW == W && (OH * OW * 2) % 16 == 0 && (uintptr_t)w->ptr % 16 == 0) ||
                            (C >= 4 * K && (K <= 64 || OH * OW <= 256)) ||
                            (K > 64 && !getenv("MJT_CONV_NO_IGEMM") && ((K + 127) / 128) * ((N * OH * OW + 63) / 64) >= 256)));
    if (mfma_ok) {
        // Rows per workgroup: a workgroup walks RPW output rows as NFULL tiles of TR rows plus one
        // shorter tile.  Pick the RPW that minimises (rounds of workgroups over the compute units) x
        // (accumulator tiles a workgroup computes, plus a per-tile overhead worth half a tile column).
        const int64_t TR = WPX * TRW, KPARTS = Kg / (16 * MT * WKO);
        const int64_t cus = c.dry_run || c.prop.multiProcessorCount <= 0 ? 256 : c.prop.multiProcessorCount;
        auto tail_of = [&](int64_t rpw, int64_t* trw_t, int64_t* nt_t) {
            const int64_t t = rpw % TR;
            *trw_t = (t + WPX - 1) / WPX;
            *nt_t = (*trw_t * OW + 15) / 16;
        };
        int64_t RPW = TR;
        {
            // Workgroups of at most four waves whose LDS is at most half a compute unit's run two to a compute unit, each
            // SIMD then holding two waves that fill each other's gaps: a pair gets through its work in 1.4 times the time
            // of one workgroup alone (64 x 64 x 56 x 56 3x3 -> 64: 256 workgroups of 14 rows 29.7 us, 448 of 8 rows 25.1,
            // 896 of 4 rows 28.4; 64 x 256 x 56 x 56 -> 64: 91.9 -> 75.9 us per call).  Such a grid pays for more, shorter
            // workgroups; a workgroup's set-up counts as one accumulator tile there, a short last tile as half a one more.
            const int64_t lds_need = 2 * LROWS * LCOLS * CBLK * 2 + 8 * (64 * 16 * MT * WKO) + 1024;
            const bool pairs = WPX * WKO <= 4 && lds_need <= lds_total / 2;
            double best = 1e300;
            for (int64_t r = TR; r <= OH || r == TR; r++) {
                int64_t trw_t, nt_t;
                tail_of(r, &trw_t, &nt_t);
                const int64_t wgs = N * ((OH + r - 1) / r) * KPARTS;
                const int64_t ntiles = r / TR + (trw_t ? 1 : 0);
                const double work = (double)(r / TR) * NT + nt_t + 0.5 * ntiles;
                double cost;
                if (pairs && wgs > cus)
                    cost = (double)((wgs + 2 * cus - 1) / (2 * cus)) * 1.4 * (work + 1.0 + (trw_t ? 0.5 : 0.0));
                else
                    cost = (double)((wgs + cus - 1) / cus) * work;
                if (cost < best - 1e-9) { best = cost; RPW = r; }
            }
            const char* e = getenv("MJT_CONV_RPW");
            if (e && *e && atoi(e) >= TR) RPW = atoi(e);
        }
        int64_t TAIL_TRW, TAIL_NT;
        tail_of(RPW, &TAIL_TRW, &TAIL_NT);
        const int64_t NFULL = RPW / TR;
        const int64_t TAIL_LROWS = TAIL_TRW ? lds_rows(TAIL_TRW) : 0;
        std::ostringstream key;
        const int64_t slab = 64 * 16 * MT * WKO;
        const int64_t spare = 1024;
        int64_t NSLAB = (lds_total - 2 * LROWS * LCOLS * CBLK * 2 - spare) / slab;
        if (NSLAB > 8) NSLAB = 8;
        MJT_CHECK(NSLAB >= 3, "conv: internal: no room for the weight ring");
        const int stage_depth = 4;                          // steps between asking for an input row and writing it to LDS (2-7: +-2 us)
        const int abl = getenv("MJT_ABLATE_CONV") ? atoi(getenv("MJT_ABLATE_CONV")) : 0;   // timing-only ablations (bench.py --ablate): results are wrong
        MJT_CHECK(abl == 0 || abl == 1 || abl == 2 || abl == 3 || abl == 7 || abl == 16 || abl == 17,
                  "conv: MJT_ABLATE_CONV must be one of 0, 1, 2, 3, 7, 16, 17");
        std::ostringstream geo_g;                        // the kernel's K_ is a group's; XC_ / YK_ are the strides of x and y between images
        geo_g << geo.str() << "#undef K_\n#define K_ " << Kg << "\n#define XC_ " << C * G << "\n#define YK_ " << K << "\n";
        key << "mfma|" << half << "|" << geo_g.str() << TRW << "|" << (y->dtype != MJT_FLOAT32) << "|" << WKO << "|" << WPX << "|" << RPW << "|" << MT << "|" << WPS
            << "|" << stage_depth << "|" << CBLK << "|" << NSLAB << "|" << abl;
        JitKernel* k = cached(key.str());
        JitKernel* kp = cached(key.str() + "|pack");
        if (!k || !kp) {
            std::ostringstream name;
            name << "mjt_conv_mfma_" << (half ? "f16" : "bf16") << "_c" << C << "_k" << Kg << (G > 1 ? "_g" + std::to_string(G) : std::string()) << "_" << H << "x" << W << "_r" << R << "x" << S << "_s"
                 << p->stride_h << "x" << p->stride_w << "_p" << p->pad_h << "x" << p->pad_w << "_d" << p->dil_h << "x"
                 << p->dil_w << "_rows" << RPW << (y->dtype == MJT_FLOAT32 ? "_of32" : half ? "_of16" : "_obf16");
            std::ostringstream src;
            src << "#define ENTRY " << name.str() << "\n#define ENTRY_PACK " << name.str() << "_pack\n" << geo_g.str()
                << "#define MT " << MT << "\n#define WKO " << WKO << "\n#define WPX " << WPX << "\n#define TRW " << TRW << "\n#define NT " << NT << "\n#define LROWS " << LROWS << "\n#define LCOLS " << LCOLS
                << "\n#define RPW " << RPW << "\n#define NFULL " << NFULL << "\n#define TAIL_TRW " << TAIL_TRW << "\n#define TAIL_NT "
                << TAIL_NT << "\n#define TAIL_LROWS " << TAIL_LROWS << "\n#define Y_BF16 " << (y->dtype != MJT_FLOAT32 ? 1 : 0) << "\n#define IN_F16 " << (half ? 1 : 0)
                << "\n#define ABL " << abl << "\n#define WPS " << WPS << "\n#define CB " << CBLK << "\n#define NS " << NSLAB << "\n#define STAGE_DEPTH " << stage_depth << "\n";
            src << embedded_source("conv_mfma.h") << "\n";
            k = jit_get(src.str(), name.str());
            kp = new JitKernel();
            kp->name = name.str() + "_pack";
            kp->module = k->module;
            if (!c.dry_run) HIP_CHECK(hipModuleGetFunction(&kp->fn, k->module, kp->name.c_str()));
            remember(key.str(), k);
            remember(key.str() + "|pack", kp);
        }
        // The kernel keeps loads and LDS reads under way in registers behind the compiler's back (it takes a spelled-out load
        // for finished when issued).  That is sound while the compiler moves no register aside; a build that needed more
        // registers than a wave has (accumulation registers beyond the accumulators, scratch memory) may have moved one
        // whose load had not landed, so such a build is not run: the convolution takes the routes below.
        const bool regs_ok = k->spilled == 0 && k->agprs >= 0 && k->agprs <= MT * NT * 4;
        if (regs_ok) {
            size_t wbytes = (size_t)numel(w) * 2;
            if (pack_mode) MJT_CHECK(packed && (uintptr_t)packed % 16 == 0, "conv: packed weights must be a 16-byte aligned device buffer");
            if (!pack_mode && !c.dry_run && wbytes > g_wpack_bytes) {
                if (g_wpack) {
                    HIP_CHECK(hipStreamSynchronize(c.stream));
                    HIP_CHECK(hipFree(g_wpack));
                }
                HIP_CHECK(hipMalloc(&g_wpack, wbytes));
                g_wpack_bytes = wbytes;
            }
            const int64_t ranges = N * ((OH + RPW - 1) / RPW);
            const int64_t ranges8 = (ranges + 7) / 8 * 8;
            const int64_t blocks = ranges8 * KPARTS;
            MJT_CHECK(blocks < (int64_t(1) << 31), "conv: launch too large");
            const int64_t wg = Kg * C * R * S;               // weights of one group
            int64_t pblocks = (wg + 255) / 256;
            if (pblocks > 2048) pblocks = 2048;
            // one launch for all groups (the group is the grid's second axis)
            char* wdst = (char*)(pack_mode ? packed : g_wpack);
            if (pack_mode != 2) {
                std::vector<uint64_t> pa{bits_of_ptr(w->ptr), bits_of_ptr(wdst), 0, 0};
                jit_launch(kp, (unsigned)pblocks, (unsigned)G, 256, 0, pa);
            }
            if (pack_mode != 1) {
                std::vector<uint64_t> a{bits_of_ptr(x->ptr), bits_of_ptr(wdst), bits_of_ptr(y->ptr), (uint64_t)N};
                jit_launch(k, (unsigned)blocks, (unsigned)G, (unsigned)(64 * WPX * WKO), 0, a);
            }
            return;
        }
    }

    if (pack_mode) MJT_FAIL(MJT_ERR_UNSUPPORTED, "conv: this convolution does not run on packed weights (mjt_conv2d_meta takes it)");

    // ---- column matrices x weights on the GEMM kernel -----------------------------------
    // What the MFMA convolution kernel does not take (float32, odd widths, channel counts that are no multiple of 64,
    // tiles that do not fit) and is large enough to matter: y[n] [K, P] = w [K, C*R*S] x cols[n] [C*R*S, P], cols = the
    // shifted input planes written by one reindex per chunk of images (a 1x1 convolution of stride 1 without padding
    // reads x itself), the product on kernels/gemm_mfma.h with the weights shared across the batch.  Rows of cols are
    // padded to a multiple of 16 bytes when the pixel count is not one (the GEMM kernel's fast path wants aligned rows).
    const int64_t P = OH * OW, CRS = C * R * S;
    if (G == 1 && !getenv("MJT_NO_FASTPATH") && !getenv("MJT_CONV_NO_GEMM") && (double)N * K * P * CRS >= (double)(1 << 22) &&
        P < (int64_t(1) << 31) && CRS < (int64_t(1) << 31) && matmul_available()) {
        const int64_t esz = dtype_size(x->dtype);
        const int64_t Ppad = (P * esz + 15) / 16 * 16 / esz;
        const bool plain = R == 1 && S == 1 && p->stride_h == 1 && p->stride_w == 1 && p->pad_h == 0 && p->pad_w == 0 && Ppad == P && OH == H && OW == W;
        auto view = [](void* ptr, int dtype, std::initializer_list<int64_t> shape) {
            mjt_tensor t;
            memset(&t, 0, sizeof(t));
            t.ptr = ptr;
            t.dtype = dtype;
            for (int64_t e : shape) t.shape[t.ndim++] = e;
            return t;
        };
        // The product's MFMA kernel wants operand rows that are 16-byte multiples at 16-byte aligned addresses.  Weight
        // rows that are not (3 x 7 x 7 float32 taps: 588 bytes) are copied into rows padded with zeros once per call.
        const void* wmat = w->ptr;
        int64_t lda = CRS;
        if ((CRS * esz) % 16 || (uintptr_t)w->ptr % 16) {
            lda = (CRS * esz + 15) / 16 * 16 / esz;
            void* wpad = conv_scratch(4, (size_t)(K * lda * esz));
            mjt_tensor tw = view(w->ptr, w->dtype, {K, CRS}), tp = view(wpad, w->dtype, {K, lda});
            const char* widx[2] = {"i0", "i1"};                 // columns past CRS lie outside w: overflow value 0
            if (mjt_reindex(&tw, &tp, 2, widx, 0.0, 0, nullptr, 0, nullptr) != MJT_OK)
                MJT_FAIL(MJT_ERR_DEVICE, "conv: padding the weight rows failed: " << mjt_last_error());
            wmat = wpad;
        }
        if (flat && !plain) {
            const int64_t osz = dtype_size(y->dtype);
            void* cols = conv_scratch(0, (size_t)(CRS * NP0 * esz));
            void* yt = conv_scratch(5, (size_t)(K * NP0 * osz));
            const std::string ih = "i4*" + std::to_string(p->stride_h) + "-" + std::to_string(p->pad_h) + "+i1*" + std::to_string(p->dil_h);
            const std::string iw = "i5*" + std::to_string(p->stride_w) + "-" + std::to_string(p->pad_w) + "+i2*" + std::to_string(p->dil_w);
            const char* cidx[4] = {"i3", "i0", ih.c_str(), iw.c_str()};
            mjt_tensor tx = view(x->ptr, x->dtype, {N, C, H, W}), tc = view(cols, x->dtype, {C, R, S, N, OH, OW});
            if (mjt_reindex(&tx, &tc, 4, cidx, 0.0, 0, nullptr, 0, nullptr) != MJT_OK)
                MJT_FAIL(MJT_ERR_DEVICE, "conv: writing the column matrices failed: " << mjt_last_error());
            gemm_launch(x->dtype, y->dtype, wmat, cols, yt, K, NP0, CRS, lda, NP0, NP0, 0, 0, 0, 1, true, false);
            const char* pidx[3] = {"i1", "i0", "i2"};
            mjt_tensor tt = view(yt, y->dtype, {K, N, P}), ty = view(y->ptr, y->dtype, {N, K, P});
            if (mjt_reindex(&tt, &ty, 3, pidx, 0.0, 0, nullptr, 0, nullptr) != MJT_OK)
                MJT_FAIL(MJT_ERR_DEVICE, "conv: rearranging the product failed: " << mjt_last_error());
            set_last_kernel("conv_as_batch_gemm");
            return;
        }
        // The product kernel gathers its second operand from x on the fly (kernels/gemm_mfma.h with CONV): no column
        // matrices.  float32 convolutions, and the 16-bit ones the MFMA convolution kernel above does not take (odd widths,
        // channel counts that are no multiple of 32 / 64, long rows).  Offsets inside x and y and the column number are
        // 32-bit there, rows and columns of the image and the reach of the taps 14-bit.
        const bool ig16 = x->dtype == MJT_BFLOAT16 || x->dtype == MJT_FLOAT16;
        const int64_t cus = c.dry_run || c.prop.multiProcessorCount <= 0 ? 256 : c.prop.multiProcessorCount;
        const int64_t NP = N * P, tiles64 = ((K + 63) / 64) * ((NP + 63) / 64);
        // (16-bit operands with a long sum and fewer 64 x 64 tiles than compute units stay on the column matrices, whose
        // product picks its tiles for a part-filled chip: 32 x 512 x 7 x 7 3x3 -> 512, 200 tiles: 102 us here, 71 there)
        const bool ig_fits = !ig16 || tiles64 >= cus || CRS <= 1024;
        if (!plain && ((x->dtype == MJT_FLOAT32 && y->dtype == MJT_FLOAT32) || ig16) && ig_fits && !getenv("MJT_CONV_NO_IGEMM") &&
            numel(x) < (int64_t(1) << 31) && numel(y) < (int64_t(1) << 31) && H < 16384 && W < 16384 &&
            (R - 1) * p->dil_h < 16384 && (S - 1) * p->dil_w < 16384 && p->pad_h < 16384 && p->pad_w < 16384 &&
            OH * p->stride_h < 16384 && OW * p->stride_w < 16384) {
            // Tile, float32: 64 output channels x 64 pixels, or 128 x 128 when there are more than 64 output channels and
            // enough tiles of that size for every compute unit.  Measured (us, tiles 64x64 / 64x128 / 128x64 / 128x128):
            // 64x64x56x56 3x3 -> 64: 202 / 244 / 381 / 365; 64x3x224x224 7x7 stride 2 -> 64: 228 / 254 / 426 / 379;
            // 64x128x28x28 3x3 -> 128: 208 / 246 / 214 / 192; 64x512x7x7 3x3 -> 512: 272 / 335 / 273 / 469.  Small tiles
            // win because four workgroups then share a compute unit: the gather's address arithmetic of one overlaps the
            // MFMAs of another.
            // 16-bit: the gather bounds the kernel and every 64 rows of output channels repeat it, so 128 x 64 when
            // such tiles fill the chip (us, 64x64 / 128x64 / 256x64 / column matrices: 64x1024x14x14 1x1 -> 256: 51 / 37 /
            // 36 / 68; 64x256x13x13 3x3 -> 384: 116 / 76 / 139 / 103; 64x64x27x27 3x3 stride 2 -> 128: 20 / 18 / 23 / 29;
            // 64x48x28x28 3x3 -> 96: 40 / 35 / 67 / 69; 64x3x224x224 7x7 stride 2 -> 64: 136 / - / - / 285).
            const bool big = !ig16 && K > 64 && ((K + 127) / 128) * ((NP + 127) / 128) >= cus;
            const bool tall = ig16 && K > 64 && ((K + 127) / 128) * ((NP + 63) / 64) >= cus;
            const int MI = big || tall ? 2 : 1, NI = big ? 2 : 1;
            const int in = x->dtype == MJT_BFLOAT16 ? 0 : x->dtype == MJT_FLOAT16 ? 1 : 2;
            const int out = y->dtype == MJT_BFLOAT16 ? 0 : y->dtype == MJT_FLOAT16 ? 1 : 2;
            std::ostringstream key;
            key << "igemm|" << geo.str() << MI << NI << in << out;
            JitKernel* k = cached(key.str());
            if (!k) {
                std::ostringstream name;
                name << "mjt_conv_igemm_" << mjt_dtype_name(x->dtype) << (y->dtype != x->dtype ? "_of32" : "") << "_c" << C << "_k" << K << "_" << H << "x" << W << "_r" << R << "x" << S << "_s" << p->stride_h << "x"
                     << p->stride_w << "_p" << p->pad_h << "x" << p->pad_w << "_d" << p->dil_h << "x" << p->dil_w << "_" << 64 * MI << "x" << 64 * NI;
                std::ostringstream src;
                src << "#define ENTRY " << name.str() << "\n#define CONV 1\n#define IN " << in << "\n#define OUT " << out << "\n#define MI " << MI << "\n#define NI " << NI
                    << "\n#define A_KCONT 1\n#define B_KCONT 0\n" << geo.str();
                src << embedded_source("gemm_mfma.h") << "\n";
                k = jit_get(src.str(), name.str());
                remember(key.str(), k);
            }
            const int64_t tiles = ((K + 64 * MI - 1) / (64 * MI)) * ((NP + 64 * NI - 1) / (64 * NI));
            const int64_t grid = (tiles + 7) / 8 * 8;
            MJT_CHECK(grid < (int64_t(1) << 31), "conv: launch too large");
            std::vector<uint64_t> a{bits_of_ptr(wmat), bits_of_ptr(x->ptr), bits_of_ptr(y->ptr), (uint64_t)K, (uint64_t)NP, (uint64_t)CRS,
                                    (uint64_t)lda, 0, 0, 0, 0, 0};
            jit_launch(k, (unsigned)grid, 1, 256, 0, a);
            return;
        }
        int64_t chunk = (int64_t(1) << 30) / (CRS * Ppad * esz);
        if (const char* e = getenv("MJT_CONV_GEMM_CHUNK"))      // images per chunk, for tests of the chunk loop
            if (atoi(e) >= 1) chunk = atoi(e);
        if (chunk < 1) chunk = 1;
        if (chunk > N) chunk = N;
        if (chunk > 65535) chunk = 65535;                       // the images of a chunk are the batch of one product launch
        void* cols = plain ? nullptr : conv_scratch(0, (size_t)(chunk * CRS * Ppad * esz));
        // index strings of the column matrices: [n, c, kh, kw, oh, ow] when a row needs no padding (the window
        // pattern of the reindex fast path), else [n, c, kh, kw, pixel] with the pixel split by division and
        // remainder and the padding marked as overflow
        std::string sh, sw, over;
        if (Ppad == P) {
            sh = "i4*" + std::to_string(p->stride_h) + "-" + std::to_string(p->pad_h) + "+i2*" + std::to_string(p->dil_h);
            sw = "i5*" + std::to_string(p->stride_w) + "-" + std::to_string(p->pad_w) + "+i3*" + std::to_string(p->dil_w);
        } else {
            sh = "i4/" + std::to_string(OW) + "*" + std::to_string(p->stride_h) + "-" + std::to_string(p->pad_h) + "+i2*" + std::to_string(p->dil_h);
            sw = "i4%" + std::to_string(OW) + "*" + std::to_string(p->stride_w) + "-" + std::to_string(p->pad_w) + "+i3*" + std::to_string(p->dil_w);
            over = "i4>=" + std::to_string(P);
        }
        const char* idx[4] = {"i0", "i1", sh.c_str(), sw.c_str()};
        const char* ovc[1] = {over.c_str()};

        for (int64_t n0 = 0; n0 < N; n0 += chunk) {
            const int64_t nb = N - n0 < chunk ? N - n0 : chunk;
            char* xn = (char*)x->ptr + n0 * C * H * W * esz;
            if (!plain) {
                mjt_tensor tx = view(xn, x->dtype, {nb, C, H, W});
                mjt_tensor tc = Ppad == P ? view(cols, x->dtype, {nb, C, R, S, OH, OW}) : view(cols, x->dtype, {nb, C, R, S, Ppad});
                if (mjt_reindex(&tx, &tc, 4, idx, 0.0, Ppad == P ? 0 : 1, ovc, 0, nullptr) != MJT_OK)
                    MJT_FAIL(MJT_ERR_DEVICE, "conv: writing the column matrices failed: " << mjt_last_error());
            }
            char* yn = (char*)y->ptr + n0 * K * P * dtype_size(y->dtype);
            // a short sum (a 1x1 convolution, few channels) is bound by how many workgroups a compute unit holds, not by
            // operand reuse: tiles of 128 x 128 (64 for at most 64 output channels or pixels, or when there would be fewer
            // tiles than compute units; at most 64 output channels with four or more 64 x 128 tiles per compute unit:
            // 64 x 64), and the direct-copy kernel from two stages of the sum on, its 256 x 256 tiles from four
            // (16-bit operands, us with / without the tile named here: 64 x 64 x 56 x 56 -> 256: 43 / 55;
            // 64 x 512 x 28 x 28 -> 64: 19 / 37; 64 x 256 x 56 x 56 -> 64: 37 / 44 with 64 x 128;
            // general kernel / direct-copy kernel on 128 x 128 tiles: 64 x 512 x 28 x 28 -> 128: 21.8 / 19.8; -> 512: 77 / 64;
            // 64 x 256 x 56 x 56 -> 128: 56 / 47; 64 x 128 x 28 x 28 -> 512: 32 / 26)
            const bool short_sum = CRS <= 1024 && esz == 2 && !getenv("MJT_CONV_GEMM_NO_HINT");
            const int64_t cus = ctx().dry_run || ctx().prop.multiProcessorCount <= 0 ? 256 : ctx().prop.multiProcessorCount;
            const bool few = ((K + 127) / 128) * ((P + 127) / 128) * nb < cus;       // tiles of 128 x 128 would leave compute units idle
            const bool many = ((P + 127) / 128) * nb >= 4 * cus;                     // plenty of 64 x 128 tiles
            const int tile_m = !short_sum ? 0 : K <= 64 || few ? 64 : 128;
            const int tile_n = !short_sum ? 0 : P <= 64 || few || (K <= 64 && many) ? 64 : 128;
            gemm_launch(x->dtype, y->dtype, wmat, plain ? (void*)xn : cols, yn, K, P, CRS, lda, Ppad, P, 0, CRS * Ppad, K * P, nb, true, false,
                        tile_m, tile_n, !short_sum || CRS >= 128);
        }
        set_last_kernel(plain ? "conv_as_gemm" : "conv_as_reindex_gemm");
        return;
    }

    // ---- direct path ----------------------------------------------------------------
    const bool idx32 = numel(x) < (int64_t(1) << 31) && numel(y) < (int64_t(1) << 31) - 256 && numel(w) < (int64_t(1) << 31);
    std::ostringstream key;
    key << "direct|" << geo.str() << x->dtype << "|" << y->dtype << "|" << G << "|" << idx32;
    JitKernel* k = cached(key.str());
    if (!k) {
        std::ostringstream name;
        name << "mjt_conv_direct_" << mjt_dtype_name(x->dtype) << "_" << mjt_dtype_name(y->dtype) << "_c" << C << "_k" << K
             << "_" << H << "x" << W << "_r" << R << "x" << S << "_s" << p->stride_h << "x" << p->stride_w << "_p" << p->pad_h
             << "x" << p->pad_w << "_d" << p->dil_h << "x" << p->dil_w;
        if (G > 1) name << "_g" << G;
        if (!idx32) name << "_i64";
        std::ostringstream src;
        src << "#define ENTRY " << name.str() << "\n#define TIN " << dtype_cname(x->dtype) << "\n#define TOUT "
            << dtype_cname(y->dtype) << "\n#define G_ " << G << "\n#define IDX " << (idx32 ? "int" : "long long")
            << "\n" << geo.str();
        src << embedded_source("prelude.h") << "\n" << embedded_source("conv_direct.h") << "\n";
        k = jit_get(src.str(), name.str());
        remember(key.str(), k);
    }
    const int64_t total = numel(y);
    const int64_t blocks = (total + 255) / 256;
    MJT_CHECK(blocks < (int64_t(1) << 31), "conv: launch too large");
    std::vector<uint64_t> a{bits_of_ptr(x->ptr), bits_of_ptr(w->ptr), bits_of_ptr(y->ptr), (uint64_t)total};
    jit_launch(k, (unsigned)blocks, 1, 256, 0, a);
}

// The buffer of per-slice partial weight gradients, grown to `bytes`.
static void* wgrad_partials(size_t bytes) {
    Context& c = ctx();
    if (c.dry_run) return (void*)(uintptr_t)0x1000;
    if (bytes > g_wgrad_bytes) {
        if (g_wgrad_part) {
            HIP_CHECK(hipStreamSynchronize(c.stream));
            HIP_CHECK(hipFree(g_wgrad_part));
            g_wgrad_part = nullptr;
            g_wgrad_bytes = 0;
        }
        HIP_CHECK(hipMalloc(&g_wgrad_part, bytes));
        g_wgrad_bytes = bytes;
    }
    return g_wgrad_part;
}

// [slices, numel(dw)] float partial sums summed over axis 0 into dw, rounded once if dw is a 16-bit type.
static void fold_wgrad_slices(void* part, int64_t slices, const mjt_tensor* dw) {
    mjt_tensor tp, td;
    memset(&tp, 0, sizeof(tp));
    memset(&td, 0, sizeof(td));
    tp.ptr = part;
    tp.dtype = MJT_FLOAT32;
    tp.ndim = 2;
    tp.shape[0] = slices;
    tp.shape[1] = numel(dw);
    td.ptr = dw->ptr;
    td.dtype = dw->dtype;
    td.ndim = 1;
    td.shape[0] = numel(dw);
    if (mjt_reduce(&tp, &td, MJT_OP_ADD, 0b01) != MJT_OK) MJT_FAIL(MJT_ERR_DEVICE, "conv wgrad: folding the partial sums failed: " << mjt_last_error());
}

// The direct weight-gradient kernel (kernels/conv_wgrad_direct.h): any groups, any geometry, float32 / bfloat16 / float16.
static void conv_wgrad_direct(const mjt_tensor* x, const mjt_tensor* dy, const mjt_tensor* dw, const mjt_conv_params* p, int64_t G) {
    const int64_t N = x->shape[0], C = x->shape[1] / G, H = x->shape[2], W = x->shape[3];
    const int64_t K = dy->shape[1], OH = dy->shape[2], OW = dy->shape[3], R = dw->shape[2], S = dw->shape[3];
    const bool flt = x->dtype == MJT_FLOAT32 || x->dtype == MJT_BFLOAT16 || x->dtype == MJT_FLOAT16;
    if (!flt || dy->dtype != x->dtype || !(dw->dtype == MJT_FLOAT32 || dw->dtype == x->dtype))
        MJT_FAIL(MJT_ERR_UNSUPPORTED, "conv wgrad: x and dy must share one of float32 / bfloat16 / float16 and dw be of that type or float32");
    MJT_CHECK(H * W < (int64_t(1) << 31) && OH * OW < (int64_t(1) << 31), "conv wgrad: image too large");
    if (N == 0 || OH * OW == 0) {                                // a sum over nothing: zeros, written by the reduce kernel
        fold_wgrad_slices(wgrad_partials(4), 0, dw);
        return;
    }
    const int64_t taps = R * S;
    const int64_t TCH = taps <= 49 ? taps : 32;
    int64_t CT = taps <= 49 ? 40 / taps : 1;
    if (CT > 4) CT = 4;
    if (CT > C) CT = C;
    if (CT < 1) CT = 1;
    const int64_t per_slice = K * ((C + CT - 1) / CT) * ((taps + TCH - 1) / TCH);
    Context& c = ctx();
    const int64_t cus = c.dry_run || c.prop.multiProcessorCount <= 0 ? 256 : c.prop.multiProcessorCount;
    // slices of whole images: about four workgroups per compute unit, at least a thousand positions per slice
    int64_t slices = (4 * cus + per_slice - 1) / per_slice;
    if (slices > N * OH * OW / 1024) slices = N * OH * OW / 1024;
    if (slices > N) slices = N;
    if (slices < 1) slices = 1;
    const int64_t ips = (N + slices - 1) / slices;
    slices = (N + ips - 1) / ips;
    MJT_CHECK(slices * per_slice < (int64_t(1) << 31), "conv wgrad: launch too large");

    std::ostringstream key;
    key << "wgrad_direct|" << x->dtype << "|" << C << "|" << H << "|" << W << "|" << K << "|" << R << "|" << S << "|" << OH << "|" << OW << "|"
        << p->stride_h << "|" << p->stride_w << "|" << p->pad_h << "|" << p->pad_w << "|" << p->dil_h << "|" << p->dil_w << "|" << G << "|" << CT;
    JitKernel* k = cached(key.str());
    if (!k) {
        std::ostringstream name;
        name << "mjt_conv_wgrad_direct_" << mjt_dtype_name(x->dtype) << "_c" << C << "_k" << K << "_" << H << "x" << W << "_r" << R << "x" << S << "_s"
             << p->stride_h << "x" << p->stride_w << "_p" << p->pad_h << "x" << p->pad_w << "_d" << p->dil_h << "x" << p->dil_w << "_g" << G;
        std::ostringstream src;
        src << "#define ENTRY " << name.str() << "\n#define TIN " << dtype_cname(x->dtype) << "\n#define C_ " << C << "\n#define H_ " << H
            << "\n#define W_ " << W << "\n#define K_ " << K << "\n#define R_ " << R << "\n#define S_ " << S << "\n#define OH_ " << OH
            << "\n#define OW_ " << OW << "\n#define SH " << p->stride_h << "\n#define SW " << p->stride_w << "\n#define PH " << p->pad_h
            << "\n#define PW " << p->pad_w << "\n#define DH " << p->dil_h << "\n#define DW " << p->dil_w << "\n#define G_ " << G
            << "\n#define CT " << CT << "\n#define TCH " << TCH << "\n";
        src << embedded_source("prelude.h") << "\n" << embedded_source("conv_wgrad_direct.h") << "\n";
        k = jit_get(src.str(), name.str());
        remember(key.str(), k);
    }
    const bool in_place = slices == 1 && dw->dtype == MJT_FLOAT32;       // one slice of float sums is the result
    void* part = in_place ? dw->ptr : wgrad_partials((size_t)slices * (size_t)numel(dw) * 4);
    std::vector<uint64_t> a{bits_of_ptr(x->ptr), bits_of_ptr(dy->ptr), bits_of_ptr(part), (uint64_t)N, (uint64_t)ips, 0};
    jit_launch(k, (unsigned)(slices * per_slice), 1, 256, 0, a);
    if (!in_place) fold_wgrad_slices(part, slices, dw);
    set_last_kernel(k->name.c_str());
}

// Weight gradient: dw[k,c,r,s] = sum_{n,oh,ow} dy[n,k,oh,ow] * x[n,c,oh*sh-ph+r*dh,ow*sw-pw+s*dw].
// With `any_shape` (the grouped entry point) what the MFMA kernel does not cover runs on the direct kernel instead of
// being handed back; G > 1: x has G groups of dw->shape[1] channels, dy G groups of K / G (python/jittor/nn.py:1272-1294).
void conv_wgrad_impl(const mjt_tensor* x, const mjt_tensor* dy, const mjt_tensor* dw, const mjt_conv_params* p, int64_t G, bool any_shape) {
    require_init();
    check_tensor(x, "conv wgrad x");
    check_tensor(dy, "conv wgrad dy");
    check_tensor(dw, "conv wgrad dw");
    MJT_CHECK(p, "conv wgrad: null parameters");
    MJT_CHECK(x->ndim == 4 && dy->ndim == 4 && dw->ndim == 4, "conv wgrad: x, dy and dw must have rank 4");
    MJT_CHECK(p->stride_h >= 1 && p->stride_w >= 1 && p->dil_h >= 1 && p->dil_w >= 1 && p->pad_h >= 0 && p->pad_w >= 0,
              "conv wgrad: bad stride / padding / dilation");
    MJT_CHECK(G >= 1, "conv wgrad: groups must be positive");
    const int64_t N = x->shape[0], H = x->shape[2], W = x->shape[3];
    const int64_t K = dy->shape[1], OH = dy->shape[2], OW = dy->shape[3];
    const int64_t R = dw->shape[2], S = dw->shape[3];
    MJT_CHECK(x->shape[1] % G == 0 && K % G == 0, "conv wgrad: " << x->shape[1] << " input and " << K << " output channels do not split into " << G << " groups");
    const int64_t C = x->shape[1] / G;                           // input channels per group
    MJT_CHECK(dy->shape[0] == N, "conv wgrad: dy has " << dy->shape[0] << " images, x " << N);
    MJT_CHECK(dw->shape[0] == K && dw->shape[1] == C, "conv wgrad: dw shape " << shape_str(dw) << " != [" << K << "," << C << ",R,S]");
    MJT_CHECK(OH == (H + 2 * p->pad_h - p->dil_h * (R - 1) - 1) / p->stride_h + 1 &&
                  OW == (W + 2 * p->pad_w - p->dil_w * (S - 1) - 1) / p->stride_w + 1,
              "conv wgrad: dy shape " << shape_str(dy) << " does not follow from x " << shape_str(x) << " and the " << R << "x" << S
                                      << " kernel");
    if (numel(dw) == 0) return;
    // what the MFMA kernel covers; anything else is for the caller's general path
    const int64_t KG = K % 256 == 0 ? 4 : K % 128 == 0 ? 2 : 1;
    const int64_t CTW = 8 / KG;
    const bool half = x->dtype == MJT_FLOAT16;
    const bool ok = G == 1 && (x->dtype == MJT_BFLOAT16 || half) && dy->dtype == x->dtype && (dw->dtype == MJT_FLOAT32 || dw->dtype == x->dtype) &&
                    p->stride_w == 1 && p->pad_w <= 2 && (S - 1) * p->dil_w - p->pad_w <= 4 && K % 64 == 0 && C % 16 == 0 && (C % (16 * CTW) == 0 || C % (16 * CTW) >= 8 * CTW) && R * S <= 9 && OW % 2 == 0 &&
                    W % 2 == 0 && N >= 1 && numel(x) * 2 < (int64_t(1) << 31) && numel(dy) * 2 < (int64_t(1) << 31) &&
                    (uintptr_t)x->ptr % 4 == 0 && (uintptr_t)dy->ptr % 16 == 0 &&
                    !getenv("MJT_NO_FASTPATH");
    if (!ok && any_shape) {
        conv_wgrad_direct(x, dy, dw, p, G);
        return;
    }
    if (!ok)
        MJT_FAIL(MJT_ERR_UNSUPPORTED, "conv wgrad: only bfloat16 or float16 operands with horizontal stride 1, column shifts of the taps within -2 .. 4, at most 9 taps, "
                                      "K % 64 == 0, C % 16 == 0 (the last block of " << 16 * CTW << " channels at least half full), even OW and tensors below 2 GB run on the MFMA kernel");
    Context& c = ctx();
    const int64_t cus = c.dry_run || c.prop.multiProcessorCount <= 0 ? 256 : c.prop.multiProcessorCount;
    const int64_t blocks_per_slice = (K / (64 * KG)) * ((C + 16 * CTW - 1) / (16 * CTW));   // the last block of channels may be partly idle
    // slices of consecutive output rows of the batch (a part of an image, or several images): enough workgroups for every
    // compute unit, at least 4 rows per slice (with whole images per slice, 64 x 64 x 56 x 56 with 3x3 taps ran 64
    // workgroups: 158 us)
    const int64_t rows = N * OH;
    int64_t slices = (cus + blocks_per_slice - 1) / blocks_per_slice;
    if (slices > (rows + 3) / 4) slices = (rows + 3) / 4;
    if (slices < 1) slices = 1;
    int64_t rps = (rows + slices - 1) / slices;
    if (const char* e = getenv("MJT_WGRAD_IPS"))             // images per slice, for experiments
        if (atoi(e) >= 1) rps = (atoi(e) < N ? atoi(e) : N) * OH;
    if (const char* e = getenv("MJT_WGRAD_RPS"))             // rows per slice, likewise
        if (atoi(e) >= 1) rps = atoi(e) < rows ? atoi(e) : rows;
    slices = (rows + rps - 1) / rps;

    const int abl = getenv("MJT_ABLATE_WGRAD") ? atoi(getenv("MJT_ABLATE_WGRAD")) : 0;    // timing-only ablations (bench.py --ablate): results are wrong
    MJT_CHECK(abl >= 0 && abl <= 63, "conv wgrad: MJT_ABLATE_WGRAD must be 0 .. 63");
    std::ostringstream key;
    key << "wgrad|" << abl << "|" << C << "|" << H << "|" << W << "|" << K << "|" << R << "|" << S << "|" << OH << "|" << OW << "|" << p->stride_h << "|"
        << p->pad_h << "|" << p->pad_w << "|" << p->dil_h << "|" << p->dil_w << "|" << KG << "|" << half;
    JitKernel* k = cached(key.str());
    if (!k) {
        std::ostringstream name;
        name << "mjt_conv_wgrad_mfma_" << (half ? "f16" : "bf16") << "_c" << C << "_k" << K << "_" << H << "x" << W << "_r" << R << "x" << S << "_s" << p->stride_h
             << "x1_p" << p->pad_h << "x" << p->pad_w << "_d" << p->dil_h << "x" << p->dil_w;
        std::ostringstream src;
        src << "#define ENTRY " << name.str() << "\n#define C_ " << C << "\n#define H_ " << H << "\n#define W_ " << W << "\n#define K_ " << K
            << "\n#define R_ " << R << "\n#define S_ " << S << "\n#define OH_ " << OH << "\n#define OW_ " << OW << "\n#define SH "
            << p->stride_h << "\n#define PH " << p->pad_h << "\n#define PW " << p->pad_w << "\n#define DH " << p->dil_h << "\n#define DW "
            << p->dil_w << "\n#define KG " << KG << "\n#define IN_F16 " << (half ? 1 : 0) << "\n#define ABL " << abl << "\n";
        src << embedded_source("conv_wgrad_mfma.h") << "\n";
        k = jit_get(src.str(), name.str());
        remember(key.str(), k);
    }
    // (as in the forward kernel: a build that had to move registers aside is not run; its accumulators are vector registers)
    if (k->spilled != 0 || k->agprs != 0) {
        if (any_shape) {
            conv_wgrad_direct(x, dy, dw, p, G);
            return;
        }
        MJT_FAIL(MJT_ERR_UNSUPPORTED, "conv wgrad: the MFMA kernel for this shape needs more registers than a wave has");
    }
    void* part = wgrad_partials((size_t)slices * (size_t)numel(dw) * 4);
    std::vector<uint64_t> a{bits_of_ptr(x->ptr), bits_of_ptr(dy->ptr), bits_of_ptr(part), (uint64_t)N, (uint64_t)rps, 0};
    jit_launch(k, (unsigned)((slices + 7) / 8 * 8 * blocks_per_slice), 1, 512, 0, a);
    fold_wgrad_slices(part, slices, dw);
    set_last_kernel(k->name.c_str());
}

}  // namespace mjt

extern "C" int mjt_conv2d_meta_wgrad(const mjt_tensor* x, const mjt_tensor* dy, const mjt_tensor* dw, const mjt_conv_params* p) {
    return mjt::guarded([&] { mjt::conv_wgrad_impl(x, dy, dw, p, 1, false); });
}

extern "C" int mjt_conv2d_meta_wgrad_grouped(const mjt_tensor* x, const mjt_tensor* dy, const mjt_tensor* dw, const mjt_conv_params* p,
                                             int groups) {
    return mjt::guarded([&] { mjt::conv_wgrad_impl(x, dy, dw, p, groups, true); });
}

namespace mjt {
// Input gradient of the convolution y = conv(x, w): dx[n,c,h,w] = sum over (k, r, s) of dy[n,k,oh,ow] * w[k,c,r,s] with
// h = oh*sh - ph + r*dh, w = ow*sw - pw + s*dw.  It is itself a convolution of dy, run on the forward kernels:
//   * stride 1: with the weights transposed and their taps flipped, padding d*(R-1) - p;
//   * a stride without dilation, H and W multiples of it: one stride-1 convolution per stride phase.  The rows
//     h = sh*i + a of dx see only the taps r = r_a + sh*u (r_a = (a + ph) % sh, u = 0 .. U_a - 1) and
//     dx[sh*i + a] = sum_u dy[i + d_a - u] * w[r_a + sh*u] with d_a = (a + ph) / sh: a convolution of dy with U_a taps
//     (flipped) and left padding U_a - 1 - d_a, likewise for columns.  No product has a zero factor; the phases
//     are written one after the other and interleaved by one reindex;
//   * otherwise: dy with sh-1 (sw-1) zeros between its rows (columns), then as for stride 1.
void conv_dgrad_impl(const mjt_tensor* dy, const mjt_tensor* w, const mjt_tensor* dx, const mjt_conv_params* p) {
    require_init();
    check_tensor(dy, "conv dgrad dy");
    check_tensor(w, "conv dgrad w");
    check_tensor(dx, "conv dgrad dx");
    MJT_CHECK(p, "conv dgrad: null parameters");
    MJT_CHECK(dy->ndim == 4 && w->ndim == 4 && dx->ndim == 4, "conv dgrad: dy, w and dx must have rank 4");
    MJT_CHECK(dy->dtype == w->dtype && (dy->dtype == MJT_BFLOAT16 || dy->dtype == MJT_FLOAT16 || dy->dtype == MJT_FLOAT32),
              "conv dgrad: dy and w must both be bfloat16, float16 or float32");
    MJT_CHECK(dx->dtype == MJT_FLOAT32 || dx->dtype == dy->dtype, "conv dgrad: dx must be float32 or the operands' dtype");
    const int64_t N = dx->shape[0], C = dx->shape[1], H = dx->shape[2], W = dx->shape[3];
    const int64_t K = w->shape[0], R = w->shape[2], S = w->shape[3];
    const int64_t sh = p->stride_h, sw = p->stride_w, ph = p->pad_h, pw = p->pad_w, dh = p->dil_h, dw = p->dil_w;
    MJT_CHECK(sh >= 1 && sw >= 1 && dh >= 1 && dw >= 1 && ph >= 0 && pw >= 0, "conv dgrad: bad stride / padding / dilation");
    MJT_CHECK(w->shape[1] == C, "conv dgrad: weight channels " << w->shape[1] << " != dx channels " << C);
    const int64_t OH = (H + 2 * ph - dh * (R - 1) - 1) / sh + 1, OW = (W + 2 * pw - dw * (S - 1) - 1) / sw + 1;
    MJT_CHECK(dy->shape[0] == N && dy->shape[1] == K && dy->shape[2] == OH && dy->shape[3] == OW,
              "conv dgrad: dy shape " << shape_str(dy) << " != [" << N << "," << K << "," << OH << "," << OW << "]");
    MJT_CHECK(dh * (R - 1) >= ph && dw * (S - 1) >= pw, "conv dgrad: padding beyond the taps' reach is not supported");
    if (N == 0 || C == 0) return;
    const int64_t esz = dtype_size(w->dtype);
    auto view = [](void* ptr, int dtype, std::initializer_list<int64_t> shape) {
        mjt_tensor t;
        memset(&t, 0, sizeof(t));
        t.ptr = ptr;
        t.dtype = dtype;
        for (int64_t e : shape) t.shape[t.ndim++] = e;
        return t;
    };
    auto reindex = [&](const mjt_tensor& src, const mjt_tensor& dst, std::initializer_list<std::string> idx, std::initializer_list<std::string> over) {
        std::vector<const char*> ip, op;
        for (const std::string& e : idx) ip.push_back(e.c_str());
        for (const std::string& e : over) op.push_back(e.c_str());
        if (mjt_reindex(&src, &dst, (int)ip.size(), ip.data(), 0.0, (int)op.size(), op.data(), 0, nullptr) != MJT_OK)
            MJT_FAIL(MJT_ERR_DEVICE, "conv dgrad: a rearrangement failed: " << mjt_last_error());
    };
    auto str = [](int64_t v) { return std::to_string(v); };
    void* wbuf = conv_scratch(2, (size_t)(numel(w) * esz));

    // the taps of each stride phase along one axis: first tap, number of taps, left padding (-1: not expressible)
    struct Phase { int64_t first, taps, pad; };
    auto phases = [](int64_t stride, int64_t pad, int64_t taps) {
        std::vector<Phase> v;
        for (int64_t a = 0; a < stride; a++) {
            Phase q;
            q.first = (a + pad) % stride;
            q.taps = q.first < taps ? (taps - q.first + stride - 1) / stride : 0;
            q.pad = q.taps ? q.taps - 1 - (a + pad) / stride : 0;
            v.push_back(q);
        }
        return v;
    };
    bool by_phase = (sh > 1 || sw > 1) && dh == 1 && dw == 1 && H % sh == 0 && W % sw == 0 && !getenv("MJT_CONV_DGRAD_NO_PHASES");
    std::vector<Phase> rows, cols;
    if (by_phase) {
        rows = phases(sh, ph, R);
        cols = phases(sw, pw, S);
        for (const Phase& q : rows) by_phase = by_phase && q.pad >= 0;
        for (const Phase& q : cols) by_phase = by_phase && q.pad >= 0;
    }
    if (by_phase) {
        const int64_t Hs = H / sh, Ws = W / sw, dsz = dtype_size(dx->dtype);
        const int64_t plane = N * C * Hs * Ws;
        char* part = (char*)conv_scratch(3, (size_t)(sh * sw * plane * dsz));
        const mjt_conv_params unit = {1, 1, 0, 0, 1, 1};
        std::string kernels;
        // The weights of all phases in one pass (the phases partition the taps): w [K,C,R,S] -> one block [C,K,U,V] per
        // phase, the phase's taps flipped, the blocks one after the other.  Seen from the flat offset i0 of that buffer,
        // block p covers [off_p, off_p + C*K*U*V) and its element (c, k, u, v) reads w[k, c, first_r + sh*(U-1-u),
        // first_c + sw*(V-1-v)]: four index expressions, each a chain of conditions on i0.
        std::vector<int64_t> woff((size_t)(sh * sw), -1);
        {
            std::string ek = "0", ec = "0", er = "0", es = "0";
            int64_t off = 0;
            std::vector<std::array<std::string, 4>> pieces;
            std::vector<int64_t> ends;
            for (int64_t a = 0; a < sh; a++)
                for (int64_t b = 0; b < sw; b++) {
                    const Phase &qr = rows[a], &qc = cols[b];
                    if (qr.taps == 0 || qc.taps == 0) continue;
                    woff[(size_t)(a * sw + b)] = off;
                    const int64_t U = qr.taps, V = qc.taps;
                    const std::string l = "(i0-" + str(off) + ")";
                    pieces.push_back({l + "/" + str(U * V) + "%" + str(K), l + "/" + str(K * U * V),
                                      str(qr.first) + "+" + str(sh) + "*(" + str(U - 1) + "-" + l + "/" + str(V) + "%" + str(U) + ")",
                                      str(qc.first) + "+" + str(sw) + "*(" + str(V - 1) + "-" + l + "%" + str(V) + ")"});
                    off += C * K * U * V;
                    ends.push_back(off);
                }
            if (!pieces.empty()) {
                std::array<std::string, 4> e = pieces.back();
                for (int i = (int)pieces.size() - 2; i >= 0; i--)
                    for (int j = 0; j < 4; j++) e[j] = "(i0<" + str(ends[i]) + " ? " + pieces[i][j] + " : " + e[j] + ")";
                mjt_tensor tall = view(wbuf, w->dtype, {off});
                reindex(*w, tall, {e[0], e[1], e[2], e[3]}, {});
            }
        }
        for (int64_t a = 0; a < sh; a++)
            for (int64_t b = 0; b < sw; b++) {
                const Phase &qr = rows[a], &qc = cols[b];
                mjt_tensor ty = view(part + (a * sw + b) * plane * dsz, dx->dtype, {N, C, Hs, Ws});
                if (qr.taps == 0 || qc.taps == 0) {                 // no tap reaches these positions: zeros
                    reindex(*dy, ty, {"0", "0", "0", "0"}, {"1"});
                    continue;
                }
                mjt_tensor tw = view((char*)wbuf + woff[(size_t)(a * sw + b)] * esz, w->dtype, {C, K, qr.taps, qc.taps});
                mjt_conv_params q = unit;
                q.pad_h = (int32_t)qr.pad;
                q.pad_w = (int32_t)qc.pad;
                conv_impl(dy, &tw, &ty, &q, 1, true);
                if (kernels.empty()) kernels = mjt_last_kernel();
            }
        mjt_tensor tp = view(part, dx->dtype, {sh * sw, N, C, Hs, Ws});
        reindex(tp, *dx, {"i2%" + str(sh) + "*" + str(sw) + "+i3%" + str(sw), "i0", "i1", "i2/" + str(sh), "i3/" + str(sw)}, {});
        set_last_kernel(("conv_dgrad_phases:" + kernels).c_str());
        return;
    }
    mjt_tensor tw = view(wbuf, w->dtype, {C, K, R, S});
    reindex(*w, tw, {"i1", "i0", str(R - 1) + "-i2", str(S - 1) + "-i3"}, {});
    const mjt_conv_params q = {1, 1, (int32_t)(dh * (R - 1) - ph), (int32_t)(dw * (S - 1) - pw), (int32_t)dh, (int32_t)dw};
    if (sh == 1 && sw == 1) {
        conv_impl(dy, &tw, dx, &q, 1);
        return;
    }
    const int64_t ZH = H + 2 * ph - dh * (R - 1), ZW = W + 2 * pw - dw * (S - 1);
    mjt_tensor tz = view(conv_scratch(3, (size_t)(N * K * ZH * ZW * esz)), dy->dtype, {N, K, ZH, ZW});
    reindex(*dy, tz, {"i0", "i1", "i2/" + str(sh), "i3/" + str(sw)}, {"i2%" + str(sh) + "!=0", "i3%" + str(sw) + "!=0"});
    conv_impl(&tz, &tw, dx, &q, 1);
}
}  // namespace mjt

extern "C" int mjt_conv2d_meta_dgrad(const mjt_tensor* dy, const mjt_tensor* w, const mjt_tensor* dx, const mjt_conv_params* p) {
    return mjt::guarded([&] { mjt::conv_dgrad_impl(dy, w, dx, p); });
}

extern "C" int mjt_conv2d_meta(const mjt_tensor* x, const mjt_tensor* w, const mjt_tensor* y, const mjt_conv_params* p) {
    return mjt::guarded([&] { mjt::conv_impl(x, w, y, p, 1); });
}

extern "C" int mjt_conv2d_meta_pack(const mjt_tensor* x, const mjt_tensor* w, const mjt_tensor* y, const mjt_conv_params* p,
                                    void* packed, size_t packed_bytes) {
    return mjt::guarded([&] {
        mjt::check_tensor(w, "conv w");
        MJT_CHECK(packed_bytes >= (size_t)mjt::numel(w) * mjt::dtype_size(w->dtype), "conv: the packed weights need as many bytes as w");
        mjt::conv_impl(x, w, y, p, 1, false, 1, packed);
    });
}

extern "C" int mjt_conv2d_meta_packed(const mjt_tensor* x, const mjt_tensor* w, const void* packed, const mjt_tensor* y,
                                      const mjt_conv_params* p) {
    return mjt::guarded([&] { mjt::conv_impl(x, w, y, p, 1, false, 2, const_cast<void*>(packed)); });
}

extern "C" int mjt_conv2d_meta_grouped(const mjt_tensor* x, const mjt_tensor* w, const mjt_tensor* y, const mjt_conv_params* p,
                                       int groups) {
    return mjt::guarded([&] { mjt::conv_impl(x, w, y, p, groups); });
}
