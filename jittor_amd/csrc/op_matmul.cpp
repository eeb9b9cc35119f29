// Matrix product behind the reference's matmul relay.
//
// The reference recognises broadcast * broadcast -> reduce.add over 2-d
// operands (opt/tuner/matmul_tuner.cc:16-104) and relays it to a library GEMM:
// cublas_matmul(a, b, trans_a, trans_b) on the GPU
// (extern/cuda/cublas/ops/cublas_matmul_op.cc:27-56, batched form
// cublas_batched_matmul_op.cc:63-85).  Here the product runs on the library's
// own kernels: kernels/gemm_mfma.h (MFMA, LDS-tiled; bfloat16, float16 and
// float32 operands whose rows are 16-byte aligned) and kernels/gemm_plain.h
// (everything else, float64 included).  Float accumulation for every input
// type (double for float64).
#include "common.h"
#include <cmath>
#include <mutex>
#include <unordered_map>

namespace mjt {

void launch_fill_pattern(void* dst, uint64_t pattern, int elem_size, size_t n);

namespace {
std::mutex g_mu;
std::unordered_map<std::string, JitKernel*> g_kernels;
void forget() {   // the kernels belong to the run-time compiler's cache, which mjt_shutdown empties
    std::lock_guard<std::mutex> lock(g_mu);
    g_kernels.clear();
}
const bool g_registered = (at_shutdown(&forget), true);

JitKernel* cached(const std::string& key) {
    std::lock_guard<std::mutex> lock(g_mu);
    auto it = g_kernels.find(key);
    return it == g_kernels.end() ? nullptr : it->second;
}
void remember(const std::string& key, JitKernel* k) {
    std::lock_guard<std::mutex> lock(g_mu);
    g_kernels.emplace(key, k);
}
int env_int(const char* name, int dflt) {
    const char* v = getenv(name);
    return v && *v ? atoi(v) : dflt;
}
}  // namespace

// One strided-batched product C[b] = A'[b] * B'[b] over plain pointers: M x K times K x N, leading dimensions and
// batch strides in elements (a batch stride of 0 shares the operand).  a_kcont / b_kcont: the operand's memory has
// k innermost (a as given, b transposed).
void gemm_launch(int in_dtype, int out_dtype, const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t K,
                 int64_t lda, int64_t ldb, int64_t ldc, int64_t sa, int64_t sb, int64_t sc, int64_t batch, bool a_kcont,
                 bool b_kcont, int tile_m = 0, int tile_n = 0, bool allow_direct = true) {
    Context& c = ctx();
    const int esz = dtype_size(in_dtype);
    const bool mfma_type = in_dtype == MJT_BFLOAT16 || in_dtype == MJT_FLOAT16 || in_dtype == MJT_FLOAT32;
    const bool out_ok = out_dtype == MJT_FLOAT32 || (out_dtype == in_dtype && esz == 2);
    auto al16 = [&](const void* p, int64_t ld, int64_t stride) {
        return (uintptr_t)p % 16 == 0 && (ld * esz) % 16 == 0 && (stride * esz) % 16 == 0;
    };
    const bool fast = mfma_type && out_ok && !getenv("MJT_GEMM_PLAIN") && al16(A, lda, sa) && al16(B, ldb, sb) &&
                      M < (int64_t(1) << 31) && N < (int64_t(1) << 31) && K < (int64_t(1) << 31) && batch < 65536;
    std::vector<uint64_t> args{bits_of_ptr(A), bits_of_ptr(B), bits_of_ptr(C), (uint64_t)M, (uint64_t)N, (uint64_t)K,
                               (uint64_t)lda, (uint64_t)ldb, (uint64_t)ldc, (uint64_t)sa, (uint64_t)sb, (uint64_t)sc};
    // 16-bit operands, K a multiple of 64 and enough tiles of 256 x 256 to go round: the kernel whose operands reach LDS
    // without passing through registers (any of the four layouts).  Offsets inside an operand's tile are 32-bit there:
    // 256 rows of an operand with k innermost, all K rows of one with m or n innermost.
    auto fits32 = [&](bool kcont, int64_t ld) { return (kcont ? ld * 2 * 256 : ld * 2 * K) < (int64_t(1) << 31); };
    if (fast && allow_direct && esz == 2 && K % 64 == 0 && !getenv("MJT_GEMM_NO_DMA") && fits32(a_kcont, lda) && fits32(b_kcont, ldb)) {
        const int64_t cus = c.dry_run || c.prop.multiProcessorCount <= 0 ? 256 : c.prop.multiProcessorCount;
        // 256 x 256 tiles on two stage buffers, or 128 x 128 tiles on a ring of four (a 128-tile's stage is a quarter of
        // the MFMA time, so more stages have to be on their way): the smaller tile where the larger one leaves compute
        // units without work
        int tile = 0;
        // a caller that names its tile has measured the general kernel against the 256 x 256 tiles; 128 x 128 tiles of this
        // kernel are still better than the general kernel's from two stages on (measured on 1x1 convolutions below)
        const bool hinted = tile_m || tile_n;
        const int smallest = hinted && !(tile_m == 128 && tile_n == 128 && K >= 128) ? 256 : 128;
        for (int t = 256; t >= smallest && !tile; t /= 2) {
            const int64_t tm = (M + t - 1) / t, tn = (N + t - 1) / t;
            const double edge = ((double)M * N) / ((double)tm * t * tn * t);
            const double tiles = (double)tm * tn * batch;
            const double util = tiles / (std::ceil(tiles / cus) * cus);
            // (a sum of fewer than four stages does not fill the time a 256 x 256 tile's operands take to arrive, and only
            // one such workgroup fits a compute unit)
            if (edge >= 0.85 && util >= (t == 256 ? 0.7 : 0.25) && (t == 128 || K >= 256)) tile = t;
        }
        if (const char* e = getenv("MJT_GEMM_DMA")) tile = atoi(e) == 128 ? 128 : 256;
        if (tile) {
            const int64_t tm = (M + tile - 1) / tile, tn = (N + tile - 1) / tile;
            const int in = in_dtype == MJT_BFLOAT16 ? 0 : 1;
            const int out = out_dtype == MJT_BFLOAT16 ? 0 : out_dtype == MJT_FLOAT16 ? 1 : 2;
            // a short sum on 128 x 128 tiles: two stage buffers, so that a compute unit holds two workgroups and one
            // computes or stores while the other waits for its operands
            // 128 x 128 tiles: with more tiles than compute units two stage buffers, so that a compute unit holds two
            // workgroups and one computes or stores while the other waits for its operands (us, ring of four / two
            // workgroups: 3072 x 3072 x 1024 35.4 / 31.7; 8192 x 1024 x 1024 26.8 / 22.1; 64 x 512 x 28 x 28 -> 512 as a
            // product 82.3 / 63.7); with at most one tile each a ring of four (2048^3 21.7 / 24.8; 1536^3 15.3 / 20.5)
            const int nbuf = tile == 256 ? 2 : (double)tm * tn * batch > (double)cus ? 2 : 4, wpe = tile == 128 && nbuf == 2 ? 2 : 1;
            std::ostringstream key;
            key << "gemmd|" << in << out << a_kcont << b_kcont << tile << nbuf;
            JitKernel* k = cached(key.str());
            if (!k) {
                std::ostringstream name;
                name << "mjt_gemm_mfma_" << mjt_dtype_name(in_dtype) << "_" << mjt_dtype_name(out_dtype) << "_" << tile << "x" << tile << (a_kcont ? "_n" : "_t")
                     << (b_kcont ? "t" : "n") << "_direct" << (wpe == 2 ? "2" : "");
                std::ostringstream src;
                src << "#define ENTRY " << name.str() << "\n#define IN " << in << "\n#define OUT " << out << "\n#define A_KCONT " << (a_kcont ? 1 : 0)
                    << "\n#define B_KCONT " << (b_kcont ? 1 : 0) << "\n#define TILE " << tile << "\n#define NBUF " << nbuf << "\n#define WPE " << wpe << "\n";
                src << embedded_source("gemm_dma.h") << "\n";
                k = jit_get(src.str(), name.str());
                remember(key.str(), k);
            }
            // (the kernel keeps LDS reads under way in registers behind the compiler's back: a build that had to move
            // registers aside, into accumulation registers beyond the tile / 256 accumulators or into scratch memory,
            // is not run; the general kernel below takes the product)
            if (k->spilled == 0 && k->agprs >= 0 && k->agprs <= tile * tile / 256) {
                const int64_t grid = (tm * tn + 7) / 8 * 8;
                MJT_CHECK(grid < (int64_t(1) << 31), "matmul: launch too large");
                jit_launch(k, (unsigned)grid, (unsigned)batch, 256, 0, args);
                return;
            }
        }
    }
    if (fast) {
        // Tile: the largest of 64 MI x 64 NI (MI, NI in 1, 2, 4) that still gives every compute unit work and wastes
        // little on the edges; larger tiles read each operand element less often.
        const int64_t cus = c.dry_run || c.prop.multiProcessorCount <= 0 ? 256 : c.prop.multiProcessorCount;
        int best_mi = 1, best_ni = 1;
        double best = -1.0;
        for (int mi = 4; mi >= 1; mi /= 2)
            for (int ni = 4; ni >= 1; ni /= 2) {
                const int64_t tm = (M + 64 * mi - 1) / (64 * mi), tn = (N + 64 * ni - 1) / (64 * ni);
                const double tiles = (double)tm * tn * batch;
                const double edge = ((double)M * N) / ((double)tm * 64 * mi * tn * 64 * ni);
                const double waves = std::ceil(tiles / cus);
                const double util = tiles / (waves * cus);
                const double reuse = 1.0 / (1.0 / (64.0 * mi) + 1.0 / (64.0 * ni)) / 128.0;   // 1 for 256 x 256
                const double score = edge * util * (0.55 + 0.45 * reuse);
                if (score > best) { best = score; best_mi = mi; best_ni = ni; }
            }
        // the caller's tile, if it names one (tile_m x tile_n of 64, 128 or 256)
        if (tile_m == 64 || tile_m == 128 || tile_m == 256) best_mi = tile_m / 64;
        if (tile_n == 64 || tile_n == 128 || tile_n == 256) best_ni = tile_n / 64;
        const int MI = best_mi, NI = best_ni;
        const int in = in_dtype == MJT_BFLOAT16 ? 0 : in_dtype == MJT_FLOAT16 ? 1 : 2;
        const int out = out_dtype == MJT_BFLOAT16 ? 0 : out_dtype == MJT_FLOAT16 ? 1 : 2;
        const bool one_stage = K <= (esz == 2 ? 64 : 32) && !getenv("MJT_GEMM_TWO_BUFFERS");       // a single stage of the kernel's k loop
        std::ostringstream key;
        key << "gemm|" << in << out << MI << NI << a_kcont << b_kcont << one_stage;
        JitKernel* k = cached(key.str());
        if (!k) {
            std::ostringstream name;
            name << "mjt_gemm_mfma_" << mjt_dtype_name(in_dtype) << "_" << mjt_dtype_name(out_dtype) << "_" << 64 * MI << "x" << 64 * NI
                 << (a_kcont ? "_n" : "_t") << (b_kcont ? "t" : "n") << (one_stage ? "_k1" : "");
            std::ostringstream src;
            src << "#define NBUF " << (one_stage ? 1 : 2) << "\n";
            src << "#define ENTRY " << name.str() << "\n#define IN " << in << "\n#define OUT " << out << "\n#define MI " << MI
                << "\n#define NI " << NI << "\n#define A_KCONT " << (a_kcont ? 1 : 0) << "\n#define B_KCONT " << (b_kcont ? 1 : 0) << "\n";
            src << embedded_source("gemm_mfma.h") << "\n";
            k = jit_get(src.str(), name.str());
            remember(key.str(), k);
        }
        const int64_t tiles = ((M + 64 * MI - 1) / (64 * MI)) * ((N + 64 * NI - 1) / (64 * NI));
        const int64_t grid = (tiles + 7) / 8 * 8;
        MJT_CHECK(grid < (int64_t(1) << 31), "matmul: launch too large");
        jit_launch(k, (unsigned)grid, (unsigned)batch, 256, 0, args);
        return;
    }
    std::ostringstream key;
    key << "gemmp|" << in_dtype << "|" << out_dtype << a_kcont << b_kcont;
    JitKernel* k = cached(key.str());
    if (!k) {
        std::ostringstream name;
        name << "mjt_gemm_plain_" << mjt_dtype_name(in_dtype) << "_" << mjt_dtype_name(out_dtype) << (a_kcont ? "_n" : "_t") << (b_kcont ? "t" : "n");
        std::ostringstream src;
        src << "#define ENTRY " << name.str() << "\n#define TIN " << dtype_cname(in_dtype) << "\n#define TOUT " << dtype_cname(out_dtype)
            << "\n#define TACC " << (in_dtype == MJT_FLOAT64 ? "double" : "float") << "\n#define A_KCONT " << (a_kcont ? 1 : 0)
            << "\n#define B_KCONT " << (b_kcont ? 1 : 0) << "\n";
        src << embedded_source("prelude.h") << "\n" << embedded_source("gemm_plain.h") << "\n";
        k = jit_get(src.str(), name.str());
        remember(key.str(), k);
    }
    MJT_CHECK(batch < 65536 && (M + 63) / 64 < 65536, "matmul: launch too large");
    set_last_kernel(k->name.c_str());
    if (c.dry_run) return;
    size_t size = args.size() * sizeof(uint64_t);
    void* config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, (void*)args.data(), HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END};
    HIP_CHECK(hipModuleLaunchKernel(k->fn, (unsigned)((N + 63) / 64), (unsigned)((M + 63) / 64), (unsigned)batch, 256, 1, 1, 0, c.stream,
                                    nullptr, config));
}

// With `share_a` every matrix of the batch is multiplied by the first matrix of a (batch stride 0: the weights of a
// convolution against the column matrices of a chunk of images).
void matmul_impl(const mjt_tensor* a, const mjt_tensor* b, const mjt_tensor* c, int trans_a, int trans_b, bool share_a) {
    require_init();
    MJT_CHECK(a && b && c, "matmul: null tensor");
    // the relay's own checks (cublas_matmul_op.cc:34-52)
    // 2-d operands, or the same leading (batch) extents on all three (cublas_batched_matmul_op.cc:63-85)
    MJT_CHECK(a->ndim >= 2 && a->ndim == b->ndim && a->ndim == c->ndim, "matmul: operands must have the same rank >= 2");
    const int nd = a->ndim;
    int64_t batch = 1;
    for (int i = 0; i < nd - 2; i++) {
        MJT_CHECK(a->shape[i] == b->shape[i] && a->shape[i] == c->shape[i], "matmul: batch extents differ at axis " << i);
        batch *= a->shape[i];
    }
    auto is_float = [](int d) { return d == MJT_FLOAT32 || d == MJT_FLOAT64 || d == MJT_FLOAT16 || d == MJT_BFLOAT16; };
    MJT_CHECK(is_float(a->dtype) && a->dtype == b->dtype, "matmul: type of two inputs should be the same (float)");
    // the result has the inputs' type; float32 is also accepted for 16-bit inputs (the sum before it is narrowed)
    MJT_CHECK(c->dtype == a->dtype || (c->dtype == MJT_FLOAT32 && dtype_size(a->dtype) == 2), "matmul: result dtype");
    int64_t n = a->shape[nd - 2], m = a->shape[nd - 1], m2 = b->shape[nd - 2], k = b->shape[nd - 1];
    if (trans_a) std::swap(n, m);
    if (trans_b) std::swap(m2, k);
    MJT_CHECK(m == m2, "matmul: inner extents " << m << " and " << m2 << " differ");
    MJT_CHECK(c->shape[nd - 2] == n && c->shape[nd - 1] == k,
              "matmul: result shape " << shape_str(c) << " does not end in [" << n << "," << k << "]");
    MJT_CHECK(n < (int64_t(1) << 31) && m < (int64_t(1) << 31) && k < (int64_t(1) << 31) && batch < (int64_t(1) << 31),
              "matmul: extent too large");
    if (batch == 0) return;
    if (n == 0 || k == 0) return;
    Context& ctxt = ctx();
    if (!ctxt.dry_run) MJT_CHECK(a->ptr && b->ptr && c->ptr, "matmul: null data");
    if (m == 0) {                                             // an empty sum
        if (!ctxt.dry_run) launch_fill_pattern(c->ptr, 0, dtype_size(c->dtype), (size_t)batch * n * k);
        return;
    }
    // c[n,k] = a'[n,m] * b'[m,k]: rows n, columns k, sum over m
    const int64_t lda = a->shape[nd - 1], ldb = b->shape[nd - 1];
    const int64_t per_launch = 65535;                         // the batch rides on a grid axis
    for (int64_t b0 = 0; b0 < batch; b0 += per_launch) {
        const int64_t nb = batch - b0 < per_launch ? batch - b0 : per_launch;
        const char* pa = (const char*)a->ptr + (share_a ? 0 : b0 * n * m * dtype_size(a->dtype));
        const char* pb = (const char*)b->ptr + b0 * m * k * dtype_size(b->dtype);
        char* pc = (char*)c->ptr + b0 * n * k * dtype_size(c->dtype);
        gemm_launch(a->dtype, c->dtype, pa, pb, pc, n, k, m, lda, ldb, k, share_a ? 0 : n * m, m * k, n * k, nb, !trans_a, trans_b != 0);
    }
}

}  // namespace mjt

extern "C" int mjt_matmul(const mjt_tensor* a, const mjt_tensor* b, const mjt_tensor* c, int trans_a, int trans_b) {
    return mjt::guarded([&] { mjt::matmul_impl(a, b, c, trans_a, trans_b, false); });
}

namespace mjt {
bool matmul_available() { return true; }
}  // namespace mjt

extern "C" int mjt_matmul_available(void) { return 1; }
