// Hand-written fast kernels behind mjt_reindex / mjt_reindex_reduce: the
// sliding-window gather (LDS-staged input tile) and the one-axis scatter
// (LDS-privatised bins).  Both are chosen from the parsed index expressions;
// anything they do not cover goes to the generic kernels.
#include "common.h"
#include "expr.h"
#include <algorithm>
#include <mutex>
#include <sstream>
#include <unordered_map>

namespace mjt {

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

// y = x with its axes in another order (every index expression is one output coordinate, each used once): tiles through
// LDS when x's innermost axis is not y's (kernels/permute_tiles.h); otherwise the generic kernel already moves runs.
bool try_permute(const mjt_tensor* x, const mjt_tensor* y, const std::vector<Affine>& aff) {
    if (getenv("MJT_NO_FASTPATH") || getenv("MJT_NO_PERMUTE")) return false;
    const int n = x->ndim;
    if (n != y->ndim || n < 2) return false;
    const int64_t esz = dtype_size(x->dtype);
    if (esz != 2 && esz != 4 && esz != 8) return false;
    // perm[d]: the output axis that indexes x's axis d
    std::vector<int> perm(n, -1);
    std::vector<bool> used(n, false);
    for (int d = 0; d < n; d++) {
        if (aff[d].c0 != 0) return false;
        for (int j = 0; j < 10; j++) {
            if (aff[d].coef[j] == 0) continue;
            if (aff[d].coef[j] != 1 || perm[d] >= 0 || j >= n || used[j]) return false;
            perm[d] = j;
            used[j] = true;
        }
        if (perm[d] < 0 || y->shape[perm[d]] != x->shape[d]) return false;
    }
    if (numel(x) < (1 << 16) || numel(x) >= (int64_t(1) << 40)) return false;
    // drop axes of extent 1; merge x axes d, d+1 that follow each other in y as well (only axes of extent 1 between them)
    std::vector<int64_t> ext;        // extents of the merged x axes
    std::vector<int> first_y, last_y;   // the output axes a merged x axis covers
    for (int d = 0; d < n; d++) {
        if (x->shape[d] == 1) continue;
        bool merge = !ext.empty() && perm[d] > last_y.back();
        for (int j = merge ? last_y.back() + 1 : 0; merge && j < perm[d]; j++) merge = y->shape[j] == 1;
        if (merge) {
            ext.back() *= x->shape[d];
            last_y.back() = perm[d];
        } else {
            ext.push_back(x->shape[d]);
            first_y.push_back(perm[d]);
            last_y.push_back(perm[d]);
        }
    }
    const int m = (int)ext.size();
    if (m < 2 || m > 6) return false;
    // order of the merged axes in y
    std::vector<int> order(m);                       // order[k]: merged x axis that is k-th in y
    for (int k = 0; k < m; k++) order[k] = k;
    std::sort(order.begin(), order.end(), [&](int a, int b) { return first_y[a] < first_y[b]; });
    std::vector<int64_t> xstr(m), ystr(m);
    {
        int64_t s = 1;
        for (int d = m - 1; d >= 0; d--) { xstr[d] = s; s *= ext[d]; }
        s = 1;
        for (int k = m - 1; k >= 0; k--) { ystr[order[k]] = s; s *= ext[order[k]]; }
    }
    const int A = m - 1, B = order[m - 1];           // x's innermost axis; the x axis that is innermost in y
    if (A == B) return false;                        // rows stay rows: nothing to transpose
    if (ext[A] < 16 || ext[B] < 16) return false;    // thin tiles: the generic kernel does as well
    std::ostringstream key;
    key << "perm|" << esz;
    for (int d = 0; d < m; d++) key << "|" << ext[d] << "," << ystr[d];
    JitKernel* k = cached(key.str());
    const int64_t TA = (ext[A] + 63) / 64, TBN = (ext[B] + 63) / 64;
    int64_t others = 1;
    if (!k) {
        std::ostringstream oe, ox, oy, name;
        int noth = 0;
        for (int d = 0; d < m; d++) {
            if (d == A || d == B) continue;
            oe << (noth ? ", " : "") << ext[d];
            ox << (noth ? ", " : "") << xstr[d];
            oy << (noth ? ", " : "") << ystr[d];
            noth++;
        }
        uint64_t h = 1469598103934665603ull;
        for (unsigned char ch : key.str()) {
            h ^= ch;
            h *= 1099511628211ull;
        }
        char buf[32];
        snprintf(buf, sizeof(buf), "%016llx", (unsigned long long)h);
        name << "mjt_permute_b" << esz << "_" << ext[B] << "x" << ext[A] << "_" << buf;
        std::ostringstream src;
        src << "#define ENTRY " << name.str() << "\n#define TB " << (esz == 4 ? "unsigned" : esz == 2 ? "unsigned short" : "unsigned long long")
            << "\n#define LA " << ext[A] << "LL\n#define LB " << ext[B] << "LL\n#define XSTR_B " << xstr[B] << "LL\n#define YSTR_A " << ystr[A]
            << "LL\n#define NOTH " << noth << "\n#define OEXT " << oe.str() << "\n#define OXS " << ox.str() << "\n#define OYS " << oy.str() << "\n";
        src << embedded_source("permute_tiles.h") << "\n";
        k = jit_get(src.str(), name.str());
        remember(key.str(), k);
    }
    for (int d = 0; d < m; d++)
        if (d != A && d != B) others *= ext[d];
    const int64_t blocks = TA * TBN * others;
    if (blocks >= (int64_t(1) << 31)) return false;
    std::vector<uint64_t> args{bits_of_ptr(x->ptr), bits_of_ptr(y->ptr), 0, 0};
    jit_launch(k, (unsigned)blocks, 1, 256, 0, args);
    return true;
}

// y[b.., oh, ow, kh, kw] = x[b.., oh*SH + kh*DH + CH, ow*SW + kw*DW + CW]
bool try_window_gather(const mjt_tensor* x, const mjt_tensor* y, const std::vector<Affine>& aff, double overflow_value) {
    if (getenv("MJT_NO_FASTPATH")) return false;
    const int XD = x->ndim, YD = y->ndim;
    if (XD < 2 || YD != XD + 2) return false;
    const int nb = XD - 2;
    int esz = dtype_size(x->dtype);
    if (esz != 4 && esz != 2 && esz != 8) return false;
    // batch axes: identity
    for (int d = 0; d < nb; d++) {
        if (aff[d].c0 != 0 || x->shape[d] != y->shape[d]) return false;
        for (int k = 0; k < YD; k++)
            if (aff[d].coef[k] != (k == d ? 1 : 0)) return false;
    }
    const int a_oh = nb, a_ow = nb + 1, a_kh = nb + 2, a_kw = nb + 3;
    const Affine& ah = aff[nb];
    const Affine& aw = aff[nb + 1];
    for (int k = 0; k < YD; k++) {
        if (k != a_oh && k != a_kh && ah.coef[k]) return false;
        if (k != a_ow && k != a_kw && aw.coef[k]) return false;
    }
    const int64_t SH = ah.coef[a_oh], DH = ah.coef[a_kh], CH = ah.c0;
    const int64_t SW = aw.coef[a_ow], DW = aw.coef[a_kw], CW = aw.c0;
    if (SH < 1 || SW < 1 || DH < 1 || DW < 1 || SH > 8 || SW > 8 || DH > 8 || DW > 8) return false;
    const int64_t H = x->shape[nb], W = x->shape[nb + 1];
    const int64_t OH = y->shape[a_oh], OW = y->shape[a_ow], KH = y->shape[a_kh], KW = y->shape[a_kw];
    if (KH * KW > 64 || KH * KW < 2 || OH < 1 || OW < 1) return false;
    if (H * W >= (int64_t(1) << 30) || OH * OW * KH * KW >= (int64_t(1) << 30)) return false;
    if (H * W * esz >= (int64_t(1) << 31) || OH * OW * KH * KW * esz >= (int64_t(1) << 31)) return false;   // byte offsets inside a plane are 31-bit
    if (std::abs(CH) > 64 || std::abs(CW) > 64) return false;
    int64_t planes = 1;
    for (int d = 0; d < nb; d++) planes *= x->shape[d];
    const int64_t rowlen = OW * KH * KW;
    int vec = 16 / esz;
    while (vec > 1 && (rowlen % vec != 0 || (uintptr_t)y->ptr % (size_t)(vec * esz) != 0)) vec /= 2;
    // rows per workgroup: aim at ~16 KB of output per workgroup (many workgroups in flight), keep the
    // lanes of the last store round busy, and start every workgroup's run of y on a vector boundary
    const int64_t LW = (OW - 1) * SW + (KW - 1) * DW + 1;
    auto tile_rows = [&](int64_t th) { return (th - 1) * SH + (KH - 1) * DH + 1; };
    const int wthreads = 256;
    int64_t TH = 0;
    double best = -1.0;
    for (int64_t th = 1; th <= OH; th++) {
        if ((th * rowlen) % vec != 0 && th != OH) continue;
        if (tile_rows(th) * LW * esz > 24 * 1024) break;       // two of them in LDS
        const int64_t nv = th * rowlen / vec;
        const double lanes = (double)nv / (double)(((nv + wthreads - 1) / wthreads) * wthreads);
        const double bytes = (double)(th * rowlen * esz);
        const double size_score = bytes < 16384.0 ? bytes / 16384.0 : 16384.0 / bytes;
        const double tail = (double)OH / (double)(((OH + th - 1) / th) * th);     // rows wasted in the last tile
        const double score = lanes * tail * (0.5 + 0.5 * size_score);
        if (score > best) { best = score; TH = th; }
    }
    if (TH == 0) return false;
    if (env_int("MJT_WINDOW_TH", 0) > 0 && env_int("MJT_WINDOW_TH", 0) <= OH) TH = env_int("MJT_WINDOW_TH", 0);
    const int64_t LH = tile_rows(TH);
    const int64_t tiles = (OH + TH - 1) / TH;
    if (planes * tiles >= (int64_t(1) << 31)) return false;
    // Tiles per workgroup.  One: consecutive tiles then go to different compute units at about the same time and the
    // output, which is most of the traffic, reaches memory as one ascending stream.  With several tiles per
    // workgroup the kernel prefetches the next tile's input behind the current tile's stores, but every workgroup
    // then writes a stream of its own and the 3x3 im2col of [32,64,56,56] is 20 % slower (55 against 45 us).
    int64_t TPW = env_int("MJT_WINDOW_TPW", 1);
    if (TPW < 1 || TPW > tiles) TPW = tiles;
    const int64_t parts = (tiles + TPW - 1) / TPW;

    // overflow value as raw bits of Tx(overflow_value); dtypes without an encoding here take the generic kernel
    // (decided before a kernel is compiled for them)
    uint64_t ovbits = 0;
    switch (x->dtype) {
        case MJT_FLOAT32: { float f = (float)overflow_value; uint32_t u; memcpy(&u, &f, 4); ovbits = u; break; }
        case MJT_FLOAT64: ovbits = bits_of(overflow_value); break;
        case MJT_BFLOAT16: { float f = (float)overflow_value; uint32_t u; memcpy(&u, &f, 4); ovbits = u >> 16; break; }
        case MJT_FLOAT16: return false;
        case MJT_INT32: case MJT_INT64: case MJT_INT16: ovbits = (uint64_t)(int64_t)overflow_value; break;
        case MJT_UINT32: case MJT_UINT64: case MJT_UINT16: ovbits = (uint64_t)overflow_value; break;
        default: return false;
    }
    if (esz < 8) ovbits &= (1ull << (8 * esz)) - 1;
    std::ostringstream key;
    key << "win|" << esz << "|" << vec << "|" << H << "," << W << "," << OH << "," << OW << "," << KH << "," << KW << ","
        << SH << "," << SW << "," << DH << "," << DW << "," << CH << "," << CW << "," << TH << "," << wthreads << "," << TPW;
    JitKernel* k = cached(key.str());
    if (!k) {
        std::ostringstream name;
        name << "mjt_window_gather_b" << esz << "_" << H << "x" << W << "_k" << KH << "x" << KW << "_s" << SH << "x" << SW
             << "_d" << DH << "x" << DW << "_o" << OH << "x" << OW << "_t" << TH << "x" << TPW;
        std::ostringstream src;
        src << "#define ENTRY " << name.str() << "\n#define TB " << (esz == 4 ? "unsigned" : esz == 2 ? "unsigned short" : "unsigned long long")
            << "\n#define VEC " << vec << "\n#define H " << H << "\n#define W " << W << "\n#define OH " << OH
            << "\n#define OW " << OW << "\n#define KH " << KH << "\n#define KW " << KW << "\n#define SH " << SH
            << "\n#define SW " << SW << "\n#define DH " << DH << "\n#define DW " << DW << "\n#define CH (" << CH
            << ")\n#define CW (" << CW << ")\n#define WTHREADS " << wthreads << "\n#define TH " << TH << "\n#define TPW " << TPW << "\n#define LH " << LH << "\n#define LW " << LW << "\n";
        src << embedded_source("prelude.h") << "\n" << embedded_source("window_gather.h") << "\n";
        k = jit_get(src.str(), name.str());
        remember(key.str(), k);
    }
    std::vector<uint64_t> args{bits_of_ptr(x->ptr), bits_of_ptr(y->ptr), ovbits, (uint64_t)planes};
    jit_launch(k, (unsigned)(planes * parts), 1, (unsigned)wthreads, 0, args);
    return true;
}

// Column matrices of a convolution: y [G, C, KH, KW, NB, OH, OW] (without the G axis: one group; without the NB axis:
// one image per group) = x [G * NB, C, H, W] read at (oh*SH + kh*DH + CH, ow*SW + kw*DW + CW), kernels/im2col_planes.h.
// Against the generic gather (us; bf16, 3x3, 64 images): 128 x 28 x 28 per image 92 -> 32; 256 x 14 x 14 in chunks of 16
// images 53 -> 21; 512 x 7 x 7, the whole batch side by side 29 -> 19.  With streaming stores the kernel itself is no
// faster and the product that reads y next loses a fifth (54.7 -> 67.8, 27.4 -> 36.7, 31.7 -> 44.5 us).
bool try_im2col_planes(const mjt_tensor* x, const mjt_tensor* y, const std::vector<Affine>& aff, double overflow_value) {
    if (getenv("MJT_NO_FASTPATH") || getenv("MJT_NO_IM2COL_PLANES")) return false;
    const int YD = y->ndim;
    if (x->ndim != 4 || (YD != 6 && YD != 7)) return false;
    const int esz = dtype_size(x->dtype);
    if (esz != 2 && esz != 4) return false;
    // which axes of y are the group, the channel, the taps, the image inside its group and the pixel
    int a_g = -1, a_c, a_kh, a_kw, a_i = -1, a_oh, a_ow;
    if (YD == 7) { a_g = 0; a_c = 1; a_kh = 2; a_kw = 3; a_i = 4; a_oh = 5; a_ow = 6; }
    else if (aff[0].coef[0] == 1) { a_g = 0; a_c = 1; a_kh = 2; a_kw = 3; a_oh = 4; a_ow = 5; }      // [N, C, KH, KW, OH, OW]
    else { a_c = 0; a_kh = 1; a_kw = 2; a_i = 3; a_oh = 4; a_ow = 5; }                                // [C, KH, KW, N, OH, OW]
    const int64_t G = a_g >= 0 ? y->shape[a_g] : 1, NB = a_i >= 0 ? y->shape[a_i] : 1, C = y->shape[a_c];
    const int64_t KH = y->shape[a_kh], KW = y->shape[a_kw], OH = y->shape[a_oh], OW = y->shape[a_ow];
    const int64_t H = x->shape[2], W = x->shape[3];
    if (x->shape[0] != G * NB || x->shape[1] != C) return false;
    // the image: NB * g + i; the channel: c; rows and columns: stride * pixel + dilation * tap + constant
    for (int k = 0; k < YD; k++) {
        if (aff[0].coef[k] != (k == a_g ? NB : k == a_i ? 1 : 0)) return false;
        if (aff[1].coef[k] != (k == a_c ? 1 : 0)) return false;
        if (k != a_oh && k != a_kh && aff[2].coef[k]) return false;
        if (k != a_ow && k != a_kw && aff[3].coef[k]) return false;
    }
    if (aff[0].c0 != 0 || aff[1].c0 != 0) return false;
    const int64_t SH = aff[2].coef[a_oh], DH = aff[2].coef[a_kh], CH = aff[2].c0;
    const int64_t SW = aff[3].coef[a_ow], DW = aff[3].coef[a_kw], CW = aff[3].c0;
    if (SH < 1 || SW < 1 || DH < 1 || DW < 1 || SH > 8 || SW > 8 || DH > 8 || DW > 8) return false;
    // (a single tap is a transposition of whole planes, which the generic kernel moves as runs: 64 x 512 x 14 x 14 as one
    // group 38 us there against 47 here for the 1x1 convolution that follows it included)
    if (std::abs(CH) > 64 || std::abs(CW) > 64 || KH * KW > 121 || KH * KW < 2 || OH < 1 || OW < 1) return false;
    const int64_t LH = (OH - 1) * SH + (KH - 1) * DH + 1, LW = (OW - 1) * SW + (KW - 1) * DW + 1;
    const int64_t P = OH * OW, run = NB * P;
    if (NB * LH * LW * esz > 48 * 1024) return false;           // the planes of a group sit in LDS together
    if (run * KH * KW >= (int64_t(1) << 31) || H * W >= (int64_t(1) << 30) || G * C >= (int64_t(1) << 31)) return false;
    int vec = 16 / esz;
    while (vec > 1 && (run % vec != 0 || (uintptr_t)y->ptr % (size_t)(vec * esz) != 0)) vec /= 2;
    // the overflow value as raw bits of x's type
    uint64_t ovbits = 0;
    switch (x->dtype) {
        case MJT_FLOAT32: { float f = (float)overflow_value; uint32_t u; memcpy(&u, &f, 4); ovbits = u; break; }
        case MJT_BFLOAT16: { float f = (float)overflow_value; uint32_t u; memcpy(&u, &f, 4); ovbits = u >> 16; break; }
        case MJT_FLOAT16: if (overflow_value != 0.0) return false; break;
        case MJT_INT32: case MJT_INT16: ovbits = (uint64_t)(int64_t)overflow_value; break;
        case MJT_UINT32: case MJT_UINT16: ovbits = (uint64_t)overflow_value; break;
        default: return false;
    }
    ovbits &= (1ull << (8 * esz)) - 1;
    const int threads = 256;
    std::ostringstream key;
    key << "i2cp|" << esz << "|" << vec << "|" << H << "," << W << "," << OH << "," << OW << "," << KH << "," << KW << "," << SH << "," << SW << ","
        << DH << "," << DW << "," << CH << "," << CW << "," << NB;
    JitKernel* k = cached(key.str());
    if (!k) {
        std::ostringstream name;
        name << "mjt_im2col_planes_b" << esz << "_" << H << "x" << W << "_k" << KH << "x" << KW << "_s" << SH << "x" << SW << "_d" << DH << "x" << DW
             << "_c" << CH << "x" << CW << "_o" << OH << "x" << OW << "_n" << NB << "_v" << vec;
        std::string nm = name.str();
        for (char& ch : nm)
            if (ch == '-') ch = 'm';
        std::ostringstream src;
        src << "#define ENTRY " << nm << "\n#define TB " << (esz == 4 ? "unsigned" : "unsigned short") << "\n#define VEC " << vec << "\n#define H " << H
            << "\n#define W " << W << "\n#define OH " << OH << "\n#define OW " << OW << "\n#define KH " << KH << "\n#define KW " << KW << "\n#define SH " << SH
            << "\n#define SW " << SW << "\n#define DH " << DH << "\n#define DW " << DW << "\n#define CH (" << CH << ")\n#define CW (" << CW
            << ")\n#define NB " << NB << "\n#define LH " << LH << "\n#define LW " << LW << "\n#define THREADS " << threads << "\n";
        src << embedded_source("prelude.h") << "\n" << embedded_source("im2col_planes.h") << "\n";
        k = jit_get(src.str(), nm);
        remember(key.str(), k);
    }
    std::vector<uint64_t> args{bits_of_ptr(x->ptr), bits_of_ptr(y->ptr), ovbits, (uint64_t)C};
    jit_launch(k, (unsigned)(G * C), 1, (unsigned)threads, 0, args);
    return true;
}

// x[idx[i]] = OP(x[idx[i]], y[i]); fills x with the identity first.
void launch_fill_pattern(void* dst, uint64_t pattern, int elem_size, size_t n);

bool try_scatter_1d(const mjt_tensor* y, const mjt_tensor* x, int op, const mjt_tensor* index) {
    if (getenv("MJT_NO_FASTPATH")) return false;
    int mode = op == MJT_OP_ADD ? 0 : op == MJT_OP_MAXIMUM ? 1 : op == MJT_OP_MINIMUM ? 2 : -1;
    if (mode < 0) return false;
    if (x->dtype != MJT_FLOAT32 && x->dtype != MJT_INT32 && x->dtype != MJT_UINT32) return false;
    if (index->dtype != MJT_INT32 && index->dtype != MJT_INT64) return false;
    if (x->ndim != 1 || y->ndim != 1) return false;
    const int64_t n = numel(y), bins = numel(x);
    if (bins >= (int64_t(1) << 31) || n >= (int64_t(1) << 36)) return false;
    if ((uintptr_t)y->ptr % 16 || (uintptr_t)index->ptr % 32 || (uintptr_t)x->ptr % 4) return false;
    Context& c = ctx();
    int logw = 14;                                            // 16384 bins: 64 KB (128 KB for float sums) of LDS per private copy
    while (logw > 8 && (int64_t(1) << (logw - 1)) >= bins) logw--;
    const int64_t W = int64_t(1) << logw;
    const int64_t NB = (bins + W - 1) / W;
    const int nthreads = 1024;
    if (NB > 512) return false;                               // per-bucket tables live in LDS, one loading thread per bucket
    int64_t nbmax = 1;
    while (nbmax < NB) nbmax *= 2;
    // Measured on the 2^24 -> 2^20 Zipf(1.1) scatter; every neighbouring value was slower.  list entries per list
    // item of the tail pass: 16384 -> 23 us, 24576 -> 17.5, 32768 -> 18.3, 40960 -> 22 (tail pass); loads in flight
    // per thread there: 8 (16 and 24 spill registers); threads of a main workgroup that only append to the lists:
    // 64 -> 48 us, 128 -> 41, 256 -> 40 (main pass); elements per thread and round: 4 -> 44-48 us, 8 -> 40.
    const int64_t cold_target = 24576;
    const int ldepth = 8, mdepth = 8;
    const int ept = 8, nflush = 256;
    const int abl = env_int("MJT_ABLATE_SCATTER", 0);      // timing-only ablations (bench.py --ablate): results are wrong
    const int acc64 = mode == 0 && x->dtype == MJT_FLOAT32;  // float sums in double: the one fast float atomic of the LDS
    // staging entries: what the private copy and the per-bucket table leave of the 160 KB of LDS, in two areas
    const int64_t lds_left = 160 * 1024 - 1024 - W * (acc64 ? 8 : 4) - (nbmax + 1) * 4;
    int64_t scap = lds_left / 16 / 64 * 64;
    if (scap > 4096) scap = 4096;
    if (scap < 64 || scap * 16 > lds_left) return false;
    // identity
    uint32_t ident = 0;
    if (mode) {
        if (x->dtype == MJT_FLOAT32) ident = mode == 1 ? 0xff7fffffu : 0x7f7fffffu;
        else if (x->dtype == MJT_INT32) ident = mode == 1 ? 0x80000000u : 0x7fffffffu;
        else ident = mode == 1 ? 0u : 0xffffffffu;
    }
    // geometry of the main pass
    int64_t G1 = (int64_t)c.prop.multiProcessorCount;
    if (G1 > 512) G1 = 512;
    const int64_t chunk = (int64_t)nthreads * 4;
    const int64_t per = ((n + G1 - 1) / G1 + chunk - 1) / chunk * chunk;
    G1 = n ? (n + per - 1) / per : 1;
    // items of the tail pass: at most one list item per bucket plus population / cold_target, and the merge items
    // (bins of a bucket / 256 per bucket that was some main workgroup's hot one)
    const int64_t mseg = W < 256 ? 1 : W / 256;
    const int64_t tail_items = NB + n / cold_target + 1 + (NB < G1 ? NB : G1) * mseg;
    int64_t tail_wgs = (int64_t)c.prop.multiProcessorCount;   // one per compute unit (by its LDS)
    if (tail_wgs > tail_items) tail_wgs = tail_items;
    // A list holds four times its share of a uniformly spread input, plus 512 bytes: all workgroups append to
    // the lists of one bucket at about the same position, and lists that lie a power of two apart (32 KB for
    // 2^24 elements into 2^20 bins) put those appends into the same memory channels (main pass 40 instead of 44 us).
    // Three times the share is as fast, twice overflows the Zipf head's lists (tail pass 37 us), eight times spreads
    // the appends over 1 GB and the main pass takes 59 us.
    int64_t CAP = NB > 1 ? (4 * per / NB + 63) / 64 * 64 + 64 : 64;
    if (CAP > per) CAP = (per + 63) / 64 * 64;

    std::ostringstream key;
    key << "sc1|" << x->dtype << "|" << index->dtype << "|" << mode << "|" << logw << "|" << nbmax << "|" << nthreads << "|" << nflush << "|" << ept
        << "|" << scap << "|" << cold_target << "|" << acc64 << "|" << (bins % W == 0) << "|" << abl << "|" << ldepth << "|" << mdepth;
    static const char* parts[] = {"main", "tail", "reset"};
    JitKernel* ks[3];
    bool have = true;
    for (int i = 0; i < 3; i++) have = (ks[i] = cached(key.str() + "|" + parts[i])) != nullptr && have;
    if (!have) {
        std::ostringstream name;
        name << "mjt_scatter1d_" << mjt_op_name(op) << "_" << mjt_dtype_name(x->dtype) << "_" << mjt_dtype_name(index->dtype)
             << "_w" << W << "_b" << nbmax << "_e" << ept << "_s" << scap;
        std::ostringstream src;
        src << "#define ENTRY_MAIN " << name.str() << "_main\n#define ENTRY_TAIL " << name.str() << "_tail\n#define ENTRY_RESET "
            << name.str() << "_reset\n#define LDEPTH " << ldepth << "\n#define MDEPTH " << mdepth << "\n#define ABL " << abl << "\n#define COLD_TARGET " << cold_target
            << "u\n#define TX " << dtype_cname(x->dtype) << "\n#define TE " << dtype_cname(index->dtype) << "\n#define WBINS "
            << W << "\n#define LOGW " << logw << "\n#define NBMAX " << nbmax << "\n#define NTHREADS " << nthreads
            << "\n#define EXACT_BINS " << (bins % W == 0 ? 1 : 0) << "\n#define NFLUSH " << nflush << "\n#define EPT " << ept << "\n#define SCAP " << scap << "\n#define ACC64 " << acc64
            << "\n#define MODE " << mode << "\n#define IDENT_BITS " << ident << "u\n";
        src << embedded_source("prelude.h") << "\n" << embedded_source("scatter1d.h") << "\n";
        JitKernel* first = jit_get(src.str(), name.str() + "_main");
        for (int i = 0; i < 3; i++) {
            JitKernel* k = i == 0 ? first : new JitKernel();
            if (i) {
                k->name = name.str() + "_" + parts[i];
                k->module = first->module;
                if (!c.dry_run) HIP_CHECK(hipModuleGetFunction(&k->fn, first->module, k->name.c_str()));
            }
            ks[i] = k;
            remember(key.str() + "|" + parts[i], k);
        }
    }
    // scratch layout
    auto align = [](size_t v) { return (v + 255) / 256 * 256; };
    const size_t off_hotof = 0;
    const size_t off_novf = off_hotof + align((size_t)G1 * 4);
    const size_t off_counts = off_novf + align((size_t)G1 * 4);
    const size_t off_pmain = off_counts + align((size_t)G1 * NB * 4);
    const size_t off_lists = off_pmain + align((size_t)G1 * W * 4);
    const size_t off_ovf = off_lists + align(NB > 1 ? (size_t)G1 * NB * CAP * 8 : 0);
    const size_t off_dbg = off_ovf + align(NB > 1 ? (size_t)G1 * per * 8 : 0);
    const size_t total = off_dbg + ((abl & 256) ? 512 * 64 : 0);
    // about 40 bytes of scratch per input element: when that is more than a sixteenth of the device's memory, or
    // the arena cannot grow, the generic kernel (global atomics, no scratch) takes the call
    if (!c.dry_run && total > c.prop.totalGlobalMem / 16) return false;
    char* base;
    try {
        base = (char*)scratch(total);
    } catch (const Error&) {
        (void)hipGetLastError();
        return false;
    }
    // The main pass writes the identity into x beside its stream (each workgroup a slice); with few main
    // workgroups and many bins that would take longer than the stream, and a launch of its own fills x.
    const bool fill_in_main = bins <= G1 * 65536;
    // ks[0]->state: [0] calls completed with this code object (its parity names the tally set of the next call),
    // [1] 1 when both tally sets are known to be zero or about to be cleared by a tail pass that was launched
    JitKernel* owner = ks[0];
    std::vector<uint64_t> a{bits_of_ptr(x->ptr), bits_of_ptr(y->ptr), bits_of_ptr(index->ptr), (uint64_t)n, (uint64_t)bins,
                            (uint64_t)(fill_in_main ? 1 : 0), (uint64_t)per, (uint64_t)G1, (uint64_t)NB, (uint64_t)CAP,
                            bits_of_ptr(base + off_counts), bits_of_ptr(base + off_lists), bits_of_ptr(base + off_pmain),
                            owner->state[0] & 1, bits_of_ptr(base + off_hotof), bits_of_ptr(base + off_ovf),
                            bits_of_ptr(base + off_novf), bits_of_ptr(base + off_dbg), 0, 0};
    if (!owner->state[1]) jit_launch(ks[2], 1, 1, (unsigned)nthreads, 0, a);
    owner->state[1] = 0;                                      // until the tail pass of this call is under way
    if (!fill_in_main) launch_fill_pattern(x->ptr, ident, 4, (size_t)bins);
    jit_launch(ks[0], (unsigned)G1, 1, (unsigned)nthreads, 0, a);
    jit_launch(ks[1], (unsigned)tail_wgs, 1, (unsigned)nthreads, 0, a);
    owner->state[0]++;
    owner->state[1] = 1;
    if ((abl & 256) && !c.dry_run && owner->state[0] == 30) {   // development only: when each tail workgroup did what
        HIP_CHECK(hipStreamSynchronize(c.stream));
        std::vector<uint64_t> d((size_t)tail_wgs * 8);
        HIP_CHECK(hipMemcpy(d.data(), base + off_dbg, d.size() * 8, hipMemcpyDeviceToHost));
        uint64_t t0 = ~0ull;
        for (int64_t i = 0; i < tail_wgs; i++) t0 = std::min(t0, d[i * 8]);
        for (int64_t i = 0; i < tail_wgs; i++)
            fprintf(stderr, "tailwg %3d kind %d start %6.2f plan %6.2f lists %6.2f end %6.2f xcc %d hwid %08x\n", (int)i, (int)d[i * 8 + 3],
                    (d[i * 8] - t0) * 0.01, (d[i * 8 + 1] - t0) * 0.01, d[i * 8 + 4] ? (d[i * 8 + 4] - t0) * 0.01 : 0.0, (d[i * 8 + 2] - t0) * 0.01,
                    (int)d[i * 8 + 5], (unsigned)d[i * 8 + 6]);
    }
    return true;
}

}  // namespace mjt
