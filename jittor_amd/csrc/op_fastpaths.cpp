// Hand-written fast kernels behind mjt_reindex / mjt_reindex_reduce: the
// sliding-window gather (LDS-staged input tile) and the one-axis scatter
// (LDS-privatised bins).  Both are chosen from the parsed index expressions;
// anything they do not cover goes to the generic kernels.
#include "common.h"
#include "expr.h"
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
int env_int(const char* name, int dflt) {
    const char* v = getenv(name);
    return v && *v ? atoi(v) : dflt;
}
}  // namespace

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
    if (std::abs(CH) > 64 || std::abs(CW) > 64) return false;
    int64_t planes = 1;
    for (int d = 0; d < nb; d++) planes *= x->shape[d];
    const int64_t rowlen = OW * KH * KW;
    int vec = 16 / esz;
    while (vec > 1 && (rowlen % vec != 0 || (uintptr_t)y->ptr % (size_t)(vec * esz) != 0)) vec /= 2;
    // rows per workgroup: LDS tile <= 24 KB, and at least ~4 workgroups per CU when possible
    const int64_t LW = (OW - 1) * SW + (KW - 1) * DW + 1;
    int64_t TH = OH;
    auto tile_rows = [&](int64_t th) { return (th - 1) * SH + (KH - 1) * DH + 1; };
    while (TH > 1 && tile_rows(TH) * LW * esz > 24 * 1024) TH = (TH + 1) / 2;
    if (tile_rows(TH) * LW * esz > 48 * 1024) return false;
    const int64_t cu = ctx().prop.multiProcessorCount;
    while (TH > 4 && planes * ((OH + TH - 1) / TH) < cu * 4) TH = (TH + 1) / 2;
    // a workgroup's run of y must start on a vector boundary
    while (TH < OH && (TH * rowlen) % vec != 0) TH++;
    const int64_t LH = tile_rows(TH);
    const int64_t tiles = (OH + TH - 1) / TH;
    if (planes * tiles >= (int64_t(1) << 31)) return false;

    std::ostringstream key;
    key << "win|" << esz << "|" << vec << "|" << H << "," << W << "," << OH << "," << OW << "," << KH << "," << KW << ","
        << SH << "," << SW << "," << DH << "," << DW << "," << CH << "," << CW << "," << TH;
    JitKernel* k = cached(key.str());
    if (!k) {
        std::ostringstream name;
        name << "mjt_window_gather_b" << esz << "_" << H << "x" << W << "_k" << KH << "x" << KW << "_s" << SH << "x" << SW
             << "_d" << DH << "x" << DW << "_o" << OH << "x" << OW << "_t" << TH;
        std::ostringstream src;
        src << "#define ENTRY " << name.str() << "\n#define TB " << (esz == 4 ? "unsigned" : esz == 2 ? "unsigned short" : "unsigned long long")
            << "\n#define VEC " << vec << "\n#define H " << H << "\n#define W " << W << "\n#define OH " << OH
            << "\n#define OW " << OW << "\n#define KH " << KH << "\n#define KW " << KW << "\n#define SH " << SH
            << "\n#define SW " << SW << "\n#define DH " << DH << "\n#define DW " << DW << "\n#define CH (" << CH
            << ")\n#define CW (" << CW << ")\n#define TH " << TH << "\n#define LH " << LH << "\n#define LW " << LW << "\n";
        src << embedded_source("prelude.h") << "\n" << embedded_source("window_gather.h") << "\n";
        k = jit_get(src.str(), name.str());
        remember(key.str(), k);
    }
    // overflow value as raw bits of Tx(overflow_value)
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
    std::vector<uint64_t> args{bits_of_ptr(x->ptr), bits_of_ptr(y->ptr), ovbits, (uint64_t)planes};
    jit_launch(k, (unsigned)(planes * tiles), 1, 256, 0, args);
    return true;
}

// x[idx[i]] = OP(x[idx[i]], y[i]); fills x with the identity first.
void launch_fill_pattern(void* dst, uint64_t pattern, int elem_size, size_t n);

static void* g_lo = nullptr;   // device int: start of the privatised window

bool try_scatter_1d(const mjt_tensor* y, const mjt_tensor* x, int op, const mjt_tensor* index) {
    if (getenv("MJT_NO_FASTPATH")) return false;
    int mode = op == MJT_OP_ADD ? 0 : op == MJT_OP_MAXIMUM ? 1 : op == MJT_OP_MINIMUM ? 2 : -1;
    if (mode < 0) return false;
    if (x->dtype != MJT_FLOAT32 && x->dtype != MJT_INT32 && x->dtype != MJT_UINT32) return false;
    if (index->dtype != MJT_INT32 && index->dtype != MJT_INT64) return false;
    if (x->ndim != 1 || y->ndim != 1) return false;
    const int64_t n = numel(y), bins = numel(x);
    if (bins >= (int64_t(1) << 31)) return false;
    if ((uintptr_t)y->ptr % 16 || (uintptr_t)index->ptr % 32) return false;
    Context& c = ctx();
    int wbins = env_int("MJT_SCATTER_WBINS", 16384);
    while (wbins > 256 && wbins / 2 >= bins) wbins /= 2;
    int nthreads = env_int("MJT_SCATTER_THREADS", 1024);
    int per_cu = env_int("MJT_SCATTER_WG_PER_CU", 2);
    // identity
    uint32_t ident = 0;
    if (mode) {
        if (x->dtype == MJT_FLOAT32) ident = mode == 1 ? 0xff7fffffu : 0x7f7fffffu;
        else if (x->dtype == MJT_INT32) ident = mode == 1 ? 0x80000000u : 0x7fffffffu;
        else ident = mode == 1 ? 0u : 0xffffffffu;
    }
    std::ostringstream key;
    key << "sc1|" << x->dtype << "|" << index->dtype << "|" << mode << "|" << wbins << "|" << nthreads;
    JitKernel* k = cached(key.str());
    JitKernel* ks = cached(key.str() + "|sample");
    if (!k || !ks) {
        std::ostringstream name;
        name << "mjt_scatter1d_" << mjt_op_name(op) << "_" << mjt_dtype_name(x->dtype) << "_" << mjt_dtype_name(index->dtype)
             << "_w" << wbins << "_t" << nthreads;
        std::ostringstream src;
        src << "#define ENTRY " << name.str() << "\n#define ENTRY_SAMPLE " << name.str() << "_sample\n#define TX "
            << dtype_cname(x->dtype) << "\n#define TE " << dtype_cname(index->dtype) << "\n#define WBINS " << wbins
            << "\n#define NTHREADS " << nthreads << "\n#define MODE " << mode << "\n#define IDENT_BITS " << ident << "u\n";
        src << embedded_source("prelude.h") << "\n" << embedded_source("atomics.h") << "\n" << embedded_source("scatter1d.h")
            << "\n";
        k = jit_get(src.str(), name.str());
        // second entry point of the same module
        ks = new JitKernel();
        ks->name = name.str() + "_sample";
        ks->module = k->module;
        if (!c.dry_run) HIP_CHECK(hipModuleGetFunction(&ks->fn, k->module, ks->name.c_str()));
        remember(key.str(), k);
        remember(key.str() + "|sample", ks);
    }
    if (!g_lo && !c.dry_run) {
        HIP_CHECK(hipMalloc(&g_lo, 256));
    }
    launch_fill_pattern(x->ptr, ident, 4, (size_t)bins);
    int64_t groups = (int64_t)c.prop.multiProcessorCount * per_cu;
    int64_t chunk = (int64_t)nthreads * 4;
    int64_t per = ((n + groups - 1) / groups + chunk - 1) / chunk * chunk;
    groups = (n + per - 1) / per;
    std::vector<uint64_t> args{bits_of_ptr(x->ptr), bits_of_ptr(y->ptr), bits_of_ptr(index->ptr), (uint64_t)n,
                               (uint64_t)bins,      bits_of_ptr(g_lo),   (uint64_t)per,            0};
    if (bins > wbins) {
        jit_launch(ks, 1, 1, 1024, 0, args);
    } else {
        launch_fill_pattern(g_lo, 0, 4, 1);
    }
    jit_launch(k, (unsigned)groups, 1, (unsigned)nthreads, 0, args);
    return true;
}

}  // namespace mjt
