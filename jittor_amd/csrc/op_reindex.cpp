// mjt_reindex / mjt_reindex_reduce: host side of the gather and scatter ops
// (reference: python/jittor/src/ops/reindex_op.cc:82-139,
// python/jittor/src/ops/reindex_reduce_op.cc:65-131).
//
// Index strings are parsed once per distinct op description (the role of the
// reference's jit key, ops/reindex_op.cc:93-108) and kept in a plan: the
// parsed expressions, their affine form when they have one, and the kernel
// that was specialised for them.  A plan first tries the hand-written fast
// kernels (sliding-window gather, one-axis scatter with LDS-privatised bins)
// and otherwise uses the generic kernel with the expressions pasted in.
#include "common.h"
#include <functional>
#include "expr.h"
#include <mutex>
#include <unordered_map>

namespace mjt {

// fast paths, aot_kernels.hip
bool try_window_gather(const mjt_tensor* x, const mjt_tensor* y, const std::vector<Affine>& aff, double overflow_value);
bool try_permute(const mjt_tensor* x, const mjt_tensor* y, const std::vector<Affine>& aff);
bool try_im2col_planes(const mjt_tensor* x, const mjt_tensor* y, const std::vector<Affine>& aff, double overflow_value);
bool try_scatter_1d(const mjt_tensor* y, const mjt_tensor* x, int op, const mjt_tensor* index);
void launch_fill_pattern(void* dst, uint64_t pattern, int elem_size, size_t n);

namespace {

struct Plan {
    std::vector<std::unique_ptr<Expr>> idx, ofc;
    bool all_affine = false;      // every index is affine and there are no overflow conditions / extras
    bool plain_e0 = false;        // scatter: indexes == ["@e0(i0)"] style one-axis lookup of a 1-d extra
    std::unordered_map<std::string, JitKernel*> kernels;   // by (vec, use64)
};

std::mutex g_mu;
std::unordered_map<std::string, std::unique_ptr<Plan>> g_plans;
void forget() {   // plans hold kernels of the run-time compiler's cache, which mjt_shutdown empties
    std::lock_guard<std::mutex> lock(g_mu);
    g_plans.clear();
}
const bool g_registered = (at_shutdown(&forget), true);

std::string plan_key(bool scatter, int op, const mjt_tensor* x, const mjt_tensor* y, int n_idx, const char* const* idx,
                     int n_ofc, const char* const* ofc, int n_ex, const mjt_tensor* ex) {
    std::string k;
    k.reserve(256);
    k += scatter ? "S" : "G";
    k += std::to_string(op) + "|" + std::to_string(x->dtype) + "|" + std::to_string(x->ndim) + "|" + std::to_string(y->ndim);
    for (int i = 0; i < n_idx; i++) {
        k += "\x1f";
        k += idx[i];
    }
    k += "\x1e";
    for (int i = 0; i < n_ofc; i++) {
        k += "\x1f";
        k += ofc[i];
    }
    k += "\x1e";
    for (int i = 0; i < n_ex; i++) k += std::to_string(ex[i].dtype) + ":" + std::to_string(ex[i].ndim) + ",";
    return k;
}

Plan* get_plan(const std::string& key, const mjt_tensor* x, const mjt_tensor* y, int loop_rank, int n_idx,
               const char* const* idx, int n_ofc, const char* const* ofc, int n_ex, const mjt_tensor* ex) {
    std::lock_guard<std::mutex> lock(g_mu);
    auto it = g_plans.find(key);
    if (it != g_plans.end()) return it->second.get();
    auto plan = std::make_unique<Plan>();
    ExprEnv env;
    env.n_loop = loop_rank;
    env.xdim = x->ndim;
    env.ydim = y->ndim;
    for (int i = 0; i < n_ex; i++) env.extra_rank.push_back(ex[i].ndim);
    bool pure = n_ofc == 0;
    for (int i = 0; i < n_idx; i++) {
        MJT_CHECK(idx[i], "null index expression");
        plan->idx.push_back(parse_expr(idx[i]));
        validate_expr(*plan->idx.back(), env);
        pure = pure && is_pure(*plan->idx.back());
    }
    for (int i = 0; i < n_ofc; i++) {
        MJT_CHECK(ofc[i], "null overflow condition");
        plan->ofc.push_back(parse_expr(ofc[i]));
        validate_expr(*plan->ofc.back(), env);
    }
    plan->all_affine = pure;
    if (n_idx == 1 && n_ofc == 0 && n_ex >= 1 && ex[0].ndim == 1 && loop_rank == 1) {
        const Expr& e = *plan->idx[0];
        plan->plain_e0 = e.kind == Expr::EXTRA && e.extra == 0 && e.kids.size() == 1 && e.kids[0]->kind == Expr::VAR &&
                         e.kids[0]->text == "i0";
    }
    Plan* raw = plan.get();
    g_plans.emplace(key, std::move(plan));
    return raw;
}

int pick_vec(int elem_size, int64_t last, const void* p) {
    int vec = std::min(8, 16 / elem_size);
    while (vec > 1 && (last % vec != 0 || ((uintptr_t)p % (size_t)(vec * elem_size)) != 0)) vec /= 2;
    return vec;
}

// Specialises (once per plan and variant) and launches the generic kernel.
// An element-wise prologue of a scatter: the parameter words it needs, a key, and the macro definitions
// (SC_PROLOGUE 1, MJT_SC_SCALARS, MJT_SC_VALUE) given the index of its first parameter word.
struct ScatterPrologue {
    std::vector<uint64_t> args;
    std::string key;
    std::function<std::string(int)> defs;
};

// With z: the gather is fused with a reduce (rop) over y's last nred axes; y then only gives the loop shape.
// With sp (scatter only): y's values are computed by the prologue, y gives the loop shape and dtype.
void run_generic(Plan* plan, bool scatter, int op, const mjt_tensor* x, const mjt_tensor* y, double overflow_value,
                 int n_ex, const mjt_tensor* ex, const mjt_tensor* z = nullptr, int rop = 0, int nred = 0,
                 const ScatterPrologue* sp = nullptr) {
    // the loop runs over y (gather output / scatter input)
    const int LD = y->ndim, XD = x->ndim;
    int64_t yn = numel(y), xn = numel(x);
    if (yn == 0) return;
    int64_t biggest = std::max(xn, yn);
    for (int i = 0; i < n_ex; i++) biggest = std::max(biggest, numel(&ex[i]));
    bool use64 = biggest >= (int64_t(1) << 31);   // index_t rule of op.cc:158-192
    int vec = z || sp ? 1 : pick_vec(dtype_size(x->dtype), y->shape[LD - 1], y->ptr);
    // a gather into rows that do not divide into 16-byte vectors (a padded or cropped innermost axis) still stores 16 bytes
    // per lane when y as a whole does: the kernel then decodes every element by itself
    bool flat = false;
    if (!z && !sp && !scatter && xn > 0 && vec * dtype_size(x->dtype) < 16 && !getenv("MJT_REINDEX_NO_FLAT")) {
        const int fv = std::min(8, 16 / dtype_size(x->dtype));
        if (yn % fv == 0 && (uintptr_t)y->ptr % 16 == 0) {
            vec = fv;
            flat = true;
        }
    }
    int64_t rtail = 1;
    for (int i = LD - nred; z && i < LD; i++) rtail *= y->shape[i];

    // parameter block: a[0] x, a[1] y, a[2] nvec, a[3] overflow value,
    // then yshape[LD], ydiv[LD], xshape[XD], per extra: pointer, shape[rank]
    std::vector<uint64_t> args{bits_of_ptr(x->ptr), bits_of_ptr(z ? z->ptr : y->ptr), (uint64_t)(z ? yn / rtail : yn / vec),
                               bits_of(overflow_value)};
    int p_ys = (int)args.size();
    for (int i = 0; i < LD; i++) args.push_back((uint64_t)y->shape[i]);
    int p_yd = (int)args.size();
    for (int i = 0; i < LD; i++) args.push_back(pack_divmod((uint64_t)y->shape[i]));
    int p_xs = (int)args.size();
    for (int i = 0; i < XD; i++) args.push_back((uint64_t)x->shape[i]);
    std::vector<int> p_ex(n_ex);
    for (int k = 0; k < n_ex; k++) {
        p_ex[k] = (int)args.size();
        args.push_back(bits_of_ptr(ex[k].ptr));
        for (int i = 0; i < ex[k].ndim; i++) args.push_back((uint64_t)ex[k].shape[i]);
    }

    int p_tail = 0;
    if (z) {
        p_tail = (int)args.size();
        args.push_back((uint64_t)rtail);
        args.push_back(bits_of(rtail ? 1.0 / (double)rtail : 0.0));
    }
    int p_sp = 0;
    if (sp) {
        p_sp = (int)args.size();
        args.insert(args.end(), sp->args.begin(), sp->args.end());
    }
    // a short tail (a pooling window) is unrolled, the folded extents are literals in the kernel; window rows of 4 to 8
    // elements are loaded as vectors where a wave finds them all in range and adjacent (8 x 8 mean over [64,128,64,64]:
    // 59 -> 22.5 us; rows of 2 or 3 gain nothing: 25.9 against 25.7 us for 2 x 2, and with padding nearly every wave has a
    // lane at the border).  One output per lane:
    // with 2 / 4 / 8 adjacent outputs per lane a 2 x 2 maximum over [64,128,64,64] took 36 / 65 / 79 us against 27
    // (neighbouring lanes then read further apart)
    const int rt_c = z && rtail <= 64 && xn > 0 && !getenv("MJT_GATHER_REDUCE_LOOP") ? (int)rtail : 0;
    const int ov = 1;
    std::string vkey = std::to_string(vec) + (use64 ? "L" : "I") + (flat ? "F" : "") + (xn > 0 ? "" : "E");
    if (sp) vkey += "|P" + sp->key;
    if (z) {
        vkey += "|R" + std::to_string(rop) + "," + std::to_string(z->dtype) + "," + std::to_string(nred) + "," + std::to_string(rt_c) + "," + std::to_string(ov);
        for (int i = LD - nred; i < LD; i++) vkey += "," + std::to_string(y->shape[i]);
    }
    JitKernel* kern = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_mu);
        auto it = plan->kernels.find(vkey);
        if (it != plan->kernels.end()) kern = it->second;
    }
    if (!kern) {
        const char* IT = use64 ? "long long" : "int";
        std::ostringstream setup, dec, index;
        setup << "const index_t XDIM = " << XD << "; const index_t YDIM = " << LD << "; (void)XDIM; (void)YDIM; ";
        auto shapes = [&](const char* n, int rank, int base) {
            for (int i = 0; i < rank; i++)
                setup << "const index_t " << n << "shape" << i << " = (index_t)(unsigned long long)p.a[" << base + i << "]; (void)" << n
                      << "shape" << i << "; ";
            setup << "const index_t " << n << "stride" << rank - 1 << " = 1; (void)" << n << "stride" << rank - 1 << "; ";
            for (int i = rank - 2; i >= 0; i--)
                setup << "const index_t " << n << "stride" << i << " = " << n << "stride" << i + 1 << " * " << n << "shape"
                      << i + 1 << "; (void)" << n << "stride" << i << "; ";
        };
        shapes("y", LD, p_ys);
        shapes("x", XD, p_xs);
        for (int k = 0; k < n_ex; k++) {
            std::string n = "e" + std::to_string(k);
            setup << "const " << dtype_cname(ex[k].dtype) << "* __restrict__ " << n << "p = (const "
                  << dtype_cname(ex[k].dtype) << "*)p.a[" << p_ex[k] << "]; (void)" << n << "p; ";
            shapes(n.c_str(), ex[k].ndim, p_ex[k] + 1);
        }
        dec << IT << " rem_ = e; ";
        for (int a = LD - 1; a >= 0; a--) {
            std::string cname = a == LD - 1 ? std::string("ilast_") : "i" + std::to_string(a);
            if (a == 0) {
                dec << "const " << IT << " " << cname << " = rem_; ";
            } else if (use64) {
                dec << "const " << IT << " q" << a << "_ = rem_ / yshape" << a << "; const " << IT << " " << cname
                    << " = rem_ - q" << a << "_ * yshape" << a << "; rem_ = q" << a << "_; ";
            } else {
                dec << "const int q" << a << "_ = (int)mjt_div((unsigned)rem_, mjt_unpack_divmod((unsigned long long)p.a[" << p_yd + a
                    << "], 0)); const int " << cname << " = rem_ - q" << a << "_ * yshape" << a << "; rem_ = q" << a
                    << "_; ";
            }
            if (a != LD - 1) dec << "(void)" << cname << "; ";
        }
        // the same coordinates for a gather that folds its last nred axes: the kept ones from the output's offset o_, the
        // folded ones from the tail offset r
        std::ostringstream dec_kept, dec_tail;
        if (z) {
            dec_kept << IT << " rem_ = o_; (void)rem_; ";
            for (int a = LD - nred - 1; a >= 0; a--) {
                if (a == 0) {
                    dec_kept << "const " << IT << " i0 = rem_; ";
                } else if (use64) {
                    dec_kept << "const " << IT << " q" << a << "_ = rem_ / yshape" << a << "; const " << IT << " i" << a
                             << " = rem_ - q" << a << "_ * yshape" << a << "; rem_ = q" << a << "_; ";
                } else {
                    dec_kept << "const int q" << a << "_ = (int)mjt_div((unsigned)rem_, mjt_unpack_divmod((unsigned long long)p.a["
                             << p_yd + a << "], 0)); const int i" << a << " = rem_ - q" << a << "_ * yshape" << a << "; rem_ = q" << a
                             << "_; ";
                }
                dec_kept << "(void)i" << a << "; ";
            }
            dec_tail << IT << " rt_ = r; (void)rt_; ";
            for (int a = LD - 1; a >= LD - nred; a--) {
                if (a == LD - nred) dec_tail << "const " << IT << " i" << a << " = rt_; ";
                else dec_tail << "const " << IT << " i" << a << " = rt_ % " << y->shape[a] << "; rt_ /= " << y->shape[a] << "; ";
                dec_tail << "(void)i" << a << "; ";
            }
        }
        for (int dd = 0; dd < XD; dd++)
            index << "const index_t xid" << dd << " = (index_t)(" << emit_c(*plan->idx[dd]) << "); ";
        index << "const index_t xid = 0";
        for (int dd = 0; dd < XD; dd++) index << " + xid" << dd << " * xstride" << dd;
        // combined without short-circuit evaluation: that would put a branch between the loads of a lane's elements
        index << "; bool ov_ = false";
        for (int dd = 0; dd < XD; dd++) index << " | (xid" << dd << " < 0) | (xid" << dd << " >= xshape" << dd << ")";
        for (auto& c : plan->ofc) index << " | (bool)(" << emit_c(*c) << ")";
        index << "; ";

        std::ostringstream frag;
        frag << "#define TX " << dtype_cname(x->dtype) << "\n#define index_t " << IT << "\n#define VEC " << vec
             << "\n#define NPARAM " << args.size() << "\n#define SCATTER " << (scatter ? 1 : 0) << "\n";
        frag << "#define MJT_RX_LASTVAR i" << LD - 1 << "\n";
        frag << "#define MJT_RX_SETUP " << setup.str() << "\n";
        frag << "#define MJT_RX_DECODE " << dec.str() << "\n";
        if (z)
            frag << "#define MJT_RX_DECODE_KEPT " << dec_kept.str() << "\n#define MJT_RX_DECODE_TAIL " << dec_tail.str()
                 << "\n#define RTAIL_C " << rt_c << "\n#define OV " << ov << "\n#define TAIL_IN "
                 << (rt_c && y->shape[LD - 1] >= 4 && y->shape[LD - 1] <= 8 && !getenv("MJT_GATHER_REDUCE_NO_RUNS") ? y->shape[LD - 1] : 1) << "\n";
        frag << "#define MJT_RX_INDEX " << index.str() << "\n";
        if (scatter) frag << "#define ATOMIC_UPDATE(addr, v) mjt_atomic_" << mjt_op_name(op) << "<TX>((addr), (v))\n";
        frag << "#define REDUCE_TAIL " << (z ? 1 : 0) << "\n#define FLAT_VEC " << (flat ? 1 : 0) << "\n#define SAFE_LOAD "
             << (xn > 0 ? 1 : 0) << "\n";
        if (sp) frag << sp->defs(p_sp);
        else frag << "#define SC_PROLOGUE 0\n";
        if (z) {
            // accumulator as in the reduce kernels: z's type, float for 16-bit float results
            const int ta = z->dtype == MJT_FLOAT16 || z->dtype == MJT_BFLOAT16 ? MJT_FLOAT32 : z->dtype;
            const std::string opn = rop == MJT_OP_MEAN ? "add" : mjt_op_name(rop);
            frag << "#define TZ " << dtype_cname(z->dtype) << "\n#define TACC " << dtype_cname(ta) << "\n#define P_RTAIL " << p_tail
                 << "\n#define P_RCOUNT " << p_tail + 1 << "\n#define INIT mjt_init_" << opn << "<TACC>()\n";
            if (rop == MJT_OP_MEAN) frag << "#define COMBINE(a, x) ((a) + TACC(x) * TACC(rcount))\n";
            else frag << "#define COMBINE(a, x) mjt_" << opn << "<TACC>((a), (x))\n";
        }
        uint64_t h = 1469598103934665603ull;
        for (unsigned char ch : frag.str()) {
            h ^= ch;
            h *= 1099511628211ull;
        }
        char name[96];
        snprintf(name, sizeof(name), "mjt_%s_%016llx",
                 scatter ? (std::string("reindex_reduce_") + mjt_op_name(op)).c_str()
                         : z ? (std::string("reindex_then_") + mjt_op_name(rop)).c_str() : "reindex",
                 (unsigned long long)h);
        std::string src = std::string("#define ENTRY ") + name + "\n" + frag.str() + embedded_source("prelude.h") + "\n" +
                          (scatter ? std::string(embedded_source("atomics.h")) + "\n" : std::string()) +
                          embedded_source("reindex.h") + "\n";
        kern = jit_get(src, name);
        std::lock_guard<std::mutex> lock(g_mu);
        plan->kernels.emplace(vkey, kern);
    }
    int64_t nvec = z ? (yn / rtail + ov - 1) / ov : yn / vec;
    int64_t blocks = (nvec + 255) / 256;
    MJT_CHECK(blocks < (int64_t(1) << 31), "reindex: launch too large");
    jit_launch(kern, (unsigned)blocks, 1, 256, 0, args);
}

// A scatter through a window pattern (x[b.., oh*SH + kh*DH + CH, ow*SW + kw*DW + CW] op= y[b.., oh, ow, kh, kw], no
// overflow conditions, no extras: the gradient of pooling) runs as a gather over x: every element of x folds the windows
// that reach it (kernels/window_scatter.h) -- no atomic updates, no identity fill.  Measured on the gradient of a 3x3
// stride-2 maximum pooling of [64,64,112,112] float32: 1042 us of queued atomic adds (plus 20 us of fill) against 139 us.  Returns false when the pattern is another one; the caller then fills and scatters.
bool try_window_scatter(Plan* plan, int op, const mjt_tensor* x, const mjt_tensor* y, int n_ofc, int n_ex, const ScatterPrologue* sp) {
    if (getenv("MJT_NO_FASTPATH") || getenv("MJT_NO_WINDOW_SCATTER")) return false;
    if (n_ofc != 0 || n_ex != 0 || !plan->all_affine) return false;
    if (op != MJT_OP_ADD && op != MJT_OP_MAXIMUM && op != MJT_OP_MINIMUM && op != MJT_OP_MULTIPLY) return false;
    if (x->dtype == MJT_BOOL) return false;
    const int XD = x->ndim, YD = y->ndim, nb = XD - 2;
    if (XD < 2 || YD != XD + 2) return false;
    if (numel(x) == 0 || numel(y) == 0) return false;
    std::vector<int64_t> xs(x->shape, x->shape + XD), ys(y->shape, y->shape + YD);
    std::vector<Affine> aff(XD);
    for (int i = 0; i < XD; i++)
        if (!affine_of(*plan->idx[i], xs, ys, &aff[i])) return false;
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
    const int64_t SH = ah.coef[a_oh], DH = ah.coef[a_kh], CH = ah.c0, SW = aw.coef[a_ow], DW = aw.coef[a_kw], CW = aw.c0;
    if (SH < 1 || SW < 1 || DH < 1 || DW < 1 || SH > 8 || SW > 8 || DH > 8 || DW > 8) return false;
    if (CH < -64 || CH > 64 || CW < -64 || CW > 64) return false;
    const int64_t KH = y->shape[a_kh], KW = y->shape[a_kw];
    if (KH < 1 || KW < 1 || KH * KW > 64) return false;
    const int64_t NCH = (KH - 1) * DH / SH + 1, NCW = (KW - 1) * DW / SW + 1;
    if (NCH * NCW > 16) return false;

    int64_t biggest = std::max(numel(x), numel(y));
    const bool use64 = biggest >= (int64_t(1) << 31);
    const int64_t xn = numel(x);
    std::vector<uint64_t> args{bits_of_ptr(x->ptr), bits_of_ptr(y->ptr), (uint64_t)xn, 0};
    const int p_ys = (int)args.size();
    for (int i = 0; i < YD; i++) args.push_back((uint64_t)y->shape[i]);
    const int p_xs = (int)args.size();
    for (int i = 0; i < XD; i++) args.push_back((uint64_t)x->shape[i]);
    const int p_sp = (int)args.size();
    if (sp) args.insert(args.end(), sp->args.begin(), sp->args.end());

    // elements of a row of x per lane: one 16-byte store when the rows and the pointer allow it
    int wvec = std::min(8, 16 / dtype_size(x->dtype));
    while (wvec > 1 && (x->shape[XD - 1] % wvec != 0 || (uintptr_t)x->ptr % (size_t)(wvec * dtype_size(x->dtype)) != 0)) wvec /= 2;
    while (wvec > 1 && NCH * NCW * wvec > 32) wvec /= 2;                  // at most 32 candidate windows per lane
    // without a prologue the candidates are loads from y itself, far apart for neighbouring elements of x: more of them
    // per lane coalesce worse (3x3 stride-2 windows into [64,64,112,112]: 230 us with four elements per lane, 175 with one)
    if (!sp) wvec = 1;
    std::ostringstream vk;
    vk << "WS" << op << (use64 ? "L" : "I") << wvec << "|" << SH << "," << SW << "," << DH << "," << DW << "," << CH << "," << CW << "," << KH << "," << KW;
    for (int i = 0; i < XD; i++) vk << "," << x->shape[i];
    vk << "," << y->shape[a_oh] << "," << y->shape[a_ow];
    if (sp) vk << "|P" << sp->key;
    const std::string vkey = vk.str();
    JitKernel* kern = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_mu);
        auto it = plan->kernels.find(vkey);
        if (it != plan->kernels.end()) kern = it->second;
    }
    if (!kern) {
        const char* IT = use64 ? "long long" : "int";
        std::ostringstream setup, batch;
        setup << "const index_t XDIM = " << XD << "; const index_t YDIM = " << YD << "; (void)XDIM; (void)YDIM; ";
        auto shapes = [&](const char* n, int rank, int base) {
            for (int i = 0; i < rank; i++)
                setup << "const index_t " << n << "shape" << i << " = (index_t)(unsigned long long)p.a[" << base + i << "]; (void)" << n
                      << "shape" << i << "; ";
            setup << "const index_t " << n << "stride" << rank - 1 << " = 1; (void)" << n << "stride" << rank - 1 << "; ";
            for (int i = rank - 2; i >= 0; i--)
                setup << "const index_t " << n << "stride" << i << " = " << n << "stride" << i + 1 << " * " << n << "shape"
                      << i + 1 << "; (void)" << n << "stride" << i << "; ";
        };
        shapes("y", YD, p_ys);
        shapes("x", XD, p_xs);
        batch << IT << " rem_ = plane_; (void)rem_; ";
        for (int a = nb - 1; a >= 0; a--) {
            if (a == 0) batch << "const " << IT << " i0 = rem_; ";
            else batch << "const " << IT << " i" << a << " = rem_ % " << x->shape[a] << "; rem_ /= " << x->shape[a] << "; ";
            batch << "(void)i" << a << "; ";
        }
        const int ta = x->dtype == MJT_FLOAT16 || x->dtype == MJT_BFLOAT16 ? MJT_FLOAT32 : x->dtype;
        std::ostringstream frag;
        frag << "#define TX " << dtype_cname(x->dtype) << "\n#define TACC " << dtype_cname(ta) << "\n#define index_t " << IT << "\n#define VEC " << wvec
             << "\n#define NPARAM " << args.size() << "\n#define NB " << nb << "\n#define KH " << KH << "\n#define KW " << KW << "\n#define SH " << SH << "\n#define SW " << SW
             << "\n#define DH " << DH << "\n#define DW " << DW << "\n#define CH " << CH << "\n#define CW " << CW << "\n#define NCH " << NCH
             << "\n#define NCW " << NCW << "\n";
        // extents as literals: the lane's coordinates come from divisions by them
        frag << "#define xshape_h " << x->shape[nb] << "\n#define xshape_w " << x->shape[nb + 1] << "\n#define yshape_oh " << y->shape[a_oh]
             << "\n#define yshape_ow " << y->shape[a_ow] << "\n";
        frag << "#define I_OH i" << a_oh << "\n#define I_OW i" << a_ow << "\n#define I_KH i" << a_kh << "\n#define I_KW i" << a_kw << "\n";
        frag << "#define MJT_RX_SETUP " << setup.str() << "\n#define MJT_WS_BATCH " << batch.str() << "\n";
        frag << "#define INIT mjt_init_" << mjt_op_name(op) << "<TACC>()\n#define COMBINE(a, v) mjt_" << mjt_op_name(op) << "<TACC>((a), (v))\n";
        if (sp) frag << sp->defs(p_sp);
        else frag << "#define SC_PROLOGUE 0\n";
        uint64_t h = 1469598103934665603ull;
        for (unsigned char ch : frag.str()) {
            h ^= ch;
            h *= 1099511628211ull;
        }
        char name[96];
        snprintf(name, sizeof(name), "mjt_window_scatter_%s_%016llx", mjt_op_name(op), (unsigned long long)h);
        std::string src = std::string("#define ENTRY ") + name + "\n" + frag.str() + embedded_source("prelude.h") + "\n" +
                          embedded_source("window_scatter.h") + "\n";
        kern = jit_get(src, name);
        std::lock_guard<std::mutex> lock(g_mu);
        plan->kernels.emplace(vkey, kern);
    }
    const int64_t blocks = (xn / wvec + 255) / 256;
    if (blocks >= (int64_t(1) << 31)) return false;
    jit_launch(kern, (unsigned)blocks, 1, 256, 0, args);
    return true;
}

void check_extras(int n_ex, const mjt_tensor* ex) {
    MJT_CHECK(n_ex >= 0 && n_ex <= 16, "too many extras");
    MJT_CHECK(n_ex == 0 || ex, "null extras");
    for (int i = 0; i < n_ex; i++) check_tensor(&ex[i], "extras");
}

// bit pattern of init_OP for dtype (type/common_op_type.cc:116-117,142-151;
// 16-bit floats: type/fp16_op_type.cc:111-112)
uint64_t identity_bits(int op, int dtype) {
    auto fbits = [&](double v) -> uint64_t {
        if (dtype == MJT_FLOAT64) return bits_of(v);
        float f = (float)v;
        uint32_t u;
        memcpy(&u, &f, 4);
        if (dtype == MJT_FLOAT32) return u;
        if (dtype == MJT_BFLOAT16) return u >> 16;
        // float16: only 0, 1 and +-32768 are needed
        if (v == 0) return 0;
        if (v == 1) return 0x3c00;
        return v > 0 ? 0x7800 : 0xf800;
    };
    bool fl = dtype_is_float(dtype);
    int sz = dtype_size(dtype);
    uint64_t ones = sz == 8 ? ~0ull : ((1ull << (8 * sz)) - 1);
    switch (op) {
        case MJT_OP_MULTIPLY: return fl ? fbits(1.0) : 1;
        case MJT_OP_MAXIMUM:
            if (dtype == MJT_FLOAT32) return fbits(-3.402823466e+38);
            if (dtype == MJT_FLOAT64) return fbits(-1.7976931348623157e+308);
            if (fl) return fbits(-32768.0);
            if (dtype == MJT_BOOL || dtype_is_unsigned(dtype)) return 0;
            return 1ull << (8 * sz - 1);
        case MJT_OP_MINIMUM:
            if (dtype == MJT_FLOAT32) return fbits(3.402823466e+38);
            if (dtype == MJT_FLOAT64) return fbits(1.7976931348623157e+308);
            if (fl) return fbits(32768.0);
            if (dtype == MJT_BOOL) return 1;
            if (dtype_is_unsigned(dtype)) return ones;
            return ones >> 1;
        case MJT_OP_LOGICAL_AND: return fl ? fbits(1.0) : 1;
        case MJT_OP_BITWISE_AND: return dtype == MJT_BOOL ? 1 : (fl ? fbits(-1.0) : ones);
        default: return 0;   // add, subtract, void, logical_or/xor, bitwise_or/xor and the rest start from 0
    }
}

}  // namespace

void reindex_impl(const mjt_tensor* x, const mjt_tensor* y, int n_idx, const char* const* idx, double overflow_value,
                  int n_ofc, const char* const* ofc, int n_ex, const mjt_tensor* ex) {
    require_init();
    check_tensor(x, "reindex x");
    check_tensor(y, "reindex y");
    check_extras(n_ex, ex);
    MJT_CHECK(n_idx == x->ndim, "Number of x's shape and indexes should be the same. (x rank " << x->ndim << ", "
                                                                                             << n_idx << " indexes)");
    MJT_CHECK(n_idx == 0 || idx, "null indexes");
    MJT_CHECK(n_ofc >= 0 && (n_ofc == 0 || ofc), "null overflow conditions");
    MJT_CHECK(x->dtype == y->dtype, "reindex: y dtype must equal x dtype");
    std::string key = plan_key(false, 0, x, y, n_idx, idx, n_ofc, ofc, n_ex, ex);
    Plan* plan = get_plan(key, x, y, y->ndim, n_idx, idx, n_ofc, ofc, n_ex, ex);
    if (numel(y) == 0) return;
    if (plan->all_affine && numel(x) > 0) {
        std::vector<int64_t> xs(x->shape, x->shape + x->ndim), ys(y->shape, y->shape + y->ndim);
        std::vector<Affine> aff(n_idx);
        bool ok = true;
        for (int i = 0; i < n_idx && ok; i++) ok = affine_of(*plan->idx[i], xs, ys, &aff[i]);
        if (ok && n_ofc == 0 && try_permute(x, y, aff)) return;
        if (ok && try_window_gather(x, y, aff, overflow_value)) return;
        if (ok && try_im2col_planes(x, y, aff, overflow_value)) return;
    }
    run_generic(plan, false, 0, x, y, overflow_value, n_ex, ex);
}

// reduce(reindex(x), rop) over the last nred axes of the reindex result, whose shape yshape gives (its pointer is unused)
void reindex_then_reduce_impl(const mjt_tensor* x, const mjt_tensor* yshape, const mjt_tensor* z, int rop, int nred, int n_idx,
                              const char* const* idx, double overflow_value, int n_ofc, const char* const* ofc, int n_ex,
                              const mjt_tensor* ex) {
    require_init();
    check_tensor(x, "reindex_then_reduce x");
    check_tensor(z, "reindex_then_reduce z");
    check_extras(n_ex, ex);
    MJT_CHECK(yshape && yshape->ndim >= 1 && yshape->ndim <= MJT_MAX_DIM, "reindex_then_reduce: bad loop shape");
    MJT_CHECK(n_idx == x->ndim, "Number of x's shape and indexes should be the same. (x rank " << x->ndim << ", " << n_idx << " indexes)");
    MJT_CHECK(n_idx == 0 || idx, "null indexes");
    MJT_CHECK(n_ofc >= 0 && (n_ofc == 0 || ofc), "null overflow conditions");
    MJT_CHECK(nred >= 1 && nred <= yshape->ndim, "reindex_then_reduce: " << nred << " reduced axes of " << yshape->ndim);
    MJT_CHECK(rop == MJT_OP_ADD || rop == MJT_OP_MEAN || rop == MJT_OP_MAXIMUM || rop == MJT_OP_MINIMUM || rop == MJT_OP_MULTIPLY,
              "reindex_then_reduce: op must be add, mean, maximum, minimum or multiply");
    MJT_CHECK(z->dtype != MJT_BOOL, "reindex_then_reduce: accumulator dtype bool is not supported");
    int64_t kept = 1;
    for (int i = 0; i < yshape->ndim - nred; i++) kept *= yshape->shape[i];
    MJT_CHECK(numel(z) == kept, "reindex_then_reduce: z has " << numel(z) << " elements, the kept axes give " << kept);
    if (kept == 0) return;
    if (numel(yshape) == 0) {                         // nothing folds into z: every element is the identity
        launch_fill_pattern(z->ptr, identity_bits(rop == MJT_OP_MEAN ? MJT_OP_ADD : rop, z->dtype), dtype_size(z->dtype), (size_t)kept);
        return;
    }
    mjt_tensor y = *yshape;
    y.dtype = x->dtype;
    y.ptr = z->ptr;                                   // never dereferenced: only its shape is used
    std::string key = plan_key(false, 0, x, &y, n_idx, idx, n_ofc, ofc, n_ex, ex);
    Plan* plan = get_plan(key, x, &y, y.ndim, n_idx, idx, n_ofc, ofc, n_ex, ex);
    run_generic(plan, false, 0, x, &y, overflow_value, n_ex, ex, z, rop, nred);
}

// reindex_reduce whose input is computed by an element-wise group (desc: the group over y's shape, one output var)
void fused_reindex_reduce_impl(const mjt_fused_desc* d, const mjt_tensor* x, int op, int n_idx, const char* const* idx, int n_ofc,
                               const char* const* ofc, int n_ex, const mjt_tensor* ex) {
    require_init();
    check_tensor(x, "fused reindex_reduce x");
    check_extras(n_ex, ex);
    std::vector<int> inputs;
    fused_validate(d, &inputs, false, true);
    int out = -1;
    for (int i = 0; i < d->n_vars; i++)
        if (d->vars[i].role == MJT_VAR_OUTPUT) {
            MJT_CHECK(out < 0, "fused reindex_reduce: the group must have exactly one output var (the scattered values)");
            out = i;
        }
    MJT_CHECK(out >= 0, "fused reindex_reduce: the group has no output var");
    MJT_CHECK((op >= MJT_OP_POW && op < MJT_OP_MEAN) || op == MJT_OP_VOID,
              "reindex_reduce: op must be a binary op other than mean, or void");
    MJT_CHECK(n_idx == x->ndim, "Number of shape and indexes should be the same. (shape rank " << x->ndim << ", " << n_idx << " indexes)");
    MJT_CHECK(n_idx == 0 || idx, "null indexes");
    MJT_CHECK(n_ofc >= 0 && (n_ofc == 0 || ofc), "null overflow conditions");
    MJT_CHECK(d->vars[out].dtype == x->dtype, "fused reindex_reduce: x dtype must equal the group's output dtype");
    mjt_tensor y{};                                   // the virtual scatter input
    y.ptr = x->ptr;                                   // never dereferenced
    y.dtype = x->dtype;
    y.ndim = d->ndim;
    for (int i = 0; i < d->ndim; i++) y.shape[i] = d->shape[i];
    std::string key = plan_key(true, op, x, &y, n_idx, idx, n_ofc, ofc, n_ex, ex);
    Plan* plan = get_plan(key, x, &y, y.ndim, n_idx, idx, n_ofc, ofc, n_ex, ex);
    const int64_t xn = numel(x);
    if (xn == 0) return;

    ScatterPrologue sp;
    std::ostringstream key2;
    std::vector<int> slot(d->n_vars, -1);
    for (int i = 0; i < d->n_vars; i++) {
        const mjt_fused_var& fv = d->vars[i];
        key2 << fv.role << ":" << fv.dtype << ":" << fv.bcast_mask << ";";
        if (fv.role == MJT_VAR_INPUT || fv.role == MJT_VAR_GATHERED) {
            slot[i] = (int)sp.args.size();
            sp.args.push_back(bits_of_ptr(fv.ptr));
        } else if (fv.role == MJT_VAR_SCALAR) {
            slot[i] = (int)sp.args.size();
            sp.args.push_back(dtype_is_float(fv.dtype) ? bits_of(fv.fvalue) : (uint64_t)fv.ivalue);
        }
    }
    for (int k = 0; k < d->n_ops; k++) {
        const mjt_fused_op& o = d->ops[k];
        key2 << o.kind << ":" << o.op << ":" << o.in[0] << ":" << (o.kind >= MJT_FOP_BINARY ? o.in[1] : -1) << ":"
             << (o.kind == MJT_FOP_TERNARY ? o.in[2] : -1) << ">" << o.out << ";";
    }
    sp.key = key2.str();
    sp.defs = [d, slot, out](int base) {
        std::ostringstream scal, val;
        for (int i = 0; i < d->n_vars; i++) {
            const mjt_fused_var& fv = d->vars[i];
            const char* T = dtype_cname(fv.dtype);
            if (fv.role == MJT_VAR_SCALAR) {
                if (dtype_is_float(fv.dtype))
                    scal << "const " << T << " v" << i << " = (" << T << ")__longlong_as_double((long long)(unsigned long long)p.a["
                         << base + slot[i] << "]); ";
                else
                    scal << "const " << T << " v" << i << " = (" << T << ")(long long)(unsigned long long)p.a[" << base + slot[i] << "]; ";
            } else if (fv.role == MJT_VAR_GATHERED) {
                val << "const " << T << " v" << i << " = ((const " << T << "*)p.a[" << base + slot[i] << "])[xid]; ";
            } else if (fv.role == MJT_VAR_INPUT) {
                // offset inside a tensor that has extent 1 along the axes of its mask: Horner over the other axes
                std::string off = "(index_t)0";
                bool full = true;
                for (int a = 0; a < d->ndim; a++)
                    if ((fv.bcast_mask >> a & 1) && d->shape[a] != 1) full = false;
                if (full) {
                    off = "e_";
                } else {
                    for (int a = 0; a < d->ndim; a++)
                        if (!(fv.bcast_mask >> a & 1) && d->shape[a] != 1)
                            off = "(" + off + " * yshape" + std::to_string(a) + " + i" + std::to_string(a) + ")";
                }
                val << "const " << T << " v" << i << " = ((const " << T << "*)p.a[" << base + slot[i] << "])[" << off << "]; ";
            }
        }
        std::ostringstream defs;
        defs << "#define SC_PROLOGUE 1\n#define MJT_SC_SCALARS " << scal.str() << "\n#define MJT_SC_VALUE " << val.str()
             << fused_emit_ops(d, false) << "const TX val_ = (TX)(v" << out << ");\n";
        return defs.str();
    };
    if (numel(&y) > 0 && try_window_scatter(plan, op, x, &y, n_ofc, n_ex, &sp)) return;
    launch_fill_pattern(x->ptr, op == MJT_OP_VOID ? 0 : identity_bits(op, x->dtype), dtype_size(x->dtype), (size_t)xn);
    if (numel(&y) == 0) return;
    run_generic(plan, true, op, x, &y, 0.0, n_ex, ex, nullptr, 0, 0, &sp);
}

void reindex_reduce_impl(const mjt_tensor* y, const mjt_tensor* x, int op, int n_idx, const char* const* idx, int n_ofc,
                         const char* const* ofc, int n_ex, const mjt_tensor* ex) {
    require_init();
    check_tensor(y, "reindex_reduce y");
    check_tensor(x, "reindex_reduce x");
    check_extras(n_ex, ex);
    // ASSERT((ns.is_binary() && ns!=ns_mean) || ns == ns_void), ops/reindex_reduce_op.cc:34
    MJT_CHECK((op >= MJT_OP_POW && op < MJT_OP_MEAN) || op == MJT_OP_VOID,
              "reindex_reduce: op must be a binary op other than mean, or void");
    MJT_CHECK(n_idx == x->ndim, "Number of shape and indexes should be the same. (shape rank " << x->ndim << ", " << n_idx
                                                                                              << " indexes)");
    MJT_CHECK(n_idx == 0 || idx, "null indexes");
    MJT_CHECK(n_ofc >= 0 && (n_ofc == 0 || ofc), "null overflow conditions");
    MJT_CHECK(x->dtype == y->dtype, "reindex_reduce: x dtype must equal y dtype");
    std::string key = plan_key(true, op, x, y, n_idx, idx, n_ofc, ofc, n_ex, ex);
    Plan* plan = get_plan(key, x, y, y->ndim, n_idx, idx, n_ofc, ofc, n_ex, ex);
    int64_t xn = numel(x);
    if (xn == 0) return;
    if (plan->plain_e0 && numel(y) > 0 && numel(&ex[0]) == numel(y) && try_scatter_1d(y, x, op, &ex[0])) return;
    if (numel(y) > 0 && try_window_scatter(plan, op, x, y, n_ofc, n_ex, nullptr)) return;
    // "void" skips the initialisation in the reference (ops/reindex_reduce_op.cc:113-120), which leaves the
    // elements no update reaches unspecified; here they are zero, so that results do not depend on what the
    // buffer held before
    launch_fill_pattern(x->ptr, op == MJT_OP_VOID ? 0 : identity_bits(op, x->dtype), dtype_size(x->dtype), (size_t)xn);
    run_generic(plan, true, op, x, y, 0.0, n_ex, ex);
}

}  // namespace mjt

extern "C" int mjt_reindex(const mjt_tensor* x, const mjt_tensor* y, int n_indexes, const char* const* indexes,
                           double overflow_value, int n_overflow_conditions, const char* const* overflow_conditions,
                           int n_extras, const mjt_tensor* extras) {
    return mjt::guarded([&] {
        mjt::reindex_impl(x, y, n_indexes, indexes, overflow_value, n_overflow_conditions, overflow_conditions, n_extras,
                          extras);
    });
}

extern "C" int mjt_reindex_then_reduce(const mjt_tensor* x, const mjt_tensor* yshape, const mjt_tensor* z, int op, int n_reduced,
                                       int n_indexes, const char* const* indexes, double overflow_value,
                                       int n_overflow_conditions, const char* const* overflow_conditions, int n_extras,
                                       const mjt_tensor* extras) {
    return mjt::guarded([&] {
        mjt::reindex_then_reduce_impl(x, yshape, z, op, n_reduced, n_indexes, indexes, overflow_value, n_overflow_conditions,
                                      overflow_conditions, n_extras, extras);
    });
}

extern "C" int mjt_fused_reindex_reduce(const mjt_fused_desc* desc, const mjt_tensor* x, int op, int n_indexes,
                                        const char* const* indexes, int n_overflow_conditions,
                                        const char* const* overflow_conditions, int n_extras, const mjt_tensor* extras) {
    return mjt::guarded([&] {
        mjt::fused_reindex_reduce_impl(desc, x, op, n_indexes, indexes, n_overflow_conditions, overflow_conditions, n_extras, extras);
    });
}

extern "C" int mjt_reindex_reduce(const mjt_tensor* y, const mjt_tensor* x, int op, int n_indexes,
                                  const char* const* indexes, int n_overflow_conditions,
                                  const char* const* overflow_conditions, int n_extras, const mjt_tensor* extras) {
    return mjt::guarded([&] {
        mjt::reindex_reduce_impl(y, x, op, n_indexes, indexes, n_overflow_conditions, overflow_conditions, n_extras,
                                 extras);
    });
}
