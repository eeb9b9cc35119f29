// mjt_reduce: host side of the axis-set reduction
// (reference: python/jittor/src/ops/reduce_op.cc:257-337 for masks and
// shapes, :374-399 for the loop nest this replaces).
#include "common.h"
#include <mutex>
#include <unordered_map>

namespace mjt {

namespace {

struct Axis {
    int64_t size;
    int64_t stride;
};

std::mutex g_mu;
std::unordered_map<std::string, JitKernel*> g_kernels;

bool reducible(int op) {
    switch (op) {
        case MJT_OP_ADD: case MJT_OP_MULTIPLY: case MJT_OP_MAXIMUM: case MJT_OP_MINIMUM:
        case MJT_OP_LOGICAL_AND: case MJT_OP_LOGICAL_OR: case MJT_OP_LOGICAL_XOR:
        case MJT_OP_BITWISE_AND: case MJT_OP_BITWISE_OR: case MJT_OP_BITWISE_XOR: case MJT_OP_MEAN:
            return true;
        default:
            return false;
    }
}

int env_int(const char* n, int d) {
    const char* v = getenv(n);
    return v && *v ? atoi(v) : d;
}

struct Variant {
    int tx, ty, op, nk, nr, vec, g, unr, nt;
    bool row, split, use64, second;   // second: folding partials (TX == TY, plain merge)
};

JitKernel* get_kernel(const Variant& v) {
    std::ostringstream key;
    key << v.tx << "," << v.ty << "," << v.op << "," << v.nk << "," << v.nr << "," << v.vec << "," << v.g << ","
        << v.row << v.split << v.use64 << v.second << "," << v.unr << "," << v.nt;
    std::lock_guard<std::mutex> lock(g_mu);
    auto it = g_kernels.find(key.str());
    if (it != g_kernels.end()) return it->second;
    const char* opn = mjt_op_name(v.op);
    std::string merge_op = v.op == MJT_OP_MEAN ? "add" : opn;
    std::ostringstream name;
    name << "mjt_reduce_" << (v.row ? "row_" : "col_") << opn << "_" << mjt_dtype_name(v.tx) << "_"
         << mjt_dtype_name(v.ty) << "_k" << v.nk << "r" << v.nr << "v" << v.vec << "g" << v.g
         << (v.split ? "_split" : "") << (v.second ? "_fold" : "") << (v.use64 ? "_i64" : "");
    std::ostringstream src;
    src << "#define ENTRY " << name.str() << "\n";
    src << "#define TX " << dtype_cname(v.tx) << "\n#define TY " << dtype_cname(v.ty) << "\n";
    src << "#define index_t " << (v.use64 ? "long long" : "int") << "\n#define USE64 " << (v.use64 ? 1 : 0) << "\n";
    src << "#define NK " << v.nk << "\n#define NR " << v.nr << "\n#define VEC " << v.vec << "\n#define G " << v.g
        << "\n#define SPLIT " << (v.split ? 1 : 0) << "\n#define ROW " << (v.row ? 1 : 0) << "\n";
    src << "#define UNR " << v.unr << "\n#define MJT_LD " << (v.nt ? "mjt_load_nt" : "mjt_load") << "\n";
    src << "#define MERGE(a, b) mjt_" << merge_op << "<TY>((a), (b))\n";
    if (v.second || v.op != MJT_OP_MEAN)
        src << "#define COMBINE(a, x) mjt_" << (v.second ? merge_op : std::string(opn)) << "<TY>((a), (x))\n";
    else   // (acc + Ty(x) * Ty(rcount)), type/common_op_type.cc:141
        src << "#define COMBINE(a, x) ((a) + TY(x) * TY(rcount))\n";
    src << "#define INIT mjt_init_" << merge_op << "<TY>()\n";
    src << embedded_source("prelude.h") << "\n" << embedded_source("reduce.h") << "\n";
    JitKernel* k = jit_get(src.str(), name.str());
    g_kernels.emplace(key.str(), k);
    return k;
}

int pick_vec(int elem_size, int64_t run, const void* p, const void* q, int out_size) {
    int vec = 16 / elem_size;
    if (vec > 8) vec = 8;
    while (vec > 1 && (run % vec != 0 || ((uintptr_t)p % (size_t)(vec * elem_size)) != 0 ||
                       (q && ((uintptr_t)q % (size_t)(vec * out_size)) != 0)))
        vec /= 2;
    return vec;
}

void fill_axes(std::vector<uint64_t>& a, const std::vector<Axis>& kept, const std::vector<Axis>& red) {
    for (size_t i = 0; i < kept.size(); i++) {
        a[8 + 0 * 5 + i] = (uint64_t)kept[i].size;
        a[8 + 1 * 5 + i] = (uint64_t)kept[i].stride;
        a[8 + 2 * 5 + i] = pack_divmod((uint64_t)kept[i].size);
    }
    for (size_t i = 0; i < red.size(); i++) {
        a[8 + 3 * 5 + i] = (uint64_t)red[i].size;
        a[8 + 4 * 5 + i] = (uint64_t)red[i].stride;
        a[8 + 5 * 5 + i] = pack_divmod((uint64_t)red[i].size);
    }
}

// One launch of the row or column kernel.  Returns nothing; partials (when
// S > 1) are written to `out` as [O, S] (row) or [S, O] (column).
void launch(bool row, int tx, int ty, int op, bool second, const void* x, void* out, int64_t O, int64_t S,
            const std::vector<Axis>& kept, const std::vector<Axis>& red, double rcount, bool use64, int vec, int g,
            int64_t per, int64_t total, bool stream = false) {
    // inputs larger than the caches are streamed (read once, non-temporal loads)
    Variant v{tx, ty, op, (int)kept.size(), (int)red.size(), vec, g, env_int("MJT_REDUCE_UNR", 8),
              env_int("MJT_REDUCE_NT", stream ? 1 : 0), row, S > 1, use64, second};
    JitKernel* k = get_kernel(v);
    std::vector<uint64_t> a(8 + 6 * 5, 0);
    a[0] = bits_of_ptr(x);
    a[1] = bits_of_ptr(out);
    a[2] = (uint64_t)O;
    a[3] = (uint64_t)S;
    a[4] = bits_of(rcount);
    a[5] = (uint64_t)per;
    a[6] = (uint64_t)total;
    fill_axes(a, kept, red);
    int64_t blocks = row ? (O + (256 / g) - 1) / (256 / g) : ((O / vec) + 255) / 256;
    MJT_CHECK(blocks < (int64_t(1) << 31) && S < 65536, "reduce: launch too large");
    jit_launch(k, (unsigned)blocks, (unsigned)S, 256, 0, a);
}

}  // namespace

void reduce_impl(const mjt_tensor* x, const mjt_tensor* y, int op, uint32_t reduce_mask) {
    require_init();
    check_tensor(x, "reduce x");
    check_tensor(y, "reduce y");
    MJT_CHECK(op >= 0 && op < MJT_OP_COUNT && reducible(op),
              "reduce: op '" << (mjt_op_name(op) ? mjt_op_name(op) : "?") << "' is not an associative binary op");
    MJT_CHECK(reduce_mask != 0 && (reduce_mask >> x->ndim) == 0, "reduce: reduce_mask " << reduce_mask
                                                                                       << " does not fit rank " << x->ndim);
    MJT_CHECK(dtype_size(y->dtype) >= 1 && y->dtype != MJT_FLOAT16 && y->dtype != MJT_BFLOAT16 && y->dtype != MJT_BOOL,
              "reduce: accumulator dtype " << mjt_dtype_name(y->dtype) << " is not supported");
    int64_t xn = numel(x), O = 1;
    for (int d = 0; d < x->ndim; d++)
        if (!(reduce_mask >> d & 1)) O *= x->shape[d];
    MJT_CHECK(numel(y) == O, "reduce: y has " << numel(y) << " elements, kept axes of x" << shape_str(x) << " give " << O);
    if (O == 0) return;
    Context& c = ctx();

    // merge axes: drop extent-1 axes, fuse neighbours of equal kind
    std::vector<Axis> kept, red;
    {
        int64_t stride = 1;
        int last_kind = -1;   // kind of the most recently pushed axis (0 kept, 1 reduced)
        std::vector<Axis>* last = nullptr;
        for (int d = x->ndim - 1; d >= 0; d--) {
            int64_t n = x->shape[d];
            int kind = (reduce_mask >> d) & 1;
            if (n != 1) {
                std::vector<Axis>& dst = kind ? red : kept;
                if (last_kind == kind && last == &dst)
                    dst.front().size *= n;          // contiguous with the axis merged last
                else
                    dst.insert(dst.begin(), Axis{n, stride});
                last_kind = kind;
                last = &dst;
            }
            stride *= n;
        }
    }
    MJT_CHECK(kept.size() <= 5 && red.size() <= 5, "reduce: more than 5 alternating axis groups");
    int64_t R = 1;
    for (auto& a : red) R *= a.size;
    double rcount = xn ? (double)O / (double)xn : 0.0;
    int tx = x->dtype, ty = y->dtype;
    int tsz = dtype_size(ty);

    if (xn == 0 || red.empty()) {
        // nothing to fold (empty reduced axis -> identity; extent-1 reduced axes -> copy with conversion):
        // run the column kernel over a reduced axis of extent R (0 or 1)
        std::vector<Axis> r1{Axis{xn == 0 ? 0 : 1, 0}};
        std::vector<Axis> k1{Axis{O, 1}};
        launch(false, tx, ty, op, false, x->ptr ? x->ptr : y->ptr, y->ptr, O, 1, k1, r1, rcount, false, 1, 1,
               r1[0].size, r1[0].size);
        return;
    }
    bool use64 = xn >= (int64_t(1) << 31);
    bool row = red.back().stride == 1;   // innermost merged axis is reduced
    const bool stream = xn * (int64_t)dtype_size(tx) >= (int64_t(64) << 20);
    const int64_t cu = c.prop.multiProcessorCount;

    if (row) {
        int64_t L = red.back().size;
        int vec = pick_vec(dtype_size(tx), L, x->ptr, nullptr, 0);
        for (auto& a : kept)
            if (a.stride % vec) vec = 1;
        for (size_t i = 0; i + 1 < red.size(); i++)
            if (red[i].stride % vec) vec = 1;
        int g = 64;
        while (g > 1 && (int64_t)(g / 2) * vec * 2 > L) g /= 2;   // at least ~2 loads per lane, else shrink the group
        if (R >= 4096) g = 64;
        int64_t nL = (L + (int64_t)g * vec - 1) / ((int64_t)g * vec);
        int64_t total = (R / L) * nL;
        int64_t groups = O;
        int64_t target = cu * 16;               // groups of 64 lanes wanted in flight
        int64_t S = 1;
        if (groups * g < target * 64 && total > 8) {
            S = (target * 64 + groups * g - 1) / (groups * g);
            if (S > total / 4) S = total / 4;
            if (S > 1024) S = 1024;
            if (S < 1) S = 1;
        }
        int64_t per = (total + S - 1) / S;
        S = (total + per - 1) / per;
        if (S == 1) {
            launch(true, tx, ty, op, false, x->ptr, y->ptr, O, 1, kept, red, rcount, use64, vec, g, per, total, stream);
        } else {
            void* part = scratch((size_t)O * S * tsz);
            launch(true, tx, ty, op, false, x->ptr, part, O, S, kept, red, rcount, use64, vec, g, per, total, stream);
            // fold [O, S] along the last axis
            std::vector<Axis> k2{Axis{O, S}}, r2{Axis{S, 1}};
            int vec2 = pick_vec(tsz, S, part, nullptr, 0);
            int g2 = 64;
            while (g2 > 1 && (int64_t)(g2 / 2) * vec2 >= S) g2 /= 2;
            int64_t nL2 = (S + (int64_t)g2 * vec2 - 1) / ((int64_t)g2 * vec2);
            launch(true, ty, ty, op, true, part, y->ptr, O, 1, k2, r2, rcount, false, vec2, g2, nL2, nL2);
        }
    } else {
        int64_t Lk = kept.back().size;
        int vec = pick_vec(dtype_size(tx), Lk, x->ptr, y->ptr, tsz);
        for (size_t i = 0; i + 1 < kept.size(); i++)
            if (kept[i].stride % vec) vec = 1;
        for (auto& a : red)
            if (a.stride % vec) vec = 1;
        int64_t threads = O / vec;
        int64_t target = cu * 256 * 4;
        int64_t S = 1;
        if (threads < target && R > 16) {
            S = (target + threads - 1) / threads;
            if (S > R / 8) S = R / 8;
            if (S > 1024) S = 1024;
            if (S < 1) S = 1;
        }
        int64_t per = (R + S - 1) / S;
        S = (R + per - 1) / per;
        if (S == 1) {
            launch(false, tx, ty, op, false, x->ptr, y->ptr, O, 1, kept, red, rcount, use64, vec, 1, per, R, stream);
        } else {
            void* part = scratch((size_t)O * S * tsz);
            launch(false, tx, ty, op, false, x->ptr, part, O, S, kept, red, rcount, use64, vec, 1, per, R, stream);
            std::vector<Axis> k2{Axis{O, 1}}, r2{Axis{S, O}};
            int vec2 = pick_vec(tsz, O, part, y->ptr, tsz);
            launch(false, ty, ty, op, true, part, y->ptr, O, 1, k2, r2, rcount, false, vec2, 1, S, S);
        }
    }
}

}  // namespace mjt

extern "C" int mjt_reduce(const mjt_tensor* x, const mjt_tensor* y, int op, uint32_t reduce_mask) {
    return mjt::guarded([&] { mjt::reduce_impl(x, y, op, reduce_mask); });
}
