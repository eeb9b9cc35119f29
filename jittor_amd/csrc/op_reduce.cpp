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
void forget() {   // the kernels belong to the run-time compiler's cache, which mjt_shutdown empties
    std::lock_guard<std::mutex> lock(g_mu);
    g_kernels.clear();
}
const bool g_registered = (at_shutdown(&forget), true);

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

// element-wise prologue of a reduce: macro text for the kernel, its cache key, its parameter words
struct Prologue {
    std::string defs, key;
    std::vector<uint64_t> args;
    std::vector<std::pair<const void*, int>> inputs;   // (pointer, element size) of every tensor it loads
};

// 16-bit float results are accumulated in float32 and rounded once, at the store
int acc_dtype(int ty) { return ty == MJT_FLOAT16 || ty == MJT_BFLOAT16 ? MJT_FLOAT32 : ty; }

// The fixed scratch array behind mjt_reduce_static.  In host code the array's name is only a handle: its device
// address is looked up once per device (every device holds its own copy at its own address) and that pointer is
// what kernels get.
static __device__ __align__(256) __attribute__((used)) unsigned char g_static_scratch[MJT_STATIC_SCRATCH_BYTES];
constexpr int kMaxDevices = 64;
void* g_static_ptr[kMaxDevices] = {};

struct Variant {
    int tx, ty, op, nk, nr, vec, g, unr, nt;
    bool row, split, use64, second;   // second: folding partials (TX == TY, plain merge)
    const Prologue* pro;
    bool tsplit = false;              // column kernel: partials as [O, S] instead of [S, O]
};

// may_build == false: only a kernel that is already loaded is returned (no compiler, no module load)
JitKernel* get_kernel(const Variant& v, bool may_build = true) {
    std::ostringstream key;
    key << v.tx << "," << v.ty << "," << v.op << "," << v.nk << "," << v.nr << "," << v.vec << "," << v.g << ","
        << v.row << v.split << v.use64 << v.second << v.tsplit << "," << v.unr << "," << v.nt;
    if (v.pro) key << "|" << v.pro->key;
    std::lock_guard<std::mutex> lock(g_mu);
    auto it = g_kernels.find(key.str());
    if (it != g_kernels.end()) return it->second;
    const char* opn = mjt_op_name(v.op);
    std::string merge_op = v.op == MJT_OP_MEAN ? "add" : opn;
    std::ostringstream name;
    name << "mjt_reduce_" << (v.row ? "row_" : "col_") << opn << "_" << mjt_dtype_name(v.tx) << "_"
         << mjt_dtype_name(v.ty) << "_k" << v.nk << "r" << v.nr << "v" << v.vec << "g" << v.g
         << (v.split ? (v.tsplit ? "_tsplit" : "_split") : "") << (v.second ? "_fold" : "") << (v.use64 ? "_i64" : "");
    if (v.pro) {
        uint64_t h = 1469598103934665603ull;
        for (unsigned char ch : v.pro->key) {
            h ^= ch;
            h *= 1099511628211ull;
        }
        char buf[32];
        snprintf(buf, sizeof(buf), "_pro%016llx", (unsigned long long)h);
        name << buf;
    }
    std::ostringstream src;
    src << "#define ENTRY " << name.str() << "\n";
    src << "#define TX " << dtype_cname(v.tx) << "\n#define TY " << dtype_cname(v.ty) << "\n#define TACC " << dtype_cname(acc_dtype(v.ty)) << "\n";
    src << "#define index_t " << (v.use64 ? "long long" : "int") << "\n#define USE64 " << (v.use64 ? 1 : 0) << "\n";
    src << "#define NK " << v.nk << "\n#define NR " << v.nr << "\n#define VEC " << v.vec << "\n#define G " << v.g
        << "\n#define SPLIT " << (v.split ? 1 : 0) << "\n#define SPLIT_T " << (v.tsplit ? 1 : 0) << "\n#define ROW " << (v.row ? 1 : 0) << "\n";
    src << "#define UNR " << v.unr << "\n#define MJT_LD " << (v.nt ? "mjt_load_nt" : "mjt_load") << "\n";
    src << "#define MERGE(a, b) mjt_" << merge_op << "<TACC>((a), (b))\n";
    if (v.second || v.op != MJT_OP_MEAN)
        src << "#define COMBINE(a, x) mjt_" << (v.second ? merge_op : std::string(opn)) << "<TACC>((a), (x))\n";
    else   // (acc + Ty(x) * Ty(rcount)), type/common_op_type.cc:141
        src << "#define COMBINE(a, x) ((a) + TACC(x) * TACC(rcount))\n";
    src << "#define INIT mjt_init_" << merge_op << "<TACC>()\n";
    if (v.pro) src << v.pro->defs;
    src << embedded_source("prelude.h") << "\n" << embedded_source("reduce.h") << "\n";
    JitKernel* k = may_build ? jit_get(src.str(), name.str()) : jit_lookup(src.str());
    if (!k)
        throw Error{MJT_ERR_NOT_READY, "reduce: kernel " + name.str() + " is not loaded yet and this entry point may not build it: "
                                       "call mjt_reduce once with a descriptor of the same kind first"};
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

// same with a prologue: every tensor it loads must take the vector width
int pick_vec_pro(const Prologue* pro, int elem_size, int64_t run, const void* p, const void* q, int out_size) {
    if (!pro) return pick_vec(elem_size, run, p, q, out_size);
    int widest = 1;
    for (auto& in : pro->inputs) widest = in.second > widest ? in.second : widest;
    int vec = pick_vec(widest, run, nullptr, q, out_size);
    for (auto& in : pro->inputs)
        while (vec > 1 && (uintptr_t)in.first % (size_t)(vec * in.second)) vec /= 2;
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
// S > 1) are written to `out` as [O, S] by both kernels.
void launch(bool row, int tx, int ty, int op, bool second, const void* x, void* out, int64_t O, int64_t S,
            const std::vector<Axis>& kept, const std::vector<Axis>& red, double rcount, bool use64, int vec, int g,
            int64_t per, int64_t total, bool stream = false, const Prologue* pro = nullptr, bool may_build = true, bool tsplit = false) {
    // inputs larger than the caches are streamed (read once, non-temporal loads)
    // loads in flight per lane: 8, or as many as a row gives a lane when that is fewer (the unrolled loop only takes whole batches)
    int unr = 8;
    if (row && !red.empty()) {
        const int64_t per_lane = red.back().size / ((int64_t)g * vec);
        while (unr > 1 && unr > per_lane) unr /= 2;
    }
    Variant v{tx, ty, op, (int)kept.size(), (int)red.size(), vec, g, unr,
              stream ? 1 : 0, row, S > 1, use64, second, pro};
    v.tsplit = tsplit && !row && S > 1;
    JitKernel* k = get_kernel(v, may_build);
    std::vector<uint64_t> a(8 + 6 * 5, 0);
    a[0] = bits_of_ptr(x);
    a[1] = bits_of_ptr(out);
    a[2] = (uint64_t)O;
    a[3] = (uint64_t)S;
    a[4] = bits_of(rcount);
    a[5] = (uint64_t)per;
    a[6] = (uint64_t)total;
    fill_axes(a, kept, red);
    if (pro) a.insert(a.end(), pro->args.begin(), pro->args.end());
    const int64_t blk = row && g > 256 ? g : 256;              // lanes per workgroup
    const int64_t txl = !row && g > 1 ? g : 256;                // column kernel: lanes across the outputs
    int64_t blocks = row ? (O + (blk / g) - 1) / (blk / g) : ((O / vec) + txl - 1) / txl;
    const int64_t grid_y = row ? S : (S + 256 / txl - 1) / (256 / txl);
    MJT_CHECK(blocks < (int64_t(1) << 31) && grid_y < 65536, "reduce: launch too large");
    jit_launch(k, (unsigned)blocks, (unsigned)grid_y, (unsigned)blk, 0, a);
}

}  // namespace

// fixed_scratch: the allocation-free variant (partials in the fixed array, only kernels that are already loaded)
void reduce_core(const mjt_tensor* x, const mjt_tensor* y, int op, uint32_t reduce_mask, const Prologue* pro,
                 bool fixed_scratch = false) {
    require_init();
    const bool mb = !fixed_scratch;
    auto partials = [&](size_t bytes) -> void* {
        if (!fixed_scratch) return scratch(bytes);
        Context& cc = ctx();
        if (bytes > MJT_STATIC_SCRATCH_BYTES)
            MJT_FAIL(MJT_ERR_UNSUPPORTED, "mjt_reduce_static: this reduction is split into " << bytes << " bytes of partial results; "
                                          "the fixed scratch array holds " << MJT_STATIC_SCRATCH_BYTES << " (use mjt_reduce)");
        if (cc.dry_run) return (void*)(uintptr_t)0x1000;
        void* ptr = cc.device >= 0 && cc.device < kMaxDevices ? g_static_ptr[cc.device] : nullptr;
        if (!ptr) MJT_FAIL(MJT_ERR_NOT_INIT, "mjt_reduce_static: the fixed scratch array was not set up on device " << cc.device);
        return ptr;
    };
    if (!pro) check_tensor(x, "reduce x");
    check_tensor(y, "reduce y");
    MJT_CHECK(op >= 0 && op < MJT_OP_COUNT && reducible(op),
              "reduce: op '" << (mjt_op_name(op) ? mjt_op_name(op) : "?") << "' is not an associative binary op");
    MJT_CHECK(reduce_mask != 0 && (reduce_mask >> x->ndim) == 0, "reduce: reduce_mask " << reduce_mask
                                                                                       << " does not fit rank " << x->ndim);
    MJT_CHECK(dtype_size(y->dtype) >= 1 && y->dtype != MJT_BOOL,
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
    const int ta = acc_dtype(ty);              // type of the partials of a split reduction
    int tsz = dtype_size(ty);
    const int asz = dtype_size(ta);

    if (xn == 0 || red.empty()) {
        // nothing to fold (empty reduced axis -> identity; extent-1 reduced axes -> copy with conversion):
        // run the column kernel over a reduced axis of extent R (0 or 1)
        std::vector<Axis> r1{Axis{xn == 0 ? 0 : 1, 0}};
        std::vector<Axis> k1{Axis{O, 1}};
        launch(false, tx, ty, op, false, x->ptr ? x->ptr : y->ptr, y->ptr, O, 1, k1, r1, rcount, O >= (int64_t(1) << 31), 1, 1,
               r1[0].size, r1[0].size, false, xn ? pro : nullptr, mb);
        return;
    }
    bool use64 = xn >= (int64_t(1) << 31);
    bool row = red.back().stride == 1;   // innermost merged axis is reduced
    const bool stream = xn * (int64_t)dtype_size(tx) >= (int64_t(64) << 20);
    const int64_t cu = c.prop.multiProcessorCount;

    if (row) {
        int64_t L = red.back().size;
        int vec = pick_vec_pro(pro, dtype_size(tx), L, x->ptr, nullptr, 0);
        for (auto& a : kept)
            if (a.stride % vec) vec = 1;
        for (size_t i = 0; i + 1 < red.size(); i++)
            if (red[i].stride % vec) vec = 1;
        int g = 64;
        while (g > 1 && (int64_t)(g / 2) * vec * 2 > L) g /= 2;   // at least ~2 loads per lane, else shrink the group
        if (R >= 4096) g = 64;
        // long rows streamed from memory: up to eight waves per row while every lane keeps at least two loads (measured
        // on an [8192, 4096] float32 sum: 64 lanes per row 22.3 us, 128 21.1, 256 20.8, 512 20.2; with a single load per
        // lane the fixed cost of a lane dominates: [65536, 1024] with 256 lanes 48 us against 39)
        if (stream && g == 64)
            while (g < 512 && (int64_t)g * 2 * vec * 2 <= L) g *= 2;
        if (env_int("MJT_REDUCE_G", 0) >= 64) g = env_int("MJT_REDUCE_G", 0);
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
            launch(true, tx, ty, op, false, x->ptr, y->ptr, O, 1, kept, red, rcount, use64, vec, g, per, total, stream, pro, mb);
        } else {
            void* part = partials((size_t)O * S * asz);
            launch(true, tx, ta, op, false, x->ptr, part, O, S, kept, red, rcount, use64, vec, g, per, total, stream, pro, mb);
            // fold [O, S] along the last axis
            std::vector<Axis> k2{Axis{O, S}}, r2{Axis{S, 1}};
            int vec2 = pick_vec(asz, S, part, nullptr, 0);
            int g2 = 64;
            while (g2 > 1 && (int64_t)(g2 / 2) * vec2 >= S) g2 /= 2;
            int64_t nL2 = (S + (int64_t)g2 * vec2 - 1) / ((int64_t)g2 * vec2);
            launch(true, ta, ty, op, true, part, y->ptr, O, 1, k2, r2, rcount, false, vec2, g2, nL2, nL2, false, nullptr, mb);
        }
    } else {
        int64_t Lk = kept.back().size;
        int vec = pick_vec_pro(pro, dtype_size(tx), Lk, x->ptr, y->ptr, tsz);
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
            launch(false, tx, ty, op, false, x->ptr, y->ptr, O, 1, kept, red, rcount, use64, vec, 1, per, R, stream, pro, mb);
        } else {
            // lanes across the outputs: all 256 (g = 1), or with fewer vectors of outputs the power of two that holds them
            int gx = 1;
            if (threads < 256) {
                gx = 2;
                while (gx < threads) gx *= 2;
            }
            void* part = partials((size_t)O * S * asz);
            const bool tsplit = S >= 16;                 // many slices: partials as [O, S], folded by the row kernel
            launch(false, tx, ta, op, false, x->ptr, part, O, S, kept, red, rcount, use64, vec, gx, per, R, stream, pro, mb, tsplit);
            if (tsplit) {
                std::vector<Axis> k2{Axis{O, S}}, r2{Axis{S, 1}};
                int vec2 = pick_vec(asz, S, part, nullptr, 0);
                int g2 = 64;
                while (g2 > 1 && (int64_t)(g2 / 2) * vec2 >= S) g2 /= 2;
                int64_t nL2 = (S + (int64_t)g2 * vec2 - 1) / ((int64_t)g2 * vec2);
                launch(true, ta, ty, op, true, part, y->ptr, O, 1, k2, r2, rcount, false, vec2, g2, nL2, nL2, false, nullptr, mb);
            } else {                                     // a few slices [S, O]: each output's lane walks them
                std::vector<Axis> k2{Axis{O, 1}}, r2{Axis{S, O}};
                int vec2 = pick_vec(asz, O, part, y->ptr, tsz);
                launch(false, ta, ty, op, true, part, y->ptr, O, 1, k2, r2, rcount, false, vec2, 1, S, S, false, nullptr, mb);
            }
        }
    }
}

void reduce_impl(const mjt_tensor* x, const mjt_tensor* y, int op, uint32_t reduce_mask) {
    reduce_core(x, y, op, reduce_mask, nullptr);
}

// Looks up where this device keeps the fixed scratch array.  Runs once per device, with that device current
// (mjt_init calls it after hipSetDevice).
// Never fails: a device outside the table, or one whose copy of the array cannot be found, leaves its entry null, and
// mjt_reduce_static then reports MJT_ERR_NOT_INIT for that device while every other entry point works.
void reduce_static_setup(int device) {
    if (device < 0 || device >= kMaxDevices || g_static_ptr[device]) return;
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_static_scratch)) != hipSuccess) {
        (void)hipGetLastError();
        return;
    }
    g_static_ptr[device] = ptr;
}

// Reduce whose input is produced element by element from other tensors: the group's single output var
// is never written to memory.
void fused_reduce_impl(const mjt_fused_desc* d, const mjt_tensor* y, int op, uint32_t reduce_mask) {
    require_init();
    std::vector<int> inputs;
    fused_validate(d, &inputs, false);
    int out = -1;
    for (int i = 0; i < d->n_vars; i++)
        if (d->vars[i].role == MJT_VAR_OUTPUT) {
            MJT_CHECK(out < 0, "fused reduce: the group must have exactly one output var (the reduce input)");
            out = i;
        }
    MJT_CHECK(out >= 0, "fused reduce: the group has no output var");
    // a tensor input is either full-shape or broadcast along exactly the reduced axes (one value per output)
    uint32_t live_mask = 0, red_live = 0;          // axes of extent > 1; those of them that are reduced
    for (int a = 0; a < d->ndim; a++)
        if (d->shape[a] != 1) {
            live_mask |= 1u << a;
            if (reduce_mask >> a & 1) red_live |= 1u << a;
        }
    for (int id : inputs) {
        const uint32_t m = d->vars[id].bcast_mask & live_mask;
        if (m != 0 && m != red_live)
            MJT_FAIL(MJT_ERR_UNSUPPORTED, "fused reduce: input var " << id << " is broadcast along axes other than the reduced ones");
    }
    Prologue pro;
    const int base = 8 + 6 * 5;
    std::ostringstream scal, loads, elems, key, per_out;
    std::vector<int> slot(d->n_vars, -1);
    for (int i = 0; i < d->n_vars; i++) {
        const mjt_fused_var& fv = d->vars[i];
        const char* T = dtype_cname(fv.dtype);
        key << fv.role << ":" << fv.dtype << ";";
        if (fv.role == MJT_VAR_INPUT) {
            slot[i] = base + (int)pro.args.size();
            pro.args.push_back(bits_of_ptr(fv.ptr));
            if ((fv.bcast_mask & live_mask) == 0 || red_live == 0) {
                pro.inputs.emplace_back(fv.ptr, dtype_size(fv.dtype));
                loads << "mjt_pack<" << T << ", VEC> in" << i << "; MJT_LD(in" << i << ", (const " << T << "*)p.a[" << slot[i]
                      << "] + o_); ";
                elems << "const " << T << " v" << i << " = in" << i << ".v[k]; ";
            } else {
                // one value per output: a scalar per lane group in the row kernel, VEC adjacent outputs per lane in
                // the column kernel (scalar loads there: the outputs' alignment is not part of the vector-width choice)
                key << "P";
                per_out << "T_ROWCOL(" << T << ", " << i << ", " << slot[i] << ") ";
                elems << "const " << T << " v" << i << " = V_ROWCOL(" << i << "); ";
            }
        } else if (fv.role == MJT_VAR_SCALAR) {
            slot[i] = base + (int)pro.args.size();
            if (dtype_is_float(fv.dtype)) {
                pro.args.push_back(bits_of(fv.fvalue));
                scal << "const " << T << " v" << i << " = (" << T << ")__longlong_as_double((long long)(unsigned long long)p.a["
                     << slot[i] << "]); ";
            } else {
                pro.args.push_back((uint64_t)fv.ivalue);
                scal << "const " << T << " v" << i << " = (" << T << ")(long long)(unsigned long long)p.a[" << slot[i] << "]; ";
            }
        }
    }
    for (int k = 0; k < d->n_ops; k++) {
        const mjt_fused_op& o = d->ops[k];
        key << o.kind << ":" << o.op << ":" << o.in[0] << ":" << (o.kind >= MJT_FOP_BINARY ? o.in[1] : -1) << ":"
            << (o.kind == MJT_FOP_TERNARY ? o.in[2] : -1) << ">" << o.out << ";";
    }
    std::ostringstream defs;
    defs << "#if ROW\n#define T_ROWCOL(T, i, slot) const T r##i = ((const T*)p.a[slot])[o];\n#define V_ROWCOL(i) r##i\n#else\n"
         << "#define T_ROWCOL(T, i, slot) T r##i[VEC]; _Pragma(\"unroll\") for (int k = 0; k < VEC; k++) r##i[k] = ((const T*)p.a[slot])[o + k];\n"
         << "#define V_ROWCOL(i) r##i[k]\n#endif\n"
         << "#define MJT_PRO_PER_OUTPUT " << per_out.str() << "\n";
    defs << "#define NPRO " << pro.args.size() << "\n#define MJT_PRO_SCALARS " << scal.str() << "\n"
         << "#define MJT_RD(dst, off) do { const index_t o_ = (off); " << loads.str()
         << "_Pragma(\"unroll\") for (int k = 0; k < VEC; k++) { " << elems.str() << fused_emit_ops(d, false) << "(dst).v[k] = (TX)(v"
         << out << "); } } while (0)\n";
    pro.defs = defs.str();
    pro.key = key.str();
    mjt_tensor x{};                        // the virtual reduce input: dtype of the group's output, shape of the group
    x.ptr = nullptr;
    x.dtype = d->vars[out].dtype;
    x.ndim = d->ndim;
    for (int i = 0; i < d->ndim; i++) x.shape[i] = d->shape[i];
    dtype_size(x.dtype);
    reduce_core(&x, y, op, reduce_mask, &pro);
}

}  // namespace mjt

extern "C" int mjt_fused_reduce(const mjt_fused_desc* desc, const mjt_tensor* y, int op, uint32_t reduce_mask) {
    return mjt::guarded([&] { mjt::fused_reduce_impl(desc, y, op, reduce_mask); });
}

extern "C" int mjt_reduce_static(const mjt_tensor* x, const mjt_tensor* y, int op, uint32_t reduce_mask) {
    return mjt::guarded([&] { mjt::reduce_core(x, y, op, reduce_mask, nullptr, true); });
}

extern "C" int mjt_reduce(const mjt_tensor* x, const mjt_tensor* y, int op, uint32_t reduce_mask) {
    return mjt::guarded([&] { mjt::reduce_impl(x, y, op, reduce_mask); });
}
