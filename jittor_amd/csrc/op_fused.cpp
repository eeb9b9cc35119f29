// mjt_fused_elementwise: host side of the fused broadcast + element-wise
// group (reference: python/jittor/src/fused_op.cc:41-118 builds the group,
// op_compiler.cc:839-1045 stitches the member kernels into one loop nest).
#include "common.h"
#include <mutex>
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

bool is_unary_op(int op) { return op >= MJT_OP_ABS && op <= MJT_OP_SIGMOID; }
bool is_binary_op(int op) { return op >= MJT_OP_POW && op <= MJT_OP_MEAN; }

struct MergedDim {
    int64_t size;
    std::vector<int> bcast;   // per input tensor: 1 when broadcast along this axis
};

std::string vname(int i) { return "v" + std::to_string(i); }

}  // namespace

int64_t fused_validate(const mjt_fused_desc* d, std::vector<int>* inputs_out, bool outputs_need_data, bool allow_gathered) {
    MJT_CHECK(d, "fused: null descriptor");
    MJT_CHECK(d->ndim >= 1 && d->ndim <= MJT_MAX_DIM, "fused: rank " << d->ndim);
    MJT_CHECK(d->n_vars > 0 && d->n_ops > 0 && d->vars && d->ops, "fused: empty group");
    MJT_CHECK(d->n_vars <= 256 && d->n_ops <= 256, "fused: group too large");
    int64_t total = 1;
    for (int i = 0; i < d->ndim; i++) {
        MJT_CHECK(d->shape[i] >= 0, "fused: negative extent");
        total *= d->shape[i];
    }
    const int nv = d->n_vars;
    std::vector<int> defined(nv, 0);
    std::vector<int>& inputs = *inputs_out;          // var ids of tensor inputs
    for (int i = 0; i < nv; i++) {
        const mjt_fused_var& v = d->vars[i];
        dtype_size(v.dtype);
        MJT_CHECK(v.role >= MJT_VAR_INPUT && v.role <= (allow_gathered ? MJT_VAR_GATHERED : MJT_VAR_SCALAR),
                  "fused: var " << i << " has role " << v.role);
        if (v.role == MJT_VAR_GATHERED) {
            MJT_CHECK(total == 0 || v.ptr, "fused: gathered var " << i << " has no data");
            defined[i] = 1;
        }
        if (v.role == MJT_VAR_INPUT) {
            MJT_CHECK(total == 0 || v.ptr, "fused: input var " << i << " has no data");
            MJT_CHECK((v.bcast_mask >> d->ndim) == 0, "fused: bcast_mask of var " << i << " exceeds the rank");
            defined[i] = 1;
            inputs.push_back(i);
        } else if (v.role == MJT_VAR_SCALAR) {
            defined[i] = 1;
        } else if (v.role == MJT_VAR_OUTPUT) {
            MJT_CHECK(!outputs_need_data || total == 0 || v.ptr, "fused: output var " << i << " has no data");
        }
    }
    for (int k = 0; k < d->n_ops; k++) {
        const mjt_fused_op& o = d->ops[k];
        int nin = o.kind == MJT_FOP_UNARY || o.kind == MJT_FOP_BROADCAST ? 1 : o.kind == MJT_FOP_BINARY ? 2 : 3;
        MJT_CHECK(o.kind >= MJT_FOP_UNARY && o.kind <= MJT_FOP_BROADCAST, "fused: op " << k << " has kind " << o.kind);
        for (int j = 0; j < nin; j++) {
            MJT_CHECK(o.in[j] >= 0 && o.in[j] < nv, "fused: op " << k << " input " << j << " out of range");
            MJT_CHECK(defined[o.in[j]], "fused: op " << k << " reads var " << o.in[j] << " before it is produced");
        }
        MJT_CHECK(o.out >= 0 && o.out < nv, "fused: op " << k << " output out of range");
        const mjt_fused_var& ov = d->vars[o.out];
        MJT_CHECK(ov.role == MJT_VAR_INTERMEDIATE || ov.role == MJT_VAR_OUTPUT,
                  "fused: op " << k << " writes var " << o.out << " which is not an intermediate or output");
        MJT_CHECK(!defined[o.out], "fused: var " << o.out << " is produced twice");
        if (o.kind == MJT_FOP_UNARY) MJT_CHECK(is_unary_op(o.op), "fused: op " << k << ": " << o.op << " is not a unary op");
        if (o.kind == MJT_FOP_BINARY) MJT_CHECK(is_binary_op(o.op), "fused: op " << k << ": " << o.op << " is not a binary op");
        if (o.kind == MJT_FOP_BROADCAST)
            MJT_CHECK(d->vars[o.in[0]].dtype == ov.dtype, "fused: broadcast op " << k << " changes dtype");
        defined[o.out] = 1;
    }
    for (int i = 0; i < nv; i++) MJT_CHECK(defined[i], "fused: var " << i << " is never produced");
    return total;
}

// The op chain for one element as C statements: every var i becomes `vI`; intermediates keep the natural
// type of their expression, outputs take their dtype (and are also written to `outI.v[k]` when
// store_outputs is set).
std::string fused_emit_ops(const mjt_fused_desc* d, bool store_outputs) {
    std::ostringstream body;
    for (int k = 0; k < d->n_ops; k++) {
        const mjt_fused_op& o = d->ops[k];
        const mjt_fused_var& ov = d->vars[o.out];
        const char* Tz = dtype_cname(ov.dtype);
        std::string expr;
        if (o.kind == MJT_FOP_BROADCAST) {
            expr = vname(o.in[0]);
        } else if (o.kind == MJT_FOP_UNARY) {
            expr = std::string("mjt_") + mjt_op_name(o.op) + "<" + Tz + ">(" + vname(o.in[0]) + ")";
        } else if (o.kind == MJT_FOP_BINARY) {
            expr = std::string("mjt_") + mjt_op_name(o.op) + "<" + Tz + ">(" + vname(o.in[0]) + ", " + vname(o.in[1]) + ")";
        } else {
            expr = std::string("(") + vname(o.in[0]) + " ? (" + Tz + ")(" + vname(o.in[1]) + ") : (" + Tz + ")(" +
                   vname(o.in[2]) + "))";
        }
        // bool results are wrapped in (bool)(...) (type/common_op_type.cc:161); outputs take the
        // declared dtype, intermediates keep the natural type of the expression
        if (ov.dtype == MJT_BOOL) expr = "(bool)(" + expr + ")";
        if (ov.role == MJT_VAR_OUTPUT) {
            body << "const " << Tz << " " << vname(o.out) << " = (" << Tz << ")(" << expr << "); ";
            if (store_outputs) body << "out" << o.out << ".v[k] = " << vname(o.out) << "; ";
        } else {
            body << "const auto " << vname(o.out) << " = " << expr << "; ";
        }
    }
    return body.str();
}

void fused_impl(const mjt_fused_desc* d) {
    require_init();
    std::vector<int> inputs;          // var ids of tensor inputs
    const int64_t total = fused_validate(d, &inputs, true);
    const int nv = d->n_vars;
    if (total == 0) return;

    // ---- merge axes: drop extent-1 axes, fuse neighbours on which every input agrees -------
    std::vector<MergedDim> dims;
    for (int a = 0; a < d->ndim; a++) {
        if (d->shape[a] == 1) continue;
        MergedDim m;
        m.size = d->shape[a];
        for (int id : inputs) m.bcast.push_back((d->vars[id].bcast_mask >> a) & 1);
        if (!dims.empty() && dims.back().bcast == m.bcast)
            dims.back().size *= m.size;
        else
            dims.push_back(m);
    }
    if (dims.empty()) {
        MergedDim m;
        m.size = 1;
        m.bcast.assign(inputs.size(), 0);
        dims.push_back(m);
    }
    const int nd = (int)dims.size();
    bool use64 = total >= (int64_t(1) << 31);

    // ---- vector width ----------------------------------------------------------
    int maxsize = 1;
    for (int i = 0; i < nv; i++)
        if (d->vars[i].role == MJT_VAR_INPUT || d->vars[i].role == MJT_VAR_OUTPUT)
            maxsize = std::max(maxsize, dtype_size(d->vars[i].dtype));
    int vec = std::min(8, 16 / maxsize);
    auto aligned = [&](int v) {
        if (dims.back().size % v) return false;
        for (int i = 0; i < nv; i++) {
            const mjt_fused_var& fv = d->vars[i];
            if (fv.role == MJT_VAR_OUTPUT && (uintptr_t)fv.ptr % (size_t)(v * dtype_size(fv.dtype))) return false;
        }
        for (size_t k = 0; k < inputs.size(); k++) {
            const mjt_fused_var& fv = d->vars[inputs[k]];
            if (dims.back().bcast[k]) continue;   // scalar load per lane
            if ((uintptr_t)fv.ptr % (size_t)(v * dtype_size(fv.dtype))) return false;
        }
        return true;
    };
    while (vec > 1 && !aligned(vec)) vec /= 2;
    int64_t nvec = total / vec;
    // measured on MI355X: one vector per lane is fastest for the chain workloads (more vectors per
    // lane cost registers and occupancy); outputs too large to be re-read from cache are stored
    // non-temporally, loads stay plain; and such streams run best as single-wave workgroups, which the dispatcher
    // hands out in address order 1 KB at a time (x[64,512,1024] float32 through an 11-op chain: 256 lanes 44.4 us,
    // 128 lanes 44.1, 64 lanes 43.1, 512 lanes 45.2, 1024 lanes 49.9)
    // A kernel that streams no input of the output's size (a broadcast, a fill) is a pure store stream and wants 4 KB per
    // workgroup: [512,1] spread over [64,512,1024] float32 takes 30.4 us with 64 lanes, 20.2 with 128 or 256
    const bool streams = total * maxsize >= (int64_t(32) << 20);
    bool reads_stream = false;
    for (size_t k = 0; k < inputs.size(); k++) {
        bool full = true;
        for (int a = 0; a < nd; a++)
            if (dims[a].size > 1 && dims[a].bcast[k]) full = false;
        reads_stream = reads_stream || full;
    }
    int block = streams && reads_stream ? 64 : 256;
    int unroll = 1;
    int nt = streams ? 2 : 0;   // bit 0: non-temporal loads, bit 1: non-temporal stores

    // ---- parameter block layout ---------------------------------------------------
    // a[0] nvec | per merged axis: extent, divider | per var: pointer or scalar bits
    // | per (input with broadcast, merged axis): stride in elements
    std::vector<uint64_t> args;
    args.push_back((uint64_t)nvec);
    std::vector<int> p_dim(nd), p_var(nv, -1);
    for (int a = 0; a < nd; a++) {
        p_dim[a] = (int)args.size();
        args.push_back((uint64_t)dims[a].size);
        args.push_back(pack_divmod((uint64_t)dims[a].size));
    }
    for (int i = 0; i < nv; i++) {
        const mjt_fused_var& fv = d->vars[i];
        if (fv.role == MJT_VAR_INTERMEDIATE) continue;
        p_var[i] = (int)args.size();
        if (fv.role == MJT_VAR_SCALAR) {
            if (dtype_is_float(fv.dtype)) args.push_back(bits_of(fv.fvalue));
            else args.push_back((uint64_t)fv.ivalue);
        } else
            args.push_back(bits_of_ptr(fv.ptr));
    }
    std::vector<std::vector<int>> p_stride(inputs.size());
    bool need_decode = false;
    for (size_t k = 0; k < inputs.size(); k++) {
        bool any = false;
        for (int a = 0; a < nd; a++) any |= dims[a].bcast[k] != 0;
        if (!any) continue;
        need_decode = true;
        int64_t stride = 1;
        std::vector<int64_t> st(nd, 0);
        for (int a = nd - 1; a >= 0; a--) {
            if (!dims[a].bcast[k]) {
                st[a] = stride;
                stride *= dims[a].size;
            }
        }
        for (int a = 0; a < nd; a++) {
            p_stride[k].push_back((int)args.size());
            args.push_back((uint64_t)st[a]);
        }
    }

    // ---- static key -----------------------------------------------------------------
    std::ostringstream key;
    key << nd << "|" << vec << "|" << unroll << "|" << use64 << "|" << block << "|" << nt << "|";
    for (int a = 0; a < nd; a++) {
        for (int b : dims[a].bcast) key << b;
        key << ",";
    }
    for (int i = 0; i < nv; i++) key << d->vars[i].role << ":" << d->vars[i].dtype << ";";
    for (int k = 0; k < d->n_ops; k++) {
        const mjt_fused_op& o = d->ops[k];
        key << o.kind << ":" << o.op << ":" << o.in[0] << ":" << (o.kind >= MJT_FOP_BINARY ? o.in[1] : -1) << ":"
            << (o.kind == MJT_FOP_TERNARY ? o.in[2] : -1) << ">" << o.out << ";";
    }
    JitKernel* kern = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_mu);
        auto it = g_kernels.find(key.str());
        if (it != g_kernels.end()) kern = it->second;
    }
    if (!kern) {
        const char* IT = use64 ? "long long" : "int";
        std::ostringstream scal, dec, loads, body, stores;
        for (int i = 0; i < nv; i++) {
            const mjt_fused_var& fv = d->vars[i];
            if (fv.role != MJT_VAR_SCALAR) continue;
            const char* T = dtype_cname(fv.dtype);
            if (dtype_is_float(fv.dtype))
                scal << "const " << T << " " << vname(i) << " = (" << T << ")__longlong_as_double((long long)(unsigned long long)p.a["
                     << p_var[i] << "]); ";
            else
                scal << "const " << T << " " << vname(i) << " = (" << T << ")(long long)(unsigned long long)p.a[" << p_var[i] << "]; ";
        }
        if (need_decode) {
            dec << IT << " rem_ = e; ";
            for (int a = nd - 1; a >= 0; a--) {
                if (a == 0) {
                    dec << "const " << IT << " c0 = rem_; ";
                } else if (use64) {
                    dec << "const " << IT << " q" << a << " = rem_ / (" << IT << ")(unsigned long long)p.a[" << p_dim[a] << "]; const " << IT
                        << " c" << a << " = rem_ - q" << a << " * (" << IT << ")(unsigned long long)p.a[" << p_dim[a] << "]; rem_ = q" << a
                        << "; ";
                } else {
                    dec << "const int q" << a << " = (int)mjt_div((unsigned)rem_, mjt_unpack_divmod((unsigned long long)p.a[" << p_dim[a] + 1
                        << "], 0)); const int c" << a << " = rem_ - q" << a << " * (int)(unsigned long long)p.a[" << p_dim[a] << "]; rem_ = q"
                        << a << "; ";
                }
            }
        }
        for (size_t k = 0; k < inputs.size(); k++) {
            int id = inputs[k];
            const char* T = dtype_cname(d->vars[id].dtype);
            std::string off = "e";
            if (!p_stride[k].empty()) {
                off = "(";
                for (int a = 0; a < nd; a++) {
                    if (dims[a].bcast[k]) continue;
                    off += "c" + std::to_string(a) + " * (" + IT + ")(unsigned long long)p.a[" + std::to_string(p_stride[k][a]) + "] + ";
                }
                off += "0)";
            }
            if (dims.back().bcast[k] && vec > 1) {
                loads << "const " << T << " s" << id << " = ((const " << T << "*)p.a[" << p_var[id] << "])[" << off << "]; ";
            } else {
                loads << "mjt_pack<" << T << ", VEC> in" << id << "; MJT_LD(in" << id << ", (const " << T << "*)p.a["
                      << p_var[id] << "] + " << off << "); ";
            }
        }
        for (int i = 0; i < nv; i++)
            if (d->vars[i].role == MJT_VAR_OUTPUT)
                loads << "mjt_pack<" << dtype_cname(d->vars[i].dtype) << ", VEC> out" << i << "; ";
        for (size_t k = 0; k < inputs.size(); k++) {
            int id = inputs[k];
            const char* T = dtype_cname(d->vars[id].dtype);
            if (dims.back().bcast[k] && vec > 1)
                body << "const " << T << " " << vname(id) << " = s" << id << "; ";
            else
                body << "const " << T << " " << vname(id) << " = in" << id << ".v[k]; ";
        }
        body << fused_emit_ops(d, true);
        for (int i = 0; i < nv; i++)
            if (d->vars[i].role == MJT_VAR_OUTPUT)
                stores << "MJT_ST((" << dtype_cname(d->vars[i].dtype) << "*)p.a[" << p_var[i] << "] + e, out" << i << "); ";

        std::ostringstream frag;
        frag << "#define VEC " << vec << "\n#define UNROLL " << unroll << "\n#define index_t " << IT << "\n#define NPARAM "
             << args.size() << "\n#define BLOCK " << block << "\n#define MJT_LD " << ((nt & 1) ? "mjt_load_nt" : "mjt_load")
             << "\n#define MJT_ST " << ((nt & 2) ? "mjt_store_nt" : "mjt_store") << "\n";
        frag << "#define MJT_FUSED_SCALARS " << scal.str() << "\n";
        frag << "#define MJT_FUSED_DECODE " << dec.str() << "\n";
        frag << "#define MJT_FUSED_LOADS " << loads.str() << "\n";
        frag << "#define MJT_FUSED_BODY " << body.str() << "\n";
        frag << "#define MJT_FUSED_STORES " << stores.str() << "\n";
        uint64_t h = 1469598103934665603ull;
        for (unsigned char c : frag.str()) {
            h ^= c;
            h *= 1099511628211ull;
        }
        char name[64];
        snprintf(name, sizeof(name), "mjt_fused_%dops_%016llx", d->n_ops, (unsigned long long)h);
        std::string src = std::string("#define ENTRY ") + name + "\n" + frag.str() + embedded_source("prelude.h") + "\n" +
                          embedded_source("fused.h") + "\n";
        kern = jit_get(src, name);
        std::lock_guard<std::mutex> lock(g_mu);
        g_kernels.emplace(key.str(), kern);
    }
    int64_t per_block = (int64_t)block * unroll;
    int64_t blocks = (nvec + per_block - 1) / per_block;
    MJT_CHECK(blocks < (int64_t(1) << 31), "fused: launch too large");
    jit_launch(kern, (unsigned)blocks, 1, (unsigned)block, 0, args);
}

}  // namespace mjt

extern "C" int mjt_fused_elementwise(const mjt_fused_desc* desc) {
    return mjt::guarded([&] { mjt::fused_impl(desc); });
}
