// Runtime services of libmjt.so: device context, memory, events, error text
// and the run-time kernel specialiser (hiprtc + module cache).
//
// The specialiser plays the role of the reference's op compiler + jit cache
// (python/jittor/src/op_compiler.cc:1096-1100, jit_compiler.cc:195-274,
// op.cc:264-281): a kernel is identified by its complete source text, built
// once per process (and kept on disk), then looked up on every launch.
#include "common.h"
#include <hip/hiprtc.h>
#include <mutex>
#include <unordered_map>
#include <fstream>
#include <sys/stat.h>
#include <unistd.h>

namespace mjt {

static thread_local std::string g_error;
static thread_local std::string g_last_kernel;
static Context g_ctx;
static std::mutex g_jit_mutex;
static std::unordered_map<std::string, JitKernel*> g_jit_cache;
static int64_t g_jit_compiled = 0, g_jit_hits = 0;

std::recursive_mutex& api_mutex() {
    static std::recursive_mutex m;
    return m;
}

int set_error(int code, const std::string& msg) {
    g_error = msg;
    return code;
}
void set_last_kernel(const char* name) { g_last_kernel = name; }

Context& ctx() { return g_ctx; }

void require_init() {
    if (!g_ctx.ready) MJT_FAIL(MJT_ERR_NOT_INIT, "mjt_init() has not been called");
}
void require_device() {
    require_init();
    if (g_ctx.dry_run) MJT_FAIL(MJT_ERR_NOT_INIT, "compile-only mode (mjt_init(-1)) has no device");
}

static std::vector<void (*)()>& shutdown_hooks() {
    static std::vector<void (*)()> hooks;      // built on first use: registration runs during static initialisation
    return hooks;
}
void at_shutdown(void (*fn)()) { shutdown_hooks().push_back(fn); }

void* scratch(size_t bytes) {
    Context& c = ctx();
    if (c.dry_run) return (void*)(uintptr_t)0x1000;
    if (bytes > c.scratch_bytes) {
        if (c.scratch) {
            HIP_CHECK(hipStreamSynchronize(c.stream));
            HIP_CHECK(hipFree(c.scratch));
            c.scratch = nullptr;
            c.scratch_bytes = 0;
        }
        size_t want = bytes < (size_t(8) << 20) ? (size_t(8) << 20) : bytes;
        HIP_CHECK(hipMalloc(&c.scratch, want));
        c.scratch_bytes = want;
    }
    return c.scratch;
}

// ---- dtype tables ------------------------------------------------------------
static const char* k_dtype_names[MJT_DTYPE_COUNT] = {
    "void", "bool", "int8", "int16", "int32", "int64", "uint8", "uint16", "uint32",
    "uint64", "float16", "float32", "float64", "bfloat16"};
static const int k_dtype_sizes[MJT_DTYPE_COUNT] = {0, 1, 1, 2, 4, 8, 1, 2, 4, 8, 2, 4, 8, 2};
static const char* k_op_names[MJT_OP_COUNT] = {
    "pow", "maximum", "minimum", "add", "subtract", "multiply", "divide", "floor_divide",
    "mod", "less", "less_equal", "greater", "greater_equal", "equal", "not_equal",
    "left_shift", "right_shift", "logical_and", "logical_or", "logical_xor", "bitwise_and",
    "bitwise_or", "bitwise_xor", "mean", "abs", "negative", "logical_not", "bitwise_not",
    "log", "exp", "sqrt", "round", "floor", "ceil", "round_int", "floor_int", "ceil_int",
    "cast", "sin", "asin", "sinh", "asinh", "tan", "atan", "tanh", "atanh", "cos", "acos",
    "cosh", "acosh", "erf", "erfinv", "sigmoid", "void"};

int dtype_size(int d) {
    if (d <= 0 || d >= MJT_DTYPE_COUNT) MJT_FAIL(MJT_ERR_INVALID, "bad dtype code " << d);
    return k_dtype_sizes[d];
}
const char* dtype_cname(int d) {
    dtype_size(d);
    return d == MJT_BOOL ? "bool" : k_dtype_names[d];
}
bool dtype_is_float(int d) {
    return d == MJT_FLOAT16 || d == MJT_FLOAT32 || d == MJT_FLOAT64 || d == MJT_BFLOAT16;
}
bool dtype_is_int(int d) { return d >= MJT_INT8 && d <= MJT_UINT64; }
bool dtype_is_unsigned(int d) { return d >= MJT_UINT8 && d <= MJT_UINT64; }

int64_t numel(const mjt_tensor* t) {
    int64_t n = 1;
    for (int i = 0; i < t->ndim; i++) n *= t->shape[i];
    return n;
}
void check_tensor(const mjt_tensor* t, const char* what) {
    MJT_CHECK(t != nullptr, what << ": null tensor descriptor");
    MJT_CHECK(t->ndim >= 1 && t->ndim <= MJT_MAX_DIM, what << ": rank " << t->ndim << " outside 1.." << MJT_MAX_DIM);
    dtype_size(t->dtype);
    for (int i = 0; i < t->ndim; i++)
        MJT_CHECK(t->shape[i] >= 0, what << ": negative extent " << shape_str(t));
    MJT_CHECK(numel(t) == 0 || t->ptr != nullptr, what << ": null data pointer");
}
std::string shape_str(const mjt_tensor* t) {
    std::ostringstream os;
    os << "[";
    for (int i = 0; i < t->ndim; i++) os << t->shape[i] << ",";
    os << "]";
    return os.str();
}

uint64_t pack_divmod(uint64_t d) {
    if (d == 0) d = 1;
    unsigned shift = 0;
    while ((uint64_t(1) << shift) < d) shift++;
    uint64_t mul = ((uint64_t(1) << 32) * ((uint64_t(1) << shift) - d)) / d + 1;
    return (uint64_t(shift) << 32) | (mul & 0xffffffffull);
}

// ---- run-time specialisation ---------------------------------------------------
static uint64_t fnv1a(const std::string& s, uint64_t seed) {
    uint64_t h = seed;
    for (unsigned char c : s) {
        h ^= c;
        h *= 1099511628211ull;
    }
    return h;
}

static std::string cache_dir() {
    const char* env = getenv("MJT_CACHE_DIR");
    std::string d;
    if (env && *env)
        d = env;
    else {
        const char* home = getenv("HOME");
        d = std::string(home && *home ? home : "/tmp") + "/.cache/mjt";
    }
    std::string cur;
    for (size_t i = 0; i <= d.size(); i++) {
        if (i == d.size() || d[i] == '/') {
            if (!cur.empty()) mkdir(cur.c_str(), 0755);
        }
        if (i < d.size()) cur.push_back(d[i]);
    }
    return d;
}

static std::vector<char> compile_source(const std::string& source, const std::string& file) {
    hiprtcProgram prog;
    if (hiprtcCreateProgram(&prog, source.c_str(), file.c_str(), 0, nullptr, nullptr) != HIPRTC_SUCCESS)
        MJT_FAIL(MJT_ERR_COMPILE, "hiprtcCreateProgram failed");
    std::string arch = std::string("--offload-arch=") + ctx().prop.gcnArchName;
    // packed fp32 instruction selection is switched off for every device build
    const char* opts[] = {arch.c_str(), "-O3", "-std=c++17", "-munsafe-fp-atomics",
                          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
    hiprtcResult r = hiprtcCompileProgram(prog, sizeof(opts) / sizeof(opts[0]), opts);
    if (r != HIPRTC_SUCCESS) {
        size_t n = 0;
        hiprtcGetProgramLogSize(prog, &n);
        std::string log(n, '\0');
        if (n) hiprtcGetProgramLog(prog, &log[0]);
        hiprtcDestroyProgram(&prog);
        if (getenv("MJT_DUMP_FAILED")) {
            std::ofstream f(std::string(getenv("MJT_DUMP_FAILED")));
            f << source;
        }
        MJT_FAIL(MJT_ERR_COMPILE, "kernel specialisation failed (" << file << "):\n" << log);
    }
    size_t size = 0;
    hiprtcGetCodeSize(prog, &size);
    std::vector<char> code(size);
    hiprtcGetCode(prog, code.data());
    hiprtcDestroyProgram(&prog);
    return code;
}

// Writes a code object under its final name only when every byte reached the file.
static void store_code(const std::string& path, const std::vector<char>& code) {
    std::string tmp = path + "." + std::to_string((long)getpid());
    std::ofstream f(tmp, std::ios::binary);
    f.write(code.data(), (std::streamsize)code.size());
    f.close();
    if (f.good()) rename(tmp.c_str(), path.c_str());
    else unlink(tmp.c_str());
}

// The register figures of `entry` in a code object's metadata (a MessagePack map per kernel whose keys come in
// alphabetical order: .agpr_count first, .symbol and .vgpr_spill_count behind it).
static void read_register_use(const std::vector<char>& code, const std::string& entry, int* agprs, int* spilled) {
    *agprs = *spilled = -1;
    const std::string blob(code.begin(), code.end());
    auto value_at = [&](size_t pos) -> int {                  // an unsigned integer of up to 16 bits
        if (pos >= blob.size()) return -1;
        const unsigned char t = (unsigned char)blob[pos];
        if (t < 0x80) return t;
        if (t == 0xcc && pos + 1 < blob.size()) return (unsigned char)blob[pos + 1];
        if (t == 0xcd && pos + 2 < blob.size()) return ((unsigned char)blob[pos + 1] << 8) | (unsigned char)blob[pos + 2];
        return -1;
    };
    const std::string k_agpr = "\xab.agpr_count", k_sym = "\xa7.symbol", k_spill = "\xb1.vgpr_spill_count";
    const std::string want = entry + ".kd";
    for (size_t at = blob.find(k_agpr); at != std::string::npos; at = blob.find(k_agpr, at + 1)) {
        const size_t next = blob.find(k_agpr, at + 1);
        const size_t sym = blob.find(k_sym, at), sp = blob.find(k_spill, at);
        if (sym == std::string::npos || sp == std::string::npos || (next != std::string::npos && (sym > next || sp > next))) continue;
        size_t v = sym + k_sym.size();                        // the name: a string of up to 31, 255 or 65535 bytes
        if (v >= blob.size()) continue;
        const unsigned char t = (unsigned char)blob[v];
        size_t len = 0;
        if ((t & 0xe0) == 0xa0) { len = t & 0x1f; v += 1; }
        else if (t == 0xd9 && v + 1 < blob.size()) { len = (unsigned char)blob[v + 1]; v += 2; }
        else if (t == 0xda && v + 2 < blob.size()) { len = ((unsigned char)blob[v + 1] << 8) | (unsigned char)blob[v + 2]; v += 3; }
        else continue;
        if (len != want.size() || blob.compare(v, len, want) != 0) continue;
        *agprs = value_at(at + k_agpr.size());
        *spilled = value_at(sp + k_spill.size());
        return;
    }
}

JitKernel* jit_get(const std::string& source, const std::string& entry) {
    require_init();
    std::lock_guard<std::mutex> lock(g_jit_mutex);
    auto it = g_jit_cache.find(source);
    if (it != g_jit_cache.end()) {
        g_jit_hits++;
        return it->second;
    }
    std::string key = source + "\n//" + ctx().prop.gcnArchName;
    char hash[40];
    snprintf(hash, sizeof(hash), "%016llx%016llx", (unsigned long long)fnv1a(key, 1469598103934665603ull),
             (unsigned long long)fnv1a(key, 0x9e3779b97f4a7c15ull));
    std::vector<char> code;
    std::string path;
    bool use_disk = !getenv("MJT_NO_DISK_CACHE");
    if (use_disk) {
        path = cache_dir() + "/" + entry + "_" + hash + ".hsaco";
        std::ifstream f(path, std::ios::binary);
        if (f) code.assign(std::istreambuf_iterator<char>(f), std::istreambuf_iterator<char>());
    }
    if (const char* dump = getenv("MJT_DUMP_DIR")) {
        // development aid: keep the generated source next to its name
        std::ofstream f(std::string(dump) + "/" + entry + ".hip");
        f << source;
    }
    const bool from_disk = !code.empty();
    if (code.empty()) {
        code = compile_source(source, entry + ".hip");
        g_jit_compiled++;
        if (use_disk) {
            store_code(path, code);
        }
    }
    JitKernel* k = new JitKernel();
    k->name = entry;
    read_register_use(code, entry, &k->agprs, &k->spilled);
    if (!ctx().dry_run) {
        hipError_t e = hipModuleLoadData(&k->module, code.data());
        if (e != hipSuccess && from_disk) {
            // a cached file that does not load (truncated by a full disk, written by another build): drop it,
            // build from source and try once more
            (void)hipGetLastError();
            unlink(path.c_str());
            code = compile_source(source, entry + ".hip");
            g_jit_compiled++;
            store_code(path, code);
            read_register_use(code, entry, &k->agprs, &k->spilled);
            e = hipModuleLoadData(&k->module, code.data());
        }
        if (e != hipSuccess) {
            delete k;
            MJT_FAIL(MJT_ERR_DEVICE, "hipModuleLoadData(" << entry << "): " << hipGetErrorString(e));
        }
        HIP_CHECK(hipModuleGetFunction(&k->fn, k->module, entry.c_str()));
    }
    g_jit_cache.emplace(source, k);
    return k;
}

JitKernel* jit_lookup(const std::string& source) {
    std::lock_guard<std::mutex> lock(g_jit_mutex);
    auto it = g_jit_cache.find(source);
    return it == g_jit_cache.end() ? nullptr : it->second;
}

void jit_launch(JitKernel* k, unsigned grid_x, unsigned grid_y, unsigned block, unsigned shmem,
                const std::vector<uint64_t>& args) {
    size_t size = args.size() * sizeof(uint64_t);
    void* config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, (void*)args.data(), HIP_LAUNCH_PARAM_BUFFER_SIZE, &size,
                      HIP_LAUNCH_PARAM_END};
    set_last_kernel(k->name.c_str());
    if (ctx().dry_run) return;
    HIP_CHECK(hipModuleLaunchKernel(k->fn, grid_x, grid_y, 1, block, 1, 1, shmem, ctx().stream, nullptr, config));
}

// defined in aot_kernels.hip
void launch_copy(void* dst, const void* src, size_t bytes);
void launch_fill_u32(void* dst, uint32_t pattern, size_t n_words);

}  // namespace mjt

using namespace mjt;

extern "C" {

int mjt_init(int device) {
    return guarded([&] {
        Context& c = ctx();
        if (c.ready && c.device == device) return;
        MJT_CHECK(!c.ready, "mjt_init: already initialised on device " << c.device);
        if (device == -1) {
            // compile-only mode: no device is touched
            memset(&c.prop, 0, sizeof(c.prop));
            strcpy(c.prop.gcnArchName, "gfx950");
            c.prop.multiProcessorCount = 256;
            c.device = -1;
            c.dry_run = true;
            c.ready = true;
            return;
        }
        int n = 0;
        HIP_CHECK(hipGetDeviceCount(&n));
        MJT_CHECK(device >= 0 && device < n, "mjt_init: device " << device << " of " << n);
        HIP_CHECK(hipSetDevice(device));
        HIP_CHECK(hipGetDeviceProperties(&c.prop, device));
        MJT_CHECK(strncmp(c.prop.gcnArchName, "gfx950", 6) == 0,
                  "mjt_init: this library is built for gfx950 only; device is " << c.prop.gcnArchName);
        HIP_CHECK(hipStreamCreateWithFlags(&c.stream, hipStreamNonBlocking));
        reduce_static_setup(device);
        c.device = device;
        c.ready = true;
    });
}

void mjt_shutdown(void) {
    Context& c = ctx();
    if (!c.ready) return;
    if (!c.dry_run) (void)hipStreamSynchronize(c.stream);
    for (auto fn : shutdown_hooks()) fn();
    {
        std::lock_guard<std::mutex> lock(g_jit_mutex);
        for (auto& kv : g_jit_cache) {
            if (kv.second->module) (void)hipModuleUnload(kv.second->module);
            delete kv.second;
        }
        g_jit_cache.clear();
    }
    if (c.scratch && !c.dry_run) (void)hipFree(c.scratch);
    c.scratch = nullptr;
    c.scratch_bytes = 0;
    if (!c.dry_run) (void)hipStreamDestroy(c.stream);
    c.dry_run = false;
    c.stream = nullptr;
    c.ready = false;
    c.device = -1;
}

const char* mjt_last_error(void) { return g_error.c_str(); }
const char* mjt_last_kernel(void) { return g_last_kernel.c_str(); }

int mjt_get_device_info(mjt_device_info* out) {
    return guarded([&] {
        require_init();
        MJT_CHECK(out, "null output");
        memset(out, 0, sizeof(*out));
        const hipDeviceProp_t& p = ctx().prop;
        strncpy(out->name, p.name, sizeof(out->name) - 1);
        strncpy(out->arch, p.gcnArchName, sizeof(out->arch) - 1);
        out->compute_units = p.multiProcessorCount;
        out->clock_khz = p.clockRate;
        out->mem_clock_khz = p.memoryClockRate;
        out->mem_bus_bits = p.memoryBusWidth;
        out->lds_bytes_per_block = (int32_t)p.sharedMemPerBlock;
        out->wavefront = p.warpSize;
        out->hbm_bytes = p.totalGlobalMem;
        out->l2_bytes = p.l2CacheSize;
    });
}

const char* mjt_dtype_name(int d) { return (d >= 0 && d < MJT_DTYPE_COUNT) ? k_dtype_names[d] : nullptr; }
const char* mjt_op_name(int o) { return (o >= 0 && o < MJT_OP_COUNT) ? k_op_names[o] : nullptr; }
int mjt_dtype_from_name(const char* name) {
    if (!name) return MJT_ERR_INVALID;
    for (int i = 0; i < MJT_DTYPE_COUNT; i++)
        if (!strcmp(name, k_dtype_names[i])) return i;
    return set_error(MJT_ERR_INVALID, std::string("unknown dtype ") + name);
}
int mjt_op_from_name(const char* name) {
    if (!name) return MJT_ERR_INVALID;
    for (int i = 0; i < MJT_OP_COUNT; i++)
        if (!strcmp(name, k_op_names[i])) return i;   // "void" resolves to MJT_OP_VOID (dtype void is not an op)
    return set_error(MJT_ERR_INVALID, std::string("unknown op ") + name);
}

int mjt_alloc(size_t bytes, void** out) {
    return guarded([&] {
        require_device();
        MJT_CHECK(out, "null output");
        *out = nullptr;
        if (bytes == 0) bytes = 256;
        HIP_CHECK(hipMalloc(out, bytes));
    });
}
int mjt_free(void* p) {
    return guarded([&] {
        require_device();
        if (!p) return;
        HIP_CHECK(hipStreamSynchronize(ctx().stream));
        HIP_CHECK(hipFree(p));
    });
}
int mjt_h2d(void* dst, const void* src, size_t bytes) {
    return guarded([&] {
        require_device();
        if (!bytes) return;
        HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx().stream));
        HIP_CHECK(hipStreamSynchronize(ctx().stream));
    });
}
int mjt_d2h(void* dst, const void* src, size_t bytes) {
    return guarded([&] {
        require_device();
        if (!bytes) return;
        HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx().stream));
        HIP_CHECK(hipStreamSynchronize(ctx().stream));
    });
}
int mjt_d2d(void* dst, const void* src, size_t bytes) {
    return guarded([&] {
        require_device();
        if (!bytes) return;
        launch_copy(dst, src, bytes);
    });
}
int mjt_fill_u32(void* dst, uint32_t pattern, size_t n_words) {
    return guarded([&] {
        require_device();
        if (!n_words) return;
        launch_fill_u32(dst, pattern, n_words);
    });
}
int mjt_sync(void) {
    return guarded([&] {
        require_device();
        HIP_CHECK(hipStreamSynchronize(ctx().stream));
    });
}

int mjt_event_create(void** ev) {
    return guarded([&] {
        require_device();
        hipEvent_t e;
        HIP_CHECK(hipEventCreate(&e));
        *ev = (void*)e;
    });
}
int mjt_event_record(void* ev) {
    return guarded([&] {
        require_device();
        HIP_CHECK(hipEventRecord((hipEvent_t)ev, ctx().stream));
    });
}
int mjt_event_elapsed_ms(void* start, void* stop, float* ms) {
    return guarded([&] {
        require_device();
        HIP_CHECK(hipEventSynchronize((hipEvent_t)stop));
        HIP_CHECK(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    });
}
int mjt_event_destroy(void* ev) {
    return guarded([&] {
        require_device();
        HIP_CHECK(hipEventDestroy((hipEvent_t)ev));
    });
}

int mjt_jit_stats(int64_t* compiled, int64_t* cache_hits) {
    if (compiled) *compiled = g_jit_compiled;
    if (cache_hits) *cache_hits = g_jit_hits;
    return MJT_OK;
}

}  // extern "C"
