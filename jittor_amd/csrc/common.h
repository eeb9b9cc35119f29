// Internal declarations shared by the translation units of libmjt.so.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>
#include <sstream>
#include "../../include/mjt.h"

namespace mjt {

// ---- errors ----------------------------------------------------------------
int set_error(int code, const std::string& msg);
void set_last_kernel(const char* name);

struct Error {
    int code;
    std::string msg;
};

#define MJT_FAIL(code, ...)                                 \
    do {                                                    \
        std::ostringstream _os;                             \
        _os << __VA_ARGS__;                                 \
        throw ::mjt::Error{(code), _os.str()};              \
    } while (0)

#define MJT_CHECK(cond, ...)                                \
    do {                                                    \
        if (!(cond)) MJT_FAIL(MJT_ERR_INVALID, __VA_ARGS__); \
    } while (0)

#define HIP_CHECK(expr)                                                        \
    do {                                                                       \
        hipError_t _e = (expr);                                                \
        if (_e != hipSuccess)                                                  \
            MJT_FAIL(MJT_ERR_DEVICE, #expr << ": " << hipGetErrorString(_e));  \
    } while (0)

// Every extern "C" entry point runs its body through this guard so that no
// exception crosses the C boundary.  The guard also takes the library's one lock: the context, the scratch arena
// and the growing device buffers of the convolution paths are process-wide, and work is queued on one stream, so
// calls from several host threads run one after the other (the lock is recursive: an entry point may call another).
std::recursive_mutex& api_mutex();
template <class F> int guarded(F&& f) {
    std::lock_guard<std::recursive_mutex> lock(api_mutex());
    try {
        f();
        return MJT_OK;
    } catch (const Error& e) {
        return set_error(e.code, e.msg);
    } catch (const std::exception& e) {
        return set_error(MJT_ERR_INVALID, e.what());
    } catch (...) {
        return set_error(MJT_ERR_INVALID, "unknown failure");
    }
}

// ---- device context --------------------------------------------------------
struct Context {
    bool ready = false;
    bool dry_run = false;         // device -1: specialise and compile kernels, launch nothing
    int device = -1;
    hipStream_t stream = nullptr;
    hipDeviceProp_t prop;
    void* scratch = nullptr;      // partial results of two-pass reductions etc.
    size_t scratch_bytes = 0;
};
Context& ctx();
void require_init();
void require_device();
void* scratch(size_t bytes);      // grows the scratch arena when needed
// mjt_shutdown runs these first, while the stream and the kernel modules still exist: whatever a file keeps
// beyond a call (kernel look-up tables, device buffers, library handles) is dropped there
void at_shutdown(void (*fn)());

// ---- dtype helpers ---------------------------------------------------------
int dtype_size(int dtype);
const char* dtype_cname(int dtype);          // type name inside generated kernels
bool dtype_is_float(int dtype);
bool dtype_is_int(int dtype);                // integer, excluding bool
bool dtype_is_unsigned(int dtype);
int64_t numel(const mjt_tensor* t);
void check_tensor(const mjt_tensor* t, const char* what);
std::string shape_str(const mjt_tensor* t);

// multiply-shift divider, packed as (shift << 32 | mul); see prelude.h
uint64_t pack_divmod(uint64_t d);

// ---- run-time specialisation ----------------------------------------------
struct JitKernel {
    hipModule_t module = nullptr;
    hipFunction_t fn = nullptr;
    std::string name;
    uint64_t state[2] = {0, 0};   // for the launcher of kernels that keep state in their code object's device memory
    // what the code object's metadata says of the entry point: accumulation registers in use and vector registers
    // moved to scratch memory (-1: not found)
    int agprs = -1, spilled = -1;
};
// Compiles `source` (which must define extern "C" __global__ `entry`) for the
// current device, or returns the cached kernel for an identical source.
JitKernel* jit_get(const std::string& source, const std::string& entry);
// The cached kernel for `source`, or nullptr: never compiles, never loads.
JitKernel* jit_lookup(const std::string& source);
// per-device set-up of the fixed scratch array behind mjt_reduce_static (op_reduce.cpp); called by mjt_init
void reduce_static_setup(int device);
// Launch with a parameter block of 8-byte words.
void jit_launch(JitKernel* k, unsigned grid_x, unsigned grid_y, unsigned block, unsigned shmem,
                const std::vector<uint64_t>& args);

// embedded kernel sources (generated from csrc/kernels/)
const char* embedded_source(const char* name);

// shared by the fused element-wise group and the reduce with an element-wise prologue (op_fused.cpp)
int64_t fused_validate(const mjt_fused_desc* d, std::vector<int>* inputs, bool outputs_need_data,
                       bool allow_gathered = false);   // returns the element count
std::string fused_emit_ops(const mjt_fused_desc* d, bool store_outputs);

// plan cache: per entry point, a string key maps to a prepared plan object
// (parsed expressions, chosen kernel); see op_*.cpp

inline uint64_t bits_of(double v) { uint64_t u; memcpy(&u, &v, 8); return u; }
inline uint64_t bits_of_ptr(const void* p) { return (uint64_t)(uintptr_t)p; }

}  // namespace mjt
