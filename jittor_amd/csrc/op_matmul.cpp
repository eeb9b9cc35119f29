// Plain matrix product behind the reference's matmul relay.
//
// The reference recognises broadcast * broadcast -> reduce.add over 2-d
// operands (opt/tuner/matmul_tuner.cc:16-104) and relays it to a library GEMM:
// cublas_matmul(a, b, trans_a, trans_b) on the GPU
// (extern/cuda/cublas/ops/cublas_matmul_op.cc:27-56, one GemmEx call with the
// row-major operands swapped, :118-126).  The counterpart here is rocBLAS'
// gemm_ex, opened on first use so that a process that never multiplies matrices
// never loads the library.  Float accumulation for every input type.
#include "common.h"
#include <dlfcn.h>
#include <mutex>
#include <rocblas/rocblas.h>

namespace mjt {

void launch_fill_pattern(void* dst, uint64_t pattern, int elem_size, size_t n);

namespace {
struct Blas {
    void* so = nullptr;
    rocblas_handle handle = nullptr;
    decltype(&rocblas_create_handle) create = nullptr;
    decltype(&rocblas_set_stream) set_stream = nullptr;
    decltype(&rocblas_gemm_ex) gemm_ex = nullptr;
    decltype(&rocblas_gemm_strided_batched_ex) gemm_batched = nullptr;
    bool tried = false;
};
Blas g_blas;
std::mutex g_mu;

bool blas_load() {
    std::lock_guard<std::mutex> lock(g_mu);
    if (g_blas.tried) return g_blas.gemm_ex != nullptr;
    g_blas.tried = true;
    const char* names[] = {"librocblas.so.5", "librocblas.so", "/opt/rocm/lib/librocblas.so"};
    for (const char* n : names) {
        g_blas.so = dlopen(n, RTLD_NOW | RTLD_LOCAL);
        if (g_blas.so) break;
    }
    if (!g_blas.so) return false;
    g_blas.create = (decltype(g_blas.create))dlsym(g_blas.so, "rocblas_create_handle");
    g_blas.set_stream = (decltype(g_blas.set_stream))dlsym(g_blas.so, "rocblas_set_stream");
    auto gemm = (decltype(g_blas.gemm_ex))dlsym(g_blas.so, "rocblas_gemm_ex");
    g_blas.gemm_batched = (decltype(g_blas.gemm_batched))dlsym(g_blas.so, "rocblas_gemm_strided_batched_ex");
    if (!g_blas.create || !g_blas.set_stream || !gemm || !g_blas.gemm_batched) return false;
    g_blas.gemm_ex = gemm;
    return true;
}

rocblas_datatype blas_type(int dtype) {
    switch (dtype) {
        case MJT_FLOAT32: return rocblas_datatype_f32_r;
        case MJT_FLOAT64: return rocblas_datatype_f64_r;
        case MJT_FLOAT16: return rocblas_datatype_f16_r;
        default: return rocblas_datatype_bf16_r;
    }
}
}  // namespace

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
    if (ctxt.dry_run) return;
    MJT_CHECK(a->ptr && b->ptr && c->ptr, "matmul: null data");
    if (m == 0) {                                             // an empty sum
        launch_fill_pattern(c->ptr, 0, dtype_size(c->dtype), (size_t)batch * n * k);
        return;
    }
    if (!blas_load()) MJT_FAIL(MJT_ERR_UNSUPPORTED, "matmul: rocBLAS is not available");
    {
        std::lock_guard<std::mutex> lock(g_mu);
        if (!g_blas.handle && g_blas.create(&g_blas.handle) != rocblas_status_success)
            MJT_FAIL(MJT_ERR_DEVICE, "matmul: rocblas_create_handle failed");
        // every call: the library's stream changes when it is shut down and bound again
        if (g_blas.set_stream(g_blas.handle, ctxt.stream) != rocblas_status_success) MJT_FAIL(MJT_ERR_DEVICE, "matmul: rocblas_set_stream failed");
    }
    // Row-major c[n,k] = a * b is column-major c^T[k,n] = b^T * a^T: the operands trade places and keep
    // their own transposition flags (cublas_matmul_op.cc:118-126).
    const float alpha_f = 1.0f, beta_f = 0.0f;
    const double alpha_d = 1.0, beta_d = 0.0;
    const bool f64 = a->dtype == MJT_FLOAT64;
    const void* alpha = f64 ? (const void*)&alpha_d : (const void*)&alpha_f;
    const void* beta = f64 ? (const void*)&beta_d : (const void*)&beta_f;
    const rocblas_operation opb = trans_b ? rocblas_operation_transpose : rocblas_operation_none;
    const rocblas_operation opa = trans_a ? rocblas_operation_transpose : rocblas_operation_none;
    const rocblas_int ldb = (rocblas_int)(trans_b ? m : k), lda = (rocblas_int)(trans_a ? n : m);
    const rocblas_datatype tc = f64 ? rocblas_datatype_f64_r : rocblas_datatype_f32_r;
    rocblas_status st;
    if (batch == 1)
        st = g_blas.gemm_ex(g_blas.handle, opb, opa, (rocblas_int)k, (rocblas_int)n, (rocblas_int)m, alpha, b->ptr,
                            blas_type(b->dtype), ldb, a->ptr, blas_type(a->dtype), lda, beta, c->ptr, blas_type(c->dtype),
                            (rocblas_int)k, c->ptr, blas_type(c->dtype), (rocblas_int)k, tc, rocblas_gemm_algo_standard, 0, 0);
    else
        st = g_blas.gemm_batched(g_blas.handle, opb, opa, (rocblas_int)k, (rocblas_int)n, (rocblas_int)m, alpha, b->ptr,
                                 blas_type(b->dtype), ldb, (rocblas_stride)(m * k), a->ptr, blas_type(a->dtype), lda,
                                 (rocblas_stride)(share_a ? 0 : n * m), beta, c->ptr, blas_type(c->dtype), (rocblas_int)k,
                                 (rocblas_stride)(n * k), c->ptr, blas_type(c->dtype), (rocblas_int)k, (rocblas_stride)(n * k),
                                 (rocblas_int)batch, tc, rocblas_gemm_algo_standard, 0, 0);
    if (st != rocblas_status_success) MJT_FAIL(MJT_ERR_DEVICE, "matmul: rocBLAS returned " << (int)st);
    set_last_kernel(batch == 1 ? "rocblas_gemm_ex" : "rocblas_gemm_strided_batched_ex");
}

}  // namespace mjt

extern "C" int mjt_matmul(const mjt_tensor* a, const mjt_tensor* b, const mjt_tensor* c, int trans_a, int trans_b) {
    return mjt::guarded([&] { mjt::matmul_impl(a, b, c, trans_a, trans_b, false); });
}

namespace mjt {
bool matmul_available() { return blas_load(); }
}  // namespace mjt

extern "C" int mjt_matmul_available(void) {
    return mjt::blas_load() ? 1 : 0;
}
