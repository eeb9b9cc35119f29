/* mjt.h -- C ABI of libmjt.so: the MI355X (gfx950) execution path for
 * Jittor's meta-operators.
 *
 * Every entry point returns 0 on success or a negative mjt_status; the text
 * of the last failure on the calling thread is available from
 * mjt_last_error().  Nothing throws or aborts across this boundary.  All
 * tensor buffers are dense, row-major device memory owned by the caller
 * (the reference allocates every group output before calling the kernel,
 * python/jittor/src/executor.cc:575-577, and kernels only read
 * Var::mem_ptr/shape/dtype, python/jittor/src/var.h:18-49).  Work is queued
 * on one stream per device and is asynchronous; mjt_sync() waits for it.
 * Entry points may be called from several host threads: the library takes
 * one lock per call, so the calls (and the kernels they queue) run one after
 * the other.
 *
 * Paths in the citations below are relative to python/jittor/src/ of the
 * reference tree.
 */
#ifndef MJT_H_
#define MJT_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MJT_MAX_DIM 10 /* ops/reindex_op.cc:43: at most 10 dims */

typedef enum {
    MJT_OK = 0,
    MJT_ERR_INVALID = -1,   /* bad descriptor (the reference's CHECK/ASSERT) */
    MJT_ERR_UNSUPPORTED = -2,
    MJT_ERR_COMPILE = -3,   /* runtime kernel specialisation failed */
    MJT_ERR_DEVICE = -4,    /* HIP runtime error */
    MJT_ERR_NOT_INIT = -5,
    MJT_ERR_NOT_READY = -6  /* an allocation-free entry point would have to build or load a kernel */
} mjt_status;

/* dtype codes: order of misc/nano_string.h:17-31 */
typedef enum {
    MJT_VOID = 0, MJT_BOOL, MJT_INT8, MJT_INT16, MJT_INT32, MJT_INT64,
    MJT_UINT8, MJT_UINT16, MJT_UINT32, MJT_UINT64, MJT_FLOAT16, MJT_FLOAT32,
    MJT_FLOAT64, MJT_BFLOAT16, MJT_DTYPE_COUNT
} mjt_dtype;

/* op codes: order of misc/nano_string.h:33-89 (binary ops, then unary ops).
 * MJT_OP_VOID is the "void" reduce op of ops/reindex_reduce_op.cc:34. */
typedef enum {
    MJT_OP_POW = 0, MJT_OP_MAXIMUM, MJT_OP_MINIMUM, MJT_OP_ADD,
    MJT_OP_SUBTRACT, MJT_OP_MULTIPLY, MJT_OP_DIVIDE, MJT_OP_FLOOR_DIVIDE,
    MJT_OP_MOD, MJT_OP_LESS, MJT_OP_LESS_EQUAL, MJT_OP_GREATER,
    MJT_OP_GREATER_EQUAL, MJT_OP_EQUAL, MJT_OP_NOT_EQUAL, MJT_OP_LEFT_SHIFT,
    MJT_OP_RIGHT_SHIFT, MJT_OP_LOGICAL_AND, MJT_OP_LOGICAL_OR,
    MJT_OP_LOGICAL_XOR, MJT_OP_BITWISE_AND, MJT_OP_BITWISE_OR,
    MJT_OP_BITWISE_XOR, MJT_OP_MEAN,
    MJT_OP_ABS, MJT_OP_NEGATIVE, MJT_OP_LOGICAL_NOT, MJT_OP_BITWISE_NOT,
    MJT_OP_LOG, MJT_OP_EXP, MJT_OP_SQRT, MJT_OP_ROUND, MJT_OP_FLOOR,
    MJT_OP_CEIL, MJT_OP_ROUND_INT, MJT_OP_FLOOR_INT, MJT_OP_CEIL_INT,
    MJT_OP_CAST, MJT_OP_SIN, MJT_OP_ASIN, MJT_OP_SINH, MJT_OP_ASINH,
    MJT_OP_TAN, MJT_OP_ATAN, MJT_OP_TANH, MJT_OP_ATANH, MJT_OP_COS,
    MJT_OP_ACOS, MJT_OP_COSH, MJT_OP_ACOSH, MJT_OP_ERF, MJT_OP_ERFINV,
    MJT_OP_SIGMOID, MJT_OP_VOID, MJT_OP_COUNT
} mjt_op;

/* Dense row-major tensor: the fields a kernel reads from a reference Var
 * (var.h:18-49: mem_ptr, shape, dtype; no strides). */
typedef struct {
    void*   ptr;
    int32_t dtype;               /* mjt_dtype */
    int32_t ndim;                /* 1..MJT_MAX_DIM */
    int64_t shape[MJT_MAX_DIM];
} mjt_tensor;

typedef struct {
    char     name[256];
    char     arch[64];
    int32_t  compute_units;
    int32_t  clock_khz;
    int32_t  mem_clock_khz;
    int32_t  mem_bus_bits;
    int32_t  lds_bytes_per_block;
    int32_t  wavefront;
    uint64_t hbm_bytes;
    uint64_t l2_bytes;
} mjt_device_info;

/* ---- runtime ---------------------------------------------------------- */
/* device >= 0: bind to that gfx950 device.  device == -1: compile-only mode
 * for build checks on a machine without a GPU -- every entry point validates
 * its descriptors and specialises + compiles its kernels for gfx950, but
 * nothing is allocated or launched. */
int         mjt_init(int device);
void        mjt_shutdown(void);
const char* mjt_last_error(void);
int         mjt_get_device_info(mjt_device_info* out);
const char* mjt_dtype_name(int dtype);
const char* mjt_op_name(int op);
int         mjt_dtype_from_name(const char* name);   /* <0 if unknown */
int         mjt_op_from_name(const char* name);      /* <0 if unknown */

/* Device memory.  Replaces Var::alloc / Allocator::alloc (var.cc:114-127). */
int mjt_alloc(size_t bytes, void** out);
int mjt_free(void* p);
int mjt_h2d(void* dst, const void* src, size_t bytes);   /* synchronous */
int mjt_d2h(void* dst, const void* src, size_t bytes);   /* synchronous */
int mjt_d2d(void* dst, const void* src, size_t bytes);   /* copy kernel, async */
int mjt_fill_u32(void* dst, uint32_t pattern, size_t n_words); /* async */
int mjt_sync(void);

/* Timing on the library's stream (the role of Profiler::record_and_run,
 * profiler/profiler.cc:229-347). */
int mjt_event_create(void** ev);
int mjt_event_record(void* ev);
int mjt_event_elapsed_ms(void* start, void* stop, float* ms); /* waits for stop */
int mjt_event_destroy(void* ev);

/* ---- ReduceOp: ops/reduce_op.cc:374-399 -------------------------------
 * y = reduce(x, op) over the axes set in reduce_mask (bit d = axis d of x is
 * reduced, ops/reduce_op.h:14).  y->shape is the kept axes (with or without
 * 1s for reduced axes: only the element count is checked).  Accumulation is
 * in y->dtype starting from the identity init_OP
 * (type/common_op_type.cc:116-117,142-151: lowest()/max() for max/min). */
int mjt_reduce(const mjt_tensor* x, const mjt_tensor* y, int op, uint32_t reduce_mask);

/* mjt_reduce for callers that may not allocate device memory (code under HIP
 * graph capture, serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  Same arguments, same kernels and the same
 * results as mjt_reduce; the partial results of a two-pass reduction go to a
 * fixed array in device memory (MJT_STATIC_SCRATCH_BYTES per device, held
 * until the process ends) instead of the growing scratch arena.  The call
 * allocates nothing: a reduction whose partial results need more than the
 * array holds fails with MJT_ERR_UNSUPPORTED, and one whose kernels are not
 * loaded yet with MJT_ERR_NOT_READY (run mjt_reduce once with a descriptor
 * of the same dtypes, op, mask and shape beforehand, outside the region that
 * may not allocate: building and loading a kernel allocates).  All calls on a
 * device share the array: calls that overlap in time on one device race;
 * calls queued on the library's stream do not overlap.  Nothing in the array
 * has to be cleared between calls (every partial result is written before
 * it is read). */
#define MJT_STATIC_SCRATCH_BYTES (4u << 20)
int mjt_reduce_static(const mjt_tensor* x, const mjt_tensor* y, int op, uint32_t reduce_mask);

/* ---- ReindexOp: ops/reindex_op.cc:111-139 -----------------------------
 * y[i..] = overflow ? Tx(overflow_value) : x[idx_0(i..), ..., idx_{XDIM-1}(i..)]
 * indexes[d] and overflow_conditions[k] are C integer expressions over
 * i0..i{YDIM-1}, xshapeK, yshapeK, xstrideK, ystrideK, XDIM, YDIM and
 * @eK(a,b,..) = extras[K] at that coordinate (ops/reindex_op.h:58-68,
 * op_compiler.cc:665-699).  n_indexes must equal x->ndim
 * (ops/reindex_op.cc:83).  y->dtype must equal x->dtype. */
int mjt_reindex(const mjt_tensor* x, const mjt_tensor* y,
                int n_indexes, const char* const* indexes,
                double overflow_value,
                int n_overflow_conditions, const char* const* overflow_conditions,
                int n_extras, const mjt_tensor* extras);

/* ---- ReindexReduceOp: ops/reindex_reduce_op.cc:93-131 -----------------
 * x (the output, shape given) is filled with init_OP, then for every
 * coordinate of y (the input): x[idx(i..)] = OP(x[idx(i..)], y[i..]) unless
 * overflow.  op is a binary op other than mean, or MJT_OP_VOID
 * (ops/reindex_reduce_op.cc:34).  n_indexes must equal x->ndim (:66).
 * Updates are applied with device atomics: for float add the summation
 * order is not the reference's sequential order. */
int mjt_reindex_reduce(const mjt_tensor* y, const mjt_tensor* x, int op,
                       int n_indexes, const char* const* indexes,
                       int n_overflow_conditions, const char* const* overflow_conditions,
                       int n_extras, const mjt_tensor* extras);

/* ReindexOp fused with the ReduceOp that consumes it: z = reduce(reindex(x,
 * yshape, indexes, overflow_value, overflow_conditions, extras), op) over the
 * last n_reduced axes of the reindex result, which is never written (the
 * reference fuses a reindex -- a broadcast-type op -- with its consumer,
 * executor.cc:555; this is the pooling group of python/jittor/pool.py:200-208).
 * yshape gives the shape of the reindex result (its pointer is not used);
 * z holds the kept axes, accumulation in z's dtype (float32 for 16-bit float
 * results, rounded once) from the identity of op; op is add, mean, maximum,
 * minimum or multiply. */
int mjt_reindex_then_reduce(const mjt_tensor* x, const mjt_tensor* yshape, const mjt_tensor* z,
                            int op, int n_reduced,
                            int n_indexes, const char* const* indexes, double overflow_value,
                            int n_overflow_conditions, const char* const* overflow_conditions,
                            int n_extras, const mjt_tensor* extras);

/* ---- fused element-wise group: fused_op.h:29-60 -----------------------
 * One kernel for a group of broadcast / unary / binary / ternary ops
 * (ops/broadcast_to_op.cc:177-194, ops/unary_op.cc:1021-1027,
 * ops/binary_op.cc:563-570, ops/ternary_op.cc:84-95) over one iteration
 * space.  vars[] mirrors FusedOp::vars (role 0 input / 1 intermediate /
 * 2 output, fused_op.h:13-20) plus by-value scalars (ops/array_op.cc:56-60);
 * ops[] is FusedOp::ops in topological order. */
typedef enum {
    MJT_VAR_INPUT = 0, MJT_VAR_INTERMEDIATE = 1, MJT_VAR_OUTPUT = 2,
    MJT_VAR_SCALAR = 3,
    /* mjt_fused_reindex_reduce only: a tensor of the scatter target's shape read through the scatter's own index
     * program (the reindex of the forward pass, recomputed instead of stored) */
    MJT_VAR_GATHERED = 4
} mjt_var_role;

typedef struct {
    int32_t role;        /* mjt_var_role */
    int32_t dtype;
    void*   ptr;         /* input / output */
    double  fvalue;      /* scalar: value when dtype is floating */
    int64_t ivalue;      /* scalar: value when dtype is integer / bool */
    /* inputs only: axes (of the iteration space) along which this tensor has
     * extent 1 and is broadcast; 0 for a full-size tensor */
    uint32_t bcast_mask;
    uint32_t reserved;
} mjt_fused_var;

typedef enum {
    MJT_FOP_UNARY = 0, MJT_FOP_BINARY = 1, MJT_FOP_TERNARY = 2,
    MJT_FOP_BROADCAST = 3
} mjt_fused_kind;

typedef struct {
    int32_t kind;        /* mjt_fused_kind */
    int32_t op;          /* mjt_op for unary / binary */
    int32_t in[3];       /* indices into vars[]; ternary: cond, x, y */
    int32_t out;         /* index into vars[] */
} mjt_fused_op;

typedef struct {
    int32_t ndim;
    int64_t shape[MJT_MAX_DIM];   /* iteration space = shape of every output */
    int32_t n_vars;
    const mjt_fused_var* vars;
    int32_t n_ops;
    const mjt_fused_op* ops;
} mjt_fused_desc;

int mjt_fused_elementwise(const mjt_fused_desc* desc);

/* A fused group that ends in a reduce (executor.cc:555 lets element, broadcast
 * and reduce ops share a group; fused_op.cc:41-118): `desc` describes the
 * element-wise part over the shape of the reduce input and has exactly one
 * output var -- the reduce input, which is never written to memory (its ptr
 * is ignored).  A tensor input has the full shape (bcast_mask 0) or is
 * broadcast along exactly the reduced axes (bcast_mask == reduce_mask on the
 * axes of extent > 1: one value per output, e.g. the mean inside a variance);
 * scalars are by value; other groups return MJT_ERR_UNSUPPORTED and run as
 * mjt_fused_elementwise followed by mjt_reduce.  y, op and reduce_mask as in
 * mjt_reduce. */
int mjt_fused_reduce(const mjt_fused_desc* desc, const mjt_tensor* y, int op, uint32_t reduce_mask);

/* A fused group that ends in a ReindexReduceOp (element, broadcast, reindex and
 * reduce-type ops share a group in the reference, executor.cc:555; this is the
 * gradient of pooling, python/jittor/pool.py:200-208 differentiated): `desc`
 * describes the element-wise part over the shape of the scatter's input y and
 * has exactly one output var -- that input, never written to memory.  Tensor
 * inputs have y's shape or are broadcast along the axes of their bcast_mask;
 * MJT_VAR_GATHERED inputs have x's shape and are read at the element the
 * scatter's index program points to.  x, op and the index program as in
 * mjt_reindex_reduce (x's dtype is the output var's). */
int mjt_fused_reindex_reduce(const mjt_fused_desc* desc, const mjt_tensor* x, int op,
                             int n_indexes, const char* const* indexes,
                             int n_overflow_conditions, const char* const* overflow_conditions,
                             int n_extras, const mjt_tensor* extras);

/* ---- where ------------------------------------------------------------
 * The positions of the non-zero elements of `cond` (any dtype; -0.0 is zero,
 * NaN is not), in row-major order, as one int32 tensor per axis of cond
 * (python/jittor/src/ops/where_op.cc:20-60; what x[mask] and x[mask] = v with a
 * boolean mask are built from).  The length of the result depends on the
 * data: mjt_where_count returns it (one counting pass and a synchronous
 * 8-byte copy, as the reference's executor fixes the op's uncertain shape once
 * it has run), the caller allocates cond->ndim tensors int32 [count] and
 * passes them to mjt_where, which writes at most `count` positions. */
int mjt_where_count(const mjt_tensor* cond, int64_t* count);
int mjt_where(const mjt_tensor* cond, int64_t count, const mjt_tensor* outs);

/* ---- meta-op convolution ----------------------------------------------
 * The group reindex + broadcast + multiply + reduce.add that
 * python/jittor/nn.py:1251-1262 builds and opt/tuner/conv_tuner.cc:218-411
 * recognises; the parameters are the ones the matcher solves for
 * (conv_tuner.cc:333-356).  x [N,C,H,W], w [K,C,R,S], y [N,K,OH,OW].
 * x and w are bfloat16, float16 or float32 (same dtype); y is float32 (the
 * accumulator) or x's dtype (narrowed by truncation for bfloat16,
 * type/fp16_compute.h:238-241, by rounding to nearest even for float16,
 * :147-198).  Out-of-range taps contribute 0. */
typedef struct {
    int32_t stride_h, stride_w, pad_h, pad_w, dil_h, dil_w;
} mjt_conv_params;

int mjt_conv2d_meta(const mjt_tensor* x, const mjt_tensor* w, const mjt_tensor* y,
                    const mjt_conv_params* p);

/* The same convolution with the weights prepared once.  The reference's relay
 * target prepares per jit key and keeps what it prepared across calls
 * (extern/cuda/cudnn/ops/cudnn_conv_op.cc:218-299: the algorithm found for a
 * key is cached and reused); here what can be kept is the rearrangement of w
 * into the order the MFMA kernel consumes, which mjt_conv2d_meta otherwise
 * repeats on every call.
 *   mjt_conv2d_meta_pack    writes that rearrangement of w into `packed`
 *                           (device memory, 16-byte aligned, at least as many
 *                           bytes as w; x and y give the shapes of the calls
 *                           that will follow, their data is not touched);
 *   mjt_conv2d_meta_packed  is mjt_conv2d_meta on weights packed by
 *                           mjt_conv2d_meta_pack for the same shapes, dtypes
 *                           and parameters (w gives the shape; its data is
 *                           not read).
 * Both return MJT_ERR_UNSUPPORTED for a convolution that does not run on
 * packed weights (float32, channel counts or widths the MFMA kernel does not
 * take, 1x1 convolutions sent to the matrix product): call mjt_conv2d_meta. */
int mjt_conv2d_meta_pack(const mjt_tensor* x, const mjt_tensor* w, const mjt_tensor* y,
                         const mjt_conv_params* p, void* packed, size_t packed_bytes);
int mjt_conv2d_meta_packed(const mjt_tensor* x, const mjt_tensor* w, const void* packed,
                           const mjt_tensor* y, const mjt_conv_params* p);

/* The grouped form (python/jittor/nn.py:1272-1294: reindex(x) * reindex(w) ->
 * reindex_reduce.add, the group count handed to the tuner as compile option
 * "G"): x [N, groups*Cg, H, W], w [K, Cg, R, S], y [N, K, OH, OW]; output
 * channel k reads the Cg input channels of group k / (K / groups).
 * groups == 1 is mjt_conv2d_meta. */
int mjt_conv2d_meta_grouped(const mjt_tensor* x, const mjt_tensor* w, const mjt_tensor* y,
                            const mjt_conv_params* p, int groups);

/* Input gradient of the same convolution (the pattern reindex_reduce.add of
 * broadcast(dy) * broadcast(w) back into x's shape that jt.grad builds;
 * opt/tuner/conv_tuner.cc:375-397 relays it to a backward-x library op,
 * extern/cuda/cudnn/ops/cudnn_conv_backward_x_op.cc):
 *   dx[n,c,h,w] = sum over (k,r,s) with h = oh*sh-ph+r*dh, w = ow*sw-pw+s*dw of dy[n,k,oh,ow] * w[k,c,r,s]
 * dy [N,K,OH,OW] and w [K,C,R,S] bfloat16, float16 or float32 (same dtype), dx
 * [N,C,H,W] float32 or their dtype; p is the forward convolution's.  Runs on
 * the forward kernels: with transposed, flipped weights for stride 1; for a
 * stride (no dilation, H and W multiples of it) as one stride-1 convolution
 * per stride phase on that phase's taps, so that no product has a zero
 * factor; otherwise on dy spread out with zeros.  Padding beyond the taps'
 * reach (p > d*(R-1)) is rejected. */
int mjt_conv2d_meta_dgrad(const mjt_tensor* dy, const mjt_tensor* w, const mjt_tensor* dx,
                          const mjt_conv_params* p);

/* Weight gradient of the same convolution (the pattern
 * reindex(x) * broadcast(dy) -> reduce.add over (n, oh, ow) that jt.grad builds;
 * opt/tuner/conv_tuner.cc:375-397 relays it to a backward-w library op,
 * extern/cuda/cudnn/ops/cudnn_conv_backward_w_op.cc):
 *   dw[k,c,r,s] = sum_{n,oh,ow} dy[n,k,oh,ow] * x[n,c,oh*sh-ph+r*dh,ow*sw-pw+s*dw]
 * x [N,C,H,W] and dy [N,K,OH,OW] bfloat16 or float16, dw [K,C,R,S] float32 or their dtype
 * (float32 accumulation, rounded once).  One MFMA kernel plus a reduce over
 * slices of images; shapes it does not cover (horizontal stride > 1, more
 * than 9 taps, left padding > 2, K % 64 != 0, an odd OW or W, a geometry whose
 * kernel would need more registers than a wave has, ...) return MJT_ERR_UNSUPPORTED
 * and are the caller's to run through mjt_matmul or mjt_conv2d_meta. */
int mjt_conv2d_meta_wgrad(const mjt_tensor* x, const mjt_tensor* dy, const mjt_tensor* dw,
                          const mjt_conv_params* p);

/* The same gradient for any geometry and for grouped convolutions
 * (python/jittor/nn.py:1272-1294: x has `groups` groups of dw->shape[1] channels,
 * dy `groups` groups of K / groups; the reference's tuner relays the grouped
 * pattern to the same backward-w library op with a group count,
 * opt/tuner/conv_tuner.cc:375-397):
 *   dw[k,c,r,s] = sum_{n,oh,ow} dy[n,k,oh,ow] * x[n,(k/(K/groups))*C+c,oh*sh-ph+r*dh,ow*sw-pw+s*dw]
 * float32, bfloat16 or float16 operands (float32 products and sums, rounded
 * once).  With groups == 1 shapes the MFMA kernel covers run on it; everything
 * else runs on a direct kernel (one workgroup per output channel x up to four
 * input channels x slice of images, sums kept in registers). */
int mjt_conv2d_meta_wgrad_grouped(const mjt_tensor* x, const mjt_tensor* dy, const mjt_tensor* dw,
                                  const mjt_conv_params* p, int groups);

/* ---- matrix product ---------------------------------------------------
 * c[n,k] = op(a) * op(b) for 2-d float operands of one dtype, op = transpose
 * when the flag is set: the call the reference relays the pattern
 * broadcast * broadcast -> reduce.add to (opt/tuner/matmul_tuner.cc:16-104 ->
 * cublas_matmul, extern/cuda/cublas/ops/cublas_matmul_op.cc:27-56,118-126).
 * With more than two dims the leading extents must be equal on a, b and c and
 * count as a batch of products (cublas_batched_matmul_op.cc:63-85,113-166).
 * c has the inputs' dtype, or float32 for 16-bit inputs; the accumulator is
 * float32 (float64 for float64).  The product runs on the library's own
 * kernels: an LDS-tiled MFMA kernel for bfloat16 / float16 / float32 operands
 * whose rows are multiples of 16 bytes, a plain kernel for the rest (float64,
 * unaligned rows).  mjt_matmul_available() is kept for callers written
 * against an earlier build that relayed to a vendor library: it returns 1. */
int mjt_matmul(const mjt_tensor* a, const mjt_tensor* b, const mjt_tensor* c, int trans_a, int trans_b);
int mjt_matmul_available(void);

/* ---- index-expression helper ------------------------------------------
 * Parses one index expression (the language of opt/expr.h:38-143 restricted
 * to what ops/reindex_op.h:58-68 allows) and, when it is affine in i0..i9
 * with integer coefficients, returns c0 and coef[0..9].  Used by the host
 * side to recognise the convolution pattern the way ConvTuner does
 * (conv_tuner.cc:312-338).  Returns 1 if affine, 0 if valid but not affine,
 * <0 on a syntax error.  Shapes are needed to fold xshapeK / yshapeK. */
int mjt_expr_affine(const char* expr, const mjt_tensor* x, const mjt_tensor* y,
                    int64_t* c0, int64_t coef[MJT_MAX_DIM]);

/* Number of kernels specialised at run time so far, and how many launches
 * reused one (the role of jit_ops / jit_fused_ops, op.cc:30, fused_op.cc:18). */
int mjt_jit_stats(int64_t* compiled, int64_t* cache_hits);

/* Name of the device kernel the most recent entry-point call on this thread
 * launched (for profiles). */
const char* mjt_last_kernel(void);

#ifdef __cplusplus
}
#endif
#endif /* MJT_H_ */
