// One kernel for a fused group of broadcast / unary / binary / ternary ops
// (reference: python/jittor/src/fused_op.h:29-60; member kernels
// ops/broadcast_to_op.cc:177-194, ops/unary_op.cc:1021-1027,
// ops/binary_op.cc:563-570, ops/ternary_op.cc:84-95; intermediates live in
// registers as the reference's remove_intermediate pass arranges,
// opt/pass/remove_intermediate_pass.cc:26-47).
//
// The host generates four code fragments and the constants below:
//   VEC, UNROLL, BLOCK, index_t, NPARAM, MJT_LD / MJT_ST (plain or non-temporal access)
//   MJT_FUSED_DECODE   coordinates c0..c{n-1} of element e (only when a
//                      broadcast input needs them)
//   MJT_FUSED_LOADS    one vector (or scalar, when broadcast along the
//                      innermost axis) load per input tensor
//   MJT_FUSED_BODY     the op chain for lane element k, in topological order
//   MJT_FUSED_STORES   one vector store per output tensor
//
// Each lane owns VEC adjacent elements of the innermost axis, so full-size
// tensors move as 16-byte vectors; a workgroup covers UNROLL contiguous
// BLOCK*VEC-element runs, which keeps UNROLL independent loads in flight per
// lane.

struct Params { void* a[NPARAM]; };   // 8-byte words; typed as pointers so loads/stores use the global address space

extern "C" __global__ __launch_bounds__(BLOCK) void ENTRY(Params p) {
    const index_t nvec = (index_t)(unsigned long long)p.a[0];
    MJT_FUSED_SCALARS
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        const index_t j = ((index_t)blockIdx.x * UNROLL + u) * BLOCK + threadIdx.x;
        if (j < nvec) {
            const index_t e = j * VEC;
            MJT_FUSED_DECODE
            MJT_FUSED_LOADS
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                MJT_FUSED_BODY
            }
            MJT_FUSED_STORES
        }
    }
}
