// Matrix product without alignment requirements, for what kernels/gemm_mfma.h does not take
// (float64, leading dimensions or pointers that are not multiples of 16 bytes):
//   C[b][M][N] = sum_k A'[b][M][K] * B'[b][K][N]
// A workgroup of 256 lanes owns a 64 x 64 tile of C, a lane 4 x 4 of it; K in stages of 16 through LDS.
// Supplied by the host: TIN, TOUT (element types), TACC (float, or double for float64), A_KCONT, B_KCONT.
struct Params { void* a[12]; };   // as in kernels/gemm_mfma.h

__device__ __forceinline__ TACC mjt_to_acc(double v) { return (TACC)v; }
__device__ __forceinline__ TACC mjt_to_acc(float v) { return (TACC)v; }
__device__ __forceinline__ TACC mjt_to_acc(bfloat16 v) { return (TACC)(float)v; }
__device__ __forceinline__ TACC mjt_to_acc(float16 v) { return (TACC)(float)v; }

extern "C" __global__ __launch_bounds__(256) void ENTRY(Params p) {
    const int M = (int)(long long)p.a[3], N = (int)(long long)p.a[4], K = (int)(long long)p.a[5];
    const long long lda = (long long)p.a[6], ldb = (long long)p.a[7], ldc = (long long)p.a[8];
    const TIN* __restrict__ A = (const TIN*)p.a[0] + (long long)blockIdx.z * (long long)p.a[9];
    const TIN* __restrict__ B = (const TIN*)p.a[1] + (long long)blockIdx.z * (long long)p.a[10];
    TOUT* __restrict__ C = (TOUT*)p.a[2] + (long long)blockIdx.z * (long long)p.a[11];
    __shared__ TACC as[16][64 + 1], bs[16][64 + 1];
    const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    TACC acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = (TACC)0;
    for (int k0 = 0; k0 < K; k0 += 16) {
        // 1024 elements of each operand tile, 4 per lane; the lanes run along the operand's innermost axis
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int e = tid + i * 256;
            int row, k;
            if (A_KCONT) { k = e & 15; row = e >> 4; } else { row = e & 63; k = e >> 6; }
            TACC v = (TACC)0;
            if (m0 + row < M && k0 + k < K)
                v = mjt_to_acc(A[A_KCONT ? (long long)(m0 + row) * lda + (k0 + k) : (long long)(k0 + k) * lda + (m0 + row)]);
            as[k][row] = v;
            int col;
            if (B_KCONT) { k = e & 15; col = e >> 4; } else { col = e & 63; k = e >> 6; }
            v = (TACC)0;
            if (n0 + col < N && k0 + k < K)
                v = mjt_to_acc(B[B_KCONT ? (long long)(n0 + col) * ldb + (k0 + k) : (long long)(k0 + k) * ldb + (n0 + col)]);
            bs[k][col] = v;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < 16; k++) {
            TACC a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; i++) { a[i] = as[k][ty * 4 + i]; b[i] = bs[k][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) acc[i][j] += a[i] * b[j];
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int row = m0 + ty * 4 + i, col = n0 + tx * 4 + j;
            if (row < M && col < N) C[(long long)row * ldc + col] = (TOUT)acc[i][j];
        }
}
