// Direct form of the weight gradient of the meta-op convolution, for what the MFMA kernel does not cover: grouped
// and depthwise convolutions (python/jittor/nn.py:1272-1294), float32 operands, any stride / padding / dilation.
//   dw[ko, c, r, s] = sum over n, oh, ow of dy[n, ko, oh, ow] * x[n, g*C_ + c, oh*SH - PH + r*DH, ow*SW - PW + s*DW]
// with g = ko / (K_ / G_), out-of-range x reading as zero (the gradient of reindex's overflow value is nothing).
// One workgroup owns output channel ko, CT input channels of its group, TCH taps and a slice of the images; its
// lanes walk the (n, oh, ow) positions of the slice (coalesced along ow in dy and in x), keep CT*TCH float sums in
// registers and fold them at the end: across the wave with shuffles, across the waves through LDS.  The host sums the
// slices.  Supplied by the host: TIN, the geometry (C_ = input channels per group, K_ = all output channels), G_, CT,
// TCH (taps per workgroup; NTCH = chunks of taps).

struct Params { void* a[6]; };   // x, dy, partial sums (float, [slice][K_][C_][R_][S_]), images, images per slice, unused

constexpr int TAPS = R_ * S_;
constexpr int NTCH = (TAPS + TCH - 1) / TCH;
constexpr int CTILES = (C_ + CT - 1) / CT;
constexpr int OHW = OH_ * OW_;

extern "C" __global__ __launch_bounds__(256) void ENTRY(Params p) {
    const TIN* __restrict__ xp = (const TIN*)p.a[0];
    const TIN* __restrict__ dyp = (const TIN*)p.a[1];
    float* __restrict__ part = (float*)p.a[2];
    const long long n_img = (long long)(unsigned long long)p.a[3];
    const long long ips = (long long)(unsigned long long)p.a[4];
    unsigned id = blockIdx.x;
    const int tch = NTCH > 1 ? (int)(id % NTCH) : 0;
    id /= NTCH;
    const int ctile = (int)(id % CTILES);
    id /= CTILES;
    const int ko = (int)(id % K_);
    const long long slice = id / K_;
    const long long n0 = slice * ips;
    const long long n1 = n0 + ips < n_img ? n0 + ips : n_img;
    const int c0 = ctile * CT;
    const int t0 = tch * TCH;
    const long long cbase = (long long)(ko / (K_ / G_)) * C_ + c0;          // first input channel of this workgroup

    float acc[CT][TCH];
#pragma unroll
    for (int c = 0; c < CT; c++)
#pragma unroll
        for (int t = 0; t < TCH; t++) acc[c][t] = 0.0f;

    const long long npos = (n1 - n0) * OHW;
    for (long long q = threadIdx.x; q < npos; q += 256) {
        const long long n = n0 + q / OHW;
        const int pos = (int)(q % OHW);
        const int oh = pos / OW_, ow = pos - oh * OW_;
        const float dyv = (float)dyp[(n * K_ + ko) * OHW + pos];
        const TIN* __restrict__ xn = xp + (n * ((long long)C_ * G_) + cbase) * ((long long)H_ * W_);
#pragma unroll
        for (int t = 0; t < TCH; t++) {
            const int tap = t0 + t;
            if (TAPS % TCH != 0 && tap >= TAPS) break;
            const int r = tap / S_, s = tap - r * S_;
            const int ih = oh * SH - PH + r * DH, iw = ow * SW - PW + s * DW;
            const bool in = ih >= 0 && ih < H_ && iw >= 0 && iw < W_;
            const int off = in ? ih * W_ + iw : 0;
#pragma unroll
            for (int c = 0; c < CT; c++) {
                if (C_ % CT != 0 && c0 + c >= C_) break;
                const float xv = in ? (float)xn[(long long)c * (H_ * W_) + off] : 0.0f;
                acc[c][t] = acc[c][t] + dyv * xv;
            }
        }
    }

    __shared__ float fold[4][CT * TCH];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int c = 0; c < CT; c++)
#pragma unroll
        for (int t = 0; t < TCH; t++) {
            float v = acc[c][t];
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) v = v + __shfl_xor(v, off, 64);
            if (lane == 0) fold[wave][c * TCH + t] = v;
        }
    __syncthreads();
    for (int i = threadIdx.x; i < CT * TCH; i += 256) {
        const int c = i / TCH, t = i - c * TCH;
        if (c0 + c >= C_ || t0 + t >= TAPS) continue;
        const float v = (fold[0][i] + fold[1][i]) + (fold[2][i] + fold[3][i]);
        part[((slice * K_ + ko) * C_ + c0 + c) * TAPS + t0 + t] = v;
    }
}
