// Direct form of the meta-op convolution for shapes the MFMA kernel does not
// cover: one lane per output element, the reference's loop order (c, kh, kw)
// with float products and a float32 accumulator
// (python/jittor/nn.py:1251-1262, python/jittor/src/ops/reduce_op.cc:374-399).
// With G_ > 1 the channels fall into G_ groups: output channel ko belongs to group ko / (K_ / G_) and
// sees the C_ input channels of that group only (python/jittor/nn.py:1272-1294); x has C_ * G_ channels.
// Supplied by the host: TIN (element type of x and w), TOUT, G_, IDX (int when every element index fits 31 bits,
// else long long: 64-bit index arithmetic costs a third of this kernel's time) and the geometry (C_ = channels per group).

struct Params { void* a[4]; };   // 8-byte words; typed as pointers so loads/stores use the global address space   // x, w, y, number of outputs

extern "C" __global__ __launch_bounds__(256) void ENTRY(Params p) {
    const TIN* __restrict__ xp = (const TIN*)p.a[0];
    const TIN* __restrict__ wp = (const TIN*)p.a[1];
    TOUT* __restrict__ yp = (TOUT*)p.a[2];
    const IDX total = (IDX)(unsigned long long)p.a[3];
    const IDX o = (IDX)blockIdx.x * 256 + threadIdx.x;
    if (o >= total) return;
    const int ow = (int)(o % OW_);
    const int oh = (int)((o / OW_) % OH_);
    const int ko = (int)((o / ((IDX)OW_ * OH_)) % K_);
    const IDX n = o / ((IDX)OW_ * OH_ * K_);
    const int cbase = (ko / (K_ / G_)) * C_;          // first input channel of ko's group
    float acc = 0.0f;
    for (int c = 0; c < C_; c++)
        for (int kh = 0; kh < R_; kh++)
            for (int kw = 0; kw < S_; kw++) {
                const int ih = oh * SH - PH + kh * DH, iw = ow * SW - PW + kw * DW;
                const bool ov = ih < 0 || ih >= H_ || iw < 0 || iw >= W_;
                const float xv = ov ? 0.0f : (float)xp[((n * (C_ * G_) + cbase + c) * H_ + ih) * W_ + iw];
                const float wv = (float)wp[(((IDX)ko * C_ + c) * R_ + kh) * S_ + kw];
                acc = acc + xv * wv;
            }
    yp[o] = (TOUT)acc;
}
