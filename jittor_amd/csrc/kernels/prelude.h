// Device-side prelude shared by every kernel that is specialised at run time.
// It holds the per-dtype formulas of the element-wise vocabulary
// (reference: python/jittor/src/type/common_op_type.cc:82-152, CPU column),
// the 16-bit float storage types (type/fp16_compute.h:144-252), vector
// load/store helpers and a multiply-shift divider.  gfx950 only.

typedef bool               mjt_bool;
typedef signed char        int8;
typedef short              int16;
typedef int                int32;
typedef long long          int64;
typedef unsigned char      uint8;
typedef unsigned short     uint16;
typedef unsigned int       uint32;
typedef unsigned long long uint64;
typedef float              float32;
typedef double             float64;

// bfloat16 <- float keeps the upper 16 bits (truncation), as the reference's
// CPU struct does (type/fp16_compute.h:238-241).
struct bfloat16 {
    unsigned short x;
    __device__ __forceinline__ bfloat16() {}
    __device__ __forceinline__ bfloat16(float f) { x = (unsigned short)(__float_as_uint(f) >> 16); }
    __device__ __forceinline__ bfloat16(double f) { x = (unsigned short)(__float_as_uint((float)f) >> 16); }
    __device__ __forceinline__ bfloat16(int f) { x = (unsigned short)(__float_as_uint((float)f) >> 16); }
    __device__ __forceinline__ bfloat16(long long f) { x = (unsigned short)(__float_as_uint((float)f) >> 16); }
    __device__ __forceinline__ bfloat16(bool f) { x = (unsigned short)(__float_as_uint((float)f) >> 16); }
    __device__ __forceinline__ operator float() const { return __uint_as_float(((unsigned)x) << 16); }
};
// float16 <- float rounds to nearest even (type/fp16_compute.h:147-198).
struct float16 {
    _Float16 h;
    __device__ __forceinline__ float16() {}
    __device__ __forceinline__ float16(float f) { h = (_Float16)f; }
    __device__ __forceinline__ float16(double f) { h = (_Float16)(float)f; }
    __device__ __forceinline__ float16(int f) { h = (_Float16)(float)f; }
    __device__ __forceinline__ float16(long long f) { h = (_Float16)(float)f; }
    __device__ __forceinline__ float16(bool f) { h = (_Float16)(float)f; }
    __device__ __forceinline__ operator float() const { return (float)h; }
};

template <class T> struct mjt_limits;
#define MJT_LIM(T, LO, HI) template <> struct mjt_limits<T> { \
    static __device__ __forceinline__ T lowest() { return LO; } \
    static __device__ __forceinline__ T max() { return HI; } };
MJT_LIM(bool, false, true)
MJT_LIM(int8, (int8)-128, (int8)127)
MJT_LIM(int16, (int16)-32768, (int16)32767)
MJT_LIM(int32, (-2147483647 - 1), 2147483647)
MJT_LIM(int64, (-9223372036854775807LL - 1), 9223372036854775807LL)
MJT_LIM(uint8, (uint8)0, (uint8)255)
MJT_LIM(uint16, (uint16)0, (uint16)65535)
MJT_LIM(uint32, 0u, 4294967295u)
MJT_LIM(uint64, 0ull, 18446744073709551615ull)
MJT_LIM(float32, -3.402823466e+38f, 3.402823466e+38f)
MJT_LIM(float64, -1.7976931348623157e+308, 1.7976931348623157e+308)
// 16-bit floats use +-32768 on the reference's CPU path (type/fp16_op_type.cc:111-112)
MJT_LIM(float16, float16(-32768.0f), float16(32768.0f))
MJT_LIM(bfloat16, bfloat16(-32768.0f), bfloat16(32768.0f))

// ---- integer divider: q = n / d for 0 <= n < 2^31, d >= 1 ----------------
struct mjt_divmod { unsigned mul; unsigned shift; unsigned div; };
__device__ __forceinline__ unsigned mjt_div(unsigned n, mjt_divmod d) {
    return (__umulhi(n, d.mul) + n) >> d.shift;
}
__device__ __forceinline__ mjt_divmod mjt_unpack_divmod(unsigned long long packed, unsigned div) {
    mjt_divmod d; d.mul = (unsigned)(packed & 0xffffffffull); d.shift = (unsigned)(packed >> 32); d.div = div; return d;
}

// ---- vector access ---------------------------------------------------------
template <int BYTES> struct mjt_vec_t;
template <> struct mjt_vec_t<1> { typedef unsigned char type; };
template <> struct mjt_vec_t<2> { typedef unsigned short type; };
template <> struct mjt_vec_t<4> { typedef unsigned int type; };
typedef unsigned int mjt_u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int mjt_u32x4 __attribute__((ext_vector_type(4)));
template <> struct mjt_vec_t<8> { typedef mjt_u32x2 type; };
template <> struct mjt_vec_t<16> { typedef mjt_u32x4 type; };
template <> struct mjt_vec_t<32> { struct type { mjt_u32x4 a, b; }; };

template <class T, int N> struct mjt_pack {
    T v[N];
};
template <class T, int N>
__device__ __forceinline__ void mjt_load(mjt_pack<T, N>& dst, const T* p) {
    typedef typename mjt_vec_t<sizeof(T) * N>::type V;
    *reinterpret_cast<V*>(&dst) = *reinterpret_cast<const V*>(p);
}
template <class T, int N>
__device__ __forceinline__ void mjt_store(T* p, const mjt_pack<T, N>& src) {
    typedef typename mjt_vec_t<sizeof(T) * N>::type V;
    *reinterpret_cast<V*>(p) = *reinterpret_cast<const V*>(&src);
}
// Streaming store: non-temporal and system scope (sc0 sc1 nt), for results that are written once and not read back by the
// kernel.  On MI355X this is the fastest policy for large outputs (a fill of 231 MB: 6.9 TB/s against 6.6 for plain
// non-temporal stores and 6.5 for ordinary ones).  Spelled out because the non-temporal builtin sets nt only.
template <class T, int N>
__device__ __forceinline__ void mjt_store_nt(T* p, const mjt_pack<T, N>& src) {
    constexpr int BYTES = (int)(sizeof(T) * N);
    if constexpr (BYTES == 16) {
        asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1 nt" : : "v"(p), "v"(*reinterpret_cast<const mjt_u32x4*>(&src)) : "memory");
    } else if constexpr (BYTES == 8) {
        typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
        asm volatile("global_store_dwordx2 %0, %1, off sc0 sc1 nt" : : "v"(p), "v"(*reinterpret_cast<const u32x2*>(&src)) : "memory");
    } else if constexpr (BYTES == 4) {
        asm volatile("global_store_dword %0, %1, off sc0 sc1 nt" : : "v"(p), "v"(*reinterpret_cast<const unsigned*>(&src)) : "memory");
    } else if constexpr (BYTES == 2) {
        asm volatile("global_store_short %0, %1, off sc0 sc1 nt" : : "v"(p), "v"((unsigned)*reinterpret_cast<const unsigned short*>(&src)) : "memory");
    } else if constexpr (BYTES == 1) {
        asm volatile("global_store_byte %0, %1, off sc0 sc1 nt" : : "v"(p), "v"((unsigned)*reinterpret_cast<const unsigned char*>(&src)) : "memory");
    } else {
        mjt_store(p, src);
    }
}
template <class T, int N>
__device__ __forceinline__ void mjt_load_nt(mjt_pack<T, N>& dst, const T* p) {
    if constexpr (sizeof(T) * N <= 16) {
        typedef typename mjt_vec_t<sizeof(T) * N>::type V;
        *reinterpret_cast<V*>(&dst) = __builtin_nontemporal_load(reinterpret_cast<const V*>(p));
    } else {
        mjt_load(dst, p);
    }
}

// ---- element-wise formulas -------------------------------------------------
// Each returns the natural C++ type of the reference's expression; the caller
// converts to the destination dtype on store.  Fused intermediates are `auto`
// temporaries in the reference (opt/kernel_ir.cc:958-968), so they keep that
// natural type here as well.
template <class T> struct mjt_is_f32 { static const bool v = false; };
template <> struct mjt_is_f32<float> { static const bool v = true; };
template <class T> struct mjt_is_f64 { static const bool v = false; };
template <> struct mjt_is_f64<double> { static const bool v = true; };
template <class T> struct mjt_is_fp { static const bool v = false; };
template <> struct mjt_is_fp<float> { static const bool v = true; };
template <> struct mjt_is_fp<double> { static const bool v = true; };
template <> struct mjt_is_fp<float16> { static const bool v = true; };
template <> struct mjt_is_fp<bfloat16> { static const bool v = true; };

// math in the working precision of the argument (std:: overload rules:
// float stays float, 16-bit floats go through float, integers use double)
template <class T> struct mjt_mt { typedef double type; };
template <> struct mjt_mt<float> { typedef float type; };
template <> struct mjt_mt<float16> { typedef float type; };
template <> struct mjt_mt<bfloat16> { typedef float type; };
#define MJT_M(T) typename mjt_mt<T>::type

// exp in float, branch-free: n = rint(x*log2(e)); the reduced argument
// x*log2(e) - n comes from two fused multiply-adds with log2(e) split in two
// floats, so it carries one rounding of 2^-25; then the hardware exp2 and a
// scaling by 2^n (about 1.5 ulp in all).  Beyond |x| = 150, where e^x and 2^x
// are both 0 or inf, and for NaN, exp2(x) itself is the answer.
__device__ __forceinline__ float mjt_expf(float x) {
    const bool far = !(__builtin_fabsf(x) <= 150.0f);
    const float n = __builtin_rintf(x * 0x1.715476p+0f);
    const float f = __builtin_fmaf(x, 0x1.4ae0c0p-26f, __builtin_fmaf(x, 0x1.715476p+0f, -n));
    return __builtin_ldexpf(__builtin_amdgcn_exp2f(far ? x : f), far ? 0 : (int)n);
}
// 1/d for finite d >= 1: hardware reciprocal and one Newton step (within 1 ulp)
__device__ __forceinline__ float mjt_rcp_ge1(float d) {
    const float r = __builtin_amdgcn_rcpf(d);
    return __builtin_fmaf(__builtin_fmaf(-d, r, 1.0f), r, r);
}

#define MJT_MATH1(NAME, F32, F64) \
    __device__ __forceinline__ float mjt_m_##NAME(float x) { return F32(x); } \
    __device__ __forceinline__ double mjt_m_##NAME(double x) { return F64(x); }
MJT_MATH1(log, logf, log) MJT_MATH1(exp, mjt_expf, exp) MJT_MATH1(sqrt, sqrtf, sqrt)
MJT_MATH1(round, roundf, round) MJT_MATH1(floor, floorf, floor) MJT_MATH1(ceil, ceilf, ceil)
MJT_MATH1(sin, sinf, sin) MJT_MATH1(asin, asinf, asin) MJT_MATH1(sinh, sinhf, sinh)
MJT_MATH1(asinh, asinhf, asinh) MJT_MATH1(tan, tanf, tan) MJT_MATH1(atan, atanf, atan)
MJT_MATH1(tanh, tanhf, tanh) MJT_MATH1(atanh, atanhf, atanh) MJT_MATH1(cos, cosf, cos)
MJT_MATH1(acos, acosf, acos) MJT_MATH1(cosh, coshf, cosh) MJT_MATH1(acosh, acoshf, acosh)
MJT_MATH1(erf, erff, erf)

// misc/cpu_math.cc:18-52: rational start, two Newton steps
template <class T> __device__ __forceinline__ T mjt_erfinv_t(T y) {
    const T a0 = T(0.886226899), a1 = T(-1.645349621), a2 = T(0.914624893), a3 = T(-0.140543331);
    const T b0 = T(-2.118377725), b1 = T(1.442710462), b2 = T(-0.329097515), b3 = T(0.012229801);
    const T c0 = T(-1.970840454), c1 = T(-1.624906493), c2 = T(3.429567803), c3 = T(1.641345311);
    const T d0 = T(3.543889200), d1 = T(1.637067800);
    T ya = y < T(0) ? -y : y;
    if (ya > T(1)) return T(__builtin_nanf(""));
    if (ya == T(1)) return y < T(0) ? T(-__builtin_inff()) : T(__builtin_inff());
    T x;
    if (ya <= T(0.7)) {
        T z = y * y;
        T num = (((a3 * z + a2) * z + a1) * z + a0);
        T dem = ((((b3 * z + b2) * z + b1) * z + b0) * z + T(1));
        x = y * num / dem;
    } else {
        T z = mjt_m_sqrt(-mjt_m_log((T(1) - ya) / T(2)));
        T num = ((c3 * z + c2) * z + c1) * z + c0;
        T dem = (d1 * z + d0) * z + T(1);
        x = (y < T(0) ? -num : num) / dem;
    }
    const T k = T(2) / T(1.7724538509055159);
    x = x - (mjt_m_erf(x) - y) / (k * mjt_m_exp(-x * x));
    x = x - (mjt_m_erf(x) - y) / (k * mjt_m_exp(-x * x));
    return x;
}

#define MJT_UN(NAME) template <class Tz, class X> __device__ __forceinline__ auto mjt_##NAME(X x)
MJT_UN(logical_not) { return !x; }
MJT_UN(bitwise_not) { return ~x; }
MJT_UN(negative) { return -x; }
template <class Tz> __device__ __forceinline__ auto mjt_abs(float x) { return fabsf(x); }
template <class Tz> __device__ __forceinline__ auto mjt_abs(double x) { return fabs(x); }
template <class Tz> __device__ __forceinline__ auto mjt_abs(float16 x) { return fabsf((float)x); }
template <class Tz> __device__ __forceinline__ auto mjt_abs(bfloat16 x) { return fabsf((float)x); }
template <class Tz> __device__ __forceinline__ auto mjt_abs(long long x) { return x < 0 ? -x : x; }
template <class Tz> __device__ __forceinline__ auto mjt_abs(unsigned long long x) { return x; }
template <class Tz> __device__ __forceinline__ auto mjt_abs(unsigned x) { return x; }
template <class Tz> __device__ __forceinline__ auto mjt_abs(int x) { return x < 0 ? -x : x; }
MJT_UN(log) { return mjt_m_log((MJT_M(Tz))(Tz(x))); }
MJT_UN(exp) { return mjt_m_exp((MJT_M(Tz))(Tz(x))); }
MJT_UN(sqrt) { return mjt_m_sqrt((MJT_M(Tz))(Tz(x))); }
#define MJT_UN_M(NAME) MJT_UN(NAME) { return Tz(mjt_m_##NAME((MJT_M(X))(x))); }
MJT_UN_M(round) MJT_UN_M(floor) MJT_UN_M(ceil)
MJT_UN(round_int) { return Tz(mjt_m_round((MJT_M(X))(x))); }
MJT_UN(floor_int) { return Tz(mjt_m_floor((MJT_M(X))(x))); }
MJT_UN(ceil_int) { return Tz(mjt_m_ceil((MJT_M(X))(x))); }
MJT_UN_M(sin) MJT_UN_M(asin) MJT_UN_M(sinh) MJT_UN_M(asinh) MJT_UN_M(tan) MJT_UN_M(atan)
MJT_UN_M(tanh) MJT_UN_M(atanh) MJT_UN_M(cos) MJT_UN_M(acos) MJT_UN_M(cosh) MJT_UN_M(acosh)
MJT_UN_M(erf)
MJT_UN(erfinv) { return mjt_erfinv_t((MJT_M(X))(x)); }
MJT_UN(cast) { return Tz(x); }
// Tz(1.0f/(1.0f+exp(min(Tz(-x), Tz(30 | 300)))))
MJT_UN(sigmoid) {
    typedef MJT_M(Tz) M;
    M t = (M)(Tz(-x));
    M lim = (M)(Tz(mjt_is_f32<Tz>::v ? 30 : 300));
    M m = (lim < t) ? lim : t;
    if constexpr (mjt_is_f32<Tz>::v) return mjt_rcp_ge1(1.0f + mjt_expf(m));   // denominator in [1, 1+e^30]
    else return Tz(1.0f / (1.0f + mjt_m_exp(m)));
}

#define MJT_BIN(NAME) template <class Tz, class X, class Y> __device__ __forceinline__ auto mjt_##NAME(X x, Y y)
MJT_BIN(add) { return x + y; }
MJT_BIN(subtract) { return x - y; }
MJT_BIN(multiply) { return x * y; }
MJT_BIN(divide) { return Tz(Tz(x) / Tz(y)); }
MJT_BIN(floor_divide) { return Tz(Tz(x) / Tz(y)); }
template <class Tz, class X, class Y, bool FP32, bool FP64> struct mjt_mod_impl {
    static __device__ __forceinline__ auto f(X x, Y y) { return x % y; } };
template <class Tz, class X, class Y, bool FP64> struct mjt_mod_impl<Tz, X, Y, true, FP64> {
    static __device__ __forceinline__ auto f(X x, Y y) { return x - floorf(x / y) * y; } };
template <class Tz, class X, class Y> struct mjt_mod_impl<Tz, X, Y, false, true> {
    static __device__ __forceinline__ auto f(X x, Y y) { return x - floor(x / y) * y; } };
// float32 result: x-floor(x/y)*y; float64 x: same in double; else C remainder
MJT_BIN(mod) { return mjt_mod_impl<Tz, X, Y, mjt_is_f32<Tz>::v, mjt_is_f64<X>::v>::f(x, y); }
template <class X, class Y, bool BOTHF> struct mjt_pow_impl {
    static __device__ __forceinline__ auto f(X x, Y y) { return pow((double)x, (double)y); } };
template <class X, class Y> struct mjt_pow_impl<X, Y, true> {
    static __device__ __forceinline__ auto f(X x, Y y) { return powf((float)x, (float)y); } };
template <class T> struct mjt_is_f32like { static const bool v = false; };
template <> struct mjt_is_f32like<float> { static const bool v = true; };
template <> struct mjt_is_f32like<float16> { static const bool v = true; };
template <> struct mjt_is_f32like<bfloat16> { static const bool v = true; };
MJT_BIN(pow) { return mjt_pow_impl<X, Y, mjt_is_f32like<X>::v && mjt_is_f32like<Y>::v>::f(x, y); }
// std::max(a,b) = (a<b)?b:a ; std::min(a,b) = (b<a)?b:a
MJT_BIN(maximum) { Tz a = Tz(x), b = Tz(y); return (a < b) ? b : a; }
MJT_BIN(minimum) { Tz a = Tz(x), b = Tz(y); return (b < a) ? b : a; }
MJT_BIN(less) { return x < y; }
MJT_BIN(less_equal) { return x <= y; }
MJT_BIN(greater) { return x > y; }
MJT_BIN(greater_equal) { return x >= y; }
MJT_BIN(equal) { return x == y; }
MJT_BIN(not_equal) { return x != y; }
MJT_BIN(left_shift) { return x << y; }
MJT_BIN(right_shift) { return x >> y; }
MJT_BIN(logical_and) { return x && y; }
MJT_BIN(logical_or) { return x || y; }
MJT_BIN(logical_xor) { return bool(x) != bool(y); }
MJT_BIN(bitwise_and) { return x & y; }
MJT_BIN(bitwise_or) { return x | y; }
MJT_BIN(bitwise_xor) { return x ^ y; }
// as a plain binary op rcount is 1
MJT_BIN(mean) { return x + Tz(y) * Tz(1); }
MJT_BIN(void) { return y; }

// comparisons of the 16-bit float structs go through float
__device__ __forceinline__ bool operator<(bfloat16 a, bfloat16 b) { return (float)a < (float)b; }
__device__ __forceinline__ bool operator<(float16 a, float16 b) { return (float)a < (float)b; }

// reduce identities (type/common_op_type.cc:116-117,142-151)
template <class T> __device__ __forceinline__ T mjt_init_add() { return T(0); }
template <class T> __device__ __forceinline__ T mjt_init_mean() { return T(0); }
template <class T> __device__ __forceinline__ T mjt_init_void() { return T(0); }
template <class T> __device__ __forceinline__ T mjt_init_subtract() { return T(0); }
template <class T> __device__ __forceinline__ T mjt_init_multiply() { return T(1); }
template <class T> __device__ __forceinline__ T mjt_init_maximum() { return mjt_limits<T>::lowest(); }
template <class T> __device__ __forceinline__ T mjt_init_minimum() { return mjt_limits<T>::max(); }
template <class T> __device__ __forceinline__ T mjt_init_logical_and() { return T(true); }
template <class T> __device__ __forceinline__ T mjt_init_logical_or() { return T(false); }
template <class T> __device__ __forceinline__ T mjt_init_logical_xor() { return T(false); }
template <class T> __device__ __forceinline__ T mjt_init_bitwise_and() { return T(-1); }
template <class T> __device__ __forceinline__ T mjt_init_bitwise_or() { return T(0); }
template <class T> __device__ __forceinline__ T mjt_init_bitwise_xor() { return T(0); }
