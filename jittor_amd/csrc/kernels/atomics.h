// Device atomics for the scatter update x[idx] = OP(x[idx], v)
// (reference: python/jittor/src/ops/reindex_reduce_op.cc:123-130 is a
// sequential read-modify-write; on a GPU the reference's passes turn it into
// atomicAdd / cuda_atomic_max / cuda_atomic_min, misc/cuda_atomic.h:16-84).
// Hardware atomics are used where gfx950 has them (32/64-bit integer
// add/min/max/and/or/xor, float and double add); float max/min use the
// order-preserving integer view of IEEE floats; everything else is a
// compare-and-swap loop on the containing 32- or 64-bit word.

template <class T, class F>
__device__ __forceinline__ void mjt_atomic_cas(T* addr, T val, F f) {
    if constexpr (sizeof(T) == 8) {
        unsigned long long* a = (unsigned long long*)addr;
        unsigned long long old = *a, assumed;
        do {
            assumed = old;
            T cur;
            __builtin_memcpy(&cur, &assumed, 8);
            T nv = (T)f(cur, val);
            unsigned long long nb;
            __builtin_memcpy(&nb, &nv, 8);
            if (nb == assumed) break;
            old = atomicCAS(a, assumed, nb);
        } while (old != assumed);
    } else if constexpr (sizeof(T) == 4) {
        unsigned* a = (unsigned*)addr;
        unsigned old = *a, assumed;
        do {
            assumed = old;
            T cur;
            __builtin_memcpy(&cur, &assumed, 4);
            T nv = (T)f(cur, val);
            unsigned nb;
            __builtin_memcpy(&nb, &nv, 4);
            if (nb == assumed) break;
            old = atomicCAS(a, assumed, nb);
        } while (old != assumed);
    } else {
        // 1- and 2-byte elements: update inside the aligned 32-bit word
        unsigned long long ad = (unsigned long long)addr;
        unsigned* a = (unsigned*)(ad & ~3ull);
        const unsigned shift = (unsigned)(ad & 3ull) * 8u;
        const unsigned mask = (sizeof(T) == 1 ? 0xffu : 0xffffu) << shift;
        unsigned old = *a, assumed;
        do {
            assumed = old;
            unsigned curbits = (assumed & mask) >> shift;
            T cur;
            __builtin_memcpy(&cur, &curbits, sizeof(T));
            T nv = (T)f(cur, val);
            unsigned nb = 0;
            __builtin_memcpy(&nb, &nv, sizeof(T));
            unsigned word = (assumed & ~mask) | (nb << shift);
            if (word == assumed) break;
            old = atomicCAS(a, assumed, word);
        } while (old != assumed);
    }
}

// ---- add ---------------------------------------------------------------------
template <class T> __device__ __forceinline__ void mjt_atomic_add(T* a, T v) {
    mjt_atomic_cas(a, v, [](T x, T y) { return mjt_add<T>(x, y); });
}
template <> __device__ __forceinline__ void mjt_atomic_add<float>(float* a, float v) { unsafeAtomicAdd(a, v); }
template <> __device__ __forceinline__ void mjt_atomic_add<double>(double* a, double v) { unsafeAtomicAdd(a, v); }
template <> __device__ __forceinline__ void mjt_atomic_add<int>(int* a, int v) { atomicAdd(a, v); }
template <> __device__ __forceinline__ void mjt_atomic_add<unsigned>(unsigned* a, unsigned v) { atomicAdd(a, v); }
template <> __device__ __forceinline__ void mjt_atomic_add<long long>(long long* a, long long v) {
    atomicAdd((unsigned long long*)a, (unsigned long long)v);
}
template <> __device__ __forceinline__ void mjt_atomic_add<unsigned long long>(unsigned long long* a, unsigned long long v) {
    atomicAdd(a, v);
}

// ---- maximum / minimum ----------------------------------------------------------
// std::max(cur, v) keeps cur when v is NaN (the comparison is false), so NaN
// updates are dropped.  Non-negative floats order like signed integers,
// negative floats order inversely like unsigned integers.
template <class T> __device__ __forceinline__ void mjt_atomic_maximum(T* a, T v) {
    mjt_atomic_cas(a, v, [](T x, T y) { return mjt_maximum<T>(x, y); });
}
template <class T> __device__ __forceinline__ void mjt_atomic_minimum(T* a, T v) {
    mjt_atomic_cas(a, v, [](T x, T y) { return mjt_minimum<T>(x, y); });
}
template <> __device__ __forceinline__ void mjt_atomic_maximum<float>(float* a, float v) {
    if (v != v) return;
    unsigned b = __float_as_uint(v);
    if (b >> 31) atomicMin((unsigned*)a, b); else atomicMax((int*)a, (int)b);
}
template <> __device__ __forceinline__ void mjt_atomic_minimum<float>(float* a, float v) {
    if (v != v) return;
    unsigned b = __float_as_uint(v);
    if (b >> 31) atomicMax((unsigned*)a, b); else atomicMin((int*)a, (int)b);
}
template <> __device__ __forceinline__ void mjt_atomic_maximum<double>(double* a, double v) {
    if (v != v) return;
    unsigned long long b = (unsigned long long)__double_as_longlong(v);
    if (b >> 63) atomicMin((unsigned long long*)a, b); else atomicMax((long long*)a, (long long)b);
}
template <> __device__ __forceinline__ void mjt_atomic_minimum<double>(double* a, double v) {
    if (v != v) return;
    unsigned long long b = (unsigned long long)__double_as_longlong(v);
    if (b >> 63) atomicMax((unsigned long long*)a, b); else atomicMin((long long*)a, (long long)b);
}
#define MJT_ATOMIC_INT_MINMAX(T) \
    template <> __device__ __forceinline__ void mjt_atomic_maximum<T>(T* a, T v) { atomicMax(a, v); } \
    template <> __device__ __forceinline__ void mjt_atomic_minimum<T>(T* a, T v) { atomicMin(a, v); }
MJT_ATOMIC_INT_MINMAX(int) MJT_ATOMIC_INT_MINMAX(unsigned) MJT_ATOMIC_INT_MINMAX(long long)
MJT_ATOMIC_INT_MINMAX(unsigned long long)

// ---- bitwise ---------------------------------------------------------------------
#define MJT_ATOMIC_BITWISE(NAME, HW) \
    template <class T> __device__ __forceinline__ void mjt_atomic_##NAME(T* a, T v) { \
        mjt_atomic_cas(a, v, [](T x, T y) { return mjt_##NAME<T>(x, y); }); } \
    template <> __device__ __forceinline__ void mjt_atomic_##NAME<int>(int* a, int v) { HW(a, v); } \
    template <> __device__ __forceinline__ void mjt_atomic_##NAME<unsigned>(unsigned* a, unsigned v) { HW(a, v); } \
    template <> __device__ __forceinline__ void mjt_atomic_##NAME<unsigned long long>(unsigned long long* a, unsigned long long v) { HW(a, v); } \
    template <> __device__ __forceinline__ void mjt_atomic_##NAME<long long>(long long* a, long long v) { HW((unsigned long long*)a, (unsigned long long)v); }
MJT_ATOMIC_BITWISE(bitwise_and, atomicAnd)
MJT_ATOMIC_BITWISE(bitwise_or, atomicOr)
MJT_ATOMIC_BITWISE(bitwise_xor, atomicXor)

// ---- everything else: compare-and-swap with the element-wise formula ---------------
#define MJT_ATOMIC_GENERIC(NAME) \
    template <class T> __device__ __forceinline__ void mjt_atomic_##NAME(T* a, T v) { \
        mjt_atomic_cas(a, v, [](T x, T y) { return mjt_##NAME<T>(x, y); }); }
MJT_ATOMIC_GENERIC(multiply) MJT_ATOMIC_GENERIC(subtract) MJT_ATOMIC_GENERIC(divide)
MJT_ATOMIC_GENERIC(floor_divide) MJT_ATOMIC_GENERIC(mod) MJT_ATOMIC_GENERIC(pow)
MJT_ATOMIC_GENERIC(less) MJT_ATOMIC_GENERIC(less_equal) MJT_ATOMIC_GENERIC(greater)
MJT_ATOMIC_GENERIC(greater_equal) MJT_ATOMIC_GENERIC(equal) MJT_ATOMIC_GENERIC(not_equal)
MJT_ATOMIC_GENERIC(left_shift) MJT_ATOMIC_GENERIC(right_shift) MJT_ATOMIC_GENERIC(logical_and)
MJT_ATOMIC_GENERIC(logical_or) MJT_ATOMIC_GENERIC(logical_xor)
// "void": plain store, the value written last stays
template <class T> __device__ __forceinline__ void mjt_atomic_void(T* a, T v) { *a = v; }
