// One-axis scatter  x[idx[i]] = OP(x[idx[i]], y[i])  for i in [0, n), idx a
// 1-d integer tensor (the pattern jt.histc and jt.scatter produce,
// reference: python/jittor/misc.py:2233; semantics
// python/jittor/src/ops/reindex_reduce_op.cc:93-131).
//
// Scattered global atomics run at about 2e10 updates/s on this chip whatever
// their scope, and a hot bin serialises them further, so this path uses none
// on its main route.  The bin axis is cut into buckets of WBINS bins (one
// bucket fits in LDS):
//   sample  a strided sample of the indices votes for the bucket that receives
//           the most updates (the "hot" bucket);
//   main    every workgroup streams its share of (idx, y): updates of the hot
//           bucket are applied to a private LDS copy of that bucket, all other
//           updates are appended to per-(workgroup, bucket) lists in scratch
//           memory (list cursors are LDS counters); at the end the private
//           copy and the list lengths are written out;
//   cold    workgroup (bucket, split) folds the lists of its bucket into a
//           private LDS copy and writes it out
//           (the number of workgroups per bucket follows the bucket's population;
//           entries that did not fit a list -- rare: a second hot region -- sit in
//           one overflow list that the first workgroup of each bucket scans);
//   final   x[bin] = merge of the partial copies of its bucket (plain stores:
//           x needs no prior fill).
//
// Supplied by the host: TX (4-byte element type), TE (index type), WBINS
// (power of two), LOGW, NBMAX (bound on the bucket count), NTHREADS, NHOT (bins kept in
// registers), MODE (0 add,
// 1 maximum, 2 minimum),
// IDENT_BITS (bit pattern of the identity).

struct Params { void* a[16]; };   // 8-byte words; typed as pointers so loads/stores use the global address space
// a[0] x          a[1] y           a[2] idx        a[3] n          a[4] bins
// a[5] control    a[6] per (elements per main workgroup)           a[7] G1 (main workgroups)
// a[8] NB (buckets)  a[9] CAP (list capacity)  a[10] counts  a[11] lists
// a[12] partial_main  a[13] partial_cold  a[14] unused  a[15] overflow list
// control: int[0] hot bucket, unsigned[1] overflow count, unsigned[64 + b] list entries of bucket b

struct mjt_pair { int bin; TX val; };

#if MODE == 0
#define LDS_UPDATE(addr, v) atomicAdd((addr), (v))
#define GLB_UPDATE(addr, v) mjt_atomic_add<TX>((addr), (v))
#define MERGE2(a, b) ((a) + (b))
#elif MODE == 1
#define LDS_UPDATE(addr, v) mjt_lds_max((addr), (v))
#define GLB_UPDATE(addr, v) mjt_atomic_maximum<TX>((addr), (v))
#define MERGE2(a, b) (((a) < (b)) ? (b) : (a))
#else
#define LDS_UPDATE(addr, v) mjt_lds_min((addr), (v))
#define GLB_UPDATE(addr, v) mjt_atomic_minimum<TX>((addr), (v))
#define MERGE2(a, b) (((b) < (a)) ? (b) : (a))
#endif

// std::max(cur, v) keeps cur when v is NaN: NaN updates are dropped
__device__ __forceinline__ void mjt_lds_max(float* a, float v) {
    if (v != v) return;
    unsigned b = __float_as_uint(v);
    if (b >> 31) atomicMin((unsigned*)a, b); else atomicMax((int*)a, (int)b);
}
__device__ __forceinline__ void mjt_lds_min(float* a, float v) {
    if (v != v) return;
    unsigned b = __float_as_uint(v);
    if (b >> 31) atomicMax((unsigned*)a, b); else atomicMin((int*)a, (int)b);
}
__device__ __forceinline__ void mjt_lds_max(int* a, int v) { atomicMax(a, v); }
__device__ __forceinline__ void mjt_lds_min(int* a, int v) { atomicMin(a, v); }
__device__ __forceinline__ void mjt_lds_max(unsigned* a, unsigned v) { atomicMax(a, v); }
__device__ __forceinline__ void mjt_lds_min(unsigned* a, unsigned v) { atomicMin(a, v); }

__device__ __forceinline__ TX mjt_ident() {
    TX t;
    unsigned ib = IDENT_BITS;
    __builtin_memcpy(&t, &ib, 4);
    return t;
}

// ---- sample -------------------------------------------------------------------------
extern "C" __global__ __launch_bounds__(1024) void ENTRY_SAMPLE(Params p) {
    const TE* __restrict__ ip = (const TE*)p.a[2];
    const long long n = (long long)(unsigned long long)p.a[3];
    const long long bins = (long long)(unsigned long long)p.a[4];
    int* control = (int*)p.a[5];
    const int NB = (int)(unsigned long long)p.a[8];
    __shared__ int votes[1024];
    __shared__ int best_votes, best_slot;
    const int group = (NB + 1023) / 1024;            // buckets per counter when there are more than 1024
    votes[threadIdx.x] = 0;
    if (threadIdx.x == 0) { best_votes = -1; best_slot = 0; }
    __syncthreads();
    // 32 runs of 64 consecutive indices spread over the input (a lone workgroup can pull only a few
    // tens of GB/s, and every isolated 4-byte sample would cost a whole 128-byte line)
    long long b[2];
    const long long runs = 32, run_stride = n / runs;
#pragma unroll
    for (int k = 0; k < 2; k++) {
        const long long r = k * 16 + (threadIdx.x >> 6);
        const long long pos = run_stride >= 64 ? r * run_stride + (threadIdx.x & 63) : (long long)threadIdx.x + k * 1024;
        b[k] = pos < n ? (long long)ip[pos] : -1;
    }
#pragma unroll
    for (int k = 0; k < 2; k++)
        if (b[k] >= 0 && b[k] < bins) atomicAdd(&votes[(int)(b[k] >> LOGW) / group], 1);
    __syncthreads();
    atomicMax(&best_votes, votes[threadIdx.x]);
    __syncthreads();
    if (votes[threadIdx.x] == best_votes) atomicMax(&best_slot, (int)threadIdx.x);
    __syncthreads();
    if (threadIdx.x == 0) {
        control[0] = best_slot * group;
        control[1] = 0;
    }
    for (int t = threadIdx.x; t < NB; t += 1024) control[64 + t] = 0;
}

// ---- main ---------------------------------------------------------------------------
extern "C" __global__ __launch_bounds__(NTHREADS) void ENTRY_MAIN(Params p) {
    const TX* __restrict__ yp = (const TX*)p.a[1];
    const TE* __restrict__ ip = (const TE*)p.a[2];
    const long long n = (long long)(unsigned long long)p.a[3];
    const long long bins = (long long)(unsigned long long)p.a[4];
    int* control = (int*)p.a[5];
    const long long per = (long long)(unsigned long long)p.a[6];
    const int NB = (int)(unsigned long long)p.a[8];
    const unsigned CAP = (unsigned)(unsigned long long)p.a[9];
    unsigned* __restrict__ counts = (unsigned*)p.a[10];
    mjt_pair* __restrict__ lists = (mjt_pair*)p.a[11];
    TX* __restrict__ pmain = (TX*)p.a[12];
    mjt_pair* __restrict__ ovf = (mjt_pair*)p.a[15];
    __shared__ TX win[WBINS];
    __shared__ unsigned cursor[NBMAX];
    __shared__ unsigned cand[NTHREADS];
    __shared__ int hotbin_s[NHOT];
    const long long hot = control[0];
    const TX ident = mjt_ident();
    const long long begin = (long long)blockIdx.x * per;
    const long long end = begin + per < n ? begin + per : n;
    const int lane = threadIdx.x & 63;

    // Phase 0: the NHOT most frequent bins of the hot bucket in the first 4*NTHREADS elements of this
    // workgroup's share.  Same-address LDS atomics serialise, so these bins are accumulated in
    // registers instead and folded into the private copy once per wave at the end.
    unsigned* hist = (unsigned*)win;
    for (int t = threadIdx.x; t < WBINS; t += NTHREADS) hist[t] = 0;
    for (int t = threadIdx.x; t < NB; t += NTHREADS) cursor[t] = 0;
    __syncthreads();
    {
        const long long i0 = begin + (long long)threadIdx.x * 4;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const long long b = i0 + k < end ? (long long)ip[i0 + k] : -1;
            if (b >= 0 && b < bins && (b >> LOGW) == hot) atomicAdd(&hist[b & (WBINS - 1)], 1u);
        }
    }
    __syncthreads();
    {
        unsigned best = 0;                                   // (count << LOGW) | local bin
        for (int t = threadIdx.x; t < WBINS; t += NTHREADS) {
            const unsigned c = (hist[t] << LOGW) | (unsigned)t;
            best = c > best ? c : best;
        }
        cand[threadIdx.x] = best;
    }
    __syncthreads();
    if (threadIdx.x < 64) {
        unsigned mine[NTHREADS / 64];
#pragma unroll
        for (int k = 0; k < NTHREADS / 64; k++) mine[k] = cand[k * 64 + lane];
        for (int r = 0; r < NHOT; r++) {
            unsigned m = 0;
#pragma unroll
            for (int k = 0; k < NTHREADS / 64; k++) m = mine[k] > m ? mine[k] : m;
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                const unsigned o = (unsigned)__shfl_xor((int)m, off, 64);
                m = o > m ? o : m;
            }
#pragma unroll
            for (int k = 0; k < NTHREADS / 64; k++) if (mine[k] == m) mine[k] = 0;
            // at least 1/128 of the sample, else the slot stays unused
            if (lane == 0) hotbin_s[r] = (m >> LOGW) >= (4 * NTHREADS) / 128 ? (int)(m & (WBINS - 1)) : -1;
        }
    }
    __syncthreads();
    int hotbin[NHOT];
    TX hotacc[NHOT];
#pragma unroll
    for (int r = 0; r < NHOT; r++) { hotbin[r] = hotbin_s[r]; hotacc[r] = ident; }
    for (int t = threadIdx.x; t < WBINS; t += NTHREADS) win[t] = ident;
    __syncthreads();

    mjt_pair* __restrict__ mylists = lists + (size_t)blockIdx.x * NB * CAP;
    auto update = [&](long long b, TX v) {
        if (b < 0 || b >= bins) return;                      // overflow: skipped
        const long long bucket = b >> LOGW;
        const int local = (int)(b & (WBINS - 1));
        if (bucket == hot) {
            bool taken = false;
#pragma unroll
            for (int r = 0; r < NHOT; r++) {
                const bool hit = local == hotbin[r];
#if MODE == 0
                hotacc[r] = hit ? hotacc[r] + v : hotacc[r];
#elif MODE == 1
                hotacc[r] = (hit && hotacc[r] < v) ? v : hotacc[r];     // false for NaN: dropped
#else
                hotacc[r] = (hit && v < hotacc[r]) ? v : hotacc[r];
#endif
                taken = taken || hit;
            }
            if (!taken) { LDS_UPDATE(&win[local], v); }
        } else {
            const unsigned pos = atomicAdd(&cursor[bucket], 1u);
            mjt_pair e;
            if (pos < CAP) {
                e.bin = local;
                e.val = v;
                mylists[(size_t)bucket * CAP + pos] = e;
            } else {
                const unsigned g = atomicAdd((unsigned*)control + 1, 1u);
                e.bin = (int)b;
                e.val = v;
                ovf[g] = e;
            }
        }
    };
    // per is a multiple of 4*NTHREADS and the bases are 16-byte aligned: full vectors first
    long long i = begin + (long long)threadIdx.x * 4;
    for (; i + 3 < end; i += (long long)NTHREADS * 4) {
        mjt_pack<TX, 4> v;
        mjt_pack<TE, 4> id;
        mjt_load_nt(v, yp + i);
        mjt_load_nt(id, ip + i);
#pragma unroll
        for (int k = 0; k < 4; k++) update((long long)id.v[k], v.v[k]);
    }
    for (; i < end; i++) update((long long)ip[i], yp[i]);    // ragged tail of the last workgroup
    // fold the register accumulators: xor-shuffle tree, then one LDS update per wave and bin
#pragma unroll
    for (int r = 0; r < NHOT; r++) {
        TX a = hotacc[r];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            int ob = __shfl_xor(*reinterpret_cast<int*>(&a), off, 64);
            const TX o = *reinterpret_cast<TX*>(&ob);
            a = MERGE2(a, o);
        }
        if (lane == 0 && hotbin[r] >= 0) { LDS_UPDATE(&win[hotbin[r]], a); }
    }
    __syncthreads();
    TX* __restrict__ out = pmain + (size_t)blockIdx.x * WBINS;
    for (int t = threadIdx.x * 4; t < WBINS; t += NTHREADS * 4) {
        mjt_pack<TX, 4> o;
#pragma unroll
        for (int k = 0; k < 4; k++) o.v[k] = win[t + k];
        mjt_store(out + t, o);
    }
    for (int t = threadIdx.x; t < NB; t += NTHREADS) {
        const unsigned c = cursor[t] < CAP ? cursor[t] : CAP;
        counts[(size_t)blockIdx.x * NB + t] = c;
        if (c) atomicAdd((unsigned*)control + 64 + t, c);     // bucket populations, read by the cold plan
    }
}


// Work plan of the cold pass, recomputed identically by every workgroup that needs it:
// bucket b is folded by nsplit[b] workgroups (list entries / COLD_TARGET, at least 1, at most
// G1), the hot bucket by none; first[b] is the index of its first partial copy.
struct mjt_plan {
    unsigned nsplit[NBMAX];
    unsigned first[NBMAX + 1];
};
// In-place inclusive scan of arr[0..n), n <= blockDim.x <= 1024: xor-free shuffle scan inside each
// wave, then the wave totals.
__device__ __forceinline__ void mjt_block_scan(unsigned* arr, int n, unsigned* wsum) {
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    unsigned v = t < n ? arr[t] : 0u;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const unsigned o = (unsigned)__shfl_up((int)v, off, 64);
        if (lane >= off) v += o;
    }
    if (lane == 63) wsum[wave] = v;
    __syncthreads();
    unsigned base = 0;
    for (int w = 0; w < wave; w++) base += wsum[w];
    if (t < n) arr[t] = v + base;
    __syncthreads();
}

__device__ __forceinline__ void mjt_make_plan(mjt_plan& plan, const unsigned* __restrict__ pop, int G1, int NB, int hot,
                                              unsigned* wsum) {
    for (int b = threadIdx.x; b < NB; b += blockDim.x) {
        unsigned k = b == hot ? 0u : (pop[b] + COLD_TARGET - 1) / COLD_TARGET;
        if (b != hot && k < 1) k = 1;
        if (k > (unsigned)G1) k = (unsigned)G1;
        plan.nsplit[b] = k;
        plan.first[b + 1] = k;
    }
    if (threadIdx.x == 0) plan.first[0] = 0;
    __syncthreads();
    if (NB <= (int)blockDim.x) {
        mjt_block_scan(plan.first + 1, NB, wsum);            // first[b + 1] = nsplit[0] + ... + nsplit[b]
    } else {
        if (threadIdx.x == 0)
            for (int b = 0; b < NB; b++) plan.first[b + 1] += plan.first[b];
        __syncthreads();
    }
}

// ---- cold: workgroup (bucket, split) folds the lists of main workgroups split, split+nsplit, ... ----------
extern "C" __global__ __launch_bounds__(NTHREADS) void ENTRY_COLD(Params p) {
    const int* control = (const int*)p.a[5];
    const int G1 = (int)(unsigned long long)p.a[7];
    const int NB = (int)(unsigned long long)p.a[8];
    const unsigned CAP = (unsigned)(unsigned long long)p.a[9];
    const unsigned* __restrict__ counts = (const unsigned*)p.a[10];
    const mjt_pair* __restrict__ lists = (const mjt_pair*)p.a[11];
    TX* __restrict__ pcold = (TX*)p.a[13];
    const mjt_pair* __restrict__ ovf = (const mjt_pair*)p.a[15];
    __shared__ TX win[WBINS];
    __shared__ unsigned prefix[512];                         // running totals of the list lengths (G1 <= 512)
    __shared__ mjt_plan plan;
    __shared__ unsigned wsum[16];
    const int hot = control[0];
    mjt_make_plan(plan, (const unsigned*)control + 64, G1, NB, hot, wsum);
    if (blockIdx.x >= plan.first[NB]) return;
    int bucket = 0;
    {
        int lo = 0, hi = NB - 1;                              // first bucket whose running total exceeds blockIdx.x
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (plan.first[mid + 1] > blockIdx.x) hi = mid; else lo = mid + 1;
        }
        bucket = lo;
    }
    const int split = (int)(blockIdx.x - plan.first[bucket]);
    const int SPLIT = (int)plan.nsplit[bucket];
    const TX ident = mjt_ident();
    for (int t = threadIdx.x; t < WBINS; t += NTHREADS) win[t] = ident;
    const int nsrc = (G1 - split + SPLIT - 1) / SPLIT;       // lists this workgroup folds
    for (int t = threadIdx.x; t < nsrc; t += NTHREADS) prefix[t] = counts[(size_t)(split + t * SPLIT) * NB + bucket];
    __syncthreads();
    mjt_block_scan(prefix, nsrc, wsum);
    const unsigned total = nsrc ? prefix[nsrc - 1] : 0;
    for (unsigned q0 = threadIdx.x; q0 < total; q0 += NTHREADS * 4) {
        mjt_pair e[4];
        bool live[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {                        // four independent reads in flight per lane
            const unsigned q = q0 + u * NTHREADS;
            live[u] = q < total;
            int lo = 0, hi = nsrc - 1;                       // first list whose running total exceeds q
            while (lo < hi) {
                const int mid = (lo + hi) >> 1;
                if (prefix[mid] > q) hi = mid; else lo = mid + 1;
            }
            const unsigned within = q - (lo ? prefix[lo - 1] : 0);
            if (live[u]) e[u] = lists[((size_t)(split + lo * SPLIT) * NB + bucket) * CAP + within];
        }
#pragma unroll
        for (int u = 0; u < 4; u++)
            if (live[u]) { LDS_UPDATE(&win[e[u].bin], e[u].val); }
    }
    // entries that did not fit a list: the first workgroup of the bucket scans the overflow list
    if (split == 0) {
        const unsigned novf = ((const unsigned*)control)[1];
        for (unsigned q = threadIdx.x; q < novf; q += NTHREADS) {
            const mjt_pair e = ovf[q];
            if ((e.bin >> LOGW) == bucket) { LDS_UPDATE(&win[e.bin & (WBINS - 1)], e.val); }
        }
    }
    __syncthreads();
    TX* __restrict__ out = pcold + (size_t)blockIdx.x * WBINS;
    for (int t = threadIdx.x * 4; t < WBINS; t += NTHREADS * 4) {
        mjt_pack<TX, 4> o;
#pragma unroll
        for (int k = 0; k < 4; k++) o.v[k] = win[t + k];
        mjt_store(out + t, o);
    }
}

// ---- final: x[bin] = merge of the partial copies of its bucket --------------------------------
// workgroup = (bucket, segment of 256 bins); 64 lanes x 4 bins across, 4 groups of partials down
extern "C" __global__ __launch_bounds__(256) void ENTRY_FINAL(Params p) {
    TX* __restrict__ xp = (TX*)p.a[0];
    const long long bins = (long long)(unsigned long long)p.a[4];
    const int* control = (const int*)p.a[5];
    const int G1 = (int)(unsigned long long)p.a[7];
    const TX* __restrict__ pmain = (const TX*)p.a[12];
    const TX* __restrict__ pcold = (const TX*)p.a[13];
    const int NB = (int)(unsigned long long)p.a[8];
    constexpr int SEGS = WBINS / 256;
    const int bucket = blockIdx.x / SEGS, seg = blockIdx.x - bucket * SEGS;
    const bool hot = bucket == control[0];
    __shared__ mjt_plan plan;
    __shared__ unsigned wsum[16];
    if (NB > 1) mjt_make_plan(plan, (const unsigned*)control + 64, G1, NB, control[0], wsum);
    const TX* __restrict__ src = hot ? pmain : pcold + (size_t)plan.first[bucket] * WBINS;
    const int P = hot ? G1 : (int)plan.nsplit[bucket];
    const int lane = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const int t = seg * 256 + lane * 4;
    const TX ident = mjt_ident();
    TX acc[4] = {ident, ident, ident, ident};
#pragma unroll 8
    for (int j = grp; j < P; j += 4) {
        mjt_pack<TX, 4> v;
        mjt_load(v, src + (size_t)j * WBINS + t);
#pragma unroll
        for (int k = 0; k < 4; k++) acc[k] = MERGE2(acc[k], v.v[k]);
    }
    __shared__ TX comb[4][256];
#pragma unroll
    for (int k = 0; k < 4; k++) comb[grp][lane * 4 + k] = acc[k];
    __syncthreads();
    if (grp == 0) {
        const long long b0 = (long long)bucket * WBINS + t;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            TX r = comb[0][lane * 4 + k];
            r = MERGE2(r, comb[1][lane * 4 + k]);
            r = MERGE2(r, comb[2][lane * 4 + k]);
            r = MERGE2(r, comb[3][lane * 4 + k]);
            if (b0 + k < bins) xp[b0 + k] = r;
        }
    }
}

