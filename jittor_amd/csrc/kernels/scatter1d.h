// One-axis scatter  x[idx[i]] = OP(x[idx[i]], y[i])  for i in [0, n), idx a
// 1-d integer tensor (the pattern jt.histc and jt.scatter produce,
// reference: python/jittor/misc.py:2233; semantics
// python/jittor/src/ops/reindex_reduce_op.cc:93-131).
//
// Scattered global atomics run at about 2e10 updates/s on this chip whatever
// their scope, and a hot bin serialises them further, so this path uses none.
// The bin axis is cut into buckets of WBINS bins (one bucket fits in LDS):
//   main    every workgroup streams its share of (idx, y) in rounds of
//           NP*EPT elements.  A sample of its own indices picks the bucket
//           that receives most of its updates (its "hot" bucket); updates of
//           that bucket go to a private LDS copy.  All other updates are put
//           into an LDS staging area (a wave takes its slots of a round with
//           one LDS atomic), and a few waves that load no input append what
//           the previous round staged to the workgroup's per-bucket lists in
//           scratch memory.  At the end the private copy, the list lengths and
//           the hot bucket's number are written out;
//   plan    one workgroup sums the list lengths per bucket and lays out the
//           work of the cold pass;
//   cold    a fixed number of workgroups walks the work items.  A list item
//           (bucket, split) folds the lists of its bucket written by main
//           workgroups split, split + nsplit, ... into a private LDS copy and
//           writes it out; the number of list items per bucket follows the
//           bucket's population.  Entries that did not fit a list (rare: a
//           second hot region) sit in per-workgroup overflow lists that item
//           (bucket, 0) scans.  A merge item merges a segment of the private
//           copies of 32 main workgroups that had the same hot bucket;
//   final   x[bin] = merge of the partial copies of its bucket (plain stores:
//           x needs no prior fill).
// Workgroups of one launch share nothing, so no buffer has to be cleared
// beforehand and no global atomic is issued.
//
// Supplied by the host: TX (4-byte element type), TE (index type), WBINS
// (power of two), LOGW, NBMAX (power of two >= bucket count, <= NTHREADS),
// NTHREADS, NFLUSH (threads that only store), EPT (elements per thread and
// round, multiple of 4), SCAP (entries of each of the two staging areas), MODE (0 add, 1 maximum, 2 minimum), ACC64, COLD_TARGET,
// EXACT_BINS (the bin count is a multiple of WBINS),
// IDENT_BITS (bit pattern of the identity).

struct Params { void* a[20]; };   // 8-byte words; typed as pointers so loads/stores use the global address space
// a[0] x          a[1] y           a[2] idx        a[3] n          a[4] bins
// a[5] plan (written by the plan kernel)
// a[6] per (elements per main workgroup)           a[7] G1 (main workgroups)
// a[8] NB (buckets)  a[9] CAP (list capacity)  a[10] counts[G1][NB]  a[11] lists[NB][G1][CAP]
// a[12] partial_main[G1][WBINS]  a[13] partial_cold[items][WBINS]  a[14] hotof[G1]
// a[15] overflow lists[G1][per]   a[16] novf[G1]

struct mjt_pair { int bin; TX val; };

// TA: type partial results are merged in.  TW: type of the private copies in LDS.
// add: a float LDS add costs 3 cycles per lane on this chip, a double one 0.25 (0.6 with the same-address
// conflicts of a Zipf head), so float sums are kept in double: faster, and each partial sum is rounded
// once, when it is written out.
// maximum / minimum: the copies hold order-preserving integer keys, so one integer LDS atomic serves every
// sign; NaN updates are dropped (std::max(cur, v) keeps cur when v is NaN).
#if ACC64
typedef double TA;
#else
typedef TX TA;
#endif
#if MODE == 0
typedef TA TW;
#define MERGE2(a, b) ((a) + (b))
__device__ __forceinline__ TW mjt_win_from(TX v) { return (TW)v; }
__device__ __forceinline__ TX mjt_win_read(TW w) { return (TX)w; }
__device__ __forceinline__ void mjt_win_update(TW* a, TX v) { atomicAdd(a, (TW)v); }
#else
typedef int TW;
#if MODE == 1
#define MERGE2(a, b) (((a) < (b)) ? (b) : (a))
#else
#define MERGE2(a, b) (((b) < (a)) ? (b) : (a))
#endif
__device__ __forceinline__ int mjt_win_from(float v) {
    const int b = __float_as_int(v);
    return b ^ ((b >> 31) & 0x7fffffff);
}
__device__ __forceinline__ int mjt_win_from(int v) { return v; }
__device__ __forceinline__ int mjt_win_from(unsigned v) { return (int)(v ^ 0x80000000u); }
__device__ __forceinline__ void mjt_win_to(int k, float& v) { v = __int_as_float(k ^ ((k >> 31) & 0x7fffffff)); }
__device__ __forceinline__ void mjt_win_to(int k, int& v) { v = k; }
__device__ __forceinline__ void mjt_win_to(int k, unsigned& v) { v = (unsigned)k ^ 0x80000000u; }
__device__ __forceinline__ TX mjt_win_read(TW w) { TX v; mjt_win_to(w, v); return v; }
__device__ __forceinline__ bool mjt_is_nan(float v) { return v != v; }
__device__ __forceinline__ bool mjt_is_nan(int) { return false; }
__device__ __forceinline__ bool mjt_is_nan(unsigned) { return false; }
__device__ __forceinline__ void mjt_win_update(TW* a, TX v) {
    if (mjt_is_nan(v)) return;
#if MODE == 1
    atomicMax(a, mjt_win_from(v));
#else
    atomicMin(a, mjt_win_from(v));
#endif
}
#endif

__device__ __forceinline__ TX mjt_ident() {
    TX t;
    unsigned ib = IDENT_BITS;
    __builtin_memcpy(&t, &ib, 4);
    return t;
}

// Inclusive scan of one 64-bit value per thread over the workgroup (NTHREADS <= 1024): shuffle scan
// inside each wave, then the wave totals through wsum (16 words of LDS that nobody else touches between
// two barriers around this call).  Contains one barrier.
__device__ __forceinline__ unsigned long long mjt_block_scan_value(unsigned long long v, unsigned long long* wsum) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const unsigned long long o = __shfl_up(v, off, 64);
        if (lane >= off) v += o;
    }
    if (lane == 63) wsum[wave] = v;
    __syncthreads();
    unsigned long long base = 0;
    for (int w = 0; w < wave; w++) base += wsum[w];
    return v + base;
}

// ---- main ---------------------------------------------------------------------------
template <bool V> struct mjt_flag { static constexpr bool value = V; };
constexpr int NP = NTHREADS - NFLUSH;                        // threads that load input; the others append to the lists

extern "C" __global__ __launch_bounds__(NTHREADS) void ENTRY_MAIN(Params p) {
    const TX* __restrict__ yp = (const TX*)p.a[1];
    const TE* __restrict__ ip = (const TE*)p.a[2];
    const long long n = (long long)(unsigned long long)p.a[3];
    const long long bins = (long long)(unsigned long long)p.a[4];
    const long long per = (long long)(unsigned long long)p.a[6];
    const int NB = (int)(unsigned long long)p.a[8];
    const unsigned CAP = (unsigned)(unsigned long long)p.a[9];
    unsigned* __restrict__ counts = (unsigned*)p.a[10];
    mjt_pair* __restrict__ lists = (mjt_pair*)p.a[11];
    TX* __restrict__ pmain = (TX*)p.a[12];
    int* __restrict__ hotof = (int*)p.a[14];
    mjt_pair* __restrict__ ovf = (mjt_pair*)p.a[15] + (size_t)blockIdx.x * per;
    unsigned* __restrict__ novf = (unsigned*)p.a[16];
    __shared__ TW win[WBINS];
    __shared__ mjt_pair staging[2][SCAP];  // updates of a round on their way to the lists, by round parity
    __shared__ unsigned cursor[NBMAX + 1]; // list lengths (votes during the sample); the last one is a dummy
    __shared__ unsigned best, staged[3], ovf_len;        // staged: entries of a round, by round number mod 3
    const TX ident = mjt_ident();
    const long long begin = (long long)blockIdx.x * per;
    const long long end = begin + per < n ? begin + per : n;
    const int lane = threadIdx.x & 63;

    for (int t = threadIdx.x; t < NBMAX; t += NTHREADS) cursor[t] = 0;
    for (int t = threadIdx.x; t < WBINS; t += NTHREADS) win[t] = mjt_win_from(ident);
    if (threadIdx.x == 0) { best = 0; staged[0] = 0; staged[1] = 0; staged[2] = 0; ovf_len = 0; }
    __syncthreads();
    unsigned hot = 0;                                         // the hot bucket, voted below (used by the producers only)

    // lists of one bucket are neighbours in memory: the cold item that folds them then touches few pages
    mjt_pair* __restrict__ mylists = lists + (size_t)blockIdx.x * CAP;
    const size_t bucket_stride = (size_t)gridDim.x * CAP;
    // next entry of its bucket's list, or of the overflow list once that is full
    auto append = [&](mjt_pair e) {
        const int b = e.bin >> LOGW;
        const unsigned pos = atomicAdd(&cursor[b], 1u);
        if (pos < CAP) mylists[(size_t)b * bucket_stride + pos] = e;
        else ovf[atomicAdd(&ovf_len, 1u)] = e;
    };
    // Rounds of NP*EPT elements, one barrier each.  Producers (threads < NP) load input, apply the updates of
    // the hot bucket to the private copy and put every other update into the staging area of the round's
    // parity; flushers (the last NFLUSH threads) append what the previous round staged to the lists and load
    // nothing.  The split matters: memory operations of a wave complete in order, so in a wave that both
    // loads and stores every wait for loaded data is also a wait for the acknowledgement of earlier stores.
    const long long end4 = begin + ((end - begin) & ~3ll);
    constexpr long long STEP = (long long)NP * EPT;
    const int rounds = 2 * (int)((end4 - begin + 2 * STEP - 1) / (2 * STEP)) + (end4 < end ? 1 : 0);
    if (threadIdx.x >= NP) {
        __syncthreads();                                      // the three barriers of the producers' vote
        __syncthreads();
        __syncthreads();
        int prev3 = 2, next3 = 1;                             // (r - 1) mod 3, (r + 1) mod 3
        for (int r = 0; r <= rounds; r++) {
            if (r > 0) {                                      // drain what round r-1 staged
                const unsigned total = staged[prev3];
                const unsigned m = total < SCAP ? total : SCAP;
                // FDEPTH entries per thread at a time: their LDS reads, their list cursors and their stores each
                // go out back to back (one entry at a time would cost two LDS round trips per entry in a row)
                constexpr int FDEPTH = 4;
                for (unsigned t0 = threadIdx.x - NP; t0 < m; t0 += NFLUSH * FDEPTH) {
                    mjt_pair e[FDEPTH];
                    unsigned pos[FDEPTH];
#pragma unroll
                    for (int u = 0; u < FDEPTH; u++) {
                        const unsigned t = t0 + u * NFLUSH;
                        e[u] = staging[(r - 1) & 1][t < m ? t : 0];
                        if (t >= m) e[u].bin = NBMAX << LOGW;    // a cursor of its own that nobody reads
                    }
#pragma unroll
                    for (int u = 0; u < FDEPTH; u++) pos[u] = atomicAdd(&cursor[e[u].bin >> LOGW], 1u);
#pragma unroll
                    for (int u = 0; u < FDEPTH; u++) {
                        const int b = e[u].bin >> LOGW;
                        if (b < NBMAX) {
                            if (pos[u] < CAP) mylists[(size_t)b * bucket_stride + pos[u]] = e[u];
                            else ovf[atomicAdd(&ovf_len, 1u)] = e[u];
                        }
                    }
                }
            }
            if (threadIdx.x == NP) staged[next3] = 0;         // drained one round ago, used from the next round on
            prev3 = prev3 == 2 ? 0 : prev3 + 1;
            next3 = next3 == 2 ? 0 : next3 + 1;
            __syncthreads();                                  // (r == rounds: matches the producers' closing barrier)
        }
    } else {
        constexpr unsigned SKIP = 0xffffffffu;                // index of an element that takes no part: its bucket is none
        // one round of a producer over EPT elements; cnt = staged[round number mod 3]
        auto round = [&](int r, unsigned* cnt, const unsigned (&idx)[EPT], const TX (&val)[EPT]) {
            // hot bucket: private copy.  Every other element takes a staging slot: the wave counts them with
            // ballots and takes all its slots of the round with a single LDS atomic.
            bool cold[EPT];
            unsigned long long mask[EPT];
            unsigned before[EPT], total = 0;
#pragma unroll
            for (int k = 0; k < EPT; k++) {
                const unsigned bucket = idx[k] >> LOGW;
                if (bucket == hot) mjt_win_update(&win[idx[k] & (WBINS - 1)], val[k]);
                cold[k] = bucket != hot && bucket < (unsigned)NB;
                mask[k] = __builtin_amdgcn_ballot_w64(cold[k]);
                before[k] = total;
                total += (unsigned)__popcll(mask[k]);
            }
            unsigned base = 0;
            if (total) {
                if (lane == 0) base = atomicAdd(cnt, total);
                base = (unsigned)__shfl((int)base, 0, 64);
            }
#pragma unroll
            for (int k = 0; k < EPT; k++) {
                if (cold[k]) {
                    const unsigned slot = base + before[k] +
                        __builtin_amdgcn_mbcnt_hi((unsigned)(mask[k] >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)mask[k], 0u));
                    mjt_pair e;
                    e.bin = (int)idx[k];
                    e.val = val[k];
                    if (slot < SCAP) staging[r & 1][slot] = e;
                    else append(e);                          // more than the staging area holds: straight to memory
                }
            }
            __syncthreads();
        };
        // The loads of a round are issued two rounds ahead and unconditionally (a load under a branch would
        // make every later wait a wait for all loads in flight): past the end they re-read the start of the
        // input and are ignored.
        mjt_pack<TX, 4> vva[EPT / 4], vvb[EPT / 4];
        mjt_pack<TE, 4> ida[EPT / 4], idb[EPT / 4];
        auto fetch = [&](long long r0, mjt_pack<TX, 4> (&vv)[EPT / 4], mjt_pack<TE, 4> (&id)[EPT / 4]) {
#pragma unroll
            for (int v = 0; v < EPT / 4; v++) {
                const long long i = r0 + ((long long)v * NP + threadIdx.x) * 4;
                const long long ic = i < end4 ? i : 0;
                mjt_load_nt(vv[v], yp + ic);
                mjt_load_nt(id[v], ip + ic);
            }
        };
        // FULL: every vector of the round lies inside the share (no per-vector test)
        auto step = [&](auto full, int r, unsigned* cnt, long long r0, mjt_pack<TX, 4> (&vv)[EPT / 4], mjt_pack<TE, 4> (&id)[EPT / 4]) {
            constexpr bool FULL = decltype(full)::value;
            unsigned idx[EPT];
            TX val[EPT];
#pragma unroll
            for (int v = 0; v < EPT / 4; v++) {
                const long long i = r0 + ((long long)v * NP + threadIdx.x) * 4;
                const bool present = FULL || i < end4;
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    // overflow (index outside [0, bins)): skipped.  When the bins fill their buckets exactly and the
                    // index has 32 bits, an index outside the bins is an index outside the buckets: the test
                    // against the bucket count in `round` covers it.
                    bool inside = true;
                    if constexpr (sizeof(TE) != 4) inside = (unsigned long long)id[v].v[k] < (unsigned long long)bins;
                    else if constexpr (!EXACT_BINS) inside = (unsigned)id[v].v[k] < (unsigned)bins;   // bins < 2^31
                    idx[v * 4 + k] = (present && inside) ? (unsigned)id[v].v[k] : SKIP;
                    val[v * 4 + k] = vv[v].v[k];
                }
            }
            fetch(r0 + 2 * STEP, vv, id);
            round(r, cnt, idx, val);
        };
        fetch(begin, vva, ida);
        fetch(begin + STEP, vvb, idb);
        // The hot bucket: a vote among 256 indices of the first round (already on their way: no extra memory
        // round trip before the stream starts).
        if (threadIdx.x < 256 && begin + (long long)threadIdx.x * 4 < end4) {
            bool inside;
            if constexpr (sizeof(TE) == 4) inside = (unsigned)ida[0].v[0] < (unsigned)bins;
            else inside = (unsigned long long)ida[0].v[0] < (unsigned long long)bins;
            if (inside) atomicAdd(&cursor[(unsigned)ida[0].v[0] >> LOGW], 1u);
        }
        __syncthreads();
        for (int t = threadIdx.x; t < NB; t += NP)
            if (cursor[t]) atomicMax(&best, (cursor[t] << 12) | (unsigned)(4095 - t));   // ties: the lowest bucket
        __syncthreads();
        hot = best ? 4095u - (best & 4095u) : 0u;
        for (int t = threadIdx.x; t < NBMAX; t += NP) cursor[t] = 0;
        __syncthreads();
        int r = 0, r3 = 0;                                    // r3 = r mod 3
        long long r0 = begin;
        for (; r0 + 2 * STEP <= end4; r0 += 2 * STEP) {       // pairs of whole rounds
            step(mjt_flag<true>(), r++, &staged[r3], r0, vva, ida);
            r3 = r3 == 2 ? 0 : r3 + 1;
            step(mjt_flag<true>(), r++, &staged[r3], r0 + STEP, vvb, idb);
            r3 = r3 == 2 ? 0 : r3 + 1;
        }
        for (; r0 < end4; r0 += 2 * STEP) {                   // the ragged end
            step(mjt_flag<false>(), r++, &staged[r3], r0, vva, ida);
            r3 = r3 == 2 ? 0 : r3 + 1;
            step(mjt_flag<false>(), r++, &staged[r3], r0 + STEP, vvb, idb);   // possibly past the end: a round of skipped elements
            r3 = r3 == 2 ? 0 : r3 + 1;
        }
        if (end4 < end) {                                     // the last 1..3 elements of the input
            unsigned idx[EPT];
            TX val[EPT];
#pragma unroll
            for (int k = 0; k < EPT; k++) { idx[k] = SKIP; val[k] = ident; }
            const long long i = end4 + threadIdx.x;
            if (i < end) {
                const long long b = (long long)ip[i];
                idx[0] = (unsigned long long)b < (unsigned long long)bins ? (unsigned)b : SKIP;
                val[0] = yp[i];
            }
            round(r, &staged[r3], idx, val);
        }
        __syncthreads();                                      // the flushers have drained the last round
    }
    __syncthreads();
    TX* __restrict__ out = pmain + (size_t)blockIdx.x * WBINS;
    for (int t = threadIdx.x * 4; t < WBINS; t += NTHREADS * 4) {
        mjt_pack<TX, 4> o;
#pragma unroll
        for (int k = 0; k < 4; k++) o.v[k] = mjt_win_read(win[t + k]);
        mjt_store(out + t, o);
    }
    for (int t = threadIdx.x; t < NB; t += NTHREADS) {
        const unsigned c = cursor[t];
        counts[(size_t)blockIdx.x * NB + t] = c < CAP ? c : CAP;
    }
    if (threadIdx.x == 0) {
        hotof[blockIdx.x] = (int)hot;
        novf[blockIdx.x] = ovf_len;
    }
}

// Work plan of the cold pass, computed identically by every cold workgroup.  Bucket b has nsplit[b] list
// items (list entries / COLD_TARGET, at least 1 when it has entries, at most G1), each producing one
// partial copy, followed by nmerge[b] * MSEG merge items: the partial copies of MERGE_ROWS main workgroups
// whose hot bucket it was are merged into one, MSEG items sharing the work by segments of MBINS bins (one
// compute unit pulls little more than 100 GB/s: an item should not read more than about 100 KB).
// first[b] is the number of the bucket's first item, pfirst[b] of its first partial copy; first[NBMAX] and
// pfirst[NBMAX] are the totals.
constexpr int MERGE_ROWS = 32;
constexpr int MBINS = WBINS < 2048 ? WBINS : 2048;
constexpr int MSEG = WBINS / MBINS;
struct mjt_plan {
    unsigned nsplit[NBMAX];
    unsigned nmerge[NBMAX];
    unsigned first[NBMAX + 1];
    unsigned pfirst[NBMAX + 1];
};

__device__ __forceinline__ void mjt_make_plan(mjt_plan& plan, const unsigned* __restrict__ counts,
                                              const int* __restrict__ hotof, int G1, int NB, unsigned long long* wsum) {
    for (int b = threadIdx.x; b < NBMAX; b += NTHREADS) { plan.nsplit[b] = 0; plan.nmerge[b] = 0; }   // populations first
    __syncthreads();
    {
        const int b = threadIdx.x & (NBMAX - 1);
        unsigned sum = 0;
        if (b < NB) {                                         // independent loads, several in flight
            constexpr int RSTEP = NTHREADS / NBMAX;
            for (int r0 = threadIdx.x / NBMAX; r0 < G1; r0 += 16 * RSTEP) {
                unsigned c[16];
#pragma unroll
                for (int u = 0; u < 16; u++) c[u] = r0 + u * RSTEP < G1 ? counts[(size_t)(r0 + u * RSTEP) * NB + b] : 0u;
#pragma unroll
                for (int u = 0; u < 16; u++) sum += c[u];
            }
        }
        if (sum) atomicAdd(&plan.nsplit[b], sum);
        for (int j = threadIdx.x; j < G1; j += NTHREADS) atomicAdd(&plan.nmerge[hotof[j]], 1u);
    }
    __syncthreads();
    const int b = threadIdx.x;
    unsigned k = 0, m = 0;
    if (b < NBMAX) {
        k = (plan.nsplit[b] + COLD_TARGET - 1) / COLD_TARGET;
        if (k > (unsigned)G1) k = (unsigned)G1;
        m = (plan.nmerge[b] + MERGE_ROWS - 1) / MERGE_ROWS;
    }
    // items in the low word, partial copies in the high word
    const unsigned long long mine = (unsigned long long)(k + m * MSEG) | ((unsigned long long)(k + m) << 32);
    const unsigned long long incl = mjt_block_scan_value(mine, wsum);
    if (b < NBMAX) {
        plan.nsplit[b] = k;
        plan.nmerge[b] = m;
        plan.first[b] = (unsigned)incl - (k + m * MSEG);
        plan.pfirst[b] = (unsigned)(incl >> 32) - (k + m);
    }
    if (b == NBMAX - 1) {
        plan.first[NBMAX] = (unsigned)incl;
        plan.pfirst[NBMAX] = (unsigned)(incl >> 32);
    }
    __syncthreads();
}

// ---- plan: one workgroup computes the work plan of the cold pass -------------------------------------------
// layout of the plan in memory, in words: nsplit[NBMAX], nmerge[NBMAX], first[NBMAX + 1], pfirst[NBMAX + 1], any_ovf
extern "C" __global__ __launch_bounds__(NTHREADS) void ENTRY_PLAN(Params p) {
    unsigned* __restrict__ planout = (unsigned*)p.a[5];
    const int G1 = (int)(unsigned long long)p.a[7];
    const int NB = (int)(unsigned long long)p.a[8];
    const unsigned* __restrict__ counts = (const unsigned*)p.a[10];
    const int* __restrict__ hotof = (const int*)p.a[14];
    const unsigned* __restrict__ novf = (const unsigned*)p.a[16];
    __shared__ mjt_plan plan;
    __shared__ unsigned long long wsum[16];
    __shared__ unsigned any_ovf;
    if (threadIdx.x == 0) any_ovf = 0;
    mjt_make_plan(plan, counts, hotof, G1, NB, wsum);
    for (int w = threadIdx.x; w < G1; w += NTHREADS)
        if (novf[w]) any_ovf = 1;
    __syncthreads();
    for (int t = threadIdx.x; t < NBMAX; t += NTHREADS) {
        planout[t] = plan.nsplit[t];
        planout[NBMAX + t] = plan.nmerge[t];
    }
    for (int t = threadIdx.x; t <= NBMAX; t += NTHREADS) {
        planout[2 * NBMAX + t] = plan.first[t];
        planout[3 * NBMAX + 1 + t] = plan.pfirst[t];
    }
    if (threadIdx.x == 0) planout[4 * NBMAX + 2] = any_ovf;
}

// ---- cold: folds the lists into partial copies, and the partial copies of main MERGE_ROWS at a time ----------
extern "C" __global__ __launch_bounds__(NTHREADS) void ENTRY_COLD(Params p) {
    const unsigned* __restrict__ planin = (const unsigned*)p.a[5];
    const long long per = (long long)(unsigned long long)p.a[6];
    const int G1 = (int)(unsigned long long)p.a[7];
    const int NB = (int)(unsigned long long)p.a[8];
    const unsigned CAP = (unsigned)(unsigned long long)p.a[9];
    const unsigned* __restrict__ counts = (const unsigned*)p.a[10];
    const mjt_pair* __restrict__ lists = (const mjt_pair*)p.a[11];
    const TX* __restrict__ pmain = (const TX*)p.a[12];
    TX* __restrict__ pcold = (TX*)p.a[13];
    const int* __restrict__ hotof = (const int*)p.a[14];
    const mjt_pair* __restrict__ ovf = (const mjt_pair*)p.a[15];
    const unsigned* __restrict__ novf = (const unsigned*)p.a[16];
    // the private copy of a list item, or the rows of a merge item on their way to being combined
    constexpr size_t WIN_BYTES = sizeof(TW) * WBINS > sizeof(TA) * NTHREADS * 4 ? sizeof(TW) * WBINS : sizeof(TA) * NTHREADS * 4;
    __shared__ __attribute__((aligned(16))) unsigned char win_bytes[WIN_BYTES];
    TW* win = (TW*)win_bytes;
    __shared__ mjt_plan plan;
    __shared__ unsigned length[512];                          // lengths of the lists of an item (G1 <= 512)
    __shared__ int rows[MERGE_ROWS];
    __shared__ unsigned novf_s[512];                          // entries of each main workgroup's overflow list
    __shared__ unsigned long long wsum[16];
    __shared__ unsigned any_ovf, nmatch;
    for (int t = threadIdx.x; t < G1; t += NTHREADS) novf_s[t] = novf[t];
    for (int t = threadIdx.x; t < NBMAX; t += NTHREADS) {
        plan.nsplit[t] = planin[t];
        plan.nmerge[t] = planin[NBMAX + t];
    }
    for (int t = threadIdx.x; t <= NBMAX; t += NTHREADS) {
        plan.first[t] = planin[2 * NBMAX + t];
        plan.pfirst[t] = planin[3 * NBMAX + 1 + t];
    }
    if (threadIdx.x == 0) any_ovf = planin[4 * NBMAX + 2];
    // fetched together with the plan: a merge item then has one memory round trip less in front of its rows
    const int my_hot = (int)threadIdx.x < G1 ? hotof[threadIdx.x] : -1;
    __syncthreads();
    const TX ident = mjt_ident();
    for (unsigned item = blockIdx.x; item < plan.first[NBMAX]; item += gridDim.x) {
        int bucket;
        {
            int lo = 0, hi = NBMAX - 1;                       // the last bucket whose first item is <= item: it has items,
            while (lo < hi) {                                 // buckets without share `first` with their successor
                const int mid = (lo + hi + 1) >> 1;
                if (plan.first[mid] <= item) lo = mid; else hi = mid - 1;
            }
            bucket = lo;
        }
        const int within = (int)(item - plan.first[bucket]);
        const int SPLIT = (int)plan.nsplit[bucket];
        if (within >= SPLIT) {
            // merge item: segment sgm of the partial copies of main workgroups number g*MERGE_ROWS ... of this bucket
            const int g = (within - SPLIT) / MSEG, sgm = (within - SPLIT) - g * MSEG;
            const unsigned match = my_hot == bucket ? 1u : 0u;
            const unsigned incl = (unsigned)mjt_block_scan_value(match, wsum);
            if (match && (int)(incl - 1) / MERGE_ROWS == g) rows[(incl - 1) % MERGE_ROWS] = threadIdx.x;
            if (threadIdx.x == NTHREADS - 1) nmatch = incl;
            __syncthreads();
            const int nrows = (int)nmatch - g * MERGE_ROWS < MERGE_ROWS ? (int)nmatch - g * MERGE_ROWS : MERGE_ROWS;
            // MBINS / 4 threads across, the rows dealt to the groups of MBINS / 4 threads; combined through LDS
            constexpr int ACROSS = MBINS / 4, GROUPS = NTHREADS / ACROSS;
            const int col = threadIdx.x % ACROSS, grp = threadIdx.x / ACROSS;
            const int t = sgm * MBINS + col * 4;
            TA acc[4] = {(TA)ident, (TA)ident, (TA)ident, (TA)ident};
            // all rows of the thread in flight at once
            constexpr int RPT = (MERGE_ROWS + GROUPS - 1) / GROUPS;
            mjt_pack<TX, 4> v[RPT];
#pragma unroll
            for (int j = 0; j < RPT; j++) {
                const int r = grp + j * GROUPS;
                mjt_load(v[j], pmain + (size_t)rows[r < nrows ? r : 0] * WBINS + t);
            }
#pragma unroll
            for (int j = 0; j < RPT; j++)
                if (grp + j * GROUPS < nrows) {
#pragma unroll
                    for (int k = 0; k < 4; k++) acc[k] = MERGE2(acc[k], (TA)v[j].v[k]);
                }
            TA* comb = (TA*)win_bytes;                        // GROUPS x MBINS = NTHREADS * 4 values
#pragma unroll
            for (int k = 0; k < 4; k++) comb[grp * MBINS + col * 4 + k] = acc[k];
            __syncthreads();
            if (grp == 0) {
                mjt_pack<TX, 4> o;
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    TA r = comb[col * 4 + k];
                    for (int q = 1; q < GROUPS; q++) r = MERGE2(r, comb[q * MBINS + col * 4 + k]);
                    o.v[k] = (TX)r;
                }
                mjt_store(pcold + (size_t)(plan.pfirst[bucket] + SPLIT + g) * WBINS + t, o);
            }
            __syncthreads();
            continue;
        }
        const int split = within;
        TX* __restrict__ out = pcold + (size_t)(plan.pfirst[bucket] + split) * WBINS;
        for (int t = threadIdx.x; t < WBINS; t += NTHREADS) win[t] = mjt_win_from(ident);
        const int nsrc = (G1 - split + SPLIT - 1) / SPLIT;       // lists this item folds
        for (int t = threadIdx.x; t < nsrc; t += NTHREADS) length[t] = counts[(size_t)(split + t * SPLIT) * NB + bucket];
        __syncthreads();
        // Each wave walks whole lists (no search for the list an entry belongs to), 64 consecutive entries per
        // load and DEPTH loads in flight; when the item has fewer lists than waves, several waves share a list.
        {
            constexpr int WAVES = NTHREADS / 64, DEPTH = 8;
            const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
            int wpl = 1;                                          // waves per list
            while (wpl * 2 * nsrc <= WAVES) wpl *= 2;
            const unsigned first_off = (unsigned)(wave % wpl) * 64u, off_step = (unsigned)wpl * 64u;
            const int list_step = WAVES / wpl;
            int li = wave / wpl;
            unsigned off = first_off;
            while (li < nsrc) {
                mjt_pair e[DEPTH];
#pragma unroll
                for (int d = 0; d < DEPTH; d++) {
                    e[d].bin = -1;
                    if (li < nsrc) {
                        const unsigned c = length[li];
                        const unsigned q = off + lane;
                        if (q < c) e[d] = lists[((size_t)bucket * G1 + (split + li * SPLIT)) * CAP + q];
                        off += off_step;
                        if (off >= c) { li += list_step; off = first_off; }
                    }
                }
#pragma unroll
                for (int d = 0; d < DEPTH; d++)
                    if (e[d].bin >= 0) mjt_win_update(&win[e[d].bin & (WBINS - 1)], e[d].val);
            }
        }
        // entries that did not fit a list: the first item of the bucket scans the overflow lists
        if (split == 0 && any_ovf) {
            for (int w = 0; w < G1; w++) {
                const unsigned c = novf_s[w];                 // (from LDS: a load from memory per workgroup would be a chain of round trips)
                const mjt_pair* __restrict__ l = ovf + (size_t)w * per;
                for (unsigned q = threadIdx.x; q < c; q += NTHREADS) {
                    const mjt_pair e = l[q];
                    if ((e.bin >> LOGW) == bucket) mjt_win_update(&win[e.bin & (WBINS - 1)], e.val);
                }
            }
        }
        __syncthreads();
        for (int t = threadIdx.x * 4; t < WBINS; t += NTHREADS * 4) {
            mjt_pack<TX, 4> o;
#pragma unroll
            for (int k = 0; k < 4; k++) o.v[k] = mjt_win_read(win[t + k]);
            mjt_store(out + t, o);
        }
        __syncthreads();
    }
}

// ---- final: x[bin] = merge of the partial copies of its bucket --------------------------------
// workgroup = (bucket, segment of 256 bins); 64 lanes x 4 bins across, 4 groups of partial copies down
extern "C" __global__ __launch_bounds__(256) void ENTRY_FINAL(Params p) {
    TX* __restrict__ xp = (TX*)p.a[0];
    const long long bins = (long long)(unsigned long long)p.a[4];
    const unsigned* __restrict__ planin = (const unsigned*)p.a[5];
    const TX* __restrict__ pcold = (const TX*)p.a[13];
    constexpr int SEGS = WBINS / 256;
    const int bucket = blockIdx.x / SEGS, seg = blockIdx.x - bucket * SEGS;
    const int lane = threadIdx.x & 63, grp = threadIdx.x >> 6;
    const int t = seg * 256 + lane * 4;
    const int P = (int)(planin[bucket] + planin[NBMAX + bucket]);
    const size_t first = planin[3 * NBMAX + 1 + bucket];
    const TA ident = (TA)mjt_ident();
    TA acc[4] = {ident, ident, ident, ident};
#pragma unroll 8
    for (int j = grp; j < P; j += 4) {
        mjt_pack<TX, 4> v;
        mjt_load(v, pcold + (first + j) * WBINS + t);
#pragma unroll
        for (int k = 0; k < 4; k++) acc[k] = MERGE2(acc[k], (TA)v.v[k]);
    }
    __shared__ TA comb[4][256];
#pragma unroll
    for (int k = 0; k < 4; k++) comb[grp][lane * 4 + k] = acc[k];
    __syncthreads();
    if (grp == 0) {
        const long long b0 = (long long)bucket * WBINS + t;
#pragma unroll
        for (int k = 0; k < 4; k++) {
            TA r = comb[0][lane * 4 + k];
            r = MERGE2(r, comb[1][lane * 4 + k]);
            r = MERGE2(r, comb[2][lane * 4 + k]);
            r = MERGE2(r, comb[3][lane * 4 + k]);
            if (b0 + k < bins) xp[b0 + k] = (TX)r;
        }
    }
}
