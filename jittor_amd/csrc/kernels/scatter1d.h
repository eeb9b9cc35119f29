// One-axis scatter  x[idx[i]] = OP(x[idx[i]], y[i])  for i in [0, n), idx a
// 1-d integer tensor (the pattern jt.histc and jt.scatter produce,
// reference: python/jittor/misc.py:2233; semantics
// python/jittor/src/ops/reindex_reduce_op.cc:93-131).
//
// Scattered global atomics run at about 2e10 updates/s on this chip whatever
// their scope (contiguous ones, 64 neighbouring bins per wave instruction, at
// 2-4e11/s), and a hot bin serialises them further, so no update of the input
// is a global atomic.  The bin axis is cut into buckets of WBINS bins (one
// bucket fits in LDS); two launches:
//   main    every workgroup streams its share of (idx, y) in rounds of
//           NP*EPT elements.  A sample of its own indices picks the bucket
//           that receives most of its updates (its "hot" bucket); updates of
//           that bucket go to a private LDS copy.  All other updates are put
//           into an LDS staging area (a wave takes its slots of a round with
//           one LDS atomic), and a few waves that load no input append what
//           the previous round staged to the workgroup's per-bucket lists in
//           scratch memory.  Those waves also write the identity into the
//           workgroup's slice of x.  At the end the private copy, the list
//           lengths and the hot bucket's number are written out, and the
//           lengths and the hot bucket are added to the tallies below;
//   tail    every workgroup reads the tallies (list entries and private
//           copies per bucket), lays out the work items from them and walks
//           its items.  A list item (bucket, split) folds the lists of its
//           bucket written by main workgroups split, split + nsplit, ... into
//           an LDS copy; the number of list items per bucket follows the
//           bucket's population.  Entries that did not fit a list (rare: a
//           second hot region) sit in per-workgroup overflow lists that item
//           (bucket, 0) scans.  A merge item merges a segment of MB bins of
//           all private copies of the bucket.  An item that is the only one
//           to reach its bins stores them; otherwise the items of a bucket
//           combine in x through contiguous atomics (a wave instruction
//           updates 64 neighbouring bins) on top of the identity.
// The tallies are two sets of counters in device memory that belong to this
// code object: a call uses set `slot` (its number modulo 2), and the tail pass
// of a call clears the other set, so the counters are zero when main starts
// and nothing has to be cleared in a launch of its own (ENTRY_RESET clears
// both: first call, and after a call that did not finish).
//
// Supplied by the host: TX (4-byte element type), TE (index type), WBINS
// (power of two), LOGW, NBMAX (power of two >= bucket count, <= NTHREADS / 2),
// NTHREADS, NFLUSH (threads that only store), EPT (elements per thread and
// round, multiple of 4), SCAP (entries of each of the two staging areas), MODE (0 add, 1 maximum, 2 minimum), ACC64, COLD_TARGET,
// EXACT_BINS (the bin count is a multiple of WBINS),
// IDENT_BITS (bit pattern of the identity).

// ABL (0 in production): timing-only ablations, results are wrong with any bit set.  1 the tail pass stores
// instead of combining through atomics, 2 list items read no lists, 4 no merge items, 8 the main pass
// stores no list entries, 16 stages none, 32 leaves the private copy alone, 64 neither fills x nor tallies.
#ifndef ABL
#define ABL 0
#endif
#ifndef MDEPTH
#define MDEPTH 8
#endif
#ifndef LDEPTH
#define LDEPTH 16
#endif

struct Params { void* a[20]; };   // 8-byte words; typed as pointers so loads/stores use the global address space
// a[0] x          a[1] y           a[2] idx        a[3] n          a[4] bins
// a[5] fill (1: main writes the identity into x)
// a[6] per (elements per main workgroup)           a[7] G1 (main workgroups)
// a[8] NB (buckets)  a[9] CAP (list capacity)  a[10] counts[G1][NB]  a[11] lists[NB][G1][CAP]
// a[12] partial_main[MSEG][G1][MB]  a[13] slot (tally set of this call)  a[14] hotof[G1]
// a[15] overflow lists[G1][per]   a[16] novf[G1]

// Tallies of the main pass: [set][b] list entries of bucket b, [set][NBMAX + b] main workgroups whose hot bucket
// was b, [set][2 * NBMAX] main workgroups that wrote an overflow list.
// Each set exists TSUB times (a main workgroup adds to copy number blockIdx % TSUB, the tail pass sums the
// copies): hundreds of atomics on one address queue up at the memory.
constexpr int TSUB = 16, TALLY = 2 * NBMAX + 1;
__device__ unsigned mjt_tally[2][TSUB][TALLY];

struct mjt_pair { int bin; TX val; };
// The private copies in memory: partial_main[segment][main workgroup][MB] -- a merge item reads segment s of every
// copy, which is one contiguous piece this way (as rows of whole copies its reads were 1 KB pieces 64 KB apart).
constexpr int MB = WBINS < 256 ? WBINS : 256;                 // bins of a merge item
constexpr int MSEG = WBINS / MB;

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
    TX* __restrict__ xp = (TX*)p.a[0];
    const TX* __restrict__ yp = (const TX*)p.a[1];
    const TE* __restrict__ ip = (const TE*)p.a[2];
    const long long n = (long long)(unsigned long long)p.a[3];
    const long long bins = (long long)(unsigned long long)p.a[4];
    const bool fill = p.a[5] != nullptr;
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
        if (fill && !(ABL & 64)) {                            // the identity into this workgroup's slice of x
            const long long slice = (bins + gridDim.x - 1) / gridDim.x;
            const long long f0 = (long long)blockIdx.x * slice, f1 = f0 + slice < bins ? f0 + slice : bins;
            for (long long t = f0 + (threadIdx.x - NP); t < f1; t += NFLUSH) xp[t] = ident;
        }
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
                        if (b < NBMAX && !(ABL & 8)) {
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
                if (bucket == hot && !(ABL & 32)) mjt_win_update(&win[idx[k] & (WBINS - 1)], val[k]);
                cold[k] = bucket != hot && bucket < (unsigned)NB && !(ABL & 16);
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
    for (int t = threadIdx.x * 4; t < WBINS; t += NTHREADS * 4) {
        mjt_pack<TX, 4> o;
#pragma unroll
        for (int k = 0; k < 4; k++) o.v[k] = mjt_win_read(win[t + k]);
        mjt_store(pmain + ((size_t)(t / MB) * gridDim.x + blockIdx.x) * MB + t % MB, o);
    }
    unsigned* __restrict__ tally = mjt_tally[(unsigned)(unsigned long long)p.a[13] & 1u][blockIdx.x % TSUB];
    for (int t = threadIdx.x; t < NB; t += NTHREADS) {
        const unsigned c = cursor[t] < CAP ? cursor[t] : CAP;
        counts[(size_t)blockIdx.x * NB + t] = c;
        if (c && !(ABL & 64)) atomicAdd(&tally[t], c);
    }
    if (threadIdx.x == 0) {
        hotof[blockIdx.x] = (int)hot;
        novf[blockIdx.x] = ovf_len;
        atomicAdd(&tally[NBMAX + hot], 1u);
        if (ovf_len) atomicAdd(&tally[2 * NBMAX], 1u);
    }
}

// ---- updates of x by the tail pass ------------------------------------------------------------------------
// x holds the identity or what other items have put there; float maxima and minima go through the
// order-preserving integer view of IEEE floats (non-negative floats order like signed integers, negative
// ones inversely like unsigned integers).
#if MODE == 0
__device__ __forceinline__ void mjt_x_update(float* a, float v) { unsafeAtomicAdd(a, v); }
__device__ __forceinline__ void mjt_x_update(int* a, int v) { atomicAdd(a, v); }
__device__ __forceinline__ void mjt_x_update(unsigned* a, unsigned v) { atomicAdd(a, v); }
#elif MODE == 1
__device__ __forceinline__ void mjt_x_update(float* a, float v) {
    const unsigned b = __float_as_uint(v);
    if (b >> 31) atomicMin((unsigned*)a, b); else atomicMax((int*)a, (int)b);
}
__device__ __forceinline__ void mjt_x_update(int* a, int v) { atomicMax(a, v); }
__device__ __forceinline__ void mjt_x_update(unsigned* a, unsigned v) { atomicMax(a, v); }
#else
__device__ __forceinline__ void mjt_x_update(float* a, float v) {
    const unsigned b = __float_as_uint(v);
    if (b >> 31) atomicMax((unsigned*)a, b); else atomicMin((int*)a, (int)b);
}
__device__ __forceinline__ void mjt_x_update(int* a, int v) { atomicMin(a, v); }
__device__ __forceinline__ void mjt_x_update(unsigned* a, unsigned v) { atomicMin(a, v); }
#endif

// ---- reset: both tally sets to zero ----------------------------------------------------------------------
extern "C" __global__ __launch_bounds__(NTHREADS) void ENTRY_RESET(Params) {
    unsigned* t = &mjt_tally[0][0][0];
    for (int i = threadIdx.x; i < 2 * TSUB * TALLY; i += NTHREADS) t[i] = 0;
}

// ---- tail: folds the lists and merges the private copies of main into x -----------------------------------
// Work plan, computed identically by every workgroup from the tallies.  Bucket b has nsplit[b] list items
// (list entries / COLD_TARGET, at least 1 when it has entries, at most G1) followed, when main workgroups had
// it as their hot bucket, by MSEG merge items: one per segment of MB bins, each over all private copies of
// the bucket (one compute unit pulls little more than 100 GB/s: an item should not read more than a few
// hundred KB).  The list items of all buckets come first (they take longest), the merge items after them:
// first[b] is the number of the bucket's first list item, mfirst[b] of its first merge item; first[NBMAX] is
// the number of list items, mfirst[NBMAX] the total.
struct mjt_plan {
    unsigned nsplit[NBMAX];
    unsigned nrows[NBMAX];
    unsigned first[NBMAX + 1];
    unsigned mfirst[NBMAX + 1];
};

extern "C" __global__ __launch_bounds__(NTHREADS) void ENTRY_TAIL(Params p) {
    TX* __restrict__ xp = (TX*)p.a[0];
    const long long bins = (long long)(unsigned long long)p.a[4];
    const long long per = (long long)(unsigned long long)p.a[6];
    const int G1 = (int)(unsigned long long)p.a[7];
    const int NB = (int)(unsigned long long)p.a[8];
    const unsigned CAP = (unsigned)(unsigned long long)p.a[9];
    const unsigned* __restrict__ counts = (const unsigned*)p.a[10];
    const mjt_pair* __restrict__ lists = (const mjt_pair*)p.a[11];
    const TX* __restrict__ pmain = (const TX*)p.a[12];
    const unsigned slot = (unsigned)(unsigned long long)p.a[13] & 1u;
    const int* __restrict__ hotof = (const int*)p.a[14];
    const mjt_pair* __restrict__ ovf = (const mjt_pair*)p.a[15];
    const unsigned* __restrict__ novf = (const unsigned*)p.a[16];
#if ABL & 256
    unsigned long long* dbg = (unsigned long long*)p.a[17] + (size_t)blockIdx.x * 8;
    const unsigned long long dbg_t0 = wall_clock64();
    unsigned long long dbg_t1 = 0, dbg_kind = 0, dbg_t2 = 0;
#endif
    // the private copy of a list item, or the partial results of a merge item on their way to being combined
    constexpr int GROUPS = NTHREADS / (MB / 4);               // a merge item: MB / 4 threads across, GROUPS sets of rows
    constexpr size_t WIN_BYTES = sizeof(TW) * WBINS > sizeof(TA) * GROUPS * MB ? sizeof(TW) * WBINS : sizeof(TA) * GROUPS * MB;
    // At least half of a compute unit's LDS, so that a compute unit takes one workgroup: the dispatcher fills a
    // compute unit before it goes to the next, and two items on one compute unit share its path to memory
    // while other compute units have none (measured with 64 KB copies: 24 us instead of 15).
    constexpr size_t WIN_ALLOC = WIN_BYTES > 84 * 1024 ? WIN_BYTES : 84 * 1024;
    __shared__ __attribute__((aligned(16))) unsigned char win_bytes[WIN_ALLOC];
    TW* win = (TW*)win_bytes;
    __shared__ mjt_plan plan;
    __shared__ unsigned length[512];                          // lengths of the lists of an item (G1 <= 512)
    __shared__ int rows[512];                                 // main workgroups whose private copies an item merges
    __shared__ unsigned novf_s[512];                          // entries of each main workgroup's overflow list
    __shared__ unsigned long long wsum[16];
    __shared__ unsigned any_ovf, nmatch;
    for (int t = threadIdx.x; t < TALLY; t += NTHREADS) {     // the copies of a counter: loads in flight together
        unsigned c[TSUB], sum = 0;
#pragma unroll
        for (int u = 0; u < TSUB; u++) c[u] = mjt_tally[slot][u][t];
#pragma unroll
        for (int u = 0; u < TSUB; u++) sum += c[u];
        if (t < NBMAX) plan.nsplit[t] = sum;
        else if (t < 2 * NBMAX) plan.nrows[t - NBMAX] = sum;
        else any_ovf = sum;
    }
    for (int t = threadIdx.x; t < G1; t += NTHREADS) novf_s[t] = novf[t];
    // fetched together with the tallies: a merge item then has one memory round trip less in front of its rows
    const int my_hot = (int)threadIdx.x < G1 ? hotof[threadIdx.x] : -1;
    if (blockIdx.x == 0)                                      // the next call's set: nobody reads or adds to it now
        for (int t = threadIdx.x; t < TSUB * TALLY; t += NTHREADS) (&mjt_tally[slot ^ 1u][0][0])[t] = 0;
    __syncthreads();
    {
        const int b = threadIdx.x;
        unsigned k = 0, m = 0;
        if (b < NBMAX) {
            k = (plan.nsplit[b] + COLD_TARGET - 1) / COLD_TARGET;
            if (k > (unsigned)G1) k = (unsigned)G1;
            m = plan.nrows[b] ? (unsigned)MSEG : 0u;
        }
        // list items in the low word, merge items in the high word
        const unsigned long long incl = mjt_block_scan_value((unsigned long long)k | ((unsigned long long)m << 32), wsum);
        if (b < NBMAX) {
            plan.nsplit[b] = k;
            plan.first[b] = (unsigned)incl - k;
            plan.mfirst[b] = (unsigned)(incl >> 32) - m;
        }
        if (b == NBMAX - 1) {
            plan.first[NBMAX] = (unsigned)incl;
            plan.mfirst[NBMAX] = (unsigned)(incl >> 32);
        }
        __syncthreads();
        if (b < NBMAX + 1) plan.mfirst[b] += plan.first[NBMAX];
        __syncthreads();
    }
    const TX ident = mjt_ident();
#if ABL & 256
    dbg_t1 = wall_clock64();
#endif
    for (unsigned item = blockIdx.x; item < plan.mfirst[NBMAX]; item += gridDim.x) {
        const bool merge = item >= plan.first[NBMAX];
#if ABL & 256
        dbg_kind = merge ? 2 : 1;
#endif
        const unsigned* __restrict__ firsts = merge ? plan.mfirst : plan.first;
        int bucket;
        {
            int lo = 0, hi = NBMAX - 1;                       // the last bucket whose first item is <= item: it has items,
            while (lo < hi) {                                 // buckets without share `first` with their successor
                const int mid = (lo + hi + 1) >> 1;
                if (firsts[mid] <= item) lo = mid; else hi = mid - 1;
            }
            bucket = lo;
        }
        const int within = (int)(item - firsts[bucket]);
        const int SPLIT = (int)plan.nsplit[bucket];
        // more than one item reaches the bins of this bucket: they combine in x through atomics
        const bool shared = SPLIT + (plan.nrows[bucket] ? 1 : 0) > 1;
        const long long bin0 = (long long)bucket * WBINS;
        if (merge) {
            // merge item: segment sgm of all private copies of this bucket
            if (ABL & 4) continue;
            const int sgm = within;
            const unsigned match = my_hot == bucket ? 1u : 0u;
            const unsigned incl = (unsigned)mjt_block_scan_value(match, wsum);
            if (match) rows[incl - 1] = threadIdx.x;
            if (threadIdx.x == NTHREADS - 1) nmatch = incl;
            __syncthreads();
            const int nrows = (int)nmatch;
            constexpr int ACROSS = MB / 4;
            const int col = threadIdx.x % ACROSS, grp = threadIdx.x / ACROSS;
            TA acc[4] = {(TA)ident, (TA)ident, (TA)ident, (TA)ident};
            constexpr int RPT = MDEPTH;                       // rows of a thread in flight at once
            for (int r0 = 0; r0 < nrows; r0 += GROUPS * RPT) {
                mjt_pack<TX, 4> v[RPT];
#pragma unroll
                for (int j = 0; j < RPT; j++) {
                    const int r = r0 + grp + j * GROUPS;
                    mjt_load(v[j], pmain + ((size_t)sgm * G1 + rows[r < nrows ? r : 0]) * MB + col * 4);
                }
#pragma unroll
                for (int j = 0; j < RPT; j++)
                    if (r0 + grp + j * GROUPS < nrows) {
#pragma unroll
                        for (int k = 0; k < 4; k++) acc[k] = MERGE2(acc[k], (TA)v[j].v[k]);
                    }
            }
            TA* comb = (TA*)win_bytes;                        // GROUPS x MB values
#pragma unroll
            for (int k = 0; k < 4; k++) comb[grp * MB + col * 4 + k] = acc[k];
            __syncthreads();
            if (threadIdx.x < MB) {                           // one bin per thread: neighbouring lanes, neighbouring bins
                TA r = comb[threadIdx.x];
                for (int q = 1; q < GROUPS; q++) r = MERGE2(r, comb[q * MB + threadIdx.x]);
                const long long bin = bin0 + sgm * MB + threadIdx.x;
                if (EXACT_BINS || bin < bins) {
                    if (!shared || (ABL & 1)) xp[bin] = (TX)r;
                    else if ((TX)r != ident) mjt_x_update(xp + bin, (TX)r);
                }
            }
            __syncthreads();
            continue;
        }
        const int split = within;
        for (int t = threadIdx.x; t < WBINS; t += NTHREADS) win[t] = mjt_win_from(ident);
        const int nsrc = (G1 - split + SPLIT - 1) / SPLIT;       // lists this item folds
        for (int t = threadIdx.x; t < nsrc; t += NTHREADS) length[t] = counts[(size_t)(split + t * SPLIT) * NB + bucket];
        __syncthreads();
        // Each wave walks whole lists (no search for the list an entry belongs to), 128 consecutive entries per
        // load (two per lane: a list starts at a multiple of 16 bytes) and all of DEPTH loads in flight before
        // the first is used: the pass is bound by memory round trips, not by bandwidth.  When the item has fewer
        // lists than waves, several waves share a list.
        {
            constexpr int WAVES = NTHREADS / 64, DEPTH = LDEPTH;
            const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
            int wpl = 1;                                          // waves per list
            while (wpl * 2 * nsrc <= WAVES) wpl *= 2;
            const unsigned first_off = (unsigned)(wave % wpl) * 128u, off_step = (unsigned)wpl * 128u;
            const int list_step = WAVES / wpl;
            int li = wave / wpl;
            unsigned off = first_off;
            const mjt_pair* __restrict__ blists = lists + (size_t)bucket * G1 * CAP;   // G1 * CAP < 2^29 entries
            while (li < nsrc && !(ABL & 2)) {
                mjt_pack<mjt_pair, 2> e[DEPTH];
#pragma unroll
                for (int d = 0; d < DEPTH; d++) {
                    e[d].v[0].bin = -1;
                    e[d].v[1].bin = -1;
                    if (li < nsrc) {
                        const unsigned c = length[li];
                        const unsigned q = off + 2 * lane;
                        // (nothing loaded is modified afterwards: that would be a wait for the load)
                        const mjt_pair* src = blists + ((unsigned)(split + li * SPLIT) * CAP + q);
                        if (q + 1 < c) mjt_load(e[d], src);
                        else if (q < c) e[d].v[0] = *src;
                        off += off_step;
                        if (off >= c) { li += list_step; off = first_off; }
                    }
                }
#pragma unroll
                for (int d = 0; d < DEPTH; d++) {
                    if (e[d].v[0].bin >= 0) mjt_win_update(&win[e[d].v[0].bin & (WBINS - 1)], e[d].v[0].val);
                    if (e[d].v[1].bin >= 0) mjt_win_update(&win[e[d].v[1].bin & (WBINS - 1)], e[d].v[1].val);
                }
            }
        }
#if ABL & 256
        __syncthreads();
        dbg_t2 = wall_clock64();
#endif
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
        for (int t = threadIdx.x; t < WBINS; t += NTHREADS) {
            const long long bin = bin0 + t;
            if (EXACT_BINS || bin < bins) {
                const TW w = win[t];
                if (!shared || (ABL & 1)) xp[bin] = mjt_win_read(w);
                else if (w != mjt_win_from(ident)) mjt_x_update(xp + bin, mjt_win_read(w));
            }
        }
        __syncthreads();
    }
#if ABL & 256
    if (threadIdx.x == 0) {
        dbg[0] = dbg_t0; dbg[1] = dbg_t1; dbg[2] = wall_clock64(); dbg[3] = dbg_kind; dbg[4] = dbg_t2;
        unsigned smid;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(smid));
        dbg[5] = smid;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(smid));
        dbg[6] = smid;
    }
#endif
}
