// top_k along the last axis of strided views for gfx950.
//
// Selection kernel (rows up to 65536 elements, limit up to 1024): one workgroup of 256 or
// 1024 threads per row reads the row exactly once into registers, takes a bound that at
// least `limit` elements reach from samples of its threads' maxima, compacts the elements
// that reach it into LDS and orders those few by sorted runs and rank merging; a row with
// too many survivors (long runs of equal values, a limit that is a large part of the row)
// is selected exactly, by a most-significant-digit radix select over LDS histograms: from
// its registers when the row is short, by a second kernel from spilled candidates or the
// row itself otherwise.  Among equal values the lowest index always comes first.
//
// Around it: one wavefront per row for rows of up to 1024 elements and limits up to 32, one
// thread per row for many very short rows, kernels for rows that lie side by side in memory
// (an outer axis), two levels of selection for rows longer than one workgroup holds.
// Limits above 1024, or that are a large part of a short row, go through the stable
// argsort and keep the first `limit` entries of each row.
#include <cstring>
#include <limits>
#include <type_traits>

#include "common.hip.h"

// This file is compiled three times, once for each width of element, so that the three sets of
// kernels compile side by side: part 0 (this file on its own) holds the 32-bit elements and
// everything that is not a template, the entry points included; topk_wide.hip includes it as
// part 1 for the 64-bit elements, topk_narrow.hip as part 2 for the 16-bit ones.
#ifndef DLFX_TOPK_PART
#define DLFX_TOPK_PART 0
#endif

namespace dlfx {

// from sort.hip
size_t argsort_scratch_bytes_impl(int dtype, int64_t m, int64_t n);
int argsort_contiguous(hipStream_t stream, int dir, int dtype, int rank, const int64_t* dims,
                       const void* x, const int64_t* x_strides, void* y_contig, int32_t* idx_contig,
                       void* scratch, size_t scratch_bytes);

namespace {

constexpr int kRadix = 256;
constexpr int kMaxLimit = 1024;

#ifdef DLFX_TOPK_TIMING
// Debug builds only: shader-clock cycles spent by thread 0 of every workgroup in each phase.
constexpr int kPhaseSlots = 8192;
__device__ unsigned long long g_topk_cycles[kPhaseSlots * 8];
#define DLFX_PHASE(i) do { if (threadIdx.x == 0) { const long long now_ = clock64(); g_topk_cycles[(blockIdx.x % kPhaseSlots) * 8 + (i)] += static_cast<unsigned long long>(now_ - phase_t_); phase_t_ = now_; } } while (0)
#define DLFX_PHASE_BEGIN() long long phase_t_ = clock64()
#else
#define DLFX_PHASE(i) do { } while (0)
#define DLFX_PHASE_BEGIN() do { } while (0)
#endif

enum KeyKind { kKeyInt = 0, kKeyFloat = 1 };

template <typename K>
struct KeyBits;
template <> struct KeyBits<uint32_t> { static constexpr uint32_t kSign = 0x80000000u; };
template <> struct KeyBits<uint64_t> { static constexpr uint64_t kSign = 0x8000000000000000ull; };

// Larger image <=> better candidate.
template <typename K>
__device__ __forceinline__ K to_ord(K bits, int kind, int largest) {
    constexpr K S = KeyBits<K>::kSign;
    if (kind == kKeyFloat && (bits << 1) == 0) bits = 0;          // -0.0 and +0.0 are one value
    K k = (kind == kKeyFloat) ? ((bits & S) ? ~bits : (bits | S)) : (bits ^ S);
    return largest ? k : ~k;
}
template <typename K>
__device__ __forceinline__ K from_ord(K k, int kind, int largest) {
    constexpr K S = KeyBits<K>::kSign;
    if (!largest) k = ~k;
    return (kind == kKeyFloat) ? ((k & S) ? (k & ~S) : ~k) : (k ^ S);
}

// Elements are stored as S and handled as K-wide bit patterns: S is K itself for four- and
// eight-byte types; IEEE half and int16 are stored as 16 bits and widened (exactly, order
// preserved) to the bits of a float or an int32 at the load, narrowed again at the store.
template <typename K, typename S>
__device__ __forceinline__ K widen_bits(S s, int kind) {
    if constexpr (sizeof(S) == sizeof(K)) {
        return s;
    } else {
        if (kind == kKeyFloat) return bit_cast<uint32_t>(static_cast<float>(bit_cast<half_t>(s)));
        return static_cast<uint32_t>(static_cast<int32_t>(static_cast<int16_t>(s)));
    }
}
template <typename S, typename K>
__device__ __forceinline__ S narrow_bits(K bits, int kind) {
    if constexpr (sizeof(S) == sizeof(K)) {
        return bits;
    } else {
        if (kind == kKeyFloat) return bit_cast<uint16_t>(static_cast<half_t>(bit_cast<float>(bits)));
        return static_cast<uint16_t>(bits);
    }
}

template <typename K, typename S = K>
struct TopkIo {
    const S* x;
    DimMap xmap;
    int64_t sx;
    S* y;
    DimMap ymap;
    int64_t sy;
    void* idx;
    DimMap imap;
    int64_t si;
    int idx64, kind, largest;
    // segmented rows (first stage of long rows): row r of the launch is segment r % segs of a
    // longer row; the last segment of each has last_n elements instead of n.  0 or 1: plain rows.
    int64_t segs, last_n;
    // rows side by side in memory: workgroup b takes block (b % 8) * xcd_blocks + b / 8, so that
    // neighbouring rows, which share cache lines, run on one XCD (0: workgroup b takes block b)
    int64_t xcd_blocks;
};

constexpr int kCandCap = 4096;     // candidates kept after the pre-filter (4-byte keys; half for 8-byte keys)
template <typename K> constexpr int cand_cap() { return sizeof(K) == 4 ? kCandCap : kCandCap / 2; }
constexpr int kAmbMax = 64;        // members of the deciding digit that are ranked directly
constexpr int kSelectThreads = 256; // threads that run the exact selection among candidates
constexpr uint32_t kRowDone = 0u, kRowWhole = 0xffffffffu;   // per-row hand-over state (else: candidate count)

template <typename K, int CAND = cand_cap<K>()>
struct TopkShared {
    uint32_t hist[kRadix];
    uint32_t wave_tot[kRadix / kWave];
    uint32_t scan_tot[32];
    uint32_t sel_digit, sel_k, sel_ties, count;
    K out_ord[kMaxLimit];
    uint32_t out_idx[kMaxLimit];
    uint32_t rank[kMaxLimit];
    K amb_ord[kAmbMax];
    uint32_t amb_idx[kAmbMax];
    K and_bits[16], or_bits[16];
    uint32_t amb_count;
    K cand_ord[CAND];                       // (rows no longer than the capacity keep at most what is merged by rank)
    uint32_t cand_idx[CAND];
    unsigned long long pack[sizeof(K) == 4 ? 512 : 1];      // sorted runs of (image, ~index) words, 4-byte keys
};

// Synchronises the TEAM threads that run a selection.  A single wave needs no hardware
// barrier: its LDS accesses execute in program order, the fence only stops the compiler
// from moving them across this point.
template <int TEAM>
__device__ __forceinline__ void team_sync() {
    if constexpr (TEAM <= kWave) {
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
        __builtin_amdgcn_wave_barrier();
    } else {
        __syncthreads();
    }
}

// Appends the items flagged `take` of the calling wave to an LDS list whose length is
// *counter: one atomic per wave, slots in lane order.  Returns the slot (valid when take).
__device__ __forceinline__ uint32_t wave_append(uint32_t* counter, bool take) {
    const unsigned long long m = __ballot(take);
    if (m == 0ull) return 0u;
    const int lane = lane_id();
    const int first = __ffsll(static_cast<long long>(m)) - 1;
    uint32_t base = 0;
    if (lane == first) base = atomicAdd(counter, static_cast<uint32_t>(__popcll(m)));
    base = __shfl(base, first, kWave);
    return base + static_cast<uint32_t>(__popcll(m & ((1ull << lane) - 1ull)));
}

// One radix-select step over the values val(i) of the items for which part(i)
// holds: picks the digit (at `shift`) that contains the kk-th largest
// participating value.  Results: sm.sel_digit, sm.sel_k (rank inside that
// digit), sm.sel_ties (its population).  sm.hist must be all zero on entry and is
// all zero again on return.
template <int BLOCK, int ITEMS, bool ROLLED, typename K, int CAND, typename Val, typename Part>
__device__ __forceinline__ void select_digit(TopkShared<K, CAND>& sm, int nitems, int shift, uint32_t kk, Val val, Part part) {
    const int tid = threadIdx.x;
    const int lane = lane_id();
    (void)lane;
    auto count_item = [&](int i) {
        // callers skip bytes in which all items agree, so a digit shared by everyone (the one
        // case that would serialise these adds) does not reach this point
        if (part(i)) atomicAdd(&sm.hist[static_cast<uint32_t>(val(i) >> shift) & 0xffu], 1u);
    };
    if constexpr (ROLLED) {
#pragma unroll 1
        for (int i = 0; i < nitems; ++i) count_item(i);
    } else {
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) count_item(i);
    }
    team_sync<BLOCK>();
    if (tid < kWave) {
        // lane l owns digits 255-4l .. 252-4l (descending), so a scan over lanes is a suffix sum over digits
        uint32_t h[4], run = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int d = kRadix - 1 - (4 * lane + j);
            h[j] = sm.hist[d];
            sm.hist[d] = 0;
            run += h[j];
        }
        const uint32_t incl = wave_scan_inclusive(run, 0u, [](uint32_t a, uint32_t b) { return a + b; });
        uint32_t above = incl - run;                  // participants with a digit above this lane's four
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (above < kk && above + h[j] >= kk) {
                sm.sel_digit = kRadix - 1 - (4 * lane + j);
                sm.sel_k = kk - above;
                sm.sel_ties = h[j];
            }
            above += h[j];
        }
    }
    team_sync<BLOCK>();
}

// The kk-th largest of the values val(i) over the items with part(i): most significant
// byte first.  Returns the value; *rank_in_ties / *ties describe how many of the elements
// equal to it still have to be taken and how many there are.
template <int BLOCK, int ITEMS, bool ROLLED, typename V, typename K, int CAND, typename Val, typename Valid>
__device__ __forceinline__ V kth_largest(TopkShared<K, CAND>& sm, int nitems, uint32_t kk, Val val, Valid valid,
                                         uint32_t* rank_in_ties, uint32_t* ties,
                                         int first_pass = static_cast<int>(sizeof(V)) - 1, V known_high = 0) {
    // bytes above first_pass are the same (known_high) in every participating value
    V prefix = known_high;
#pragma unroll 1
    for (int pass = first_pass; pass >= 0; --pass) {
        const int shift = 8 * pass;
        const V hi_mask = (pass == static_cast<int>(sizeof(V)) - 1) ? V(0) : static_cast<V>(~V(0) << (shift + 8));
        select_digit<BLOCK, ITEMS, ROLLED>(sm, nitems, shift, kk, val, [&](int i) {
            return valid(i) && ((val(i) ^ prefix) & hi_mask) == 0;
        });
        prefix |= static_cast<V>(sm.sel_digit) << shift;
        kk = sm.sel_k;
        *ties = sm.sel_ties;
    }
    *rank_in_ties = kk;
    return prefix;
}

template <typename K, typename S>
__device__ __forceinline__ void emit_one(const TopkIo<K, S>& io, S* yr, int64_t ir, const S* xr, int j, K ord, uint32_t ix) {
    K bits = from_ord<K>(ord, io.kind, io.largest);
    S out = narrow_bits<S, K>(bits, io.kind);
    if (io.kind == kKeyFloat && (bits << 1) == 0) out = xr[static_cast<int64_t>(ix) * io.sx];   // keep the zero's sign
    yr[j * io.sy] = out;
    if (io.idx64) static_cast<int64_t*>(io.idx)[ir + j * io.si] = static_cast<int64_t>(ix);
    else static_cast<int32_t*>(io.idx)[ir + j * io.si] = static_cast<int32_t>(ix);
}

// "entry j beats (o, x)": larger image, then lower index.
template <typename K>
__device__ __forceinline__ uint32_t beats(K oj, uint32_t xj, K o, uint32_t x) {
    if constexpr (sizeof(K) == 4) {
        // one 64-bit comparison of (image, ~index)
        const uint64_t a = (static_cast<uint64_t>(oj) << 32) | static_cast<uint32_t>(~xj);
        const uint64_t b = (static_cast<uint64_t>(o) << 32) | static_cast<uint32_t>(~x);
        return a > b ? 1u : 0u;
    } else {
        return (oj > o || (oj == o && xj < x)) ? 1u : 0u;
    }
}

// For each of `count` (image, index) entries held in LDS: sm.rank[e] = number of entries that
// beat it (entries are distinct).  Quadratic: small counts.  Ends with a barrier.
template <int BLOCK, typename K, int CAND>
__device__ __forceinline__ void compute_ranks(TopkShared<K, CAND>& sm, const K* e_ord, const uint32_t* e_idx, int count) {
    const int tid = threadIdx.x;
    for (int i = tid; i < count; i += BLOCK) sm.rank[i] = 0;
    team_sync<BLOCK>();
    int cp = 1;
    while (cp < count) cp <<= 1;
    // BLOCK / cp threads share one entry (one thread when there are more entries than threads),
    // each scanning a slice of the others; eight independent LDS reads in flight
    const int parts = cp <= BLOCK ? BLOCK / cp : 1;
    const int per = (count + parts - 1) / parts;
    for (int e0 = 0; e0 < count; e0 += BLOCK) {
        const int e = e0 + (parts > 1 ? (tid & (cp - 1)) : tid);
        const int part = parts > 1 ? tid / cp : 0;
        if (e < count) {
            const K o = e_ord[e];
            const uint32_t x = e_idx[e];
            const int lo = part * per;
            const int hi = lo + per < count ? lo + per : count;
            uint32_t r = 0;
            int j = lo;
            for (; j + 8 <= hi; j += 8) {
                K oj[8];
                uint32_t xj[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) { oj[u] = e_ord[j + u]; xj[u] = e_idx[j + u]; }
#pragma unroll
                for (int u = 0; u < 8; ++u) r += beats<K>(oj[u], xj[u], o, x);
            }
            for (; j < hi; ++j) r += beats<K>(e_ord[j], e_idx[j], o, x);
            if (parts > 1) { if (r) atomicAdd(&sm.rank[e], r); }
            else sm.rank[e] = r;
        }
        if (parts > 1) break;
    }
    team_sync<BLOCK>();
}

// Sorts one (image, index) entry per lane across the wavefront, best entry in lane 0.
template <typename K>
__device__ __forceinline__ void wave_sort_entries(K& o, uint32_t& x) {
    wave_bitonic<kWave>([&](auto jc, bool keep_better) {
        constexpr int J = decltype(jc)::value;
        const K oo = lane_xor_const<J>(o);
        const uint32_t xo = lane_xor_const<J>(x);
        if (keep_better == (beats<K>(oo, xo, o, x) != 0u)) {
            o = oo;
            x = xo;
        }
    });
}

constexpr int kMergeMax = 512;       // entries up to which sorted runs are merged by rank
static_assert(sizeof(TopkShared<uint32_t>::pack) == kMergeMax * 8, "room for kMergeMax packed entries");
constexpr int kCountMax = 20;        // entries up to which ranks are counted directly

// Orders `count` distinct (image, index) entries held in LDS, best first, and writes those
// ranked below `limit` to the outputs.  The arrays must have room for count rounded up to a
// multiple of 64 and are overwritten.  Each wave sorts runs of 64 entries in registers; the
// rank of an entry is its position in its run plus, for every other run, the number of that
// run's entries that beat it, found by bisection.  All threads of the team must call.
struct KeepImage {
    template <typename K>
    __device__ __forceinline__ K operator()(K v) const { return v; }
};

// `image_of` maps what e_ord holds to the image (the identity unless the caller stored
// something cheaper to produce).
// 4-byte images travel through the ranking as one 64-bit word (image, ~index) in `e_pack`
// (room for kMergeMax words): an entry beats another exactly when its word is larger, one
// LDS read and one comparison per probe.  8-byte images keep the two arrays.
template <int BLOCK, typename K, typename S, typename ImageOf = KeepImage>
__device__ __forceinline__ void merge_rank_emit(K* e_ord, uint32_t* e_idx, unsigned long long* e_pack, int count, int limit,
                                                const TopkIo<K, S>& io, int64_t row, const S* xr,
                                                ImageOf image_of = ImageOf()) {
    constexpr bool PACKED = sizeof(K) == 4;
    constexpr int WAVES = BLOCK / kWave;
    const int tid = threadIdx.x;
    const int lane = lane_id();
    const int w = tid / kWave;
    const int runs = (count + kWave - 1) / kWave;
    S* yr = io.y + io.ymap.at(row);
    const int64_t ir = io.imap.at(row);
    if (count <= kCountMax) {
        // a handful of entries: the first wave counts, for each, the entries that beat it
        if (w == 0) {
            const K o = lane < count ? image_of(e_ord[lane]) : K(0);
            const uint32_t x = lane < count ? e_idx[lane] : 0xffffffffu;
            uint32_t rank = 0;
            for (int j = 0; j < count; ++j) rank += beats<K>(lane_read(o, j), lane_read(x, j), o, x);
            if (lane < count && rank < static_cast<uint32_t>(limit)) emit_one<K>(io, yr, ir, xr, static_cast<int>(rank), o, x);
        }
        return;
    }
    for (int r = w; r < runs; r += WAVES) {
        const int e = r * kWave + lane;
        K o = e < count ? image_of(e_ord[e]) : K(0);
        uint32_t x = e < count ? e_idx[e] : 0xffffffffu;      // padding: beaten by every entry
        wave_sort_entries<K>(o, x);
        if (runs == 1) {
            if (lane < limit && lane < count) emit_one<K>(io, yr, ir, xr, lane, o, x);
        } else if constexpr (PACKED) {
            e_pack[e] = (static_cast<unsigned long long>(o) << 32) | static_cast<uint32_t>(~x);
        } else {
            e_ord[e] = o;
            e_idx[e] = x;
        }
    }
    if (runs == 1) return;
    team_sync<BLOCK>();
    for (int e = tid; e < count; e += BLOCK) {
        K o;
        uint32_t x;
        unsigned long long mine_word = 0ull;
        if constexpr (PACKED) {
            mine_word = e_pack[e];
            o = static_cast<K>(mine_word >> 32);
            x = ~static_cast<uint32_t>(mine_word);
        } else {
            o = e_ord[e];
            x = e_idx[e];
        }
        const int mine = e / kWave;
        uint32_t rank = static_cast<uint32_t>(e % kWave);
        // U bisections at a time keep U independent LDS reads in flight; indices are only
        // read in the steps where some image ties with this entry's
        auto bisect = [&](auto uc, int first_other) {
            constexpr int U = decltype(uc)::value;
            int base[U];
            uint32_t c[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int other = first_other + u;
                base[u] = (other < mine ? other : other + 1) * kWave;
                c[u] = 0u;
            }
            auto probe = [&](int step) {      // step 0: the last probe, which decides 63 against 64
                if constexpr (PACKED) {
                    unsigned long long pj[U];
#pragma unroll
                    for (int u = 0; u < U; ++u) pj[u] = e_pack[base[u] + static_cast<int>(c[u]) + (step ? step - 1 : 0)];
#pragma unroll
                    for (int u = 0; u < U; ++u) c[u] += pj[u] > mine_word ? static_cast<uint32_t>(step ? step : 1) : 0u;
                    return;
                }
                K oj[U];
                uint32_t xj[U];
                bool tie = false;
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    oj[u] = e_ord[base[u] + static_cast<int>(c[u]) + (step ? step - 1 : 0)];
                    xj[u] = 0xffffffffu;
                    tie = tie || oj[u] == o;
                }
                if (tie) {
#pragma unroll
                    for (int u = 0; u < U; ++u) xj[u] = e_idx[base[u] + static_cast<int>(c[u]) + (step ? step - 1 : 0)];
                }
#pragma unroll
                for (int u = 0; u < U; ++u)
                    c[u] += (oj[u] > o || (oj[u] == o && xj[u] < x)) ? static_cast<uint32_t>(step ? step : 1) : 0u;
            };
#pragma unroll
            for (int step = 32; step >= 1; step >>= 1) probe(step);
            probe(0);
#pragma unroll
            for (int u = 0; u < U; ++u) rank += c[u];
        };
        // all the other runs (at most seven: kMergeMax / 64 - 1) are bisected side by side
        static_assert(kMergeMax / kWave - 1 == 7, "one case per possible number of other runs");
        switch (runs - 1) {
        case 7: bisect(std::integral_constant<int, 7>(), 0); break;
        case 6: bisect(std::integral_constant<int, 6>(), 0); break;
        case 5: bisect(std::integral_constant<int, 5>(), 0); break;
        case 4: bisect(std::integral_constant<int, 4>(), 0); break;
        case 3: bisect(std::integral_constant<int, 3>(), 0); break;
        case 2: bisect(std::integral_constant<int, 2>(), 0); break;
        case 1: bisect(std::integral_constant<int, 1>(), 0); break;
        default: break;
        }
        if (rank < static_cast<uint32_t>(limit)) emit_one<K>(io, yr, ir, xr, static_cast<int>(rank), o, x);
    }
}


// Exact selection of the `limit` best of the items (ord(i), idx(i)), best = larger image,
// then lower index; writes them in that order.  Padding items carry image 0 and an index
// that is not below the row length: they lose every tie, and limit <= row length, so no
// validity test is needed.
//
// Radix select from the first byte in which the items differ; as soon as the digit that
// holds the limit-th best has at most kAmbMax members, those members are ranked
// directly (by image, then index) instead of refining further.
template <int BLOCK, int ITEMS, bool ROLLED, typename K, int CAND, typename S, typename Ord, typename Idx>
__device__ __forceinline__ void select_and_emit(TopkShared<K, CAND>& sm, const TopkIo<K, S>& io, int64_t row, const S* xr,
                                                int limit, int nitems, Ord ord, Idx idx) {
    const int tid = threadIdx.x;
    const int lane = lane_id();
    const int w = tid / kWave;
    constexpr int WAVES = BLOCK / kWave;
    auto for_items = [&](auto&& body) {
        if constexpr (ROLLED) {
#pragma unroll 1
            for (int i = 0; i < nitems; ++i) body(i);
        } else {
#pragma unroll
            for (int i = 0; i < ITEMS; ++i) body(i);
        }
    };
    if (tid == 0) { sm.count = 0; sm.amb_count = 0; }

    // ---- bytes in which every item agrees need no pass.  Padding (image 0) is left out of
    // the comparison; should the limit reach into the padding-valued items, nothing is skipped.
    K all_and = ~K(0), all_or = 0;
    uint32_t nonzero = 0;
    for_items([&](int i) {
        const K o = ord(i);
        if (o != 0) { all_and &= o; all_or |= o; }
        nonzero += static_cast<uint32_t>(__popcll(__ballot(o != 0)));
    });
    all_and = wave_reduce(all_and, [](K a, K b) { return a & b; });
    all_or = wave_reduce(all_or, [](K a, K b) { return a | b; });
    if (lane == 0) { sm.and_bits[w] = all_and; sm.or_bits[w] = all_or; sm.scan_tot[w] = nonzero; }
    team_sync<BLOCK>();
    nonzero = 0;
    for (int i = 0; i < WAVES; ++i) { all_and &= sm.and_bits[i]; all_or |= sm.or_bits[i]; nonzero += sm.scan_tot[i]; }
    team_sync<BLOCK>();            // scan_tot is reused below
    const K differ = (nonzero >= static_cast<uint32_t>(limit)) ? static_cast<K>(all_and ^ all_or) : ~K(0);

    K prefix = 0, decided = 0;
    uint32_t kk = static_cast<uint32_t>(limit), ties = nonzero;
#pragma unroll 1
    for (int pass = static_cast<int>(sizeof(K)) - 1; pass >= 0; --pass) {
        const int shift = 8 * pass;
        if (((differ >> shift) & 0xffu) == 0) {
            // all (non-padding) items share this byte
            prefix |= all_and & (static_cast<K>(0xffu) << shift);
            decided = static_cast<K>(~K(0) << shift);
            continue;
        }
        select_digit<BLOCK, ITEMS, ROLLED>(sm, nitems, shift, kk, ord, [&](int i) { return ((ord(i) ^ prefix) & decided) == 0; });
        prefix |= static_cast<K>(sm.sel_digit) << shift;
        decided = static_cast<K>(~K(0) << shift);
        kk = sm.sel_k;
        ties = sm.sel_ties;
        if (ties <= kAmbMax) break;
    }
    // now: (image & decided) > prefix  -> in;  == prefix -> one of `ties` items of which kk are in;  < prefix -> out

    if (ties <= kAmbMax) {
        // two sweeps, no atomics: every wave counts its winners / deciding-digit members with
        // ballots, the counts are prefix-summed over the team's waves, then each item is placed
        // at wave offset + number of such items before it in the wave
        const unsigned long long lt_mask = (1ull << lane) - 1ull;
        uint32_t n_in = 0, n_amb = 0;
        for_items([&](int i) {
            const K hi = ord(i) & decided;
            n_in += static_cast<uint32_t>(__popcll(__ballot(hi > prefix)));
            n_amb += static_cast<uint32_t>(__popcll(__ballot(hi == prefix)));
        });
        if (lane == 0) { sm.scan_tot[w] = n_in; sm.scan_tot[WAVES + w] = n_amb; }
        team_sync<BLOCK>();
        uint32_t b_in = 0, b_amb = 0;
        for (int i = 0; i < w; ++i) { b_in += sm.scan_tot[i]; b_amb += sm.scan_tot[WAVES + i]; }
        for_items([&](int i) {
            const K o = ord(i);
            const K hi = o & decided;
            const bool in = hi > prefix, maybe = hi == prefix;
            const unsigned long long m_in = __ballot(in), m_amb = __ballot(maybe);
            if (in) {
                const uint32_t slot = b_in + static_cast<uint32_t>(__popcll(m_in & lt_mask));
                if (slot < kMaxLimit) { sm.out_ord[slot] = o; sm.out_idx[slot] = idx(i); }
            }
            if (maybe) {
                const uint32_t slot = b_amb + static_cast<uint32_t>(__popcll(m_amb & lt_mask));
                if (slot < kAmbMax) { sm.amb_ord[slot] = o; sm.amb_idx[slot] = idx(i); }
            }
            b_in += static_cast<uint32_t>(__popcll(m_in));
            b_amb += static_cast<uint32_t>(__popcll(m_amb));
        });
        if (tid == 0) sm.count = static_cast<uint32_t>(limit) - kk;     // winners above the deciding digit
        team_sync<BLOCK>();
        if (kk == ties) {
            // the whole digit is in
            for (int e0 = 0; e0 < static_cast<int>(ties); e0 += BLOCK) {
                const int e = e0 + tid;
                const bool in = e < static_cast<int>(ties);
                const uint32_t slot = wave_append(&sm.count, in);
                if (in && slot < kMaxLimit) {
                    sm.out_ord[slot] = sm.amb_ord[e];
                    sm.out_idx[slot] = sm.amb_idx[e];
                }
            }
        } else {
            compute_ranks<BLOCK, K>(sm, sm.amb_ord, sm.amb_idx, static_cast<int>(ties));
            for (int e0 = 0; e0 < static_cast<int>(ties); e0 += BLOCK) {
                const int e = e0 + tid;
                const bool in = e < static_cast<int>(ties) && sm.rank[e] < kk;
                const uint32_t slot = wave_append(&sm.count, in);
                if (in && slot < kMaxLimit) {
                    sm.out_ord[slot] = sm.amb_ord[e];
                    sm.out_idx[slot] = sm.amb_idx[e];
                }
            }
        }
    } else {
        // more than kAmbMax items share the threshold image: take the kk lowest indices
        // among them, i.e. the kk largest images of ~index (indices are below 2^24 here)
        uint32_t k2 = 0, t2 = 0;
        const K threshold = prefix;
        const uint32_t inv = kth_largest<BLOCK, ITEMS, ROLLED, uint32_t>(
            sm, nitems, kk, [&](int i) { return ~idx(i); }, [&](int i) { return ord(i) == threshold && idx(i) < (1u << 24); },
            &k2, &t2, 2, 0xff000000u);
        const uint32_t idx_limit = ~inv;
        for_items([&](int i) {
            const uint32_t ix = idx(i);
            const K o = ord(i);
            const bool in = o > threshold || (o == threshold && ix <= idx_limit);
            const uint32_t slot = wave_append(&sm.count, in);
            if (in && slot < kMaxLimit) {
                sm.out_ord[slot] = o;
                sm.out_idx[slot] = ix;
            }
        });
    }
    team_sync<BLOCK>();

    // ---- order the winners: best first
    if (limit <= kMergeMax) {
        merge_rank_emit<BLOCK, K>(sm.out_ord, sm.out_idx, sm.pack, limit, limit, io, row, xr);
        return;
    }
    int kp = 1;
    while (kp < limit) kp <<= 1;
    for (int i = limit + tid; i < kp; i += BLOCK) {
        sm.out_ord[i] = 0;
        sm.out_idx[i] = 0xffffffffu;      // padding: worse than any real entry
    }
    team_sync<BLOCK>();
    for (int size = 2; size <= kp; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            for (int t = tid; t < kp / 2; t += BLOCK) {
                const int i = (t / stride) * 2 * stride + (t % stride);
                const int j = i + stride;
                const K oi = sm.out_ord[i], oj = sm.out_ord[j];
                const uint32_t xi = sm.out_idx[i], xj = sm.out_idx[j];
                const bool j_better = oj > oi || (oj == oi && xj < xi);
                const bool best_first = (i & size) == 0;
                if (j_better == best_first) {
                    sm.out_ord[i] = oj; sm.out_ord[j] = oi;
                    sm.out_idx[i] = xj; sm.out_idx[j] = xi;
                }
            }
            team_sync<BLOCK>();
        }
    }
    S* yr = io.y + io.ymap.at(row);
    const int64_t ir = io.imap.at(row);
    for (int j = tid; j < limit; j += BLOCK) emit_one<K>(io, yr, ir, xr, j, sm.out_ord[j], sm.out_idx[j]);
}

// E: the element type in memory.  type: its K-wide bit pattern; storage: its bits in memory;
// score: the arithmetic type elements are compared in.
template <typename E> struct BitsOf;
template <> struct BitsOf<float>   { using type = uint32_t; using storage = uint32_t; using score = float;   static constexpr int kind = kKeyFloat; };
template <> struct BitsOf<int32_t> { using type = uint32_t; using storage = uint32_t; using score = int32_t; static constexpr int kind = kKeyInt; };
template <> struct BitsOf<double>  { using type = uint64_t; using storage = uint64_t; using score = double;  static constexpr int kind = kKeyFloat; };
template <> struct BitsOf<int64_t> { using type = uint64_t; using storage = uint64_t; using score = int64_t; static constexpr int kind = kKeyInt; };
template <> struct BitsOf<half_t>  { using type = uint32_t; using storage = uint16_t; using score = float;   static constexpr int kind = kKeyFloat; };
template <> struct BitsOf<int16_t> { using type = uint32_t; using storage = uint16_t; using score = int32_t; static constexpr int kind = kKeyInt; };

// Short rows and small limits: one wavefront per row, four rows per workgroup, no workgroup
// barrier.  A row of at most 64 * ITEMS elements lives in the wave's registers as images.  The
// limit-th largest of the 64 lane maxima (distinct elements of the row) has at least `limit`
// elements at or above it; what reaches it - usually a few more than `limit` entries - is
// gathered through a 64-entry LDS buffer of the wave and ordered by one wave sort (or by
// counting, when there is only a handful).  When more than 64 elements reach the bound (long
// runs of equal values), the wave takes the `limit` best one after the other instead: exact
// for any input, and only slow where it is needed.
constexpr int kWaveRowMax = 1024;       // longest row topk_rows_wave takes (beyond, the pre-filter of topk_select with 256 threads a row is as fast or faster)
constexpr int kWaveRowLimit = 32;       // largest limit: the limit-th of 64 lane maxima lets about 45 entries through at 32, more than the 64 the buffer holds from 40 on
constexpr int kWaveSortItems = 4;       // rows of up to 64 * this many elements can be ordered whole by the wave

template <typename E, int ITEMS>
__global__ __launch_bounds__(256) void topk_rows_wave(TopkIo<typename BitsOf<E>::type, typename BitsOf<E>::storage> io,
                                                      int64_t rows, int64_t n, int limit) {
    using K = typename BitsOf<E>::type;
    using S = typename BitsOf<E>::storage;
    constexpr int kind = BitsOf<E>::kind;
    __shared__ K cand_ord[4][kWave];
    __shared__ uint32_t cand_idx[4][kWave];
    const int lane = lane_id();
    const int w = threadIdx.x / kWave;
    const int64_t block = io.xcd_blocks ? static_cast<int64_t>(blockIdx.x % 8) * io.xcd_blocks + blockIdx.x / 8 : blockIdx.x;
    const int64_t row = block * 4 + w;
    if (row >= rows) return;                               // whole waves leave; nothing below synchronises the workgroup
    const S* xr = io.x + io.xmap.at(row);
    S* yr = io.y + io.ymap.at(row);
    const int64_t ir = io.imap.at(row);
    const uint32_t n32 = static_cast<uint32_t>(n);
    const K flip = io.largest ? K(0) : (kind == kKeyFloat ? KeyBits<K>::kSign : ~K(0));

    // element i * 64 + lane is item i of the lane; padding carries image 0 and an index past the row
    K ord[ITEMS];
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        const uint32_t e = static_cast<uint32_t>(i * kWave + lane);
        ord[i] = e < n32 ? to_ord<K>(static_cast<K>(widen_bits<K, S>(xr[static_cast<int64_t>(e) * io.sx], kind) ^ flip), kind, 1) : K(0);
    }
    // rows of up to 256 elements and a limit for which the bound below is weak (or cannot be
    // formed: it is one of 64 lane maxima), and rows the bound fails on: order the whole row
    auto order_row = [&]() {
        uint32_t ix[ITEMS];
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) ix[i] = static_cast<uint32_t>(i * kWave + lane);      // padding: image 0, index past the row
        wave_bitonic_items<true, ITEMS>(ord, ix, [](K ka, uint32_t ia, K kb, uint32_t ib) { return beats<K>(ka, ia, kb, ib) != 0u; });
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
            const int e = i * kWave + lane;
            if (e < limit) emit_one<K>(io, yr, ir, xr, e, ord[i], ix[i]);
        }
    };
    if constexpr (ITEMS <= kWaveSortItems) {
        if (limit > kWaveRowLimit) {
            order_row();
            return;
        }
    }
    K best = 0;
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) best = ord[i] > best ? ord[i] : best;
    const K bound = lane_get(wave_sort_descending(best), limit - 1);
    uint32_t count = 0;
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) count += static_cast<uint32_t>(__popcll(__ballot(ord[i] >= bound)));

    if (count <= static_cast<uint32_t>(kWave)) {
        const unsigned long long lt_mask = (1ull << lane) - 1ull;
        uint32_t base = 0;
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
            const bool pass = ord[i] >= bound;
            const unsigned long long m = __ballot(pass);
            if (m != 0ull) {
                if (pass) {
                    const uint32_t slot = base + static_cast<uint32_t>(__popcll(m & lt_mask));
                    cand_ord[w][slot] = ord[i];
                    cand_idx[w][slot] = static_cast<uint32_t>(i * kWave + lane);
                }
                base += static_cast<uint32_t>(__popcll(m));
            }
        }
        team_sync<kWave>();
        const bool live = static_cast<uint32_t>(lane) < count;
        K o = live ? cand_ord[w][lane] : K(0);
        uint32_t x = live ? cand_idx[w][lane] : 0xffffffffu;
        uint32_t rank;
        if (count <= static_cast<uint32_t>(kCountMax)) {
            rank = 0;
            for (uint32_t j = 0; j < count; ++j) rank += beats<K>(lane_read(o, static_cast<int>(j)), lane_read(x, static_cast<int>(j)), o, x);
        } else {
            wave_sort_entries<K>(o, x);
            rank = static_cast<uint32_t>(lane);
        }
        if (live && rank < static_cast<uint32_t>(limit)) emit_one<K>(io, yr, ir, xr, static_cast<int>(rank), o, x);
        return;
    }

    if constexpr (ITEMS <= kWaveSortItems) {
        order_row();
        return;
    }
    // more than a wave's worth of entries reach the bound: take the best entry that comes
    // after the one taken last, `limit` times (entries are ordered by image, then by lower index)
    K last_o = ~K(0);
    uint32_t last_x = 0;
    bool first = true;
    for (int j = 0; j < limit; ++j) {
        K bo = 0;
        uint32_t bx = 0xffffffffu;
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
            const uint32_t e = static_cast<uint32_t>(i * kWave + lane);
            const bool after = first || beats<K>(last_o, last_x, ord[i], e) != 0u;      // not taken yet
            if (e < n32 && after && beats<K>(ord[i], e, bo, bx) != 0u) {
                bo = ord[i];
                bx = e;
            }
        }
        struct Entry {
            K o;
            uint32_t x;
        };
        const Entry top = wave_reduce(Entry{bo, bx}, [](Entry a, Entry b) { return beats<K>(b.o, b.x, a.o, a.x) ? b : a; });
        if (lane == 0) emit_one<K>(io, yr, ir, xr, j, top.o, top.x);
        last_o = top.o;
        last_x = top.x;
        first = false;
    }
}

// Rows that lie side by side in memory (the axis is an outer dimension of the tensor, the
// innermost row dimension has stride 1) and a limit of at most 16: one thread per row and
// segment of the axis, so the 64 lanes of a wave read 64 neighbouring elements whatever the
// stride along the axis.  A thread keeps the KMAX best (image, index) entries it has seen in
// registers, ordered; an element enters only when it beats the last of them.  SEG waves share
// 64 rows, each scanning a contiguous piece of the axis; their lists meet in LDS and the first
// wave merges and writes them.  No scratch, any row length.
constexpr int kColsLimit = 16;         // largest limit topk_cols takes
constexpr int kThreadRowLimit = 8;     // ... and topk_rows_thread
// longest row topk_rows_thread takes with 4-byte keys, half of it with 8-byte keys
// (dlfx_set_tuning "topk_thread_rows"); beyond, a wave per row has enough rows in flight and wins
}  // namespace
#if DLFX_TOPK_PART == 0
int g_topk_thread_rows = 256;
int g_topk_cols_waves = 0;            // dlfx_set_tuning "topk_cols_waves": 1, 4 or 8 wavefronts a block of 64 rows in topk_cols (0: by the shape)
#else
extern int g_topk_thread_rows;
extern int g_topk_cols_waves;
#endif
namespace {

template <typename K, int KMAX>
__device__ __forceinline__ void cols_insert(K (&lo)[KMAX], uint32_t (&li)[KMAX], K o, uint32_t x) {
    if (beats<K>(o, x, lo[KMAX - 1], li[KMAX - 1]) == 0u) return;
#pragma unroll
    for (int p = 0; p < KMAX; ++p) {
        const bool b = beats<K>(o, x, lo[p], li[p]) != 0u;
        const K to = lo[p];
        const uint32_t tx = li[p];
        lo[p] = b ? o : to;
        li[p] = b ? x : tx;
        o = b ? to : o;
        x = b ? tx : x;
    }
}

// The same for an element that comes after every entry of a full list (a higher index than all
// of them, no placeholder left): it enters before the entries with a smaller image, and a tie
// never moves it forward - one comparison per entry instead of the (image, index) pair's.
template <typename K, int KMAX>
__device__ __forceinline__ void cols_insert_later(K (&lo)[KMAX], uint32_t (&li)[KMAX], K o, uint32_t x) {
    if (!(o > lo[KMAX - 1])) return;
    bool b = false;
#pragma unroll
    for (int p = 0; p < KMAX; ++p) {
        b = b || o > lo[p];                 // (behind the place where it entered every entry moves down one place, ties included)
        const K to = lo[p];
        const uint32_t tx = li[p];
        lo[p] = b ? o : to;
        li[p] = b ? x : tx;
        o = b ? to : o;
        x = b ? tx : x;
    }
}

template <typename E, int KMAX, int SEG>
__global__ __launch_bounds__(kWave * SEG) void topk_cols(TopkIo<typename BitsOf<E>::type, typename BitsOf<E>::storage> io,
                                                         int64_t rows, int64_t n, int limit) {
    using K = typename BitsOf<E>::type;
    using S = typename BitsOf<E>::storage;
    constexpr int kind = BitsOf<E>::kind;
    constexpr int kUnroll = 8;
    __shared__ K s_ord[SEG > 1 ? SEG - 1 : 1][KMAX][kWave];
    __shared__ uint32_t s_idx[SEG > 1 ? SEG - 1 : 1][KMAX][kWave];
    const int lane = threadIdx.x % kWave;
    const int seg = threadIdx.x / kWave;
    // workgroups are dealt to the 8 XCDs in turn: give each XCD one contiguous range of rows,
    // so that the pieces of a page (and of a cache line) are fetched through one L2 and TLB
    const int64_t per_xcd = gridDim.x / 8;                 // the grid is a multiple of 8
    const int64_t block = static_cast<int64_t>(blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    const int64_t row = block * kWave + lane;
    const bool live = row < rows;
    const S* xr = io.x + (live ? io.xmap.at(row) : 0);
    const K flip = io.largest ? K(0) : (kind == kKeyFloat ? KeyBits<K>::kSign : ~K(0));

    K lo[KMAX];
    uint32_t li[KMAX];
#pragma unroll
    for (int p = 0; p < KMAX; ++p) {
        lo[p] = K(0);                    // beaten by every element of the row (lower index)
        li[p] = 0xffffffffu;
    }
    const int64_t chunk = (n + SEG - 1) / SEG;
    const int64_t j0 = seg * chunk;
    const int64_t j1 = j0 + chunk < n ? j0 + chunk : n;
    // (a wavefront runs an insertion wherever one of its 64 rows needs it, which is nearly
    // everywhere: the kernel is bound by vector ALU work - fp32 [32, 512, 56, 56] along axis 1,
    // limit 5: 5700 instructions a wavefront and 64 positions - so the list is exactly as long as
    // the limit asks and, once it is full, entries are compared by their images alone)
    constexpr int kFill = (KMAX + kUnroll - 1) / kUnroll * kUnroll;      // the list is full after so many elements
    for (int64_t j = j0; j < j1; j += kUnroll) {
        K o[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const bool in = live && j + u < j1;
            o[u] = in ? to_ord<K>(static_cast<K>(widen_bits<K, S>(load_stream(xr + (j + u) * io.sx), kind) ^ flip), kind, 1) : K(0);
        }
        // (lists of more than 8 entries keep the one insertion: two unrolled copies of it cost them
        // registers and a wavefront per SIMD - int64 [16, 80, 160, 160], limit 16: 406 -> 650 us)
        if (KMAX > 8 || j - j0 < kFill) {
#pragma unroll
            for (int u = 0; u < kUnroll; ++u)
                cols_insert<K, KMAX>(lo, li, o[u], (live && j + u < j1) ? static_cast<uint32_t>(j + u) : 0xffffffffu);
        } else {
#pragma unroll
            for (int u = 0; u < kUnroll; ++u) cols_insert_later<K, KMAX>(lo, li, o[u], static_cast<uint32_t>(j + u));
        }
    }
    if constexpr (SEG > 1) {
        if (seg > 0) {
#pragma unroll
            for (int p = 0; p < KMAX; ++p) {
                s_ord[seg - 1][p][lane] = lo[p];
                s_idx[seg - 1][p][lane] = li[p];
            }
        }
        __syncthreads();
        if (seg > 0) return;
        for (int s = 0; s < SEG - 1; ++s) {
#pragma unroll
            for (int p = 0; p < KMAX; ++p) cols_insert<K, KMAX>(lo, li, s_ord[s][p][lane], s_idx[s][p][lane]);
        }
    }
    if (!live) return;
    S* yr = io.y + io.ymap.at(row);
    const int64_t ir = io.imap.at(row);
#pragma unroll
    for (int p = 0; p < KMAX; ++p)
        if (p < limit) emit_one<K>(io, yr, ir, xr, p, lo[p], li[p]);
}

// Many short contiguous rows and a limit of at most 8: one thread per row again, but the rows
// lie one after the other in memory, so a wavefront reads its 64 rows in pieces of 32 elements
// with coalesced loads (a half-wave per row piece), passes them through its own slab of LDS
// (row pitch 33: no bank conflicts either way), and every lane then walks its own row and
// keeps the KMAX best entries in the ordered register list of topk_cols.  The work per element
// does not depend on the row length, where a wave per row pays its fixed cost for every row.
constexpr int kThreadRowChunk = 32;

template <typename E, int KMAX, bool ONE_RUN>
__global__ __launch_bounds__(256) void topk_rows_thread(TopkIo<typename BitsOf<E>::type, typename BitsOf<E>::storage> io,
                                                        int64_t rows, int64_t n, int limit, int64_t row_pitch) {
    using K = typename BitsOf<E>::type;
    using S = typename BitsOf<E>::storage;
    constexpr int kind = BitsOf<E>::kind;
    constexpr int C = kThreadRowChunk;
    __shared__ S slab[4][kWave * (C + 1)];
    const int lane = lane_id();
    const int w = threadIdx.x / kWave;
    const int64_t row0 = (static_cast<int64_t>(blockIdx.x) * 4 + w) * kWave;
    if (row0 >= rows) return;                              // whole waves leave; nothing below synchronises the workgroup
    const int64_t row = row0 + lane;
    const bool live = row < rows;
    const int n32 = static_cast<int>(n);
    const K flip = io.largest ? K(0) : (kind == kKeyFloat ? KeyBits<K>::kSign : ~K(0));
    S* mine = slab[w];

    K lo[KMAX];
    uint32_t li[KMAX];
#pragma unroll
    for (int p = 0; p < KMAX; ++p) {
        lo[p] = K(0);                    // beaten by every element of the row (lower index)
        li[p] = 0xffffffffu;
    }
    const int half = lane / C, col = lane % C;             // C == 32: lanes 0-31 one row piece, lanes 32-63 the next
    // rows shorter than a piece that follow each other without a gap: the wave's 64 rows are
    // one run of 64 * n elements, read 64 at a time (a piece per row would leave most lanes idle)
    // (ONE_RUN, chosen by the host: n < 32 and the row pitch equals n)
    const int run = static_cast<int>((rows - row0 < kWave ? rows - row0 : kWave) * n);
    const float inv_n = 1.0f / static_cast<float>(n32);
    for (int c0 = 0; c0 < n32; c0 += C) {
        S in[C];
        if constexpr (ONE_RUN) {
#pragma unroll
            for (int t = 0; t < C; ++t) {
                const int f = t * kWave + lane;
                in[t] = (t < n32 && f < run) ? io.x[row0 * row_pitch + f] : S(0);
            }
#pragma unroll
            for (int t = 0; t < C; ++t) {
                const int f = t * kWave + lane;
                const int r = static_cast<int>((static_cast<float>(f) + 0.5f) * inv_n);      // f / n, exact for f < 2048
                if (t < n32 && f < run) mine[r * (C + 1) + (f - r * n32)] = in[t];
            }
        } else {
#pragma unroll
            for (int t = 0; t < C; ++t) {
                const int r = 2 * t + half;
                const bool ok = row0 + r < rows && c0 + col < n32;
                // (no non-temporal hint: pieces of rows that are not whole cache lines share lines, and a line two
                // such loads share is fetched twice - fp32 [500000, 200], limit 1: 117 us with the hint, 107 without)
                in[t] = ok ? io.x[(row0 + r) * row_pitch + (c0 + col)] : S(0);
            }
#pragma unroll
            for (int t = 0; t < C; ++t) mine[(2 * t + half) * (C + 1) + col] = in[t];
        }
        team_sync<kWave>();
#pragma unroll
        for (int j = 0; j < C; ++j) {
            if (c0 + j < n32) {                            // the same for every lane: a scalar branch past the row's end
                const K o = live ? to_ord<K>(static_cast<K>(widen_bits<K, S>(mine[lane * (C + 1) + j], kind) ^ flip), kind, 1) : K(0);
                cols_insert<K, KMAX>(lo, li, o, live ? static_cast<uint32_t>(c0 + j) : 0xffffffffu);
            }
        }
        team_sync<kWave>();
    }
    if (!live) return;
    const S* xr = io.x + row * row_pitch;
    S* yr = io.y + io.ymap.at(row);
    const int64_t ir = io.imap.at(row);
#pragma unroll
    for (int p = 0; p < KMAX; ++p)
        if (p < limit) emit_one<K>(io, yr, ir, xr, p, lo[p], li[p]);
}

// Rows of at most 64 elements side by side in memory and a limit the register lists of
// topk_cols do not take: a workgroup reads 64 neighbouring rows with coalesced loads (64 rows
// wide, one axis position at a time) into an LDS tile of images (pitch 65: no bank conflicts
// either way), each wavefront orders sixteen of them whole (lane l holds element l), and the
// winners leave the way the rows came, `limit` axis positions deep.
template <typename E>
__global__ __launch_bounds__(256) void topk_cols_wave(TopkIo<typename BitsOf<E>::type, typename BitsOf<E>::storage> io,
                                                      int64_t rows, int64_t n, int limit) {
    using K = typename BitsOf<E>::type;
    using S = typename BitsOf<E>::storage;
    constexpr int kind = BitsOf<E>::kind;
    constexpr int kPitch = kWave + 1;
    __shared__ K images[kWave * kPitch];
    __shared__ uint32_t places[kWave * kPitch];
    const int lane = lane_id();
    const int w = threadIdx.x / kWave;
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * kWave;
    const int r = lane;                                    // this thread's row of the tile in the load and store phases
    const bool row_live = row0 + r < rows;
    const int n32 = static_cast<int>(n);
    const K flip = io.largest ? K(0) : (kind == kKeyFloat ? KeyBits<K>::kSign : ~K(0));
    const S* xr = io.x + (row_live ? io.xmap.at(row0 + r) : 0);
    for (int a = w; a < n32; a += 4)
        images[a * kPitch + r] = row_live ? to_ord<K>(static_cast<K>(widen_bits<K, S>(load_stream(xr + static_cast<int64_t>(a) * io.sx), kind) ^ flip), kind, 1) : K(0);
    __syncthreads();
    for (int q = w; q < kWave; q += 4) {                   // row q of the tile, element `lane`
        K ord[1] = {lane < n32 ? images[lane * kPitch + q] : K(0)};
        uint32_t ix[1] = {static_cast<uint32_t>(lane)};    // padding: image 0 and an index past the row
        wave_bitonic_items<true, 1>(ord, ix, [](K ka, uint32_t ia, K kb, uint32_t ib) { return beats<K>(ka, ia, kb, ib) != 0u; });
        images[lane * kPitch + q] = ord[0];
        places[lane * kPitch + q] = ix[0];
    }
    __syncthreads();
    if (!row_live) return;
    S* yr = io.y + io.ymap.at(row0 + r);
    const int64_t ir = io.imap.at(row0 + r);
    for (int a = w; a < limit; a += 4) emit_one<K>(io, yr, ir, xr, a, images[a * kPitch + r], places[a * kPitch + r]);
}

// E: the element type.  LOAD says how a row is read (the host decides): kLoadAligned - the axis
// is contiguous and every row starts on a 16-byte boundary, so rows are read with 128-bit loads
// off one base register; kLoadShifted - contiguous rows that start anywhere (an odd row length)
// are laid out from the boundary before them: position p of that layout is element p - shift,
// the positions below `shift` are padding, and every whole vector of the row is still one
// aligned load; kLoadStrided - element by element, any stride.
//
// Elements are held as scores of type T: the element itself when the largest are wanted,
// its order-reversing image otherwise (sign flip for floats, complement for integers), so
// the kernel always looks for the largest scores and compares them natively.
constexpr int kLoadStrided = 0, kLoadAligned = 1, kLoadShifted = 2;

template <typename E, int BLOCK, int ITEMS, int LOAD>
__global__ __launch_bounds__(BLOCK) __attribute__((amdgpu_waves_per_eu(BLOCK >= 1024 && sizeof(typename BitsOf<E>::type) == 4 && ITEMS <= 32 ? 8 : 1)))
void topk_select(TopkIo<typename BitsOf<E>::type, typename BitsOf<E>::storage> io, int64_t n, int limit,
                 uint32_t* __restrict__ row_state, typename BitsOf<E>::type* __restrict__ spill_ord,
                 uint32_t* __restrict__ spill_idx) {
    using K = typename BitsOf<E>::type;
    using S = typename BitsOf<E>::storage;
    using T = typename BitsOf<E>::score;
    constexpr int kind = BitsOf<E>::kind;
    constexpr int V = (16 / sizeof(S) < ITEMS) ? 16 / sizeof(S) : ITEMS;
    constexpr int G = ITEMS / V;
    constexpr int WAVES = BLOCK / kWave;
    using VecT = Vec<S, V>;
    constexpr int CAP = cand_cap<K>();
    // A row whose items are no more than the candidates a longer row may leave never hands
    // anything to a second kernel: it keeps the survivors it can rank here (kMergeMax) and
    // otherwise selects from its registers.
    constexpr bool kShort = BLOCK * ITEMS <= CAP;
    constexpr uint32_t kCap = static_cast<uint32_t>(kShort ? kMergeMax : CAP);
    __shared__ TopkShared<K, static_cast<int>(kCap)> sm;

    const int tid = threadIdx.x;
    const int lane = lane_id();
    const int w = tid / kWave;
    const int64_t row = blockIdx.x;
    if (io.segs > 1 && row % io.segs == io.segs - 1) n = io.last_n;
    const S* xr = io.x + io.xmap.at(row);
    if (tid < kRadix) sm.hist[tid] = 0;
    DLFX_PHASE_BEGIN();

    // item (g, e) of thread t is position ((g*BLOCK + t)*V + e) of the row: element position - shift
    // (padding before the row gets an index far beyond it, like the padding behind it)
    const uint32_t n32 = static_cast<uint32_t>(n);        // rows here have at most 65536 elements
    const uint32_t shift = LOAD == kLoadShifted ? static_cast<uint32_t>((reinterpret_cast<uintptr_t>(xr) / sizeof(S)) % V) : 0u;
    const uint32_t end32 = n32 + shift;                   // positions [shift, end32) are the row
    const uint32_t tid_v = static_cast<uint32_t>(tid) * V;
    auto index_of = [&](int i) -> uint32_t {
        return tid_v + static_cast<uint32_t>((i / V) * (BLOCK * V) + (i % V)) - shift;
    };
    const K flip = io.largest ? K(0) : (kind == kKeyFloat ? KeyBits<K>::kSign : ~K(0));
    const T worst = std::is_integral<T>::value ? std::numeric_limits<T>::lowest() : -std::numeric_limits<T>::infinity();
    auto score_of = [&](S stored) -> T { return bit_cast<T>(static_cast<K>(widen_bits<K, S>(stored, kind) ^ flip)); };
    // order-preserving unsigned image of a score (scores are always maximised)
    auto ord_of = [&](T sc) -> K { return to_ord<K>(bit_cast<K>(sc), kind, 1); };

    T sc[ITEMS];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const uint32_t i0 = tid_v + static_cast<uint32_t>(g * (BLOCK * V));
        if (LOAD != kLoadStrided && i0 >= shift && i0 + V <= end32) {
            const VecT a = load_stream(reinterpret_cast<const VecT*>(xr + i0 - shift));
#pragma unroll
            for (int e = 0; e < V; ++e) sc[g * V + e] = score_of(a.v[e]);
        } else {
#pragma unroll
            for (int e = 0; e < V; ++e) {
                const uint32_t ix = i0 + e - shift;
                const int64_t at = LOAD != kLoadStrided ? static_cast<int64_t>(ix) : static_cast<int64_t>(ix) * io.sx;
                sc[g * V + e] = (ix < n32) ? score_of(xr[at]) : worst;
            }
        }
    }
    // ---- pre-filter.  The largest element of each thread is a distinct element of the
    // row, and so is the largest of any group of threads.  A bound that provably has at
    // least `limit` elements at or above it comes from 16 or 64 such samples:
    //   * limit <= the number of waves: the limit-th largest of the wave maxima;
    //   * limit <= four times that: the limit-th largest of the maxima of 16-lane rows;
    //   * above: every wave sorts its 64 thread maxima; the value at position p*s - 1 of a
    //     wave has p*s elements at or above it.  SPW such samples per wave (p = 1..SPW, four
    //     from each of sixteen waves, sixteen from each of four: 64 in all) are
    //     sorted together: the m-th largest sample has at least m*s elements at or above
    //     it (q samples of one wave among the first m stand for q*s elements of that
    //     wave), so with m*s >= limit it cannot exceed the limit-th largest element.
    // Everything below the bound is out; what is left is usually 1 to 2 times `limit`.
    constexpr int SPW = kWave / WAVES;                 // samples a wave gives in the third form: 64 in all
    static_assert(WAVES <= 16 && SPW * WAVES == kWave, "the samples of all waves fill one wave");
    T tmax = worst;
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) tmax = sc[i] > tmax ? sc[i] : tmax;
    // NaNs compare false with everything, so the comparisons below would drop them, while
    // the radix selection (and the sort) place them by their bit pattern, above +inf or
    // below -inf.  A row that holds one is therefore selected exactly (short rows from the
    // registers below, long rows by topk_finish from the row itself); the sum of a thread's scores is NaN exactly when one of them is, or when
    // infinities of both signs meet, which only costs that row the slower path.
    bool nan_seen = false;
    if constexpr (!std::is_integral<T>::value) {
        T sum = T(0);
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) sum += sc[i];
        nan_seen = sum != sum;
    }
    T* red = reinterpret_cast<T*>(sm.out_ord);
    if (tid == 0) sm.count = 0u;
    DLFX_PHASE(0);            // loads and thread maxima
    auto larger = [](T a, T b) { return a > b ? a : b; };
    // (a row shorter than the workgroup's first vectors leaves the last waves and 16-lane rows
    // without elements: a sample from there bounds nothing, so only the full ones count)
    const int full_waves = static_cast<int>(end32 / static_cast<uint32_t>(kWave * V));
    const int full_rows = static_cast<int>(end32 / static_cast<uint32_t>(16 * V));
    int samples, mth;
    if (limit <= WAVES && limit <= full_waves) {
        const T wmax = wave_reduce(tmax, larger);
        if (lane == 0) red[w] = wmax;
        samples = WAVES;
        mth = limit;
    } else if (limit <= 4 * WAVES && limit <= full_rows) {
        const T rmax = group_reduce(tmax, 16, larger);
        if ((lane & 15) == 0) red[w * 4 + (lane >> 4)] = rmax;
        samples = 4 * WAVES;
        mth = limit;
    } else if (ITEMS >= 2 && 2 * limit > BLOCK) {
        // A limit above half the number of threads would take its bound from the weakest thread
        // maxima of every wave, which most of the row exceeds.  The two halves of a thread's
        // items are sampled as threads of their own instead: twice as many waves of maxima,
        // half as many samples from each, all from the upper half of its 64.
        constexpr int HALF = SPW / 2;
        const int stride = (limit + 63) / 64;
        T first_half = worst, second_half = worst;
#pragma unroll
        for (int i = 0; i < ITEMS; i += 2) {               // (every other item: a short row fills both halves)
            first_half = larger(first_half, sc[i]);
            if (i + 1 < ITEMS) second_half = larger(second_half, sc[i + 1]);
        }
        const T sorted_first = wave_sort_descending(first_half), sorted_second = wave_sort_descending(second_half);
#pragma unroll
        for (int p = 1; p <= HALF; ++p) {
            if (lane + 1 == p * stride) {
                red[w * SPW + p - 1] = sorted_first;
                red[w * SPW + HALF + p - 1] = sorted_second;
            }
        }
        samples = kWave;
        mth = (limit + stride - 1) / stride;                                       // <= 64
    } else {
        // (the last sample of a wave is its thread maximum number SPW * stride <= 64; a limit
        // above the workgroup's size has no bound and is given none below)
        constexpr int kMaxStride = kWave / SPW;
        const int stride = (limit + 31) / 32 <= kMaxStride ? (limit + 31) / 32 : (limit + 63) / 64;
        const T sorted = wave_sort_descending(tmax);
#pragma unroll
        for (int p = 1; p <= SPW; ++p)
            if (lane + 1 == p * stride) red[w * SPW + p - 1] = sorted;
        samples = kWave;
        mth = (limit + stride - 1) / stride;                                       // <= 64
    }
    __syncthreads();
    T bound;
    if (samples == WAVES) {
        // sixteen samples: every wave orders them itself (ten exchange steps)
        bound = lane < WAVES ? red[lane] : worst;
        bound = lane_get(wave_sort_descending<16>(bound), mth - 1);
    } else {
        // one wave orders the samples; the others wait (sixteen waves sorting the same
        // samples would only compete for the issue slots of the row that shares this
        // compute unit)
        if (w == 0) {
            T b = wave_sort_descending(lane < samples ? red[lane] : worst);
            b = lane_get(b, (mth - 1) & (kWave - 1));
            if (limit > BLOCK) b = worst;
            if (lane == 0) red[kWave] = b;
        }
        __syncthreads();
        bound = red[kWave];
    }
    DLFX_PHASE(1);            // bound
    // ---- survivors go to LDS as (image, index).  A wave counts its survivors with one
    // ballot per item, reserves that many slots with one atomic and places every survivor
    // at the wave's base + the number of the wave's survivors before it; their order in
    // LDS does not matter (they are ranked by image and index afterwards).  The ballots
    // are kept in scalar registers for the second sweep while there are few enough.  What
    // is stored is the score's bit pattern; its image is formed when the few survivors
    // are read back.  A wave none of whose thread maxima reaches the bound has none.
    constexpr bool kKeepMasks = ITEMS <= 32;
    unsigned long long masks[kKeepMasks ? ITEMS : 1];
    uint32_t wave_count = 0;
    if (__ballot(tmax >= bound) != 0ull) {
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
            const unsigned long long m = __ballot(sc[i] >= bound);
            if constexpr (kKeepMasks) masks[i] = m;
            wave_count += static_cast<uint32_t>(__popcll(m));
        }
    }
    if (__ballot(nan_seen) != 0ull) wave_count = kCap + 1u;       // more than fits: the row goes to topk_finish
    if (wave_count != 0u) {
        uint32_t base = 0;
        if (lane == 0) base = atomicAdd(&sm.count, wave_count);
        base = lane_read(base, 0);
        if (base + wave_count <= kCap) {
            const unsigned long long lt_mask = (1ull << lane) - 1ull;
#pragma unroll
            for (int i = 0; i < ITEMS; ++i) {
                unsigned long long m;
                if constexpr (kKeepMasks) m = masks[i];
                else m = __ballot(sc[i] >= bound);
                if (m != 0ull) {
                    if (sc[i] >= bound) {
                        const uint32_t slot = base + static_cast<uint32_t>(__popcll(m & lt_mask));
                        sm.cand_ord[slot] = bit_cast<K>(sc[i]);
                        sm.cand_idx[slot] = index_of(i);
                    }
                    base += static_cast<uint32_t>(__popcll(m));
                }
            }
        }
    }
    __syncthreads();
    const uint32_t total = sm.count;              // above the capacity: not all were stored
    DLFX_PHASE(2);            // compaction
    // What happens next depends on how many survived:
    //   * up to kMergeMax: ordered here by sorted runs and ranks, answer written (handing
    //     them to a second kernel with small workgroups was measured: slower);
    //   * up to kCandCap: they are handed, through global memory, to topk_finish, whose
    //     small workgroups hide the latency of an exact radix selection much better than
    //     this one (which holds a whole row) could;
    //   * more (long runs of equal values, adversarial order), or a limit the bound does
    //     not hold for: topk_finish selects from the row itself.
    if (total <= static_cast<uint32_t>(kMergeMax) && limit <= BLOCK) {
        if (tid == 0) row_state[row] = kRowDone;
        merge_rank_emit<BLOCK, K>(sm.cand_ord, sm.cand_idx, sm.pack, static_cast<int>(total), limit, io, row, xr,
                                  [&](K bits) { return ord_of(bit_cast<T>(bits)); });
        DLFX_PHASE(3);        // ordering and output
    } else if constexpr (kShort) {
        // a short row whose survivors are too many to rank (or that holds a NaN): exact
        // selection from the registers, no second kernel
        __syncthreads();                          // every thread has read the count select_and_emit clears
        if (tid == 0) row_state[row] = kRowDone;
        select_and_emit<BLOCK, ITEMS, false>(sm, io, row, xr, limit, ITEMS,
                                             [&](int i) { return index_of(i) < n32 ? ord_of(sc[i]) : K(0); }, index_of);
    } else if (total <= CAP && limit <= BLOCK) {
        if (tid == 0) row_state[row] = total;
        K* so = spill_ord + row * CAP;
        uint32_t* si = spill_idx + row * CAP;
        for (uint32_t i = tid; i < total; i += BLOCK) {
            so[i] = ord_of(bit_cast<T>(sm.cand_ord[i]));
            si[i] = sm.cand_idx[i];
        }
    } else {
        if (tid == 0) row_state[row] = kRowWhole;
    }
}

// Second stage of the selection for rows topk_select did not finish: exact selection among the row's
// spilled candidates, or over the whole row when it has to be.
template <typename E>
__global__ __launch_bounds__(kSelectThreads) void topk_finish(
    TopkIo<typename BitsOf<E>::type, typename BitsOf<E>::storage> io, int64_t n, int limit, const uint32_t* __restrict__ row_state,
    const typename BitsOf<E>::type* __restrict__ spill_ord, const uint32_t* __restrict__ spill_idx) {
    using K = typename BitsOf<E>::type;
    using S = typename BitsOf<E>::storage;
    constexpr int kind = BitsOf<E>::kind;
    constexpr int SEL = kSelectThreads;
    __shared__ TopkShared<K> sm;
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x;
    const uint32_t state = row_state[row];
    if (state == kRowDone) return;
    if (io.segs > 1 && row % io.segs == io.segs - 1) n = io.last_n;
    const S* xr = io.x + io.xmap.at(row);
    if (tid < kRadix) sm.hist[tid] = 0;
    if (state != kRowWhole) {
        const uint32_t total = state;
        constexpr int CAP = cand_cap<K>();
        const K* so = spill_ord + row * CAP;
        const uint32_t* si = spill_idx + row * CAP;
        for (uint32_t i = tid; i < total; i += SEL) {
            sm.cand_ord[i] = so[i];
            sm.cand_idx[i] = si[i];
        }
        __syncthreads();
        if (total <= static_cast<uint32_t>(kMergeMax)) {
            merge_rank_emit<SEL, K>(sm.cand_ord, sm.cand_idx, sm.pack, static_cast<int>(total), limit, io, row, xr);
            return;
        }
        const int per_thread = static_cast<int>((total + SEL - 1) / SEL);
        select_and_emit<SEL, CAP / SEL, true>(
            sm, io, row, xr, limit, per_thread,
            [&](int j) { const uint32_t s2 = j * SEL + tid; return s2 < total ? sm.cand_ord[s2] : K(0); },
            [&](int j) { const uint32_t s2 = j * SEL + tid; return s2 < total ? sm.cand_idx[s2] : 0xffffffffu; });
    } else {
        __syncthreads();
        const uint32_t n32 = static_cast<uint32_t>(n);
        const K flip = io.largest ? K(0) : (kind == kKeyFloat ? KeyBits<K>::kSign : ~K(0));
        const int per_thread = static_cast<int>((n32 + SEL - 1) / SEL);
        select_and_emit<SEL, 1, true>(
            sm, io, row, xr, limit, per_thread,
            [&](int j) {
                const uint32_t ix = j * SEL + tid;
                return ix < n32 ? to_ord<K>(static_cast<K>(widen_bits<K, S>(xr[static_cast<int64_t>(ix) * io.sx], kind) ^ flip), kind, 1) : K(0);
            },
            [&](int j) { return static_cast<uint32_t>(j * SEL + tid); });
    }
}

// Fallback epilogue: first `limit` entries of each row of a full stable argsort.
template <typename K, typename S>
__global__ __launch_bounds__(256) void topk_take(const S* __restrict__ ys, const int32_t* __restrict__ is,
                                                  int64_t m, int64_t n, int64_t limit, TopkIo<K, S> io) {
    const int64_t g = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (g >= m * limit) return;
    const int64_t row = g / limit, j = g - row * limit;
    io.y[io.ymap.at(row) + j * io.sy] = ys[row * n + j];
    const int32_t ix = is[row * n + j];
    if (io.idx64) static_cast<int64_t*>(io.idx)[io.imap.at(row) + j * io.si] = ix;
    else static_cast<int32_t*>(io.idx)[io.imap.at(row) + j * io.si] = ix;
}

// Scratch of the selection path: one state word per row and room for kCandCap spilled
// candidates per row (rows no longer than kCandCap finish in one kernel and need none).
struct SelectLayout {
    size_t state_off, ord_off, idx_off, total;
};
SelectLayout select_layout(size_t key_size, int64_t m, int64_t n) {
    SelectLayout l{0, 0, 0, 0};
    const int64_t cap = key_size == 4 ? kCandCap : kCandCap / 2;
    l.ord_off = align_up(static_cast<size_t>(m) * 4, 256);
    if (n <= cap) {
        l.idx_off = l.ord_off;
        l.total = l.ord_off;
        return l;
    }
    l.idx_off = l.ord_off + align_up(static_cast<size_t>(m) * cap * key_size, 256);
    l.total = l.idx_off + align_up(static_cast<size_t>(m) * cap * 4, 256);
    return l;
}

bool selection_fits(size_t key_size, int64_t n, int64_t limit) {
    if (limit > kMaxLimit) return false;
    // more than an eighth of a short row: no bound keeps few enough candidates, and the row's
    // whole sort on chip (one workgroup, one read) takes half the time of the exact selection
    if (n <= 4096 && limit > 256 && limit * 8 > n) return false;
    return n <= (key_size == 4 ? 65536 : 32768);
}

// The selection kernels over `m` rows of `n` elements (n within selection_fits).
template <typename T>
int launch_select(hipStream_t stream, const TopkIo<typename BitsOf<T>::type, typename BitsOf<T>::storage>& io, int64_t m, int64_t n,
                  int64_t limit, void* scratch, size_t scratch_bytes) {
    using K = typename BitsOf<T>::type;
    using S = typename BitsOf<T>::storage;
    const dim3 grid(static_cast<unsigned>(m));
    const int lim = static_cast<int>(limit);
    bool aligned = io.sx == 1 && reinterpret_cast<uintptr_t>(io.x) % 16 == 0;
    for (int i = 0; i < io.xmap.rank; ++i) aligned = aligned && io.xmap.strides[i] % (16 / static_cast<int64_t>(sizeof(S))) == 0;
    const SelectLayout sl = select_layout(sizeof(K), m, n);
    if (sl.total && (!scratch || scratch_bytes < sl.total)) return DLFX_ERR_SCRATCH_TOO_SMALL;
    char* sbase = static_cast<char*>(scratch);
    uint32_t* row_state = reinterpret_cast<uint32_t*>(sbase + sl.state_off);
    K* spill_ord = reinterpret_cast<K*>(sbase + sl.ord_off);
    uint32_t* spill_idx = reinterpret_cast<uint32_t*>(sbase + sl.idx_off);
    if (n <= kWaveRowMax && (lim <= kWaveRowLimit || n <= kWaveSortItems * kWave)) {      // at most 256 elements: a wave can order the whole row, whatever the limit
        TopkIo<K, S> wio = io;
        int64_t wblocks = ceil_div(m, 4);
        if (io.sx != 1 && io.sx != -1 && io.xmap.rank >= 1 && io.xmap.strides[io.xmap.rank - 1] == 1 && wblocks >= 64) {
            wio.xcd_blocks = ceil_div(wblocks, 8);
            wblocks = wio.xcd_blocks * 8;
        }
        const dim3 wgrid(static_cast<unsigned>(wblocks));
#define DLFX_TOPK_WAVE(ITEMS) topk_rows_wave<T, ITEMS><<<wgrid, dim3(256), 0, stream>>>(wio, m, n, lim)
        if (n <= 64) DLFX_TOPK_WAVE(1);
        else if (n <= 128) DLFX_TOPK_WAVE(2);
        else if (n <= 256) DLFX_TOPK_WAVE(4);
        else if (n <= 512) DLFX_TOPK_WAVE(8);
        else DLFX_TOPK_WAVE(16);
#undef DLFX_TOPK_WAVE
        DLFX_CHECK_LAUNCH();
        return DLFX_OK;
    }
#define DLFX_TOPK(BLOCK, ITEMS)                                                                     \
do {                                                                                            \
    if (load == kLoadAligned) topk_select<T, BLOCK, ITEMS, kLoadAligned><<<grid, dim3(BLOCK), 0, stream>>>(io, n, lim, row_state, spill_ord, spill_idx); \
    else if (load == kLoadShifted) topk_select<T, BLOCK, ITEMS, kLoadShifted><<<grid, dim3(BLOCK), 0, stream>>>(io, n, lim, row_state, spill_ord, spill_idx); \
    else topk_select<T, BLOCK, ITEMS, kLoadStrided><<<grid, dim3(BLOCK), 0, stream>>>(io, n, lim, row_state, spill_ord, spill_idx);      \
} while (0)
    // Contiguous rows off a 16-byte boundary are laid out from the boundary before them, which
    // takes up to a vector less one element more room: the size class is picked for that, unless
    // it would take the row beyond what the kernel holds or into the classes that hand
    // candidates to topk_finish through scratch the caller was not asked for.
    int load = aligned ? kLoadAligned : kLoadStrided;
    int64_t np = n;
    if (!aligned && io.sx == 1 && n > 8192) {           // (shorter rows measured the same or faster element by element)
        const int64_t padded = n + 16 / static_cast<int64_t>(sizeof(S)) - 1;
        if (padded <= (sizeof(K) == 4 ? 65536 : 32768) && (padded <= cand_cap<K>() || n > cand_cap<K>())) {
            load = kLoadShifted;
            np = padded;
        }
    }
    // (rows of up to 8192 elements are never read in the shifted layout)
#define DLFX_TOPK_SHORT(BLOCK, ITEMS)                                                               \
do {                                                                                            \
    if (load == kLoadAligned) topk_select<T, BLOCK, ITEMS, kLoadAligned><<<grid, dim3(BLOCK), 0, stream>>>(io, n, lim, row_state, spill_ord, spill_idx); \
    else topk_select<T, BLOCK, ITEMS, kLoadStrided><<<grid, dim3(BLOCK), 0, stream>>>(io, n, lim, row_state, spill_ord, spill_idx);      \
} while (0)
    if (np <= 1024) DLFX_TOPK_SHORT(256, 4);
    else if (np <= 2048) {
        // (a limit above the workgroup's size has no bound from the pre-filter: the larger workgroup takes those)
        if (lim <= 256) DLFX_TOPK_SHORT(256, 8);
        else DLFX_TOPK_SHORT(1024, 2);
    } else if (np <= 4096) {
        if (lim <= 256 && sizeof(K) == 4) DLFX_TOPK_SHORT(256, 16);
        else DLFX_TOPK_SHORT(1024, 4);
    }
    else if (np <= 8192) DLFX_TOPK_SHORT(1024, 8);
#undef DLFX_TOPK_SHORT
    else if (np <= 16384) DLFX_TOPK(1024, 16);
    else if (np <= 32768) {
        DLFX_TOPK(1024, 32);
    } else {
        if constexpr (sizeof(K) == 4) DLFX_TOPK(1024, 64);
        else return DLFX_ERR_TOO_LARGE;
    }
#undef DLFX_TOPK
    DLFX_CHECK_LAUNCH();
    if (n > cand_cap<K>()) {
        topk_finish<T><<<grid, dim3(kSelectThreads), 0, stream>>>(io, n, lim, row_state, spill_ord, spill_idx);
        DLFX_CHECK_LAUNCH();
    }
    return DLFX_OK;
}

// ---------------------------------------------------------------- rows longer than the selection kernel takes
// A long row is cut into segments the selection kernel takes (a launch of m * segs "rows"); each
// leaves its `limit` best as (value, index within the segment) in scratch, ordered, so that
// among equal values a lower place in the candidate array means a lower index in the row.
// top_k of the m rows of segs * limit candidates (this routine again) then yields the values
// and the places of the winners, and topk_places_to_indices turns places into row indices.
struct LongPlan {
    bool ok;
    int64_t seg_len, segs, last_n;
    int64_t keep;                      // what every segment leaves: `limit`, or one more (below)
    size_t val_off, idx_off, pos_off, rest_off, total;
};

size_t top_k_scratch_impl(int dtype, int64_t m, int64_t n, int64_t limit);

LongPlan long_plan(int dtype, size_t elem_size, size_t key_size, int64_t m, int64_t n, int64_t limit) {
    LongPlan p{};
    const int64_t cap = key_size == 4 ? 65536 : 32768;
    if (n <= cap || limit > kMaxLimit) return p;
    int64_t segs = ceil_div(n, cap);
    p.seg_len = align_up(static_cast<size_t>(ceil_div(n, segs)), 8);      // segments start on 16-byte boundaries when the row does
    p.segs = ceil_div(n, p.seg_len);
    p.last_n = n - (p.segs - 1) * p.seg_len;
    // The winners lie in the candidate array as sorted runs, one per segment.  The selection
    // kernel gives a thread four neighbouring elements out of every 4096, so with runs of a length
    // that divides 4096 a thread would hold the same ranks of every run - a few threads all the
    // heads - and the bound it takes from samples of the threads' maxima would let thousands
    // through ([1, 2^24], limit 256: 250 us; limit 257: 68 us).  An even limit therefore keeps one
    // winner more per segment: runs of odd length, which shift from one group of 4096 to the next.
    p.keep = (limit % 2 == 0 && limit < kMaxLimit) ? limit + 1 : limit;
    if (p.segs < 2 || p.last_n < p.keep || p.segs * p.keep > n / 2 || m * p.segs > 0x7fffffffLL) return p;
    const size_t cands = static_cast<size_t>(m) * p.segs * p.keep;
    p.val_off = 0;
    p.idx_off = align_up(cands * elem_size, 256);
    p.pos_off = p.idx_off + align_up(cands * 4, 256);
    p.rest_off = p.pos_off + align_up(static_cast<size_t>(m) * limit * 4, 256);
    const size_t first = select_layout(key_size, m * p.segs, p.seg_len).total;
    const size_t second = top_k_scratch_impl(dtype, m, p.segs * p.keep, limit);
    p.total = p.rest_off + (first > second ? first : second);
    p.ok = true;
    return p;
}

__global__ __launch_bounds__(256) void topk_places_to_indices(const int32_t* __restrict__ place, const uint32_t* __restrict__ cand_idx,
                                                              int64_t rows, int limit, int64_t keep, int64_t segs, int64_t seg_len,
                                                              void* idx, DimMap imap, int64_t si, int idx64) {
    const int64_t g = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (g >= rows * limit) return;
    const int64_t row = g / limit;
    const int j = static_cast<int>(g - row * limit);
    const int64_t p = place[g];                        // among the row's segs * keep candidates
    const int64_t ix = (p / keep) * seg_len + cand_idx[row * segs * keep + p];
    const int64_t at = imap.at(row) + j * si;
    if (idx64) static_cast<int64_t*>(idx)[at] = ix;
    else static_cast<int32_t*>(idx)[at] = static_cast<int32_t>(ix);
}

template <typename T>
int run_top_k(hipStream_t stream, int64_t limit, int dir, int dtype, int index_dtype,
              int rank, const int64_t* x_dims, const int64_t* y_dims,
              const void* x, const int64_t* xs, void* y, const int64_t* ys, void* idx, const int64_t* is,
              void* scratch, size_t scratch_bytes) {
    using K = typename BitsOf<T>::type;
    using S = typename BitsOf<T>::storage;
    const int64_t n = x_dims[rank - 1];
    const int64_t m = view_size(rank, x_dims) / n;
    TopkIo<K, S> io;
    std::memset(&io, 0, sizeof(io));
    io.x = static_cast<const S*>(x);
    io.y = static_cast<S*>(y);
    io.idx = idx;
    if (!make_dim_map(x_dims, xs, 0, rank - 1, &io.xmap) || !make_dim_map(y_dims, ys, 0, rank - 1, &io.ymap) ||
        !make_dim_map(y_dims, is, 0, rank - 1, &io.imap))
        return DLFX_ERR_RANK;
    io.sx = xs[rank - 1];
    io.sy = ys[rank - 1];
    io.si = is[rank - 1];
    io.idx64 = index_dtype == DLFX_I64;
    io.kind = BitsOf<T>::kind;
    io.largest = dir ? 1 : 0;
    if (m > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;

    // rows side by side in memory, small limit: one thread per row (and segment of the axis)
    // (limits of 9 to 16 only on rows of up to 256 elements: beyond, a wave per row with neighbouring rows on one XCD is faster)
    if (limit <= kColsLimit && (limit <= 8 || n <= 256) && io.sx != 1 && io.sx != -1 && m >= 16384 && n <= 0x7fffffffLL && io.xmap.rank >= 1 &&
        io.xmap.strides[io.xmap.rank - 1] == 1 && io.xmap.dims[io.xmap.rank - 1] >= kWave) {
        const int lim = static_cast<int>(limit);
        const int64_t blocks = ceil_div(m, static_cast<int64_t>(kWave));
        // wavefronts that share a block of 64 rows, each with a piece of the axis (measured on fp32, axes of 64 to
        // 2048 positions, 500 to 16400 blocks: eight while the blocks are few - and for limits of one or two, whose
        // lists are cheap to merge, up to 5000 blocks -, four beyond; one only for axes too short to cut)
        int seg = n < 64 ? 1 : blocks < (lim <= 2 ? 5000 : 1024) ? 8 : 4;
        if (g_topk_cols_waves) seg = g_topk_cols_waves;
        const dim3 cgrid(static_cast<unsigned>(ceil_div(blocks, 8) * 8));
#define DLFX_TOPK_COLS(KMAX)                                                                        \
    do {                                                                                            \
        if (seg == 1) topk_cols<T, KMAX, 1><<<cgrid, dim3(kWave), 0, stream>>>(io, m, n, lim);      \
        else if (seg == 4) topk_cols<T, KMAX, 4><<<cgrid, dim3(kWave * 4), 0, stream>>>(io, m, n, lim); \
        else topk_cols<T, KMAX, 8><<<cgrid, dim3(kWave * 8), 0, stream>>>(io, m, n, lim);           \
    } while (0)
        if (lim <= 1) DLFX_TOPK_COLS(1);
        else if (lim <= 2) DLFX_TOPK_COLS(2);
        else if (lim <= 3) DLFX_TOPK_COLS(3);
        else if (lim <= 4) DLFX_TOPK_COLS(4);
        else if (lim <= 5) DLFX_TOPK_COLS(5);
        else if (lim <= 6) DLFX_TOPK_COLS(6);
        else if (lim <= 8) DLFX_TOPK_COLS(8);
        else if (lim <= 12) DLFX_TOPK_COLS(12);
        else DLFX_TOPK_COLS(16);
#undef DLFX_TOPK_COLS
        DLFX_CHECK_LAUNCH();
        return DLFX_OK;
    }

    // short rows side by side in memory, a limit beyond the register lists: LDS tiles of 64 rows
    if (n <= kWave && m >= 4096 && io.sx != 1 && io.sx != -1 && io.xmap.rank >= 1 && io.xmap.strides[io.xmap.rank - 1] == 1 &&
        io.xmap.dims[io.xmap.rank - 1] >= kWave) {
        topk_cols_wave<T><<<dim3(static_cast<unsigned>(ceil_div(m, static_cast<int64_t>(kWave)))), dim3(256), 0, stream>>>(
            io, m, n, static_cast<int>(limit));
        DLFX_CHECK_LAUNCH();
        return DLFX_OK;
    }

    // many short rows one after the other in memory, small limit: one thread per row
    if (limit <= kThreadRowLimit && io.sx == 1 && io.xmap.rank <= 1 && m >= 16384 &&
        n <= (sizeof(K) == 4 ? g_topk_thread_rows : g_topk_thread_rows / 2)) {
        const int lim = static_cast<int>(limit);
        const int64_t pitch = io.xmap.rank ? io.xmap.strides[0] : 0;
        const int64_t blocks = ceil_div(m, static_cast<int64_t>(4 * kWave));
        const dim3 rgrid(static_cast<unsigned>(blocks));
        const bool one_run = n < kThreadRowChunk && pitch == n;
#define DLFX_TOPK_THREAD(KMAX)                                                                      \
    do {                                                                                            \
        if (one_run) topk_rows_thread<T, KMAX, true><<<rgrid, dim3(256), 0, stream>>>(io, m, n, lim, pitch);  \
        else topk_rows_thread<T, KMAX, false><<<rgrid, dim3(256), 0, stream>>>(io, m, n, lim, pitch);         \
    } while (0)
        if (lim <= 1) DLFX_TOPK_THREAD(1);
        else if (lim <= 2) DLFX_TOPK_THREAD(2);
        else if (lim <= 3) DLFX_TOPK_THREAD(3);
        else if (lim <= 4) DLFX_TOPK_THREAD(4);
        else if (lim <= 5) DLFX_TOPK_THREAD(5);
        else if (lim <= 6) DLFX_TOPK_THREAD(6);
        else DLFX_TOPK_THREAD(8);
#undef DLFX_TOPK_THREAD
        DLFX_CHECK_LAUNCH();
        return DLFX_OK;
    }

    if (selection_fits(sizeof(K), n, limit)) return launch_select<T>(stream, io, m, n, limit, scratch, scratch_bytes);

    // rows too long for the selection kernel: select within segments, then among their winners
    const LongPlan lp = long_plan(dtype, sizeof(S), sizeof(K), m, n, limit);
    if (lp.ok && io.xmap.rank < kMaxRank) {
        if (!scratch || scratch_bytes < lp.total) return DLFX_ERR_SCRATCH_TOO_SMALL;
        const int lim = static_cast<int>(limit);
        char* base = static_cast<char*>(scratch);
        S* cand_val = reinterpret_cast<S*>(base + lp.val_off);
        uint32_t* cand_idx = reinterpret_cast<uint32_t*>(base + lp.idx_off);
        int32_t* place = reinterpret_cast<int32_t*>(base + lp.pos_off);
        TopkIo<K, S> io1 = io;
        io1.xmap.dims[io1.xmap.rank] = lp.segs;                    // innermost: row r of the launch is segment r % segs
        io1.xmap.strides[io1.xmap.rank] = lp.seg_len * io.sx;
        io1.xmap.rank += 1;
        io1.y = cand_val;
        io1.idx = cand_idx;
        io1.ymap.rank = io1.imap.rank = 1;
        io1.ymap.dims[0] = io1.imap.dims[0] = m * lp.segs;
        io1.ymap.strides[0] = io1.imap.strides[0] = lp.keep;
        io1.sy = io1.si = 1;
        io1.idx64 = 0;
        io1.segs = lp.segs;
        io1.last_n = lp.last_n;
        int st = launch_select<T>(stream, io1, m * lp.segs, lp.seg_len, lp.keep, base + lp.rest_off, scratch_bytes - lp.rest_off);
        if (st != DLFX_OK) return st;
        int64_t c_dims[64], c_strides[64], p_strides[64];
        for (int i = 0; i < rank; ++i) c_dims[i] = x_dims[i];
        c_dims[rank - 1] = lp.segs * lp.keep;
        int64_t cs = 1, ps = 1;
        for (int i = rank - 1; i >= 0; --i) {
            c_strides[i] = cs;
            cs *= c_dims[i];
            p_strides[i] = ps;
            ps *= y_dims[i];
        }
        st = run_top_k<T>(stream, limit, dir, dtype, DLFX_I32, rank, c_dims, y_dims, cand_val, c_strides, y, ys, place, p_strides,
                          base + lp.rest_off, scratch_bytes - lp.rest_off);
        if (st != DLFX_OK) return st;
        const int64_t outs = m * limit;
        topk_places_to_indices<<<dim3(static_cast<unsigned>(ceil_div(outs, 256))), dim3(256), 0, stream>>>(
            place, cand_idx, m, lim, lp.keep, lp.segs, lp.seg_len, idx, io.imap, io.si, io.idx64);
        DLFX_CHECK_LAUNCH();
        return DLFX_OK;
    }

    // full stable argsort into scratch, then keep the head of each row
    const size_t ysz = align_up(static_cast<size_t>(m) * n * sizeof(S), 256);
    const size_t isz = align_up(static_cast<size_t>(m) * n * 4, 256);
    const size_t need = ysz + isz + argsort_scratch_bytes_impl(dtype, m, n);
    if (!scratch || scratch_bytes < need) return DLFX_ERR_SCRATCH_TOO_SMALL;
    char* base = static_cast<char*>(scratch);
    S* ysorted = reinterpret_cast<S*>(base);
    int32_t* isorted = reinterpret_cast<int32_t*>(base + ysz);
    int st = argsort_contiguous(stream, dir ? 1 : 0, dtype, rank, x_dims, x, xs, ysorted, isorted,
                                base + ysz + isz, scratch_bytes - ysz - isz);
    if (st != DLFX_OK) return st;
    const int64_t total = m * limit;
    if (ceil_div(total, 256) > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
    topk_take<K, S><<<dim3(static_cast<unsigned>(ceil_div(total, 256))), dim3(256), 0, stream>>>(ysorted, isorted, m, n, limit, io);
    DLFX_CHECK_LAUNCH();
    return DLFX_OK;
}

}  // namespace

#if DLFX_TOPK_PART == 0
bool set_topk_tuning(const char* key, int64_t value) {
    if (!std::strcmp(key, "topk_cols_waves") && (value == 0 || value == 1 || value == 4 || value == 8)) {
        g_topk_cols_waves = static_cast<int>(value);
        return true;
    }
    if (!std::strcmp(key, "topk_thread_rows") && value >= 0 && value <= 65536) {
        g_topk_thread_rows = static_cast<int>(value);
        return true;
    }
    return false;
}
#endif

// the other widths' translation units
#define DLFX_TOPK_ARGS                                                                                              \
    hipStream_t s, int64_t limit, int dir, int dtype, int index_dtype, int rank, const int64_t *x_dims,             \
        const int64_t *y_dims, const void *xp, const int64_t *x_strides, void *yp, const int64_t *y_strides, void *ip, \
        const int64_t *i_strides, void *scratch, size_t scratch_bytes
#define DLFX_TOPK_PASS s, limit, dir, dtype, index_dtype, rank, x_dims, y_dims, xp, x_strides, yp, y_strides, ip, i_strides, scratch, scratch_bytes
int top_k_wide(DLFX_TOPK_ARGS);
int top_k_narrow(DLFX_TOPK_ARGS);
#if DLFX_TOPK_PART == 1
int top_k_wide(DLFX_TOPK_ARGS) {
    return dtype == DLFX_F64 ? run_top_k<double>(DLFX_TOPK_PASS) : run_top_k<int64_t>(DLFX_TOPK_PASS);
}
#elif DLFX_TOPK_PART == 2
int top_k_narrow(DLFX_TOPK_ARGS) {
    return dtype == DLFX_F16 ? run_top_k<half_t>(DLFX_TOPK_PASS) : run_top_k<int16_t>(DLFX_TOPK_PASS);
}
#endif
}  // namespace dlfx

using namespace dlfx;

#if defined(DLFX_TOPK_TIMING) && DLFX_TOPK_PART == 0
extern "C" void dlfx_debug_topk_phases(unsigned long long* out, int reset) {
    static unsigned long long host[dlfx::kPhaseSlots * 8];
    if (out) {
        (void)hipMemcpyFromSymbol(host, HIP_SYMBOL(dlfx::g_topk_cycles), sizeof(host));
        for (int i = 0; i < 8; ++i) out[i] = 0;
        for (int b = 0; b < dlfx::kPhaseSlots; ++b)
            for (int i = 0; i < 8; ++i) out[i] += host[b * 8 + i];
    }
    if (reset) {
        std::memset(host, 0, sizeof(host));
        (void)hipMemcpyToSymbol(HIP_SYMBOL(dlfx::g_topk_cycles), host, sizeof(host));
    }
}
#endif

namespace dlfx {
namespace {
size_t top_k_scratch_impl(int dtype, int64_t m, int64_t n, int64_t limit) {
    const size_t es = dtype_size(dtype);
    if (!es || dtype == DLFX_BOOL || m <= 0 || n <= 0) return 0;
    const size_t ks = es < 4 ? 4 : es;            // 16-bit elements are selected as 32-bit keys
    if (selection_fits(ks, n, limit)) return select_layout(ks, m, n).total;
    const LongPlan lp = long_plan(dtype, es, ks, m, n, limit);
    if (lp.ok) return lp.total;
    return align_up(static_cast<size_t>(m) * n * es, 256) + align_up(static_cast<size_t>(m) * n * 4, 256) +
           argsort_scratch_bytes_impl(dtype, m, n);
}
}  // namespace
}  // namespace dlfx

#if DLFX_TOPK_PART == 0
extern "C" size_t dlfx_top_k_scratch_bytes(int dtype, int64_t m, int64_t n, int64_t limit) {
    return top_k_scratch_impl(dtype, m, n, limit);
}

extern "C" int dlfx_top_k(dlfx_stream_t stream, int64_t limit, int dir, int dtype, int index_dtype,
                          int rank, const int64_t* x_dims, const int64_t* y_dims,
                          const void* x, int64_t x_offset, const int64_t* x_strides,
                          void* y, int64_t y_offset, const int64_t* y_strides,
                          void* idx, int64_t i_offset, const int64_t* i_strides,
                          void* scratch, size_t scratch_bytes) {
    if (!x || !y || !idx || rank < 1) return DLFX_ERR_INVALID_ARGUMENT;
    if (!view_ok(rank, x_dims, x_strides) || !view_ok(rank, y_dims, y_strides) || !view_ok(rank, y_dims, i_strides))
        return DLFX_ERR_INVALID_ARGUMENT;
    for (int i = 0; i + 1 < rank; ++i)
        if (x_dims[i] != y_dims[i]) return DLFX_ERR_INVALID_ARGUMENT;
    if (limit < 1 || limit > x_dims[rank - 1] || y_dims[rank - 1] != limit) return DLFX_ERR_INVALID_ARGUMENT;
    if (index_dtype != DLFX_I32 && index_dtype != DLFX_I64) return DLFX_ERR_UNSUPPORTED_DTYPE;
    if (x_dims[rank - 1] > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
    const size_t es = dtype_size(dtype);
    if (!es) return DLFX_ERR_UNSUPPORTED_DTYPE;
    const void* xp = static_cast<const char*>(x) + x_offset * static_cast<int64_t>(es);
    void* yp = static_cast<char*>(y) + y_offset * static_cast<int64_t>(es);
    void* ip = static_cast<char*>(idx) + i_offset * (index_dtype == DLFX_I64 ? 8 : 4);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (dtype) {
    case DLFX_F32: return run_top_k<float>(DLFX_TOPK_PASS);
    case DLFX_I32: return run_top_k<int32_t>(DLFX_TOPK_PASS);
    case DLFX_F64:
    case DLFX_I64: return top_k_wide(DLFX_TOPK_PASS);
    case DLFX_F16:
    case DLFX_I16: return top_k_narrow(DLFX_TOPK_PASS);
    default: return DLFX_ERR_UNSUPPORTED_DTYPE;
    }
}
#endif
