// The bucket route of sort / argsort for rows longer than one workgroup holds (gfx950).
//
// A row is cut by value into at most 256 buckets of at most 5120 keys (rows of up to 131072 keys:
// 2560; rows longer than 1.1 M keys: 10240), and every bucket is then sorted on chip, so the keys cross HBM four times (plus one read
// for the histogram) however wide they are:
//   1. split_sample     1024 keys of every row, from 256 evenly spaced places, give the range of
//                       its keys (a few stray keys at either end left aside); 4096 "fine bins"
//                       resolve that range, keys outside it share the first or the last bin.
//   2. split_histogram  one read of the input: a fine-bin histogram of every chunk of 32768 keys
//                       (LDS atomics).
//   3. split_plan       per row: the chunks' histograms add up to the row's; neighbouring fine
//                       bins are merged into buckets of equal depth (bucket of a bin = keys
//                       before it / target, and a new bucket after a long run of empty bins), so
//                       skewed rows - floats with their exponents, clustered integers - still
//                       give even buckets.  Every chunk's histogram becomes the place of its keys
//                       inside each bucket, and the buckets of all rows are listed for the last
//                       step.  A row with a fine bin fuller than a workgroup holds gets buckets
//                       larger than that - each such bin one to itself where the bucket
//                       numbers allow (decided here, on the device, row by row; below).
//   4. split_pass       one workgroup per chunk: a tile of 4096 keys finds each key's bucket
//                       (table in LDS) and its slot among the tile's keys of that bucket with one
//                       LDS atomic, lays the tile out by bucket in LDS and writes it as runs to
//                       where split_plan said the chunk's keys of each bucket go: workgroups
//                       exchange nothing.  The order inside a run is whatever the atomics gave:
//                       not stable, and it need not be.
//   5. split_finish     resident workgroups take buckets from the list: the keys' offsets from
//                       the bucket minimum, scaled to 8192 (4096) bins, are counted and placed
//                       with LDS atomics; what shares a bin (about one other key) is ranked by
//                       comparing whole (key, index) entries, which also restores the stable
//                       order of equal keys; the bucket leaves for the strided outputs.
//   6. split_finish_crowded  buckets with a bin too crowded for that (many equal or clustered
//                       keys) take the stable digit passes of sort_in_workgroup instead, for
//                       pairs first by index, then by key.
// Rows that evenly spaced fine bins do not cut:
//   * one value repeated more often than a workgroup holds makes a bucket larger than that.  The
//     row is then moved by split_pass_stable (ranks in element order instead of atomics), which
//     writes the entries of such buckets straight to the outputs: a bucket of one value arrives
//     sorted, in index order, and is done.
//   * distinct keys packed more tightly than the bins resolve: split_sample sees them in its
//     sample and marks the row, split_remap gives it a map made from the quantiles of a larger
//     sample (PiecewiseMap), and steps 2 to 6 run as for any row, the stable pass moving it.
//   * what is left - an oversized bucket of several values that the sample did not show - is
//     sorted by the one workgroup of split_finish_crowded that draws it: stable digit passes over
//     the digits that vary in it, window by window, between the scratch buffer and the bucket's
//     place in the outputs.
// Ranking with an LDS atomic costs a few instructions per key where wave-wide digit matching
// costs about fifty per digit, which is what bounds the digit passes.
#include <cstddef>
#include <cstring>

#include "sort_common.hip.h"

namespace dlfx {
namespace {

#ifdef SPLIT_TIMING
// Debug builds only: shader-clock cycles spent by thread 0 of every workgroup in each phase.
constexpr int kPhaseSlots = 4096;
__device__ unsigned long long g_split_cycles[kPhaseSlots * 16];
#define SPLIT_PHASE(i) do { if (threadIdx.x == 0) { const long long now_ = clock64(); g_split_cycles[(blockIdx.x % kPhaseSlots) * 16 + (i)] += static_cast<unsigned long long>(now_ - phase_t_); phase_t_ = now_; } } while (0)
#define SPLIT_PHASE_BEGIN() long long phase_t_ = clock64()
#else
#define SPLIT_PHASE(i) do { } while (0)
#define SPLIT_PHASE_BEGIN() do { } while (0)
#endif

constexpr int kFineBits = 12;
constexpr int kFine = 1 << kFineBits;                 // fine bins per row
constexpr int kMaxBuckets = 256;
constexpr int kSplitBlock = 256;
constexpr int kSplitItems = 16;                       // keys per thread of a split_pass tile
constexpr int kSplitTile = kSplitBlock * kSplitItems;
constexpr int kChunk = 8 * kSplitTile;                // keys one split_pass workgroup takes (32768)
// Threads of a split_pass workgroup (16 keys each make its tile): 256, 512 or 1024.  A tile leaves
// as one run per bucket, so its keys spread over the row's buckets decide how long the runs
// are; short runs (128 bytes for 8-byte keys in 256 buckets) cost write bandwidth, larger tiles
// cost LDS and occupancy.  Measured on [256, 2^20] int64: 1476 / 1235 / 1044 us (keys),
// 2197 / 1698 / 1540 us (pairs; at 1024 threads the indices pass through LDS after the keys); on
// [1024, 65536] fp32 (32 buckets): 118 / 118 / 157 us (keys), 193 / 178 / 203 us (pairs).
template <typename K, bool PAIRS>
constexpr int kPassBlockMax = sizeof(K) == 8 ? 1024 : 512;
template <typename K, bool PAIRS>
int pass_block(int64_t n, int cap) {
    const int64_t buckets = ceil_div(n * 5, static_cast<int64_t>(cap) * 4);       // buckets fill to about 4/5
    int block = 256;
    const int64_t run_bytes = 1024;                        // what a tile should write per bucket at least
    while (block < kPassBlockMax<K, PAIRS> && static_cast<int64_t>(block) * kSplitItems * static_cast<int64_t>(sizeof(K)) < run_bytes * buckets) block *= 2;
    return block;
}
// split_finish comes in three sizes: four wavefronts for buckets of up to 2560 keys (rows of up
// to 131072 keys: more, smaller workgroups on a compute unit hide each other's waits better),
// eight for buckets of up to 5120 (rows of up to 1.1 M keys), sixteen for buckets of up to 10240
// (rows of up to about 2.4 M keys; measured at 2^20 int64 keys: the scatter pass gains from the
// longer runs, 1049 -> 973 us, but the finish loses more, 1413 -> 1577 us, so the size is kept
// for rows the eight-wavefront size cannot take).
constexpr int kFinishItems = 10;
constexpr int finish_cap(int waves) { return waves * kWave * kFinishItems; }      // keys a bucket may hold
constexpr int finish_bins(int waves) { return waves * 1024; }                     // counting bins, two 16-bit counters a word
constexpr int kCapHuge = finish_cap(16);
constexpr int64_t kSmallCapRows = 131072;             // longest row that takes the small size
constexpr int64_t kLargeCapRows = 1100000;            // longest row that takes the eight-wavefront size
constexpr int64_t kLargeCapFloatRows = 700000;        // ... of floats, which seldom fill their fine bins as evenly as integers do
// Wavefronts of the finishing workgroup for rows of n keys, and what a bucket may hold then.
inline int finish_waves(int64_t n, bool floats) {
    return n <= kSmallCapRows ? 4 : n <= (floats ? kLargeCapFloatRows : kLargeCapRows) ? 8 : 16;
}
constexpr int kNear = 2;                              // entries of a bin compared without a loop
constexpr int64_t kFrontRows = 512;                   // fewest rows of a call that split_front takes (two a compute unit)
// A bucket larger than a workgroup holds is listed once per window of this many entries, so that
// a bucket of one repeated value (a constant row is one bucket) is copied out by many workgroups.
constexpr uint32_t kOverWindow = 32768;
constexpr uint32_t kNoWindow = 0xffffffffu;           // an entry of the list that is a whole (crowded) bucket
// What split_finish_crowded walks: {bucket id = row * 256 + b, window} entries, and the OR and
// the AND of the keys of every oversized bucket (split_plan sets them to zero and all ones,
// split_pass_stable gathers them): equal means one repeated value.
struct CrowdedList {
    uint2* items;
    unsigned long long* range;             // [2 id]: OR of the bucket's keys, [2 id + 1]: AND
};

// A row whose keys cluster more tightly than evenly spaced fine bins resolve gets a map made from
// the quantiles of a sample instead: the sorted sample's every 16th key bounds a segment, 256 of
// them, and a segment has 16 fine bins - the first for the bounding key itself (a value repeated
// so often that it bounds segments gets a bin, and then a bucket, to itself), the others spread
// evenly over the keys up to the next bound.
constexpr int kSegments = 256;
constexpr int kSegmentBins = kFine / kSegments;
constexpr int kQuantileSample = kSegments * 16;       // keys sampled for the bounds
struct alignas(16) PiecewiseMap {
    unsigned long long bound[kSegments];   // bound[0] = 0: every key has a segment
    uint8_t shift[kSegments];              // bin of a key above its bound: 1 + min((key - bound - 1) >> shift, 14)
};

// What split_sample and split_plan decide for a row.
struct alignas(16) SplitRow {
    uint32_t route;                        // 1: this row takes the bucket route, 0: the digit passes
    uint32_t shift;                        // by key image: fine bin = min((key - base) >> shift, kFine - 1), 0 below base
    unsigned long long base;               // keys below share the first fine bin (both ways)
    uint32_t n_buckets;
    uint32_t by_value;                     // 1 (floats only): fine bin = (value - lo) * scale between base and top
    unsigned long long top;                // by value: keys from here up share the last fine bin
    unsigned long long lo_bits, scale_bits;    // by value: lo and scale as a float's / double's bits
    unsigned long long gap_lo, gap_hi;     // by key image, floats: keys in [gap_lo, gap_hi) count as gap_lo and the keys above move down by
                                           // the width of the gap (none: both all ones)
    uint32_t piecewise, unused[3];         // 1: none of the above - the row's PiecewiseMap says where a key goes
    uint32_t begin[kMaxBuckets + 4];       // first position of each bucket in the row; begin[n_buckets] = n
    uint8_t bucket_of[kFine];              // fine bin -> bucket (16-byte aligned: tiles load it as vectors)
};
static_assert(offsetof(SplitRow, bucket_of) % 16 == 0 && sizeof(SplitRow) % 16 == 0, "vector loads of the table");

template <typename K> struct FloatOf;
template <> struct FloatOf<uint32_t> { using type = float; };
template <> struct FloatOf<uint64_t> { using type = double; };

// The fine bin of a key, monotone in the key whatever the key: keys outside the sampled range
// land in the first or last bins, so nothing has to be verified afterwards - a poor sample costs
// balance, not order.  Two ways to spread the range over the bins: evenly over the key images
// (integers; floats whose magnitudes spread over many binades - an image is about the
// logarithm of its float), or evenly over the values (floats that spread evenly as numbers:
// uniform or bell-shaped data, data on both sides of zero, where most images would crowd into
// the few bins of the largest binades).  split_sample picks per row.  By key image, a float row
// with values on both sides of zero would spend most bins on the images between its smallest
// negative and positive magnitudes, where it has next to no keys: split_sample finds that gap
// and the map closes it up.
template <typename K>
struct FineMap {
    using F = typename FloatOf<K>::type;
    K base, top, gap_lo, gap_hi, less;     // less: -(gap_hi + base), what the image with the gap taken out is short of
    F lo, scale;
    uint32_t shift, by_value, piecewise;
    int descending;
    const K* bound = nullptr;              // piecewise: the map's bounds and shifts (in LDS)
    const uint8_t* bound_shift = nullptr;
    template <typename Row>                // a SplitRow, or the FineRange that goes into one
    __device__ FineMap(const Row& r, int desc)
        : base(static_cast<K>(r.base)), top(static_cast<K>(r.top)), gap_lo(static_cast<K>(r.gap_lo)), gap_hi(static_cast<K>(r.gap_hi)),
          less(static_cast<K>(K(0) - static_cast<K>(r.gap_hi) - static_cast<K>(r.base))),
          lo(bit_cast<F>(static_cast<K>(r.lo_bits))), scale(bit_cast<F>(static_cast<K>(r.scale_bits))), shift(r.shift),
          by_value(r.by_value), piecewise(r.piecewise), descending(desc) {}
    // by the row's PiecewiseMap: the last segment whose bound is not above the key, then the bin inside it
    __device__ __forceinline__ uint32_t bin_piecewise(K key) const {
        uint32_t j = 0;
#pragma unroll
        for (int step = kSegments / 2; step > 0; step >>= 1) j += bound[j + step] <= key ? static_cast<uint32_t>(step) : 0u;
        const K above = static_cast<K>(key - bound[j]);
        const K sub = static_cast<K>(static_cast<K>(above - 1) >> bound_shift[j]);
        return j * kSegmentBins + (above == 0 ? 0u : 1u + (sub < K(kSegmentBins - 2) ? static_cast<uint32_t>(sub) : static_cast<uint32_t>(kSegmentBins - 2)));
    }
    // MODE: 0 by key image, 1 by value, 2 piecewise (what the row's record says; the kernels branch once per workgroup)
    template <int MODE, bool GAP>
    __device__ __forceinline__ uint32_t bin_as(K key) const {
        if constexpr (MODE == 2) return bin_piecewise(key);
        else return bin<MODE == 1, GAP>(key);
    }
    // the number a float key stands for, increasing with the key (so negated for descending sorts)
    __device__ __forceinline__ static F value_of(K key, int desc) {
        const F x = bit_cast<F>(decode_key<K>(key, kKeyFloat, desc));
        return desc ? -x : x;
    }
    // BY_VALUE must equal by_value: the kernels branch once per workgroup, not once per key.
    // GAP: the row may have a gap (the host knows which rows can) - otherwise no code for it.
    // With the gap taken out, the image of a key is min(key, gap_lo) + max(key, gap_hi) - gap_hi:
    // monotone, the key itself below the gap (where base lies) and when there is no gap.
    template <bool BY_VALUE, bool GAP>
    __device__ __forceinline__ uint32_t bin(K key) const {
        uint32_t f;
        if constexpr (BY_VALUE) {
            // between base and top the value is finite; subtraction, scaling and truncation are
            // all monotone, so the bin never decreases as the key grows
            const F t = (value_of(key, descending) - lo) * scale;
            int b = static_cast<int>(t);
            b = b < 0 ? 0 : b;
            f = b < kFine - 1 ? static_cast<uint32_t>(b) : static_cast<uint32_t>(kFine - 1);
            f = key >= top ? static_cast<uint32_t>(kFine - 1) : f;
        } else if constexpr (GAP) {
            // base lies below the gap: a key held between base and gap_lo, plus one held above
            // gap_hi, less gap_hi and base, is the image's distance from base - no test for keys
            // under base, and as many operations as without a gap
            const K below = clamp_between(key, base, gap_lo), above = key > gap_hi ? key : gap_hi;
            const K off = static_cast<K>(below + above + less) >> shift;
            return off < static_cast<K>(kFine - 1) ? static_cast<uint32_t>(off) : static_cast<uint32_t>(kFine - 1);
        } else {
            const K off = static_cast<K>(key - base) >> shift;
            f = off < static_cast<K>(kFine - 1) ? static_cast<uint32_t>(off) : static_cast<uint32_t>(kFine - 1);
        }
        return key < base ? 0u : f;
    }
    // min(max(x, lo), hi) for lo <= hi: one instruction for 32-bit keys (the compiler cannot know that lo <= hi)
    __device__ __forceinline__ static K clamp_between(K x, K lo, K hi) {
        if constexpr (sizeof(K) == 4) {
            uint32_t r;
            asm("v_med3_u32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "s"(lo), "v"(hi));      // (one scalar operand an instruction)
            return r;
        } else {
            const K up = x > lo ? x : lo;
            return up < hi ? up : hi;
        }
    }
    __device__ __forceinline__ uint32_t operator()(K key) const { return by_value ? bin<true, true>(key) : bin<false, true>(key); }
};

template <typename T, typename Join>
__device__ __forceinline__ T block_reduce(T v, Join join, T* lds, int waves) {
    v = wave_reduce(v, join);
    __syncthreads();                                   // the previous use of `lds` is over
    if (lane_id() == 0) lds[threadIdx.x / kWave] = v;
    __syncthreads();
    T r = lds[0];
    for (int i = 1; i < waves; ++i) r = join(r, lds[i]);
    return r;
}

// The fourth smallest (SMALLEST) or fourth largest of the 256 keys a wavefront holds, four a
// lane: the best is found and one instance of it struck out, three times over, and the best of
// what is left is the answer (a full sort of the 256 keys cost three times as much).
template <bool SMALLEST, typename K>
__device__ __forceinline__ K wave_fourth(const K (&key)[4]) {
    constexpr K out = SMALLEST ? ~K(0) : K(0);         // a struck-out entry: never better than a key
    auto better = [](K a, K b) { return SMALLEST ? (a < b ? a : b) : (a > b ? a : b); };
    K left[4] = {key[0], key[1], key[2], key[3]};
    K best = out;
#pragma unroll
    for (int round = 0; round < 4; ++round) {
        const K mine = better(better(left[0], left[1]), better(left[2], left[3]));
        best = wave_reduce(mine, better);
        if (round == 3) break;
        const unsigned long long holders = __ballot(mine == best);
        if (lane_id() == __ffsll(static_cast<long long>(holders)) - 1) {     // the first lane that holds it strikes one out
            bool struck = false;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const bool hit = !struck && left[u] == best;
                left[u] = hit ? out : left[u];
                struck = struck || hit;
            }
        }
    }
    return best;
}

// ------------------------------------------------------------------ 1. the range of a row's keys
// MAP (the host knows): 0 for rows spread by key image and nothing else (integers, short float
// rows); 1 for float rows of middling length, whose images may have the gap around zero closed
// up; 2 for longer float rows, by key image as they are or by value.  The kernels carry no code for what their
// MAP leaves out.
constexpr int kMapPlain = 0, kMapGap = 1, kMapValue = 2, kMapAny = 3, kMapPiecewise = 4;      // (any: what the row's record says, as the kernel runs)

// How a row's keys spread over its fine bins (the part of SplitRow that split_sample decides).
struct FineRange {
    uint32_t shift, by_value, piecewise;
    unsigned long long base, top, lo_bits, scale_bits, gap_lo, gap_hi;
    __device__ __forceinline__ void store(SplitRow& out) const {
        out.piecewise = piecewise;
        out.shift = shift;
        out.base = base;
        out.by_value = by_value;
        out.gap_lo = gap_lo;
        out.gap_hi = gap_hi;
        out.top = top;
        out.lo_bits = lo_bits;
        out.scale_bits = scale_bits;
    }
};

// The sample of row `xrow` and what it says, worked out by a workgroup of BLOCK threads (every
// thread returns the same answer).  The sample is that of 256 threads whatever BLOCK is: further
// wavefronts repeat the first four, which changes no minimum or maximum, and the lists of what
// every wavefront offers are those of the first four.
//
// The sample also shows whether the row's keys cluster more tightly than the chosen map resolves:
// a fine bin that holds so many of the sample's keys that it promises more than a bucket may
// hold, and keys that differ among them (one value repeated is no trouble: its bucket is done
// when it has been moved).  Such a row is marked `piecewise`.  sample_hist: kFine words of LDS,
// zero on entry and on return.
template <typename K, int MAP, int BLOCK>
__device__ __forceinline__ FineRange sample_row(const PassIo<K>& io, const K* __restrict__ xrow, int64_t n, uint32_t cap, uint32_t* __restrict__ sample_hist) {
    static_assert(BLOCK % kSplitBlock == 0 && (MAP != kMapValue || BLOCK == kSplitBlock), "whole repeats of the sampling threads");
    __shared__ K red[BLOCK / kWave];
    const int st = threadIdx.x % kSplitBlock;          // the sampling thread this one is (or repeats)
    // 1024 keys: four neighbours (one memory line when the row is contiguous) at each of 256
    // evenly spaced places, the last of them the row's last keys, so that a sorted row shows
    // its whole range
    K key[4];
    int64_t e0 = (static_cast<int64_t>(st) * n) / kSplitBlock;
    if (st == kSplitBlock - 1 || e0 > n - 4) e0 = n - 4;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int64_t j = static_cast<int64_t>(st) * 4 + u;
        const int64_t e = n >= 1024 ? e0 + u : (j < n ? j : n - 1);
        key[u] = key_of_element<K>(io, xrow[e * io.sx]);
    }
    // every wave offers the 4th smallest and the 4th largest of its 256 keys: three stray keys
    // per wave at either end (a few zeros among positive values, a few huge ones) do not stretch
    // the range the fine bins resolve
    auto smaller = [](K a, K b) { return a < b ? a : b; };
    auto larger = [](K a, K b) { return a > b ? a : b; };
    K lo, hi;
    if (n < 64) {                                      // too few keys for that: the plain range
        lo = wave_reduce(smaller(smaller(key[0], key[1]), smaller(key[2], key[3])), smaller);
        hi = wave_reduce(larger(larger(key[0], key[1]), larger(key[2], key[3])), larger);
    } else {
        lo = wave_fourth<true>(key);
        hi = wave_fourth<false>(key);
    }
    lo = block_reduce(lo, smaller, red, BLOCK / kWave);
    hi = block_reduce(hi, larger, red, BLOCK / kWave);
    // Float rows: the images of negative and of positive values lie either side of the middle
    // of the key range, those of the smallest magnitudes next to it and the two zeros at it.
    // Every wave offers the nearest of its keys below the zeros and the nearest above them; the
    // second nearest of the four on each side bound the gap (one stray tiny value a side does not
    // count, and zeros never do).  Keys inside it - zeros, a few tiny values - share a fine bin.
    K gap_lo = ~K(0), gap_hi = ~K(0);
    if constexpr (MAP == kMapGap) {
        constexpr K zero_hi = K(1) << (8 * sizeof(K) - 1), zero_lo = zero_hi - 1;      // keys of +0.0 and -0.0 (either way round)
        K under_mine = K(0), over_mine = ~K(0);        // this lane's nearest key below the zeros, and above them
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (key[u] < zero_lo) under_mine = larger(under_mine, key[u]);
            if (key[u] > zero_hi) over_mine = smaller(over_mine, key[u]);
        }
        __shared__ K near[2][kSplitBlock / kWave];
        const K wave_under = wave_reduce(under_mine, larger), wave_over = wave_reduce(over_mine, smaller);
        if (lane_id() == 0 && threadIdx.x < kSplitBlock) {
            near[0][threadIdx.x / kWave] = wave_under;
            near[1][threadIdx.x / kWave] = wave_over;
        }
        __syncthreads();
        K under[2] = {K(0), K(0)}, over[2] = {~K(0), ~K(0)};       // nearest and second nearest
        for (int w = 0; w < kSplitBlock / kWave; ++w) {
            const K a = near[0][w], b = near[1][w];
            if (a > under[0]) { under[1] = under[0]; under[0] = a; } else if (a > under[1]) under[1] = a;
            if (b < over[0]) { over[1] = over[0]; over[0] = b; } else if (b < over[1]) over[1] = b;
        }
        const K nearest_under = under[1], nearest_over = over[1];
        // worth closing when it lies inside the range and is at least half of it (a bit of bin width or more)
        if (n >= 1024 && nearest_under != K(0) && nearest_under >= lo && nearest_over <= hi &&
            static_cast<K>(nearest_over - nearest_under) >= static_cast<K>(static_cast<K>(hi - lo) / 2)) {
            gap_lo = nearest_under;
            gap_hi = nearest_over;
        }
    }
    // that range takes the middle half of the fine bins; a quarter on either side is left for
    // keys outside it (beyond those, keys share the first or last bin)
    FineRange map;
    {
        map.gap_lo = static_cast<unsigned long long>(gap_lo);
        map.gap_hi = static_cast<unsigned long long>(gap_hi);
        const K gap = static_cast<K>(gap_hi - gap_lo);         // lo is below the gap, hi above it
        const unsigned long long range = static_cast<unsigned long long>(static_cast<K>(hi - lo - gap));
        const int width = range ? 64 - __builtin_clzll(range) : 0;
        map.shift = width > kFineBits - 1 ? static_cast<uint32_t>(width - (kFineBits - 1)) : 0u;
        const K margin = static_cast<K>(K(kFine / 4) << map.shift);
        map.base = static_cast<unsigned long long>(lo > margin ? static_cast<K>(lo - margin) : K(0));
        map.by_value = 0u;
        map.top = 0ull;
        map.lo_bits = map.scale_bits = 0ull;
    }
    if constexpr (MAP == kMapValue) {
        // the same range spread evenly over the values instead - taken when, by key image, the
        // sample's fullest cell of 16 bins promises a fine bin of more than a quarter of what a
        // bucket holds (the row might not fit the route, or only in lopsided buckets) and the
        // values crowd their fullest cell less; otherwise the cheaper image arithmetic stays
        using F = typename FloatOf<K>::type;
        const F xl = FineMap<K>::value_of(lo, io.descending), xh = FineMap<K>::value_of(hi, io.descending);
        const F w = xh - xl;
        const F first = xl - w * F(0.5), last = xh + w * F(0.5);
        if (w > F(0) && w - w == F(0) && first - first == F(0) && last - last == F(0)) {       // all finite
            FineRange by_value = map;
            by_value.by_value = 1u;
            by_value.lo_bits = static_cast<unsigned long long>(bit_cast<K>(first));
            by_value.scale_bits = static_cast<unsigned long long>(bit_cast<K>(static_cast<F>(kFine) / (w * F(2))));
            // the keys of `first` and `last` (the element value is the negated one when descending)
            by_value.base = static_cast<unsigned long long>(key_of_element<K>(io, bit_cast<K>(io.descending ? -first : first)));
            by_value.top = static_cast<unsigned long long>(key_of_element<K>(io, bit_cast<K>(io.descending ? -last : last)));
            static_assert(kFine / 16 == kSplitBlock, "a thread per cell");
            __shared__ uint32_t cells[2][kFine / 16];
            for (int i = threadIdx.x; i < 2 * (kFine / 16); i += kSplitBlock) (&cells[0][0])[i] = 0u;
            __syncthreads();
            const FineMap<K> by_image_map(map, io.descending), by_value_map(by_value, io.descending);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                atomicAdd(&cells[0][by_image_map(key[u]) >> 4], 1u);
                atomicAdd(&cells[1][by_value_map(key[u]) >> 4], 1u);
            }
            __syncthreads();
            uint32_t worst_image = cells[0][threadIdx.x], worst_value = cells[1][threadIdx.x];      // kFine / 16 == kSplitBlock
            __shared__ uint32_t red32[kSplitBlock / kWave];
            worst_image = block_reduce(worst_image, [](uint32_t a, uint32_t b) { return a > b ? a : b; }, red32, kSplitBlock / kWave);
            worst_value = block_reduce(worst_value, [](uint32_t a, uint32_t b) { return a > b ? a : b; }, red32, kSplitBlock / kWave);
            if (worst_value < worst_image && static_cast<unsigned long long>(worst_image) * static_cast<unsigned long long>(n) > static_cast<unsigned long long>(cap) * kFine) map = by_value;
        }
    }
    map.piecewise = 0u;
    if (n > static_cast<int64_t>(cap)) {
        const FineMap<K> chosen(map, io.descending);
        const bool sampler = threadIdx.x < kSplitBlock;    // (further threads repeat these keys)
        uint32_t f[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            f[u] = chosen(key[u]);
            if (sampler) atomicAdd(&sample_hist[f[u]], 1u);
        }
        __syncthreads();
        // (what a full bucket's worth of keys shows in the sample, and four standard deviations of
        // that count more - twice that at most; eight at least, which evenly spread keys never reach by chance)
        const float full = static_cast<float>(cap) * 1024.0f / static_cast<float>(n);
        const float margin = 4.0f * sqrtf(full) + 1.0f;
        const uint32_t by_size = static_cast<uint32_t>(full + (margin < full ? margin : full)) + 1u;
        const uint32_t many = by_size > 8u ? by_size : 8u;
        bool crowded[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) crowded[u] = sampler && sample_hist[f[u]] >= many;
        __syncthreads();
        // every crowded bin's word now takes one of the bin's keys (folded to 32 bits), whichever lands last ...
        auto folded = [](K k) { return static_cast<uint32_t>(k) ^ static_cast<uint32_t>(static_cast<unsigned long long>(k) >> 32); };
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (crowded[u]) sample_hist[f[u]] = folded(key[u]);
        __syncthreads();
        // ... and a key of the bin that differs from it says that the bin holds more than one value
        bool mixed = false;
#pragma unroll
        for (int u = 0; u < 4; ++u) mixed = mixed || (crowded[u] && sample_hist[f[u]] != folded(key[u]));
        map.piecewise = __syncthreads_or(mixed ? 1 : 0) ? 1u : 0u;
        if (sampler) {
#pragma unroll
            for (int u = 0; u < 4; ++u) sample_hist[f[u]] = 0u;
        }
        __syncthreads();
    }
    return map;
}

template <typename K, int MAP>
__global__ __launch_bounds__(kSplitBlock) void split_sample(PassIo<K> io, int64_t n, uint32_t cap, SplitRow* __restrict__ rows, uint32_t* __restrict__ counters) {
    __shared__ uint32_t sample_hist[kFine];
    const int64_t row = blockIdx.x;
    if (row == 0 && threadIdx.x < 4) counters[threadIdx.x] = 0u;      // what the later launches of this sort count up from
    for (int i = threadIdx.x; i < kFine; i += kSplitBlock) sample_hist[i] = 0u;
    const FineRange map = sample_row<K, MAP, kSplitBlock>(io, io.x + io.xmap.at(row), n, cap, sample_hist);
    if (threadIdx.x == 0) {
        rows[row].route = 0u;
        map.store(rows[row]);
        // counters[4]: not zero when some row of the call has a piecewise map.  split_plan leaves
        // it zero for the next sort; whatever else it may hold at first (new scratch memory)
        // only makes split_remap look at every row's record once.
        if (map.piecewise != 0u) atomicOr(&counters[4], 1u);
    }
}

// ------------------------------------------------------------------ 2. fine-bin histograms
// One workgroup per chunk of kChunk keys of a row: the chunk's fine-bin histogram, two 16-bit
// counts a word (a count is at most kChunk).  split_plan adds the chunks up for the row's
// histogram and turns each chunk's into its keys per bucket, so that split_pass needs no
// communication between workgroups.
// Elements [lo, hi) of a row counted into hist[kFine] (LDS, which the caller has cleared) by a
// workgroup of BLOCK threads.  STREAM: the elements are not read again soon (non-temporal loads).
template <typename K, int MAP, int BLOCK, bool STREAM>
__device__ __forceinline__ void count_fine_bins(const PassIo<K>& io, const K* __restrict__ xrow, int64_t lo, int64_t hi,
                                                const FineMap<K>& fine_of, uint32_t* __restrict__ hist) {
    constexpr int U = 32 / sizeof(K);                 // keys per thread and batch (64 bytes measured: no faster)
    // batches of BLOCK x U keys; the next batch's keys are on their way while this one is counted
    // (no branches in the loads: a key beyond the range's end reads its first key and is never counted)
    constexpr int64_t BATCH = static_cast<int64_t>(BLOCK) * U;
    // (whole batches of a contiguous, aligned row move as 16-byte accesses: which thread counts
    // which key does not matter here)
    constexpr int VK = 16 / sizeof(K);
    using VecK = Vec<K, VK>;
    const bool vectors = io.sx == 1 && reinterpret_cast<uintptr_t>(xrow + lo) % 16 == 0;
    auto load_batch = [&](int64_t b0, K (&key)[U]) __attribute__((always_inline)) {
        if (vectors && b0 + BATCH <= hi) {
            const VecK* src = reinterpret_cast<const VecK*>(xrow + b0);
#pragma unroll
            for (int v = 0; v < U / VK; ++v) {
                VecK a;
                if constexpr (STREAM) a = load_stream(&src[threadIdx.x + v * BLOCK]);      // (non-temporal: 71 -> 50 us on [1024, 65536] fp32)
                else a = src[threadIdx.x + v * BLOCK];
#pragma unroll
                for (int e = 0; e < VK; ++e) key[v * VK + e] = a.v[e];
            }
            return;
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t i = b0 + threadIdx.x + static_cast<int64_t>(u) * BLOCK;
            key[u] = xrow[(i < hi ? i : lo) * io.sx];
        }
    };
    auto count_chunk = [&](auto mode_tag) __attribute__((always_inline)) {
    constexpr int MODE = decltype(mode_tag)::value;
    constexpr bool GAP = MAP == kMapGap;               // (a branch per workgroup on whether the row has a gap: more registers, slower)
    K key[U];
    load_batch(lo, key);
    for (int64_t b0 = lo; b0 < hi; b0 += BATCH) {
        K ahead[U];
        if (b0 + BATCH < hi) load_batch(b0 + BATCH, ahead);
        const bool full = b0 + BATCH <= hi;
        uint32_t f[U];
#pragma unroll
        for (int u = 0; u < U; ++u) f[u] = fine_of.template bin_as<MODE, GAP>(key_of_element<K>(io, key[u]));
        // a wave whose keys all share one fine bin (narrow ranges, few distinct values) adds once
        const uint32_t f0 = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(f[0])));
        bool same = full;
#pragma unroll
        for (int u = 0; u < U; ++u) same = same && f[u] == f0;
        if (__ballot(!same) == 0ull) {
            if (lane_id() == 0) atomicAdd(&hist[f0], static_cast<uint32_t>(U * kWave));
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (full || b0 + threadIdx.x + static_cast<int64_t>(u) * BLOCK < hi) atomicAdd(&hist[f[u]], 1u);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) key[u] = ahead[u];
    }
    };
    if constexpr (MAP == kMapPiecewise) count_chunk(std::integral_constant<int, 2>());
    else if (MAP == kMapValue && fine_of.by_value) count_chunk(std::integral_constant<int, MAP == kMapValue ? 1 : 0>());
    else count_chunk(std::integral_constant<int, 0>());
}

template <typename K, int MAP>
__global__ __launch_bounds__(kSplitBlock) void split_histogram(PassIo<K> io, int64_t n, int64_t chunks_per_row,
                                                               const SplitRow* __restrict__ rows, uint32_t* __restrict__ chunk_fine,
                                                               const PiecewiseMap* __restrict__ maps) {
    __shared__ uint32_t hist[kFine];
    for (int i = threadIdx.x; i < kFine; i += kSplitBlock) hist[i] = 0;
    __syncthreads();
    const int64_t row = blockIdx.x / chunks_per_row;
    const int64_t c = blockIdx.x - row * chunks_per_row;
    const K* xrow = io.x + io.xmap.at(row);
    FineMap<K> fine_of(rows[row], io.descending);
    const int64_t lo = c * kChunk;
    const int64_t hi = (lo + kChunk < n) ? lo + kChunk : n;
    if (fine_of.piecewise != 0u) {                     // (seldom) by the map split_remap made for the row
        __shared__ K bound[kSegments];
        __shared__ uint8_t bound_shift[kSegments];
        static_assert(kSplitBlock == kSegments, "a thread a segment");
        bound[threadIdx.x] = static_cast<K>(maps[row].bound[threadIdx.x]);
        bound_shift[threadIdx.x] = maps[row].shift[threadIdx.x];
        __syncthreads();
        fine_of.bound = bound;
        fine_of.bound_shift = bound_shift;
        count_fine_bins<K, kMapPiecewise, kSplitBlock, true>(io, xrow, lo, hi, fine_of, hist);
    } else {
        count_fine_bins<K, MAP, kSplitBlock, true>(io, xrow, lo, hi, fine_of, hist);
    }
    __syncthreads();
    uint32_t* g = chunk_fine + static_cast<int64_t>(blockIdx.x) * (kFine / 2);
    for (int i = threadIdx.x; i < kFine / 2; i += kSplitBlock) g[i] = hist[2 * i] | (hist[2 * i + 1] << 16);
}

// ------------------------------------------------------------------ 3. buckets of equal depth
// One workgroup per row; thread t owns fine bins [16 t, 16 t + 16).  For every row,
// chunk_base[chunk][b] receives the row position where that chunk's keys of bucket b go: the
// bucket's start plus what the row's earlier chunks hold of it.  Buckets that a workgroup of
// split_finish holds are appended to bucket_list (counters[2] entries); a row with a fine bin
// fuller than that (one value repeated many times, keys clustered more tightly than the fine
// bins resolve) has buckets that are larger: those go on the list split_finish_crowded walks
// (counters[1] entries) and the row is marked route 2, which for pairs makes split_pass_stable
// move it, so that every bucket of the row arrives in index order.
template <int BLOCK>
struct PlanShared {
    uint32_t red[BLOCK / kWave];
    uint32_t listed[2][kSplitBlock / kWave + 1];      // buckets of this row for either list by wavefront, and where they go
    uint32_t last_count[kSplitBlock];                 // every planning thread's last fine bin
    uint32_t last_bucket[kSplitBlock];
    uint32_t begin[kMaxBuckets + 1];
};

// What packing a row's fine bins into buckets one by one needs (plan_buckets, when its formula
// asks for more buckets than there are).
struct PackShared {
    uint32_t prefix[kFine + 1];                        // keys before every fine bin
    uint16_t next[kFine];                              // the bin after the fullest bucket that starts at a bin
    uint16_t start[kMaxBuckets + 2];                   // first bin of every bucket
    uint32_t buckets;
};

// The buckets of row `row` from its fine-bin counts: planning thread t (the first 256 threads of
// a workgroup of BLOCK) brings the counts of fine bins [16 t, 16 t + 16) in cnt[] and receives
// their buckets in bucket[]; the other threads bring zeros and only keep the barriers company.
// The row's record, its table and its buckets' places (also sm.begin) are written, the buckets
// listed.  Returns the number of buckets.
template <int BLOCK>
__device__ __forceinline__ uint32_t plan_buckets(PlanShared<BLOCK>& sm, const uint32_t (&cnt)[kFine / kSplitBlock], uint32_t (&bucket)[kFine / kSplitBlock],
                                                 int64_t n, uint32_t cap, int64_t row, SplitRow& info, uint32_t* __restrict__ counters,
                                                 uint4* __restrict__ bucket_list, CrowdedList crowded, uint32_t* route_out = nullptr, bool piecewise = false,
                                                 PackShared* pack = nullptr) {
    constexpr int PER = kFine / kSplitBlock;          // 16
    constexpr int WAVES = BLOCK / kWave;
    const int w = threadIdx.x / kWave;
    const bool planner = threadIdx.x < kSplitBlock;
    uint32_t sum = 0, biggest = 0;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        sum += cnt[i];
        biggest = cnt[i] > biggest ? cnt[i] : biggest;
    }
    if (planner) sm.last_count[threadIdx.x] = cnt[PER - 1];
    biggest = block_reduce(biggest, [](uint32_t a, uint32_t b) { return a > b ? a : b; }, sm.red, WAVES);
    // exclusive prefix of the thread sums
    const uint32_t incl = wave_scan_inclusive(sum, 0u, [](uint32_t a, uint32_t b) { return a + b; });
    __syncthreads();
    if (lane_id() == kWave - 1) sm.red[w] = incl;
    __syncthreads();
    uint32_t before = incl - sum;
    for (int i = 0; i < w; ++i) before += sm.red[i];

    // A bin goes to bucket (keys before it) / target plus the cuts at or before it: bit i of
    // `cut_at` makes bin i of this thread open a new bucket whatever the count says.  Returns
    // the number of buckets.
    auto assign = [&](uint32_t target, uint32_t cut_at) __attribute__((always_inline)) -> uint32_t {
        const uint32_t cuts = static_cast<uint32_t>(__popc(cut_at));
        const uint32_t cuts_incl = wave_scan_inclusive(cuts, 0u, [](uint32_t a, uint32_t b) { return a + b; });
        __syncthreads();
        if (lane_id() == kWave - 1) sm.red[w] = cuts_incl;
        __syncthreads();
        uint32_t extra = cuts_incl - cuts;
        for (int i = 0; i < w; ++i) extra += sm.red[i];
        uint32_t run = before;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            extra += (cut_at >> i) & 1u;
            bucket[i] = run / target + extra;
            run += cnt[i];
        }
        if (planner) sm.last_bucket[threadIdx.x] = bucket[PER - 1];
        __syncthreads();
        return sm.last_bucket[kSplitBlock - 1] + 1;
    };

    // Where at least kGapBins empty bins lie between two populated ones a new bucket starts
    // whatever the counts say: stray keys far from the rest (a few zeros below positive values)
    // then do not stretch the range of the bucket next to them, which split_finish resolves with
    // a fixed number of counting bins.
    constexpr int kGapBins = 64;
    uint32_t gap_cuts = 0;
    {
        int last = -1;                                 // last populated bin of this thread
#pragma unroll
        for (int i = 0; i < PER; ++i)
            if (cnt[i]) last = static_cast<int>(threadIdx.x) * PER + i;
        int seen = wave_scan_inclusive(last, -1, [](int a, int b) { return a > b ? a : b; });
        __syncthreads();
        if (lane_id() == kWave - 1) sm.red[w] = static_cast<uint32_t>(seen);
        __syncthreads();
        int prev = __shfl_up(seen, 1, kWave);          // last populated bin before this thread's first
        if (lane_id() == 0) prev = -1;
        for (int i = 0; i < w; ++i) prev = static_cast<int>(sm.red[i]) > prev ? static_cast<int>(sm.red[i]) : prev;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int bin = static_cast<int>(threadIdx.x) * PER + i;
            if (cnt[i]) {
                if (prev >= 0 && bin - prev > kGapBins) gap_cuts |= 1u << i;
                prev = bin;
            }
        }
    }

    // Every fine bin leaves room in a bucket: buckets of (keys before) / (cap - largest bin) hold
    // fewer than cap keys each.
    // (a row with a piecewise map is moved by split_pass_stable whatever its buckets: the plain pass carries no code for that map)
    uint32_t route = piecewise ? 2u : 1u, n_buckets = kMaxBuckets + 1;
    if (biggest < cap) {
        n_buckets = assign(cap - biggest, gap_cuts);
        if (n_buckets > static_cast<uint32_t>(kMaxBuckets)) n_buckets = assign(cap - biggest, 0u);
    }
    if (n_buckets > static_cast<uint32_t>(kMaxBuckets) && biggest < cap && pack != nullptr) {
        // Too many buckets that way (a long row: the formula leaves room for the row's largest bin
        // in every bucket): the bins are packed one bucket after the other instead, each bucket
        // taking bins while they fit.  Every bin finds where the fullest bucket that starts
        // with it ends (bisection over the prefix sums); one thread then walks from bucket to
        // bucket - 256 dependent steps at most, on this path only.
        if (planner) {
            uint32_t run = before;
#pragma unroll
            for (int i = 0; i < PER; ++i) {
                pack->prefix[threadIdx.x * PER + i] = run;
                run += cnt[i];
            }
            if (threadIdx.x == kSplitBlock - 1) pack->prefix[kFine] = run;
        }
        __syncthreads();
        if (planner) {
#pragma unroll 1
            for (int i = 0; i < PER; ++i) {
                const int bin = static_cast<int>(threadIdx.x) * PER + i;
                const uint32_t most = pack->prefix[bin] + cap;
                int lo = bin + 1, hi = kFine;                          // the answer lies in [lo, hi]: every bin alone fits
                while (lo < hi) {
                    const int mid = (lo + hi + 1) >> 1;
                    if (pack->prefix[mid] <= most) lo = mid;
                    else hi = mid - 1;
                }
                pack->next[bin] = static_cast<uint16_t>(lo);
            }
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            uint32_t b = 0;
            int pos = 0;
            while (pos < kFine && b <= static_cast<uint32_t>(kMaxBuckets)) {
                pack->start[b++] = static_cast<uint16_t>(pos);
                pos = pack->next[pos];
            }
            pack->start[b < static_cast<uint32_t>(kMaxBuckets) + 1u ? b : static_cast<uint32_t>(kMaxBuckets) + 1u] = static_cast<uint16_t>(kFine);
            pack->buckets = pos < kFine ? static_cast<uint32_t>(kMaxBuckets) + 1u : b;
        }
        __syncthreads();
        const uint32_t packed = pack->buckets;
        if (packed <= static_cast<uint32_t>(kMaxBuckets)) {
            if (planner) {
                const int first_bin = static_cast<int>(threadIdx.x) * PER;
                uint32_t lo = 0, hi = packed - 1u;                     // the bucket of this thread's first bin
                while (lo < hi) {
                    const uint32_t mid = (lo + hi + 1u) >> 1;
                    if (static_cast<int>(pack->start[mid]) <= first_bin) lo = mid;
                    else hi = mid - 1u;
                }
#pragma unroll
                for (int i = 0; i < PER; ++i) {
                    while (lo + 1u < packed && first_bin + i >= static_cast<int>(pack->start[lo + 1u])) ++lo;
                    bucket[i] = lo;
                }
                sm.last_bucket[threadIdx.x] = bucket[PER - 1];
            }
            __syncthreads();
            n_buckets = packed;
        }
    }
    if (n_buckets > static_cast<uint32_t>(kMaxBuckets)) {
        // Some fine bin does not (or too many buckets would be needed): the row gets buckets of
        // cap * 3/4 keys plus a bin of less than cap / 4 - or of n / 224 keys when that is more,
        // which 256 buckets always hold - and every fuller bin a bucket to itself while the
        // bucket numbers allow it; a bucket larger than cap is finished by split_finish_crowded
        // (a bucket of one value costs next to nothing there).
        route = 2u;
        const uint32_t heavy = cap / 4;
        uint32_t heavy_cuts = 0;
        uint32_t prev = (planner && threadIdx.x != 0) ? sm.last_count[threadIdx.x - 1] : 0u;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            if (cnt[i] >= heavy || prev >= heavy) heavy_cuts |= 1u << i;
            prev = cnt[i];
        }
        if (!planner) heavy_cuts = 0u;
        const uint32_t by_count = static_cast<uint32_t>((n + 223) / 224);
        const uint32_t target = cap - heavy > by_count ? cap - heavy : by_count;
        n_buckets = assign(target, heavy_cuts);
        if (n_buckets > static_cast<uint32_t>(kMaxBuckets)) n_buckets = assign(target, 0u);      // at most 224
    }
    // a bin opens every bucket after its predecessor's up to its own (the starts are put together
    // in LDS: the threads read one another's just below)
    if (planner) {
        uint32_t prev_bucket = threadIdx.x == 0 ? 0u : sm.last_bucket[threadIdx.x - 1];
        if (threadIdx.x == 0) sm.begin[0] = 0u;
        uint32_t run = before;
        uint32_t packed[PER / 4];                     // this thread's 16 table bytes: one store
#pragma unroll
        for (int i = 0; i < PER / 4; ++i) packed[i] = 0u;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            packed[i / 4] |= bucket[i] << (8 * (i % 4));
            for (uint32_t k = prev_bucket + 1; k <= bucket[i]; ++k) sm.begin[k] = run;
            prev_bucket = bucket[i];
            run += cnt[i];
        }
        static_assert(PER == 16 && offsetof(SplitRow, bucket_of) % 16 == 0, "a thread's bins are one aligned 16-byte piece of the table");
        reinterpret_cast<uint4*>(info.bucket_of)[threadIdx.x] = make_uint4(packed[0], packed[1], packed[2], packed[3]);
    }
    if (route_out) *route_out = route;
    if (threadIdx.x == kSplitBlock - 1) {
        info.n_buckets = n_buckets;
        sm.begin[n_buckets] = static_cast<uint32_t>(n);
        info.route = route;
        if (route == 2u) atomicAdd(&counters[3], 1u);      // split_pass_stable has something to do
    }
    __syncthreads();
    for (uint32_t k = threadIdx.x; k <= n_buckets; k += BLOCK) info.begin[k] = sm.begin[k];
    // The buckets that hold anything, in no particular order, on the list of the kernel that
    // finishes them: split_finish those that fit its workgroup, split_finish_crowded the others.
    {
        uint32_t b0 = 0, size = 0;
        if (threadIdx.x < n_buckets) {
            b0 = sm.begin[threadIdx.x];
            size = sm.begin[threadIdx.x + 1] - b0;
        }
        const bool fits_finish = size != 0u && size <= cap;
        const uint32_t windows = size > cap ? (size + kOverWindow - 1) / kOverWindow : 0u;      // list entries of an oversized bucket
        const unsigned long long fit_lanes = __ballot(fits_finish);
        const uint32_t windows_incl = wave_scan_inclusive(windows, 0u, [](uint32_t a, uint32_t b) { return a + b; });
        if (planner) {
            if (lane_id() == 0) sm.listed[0][w] = static_cast<uint32_t>(__popcll(fit_lanes));
            if (lane_id() == kWave - 1) sm.listed[1][w] = windows_incl;
        }
        __syncthreads();
        if (threadIdx.x < 2) {
            uint32_t total = 0;
            for (int i = 0; i < kSplitBlock / kWave; ++i) {
                const uint32_t c = sm.listed[threadIdx.x][i];
                sm.listed[threadIdx.x][i] = total;
                total += c;
            }
            sm.listed[threadIdx.x][kSplitBlock / kWave] = total ? atomicAdd(&counters[threadIdx.x == 0 ? 2 : 1], total) : 0u;
        }
        __syncthreads();
        const unsigned long long below = (1ull << lane_id()) - 1ull;
        const uint32_t id = static_cast<uint32_t>(row) * kMaxBuckets + threadIdx.x;
        if (fits_finish)
            bucket_list[sm.listed[0][kSplitBlock / kWave] + sm.listed[0][w] + static_cast<uint32_t>(__popcll(fit_lanes & below))] = make_uint4(static_cast<uint32_t>(row), b0, size, id);
        if (windows != 0u) {
            uint2* at = crowded.items + sm.listed[1][kSplitBlock / kWave] + sm.listed[1][w] + (windows_incl - windows);
            for (uint32_t i = 0; i < windows; ++i) at[i] = make_uint2(id, i);
            crowded.range[2 * id] = 0ull;
            crowded.range[2 * id + 1] = ~0ull;
        }
    }
    return n_buckets;
}

// The plan of row `row` from its chunks' fine-bin histograms, by a workgroup of BLOCK threads:
// groups of 256 threads take the chunks in turn (thread t of a group owns fine bins [16 t,
// 16 t + 16) of its chunks), each with the histograms of eight chunks in flight - what bounds the
// plan of a long row is the latency of these loads (they miss the L2: other compute units'
// workgroups wrote them), not their number.  per_chunk: chunks_per_row x 256 words of LDS.
constexpr int kPlanChunks = 8;
template <int BLOCK>
__device__ __forceinline__ void plan_row(PlanShared<BLOCK>& sm, PackShared& pack, uint32_t* __restrict__ row_hist, uint32_t* __restrict__ per_chunk, int64_t row, int64_t n,
                                         uint32_t cap, int64_t chunks_per_row,
                                         const uint32_t* __restrict__ chunk_fine, SplitRow* __restrict__ rows, uint32_t* __restrict__ counters,
                                         uint4* __restrict__ bucket_list, CrowdedList crowded, uint32_t* __restrict__ chunk_base, bool piecewise) {
    constexpr int PER = kFine / kSplitBlock;          // 16
    constexpr int GROUPS = BLOCK / kSplitBlock;
    const int group = threadIdx.x / kSplitBlock, t = threadIdx.x % kSplitBlock;
    const uint32_t* f = chunk_fine + row * chunks_per_row * (kFine / 2) + t * (PER / 2);
    auto chunk_words = [&](int64_t c, uint32_t (&w)[PER / 2]) __attribute__((always_inline)) {
        const uint4 a = reinterpret_cast<const uint4*>(f + c * (kFine / 2))[0], b = reinterpret_cast<const uint4*>(f + c * (kFine / 2))[1];
        w[0] = a.x; w[1] = a.y; w[2] = a.z; w[3] = a.w; w[4] = b.x; w[5] = b.y; w[6] = b.z; w[7] = b.w;
    };
    // ---- the row's histogram: every group adds up its chunks, the groups add up in LDS
    uint32_t cnt[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) cnt[i] = 0;
    if constexpr (GROUPS > 1) {
        for (int i = threadIdx.x; i < kFine; i += BLOCK) row_hist[i] = 0u;
    }
    for (int64_t i = threadIdx.x; i < chunks_per_row * kMaxBuckets; i += BLOCK) per_chunk[i] = 0u;
    for (int64_t c0 = group; c0 < chunks_per_row; c0 += kPlanChunks * GROUPS) {
        uint32_t w[kPlanChunks][PER / 2];
#pragma unroll
        for (int j = 0; j < kPlanChunks; ++j)
            if (c0 + j * GROUPS < chunks_per_row) chunk_words(c0 + j * GROUPS, w[j]);
#pragma unroll
        for (int j = 0; j < kPlanChunks; ++j) {
            if (c0 + j * GROUPS >= chunks_per_row) break;
#pragma unroll
            for (int i = 0; i < PER / 2; ++i) {
                cnt[2 * i] += w[j][i] & 0xffffu;
                cnt[2 * i + 1] += w[j][i] >> 16;
            }
        }
    }
    if constexpr (GROUPS > 1) {
        __syncthreads();
#pragma unroll
        for (int i = 0; i < PER; ++i)
            if (cnt[i]) atomicAdd(&row_hist[t * PER + i], cnt[i]);
        __syncthreads();
#pragma unroll
        for (int i = 0; i < PER; ++i) cnt[i] = group == 0 ? row_hist[t * PER + i] : 0u;
        __syncthreads();                               // row_hist is free: the planners' buckets go there next
    }
    uint32_t bucket[PER];
    const uint32_t n_buckets = plan_buckets<BLOCK>(sm, cnt, bucket, n, cap, row, rows[row], counters, bucket_list, crowded, nullptr, piecewise, &pack);
    if constexpr (GROUPS > 1) {
        // every group needs the buckets of its threads' bins
        if (group == 0) {
#pragma unroll
            for (int i = 0; i < PER; ++i) row_hist[t * PER + i] = bucket[i];
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < PER; ++i) bucket[i] = row_hist[t * PER + i];
    }
    // ---- each chunk's keys per bucket.  A thread's 16 bins lie in two buckets at most as a rule -
    // the bins up to the first change of bucket (left_bins) and the rest: two sums and two LDS
    // atomics a chunk.
    uint32_t left_bins = (1u << PER) - 1u;
    int changes = 0;
#pragma unroll
    for (int i = 0; i + 1 < PER; ++i) {
        if (bucket[i + 1] != bucket[i]) {
            if (changes == 0) left_bins = (2u << i) - 1u;
            ++changes;
        }
    }
    const bool two_at_most = changes <= 1;
    for (int64_t c0 = group; c0 < chunks_per_row; c0 += kPlanChunks * GROUPS) {
        uint32_t w[kPlanChunks][PER / 2];
#pragma unroll
        for (int j = 0; j < kPlanChunks; ++j)
            if (c0 + j * GROUPS < chunks_per_row) chunk_words(c0 + j * GROUPS, w[j]);
#pragma unroll
        for (int j = 0; j < kPlanChunks; ++j) {
            const int64_t c = c0 + j * GROUPS;
            if (c >= chunks_per_row) break;
            uint32_t* into = per_chunk + c * kMaxBuckets;
            if (two_at_most) {
                uint32_t total = 0, left = 0;
#pragma unroll
                for (int i = 0; i < PER; ++i) {
                    const uint32_t count = (i & 1) ? (w[j][i / 2] >> 16) : (w[j][i / 2] & 0xffffu);
                    total += count;
                    left += ((left_bins >> i) & 1u) ? count : 0u;
                }
                if (left) atomicAdd(&into[bucket[0]], left);
                if (total != left) atomicAdd(&into[bucket[PER - 1]], total - left);
            } else {
                uint32_t acc = 0;
#pragma unroll
                for (int i = 0; i < PER; ++i) {
                    acc += (i & 1) ? (w[j][i / 2] >> 16) : (w[j][i / 2] & 0xffffu);
                    if (i == PER - 1 || bucket[i + 1] != bucket[i]) {
                        if (acc) atomicAdd(&into[bucket[i]], acc);
                        acc = 0;
                    }
                }
            }
        }
    }
    __syncthreads();
    // ---- and from them where every chunk writes each bucket: thread b carries bucket b through the chunks
    if (threadIdx.x < kMaxBuckets) {
        uint32_t next = threadIdx.x < n_buckets ? sm.begin[threadIdx.x] : 0u;
        for (int64_t c = 0; c < chunks_per_row; ++c) {
            chunk_base[(row * chunks_per_row + c) * kMaxBuckets + threadIdx.x] = next;
            next += per_chunk[c * kMaxBuckets + threadIdx.x];
        }
    }
}

// (BLOCK: 256 for rows of up to eight chunks - all their histograms are in flight at once anyway - and 1024 beyond)
template <int BLOCK>
__global__ __launch_bounds__(BLOCK) void split_plan(int64_t n, uint32_t cap, int64_t chunks_per_row, const uint32_t* __restrict__ chunk_fine,
                                                    SplitRow* __restrict__ rows, uint32_t* __restrict__ counters,
                                                    uint4* __restrict__ bucket_list, CrowdedList crowded,
                                                    uint32_t* __restrict__ chunk_base) {
    __shared__ PlanShared<BLOCK> sm;
    __shared__ PackShared pack;
    __shared__ uint32_t row_hist[BLOCK > kSplitBlock ? kFine : 1];
    extern __shared__ uint32_t per_chunk[];            // chunks_per_row x 256 words
    const int64_t row = blockIdx.x;
    if (row == 0 && threadIdx.x == 0) counters[4] = 0u;       // split_remap has read it: zero again for the next sort that uses this memory
    plan_row<BLOCK>(sm, pack, row_hist, per_chunk, row, n, cap, chunks_per_row, chunk_fine, rows, counters, bucket_list, crowded, chunk_base, rows[row].piecewise != 0u);
}

// ------------------------------------------------------------------ 3b. rows whose keys cluster
// The rows split_sample marked `piecewise` (as a rule none: counters[4] is then zero and every
// workgroup leaves at once).  split_remap, a workgroup per such row: a sample of 4096 of the
// row's keys sorted on chip, and the row's PiecewiseMap from it; split_histogram and split_plan
// then treat the row like any other, by that map.  Where split_front stands for those launches
// (it leaves such a row alone), split_replan does the whole of it instead: a workgroup makes the
// row's map, counts the row into the map's fine bins and plans it.
template <typename K>
struct RemapShared {
    SmallShared<K, false, kQuantileSample / kSplitBlock, kSplitBlock / kWave> sorter;
    K bound[kSegments + 1];                            // [kSegments]: the sample's largest key
    uint8_t bound_shift[kSegments];
};

// The PiecewiseMap of a row into sm.bound / sm.bound_shift, by a workgroup of kSplitBlock threads
// (no barrier after the last writes).
template <typename K>
__device__ __forceinline__ void piecewise_map_of(RemapShared<K>& sm, const PassIo<K>& io, const K* __restrict__ xrow, int64_t n) {
    constexpr int ITEMS = kQuantileSample / kSplitBlock;      // 16
    static_assert(kQuantileSample / kSegments == 16 && kSplitBlock == kSegments, "every 16th key of the sorted sample bounds a segment; a thread a segment");
    const int tid = threadIdx.x;
    const int seg = (tid / kWave) * kWave * ITEMS + lane_id();
    // ---- the sample, sorted: one key from each of 4096 equal stretches of the row, at a place
    // inside the stretch that changes from stretch to stretch (a row that repeats with some period
    // shows all its phases)
    K key[ITEMS];
    uint32_t none[1] = {0u};
    K ors = 0, ands = ~K(0);
    const int64_t stretch = n / kQuantileSample;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const uint32_t p = static_cast<uint32_t>(seg + k * kWave);
        int64_t e = (static_cast<int64_t>(p) * n) / kQuantileSample;
        if (stretch > 1) e += static_cast<int64_t>((p * 2654435761u) >> 8) % stretch;
        key[k] = key_of_element<K>(io, xrow[e * io.sx]);
        ors |= key[k];
        ands &= key[k];
    }
    sort_in_workgroup<K, false, ITEMS, kSplitBlock / kWave>(sm.sorter, key, none, ors, ands, kQuantileSample, KeyTraits<K>::kPasses);
    // ---- bounds: key k of this thread is the sorted sample's entry seg + 64 k
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const int at = seg + k * kWave;
        if (at % 16 == 0) sm.bound[at / 16] = at == 0 ? K(0) : key[k];
        if (at == kQuantileSample - 1) sm.bound[kSegments] = key[k];
    }
    __syncthreads();
    // the keys above a bound, up to the next one, share 15 bins: 1 + ((key - bound - 1) >> shift), at most 15
    const K lo = sm.bound[tid], hi = sm.bound[tid + 1];
    uint32_t shift = 0;
    if (hi > lo) {
        const unsigned long long widest = static_cast<unsigned long long>(static_cast<K>(hi - lo - 1));
        const int bits = widest ? 64 - __builtin_clzll(widest) : 0;
        shift = bits > 4 ? static_cast<uint32_t>(bits - 4) : 0u;
    }
    sm.bound_shift[tid] = static_cast<uint8_t>(shift);
}

template <typename K>
__global__ __launch_bounds__(kSplitBlock) void split_remap(PassIo<K> io, int64_t m, int64_t n, const SplitRow* __restrict__ rows,
                                                           const uint32_t* __restrict__ counters, PiecewiseMap* __restrict__ maps) {
    __shared__ RemapShared<K> sm;
    if (counters[4] == 0u) return;
    const int tid = threadIdx.x;
    for (int64_t row = blockIdx.x; row < m; row += gridDim.x) {
        if (rows[row].piecewise == 0u) continue;
        __syncthreads();                               // the row before has left LDS
        piecewise_map_of<K>(sm, io, io.x + io.xmap.at(row), n);
        maps[row].bound[tid] = static_cast<unsigned long long>(sm.bound[tid]);
        maps[row].shift[tid] = sm.bound_shift[tid];
    }
}

template <typename K>
__global__ __launch_bounds__(kSplitBlock) void split_replan(PassIo<K> io, int64_t m, int64_t n, uint32_t cap, SplitRow* __restrict__ rows,
                                                            uint32_t* __restrict__ counters, uint4* __restrict__ bucket_list, CrowdedList crowded,
                                                            PiecewiseMap* __restrict__ maps) {
    __shared__ RemapShared<K> sm;
    __shared__ uint32_t hist[kFine];
    __shared__ PlanShared<kSplitBlock> plan;
    if (counters[4] == 0u) return;
    const int tid = threadIdx.x;
    for (int64_t row = blockIdx.x; row < m; row += gridDim.x) {
        SplitRow& info = rows[row];
        if (info.piecewise == 0u) continue;
        const K* xrow = io.x + io.xmap.at(row);
        __syncthreads();                               // the row before has left LDS
        piecewise_map_of<K>(sm, io, xrow, n);
        maps[row].bound[tid] = static_cast<unsigned long long>(sm.bound[tid]);      // (split_pass_stable reads it)
        maps[row].shift[tid] = sm.bound_shift[tid];
        for (int i = tid; i < kFine; i += kSplitBlock) hist[i] = 0u;
        __syncthreads();
        FineMap<K> fine_of(info, io.descending);
        fine_of.bound = sm.bound;
        fine_of.bound_shift = sm.bound_shift;
        count_fine_bins<K, kMapPiecewise, kSplitBlock, false>(io, xrow, 0, n, fine_of, hist);
        __syncthreads();
        constexpr int PER = kFine / kSplitBlock;
        uint32_t cnt[PER], bucket[PER];
#pragma unroll
        for (int i = 0; i < PER; ++i) cnt[i] = hist[tid * PER + i];
        (void)plan_buckets<kSplitBlock>(plan, cnt, bucket, n, cap, row, info, counters, bucket_list, crowded, nullptr, true);
    }
}

// Where bucket `id` = row * 256 + b lies: {row, first position in the row, entries, id}.
__device__ __forceinline__ uint4 bucket_at(const SplitRow* __restrict__ infos, uint32_t id) {
    const uint32_t row = id / kMaxBuckets, b = id % kMaxBuckets;
    const SplitRow& info = infos[row];
    const uint32_t b0 = info.begin[b];
    return make_uint4(row, b0, info.begin[b + 1] - b0, id);
}

// Entry `at` of the sorted row goes to the strided outputs (unit strides: plain 32-bit offsets
// from the row's start, the case every contiguous output takes).
template <typename K, bool PAIRS>
__device__ __forceinline__ void emit_entry(const PassIo<K>& io, const K* xrow, K* yrow, int64_t irow, int64_t at, K key, uint32_t val) {
    if (yrow) {
        K bits = decode_key<K>(key, io.kind, io.descending);
        if constexpr (PAIRS) {
            if (io.restore_zero && static_cast<K>(bits << 1) == 0) bits = xrow[static_cast<int64_t>(val) * io.sx];
        }
        if (io.sy == 1) yrow[static_cast<uint32_t>(at)] = bits;
        else yrow[at * io.sy] = bits;
    }
    if constexpr (PAIRS) {
        if (io.idx) {
            if (io.si == 1 && !io.idx64) (static_cast<int32_t*>(io.idx) + irow)[static_cast<uint32_t>(at)] = static_cast<int32_t>(val);
            else if (io.idx64) static_cast<int64_t*>(io.idx)[irow + at * io.si] = static_cast<int64_t>(val);
            else static_cast<int32_t*>(io.idx)[irow + at * io.si] = static_cast<int32_t>(val);
        }
    }
}

// ------------------------------------------------------------------ 4. one pass: chunk -> buckets
// The largest tile of 8-byte keys with indices does not fit LDS twice over: its indices pass
// through the space its keys have left (the threads keep where everything goes in registers).
template <typename K, bool PAIRS, int BLOCK>
constexpr bool kPassInTurn = PAIRS && sizeof(K) == 8 && BLOCK == 1024;

template <typename K, bool PAIRS, int BLOCK, bool STABLE = false>
struct SplitShared {
    uint32_t table[kFine / 4];                 // bucket_of, four fine bins a word
    uint32_t hist[kMaxBuckets];                // keys of the tile per bucket
    uint32_t start[kMaxBuckets];               // where each bucket begins in the tile
    int32_t dst_base[kMaxBuckets];             // row position of a bucket's share of this tile minus start
    uint32_t scan_tmp[kMaxBuckets / kWave];
    K keys[BLOCK * kSplitItems];
    uint32_t vals[PAIRS && !kPassInTurn<K, PAIRS, BLOCK> ? BLOCK * kSplitItems : 1];
    // the stable pass: every wavefront's count of each bucket, which buckets are larger than a
    // workgroup holds, and
    uint32_t wave_hist[STABLE ? BLOCK / kWave : 1][kMaxBuckets];
    uint32_t oversized[STABLE ? kMaxBuckets : 1];
    K mixed[STABLE ? kMaxBuckets : 1];        // ... the bits in which neighbouring entries of such a bucket differ in this tile
    K bound[STABLE ? kSegments : 1];           // the row's PiecewiseMap, if it has one
    uint8_t bound_shift[STABLE ? kSegments : 4];
    uint8_t bucket_at[STABLE ? BLOCK * kSplitItems : 4];      // the bucket of every entry of the tile as laid out
};

// What the stable pass needs beyond the plain one.
template <typename K>
struct StablePass {
    uint32_t cap = 0;                          // the most entries of a bucket that split_finish takes
    unsigned long long* range = nullptr;       // CrowdedList::range
    const PiecewiseMap* map = nullptr;         // the row's, if SplitRow::piecewise says so
    // the row's outputs (what emit_entry reads from PassIo, by value)
    K* yrow = nullptr;                         // the row of the value output, if there is one
    void* idx = nullptr;                       // the index output, if there is one
    int64_t irow = 0, sx = 1, sy = 1, si = 1;  // where its row starts; the strides
    int idx64 = 0, kind = 0, descending = 0, restore_zero = 0;
    bool direct = false;                       // the oversized buckets' entries go straight to the outputs
    __device__ __forceinline__ void emit(const K* xrow, int64_t at, K key, uint32_t val) const {
        if (yrow) {
            K bits = decode_key<K>(key, kind, descending);
            if (restore_zero && static_cast<K>(bits << 1) == 0) bits = xrow[static_cast<int64_t>(val) * sx];
            yrow[at * sy] = bits;
        }
        if (idx) {
            if (idx64) static_cast<int64_t*>(idx)[irow + at * si] = static_cast<int64_t>(val);
            else static_cast<int32_t*>(idx)[irow + at * si] = static_cast<int32_t>(val);
        }
    }
};

// A workgroup moves a range of a row (split_pass: a chunk of kChunk keys) in tiles of BLOCK x 16
// keys: where the range's keys of each bucket go is known (chunk_base), so the workgroup carries
// the running positions itself from tile to tile and nothing passes between workgroups.  A tile's keys find their bucket (table in LDS)
// and their slot among the tile's keys of that bucket with one LDS atomic each, the tile is laid
// out by bucket in LDS and written as runs; once it lies in LDS the registers already receive
// the next tile's keys.  The order inside a run is whatever the atomics gave.
//
// STABLE (rows with buckets larger than a workgroup holds, SplitRow::route 2): a key's slot is
// its rank in element order instead (wave-wide matching of bucket numbers, as the digit passes
// rank; wavefront w takes elements [1024 w, 1024 w + 1024) of the tile), so every bucket receives
// its entries in index order and a bucket of one repeated value arrives sorted.  The entries of
// the oversized buckets go straight to their places in the outputs when those do not overlap
// the input (a bucket of one value is then done: a constant row costs one crossing), and the
// OR and the AND of the keys of every oversized bucket are left in `range`.
template <typename K, bool PAIRS, int BLOCK, int MAP, bool STREAM, bool STABLE = false>
__device__ __forceinline__ void scatter_to_buckets(SplitShared<K, PAIRS, BLOCK, STABLE>& sm, const PassIo<K>& io, int64_t n, int64_t row, const SplitRow& info,
                                                   int64_t chunk_lo, int64_t chunk_hi, const uint32_t* __restrict__ places, StablePass<K> stable = {}) {
    constexpr int ITEMS = kSplitItems;
    constexpr int TILE = BLOCK * kSplitItems;
    constexpr int WAVES = BLOCK / kWave;
    constexpr bool IN_TURN = kPassInTurn<K, PAIRS, BLOCK>;
    static_assert(!(STABLE && IN_TURN), "the stable pass writes keys and indices together");
    const int tid = threadIdx.x;
    const int lane = lane_id();
    const int w = tid / kWave;
    FineMap<K> fine_of(info, io.descending);
    const K* xrow = io.x + io.xmap.at(row);
    const int64_t row_off = row * n;
    if constexpr (STABLE) {
        fine_of.bound = sm.bound;
        fine_of.bound_shift = sm.bound_shift;
        if (fine_of.piecewise != 0u && tid < kSegments) {
            sm.bound[tid] = static_cast<K>(stable.map->bound[tid]);
            sm.bound_shift[tid] = stable.map->shift[tid];
        }
    }
    // element of the tile that this thread's item k is
    auto element_of = [&](int k) __attribute__((always_inline)) { return STABLE ? w * (kWave * ITEMS) + k * kWave + lane : tid + k * BLOCK; };

    // (no branches: an element beyond the chunk's end reads the tile's first element instead and is never used)
    auto load_tile = [&](int64_t tile_base, K (&key)[ITEMS]) __attribute__((always_inline)) {
        const int valid = static_cast<int>((chunk_hi - tile_base < TILE) ? chunk_hi - tile_base : TILE);
        const K* src = xrow + tile_base * io.sx;
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) {
            const int e = element_of(k);
            const K* at = &src[static_cast<int64_t>(e < valid ? e : 0) * io.sx];
            if constexpr (sizeof(K) == 4 && STREAM) key[k] = load_stream(at);       // (non-temporal loads measured: a gain for 4-byte keys,
            else key[k] = *at;                                                      // a loss of 7 % for 8-byte keys)
        }
    };

    K key[ITEMS];
    load_tile(chunk_lo, key);
    // threads 0 .. 255 each own a bucket (and 16 bytes of the table)
    const bool owner = tid < kMaxBuckets;
    uint32_t next = 0;                                 // where this chunk's coming keys of bucket tid go
    if (owner) {
        reinterpret_cast<uint4*>(sm.table)[tid] = reinterpret_cast<const uint4*>(info.bucket_of)[tid];
        sm.hist[tid] = 0u;
        next = places[tid];
        if constexpr (STABLE) {
            sm.oversized[tid] = (tid < static_cast<int>(info.n_buckets) && info.begin[tid + 1] - info.begin[tid] > stable.cap) ? 1u : 0u;
            sm.mixed[tid] = K(0);
        }
    }
    if constexpr (STABLE)
        for (int i = tid; i < WAVES * kMaxBuckets; i += BLOCK) (&sm.wave_hist[0][0])[i] = 0u;
    // (stable) bucket numbers lie below n_buckets: only those bits are matched; elements beyond the
    // chunk's end count as the last bucket's, after every element of the chunk
    const uint32_t last_bucket = info.n_buckets - 1u;
    const uint32_t vary = last_bucket != 0u ? (2u << (31 - __builtin_clz(last_bucket))) - 1u : 0u;
    const bool direct = STABLE && stable.direct;
    __syncthreads();

    auto move_chunk = [&](auto mode_tag) __attribute__((always_inline)) {
    constexpr int MODE = decltype(mode_tag)::value;
    constexpr bool GAP = MAP == kMapGap || MAP == kMapAny;
    for (int64_t tile_base = chunk_lo; tile_base < chunk_hi; tile_base += TILE) {
        const int valid = static_cast<int>((chunk_hi - tile_base < TILE) ? chunk_hi - tile_base : TILE);
        const bool full = valid == TILE;
        SPLIT_PHASE_BEGIN();
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) key[k] = key_of_element<K>(io, key[k]);
        SPLIT_PHASE(0);

        // ---- bucket of every key (table), then its slot among the tile's keys of that bucket:
        // one LDS atomic each, eight lookups issued before their eight atomics
        uint32_t where[ITEMS];                     // bucket << 16 | slot, later the key's place in the tile
        if constexpr (STABLE) {
            uint32_t rank[ITEMS];
#pragma unroll
            for (int k = 0; k < ITEMS; ++k) {
                const uint32_t f = fine_of.template bin_as<MODE, GAP>(key[k]);
                where[k] = (sm.table[f >> 2] >> (8u * (f & 3u))) & 0xffu;
                if (!full && element_of(k) >= valid) where[k] = last_bucket;
            }
            rank_by_digit<ITEMS>(sm.wave_hist[w], where, vary, rank);
#pragma unroll
            for (int k = 0; k < ITEMS; ++k) where[k] = (where[k] << 16) | rank[k];
        } else {
#pragma unroll
        for (int k0 = 0; k0 < ITEMS; k0 += 8) {
#pragma unroll
            for (int k = k0; k < k0 + 8; ++k) {
                const uint32_t f = fine_of.template bin_as<MODE, GAP>(key[k]);
                where[k] = (sm.table[f >> 2] >> (8u * (f & 3u))) & 0xffu;
            }
#pragma unroll
            for (int k = k0; k < k0 + 8; ++k)
                if (full || tid + k * BLOCK < valid) where[k] = (where[k] << 16) | atomicAdd(&sm.hist[where[k]], 1u);
        }
        }
        __syncthreads();
        SPLIT_PHASE(1);

        // ---- thread b owns bucket b: its place in the tile and in the row
        uint32_t own_start = 0, own_count = 0;         // (stable) ... and how many entries of the chunk it has in the tile
        {
            uint32_t count = 0, incl = 0;
            if (owner) {
                if constexpr (STABLE) {
                    // each wavefront's share of the bucket starts after the shares of the wavefronts before
#pragma unroll
                    for (int i = 0; i < WAVES; ++i) {
                        const uint32_t c = sm.wave_hist[i][tid];
                        sm.wave_hist[i][tid] = count;
                        count += c;
                    }
                } else {
                    count = sm.hist[tid];
                }
                incl = wave_scan_inclusive(count, 0u, [](uint32_t a, uint32_t b) { return a + b; });
                if (lane == kWave - 1) sm.scan_tmp[w] = incl;
                sm.hist[tid] = 0u;                         // for the next tile
            }
            __syncthreads();
            if (owner) {
                uint32_t pre = 0;
                for (int i = 0; i < w; ++i) pre += sm.scan_tmp[i];
                const uint32_t start = pre + incl - count;
                sm.start[tid] = start;
                sm.dst_base[tid] = static_cast<int32_t>(next) - static_cast<int32_t>(start);
                next += count;
                if constexpr (STABLE) {
                    own_start = start;
                    own_count = (!full && tid == static_cast<int>(last_bucket)) ? count - static_cast<uint32_t>(TILE - valid) : count;
                }
            }
        }
        __syncthreads();
        SPLIT_PHASE(2);

        // ---- lay the tile out by bucket (bucket starts read first, then the stores)
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) {
            // (stable: the bucket stays in the upper half, for the table of buckets beside the tile)
            if constexpr (STABLE) where[k] = (where[k] & 0xffff0000u) | (sm.start[where[k] >> 16] + sm.wave_hist[w][where[k] >> 16] + (where[k] & 0xffffu));
            else where[k] = sm.start[where[k] >> 16] + (where[k] & 0xffffu);
        }
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) {
            if (full || element_of(k) < valid) {
                const uint32_t at_tile = STABLE ? (where[k] & 0xffffu) : where[k];
                sm.keys[at_tile] = key[k];
                if constexpr (PAIRS && !IN_TURN) sm.vals[at_tile] = static_cast<uint32_t>(tile_base) + static_cast<uint32_t>(element_of(k));
                if constexpr (STABLE) sm.bucket_at[at_tile] = static_cast<uint8_t>(where[k] >> 16);
            }
        }
        __syncthreads();
        SPLIT_PHASE(3);
        if constexpr (STABLE)
            for (int i = tid; i < WAVES * kMaxBuckets; i += BLOCK) (&sm.wave_hist[0][0])[i] = 0u;      // for the next tile
        // the tile is in LDS: the registers take the next tile, whose keys arrive while this one is written
        if (tile_base + TILE < chunk_hi) load_tile(tile_base + TILE, key);

        // ---- write runs: thread tid takes tile positions tid, tid + BLOCK, ...; eight at a time, the
        // reads of each step issued for all eight before the next step uses them
        if constexpr (STABLE) {
            K* dk = io.kbuf[0] + row_off;
            uint32_t* dv = PAIRS ? io.vbuf[0] + row_off : nullptr;
            constexpr int G = sizeof(K) == 8 ? (PAIRS ? 2 : 4) : 8;      // tile positions a thread handles at a time (registers)
            const K own_first = (owner && own_count != 0u) ? sm.keys[own_start] : K(0);
#pragma unroll
            for (int k0 = 0; k0 < ITEMS; k0 += G) {
                K out[G], before[G];
                uint32_t pay[PAIRS ? G : 1], b[G], first[G], big[G];
                int32_t at[G];
#pragma unroll
                for (int j = 0; j < G; ++j) {
                    const int p = (k0 + j) * BLOCK + tid;
                    out[j] = sm.keys[p];
                    before[j] = sm.keys[p > 0 ? p - 1 : 0];
                    if constexpr (PAIRS) pay[j] = sm.vals[p];
                }
#pragma unroll
                for (int j = 0; j < G; ++j) b[j] = sm.bucket_at[(k0 + j) * BLOCK + tid];
#pragma unroll
                for (int j = 0; j < G; ++j) {
                    at[j] = sm.dst_base[b[j]] + ((k0 + j) * BLOCK + tid);
                    first[j] = sm.start[b[j]];
                    big[j] = sm.oversized[b[j]];
                }
#pragma unroll
                for (int j = 0; j < G; ++j) {
                    const uint32_t p = static_cast<uint32_t>((k0 + j) * BLOCK + tid);
                    if (!full && p >= static_cast<uint32_t>(valid)) continue;
                    if (big[j] != 0u) {
                        if (p > first[j] && before[j] != out[j]) atomicOr(&sm.mixed[b[j]], static_cast<K>(before[j] ^ out[j]));
                        if (direct) {
                            stable.emit(xrow, at[j], out[j], PAIRS ? pay[j] : 0u);
                            continue;
                        }
                    }
                    dk[at[j]] = out[j];
                    if constexpr (PAIRS) dv[at[j]] = pay[j];
                }
            }
            __syncthreads();                               // the tile in LDS has left, every mixed bucket is marked
            if (owner && own_count != 0u && sm.oversized[tid] != 0u) {
                // the OR and the AND of the bucket's keys in this tile, from one of them and the bits that vary
                const K vary_here = sm.mixed[tid];
                sm.mixed[tid] = K(0);
                const uint32_t id = static_cast<uint32_t>(row) * kMaxBuckets + tid;
                atomicOr(&stable.range[2 * id], static_cast<unsigned long long>(static_cast<K>(own_first | vary_here)));
                atomicAnd(&stable.range[2 * id + 1], static_cast<unsigned long long>(static_cast<K>(own_first & ~vary_here)) | ~static_cast<unsigned long long>(~K(0)));
            }
            continue;
        } else {
            K* dk = io.kbuf[0] + row_off;
            uint32_t* dv = PAIRS ? io.vbuf[0] + row_off : nullptr;
            int32_t at[ITEMS];                         // where tile position k * BLOCK + tid goes in the row
#pragma unroll
            for (int k0 = 0; k0 < ITEMS; k0 += 8) {
                K out[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) out[j] = sm.keys[(k0 + j) * BLOCK + tid];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t f = fine_of.template bin_as<MODE, GAP>(out[j]);
                    at[k0 + j] = static_cast<int32_t>((sm.table[f >> 2] >> (8u * (f & 3u))) & 0xffu);
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) at[k0 + j] = sm.dst_base[at[k0 + j]] + ((k0 + j) * BLOCK + tid);
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    if (full || (k0 + j) * BLOCK + tid < valid) dk[at[k0 + j]] = out[j];
                if constexpr (PAIRS && !IN_TURN) {
                    uint32_t pay[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) pay[j] = sm.vals[(k0 + j) * BLOCK + tid];
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        if (full || (k0 + j) * BLOCK + tid < valid) dv[at[k0 + j]] = pay[j];
                }
            }
            if constexpr (IN_TURN) {
                // the keys have left: their space takes the indices, laid out the same way
                uint32_t* turn = reinterpret_cast<uint32_t*>(sm.keys);
                __syncthreads();
#pragma unroll
                for (int k = 0; k < ITEMS; ++k)
                    if (full || tid + k * BLOCK < valid) turn[where[k]] = static_cast<uint32_t>(tile_base) + static_cast<uint32_t>(tid + k * BLOCK);
                __syncthreads();
#pragma unroll
                for (int k0 = 0; k0 < ITEMS; k0 += 8) {
                    uint32_t pay[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) pay[j] = turn[(k0 + j) * BLOCK + tid];
#pragma unroll
                    for (int j = 0; j < 8; ++j)
                        if (full || (k0 + j) * BLOCK + tid < valid) dv[at[k0 + j]] = pay[j];
                }
            }
        }
        SPLIT_PHASE(5);
        __syncthreads();                                   // the tile in LDS has left
    }
    };
    if constexpr (MAP == kMapAny) {
        if (fine_of.piecewise) move_chunk(std::integral_constant<int, 2>());
        else if (fine_of.by_value) move_chunk(std::integral_constant<int, 1>());
        else move_chunk(std::integral_constant<int, 0>());
    } else {
        if (MAP == kMapValue && fine_of.by_value) move_chunk(std::integral_constant<int, MAP == kMapValue ? 1 : 0>());
        else move_chunk(std::integral_constant<int, 0>());
    }
}

// One workgroup per chunk (kChunk keys): elements [chunk_lo, chunk_hi) of row `row` go to their
// buckets, places[b] being the row position of the first of them that belongs to bucket b.
template <typename K, bool PAIRS, int BLOCK, int MAP>
__global__ __launch_bounds__(BLOCK) __attribute__((amdgpu_waves_per_eu(4))) void split_pass(PassIo<K> io, int64_t n, int64_t chunks_per_row,
                                                          const SplitRow* __restrict__ infos, const uint32_t* __restrict__ chunk_base) {
    static_assert(kChunk % (BLOCK * kSplitItems) == 0, "whole tiles a chunk");
    __shared__ SplitShared<K, PAIRS, BLOCK> sm;
    const int64_t row = blockIdx.x / chunks_per_row;
    const int64_t c = blockIdx.x - row * chunks_per_row;
    const SplitRow& info = infos[row];
    if (info.route != 1u) return;                      // (a row with buckets larger than a workgroup holds: split_pass_stable)
    const int64_t chunk_lo = c * kChunk;
    const int64_t chunk_hi = (chunk_lo + kChunk < n) ? chunk_lo + kChunk : n;
    scatter_to_buckets<K, PAIRS, BLOCK, MAP, true>(sm, io, n, row, info, chunk_lo, chunk_hi, chunk_base + static_cast<int64_t>(blockIdx.x) * kMaxBuckets);
}

// Steps 1 to 4 for a whole row by one workgroup, for calls of many rows that are not too long
// (at least two rows per compute unit, rows of up to 131072 keys): the row's range from its
// sample, its fine-bin histogram in LDS (no chunks, no tables in memory), its buckets, and the
// scatter, for which the row is read a second time - out of the caches as a rule, the same
// workgroup having just read it.  Three launches fewer, one crossing of HBM less, and what one
// workgroup waits for (the sample, the dependent steps of the plan) the others on its compute
// unit fill.  Rows of pairs with buckets larger than a workgroup holds are left to
// split_pass_stable.
template <typename K, bool PAIRS, int BLOCK, int MAP>
__global__ __launch_bounds__(BLOCK) __attribute__((amdgpu_waves_per_eu(4))) void split_front(PassIo<K> io, int64_t n, uint32_t cap, SplitRow* __restrict__ rows,
                                                           uint32_t* __restrict__ counters, uint4* __restrict__ bucket_list,
                                                           CrowdedList crowded) {
    static_assert(MAP != kMapValue, "rows short enough for the smallest buckets");
    __shared__ SplitShared<K, PAIRS, BLOCK> sm;
    __shared__ PlanShared<BLOCK> plan;
    static_assert(sizeof(sm.keys) >= kFine * sizeof(uint32_t), "the histogram lies where the tiles will");
    uint32_t* hist = reinterpret_cast<uint32_t*>(sm.keys);
    const int64_t row = blockIdx.x;
    const K* xrow = io.x + io.xmap.at(row);
    SplitRow& info = rows[row];
    for (int i = threadIdx.x; i < kFine; i += BLOCK) hist[i] = 0u;
    const FineRange range = sample_row<K, MAP, BLOCK>(io, xrow, n, cap, hist);
    if (threadIdx.x == 0) {
        range.store(info);
        if (range.piecewise != 0u) {                   // split_replan counts and plans such a row
            info.route = 0u;
            atomicOr(&counters[4], 1u);
        }
    }
    if (range.piecewise != 0u) return;
    count_fine_bins<K, MAP, BLOCK, false>(io, xrow, 0, n, FineMap<K>(range, io.descending), hist);
    __syncthreads();
    constexpr int PER = kFine / kSplitBlock;
    uint32_t cnt[PER], bucket[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) cnt[i] = threadIdx.x < kSplitBlock ? hist[threadIdx.x * PER + i] : 0u;
    uint32_t route = 0;
    (void)plan_buckets<BLOCK>(plan, cnt, bucket, n, cap, row, info, counters, bucket_list, crowded, &route);
    if (route != 1u) return;
    __syncthreads();                                   // the row's record and table are in memory, the histogram has been read
    scatter_to_buckets<K, PAIRS, BLOCK, MAP, true>(sm, io, n, row, info, 0, n, plan.begin);
}

__global__ void split_clear(uint32_t* __restrict__ counters) {
    if (threadIdx.x < 8) counters[threadIdx.x] = 0u;      // what the later launches of this sort count up from
}

// The stable pass for the rows that have buckets larger than a workgroup holds (SplitRow::route
// 2).  A small grid walks the units - chunks, or whole rows when split_front made the plan and
// left no chunk tables - so the launch costs little in the usual case of no such row.
constexpr int kStableBlock = 512;
template <typename K, bool PAIRS>
__global__ __launch_bounds__(kStableBlock) void split_pass_stable(PassIo<K> io, int64_t n, uint32_t cap, int64_t chunks_per_row, int64_t units,
                                                                  const SplitRow* __restrict__ infos, const uint32_t* __restrict__ counters,
                                                                  const uint32_t* __restrict__ chunk_base, unsigned long long* __restrict__ range,
                                                                  const PiecewiseMap* __restrict__ maps) {
    static_assert(kChunk % (kStableBlock * kSplitItems) == 0, "whole tiles a chunk");
    __shared__ SplitShared<K, PAIRS, kStableBlock, true> sm;
    if (counters[3] == 0u) return;                     // no such row in this call
    for (int64_t unit = blockIdx.x; unit < units; unit += gridDim.x) {
        const int64_t row = chunk_base ? unit / chunks_per_row : unit;
        const int64_t c = chunk_base ? unit - row * chunks_per_row : 0;
        const SplitRow& info = infos[row];
        if (info.route != 2u) continue;
        const int64_t chunk_lo = c * kChunk;
        const int64_t chunk_hi = (chunk_base && chunk_lo + kChunk < n) ? chunk_lo + kChunk : n;
        __syncthreads();                               // the unit before has left the tables
        scatter_to_buckets<K, PAIRS, kStableBlock, kMapAny, false, true>(sm, io, n, row, info, chunk_lo, chunk_hi,
                                                                        chunk_base ? chunk_base + unit * kMaxBuckets : info.begin,
                                                                        StablePass<K>{cap, range, maps + row, io.y ? io.y + io.ymap.at(row) : nullptr, PAIRS ? io.idx : nullptr,
                                                                                      (PAIRS && io.idx) ? io.imap.at(row) : 0, io.sx, io.sy, io.si, io.idx64,
                                                                                      io.kind, io.descending, PAIRS ? io.restore_zero : 0, io.x_intact != 0});
    }
}

// ------------------------------------------------------------------ 5. a bucket, on chip
// Whether split_finish keeps every entry's bin beside it in LDS (two bytes an entry) instead of
// working it out again from the key when the entry is ranked; 8-byte keys with indices have no
// room for that with two workgroups on a compute unit.
template <typename K, bool PAIRS, int WAVES>
constexpr bool kKeepBins = !(PAIRS && sizeof(K) == 8 && WAVES >= 8);

template <typename K, bool PAIRS, int WAVES>
struct FinishShared {
    uint32_t bins[finish_bins(WAVES) / 2];     // two 16-bit counters a word: counts, then bin starts, then bin ends
    K keys[finish_cap(WAVES)];
    uint32_t vals[PAIRS ? finish_cap(WAVES) : 1];
    uint16_t bin_at[kKeepBins<K, PAIRS, WAVES> ? finish_cap(WAVES) : 1];
    K red_key[WAVES];
    uint32_t red_val[WAVES], red32[WAVES];
    uint32_t crowded;
};

// Workgroup g takes entries g, g + G, ... of the bucket list (what split_plan wrote: row, first
// position, size of every bucket); once a bucket lies in LDS the registers already receive the
// next one's entries.  A bucket whose bins are too crowded to rank by comparison is put on
// `crowded_list` (counters[1] entries) for split_finish_crowded.
template <typename K, bool PAIRS, int WAVES>
__global__ __launch_bounds__(WAVES * kWave) __attribute__((amdgpu_waves_per_eu(4))) void split_finish(PassIo<K> io, int64_t n,
                                                             uint32_t compare_max, uint32_t* __restrict__ counters,
                                                             const uint4* __restrict__ bucket_list, uint2* __restrict__ crowded_list) {
    constexpr int ITEMS = kFinishItems;
    constexpr int T = WAVES * kWave;
    constexpr int kBins = finish_bins(WAVES);
    constexpr int kBinBits = WAVES == 16 ? 14 : WAVES == 8 ? 13 : 12;
    static_assert(kBins == 1 << kBinBits, "bins and their bits");
    constexpr int WORDS = kBins / 2 / T;       // counter words a thread scans (8)
    constexpr bool KEEP = kKeepBins<K, PAIRS, WAVES>;
    __shared__ FinishShared<K, PAIRS, WAVES> sm;
    const int tid = threadIdx.x;
    const int lane = lane_id();
    const int w = tid / kWave;
    const int seg = w * kWave * ITEMS + lane;              // item k of this thread is entry seg + 64 k of the bucket
    const int64_t total = counters[2];                     // buckets on the list
    const int64_t step = gridDim.x;

    // (no branches: an entry beyond the bucket's end reads its first entry instead and is never used)
    auto load_bucket = [&](const uint4& d, K (&key)[ITEMS], uint32_t (&val)[PAIRS ? ITEMS : 1]) __attribute__((always_inline)) {
        const K* src = io.kbuf[0] + static_cast<int64_t>(d.x) * n + d.y;
        const uint32_t* vsrc = PAIRS ? io.vbuf[0] + static_cast<int64_t>(d.x) * n + d.y : nullptr;
        const int size = static_cast<int>(d.z);
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) {
            const int e = seg + k * kWave;
            key[k] = src[e < size ? e : 0];
            if constexpr (PAIRS) val[k] = vsrc[e < size ? e : 0];
        }
    };

    int64_t v = blockIdx.x;
    if (v >= total) return;
    uint4 cur = bucket_list[v];
    K key[ITEMS];
    uint32_t val[PAIRS ? ITEMS : 1];
    load_bucket(cur, key, val);
    int dirty_words = kBins / 2;                           // counter words that are not zero
    for (;;) {
        SPLIT_PHASE_BEGIN();
        const int64_t vn = v + step;
        uint4 nxt = cur;
        if (vn < total) nxt = bucket_list[vn];             // on its way while this bucket is counted
        const int valid = static_cast<int>(cur.z);
        const int64_t begin = cur.y;
        const int64_t row = cur.x;

        // ---- smallest key (and index): the origin of the offsets
        K lo = ~K(0);
        uint32_t vlo = ~0u;
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) {
            if (seg + k * kWave < valid) {
                lo = key[k] < lo ? key[k] : lo;
                if constexpr (PAIRS) vlo = val[k] < vlo ? val[k] : vlo;
            }
        }
        if (dirty_words == kBins / 2) {                    // what the bucket before used
#pragma unroll
            for (int i = 0; i < kBins / 2 / T; ++i) sm.bins[tid + i * T] = 0u;
        } else {
            for (int i = tid; i < dirty_words; i += T) sm.bins[i] = 0u;
        }
        lo = wave_reduce(lo, [](K a, K c) { return a < c ? a : c; });
        if constexpr (PAIRS) vlo = wave_reduce(vlo, [](uint32_t a, uint32_t c) { return a < c ? a : c; });
        if (lane == 0) {
            sm.red_key[w] = lo;
            if constexpr (PAIRS) sm.red_val[w] = vlo;
        }
        if (tid == 0) sm.crowded = 0u;
        __syncthreads();
#pragma unroll
        for (int i = 0; i < WAVES; ++i) {
            lo = sm.red_key[i] < lo ? sm.red_key[i] : lo;
            if constexpr (PAIRS) vlo = sm.red_val[i] < vlo ? sm.red_val[i] : vlo;
        }
        __syncthreads();                                   // red_key / red_val are reused at once
        // ---- OR of all offsets: its leading bit bounds them, its trailing zeros carry nothing (quantised values)
        K ors = 0;
        uint32_t vors = 0;
#pragma unroll
        for (int k = 0; k < ITEMS; ++k)
            if (seg + k * kWave < valid) {
                ors |= static_cast<K>(key[k] - lo);
                if constexpr (PAIRS) vors |= val[k] - vlo;
            }
        ors = wave_reduce(ors, [](K a, K c) { return static_cast<K>(a | c); });
        if constexpr (PAIRS) vors = wave_reduce(vors, [](uint32_t a, uint32_t c) { return a | c; });
        if (lane == 0) {
            sm.red_key[w] = ors;
            if constexpr (PAIRS) sm.red_val[w] = vors;
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < WAVES; ++i) {
            ors |= sm.red_key[i];
            if constexpr (PAIRS) vors |= sm.red_val[i];
        }

        // The word an entry is binned by: its key's offset from the smallest key without the
        // zero bits; for pairs, when there is room, that offset with the index's offset below it,
        // so that equal keys spread over bins in index order instead of crowding one.
        const int zeros = ors ? __builtin_ctzll(static_cast<unsigned long long>(ors)) : 0;
        const int key_bits = ors ? 64 - __builtin_clzll(static_cast<unsigned long long>(ors)) - zeros : 0;
        int idx_bits = 0;
        bool packed = false;                               // the word fits a key's width
        if constexpr (PAIRS) {
            idx_bits = vors ? 32 - __builtin_clz(vors) : 0;
            packed = idx_bits != 0 && key_bits + idx_bits <= static_cast<int>(8 * sizeof(K));
            if (key_bits + idx_bits > 64) idx_bits = 0;    // wide keys seldom repeat
        }
        const int width = key_bits + idx_bits;
        const int down = width > kBinBits ? width - kBinBits : 0;      // words >> down lie below kBins
        // a bucket whose words are narrower than that (quantised values, small integers) uses the
        // first 2^width bins only: the others are neither scanned now nor cleared afterwards
        // (the smallest buckets only: the larger ones measured 2.5 % slower with the test in their loops)
        constexpr bool kNarrow = WAVES == 4;
        const int used_words = (!kNarrow || width >= kBinBits) ? kBins / 2 : (width > 4 ? (1 << width) / 2 : WORDS);
        dirty_words = used_words;
        SPLIT_PHASE(8);

        // The rest of the bucket's work in two forms.  PACKED (pairs whose word fits a key's
        // width): the word alone stands for the entry from here on - it is unique, orders the
        // entries as (key, index) does, and gives both back when the entry leaves - so LDS holds
        // one word per entry and ranking is one comparison.  Otherwise keys (and indices) are
        // kept as they are and entries of a bin are told apart by comparing them whole.
        auto finish = [&](auto packed_tag) __attribute__((always_inline)) {
            constexpr bool PACKED = decltype(packed_tag)::value;
            constexpr bool VALS = PAIRS && !PACKED;              // indices travel beside the keys
            constexpr bool KEPT = KEEP && !PACKED;               // bins kept beside the entries
            auto bin_of = [&](K k1, uint32_t v1) __attribute__((always_inline)) -> uint32_t {
                if constexpr (PACKED) {
                    return static_cast<uint32_t>(k1 >> down);
                } else {
                    unsigned long long word = static_cast<unsigned long long>(static_cast<K>(k1 - lo) >> zeros);
                    if constexpr (PAIRS) {
                        if (idx_bits) word = (word << idx_bits) | static_cast<unsigned long long>(v1 - vlo);
                    }
                    return static_cast<uint32_t>(word >> down);
                }
            };
            // entries that share a bin are told apart by comparison, unless the bin says it all
            const bool compare = down != 0 || (VALS && idx_bits == 0 && vors != 0u);
            if constexpr (PACKED) {
#pragma unroll
                for (int k = 0; k < ITEMS; ++k)
                    key[k] = static_cast<K>(static_cast<K>(static_cast<K>(key[k] - lo) >> zeros) << idx_bits) | static_cast<K>(val[k] - vlo);
            }

            // ---- count
            uint32_t bin[ITEMS];
#pragma unroll
            for (int k = 0; k < ITEMS; ++k) bin[k] = bin_of(key[k], VALS ? val[k] : 0u);
#pragma unroll
            for (int k = 0; k < ITEMS; ++k)
                if (seg + k * kWave < valid) atomicAdd(&sm.bins[bin[k] >> 1], 1u << (16u * (bin[k] & 1u)));
            __syncthreads();
            SPLIT_PHASE(9);

            // ---- counts -> bin starts (exclusive prefix over the bins), and the fullest bin
            {
                uint32_t words[WORDS] = {};
                uint32_t sum = 0, fullest = 0;
                const bool in_use = !kNarrow || tid * WORDS < used_words;
                if (in_use) {
#pragma unroll
                    for (int i = 0; i < WORDS; ++i) words[i] = sm.bins[tid * WORDS + i];
                }
#pragma unroll
                for (int i = 0; i < WORDS; ++i) {
                    const uint32_t c0 = words[i] & 0xffffu, c1 = words[i] >> 16;
                    sum += c0 + c1;
                    fullest = c0 > fullest ? c0 : fullest;
                    fullest = c1 > fullest ? c1 : fullest;
                }
                const uint32_t incl = wave_scan_inclusive(sum, 0u, [](uint32_t a, uint32_t c) { return a + c; });
                if (lane == kWave - 1) sm.red32[w] = incl;
                fullest = wave_reduce(fullest, [](uint32_t a, uint32_t c) { return a > c ? a : c; });
                if (lane == 0 && fullest > compare_max) atomicMax(&sm.crowded, fullest);
                __syncthreads();
                uint32_t run = incl - sum;
                for (int i = 0; i < w; ++i) run += sm.red32[i];
                if (in_use) {
#pragma unroll
                    for (int i = 0; i < WORDS; ++i) {
                        const uint32_t c0 = words[i] & 0xffffu, c1 = words[i] >> 16;
                        sm.bins[tid * WORDS + i] = run | ((run + c0) << 16);
                        run += c0 + c1;
                    }
                }
            }
            __syncthreads();
            SPLIT_PHASE(10);

            if (compare && sm.crowded != 0u) {
                // many equal or clustered keys: the stable digit passes of split_finish_crowded take this bucket
                if (tid == 0) crowded_list[atomicAdd(&counters[1], 1u)] = make_uint2(cur.w, kNoWindow);
                if (vn < total) load_bucket(nxt, key, val);
                return;
            }
            // ---- place: the atomic hands out the next free entry of the bin, whose word ends up at its end
            {
                uint32_t old[ITEMS];
#pragma unroll
                for (int k = 0; k < ITEMS; ++k)
                    if (seg + k * kWave < valid) old[k] = atomicAdd(&sm.bins[bin[k] >> 1], 1u << (16u * (bin[k] & 1u)));
#pragma unroll
                for (int k = 0; k < ITEMS; ++k) {
                    if (seg + k * kWave < valid) {
                        const uint32_t pos = (old[k] >> (16u * (bin[k] & 1u))) & 0xffffu;
                        sm.keys[pos] = key[k];
                        if constexpr (VALS) sm.vals[pos] = val[k];
                        if constexpr (KEPT) {
                            if (compare) sm.bin_at[pos] = static_cast<uint16_t>(bin[k]);
                        }
                    }
                }
            }
            __syncthreads();
            SPLIT_PHASE(11);
            // the bucket is in LDS: the registers take the next bucket, whose entries arrive while
            // this one is ranked and written
            if (vn < total) load_bucket(nxt, key, val);

            const K* xrow = io.x + io.xmap.at(row);
            K* yrow = io.y ? io.y + io.ymap.at(row) : nullptr;
            const int64_t irow = (PAIRS && io.idx) ? io.imap.at(row) : 0;
            const K idx_mask = static_cast<K>((K(1) << idx_bits) - 1);
            // entry `at` of the row leaves: a packed word gives its key and index back first
            auto emit = [&](int64_t at, K k1, uint32_t v1) __attribute__((always_inline)) {
                if constexpr (PACKED)
                    emit_entry<K, PAIRS>(io, xrow, yrow, irow, at, static_cast<K>(lo + static_cast<K>(static_cast<K>(k1 >> idx_bits) << zeros)),
                                         vlo + static_cast<uint32_t>(k1 & idx_mask));
                else
                    emit_entry<K, PAIRS>(io, xrow, yrow, irow, at, k1, v1);
            };
            // ---- rank inside the bin and write: thread tid takes entries tid, tid + T, ...; five at
            // a time, each step reading for all five before the next step looks at what came back
            constexpr int B = 5;
            static_assert(ITEMS % B == 0, "whole batches");
#pragma unroll 1
            for (int k0 = 0; k0 < ITEMS; k0 += B) {
                if (k0 * T >= valid) break;                // (uniform) nothing left
                K mine[B];
                uint32_t mine_v[VALS ? B : 1] = {};
                uint32_t mine_b[B];
#pragma unroll
                for (int j = 0; j < B; ++j) {
                    const int pos = (k0 + j) * T + tid;
                    const int at = pos < valid ? pos : 0;
                    mine[j] = sm.keys[at];
                    if constexpr (VALS) mine_v[j] = sm.vals[at];
                    if constexpr (KEPT) mine_b[j] = sm.bin_at[at];
                }
                if (!compare) {
#pragma unroll
                    for (int j = 0; j < B; ++j)
                        if ((k0 + j) * T + tid < valid) emit(begin + (k0 + j) * T + tid, mine[j], VALS ? mine_v[j] : 0u);
                    continue;
                }
                int first[B], end[B], ahead[B];
#pragma unroll
                for (int j = 0; j < B; ++j) {
                    uint32_t b1;
                    if constexpr (KEPT) b1 = mine_b[j];
                    else b1 = bin_of(mine[j], VALS ? mine_v[j] : 0u);
                    end[j] = static_cast<int>((sm.bins[b1 >> 1] >> (16u * (b1 & 1u))) & 0xffffu);
                    const uint32_t b0 = b1 - 1u;
                    first[j] = b1 == 0u ? 0 : static_cast<int>((sm.bins[b0 >> 1] >> (16u * (b0 & 1u))) & 0xffffu);
                    ahead[j] = 0;
                }
                // the first kNear entries of the bin without a loop (a bin seldom holds more)
#pragma unroll
                for (int i = 0; i < kNear; ++i) {
                    K other[B];
                    uint32_t other_v[VALS ? B : 1] = {};
#pragma unroll
                    for (int j = 0; j < B; ++j) {
                        const int q = first[j] + i < valid ? first[j] + i : 0;
                        other[j] = sm.keys[q];
                        if constexpr (VALS) other_v[j] = sm.vals[q];
                    }
#pragma unroll
                    for (int j = 0; j < B; ++j) {
                        const int q = first[j] + i;
                        bool before = other[j] < mine[j];
                        if constexpr (!PACKED) {               // (packed words are all different)
                            if (other[j] == mine[j]) {
                                if constexpr (VALS) before = other_v[j] < mine_v[j];
                                else before = q < (k0 + j) * T + tid;
                            }
                        }
                        ahead[j] += (q < end[j] && before) ? 1 : 0;
                    }
                }
#pragma unroll
                for (int j = 0; j < B; ++j) {
                    const int pos = (k0 + j) * T + tid;
                    if (pos >= valid) continue;
                    for (int q = first[j] + kNear; q < end[j]; ++q) {          // the rest of a fuller bin
                        const K other = sm.keys[q];
                        bool before = other < mine[j];
                        if constexpr (!PACKED) {
                            if (other == mine[j]) {
                                if constexpr (VALS) before = sm.vals[q] < mine_v[j];
                                else before = q < pos;
                            }
                        }
                        ahead[j] += before ? 1 : 0;
                    }
                    emit(begin + first[j] + ahead[j], mine[j], VALS ? mine_v[j] : 0u);
                }
            }
            SPLIT_PHASE(12);
        };
        if (PAIRS && packed) finish(std::integral_constant<bool, PAIRS>());
        else finish(std::false_type());
        if (vn >= total) break;
        v = vn;
        cur = nxt;
        __syncthreads();                                   // the bucket in LDS has left
    }
}

// ------------------------------------------------------------------ 6. what split_finish does not take
// A bucket larger than a workgroup holds, sorted by the one workgroup that drew it from the list.
// Its entries lie in kbuf[0] / vbuf[0] ("side A"), pairs in index order (split_pass_stable).  The
// bucket's place in the outputs ("side B": the value output and / or the index output, whatever
// their strides) is the only other memory that is certainly there, so the stable digit passes
// below ping-pong between the two: key images travel through the value output as they are and
// are decoded by the last pass, which always goes from A to B; without a value output the keys
// of side B are read again from the input through the indices (possible while the input is
// intact).  Digits that are the same in the whole bucket are left out - a bucket of one repeated
// value is just copied - and an even number of passes is preceded by a plain copy to B.
template <typename K, bool PAIRS>
struct OversizedIo {
    // (what it needs of PassIo, by value: a reference to the kernel's argument block made the
    // compiler keep a private copy of the whole block in scratch memory)
    const K* xrow;
    K* yrow;
    void* idx;
    int64_t irow, sx, sy, si;
    int idx64, kind, descending, canon_zero, restore_zero;
    K* ak;                                             // side A
    uint32_t* av;
    __device__ __forceinline__ K image_of(K bits) const {
        if (canon_zero && static_cast<K>(bits << 1) == 0) bits = 0;
        return encode_key<K>(bits, kind, descending);
    }
    // (values: side B holds what split_pass_stable emitted - values, not key images)
    __device__ __forceinline__ void read(bool side_b, int64_t at, K* key, uint32_t* val, bool values = false) const {
        if (!side_b) {
            *key = ak[at];
            if constexpr (PAIRS) *val = av[at];
            return;
        }
        if constexpr (PAIRS) {
            *val = idx64 ? static_cast<uint32_t>(static_cast<const int64_t*>(idx)[irow + at * si])
                         : static_cast<uint32_t>(static_cast<const int32_t*>(idx)[irow + at * si]);
            *key = yrow ? yrow[at * sy] : image_of(xrow[static_cast<int64_t>(*val) * sx]);
        } else {
            *key = yrow[at * sy];
        }
        if (values && yrow) *key = image_of(*key);
    }
    __device__ __forceinline__ void write(bool side_b, int64_t at, K key, uint32_t val) const {
        if (!side_b) {
            ak[at] = key;
            if constexpr (PAIRS) av[at] = val;
            return;
        }
        if (yrow) yrow[at * sy] = key;
        if constexpr (PAIRS) {
            if (idx64) static_cast<int64_t*>(idx)[irow + at * si] = static_cast<int64_t>(val);
            else static_cast<int32_t*>(idx)[irow + at * si] = static_cast<int32_t>(val);
        }
    }
    // entry `at` of the sorted row leaves for good
    __device__ __forceinline__ void emit(int64_t at, K key, uint32_t val) const {
        if (yrow) {
            K bits = decode_key<K>(key, kind, descending);
            if constexpr (PAIRS) {
                if (restore_zero && static_cast<K>(bits << 1) == 0) bits = xrow[static_cast<int64_t>(val) * sx];
            }
            yrow[at * sy] = bits;
        }
        if constexpr (PAIRS) {
            if (idx) {
                if (idx64) static_cast<int64_t*>(idx)[irow + at * si] = static_cast<int64_t>(val);
                else static_cast<int32_t*>(idx)[irow + at * si] = static_cast<int32_t>(val);
            }
        }
    }
};

// Returns false, having done nothing, for the one case it does not take: an index-only argsort
// whose index output overwrites the input (side B cannot hold keys and they cannot be read again
// either); the caller then sorts the bucket where it lies.
template <typename K, bool PAIRS, int WAVES>
__device__ __forceinline__ bool sort_oversized(SmallShared<K, PAIRS, kFinishItems, WAVES>& sm, const PassIo<K>& io, int64_t n, int64_t row, int64_t begin, int64_t size, bool in_b,
                                               unsigned long long ors, unsigned long long ands, const K* xrow, K* yrow, int64_t irow) {
    constexpr int ITEMS = kFinishItems;
    constexpr int T = WAVES * kWave;
    constexpr int WINDOW = T * ITEMS;
    __shared__ uint32_t digit_at[kRadix];              // where the next entry of each digit goes
    const int tid = threadIdx.x;
    const int lane = lane_id();
    const int w = tid / kWave;
    const int seg = w * kWave * ITEMS + lane;
    OversizedIo<K, PAIRS> mem{xrow, yrow, PAIRS ? io.idx : nullptr, irow, io.sx, io.sy, io.si, io.idx64, io.kind, io.descending, io.canon_zero,
                              io.restore_zero, io.kbuf[0] + row * n, PAIRS ? io.vbuf[0] + row * n : nullptr};
    const bool x_intact = io.x_intact != 0;

    // ---- the bits that differ inside the bucket (split_pass_stable gathered its keys' OR and AND)
    const K all = static_cast<K>(ands);
    const K differ = static_cast<K>(static_cast<K>(ors) & ~all);
    constexpr int U = WAVES >= 16 ? 2 : 8;             // entries in flight a thread where the bucket is only streamed
    int passes = 0;
    for (int p = 0; p < KeyTraits<K>::kPasses; ++p) passes += (static_cast<uint32_t>(differ >> (8 * p)) & 0xffu) != 0u ? 1 : 0;

    auto emit = [&](int64_t at, K k1, uint32_t v1) __attribute__((always_inline)) { mem.emit(at, k1, v1); };
    if (passes == 0) {                                 // one value: pairs are in index order already
        if (in_b) return true;
        for (int64_t i = tid; i < size; i += T) {
            K k1;
            uint32_t v1 = 0;
            mem.read(false, begin + i, &k1, &v1);
            emit(begin + i, k1, v1);
        }
        return true;
    }
    if (PAIRS && !mem.yrow && !x_intact) return false;

    bool from_b = in_b, b_values = in_b;               // (values: side B still holds what split_pass_stable emitted)
    if ((passes % 2 == 0) != in_b) {                   // so that the last pass goes from A to B
        for (int64_t i0 = 0; i0 < size; i0 += U * T) {
            K k1[U];
            uint32_t v1[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int64_t i = i0 + u * T + tid;
                v1[u] = 0u;
                mem.read(from_b, begin + (i < size ? i : 0), &k1[u], &v1[u], b_values);
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int64_t i = i0 + u * T + tid;
                if (i < size) mem.write(!from_b, begin + i, k1[u], v1[u]);
            }
        }
        from_b = !from_b;
        b_values = false;
        __syncthreads();
    }
    int left = passes;
    for (int p = 0; p < KeyTraits<K>::kPasses; ++p) {
        const int shift = 8 * p;
        const uint32_t vary = static_cast<uint32_t>(differ >> shift) & 0xffu;
        if (vary == 0u) continue;
        const bool last = --left == 0;
        // ---- how many entries carry each digit, and from that where each digit's run starts
        for (int i = tid; i < kRadix; i += T) digit_at[i] = 0u;
        __syncthreads();
        for (int64_t i0 = 0; i0 < size; i0 += U * T) {
            K k1[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int64_t i = i0 + u * T + tid;
                uint32_t v1 = 0;
                mem.read(from_b, begin + (i < size ? i : 0), &k1[u], &v1, b_values);
            }
#pragma unroll
            for (int u = 0; u < U; ++u)
                if (i0 + u * T + tid < size) atomicAdd(&digit_at[static_cast<uint32_t>(k1[u] >> shift) & 0xffu], 1u);
        }
        __syncthreads();
        {
            const uint32_t count = tid < kRadix ? digit_at[tid] : 0u;
            const uint32_t incl = wave_scan_inclusive(count, 0u, [](uint32_t a, uint32_t b) { return a + b; });
            if (tid < kRadix && lane == kWave - 1) sm.scan_tmp[w] = incl;
            __syncthreads();
            if (tid < kRadix) {
                uint32_t run = incl - count;
                for (int i = 0; i < w; ++i) run += sm.scan_tmp[i];
                digit_at[tid] = run;
            }
        }
        // ---- window by window, in order: stable ranks inside the window, runs carried along
        for (int64_t lo = 0; lo < size; lo += WINDOW) {
            for (int i = tid; i < WAVES * kRadix; i += T) (&sm.wave_hist[0][0])[i] = 0u;
            K key[ITEMS];
            uint32_t val[PAIRS ? ITEMS : 1];
            uint32_t digit[ITEMS], rank[ITEMS];
#pragma unroll
            for (int k = 0; k < ITEMS; ++k) {
                const int64_t e = lo + seg + k * kWave;
                key[k] = all;                          // padding agrees with the bucket in every bit that does not vary
                if constexpr (PAIRS) val[k] = 0u;
                if (e < size) mem.read(from_b, begin + e, &key[k], &val[PAIRS ? k : 0], b_values);
                digit[k] = static_cast<uint32_t>(key[k] >> shift) & 0xffu;
            }
            __syncthreads();                           // zeroed counts and digit_at are in place
            rank_by_digit<ITEMS>(sm.wave_hist[w], digit, vary, rank);
            __syncthreads();
            if (tid < kRadix) {
                uint32_t run = digit_at[tid];
#pragma unroll
                for (int i = 0; i < WAVES; ++i) {
                    const uint32_t count = sm.wave_hist[i][tid];
                    sm.wave_hist[i][tid] = run;
                    run += count;
                }
                digit_at[tid] = run;                   // (padding of the last window counts too: never used again)
            }
            __syncthreads();
#pragma unroll
            for (int k = 0; k < ITEMS; ++k) {
                if (lo + seg + k * kWave < size) {
                    const int64_t at = begin + sm.wave_hist[w][digit[k]] + rank[k];
                    if (last) emit(at, key[k], PAIRS ? val[k] : 0u);
                    else mem.write(!from_b, at, key[k], PAIRS ? val[k] : 0u);
                }
            }
            __syncthreads();
        }
        from_b = !from_b;
        b_values = false;
    }
    return true;
}

// The buckets split_finish left: stable digit passes on chip - for pairs first by index (the
// entries arrive in no particular order), then by key - and the buckets larger than a workgroup
// holds, which split_plan put on the same list, an entry per window of kOverWindow entries.
//
// split_pass_stable left the smallest and the largest key of every oversized bucket: when they
// are equal - one repeated value, whose pairs arrived in index order - every window of the bucket
// is copied out as it lies, by as many workgroups as the bucket has windows; otherwise the
// workgroup that draws the bucket's first window sorts it whole (sort_oversized).
template <typename K, bool PAIRS, int WAVES>
__global__ __launch_bounds__(WAVES * kWave) void split_finish_crowded(PassIo<K> io, int64_t n, const SplitRow* __restrict__ infos,
                                                                     const uint32_t* __restrict__ counters, CrowdedList crowded) {
    constexpr int ITEMS = kFinishItems;
    constexpr int T = WAVES * kWave;
    __shared__ SmallShared<K, PAIRS, ITEMS, WAVES> sm;
    const uint32_t listed = counters[1];
    const int lane = lane_id();
    const int seg = (threadIdx.x / kWave) * kWave * ITEMS + lane;
    for (uint32_t i = blockIdx.x; i < listed; i += gridDim.x) {
        const uint2 item = crowded.items[i];
        const uint4 at = bucket_at(infos, item.x);
        const int64_t at_row = at.x, at_begin = at.y;
        if (item.y != kNoWindow) {
            const int64_t size = at.z;
            const K* ak = io.kbuf[0] + at_row * n + at_begin;
            const uint32_t* av = PAIRS ? io.vbuf[0] + at_row * n + at_begin : nullptr;
            const K* xrow = io.x + io.xmap.at(at_row);
            K* yrow = io.y ? io.y + io.ymap.at(at_row) : nullptr;
            const int64_t irow = (PAIRS && io.idx) ? io.imap.at(at_row) : 0;
            if (static_cast<K>(crowded.range[2 * item.x]) != static_cast<K>(crowded.range[2 * item.x + 1])) {
                if (item.y == 0u) {
                    (void)sort_oversized<K, PAIRS, WAVES>(sm, io, n, at_row, at_begin, size, io.x_intact != 0, crowded.range[2 * item.x], crowded.range[2 * item.x + 1], xrow, yrow, irow);      // (what it does not take: split_finish_in_place)
                    __syncthreads();
                }
                continue;
            }
            if (io.x_intact) continue;                 // one value, and split_pass_stable wrote it to the outputs
            const int64_t lo = static_cast<int64_t>(item.y) * kOverWindow;
            const int64_t hi = lo + kOverWindow < size ? lo + kOverWindow : size;
            constexpr int U = WAVES >= 16 ? 2 : 8;                     // entries in flight a thread (the registers of 1024 threads allow two)
            for (int64_t e0 = lo; e0 < hi; e0 += U * T) {
                K key[U];
                uint32_t val[PAIRS ? U : 1];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int64_t e = e0 + u * T + threadIdx.x;
                    key[u] = ak[e < hi ? e : lo];
                    if constexpr (PAIRS) val[u] = av[e < hi ? e : lo];
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int64_t e = e0 + u * T + threadIdx.x;
                    if (e < hi) emit_entry<K, PAIRS>(io, xrow, yrow, irow, at_begin + e, key[u], PAIRS ? val[u] : 0u);
                }
            }
            continue;
        }
        const int valid = static_cast<int>(at.z);
        const K* src = io.kbuf[0] + at_row * n + at_begin;
        const uint32_t* vsrc = PAIRS ? io.vbuf[0] + at_row * n + at_begin : nullptr;
        K key[ITEMS];
        uint32_t val[PAIRS ? ITEMS : 1];
        K ors = 0, ands = ~K(0), vors = 0, vands = ~K(0);
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) {
            const int e = seg + k * kWave;
            key[k] = ~K(0);                                    // padding sorts last, by index and by key
            if constexpr (PAIRS) val[k] = ~0u;
            if (e < valid) {
                key[k] = src[e];
                ors |= key[k];
                ands &= key[k];
                if constexpr (PAIRS) {
                    val[k] = vsrc[e];
                    vors |= static_cast<K>(val[k]);
                    vands &= static_cast<K>(val[k]);
                }
            }
        }
        if constexpr (PAIRS) {
            sort_in_workgroup<K, PAIRS, ITEMS, WAVES, true>(sm, key, val, vors, vands, valid, 4);
            __syncthreads();
        }
        sort_in_workgroup<K, PAIRS, ITEMS, WAVES>(sm, key, val, ors, ands, valid, KeyTraits<K>::kPasses);
        const K* xrow = io.x + io.xmap.at(at_row);
        K* yrow = io.y ? io.y + io.ymap.at(at_row) : nullptr;
        const int64_t irow = (PAIRS && io.idx) ? io.imap.at(at_row) : 0;
#pragma unroll
        for (int k = 0; k < ITEMS; ++k)
            if (seg + k * kWave < valid) emit_entry<K, PAIRS>(io, xrow, yrow, irow, at_begin + seg + k * kWave, key[k], PAIRS ? val[k] : 0u);
        __syncthreads();
    }
}

// The oversized buckets of several values that sort_oversized leaves: an index-only argsort
// whose index output overwrites its input (the host launches this kernel for such calls only).
// The bucket is sorted where it lies - neighbouring halves of windows sorted together on chip,
// odd and even pairs in turn, as many rounds as there are halves - and then copied out: slow
// (the work grows with the square of the bucket), and only for this combination.
template <typename K, int WAVES>
__global__ __launch_bounds__(WAVES * kWave) void split_finish_in_place(PassIo<K> io, int64_t n, const SplitRow* __restrict__ infos,
                                                                      const uint32_t* __restrict__ counters, CrowdedList crowded) {
    constexpr int ITEMS = kFinishItems;
    constexpr int T = WAVES * kWave, WINDOW = T * ITEMS, HALF = WINDOW / 2;
    __shared__ SmallShared<K, true, ITEMS, WAVES> sm;
    const uint32_t listed = counters[1];
    const int lane = lane_id();
    const int w = threadIdx.x / kWave;
    const int seg = w * kWave * ITEMS + lane;
    for (uint32_t i = blockIdx.x; i < listed; i += gridDim.x) {
        // the first window's entry stands for its bucket; a bucket of one value has been copied out
        const uint2 item = crowded.items[i];
        if (item.y != 0u || static_cast<K>(crowded.range[2 * item.x]) == static_cast<K>(crowded.range[2 * item.x + 1])) continue;
        const uint4 at = bucket_at(infos, item.x);
        const int64_t size = at.z;
        K* ak = io.kbuf[0] + static_cast<int64_t>(at.x) * n + at.y;
        uint32_t* av = io.vbuf[0] + static_cast<int64_t>(at.x) * n + at.y;
        const int64_t halves = (size + HALF - 1) / HALF;
#pragma unroll 1
        for (int64_t round = 0; round < halves; ++round) {
#pragma unroll 1
            for (int64_t h = round & 1; h < halves; h += 2) {
                const int64_t lo = h * HALF;
                const int valid = static_cast<int>(size - lo < WINDOW ? size - lo : WINDOW);
                if (valid <= HALF && round > 0) continue;       // a lone last half: sorted since the first round
                K key[ITEMS];
                uint32_t val[ITEMS];
                K ors = 0, ands = ~K(0), vors = 0, vands = ~K(0);
#pragma unroll
                for (int k = 0; k < ITEMS; ++k) {
                    const int e = seg + k * kWave;
                    key[k] = ~K(0);                            // padding sorts last, by index and by key
                    val[k] = ~0u;
                    if (e < valid) {
                        key[k] = ak[lo + e];
                        val[k] = av[lo + e];
                        ors |= key[k];
                        ands &= key[k];
                        vors |= static_cast<K>(val[k]);
                        vands &= static_cast<K>(val[k]);
                    }
                }
                sort_in_workgroup<K, true, ITEMS, WAVES, true>(sm, key, val, vors, vands, valid, 4);
                __syncthreads();
                sort_in_workgroup<K, true, ITEMS, WAVES>(sm, key, val, ors, ands, valid, KeyTraits<K>::kPasses);
#pragma unroll
                for (int k = 0; k < ITEMS; ++k) {
                    const int e = seg + k * kWave;
                    if (e < valid) {
                        ak[lo + e] = key[k];
                        av[lo + e] = val[k];
                    }
                }
                __syncthreads();
            }
        }
        const K* xrow = io.x + io.xmap.at(at.x);
        const int64_t irow = io.imap.at(at.x);
        for (int64_t e = threadIdx.x; e < size; e += T) emit_entry<K, true>(io, xrow, nullptr, irow, static_cast<int64_t>(at.y) + e, ak[e], av[e]);
        __syncthreads();
    }
}

struct SplitLayout {
    int64_t chunks_per_row;
    size_t counters_off, rows_off, list_off, crowded_off, state_off, fine_off, base_off, maps_off, total;
};

SplitLayout split_layout(int64_t m, int64_t n) {
    SplitLayout l;
    l.chunks_per_row = ceil_div(n, static_cast<int64_t>(kChunk));
    size_t off = 0;
    l.counters_off = off;        // [1] buckets on the list of split_finish_crowded, [2] on that of split_finish
    off += 256;
    l.rows_off = off;
    off += align_up(static_cast<size_t>(m) * sizeof(SplitRow), 256);
    l.list_off = off;            // {row, begin, size, id} of every bucket
    off += align_up(static_cast<size_t>(m) * kMaxBuckets * 16, 256);
    l.crowded_off = off;         // {id, window}: a bucket is crowded or oversized, and an oversized one has a window per kOverWindow entries
    static_assert(kOverWindow == kChunk, "as many windows a row as chunks, at most");
    off += align_up(static_cast<size_t>(m) * (kMaxBuckets + l.chunks_per_row) * 8, 256);
    l.state_off = off;           // OR and AND of the keys of every (oversized) bucket
    off += align_up(static_cast<size_t>(m) * kMaxBuckets * 16, 256);
    l.fine_off = off;            // fine-bin histogram of every chunk, two counts a word
    off += align_up(static_cast<size_t>(m) * l.chunks_per_row * (kFine / 2) * 4, 256);
    l.base_off = off;            // where every chunk writes each bucket
    off += align_up(static_cast<size_t>(m) * l.chunks_per_row * kMaxBuckets * 4, 256);
    l.maps_off = off;            // the maps of rows whose keys cluster
    off += align_up(static_cast<size_t>(m) * sizeof(PiecewiseMap), 256);
    l.total = off;
    return l;
}

}  // namespace

// Whether rows of n keys can take the bucket route at all (each row then decides on the device).
// (the longest rows: nine tenths of what 256 of the largest buckets hold - fine bins do not fill
// buckets to the brim, and a row that needs more buckets than there are gets oversized ones)
constexpr int64_t kLongestRow = static_cast<int64_t>(kMaxBuckets) * kCapHuge / 10 * 9;
bool split_route_takes(size_t key_size, int64_t m, int64_t n) {
    return (key_size == 4 || key_size == 8) && n <= kLongestRow &&
           m * kMaxBuckets <= 0x7fffffffLL && m * ceil_div(n, static_cast<int64_t>(kChunk)) <= 0x7fffffffLL;
}

size_t split_scratch_bytes(size_t key_size, bool pairs, int64_t m, int64_t n) {
    (void)key_size;
    (void)pairs;              // keys and indices travel through the caller's first ping-pong buffers
    return split_layout(m, n).total;
}

// Enqueues the bucket route, which sorts every row of the call; keys (and indices) travel through
// io.kbuf[0] (and io.vbuf[0]).
template <typename K>
int run_split(hipStream_t stream, const PassIo<K>& io, bool pairs, int64_t m, int64_t n, void* scratch, int compare_max) {
    const SplitLayout l = split_layout(m, n);
    char* base = static_cast<char*>(scratch);
    uint32_t* counters = reinterpret_cast<uint32_t*>(base + l.counters_off);
    SplitRow* rows = reinterpret_cast<SplitRow*>(base + l.rows_off);
    uint4* list = reinterpret_cast<uint4*>(base + l.list_off);
    const CrowdedList crowded = {reinterpret_cast<uint2*>(base + l.crowded_off), reinterpret_cast<unsigned long long*>(base + l.state_off)};
    uint32_t* fine = reinterpret_cast<uint32_t*>(base + l.fine_off);
    uint32_t* chunk_base = reinterpret_cast<uint32_t*>(base + l.base_off);
    PiecewiseMap* maps = reinterpret_cast<PiecewiseMap*>(base + l.maps_off);

    const int waves = finish_waves(n, io.kind == kKeyFloat);
    const int cap = finish_cap(waves);
    // Float rows beyond the smallest size may be spread by value (split_sample decides per row).
    // The smallest may have the gap around zero closed up once they are long enough for it to
    // pay: a quarter of a binade, the bin of an open gap, holds some 4 % of a bell-shaped row -
    // not much beside a bucket while the row has under a dozen buckets' worth of keys, and the
    // finer bins of the closed gap would only split the thin tails into many small buckets
    // (measured on normal rows: open gap ahead up to 24 000 keys, closed from 32 768).
    // Doubles always: their sign and exponent alone fill the 12 bits of a fine bin's number, so with
    // the gap open a row on both sides of zero has one bin to a binade or less, and a bell-shaped
    // row a bin fuller than a bucket (N(0,1) doubles, rows of 10 000: 15 Gkeys/s with the gap open).
    const int map = io.kind != kKeyFloat ? kMapPlain : waves > 4 ? kMapValue : (sizeof(K) == 8 || n >= 12 * static_cast<int64_t>(cap)) ? kMapGap : kMapPlain;
    auto with_map = [&](auto&& launch_with) {
        if (map == kMapPlain) launch_with(std::integral_constant<int, kMapPlain>());
        else if (map == kMapGap) launch_with(std::integral_constant<int, kMapGap>());
        else launch_with(std::integral_constant<int, kMapValue>());
    };
    // Many rows of 4-byte keys that take the smallest buckets: one workgroup makes a row's plan and
    // moves the row (split_front); otherwise the steps are launches of their own, a workgroup a chunk.
    const bool front = sizeof(K) == 4 && waves == 4 && m >= kFrontRows;
    if (!front) {
        with_map([&](auto map_tag) {
            split_sample<K, decltype(map_tag)::value><<<dim3(static_cast<unsigned>(m)), dim3(kSplitBlock), 0, stream>>>(io, n, static_cast<uint32_t>(cap), rows, counters);
        });
        DLFX_CHECK_LAUNCH();
    } else {
        split_clear<<<dim3(1), dim3(kWave), 0, stream>>>(counters);
        DLFX_CHECK_LAUNCH();
    }
    const dim3 chunks(static_cast<unsigned>(m * l.chunks_per_row));
    // rows whose keys cluster get their maps (as a rule none: every workgroup leaves at once)
    auto remap_rows = [&]() -> int {
        split_remap<K><<<dim3(static_cast<unsigned>(m < 1024 ? m : 1024)), dim3(kSplitBlock), 0, stream>>>(io, m, n, rows, counters, maps);
        DLFX_CHECK_LAUNCH();
        return DLFX_OK;
    };
    if (!front) {
        const int status = remap_rows();
        if (status != DLFX_OK) return status;
        with_map([&](auto map_tag) {
            split_histogram<K, decltype(map_tag)::value><<<chunks, dim3(kSplitBlock), 0, stream>>>(io, n, l.chunks_per_row, rows, fine, maps);
        });
        DLFX_CHECK_LAUNCH();
        const size_t per_chunk_bytes = static_cast<size_t>(l.chunks_per_row) * kMaxBuckets * sizeof(uint32_t);      // (at most 80 chunks: 80 KB)
        if (l.chunks_per_row <= kPlanChunks)
            split_plan<kSplitBlock><<<dim3(static_cast<unsigned>(m)), dim3(kSplitBlock), per_chunk_bytes, stream>>>(n, static_cast<uint32_t>(cap), l.chunks_per_row, fine, rows, counters, list, crowded, chunk_base);
        else
            split_plan<1024><<<dim3(static_cast<unsigned>(m)), dim3(1024), per_chunk_bytes, stream>>>(n, static_cast<uint32_t>(cap), l.chunks_per_row, fine, rows, counters, list, crowded, chunk_base);
        DLFX_CHECK_LAUNCH();
    }
    // split_finish: as many workgroups as the device holds at once, each walking its share of the buckets
    const int64_t buckets = m * kMaxBuckets;
    const uint32_t limit = static_cast<uint32_t>(compare_max);
    auto launch = [&](auto pairs_tag, auto waves_tag) -> int {
        constexpr bool PAIRS = decltype(pairs_tag)::value;
        constexpr int WAVES = decltype(waves_tag)::value;
        const int64_t finish_room = resident_workgroups(split_finish<K, PAIRS, WAVES>, WAVES * kWave);
        if (finish_room <= 0) return DLFX_ERR_LAUNCH;
        const dim3 fgrid(static_cast<unsigned>(buckets < finish_room ? buckets : finish_room));
        const int block = pass_block<K, PAIRS>(n, cap);
        auto pass_of = [&](auto block_tag) {
            constexpr int BLOCK = decltype(block_tag)::value;
            with_map([&](auto map_tag) {
                constexpr int MAP = decltype(map_tag)::value;
                if constexpr (sizeof(K) == 4 && WAVES == 4 && MAP != kMapValue && BLOCK <= 512) {
                    if (front) {
                        split_front<K, PAIRS, BLOCK, MAP><<<dim3(static_cast<unsigned>(m)), dim3(BLOCK), 0, stream>>>(
                            io, n, static_cast<uint32_t>(cap), rows, counters, list, crowded);
                        return;
                    }
                }
                split_pass<K, PAIRS, BLOCK, MAP><<<chunks, dim3(BLOCK), 0, stream>>>(io, n, l.chunks_per_row, rows, chunk_base);
            });
        };
        if (block == 256) pass_of(std::integral_constant<int, 256>());
        else if (block == 512) pass_of(std::integral_constant<int, 512>());
        else if constexpr (kPassBlockMax<K, PAIRS> >= 1024) pass_of(std::integral_constant<int, 1024>());
        DLFX_CHECK_LAUNCH();
        if (front) {
            split_replan<K><<<dim3(static_cast<unsigned>(m < 1024 ? m : 1024)), dim3(kSplitBlock), 0, stream>>>(
                io, m, n, static_cast<uint32_t>(cap), rows, counters, list, crowded, maps);
            DLFX_CHECK_LAUNCH();
        }
        {
            // rows with buckets larger than a workgroup holds (as a rule none: every workgroup leaves at once)
            const int64_t units = front ? m : m * l.chunks_per_row;
            split_pass_stable<K, PAIRS><<<dim3(static_cast<unsigned>(units < 1024 ? units : 1024)), dim3(kStableBlock), 0, stream>>>(
                io, n, static_cast<uint32_t>(cap), l.chunks_per_row, units, rows, counters, front ? nullptr : chunk_base, crowded.range, maps);
            DLFX_CHECK_LAUNCH();
        }
        split_finish<K, PAIRS, WAVES><<<fgrid, dim3(WAVES * kWave), 0, stream>>>(io, n, limit, counters, list, crowded.items);
        DLFX_CHECK_LAUNCH();
        // (a smaller grid for this launch, which as a rule finds little to do, was measured: the
        // same for the benchmark rows, up to 15 % slower on bell-shaped rows, whose buckets are often crowded)
        split_finish_crowded<K, PAIRS, WAVES><<<fgrid, dim3(WAVES * kWave), 0, stream>>>(io, n, rows, counters, crowded);
        DLFX_CHECK_LAUNCH();
        if constexpr (PAIRS) {
            if (!io.y && !io.x_intact) {       // what sort_oversized cannot take (an index-only argsort written over its input)
                split_finish_in_place<K, WAVES><<<fgrid, dim3(WAVES * kWave), 0, stream>>>(io, n, rows, counters, crowded);
                DLFX_CHECK_LAUNCH();
            }
        }
        return DLFX_OK;
    };
    using Huge = std::integral_constant<int, 16>;
    using Large = std::integral_constant<int, 8>;
    using Small = std::integral_constant<int, 4>;
    if (pairs) return waves == 4 ? launch(std::true_type(), Small()) : waves == 8 ? launch(std::true_type(), Large()) : launch(std::true_type(), Huge());
    return waves == 4 ? launch(std::false_type(), Small()) : waves == 8 ? launch(std::false_type(), Large()) : launch(std::false_type(), Huge());
}

template int run_split<uint32_t>(hipStream_t, const PassIo<uint32_t>&, bool, int64_t, int64_t, void*, int);
template int run_split<uint64_t>(hipStream_t, const PassIo<uint64_t>&, bool, int64_t, int64_t, void*, int);

}  // namespace dlfx

#ifdef SPLIT_TIMING
extern "C" void dlfx_debug_split_phases(unsigned long long* out, int reset) {
    static unsigned long long host[dlfx::kPhaseSlots * 16];
    if (out) {
        (void)hipMemcpyFromSymbol(host, HIP_SYMBOL(dlfx::g_split_cycles), sizeof(host));
        for (int i = 0; i < 16; ++i) out[i] = 0;
        for (int b = 0; b < dlfx::kPhaseSlots; ++b)
            for (int i = 0; i < 16; ++i) out[i] += host[b * 16 + i];
    }
    if (reset) {
        for (auto& v : host) v = 0;
        (void)hipMemcpyToSymbol(HIP_SYMBOL(dlfx::g_split_cycles), host, sizeof(host));
    }
}
#endif
