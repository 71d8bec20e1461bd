// scan (cumsum / cumprod / cummax / cummin) over strided views for gfx950.
//
// Two kernels:
//   * scan_rows: the scanned axis is walked by whole workgroups.  A row is cut
//     into tiles of 256 x ITEMS elements; every tile is read once and written
//     once.  Inside a tile each wave owns a contiguous segment that it loads
//     with 128-bit accesses and scans with DPP row shifts / broadcasts; tiles of
//     one row are chained with decoupled look-back (aggregate / inclusive-prefix
//     words published with agent-scope atomics).  Waits when the output does not
//     overlap the input are bounded by a poll limit: a tile that polled a
//     predecessor's state too long computes that predecessor's aggregate from
//     the input itself, and a tile that polled too long for the word that says
//     a slice of states has been cleared reads and publishes no state of that
//     slice (its predecessors there are folded from the input, its successors
//     time out on it the same way).  When the output does overlap the input
//     (in-place scan) tile numbers are drawn from a per-row atomic ticket, so a
//     tile only waits for tiles that are running; that wait has no limit.
//   * scan_cols: many rows, scanned axis strided, a kept axis contiguous (e.g.
//     cumsum over C of NCHW).  Lanes run along the kept axis so each load is a
//     contiguous segment, the four waves of a workgroup take consecutive
//     chunks of the scanned axis and exchange chunk totals through LDS.
#include <atomic>
#include <chrono>
#include <cstring>
#include <limits>
#include <type_traits>

#include <unistd.h>

#include "common.hip.h"

namespace dlfx {
namespace {

enum ScanKind { kScanAdd = 0, kScanMul = 1, kScanMax = 2, kScanMin = 3 };
constexpr int kBlock = 256;
constexpr int kWaves = kBlock / kWave;

template <typename T, int K>
struct ScanOp {
    __device__ static __forceinline__ T identity() {
        if constexpr (K == kScanAdd) return T(0);
        else if constexpr (K == kScanMul) return T(1);
        else if constexpr (K == kScanMax) return std::numeric_limits<T>::lowest();
        else return std::numeric_limits<T>::max();
    }
    __device__ static __forceinline__ T apply(T a, T b) {
        if constexpr (K == kScanAdd) {
            if constexpr (std::is_integral<T>::value) {
                using U = typename std::make_unsigned<T>::type;
                return static_cast<T>(static_cast<U>(a) + static_cast<U>(b));
            } else return a + b;
        } else if constexpr (K == kScanMul) {
            if constexpr (std::is_integral<T>::value) {
                using U = typename std::make_unsigned<T>::type;
                return static_cast<T>(static_cast<U>(a) * static_cast<U>(b));
            } else return a * b;
        } else if constexpr (K == kScanMax) {
            return (a < b) ? b : a;
        } else {
            return (b < a) ? b : a;
        }
    }
};

// ------------------------------------------------------------------ look-back state
constexpr uint32_t kInvalid = 0, kAggregate = 1, kInclusive = 2;
// polls of one predecessor's state before a tile stops waiting for it (dlfx_set_tuning "scan_poll_limit")
int g_poll_limit = 2048;

// 4-byte values travel with their flag in one 64-bit word.
template <typename T, int SIZE = sizeof(T)>
struct TileState;

template <typename T>
struct TileState<T, 4> {
    unsigned long long* words;
    static size_t bytes(int64_t tiles) { return static_cast<size_t>(tiles) * 8; }
    __host__ __device__ void bind(void* base, int64_t) { words = static_cast<unsigned long long*>(base); }
    __device__ __forceinline__ void clear(int64_t i) { words[i] = 0ull; }
    // the same from inside the launch that goes on to use the states
    __device__ __forceinline__ void clear_shared(int64_t i) { __hip_atomic_store(&words[i], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
    __device__ __forceinline__ void publish(int64_t i, uint32_t flag, T v) {
        unsigned long long w = (static_cast<unsigned long long>(flag) << 32) | bit_cast<uint32_t>(v);
        __hip_atomic_store(&words[i], w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __device__ __forceinline__ uint32_t read(int64_t i, T* v) {
        unsigned long long w = __hip_atomic_load(&words[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *v = bit_cast<T>(static_cast<uint32_t>(w));
        return static_cast<uint32_t>(w >> 32);
    }
};

// 8- and 16-byte values: one 64-bit word per 32 bits of the value, each carrying the flag in
// its upper half, all written and read with relaxed atomics (no fences, so no cache
// write-backs or invalidations on the polling path).  A value is taken only when all of its
// words carry the same flag: every state of a tile is written once and the states follow one
// another, so equal flags mean the words belong to one state; anything else reads as "not
// there yet" and is polled again.
template <typename T, int WORDS>
struct TileStateWords {
    struct Parts {
        uint32_t w[WORDS];
    };
    unsigned long long* words;
    static size_t bytes(int64_t tiles) { return static_cast<size_t>(tiles) * WORDS * 8; }
    __host__ __device__ void bind(void* base, int64_t) { words = static_cast<unsigned long long*>(base); }
    __device__ __forceinline__ void clear(int64_t i) {
#pragma unroll
        for (int k = 0; k < WORDS; ++k) words[i * WORDS + k] = 0ull;
    }
    __device__ __forceinline__ void clear_shared(int64_t i) {
#pragma unroll
        for (int k = 0; k < WORDS; ++k) __hip_atomic_store(&words[i * WORDS + k], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __device__ __forceinline__ void publish(int64_t i, uint32_t flag, T v) {
        const Parts p = bit_cast<Parts>(v);
#pragma unroll
        for (int k = 0; k < WORDS; ++k)
            __hip_atomic_store(&words[i * WORDS + k], (static_cast<unsigned long long>(flag) << 32) | p.w[k], __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
    }
    __device__ __forceinline__ uint32_t read(int64_t i, T* v) {
        unsigned long long w[WORDS];
#pragma unroll
        for (int k = 0; k < WORDS; ++k) w[k] = __hip_atomic_load(&words[i * WORDS + k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const uint32_t f = static_cast<uint32_t>(w[0] >> 32);
        Parts p;
        bool whole = true;
#pragma unroll
        for (int k = 0; k < WORDS; ++k) {
            whole = whole && static_cast<uint32_t>(w[k] >> 32) == f;
            p.w[k] = static_cast<uint32_t>(w[k]);
        }
        if (!whole) return kInvalid;
        *v = bit_cast<T>(p);
        return f;
    }
};
template <typename T> struct TileState<T, 8> : TileStateWords<T, 2> {};
template <typename T> struct TileState<T, 16> : TileStateWords<T, 4> {};

template <typename T>
__global__ __launch_bounds__(kBlock) void scan_init(unsigned* ticket, int64_t rows, TileState<T> st, int64_t tiles) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (i < rows) ticket[i] = 0u;
    if (i < tiles) st.clear(i);
}

// Tile states cleared by the scan launch itself.  The states are cut into slices of kSliceTiles;
// workgroup s of the launch clears slice s before anything else and then stores the call's
// nonce into ready[s].  A state is published, or read, only once its slice's word has been seen
// to hold the nonce: what the scratch held before the call (anything) cannot pass for a state
// of this call.  Workgroup s never waits before it clears and the host takes this path only when
// the clearing workgroups are fewer than the device holds at once, so they should all be running
// when any tile asks; nothing in HIP promises the order in which workgroups start, though, so
// the wait gives up after `limit` polls and the tile then leaves that slice's states alone
// (scan_tile).  The nonce is a kernel argument: a recorded launch replayed from a graph would
// meet its own nonce from the replay before, so launches under stream capture clear the states
// with a launch of their own (ready == nullptr), as do in-place scans, whose tickets need
// clearing too.
constexpr int64_t kSliceTiles = 1024;
struct ClearedBy {
    unsigned long long* ready;
    unsigned long long nonce;
    __device__ __forceinline__ bool seen(int64_t slice) const {
        return __hip_atomic_load(&ready[slice], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == nonce;
    }
    // True once slice `slice` is known to be cleared (`early` is an earlier load of its word),
    // false when `limit` polls did not show it.
    __device__ __forceinline__ bool await(int64_t slice, unsigned long long early, int limit) const {
        if (early != nonce) {
            int polls = 0;
            while (!seen(slice)) {
                if (polls++ >= limit) return false;
                __builtin_amdgcn_s_sleep(1);
            }
        }
        // What follows are agent-scope atomics on the states, which go to the same coherence
        // point as this load and are issued after it has returned (every later access depends on
        // the branch above): the compiler alone has to keep them behind it (a cache-invalidating
        // agent-scope fence here costs more than the separate clearing launch did).
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        return true;
    }
};

// Elements per memory access: 16 bytes of the arithmetic type, or of the stored type when input
// and output are both 16-bit (half scans compute in fp32 but should still move 16 bytes at a time).
template <typename T, typename X, typename Y>
constexpr int scan_vec() { return (sizeof(X) == 2 && sizeof(Y) == 2) ? 8 : vec_width<T>(); }

// What a scan folds for an input element: the element itself, or (scan_nonzero,
// gpgpu/include/gdnn.h:131-136) one for every element that is not zero.
template <typename T, typename X, bool NZ>
__device__ __forceinline__ T scan_input(X x) {
    if constexpr (NZ) return x != X(0) ? T(1) : T(0);
    else return static_cast<T>(x);
}

// ------------------------------------------------------------------ row kernels
template <typename T>
struct RowScanShared {
    T wave_total[16];
    T tile_prefix;
    unsigned next_tile;
};

// One tile: tile `t` of row `row`.  Element order inside a tile: wave w owns
// [w*64*ITEMS, (w+1)*64*ITEMS); within it, vector k of lane l covers elements
// (k*64 + l)*V .. +V.  CHAINED tiles publish / look back through `st`.
template <typename T, int K, int ITEMS, bool CHAINED, bool SELF_HELP, int BLOCK = kBlock, typename X = T, bool NZ = false,
          typename Y = T, bool PAD = false>
__device__ __forceinline__ void scan_tile(
    const X* __restrict__ x, Y* __restrict__ y, const DimMap& xmap, const DimMap& ymap, int64_t sx, int64_t sy,
    const DimMap& xaxis, int64_t n, int64_t tiles_per_row, int exclusive, int64_t row, int64_t t, int poll_limit,
    TileState<T>& st, RowScanShared<T>& sm, const ClearedBy& cb = ClearedBy{nullptr, 0ull}, unsigned long long ready_early = 0ull) {
    // where element i of a row lives: i * sx, or (scan_nonzero over a flattened view whose
    // dimensions do not merge) wherever the row-major walk of `xaxis` puts it
    auto x_at = [&](int64_t i) -> int64_t {
        if constexpr (NZ) return xaxis.at(i);
        else return i * sx;
    };
    using Op = ScanOp<T, K>;
    constexpr int V = (scan_vec<T, X, Y>() < ITEMS) ? scan_vec<T, X, Y>() : ITEMS;
    constexpr int KV = ITEMS / V;
    constexpr int64_t TILE = static_cast<int64_t>(BLOCK) * ITEMS;
    using VecX = Vec<X, V>;

    const int lane = lane_id();
    const int w = threadIdx.x / kWave;
    const int64_t tile_base = t * TILE;

    const X* xr = x + xmap.at(row);
    Y* yr = y + ymap.at(row);
    // A unit-stride row that does not start on a vector boundary (PAD: the host found such
    // rows) is tiled from the boundary before it: position j of that tiling is element
    // j - shift of the row, positions below `shift` hold the identity, and every whole vector
    // of the row is aligned in memory.  Elsewhere shift is 0 and positions are elements.
    const int shift = PAD ? static_cast<int>((reinterpret_cast<uintptr_t>(xr) / sizeof(X)) % V) : 0;
    const int64_t n_pos = n + shift;                       // positions of the row: [shift, n_pos)
    const int64_t seg = tile_base + static_cast<int64_t>(w) * kWave * ITEMS;

    // ---- load
    T vals[ITEMS];
    // whole vectors of an aligned unit-stride row move as one access; the row's first and last,
    // partial vectors (and what lies past the row in its last tile) element by element
    const bool x_vec = sx == 1 && (reinterpret_cast<uintptr_t>(xr - shift + seg) % (sizeof(X) * V) == 0);
    const VecX* pv = reinterpret_cast<const VecX*>(xr - shift + seg);
    const bool full = tile_base >= shift && n_pos - tile_base >= TILE;      // every position of the tile is an element of the row
    // A row walked backwards (stride -1: the reverse scans): elements [i, i + V) of the row are the
    // vector that ends at xr - i in memory, last element first.
    const bool x_rev = !PAD && sx == -1 && (reinterpret_cast<uintptr_t>(xr - seg - (V - 1)) % (sizeof(X) * V) == 0);
    const VecX* pr = reinterpret_cast<const VecX*>(xr - seg - (V - 1));
    if (full && x_vec) {
        // the common case apart: all loads issued back to back, nothing to test per vector
#pragma unroll
        for (int k = 0; k < KV; ++k) {
            VecX a = load_stream(&pv[k * kWave + lane]);
#pragma unroll
            for (int e = 0; e < V; ++e) vals[k * V + e] = scan_input<T, X, NZ>(a.v[e]);
        }
    } else if (full && x_rev) {
#pragma unroll
        for (int k = 0; k < KV; ++k) {
            VecX a = load_stream(pr - (k * kWave + lane));
#pragma unroll
            for (int e = 0; e < V; ++e) vals[k * V + e] = scan_input<T, X, NZ>(a.v[V - 1 - e]);
        }
    } else
#pragma unroll
    for (int k = 0; k < KV; ++k) {
        const int64_t i0 = seg + static_cast<int64_t>(k * kWave + lane) * V;
        if (x_vec && i0 >= shift && i0 + V <= n_pos) {
            VecX a = load_stream(&pv[k * kWave + lane]);
#pragma unroll
            for (int e = 0; e < V; ++e) vals[k * V + e] = scan_input<T, X, NZ>(a.v[e]);
        } else if (x_rev && i0 + V <= n_pos) {
            VecX a = load_stream(pr - (k * kWave + lane));
#pragma unroll
            for (int e = 0; e < V; ++e) vals[k * V + e] = scan_input<T, X, NZ>(a.v[V - 1 - e]);
        } else {
#pragma unroll
            for (int e = 0; e < V; ++e)
                vals[k * V + e] = (i0 + e >= shift && i0 + e < n_pos) ? scan_input<T, X, NZ>(xr[x_at(i0 + e - shift)]) : Op::identity();
        }
    }
    // ---- scan inside the wave: vals[] become inclusive prefixes within the wave segment
    T carry = Op::identity();
#pragma unroll
    for (int k = 0; k < KV; ++k) {
#pragma unroll
        for (int e = 1; e < V; ++e) vals[k * V + e] = Op::apply(vals[k * V + e - 1], vals[k * V + e]);
        const T lane_total = vals[k * V + V - 1];
        const T incl = wave_scan_inclusive(lane_total, Op::identity(), [](T a, T b) { return Op::apply(a, b); });
        T excl = lane_get(incl, lane - 1 < 0 ? 0 : lane - 1);
        if (lane == 0) excl = Op::identity();
        const T base = Op::apply(carry, excl);
#pragma unroll
        for (int e = 0; e < V; ++e) vals[k * V + e] = Op::apply(base, vals[k * V + e]);
        carry = Op::apply(carry, lane_read(incl, kWave - 1));
    }
    if (lane == 0) sm.wave_total[w] = carry;
    __syncthreads();

    T wave_prefix = Op::identity();
    T aggregate = Op::identity();
#pragma unroll
    for (int i = 0; i < BLOCK / kWave; ++i) {
        const T wt = sm.wave_total[i];
        if (i < w) wave_prefix = Op::apply(wave_prefix, wt);
        aggregate = Op::apply(aggregate, wt);
    }

    // ---- chain tiles of this row
    T tile_prefix = Op::identity();
    if (CHAINED) {
        if (w == 0) {
            const int64_t sbase = row * tiles_per_row;
            // States [cleared_from, this tile's] are known to be cleared (when this launch clears
            // them itself); states below dead_below are never read: the word of their slice did
            // not show the nonce in time, so whatever they hold may be older than this call.
            int64_t cleared_from = 0, dead_below = 0;
            bool publishes = true;
            if (cb.ready) {
                const int64_t slice = (sbase + t) / kSliceTiles;
                if (cb.await(slice, ready_early, poll_limit)) {
                    cleared_from = slice * kSliceTiles;
                } else {
                    // not even this tile's own slice: nothing is published (the slice's clearing
                    // would wipe it or, worse, come first and leave it) and every predecessor
                    // is folded from the input
                    publishes = false;
                    cleared_from = dead_below = sbase + t;
                }
            }
            if (lane == 0 && publishes) st.publish(sbase + t, t == 0 ? kInclusive : kAggregate, aggregate);
            T excl = Op::identity();
            if (t > 0) {
                int64_t pos = t - 1;
                for (;;) {
                    // the states this step of the look-back reads reach back to pos - 63 or to the row's first
                    const int64_t lowest = sbase + (pos >= kWave - 1 ? pos - (kWave - 1) : 0);
                    while (lowest < cleared_from && cleared_from > dead_below) {
                        const int64_t slice = (cleared_from - 1) / kSliceTiles;
                        if (cb.await(slice, 0ull, poll_limit)) cleared_from = slice * kSliceTiles;
                        else dead_below = cleared_from;
                    }
                    const int64_t idx = pos - lane;
                    T v = Op::identity();
                    uint32_t f = kInclusive;          // before the row: an inclusive identity
                    if (idx >= 0 && sbase + idx < dead_below) {
                        f = kInvalid;                  // (only with SELF_HELP: this launch clears its states only then)
                    } else if (idx >= 0) {
                        f = st.read(sbase + idx, &v);
                        if constexpr (SELF_HELP) {
                            for (int polls = 0; f == kInvalid && polls < poll_limit; ++polls) {
                                __builtin_amdgcn_s_sleep(1);
                                f = st.read(sbase + idx, &v);
                            }
                        } else {
                            while (f == kInvalid) {
                                __builtin_amdgcn_s_sleep(1);
                                f = st.read(sbase + idx, &v);
                            }
                        }
                    }
                    if constexpr (SELF_HELP) {
                        // predecessors that still have nothing published: fold their tile of
                        // the input here (the input is not being overwritten in this mode)
                        unsigned long long stuck = __ballot(f == kInvalid);
                        while (stuck != 0ull) {
                            const int l = __ffsll(static_cast<long long>(stuck)) - 1;
                            stuck &= stuck - 1;
                            const int64_t pfirst = (pos - l) * TILE;                       // positions [pfirst, pfirst + TILE)
                            const int64_t pbase = pfirst > shift ? pfirst - shift : 0;     // elements [pbase, pend)
                            const int64_t pend = pfirst + TILE - shift < n ? pfirst + TILE - shift : n;
                            T a = Op::identity();
                            for (int64_t i = pbase + lane; i < pend; i += kWave) a = Op::apply(a, scan_input<T, X, NZ>(xr[x_at(i)]));
                            a = wave_reduce(a, [](T p, T q) { return Op::apply(p, q); });
                            if (lane == l) {
                                v = a;
                                f = kAggregate;
                            }
                        }
                    }
                    const unsigned long long incl_mask = __ballot(f == kInclusive);
                    const int first = __ffsll(static_cast<long long>(incl_mask)) - 1;   // >= 0: some lane is inclusive
                    const T contrib = (first < 0 || lane <= first) ? v : Op::identity();
                    const T red = wave_reduce(contrib, [](T a, T b) { return Op::apply(a, b); });
                    excl = Op::apply(red, excl);
                    if (incl_mask != 0ull) break;
                    pos -= kWave;
                }
                if (lane == 0 && publishes) st.publish(sbase + t, kInclusive, Op::apply(excl, aggregate));
            }
            if (lane == 0) sm.tile_prefix = excl;
        }
        __syncthreads();
        tile_prefix = sm.tile_prefix;
    }

    // ---- combine and store
    const T pre = Op::apply(tile_prefix, wave_prefix);
    if (exclusive) {
        // element i receives the prefix of everything before it: shift by one element
        // inside the lane's vector, and take the previous lane / vector for e == 0
#pragma unroll
        for (int k = KV - 1; k >= 0; --k) {
            const T last = vals[k * V + V - 1];
            T prev = lane_get(last, lane - 1 < 0 ? 0 : lane - 1);
            T prev_vec_end = (k > 0) ? lane_read(vals[(k > 0 ? k - 1 : 0) * V + V - 1], kWave - 1) : Op::identity();
            if (lane == 0) prev = prev_vec_end;
#pragma unroll
            for (int e = V - 1; e > 0; --e) vals[k * V + e] = vals[k * V + e - 1];
            vals[k * V] = prev;
        }
    }
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) vals[i] = Op::apply(pre, vals[i]);

    using VecY = Vec<Y, V>;
    const bool y_vec = sy == 1 && (reinterpret_cast<uintptr_t>(yr - shift + seg) % (sizeof(Y) * V) == 0);
    VecY* qv = reinterpret_cast<VecY*>(yr - shift + seg);
    const bool y_rev = !PAD && sy == -1 && (reinterpret_cast<uintptr_t>(yr - seg - (V - 1)) % (sizeof(Y) * V) == 0);
    VecY* qr = reinterpret_cast<VecY*>(yr - seg - (V - 1));
    if (full && y_vec) {
#pragma unroll
        for (int k = 0; k < KV; ++k) {
            VecY a;
#pragma unroll
            for (int e = 0; e < V; ++e) a.v[e] = static_cast<Y>(vals[k * V + e]);
            store_stream(&qv[k * kWave + lane], a);
        }
    } else if (full && y_rev) {
#pragma unroll
        for (int k = 0; k < KV; ++k) {
            VecY a;
#pragma unroll
            for (int e = 0; e < V; ++e) a.v[V - 1 - e] = static_cast<Y>(vals[k * V + e]);
            store_stream(qr - (k * kWave + lane), a);
        }
    } else
#pragma unroll
    for (int k = 0; k < KV; ++k) {
        const int64_t i0 = seg + static_cast<int64_t>(k * kWave + lane) * V;
        if (y_vec && i0 >= shift && i0 + V <= n_pos) {
            VecY a;
#pragma unroll
            for (int e = 0; e < V; ++e) a.v[e] = static_cast<Y>(vals[k * V + e]);
            store_stream(&qv[k * kWave + lane], a);
        } else if (y_rev && i0 + V <= n_pos) {
            VecY a;
#pragma unroll
            for (int e = 0; e < V; ++e) a.v[V - 1 - e] = static_cast<Y>(vals[k * V + e]);
            store_stream(qr - (k * kWave + lane), a);
        } else {
#pragma unroll
            for (int e = 0; e < V; ++e)
                if (i0 + e >= shift && i0 + e < n_pos) yr[(i0 + e - shift) * sy] = static_cast<Y>(vals[k * V + e]);
        }
    }
}

// Rows of a single tile: workgroup b scans row b.
template <typename T, int K, int ITEMS, typename X, bool NZ, typename Y, bool PAD>
__global__ __launch_bounds__(kBlock) void scan_rows_single(
    const X* __restrict__ x, Y* __restrict__ y, DimMap xmap, DimMap ymap, int64_t sx, int64_t sy, DimMap xaxis,
    int64_t n, int exclusive) {
    __shared__ RowScanShared<T> sm;
    TileState<T> st;
    scan_tile<T, K, ITEMS, false, false, kBlock, X, NZ, Y, PAD>(x, y, xmap, ymap, sx, sy, xaxis, n, 1, exclusive, blockIdx.x, 0, 0, st, sm);
}

// Short rows: LANES lanes per row (one lane, a quad, a DPP row of 16 lanes, or a whole wavefront), ITEMS elements
// per lane in vectors of V, no workgroup barrier and no LDS; a 256-thread workgroup takes
// 256 / LANES rows.  Element (v * LANES + l) * V + j is item (v, j) of lane l of the group.
template <typename T, int K, int LANES, int ITEMS, typename X, bool NZ, typename Y>
__global__ __launch_bounds__(kBlock) void scan_rows_group(
    const X* __restrict__ x, Y* __restrict__ y, DimMap xmap, DimMap ymap, int64_t sx, int64_t sy,
    int64_t rows, int64_t n, int exclusive, int pad, int plain) {
    static_assert(LANES == 1 || LANES == 4 || LANES == 16 || LANES == kWave, "a thread, a quad, a DPP row or a wavefront");
    using Op = ScanOp<T, K>;
    constexpr int V0 = (scan_vec<T, X, Y>() < ITEMS) ? scan_vec<T, X, Y>() : ITEMS;
    constexpr int V = ITEMS % V0 == 0 ? V0 : V0 / 2;      // (12 items of a 16-bit type: vectors of 4)
    static_assert(ITEMS % V == 0, "whole vectors per lane");
    constexpr int KV = ITEMS / V;
    using VecX = Vec<X, V>;
    using VecY = Vec<Y, V>;
    const int lane = lane_id();
    const int l = lane & (LANES - 1);
    const int64_t row = (static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x) / LANES;
    const bool live = row < rows;                       // whole groups are live or not
    const X* xr = x + (live ? xmap.at(row) : 0);
    Y* yr = y + (live ? ymap.at(row) : 0);
    // a row that does not start on a vector boundary (pad != 0: the host found such rows) is laid
    // out from the boundary before it, as in scan_tile: position e is element e - shift
    const int shift = pad ? static_cast<int>((reinterpret_cast<uintptr_t>(xr) / sizeof(X)) % V) : 0;
    const int64_t count = live ? n + shift : 0;            // positions [shift, count) are the row

    // whole vectors of an aligned unit-stride row move as one access, the row's first and last,
    // partial vectors element by element
    const bool x_vec = sx == 1 && reinterpret_cast<uintptr_t>(xr - shift) % (sizeof(X) * V) == 0;
    const bool y_vec = sy == 1 && reinterpret_cast<uintptr_t>(yr - shift) % (sizeof(Y) * V) == 0;
    // a row walked backwards that ends on a vector boundary: whole vectors, last element first
    const bool x_rev = !pad && sx == -1 && reinterpret_cast<uintptr_t>(xr - (V - 1)) % (sizeof(X) * V) == 0;
    const bool y_rev = !pad && sy == -1 && reinterpret_cast<uintptr_t>(yr - (V - 1)) % (sizeof(Y) * V) == 0;
    T vals[ITEMS];
#pragma unroll
    for (int v = 0; v < KV; ++v) {
        const int64_t e0 = static_cast<int64_t>(v * LANES + l) * V;
        if (x_vec && e0 >= shift && e0 + V <= count) {
            // (plain: without the non-temporal hint, for rows that are not whole cache lines - where one access takes
            // part of a line and another the rest, the hint has the line fetched twice: fp32 [500000, 100] 82 -> 75 us)
            const VecX* from = reinterpret_cast<const VecX*>(xr - shift + e0);
            const VecX a = plain ? *from : load_stream(from);
#pragma unroll
            for (int j = 0; j < V; ++j) vals[v * V + j] = scan_input<T, X, NZ>(a.v[j]);
        } else if (x_rev && e0 + V <= count) {
            const VecX a = load_stream(reinterpret_cast<const VecX*>(xr - e0 - (V - 1)));
#pragma unroll
            for (int j = 0; j < V; ++j) vals[v * V + j] = scan_input<T, X, NZ>(a.v[V - 1 - j]);
        } else {
#pragma unroll
            for (int j = 0; j < V; ++j)
                vals[v * V + j] = (e0 + j >= shift && e0 + j < count) ? scan_input<T, X, NZ>(xr[(e0 + j - shift) * sx]) : Op::identity();
        }
    }
    auto combine = [](T a, T b) { return Op::apply(a, b); };
    T carry = Op::identity();
#pragma unroll
    for (int v = 0; v < KV; ++v) {
#pragma unroll
        for (int j = 1; j < V; ++j) vals[v * V + j] = Op::apply(vals[v * V + j - 1], vals[v * V + j]);
        const T lane_total = vals[v * V + V - 1];
        T incl;
        if constexpr (LANES == 1) {
            incl = lane_total;
        } else if constexpr (LANES == 4) {
            // shifts within a DPP row cross quads: what comes from another quad is dropped
            const T s1 = dpp_fetch<kRowShr1>(lane_total, Op::identity());
            incl = combine(l >= 1 ? s1 : Op::identity(), lane_total);
            const T s2 = dpp_fetch<kRowShr2>(incl, Op::identity());
            incl = combine(l >= 2 ? s2 : Op::identity(), incl);
        } else if constexpr (LANES == 16) {
            incl = combine(dpp_fetch<kRowShr1>(lane_total, Op::identity()), lane_total);
            incl = combine(dpp_fetch<kRowShr2>(incl, Op::identity()), incl);
            incl = combine(dpp_fetch<kRowShr4>(incl, Op::identity()), incl);
            incl = combine(dpp_fetch<kRowShr8>(incl, Op::identity()), incl);
        } else {
            incl = wave_scan_inclusive(lane_total, Op::identity(), combine);
        }
        T before = lane_get(incl, lane - 1 < 0 ? 0 : lane - 1);     // the lanes before this one in the group
        if (l == 0) before = Op::identity();
        const T base = Op::apply(carry, before);
        const T group_total = lane_get(incl, lane | (LANES - 1));
        if (exclusive) {
#pragma unroll
            for (int j = V - 1; j > 0; --j) vals[v * V + j] = Op::apply(base, vals[v * V + j - 1]);
            vals[v * V] = base;
        } else {
#pragma unroll
            for (int j = 0; j < V; ++j) vals[v * V + j] = Op::apply(base, vals[v * V + j]);
        }
        carry = Op::apply(carry, group_total);
    }
#pragma unroll
    for (int v = 0; v < KV; ++v) {
        const int64_t e0 = static_cast<int64_t>(v * LANES + l) * V;
        if (y_vec && e0 >= shift && e0 + V <= count) {
            VecY a;
#pragma unroll
            for (int j = 0; j < V; ++j) a.v[j] = static_cast<Y>(vals[v * V + j]);
            store_stream(reinterpret_cast<VecY*>(yr - shift + e0), a);
        } else if (y_rev && e0 + V <= count) {
            VecY a;
#pragma unroll
            for (int j = 0; j < V; ++j) a.v[V - 1 - j] = static_cast<Y>(vals[v * V + j]);
            store_stream(reinterpret_cast<VecY*>(yr - e0 - (V - 1)), a);
        } else {
#pragma unroll
            for (int j = 0; j < V; ++j)
                if (e0 + j >= shift && e0 + j < count) yr[(e0 + j - shift) * sy] = static_cast<Y>(vals[v * V + j]);
        }
    }
}

// Rows of several tiles.  Workgroup b belongs to row b / tiles_per_row.  With
// TICKET the tile of the row is drawn from that row's atomic counter (in-place
// scans); without, it is the workgroup's position in the row and waits are
// bounded by self-help.
template <typename T, int K, int ITEMS, bool TICKET, int BLOCK, typename X, bool NZ, typename Y, bool PAD>
__global__ __launch_bounds__(BLOCK) void scan_rows_chained(
    const X* __restrict__ x, Y* __restrict__ y, DimMap xmap, DimMap ymap, int64_t sx, int64_t sy, DimMap xaxis,
    int64_t n, int64_t tiles_per_row, int exclusive, int poll_limit, unsigned* ticket, TileState<T> st, ClearedBy cb) {
    __shared__ RowScanShared<T> sm;
    const int64_t row = blockIdx.x / tiles_per_row;
    int64_t t = blockIdx.x - row * tiles_per_row;
    unsigned long long ready_early = 0ull;
    if constexpr (!TICKET) {
        if (cb.ready) {
            const int64_t tiles = gridDim.x;
            if (static_cast<int64_t>(blockIdx.x) * kSliceTiles < tiles) {
                // this workgroup's slice of the states: cleared, made visible, announced
                for (int64_t i = threadIdx.x; i < kSliceTiles; i += BLOCK) {
                    const int64_t idx = static_cast<int64_t>(blockIdx.x) * kSliceTiles + i;
                    if (idx < tiles) st.clear_shared(idx);
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
                __syncthreads();
                if (threadIdx.x == 0) __hip_atomic_store(&cb.ready[blockIdx.x], cb.nonce, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
            }
            // asked for now, looked at when the tile has been loaded and scanned
            ready_early = __hip_atomic_load(&cb.ready[blockIdx.x / kSliceTiles], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    if constexpr (TICKET) {
        if (threadIdx.x == 0) sm.next_tile = atomicAdd(&ticket[row], 1u);
        __syncthreads();
        t = sm.next_tile;
    }
    scan_tile<T, K, ITEMS, true, !TICKET, BLOCK, X, NZ, Y, PAD>(x, y, xmap, ymap, sx, sy, xaxis, n, tiles_per_row, exclusive, row, t, poll_limit, st, sm,
                                                                TICKET ? ClearedBy{nullptr, 0ull} : cb, ready_early);
}

// ------------------------------------------------------------------ column kernel
// One lane per row ("column"), four waves along the scanned axis.  Each pass of
// the loop covers kWaves * chunk positions of the axis: thread (lx, ty) scans
// positions [s + ty*chunk, s + (ty+1)*chunk) in registers.
constexpr int kColsChunk = 16;      // rows of a column a wave scans per round (4, 8 and 32 measured: slower)

// Few columns and a long axis would leave the chip to a handful of workgroups walking the whole
// axis one round after the other: the axis is then cut into segments of seg_len positions, a
// workgroup per (block of 64 columns, segment).  scan_cols_partials leaves every segment's
// total per column in `partials` ([segment][column]); scan_cols starts a segment from what the
// segments before it add up to.  The input is read twice - three crossings instead of two -
// by as many workgroups as fill the device.
// Where a lane's column is at a position of the axis.  A position is the same for a whole
// wavefront, so with NARROW (every column starts less than 4 GB after the base: the host checks
// the view) the address is a scalar base - the position's offset, worked out once a wavefront -
// plus the lane's 32-bit offset, the form that a global access takes as it is: no pair of vector
// registers per access in flight for its address, which is what kept these kernels at 118
// registers and four wavefronts a SIMD.
template <typename P, bool NARROW>
struct ColumnAt {
    P* base;
    uint32_t lane_bytes;
    int64_t step_bytes;
    __device__ __forceinline__ ColumnAt(P* origin, int64_t column_offset, int64_t axis_stride) {
        if constexpr (NARROW) {
            base = origin;
            lane_bytes = static_cast<uint32_t>(column_offset * static_cast<int64_t>(sizeof(P)));
        } else {
            base = origin + column_offset;
            lane_bytes = 0;
        }
        step_bytes = axis_stride * static_cast<int64_t>(sizeof(P));
    }
    // the same by a running pointer: `row` is where position p starts, `next` moves it one position on
    // (an address worked out per position from p * stride keeps a product per position in scalar
    // registers for the whole loop once the compiler has unrolled it)
    using Row = std::conditional_t<std::is_const<P>::value, const char, char>*;
    __device__ __forceinline__ Row row(int64_t position) const { return reinterpret_cast<Row>(base) + position * step_bytes; }
    __device__ __forceinline__ Row next(Row r) const { return r + step_bytes; }
    __device__ __forceinline__ P* in_row(Row r) const {
        if constexpr (NARROW) return reinterpret_cast<P*>(r + static_cast<uint64_t>(lane_bytes));
        else return reinterpret_cast<P*>(r);
    }
    __device__ __forceinline__ P* at(int64_t position) const {
        using Byte = std::conditional_t<std::is_const<P>::value, const char, char>;
        Byte* row = reinterpret_cast<Byte*>(base) + position * step_bytes;
        if constexpr (NARROW) return reinterpret_cast<P*>(row + static_cast<uint64_t>(lane_bytes));
        else return reinterpret_cast<P*>(row);
    }
};

struct ColSegments {
    int64_t seg_len, segs, col_blocks;     // one segment: seg_len = n, segs = 1
};

template <typename T, int K, typename X, bool NZ, int C, bool NARROW>
__global__ __launch_bounds__(kBlock) void scan_cols_partials(
    const X* __restrict__ x, DimMap xmap, int64_t sx, int64_t m, int64_t n, ColSegments cut, T* __restrict__ partials) {
    using Op = ScanOp<T, K>;
    using VecX = Vec<X, C>;
    constexpr int R = kColsChunk;
    __shared__ T totals[kWaves][C][kWave];
    const int lx = threadIdx.x & (kWave - 1);
    // (NARROW: the wavefront's number as a scalar, so that positions and their offsets are scalars too)
    const int ty = NARROW ? __builtin_amdgcn_readfirstlane(threadIdx.x / kWave) : threadIdx.x / kWave;
    const int64_t col_block = blockIdx.x % cut.col_blocks, seg = blockIdx.x / cut.col_blocks;
    const int64_t col = (col_block * kWave + lx) * C;
    const bool live = col < m;
    const ColumnAt<const X, NARROW> xc(x, live ? xmap.at(col) : 0, sx);
    const int64_t lo = seg * cut.seg_len;
    const int64_t hi = lo + cut.seg_len < n ? lo + cut.seg_len : n;
    T sum[C];
#pragma unroll
    for (int c = 0; c < C; ++c) sum[c] = Op::identity();
    // wave ty takes positions lo + 16 ty, + 64, ...: sixteen loads in flight a lane
    for (int64_t p0 = lo + static_cast<int64_t>(ty) * R; p0 < hi; p0 += static_cast<int64_t>(kWaves) * R) {
        T v[R * C];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int64_t p = p0 + r;
            if (live && p < hi) {
                const VecX a = load_stream(reinterpret_cast<const VecX*>(xc.at(p)));
#pragma unroll
                for (int c = 0; c < C; ++c) v[r * C + c] = scan_input<T, X, NZ>(a.v[c]);
            } else {
#pragma unroll
                for (int c = 0; c < C; ++c) v[r * C + c] = Op::identity();
            }
        }
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int c = 0; c < C; ++c) sum[c] = Op::apply(sum[c], v[r * C + c]);
    }
#pragma unroll
    for (int c = 0; c < C; ++c) totals[ty][c][lx] = sum[c];
    __syncthreads();
    if (ty == 0 && live) {
#pragma unroll
        for (int c = 0; c < C; ++c) {
            T all = totals[0][c][lx];
#pragma unroll
            for (int i = 1; i < kWaves; ++i) all = Op::apply(all, totals[i][c][lx]);
            partials[seg * m + col + c] = all;
        }
    }
}

// C columns that lie side by side in memory per lane (one access of C elements: a wavefront's
// access to a position of the axis is then 64 C elements wide - with one two-byte element per
// lane it is 128 bytes, and such scans ran at the element rate of fp32 or below).
#ifndef DLFX_SCAN_COLS_WAVES
#define DLFX_SCAN_COLS_WAVES 5
#endif
template <typename T, int K, typename X, bool NZ, typename Y, int C, bool NARROW>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(1, DLFX_SCAN_COLS_WAVES))) void scan_cols(
    const X* __restrict__ x, Y* __restrict__ y, DimMap xmap, DimMap ymap, int64_t sx, int64_t sy,
    int64_t m, int64_t n, int chunk, int exclusive, ColSegments cut, const T* __restrict__ partials) {
    using Op = ScanOp<T, K>;
    using VecX = Vec<X, C>;
    using VecY = Vec<Y, C>;
    constexpr int R = kColsChunk;
    __shared__ T totals[2][kWaves][C][kWave];

    const int lx = threadIdx.x & (kWave - 1);
    // (NARROW: the wavefront's number as a scalar, so that positions and their offsets are scalars too)
    const int ty = NARROW ? __builtin_amdgcn_readfirstlane(threadIdx.x / kWave) : threadIdx.x / kWave;
    const int64_t col_block = blockIdx.x % cut.col_blocks, seg = blockIdx.x / cut.col_blocks;
    const int64_t col = (col_block * kWave + lx) * C;
    const bool live = col < m;
    const ColumnAt<const X, NARROW> xc(x, live ? xmap.at(col) : 0, sx);
    const ColumnAt<Y, NARROW> yc(y, live ? ymap.at(col) : 0, sy);
    const int64_t lo = seg * cut.seg_len;
    const int64_t hi = lo + cut.seg_len < n ? lo + cut.seg_len : n;        // this workgroup scans positions [lo, hi)

    T carry[C];
#pragma unroll
    for (int c = 0; c < C; ++c) carry[c] = Op::identity();
    if (cut.segs > 1 && live) {
        // what the segments before this one add up to (their totals, in order: four loads in flight)
        for (int64_t s0 = 0; s0 < seg; s0 += 4) {
            T part[4 * C];
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int c = 0; c < C; ++c) part[j * C + c] = s0 + j < seg ? partials[(s0 + j) * m + col + c] : Op::identity();
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int c = 0; c < C; ++c) carry[c] = Op::apply(carry[c], part[j * C + c]);
        }
    }
    int buf = 0;
    const int64_t step = static_cast<int64_t>(kWaves) * chunk;
    // the wave's chunk of the next round is on its way while this round is scanned and stored
    // (kept as loaded: two-byte elements wait two to a register)
    auto load_chunk = [&](int64_t s, VecX* v) __attribute__((always_inline)) {
        const int64_t p0 = s + static_cast<int64_t>(ty) * chunk;
        auto xrow = xc.row(p0);
#pragma unroll
        for (int r = 0; r < R; ++r, xrow = xc.next(xrow)) {
            const int64_t p = p0 + r;
            if (live && r < chunk && p < hi) {
                v[r] = load_stream(reinterpret_cast<const VecX*>(xc.in_row(xrow)));
            } else {
#pragma unroll
                for (int c = 0; c < C; ++c) v[r].v[c] = static_cast<X>(Op::identity());      // (folds as the identity, also where scan_input maps elements to 0 / 1)
            }
        }
    };
    VecX ahead[R];
    load_chunk(lo, ahead);
    for (int64_t s = lo; s < hi; s += step, buf ^= 1) {
        const int64_t p0 = s + static_cast<int64_t>(ty) * chunk;
        T v[R * C];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int c = 0; c < C; ++c) v[r * C + c] = scan_input<T, X, NZ>(ahead[r].v[c]);
        if (s + step < hi) load_chunk(s + step, ahead);
#pragma unroll
        for (int i = C; i < R * C; ++i) v[i] = Op::apply(v[i - C], v[i]);
#pragma unroll
        for (int c = 0; c < C; ++c) totals[buf][ty][c][lx] = v[(R - 1) * C + c];
        __syncthreads();
        T pre[C];
#pragma unroll
        for (int c = 0; c < C; ++c) {
            pre[c] = carry[c];
            T all = Op::identity();
#pragma unroll
            for (int i = 0; i < kWaves; ++i) {
                const T tv = totals[buf][i][c][lx];
                if (i < ty) pre[c] = Op::apply(pre[c], tv);
                all = Op::apply(all, tv);
            }
            carry[c] = Op::apply(carry[c], all);
        }
        if (live) {
            auto yrow = yc.row(p0);
            if (exclusive) {
#pragma unroll
                for (int r = 0; r < R; ++r, yrow = yc.next(yrow)) {
                    const int64_t p = p0 + r;
                    VecY out;
#pragma unroll
                    for (int c = 0; c < C; ++c)
                        out.v[c] = static_cast<Y>((r == 0) ? pre[c] : Op::apply(pre[c], v[(r > 0 ? r - 1 : 0) * C + c]));
                    if (r < chunk && p < hi) store_stream(reinterpret_cast<VecY*>(yc.in_row(yrow)), out);
                }
            } else {
#pragma unroll
                for (int r = 0; r < R; ++r, yrow = yc.next(yrow)) {
                    const int64_t p = p0 + r;
                    VecY out;
#pragma unroll
                    for (int c = 0; c < C; ++c) out.v[c] = static_cast<Y>(Op::apply(pre[c], v[r * C + c]));
                    if (r < chunk && p < hi) store_stream(reinterpret_cast<VecY*>(yc.in_row(yrow)), out);
                }
            }
        }
    }
}

// Short axes (up to 32 positions) beside many columns: a lane scans a whole column in registers,
// all its loads in flight at once, 256 columns a workgroup and no barrier (the kernel above
// gives such an axis to four wavefronts a position or two each: fp32 [8, 21, 512, 512] along
// axis 1 141 us, [64, 3, 224, 224] 184 us).
template <typename T, int K, typename X, bool NZ, typename Y, int N, int C, bool NARROW>
__global__ __launch_bounds__(kBlock) void scan_cols_thread(
    const X* __restrict__ x, Y* __restrict__ y, DimMap xmap, DimMap ymap, int64_t sx, int64_t sy, int64_t m, int n, int exclusive) {
    using Op = ScanOp<T, K>;
    using VecX = Vec<X, C>;
    using VecY = Vec<Y, C>;
    const int64_t col = (static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x) * C;
    if (col >= m) return;
    const ColumnAt<const X, NARROW> xc(x, xmap.at(col), sx);
    const ColumnAt<Y, NARROW> yc(y, ymap.at(col), sy);
    T v[N * C];
#pragma unroll
    for (int r = 0; r < N; ++r) {
        if (r < n) {
            const VecX a = load_stream(reinterpret_cast<const VecX*>(xc.at(r)));
#pragma unroll
            for (int c = 0; c < C; ++c) v[r * C + c] = scan_input<T, X, NZ>(a.v[c]);
        } else {
#pragma unroll
            for (int c = 0; c < C; ++c) v[r * C + c] = Op::identity();
        }
    }
    T run[C];
#pragma unroll
    for (int c = 0; c < C; ++c) run[c] = Op::identity();
#pragma unroll
    for (int r = 0; r < N; ++r) {
        VecY out;
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const T before = run[c];
            run[c] = Op::apply(run[c], v[r * C + c]);
            out.v[c] = static_cast<Y>(exclusive ? before : run[c]);
        }
        if (r < n) store_stream(reinterpret_cast<VecY*>(yc.at(r)), out);
    }
}

// ------------------------------------------------------------------ host side
// Joint merge of the leading dimensions [0, e) of two stride sets that share
// extents: neighbours merge only when both walks allow it.
bool make_dim_map2(const int64_t* dims, const int64_t* sx, const int64_t* sy, int e, DimMap* mx, DimMap* my) {
    int r = 0;
    int64_t d[64], a[64], b[64];
    for (int i = 0; i < e; ++i) {
        if (dims[i] == 1) continue;
        if (r > 0 && a[r - 1] == sx[i] * dims[i] && b[r - 1] == sy[i] * dims[i]) {
            d[r - 1] *= dims[i];
            a[r - 1] = sx[i];
            b[r - 1] = sy[i];
        } else {
            if (r == 64) return false;
            d[r] = dims[i];
            a[r] = sx[i];
            b[r] = sy[i];
            ++r;
        }
    }
    if (r > kMaxRank) return false;
    mx->rank = my->rank = r;
    for (int i = 0; i < kMaxRank; ++i) {
        mx->dims[i] = my->dims[i] = i < r ? d[i] : 1;
        mx->strides[i] = i < r ? a[i] : 0;
        my->strides[i] = i < r ? b[i] : 0;
    }
    return true;
}

#ifndef DLFX_SCAN_CHAIN_BLOCK
#define DLFX_SCAN_CHAIN_BLOCK 512
#endif
#ifndef DLFX_SCAN_CHAIN_BYTES
#define DLFX_SCAN_CHAIN_BYTES 131072
#endif
constexpr int kChainBlock = DLFX_SCAN_CHAIN_BLOCK;
constexpr int64_t kChainTileBytes = DLFX_SCAN_CHAIN_BYTES;

#ifndef DLFX_SCAN_GROUP_ROW_MAX
#define DLFX_SCAN_GROUP_ROW_MAX 768
#endif
constexpr int64_t kGroupRowMax = DLFX_SCAN_GROUP_ROW_MAX;      // longest row (in slots) a group of lanes scans
constexpr int64_t kMaxPad = 15;        // the most positions a row gains when it is tiled from the vector boundary before it

// Elements per tile: 256 bytes per thread for chained rows, less for short rows.
int64_t tile_elems(size_t elem_size, int64_t n) {
    const int64_t full = 256 * (256 / static_cast<int64_t>(elem_size));
    if (n > full) return kChainTileBytes / static_cast<int64_t>(elem_size);
    // the smallest of 1, 4, 8, 16, 32, 64 elements per thread that holds the row
    for (int64_t tile = 256; tile < full; tile *= (tile == 256 ? 4 : 2))
        if (n <= tile) return tile;
    return full;
}

// How scan_cols cuts the axis of m columns of n positions: not at all while the blocks of 64
// columns alone give the device enough workgroups (or the axis is short); otherwise into segments
// of whole rounds (64 positions), about 1024 workgroups in all, no segment under 512 positions.
#ifndef DLFX_SCAN_COLS_WANT
#define DLFX_SCAN_COLS_WANT 1024
#endif
#ifndef DLFX_SCAN_COLS_FEW
#define DLFX_SCAN_COLS_FEW 64
#endif
#ifndef DLFX_SCAN_COLS_MIN_SEG
#define DLFX_SCAN_COLS_MIN_SEG 512
#endif
ColSegments col_segments(int64_t m, int64_t n, int per_lane = 1) {
    ColSegments c;
    c.col_blocks = ceil_div(m, static_cast<int64_t>(kWave) * per_lane);
    c.seg_len = n;
    c.segs = 1;
    if (c.col_blocks >= 512 || n < 2048) return c;
    int64_t want = ceil_div(static_cast<int64_t>(DLFX_SCAN_COLS_WANT), c.col_blocks);
    // (a segment starts from the totals of those before it, read one after the other: up to 32 segments
    // may be as short as 128 positions, more than that only of 512 and more)
    int64_t most = n / DLFX_SCAN_COLS_MIN_SEG;
    const int64_t few = n / 128 < DLFX_SCAN_COLS_FEW ? n / 128 : DLFX_SCAN_COLS_FEW;
    if (most < few) most = few;
    if (want > most) want = most;
    if (want < 2) return c;
    c.seg_len = align_up(static_cast<size_t>(ceil_div(n, want)), static_cast<size_t>(kWaves * kColsChunk));
    c.segs = ceil_div(n, c.seg_len);
    if (c.segs < 2) {
        c.seg_len = n;
        c.segs = 1;
    }
    return c;
}

constexpr int kColsPerLaneMax = 2;
int g_cols_per_lane = 0;           // dlfx_set_tuning "scan_cols_per_lane": at most so many (0: as the kernels choose)
#ifndef DLFX_SCAN_COLS_BYTES
#define DLFX_SCAN_COLS_BYTES 4
#endif
constexpr size_t kColsAccessBytes = DLFX_SCAN_COLS_BYTES;      // widest access of a lane to its columns

// (the most that any number of columns per lane asks for: the query does not see the strides)
size_t col_partials_bytes(size_t elem_size, int64_t m, int64_t n) {
    size_t most = 0;
    for (int per_lane = 1; per_lane <= kColsPerLaneMax; per_lane *= 2) {
        const ColSegments c = col_segments(m, n, per_lane);
        const size_t bytes = c.segs > 1 ? static_cast<size_t>(c.segs) * static_cast<size_t>(m) * elem_size : 0;
        if (bytes > most) most = bytes;
    }
    return most;
}

struct ScanLayout {
    bool chained;                          // rows too long for one workgroup's registers: tiles with states
    int64_t tiles_per_row, tiles;
    size_t ticket_off, state_off, ready_off, total;
};

ScanLayout scan_layout(size_t elem_size, int64_t m, int64_t n) {
    ScanLayout l;
    l.chained = n > 256 * (256 / static_cast<int64_t>(elem_size));
    l.tiles_per_row = ceil_div(n, tile_elems(elem_size, n));
    l.tiles = m * l.tiles_per_row;
    l.ticket_off = 0;
    l.state_off = align_up(static_cast<size_t>(m) * 4, 256);
    l.ready_off = 0;
    if (!l.chained) {
        l.total = 0;
    } else {
        const size_t sb = static_cast<size_t>(l.tiles) * 2 * elem_size;      // a 64-bit word per 32 bits of the value
        l.ready_off = l.state_off + align_up(sb, 256);                       // a word per slice of states
        l.total = l.ready_off + align_up(static_cast<size_t>(ceil_div(l.tiles, kSliceTiles)) * 8, 256);
    }
    return l;
}

// True when the byte ranges the two views touch intersect.
template <typename X, typename T>
bool views_overlap(int rank, const int64_t* dims, const X* x, const int64_t* sx, const T* y, const int64_t* sy) {
    int64_t xlo = 0, xhi = 0, ylo = 0, yhi = 0;
    for (int i = 0; i < rank; ++i) {
        const int64_t ex = (dims[i] - 1) * sx[i], ey = (dims[i] - 1) * sy[i];
        if (ex > 0) xhi += ex; else xlo += ex;
        if (ey > 0) yhi += ey; else ylo += ey;
    }
    const char* xb = reinterpret_cast<const char*>(x + xlo);
    const char* xe = reinterpret_cast<const char*>(x + xhi + 1);
    const char* yb = reinterpret_cast<const char*>(y + ylo);
    const char* ye = reinterpret_cast<const char*>(y + yhi + 1);
    return xb < ye && yb < xe;
}

// A 64-bit value no earlier call of this process has used and, started from the clock and the
// process, no other process is likely to have left in reused memory; never zero.
unsigned long long next_nonce() {
    static std::atomic<unsigned long long> counter{[] {
        unsigned long long z = static_cast<unsigned long long>(std::chrono::steady_clock::now().time_since_epoch().count());
        z ^= static_cast<unsigned long long>(reinterpret_cast<uintptr_t>(&g_poll_limit)) << 17;
        z ^= static_cast<unsigned long long>(getpid()) << 40;
        z += 0x9e3779b97f4a7c15ull;                       // splitmix64
        z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
        z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
        return z ^ (z >> 31);
    }()};
    unsigned long long v;
    do v = counter.fetch_add(0x9e3779b97f4a7c15ull, std::memory_order_relaxed); while (v == 0ull);
    return v;
}

template <typename T, int K, typename X = T, bool NZ = false, typename Y = T>
int launch_scan(hipStream_t stream, int64_t m, int64_t n, int exclusive, int rank, const int64_t* dims,
                const X* x, const int64_t* x_strides, Y* y, const int64_t* y_strides,
                void* scratch, size_t scratch_bytes, const DimMap* x_axis = nullptr) {
    DimMap xmap, ymap;
    if (!make_dim_map2(dims, x_strides, y_strides, rank - 1, &xmap, &ymap)) return DLFX_ERR_RANK;
    DimMap xaxis;
    if (x_axis) {
        xaxis = *x_axis;
    } else {
        const int64_t one_dim[1] = {n}, one_stride[1] = {rank ? x_strides[rank - 1] : 1};
        make_dim_map(one_dim, one_stride, 0, 1, &xaxis);
        if (xaxis.rank == 0) {          // n == 1
            xaxis.rank = 1;
            xaxis.dims[0] = 1;
            xaxis.strides[0] = one_stride[0];
        }
    }
    const bool axis_general = xaxis.rank > 1;
    const int64_t sx = axis_general ? 0 : xaxis.strides[0];
    const int64_t sy = rank ? y_strides[rank - 1] : 1;

    // Many rows with a contiguous kept axis and a strided scanned axis: column kernel.
    const bool axis_unit = (sx == 1 || sx == -1 || n == 1) && (sy == 1 || sy == -1 || n == 1);
    const bool inner_unit = xmap.rank >= 1 && xmap.strides[xmap.rank - 1] == 1 && ymap.strides[ymap.rank - 1] == 1 &&
                            xmap.dims[xmap.rank - 1] >= 16;
    // Unit-stride rows that do not all start on a vector boundary are laid out from the boundary
    // before each row (scan_tile, scan_rows_group), which can make a row up to one vector less
    // one element longer.
    int pad = 0;
    if (!NZ && !axis_general && sx == 1 && sy == 1) {
        constexpr int VX = scan_vec<T, X, Y>();
        bool aligned = reinterpret_cast<uintptr_t>(x) % (sizeof(X) * VX) == 0;
        for (int i = 0; i < xmap.rank; ++i) aligned = aligned && xmap.strides[i] % VX == 0;
        if (!aligned) pad = VX - 1;
    }
    // Short rows along a unit-stride axis: a group of lanes per row (rows of up to 768 elements;
    // a workgroup per row would leave most of its threads, or of the chip, idle).
    if (!axis_general && axis_unit && n + pad <= kGroupRowMax && m >= 4) {
        const int64_t np = n + pad;
        const int64_t lanes = np <= 4 ? 1 : np <= 32 ? 4 : np <= 192 ? 16 : kWave;
        const int64_t blocks = ceil_div(m * lanes, kBlock);
        if (blocks > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
        const dim3 grid(static_cast<unsigned>(blocks)), block(kBlock);
        const int64_t row_bytes = n * static_cast<int64_t>(sizeof(X));
        const int plain = row_bytes < 512 || row_bytes % 128 != 0;
#define DLFX_SCAN_GROUP(LANES, ITEMS) \
    scan_rows_group<T, K, LANES, ITEMS, X, NZ, Y><<<grid, block, 0, stream>>>(x, y, xmap, ymap, sx, sy, m, n, exclusive, pad, plain)
        if (np <= 4) DLFX_SCAN_GROUP(1, 4);
        else if (np <= 16) DLFX_SCAN_GROUP(4, 4);
        else if (np <= 32) DLFX_SCAN_GROUP(4, 8);
        else if (np <= 64) DLFX_SCAN_GROUP(16, 4);
        else if (np <= 128) DLFX_SCAN_GROUP(16, 8);
        else if (np <= 192) DLFX_SCAN_GROUP(16, 12);
        else if (np <= 256) DLFX_SCAN_GROUP(kWave, 4);
        else if (np <= 512) DLFX_SCAN_GROUP(kWave, 8);
        else DLFX_SCAN_GROUP(kWave, 12);
#undef DLFX_SCAN_GROUP
        DLFX_CHECK_LAUNCH();
        return DLFX_OK;
    }
    const bool short_rows = n <= 64 && m >= 256;
    // (columns side by side in memory: from 64 of them; from 8 when the axis has a million positions or more -
    // [4194304, 16] fp32 along the first axis: 309 GB/s as strided rows, 1643 GB/s as columns, three lanes in
    // four idle; [262144, 16]: 674 against 497)
    const bool use_cols = !axis_general && (short_rows || (!axis_unit && (m >= 64 || (m >= 8 && n >= (1 << 20))) && (inner_unit || n < 4096)));
    // Columns per lane: as many neighbours in memory as make an access of DLFX_SCAN_COLS_BYTES, where every
    // such group of columns starts on a boundary of its own size at every position of the axis.
    int per_lane = 1;
    if (use_cols && !std::is_class<X>::value && !std::is_class<Y>::value) {
        for (int c = g_cols_per_lane ? g_cols_per_lane : kColsPerLaneMax; c > 1 && per_lane == 1; c /= 2) {
            if (sizeof(X) * c > kColsAccessBytes || sizeof(Y) * c > kColsAccessBytes) continue;
            bool ok = xmap.rank >= 1 && xmap.strides[xmap.rank - 1] == 1 && ymap.strides[ymap.rank - 1] == 1 &&
                      xmap.dims[xmap.rank - 1] % c == 0 && sx % c == 0 && sy % c == 0 &&
                      reinterpret_cast<uintptr_t>(x) % (sizeof(X) * c) == 0 && reinterpret_cast<uintptr_t>(y) % (sizeof(Y) * c) == 0;
            for (int i = 0; ok && i + 1 < xmap.rank; ++i) ok = xmap.strides[i] % c == 0 && ymap.strides[i] % c == 0;
            if (ok) per_lane = c;
        }
    }
    // Every column within 4 GB after the base, in input and output: scalar base + 32-bit lane offset.
    bool narrow = use_cols;
    {
        int64_t span_x = 0, span_y = 0;
        for (int i = 0; narrow && i < xmap.rank; ++i) {
            narrow = xmap.strides[i] >= 0 && ymap.strides[i] >= 0;
            span_x += (xmap.dims[i] - 1) * xmap.strides[i];
            span_y += (ymap.dims[i] - 1) * ymap.strides[i];
        }
        narrow = narrow && static_cast<uint64_t>(span_x) * sizeof(X) < (1ull << 32) && static_cast<uint64_t>(span_y) * sizeof(Y) < (1ull << 32);
    }
    if (!narrow) per_lane = 1;
    const ColSegments cut = col_segments(m, n, per_lane);
    // One column a lane: the kernel that walks the axis in rounds is faster with an address of its own
    // per lane and access (fp32 [32, 512, 56, 56] along axis 1: 77 against 82 us with scalar bases - the
    // compiler runs out of scalar registers for the bases of 32 accesses and parks them in vector
    // registers), the kernel that holds a short axis whole with scalar bases (60 against 65 us at
    // [8, 21, 512, 512]).  Two columns a lane need the registers that the scalar bases leave free.
    const bool thread_kernel = use_cols && n <= 32 && m >= 4096;
    auto with_cols = [&](auto&& launch) {
        constexpr bool kScalars = !std::is_class<X>::value && !std::is_class<Y>::value;
        if constexpr (kScalars && sizeof(X) * 4 <= kColsAccessBytes && sizeof(Y) * 4 <= kColsAccessBytes) {
            if (per_lane == 4) { launch(std::integral_constant<int, 4>(), std::true_type()); return; }
        }
        if constexpr (kScalars && sizeof(X) * 2 <= kColsAccessBytes && sizeof(Y) * 2 <= kColsAccessBytes) {
            if (per_lane == 2) { launch(std::integral_constant<int, 2>(), std::true_type()); return; }
        }
        if (narrow && thread_kernel) launch(std::integral_constant<int, 1>(), std::true_type());
        else launch(std::integral_constant<int, 1>(), std::false_type());
    };
    if (thread_kernel) {
        const int64_t blocks = ceil_div(m, static_cast<int64_t>(kBlock) * per_lane);
        if (blocks > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
        const dim3 grid(static_cast<unsigned>(blocks)), block(kBlock);
        with_cols([&](auto c, auto nw) {
            constexpr int C = decltype(c)::value;
            constexpr bool NW = decltype(nw)::value;
#define DLFX_SCAN_THREAD(N) scan_cols_thread<T, K, X, NZ, Y, N, C, NW><<<grid, block, 0, stream>>>(x, y, xmap, ymap, sx, sy, m, static_cast<int>(n), exclusive)
            if (n <= 4) DLFX_SCAN_THREAD(4);
            else if (n <= 8) DLFX_SCAN_THREAD(8);
            else if (n <= 16) DLFX_SCAN_THREAD(16);
            else DLFX_SCAN_THREAD(32);
#undef DLFX_SCAN_THREAD
        });
        DLFX_CHECK_LAUNCH();
        return DLFX_OK;
    }
    if (use_cols) {
        int chunk = static_cast<int>(ceil_div(n, kWaves) < kColsChunk ? ceil_div(n, kWaves) : kColsChunk);
        const int64_t blocks = cut.col_blocks * cut.segs;
        if (blocks > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
        T* partials = static_cast<T*>(scratch);
        if (cut.segs > 1) {
            if (!scratch || scratch_bytes < col_partials_bytes(sizeof(T), m, n)) return DLFX_ERR_SCRATCH_TOO_SMALL;
            with_cols([&](auto c, auto nw) {
                if constexpr (decltype(c)::value == 1 && decltype(nw)::value) return;        // (the short-axis kernel's combination)
                else scan_cols_partials<T, K, X, NZ, decltype(c)::value, decltype(nw)::value><<<dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0, stream>>>(x, xmap, sx, m, n, cut, partials);
            });
            DLFX_CHECK_LAUNCH();
        }
        with_cols([&](auto c, auto nw) {
            if constexpr (decltype(c)::value == 1 && decltype(nw)::value) return;
            else scan_cols<T, K, X, NZ, Y, decltype(c)::value, decltype(nw)::value><<<dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0, stream>>>(
                x, y, xmap, ymap, sx, sy, m, n, chunk, exclusive, cut, partials);
        });
        DLFX_CHECK_LAUNCH();
        return DLFX_OK;
    }

    const ScanLayout l = scan_layout(sizeof(T), m, n + pad);
    if (l.tiles > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
    if (scratch_bytes < l.total || (l.total && !scratch)) return DLFX_ERR_SCRATCH_TOO_SMALL;
    const int64_t tile = tile_elems(sizeof(T), n + pad);
    constexpr int FULL = 256 / sizeof(T);
    const dim3 block(kBlock);
    if (!l.chained) {
        const dim3 grid(static_cast<unsigned>(m));
        auto single = [&](auto items) {
            constexpr int ITEMS = decltype(items)::value;
            if constexpr (ITEMS <= FULL) {
                if constexpr (!NZ) {
                    if (pad) {
                        scan_rows_single<T, K, ITEMS, X, NZ, Y, true><<<grid, block, 0, stream>>>(x, y, xmap, ymap, sx, sy, xaxis, n, exclusive);
                        return;
                    }
                }
                scan_rows_single<T, K, ITEMS, X, NZ, Y, false><<<grid, block, 0, stream>>>(x, y, xmap, ymap, sx, sy, xaxis, n, exclusive);
            }
        };
        switch (tile / 256) {
        case 1: single(std::integral_constant<int, 1>()); break;
        case 4: single(std::integral_constant<int, 4>()); break;
        case 8: single(std::integral_constant<int, 8>()); break;
        case 16: single(std::integral_constant<int, 16>()); break;
        case 32: single(std::integral_constant<int, 32>()); break;
        default: single(std::integral_constant<int, 64>()); break;
        }
        DLFX_CHECK_LAUNCH();
        return DLFX_OK;
    }
    unsigned* ticket = reinterpret_cast<unsigned*>(static_cast<char*>(scratch) + l.ticket_off);
    TileState<T> st;
    st.bind(static_cast<char*>(scratch) + l.state_off, l.tiles);
    const bool in_place = views_overlap(rank, dims, x, x_strides, y, y_strides);
    constexpr int CI = static_cast<int>(kChainTileBytes / sizeof(T) / kChainBlock);
    const bool padded = !NZ && pad != 0;
    // The scan launch clears the tile states itself, except where that cannot work: under stream
    // capture (a replayed launch would carry the nonce of the replay before it), in place (the
    // rows' tickets need clearing before any workgroup runs), and when there are more slices to
    // clear than the device holds workgroups at once (the clearing workgroups, the first of the
    // launch, should all be running when a tile asks for their word; 256 run on any gfx950).
    ClearedBy cb{nullptr, 0ull};
    bool clears_itself = !in_place && !stream_is_capturing(stream);
    if (clears_itself && ceil_div(l.tiles, kSliceTiles) > 256) {
        int64_t room = 0;
        if constexpr (!NZ) {
            if (padded) room = resident_workgroups(scan_rows_chained<T, K, CI, false, kChainBlock, X, NZ, Y, true>, kChainBlock);
        }
        if (!padded) room = resident_workgroups(scan_rows_chained<T, K, CI, false, kChainBlock, X, NZ, Y, false>, kChainBlock);
        clears_itself = ceil_div(l.tiles, kSliceTiles) <= room;
    }
    if (clears_itself) {
        cb.ready = reinterpret_cast<unsigned long long*>(static_cast<char*>(scratch) + l.ready_off);
        cb.nonce = next_nonce();
    } else {
        scan_init<T><<<dim3(static_cast<unsigned>(ceil_div(l.tiles, kBlock))), block, 0, stream>>>(ticket, m, st, l.tiles);
        DLFX_CHECK_LAUNCH();
    }
    const dim3 grid(static_cast<unsigned>(l.tiles));
    const dim3 cblock(kChainBlock);
    // rows off a vector boundary have kernels of their own: the aligned ones carry none of that arithmetic
    auto chained = [&](auto ticketed, auto padded) {
        scan_rows_chained<T, K, CI, decltype(ticketed)::value, kChainBlock, X, NZ, Y, decltype(padded)::value><<<grid, cblock, 0, stream>>>(
            x, y, xmap, ymap, sx, sy, xaxis, n, l.tiles_per_row, exclusive, g_poll_limit, ticket, st, cb);
    };
    bool launched = false;
    if constexpr (!NZ) {
        if (pad) {
            if (in_place) chained(std::true_type(), std::true_type());
            else chained(std::false_type(), std::true_type());
            launched = true;
        }
    }
    if (!launched) {
        if (in_place) chained(std::true_type(), std::false_type());
        else chained(std::false_type(), std::false_type());
    }
    DLFX_CHECK_LAUNCH();
    return DLFX_OK;
}

}  // namespace
}  // namespace dlfx

using namespace dlfx;

namespace dlfx {
bool set_scan_tuning(const char* key, int64_t value) {
    if (!std::strcmp(key, "scan_cols_per_lane") && (value == 0 || value == 1 || value == 2)) {
        g_cols_per_lane = static_cast<int>(value);
        return true;
    }
    if (!std::strcmp(key, "scan_poll_limit") && value >= 0 && value <= (1 << 30)) {
        g_poll_limit = static_cast<int>(value);
        return true;
    }
    return false;
}
}  // namespace dlfx

extern "C" size_t dlfx_scan_scratch_bytes(int dtype, int64_t m, int64_t n) {
    size_t es = dtype_size(dtype);
    if (dtype == DLFX_F16) es = 4;                  // scanned as fp32
    if (es < 4 || m <= 0 || n <= 0) return 0;
    const size_t rows = dlfx::scan_layout(es, m, n + dlfx::kMaxPad).total;       // rows off a vector boundary take up to a vector more
    const size_t cols = dlfx::col_partials_bytes(es, m, n);                       // (an axis that is not the innermost, cut into segments)
    return rows > cols ? rows : cols;
}

extern "C" int dlfx_scan(dlfx_stream_t stream, const char* name, int dtype, int64_t m, int64_t n,
                         int exclusive, int rank, const int64_t* dims,
                         const void* x, int64_t x_offset, const int64_t* x_strides,
                         void* y, int64_t y_offset, const int64_t* y_strides,
                         void* scratch, size_t scratch_bytes) {
    if (!name || !x || !y || m <= 0 || n <= 0) return DLFX_ERR_INVALID_ARGUMENT;
    if (!view_ok(rank, dims, x_strides) || !view_ok(rank, dims, y_strides)) return DLFX_ERR_INVALID_ARGUMENT;
    if (rank < 1 || dims[rank - 1] != n || view_size(rank, dims) != m * n) return DLFX_ERR_INVALID_ARGUMENT;
    int kind;
    if (!std::strcmp(name, "cumsum")) kind = kScanAdd;
    else if (!std::strcmp(name, "cumprod")) kind = kScanMul;
    else if (!std::strcmp(name, "cummax")) kind = kScanMax;
    else if (!std::strcmp(name, "cummin")) kind = kScanMin;
    else return DLFX_ERR_UNKNOWN_OP;
    hipStream_t s = static_cast<hipStream_t>(stream);
#ifdef DLFX_SCAN_FEW_TYPES
    // (a build for experiments, minutes faster to compile: running sums of fp32 and half only)
    if (dtype == DLFX_F16 && kind == kScanMax)
        return launch_scan<float, kScanMax, half_t, false, half_t>(s, m, n, exclusive, rank, dims, static_cast<const half_t*>(x) + x_offset, x_strides,
                                                                  static_cast<half_t*>(y) + y_offset, y_strides, scratch, scratch_bytes);
    if (kind != kScanAdd) return DLFX_ERR_UNSUPPORTED_DTYPE;
    if (dtype == DLFX_F16)
        return launch_scan<float, kScanAdd, half_t, false, half_t>(s, m, n, exclusive, rank, dims, static_cast<const half_t*>(x) + x_offset, x_strides,
                                                                  static_cast<half_t*>(y) + y_offset, y_strides, scratch, scratch_bytes);
    if (dtype == DLFX_F32)
        return launch_scan<float, kScanAdd>(s, m, n, exclusive, rank, dims, static_cast<const float*>(x) + x_offset, x_strides,
                                            static_cast<float*>(y) + y_offset, y_strides, scratch, scratch_bytes);
    return DLFX_ERR_UNSUPPORTED_DTYPE;
#else
    if (dtype == DLFX_F16) {
        // half elements are scanned in fp32: one rounding per output instead of one per step
        const half_t* xp = static_cast<const half_t*>(x) + x_offset;
        half_t* yp = static_cast<half_t*>(y) + y_offset;
        switch (kind) {
        case kScanAdd: return launch_scan<float, kScanAdd, half_t, false, half_t>(s, m, n, exclusive, rank, dims, xp, x_strides, yp, y_strides, scratch, scratch_bytes);
        case kScanMul: return launch_scan<float, kScanMul, half_t, false, half_t>(s, m, n, exclusive, rank, dims, xp, x_strides, yp, y_strides, scratch, scratch_bytes);
        case kScanMax: return launch_scan<float, kScanMax, half_t, false, half_t>(s, m, n, exclusive, rank, dims, xp, x_strides, yp, y_strides, scratch, scratch_bytes);
        default:       return launch_scan<float, kScanMin, half_t, false, half_t>(s, m, n, exclusive, rank, dims, xp, x_strides, yp, y_strides, scratch, scratch_bytes);
        }
    }
    if (dtype == DLFX_C64 || dtype == DLFX_C128) {
        // running sums and products of complex elements; complex numbers are not ordered
        if (kind != kScanAdd && kind != kScanMul) return DLFX_ERR_UNSUPPORTED_DTYPE;
        auto run = [&](auto tag) {
            using T = decltype(tag);
            const T* xp = static_cast<const T*>(x) + x_offset;
            T* yp = static_cast<T*>(y) + y_offset;
            if (kind == kScanAdd) return launch_scan<T, kScanAdd>(s, m, n, exclusive, rank, dims, xp, x_strides, yp, y_strides, scratch, scratch_bytes);
            return launch_scan<T, kScanMul>(s, m, n, exclusive, rank, dims, xp, x_strides, yp, y_strides, scratch, scratch_bytes);
        };
        return dtype == DLFX_C64 ? run(Cx<float>()) : run(Cx<double>());
    }
    return dispatch_dtype(dtype, [&](auto tag) {
        using T = decltype(tag);
        const T* xp = static_cast<const T*>(x) + x_offset;
        T* yp = static_cast<T*>(y) + y_offset;
        switch (kind) {
        case kScanAdd: return launch_scan<T, kScanAdd>(s, m, n, exclusive, rank, dims, xp, x_strides, yp, y_strides, scratch, scratch_bytes);
        case kScanMul: return launch_scan<T, kScanMul>(s, m, n, exclusive, rank, dims, xp, x_strides, yp, y_strides, scratch, scratch_bytes);
        case kScanMax: return launch_scan<T, kScanMax>(s, m, n, exclusive, rank, dims, xp, x_strides, yp, y_strides, scratch, scratch_bytes);
        default:       return launch_scan<T, kScanMin>(s, m, n, exclusive, rank, dims, xp, x_strides, yp, y_strides, scratch, scratch_bytes);
        }
    });
#endif
}

extern "C" size_t dlfx_scan_nonzero_scratch_bytes(int dtype, int64_t m, int64_t n) {
    if (!dtype_size(dtype) || m <= 0 || n <= 0) return 0;
    return scan_layout(4, m, n + kMaxPad).total;
}

extern "C" int dlfx_scan_nonzero(dlfx_stream_t stream, int dtype, int64_t m, int64_t n,
                                 int exclusive, int rank, const int64_t* dims,
                                 const void* x, int64_t x_offset, const int64_t* x_strides,
                                 int32_t* y, int64_t y_offset, const int64_t* y_strides,
                                 void* scratch, size_t scratch_bytes) {
    if (!x || !y || m <= 0 || n <= 0) return DLFX_ERR_INVALID_ARGUMENT;
    if (!view_ok(rank, dims, x_strides) || !view_ok(rank, dims, y_strides)) return DLFX_ERR_INVALID_ARGUMENT;
    if (rank < 1 || rank > 64 || view_size(rank, dims) != m * n) return DLFX_ERR_INVALID_ARGUMENT;
    if (n > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;       // counts are 32-bit, as in the reference
    // the scanned elements are the trailing dimensions whose product is n, walked in row-major
    // order (nonzero() scans a whole tensor as one row: reduce.h:426-429)
    int split = rank;
    int64_t prod = 1;
    while (split > 0 && prod < n) prod *= dims[--split];
    if (prod != n) return DLFX_ERR_INVALID_ARGUMENT;
    if (split == rank) split = rank - 1;                   // n == 1
    DimMap xaxis, yaxis;
    if (!make_dim_map(dims, x_strides, split, rank, &xaxis) || !make_dim_map(dims, y_strides, split, rank, &yaxis))
        return DLFX_ERR_RANK;
    if (yaxis.rank > 1) return DLFX_ERR_RANK;              // the counts must be walked with one stride
    if (xaxis.rank == 0) {
        xaxis.rank = 1;
        xaxis.dims[0] = 1;
        xaxis.strides[0] = 1;
    }
    int64_t d2[64], xs2[64], ys2[64];
    for (int i = 0; i < split; ++i) {
        d2[i] = dims[i];
        xs2[i] = x_strides[i];
        ys2[i] = y_strides[i];
    }
    d2[split] = n;
    xs2[split] = xaxis.rank == 1 ? xaxis.strides[0] : 0;
    ys2[split] = yaxis.rank == 1 ? yaxis.strides[0] : 1;
    hipStream_t s = static_cast<hipStream_t>(stream);
#ifdef DLFX_SCAN_FEW_TYPES
    return DLFX_ERR_UNSUPPORTED_DTYPE;
#endif
    auto run = [&](auto tag) {
        using X = decltype(tag);
        return launch_scan<int32_t, kScanAdd, X, true>(s, m, n, exclusive, split + 1, d2, static_cast<const X*>(x) + x_offset,
                                                       xs2, y + y_offset, ys2, scratch, scratch_bytes, &xaxis);
    };
    if (dtype == DLFX_F16) return run(half_t());
    if (dtype == DLFX_BOOL) return run(uint8_t());
    if (dtype == DLFX_I16) return DLFX_ERR_UNSUPPORTED_DTYPE;
    return dispatch_dtype(dtype, run);
}
