// softmax / logsoftmax / hardmax over the rows of a contiguous [m, n] matrix
// (gpgpu/include/gdnn.h:253-264; host semantics dlf/include/tensor/dnn_detail.h:266-350:
// subtract the row maximum, exponentiate, divide by the sum; logsoftmax x - max - log(sum);
// hardmax a one at the first occurrence of the maximum and zeros elsewhere; hardmax also takes
// int32 / int64 rows, gpgpu/src/gdnn.cpp:1888-1900).
//
// A row is read once: it lives in the registers of a team of threads (1, 4 or 16 lanes for
// the shortest rows, one wavefront up to 2048 elements, a 256-thread workgroup up to 6144, a
// 1024-thread workgroup up to 32768 four-byte elements, and up to 65536 when there are
// enough rows for every compute unit) between the load, the two team-wide reductions and the
// store.  Longer rows are streamed twice (running maximum and rescaled sum first, then the
// outputs), a few long rows cut into tiles over the whole device.  Bandwidth bound; exp and log in the
// element type, sums in it as well (tree order), as the reference's row loops do.  IEEE half
// rows are widened to float at the load and rounded once at the store.
#include <cmath>
#include <cstring>
#include <limits>
#include <type_traits>

#include "common.hip.h"

namespace dlfx {
namespace {

enum SoftKind { kSoftmax = 0, kLogSoftmax = 1, kHardmax = 2 };

// The arithmetic type for rows stored as S.
template <typename S> struct ComputeOf { using type = S; };
template <> struct ComputeOf<half_t> { using type = float; };

template <typename T> __device__ __forceinline__ T exp_of(T v);
template <> __device__ __forceinline__ float exp_of<float>(float v) { return expf(v); }
template <> __device__ __forceinline__ double exp_of<double>(double v) { return exp(v); }
template <typename T> __device__ __forceinline__ T log_of(T v);
template <> __device__ __forceinline__ float log_of<float>(float v) { return logf(v); }
template <> __device__ __forceinline__ double log_of<double>(double v) { return log(v); }

// (maximum, first index holding it) with the serial loop's rules (dnn_detail.h:334-346):
// strict comparison, so the first occurrence wins; a NaN in position 0 is never displaced and
// a NaN elsewhere never wins.
template <typename T>
struct MaxAt {
    T v;
    int32_t i;
};
template <typename T>
__device__ __forceinline__ MaxAt<T> max_at_of(T x, int64_t j) {
    if (x != x) {
        if (j == 0) return {std::numeric_limits<T>::infinity(), -1};
        return {-std::numeric_limits<T>::infinity(), std::numeric_limits<int32_t>::max()};
    }
    return {x, static_cast<int32_t>(j)};
}
template <typename T>
__device__ __forceinline__ MaxAt<T> max_at_join(MaxAt<T> a, MaxAt<T> b) {
    const bool take_b = b.v > a.v || (b.v == a.v && b.i < a.i);
    return take_b ? b : a;
}

// Reduction over the TEAM threads that share a row (part of a wavefront, one, or a whole workgroup through
// LDS); every thread receives the result.  `slot` separates the teams of a workgroup.
template <int TEAM, typename V, typename Join>
__device__ __forceinline__ V team_reduce(V v, Join join, V* lds) {
    if constexpr (TEAM < kWave) v = group_reduce(v, TEAM, join);      // one lane, a quad, or a DPP row of 16 lanes
    else v = wave_reduce(v, join);
    if constexpr (TEAM > kWave) {
        constexpr int WAVES = TEAM / kWave;
        const int w = threadIdx.x / kWave;
        __syncthreads();                       // the previous use of `lds` is over
        if (lane_id() == 0) lds[w] = v;
        __syncthreads();
        v = lds[0];
#pragma unroll
        for (int i = 1; i < WAVES; ++i) v = join(v, lds[i]);
    }
    return v;
}

// Rows held in registers.  TEAM threads per row, ITEMS elements per thread in 128-bit accesses
// of V elements: item k of thread t sits at position ((k / V) * TEAM + t) * V + k % V of its
// row.  A row that starts on a 16-byte boundary has element i at position i.  Rows that do not
// (PAD: the host found that rows may not - a row length that is no multiple of V, a base
// off the boundary) are laid out from the boundary before them: element i at position
// i + shift, so that every whole vector of the row is still one aligned access; the vectors at
// a row's two ends, when partial, move element by element.  Without PAD none of that arithmetic
// is compiled in: n is a multiple of V and a vector lies in the row or past it.
template <typename S, int TEAM, int ITEMS, int KIND, bool PAD>
__global__ __launch_bounds__(TEAM > 256 ? TEAM : 256)
__attribute__((amdgpu_waves_per_eu(TEAM >= 1024 && sizeof(typename ComputeOf<S>::type) * ITEMS <= 128 ? 8 : 1)))      // two 1024-thread rows per CU
void softmax_rows(const S* x, S* y, int64_t m, int64_t n) {          // y may be x: no restrict
    using T = typename ComputeOf<S>::type;
    constexpr int BLOCK = TEAM > 256 ? TEAM : 256;
    constexpr int V = 16 / static_cast<int>(sizeof(S));
    static_assert(ITEMS % V == 0, "whole vectors per thread");
    constexpr int G = ITEMS / V;
    using VecT = Vec<S, V>;
    __shared__ alignas(16) unsigned char lds_raw[(TEAM > kWave ? TEAM / kWave : 1) * sizeof(MaxAt<T>)];

    const int t = threadIdx.x % TEAM;
    const int64_t row = static_cast<int64_t>(blockIdx.x) * (BLOCK / TEAM) + threadIdx.x / TEAM;
    const bool live = row < m;                           // whole teams are live or not
    const S* xr = x + (live ? row : 0) * n;
    S* yr = y + (live ? row : 0) * n;
    const T lowest = std::is_integral<T>::value ? std::numeric_limits<T>::lowest() : -std::numeric_limits<T>::infinity();
    const int32_t shift = PAD ? static_cast<int32_t>((reinterpret_cast<uintptr_t>(xr) / sizeof(S)) % V) : 0;
    const bool y_like_x = !PAD || static_cast<int32_t>((reinterpret_cast<uintptr_t>(yr) / sizeof(S)) % V) == shift;
    const int32_t n32 = static_cast<int32_t>(n);          // rows here have at most 32768 elements
    const int32_t end32 = n32 + shift;                    // positions [shift, end32) are the row
    auto index_of = [&](int k) -> int32_t { return ((k / V) * TEAM + t) * V + k % V - shift; };
    auto in_row = [&](int k) -> bool { return static_cast<uint32_t>(index_of(k)) < static_cast<uint32_t>(n32); };

    // A vector that holds the row's first or last elements also holds the neighbouring row's:
    // it is read whole all the same (and what is not the row's dropped) unless it reaches
    // outside the tensor, which only the first and the last row's end vectors can.
    const S* const tensor_end = x + m * n;
    T v[ITEMS];
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const int32_t p0 = (g * TEAM + t) * V;
        const S* at = xr - shift + p0;
        if constexpr (!PAD) {
            if (live && p0 < n32) {
                const VecT a = load_stream(reinterpret_cast<const VecT*>(at));
#pragma unroll
                for (int e = 0; e < V; ++e) v[g * V + e] = static_cast<T>(a.v[e]);
            } else {
#pragma unroll
                for (int e = 0; e < V; ++e) v[g * V + e] = lowest;
            }
        } else if (live && p0 + V > shift && p0 < end32 && at >= x && at + V <= tensor_end) {
            const VecT a = load_stream(reinterpret_cast<const VecT*>(at));
#pragma unroll
            for (int e = 0; e < V; ++e) v[g * V + e] = (p0 + e >= shift && p0 + e < end32) ? static_cast<T>(a.v[e]) : lowest;
        } else {
#pragma unroll
            for (int e = 0; e < V; ++e)
                v[g * V + e] = (live && p0 + e >= shift && p0 + e < end32) ? static_cast<T>(load_stream(&xr[p0 + e - shift])) : lowest;
        }
    }

    // Whether the row starts with a NaN, read now: in place, another wave of the team may store
    // element 0 as soon as it has left the last team reduction.
    const bool leading_nan = live && xr[0] != xr[0];

    if constexpr (KIND == kHardmax) {
        // the serial loop (dnn_detail.h:334-346) keeps the first element that is strictly larger
        // than everything before it: the first occurrence of the largest non-NaN value, or
        // position 0 when the row starts with a NaN (nothing compares larger than a NaN)
        T mx = lowest;
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) mx = (mx < v[k]) ? v[k] : mx;
        mx = team_reduce<TEAM>(mx, [](T a, T b) { return (a < b) ? b : a; }, reinterpret_cast<T*>(lds_raw));
        int32_t hot = std::numeric_limits<int32_t>::max();
#pragma unroll
        for (int k = ITEMS - 1; k >= 0; --k)
            if (v[k] == mx && in_row(k)) hot = index_of(k);      // this thread's indices grow with k
        hot = team_reduce<TEAM>(hot, [](int32_t a, int32_t b) { return a < b ? a : b; }, reinterpret_cast<int32_t*>(lds_raw));
        if (hot >= n32 || leading_nan) hot = 0;                            // all NaN or -inf, or a leading NaN
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) v[k] = index_of(k) == hot ? T(1) : T(0);
    } else {
        // the reference starts from px[0] and uses std::max, which keeps its first argument when
        // the comparison fails: a NaN spreads only from position 0; other NaNs are skipped
        T mx = lowest;
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) mx = (mx < v[k]) ? v[k] : mx;
        mx = team_reduce<TEAM>(mx, [](T a, T b) { return (a < b) ? b : a; }, reinterpret_cast<T*>(lds_raw));
        if (leading_nan) mx = static_cast<T>(xr[0]);           // stores only follow the next team reduction
        T sum = T(0);
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) {
            const T e = in_row(k) ? exp_of<T>(v[k] - mx) : T(0);
            if constexpr (KIND == kSoftmax) v[k] = e;
            sum += e;
        }
        sum = team_reduce<TEAM>(sum, [](T a, T b) { return a + b; }, reinterpret_cast<T*>(lds_raw));
        if constexpr (KIND == kSoftmax) {
#pragma unroll
            for (int k = 0; k < ITEMS; ++k) v[k] = v[k] / sum;
        } else {
            // (x - max) - log(sum) in this order: x - max is exact for nearby values, max + log(sum)
            // would round at the magnitude of max
            const T lsum = log_of<T>(sum);
#pragma unroll
            for (int k = 0; k < ITEMS; ++k) v[k] = (v[k] - mx) - lsum;
        }
    }

#pragma unroll
    for (int g = 0; g < G; ++g) {
        const int32_t p0 = (g * TEAM + t) * V;
        if (!live) continue;
        if constexpr (!PAD) {
            if (p0 < n32) {
                VecT a;
#pragma unroll
                for (int e = 0; e < V; ++e) a.v[e] = static_cast<S>(v[g * V + e]);
                store_stream(reinterpret_cast<VecT*>(yr + p0), a);
            }
        } else if (y_like_x && p0 >= shift && p0 + V <= end32) {
            VecT a;
#pragma unroll
            for (int e = 0; e < V; ++e) a.v[e] = static_cast<S>(v[g * V + e]);
            store_stream(reinterpret_cast<VecT*>(yr - shift + p0), a);
        } else {
#pragma unroll
            for (int e = 0; e < V; ++e)
                if (p0 + e >= shift && p0 + e < end32) store_stream(&yr[p0 + e - shift], static_cast<S>(v[g * V + e]));
        }
    }
}

constexpr int kStreamBatch = 8;

// Rows too long for registers: one 1024-thread workgroup per row, two passes over the row.
template <typename S, int KIND>
__global__ __launch_bounds__(1024) void softmax_rows_streamed(const S* x, S* y, int64_t n) {
    using T = typename ComputeOf<S>::type;
    constexpr int TEAM = 1024;
    __shared__ alignas(16) unsigned char lds_raw[(TEAM / kWave) * sizeof(MaxAt<T>)];
    const int t = threadIdx.x;
    const S* xr = x + static_cast<int64_t>(blockIdx.x) * n;
    S* yr = y + static_cast<int64_t>(blockIdx.x) * n;
    const T lowest = std::is_integral<T>::value ? std::numeric_limits<T>::lowest() : -std::numeric_limits<T>::infinity();
    if constexpr (KIND == kHardmax) {
        MaxAt<T> best = {lowest, std::numeric_limits<int32_t>::max()};
        for (int64_t i = t; i < n; i += TEAM) best = max_at_join(best, max_at_of(static_cast<T>(xr[i]), i));
        best = team_reduce<TEAM>(best, [](MaxAt<T> a, MaxAt<T> b) { return max_at_join(a, b); },
                                 reinterpret_cast<MaxAt<T>*>(lds_raw));
        const int64_t hot = best.i < 0 ? 0 : best.i;
        for (int64_t i = t; i < n; i += TEAM) yr[i] = i == hot ? S(1) : S(0);
    } else {
        // running maximum and the sum of exp(x - maximum), rescaled whenever the maximum moves
        T mx = lowest, sum = T(0);
        for (int64_t i = t; i < n; i += TEAM * kStreamBatch) {              // kStreamBatch loads in flight per thread
            S in[kStreamBatch];
#pragma unroll
            for (int u = 0; u < kStreamBatch; ++u) {
                const int64_t j = i + static_cast<int64_t>(u) * TEAM;
                if (j < n) in[u] = load_stream(&xr[j]);
            }
#pragma unroll
            for (int u = 0; u < kStreamBatch; ++u) {
                if (i + static_cast<int64_t>(u) * TEAM >= n) break;
                const T xv = static_cast<T>(in[u]);
                if (mx < xv) {
                    sum = sum * exp_of<T>(mx - xv);          // exp(-inf) = 0 on the first element
                    mx = xv;
                }
                if (xv != lowest || mx != lowest) sum += exp_of<T>(xv - mx);     // -inf before any finite element adds nothing
            }
        }
        T row_max = team_reduce<TEAM>(mx, [](T a, T b) { return (a < b) ? b : a; }, reinterpret_cast<T*>(lds_raw));
        sum = (mx == lowest) ? T(0) : sum * exp_of<T>(mx - row_max);
        if (xr[0] != xr[0]) row_max = static_cast<T>(xr[0]);             // a NaN in position 0 is the reference's maximum
        sum = team_reduce<TEAM>(sum, [](T a, T b) { return a + b; }, reinterpret_cast<T*>(lds_raw));
        const T lsum = log_of<T>(sum);
        for (int64_t i = t; i < n; i += TEAM * kStreamBatch) {
            S in[kStreamBatch];
#pragma unroll
            for (int u = 0; u < kStreamBatch; ++u) {
                const int64_t j = i + static_cast<int64_t>(u) * TEAM;
                if (j < n) in[u] = load_stream(&xr[j]);
            }
#pragma unroll
            for (int u = 0; u < kStreamBatch; ++u) {
                const int64_t j = i + static_cast<int64_t>(u) * TEAM;
                if (j >= n) break;
                const T xv = static_cast<T>(in[u]);
                store_stream(&yr[j], static_cast<S>(KIND == kSoftmax ? exp_of<T>(xv - row_max) / sum : (xv - row_max) - lsum));
            }
        }
    }
}

// Few long rows: a row is cut into tiles so that the whole device works on it.  A first kernel
// leaves one record per tile in scratch, a second one folds a row's records (every workgroup of
// the row does, they are few) and writes its own tile.  A workgroup only ever writes the tile
// it read, and what the second kernel needs from other places of the row (the first element,
// for the NaN rule) travels in the records, so y may be x.
template <typename T>
struct SoftPartial {
    T mx, sum, first;          // soft kinds: running maximum, sum of exp(x - mx), the row's first element (tile 0)
    MaxAt<T> best;             // hardmax
};

constexpr int kSplitBatch = 8;

struct SplitPlan {
    int64_t tiles, tile_len;
};

// about 2048 workgroups in all, tiles of at least 8192 elements
inline SplitPlan split_plan(int64_t m, int64_t n) {
    int64_t tiles = ceil_div(2048, m);
    const int64_t most = ceil_div(n, 8192);
    if (tiles > most) tiles = most;
    if (tiles < 1) tiles = 1;
    SplitPlan p;
    p.tile_len = ceil_div(n, tiles);
    p.tiles = ceil_div(n, p.tile_len);
    return p;
}

template <typename S, int KIND>
__global__ __launch_bounds__(1024) void softmax_split_partials(const S* __restrict__ x, int64_t n, int64_t tiles, int64_t tile_len,
                                                               SoftPartial<typename ComputeOf<S>::type>* __restrict__ part) {
    using T = typename ComputeOf<S>::type;
    constexpr int TEAM = 1024;
    __shared__ alignas(16) unsigned char lds_raw[(TEAM / kWave) * sizeof(MaxAt<T>)];
    const int t = threadIdx.x;
    const int64_t row = blockIdx.x / tiles, tile = blockIdx.x - row * tiles;
    const S* xr = x + row * n;
    const int64_t i0 = tile * tile_len, i1 = i0 + tile_len < n ? i0 + tile_len : n;
    const T lowest = std::is_integral<T>::value ? std::numeric_limits<T>::lowest() : -std::numeric_limits<T>::infinity();
    SoftPartial<T> out;
    out.mx = lowest;
    out.sum = T(0);
    out.first = static_cast<T>(xr[0]);
    out.best = {lowest, std::numeric_limits<int32_t>::max()};
    if constexpr (KIND == kHardmax) {
        MaxAt<T> best = out.best;
        for (int64_t i = i0 + t; i < i1; i += TEAM) best = max_at_join(best, max_at_of(static_cast<T>(xr[i]), i));
        out.best = team_reduce<TEAM>(best, [](MaxAt<T> a, MaxAt<T> b) { return max_at_join(a, b); },
                                     reinterpret_cast<MaxAt<T>*>(lds_raw));
    } else {
        T mx = lowest, sum = T(0);
        for (int64_t i = i0 + t; i < i1; i += TEAM * kSplitBatch) {           // kSplitBatch loads in flight per thread
            S in[kSplitBatch];
#pragma unroll
            for (int u = 0; u < kSplitBatch; ++u) {
                const int64_t j = i + static_cast<int64_t>(u) * TEAM;
                if (j < i1) in[u] = load_stream(&xr[j]);
            }
#pragma unroll
            for (int u = 0; u < kSplitBatch; ++u) {
                if (i + static_cast<int64_t>(u) * TEAM >= i1) break;
                const T xv = static_cast<T>(in[u]);
                if (mx < xv) {
                    sum = sum * exp_of<T>(mx - xv);
                    mx = xv;
                }
                if (xv != lowest || mx != lowest) sum += exp_of<T>(xv - mx);
            }
        }
        const T tile_max = team_reduce<TEAM>(mx, [](T a, T b) { return (a < b) ? b : a; }, reinterpret_cast<T*>(lds_raw));
        sum = (mx == lowest) ? T(0) : sum * exp_of<T>(mx - tile_max);
        out.mx = tile_max;
        out.sum = team_reduce<TEAM>(sum, [](T a, T b) { return a + b; }, reinterpret_cast<T*>(lds_raw));
    }
    if (t == 0) part[blockIdx.x] = out;
}

template <typename S, int KIND>
__global__ __launch_bounds__(1024) void softmax_split_apply(const S* x, S* y, int64_t n, int64_t tiles,
                                                            int64_t tile_len,
                                                            const SoftPartial<typename ComputeOf<S>::type>* __restrict__ part) {
    using T = typename ComputeOf<S>::type;
    constexpr int TEAM = 1024;
    __shared__ alignas(16) unsigned char lds_raw[(TEAM / kWave) * sizeof(MaxAt<T>)];
    const int t = threadIdx.x;
    const int64_t row = blockIdx.x / tiles, tile = blockIdx.x - row * tiles;
    const S* xr = x + row * n;
    S* yr = y + row * n;
    const SoftPartial<T>* pr = part + row * tiles;
    const int64_t i0 = tile * tile_len, i1 = i0 + tile_len < n ? i0 + tile_len : n;
    const T lowest = std::is_integral<T>::value ? std::numeric_limits<T>::lowest() : -std::numeric_limits<T>::infinity();
    if constexpr (KIND == kHardmax) {
        MaxAt<T> best = {lowest, std::numeric_limits<int32_t>::max()};
        for (int64_t p = t; p < tiles; p += TEAM) best = max_at_join(best, pr[p].best);
        best = team_reduce<TEAM>(best, [](MaxAt<T> a, MaxAt<T> b) { return max_at_join(a, b); },
                                 reinterpret_cast<MaxAt<T>*>(lds_raw));
        const int64_t hot = best.i < 0 ? 0 : best.i;
        for (int64_t i = i0 + t; i < i1; i += TEAM) yr[i] = i == hot ? S(1) : S(0);
    } else {
        T mx = lowest, sum = T(0);
        for (int64_t p = t; p < tiles; p += TEAM) {
            const T pm = pr[p].mx, ps = pr[p].sum;
            if (mx < pm) {
                sum = sum * exp_of<T>(mx - pm);
                mx = pm;
            }
            if (pm != lowest) sum += ps * exp_of<T>(pm - mx);
        }
        T row_max = team_reduce<TEAM>(mx, [](T a, T b) { return (a < b) ? b : a; }, reinterpret_cast<T*>(lds_raw));
        sum = (mx == lowest) ? T(0) : sum * exp_of<T>(mx - row_max);
        const T first = pr[0].first;
        if (first != first) row_max = first;                      // a NaN in position 0 is the reference's maximum
        sum = team_reduce<TEAM>(sum, [](T a, T b) { return a + b; }, reinterpret_cast<T*>(lds_raw));
        const T lsum = log_of<T>(sum);
        for (int64_t i = i0 + t; i < i1; i += TEAM * kSplitBatch) {
            S in[kSplitBatch];
#pragma unroll
            for (int u = 0; u < kSplitBatch; ++u) {
                const int64_t j = i + static_cast<int64_t>(u) * TEAM;
                if (j < i1) in[u] = load_stream(&xr[j]);
            }
#pragma unroll
            for (int u = 0; u < kSplitBatch; ++u) {
                const int64_t j = i + static_cast<int64_t>(u) * TEAM;
                if (j >= i1) break;
                const T xv = static_cast<T>(in[u]);
                store_stream(&yr[j], static_cast<S>(KIND == kSoftmax ? exp_of<T>(xv - row_max) / sum : (xv - row_max) - lsum));
            }
        }
    }
}

// rows at most this long are held in registers by one workgroup
template <typename T>
constexpr int64_t register_row_limit() { return sizeof(typename ComputeOf<T>::type) == 4 ? 1024 * 32 : 1024 * 16; }
constexpr int64_t kSplitMaxRows = 256;        // from this many rows on (one per compute unit), a workgroup per row is as fast

template <typename T>
size_t split_scratch_bytes(int64_t m, int64_t n) {
    if (n <= register_row_limit<T>() || m >= kSplitMaxRows) return 0;
    const SplitPlan p = split_plan(m, n);
    if (p.tiles < 2) return 0;
    return static_cast<size_t>(m * p.tiles) * sizeof(SoftPartial<typename ComputeOf<T>::type>);
}

template <typename T, int KIND>
int launch_softmax(hipStream_t stream, int64_t m, int64_t n, const T* x, T* y, void* scratch, size_t scratch_bytes) {
    constexpr int V = 16 / static_cast<int>(sizeof(T));
    constexpr int kRegisterBytes = static_cast<int>(sizeof(typename ComputeOf<T>::type));
    // rows all start on a 16-byte boundary, or are laid out from the boundary before them (softmax_rows),
    // which can make a row up to V - 1 positions longer
    const bool aligned = n % V == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0;
    const int pad = aligned ? 0 : V - 1;
    const int64_t np = n + pad;
    // wavefront teams: 4 rows per workgroup
#define DLFX_WAVE_ROWS(ITEMS)                                                                                   \
    do {                                                                                                        \
        const dim3 grid(static_cast<unsigned>(ceil_div(m, 4)));                                                 \
        if (pad) softmax_rows<T, kWave, ITEMS, KIND, true><<<grid, dim3(256), 0, stream>>>(x, y, m, n);         \
        else softmax_rows<T, kWave, ITEMS, KIND, false><<<grid, dim3(256), 0, stream>>>(x, y, m, n);            \
        DLFX_CHECK_LAUNCH();                                                                                    \
        return DLFX_OK;                                                                                         \
    } while (0)
#define DLFX_BLOCK_ROWS(ITEMS)                                                                                  \
    do {                                                                                                        \
        const dim3 grid(static_cast<unsigned>(m));                                                              \
        if (pad) softmax_rows<T, 1024, ITEMS, KIND, true><<<grid, dim3(1024), 0, stream>>>(x, y, m, n);         \
        else softmax_rows<T, 1024, ITEMS, KIND, false><<<grid, dim3(1024), 0, stream>>>(x, y, m, n);            \
        DLFX_CHECK_LAUNCH();                                                                                    \
        return DLFX_OK;                                                                                         \
    } while (0)
    if (ceil_div(m, 4) > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
    // very short rows: one, four or sixteen lanes per row (V elements each), 256, 64 or 16 rows per workgroup
#define DLFX_LANE_ROWS(TEAM, ITEMS)                                                                             \
    do {                                                                                                        \
        const dim3 grid(static_cast<unsigned>(ceil_div(m, 256 / TEAM)));                                        \
        if (pad) softmax_rows<T, TEAM, ITEMS, KIND, true><<<grid, dim3(256), 0, stream>>>(x, y, m, n);          \
        else softmax_rows<T, TEAM, ITEMS, KIND, false><<<grid, dim3(256), 0, stream>>>(x, y, m, n);             \
        DLFX_CHECK_LAUNCH();                                                                                    \
        return DLFX_OK;                                                                                         \
    } while (0)
    // (slots of a row: V, 4 V, 16 V, 32 V, 48 V, 64 V, 128 V, 192 V, 256 V, 384 V, then 2048, 3072, 4096, 6144 and 8192 to 32768 in steps of at most half)
    if (np <= V) DLFX_LANE_ROWS(1, V);
    if (np <= 4 * V) DLFX_LANE_ROWS(4, V);
    if (np <= 16 * V) DLFX_LANE_ROWS(16, V);
    if (np <= 32 * V) DLFX_LANE_ROWS(16, 2 * V);
    if (np <= 48 * V) DLFX_LANE_ROWS(16, 3 * V);
#undef DLFX_LANE_ROWS
    if (np <= kWave * V) DLFX_WAVE_ROWS(V);
    if (np <= kWave * 2 * V) DLFX_WAVE_ROWS(2 * V);
    if (np <= kWave * 3 * V) DLFX_WAVE_ROWS(3 * V);
    if (np <= kWave * 4 * V) DLFX_WAVE_ROWS(4 * V);
    if (np <= kWave * 6 * V && kWave * 6 * V < kWave * 32) DLFX_WAVE_ROWS(6 * V);
    if (np <= kWave * 32) DLFX_WAVE_ROWS(32);
    // a workgroup of 256 threads per row up to 8192 slots: a row of 2049 elements would leave
    // most of 1024 threads without any
#define DLFX_TEAM_ROWS(ITEMS)                                                                                   \
    do {                                                                                                        \
        const dim3 grid(static_cast<unsigned>(m));                                                              \
        if (pad) softmax_rows<T, 256, ITEMS, KIND, true><<<grid, dim3(256), 0, stream>>>(x, y, m, n);           \
        else softmax_rows<T, 256, ITEMS, KIND, false><<<grid, dim3(256), 0, stream>>>(x, y, m, n);              \
        DLFX_CHECK_LAUNCH();                                                                                    \
        return DLFX_OK;                                                                                         \
    } while (0)
    if constexpr (V <= 4) {
        if (np <= 256 * 12) DLFX_TEAM_ROWS(12);
    }
    if (np <= 256 * 16) DLFX_TEAM_ROWS(16);
    if constexpr (kRegisterBytes == 4) {
        if (np <= 256 * 24) DLFX_TEAM_ROWS(24);
    }
#undef DLFX_TEAM_ROWS
    if (np <= 1024 * 8) DLFX_BLOCK_ROWS(8);
    if constexpr (V <= 4) {
        if (np <= 1024 * 12) DLFX_BLOCK_ROWS(12);
    }
    if (np <= 1024 * 16) DLFX_BLOCK_ROWS(16);
    if (np <= 1024 * 24 && kRegisterBytes == 4) DLFX_BLOCK_ROWS(24);
    if (np <= 1024 * 32 && kRegisterBytes == 4) DLFX_BLOCK_ROWS(32);
    // Longer rows, when there is at least one for every compute unit: up to 64 registers a thread
    // hold the row (one workgroup on a compute unit), which reads it once where the streamed
    // kernel reads it twice.
    if (m >= kSplitMaxRows) {
        if constexpr (kRegisterBytes == 4) {
            if (np <= 1024 * 40) DLFX_BLOCK_ROWS(40);
            if (np <= 1024 * 48) DLFX_BLOCK_ROWS(48);
            if (np <= 1024 * 56) DLFX_BLOCK_ROWS(56);
            if (np <= 1024 * 64) DLFX_BLOCK_ROWS(64);
        } else {
            if (np <= 1024 * 24) DLFX_BLOCK_ROWS(24);
            if (np <= 1024 * 32) DLFX_BLOCK_ROWS(32);
        }
    }
#undef DLFX_WAVE_ROWS
#undef DLFX_BLOCK_ROWS
    const size_t need = split_scratch_bytes<T>(m, n);
    if (need && scratch && scratch_bytes >= need && reinterpret_cast<uintptr_t>(scratch) % 16 == 0) {
        using P = SoftPartial<typename ComputeOf<T>::type>;
        const SplitPlan p = split_plan(m, n);
        const dim3 grid(static_cast<unsigned>(m * p.tiles));
        softmax_split_partials<T, KIND><<<grid, dim3(1024), 0, stream>>>(x, n, p.tiles, p.tile_len, static_cast<P*>(scratch));
        DLFX_CHECK_LAUNCH();
        softmax_split_apply<T, KIND><<<grid, dim3(1024), 0, stream>>>(x, y, n, p.tiles, p.tile_len, static_cast<const P*>(scratch));
        DLFX_CHECK_LAUNCH();
        return DLFX_OK;
    }
    softmax_rows_streamed<T, KIND><<<dim3(static_cast<unsigned>(m)), dim3(1024), 0, stream>>>(x, y, n);
    DLFX_CHECK_LAUNCH();
    return DLFX_OK;
}

}  // namespace
}  // namespace dlfx

using namespace dlfx;

extern "C" size_t dlfx_softmax_scratch_bytes(int dtype, int64_t m, int64_t n) {
    if (m <= 0 || n <= 0 || m > 0x7fffffffLL || n > 0x7fffffffLL) return 0;
    switch (dtype) {
    case DLFX_F32: return split_scratch_bytes<float>(m, n);
    case DLFX_F64: return split_scratch_bytes<double>(m, n);
    case DLFX_F16: return split_scratch_bytes<half_t>(m, n);
    case DLFX_I32: return split_scratch_bytes<int32_t>(m, n);
    case DLFX_I64: return split_scratch_bytes<int64_t>(m, n);
    default: return 0;
    }
}

extern "C" int dlfx_softmax(dlfx_stream_t stream, const char* name, int dtype, int64_t m, int64_t n,
                            const void* x, int64_t x_offset, void* y, int64_t y_offset,
                            void* scratch, size_t scratch_bytes) {
    if (!name || !x || !y || m <= 0 || n <= 0) return DLFX_ERR_INVALID_ARGUMENT;
    if (m > 0x7fffffffLL || n > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
    int kind;
    if (!std::strcmp(name, "softmax")) kind = kSoftmax;
    else if (!std::strcmp(name, "logsoftmax")) kind = kLogSoftmax;
    else if (!std::strcmp(name, "hardmax")) kind = kHardmax;
    else return DLFX_ERR_UNKNOWN_OP;
    const bool integer = dtype == DLFX_I32 || dtype == DLFX_I64;
    if (dtype != DLFX_F32 && dtype != DLFX_F64 && dtype != DLFX_F16 && !(integer && kind == kHardmax))
        return DLFX_ERR_UNSUPPORTED_DTYPE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    auto run = [&](auto tag) {
        using T = decltype(tag);
        const T* xp = static_cast<const T*>(x) + x_offset;
        T* yp = static_cast<T*>(y) + y_offset;
        if constexpr (!std::is_integral<T>::value) {
            if (kind == kSoftmax) return launch_softmax<T, kSoftmax>(s, m, n, xp, yp, scratch, scratch_bytes);
            if (kind == kLogSoftmax) return launch_softmax<T, kLogSoftmax>(s, m, n, xp, yp, scratch, scratch_bytes);
        }
        return launch_softmax<T, kHardmax>(s, m, n, xp, yp, scratch, scratch_bytes);
    };
    switch (dtype) {
    case DLFX_F32: return run(float());
    case DLFX_F64: return run(double());
    case DLFX_F16: return run(half_t());
    case DLFX_I32: return run(int32_t());
    default: return run(int64_t());
    }
}
