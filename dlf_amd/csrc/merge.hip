// merge: two tensors sorted along their last axis -> one sorted tensor
// (gpgpu/include/gdnn.h:147-155; host semantics dlf/include/tensor/reorder_detail.h:346-368:
// the merged row takes an element of the second input only when it compares strictly before
// the first input's current element, so equal elements keep "first input first").
//
// Merge path in two kernels.  merge_partition finds, for every tile boundary of every output
// row, how many elements of the first input lie before it (one 9-way search per boundary by
// eight lanes, all of them in flight at once).  merge_tiles loads the two input pieces of a tile into LDS
// with coalesced loads, every thread finds its own split by a search in LDS, merges kItems
// outputs serially, and the tile leaves through LDS again so that stores are coalesced.
// Bandwidth bound: every input element is read once and every output element written once.
// Output rows of up to 2048 elements skip the partition: merge_rows_small packs several rows
// into a workgroup.
#include <type_traits>

#include "common.hip.h"

namespace dlfx {
namespace {

constexpr int kBlock = 256;
#ifndef DLFX_MERGE_TILE_BYTES
#define DLFX_MERGE_TILE_BYTES 16384
#endif
// outputs per thread / per tile: 16 KB tiles (16 four-byte or 8 eight-byte elements per thread)
constexpr int items_of(size_t elem_size) { return static_cast<int>(DLFX_MERGE_TILE_BYTES / kBlock / elem_size); }
constexpr int tile_of(size_t elem_size) { return kBlock * items_of(elem_size); }

template <typename T, bool DESC>
__device__ __forceinline__ bool before(T a, T b) {       // a sorts strictly before b
    return DESC ? a > b : a < b;
}

// Number of elements of x among the first `diag` outputs of merging x[0, na) and y[0, nb).
template <typename T, bool DESC, typename GetX, typename GetY>
__device__ __forceinline__ int64_t merge_split(int64_t diag, int64_t na, int64_t nb, GetX x, GetY y) {
    int64_t lo = diag > nb ? diag - nb : 0;
    int64_t hi = diag < na ? diag : na;
    while (lo < hi) {
        const int64_t mid = (lo + hi) >> 1;
        if (before<T, DESC>(y(diag - 1 - mid), x(mid))) hi = mid;
        else lo = mid + 1;
    }
    return lo;
}

struct MergeViews {
    DimMap xrows, yrows, zrows;
    int64_t sx, sy, sz;
    int64_t na, nb;
};

// Four lanes per tile boundary probe four evenly spaced split candidates at once: a boundary
// takes about log5 of the row length dependent memory round trips instead of log2.  The kernel
// is bound by the cache lines its probes fetch as much as by those round trips: with 16 384
// boundaries, 8 lanes each (log9) measured 3 to 4 % slower, 16 lanes 7 % slower, 64 lanes
// fetched as many cache lines as the merge itself moves; 1 lane (plain bisection) 5 % slower.
constexpr int kProbe = 4;

template <typename T, bool DESC>
__global__ __launch_bounds__(kBlock) void merge_partition(const T* __restrict__ x, const T* __restrict__ y, MergeViews v,
                                                          int64_t rows, int64_t bounds_per_row,
                                                          int32_t* __restrict__ split) {
    constexpr int kTile = tile_of(sizeof(T));
    const int lane = lane_id();
    const int sub = lane % kProbe;
    const int group_lane0 = lane - sub;
    const int64_t g = (static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x) / kProbe;
    const bool live = g < rows * bounds_per_row;
    const int64_t row = live ? g / bounds_per_row : 0;
    const int64_t t = live ? g - row * bounds_per_row : 0;
    const int64_t n = v.na + v.nb;
    int64_t diag = t * kTile;
    if (diag > n) diag = n;
    const T* xr = x + v.xrows.at(row);
    const T* yr = y + v.yrows.at(row);
    // smallest split i in [lo, hi] for which y[diag - 1 - i] sorts strictly before x[i]
    // (hi when there is none): the predicate is false up to the answer and true from it on
    int64_t lo = diag > v.nb ? diag - v.nb : 0;
    int64_t hi = diag < v.na ? diag : v.na;
    if (!live) hi = lo;
    while (__ballot(lo < hi) != 0ull) {
        const bool open = lo < hi;
        const int64_t span = hi - lo;
        const int64_t mid = lo + (span * (sub + 1)) / (kProbe + 1);            // < hi while the search is open
        bool y_first = false;
        if (open) y_first = before<T, DESC>(yr[(diag - 1 - mid) * v.sy], xr[mid * v.sx]);
        const unsigned votes = static_cast<unsigned>(__ballot(y_first) >> group_lane0) & ((1u << kProbe) - 1u);
        const int f = votes ? __ffs(static_cast<int>(votes)) - 1 : kProbe;     // first candidate that holds
        const int64_t at_f = lane_get(mid, group_lane0 + (f < kProbe ? f : kProbe - 1));
        const int64_t below = lane_get(mid, group_lane0 + (f > 0 ? f - 1 : 0));
        if (open) {
            if (f < kProbe) hi = at_f;
            if (f > 0) lo = below + 1;
        }
    }
    if (live && sub == 0) split[g] = static_cast<int32_t>(lo);
}

template <typename T, bool DESC>
__global__ __launch_bounds__(kBlock) void merge_tiles(const T* __restrict__ x, const T* __restrict__ y, T* __restrict__ z,
                                                      MergeViews v, int64_t tiles_per_row,
                                                      const int32_t* __restrict__ split) {
    constexpr int kItems = items_of(sizeof(T));
    constexpr int kTile = tile_of(sizeof(T));
    // one unused word after every 32: threads that walk the tile 8 or 16 words apart (their
    // merge positions, their runs of outputs) then spread over all LDS banks
    __shared__ T buf[kTile + kTile / 32];
    auto at = [](int p) { return p + (p >> 5); };
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x / tiles_per_row;
    const int64_t t = blockIdx.x - row * tiles_per_row;
    const int64_t n = v.na + v.nb;
    const int64_t d0 = t * kTile;
    const int64_t d1 = (d0 + kTile < n) ? d0 + kTile : n;
    const int32_t* sp = split + row * (tiles_per_row + 1) + t;
    const int64_t i0 = sp[0], i1 = sp[1];
    const int64_t j0 = d0 - i0, j1 = d1 - i1;
    const int ca = static_cast<int>(i1 - i0), cb = static_cast<int>(j1 - j0);     // ca + cb <= kTile
    const T* xr = x + v.xrows.at(row) + i0 * v.sx;
    const T* yr = y + v.yrows.at(row) + j0 * v.sy;

    // the tile's piece of x, then its piece of y
    // (tile position k < ca comes from x, the others from y; all loads are issued before the
    // first one is used)
    const int total = ca + cb;
    T in[kItems];
#pragma unroll
    for (int e = 0; e < kItems; ++e) {
        int k = e * kBlock + tid;
        if (k >= total) k = total - 1;            // past the tile: a valid element, not stored
        const T* p = k < ca ? xr + k * v.sx : yr + (k - ca) * v.sy;
        in[e] = load_stream(p);
    }
#pragma unroll
    for (int e = 0; e < kItems; ++e) {
        const int k = e * kBlock + tid;
        if (k < total) buf[at(k)] = in[e];
    }
    __syncthreads();

    int diag = tid * kItems;
    if (diag > total) diag = total;
    int i = static_cast<int>(merge_split<T, DESC>(
        diag, ca, cb, [&](int64_t k) { return buf[at(static_cast<int>(k))]; },
        [&](int64_t k) { return buf[at(ca + static_cast<int>(k))]; }));
    int j = diag - i;
    // both heads live in registers; every step reloads only the one it consumed (an exhausted
    // side reads a valid slot whose value is never taken)
    T out[kItems];
    T xv = buf[at(i < ca ? i : 0)], yv = buf[at(j < cb ? ca + j : 0)];
#pragma unroll
    for (int e = 0; e < kItems; ++e) {
        const bool has_x = i < ca, has_y = j < cb;
        const bool take_y = has_y && (!has_x || before<T, DESC>(yv, xv));
        out[e] = take_y ? yv : xv;
        i += take_y ? 0 : 1;
        j += take_y ? 1 : 0;
        int next = take_y ? ca + j : i;
        if (next >= total) next = 0;
        const T nv = buf[at(next)];
        if (take_y) yv = nv;
        else xv = nv;
    }
    __syncthreads();
#pragma unroll
    for (int e = 0; e < kItems; ++e)
        if (tid * kItems + e < total) buf[at(tid * kItems + e)] = out[e];
    __syncthreads();
    T* zr = z + v.zrows.at(row) + d0 * v.sz;
#pragma unroll
    for (int e = 0; e < kItems; ++e) out[e] = buf[at(e * kBlock + tid)];
#pragma unroll
    for (int e = 0; e < kItems; ++e)
        if (e * kBlock + tid < total) store_stream(&zr[static_cast<int64_t>(e * kBlock + tid) * v.sz], out[e]);
}

// Short rows: several rows per workgroup.  A row of n <= 256 * ITEMS outputs belongs to a team
// of 2^lg consecutive threads (ITEMS outputs each), a workgroup holds 256 >> lg rows, each in
// its own slab of LDS.  No partition pass and no scratch: a row is one tile whose split is
// known (all of x, all of y).  The steps are those of merge_tiles.
template <typename T, bool DESC, int ITEMS>
__global__ __launch_bounds__(kBlock) void merge_rows_small(const T* __restrict__ x, const T* __restrict__ y, T* __restrict__ z,
                                                           MergeViews v, int64_t rows, int lg) {
    __shared__ T buf[kBlock * ITEMS + kBlock * ITEMS / 32];
    auto at = [](int p) { return p + (p >> 5); };
    const int tid = threadIdx.x;
    const int team = 1 << lg;
    const int sub = tid & (team - 1);
    const int base = (tid - sub) * ITEMS;                         // the row's slab
    const int64_t row = static_cast<int64_t>(blockIdx.x) * (kBlock >> lg) + (tid >> lg);
    const bool live = row < rows;
    const int na = static_cast<int>(v.na), nb = static_cast<int>(v.nb), n = na + nb;
    const T* xr = x + (live ? v.xrows.at(row) : 0);
    const T* yr = y + (live ? v.yrows.at(row) : 0);

    T in[ITEMS];
#pragma unroll
    for (int e = 0; e < ITEMS; ++e) {
        const int k = e * team + sub;
        if (live && k < n) in[e] = load_stream(k < na ? xr + k * v.sx : yr + (k - na) * v.sy);
    }
#pragma unroll
    for (int e = 0; e < ITEMS; ++e) {
        const int k = e * team + sub;
        if (live && k < n) buf[at(base + k)] = in[e];
    }
    __syncthreads();

    int diag = sub * ITEMS;
    if (diag > n) diag = n;
    int i = 0;
    if (live)
        i = static_cast<int>(merge_split<T, DESC>(
            diag, na, nb, [&](int64_t k) { return buf[at(base + static_cast<int>(k))]; },
            [&](int64_t k) { return buf[at(base + na + static_cast<int>(k))]; }));
    int j = diag - i;
    T out[ITEMS];
    T xv = buf[at(base + (i < na ? i : 0))], yv = buf[at(base + (j < nb ? na + j : 0))];
#pragma unroll
    for (int e = 0; e < ITEMS; ++e) {
        const bool has_x = i < na, has_y = j < nb;
        const bool take_y = has_y && (!has_x || before<T, DESC>(yv, xv));
        out[e] = take_y ? yv : xv;
        i += take_y ? 0 : 1;
        j += take_y ? 1 : 0;
        int next = take_y ? na + j : i;
        if (next >= n) next = 0;
        const T nv = buf[at(base + next)];
        if (take_y) yv = nv;
        else xv = nv;
    }
    __syncthreads();
#pragma unroll
    for (int e = 0; e < ITEMS; ++e)
        if (sub * ITEMS + e < n) buf[at(base + sub * ITEMS + e)] = out[e];
    __syncthreads();
    if (!live) return;
    T* zr = z + v.zrows.at(row);
#pragma unroll
    for (int e = 0; e < ITEMS; ++e) {
        const int k = e * team + sub;
        if (k < n) out[e] = buf[at(base + k)];
    }
#pragma unroll
    for (int e = 0; e < ITEMS; ++e) {
        const int k = e * team + sub;
        if (k < n) store_stream(&zr[static_cast<int64_t>(k) * v.sz], out[e]);
    }
}

constexpr int kSmallRowMax = kBlock * 8;        // longest output row merge_rows_small takes

template <typename T, bool DESC>
int launch_merge_small(hipStream_t stream, int64_t m, const MergeViews& v, const T* x, const T* y, T* z) {
    const int n = static_cast<int>(v.na + v.nb);
    const int items = n <= 256 ? 4 : 8;
    int lg = 0;
    while ((items << lg) < n) ++lg;                               // team = 2^lg threads, at most 256
    const int64_t blocks = ceil_div(m, static_cast<int64_t>(kBlock >> lg));
    if (blocks > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
    const dim3 grid(static_cast<unsigned>(blocks));
    if (items == 4) merge_rows_small<T, DESC, 4><<<grid, dim3(kBlock), 0, stream>>>(x, y, z, v, m, lg);
    else merge_rows_small<T, DESC, 8><<<grid, dim3(kBlock), 0, stream>>>(x, y, z, v, m, lg);
    DLFX_CHECK_LAUNCH();
    return DLFX_OK;
}

struct MergeLayout {
    int64_t tiles_per_row;
    size_t total;
};

MergeLayout merge_layout(size_t elem_size, int64_t m, int64_t n) {
    MergeLayout l;
    l.tiles_per_row = ceil_div(n, tile_of(elem_size));
    if (l.tiles_per_row < 1) l.tiles_per_row = 1;
    l.total = align_up(static_cast<size_t>(m) * (l.tiles_per_row + 1) * 4, 256);
    return l;
}

template <typename T>
int launch_merge(hipStream_t stream, int dir, int64_t m, const MergeViews& v, const T* x, const T* y, T* z,
                 void* scratch, size_t scratch_bytes) {
    const int64_t n = v.na + v.nb;
    if (n > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;       // splits are 32-bit
    if (n <= kSmallRowMax) return dir ? launch_merge_small<T, true>(stream, m, v, x, y, z) : launch_merge_small<T, false>(stream, m, v, x, y, z);
    const MergeLayout l = merge_layout(sizeof(T), m, n);
    if (m * l.tiles_per_row > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
    if (!scratch || scratch_bytes < l.total) return DLFX_ERR_SCRATCH_TOO_SMALL;
    int32_t* split = static_cast<int32_t*>(scratch);
    const int64_t bounds = m * (l.tiles_per_row + 1);
    const dim3 pgrid(static_cast<unsigned>(ceil_div(bounds * kProbe, kBlock))), tgrid(static_cast<unsigned>(m * l.tiles_per_row));
    if (dir) {
        merge_partition<T, true><<<pgrid, dim3(kBlock), 0, stream>>>(x, y, v, m, l.tiles_per_row + 1, split);
        DLFX_CHECK_LAUNCH();
        merge_tiles<T, true><<<tgrid, dim3(kBlock), 0, stream>>>(x, y, z, v, l.tiles_per_row, split);
    } else {
        merge_partition<T, false><<<pgrid, dim3(kBlock), 0, stream>>>(x, y, v, m, l.tiles_per_row + 1, split);
        DLFX_CHECK_LAUNCH();
        merge_tiles<T, false><<<tgrid, dim3(kBlock), 0, stream>>>(x, y, z, v, l.tiles_per_row, split);
    }
    DLFX_CHECK_LAUNCH();
    return DLFX_OK;
}

}  // namespace
}  // namespace dlfx

using namespace dlfx;

extern "C" size_t dlfx_merge_scratch_bytes(int dtype, int64_t m, int64_t n) {
    if (!dtype_size(dtype) || dtype == DLFX_BOOL || m <= 0 || n <= 0) return 0;
    return merge_layout(dtype_size(dtype), m, n).total;
}

extern "C" int dlfx_merge(dlfx_stream_t stream, int dir, int dtype, int rank,
                          const int64_t* x_dims, const int64_t* x_strides, const void* x, int64_t x_offset,
                          const int64_t* y_dims, const int64_t* y_strides, const void* y, int64_t y_offset,
                          const int64_t* z_dims, const int64_t* z_strides, void* z, int64_t z_offset,
                          void* scratch, size_t scratch_bytes) {
    if (!x || !y || !z || rank < 1) return DLFX_ERR_INVALID_ARGUMENT;
    if (!view_ok(rank, z_dims, z_strides)) return DLFX_ERR_INVALID_ARGUMENT;
    if (!x_dims || !y_dims || !x_strides || !y_strides) return DLFX_ERR_INVALID_ARGUMENT;
    // the inputs share the output's leading extents; their last extents add up to the output's
    // (an input may be empty along the axis)
    for (int i = 0; i < rank - 1; ++i)
        if (x_dims[i] != z_dims[i] || y_dims[i] != z_dims[i]) return DLFX_ERR_INVALID_ARGUMENT;
    const int64_t na = x_dims[rank - 1], nb = y_dims[rank - 1];
    if (na < 0 || nb < 0 || na + nb != z_dims[rank - 1]) return DLFX_ERR_INVALID_ARGUMENT;
    MergeViews v;
    if (!make_dim_map(z_dims, x_strides, 0, rank - 1, &v.xrows) || !make_dim_map(z_dims, y_strides, 0, rank - 1, &v.yrows) ||
        !make_dim_map(z_dims, z_strides, 0, rank - 1, &v.zrows))
        return DLFX_ERR_RANK;
    v.sx = x_strides[rank - 1];
    v.sy = y_strides[rank - 1];
    v.sz = z_strides[rank - 1];
    v.na = na;
    v.nb = nb;
    const int64_t m = view_size(rank, z_dims) / z_dims[rank - 1];
    if (dtype == DLFX_BOOL) return DLFX_ERR_UNSUPPORTED_DTYPE;
    return dispatch_dtype16(dtype, [&](auto tag) {
        using T = decltype(tag);
        return launch_merge<T>(static_cast<hipStream_t>(stream), dir, m, v, static_cast<const T*>(x) + x_offset,
                               static_cast<const T*>(y) + y_offset, static_cast<T*>(z) + z_offset, scratch, scratch_bytes);
    });
}
