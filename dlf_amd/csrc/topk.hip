// top_k along the last axis of strided views for gfx950.
//
// Selection kernel (rows up to 65536 elements, limit up to 1024): one workgroup
// per row reads the row exactly once into registers as order-preserving
// unsigned keys, finds the limit-th best key with a most-significant-digit
// radix select over LDS histograms (no further global reads), breaks ties at
// the threshold by lowest source index with the same select over the indices,
// compacts the winners into LDS, orders them with a bitonic network and writes
// values and indices.  Among equal values the lowest index always comes first.
//
// Anything larger goes through the stable segmented argsort and keeps the first
// `limit` entries of each row.
#include <cstring>
#include <type_traits>

#include "common.hip.h"

namespace dlfx {

// from sort.hip
size_t argsort_scratch_bytes_impl(int dtype, int64_t m, int64_t n);
int argsort_contiguous(hipStream_t stream, int dir, int dtype, int rank, const int64_t* dims,
                       const void* x, const int64_t* x_strides, void* y_contig, int32_t* idx_contig,
                       void* scratch, size_t scratch_bytes);

namespace {

constexpr int kRadix = 256;
constexpr int kMaxLimit = 1024;

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

template <typename K>
struct TopkIo {
    const K* x;
    DimMap xmap;
    int64_t sx;
    K* y;
    DimMap ymap;
    int64_t sy;
    void* idx;
    DimMap imap;
    int64_t si;
    int idx64, kind, largest;
};

constexpr int kCandCap = 4096;     // candidates kept in LDS after the pre-filter

template <typename K>
struct TopkShared {
    uint32_t hist[kRadix];
    uint32_t wave_tot[kRadix / kWave];
    uint32_t scan_tot[16];
    uint32_t sel_digit, sel_k, sel_ties, count;
    K out_ord[kMaxLimit];
    uint32_t out_idx[kMaxLimit];
    K cand_ord[kCandCap];
    uint32_t cand_idx[kCandCap];
};

// One radix-select step over the values val(i) of the items for which part(i)
// holds: picks the digit (at `shift`) that contains the kk-th largest
// participating value.  Results: sm.sel_digit, sm.sel_k (rank inside that
// digit), sm.sel_ties (its population).  sm.hist must be all zero on entry and is
// all zero again on return.
template <int BLOCK, int ITEMS, bool ROLLED, typename K, typename Val, typename Part>
__device__ __forceinline__ void select_digit(TopkShared<K>& sm, int shift, uint32_t kk, Val val, Part part) {
    const int tid = threadIdx.x;
    const int lane = lane_id();
    auto count_item = [&](int i) {
        const bool in = part(i);
        const uint32_t d = static_cast<uint32_t>(val(i) >> shift) & 0xffu;
        // a wave whose participants all share the digit adds once
        const unsigned long long in_mask = __ballot(in);
        if (in_mask == 0ull) return;
        const int first = __ffsll(static_cast<long long>(in_mask)) - 1;
        const uint32_t d0 = __shfl(d, first, kWave);
        if (__ballot(in && d != d0) == 0ull) {
            if (lane == first) atomicAdd(&sm.hist[d0], static_cast<uint32_t>(__popcll(in_mask)));
        } else if (in) {
            atomicAdd(&sm.hist[d], 1u);
        }
    };
    if constexpr (ROLLED) {
#pragma unroll 1
        for (int i = 0; i < ITEMS; ++i) count_item(i);
    } else {
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) count_item(i);
    }
    __syncthreads();
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
    __syncthreads();
}

// The kk-th largest of the values val(i) over the items with part(i): most significant
// byte first.  Returns the value; *rank_in_ties / *ties describe how many of the elements
// equal to it still have to be taken and how many there are.
template <int BLOCK, int ITEMS, bool ROLLED, typename V, typename K, typename Val, typename Valid>
__device__ __forceinline__ V kth_largest(TopkShared<K>& sm, uint32_t kk, Val val, Valid valid,
                                         uint32_t* rank_in_ties, uint32_t* ties) {
    V prefix = 0;
#pragma unroll 1
    for (int pass = static_cast<int>(sizeof(V)) - 1; pass >= 0; --pass) {
        const int shift = 8 * pass;
        const V hi_mask = (pass == static_cast<int>(sizeof(V)) - 1) ? V(0) : static_cast<V>(~V(0) << (shift + 8));
        select_digit<BLOCK, ITEMS, ROLLED>(sm, shift, kk, val, [&](int i) {
            return valid(i) && ((val(i) ^ prefix) & hi_mask) == 0;
        });
        prefix |= static_cast<V>(sm.sel_digit) << shift;
        kk = sm.sel_k;
        *ties = sm.sel_ties;
    }
    *rank_in_ties = kk;
    return prefix;
}

// Exact selection of the `limit` best of the items (ord(i), idx(i)), best = larger image,
// then lower index; writes them in that order.  Padding items carry image 0 and an index
// that is not below the row length: they lose every tie, and limit <= row length, so no
// validity test is needed.
template <int BLOCK, int ITEMS, bool ROLLED, typename K, typename Ord, typename Idx>
__device__ __forceinline__ void select_and_emit(TopkShared<K>& sm, const TopkIo<K>& io, int64_t row, const K* xr,
                                                int limit, Ord ord, Idx idx) {
    const int tid = threadIdx.x;
    if (tid == 0) sm.count = 0;

    uint32_t kk = 0, ties = 0;
    const K threshold = kth_largest<BLOCK, ITEMS, ROLLED, K>(sm, static_cast<uint32_t>(limit), ord, [](int) { return true; }, &kk, &ties);
    // kk of the `ties` elements equal to the threshold are taken: those with the lowest indices,
    // i.e. the kk largest images of ~index
    uint32_t idx_limit = 0xffffffffu;
    if (kk < ties) {
        uint32_t k2 = 0, t2 = 0;
        const uint32_t inv = kth_largest<BLOCK, ITEMS, ROLLED, uint32_t>(
            sm, kk, [&](int i) { return ~idx(i); }, [&](int i) { return ord(i) == threshold; }, &k2, &t2);
        idx_limit = ~inv;
    }

    // ---- compact the winners
    auto take = [&](int i) {
        const uint32_t ix = idx(i);
        const K o = ord(i);
        if (o > threshold || (o == threshold && ix <= idx_limit)) {
            const uint32_t slot = atomicAdd(&sm.count, 1u);
            if (slot < kMaxLimit) {
                sm.out_ord[slot] = o;
                sm.out_idx[slot] = ix;
            }
        }
    };
    if constexpr (ROLLED) {
#pragma unroll 1
        for (int i = 0; i < ITEMS; ++i) take(i);
    } else {
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) take(i);
    }
    int kp = 1;
    while (kp < limit) kp <<= 1;
    __syncthreads();
    for (int i = limit + tid; i < kp; i += BLOCK) {
        sm.out_ord[i] = 0;
        sm.out_idx[i] = 0xffffffffu;      // padding: worse than any real entry
    }
    __syncthreads();

    // ---- bitonic network: best first (larger image, then lower index)
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
            __syncthreads();
        }
    }

    // ---- write
    K* yr = io.y + io.ymap.at(row);
    const int64_t ir = io.imap.at(row);
    for (int j = tid; j < limit; j += BLOCK) {
        const uint32_t ix = sm.out_idx[j];
        K bits = from_ord<K>(sm.out_ord[j], io.kind, io.largest);
        if (io.kind == kKeyFloat && (bits << 1) == 0) bits = xr[static_cast<int64_t>(ix) * io.sx];   // keep the zero's sign
        yr[j * io.sy] = bits;
        if (io.idx64) static_cast<int64_t*>(io.idx)[ir + j * io.si] = static_cast<int64_t>(ix);
        else static_cast<int32_t*>(io.idx)[ir + j * io.si] = static_cast<int32_t>(ix);
    }
}

// ALIGNED: the axis is contiguous and every row starts on a 16-byte boundary (checked on the
// host), so rows are read with 128-bit loads off one base register.
template <typename K, int BLOCK, int ITEMS, bool ALIGNED>
__global__ __launch_bounds__(BLOCK) void topk_select(TopkIo<K> io, int64_t n, int limit) {
    constexpr int V = (16 / sizeof(K) < ITEMS) ? 16 / sizeof(K) : ITEMS;
    constexpr int G = ITEMS / V;
    constexpr int WAVES = BLOCK / kWave;
    using VecT = Vec<K, V>;
    __shared__ TopkShared<K> sm;

    const int tid = threadIdx.x;
    const int lane = lane_id();
    const int w = tid / kWave;
    const int64_t row = blockIdx.x;
    const K* xr = io.x + io.xmap.at(row);
    if (tid < kRadix) sm.hist[tid] = 0;

    // item (g, e) of thread t is element ((g*BLOCK + t)*V + e) of the row
    const uint32_t n32 = static_cast<uint32_t>(n);        // rows here have at most 65536 elements
    const uint32_t tid_v = static_cast<uint32_t>(tid) * V;
    auto index_of = [&](int i) -> uint32_t {
        return tid_v + static_cast<uint32_t>((i / V) * (BLOCK * V) + (i % V));
    };
    auto in_row = [&](int i) -> bool { return index_of(i) < n32; };

    if constexpr (BLOCK * ITEMS <= kCandCap) {
        // short rows: select straight from registers
        K ord[ITEMS];
#pragma unroll
        for (int i = 0; i < ITEMS; ++i)
            ord[i] = in_row(i) ? to_ord<K>(xr[static_cast<int64_t>(index_of(i)) * io.sx], io.kind, io.largest) : K(0);
        __syncthreads();
        select_and_emit<BLOCK, ITEMS, false>(sm, io, row, xr, limit, [&](int i) { return ord[i]; }, index_of);
    } else {
        K ord[ITEMS];
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const uint32_t i0 = tid_v + static_cast<uint32_t>(g * (BLOCK * V));
            if (ALIGNED && i0 + V <= n32) {
                const VecT a = *reinterpret_cast<const VecT*>(xr + i0);
#pragma unroll
                for (int e = 0; e < V; ++e) ord[g * V + e] = to_ord<K>(a.v[e], io.kind, io.largest);
            } else {
#pragma unroll
                for (int e = 0; e < V; ++e) {
                    const int64_t at = ALIGNED ? static_cast<int64_t>(i0 + e) : static_cast<int64_t>(i0 + e) * io.sx;
                    ord[g * V + e] = (i0 + e < n32) ? to_ord<K>(xr[at], io.kind, io.largest) : K(0);
                }
            }
        }
        // ---- pre-filter.  Split the threads into `groups` >= limit groups; the largest
        // element each group holds gives `groups` distinct elements, so the smallest of those
        // maxima cannot exceed the limit-th largest element of the row: everything below it is
        // out.  What is left is usually a few times `limit` elements.
        K tmax = 0;
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) tmax = ord[i] > tmax ? ord[i] : tmax;      // padding is 0
        int groups = 1;
        while (groups < limit && groups < BLOCK) groups <<= 1;
        const int span = BLOCK / groups;               // threads per group, a power of two
        auto kmax = [](K a, K b) { return a > b ? a : b; };
        auto kmin = [](K a, K b) { return a < b ? a : b; };
        K bound;
        if (span >= kWave) {
            const K wmax = wave_reduce(tmax, kmax);
            if (lane == 0) sm.cand_ord[w] = wmax;
            __syncthreads();
            bound = ~K(0);
            const int wpg = span / kWave;              // waves per group
            for (int g0 = 0; g0 < WAVES; g0 += wpg) {
                K gm = 0;
                for (int j = 0; j < wpg; ++j) gm = kmax(gm, sm.cand_ord[g0 + j]);
                bound = kmin(bound, gm);
            }
        } else {
            const K gmax = group_reduce(tmax, span, kmax);
            const K wmin = wave_reduce(gmax, kmin);
            if (lane == 0) sm.cand_ord[w] = wmin;
            __syncthreads();
            bound = ~K(0);
            for (int j = 0; j < WAVES; ++j) bound = kmin(bound, sm.cand_ord[j]);
        }
        uint32_t mine = 0;
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) mine += (ord[i] >= bound) ? 1u : 0u;
        const uint32_t incl = wave_scan_inclusive(mine, 0u, [](uint32_t a, uint32_t b) { return a + b; });
        if (lane == kWave - 1) sm.scan_tot[w] = incl;
        __syncthreads();
        uint32_t before = incl - mine, total = 0;
        for (int i = 0; i < WAVES; ++i) {
            const uint32_t t = sm.scan_tot[i];
            if (i < w) before += t;
            total += t;
        }
        if (total <= kCandCap && limit <= BLOCK) {
#pragma unroll
            for (int i = 0; i < ITEMS; ++i) {
                if (ord[i] >= bound) {
                    sm.cand_ord[before] = ord[i];
                    sm.cand_idx[before] = index_of(i);
                    ++before;
                }
            }
            __syncthreads();
            constexpr int CI = kCandCap / BLOCK;
            K cord[CI];
            uint32_t cidx[CI];
#pragma unroll
            for (int j = 0; j < CI; ++j) {
                const uint32_t slot = j * BLOCK + tid;
                cord[j] = slot < total ? sm.cand_ord[slot] : K(0);
                cidx[j] = slot < total ? sm.cand_idx[slot] : 0xffffffffu;
            }
            select_and_emit<BLOCK, CI, false>(sm, io, row, xr, limit, [&](int j) { return cord[j]; },
                                       [&](int j) { return cidx[j]; });
        } else {
            // the filter kept too much (e.g. long runs of equal values): exact selection over the
            // whole row, re-reading elements (they are cache resident) instead of holding them
            __syncthreads();
            select_and_emit<BLOCK, ITEMS, true>(
                sm, io, row, xr, limit,
                [&](int i) { return in_row(i) ? to_ord<K>(xr[static_cast<int64_t>(index_of(i)) * io.sx], io.kind, io.largest) : K(0); },
                index_of);
        }
    }
}

// Fallback epilogue: first `limit` entries of each row of a full stable argsort.
template <typename K>
__global__ __launch_bounds__(256) void topk_take(const K* __restrict__ ys, const int32_t* __restrict__ is,
                                                  int64_t m, int64_t n, int64_t limit, TopkIo<K> io) {
    const int64_t g = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (g >= m * limit) return;
    const int64_t row = g / limit, j = g - row * limit;
    io.y[io.ymap.at(row) + j * io.sy] = ys[row * n + j];
    const int32_t ix = is[row * n + j];
    if (io.idx64) static_cast<int64_t*>(io.idx)[io.imap.at(row) + j * io.si] = ix;
    else static_cast<int32_t*>(io.idx)[io.imap.at(row) + j * io.si] = ix;
}

bool selection_fits(size_t key_size, int64_t n, int64_t limit) {
    if (limit > kMaxLimit) return false;
    return n <= (key_size == 4 ? 65536 : 32768);
}

template <typename K>
int run_top_k(hipStream_t stream, int64_t limit, int dir, int kind, int dtype, int index_dtype,
              int rank, const int64_t* x_dims, const int64_t* y_dims,
              const void* x, const int64_t* xs, void* y, const int64_t* ys, void* idx, const int64_t* is,
              void* scratch, size_t scratch_bytes) {
    const int64_t n = x_dims[rank - 1];
    const int64_t m = view_size(rank, x_dims) / n;
    TopkIo<K> io;
    std::memset(&io, 0, sizeof(io));
    io.x = static_cast<const K*>(x);
    io.y = static_cast<K*>(y);
    io.idx = idx;
    if (!make_dim_map(x_dims, xs, 0, rank - 1, &io.xmap) || !make_dim_map(y_dims, ys, 0, rank - 1, &io.ymap) ||
        !make_dim_map(y_dims, is, 0, rank - 1, &io.imap))
        return DLFX_ERR_RANK;
    io.sx = xs[rank - 1];
    io.sy = ys[rank - 1];
    io.si = is[rank - 1];
    io.idx64 = index_dtype == DLFX_I64;
    io.kind = kind;
    io.largest = dir ? 1 : 0;
    if (m > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;

    if (selection_fits(sizeof(K), n, limit)) {
        const dim3 grid(static_cast<unsigned>(m));
        const int lim = static_cast<int>(limit);
        bool aligned = io.sx == 1 && reinterpret_cast<uintptr_t>(io.x) % 16 == 0;
        for (int i = 0; i < io.xmap.rank; ++i) aligned = aligned && io.xmap.strides[i] % (16 / static_cast<int64_t>(sizeof(K))) == 0;
#define DLFX_TOPK(BLOCK, ITEMS)                                                                     \
    do {                                                                                            \
        if (aligned) topk_select<K, BLOCK, ITEMS, true><<<grid, dim3(BLOCK), 0, stream>>>(io, n, lim); \
        else topk_select<K, BLOCK, ITEMS, false><<<grid, dim3(BLOCK), 0, stream>>>(io, n, lim);      \
    } while (0)
        if (n <= 256) DLFX_TOPK(256, 1);
        else if (n <= 1024) DLFX_TOPK(256, 4);
        else if (n <= 2048) DLFX_TOPK(1024, 2);
        else if (n <= 4096) DLFX_TOPK(1024, 4);
        else if (n <= 8192) DLFX_TOPK(1024, 8);
        else if (n <= 16384) DLFX_TOPK(1024, 16);
        else if (n <= 32768) {
            if (lim <= 512) DLFX_TOPK(512, 64);
            else DLFX_TOPK(1024, 32);
        } else {
            if constexpr (sizeof(K) == 4) DLFX_TOPK(1024, 64);
            else return DLFX_ERR_TOO_LARGE;
        }
#undef DLFX_TOPK
        DLFX_CHECK_LAUNCH();
        return DLFX_OK;
    }

    // full stable argsort into scratch, then keep the head of each row
    const size_t ysz = align_up(static_cast<size_t>(m) * n * sizeof(K), 256);
    const size_t isz = align_up(static_cast<size_t>(m) * n * 4, 256);
    const size_t need = ysz + isz + argsort_scratch_bytes_impl(dtype, m, n);
    if (!scratch || scratch_bytes < need) return DLFX_ERR_SCRATCH_TOO_SMALL;
    char* base = static_cast<char*>(scratch);
    K* ysorted = reinterpret_cast<K*>(base);
    int32_t* isorted = reinterpret_cast<int32_t*>(base + ysz);
    int st = argsort_contiguous(stream, dir ? 1 : 0, dtype, rank, x_dims, x, xs, ysorted, isorted,
                                base + ysz + isz, scratch_bytes - ysz - isz);
    if (st != DLFX_OK) return st;
    const int64_t total = m * limit;
    if (ceil_div(total, 256) > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
    topk_take<K><<<dim3(static_cast<unsigned>(ceil_div(total, 256))), dim3(256), 0, stream>>>(ysorted, isorted, m, n, limit, io);
    DLFX_CHECK_LAUNCH();
    return DLFX_OK;
}

}  // namespace
}  // namespace dlfx

using namespace dlfx;

extern "C" size_t dlfx_top_k_scratch_bytes(int dtype, int64_t m, int64_t n, int64_t limit) {
    const size_t es = dtype_size(dtype);
    if (!es || m <= 0 || n <= 0) return 0;
    if (selection_fits(es, n, limit)) return 0;
    return align_up(static_cast<size_t>(m) * n * es, 256) + align_up(static_cast<size_t>(m) * n * 4, 256) +
           argsort_scratch_bytes_impl(dtype, m, n);
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
    case DLFX_F32: return run_top_k<uint32_t>(s, limit, dir, kKeyFloat, dtype, index_dtype, rank, x_dims, y_dims, xp, x_strides, yp, y_strides, ip, i_strides, scratch, scratch_bytes);
    case DLFX_I32: return run_top_k<uint32_t>(s, limit, dir, kKeyInt, dtype, index_dtype, rank, x_dims, y_dims, xp, x_strides, yp, y_strides, ip, i_strides, scratch, scratch_bytes);
    case DLFX_F64: return run_top_k<uint64_t>(s, limit, dir, kKeyFloat, dtype, index_dtype, rank, x_dims, y_dims, xp, x_strides, yp, y_strides, ip, i_strides, scratch, scratch_bytes);
    case DLFX_I64: return run_top_k<uint64_t>(s, limit, dir, kKeyInt, dtype, index_dtype, rank, x_dims, y_dims, xp, x_strides, yp, y_strides, ip, i_strides, scratch, scratch_bytes);
    default: return DLFX_ERR_UNSUPPORTED_DTYPE;
    }
}
