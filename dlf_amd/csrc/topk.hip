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
template <> struct KeyBits<uint32_t> { static constexpr int kBytes = 4; static constexpr uint32_t kSign = 0x80000000u; };
template <> struct KeyBits<uint64_t> { static constexpr int kBytes = 8; static constexpr uint64_t kSign = 0x8000000000000000ull; };

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

template <typename K>
struct TopkShared {
    uint32_t hist[kRadix];
    uint32_t wave_tot[kRadix / kWave];
    uint32_t sel_digit, sel_k, sel_ties, count;
    K out_ord[kMaxLimit];
    uint32_t out_idx[kMaxLimit];
};

// One radix-select step over the values val(i) of the items for which part(i)
// holds: picks the digit (at `shift`) that contains the kk-th largest
// participating value.  Results: sm.sel_digit, sm.sel_k (rank inside that
// digit), sm.sel_ties (its population).
template <int BLOCK, int ITEMS, typename K, typename Val, typename Part>
__device__ __forceinline__ void select_digit(TopkShared<K>& sm, int shift, uint32_t kk, Val val, Part part) {
    const int tid = threadIdx.x;
    const int lane = lane_id();
    for (int i = tid; i < kRadix; i += BLOCK) sm.hist[i] = 0;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        const bool in = part(i);
        const uint32_t d = static_cast<uint32_t>(val(i) >> shift) & 0xffu;
        // a wave whose participants all share the digit adds once
        const unsigned long long in_mask = __ballot(in);
        if (in_mask == 0ull) continue;
        const int first = __ffsll(static_cast<long long>(in_mask)) - 1;
        const uint32_t d0 = __shfl(d, first, kWave);
        if (__ballot(in && d != d0) == 0ull) {
            if (lane == first) atomicAdd(&sm.hist[d0], static_cast<uint32_t>(__popcll(in_mask)));
        } else if (in) {
            atomicAdd(&sm.hist[d], 1u);
        }
    }
    __syncthreads();
    // thread t < 256 looks at digit 255 - t, so an inclusive scan over t is a suffix sum over digits
    const uint32_t d = kRadix - 1 - tid;
    const int w = tid / kWave;
    uint32_t h = 0, incl = 0;
    if (tid < kRadix) {
        h = sm.hist[d];
        incl = wave_scan_inclusive(h, 0u, [](uint32_t a, uint32_t b) { return a + b; });
        if (lane == kWave - 1) sm.wave_tot[w] = incl;
    }
    __syncthreads();
    if (tid < kRadix) {
        for (int i = 0; i < w; ++i) incl += sm.wave_tot[i];
        const uint32_t above = incl - h;              // participants with a larger digit
        if (incl >= kk && above < kk) {
            sm.sel_digit = d;
            sm.sel_k = kk - above;
            sm.sel_ties = h;
        }
    }
    __syncthreads();
}

template <typename K, int BLOCK, int ITEMS>
__global__ __launch_bounds__(BLOCK) void topk_select(TopkIo<K> io, int64_t n, int limit) {
    constexpr int V = (16 / sizeof(K) < ITEMS) ? 16 / sizeof(K) : ITEMS;
    constexpr int G = ITEMS / V;
    using VecT = Vec<K, V>;
    __shared__ TopkShared<K> sm;

    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x;
    const K* xr = io.x + io.xmap.at(row);

    // item (g, e) of thread t is element ((g*BLOCK + t)*V + e) of the row
    K ord[ITEMS];
    const bool vec_ok = io.sx == 1 && (reinterpret_cast<uintptr_t>(xr) % (sizeof(K) * V) == 0);
#pragma unroll
    for (int g = 0; g < G; ++g) {
        const int64_t i0 = (static_cast<int64_t>(g) * BLOCK + tid) * V;
        if (vec_ok && i0 + V <= n) {
            const VecT a = *reinterpret_cast<const VecT*>(xr + i0);
#pragma unroll
            for (int e = 0; e < V; ++e) ord[g * V + e] = to_ord<K>(a.v[e], io.kind, io.largest);
        } else {
#pragma unroll
            for (int e = 0; e < V; ++e)
                ord[g * V + e] = (i0 + e < n) ? to_ord<K>(xr[(i0 + e) * io.sx], io.kind, io.largest) : K(0);
        }
    }
    auto index_of = [&](int i) -> uint32_t {
        return static_cast<uint32_t>((static_cast<int64_t>(i / V) * BLOCK + tid) * V + (i % V));
    };
    if (tid == 0) sm.count = 0;

    // ---- threshold key: the limit-th largest image
    K prefix = 0;
    uint32_t kk = static_cast<uint32_t>(limit);
    uint32_t ties = 0;
#pragma unroll 1
    for (int pass = KeyBits<K>::kBytes - 1; pass >= 0; --pass) {
        const int shift = 8 * pass;
        const K hi_mask = (pass == KeyBits<K>::kBytes - 1) ? K(0) : (~K(0) << (shift + 8));
        select_digit<BLOCK, ITEMS>(sm, shift, kk, [&](int i) { return ord[i]; }, [&](int i) {
            return index_of(i) < n && ((ord[i] ^ prefix) & hi_mask) == 0;
        });
        prefix |= static_cast<K>(sm.sel_digit) << shift;
        kk = sm.sel_k;
        ties = sm.sel_ties;
        __syncthreads();
    }
    // kk of the `ties` elements equal to the threshold are taken: those with the lowest indices
    uint32_t idx_limit = 0xffffffffu;
    if (kk < ties) {
        uint32_t iprefix = 0;        // select over ~index: the largest images are the lowest indices
#pragma unroll 1
        for (int pass = 3; pass >= 0; --pass) {
            const int shift = 8 * pass;
            const uint32_t hi_mask = (pass == 3) ? 0u : (~0u << (shift + 8));
            select_digit<BLOCK, ITEMS>(sm, shift, kk, [&](int i) { return ~index_of(i); }, [&](int i) {
                return index_of(i) < n && ord[i] == prefix && ((~index_of(i) ^ iprefix) & hi_mask) == 0;
            });
            iprefix |= sm.sel_digit << shift;
            kk = sm.sel_k;
            __syncthreads();
        }
        idx_limit = ~iprefix;
    }

    // ---- compact the winners
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        const uint32_t ix = index_of(i);
        if (ix < n && (ord[i] > prefix || (ord[i] == prefix && ix <= idx_limit))) {
            const uint32_t slot = atomicAdd(&sm.count, 1u);
            if (slot < kMaxLimit) {
                sm.out_ord[slot] = ord[i];
                sm.out_idx[slot] = ix;
            }
        }
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
                const bool descending_block = (i & size) == 0;      // best first in this block
                if (j_better == descending_block) {
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
#define DLFX_TOPK(BLOCK, ITEMS) topk_select<K, BLOCK, ITEMS><<<grid, dim3(BLOCK), 0, stream>>>(io, n, lim)
        if (n <= 256) DLFX_TOPK(256, 1);
        else if (n <= 1024) DLFX_TOPK(256, 4);
        else if (n <= 2048) DLFX_TOPK(1024, 2);
        else if (n <= 4096) DLFX_TOPK(1024, 4);
        else if (n <= 8192) DLFX_TOPK(1024, 8);
        else if (n <= 16384) DLFX_TOPK(1024, 16);
        else if (n <= 32768) DLFX_TOPK(1024, 32);
        else {
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
