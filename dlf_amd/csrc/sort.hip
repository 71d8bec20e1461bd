// sort / argsort along the last axis of strided views for gfx950.
//
// Segmented least-significant-digit radix sort, 8 bits per pass, every row an
// independent segment:
//   1. sort_histogram: one read of the input builds, per row, the digit
//      histograms of every pass (they do not depend on the order of the keys).
//   2. sort_bases: exclusive scan of each histogram -> where each digit's run
//      starts inside the row.
//   3. sort_pass (once per digit): a tile of keys is ranked with wave-wide
//      digit matching (stable), gathered in LDS in its locally sorted order and
//      written out in runs; the offset of a tile inside a digit's run comes from
//      the counts of the row's earlier tiles, chained with decoupled look-back
//      over per-tile, per-digit status words.
// Keys are order-preserving unsigned images of the elements (sign flip for
// integers, sign-magnitude flip for floats, complemented for descending order),
// so equal elements keep their source order in both directions.  The first
// pass reads the strided input, the last pass writes the strided outputs; the
// passes in between ping-pong through contiguous scratch.
//
// No wait is unbounded: a tile that polled an earlier tile's status too long
// counts that tile's digits itself from the pass input, which nothing writes
// during the pass.
#include <cstring>
#include <type_traits>

#include "common.hip.h"

namespace dlfx {
namespace {

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / kWave;
constexpr int kRadix = 256;
constexpr int64_t kMaxRow = (int64_t(1) << 27) - 1;   // counts share a status word with 5 tag bits

int g_sort_poll_limit = 2048;

enum KeyKind { kKeyInt = 0, kKeyFloat = 1 };

template <typename K>
struct KeyTraits;
template <>
struct KeyTraits<uint32_t> {
    static constexpr int kPasses = 4;
    static constexpr uint32_t kSign = 0x80000000u;
};
template <>
struct KeyTraits<uint64_t> {
    static constexpr int kPasses = 8;
    static constexpr uint64_t kSign = 0x8000000000000000ull;
};

template <typename K>
__device__ __forceinline__ K encode_key(K bits, int kind, int descending) {
    constexpr K S = KeyTraits<K>::kSign;
    K k = (kind == kKeyFloat) ? ((bits & S) ? ~bits : (bits | S)) : (bits ^ S);
    return descending ? ~k : k;
}
template <typename K>
__device__ __forceinline__ K decode_key(K k, int kind, int descending) {
    constexpr K S = KeyTraits<K>::kSign;
    if (descending) k = ~k;
    return (kind == kKeyFloat) ? ((k & S) ? (k & ~S) : ~k) : (k ^ S);
}

// Where a pass reads its keys and writes them.
template <typename K>
struct PassIo {
    // input
    const K* src_keys;        // contiguous [m][n] (null on the first pass)
    const uint32_t* src_vals; // contiguous [m][n] (null on the first pass / keys only)
    const K* x;               // strided input, read on the first pass
    DimMap xmap;
    int64_t sx;
    // output
    K* dst_keys;              // contiguous [m][n] (null on the last pass)
    uint32_t* dst_vals;
    K* y;                     // strided value output of the last pass (may be null)
    DimMap ymap;
    int64_t sy;
    void* idx;                // strided index output of the last pass (may be null)
    DimMap imap;
    int64_t si;
    int idx64;
    int first, last;
    int kind, descending;
    int canon_zero;           // argsort of floats: -0.0 and +0.0 are one key
    int restore_zero;         // ... and the value written for a zero key is re-read from x
};

template <typename K>
__device__ __forceinline__ K load_key(const PassIo<K>& io, int64_t row, int64_t row_n, const K* xrow, int64_t i) {
    if (io.first) {
        K bits = xrow[i * io.sx];
        if (io.canon_zero && (bits << 1) == 0) bits = 0;      // -0.0 -> +0.0
        return encode_key<K>(bits, io.kind, io.descending);
    }
    return io.src_keys[row * row_n + i];
}

// ------------------------------------------------------------------ histograms
template <typename K>
__global__ __launch_bounds__(kBlock) void sort_histogram(PassIo<K> io, int64_t n, int64_t chunk, int64_t chunks_per_row,
                                                         uint32_t* __restrict__ ghist) {
    constexpr int P = KeyTraits<K>::kPasses;
    __shared__ uint32_t hist[P][kRadix];
    for (int i = threadIdx.x; i < P * kRadix; i += kBlock) (&hist[0][0])[i] = 0;
    __syncthreads();
    const int64_t row = blockIdx.x / chunks_per_row;
    const int64_t c = blockIdx.x - row * chunks_per_row;
    const K* xrow = io.x + io.xmap.at(row);
    const int64_t lo = c * chunk;
    const int64_t hi = (lo + chunk < n) ? lo + chunk : n;
    const int lane = lane_id();
    for (int64_t i0 = lo + (threadIdx.x - lane); i0 < hi; i0 += kBlock) {
        const int64_t i = i0 + lane;
        const bool live = i < hi;
        K key = 0;
        if (live) key = load_key<K>(io, row, n, xrow, i);
        const unsigned long long live_mask = __ballot(live);
#pragma unroll
        for (int p = 0; p < P; ++p) {
            const uint32_t d = static_cast<uint32_t>(key >> (8 * p)) & 0xffu;
            // a wave whose live keys share the digit adds once instead of 64 times to one word
            const uint32_t d0 = __builtin_amdgcn_readfirstlane(d);
            const bool uniform = __ballot(live && d != d0) == 0ull && (live_mask & 1ull);
            if (uniform) {
                if (lane == 0) atomicAdd(&hist[p][d0], static_cast<uint32_t>(__popcll(live_mask)));
            } else if (live) {
                atomicAdd(&hist[p][d], 1u);
            }
        }
    }
    __syncthreads();
    uint32_t* g = ghist + row * (P * kRadix);
    for (int i = threadIdx.x; i < P * kRadix; i += kBlock) {
        const uint32_t v = (&hist[0][0])[i];
        if (v) atomicAdd(&g[i], v);
    }
}

// In place: histogram -> exclusive prefix (start of each digit's run in the row).
__global__ __launch_bounds__(kRadix) void sort_bases(uint32_t* __restrict__ ghist) {
    __shared__ uint32_t wave_tot[kRadix / kWave];
    uint32_t* g = ghist + static_cast<int64_t>(blockIdx.x) * kRadix;
    const uint32_t v = g[threadIdx.x];
    const uint32_t incl = wave_scan_inclusive(v, 0u, [](uint32_t a, uint32_t b) { return a + b; });
    const int w = threadIdx.x / kWave;
    if (lane_id() == kWave - 1) wave_tot[w] = incl;
    __syncthreads();
    uint32_t pre = 0;
    for (int i = 0; i < w; ++i) pre += wave_tot[i];
    g[threadIdx.x] = pre + incl - v;
}

__global__ __launch_bounds__(kBlock) void sort_clear(uint32_t* __restrict__ p, int64_t words) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (i < words) p[i] = 0u;
}

// ------------------------------------------------------------------ one pass
// Status word of (tile, digit): [tag:4 | inclusive:1 | count:27]; a word is valid
// for pass p when its tag is p + 1, so the array is cleared once per sort.
constexpr uint32_t kCountMask = (1u << 27) - 1;
__device__ __forceinline__ uint32_t make_status(int pass, bool inclusive, uint32_t count) {
    return (static_cast<uint32_t>(pass + 1) << 28) | (inclusive ? (1u << 27) : 0u) | count;
}

template <typename K, bool PAIRS, int ITEMS>
struct PassShared {
    uint32_t wave_hist[kWaves][kRadix];       // per-wave digit counts, then per-wave offsets
    uint32_t help_hist[kRadix];               // digits of an earlier tile counted here when it is late
    uint32_t digit_start[kRadix];             // first tile-local position of each digit
    int64_t dst_base[kRadix];                 // global position of that digit's run start minus digit_start
    uint32_t scan_tmp[kWaves];
    int help_tile;
    K keys[kBlock * ITEMS];
    uint32_t vals[PAIRS ? kBlock * ITEMS : 1];
};

template <typename K, bool PAIRS, int ITEMS>
__global__ __launch_bounds__(kBlock) void sort_pass(PassIo<K> io, int pass, int64_t n, int64_t tiles_per_row,
                                                    const uint32_t* __restrict__ gbase,
                                                    uint32_t* __restrict__ status, int poll_limit) {
    constexpr int P = KeyTraits<K>::kPasses;
    constexpr int TILE = kBlock * ITEMS;
    constexpr int W = 4;    // status words of earlier tiles fetched per look-back step
    __shared__ PassShared<K, PAIRS, ITEMS> sm;

    const int tid = threadIdx.x;
    const int lane = lane_id();
    const int w = tid / kWave;
    const int64_t row = blockIdx.x / tiles_per_row;
    const int64_t t = blockIdx.x - row * tiles_per_row;
    const int64_t tile_base = t * TILE;
    const int valid = static_cast<int>((n - tile_base < TILE) ? n - tile_base : TILE);
    const K* xrow = io.first ? io.x + io.xmap.at(row) : nullptr;
    const int shift = 8 * pass;

    for (int i = tid; i < kWaves * kRadix; i += kBlock) (&sm.wave_hist[0][0])[i] = 0;
    if (tid == 0) sm.help_tile = -1;

    // ---- load: wave w owns [w*64*ITEMS, ...), item k of lane l is element k*64 + l of it
    K key[ITEMS];
    uint32_t val[PAIRS ? ITEMS : 1];
    const int seg = w * kWave * ITEMS;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const int li = seg + k * kWave + lane;
        const int64_t i = tile_base + li;
        if (li < valid) {
            key[k] = load_key<K>(io, row, n, xrow, i);
            if constexpr (PAIRS) val[k] = io.first ? static_cast<uint32_t>(i) : io.src_vals[row * n + i];
        } else {
            key[k] = ~K(0);      // padding sorts last and is never stored
            if constexpr (PAIRS) val[k] = 0;
        }
    }
    __syncthreads();

    // ---- rank inside the wave, in element order (stable)
    uint32_t rank[ITEMS];
    const unsigned long long lt_mask = (1ull << lane) - 1ull;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const uint32_t d = static_cast<uint32_t>(key[k] >> shift) & 0xffu;
        unsigned long long peers = ~0ull;
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            const bool bit = (d >> b) & 1u;
            const unsigned long long vote = __ballot(bit);
            peers &= bit ? vote : ~vote;
        }
        const uint32_t before = static_cast<uint32_t>(__popcll(peers & lt_mask));
        const uint32_t cnt = static_cast<uint32_t>(__popcll(peers));
        const uint32_t seen = sm.wave_hist[w][d];          // same word for all peers: a broadcast read
        rank[k] = seen + before;
        __builtin_amdgcn_wave_barrier();
        if (before == 0) sm.wave_hist[w][d] = seen + cnt;
        __builtin_amdgcn_wave_barrier();
    }
    __syncthreads();

    // ---- thread d owns digit d: wave offsets, tile count, position of the digit in the tile
    uint32_t count = 0;
#pragma unroll
    for (int i = 0; i < kWaves; ++i) {
        const uint32_t c = sm.wave_hist[i][tid];
        sm.wave_hist[i][tid] = count;
        count += c;
    }
    if (tid == kRadix - 1) count -= static_cast<uint32_t>(TILE - valid);     // padding is not part of the row
    const int64_t srow = (row * tiles_per_row) * kRadix;
    uint32_t* my_status = status + srow + t * kRadix + tid;
    if (t + 1 < tiles_per_row)
        __hip_atomic_store(my_status, make_status(pass, t == 0, count), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    {
        uint32_t padded = count + (tid == kRadix - 1 ? static_cast<uint32_t>(TILE - valid) : 0u);
        const uint32_t incl = wave_scan_inclusive(padded, 0u, [](uint32_t a, uint32_t b) { return a + b; });
        if (lane == kWave - 1) sm.scan_tmp[w] = incl;
        __syncthreads();
        uint32_t pre = 0;
        for (int i = 0; i < w; ++i) pre += sm.scan_tmp[i];
        sm.digit_start[tid] = pre + incl - padded;
    }

    // ---- look back over the row's earlier tiles for digit `tid`
    uint32_t before_tiles = 0;
    {
        int64_t p = t - 1;
        bool done = (t == 0);
        const uint32_t want_tag = static_cast<uint32_t>(pass + 1);
        for (;;) {
            int stuck = -1;
            while (!done) {
                uint32_t sw[W];
#pragma unroll
                for (int i = 0; i < W; ++i) {
                    const int64_t q = p - i;
                    sw[i] = (q >= 0) ? __hip_atomic_load(status + srow + q * kRadix + tid, __ATOMIC_RELAXED,
                                                         __HIP_MEMORY_SCOPE_AGENT)
                                     : make_status(pass, true, 0u);
                }
#pragma unroll
                for (int i = 0; i < W; ++i) {
                    if (done || stuck >= 0) continue;
                    const int64_t q = p - i;
                    uint32_t s = sw[i];
                    for (int polls = 0; (s >> 28) != want_tag && polls < poll_limit; ++polls) {
                        __builtin_amdgcn_s_sleep(1);
                        s = __hip_atomic_load(status + srow + q * kRadix + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                    if ((s >> 28) != want_tag) {
                        stuck = static_cast<int>(q);
                        p = q;                    // resume at this tile
                    } else {
                        before_tiles += s & kCountMask;
                        if (s & (1u << 27)) done = true;
                    }
                }
                if (stuck >= 0) break;
                p -= W;
            }
            // anyone still waiting?  then the whole workgroup counts that tile's digits itself
            if (stuck >= 0) atomicMax(&sm.help_tile, stuck);
            __syncthreads();
            const int help = sm.help_tile;
            if (help < 0) break;
            sm.help_hist[tid] = 0;
            __syncthreads();
            {
                const int64_t hb = static_cast<int64_t>(help) * TILE;
                const int hv = static_cast<int>((n - hb < TILE) ? n - hb : TILE);
                for (int li = tid; li < hv; li += kBlock) {
                    const K hk = load_key<K>(io, row, n, xrow, hb + li);
                    atomicAdd(&sm.help_hist[static_cast<uint32_t>(hk >> shift) & 0xffu], 1u);
                }
            }
            __syncthreads();
            if (stuck == help) {
                before_tiles += sm.help_hist[tid];
                p = static_cast<int64_t>(help) - 1;
                if (p < 0) done = true;
            }
            __syncthreads();
            if (tid == 0) sm.help_tile = -1;
            __syncthreads();
        }
    }
    if (t > 0 && t + 1 < tiles_per_row)
        __hip_atomic_store(my_status, make_status(pass, true, before_tiles + count), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    sm.dst_base[tid] = static_cast<int64_t>(gbase[(row * P + pass) * kRadix + tid]) + before_tiles -
                       static_cast<int64_t>(sm.digit_start[tid]);
    __syncthreads();

    // ---- gather the tile in its locally sorted order
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const uint32_t d = static_cast<uint32_t>(key[k] >> shift) & 0xffu;
        const uint32_t pos = sm.digit_start[d] + sm.wave_hist[w][d] + rank[k];
        sm.keys[pos] = key[k];
        if constexpr (PAIRS) sm.vals[pos] = val[k];
    }
    __syncthreads();

    // ---- write runs
    const int64_t row_off = row * n;
    K* yrow = (io.last && io.y) ? io.y + io.ymap.at(row) : nullptr;
    const int64_t irow = (io.last && io.idx) ? io.imap.at(row) : 0;
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const int lp = k * kBlock + tid;
        if (lp >= valid) continue;
        const K kk = sm.keys[lp];
        const uint32_t d = static_cast<uint32_t>(kk >> shift) & 0xffu;
        const int64_t dst = sm.dst_base[d] + lp;
        if (!io.last) {
            io.dst_keys[row_off + dst] = kk;
            if constexpr (PAIRS) io.dst_vals[row_off + dst] = sm.vals[lp];
        } else {
            uint32_t v = 0;
            if constexpr (PAIRS) v = sm.vals[lp];
            if (yrow) {
                K bits = decode_key<K>(kk, io.kind, io.descending);
                if constexpr (PAIRS) {
                    if (io.restore_zero && (bits << 1) == 0) bits = io.x[io.xmap.at(row) + static_cast<int64_t>(v) * io.sx];
                }
                yrow[dst * io.sy] = bits;
            }
            if constexpr (PAIRS) {
                if (io.idx) {
                    if (io.idx64) static_cast<int64_t*>(io.idx)[irow + dst * io.si] = static_cast<int64_t>(v);
                    else static_cast<int32_t*>(io.idx)[irow + dst * io.si] = static_cast<int32_t>(v);
                }
            }
        }
    }
}

// ------------------------------------------------------------------ host side
template <typename K>
constexpr int tile_items() { return 64 / sizeof(K); }       // 16 x u32 or 8 x u64 per thread

struct SortLayout {
    int64_t tiles_per_row;
    size_t hist_off, hist_bytes, status_off, status_bytes, keys_off[2], vals_off[2], total;
};

SortLayout sort_layout(size_t key_size, bool pairs, int64_t m, int64_t n) {
    SortLayout l;
    const int passes = key_size == 4 ? 4 : 8;
    const int64_t tile = kBlock * (64 / static_cast<int64_t>(key_size));
    l.tiles_per_row = ceil_div(n, tile);
    size_t off = 0;
    l.hist_off = off;
    l.hist_bytes = static_cast<size_t>(m) * passes * kRadix * 4;
    off += align_up(l.hist_bytes, 256);
    l.status_off = off;
    l.status_bytes = l.tiles_per_row > 1 ? static_cast<size_t>(m) * l.tiles_per_row * kRadix * 4 : 0;
    off += align_up(l.status_bytes, 256);
    for (int i = 0; i < 2; ++i) {
        l.keys_off[i] = off;
        off += align_up(static_cast<size_t>(m) * n * key_size, 256);
    }
    for (int i = 0; i < 2; ++i) {
        l.vals_off[i] = off;
        if (pairs) off += align_up(static_cast<size_t>(m) * n * 4, 256);
    }
    l.total = off;
    return l;
}

template <typename T>
bool ranges_overlap(int rank, const int64_t* dims, const T* x, const int64_t* sx, const T* y, const int64_t* sy) {
    int64_t xlo = 0, xhi = 0, ylo = 0, yhi = 0;
    for (int i = 0; i < rank; ++i) {
        const int64_t ex = (dims[i] - 1) * sx[i], ey = (dims[i] - 1) * sy[i];
        if (ex > 0) xhi += ex; else xlo += ex;
        if (ey > 0) yhi += ey; else ylo += ey;
    }
    return !(x + xhi < y + ylo || y + yhi < x + xlo);
}

struct SortArgs {
    int dir, kind;
    int rank;
    const int64_t* dims;
    const void* x; const int64_t* xs;
    void* y; const int64_t* ys;
    void* idx; const int64_t* is; int idx64;
    bool pairs;
};

template <typename K>
int run_sort(hipStream_t stream, const SortArgs& a, void* scratch, size_t scratch_bytes) {
    constexpr int P = KeyTraits<K>::kPasses;
    constexpr int ITEMS = tile_items<K>();
    const int64_t n = a.dims[a.rank - 1];
    const int64_t m = view_size(a.rank, a.dims) / n;
    if (n > kMaxRow) return DLFX_ERR_TOO_LARGE;
    const SortLayout l = sort_layout(sizeof(K), a.pairs, m, n);
    if (m * l.tiles_per_row > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
    if (!scratch || scratch_bytes < l.total) return DLFX_ERR_SCRATCH_TOO_SMALL;
    char* base = static_cast<char*>(scratch);

    PassIo<K> io;
    std::memset(&io, 0, sizeof(io));
    io.x = static_cast<const K*>(a.x);
    if (!make_dim_map(a.dims, a.xs, 0, a.rank - 1, &io.xmap)) return DLFX_ERR_RANK;
    io.sx = a.xs[a.rank - 1];
    io.y = static_cast<K*>(a.y);
    if (a.y) {
        if (!make_dim_map(a.dims, a.ys, 0, a.rank - 1, &io.ymap)) return DLFX_ERR_RANK;
        io.sy = a.ys[a.rank - 1];
    }
    io.idx = a.idx;
    if (a.idx) {
        if (!make_dim_map(a.dims, a.is, 0, a.rank - 1, &io.imap)) return DLFX_ERR_RANK;
        io.si = a.is[a.rank - 1];
    }
    io.idx64 = a.idx64;
    io.kind = a.kind;
    io.descending = a.dir ? 1 : 0;
    // -0.0 and +0.0 compare equal, so a stable argsort must order them by index: both
    // get +0.0's key and the value output re-reads the element (not possible when the
    // value output overwrites the input; then the two zeros order by sign)
    const bool y_over_x = a.y && ranges_overlap<K>(a.rank, a.dims, static_cast<const K*>(a.x), a.xs, static_cast<const K*>(a.y), a.ys);
    io.canon_zero = (a.pairs && a.kind == kKeyFloat && !y_over_x) ? 1 : 0;
    io.restore_zero = (io.canon_zero && a.y) ? 1 : 0;

    uint32_t* ghist = reinterpret_cast<uint32_t*>(base + l.hist_off);
    uint32_t* status = reinterpret_cast<uint32_t*>(base + l.status_off);
    const int64_t clear_words = static_cast<int64_t>((l.status_off + l.status_bytes) / 4);   // histograms + status
    sort_clear<<<dim3(static_cast<unsigned>(ceil_div(clear_words, kBlock))), dim3(kBlock), 0, stream>>>(ghist, clear_words);
    DLFX_CHECK_LAUNCH();

    io.first = 1;
    const int64_t chunk = 32768;
    const int64_t chunks_per_row = ceil_div(n, chunk);
    if (m * chunks_per_row > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
    sort_histogram<K><<<dim3(static_cast<unsigned>(m * chunks_per_row)), dim3(kBlock), 0, stream>>>(io, n, chunk, chunks_per_row, ghist);
    DLFX_CHECK_LAUNCH();
    sort_bases<<<dim3(static_cast<unsigned>(m * P)), dim3(kRadix), 0, stream>>>(ghist);
    DLFX_CHECK_LAUNCH();

    K* kbuf[2] = {reinterpret_cast<K*>(base + l.keys_off[0]), reinterpret_cast<K*>(base + l.keys_off[1])};
    uint32_t* vbuf[2] = {reinterpret_cast<uint32_t*>(base + l.vals_off[0]), reinterpret_cast<uint32_t*>(base + l.vals_off[1])};
    const dim3 grid(static_cast<unsigned>(m * l.tiles_per_row));
    for (int p = 0; p < P; ++p) {
        io.first = (p == 0);
        io.last = (p == P - 1);
        io.src_keys = io.first ? nullptr : kbuf[(p - 1) & 1];
        io.src_vals = (io.first || !a.pairs) ? nullptr : vbuf[(p - 1) & 1];
        io.dst_keys = io.last ? nullptr : kbuf[p & 1];
        io.dst_vals = (io.last || !a.pairs) ? nullptr : vbuf[p & 1];
        if (a.pairs)
            sort_pass<K, true, ITEMS><<<grid, dim3(kBlock), 0, stream>>>(io, p, n, l.tiles_per_row, ghist, status, g_sort_poll_limit);
        else
            sort_pass<K, false, ITEMS><<<grid, dim3(kBlock), 0, stream>>>(io, p, n, l.tiles_per_row, ghist, status, g_sort_poll_limit);
        DLFX_CHECK_LAUNCH();
    }
    return DLFX_OK;
}

int sort_entry(hipStream_t stream, int dtype, const SortArgs& a0, void* scratch, size_t scratch_bytes) {
    SortArgs a = a0;
    switch (dtype) {
    case DLFX_F32: a.kind = kKeyFloat; return run_sort<uint32_t>(stream, a, scratch, scratch_bytes);
    case DLFX_I32: a.kind = kKeyInt;   return run_sort<uint32_t>(stream, a, scratch, scratch_bytes);
    case DLFX_F64: a.kind = kKeyFloat; return run_sort<uint64_t>(stream, a, scratch, scratch_bytes);
    case DLFX_I64: a.kind = kKeyInt;   return run_sort<uint64_t>(stream, a, scratch, scratch_bytes);
    default: return DLFX_ERR_UNSUPPORTED_DTYPE;
    }
}

}  // namespace

bool set_sort_tuning(const char* key, int64_t value) {
    if (!std::strcmp(key, "sort_poll_limit") && value >= 0 && value <= (1 << 30)) {
        g_sort_poll_limit = static_cast<int>(value);
        return true;
    }
    return false;
}

// Used by top_k for rows or limits its selection kernel does not take: stable
// argsort of a strided view into contiguous value and int32 index arrays.
int argsort_contiguous(hipStream_t stream, int dir, int dtype, int rank, const int64_t* dims,
                       const void* x, const int64_t* x_strides, void* y_contig, int32_t* idx_contig,
                       void* scratch, size_t scratch_bytes) {
    if (rank < 1 || rank > 64) return DLFX_ERR_INVALID_ARGUMENT;
    int64_t cs[64];
    int64_t acc = 1;
    for (int i = rank - 1; i >= 0; --i) {
        cs[i] = acc;
        acc *= dims[i];
    }
    SortArgs a{};
    a.dir = dir;
    a.rank = rank;
    a.dims = dims;
    a.x = x;
    a.xs = x_strides;
    a.y = y_contig;
    a.ys = cs;
    a.idx = idx_contig;
    a.is = cs;
    a.idx64 = 0;
    a.pairs = true;
    return sort_entry(stream, dtype, a, scratch, scratch_bytes);
}


size_t argsort_scratch_bytes_impl(int dtype, int64_t m, int64_t n) {
    const size_t es = dtype_size(dtype);
    if (!es || m <= 0 || n <= 0) return 0;
    return sort_layout(es, true, m, n).total;
}

}  // namespace dlfx

using namespace dlfx;

extern "C" size_t dlfx_sort_scratch_bytes(int dtype, int64_t m, int64_t n) {
    const size_t es = dtype_size(dtype);
    if (!es || m <= 0 || n <= 0) return 0;
    return sort_layout(es, false, m, n).total;
}

extern "C" int dlfx_sort(dlfx_stream_t stream, int dir, int dtype, int rank, const int64_t* dims,
                         const void* x, int64_t x_offset, const int64_t* x_strides,
                         void* y, int64_t y_offset, const int64_t* y_strides,
                         void* scratch, size_t scratch_bytes) {
    if (!x || !y || rank < 1) return DLFX_ERR_INVALID_ARGUMENT;
    if (!view_ok(rank, dims, x_strides) || !view_ok(rank, dims, y_strides)) return DLFX_ERR_INVALID_ARGUMENT;
    const size_t es = dtype_size(dtype);
    if (!es) return DLFX_ERR_UNSUPPORTED_DTYPE;
    SortArgs a{};
    a.dir = dir;
    a.rank = rank;
    a.dims = dims;
    a.x = static_cast<const char*>(x) + x_offset * static_cast<int64_t>(es);
    a.xs = x_strides;
    a.y = static_cast<char*>(y) + y_offset * static_cast<int64_t>(es);
    a.ys = y_strides;
    a.pairs = false;
    return sort_entry(static_cast<hipStream_t>(stream), dtype, a, scratch, scratch_bytes);
}

extern "C" size_t dlfx_argsort_scratch_bytes(int dtype, int64_t m, int64_t n) {
    return argsort_scratch_bytes_impl(dtype, m, n);
}

extern "C" int dlfx_argsort(dlfx_stream_t stream, int dir, int dtype, int index_dtype,
                            int rank, const int64_t* dims,
                            const void* x, int64_t x_offset, const int64_t* x_strides,
                            void* y, int64_t y_offset, const int64_t* y_strides,
                            void* idx, int64_t i_offset, const int64_t* i_strides,
                            void* scratch, size_t scratch_bytes) {
    if (!x || !idx || rank < 1) return DLFX_ERR_INVALID_ARGUMENT;
    if (!view_ok(rank, dims, x_strides) || !view_ok(rank, dims, i_strides)) return DLFX_ERR_INVALID_ARGUMENT;
    if (y && !view_ok(rank, dims, y_strides)) return DLFX_ERR_INVALID_ARGUMENT;
    if (index_dtype != DLFX_I32 && index_dtype != DLFX_I64) return DLFX_ERR_UNSUPPORTED_DTYPE;
    const size_t es = dtype_size(dtype);
    if (!es) return DLFX_ERR_UNSUPPORTED_DTYPE;
    SortArgs a{};
    a.dir = dir;
    a.rank = rank;
    a.dims = dims;
    a.x = static_cast<const char*>(x) + x_offset * static_cast<int64_t>(es);
    a.xs = x_strides;
    a.y = y ? static_cast<char*>(y) + y_offset * static_cast<int64_t>(es) : nullptr;
    a.ys = y_strides;
    a.idx64 = index_dtype == DLFX_I64;
    a.idx = static_cast<char*>(idx) + i_offset * (a.idx64 ? 8 : 4);
    a.is = i_strides;
    a.pairs = true;
    return sort_entry(static_cast<hipStream_t>(stream), dtype, a, scratch, scratch_bytes);
}
