// sort / argsort along the last axis of strided views for gfx950.
//
// Which way a row goes: rows of up to 64 / 512 elements are sorted by one wavefront in
// registers, rows of up to 4096 (16-bit keys), 8192 (8-byte) or 16384 (4-byte keys) by one workgroup
// on chip, longer rows of 4- and 8-byte keys by the bucket route of sort_split.hip (run_split),
// which sorts every row of such a call.  What is left - 16-bit keys, rows longer than 256 of the
// largest buckets hold (about 2.6 million keys) - is sorted here:
//
// Segmented least-significant-digit radix sort, 8 bits per pass, every row an
// independent segment:
//   1. sort_histogram: one read of the input builds, per row, the digit
//      histograms of every pass (they do not depend on the order of the keys);
//      the workgroup that adds a row's last chunk turns each histogram into its
//      exclusive scan -> where each digit's run starts inside the row.
//   2. sort_pass (once per digit): a tile of keys is ranked with wave-wide
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

#include "sort_common.hip.h"

namespace dlfx {
namespace {

#ifndef DLFX_SORT_WAVES
#define DLFX_SORT_WAVES 4
#endif
constexpr int kBlock = 256;
#ifndef DLFX_SORT_PASS_BLOCK
#define DLFX_SORT_PASS_BLOCK 256
#endif
constexpr int kPassBlock = DLFX_SORT_PASS_BLOCK;       // threads of a sort_pass workgroup
constexpr int kPassWaves = kPassBlock / kWave;
constexpr int64_t kMaxRow = (int64_t(1) << 27) - 1;   // counts share a status word with 5 tag bits

int g_sort_poll_limit = 2048;

#ifdef DLFX_SORT_TIMING
// Debug builds only: shader-clock cycles spent by thread 0 of every workgroup in each phase.
constexpr int kPhaseSlots = 16384;
__device__ unsigned long long g_phase_cycles[kPhaseSlots * 8];
#define DLFX_PHASE(i) do { if (threadIdx.x == 0) { const long long now_ = clock64(); g_phase_cycles[(blockIdx.x % kPhaseSlots) * 8 + (i)] += static_cast<unsigned long long>(now_ - phase_t_); phase_t_ = now_; } } while (0)
#define DLFX_PHASE_BEGIN() long long phase_t_ = clock64()
#else
#define DLFX_PHASE(i) do { } while (0)
#define DLFX_PHASE_BEGIN() do { } while (0)
#endif

// ------------------------------------------------------------------ bases
// In place: one histogram of a row -> exclusive prefix (start of each digit's run in the row),
// by the 256 threads of a workgroup.  *moves receives the bits of the digit that are not the
// same in all keys of the row: none means the pass would not change the order of the row (the
// row then skips it), and the ranking only needs to look at those bits.  `all_bits` forces
// every pass of every row to run.  The counts were added by other workgroups of this launch:
// they are read where those additions were made, past this part's own cache.
__device__ __forceinline__ void bases_of_pass(uint32_t* __restrict__ g, uint32_t* __restrict__ moves, int all_bits) {
    __shared__ uint32_t wave_tot[kRadix / kWave];
    __shared__ uint32_t wave_or[kRadix / kWave], wave_and[kRadix / kWave];
    __syncthreads();                                   // the pass before has left these words
    const uint32_t v = __hip_atomic_load(g + threadIdx.x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint32_t incl = wave_scan_inclusive(v, 0u, [](uint32_t a, uint32_t b) { return a + b; });
    const uint32_t ors = wave_reduce(v ? threadIdx.x : 0u, [](uint32_t a, uint32_t b) { return a | b; });
    const uint32_t ands = wave_reduce(v ? threadIdx.x : 0xffu, [](uint32_t a, uint32_t b) { return a & b; });
    const int w = threadIdx.x / kWave;
    if (lane_id() == kWave - 1) {
        wave_tot[w] = incl;
        wave_or[w] = ors;
        wave_and[w] = ands;
    }
    __syncthreads();
    uint32_t pre = 0;
    for (int i = 0; i < w; ++i) pre += wave_tot[i];
    g[threadIdx.x] = pre + incl - v;
    if (threadIdx.x == 0) {
        uint32_t o = 0, a = 0xffu;
        for (int i = 0; i < kRadix / kWave; ++i) {
            o |= wave_or[i];
            a &= wave_and[i];
        }
        *moves = all_bits ? 0xffu : (o ^ a);
    }
}

// ------------------------------------------------------------------ histograms
// One read of the input builds the digit histograms of every pass for a chunk of a row.
// Each workgroup keeps kHistCopies interleaved copies of every histogram (a lane adds to copy
// lane % kHistCopies), so that the few distinct values of a low-entropy digit do not
// serialise all 64 lanes on one LDS word; a digit that is the same in a whole batch of
// keys (constant bytes: small integers, narrow float ranges) is added once per wave.
template <typename K>
__global__ __launch_bounds__(kBlock) void sort_histogram(PassIo<K> io, int64_t n, int64_t chunk, int64_t chunks_per_row, int64_t units,
                                                         uint32_t* __restrict__ ghist, uint32_t* __restrict__ arrived,
                                                         uint32_t* __restrict__ moves, int all_bits) {
    constexpr int P = KeyTraits<K>::kPasses;
    static_assert(kBlock == kRadix, "a thread per digit when the row's histograms are scanned");
    __shared__ uint32_t last_chunk;
    constexpr int U = 32 / sizeof(K);                 // keys in flight per thread
    constexpr int R = 32 / P;                         // copies: 8 (32-bit keys) or 4 (64-bit keys): 32 KB
    __shared__ uint32_t hist[P * kRadix * R];
    for (int64_t unit = blockIdx.x; unit < units; unit += gridDim.x) {       // (row, chunk) pairs
    const int64_t row = unit / chunks_per_row;
    __syncthreads();                                   // the previous unit's histogram has left
    for (int i = threadIdx.x; i < P * kRadix * R; i += kBlock) hist[i] = 0;
    __syncthreads();
    const int64_t c = unit - row * chunks_per_row;
    const K* xrow = io.x + io.xmap.at(row);
    const int64_t lo = c * chunk;
    const int64_t hi = (lo + chunk < n) ? lo + chunk : n;
    const int lane = lane_id();
    const int copy = lane % R;
    // wave-uniform trip count: every wave walks whole batches of U * 256 keys
    for (int64_t b0 = lo; b0 < hi; b0 += static_cast<int64_t>(kBlock) * U) {
        const int64_t i0 = b0 + threadIdx.x;
        K key[U];
        const bool whole = b0 + static_cast<int64_t>(kBlock) * U <= hi;
        if (whole) {
#pragma unroll
            for (int u = 0; u < U; ++u) key[u] = xrow[(i0 + static_cast<int64_t>(u) * kBlock) * io.sx];
#pragma unroll
            for (int u = 0; u < U; ++u) key[u] = key_of_element<K>(io, key[u]);
            const K key0 = lane_read(key[0], 0);
            K diff = 0;
#pragma unroll
            for (int u = 0; u < U; ++u) diff |= key[u] ^ key0;
#pragma unroll
            for (int p = 0; p < P; ++p) {
                uint32_t* h = hist + p * kRadix * R;
                if (__ballot(((diff >> (8 * p)) & 0xffu) != 0) == 0ull) {
                    if (lane == 0) atomicAdd(&h[(static_cast<uint32_t>(key0 >> (8 * p)) & 0xffu) * R], static_cast<uint32_t>(U * kWave));
                } else {
#pragma unroll
                    for (int u = 0; u < U; ++u) atomicAdd(&h[(static_cast<uint32_t>(key[u] >> (8 * p)) & 0xffu) * R + copy], 1u);
                }
            }
        } else {
            for (int u = 0; u < U; ++u) {
                const int64_t i = i0 + static_cast<int64_t>(u) * kBlock;
                if (i < hi) {
                    const K k1 = key_of_element<K>(io, xrow[i * io.sx]);
#pragma unroll
                    for (int p = 0; p < P; ++p)
                        atomicAdd(&hist[p * kRadix * R + (static_cast<uint32_t>(k1 >> (8 * p)) & 0xffu) * R + copy], 1u);
                }
            }
        }
    }
    __syncthreads();
    uint32_t* g = ghist + row * (P * kRadix);
    for (int i = threadIdx.x; i < P * kRadix; i += kBlock) {
        uint32_t v = 0;
#pragma unroll
        for (int r = 0; r < R; ++r) v += hist[i * R + r];
        if (v) atomicAdd(&g[i], v);
    }
    // The workgroup that brings the row's last chunk scans the row's histograms.  The additions
    // are made where the whole device sees them, so it is enough that each workgroup's have
    // been carried out before it counts its chunk (no cache is written back or emptied for
    // this: with thousands of workgroups that costs more than the histograms), and that the
    // last one reads the sums in the same place (bases_of_pass does).
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    if (threadIdx.x == 0) last_chunk = atomicAdd(&arrived[row], 1u) == static_cast<uint32_t>(chunks_per_row - 1) ? 1u : 0u;
    __syncthreads();
    if (last_chunk) {
        for (int p = 0; p < P; ++p) bases_of_pass(g + p * kRadix, moves + row * P + p, all_bits);
    }
    }
}

__global__ __launch_bounds__(kBlock) void sort_clear(uint32_t* __restrict__ p, int64_t words) {
    const int64_t i = (static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x) * 4;
    if (i + 4 <= words) *reinterpret_cast<uint4*>(p + i) = make_uint4(0u, 0u, 0u, 0u);
    else for (int64_t j = i; j < words; ++j) p[j] = 0u;
}

// ------------------------------------------------------------------ one pass
template <typename K, bool PAIRS, int ITEMS>
struct PassShared {
    uint32_t wave_hist[kPassWaves][kRadix];       // per-wave digit counts, then per-wave offsets
    uint32_t help_hist[kRadix];               // digits of an earlier tile counted here when it is late
    int32_t dst_base[kRadix];                 // row position of that digit's run start minus digit_start
    uint32_t scan_tmp[kPassWaves];
    int help_tile;
    K keys[kPassBlock * ITEMS];
    uint32_t vals[PAIRS ? kPassBlock * ITEMS : 1];
};

// Pass `pass` of the sort (digit = bits [8 pass, 8 pass + 8) of the key).  LAST: the pass of
// the most significant digit, which every row runs and which writes the strided outputs.
// Rows are independent: a row leaves out the passes that would not move its keys, the first
// pass it runs reads the strided input, and its place in the ping-pong buffers alternates
// over the passes it does run.
template <typename K, bool PAIRS, int ITEMS, bool LAST>
__global__ __launch_bounds__(kPassBlock) __attribute__((amdgpu_waves_per_eu(DLFX_SORT_WAVES))) void sort_pass(PassIo<K> io, int pass, int64_t rows, int64_t n, int64_t tiles_per_row,
                                                    const uint32_t* __restrict__ gbase,
                                                    const uint32_t* __restrict__ moves,
                                                    uint32_t* __restrict__ status, int poll_limit) {
    constexpr int P = KeyTraits<K>::kPasses;
    constexpr int TILE = kPassBlock * ITEMS;
    constexpr int W = 4;    // status words of earlier tiles fetched per look-back step
    __shared__ PassShared<K, PAIRS, ITEMS> sm;

    // workgroups are handed out in index order and dealt round-robin over the chip's eight
    // parts: tile t of every row comes before tile t + 1 of any row, so a tile's predecessors
    // in its row have usually finished when it looks back, and the tiles of a row share a
    // second-level cache when the number of rows is a multiple of eight.
    for (int64_t unit = blockIdx.x; unit < rows * tiles_per_row; unit += gridDim.x) {
    if (unit != static_cast<int64_t>(blockIdx.x)) __syncthreads();      // the previous tile has left LDS
    const int64_t t = unit / rows;
    const int64_t row = unit - t * rows;
    const uint32_t* row_moves = moves + row * P;
    const int tag = pass;
    int ran = 0;            // passes before this one that this row ran
    for (int p = 0; p < pass; ++p) ran += row_moves[p] ? 1 : 0;
    if (!LAST && row_moves[pass] == 0u) continue;
    const bool first = ran == 0;
    const K* __restrict__ src_keys = first ? nullptr : io.kbuf[(ran - 1) & 1];
    const uint32_t* __restrict__ src_vals = first ? nullptr : io.vbuf[(ran - 1) & 1];
    K* __restrict__ dst_keys = io.kbuf[ran & 1];
    uint32_t* __restrict__ dst_vals = io.vbuf[ran & 1];

    const int tid = threadIdx.x;
    const int lane = lane_id();
    const int w = tid / kWave;
    const int64_t tile_base = t * TILE;
    const int valid = static_cast<int>((n - tile_base < TILE) ? n - tile_base : TILE);
    const bool full = valid == TILE;
    const K* xrow = io.x + io.xmap.at(row);
    const int64_t row_off = row * n;
    const int shift = 8 * pass;

    DLFX_PHASE_BEGIN();
    for (int i = tid; i < kPassWaves * kRadix; i += kPassBlock) (&sm.wave_hist[0][0])[i] = 0;
    if (tid == 0) sm.help_tile = -1;

    // ---- load: wave w owns [w*64*ITEMS, ...), item k of lane l is element k*64 + l of it.
    // All loads are issued before the first key is used.
    K key[ITEMS];
    uint32_t val[PAIRS ? ITEMS : 1];
    const int seg = w * kWave * ITEMS + lane;
    if (first) {
        const K* src = xrow + (tile_base + seg) * io.sx;
        const int64_t step = io.sx * kWave;
        if (full) {
#pragma unroll
            for (int k = 0; k < ITEMS; ++k) key[k] = src[k * step];
        } else {
#pragma unroll
            for (int k = 0; k < ITEMS; ++k) {
                key[k] = 0;
                if (seg + k * kWave < valid) key[k] = src[k * step];
            }
        }
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) {
            key[k] = key_of_element<K>(io, key[k]);
            if constexpr (PAIRS) val[k] = static_cast<uint32_t>(tile_base) + static_cast<uint32_t>(seg + k * kWave);
        }
    } else {
        const K* src = src_keys + row_off + tile_base + seg;
        if (full) {
#pragma unroll
            for (int k = 0; k < ITEMS; ++k) key[k] = src[k * kWave];
        } else {
#pragma unroll
            for (int k = 0; k < ITEMS; ++k) {
                key[k] = 0;
                if (seg + k * kWave < valid) key[k] = src[k * kWave];
            }
        }
        if constexpr (PAIRS) {
            const uint32_t* vsrc = src_vals + row_off + tile_base + seg;
            if (full) {
#pragma unroll
                for (int k = 0; k < ITEMS; ++k) val[k] = vsrc[k * kWave];
            } else {
#pragma unroll
                for (int k = 0; k < ITEMS; ++k) {
                    val[k] = 0;
                    if (seg + k * kWave < valid) val[k] = vsrc[k * kWave];
                }
            }
        }
    }
    if (!full) {
#pragma unroll
        for (int k = 0; k < ITEMS; ++k)
            if (seg + k * kWave >= valid) key[k] = ~K(0);      // padding sorts last and is never stored
    }
    __syncthreads();
    DLFX_PHASE(0);

    // ---- rank inside the wave, in element order (stable).  The lanes whose digit equals this
    // lane's are found with one ballot per digit bit that varies in the row (padding differs
    // in other bits too, so a tile with padding looks at all of them); two items at a time, so
    // that the two independent chains fill each other's wait states.  The items then take their ranks from
    // the wave's running digit counts one after the other: the first lane of each group of
    // equal digits moves the count on.
    const uint32_t vary = full ? row_moves[pass] : 0xffu;
    uint32_t rank[ITEMS];
    static_assert(ITEMS % 2 == 0, "items are ranked in pairs");
#pragma unroll
    for (int k0 = 0; k0 < ITEMS; k0 += 2) {
        uint32_t d[2], before[2], cnt[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) d[j] = static_cast<uint32_t>(key[k0 + j] >> shift) & 0xffu;
        uint32_t peers_lo[2] = {0xffffffffu, 0xffffffffu}, peers_hi[2] = {0xffffffffu, 0xffffffffu};
        for (uint32_t bits = vary; bits != 0u; bits &= bits - 1u) {
            const uint32_t b = static_cast<uint32_t>(__builtin_ctz(bits));
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int32_t ones = __builtin_amdgcn_sbfe(static_cast<int32_t>(d[j]), b, 1u);     // all ones when the bit is set
                const unsigned long long vote = __ballot(ones < 0);
                peers_lo[j] &= ~(static_cast<uint32_t>(vote) ^ static_cast<uint32_t>(ones));
                peers_hi[j] &= ~(static_cast<uint32_t>(vote >> 32) ^ static_cast<uint32_t>(ones));
            }
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            before[j] = __builtin_amdgcn_mbcnt_hi(peers_hi[j], __builtin_amdgcn_mbcnt_lo(peers_lo[j], 0u));
            cnt[j] = static_cast<uint32_t>(__popc(peers_lo[j]) + __popc(peers_hi[j]));
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const uint32_t seen = sm.wave_hist[w][d[j]];          // same word for all peers: a broadcast read
            rank[k0 + j] = seen + before[j];
            __builtin_amdgcn_wave_barrier();
            if (before[j] == 0) sm.wave_hist[w][d[j]] = seen + cnt[j];
            __builtin_amdgcn_wave_barrier();
        }
    }
    __syncthreads();
    DLFX_PHASE(1);

    // ---- thread d owns digit d: tile count, position of the digit in the tile, wave offsets
    // (threads beyond the 256 digits idle through this part, except at the barriers)
    const bool owner = tid < kRadix;
    const int dg = owner ? tid : 0;
    uint32_t wave_count[kPassWaves];
    uint32_t count = 0;
#pragma unroll
    for (int i = 0; i < kPassWaves; ++i) {
        wave_count[i] = sm.wave_hist[i][dg];
        count += wave_count[i];
    }
    const uint32_t padded = count;
    if (tid == kRadix - 1) count -= static_cast<uint32_t>(TILE - valid);     // padding is not part of the row
    const int64_t srow = (row * tiles_per_row) * kRadix;
    uint32_t* my_status = status + srow + t * kRadix + dg;
    if (owner && t + 1 < tiles_per_row)
        __hip_atomic_store(my_status, make_status(tag, t == 0, count), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // the status words of the W tiles before this one are requested now and looked at after
    // the tile has been gathered, so that their latency is not waited for
    uint32_t sw[W];
    int64_t p = t - 1;
    auto fetch = [&]() {
#pragma unroll
        for (int i = 0; i < W; ++i) {
            const int64_t q = p - i;
            sw[i] = (q >= 0) ? __hip_atomic_load(status + srow + q * kRadix + dg, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                             : make_status(tag, true, 0u);
        }
    };
    bool done = (t == 0) || !owner;
    if (!done) fetch();
    uint32_t start;
    {
        const uint32_t incl = wave_scan_inclusive(padded, 0u, [](uint32_t a, uint32_t b) { return a + b; });
        if (owner && lane == kWave - 1) sm.scan_tmp[w] = incl;
        __syncthreads();
        uint32_t pre = 0;
        for (int i = 0; i < w && i < kRadix / kWave; ++i) pre += sm.scan_tmp[i];
        start = pre + incl - padded;
        uint32_t run = start;
        if (owner) {
#pragma unroll
            for (int i = 0; i < kPassWaves; ++i) {
                sm.wave_hist[i][tid] = run;        // tile position of the first key of wave i with this digit
                run += wave_count[i];
            }
        }
    }
    __syncthreads();
    DLFX_PHASE(2);

    // ---- gather the tile in its locally sorted order
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const uint32_t d = static_cast<uint32_t>(key[k] >> shift) & 0xffu;
        const uint32_t pos = sm.wave_hist[w][d] + rank[k];
        sm.keys[pos] = key[k];
        if constexpr (PAIRS) sm.vals[pos] = val[k];
    }
    DLFX_PHASE(3);

    // ---- look back over the row's earlier tiles for digit `tid`
    uint32_t before_tiles = 0;
    {
        bool refetch = false;
        const uint32_t want_tag = static_cast<uint32_t>(tag + 1);
        for (;;) {
            int stuck = -1;
            while (!done) {
                if (refetch) {
                    fetch();
                    refetch = false;
                }
#pragma unroll
                for (int i = 0; i < W; ++i) {
                    if (done || stuck >= 0) continue;
                    const int64_t q = p - i;
                    uint32_t s = sw[i];
                    for (int polls = 0; (s >> 28) != want_tag && polls < poll_limit; ++polls) {
                        __builtin_amdgcn_s_sleep(1);
                        s = __hip_atomic_load(status + srow + q * kRadix + dg, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                    if ((s >> 28) != want_tag) {
                        stuck = static_cast<int>(q);
                    } else {
                        before_tiles += s & kCountMask;
                        if (s & (1u << 27)) done = true;
                    }
                }
                refetch = true;
                if (stuck >= 0) {
                    p = stuck;                    // resume at this tile
                    break;
                }
                p -= W;
            }
            // anyone still waiting?  then the whole workgroup counts that tile's digits itself
            if (stuck >= 0) atomicMax(&sm.help_tile, stuck);
            __syncthreads();
            const int help = sm.help_tile;
            if (help < 0) break;
            if (owner) sm.help_hist[tid] = 0;
            __syncthreads();
            {
                const int64_t hb = static_cast<int64_t>(help) * TILE;
                const int hv = static_cast<int>((n - hb < TILE) ? n - hb : TILE);
                for (int li = tid; li < hv; li += kPassBlock) {
                    const K hk = first ? key_of_element<K>(io, xrow[(hb + li) * io.sx]) : src_keys[row_off + hb + li];
                    atomicAdd(&sm.help_hist[static_cast<uint32_t>(hk >> shift) & 0xffu], 1u);
                }
            }
            __syncthreads();
            if (stuck == help) {
                before_tiles += sm.help_hist[dg];
                p = static_cast<int64_t>(help) - 1;
                if (p < 0) done = true;
            }
            __syncthreads();
            if (tid == 0) sm.help_tile = -1;
            __syncthreads();
        }
    }
    if (owner && t > 0 && t + 1 < tiles_per_row)
        __hip_atomic_store(my_status, make_status(tag, true, before_tiles + count), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (owner) sm.dst_base[tid] = static_cast<int32_t>(gbase[(row * P + pass) * kRadix + tid] + before_tiles) - static_cast<int32_t>(start);
    __syncthreads();
    DLFX_PHASE(4);

    // ---- write runs: thread t takes tile positions t, t + 256, ...
    K out[ITEMS];
    int32_t at[ITEMS];
    uint32_t pay[PAIRS ? ITEMS : 1];
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) out[k] = sm.keys[k * kPassBlock + tid];
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) at[k] = sm.dst_base[static_cast<uint32_t>(out[k] >> shift) & 0xffu] + (k * kPassBlock + tid);
    if constexpr (PAIRS) {
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) pay[k] = sm.vals[k * kPassBlock + tid];
    }
    if (!LAST) {
        K* dk = dst_keys + row_off;
#pragma unroll
        for (int k = 0; k < ITEMS; ++k)
            if (full || k * kPassBlock + tid < valid) dk[at[k]] = out[k];
        if constexpr (PAIRS) {
            uint32_t* dv = dst_vals + row_off;
#pragma unroll
            for (int k = 0; k < ITEMS; ++k)
                if (full || k * kPassBlock + tid < valid) dv[at[k]] = pay[k];
        }
    } else if constexpr (LAST) {
        if (io.y) {
            K* yrow = io.y + io.ymap.at(row);
#pragma unroll
            for (int k = 0; k < ITEMS; ++k) {
                K bits = decode_key<K>(out[k], io.kind, io.descending);
                if constexpr (PAIRS) {
                    if (io.restore_zero && static_cast<K>(bits << 1) == 0 && (full || k * kPassBlock + tid < valid))
                        bits = xrow[static_cast<int64_t>(pay[k]) * io.sx];
                }
                if (full || k * kPassBlock + tid < valid) yrow[at[k] * io.sy] = bits;
            }
        }
        if constexpr (PAIRS) {
            if (io.idx) {
                const int64_t irow = io.imap.at(row);
                if (io.idx64) {
                    int64_t* ip = static_cast<int64_t*>(io.idx) + irow;
#pragma unroll
                    for (int k = 0; k < ITEMS; ++k)
                        if (full || k * kPassBlock + tid < valid) ip[at[k] * io.si] = static_cast<int64_t>(pay[k]);
                } else {
                    int32_t* ip = static_cast<int32_t*>(io.idx) + irow;
#pragma unroll
                    for (int k = 0; k < ITEMS; ++k)
                        if (full || k * kPassBlock + tid < valid) ip[at[k] * io.si] = static_cast<int32_t>(pay[k]);
                }
            }
        }
    }
    DLFX_PHASE(5);
    }
}

// ------------------------------------------------------------------ rows that fit one workgroup
// A row of at most 64 * WAVES * ITEMS keys is read once, sorted through all its passes in LDS and
// registers and written once: no histogram pass, no scratch traffic, no chaining between
// tiles.  The passes are those of sort_pass without the parts that connect tiles: rank inside
// the wave with ballots over the digit bits that vary in the row, digit starts from the
// waves' counts (four waves; eight or sixteen for rows beyond 4096 keys), scatter through LDS, reload in element order.  Digits that are the same in
// the whole row are skipped.  Element e of the row is item e / 64 % ITEMS of lane e % 64 of
// wave e / (64 * ITEMS), before and after every pass.
template <typename K, bool PAIRS, int ITEMS, int WAVES = 4>
__global__ __launch_bounds__(WAVES * kWave) void sort_rows_small(PassIo<K> io, int64_t rows, int64_t n) {
    constexpr int P = KeyTraits<K>::kPasses;
    static_assert(ITEMS % 2 == 0, "items are ranked in pairs");
    __shared__ SmallShared<K, PAIRS, ITEMS, WAVES> sm;
    const int tid = threadIdx.x;
    const int lane = lane_id();
    const int w = tid / kWave;
    const int64_t row = block_of(io);
    if (row >= rows) return;                               // (the grid is rounded up to a multiple of 8)
    const K* xrow = io.x + io.xmap.at(row);
    const int valid = static_cast<int>(n);
    const int seg = w * kWave * ITEMS + lane;

    K key[ITEMS];
    uint32_t val[PAIRS ? ITEMS : 1];
    K ors = 0, ands = ~K(0);
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        const int e = seg + k * kWave;
        key[k] = ~K(0);                                   // padding sorts last in every pass that runs
        if (e < valid) {
            key[k] = key_of_element<K>(io, xrow[static_cast<int64_t>(e) * io.sx]);
            ors |= key[k];
            ands &= key[k];
        }
        if constexpr (PAIRS) val[k] = static_cast<uint32_t>(e);
    }
    sort_in_workgroup<K, PAIRS, ITEMS, WAVES>(sm, key, val, ors, ands, valid, P);

    // ---- write
    if (io.y) {
        K* yrow = io.y + io.ymap.at(row);
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) {
            const int e = seg + k * kWave;
            if (e < valid) {
                K bits = decode_key<K>(key[k], io.kind, io.descending);
                if constexpr (PAIRS) {
                    if (io.restore_zero && static_cast<K>(bits << 1) == 0) bits = xrow[static_cast<int64_t>(val[k]) * io.sx];
                }
                yrow[static_cast<int64_t>(e) * io.sy] = bits;
            }
        }
    }
    if constexpr (PAIRS) {
        if (io.idx) {
            const int64_t irow = io.imap.at(row);
#pragma unroll
            for (int k = 0; k < ITEMS; ++k) {
                const int e = seg + k * kWave;
                if (e < valid) {
                    if (io.idx64) static_cast<int64_t*>(io.idx)[irow + static_cast<int64_t>(e) * io.si] = static_cast<int64_t>(val[k]);
                    else static_cast<int32_t*>(io.idx)[irow + static_cast<int64_t>(e) * io.si] = static_cast<int32_t>(val[k]);
                }
            }
        }
    }
}

// One exchange of the (key, index) networks below: the lane takes the entry of lane ^ J when
// that entry comes first (smaller key, then smaller index - a total order, hence stable) and
// this lane keeps the first of the two, or when it does not and this lane keeps the second.
template <bool PAIRS, int J, typename K>
__device__ __forceinline__ void exchange_entry(K& key, uint32_t& idx, bool keep_first) {
    const K other_key = lane_xor_const<J>(key);
    bool other_first = other_key < key;
    if constexpr (PAIRS) {
        const uint32_t other_idx = lane_xor_const<J>(idx);
        other_first = other_first || (other_key == key && other_idx < idx);
        if (keep_first == other_first) {
            key = other_key;
            idx = other_idx;
        }
    } else {
        if (keep_first == other_first) key = other_key;
    }
}

// Rows of at most 64 elements: a group of WIDTH = 4, 8, 16, 32 or 64 lanes per row, one element
// per lane, a bitonic network over (key, index) pairs - a total order, so the result is the
// stable one.  256 / WIDTH rows per workgroup, no LDS, no barrier.
template <typename K, bool PAIRS, int WIDTH>
__global__ __launch_bounds__(256) void sort_rows_wave(PassIo<K> io, int64_t rows, int64_t n) {
    const int at = lane_id() % WIDTH;
    const int64_t row = block_of(io) * (256 / WIDTH) + threadIdx.x / WIDTH;
    const bool row_live = row < rows;                      // lanes of absent rows still take part in the exchanges
    const K* xrow = io.x + (row_live ? io.xmap.at(row) : 0);
    const bool live = row_live && at < n;
    K key = live ? key_of_element<K>(io, xrow[static_cast<int64_t>(at) * io.sx]) : ~K(0);   // padding sorts last
    uint32_t idx = static_cast<uint32_t>(at);
    wave_bitonic<WIDTH, true>([&](auto jc, bool keep_first) { exchange_entry<PAIRS, decltype(jc)::value>(key, idx, keep_first); });
    if (!live) return;                                     // the first n lanes of the group hold the row in order
    if (io.y) {
        K bits = decode_key<K>(key, io.kind, io.descending);
        if constexpr (PAIRS) {
            if (io.restore_zero && static_cast<K>(bits << 1) == 0) bits = xrow[static_cast<int64_t>(idx) * io.sx];
        }
        io.y[io.ymap.at(row) + static_cast<int64_t>(at) * io.sy] = bits;
    }
    if constexpr (PAIRS) {
        if (io.idx) {
            const int64_t where = io.imap.at(row) + static_cast<int64_t>(at) * io.si;
            if (io.idx64) static_cast<int64_t*>(io.idx)[where] = static_cast<int64_t>(idx);
            else static_cast<int32_t*>(io.idx)[where] = static_cast<int32_t>(idx);
        }
    }
}

// Rows of 65 to 64 * ITEMS elements: still one wavefront per row and no LDS.  Element
// i * 64 + lane is item i of the lane (coalesced loads and stores); the bitonic network runs
// over that index: exchanges at a distance below 64 cross lanes, the others pair two items of
// one lane, with a direction known at compile time.
template <typename K, bool PAIRS, int ITEMS>
__global__ __launch_bounds__(256) void sort_rows_wave_items(PassIo<K> io, int64_t rows, int64_t n) {
    const int lane = lane_id();
    const int64_t row = block_of(io) * 4 + threadIdx.x / kWave;
    if (row >= rows) return;
    const K* xrow = io.x + io.xmap.at(row);
    const int n32 = static_cast<int>(n);
    K key[ITEMS];
    uint32_t idx[ITEMS];
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        const int e = i * kWave + lane;
        key[i] = e < n32 ? key_of_element<K>(io, xrow[static_cast<int64_t>(e) * io.sx]) : ~K(0);   // padding sorts last
        idx[i] = static_cast<uint32_t>(e);
    }
    wave_bitonic_items<PAIRS, ITEMS>(key, idx, [](K ka, uint32_t ia, K kb, uint32_t ib) {      // a strictly before b
        if constexpr (PAIRS) return ka < kb || (ka == kb && ia < ib);
        else return ka < kb;
    });
    K* yrow = io.y ? io.y + io.ymap.at(row) : nullptr;
    const int64_t irow = (PAIRS && io.idx) ? io.imap.at(row) : 0;
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        const int e = i * kWave + lane;
        if (e >= n32) continue;                            // the first n places hold the row in order
        if (yrow) {
            K bits = decode_key<K>(key[i], io.kind, io.descending);
            if constexpr (PAIRS) {
                if (io.restore_zero && static_cast<K>(bits << 1) == 0) bits = xrow[static_cast<int64_t>(idx[i]) * io.sx];
            }
            yrow[static_cast<int64_t>(e) * io.sy] = bits;
        }
        if constexpr (PAIRS) {
            if (io.idx) {
                const int64_t at = irow + static_cast<int64_t>(e) * io.si;
                if (io.idx64) static_cast<int64_t*>(io.idx)[at] = static_cast<int64_t>(idx[i]);
                else static_cast<int32_t*>(io.idx)[at] = static_cast<int32_t>(idx[i]);
            }
        }
    }
}

// Rows of at most 64 elements that lie side by side in memory (the axis is an outer
// dimension): a workgroup takes 64 neighbouring rows, reads them with coalesced loads (64
// rows wide, one axis position at a time) into LDS, each wavefront sorts sixteen of them with the
// network of sort_rows_wave (lane l holds element l; pitch 65 keeps both access patterns
// free of bank conflicts), and the tile leaves the way it came.
template <typename K, bool PAIRS>
__global__ __launch_bounds__(256) void sort_cols_wave(PassIo<K> io, int64_t rows, int64_t n) {
    constexpr int kPitch = kWave + 1;
    __shared__ K keys[kWave * kPitch];
    __shared__ uint32_t places[PAIRS ? kWave * kPitch : 1];
    const int lane = lane_id();
    const int w = threadIdx.x / kWave;
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * kWave;
    const int r = lane;                                    // this thread's row of the tile in the load and store phases
    const bool row_live = row0 + r < rows;
    const int n32 = static_cast<int>(n);
    const K* xrow = io.x + (row_live ? io.xmap.at(row0 + r) : 0);
    for (int a = w; a < n32; a += 4)
        keys[a * kPitch + r] = row_live ? key_of_element<K>(io, xrow[static_cast<int64_t>(a) * io.sx]) : ~K(0);
    __syncthreads();
    for (int q = w; q < kWave; q += 4) {                   // row q of the tile, element `lane`
        K key = lane < n32 ? keys[lane * kPitch + q] : ~K(0);      // padding sorts last
        uint32_t idx = static_cast<uint32_t>(lane);
        wave_bitonic<kWave, true>([&](auto jc, bool keep_first) { exchange_entry<PAIRS, decltype(jc)::value>(key, idx, keep_first); });
        if (lane < n32) {
            K bits = decode_key<K>(key, io.kind, io.descending);
            if constexpr (PAIRS) {
                if (io.restore_zero && static_cast<K>(bits << 1) == 0 && row0 + q < rows)
                    bits = io.x[io.xmap.at(row0 + q) + static_cast<int64_t>(idx) * io.sx];
                places[lane * kPitch + q] = idx;
            }
            keys[lane * kPitch + q] = bits;
        }
    }
    __syncthreads();
    if (!row_live) return;
    if (io.y) {
        K* yrow = io.y + io.ymap.at(row0 + r);
        for (int a = w; a < n32; a += 4) yrow[static_cast<int64_t>(a) * io.sy] = keys[a * kPitch + r];
    }
    if constexpr (PAIRS) {
        if (io.idx) {
            const int64_t irow = io.imap.at(row0 + r);
            for (int a = w; a < n32; a += 4) {
                const int64_t at = irow + static_cast<int64_t>(a) * io.si;
                if (io.idx64) static_cast<int64_t*>(io.idx)[at] = static_cast<int64_t>(places[a * kPitch + r]);
                else static_cast<int32_t*>(io.idx)[at] = static_cast<int32_t>(places[a * kPitch + r]);
            }
        }
    }
}

// The same for rows of 65 to 64 * ITEMS elements (4-byte keys; 8-byte keys with two items): a tile of 16 neighbouring rows,
// read 16 rows wide (64 bytes a position, where a wavefront per row reads every element of its
// row from a cache line of its own: fp32 [32, 512, 56, 56] along axis 1 440 us), each wavefront
// sorts four of them with the network of sort_rows_wave_items (pitch 17: a wavefront's accesses
// to one row of the tile fall into different banks), and the tile leaves the way it came.
template <typename K, bool PAIRS, int ITEMS>
__global__ __launch_bounds__(256) void sort_cols_tile(PassIo<K> io, int64_t rows, int64_t n) {
    constexpr int kTile = 16, kPitch = kTile + 1;
    __shared__ K keys[ITEMS * kWave * kPitch];
    __shared__ uint32_t places[PAIRS ? ITEMS * kWave * kPitch : 1];
    const int lane = lane_id();
    const int w = threadIdx.x / kWave;
    const int64_t row0 = block_of(io) * kTile;
    if (row0 >= rows) return;
    const int r = threadIdx.x % kTile;                     // this thread's row of the tile in the load and store phases
    const int a0 = threadIdx.x / kTile;                    // ... and its first position of the axis
    const bool row_live = row0 + r < rows;
    const int n32 = static_cast<int>(n);
    const K* xrow = io.x + (row_live ? io.xmap.at(row0 + r) : 0);
    for (int a = a0; a < n32; a += 256 / kTile)
        keys[a * kPitch + r] = row_live ? key_of_element<K>(io, xrow[static_cast<int64_t>(a) * io.sx]) : ~K(0);
    __syncthreads();
    for (int q = w; q < kTile; q += 4) {                   // row q of the tile: element i * 64 + lane is item i of the lane
        K key[ITEMS];
        uint32_t idx[ITEMS];
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
            const int e = i * kWave + lane;
            key[i] = e < n32 ? keys[e * kPitch + q] : ~K(0);       // padding sorts last
            idx[i] = static_cast<uint32_t>(e);
        }
        wave_bitonic_items<PAIRS, ITEMS>(key, idx, [](K ka, uint32_t ia, K kb, uint32_t ib) {      // a strictly before b
            if constexpr (PAIRS) return ka < kb || (ka == kb && ia < ib);
            else return ka < kb;
        });
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
            const int e = i * kWave + lane;
            if (e >= n32) continue;
            K bits = decode_key<K>(key[i], io.kind, io.descending);
            if constexpr (PAIRS) {
                if (io.restore_zero && static_cast<K>(bits << 1) == 0 && row0 + q < rows)
                    bits = io.x[io.xmap.at(row0 + q) + static_cast<int64_t>(idx[i]) * io.sx];
                places[e * kPitch + q] = idx[i];
            }
            keys[e * kPitch + q] = bits;
        }
    }
    __syncthreads();
    if (!row_live) return;
    if (io.y) {
        K* yrow = io.y + io.ymap.at(row0 + r);
        for (int a = a0; a < n32; a += 256 / kTile) yrow[static_cast<int64_t>(a) * io.sy] = keys[a * kPitch + r];
    }
    if constexpr (PAIRS) {
        if (io.idx) {
            const int64_t irow = io.imap.at(row0 + r);
            for (int a = a0; a < n32; a += 256 / kTile) {
                const int64_t at = irow + static_cast<int64_t>(a) * io.si;
                if (io.idx64) static_cast<int64_t*>(io.idx)[at] = static_cast<int64_t>(places[a * kPitch + r]);
                else static_cast<int32_t*>(io.idx)[at] = static_cast<int32_t>(places[a * kPitch + r]);
            }
        }
    }
}

// longest row sorted by one wavefront (dlfx_set_tuning "sort_wave_rows": 64, 128, 256 or 512)
int g_sort_wave_rows = 512;

// longest row sort_rows_small takes: four wavefronts hold 4096 keys, eight hold 8192 (4- and
// 8-byte keys: [4096, 8192] fp32 sorts in 245 us against 485 us by the bucket route, argsort
// 260 against 590; int64 235 against 280, argsort 260 against 340), sixteen hold 16384 4-byte
// keys ([2048, 16384] fp32 301 against 362 us, argsort 355 against 434; [2796, 12000] 333
// against 401; int32 the same within 5 %)
constexpr int64_t small_row(size_t key_size) { return key_size == 4 ? 16384 : key_size == 8 ? 8192 : 4096; }

int g_sort_buckets = 1;                  // 1: rows the bucket route takes go that way (dlfx_set_tuning "sort_buckets")
int g_sort_compare_max = 32;             // fullest counting bin of a bucket that is still ranked by comparison (fuller ones cost more that way than the digit passes do: 16 to 48 measured alike, 96 up to 11 % slower on N(0,1) floats, 8 slower again)

template <typename K, bool PAIRS>
int launch_small(hipStream_t stream, const PassIo<K>& io_in, int64_t m, int64_t n) {
    PassIo<K> io = io_in;
    const dim3 block(256);
    // rows side by side in memory: neighbouring rows to the same XCD
    const bool side_by_side = io.sx != 1 && io.sx != -1 && io.xmap.rank >= 1 && io.xmap.strides[io.xmap.rank - 1] == 1;
    auto grid_for = [&](int64_t rows_per_block) {
        int64_t blocks = ceil_div(m, rows_per_block);
        io.xcd_blocks = 0;
        if (side_by_side && blocks >= 64) {
            io.xcd_blocks = ceil_div(blocks, 8);
            blocks = io.xcd_blocks * 8;
        }
        return dim3(static_cast<unsigned>(blocks));
    };
    // eight items per lane pay off except for 4-byte keys that carry an index
    const bool wave_items8 = g_sort_wave_rows >= 8 * kWave && !(PAIRS && sizeof(K) == 4);
    // (tiles of 16 rows: the innermost run of rows at least that long, and rows enough for a few tiles a compute
    // unit.  Keys alone, rows of up to 256 elements: fp32 [8, 128, 256, 256] along axis 1 482 -> 268 us,
    // [256, 100000] along axis 0 183 -> 112 us.  With indices the tile costs LDS that the wavefront-per-row
    // kernels do not need and was slower from 129 elements on (317 -> 353 us at 200, 527 -> 609 us at 256) and
    // within 8 % below; eight items a lane lost both ways at 300 elements (222 -> 282 us); a row that fills
    // little of four items a lane - 129 to 160 elements - gains nothing either)
    const bool tiles = !PAIRS && side_by_side && (sizeof(K) == 4 || sizeof(K) == 8) && n > kWave && n <= (sizeof(K) == 4 ? 4 : 2) * kWave &&
                       !(n > 2 * kWave && n <= 160) && m >= 4096 && io.xmap.dims[io.xmap.rank - 1] >= 16;
    if (side_by_side && n <= kWave && m >= 4096) sort_cols_wave<K, PAIRS><<<dim3(static_cast<unsigned>(ceil_div(m, kWave))), block, 0, stream>>>(io, m, n);
    else if (tiles) {
        if constexpr (!PAIRS && sizeof(K) >= 4) {
            const dim3 g = grid_for(16);
            if (n <= 2 * kWave) sort_cols_tile<K, PAIRS, 2><<<g, block, 0, stream>>>(io, m, n);
            else if constexpr (sizeof(K) == 4) sort_cols_tile<K, PAIRS, 4><<<g, block, 0, stream>>>(io, m, n);
        }
    }
    else if (n <= 4) { const dim3 g = grid_for(64); sort_rows_wave<K, PAIRS, 4><<<g, block, 0, stream>>>(io, m, n); }
    else if (n <= 8) { const dim3 g = grid_for(32); sort_rows_wave<K, PAIRS, 8><<<g, block, 0, stream>>>(io, m, n); }
    else if (n <= 16) { const dim3 g = grid_for(16); sort_rows_wave<K, PAIRS, 16><<<g, block, 0, stream>>>(io, m, n); }
    else if (n <= 32) { const dim3 g = grid_for(8); sort_rows_wave<K, PAIRS, 32><<<g, block, 0, stream>>>(io, m, n); }
    else if (n <= kWave) { const dim3 g = grid_for(4); sort_rows_wave<K, PAIRS, kWave><<<g, block, 0, stream>>>(io, m, n); }
    else if (n <= 2 * kWave && g_sort_wave_rows >= 2 * kWave) { const dim3 g = grid_for(4); sort_rows_wave_items<K, PAIRS, 2><<<g, block, 0, stream>>>(io, m, n); }
    else if (n <= 4 * kWave && g_sort_wave_rows >= 4 * kWave) { const dim3 g = grid_for(4); sort_rows_wave_items<K, PAIRS, 4><<<g, block, 0, stream>>>(io, m, n); }
    else if (n <= 8 * kWave && wave_items8) { const dim3 g = grid_for(4); sort_rows_wave_items<K, PAIRS, 8><<<g, block, 0, stream>>>(io, m, n); }
    else if (n <= 512) { const dim3 g = grid_for(1); sort_rows_small<K, PAIRS, 2><<<g, block, 0, stream>>>(io, m, n); }
    else if (n <= 1024) { const dim3 g = grid_for(1); sort_rows_small<K, PAIRS, 4><<<g, block, 0, stream>>>(io, m, n); }
    else if (n <= 1536) { const dim3 g = grid_for(1); sort_rows_small<K, PAIRS, 6><<<g, block, 0, stream>>>(io, m, n); }
    else if (n <= 2048) { const dim3 g = grid_for(1); sort_rows_small<K, PAIRS, 8><<<g, block, 0, stream>>>(io, m, n); }
    else if (n <= 2560) { const dim3 g = grid_for(1); sort_rows_small<K, PAIRS, 10><<<g, block, 0, stream>>>(io, m, n); }
    else if (n <= 3072) { const dim3 g = grid_for(1); sort_rows_small<K, PAIRS, 12><<<g, block, 0, stream>>>(io, m, n); }
    else if (n <= 3584 && !(PAIRS && sizeof(K) == 8)) { const dim3 g = grid_for(1); sort_rows_small<K, PAIRS, 14><<<g, block, 0, stream>>>(io, m, n); }
    else if (n <= 4096) {
        // (16 8-byte keys a thread with their indices: eight wavefronts of 8 keep them in registers)
        const dim3 g = grid_for(1);
        if constexpr (PAIRS && sizeof(K) == 8) sort_rows_small<K, PAIRS, 8, 8><<<g, dim3(8 * kWave), 0, stream>>>(io, m, n);
        else sort_rows_small<K, PAIRS, 16><<<g, block, 0, stream>>>(io, m, n);
    }
    else if constexpr (sizeof(K) >= 4) {
        // eight wavefronts, 10, 12 or 16 keys a thread: 5120, 6144 or 8192 slots; sixteen for 4-byte
        // keys beyond that, 10, 12, 14 or 16 keys a thread: 10240, 12288, 14336 or 16384 slots
        const dim3 g = grid_for(1), wide(8 * kWave);
        if (n <= 5120) sort_rows_small<K, PAIRS, 10, 8><<<g, wide, 0, stream>>>(io, m, n);
        else if (n <= 6144) sort_rows_small<K, PAIRS, 12, 8><<<g, wide, 0, stream>>>(io, m, n);
        else if (n <= 8192) sort_rows_small<K, PAIRS, 16, 8><<<g, wide, 0, stream>>>(io, m, n);
        else if constexpr (sizeof(K) == 4) {
            const dim3 widest(16 * kWave);
            if (n <= 10240) sort_rows_small<K, PAIRS, 10, 16><<<g, widest, 0, stream>>>(io, m, n);
            else if (n <= 12288) sort_rows_small<K, PAIRS, 12, 16><<<g, widest, 0, stream>>>(io, m, n);
            else if (n <= 14336) sort_rows_small<K, PAIRS, 14, 16><<<g, widest, 0, stream>>>(io, m, n);
            else sort_rows_small<K, PAIRS, 16, 16><<<g, widest, 0, stream>>>(io, m, n);
        }
    }
    DLFX_CHECK_LAUNCH();
    return DLFX_OK;
}

// ------------------------------------------------------------------ host side
// Keys per thread: 16, or 8 for 64-bit keys that carry an index (LDS and registers then
// still allow four workgroups per compute unit).
constexpr int tile_items(size_t key_size, bool pairs) { return ((key_size == 8 && pairs) ? 8 : 16) * 256 / kPassBlock; }

struct SortLayout {
    int64_t tiles_per_row;
    size_t moves_off, arrived_off, hist_off, hist_bytes, status_off, status_bytes, split_off, split_bytes, keys_off[2], vals_off[2], total;
};

// Rows longer than one workgroup sorts on chip take the bucket route when their shape allows
// it (and dlfx_set_tuning has not switched it off): it sorts every row of the call, needs one
// pair of ping-pong buffers and its own tables, and none of the digit passes' tables.
bool takes_bucket_route(size_t key_size, int64_t m, int64_t n) {
    return key_size >= 4 && g_sort_buckets != 0 && n > small_row(key_size) && split_route_takes(key_size, m, n);
}

SortLayout sort_layout(size_t key_size, bool pairs, int64_t m, int64_t n) {
    SortLayout l;
    const int passes = static_cast<int>(key_size);          // one per key byte
    const int64_t tile = kPassBlock * tile_items(key_size, pairs);
    const bool buckets = takes_bucket_route(key_size, m, n);
    l.tiles_per_row = ceil_div(n, tile);
    size_t off = 0;
    l.moves_off = off;           // one word per (row, pass): does the pass move the row's keys
    if (!buckets) off += align_up(static_cast<size_t>(m) * passes * 4, 256);
    l.arrived_off = off;         // chunks of each row counted so far; cleared with the histograms and the status words after it
    if (!buckets) off += align_up(static_cast<size_t>(m) * 4, 256);
    l.hist_off = off;
    l.hist_bytes = buckets ? 0 : static_cast<size_t>(m) * passes * kRadix * 4;
    off += align_up(l.hist_bytes, 256);
    l.status_off = off;
    l.status_bytes = (!buckets && l.tiles_per_row > 1) ? static_cast<size_t>(m) * l.tiles_per_row * kRadix * 4 : 0;
    off += align_up(l.status_bytes, 256);
    l.split_off = off;           // tables of the bucket route
    l.split_bytes = buckets ? split_scratch_bytes(key_size, pairs, m, n) : 0;
    off += align_up(l.split_bytes, 256);
    for (int i = 0; i < 2; ++i) {
        l.keys_off[i] = off;
        if (i == 0 || !buckets) off += align_up(static_cast<size_t>(m) * n * key_size, 256);
    }
    for (int i = 0; i < 2; ++i) {
        l.vals_off[i] = off;
        if (pairs && (i == 0 || !buckets)) off += align_up(static_cast<size_t>(m) * n * 4, 256);
    }
    l.total = off;
    return l;
}

// True when the bytes the two views touch intersect (views of different element types).
bool bytes_overlap(int rank, const int64_t* dims, const void* x, const int64_t* sx, size_t ex, const void* y, const int64_t* sy, size_t ey) {
    int64_t xlo = 0, xhi = 0, ylo = 0, yhi = 0;
    for (int i = 0; i < rank; ++i) {
        const int64_t dx = (dims[i] - 1) * sx[i], dy = (dims[i] - 1) * sy[i];
        if (dx > 0) xhi += dx; else xlo += dx;
        if (dy > 0) yhi += dy; else ylo += dy;
    }
    const char* xb = static_cast<const char*>(x) + xlo * static_cast<int64_t>(ex);
    const char* xe = static_cast<const char*>(x) + (xhi + 1) * static_cast<int64_t>(ex);
    const char* yb = static_cast<const char*>(y) + ylo * static_cast<int64_t>(ey);
    const char* ye = static_cast<const char*>(y) + (yhi + 1) * static_cast<int64_t>(ey);
    return xb < ye && yb < xe;
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
    constexpr int IK = tile_items(sizeof(K), false), IP = tile_items(sizeof(K), true);
    const int64_t n = a.dims[a.rank - 1];
    const int64_t m = view_size(a.rank, a.dims) / n;
    if (n > kMaxRow) return DLFX_ERR_TOO_LARGE;
    const SortLayout l = sort_layout(sizeof(K), a.pairs, m, n);
    if (m * l.tiles_per_row > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
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
    const bool i_over_x = a.idx && bytes_overlap(a.rank, a.dims, a.x, a.xs, sizeof(K), a.idx, a.is, a.idx64 ? 8 : 4);
    io.x_intact = (!y_over_x && !i_over_x) ? 1 : 0;

    // short rows: one workgroup sorts a row on chip.  A workgroup reads its whole row before it
    // writes, so sorting in place is fine; an output that overlaps the input in any other way
    // (one row's output over another row's input) takes the general path.
    bool same_view = a.y == a.x;
    for (int i = 0; i < a.rank && same_view; ++i) same_view = a.xs[i] == a.ys[i] || a.dims[i] == 1;
    if (n <= small_row(sizeof(K)) && (!y_over_x || same_view)) {
        if (m > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
        return a.pairs ? launch_small<K, true>(stream, io, m, n) : launch_small<K, false>(stream, io, m, n);
    }
    if (!scratch || scratch_bytes < l.total) return DLFX_ERR_SCRATCH_TOO_SMALL;

    io.kbuf[0] = reinterpret_cast<K*>(base + l.keys_off[0]);
    io.kbuf[1] = reinterpret_cast<K*>(base + l.keys_off[1]);
    io.vbuf[0] = a.pairs ? reinterpret_cast<uint32_t*>(base + l.vals_off[0]) : nullptr;
    io.vbuf[1] = a.pairs ? reinterpret_cast<uint32_t*>(base + l.vals_off[1]) : nullptr;

    // The bucket route sorts every row of the call (rows that do not cut into buckets a workgroup
    // holds are finished by one workgroup per oversized bucket, decided on the device).
    if constexpr (sizeof(K) >= 4) {
        if (l.split_bytes != 0) return run_split<K>(stream, io, a.pairs, m, n, base + l.split_off, g_sort_compare_max);
    }

    uint32_t* moves = reinterpret_cast<uint32_t*>(base + l.moves_off);
    uint32_t* arrived = reinterpret_cast<uint32_t*>(base + l.arrived_off);
    uint32_t* ghist = reinterpret_cast<uint32_t*>(base + l.hist_off);
    uint32_t* status = reinterpret_cast<uint32_t*>(base + l.status_off);
    {
        const int64_t clear_words = static_cast<int64_t>((l.status_off + l.status_bytes - l.arrived_off) / 4);   // counts, histograms, status
        sort_clear<<<dim3(static_cast<unsigned>(ceil_div(clear_words, kBlock * 4))), dim3(kBlock), 0, stream>>>(arrived, clear_words);
        DLFX_CHECK_LAUNCH();
    }

    const int64_t chunk = 32768;
    const int64_t chunks_per_row = ceil_div(n, chunk);
    if (m * chunks_per_row > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
    // a pass that moves nothing may only be left out when no pass reads the input while
    // another tile of the same pass writes the output over it
    sort_histogram<K><<<dim3(static_cast<unsigned>(m * chunks_per_row)), dim3(kBlock), 0, stream>>>(io, n, chunk, chunks_per_row, m * chunks_per_row, ghist,
                                                                                    arrived, moves, y_over_x ? 1 : 0);
    DLFX_CHECK_LAUNCH();

    const dim3 grid(static_cast<unsigned>(m * l.tiles_per_row));
    for (int p = 0; p < P; ++p) {
        if (p < P - 1) {
            if (a.pairs)
                sort_pass<K, true, IP, false><<<grid, dim3(kPassBlock), 0, stream>>>(io, p, m, n, l.tiles_per_row, ghist, moves, status, g_sort_poll_limit);
            else
                sort_pass<K, false, IK, false><<<grid, dim3(kPassBlock), 0, stream>>>(io, p, m, n, l.tiles_per_row, ghist, moves, status, g_sort_poll_limit);
        } else {
            if (a.pairs)
                sort_pass<K, true, IP, true><<<grid, dim3(kPassBlock), 0, stream>>>(io, p, m, n, l.tiles_per_row, ghist, moves, status, g_sort_poll_limit);
            else
                sort_pass<K, false, IK, true><<<grid, dim3(kPassBlock), 0, stream>>>(io, p, m, n, l.tiles_per_row, ghist, moves, status, g_sort_poll_limit);
        }
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
    case DLFX_F16: a.kind = kKeyFloat; return run_sort<uint16_t>(stream, a, scratch, scratch_bytes);
    case DLFX_I16: a.kind = kKeyInt;   return run_sort<uint16_t>(stream, a, scratch, scratch_bytes);
    default: return DLFX_ERR_UNSUPPORTED_DTYPE;
    }
}

}  // namespace

bool set_sort_tuning(const char* key, int64_t value) {
    if (!std::strcmp(key, "sort_poll_limit") && value >= 0 && value <= (1 << 30)) {
        g_sort_poll_limit = static_cast<int>(value);
        return true;
    }
    if (!std::strcmp(key, "sort_buckets") && value >= 0 && value <= 1) {
        g_sort_buckets = static_cast<int>(value);
        return true;
    }
    if (!std::strcmp(key, "sort_compare_max") && value >= 0 && value <= 4096) {
        g_sort_compare_max = static_cast<int>(value);
        return true;
    }
    if (!std::strcmp(key, "sort_wave_rows") && value >= 0 && value <= 512) {
        g_sort_wave_rows = static_cast<int>(value);
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
    const size_t es = dtype == DLFX_BOOL ? 0 : dtype_size(dtype);
    if (!es || m <= 0 || n <= 0) return 0;
    return sort_layout(es, true, m, n).total;
}

}  // namespace dlfx

using namespace dlfx;

extern "C" size_t dlfx_sort_scratch_bytes(int dtype, int64_t m, int64_t n) {
    const size_t es = dtype == DLFX_BOOL ? 0 : dtype_size(dtype);
    if (!es || m <= 0 || n <= 0) return 0;
    return sort_layout(es, false, m, n).total;
}

extern "C" int dlfx_sort(dlfx_stream_t stream, int dir, int dtype, int rank, const int64_t* dims,
                         const void* x, int64_t x_offset, const int64_t* x_strides,
                         void* y, int64_t y_offset, const int64_t* y_strides,
                         void* scratch, size_t scratch_bytes) {
    if (!x || !y || rank < 1) return DLFX_ERR_INVALID_ARGUMENT;
    if (!view_ok(rank, dims, x_strides) || !view_ok(rank, dims, y_strides)) return DLFX_ERR_INVALID_ARGUMENT;
    const size_t es = dtype == DLFX_BOOL ? 0 : dtype_size(dtype);
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
    const size_t es = dtype == DLFX_BOOL ? 0 : dtype_size(dtype);
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

#ifdef DLFX_SORT_TIMING
extern "C" void dlfx_debug_sort_phases(unsigned long long* out, int reset) {
    static unsigned long long host[dlfx::kPhaseSlots * 8];
    if (out) {
        (void)hipMemcpyFromSymbol(host, HIP_SYMBOL(dlfx::g_phase_cycles), sizeof(host));
        for (int i = 0; i < 8; ++i) out[i] = 0;
        for (int b = 0; b < dlfx::kPhaseSlots; ++b)
            for (int i = 0; i < 8; ++i) out[i] += host[b * 8 + i];
    }
    if (reset) {
        for (auto& v : host) v = 0;
        (void)hipMemcpyToSymbol(HIP_SYMBOL(dlfx::g_phase_cycles), host, sizeof(host));
    }
}
#endif
