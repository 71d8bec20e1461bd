// Declarations shared by the sort kernels: order-preserving key images, the description of
// what a sort reads and writes, and the entry of the bucket route (sort_split.hip) that
// sort.hip calls.
#pragma once

#include "common.hip.h"

namespace dlfx {

enum KeyKind { kKeyInt = 0, kKeyFloat = 1 };

template <typename K>
struct KeyTraits;
template <>
struct KeyTraits<uint16_t> {
    static constexpr int kPasses = 2;
    static constexpr uint16_t kSign = 0x8000u;
};
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

// What the passes of one sort read and write.
template <typename K>
struct PassIo {
    const K* x;               // strided input, read by the first pass that runs
    DimMap xmap;
    int64_t sx;
    K* kbuf[2];               // contiguous [m][n] ping-pong buffers between passes
    uint32_t* vbuf[2];        // ... and their index payloads (argsort)
    K* y;                     // strided value output of the last pass (may be null)
    DimMap ymap;
    int64_t sy;
    void* idx;                // strided index output of the last pass (may be null)
    DimMap imap;
    int64_t si;
    int idx64;
    int kind, descending;
    int canon_zero;           // argsort of floats: -0.0 and +0.0 are one key
    int restore_zero;         // ... and the value written for a zero key is re-read from x
    int x_intact;             // no output overlaps the input: x can still be read once outputs are being written
    // rows side by side in memory (the axis is an outer dimension): workgroups are dealt to the
    // 8 XCDs in turn, so workgroup b takes block (b % 8) * xcd_blocks + b / 8 and neighbouring
    // rows, which share cache lines, meet in one L2 (0: workgroup b takes block b)
    int64_t xcd_blocks;
};

template <typename K>
__device__ __forceinline__ int64_t block_of(const PassIo<K>& io) {
    if (io.xcd_blocks == 0) return blockIdx.x;
    return static_cast<int64_t>(blockIdx.x % 8) * io.xcd_blocks + blockIdx.x / 8;
}

template <typename K>
__device__ __forceinline__ K key_of_element(const PassIo<K>& io, K bits) {
    if (io.canon_zero && static_cast<K>(bits << 1) == 0) bits = 0;      // -0.0 -> +0.0
    return encode_key<K>(bits, io.kind, io.descending);
}


// The per-(tile, digit) status words that chain the tiles of a row: [tag:4 | inclusive:1 | count:27];
// a word is valid for the launch whose tag it carries, so the array is cleared once per sort.
constexpr uint32_t kCountMask = (1u << 27) - 1;
__device__ __forceinline__ uint32_t make_status(int tag, bool inclusive, uint32_t count) {
    return (static_cast<uint32_t>(tag + 1) << 28) | (inclusive ? (1u << 27) : 0u) | count;
}

constexpr int kRadix = 256;

// ------------------------------------------------------------------ the bucket route (sort_split.hip)
// Whether rows of n keys may take it, the scratch it needs beside the caller's first pair of
// ping-pong buffers, and its launches: every row of the call is sorted by it.
bool split_route_takes(size_t key_size, int64_t m, int64_t n);
size_t split_scratch_bytes(size_t key_size, bool pairs, int64_t m, int64_t n);
template <typename K>
int run_split(hipStream_t stream, const PassIo<K>& io, bool pairs, int64_t m, int64_t n, void* scratch, int compare_max);

// ------------------------------------------------------------------ stable ranks by digit
// Every wavefront of a workgroup ranks its ITEMS x 64 elements, item k of lane l being element
// k * 64 + l of the wavefront's share: rank[k] = how many earlier elements of the wavefront
// carry the same digit d[k] (wave-wide matching over the bits of `vary`; all other bits must
// agree in every element).  wave_hist[w][*] must be zero on entry (and that visible); on return
// (no barrier inside) row w holds the wavefront's count of every digit.
template <int ITEMS>
__device__ __forceinline__ void rank_by_digit(uint32_t* __restrict__ wave_hist_row, const uint32_t (&d)[ITEMS], uint32_t vary, uint32_t (&rank)[ITEMS]) {
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
        uint32_t peers_lo = 0xffffffffu, peers_hi = 0xffffffffu;
        for (uint32_t bits = vary; bits != 0u; bits &= bits - 1u) {
            const uint32_t b = static_cast<uint32_t>(__builtin_ctz(bits));
            const int32_t ones = __builtin_amdgcn_sbfe(static_cast<int32_t>(d[k]), b, 1u);
            const unsigned long long vote = __ballot(ones < 0);
            peers_lo &= ~(static_cast<uint32_t>(vote) ^ static_cast<uint32_t>(ones));
            peers_hi &= ~(static_cast<uint32_t>(vote >> 32) ^ static_cast<uint32_t>(ones));
        }
        const uint32_t before = __builtin_amdgcn_mbcnt_hi(peers_hi, __builtin_amdgcn_mbcnt_lo(peers_lo, 0u));
        const uint32_t cnt = static_cast<uint32_t>(__popc(peers_lo) + __popc(peers_hi));
        const uint32_t seen = wave_hist_row[d[k]];
        rank[k] = seen + before;
        __builtin_amdgcn_wave_barrier();
        if (before == 0) wave_hist_row[d[k]] = seen + cnt;
        __builtin_amdgcn_wave_barrier();
    }
}

// ------------------------------------------------------------------ a sort that stays in one workgroup
constexpr int kSmallMoves = 256;         // keys that the run walk of sort_in_workgroup may move (one thread each)

template <typename K, bool PAIRS, int ITEMS, int WAVES = 4>
struct SmallShared {
    uint32_t n_moves;
    uint2 moves[kSmallMoves];
    uint32_t wave_hist[WAVES][kRadix];
    uint32_t scan_tmp[kRadix / kWave];
    K wave_or[WAVES], wave_and[WAVES];
    K keys[WAVES * kWave * ITEMS];
    uint32_t vals[PAIRS ? WAVES * kWave * ITEMS : 1];
};

// The passes of a workgroup-resident sort: key[] / val[] hold the row (or bucket) in element
// order before and after; `ors` / `ands` are this thread's OR / AND over its valid keys, `top`
// the number of low digits that may differ (digits from `top` up are known to be equal),
// `valid` the number of keys that are not padding.  The workgroup has WAVES wavefronts (4 or 8).
//
// When more digits vary than `valid` distinct keys need to tell most of them apart (about as
// many bits as the square of `valid` has, so that evenly spread keys leave a few pairs that
// agree), the leading ones of the varying digits are sorted first.  Keys that then agree with
// a neighbour in all of those digits form short runs, in source order; every key of such a run
// finds its place by comparing whole keys with the run's other members (at most kNear to
// either side), and the lower digits never ran.  A longer run makes every digit run from that
// arrangement, which the passes so far left in source order among equal keys.
//
// BY_VAL (pairs only): the digits are taken from val[] instead of key[] - the same stable passes
// ordering the entries by their 32-bit payload, `ors` / `ands` / `top` then describe the payloads
// (in a K).  Sorting by payload and then by key gives the order by (key, payload) whatever order
// the entries arrived in.
template <typename K, bool PAIRS, int ITEMS, int WAVES = 4, bool BY_VAL = false>
__device__ __forceinline__ void sort_in_workgroup(SmallShared<K, PAIRS, ITEMS, WAVES>& sm, K (&key)[ITEMS], uint32_t (&val)[PAIRS ? ITEMS : 1],
                                                  K ors, K ands, int valid, int top) {
    static_assert(WAVES * kWave >= kRadix, "a thread per digit");
    static_assert(PAIRS || !BY_VAL, "only pairs have a payload to sort by");
    auto word = [&](int k) -> K {
        if constexpr (BY_VAL) return static_cast<K>(val[k]);
        else return key[k];
    };
    const bool padded = valid < WAVES * kWave * ITEMS;
    const int tid = threadIdx.x;
    const int lane = lane_id();
    const int w = tid / kWave;
    const int seg = w * kWave * ITEMS + lane;
    ors = wave_reduce(ors, [](K a, K b) { return static_cast<K>(a | b); });
    ands = wave_reduce(ands, [](K a, K b) { return static_cast<K>(a & b); });
    if (lane == 0) {
        sm.wave_or[w] = ors;
        sm.wave_and[w] = ands;
    }
    if (tid == 0) sm.n_moves = 0u;
    __syncthreads();
    K any = 0, all = ~K(0);
#pragma unroll
    for (int i = 0; i < WAVES; ++i) {
        any |= sm.wave_or[i];
        all &= sm.wave_and[i];
    }
    const K differ = static_cast<K>(any & ~all);
    const bool owner = tid < kRadix;                       // thread d < 256 owns digit d

    int first = 0;                                         // lowest digit of this round of passes
    if constexpr (sizeof(K) > 4 && !BY_VAL) {
        const int enough = (2 * (32 - __builtin_clz(static_cast<uint32_t>(valid > 1 ? valid - 1 : 1))) - 2 + 7) / 8;
        int varying = 0;
        for (int p = top - 1; p >= 0; --p) {
            if ((static_cast<uint32_t>(differ >> (8 * p)) & 0xffu) != 0u && ++varying == enough) first = p;
        }
        if (varying <= enough) first = 0;
    }

    for (;;) {
        for (int pass = first; pass < top; ++pass) {
            const int shift = 8 * pass;
            const uint32_t moves = static_cast<uint32_t>(differ >> shift) & 0xffu;
            if (moves == 0u) continue;                        // this digit is the same in the whole row
            const uint32_t vary = padded ? 0xffu : moves;     // padding differs from the row in other bits too
            for (int i = tid; i < WAVES * kRadix; i += WAVES * kWave) (&sm.wave_hist[0][0])[i] = 0;
            __syncthreads();

            // ---- rank inside the wave, in element order
            uint32_t rank[ITEMS];
#pragma unroll
            for (int k0 = 0; k0 < ITEMS; k0 += 2) {
                uint32_t d[2], before[2], cnt[2];
#pragma unroll
                for (int j = 0; j < 2; ++j) d[j] = static_cast<uint32_t>(word(k0 + j) >> shift) & 0xffu;
                uint32_t peers_lo[2] = {0xffffffffu, 0xffffffffu}, peers_hi[2] = {0xffffffffu, 0xffffffffu};
                for (uint32_t bits = vary; bits != 0u; bits &= bits - 1u) {
                    const uint32_t b = static_cast<uint32_t>(__builtin_ctz(bits));
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        const int32_t ones = __builtin_amdgcn_sbfe(static_cast<int32_t>(d[j]), b, 1u);
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
                    const uint32_t seen = sm.wave_hist[w][d[j]];
                    rank[k0 + j] = seen + before[j];
                    __builtin_amdgcn_wave_barrier();
                    if (before[j] == 0) sm.wave_hist[w][d[j]] = seen + cnt[j];
                    __builtin_amdgcn_wave_barrier();
                }
            }
            __syncthreads();

            // ---- thread d owns digit d: where the digit starts in the row, and each wave's share of it
            {
                uint32_t wave_count[WAVES];
                uint32_t count = 0;
                if (owner) {
#pragma unroll
                    for (int i = 0; i < WAVES; ++i) {
                        wave_count[i] = sm.wave_hist[i][tid];
                        count += wave_count[i];
                    }
                }
                const uint32_t incl = wave_scan_inclusive(count, 0u, [](uint32_t a, uint32_t b) { return a + b; });
                if (owner && lane == kWave - 1) sm.scan_tmp[w] = incl;
                __syncthreads();
                if (owner) {
                    uint32_t run = incl - count;
                    for (int i = 0; i < w; ++i) run += sm.scan_tmp[i];
#pragma unroll
                    for (int i = 0; i < WAVES; ++i) {
                        sm.wave_hist[i][tid] = run;
                        run += wave_count[i];
                    }
                }
            }
            __syncthreads();

            // ---- scatter to the sorted position, reload in element order
#pragma unroll
            for (int k = 0; k < ITEMS; ++k) {
                const uint32_t pos = sm.wave_hist[w][static_cast<uint32_t>(word(k) >> shift) & 0xffu] + rank[k];
                sm.keys[pos] = key[k];
                if constexpr (PAIRS) sm.vals[pos] = val[k];
            }
            __syncthreads();
#pragma unroll
            for (int k = 0; k < ITEMS; ++k) {
                key[k] = sm.keys[seg + k * kWave];
                if constexpr (PAIRS) val[k] = sm.vals[seg + k * kWave];
            }
            // (the three barriers of the next pass lie between these reads and its scatter)
        }
        if (first == 0) break;
        // Runs of neighbours that agree in every digit sorted so far.  Keys with such a neighbour
        // are few: each walks its run (the tile holds what the registers hold), and the ones that
        // have to move are listed.
        constexpr int kNear = 3;
        const int sh = 8 * first;
        uint32_t near = 0;                                 // bit k: item k has a neighbour of its run
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) {
            const int e = seg + k * kWave;
            if (e < valid) {
                const K lead = key[k] >> sh;
                const bool left = e > 0 && (sm.keys[e - 1] >> sh) == lead;
                const bool right = e + 1 < valid && (sm.keys[e + 1] >> sh) == lead;
                if (left || right) near |= 1u << k;
            }
        }
        bool longer = false;
        for (; near != 0u; near &= near - 1u) {
            const int e = seg + __builtin_ctz(near) * kWave;
            const K mine = sm.keys[e];
            const K lead = mine >> sh;
            int before = 0, ahead = 0;                     // members of the run to the left; of the whole run that come first
            int j = e - 1;
            for (; j >= 0 && before < kNear; --j, ++before) {
                const K other = sm.keys[j];
                if ((other >> sh) != lead) break;
                ahead += other <= mine ? 1 : 0;
            }
            if (before == kNear && j >= 0 && (sm.keys[j] >> sh) == lead) longer = true;
            int after = 0;
            for (j = e + 1; j < valid && after < kNear; ++j, ++after) {
                const K other = sm.keys[j];
                if ((other >> sh) != lead) break;
                ahead += other < mine ? 1 : 0;
            }
            if (after == kNear && j < valid && (sm.keys[j] >> sh) == lead) longer = true;
            const int dest = e - before + ahead;
            if (dest != e) {
                const uint32_t slot = atomicAdd(&sm.n_moves, 1u);
                if (slot < static_cast<uint32_t>(kSmallMoves)) sm.moves[slot] = make_uint2(static_cast<uint32_t>(e), static_cast<uint32_t>(dest));
                else longer = true;
            }
        }
        if (__syncthreads_or(longer ? 1 : 0)) {            // a run too long, or too many moves: every digit runs
            first = 0;
            continue;
        }
        const int n_moves = static_cast<int>(sm.n_moves);
        if (n_moves != 0) {
            uint2 mv = make_uint2(0u, 0u);
            K moved_key = 0;
            uint32_t moved_val = 0;
            if (tid < n_moves) {
                mv = sm.moves[tid];
                moved_key = sm.keys[mv.x];
                if constexpr (PAIRS) moved_val = sm.vals[mv.x];
            }
            __syncthreads();
            if (tid < n_moves) {
                sm.keys[mv.y] = moved_key;
                if constexpr (PAIRS) sm.vals[mv.y] = moved_val;
            }
            __syncthreads();
#pragma unroll
            for (int k = 0; k < ITEMS; ++k) {
                key[k] = sm.keys[seg + k * kWave];
                if constexpr (PAIRS) val[k] = sm.vals[seg + k * kWave];
            }
        }
        break;
    }
}


}  // namespace dlfx
