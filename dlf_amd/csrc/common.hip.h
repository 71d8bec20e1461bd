// Shared device and host helpers for the gfx950 axis-primitive kernels.
//
// Everything here assumes CDNA4: 64-lane wavefronts, DPP row operations and
// row broadcasts, 160 KB of LDS per compute unit.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "../../include/dlfx.h"

namespace dlfx {

constexpr int kWave = 64;
constexpr int kMaxRank = DLFX_MAX_RANK;

// ------------------------------------------------------------------ views
// A group of merged dimensions: flat index -> element offset by a div/mod walk
// from the innermost extent outwards.  rank 0 maps every index to 0.
struct DimMap {
    int rank;
    int64_t dims[kMaxRank];
    int64_t strides[kMaxRank];

    // (always inlined: an out-of-line call takes the address of its map, and a kernel whose
    // argument block holds the map then keeps a private copy of the whole block in scratch memory)
    __host__ __device__ __attribute__((always_inline)) int64_t at(int64_t flat) const {
        if (rank == 1) return flat * strides[0];
        int64_t off = 0;
        for (int i = rank - 1; i > 0; --i) {
            int64_t d = dims[i];
            int64_t q = flat / d;
            off += (flat - q * d) * strides[i];
            flat = q;
        }
        if (rank > 0) off += flat * strides[0];
        return off;
    }
    __host__ __device__ int64_t size() const {
        int64_t s = 1;
        for (int i = 0; i < rank; ++i) s *= dims[i];
        return s;
    }
};

// Host side: copy dims [b, e) of a view into a DimMap, dropping extent-1
// dimensions and merging neighbours that walk memory as one dimension.
// Returns false when more than kMaxRank dimensions remain.
inline bool make_dim_map(const int64_t* dims, const int64_t* strides, int b, int e, DimMap* out) {
    int r = 0;
    int64_t d[64], s[64];
    for (int i = b; i < e; ++i) {
        if (dims[i] == 1) continue;
        if (r > 0 && s[r - 1] == strides[i] * dims[i]) {
            d[r - 1] *= dims[i];
            s[r - 1] = strides[i];
        } else {
            if (r == 64) return false;
            d[r] = dims[i];
            s[r] = strides[i];
            ++r;
        }
    }
    if (r > kMaxRank) return false;
    out->rank = r;
    for (int i = 0; i < kMaxRank; ++i) {
        out->dims[i] = i < r ? d[i] : 1;
        out->strides[i] = i < r ? s[i] : 0;
    }
    return true;
}

// ------------------------------------------------------------------ bit casts / DPP
template <typename To, typename From>
__device__ __forceinline__ To bit_cast(const From& f) {
    static_assert(sizeof(To) == sizeof(From), "size mismatch");
    return __builtin_bit_cast(To, f);
}

template <int N>
struct Words {
    int w[N];
};

// Complex element (the reference's float2 / double2, std::complex on the host): real part first.
template <typename F>
struct alignas(2 * sizeof(F)) Cx {
    F re, im;
    Cx() = default;
    __host__ __device__ constexpr Cx(F r, F i = F(0)) : re(r), im(i) {}
    template <typename G>
    __host__ __device__ explicit constexpr Cx(const Cx<G>& o) : re(static_cast<F>(o.re)), im(static_cast<F>(o.im)) {}
};
template <typename F>
__host__ __device__ __forceinline__ Cx<F> operator+(Cx<F> a, Cx<F> b) { return {a.re + b.re, a.im + b.im}; }
template <typename F>
__host__ __device__ __forceinline__ Cx<F> operator*(Cx<F> a, Cx<F> b) {
    return {a.re * b.re - a.im * b.im, a.re * b.im + a.im * b.re};
}
template <typename F>
__host__ __device__ __forceinline__ bool operator==(Cx<F> a, Cx<F> b) { return a.re == b.re && a.im == b.im; }
template <typename F>
__host__ __device__ __forceinline__ bool operator!=(Cx<F> a, Cx<F> b) { return !(a == b); }
template <typename T> struct IsComplex : std::false_type {};
template <typename F> struct IsComplex<Cx<F>> : std::true_type {};

// Cross-lane helpers move whole 32-bit words; a 2-byte value rides in the low half of one.
template <typename T>
__device__ __forceinline__ int widen16(T v) {
    static_assert(sizeof(T) == 2, "2-byte values only");
    return static_cast<int>(bit_cast<unsigned short>(v));
}
template <typename T>
__device__ __forceinline__ T narrow16(int w) {
    return bit_cast<T>(static_cast<unsigned short>(w));
}

// Value of `v` in the lane the DPP control selects; lanes whose source is
// outside the row (or masked off by ROW_MASK) receive `fill`.
template <int CTRL, int ROW_MASK = 0xf, int BANK_MASK = 0xf, typename T>
__device__ __forceinline__ T dpp_fetch(T v, T fill) {
    if constexpr (sizeof(T) == 2) {
        return narrow16<T>(__builtin_amdgcn_update_dpp(widen16(fill), widen16(v), CTRL, ROW_MASK, BANK_MASK, false));
    } else {
    static_assert(sizeof(T) % 4 == 0, "whole 32-bit words only");
    constexpr int N = sizeof(T) / 4;
    Words<N> a = bit_cast<Words<N>>(v), f = bit_cast<Words<N>>(fill), r;
#pragma unroll
    for (int i = 0; i < N; ++i)
        r.w[i] = __builtin_amdgcn_update_dpp(f.w[i], a.w[i], CTRL, ROW_MASK, BANK_MASK, false);
    return bit_cast<T>(r);
    }
}

template <typename T>
__device__ __forceinline__ T lane_xor(T v, int mask) {
    if constexpr (sizeof(T) == 2) {
        return narrow16<T>(__shfl_xor(widen16(v), mask, kWave));
    } else {
        constexpr int N = sizeof(T) / 4;
        Words<N> a = bit_cast<Words<N>>(v);
#pragma unroll
        for (int i = 0; i < N; ++i) a.w[i] = __shfl_xor(a.w[i], mask, kWave);
        return bit_cast<T>(a);
    }
}

template <typename T>
__device__ __forceinline__ T lane_get(T v, int lane) {
    if constexpr (sizeof(T) == 2) {
        return narrow16<T>(__shfl(widen16(v), lane, kWave));
    } else {
        constexpr int N = sizeof(T) / 4;
        Words<N> a = bit_cast<Words<N>>(v);
#pragma unroll
        for (int i = 0; i < N; ++i) a.w[i] = __shfl(a.w[i], lane, kWave);
        return bit_cast<T>(a);
    }
}

// Broadcast of one lane's value through a scalar register (lane is uniform).
template <typename T>
__device__ __forceinline__ T lane_read(T v, int lane) {
    if constexpr (sizeof(T) == 2) {
        return narrow16<T>(__builtin_amdgcn_readlane(widen16(v), lane));
    } else {
        constexpr int N = sizeof(T) / 4;
        Words<N> a = bit_cast<Words<N>>(v);
#pragma unroll
        for (int i = 0; i < N; ++i) a.w[i] = __builtin_amdgcn_readlane(a.w[i], lane);
        return bit_cast<T>(a);
    }
}

// DPP controls used below.
constexpr int kQuadXor1 = 0xB1;      // quad_perm [1,0,3,2]
constexpr int kQuadXor2 = 0x4E;      // quad_perm [2,3,0,1]
constexpr int kRowHalfMirror = 0x141;
constexpr int kRowMirror = 0x140;
constexpr int kRowShr1 = 0x111, kRowShr2 = 0x112, kRowShr4 = 0x114, kRowShr8 = 0x118;
constexpr int kRowBcast15 = 0x142, kRowBcast31 = 0x143;

// Value of `v` in lane (lane ^ J), J a power of two.  Distances below 16 stay inside a DPP
// row and cost one or two moves; 16 and 32 cross rows with one lane-swap instruction and a select.
template <int J, typename T>
__device__ __forceinline__ T lane_xor_const(T v) {
    if constexpr (J == 1) return dpp_fetch<kQuadXor1>(v, v);
    else if constexpr (J == 2) return dpp_fetch<kQuadXor2>(v, v);
    else if constexpr (J == 4) {
        // banks are groups of four lanes: even banks take lane + 4, odd banks lane - 4
        const T up = dpp_fetch<0x104, 0xf, 0x5>(v, v);        // row_shl:4 into banks 0 and 2
        return dpp_fetch<0x114, 0xf, 0xa>(v, up);             // row_shr:4 into banks 1 and 3
    } else if constexpr (J == 8) return dpp_fetch<0x128>(v, v);   // row_ror:8
    else {
        // v_permlane16_swap exchanges the odd rows of its first operand with the even rows of
        // its second, v_permlane32_swap the upper half of the first with the lower half of the
        // second: with both operands holding v, the first result carries v's even rows (lower
        // half) twice and the second its odd rows (upper half) twice.
        static_assert(J == 16 || J == 32, "power-of-two distance inside a wavefront");
        const bool upper = (__lane_id() & J) != 0;
        auto word = [&](int w) -> int {
            const unsigned u = static_cast<unsigned>(w);
            if constexpr (J == 16) {
                const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
                return static_cast<int>(upper ? r[0] : r[1]);
            } else {
                const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
                return static_cast<int>(upper ? r[0] : r[1]);
            }
        };
        if constexpr (sizeof(T) == 2) {
            return narrow16<T>(word(widen16(v)));
        } else {
            constexpr int N = sizeof(T) / 4;
            Words<N> a = bit_cast<Words<N>>(v);
#pragma unroll
            for (int i = 0; i < N; ++i) a.w[i] = word(a.w[i]);
            return bit_cast<T>(a);
        }
    }
}

// Bitonic network over aligned groups of WIDTH lanes (a power of two, at most 64); the group
// that starts at lane 0 ends up best-first.  `exchange(J, keep_better)` must replace the lane's
// item by the item of lane ^ J when that one is better and keep_better holds, or when it is not
// better and keep_better does not hold.
// SAME_WAY: every group of WIDTH lanes ends in the same direction (first item in its lowest
// lane); otherwise neighbouring groups end in opposite directions, as a later merge wants.
template <int WIDTH, bool SAME_WAY = false, typename Exchange>
__device__ __forceinline__ void wave_bitonic(Exchange exchange) {
    const int lane = __lane_id();
    auto step = [&](auto jc, int k) {
        constexpr int J = decltype(jc)::value;
        const bool up = (SAME_WAY && k == WIDTH) ? true : (lane & k) == 0;
        exchange(jc, ((lane & J) == 0) == up);
    };
#pragma unroll
    for (int k = 2; k <= WIDTH; k <<= 1) {
        if (k >= 64) step(std::integral_constant<int, 32>(), k);
        if (k >= 32) step(std::integral_constant<int, 16>(), k);
        if (k >= 16) step(std::integral_constant<int, 8>(), k);
        if (k >= 8) step(std::integral_constant<int, 4>(), k);
        if (k >= 4) step(std::integral_constant<int, 2>(), k);
        step(std::integral_constant<int, 1>(), k);
    }
}

// Sorts one value per lane, largest in lane 0 of each even group of WIDTH lanes.
template <int WIDTH = kWave, typename T>
__device__ __forceinline__ T wave_sort_descending(T v) {
    wave_bitonic<WIDTH>([&](auto jc, bool keep_better) {
        const T other = lane_xor_const<decltype(jc)::value>(v);
        v = (keep_better == (other > v)) ? other : v;
    });
    return v;
}

template <typename T>
__device__ __forceinline__ T lane_xor_any(T v, int j) {      // j is a constant after unrolling
    switch (j) {
        case 1: return lane_xor_const<1>(v);
        case 2: return lane_xor_const<2>(v);
        case 4: return lane_xor_const<4>(v);
        case 8: return lane_xor_const<8>(v);
        case 16: return lane_xor_const<16>(v);
        default: return lane_xor_const<32>(v);
    }
}

// Bitonic network over the 64 * ITEMS (key, index) entries of a wavefront; entry i * 64 + lane
// is item i of the lane and ends up holding the entry of that rank in the order `first`
// (first(ka, ia, kb, ib): entry a comes strictly before entry b).  Exchanges at a distance
// below 64 cross lanes; the others pair two items of one lane, with a direction known at
// compile time.  The indices travel only when PAIRS is set.
template <bool PAIRS, int ITEMS, typename K, typename First>
__device__ __forceinline__ void wave_bitonic_items(K (&key)[ITEMS], uint32_t (&idx)[ITEMS], First first) {
    constexpr int N = kWave * ITEMS;
    const int lane = __lane_id();
#pragma unroll
    for (int k = 2; k <= N; k <<= 1) {
#pragma unroll
        for (int j = k >> 1; j >= 1; j >>= 1) {
            if (j >= kWave) {
                const int jj = j / kWave;
#pragma unroll
                for (int i = 0; i < ITEMS; ++i) {
                    if (i & jj) continue;
                    const int o = i | jj;
                    const bool ascending = ((i * kWave) & k) == 0;
                    const bool swap = ascending ? first(key[o], idx[o], key[i], idx[i]) : first(key[i], idx[i], key[o], idx[o]);
                    const K ka = key[i], kb = key[o];
                    key[i] = swap ? kb : ka;
                    key[o] = swap ? ka : kb;
                    if constexpr (PAIRS) {
                        const uint32_t ia = idx[i], ib = idx[o];
                        idx[i] = swap ? ib : ia;
                        idx[o] = swap ? ia : ib;
                    }
                }
            } else {
                const bool low = (lane & j) == 0;
#pragma unroll
                for (int i = 0; i < ITEMS; ++i) {
                    const bool ascending = k < kWave ? (lane & k) == 0 : ((i * kWave) & k) == 0;
                    const bool keep_first = low == ascending;
                    const K other_key = lane_xor_any(key[i], j);
                    if constexpr (PAIRS) {
                        const uint32_t other_idx = lane_xor_any(idx[i], j);
                        if (keep_first == first(other_key, other_idx, key[i], idx[i])) {
                            key[i] = other_key;
                            idx[i] = other_idx;
                        }
                    } else {
                        if (keep_first == first(other_key, 0u, key[i], 0u)) key[i] = other_key;
                    }
                }
            }
        }
    }
}

// All-lanes reduction over a wavefront with a commutative `join`.
template <typename T, typename Join>
__device__ __forceinline__ T wave_reduce(T v, Join join) {
    v = join(v, dpp_fetch<kQuadXor1>(v, v));
    v = join(v, dpp_fetch<kQuadXor2>(v, v));
    v = join(v, dpp_fetch<kRowHalfMirror>(v, v));
    v = join(v, dpp_fetch<kRowMirror>(v, v));
    v = join(v, lane_xor_const<16>(v));
    v = join(v, lane_xor_const<32>(v));
    return v;
}

// Reduction over aligned groups of `width` lanes (power of two, <= 64); every
// lane of a group ends with the group's result.
template <typename T, typename Join>
__device__ __forceinline__ T group_reduce(T v, int width, Join join) {
    if (width > 1) v = join(v, dpp_fetch<kQuadXor1>(v, v));
    if (width > 2) v = join(v, dpp_fetch<kQuadXor2>(v, v));
    if (width > 4) v = join(v, dpp_fetch<kRowHalfMirror>(v, v));
    if (width > 8) v = join(v, dpp_fetch<kRowMirror>(v, v));
    if (width > 16) v = join(v, lane_xor_const<16>(v));
    if (width > 32) v = join(v, lane_xor_const<32>(v));
    return v;
}

// Inclusive scan over a wavefront: lane i receives op(v0, ..., vi) with the
// operands in lane order.  `id` is the operator's identity.
template <typename T, typename Op>
__device__ __forceinline__ T wave_scan_inclusive(T v, T id, Op op) {
    v = op(dpp_fetch<kRowShr1>(v, id), v);
    v = op(dpp_fetch<kRowShr2>(v, id), v);
    v = op(dpp_fetch<kRowShr4>(v, id), v);
    v = op(dpp_fetch<kRowShr8>(v, id), v);
    v = op(dpp_fetch<kRowBcast15, 0xa>(v, id), v);
    v = op(dpp_fetch<kRowBcast31, 0xc>(v, id), v);
    return v;
}

__device__ __forceinline__ int lane_id() { return __lane_id(); }

// ------------------------------------------------------------------ vectors
template <typename T, int N>
struct alignas(sizeof(T) * N) Vec {
    T v[N];
};

// Elements per 128-bit load.
template <typename T>
constexpr int vec_width() { return 16 / sizeof(T); }

// Streaming accesses: data that is touched once is loaded / stored with the non-temporal
// hint so that it does not displace what the caches could reuse.  On MI355X this alone
// lifts a read-only stream from about 5.9 to 6.6 TB/s.
template <typename T, int N>
__device__ __forceinline__ Vec<T, N> load_stream(const Vec<T, N>* p) {
    if constexpr (std::is_class<T>::value) {
        // structs travel as the 32-bit words they are made of
        constexpr int W = N * static_cast<int>(sizeof(T)) / 4;
        return bit_cast<Vec<T, N>>(load_stream(reinterpret_cast<const Vec<uint32_t, W>*>(p)));
    } else if constexpr (N == 1) {
        Vec<T, 1> r;
        r.v[0] = __builtin_nontemporal_load(reinterpret_cast<const T*>(p));
        return r;
    } else {
        typedef T NV __attribute__((ext_vector_type(N)));
        const NV nv = __builtin_nontemporal_load(reinterpret_cast<const NV*>(p));
        Vec<T, N> r;
#pragma unroll
        for (int e = 0; e < N; ++e) r.v[e] = nv[e];
        return r;
    }
}
template <typename T, int N>
__device__ __forceinline__ void store_stream(Vec<T, N>* p, const Vec<T, N>& v) {
    if constexpr (std::is_class<T>::value) {
        constexpr int W = N * static_cast<int>(sizeof(T)) / 4;
        store_stream(reinterpret_cast<Vec<uint32_t, W>*>(p), bit_cast<Vec<uint32_t, W>>(v));
    } else if constexpr (N == 1) {
        __builtin_nontemporal_store(v.v[0], reinterpret_cast<T*>(p));
    } else {
        typedef T NV __attribute__((ext_vector_type(N)));
        NV nv;
#pragma unroll
        for (int e = 0; e < N; ++e) nv[e] = v.v[e];
        __builtin_nontemporal_store(nv, reinterpret_cast<NV*>(p));
    }
}
template <typename T>
__device__ __forceinline__ T load_stream(const T* p) {
    if constexpr (std::is_class<T>::value) return load_stream(reinterpret_cast<const Vec<T, 1>*>(p)).v[0];
    else return __builtin_nontemporal_load(p);
}
template <typename T>
__device__ __forceinline__ void store_stream(T* p, T v) {
    if constexpr (std::is_class<T>::value) {
        Vec<T, 1> one;
        one.v[0] = v;
        store_stream(reinterpret_cast<Vec<T, 1>*>(p), one);
    } else {
        __builtin_nontemporal_store(v, p);
    }
}

// ------------------------------------------------------------------ host launch helpers
inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// Records a HIP failure for dlfx_last_hip_error and returns DLFX_ERR_LAUNCH.
int record_hip_error(hipError_t e);

#define DLFX_CHECK_LAUNCH()                                      \
    do {                                                         \
        hipError_t e_ = hipGetLastError();                       \
        if (e_ != hipSuccess) return dlfx::record_hip_error(e_); \
    } while (0)

// Workgroups of `kernel` that the current device holds at once (0 when HIP cannot tell).
template <typename Kernel>
int64_t resident_workgroups(Kernel kernel, int block) {
    int device = 0, units = 0, per_unit = 0;
    if (hipGetDevice(&device) != hipSuccess) return 0;
    if (hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) return 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_unit, kernel, block, 0) != hipSuccess) return 0;
    return static_cast<int64_t>(units) * per_unit;
}

// True when launches into `stream` are being recorded into a graph (or that cannot be told).
inline bool stream_is_capturing(hipStream_t stream) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
        (void)hipGetLastError();
        return true;
    }
    return status != hipStreamCaptureStatusNone;
}

// Common argument validation for a strided view.
inline bool view_ok(int rank, const int64_t* dims, const int64_t* strides) {
    if (rank < 0 || rank > 64) return false;
    if (rank > 0 && (!dims || !strides)) return false;
    for (int i = 0; i < rank; ++i)
        if (dims[i] <= 0) return false;
    return true;
}

inline int64_t view_size(int rank, const int64_t* dims) {
    int64_t s = 1;
    for (int i = 0; i < rank; ++i) s *= dims[i];
    return s;
}

template <typename F>
inline int dispatch_dtype(int dtype, F&& f) {
    switch (dtype) {
    case DLFX_F32: return f(float());
    case DLFX_F64: return f(double());
    case DLFX_I32: return f(int32_t());
    case DLFX_I64: return f(int64_t());
    default: return DLFX_ERR_UNSUPPORTED_DTYPE;
    }
}

using half_t = _Float16;      // IEEE half as a native scalar type

// The four wide types plus half.
template <typename F>
inline int dispatch_dtype_half(int dtype, F&& f) {
    if (dtype == DLFX_F16) return f(half_t());
    return dispatch_dtype(dtype, f);
}

// The four wide types plus the two 16-bit ones.
template <typename F>
inline int dispatch_dtype16(int dtype, F&& f) {
    switch (dtype) {
    case DLFX_F16: return f(half_t());
    case DLFX_I16: return f(int16_t());
    default: return dispatch_dtype(dtype, f);
    }
}

inline size_t dtype_size(int dtype) {
    switch (dtype) {
    case DLFX_F32: case DLFX_I32: return 4;
    case DLFX_F64: case DLFX_I64: case DLFX_C64: return 8;
    case DLFX_C128: return 16;
    case DLFX_F16: case DLFX_I16: return 2;
    case DLFX_BOOL: return 1;
    default: return 0;
    }
}

}  // namespace dlfx
