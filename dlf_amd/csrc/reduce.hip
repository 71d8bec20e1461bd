// reduce / arg_reduce over strided views for gfx950.
//
// Three row shapes get their own kernels:
//   * rows whose reduced elements are contiguous in memory: 128-bit loads, a
//     group of 1..64 lanes per row (short rows), or one or more 256-thread
//     workgroups per row (long rows) with a small second stage;
//   * reductions across a strided axis while a kept axis is contiguous
//     ("columns"): lanes run along the contiguous kept axis so every load
//     instruction is a contiguous 256-byte segment, four waves split the
//     reduced axis and combine through LDS;
//   * anything else: the row kernels with per-element address computation.
// All of them are bandwidth bound; fp32 sums accumulate in fp64 registers.
#include <atomic>
#include <cmath>
#include <cstring>
#include <limits>
#include <type_traits>

#include "common.hip.h"

namespace dlfx {
namespace {

enum JoinKind { kAdd = 0, kMul = 1, kMax = 2, kMin = 3 };
enum MapKind { kMapId = 0, kMapExp = 1, kMapAbs = 2, kMapSquare = 3, kMapNorm = 4 };     // norm: |x|^2, x*x for reals
enum FinalKind { kFinalId = 0, kFinalMean = 1, kFinalLog = 2, kFinalSqrt = 3 };

constexpr int kBlock = 256;

template <typename T, int J>
struct AccType { using type = T; };
template <> struct AccType<float, kAdd> { using type = double; };
template <> struct AccType<float, kMul> { using type = double; };
template <int J> struct AccType<half_t, J> { using type = float; };       // half: every fold in fp32, one rounding at the end

// numeric_limits for the element types (the host library has none for half)
template <typename T> struct Limits {
    __host__ __device__ static constexpr T lowest() { return std::numeric_limits<T>::lowest(); }
    __host__ __device__ static constexpr T max() { return std::numeric_limits<T>::max(); }
    __host__ __device__ static constexpr T infinity() { return std::numeric_limits<T>::infinity(); }
};
template <> struct Limits<half_t> {
    __host__ __device__ static constexpr half_t lowest() { return static_cast<half_t>(-65504.0f); }
    __host__ __device__ static constexpr half_t max() { return static_cast<half_t>(65504.0f); }
    __host__ __device__ static constexpr half_t infinity() { return static_cast<half_t>(__builtin_inff()); }
};

template <typename T>
__device__ __forceinline__ T wrap_add(T a, T b) {
    if constexpr (std::is_integral<T>::value) {
        using U = typename std::make_unsigned<T>::type;
        return static_cast<T>(static_cast<U>(a) + static_cast<U>(b));
    } else {
        return a + b;
    }
}
template <typename T>
__device__ __forceinline__ T wrap_mul(T a, T b) {
    if constexpr (std::is_integral<T>::value) {
        using U = typename std::make_unsigned<T>::type;
        return static_cast<T>(static_cast<U>(a) * static_cast<U>(b));
    } else {
        return a * b;
    }
}

// Map -> fold -> Final of the reducer table (dlf/include/tensor/xfn.h:661-805).
template <typename T, int J, int M>
struct ValueReducer {
    using in_t = T;
    using acc_t = typename AccType<T, J>::type;
    using out_t = T;
    using param_t = int;      // no run-time parameter

    __device__ static __forceinline__ acc_t identity() {
        if constexpr (J == kAdd) return acc_t(0);
        else if constexpr (J == kMul) return acc_t(1);
        else if constexpr (J == kMax) return (M == kMapAbs) ? acc_t(0) : static_cast<acc_t>(Limits<T>::lowest());
        else return static_cast<acc_t>(Limits<T>::max());
    }
    __device__ static __forceinline__ acc_t map(T x, int64_t, param_t) {
        if constexpr (M == kMapExp) {
            if constexpr (std::is_same<T, float>::value || std::is_same<T, half_t>::value) return static_cast<acc_t>(expf(static_cast<float>(x)));
            else return static_cast<acc_t>(exp(static_cast<double>(x)));
        } else if constexpr (M == kMapAbs) {
            if constexpr (std::is_integral<T>::value) {
                using U = typename std::make_unsigned<T>::type;
                return x < 0 ? static_cast<T>(U(0) - static_cast<U>(x)) : x;
            } else {
                return x < T(0) ? -static_cast<acc_t>(x) : static_cast<acc_t>(x);
            }
        } else if constexpr (M == kMapSquare) {
            acc_t v = static_cast<acc_t>(x);
            return wrap_mul(v, v);
        } else {
            return static_cast<acc_t>(x);
        }
    }
    __device__ static __forceinline__ acc_t join(acc_t a, acc_t b) {
        if constexpr (J == kAdd) return wrap_add(a, b);
        else if constexpr (J == kMul) return wrap_mul(a, b);
        else if constexpr (J == kMax) return (a < b) ? b : a;
        else return (b < a) ? b : a;
    }
    __device__ static __forceinline__ out_t finish(acc_t a, int64_t n, int final_op) {
        if constexpr (std::is_integral<T>::value) {
            if (final_op == kFinalMean) return static_cast<T>(a / static_cast<T>(n));
            return static_cast<T>(a);
        } else {
            double v = static_cast<double>(a);
            if (final_op == kFinalMean) v = v / static_cast<double>(n);
            else if (final_op == kFinalLog) v = log(v);
            else if (final_op == kFinalSqrt) v = sqrt(v);
            return static_cast<T>(v);
        }
    }
};

// The same table over complex elements (std::complex on the reference's host side: abs and
// norm give a real value held in a complex, exp / log / sqrt are the principal complex
// functions, mean divides by (n, 0)).  Both parts accumulate in fp64.  Ordering reducers
// (max, min, amax, amin) have no meaning here and are rejected by the caller.
template <typename F, int J, int M>
struct ComplexReducer {
    using in_t = Cx<F>;
    using acc_t = Cx<double>;
    using out_t = Cx<F>;
    using param_t = int;

    __device__ static __forceinline__ acc_t identity() { return J == kMul ? acc_t(1.0, 0.0) : acc_t(0.0, 0.0); }
    __device__ static __forceinline__ acc_t map(in_t x, int64_t, param_t) {
        if constexpr (M == kMapExp) {
            if constexpr (std::is_same<F, float>::value) {
                const float e = expf(x.re);
                float s, c;
                sincosf(x.im, &s, &c);
                return acc_t(static_cast<double>(e * c), static_cast<double>(e * s));
            } else {
                const double e = exp(x.re);
                double s, c;
                sincos(x.im, &s, &c);
                return acc_t(e * c, e * s);
            }
        } else if constexpr (M == kMapAbs) {
            return acc_t(hypot(static_cast<double>(x.re), static_cast<double>(x.im)), 0.0);
        } else if constexpr (M == kMapSquare) {
            const acc_t v(x);
            return v * v;
        } else if constexpr (M == kMapNorm) {
            const acc_t v(x);
            return acc_t(v.re * v.re + v.im * v.im, 0.0);
        } else {
            return acc_t(x);
        }
    }
    __device__ static __forceinline__ acc_t join(acc_t a, acc_t b) { return J == kMul ? a * b : a + b; }
    __device__ static __forceinline__ out_t finish(acc_t a, int64_t n, int final_op) {
        if (final_op == kFinalMean) {
            a = acc_t(a.re / static_cast<double>(n), a.im / static_cast<double>(n));
        } else if (final_op == kFinalLog) {
            a = acc_t(log(hypot(a.re, a.im)), atan2(a.im, a.re));
        } else if (final_op == kFinalSqrt) {
            // principal square root: non-negative real part, imaginary part with the sign of a.im
            const double mod = hypot(a.re, a.im);
            const double big = sqrt((mod + fabs(a.re)) * 0.5);
            const double small = big > 0.0 ? fabs(a.im) / (2.0 * big) : 0.0;
            a = a.re >= 0.0 ? acc_t(big, copysign(small, a.im)) : acc_t(small, copysign(big, a.im));
        }
        return out_t(a);
    }
};

template <typename T>
struct ArgAcc {
    T v;
    int32_t i;
};

// argmax / argmin with the serial loop's semantics
// (dlf/include/tensor/reduce_detail.h:107-132): strict comparison, so the first
// occurrence wins; a NaN in position 0 is never displaced, a NaN elsewhere
// never wins.
template <typename T, bool MAX, typename I>
struct ArgReducer {
    using in_t = T;
    using acc_t = ArgAcc<T>;
    using out_t = I;
    using param_t = int;

    __device__ static __forceinline__ acc_t identity() {
        // weakest possible value, so that any element (even -inf / +inf) ties or wins;
        // ties go to the lower index, and every real index is below this one
        if constexpr (std::is_integral<T>::value)
            return {MAX ? std::numeric_limits<T>::lowest() : std::numeric_limits<T>::max(),
                    std::numeric_limits<int32_t>::max()};
        else
            return {MAX ? static_cast<T>(-Limits<T>::infinity()) : Limits<T>::infinity(),
                    std::numeric_limits<int32_t>::max()};
    }
    __device__ static __forceinline__ acc_t map(T x, int64_t j, param_t) {
        if constexpr (!std::is_integral<T>::value) {
            if (x != x) {
                if (j == 0)
                    return {MAX ? Limits<T>::infinity() : static_cast<T>(-Limits<T>::infinity()), -1};
                return identity();
            }
        }
        return {x, static_cast<int32_t>(j)};
    }
    __device__ static __forceinline__ acc_t join(acc_t a, acc_t b) {
        bool take_b = MAX ? (b.v > a.v) : (b.v < a.v);
        take_b = take_b || (b.v == a.v && b.i < a.i);
        return take_b ? b : a;
    }
    __device__ static __forceinline__ out_t finish(acc_t a, int64_t, int) {
        return static_cast<I>(a.i < 0 ? 0 : a.i);
    }
};

// count: number of elements equal to a value (dlf/include/tensor/reduce.h:151-158: Map
// x == value ? 1 : 0, fold +).  The value is the reducer's run-time parameter.
template <typename T>
struct CountReducer {
    using in_t = T;
    using acc_t = int32_t;
    using out_t = int32_t;
    using param_t = T;

    __device__ static __forceinline__ acc_t identity() { return 0; }
    __device__ static __forceinline__ acc_t map(T x, int64_t, param_t value) { return x == value ? 1 : 0; }
    __device__ static __forceinline__ acc_t join(acc_t a, acc_t b) { return wrap_add(a, b); }
    __device__ static __forceinline__ out_t finish(acc_t a, int64_t, int) { return a; }
};

// --------------------------------------------------------------------------
// One row's contiguous elements, visited by `width` cooperating lanes (lane
// `g` of the group) restricted to 128-bit vectors [v_lo, v_hi) of the aligned
// body; with_head / with_tail add the unaligned ends of the row.
template <typename R, bool STREAM = true>
__device__ __forceinline__ typename R::acc_t
row_partial_contig(const typename R::in_t* __restrict__ p, int64_t n, int g, int width,
                   int64_t part, int64_t parts, typename R::param_t prm, int64_t first_index = 0) {
    using T = typename R::in_t;
    using acc_t = typename R::acc_t;
    constexpr int V = vec_width<T>();
    using VecT = Vec<T, V>;

    auto fetch = [](const VecT* q) __attribute__((always_inline)) { if constexpr (STREAM) return load_stream(q); else return *q; };
    acc_t acc = R::identity();
    const uintptr_t addr = reinterpret_cast<uintptr_t>(p) / sizeof(T);
    int64_t head = (V - static_cast<int64_t>(addr % V)) % V;
    if (head > n) head = n;
    const int64_t nv = (n - head) / V;
    const int64_t tail_start = head + nv * V;

    const int64_t per = (nv + parts - 1) / parts;
    const int64_t v_lo = part * per;
    const int64_t v_hi = (v_lo + per < nv) ? v_lo + per : nv;

    const VecT* __restrict__ pv = reinterpret_cast<const VecT*>(p + head);
    int64_t v = v_lo + g;
    // four independent 128-bit loads in flight per lane
    for (; v + 3 * static_cast<int64_t>(width) < v_hi; v += 4 * static_cast<int64_t>(width)) {
        VecT a = fetch(&pv[v]), b = fetch(&pv[v + width]), c = fetch(&pv[v + 2 * width]),
             d = fetch(&pv[v + 3 * width]);
        const int64_t j0 = first_index + head + v * V;
#pragma unroll
        for (int e = 0; e < V; ++e) acc = R::join(acc, R::map(a.v[e], j0 + e, prm));
#pragma unroll
        for (int e = 0; e < V; ++e) acc = R::join(acc, R::map(b.v[e], j0 + static_cast<int64_t>(width) * V + e, prm));
#pragma unroll
        for (int e = 0; e < V; ++e) acc = R::join(acc, R::map(c.v[e], j0 + 2 * static_cast<int64_t>(width) * V + e, prm));
#pragma unroll
        for (int e = 0; e < V; ++e) acc = R::join(acc, R::map(d.v[e], j0 + 3 * static_cast<int64_t>(width) * V + e, prm));
    }
    // what is left, at most three vectors a lane, again with all loads in flight (rows of a few
    // vectors a lane - many short rows - consist of little else)
    if (v < v_hi) {
        const bool two = v + static_cast<int64_t>(width) < v_hi, three = v + 2 * static_cast<int64_t>(width) < v_hi;
        VecT a = fetch(&pv[v]), b = a, c = a;
        if (two) b = fetch(&pv[v + width]);
        if (three) c = fetch(&pv[v + 2 * width]);
        const int64_t j0 = first_index + head + v * V;
#pragma unroll
        for (int e = 0; e < V; ++e) acc = R::join(acc, R::map(a.v[e], j0 + e, prm));
        if (two) {
#pragma unroll
            for (int e = 0; e < V; ++e) acc = R::join(acc, R::map(b.v[e], j0 + static_cast<int64_t>(width) * V + e, prm));
        }
        if (three) {
#pragma unroll
            for (int e = 0; e < V; ++e) acc = R::join(acc, R::map(c.v[e], j0 + 2 * static_cast<int64_t>(width) * V + e, prm));
        }
    }
    if (part == 0)
        for (int64_t j = g; j < head; j += width) acc = R::join(acc, R::map(p[j], first_index + j, prm));
    if (part == parts - 1)
        for (int64_t j = tail_start + g; j < n; j += width) acc = R::join(acc, R::map(p[j], first_index + j, prm));
    return acc;
}

template <typename R>
__device__ __forceinline__ typename R::acc_t
row_partial_strided(const typename R::in_t* __restrict__ p, const DimMap& red, int64_t n, int g,
                    int width, int64_t part, int64_t parts, typename R::param_t prm) {
    typename R::acc_t acc = R::identity();
    const int64_t per = (n + parts - 1) / parts;
    const int64_t lo = part * per;
    const int64_t hi = (lo + per < n) ? lo + per : n;
    // (two dimensions of fewer than 2^32 elements are told apart with one 32-bit division; four loads in flight)
    const bool two = red.rank == 2 && n <= 0xffffffffLL;
    const uint32_t inner = static_cast<uint32_t>(red.rank == 2 ? red.dims[1] : 1);
    auto where = [&](int64_t j) __attribute__((always_inline)) -> int64_t {
        if (two) {
            const uint32_t q = static_cast<uint32_t>(j) / inner, r = static_cast<uint32_t>(j) - q * inner;
            return static_cast<int64_t>(q) * red.strides[0] + static_cast<int64_t>(r) * red.strides[1];
        }
        return red.at(j);
    };
    int64_t j = lo + g;
    for (; j + 3 * static_cast<int64_t>(width) < hi; j += 4 * static_cast<int64_t>(width)) {
        typename R::in_t v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = p[where(j + u * static_cast<int64_t>(width))];
#pragma unroll
        for (int u = 0; u < 4; ++u) acc = R::join(acc, R::map(v[u], j + u * static_cast<int64_t>(width), prm));
    }
    for (; j < hi; j += width) acc = R::join(acc, R::map(p[where(j)], j, prm));
    return acc;
}

// Short rows: 2^log2g lanes per row, 256 >> log2g rows per workgroup.
// STREAM: the loads carry the non-temporal hint.  Not where a wavefront's access takes part of a
// cache line and another access the rest (rows that are not whole lines, or shorter than the 64
// bytes a lane group reads of each row at a time times a few): the line was then fetched twice -
// fp32 [2867200, 56] 229 us with the hint, 148 us without, [4194304, 16] 77 against 46 us,
// [500000, 100] 59 against 34 us; rows of whole lines from 512 bytes on are faster with it
// (int64 [1048576, 64] 81 against 92 us).
template <typename R, bool CONTIG, bool STREAM>
__global__ __launch_bounds__(kBlock) void reduce_rows_group(
    const typename R::in_t* __restrict__ x, DimMap kept, DimMap red, int64_t m, int64_t n, int log2g,
    typename R::out_t* __restrict__ y, DimMap ymap, int final_op, typename R::param_t prm) {
    const int width = 1 << log2g;
    const int64_t row = static_cast<int64_t>(blockIdx.x) * (kBlock >> log2g) + (threadIdx.x >> log2g);
    const int g = threadIdx.x & (width - 1);
    typename R::acc_t acc = R::identity();
    if (row < m) {
        const typename R::in_t* p = x + kept.at(row);
        if constexpr (CONTIG) acc = row_partial_contig<R, STREAM>(p, n, g, width, 0, 1, prm);
        else acc = row_partial_strided<R>(p, red, n, g, width, 0, 1, prm);
    }
    acc = group_reduce(acc, width, [](typename R::acc_t a, typename R::acc_t b) { return R::join(a, b); });
    if (row < m && g == 0) y[ymap.at(row)] = R::finish(acc, n, final_op);
}

template <typename R>
__device__ __forceinline__ typename R::acc_t block_reduce(typename R::acc_t acc) {
    using acc_t = typename R::acc_t;
    __shared__ acc_t sm[kBlock / kWave];
    acc = wave_reduce(acc, [](acc_t a, acc_t b) { return R::join(a, b); });
    const int w = threadIdx.x / kWave;
    if (lane_id() == 0) sm[w] = acc;
    __syncthreads();
    acc_t r = sm[0];
#pragma unroll
    for (int i = 1; i < kBlock / kWave; ++i) r = R::join(r, sm[i]);
    return r;
}

// Long rows: `parts` workgroups per row.  parts == 1 writes the result,
// otherwise each workgroup leaves one partial accumulator in `partial`.
// LAYOUT of a row: kRowStrided - any view of the reduced dimensions, element by element;
// kRowContig - one contiguous run; kRowRuns - contiguous runs of the innermost reduced dimension
// (statistics per channel of an NCHW tensor: 32 runs of 3136 elements a row), a group of lanes
// taking a run at a time with the vector loads of the contiguous case.
constexpr int kRowStrided = 0, kRowContig = 1, kRowRuns = 2;
template <typename R, int LAYOUT, bool STREAM = true>
__global__ __launch_bounds__(kBlock) void reduce_rows_block(
    const typename R::in_t* __restrict__ x, DimMap kept, DimMap red, int64_t n, int64_t parts,
    typename R::out_t* __restrict__ y, DimMap ymap, int final_op,
    typename R::acc_t* __restrict__ partial, typename R::param_t prm) {
    const int64_t row = blockIdx.x / parts;
    const int64_t part = blockIdx.x - row * parts;
    const typename R::in_t* p = x + kept.at(row);
    typename R::acc_t acc;
    if constexpr (LAYOUT == kRowContig) {
        acc = row_partial_contig<R>(p, n, threadIdx.x, kBlock, part, parts, prm);
    } else if constexpr (LAYOUT == kRowRuns) {
        acc = R::identity();
        const int last = red.rank - 1;
        const int64_t run = red.dims[last], runs = n / run;
        DimMap outer = red;
        outer.rank = last;
        // 64 lanes a run from 256 elements, 16 from 64, 4 below
        const int lanes = run >= 256 ? kWave : run >= 64 ? 16 : 4;
        const int64_t groups = kBlock / lanes;
        // long runs are handed out in pieces of 4096 elements: a few long runs a row (statistics per
        // channel of [64, 3, 224, 224]: 64 runs of 50176 elements, of [8, 16, 32, 64, 64]: 8 runs of
        // 131072) would otherwise leave most groups of most of the row's workgroups without work
        const int64_t piece = run > 8192 ? 4096 : run;
        const int64_t pieces = (run + piece - 1) / piece;
        for (int64_t it = part * groups + threadIdx.x / lanes; it < runs * pieces; it += parts * groups) {
            const int64_t r = it / pieces, at = (it - r * pieces) * piece;
            const int64_t len = run - at < piece ? run - at : piece;
            acc = R::join(acc, row_partial_contig<R, STREAM>(p + outer.at(r) + at, len, threadIdx.x % lanes, lanes, 0, 1, prm, r * run + at));
        }
    } else {
        acc = row_partial_strided<R>(p, red, n, threadIdx.x, kBlock, part, parts, prm);
    }
    acc = block_reduce<R>(acc);
    if (threadIdx.x == 0) {
        if (parts == 1) y[ymap.at(row)] = R::finish(acc, n, final_op);
        else partial[blockIdx.x] = acc;
    }
}

// Second stage for few rows: a workgroup per row, every thread's loads of partials in flight at
// once (one wave walking 2048 partials of a single row took 10 us, as long as a fiftieth of the
// first stage over 4 GB).
template <typename R>
__global__ __launch_bounds__(kBlock) void reduce_finalize_block(
    const typename R::acc_t* __restrict__ partial, int64_t n, int64_t parts,
    typename R::out_t* __restrict__ y, DimMap ymap, int final_op) {
    using acc_t = typename R::acc_t;
    const int64_t row = blockIdx.x;
    const acc_t* p = partial + row * parts;
    acc_t acc = R::identity();
    int64_t i = threadIdx.x;
    for (; i + 7 * kBlock < parts; i += 8 * kBlock) {
        acc_t v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = p[i + u * kBlock];
#pragma unroll
        for (int u = 0; u < 8; ++u) acc = R::join(acc, v[u]);
    }
    for (; i < parts; i += kBlock) acc = R::join(acc, p[i]);
    acc = block_reduce<R>(acc);
    if (threadIdx.x == 0) y[ymap.at(row)] = R::finish(acc, n, final_op);
}

// Second stage: one wave per row folds that row's `parts` partials.
template <typename R>
__global__ __launch_bounds__(kBlock) void reduce_finalize(
    const typename R::acc_t* __restrict__ partial, int64_t m, int64_t n, int64_t parts,
    typename R::out_t* __restrict__ y, DimMap ymap, int final_op) {
    using acc_t = typename R::acc_t;
    const int64_t row = static_cast<int64_t>(blockIdx.x) * (kBlock / kWave) + threadIdx.x / kWave;
    acc_t acc = R::identity();
    if (row < m)
        for (int64_t i = lane_id(); i < parts; i += kWave) acc = R::join(acc, partial[row * parts + i]);
    acc = wave_reduce(acc, [](acc_t a, acc_t b) { return R::join(a, b); });
    if (row < m && lane_id() == 0) y[ymap.at(row)] = R::finish(acc, n, final_op);
}

// Columns: kept axis of extent L is contiguous, lanes run along it; the four
// waves of a workgroup take reduced indices ty, ty+4, ... of slice `part`.
// A lane takes C neighbouring columns in one access (C = 2 for two-byte elements where every
// pair starts on a 4-byte boundary: with one such element per lane a wavefront's access is
// 128 bytes wide and the kernel runs at the element rate of fp32).
template <typename R, int C>
__global__ __launch_bounds__(kBlock) void reduce_cols(
    const typename R::in_t* __restrict__ x, DimMap outer, int64_t L, DimMap red, int64_t n,
    int64_t col_blocks, int64_t parts, typename R::out_t* __restrict__ y, DimMap ymap, int final_op,
    typename R::acc_t* __restrict__ partial, typename R::param_t prm) {
    using acc_t = typename R::acc_t;
    using in_t = typename R::in_t;
    using VecIn = Vec<in_t, C>;
    constexpr int TY = kBlock / kWave;
    __shared__ acc_t sm[TY][C][kWave];
    const int lx = threadIdx.x & (kWave - 1);
    const int ty = threadIdx.x / kWave;
    int64_t b = blockIdx.x;
    const int64_t part = b % parts;
    b /= parts;
    const int64_t cb = b % col_blocks;
    const int64_t o = b / col_blocks;
    const int64_t c = (cb * kWave + lx) * C;

    const int64_t per = (n + parts - 1) / parts;
    const int64_t lo = part * per;
    const int64_t hi = (lo + per < n) ? lo + per : n;

    acc_t acc[C];
#pragma unroll
    for (int k = 0; k < C; ++k) acc[k] = R::identity();
    if (c < L) {
        const in_t* __restrict__ p = x + outer.at(o) + c;
        auto fold = [&](const VecIn& v, int64_t j) __attribute__((always_inline)) {
#pragma unroll
            for (int k = 0; k < C; ++k) acc[k] = R::join(acc[k], R::map(v.v[k], j, prm));
        };
        if (red.rank == 1) {
            const int64_t s = red.strides[0];
            int64_t j = lo + ty;
            // row loads a lane keeps in flight: four when the launch fills the chip several times
            // over (measured: deeper queues then only slow the memory system down), eight when
            // few wavefronts have to cover the latency
            auto rows_at_once = [&](auto depth) __attribute__((always_inline)) {
                constexpr int U = decltype(depth)::value;
                for (; j + (U - 1) * TY < hi; j += U * TY) {
                    VecIn v[U];
#pragma unroll
                    for (int u = 0; u < U; ++u) v[u] = load_stream(reinterpret_cast<const VecIn*>(&p[(j + u * TY) * s]));
#pragma unroll
                    for (int u = 0; u < U; ++u) fold(v[u], j + u * TY);
                }
            };
            if (gridDim.x >= 1024) rows_at_once(std::integral_constant<int, 4>());
            else rows_at_once(std::integral_constant<int, 8>());
            for (; j < hi; j += TY) fold(load_stream(reinterpret_cast<const VecIn*>(&p[j * s])), j);
        } else {
            // several reduced dimensions that do not merge (batch and height of an NCHW tensor): eight loads in
            // flight; two dimensions of fewer than 2^32 elements are told apart with one 32-bit division
            const bool two = red.rank == 2 && n <= 0xffffffffLL;
            const uint32_t inner = static_cast<uint32_t>(red.dims[1]);
            auto where = [&](int64_t j) __attribute__((always_inline)) -> int64_t {
                if (two) {
                    const uint32_t q = static_cast<uint32_t>(j) / inner, r = static_cast<uint32_t>(j) - q * inner;
                    return static_cast<int64_t>(q) * red.strides[0] + static_cast<int64_t>(r) * red.strides[1];
                }
                return red.at(j);
            };
            constexpr int U = 8;
            int64_t j = lo + ty;
            for (; j + (U - 1) * TY < hi; j += U * TY) {
                VecIn v[U];
#pragma unroll
                for (int u = 0; u < U; ++u) v[u] = load_stream(reinterpret_cast<const VecIn*>(&p[where(j + u * TY)]));
#pragma unroll
                for (int u = 0; u < U; ++u) fold(v[u], j + u * TY);
            }
            for (; j < hi; j += TY) fold(*reinterpret_cast<const VecIn*>(&p[where(j)]), j);
        }
    }
#pragma unroll
    for (int k = 0; k < C; ++k) sm[ty][k][lx] = acc[k];
    __syncthreads();
    if (ty == 0 && c < L) {
#pragma unroll
        for (int k = 0; k < C; ++k) {
            acc_t all = acc[k];
#pragma unroll
            for (int i = 1; i < TY; ++i) all = R::join(all, sm[i][k][lx]);
            const int64_t row = o * L + c + k;
            if (parts == 1) y[ymap.at(row)] = R::finish(all, n, final_op);
            else partial[row * parts + part] = all;
        }
    }
}

// Columns beside a short reduced axis (up to 32 elements, one stride): a lane reduces a whole
// column, all its loads in flight at once, 256 columns a workgroup and no barrier (reduce_cols
// gives such an axis to four wavefronts an element or two each: fp32 [64, 3, 224, 224] over
// axis 1 54 us, [8, 21, 512, 512] 60 us).  C neighbouring columns a lane, as above.
template <typename R, int N, int C>
__global__ __launch_bounds__(kBlock) void reduce_cols_thread(
    const typename R::in_t* __restrict__ x, DimMap outer, int64_t L, int64_t stride, int n, int64_t col_blocks,
    typename R::out_t* __restrict__ y, DimMap ymap, int final_op, typename R::param_t prm) {
    using VecIn = Vec<typename R::in_t, C>;
    const int64_t cb = blockIdx.x % col_blocks, o = blockIdx.x / col_blocks;
    const int64_t c = (cb * kBlock + threadIdx.x) * C;
    if (c >= L) return;
    const typename R::in_t* __restrict__ p = x + outer.at(o) + c;
    VecIn v[N];
#pragma unroll
    for (int j = 0; j < N; ++j) v[j] = load_stream(reinterpret_cast<const VecIn*>(&p[(j < n ? j : 0) * stride]));
#pragma unroll
    for (int k = 0; k < C; ++k) {
        typename R::acc_t acc = R::identity();
#pragma unroll
        for (int j = 0; j < N; ++j)
            if (j < n) acc = R::join(acc, R::map(v[j].v[k], j, prm));
        y[ymap.at(o * L + c + k)] = R::finish(acc, n, final_op);
    }
}

// --------------------------------------------------------------------------
// The classification head in one read: per row of logits its sum, maximum, first arg-maximum,
// log-sum-exp and `limit` best entries, each exactly what the separate reduce / arg_reduce /
// top_k call gives (the same reducers; the same order among the best: larger value first,
// -0.0 and +0.0 one value, NaNs by their bit pattern, lower index first among equals).
// One wavefront holds one row (element i * 64 + lane is item i of the lane).
template <int ITEMS>
__global__ __launch_bounds__(kWave) void logits_head_rows(
    const float* __restrict__ x, int64_t row_stride, int64_t m, int64_t n, float* __restrict__ sum_out,
    float* __restrict__ max_out, int32_t* __restrict__ argmax_out, float* __restrict__ lse_out, int limit,
    float* __restrict__ best_out, int32_t* __restrict__ best_idx) {
    using Sum = ValueReducer<float, kAdd, kMapId>;
    using Max = ValueReducer<float, kMax, kMapId>;
    using Lse = ValueReducer<float, kAdd, kMapExp>;
    using Arg = ArgReducer<float, true, int32_t>;
    const int64_t row = blockIdx.x;
    const int lane = lane_id();
    const float* xr = x + row * row_stride;
    const uint32_t n32 = static_cast<uint32_t>(n);
    float v[ITEMS];
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        const uint32_t e = static_cast<uint32_t>(i * kWave + lane);
        v[i] = xr[e < n32 ? e : 0u];                         // (past the row: its first element again, never used)
    }
    Sum::acc_t a_sum = Sum::identity();
    Max::acc_t a_max = Max::identity();
    Lse::acc_t a_lse = Lse::identity();
    Arg::acc_t a_arg = Arg::identity();
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        const uint32_t e = static_cast<uint32_t>(i * kWave + lane);
        if (e < n32) {
            a_sum = Sum::join(a_sum, Sum::map(v[i], e, 0));
            a_max = Max::join(a_max, Max::map(v[i], e, 0));
            if (lse_out) a_lse = Lse::join(a_lse, Lse::map(v[i], e, 0));
            a_arg = Arg::join(a_arg, Arg::map(v[i], e, 0));
        }
    }
    a_sum = wave_reduce(a_sum, [](Sum::acc_t a, Sum::acc_t b) { return Sum::join(a, b); });
    a_max = wave_reduce(a_max, [](Max::acc_t a, Max::acc_t b) { return Max::join(a, b); });
    if (lse_out) a_lse = wave_reduce(a_lse, [](Lse::acc_t a, Lse::acc_t b) { return Lse::join(a, b); });
    a_arg = wave_reduce(a_arg, [](Arg::acc_t a, Arg::acc_t b) { return Arg::join(a, b); });
    if (lane == 0) {
        if (sum_out) sum_out[row] = Sum::finish(a_sum, n, kFinalId);
        if (max_out) max_out[row] = Max::finish(a_max, n, kFinalId);
        if (lse_out) lse_out[row] = Lse::finish(a_lse, n, kFinalLog);
        if (argmax_out) argmax_out[row] = Arg::finish(a_arg, n, kFinalId);
    }
    if (limit <= 0) return;

    // ---- the best `limit` entries: `limit` times the best entry that comes after the one taken
    // last, entries ordered by image (larger first), then by lower index
    uint32_t ord[ITEMS];
#pragma unroll
    for (int i = 0; i < ITEMS; ++i) {
        uint32_t bits = bit_cast<uint32_t>(v[i]);
        if ((bits << 1) == 0u) bits = 0u;                    // -0.0 and +0.0 are one value
        ord[i] = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
    }
    struct Entry {
        uint32_t o, x;
    };
    auto beats = [](uint32_t oa, uint32_t xa, uint32_t ob, uint32_t xb) { return oa > ob || (oa == ob && xa < xb); };
    Entry last = {0xffffffffu, 0u};
    for (int j = 0; j < limit; ++j) {
        Entry mine = {0u, 0xffffffffu};
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
            const uint32_t e = static_cast<uint32_t>(i * kWave + lane);
            const bool after = j == 0 || beats(last.o, last.x, ord[i], e);       // not taken yet
            if (e < n32 && after && beats(ord[i], e, mine.o, mine.x)) mine = {ord[i], e};
        }
        const Entry top = wave_reduce(mine, [beats](Entry a, Entry b) { return beats(b.o, b.x, a.o, a.x) ? b : a; });
        if (lane == 0) {
            if (best_out) best_out[row * limit + j] = xr[top.x];                 // the element itself (a zero keeps its sign)
            if (best_idx) best_idx[row * limit + j] = static_cast<int32_t>(top.x);
        }
        last = top;
    }
}

// --------------------------------------------------------------------------
// Host-side planning.

struct ReducePlan {
    DimMap kept, red, ymap;
    int64_t m, n;
};

int next_pow2_log(int64_t v) {
    int l = 0;
    while ((int64_t(1) << l) < v) ++l;
    return l;
}

// Workgroups per row for the long-row kernel; a function of (m, n) only so the
// scratch query and the launch agree.
int64_t row_parts(int64_t m, int64_t n) {
    if (m >= 1024) return 1;
    int64_t want = ceil_div(2048, m);
    int64_t cap = n / 16384;
    if (cap < 1) cap = 1;
    return want < cap ? want : cap;
}

#ifndef DLFX_REDUCE_COLS_MIN_RUN
#define DLFX_REDUCE_COLS_MIN_RUN 48
#endif
#ifndef DLFX_REDUCE_COLS_SHORT_AXIS
#define DLFX_REDUCE_COLS_SHORT_AXIS 8
#endif
#ifndef DLFX_REDUCE_SHORT_RUNS
#define DLFX_REDUCE_SHORT_RUNS 1024
#endif
int64_t col_parts(int64_t base_blocks, int64_t n) {
    if (base_blocks >= 1024) return 1;
    int64_t want = ceil_div(2048, base_blocks);
    int64_t cap = n / 64;
    if (cap < 1) cap = 1;
    return want < cap ? want : cap;
}

size_t partial_bound_bytes(int64_t m) {
    if (m >= 65536) return 0;
    return static_cast<size_t>(m + 133120) * 16;
}

template <typename R>
int launch_reduce(hipStream_t stream, const ReducePlan& pl, const typename R::in_t* x,
                  typename R::out_t* y, int final_op, void* scratch, size_t scratch_bytes,
                  typename R::param_t prm = typename R::param_t()) {
    using acc_t = typename R::acc_t;
    using T = typename R::in_t;
    const int64_t m = pl.m, n = pl.n;
    acc_t* partial = static_cast<acc_t*>(scratch);

    const bool contig = pl.red.rank == 0 || (pl.red.rank == 1 && pl.red.strides[0] == 1);
    const bool cols = !contig && pl.kept.rank >= 1 && pl.kept.strides[pl.kept.rank - 1] == 1 &&
                      pl.kept.dims[pl.kept.rank - 1] >= 16 &&
                      // (a short run of columns beside a short reduced axis: a lane a row keeps the lanes busy, where a
                      // block of 64 columns a workgroup leaves most of them idle - fp32 [4096, 50, 3, 17] over axis 2: 78 us)
                      (pl.kept.dims[pl.kept.rank - 1] >= DLFX_REDUCE_COLS_MIN_RUN || n > DLFX_REDUCE_COLS_SHORT_AXIS);

    if (cols) {
        DimMap outer = pl.kept;
        const int64_t L = outer.dims[outer.rank - 1];
        outer.rank -= 1;
        outer.dims[outer.rank] = 1;
        outer.strides[outer.rank] = 0;
        // two-byte elements: two neighbouring columns a lane where every pair starts on a 4-byte boundary
        // (from 128 columns on: fewer leave half the lanes of the one block of columns without work)
        bool pairs = sizeof(T) == 2 && !std::is_class<T>::value && L % 2 == 0 && L >= 128 && reinterpret_cast<uintptr_t>(x) % 4 == 0;
        for (int i = 0; pairs && i < outer.rank; ++i) pairs = outer.strides[i] % 2 == 0;
        for (int i = 0; pairs && i < pl.red.rank; ++i) pairs = pl.red.strides[i] % 2 == 0;
        auto with_cols = [&](auto&& launch) {
            if constexpr (sizeof(T) == 2 && !std::is_class<T>::value) {
                if (pairs) { launch(std::integral_constant<int, 2>()); return; }
            }
            launch(std::integral_constant<int, 1>());
        };
        const int per_lane = pairs ? 2 : 1;
        if (n <= 32 && pl.red.rank == 1 && m >= 4096) {
            const int64_t wide_blocks = ceil_div(L, static_cast<int64_t>(kBlock) * per_lane);
            const int64_t blocks = (m / L) * wide_blocks;
            if (blocks > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
            const dim3 grid(static_cast<unsigned>(blocks)), block(kBlock);
            with_cols([&](auto cols_per_lane) {
                constexpr int C = decltype(cols_per_lane)::value;
#define DLFX_REDUCE_THREAD(N) reduce_cols_thread<R, N, C><<<grid, block, 0, stream>>>(x, outer, L, pl.red.strides[0], static_cast<int>(n), wide_blocks, y, pl.ymap, final_op, prm)
                if (n <= 4) DLFX_REDUCE_THREAD(4);
                else if (n <= 8) DLFX_REDUCE_THREAD(8);
                else if (n <= 16) DLFX_REDUCE_THREAD(16);
                else DLFX_REDUCE_THREAD(32);
#undef DLFX_REDUCE_THREAD
            });
            DLFX_CHECK_LAUNCH();
            return DLFX_OK;
        }
        const int64_t col_blocks = ceil_div(L, static_cast<int64_t>(kWave) * per_lane);
        const int64_t base_blocks = (m / L) * col_blocks;
        const int64_t parts = col_parts(base_blocks * per_lane, n);      // (as many slices as one column a lane would get: what the scratch query allows for)
        if (base_blocks * parts > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
        if (parts > 1 && scratch_bytes < static_cast<size_t>(m * parts) * sizeof(acc_t))
            return DLFX_ERR_SCRATCH_TOO_SMALL;
        with_cols([&](auto cols_per_lane) {
            reduce_cols<R, decltype(cols_per_lane)::value><<<dim3(static_cast<unsigned>(base_blocks * parts)), dim3(kBlock), 0, stream>>>(
                x, outer, L, pl.red, n, col_blocks, parts, y, pl.ymap, final_op, partial, prm);
        });
        DLFX_CHECK_LAUNCH();
        if (parts > 1) {
            reduce_finalize<R><<<dim3(static_cast<unsigned>(ceil_div(m, kBlock / kWave))), dim3(kBlock), 0, stream>>>(
                partial, m, n, parts, y, pl.ymap, final_op);
            DLFX_CHECK_LAUNCH();
        }
        return DLFX_OK;
    }

    const int64_t short_limit = 8192;
    // rows made of contiguous runs (the innermost reduced dimension has stride 1 and at least 16 elements)
    const bool runs = !contig && pl.red.rank >= 2 && pl.red.strides[pl.red.rank - 1] == 1 && pl.red.dims[pl.red.rank - 1] >= 16;
    // (short rows of runs take the long rows' kernel, a workgroup a row, from 1024 elements: element by element
    // with a division per element - fp32 [32, 512, 56, 56] over {0, 3} - they took 76 us)
    if (n <= short_limit && !(runs && n >= DLFX_REDUCE_SHORT_RUNS)) {
        const int per_lane = contig ? vec_width<T>() * 4 : 8;
        int log2g = next_pow2_log(ceil_div(n, per_lane));
        if (log2g > 6) log2g = 6;
        const int64_t blocks = ceil_div(m, kBlock >> log2g);
        if (blocks > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
        const int64_t row_bytes = n * static_cast<int64_t>(sizeof(T));
        if (contig && row_bytes >= 512 && row_bytes % 128 == 0)
            reduce_rows_group<R, true, true><<<dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0, stream>>>(
                x, pl.kept, pl.red, m, n, log2g, y, pl.ymap, final_op, prm);
        else if (contig)
            reduce_rows_group<R, true, false><<<dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0, stream>>>(
                x, pl.kept, pl.red, m, n, log2g, y, pl.ymap, final_op, prm);
        else
            reduce_rows_group<R, false, true><<<dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0, stream>>>(
                x, pl.kept, pl.red, m, n, log2g, y, pl.ymap, final_op, prm);
        DLFX_CHECK_LAUNCH();
        return DLFX_OK;
    }

    const int64_t parts = row_parts(m, n);
    if (m * parts > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
    if (parts > 1 && scratch_bytes < static_cast<size_t>(m * parts) * sizeof(acc_t))
        return DLFX_ERR_SCRATCH_TOO_SMALL;
    if (contig)
        reduce_rows_block<R, kRowContig><<<dim3(static_cast<unsigned>(m * parts)), dim3(kBlock), 0, stream>>>(
            x, pl.kept, pl.red, n, parts, y, pl.ymap, final_op, partial, prm);
    else if (runs && (pl.red.dims[pl.red.rank - 1] * static_cast<int64_t>(sizeof(T)) < 512 || pl.red.dims[pl.red.rank - 1] * static_cast<int64_t>(sizeof(T)) % 128 != 0))
        // (runs that are not whole cache lines: without the non-temporal hint, as in reduce_rows_group)
        reduce_rows_block<R, kRowRuns, false><<<dim3(static_cast<unsigned>(m * parts)), dim3(kBlock), 0, stream>>>(
            x, pl.kept, pl.red, n, parts, y, pl.ymap, final_op, partial, prm);
    else if (runs)
        reduce_rows_block<R, kRowRuns><<<dim3(static_cast<unsigned>(m * parts)), dim3(kBlock), 0, stream>>>(
            x, pl.kept, pl.red, n, parts, y, pl.ymap, final_op, partial, prm);
    else
        reduce_rows_block<R, kRowStrided><<<dim3(static_cast<unsigned>(m * parts)), dim3(kBlock), 0, stream>>>(
            x, pl.kept, pl.red, n, parts, y, pl.ymap, final_op, partial, prm);
    DLFX_CHECK_LAUNCH();
    if (parts > 1) {
        if (m <= 64 && parts >= 256)
            reduce_finalize_block<R><<<dim3(static_cast<unsigned>(m)), dim3(kBlock), 0, stream>>>(partial, n, parts, y, pl.ymap, final_op);
        else
            reduce_finalize<R><<<dim3(static_cast<unsigned>(ceil_div(m, kBlock / kWave))), dim3(kBlock), 0, stream>>>(
                partial, m, n, parts, y, pl.ymap, final_op);
        DLFX_CHECK_LAUNCH();
    }
    return DLFX_OK;
}

struct ReduceOp {
    const char* name;
    int join, map, final_op;
    bool float_only;
};

const ReduceOp kReduceOps[] = {
    {"reduce_sum", kAdd, kMapId, kFinalId, false},
    {"reduce_mean", kAdd, kMapId, kFinalMean, false},
    {"reduce_max", kMax, kMapId, kFinalId, false},
    {"reduce_min", kMin, kMapId, kFinalId, false},
    {"reduce_log_sum_exp", kAdd, kMapExp, kFinalLog, true},
    {"reduce_sum_exp", kAdd, kMapExp, kFinalId, true},
    {"reduce_log_sum", kAdd, kMapId, kFinalLog, true},
    {"reduce_prod", kMul, kMapId, kFinalId, false},
    {"reduce_asum", kAdd, kMapAbs, kFinalId, false},
    {"reduce_sum_square", kAdd, kMapSquare, kFinalId, false},
    {"reduce_nrm2", kAdd, kMapNorm, kFinalSqrt, true},
    {"reduce_amax", kMax, kMapAbs, kFinalId, false},
    {"reduce_amin", kMin, kMapAbs, kFinalId, false},
};

template <typename T>
int launch_reduce_typed(hipStream_t stream, const ReduceOp& op, const ReducePlan& pl, const T* x, T* y,
                        void* scratch, size_t scratch_bytes) {
#define DLFX_CASE(J, M)                                                                       \
    if (op.join == J && op.map == M)                                                          \
        return launch_reduce<ValueReducer<T, J, M>>(stream, pl, x, y, op.final_op, scratch, scratch_bytes);
    DLFX_CASE(kAdd, kMapId)
    DLFX_CASE(kAdd, kMapAbs)
    DLFX_CASE(kAdd, kMapSquare)
    if (op.join == kAdd && op.map == kMapNorm)           // |x|^2 of a real is its square
        return launch_reduce<ValueReducer<T, kAdd, kMapSquare>>(stream, pl, x, y, op.final_op, scratch, scratch_bytes);
    DLFX_CASE(kMul, kMapId)
    DLFX_CASE(kMax, kMapId)
    DLFX_CASE(kMin, kMapId)
    DLFX_CASE(kMax, kMapAbs)
    DLFX_CASE(kMin, kMapAbs)
    if constexpr (!std::is_integral<T>::value) {
        DLFX_CASE(kAdd, kMapExp)
    }
#undef DLFX_CASE
    return DLFX_ERR_UNKNOWN_OP;
}

template <typename F>
int launch_reduce_complex(hipStream_t stream, const ReduceOp& op, const ReducePlan& pl, const Cx<F>* x, Cx<F>* y,
                          void* scratch, size_t scratch_bytes) {
#define DLFX_CASE(J, M)                                                                       \
    if (op.join == J && op.map == M)                                                          \
        return launch_reduce<ComplexReducer<F, J, M>>(stream, pl, x, y, op.final_op, scratch, scratch_bytes);
    DLFX_CASE(kAdd, kMapId)
    DLFX_CASE(kAdd, kMapAbs)
    DLFX_CASE(kAdd, kMapSquare)
    DLFX_CASE(kAdd, kMapNorm)
    DLFX_CASE(kAdd, kMapExp)
    DLFX_CASE(kMul, kMapId)
#undef DLFX_CASE
    return DLFX_ERR_UNSUPPORTED_DTYPE;      // max / min / amax / amin: complex numbers are not ordered
}

}  // namespace
}  // namespace dlfx

using namespace dlfx;

extern "C" size_t dlfx_reduce_scratch_bytes(int dtype, int64_t m, int64_t n) {
    (void)dtype;
    (void)n;
    if (m <= 0) return 0;
    return partial_bound_bytes(m);
}

namespace {

int reduce_entry(dlfx_stream_t stream, const char* name, int dtype, int64_t m, int64_t n,
                 int x_rank, const int64_t* x_dims, const int64_t* x_strides,
                 const void* x, int64_t x_offset,
                 int y_rank, const int64_t* y_dims, const int64_t* y_strides,
                 void* y, int64_t y_offset, void* scratch, size_t scratch_bytes) {
    if (!name || !x || !y || m <= 0 || n <= 0) return DLFX_ERR_INVALID_ARGUMENT;
    if (!view_ok(x_rank, x_dims, x_strides) || !view_ok(y_rank, y_dims, y_strides))
        return DLFX_ERR_INVALID_ARGUMENT;
    if (view_size(x_rank, x_dims) != m * n || view_size(y_rank, y_dims) != m) return DLFX_ERR_INVALID_ARGUMENT;
    const ReduceOp* op = nullptr;
    for (const auto& o : kReduceOps)
        if (!std::strcmp(o.name, name)) op = &o;
    if (!op) return DLFX_ERR_UNKNOWN_OP;
    if (op->float_only && (dtype == DLFX_I32 || dtype == DLFX_I64)) return DLFX_ERR_UNSUPPORTED_DTYPE;
    if (dtype == DLFX_I16 || dtype == DLFX_BOOL) return DLFX_ERR_UNSUPPORTED_DTYPE;        // as the reference's instantiations

    // the reduced extents are the trailing dimensions whose product is n
    int split = x_rank;
    int64_t prod = 1;
    while (split > 0 && prod < n) prod *= x_dims[--split];
    if (prod != n) return DLFX_ERR_INVALID_ARGUMENT;

    ReducePlan pl;
    pl.m = m;
    pl.n = n;
    if (!make_dim_map(x_dims, x_strides, 0, split, &pl.kept) ||
        !make_dim_map(x_dims, x_strides, split, x_rank, &pl.red) ||
        !make_dim_map(y_dims, y_strides, 0, y_rank, &pl.ymap))
        return DLFX_ERR_RANK;

    if (dtype == DLFX_C64)
        return launch_reduce_complex<float>(static_cast<hipStream_t>(stream), *op, pl, static_cast<const Cx<float>*>(x) + x_offset,
                                            static_cast<Cx<float>*>(y) + y_offset, scratch, scratch_bytes);
    if (dtype == DLFX_C128)
        return launch_reduce_complex<double>(static_cast<hipStream_t>(stream), *op, pl, static_cast<const Cx<double>*>(x) + x_offset,
                                             static_cast<Cx<double>*>(y) + y_offset, scratch, scratch_bytes);
    return dispatch_dtype_half(dtype, [&](auto tag) {
        using T = decltype(tag);
        return launch_reduce_typed<T>(static_cast<hipStream_t>(stream), *op, pl,
                                      static_cast<const T*>(x) + x_offset, static_cast<T*>(y) + y_offset,
                                      scratch, scratch_bytes);
    });
}

// Partial accumulators of dlfx_reduce_static: one copy of this array lives on every device the
// library runs on, from the load of the code object to the end of the process.  The size is
// partial_bound_bytes() of the largest row count that needs partials (65535), rounded up to 256.
constexpr size_t kStaticScratchBytes = 3178496;
static_assert(kStaticScratchBytes == DLFX_REDUCE_STATIC_SCRATCH_BYTES, "header and array disagree");
static_assert(kStaticScratchBytes % 256 == 0 && kStaticScratchBytes >= (65535 + 133120) * 16, "array too small");
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// The array's address on each device.  In host code the name `scratch` is only a handle for
// hipGetSymbolAddress: every device has its own copy at its own address, looked up once with
// that device current and kept here; kernels are only ever given these pointers.
constexpr int kMaxDevices = 64;
std::atomic<void*> g_static_scratch[kMaxDevices];

int static_scratch_of_current_device(hipStream_t stream, void** out) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return record_hip_error(e);
    if (dev < 0 || dev >= kMaxDevices) return DLFX_ERR_INVALID_ARGUMENT;
    void* p = g_static_scratch[dev].load(std::memory_order_acquire);
    if (!p) {
        // the lookup may load the code object: not something to do while a graph is being recorded
        if (stream_is_capturing(stream)) return DLFX_ERR_CAPTURING;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return record_hip_error(e);
        if (!p) return record_hip_error(hipErrorInvalidSymbol);
        g_static_scratch[dev].store(p, std::memory_order_release);   // racing threads store the same address
    }
    *out = p;
    return DLFX_OK;
}

}  // namespace

extern "C" int dlfx_reduce(dlfx_stream_t stream, const char* name, int dtype, int64_t m, int64_t n,
                           int x_rank, const int64_t* x_dims, const int64_t* x_strides,
                           const void* x, int64_t x_offset,
                           int y_rank, const int64_t* y_dims, const int64_t* y_strides,
                           void* y, int64_t y_offset, void* scratch_arg, size_t scratch_bytes) {
    return reduce_entry(stream, name, dtype, m, n, x_rank, x_dims, x_strides, x, x_offset,
                        y_rank, y_dims, y_strides, y, y_offset, scratch_arg, scratch_bytes);
}

extern "C" int dlfx_reduce_static(dlfx_stream_t stream, const char* name, int dtype, int64_t m, int64_t n,
                                  int x_rank, const int64_t* x_dims, const int64_t* x_strides,
                                  const void* x, int64_t x_offset,
                                  int y_rank, const int64_t* y_dims, const int64_t* y_strides,
                                  void* y, int64_t y_offset) {
    if (m <= 0 || n <= 0) return DLFX_ERR_INVALID_ARGUMENT;
    // Same bound as the caller of dlfx_reduce would have to provide; beyond the array: refuse.
    if (partial_bound_bytes(m) > kStaticScratchBytes) return DLFX_ERR_TOO_LARGE;
    void* ptr = nullptr;
    const int st = static_scratch_of_current_device(static_cast<hipStream_t>(stream), &ptr);
    if (st != DLFX_OK) return st;
    // Partials are written by the first kernel before the second reads them: nothing to clear.
    return reduce_entry(stream, name, dtype, m, n, x_rank, x_dims, x_strides, x, x_offset,
                        y_rank, y_dims, y_strides, y, y_offset, ptr, kStaticScratchBytes);
}

extern "C" size_t dlfx_arg_reduce_scratch_bytes(int dtype, int64_t n_rows, int64_t k) {
    (void)dtype;
    (void)k;
    if (n_rows <= 0) return 0;
    return partial_bound_bytes(n_rows);
}

extern "C" int dlfx_arg_reduce(dlfx_stream_t stream, const char* name, int dtype, int index_dtype,
                               int64_t n_rows, int64_t k,
                               int x_rank, const int64_t* x_dims, const int64_t* x_strides,
                               const void* x, int64_t x_offset,
                               int y_rank, const int64_t* y_dims, const int64_t* y_strides,
                               void* y, int64_t y_offset, void* scratch, size_t scratch_bytes) {
    if (!name || !x || !y || n_rows <= 0 || k <= 0) return DLFX_ERR_INVALID_ARGUMENT;
    if (!view_ok(x_rank, x_dims, x_strides) || !view_ok(y_rank, y_dims, y_strides))
        return DLFX_ERR_INVALID_ARGUMENT;
    if (x_rank < 1 || x_dims[x_rank - 1] != k) return DLFX_ERR_INVALID_ARGUMENT;
    if (view_size(x_rank, x_dims) != n_rows * k || view_size(y_rank, y_dims) != n_rows)
        return DLFX_ERR_INVALID_ARGUMENT;
    if (k > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
    bool want_max;
    if (!std::strcmp(name, "argmax")) want_max = true;
    else if (!std::strcmp(name, "argmin")) want_max = false;
    else return DLFX_ERR_UNKNOWN_OP;
    if (index_dtype != DLFX_I32 && index_dtype != DLFX_I64) return DLFX_ERR_UNSUPPORTED_DTYPE;
    if (dtype == DLFX_BOOL) return DLFX_ERR_UNSUPPORTED_DTYPE;

    ReducePlan pl;
    pl.m = n_rows;
    pl.n = k;
    if (!make_dim_map(x_dims, x_strides, 0, x_rank - 1, &pl.kept) ||
        !make_dim_map(x_dims, x_strides, x_rank - 1, x_rank, &pl.red) ||
        !make_dim_map(y_dims, y_strides, 0, y_rank, &pl.ymap))
        return DLFX_ERR_RANK;

    hipStream_t s = static_cast<hipStream_t>(stream);
    return dispatch_dtype16(dtype, [&](auto tag) {
        using T = decltype(tag);
        const T* xp = static_cast<const T*>(x) + x_offset;
        if (index_dtype == DLFX_I32) {
            int32_t* yp = static_cast<int32_t*>(y) + y_offset;
            if (want_max) return launch_reduce<ArgReducer<T, true, int32_t>>(s, pl, xp, yp, 0, scratch, scratch_bytes);
            return launch_reduce<ArgReducer<T, false, int32_t>>(s, pl, xp, yp, 0, scratch, scratch_bytes);
        }
        int64_t* yp = static_cast<int64_t*>(y) + y_offset;
        if (want_max) return launch_reduce<ArgReducer<T, true, int64_t>>(s, pl, xp, yp, 0, scratch, scratch_bytes);
        return launch_reduce<ArgReducer<T, false, int64_t>>(s, pl, xp, yp, 0, scratch, scratch_bytes);
    });
}

extern "C" size_t dlfx_count_scratch_bytes(int dtype, int64_t m, int64_t n) {
    (void)dtype;
    (void)n;
    if (m <= 0) return 0;
    return partial_bound_bytes(m);
}

extern "C" int dlfx_count(dlfx_stream_t stream, int dtype, int64_t m, int64_t n, const void* value,
                          int x_rank, const int64_t* x_dims, const int64_t* x_strides,
                          const void* x, int64_t x_offset,
                          int y_rank, const int64_t* y_dims, const int64_t* y_strides,
                          int32_t* y, int64_t y_offset, void* scratch, size_t scratch_bytes) {
    if (!value || !x || !y || m <= 0 || n <= 0) return DLFX_ERR_INVALID_ARGUMENT;
    if (!view_ok(x_rank, x_dims, x_strides) || !view_ok(y_rank, y_dims, y_strides))
        return DLFX_ERR_INVALID_ARGUMENT;
    if (view_size(x_rank, x_dims) != m * n || view_size(y_rank, y_dims) != m) return DLFX_ERR_INVALID_ARGUMENT;
    if (n > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;       // counts are 32-bit, as in the reference
    if (dtype == DLFX_I16 || dtype == DLFX_BOOL) return DLFX_ERR_UNSUPPORTED_DTYPE;

    int split = x_rank;
    int64_t prod = 1;
    while (split > 0 && prod < n) prod *= x_dims[--split];
    if (prod != n) return DLFX_ERR_INVALID_ARGUMENT;

    ReducePlan pl;
    pl.m = m;
    pl.n = n;
    if (!make_dim_map(x_dims, x_strides, 0, split, &pl.kept) ||
        !make_dim_map(x_dims, x_strides, split, x_rank, &pl.red) ||
        !make_dim_map(y_dims, y_strides, 0, y_rank, &pl.ymap))
        return DLFX_ERR_RANK;

    auto count_as = [&](auto tag) {
        using T = decltype(tag);
        T v;
        std::memcpy(&v, value, sizeof(T));
        return launch_reduce<CountReducer<T>>(static_cast<hipStream_t>(stream), pl,
                                              static_cast<const T*>(x) + x_offset, y + y_offset, kFinalId,
                                              scratch, scratch_bytes, v);
    };
    if (dtype == DLFX_C64) return count_as(Cx<float>());
    if (dtype == DLFX_C128) return count_as(Cx<double>());
    return dispatch_dtype_half(dtype, count_as);
}

extern "C" int dlfx_logits_head(dlfx_stream_t stream, int dtype, int64_t m, int64_t n,
                                const void* x, int64_t x_offset, int64_t row_stride,
                                void* sum, void* max, int32_t* argmax, void* log_sum_exp,
                                int64_t k, void* best_values, int32_t* best_indices) {
    if (!x || m <= 0 || n <= 0 || k < 0 || row_stride < n) return DLFX_ERR_INVALID_ARGUMENT;
    if (dtype != DLFX_F32) return DLFX_ERR_UNSUPPORTED_DTYPE;
    if (n > DLFX_LOGITS_HEAD_MAX_N || k > DLFX_LOGITS_HEAD_MAX_K || k > n || m > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
    if (k > 0 && !best_values && !best_indices) return DLFX_ERR_INVALID_ARGUMENT;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const float* xp = static_cast<const float*>(x) + x_offset;
    const dim3 grid(static_cast<unsigned>(m)), block(kWave);
    auto launch = [&](auto items) {
        constexpr int ITEMS = decltype(items)::value;
        logits_head_rows<ITEMS><<<grid, block, 0, s>>>(xp, row_stride, m, n, static_cast<float*>(sum), static_cast<float*>(max), argmax,
                                                        static_cast<float*>(log_sum_exp), static_cast<int>(k),
                                                        static_cast<float*>(best_values), best_indices);
    };
    if (n <= 4 * kWave) launch(std::integral_constant<int, 4>());
    else if (n <= 8 * kWave) launch(std::integral_constant<int, 8>());
    else if (n <= 16 * kWave) launch(std::integral_constant<int, 16>());
    else launch(std::integral_constant<int, 32>());
    DLFX_CHECK_LAUNCH();
    return DLFX_OK;
}
