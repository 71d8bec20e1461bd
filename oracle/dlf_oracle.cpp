// TEST INFRASTRUCTURE ONLY -- CPU oracle for the axis primitives.
//
// This file restates, on the host, what the dlf CPU Tensor path computes for
// reduce / arg_reduce / scan / sort / argsort / top_k over strided views, plus
// fp64 evaluators that tolerance checks compare against.  Nothing in the
// shipped library may link, load or call it: only the test-suite, the smoke
// check and the benchmark's cpu_baseline leg do.
//
// Every entry point takes the same view description the GPU boundary takes:
// rank, extents, strides (signed, in elements) and an element offset.
//
// Reference lines each function follows (paths relative to the dlf tree):
//   reduce        dlf/include/tensor/reduce_detail.h:40-68, utility.h:143-150,
//                 reducers dlf/include/tensor/xfn.h:661-805
//   arg_reduce    dlf/include/tensor/reduce_detail.h:107-132
//   scan          dlf/include/tensor/reduce_detail.h:171-242
//   sort          dlf/include/tensor/reorder_detail.h:511-615
//   argsort       dlf/include/tensor/reorder_detail.h:681-772 (serial leaves
//                 and serial merge, which are stable)
//   top_k (heap)  dlf/include/tensor/reorder_detail.h:969-1060
//   count         dlf/include/tensor/reduce.h:151-158
//   scan_nonzero, gather_indices   dlf/include/tensor/reduce.h:381-418
//   merge         dlf/include/tensor/reorder_detail.h:346-368
//   softmax, logsoftmax, hardmax   dlf/include/tensor/dnn_detail.h:266-350
//   complex elements: the same reduce / scan / count templates instantiated with
//                 std::complex<float|double> (functors dlf/include/tensor/xfn.h:73-170)
//
// Pinning status (what independent evidence fixes each function):
//   reduce, arg_reduce, scan, sort, top_k values+indices on tie-free input:
//       literal vectors held by the reference's own tests (tests/golden/*.json)
//       and numpy library routines on random input.
//   argsort / top_k tie order: NOT pinned by any reference test (the
//       reference concedes the indices may differ).  The rule used here is
//       "lowest index first" (std::stable_sort); it is pinned against numpy's
//       stable argsort, not against the reference.  parity unpinned w.r.t. the
//       reference for tie order only.
//   count, nonzero, merge, softmax family: literal vectors of the reference's tests
//       (tests/golden/reference_vectors.json) and numpy / scipy closed forms.
//   complex reduce / scan / count: the reference's literal nrm2 vector
//       (dlf/test/UniformTest.cpp:2060-2063) and numpy complex128 closed forms; the
//       reference holds no other complex vector for this path.
//   16-bit elements never reach this file: the Python wrapper widens them exactly to the
//       32-bit types (oracle.py), which numpy on the 16-bit arrays pins.
//   fp32 sum/scan rounding: the reference's association depends on TBB's
//       run-time range splitting; the restatement uses one valid schedule
//       (recursive halving down to 1024-element leaves) and parity is judged
//       against the fp64 evaluators with a stated tolerance.

#include <algorithm>
#include <cmath>
#include <complex>
#include <cstdint>
#include <cstring>
#include <functional>
#include <limits>
#include <numeric>
#include <string>
#include <utility>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

constexpr int64_t kGrain = 1024;   // utility.h:28-34 (release build)

struct View {
    int rank;
    const int64_t* dims;
    const int64_t* strides;
    int64_t offset;
    bool contiguous;   // row-major dense: the reference then walks a raw pointer (map.h:5-41)

    View(int r, const int64_t* d, const int64_t* s, int64_t o) : rank(r), dims(d), strides(s), offset(o) {
        contiguous = true;
        int64_t size = 1;
        for (int i = rank - 1; i >= 0; --i) {
            if (dims[i] != 1 && strides[i] != size) contiguous = false;
            size *= dims[i];
        }
    }

    // Shape::linear_offset: row-major unravel of a flat index, then dot with strides.
    int64_t at(int64_t flat) const {
        if (contiguous) return offset + flat;
        int64_t off = offset;
        for (int i = rank - 1; i >= 0; --i) {
            int64_t d = dims[i];
            off += (flat % d) * strides[i];
            flat /= d;
        }
        return off;
    }
    int64_t last_extent() const { return rank ? dims[rank - 1] : 1; }
    int64_t last_stride() const { return rank ? strides[rank - 1] : 1; }
    int64_t size() const {
        int64_t s = 1;
        for (int i = 0; i < rank; ++i) s *= dims[i];
        return s;
    }
};

// ---------------------------------------------------------------- reducers
enum class Red { Sum, Mean, Max, Min, LogSumExp, SumExp, Prod, ASum, SumSquare, Nrm2, LogSum, AMax, AMin };

bool parse_reduce(const char* name, Red* r) {
    static const std::pair<const char*, Red> table[] = {
        {"reduce_sum", Red::Sum}, {"reduce_mean", Red::Mean}, {"reduce_max", Red::Max},
        {"reduce_min", Red::Min}, {"reduce_log_sum_exp", Red::LogSumExp},
        {"reduce_sum_exp", Red::SumExp}, {"reduce_prod", Red::Prod},
        {"reduce_asum", Red::ASum}, {"reduce_sum_square", Red::SumSquare},
        {"reduce_nrm2", Red::Nrm2}, {"reduce_log_sum", Red::LogSum},
        {"reduce_amax", Red::AMax}, {"reduce_amin", Red::AMin}};
    for (auto& e : table)
        if (!std::strcmp(name, e.first)) { *r = e.second; return true; }
    return false;
}

// std::complex elements (float2 / double2 on the device side): the reducer table instantiated
// with T = std::complex<F> as the reference's host templates do (abs and norm yield a real
// value converted back to T, exp / log / sqrt are the std::complex functions, mean divides by
// T(n)); the ordering reducers do not compile there and are rejected here.
template <typename T> struct is_complex : std::false_type {};
template <typename F> struct is_complex<std::complex<F>> : std::true_type {};

template <typename T> T t_abs(T x) { return x < 0 ? T(-x) : x; }
template <typename T> T t_exp(T x) { return static_cast<T>(std::exp(static_cast<double>(x))); }
template <> float  t_exp<float>(float x)   { return std::exp(x); }
template <> double t_exp<double>(double x) { return std::exp(x); }
template <typename T> T t_log(T x) { return static_cast<T>(std::log(static_cast<double>(x))); }
template <> float  t_log<float>(float x)   { return std::log(x); }
template <> double t_log<double>(double x) { return std::log(x); }
template <typename T> T t_sqrt(T x) { return static_cast<T>(std::sqrt(static_cast<double>(x))); }
template <> float  t_sqrt<float>(float x)  { return std::sqrt(x); }

template <typename T> T red_identity(Red r) {
    if constexpr (is_complex<T>::value) return r == Red::Prod ? T(1) : T(0);
    else
    switch (r) {
    case Red::Max: return std::numeric_limits<T>::lowest();
    case Red::Min: case Red::AMin: return std::numeric_limits<T>::max();
    case Red::Prod: return T(1);
    default: return T(0);
    }
}
template <typename T> T red_map(Red r, T x) {
    if constexpr (is_complex<T>::value) {
        switch (r) {
        case Red::LogSumExp: case Red::SumExp: return std::exp(x);
        case Red::ASum: return T(std::abs(x));
        case Red::SumSquare: return x * x;
        case Red::Nrm2: return T(std::norm(x));
        default: return x;
        }
    } else
    switch (r) {
    case Red::LogSumExp: case Red::SumExp: return t_exp(x);
    case Red::ASum: case Red::AMax: case Red::AMin: return t_abs(x);
    case Red::SumSquare: case Red::Nrm2: return T(x * x);
    default: return x;
    }
}
template <typename T> T red_join(Red r, T a, T b) {
    if constexpr (is_complex<T>::value) return r == Red::Prod ? a * b : a + b;
    else
    switch (r) {
    case Red::Max: return std::max(a, b);
    case Red::Min: return std::min(a, b);
    case Red::Prod: return T(a * b);
    case Red::AMax: return (t_abs(a) < t_abs(b)) ? b : a;
    case Red::AMin: return (t_abs(a) < t_abs(b)) ? a : b;
    default: return T(a + b);
    }
}
template <typename T> T red_final(Red r, T acc, int64_t n) {
    if constexpr (is_complex<T>::value) {
        switch (r) {
        case Red::Mean: return acc / T(static_cast<typename T::value_type>(n));
        case Red::LogSumExp: case Red::LogSum: return std::log(acc);
        case Red::Nrm2: return std::sqrt(acc);
        default: return acc;
        }
    } else
    switch (r) {
    case Red::Mean: return T(acc / static_cast<T>(n));
    case Red::LogSumExp: case Red::LogSum: return t_log(acc);
    case Red::Nrm2: return t_sqrt(acc);
    default: return acc;
    }
}

// One row of do_reduce: ranges longer than the grain split in halves and join
// with the reducer; leaves fold left to right starting from the identity.
template <typename T>
T reduce_range(Red r, const T* x, const View& xv, int64_t row_first, int64_t lo, int64_t hi) {
    if (hi - lo > kGrain) {
        int64_t mid = lo + (hi - lo) / 2;
        T a = reduce_range(r, x, xv, row_first, lo, mid);
        T b = reduce_range(r, x, xv, row_first, mid, hi);
        return red_join(r, a, b);
    }
    T acc = red_identity<T>(r);
    for (int64_t j = lo; j < hi; ++j)
        acc = red_join(r, acc, red_map(r, x[xv.at(row_first + j)]));
    return acc;
}

template <typename T>
int do_reduce(Red r, int64_t m, int64_t n, const View& xv, const T* x, const View& yv, T* y) {
    if (m * n < kGrain) {
        for (int64_t i = 0; i < m; ++i) {
            T acc = red_identity<T>(r);
            for (int64_t j = 0; j < n; ++j)
                acc = red_join(r, acc, red_map(r, x[xv.at(i * n + j)]));
            y[yv.at(i)] = red_final(r, acc, n);
        }
        return 0;
    }
    if (m == 1) {
        // A single long row: leaves in parallel, joined in the same tree order.
        int64_t leaves = (n + kGrain - 1) / kGrain;
        if (leaves > 64) {
            // split the top of the tree over threads; each subtree is the serial recursion
            int64_t parts = 64;
            std::vector<T> partial(parts);
            std::vector<int64_t> cut(parts + 1);
            // cuts follow the recursive halving so the association is unchanged
            std::function<void(int64_t, int64_t, int64_t, int64_t)> mk =
                [&](int64_t lo, int64_t hi, int64_t p0, int64_t p1) {
                    if (p1 - p0 == 1) { cut[p0] = lo; cut[p1] = hi; return; }
                    int64_t mid = lo + (hi - lo) / 2, pm = p0 + (p1 - p0) / 2;
                    mk(lo, mid, p0, pm); mk(mid, hi, pm, p1);
                };
            mk(0, n, 0, parts);
#pragma omp parallel for schedule(dynamic, 1)
            for (int64_t p = 0; p < parts; ++p)
                partial[p] = reduce_range(r, x, xv, 0, cut[p], cut[p + 1]);
            std::function<T(int64_t, int64_t)> join = [&](int64_t p0, int64_t p1) -> T {
                if (p1 - p0 == 1) return partial[p0];
                int64_t pm = p0 + (p1 - p0) / 2;
                return red_join(r, join(p0, pm), join(pm, p1));
            };
            y[yv.at(0)] = red_final(r, join(0, parts), n);
            return 0;
        }
    }
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < m; ++i)
        y[yv.at(i)] = red_final(r, reduce_range(r, x, xv, i * n, 0, n), n);
    return 0;
}

// fp64 evaluation of the same reducer on the same elements (one double per row).
template <typename T>
int do_reduce_f64(Red r, int64_t m, int64_t n, const View& xv, const T* x, double* y) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < m; ++i) {
        long double acc;
        bool first = true;
        acc = (r == Red::Prod) ? 1.0L : 0.0L;
        for (int64_t j = 0; j < n; ++j) {
            double v = static_cast<double>(x[xv.at(i * n + j)]);
            switch (r) {
            case Red::Max: acc = first ? v : std::max<long double>(acc, v); break;
            case Red::Min: acc = first ? v : std::min<long double>(acc, v); break;
            case Red::AMax: acc = first ? std::fabs(v) : std::max<long double>(acc, std::fabs(v)); break;
            case Red::AMin: acc = first ? std::fabs(v) : std::min<long double>(acc, std::fabs(v)); break;
            case Red::Prod: acc *= v; break;
            case Red::LogSumExp: case Red::SumExp: acc += std::exp(v); break;
            case Red::ASum: acc += std::fabs(v); break;
            case Red::SumSquare: case Red::Nrm2: acc += v * v; break;
            default: acc += v; break;
            }
            first = false;
        }
        switch (r) {
        case Red::Mean: acc /= static_cast<long double>(n); break;
        case Red::LogSumExp: case Red::LogSum: acc = std::log(static_cast<double>(acc)); break;
        case Red::Nrm2: acc = std::sqrt(static_cast<double>(acc)); break;
        default: break;
        }
        y[i] = static_cast<double>(acc);
    }
    return 0;
}

// ---------------------------------------------------------------- arg reduce
template <typename T>
int do_arg_reduce(bool want_max, int64_t rows, int64_t k, const View& xv, const T* x,
                  const View& yv, int32_t* y) {
    const int64_t sk = xv.last_stride();
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < rows; ++i) {
        const T* px = x + xv.at(i * k);
        T acc = *px;
        int32_t index = 0;
        for (int64_t ik = 1; ik < k; ++ik) {
            px += sk;
            bool better = want_max ? (*px > acc) : (*px < acc);
            if (better) { acc = *px; index = static_cast<int32_t>(ik); }
        }
        y[yv.at(i)] = index;
    }
    return 0;
}

// ---------------------------------------------------------------- scan
enum class Scn { Sum, Prod, Max, Min };
bool parse_scan(const char* name, Scn* s) {
    if (!std::strcmp(name, "cumsum")) { *s = Scn::Sum; return true; }
    if (!std::strcmp(name, "cumprod")) { *s = Scn::Prod; return true; }
    if (!std::strcmp(name, "cummax")) { *s = Scn::Max; return true; }
    if (!std::strcmp(name, "cummin")) { *s = Scn::Min; return true; }
    return false;
}
template <typename T> T scan_identity(Scn s) {
    if constexpr (is_complex<T>::value) return s == Scn::Prod ? T(1) : T(0);
    else
    switch (s) {
    case Scn::Prod: return T(1);
    case Scn::Max: return std::numeric_limits<T>::lowest();
    case Scn::Min: return std::numeric_limits<T>::max();
    default: return T(0);
    }
}
template <typename T> T scan_op(Scn s, T a, T b) {
    if constexpr (is_complex<T>::value) return s == Scn::Prod ? a * b : a + b;
    else
    switch (s) {
    case Scn::Prod: return T(a * b);
    case Scn::Max: return std::max(a, b);
    case Scn::Min: return std::min(a, b);
    default: return T(a + b);   // built with -fwrapv: integer sums wrap
    }
}

// serial_scan over [first, first+len) of one row; when `write` is false only the
// running value is produced (the pre-scan pass of a two-pass parallel scan).
template <typename T>
T serial_scan(Scn s, int64_t len, int64_t flat, bool exclusive, bool write, T acc,
              const View& xv, const T* x, const View& yv, T* y) {
    const T* px = x + xv.at(flat);
    T* py = y + yv.at(flat);
    const int64_t ix = xv.last_stride(), iy = yv.last_stride();
    for (; len > 0; --len, px += ix, py += iy) {
        if (write && exclusive) *py = acc;
        acc = scan_op(s, acc, *px);
        if (write && !exclusive) *py = acc;
    }
    return acc;
}

template <typename T>
int do_scan(Scn s, int64_t m, int64_t n, bool exclusive, const View& xv, const T* x,
            const View& yv, T* y) {
    const T id = scan_identity<T>(s);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < m; ++i) {
        if (n < kGrain) {
            serial_scan(s, n, i * n, exclusive, true, id, xv, x, yv, y);
            continue;
        }
        // Two-pass schedule of a parallel scan with 1024-element chunks: chunk
        // totals first, a serial scan of the totals, then the final pass with
        // each chunk starting from its carried-in value.
        const int64_t chunks = (n + kGrain - 1) / kGrain;
        std::vector<T> total(chunks);
        for (int64_t c = 0; c < chunks; ++c) {
            int64_t lo = c * kGrain, len = std::min(kGrain, n - lo);
            total[c] = serial_scan(s, len, i * n + lo, exclusive, false, id, xv, x, yv, y);
        }
        T carry = id;
        for (int64_t c = 0; c < chunks; ++c) {
            int64_t lo = c * kGrain, len = std::min(kGrain, n - lo);
            // x and y may alias, so the chunk total was taken before any write
            T next = scan_op(s, carry, total[c]);
            serial_scan(s, len, i * n + lo, exclusive, true, carry, xv, x, yv, y);
            carry = next;
        }
    }
    return 0;
}

template <typename T>
int do_scan_f64(Scn s, int64_t m, int64_t n, bool exclusive, const View& xv, const T* x,
                double* y, double* abs_prefix) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < m; ++i) {
        long double acc = (s == Scn::Prod) ? 1.0L : 0.0L, mag = 0.0L;
        bool first = true;
        const T* px = x + xv.at(i * n);
        const int64_t ix = xv.last_stride();
        for (int64_t j = 0; j < n; ++j, px += ix) {
            long double v = static_cast<long double>(*px);
            if (exclusive) {
                y[i * n + j] = (first && (s == Scn::Max || s == Scn::Min))
                                   ? static_cast<double>(scan_identity<T>(s)) : static_cast<double>(acc);
                if (abs_prefix) abs_prefix[i * n + j] = static_cast<double>(mag);
            }
            switch (s) {
            case Scn::Prod: acc *= v; break;
            case Scn::Max: acc = first ? v : std::max(acc, v); break;
            case Scn::Min: acc = first ? v : std::min(acc, v); break;
            default: acc += v; break;
            }
            mag += std::fabs(static_cast<double>(v));
            first = false;
            if (!exclusive) {
                y[i * n + j] = static_cast<double>(acc);
                if (abs_prefix) abs_prefix[i * n + j] = static_cast<double>(mag);
            }
        }
    }
    return 0;
}

// ---------------------------------------------------------------- sort
constexpr int64_t kSortCutOff = 500;     // reorder_detail.h:511
constexpr int64_t kArgsortCutOff = 100;  // reorder_detail.h:679

template <typename T, typename Cmp>
void merge_sort_row(std::vector<T>& buf, std::vector<T>& aux, int64_t lo, int64_t hi, Cmp cmp) {
    const int64_t n = hi - lo;
    if (n <= kSortCutOff) {
        std::sort(buf.begin() + lo, buf.begin() + hi, cmp);
        return;
    }
    const int64_t mid = lo + n / 2;
    merge_sort_row(buf, aux, lo, mid, cmp);
    merge_sort_row(buf, aux, mid, hi, cmp);
    std::merge(buf.begin() + lo, buf.begin() + mid, buf.begin() + mid, buf.begin() + hi,
               aux.begin() + lo, cmp);
    std::copy(aux.begin() + lo, aux.begin() + hi, buf.begin() + lo);
}

template <typename T>
int do_sort(int dir, const View& xv, const T* x, const View& yv, T* y) {
    const int64_t n = xv.last_extent();
    const int64_t m = xv.size() / n;
    const int64_t ix = xv.last_stride(), iy = yv.last_stride();
#pragma omp parallel for schedule(dynamic, 1)
    for (int64_t b = 0; b < m; ++b) {
        std::vector<T> buf(n), aux(n);
        const T* px = x + xv.at(b * n);
        for (int64_t j = 0; j < n; ++j) buf[j] = px[j * ix];
        if (dir) merge_sort_row(buf, aux, 0, n, std::greater<T>());
        else     merge_sort_row(buf, aux, 0, n, std::less<T>());
        T* py = y + yv.at(b * n);
        for (int64_t j = 0; j < n; ++j) py[j * iy] = buf[j];
    }
    return 0;
}

// Stable arg merge sort: insertion leaves placed with an upper bound (equal keys
// keep arrival order), merges take from the right run only on a strict win.
template <typename T, typename Cmp>
void arg_merge_sort_row(std::vector<T>& key, std::vector<int32_t>& idx, std::vector<T>& kaux,
                        std::vector<int32_t>& iaux, int64_t lo, int64_t hi, Cmp cmp) {
    const int64_t n = hi - lo;
    if (n <= kArgsortCutOff) {
        for (int64_t i = lo + 1; i < hi; ++i) {
            T kv = key[i];
            int32_t iv = idx[i];
            int64_t pos = std::upper_bound(key.begin() + lo, key.begin() + i, kv, cmp) - key.begin();
            for (int64_t j = i; j > pos; --j) { key[j] = key[j - 1]; idx[j] = idx[j - 1]; }
            key[pos] = kv;
            idx[pos] = iv;
        }
        return;
    }
    const int64_t mid = lo + n / 2;
    arg_merge_sort_row(key, idx, kaux, iaux, lo, mid, cmp);
    arg_merge_sort_row(key, idx, kaux, iaux, mid, hi, cmp);
    int64_t a = lo, b = mid, o = lo;
    while (a < mid && b < hi) {
        if (cmp(key[b], key[a])) { kaux[o] = key[b]; iaux[o] = idx[b]; ++b; }
        else                     { kaux[o] = key[a]; iaux[o] = idx[a]; ++a; }
        ++o;
    }
    for (; a < mid; ++a, ++o) { kaux[o] = key[a]; iaux[o] = idx[a]; }
    for (; b < hi; ++b, ++o)  { kaux[o] = key[b]; iaux[o] = idx[b]; }
    std::copy(kaux.begin() + lo, kaux.begin() + hi, key.begin() + lo);
    std::copy(iaux.begin() + lo, iaux.begin() + hi, idx.begin() + lo);
}

template <typename T>
int do_argsort(int dir, const View& xv, const T* x, const View* yv, T* y,
               const View& iv, int32_t* idx_out) {
    const int64_t n = xv.last_extent();
    const int64_t m = xv.size() / n;
    const int64_t ix = xv.last_stride(), ii = iv.last_stride();
#pragma omp parallel for schedule(dynamic, 1)
    for (int64_t b = 0; b < m; ++b) {
        std::vector<T> key(n), kaux(n);
        std::vector<int32_t> idx(n), iaux(n);
        const T* px = x + xv.at(b * n);
        for (int64_t j = 0; j < n; ++j) { key[j] = px[j * ix]; idx[j] = static_cast<int32_t>(j); }
        if (dir) arg_merge_sort_row(key, idx, kaux, iaux, 0, n, std::greater<T>());
        else     arg_merge_sort_row(key, idx, kaux, iaux, 0, n, std::less<T>());
        if (y) {
            T* py = y + yv->at(b * n);
            const int64_t iy = yv->last_stride();
            for (int64_t j = 0; j < n; ++j) py[j * iy] = key[j];
        }
        int32_t* pi = idx_out + iv.at(b * n);
        for (int64_t j = 0; j < n; ++j) pi[j * ii] = idx[j];
    }
    return 0;
}

// ---------------------------------------------------------------- top-k
// Heap selection as the reference does it: 1-based binary heap whose root is the
// weakest kept element; a candidate replaces the root only on a strict win.
template <typename T, typename Cmp>
void sift_down(std::pair<T, int64_t>* h1, int64_t k, int64_t i, Cmp cmp) {
    for (;;) {
        int64_t l = 2 * i, r = 2 * i + 1, j = i;
        if (l <= k && cmp(h1[j].first, h1[l].first)) j = l;
        if (r <= k && cmp(h1[j].first, h1[r].first)) j = r;
        if (j == i) return;
        std::swap(h1[i], h1[j]);
        i = j;
    }
}

template <typename T, typename Cmp>
void heap_select(int64_t n, int64_t k, const T* px, int64_t ix, Cmp cmp,
                 std::vector<std::pair<T, int64_t>>& heap) {
    heap.clear();
    heap.reserve(k);
    for (int64_t i = 0; i < k; ++i) heap.emplace_back(px[i * ix], i);
    auto* h1 = heap.data() - 1;
    for (int64_t i = k / 2; i > 0; --i) sift_down(h1, k, i, cmp);
    for (int64_t i = k; i < n; ++i) {
        T v = px[i * ix];
        if (cmp(v, heap.front().first)) {
            heap.front() = {v, i};
            sift_down(h1, k, 1, cmp);
        }
    }
}

template <typename T, typename I>
int do_top_k(int mode, int largest, int sorted, int64_t k, const View& xv, const T* x,
             const View& yv, T* y, const View& iv, I* idx) {
    const int64_t n = xv.last_extent();
    const int64_t m = xv.size() / n;
    const int64_t ix = xv.last_stride(), iy = yv.last_stride(), ii = iv.last_stride();
#pragma omp parallel for schedule(dynamic, 4)
    for (int64_t b = 0; b < m; ++b) {
        const T* px = x + xv.at(b * n);
        T* py = y + yv.at(b * k);
        I* pi = idx + iv.at(b * k);
        std::vector<std::pair<T, int64_t>> sel;
        if (mode == 0) {
            // reference algorithm: heap, then sort the k survivors by value only
            if (largest) heap_select(n, k, px, ix, std::greater<T>(), sel);
            else         heap_select(n, k, px, ix, std::less<T>(), sel);
            if (sorted) {
                if (largest) std::sort(sel.begin(), sel.end(), [](auto& a, auto& b2) { return a.first > b2.first; });
                else         std::sort(sel.begin(), sel.end(), [](auto& a, auto& b2) { return a.first < b2.first; });
            }
        } else {
            // specification rule: first k of a stable sort (lowest index wins ties)
            std::vector<int64_t> order(n);
            std::iota(order.begin(), order.end(), int64_t(0));
            auto by = [&](int64_t a, int64_t c) {
                T va = px[a * ix], vc = px[c * ix];
                return largest ? (va > vc) : (va < vc);
            };
            std::stable_sort(order.begin(), order.end(), by);
            sel.reserve(k);
            for (int64_t j = 0; j < k; ++j) sel.emplace_back(px[order[j] * ix], order[j]);
        }
        for (int64_t j = 0; j < k; ++j) {
            py[j * iy] = sel[j].first;
            pi[j * ii] = static_cast<I>(sel[j].second);
        }
    }
    return 0;
}

template <typename F>
int by_dtype(int dtype, F&& f) {
    switch (dtype) {
    case 0: return f(float());
    case 1: return f(double());
    case 2: return f(int32_t());
    case 3: return f(int64_t());
    default: return -2;
    }
}

// dtype codes 7 / 8: complex of floats / doubles (reduce, count and scan only)
template <typename F>
int by_dtype_complex(int dtype, F&& f) {
    if (dtype == 7) return f(std::complex<float>());
    if (dtype == 8) return f(std::complex<double>());
    return by_dtype(dtype, f);
}
bool complex_dtype(int dtype) { return dtype == 7 || dtype == 8; }
bool ordered_only(Red r) { return r == Red::Max || r == Red::Min || r == Red::AMax || r == Red::AMin; }

}  // namespace

extern "C" {

int dlf_oracle_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void dlf_oracle_set_threads(int n) {
#ifdef _OPENMP
    omp_set_num_threads(n);
#else
    (void)n;
#endif
}

int dlf_oracle_reduce(const char* name, int dtype, int64_t m, int64_t n,
                      int x_rank, const int64_t* x_dims, const int64_t* x_strides,
                      const void* x, int64_t x_offset,
                      int y_rank, const int64_t* y_dims, const int64_t* y_strides,
                      void* y, int64_t y_offset) {
    Red r;
    if (!parse_reduce(name, &r)) return -1;
    View xv(x_rank, x_dims, x_strides, x_offset), yv(y_rank, y_dims, y_strides, y_offset);
    if (complex_dtype(dtype) && ordered_only(r)) return -2;
    return by_dtype_complex(dtype, [&](auto tag) {
        using T = decltype(tag);
        return do_reduce<T>(r, m, n, xv, static_cast<const T*>(x), yv, static_cast<T*>(y));
    });
}

int dlf_oracle_reduce_f64(const char* name, int dtype, int64_t m, int64_t n,
                          int x_rank, const int64_t* x_dims, const int64_t* x_strides,
                          const void* x, int64_t x_offset, double* y) {
    Red r;
    if (!parse_reduce(name, &r)) return -1;
    View xv(x_rank, x_dims, x_strides, x_offset);
    return by_dtype(dtype, [&](auto tag) {
        using T = decltype(tag);
        return do_reduce_f64<T>(r, m, n, xv, static_cast<const T*>(x), y);
    });
}

int dlf_oracle_arg_reduce(const char* name, int dtype, int64_t rows, int64_t k,
                          int x_rank, const int64_t* x_dims, const int64_t* x_strides,
                          const void* x, int64_t x_offset,
                          int y_rank, const int64_t* y_dims, const int64_t* y_strides,
                          int32_t* y, int64_t y_offset) {
    bool want_max;
    if (!std::strcmp(name, "argmax")) want_max = true;
    else if (!std::strcmp(name, "argmin")) want_max = false;
    else return -1;
    View xv(x_rank, x_dims, x_strides, x_offset), yv(y_rank, y_dims, y_strides, y_offset);
    return by_dtype(dtype, [&](auto tag) {
        using T = decltype(tag);
        return do_arg_reduce<T>(want_max, rows, k, xv, static_cast<const T*>(x), yv, y);
    });
}

int dlf_oracle_scan(const char* name, int dtype, int64_t m, int64_t n, int exclusive,
                    int rank, const int64_t* dims,
                    const void* x, int64_t x_offset, const int64_t* x_strides,
                    void* y, int64_t y_offset, const int64_t* y_strides) {
    Scn s;
    if (!parse_scan(name, &s)) return -1;
    View xv(rank, dims, x_strides, x_offset), yv(rank, dims, y_strides, y_offset);
    if (complex_dtype(dtype) && (s == Scn::Max || s == Scn::Min)) return -2;
    return by_dtype_complex(dtype, [&](auto tag) {
        using T = decltype(tag);
        return do_scan<T>(s, m, n, exclusive != 0, xv, static_cast<const T*>(x), yv, static_cast<T*>(y));
    });
}

// y (and abs_prefix when non-null: running sum of |x|) are contiguous [m][n] doubles.
int dlf_oracle_scan_f64(const char* name, int dtype, int64_t m, int64_t n, int exclusive,
                        int rank, const int64_t* dims,
                        const void* x, int64_t x_offset, const int64_t* x_strides,
                        double* y, double* abs_prefix) {
    Scn s;
    if (!parse_scan(name, &s)) return -1;
    View xv(rank, dims, x_strides, x_offset);
    return by_dtype(dtype, [&](auto tag) {
        using T = decltype(tag);
        return do_scan_f64<T>(s, m, n, exclusive != 0, xv, static_cast<const T*>(x), y, abs_prefix);
    });
}

int dlf_oracle_sort(int dir, int dtype, int rank, const int64_t* dims,
                    const void* x, int64_t x_offset, const int64_t* x_strides,
                    void* y, int64_t y_offset, const int64_t* y_strides) {
    View xv(rank, dims, x_strides, x_offset), yv(rank, dims, y_strides, y_offset);
    return by_dtype(dtype, [&](auto tag) {
        using T = decltype(tag);
        return do_sort<T>(dir, xv, static_cast<const T*>(x), yv, static_cast<T*>(y));
    });
}

// y may be null (index-only argsort).
int dlf_oracle_argsort(int dir, int dtype, int rank, const int64_t* dims,
                       const void* x, int64_t x_offset, const int64_t* x_strides,
                       void* y, int64_t y_offset, const int64_t* y_strides,
                       int32_t* idx, int64_t i_offset, const int64_t* i_strides) {
    View xv(rank, dims, x_strides, x_offset), iv(rank, dims, i_strides, i_offset);
    View yv(rank, dims, y_strides ? y_strides : x_strides, y_offset);
    return by_dtype(dtype, [&](auto tag) {
        using T = decltype(tag);
        return do_argsort<T>(dir, xv, static_cast<const T*>(x), y ? &yv : nullptr,
                             static_cast<T*>(y), iv, idx);
    });
}

// mode 0: the reference's heap algorithm (values are well defined, tie indices are
// whatever the heap leaves); mode 1: specification order (stable, lowest index).
// index_bytes selects int32 or int64 index output.
int dlf_oracle_top_k(int mode, int64_t limit, int largest, int sorted, int dtype,
                     int rank, const int64_t* x_dims, const int64_t* y_dims,
                     const void* x, int64_t x_offset, const int64_t* x_strides,
                     void* y, int64_t y_offset, const int64_t* y_strides,
                     void* idx, int64_t i_offset, const int64_t* i_strides, int index_bytes) {
    View xv(rank, x_dims, x_strides, x_offset), yv(rank, y_dims, y_strides, y_offset),
         iv(rank, y_dims, i_strides, i_offset);
    if (limit > xv.last_extent() || limit != yv.last_extent()) return -3;
    return by_dtype(dtype, [&](auto tag) {
        using T = decltype(tag);
        if (index_bytes == 8)
            return do_top_k<T, int64_t>(mode, largest, sorted, limit, xv, static_cast<const T*>(x), yv,
                                        static_cast<T*>(y), iv, static_cast<int64_t*>(idx));
        return do_top_k<T, int32_t>(mode, largest, sorted, limit, xv, static_cast<const T*>(x), yv,
                                    static_cast<T*>(y), iv, static_cast<int32_t*>(idx));
    });
}

// count (dlf/include/tensor/reduce.h:151-158): reduce with identity 0, Map x == value ? 1 : 0,
// fold +, over the permuted view that prepare_reduce builds; integer addition, so the order
// of the fold does not matter.
int dlf_oracle_count(int dtype, int64_t m, int64_t n, const void* value,
                     int x_rank, const int64_t* x_dims, const int64_t* x_strides,
                     const void* x, int64_t x_offset,
                     int y_rank, const int64_t* y_dims, const int64_t* y_strides,
                     int32_t* y, int64_t y_offset) {
    View xv(x_rank, x_dims, x_strides, x_offset), yv(y_rank, y_dims, y_strides, y_offset);
    return by_dtype_complex(dtype, [&](auto tag) {
        using T = decltype(tag);
        T v;
        std::memcpy(&v, value, sizeof(T));
        const T* xp = static_cast<const T*>(x);
#pragma omp parallel for schedule(static)
        for (int64_t i = 0; i < m; ++i) {
            int32_t acc = 0;
            for (int64_t j = 0; j < n; ++j) acc += xp[xv.at(i * n + j)] == v ? 1 : 0;
            y[yv.at(i)] = acc;
        }
        return 0;
    });
}

// First half of nonzero() (dlf/include/tensor/reduce.h:383-386): indices = (x != 0), then
// cumsum(indices, indices) along the last axis.
int dlf_oracle_scan_nonzero(int dtype, int64_t m, int64_t n, int exclusive,
                            int rank, const int64_t* dims,
                            const void* x, int64_t x_offset, const int64_t* x_strides,
                            int32_t* y, int64_t y_offset, const int64_t* y_strides) {
    View xv(rank, dims, x_strides, x_offset), yv(rank, dims, y_strides, y_offset);
    return by_dtype(dtype, [&](auto tag) {
        using T = decltype(tag);
        const T* xp = static_cast<const T*>(x);
        for (int64_t i = 0; i < m; ++i) {
            int32_t acc = 0;
            for (int64_t j = 0; j < n; ++j) {
                const int32_t flag = xp[xv.at(i * n + j)] != T(0) ? 1 : 0;
                if (exclusive) {
                    y[yv.at(i * n + j)] = acc;
                    acc += flag;
                } else {
                    acc += flag;
                    y[yv.at(i * n + j)] = acc;
                }
            }
        }
        return 0;
    });
}

// Second half of nonzero() (dlf/include/tensor/reduce.h:404-417): for every element i whose
// running count differs from its predecessor's, the coordinates of flat index i go to column
// prev of a [rank, n] matrix (row_major) or to row prev of an [n, rank] matrix.
int dlf_oracle_gather_indices(int64_t m, int64_t n, int row_major, int rank, const int64_t* dims,
                              const int32_t* idx, int32_t* out) {
    for (int64_t i = 0; i < m; ++i) {
        const int32_t curr = idx[i];
        const int32_t prev = i == 0 ? 0 : idx[i - 1];
        if (curr != prev) {
            int64_t temp = i;
            for (int j = rank; --j >= 0;) {
                const int64_t id = row_major ? (n * j + prev) : (static_cast<int64_t>(prev) * rank + j);
                out[id] = static_cast<int32_t>(temp % dims[j]);
                temp /= dims[j];
            }
        }
    }
    return 0;
}

// merge (dlf/include/tensor/reorder_detail.h:346-368, 470-494): per row, the serial merge that
// takes y's element only when comp(y, x); the parallel split of longer rows produces the same
// sequence because it cuts x at a pivot and y at lower_bound of that pivot (394-449).
int dlf_oracle_merge(int dir, int dtype, int rank,
                     const int64_t* x_dims, const int64_t* x_strides, const void* x, int64_t x_offset,
                     const int64_t* y_dims, const int64_t* y_strides, const void* y, int64_t y_offset,
                     const int64_t* z_dims, const int64_t* z_strides, void* z, int64_t z_offset) {
    View xv(rank, x_dims, x_strides, x_offset), yv(rank, y_dims, y_strides, y_offset), zv(rank, z_dims, z_strides, z_offset);
    const int64_t na = x_dims[rank - 1], nb = y_dims[rank - 1], n = na + nb;
    if (n != z_dims[rank - 1]) return -3;
    const int64_t rows = zv.size() / n;
    return by_dtype(dtype, [&](auto tag) {
        using T = decltype(tag);
        const T* xp = static_cast<const T*>(x);
        const T* yp = static_cast<const T*>(y);
        T* zp = static_cast<T*>(z);
        auto comp = [dir](T a, T b) { return dir ? a > b : a < b; };
#pragma omp parallel for schedule(static)
        for (int64_t r = 0; r < rows; ++r) {
            int64_t i = 0, j = 0, k = 0;
            const int64_t xb = na ? xv.at(r * na) : 0, yb = nb ? yv.at(r * nb) : 0, zb = zv.at(r * n);
            const int64_t sx = xv.last_stride(), sy = yv.last_stride(), sz = zv.last_stride();
            while (i < na && j < nb) {
                if (comp(yp[yb + j * sy], xp[xb + i * sx])) zp[zb + (k++) * sz] = yp[yb + (j++) * sy];
                else zp[zb + (k++) * sz] = xp[xb + (i++) * sx];
            }
            while (i < na) zp[zb + (k++) * sz] = xp[xb + (i++) * sx];
            while (j < nb) zp[zb + (k++) * sz] = yp[yb + (j++) * sy];
        }
        return 0;
    });
}

// softmax / logsoftmax / hardmax on the rows of a contiguous [m, n] matrix, in place, as the
// reference's row loops (dlf/include/tensor/dnn_detail.h:266-350): serial maximum from px[0]
// with std::max, serial sum in the element type.  kind: 0 softmax, 1 logsoftmax, 2 hardmax.
int dlf_oracle_softmax(int kind, int dtype, int64_t m, int64_t n, void* x) {
    if (dtype != 0 && dtype != 1 && !(kind == 2 && (dtype == 2 || dtype == 3))) return -2;
    auto run = [&](auto tag) {
        using T = decltype(tag);
        using F = std::conditional_t<std::is_integral<T>::value, double, T>;     // integers reach hardmax only
        T* base = static_cast<T*>(x);
#pragma omp parallel for schedule(static)
        for (int64_t b = 0; b < m; ++b) {
            T* px = base + b * n;
            if (kind == 2) {
                T amax = px[0];
                int64_t imax = 0;
                for (int64_t i = 0; i < n; ++i) {
                    if (px[i] > amax) {
                        amax = px[i];
                        imax = i;
                    }
                    px[i] = 0;
                }
                px[imax] = 1;
                continue;
            }
            T amax = px[0];
            for (int64_t i = 1; i < n; ++i) amax = std::max(amax, px[i]);
            F asum = 0;
            if (kind == 0) {
                for (int64_t i = 0; i < n; ++i) {
                    px[i] = static_cast<T>(std::exp(static_cast<F>(px[i] - amax)));
                    asum += px[i];
                }
                for (int64_t i = 0; i < n; ++i) px[i] = static_cast<T>(px[i] / asum);
            } else {
                for (int64_t i = 0; i < n; ++i) asum += std::exp(static_cast<F>(px[i] - amax));
                asum = std::log(asum);
                for (int64_t i = 0; i < n; ++i) px[i] = static_cast<T>(px[i] - amax - asum);
            }
        }
        return 0;
    };
    switch (dtype) {
    case 0: return run(float());
    case 1: return run(double());
    case 2: return run(int32_t());
    default: return run(int64_t());
    }
}

}  // extern "C"
