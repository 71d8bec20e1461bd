// copy / fill over strided views for gfx950: the layout steps the axis primitives' front-ends
// take on the device (a strided view into row-major storage before the in-place softmax family,
// the copy that sort / argsort of an extent-1 axis degenerates to, zero indices).
//
// Elements are moved as opaque 1, 2, 4, 8 or 16-byte words, so one set of kernels serves every
// element type.  Dimensions are merged jointly over source and destination; a thread walks four
// elements a workgroup-width apart, so neighbouring lanes touch neighbouring elements of the
// innermost dimension and accesses coalesce whenever that dimension is contiguous on a side.
#include <cstring>

#include "common.hip.h"

namespace dlfx {
namespace {

constexpr int kCopyBlock = 256;
constexpr int kCopyItems = 4;

// The same extents walked with two stride sets.
struct DimMap2 {
    int rank;
    int64_t dims[kMaxRank];
    int64_t xs[kMaxRank];
    int64_t ys[kMaxRank];
};

// Drops extent-1 dimensions and merges neighbours that both views walk as one dimension.
bool make_dim_map2(int rank, const int64_t* dims, const int64_t* xs, const int64_t* ys, DimMap2* out) {
    int r = 0;
    int64_t d[64], a[64], b[64];
    for (int i = 0; i < rank; ++i) {
        if (dims[i] == 1) continue;
        if (r > 0 && a[r - 1] == xs[i] * dims[i] && b[r - 1] == ys[i] * dims[i]) {
            d[r - 1] *= dims[i];
            a[r - 1] = xs[i];
            b[r - 1] = ys[i];
        } else {
            d[r] = dims[i];
            a[r] = xs[i];
            b[r] = ys[i];
            ++r;
        }
    }
    if (r > kMaxRank) return false;
    out->rank = r;
    for (int i = 0; i < kMaxRank; ++i) {
        out->dims[i] = i < r ? d[i] : 1;
        out->xs[i] = i < r ? a[i] : 0;
        out->ys[i] = i < r ? b[i] : 0;
    }
    return true;
}

template <int RANK>
__device__ __forceinline__ void offsets_of(const DimMap2& dm, int64_t flat, int64_t* xo, int64_t* yo) {
    int64_t a = 0, b = 0;
#pragma unroll
    for (int i = RANK - 1; i > 0; --i) {
        const int64_t d = dm.dims[i];
        const int64_t q = flat / d;
        const int64_t r = flat - q * d;
        a += r * dm.xs[i];
        b += r * dm.ys[i];
        flat = q;
    }
    if (RANK > 0) {
        a += flat * dm.xs[0];
        b += flat * dm.ys[0];
    }
    *xo = a;
    *yo = b;
}

template <typename E, int RANK>
__global__ __launch_bounds__(kCopyBlock) void copy_strided(const E* __restrict__ x, E* __restrict__ y, DimMap2 dm, int64_t total) {
    const int64_t base = static_cast<int64_t>(blockIdx.x) * (kCopyBlock * kCopyItems) + threadIdx.x;
    E v[kCopyItems];
    int64_t yo[kCopyItems];
#pragma unroll
    for (int k = 0; k < kCopyItems; ++k) {
        const int64_t id = base + k * kCopyBlock;
        if (id < total) {
            int64_t xo;
            offsets_of<RANK>(dm, id, &xo, &yo[k]);
            v[k] = x[xo];
        }
    }
#pragma unroll
    for (int k = 0; k < kCopyItems; ++k)
        if (base + k * kCopyBlock < total) y[yo[k]] = v[k];
}

// Both sides dense in the same order: one 128-bit non-temporal load and store per thread, the
// fastest read + write stream this device gives (about 6.2 TB/s; what the scans and other
// two-way streams of the library are measured against).  `vectors` 16-byte units.
__global__ __launch_bounds__(kCopyBlock) void copy_dense(const Vec<uint32_t, 4>* __restrict__ x, Vec<uint32_t, 4>* __restrict__ y, int64_t vectors) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * kCopyBlock + threadIdx.x;
    if (i < vectors) store_stream(y + i, load_stream(x + i));
}

template <typename E, int RANK>
__global__ __launch_bounds__(kCopyBlock) void fill_strided(E* __restrict__ y, DimMap2 dm, int64_t total, E value) {
    const int64_t base = static_cast<int64_t>(blockIdx.x) * (kCopyBlock * kCopyItems) + threadIdx.x;
#pragma unroll
    for (int k = 0; k < kCopyItems; ++k) {
        const int64_t id = base + k * kCopyBlock;
        if (id < total) {
            int64_t xo, yo;
            offsets_of<RANK>(dm, id, &xo, &yo);
            y[yo] = value;
        }
    }
}

template <typename F>
int dispatch_width(size_t bytes, F&& f) {
    switch (bytes) {
    case 1: return f(uint8_t());
    case 2: return f(uint16_t());
    case 4: return f(uint32_t());
    case 8: return f(uint64_t());
    case 16: return f(Vec<uint32_t, 4>());
    default: return DLFX_ERR_UNSUPPORTED_DTYPE;
    }
}

template <typename F>
int dispatch_rank(int rank, F&& f) {
    switch (rank) {
    case 0: case 1: return f(std::integral_constant<int, 1>());
    case 2: return f(std::integral_constant<int, 2>());
    case 3: return f(std::integral_constant<int, 3>());
    case 4: return f(std::integral_constant<int, 4>());
    default: return f(std::integral_constant<int, kMaxRank>());
    }
}

}  // namespace
}  // namespace dlfx

using namespace dlfx;

extern "C" int dlfx_copy(dlfx_stream_t stream, int dtype, int rank, const int64_t* dims,
                         const void* x, int64_t x_offset, const int64_t* x_strides,
                         void* y, int64_t y_offset, const int64_t* y_strides) {
    if (!x || !y) return DLFX_ERR_INVALID_ARGUMENT;
    if (!view_ok(rank, dims, x_strides) || !view_ok(rank, dims, y_strides)) return DLFX_ERR_INVALID_ARGUMENT;
    const size_t width = dtype_size(dtype);
    if (width == 0) return DLFX_ERR_UNSUPPORTED_DTYPE;
    DimMap2 dm;
    if (!make_dim_map2(rank, dims, x_strides, y_strides, &dm)) return DLFX_ERR_RANK;
    const int64_t total = view_size(rank, dims);
    const int64_t blocks = ceil_div(total, kCopyBlock * kCopyItems);
    if (blocks > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const char* xp = static_cast<const char*>(x) + x_offset * static_cast<int64_t>(width);
    char* yp = static_cast<char*>(y) + y_offset * static_cast<int64_t>(width);
    if (dm.rank == 0 || (dm.rank == 1 && dm.xs[0] == 1 && dm.ys[0] == 1)) {
        // both sides dense in the same order: a streaming copy kernel when everything is a
        // whole number of aligned 16-byte vectors, else one device-to-device copy
        if (xp == yp) return DLFX_OK;
        const size_t bytes = static_cast<size_t>(total) * width;
        const bool vectors = bytes % 16 == 0 && reinterpret_cast<uintptr_t>(xp) % 16 == 0 && reinterpret_cast<uintptr_t>(yp) % 16 == 0;
        if (vectors && ceil_div(static_cast<int64_t>(bytes / 16), kCopyBlock) <= 0x7fffffffLL) {
            const int64_t count = static_cast<int64_t>(bytes / 16);
            copy_dense<<<dim3(static_cast<unsigned>(ceil_div(count, kCopyBlock))), dim3(kCopyBlock), 0, s>>>(
                reinterpret_cast<const Vec<uint32_t, 4>*>(xp), reinterpret_cast<Vec<uint32_t, 4>*>(yp), count);
            DLFX_CHECK_LAUNCH();
            return DLFX_OK;
        }
        hipError_t e = hipMemcpyAsync(yp, xp, bytes, hipMemcpyDeviceToDevice, s);
        if (e != hipSuccess) return record_hip_error(e);
        return DLFX_OK;
    }
    return dispatch_width(width, [&](auto tag) {
        using E = decltype(tag);
        return dispatch_rank(dm.rank, [&](auto r) {
            constexpr int R = decltype(r)::value;
            copy_strided<E, R><<<dim3(static_cast<unsigned>(blocks)), dim3(kCopyBlock), 0, s>>>(
                reinterpret_cast<const E*>(xp), reinterpret_cast<E*>(yp), dm, total);
            DLFX_CHECK_LAUNCH();
            return static_cast<int>(DLFX_OK);
        });
    });
}

extern "C" int dlfx_fill(dlfx_stream_t stream, int dtype, int rank, const int64_t* dims, const int64_t* strides,
                         void* x, int64_t x_offset, const void* value) {
    if (!x || !value) return DLFX_ERR_INVALID_ARGUMENT;
    if (!view_ok(rank, dims, strides)) return DLFX_ERR_INVALID_ARGUMENT;
    const size_t width = dtype_size(dtype);
    if (width == 0) return DLFX_ERR_UNSUPPORTED_DTYPE;
    DimMap2 dm;
    if (!make_dim_map2(rank, dims, strides, strides, &dm)) return DLFX_ERR_RANK;
    const int64_t total = view_size(rank, dims);
    const int64_t blocks = ceil_div(total, kCopyBlock * kCopyItems);
    if (blocks > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    char* xp = static_cast<char*>(x) + x_offset * static_cast<int64_t>(width);
    return dispatch_width(width, [&](auto tag) {
        using E = decltype(tag);
        E v;
        std::memcpy(&v, value, sizeof(E));           // the element is read before the call returns
        return dispatch_rank(dm.rank, [&](auto r) {
            constexpr int R = decltype(r)::value;
            fill_strided<E, R><<<dim3(static_cast<unsigned>(blocks)), dim3(kCopyBlock), 0, s>>>(
                reinterpret_cast<E*>(xp), dm, total, v);
            DLFX_CHECK_LAUNCH();
            return static_cast<int>(DLFX_OK);
        });
    });
}
