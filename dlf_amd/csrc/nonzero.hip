// gather_indices: the coordinate list of the non-zero elements of a tensor, from the
// running count of non-zero elements (second half of nonzero(),
// dlf/include/tensor/reduce.h:381-418 on the host, gpgpu/src/kernels/dnn/xgather.cl:226-271
// for the device contract).  One thread per element: reading the counts is the traffic,
// the coordinates of the (usually few) non-zero elements are scattered writes.
#include "common.hip.h"

namespace dlfx {
namespace {

constexpr int kBlock = 256;

struct Extents {
    int rank;
    int32_t dims[kMaxRank];
};

// Each thread takes kPer consecutive elements: 128-bit loads of their counts, the count
// before them from the neighbouring lane (or memory at a wave's first lane), the coordinates
// of the first element by division and of the others by stepping the innermost coordinate.
constexpr int kPer = 4;

// RANK: the tensor's rank when it is 1 to 4 (the loops over dimensions then unroll to exactly
// that many steps and the coordinates of an element leave in one store where they are
// adjacent), 0 for any rank up to kMaxRank.
template <bool VEC, int RANK>
__global__ __launch_bounds__(kBlock) void gather_indices_kernel(int64_t m, int64_t n, int row_major, Extents ext,
                                                                const int32_t* __restrict__ counts,
                                                                int32_t* __restrict__ out) {
    const int64_t i0 = (static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x) * kPer;
    int32_t c[kPer];
    if (VEC && i0 + kPer <= m) {
        Vec<int32_t, 4> v[kPer / 4];
#pragma unroll
        for (int q = 0; q < kPer / 4; ++q) v[q] = load_stream(reinterpret_cast<const Vec<int32_t, 4>*>(counts + i0) + q);
#pragma unroll
        for (int e = 0; e < kPer; ++e) c[e] = v[e / 4].v[e % 4];
    } else {
#pragma unroll
        for (int e = 0; e < kPer; ++e) c[e] = i0 + e < m ? counts[i0 + e] : (e ? c[e - 1] : 0);     // past the end: no further non-zero element
    }
    // the count just before this thread's elements
    int32_t before = __shfl_up(c[kPer - 1], 1, kWave);
    if (lane_id() == 0) before = (i0 == 0 || i0 > m) ? 0 : counts[i0 - 1];

    // coordinates of element i0
    constexpr int SLOTS = RANK ? RANK : kMaxRank;
    const int rank = RANK ? RANK : ext.rank;
    int32_t coord[SLOTS];
    if (m <= 0xffffffffLL) {
        // 32-bit division is several times cheaper than 64-bit division here
        // (loops run over all kMaxRank slots so that the coordinates stay in registers)
        uint32_t rest = static_cast<uint32_t>(i0);
#pragma unroll
        for (int j = SLOTS - 1; j >= 0; --j) {
            coord[j] = 0;
            if (j < rank) {          // the same for every thread: dimensions past the rank cost nothing
                const uint32_t d = static_cast<uint32_t>(ext.dims[j]);
                const uint32_t q = rest / d;
                coord[j] = static_cast<int32_t>(rest - q * d);
                rest = q;
            }
        }
    } else {
        int64_t rest = i0;
#pragma unroll
        for (int j = SLOTS - 1; j >= 0; --j) {
            coord[j] = 0;
            if (j < rank) {
                const int64_t d = ext.dims[j];
                const int64_t q = rest / d;
                coord[j] = static_cast<int32_t>(rest - q * d);
                rest = q;
            }
        }
    }
    if (i0 >= m) return;
    if (__ballot(c[kPer - 1] != before) == 0ull) return;      // no lane of this wave holds a non-zero element
    int32_t prev = before;
#pragma unroll
    for (int e = 0; e < kPer; ++e) {
        if (i0 + e >= m) break;
        const int32_t curr = c[e];
        // counts that do not belong to this n are never written outside [rank, n]
        if (curr != prev && prev >= 0 && prev < n) {
            int32_t* cell = out + static_cast<int64_t>(prev) * rank;
            bool stored = false;
            if constexpr (RANK == 2 || RANK == 4) {
                // the coordinates of one element are adjacent: one 8- or 16-byte store
                if (!row_major && reinterpret_cast<uintptr_t>(cell) % (RANK * 4) == 0) {
                    Vec<int32_t, RANK> v;
#pragma unroll
                    for (int j = 0; j < RANK; ++j) v.v[j] = coord[j];
                    *reinterpret_cast<Vec<int32_t, RANK>*>(cell) = v;
                    stored = true;
                }
            }
            if (!stored) {
#pragma unroll
                for (int j = 0; j < SLOTS; ++j) {
                    if (j < rank) {
                        if (row_major) out[n * j + prev] = coord[j];
                        else cell[j] = coord[j];
                    }
                }
            }
        }
        prev = curr;
        // step to the next element in row-major order
        bool carry = true;
#pragma unroll
        for (int j = SLOTS - 1; j >= 0; --j) {
            if (j < rank && carry) {
                carry = ++coord[j] >= ext.dims[j];
                if (carry) coord[j] = 0;
            }
        }
    }
}

}  // namespace
}  // namespace dlfx

using namespace dlfx;

extern "C" int dlfx_gather_indices(dlfx_stream_t stream, int64_t m, int64_t n, int row_major,
                                   int rank, const int64_t* dims,
                                   const int32_t* indices, int64_t indices_offset,
                                   int32_t* output, int64_t output_offset) {
    if (!indices || !output || m <= 0 || n < 0 || rank < 1 || !dims) return DLFX_ERR_INVALID_ARGUMENT;
    if (rank > kMaxRank) return DLFX_ERR_RANK;
    Extents ext;
    ext.rank = rank;
    int64_t size = 1;
    for (int j = 0; j < kMaxRank; ++j) {
        const int64_t d = j < rank ? dims[j] : 1;
        if (d <= 0 || d > 0x7fffffffLL) return DLFX_ERR_INVALID_ARGUMENT;
        ext.dims[j] = static_cast<int32_t>(d);
        size *= d;
    }
    if (size != m) return DLFX_ERR_INVALID_ARGUMENT;
    if (n == 0) return DLFX_OK;
    const int64_t blocks = ceil_div(m, static_cast<int64_t>(kBlock) * kPer);
    if (blocks > 0x7fffffffLL) return DLFX_ERR_TOO_LARGE;
    const int32_t* counts = indices + indices_offset;
    const dim3 grid(static_cast<unsigned>(blocks)), block(kBlock);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool vec = reinterpret_cast<uintptr_t>(counts) % 16 == 0;
#define DLFX_GATHER(RANK)                                                                                                       \
    do {                                                                                                                        \
        if (vec) gather_indices_kernel<true, RANK><<<grid, block, 0, s>>>(m, n, row_major ? 1 : 0, ext, counts, output + output_offset);  \
        else gather_indices_kernel<false, RANK><<<grid, block, 0, s>>>(m, n, row_major ? 1 : 0, ext, counts, output + output_offset);    \
    } while (0)
    switch (rank) {
    case 1: DLFX_GATHER(1); break;
    case 2: DLFX_GATHER(2); break;
    case 3: DLFX_GATHER(3); break;
    case 4: DLFX_GATHER(4); break;
    default: DLFX_GATHER(0); break;
    }
#undef DLFX_GATHER
    DLFX_CHECK_LAUNCH();
    return DLFX_OK;
}
