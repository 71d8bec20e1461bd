// Host veneer: dlf's gpgpu::dnn entry points for the axis primitives, forwarding
// to the C ABI in dlfx.h.  Signatures follow gpgpu/include/gdnn.h:108-182 so
// that dlf's tensor front-ends (dlf/include/tensor/reduce_detail.h:91-101,
// 134-147, 244-253; reorder_detail.h:617-627, 667-677, 951-963, 1062-1073)
// compile against it unchanged: sizes and strides are std::vector<size_t>
// (negative steps wrapped), scratch comes from the context's temporary-buffer
// stack, failures surface as exceptions, and `event`, when given, brackets the
// work of the call.
#pragma once

#include <cstdint>
#include <string>
#include <type_traits>
#include <vector>

#include <complex>

#include "dlfx.h"
#include "gblas_half.h"
#include "gpgpu.h"

namespace gpgpu { namespace dnn {

namespace detail {

template <typename T> struct dtype_of;
template <> struct dtype_of<float>   { static constexpr int value = DLFX_F32; };
template <> struct dtype_of<double>  { static constexpr int value = DLFX_F64; };
template <> struct dtype_of<int32_t> { static constexpr int value = DLFX_I32; };
template <> struct dtype_of<int64_t> { static constexpr int value = DLFX_I64; };
template <> struct dtype_of<int16_t> { static constexpr int value = DLFX_I16; };
template <> struct dtype_of<blas::half> { static constexpr int value = DLFX_F16; };
template <> struct dtype_of<std::complex<float>>  { static constexpr int value = DLFX_C64; };     // float2
template <> struct dtype_of<std::complex<double>> { static constexpr int value = DLFX_C128; };    // double2

// size_t strides that wrapped for a negative step come back as the negative number
inline std::vector<int64_t> signed_vec(const std::vector<size_t>& v) {
    std::vector<int64_t> r(v.size());
    for (size_t i = 0; i < v.size(); ++i) r[i] = static_cast<int64_t>(v[i]);
    return r;
}

struct EventScope {
    const Queue& q;
    Event* e;
    EventScope(const Queue& queue, Event* event) : q(queue), e(event) {
        if (e) check_hip(hipEventRecord(e->start(), q.stream()), "hipEventRecord");
    }
    void done() { if (e) check_hip(hipEventRecord(e->end(), q.stream()), "hipEventRecord"); }
};

}  // namespace detail

template <typename T>
void reduce(const std::string& name, const size_t m, const size_t n,
            const std::vector<size_t>& x_dims, const std::vector<size_t>& x_strides,
            const Buffer<T>& x_buffer, const size_t x_offset,
            const std::vector<size_t>& y_dims, const std::vector<size_t>& y_strides,
            Buffer<T>& y_buffer, const size_t y_offset,
            const Queue& queue = gpgpu::current::queue(), Event* event = nullptr) {
    const int dt = detail::dtype_of<T>::value;
    auto xd = detail::signed_vec(x_dims), xs = detail::signed_vec(x_strides);
    auto yd = detail::signed_vec(y_dims), ys = detail::signed_vec(y_strides);
    auto tmp = queue.context().getTemporaryBuffer<char>(dlfx_reduce_scratch_bytes(dt, m, n));
    detail::EventScope ev(queue, event);
    check_status(dlfx_reduce(queue.stream(), name.c_str(), dt, m, n,
                             static_cast<int>(xd.size()), xd.data(), xs.data(), x_buffer.data(), x_offset,
                             static_cast<int>(yd.size()), yd.data(), ys.data(), y_buffer.data(), y_offset,
                             tmp.bytes(), tmp.byte_size()), "gpgpu::dnn::reduce");
    ev.done();
}

// Not in the reference: sum, max, first arg-maximum, log-sum-exp and the k best entries of
// every row of an [m, n] fp32 matrix in one launch (dlfx_logits_head).  Row r starts at
// x_offset + r * row_stride; outputs are dense and any may be null.
inline void logits_head(const size_t m, const size_t n,
                        const Buffer<float>& x_buffer, const size_t x_offset, const size_t row_stride,
                        Buffer<float>* sum, Buffer<float>* max, Buffer<int>* argmax, Buffer<float>* log_sum_exp,
                        const size_t k, Buffer<float>* best_values, Buffer<int>* best_indices,
                        const Queue& queue = gpgpu::current::queue(), Event* event = nullptr) {
    detail::EventScope ev(queue, event);
    check_status(dlfx_logits_head(queue.stream(), DLFX_F32, m, n, x_buffer.data(), x_offset, row_stride,
                                  sum ? sum->data() : nullptr, max ? max->data() : nullptr,
                                  argmax ? argmax->data() : nullptr, log_sum_exp ? log_sum_exp->data() : nullptr, k,
                                  best_values ? best_values->data() : nullptr, best_indices ? best_indices->data() : nullptr),
                 "gpgpu::dnn::logits_head");
    ev.done();
}

template <typename T>
void arg_reduce(const std::string& name, const size_t n, const size_t k,
                const std::vector<size_t>& x_dims, const std::vector<size_t>& x_strides,
                const Buffer<T>& x_buffer, const size_t x_offset,
                const std::vector<size_t>& y_dims, const std::vector<size_t>& y_strides,
                Buffer<int>& y_buffer, const size_t y_offset,
                const Queue& queue = gpgpu::current::queue(), Event* event = nullptr) {
    const int dt = detail::dtype_of<T>::value;
    auto xd = detail::signed_vec(x_dims), xs = detail::signed_vec(x_strides);
    auto yd = detail::signed_vec(y_dims), ys = detail::signed_vec(y_strides);
    auto tmp = queue.context().getTemporaryBuffer<char>(dlfx_arg_reduce_scratch_bytes(dt, n, k));
    detail::EventScope ev(queue, event);
    check_status(dlfx_arg_reduce(queue.stream(), name.c_str(), dt, DLFX_I32, n, k,
                                 static_cast<int>(xd.size()), xd.data(), xs.data(), x_buffer.data(), x_offset,
                                 static_cast<int>(yd.size()), yd.data(), ys.data(), y_buffer.data(), y_offset,
                                 tmp.bytes(), tmp.byte_size()), "gpgpu::dnn::arg_reduce");
    ev.done();
}

template <typename T>
void scan(const std::string& name, const size_t m, const size_t n,
          const bool exclusive, const std::vector<size_t>& dims,
          const Buffer<T>& x_buffer, const size_t x_offset, const std::vector<size_t>& x_strides,
          Buffer<T>& y_buffer, const size_t y_offset, const std::vector<size_t>& y_strides,
          const Queue& queue = gpgpu::current::queue(), Event* event = nullptr) {
    const int dt = detail::dtype_of<T>::value;
    auto d = detail::signed_vec(dims), xs = detail::signed_vec(x_strides), ys = detail::signed_vec(y_strides);
    auto tmp = queue.context().getTemporaryBuffer<char>(dlfx_scan_scratch_bytes(dt, m, n));
    detail::EventScope ev(queue, event);
    check_status(dlfx_scan(queue.stream(), name.c_str(), dt, m, n, exclusive ? 1 : 0,
                           static_cast<int>(d.size()), d.data(), x_buffer.data(), x_offset, xs.data(),
                           y_buffer.data(), y_offset, ys.data(), tmp.bytes(), tmp.byte_size()), "gpgpu::dnn::scan");
    ev.done();
}

template <typename T>
void sort(const int dir, const std::vector<size_t>& dims,
          const Buffer<T>& x_buffer, const size_t x_offset, const std::vector<size_t>& x_strides,
          Buffer<T>& y_buffer, const size_t y_offset, const std::vector<size_t>& y_strides,
          const Queue& queue = gpgpu::current::queue(), Event* event = nullptr) {
    const int dt = detail::dtype_of<T>::value;
    auto d = detail::signed_vec(dims), xs = detail::signed_vec(x_strides), ys = detail::signed_vec(y_strides);
    const int64_t n = d.empty() ? 1 : d.back();
    int64_t m = 1;
    for (size_t i = 0; i + 1 < d.size(); ++i) m *= d[i];
    auto tmp = queue.context().getTemporaryBuffer<char>(dlfx_sort_scratch_bytes(dt, m, n));
    detail::EventScope ev(queue, event);
    check_status(dlfx_sort(queue.stream(), dir, dt, static_cast<int>(d.size()), d.data(),
                           x_buffer.data(), x_offset, xs.data(), y_buffer.data(), y_offset, ys.data(),
                           tmp.bytes(), tmp.byte_size()), "gpgpu::dnn::sort");
    ev.done();
}

template <typename T>
void argsort(const int dir, const std::vector<size_t>& dims,
             const Buffer<T>& x_buffer, const size_t x_offset, const std::vector<size_t>& x_strides,
             Buffer<int32_t>& i_buffer, const size_t i_offset, const std::vector<size_t>& i_strides,
             const Queue& queue = gpgpu::current::queue(), Event* event = nullptr) {
    const int dt = detail::dtype_of<T>::value;
    auto d = detail::signed_vec(dims), xs = detail::signed_vec(x_strides), is = detail::signed_vec(i_strides);
    const int64_t n = d.empty() ? 1 : d.back();
    int64_t m = 1;
    for (size_t i = 0; i + 1 < d.size(); ++i) m *= d[i];
    auto tmp = queue.context().getTemporaryBuffer<char>(dlfx_argsort_scratch_bytes(dt, m, n));
    detail::EventScope ev(queue, event);
    check_status(dlfx_argsort(queue.stream(), dir, dt, DLFX_I32, static_cast<int>(d.size()), d.data(),
                              x_buffer.data(), x_offset, xs.data(), nullptr, 0, nullptr,
                              i_buffer.data(), i_offset, is.data(), tmp.bytes(), tmp.byte_size()), "gpgpu::dnn::argsort");
    ev.done();
}

template <typename T>
void argsort(const int dir, const std::vector<size_t>& dims,
             const Buffer<T>& x_buffer, const size_t x_offset, const std::vector<size_t>& x_strides,
             Buffer<T>& y_buffer, const size_t y_offset, const std::vector<size_t>& y_strides,
             Buffer<int32_t>& i_buffer, const size_t i_offset, const std::vector<size_t>& i_strides,
             const Queue& queue = gpgpu::current::queue(), Event* event = nullptr) {
    const int dt = detail::dtype_of<T>::value;
    auto d = detail::signed_vec(dims), xs = detail::signed_vec(x_strides), ys = detail::signed_vec(y_strides),
         is = detail::signed_vec(i_strides);
    const int64_t n = d.empty() ? 1 : d.back();
    int64_t m = 1;
    for (size_t i = 0; i + 1 < d.size(); ++i) m *= d[i];
    auto tmp = queue.context().getTemporaryBuffer<char>(dlfx_argsort_scratch_bytes(dt, m, n));
    detail::EventScope ev(queue, event);
    check_status(dlfx_argsort(queue.stream(), dir, dt, DLFX_I32, static_cast<int>(d.size()), d.data(),
                              x_buffer.data(), x_offset, xs.data(), y_buffer.data(), y_offset, ys.data(),
                              i_buffer.data(), i_offset, is.data(), tmp.bytes(), tmp.byte_size()), "gpgpu::dnn::argsort");
    ev.done();
}

template <typename T>
void top_k(const size_t limit, const int dir,
           const std::vector<size_t>& x_dims, const std::vector<size_t>& y_dims,
           const Buffer<T>& x_buffer, const size_t x_offset, const std::vector<size_t>& x_strides,
           Buffer<T>& y_buffer, const size_t y_offset, const std::vector<size_t>& y_strides,
           Buffer<int32_t>& i_buffer, const size_t i_offset, const std::vector<size_t>& i_strides,
           const Queue& queue = gpgpu::current::queue(), Event* event = nullptr) {
    const int dt = detail::dtype_of<T>::value;
    auto xd = detail::signed_vec(x_dims), yd = detail::signed_vec(y_dims);
    auto xs = detail::signed_vec(x_strides), ys = detail::signed_vec(y_strides), is = detail::signed_vec(i_strides);
    const int64_t n = xd.empty() ? 1 : xd.back();
    int64_t m = 1;
    for (size_t i = 0; i + 1 < xd.size(); ++i) m *= xd[i];
    auto tmp = queue.context().getTemporaryBuffer<char>(dlfx_top_k_scratch_bytes(dt, m, n, limit));
    detail::EventScope ev(queue, event);
    check_status(dlfx_top_k(queue.stream(), limit, dir, dt, DLFX_I32, static_cast<int>(xd.size()), xd.data(), yd.data(),
                            x_buffer.data(), x_offset, xs.data(), y_buffer.data(), y_offset, ys.data(),
                            i_buffer.data(), i_offset, is.data(), tmp.bytes(), tmp.byte_size()), "gpgpu::dnn::top_k");
    ev.done();
}

// gpgpu/include/gdnn.h:253-264: in place on the rows of a contiguous [m, n] matrix
namespace detail {
template <typename T>
void softmax_family(const char* name, const size_t m, const size_t n, const Buffer<T>& x_buffer, const size_t x_offset,
                    Buffer<T>& y_buffer, const size_t y_offset, const Queue& queue, Event* event) {
    const int dt = dtype_of<T>::value;
    auto tmp = queue.context().getTemporaryBuffer<char>(dlfx_softmax_scratch_bytes(dt, m, n));      // only few, long rows need any
    EventScope ev(queue, event);
    check_status(dlfx_softmax(queue.stream(), name, dt, m, n, x_buffer.data(), x_offset,
                              y_buffer.data(), y_offset, tmp.bytes(), tmp.byte_size()), name);
    ev.done();
}
}  // namespace detail
template <typename T>
void softmax(const size_t m, const size_t n, Buffer<T>& x_buffer, const size_t x_offset,
             const Queue& queue = gpgpu::current::queue(), Event* event = nullptr) {
    detail::softmax_family("softmax", m, n, x_buffer, x_offset, x_buffer, x_offset, queue, event);
}
// Out of place (no counterpart in the reference, whose routine works in place only): rows of the
// contiguous [m, n] matrix at x go to y, which may be the same buffer.
template <typename T>
void softmax(const size_t m, const size_t n, const Buffer<T>& x_buffer, const size_t x_offset,
        Buffer<T>& y_buffer, const size_t y_offset,
        const Queue& queue = gpgpu::current::queue(), Event* event = nullptr) {
    detail::softmax_family("softmax", m, n, x_buffer, x_offset, y_buffer, y_offset, queue, event);
}
template <typename T>
void logsoftmax(const size_t m, const size_t n, Buffer<T>& x_buffer, const size_t x_offset,
                const Queue& queue = gpgpu::current::queue(), Event* event = nullptr) {
    detail::softmax_family("logsoftmax", m, n, x_buffer, x_offset, x_buffer, x_offset, queue, event);
}
// Out of place (no counterpart in the reference, whose routine works in place only): rows of the
// contiguous [m, n] matrix at x go to y, which may be the same buffer.
template <typename T>
void logsoftmax(const size_t m, const size_t n, const Buffer<T>& x_buffer, const size_t x_offset,
        Buffer<T>& y_buffer, const size_t y_offset,
        const Queue& queue = gpgpu::current::queue(), Event* event = nullptr) {
    detail::softmax_family("logsoftmax", m, n, x_buffer, x_offset, y_buffer, y_offset, queue, event);
}
template <typename T>
void hardmax(const size_t m, const size_t n, Buffer<T>& x_buffer, const size_t x_offset,
             const Queue& queue = gpgpu::current::queue(), Event* event = nullptr) {
    detail::softmax_family("hardmax", m, n, x_buffer, x_offset, x_buffer, x_offset, queue, event);
}
// Out of place (no counterpart in the reference, whose routine works in place only): rows of the
// contiguous [m, n] matrix at x go to y, which may be the same buffer.
template <typename T>
void hardmax(const size_t m, const size_t n, const Buffer<T>& x_buffer, const size_t x_offset,
        Buffer<T>& y_buffer, const size_t y_offset,
        const Queue& queue = gpgpu::current::queue(), Event* event = nullptr) {
    detail::softmax_family("hardmax", m, n, x_buffer, x_offset, y_buffer, y_offset, queue, event);
}

// gpgpu/include/gdnn.h:14-17 (routine xcopy.cpp:59-81): strided view to strided view
template <typename T>
void copy(const size_t n, const std::vector<size_t>& dims,
          const Buffer<T>& x_buffer, const size_t x_offset, const std::vector<size_t>& x_stride,
          Buffer<T>& y_buffer, const size_t y_offset, const std::vector<size_t>& y_stride,
          const Queue& queue = gpgpu::current::queue(), Event* event = nullptr) {
    auto d = detail::signed_vec(dims), xs = detail::signed_vec(x_stride), ys = detail::signed_vec(y_stride);
    size_t size = 1;
    for (auto e : dims) size *= e;
    if (size != n || x_stride.size() != dims.size() || y_stride.size() != dims.size())
        throw LogicError("gpgpu::dnn::copy: extents, strides and n disagree");
    detail::EventScope ev(queue, event);
    if (n != 0)            // an empty view: nothing to move
        check_status(dlfx_copy(queue.stream(), detail::dtype_of<T>::value, static_cast<int>(d.size()), d.data(),
                               x_buffer.data(), x_offset, xs.data(), y_buffer.data(), y_offset, ys.data()), "gpgpu::dnn::copy");
    ev.done();
}

// gpgpu/include/gdnn.h:9-11 (xcopy.cpp:15-55, kernel xcopy.cl:8-26): y_size elements; a shorter x repeats
template <typename T>
void copy(const size_t x_size, const Buffer<T>& x_buffer, const size_t x_offset,
          const size_t y_size, Buffer<T>& y_buffer, const size_t y_offset,
          const Queue& queue = gpgpu::current::queue(), Event* event = nullptr) {
    if (x_size == 0 || y_size == 0) throw RuntimeErrorCode(DLFX_ERR_INVALID_ARGUMENT, "gpgpu::dnn::copy");
    detail::EventScope ev(queue, event);
    const int dt = detail::dtype_of<T>::value;
    if (x_size >= y_size) {
        const int64_t d[1] = {static_cast<int64_t>(y_size)}, one[1] = {1};
        check_status(dlfx_copy(queue.stream(), dt, 1, d, x_buffer.data(), x_offset, one, y_buffer.data(), y_offset, one),
                     "gpgpu::dnn::copy");
    } else {
        const size_t reps = y_size / x_size, rest = y_size % x_size;
        const int64_t d[2] = {static_cast<int64_t>(reps), static_cast<int64_t>(x_size)};
        const int64_t xs[2] = {0, 1}, ys[2] = {static_cast<int64_t>(x_size), 1};
        check_status(dlfx_copy(queue.stream(), dt, 2, d, x_buffer.data(), x_offset, xs, y_buffer.data(), y_offset, ys),
                     "gpgpu::dnn::copy");
        if (rest) {
            const int64_t dr[1] = {static_cast<int64_t>(rest)}, one[1] = {1};
            check_status(dlfx_copy(queue.stream(), dt, 1, dr, x_buffer.data(), x_offset, one, y_buffer.data(),
                                   y_offset + reps * x_size, one), "gpgpu::dnn::copy");
        }
    }
    ev.done();
}

// gpgpu/include/gdnn.h:20-22
template <typename T>
void fill(const size_t n, Buffer<T>& x_buffer, const size_t x_offset, const T value,
          const Queue& queue = gpgpu::current::queue(), Event* event = nullptr) {
    const int64_t d[1] = {static_cast<int64_t>(n)}, one[1] = {1};
    detail::EventScope ev(queue, event);
    if (n != 0)
        check_status(dlfx_fill(queue.stream(), detail::dtype_of<T>::value, 1, d, one, x_buffer.data(), x_offset, &value),
                     "gpgpu::dnn::fill");
    ev.done();
}

// gpgpu/include/gdnn.h:24-26
template <typename T>
void fill(const size_t n, const std::vector<size_t>& dims, const std::vector<size_t>& strides,
          Buffer<T>& x_buffer, const size_t x_offset, const T value,
          const Queue& queue = gpgpu::current::queue(), Event* event = nullptr) {
    auto d = detail::signed_vec(dims), st = detail::signed_vec(strides);
    size_t size = 1;
    for (auto e : dims) size *= e;
    if (size != n || strides.size() != dims.size()) throw LogicError("gpgpu::dnn::fill: extents, strides and n disagree");
    detail::EventScope ev(queue, event);
    if (n != 0)
        check_status(dlfx_fill(queue.stream(), detail::dtype_of<T>::value, static_cast<int>(d.size()), d.data(), st.data(),
                               x_buffer.data(), x_offset, &value), "gpgpu::dnn::fill");
    ev.done();
}

// gpgpu/include/gdnn.h:147-155
template <typename T>
void merge(const int dir,
           const std::vector<size_t>& x_dims, const std::vector<size_t>& x_strides,
           const Buffer<T>& x_buffer, const size_t x_offset,
           const std::vector<size_t>& y_dims, const std::vector<size_t>& y_strides,
           const Buffer<T>& y_buffer, const size_t y_offset,
           const std::vector<size_t>& z_dims, const std::vector<size_t>& z_strides,
           Buffer<T>& z_buffer, const size_t z_offset,
           const Queue& queue = gpgpu::current::queue(), Event* event = nullptr) {
    const int dt = detail::dtype_of<T>::value;
    if (x_dims.size() != z_dims.size() || y_dims.size() != z_dims.size() || z_dims.empty())
        throw LogicError("gpgpu::dnn::merge: ranks differ");
    auto xd = detail::signed_vec(x_dims), xs = detail::signed_vec(x_strides);
    auto yd = detail::signed_vec(y_dims), ys = detail::signed_vec(y_strides);
    auto zd = detail::signed_vec(z_dims), zs = detail::signed_vec(z_strides);
    const size_t n = z_dims.back();
    size_t m = 1;
    for (size_t i = 0; i + 1 < z_dims.size(); ++i) m *= z_dims[i];
    auto tmp = queue.context().getTemporaryBuffer<char>(dlfx_merge_scratch_bytes(dt, m, n));
    detail::EventScope ev(queue, event);
    check_status(dlfx_merge(queue.stream(), dir, dt, static_cast<int>(zd.size()),
                            xd.data(), xs.data(), x_buffer.data(), x_offset,
                            yd.data(), ys.data(), y_buffer.data(), y_offset,
                            zd.data(), zs.data(), z_buffer.data(), z_offset,
                            tmp.bytes(), tmp.byte_size()), "gpgpu::dnn::merge");
    ev.done();
}

// gpgpu/include/gdnn.h:116-122
template <typename T>
void count(const size_t m, const size_t n, const T value,
           const std::vector<size_t>& x_dims, const std::vector<size_t>& x_strides,
           const Buffer<T>& x_buffer, const size_t x_offset,
           const std::vector<size_t>& y_dims, const std::vector<size_t>& y_strides,
           Buffer<int>& y_buffer, const size_t y_offset,
           const Queue& queue = gpgpu::current::queue(), Event* event = nullptr) {
    const int dt = detail::dtype_of<T>::value;
    auto xd = detail::signed_vec(x_dims), xs = detail::signed_vec(x_strides);
    auto yd = detail::signed_vec(y_dims), ys = detail::signed_vec(y_strides);
    auto tmp = queue.context().getTemporaryBuffer<char>(dlfx_count_scratch_bytes(dt, m, n));
    detail::EventScope ev(queue, event);
    check_status(dlfx_count(queue.stream(), dt, m, n, &value,
                            static_cast<int>(xd.size()), xd.data(), xs.data(), x_buffer.data(), x_offset,
                            static_cast<int>(yd.size()), yd.data(), ys.data(), y_buffer.data(), y_offset,
                            tmp.bytes(), tmp.byte_size()), "gpgpu::dnn::count");
    ev.done();
}

// gpgpu/include/gdnn.h:131-136
template <typename T>
void scan_nonzero(const size_t m, const size_t n,
                  const bool exclusive, const std::vector<size_t>& dims,
                  const Buffer<T>& x_buffer, const size_t x_offset, const std::vector<size_t>& x_strides,
                  Buffer<int32_t>& y_buffer, const size_t y_offset, const std::vector<size_t>& y_strides,
                  const Queue& queue = gpgpu::current::queue(), Event* event = nullptr) {
    const int dt = detail::dtype_of<T>::value;
    auto d = detail::signed_vec(dims), xs = detail::signed_vec(x_strides), ys = detail::signed_vec(y_strides);
    auto tmp = queue.context().getTemporaryBuffer<char>(dlfx_scan_nonzero_scratch_bytes(dt, m, n));
    detail::EventScope ev(queue, event);
    check_status(dlfx_scan_nonzero(queue.stream(), dt, m, n, exclusive ? 1 : 0,
                                   static_cast<int>(d.size()), d.data(), x_buffer.data(), x_offset, xs.data(),
                                   y_buffer.data(), y_offset, ys.data(), tmp.bytes(), tmp.byte_size()),
                 "gpgpu::dnn::scan_nonzero");
    ev.done();
}

// gpgpu/include/gdnn.h:328-332
inline void gather_indices(const size_t m, const size_t n, const bool row_major,
                           const std::vector<size_t>& dims,
                           const Buffer<int32_t>& indices, const size_t indices_offset,
                           Buffer<int32_t>& output, const size_t output_offset,
                           const Queue& queue = gpgpu::current::queue(), Event* event = nullptr) {
    auto d = detail::signed_vec(dims);
    detail::EventScope ev(queue, event);
    check_status(dlfx_gather_indices(queue.stream(), m, n, row_major ? 1 : 0, static_cast<int>(d.size()), d.data(),
                                     indices.data(), indices_offset, output.data(), output_offset),
                 "gpgpu::dnn::gather_indices");
    ev.done();
}

}}  // namespace gpgpu::dnn
