// Host veneer: a compact DevTensor plus the tensor-level front-ends of the axis
// primitives, so that code written against dlf's tensor API for this path
// (reduce_sum(dev(X), {1}), argmax(X, axis), cumsum(X, axis, exclusive,
// reverse), sorted(X, axis), argsort(X, Y, I, axis), top_k(X, Y, I, k, axis))
// reads the same here.
//
// Follows dlf/include/tensor/shape.h:51-366, dlf/src/tensor/shape.cpp:21-135,
// 362-460 (Shape), dlf/include/tensor/device.h:14-234 (DevTensor), reduce.h:68-377,
// reduce_detail.h:9-38,149-165, reorder.h:439-513,1120-1300 (front-ends).  Only
// what the path needs is here; a tensor and its views share one gpgpu::Buffer.
#pragma once

#include <algorithm>
#include <cassert>
#include <initializer_list>
#include <limits>
#include <numeric>
#include <string>
#include <utility>
#include <vector>

#include "gdnn.h"

namespace dlf {

class shape_error : public std::logic_error {
public:
    using std::logic_error::logic_error;
};

namespace detail {
inline void norm_axis(const int rank, int& axis) {
    if (axis < 0) axis += rank;
    if (axis < 0 || axis >= rank) throw shape_error("axis has incorrect value");
}
inline void norm_axes(const int rank, std::vector<int>& axes, bool allow_duplicates = false) {
    for (auto& k : axes) norm_axis(rank, k);
    if (!allow_duplicates) {
        auto s = axes;
        std::sort(s.begin(), s.end());
        if (std::adjacent_find(s.begin(), s.end()) != s.end()) throw shape_error("axes has duplicates");
    }
}
}  // namespace detail

// Extents, strides (size_t: a negative step wraps, as in the reference) and an offset.
class Shape {
    std::vector<size_t> extents_, strides_;
    size_t offset_ = 0;
public:
    Shape() = default;
    Shape(std::initializer_list<size_t> e) : Shape(std::vector<size_t>(e)) {}
    explicit Shape(std::vector<size_t> e) : extents_(std::move(e)), strides_(extents_.size()) {
        size_t size = 1;
        for (size_t i = extents_.size(); i-- != 0;) {
            if (extents_[i] == 0) throw shape_error("extent must be positive");
            strides_[i] = size;
            size *= extents_[i];
        }
    }
    static Shape as_strided(std::vector<size_t> e, std::vector<size_t> s, size_t offset) {
        if (e.size() != s.size()) throw shape_error("as_strided: rank mismatch");
        Shape r;
        r.extents_ = std::move(e);
        r.strides_ = std::move(s);
        r.offset_ = offset;
        return r;
    }
    size_t rank() const noexcept { return extents_.size(); }
    size_t size() const noexcept { return std::accumulate(extents_.begin(), extents_.end(), size_t(1), std::multiplies<size_t>()); }
    size_t offset() const noexcept { return offset_; }
    const std::vector<size_t>& extents() const noexcept { return extents_; }
    const std::vector<size_t>& strides() const noexcept { return strides_; }
    size_t extent(int i) const { return extents_[i < 0 ? i + rank() : i]; }
    size_t stride(int i) const { return strides_[i < 0 ? i + rank() : i]; }
    bool operator==(const Shape& o) const noexcept { return extents_ == o.extents_; }
    bool operator!=(const Shape& o) const noexcept { return !(*this == o); }
    // Row-major dense: every stride is the product of the extents after it (shape.cpp:126-135).
    bool is_contiguous() const noexcept {
        size_t size = 1;
        for (size_t i = rank(); i-- != 0;) {
            if (extents_[i] != 1 && strides_[i] != size) return false;
            size *= extents_[i];
        }
        return true;
    }

    size_t linear_offset(size_t index) const noexcept {
        size_t off = offset_;
        for (size_t i = rank(); i-- != 0;) {
            off += (index % extents_[i]) * strides_[i];
            index /= extents_[i];
        }
        return off;
    }
    Shape transpose(const std::vector<size_t>& perm) const {
        std::vector<size_t> sorted = perm;
        std::sort(sorted.begin(), sorted.end());
        for (size_t i = 0; i < sorted.size(); ++i)
            if (sorted.size() != rank() || sorted[i] != i) throw shape_error("transpose: invalid permutation");
        std::vector<size_t> e(rank()), s(rank());
        for (size_t i = 0; i < rank(); ++i) { e[i] = extents_[perm[i]]; s[i] = strides_[perm[i]]; }
        return as_strided(std::move(e), std::move(s), offset_);
    }
    Shape transpose() const {
        if (rank() == 1) return as_strided({extents_[0], 1}, {strides_[0], 0}, offset_);
        std::vector<size_t> perm(rank());
        std::iota(perm.rbegin(), perm.rend(), size_t(0));
        return transpose(perm);
    }
    // One axis: [start, end) with a non-zero step, numpy/ONNX conventions (shape.cpp:386-460).
    Shape slice(int axis, int start, int end, int step = 1) const {
        detail::norm_axis(static_cast<int>(rank()), axis);
        if (step == 0) throw shape_error("slice: step cannot be 0");
        const int dim = static_cast<int>(extents_[axis]);
        auto clamp = [](int v, int lo, int hi) { return std::max(lo, std::min(hi, v)); };
        if (start < 0) start += dim;
        start = step < 0 ? clamp(start, 0, dim - 1) : clamp(start, 0, dim);
        if (end < 0) end += dim;
        end = step < 0 ? clamp(end, -1, dim) : clamp(end, 0, dim);
        int count = (end - start - (step < 0 ? -1 : 1)) / step + 1;
        if (count < 0) throw shape_error("slice: incorrect start and end value");
        if (count == 0) count = 1;
        Shape r = *this;
        r.extents_[axis] = static_cast<size_t>(count);
        r.strides_[axis] = strides_[axis] * static_cast<size_t>(static_cast<long long>(step));   // wraps for step < 0
        r.offset_ = offset_ + static_cast<size_t>(start) * strides_[axis];
        return r;
    }
};

// Row-major host tensor.
template <typename T>
class Tensor {
    Shape shape_;
    std::vector<T> data_;
public:
    Tensor() = default;
    explicit Tensor(Shape shape) : shape_(std::move(shape)), data_(shape_.size()) {}
    Tensor(Shape shape, std::initializer_list<T> v) : shape_(std::move(shape)), data_(v) {
        if (data_.size() != shape_.size()) throw shape_error("initializer does not match the shape");
    }
    Tensor(Shape shape, std::vector<T> v) : shape_(std::move(shape)), data_(std::move(v)) {
        if (data_.size() != shape_.size()) throw shape_error("data does not match the shape");
    }
    Tensor& range(T start = T(0)) { std::iota(data_.begin(), data_.end(), start); return *this; }
    const Shape& shape() const noexcept { return shape_; }
    size_t rank() const noexcept { return shape_.rank(); }
    size_t size() const noexcept { return data_.size(); }
    size_t extent(int i) const { return shape_.extent(i); }
    T* data() noexcept { return data_.data(); }
    const T* data() const noexcept { return data_.data(); }
    const std::vector<T>& values() const noexcept { return data_; }
    bool operator==(const Tensor& o) const { return shape_ == o.shape_ && data_ == o.data_; }
    bool operator!=(const Tensor& o) const { return !(*this == o); }
};

// Device tensor or view: a Shape over a shared gpgpu::Buffer.
template <typename T>
class DevTensor {
    Shape shape_;
    gpgpu::Buffer<T> data_;
public:
    using value_type = T;
    DevTensor() = default;
    explicit DevTensor(Shape shape) : shape_(std::move(shape)), data_(shape_.size()) {}
    DevTensor(Shape shape, gpgpu::Buffer<T> buffer) : shape_(std::move(shape)), data_(std::move(buffer)) {}
    explicit DevTensor(const Tensor<T>& host) : shape_(host.shape()), data_(host.size()) {
        data_.write(gpgpu::current::queue(), host.data(), host.size());
    }
    const Shape& shape() const noexcept { return shape_; }
    size_t rank() const noexcept { return shape_.rank(); }
    size_t size() const noexcept { return shape_.size(); }
    size_t extent(int i) const { return shape_.extent(i); }
    gpgpu::Buffer<T>& data() noexcept { return data_; }
    const gpgpu::Buffer<T>& data() const noexcept { return data_; }

    // (Re)allocate as a dense tensor of `shape`; storage is kept when it is large enough.
    void resize(const Shape& shape) {
        if (!data_ || data_.size() < shape.size()) data_ = gpgpu::Buffer<T>(shape.size());
        shape_ = Shape(shape.extents());
    }
    // Drops the storage; the tensor is empty afterwards (device.h: DevTensor::clear).
    void clear() {
        data_ = gpgpu::Buffer<T>();
        shape_ = Shape();
    }
    bool empty() const noexcept { return !data_; }
    DevTensor view(Shape shape) const { return DevTensor(std::move(shape), data_); }
    DevTensor transpose() const { return view(shape_.transpose()); }
    DevTensor transpose(const std::vector<size_t>& perm) const { return view(shape_.transpose(perm)); }
    DevTensor slice(int axis, int start, int end, int step = 1) const { return view(shape_.slice(axis, start, end, step)); }

    // Host copy of the viewed elements in row-major order.
    Tensor<T> read() const {
        std::vector<T> all(data_.size());
        data_.read(gpgpu::current::queue(), all.data(), all.size());
        std::vector<T> out(size());
        for (size_t i = 0; i < out.size(); ++i) out[i] = all[shape_.linear_offset(i)];
        return Tensor<T>(Shape(shape_.extents()), std::move(out));
    }
};

template <typename T>
inline DevTensor<T> dev(const Tensor<T>& host) { return DevTensor<T>(host); }

// ---------------------------------------------------------------- views
template <typename T>
DevTensor<T> moveaxis(const DevTensor<T>& X, int source, int destination) {
    const int rank = static_cast<int>(X.rank());
    detail::norm_axis(rank, source);
    detail::norm_axis(rank, destination);
    std::vector<size_t> order;
    for (int k = 0; k < rank; ++k)
        if (k != source) order.push_back(k);
    order.insert(order.begin() + destination, source);
    return X.transpose(order);
}

template <typename T>
DevTensor<T> flip(const DevTensor<T>& X, int axis) {
    return X.slice(axis, -1, std::numeric_limits<int>::lowest(), -1);
}

// ---------------------------------------------------------------- reduce
namespace detail {
template <typename T>
Shape prepare_reduce(const DevTensor<T>& X, DevTensor<T>& Y, std::vector<int> axes, bool keepdims, size_t* m, size_t* n) {
    const int rank = static_cast<int>(X.rank());
    norm_axes(rank, axes, true);
    auto reduced = [&](int i) { return axes.empty() || std::find(axes.begin(), axes.end(), i) != axes.end(); };
    std::vector<size_t> out_dims, perm;
    *m = *n = 1;
    for (int i = 0; i < rank; ++i) {
        if (!reduced(i)) { out_dims.push_back(X.extent(i)); perm.push_back(i); }
        else if (keepdims) out_dims.push_back(1);
    }
    for (int i = 0; i < rank; ++i) {
        if (reduced(i)) { perm.push_back(i); *n *= X.extent(i); }
        else *m *= X.extent(i);
    }
    Y.resize(Shape(out_dims));
    return X.shape().transpose(perm);
}
}  // namespace detail

template <typename T>
void reduce(const std::string& name, const DevTensor<T>& X, DevTensor<T>& Y, std::vector<int> axes = {}, bool keepdims = false) {
    size_t m, n;
    const Shape xs = detail::prepare_reduce(X, Y, std::move(axes), keepdims, &m, &n);
    gpgpu::dnn::reduce(name, m, n, xs.extents(), xs.strides(), X.data(), xs.offset(),
                       Y.shape().extents(), Y.shape().strides(), Y.data(), Y.shape().offset());
}

#define DLF_DEFINE_REDUCE_OP(fn)                                                                       \
    template <typename T>                                                                              \
    inline void fn(const DevTensor<T>& X, DevTensor<T>& Y, std::vector<int> axes = {}, bool keepdims = false) { \
        reduce(#fn, X, Y, std::move(axes), keepdims);                                                  \
    }                                                                                                  \
    template <typename T>                                                                              \
    inline DevTensor<T> fn(const DevTensor<T>& X, std::vector<int> axes = {}, bool keepdims = false) { \
        DevTensor<T> Y;                                                                                \
        reduce(#fn, X, Y, std::move(axes), keepdims);                                                  \
        return Y;                                                                                      \
    }
DLF_DEFINE_REDUCE_OP(reduce_max)
DLF_DEFINE_REDUCE_OP(reduce_min)
DLF_DEFINE_REDUCE_OP(reduce_amax)
DLF_DEFINE_REDUCE_OP(reduce_amin)
DLF_DEFINE_REDUCE_OP(reduce_sum)
DLF_DEFINE_REDUCE_OP(reduce_asum)
DLF_DEFINE_REDUCE_OP(reduce_mean)
DLF_DEFINE_REDUCE_OP(reduce_sum_square)
DLF_DEFINE_REDUCE_OP(reduce_nrm2)
DLF_DEFINE_REDUCE_OP(reduce_log_sum)
DLF_DEFINE_REDUCE_OP(reduce_sum_exp)
DLF_DEFINE_REDUCE_OP(reduce_log_sum_exp)
DLF_DEFINE_REDUCE_OP(reduce_prod)
#undef DLF_DEFINE_REDUCE_OP

// ---------------------------------------------------------------- count / nonzero
// dlf/include/tensor/reduce.h:160-198
template <typename T>
void count(const DevTensor<T>& X, DevTensor<int>& Y, const T& value, std::vector<int> axes = {}, bool keepdims = false) {
    size_t m, n;
    DevTensor<T> shape_only;       // prepare_reduce sizes an output of X's type; only its shape is used
    const Shape xs = detail::prepare_reduce(X, shape_only, std::move(axes), keepdims, &m, &n);
    Y.resize(shape_only.shape());
    gpgpu::dnn::count(m, n, value, xs.extents(), xs.strides(), X.data(), xs.offset(),
                      Y.shape().extents(), Y.shape().strides(), Y.data(), Y.shape().offset());
}
template <typename T>
inline DevTensor<int> count(const DevTensor<T>& X, const T& value, std::vector<int> axes = {}, bool keepdims = false) {
    DevTensor<int> Y;
    count(X, Y, value, std::move(axes), keepdims);
    return Y;
}

// dlf/include/tensor/reduce.h:419-450: running count of the non-zero elements of the whole
// tensor, one read of the total, then the coordinates.  Y becomes [n, rank], or [rank, n] when
// row_major; an input without non-zero elements leaves Y empty.
template <typename T>
void nonzero(const DevTensor<T>& X, DevTensor<int32_t>& Y, bool row_major = false) {
    auto counts = gpgpu::current::context().getTemporaryBuffer<int32_t>(X.size());
    const Shape counts_shape(X.shape().extents());
    gpgpu::dnn::scan_nonzero(1, X.size(), false, X.shape().extents(), X.data(), X.shape().offset(), X.shape().strides(),
                             counts, counts.offset(), counts_shape.strides());
    int32_t n = 0;
    counts.read(gpgpu::current::queue(), &n, 1, counts.offset() + X.size() - 1);
    if (n == 0) {
        Y.clear();
        return;
    }
    if (row_major) Y.resize(Shape({X.rank(), static_cast<size_t>(n)}));
    else Y.resize(Shape({static_cast<size_t>(n), X.rank()}));
    gpgpu::dnn::gather_indices(X.size(), n, row_major, X.shape().extents(), counts, counts.offset(),
                               Y.data(), Y.shape().offset());
}
template <typename T>
inline DevTensor<int32_t> nonzero(const DevTensor<T>& X, bool row_major = false) {
    DevTensor<int32_t> Y;
    nonzero(X, Y, row_major);
    return Y;
}

// ---------------------------------------------------------------- argmax / argmin
namespace detail {
template <typename T>
void arg_reduce(const DevTensor<T>& X, DevTensor<int>& Y, int axis, bool keepdims, const char* name) {
    norm_axis(static_cast<int>(X.rank()), axis);
    auto y_dims = X.shape().extents();
    if (keepdims) y_dims[axis] = 1;
    else y_dims.erase(y_dims.begin() + axis);
    const auto xv = moveaxis(X, axis, -1);
    Y.resize(Shape(y_dims));
    const size_t k = xv.shape().extent(-1);
    gpgpu::dnn::arg_reduce(name, xv.size() / k, k, xv.shape().extents(), xv.shape().strides(), xv.data(),
                           xv.shape().offset(), Y.shape().extents(), Y.shape().strides(), Y.data(), Y.shape().offset());
}
}  // namespace detail

template <typename T>
inline DevTensor<int> argmax(const DevTensor<T>& X, int axis, bool keepdims = true) {
    DevTensor<int> Y;
    detail::arg_reduce(X, Y, axis, keepdims, "argmax");
    return Y;
}
template <typename T>
inline DevTensor<int> argmin(const DevTensor<T>& X, int axis, bool keepdims = true) {
    DevTensor<int> Y;
    detail::arg_reduce(X, Y, axis, keepdims, "argmin");
    return Y;
}

// ---------------------------------------------------------------- scan
template <typename T>
void scan(const std::string& name, const DevTensor<T>& X, DevTensor<T>& Y, int axis, bool exclusive, bool reverse) {
    detail::norm_axis(static_cast<int>(X.rank()), axis);
    const size_t n = X.extent(axis), m = X.size() / n;
    if (&X != &Y) Y.resize(X.shape());
    auto xt = moveaxis(X, axis, -1), yt = moveaxis(Y, axis, -1);
    if (reverse) { xt = flip(xt, -1); yt = flip(yt, -1); }
    gpgpu::dnn::scan(name, m, n, exclusive, xt.shape().extents(), xt.data(), xt.shape().offset(), xt.shape().strides(),
                     yt.data(), yt.shape().offset(), yt.shape().strides());
}
template <typename T>
inline DevTensor<T> cumsum(const DevTensor<T>& X, int axis = -1, bool exclusive = false, bool reverse = false) {
    DevTensor<T> Y;
    scan("cumsum", X, Y, axis, exclusive, reverse);
    return Y;
}
template <typename T>
inline DevTensor<T> cumprod(const DevTensor<T>& X, int axis = -1, bool exclusive = false, bool reverse = false) {
    DevTensor<T> Y;
    scan("cumprod", X, Y, axis, exclusive, reverse);
    return Y;
}
template <typename T>
inline void cumsum(const DevTensor<T>& X, DevTensor<T>& Y, int axis = -1, bool exclusive = false, bool reverse = false) {
    scan("cumsum", X, Y, axis, exclusive, reverse);
}

// ---------------------------------------------------------------- reorder
// dlf/include/tensor/reorder.h reorder(X, Y) on device tensors: the viewed elements of X in
// row-major order in Y, copied on the device (gpgpu::dnn::copy).
template <typename T>
void reorder(const DevTensor<T>& X, DevTensor<T>& Y) {
    // Y may be X itself or another tensor over X's buffer (a view): the copy kernels do not take
    // overlapping views, so the elements then go through a tensor of their own
    const bool shared = &X == &Y || (!X.empty() && !Y.empty() && X.data().data() == Y.data().data());
    if (&X == &Y && X.shape().is_contiguous()) return;
    DevTensor<T> out;
    DevTensor<T>& dst = shared ? out : Y;
    dst.resize(X.shape());
    if (X.size() != 0)
        gpgpu::dnn::copy(X.size(), X.shape().extents(), X.data(), X.shape().offset(), X.shape().strides(),
                         dst.data(), dst.shape().offset(), dst.shape().strides());
    if (shared) Y = std::move(out);
}

// ---------------------------------------------------------------- sort / argsort / top_k
namespace detail {
template <typename T>
void copy_dense(const DevTensor<T>& X, DevTensor<T>& Y) {
    if (&X == &Y) return;
    reorder(X, Y);
}
inline void zero_indices(DevTensor<int32_t>& I) {
    gpgpu::dnn::fill(I.size(), I.data(), I.shape().offset(), int32_t(0));
}
}  // namespace detail

// dir: false ascending (less), true descending (greater)
template <typename T>
void sort(const DevTensor<T>& X, DevTensor<T>& Y, int axis = -1, bool descending = false) {
    detail::norm_axis(static_cast<int>(X.rank()), axis);
    if (X.extent(axis) > 1) {
        if (&X != &Y) Y.resize(X.shape());
        const auto xv = moveaxis(X, axis, -1);
        auto yv = moveaxis(Y, axis, -1);
        gpgpu::dnn::sort(descending ? 1 : 0, xv.shape().extents(), xv.data(), xv.shape().offset(), xv.shape().strides(),
                         yv.data(), yv.shape().offset(), yv.shape().strides());
    } else {
        detail::copy_dense(X, Y);
    }
}
template <typename T>
inline DevTensor<T> sorted(const DevTensor<T>& X, int axis = -1, bool descending = false) {
    DevTensor<T> Y;
    sort(X, Y, axis, descending);
    return Y;
}

template <typename T>
void argsort(const DevTensor<T>& X, DevTensor<int32_t>& I, int axis = -1, bool descending = false) {
    detail::norm_axis(static_cast<int>(X.rank()), axis);
    I.resize(X.shape());
    if (X.extent(axis) > 1) {
        const auto xv = moveaxis(X, axis, -1);
        auto iv = moveaxis(I, axis, -1);
        gpgpu::dnn::argsort(descending ? 1 : 0, xv.shape().extents(), xv.data(), xv.shape().offset(), xv.shape().strides(),
                            iv.data(), iv.shape().offset(), iv.shape().strides());
    } else {
        detail::zero_indices(I);
    }
}
template <typename T>
void argsort(const DevTensor<T>& X, DevTensor<T>& Y, DevTensor<int32_t>& I, int axis = -1, bool descending = false) {
    detail::norm_axis(static_cast<int>(X.rank()), axis);
    if (&X != &Y) Y.resize(X.shape());
    I.resize(X.shape());
    if (X.extent(axis) > 1) {
        const auto xv = moveaxis(X, axis, -1);
        auto yv = moveaxis(Y, axis, -1);
        auto iv = moveaxis(I, axis, -1);
        gpgpu::dnn::argsort(descending ? 1 : 0, xv.shape().extents(), xv.data(), xv.shape().offset(), xv.shape().strides(),
                            yv.data(), yv.shape().offset(), yv.shape().strides(),
                            iv.data(), iv.shape().offset(), iv.shape().strides());
    } else {
        detail::copy_dense(X, Y);
        detail::zero_indices(I);
    }
}
template <typename T>
inline DevTensor<int32_t> argsort(const DevTensor<T>& X, int axis = -1, bool descending = false) {
    DevTensor<int32_t> I;
    argsort(X, I, axis, descending);
    return I;
}

template <typename T>
void top_k(const DevTensor<T>& X, DevTensor<T>& Y, DevTensor<int32_t>& I, size_t k, int axis = -1, bool largest = true) {
    detail::norm_axis(static_cast<int>(X.rank()), axis);
    k = std::min(k, X.extent(axis));
    auto out_dims = X.shape().extents();
    out_dims[axis] = k;
    Y.resize(Shape(out_dims));
    I.resize(Shape(out_dims));
    const auto xv = moveaxis(X, axis, -1);
    auto yv = moveaxis(Y, axis, -1);
    auto iv = moveaxis(I, axis, -1);
    gpgpu::dnn::top_k(k, largest ? 1 : 0, xv.shape().extents(), yv.shape().extents(),
                      xv.data(), xv.shape().offset(), xv.shape().strides(),
                      yv.data(), yv.shape().offset(), yv.shape().strides(),
                      iv.data(), iv.shape().offset(), iv.shape().strides());
}
template <typename T>
inline std::pair<DevTensor<T>, DevTensor<int32_t>> top_k(const DevTensor<T>& X, size_t k, int axis = -1, bool largest = true) {
    DevTensor<T> Y;
    DevTensor<int32_t> I;
    top_k(X, Y, I, k, axis, largest);
    return {std::move(Y), std::move(I)};
}

// ---------------------------------------------------------------- softmax family
// dlf/include/tensor/dnn.h:447-531: rows are everything from `axis` on (default 1); the input
// is first copied into Y in row-major order (the reference's reorder(X, Y)), then normalised
// in place.
namespace dnn {
namespace detail {
// A dense input goes straight through the out-of-place routine; any other view is first laid out
// row-major in Y on the device (the reference's reorder(X, Y)) and normalised in place there.
template <typename T, typename Fn>
void normalize_rows(const DevTensor<T>& X, DevTensor<T>& Y, int axis, Fn fn) {
    dlf::detail::norm_axis(static_cast<int>(X.rank()), axis);
    size_t m = 1;
    for (int i = 0; i < axis; ++i) m *= X.extent(i);
    const size_t n = X.size() / m;
    if (X.shape().is_contiguous()) {
        if (&X != &Y) Y.resize(X.shape());
        fn(m, n, X.data(), X.shape().offset(), Y.data(), Y.shape().offset());
    } else {
        reorder(X, Y);
        fn(m, n, Y.data(), Y.shape().offset(), Y.data(), Y.shape().offset());
    }
}
}  // namespace detail
#define DLF_DEFINE_ROW_NORMALIZER(fn)                                                                     \
    template <typename T>                                                                                 \
    void fn(const DevTensor<T>& X, DevTensor<T>& Y, int axis = 1) {                                       \
        detail::normalize_rows(X, Y, axis, [](size_t m, size_t n, const gpgpu::Buffer<T>& x, size_t xo,  \
                                              gpgpu::Buffer<T>& y, size_t yo) { gpgpu::dnn::fn(m, n, x, xo, y, yo); }); \
    }
DLF_DEFINE_ROW_NORMALIZER(softmax)
DLF_DEFINE_ROW_NORMALIZER(logsoftmax)
DLF_DEFINE_ROW_NORMALIZER(hardmax)
#undef DLF_DEFINE_ROW_NORMALIZER
template <typename T>
inline DevTensor<T> softmax(const DevTensor<T>& X, int axis = 1) { DevTensor<T> Y; softmax(X, Y, axis); return Y; }
template <typename T>
inline DevTensor<T> logsoftmax(const DevTensor<T>& X, int axis = 1) { DevTensor<T> Y; logsoftmax(X, Y, axis); return Y; }
template <typename T>
inline DevTensor<T> hardmax(const DevTensor<T>& X, int axis = 1) { DevTensor<T> Y; hardmax(X, Y, axis); return Y; }
}  // namespace dnn

// ---------------------------------------------------------------- merge
// dlf/include/tensor/reorder.h:1061-1114: A and B are sorted along `axis`; C receives the
// merged rows (descending: both inputs sorted descending, the reference's comp = greater).
template <typename T>
void merge(const DevTensor<T>& A, const DevTensor<T>& B, DevTensor<T>& C, int axis = -1, bool descending = false) {
    const int rank = static_cast<int>(A.rank());
    if (static_cast<int>(B.rank()) != rank) throw shape_error("merge: incompatible shape");
    detail::norm_axis(rank, axis);
    std::vector<size_t> dims(rank);
    for (int i = 0; i < rank; ++i) {
        if (i == axis) dims[i] = A.extent(i) + B.extent(i);
        else if (A.extent(i) != B.extent(i)) throw shape_error("merge: incompatible shape");
        else dims[i] = A.extent(i);
    }
    C.resize(Shape(dims));
    const auto a = moveaxis(A, axis, -1), b = moveaxis(B, axis, -1), c = moveaxis(C, axis, -1);
    gpgpu::dnn::merge(descending ? 1 : 0,
                      a.shape().extents(), a.shape().strides(), a.data(), a.shape().offset(),
                      b.shape().extents(), b.shape().strides(), b.data(), b.shape().offset(),
                      c.shape().extents(), c.shape().strides(), C.data(), c.shape().offset());
}
template <typename T>
inline DevTensor<T> merge(const DevTensor<T>& A, const DevTensor<T>& B, int axis = -1, bool descending = false) {
    DevTensor<T> C;
    merge(A, B, C, axis, descending);
    return C;
}

}  // namespace dlf
