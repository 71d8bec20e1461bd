// Host veneer: the subset of dlf's gpgpu runtime objects that the axis
// primitives' call surface touches, implemented directly on HIP.
//
// Mirrors gpgpu/include/gpgpu.h (exceptions :21-121, Queue/Event :593-637,
// Buffer<T> :639-698, TemporaryBuffer<T> :710-746, current:: :828-857) and
// gpgpu/src/gpgpu.cpp:139-229 (thread-local current queue, LIFO temporary
// buffers).  Only HIP is behind it: no OpenCL/CUDA back-ends, no run-time
// kernel compilation, no program cache.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "dlfx.h"

namespace gpgpu {

// ---------------------------------------------------------------- errors
class Error : public std::runtime_error {
public:
    explicit Error(const std::string& what) : std::runtime_error(what) {}
};

// A HIP runtime call failed (reference: APIError).
class APIError : public Error {
    int status_;
public:
    APIError(int status, const std::string& where)
        : Error("HIP error " + std::to_string(status) + " (" + hipGetErrorString(static_cast<hipError_t>(status)) +
                ") in " + where), status_(status) {}
    int status() const noexcept { return status_; }
};

// A routine rejected its arguments or failed to launch (reference: RuntimeErrorCode).
class RuntimeErrorCode : public Error {
    int status_;
public:
    RuntimeErrorCode(int status, const std::string& where)
        : Error(where + ": " + dlfx_status_string(status)), status_(status) {}
    int status() const noexcept { return status_; }
};

// Misuse of the veneer itself, e.g. temporary buffers released out of order (reference: LogicError).
class LogicError : public Error {
public:
    explicit LogicError(const std::string& what) : Error(what) {}
};

inline void check_hip(hipError_t e, const char* where) {
    if (e != hipSuccess) throw APIError(static_cast<int>(e), where);
}

inline void check_status(int status, const char* where) {
    if (status == DLFX_OK) return;
    if (status == DLFX_ERR_LAUNCH) throw APIError(dlfx_last_hip_error(), where);
    throw RuntimeErrorCode(status, where);
}

// ---------------------------------------------------------------- context
template <typename T> class TemporaryBuffer;
class Queue;

namespace detail {
// One device and one scratch arena: a bump allocator whose allocations are released in LIFO order.
struct ContextState {
    int device = 0;
    std::shared_ptr<void> arena;
    size_t capacity = 0, top = 0;
    std::vector<std::shared_ptr<void>> retired;    // arenas outgrown while temporaries were live

    void release(size_t prev_top, size_t end) {
        if (end != top) throw LogicError("TemporaryBuffer: released out of order");
        top = prev_top;
        if (top == 0) retired.clear();
    }
};
// Host transfers issued through Buffer::read, for tests that must prove a path stays on the device.
inline size_t& device_to_host_reads() {
    static thread_local size_t n = 0;
    return n;
}
}  // namespace detail

// A handle to a device context (reference: gpgpu.h Context, :480-590): copies share the state.
// Queues created from one context share its scratch arena, as in the reference; work that may
// overlap in time on different queues therefore needs queues of different contexts.
class Context {
    std::shared_ptr<detail::ContextState> s_;
public:
    explicit Context(int device = 0) : s_(std::make_shared<detail::ContextState>()) {
        s_->device = device;
        check_hip(hipSetDevice(device), "hipSetDevice");
    }
    int device() const noexcept { return s_->device; }
    bool operator==(const Context& o) const noexcept { return s_ == o.s_; }
    bool operator!=(const Context& o) const noexcept { return s_ != o.s_; }
    size_t temporary_bytes_in_use() const noexcept { return s_->top; }

    // gpgpu.h:573-574, gpgpu.cpp:189-214
    template <typename T>
    TemporaryBuffer<T> getTemporaryBuffer(size_t size) const;
    // gpgpu.h:555-559: a new in-order queue on this context's device
    Queue createQueue() const;
};

// ---------------------------------------------------------------- queue / event
// An in-order stream of work on one device; it knows the context it was created on
// (reference: Queue::context(), gpgpu.h:609), which is where routines take their scratch.
class Queue {
    struct Holder {
        hipStream_t stream = nullptr;
        bool owned = false;
        ~Holder() { if (owned && stream) (void)hipStreamDestroy(stream); }
    };
    Context ctx_;
    std::shared_ptr<Holder> h_;
    static int current_device() {
        int d = 0;
        check_hip(hipGetDevice(&d), "hipGetDevice");
        return d;
    }
    friend class Context;
    Queue(Context ctx, bool) : ctx_(std::move(ctx)), h_(std::make_shared<Holder>()) {
        check_hip(hipStreamCreate(&h_->stream), "hipStreamCreate");
        h_->owned = true;
    }
public:
    // A new stream on the current device with a context (and scratch arena) of its own.
    Queue() : Queue(Context(current_device()), true) {}
    // Wraps an existing stream without taking ownership (nullptr = the default stream); the
    // queue gets a context of its own.
    explicit Queue(hipStream_t s) : ctx_(current_device()), h_(std::make_shared<Holder>()) { h_->stream = s; }
    hipStream_t stream() const noexcept { return h_->stream; }
    const Context& context() const noexcept { return ctx_; }
    void finish() const { check_hip(hipStreamSynchronize(h_->stream), "hipStreamSynchronize"); }
    bool operator==(const Queue& o) const noexcept { return h_ == o.h_; }
    bool operator!=(const Queue& o) const noexcept { return h_ != o.h_; }
};

inline Queue Context::createQueue() const { return Queue(*this, true); }

// Start/end markers around the last kernel of a routine.
class Event {
    struct Holder {
        hipEvent_t start = nullptr, end = nullptr;
        Holder() {
            check_hip(hipEventCreate(&start), "hipEventCreate");
            check_hip(hipEventCreate(&end), "hipEventCreate");
        }
        ~Holder() { (void)hipEventDestroy(start); (void)hipEventDestroy(end); }
    };
    std::shared_ptr<Holder> h_ = std::make_shared<Holder>();
public:
    hipEvent_t start() const noexcept { return h_->start; }
    hipEvent_t end() const noexcept { return h_->end; }
    void waitForCompletion() const { check_hip(hipEventSynchronize(h_->end), "hipEventSynchronize"); }
    float getElapsedTime() const {          // milliseconds
        waitForCompletion();
        float ms = 0;
        check_hip(hipEventElapsedTime(&ms, h_->start, h_->end), "hipEventElapsedTime");
        return ms;
    }
};

// ---------------------------------------------------------------- buffers
// Typed device memory shared by reference; offset() is non-zero only for
// temporary buffers carved out of a context's scratch arena.
template <typename T>
class Buffer {
protected:
    std::shared_ptr<void> mem_;
    size_t size_ = 0;      // elements
    size_t offset_ = 0;    // elements from mem_
public:
    Buffer() = default;
    explicit Buffer(size_t size) : size_(size) {
        void* p = nullptr;
        check_hip(hipMalloc(&p, (size ? size : 1) * sizeof(T)), "hipMalloc");
        mem_ = std::shared_ptr<void>(p, [](void* q) { (void)hipFree(q); });
    }
    Buffer(std::shared_ptr<void> mem, size_t size, size_t offset) : mem_(std::move(mem)), size_(size), offset_(offset) {}

    size_t size() const noexcept { return size_; }
    size_t offset() const noexcept { return offset_; }
    T* data() const noexcept { return static_cast<T*>(mem_.get()); }       // start of the allocation
    explicit operator bool() const noexcept { return static_cast<bool>(mem_); }

    void read(const Queue& q, T* host, size_t n, size_t offset = 0) const {
        if (offset + n > size_ + offset_) throw LogicError("Buffer::read: range exceeds the buffer");
        check_hip(hipMemcpyAsync(host, data() + offset, n * sizeof(T), hipMemcpyDeviceToHost, q.stream()), "hipMemcpyAsync");
        q.finish();
        ++detail::device_to_host_reads();
    }
    void write(const Queue& q, const T* host, size_t n, size_t offset = 0) {
        if (offset + n > size_ + offset_) throw LogicError("Buffer::write: range exceeds the buffer");
        check_hip(hipMemcpyAsync(data() + offset, host, n * sizeof(T), hipMemcpyHostToDevice, q.stream()), "hipMemcpyAsync");
        q.finish();
    }
    void copyTo(const Queue& q, Buffer<T>& dst, size_t n, size_t src_offset = 0, size_t dst_offset = 0) const {
        check_hip(hipMemcpyAsync(dst.data() + dst_offset, data() + src_offset, n * sizeof(T), hipMemcpyDeviceToDevice,
                                 q.stream()), "hipMemcpyAsync");
    }
};

// A bump allocation from the context's arena, released in LIFO order when it
// goes out of scope; releasing out of order throws (gpgpu.cpp:208-214).
template <typename T>
class TemporaryBuffer : public Buffer<T> {
    std::shared_ptr<detail::ContextState> ctx_;
    size_t bytes_begin_ = 0, bytes_end_ = 0, prev_top_ = 0;   // prev_top_: the arena's top before this allocation
public:
    TemporaryBuffer(std::shared_ptr<detail::ContextState> ctx, std::shared_ptr<void> mem, size_t size, size_t byte_begin,
                    size_t byte_end, size_t prev_top)
        : Buffer<T>(std::move(mem), size, byte_begin / sizeof(T)), ctx_(std::move(ctx)), bytes_begin_(byte_begin),
          bytes_end_(byte_end), prev_top_(prev_top) {}
    TemporaryBuffer(const TemporaryBuffer&) = delete;
    TemporaryBuffer& operator=(const TemporaryBuffer&) = delete;
    TemporaryBuffer(TemporaryBuffer&& o) noexcept
        : Buffer<T>(std::move(o)), ctx_(std::move(o.ctx_)), bytes_begin_(o.bytes_begin_), bytes_end_(o.bytes_end_),
          prev_top_(o.prev_top_) {
        o.ctx_ = nullptr;
    }
    ~TemporaryBuffer() noexcept(false) {
        if (ctx_) ctx_->release(prev_top_, bytes_end_);
    }
    // This allocation's own bytes (Buffer::data() is the start of the whole arena).
    void* bytes() const noexcept { return static_cast<char*>(this->mem_.get()) + bytes_begin_; }
    size_t byte_size() const noexcept { return bytes_end_ - bytes_begin_; }
};

template <typename T>
TemporaryBuffer<T> Context::getTemporaryBuffer(size_t size) const {
    detail::ContextState& c = *s_;
    const size_t align = 256;
    const size_t prev_top = c.top;
    const size_t begin = (c.top + align - 1) / align * align;
    const size_t end = begin + (size ? size : 1) * sizeof(T);
    if (end > c.capacity) {
        // grow: earlier temporaries keep their (retired) arena alive through their shared_ptr
        size_t cap = c.capacity ? c.capacity : (size_t(1) << 20);
        while (cap < end) cap *= 2;
        void* p = nullptr;
        check_hip(hipMalloc(&p, cap), "hipMalloc");
        if (c.arena) c.retired.push_back(c.arena);
        c.arena = std::shared_ptr<void>(p, [](void* q) { (void)hipFree(q); });
        c.capacity = cap;
    }
    c.top = end;
    return TemporaryBuffer<T>(s_, c.arena, size, begin, end, prev_top);
}

// ---------------------------------------------------------------- thread-local current objects
namespace current {

// The calling thread's queue, created with its context on first use (gpgpu.cpp:155-168).
inline const Queue& queue() {
    thread_local Queue q = Context(0).createQueue();
    return q;
}

inline const Context& context() { return queue().context(); }

}  // namespace current
}  // namespace gpgpu
