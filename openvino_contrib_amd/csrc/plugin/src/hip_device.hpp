// Errors and RAII device objects of the plugin layer.  Everything below goes through the C ABI of
// libhipattn (include/hipattn.h); this layer contains no HIP call of its own.
//
// Counterparts in the reference: throw_ov_exception with file:line(function)
// (modules/nvidia_plugin/src/error.cpp:13-29), CUDA::Stream / Allocation / Event
// (src/cuda/runtime.hpp:188-285, src/cuda/event.hpp:11-29).
#pragma once

#include <cstddef>
#include <memory>
#include <string>

#include "hipattn.h"
#include "openvino/core/except.hpp"

namespace ov {
namespace hip_gpu {

[[noreturn]] inline void throw_ov_exception(const std::string& msg, const char* file, int line, const char* func) {
    OPENVINO_THROW(file, ":", line, "(", func, "): ", msg);
}

#define HIP_PLUGIN_THROW(msg) ::ov::hip_gpu::throw_ov_exception((msg), __FILE__, __LINE__, __func__)
#define HIP_PLUGIN_ASSERT(cond, msg) \
    do {                             \
        if (!(cond)) HIP_PLUGIN_THROW(std::string("assertion `" #cond "` failed: ") + (msg)); \
    } while (0)

inline void throw_if_error(hipattn_status st, const char* file, int line, const char* func) {
    if (st != HIPATTN_OK)
        throw_ov_exception(std::string(hipattn_status_string(st)) + ": " + hipattn_last_error_string(), file, line, func);
}
#define HIP_PLUGIN_CHECK(expr) ::ov::hip_gpu::throw_if_error((expr), __FILE__, __LINE__, __func__)

class Stream {
public:
    Stream() { HIP_PLUGIN_CHECK(hipattn_stream_create(&stream_)); }
    ~Stream() {
        if (stream_) hipattn_stream_destroy(stream_);
    }
    Stream(const Stream&) = delete;
    Stream& operator=(const Stream&) = delete;
    hipattn_stream get() const { return stream_; }
    void synchronize() const { HIP_PLUGIN_CHECK(hipattn_stream_synchronize(stream_)); }
    void upload(void* dst, const void* src, size_t bytes) const {
        HIP_PLUGIN_CHECK(hipattn_memcpy_h2d_async(dst, src, bytes, stream_));
    }
    void download(void* dst, const void* src, size_t bytes) const {
        HIP_PLUGIN_CHECK(hipattn_memcpy_d2h_async(dst, src, bytes, stream_));
    }
    void transfer(void* dst, const void* src, size_t bytes) const {
        HIP_PLUGIN_CHECK(hipattn_memcpy_d2d_async(dst, src, bytes, stream_));
    }
    void fill(void* dst, int byte_value, size_t bytes) const {
        HIP_PLUGIN_CHECK(hipattn_fill_async(dst, byte_value, bytes, stream_));
    }

private:
    hipattn_stream stream_ = nullptr;
};

// Grow-only device buffer: reallocates when asked for more than it holds.
class Allocation {
public:
    Allocation() = default;
    ~Allocation() { release(); }
    Allocation(const Allocation&) = delete;
    Allocation& operator=(const Allocation&) = delete;
    void* reserve(size_t bytes) {
        if (bytes > capacity_) {
            release();
            HIP_PLUGIN_CHECK(hipattn_malloc(&ptr_, bytes));
            capacity_ = bytes;
        }
        return ptr_;
    }
    void* get() const { return ptr_; }
    size_t capacity() const { return capacity_; }

private:
    void release() {
        if (ptr_) hipattn_free(ptr_);
        ptr_ = nullptr;
        capacity_ = 0;
    }
    void* ptr_ = nullptr;
    size_t capacity_ = 0;
};

// An executable graph recorded from a stream (CUDA::GraphExec in the reference, src/cuda/graph.hpp).
class Graph {
public:
    Graph() = default;
    ~Graph() { reset(); }
    Graph(const Graph&) = delete;
    Graph& operator=(const Graph&) = delete;
    static void begin_capture(const Stream& s) { HIP_PLUGIN_CHECK(hipattn_stream_begin_capture(s.get())); }
    // ends the capture on `s` and keeps what was recorded; returns false (and keeps nothing) when the
    // recording could not be turned into an executable graph
    bool end_capture(const Stream& s) {
        reset();
        return hipattn_stream_end_capture(s.get(), &graph_) == HIPATTN_OK && graph_ != nullptr;
    }
    void launch(const Stream& s) const { HIP_PLUGIN_CHECK(hipattn_graph_launch(graph_, s.get())); }
    explicit operator bool() const { return graph_ != nullptr; }
    void reset() {
        if (graph_) hipattn_graph_destroy(graph_);
        graph_ = nullptr;
    }

private:
    hipattn_graph graph_ = nullptr;
};

class Event {
public:
    Event() { HIP_PLUGIN_CHECK(hipattn_event_create(&event_)); }
    ~Event() {
        if (event_) hipattn_event_destroy(event_);
    }
    Event(const Event&) = delete;
    Event& operator=(const Event&) = delete;
    void record(const Stream& s) const { HIP_PLUGIN_CHECK(hipattn_event_record(event_, s.get())); }
    void synchronize() const { HIP_PLUGIN_CHECK(hipattn_event_synchronize(event_)); }
    float elapsed_ms_until(const Event& stop) const {
        float ms = 0.f;
        HIP_PLUGIN_CHECK(hipattn_event_elapsed_ms(event_, stop.event_, &ms));
        return ms;
    }

private:
    hipattn_event event_ = nullptr;
};

}  // namespace hip_gpu
}  // namespace ov
