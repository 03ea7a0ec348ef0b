// Minimal HIP runtime wrapper for the host mirror: the subset of the reference's CUDA wrapper the FFN path uses
// (src/cuda.rs: Cuda::allocate / stream / event / copy_device / zero_device, Buffer::{ptr,len,upload,download,zero},
// Stream::{raw,synchronize,capture}, Event::{record,wait,elapsed_since}, Graph::launch).  All handles stay on the thread
// that made them; buffers free themselves.
#pragma once
#include <hip/hip_runtime_api.h>
#include <cstdint>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

namespace tf {

struct Error : std::runtime_error { using std::runtime_error::runtime_error; };
inline void check(hipError_t e, const char* what) {
    if (e != hipSuccess) throw Error(std::string(what) + ": " + hipGetErrorString(e));
}
inline void ensure(bool ok, const char* what) { if (!ok) throw Error(what); }

class Stream {
public:
    Stream() { check(hipStreamCreateWithFlags(&s_, hipStreamNonBlocking), "stream"); }
    ~Stream() { if (s_) hipStreamDestroy(s_); }
    Stream(const Stream&) = delete;
    Stream& operator=(const Stream&) = delete;
    hipStream_t raw() const { return s_; }
    void synchronize() const { check(hipStreamSynchronize(s_), "stream synchronize"); }
private:
    hipStream_t s_ = nullptr;
};

class Event {
public:
    explicit Event(bool timing = false) { check(hipEventCreateWithFlags(&e_, timing ? hipEventDefault : hipEventDisableTiming), "event"); }
    ~Event() { if (e_) hipEventDestroy(e_); }
    Event(const Event&) = delete;
    Event& operator=(const Event&) = delete;
    void record(hipStream_t s) const { check(hipEventRecord(e_, s), "event record"); }
    void wait(hipStream_t s) const { check(hipStreamWaitEvent(s, e_, 0), "event wait"); }
    void synchronize() const { check(hipEventSynchronize(e_), "event synchronize"); }
    hipEvent_t raw() const { return e_; }
    float elapsed_since(const Event& earlier) const { float ms = 0; check(hipEventElapsedTime(&ms, earlier.e_, e_), "elapsed"); return ms; }
private:
    hipEvent_t e_ = nullptr;
};

template <class T>
class Buffer {
public:
    Buffer() = default;
    explicit Buffer(size_t len) : len_(len) { if (len) check(hipMalloc(&p_, len * sizeof(T)), "allocate"); }
    ~Buffer() { if (p_) hipFree(p_); }
    Buffer(Buffer&& o) noexcept : p_(o.p_), len_(o.len_) { o.p_ = nullptr; o.len_ = 0; }
    Buffer& operator=(Buffer&& o) noexcept { if (this != &o) { if (p_) hipFree(p_); p_ = o.p_; len_ = o.len_; o.p_ = nullptr; o.len_ = 0; } return *this; }
    Buffer(const Buffer&) = delete;
    Buffer& operator=(const Buffer&) = delete;
    uint64_t ptr() const { return (uint64_t)p_; }
    T* data() const { return (T*)p_; }
    size_t len() const { return len_; }
    size_t bytes() const { return len_ * sizeof(T); }
    void upload(const T* host, size_t n) { ensure(n == len_, "upload length"); check(hipMemcpy(p_, host, n * sizeof(T), hipMemcpyHostToDevice), "upload"); }
    void upload(const std::vector<T>& host) { upload(host.data(), host.size()); }
    void download(T* host, size_t n) const { ensure(n <= len_, "download length"); check(hipMemcpy(host, p_, n * sizeof(T), hipMemcpyDeviceToHost), "download"); }
    std::vector<T> download() const { std::vector<T> v(len_); download(v.data(), len_); return v; }
    void zero() { if (len_) check(hipMemset(p_, 0, bytes()), "zero"); }
    void fill_bytes(int value) { if (len_) check(hipMemset(p_, value, bytes()), "fill"); }
private:
    void* p_ = nullptr;
    size_t len_ = 0;
};

// A captured stream section replayed as one graph launch (src/cuda.rs:2068-2153).
class Graph {
public:
    Graph() = default;
    ~Graph() { if (exec_) hipGraphExecDestroy(exec_); if (graph_) hipGraphDestroy(graph_); }
    Graph(const Graph&) = delete;
    Graph& operator=(const Graph&) = delete;
    template <class F>
    void capture(const Stream& s, F&& body) {
        check(hipStreamBeginCapture(s.raw(), hipStreamCaptureModeThreadLocal), "begin capture");
        try { body(); } catch (...) { hipGraph_t g = nullptr; hipStreamEndCapture(s.raw(), &g); if (g) hipGraphDestroy(g); throw; }
        check(hipStreamEndCapture(s.raw(), &graph_), "end capture");
        check(hipGraphInstantiate(&exec_, graph_, nullptr, nullptr, 0), "instantiate graph");
    }
    bool ready() const { return exec_ != nullptr; }
    void launch(const Stream& s) const { check(hipGraphLaunch(exec_, s.raw()), "graph launch"); }
private:
    hipGraph_t graph_ = nullptr;
    hipGraphExec_t exec_ = nullptr;
};

}  // namespace tf
