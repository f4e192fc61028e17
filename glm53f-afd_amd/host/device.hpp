// Minimal device memory, streams and events over the HIP runtime: the C++ counterpart of the reference's
// crates/glm53f-kda/src/device.rs:1-331 and src/cuda.rs:1-55 (DeviceBuffer, Stream, Event, Error, device_count,
// attribute, mem_info). Header only; link with amdhip64.
#ifndef GLM53F_KDA_HOST_DEVICE_HPP
#define GLM53F_KDA_HOST_DEVICE_HPP

#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdint>
#include <string>
#include <utility>
#include <vector>

namespace glm53f_kda {

/// What went wrong: nothing, an argument rejected on the host (device.rs `Error::Invalid`), or a runtime
/// error code (device.rs `Error::Cuda`, here a hipError_t).
struct Error {
    enum Kind { Ok, Invalid, Hip };
    Kind kind = Ok;
    int code = 0;
    std::string what;

    static Error ok() { return {}; }
    static Error invalid(std::string msg) { return {Invalid, 1, std::move(msg)}; }
    static Error hip(int code, std::string msg) { return {Hip, code, std::move(msg)}; }
    bool is_ok() const { return kind == Ok; }
    explicit operator bool() const { return kind == Ok; }
};

inline Error check_hip(hipError_t e, const char* what) {
    if (e == hipSuccess) return Error::ok();
    return Error::hip((int)e, std::string(what) + ": " + hipGetErrorString(e));
}

inline int device_count() {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return n;
}

inline Error attribute(hipDeviceAttribute_t attr, int device, int* value) {
    return check_hip(hipDeviceGetAttribute(value, attr, device), "hipDeviceGetAttribute");
}

inline Error mem_info(size_t* free_bytes, size_t* total_bytes) {
    return check_hip(hipMemGetInfo(free_bytes, total_bytes), "hipMemGetInfo");
}

/// Device memory that frees itself (hipFree waits for the device, as the reference's cudaFree does).
class DeviceBuffer {
  public:
    DeviceBuffer() = default;
    DeviceBuffer(const DeviceBuffer&) = delete;
    DeviceBuffer& operator=(const DeviceBuffer&) = delete;
    DeviceBuffer(DeviceBuffer&& o) noexcept : ptr_(o.ptr_), bytes_(o.bytes_) { o.ptr_ = nullptr; o.bytes_ = 0; }
    DeviceBuffer& operator=(DeviceBuffer&& o) noexcept {
        if (this != &o) {
            release();
            ptr_ = o.ptr_; bytes_ = o.bytes_;
            o.ptr_ = nullptr; o.bytes_ = 0;
        }
        return *this;
    }
    ~DeviceBuffer() { release(); }

    /// Uninitialized memory. Zero bytes is allowed: an empty buffer.
    static Error alloc(size_t bytes, DeviceBuffer* out) {
        DeviceBuffer b;
        if (bytes > 0) {
            Error e = check_hip(hipMalloc(&b.ptr_, bytes), "hipMalloc");
            if (!e) return e;
        }
        b.bytes_ = bytes;
        *out = std::move(b);
        return Error::ok();
    }
    static Error zeroed(size_t bytes, DeviceBuffer* out) {
        Error e = alloc(bytes, out);
        if (!e || bytes == 0) return e;
        return check_hip(hipMemset(out->ptr_, 0, bytes), "hipMemset");
    }
    template <typename T>
    static Error from_slice(const std::vector<T>& xs, DeviceBuffer* out) {
        Error e = alloc(xs.size() * sizeof(T), out);
        if (!e) return e;
        return out->upload(xs);
    }

    size_t bytes() const { return bytes_; }
    const void* as_ptr() const { return ptr_; }
    /// Element `offset` of the buffer seen as an array of T.
    template <typename T>
    T* ptr(size_t offset = 0) const { return reinterpret_cast<T*>(ptr_) + offset; }

    /// Synchronous copies (they wait for the device's earlier work on the default stream).
    template <typename T>
    Error upload(const std::vector<T>& xs) { return upload_at<T>(0, xs); }
    template <typename T>
    Error upload_at(size_t offset, const std::vector<T>& xs) {
        if ((offset + xs.size()) * sizeof(T) > bytes_) return Error::invalid("upload beyond the buffer");
        if (xs.empty()) return Error::ok();
        return check_hip(hipMemcpy(ptr<T>(offset), xs.data(), xs.size() * sizeof(T), hipMemcpyHostToDevice), "hipMemcpy");
    }
    template <typename T>
    Error download(size_t n, std::vector<T>* out, size_t offset = 0) const {
        if ((offset + n) * sizeof(T) > bytes_) return Error::invalid("download beyond the buffer");
        out->resize(n);
        if (n == 0) return Error::ok();
        return check_hip(hipMemcpy(out->data(), ptr<T>(offset), n * sizeof(T), hipMemcpyDeviceToHost), "hipMemcpy");
    }
    template <typename T>
    Error to_vec(std::vector<T>* out) const { return download<T>(bytes_ / sizeof(T), out); }

  private:
    void release() {
        if (ptr_ != nullptr) (void)hipFree(ptr_);
        ptr_ = nullptr;
        bytes_ = 0;
    }
    void* ptr_ = nullptr;
    size_t bytes_ = 0;
};

/// A HIP stream at the default priority. `Stream::null()` is the default stream.
class Stream {
  public:
    Stream(const Stream&) = delete;
    Stream& operator=(const Stream&) = delete;
    Stream(Stream&& o) noexcept : s_(o.s_), owned_(o.owned_) { o.s_ = nullptr; o.owned_ = false; }
    ~Stream() {
        if (owned_ && s_ != nullptr) (void)hipStreamDestroy(s_);
    }
    static Stream null() { return Stream(nullptr, false); }
    static Error create(Stream* out) {
        hipStream_t s = nullptr;
        Error e = check_hip(hipStreamCreate(&s), "hipStreamCreate");
        if (!e) return e;
        out->~Stream();
        new (out) Stream(s, true);
        return Error::ok();
    }
    hipStream_t raw() const { return s_; }
    Error synchronize() const { return check_hip(hipStreamSynchronize(s_), "hipStreamSynchronize"); }

  private:
    Stream(hipStream_t s, bool owned) : s_(s), owned_(owned) {}
    hipStream_t s_ = nullptr;
    bool owned_ = false;
};

/// A timing event.
class Event {
  public:
    Event() { (void)hipEventCreate(&e_); }
    Event(const Event&) = delete;
    Event& operator=(const Event&) = delete;
    ~Event() {
        if (e_ != nullptr) (void)hipEventDestroy(e_);
    }
    Error record(const Stream& s) { return check_hip(hipEventRecord(e_, s.raw()), "hipEventRecord"); }
    Error synchronize() { return check_hip(hipEventSynchronize(e_), "hipEventSynchronize"); }
    /// Milliseconds from `start` to this event (both recorded and complete).
    Error elapsed_since(const Event& start, float* ms) {
        return check_hip(hipEventElapsedTime(ms, start.e_, e_), "hipEventElapsedTime");
    }

  private:
    hipEvent_t e_ = nullptr;
};

}  // namespace glm53f_kda

#endif  // GLM53F_KDA_HOST_DEVICE_HPP
