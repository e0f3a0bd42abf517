// Shared host-side plumbing for the MI355X IVFPQ / Flat search library: status codes, error
// capture, RAII device buffers and the stream every kernel of an index is launched on.
#pragma once
#include <atomic>
#include <mutex>
#include <unordered_map>
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <stdexcept>
#include <string>
#include <vector>

namespace ixa {

// Numeric values follow the reference's APP_ERROR enum (FR/common/ErrorCode.h:26-73).
enum Status : int {
    kOk = 0,
    kErrBadAlloc = 1001,        // APP_ERR_ACL_BAD_ALLOC
    kErrOpExecFailed = 1017,    // APP_ERR_ACL_OP_EXEC_FAILED
    kErrInvalidParam = 2001,    // APP_ERR_INVALID_PARAM
    kErrNotImplemented = 2008,  // APP_ERR_NOT_IMPLEMENT
    kErrIllegalOperation = 2009,
    kErrInner = 2010,           // APP_ERR_INNER_ERROR
    kErrIndexNotInit = 2016,    // APP_ERR_INDEX_NOT_INIT
};

constexpr int kMetricInnerProduct = 0;  // faiss::METRIC_INNER_PRODUCT
constexpr int kMetricL2 = 1;            // faiss::METRIC_L2

struct Error : std::runtime_error {
    int code;
    Error(int c, const std::string &m) : std::runtime_error(m), code(c) {}
};

[[noreturn]] inline void fail(int code, const char *fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    throw Error(code, buf);
}

#define IXA_REQUIRE(cond, code, ...)        \
    do {                                    \
        if (!(cond)) {                      \
            ::ixa::fail((code), __VA_ARGS__); \
        }                                   \
    } while (0)

#define IXA_HIP(expr)                                                                                   \
    do {                                                                                                \
        hipError_t e_ = (expr);                                                                         \
        if (e_ != hipSuccess) {                                                                         \
            ::ixa::fail(e_ == hipErrorOutOfMemory ? ::ixa::kErrBadAlloc : ::ixa::kErrOpExecFailed,      \
                        "HIP error %d (%s) at %s:%d: %s", (int)e_, hipGetErrorString(e_), __FILE__, __LINE__, \
                        #expr);                                                                         \
        }                                                                                               \
    } while (0)

// Waits for the stream.  A launch the device rejects (a grid or LDS size it cannot run) is reported by
// no later call except hipGetLastError, so that is asked first: a kernel that never ran must not pass
// for one that did.
inline void sync_stream(hipStream_t s)
{
    IXA_HIP(hipGetLastError());
    IXA_HIP(hipStreamSynchronize(s));
}

// Raises a kernel's limit of dynamic LDS to at least `bytes` (every kernel starts at 48 KB).  The limit only ever
// grows: launches from several threads never find it lowered under them, and a launch whose size is covered already
// costs no runtime call.
inline void require_dynamic_lds(const void *kern, size_t bytes)
{
    if (bytes <= 48 * 1024) {
        return;
    }
    static std::mutex mu;
    static std::unordered_map<const void *, size_t> limit;
    std::lock_guard<std::mutex> lock(mu);
    size_t &have = limit[kern];
    if (bytes > have) {
        IXA_HIP(hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
        have = bytes;
    }
}

// Owning device allocation.  Grows by reallocation (contents are NOT preserved by resize()).  borrow() makes it a
// non-owning window onto another buffer's memory instead (a search view of an index reads the owner's data).
template <typename T>
class DeviceBuffer {
public:
    DeviceBuffer() = default;
    explicit DeviceBuffer(size_t n) { resize(n); }
    DeviceBuffer(const DeviceBuffer &) = delete;
    DeviceBuffer &operator=(const DeviceBuffer &) = delete;
    DeviceBuffer(DeviceBuffer &&o) noexcept : p_(o.p_), n_(o.n_), cap_(o.cap_), borrowed_(o.borrowed_)
    {
        o.p_ = nullptr;
        o.n_ = o.cap_ = 0;
        o.borrowed_ = false;
    }
    DeviceBuffer &operator=(DeviceBuffer &&o) noexcept
    {
        if (this != &o) {
            release();
            p_ = o.p_;
            n_ = o.n_;
            cap_ = o.cap_;
            borrowed_ = o.borrowed_;
            o.p_ = nullptr;
            o.n_ = o.cap_ = 0;
            o.borrowed_ = false;
        }
        return *this;
    }
    ~DeviceBuffer() { release(); }

    // After resize the buffer holds n elements of unspecified content.
    void resize(size_t n)
    {
        if (n > cap_) {
            release();
            void *p = nullptr;
            IXA_HIP(hipMalloc(&p, n * sizeof(T)));
            p_ = static_cast<T *>(p);
            cap_ = n;
        }
        n_ = n;
    }
    void release()
    {
        if (p_ && !borrowed_) {
            (void)hipFree(p_);
        }
        p_ = nullptr;
        n_ = cap_ = 0;
        borrowed_ = false;
    }
    // This buffer becomes a window onto o's memory: valid until o reallocates or dies.
    void borrow(const DeviceBuffer &o)
    {
        release();
        p_ = o.p_;
        n_ = cap_ = o.n_;
        borrowed_ = p_ != nullptr;
    }
    T *data() const { return p_; }
    size_t size() const { return n_; }
    size_t bytes() const { return n_ * sizeof(T); }

    void upload(const T *host, size_t n, hipStream_t s)
    {
        resize(n);
        if (n) {
            IXA_HIP(hipMemcpyAsync(p_, host, n * sizeof(T), hipMemcpyHostToDevice, s));
        }
    }
    void download(T *host, size_t n, hipStream_t s) const
    {
        if (n) {
            IXA_HIP(hipMemcpyAsync(host, p_, n * sizeof(T), hipMemcpyDeviceToHost, s));
            sync_stream(s);
        }
    }

private:
    T *p_ = nullptr;
    size_t n_ = 0, cap_ = 0;
    bool borrowed_ = false;
};

// Page-locked host memory for the small copies of latency-bound paths (a copy to or from pageable memory
// goes through a staging buffer of the runtime).  Grows by reallocation; contents are not preserved.
class PinnedBuffer {
public:
    PinnedBuffer() = default;
    PinnedBuffer(const PinnedBuffer &) = delete;
    PinnedBuffer &operator=(const PinnedBuffer &) = delete;
    ~PinnedBuffer()
    {
        if (p_) {
            (void)hipHostFree(p_);
        }
    }
    void *reserve(size_t bytes)
    {
        if (bytes > cap_) {
            if (p_) {
                (void)hipHostFree(p_);
                p_ = nullptr;
                cap_ = 0;
            }
            const size_t want = bytes + bytes / 2 + 4096;
            IXA_HIP(hipHostMalloc(&p_, want, hipHostMallocDefault));
            cap_ = want;
        }
        return p_;
    }

private:
    void *p_ = nullptr;
    size_t cap_ = 0;
};

inline int64_t round_up(int64_t v, int64_t m) { return (v + m - 1) / m * m; }
inline int pow2_ceil(int v)
{
    int p = 1;
    while (p < v) {
        p <<= 1;
    }
    return p;
}

}  // namespace ixa
