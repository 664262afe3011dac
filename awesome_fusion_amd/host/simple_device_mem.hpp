// Owning buffers of the harness.  The two names and GetBuffer() are those the reference's driver uses
// (/root/reference/bfAintBGemm/simple_device_mem.hpp:5-40), so its main() reads the same with these; the
// implementation is one owning template over an allocation policy instead of a virtual base, is movable, and —
// unlike the reference, which discards hipMalloc's result (:20) — keeps the allocation status for the caller.
#pragma once
#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdlib>
#include <utility>

namespace bfaintb_host {

// Device memory through the HIP runtime.
struct DevicePolicy {
    static hipError_t acquire(void** out, std::size_t bytes) { return bytes ? hipMalloc(out, bytes) : hipSuccess; }
    static void release(void* p) { (void)hipFree(p); }
};

// Pageable host memory; a zero-byte request still yields a distinct pointer.
struct HostPolicy {
    static hipError_t acquire(void** out, std::size_t bytes)
    {
        *out = std::malloc(bytes ? bytes : 1);
        return *out ? hipSuccess : hipErrorOutOfMemory;
    }
    static void release(void* p) { std::free(p); }
};

template <typename Policy>
class OwnedBuffer {
public:
    explicit OwnedBuffer(std::size_t bytes) : bytes_(bytes)
    {
        status_ = Policy::acquire(&ptr_, bytes);
        if (status_ != hipSuccess) ptr_ = nullptr;
    }
    OwnedBuffer(OwnedBuffer&& other) noexcept : ptr_(std::exchange(other.ptr_, nullptr)), bytes_(other.bytes_), status_(other.status_) {}
    OwnedBuffer(const OwnedBuffer&) = delete;
    OwnedBuffer& operator=(const OwnedBuffer&) = delete;
    OwnedBuffer& operator=(OwnedBuffer&&) = delete;
    ~OwnedBuffer()
    {
        if (ptr_ != nullptr) Policy::release(ptr_);
    }

    void* GetBuffer() const { return ptr_; }
    std::size_t GetSize() const { return bytes_; }
    hipError_t Status() const { return status_; }

private:
    void* ptr_ = nullptr;
    std::size_t bytes_ = 0;
    hipError_t status_ = hipSuccess;
};

}  // namespace bfaintb_host

using SimpleDeviceMem = bfaintb_host::OwnedBuffer<bfaintb_host::DevicePolicy>;
using SimpleHostMem = bfaintb_host::OwnedBuffer<bfaintb_host::HostPolicy>;
