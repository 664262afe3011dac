// RAII buffers of the harness: same class names and GetBuffer() as
// /root/reference/bfAintBGemm/simple_device_mem.hpp:5-40.  Unlike the reference (hipMalloc result
// discarded, :20) an allocation failure is recorded and can be asked for.
#pragma once
#include <hip/hip_runtime.h>
#include <cstddef>
#include <cstdlib>

struct SimpleMem {
    SimpleMem() = default;
    explicit SimpleMem(std::size_t mem_size) : p_mem_{nullptr}, size_{mem_size} {}
    virtual void* GetBuffer() = 0;
    virtual ~SimpleMem() {}
    std::size_t GetSize() const { return size_; }
    SimpleMem(const SimpleMem&) = delete;
    SimpleMem& operator=(const SimpleMem&) = delete;
    void* p_mem_ = nullptr;
    std::size_t size_ = 0;
};

struct SimpleDeviceMem : SimpleMem {
    SimpleDeviceMem() = delete;
    explicit SimpleDeviceMem(std::size_t mem_size) : SimpleMem(mem_size)
    {
        status_ = mem_size ? hipMalloc(&p_mem_, mem_size) : hipSuccess;
        if (status_ != hipSuccess) p_mem_ = nullptr;
    }
    void* GetBuffer() override { return p_mem_; }
    hipError_t Status() const { return status_; }
    ~SimpleDeviceMem() override { if (p_mem_) (void)hipFree(p_mem_); }
    hipError_t status_ = hipSuccess;
};

struct SimpleHostMem : SimpleMem {
    SimpleHostMem() = delete;
    explicit SimpleHostMem(std::size_t mem_size) : SimpleMem(mem_size) { p_mem_ = std::malloc(mem_size ? mem_size : 1); }
    void* GetBuffer() override { return p_mem_; }
    ~SimpleHostMem() override { std::free(p_mem_); }
};
