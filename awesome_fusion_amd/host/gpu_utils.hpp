// GPU_CHECK_ERROR of the harness (/root/reference/bfAintBGemm/gpu_utils.hpp:5-11): print the failing
// call.  The reference then calls exit(0), which reports success to the shell; this one exits 1.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>

#define GPU_CHECK_ERROR(call)                                                                                \
    do {                                                                                                     \
        hipError_t err_ = (call);                                                                            \
        if (err_ != hipSuccess) {                                                                            \
            std::printf("[hip error](%d: %s), failed to call %s \n", (int)err_, hipGetErrorString(err_), #call); \
            std::exit(EXIT_FAILURE);                                                                         \
        }                                                                                                    \
    } while (0)
