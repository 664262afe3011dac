// The bfAintBGemm driver: command line, buffers, data, timing, metrics and (optionally) validation.
// Same flow and positional command line as /root/reference/bfAintBGemm/bfAintBGemm.cc:36-217:
//
//   bfAintBGemm [validation] [m n k] [lda ldb ldc] [weight_bits group_size data seed loops arith]
//
// with the reference's defaults (validation 0, m 32, n 128, k 512, ld = k, n, n; 10 warm-up and 10
// timed launches inside one event pair on the null stream, :103-104,151-186).  Where the reference
// loads a code object and calls hipModuleLaunchKernel with a packed argument block (:65-66,119-152),
// this driver calls bfaintb_gemm from the C ABI with the same arguments in the same order.
//   data = 0  the reference's test regime: A, B and scale all integers in {-2,-1,0,1} (random_gen.hpp:24,37,50)
//   data = 1  A ~ N(0,1); B uniform integers over the code range; scale uniform in [0.001, 0.01] (8-bit)
//             or [0.001, 0.02] (4-bit); scales per column or per group of `group_size` rows
//   arith = 0 this library's contract: bf16 scales, round-to-nearest-even conversions on host and device
//   arith = 1 the reference's own: A narrowed by truncation (mem_transfer<bfloat16, float>, bfAintBGemm.cc:88), fp32 scales
//             on the device (:27,101), bfaintb_gemm_reference (truncating kernel arithmetic); 8-bit codes, per column only.
//             With data = 0 the validation is the reference's, operand for operand (:198-214).
// Metrics are the reference's (:186-195) in decimal units with the scale bytes counted.
// Validation compares with a host GEMM supplied by the caller of driver_main: the shipped binary passes the
// harness's own gemm_rrr (host_ref.hpp), the test build the CPU checker's.  Return code: 0, 1 when a launch
// or the validation failed, 2 for a bad command line.
#pragma once
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <iostream>
#include <vector>

#include "../../include/bfaintb_gemm.h"
#include "datatype.hpp"
#include "gemm_tensor_layout.hpp"
#include "gpu_utils.hpp"
#include "mem_transfer.hpp"
#include "random_gen.hpp"
#include "simple_device_mem.hpp"
#include "validation.hpp"

namespace bfaintb_host {

using Row = gemm_layout::gemm::RowMajor;
using Col = gemm_layout::gemm::ColumnMajor;
using ALayout = Row;
using BLayout = Row;
using ScaleLayout = Row;
using CLayout = Row;
using ADataType = bfloat16;
using BDataType = std::int8_t;
using ScaleDataType = bfloat16;  // the reference keeps fp32 scales on the device (bfAintBGemm.cc:27); this build's contract is bf16
using CDataType = bfloat16;

// A host GEMM with the signature of the reference's gemm_rrr (host_ref.hpp:3-13).
struct HostChecker {
    void (*gemm_rrr)(float* c, const float* a, const float* b, const float* scale, std::size_t m, std::size_t n, std::size_t k,
                     std::size_t lda, std::size_t ldb, std::size_t ldc);
};

struct DriverResult {
    float ms_per_launch = 0.f;
    double tflops = 0.0, gbs = 0.0;
    int validated = -1;  // -1 not asked, 0 fail, 1 valid
};

inline int driver_main(int argc, char** argv, const HostChecker* checker, DriverResult* result = nullptr)
{
    int validation = 0, m = 32, n = 64 * 2, k = 256 * 2;
    if (argc >= 2) validation = std::atoi(argv[1]);
    if (argc >= 5) { m = std::atoi(argv[2]); n = std::atoi(argv[3]); k = std::atoi(argv[4]); }
    int lda = k, ldb = n, ldc = n;
    if (argc >= 8) { lda = std::atoi(argv[5]); ldb = std::atoi(argv[6]); ldc = std::atoi(argv[7]); }
    int weight_bits = 8, group_size = 0, data = 0, total_loop = 10;
    unsigned long long seed = 0;
    if (argc >= 9) weight_bits = std::atoi(argv[8]);
    if (argc >= 10) group_size = std::atoi(argv[9]);
    if (argc >= 11) data = std::atoi(argv[10]);
    if (argc >= 12) seed = std::strtoull(argv[11], nullptr, 10);
    if (argc >= 13) total_loop = std::atoi(argv[12]);
    const bool ref_arith = argc >= 14 && std::atoi(argv[13]) != 0;
    if (ref_arith && (weight_bits != 8 || group_size != 0)) { std::printf("arith 1 is 8-bit codes with one scale per column\n"); return 2; }
    const std::size_t scale_elem_bytes = ref_arith ? sizeof(float) : sizeof(ScaleDataType);
    const int warm_ups = 10;
    if (m <= 0 || n <= 0 || k <= 0 || total_loop <= 0) { std::printf("bad sizes\n"); return 2; }
    if (validation && (checker == nullptr || checker->gemm_rrr == nullptr)) {
        std::printf("validation requested, but driver_main was given no host GEMM to compare with\n");
        return 2;
    }
    const int groups = group_size ? k / group_size : 1;
    const int qlo = weight_bits == 8 ? -128 : -8, qhi = weight_bits == 8 ? 127 : 7;

    GPU_CHECK_ERROR(hipSetDevice(0));

    const std::size_t a_elems = gemm_layout::matrix_space_size(m, k, lda, ALayout{});
    const std::size_t b_elems = gemm_layout::matrix_space_size(k, n, ldb, BLayout{});
    const std::size_t c_elems = gemm_layout::matrix_space_size(m, n, ldc, CLayout{});
    const std::size_t s_elems = (std::size_t)groups * n;
    const std::size_t b_bytes = weight_bits == 8 ? b_elems : (std::size_t)k * (ldb / 2);

    SimpleDeviceMem a_device_buf(sizeof(ADataType) * a_elems);
    SimpleDeviceMem b_device_buf(b_bytes);
    SimpleDeviceMem c_device_buf(sizeof(CDataType) * c_elems);
    SimpleDeviceMem scale_device_buf(scale_elem_bytes * s_elems);
    GPU_CHECK_ERROR(a_device_buf.Status()); GPU_CHECK_ERROR(b_device_buf.Status());
    GPU_CHECK_ERROR(c_device_buf.Status()); GPU_CHECK_ERROR(scale_device_buf.Status());

    SimpleHostMem a_host_buf(sizeof(float) * a_elems), b_host_buf(sizeof(float) * (std::size_t)k * ldb);
    SimpleHostMem c_host_buf(sizeof(float) * c_elems), scale_host_buf(sizeof(float) * s_elems);
    float* a_f = static_cast<float*>(a_host_buf.GetBuffer());
    float* b_f = static_cast<float*>(b_host_buf.GetBuffer());
    float* s_f = static_cast<float*>(scale_host_buf.GetBuffer());
    for (std::size_t i = 0; i < a_elems; ++i) a_f[i] = 0.f;
    for (std::size_t i = 0; i < (std::size_t)k * ldb; ++i) b_f[i] = 0.f;

    if (data == 0) {
        rand_vector_2d_int_a(a_f, m, k, lda, seed * 3 + 1);
        rand_vector_2d_int_range(b_f, k, n, ldb, qlo < -2 ? -2 : qlo, 1, seed * 3 + 2);
        rand_vector_2d_int_scale(s_f, groups, n, n, seed * 3 + 3);
    } else {
        rand_vector_2d_normal(a_f, m, k, lda, seed * 3 + 1);
        rand_vector_2d_int_range(b_f, k, n, ldb, qlo, qhi, seed * 3 + 2);
        rand_vector_2d(s_f, groups, n, n, 0.001f, weight_bits == 8 ? 0.01f : 0.02f, seed * 3 + 3);
    }

    SimpleHostMem a_host_buf_to_device(sizeof(ADataType) * a_elems), b_host_buf_to_device(b_bytes);
    SimpleHostMem scale_host_buf_to_device(sizeof(ScaleDataType) * s_elems), c_host_buf_from_device(sizeof(CDataType) * c_elems);
    if (ref_arith) mem_transfer<ADataType, float, SimpleHostMem, SimpleHostMem>(a_host_buf_to_device, a_host_buf, a_elems);
    else mem_transfer_bf16_rne(a_host_buf_to_device, a_host_buf, a_elems);
    mem_transfer_bf16_rne(scale_host_buf_to_device, scale_host_buf, s_elems);  // unused with arith 1: the fp32 scales go as they are
    if (weight_bits == 8) mem_transfer<BDataType, float, SimpleHostMem, SimpleHostMem>(b_host_buf_to_device, b_host_buf, b_elems);
    else mem_transfer_int4(b_host_buf_to_device, b_host_buf, k, n, ldb);

    GPU_CHECK_ERROR(hipMemcpy(a_device_buf.GetBuffer(), a_host_buf_to_device.GetBuffer(), sizeof(ADataType) * a_elems, hipMemcpyHostToDevice));
    GPU_CHECK_ERROR(hipMemcpy(b_device_buf.GetBuffer(), b_host_buf_to_device.GetBuffer(), b_bytes, hipMemcpyHostToDevice));
    GPU_CHECK_ERROR(hipMemcpy(scale_device_buf.GetBuffer(), ref_arith ? scale_host_buf.GetBuffer() : scale_host_buf_to_device.GetBuffer(),
                              scale_elem_bytes * s_elems, hipMemcpyHostToDevice));
    GPU_CHECK_ERROR(hipMemset(c_device_buf.GetBuffer(), 0, sizeof(CDataType) * c_elems));

    const std::size_t ws_bytes = bfaintb_gemm_workspace_bytes(m, n, k, weight_bits, group_size);
    SimpleDeviceMem workspace(ws_bytes);
    GPU_CHECK_ERROR(workspace.Status());
    int rc = bfaintb_workspace_init(workspace.GetBuffer(), ws_bytes, nullptr);
    if (rc) { std::printf("bfaintb_workspace_init: %s\n", bfaintb_error_string(rc)); return 1; }

    auto launch = [&]() {
        if (ref_arith)
            return bfaintb_gemm_reference(c_device_buf.GetBuffer(), a_device_buf.GetBuffer(), b_device_buf.GetBuffer(),
                                          static_cast<const float*>(scale_device_buf.GetBuffer()), m, n, k, lda, ldb, ldc,
                                          workspace.GetBuffer(), ws_bytes, nullptr);
        return bfaintb_gemm(c_device_buf.GetBuffer(), a_device_buf.GetBuffer(), b_device_buf.GetBuffer(), scale_device_buf.GetBuffer(),
                            m, n, k, lda, ldb, ldc, weight_bits, group_size, workspace.GetBuffer(), ws_bytes, nullptr);
    };
    for (int i = 0; i < warm_ups; i++) {
        rc = launch();
        if (rc) { std::printf("bfaintb_gemm failed: [%d] %s\n", rc, bfaintb_error_string(rc)); return 1; }
    }
    hipEvent_t evt_00, evt_11;
    GPU_CHECK_ERROR(hipEventCreate(&evt_00));
    GPU_CHECK_ERROR(hipEventCreate(&evt_11));
    GPU_CHECK_ERROR(hipDeviceSynchronize());
    GPU_CHECK_ERROR(hipEventRecord(evt_00, nullptr));
    int timed_rc = 0;  // the first non-zero return code of the timed launches
    for (int i = 0; i < total_loop; i++) {
        const int r = launch();
        if (r && !timed_rc) timed_rc = r;
    }
    GPU_CHECK_ERROR(hipEventRecord(evt_11, nullptr));
    GPU_CHECK_ERROR(hipEventSynchronize(evt_11));
    GPU_CHECK_ERROR(hipDeviceSynchronize());
    if (timed_rc) { std::printf("bfaintb_gemm failed in the timed loop: [%d] %s\n", timed_rc, bfaintb_error_string(timed_rc)); return 1; }
    float elapsed_ms = 0.f;
    GPU_CHECK_ERROR(hipEventElapsedTime(&elapsed_ms, evt_00, evt_11));
    GPU_CHECK_ERROR(hipEventDestroy(evt_00));
    GPU_CHECK_ERROR(hipEventDestroy(evt_11));

    const float time_per_loop = elapsed_ms / total_loop;
    const double flops = 2.0 * m * n * k;
    const double bytes = 2.0 * ((double)m * k + (double)m * n) + (double)n * k * weight_bits / 8.0 + 2.0 * groups * n;
    const double tflops = flops / (time_per_loop * 1e-3) / 1e12;
    const double bw_gbs = bytes / (time_per_loop * 1e-3) / 1e9;
    std::printf("m: %d, n: %d, k: %d, time: %.3f ms, tflops: %.3f, bw: %.3f GB/s\n", m, n, k, time_per_loop, tflops, bw_gbs);
    const bool decode = bfaintb_gemm_variant(m, n, k, weight_bits, group_size) == BFAINTB_VARIANT_DECODE;
    std::cout << "layouts A/B/scale/C: " << ALayout{} << "/" << BLayout{} << "/" << ScaleLayout{} << "/" << CLayout{}
              << ", weight_bits " << weight_bits << ", group_size " << group_size << (ref_arith ? ", reference arithmetic" : "") << ", variant " << (decode ? "decode" : "prefill")
              << ", roofline: " << (decode ? 100.0 * bw_gbs / 8000.0 : 100.0 * tflops / 2500.0) << " % of "
              << (decode ? "8000 GB/s HBM" : "2500 TFLOP/s bf16 MFMA") << " (cache-hot: the same buffers every launch)\n\n";
    if (result) { result->ms_per_launch = time_per_loop; result->tflops = tflops; result->gbs = bw_gbs; }

    if (validation) {
        GPU_CHECK_ERROR(hipMemcpy(c_host_buf_from_device.GetBuffer(), c_device_buf.GetBuffer(), sizeof(CDataType) * c_elems, hipMemcpyDeviceToHost));
        const bfloat16* a_dev = static_cast<const bfloat16*>(a_host_buf_to_device.GetBuffer());
        const bfloat16* s_dev = static_cast<const bfloat16*>(scale_host_buf_to_device.GetBuffer());
        // what the device multiplies: bf16 activations and bf16 dequantised weights W = bf16(q * scale)
        std::vector<float> a_seen(a_elems), w_seen((std::size_t)k * n), ones(n, 1.0f), c_ref((std::size_t)m * n);
        for (std::size_t i = 0; i < a_elems; ++i) a_seen[i] = type_convert<float>(a_dev[i]);
        for (int ik = 0; ik < k; ++ik)
            for (int in = 0; in < n; ++in) {
                const float q = b_f[(std::size_t)ik * ldb + in];
                if (ref_arith) {  // fp32 scale, product narrowed by truncation
                    w_seen[(std::size_t)ik * n + in] = type_convert<float>(type_convert<bfloat16, float>(q * s_f[in]));
                } else {
                    const float s = type_convert<float>(s_dev[(std::size_t)(group_size ? ik / group_size : 0) * n + in]);
                    w_seen[(std::size_t)ik * n + in] = type_convert<float>(bf16_convert_rtn<bfloat16, float>(q * s));
                }
            }
        if (ref_arith && data == 0) {
            // the reference's own check, operand for operand: the host's float A, float B and float scales (bfAintBGemm.cc:200-209)
            std::vector<float> b_dense((std::size_t)k * n);
            for (int ik = 0; ik < k; ++ik)
                for (int in = 0; in < n; ++in) b_dense[(std::size_t)ik * n + in] = b_f[(std::size_t)ik * ldb + in];
            checker->gemm_rrr(c_ref.data(), a_f, b_dense.data(), s_f, m, n, k, lda, n, n);
        } else {
            checker->gemm_rrr(c_ref.data(), a_seen.data(), w_seen.data(), ones.data(), m, n, k, lda, n, n);
        }
        std::vector<bfloat16> c_dev((std::size_t)m * n);
        const bfloat16* c_raw = static_cast<const bfloat16*>(c_host_buf_from_device.GetBuffer());
        for (int im = 0; im < m; ++im)
            for (int in = 0; in < n; ++in) c_dev[(std::size_t)im * n + in] = c_raw[(std::size_t)im * ldc + in];
        bool res;
        if (data == 0) {
            // the reference's own criterion (exact small-integer data)
            res = valid_vector<CDataType>(c_ref.data(), c_dev.data(), m * n);
        } else {
            // sum_k |a*w| per output, from the same host routine: 12 * 2^-24 of it covers the rounding error of an fp32 sum of those
            // terms on both sides (measured worst: 4.4 such units for the sequential host sum, 1.3 for the device); only outputs
            // that cancel to almost nothing (below an eighth of the rms of C) may lean on it
            std::vector<float> noise((std::size_t)m * n);
            for (auto& v : a_seen) v = std::fabs(v);
            for (auto& v : w_seen) v = std::fabs(v);
            checker->gemm_rrr(noise.data(), a_seen.data(), w_seen.data(), ones.data(), m, n, k, lda, n, n);
            double sq = 0.0;
            for (const float v : c_ref) sq += (double)v * v;
            const float near_zero = 0.125f * (float)std::sqrt(sq / ((double)m * n));
            const float noise_scale = 12.0f * std::ldexp(1.0f, -24);
            for (std::size_t i = 0; i < noise.size(); ++i) noise[i] = std::fabs(c_ref[i]) < near_zero ? noise[i] * noise_scale : 0.0f;
            const UlpReport rep = valid_vector_ulp(c_ref.data(), c_dev.data(), (long)m * n, 2.0, 1e-3, 1e-2, noise.data());
            // outputs that cancel to almost nothing: at most 2 in 10^4 (plus three), each within the noise bound
            const long allowed = (long)((double)m * n * 2e-4) + 3;
            std::printf("ulp check: %ld of %ld outside 2 bf16 ULP (or 1e-2 relative below 1e-3), %ld more only within the fp32 summation "
                        "noise (allowed %ld), worst %.3f ULP at %ld\n", rep.failing, (long)m * n, rep.cancelling, allowed, rep.worst_ulp,
                        rep.worst_index);
            res = rep.failing == 0 && rep.cancelling <= allowed;
        }
        std::printf(",%s \n", res ? "valid" : "fail");
        if (result) result->validated = res ? 1 : 0;
        return res ? 0 : 1;
    }
    return 0;
}

}  // namespace bfaintb_host
