// Test build of the driver: the product's driver_main plus the CPU checker's gemm_rrr restatement
// (oracle/bfaintb_oracle.c) as the host GEMM, which is what enables `validation 1` — the analogue of
// the reference binary validating itself against host_ref.hpp
// (/root/reference/bfAintBGemm/bfAintBGemm.cc:198-214).  Lives under tests/ because only tests may
// link the checker.
#include "../../awesome_fusion_amd/host/bfAintBGemm_driver.hpp"

extern "C" void orc_gemm_rrr(float* c, const float* a, const float* b, const float* scale, std::size_t m, std::size_t n,
                             std::size_t k, std::size_t lda, std::size_t ldb, std::size_t ldc);

int main(int argc, char** argv)
{
    const bfaintb_host::HostChecker checker{&orc_gemm_rrr};
    return bfaintb_host::driver_main(argc, argv, &checker);
}
