// bfAintBGemm: benchmark driver for the MI355X library (see bfAintBGemm_driver.hpp for the command
// line, which is the reference's, /root/reference/bfAintBGemm/bfAintBGemm.cc:38-58, plus trailing
// extras).  `bfAintBGemm 1 ...` validates the device result against the harness's own host GEMM
// (host_ref.hpp), as the reference binary does (bfAintBGemm.cc:198-214).
#include "bfAintBGemm_driver.hpp"
#include "host_ref.hpp"

int main(int argc, char** argv)
{
    const bfaintb_host::HostChecker checker{&gemm_rrr};
    return bfaintb_host::driver_main(argc, argv, &checker);
}
