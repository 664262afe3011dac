// bfAintBGemm: benchmark driver for the MI355X library (see bfAintBGemm_driver.hpp for the command
// line, which is the reference's, /root/reference/bfAintBGemm/bfAintBGemm.cc:38-58, plus trailing
// extras).  This binary carries no host GEMM, so it times and reports but does not validate.
#include "bfAintBGemm_driver.hpp"

int main(int argc, char** argv) { return bfaintb_host::driver_main(argc, argv, nullptr); }
