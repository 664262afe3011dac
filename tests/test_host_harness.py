"""The C++ host harness and driver: unit checks on the CPU, end-to-end validation runs on the GPU."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CHECK = os.path.join(ROOT, "tests", "driver_check", "bfAintBGemm_check")
DRIVER = os.path.join(ROOT, "awesome_fusion_amd", "host", "bfAintBGemm")


def test_host_harness_cpp_unit_checks(tmp_path):
    subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "liboracle.so"], check=True, capture_output=True)
    exe = str(tmp_path / "test_host_harness")
    subprocess.run(["g++", "-std=c++17", "-O1", "-ffp-contract=off", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include", "-w",
                    os.path.join(ROOT, "tests", "cpp", "test_host_harness.cc"), "-o", exe,
                    "-L" + os.path.join(ROOT, "oracle"), "-loracle", "-Wl,-rpath," + os.path.join(ROOT, "oracle"),
                    "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,/opt/rocm/lib"], check=True)
    r = subprocess.run([exe], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout[-3000:]
    assert "all checks passed" in r.stdout


def test_driver_and_check_build_compile():
    subprocess.run(["make", "-C", os.path.join(ROOT, "awesome_fusion_amd", "host")], check=True, capture_output=True)
    subprocess.run(["make", "-C", os.path.join(ROOT, "tests", "driver_check")], check=True, capture_output=True)
    assert os.path.exists(DRIVER) and os.path.exists(CHECK)


def run(exe, *args):
    return subprocess.run([exe] + [str(a) for a in args], capture_output=True, text=True, timeout=120)


@pytest.mark.gpu
@pytest.mark.parametrize("args", [
    (1,),                                              # the reference's defaults: m 32, n 128, k 512, data in {-2..1}
    (1, 64, 128, 256),                                 # small-integer regime, prefill variant
    (1, 64, 128, 256, 256, 128, 128, 8, 0, 1, 0),      # config 1: N(0,1) x int8 uniform, per-channel scales, seed 0
    (1, 1, 4096, 4096, 4096, 4096, 4096, 8, 0, 1, 0),  # config 2: decode
    (1, 16, 1024, 2048, 2048, 1024, 1024, 4, 128, 1, 3),   # int4, group 128, decode
    (1, 96, 512, 1024, 1032, 528, 520, 4, 128, 1, 4),  # int4 prefill with padded leading dimensions
    # arith = 1: the reference's harness as it is — truncated A, fp32 scales on the device, bfaintb_gemm_reference
    (1, 32, 128, 512, 512, 128, 128, 8, 0, 0, 0, 10, 1),       # its defaults and data: validated exactly as bfAintBGemm.cc:198-214 does
    (1, 300, 528, 256, 256, 528, 528, 8, 0, 0, 5, 10, 1),      # the same regime on the tiled kernel (k small enough that every
                                                               # sum fits bf16: truncated larger sums fail the reference's 1e-3
                                                               # criterion, for its own kernel as for this one)
    (1, 64, 128, 256, 256, 128, 128, 8, 0, 1, 0, 10, 1),       # config 1 data
    (1, 1, 4096, 4096, 4096, 4096, 4096, 8, 0, 1, 0, 10, 1),   # config 2: decode
])
def test_driver_validates_against_host_gemm(args):
    assert os.path.exists(CHECK), "build tests/driver_check first (make -C tests/driver_check)"
    r = run(CHECK, *args)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert ",valid" in r.stdout
    assert "tflops:" in r.stdout and "bw:" in r.stdout  # the reference's report line


@pytest.mark.gpu
def test_plain_driver_times_but_refuses_validation():
    r = run(DRIVER, 0, 32, 128, 512)
    assert r.returncode == 0 and "m: 32, n: 128, k: 512, time:" in r.stdout
    r = run(DRIVER, 1)
    assert r.returncode == 2 and "without a host GEMM" in r.stdout


@pytest.mark.gpu
def test_driver_reports_library_errors():
    r = run(DRIVER, 0, 32, 100, 512)  # n not a multiple of 16
    assert r.returncode == 1 and "bfaintb_gemm failed" in r.stdout
