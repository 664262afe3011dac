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


def test_shipped_host_gemm_matches_the_reference_fixtures(tmp_path, golden_dir):
    """host/host_ref.hpp's gemm_rrr (what the shipped driver validates against), compiled as it is and called through
    ctypes, against outputs the reference's own compiled gemm_rrr wrote into the fixtures: bit for bit, padded leading
    dimensions included."""
    import ctypes as C
    import numpy as np
    src = tmp_path / "wrap.cc"
    src.write_text('#include "%s"\nextern "C" void shipped_gemm_rrr(float* c, const float* a, const float* b, const float* s, '
                   'std::size_t m, std::size_t n, std::size_t k, std::size_t lda, std::size_t ldb, std::size_t ldc) '
                   '{ gemm_rrr(c, a, b, s, m, n, k, lda, ldb, ldc); }\n' % os.path.join(ROOT, "awesome_fusion_amd", "host", "host_ref.hpp"))
    so = str(tmp_path / "libshipped_ref.so")
    subprocess.run(["g++", "-std=c++17", "-O2", "-ffp-contract=off", "-shared", "-fPIC", str(src), "-o", so], check=True)
    fn = C.CDLL(so).shipped_gemm_rrr
    fp = C.POINTER(C.c_float)
    fn.argtypes = [fp, fp, fp, fp] + [C.c_size_t] * 6

    def call(a, b, s, lda=None, ldb=None, ldc=None):
        m, k = a.shape
        n = s.shape[0]
        lda, ldb, ldc = lda or k, ldb or n, ldc or n
        ap = np.zeros((m, lda), np.float32); ap[:, :k] = a
        bp = np.zeros((k, ldb), np.float32); bp[:, :n] = b
        c = np.full((m, ldc), np.float32(-7))
        fn(c.ctypes.data_as(fp), ap.ctypes.data_as(fp), bp.ctypes.data_as(fp), np.ascontiguousarray(s).ctypes.data_as(fp), m, n, k, lda, ldb, ldc)
        assert (c[:, n:] == -7).all()
        return np.ascontiguousarray(c[:, :n])

    from helpers import widen
    g = np.load(f"{golden_dir}/c1_seed0.npz")
    for lds in ((None, None, None), (264, 136, 144)):
        c = call(widen(g["a_bf"]), g["q"].astype(np.float32), widen(g["s_bf"]), *lds)
        assert np.array_equal(c.view(np.uint32), g["c_rrr"].view(np.uint32))
    g = np.load(f"{golden_dir}/int_regime_seed1.npz")
    assert np.array_equal(call(g["a"], g["b"], g["s"]).view(np.uint32), g["c"].view(np.uint32))
    # a transposed-operand or dropped-scale slip fails here: one non-zero product
    a = np.zeros((3, 8), np.float32); a[1, 5] = 3
    b = np.zeros((8, 4), np.float32); b[5, 2] = 7
    want = np.zeros((3, 4), np.float32); want[1, 2] = 3 * (7 * np.float32(0.5))
    assert np.array_equal(call(a, b, np.array([1, 1, 0.5, 1], np.float32)), want)


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
@pytest.mark.parametrize("args", [
    (0, 32, 128, 512),                                 # timing only
    (1,),                                              # validation on the reference's defaults, its own data regime
    (1, 32, 128, 512, 512, 128, 128, 8, 0, 0, 0, 10, 1),   # the reference's check operand for operand (arith = 1)
    (1, 64, 128, 256, 256, 128, 128, 8, 0, 1, 0),      # config 1
    (1, 1, 4096, 4096, 4096, 4096, 4096, 8, 0, 1, 0),  # config 2
])
def test_shipped_driver_times_and_validates_itself(args):
    """The shipped binary (no checker linked: its host GEMM is host/host_ref.hpp) behaves like the reference's:
    `validation` != 0 runs the host GEMM and prints ,valid (bfAintBGemm.cc:198-214)."""
    r = run(DRIVER, *args)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert "time:" in r.stdout and "tflops:" in r.stdout and "bw:" in r.stdout
    assert (",valid" in r.stdout) == bool(args[0])


@pytest.mark.gpu
def test_driver_reports_library_errors():
    r = run(DRIVER, 0, 32, 100, 512)  # n not a multiple of 16
    assert r.returncode == 1 and "bfaintb_gemm failed" in r.stdout
