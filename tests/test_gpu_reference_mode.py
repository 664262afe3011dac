"""bfaintb_gemm_reference on a real MI355X: the reference kernel's own arithmetic — fp32 scales, W = trunc_bf16(q * scale),
C = trunc_bf16(sum) (bf16gemm_kernel_gfx90a.s:18-55, 597-611) — in every kernel that serves it.

What pins it: the oracle's dequantisation with fp32 scales and truncation (one-hot activations expose W bit for bit: a
bf16-rounded scale or a round-to-nearest narrowing fails), the reference's integer regime with sums that need more than
8 significant bits (exact in fp32, so C must equal the truncated exact integer bit for bit: a rounding epilogue fails),
and on random data the two properties truncation has: within one bf16 unit of the fp32 sequential-K sum, never larger
in magnitude.
"""
import numpy as np
import pytest

import oracle
from helpers import Workspace, from_dev_u16, to_dev, widen

pytestmark = pytest.mark.gpu
_ws = Workspace()


@pytest.fixture(scope="module")
def af():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a device"
    import awesome_fusion_amd as af
    af.lib()  # raises if the HIP library was not built: no fallback
    return af


class RefProblem:
    """Inputs as the reference's harness holds them on the device: bf16 A, excess-128 B, fp32 scales."""

    def __init__(self, m, n, k, seed, regime="normal"):
        rng = np.random.Generator(np.random.PCG64(seed))
        self.m, self.n, self.k = m, n, k
        if regime == "normal":
            a = rng.standard_normal((m, k), dtype=np.float32)
            q = rng.integers(-128, 128, size=(k, n)).astype(np.int8)
            self.scale = rng.uniform(0.001, 0.01, size=n).astype(np.float32)  # 24 significant bits: not bf16 values
        else:  # integers: every product and every partial sum is exact in fp32
            a = rng.integers(-64, 64, size=(m, k)).astype(np.float32)
            q = rng.integers(-2, 2, size=(k, n)).astype(np.int8)
            self.scale = rng.integers(-2, 2, size=n).astype(np.float32)
        self.a_bf = oracle.f32_to_bf16_rtz(a)  # the reference's host conversion (datatype.hpp:46-55)
        self.q = q
        self.b_bytes = oracle.mem_transfer_int8(q.astype(np.float32))
        self.w_bf = oracle.dequant(self.b_bytes, self.scale, k, n, 8, 0, rtz=True)

    def sums(self, threads=8):
        return oracle.gemm_bf16_rows(self.a_bf, self.w_bf, threads=threads)

    def abs_sums(self):
        """sum_k |A||W|: the scale of the fp32 rounding errors two summation orders may differ by."""
        return np.abs(widen(self.a_bf)) @ np.abs(widen(self.w_bf))


def run(af, p, which=0, split=0, ldc=None):
    import torch
    c = torch.full((p.m, p.n if ldc is None else ldc), 0x7FC0, dtype=torch.int16, device="cuda")
    ws = _ws.get(af.workspace_bytes(p.m, p.n, p.k, 8, 0, which, split))
    af.gemm_reference(c, to_dev(p.a_bf), to_dev(p.b_bytes), torch.from_numpy(p.scale).cuda(), p.m, p.n, p.k, ldc=ldc, workspace=ws,
                      which=which, force_split_k=split)
    torch.cuda.synchronize()
    return from_dev_u16(c)


def assert_truncated(sums, abs_sums, c_bits, what):
    """|C - sum| < 1 bf16 unit of the sum (plus fp32 summation-order noise), and |C| <= |sum| up to that noise."""
    ref = np.asarray(sums, np.float64)
    got = widen(c_bits).astype(np.float64)
    _, e = np.frexp(np.abs(ref))
    ulp = np.ldexp(1.0, e - 8)                    # bf16: 8 significant bits
    noise = 1e-6 * np.asarray(abs_sums, np.float64) + 1e-30   # 16 fp32 units of the terms' magnitude: two summation orders
    err = np.abs(got - ref)
    bad = np.flatnonzero(err.ravel() >= (ulp + noise).ravel())
    assert bad.size == 0, f"{what}: {bad.size} outputs off by a bf16 unit or more, worst {np.max(err / ulp):.3f}"
    grown = np.flatnonzero((np.abs(got) > np.abs(ref) + noise).ravel())
    assert grown.size == 0, f"{what}: {grown.size} outputs larger in magnitude than the sum: not truncated"
    # and truncation it is, not rounding to nearest: about half of the outputs sit more than half a unit below the sum
    far = np.count_nonzero(err > 0.5 * ulp + noise)
    assert far > 0.3 * ref.size, f"{what}: only {far} of {ref.size} outputs more than half a unit from the sum"


VARIANTS = [("decode", 16, 0), ("decode", 32, 0), ("decode", 64, 0), ("prefill_256", 64, 0), ("prefill_128", 64, 0)]


@pytest.mark.parametrize("which,m,split", VARIANTS)
def test_dequantisation_is_the_reference_kernels_bit_for_bit(af, which, m, split):
    """One-hot activations: C[i, :] = W[k_i, :], nothing to sum and nothing left to truncate."""
    which = {"decode": af.DECODE, "prefill_256": af.PREFILL_256, "prefill_128": af.PREFILL_128}[which]
    k, n = 256, 512
    p = RefProblem(m, n, k, seed=11)
    bf = oracle.dequant(p.b_bytes, oracle.f32_to_bf16_rne(p.scale.reshape(1, n)), k, n, 8, 0)
    assert np.count_nonzero(bf != p.w_bf) > 0.2 * k * n, "the test data must tell the two contracts apart"
    for base in range(0, k, m):
        a = np.zeros((m, k), np.float32)
        rows = (base + np.arange(m)) % k
        a[np.arange(m), rows] = 1.0
        p.a_bf = oracle.f32_to_bf16_rtz(a)
        assert np.array_equal(run(af, p, which, split), p.w_bf[rows]), f"rows {base}.. differ"


@pytest.mark.parametrize("m,n,k,which,split", [
    (1, 512, 2048, "decode", 0), (8, 256, 4096, "decode", 4), (32, 528, 1024, "decode", 2), (100, 272, 512, "decode", 0),
    (300, 528, 512, "prefill_256", 0), (300, 528, 512, "prefill_128", 0), (64, 128, 256, "auto", 0), (2100, 2064, 256, "auto", 0)])
def test_integer_regime_is_exact_and_truncated(af, m, n, k, which, split):
    """Integers keep every fp32 sum exact whatever the order, so C is the truncated exact sum bit for bit — in every
    kernel, with and without split-K.  Sums reach a few thousand: most need more than bf16's 8 bits."""
    which = {"auto": af.AUTO, "decode": af.DECODE, "prefill_256": af.PREFILL_256, "prefill_128": af.PREFILL_128}[which]
    p = RefProblem(m, n, k, seed=m + n + k, regime="int")
    exact = (p.a_bf.astype(np.uint32) << 16).view(np.float32).astype(np.float64) @ (p.q.astype(np.float64) * p.scale.astype(np.float64))
    assert np.max(np.abs(exact)) < 2 ** 24
    want = oracle.f32_to_bf16_rtz(exact.astype(np.float32))
    assert np.count_nonzero(want != oracle.f32_to_bf16_rne(exact.astype(np.float32))) > 0.05 * m * n, "sums must not all fit bf16"
    # gemm_rrr on the reference's own operands (float A, float B, float scale) gives the same integers
    assert np.array_equal(oracle.gemm_rrr(widen(p.a_bf), p.q.astype(np.float32), p.scale), exact.astype(np.float32))
    assert np.array_equal(run(af, p, which, split), want)


@pytest.mark.parametrize("m,n,k,which", [
    (1, 4096, 4096, "auto"), (16, 1040, 2048, "auto"), (80, 528, 1024, "auto"), (700, 784, 448, "auto"),
    (260, 272, 320, "prefill_256"), (260, 272, 320, "prefill_128"), (4096, 4096, 4096, "auto")])
def test_random_data_is_within_one_unit_and_never_larger(af, m, n, k, which):
    which = {"auto": af.AUTO, "prefill_256": af.PREFILL_256, "prefill_128": af.PREFILL_128}[which]
    p = RefProblem(m, n, k, seed=3 * m + n)
    assert_truncated(p.sums(threads=16), p.abs_sums(), run(af, p, which), f"reference arithmetic {m}x{n}x{k}")


def test_padding_of_c_is_left_alone(af):
    p = RefProblem(40, 272, 256, seed=5)
    c = run(af, p, ldc=288)
    assert np.all(c[:, 272:] == 0x7FC0)
    assert np.array_equal(c[:, :272], run(af, p))
