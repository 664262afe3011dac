"""Shared test plumbing: seeded inputs in the wire formats, device round trips, comparisons.

Inputs are made with numpy's PCG64 and converted with the oracle's restatements of the reference's
host converters; the GPU side is reached only through the C ABI (awesome_fusion_amd.gemm is a
ctypes shim over it).
"""
import numpy as np

import oracle


def widen(bits):
    return (np.asarray(bits, np.uint16).astype(np.uint32) << 16).view(np.float32)


class Problem:
    """One GEMM instance in device wire formats plus what the oracle needs."""

    def __init__(self, m, n, k, bits=8, group_size=0, seed=0, scale_lo=0.001, scale_hi=0.01, regime="normal"):
        rng = np.random.Generator(np.random.PCG64(seed))
        self.m, self.n, self.k, self.bits, self.group_size = m, n, k, bits, group_size
        groups = k // group_size if group_size else 1
        lo, hi = (-128, 128) if bits == 8 else (-8, 8)
        if regime == "normal":
            a = rng.standard_normal((m, k), dtype=np.float32)
            q = rng.integers(lo, hi, size=(k, n), dtype=np.int64).astype(np.int8)
            s = rng.uniform(scale_lo, scale_hi, size=(groups, n)).astype(np.float32)
        elif regime == "small_int":  # the reference's own test data: everything in {-2,-1,0,1}
            a = rng.integers(-2, 2, size=(m, k)).astype(np.float32)
            q = rng.integers(-2, 2, size=(k, n)).astype(np.int8)
            s = rng.integers(-2, 2, size=(groups, n)).astype(np.float32)
        else:
            raise ValueError(regime)
        self.a_bf = oracle.f32_to_bf16_rne(a)
        self.q = q
        self.s_bf = oracle.f32_to_bf16_rne(s)
        if bits == 8:
            self.b_bytes = oracle.mem_transfer_int8(q.astype(np.float32))
        else:
            self.b_bytes = oracle.pack_int4(q)
        self._w = None
        self.bias_bf = None  # optional bf16 [n] bias (set by with_bias)
        self.residual_bf = None  # optional bf16 [m, n] residual (set by with_residual)

    def with_bias(self, seed=1, lo=-1.0, hi=1.0):
        rng = np.random.Generator(np.random.PCG64(seed))
        self.bias_bf = oracle.f32_to_bf16_rne(rng.uniform(lo, hi, size=(self.n,)).astype(np.float32))
        return self

    def with_residual(self, seed=2, lo=-2.0, hi=2.0):
        rng = np.random.Generator(np.random.PCG64(seed))
        self.residual_bf = oracle.f32_to_bf16_rne(rng.uniform(lo, hi, size=(self.m, self.n)).astype(np.float32))
        return self

    @property
    def w_bf(self):
        if self._w is None:
            self._w = oracle.dequant(self.b_bytes, self.s_bf, self.k, self.n, self.bits, self.group_size)
        return self._w

    def c_ref(self, rows=None, threads=8):
        a = self.a_bf if rows is None else self.a_bf[rows]
        return oracle.gemm_bf16_rows(a, self.w_bf, threads=threads)


def to_dev(x):
    import torch
    x = np.ascontiguousarray(x)
    if x.dtype == np.uint16:
        return torch.from_numpy(x.view(np.int16)).cuda()
    return torch.from_numpy(x).cuda()


def from_dev_u16(t):
    return t.cpu().numpy().view(np.uint16)


class Workspace:
    """A zero-initialised device scratch, grown on demand."""

    def __init__(self):
        self.t = None

    def get(self, nbytes):
        import torch
        import awesome_fusion_amd as af
        if nbytes == 0:
            return None
        if self.t is None or self.t.numel() < nbytes:
            self.t = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device="cuda")
            af.workspace_init(self.t)
        return self.t


_ws = Workspace()


def run_gemm(p, which=0, force_split_k=0, lda=None, ldb=None, ldc=None, a_dev=None, b_dev=None, s_dev=None, c_fill=None, activation=0):
    """Runs the library on Problem p; returns C as uint16 bits [m, ldc or n]."""
    import torch
    import awesome_fusion_amd as af
    m, n, k = p.m, p.n, p.k
    a_dev = to_dev(p.a_bf) if a_dev is None else a_dev
    b_dev = to_dev(p.b_bytes) if b_dev is None else b_dev
    s_dev = to_dev(p.s_bf) if s_dev is None else s_dev
    ldc_ = (n // 2 if activation else n) if ldc is None else ldc
    c_dev = torch.full((m, ldc_), 0x7FC0 if c_fill is None else c_fill, dtype=torch.int16, device="cuda")
    ws = _ws.get(af.workspace_bytes(m, n, k, p.bits, p.group_size, which, force_split_k))
    bias_dev = None if p.bias_bf is None else to_dev(p.bias_bf)
    res_dev = None if p.residual_bf is None else to_dev(p.residual_bf)
    af.gemm(c_dev, a_dev, b_dev, s_dev, m, n, k, lda, ldb, ldc, p.bits, p.group_size, ws, None, None, which, force_split_k,
            bias=bias_dev, residual=res_dev, activation=activation)
    torch.cuda.synchronize()
    return from_dev_u16(c_dev)


def ulp_violations(c_ref, c_bits, max_ulp=2.0, small_abs=1e-3, small_rel=1e-2):
    """Flat indices failing the stated acceptance bound: |err| <= 2 bf16 ULP of the fp32-accumulated
    oracle, or relative error <= 1e-2 where |ref| < 1e-3.  (numpy twin of the oracle's C checker.)"""
    r = np.asarray(c_ref, np.float32).ravel().astype(np.float64)
    p = widen(np.asarray(c_bits, np.uint16).ravel()).astype(np.float64)
    err = np.abs(p - r)
    _, e = np.frexp(np.abs(r))
    ulp = np.ldexp(1.0, np.maximum(e - 1, -126) - 7)
    ulp[r == 0] = np.ldexp(1.0, -133)
    ok = (err <= max_ulp * ulp) | ((np.abs(r) < small_abs) & (err <= small_rel * np.abs(r)))
    ok &= np.isfinite(p)
    return np.nonzero(~ok)[0], err / ulp


# what every assert_close_ulp call found, for the acceptance report (tests/conftest.py writes it out at the end of a GPU session)
ACCEPTANCE_LOG = []
NOISE_FACTOR = 2.0   # the escape below: this many times 2^-24 * sum_k |a_k w_k| on top of 2 ULP (worst seen over the GPU suite: 0.61)
NEAR_ZERO = 0.125    # ... and only for outputs below this fraction of rms(C)


def allowed_outside(outputs, rate=3e-5):
    """How many outputs of a check may take the near-zero escape: the rate seen at the full-size benchmark shapes is
    1.4e-5 to 2.1e-5 of the outputs (228 of 16.7 M at config 4, 98 of 4.6 M at config 5); allowed is 3e-5 of them plus
    four standard deviations of a count of that mean, and a handful for small problems — so that a kernel whose
    cancelling outputs are a few times worse than today's fails at the sizes where it can be told from chance
    (config 4: 593 allowed against 228 seen; the old cap of 2e-4 allowed 3355)."""
    mean = rate * outputs
    return max(3, int(mean + 4.0 * np.sqrt(mean)))


def assert_close_ulp(p, c_bits, what, rows=None, threads=8):
    """The acceptance bound of this build: every output within 2 bf16 ULP of the fp32
    sequential-K oracle, or within 1e-2 relative where |ref| < 1e-3.

    No summation order other than the oracle's own can meet that bound for outputs that cancel to
    (almost) nothing: there a bf16 ULP is smaller than the fp32 rounding noise of the K-term sum on
    EITHER side.  Such outputs are rare (counted, capped by allowed_outside(), and recorded in
    ACCEPTANCE_LOG); each must be small (|ref| < rms(C) * NEAR_ZERO: an output of ordinary size has no such excuse)
    and must lie within 2 ULP + NOISE_FACTOR * 2^-24 * sum_k |a_k w_k| of the fp64-accumulated value.  The second
    term is a few times the rounding error an fp32 sum of those terms makes in any order (measured worst
    over the benchmark shapes: 1.3 of these units for the device, 4.4 for the sequential oracle); one
    dropped or doubled term of ordinary size is a thousand of them.
    Returns (worst error in ULP among the outputs inside the bound, number of outputs that took the escape)."""
    a = p.a_bf if rows is None else p.a_bf[rows]
    c_ref = oracle.gemm_bf16_rows(a, p.w_bf, threads=threads)
    bias = None if p.bias_bf is None else widen(p.bias_bf)
    if bias is not None:
        c_ref = (c_ref + bias[None, :]).astype(np.float32)  # one fp32 addition after the sum, before the rounding to bf16
    res = None if p.residual_bf is None else widen(p.residual_bf if rows is None else p.residual_bf[rows])
    if res is not None:
        c_ref = (c_ref + res).astype(np.float32)            # and one more for the residual
    bad, ulps = ulp_violations(c_ref, c_bits)
    nbad_c, _, _ = oracle.check_ulp(c_ref, c_bits)
    assert nbad_c == len(bad), "C and numpy acceptance checks disagree"
    # (a handful is always allowed: over 4000 random problems of a few thousand outputs each, six had 2 or 3 such outputs)
    assert len(bad) <= allowed_outside(c_ref.size), \
        f"{what}: {len(bad)} of {c_ref.size} outputs outside 2 ULP (worst {ulps.max():.2f} ULP)"
    worst_units = 0.0
    if len(bad):
        n = c_ref.shape[1]
        rms = float(np.sqrt(np.mean(c_ref.astype(np.float64) ** 2)))
        af_, wf_ = widen(a).astype(np.float64), widen(p.w_bf).astype(np.float64)
        got = widen(np.asarray(c_bits, np.uint16).ravel()[bad]).astype(np.float64)
        for flat, g in zip(bad, got):
            i, j = divmod(int(flat), n)
            assert abs(float(c_ref[i, j])) < NEAR_ZERO * rms, \
                f"{what}: output ({i},{j}) = {g!r} is outside 2 ULP of {c_ref[i, j]!r} and not near zero (rms of C {rms:.3g})"
            terms = af_[i] * wf_[:, j]
            exact = terms.sum() + (0.0 if bias is None else float(bias[j])) + (0.0 if res is None else float(res[i, j]))
            _, e = np.frexp(abs(exact))
            unit = 2.0 ** -24 * np.abs(terms).sum()
            tol = 2.0 * np.ldexp(1.0, max(int(e) - 1, -126) - 7) + NOISE_FACTOR * unit
            worst_units = max(worst_units, abs(g - exact) / unit)
            assert abs(g - exact) <= tol, f"{what}: output ({i},{j}) = {g!r}, exact {exact!r}, fp32 oracle " \
                                          f"{c_ref[i, j]!r}: off by {abs(g - exact):.3e} > {tol:.3e}"
    ok_ulps = np.delete(ulps, bad)
    worst = float(ok_ulps.max()) if ok_ulps.size else 0.0
    ACCEPTANCE_LOG.append({"what": what, "m": int(c_ref.shape[0]), "n": p.n, "k": p.k, "weight_bits": p.bits, "group_size": p.group_size,
                           "outputs": int(c_ref.size), "outside_2ulp": int(len(bad)), "worst_ulp_inside": round(worst, 3),
                           "worst_outside_vs_fp64_in_units_of_2^-24_sum_abs": round(float(worst_units), 3)})
    return worst, len(bad)


def gated_reference(p, rows=None, threads=8):
    """fp64 silu(gate) * up (+ residual) from the oracle's fp32 sums (+ bias): columns (2j, 2j+1) of the problem are
    (gate, up) of output column j.  Also returns the tolerance that goes with it: 2 bf16 ULP of the result plus what
    the fp32 summation noise of either sum (sqrt(K) * 2^-24 * sum_k |a_k w_k|) can move it by, plus 4e-6 relative
    for the device's fast exponential and reciprocal, plus an absolute floor of 1e-30 * (1 + |gate * up|): the hardware's
    exponential and reciprocal flush subnormal results, so silu of a gate below about -87 comes out as zero where the
    exact value is of the order of 1e-36."""
    a = p.a_bf if rows is None else p.a_bf[rows]
    s_ref = oracle.gemm_bf16_rows(a, p.w_bf, threads=threads)
    if p.bias_bf is not None:
        s_ref = (s_ref + widen(p.bias_bf)[None, :]).astype(np.float32)
    absum = oracle.gemm_bf16_rows(a & 0x7FFF, p.w_bf & 0x7FFF, threads=threads).astype(np.float64)
    noise = np.sqrt(p.k) * 2.0 ** -24 * absum + np.abs(s_ref) * 2.0 ** -23
    g, u = s_ref[:, 0::2].astype(np.float64), s_ref[:, 1::2].astype(np.float64)
    sig = 1.0 / (1.0 + np.exp(-g))
    out = g * sig * u
    dsilu = sig * (1.0 + g * (1.0 - sig))
    moved = np.abs(dsilu * u) * noise[:, 0::2] + np.abs(g * sig) * noise[:, 1::2]
    if p.residual_bf is not None:
        out = out + widen(p.residual_bf if rows is None else p.residual_bf[rows]).astype(np.float64)
    _, e = np.frexp(np.abs(out))
    ulp = np.ldexp(1.0, np.maximum(e - 1, -126) - 7)
    return out, 2.0 * ulp + 1.1 * moved + 4e-6 * np.abs(out) + 1e-30 * (1.0 + np.abs(g * u))


def assert_close_gated(p, c_bits, what, rows=None, threads=8):
    out, tol = gated_reference(p, rows, threads)
    got = widen(np.asarray(c_bits, np.uint16)).astype(np.float64)
    assert got.shape == out.shape, f"{what}: shape {got.shape} against {out.shape}"
    bad = np.abs(got - out) > tol
    assert not bad.any(), f"{what}: {int(bad.sum())} of {out.size} gated outputs off; worst {np.max(np.abs(got - out) / tol):.2f} x tolerance"
    return float(np.max(np.abs(got - out) / tol))
