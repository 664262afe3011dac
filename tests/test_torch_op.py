"""The PyTorch binding (awesome_fusion_amd/torch_op.py): registration, shape inference and the host-side
quantiser on the CPU; the operator and the linear layer against the oracle on the GPU."""
import numpy as np
import pytest
import torch

import awesome_fusion_amd.torch_op as top
from helpers import Problem, assert_close_ulp, run_gemm, widen


def _args(m=4, n=32, k=64, bits=8, group=0, device="cpu"):
    groups = k // group if group else 1
    return (torch.zeros((m, k), dtype=torch.bfloat16, device=device), torch.zeros((k, n * bits // 8), dtype=torch.uint8, device=device),
            torch.zeros((groups, n), dtype=torch.bfloat16, device=device), bits, group)


def test_operator_is_registered_and_infers_shapes():
    assert hasattr(torch.ops.awesome_fusion, "bfaintb_gemm")
    out = torch.ops.awesome_fusion.bfaintb_gemm(*_args(5, 48, 128, 4, 64, device="meta"))
    assert out.shape == (5, 48) and out.dtype == torch.bfloat16 and out.device.type == "meta"


def test_operator_rejects_bad_arguments_and_cpu_tensors():
    a, b, s, bits, g = _args()
    with pytest.raises(RuntimeError):           # no CPU implementation, and no silent fallback
        torch.ops.awesome_fusion.bfaintb_gemm(a, b, s, bits, g)
    with pytest.raises(Exception):
        torch.ops.awesome_fusion.bfaintb_gemm(a.float(), b, s, bits, g)
    with pytest.raises(Exception):
        torch.ops.awesome_fusion.bfaintb_gemm(a, b, s[:, :16], bits, g)
    with pytest.raises(Exception):
        torch.ops.awesome_fusion.bfaintb_gemm(a, b, s, 5, g)


@pytest.mark.parametrize("bits,group", [(8, 0), (8, 64), (4, 0), (4, 32)])
def test_quantize_weight_wire_format_and_error_bound(bits, group):
    gen = torch.Generator().manual_seed(3)
    w = torch.randn((48, 128), generator=gen) * 0.05            # [n_out, k_in]
    b, s = top.quantize_weight(w, bits, group)
    k, n = 128, 48
    groups = k // group if group else 1
    assert b.shape == (k, n * bits // 8) and b.dtype == torch.uint8 and s.shape == (groups, n) and s.dtype == torch.bfloat16
    bn = b.numpy()
    if bits == 8:
        q = bn.astype(np.int16) - 128                            # excess-128 (mem_transfer.hpp:30)
    else:
        q = np.empty((k, n), np.int16)
        q[:, 0::2] = (bn & 15).astype(np.int16) - 8              # even column in the low nibble, excess-8
        q[:, 1::2] = (bn >> 4).astype(np.int16) - 8
    sf = s.float().numpy()
    rows_per = group if group else k
    deq = q.astype(np.float32) * np.repeat(sf, rows_per, axis=0)
    err = np.abs(deq - w.t().numpy())
    assert np.all(err <= 0.5 * np.repeat(sf, rows_per, axis=0) * 1.01 + 1e-7), "more than half a step off"
    assert q.min() >= (-128 if bits == 8 else -8) and q.max() <= (127 if bits == 8 else 7)


@pytest.mark.gpu
@pytest.mark.parametrize("m,n,k,bits,group", [(1, 4096, 4096, 8, 0), (7, 528, 1024, 4, 128), (300, 512, 512, 8, 0)])
def test_operator_matches_library_and_oracle(m, n, k, bits, group):
    p = Problem(m, n, k, bits, group, seed=500 + m)
    a = torch.from_numpy(p.a_bf.view(np.int16)).cuda().view(torch.bfloat16)
    b = torch.from_numpy(p.b_bytes).cuda()
    s = torch.from_numpy(p.s_bf.view(np.int16)).cuda().view(torch.bfloat16)
    for _ in range(2):  # the second call reuses the cached workspace
        c = torch.ops.awesome_fusion.bfaintb_gemm(a, b, s, bits, group)
        torch.cuda.synchronize()
        bits_out = c.view(torch.int16).cpu().numpy().view(np.uint16)
        assert np.array_equal(bits_out, run_gemm(p)), "operator and direct C-ABI call disagree"
    assert_close_ulp(p, bits_out, f"torch operator m={m}")


@pytest.mark.gpu
def test_quant_linear_forward():
    torch.manual_seed(0)
    lin = torch.nn.Linear(512, 256, bias=True).cuda()
    ql = top.QuantLinear.from_float(lin, weight_bits=8, group_size=128)
    x = torch.randn((2, 5, 512), device="cuda")
    y = ql(x)
    assert y.shape == (2, 5, 256) and y.dtype == torch.bfloat16
    # against torch arithmetic on the dequantised weights (bf16 inputs, fp32 accumulate): loose, the tight
    # comparison against the oracle is the operator test above
    q = ql.qweight.to(torch.int16) - 128
    w = (q.float() * ql.scales.float().repeat_interleave(128, dim=0)).to(torch.bfloat16).float()
    ref = x.to(torch.bfloat16).float().reshape(-1, 512) @ w + ql.bias.float()  # the kernel adds the bias to its fp32 sums
    assert torch.allclose(y.float().reshape(-1, 256), ref, rtol=2e-2, atol=2e-2)
    # and the quantised layer tracks the float layer it came from
    assert (y.float() - lin(x)).abs().max() < 0.05


def test_prepacked_operator_is_registered_and_infers_shapes():
    a = torch.zeros((5, 128), dtype=torch.bfloat16, device="meta")
    packed = torch.zeros(128 * 48 // 2, dtype=torch.uint8, device="meta")
    s = torch.zeros((2, 48), dtype=torch.bfloat16, device="meta")
    out = torch.ops.awesome_fusion.bfaintb_gemm_prepacked(a, packed, s, 4, 64)
    assert out.shape == (5, 48) and out.dtype == torch.bfloat16
    with pytest.raises(Exception):
        torch.ops.awesome_fusion.bfaintb_gemm_prepacked(a, packed[:-1], s, 4, 64)
    with pytest.raises(RuntimeError):           # no CPU implementation
        torch.ops.awesome_fusion.bfaintb_gemm_prepacked(a.to("cpu"), packed.to("cpu"), s.to("cpu"), 4, 64)


@pytest.mark.gpu
@pytest.mark.parametrize("m,n,k,bits,group", [(1, 4096, 4096, 8, 0), (7, 528, 1024, 4, 128), (600, 512, 512, 8, 0)])
def test_prepacked_operator_matches_oracle(m, n, k, bits, group):
    p = Problem(m, n, k, bits, group, seed=700 + m)
    a = torch.from_numpy(p.a_bf.view(np.int16)).cuda().view(torch.bfloat16)
    s = torch.from_numpy(p.s_bf.view(np.int16)).cuda().view(torch.bfloat16)
    packed = top.prepack_weight(torch.from_numpy(p.b_bytes).cuda(), bits)
    c = torch.ops.awesome_fusion.bfaintb_gemm_prepacked(a, packed, s, bits, group)
    torch.cuda.synchronize()
    assert_close_ulp(p, c.view(torch.int16).cpu().numpy().view(np.uint16), f"prepacked torch operator m={m}")


@pytest.mark.gpu
def test_quant_linear_prepacked_matches_row_major_layer():
    torch.manual_seed(1)
    lin = torch.nn.Linear(512, 256, bias=True).cuda()
    ql = top.QuantLinear.from_float(lin, weight_bits=4, group_size=128)
    x = torch.randn((3, 512), device="cuda")
    y_row = ql(x)
    y_packed = ql.prepack()(x)
    assert ql.prepacked and ql.qweight.dim() == 1
    # same weights, same fp32 accumulation up to summation order: within a bf16 ULP or two of each other
    assert torch.allclose(y_row.float(), y_packed.float(), rtol=2e-2, atol=2e-3)


@pytest.mark.gpu
def test_quant_linear_residual_is_added_before_the_rounding():
    torch.manual_seed(2)
    lin = torch.nn.Linear(512, 256, bias=True).cuda()
    ql = top.QuantLinear.from_float(lin, weight_bits=8, group_size=0)
    x = torch.randn((6, 512), device="cuda")
    r = torch.randn((6, 256), device="cuda").to(torch.bfloat16)
    y = ql(x, residual=r)
    q = ql.qweight.to(torch.int16) - 128
    w = (q.float() * ql.scales.float()).to(torch.bfloat16).float()
    ref = x.to(torch.bfloat16).float() @ w + ql.bias.float() + r.float()
    assert torch.allclose(y.float(), ref, rtol=2e-2, atol=2e-2)
    assert torch.allclose(ql.prepack()(x, residual=r).float(), y.float(), rtol=2e-2, atol=2e-3)
    out = torch.ops.awesome_fusion.bfaintb_gemm(torch.zeros((6, 512), dtype=torch.bfloat16, device="meta"), ql.qweight.to("meta") if not ql.prepacked else torch.zeros((512, 256), dtype=torch.uint8, device="meta"),
                                                ql.scales.to("meta"), 8, 0, None, torch.zeros((6, 256), dtype=torch.bfloat16, device="meta"))
    assert out.shape == (6, 256)


def test_gated_operator_infers_half_width():
    a, b, s_, bits, g = _args(5, 64, 128, 8, 0, device="meta")
    out = torch.ops.awesome_fusion.bfaintb_gemm(a, b, s_, bits, g, None, None, 1)
    assert out.shape == (5, 32)
    with pytest.raises(Exception):
        torch.ops.awesome_fusion.bfaintb_gemm(a, b, s_, bits, g, None, None, 2)


@pytest.mark.gpu
def test_gated_mlp_against_torch():
    """A LLaMA-style gated MLP front half, y = silu(x Wg) * (x Wu), as one GEMM over interleaved (gate, up) columns."""
    torch.manual_seed(3)
    k, n = 512, 256
    wg, wu = torch.randn((n, k)) * 0.05, torch.randn((n, k)) * 0.05
    w = torch.stack((wg, wu), dim=1).reshape(2 * n, k)            # rows 2j, 2j+1 = gate_j, up_j  ->  columns of B
    b, s = top.quantize_weight(w, 8, 0)
    x = torch.randn((9, k)).to(torch.bfloat16)
    y = torch.ops.awesome_fusion.bfaintb_gemm(x.cuda(), b.cuda(), s.cuda(), 8, 0, None, None, 1)
    assert y.shape == (9, n)
    wq = ((b.to(torch.int16) - 128).float() * s.float()).to(torch.bfloat16).float()   # [k, 2n]
    sums = x.float() @ wq
    ref = torch.nn.functional.silu(sums[:, 0::2]) * sums[:, 1::2]
    assert torch.allclose(y.float().cpu(), ref, rtol=2e-2, atol=2e-3)
    yp = torch.ops.awesome_fusion.bfaintb_gemm_prepacked(x.cuda(), top.prepack_weight(b.cuda(), 8), s.cuda(), 8, 0, None, None, 1)
    assert torch.allclose(yp.float(), y.float(), rtol=2e-2, atol=2e-3)
