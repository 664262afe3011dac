"""PyTorch binding of the bfAintBGemm C ABI: a custom operator and a linear layer built on it.

The reference is a stand-alone harness with no framework side; its README names the intended use
("gemm fusion for llm", /root/reference/README.md:2) and its argument block is that of a linear layer's
forward pass: activations A [m, k], weights B [k, n], per-output-channel scale, output C [m, n]
(/root/reference/bfAintBGemm/bfAintBGemm.cc:17-28,119-133).  This module lets such a layer call the
library:

    torch.ops.awesome_fusion.bfaintb_gemm(a, b, scale, weight_bits, group_size, bias=None, residual=None, activation=0) -> c
    torch.ops.awesome_fusion.bfaintb_gemm_prepacked(a, packed, scale, weight_bits, group_size, bias=None, residual=None, activation=0) -> c

``a`` bf16 [m, k] (row stride a multiple of 8 elements), ``b`` uint8 [k, n] (8-bit, excess-128) or
[k, n/2] (4-bit, excess-8, even column in the low nibble), ``scale`` bf16 [groups, n], ``bias`` bf16 [n] and
``residual`` bf16 [m, n] (added to the fp32 sums before the one rounding, inside the kernel); returns bf16 [m, n].  torch supplies the output tensor, the current stream and a per-(device, stream) split-K
workspace; all arithmetic happens in ``libbfaintb_gemm.so``.  There is no CPU implementation: on a CPU
tensor the operator raises.

``quantize_weight`` (host-side helper, symmetric round-to-nearest) and ``QuantLinear`` are conveniences
for trying the kernel on a float model; the quantiser is not part of the reference either.
"""
from typing import Optional

import torch

from .gemm import (gemm as _gemm, gemm_prepacked as _gemm_prepacked, prepack as _prepack, prepack_bytes as _prepack_bytes,
                   prepack_colmajor as _prepack_colmajor,
                   prepacked_workspace_bytes as _prepacked_workspace_bytes,
                   workspace_bytes as _workspace_bytes, workspace_init as _workspace_init)

_LIB_NAME = "awesome_fusion"
_workspaces = {}


def _workspace(device, nbytes):
    """One split-K workspace per (device, stream): calls ordered on a stream may share it, calls on
    different streams may overlap and must not."""
    if nbytes == 0:
        return None
    key = (device.index, torch.cuda.current_stream(device).cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 4 << 20), dtype=torch.uint8, device=device)
        _workspace_init(ws)
        _workspaces[key] = ws
    return ws


def _check(a, b, scale, weight_bits, group_size, bias=None):
    if a.dim() != 2 or b.dim() != 2 or scale.dim() != 2:
        raise ValueError("bfaintb_gemm: a [m, k], b [k, n*bits/8], scale [groups, n] must be 2-D")
    if a.dtype != torch.bfloat16 or scale.dtype != torch.bfloat16 or b.dtype != torch.uint8:
        raise TypeError("bfaintb_gemm: a and scale must be bfloat16, b uint8")
    if weight_bits not in (8, 4):
        raise ValueError("bfaintb_gemm: weight_bits must be 8 or 4")
    k = a.shape[1]
    n = b.shape[1] * (8 // weight_bits)
    groups = k // group_size if group_size else 1
    if b.shape[0] != k or tuple(scale.shape) != (groups, n):
        raise ValueError(f"bfaintb_gemm: shapes do not agree: a {tuple(a.shape)}, b {tuple(b.shape)}, scale {tuple(scale.shape)}")
    if bias is not None and (bias.dtype != torch.bfloat16 or tuple(bias.shape) != (n,)):
        raise ValueError("bfaintb_gemm: bias must be bfloat16 [n]")
    return a.shape[0], n, k


def _out_cols(n, activation):
    """Columns of the output: n, or n / 2 for the SiLU-gate epilogue (activation = 1: columns 2j and 2j+1 of the weights
    are the gate and up projections of output column j)."""
    if activation not in (0, 1):
        raise ValueError("bfaintb_gemm: activation must be 0 (none) or 1 (SiLU gate)")
    return n // 2 if activation == 1 else n


def _check_residual(residual, m, n):
    if residual is None:
        return None
    if residual.dtype != torch.bfloat16 or tuple(residual.shape) != (m, n):
        raise ValueError("bfaintb_gemm: residual must be bfloat16 [m, n]")
    return residual.contiguous()


@torch.library.custom_op(f"{_LIB_NAME}::bfaintb_gemm", mutates_args=())
def bfaintb_gemm(a: torch.Tensor, b: torch.Tensor, scale: torch.Tensor, weight_bits: int, group_size: int,
                 bias: Optional[torch.Tensor] = None, residual: Optional[torch.Tensor] = None, activation: int = 0) -> torch.Tensor:
    m, n, k = _check(a, b, scale, weight_bits, group_size, bias)
    n_out = _out_cols(n, activation)
    residual = _check_residual(residual, m, n_out)
    if not a.is_cuda:
        raise RuntimeError("bfaintb_gemm runs on the GPU only (no CPU implementation)")
    if a.stride(1) != 1 or a.stride(0) % 8 != 0 or a.data_ptr() % 16 != 0:
        a = a.contiguous()
    b = b.contiguous()
    scale = scale.contiguous()
    if bias is not None:
        bias = bias.contiguous()
    c = torch.empty((m, n_out), dtype=torch.bfloat16, device=a.device)
    if m == 0 or n == 0:
        return c
    with torch.cuda.device(a.device):
        need = _workspace_bytes(m, n, k, weight_bits, group_size)
        ws = _workspace(a.device, need)
        _gemm(c, a, b, scale, m, n, k, lda=a.stride(0), weight_bits=weight_bits, group_size=group_size, workspace=ws,
              workspace_nbytes=0 if ws is None else ws.numel(), bias=bias, residual=residual, activation=activation)
    return c


@bfaintb_gemm.register_fake
def _(a, b, scale, weight_bits, group_size, bias=None, residual=None, activation=0):
    m, n, _k = _check(a, b, scale, weight_bits, group_size, bias)
    _check_residual(residual, m, _out_cols(n, activation))
    return a.new_empty((m, _out_cols(n, activation)))


@torch.library.custom_op(f"{_LIB_NAME}::bfaintb_gemm_prepacked", mutates_args=())
def bfaintb_gemm_prepacked(a: torch.Tensor, packed: torch.Tensor, scale: torch.Tensor, weight_bits: int, group_size: int,
                           bias: Optional[torch.Tensor] = None, residual: Optional[torch.Tensor] = None,
                           activation: int = 0) -> torch.Tensor:
    """The same product with the weights in the library's pre-packed order (``prepack_weight``): ``packed`` is a flat
    uint8 tensor of k * n * weight_bits / 8 bytes, n is taken from ``scale``."""
    m, n, k = _check_prepacked(a, packed, scale, weight_bits, group_size, bias)
    n_out = _out_cols(n, activation)
    residual = _check_residual(residual, m, n_out)
    if not a.is_cuda:
        raise RuntimeError("bfaintb_gemm_prepacked runs on the GPU only (no CPU implementation)")
    if a.stride(1) != 1 or a.stride(0) % 8 != 0 or a.data_ptr() % 16 != 0:
        a = a.contiguous()
    packed = packed.contiguous()
    scale = scale.contiguous()
    if bias is not None:
        bias = bias.contiguous()
    c = torch.empty((m, n_out), dtype=torch.bfloat16, device=a.device)
    if m == 0 or n == 0:
        return c
    with torch.cuda.device(a.device):
        ws = _workspace(a.device, _prepacked_workspace_bytes(m, n, k, weight_bits, group_size))
        _gemm_prepacked(c, a, packed, scale, m, n, k, lda=a.stride(0), weight_bits=weight_bits, group_size=group_size, bias=bias,
                        workspace=ws, residual=residual, activation=activation)
    return c


def _check_prepacked(a, packed, scale, weight_bits, group_size, bias=None):
    if a.dim() != 2 or scale.dim() != 2 or packed.dim() != 1:
        raise ValueError("bfaintb_gemm_prepacked: a [m, k], packed [k*n*bits/8], scale [groups, n]")
    if a.dtype != torch.bfloat16 or scale.dtype != torch.bfloat16 or packed.dtype != torch.uint8:
        raise TypeError("bfaintb_gemm_prepacked: a and scale must be bfloat16, packed uint8")
    if weight_bits not in (8, 4):
        raise ValueError("bfaintb_gemm_prepacked: weight_bits must be 8 or 4")
    k, n = a.shape[1], scale.shape[1]
    groups = k // group_size if group_size else 1
    if scale.shape[0] != groups or packed.numel() != k * n * weight_bits // 8:
        raise ValueError(f"bfaintb_gemm_prepacked: shapes do not agree: a {tuple(a.shape)}, packed {packed.numel()} bytes, scale {tuple(scale.shape)}")
    if bias is not None and (bias.dtype != torch.bfloat16 or tuple(bias.shape) != (n,)):
        raise ValueError("bfaintb_gemm_prepacked: bias must be bfloat16 [n]")
    return a.shape[0], n, k


@bfaintb_gemm_prepacked.register_fake
def _(a, packed, scale, weight_bits, group_size, bias=None, residual=None, activation=0):
    m, n, _k = _check_prepacked(a, packed, scale, weight_bits, group_size, bias)
    _check_residual(residual, m, _out_cols(n, activation))
    return a.new_empty((m, _out_cols(n, activation)))


def prepack_weight(b, weight_bits=8, column_major=False):
    """Codes ``b`` on the GPU -> flat packed tensor for ``bfaintb_gemm_prepacked``.  Row-major: uint8 [k, n*bits/8];
    ``column_major``: uint8 [n, k*bits/8] — one row per output feature, the way a Linear keeps its weight (4-bit: two
    consecutive k per byte, low nibble first)."""
    per_byte = 8 // weight_bits
    if column_major:
        n, k = b.shape[0], b.shape[1] * per_byte
    else:
        k, n = b.shape[0], b.shape[1] * per_byte
    nbytes = _prepack_bytes(n, k, weight_bits)
    if nbytes == 0:
        raise ValueError("prepack_weight: the packed order needs n % 16 == 0 and k % 64 == 0 (k % 128 == 0 for 4-bit codes)")
    packed = torch.empty(nbytes, dtype=torch.uint8, device=b.device)
    with torch.cuda.device(b.device):
        if column_major:
            _prepack_colmajor(packed, b.contiguous(), n, k, weight_bits=weight_bits)
        else:
            _prepack(packed, b.contiguous(), n, k, weight_bits=weight_bits)
    return packed


def quantize_weight(weight, weight_bits=8, group_size=0):
    """float weight [n_out, k_in] (a torch Linear's layout) -> (b uint8 [k, n*bits/8], scale bf16 [groups, n]).

    Symmetric: scale = max|w| over the group / qmax, rounded to bf16 first, q = round(w / scale) clamped to the
    code range, stored in the library's wire format (excess-128 bytes; excess-8 nibbles, even column low)."""
    w = weight.detach().float().t().contiguous()  # [k, n]
    k, n = w.shape
    g = group_size if group_size else k
    if k % g or (weight_bits == 4 and n % 2):
        raise ValueError("quantize_weight: group_size must divide k; 4-bit needs an even n")
    qmax = 127 if weight_bits == 8 else 7
    wg = w.view(k // g, g, n)
    scale = (wg.abs().amax(dim=1) / qmax).clamp_min(1e-12).to(torch.bfloat16)  # [groups, n]
    q = torch.round(wg / scale.float()[:, None, :]).clamp_(-qmax - 1, qmax).view(k, n).to(torch.int16)
    if weight_bits == 8:
        b = (q + 128).to(torch.uint8)
    else:
        u = (q + 8).to(torch.uint8)
        b = (u[:, 0::2] | (u[:, 1::2] << 4)).contiguous()
    return b, scale


class QuantLinear(torch.nn.Module):
    """y = x @ dequant(B, scale) (+ bias): a Linear whose weight lives as int8/int4 codes and bf16 scales.

    The bias, if any, is added inside the kernel, to the fp32 sums."""

    def __init__(self, in_features, out_features, weight_bits=8, group_size=0, bias=False, device=None):
        super().__init__()
        if out_features % 16 or in_features % 8:
            raise ValueError("QuantLinear: the kernels need out_features % 16 == 0 (rows of B stay 16-byte aligned) and in_features % 8 == 0")
        groups = in_features // group_size if group_size else 1
        self.in_features, self.out_features = in_features, out_features
        self.weight_bits, self.group_size = weight_bits, group_size
        self.prepacked = False
        self.register_buffer("qweight", torch.zeros((in_features, out_features * weight_bits // 8), dtype=torch.uint8, device=device))
        self.register_buffer("scales", torch.zeros((groups, out_features), dtype=torch.bfloat16, device=device))
        self.bias = torch.nn.Parameter(torch.zeros(out_features, dtype=torch.bfloat16, device=device)) if bias else None

    @classmethod
    def from_float(cls, linear, weight_bits=8, group_size=0):
        q = cls(linear.in_features, linear.out_features, weight_bits, group_size, linear.bias is not None, linear.weight.device)
        b, s = quantize_weight(linear.weight, weight_bits, group_size)
        q.qweight.copy_(b)
        q.scales.copy_(s)
        if linear.bias is not None:
            q.bias.data.copy_(linear.bias.detach().to(torch.bfloat16))
        return q

    def prepack(self):
        """Switches the layer to the pre-packed weight order (on the GPU, once): the row-major codes are replaced."""
        if not self.prepacked:
            self.qweight = prepack_weight(self.qweight, self.weight_bits)
            self.prepacked = True
        return self

    def forward(self, x, residual=None):
        """``residual`` (same shape as the output, bf16) is added inside the kernel, before the rounding."""
        lead = x.shape[:-1]
        op = torch.ops.awesome_fusion.bfaintb_gemm_prepacked if self.prepacked else torch.ops.awesome_fusion.bfaintb_gemm
        if residual is not None:
            residual = residual.reshape(-1, self.out_features).to(torch.bfloat16)
        y = op(x.reshape(-1, self.in_features).to(torch.bfloat16), self.qweight, self.scales, self.weight_bits, self.group_size,
               self.bias, residual)
        return y.reshape(*lead, self.out_features)
