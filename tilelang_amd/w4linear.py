"""W4A16 linear layer on the dequantize-GEMV / GEMM kernels: the caller either side of ``dequantize_gemv``.

The weights are quantised once, per (output row, group of ``group_size`` consecutive k), to uint4 codes with an
fp16 scale and either the fixed zero point 8 (``w = (q - 8) * s``, the decode of
examples/dequantize_gemm/quantize/lop3.py:41-75 and the quantiser of ``gen_quant4``,
examples/dequantize_gemm/quantize/utils.py:1-47) or an fp16 integer-valued zero point per group
(``w = (q - z) * s``, lop3.py:136-176), packed two per byte with the even k in the low nibble
(``general_compress``, utils.py:50-67).  ``forward`` is one kernel launch whatever the batch: the library routes
M = 1..2 to the streaming GEMV, small batches to the register-resident / direct-to-LDS kernels and large ones to
the MFMA GEMM.  Same shape of layer as ``BitLinearBitBLAS`` (examples/bitnet-1.58b/utils_quant.py:34-209) with the
4-bit weight format of the dequantize examples instead of the ternary one.
"""

from __future__ import annotations

import torch
from torch import nn

from . import kernels, quantize


def quantize_w4(weight: torch.Tensor, group_size: int = 128, with_zeros: bool = False):
    """``weight[N, K]`` -> ``(codes[N, K] uint8 in 0..15, scale[N, K/g] fp16, zeros[N, K/g] fp16 or None)``.

    Without zeros: the symmetric rule of ``gen_quant4`` restricted to what fits a nibble: ``s = absmax / 7``,
    ``q = clamp(round(w / s) + 8, 1, 15)``.  With zeros: the asymmetric min/max rule, ``s = (max - min) / 15``,
    ``z = clamp(round(-min / s), 0, 15)`` (integer-valued, so ``q - z`` is exact in fp16),
    ``q = clamp(round(w / s) + z, 0, 15)``.
    """
    N, K = weight.shape
    if K % group_size:
        raise ValueError(f"quantize_w4: K={K} is not a multiple of group_size={group_size}")
    g = weight.float().reshape(N, K // group_size, group_size)
    if with_zeros:
        lo = g.amin(dim=2, keepdim=True).clamp(max=0)
        hi = g.amax(dim=2, keepdim=True).clamp(min=0)
        s = ((hi - lo) / 15).clamp(min=1e-8).half().float()
        z = torch.round(-lo / s).clamp(0, 15)
        q = (torch.round(g / s) + z).clamp(0, 15)
        return (q.reshape(N, K).to(torch.uint8), s.reshape(N, -1).half().contiguous(), z.reshape(N, -1).half().contiguous())
    s = (g.abs().amax(dim=2, keepdim=True) / 7).clamp(min=1e-8).half().float()
    q = (torch.round(g / s) + 8).clamp(1, 15)
    return q.reshape(N, K).to(torch.uint8), s.reshape(N, -1).half().contiguous(), None


def dequantize_w4_reference(codes: torch.Tensor, scale: torch.Tensor, zeros: torch.Tensor | None, group_size: int) -> torch.Tensor:
    """Torch restatement of the tile the kernels multiply with: ``fp16((q - 8) * s)`` or ``fp16(fp16(q - z) * s)``."""
    N, K = codes.shape
    s = scale.repeat_interleave(group_size, dim=1)
    if zeros is None:
        return ((codes.to(torch.float16) - 8).float() * s.float()).half()
    z = zeros.repeat_interleave(group_size, dim=1)
    return ((codes.to(torch.float16) - z).float() * s.float()).half()


class W4A16Linear(nn.Module):
    """``out = x @ dequant(qweight, scales[, zeros]).T (+ bias)`` in fp16 with fp32 accumulation."""

    def __init__(self, in_features: int, out_features: int, group_size: int = 128, with_zeros: bool = False, bias: bool = False):
        super().__init__()
        if in_features % 128 != 0:
            raise ValueError(f"W4A16Linear: in_features={in_features} must be a multiple of 128")
        if in_features % group_size != 0 or group_size % 32 != 0:
            raise ValueError(f"W4A16Linear: group_size={group_size} must divide in_features and be a multiple of 32")
        self.in_features, self.out_features = in_features, out_features
        self.group_size, self.with_zeros = group_size, with_zeros
        groups = in_features // group_size
        self.register_buffer("qweight", torch.zeros((out_features, in_features // 2), dtype=torch.int8))
        self.register_buffer("scales", torch.ones((out_features, groups), dtype=torch.float16))
        self.register_buffer("zeros", torch.full((out_features, groups), 8.0, dtype=torch.float16) if with_zeros else None)
        # buffers, so that .to(device) and state_dict carry them with the packed weights
        self.register_buffer("bias", torch.zeros((out_features,), dtype=torch.float16) if bias else None)
        self._kernels = {}

    @classmethod
    def from_linear(cls, linear: nn.Module, group_size: int = 128, with_zeros: bool = False) -> "W4A16Linear":
        """From a layer holding the fp weight (``.weight [out, in]``, optional ``.bias``)."""
        layer = cls(linear.in_features, linear.out_features, group_size=group_size, with_zeros=with_zeros,
                    bias=getattr(linear, "bias", None) is not None)
        layer.load_float_weight(linear.weight, getattr(linear, "bias", None))
        return layer

    def load_float_weight(self, weight: torch.Tensor, bias: torch.Tensor | None = None) -> None:
        dev = self.qweight.device
        codes, s, z = quantize_w4(weight.detach().cpu(), self.group_size, self.with_zeros)
        self.qweight = quantize.general_compress(codes.to(torch.int8), 4).to(dev).contiguous()
        self.scales = s.to(dev)
        if self.with_zeros:
            self.zeros = z.to(dev)
        self.bias = None if bias is None else bias.detach().to(device=dev, dtype=torch.float16)

    def _get_kernel(self, M: int):
        k = self._kernels.get(M)
        if k is None:
            k = kernels.dequantize_gemv(M, self.out_features, self.in_features, group_size=self.group_size,
                                        source_format="uint" if self.with_zeros else "int", with_scaling=True,
                                        with_zeros=self.with_zeros)
            self._kernels[M] = k
        return k

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        x = input.reshape(-1, self.in_features)
        if x.dtype != torch.float16:
            x = x.to(torch.float16)
        x = x.contiguous()
        out = torch.empty((x.shape[0], self.out_features), dtype=torch.float16, device=x.device)
        kern = self._get_kernel(x.shape[0])
        if self.with_zeros:
            kern(x, self.qweight, self.scales, self.zeros, out)
        else:
            kern(x, self.qweight, self.scales, out)
        if self.bias is not None:
            out += self.bias.view(1, -1).expand_as(out)
        return out.reshape(*input.shape[:-1], self.out_features)
