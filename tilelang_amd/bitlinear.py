"""BitLinear (BitNet b1.58) layer on the W2A8 kernels: the caller either side of the int8 x 2-bit GEMM.

Twin of ``BitLinearBitBLAS`` of examples/bitnet-1.58b/utils_quant.py:34-209 with the BitBLAS operator replaced by
``libdqgemm.so``: the weights are quantised once to ternary codes (``weight_quant``, :149-154), packed four per
byte (and interleaved for the fast decoder, as the reference's kernels expect), and ``forward`` is two kernel
launches: the activation quantiser (:156-163) and the GEMM with the fused ``post_quant_process`` epilogue
(:165-170).  BitBLAS's own weight transform (``transform_weight``) is third-party and absent; the packed layout
here is the reference examples' ``general_compress`` + ``interleave_weight``.
"""

from __future__ import annotations

import torch
from torch import nn

from . import kernels, quantize


def weight_quant(weight: torch.Tensor) -> torch.Tensor:
    """``round(W / mean|W|)`` clamped to {-1, 0, 1} as int8 (utils_quant.py:149-154)."""
    weight = weight.float()
    s = 1 / weight.abs().mean().clamp(min=1e-5)
    return (weight * s).round().clamp(-1, 1).type(torch.int8)


def activation_quant_reference(x: torch.Tensor, num_bits: int = 8):
    """Torch restatement of utils_quant.py:156-163 (used where no GPU kernel applies, e.g. CPU tensors)."""
    x = x.float()
    qn, qp = -(2 ** (num_bits - 1)), 2 ** (num_bits - 1) - 1
    s = qp / x.abs().max(dim=-1, keepdim=True).values.clamp(min=1e-5)
    return (x * s).round().clamp(qn, qp).type(torch.int8), s


class BitLinear(nn.Module):
    """``out = ((x_q @ W_q.T) / s_a) / s_w (+ bias)`` in fp16 with int8 activations and ternary weights."""

    def __init__(self, in_features: int, out_features: int, weight_bits: int = 1, input_bits: int = 8, interleave: bool = True,
                 prefill_fragments: bool = False):
        """``prefill_fragments``: hold the packed weights in the matrix instruction's operand order
        (``quantize.prepack_i2_fragments``: ``[ceil(out/32), in/128, 64, 16]`` bytes) INSTEAD of row-major: one copy,
        read at every batch size (decode kernel, K-sliced kernel, tiled kernel), about 10 % faster at a few hundred
        rows.  Needs ``in_features % 2048 == 0``; otherwise the layer keeps the row-major words.  Same results bit for
        bit."""
        super().__init__()
        if input_bits != 8:
            raise ValueError("BitLinear: only 8-bit activations are built")
        if in_features % 128 != 0:
            raise ValueError(f"BitLinear: in_features={in_features} must be a multiple of 128")
        self.in_features, self.out_features = in_features, out_features
        self.weight_bits, self.input_bits = weight_bits, input_bits
        self.interleave = interleave
        self.prefill_fragments = bool(prefill_fragments) and in_features % 2048 == 0 and in_features < 131072
        shape = ((out_features + 31) // 32, in_features // 128, 64, 16) if self.prefill_fragments else (out_features, in_features // 4)
        self.register_buffer("qweight", torch.zeros(shape, dtype=torch.int8))
        self.register_buffer("sw", torch.ones((), dtype=torch.float32))
        self._sw_value = 1.0
        self.bias = None
        self._kernels = {}

    @classmethod
    def from_bit_linear(cls, bitlinear, interleave: bool = True, prefill_fragments: bool = False) -> "BitLinear":
        """From a layer holding the latent fp weight (``.weight [out, in]``, optional ``.bias``), utils_quant.py:99-109."""
        layer = cls(bitlinear.in_features, bitlinear.out_features, interleave=interleave, prefill_fragments=prefill_fragments)
        layer.load_float_weight(bitlinear.weight, getattr(bitlinear, "bias", None))
        return layer

    def load_float_weight(self, weight: torch.Tensor, bias: torch.Tensor | None = None) -> None:
        """``create_bitblas_weights`` with one weight group (utils_quant.py:111-137): s_w, ternary codes, packing."""
        sw = 1 / weight.float().abs().mean().clamp(min=1e-5)
        codes = (weight_quant(weight).to(torch.int16) + 2).to(torch.int8)  # offset-binary: c = w + 2
        packed = quantize.general_compress(codes.cpu(), source_bits=2)
        if self.interleave:
            packed = quantize.interleave_weight(packed, 2, "int8")
        self.load_packed_weight(packed, sw, bias)

    def load_packed_weight(self, packed_rowmajor: torch.Tensor, sw, bias: torch.Tensor | None = None) -> None:
        """Row-major packed words ``[out, in/4]`` (interleaved or not, as the layer was built) and the weight scale;
        stored in the layer's own order."""
        packed = packed_rowmajor.contiguous()
        if self.prefill_fragments:
            packed = quantize.prepack_i2_fragments(packed)
        self.qweight = packed.to(self.qweight.device).contiguous()
        self.sw = torch.as_tensor(sw, dtype=torch.float32).to(self.sw.device)
        self._sw_value = float(self.sw)
        self.bias = None if bias is None else bias.detach().to(self.qweight.device)
        self._kernels.clear()

    def rowmajor_weight(self) -> torch.Tensor:
        """The packed words ``[out, in/4]`` whatever order the layer holds them in."""
        if self.prefill_fragments:
            return quantize.unpack_i2_fragments(self.qweight, self.out_features)
        return self.qweight

    def _load_from_state_dict(self, *args, **kwargs):
        super()._load_from_state_dict(*args, **kwargs)
        # the weight scale is baked into the kernels as a number
        self._sw_value = float(self.sw)
        self._kernels.clear()

    def _get_kernels(self, M: int):
        k = self._kernels.get(M)
        if k is None:
            k = (kernels.bitnet_activation_quant(M, self.in_features),
                 kernels.bitlinear_int8xint2(M, self.out_features, self.in_features, self._sw_value, convention="offset",
                                             interleaved=self.interleave, weight_fragments=self.prefill_fragments))
            self._kernels[M] = k
        return k

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        x = input.reshape(-1, self.in_features)
        if x.dtype != torch.float16:
            x = x.to(torch.float16)
        quant, gemm = self._get_kernels(x.shape[0])
        x_q, s_a = quant(x.contiguous())
        out = gemm(x_q, self.qweight, s_a)
        if self.bias is not None:
            out += self.bias.view(1, -1).expand_as(out)
        return out.reshape(*input.shape[:-1], self.out_features)
