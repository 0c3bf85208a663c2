"""torch-CPU restatement of the reference's ``ref_program``s.  TEST INFRASTRUCTURE ONLY.

Used as the timed CPU baseline (``bench.py``'s ``cpu_baseline`` leg) and cross-checked
against ``oracle/dq_oracle.py`` in the tests; nothing that ships may import it.  Same
structure as the reference programs: unpack / dequantise with torch ops, ``torch.matmul``
in fp32, cast (examples/dequantize_gemm/example_dequant_gemv_fp16xint4.py:207-214,
example_dequant_gemm_bf16_mxfp4_cdna4.py:254-267,
examples/bitnet-1.58b/kernel_benchmark/tilelang_bitnet_158_int8xint2_decode.py:245-258).
"""

from __future__ import annotations

import torch

_E2M1 = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0])


def unpack_u4(qB: torch.Tensor) -> torch.Tensor:
    u = qB.view(torch.uint8)
    return torch.stack((u & 0x0F, u >> 4), dim=-1).reshape(u.shape[0], u.shape[1] * 2)


def dequant_w4a16(qB, Scale, Zeros=None, group: int = 128):
    """``W = ((q - 8) * s).half()`` or ``((q - z).half() * s).half()``, fp16 [N, K]."""
    q = unpack_u4(qB).to(torch.half)
    s = Scale.repeat_interleave(group, dim=1)
    if Zeros is None:
        return (q - 8) * s
    return (q - Zeros.repeat_interleave(group, dim=1)) * s


def matmul_f32(A, W, out_dtype):
    """The matmul half of every ``ref_program``: ``A.float() @ W.float().T`` cast to ``out_dtype``."""
    return torch.matmul(A.float(), W.float().T).to(out_dtype)


def ref_w4a16(A, qB, Scale, Zeros=None, group: int = 128):
    """``C = A.float() @ W.float().T -> fp16`` with ``W`` of ``dequant_w4a16``."""
    return matmul_f32(A, dequant_w4a16(qB, Scale, Zeros, group), torch.half)


def dequant_mxfp4_e2m1(qB, Scale, scale_bias: int = 127):
    """``W = lut[q] * 2**(Scale - bias)``, fp32 [N, K] (exactly representable in bf16)."""
    W = _E2M1[unpack_u4(qB).long()]
    return W * torch.exp2(Scale.float() - scale_bias).repeat_interleave(32, dim=1)


def ref_mxfp4_e2m1(A, qB, Scale, scale_bias: int = 127):
    """``C = A.float() @ (lut[q] * 2**(Scale - bias)).T -> bf16``."""
    return matmul_f32(A, dequant_mxfp4_e2m1(qB, Scale, scale_bias), torch.bfloat16)


def dequant_bitnet(qB, zero_point: int = 2):
    """2-bit codes ``c = w + zero_point`` four per byte, low bits first -> fp32 [N, K]."""
    u = qB.view(torch.uint8)
    c = torch.stack((u & 3, (u >> 2) & 3, (u >> 4) & 3, u >> 6), dim=-1).reshape(u.shape[0], u.shape[1] * 4)
    return c.to(torch.float32) - zero_point


def bitnet_epilogue(acc, s_a, s_w):
    return ((acc / s_a.reshape(-1, 1)) / s_w).to(torch.half)


def ref_bitnet(A, qB, s_a, s_w, zero_point: int = 2):
    """``out = ((A.float() @ W.float().T) / s_a) / s_w -> fp16`` with 2-bit codes ``c = w + zero_point``."""
    return bitnet_epilogue(torch.matmul(A.float(), dequant_bitnet(qB, zero_point).T), s_a, s_w)
