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


def ref_w4a16(A, qB, Scale, Zeros=None, group: int = 128):
    """``C = A.float() @ W.float().T -> fp16`` with ``W = ((q - 8) * s).half()`` or ``((q - z).half() * s).half()``."""
    q = unpack_u4(qB).to(torch.half)
    s = Scale.repeat_interleave(group, dim=1)
    if Zeros is None:
        W = (q - 8) * s
    else:
        W = (q - Zeros.repeat_interleave(group, dim=1)) * s
    return torch.matmul(A.float(), W.float().T).to(torch.half)


def ref_mxfp4_e2m1(A, qB, Scale, scale_bias: int = 127):
    """``C = A.float() @ (lut[q] * 2**(Scale - bias)).T -> bf16``."""
    W = _E2M1[unpack_u4(qB).long()]
    W = W * torch.exp2(Scale.float() - scale_bias).repeat_interleave(32, dim=1)
    return torch.matmul(A.float(), W.T).to(torch.bfloat16)


def ref_bitnet(A, qB, s_a, s_w, zero_point: int = 2):
    """``out = ((A.float() @ W.float().T) / s_a) / s_w -> fp16`` with 2-bit codes ``c = w + zero_point``."""
    u = qB.view(torch.uint8)
    c = torch.stack((u & 3, (u >> 2) & 3, (u >> 4) & 3, u >> 6), dim=-1).reshape(u.shape[0], u.shape[1] * 4)
    W = c.to(torch.float32) - zero_point
    acc = torch.matmul(A.float(), W.T)
    return ((acc / s_a.reshape(-1, 1)) / s_w).to(torch.half)
