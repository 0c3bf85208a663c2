"""Seeded synthetic inputs of the benchmark configurations (numpy, host memory).

One generator per weight format; shapes and distributions are the ones the benchmark
configurations name.  Everything is derived from ``numpy.random.default_rng(seed)`` so the
same call gives the same bytes on any machine; callers move the arrays to the GPU.
bf16 tensors are returned as ``uint16`` bit patterns (view them as ``torch.bfloat16``).
"""

from __future__ import annotations

import numpy as np


def _bf16_bits(x: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((u + (((u >> 16) & 1) + 0x7FFF)) >> 16).astype(np.uint16)


def pack_nibbles(q: np.ndarray) -> np.ndarray:
    """[N, K] values 0..15 -> [N, K/2] uint8, even k in the low nibble."""
    q = q.astype(np.uint8)
    return (q[:, 0::2] | (q[:, 1::2] << 4)).astype(np.uint8)


def pack_crumbs(c: np.ndarray) -> np.ndarray:
    """[N, K] values 0..3 -> [N, K/4] uint8, element 4j+i at bits 2i of byte j."""
    c = c.astype(np.uint8)
    return (c[:, 0::4] | (c[:, 1::4] << 2) | (c[:, 2::4] << 4) | (c[:, 3::4] << 6)).astype(np.uint8)


def w4a16(M: int, N: int, K: int, group: int = 128, seed: int = 0, scale_range=(0.005, 0.02), zeros_range=None):
    """A fp16 [M,K] ~ N(0,1); q uniform 0..15 packed [N,K/2]; fp16 Scale [N,K/group] uniform in ``scale_range``;
    optional fp16 Zeros [N,K/group], integer valued, uniform in ``zeros_range`` (inclusive)."""
    rng = np.random.default_rng(seed)
    A = rng.standard_normal((M, K), dtype=np.float32).astype(np.float16)
    q = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    B = pack_nibbles(q)
    S = rng.uniform(scale_range[0], scale_range[1], size=(N, K // group)).astype(np.float16)
    out = {"A": A, "B": B, "Scale": S}
    if zeros_range is not None:
        out["Zeros"] = rng.integers(zeros_range[0], zeros_range[1] + 1, size=(N, K // group)).astype(np.float16)
    return out


def mxfp4(M: int, N: int, K: int, seed: int = 0, scale_exp_range=(-8, 0), scale_bias: int = 127, scale_size: int = 32):
    """A bf16 [M,K] ~ N(0,1) (uint16 bits); e2m1 codes uniform over 16 values packed [N,K/2];
    Scale uint8 [N,K/scale_size] = scale_bias + e, e uniform in ``scale_exp_range`` (inclusive)."""
    rng = np.random.default_rng(seed)
    A = _bf16_bits(rng.standard_normal((M, K), dtype=np.float32))
    codes = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    B = pack_nibbles(codes)
    e = rng.integers(scale_exp_range[0], scale_exp_range[1] + 1, size=(N, K // scale_size))
    S = (e + scale_bias).astype(np.uint8)
    return {"A": A, "B": B, "Scale": S}


def mxfp4_mxfp4(M: int, N: int, K: int, seed: int = 0, scale_exp_range=(-8, 0), scale_size: int = 32):
    """Both operands block-scaled fp4: e2m1 codes uniform over 16 values packed [M,K/2] and [N,K/2];
    E8M0 scales uint8 [M,K/scale_size], [N,K/scale_size] = 127 + e, e uniform in ``scale_exp_range`` (inclusive)."""
    rng = np.random.default_rng(seed)
    A = pack_nibbles(rng.integers(0, 16, size=(M, K), dtype=np.uint8))
    B = pack_nibbles(rng.integers(0, 16, size=(N, K), dtype=np.uint8))
    SA = (rng.integers(scale_exp_range[0], scale_exp_range[1] + 1, size=(M, K // scale_size)) + 127).astype(np.uint8)
    SB = (rng.integers(scale_exp_range[0], scale_exp_range[1] + 1, size=(N, K // scale_size)) + 127).astype(np.uint8)
    return {"A": A, "B": B, "SFA": SA, "SFB": SB}


def bitnet(M: int, N: int, K: int, seed: int = 0, zero_point: int = 2):
    """A int8 [M,K] uniform -127..127 with fp32 per-row scale s_a [M]; ternary W in {-1,0,1} (p = 1/3 each),
    stored as 2-bit codes ``w + zero_point`` four per byte [N,K/4]; fp32 per-tensor weight scale s_w."""
    rng = np.random.default_rng(seed)
    A = rng.integers(-127, 128, size=(M, K)).astype(np.int8)
    W = rng.integers(-1, 2, size=(N, K)).astype(np.int8)
    B = pack_crumbs((W.astype(np.int16) + zero_point).astype(np.uint8))
    s_a = rng.uniform(0.5, 50.0, size=(M,)).astype(np.float32)
    s_w = np.float32(rng.uniform(0.5, 4.0))
    return {"A": A, "B": B, "W": W, "s_a": s_a, "s_w": s_w}


def int8_int4(M: int, N: int, K: int, seed: int = 0):
    """A int8 [M,K] uniform -128..127; B uint8 [N,K/2] uniform bytes (two int4 each)."""
    rng = np.random.default_rng(seed)
    A = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    B = rng.integers(0, 256, size=(N, K // 2)).astype(np.uint8)
    return {"A": A, "B": B}


def int4_int4(M: int, N: int, K: int, seed: int = 0):
    """Logical int4 operands uniform -8..7 as int8 [M,K], [N,K] (pack with ``quantize.pack_int4``)."""
    rng = np.random.default_rng(seed)
    return {
        "A_logical": rng.integers(-8, 8, size=(M, K)).astype(np.int8),
        "B_logical": rng.integers(-8, 8, size=(N, K)).astype(np.int8),
    }


# ---- algorithmic work of each configuration (bytes touched once, 2*M*N*K operations) -----

def w4a16_bytes(M: int, N: int, K: int, group: int = 128, zeros: bool = False) -> int:
    sz = 2 * N * (K // group)
    return N * K // 2 + sz * (2 if zeros else 1) + 2 * M * K + 2 * M * N


def mxfp4_bytes(M: int, N: int, K: int, scale_size: int = 32) -> int:
    return 2 * M * K + N * K // 2 + N * (K // scale_size) + 2 * M * N


def mxfp4_mxfp4_bytes(M: int, N: int, K: int, scale_size: int = 32) -> int:
    return (M + N) * (K // 2 + K // scale_size) + 2 * M * N


def bitnet_bytes(M: int, N: int, K: int) -> int:
    return N * K // 4 + M * K + 2 * M * N + 4 * M + 4


def flops(M: int, N: int, K: int) -> int:
    return 2 * M * N * K
