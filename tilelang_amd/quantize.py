"""Host-side weight packing and layout helpers (one-off, torch ops, any device).

Same names and argument meaning as the helpers the reference's examples import:
``general_compress`` / ``interleave_weight`` (examples/dequantize_gemm/quantize/utils.py:50-125),
``pack_int4`` (examples/gemm_int4/example_tilelang_gemm_int4.py:59-67), the e2m1
helpers of examples/dequantize_gemm/quantize/nvfp4.py:120-177, and ``gen_quant4``
(examples/dequantize_gemm/quantize/utils.py:1-47) with a packer from its layout to this library's, and the offline
re-ordering of packed uint4 weights into the matrix instruction's operand order (``prepack_w4_fragments``).
"""

from __future__ import annotations

import torch

FP4_E2M1_VALUES = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0)


def general_compress(lowprecision_weight: torch.Tensor, source_bits: int = 4, storage_dtype=None) -> torch.Tensor:
    """Pack ``8 // source_bits`` fields per byte, field ``k`` of a byte at bit ``source_bits * k``."""
    if storage_dtype is None:
        storage_dtype = torch.int8
    epb = 8 // source_bits
    w = lowprecision_weight
    if w.dtype == torch.float16:
        w = w.to(torch.int8)
    if w.shape[-1] % epb:
        raise ValueError(f"last dimension {w.shape[-1]} is not a multiple of {epb}")
    fields = w.to(torch.int32).reshape(*w.shape[:-1], w.shape[-1] // epb, epb)
    packed = torch.zeros(fields.shape[:-1], dtype=torch.int32, device=w.device)
    for k in range(epb):  # OR without masking the field, as the reference does for signed inputs
        packed |= (fields[..., k] << (source_bits * k)) & 0xFF
    return packed.to(torch.uint8).view(torch.int8).to(storage_dtype)


def interleave_weight(qweight: torch.Tensor, nbits: int = 4, target_dtype: str = "float16") -> torch.Tensor:
    """Permute every 32-bit word so the fast 16-bit / 8-bit decoders emit natural element order.

    Element ``e`` of a word moves to bit ``(e % G) * stride + (e // G) * nbits`` (stride 16, G 2 for a
    float16 target; stride 8, G 4 for int8), plus the extra byte shuffles of the 1-bit and
    (2-bit, float16) cases.
    """
    if target_dtype not in ("float16", "int8"):
        raise ValueError(target_dtype)
    orig_shape, orig_dtype = qweight.shape, qweight.dtype
    q = qweight.contiguous().view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    stride = 8 if target_dtype == "int8" else 16
    groups = 32 // stride
    mask = (1 << nbits) - 1
    out = torch.zeros_like(q)
    for e in range(32 // nbits):
        dst = (e % groups) * stride + (e // groups) * nbits
        out |= ((q >> (nbits * e)) & mask) << dst

    def move(x, src_mask, right, left):
        return ((x & src_mask) >> right) << left

    if nbits == 1 and target_dtype == "int8":
        out = (out & 0xF0F00F0F) | move(out, 0x000000F0, 4, 16) | move(out, 0x0000F000, 12, 24) \
            | move(out, 0x000F0000, 16, 4) | move(out, 0x0F000000, 24, 12)
    elif nbits == 2 and target_dtype == "float16":
        out = (out & 0xFF0000FF) | move(out, 0x0000FF00, 8, 16) | move(out, 0x00FF0000, 16, 8)
    elif nbits == 1 and target_dtype == "float16":
        out = (out & 0xF000000F) | move(out, 0x000000F0, 4, 8) | move(out, 0x00000F00, 8, 16) \
            | move(out, 0x0000F000, 12, 24) | move(out, 0x000F0000, 16, 4) | move(out, 0x00F00000, 20, 12) \
            | move(out, 0x0F000000, 24, 20)
    out = out & 0xFFFFFFFF
    out = torch.where(out >= 2**31, out - 2**32, out).to(torch.int32)
    return out.view(orig_dtype).reshape(orig_shape)


def _require(ok: bool, exc, text: str) -> None:
    if not ok:
        raise exc(text)


def pack_int4(tensor: torch.Tensor) -> torch.Tensor:
    """Logical signed int4 held in int8 -> two per byte, even index in the low nibble."""
    _require(tensor.dtype == torch.int8, TypeError, f"pack_int4 takes int8 values in -8..7, not {tensor.dtype}")
    _require(tensor.ndim >= 1 and tensor.shape[-1] % 2 == 0, ValueError,
             f"pack_int4 puts two values in a byte: the last dimension of {tuple(tensor.shape)} must be even")
    t = tensor.to(torch.int16)
    return ((t[..., ::2] & 0x0F) | ((t[..., 1::2] & 0x0F) << 4)).to(torch.uint8).view(torch.int8).contiguous()


def encode_fp4_e2m1_values(values: torch.Tensor) -> torch.Tensor:
    """float -> raw e2m1 nibble codes (uint8)."""
    _require(isinstance(values, torch.Tensor), TypeError, f"encode_fp4_e2m1_values takes a tensor, not {type(values).__name__}")
    x = torch.nan_to_num(values.to(torch.float32), nan=0.0, posinf=6.0, neginf=-6.0)
    bounds = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0], device=x.device)
    mag = torch.bucketize(x.abs(), bounds, right=True).to(torch.int32)
    sign = ((x < 0) & (mag != 0)).to(torch.int32) << 3
    return (mag | sign).to(torch.uint8)


def pack_fp4_e2m1_codes(codes: torch.Tensor) -> torch.Tensor:
    """e2m1 codes [N, K] uint8 -> int8 storage [N, K/2], low nibble first."""
    _require(isinstance(codes, torch.Tensor) and codes.dtype == torch.uint8, TypeError,
             "pack_fp4_e2m1_codes takes a uint8 tensor of e2m1 codes")
    _require(codes.ndim == 2 and codes.shape[1] % 2 == 0, ValueError,
             f"pack_fp4_e2m1_codes takes [N, K] with K even (two codes per byte), not {tuple(codes.shape)}")
    return ((codes[:, 0::2] & 0x0F) | ((codes[:, 1::2] & 0x0F) << 4)).contiguous().view(torch.int8)


def decode_packed_fp4_e2m1(packed: torch.Tensor, cols: int | None = None) -> torch.Tensor:
    """Packed e2m1 -> float32 values."""
    _require(packed.ndim == 2, ValueError, f"decode_packed_fp4_e2m1 takes [N, K/2] bytes, not {tuple(packed.shape)}")
    width = 2 * packed.shape[1]
    _require(cols is None or cols == width, ValueError, f"{packed.shape[1]} bytes per row hold {width} codes, not {cols}")
    cols = width
    u = packed.contiguous().view(torch.uint8)
    lut = torch.tensor(FP4_E2M1_VALUES, device=packed.device, dtype=torch.float32)
    nib = torch.stack((u & 0x0F, u >> 4), dim=-1).reshape(packed.shape[0], cols)
    return lut[nib.long()]


def gen_quant4(k: int, n: int, groupsize: int = -1):
    """Random fp16 ``w[k, n]`` quantised to 4 bits per (group of ``groupsize`` consecutive k, column): returns
    ``(original_w, linear, s, q)`` like ``gen_quant4`` of examples/dequantize_gemm/quantize/utils.py:1-47 —
    ``s[k/groupsize, n]`` fp16 = group absmax * 2/16, ``q[k, n]`` int32 = ``clamp(round(w/s) + 8, 0, 16) - 8``,
    ``linear`` an ``nn.Linear(k, n, bias=False)`` whose weight is the dequantised ``(q.half() * s).T``.

    As in the reference ``maxq`` is 16, so ``q`` reaches +8 (code 16) for a group's largest positive element;
    :func:`pack_gen_quant4` deals with that when the codes have to fit a nibble.
    """
    maxq = 2**4
    if groupsize == -1:
        groupsize = k
    if k % groupsize:
        raise ValueError(f"gen_quant4: k={k} is not a multiple of groupsize={groupsize}")
    original_w = torch.randn((k, n), dtype=torch.half, device="cpu")
    grouped = original_w.reshape(k // groupsize, groupsize, n)
    s = grouped.abs().amax(dim=1, keepdim=True) * (2 / maxq)
    q = torch.clamp(torch.round(grouped / s).int() + maxq // 2, 0, maxq)
    ref = (q - maxq // 2).half() * s
    linear = torch.nn.Linear(k, n, bias=False)
    linear.weight.data = ref.reshape(k, n).t()
    return original_w, linear, s.reshape(k // groupsize, n).contiguous(), (q - maxq // 2).reshape(k, n)


def pack_gen_quant4(q: torch.Tensor, s: torch.Tensor, saturate: bool = False):
    """``gen_quant4``'s ``q[k, n]`` (values -8..8) and ``s[k/g, n]`` -> this library's W4A16 operands
    ``B[n, k/2]`` int8 (codes ``q + 8``, even k in the low nibble) and ``Scale[n, k/g]`` fp16, for
    ``dequantize_gemv(..., source_format="int", with_scaling=True)`` (``w = (code - 8) * s``).

    Code 16 (``q = +8``) does not fit a nibble: with ``saturate=False`` that raises, with ``saturate=True`` it is
    stored as 15 (the dequantised value of that element is then ``7 s`` instead of ``8 s``).
    """
    codes = (q.to(torch.int32) + 8).t().contiguous()
    if int(codes.min()) < 0 or int(codes.max()) > 16:
        raise ValueError("pack_gen_quant4: q must be in -8..8")
    if int(codes.max()) > 15:
        if not saturate:
            raise ValueError("pack_gen_quant4: code 16 does not fit 4 bits (pass saturate=True to store 15)")
        codes = codes.clamp(max=15)
    return general_compress(codes.to(torch.int8), 4), s.t().contiguous().to(torch.float16)


def prepack_w4_fragments(qweight: torch.Tensor) -> torch.Tensor:
    """Packed uint4 weights ``[N, K/2]`` -> ``[N/16, K/128, 64, 16]`` bytes in the operand order of the 16x16x32 matrix
    instruction: entry ``16*g + r`` of chunk ``c`` of block ``b`` holds bytes ``64*c + 16*g .. + 15`` of row ``16*b + r``.

    The offline weight transform in the role of the one the reference's ladder kernel consumes
    (examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:136-354, ``B_shape = (N/16, K/16, 16, 8)``): a wave
    then fetches 1 KiB contiguous straight into operand registers.  Works on plain and on interleaved words alike (whole
    16-byte pieces move).  N must be a multiple of 16, K of 128.
    """
    _require(qweight.dim() == 2, ValueError, "prepack_w4_fragments expects a 2-D packed tensor [N, K/2]")
    n, kb = qweight.shape
    _require(n % 16 == 0 and kb % 64 == 0, ValueError,
             f"prepack_w4_fragments needs N % 16 == 0 and K % 128 == 0 (got N={n}, K={2 * kb})")
    pieces = qweight.contiguous().view(torch.uint8).reshape(n // 16, 16, kb // 64, 4, 16)  # [b, r, c, g, byte]
    return pieces.permute(0, 2, 3, 1, 4).reshape(n // 16, kb // 64, 64, 16).contiguous().view(qweight.dtype)


def unpack_w4_fragments(fragments: torch.Tensor) -> torch.Tensor:
    """Inverse of ``prepack_w4_fragments``: ``[N/16, K/128, 64, 16]`` -> ``[N, K/2]``."""
    _require(fragments.dim() == 4 and fragments.shape[2:] == (64, 16), ValueError,
             "unpack_w4_fragments expects [N/16, K/128, 64, 16]")
    nb, nc = fragments.shape[:2]
    pieces = fragments.contiguous().view(torch.uint8).reshape(nb, nc, 4, 16, 16)  # [b, c, g, r, byte]
    return pieces.permute(0, 3, 1, 2, 4).reshape(nb * 16, nc * 64).contiguous().view(fragments.dtype)


def prepack_i2_fragments(qweight: torch.Tensor) -> torch.Tensor:
    """Packed 2-bit weights ``[N, K/4]`` -> ``[ceil(N/32), K/128, 64, 16]`` bytes in the operand order of the 32x32x32
    int8 matrix instruction: entry ``32*h + r`` of chunk ``c`` of block ``b`` holds bytes ``32*c + 16*h .. + 15`` of row
    ``32*b + r`` (64 codes); rows past N are zero.

    The same offline transform as :func:`prepack_w4_fragments`, for the BitNet W2A8 GEMM that slices K over the waves
    of a workgroup: a wave fetches 1 KiB contiguous straight into an operand register.  Works on plain and on
    interleaved words alike (whole 16-byte pieces move).  K must be a multiple of 128.
    """
    _require(qweight.dim() == 2, ValueError, "prepack_i2_fragments expects a 2-D packed tensor [N, K/4]")
    n, kb = qweight.shape
    _require(kb % 32 == 0, ValueError, f"prepack_i2_fragments needs K % 128 == 0 (got K={4 * kb})")
    blocks = (n + 31) // 32
    rows = qweight.contiguous().view(torch.uint8)
    if blocks * 32 != n:
        rows = torch.cat([rows, rows.new_zeros((blocks * 32 - n, kb))])
    pieces = rows.reshape(blocks, 32, kb // 32, 2, 16)  # [b, r, c, h, byte]
    return pieces.permute(0, 2, 3, 1, 4).reshape(blocks, kb // 32, 64, 16).contiguous().view(qweight.dtype)


def unpack_i2_fragments(fragments: torch.Tensor, n: int | None = None) -> torch.Tensor:
    """Inverse of :func:`prepack_i2_fragments`: ``[ceil(N/32), K/128, 64, 16]`` -> ``[N, K/4]`` (``n`` drops the padding rows)."""
    _require(fragments.dim() == 4 and fragments.shape[2:] == (64, 16), ValueError,
             "unpack_i2_fragments expects [ceil(N/32), K/128, 64, 16]")
    nb, nc = fragments.shape[:2]
    pieces = fragments.contiguous().view(torch.uint8).reshape(nb, nc, 2, 32, 16)  # [b, c, h, r, byte]
    rows = pieces.permute(0, 3, 1, 2, 4).reshape(nb * 32, nc * 32)
    if n is not None:
        _require(nb * 32 - 31 <= n <= nb * 32, ValueError, f"unpack_i2_fragments: n={n} does not fit {nb} blocks of 32 rows")
        rows = rows[:n]
    return rows.contiguous().view(fragments.dtype)

