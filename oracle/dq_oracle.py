"""CPU oracle for the dequantize-GEMM path.  TEST INFRASTRUCTURE ONLY.

Nothing that ships (the ``tilelang_amd`` package, its C-ABI library) may import this
module; only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline``
leg use it, and only as the checker.

Every function restates, in numpy, a piece of the reference's own algorithm for this
path and cites the reference file:line it follows (paths relative to the reference
checkout).  bf16 values are carried as ``uint16`` bit patterns or as exactly
representable ``float32``; fp16 uses ``np.float16``.

How each function is pinned (see tests/test_oracle_pins.py):

* decoders over finite domains (16 nibbles / 256 bytes / 65536 byte pairs) are brute
  forced against closed forms and the value tables the reference holds
  (e2m1 table: examples/dequantize_gemm/quantize/nvfp4.py:17-34,
  testing/python/amd/test_tilelang_mxfp4_gfx950.py:32,49);
* sign extension against the known answers of
  testing/python/issue/test_tilelang_u32_signed_decode.py:26-30;
* e2m1 encode/pack against
  testing/python/quantize/test_tilelang_quantize_nvfp4_scale_layout.py:881-887;
* packing by round trip and by ``fast_decode(interleave(p)) == plain_decode(p)``;
* ``decode_fp4_simple_bf16_bits``, ``decode_fp4_twiddling``, ``interleave_weight`` and ``general_compress`` also
  against vectors the reference's own torch helpers wrote (tests/golden/reference_vectors.npz: all 256 bytes, all
  65536 byte pairs, 4096 seeded words, seeded codes);
* the rounding order of the scaled / zero-point uint4 decoders and of the BitLinear epilogue against the operation
  order of the device snippets written out with exact rationals and an explicit round-to-nearest-even per fp16 /
  fp32 instruction;
* matmuls by reduction to int64 / float64 brute force on tiny shapes;
* ``prepack_w4_fragments`` is this library's own layout (the reference's ladder transform is BitBLAS's and absent): the
  index formula written as plain loops; what pins it is the kernel that reads the layout giving, bit for bit, what the
  row-major kernel gives (tests/test_w4a16_gpu.py::test_fragment_ordered_weights).

Parity unpinned by any reference test or fixture (no in-tree caller exists; the
contract is the closed form plus the operation order of the device snippets):
``dequant_u4_scale`` / ``dequant_u4_scale_zeros`` rounding order
(examples/dequantize_gemm/quantize/lop3.py:41-81,136-176,233-271,326-363) and the
BitNet 2-bit code convention (``decode_i2``, zero_point choice).  ``quantize_mxfp4``: the
reference has no MXFP4 quantiser (its example draws codes and scales at random), so the block
scale rule is the OCP Microscaling v1.0 conversion and only the element rule
(``encode_fp4_e2m1_values``) is the reference's own: parity unpinned for the scale choice, which
is pinned by closed forms instead (exact powers of two, round trip through ``mxfp4_dequant``,
idempotence, the block maximum always landing in e2m1's top binade).  ``gen_quant4_quantize`` is
pinned by its closed form (absmax scale, rint, clamp) against torch's own ops on the CPU.
``dequant_lowbit`` (2-bit / 1-bit codes to fp16): the unscaled decoders are pinned over all 65536 / 256 inputs of
``fast_decode_i2_to_f16`` / ``fast_decode_i1_to_f16`` (examples/dequantize_gemm/quantize/lop3.py:424-463, 679-746)
against closed forms, through the interleave, and by the reference's sign-extension known answers; the rounding order
of its scaled and zero-point forms (lop3.py:465-636, 748-891) has no caller, test or fixture in the reference: parity
unpinned, contract = the operation order of the device snippets, checked against float64 arithmetic with explicit
roundings on values where the orders differ.
"""

from __future__ import annotations

import numpy as np

# --------------------------------------------------------------------------------------
# small numeric helpers
# --------------------------------------------------------------------------------------


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """float32 -> bfloat16 bit pattern, round to nearest even (what torch's ``.to(bfloat16)`` does)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    exp_all_ones = (u & 0x7F800000) == 0x7F800000
    bias = ((u >> 16) & 1) + 0x7FFF
    r = np.where(exp_all_ones, u, u + bias)
    # keep NaNs quiet
    nan = exp_all_ones & ((u & 0x007FFFFF) != 0)
    out = (r >> 16).astype(np.uint16)
    return np.where(nan, ((u >> 16) | 0x0040).astype(np.uint16), out)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.asarray(b).astype(np.uint32) << 16).view(np.float32)


def round_to_bf16(x: np.ndarray) -> np.ndarray:
    """float32 -> nearest bf16 value, returned as float32."""
    return bf16_bits_to_f32(f32_to_bf16_bits(x))


# --------------------------------------------------------------------------------------
# packing / layout (host, one-off)
# --------------------------------------------------------------------------------------


def general_compress(lowp: np.ndarray, source_bits: int = 4) -> np.ndarray:
    """Pack ``8 // source_bits`` values per byte, element ``j*epb + k`` at bit ``source_bits*k``.

    Follows examples/dequantize_gemm/quantize/utils.py:50-67 (numpy twin at
    examples/bitnet-1.58b/kernel_benchmark/tilelang_bitnet_158_int8xint2_decode.py:178-193).
    Returns int8 storage like the reference.
    """
    epb = 8 // source_bits
    v = np.asarray(lowp).astype(np.int64)
    assert v.shape[-1] % epb == 0
    v = v.reshape(*v.shape[:-1], v.shape[-1] // epb, epb)
    out = np.zeros(v.shape[:-1], dtype=np.int64)
    for k in range(epb):
        # the reference shifts the (signed) int8 value without masking, then ORs
        out |= (v[..., k] << (source_bits * k)) & 0xFF
    return out.astype(np.uint8).view(np.int8)


def general_decompress(packed: np.ndarray, source_bits: int = 4) -> np.ndarray:
    """Inverse of :func:`general_compress` for unsigned fields (uint8 out, low field first)."""
    epb = 8 // source_bits
    u = np.ascontiguousarray(packed).view(np.uint8)
    mask = (1 << source_bits) - 1
    parts = [(u >> (source_bits * k)) & mask for k in range(epb)]
    return np.stack(parts, axis=-1).reshape(*u.shape[:-1], u.shape[-1] * epb)


def interleave_weight(qweight: np.ndarray, nbits: int = 4, target_dtype: str = "float16") -> np.ndarray:
    """Per-32-bit-word permutation applied before the reference's *fast* decoders.

    Follows examples/dequantize_gemm/quantize/utils.py:71-125: element ``e`` (at bit
    ``nbits*e``) moves to bit ``(e % G)*stride + (e // G)*nbits`` with ``stride`` 16/8 and
    ``G`` = 2/4 for a float16/int8 target, followed by the byte shuffles for
    (1 bit,int8), (2 bit,float16), (1 bit,float16).
    """
    assert target_dtype in ("float16", "int8")
    q = np.ascontiguousarray(qweight).view(np.uint32).astype(np.uint64)
    new = np.zeros_like(q)
    bits_stride = 8 if target_dtype == "int8" else 16
    mask = (1 << nbits) - 1
    num_groups = 32 // bits_stride
    elems_per_group = bits_stride // nbits
    for i in range(num_groups):
        for j in range(elems_per_group):
            offset = i * elems_per_group + j
            shift = (offset % num_groups) * bits_stride + (offset // num_groups) * nbits
            new |= ((q >> (nbits * offset)) & mask) << shift
    if nbits == 1 and target_dtype == "int8":
        n = new & 0xF0F00F0F
        n |= ((new & 0x000000F0) >> 4) << 16
        n |= ((new & 0x0000F000) >> 12) << 24
        n |= ((new & 0x000F0000) >> 16) << 4
        n |= ((new & 0x0F000000) >> 24) << 12
        new = n
    elif nbits == 2 and target_dtype == "float16":
        n = new & 0xFF0000FF
        n |= ((new & 0x0000FF00) >> 8) << 16
        n |= ((new & 0x00FF0000) >> 16) << 8
        new = n
    elif nbits == 1 and target_dtype == "float16":
        n = new & 0xF000000F
        n |= ((new & 0x000000F0) >> 4) << 8
        n |= ((new & 0x00000F00) >> 8) << 16
        n |= ((new & 0x0000F000) >> 12) << 24
        n |= ((new & 0x000F0000) >> 16) << 4
        n |= ((new & 0x00F00000) >> 20) << 12
        n |= ((new & 0x0F000000) >> 24) << 20
        new = n
    return (new & 0xFFFFFFFF).astype(np.uint32).view(np.int8).reshape(np.asarray(qweight).shape)


def pack_int4(logical: np.ndarray) -> np.ndarray:
    """Two signed int4 per int8 byte, even index in the low nibble.

    Follows examples/gemm_int4/example_tilelang_gemm_int4.py:59-67.
    """
    t = np.asarray(logical)
    if t.dtype != np.int8:
        raise TypeError("expected int8 logical int4 tensor")
    if t.ndim == 0 or t.shape[-1] % 2 != 0:
        raise ValueError("last dimension must be even")
    t16 = t.astype(np.int16)
    packed = (t16[..., ::2] & 0x0F) | ((t16[..., 1::2] & 0x0F) << 4)
    return packed.astype(np.uint8).view(np.int8)


# --------------------------------------------------------------------------------------
# 4-bit / 2-bit integer decoders
# --------------------------------------------------------------------------------------


def unpack_u4(packed: np.ndarray) -> np.ndarray:
    """[N, K/2] bytes -> [N, K] uint8 nibbles, low nibble = even k.

    Follows examples/dequantize_gemm/example_dequant_gemv_fp16xint4.py:207-210 and
    examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:11-13.
    """
    u = np.ascontiguousarray(packed).view(np.uint8)
    return np.stack((u & 0x0F, u >> 4), axis=-1).reshape(*u.shape[:-1], u.shape[-1] * 2)


def sign_extend(field: np.ndarray, nbit: int) -> np.ndarray:
    """Two's-complement sign extension of an ``nbit`` field held in the low bits.

    Follows examples/dequantize_gemm/quantize/quantization.py:111-117,333-343
    (shift left by ``32-nbit`` then arithmetic shift right) and
    examples/dequantize_gemm/example_dequant_gemm_w4a8.py:10-21,68-74.
    """
    f = np.asarray(field).astype(np.int64) & ((1 << nbit) - 1)
    return (((f << (32 - nbit)) & 0xFFFFFFFF).astype(np.uint32).view(np.int32) >> (32 - nbit)).astype(np.int32)


def decode_i4_signed(packed: np.ndarray) -> np.ndarray:
    """[N, K/2] -> [N, K] int8, ``q >= 8 -> q - 16`` (W4A8 and int4 x int4 operands)."""
    return sign_extend(unpack_u4(packed), 4).astype(np.int8)


def unpack_u2(packed: np.ndarray) -> np.ndarray:
    """[N, K/4] bytes -> [N, K] 2-bit codes, element ``4j+k`` at bits ``2k`` of byte ``j``."""
    return general_decompress(packed, 2)


def decode_i2(packed: np.ndarray, convention: str = "offset") -> np.ndarray:
    """2-bit codes -> int8 weights.

    ``"unsigned"``: ``c`` (decode_i2u_to_i8s, examples/dequantize_gemm/quantize/lop3.py:975-997);
    ``"offset"``: ``c - 2`` (decode_i2s_to_i8s subtracts 0x02020202, lop3.py:950-973);
    ``"twos"``: two's complement of the 2-bit field
    (examples/dequantize_gemm/quantize/quantization.py:333-343 with nbit=2).
    """
    c = unpack_u2(packed).astype(np.int16)
    if convention == "unsigned":
        return c.astype(np.int8)
    if convention == "offset":
        return (c - 2).astype(np.int8)
    if convention == "twos":
        return sign_extend(c, 2).astype(np.int8)
    raise ValueError(convention)


def fast_decode_i4_to_f16(words: np.ndarray, signed: bool) -> np.ndarray:
    """Semantics of the reference's LOP3 snippet on one uint32 -> 8 fp16, in output order.

    Follows examples/dequantize_gemm/quantize/lop3.py:6-39: for i in 0..3,
    ``h[i] = ((w >> 4i) & 0x000f000f) | 0x64006400`` as two fp16 (1024 + nibble), minus
    1032 (signed) or 1024 (unsigned).  Output element ``2i`` is the low half.
    """
    w = np.asarray(words).astype(np.uint32)
    out = np.empty(w.shape + (8,), dtype=np.float16)
    med = np.float16(1032.0 if signed else 1024.0)
    for i in range(4):
        h = ((w >> np.uint32(4 * i)) & np.uint32(0x000F000F)) | np.uint32(0x64006400)
        lo = (h & 0xFFFF).astype(np.uint16).view(np.float16)
        hi = (h >> 16).astype(np.uint16).view(np.float16)
        out[..., 2 * i] = lo - med
        out[..., 2 * i + 1] = hi - med
    return out


def fast_decode_i2_to_i8(words: np.ndarray, signed: bool) -> np.ndarray:
    """Semantics of decode_i2{u,s}_to_i8s on one uint32 -> 16 int8, in output order.

    Follows examples/dequantize_gemm/quantize/lop3.py:950-997:
    ``i8s[i] = (w >> 2i) & 0x03030303`` (minus 0x02020202 per byte when signed).
    """
    w = np.asarray(words).astype(np.uint32)
    out = np.empty(w.shape + (16,), dtype=np.int8)
    for i in range(4):
        d = (w >> np.uint32(2 * i)) & np.uint32(0x03030303)
        for b in range(4):
            v = ((d >> np.uint32(8 * b)) & 0xFF).astype(np.int16)
            out[..., 4 * i + b] = (v - (2 if signed else 0)).astype(np.int8)
    return out


def fast_decode_i4_to_i8(word_pairs: np.ndarray, signed: bool) -> np.ndarray:
    """Semantics of decode_i4{u,s}_to_i8s on two uint32 (``[..., 2]``) -> 16 int8, in output order.

    Follows examples/dequantize_gemm/quantize/lop3.py:999-1047: for i in 0..1,
    ``i8s[i] = (i4b[0] >> 4i) & 0x0f0f0f0f`` and ``i8s[i + 2] = (i4b[1] >> 4i) & 0x0f0f0f0f``; the signed decoder
    then subtracts 0x07070707 per byte with signed saturation (``__vsubss4``; its MEDIAN_NUM is 7, not 8).
    """
    w = np.asarray(word_pairs).astype(np.uint32)
    assert w.shape[-1] == 2
    out = np.empty(w.shape[:-1] + (16,), dtype=np.int8)
    for i in range(2):
        for src in range(2):
            d = (w[..., src] >> np.uint32(4 * i)) & np.uint32(0x0F0F0F0F)
            for b in range(4):
                v = ((d >> np.uint32(8 * b)) & 0xFF).astype(np.int16)
                if signed:
                    v = np.clip(v - 7, -128, 127)
                out[..., 4 * (i + 2 * src) + b] = v.astype(np.int8)
    return out


def decode_i4_fast_int8(packed_interleaved: np.ndarray, signed: bool) -> np.ndarray:
    """[N, K/2] bytes whose 32-bit words went through ``interleave_weight(., 4, "int8")`` -> int8 [N, K] as
    decode_i4{u,s}_to_i8s yields them, 16 values per pair of words (lop3.py:999-1047)."""
    p = np.ascontiguousarray(packed_interleaved).view(np.uint8)
    w = p.view(np.uint32).reshape(p.shape[0], -1, 2)
    return fast_decode_i4_to_i8(w, signed).reshape(p.shape[0], -1)


def fast_decode_i1_to_i8(halfwords: np.ndarray, signed: bool) -> np.ndarray:
    """Semantics of decode_i1{u,s}_to_i8s on one uint16 (16 one-bit codes) -> 16 int8, in output order.

    Follows examples/dequantize_gemm/quantize/lop3.py:893-948: ``i1b = (x & 0x0f0f) | ((x & 0xf0f0) << 12)``; for i
    in 0..3 ``i8s[i] = (i1b >> i) & 0x01010101``; the signed form then computes ``v + v - 1`` per byte (``2 c - 1``).
    Output element ``4 i + b`` is byte ``b`` of ``i8s[i]``.
    """
    x = np.asarray(halfwords).astype(np.uint32) & np.uint32(0xFFFF)
    i1b = (x & np.uint32(0x0F0F)) | ((x & np.uint32(0xF0F0)) << np.uint32(12))
    out = np.empty(x.shape + (16,), dtype=np.int8)
    for i in range(4):
        d = (i1b >> np.uint32(i)) & np.uint32(0x01010101)
        for b in range(4):
            v = ((d >> np.uint32(8 * b)) & 0xFF).astype(np.int16)
            out[..., 4 * i + b] = (2 * v - 1 if signed else v).astype(np.int8)
    return out


def decode_i1_fast_int8(packed_interleaved: np.ndarray, signed: bool) -> np.ndarray:
    """[N, K/8] bytes whose 32-bit words went through ``interleave_weight(., 1, "int8")`` -> int8 [N, K] as
    decode_i1{u,s}_to_i8s yields them, 16 values per halfword (lop3.py:893-948)."""
    p = np.ascontiguousarray(packed_interleaved).view(np.uint8)
    h = p.view(np.uint16)
    return fast_decode_i1_to_i8(h, signed).reshape(p.shape[0], -1)


def fast_decode_i2_to_i4(words: np.ndarray) -> np.ndarray:
    """Semantics of decode_i2{u,s}_to_i4s on one uint32 (16 two-bit codes) -> two uint32 of eight 4-bit fields each.

    Follows examples/dequantize_gemm/quantize/lop3.py:1049-1089: with N = 16, for i in 0..1
    ``i4s[i] = (i2b[0] >> 2 i) & 0x33333333``: nibble ``e`` of ``i4s[i]`` is code ``2 e + i``.  The reference's signed
    form subtracts nothing (its adjustment is commented out, :1068-1073), so both decoders return the unsigned code
    in a nibble.  Returns ``[..., 2]`` uint32.
    """
    w = np.asarray(words).astype(np.uint32)
    return np.stack([(w >> np.uint32(2 * i)) & np.uint32(0x33333333) for i in range(2)], axis=-1)


def decode_i2_fast_int4(packed: np.ndarray) -> np.ndarray:
    """[N, K/4] bytes of 2-bit codes -> [N, K/2] bytes of 4-bit fields as decode_i2{u,s}_to_i4s writes them: word ``j``
    of a row becomes words ``2 j`` and ``2 j + 1``; field ``e`` of output word ``2 j + i`` is code ``2 e + i`` of
    input word ``j`` (lop3.py:1049-1089)."""
    p = np.ascontiguousarray(packed).view(np.uint8)
    out = fast_decode_i2_to_i4(p.view(np.uint32))  # [N, W, 2]
    return np.ascontiguousarray(out.reshape(p.shape[0], -1)).view(np.uint8)


def fast_decode_i4u_to_f16_zeros_quantized(words: np.ndarray, scale, qzero) -> np.ndarray:
    """Bit-level semantics of decode_i4u_to_f16_scale_zeros_quantized on one uint32 -> 8 fp16, in output order
    (examples/dequantize_gemm/quantize/lop3.py:326-363): ``h = (w >> 4i) & 0x000f000f | 0x64006400`` as two fp16,
    plus ``(0xe400 | zero)`` as fp16 (= -(1024 + zero)) in an fp16 add, then one fp16 fma with the scale and 0."""
    w = np.asarray(words).astype(np.uint32)
    s = np.asarray(scale, dtype=np.float16).astype(np.float32)
    med = (np.uint16(0xE400) | np.asarray(qzero).astype(np.uint16)).view(np.float16).astype(np.float32)
    out = np.empty(w.shape + (8,), dtype=np.float16)
    for i in range(4):
        h = ((w >> np.uint32(4 * i)) & np.uint32(0x000F000F)) | np.uint32(0x64006400)
        for half, sh in ((0, 0), (1, 16)):
            x = ((h >> np.uint32(sh)) & 0xFFFF).astype(np.uint16).view(np.float16).astype(np.float32)
            d = (x + med).astype(np.float16).astype(np.float32)          # add.f16x2
            out[..., 2 * i + half] = (d * s + np.float32(0)).astype(np.float16)  # fma.rn.f16x2 (product exact in fp32)
    return out


def unpack_qzeros(qzeros: np.ndarray, groups: int, fmt: str = "int16") -> np.ndarray:
    """Integer zero points of the "quantized" zeros mode as int32 [N, groups].  ``"int16"``: one per group
    (lop3.py:339-341).  ``"packed4"``: 4-bit, group g in bits 4 (g % 2) of byte g / 2 (lop3.py:381-385)."""
    if fmt == "int16":
        return np.asarray(qzeros).astype(np.int16).astype(np.int32)
    b = np.ascontiguousarray(qzeros).view(np.uint8)
    z = np.stack((b & 0xF, b >> 4), axis=-1).reshape(b.shape[0], -1)
    return z[:, :groups].astype(np.int32)


def fast_decode_i2_to_f16(halfwords: np.ndarray, signed: bool, scale=None) -> np.ndarray:
    """Semantics of decode_i2{u,s}_to_f16[_scale] on one 16-bit word -> 8 fp16, in output order.

    Follows examples/dequantize_gemm/quantize/lop3.py:424-463 (and :465-500 with a scale):
    ``i2s = (x & 0x00ff) | ((x & 0xff00) << 8)``; for i in 0..3
    ``h[i] = ((i2s >> 2i) & 0x00030003) | 0x64006400`` as two fp16 (1024 + c), minus 1026 (signed) or
    1024 (unsigned), then ``fma.rn.f16x2(h, s, 0)`` when scaled.  Output element ``2i`` is the low half.
    """
    x = np.asarray(halfwords).astype(np.uint32) & np.uint32(0xFFFF)
    i2s = (x & np.uint32(0x00FF)) | ((x & np.uint32(0xFF00)) << np.uint32(8))
    out = np.empty(x.shape + (8,), dtype=np.float16)
    med = np.float16(1026.0 if signed else 1024.0)
    for i in range(4):
        h = ((i2s >> np.uint32(2 * i)) & np.uint32(0x00030003)) | np.uint32(0x64006400)
        lo = (h & 0xFFFF).astype(np.uint16).view(np.float16)
        hi = (h >> 16).astype(np.uint16).view(np.float16)
        out[..., 2 * i] = lo - med
        out[..., 2 * i + 1] = hi - med
    if scale is not None:
        out = ((out.astype(np.float32) * np.float32(np.float16(scale))) + np.float32(0.0)).astype(np.float16)
    return out


def fast_decode_i1_to_f16(bytes_: np.ndarray, signed: bool) -> np.ndarray:
    """Semantics of decode_i1{u,s}_to_f16 on one byte -> 8 fp16, in output order.

    Follows examples/dequantize_gemm/quantize/lop3.py:679-746: ``i1s = (x & 0x0f) | ((x & 0xf0) << 12)``; for i in
    0..3 ``h[i] = ((i1s >> i) & 0x00010001) | 0x64006400`` as two fp16 (1024 + c) minus 1024; the signed form then
    computes ``h + h - 1`` (``2 c - 1``).  Output element ``2i`` is the low half.
    """
    x = np.asarray(bytes_).astype(np.uint32) & np.uint32(0xFF)
    i1s = (x & np.uint32(0x0F)) | ((x & np.uint32(0xF0)) << np.uint32(12))
    out = np.empty(x.shape + (8,), dtype=np.float16)
    for i in range(4):
        h = ((i1s >> np.uint32(i)) & np.uint32(0x00010001)) | np.uint32(0x64006400)
        lo = (h & 0xFFFF).astype(np.uint16).view(np.float16) - np.float16(1024.0)
        hi = (h >> 16).astype(np.uint16).view(np.float16) - np.float16(1024.0)
        if signed:
            lo = lo + lo - np.float16(1.0)
            hi = hi + hi - np.float16(1.0)
        out[..., 2 * i] = lo
        out[..., 2 * i + 1] = hi
    return out


def decode_lowbit(packed: np.ndarray, bits: int, convention: str = "twos") -> np.ndarray:
    """1- or 2-bit codes -> integer weights (int8), element ``e`` of a byte at bit ``bits * e``.

    ``"unsigned"``: ``c``; ``"twos"``: two's complement of the field
    (examples/dequantize_gemm/quantize/quantization.py:333-343); ``"offset"``: the signed fast decoders,
    ``c - 2`` for two bits (lop3.py:430,446) and ``2 c - 1`` for one bit (lop3.py:699,719-723).
    """
    c = general_decompress(np.asarray(packed).view(np.uint8), bits).astype(np.int16)
    if convention == "unsigned":
        return c.astype(np.int8)
    if convention == "twos":
        return sign_extend(c, bits).astype(np.int8)
    if convention == "offset":
        return ((c - 2) if bits == 2 else (2 * c - 1)).astype(np.int8)
    raise ValueError(convention)


def dequant_lowbit(packed, bits: int, convention: str = "twos", scale=None, zeros=None, group: int = -1,
                   zeros_mode: str = "original") -> np.ndarray:
    """1- or 2-bit codes -> fp16 weights with the rounding order of the device snippets.

    No scale: ``w`` exact.  Scale: ``RNE16(w * s)`` (``fma.rn.f16x2(x, s, 0)``, lop3.py:465-500, 748-810).  Zeros
    ``"original"``: ``RNE16(RNE16(w - z) * s)`` (sub, then fma: lop3.py:564-599, 812-851); ``"rescale"``:
    ``RNE16(RNE16(w * s) - z)`` (fma with 0, then sub: lop3.py:601-636, 853-891; the one-bit form :719-735).
    PARITY UNPINNED by reference tests for the scaled and zero-point forms (no caller in the reference).
    """
    w = decode_lowbit(packed, bits, convention).astype(np.float32)
    if scale is None:
        return w.astype(np.float16)
    K = w.shape[-1]
    g = K if group == -1 else group
    s = _expand_groups(np.asarray(scale, dtype=np.float16), K, g).astype(np.float32)
    if zeros is None:
        return ((w * s) + np.float32(0.0)).astype(np.float16)
    z = _expand_groups(np.asarray(zeros, dtype=np.float16), K, g).astype(np.float32)
    if zeros_mode == "original":
        d = (w - z).astype(np.float16).astype(np.float32)
        return ((d * s) + np.float32(0.0)).astype(np.float16)
    if zeros_mode == "rescale":
        d = ((w * s) + np.float32(0.0)).astype(np.float16).astype(np.float32)
        return (d - z).astype(np.float16)
    raise ValueError(zeros_mode)


def dequant_u2(packed: np.ndarray, convention: str = "twos", scale: np.ndarray | None = None, group: int = -1) -> np.ndarray:
    """The two-bit case of :func:`dequant_lowbit` without zeros."""
    return dequant_lowbit(packed, 2, convention, scale, None, group)


def ref_lowbit(A, packed, bits: int, convention: str = "twos", scale=None, zeros=None, group: int = -1,
               zeros_mode: str = "original") -> np.ndarray:
    """``ref_program`` of the 1- / 2-bit GEMV: dequantise, fp32 matmul, fp16 out (the pattern of
    examples/dequantize_gemm/example_dequant_gemv_fp16xint4.py:207-217 with the narrower unpack)."""
    W = dequant_lowbit(packed, bits, convention, scale, zeros, group, zeros_mode)
    return _matmul_f32(np.asarray(A, dtype=np.float16), W).astype(np.float16)


def ref_w2a16(A, packed, convention: str = "twos", scale=None, group: int = -1) -> np.ndarray:
    return ref_lowbit(A, packed, 2, convention, scale, None, group)


# --------------------------------------------------------------------------------------
# W4A16 dequantised weight tiles (fp16), exact rounding order of the device snippets
# --------------------------------------------------------------------------------------


def _expand_groups(per_group: np.ndarray, K: int, group: int) -> np.ndarray:
    return np.repeat(np.asarray(per_group), group, axis=-1)[..., :K]


def dequant_u4_plain(packed: np.ndarray, signed: bool = False) -> np.ndarray:
    """fp16 tile of ``q`` (unsigned) or two's-complement ``sext4(q)`` with no scale.

    Follows examples/dequantize_gemm/quantize/quantization.py:310-318 (unsigned) and
    :333-343 (the GEMV example's slow path,
    examples/dequantize_gemm/example_dequant_gemv_fp16xint4.py:121-124).
    """
    q = unpack_u4(packed)
    if signed:
        return sign_extend(q, 4).astype(np.float16)
    return q.astype(np.float16)


def dequant_u4_scale(packed: np.ndarray, scale: np.ndarray, group: int) -> np.ndarray:
    """``w = RNE_fp16((q - 8) * s[n, k // group])``.

    Follows examples/dequantize_gemm/quantize/quantization.py:298-307 (``q - 8``) and
    the operation order of lop3.py:41-81: exact fp16 ``q - 8`` then one
    ``fma.rn.f16x2(x, s, 0)``, i.e. a single rounding of the exact product.
    PARITY UNPINNED by reference tests (no caller in the reference).
    """
    q = unpack_u4(packed).astype(np.float32) - 8.0
    K = q.shape[-1]
    s = _expand_groups(np.asarray(scale, dtype=np.float16), K, group).astype(np.float32)
    # fp16 x fp16 is exact in fp32, so one cast is the single rounding; "+ 0" of the
    # fma turns a -0 product into +0
    return ((q * s) + np.float32(0.0)).astype(np.float16)


def dequant_u4_scale_zeros(packed: np.ndarray, scale: np.ndarray, zeros: np.ndarray, group: int, mode: str = "original") -> np.ndarray:
    """Zero-point variants of the uint4 decoder.

    ``original``:  ``RNE16(RNE16(q - z) * s)``      (lop3.py:136-176, sub then fma)
    ``rescale``:   ``RNE16(fma(q, s, -z))``          (lop3.py:233-271)
    ``quantized``: ``RNE16((q - qz) * s)``, qz int   (lop3.py:326-363)
    ``folded``:    ``RNE16(fma(q, s, -RNE16(z * s)))``: not a reference formula; the library's cheaper form of
                   ``original`` (DQ_W4_ZEROS_FOLDED), restated here so that its tile can be checked bit for bit.
    Also examples/dequantize_gemm/quantize/quantization.py:321-330.
    PARITY UNPINNED by reference tests (no caller in the reference).
    """
    q = unpack_u4(packed).astype(np.float32)
    K = q.shape[-1]
    s = _expand_groups(np.asarray(scale, dtype=np.float16), K, group).astype(np.float32)
    if mode == "original":
        z = _expand_groups(np.asarray(zeros, dtype=np.float16), K, group).astype(np.float32)
        d = (q - z).astype(np.float16).astype(np.float32)
        return ((d * s) + np.float32(0.0)).astype(np.float16)
    if mode == "rescale":
        z = _expand_groups(np.asarray(zeros, dtype=np.float16), K, group).astype(np.float64)
        return (q.astype(np.float64) * s.astype(np.float64) - z).astype(np.float16)
    if mode == "quantized":
        qz = _expand_groups(np.asarray(zeros).astype(np.int32), K, group).astype(np.float32)
        return (((q - qz) * s) + np.float32(0.0)).astype(np.float16)
    if mode == "folded":
        z = _expand_groups(np.asarray(zeros, dtype=np.float16), K, group).astype(np.float32)
        zs = (z * s).astype(np.float16).astype(np.float64)  # z * s is exact in fp32 (11 x 11 bits): one rounding
        return (q.astype(np.float64) * s.astype(np.float64) - zs).astype(np.float16)  # exact in fp64: one rounding
    raise ValueError(mode)


# --------------------------------------------------------------------------------------
# fp4 decoders
# --------------------------------------------------------------------------------------

#: OCP e2m1 values by code (examples/dequantize_gemm/quantize/nvfp4.py:17-34,
#: examples/dequantize_gemm/quantize/mxfp.py:141-144, src/tl_templates/hip/hip_fp4.h:61-64)
E2M1_VALUES = np.array(
    [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0], dtype=np.float32
)


def encode_fp4_e2m1_values(values: np.ndarray) -> np.ndarray:
    """float -> e2m1 code (ties toward the larger magnitude at the listed thresholds).

    Follows examples/dequantize_gemm/quantize/nvfp4.py:120-138.
    """
    x = np.nan_to_num(np.asarray(values, dtype=np.float32), nan=0.0, posinf=6.0, neginf=-6.0)
    a = np.abs(x)
    mag = np.zeros(a.shape, dtype=np.int32)
    for thr, code in ((0.25, 1), (0.75, 2), (1.25, 3), (1.75, 4), (2.5, 5), (3.5, 6), (5.0, 7)):
        mag = np.where(a >= thr, code, mag)
    sign = ((x < 0) & (mag != 0)).astype(np.int32) << 3
    return (mag | sign).astype(np.uint8)


def pack_fp4_e2m1_codes(codes: np.ndarray) -> np.ndarray:
    """Low nibble = even k.  Follows examples/dequantize_gemm/quantize/nvfp4.py:141-157."""
    c = np.asarray(codes)
    if c.dtype != np.uint8 or c.ndim != 2 or c.shape[1] % 2:
        raise ValueError("codes must be 2-D uint8 with even K")
    return ((c[:, 0::2] & 0x0F) | ((c[:, 1::2] & 0x0F) << 4)).astype(np.uint8)


def decode_fp4_e2m1(packed: np.ndarray) -> np.ndarray:
    """Plain low-first e2m1 -> float32 values.  Follows nvfp4.py:160-177, mxfp.py:136-157."""
    return E2M1_VALUES[unpack_u4(packed).astype(np.int64)]


def decode_fp4_simple_bf16_bits(packed: np.ndarray, scale: np.ndarray | None = None, scale_size: int | None = None) -> np.ndarray:
    """"Simple" fp4 -> bf16 bit pattern ``(s<<15) | ((E+126)<<7) | (m<<6)`` for every E.

    Follows examples/dequantize_gemm/dequantize_utils.py:57-84 (torch_convert) and
    examples/dequantize_gemm/example_dequant_gemm_bf16_mxfp4_cdna4.py:26-41.  Codes
    0..7 give 0.5, 0.75, 1, 1.5, 2, 3, 4, 6 (no zero, no subnormal).  With ``scale`` the
    per-block byte is added to the exponent and clamped to 255
    (examples/dequantize_gemm/quantize/quantization.py:30-73).
    """
    f4 = unpack_u4(packed).astype(np.int32)
    sign = f4 >> 3
    exponent = ((f4 & 6) >> 1) + 126
    if scale_size is not None:
        idx = np.arange(f4.shape[-1]) // scale_size
        exponent = np.minimum(exponent + np.asarray(scale).astype(np.int32)[:, idx], 255)
    mant = (f4 & 1) << 6
    return ((sign << 15) | (exponent << 7) | mant).astype(np.uint16)


def decode_fp4_simple_f16(packed: np.ndarray) -> np.ndarray:
    """"Simple" fp4 -> fp16 ``(s<<15) | ((E+14)<<10) | (m<<9)``.

    Follows examples/dequantize_gemm/example_dequant_gemm_fp4_hopper.py:10-41.
    """
    f4 = unpack_u4(packed).astype(np.int32)
    bits = ((f4 >> 3) << 15) | ((((f4 & 6) >> 1) + 14) << 10) | ((f4 & 1) << 9)
    return bits.astype(np.uint16).view(np.float16)


def decode_fp4_twiddling(packed: np.ndarray) -> np.ndarray:
    """"Twiddled" fp4 layout -> float32 values (true e2m1), 4 outputs per byte pair.

    Follows examples/dequantize_gemm/dequantize_utils.py:4-54: ``w = (b[2j] << 8) | b[2j+1]``,
    position p of output ``4j+p`` selects bits with mask 0x81C0 after shifts 0/3/6, and
    p=3 gathers ``(w<<1)&0x8000 | (w>>3)&0x0180 | (w>>7)&0x0040``; the pattern is a bf16
    which is multiplied by 2**126.
    """
    u = np.ascontiguousarray(packed).view(np.uint8).astype(np.uint32)
    assert u.ndim == 2 and u.shape[1] % 2 == 0
    w = (u[:, 0::2] << 8) | u[:, 1::2]
    mask = 0x81C0
    r0 = w & mask
    r1 = (w << 3) & mask
    r2 = (w << 6) & mask
    r3 = ((w << 1) & 0x8000) | ((w >> 3) & 0x0180) | ((w >> 7) & 0x0040)
    bits = np.stack((r0, r1, r2, r3), axis=-1).reshape(u.shape[0], u.shape[1] * 2) & 0xFFFF
    # bf16 * 2**126 is exact (the product has at most 2 significant bits), including the
    # bf16 subnormal inputs of codes 1 and 9
    return (bf16_bits_to_f32(bits.astype(np.uint16)).astype(np.float64) * 2.0**126).astype(np.float32)


def twiddle_pack_fp4(codes: np.ndarray) -> np.ndarray:
    """Inverse of :func:`decode_fp4_twiddling`'s bit map: e2m1 codes [N, K] -> bytes [N, K/2].

    Not in the reference (its inputs are random bytes); derived from the masks above so
    that round-trip tests can feed known codes.
    """
    c = np.asarray(codes).astype(np.uint32)
    assert c.ndim == 2 and c.shape[1] % 4 == 0
    c = c.reshape(c.shape[0], -1, 4)
    s, e, m = (c >> 3) & 1, (c >> 1) & 3, c & 1
    w = (s[..., 0] << 15) | (e[..., 0] << 7) | (m[..., 0] << 6)
    w |= (s[..., 1] << 12) | (e[..., 1] << 4) | (m[..., 1] << 3)
    w |= (s[..., 2] << 9) | (e[..., 2] << 1) | m[..., 2]
    w |= (s[..., 3] << 14) | (e[..., 3] << 10) | (m[..., 3] << 13)
    out = np.stack((w >> 8, w & 0xFF), axis=-1).reshape(c.shape[0], -1)
    return out.astype(np.uint8)


def mxfp4_dequant(packed: np.ndarray, scale: np.ndarray, fmt: str = "e2m1", scale_size: int = 32, scale_bias: int = 0) -> np.ndarray:
    """fp4 weights times the per-block power-of-two scale, as float32 (exact).

    ``fmt``: ``"e2m1"`` plain nibbles (a13), ``"twiddling"`` (a12), ``"simple"`` (a11).
    The reference multiplies by ``2 ** Scale`` with the raw, unbiased byte
    (examples/dequantize_gemm/example_dequant_gemm_bf16_mxfp4_cdna4.py:254-267) ->
    ``scale_bias=0``; an E8M0 scale is ``2 ** (Scale - 127)`` -> ``scale_bias=127``.
    """
    if fmt == "e2m1":
        w = decode_fp4_e2m1(packed)
    elif fmt == "twiddling":
        w = decode_fp4_twiddling(packed)
    elif fmt == "simple":
        w = bf16_bits_to_f32(decode_fp4_simple_bf16_bits(packed))
    else:
        raise ValueError(fmt)
    K = w.shape[1]
    e = np.asarray(scale).astype(np.int64)[:, np.arange(K) // scale_size] - scale_bias
    return (w.astype(np.float64) * np.exp2(e.astype(np.float64))).astype(np.float32)


# --------------------------------------------------------------------------------------
# ref_programs: dequantise -> fp32 / integer matmul -> cast
# --------------------------------------------------------------------------------------


def _matmul_f32(a: np.ndarray, w: np.ndarray) -> np.ndarray:
    return np.matmul(np.asarray(a, dtype=np.float32), np.asarray(w, dtype=np.float32).T)


def _matmul_int(a: np.ndarray, w: np.ndarray) -> np.ndarray:
    """Exact integer A @ W.T; every partial sum is an integer below 2**53, so float64 BLAS is exact."""
    a64 = np.asarray(a).astype(np.float64)
    w64 = np.asarray(w).astype(np.float64)
    bound = float(np.abs(a64).max(initial=0)) * float(np.abs(w64).max(initial=0)) * a64.shape[-1]
    assert bound < 2**53
    return np.rint(np.matmul(a64, w64.T)).astype(np.int64)


def ref_w4a16(A, packed, scale=None, zeros=None, group: int = -1, mode: str = "scale", out_dtype=np.float16):
    """W4A16 GEMV/GEMM: ``C = A.float() @ W_deq.float().T -> out_dtype``.

    Shape of the computation follows
    examples/dequantize_gemm/example_dequant_gemv_fp16xint4.py:207-214 (unpack, matmul) and
    examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:125-131 (fp32 matmul,
    cast); ``mode``: ``"unsigned"`` (w=q), ``"signed"`` (w=sext4 q), ``"scale"`` (w=(q-8)s),
    ``"original" | "rescale" | "quantized"`` zero-point variants.
    """
    K = np.asarray(packed).shape[-1] * 2
    if group == -1:
        group = K
    if mode == "unsigned":
        W = dequant_u4_plain(packed, signed=False)
    elif mode == "signed":
        W = dequant_u4_plain(packed, signed=True)
    elif mode == "scale":
        W = dequant_u4_scale(packed, scale, group)
    else:
        W = dequant_u4_scale_zeros(packed, scale, zeros, group, mode)
    C = _matmul_f32(np.asarray(A, dtype=np.float16), W)
    return C.astype(out_dtype)


def ref_mxfp4(A_bf16_bits, packed, scale, bias_bf16_bits=None, fmt="e2m1", scale_size=32, scale_bias=0):
    """MXFP4 GEMM: ``C = A @ (decode(B) * 2**(Scale-bias)).T (+ Bias) -> bf16 bits``.

    Follows examples/dequantize_gemm/example_dequant_gemm_bf16_mxfp4_cdna4.py:254-281.
    """
    A = bf16_bits_to_f32(np.asarray(A_bf16_bits, dtype=np.uint16))
    W = mxfp4_dequant(packed, scale, fmt, scale_size, scale_bias)
    C = _matmul_f32(A, W)
    if bias_bf16_bits is not None:
        C = C + bf16_bits_to_f32(np.asarray(bias_bf16_bits, dtype=np.uint16))
    return f32_to_bf16_bits(C)


def ref_mxfp4_mxfp4(A_packed, scale_a, B_packed, scale_b, bias_bf16_bits=None, scale_size=32):
    """Block-scaled MXFP4 x MXFP4 GEMM: both operands e2m1 codes with one E8M0 byte per 32 k,
    ``C = (decode(A) * 2**(SA-127)) @ (decode(B) * 2**(SB-127)).T (+ Bias) -> bf16 bits``, the sum in float64
    (every product is exact there) rounded once to fp32 and once to bf16.

    Follows blockscaled_gemm_ref of examples/blockscaled_gemm_sm100/gemm_mxfp8_blockscaled_1d1d.py:575-620
    (``2 ** (sf - 127)`` per scale block, fp32 result) with the 4-bit element format of
    examples/dequantize_gemm/quantize/nvfp4.py:17-34.  A scale byte of 255 is NaN (E8M0).
    """
    sa = np.asarray(scale_a); sb = np.asarray(scale_b)
    A = mxfp4_dequant(A_packed, np.where(sa == 255, 127, sa), "e2m1", scale_size, 127).astype(np.float64)
    W = mxfp4_dequant(B_packed, np.where(sb == 255, 127, sb), "e2m1", scale_size, 127).astype(np.float64)
    K = A.shape[1]
    A[(sa == 255)[:, np.arange(K) // scale_size]] = np.nan
    W[(sb == 255)[:, np.arange(K) // scale_size]] = np.nan
    C = np.matmul(A, W.T).astype(np.float32)
    if bias_bf16_bits is not None:
        C = C + bf16_bits_to_f32(np.asarray(bias_bf16_bits, dtype=np.uint16))
    return f32_to_bf16_bits(C)


def ref_fp16xfp4(A, packed):
    """``Ct[N, M] = (A.float() @ simple_fp16(B).float().T -> fp16).T``.

    Follows examples/dequantize_gemm/example_dequant_gemm_fp4_hopper.py:223-228.
    """
    C = _matmul_f32(np.asarray(A, dtype=np.float16), decode_fp4_simple_f16(packed)).astype(np.float16)
    return np.ascontiguousarray(C.T)


def ref_fp16xfp4_splitk(A, packed, split: int):
    """The split-K form of the fp16 x fp4 GEMM: each K slice gives an fp32 product rounded to fp16
    (``T.copy(Ct_local, SplitC[bz, ...])``, SplitC in ``out_dtype``), and the slices are added in fp16, slice 0 first
    (``acc`` of ``out_dtype``, ``acc += SplitC[k]``): examples/dequantize_gemm/example_dequant_gemm_fp4_hopper.py:136-175.
    Returns ``C[M,N]`` fp16 (the example stores its transpose).
    """
    A = np.asarray(A, dtype=np.float16)
    W = decode_fp4_simple_f16(packed)
    K = A.shape[1]
    assert K % split == 0
    kk = K // split
    acc = None
    for z in range(split):
        part = _matmul_f32(A[:, z * kk:(z + 1) * kk], W[:, z * kk:(z + 1) * kk]).astype(np.float16)
        acc = part if acc is None else (acc.astype(np.float32) + part.astype(np.float32)).astype(np.float16)
    return acc


def ref_w4a8(A_i8, packed):
    """``Ct[N, M] int32 = (A @ sext4(B).T).T``.  Follows example_dequant_gemm_w4a8.py:68-82."""
    C = _matmul_int(np.asarray(A_i8, dtype=np.int8), decode_i4_signed(packed)).astype(np.int32)
    return np.ascontiguousarray(C.T)


def ref_int4xint4(A_packed, B_packed):
    """``C int32 = sext4(A) @ sext4(B).T``.  Follows examples/gemm_int4/example_tilelang_gemm_int4.py:92-101."""
    return _matmul_int(decode_i4_signed(A_packed), decode_i4_signed(B_packed)).astype(np.int32)


def ref_u4_int8(A_i8, packed):
    """Fine-grained int8 path: ``C int32 = A @ q.T`` with unsigned nibbles.

    Follows examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:11-13,125-131.
    """
    return _matmul_int(np.asarray(A_i8, dtype=np.int8), unpack_u4(packed)).astype(np.int32)


def ref_bitnet_int(A_i8, packed, convention: str = "offset"):
    """``C[M, N] int32 = A_int8 @ decode_i2(B).T``.

    Follows examples/bitnet-1.58b/kernel_benchmark/tilelang_bitnet_158_int8xint2_decode.py:245-258
    and ..._prefill.py:360-381 (torch matmul of the unpacked operands).
    """
    return _matmul_int(np.asarray(A_i8, dtype=np.int8), decode_i2(packed, convention)).astype(np.int32)


# --------------------------------------------------------------------------------------
# weight quantisers (the producers of the packed operands)
# --------------------------------------------------------------------------------------


def quantize_mxfp4(w: np.ndarray, scale_bias: int = 127, scale_size: int = 32):
    """bf16-representable ``w[N, K]`` -> (packed e2m1 codes uint8 [N, K/2], scale bytes uint8 [N, K/scale_size]).

    Block scale: ``e = max(floor(log2(max|w|)) - 2, -127)`` (OCP Microscaling Formats v1.0, section 6.3: shared
    exponent = exponent of the block maximum minus the exponent of the element format's largest value, 6 = 1.5 * 2^2;
    an all-zero block takes the smallest exponent, as the published ``microxcaling`` library does),
    ``byte = clamp(e + scale_bias, 0, 255)``.  Elements: ``encode_fp4_e2m1_values(w / 2**(byte - scale_bias))``
    (examples/dequantize_gemm/quantize/nvfp4.py:120-138), packed low nibble first (``:141-157``).  The layout is
    the one examples/dequantize_gemm/example_dequant_gemm_bf16_mxfp4_cdna4.py:99-103 consumes.
    """
    w = np.asarray(w, dtype=np.float32)
    N, K = w.shape
    blocks = w.reshape(N, K // scale_size, scale_size)
    amax = np.abs(blocks).max(axis=-1)
    # floor(log2(amax)) from the exponent field (exact); bf16 subnormals and zero give exponent field 0
    expf = (amax.view(np.uint32) >> 23).astype(np.int32) & 0xFF
    e = np.maximum(expf - 127 - 2, -127)
    byte = np.clip(e + scale_bias, 0, 255)
    e_used = np.clip(byte - scale_bias, -127, 126)
    scaled = blocks * np.exp2(-e_used.astype(np.float64))[..., None].astype(np.float32)  # exact: power of two
    codes = encode_fp4_e2m1_values(scaled.reshape(N, K))
    return pack_fp4_e2m1_codes(codes), byte.astype(np.uint8)


def gen_quant4_quantize(w: np.ndarray, groupsize: int = -1):
    """The deterministic part of ``gen_quant4`` (examples/dequantize_gemm/quantize/utils.py:1-47) for a given
    fp16 ``w[K, N]``: per (group of ``groupsize`` consecutive k, column n) ``s = max|w| * 2 / 16`` in fp16,
    ``q = clamp(rint(w / s) + 8, 0, 16)``, ``ref = (q - 8).half() * s``.  Returns ``(ref[K, N] fp16,
    s[K/groupsize, N] fp16, q - 8 [K, N] int32)`` — the reference's ``linear.weight.T``, ``s`` and last value.

    ``maxq`` is 16 there, not 15: the element with the largest magnitude of a group, when positive, quantises to
    ``q = 16``, which does not fit a nibble (the reference never packs this function's output).
    """
    w = np.asarray(w, dtype=np.float16)
    K, N = w.shape
    g = K if groupsize == -1 else groupsize
    wg = w.reshape(K // g, g, N)
    s = (np.abs(wg).max(axis=1, keepdims=True).astype(np.float16) * np.float16(2 / 16)).astype(np.float16)
    q = np.rint((wg / s).astype(np.float16).astype(np.float32)).astype(np.int32) + 8
    q = np.clip(q, 0, 16)
    ref = ((q - 8).astype(np.float16) * s).astype(np.float16)
    return ref.reshape(K, N), s.reshape(K // g, N), (q - 8).reshape(K, N)


# --------------------------------------------------------------------------------------
# BitLinear quantisers and epilogue
# --------------------------------------------------------------------------------------


def weight_quant(weight: np.ndarray):
    """Ternary weights.  Follows examples/bitnet-1.58b/utils_quant.py:149-154.  Returns (W_q int8, s_w)."""
    w = np.asarray(weight, dtype=np.float32)
    s = np.float32(1.0) / np.maximum(np.abs(w).mean(dtype=np.float32), np.float32(1e-5))
    return np.clip(np.rint(w * s), -1, 1).astype(np.int8), np.float32(s)


def activation_quant(x: np.ndarray, num_bits: int = 8):
    """Per-row int8 activations.  Follows examples/bitnet-1.58b/utils_quant.py:156-163.  Returns (x_q, s[M,1]).

    ``Qp / tensor`` with a Python scalar on the left is torch's ``Tensor.__rtruediv__``, i.e.
    ``tensor.reciprocal() * Qp``: two fp32 roundings, not one division (pinned against torch's own ops on the
    CPU in tests/test_oracle_pins.py).
    """
    xf = np.asarray(x, dtype=np.float32)
    qn, qp = -(2 ** (num_bits - 1)), 2 ** (num_bits - 1) - 1
    amax = np.maximum(np.abs(xf).max(axis=-1, keepdims=True), np.float32(1e-5)).astype(np.float32)
    s = ((np.float32(1.0) / amax).astype(np.float32) * np.float32(qp)).astype(np.float32)
    return np.clip(np.rint(xf * s), qn, qp).astype(np.int8), s


def post_quant_process(acc: np.ndarray, si: np.ndarray, sw) -> np.ndarray:
    """``out = (float(acc) / si) / sw -> fp16``: two fp32 divides in that order.

    Follows examples/bitnet-1.58b/utils_quant.py:165-170.
    """
    out = np.asarray(acc).astype(np.float32) / np.asarray(si, dtype=np.float32)
    out = out / np.float32(sw)
    return out.astype(np.float16)


def ref_bitnet(A_i8, packed, s_a, s_w, convention: str = "offset"):
    """BitNet W2A8 linear: exact int32 accumulation then the BitLinear epilogue -> fp16 [M, N]."""
    acc = ref_bitnet_int(A_i8, packed, convention)
    return post_quant_process(acc, np.asarray(s_a, dtype=np.float32).reshape(-1, 1), s_w)


def prepack_w4_fragments(B):
    """Packed uint4 weights [N, K/2] -> [N/16, K/128, 64, 16] bytes: entry 16 g + r of chunk c of block b holds bytes
    64 c + 16 g .. + 15 of row 16 b + r -- the operand order of the 16x16x32 matrix instruction (lane 16 g + r owns
    k = 32 g .. 32 g + 31 of a 128-k chunk of row r).  Plain loops over the index formula (test infrastructure: the
    library's torch helper and its kernel are checked against this).  In the role of the reference's offline weight
    transform, examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:178-179 (B_shape of the ladder kernel)."""
    B = np.ascontiguousarray(B).view(np.uint8)
    N, KB = B.shape
    assert N % 16 == 0 and KB % 64 == 0
    out = np.empty((N // 16, KB // 64, 64, 16), np.uint8)
    for b in range(N // 16):
        for c in range(KB // 64):
            for g in range(4):
                for r in range(16):
                    out[b, c, 16 * g + r, :] = B[16 * b + r, 64 * c + 16 * g: 64 * c + 16 * g + 16]
    return out


def prepack_i2_fragments(B):
    """Packed 2-bit weights [N, K/4] -> [ceil(N/32), K/128, 64, 16] bytes: entry 32 h + r of chunk c of block b holds bytes
    32 c + 16 h .. + 15 of row 32 b + r (rows past N: zeros) -- the operand order of the 32x32x32 int8 matrix instruction
    (lane 32 h + r owns k = 64 h .. 64 h + 63 of a 128-k chunk of row r).  Plain loops over the index formula (test
    infrastructure, as prepack_w4_fragments above); the reference has no counterpart for its BitNet kernels."""
    B = np.ascontiguousarray(B).view(np.uint8)
    N, KB = B.shape
    assert KB % 32 == 0
    blocks = (N + 31) // 32
    out = np.zeros((blocks, KB // 32, 64, 16), np.uint8)
    for b in range(blocks):
        for c in range(KB // 32):
            for h in range(2):
                for r in range(32):
                    if 32 * b + r < N:
                        out[b, c, 32 * h + r, :] = B[32 * b + r, 32 * c + 16 * h: 32 * c + 16 * h + 16]
    return out
