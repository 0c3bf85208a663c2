"""Kernel factories with the call surface of the reference's examples.

Each factory takes the example's arguments (shapes, dtype names, decode options) and
returns a :class:`~tilelang_amd.adapter.KernelAdapter` whose call signature is the
example kernel's: ``kernel(A, B_packed[, Scale[, Zeros]], C)`` on torch device tensors.
Nothing is compiled at call time: every factory binds an ahead-of-time entry point of
``libdqgemm.so``.  Tile-size / thread / stage arguments of the examples are accepted and
ignored (the kernels carry their own gfx950 tiling).
"""

from __future__ import annotations

import torch

from . import _lib
from .adapter import KernelAdapter, KernelParam

# ---- enums of include/dqgemm.h -------------------------------------------------------------
W4_UNSIGNED, W4_SIGNED, W4_OFFSET8, W4_SCALE, W4_USCALE, W4_ZEROS_ORIGINAL, W4_ZEROS_RESCALE, W4_ZEROS_FOLDED = range(8)
LAYOUT_PLAIN, LAYOUT_INTERLEAVED, LAYOUT_FRAGMENTS = 0, 1, 2
DECODER_CONVERTER = 4  # flag of call_dequantize_w4's layout: dump the tile with the fp8-converter decoder
I4_UNSIGNED, I4_TWOS, I4U_INTERLEAVED, I4S_INTERLEAVED, I2_TO_I4 = range(5)

_DTYPES = {
    "float16": torch.float16,
    "bfloat16": torch.bfloat16,
    "float32": torch.float32,
    "int8": torch.int8,
    "uint8": torch.uint8,
    "int32": torch.int32,
}


def _dtype(d) -> torch.dtype:
    if isinstance(d, torch.dtype):
        return d
    try:
        return _DTYPES[str(d)]
    except KeyError:
        raise ValueError(f"unsupported dtype {d!r}") from None


def _w4_mode(source_format: str, fast_decoding: bool, with_scaling: bool, with_zeros: bool, zeros_mode: str) -> int:
    if with_zeros:
        if not with_scaling:
            raise ValueError("with_zeros requires with_scaling")
        if zeros_mode in ("original", "quantized"):
            # "quantized": integer zero points, unpacked to fp16 in front of the kernel (see _zeros_params)
            return W4_ZEROS_ORIGINAL
        if zeros_mode == "rescale":
            return W4_ZEROS_RESCALE
        if zeros_mode == "folded":
            # (q - z) * s as one fused multiply-add per weight, fma(q, s, -rne16(z * s)): this library's own, cheaper
            # form of "original" (no counterpart in the reference); inside rtol = atol = 1e-2 of it
            return W4_ZEROS_FOLDED
        raise ValueError(f"unknown zeros_mode {zeros_mode!r}")
    if with_scaling:
        return W4_SCALE if source_format == "int" else W4_USCALE
    if fast_decoding:
        return W4_OFFSET8 if source_format == "int" else W4_UNSIGNED
    # the example's slow path sign-extends the nibble whatever source_format says
    # (examples/dequantize_gemm/example_dequant_gemv_fp16xint4.py:121-124)
    return W4_SIGNED


QZEROS_INT16, QZEROS_PACKED4 = 0, 1


def _zeros_params(N: int, groups: int, zeros_mode: str, qzeros_format: str):
    """Parameters that carry the zero points: ``(Zeros as the caller passes it, fp16 workspace or None, format)``.

    ``"original"`` / ``"rescale"``: fp16 ``Zeros[N, groups]``.  ``"quantized"``
    (examples/dequantize_gemm/quantize/lop3.py:326-420): integer zero points, ``qzeros_format="int16"`` for
    ``Zeros[N, groups]`` int16 (the ``int16_t zero_r`` of :339-341) or ``"packed4"`` for 4-bit zero points two per
    byte, ``Zeros[N, ceil(groups / 2)]`` (the extraction of :381-385; the tensor shape and the order of the groups
    inside a row are this library's convention, the reference defines no host-side tensor for them); they are
    unpacked to fp16 into a workspace in front of the kernel, which then runs its ``(q - z) * s`` decoder: the same
    bits, since ``q - qz`` is exact either way.  Reference parity of the int16 form holds for 0 <= qz <= 1023 (what
    ``0xe400 | zero_r`` can express); other values are taken as the integers they are.
    """
    if zeros_mode != "quantized":
        return KernelParam("Zeros", torch.float16, (N, groups)), None, None
    if qzeros_format == "int16":
        zp = KernelParam("Zeros", torch.int16, (N, groups))
        fmt = QZEROS_INT16
    elif qzeros_format == "packed4":
        zp = KernelParam("Zeros", torch.uint8, (N, (groups + 1) // 2), packed=True)
        fmt = QZEROS_PACKED4
    else:
        raise ValueError(f"unknown qzeros_format {qzeros_format!r} (expected 'int16' or 'packed4')")
    return zp, KernelParam("ZerosFp16", torch.float16, (N, groups)), fmt


def dequantize_gemv(
    M: int,
    N: int,
    K: int,
    in_dtype="float16",
    out_dtype="float16",
    accum_dtype="float32",
    num_bits: int = 4,
    storage_dtype="int8",
    source_format: str = "uint",
    n_partition: int = 4,
    reduce_thread: int = 32,
    fast_decoding: bool = False,
    trans_A: bool = False,
    trans_B: bool = True,
    group_size: int = -1,
    with_scaling: bool = False,
    with_zeros: bool = False,
    zeros_mode: str = "original",
    variant: int = -1,
    _formula_fast: bool | None = None,
    qzeros_format: str = "int16",
    weight_fragments: bool = False,
) -> KernelAdapter:
    """W4A16 decode GEMV / small-batch GEMM: ``C[M,N] = A[M,K] @ dequant(B[N,K/2]).T``.

    Same positional arguments as ``dequantize_gemv`` of
    examples/dequantize_gemm/example_dequant_gemv_fp16xint4.py:11-29.  Call surface:
    ``kernel(A, B, C)``; with ``with_scaling`` ``kernel(A, B, Scale, C)``; with
    ``with_zeros`` ``kernel(A, B, Scale, Zeros, C)``, ``Scale``/``Zeros`` fp16
    ``[N, K // group_size]``.

    ``num_bits`` 2 and 1 (``B[N, K * num_bits / 8]``) and ``in_dtype="int8"`` with int32 accumulation and output
    (the example's ``use_dp4a`` branch) are served by their own kernels, see ``_dequantize_gemv_lowbit`` and
    ``_dequantize_gemv_int8``; what follows describes the fp16 x 4-bit case.

    ``fast_decoding=True`` means, as in the example, that B was passed through
    ``interleave_weight(B, 4, "float16")``; otherwise B is the plain low-nibble-first
    layout.  Accumulation is always fp32.  ``source_format="int"`` with scaling is the
    zero-point-8 decode ``w = (q - 8) * s``.

    ``weight_fragments=True``: B went through ``quantize.prepack_w4_fragments`` (after ``interleave_weight`` when
    ``fast_decoding``) and is ``[N/16, K/128, 64, 16]`` bytes, the matrix instruction's operand order; read at
    M <= 16, K in {2048, 4096, 8192}, group 128 only (the library refuses other shapes).
    """
    assert trans_A is False, "Dequantize only implement for trans_A=False currently"
    assert trans_B is True, "Dequantize only implement for trans_B=TRue currently"
    if num_bits not in (1, 2, 4):
        raise ValueError("dequantize_gemv: num_bits must be 4, 2 or 1")
    if _dtype(in_dtype) == torch.int8:
        return _dequantize_gemv_int8(M, N, K, out_dtype, accum_dtype, num_bits, storage_dtype, source_format, fast_decoding,
                                     with_scaling, with_zeros, _formula_fast)
    if _dtype(in_dtype) != torch.float16 or _dtype(out_dtype) != torch.float16:
        raise ValueError("dequantize_gemv: in_dtype must be float16 (with float16 out) or int8 (with int32 out)")
    if _dtype(storage_dtype) not in (torch.int8, torch.uint8):
        raise ValueError("dequantize_gemv: storage_dtype must be int8 or uint8")
    if num_bits < 4:
        return _dequantize_gemv_lowbit(M, N, K, num_bits, storage_dtype, source_format, fast_decoding, group_size,
                                       with_scaling, with_zeros, zeros_mode, _formula_fast, qzeros_format)
    if group_size == -1:
        group_size = K
    if K % 128 != 0:
        raise ValueError(f"dequantize_gemv: K={K} must be a multiple of 128")
    if K % group_size != 0 or group_size % 32 != 0:
        raise ValueError(f"dequantize_gemv: group_size={group_size} must divide K={K} and be a multiple of 32")
    # _formula_fast (tests): pick the decode formula of the fast / slow path independently of the layout
    formula_fast = fast_decoding if _formula_fast is None else _formula_fast
    mode = _w4_mode(source_format, formula_fast, with_scaling, with_zeros, zeros_mode)
    layout = LAYOUT_INTERLEAVED if fast_decoding else LAYOUT_PLAIN
    groups = K // group_size
    b_shape = (N, K // 2)
    if weight_fragments:
        if M > 16 or N % 16 != 0 or K not in (2048, 4096, 8192) or group_size != 128 or (with_zeros and zeros_mode == "rescale"):
            raise ValueError("dequantize_gemv: fragment-ordered weights need M <= 16, N % 16 == 0, K in {2048, 4096, 8192}, "
                             "group_size 128 and a zeros_mode other than \"rescale\"")
        layout |= LAYOUT_FRAGMENTS
        b_shape = (N // 16, K // 128, 64, 16)

    params = [
        KernelParam("A", torch.float16, (M, K)),
        KernelParam("B", _dtype(storage_dtype), b_shape, packed=True),
    ]
    if with_scaling:
        params.append(KernelParam("Scale", torch.float16, (N, groups)))
    zwork, zfmt = None, None
    if with_zeros:
        zparam, zwork, zfmt = _zeros_params(N, groups, zeros_mode, qzeros_format)
        params.append(zparam)
    c_idx = len(params)
    params.append(KernelParam("C", torch.float16, (M, N)))
    # Few rows and a long K: the library cuts K over workgroups when it is given room for the slices' fp32 sums (the
    # reference's split-K kernels allocate theirs inside the kernel function,
    # examples/dequantize_gemm/example_dequant_gemm_fp4_hopper.py:141).
    ws_bytes = 0
    if variant < 0 and not weight_fragments:
        ws_bytes = int(_lib.load_library().dq_w4a16_workspace_bytes(M, N, K, group_size, mode))
    workspace_idx = []
    if ws_bytes:
        workspace_idx.append(len(params))
        params.append(KernelParam("Workspace", torch.uint8, (ws_bytes,)))
    if zwork is not None:
        workspace_idx.append(len(params))
        params.append(zwork)

    def launch(ptrs, stream):
        lib = _lib.get_library()
        a, b = ptrs[0], ptrs[1]
        s = ptrs[2] if with_scaling else None
        z = ptrs[3] if with_zeros else None
        if zwork is not None:
            if lib.call_unpack_qzeros(z, ptrs[-1], N, groups, zfmt, stream) != 0:
                return -1
            z = ptrs[-1]
        if ws_bytes:
            return lib.call_dequantize_gemv_w4a16_ws(a, b, s, z, ptrs[c_idx], ptrs[c_idx + 1], ws_bytes, M, N, K, group_size,
                                                     mode, layout, variant, stream)
        return lib.call_dequantize_gemv_w4a16(a, b, s, z, ptrs[c_idx], M, N, K, group_size, mode, layout, variant, stream)

    return KernelAdapter("dequantize_gemv", params, [], launch, _lib.last_error, workspace_idx=workspace_idx)


def _dequantize_gemv_int8(M, N, K, out_dtype, accum_dtype, num_bits, storage_dtype, source_format, fast_decoding,
                          with_scaling, with_zeros, _formula_fast) -> KernelAdapter:
    """The integer branch of :func:`dequantize_gemv` (``use_dp4a``: int8 activations, int32 accumulation,
    examples/dequantize_gemm/example_dequant_gemv_fp16xint4.py:47-48,126-133): ``C[M,N] int32 = A[M,K] int8 .
    decode(B)^T``, exact.  Two bits: every decoder and the ``interleave_weight(B, 2, "int8")`` layout of the fast path
    (the BitNet decode kernel is this case); four bits: the slow path (two's-complement nibbles) and the fast path on
    ``interleave_weight(B, 4, "int8")`` words (``"uint"``: ``w = q``; ``"int"``: ``w = q - 7``, the constant of the
    reference's decode_i4s_to_i8s)."""
    if _dtype(accum_dtype) != torch.int32 or _dtype(out_dtype) != torch.int32:
        raise ValueError("dequantize_gemv: int8 activations accumulate and return int32")
    if with_scaling or with_zeros:
        raise ValueError("dequantize_gemv: the integer branch has no scales or zeros")
    if K % 128 != 0:
        raise ValueError(f"dequantize_gemv: K={K} must be a multiple of 128")
    params = [KernelParam("A", torch.int8, (M, K)),
              KernelParam("B", _dtype(storage_dtype), (N, K * num_bits // 8), packed=True),
              KernelParam("C", torch.int32, (M, N))]
    formula_fast = fast_decoding if _formula_fast is None else _formula_fast
    if num_bits == 2:
        conv = I2_TWOS if not formula_fast else (I2_OFFSET if source_format == "int" else I2_UNSIGNED)
        layout = LAYOUT_INTERLEAVED if fast_decoding else LAYOUT_PLAIN

        def launch(ptrs, stream):
            return _lib.get_library().call_gemm_int8xint2(ptrs[0], ptrs[1], ptrs[2], M, N, K, conv, layout, None, 1.0, 0, stream)

    elif num_bits == 4:
        # slow path: two's-complement nibbles, plain words.  Fast path: the words went through
        # interleave_weight(B, 4, "int8") and decode as decode_i4u_to_i8s (w = q) or decode_i4s_to_i8s (w = q - 7)
        # (examples/dequantize_gemm/quantize/lop3.py:999-1047)
        dec = I4_TWOS if not fast_decoding else (I4S_INTERLEAVED if source_format == "int" else I4U_INTERLEAVED)

        def launch(ptrs, stream):
            return _lib.get_library().call_gemm_int8xint4(ptrs[0], ptrs[1], ptrs[2], M, N, K, dec, 0, 0, stream)

    elif num_bits == 1:
        # slow path: the sign extension of a one-bit field, w = -c.  Fast path: the words went through
        # interleave_weight(B, 1, "int8") and decode as decode_i1u_to_i8s (w = c) or decode_i1s_to_i8s (w = 2 c - 1)
        # (examples/dequantize_gemm/quantize/lop3.py:893-948)
        if M > 4:
            raise ValueError(f"dequantize_gemv: int8 x 1-bit is a decode kernel, M <= 4 (got {M})")
        if K > 65536:
            raise ValueError(f"dequantize_gemv: int8 x 1-bit is built for K <= 65536 (got {K})")
        conv = I2_TWOS if not formula_fast else (I2_OFFSET if source_format == "int" else I2_UNSIGNED)
        layout = LAYOUT_INTERLEAVED if fast_decoding else LAYOUT_PLAIN

        def launch(ptrs, stream):
            return _lib.get_library().call_gemv_int8xint1(ptrs[0], ptrs[1], ptrs[2], M, N, K, conv, layout, stream)

    else:
        raise ValueError("dequantize_gemv: int8 activations are built for num_bits 4, 2 and 1")
    return KernelAdapter("dequantize_gemv", params, [], launch, _lib.last_error)


def _dequantize_gemv_lowbit(M, N, K, num_bits, storage_dtype, source_format, fast_decoding, group_size, with_scaling,
                            with_zeros, zeros_mode, _formula_fast, qzeros_format="int16") -> KernelAdapter:
    """The ``num_bits`` = 2 and 1 cases of :func:`dequantize_gemv`: ``B[N, K * num_bits / 8]``.

    Slow path: two's-complement codes whatever ``source_format`` says
    (examples/dequantize_gemm/example_dequant_gemv_fp16xint4.py:121-124).  ``fast_decoding=True``: B went through
    ``interleave_weight(B, num_bits, "float16")`` and decodes as ``c`` (``"uint"``) or as ``c - 2`` / ``2 c - 1``
    (``"int"``, two bits / one bit; examples/dequantize_gemm/quantize/lop3.py:424-463, 679-746), times
    ``Scale[N, K/group]`` with ``with_scaling``, and with ``with_zeros`` ``(w - z) * s`` (``"original"``) or
    ``w * s - z`` (``"rescale"``) (lop3.py:564-636, 812-891).  ``zeros_mode="quantized"`` (two bits, ``"uint"``
    codes: decode_i2u_to_f16_scale_zeros_quantized, lop3.py:638-677): integer zero points in the formats of
    :func:`_zeros_params`; the decoder's ``(1024 + c) + (0xe400 | qz)`` is ``c - qz`` exactly, so they are unpacked to
    fp16 in front of the kernel, which runs ``(c - z) * s``: the same bits.  Call surface
    ``kernel(A, B[, Scale[, Zeros]], C)``.
    """
    chunk = 128 // num_bits
    if group_size == -1:
        group_size = K
    if K % 128 != 0:
        raise ValueError(f"dequantize_gemv: K={K} must be a multiple of 128")
    if K > 32768:
        raise ValueError(f"dequantize_gemv: num_bits={num_bits} is built for K <= 32768 (got {K})")
    if M > 64:
        raise ValueError(f"dequantize_gemv: num_bits={num_bits} is a decode kernel, M <= 64 (got {M})")
    if with_zeros and not with_scaling:
        raise ValueError("with_zeros requires with_scaling")
    quantized = with_zeros and zeros_mode == "quantized"
    if quantized and not (num_bits == 2 and fast_decoding and source_format == "uint"):
        raise ValueError("dequantize_gemv: zeros_mode 'quantized' below four bits is the two-bit unsigned fast decoder's "
                         "(num_bits=2, source_format='uint', fast_decoding=True)")
    if with_zeros and zeros_mode not in ("original", "rescale", "quantized"):
        raise ValueError(f"dequantize_gemv: zeros_mode {zeros_mode!r} is not built for num_bits={num_bits}")
    if with_scaling and (K % group_size != 0 or group_size % chunk != 0):
        raise ValueError(f"dequantize_gemv: group_size={group_size} must divide K={K} and be a multiple of {chunk}")
    formula_fast = fast_decoding if _formula_fast is None else _formula_fast
    if not formula_fast:
        conv = I2_TWOS
    else:
        conv = I2_OFFSET if source_format == "int" else I2_UNSIGNED
    layout = LAYOUT_INTERLEAVED if fast_decoding else LAYOUT_PLAIN
    rescale = 1 if (with_zeros and zeros_mode == "rescale") else 0
    params = [KernelParam("A", torch.float16, (M, K)),
              KernelParam("B", _dtype(storage_dtype), (N, K * num_bits // 8), packed=True)]
    if with_scaling:
        params.append(KernelParam("Scale", torch.float16, (N, K // group_size)))
    zwork, zfmt = None, None
    groups = K // group_size
    if with_zeros:
        zparam, zwork, zfmt = _zeros_params(N, groups, zeros_mode, qzeros_format)
        params.append(zparam)
    c_idx = len(params)
    params.append(KernelParam("C", torch.float16, (M, N)))
    if zwork is not None:
        params.append(zwork)

    def launch(ptrs, stream):
        lib = _lib.get_library()
        s = ptrs[2] if with_scaling else None
        z = ptrs[3] if with_zeros else None
        if zwork is not None:
            if lib.call_unpack_qzeros(z, ptrs[-1], N, groups, zfmt, stream) != 0:
                return -1
            z = ptrs[-1]
        return lib.call_dequantize_gemv_lowbit(ptrs[0], ptrs[1], s, z, ptrs[c_idx], M, N, K, group_size, num_bits,
                                               conv, layout, rescale, stream)

    return KernelAdapter("dequantize_gemv", params, [], launch, _lib.last_error,
                         workspace_idx=[-1] if zwork is not None else [])


def dequantize_w4(
    N: int,
    K: int,
    group_size: int = -1,
    source_format: str = "int",
    fast_decoding: bool = False,
    with_scaling: bool = True,
    with_zeros: bool = False,
    zeros_mode: str = "original",
    storage_dtype="int8",
    _formula_fast: bool | None = None,
    qzeros_format: str = "int16",
    decoder: str = "mask",
) -> KernelAdapter:
    """Dequantised weight tile ``W[N,K] fp16 = decode(B[N,K/2][, Scale[, Zeros]])``.

    The decode-only kernel the examples use to test a converter
    (examples/dequantize_gemm/example_dequant_gemm_w4a8.py:36-65), here for the 4-bit
    integer decoders.  ``W = kernel(B[, Scale[, Zeros]])``.  ``decoder``: which of the library's two device decoders
    writes the tile, ``"mask"`` (nibbles OR-ed into an fp16 mantissa) or ``"converter"`` (nibbles read as fp8 by the
    hardware converter); they agree bit for bit.
    """
    if decoder not in ("mask", "converter"):
        raise ValueError(f"dequantize_w4: unknown decoder {decoder!r}")
    if group_size == -1:
        group_size = K
    formula_fast = fast_decoding if _formula_fast is None else _formula_fast
    mode = _w4_mode(source_format, formula_fast, with_scaling, with_zeros, zeros_mode)
    layout = (LAYOUT_INTERLEAVED if fast_decoding else LAYOUT_PLAIN) | (DECODER_CONVERTER if decoder == "converter" else 0)
    groups = K // group_size
    params = [KernelParam("B", _dtype(storage_dtype), (N, K // 2), packed=True)]
    if with_scaling:
        params.append(KernelParam("Scale", torch.float16, (N, groups)))
    zwork, zfmt = None, None
    if with_zeros:
        zparam, zwork, zfmt = _zeros_params(N, groups, zeros_mode, qzeros_format)
        params.append(zparam)
    w_idx = len(params)
    params.append(KernelParam("W", torch.float16, (N, K)))
    if zwork is not None:
        params.append(zwork)

    def launch(ptrs, stream):
        lib = _lib.get_library()
        s = ptrs[1] if with_scaling else None
        z = ptrs[2] if with_zeros else None
        if zwork is not None:
            if lib.call_unpack_qzeros(z, ptrs[-1], N, groups, zfmt, stream) != 0:
                return -1
            z = ptrs[-1]
        return lib.call_dequantize_w4(ptrs[0], s, z, ptrs[w_idx], N, K, group_size, mode, layout, stream)

    return KernelAdapter("dequantize_w4", params, [w_idx], launch, _lib.last_error, workspace_idx=[-1] if zwork is not None else [])


FP4_E2M1, FP4_SIMPLE, FP4_TWIDDLING = 0, 1, 2
_FP4_FORMATS = {"e2m1": FP4_E2M1, "simple": FP4_SIMPLE, "twiddling": FP4_TWIDDLING}


def matmul_bf16_mxfp4(
    M: int,
    N: int,
    K: int,
    in_dtype="bfloat16",
    out_dtype="bfloat16",
    accum_dtype="float32",
    source_format="uint32",
    num_bits: int = 4,
    scale_size: int = 32,
    fast_dequant: bool = True,
    with_bias: bool = False,
    block_M: int = 256,
    block_N: int = 256,
    block_K: int = 64,
    num_stages: int = 2,
    threads: int = 256,
    split: int = 1,
    weight_format: str | None = None,
    scale_bias: int = 0,
) -> KernelAdapter:
    """MXFP4-weight GEMM: ``C[M,N] = A[M,K] @ (fp4(B[N,K/2]) * 2**(Scale[N,K/32] - scale_bias)).T (+ Bias)``.

    Same arguments as ``matmul`` of
    examples/dequantize_gemm/example_dequant_gemm_bf16_mxfp4_cdna4.py:61-79 (tile sizes, stages,
    threads and split are accepted and ignored).  ``C = kernel(A, B, Scale, Bias)`` as with the
    example's ``out_idx=[-1]``; ``Bias`` is read only when ``with_bias``.

    ``weight_format``: ``"twiddling"`` (the example's ``fast_dequant=True`` layout), ``"simple"``
    (``fast_dequant=False``) or ``"e2m1"`` (plain OCP nibbles); by default it follows
    ``fast_dequant`` like the example.  ``scale_bias=0`` multiplies by ``2**Scale`` like the
    example's reference program; ``scale_bias=127`` treats Scale as E8M0.
    """
    if num_bits != 4 or scale_size != 32:
        raise ValueError("matmul_bf16_mxfp4: num_bits must be 4 and scale_size 32")
    if _dtype(in_dtype) != torch.bfloat16 or _dtype(out_dtype) != torch.bfloat16:
        raise ValueError("matmul_bf16_mxfp4: in_dtype and out_dtype must be bfloat16")
    if K % 64 != 0:
        raise ValueError(f"matmul_bf16_mxfp4: K={K} must be a multiple of 64")
    if weight_format is None:
        weight_format = "twiddling" if fast_dequant else "simple"
    fmt = _FP4_FORMATS[weight_format]
    params = [
        KernelParam("A", torch.bfloat16, (M, K)),
        KernelParam("B", torch.uint8, (N, K // 2), packed=True),
        KernelParam("Scale", torch.uint8, (N, K // scale_size), packed=True),
        KernelParam("Bias", torch.bfloat16, (M, N)),
        KernelParam("C", torch.bfloat16, (M, N)),
    ]

    def launch(ptrs, stream):
        lib = _lib.get_library()
        bias = ptrs[3] if with_bias else None
        return lib.call_dequant_gemm_bf16_mxfp4(ptrs[0], ptrs[1], ptrs[2], bias, ptrs[4], M, N, K, scale_size, fmt, scale_bias, stream)

    return KernelAdapter("matmul_bf16_mxfp4", params, [-1], launch, _lib.last_error)


def matmul_bf16_fp4(
    M: int,
    N: int,
    K: int,
    in_dtype="bfloat16",
    out_dtype="bfloat16",
    accum_dtype="float32",
    source_format="uint32",
    num_bits: int = 4,
    fast_dequant: bool = True,
    block_M: int = 256,
    block_N: int = 128,
    block_K: int = 128,
    num_stages: int = 2,
    threads: int = 256,
    split: int = 1,
    weight_format: str | None = None,
) -> KernelAdapter:
    """FP4-weight GEMM without block scales: ``C[M,N] = A[M,K] @ bf16(fp4(B[N,K/2])).T``.

    Same arguments as ``matmul`` of
    examples/dequantize_gemm/example_dequant_gemm_bf16_fp4_hopper.py:46-62 (tile sizes, stages, threads and split are
    accepted and ignored) and the same call, ``C = kernel(A, qB)`` with the example's ``out_idx=[-1]``.
    ``fast_dequant=True`` reads the bit-twiddled layout that ``ref_program_twiddling`` (:348-366) decodes,
    ``fast_dequant=False`` the plain nibbles of ``ref_program_simple`` (:369-386); ``weight_format`` ("twiddling",
    "simple", "e2m1") overrides the choice as in ``matmul_bf16_mxfp4``.
    """
    if num_bits != 4:
        raise ValueError("matmul_bf16_fp4: num_bits must be 4")
    if _dtype(in_dtype) != torch.bfloat16 or _dtype(out_dtype) != torch.bfloat16:
        raise ValueError("matmul_bf16_fp4: in_dtype and out_dtype must be bfloat16")
    if K % 64 != 0:
        raise ValueError(f"matmul_bf16_fp4: K={K} must be a multiple of 64")
    if weight_format is None:
        weight_format = "twiddling" if fast_dequant else "simple"
    fmt = _FP4_FORMATS[weight_format]
    params = [
        KernelParam("A", torch.bfloat16, (M, K)),
        KernelParam("B", torch.uint8, (N, K // 2), packed=True),
        KernelParam("C", torch.bfloat16, (M, N)),
    ]

    def launch(ptrs, stream):
        return _lib.get_library().call_dequant_gemm_bf16_fp4(ptrs[0], ptrs[1], ptrs[2], M, N, K, fmt, stream)

    return KernelAdapter("matmul_bf16_fp4", params, [-1], launch, _lib.last_error)


def matmul_mxfp4_mxfp4(M: int, N: int, K: int, out_dtype="bfloat16", accum_dtype="float32", with_bias: bool = False) -> KernelAdapter:
    """Block-scaled MXFP4 x MXFP4 GEMM on the gfx950 scaled matrix instruction:
    ``C[M,N] = (e2m1(A[M,K/2]) * 2**(SFA[M,K/32] - 127)) @ (e2m1(B[N,K/2]) * 2**(SFB[N,K/32] - 127)).T (+ Bias)``.

    ``C = kernel(A, B, SFA, SFB, Bias)``: the argument order of ``mxfp8_blockscaled_gemm`` of
    examples/blockscaled_gemm_sm100/gemm_mxfp8_blockscaled_1d1d.py:17-60 (A, B ``[N, K]`` as with its
    ``transpose_B=True``, then the two scale tensors), with plain row-major E8M0 bytes instead of its packed
    group-major words, 32 k per scale, and the 4-bit element format of ``matmul_bf16_mxfp4``.  Both operands
    are what ``quantize_bf16_mxfp4(rows, K, scale_bias=127)`` writes.  ``Bias`` is read only when ``with_bias``.
    """
    if _dtype(out_dtype) != torch.bfloat16 or _dtype(accum_dtype) != torch.float32:
        raise ValueError("matmul_mxfp4_mxfp4: out_dtype must be bfloat16 and accum_dtype float32")
    if K % 128 != 0 or K < 256:
        raise ValueError(f"matmul_mxfp4_mxfp4: K={K} must be a multiple of 128 and at least 256")
    params = [
        KernelParam("A", torch.uint8, (M, K // 2), packed=True),
        KernelParam("B", torch.uint8, (N, K // 2), packed=True),
        KernelParam("SFA", torch.uint8, (M, K // 32), packed=True),
        KernelParam("SFB", torch.uint8, (N, K // 32), packed=True),
        KernelParam("Bias", torch.bfloat16, (M, N)),
        KernelParam("C", torch.bfloat16, (M, N)),
    ]

    def launch(ptrs, stream):
        lib = _lib.get_library()
        bias = ptrs[4] if with_bias else None
        return lib.call_gemm_mxfp4_mxfp4(ptrs[0], ptrs[1], ptrs[2], ptrs[3], bias, ptrs[5], M, N, K, stream)

    return KernelAdapter("matmul_mxfp4_mxfp4", params, [-1], launch, _lib.last_error)


def matmul_fp16_fp4(
    M: int,
    N: int,
    K: int,
    in_dtype="float16",
    out_dtype="float16",
    accum_dtype="float32",
    num_bits: int = 4,
    block_M: int = 128,
    block_N: int = 128,
    block_K: int = 128,
    num_stages: int = 2,
    threads: int = 256,
    split: int = 1,
    transposed_output: bool = True,
) -> KernelAdapter:
    """fp16 x "simple" fp4 GEMM: ``Ct[N,M] = (A[M,K] @ fp4_to_f16(B[N,K/2]).T).T``.

    Same arguments as ``matmul`` of examples/dequantize_gemm/example_dequant_gemm_fp4_hopper.py:110-125;
    ``Ct = kernel(A, B)`` (``out_idx=[2]``).  ``split > 1`` is the example's ``main_split`` (:136-175): K is cut
    into ``split`` slices that run on their own workgroups, their fp16 partial results are added in fp16 by a
    second kernel; the partial-result buffer (the example's ``SplitC``) is allocated here once per device.
    ``transposed_output=False`` gives ``C[M,N]``.
    """
    if num_bits != 4:
        raise ValueError("matmul_fp16_fp4: num_bits must be 4")
    if _dtype(in_dtype) != torch.float16 or _dtype(out_dtype) != torch.float16:
        raise ValueError("matmul_fp16_fp4: in_dtype and out_dtype must be float16")
    if K % 64 != 0:
        raise ValueError(f"matmul_fp16_fp4: K={K} must be a multiple of 64")
    if split < 1 or K % (64 * split) != 0:
        raise ValueError(f"matmul_fp16_fp4: K={K} must be a multiple of 64 * split (split={split})")
    out_shape = (N, M) if transposed_output else (M, N)
    params = [
        KernelParam("A", torch.float16, (M, K)),
        KernelParam("B", torch.uint8, (N, K // 2), packed=True),
        KernelParam("Ct" if transposed_output else "C", torch.float16, out_shape),
    ]
    if split == 1:
        def launch(ptrs, stream):
            return _lib.get_library().call_dequant_gemm_fp16_fp4(ptrs[0], ptrs[1], ptrs[2], M, N, K, int(transposed_output), stream)

        return KernelAdapter("matmul_fp16_fp4", params, [2], launch, _lib.last_error)

    if (M * N) % 8 != 0:
        raise ValueError(f"matmul_fp16_fp4: M * N must be a multiple of 8 when split > 1 (got {M} x {N})")
    params.append(KernelParam("SplitC", torch.float16, (split,) + out_shape))

    def launch_split(ptrs, stream):
        return _lib.get_library().call_dequant_gemm_fp16_fp4_splitk(ptrs[0], ptrs[1], ptrs[3], ptrs[2], M, N, K, split,
                                                                    int(transposed_output), stream)

    return KernelAdapter("matmul_fp16_fp4_splitk", params, [2], launch_split, _lib.last_error, workspace_idx=[3])


_DT_CODE = {torch.float16: 0, torch.bfloat16: 1, torch.int8: 2, torch.float32: 3, torch.int32: 4}


def matmul(
    M: int,
    N: int,
    K: int,
    block_M: int = 128,
    block_N: int = 128,
    block_K: int = 32,
    trans_A: bool = False,
    trans_B: bool = True,
    in_dtype="float16",
    out_dtype="float16",
    accum_dtype="float32",
    num_stages: int = 0,
    threads: int = 128,
    k_pack: int = 1,
) -> KernelAdapter:
    """Plain GEMM on the MFMA tile the dequantize GEMMs share: ``C[M,N] = op(A) @ op(B)``, ``C = kernel(A, B)``.

    Same arguments as ``matmul`` of testing/python/kernel/test_tilelang_kernel_gemm.py:5-49 (``k_pack`` from
    testing/python/amd/test_tilelang_test_amd.py:7-22): ``A`` is ``[K,M]`` when ``trans_A`` else ``[M,K]``, ``B`` is
    ``[N,K]`` when ``trans_B`` else ``[K,N]``.  float16 / bfloat16 inputs give an output of the same type or
    float32; int8 gives int32 (exact).  Accumulation is always fp32 / int32.  Tile, stage, thread and k_pack
    arguments are accepted and ignored.
    """
    it, ot = _dtype(in_dtype), _dtype(out_dtype)
    if it not in (torch.float16, torch.bfloat16, torch.int8):
        raise ValueError(f"matmul: in_dtype must be float16, bfloat16 or int8 (got {in_dtype})")
    if (it == torch.int8 and ot != torch.int32) or (it != torch.int8 and ot not in (it, torch.float32)):
        raise ValueError(f"matmul: out_dtype {out_dtype} does not go with in_dtype {in_dtype}")
    kmult = 128 if it == torch.int8 else 64
    if K % kmult != 0:
        raise ValueError(f"matmul: K={K} must be a multiple of {kmult}")
    esz = 1 if it == torch.int8 else 2
    ws_bytes = (((M * K * esz + 255) // 256 * 256) if trans_A else 0) + (0 if trans_B else (N * K * esz + 255) // 256 * 256)
    params = [
        KernelParam("A", it, (K, M) if trans_A else (M, K)),
        KernelParam("B", it, (N, K) if trans_B else (K, N)),
        KernelParam("C", ot, (M, N)),
    ]
    if ws_bytes:
        params.append(KernelParam("Workspace", torch.uint8, (ws_bytes,)))

    def launch(ptrs, stream):
        ws = ptrs[3] if ws_bytes else None
        return _lib.get_library().call_gemm_plain(ptrs[0], ptrs[1], ptrs[2], ws, M, N, K, _DT_CODE[it], _DT_CODE[ot],
                                                  int(trans_A), int(trans_B), stream)

    return KernelAdapter("matmul", params, [2], launch, _lib.last_error, workspace_idx=[3] if ws_bytes else [])


def matmul_w4_fine_grained(
    M: int,
    N: int,
    K: int,
    block_M: int = 128,
    block_N: int = 128,
    block_K: int = 32,
    in_dtype="float16",
    out_dtype="float16",
    accum_dtype="float32",
    num_stages: int = 3,
    threads: int = 128,
    num_bits: int = 4,
) -> KernelAdapter:
    """Weight-only uint4 GEMM ``C[M,N] = A[M,K] @ q(B[N,K/2]).T`` with unsigned nibbles.

    Same arguments as ``matmul`` of examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:16-29;
    ``C = kernel(A, B)``.  ``in_dtype="float16"`` gives fp16 out (fp32 accumulation);
    ``in_dtype="int8"`` gives exact int32 out.
    """
    if num_bits != 4:
        raise ValueError("matmul_w4_fine_grained: num_bits must be 4")
    it = _dtype(in_dtype)
    if it == torch.float16:
        if K % 64 != 0:
            raise ValueError(f"matmul_w4_fine_grained: K={K} must be a multiple of 64")
        params = [KernelParam("A", torch.float16, (M, K)), KernelParam("B", torch.int8, (N, K // 2), packed=True),
                  KernelParam("C", torch.float16, (M, N))]

        def launch(ptrs, stream):
            return _lib.get_library().call_dequant_gemm_w4_fp16(ptrs[0], ptrs[1], None, None, ptrs[2], M, N, K, K, W4_UNSIGNED,
                                                                LAYOUT_PLAIN, stream)
    elif it == torch.int8:
        if K % 128 != 0:
            raise ValueError(f"matmul_w4_fine_grained: K={K} must be a multiple of 128 for int8")
        params = [KernelParam("A", torch.int8, (M, K)), KernelParam("B", torch.int8, (N, K // 2), packed=True),
                  KernelParam("C", torch.int32, (M, N))]

        def launch(ptrs, stream):
            return _lib.get_library().call_gemm_int8xint4(ptrs[0], ptrs[1], ptrs[2], M, N, K, 0, 0, 0, stream)
    else:
        raise ValueError("matmul_w4_fine_grained: in_dtype must be float16 or int8")
    return KernelAdapter("matmul_w4_fine_grained", params, [2], launch, _lib.last_error)


def matmul_w4a16(M: int, N: int, K: int, group_size: int = -1, source_format: str = "int", fast_decoding: bool = False,
                 with_scaling: bool = True, with_zeros: bool = False, zeros_mode: str = "original",
                 storage_dtype="int8", qzeros_format: str = "int16") -> KernelAdapter:
    """W4A16 GEMM for any M through the 256x256 MFMA kernel (tile-exact fp16 dequantisation):
    ``kernel(A, B[, Scale[, Zeros]], C)``, same decode options as :func:`dequantize_gemv`."""
    if group_size == -1:
        group_size = K
    if K % 64 != 0:
        raise ValueError(f"matmul_w4a16: K={K} must be a multiple of 64")
    mode = _w4_mode(source_format, fast_decoding, with_scaling, with_zeros, zeros_mode)
    layout = LAYOUT_INTERLEAVED if fast_decoding else LAYOUT_PLAIN
    groups = K // group_size
    params = [KernelParam("A", torch.float16, (M, K)), KernelParam("B", _dtype(storage_dtype), (N, K // 2), packed=True)]
    if with_scaling:
        params.append(KernelParam("Scale", torch.float16, (N, groups)))
    zwork, zfmt = None, None
    if with_zeros:
        zparam, zwork, zfmt = _zeros_params(N, groups, zeros_mode, qzeros_format)
        params.append(zparam)
    c_idx = len(params)
    params.append(KernelParam("C", torch.float16, (M, N)))
    if zwork is not None:
        params.append(zwork)

    def launch(ptrs, stream):
        lib = _lib.get_library()
        s = ptrs[2] if with_scaling else None
        z = ptrs[3] if with_zeros else None
        if zwork is not None:
            if lib.call_unpack_qzeros(z, ptrs[-1], N, groups, zfmt, stream) != 0:
                return -1
            z = ptrs[-1]
        return lib.call_dequant_gemm_w4_fp16(ptrs[0], ptrs[1], s, z, ptrs[c_idx], M, N, K, group_size, mode, layout, stream)

    return KernelAdapter("matmul_w4a16", params, [], launch, _lib.last_error, workspace_idx=[-1] if zwork is not None else [])


def matmul_int8xint4(
    M: int,
    N: int,
    K: int,
    in_dtype="int8",
    out_dtype="int32",
    accum_dtype="int32",
    num_bits: int = 4,
    block_M: int = 32,
    block_N: int = 32,
    block_K: int = 128,
    num_stages: int = 1,
    threads: int = 128,
) -> KernelAdapter:
    """W4A8: ``Ct[N,M] int32 = (A[M,K] int8 @ sext4(B[N,K/2]).T).T``, exact.

    Same arguments as ``matmul_int8xint4`` of examples/dequantize_gemm/example_dequant_gemm_w4a8.py:87-100;
    ``Ct = kernel(A, B)`` (``out_idx=[2]``).
    """
    if num_bits != 4 or _dtype(in_dtype) != torch.int8 or _dtype(out_dtype) != torch.int32:
        raise ValueError("matmul_int8xint4: int8 activations, 4-bit weights and int32 output only")
    if K % 128 != 0:
        raise ValueError(f"matmul_int8xint4: K={K} must be a multiple of 128")
    params = [KernelParam("A", torch.int8, (M, K)), KernelParam("B", torch.uint8, (N, K // 2), packed=True),
              KernelParam("Ct", torch.int32, (N, M))]

    def launch(ptrs, stream):
        return _lib.get_library().call_gemm_int8xint4(ptrs[0], ptrs[1], ptrs[2], M, N, K, 1, 0, 1, stream)

    return KernelAdapter("matmul_int8xint4", params, [2], launch, _lib.last_error)


def matmul_nt_int4(M: int, N: int, K: int, block_M: int = 128, block_N: int = 128, block_K: int = 64, threads: int = 128) -> KernelAdapter:
    """int4 x int4: ``C[M,N] int32 = sext4(A[M,K/2]) @ sext4(B[N,K/2]).T``, both operands packed two per byte.

    Same arguments as ``matmul_nt_int4`` of examples/gemm_int4/example_tilelang_gemm_int4.py:17-38;
    ``C = kernel(A_packed, B_packed)`` (``out_idx=-1``).
    """
    if K % 128 != 0:
        raise ValueError(f"matmul_nt_int4: K={K} must be a multiple of 128")
    params = [KernelParam("A", torch.int8, (M, K // 2), packed=True), KernelParam("B", torch.int8, (N, K // 2), packed=True),
              KernelParam("C", torch.int32, (M, N))]

    def launch(ptrs, stream):
        return _lib.get_library().call_gemm_int8xint4(ptrs[0], ptrs[1], ptrs[2], M, N, K, 1, 1, 0, stream)

    return KernelAdapter("matmul_nt_int4", params, [-1], launch, _lib.last_error)


def matmul_nt_int4xint2(M: int, N: int, K: int) -> KernelAdapter:
    """int4 x 2-bit: ``C[M,N] int32 = sext4(A[M,K/2]) @ c(B[N,K/4]).T`` with the 2-bit codes taken unsigned, the
    operand pair that decode_i2u_to_i4s / decode_i2s_to_i4s (examples/dequantize_gemm/quantize/lop3.py:1049-1089)
    prepare for the int4 x int4 matrix instruction of examples/gemm_int4/example_tilelang_gemm_int4.py:17-38 (the
    signed decoder's adjustment is commented out in the reference, so both decode to ``w = c``).
    ``C = kernel(A_packed, B_packed)``."""
    if K % 128 != 0:
        raise ValueError(f"matmul_nt_int4xint2: K={K} must be a multiple of 128")
    params = [KernelParam("A", torch.int8, (M, K // 2), packed=True), KernelParam("B", torch.int8, (N, K // 4), packed=True),
              KernelParam("C", torch.int32, (M, N))]

    def launch(ptrs, stream):
        return _lib.get_library().call_gemm_int8xint4(ptrs[0], ptrs[1], ptrs[2], M, N, K, I2_TO_I4, 1, 0, stream)

    return KernelAdapter("matmul_nt_int4xint2", params, [-1], launch, _lib.last_error)


I2_UNSIGNED, I2_OFFSET, I2_TWOS = 0, 1, 2
_I2_CONVENTIONS = {"unsigned": I2_UNSIGNED, "offset": I2_OFFSET, "twos": I2_TWOS}


def bitnet_158_int8xint2_prefill(
    M: int,
    N: int,
    K: int,
    in_dtype="int8",
    out_dtype="int32",
    accum_dtype="int32",
    fast_decoding: bool = True,
    block_row_warps: int = 2,
    block_col_warps: int = 2,
    warp_row_tiles: int = 32,
    warp_col_tiles: int = 32,
    chunk: int = 64,
    convention: str = "unsigned",
    kernel: str | None = None,
    weight_fragments: bool = False,
) -> KernelAdapter:
    """BitNet W2A8 GEMM: ``C[M,N] int32 = A[M,K] int8 @ decode(B[N,K/4]).T``, exact; ``kernel(A, B, C)``.

    Same arguments as ``bitnet_158_int8xint2_prefill`` of examples/bitnet-1.58b/kernel_benchmark/
    tilelang_bitnet_158_int8xint2_prefill.py:72-85.  As there, ``fast_decoding=True`` takes B as
    ``interleave_weight(general_compress(W, 2), 2, "int8")`` (:372-374); ``fast_decoding=False`` takes the plain
    packing ``general_compress(W, 2)``.  ``convention``: ``"unsigned"`` (what the example's kernel decodes),
    ``"offset"`` (``w = c - 2``, ternary weights stored as ``w + 2``) or ``"twos"``.  ``kernel`` (tests and
    measurements): ``"ksliced"`` or ``"tiled"`` instead of the library's choice by shape; same bits either way.
    ``weight_fragments=True``: B went through ``quantize.prepack_i2_fragments`` (after ``interleave_weight`` when
    ``fast_decoding``) and has the shape ``[ceil(N/32), K/128, 64, 16]`` (K % 2048 == 0); every batch size has a kernel
    that reads it: the decode kernel (M <= 4), the K-sliced kernel, the direct-to-LDS tiled kernel.
    """
    if _dtype(in_dtype) != torch.int8 or _dtype(out_dtype) != torch.int32:
        raise ValueError("bitnet_158_int8xint2_prefill: int8 in, int32 out")
    if K % 128 != 0:
        raise ValueError(f"bitnet_158_int8xint2_prefill: K={K} must be a multiple of 128")
    conv = _I2_CONVENTIONS[convention]
    layout = LAYOUT_INTERLEAVED if fast_decoding else LAYOUT_PLAIN
    b_shape = (N, K // 4)
    if weight_fragments:
        _i2_fragments_ok("bitnet_158_int8xint2_prefill", K, kernel)
        layout |= LAYOUT_FRAGMENTS
        b_shape = ((N + 31) // 32, K // 128, 64, 16)
    params = [KernelParam("A", torch.int8, (M, K)), KernelParam("B", torch.int8, b_shape, packed=True),
              KernelParam("C", torch.int32, (M, N))]

    def launch(ptrs, stream):
        return _lib.get_library().call_gemm_int8xint2(ptrs[0], ptrs[1], ptrs[2], M, N, K, conv, layout, None, 1.0, choice, stream)

    choice = _i2_kernel_choice("bitnet_158_int8xint2_prefill", kernel)
    return KernelAdapter("bitnet_158_int8xint2_prefill", params, [], launch, _lib.last_error)


_I2_KERNELS = {None: 0, "ksliced": 16, "tiled": 32, "resident": 64}  # DQ_I2_KERNEL_* of include/dqgemm.h


def _i2_fragments_ok(fn: str, K: int, kernel: str | None) -> None:
    # with K a multiple of 2048 the K-sliced kernel takes every shape, so some kernel always reads the order (the
    # decode kernel at M <= 4, the direct-to-LDS tiled kernel where the problem has enough tiles, else the K-sliced one)
    if K % 2048 != 0 or K >= 131072:
        raise ValueError(f"{fn}: weight_fragments needs K % 2048 == 0 and K < 131072 (got K={K})")


def _i2_kernel_choice(fn: str, kernel: str | None) -> int:
    if kernel not in _I2_KERNELS:
        raise ValueError(f"{fn}: kernel must be None, 'ksliced', 'tiled' or 'resident' (got {kernel!r})")
    return _I2_KERNELS[kernel]


def bitlinear_int8xint2(M: int, N: int, K: int, s_w: float, convention: str = "offset", interleaved: bool = False,
                        kernel: str | None = None, weight_fragments: bool = False) -> KernelAdapter:
    """BitLinear forward after activation quantisation: ``out[M,N] fp16 = ((A int8 @ W.T) / s_a[m]) / s_w``.

    The matmul plus ``post_quant_process`` of examples/bitnet-1.58b/utils_quant.py:165-170,199-209 in one
    kernel.  ``out = kernel(A, B, s_a)`` with ``s_a`` fp32 ``[M]`` (the per-row activation scale).
    ``interleaved``: B went through ``interleave_weight(.., 2, "int8")``.  ``kernel`` and ``weight_fragments``: as for
    :func:`bitnet_158_int8xint2_prefill`.
    """
    if K % 128 != 0:
        raise ValueError(f"bitlinear_int8xint2: K={K} must be a multiple of 128")
    conv = _I2_CONVENTIONS[convention]
    choice = _i2_kernel_choice("bitlinear_int8xint2", kernel)
    layout = LAYOUT_INTERLEAVED if interleaved else LAYOUT_PLAIN
    b_shape = (N, K // 4)
    if weight_fragments:
        _i2_fragments_ok("bitlinear_int8xint2", K, kernel)
        layout |= LAYOUT_FRAGMENTS
        b_shape = ((N + 31) // 32, K // 128, 64, 16)
    params = [KernelParam("A", torch.int8, (M, K)), KernelParam("B", torch.int8, b_shape, packed=True),
              KernelParam("s_a", torch.float32, (M,)), KernelParam("out", torch.float16, (M, N))]

    def launch(ptrs, stream):
        return _lib.get_library().call_gemm_int8xint2(ptrs[0], ptrs[1], ptrs[3], M, N, K, conv, layout, ptrs[2], float(s_w),
                                                      1 | choice, stream)

    return KernelAdapter("bitlinear_int8xint2", params, [-1], launch, _lib.last_error)


def bitnet_activation_quant(M: int, K: int) -> KernelAdapter:
    """BitLinear activation quantiser: ``x_q, s = kernel(x)`` with ``x`` fp16 ``[M, K]``, ``x_q`` int8 ``[M, K]``,
    ``s`` fp32 ``[M]``: ``s = 127 / max(|x|.max(-1), 1e-5)``, ``x_q = clamp(round(x.float() * s), -128, 127)``.

    One fused kernel for ``BitLinearBitBLAS.activation_quant`` of examples/bitnet-1.58b/utils_quant.py:156-163
    (there ``s`` is ``[M, 1]``); bit-identical results.
    """
    if K % 8 != 0:
        raise ValueError(f"bitnet_activation_quant: K={K} must be a multiple of 8")
    params = [KernelParam("x", torch.float16, (M, K)), KernelParam("x_q", torch.int8, (M, K)),
              KernelParam("s", torch.float32, (M,))]

    def launch(ptrs, stream):
        return _lib.get_library().call_bitnet_activation_quant(ptrs[0], ptrs[1], ptrs[2], M, K, stream)

    return KernelAdapter("bitnet_activation_quant", params, [1, 2], launch, _lib.last_error)


def quantize_bf16_mxfp4(N: int, K: int, scale_bias: int = 127) -> KernelAdapter:
    """MXFP4 weight quantiser: ``B, Scale = kernel(W)`` with ``W`` bf16 ``[N, K]``, ``B`` uint8 ``[N, K/2]`` (e2m1
    codes, even k in the low nibble) and ``Scale`` uint8 ``[N, K/32]`` — the operands that
    :func:`matmul_bf16_mxfp4` takes and that the reference's example draws at random
    (examples/dequantize_gemm/example_dequant_gemm_bf16_mxfp4_cdna4.py:286-290).

    Per block of 32: ``e = max(floor(log2(max|w|)) - 2, -127)``, ``Scale = clamp(e + scale_bias, 0, 255)``, codes =
    ``encode_fp4_e2m1_values(w / 2**(Scale - scale_bias))`` (examples/dequantize_gemm/quantize/nvfp4.py:120-138).
    """
    if K % 32 != 0:
        raise ValueError(f"quantize_bf16_mxfp4: K={K} must be a multiple of 32")
    if not 0 <= scale_bias <= 254:
        raise ValueError(f"quantize_bf16_mxfp4: scale_bias={scale_bias} must be in 0..254")
    params = [KernelParam("W", torch.bfloat16, (N, K)), KernelParam("B", torch.uint8, (N, K // 2)),
              KernelParam("Scale", torch.uint8, (N, K // 32))]

    def launch(ptrs, stream):
        return _lib.get_library().call_quantize_bf16_mxfp4(ptrs[0], ptrs[1], ptrs[2], N, K, scale_bias, stream)

    return KernelAdapter("quantize_bf16_mxfp4", params, [1, 2], launch, _lib.last_error)


def bitnet_158_int8xint2_decode(
    M: int,
    N: int,
    K: int,
    in_dtype="int8",
    out_dtype="int32",
    accum_dtype="int32",
    fast_decoding: bool = True,
    n_partition: int = 4,
    reduce_thread: int = 32,
    convention: str = "unsigned",
) -> KernelAdapter:
    """BitNet W2A8 decode GEMV: ``C[M,N] int32 = A[M,K] int8 @ decode(B[N,K/4]).T``, exact; ``kernel(A, B, C)``.

    Same arguments as ``bitnet_158_int8xint2_decode`` of examples/bitnet-1.58b/kernel_benchmark/
    tilelang_bitnet_158_int8xint2_decode.py:66-76.  M <= 4 runs the streaming dot4 kernel, larger M the
    MFMA GEMM.  ``fast_decoding`` (B interleaved or plain) and ``convention`` as in
    :func:`bitnet_158_int8xint2_prefill`.
    """
    k = bitnet_158_int8xint2_prefill(M, N, K, in_dtype, out_dtype, accum_dtype, fast_decoding, convention=convention)
    k.name = "bitnet_158_int8xint2_decode"
    return k
