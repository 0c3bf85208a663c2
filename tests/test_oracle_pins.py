"""Pins of the CPU oracle (no GPU): golden vectors the reference's own tests hold, closed forms,
brute force over finite domains, round trips, and reduction to integer / float64 arithmetic."""

import itertools
import json
import os

from fractions import Fraction

import numpy as np
import pytest

from oracle import dq_oracle as orc

with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_known_answers.json")) as _f:
    GOLDEN = json.load(_f)
E2M1 = GOLDEN["e2m1_value_table"]["values_by_code"]
assert len(E2M1) == 16


# ---- golden vectors from the reference's tests ---------------------------------------------------

@pytest.mark.parametrize("nbit,values", [(c["nbit"], c["values"]) for c in GOLDEN["signed_subword_decode"]["cases"]])
def test_sign_extend_known_answers(nbit, values):
    """testing/python/issue/test_tilelang_u32_signed_decode.py:26-30: pack (value & mask) << (pos * nbit), decode."""
    mask = (1 << nbit) - 1
    lanes = 32 // nbit
    words = []
    for start in range(0, len(values), lanes):
        w = 0
        for pos, v in enumerate(values[start:start + lanes]):
            w |= (v & mask) << (pos * nbit)
        words.append(w)
    out = []
    for i in range(len(values)):
        field = (words[i // lanes] >> ((i % lanes) * nbit)) & mask
        out.append(int(orc.sign_extend(np.array([field]), nbit)[0]))
    assert out == values


def test_e2m1_encode_pack_known_answer():
    """testing/python/quantize/test_tilelang_quantize_nvfp4_scale_layout.py:881-887."""
    kat = GOLDEN["e2m1_encode_pack"]
    values = np.array([kat["values"]], dtype=np.float32)
    codes = orc.encode_fp4_e2m1_values(values)
    assert codes.tolist() == [kat["codes"]]
    packed = orc.pack_fp4_e2m1_codes(codes)
    assert packed.tolist() == [kat["packed_low_nibble_first"]]
    np.testing.assert_array_equal(orc.decode_fp4_e2m1(packed), values)


def test_e2m1_table_all_bytes():
    """Value table of nvfp4.py:17-34 / test_tilelang_mxfp4_gfx950.py:32,49, for all 256 bytes, low nibble first."""
    b = np.arange(256, dtype=np.uint8).reshape(1, 256)
    got = orc.decode_fp4_e2m1(b).reshape(256, 2)
    for byte in range(256):
        assert got[byte, 0] == E2M1[byte & 15] and got[byte, 1] == E2M1[byte >> 4]
        assert np.signbit(got[byte, 0]) == (byte & 8 != 0) and np.signbit(got[byte, 1]) == (byte & 0x80 != 0)


# ---- closed forms over finite domains ------------------------------------------------------------

def test_simple_fp4_closed_form():
    """bits (s<<15)|((E+126)<<7)|(m<<6) is the bf16 (-1)^s 2^(E-1) (1 + m/2) for every E; fp16 twin likewise."""
    b = np.arange(256, dtype=np.uint8).reshape(1, 256)
    bf = orc.bf16_bits_to_f32(orc.decode_fp4_simple_bf16_bits(b)).reshape(256, 2)
    h = orc.decode_fp4_simple_f16(b).astype(np.float32).reshape(256, 2)
    for byte in range(256):
        for half, nib in enumerate((byte & 15, byte >> 4)):
            s, E, m = nib >> 3, (nib >> 1) & 3, nib & 1
            want = (-1.0) ** s * 2.0 ** (E - 1) * (1 + m / 2)
            assert bf[byte, half] == want and h[byte, half] == want
    # agrees with true e2m1 except for E == 0 (0.5, 0.75 instead of 0, 0.5)
    for nib in range(16):
        if (nib >> 1) & 3:
            assert bf[nib, 0] == E2M1[nib]


def test_simple_fp4_scaled_exponent_clamp():
    """quantization.py:30-73: the scale byte adds to the exponent, clamped at 255."""
    b = np.array([[0x31, 0xF7]], dtype=np.uint8)  # 4 nibbles
    sc = np.array([[3]], dtype=np.uint8)
    got = orc.bf16_bits_to_f32(orc.decode_fp4_simple_bf16_bits(b, sc, scale_size=4))
    base = orc.bf16_bits_to_f32(orc.decode_fp4_simple_bf16_bits(b))
    np.testing.assert_array_equal(got, base * 8)
    big = orc.decode_fp4_simple_bf16_bits(b, np.array([[250]], dtype=np.uint8), scale_size=4)
    assert ((big >> 7) & 0xFF).max() == 255


def test_twiddling_all_65536_units():
    """dequantize_utils.py:4-54 over every 16-bit unit: each of the 4 outputs is the e2m1 value of the code
    gathered from the documented bit positions."""
    w = np.arange(65536, dtype=np.uint32)
    packed = np.stack((w >> 8, w & 0xFF), axis=-1).astype(np.uint8).reshape(1, -1)
    got = orc.decode_fp4_twiddling(packed).reshape(65536, 4)
    pos = [(15, 8, 7, 6), (12, 5, 4, 3), (9, 2, 1, 0), (14, 11, 10, 13)]
    lut = np.array(E2M1, dtype=np.float32)
    for p, (s, e1, e0, m) in enumerate(pos):
        code = (((w >> s) & 1) << 3) | (((w >> e1) & 1) << 2) | (((w >> e0) & 1) << 1) | ((w >> m) & 1)
        want = lut[code]
        np.testing.assert_array_equal(got[:, p], want)
        np.testing.assert_array_equal(np.signbit(got[:, p]), np.signbit(want))


def test_twiddle_pack_round_trip():
    rng = np.random.default_rng(0)
    codes = rng.integers(0, 16, size=(7, 64), dtype=np.uint8)
    np.testing.assert_array_equal(orc.decode_fp4_twiddling(orc.twiddle_pack_fp4(codes)), orc.E2M1_VALUES[codes])


def test_magic_number_int_to_fp16():
    """(0x6400 | q) is the fp16 1024 + q; minus 1032 / 1024 gives q - 8 / q exactly (lop3.py:12-24)."""
    for q in range(16):
        assert np.array([0x6400 | q], dtype=np.uint16).view(np.float16)[0] == 1024 + q
    w = np.array([0x76543210, 0xFEDCBA98], dtype=np.uint32)
    # fast decode emits nibble pairs (i, i+4)
    got_u = orc.fast_decode_i4_to_f16(w, signed=False)
    assert got_u[0].tolist() == [0, 4, 1, 5, 2, 6, 3, 7]
    assert orc.fast_decode_i4_to_f16(w, signed=True)[1].tolist() == [0, 4, 1, 5, 2, 6, 3, 7]


def test_w4_scale_single_rounding():
    """(q - 8) * s in fp16 with one rounding equals the correctly rounded exact product for all q and many s."""
    rng = np.random.default_rng(1)
    s = rng.uniform(1e-4, 2.0, size=(1, 512)).astype(np.float16)
    for q in range(16):
        packed = np.full((1, 256), q | (q << 4), dtype=np.uint8)
        got = orc.dequant_u4_scale(packed, s, group=1)
        want = np.array([np.float16(float(q - 8) * float(x)) for x in s[0]], dtype=np.float16)  # exact in float64, one rounding
        np.testing.assert_array_equal(got[0].view(np.uint16), want.view(np.uint16))


def test_w4_zeros_modes_rounding_order():
    packed = np.array([[0xF0, 0x7A]], dtype=np.uint8)  # q = 0, 15, 10, 7
    s = np.array([[0.0123]], dtype=np.float16)
    z = np.array([[7.5]], dtype=np.float16)
    q = np.array([0, 15, 10, 7], dtype=np.float64)
    orig = orc.dequant_u4_scale_zeros(packed, s, z, 4, "original")[0]
    want = [np.float16(float(np.float16(x - 7.5)) * float(s[0, 0])) for x in q]
    assert orig.tolist() == [float(v) for v in want]
    resc = orc.dequant_u4_scale_zeros(packed, s, z, 4, "rescale")[0]
    want = [np.float16(x * float(s[0, 0]) - 7.5) for x in q]
    assert resc.tolist() == [float(v) for v in want]
    quant = orc.dequant_u4_scale_zeros(packed, s, np.array([[7]]), 4, "quantized")[0]
    want = [np.float16((x - 7) * float(s[0, 0])) for x in q]
    assert quant.tolist() == [float(v) for v in want]


def _rne(x: Fraction, mant_bits: int, emin: int, emax: int) -> float:
    """Round an exact rational to the nearest value of a binary floating-point format (ties to even), written out
    with integers only: `mant_bits` stored mantissa bits, normal exponents emin..emax, subnormals below."""
    if x == 0:
        return 0.0
    sign, a = (-1.0 if x < 0 else 1.0), abs(x)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    assert Fraction(2) ** e <= a < Fraction(2) ** (e + 1)
    e = max(e, emin)
    quantum = Fraction(2) ** (e - mant_bits)
    n = a / quantum
    lo = n.numerator // n.denominator
    rem = n - lo
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and lo % 2 == 1):
        lo += 1
    val = lo * quantum
    if val >= Fraction(2) ** (emax + 1):
        return sign * float("inf")
    return sign * float(val)


def _rne16(x):
    return _rne(Fraction(x), 10, -14, 15)


def _rne32(x):
    return _rne(Fraction(x), 23, -126, 127)


def test_rne_helper_against_numpy_casts():
    rng = np.random.default_rng(11)
    xs = np.concatenate([rng.standard_normal(500) * 10.0 ** rng.integers(-8, 5, 500), [65504.0, 65519.9, 65520.0, 6e-8, 2.98e-8, 0.0]])
    for x in xs:
        assert _rne16(Fraction(float(x))) == float(np.float64(x).astype(np.float16))
        assert _rne32(Fraction(float(x))) == float(np.float64(x).astype(np.float32))


def test_w4_decoders_rounding_order_step_by_step():
    """Every scaled / zero-point uint4 decoder against its operation order written out with exact rationals and an
    explicit round-to-nearest-even per fp16 instruction (examples/dequantize_gemm/quantize/lop3.py:41-81, 136-176,
    233-271, 326-363): sub.f16x2 rounds, fma.rn.f16x2 rounds once."""
    rng = np.random.default_rng(12)
    scales = np.concatenate([rng.uniform(1e-4, 2.0, 60), [6.1e-5, 1.0, 0.013, 655.0]]).astype(np.float16)
    zeros = np.array([0.0, 7.0, 7.5, 8.0, 15.0, -3.25, 6.0, 10.0, 0.3335], dtype=np.float16)
    qz_int = [0, 1, 7, 8, 15, 100, 1023]
    for s in scales:
        S = np.array([[s]], dtype=np.float16)
        fs = Fraction(float(s))
        packed = np.array([[(2 * i) | ((2 * i + 1) << 4) for i in range(8)]], dtype=np.uint8)  # q = 0..15
        got = orc.dequant_u4_scale(packed, S, 16)[0]
        assert got.tolist() == [_rne16((q - 8) * fs) for q in range(16)]
        for z in zeros:
            Z = np.array([[z]], dtype=np.float16)
            fz = Fraction(float(z))
            got = orc.dequant_u4_scale_zeros(packed, S, Z, 16, "original")[0]
            assert got.tolist() == [_rne16(Fraction(_rne16(q - fz)) * fs) for q in range(16)]
            got = orc.dequant_u4_scale_zeros(packed, S, Z, 16, "rescale")[0]
            assert got.tolist() == [_rne16(q * fs - fz) for q in range(16)]
            # the library's folded form: z * s rounded to fp16 first, then one fused multiply-add per weight
            got = orc.dequant_u4_scale_zeros(packed, S, Z, 16, "folded")[0]
            fzs = Fraction(_rne16(fz * fs))
            assert got.tolist() == [_rne16(q * fs - fzs) for q in range(16)]
            # ... which stays within one fp16 step of z * s of the reference's "original" form
            orig = orc.dequant_u4_scale_zeros(packed, S, Z, 16, "original")[0].astype(np.float64)
            step = max(np.spacing(np.float16(abs(float(fz * fs)))), np.spacing(np.float16(15 * float(fs)))).astype(np.float64)
            assert np.abs(got.astype(np.float64) - orig).max() <= 2 * step
        for qz in qz_int:
            got = orc.dequant_u4_scale_zeros(packed, S, np.array([[qz]]), 16, "quantized")[0]
            want = [_rne16((q - qz) * fs) for q in range(16)]
            assert got.tolist() == want
            # the device snippet's own route: magic-number add, then one fma (emits nibble pairs (i, i + 4))
            w = np.array([0x76543210, 0xFEDCBA98], dtype=np.uint32)
            bits = orc.fast_decode_i4u_to_f16_zeros_quantized(w, s, qz)
            order = [0, 4, 1, 5, 2, 6, 3, 7]
            assert bits[0].tolist() == [want[i] for i in order]
            assert bits[1].tolist() == [want[8 + i] for i in order]
            # and the "original" decoder fed with fp16(qz) gives the same bits (what the library relies on)
            if qz <= 15:
                same = orc.dequant_u4_scale_zeros(packed, S, np.array([[qz]], dtype=np.float16), 16, "original")[0]
                np.testing.assert_array_equal(same.view(np.uint16), got.view(np.uint16))


def test_unpack_qzeros_formats():
    z = np.array([[3, 15, 0, 9, 7]], dtype=np.int16)
    assert orc.unpack_qzeros(z, 5, "int16").tolist() == [[3, 15, 0, 9, 7]]
    packed = np.array([[3 | (15 << 4), 0 | (9 << 4), 7]], dtype=np.uint8)
    assert orc.unpack_qzeros(packed, 5, "packed4").tolist() == [[3, 15, 0, 9, 7]]


def test_i4_to_i8_fast_decode_and_interleave():
    """decode_i4{u,s}_to_i8s (lop3.py:999-1047) over interleave_weight(., 4, "int8") words: the unsigned decoder gives
    back the plain nibbles in k order, the signed one q - 7 (its MEDIAN_NUM is 0x07070707), for every nibble value
    at every position."""
    one = orc.interleave_weight(np.array([0x76543210], dtype=np.uint32).view(np.int8), 4, "int8").view(np.uint32)[0]
    assert one == 0x73625140  # element e at byte e % 4, nibble slot e / 4
    got = orc.fast_decode_i4_to_i8(np.array([[0x73625140, 0xFBEAD9C8]], dtype=np.uint32), signed=False)[0]
    assert got.tolist() == list(range(16))
    got = orc.fast_decode_i4_to_i8(np.array([[0x73625140, 0xFBEAD9C8]], dtype=np.uint32), signed=True)[0]
    assert got.tolist() == [q - 7 for q in range(16)]
    rng = np.random.default_rng(13)
    raw = rng.integers(0, 256, size=(16, 64), dtype=np.uint8)
    raw[0, :16] = np.arange(16, dtype=np.uint8) * 17  # every nibble value in both halves
    il = orc.interleave_weight(raw.view(np.int8), 4, "int8").view(np.uint8)
    np.testing.assert_array_equal(orc.decode_i4_fast_int8(il, signed=False), orc.unpack_u4(raw).astype(np.int8))
    np.testing.assert_array_equal(orc.decode_i4_fast_int8(il, signed=True), orc.unpack_u4(raw).astype(np.int8) - 7)


def test_i1_to_i8_fast_decode_all_halfwords_and_interleave():
    """decode_i1{u,s}_to_i8s (lop3.py:893-948) over every 16-bit input, against its bit shuffle written out bit by
    bit: output element 4 i + b is input bit (i, 8 + i, 4 + i, 12 + i)[b]; the signed form is 2 c - 1.  Over words
    that went through interleave_weight(., 1, "int8") (with its extra nibble shuffle, utils.py:102-109) the decoder
    returns the codes in k order."""
    x = np.arange(65536, dtype=np.uint32)
    got_u = orc.fast_decode_i1_to_i8(x, signed=False)
    got_s = orc.fast_decode_i1_to_i8(x, signed=True)
    for i in range(4):
        for b, bit in enumerate((i, 8 + i, 4 + i, 12 + i)):
            c = ((x >> bit) & 1).astype(np.int8)
            np.testing.assert_array_equal(got_u[:, 4 * i + b], c)
            np.testing.assert_array_equal(got_s[:, 4 * i + b], 2 * c - 1)
    rng = np.random.default_rng(14)
    codes = rng.integers(0, 2, size=(8, 256)).astype(np.int8)
    codes[0, :32] = np.eye(32, dtype=np.int8)[5]  # a single set bit
    raw = orc.general_compress(codes, 1)
    il = orc.interleave_weight(raw.view(np.int8), 1, "int8").view(np.uint8)
    np.testing.assert_array_equal(orc.decode_i1_fast_int8(il, signed=False), codes)
    np.testing.assert_array_equal(orc.decode_i1_fast_int8(il, signed=True), 2 * codes - 1)
    np.testing.assert_array_equal(orc.decode_lowbit(raw, 1, "offset"), 2 * codes - 1)
    for k in range(32):  # every bit position of a word
        one = np.zeros((1, 32), dtype=np.int8)
        one[0, k] = 1
        w = orc.interleave_weight(orc.general_compress(one, 1).view(np.int8), 1, "int8").view(np.uint8)
        assert orc.decode_i1_fast_int8(w, signed=False)[0].tolist() == one[0].tolist()


def test_i2_to_i4_fast_decode():
    """decode_i2{u,s}_to_i4s (lop3.py:1049-1089): (w >> 2 i) & 0x33333333 leaves code 2 e + i in nibble e of output
    word i, for every code value at every position; nothing is subtracted (the signed adjustment is commented out in
    the reference)."""
    for k in range(16):
        for c in range(4):
            w = np.array([c << (2 * k)], dtype=np.uint32)
            out = orc.fast_decode_i2_to_i4(w)[0]
            want = [0, 0]
            want[k % 2] = c << (4 * (k // 2))
            assert out.tolist() == want
    rng = np.random.default_rng(15)
    codes = rng.integers(0, 4, size=(4, 128)).astype(np.int8)
    packed = orc.general_compress(codes, 2)
    nib = orc.unpack_u4(orc.decode_i2_fast_int4(packed))  # [4, 128] nibbles of the decoder's output
    want = codes.reshape(4, 8, 8, 2).transpose(0, 1, 3, 2).reshape(4, 128)  # per 16 codes: the even ones, then the odd ones
    np.testing.assert_array_equal(nib, want)


def test_i2_conventions():
    packed = np.array([[0b11100100]], dtype=np.uint8)  # codes 0,1,2,3 low first
    assert orc.unpack_u2(packed).tolist() == [[0, 1, 2, 3]]
    assert orc.decode_i2(packed, "unsigned").tolist() == [[0, 1, 2, 3]]
    assert orc.decode_i2(packed, "offset").tolist() == [[-2, -1, 0, 1]]
    assert orc.decode_i2(packed, "twos").tolist() == [[0, 1, -2, -1]]


def test_bf16_rounding_helper():
    x = np.array([1.0, 1.00390625, 1.01171875, 3.0e38, -2.5, 1e-40], dtype=np.float32)
    import torch

    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    np.testing.assert_array_equal(orc.f32_to_bf16_bits(x), want)


# ---- packing invariants ---------------------------------------------------------------------------

@pytest.mark.parametrize("bits", [1, 2, 4])
def test_general_compress_round_trip(bits):
    rng = np.random.default_rng(bits)
    x = rng.integers(0, 1 << bits, size=(5, 64), dtype=np.int8)
    p = orc.general_compress(x, bits)
    assert p.dtype == np.int8 and p.shape == (5, 64 * bits // 8)
    np.testing.assert_array_equal(orc.general_decompress(p, bits), x.astype(np.uint8))
    # element j*epb + k sits at bit bits*k of byte j
    epb = 8 // bits
    assert (int(p.view(np.uint8)[0, 0]) >> (bits * 1)) & ((1 << bits) - 1) == x[0, 1]
    assert epb * p.shape[1] == x.shape[1]


def test_interleave_fast_decode_equals_plain_decode():
    """fast_decode(interleave_weight(p)) == plain_decode(p) for random words (4 bit -> fp16, 2 bit -> int8)."""
    rng = np.random.default_rng(0)
    raw = rng.integers(0, 256, size=(16, 64), dtype=np.uint8)
    il = orc.interleave_weight(raw.view(np.int8), 4, "float16")
    fast = orc.fast_decode_i4_to_f16(il.view(np.uint32).reshape(16, -1), signed=False).reshape(16, -1)
    np.testing.assert_array_equal(fast, orc.unpack_u4(raw).astype(np.float16))
    il2 = orc.interleave_weight(raw.view(np.int8), 2, "int8")
    fast2 = orc.fast_decode_i2_to_i8(il2.view(np.uint32).reshape(16, -1), signed=True).reshape(16, -1)
    np.testing.assert_array_equal(fast2, orc.decode_i2(raw, "offset"))
    # a bit permutation: population count preserved, and nibble order 0,2,4,6,1,3,5,7
    assert np.unpackbits(il.view(np.uint8)).sum() == np.unpackbits(raw).sum()
    one = orc.interleave_weight(np.array([0x76543210], dtype=np.uint32).view(np.int8), 4, "float16").view(np.uint32)[0]
    assert one == 0x75316420


@pytest.mark.parametrize("nbits,target", [(1, "int8"), (2, "float16"), (1, "float16"), (2, "int8"), (4, "int8")])
def test_interleave_is_bit_permutation(nbits, target):
    for bit in range(32):
        w = np.array([1 << bit], dtype=np.uint32)
        out = orc.interleave_weight(w.view(np.int8), nbits, target).view(np.uint32)[0]
        assert bin(int(out)).count("1") == 1
    outs = {int(orc.interleave_weight(np.array([1 << b], dtype=np.uint32).view(np.int8), nbits, target).view(np.uint32)[0]) for b in range(32)}
    assert len(outs) == 32


def test_pack_int4():
    x = np.array([[-8, 7, -1, 0, 3, -4]], dtype=np.int8)
    p = orc.pack_int4(x)
    assert p.view(np.uint8).tolist() == [[0x78, 0x0F, 0xC3]]
    np.testing.assert_array_equal(orc.decode_i4_signed(p), x)
    with pytest.raises(TypeError):
        orc.pack_int4(x.astype(np.int32))
    with pytest.raises(ValueError):
        orc.pack_int4(x[:, :5])


# ---- matmuls against brute force ------------------------------------------------------------------

def test_ref_w4a16_brute_force():
    rng = np.random.default_rng(2)
    M, N, K, g = 2, 5, 64, 32
    A = rng.standard_normal((M, K)).astype(np.float16)
    B = rng.integers(0, 256, size=(N, K // 2), dtype=np.uint8)
    S = rng.uniform(0.005, 0.02, size=(N, K // g)).astype(np.float16)
    got = orc.ref_w4a16(A, B, S, group=g, mode="scale")
    for m, n in itertools.product(range(M), range(N)):
        acc = 0.0
        for k in range(K):
            q = (B[n, k // 2] >> (4 * (k % 2))) & 15
            w = np.float16(np.float64(q - 8.0) * np.float64(S[n, k // g]))
            acc += float(A[m, k]) * float(w)
        assert abs(float(got[m, n]) - acc) <= 2e-3 * max(1.0, abs(acc))


def test_ref_int_paths_brute_force():
    rng = np.random.default_rng(3)
    M, N, K = 3, 4, 32
    A = rng.integers(-128, 128, size=(M, K)).astype(np.int8)
    B4 = rng.integers(0, 256, size=(N, K // 2), dtype=np.uint8)
    B2 = rng.integers(0, 256, size=(N, K // 4), dtype=np.uint8)
    w4 = np.zeros((N, K), dtype=np.int64)
    w2 = np.zeros((N, K), dtype=np.int64)
    for n, k in itertools.product(range(N), range(K)):
        q = (int(B4[n, k // 2]) >> (4 * (k % 2))) & 15
        w4[n, k] = q - 16 if q >= 8 else q
        w2[n, k] = ((int(B2[n, k // 4]) >> (2 * (k % 4))) & 3) - 2
    a = A.astype(np.int64)
    np.testing.assert_array_equal(orc.ref_w4a8(A, B4), (a @ w4.T).T)
    np.testing.assert_array_equal(orc.ref_bitnet_int(A, B2, "offset"), a @ w2.T)
    Ap = rng.integers(0, 256, size=(M, K // 2), dtype=np.uint8)
    a4 = orc.decode_i4_signed(Ap).astype(np.int64)
    np.testing.assert_array_equal(orc.ref_int4xint4(Ap, B4), a4 @ w4.T)
    assert orc.ref_w4a8(A, B4).dtype == np.int32 and orc.ref_w4a8(A, B4).shape == (N, M)
    # the fine-grained example's int8 path (unsigned nibbles) and the unscaled fp16 tiles, nibble by nibble
    u4 = np.array([[(int(B4[n, k // 2]) >> (4 * (k % 2))) & 15 for k in range(K)] for n in range(N)], dtype=np.int64)
    np.testing.assert_array_equal(orc.ref_u4_int8(A, B4), a @ u4.T)
    assert orc.ref_u4_int8(A, B4).dtype == np.int32
    np.testing.assert_array_equal(orc.dequant_u4_plain(B4, signed=False).astype(np.int64), u4)
    np.testing.assert_array_equal(orc.dequant_u4_plain(B4, signed=True).astype(np.int64), w4)
    assert orc.dequant_u4_plain(B4).dtype == np.float16


def test_ref_mxfp4_exact_scaling_and_identity():
    rng = np.random.default_rng(4)
    N, K = 8, 64
    B = rng.integers(0, 256, size=(N, K // 2), dtype=np.uint8)
    S = rng.integers(119, 128, size=(N, K // 32), dtype=np.uint8)
    W = orc.mxfp4_dequant(B, S, "e2m1", 32, 127)
    # exact: every value is an e2m1 value times a power of two, hence a bf16
    np.testing.assert_array_equal(orc.round_to_bf16(W), W)
    eye = orc.f32_to_bf16_bits(np.eye(K, dtype=np.float32))
    C = orc.bf16_bits_to_f32(orc.ref_mxfp4(eye, B, S, fmt="e2m1", scale_bias=127))
    np.testing.assert_array_equal(C, W.T)
    # reference mode: raw exponent, 2**Scale
    W0 = orc.mxfp4_dequant(B, np.full((N, 2), 2, np.uint8), "e2m1", 32, 0)
    np.testing.assert_array_equal(W0, orc.decode_fp4_e2m1(B) * 4)


def test_ref_fp16xfp4_splitk_closed_forms():
    """One slice is the plain reference program; with small integers every partial result is exact in fp16 and the
    split form equals the unsplit one; in general it is the slice products rounded to fp16 and added in fp16 in order
    (example_dequant_gemm_fp4_hopper.py:136-175), restated here with explicit loops."""
    rng = np.random.default_rng(8)
    M, N, K = 5, 7, 256
    A = (rng.standard_normal((M, K), dtype=np.float32)).astype(np.float16)
    B = rng.integers(0, 256, size=(N, K // 2), dtype=np.uint8)
    np.testing.assert_array_equal(orc.ref_fp16xfp4_splitk(A, B, 1), orc.ref_fp16xfp4(A, B).T)
    Ai = rng.integers(-2, 3, size=(M, K)).astype(np.float16)
    Bi = B & 0x33
    np.testing.assert_array_equal(orc.ref_fp16xfp4_splitk(Ai, Bi, 4), orc.ref_fp16xfp4(Ai, Bi).T)
    W = orc.decode_fp4_simple_f16(B).astype(np.float64)
    want = np.zeros((M, N), dtype=np.float16)
    for m in range(M):
        for n in range(N):
            acc = np.float16(0)
            for z in range(4):
                part = np.float16(np.float32(np.dot(A[m, z * 64:(z + 1) * 64].astype(np.float64), W[n, z * 64:(z + 1) * 64])))
                acc = np.float16(np.float32(acc) + np.float32(part))
            want[m, n] = acc
    got = orc.ref_fp16xfp4_splitk(A, B, 4)
    # the fp32 matmul of a slice may differ from the float64 dot in the last fp32 bit, i.e. by at most one fp16 ulp
    np.testing.assert_allclose(got.astype(np.float32), want.astype(np.float32), rtol=2e-3, atol=2e-3)


def test_ref_mxfp4_mxfp4_brute_force_and_scale_linearity():
    """Block-scaled product against a plain triple loop over the e2m1 table (nvfp4.py:17-34) and 2**(sf - 127)
    (gemm_mxfp8_blockscaled_1d1d.py:602-603); with every scale at 127 it is the plain matmul of the decoded
    codes; adding one to a scale byte of A doubles that block's contribution and nothing else."""
    table = np.array([0, 0.5, 1, 1.5, 2, 3, 4, 6, -0.0, -0.5, -1, -1.5, -2, -3, -4, -6], dtype=np.float64)
    rng = np.random.default_rng(11)
    M, N, K = 3, 5, 64
    ca = rng.integers(0, 16, size=(M, K), dtype=np.uint8)
    cb = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    sa = rng.integers(120, 131, size=(M, K // 32)).astype(np.uint8)
    sb = rng.integers(120, 131, size=(N, K // 32)).astype(np.uint8)
    A, B = orc.pack_fp4_e2m1_codes(ca), orc.pack_fp4_e2m1_codes(cb)
    want = np.zeros((M, N), dtype=np.float64)
    for m in range(M):
        for n in range(N):
            for k in range(K):
                want[m, n] += table[ca[m, k]] * 2.0 ** (int(sa[m, k // 32]) - 127) * table[cb[n, k]] * 2.0 ** (int(sb[n, k // 32]) - 127)
    got = orc.bf16_bits_to_f32(orc.ref_mxfp4_mxfp4(A, sa, B, sb))
    np.testing.assert_array_equal(got, orc.round_to_bf16(want.astype(np.float32)))
    ones_a, ones_b = np.full_like(sa, 127), np.full_like(sb, 127)
    plain = table[ca] @ table[cb].T
    np.testing.assert_array_equal(orc.bf16_bits_to_f32(orc.ref_mxfp4_mxfp4(A, ones_a, B, ones_b)),
                                  orc.round_to_bf16(plain.astype(np.float32)))
    # linearity in one scale block: block 1 of A row 0 one exponent up
    sa2 = sa.copy(); sa2[0, 1] += 1
    blk = np.zeros((M, N)); 
    for n in range(N):
        blk[0, n] = sum(table[ca[0, k]] * 2.0 ** (int(sa[0, 1]) - 127) * table[cb[n, k]] * 2.0 ** (int(sb[n, 1]) - 127) for k in range(32, 64))
    got2 = orc.bf16_bits_to_f32(orc.ref_mxfp4_mxfp4(A, sa2, B, sb))
    np.testing.assert_array_equal(got2, orc.round_to_bf16((want + blk).astype(np.float32)))
    # a scale byte of 255 is NaN for the whole output row
    sa3 = sa.copy(); sa3[1, 0] = 255
    got3 = orc.bf16_bits_to_f32(orc.ref_mxfp4_mxfp4(A, sa3, B, sb))
    assert np.isnan(got3[1]).all() and np.isfinite(got3[[0, 2]]).all()


def test_activation_quant_matches_torch_ops():
    """utils_quant.py:156-163 executed with torch's own CPU ops (the reference's statements verbatim in
    tilelang_amd.bitlinear.activation_quant_reference): scales bit-identical, codes identical, ties included."""
    import torch
    from tilelang_amd import bitlinear

    rng = np.random.default_rng(11)
    x = (rng.standard_normal((96, 1024), dtype=np.float32) * rng.uniform(0.01, 30.0, size=(96, 1)).astype(np.float32)).astype(np.float16)
    x[0, :8] = np.array([0.5, -0.5, 1.5, 2.5, -2.5, 0.0, 1e-4, -1e-4], dtype=np.float16)
    x[1, :] = 0
    q, s = orc.activation_quant(x)
    tq, ts = bitlinear.activation_quant_reference(torch.from_numpy(x))
    np.testing.assert_array_equal(s.view(np.uint32), ts.numpy().view(np.uint32))
    np.testing.assert_array_equal(q, tq.numpy())


def test_bitlinear_quantisers_and_epilogue():
    rng = np.random.default_rng(5)
    x = rng.standard_normal((3, 16)).astype(np.float32) * 3
    xq, s = orc.activation_quant(x)
    assert xq.dtype == np.int8 and np.abs(xq).max() == 127 and s.shape == (3, 1)
    np.testing.assert_allclose(s[:, 0], 127.0 / np.abs(x).max(axis=1), rtol=1e-6)
    w = rng.standard_normal((4, 16)).astype(np.float32)
    wq, sw = orc.weight_quant(w)
    assert set(np.unique(wq)).issubset({-1, 0, 1}) and abs(sw - 1 / np.abs(w).mean()) < 1e-5
    acc = np.array([[100, -7]], dtype=np.int32)
    out = orc.post_quant_process(acc, np.array([[4.0]], np.float32), np.float32(2.0))
    assert out.dtype == np.float16 and out.tolist() == [[12.5, -0.875]]
    # two fp32 divisions in that order, then one rounding to fp16 (utils_quant.py:165-170), with exact rationals and
    # an explicit rounding per operation; (acc / (s_a * s_w)) would differ in the last bit for some of these
    accs = rng.integers(-1040384, 1040385, size=200)
    sas = rng.uniform(0.5, 50.0, size=200).astype(np.float32)
    sws = rng.uniform(0.5, 4.0, size=200).astype(np.float32)
    for a, sa, sw_ in zip(accs, sas, sws):
        got = orc.post_quant_process(np.array([[a]], dtype=np.int32), np.array([[sa]], np.float32), np.float32(sw_))[0, 0]
        step1 = _rne32(Fraction(int(a)) / Fraction(float(sa)))
        step2 = _rne32(Fraction(step1) / Fraction(float(sw_)))
        assert float(got) == _rne16(Fraction(step2))


def test_torch_restatement_matches_numpy_oracle():
    import torch

    from oracle import ref_torch
    from tilelang_amd import workloads

    d = workloads.w4a16(2, 64, 256, 128, seed=1, zeros_range=(6, 10))
    a, b, s, z = (torch.from_numpy(d[k]) for k in ("A", "B", "Scale", "Zeros"))
    np.testing.assert_allclose(ref_torch.ref_w4a16(a, b, s).numpy().astype(np.float32),
                               orc.ref_w4a16(d["A"], d["B"], d["Scale"], group=128, mode="scale").astype(np.float32), rtol=2e-3, atol=2e-3)
    np.testing.assert_allclose(ref_torch.ref_w4a16(a, b, s, z).numpy().astype(np.float32),
                               orc.ref_w4a16(d["A"], d["B"], d["Scale"], d["Zeros"], 128, "original").astype(np.float32), rtol=2e-3, atol=2e-3)
    m = workloads.mxfp4(8, 32, 128, seed=2, scale_bias=127)
    got = ref_torch.ref_mxfp4_e2m1(torch.from_numpy(m["A"]).view(torch.bfloat16), torch.from_numpy(m["B"]), torch.from_numpy(m["Scale"]))
    want = orc.bf16_bits_to_f32(orc.ref_mxfp4(m["A"], m["B"], m["Scale"], fmt="e2m1", scale_bias=127))
    np.testing.assert_allclose(got.float().numpy(), want, rtol=1e-2, atol=1e-2)
    bn = workloads.bitnet(4, 16, 64, seed=3)
    got = ref_torch.ref_bitnet(torch.from_numpy(bn["A"]), torch.from_numpy(bn["B"]), torch.from_numpy(bn["s_a"]), float(bn["s_w"]))
    want = orc.ref_bitnet(bn["A"], bn["B"], bn["s_a"], bn["s_w"], "offset")
    np.testing.assert_allclose(got.numpy().astype(np.float32), want.astype(np.float32), rtol=2e-3, atol=2e-3)


def _bf16_pred(x):
    """Largest bf16 value below the positive bf16 value x."""
    bits = orc.f32_to_bf16_bits(np.asarray(x, dtype=np.float32))
    return orc.bf16_bits_to_f32((bits - 1).astype(np.uint16))


def test_quantize_mxfp4_closed_forms():
    """Block scale and element codes where the mathematics fixes them: a block whose maximum is 6 * 2^e or
    4 * 2^e keeps exponent e (codes 7 / 6); every e2m1 threshold goes up, its bf16 predecessor goes down; an
    all-zero block takes the smallest exponent; the sign bit is never set on a zero magnitude."""
    for e in (-20, -8, -1, 0, 3, 17):
        blk = np.zeros((1, 32), dtype=np.float32)
        blk[0, 5] = 6.0 * 2.0**e
        blk[0, 6] = -4.0 * 2.0**e
        blk[0, 7] = 7.5 * 2.0**e   # same binade as 6: saturates
        blk[0, 8] = -1e-30         # rounds to zero: no negative zero
        B, S = orc.quantize_mxfp4(blk, scale_bias=127)
        codes = orc.unpack_u4(B)[0]
        assert S[0, 0] == 127 + e
        assert list(codes[5:9]) == [7, 8 | 6, 7, 0]
    thresholds = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0], dtype=np.float32)
    blk = np.zeros((1, 32), dtype=np.float32)
    blk[0, 0] = 6.0                                  # pins the block exponent at 0
    blk[0, 1:8] = thresholds
    blk[0, 8:15] = _bf16_pred(thresholds)
    blk[0, 15:22] = -thresholds
    B, S = orc.quantize_mxfp4(blk)
    codes = orc.unpack_u4(B)[0]
    assert S[0, 0] == 127
    assert list(codes[1:8]) == [1, 2, 3, 4, 5, 6, 7]
    assert list(codes[8:15]) == [0, 1, 2, 3, 4, 5, 6]
    assert list(codes[15:22]) == [9, 10, 11, 12, 13, 14, 15]
    B, S = orc.quantize_mxfp4(np.zeros((2, 64), dtype=np.float32), scale_bias=127)
    assert (B == 0).all() and (S == 0).all()
    B, S = orc.quantize_mxfp4(np.zeros((2, 64), dtype=np.float32), scale_bias=0)   # raw-exponent mode clamps at 0
    assert (B == 0).all() and (S == 0).all()


def test_quantize_mxfp4_round_trip_and_idempotence():
    """quantize(dequantize(codes, scales)) gives the codes and scales back whenever every block holds a code of
    e2m1's top binade (4 or 6), and quantize is idempotent on arbitrary data."""
    rng = np.random.default_rng(11)
    N, K = 16, 256
    codes = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    codes[codes == 8] = 0                                       # negative zero is never produced
    top = rng.integers(0, 32, size=(N, K // 32))
    for n in range(N):
        for b in range(K // 32):
            codes[n, b * 32 + top[n, b]] = rng.choice([6, 7, 14, 15])
    scale = rng.integers(100, 140, size=(N, K // 32)).astype(np.uint8)
    packed = orc.pack_fp4_e2m1_codes(codes)
    w = orc.mxfp4_dequant(packed, scale, fmt="e2m1", scale_size=32, scale_bias=127)
    B, S = orc.quantize_mxfp4(w, scale_bias=127)
    np.testing.assert_array_equal(S, scale)
    np.testing.assert_array_equal(B, packed)

    x = orc.round_to_bf16((rng.standard_normal((N, K)) * np.exp2(rng.integers(-12, 12, size=(N, 1)))).astype(np.float32))
    B1, S1 = orc.quantize_mxfp4(x)
    d = orc.mxfp4_dequant(B1, S1, fmt="e2m1", scale_size=32, scale_bias=127)
    B2, S2 = orc.quantize_mxfp4(d)
    np.testing.assert_array_equal(B2, B1)
    # the block maximum always lands in e2m1's top binade (scaled value in [4, 8) -> code 6 or 7), which is what
    # makes the second pass choose the same exponent
    assert ((orc.unpack_u4(B1).reshape(N, K // 32, 32) & 7).max(axis=-1) >= 6).all()
    np.testing.assert_array_equal(S2, S1)
    # error bound: half a step of the binade the scaled value falls in, or the saturation gap of the top binade
    step = np.exp2(S1.astype(np.float64) - 127)[:, :, None]
    err = np.abs(x.reshape(N, K // 32, 32) - d.reshape(N, K // 32, 32))
    assert (err <= 2.0 * step + 1e-30).all()


def test_gen_quant4_quantize_properties():
    """The deterministic part of gen_quant4: scale = group absmax / 8 exactly; the largest element of a group
    quantises to +-8; weights already on the grid come back unchanged; error at most half a step otherwise."""
    rng = np.random.default_rng(5)
    K, N, g = 256, 24, 64
    w = rng.standard_normal((K, N)).astype(np.float16)
    ref, s, q = orc.gen_quant4_quantize(w, g)
    absmax = np.abs(w.reshape(K // g, g, N)).max(axis=1)
    np.testing.assert_array_equal((s.astype(np.float32) * 8).astype(np.float16), absmax)
    assert np.abs(q).max() == 8 and (np.abs(q.reshape(K // g, g, N)).max(axis=1) == 8).all()
    step = np.repeat(s.astype(np.float32), g, axis=0)
    # half a step, plus the fp16 roundings of w / s (before the rint) and of q * s: each below 2^-8 of a step
    assert (np.abs(w.astype(np.float32) - ref.astype(np.float32)) <= 0.51 * step).all()
    # on-grid weights: j * s0 with max |j| = 8 in every group
    j = rng.integers(-8, 9, size=(K, N))
    j.reshape(K // g, g, N)[:, 0, :] = 8
    s0 = np.float16(0.0078125) * rng.integers(1, 64, size=(K // g, N)).astype(np.float16)
    w_grid = (j.astype(np.float16) * np.repeat(s0, g, axis=0)).astype(np.float16)
    ref, s, q = orc.gen_quant4_quantize(w_grid, g)
    np.testing.assert_array_equal(s, s0)
    np.testing.assert_array_equal(q, j)
    np.testing.assert_array_equal(ref, w_grid)
    # the whole-K group of groupsize = -1
    ref, s, q = orc.gen_quant4_quantize(w, -1)
    assert s.shape == (1, N) and np.abs(q).max() == 8



def test_i2_to_f16_fast_decode_all_halfwords_and_interleave():
    """decode_i2{u,s}_to_f16 (lop3.py:424-463) over all 65536 inputs against the closed form (outputs 2i, 2i+1 are
    the fields at bit 2i of byte 0 and byte 1), and fast_decode(interleave_weight(p, 2, "float16")) == plain decode."""
    x = np.arange(65536, dtype=np.uint32)
    for signed in (False, True):
        out = orc.fast_decode_i2_to_f16(x, signed)
        for i in range(4):
            lo = ((x >> (2 * i)) & 3).astype(np.float32) - (2 if signed else 0)
            hi = ((x >> (8 + 2 * i)) & 3).astype(np.float32) - (2 if signed else 0)
            np.testing.assert_array_equal(out[:, 2 * i].astype(np.float32), lo)
            np.testing.assert_array_equal(out[:, 2 * i + 1].astype(np.float32), hi)
    rng = np.random.default_rng(5)
    raw = rng.integers(0, 256, size=(8, 64), dtype=np.uint8)
    il = orc.interleave_weight(raw.view(np.int8), 2, "float16")
    fast = orc.fast_decode_i2_to_f16(il.view(np.uint16).reshape(8, -1), signed=True).reshape(8, -1)
    np.testing.assert_array_equal(fast.astype(np.float32), orc.decode_i2(raw, "offset").astype(np.float32))
    fastu = orc.fast_decode_i2_to_f16(il.view(np.uint16).reshape(8, -1), signed=False).reshape(8, -1)
    np.testing.assert_array_equal(fastu, orc.dequant_u2(raw, "unsigned"))
    # the scaled decoder rounds the product once; with signed codes the product is exact
    s = np.float16(0.0137)
    sc = orc.fast_decode_i2_to_f16(x[:4096], True, scale=s).astype(np.float64)
    exact = orc.fast_decode_i2_to_f16(x[:4096], True).astype(np.float64) * float(s)
    np.testing.assert_array_equal(sc, exact)
    scu = orc.fast_decode_i2_to_f16(x[:4096], False, scale=s)
    np.testing.assert_array_equal(scu, (orc.fast_decode_i2_to_f16(x[:4096], False).astype(np.float64) * float(s)).astype(np.float16))


def test_ref_w2a16_brute_force():
    """dequant_u2 / ref_w2a16 against a triple loop in float64 on a tiny case, every convention, with and without scales."""
    rng = np.random.default_rng(11)
    M, N, K, g = 2, 5, 128, 64
    A = rng.standard_normal((M, K)).astype(np.float16)
    packed = rng.integers(0, 256, size=(N, K // 4), dtype=np.uint8)
    S = rng.uniform(0.01, 0.05, size=(N, K // g)).astype(np.float16)
    table = {"unsigned": [0, 1, 2, 3], "offset": [-2, -1, 0, 1], "twos": [0, 1, -2, -1]}
    for conv, tab in table.items():
        for scale in (None, S):
            want = np.zeros((M, N))
            for n in range(N):
                for k in range(K):
                    c = (int(packed[n, k // 4]) >> (2 * (k % 4))) & 3
                    w = float(tab[c])
                    if scale is not None:
                        w = float(np.float16(w * float(scale[n, k // g])))
                    for m in range(M):
                        want[m, n] += float(A[m, k]) * w
            got = orc.ref_w2a16(A, packed, conv, scale, g if scale is not None else -1).astype(np.float64)
            np.testing.assert_allclose(got, want, rtol=2e-3, atol=2e-3)
    # sign extension of the reference's own known answer (test_tilelang_u32_signed_decode.py:26-30): codes 2,3,0,1 -> -2..1
    np.testing.assert_array_equal(orc.dequant_u2(np.array([[0b01001110]], dtype=np.uint8), "twos")[0], np.array([-2, -1, 0, 1], dtype=np.float16))


def test_i1_to_f16_fast_decode_all_bytes_and_interleave():
    """decode_i1{u,s}_to_f16 (lop3.py:679-746) over all 256 inputs against the closed form (outputs 2i, 2i+1 are bits i
    and 4 + i: c, or 2c - 1 signed), fast_decode(interleave_weight(p, 1, "float16")) == plain decode, and the known
    answer of the reference's own sign-extension test for one bit (0 -> 0, 1 -> -1)."""
    x = np.arange(256, dtype=np.uint32)
    for signed in (False, True):
        out = orc.fast_decode_i1_to_f16(x, signed).astype(np.float32)
        for i in range(4):
            lo = ((x >> i) & 1).astype(np.float32)
            hi = ((x >> (4 + i)) & 1).astype(np.float32)
            if signed:
                lo, hi = 2 * lo - 1, 2 * hi - 1
            np.testing.assert_array_equal(out[:, 2 * i], lo)
            np.testing.assert_array_equal(out[:, 2 * i + 1], hi)
    raw = np.random.default_rng(8).integers(0, 256, size=(8, 64), dtype=np.uint8)
    il = orc.interleave_weight(raw.view(np.int8), 1, "float16").view(np.uint8)
    fast = orc.fast_decode_i1_to_f16(il, signed=True).reshape(8, -1)
    np.testing.assert_array_equal(fast.astype(np.float32), orc.decode_lowbit(raw, 1, "offset").astype(np.float32))
    fastu = orc.fast_decode_i1_to_f16(il, signed=False).reshape(8, -1)
    np.testing.assert_array_equal(fastu.astype(np.float32), orc.decode_lowbit(raw, 1, "unsigned").astype(np.float32))
    np.testing.assert_array_equal(orc.decode_lowbit(np.array([[0b10110010]], dtype=np.uint8), 1, "twos")[0], [0, -1, 0, 0, -1, -1, 0, -1])


def test_dequant_lowbit_rounding_order():
    """Zero-point forms: original rounds (w - z) then the product; rescale rounds the product then the difference;
    checked against float64 arithmetic with explicit roundings on values chosen so that the orders differ."""
    packed = np.array([[0b11100100]], dtype=np.uint8)  # 2-bit codes 0, 1, 2, 3
    s = np.array([[0.00949859619140625]], dtype=np.float16)
    z = np.array([[0.26904296875]], dtype=np.float16)
    c = np.array([0.0, 1.0, 2.0, 3.0])
    f16 = lambda v: np.asarray(v, dtype=np.float64).astype(np.float16).astype(np.float64)
    got_o = orc.dequant_lowbit(packed, 2, "unsigned", s, z, 4, "original").astype(np.float64)[0]
    np.testing.assert_array_equal(got_o, f16(f16(c - float(z[0, 0])) * float(s[0, 0])))
    got_r = orc.dequant_lowbit(packed, 2, "unsigned", s, z, 4, "rescale").astype(np.float64)[0]
    np.testing.assert_array_equal(got_r, f16(f16(c * float(s[0, 0])) - float(z[0, 0])))
    assert not np.array_equal(got_r, f16(c * float(s[0, 0]) - float(z[0, 0])))  # a single rounding would differ


# ---- vectors written by the reference's own pure-torch helpers (tests/golden/make_vectors.py) ----------------------

def _reference_vectors():
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_vectors.npz")
    return np.load(path, allow_pickle=False)


def test_reference_vectors_torch_convert_all_bytes():
    """examples/dequantize_gemm/dequantize_utils.py:57-84 run on every byte value, plain and with block exponents
    that reach the clamp at 255."""
    v = _reference_vectors()
    np.testing.assert_array_equal(orc.decode_fp4_simple_bf16_bits(v["convert_in"]), v["convert_out_bits"])
    np.testing.assert_array_equal(orc.decode_fp4_simple_bf16_bits(v["convert_in"], v["convert_scale"], 32), v["convert_scaled_out_bits"])


def test_reference_vectors_bit_twiddling_all_units():
    """examples/dequantize_gemm/dequantize_utils.py:4-54 run on all 65 536 byte pairs."""
    v = _reference_vectors()
    want = orc.bf16_bits_to_f32(v["twiddling_out_bits"])
    got = orc.decode_fp4_twiddling(v["twiddling_in"])
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))  # bit for bit, signs of zeros included


def test_reference_vectors_interleave_weight():
    """examples/dequantize_gemm/quantize/utils.py:71-125 run on 4096 seeded words.  Its byte-shuffle branches raise
    TypeError in torch (`torch.int32(...)` is not callable), so the reference itself yields vectors for three of the
    six cases only; the other three stay pinned by fast_decode(interleave(p)) == plain_decode(p)."""
    v = _reference_vectors()
    words = v["interleave_in"]
    for nbits, target in ((4, "float16"), (4, "int8"), (2, "int8")):
        got = orc.interleave_weight(words.view(np.int8), nbits, target).view(np.int32)
        np.testing.assert_array_equal(got, v[f"interleave_{nbits}_{target}"])
    raised = [str(x) for x in v["interleave_cases_the_reference_raises_on"]]
    assert len(raised) == 3 and all("not callable" in x for x in raised)


def test_reference_vectors_general_compress():
    """examples/dequantize_gemm/quantize/utils.py:50-67 run on seeded codes for 1, 2 and 4 bits."""
    v = _reference_vectors()
    for bits in (1, 2, 4):
        got = orc.general_compress(v[f"compress_in_{bits}"], bits)
        np.testing.assert_array_equal(got.view(np.uint8), v[f"compress_out_{bits}"].view(np.uint8))


def test_reference_vectors_match_the_library_helpers():
    """The package's own host helpers (tilelang_amd.quantize) against the same vectors."""
    import torch

    from tilelang_amd import quantize

    v = _reference_vectors()
    words = v["interleave_in"]
    for nbits, target in ((4, "float16"), (4, "int8"), (2, "int8")):
        got = quantize.interleave_weight(torch.from_numpy(words.copy()).view(torch.int8), nbits, target).numpy().view(np.int32)
        np.testing.assert_array_equal(got, v[f"interleave_{nbits}_{target}"])
    for bits in (1, 2, 4):
        got = quantize.general_compress(torch.from_numpy(v[f"compress_in_{bits}"].copy()), source_bits=bits).numpy()
        np.testing.assert_array_equal(got.view(np.uint8), v[f"compress_out_{bits}"].view(np.uint8))
