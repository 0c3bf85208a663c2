// int8 x 4-bit (W4A8, int8 x uint4), int4 x int4 and int4 x 2-bit policies of the LDS-staged dequantize GEMM: see
// dq_gemm_i8.h for the matrix instruction and the epilogues.
#include "dq_gemm_i8.h"

namespace dq {

namespace {

using gemm::Params;

// ---- int8 x 4-bit ---------------------------------------------------------------------------------
// DEC = I4_TWOS: nibbles are two's complement; they are decoded as 16 x value (nibble in the top of the
// byte) and the accumulator is shifted back in the epilogue.  A_PACKED: A is packed int4 too and
// is expanded the same way while it is staged, so both operands carry the factor 16.
// DEC = I4U_INTERLEAVED / I4S_INTERLEAVED: the words went through interleave_weight(qB, 4, "int8")
// (examples/dequantize_gemm/quantize/utils.py:71-125: element e of a word at byte e % 4, nibble slot e / 4), and
// decode as decode_i4u_to_i8s (w = q) / decode_i4s_to_i8s (w = q - 7: its MEDIAN_NUM is 0x07070707)
// (examples/dequantize_gemm/quantize/lop3.py:999-1047).  The same mask and shift then yield elements 0..3 and 4..7
// in natural order, so A needs no shuffle.
enum { I4_UNSIGNED = 0, I4_TWOS = 1, I4U_INTERLEAVED = 2, I4S_INTERLEAVED = 3, I2_TO_I4 = 4 };

template <int DEC, bool A_PACKED, class EPI>
struct I4Policy : I8Mfma, gemm::NoScale, EPI {
  static constexpr int kBRowBytes = 64;
  static constexpr bool kAPacked = A_PACKED;
  static constexpr bool kNatural = DEC >= I4U_INTERLEAVED;  // decoded elements come out in k order
  __device__ static __forceinline__ uint32_t minus7(uint32_t x) {
    // bytes 0..15 -> two's-complement bytes of x - 7: with bit 7 set no byte borrows from its neighbour
    return ((x | 0x80808080u) - 0x07070707u) ^ 0x80808080u;
  }
  __device__ static __forceinline__ uint32_t even(uint32_t w) {
    if constexpr (DEC == I4_TWOS) return (w << 4) & 0xF0F0F0F0u;
    else if constexpr (DEC == I4S_INTERLEAVED) return minus7(w & 0x0F0F0F0Fu);
    else return w & 0x0F0F0F0Fu;
  }
  __device__ static __forceinline__ uint32_t odd(uint32_t w) {
    if constexpr (DEC == I4_TWOS) return w & 0xF0F0F0F0u;
    else if constexpr (DEC == I4S_INTERLEAVED) return minus7((w >> 4) & 0x0F0F0F0Fu);
    else return (w >> 4) & 0x0F0F0F0Fu;
  }
  __device__ static __forceinline__ uint4_t stage_a(uint4_t v) { return kNatural ? v : split_even_odd_bytes(v); }
  // direct-to-LDS kernel (int8 A only: a packed A is expanded on its way to LDS): the byte shuffle moves behind
  // the LDS read, fragment by fragment
  static bool dma_ok(const Params&) { return !A_PACKED; }
  __device__ static __forceinline__ Scale prep_scale(int, const Params&) { return {}; }
  using gemm::NoScale::prep_scale;
  __device__ static __forceinline__ frag_t fix_a(frag_t f) {
    return kNatural ? f : __builtin_bit_cast(frag_t, split_even_odd_bytes(__builtin_bit_cast(uint4_t, f)));
  }
  __device__ static __forceinline__ void expand_a(uint4_t v, uint4_t& lo, uint4_t& hi) {
    lo = uint4_t{even(v[0]), odd(v[0]), even(v[1]), odd(v[1])};
    hi = uint4_t{even(v[2]), odd(v[2]), even(v[3]), odd(v[3])};
  }
  __device__ static __forceinline__ frag_t decode(const uint32_t* w, int j, const Scale&) {
    const uint32_t w0 = w[2 * j], w1 = w[2 * j + 1];
    return frag_t{(int)even(w0), (int)odd(w0), (int)even(w1), (int)odd(w1)};
  }
};

// ---- int4 x 2-bit --------------------------------------------------------------------------------
// B holds 2-bit codes, A packed two's-complement int4: the operands of the int4 x int4 matrix instruction that
// decode_i2{s,u}_to_i4s feeds (examples/dequantize_gemm/quantize/lop3.py:1049-1089: i4s[i] = (w >> 2 i) & 0x33333333,
// the code kept unsigned in its nibble; the signed form's adjustment is commented out there, so both decoders are
// w = c).  Here both operands go to int8: (w >> 2 i) & 0x03030303 yields codes (i, 4 + i, 8 + i, 12 + i) of a
// 16-code word as bytes, and A's nibbles are expanded to 16 x value in that same order while they are staged (the
// even / odd nibble bytes of two words regrouped with v_perm_b32); the epilogue shifts the factor 16 out.
template <class EPI>
struct I4xI2Policy : I8Mfma, gemm::NoScale, EPI {
  static constexpr int kBRowBytes = 32;
  static constexpr bool kAPacked = true;
  static bool dma_ok(const Params&) { return false; }  // a packed A is expanded on its way to LDS
  __device__ static __forceinline__ uint4_t stage_a(uint4_t v) { return v; }
  __device__ static __forceinline__ Scale prep_scale(int, const Params&) { return {}; }
  using gemm::NoScale::prep_scale;
  __device__ static __forceinline__ frag_t fix_a(frag_t f) { return f; }
  // 16 nibbles n0..n15 in two words -> dword i = 16 x (n_i, n_{4+i}, n_{8+i}, n_{12+i})
  __device__ static __forceinline__ uint4_t expand16(uint32_t v0, uint32_t v1) {
    const uint32_t e0 = (v0 << 4) & 0xF0F0F0F0u, o0 = v0 & 0xF0F0F0F0u;  // (n0 n2 n4 n6), (n1 n3 n5 n7)
    const uint32_t e1 = (v1 << 4) & 0xF0F0F0F0u, o1 = v1 & 0xF0F0F0F0u;  // (n8 n10 n12 n14), (n9 n11 n13 n15)
    return uint4_t{__builtin_amdgcn_perm(e1, e0, 0x06040200u), __builtin_amdgcn_perm(o1, o0, 0x06040200u),
                   __builtin_amdgcn_perm(e1, e0, 0x07050301u), __builtin_amdgcn_perm(o1, o0, 0x07050301u)};
  }
  __device__ static __forceinline__ void expand_a(uint4_t v, uint4_t& lo, uint4_t& hi) {
    lo = expand16(v[0], v[1]);
    hi = expand16(v[2], v[3]);
  }
  __device__ static __forceinline__ frag_t decode(const uint32_t* w, int j, const Scale&) {
    frag_t o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = (int)((w[j] >> (2 * i)) & 0x03030303u);
    return o;
  }
};

}  // namespace

int i4_gemm(const void* A, const void* B, void* C, int M, int N, int K, int decode, int a_packed, int transposed,
            hipStream_t stream) {
  Params p = gemm::make_params(A, B, nullptr, nullptr, nullptr, C, M, N, K);
  if (decode == I2_TO_I4) {
    if (!a_packed) DQ_FAIL("int4 gemm: 2-bit codes decoded to int4 go with a packed int4 A");
    if (transposed) return gemm::launch_auto<I4xI2Policy<Int32Out<4, true>>>(p, stream);
    return gemm::launch_auto<I4xI2Policy<Int32Out<4, false>>>(p, stream);
  }
  if (a_packed) {
    if (decode != I4_TWOS) DQ_FAIL("int4 gemm: packed A is built for two's-complement int4 only");
    // both operands carry a factor 16: |sum| <= 128 * 128 * K must stay below 2^31
    if (K >= 131072) DQ_FAIL("int4 gemm: K=%d is beyond the 131071 that keep the int32 accumulation of packed operands exact", K);
    if (transposed) return gemm::launch_auto<I4Policy<I4_TWOS, true, Int32Out<8, true>>>(p, stream);
    return gemm::launch_auto<I4Policy<I4_TWOS, true, Int32Out<8, false>>>(p, stream);
  }
#define DQ_I4(DEC_, SHIFT_, TRANS_)                                           \
  do {                                                                        \
    using Pol = I4Policy<DEC_, false, Int32Out<SHIFT_, TRANS_>>;              \
    return gemm::launch_best<Pol>(p, stream);                                 \
  } while (0)
#define DQ_I4T(DEC_, SHIFT_)                  \
  do {                                        \
    if (transposed) DQ_I4(DEC_, SHIFT_, true); \
    DQ_I4(DEC_, SHIFT_, false);               \
  } while (0)
  switch (decode) {
    case I4_UNSIGNED: DQ_I4T(I4_UNSIGNED, 0);
    case I4_TWOS: DQ_I4T(I4_TWOS, 4);
    case I4U_INTERLEAVED: DQ_I4T(I4U_INTERLEAVED, 0);
    case I4S_INTERLEAVED: DQ_I4T(I4S_INTERLEAVED, 0);
    default: DQ_FAIL("int4 gemm: unknown decode %d", decode);
  }
#undef DQ_I4T
#undef DQ_I4
}

}  // namespace dq
