// fp4 (e2m1) codes and E8M0 block scales -> bf16 / fp16 operands, shared by the tiled GEMM policies and the small-batch
// MXFP4 kernel (formats: examples/dequantize_gemm/example_dequant_gemm_bf16_mxfp4_hopper.py:56-110,
// examples/dequantize_gemm/dequantize_utils.py:33-45).
#pragma once

#include "dq_common.h"

namespace dq {

// exponent byte -> fp32 power of two 2^(e + off - 127); only the exponent field matters to the
// conversion instruction.  Clamped to [2^-127, 2^127].
__device__ __forceinline__ float scale_to_f32(int e, int off) {
  int ex = e + off;
  ex = ex < 0 ? 0 : (ex > 254 ? 254 : ex);
  uint32_t bits = (uint32_t)ex << 23;
  bits = bits < 0x00400000u ? 0x00400000u : bits;  // exponent 0 means 2^-127 (a subnormal)
  return __builtin_bit_cast(float, bits);
}

// eight e2m1 nibbles (natural k order) times a power of two -> bf16, exact
__device__ __forceinline__ bf16x8_t cvt_e2m1x8(uint32_t w, float scale) {
  const bf16x2_t p0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 0);
  const bf16x2_t p1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 1);
  const bf16x2_t p2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 2);
  const bf16x2_t p3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 3);
  bf16x8_t o;
  o[0] = p0[0]; o[1] = p0[1]; o[2] = p1[0]; o[3] = p1[1];
  o[4] = p2[0]; o[5] = p2[1]; o[6] = p3[0]; o[7] = p3[1];
  return o;
}

// "twiddled" 16-bit units -> plain e2m1 nibbles (natural order), both units of the dword at once.
// unit = (byte[2j] << 8) | byte[2j+1]; code p of a unit is (s, E1, E0, m) =
// p0 (15, 8, 7, 6), p1 (12, 5, 4, 3), p2 (9, 2, 1, 0), p3 (14, 11, 10, 13)
// (examples/dequantize_gemm/dequantize_utils.py:33-45).
__device__ __forceinline__ uint32_t twiddled_to_plain(uint32_t w) {
  const uint32_t x = __builtin_amdgcn_perm(w, w, 0x02030001u);  // swap the bytes of each half
  const uint32_t c0 = ((x >> 12) & 0x00080008u) | ((x >> 6) & 0x00070007u);
  const uint32_t c1 = ((x >> 9) & 0x00080008u) | ((x >> 3) & 0x00070007u);
  const uint32_t c2 = ((x >> 6) & 0x00080008u) | (x & 0x00070007u);
  const uint32_t c3 = ((x >> 11) & 0x00080008u) | ((x >> 9) & 0x00060006u) | ((x >> 13) & 0x00010001u);
  return c0 | (c1 << 4) | (c2 << 8) | (c3 << 12);
}

// "simple" fp4: 16-bit pattern (s << 15) | ((E + bias) << MB) | (m << (MB - 1)) for every E, two
// nibbles of one byte per dword (natural k order).  `expadd` carries the bias (and the block
// exponent) already shifted into both halves.
template <int MANT_BITS>
__device__ __forceinline__ uint4_t simple_fp4x8(uint32_t w, uint32_t expadd) {
  uint4_t r;
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    const uint32_t lo = (w >> (8 * b)) & 0xFu;
    const uint32_t hi = (w >> (8 * b + 4)) & 0xFu;
    const uint32_t p = lo | (hi << 16);
    r[b] = (((p & 0x00080008u) << 12) | ((p & 0x00070007u) << (MANT_BITS - 1))) + expadd;
  }
  return r;
}

}  // namespace dq
