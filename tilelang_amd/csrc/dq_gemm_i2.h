// BitNet W2A8 (int8 x 2-bit) policies of the LDS-staged dequantize GEMM, and the choice of policy and kernel for one
// word layout and one epilogue.  The instantiations are spread over several translation units (dq_gemm_i2_*.hip),
// which compile side by side; dq_gemm_i2.hip holds the entry point that picks among them.
#pragma once

#include "dq_gemm_i8.h"

namespace dq {

// One translation unit each.  Return value as i2_gemm; the fragment-ordered one returns 1 where the direct-to-LDS
// kernel does not take the shape (no other tiled kernel reads that order).
int i2_gemm_rowmajor_bitnet(const gemm::Params& p, int convention, hipStream_t stream);
int i2_gemm_rowmajor_int32(const gemm::Params& p, int convention, hipStream_t stream);
int i2_gemm_interleaved_bitnet(const gemm::Params& p, int convention, hipStream_t stream);
int i2_gemm_interleaved_int32(const gemm::Params& p, int convention, hipStream_t stream);
int i2_gemm_fragments(const gemm::Params& p, int convention, bool interleaved, bool bitnet_epilogue, hipStream_t stream);

namespace {


// ---- int8 x 2-bit ---------------------------------------------------------------------------------
// Plain layout: packed byte j of a row holds codes 4j..4j+3 at bits 0, 2, 4, 6; (w >> 2i) & 0x03030303
// then yields elements (i, 4+i, 8+i, 12+i) of a 16-code word, and A is transposed to match.
// INTERLEAVED: words pre-permuted by interleave_weight(qw, 2, "int8") (examples/bitnet-1.58b/
// kernel_benchmark/tilelang_bitnet_158_int8xint2_decode.py:196-234: element e at byte e % 4, slot
// e / 4), the layout the reference's kernels consume; the same shift-and-mask yields elements
// 4i..4i+3 in natural order and A needs no transform.
// TOP (signed conventions, K < 131072): the codes are shifted to the top two bits of their byte instead, where the
// int8 reading of the byte is 64 sext2(c) (offset binary: c - 2 = sext2(c ^ 2), the flip in the same three-input bit
// operation as the mask): two instructions per dword instead of three, and the epilogue shifts the sum back by 6.
// FRAG: B re-ordered offline by prepack_i2_fragments (whole 16-byte pieces move, so the decode is the same); the
// direct-to-LDS kernel only.
template <int CONV, class EPI, bool INTERLEAVED, bool TOP = false, bool FRAG = false>
struct I2Policy : I8Mfma, gemm::NoScale, EPI {
  static_assert(!TOP || CONV != I2_UNSIGNED, "unsigned codes are masked in place");
  static constexpr int kBRowBytes = 32;
  static constexpr bool kBFragments = FRAG;
  static constexpr bool kAPacked = false;
  __device__ static __forceinline__ uint4_t stage_a(uint4_t v) { return INTERLEAVED ? v : transpose4x4_bytes(v); }
  __device__ static __forceinline__ void expand_a(uint4_t, uint4_t&, uint4_t&) {}
  // direct-to-LDS kernel: A lands in LDS untouched and each 16-byte fragment is transposed after the read
  __device__ static __forceinline__ Scale prep_scale(int, const Params&) { return {}; }
  using gemm::NoScale::prep_scale;
  __device__ static __forceinline__ frag_t fix_a(frag_t f) {
    return INTERLEAVED ? f : __builtin_bit_cast(frag_t, transpose4x4_bytes(__builtin_bit_cast(uint4_t, f)));
  }
  __device__ static __forceinline__ frag_t decode(const uint32_t* w, int j, const Scale&) {
    frag_t o;
    if constexpr (TOP) {
      constexpr uint32_t flip = CONV == I2_OFFSET ? 0x80808080u : 0u;
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = (int)(((w[j] << (6 - 2 * i)) & 0xC0C0C0C0u) ^ flip);
      return o;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      uint32_t d = (w[j] >> (2 * i)) & 0x03030303u;
      // each byte of d is a code 0..3: as the selector of v_perm_b32 it picks the code's int8 value out of a
      // four-byte table (offset binary: c - 2; two's complement: sext2(c)), one instruction per dword
      if constexpr (CONV == I2_OFFSET) d = __builtin_amdgcn_perm(0u, 0x0100FFFEu, d);
      else if constexpr (CONV == I2_TWOS) d = __builtin_amdgcn_perm(0u, 0xFFFE0100u, d);
      o[i] = (int)d;
    }
    return o;
  }
};

// The int8 x 2-bit policy gains from the half-height direct-to-LDS tile from 160 tiles on only.
constexpr int kI2HalfTileMin = 160;

// BITNET: out = (float(acc) / s_a[m]) / s_w -> fp16; else the raw int32.  The signed conventions use the TOP decode
// while 128 x 128 x K stays below 2^31.
template <int CONV, bool INTERLEAVED, bool BITNET, bool FRAG>
int i2_gemm_conv(const Params& p, hipStream_t stream) {
  using Plain = I2Policy<CONV, std::conditional_t<BITNET, BitnetOut, Int32Out<0, false>>, INTERLEAVED, false, FRAG>;
  auto run = [&](auto pol) -> int {
    using Pol = decltype(pol);
    if constexpr (FRAG) {
      if (gemm::dma_eligible<Pol>(p)) return gemm::launch_dma<Pol>(p, stream);
      if (gemm::dma_half_eligible<Pol>(p, kI2HalfTileMin)) return gemm::launch_dma_half<Pol>(p, stream);
      return 1;
    } else {
      return gemm::launch_best<Pol>(p, stream, kI2HalfTileMin);
    }
  };
  if constexpr (CONV != I2_UNSIGNED) {
    using Top = I2Policy<CONV, std::conditional_t<BITNET, BitnetOutS<6>, Int32Out<6, false>>, INTERLEAVED, true, FRAG>;
    if (p.K < 131072) return run(Top{});
  }
  return run(Plain{});
}

template <bool INTERLEAVED, bool BITNET, bool FRAG>
int i2_gemm_part(const Params& p, int convention, hipStream_t stream) {
  switch (convention) {
    case I2_UNSIGNED: return i2_gemm_conv<I2_UNSIGNED, INTERLEAVED, BITNET, FRAG>(p, stream);
    case I2_OFFSET: return i2_gemm_conv<I2_OFFSET, INTERLEAVED, BITNET, FRAG>(p, stream);
    case I2_TWOS: return i2_gemm_conv<I2_TWOS, INTERLEAVED, BITNET, FRAG>(p, stream);
    default: DQ_FAIL("int2 gemm: unknown code convention %d", convention);
  }
}

}  // namespace

}  // namespace dq
