// 2-bit codes -> int8 operands of the matrix instruction, and the two epilogues, shared by the int8 x 2-bit kernels
// that keep a whole output tile per wave (decoder decode_i2{u,s}_to_i8s,
// examples/dequantize_gemm/quantize/lop3.py:950-997; epilogue examples/bitnet-1.58b/utils_quant.py:165-170).
#pragma once

#include "dq_common.h"

namespace dq {

template <int CONV>
struct Codes {
  static constexpr int kShift = CONV == I2_UNSIGNED ? 0 : 6;  // the accumulators hold 2^kShift x the sum
};

// One packed dword (16 codes; interleaved words: the codes of elements 4 i .. 4 i + 3 at bit 2 i of bytes 0 .. 3) ->
// dword i of the operand.
template <int CONV>
__device__ __forceinline__ int4_t decode16(uint32_t w) {
  int4_t o;
  if constexpr (CONV == I2_UNSIGNED) {
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = (int)((w >> (2 * i)) & 0x03030303u);
  } else {
    // offset binary: flipping the code's top bit after the mask is one three-input bit operation with it
    constexpr uint32_t flip = CONV == I2_OFFSET ? 0x80808080u : 0u;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = (int)(((w << (6 - 2 * i)) & 0xC0C0C0C0u) ^ flip);
  }
  return o;
}

struct BitnetFinish {
  using out_t = half_t;
  using row_t = float;  // what a thread that finishes sums of one activation row keeps of that row
  const float* s_a;
  float s_w;
  __device__ __forceinline__ row_t row(int m) const { return s_a[m]; }
  __device__ __forceinline__ out_t finish(int acc, row_t sa) const {
    float v = (float)acc;
    v = v / sa;
    v = v / s_w;
    return (half_t)v;
  }
  __device__ __forceinline__ out_t operator()(int acc, int m) const { return finish(acc, s_a[m]); }
};
struct Int32Finish {
  using out_t = int32_t;
  using row_t = int;
  __device__ __forceinline__ row_t row(int) const { return 0; }
  __device__ __forceinline__ out_t finish(int acc, row_t) const { return acc; }
  __device__ __forceinline__ out_t operator()(int acc, int) const { return acc; }
};

}  // namespace dq
