// Shared pieces of the int8-MFMA policies of the LDS-staged dequantize GEMM (dq_gemm_core.h): the matrix
// instruction and the epilogues.  Accumulation is int32 and exact; the epilogue is either the raw int32 (optionally
// transposed, optionally shifted back where the operands were decoded as a power of two times their value) or
// BitLinear's out = (float(acc) / s_a[m]) / s_w -> fp16.
#pragma once

#include "dq_gemm_core.h"

namespace dq {

namespace {

using gemm::Params;

struct I8Mfma {
  static constexpr int kKPerBlock = 128;
  using frag_t = int4_t;
  using acc_t = int16_t_;
  __device__ static __forceinline__ acc_t mfma(frag_t a, frag_t b, acc_t c) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
  }
};

// ---- epilogues --------------------------------------------------------------------------------------
template <int SHIFT, bool TRANSPOSED>
struct Int32Out {
  static constexpr bool kTransposed = TRANSPOSED;
  using out_t = int32_t;
  __device__ static __forceinline__ out_t finish(uint32_t raw, const Params&, int, int) {
    return (int32_t)raw >> SHIFT;  // operands were decoded as 16 x value: exact
  }
};

// BitLinear: out = (float(acc) / s_a[m]) / s_w -> fp16, two fp32 divides in that order
// (examples/bitnet-1.58b/utils_quant.py:165-170).  p.S = s_a (float[M]), p.f0 = s_w.
template <int SHIFT>
struct BitnetOutS {
  static constexpr bool kTransposed = false;
  using out_t = half_t;
  __device__ static __forceinline__ out_t finish(uint32_t raw, const Params& p, int m, int) {
    float v = (float)((int32_t)raw >> SHIFT);  // operands decoded as 2^SHIFT x value: exact
    v = v / ((const float*)p.S)[m];
    v = v / p.f0;
    return (half_t)v;
  }
};
using BitnetOut = BitnetOutS<0>;


}  // namespace

}  // namespace dq
