// What the matrix pipe of this chip sustains on operands that toggle like real data: a diagnostic, not a GEMM.
//
// Every wave loads four A and four B fragments (the caller's bytes, random for a meaningful figure) once and then
// issues `iters` rounds of the 4 x 4 = 16 matrix instructions of a 128 x 128 wave tile (32x32x16 fp16 / bf16, 32x32x32
// int8, block-scaled 32x32x64 fp4), the instruction mix of the
// dequantize GEMMs' inner loop without any memory, LDS or decode work.  With one workgroup of four waves per CU the
// rate it reaches is the ceiling those kernels can approach on this device at its power limit: the published peak
// assumes the top clock, which random operands do not sustain.
#include "dq_common.h"

#include <type_traits>

namespace dq {

namespace {

enum { DT_F16 = 0, DT_BF16 = 1, DT_I8 = 2, DT_FP4 = 5 };  // DQ_DT_* of the header

template <int DT>
__global__ __launch_bounds__(256) void mfma_rate_kernel(const uint4_t* __restrict__ operands, float* __restrict__ out, int iters) {
  using frag_t = std::conditional_t<DT == DT_I8 || DT == DT_FP4, int4_t, std::conditional_t<DT == DT_BF16, bf16x8_t, half8_t>>;
  using acc_t = std::conditional_t<DT == DT_I8, int16_t_, float16_t>;
  typedef int v8i_t __attribute__((ext_vector_type(8)));
  acc_t acc[16];
#pragma unroll
  for (int i = 0; i < 16; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[i][j] = 0;
  frag_t a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = __builtin_bit_cast(frag_t, operands[(i * 256 + threadIdx.x) & 4095]);
    b[i] = __builtin_bit_cast(frag_t, operands[((i + 4) * 256 + threadIdx.x) & 4095]);
  }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if constexpr (DT == DT_FP4) {
          // e2m1 codes (every nibble is one), both block scales 1.0 (E8M0 byte 127)
          const v8i_t av = {a[i][0], a[i][1], a[i][2], a[i][3], 0, 0, 0, 0}, bv = {b[j][0], b[j][1], b[j][2], b[j][3], 0, 0, 0, 0};
          acc[i * 4 + j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, acc[i * 4 + j], 4, 4, 0, 0x7F7F7F7F, 0, 0x7F7F7F7F);
        } else if constexpr (DT == DT_I8) acc[i * 4 + j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], acc[i * 4 + j], 0, 0, 0);
        else if constexpr (DT == DT_BF16) acc[i * 4 + j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i * 4 + j], 0, 0, 0);
        else acc[i * 4 + j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[j], acc[i * 4 + j], 0, 0, 0);
      }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i)
#pragma unroll
    for (int j = 0; j < 16; ++j) s += (float)acc[i][j];
  out[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
}

}  // namespace

int mfma_rate(const void* operands, void* out, int dtype, int workgroups, int iters, hipStream_t stream) {
  const dim3 grid(workgroups), block(256);
  switch (dtype) {
    case DT_F16: hipLaunchKernelGGL(mfma_rate_kernel<DT_F16>, grid, block, 0, stream, (const uint4_t*)operands, (float*)out, iters); break;
    case DT_BF16: hipLaunchKernelGGL(mfma_rate_kernel<DT_BF16>, grid, block, 0, stream, (const uint4_t*)operands, (float*)out, iters); break;
    case DT_I8: hipLaunchKernelGGL(mfma_rate_kernel<DT_I8>, grid, block, 0, stream, (const uint4_t*)operands, (float*)out, iters); break;
    case DT_FP4: hipLaunchKernelGGL(mfma_rate_kernel<DT_FP4>, grid, block, 0, stream, (const uint4_t*)operands, (float*)out, iters); break;
    default: DQ_FAIL("mfma rate: dtype %d is not fp16, bf16, int8 or fp4", dtype);
  }
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

}  // namespace dq
