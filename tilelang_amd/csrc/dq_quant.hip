// BitLinear activation quantiser for gfx950: per-row absmax -> int8.
//
// Replaces BitLinearBitBLAS.activation_quant of examples/bitnet-1.58b/utils_quant.py:156-163 (a
// torch.compile'd elementwise + row reduction):
//     s[m]   = (1 / max(max_k |x[m, k]|, 1e-5)) * 127      (fp32; what torch's `Qp / tensor` computes)
//     q[m,k] = clamp(round_half_even(float(x[m, k]) * s[m]), -128, 127)  -> int8
// One workgroup per row; the row is read twice (the second pass is served by the caches: a row is
// 2 K bytes), all arithmetic in fp32 with the same operations, so q and s are bit-identical to the
// reference's.  HBM traffic: 2 K bytes in, K + 4 bytes out per row.
#include "dq_common.h"

namespace dq {

namespace {

__device__ __forceinline__ float wave_max(float v) {
  // butterfly over the 64 lanes with DPP row operations and a cross-row swizzle
  v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true)));
  v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true)));
  v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true)));
  v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true)));
  // all 16 lanes of a row hold the row maximum (values are >= 0, bound_ctrl zero-fill is harmless)
  v = fmaxf(v, __shfl_xor(v, 16));
  v = fmaxf(v, __shfl_xor(v, 32));
  return v;
}

__global__ __launch_bounds__(256) void activation_quant_kernel(const half_t* __restrict__ X, int8_t* __restrict__ Q,
                                                               float* __restrict__ S, int K) {
  __shared__ float wmax[4];
  const int tid = threadIdx.x;
  const half_t* x = X + (size_t)blockIdx.x * K;
  int8_t* q = Q + (size_t)blockIdx.x * K;
  const int nvec = K >> 3;  // 16-byte pieces of 8 halves

  float amax = 0.f;
  for (int v = tid; v < nvec; v += 256) {
    const half8_t h = *reinterpret_cast<const half8_t*>(x + (size_t)v * 8);
#pragma unroll
    for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf((float)h[e]));
  }
  amax = wave_max(amax);
  if ((tid & 63) == 0) wmax[tid >> 6] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(wmax[0], wmax[1]), fmaxf(wmax[2], wmax[3]));
  // Qp / tensor in torch is tensor.reciprocal() * Qp: a correctly rounded reciprocal, then a product
  const float s = (1.0f / fmaxf(amax, 1e-5f)) * 127.f;
  if (tid == 0) S[blockIdx.x] = s;

  for (int v = tid; v < nvec; v += 256) {
    const half8_t h = *reinterpret_cast<const half8_t*>(x + (size_t)v * 8);
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float r = __builtin_rintf((float)h[e] * s);  // round half to even, like torch.round
      r = fminf(fmaxf(r, -128.f), 127.f);
      const uint32_t b = (uint32_t)(int)r & 0xFFu;
      if (e < 4) lo |= b << (8 * e);
      else hi |= b << (8 * (e - 4));
    }
    *reinterpret_cast<uint2_t*>(q + (size_t)v * 8) = uint2_t{lo, hi};
  }
}

}  // namespace

int activation_quant(const void* X, void* Q, void* S, int M, int K, hipStream_t stream) {
  hipLaunchKernelGGL(activation_quant_kernel, dim3(M), dim3(256), 0, stream, (const half_t*)X, (int8_t*)Q, (float*)S, K);
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

}  // namespace dq
