// BitLinear activation quantiser for gfx950: per-row absmax -> int8.
//
// Replaces BitLinearBitBLAS.activation_quant of examples/bitnet-1.58b/utils_quant.py:156-163 (a
// torch.compile'd elementwise + row reduction):
//     s[m]   = (1 / max(max_k |x[m, k]|, 1e-5)) * 127      (fp32; what torch's `Qp / tensor` computes)
//     q[m,k] = clamp(round_half_even(float(x[m, k]) * s[m]), -128, 127)  -> int8
// One workgroup per row; the row stays in registers between the reduction and the quantisation (up to
// K = 16384; longer rows are read twice), all arithmetic in fp32 with the same operations, so q and s are
// bit-identical to the reference's.  HBM traffic: 2 K bytes in, K + 4 bytes out per row.
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

// NV > 0: a row fits NV 16-byte pieces per thread and stays in registers between the two phases; a
// workgroup walks rows blockIdx.x, blockIdx.x + gridDim.x, ... with the next row's loads in flight
// while the current one is reduced and written, so reads and writes overlap across the chip.
// NV == 0: any K, one row per workgroup, read twice (the second pass is served by the caches).
template <int NV>
__global__ __launch_bounds__(256) void activation_quant_kernel(const half_t* __restrict__ X, int8_t* __restrict__ Q,
                                                               float* __restrict__ S, int M, int K) {
  __shared__ float wmax[2][4];
  const int tid = threadIdx.x;
  const int nvec = K >> 3;  // 16-byte pieces of 8 halves
  constexpr int kHeld = NV > 0 ? NV : 1;
  half8_t cur[kHeld], nxt[kHeld];

  auto load_row = [&](half8_t (&h)[kHeld], int row) {
    const half_t* x = X + (size_t)row * K;
#pragma unroll
    for (int i = 0; i < kHeld; ++i) {
      const int v = tid + 256 * i;
      if (v < nvec) h[i] = __builtin_nontemporal_load(reinterpret_cast<const half8_t*>(x + (size_t)v * 8));
      else h[i] = half8_t{0, 0, 0, 0, 0, 0, 0, 0};
    }
  };
  auto quantise = [&](const half8_t& h, int8_t* q, int v, float s) {
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
  };
  auto row_scale = [&](float amax, int parity) {
    amax = wave_max(amax);
    if ((tid & 63) == 0) wmax[parity][tid >> 6] = amax;
    __syncthreads();  // the other parity's slots are rewritten only after the next barrier
    amax = fmaxf(fmaxf(wmax[parity][0], wmax[parity][1]), fmaxf(wmax[parity][2], wmax[parity][3]));
    // Qp / tensor in torch is tensor.reciprocal() * Qp: a correctly rounded reciprocal, then a product
    return (1.0f / fmaxf(amax, 1e-5f)) * 127.f;
  };

  if constexpr (NV > 0) {
    int row = blockIdx.x, it = 0;
    if (row < M) load_row(cur, row);
    for (; row < M; row += gridDim.x, ++it) {
      const int next_row = row + gridDim.x;
      if (next_row < M) load_row(nxt, next_row);
      float amax = 0.f;
#pragma unroll
      for (int i = 0; i < NV; ++i)
#pragma unroll
        for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf((float)cur[i][e]));
      const float s = row_scale(amax, it & 1);
      if (tid == 0) S[row] = s;
      int8_t* q = Q + (size_t)row * K;
#pragma unroll
      for (int i = 0; i < NV; ++i) {
        const int v = tid + 256 * i;
        if (v < nvec) quantise(cur[i], q, v, s);
      }
#pragma unroll
      for (int i = 0; i < NV; ++i) cur[i] = nxt[i];
    }
  } else {
    const int row = blockIdx.x;
    const half_t* x = X + (size_t)row * K;
    float amax = 0.f;
    for (int v = tid; v < nvec; v += 256) {
      const half8_t h = *reinterpret_cast<const half8_t*>(x + (size_t)v * 8);
#pragma unroll
      for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf((float)h[e]));
    }
    const float s = row_scale(amax, 0);
    if (tid == 0) S[row] = s;
    int8_t* q = Q + (size_t)row * K;
    for (int v = tid; v < nvec; v += 256) quantise(*reinterpret_cast<const half8_t*>(x + (size_t)v * 8), q, v, s);
  }
}

}  // namespace

int activation_quant(const void* X, void* Q, void* S, int M, int K, hipStream_t stream) {
  const int per_thread = (K / 8 + 255) / 256;  // 16-byte pieces per thread
  // register-resident rows: at most 2 workgroups per CU in flight, each walking several rows
  const int wgs = M < 512 ? M : 512;
#define DQ_AQ(NV_, GRID_)                                                                                              \
  hipLaunchKernelGGL(activation_quant_kernel<NV_>, dim3(GRID_), dim3(256), 0, stream, (const half_t*)X, (int8_t*)Q, \
                     (float*)S, M, K)
  if (per_thread <= 1) DQ_AQ(1, wgs);
  else if (per_thread <= 2) DQ_AQ(2, wgs);
  else if (per_thread <= 4) DQ_AQ(4, wgs);
  else if (per_thread <= 8) DQ_AQ(8, wgs);
  else DQ_AQ(0, M);
#undef DQ_AQ
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

}  // namespace dq
