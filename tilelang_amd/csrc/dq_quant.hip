// Quantisers that feed the dequantize-GEMM kernels on gfx950: the BitLinear activation quantiser
// (per-row absmax -> int8) and the MXFP4 weight quantiser (bf16 -> e2m1 codes + one shared
// power-of-two scale per 32 elements), further down.
//
// BitLinear activation quantiser.
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


// ---- MXFP4 weight quantiser ---------------------------------------------------------------------
// bf16 W[N, K] -> the operands of the MXFP4 GEMM (examples/dequantize_gemm/
// example_dequant_gemm_bf16_mxfp4_cdna4.py:99-103): e2m1 codes, two per byte along K with the even
// k in the low nibble, and one scale byte per 32 consecutive k.  Per block of 32:
//     e      = max(floor(log2(max |w|)) - 2, -127)         (2 = exponent of e2m1's largest value, 6;
//                                                           an all-zero block gets -127)
//     byte   = clamp(e + scale_bias, 0, 255)
//     code_i = e2m1(w_i / 2^(byte - scale_bias)),  magnitudes rounded at the thresholds 0.25, 0.75,
//              1.25, 1.75, 2.5, 3.5, 5.0 (a value on a threshold goes up), saturating at 6; the sign
//              bit is set only for non-zero magnitudes
// The element rule is encode_fp4_e2m1_values of examples/dequantize_gemm/quantize/nvfp4.py:120-138;
// the block scale is the OCP Microscaling v1.0 conversion (largest power of two that keeps the block
// maximum inside e2m1's range after rounding down the exponent).  The division by a power of two is
// exact, so codes and scale bytes are reproducible bit for bit.
// A lane owns 8 consecutive elements (one 16-byte load, one packed dword out), the four lanes of a
// quad own a block and agree on its maximum with two DPP steps.  HBM traffic: 2 bytes in,
// 1/2 + 1/32 byte out per element.
__device__ __forceinline__ uint32_t quad_max_u32(uint32_t v) {
  v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, true));  // quad_perm(1,0,3,2)
  v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, true));  // quad_perm(2,3,0,1)
  return v;
}

template <int U>
__global__ __launch_bounds__(256) void mxfp4_quant_kernel(const uint4_t* __restrict__ W, uint32_t* __restrict__ B,
                                                          uint8_t* __restrict__ S, size_t pieces, int scale_bias) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t p0 = (size_t)blockIdx.x * 256 + threadIdx.x; p0 < pieces; p0 += stride * U) {
    uint4_t raw[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t p = p0 + u * stride;
      // pieces is a multiple of 4 and p0 keeps the quad aligned: a quad is inside or outside as a whole
      raw[u] = p < pieces ? __builtin_nontemporal_load(W + p) : uint4_t{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const size_t p = p0 + u * stride;
      // non-negative floats order like their bit patterns: the block maximum in integer arithmetic
      uint32_t amax = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) amax = max(amax, max(raw[u][i] & 0x7FFFu, (raw[u][i] >> 16) & 0x7FFFu));
      amax = quad_max_u32(amax);
      const int e = max((int)(amax >> 7) - 129, -127);       // exponent field - 127 - 2
      const int byte = min(max(e + scale_bias, 0), 255);
      const int e_used = min(max(byte - scale_bias, -127), 126);
      // 2^-e_used (a normal float) times 1 + 2^-10: the products below stay exact (8 significant bits times 11),
      // values on a threshold move just above it and nothing else crosses one (neighbouring bf16 values are at
      // least 2^-8 apart, relatively), so the converter's round-to-nearest-even becomes "a threshold goes up"
      const float inv = __builtin_bit_cast(float, (uint32_t)(127 - e_used) << 23) * 1.0009765625f;
      uint32_t packed = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float lo = __builtin_bit_cast(float, raw[u][i] << 16) * inv;          // the bf16 pair as fp32
        const float hi = __builtin_bit_cast(float, raw[u][i] & 0xFFFF0000u) * inv;
        // v_cvt_scalef32_pk_fp4_f32: two e2m1 codes (saturating, round to nearest even) into byte i
        if (i == 0) packed = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(packed, lo, hi, 1.0f, 0);
        if (i == 1) packed = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(packed, lo, hi, 1.0f, 1);
        if (i == 2) packed = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(packed, lo, hi, 1.0f, 2);
        if (i == 3) packed = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(packed, lo, hi, 1.0f, 3);
      }
      // no negative zero: keep a nibble's sign bit only where its magnitude bits are not all clear
      const uint32_t nonzero = ((packed & 0x77777777u) + 0x77777777u) & 0x88888888u;
      packed &= nonzero | 0x77777777u;
      if (p < pieces) {
        __builtin_nontemporal_store(packed, &B[p]);  // written once, read by a later kernel: kept out of the L2
        if ((threadIdx.x & 3) == 0) S[p >> 2] = (uint8_t)byte;
      }
    }
  }
}

}  // namespace

int activation_quant(const void* X, void* Q, void* S, int M, int K, hipStream_t stream) {
  const int per_thread = (K / 8 + 255) / 256;  // 16-byte pieces per thread
  // register-resident rows: up to eight workgroups per CU, each walking rows with a grid stride (M = 2048,
  // K = 8192: 11.0 us with one row per workgroup, 12.9 us with 512 workgroups of four rows, 17.7 us with 256)
  const int wgs = M < 2048 ? M : 2048;
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

int mxfp4_quant(const void* W, void* B, void* S, int N, int K, int scale_bias, hipStream_t stream) {
  const size_t pieces = (size_t)N * K / 8;
  constexpr int kUnroll = 4;
  const size_t per_wg = 256 * kUnroll;
  size_t wgs = (pieces + per_wg - 1) / per_wg;
  if (wgs > 256 * 8) wgs = 256 * 8;  // eight workgroups per CU, each walking the matrix with a grid stride
  hipLaunchKernelGGL(mxfp4_quant_kernel<kUnroll>, dim3((unsigned)wgs), dim3(256), 0, stream, (const uint4_t*)W,
                     (uint32_t*)B, (uint8_t*)S, pieces, scale_bias);
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}


namespace {

// Integer zero points of the "quantized" zeros mode -> the fp16 Zeros[N, groups] the kernels read.  The reference's
// decoder folds the integer into the magic number, (0x6400 | q) + (0xe400 | qz) = q - qz exactly, then multiplies by
// the scale once (examples/dequantize_gemm/quantize/lop3.py:339-354); fp16(qz) is exact for 0 <= qz <= 2048 and so
// is q - fp16(qz), hence the "original" decoder fed with these zeros returns the same bits.
// PACKED = false: one int16 per group (lop3.py:339-341 reads `int16_t zero_r = *((int16_t*)zeros)` and folds it as
// `0xe400 | zero_r`, which is -(1024 + qz) for 0 <= qz <= 1023 only: the range with reference parity; other values
// are taken here as the integers they are).
// PACKED = true: 4-bit zero points, two per byte, group g in bits 4 (g % 2) of byte g / 2 of the row.  This row
// layout is the library's own convention: the reference shows only the extraction `(qzeros >> (group_offset * 4))
// & 0xf` inside its device snippet (lop3.py:381-385) and no host-side tensor shape.
template <bool PACKED>
__global__ __launch_bounds__(256) void unpack_qzeros_kernel(const void* __restrict__ QZ, half_t* __restrict__ Z, int N,
                                                            int groups) {
  const size_t total = (size_t)N * groups;
  const int row_bytes = (groups + 1) / 2;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
    int qz;
    if constexpr (PACKED) {
      const size_t n = i / groups;
      const int g = (int)(i - n * groups);
      qz = (((const uint8_t*)QZ)[n * row_bytes + (g >> 1)] >> (4 * (g & 1))) & 0xF;
    } else {
      qz = ((const int16_t*)QZ)[i];
    }
    Z[i] = (half_t)(float)qz;
  }
}

}  // namespace

int unpack_qzeros(const void* QZ, void* Z, int N, int groups, int packed, hipStream_t stream) {
  const size_t total = (size_t)N * groups;
  const unsigned blocks = (unsigned)((total + 255) / 256 < 4096 ? (total + 255) / 256 : 4096);
  if (packed) hipLaunchKernelGGL(unpack_qzeros_kernel<true>, dim3(blocks), dim3(256), 0, stream, QZ, (half_t*)Z, N, groups);
  else hipLaunchKernelGGL(unpack_qzeros_kernel<false>, dim3(blocks), dim3(256), 0, stream, QZ, (half_t*)Z, N, groups);
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

}  // namespace dq
