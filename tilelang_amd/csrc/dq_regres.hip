// W4A16 decode kernel for 2 <= M <= 16 activation rows on gfx950: activations resident in REGISTERS.
//
// Replaces the batched use (up to 16 tokens) of the kernel generated from
// examples/dequantize_gemm/example_dequant_gemv_fp16xint4.py:83-153 with the group scales / zeros
// of examples/dequantize_gemm/quantize/lop3.py:41-81,136-176.  16 activation rows of K = 8192 are
// 256 KiB: too much for the LDS of a CU, but half of its register file.  So a workgroup is 16 waves
// (1024 threads, one workgroup per CU), wave w keeps the activations of its K/16 slice in MFMA
// operand registers for the whole kernel, and only weights, scales and zeros cross the memory
// system, with the access pattern and the occupancy of the M = 1 GEMV:
//
//   * the workgroup walks blocks of 16 weight rows; the 16 waves together read each row of a block
//     contiguously (wave w: K/32 bytes at offset w K/32), lane (g = lane / 16, r = lane % 16)
//     loading 16 bytes = 32 consecutive k of row r per 128-k chunk; a lane's registers are
//     refilled with the next block's weights as soon as they are consumed;
//   * each dword is decoded to the exact fp16 tile values (decode_w4) and is the 16 x 32 operand
//     of one v_mfma_f32_16x16x32_f16 against the resident activation operand (lanes with r >= M
//     hold copies of the last row; their output columns are never stored);
//   * the 16 K-slice partials of a row block are summed through LDS in a fixed order, one barrier
//     per row block (double-buffered): results are bit-identical from run to run.
#include "dq_common.h"

namespace dq {

namespace {

// NC consecutive fp16 values (the scales of a wave's chunks) with one load.
template <int NC>
__device__ __forceinline__ uint2_t load_halves(const half_t* p) {
  if constexpr (NC == 4) return *reinterpret_cast<const uint2_t*>(p);
  else if constexpr (NC == 2) return uint2_t{*reinterpret_cast<const uint32_t*>(p), 0u};
  else return uint2_t{(uint32_t) * reinterpret_cast<const unsigned short*>(p), 0u};
}
__device__ __forceinline__ half_t pick_half(uint2_t v, int c) {
  const half2_t h = as_half2(c < 2 ? v[0] : v[1]);
  return (c & 1) ? h[1] : h[0];
}

// NC: 128-k chunks per wave (K = 2048 NC).  64 NC activation bytes per lane stay in registers.
template <int NC, int MODE, bool APERM>
__global__ __launch_bounds__(1024) void w4a16_regres_kernel(const half_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                             const half_t* __restrict__ S, const half_t* __restrict__ Z,
                                                             half_t* __restrict__ C, int M, int N, int K, int rbn) {
  __shared__ float red[2][16][256];  // [buffer][wave][lane * 4 + i]
  constexpr bool kScale = MODE >= W4_SCALE;
  constexpr bool kZeros = MODE >= W4_ZEROS_ORIGINAL;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int g = lane >> 4;
  const int r = lane & 15;
  const int nrb = (N + 15) >> 4;
  const int rb0 = blockIdx.x * rbn;
  const int nrb_wg = min(rbn, nrb - rb0);  // > 0 by construction of the grid
  const uint32_t row_bytes = (uint32_t)(K >> 1);
  const int groups_per_row = K >> 7;
  const int chunk0 = wave * NC;  // first 128-k chunk (= scale group) of this wave

  uint4_t bq[NC];
  uint2_t sc = {0u, 0u}, zp = {0u, 0u}, sc_next = {0u, 0u}, zp_next = {0u, 0u};  // NC scales / zeros of a row block
  // 32-bit byte offsets of this lane's row of the current / next row block from the (uniform) bases; N is
  // a multiple of 16 here, so every row of a block exists
  uint32_t w_off = (uint32_t)(rb0 * 16 + r) * row_bytes + (uint32_t)chunk0 * 64u + (uint32_t)g * 16u;
  uint32_t s_off = ((uint32_t)(rb0 * 16 + r) * (uint32_t)groups_per_row + (uint32_t)chunk0) * 2u;
  const unsigned char* Sb = reinterpret_cast<const unsigned char*>(S);
  const unsigned char* Zb = reinterpret_cast<const unsigned char*>(Z);
  auto load_chunk = [&](int c) {  // chunk c of the row block that w_off / s_off point at
    bq[c] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(B + w_off + c * 64));
    if (c == 0) {  // the block's scales travel with its first chunk
      if constexpr (kScale) sc_next = load_halves<NC>(reinterpret_cast<const half_t*>(Sb + s_off));
      if constexpr (kZeros) zp_next = load_halves<NC>(reinterpret_cast<const half_t*>(Zb + s_off));
    }
  };
  // the first block's weights go out before the activations are fetched
#pragma unroll
  for (int c = 0; c < NC; ++c) load_chunk(c);
  w_off += 16u * row_bytes;  // from here on they point at the next row block
  s_off += 32u * (uint32_t)groups_per_row;

  // resident activations: y[c][j] is the operand of MFMA step j of chunk c
  uint4_t y[NC][4];
  {
    const half_t* ap = A + (size_t)min(r, M - 1) * K + (size_t)chunk0 * 128 + g * 32;
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint4_t d = *reinterpret_cast<const uint4_t*>(ap + c * 128 + j * 8);
        y[c][j] = APERM ? permute_k8_16bit(d) : d;
      }
  }

  for (int rb = 0; rb < nrb_wg; ++rb) {
    float4_t acc = {0.f, 0.f, 0.f, 0.f};
    sc = sc_next;
    zp = zp_next;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const half_t s = kScale ? pick_half(sc, c) : (half_t)1.f;
      const half_t z = kZeros ? pick_half(zp, c) : (half_t)0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const half8_t x = decode_w4<MODE>(bq[c][j], s, z);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(x, __builtin_bit_cast(half8_t, y[c][j]), acc, 0, 0, 0);
      }
      // this chunk's registers are free: refill them with the next row block (kept behind the
      // arithmetic above and ahead of the next chunk's by the scheduling barriers)
      if (rb + 1 < nrb_wg) {
        __builtin_amdgcn_sched_barrier(0);
        load_chunk(c);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    w_off += 16u * row_bytes;
    s_off += 32u * (uint32_t)groups_per_row;
    // acc[i] = partial C[m = r][(rb0 + rb) * 16 + g * 4 + i] over this wave's K slice
    float* buf = &red[rb & 1][0][0];
    *reinterpret_cast<float4_t*>(buf + wave * 256 + lane * 4) = acc;
    __syncthreads();  // the other buffer is rewritten only after the next barrier
    if (tid < 256) {
      float v = buf[tid];
#pragma unroll
      for (int w = 1; w < 16; ++w) v += buf[w * 256 + tid];
      const int src_lane = tid >> 2, i = tid & 3;
      const int m = src_lane & 15;
      const int n = (rb0 + rb) * 16 + (src_lane >> 4) * 4 + i;
      if (m < M && n < N) C[(size_t)m * N + n] = (half_t)v;
    }
  }
}

template <int NC>
int launch_regres(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int mode,
                  int layout, hipStream_t stream) {
  const int nrb = (N + 15) / 16;
  const int rbn = (nrb + 255) / 256;  // one workgroup per CU, all resident at once
  const dim3 grid((nrb + rbn - 1) / rbn), block(1024);
#define DQ_LAUNCH2(MODE_, APERM_)                                                                                    \
  hipLaunchKernelGGL((w4a16_regres_kernel<NC, MODE_, APERM_>), grid, block, 0, stream, (const half_t*)A,             \
                     (const uint8_t*)B, (const half_t*)S, (const half_t*)Z, (half_t*)C, M, N, K, rbn)
#define DQ_LAUNCH_MODE(MODE_)                              \
  do {                                                     \
    if (layout == LAYOUT_PLAIN) DQ_LAUNCH2(MODE_, true);   \
    else DQ_LAUNCH2(MODE_, false);                         \
  } while (0)
  switch (mode) {
    case W4_UNSIGNED: DQ_LAUNCH_MODE(W4_UNSIGNED); break;
    case W4_SIGNED: DQ_LAUNCH_MODE(W4_SIGNED); break;
    case W4_OFFSET8: DQ_LAUNCH_MODE(W4_OFFSET8); break;
    case W4_SCALE: DQ_LAUNCH_MODE(W4_SCALE); break;
    case W4_USCALE: DQ_LAUNCH_MODE(W4_USCALE); break;
    case W4_ZEROS_ORIGINAL: DQ_LAUNCH_MODE(W4_ZEROS_ORIGINAL); break;
    case W4_ZEROS_RESCALE: DQ_LAUNCH_MODE(W4_ZEROS_RESCALE); break;
    default: DQ_FAIL("w4a16: unknown mode %d", mode);
  }
#undef DQ_LAUNCH_MODE
#undef DQ_LAUNCH2
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

}  // namespace

// Returns 1 when the shape is not covered: needs M <= 16, N a multiple of 16, K = 2048, 4096 or 8192 (whole
// 128-k chunks per wave, activations within the register budget) and group 128 when the mode reads scales
// (one scale per chunk).
int w4a16_regres(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int group,
                 int mode, int layout, hipStream_t stream) {
  if (M < 1 || M > 16 || N < 16 || N % 16 != 0) return 1;
  if (mode >= W4_SCALE && group != 128) return 1;
  if ((size_t)N * K / 2 >= (1ull << 32)) return 1;  // 32-bit lane offsets
  if (K == 8192) return launch_regres<4>(A, B, S, Z, C, M, N, K, mode, layout, stream);
  if (K == 4096) return launch_regres<2>(A, B, S, Z, C, M, N, K, mode, layout, stream);
  if (K == 2048) return launch_regres<1>(A, B, S, Z, C, M, N, K, mode, layout, stream);
  return 1;
}

}  // namespace dq
