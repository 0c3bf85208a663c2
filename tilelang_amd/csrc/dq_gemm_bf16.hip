// MXFP4-weight x bf16 GEMM for gfx950: C[M,N] bf16 = A[M,K] bf16 . (fp4(B[N,K/2]) * 2^(Scale[N,K/32] - bias))^T (+ Bias).
//
// Replaces the kernel generated from
// examples/dequantize_gemm/example_dequant_gemm_bf16_mxfp4_cdna4.py:61-246 (128x128x128 tiles,
// packed B and dequantised B both staged in LDS, software fp4 decode).  Design here:
//
//   * 256x256x64 block tile, 4 waves (2x2), 128x128 per wave = 4x4 v_mfma_f32_32x32x16_bf16
//     accumulators (256 fp32 per lane), fp32 accumulation;
//   * A and the PACKED B tile are double-buffered in LDS (32 KiB + 8 KiB per stage); the next
//     tile travels global -> registers while the current one is multiplied;
//   * B is never materialised as bf16 in memory: lane (g, c) reads the 16 packed bytes
//     k = g*32 .. g*32+31 of its weight row with one ds_read_b128 and converts each byte pair
//     with v_cvt_scalef32_pk_bf16_fp4, which applies the power-of-two block scale for free
//     (fp4 x 2^e is exact in bf16).  Lane group g owns exactly one 32-k scale block per tile.
//     The contraction index of MFMA step j is labelled k = g*32 + j*8 + e for both operands,
//     so a lane's four dwords are its four B fragments and A fragments are plain 16-byte reads;
//   * A rows are 128 B in LDS; the 16-byte pieces of a row are XOR-swizzled with the row
//     index so the 8 lanes of a ds_read_b128 phase hit 8 different bank groups;
//   * output tiles are assigned to workgroups so that each XCD (workgroup id mod 8) walks a
//     compact block of tiles and re-uses its A / B panels out of its own L2.
#include "dq_common.h"

namespace dq {

namespace {

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int kThreads = 256;
constexpr int kAStage = BM * BK * 2;       // 32 KiB
constexpr int kBStage = BN * BK / 2;       // 8 KiB
constexpr int kStage = kAStage + kBStage;  // 40 KiB
constexpr int kLdsBytes = 2 * kStage;      // 80 KiB

// ---- fp4 -> bf16 fragment decoders: one dword = 8 weights in natural k order ------------------

// exponent byte -> fp32 power of two 2^(e + off - 127); only the exponent field matters to the
// conversion instruction.  Clamped to [2^-127, 2^127].
__device__ __forceinline__ float scale_to_f32(int e, int off) {
  int ex = e + off;
  ex = ex < 0 ? 0 : (ex > 254 ? 254 : ex);
  uint32_t bits = (uint32_t)ex << 23;
  bits = bits < 0x00400000u ? 0x00400000u : bits;  // exponent 0 means 2^-127 (a subnormal)
  return __builtin_bit_cast(float, bits);
}

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
// p0 (15, 8, 7, 6), p1 (12, 5, 4, 3), p2 (9, 2, 1, 0), p3 (14, 11, 10, 13).
__device__ __forceinline__ uint32_t twiddled_to_plain(uint32_t w) {
  const uint32_t x = __builtin_amdgcn_perm(w, w, 0x02030001u);  // swap the bytes of each half
  const uint32_t c0 = ((x >> 12) & 0x00080008u) | ((x >> 6) & 0x00070007u);
  const uint32_t c1 = ((x >> 9) & 0x00080008u) | ((x >> 3) & 0x00070007u);
  const uint32_t c2 = ((x >> 6) & 0x00080008u) | (x & 0x00070007u);
  const uint32_t c3 = ((x >> 11) & 0x00080008u) | ((x >> 9) & 0x00060006u) | ((x >> 13) & 0x00010001u);
  return c0 | (c1 << 4) | (c2 << 8) | (c3 << 12);
}

// "simple" format: bf16 bits (s << 15) | ((E + 126) << 7) | (m << 6) for every E, the block
// exponent added to the exponent field.  expadd = (126 + s) << 7 replicated in both halves.
__device__ __forceinline__ bf16x8_t cvt_simplex8(uint32_t w, uint32_t expadd) {
  uint32_t r[4];
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    const uint32_t lo = (w >> (8 * b)) & 0xFu;
    const uint32_t hi = (w >> (8 * b + 4)) & 0xFu;
    const uint32_t p = lo | (hi << 16);
    r[b] = (((p & 0x00080008u) << 12) | ((p & 0x00070007u) << 6)) + expadd;
  }
  return __builtin_bit_cast(bf16x8_t, uint4_t{r[0], r[1], r[2], r[3]});
}

template <int FMT>
struct ScaleRep {
  float f;       // E2M1 / TWIDDLING: fp32 power of two
  uint32_t add;  // SIMPLE: exponent increment for both halves
};

template <int FMT>
__device__ __forceinline__ ScaleRep<FMT> make_scale(int e, int off) {
  ScaleRep<FMT> s;
  if constexpr (FMT == FP4_SIMPLE) {
    int ex = 126 + e + off - 127;
    ex = ex < 0 ? 0 : (ex > 252 ? 252 : ex);  // E adds up to 3
    s.add = ((uint32_t)ex << 7) * 0x00010001u;
    s.f = 0.f;
  } else {
    s.f = scale_to_f32(e, off);
    s.add = 0;
  }
  return s;
}

template <int FMT>
__device__ __forceinline__ bf16x8_t decode_fp4x8(uint32_t w, const ScaleRep<FMT>& s) {
  if constexpr (FMT == FP4_E2M1) return cvt_e2m1x8(w, s.f);
  else if constexpr (FMT == FP4_TWIDDLING) return cvt_e2m1x8(twiddled_to_plain(w), s.f);
  else return cvt_simplex8(w, s.add);
}

// Workgroup id -> output tile.  With T tiles and 8 XCDs, XCD x (ids x, x+8, ...) gets the
// contiguous range [x*T/8, (x+1)*T/8) of a sequence that walks the tile grid in bands of
// kGroupM tile rows, column by column inside a band.
__device__ __forceinline__ void tile_of_block(int bid, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int T = tiles_m * tiles_n;
  int pid = bid;
  if ((T & 7) == 0) pid = (bid & 7) * (T >> 3) + (bid >> 3);
  constexpr int kGroupM = 4;
  const int band = kGroupM * tiles_n;
  const int first_m = (pid / band) * kGroupM;
  const int gm = min(tiles_m - first_m, kGroupM);
  const int in_band = pid - (pid / band) * band;
  tm = first_m + in_band % gm;
  tn = in_band / gm;
}

template <int FMT, bool HAS_BIAS>
__global__ __launch_bounds__(kThreads, 1) void mxfp4_gemm_kernel(const bf16_t* __restrict__ A,
                                                                  const uint8_t* __restrict__ B,
                                                                  const uint8_t* __restrict__ S,
                                                                  const bf16_t* __restrict__ Bias,
                                                                  bf16_t* __restrict__ C, int M, int N, int K,
                                                                  int scale_off, int tiles_m, int tiles_n) {
  extern __shared__ __align__(16) unsigned char smem[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;  // 2 x 2 waves, 128 x 128 each
  const int g = lane >> 5, r = lane & 31;

  int tm, tn;
  tile_of_block(blockIdx.x, tiles_m, tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  const int KB = K / BK;
  const int scales_per_row = K >> 5;

  // ---- global -> register staging: A 8 x 16 B per thread, packed B 2 x 16 B per thread --------
  // piece q = tid + 256 i.  A: row q / 8, 16-byte piece q % 8.  B: row q / 2, piece q % 2.
  const bf16_t* a_src[8];
  int a_dst[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int q = tid + kThreads * i;
    const int row = q >> 3, piece = q & 7;
    a_src[i] = A + (size_t)min(m0 + row, M - 1) * K + piece * 8;
    a_dst[i] = row * 128 + ((piece ^ (row & 7)) << 4);
  }
  const uint8_t* b_src[2];
  int b_dst[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int q = tid + kThreads * i;
    const int row = q >> 1, piece = q & 1;
    b_src[i] = B + (size_t)min(n0 + row, N - 1) * (K >> 1) + piece * 16;
    b_dst[i] = kAStage + row * 32 + ((piece ^ ((row >> 2) & 1)) << 4);
  }
  // scale byte of lane (g, c) for n-block nb: Scale[n0 + wn*128 + nb*32 + r][kb*2 + g]
  const uint8_t* s_src[4];
#pragma unroll
  for (int nb = 0; nb < 4; ++nb)
    s_src[nb] = S + (size_t)min(n0 + wn * 128 + nb * 32 + r, N - 1) * scales_per_row + g;

  uint4_t a_reg[8], b_reg[2];
  auto load_tile = [&](int kb) {
#pragma unroll
    for (int i = 0; i < 8; ++i) a_reg[i] = *reinterpret_cast<const uint4_t*>(a_src[i] + (size_t)kb * BK);
#pragma unroll
    for (int i = 0; i < 2; ++i) b_reg[i] = *reinterpret_cast<const uint4_t*>(b_src[i] + (size_t)kb * (BK / 2));
  };
  auto store_tile = [&](int stage) {
    unsigned char* base = smem + stage * kStage;
#pragma unroll
    for (int i = 0; i < 8; ++i) *reinterpret_cast<uint4_t*>(base + a_dst[i]) = a_reg[i];
#pragma unroll
    for (int i = 0; i < 2; ++i) *reinterpret_cast<uint4_t*>(base + b_dst[i]) = b_reg[i];
  };

  // ---- fragment read offsets -----------------------------------------------------------------
  // A fragment of m-block mb, step j: row wm*128 + mb*32 + r, logical piece g*4 + j
  int a_row_off[4], a_row_sw[4];
#pragma unroll
  for (int mb = 0; mb < 4; ++mb) {
    const int row = wm * 128 + mb * 32 + r;
    a_row_off[mb] = row * 128;
    a_row_sw[mb] = row & 7;
  }
  // packed B of n-block nb: row wn*128 + nb*32 + r, piece g
  int b_off[4];
#pragma unroll
  for (int nb = 0; nb < 4; ++nb) {
    const int row = wn * 128 + nb * 32 + r;
    b_off[nb] = kAStage + row * 32 + ((g ^ ((row >> 2) & 1)) << 4);
  }

  float16_t acc[4][4];
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mb][nb][i] = 0.f;

  // ---- prologue --------------------------------------------------------------------------------
  load_tile(0);
  int sc_cur[4], sc_next[4];
#pragma unroll
  for (int nb = 0; nb < 4; ++nb) sc_cur[nb] = s_src[nb][0];
  store_tile(0);
  if (KB > 1) load_tile(1);
  __syncthreads();

  for (int kb = 0; kb < KB; ++kb) {
    const int stage = kb & 1;
    const unsigned char* base = smem + stage * kStage;
    if (kb + 1 < KB) {
      store_tile(stage ^ 1);  // tile kb+1 (loaded during the previous iteration) -> other stage
#pragma unroll
      for (int nb = 0; nb < 4; ++nb) sc_next[nb] = s_src[nb][(kb + 1) * 2];
    }
    if (kb + 2 < KB) load_tile(kb + 2);

    uint4_t bw[4];
    ScaleRep<FMT> sc[4];
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
      bw[nb] = *reinterpret_cast<const uint4_t*>(base + b_off[nb]);
      sc[nb] = make_scale<FMT>(sc_cur[nb], scale_off);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      bf16x8_t af[4], bf[4];
#pragma unroll
      for (int mb = 0; mb < 4; ++mb)
        af[mb] = *reinterpret_cast<const bf16x8_t*>(base + a_row_off[mb] + ((((g << 2) + j) ^ a_row_sw[mb]) << 4));
#pragma unroll
      for (int nb = 0; nb < 4; ++nb) bf[nb] = decode_fp4x8<FMT>(bw[nb][j], sc[nb]);
#pragma unroll
      for (int mb = 0; mb < 4; ++mb)
#pragma unroll
        for (int nb = 0; nb < 4; ++nb)
          acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[mb], bf[nb], acc[mb][nb], 0, 0, 0);
    }
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) sc_cur[nb] = sc_next[nb];
    __syncthreads();
  }

  // ---- epilogue: acc[mb][nb][i] = C[m0 + wm*128 + mb*32 + 8*(i/4) + 4*g + i%4][n0 + wn*128 + nb*32 + r]
  // Staged through LDS (every tile is consumed: the loop ended with a barrier) so that a lane
  // stores 16 contiguous bytes.  Each wave owns a 32 x (128 + 4) fp32 slab; LDS operations of
  // one wave execute in order, so no workgroup barrier is needed between the phases.
  constexpr int kSlabStride = 132;
  float* slab = reinterpret_cast<float*>(smem) + wave * (32 * kSlabStride);
#pragma unroll
  for (int mb = 0; mb < 4; ++mb) {
#pragma unroll
    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int row = 8 * (i >> 2) + 4 * g + (i & 3);
        slab[row * kSlabStride + nb * 32 + r] = acc[mb][nb][i];
      }
    __builtin_amdgcn_wave_barrier();
    // 32 rows x 128 columns = 512 pieces of 8 values: 8 per lane
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const int q = lane + 64 * it;
      const int row = q >> 4, piece = q & 15;
      const int m = m0 + wm * 128 + mb * 32 + row;
      const int n = n0 + wn * 128 + piece * 8;
      const float4_t lo = *reinterpret_cast<const float4_t*>(slab + row * kSlabStride + piece * 8);
      const float4_t hi = *reinterpret_cast<const float4_t*>(slab + row * kSlabStride + piece * 8 + 4);
      float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      if (m < M && n < N) {
        const bool full = (n + 7 < N) && ((N & 7) == 0);
        if constexpr (HAS_BIAS) {
          // reference: C = bf16(float(acc) + float(Bias))
          if (full) {
            const bf16x8_t bv = *reinterpret_cast<const bf16x8_t*>(Bias + (size_t)m * N + n);
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] += (float)bv[e];
          } else {
#pragma unroll
            for (int e = 0; e < 8; ++e)
              if (n + e < N) v[e] += (float)Bias[(size_t)m * N + n + e];
          }
        }
        bf16x8_t o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = (bf16_t)v[e];
        if (full) {
          *reinterpret_cast<bf16x8_t*>(C + (size_t)m * N + n) = o;
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (n + e < N) C[(size_t)m * N + n + e] = o[e];
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
}

}  // namespace

int mxfp4_gemm(const void* A, const void* B, const void* S, const void* Bias, void* C, int M, int N, int K, int fmt,
               int scale_bias, hipStream_t stream) {
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const dim3 grid(tiles_m * tiles_n), block(kThreads);
  const int scale_off = 127 - scale_bias;
#define DQ_MX(FMT_, BIAS_)                                                                                          \
  do {                                                                                                              \
    auto kern = mxfp4_gemm_kernel<FMT_, BIAS_>;                                                                     \
    static bool lds_limit_raised = false;                                                                           \
    if (!lds_limit_raised) {                                                                                        \
      DQ_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                                         \
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes));                     \
      lds_limit_raised = true;                                                                                      \
    }                                                                                                               \
    hipLaunchKernelGGL(kern, grid, block, kLdsBytes, stream, (const bf16_t*)A, (const uint8_t*)B, (const uint8_t*)S, \
                       (const bf16_t*)Bias, (bf16_t*)C, M, N, K, scale_off, tiles_m, tiles_n);                      \
  } while (0)
#define DQ_MX_FMT(FMT_)             \
  do {                              \
    if (Bias) DQ_MX(FMT_, true);    \
    else DQ_MX(FMT_, false);        \
  } while (0)
  switch (fmt) {
    case FP4_E2M1: DQ_MX_FMT(FP4_E2M1); break;
    case FP4_SIMPLE: DQ_MX_FMT(FP4_SIMPLE); break;
    case FP4_TWIDDLING: DQ_MX_FMT(FP4_TWIDDLING); break;
    default: DQ_FAIL("mxfp4 gemm: unknown weight format %d", fmt);
  }
#undef DQ_MX_FMT
#undef DQ_MX
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

}  // namespace dq
