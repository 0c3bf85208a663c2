// W4A16 decode GEMV / small-batch kernel for gfx950 (M up to 64 rows of activations).
//
// Replaces the kernel the reference generates from
// examples/dequantize_gemm/example_dequant_gemv_fp16xint4.py:83-153 (one thread row per
// output, K split over 32 lanes, block all-reduce).  Here the packed weights stream from
// HBM exactly once with 128-bit loads straight into the MFMA operand registers:
//
//   * a wave owns row blocks of 16 weight rows; lane (g = lane/16, r = lane%16) loads
//     16 bytes = 32 consecutive k of row r per 128-k chunk (chunk offset g*32);
//   * each of the 4 dwords is decoded in registers (exact fp16 tile values) and is the
//     16x32 operand of one v_mfma_f32_16x16x32_f16, contraction index labelled
//     k = chunk + g*32 + j*8 + {0,4,1,5,2,6,3,7}[e];
//   * activations are staged once per K tile into LDS in that same element order, so a
//     plain ds_read_b128 yields the matching 32x16 operand; the K reduction happens
//     inside the MFMA in fp32 - no shuffle tree, no atomics, run-to-run deterministic.
#include "dq_common.h"

namespace dq {

namespace {

constexpr int kChunkK = 128;  // k values covered by one 16-byte load per lane across the 4 lane groups

template <int MODE>
struct ModeTraits {
  static constexpr bool kHasScale = MODE >= W4_SCALE;
  static constexpr bool kHasZeros = MODE >= W4_ZEROS_ORIGINAL;
};

// Stage `rows` x `kt` activations starting at (m0, k0) into LDS, optionally permuting every
// aligned group of 8 along k.  LDS row stride is `lds_stride` halves (kt + 8: 16 bytes of
// padding keep the 16 rows of a ds_read_b128 phase on distinct banks).
template <int THREADS, bool APERM>
__device__ __forceinline__ void stage_a_tile(const half_t* __restrict__ A, half_t* lds, int rows, int m0, int k0, int kt,
                                             int K, int lds_stride, int tid) {
  const int vec_per_row = kt >> 3;
  const int total = rows * vec_per_row;
  for (int v = tid; v < total; v += THREADS) {
    const int row = v / vec_per_row;
    const int kv = v - row * vec_per_row;
    uint4_t d = *reinterpret_cast<const uint4_t*>(A + (size_t)(m0 + row) * K + k0 + kv * 8);
    if constexpr (APERM) d = permute_k8_16bit(d);
    *reinterpret_cast<uint4_t*>(lds + row * lds_stride + kv * 8) = d;
  }
}

template <int MB, int RB, int WAVES, int U, int MODE, bool APERM>
__global__ __launch_bounds__(WAVES * 64) void w4a16_skinny_kernel(const half_t* __restrict__ A,
                                                                   const uint8_t* __restrict__ B,
                                                                   const half_t* __restrict__ S,
                                                                   const half_t* __restrict__ Z,
                                                                   half_t* __restrict__ C, int M, int N, int K,
                                                                   int group, int KT) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  half_t* lds = reinterpret_cast<half_t*>(smem_raw);

  constexpr int THREADS = WAVES * 64;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int g = lane >> 4;
  const int r = lane & 15;

  const int m0 = blockIdx.y * (16 * MB);
  const int mrows = min(M - m0, 16 * MB);
  const int n_wg0 = blockIdx.x * (WAVES * RB * 16);
  const int n_wave0 = n_wg0 + wave * (RB * 16);

  const int lds_stride = KT + 8;
  const int groups_per_row = K / group;
  // group is a power of two, or equals K (one group per row: every index shifts to 0)
  const int gshift = (group == K) ? 31 : (31 - __builtin_clz(group));
  const size_t row_bytes = (size_t)(K >> 1);

  // Row pointers; rows past N are clamped to a valid row and masked at the store.
  const uint8_t* brow[RB];
  const half_t* srow[RB];
  const half_t* zrow[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    const int row = min(n_wave0 + rb * 16 + r, N - 1);
    brow[rb] = B + (size_t)row * row_bytes + g * 16;
    srow[rb] = ModeTraits<MODE>::kHasScale ? S + (size_t)row * groups_per_row : nullptr;
    zrow[rb] = ModeTraits<MODE>::kHasZeros ? Z + (size_t)row * groups_per_row : nullptr;
  }

  float4_t acc[RB][MB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[rb][mb] = float4_t{0.f, 0.f, 0.f, 0.f};

  const bool wave_active = n_wave0 < N;  // wave-uniform
  int a_row_off[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) a_row_off[mb] = min(mb * 16 + r, mrows - 1) * lds_stride;

  for (int k0 = 0; k0 < K; k0 += KT) {
    const int kt = min(KT, K - k0);
    if (k0 > 0) __syncthreads();  // previous tile fully consumed
    stage_a_tile<THREADS, APERM>(A, lds, mrows, m0, k0, kt, K, lds_stride, tid);
    __syncthreads();

    if (wave_active) {
      const int nch = kt / kChunkK;
      // Two register sets: the loads of batch b+1 are in flight while batch b is decoded
      // and multiplied.
      uint4_t bq0[RB][U], bq1[RB][U];
      half_t sc0[RB][U], sc1[RB][U], zp0[RB][U], zp1[RB][U];
      auto load_set = [&](uint4_t (&bq)[RB][U], half_t (&sc)[RB][U], half_t (&zp)[RB][U], int c) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int cc = min(c + u, nch - 1);  // clamped: stays in bounds, unused past nch
          const int kk = k0 + cc * kChunkK;
          const int gi = (kk + g * 32) >> gshift;
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) {
            bq[rb][u] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(brow[rb] + (kk >> 1)));
            if constexpr (ModeTraits<MODE>::kHasScale) sc[rb][u] = srow[rb][gi];
            else sc[rb][u] = (half_t)1.f;
            if constexpr (ModeTraits<MODE>::kHasZeros) zp[rb][u] = zrow[rb][gi];
            else zp[rb][u] = (half_t)0.f;
          }
        }
      };
      auto compute_set = [&](uint4_t (&bq)[RB][U], half_t (&sc)[RB][U], half_t (&zp)[RB][U], int c) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (c + u < nch) {  // wave-uniform
            const half_t* a_chunk = lds + (c + u) * kChunkK + g * 32;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              // Lanes whose activation row is past M re-read the last valid row: column m of
              // the 32x16 operand only feeds output column m, which is never stored.
              half8_t y[MB];
#pragma unroll
              for (int mb = 0; mb < MB; ++mb)
                y[mb] = *reinterpret_cast<const half8_t*>(a_chunk + a_row_off[mb] + j * 8);
#pragma unroll
              for (int rb = 0; rb < RB; ++rb) {
                const half8_t x = decode_w4<MODE>(bq[rb][u][j], sc[rb][u], zp[rb][u]);
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
                  acc[rb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(x, y[mb], acc[rb][mb], 0, 0, 0);
              }
            }
          }
        }
      };
      load_set(bq0, sc0, zp0, 0);
      for (int c = 0; c < nch; c += 2 * U) {
        if (c + U < nch) load_set(bq1, sc1, zp1, c + U);
        compute_set(bq0, sc0, zp0, c);
        if (c + 2 * U < nch) load_set(bq0, sc0, zp0, c + 2 * U);
        if (c + U < nch) compute_set(bq1, sc1, zp1, c + U);
      }
    }
  }

  if (!wave_active) return;
  // acc[rb][mb][i] = C[m0 + mb*16 + r][n_wave0 + rb*16 + g*4 + i]
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int m = mb * 16 + r;
      if (m >= mrows) continue;
      const int n = n_wave0 + rb * 16 + g * 4;
      half_t* dst = C + (size_t)(m0 + m) * N + n;
      if (((N & 3) == 0) && n + 3 < N) {
        typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
        half4_t o = {(half_t)acc[rb][mb][0], (half_t)acc[rb][mb][1], (half_t)acc[rb][mb][2], (half_t)acc[rb][mb][3]};
        *reinterpret_cast<half4_t*>(dst) = o;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < N) dst[i] = (half_t)acc[rb][mb][i];
      }
    }
  }
}

// Materialise the dequantised fp16 tile W[N, K] with the very same decoder the GEMV uses
// (one thread per 32-bit word).  `plain order` output: element k of row n.
template <int MODE, bool INTERLEAVED>
__global__ void w4_dequant_kernel(const uint8_t* __restrict__ B, const half_t* __restrict__ S,
                                  const half_t* __restrict__ Z, half_t* __restrict__ W, int N, int K, int group) {
  const size_t words_per_row = (size_t)K >> 3;
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (size_t)N * words_per_row) return;
  const size_t n = idx / words_per_row;
  const int kw = (int)(idx - n * words_per_row);
  const uint32_t w = reinterpret_cast<const uint32_t*>(B)[idx];
  const int gi = (kw * 8) / group;
  const int groups_per_row = K / group;
  half_t s = (half_t)1.f, z = (half_t)0.f;
  if constexpr (ModeTraits<MODE>::kHasScale) s = S[n * groups_per_row + gi];
  if constexpr (ModeTraits<MODE>::kHasZeros) z = Z[n * groups_per_row + gi];
  const half8_t x = decode_w4<MODE>(w, s, z);
  half_t* dst = W + n * (size_t)K + (size_t)kw * 8;
  if constexpr (INTERLEAVED) {
    *reinterpret_cast<half8_t*>(dst) = x;
  } else {
    half8_t o;
    o[0] = x[0]; o[4] = x[1]; o[1] = x[2]; o[5] = x[3];
    o[2] = x[4]; o[6] = x[5]; o[3] = x[6]; o[7] = x[7];
    *reinterpret_cast<half8_t*>(dst) = o;
  }
}

struct SkinnyPlan {
  int mb, rb, waves, u, kt;
  size_t lds_bytes;
};

template <int MB, int RB, int WAVES, int U, bool ALL_MODES>
int launch_skinny(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int group,
                  int mode, int layout, int KT, hipStream_t stream) {
  const dim3 grid((N + WAVES * RB * 16 - 1) / (WAVES * RB * 16), (M + 16 * MB - 1) / (16 * MB));
  const dim3 block(WAVES * 64);
  const int mrows = M < 16 * MB ? M : 16 * MB;
  const size_t lds_bytes = (size_t)mrows * (KT + 8) * sizeof(half_t);
#define DQ_LAUNCH(MODE_, APERM_)                                                                                     \
  do {                                                                                                               \
    auto kern = w4a16_skinny_kernel<MB, RB, WAVES, U, MODE_, APERM_>;                                                \
    if (lds_bytes > 48 * 1024)                                                                                       \
      DQ_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                                          \
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));                 \
    hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, (const half_t*)A, (const uint8_t*)B, (const half_t*)S,  \
                       (const half_t*)Z, (half_t*)C, M, N, K, group, KT);                                            \
  } while (0)
#define DQ_LAUNCH_MODE(MODE_)                 \
  do {                                        \
    if (layout == LAYOUT_PLAIN) DQ_LAUNCH(MODE_, true); \
    else DQ_LAUNCH(MODE_, false);             \
  } while (0)
  if constexpr (ALL_MODES) {
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
  } else {
    // tuning variants: the two modes of the measured configurations, plain layout only
    if (layout != LAYOUT_PLAIN) DQ_FAIL("w4a16: kernel variant supports the plain layout only");
    switch (mode) {
      case W4_SCALE: DQ_LAUNCH(W4_SCALE, true); break;
      case W4_ZEROS_ORIGINAL: DQ_LAUNCH(W4_ZEROS_ORIGINAL, true); break;
      default: DQ_FAIL("w4a16: kernel variant supports modes SCALE and ZEROS_ORIGINAL only (got %d)", mode);
    }
  }
#undef DQ_LAUNCH_MODE
#undef DQ_LAUNCH
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

}  // namespace

// Largest K tile (multiple of 128) whose staged activations fit the LDS budget.
static int pick_kt(int mrows, int K, size_t lds_budget) {
  long kt = (long)(lds_budget / (mrows * sizeof(half_t))) - 8;
  kt = (kt / kChunkK) * kChunkK;
  if (kt > K) kt = K;
  if (kt < kChunkK) kt = kChunkK;
  return (int)kt;
}

int w4a16_skinny(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int group,
                 int mode, int layout, int variant, hipStream_t stream) {
  // variant < 0: heuristic.  Otherwise an explicit (benchmarking) choice, see switch below.
  if (variant < 0) {
    if (M <= 16) variant = (N >= 8192) ? 0 : 1;
    else if (M <= 32) variant = 4;
    else variant = 5;
  }
  const size_t budget = 64 * 1024;
  switch (variant) {
    case 0: return launch_skinny<1, 1, 4, 8, true>(A, B, S, Z, C, M, N, K, group, mode, layout, pick_kt(M < 16 ? M : 16, K, budget), stream);
    case 1: return launch_skinny<1, 1, 1, 8, true>(A, B, S, Z, C, M, N, K, group, mode, layout, pick_kt(M < 16 ? M : 16, K, budget), stream);
    case 2: return launch_skinny<1, 1, 2, 8, false>(A, B, S, Z, C, M, N, K, group, mode, layout, pick_kt(M < 16 ? M : 16, K, budget), stream);
    case 3: return launch_skinny<1, 2, 4, 4, false>(A, B, S, Z, C, M, N, K, group, mode, layout, pick_kt(M < 16 ? M : 16, K, budget), stream);
    case 4: return launch_skinny<2, 2, 4, 4, true>(A, B, S, Z, C, M, N, K, group, mode, layout, pick_kt(M < 32 ? M : 32, K, budget), stream);
    case 5: return launch_skinny<4, 4, 4, 2, true>(A, B, S, Z, C, M, N, K, group, mode, layout, pick_kt(M < 64 ? M : 64, K, budget), stream);
    case 6: return launch_skinny<1, 1, 4, 4, false>(A, B, S, Z, C, M, N, K, group, mode, layout, pick_kt(M < 16 ? M : 16, K, budget), stream);
    case 7: return launch_skinny<1, 1, 8, 8, false>(A, B, S, Z, C, M, N, K, group, mode, layout, pick_kt(M < 16 ? M : 16, K, budget), stream);
    default: DQ_FAIL("w4a16: unknown kernel variant %d", variant);
  }
}

int w4_dequant(const void* B, const void* S, const void* Z, void* W, int N, int K, int group, int mode, int layout,
               hipStream_t stream) {
  const size_t words = (size_t)N * (K >> 3);
  const dim3 block(256), grid((unsigned)((words + 255) / 256));
#define DQ_DQ(MODE_)                                                                                               \
  do {                                                                                                             \
    if (layout == LAYOUT_PLAIN)                                                                                    \
      hipLaunchKernelGGL((w4_dequant_kernel<MODE_, false>), grid, block, 0, stream, (const uint8_t*)B,            \
                         (const half_t*)S, (const half_t*)Z, (half_t*)W, N, K, group);                             \
    else                                                                                                           \
      hipLaunchKernelGGL((w4_dequant_kernel<MODE_, true>), grid, block, 0, stream, (const uint8_t*)B,             \
                         (const half_t*)S, (const half_t*)Z, (half_t*)W, N, K, group);                             \
  } while (0)
  switch (mode) {
    case W4_UNSIGNED: DQ_DQ(W4_UNSIGNED); break;
    case W4_SIGNED: DQ_DQ(W4_SIGNED); break;
    case W4_OFFSET8: DQ_DQ(W4_OFFSET8); break;
    case W4_SCALE: DQ_DQ(W4_SCALE); break;
    case W4_USCALE: DQ_DQ(W4_USCALE); break;
    case W4_ZEROS_ORIGINAL: DQ_DQ(W4_ZEROS_ORIGINAL); break;
    case W4_ZEROS_RESCALE: DQ_DQ(W4_ZEROS_RESCALE); break;
    default: DQ_FAIL("w4 dequant: unknown mode %d", mode);
  }
#undef DQ_DQ
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

}  // namespace dq
