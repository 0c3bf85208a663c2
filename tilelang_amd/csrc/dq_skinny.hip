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

// Workgroup = WAVES waves sharing RB row blocks of 16 weight rows; the 128-k chunks of every K
// tile are split evenly between the waves (split-K inside the workgroup), partial 16x16 tiles are
// summed through LDS in a fixed order at the end.  G128: group size 128 (one scale per chunk).
template <int MB, int RB, int WAVES, int U, int MODE, bool APERM, bool G128>
__global__ __launch_bounds__(WAVES * 64) void w4a16_skinny_kernel(const half_t* __restrict__ A,
                                                                   const uint8_t* __restrict__ B,
                                                                   const half_t* __restrict__ S,
                                                                   const half_t* __restrict__ Z,
                                                                   half_t* __restrict__ C, int M, int N, int K,
                                                                   int group, int KT) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  half_t* lds = reinterpret_cast<half_t*>(smem_raw);

  constexpr int THREADS = WAVES * 64;
  constexpr bool kScale = ModeTraits<MODE>::kHasScale;
  constexpr bool kZeros = ModeTraits<MODE>::kHasZeros;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int g = lane >> 4;
  const int r = lane & 15;

  const int m0 = blockIdx.y * (16 * MB);
  const int mrows = min(M - m0, 16 * MB);
  const int n0 = blockIdx.x * (RB * 16);

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
    const int row = min(n0 + rb * 16 + r, N - 1);
    brow[rb] = B + (size_t)row * row_bytes + g * 16;
    srow[rb] = kScale ? S + (size_t)row * groups_per_row : nullptr;
    zrow[rb] = kZeros ? Z + (size_t)row * groups_per_row : nullptr;
  }

  float4_t acc[RB][MB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[rb][mb] = float4_t{0.f, 0.f, 0.f, 0.f};

  int a_row_off[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) a_row_off[mb] = min(mb * 16 + r, mrows - 1) * lds_stride;

  for (int k0 = 0; k0 < K; k0 += KT) {
    const int kt = min(KT, K - k0);
    if (k0 > 0) __syncthreads();  // previous tile fully consumed
    stage_a_tile<THREADS, APERM>(A, lds, mrows, m0, k0, kt, K, lds_stride, tid);
    __syncthreads();

    const int nch = kt / kChunkK;
    const int cpw = (nch + WAVES - 1) / WAVES;
    const int c_begin = wave * cpw;
    const int c_end = min(nch, c_begin + cpw);

    // Two register sets: the loads of batch b+1 are in flight while batch b is decoded and
    // multiplied.  All offsets inside a batch are compile-time constants.
    uint4_t bq0[RB][U], bq1[RB][U];
    half_t sc0[RB][U], sc1[RB][U], zp0[RB][U], zp1[RB][U];
    auto load_set = [&](uint4_t (&bq)[RB][U], half_t (&sc)[RB][U], half_t (&zp)[RB][U], int c) {
      const int nvalid = c_end - c;  // wave-uniform
      const int kk = k0 + c * kChunkK;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) {
        const uint8_t* bp = brow[rb] + (kk >> 1);
        const half_t* sp = nullptr;
        const half_t* zp_ = nullptr;
        if constexpr (G128) {
          if constexpr (kScale) sp = srow[rb] + (kk >> 7);
          if constexpr (kZeros) zp_ = zrow[rb] + (kk >> 7);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          if (u < nvalid) {
            bq[rb][u] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(bp + u * (kChunkK / 2)));
            if constexpr (G128) {
              if constexpr (kScale) sc[rb][u] = sp[u];
              if constexpr (kZeros) zp[rb][u] = zp_[u];
            } else {
              const int gi = (kk + u * kChunkK + g * 32) >> gshift;
              if constexpr (kScale) sc[rb][u] = srow[rb][gi];
              if constexpr (kZeros) zp[rb][u] = zrow[rb][gi];
            }
          }
        }
      }
    };
    auto compute_set = [&](uint4_t (&bq)[RB][U], half_t (&sc)[RB][U], half_t (&zp)[RB][U], int c) {
      const int nvalid = c_end - c;
      const half_t* a_base = lds + c * kChunkK + g * 32;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (u < nvalid) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            // Lanes whose activation row is past M re-read the last valid row: column m of the
            // 32x16 operand only feeds output column m, which is never stored.
            half8_t y[MB];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
              y[mb] = *reinterpret_cast<const half8_t*>(a_base + a_row_off[mb] + u * kChunkK + j * 8);
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
              const half8_t x = decode_w4<MODE>(bq[rb][u][j], kScale ? sc[rb][u] : (half_t)1.f,
                                                kZeros ? zp[rb][u] : (half_t)0.f);
#pragma unroll
              for (int mb = 0; mb < MB; ++mb)
                acc[rb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(x, y[mb], acc[rb][mb], 0, 0, 0);
            }
          }
        }
      }
    };
    if (c_begin < c_end) {
      load_set(bq0, sc0, zp0, c_begin);
      for (int c = c_begin; c < c_end; c += 2 * U) {
        if (c + U < c_end) load_set(bq1, sc1, zp1, c + U);
        compute_set(bq0, sc0, zp0, c);
        if (c + 2 * U < c_end) load_set(bq0, sc0, zp0, c + 2 * U);
        if (c + U < c_end) compute_set(bq1, sc1, zp1, c + U);
      }
    }
  }

  // Cross-wave reduction in a fixed order (deterministic), then the fp16 store.
  // acc[rb][mb][i] = partial C[m0 + mb*16 + r][n0 + rb*16 + g*4 + i]
  float4_t* red = reinterpret_cast<float4_t*>(smem_raw);
  if constexpr (WAVES > 1) {
    __syncthreads();  // every wave is done reading activations from LDS
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) red[((rb * MB + mb) * WAVES + wave) * 64 + lane] = acc[rb][mb];
    __syncthreads();
  }
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      constexpr int kPairs = RB * MB;
      const int pair = rb * MB + mb;
      float4_t v = acc[rb][mb];
      if constexpr (WAVES > 1) {
        // output tile `pair` is finished by wave pair % WAVES
        if ((pair % WAVES) != wave && kPairs > 1) continue;
        if (kPairs == 1 && wave != 0) continue;
        v = red[(pair * WAVES + 0) * 64 + lane];
#pragma unroll
        for (int w = 1; w < WAVES; ++w) v += red[(pair * WAVES + w) * 64 + lane];
      }
      const int m = mb * 16 + r;
      const int n = n0 + rb * 16 + g * 4;
      if (m >= mrows || n >= N) continue;
      half_t* dst = C + (size_t)(m0 + m) * N + n;
      if (((N & 3) == 0) && n + 3 < N) {
        typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
        half4_t o = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
        *reinterpret_cast<half4_t*>(dst) = o;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < N) dst[i] = (half_t)v[i];
      }
    }
  }
}

// Materialise the dequantised fp16 tile W[N, K] with the very same decoder the GEMV uses
// (one thread per 32-bit word).  `plain order` output: element k of row n.
// CVT: the decoder built on the fp8 converter (decode_w4_cvt: the streaming batch kernel and the tiled GEMM use
// it) instead of the mantissa-mask decoder (decode_w4: every other kernel); the two agree bit for bit.
template <int MODE, bool INTERLEAVED, bool CVT>
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
  half_t* dst = W + n * (size_t)K + (size_t)kw * 8;
  if constexpr (CVT) {  // element order for either word layout
    *reinterpret_cast<half8_t*>(dst) = decode_w4_cvt<MODE, INTERLEAVED, true>(w, s, w4_cvt_addend<MODE>(s, z));
    return;
  }
  const half8_t x = decode_w4<MODE>(w, s, z);
  if constexpr (INTERLEAVED) {
    *reinterpret_cast<half8_t*>(dst) = x;
  } else {
    half8_t o;
    o[0] = x[0]; o[4] = x[1]; o[1] = x[2]; o[5] = x[3];
    o[2] = x[4]; o[6] = x[5]; o[3] = x[6]; o[7] = x[7];
    *reinterpret_cast<half8_t*>(dst) = o;
  }
}

template <int MB, int RB, int WAVES, int U>
int launch_skinny(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int group,
                  int mode, int layout, int KT, hipStream_t stream) {
  const dim3 grid((N + RB * 16 - 1) / (RB * 16), (M + 16 * MB - 1) / (16 * MB));
  const dim3 block(WAVES * 64);
  const int mrows = M < 16 * MB ? M : 16 * MB;
  size_t lds_bytes = (size_t)mrows * (KT + 8) * sizeof(half_t);
  const size_t red_bytes = WAVES > 1 ? (size_t)RB * MB * WAVES * 64 * sizeof(float4_t) : 0;
  if (red_bytes > lds_bytes) lds_bytes = red_bytes;
  const bool g128 = group == 128;
#define DQ_LAUNCH2(MODE_, APERM_, G128_)                                                                             \
  do {                                                                                                               \
    auto kern = w4a16_skinny_kernel<MB, RB, WAVES, U, MODE_, APERM_, G128_>;                                         \
    static bool lds_limit_raised[kMaxDevices];                                                                       \
    if (raise_lds_limit<96 * 1024>(kern, lds_limit_raised)) return -1;                                               \
    hipLaunchKernelGGL(kern, grid, block, lds_bytes, stream, (const half_t*)A, (const uint8_t*)B, (const half_t*)S,  \
                       (const half_t*)Z, (half_t*)C, M, N, K, group, KT);                                            \
  } while (0)
#define DQ_LAUNCH(MODE_, APERM_)                  \
  do {                                            \
    if (g128) DQ_LAUNCH2(MODE_, APERM_, true);    \
    else DQ_LAUNCH2(MODE_, APERM_, false);        \
  } while (0)
#define DQ_LAUNCH_MODE(MODE_)                 \
  do {                                        \
    if (layout == LAYOUT_PLAIN) DQ_LAUNCH(MODE_, true); \
    else DQ_LAUNCH(MODE_, false);             \
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
#undef DQ_LAUNCH
#undef DQ_LAUNCH2
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

}  // namespace

// K tile (multiple of 128) for staging `mrows` activation rows in LDS: the fewest equal tiles
// that fit the budget.
static int pick_kt(int mrows, int K, size_t lds_budget) {
  long kt_max = (long)(lds_budget / (mrows * sizeof(half_t))) - 8;
  kt_max = (kt_max / kChunkK) * kChunkK;
  if (kt_max < kChunkK) kt_max = kChunkK;
  if (kt_max >= K) return K;
  const long tiles = (K + kt_max - 1) / kt_max;
  long kt = (K + tiles - 1) / tiles;
  kt = ((kt + kChunkK - 1) / kChunkK) * kChunkK;
  return (int)kt;
}

int w4a16_skinny(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int group,
                 int mode, int layout, int variant, hipStream_t stream) {
  // variant < 0: heuristic.  Otherwise an explicit (benchmarking) choice, see switch below.
  if (variant < 0) {
    if (M <= 4) variant = 0;
    else if (M <= 16) variant = 10;
    else if (M <= 32) variant = 4;
    else variant = 5;
  }
  const size_t budget = 72 * 1024;
  switch (variant) {
#define DQ_V(ID, MB_, RB_, W_, U_)                                                                  \
  case ID:                                                                                                \
    return launch_skinny<MB_, RB_, W_, U_>(A, B, S, Z, C, M, N, K, group, mode, layout,             \
                                                 pick_kt(M < 16 * MB_ ? M : 16 * MB_, K, budget), stream)
    //   id  MB RB  W  U
    DQ_V(0, 1, 1, 4, 8);
    DQ_V(4, 2, 2, 4, 4);
    DQ_V(5, 4, 4, 4, 2);
    DQ_V(10, 1, 4, 4, 2);
#undef DQ_V
    default: DQ_FAIL("w4a16: unknown kernel variant %d", variant);
  }
}

int w4_dequant(const void* B, const void* S, const void* Z, void* W, int N, int K, int group, int mode, int layout,
               hipStream_t stream) {
  const size_t words = (size_t)N * (K >> 3);
  const dim3 block(256), grid((unsigned)((words + 255) / 256));
  const bool converter = (layout & DECODER_CONVERTER) != 0;
  const int word_layout = layout & ~DECODER_CONVERTER;
#define DQ_DQ3(MODE_, IL_, CVT_)                                                                                   \
  hipLaunchKernelGGL((w4_dequant_kernel<MODE_, IL_, CVT_>), grid, block, 0, stream, (const uint8_t*)B,           \
                     (const half_t*)S, (const half_t*)Z, (half_t*)W, N, K, group)
#define DQ_DQ(MODE_)                                                                                               \
  do {                                                                                                             \
    if (word_layout == LAYOUT_PLAIN) {                                                                             \
      if (converter) DQ_DQ3(MODE_, false, true);                                                                   \
      else DQ_DQ3(MODE_, false, false);                                                                            \
    } else {                                                                                                       \
      if (converter) DQ_DQ3(MODE_, true, true);                                                                    \
      else DQ_DQ3(MODE_, true, false);                                                                             \
    }                                                                                                              \
  } while (0)
  switch (mode) {
    case W4_UNSIGNED: DQ_DQ(W4_UNSIGNED); break;
    case W4_SIGNED: DQ_DQ(W4_SIGNED); break;
    case W4_OFFSET8: DQ_DQ(W4_OFFSET8); break;
    case W4_SCALE: DQ_DQ(W4_SCALE); break;
    case W4_USCALE: DQ_DQ(W4_USCALE); break;
    case W4_ZEROS_ORIGINAL: DQ_DQ(W4_ZEROS_ORIGINAL); break;
    case W4_ZEROS_RESCALE: DQ_DQ(W4_ZEROS_RESCALE); break;
    case W4_ZEROS_FOLDED: DQ_DQ(W4_ZEROS_FOLDED); break;
    default: DQ_FAIL("w4 dequant: unknown mode %d", mode);
  }
#undef DQ_DQ
#undef DQ_DQ3
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

}  // namespace dq
