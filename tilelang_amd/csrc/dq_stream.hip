// W4A16 small-batch kernel for gfx950 (4 <= M <= 64 activation rows), direct-to-LDS streaming.
//
// Replaces the batched use of the kernel generated from
// examples/dequantize_gemm/example_dequant_gemv_fp16xint4.py:83-153 (group scales / zeros as in
// examples/dequantize_gemm/quantize/lop3.py:41-81,136-176).  The path is HBM-bound, so the
// kernel is built around keeping many bytes in flight with the access pattern the memory system
// likes, at no register cost:
//
//   * a workgroup owns 64 or 128 weight rows (4 waves x 1 or 2 blocks of 16 rows) and walks K in
//     steps of 256; the packed weights (rows x 128 B), the activations (16 MB rows x 512 B) and the
//     group scales / zeros of a step (4 B per row) travel global -> LDS with
//     global_load_lds_dwordx4 / _dword into a ring of NST stages, NST - 1 steps ahead of the
//     arithmetic; every weight DMA instruction reads 8 rows x 128 contiguous bytes;
//   * a lane's bytes land at LDS base + lane * 16 whatever its source address, so the
//     bank-conflict swizzles are applied by permuting the SOURCE addresses: 16-byte piece p of
//     weight row n sits at position p ^ ((n >> 1) & 7), piece p of activation row m at
//     (p & 16) | ((p ^ m) & 15);
//   * lane (g = lane / 16, r = lane % 16) of a wave reads one 16-byte piece of weight row r per
//     128-k chunk; each of its four dwords is decoded in registers (exact fp16 tile values,
//     decode_w4) and is the 16 x 32 operand of one v_mfma_f32_16x16x32_f16, contraction index
//     labelled k = chunk + g * 32 + j * 8 + {0,4,1,5,2,6,3,7}[e]; the matching activation
//     operand is one ds_read_b128 plus, for the plain layout, four v_perm_b32;
//   * all vector-memory loads of the loop are these DMA instructions, issued from inline assembly
//     and tracked by hand with s_waitcnt vmcnt; one workgroup barrier per step.
//
// K is not split: every wave owns its output tile, results are bit-identical from run to run.
#include "dq_common.h"

namespace dq {

namespace {

__device__ __forceinline__ void dma16(unsigned lds_addr, unsigned voff, const void* sbase) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\t" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
}
__device__ __forceinline__ void dma4(unsigned lds_addr, unsigned voff, const void* sbase) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2\n\t" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
}

constexpr int kStepK = 256;

// RBW blocks of 16 weight rows per wave: a workgroup owns 64 RBW rows.
template <int MB, int RBW>
struct StreamGeom {
  static constexpr int kRowsPerWg = 64 * RBW;
  static constexpr int kWBytes = kRowsPerWg * (kStepK / 2);  // packed weights of a stage
  static constexpr int kABytes = MB * 16 * (kStepK * 2);     // activations of a stage
  static constexpr int kSOff = kWBytes + kABytes;            // scales: 128 rows x 4 B, then zeros
  static constexpr int kStage = kSOff + 1024;
};

template <int MB, int RBW, int NST, int MODE, bool APERM>
__global__ __launch_bounds__(256) void w4a16_stream_kernel(const half_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                            const half_t* __restrict__ S, const half_t* __restrict__ Z,
                                                            half_t* __restrict__ C, int M, int N, int K) {
  extern __shared__ __align__(16) unsigned char smem[];
  using G = StreamGeom<MB, RBW>;
  constexpr int kRowsPerWg = G::kRowsPerWg;
  constexpr int kWBytes = G::kWBytes;
  constexpr int kWOps = 2 * RBW;                        // weight DMA instructions per wave per stage
  constexpr bool kScale = MODE >= W4_SCALE;
  constexpr bool kZeros = MODE >= W4_ZEROS_ORIGINAL;
  constexpr int kAOps = 2 * MB;                         // activation DMA instructions per wave per stage
  constexpr int kOps = kWOps + kAOps + (kScale ? 1 : 0);    // DMA instructions per wave per stage
  constexpr int kWaitOps = (NST - 2) * kOps;            // younger instructions when the next stage must have landed
  static_assert(kWaitOps <= 63, "vmcnt is a 6-bit counter");

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 4;
  const int r = lane & 15;
  const int n0 = blockIdx.x * kRowsPerWg;
  const int m0 = blockIdx.y * (16 * MB);
  const int mrows = min(M - m0, 16 * MB);
  const int KS = K / kStepK;
  const int groups_per_row = K >> 7;
  const unsigned lds0 = (unsigned)(size_t)smem;

  // ---- per-lane source offsets of the DMA instructions ------------------------------------------
  unsigned w_voff[kWOps], a_voff[kAOps];
#pragma unroll
  for (int i = 0; i < kWOps; ++i) {
    const int c = (wave * kWOps + i) * 64 + lane;  // LDS piece: row c / 8, position c % 8
    const int row = c >> 3, pos = c & 7;
    w_voff[i] = (unsigned)min(n0 + row, N - 1) * (unsigned)(K >> 1) + (unsigned)((pos ^ ((row >> 1) & 7)) << 4);
  }
#pragma unroll
  for (int i = 0; i < kAOps; ++i) {
    const int c = (wave * kAOps + i) * 64 + lane;  // LDS piece: row c / 32, position c % 32
    const int row = c >> 5, pos = c & 31;
    a_voff[i] = (unsigned)(m0 + min(row, mrows - 1)) * (unsigned)(K * 2) + (unsigned)((pos ^ (row & 15)) << 4);
  }
  // waves 0, 1: scales of rows 0..63 / 64..127 from the workgroup's first row; waves 2, 3: zeros (or,
  // without zeros, the scales again).  Every wave issues the same number of DMA instructions; with 64
  // rows per workgroup the second half is simply not read.
  const unsigned s_voff = (unsigned)min(n0 + (wave & 1) * 64 + lane, N - 1) * (unsigned)(groups_per_row * 2);
  const unsigned char* s_src = reinterpret_cast<const unsigned char*>((wave >= 2 && kZeros) ? Z : S);

  auto issue_stage = [&](int step, int slot) {
    const unsigned sb = lds0 + slot * G::kStage;
#pragma unroll
    for (int i = 0; i < kWOps; ++i) dma16(sb + (wave * kWOps + i) * 1024, w_voff[i], B + (size_t)step * (kStepK / 2));
#pragma unroll
    for (int i = 0; i < kAOps; ++i)
      dma16(sb + kWBytes + (wave * kAOps + i) * 1024, a_voff[i],
            reinterpret_cast<const unsigned char*>(A) + (size_t)step * (kStepK * 2));
    if constexpr (kScale) dma4(sb + G::kSOff + wave * 256, s_voff, s_src + (size_t)step * 4);
  };

  // ---- fragment read offsets inside a stage -----------------------------------------------------
  int w_off[RBW][2], sc_off[RBW], y_off[2][4];
#pragma unroll
  for (int rb = 0; rb < RBW; ++rb) {
    const int row = wave * (16 * RBW) + rb * 16 + r;
    sc_off[rb] = G::kSOff + row * 4;
#pragma unroll
    for (int u = 0; u < 2; ++u) w_off[rb][u] = row * 128 + ((((u << 2) + g) ^ ((row >> 1) & 7)) << 4);
  }
#pragma unroll
  for (int u = 0; u < 2; ++u)
#pragma unroll
    for (int j = 0; j < 4; ++j) y_off[u][j] = kWBytes + r * 512 + (u << 8) + ((((g << 2) + j) ^ r) << 4);

  float4_t acc[RBW][MB];
#pragma unroll
  for (int rb = 0; rb < RBW; ++rb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[rb][mb] = float4_t{0.f, 0.f, 0.f, 0.f};

  // All LDS operands of a step are fetched up front (registers are plentiful, waves per SIMD are
  // not): the reads of chunk 1 and of the later activation pieces return while chunk 0 is decoded.
  auto compute = [&](const unsigned char* sb) {
    uint4_t w[2][RBW], yraw[2][4][MB];
    half_t sc[2][RBW], zp[2][RBW];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
#pragma unroll
      for (int rb = 0; rb < RBW; ++rb) {
        w[u][rb] = *reinterpret_cast<const uint4_t*>(sb + w_off[rb][u]);
        sc[u][rb] = kScale ? *reinterpret_cast<const half_t*>(sb + sc_off[rb] + u * 2) : (half_t)1.f;
        zp[u][rb] = kZeros ? *reinterpret_cast<const half_t*>(sb + sc_off[rb] + 512 + u * 2) : (half_t)0.f;
      }
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          yraw[u][j][mb] = *reinterpret_cast<const uint4_t*>(sb + y_off[u][j] + mb * (16 * 512));
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < 2; ++u) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        half8_t y[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          y[mb] = __builtin_bit_cast(half8_t, APERM ? permute_k8_16bit(yraw[u][j][mb]) : yraw[u][j][mb]);
#pragma unroll
        for (int rb = 0; rb < RBW; ++rb) {
          const half8_t x = decode_w4<MODE>(w[u][rb][j], sc[u][rb], zp[u][rb]);
#pragma unroll
          for (int mb = 0; mb < MB; ++mb)
            acc[rb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(x, y[mb], acc[rb][mb], 0, 0, 0);
        }
      }
    }
  };

  // ---- prologue: stages 0 .. NST-2 in flight, stage 0 landed --------------------------------------
#pragma unroll
  for (int s = 0; s < NST - 1; ++s)
    if (s < KS) issue_stage(s, s);
  if (KS >= NST - 1) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kWaitOps) : "memory");
  else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  // Step `step` multiplies out of slot step % NST.  The slot of step - 1 was released by the barrier
  // that ended that step, so the DMA of step + NST - 1 goes there first thing.  At the end of the
  // step the stages younger than step + 1 are the NST - 2 issued last (kWaitOps instructions); in the
  // tail, where nothing is issued any more, the wave simply drains its counter.
  int slot = 0;
  for (int step = 0; step < KS; ++step) {
    const int nxt = step + NST - 1;
    if (nxt < KS) issue_stage(nxt, slot == 0 ? NST - 1 : slot - 1);
    compute(smem + slot * G::kStage);
    if (nxt < KS) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kWaitOps) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    slot = slot + 1 == NST ? 0 : slot + 1;
  }

  // acc[rb][mb][i] = C[m0 + mb*16 + r][n0 + wave*16*RBW + rb*16 + g*4 + i]
#pragma unroll
  for (int rb = 0; rb < RBW; ++rb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int m = mb * 16 + r;
      const int n = n0 + wave * (16 * RBW) + rb * 16 + g * 4;
      if (m >= mrows || n >= N) continue;
      const float4_t v = acc[rb][mb];
      half_t* dst = C + (size_t)(m0 + m) * N + n;
      if (((N & 3) == 0) && n + 3 < N) {
        typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
        const half4_t o = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
        *reinterpret_cast<half4_t*>(dst) = o;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < N) dst[i] = (half_t)v[i];
      }
    }
}

template <int MB, int RBW, int NST>
int launch_stream(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int mode,
                  int layout, hipStream_t stream) {
  constexpr int kLds = NST * StreamGeom<MB, RBW>::kStage;
  constexpr int kRowsPerWg = StreamGeom<MB, RBW>::kRowsPerWg;
  static_assert(kLds <= 160 * 1024, "LDS budget");
  const dim3 grid((N + kRowsPerWg - 1) / kRowsPerWg, (M + 16 * MB - 1) / (16 * MB));
  const dim3 block(256);
#define DQ_LAUNCH2(MODE_, APERM_)                                                                                    \
  do {                                                                                                               \
    auto kern = w4a16_stream_kernel<MB, RBW, NST, MODE_, APERM_>;                                                         \
    static bool lds_limit_raised = false; /* once per kernel: legal under stream capture afterwards */            \
    if (!lds_limit_raised) {                                                                                         \
      DQ_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),                                          \
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kLds));                           \
      lds_limit_raised = true;                                                                                       \
    }                                                                                                                \
    hipLaunchKernelGGL(kern, grid, block, kLds, stream, (const half_t*)A, (const uint8_t*)B, (const half_t*)S,       \
                       (const half_t*)Z, (half_t*)C, M, N, K);                                                       \
  } while (0)
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

// config 0, 1, 2: 16, 32, 64 activation rows and 128 weight rows per workgroup; 3, 4, 5: 16, 32, 16
// activation rows and 64 weight rows.  Returns 1 when the shape is not
// covered (the caller falls back to a kernel without these restrictions): the group size must be
// 128 when the mode reads scales, K a multiple of 256, and every operand below 4 GiB (32-bit
// lane offsets).
int w4a16_stream(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int group,
                 int mode, int layout, int config, hipStream_t stream) {
  if (K % kStepK != 0 || N < 1 || M < 1) return 1;
  if (mode >= W4_SCALE && group != 128) return 1;
  if ((size_t)N * K / 2 >= (1ull << 32) || (size_t)M * K * 2 >= (1ull << 32)) return 1;
  switch (config) {
    case 0: return launch_stream<1, 2, 6>(A, B, S, Z, C, M, N, K, mode, layout, stream);
    case 1: return launch_stream<2, 2, 4>(A, B, S, Z, C, M, N, K, mode, layout, stream);
    case 2: return launch_stream<4, 2, 3>(A, B, S, Z, C, M, N, K, mode, layout, stream);
    case 3: return launch_stream<1, 1, 4>(A, B, S, Z, C, M, N, K, mode, layout, stream);
    case 4: return launch_stream<2, 1, 3>(A, B, S, Z, C, M, N, K, mode, layout, stream);
    case 5: return launch_stream<1, 1, 6>(A, B, S, Z, C, M, N, K, mode, layout, stream);
    default: DQ_FAIL("w4a16 stream kernel: unknown configuration %d", config);
  }
}

}  // namespace dq
