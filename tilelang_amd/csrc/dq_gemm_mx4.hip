// Block-scaled MXFP4 x MXFP4 GEMM on gfx950's scaled matrix instruction.
//
// C[M,N] bf16 = (e2m1(A[M,K/2]) * 2^(SA[M,K/32] - 127)) . (e2m1(B[N,K/2]) * 2^(SB[N,K/32] - 127))^T (+ Bias), fp32
// accumulation: what blockscaled_gemm_ref of examples/blockscaled_gemm_sm100/gemm_mxfp8_blockscaled_1d1d.py:575-620
// computes, with both operands in the 4-bit format of examples/dequantize_gemm/example_dequant_gemm_bf16_mxfp4_cdna4.py
// (two e2m1 codes per byte, even k in the low nibble, one E8M0 byte per 32 k).  The reference reaches block-scaled
// matrix instructions only on NVIDIA parts (T.tcgen05_gemm_blockscaled, :134-140; examples/gemm_sm120/
// sm120_nvfp4_blockscaled_gemm.py:132-143); here v_mfma_scale_f32_32x32x64_f8f6f4 takes the packed codes and the
// scale bytes as they lie in memory, so nothing is decoded in registers at all.
//
//   * block tile 256 x 256 x 128 k, 4 waves as 2 x 2, 128 x 128 per wave = 4 x 4 accumulators of 32 x 32;
//   * both operand tiles are 256 rows x 64 bytes; they and the scale dwords (4 bytes = the 4 scale blocks of a
//     row and tile) travel global -> LDS by global_load_lds into a ring of four stages, two or three tiles ahead,
//     the loads of two consecutive tiles issued as pairs (together they cover whole 128-byte lines);
//   * lane (r, g) of a wave feeds row r with the 32 codes (16 bytes) of scale block 2 s + g in MFMA step s; the
//     16-byte pieces of a row are XOR-swizzled with (row >> 2) & 3 (on the source side of the DMA) so that a
//     ds_read_b128 phase of 16 lanes covers all banks;
//   * the instruction picks its scale out of a lane register by byte index: the row's dword is shifted right by
//     8 g once per tile, after which byte 2 s is the scale of step s for both lane halves;
//   * the loop is skewed by one step (the MFMAs of a tile's second step issue while the first operands of the
//     next tile are read), one s_waitcnt vmcnt and one barrier per tile, epilogue through LDS as in
//     dq_gemm_core.h.
#include "dq_gemm_core.h"

namespace dq {

namespace {

using gemm::Params;

typedef int v8i_t __attribute__((ext_vector_type(8)));

constexpr int kKTile = 128;                // k per tile
constexpr int kRowBytes = kKTile / 2;      // 64 packed bytes per row and tile
constexpr int kOpStage = 256 * kRowBytes;  // 16 KiB per operand
constexpr int kStage = 2 * kOpStage;       // A then B
constexpr int kStages = 4;                 // tile t lives in stage t % 4
constexpr int kRing = kStages * kStage;    // scale ring behind the operand stages
constexpr int kScaleStage = 2 * 1024;      // 256 dwords of A scales, 256 of B scales
constexpr int kPipe = kRing + kStages * kScaleStage;
constexpr int kTileOps = 10;               // DMA instructions per thread and tile: 4 A, 4 B, 2 scale

template <bool HAS_BIAS>
struct Mx4Out {
  static constexpr bool kTransposed = false;
  using out_t = bf16_t;
  __device__ static __forceinline__ out_t finish(uint32_t raw, const Params& p, int m, int n) {
    float v = __builtin_bit_cast(float, raw);
    if constexpr (HAS_BIAS) v += (float)((const bf16_t*)p.Bias)[(size_t)m * p.N + n];
    return (bf16_t)v;
  }
};

__device__ __forceinline__ float16_t mfma_scaled(uint4_t a, uint4_t b, float16_t c, int sa, int sb, int step) {
  const v8i_t av = {(int)a[0], (int)a[1], (int)a[2], (int)a[3], 0, 0, 0, 0};
  const v8i_t bv = {(int)b[0], (int)b[1], (int)b[2], (int)b[3], 0, 0, 0, 0};
  // format 4 = fp4 (e2m1) for both operands; the scale of step s is byte 2 s of the lane's scale register
  if (step == 0) return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, c, 4, 4, 0, sa, 0, sb);
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, c, 4, 4, 2, sa, 2, sb);
}

// p.A / p.Z: codes and scales of A; p.B / p.S: codes and scales of B.
template <class P>
__global__ __launch_bounds__(256, 1) void mx4_gemm_kernel(Params p) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int kMBW = 4, kNBW = 4;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int r = lane & 31, g = lane >> 5;
  const int M = p.M, N = p.N, K = p.K;
  int tm, tn;
  gemm::tile_of_block(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
  const int m0 = tm * 256, n0 = tn * 256;
  const int KB = K / kKTile;
  const unsigned lds0 = (unsigned)(size_t)smem;
  const unsigned row_bytes = (unsigned)(K >> 1);

  // ---- DMA geometry: instruction i of wave w covers rows 16 (4 w + i) .. +15 of an operand tile; lane l lands
  // at row l / 4, slot l % 4, and fetches the piece that belongs in that slot.
  unsigned a_voff[4], b_voff[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = 16 * (4 * wave + i) + (lane >> 2);
    const int piece = (lane & 3) ^ ((row >> 2) & 3);
    a_voff[i] = (unsigned)min(m0 + row, M - 1) * row_bytes + (unsigned)(piece << 4);
    b_voff[i] = (unsigned)min(n0 + row, N - 1) * row_bytes + (unsigned)(piece << 4);
  }
  const unsigned sa_voff = (unsigned)min(m0 + tid, M - 1) * (unsigned)(K >> 5);
  const unsigned sb_voff = (unsigned)min(n0 + tid, N - 1) * (unsigned)(K >> 5);
  auto issue_op = [&](int op, int kb, int stage) {
    const unsigned sbase = lds0 + stage * kStage;
    if (op < 4) {
      gemm::dma16(sbase + (wave * 4 + op) * 1024, a_voff[op], (const unsigned char*)p.A + (size_t)kb * kRowBytes);
    } else if (op < 8) {
      const int i = op - 4;
      gemm::dma16(sbase + kOpStage + (wave * 4 + i) * 1024, b_voff[i], (const unsigned char*)p.B + (size_t)kb * kRowBytes);
    } else if (op == 8) {
      gemm::dma4(lds0 + kRing + stage * kScaleStage + wave * 256, sa_voff, (const unsigned char*)p.Z + (size_t)kb * 4);
    } else {
      gemm::dma4(lds0 + kRing + stage * kScaleStage + 1024 + wave * 256, sb_voff, (const unsigned char*)p.S + (size_t)kb * 4);
    }
  };

  // ---- fragment read offsets: the swizzle key (row >> 2) & 3 depends on r only, so the four row blocks of an
  // operand sit at constant distances (32 rows x 64 B) from the first
  const int key = (r >> 2) & 3;
  int a_off[2], b_off[2];  // per step: piece 2 s + g
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    a_off[s] = (wm * 128 + r) * kRowBytes + (((2 * s + g) ^ key) << 4);
    b_off[s] = kOpStage + (wn * 128 + r) * kRowBytes + (((2 * s + g) ^ key) << 4);
  }
  const int sa_off = kRing + (wm * 128 + r) * 4;
  const int sb_off = kRing + 1024 + (wn * 128 + r) * 4;
  const int shift = 8 * g;
  auto read_frag = [&](const unsigned char* base, int off, int blk) -> uint4_t {
    return *reinterpret_cast<const uint4_t*>(base + off + blk * (32 * kRowBytes));
  };
  auto read_scale = [&](int stage, int off, int blk) -> uint32_t {  // the row's four scale bytes, unshifted
    return *reinterpret_cast<const uint32_t*>(smem + off + stage * kScaleStage + blk * 128);
  };

  float16_t acc[kMBW][kNBW];
#pragma unroll
  for (int mb = 0; mb < kMBW; ++mb)
#pragma unroll
    for (int nb = 0; nb < kNBW; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mb][nb][i] = 0.f;

  // ---- prologue: tiles 0 and 1 (KB >= 2 is checked by the launcher), instruction by instruction as a pair
#pragma unroll
  for (int op = 0; op < kTileOps; ++op) {
    issue_op(op, 0, 0);
    issue_op(op, 1, 1);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  uint4_t af_c[4], bf_c[4], af_n[4], bf_n[4];
  int sa_c[4], sb_c[4], sa_n[4], sb_n[4];
  uint32_t sa_r[4], sb_r[4];

  // A chunk = one A fragment against the four B fragments; the side work sits behind the MFMAs it hides under.
  auto chunk = [&](int q, int step, auto do_mfma_tag, auto&& side_a, auto&& side_b, auto&& side_c, auto&& side_d) {
    constexpr bool do_mfma = decltype(do_mfma_tag)::value;
    if constexpr (do_mfma) acc[q][0] = mfma_scaled(af_c[q], bf_c[0], acc[q][0], sa_c[q], sb_c[0], step);
    side_a();
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (do_mfma) acc[q][1] = mfma_scaled(af_c[q], bf_c[1], acc[q][1], sa_c[q], sb_c[1], step);
    side_b();
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (do_mfma) acc[q][2] = mfma_scaled(af_c[q], bf_c[2], acc[q][2], sa_c[q], sb_c[2], step);
    side_c();
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (do_mfma) acc[q][3] = mfma_scaled(af_c[q], bf_c[3], acc[q][3], sa_c[q], sb_c[3], step);
    side_d();
    __builtin_amdgcn_sched_barrier(0);
  };

  // One iteration = tile kb out of `stage`:
  //   chunks 0..3  MFMAs of step 1 of tile kb-1 (operands and scales already in registers); side work: read the
  //                scale dwords and the step-0 fragments of tile kb, B side first (every chunk needs all four B
  //                fragments, chunk q only A fragment q), shift the scale dwords two chunks after their reads
  //   chunks 4..7  MFMAs of step 0 of tile kb; side work: read its step-1 fragments, B side first again
  // so that no LDS read is consumed sooner than four MFMAs after it was issued,
  // A tile's rows are 64 bytes, half a cache line, and the other half is the next tile's: the loads of tiles
  // t and t + 1 (t even) are therefore issued as pairs, the same instruction for t and then for t + 1, so that
  // the second finds its lines already on their way.  An even iteration kb issues the pairs of tiles kb + 2
  // and kb + 3 (kIssue of them: 2, or 1 / 0 at the end of K) into stages (kb + 2) % 4 and (kb + 3) % 4, both
  // free since the barrier that ended iteration kb - 1; an odd iteration issues nothing.
  auto iteration = [&](int kb, auto first_tag, auto issue_tag) {
    constexpr bool first = decltype(first_tag)::value;
    constexpr int kIssue = decltype(issue_tag)::value;
    using DoMfma = std::integral_constant<bool, !first>;
    const int stage = kb & 3;
    const unsigned char* base = smem + stage * kStage;
    auto dma = [&](int op) {
      if constexpr (kIssue >= 1) issue_op(op, kb + 2, (kb + 2) & 3);
      if constexpr (kIssue >= 2) issue_op(op, kb + 3, (kb + 3) & 3);
    };
    chunk(0, 1, DoMfma{},
          [&] { for (int i = 0; i < 4; ++i) sb_r[i] = read_scale(stage, sb_off, i); },
          [&] { dma(0); },
          [&] { bf_n[0] = read_frag(base, b_off[0], 0); bf_n[1] = read_frag(base, b_off[0], 1); },
          [&] { bf_n[2] = read_frag(base, b_off[0], 2); bf_n[3] = read_frag(base, b_off[0], 3); dma(1); });
    chunk(1, 1, DoMfma{},
          [&] { for (int i = 0; i < 4; ++i) sa_r[i] = read_scale(stage, sa_off, i); },
          [&] { dma(2); },
          [&] { af_n[0] = read_frag(base, a_off[0], 0); af_n[1] = read_frag(base, a_off[0], 1); },
          [&] { af_n[2] = read_frag(base, a_off[0], 2); af_n[3] = read_frag(base, a_off[0], 3); dma(3); });
    chunk(2, 1, DoMfma{},
          [&] { for (int i = 0; i < 4; ++i) sb_n[i] = (int)(sb_r[i] >> shift); },
          [&] { dma(4); },
          [&] { for (int i = 0; i < 4; ++i) sa_n[i] = (int)(sa_r[i] >> shift); },
          [&] { dma(5); });
    chunk(3, 1, DoMfma{}, [] {}, [&] { dma(6); }, [] {}, [&] { dma(7); });
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      af_c[q] = af_n[q]; bf_c[q] = bf_n[q];
      sa_c[q] = sa_n[q]; sb_c[q] = sb_n[q];
    }
#pragma unroll
    for (int q = 0; q < 4; ++q)
      chunk(q, 0, std::true_type{},
            [&] { if (q < 2) bf_n[2 * q] = read_frag(base, b_off[1], 2 * q); else af_n[2 * (q - 2)] = read_frag(base, a_off[1], 2 * (q - 2)); },
            [&] { if (q < 2) dma(8 + q); },
            [&] { if (q < 2) bf_n[2 * q + 1] = read_frag(base, b_off[1], 2 * q + 1); else af_n[2 * (q - 2) + 1] = read_frag(base, a_off[1], 2 * (q - 2) + 1); },
            [] {});
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      af_c[q] = af_n[q]; bf_c[q] = bf_n[q];
    }
    // tile kb + 1 must have landed.  After an even iteration it was issued two iterations ago and only this
    // iteration's own loads may still be in flight; after an odd one it was issued in the iteration before, paired
    // with tile kb + 2, so everything has to land.
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kIssue * kTileOps) : "memory");
    __syncthreads();
  };

  using Zero = std::integral_constant<int, 0>;
  using One = std::integral_constant<int, 1>;
  using Two = std::integral_constant<int, 2>;
  if (KB > 3) iteration(0, std::true_type{}, Two{});
  else if (KB == 3) iteration(0, std::true_type{}, One{});
  else iteration(0, std::true_type{}, Zero{});
  iteration(1, std::false_type{}, Zero{});
  int kb = 2;
  for (; kb + 3 < KB; kb += 2) {  // steady state: an issuing iteration and a quiet one
    iteration(kb, std::false_type{}, Two{});
    iteration(kb + 1, std::false_type{}, Zero{});
  }
  if (kb + 2 < KB) {  // three tiles left: the last one still has to be fetched
    iteration(kb, std::false_type{}, One{});
    ++kb;
  }
  for (; kb < KB; ++kb) iteration(kb, std::false_type{}, Zero{});
  // step 1 of the last tile
#pragma unroll
  for (int q = 0; q < 4; ++q)
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) acc[q][nb] = mfma_scaled(af_c[q], bf_c[nb], acc[q][nb], sa_c[q], sb_c[nb], 1);

  DQ_GEMM_EPILOGUE
}

template <class P>
int launch_mx4(Params p, hipStream_t stream) {
  constexpr int kSlabs = 4 * 32 * (32 * 4 + 4) * 4;  // epilogue staging
  constexpr int kLds = kPipe > kSlabs ? kPipe : kSlabs;
  p.tiles_m = (p.M + 255) / 256;
  p.tiles_n = (p.N + 255) / 256;
  auto kern = mx4_gemm_kernel<P>;
  static bool lds_limit_raised[kMaxDevices];
  if (raise_lds_limit<kLds>(kern, lds_limit_raised)) return -1;
  hipLaunchKernelGGL(kern, dim3(p.tiles_m * p.tiles_n), dim3(256), kLds, stream, p);
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

}  // namespace

int mx4_lds_bytes() { return kPipe; }

int mxfp4_mxfp4_gemm(const void* A, const void* SA, const void* B, const void* SB, const void* Bias, void* C, int M,
                     int N, int K, hipStream_t stream) {
  // 32-bit lane offsets into A and B; the kernel's prologue issues two tiles
  if (K % kKTile != 0 || K < 2 * kKTile) DQ_FAIL("mxfp4 x mxfp4 gemm: K=%d must be a multiple of %d and at least %d", K, kKTile, 2 * kKTile);
  if ((size_t)M * (K / 2) >= (1ull << 32) || (size_t)N * (K / 2) >= (1ull << 32))
    DQ_FAIL("mxfp4 x mxfp4 gemm: packed A and B must each be smaller than 4 GiB (M=%d N=%d K=%d)", M, N, K);
  Params p = gemm::make_params(A, B, SB, SA, Bias, C, M, N, K);
  if (Bias) return launch_mx4<Mx4Out<true>>(p, stream);
  return launch_mx4<Mx4Out<false>>(p, stream);
}

}  // namespace dq
