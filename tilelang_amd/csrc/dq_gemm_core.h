// Shared skeleton of the LDS-staged dequantize-GEMM kernels for gfx950.
//
// Replaces the T.Pipelined / T.copy / T.gemm loop the reference's examples share
// (e.g. examples/dequantize_gemm/example_dequant_gemm_bf16_mxfp4_cdna4.py:231-244,
// example_dequant_gemm_w4a8.py:132-147, examples/bitnet-1.58b/kernel_benchmark/
// tilelang_bitnet_158_int8xint2_prefill.py:238-296) and the tl::gemm_ss template it lowers to
// (src/tl_templates/hip/gemm.h:158-232).  One kernel template, instantiated per weight format
// through a policy:
//
//   * block tile 256 x 256 x BK (BK = 128 bytes of A per row: 64 x 16-bit or 128 x int8), 4 waves
//     as 2 x 2, 128 x 128 per wave = 4 x 4 MFMA 32x32 accumulators (256 registers per lane);
//   * A (transformed by the policy, 16 bytes at a time, on its way through registers) and the
//     PACKED B tile are double-buffered in LDS; the next tile travels global -> registers while
//     the current one is multiplied;
//   * B is never materialised in memory at the compute type: lane (g, c) of a wave reads the
//     packed bytes of the half-tile k in [g*BK/2, (g+1)*BK/2) of its weight row and decodes them
//     in registers straight into MFMA operands.  The contraction index of MFMA step j is labelled
//     k = g*BK/2 + j*BK/8 + perm(e) for BOTH operands, where perm is whatever element order the
//     policy's cheapest decoder produces; the policy's A transform applies the same perm;
//   * A rows are 128 B in LDS, their 16-byte pieces XOR-swizzled with the row index so the 8
//     lanes of a ds_read_b128 phase hit 8 different bank groups;
//   * output tiles are assigned to workgroups so that each XCD (workgroup id mod 8) walks a
//     compact block of tiles and re-uses its A / B panels out of its own L2;
//   * the epilogue goes through LDS so that every lane stores 16 contiguous bytes (or, for the
//     transposed-output variants, contiguous runs along M).
#pragma once

#include "dq_common.h"

namespace dq {
namespace gemm {

constexpr int BM = 256, BN = 256;
constexpr int kThreads = 256;
constexpr int kARowBytes = 128;            // bytes of one A row per k-block in LDS
constexpr int kAStage = BM * kARowBytes;   // 32 KiB

struct Params {
  const void* A;
  const void* B;
  const void* S;     // scales (policy specific) or nullptr
  const void* Z;     // zeros / second scale (policy specific) or nullptr
  const void* Bias;  // optional
  void* C;
  int M, N, K;
  int tiles_m, tiles_n;
  int p0, p1;        // policy specific integers (e.g. scale exponent offset, group shift)
  float f0;          // policy specific float (e.g. 1 / weight scale)
};

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

// Policy interface (all static):
//   kBRowBytes        packed B bytes per weight row per k-block: 32 or 64
//   kAPacked          A arrives as packed int4 (64 B per row per k-block, expanded while staging)
//   kKPerBlock        k values per block (64 for 16-bit operands, 128 for int8)
//   frag_t, acc_t     MFMA operand / accumulator vector types
//   mfma(a, b, c)
//   stage_a(uint4)    transform of one 16-byte A piece (16 B of one row) on its way to LDS
//   expand_a(uint4, uint4&, uint4&)   kAPacked only: 16 packed bytes -> two 16-byte pieces
//   ScaleRaw / Scale, fetch_scale(p, row, kb, g) / prep_scale(raw, p)
//   decode(const uint32_t* words, int j, const Scale&)  -> B operand of MFMA step j; `words` are
//       the lane's kBRowBytes/2 packed bytes as dwords
//   Epilogue: out_t, kTransposed, finish(acc value, p, m, n) -> value stored
template <class P>
__global__ __launch_bounds__(kThreads, 1) void gemm_kernel(const Params p) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int kBStage = BN * P::kBRowBytes;
  constexpr int kStage = kAStage + kBStage;
  constexpr int kBPiecesPerRow = P::kBRowBytes / 16;           // 2 or 4
  constexpr int kBLoads = BN * kBPiecesPerRow / kThreads;       // 2 or 4
  constexpr int kBWords = P::kBRowBytes / 8;                    // dwords per lane: 4 or 8
  constexpr int kALoads = P::kAPacked ? 4 : 8;                  // 16-byte global loads of A per thread

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;  // 2 x 2 waves, 128 x 128 each
  const int g = lane >> 5, r = lane & 31;
  const int M = p.M, N = p.N, K = p.K;

  int tm, tn;
  tile_of_block(blockIdx.x, p.tiles_m, p.tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  const int KB = K / P::kKPerBlock;
  const size_t a_row_bytes = P::kAPacked ? (size_t)(K >> 1) : (size_t)K * (kARowBytes / P::kKPerBlock == 2 ? 2 : 1);
  const size_t b_row_bytes = (size_t)K * P::kBRowBytes / P::kKPerBlock;

  // ---- global -> register staging ---------------------------------------------------------
  // A piece q = tid + 256 i: row q / 8, 16-byte piece q % 8 of the 128-byte row.  A packed A row
  // is 64 B per block: piece q = tid + 256 i covers row q / 4, packed piece q % 4, and expands
  // to LDS pieces 2 (q % 4) and 2 (q % 4) + 1.
  const unsigned char* a_src[kALoads];
  int a_dst[kALoads], a_dst2[kALoads];
#pragma unroll
  for (int i = 0; i < kALoads; ++i) {
    const int q = tid + kThreads * i;
    if constexpr (P::kAPacked) {
      const int row = q >> 2, piece = q & 3;
      a_src[i] = (const unsigned char*)p.A + (size_t)min(m0 + row, M - 1) * a_row_bytes + piece * 16;
      a_dst[i] = row * 128 + (((2 * piece) ^ (row & 7)) << 4);
      a_dst2[i] = row * 128 + (((2 * piece + 1) ^ (row & 7)) << 4);
    } else {
      const int row = q >> 3, piece = q & 7;
      a_src[i] = (const unsigned char*)p.A + (size_t)min(m0 + row, M - 1) * a_row_bytes + piece * 16;
      a_dst[i] = row * 128 + ((piece ^ (row & 7)) << 4);
      a_dst2[i] = 0;
    }
  }
  const unsigned char* b_src[kBLoads];
  int b_dst[kBLoads];
#pragma unroll
  for (int i = 0; i < kBLoads; ++i) {
    const int q = tid + kThreads * i;
    const int row = q / kBPiecesPerRow, piece = q % kBPiecesPerRow;
    b_src[i] = (const unsigned char*)p.B + (size_t)min(n0 + row, N - 1) * b_row_bytes + piece * 16;
    // rotate the pieces of a row by (row / 4) so that 8 consecutive rows cover all bank groups
    b_dst[i] = kAStage + row * P::kBRowBytes + (((piece + (row >> (kBPiecesPerRow == 2 ? 2 : 1))) % kBPiecesPerRow) << 4);
  }

  uint4_t a_reg[kALoads], b_reg[kBLoads];
  auto load_tile = [&](int kb) {
    const size_t a_step = P::kAPacked ? 64 : 128;
#pragma unroll
    for (int i = 0; i < kALoads; ++i) a_reg[i] = *reinterpret_cast<const uint4_t*>(a_src[i] + (size_t)kb * a_step);
#pragma unroll
    for (int i = 0; i < kBLoads; ++i)
      b_reg[i] = *reinterpret_cast<const uint4_t*>(b_src[i] + (size_t)kb * P::kBRowBytes);
  };
  auto store_tile = [&](int stage) {
    unsigned char* base = smem + stage * kStage;
#pragma unroll
    for (int i = 0; i < kALoads; ++i) {
      if constexpr (P::kAPacked) {
        uint4_t lo, hi;
        P::expand_a(a_reg[i], lo, hi);
        *reinterpret_cast<uint4_t*>(base + a_dst[i]) = lo;
        *reinterpret_cast<uint4_t*>(base + a_dst2[i]) = hi;
      } else {
        *reinterpret_cast<uint4_t*>(base + a_dst[i]) = P::stage_a(a_reg[i]);
      }
    }
#pragma unroll
    for (int i = 0; i < kBLoads; ++i) *reinterpret_cast<uint4_t*>(base + b_dst[i]) = b_reg[i];
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
  // packed B of n-block nb: row wn*128 + nb*32 + r, the half of the row that belongs to group g
  int b_off[4][kBPiecesPerRow / 2];
  int w_row[4];
#pragma unroll
  for (int nb = 0; nb < 4; ++nb) {
    const int row = wn * 128 + nb * 32 + r;
    w_row[nb] = min(n0 + row, N - 1);
#pragma unroll
    for (int h = 0; h < kBPiecesPerRow / 2; ++h) {
      const int piece = g * (kBPiecesPerRow / 2) + h;
      b_off[nb][h] = kAStage + row * P::kBRowBytes + (((piece + (row >> (kBPiecesPerRow == 2 ? 2 : 1))) % kBPiecesPerRow) << 4);
    }
  }

  typename P::acc_t acc[4][4];
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mb][nb][i] = 0;

  // ---- prologue --------------------------------------------------------------------------------
  load_tile(0);
  typename P::ScaleRaw sc_cur[4], sc_next[4];
#pragma unroll
  for (int nb = 0; nb < 4; ++nb) sc_cur[nb] = P::fetch_scale(p, w_row[nb], 0, g);
  store_tile(0);
  if (KB > 1) load_tile(1);
  __syncthreads();

  for (int kb = 0; kb < KB; ++kb) {
    const int stage = kb & 1;
    const unsigned char* base = smem + stage * kStage;
    if (kb + 1 < KB) {
      store_tile(stage ^ 1);  // tile kb+1 (loaded during the previous iteration) -> other stage
#pragma unroll
      for (int nb = 0; nb < 4; ++nb) sc_next[nb] = P::fetch_scale(p, w_row[nb], kb + 1, g);
    }
    if (kb + 2 < KB) load_tile(kb + 2);

    uint32_t bw[4][kBWords];
    typename P::Scale sc[4];
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
#pragma unroll
      for (int h = 0; h < kBPiecesPerRow / 2; ++h) {
        const uint4_t v = *reinterpret_cast<const uint4_t*>(base + b_off[nb][h]);
        bw[nb][4 * h + 0] = v[0]; bw[nb][4 * h + 1] = v[1]; bw[nb][4 * h + 2] = v[2]; bw[nb][4 * h + 3] = v[3];
      }
      sc[nb] = P::prep_scale(sc_cur[nb], p);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      typename P::frag_t af[4], bf[4];
#pragma unroll
      for (int mb = 0; mb < 4; ++mb)
        af[mb] = *reinterpret_cast<const typename P::frag_t*>(base + a_row_off[mb] + ((((g << 2) + j) ^ a_row_sw[mb]) << 4));
#pragma unroll
      for (int nb = 0; nb < 4; ++nb) bf[nb] = P::decode(bw[nb], j, sc[nb]);
#pragma unroll
      for (int mb = 0; mb < 4; ++mb)
#pragma unroll
        for (int nb = 0; nb < 4; ++nb) acc[mb][nb] = P::mfma(af[mb], bf[nb], acc[mb][nb]);
    }
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) sc_cur[nb] = sc_next[nb];
    __syncthreads();
  }

  // ---- epilogue: acc[mb][nb][i] = C[m0 + wm*128 + mb*32 + 8*(i/4) + 4*g + i%4][n0 + wn*128 + nb*32 + r]
  // Staged through LDS (every tile is consumed: the loop ended with a barrier).  Each wave owns
  // a 32 x (128 + 4) slab of 32-bit values; LDS operations of one wave execute in order, so no
  // workgroup barrier is needed between the phases.
  using out_t = typename P::out_t;
  constexpr int kSlabStride = 132;
  constexpr int kOutPerPiece = 16 / sizeof(out_t);  // values per 16-byte store: 8 (16-bit) or 4 (int32)
  uint32_t* slab = reinterpret_cast<uint32_t*>(smem) + wave * (32 * kSlabStride);
#pragma unroll
  for (int mb = 0; mb < 4; ++mb) {
#pragma unroll
    for (int nb = 0; nb < 4; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int row = 8 * (i >> 2) + 4 * g + (i & 3);
        // copy the element out first: bit-casting the vector-element expression itself is unreliable
        const decltype(acc[0][0][0] + 0) elem = acc[mb][nb][i];
        uint32_t bits;
        __builtin_memcpy(&bits, &elem, 4);
        slab[row * kSlabStride + nb * 32 + r] = bits;
      }
    __builtin_amdgcn_wave_barrier();
    if constexpr (!P::kTransposed) {
      // C[M, N]: 32 rows x 128 columns, 16 bytes per lane per store
      constexpr int kPiecesPerRow = 128 / kOutPerPiece;  // 16 or 32
      constexpr int kIters = 32 * kPiecesPerRow / 64;    // 8 or 16
#pragma unroll
      for (int it = 0; it < kIters; ++it) {
        const int q = lane + 64 * it;
        const int row = q / kPiecesPerRow, piece = q % kPiecesPerRow;
        const int m = m0 + wm * 128 + mb * 32 + row;
        const int n = n0 + wn * 128 + piece * kOutPerPiece;
        uint32_t raw[kOutPerPiece];
#pragma unroll
        for (int e = 0; e < kOutPerPiece; e += 4) {
          const uint4_t v = *reinterpret_cast<const uint4_t*>(slab + row * kSlabStride + piece * kOutPerPiece + e);
          raw[e] = v[0]; raw[e + 1] = v[1]; raw[e + 2] = v[2]; raw[e + 3] = v[3];
        }
        if (m < M && n < N) {
          out_t o[kOutPerPiece];
#pragma unroll
          for (int e = 0; e < kOutPerPiece; ++e) o[e] = P::finish(raw[e], p, m, min(n + e, N - 1));
          out_t* dst = (out_t*)p.C + (size_t)m * N + n;
          if ((n + kOutPerPiece <= N) && ((N % kOutPerPiece) == 0)) {
            uint4_t pk;
            __builtin_memcpy(&pk, o, 16);
            *reinterpret_cast<uint4_t*>(dst) = pk;
          } else {
#pragma unroll
            for (int e = 0; e < kOutPerPiece; ++e)
              if (n + e < N) dst[e] = o[e];
          }
        }
      }
    } else {
      // Ct[N, M]: the slab holds 32 (m) x 128 (n); a lane gathers kOutPerPiece consecutive m of one n
      constexpr int kPiecesPerCol = 32 / kOutPerPiece;    // 4 or 8
      constexpr int kIters = 128 * kPiecesPerCol / 64;    // 8 or 16
#pragma unroll
      for (int it = 0; it < kIters; ++it) {
        const int q = lane + 64 * it;
        const int col = q / kPiecesPerCol, piece = q % kPiecesPerCol;
        const int n = n0 + wn * 128 + col;
        const int m = m0 + wm * 128 + mb * 32 + piece * kOutPerPiece;
        if (n < N && m < M) {
          out_t o[kOutPerPiece];
#pragma unroll
          for (int e = 0; e < kOutPerPiece; ++e)
            o[e] = P::finish(slab[(piece * kOutPerPiece + e) * kSlabStride + col], p, min(m + e, M - 1), n);
          out_t* dst = (out_t*)p.C + (size_t)n * M + m;
          if ((m + kOutPerPiece <= M) && ((M % kOutPerPiece) == 0)) {
            uint4_t pk;
            __builtin_memcpy(&pk, o, 16);
            *reinterpret_cast<uint4_t*>(dst) = pk;
          } else {
#pragma unroll
            for (int e = 0; e < kOutPerPiece; ++e)
              if (m + e < M) dst[e] = o[e];
          }
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
}

template <class P>
int launch(const Params& p, hipStream_t stream) {
  constexpr int kLds = 2 * (kAStage + BN * P::kBRowBytes);
  auto kern = gemm_kernel<P>;
  static bool lds_limit_raised = false;  // once per kernel: legal under stream capture afterwards
  if (!lds_limit_raised) {
    DQ_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, kLds));
    lds_limit_raised = true;
  }
  hipLaunchKernelGGL(kern, dim3(p.tiles_m * p.tiles_n), dim3(kThreads), kLds, stream, p);
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

inline Params make_params(const void* A, const void* B, const void* S, const void* Z, const void* Bias, void* C, int M,
                          int N, int K) {
  Params p{};
  p.A = A; p.B = B; p.S = S; p.Z = Z; p.Bias = Bias; p.C = C;
  p.M = M; p.N = N; p.K = K;
  p.tiles_m = (M + BM - 1) / BM;
  p.tiles_n = (N + BN - 1) / BN;
  return p;
}

// ---- building blocks shared by the policies -------------------------------------------------------

struct NoScale {
  struct ScaleRaw {};
  struct Scale {};
  __device__ static __forceinline__ ScaleRaw fetch_scale(const Params&, int, int, int) { return {}; }
  __device__ static __forceinline__ Scale prep_scale(ScaleRaw, const Params&) { return {}; }
};

struct PlainA {
  static constexpr bool kAPacked = false;
  __device__ static __forceinline__ uint4_t stage_a(uint4_t v) { return v; }
  __device__ static __forceinline__ void expand_a(uint4_t, uint4_t&, uint4_t&) {}
};

}  // namespace gemm
}  // namespace dq
