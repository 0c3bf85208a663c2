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
//     PACKED B tile live in three LDS stages; tile kb+3 travels global -> registers and tile kb+2
//     registers -> LDS while tile kb is multiplied, and the operands of every MFMA step are
//     fetched (and decoded) one step ahead, across tile boundaries too;
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

#include <type_traits>

#ifndef DQ_SWZ_SHIFT
#define DQ_SWZ_SHIFT 1
#endif

#ifndef DQ_DMA_NBW
#define DQ_DMA_NBW 4  // wave tile columns / 32 of the direct-to-LDS kernel (2 = eight waves, two per SIMD)
#endif
#ifndef DQ_DMA_MBW
#define DQ_DMA_MBW 4  // wave tile rows / 32 of the direct-to-LDS kernel (2 = 128 x 256 tiles, two workgroups per CU)
#endif

namespace dq {
namespace gemm {

constexpr int BM = 256, BN = 256;
constexpr int kThreads = 256;
constexpr int kARowBytes = 128;            // bytes of one A row per k-block in LDS
constexpr int kAStage = BM * kARowBytes;   // 32 KiB

// XOR key of the 16-byte pieces of A row `row` in LDS (rows are 128 B).
__host__ __device__ constexpr int a_swz(int row) { return (row >> DQ_SWZ_SHIFT) & 7; }

// Where 16-byte piece `piece` of packed-B row `row` sits inside the row in LDS (register-staged kernel).  Rows of
// 32 or 64 bytes: rotated by the row index so that the 16 rows of one ds_read_b128 phase cover all 64 banks.  Rows
// of 128 bytes (an operand stored at the compute type, nothing to decode): the XOR swizzle of the A rows.
template <int kPieces>
__host__ __device__ constexpr int b_piece_pos(int row, int piece) {
  if (kPieces == 8) return piece ^ a_swz(row);
  return (piece + (row >> (kPieces == 2 ? 3 : 2))) % kPieces;
}

struct Params {
  const void* A;
  const void* B;
  const void* S;     // scales (policy specific) or nullptr
  const void* Z;     // zeros / second scale (policy specific) or nullptr
  const void* Bias;  // optional
  void* C;
  int M, N, K;       // K: contraction length of this launch (of one K slice when split > 1)
  int ldk;           // k elements per stored row of A and B (= K unless the launch covers K slices)
  int split;         // K slices, each its own set of workgroups and its own M x N output behind C
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

// Split-K (examples/dequantize_gemm/example_dequant_gemm_fp4_hopper.py:136-167): workgroup ids beyond the first
// tiles_m x tiles_n belong to further K slices.  Slice z reads columns [z K, (z + 1) K) of A and B and writes the
// z-th M x N (or N x M) partial result behind C; a second kernel sums the partial results.  Plain (unpacked) A only.
template <class P>
__device__ __forceinline__ void take_k_slice(Params& p, int& bid) {
  if (p.split > 1) {
    const int tiles = p.tiles_m * p.tiles_n;
    const int z = bid / tiles;
    bid -= z * tiles;
    p.A = (const unsigned char*)p.A + (size_t)z * p.K * (kARowBytes / P::kKPerBlock);
    p.B = (const unsigned char*)p.B + (size_t)z * p.K * P::kBRowBytes / P::kKPerBlock;
    p.C = (unsigned char*)p.C + (size_t)z * p.M * p.N * sizeof(typename P::out_t);
  }
}

// Epilogue shared by both kernel variants (a macro: it uses the kernel's locals).
// acc[mb][nb][i] = C[m0 + (wm*kMBW + mb)*32 + 8*(i/4) + 4*g + i%4][n0 + (wn*kNBW + nb)*32 + r], with kMBW x kNBW
// blocks of 32 x 32 per wave (constants of the kernel that expands the macro).  Staged through
// LDS (every tile is consumed: the loop ended with a barrier) so that each lane stores 16 contiguous
// bytes.  Each wave owns a 32 x (128 + 4) slab of 32-bit values; LDS operations of one wave execute
// in order, so no workgroup barrier is needed between the phases.  Each wave owns a 32 x (32 kNBW + 4) slab.
// C is written once and not read again by the kernel: the 16-byte stores are nontemporal, which keeps the
// output from displacing operand lines in the L2 (MXFP4 GEMM 361 -> 358 us, block-scaled GEMM 147 -> 138 us).
#define DQ_GEMM_EPILOGUE \
  using out_t = typename P::out_t; \
  constexpr int kSlabStride = 32 * kNBW + 4; \
  constexpr int kOutPerPiece = 16 / sizeof(out_t); \
  uint32_t* slab = reinterpret_cast<uint32_t*>(smem) + wave * (32 * kSlabStride); \
  _Pragma("unroll") \
  for (int mb = 0; mb < kMBW; ++mb) { \
  _Pragma("unroll") \
    for (int nb = 0; nb < kNBW; ++nb) \
  _Pragma("unroll") \
      for (int i = 0; i < 16; ++i) { \
        const int row = 8 * (i >> 2) + 4 * g + (i & 3); \
        const decltype(acc[0][0][0] + 0) elem = acc[mb][nb][i]; \
        uint32_t bits; \
        __builtin_memcpy(&bits, &elem, 4); \
        slab[row * kSlabStride + nb * 32 + r] = bits; \
      } \
    __builtin_amdgcn_wave_barrier(); \
    if constexpr (!P::kTransposed) { \
      constexpr int kPiecesPerRow = 32 * kNBW / kOutPerPiece; \
      constexpr int kIters = 32 * kPiecesPerRow / 64; \
  _Pragma("unroll") \
      for (int it = 0; it < kIters; ++it) { \
        const int q = lane + 64 * it; \
        const int row = q / kPiecesPerRow, piece = q % kPiecesPerRow; \
        const int m = m0 + wm * (32 * kMBW) + mb * 32 + row; \
        const int n = n0 + wn * (32 * kNBW) + piece * kOutPerPiece; \
        uint32_t raw[kOutPerPiece]; \
  _Pragma("unroll") \
        for (int e = 0; e < kOutPerPiece; e += 4) { \
          const uint4_t v = *reinterpret_cast<const uint4_t*>(slab + row * kSlabStride + piece * kOutPerPiece + e); \
          raw[e] = v[0]; raw[e + 1] = v[1]; raw[e + 2] = v[2]; raw[e + 3] = v[3]; \
        } \
        if (m < M && n < N) { \
          out_t o[kOutPerPiece]; \
  _Pragma("unroll") \
          for (int e = 0; e < kOutPerPiece; ++e) o[e] = P::finish(raw[e], p, m, min(n + e, N - 1)); \
          out_t* dst = (out_t*)p.C + (size_t)m * N + n; \
          if ((n + kOutPerPiece <= N) && ((N % kOutPerPiece) == 0)) { \
            uint4_t pk; \
            __builtin_memcpy(&pk, o, 16); \
            __builtin_nontemporal_store(pk, reinterpret_cast<uint4_t*>(dst)); \
          } else { \
  _Pragma("unroll") \
            for (int e = 0; e < kOutPerPiece; ++e) \
              if (n + e < N) dst[e] = o[e]; \
          } \
        } \
      } \
    } else { \
      constexpr int kPiecesPerCol = 32 / kOutPerPiece; \
      constexpr int kIters = 32 * kNBW * kPiecesPerCol / 64; \
  _Pragma("unroll") \
      for (int it = 0; it < kIters; ++it) { \
        const int q = lane + 64 * it; \
        const int col = q / kPiecesPerCol, piece = q % kPiecesPerCol; \
        const int n = n0 + wn * (32 * kNBW) + col; \
        const int m = m0 + wm * (32 * kMBW) + mb * 32 + piece * kOutPerPiece; \
        if (n < N && m < M) { \
          out_t o[kOutPerPiece]; \
  _Pragma("unroll") \
          for (int e = 0; e < kOutPerPiece; ++e) \
            o[e] = P::finish(slab[(piece * kOutPerPiece + e) * kSlabStride + col], p, min(m + e, M - 1), n); \
          out_t* dst = (out_t*)p.C + (size_t)n * M + m; \
          if ((m + kOutPerPiece <= M) && ((M % kOutPerPiece) == 0)) { \
            uint4_t pk; \
            __builtin_memcpy(&pk, o, 16); \
            __builtin_nontemporal_store(pk, reinterpret_cast<uint4_t*>(dst)); \
          } else { \
  _Pragma("unroll") \
            for (int e = 0; e < kOutPerPiece; ++e) \
              if (m + e < M) dst[e] = o[e]; \
          } \
        } \
      } \
    } \
    __builtin_amdgcn_wave_barrier(); \
  } \
  /* end of epilogue */

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
// kKSplit = 2: eight waves, two per SIMD; waves 4..7 are a second copy of the pipeline (LDS stages of their own) that
// takes the odd k-blocks while waves 0..3 take the even ones, and hands its accumulators over once, through LDS,
// after the loop.  For problems that give each CU one small tile with a long K (BitNet at M = 256): the second wave
// of a SIMD runs its matrix instructions under the first one's decode and waits.  Needs an even number of k-blocks.
template <class P, int kMBW, int kNBW, int kKSplit = 1>
__global__ __launch_bounds__(kThreads * kKSplit, 1) void gemm_kernel(const Params p_in) {
  Params p = p_in;
  int bid = blockIdx.x;
  take_k_slice<P>(p, bid);
  extern __shared__ __align__(16) unsigned char smem_all[];
  static_assert(kKSplit == 1 || kKSplit == 2, "one or two copies of the pipeline");
  constexpr int BM = 64 * kMBW, BN = 64 * kNBW;  // 2 x 2 waves of kMBW x kNBW blocks of 32 x 32 (shadow the 256 x 256 default)
  constexpr int kAStage = BM * kARowBytes;
  constexpr int kBStage = BN * P::kBRowBytes;
  constexpr int kStage = kAStage + kBStage;
  constexpr int kBPiecesPerRow = P::kBRowBytes / 16;           // 2 or 4
  constexpr int kBPieces = BN * kBPiecesPerRow;                 // 16-byte pieces of a packed B tile
  constexpr int kBLoads = (kBPieces + kThreads - 1) / kThreads;
  constexpr int kBWords = P::kBRowBytes / 8;                    // dwords per lane: 4 or 8
  constexpr int kALoads = (P::kAPacked ? 4 : 8) * BM / 256;     // 16-byte global loads of A per thread

  const int tid = threadIdx.x & (kThreads - 1);
  const int kh = kKSplit == 1 ? 0 : (int)(threadIdx.x / kThreads);  // which copy of the pipeline
  unsigned char* const smem = smem_all + kh * (3 * kStage);
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;  // 2 x 2 waves
  const int g = lane >> 5, r = lane & 31;
  const int M = p.M, N = p.N, K = p.K;

  int tm, tn;
  tile_of_block(bid, p.tiles_m, p.tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  const int KB = K / P::kKPerBlock / kKSplit;  // k-blocks of this copy: kb -> global k-block kb * kKSplit + kh
  const size_t a_row_bytes = P::kAPacked ? (size_t)(p.ldk >> 1) : (size_t)p.ldk * (kARowBytes / P::kKPerBlock == 2 ? 2 : 1);
  const size_t b_row_bytes = (size_t)p.ldk * P::kBRowBytes / P::kKPerBlock;

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
      a_dst[i] = row * 128 + (((2 * piece) ^ a_swz(row)) << 4);
      a_dst2[i] = row * 128 + (((2 * piece + 1) ^ a_swz(row)) << 4);
    } else {
      const int row = q >> 3, piece = q & 7;
      a_src[i] = (const unsigned char*)p.A + (size_t)min(m0 + row, M - 1) * a_row_bytes + piece * 16;
      a_dst[i] = row * 128 + ((piece ^ a_swz(row)) << 4);
      a_dst2[i] = 0;
    }
  }
  const unsigned char* b_src[kBLoads];
  int b_dst[kBLoads];
  bool b_on[kBLoads];  // a tile narrower than the workgroup leaves some threads without a piece
#pragma unroll
  for (int i = 0; i < kBLoads; ++i) {
    const int q0 = tid + kThreads * i;
    b_on[i] = q0 < kBPieces;
    const int q = b_on[i] ? q0 : 0;
    const int row = q / kBPiecesPerRow, piece = q % kBPiecesPerRow;
    b_src[i] = (const unsigned char*)p.B + (size_t)min(n0 + row, N - 1) * b_row_bytes + piece * 16;
    b_dst[i] = kAStage + row * P::kBRowBytes + (b_piece_pos<kBPiecesPerRow>(row, piece) << 4);
  }

  uint4_t a_reg[kALoads], b_reg[kBLoads];
  auto load_tile = [&](int kb_local) {
    const int kb = kb_local * kKSplit + kh;
    const size_t a_step = P::kAPacked ? 64 : 128;
#pragma unroll
    for (int i = 0; i < kALoads; ++i) a_reg[i] = *reinterpret_cast<const uint4_t*>(a_src[i] + (size_t)kb * a_step);
#pragma unroll
    for (int i = 0; i < kBLoads; ++i)
      if (b_on[i]) b_reg[i] = *reinterpret_cast<const uint4_t*>(b_src[i] + (size_t)kb * P::kBRowBytes);
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
    for (int i = 0; i < kBLoads; ++i)
      if (b_on[i]) *reinterpret_cast<uint4_t*>(base + b_dst[i]) = b_reg[i];
  };

  // ---- fragment read offsets -----------------------------------------------------------------
  // A fragment of m-block mb, step j: row wm*128 + mb*32 + r, logical piece g*4 + j
  int a_row_off[kMBW], a_row_sw[kMBW];
#pragma unroll
  for (int mb = 0; mb < kMBW; ++mb) {
    const int row = wm * (32 * kMBW) + mb * 32 + r;
    a_row_off[mb] = row * 128;
    a_row_sw[mb] = a_swz(row);
  }
  // packed B of n-block nb: row wn*128 + nb*32 + r, the half of the row that belongs to group g
  int b_off[kNBW][kBPiecesPerRow / 2];
  int w_row[kNBW];
#pragma unroll
  for (int nb = 0; nb < kNBW; ++nb) {
    const int row = wn * (32 * kNBW) + nb * 32 + r;
    w_row[nb] = min(n0 + row, N - 1);
#pragma unroll
    for (int h = 0; h < kBPiecesPerRow / 2; ++h) {
      const int piece = g * (kBPiecesPerRow / 2) + h;
      b_off[nb][h] = kAStage + row * P::kBRowBytes + (b_piece_pos<kBPiecesPerRow>(row, piece) << 4);
    }
  }

  typename P::acc_t acc[kMBW][kNBW];
#pragma unroll
  for (int mb = 0; mb < kMBW; ++mb)
#pragma unroll
    for (int nb = 0; nb < kNBW; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mb][nb][i] = 0;

  // ---- fragment readers ---------------------------------------------------------------------
  using frag_t = typename P::frag_t;
  auto read_a = [&](const unsigned char* base, int j, frag_t (&af)[kMBW]) {
#pragma unroll
    for (int mb = 0; mb < kMBW; ++mb)
      af[mb] = *reinterpret_cast<const frag_t*>(base + a_row_off[mb] + ((((g << 2) + j) ^ a_row_sw[mb]) << 4));
  };
  auto read_b = [&](const unsigned char* base, uint32_t (&bw)[kNBW][kBWords]) {
#pragma unroll
    for (int nb = 0; nb < kNBW; ++nb)
#pragma unroll
      for (int h = 0; h < kBPiecesPerRow / 2; ++h) {
        const uint4_t v = *reinterpret_cast<const uint4_t*>(base + b_off[nb][h]);
        bw[nb][4 * h + 0] = v[0]; bw[nb][4 * h + 1] = v[1]; bw[nb][4 * h + 2] = v[2]; bw[nb][4 * h + 3] = v[3];
      }
  };

  // ---- prologue: tiles 0 and 1 in LDS, tile 2 in registers, fragments of (tile 0, step 0) ready --
  // Three LDS stages.  During iteration kb: tile kb+2 goes registers -> stage (kb+2)%3 (last read in
  // iteration kb-1, protected by the barrier that ended it), tile kb+3 goes global -> registers, tile
  // kb is multiplied out of stage kb%3, and during its last step the first fragments of tile kb+1 are
  // already fetched from stage (kb+1)%3 (written in iteration kb-1): one barrier per iteration and the
  // LDS -> register -> MFMA pipeline never drains.
  typename P::ScaleRaw sc_raw1[kNBW], sc_raw2[kNBW];  // raw scales of tiles kb+1 and kb+2
  typename P::Scale sc_c[kNBW], sc_n[kNBW];
  load_tile(0);
#pragma unroll
  for (int nb = 0; nb < kNBW; ++nb) {
    sc_c[nb] = P::prep_scale(P::fetch_scale(p, w_row[nb], kh, g), p);
    sc_raw1[nb] = P::fetch_scale(p, w_row[nb], (KB > 1 ? 1 : 0) * kKSplit + kh, g);
  }
  store_tile(0);
  if (KB > 1) {
    load_tile(1);
    store_tile(1);
  }
  if (KB > 2) load_tile(2);
  __syncthreads();

  uint32_t bw_c[kNBW][kBWords], bw_n[kNBW][kBWords];
  frag_t af_c[kMBW], bf_c[kNBW], af_n[kMBW], bf_n[kNBW];
  read_b(smem, bw_c);
  read_a(smem, 0, af_c);
#pragma unroll
  for (int nb = 0; nb < kNBW; ++nb) bf_c[nb] = P::decode(bw_c[nb], 0, sc_c[nb]);

  int stage = 0;
  for (int kb = 0; kb < KB; ++kb) {
    const int stage1 = stage == 2 ? 0 : stage + 1;
    const int stage2 = stage1 == 2 ? 0 : stage1 + 1;
    const unsigned char* base = smem + stage * kStage;
    const unsigned char* base_n = smem + stage1 * kStage;
    if (kb + 2 < KB) {
      store_tile(stage2);
#pragma unroll
      for (int nb = 0; nb < kNBW; ++nb) sc_raw2[nb] = P::fetch_scale(p, w_row[nb], (kb + 2) * kKSplit + kh, g);
    }
    if (kb + 3 < KB) load_tile(kb + 3);
    const bool has_next = kb + 1 < KB;

#pragma unroll
    for (int j = 0; j < 4; ++j) {
      // fetch and decode the operands of the next step while this step's MFMAs run
      if (j < 3) {
        read_a(base, j + 1, af_n);
#pragma unroll
        for (int nb = 0; nb < kNBW; ++nb) bf_n[nb] = P::decode(bw_c[nb], j + 1, sc_c[nb]);
        if (j == 2 && has_next) read_b(base_n, bw_n);
      } else if (has_next) {
        read_a(base_n, 0, af_n);
#pragma unroll
        for (int nb = 0; nb < kNBW; ++nb) {
          sc_n[nb] = P::prep_scale(sc_raw1[nb], p);
          bf_n[nb] = P::decode(bw_n[nb], 0, sc_n[nb]);
        }
      }
#pragma unroll
      for (int mb = 0; mb < kMBW; ++mb)
#pragma unroll
        for (int nb = 0; nb < kNBW; ++nb) acc[mb][nb] = P::mfma(af_c[mb], bf_c[nb], acc[mb][nb]);
#pragma unroll
      for (int q = 0; q < kMBW; ++q) af_c[q] = af_n[q];
#pragma unroll
      for (int q = 0; q < kNBW; ++q) bf_c[q] = bf_n[q];
    }
#pragma unroll
    for (int nb = 0; nb < kNBW; ++nb) {
      sc_c[nb] = sc_n[nb];
      sc_raw1[nb] = sc_raw2[nb];
#pragma unroll
      for (int w = 0; w < kBWords; ++w) bw_c[nb][w] = bw_n[nb][w];
    }
    stage = stage1;
    __syncthreads();
  }

  if constexpr (kKSplit == 2) {
    // the second copy hands its accumulators to the first: [wave][mb][nb][lane] behind the epilogue's slabs
    constexpr int kSlabBytes = 4 * 32 * (32 * kNBW + 4) * 4;
    typename P::acc_t* red = reinterpret_cast<typename P::acc_t*>(smem_all + ((kSlabBytes + 63) & ~63)) + wave * (kMBW * kNBW * 64) + lane;
    if (kh == 1) {
#pragma unroll
      for (int mb = 0; mb < kMBW; ++mb)
#pragma unroll
        for (int nb = 0; nb < kNBW; ++nb) red[(mb * kNBW + nb) * 64] = acc[mb][nb];
    }
    __syncthreads();  // (the loop's last barrier already saw every wave done with the stages this area overlays)
    if (kh == 1) return;
#pragma unroll
    for (int mb = 0; mb < kMBW; ++mb)
#pragma unroll
      for (int nb = 0; nb < kNBW; ++nb) acc[mb][nb] = acc[mb][nb] + red[(mb * kNBW + nb) * 64];
  }
  {
    unsigned char* const smem = smem_all;  // the slabs of the epilogue start at the front
    DQ_GEMM_EPILOGUE
  }
}

// A policy may declare `static constexpr bool kBFragments = true`: its packed B was re-ordered offline into the
// matrix instruction's operand order, B[(N + 31) / 32][K / kKPerBlock][64 lanes][16 bytes] (lane 32 h + r of a
// block: bytes 16 h .. 16 h + 15 of that k-block of row r of the block of 32; 32-byte B rows only).  Read by the
// direct-to-LDS kernel: a B load is then 1 KiB contiguous and lands in LDS as the operand it is.
template <class P, class = void>
struct BFragments : std::false_type {};
template <class P>
struct BFragments<P, std::void_t<decltype(P::kBFragments)>> : std::integral_constant<bool, P::kBFragments> {};

// ---- direct-to-LDS variant ---------------------------------------------------------------------
// For policies whose A needs no transform on its way to LDS (any per-fragment transform is P::fix_a,
// applied after the fragment is read) and whose scales are absent, one byte per 32 k or one fp16 (plus
// one fp16 zero) per 128 k (P::kScaleDma): the A and packed-B tiles, and the scales, travel
// global -> LDS with global_load_lds_dwordx4 / _dword, two tiles ahead of the MFMAs, without
// passing through registers.  A lane's 16 bytes land at LDS base + lane * 16 whatever its source
// address, so the XOR swizzle of the A rows is applied by permuting the SOURCE addresses.  These
// loads are issued from inline assembly and tracked by hand (one s_waitcnt vmcnt per tile): the
// kernel issues no other vector-memory load inside the main loop, so the counter only ever
// holds these.  Requires K % 128 == 0 and A, B smaller than 4 GiB (32-bit lane offsets).
//
// M0 is written inside the statement and is not on its clobber list: clang treats M0 as a reserved register,
// warns that a reserved register on a clobber list "may not be preserved" and promises nothing for it.  What
// keeps this sound is that the statement sets M0 itself immediately before the one instruction that reads it,
// and that nothing else in these kernels depends on M0 across the statement: they use no other LDS-direct load,
// no GWS / sendmsg, no indirect register indexing and no v_readlane / v_writelane with M0 as the lane select,
// and gfx950 LDS instructions do not read M0 (that was the pre-gfx9 bounds clamp).
__device__ __forceinline__ void dma16(unsigned lds_addr, unsigned voff, const void* sbase) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\t" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
}
__device__ __forceinline__ void dma4(unsigned lds_addr, unsigned voff, const void* sbase) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2\n\t" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
}

// kMBW = 4: 256 x 256 tile, one workgroup per CU (the default).  kMBW = 2: 128 x 256 tile, two
// workgroups per CU (76 KiB of LDS and 256 registers each) that fill each other's barrier stalls;
// measured 13 % slower on the 4096 x 8192 x 8192 MXFP4 problem (twice the decode work per MFMA,
// and the 256-register budget spills), so it is kept as a build option only.  kNBW = 2: the same
// 256 x 256 tile on eight waves (two per SIMD, wave tile 128 x 64): no spills and the same decode work,
// but every A fragment is read from LDS by twice as many waves; measured 4 % slower on that
// problem (410 us against 393 us), also a build option only (-DDQ_DMA_NBW=2).  Eight waves of 64 x 128
// (four along the rows, which keeps the LDS traffic of the four-wave form) measured the same 410 us: a
// second wave per SIMD does not buy MFMA issue slots here.
//
// kWavesM = 1 (with kMBW = 8, kNBW = 2): the same 256 x 256 tile on four waves side by side, each 256 rows x 64
// columns.  A wave then decodes only the 64 weight rows it alone multiplies (with two rows of waves every packed
// word is decoded twice per workgroup) and reads every A fragment of the tile instead: half the decode
// instructions, twice the LDS reads of A.  For policies whose decode keeps a lone wave's instruction issue busier
// than its matrix pipe (P::kTallWaves).
template <class P, int kMBW, int kNBW, int kWavesM = 2>
__global__ __launch_bounds__(64 * kWavesM * (8 / kNBW), 32 * kMBW * kWavesM == 128 ? 2 : 1) void gemm_kernel_dma(const Params p_in) {
  Params p = p_in;
  int bid = blockIdx.x;
  take_k_slice<P>(p, bid);
  extern __shared__ __align__(16) unsigned char smem[];
  static_assert(P::kBRowBytes == 32 || P::kBRowBytes == 64, "direct-to-LDS variant: 32 or 64 packed bytes per weight row per tile");
  static_assert(kWavesM == 2 ? (kMBW == 2 || kMBW == 4) : (kWavesM == 1 && kMBW == 8 && kNBW == 2), "wave tile of 64, 128 or 256 rows");
  static_assert(kNBW == 2 || kNBW == 4, "wave tile of 64 or 128 columns");
  constexpr int kWavesN = 8 / kNBW;            // waves across the 256 tile columns
  constexpr int kWaves = kWavesM * kWavesN;    // 4, or 8 (two per SIMD)
  constexpr int BM = 32 * kMBW * kWavesM;      // shadows the 256-row default
  constexpr int kAStage = BM * kARowBytes;     // 32 or 16 KiB
  constexpr int kAOps = BM / 8 / kWaves;       // A DMA instructions per wave per tile
  constexpr int kBPiecesPerRow = P::kBRowBytes / 16;          // 2 or 4
  constexpr int kBRot = kBPiecesPerRow == 2 ? 3 : 2;          // piece rotation advances every 8 or 4 rows
  constexpr int kBOps = BN * kBPiecesPerRow / 64 / kWaves;    // packed-B DMA instructions per wave per tile
  constexpr int kBStage = BN * P::kBRowBytes;  // 8 KiB
  constexpr int kStage = kAStage + kBStage;    // 40 or 24 KiB
  constexpr int kStages = 3;
  // A packed-B row of one tile is 32 bytes, a quarter of a cache line, and the next tile's row is the next 32:
  // the B loads of tiles t and t + 1 (t even) are issued as pairs, the same instruction for t and then for t + 1,
  // which halves the lines the B stream asks the L2 for.  Tile t + 1 then lands three iterations before it is
  // read, which takes a fourth B slot, so B gets a ring of its own behind the three A stages: kPairB.  Policies
  // with 64-byte rows keep A and B side by side in three stages (a fourth 16 KiB slot would not fit).
  constexpr bool kPairB = P::kBRowBytes == 32 && BM == 256 && kWaves == 4;
  constexpr int kBRing = kPairB ? kStages * kAStage : kAStage;       // where B of slot 0 starts
  constexpr int kBSlot = kPairB ? kBStage : kStage;                  // distance between B slots
  constexpr int kAStride = kPairB ? kAStage : kStage;                // distance between A stages
  // Scales that travel by DMA (P::kScaleDma): 1 = one byte per 32 k (a dword per row covers a pair of tiles),
  // 2 = one fp16 per group of 64 .. 4096 k (a dword per row covers two groups: four tiles at group 128), 3 = the same
  // for scales and for zeros.
  // Ring: 4 slots x 1 KiB (256 rows x one dword), a second ring for the zeros.
  constexpr int kRing = kPairB ? kStages * kAStage + 4 * kBStage : kStages * kStage;
  constexpr int kSOps = P::kScaleDma == 0 ? 0 : (P::kScaleDma == 3 ? 2 : 1);  // scale DMA instructions per wave per tile
  constexpr int kBWords = P::kBRowBytes / 8;   // dwords per lane and 32-row block: 4 or 8
  constexpr bool kBFrag = BFragments<P>::value;
  static_assert(!kBFrag || (P::kBRowBytes == 32 && kWaves == 4), "fragment-ordered B: 32-byte rows, four waves");

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / kWavesN, wn = wave % kWavesN;
  const int g = lane >> 5, r = lane & 31;
  const int M = p.M, N = p.N, K = p.K;

  int tm, tn;
  tile_of_block(bid, p.tiles_m, p.tiles_n, tm, tn);
  const int m0 = tm * BM, n0 = tn * BN;
  const int KB = K / P::kKPerBlock;
  const unsigned lds0 = (unsigned)(size_t)smem;  // LDS byte address of the dynamic segment

  // ---- per-lane source offsets: LDS chunk c (16 bytes) of a tile <- which global 16 bytes --------
  unsigned a_voff[kAOps], b_voff[kBOps];
#pragma unroll
  for (int i = 0; i < kAOps; ++i) {
    const int c = (wave * kAOps + i) * 64 + lane;  // A chunk: row c / 8, physical piece c % 8
    const int row = c >> 3, pp = c & 7;
    a_voff[i] = (unsigned)min(m0 + row, M - 1) * (unsigned)(p.ldk * (kARowBytes / P::kKPerBlock)) + (unsigned)((pp ^ a_swz(row)) << 4);
  }
#pragma unroll
  for (int i = 0; i < kBOps; ++i) {
    const int c = (wave * kBOps + i) * 64 + lane;  // B chunk: row c / pieces per row, physical piece c % pieces per row
    const int row = c / kBPiecesPerRow, pp = c % kBPiecesPerRow;
    // LDS position (piece + rotation) % pieces holds source piece `piece`
    b_voff[i] = (unsigned)min(n0 + row, N - 1) * (unsigned)(p.ldk * P::kBRowBytes / P::kKPerBlock) +
                (unsigned)(((pp - (row >> kBRot)) & (kBPiecesPerRow - 1)) << 4);
    if constexpr (kBFrag) {
      // instruction (wave, i) brings the 32-row block wave * kBOps + i of the tile: 1 KiB as stored, lane-linear
      const int blk = min((n0 >> 5) + wave * kBOps + i, ((N + 31) >> 5) - 1);
      b_voff[i] = (unsigned)blk * (unsigned)(p.ldk / P::kKPerBlock) * 1024u + (unsigned)lane * 16u;
    }
  }
  // fp16 scales (kScaleDma >= 2): one per 2^p0 k (p.p0 = 5 .. 12, the policy's dma_ok checks it), so a dword of a row
  // serves 2^s_ps tiles of 64 k.  Groups of 32 k (one tile per dword, the two k halves of a tile in different groups)
  // need the scales issued with every tile: not the kPairB form, which dma_eligible keeps them away from
  const int s_gshift = P::kScaleDma >= 2 ? p.p0 : 7;
  const int s_ps = s_gshift - 5;
  const unsigned s_voff = (unsigned)min(n0 + (tid & 255), N - 1) * (unsigned)(P::kScaleDma == 1 ? (K >> 5) : ((K >> s_gshift) << 1));  // waves 4..7 repeat 0..3

  // One tile = kSOps + kAOps + kBOps DMA instructions per thread: first the scale dword(s) (row tid; issued
  // with every tile although a dword serves two or four, which keeps the loop branch-free), then the A
  // chunks, then the packed-B chunks.
  constexpr int kTileOps = kSOps + kAOps + kBOps;
  auto issue_op = [&](int op, int kb, int stage) {
    const unsigned sbase = lds0 + stage * kAStride;
    const unsigned bbase = lds0 + kBRing + (kPairB ? (kb & 3) : stage) * kBSlot;
    if (op < kSOps) {
      if constexpr (P::kScaleDma == 1) {
        const int pair = kb >> 1;
        dma4(lds0 + kRing + (pair & 3) * 1024 + (wave & 3) * 256, s_voff, (const unsigned char*)p.S + (size_t)pair * 4);
      } else if constexpr (P::kScaleDma >= 2) {
        const int quad = kb >> s_ps;
        dma4(lds0 + kRing + op * 4096 + (quad & 3) * 1024 + (wave & 3) * 256, s_voff,
             (const unsigned char*)(op == 0 ? p.S : p.Z) + (size_t)quad * 4);
      }
    } else if (op < kSOps + kAOps) {
      const int i = op - kSOps;
      dma16(sbase + (wave * kAOps + i) * 1024, a_voff[i], (const unsigned char*)p.A + (size_t)kb * 128);
    } else {
      const int i = op - kSOps - kAOps;
      dma16(bbase + (wave * kBOps + i) * 1024, b_voff[i], (const unsigned char*)p.B + (size_t)kb * (kBFrag ? 1024 : P::kBRowBytes));
    }
  };
  constexpr int kWaitOps = kTileOps;  // outstanding DMA instructions of one tile

  // ---- fragment read offsets (same LDS geometry as the register-staged kernel) --------------------
  int a_row_off[kMBW], a_row_sw[kMBW], b_off[kNBW][kBPiecesPerRow / 2], s_off[kNBW];
#pragma unroll
  for (int mb = 0; mb < kMBW; ++mb) {
    const int row = wm * (32 * kMBW) + mb * 32 + r;
    a_row_off[mb] = row * 128;
    a_row_sw[mb] = a_swz(row);
  }
#pragma unroll
  for (int nb = 0; nb < kNBW; ++nb) {
    const int row = wn * (32 * kNBW) + nb * 32 + r;
#pragma unroll
    for (int h = 0; h < kBPiecesPerRow / 2; ++h) {
      const int piece = g * (kBPiecesPerRow / 2) + h;
      b_off[nb][h] = row * P::kBRowBytes + (((piece + (row >> kBRot)) & (kBPiecesPerRow - 1)) << 4);  // in its B slot
      // fragment order: block row / 32 of the tile, then the lanes as the matrix instruction numbers them
      if constexpr (kBFrag) b_off[nb][h] = (row >> 5) * 1024 + lane * 16;
    }
    s_off[nb] = kRing + row * 4 + (P::kScaleDma == 1 ? g : (P::kScaleDma >= 2 && s_gshift == 5 ? 2 * g : 0));
  }
  using frag_t = typename P::frag_t;
  auto read_a1 = [&](const unsigned char* base, int j, int mb) -> frag_t {
    return P::fix_a(*reinterpret_cast<const frag_t*>(base + a_row_off[mb] + ((((g << 2) + j) ^ a_row_sw[mb]) << 4)));
  };
  // 32 rows further down the rotation of the packed-B pieces repeats ((32 >> kBRot) % kBPiecesPerRow == 0)
  // and the scale rows are 4 bytes apart: block nb sits at a constant distance from block 0, so one
  // address per tile serves all kNBW reads through their immediate offsets
  static_assert((32 >> kBRot) % kBPiecesPerRow == 0, "B rotation must repeat every 32 rows");
  auto read_b1 = [&](const unsigned char* base, int nb, uint32_t (&bw)[kBWords]) {
#pragma unroll
    for (int h = 0; h < kBPiecesPerRow / 2; ++h) {
      const uint4_t v = *reinterpret_cast<const uint4_t*>(base + b_off[0][h] + nb * (32 * P::kBRowBytes));
      bw[4 * h + 0] = v[0]; bw[4 * h + 1] = v[1]; bw[4 * h + 2] = v[2]; bw[4 * h + 3] = v[3];
    }
  };
  // the LDS read of a scale and the arithmetic on it are separate steps, so that the read can be issued a
  // chunk ahead of its first use
  auto read_scale_byte = [&](int kb, int nb) -> int {
    if constexpr (P::kScaleDma == 1) return (smem + s_off[0] + ((kb >> 1) & 3) * 1024 + (kb & 1) * 2)[nb * 128];
    else return 0;
  };
  auto read_scale1 = [&](int kb, int nb) -> typename P::Scale {
    if constexpr (P::kScaleDma >= 2) {
      // which of the dword's two groups: with groups of 32 k the lane's half of the tile (in s_off), else the tile's
      const unsigned char* at = smem + s_off[0] + ((kb >> s_ps) & 3) * 1024 + (s_gshift == 5 ? 0 : (((kb << 6) >> s_gshift) & 1) * 2) + nb * 128;
      return P::ring_scale(at, at + 4096);
    } else {
      return P::prep_scale(read_scale_byte(kb, nb), p);
    }
  };

  typename P::acc_t acc[kMBW][kNBW];
#pragma unroll
  for (int mb = 0; mb < kMBW; ++mb)
#pragma unroll
    for (int nb = 0; nb < kNBW; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mb][nb][i] = 0;

  // ---- prologue: tiles 0 and 1 (and their scales) in flight; only tile 0 has to have landed -------
  if constexpr (kPairB) {  // scales, A of tile 0, the B pairs of tiles 0 and 1, then A of tile 1
#pragma unroll
    for (int op = 0; op < kSOps + kAOps; ++op) issue_op(op, 0, 0);
#pragma unroll
    for (int i = 0; i < kBOps; ++i) {
      issue_op(kSOps + kAOps + i, 0, 0);
      issue_op(kSOps + kAOps + i, 1, 1);
    }
#pragma unroll
    for (int op = kSOps; op < kSOps + kAOps; ++op) issue_op(op, 1, 1);
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kAOps) : "memory");
  } else {
#pragma unroll
    for (int op = 0; op < kTileOps; ++op) issue_op(op, 0, 0);
#pragma unroll
    for (int op = 0; op < kTileOps; ++op) issue_op(op, 1, 1);  // KB >= 2 because K % 128 == 0
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kWaitOps) : "memory");
  }
  __syncthreads();

  typename P::Scale sc_c[kNBW];
  uint32_t bw_c[kNBW][kBWords];
  frag_t af_c[kMBW], bf_c[kNBW], af_n[kMBW], bf_n[kNBW];

  // One iteration = tile kb out of `stage`, as 16 chunks of 4 MFMAs (one A fragment against the four
  // B fragments) kept in order by scheduling barriers; every chunk carries side work that issues in
  // the shadow of its MFMAs.  The loop is skewed by one MFMA step so that nothing waits on LDS right
  // after the barrier:
  //   chunks  0..3   MFMAs of step 3 of tile kb-1 (operands already in registers); side work: read
  //                  the packed B words, the scales and the step-0 A fragments of tile kb, decode step 0
  //   chunks  4..15  MFMAs of steps 0..2 of tile kb; side work: read / decode the operands of the next
  //                  step (the step-3 operands stay in registers for the next iteration)
  //   chunks  0..10  also issue one DMA instruction each of tile kb+2 into stage (kb+2) % 3, which
  //                  was last read in iteration kb-1 and is free since the barrier that ended it.
  // Tile kb+2 is not read before iteration kb+2: its loads have almost two iterations to land.
  // A chunk with its side work cut into four pieces, one behind each of the chunk's four MFMAs, each piece
  // fenced by scheduling barriers: left to itself the scheduler issues one MFMA, then all of the side work
  // (about 50 cycles, longer than the 32 the MFMA runs), then the other three back to back, and the matrix
  // pipe idles once per chunk.
  auto chunk4 = [&](int q, auto do_mfma_tag, auto&& side_a, auto&& side_b, auto&& side_c, auto&& side_d) {
    constexpr bool do_mfma = decltype(do_mfma_tag)::value;
    if constexpr (do_mfma) acc[q][0] = P::mfma(af_c[q], bf_c[0], acc[q][0]);
    side_a();
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (do_mfma) acc[q][1] = P::mfma(af_c[q], bf_c[1], acc[q][1]);
    side_b();
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (do_mfma) acc[q][2] = P::mfma(af_c[q], bf_c[2], acc[q][2]);
    side_c();
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (do_mfma) acc[q][3] = P::mfma(af_c[q], bf_c[3], acc[q][3]);
    side_d();
    __builtin_amdgcn_sched_barrier(0);
  };

  // odd_tag: tile kb is odd (only looked at with kPairB, where even iterations issue the B pairs of tiles
  // kb + 2 and kb + 3, the scales and A of tile kb + 2, and odd iterations A of tile kb + 2 only)
  auto iteration = [&](int kb, int stage, auto first_tag, auto next2_tag, auto odd_tag) {
    constexpr bool first = decltype(first_tag)::value;
    constexpr bool has_next2 = decltype(next2_tag)::value;
    constexpr bool odd = decltype(odd_tag)::value;
    const int stage2 = stage == 0 ? 2 : stage - 1;  // (stage + 2) % 3
    const unsigned char* base = smem + stage * kAStride;
    const unsigned char* bbase = smem + kBRing + (kPairB ? (kb & 3) : stage) * kBSlot;
    constexpr int kIterOps = !kPairB ? kTileOps : (odd ? kAOps : kSOps + kAOps + 2 * kBOps);  // issued per iteration
    if constexpr ((kMBW == 4 && kNBW == 4) || kWavesM == 1) {
      using DoMfma = std::integral_constant<bool, !first>;
      auto dma = [&](int chunk) {
        if constexpr (!kPairB) {
          if (has_next2 && chunk < kTileOps) issue_op(chunk, kb + 2, stage2);
        } else if constexpr (odd) {
          if (has_next2 && chunk < kAOps) issue_op(kSOps + chunk, kb + 2, stage2);
        } else {
          if (has_next2 && chunk < kSOps + kAOps) issue_op(chunk, kb + 2, stage2);
          else if (has_next2 && chunk < kIterOps) {
            const int j = chunk - kSOps - kAOps;  // B instruction j / 2 of tile kb + 2 + j % 2
            issue_op(kSOps + kAOps + (j >> 1), kb + 2 + (j & 1), stage2);
          }
        }
      };
      int sc_byte[4];  // scale bytes are read in chunk 0 and turned into multipliers in chunk 1
      auto fetch_b = [&](int nb) {
        read_b1(bbase, nb, bw_c[nb]);
        if constexpr (P::kScaleDma >= 2) sc_c[nb] = read_scale1(kb, nb);
        else sc_byte[nb] = read_scale_byte(kb, nb);
      };
      auto finish_scale = [&](int nb) {
        if constexpr (P::kScaleDma < 2) sc_c[nb] = P::prep_scale(sc_byte[nb], p);
      };
      auto nothing = [] {};
      if constexpr (kWavesM == 1) {
        // Eight matrix instructions (four A fragments against the wave's two B fragments) and their side work per
        // scheduling region, as a pipeline of one matrix instruction, at most one LDS read and a few vector
        // instructions.  Skewed by one step like the 2 x 2 form below.
        constexpr int kValu = 3;
        auto region = [&](int q0, auto do_mfma_tag, auto&& side) {
          if constexpr (decltype(do_mfma_tag)::value) {
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
              for (int nb = 0; nb < 2; ++nb) acc[q0 + q][nb] = P::mfma(af_c[q0 + q], bf_c[nb], acc[q0 + q][nb]);
          }
          side();
#define DQ_SPREAD_GROUP                                  \
  __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);     \
  __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);     \
  __builtin_amdgcn_sched_group_barrier(0x002, kValu, 0);
          DQ_SPREAD_GROUP DQ_SPREAD_GROUP DQ_SPREAD_GROUP DQ_SPREAD_GROUP
          DQ_SPREAD_GROUP DQ_SPREAD_GROUP DQ_SPREAD_GROUP DQ_SPREAD_GROUP
#undef DQ_SPREAD_GROUP
          __builtin_amdgcn_sched_barrier(0);
        };
        region(0, DoMfma{}, [&] {
          fetch_b(0);
          fetch_b(1);
          dma(0);
          dma(1);
#pragma unroll
          for (int q = 0; q < 4; ++q) af_n[q] = read_a1(base, 0, q);
        });
        region(4, DoMfma{}, [&] {
#pragma unroll
          for (int q = 4; q < 8; ++q) af_n[q] = read_a1(base, 0, q);
          finish_scale(0);
          finish_scale(1);
          dma(2);
          dma(3);
          bf_n[0] = P::decode(bw_c[0], 0, sc_c[0]);
          bf_n[1] = P::decode(bw_c[1], 0, sc_c[1]);
        });
#pragma unroll
        for (int q = 0; q < 8; ++q) af_c[q] = af_n[q];
        bf_c[0] = bf_n[0];
        bf_c[1] = bf_n[1];
#pragma unroll
        for (int j = 0; j < 3; ++j) {
          region(0, std::true_type{}, [&] {
#pragma unroll
            for (int q = 0; q < 4; ++q) af_n[q] = read_a1(base, j + 1, q);
            dma(4 + 4 * j);
            dma(5 + 4 * j);
            bf_n[0] = P::decode(bw_c[0], j + 1, sc_c[0]);
          });
          region(4, std::true_type{}, [&] {
#pragma unroll
            for (int q = 4; q < 8; ++q) af_n[q] = read_a1(base, j + 1, q);
            dma(6 + 4 * j);
            dma(7 + 4 * j);
            bf_n[1] = P::decode(bw_c[1], j + 1, sc_c[1]);
          });
#pragma unroll
          for (int q = 0; q < 8; ++q) af_c[q] = af_n[q];
          bf_c[0] = bf_n[0];
          bf_c[1] = bf_n[1];
        }
      } else {
      chunk4(0, DoMfma{}, [&] { fetch_b(0); fetch_b(1); }, [&] { dma(0); }, [&] { fetch_b(2); fetch_b(3); },
             [&] { af_n[0] = read_a1(base, 0, 0); });
      chunk4(1, DoMfma{}, [&] { af_n[1] = read_a1(base, 0, 1); finish_scale(0); }, [&] { dma(1); },
             [&] { af_n[2] = read_a1(base, 0, 2); finish_scale(1); }, [&] { finish_scale(2); });
      chunk4(2, DoMfma{}, [&] { af_n[3] = read_a1(base, 0, 3); finish_scale(3); }, [&] { dma(2); },
             [&] { bf_n[0] = P::decode(bw_c[0], 0, sc_c[0]); }, [&] { bf_n[1] = P::decode(bw_c[1], 0, sc_c[1]); });
      chunk4(3, DoMfma{}, [&] { bf_n[2] = P::decode(bw_c[2], 0, sc_c[2]); }, [&] { dma(3); },
             [&] { bf_n[3] = P::decode(bw_c[3], 0, sc_c[3]); }, nothing);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        af_c[q] = af_n[q];
        bf_c[q] = bf_n[q];
      }
#pragma unroll
      for (int j = 0; j < 3; ++j) {
#pragma unroll
        for (int q = 0; q < 4; ++q)
          chunk4(q, std::true_type{}, [&] { af_n[q] = read_a1(base, j + 1, q); }, [&] { dma(4 + j * 4 + q); },
                 [&] { bf_n[q] = P::decode(bw_c[q], j + 1, sc_c[q]); }, nothing);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          af_c[q] = af_n[q];
          bf_c[q] = bf_n[q];
        }
      }
      }
    } else {
#pragma unroll
    for (int q = 0; q < kMBW; ++q) {
      if constexpr (kMBW == 4) {
        if (q == 0) {
#pragma unroll
          for (int nb = 0; nb < kNBW; ++nb) {
            read_b1(bbase, nb, bw_c[nb]);
            sc_c[nb] = read_scale1(kb, nb);
          }
        } else if (q == 1) {
          af_n[0] = read_a1(base, 0, 0);
          af_n[1] = read_a1(base, 0, 1);
        } else if (q == 2) {
          af_n[2] = read_a1(base, 0, 2);
          af_n[3] = read_a1(base, 0, 3);
#pragma unroll
          for (int nb = 0; nb < kNBW / 2; ++nb) bf_n[nb] = P::decode(bw_c[nb], 0, sc_c[nb]);
        } else {
#pragma unroll
          for (int nb = kNBW / 2; nb < kNBW; ++nb) bf_n[nb] = P::decode(bw_c[nb], 0, sc_c[nb]);
        }
      } else {
        if (q == 0) {
#pragma unroll
          for (int nb = 0; nb < kNBW; ++nb) {
            read_b1(bbase, nb, bw_c[nb]);
            sc_c[nb] = read_scale1(kb, nb);
          }
          af_n[0] = read_a1(base, 0, 0);
          af_n[1] = read_a1(base, 0, 1);
        } else {
#pragma unroll
          for (int nb = 0; nb < kNBW; ++nb) bf_n[nb] = P::decode(bw_c[nb], 0, sc_c[nb]);
        }
      }
      if (has_next2 && q < kTileOps) issue_op(q, kb + 2, stage2);
      if (!first) {
#pragma unroll
        for (int nb = 0; nb < kNBW; ++nb) acc[q][nb] = P::mfma(af_c[q], bf_c[nb], acc[q][nb]);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int q = 0; q < kMBW; ++q) af_c[q] = af_n[q];
#pragma unroll
    for (int q = 0; q < kNBW; ++q) bf_c[q] = bf_n[q];
#pragma unroll
    for (int j = 0; j < 3; ++j) {
#pragma unroll
      for (int q = 0; q < kMBW; ++q) {
        const int chunk = kMBW + j * kMBW + q;
        af_n[q] = read_a1(base, j + 1, q);
#pragma unroll
        for (int nb = 0; nb < kNBW; ++nb)  // the kNBW decodes of a step spread evenly over its kMBW chunks
          if (nb * kMBW / kNBW == q) bf_n[nb] = P::decode(bw_c[nb], j + 1, sc_c[nb]);
        if (has_next2 && chunk < kTileOps) issue_op(chunk, kb + 2, stage2);
#pragma unroll
        for (int nb = 0; nb < kNBW; ++nb) acc[q][nb] = P::mfma(af_c[q], bf_c[nb], acc[q][nb]);
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int q = 0; q < kMBW; ++q) af_c[q] = af_n[q];
#pragma unroll
      for (int q = 0; q < kNBW; ++q) bf_c[q] = bf_n[q];
    }
    }
    // tile kb+1 must have landed before the next iteration reads it; tile kb+2 (issued during this
    // iteration) may still be in flight
    if (has_next2) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kIterOps) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  };

  // KB is even (K % (2 kKPerBlock) == 0): tiles come in (even, odd) pairs
  using T = std::true_type;
  using F = std::false_type;
  int stage = 0;
  int kb = 0;
  auto next_stage = [&] { stage = stage == 2 ? 0 : stage + 1; };
  if (KB > 2) {
    iteration(0, 0, T{}, T{}, F{});
    stage = 1;
    for (kb = 1; kb + 3 < KB; kb += 2) {
      iteration(kb, stage, F{}, T{}, T{});
      next_stage();
      iteration(kb + 1, stage, F{}, T{}, F{});
      next_stage();
    }
    iteration(kb, stage, F{}, T{}, T{});  // kb = KB - 3
    next_stage();
    iteration(kb + 1, stage, F{}, F{}, F{});
    next_stage();
    iteration(kb + 2, stage, F{}, F{}, T{});
  } else {  // KB == 2
    iteration(0, 0, T{}, F{}, F{});
    iteration(1, 1, F{}, F{}, T{});
  }
  // step 3 of the last tile
#pragma unroll
  for (int q = 0; q < kMBW; ++q)
#pragma unroll
    for (int nb = 0; nb < kNBW; ++nb) acc[q][nb] = P::mfma(af_c[q], bf_c[nb], acc[q][nb]);

  DQ_GEMM_EPILOGUE
}

template <class P, int kMBW = 4, int kNBW = 4, int kKSplit = 1>
int launch(Params p, hipStream_t stream) {
  constexpr int kTileM = 64 * kMBW, kTileN = 64 * kNBW;
  constexpr int kPipe = kKSplit * 3 * (kTileM * kARowBytes + kTileN * P::kBRowBytes);
  // epilogue staging, and behind it the accumulators the second copy of the pipeline hands over
  constexpr int kSlabs = ((4 * 32 * (32 * kNBW + 4) * 4 + 63) & ~63) + (kKSplit - 1) * 4 * kMBW * kNBW * 64 * 64;
  constexpr int kLds = kPipe > kSlabs ? kPipe : kSlabs;
  static_assert(kLds <= 160 * 1024, "LDS budget");
  p.tiles_m = (p.M + kTileM - 1) / kTileM;
  p.tiles_n = (p.N + kTileN - 1) / kTileN;
  auto kern = gemm_kernel<P, kMBW, kNBW, kKSplit>;
  static bool lds_limit_raised[kMaxDevices];
  if (raise_lds_limit<kLds>(kern, lds_limit_raised)) return -1;
  hipLaunchKernelGGL(kern, dim3(p.tiles_m * p.tiles_n * p.split), dim3(kThreads * kKSplit), kLds, stream, p);
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

// Tile choice by how many workgroups the 256 CUs get: 256 x 256 when that already gives about one per
// CU, else 128 x 128, else 128 x 64 (a narrower N tile repeats the weight decode less than a
// narrower M tile would).
template <class P>
int launch_auto(const Params& p, hipStream_t stream) {
  auto tiles = [&](int bm, int bn) { return (long)((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn) * p.split; };
  if (tiles(256, 256) >= 192) return launch<P, 4, 4>(p, stream);
  if (tiles(128, 128) >= 192) return launch<P, 2, 2>(p, stream);
  // at most about one small tile per CU and a long K: two copies of the pipeline per workgroup, on alternate
  // k-blocks (int8 x 2-bit at M = 256, N = K = 8192: 35 -> 28.5 us).  Integer accumulation only: there the order
  // of the K sum does not show, while a float result would no longer match the other tile shapes bit for bit.
  if constexpr (P::kBRowBytes <= 64 && std::is_same<typename P::acc_t, int16_t_>::value) {
    if (tiles(128, 64) <= 320 && (p.K / P::kKPerBlock) % 2 == 0 && p.K / P::kKPerBlock >= 8) return launch<P, 2, 1, 2>(p, stream);
  }
  return launch<P, 2, 1>(p, stream);
}

template <class P>
bool dma_eligible(const Params& p) {
  // the direct-to-LDS kernel has one tile shape (256 x 256): small problems go to the tile-size choice above
  const long tiles = (long)((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN) * p.split;
  // 32-bit lane offsets: A rows are 128 bytes per K block, packed B rows kBRowBytes
  const size_t a_bytes = (size_t)p.M * (p.ldk / P::kKPerBlock) * kARowBytes;
  const size_t b_bytes = (size_t)p.N * (p.ldk / P::kKPerBlock) * P::kBRowBytes;
  // fp16 scales of groups of 32 k go with every tile: not with the pairwise issue of the 32-byte-row form of this tile
  const bool scales_per_tile = P::kScaleDma >= 2 && P::kBRowBytes == 32 && p.p0 == 5;
  return P::dma_ok(p) && !scales_per_tile && (p.K % (2 * P::kKPerBlock) == 0) && tiles >= 192 && a_bytes < (1ull << 32) &&
         b_bytes < (1ull << 32);
}

// Problems with too few 256 x 256 tiles for the kernel above but at least `min_tiles` tiles of 128 x 256: the same
// kernel on the half-height tile (two workgroups fit a CU), which keeps the operands on the direct-to-LDS path.
// Measured at N = K = 8192 against the register-staged 128 x 128 tiles, M = 1024: MXFP4 139 -> 114 us, fp16 x uint4
// 213 -> 158 us, int8 x 2-bit 68 -> 57 us, int8 x int4 75 -> 60 us; M = 384 (96 tiles): MXFP4 90 -> 85.5 us, fp16 x
// uint4 139 -> 117 us.  The int8 x 2-bit policy gains from 160 tiles on only (M = 512: 43.5 us register-staged
// against 48.8 us; M = 640: 61 against 49 us).
constexpr int kHalfTileMin = 96;
template <class P>
bool dma_half_eligible(const Params& p, int min_tiles = kHalfTileMin) {
  const long tiles = (long)((p.M + 127) / 128) * ((p.N + BN - 1) / BN) * p.split;
  const size_t a_bytes = (size_t)p.M * (p.ldk / P::kKPerBlock) * kARowBytes;
  const size_t b_bytes = (size_t)p.N * (p.ldk / P::kKPerBlock) * P::kBRowBytes;
  return !dma_eligible<P>(p) && P::dma_ok(p) && (p.K % (2 * P::kKPerBlock) == 0) && tiles >= min_tiles &&
         a_bytes < (1ull << 32) && b_bytes < (1ull << 32);
}

template <class P, int kMBW, int kNBW, int kWavesM = 2>
int launch_dma_tile(Params p, hipStream_t stream) {
  constexpr int kWaves = kWavesM * (8 / kNBW);
  constexpr int kTileM = 32 * kMBW * kWavesM;
  constexpr bool kPairB = P::kBRowBytes == 32 && kTileM == 256 && kWaves == 4;  // as in the kernel: a fourth B slot
  constexpr int kPipe = 3 * (kTileM * kARowBytes + BN * P::kBRowBytes) + (kPairB ? BN * P::kBRowBytes : 0) + 8 * 1024;
  constexpr int kSlabs = kWaves * 32 * (32 * kNBW + 4) * 4;  // epilogue staging
  constexpr int kLds = kPipe > kSlabs ? kPipe : kSlabs;
  p.tiles_m = (p.M + kTileM - 1) / kTileM;
  p.tiles_n = (p.N + BN - 1) / BN;
  auto kern = gemm_kernel_dma<P, kMBW, kNBW, kWavesM>;
  static bool lds_limit_raised[kMaxDevices];
  if (raise_lds_limit<kLds>(kern, lds_limit_raised)) return -1;
  hipLaunchKernelGGL(kern, dim3(p.tiles_m * p.tiles_n * p.split), dim3(64 * kWaves), kLds, stream, p);
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

// P::kTallWaves: the four waves side by side (see the kernel)
template <class P, class = void>
struct TallWaves : std::false_type {};
template <class P>
struct TallWaves<P, std::void_t<decltype(P::kTallWaves)>> : std::integral_constant<bool, P::kTallWaves> {};

template <class P>
int launch_dma(const Params& p, hipStream_t stream) {
  if constexpr (TallWaves<P>::value) return launch_dma_tile<P, 8, 2, 1>(p, stream);
  else return launch_dma_tile<P, DQ_DMA_MBW, DQ_DMA_NBW>(p, stream);
}

template <class P>
int launch_dma_half(const Params& p, hipStream_t stream) {
  return launch_dma_tile<P, 2, 4>(p, stream);
}

// The tile choice of every policy that can take the direct-to-LDS path: 256 x 256 tiles there when the problem has
// enough of them, else 128 x 256 tiles there, else the register-staged kernel with the tile size launch_auto picks.
template <class P>
int launch_best(const Params& p, hipStream_t stream, int half_tile_min = kHalfTileMin) {
  if (dma_eligible<P>(p)) return launch_dma<P>(p, stream);
  if (dma_half_eligible<P>(p, half_tile_min)) return launch_dma_half<P>(p, stream);
  return launch_auto<P>(p, stream);
}

inline Params make_params(const void* A, const void* B, const void* S, const void* Z, const void* Bias, void* C, int M,
                          int N, int K) {
  Params p{};
  p.A = A; p.B = B; p.S = S; p.Z = Z; p.Bias = Bias; p.C = C;
  p.M = M; p.N = N; p.K = K;
  p.ldk = K;
  p.split = 1;
  p.tiles_m = (M + BM - 1) / BM;
  p.tiles_n = (N + BN - 1) / BN;
  return p;
}

// ---- building blocks shared by the policies -------------------------------------------------------

struct NoScale {
  static constexpr int kScaleDma = 0;  // no scales to bring in by DMA
  static bool dma_ok(const Params&) { return true; }
  struct ScaleRaw {};
  struct Scale {};
  __device__ static __forceinline__ ScaleRaw fetch_scale(const Params&, int, int, int) { return {}; }
  __device__ static __forceinline__ Scale prep_scale(ScaleRaw, const Params&) { return {}; }
};

struct PlainA {
  static constexpr bool kAPacked = false;
  static constexpr bool kPlainA = true;  // stage_a is the identity: A may go global -> LDS directly
  __device__ static __forceinline__ uint4_t stage_a(uint4_t v) { return v; }
  __device__ static __forceinline__ void expand_a(uint4_t, uint4_t&, uint4_t&) {}
  // direct-to-LDS kernel: transform of an A fragment after it is read from LDS (A lands untouched)
  template <class F>
  __device__ static __forceinline__ F fix_a(F f) { return f; }
};

}  // namespace gemm
}  // namespace dq
