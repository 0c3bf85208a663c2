// BitNet W2A8 GEMM for a few hundred activation rows on gfx950: K sliced over the eight waves of a workgroup.
//
// Replaces the prefill kernel of examples/bitnet-1.58b/kernel_benchmark/tilelang_bitnet_158_int8xint2_prefill.py:72-298
// (decoder decode_i2{u,s}_to_i8s, examples/dequantize_gemm/quantize/lop3.py:950-997; epilogue
// examples/bitnet-1.58b/utils_quant.py:165-170) where M x N gives every CU about one small output tile with the whole
// of K behind it: M = 256, N = K = 8192 is 256 tiles of 64 x 128, each a chain of 8192 k.
//
// A tiled kernel walks that chain with every wave of the workgroup in step: per 128 k a barrier, the activations
// written to LDS once and read by every wave that shares their rows, the packed weights decoded by every wave that
// shares their columns.  Here a wave owns the whole 64 x 128 tile (8 accumulators of 32 x 32, 128 registers) over one
// eighth of K, so nothing is shared and nothing waits for another wave until the eight partial sums meet:
//
//   * activations travel global -> LDS with global_load_lds_dwordx4, a block of 128 k (64 rows x 128 bytes: eight
//     instructions of 8 whole lines each) at a time into two stages of the wave's own, without passing through
//     registers.  A lane's 16 bytes land at stage + lane * 16 whatever its source address, so the bank swizzle (piece
//     p of row n at position p ^ ((n >> 1) & 7) of the row's eight) is applied by permuting the source addresses.  A
//     block's eight fragments are read into registers at its start, which frees its stage for the block after the
//     next.  No other wave touches the stages: the main loop has no barrier.
//   * weights: a load instruction that puts 32 different rows into adjacent lanes costs the load unit as much as four
//     that read whole lines (it handles a row per step, whatever the row's share of the instruction), and with 32
//     bytes per row and block that alone took as long as the matrix instructions.  So a weight load covers 16 rows x
//     64 bytes (two blocks of 128 k; lane l: row l / 4, piece l % 4), two loads X, Y per block of 32 rows, two to
//     four blocks ahead in registers; one ds_bpermute_b32 per dword regroups the lanes of a register as
//     [k half h][block b][row] and one v_permlane16_swap_b32 per dword pair exchanges the odd quarters of X with the
//     even quarters of Y, which leaves the operand of block 0 (rows 0..31 x halves 0, 1) in one register and that of
//     block 1 in the other.  Dword s of an operand feeds step s: the contraction index of step s is labelled
//     k = 64 h + 16 s + e for both operands, i.e. piece 4 h + s of an activation row's 128 bytes.
//   * both streams are issued from inline assembly and tracked by hand: loads return in order, every issue point
//     issues the same number of loads (past the end of the slice: the last block again, unused), and one
//     s_waitcnt vmcnt per block lets the loads that are younger than the ones needed stay in flight.
//   * decode: 7 instructions per 16 weights.  Signed codes are moved to the top two bits of their byte, where the
//     int8 reading of the byte is 64 sext2(c) (offset binary: c - 2 = sext2(c ^ 2), the flip in the same three-input
//     bit operation as the mask); the accumulators then hold 64 x the sum and are shifted back once, exactly.
//     Unsigned codes are masked in place.
//   * the matrix instruction takes the weights as its row operand, so a lane's four consecutive accumulator values
//     are four consecutive output columns of one row: the partial sums go to LDS as 16-byte pieces and come back as
//     two pieces (8 columns) per lane, summed over the eight K slices in integer arithmetic (any order is exact),
//     finished by the epilogue and stored 16 bytes (fp16) or 32 bytes (int32) per lane.
//
//   * FRAG: the weights were re-ordered offline into the operand order, B[(N + 31) / 32][K / 128][64 lanes][16 bytes]
//     (lane 32 h + r of block (nb, kb): bytes 32 kb + 16 h .. + 15 of row 32 nb + r, rows past N zero).  A load is then
//     1 KiB contiguous, lands as the operand it is, and nothing is regrouped; same loads at the same points of the loop.
//
// Rows beyond M or N are read as the last row (their results are not stored).
#include <type_traits>
#include <utility>

#include "dq_common.h"
#include "dq_i2_codes.h"

namespace dq {

namespace {

template <int... I, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

constexpr int kMB = 2, kNB = 4;             // wave (= workgroup) tile: 64 rows x 128 columns
constexpr int kTileM = 32 * kMB, kTileN = 32 * kNB;
constexpr int kWaves = 8;                   // K slices
constexpr int kStage = kTileM * 128;        // 8 KiB: 64 activation rows x 128 k
constexpr int kStages = 2;
constexpr int kWaveLds = kStages * kStage;
constexpr int kLds = kWaves * kWaveLds;     // 128 KiB; the partial sums (8 x 32 KiB, in two rounds of 128 KiB) reuse it
constexpr int kAOps = kTileM / 8;           // activation loads per block: 8 rows x 128 bytes each
constexpr int kWOps = 2 * kNB;              // weight loads per pair of blocks

// M0 is written inside the statement and is not on its clobber list (clang treats it as reserved); the statement sets
// it immediately before the one instruction that reads it and nothing else in this kernel depends on M0.
__device__ __forceinline__ void dma16(unsigned lds_addr, unsigned voff, const void* sbase) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\t" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
}
// The destination is written when the load returns, not when the statement ends: nothing may read it before a
// wait_loads that names it.
__device__ __forceinline__ void load16(uint4_t& dst, unsigned voff, const void* sbase) {
  asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(dst) : "v"(voff), "s"(sbase) : "memory");
}
// Names every weight register, in flight or not: a register stays allocated from its load to the last wait that
// names it, and nothing that reads one can move above the wait.
template <int N>
__device__ __forceinline__ void wait_loads(uint4_t (&w)[2][kWOps]) {
  static_assert(N >= 0 && N <= 63, "vmcnt is a 6-bit counter");
  asm volatile("s_waitcnt vmcnt(%16)"
               : "+v"(w[0][0]), "+v"(w[0][1]), "+v"(w[0][2]), "+v"(w[0][3]), "+v"(w[0][4]), "+v"(w[0][5]), "+v"(w[0][6]), "+v"(w[0][7]),
                 "+v"(w[1][0]), "+v"(w[1][1]), "+v"(w[1][2]), "+v"(w[1][3]), "+v"(w[1][4]), "+v"(w[1][5]), "+v"(w[1][6]), "+v"(w[1][7])
               : "n"(N)
               : "memory");
}

template <int CONV, bool IL, bool FRAG, class FIN>
__global__ __launch_bounds__(64 * kWaves, 1) void i2_kslice_kernel(const int8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                                   typename FIN::out_t* __restrict__ C, int M, int N, int K,
                                                                   int tiles_m, int tiles_n, FIN fin) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31;
  const int h = lane >> 5;

  // workgroup -> tile: the workgroups of an XCD (ids x, x + 8, ...) take a contiguous run of tiles, the tiles that share
  // weight rows next to each other, so that a weight line is fetched from memory by one XCD only
  const int T = tiles_m * tiles_n;
  int pid = blockIdx.x;
  if ((T & 7) == 0) pid = (pid & 7) * (T >> 3) + (pid >> 3);
  const int m0 = (pid % tiles_m) * kTileM;
  const int n0 = (pid / tiles_m) * kTileN;

  const int kslice = K / kWaves;
  const int nblk = kslice >> 7;
  const unsigned lds0 = (unsigned)(uintptr_t)smem + (unsigned)(wave * kWaveLds);  // LDS addresses are the low 32 bits
  unsigned char* const ring = smem + wave * kWaveLds;

  // ---- activations: load i of a block: lane l brings the piece that belongs at position l % 8 of row 8 i + l / 8 -----
  uint32_t a_voff[kAOps];
#pragma unroll
  for (int i = 0; i < kAOps; ++i) {
    const int row = 8 * i + (lane >> 3);
    a_voff[i] = (uint32_t)min(m0 + row, M - 1) * (uint32_t)K + (uint32_t)(((lane & 7) ^ ((row >> 1) & 7)) * 16);
  }
  // Which eighth of K a wave owns turns with the workgroup (x, x + 8, ... share an XCD), three slices per workgroup:
  // the CUs do not all walk the same stretch of the activations and of their weight rows at the same time (M = 256,
  // N = K = 8192: 23.2 -> 22.75 us; by one slice 22.9 us).  Integer sums: exact in any order.
  const int kw = (wave + 3 * (int)(blockIdx.x >> 3)) & (kWaves - 1);
  const int8_t* const a_base = A + (size_t)kw * kslice;
  auto load_a = [&](int t, int i) {  // load i of block t, into stage t % 2
    dma16(lds0 + (unsigned)((t & 1) * kStage + i * 1024), a_voff[i], a_base + min(t, nblk - 1) * 128);
  };
  // fragment (mb, s) of a block: lane (r, h) reads piece 4 h + s of row 32 mb + r
  uint32_t a_rd[4];
#pragma unroll
  for (int s = 0; s < 4; ++s) a_rd[s] = (uint32_t)r * 128u + (uint32_t)(((4 * h + s) ^ ((r >> 1) & 7)) << 4);

  // ---- weights: load o of a pair of blocks.  Row-major: rows 16 o .. + 15 of the tile, lane l has piece l % 4 (64 k of
  // the pair's 256) of row 16 o + l / 4.  Fragment order: block o % 2 of the pair for the 32 rows o / 2, 1 KiB as stored.
  uint4_t w_raw[2][kWOps];
  const int npair = nblk >> 1;
  uint32_t w_voff[kWOps];
  const uint8_t* w_base;
  if constexpr (FRAG) {
    const int row_blocks = (N + 31) >> 5;
#pragma unroll
    for (int o = 0; o < kWOps; ++o)
      w_voff[o] = ((uint32_t)min((n0 >> 5) + (o >> 1), row_blocks - 1) * (uint32_t)(K >> 7) + (uint32_t)(o & 1)) * 1024u + (uint32_t)lane * 16u;
    w_base = B + (size_t)kw * nblk * 1024;
  } else {
    const uint32_t w_row_bytes = (uint32_t)(K >> 2);
#pragma unroll
    for (int o = 0; o < kWOps; ++o) w_voff[o] = (uint32_t)min(n0 + 16 * o + (lane >> 2), N - 1) * w_row_bytes + (uint32_t)(lane & 3) * 16u;
    w_base = B + (size_t)kw * (kslice >> 2);
  }
  constexpr int kPairBytes = FRAG ? 2048 : 64;  // from one pair of blocks to the next, per load
  auto load_w = [&](auto q_tag, auto o_tag, int pair) {
    load16(w_raw[decltype(q_tag)::value][decltype(o_tag)::value], w_voff[decltype(o_tag)::value], w_base + min(pair, npair - 1) * kPairBytes);
  };
  // lane (h, b, j) = 32 h + 16 b + j of the regrouped register takes lane 4 j + 2 b + h of the loaded one
  const int w_from = ((lane & 15) * 4 + ((lane >> 4) & 1) * 2 + (lane >> 5)) * 4;
  // afterwards w_raw[q][2 nb + b] is the operand of block b of the pair: lane (r, h) holds k = 64 h .. 64 h + 63 of row r
  auto regroup_w = [&](auto q_tag) {
    constexpr int q = decltype(q_tag)::value;
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb)
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const uint32_t x = (uint32_t)__builtin_amdgcn_ds_bpermute(w_from, (int)w_raw[q][2 * nb][d]);
        const uint32_t y = (uint32_t)__builtin_amdgcn_ds_bpermute(w_from, (int)w_raw[q][2 * nb + 1][d]);
        const auto sw = __builtin_amdgcn_permlane16_swap(x, y, false, false);
        w_raw[q][2 * nb][d] = sw[0];
        w_raw[q][2 * nb + 1][d] = sw[1];
      }
  };

  int16_t_ acc[kMB][kNB];
#pragma unroll
  for (int mb = 0; mb < kMB; ++mb)
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mb][nb][i] = 0;

  // ---- issue order ------------------------------------------------------------------------------------------------
  // A block is eight groups of four matrix instructions; group g of block t is followed by load g of A(t + 2), into
  // the stage block t was read from, and every second group by one weight load: during the second block of pair P the
  // X loads of pair P + 2 (into the registers of the first block's operands, which are done), during the first block of
  // pair P + 1 its Y loads (into those of the second block's operands of pair P).  Every block thus issues twelve
  // loads, and at the start of a block the twelve of the block before may still be in flight: what it needs is older.
  // (The compiler is free to move matrix instructions across the loads; pinning them with scheduling barriers
  // measured 5 % slower.)
  constexpr int kPerBlock = kAOps + kNB;
  // The prologue issues what block 0 needs first and then twelve more loads (block 1's activations and the X loads of
  // pair 1), as the block before block 0 would have.
  static_for<kWOps>([&](auto o) { load_w(std::integral_constant<int, 0>{}, o, 0); });
#pragma unroll
  for (int i = 0; i < kAOps; ++i) load_a(0, i);
#pragma unroll
  for (int i = 0; i < kAOps; ++i) load_a(1, i);
  static_for<kNB>([&](auto nb) { load_w(std::integral_constant<int, 1>{}, std::integral_constant<int, 2 * decltype(nb)::value>{}, 1); });

  // pair `pair` of blocks out of the weight registers w_raw[q], q = pair % 2
  auto do_pair = [&](auto q_tag, int pair) __attribute__((always_inline)) {
      constexpr int q = decltype(q_tag)::value;
      static_for<2>([&](auto b_tag) {
        constexpr int b = decltype(b_tag)::value;
        const int t = 2 * pair + b;
        wait_loads<kPerBlock>(w_raw);
        if constexpr (b == 0 && !FRAG) regroup_w(q_tag);
        const unsigned char* const st = ring + b * kStage;  // t % 2 == b
        int4_t af[kMB][4];
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
          for (int mb = 0; mb < kMB; ++mb) {
            const uint4_t a = *reinterpret_cast<const uint4_t*>(st + mb * 4096 + a_rd[s]);
            // plain packing: the decoder's dword i holds elements i, 4 + i, 8 + i, 12 + i of a fragment
            af[mb][s] = __builtin_bit_cast(int4_t, IL ? a : transpose4x4_bytes(a));
          }
        // the stage is overwritten from here on: its fragments must have left it
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        static_for<8>([&](auto g_tag) {
          constexpr int g = decltype(g_tag)::value;
          constexpr int s = g >> 1;
#pragma unroll
          for (int nb = 2 * (g & 1); nb < 2 * (g & 1) + 2; ++nb) {
            const int4_t bf = decode16<CONV>(w_raw[q][2 * nb + b][s]);
#pragma unroll
            for (int mb = 0; mb < kMB; ++mb) acc[mb][nb] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf, af[mb][s], acc[mb][nb], 0, 0, 0);
          }
          load_a(t + 2, g);
          if constexpr ((g & 1) == 1) {
            constexpr int nbw = g >> 1;  // the fourth of the block's weight loads this is
            if constexpr (b == 1) load_w(q_tag, std::integral_constant<int, 2 * nbw>{}, pair + 2);
            else load_w(std::integral_constant<int, q ^ 1>{}, std::integral_constant<int, 2 * nbw + 1>{}, pair + 1);
          }
        });
      });
  };
  for (int p0 = 0; p0 < npair; p0 += 2) {
    do_pair(std::integral_constant<int, 0>{}, p0);
    if (p0 + 1 < npair) do_pair(std::integral_constant<int, 1>{}, p0 + 1);  // an odd number of pairs: K % 4096 == 2048
  }
  // The loads past the end of the slice still write the stages and their registers.
  wait_loads<0>(w_raw);

  // ---- the eight partial sums meet: round mb, every wave leaves its four 32 x 32 blocks of that round in LDS and sums
  // rows 16 (wave % 2) .. + 15 of block wave / 2 over the eight slices ------------------------------------------------
  // A block in LDS: [32 rows][8 pieces of 4 columns], piece p of row m at position p ^ (m & 7).  Accumulator register
  // group vg of lane (r, h) holds columns 8 vg + 4 h .. + 3 (the weight rows of the block) of row r (the activation).
  static_for<kMB>([&](auto mb_tag) {
    constexpr int mb = decltype(mb_tag)::value;
    __syncthreads();  // the stages, or the previous round's sums, are no longer read
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb) {
      unsigned char* const blk = smem + (nb * kWaves + wave) * 4096;
#pragma unroll
      for (int vg = 0; vg < 4; ++vg) {
        const int4_t v = {acc[mb][nb][4 * vg], acc[mb][nb][4 * vg + 1], acc[mb][nb][4 * vg + 2], acc[mb][nb][4 * vg + 3]};
        *reinterpret_cast<int4_t*>(blk + r * 128 + (((2 * vg + h) ^ (r & 7)) << 4)) = v;
      }
    }
    __syncthreads();
    const int nb = wave >> 1;
    const int row = (wave & 1) * 16 + (lane >> 2);
    const int pp = (lane & 3) * 2;  // pieces pp, pp + 1: columns 4 pp .. 4 pp + 7
    int4_t lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0};
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const unsigned char* const blk = smem + (nb * kWaves + w) * 4096 + row * 128;
      lo += *reinterpret_cast<const int4_t*>(blk + ((pp ^ (row & 7)) << 4));
      hi += *reinterpret_cast<const int4_t*>(blk + (((pp + 1) ^ (row & 7)) << 4));
    }
    const int m = m0 + mb * 32 + row;
    const int n = n0 + nb * 32 + pp * 4;
    if (m < M && n < N) {
      using out_t = typename FIN::out_t;
      constexpr int kShift = Codes<CONV>::kShift;
      out_t o[8];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        o[e] = fin(lo[e] >> kShift, m);
        o[4 + e] = fin(hi[e] >> kShift, m);
      }
      out_t* dst = C + (size_t)m * N + n;
      if (n + 8 <= N && (N & 7) == 0) {
        constexpr int kPieces = sizeof(out_t) * 8 / 16;
        uint4_t pk[kPieces];
        __builtin_memcpy(pk, o, sizeof(o));
#pragma unroll
        for (int i = 0; i < kPieces; ++i) __builtin_nontemporal_store(pk[i], reinterpret_cast<uint4_t*>(dst) + i);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (n + e < N) dst[e] = o[e];
      }
    }
  });
}

template <int CONV, bool IL, bool FRAG, class FIN>
int launch_i2_kslice(const void* A, const void* B, void* C, int M, int N, int K, FIN fin, hipStream_t stream) {
  auto kern = i2_kslice_kernel<CONV, IL, FRAG, FIN>;
  static bool raised[kMaxDevices] = {};
  if (raise_lds_limit<kLds>(kern, raised)) return -1;
  const int tiles_m = (M + kTileM - 1) / kTileM, tiles_n = (N + kTileN - 1) / kTileN;
  hipLaunchKernelGGL(kern, dim3(tiles_m * tiles_n), dim3(64 * kWaves), kLds, stream, (const int8_t*)A, (const uint8_t*)B,
                     (typename FIN::out_t*)C, M, N, K, tiles_m, tiles_n, fin);
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

}  // namespace

// 0: launched; 1: this shape is not the kernel's (the caller falls back to the tiled GEMM); -1: error.
// force: take every shape the kernel can compute, whether or not it is expected to be the faster one.
int i2_gemm_kslice(const void* A, const void* B, void* C, int M, int N, int K, int convention, int layout, const void* s_a,
                   float s_w, int bitnet_epilogue, int force, hipStream_t stream) {
  // whole pairs of blocks of 128 k per wave; with signed codes the accumulators hold 64 x the sum
  if (K % (kWaves * 256) != 0 || K >= 131072) return 1;
  // 32-bit lane offsets
  if ((uint64_t)(M + kTileM) * (uint64_t)K >= (1ull << 32) || (uint64_t)(N + kTileN) * (uint64_t)(K >> 2) >= (1ull << 32)) return 1;
  const long tiles = (long)((M + kTileM - 1) / kTileM) * ((N + kTileN - 1) / kTileN);
  // worth it where the tiles are few enough that a tiled kernel leaves each CU one long chain (measured at
  // N = K = 8192: ahead of the tiled kernel up to M = 448, level with it there, behind from M = 512 on)
  if (!force && (tiles < 64 || tiles > 448 || K < 4096)) return 1;
#define DQ_I2K(CONV_, IL_, FRAG_)                                                                                       \
  do {                                                                                                                  \
    if (bitnet_epilogue)                                                                                                \
      return launch_i2_kslice<CONV_, IL_, FRAG_>(A, B, C, M, N, K, BitnetFinish{(const float*)s_a, s_w}, stream);       \
    return launch_i2_kslice<CONV_, IL_, FRAG_>(A, B, C, M, N, K, Int32Finish{}, stream);                                \
  } while (0)
#define DQ_I2KL(CONV_)                                                  \
  do {                                                                  \
    const bool il = (layout & ~LAYOUT_FRAGMENTS) == LAYOUT_INTERLEAVED; \
    if (layout & LAYOUT_FRAGMENTS) {                                    \
      if (il) DQ_I2K(CONV_, true, true);                                \
      DQ_I2K(CONV_, false, true);                                       \
    }                                                                   \
    if (il) DQ_I2K(CONV_, true, false);                                 \
    DQ_I2K(CONV_, false, false);                                        \
  } while (0)
  switch (convention) {
    case I2_UNSIGNED: DQ_I2KL(I2_UNSIGNED);
    case I2_OFFSET: DQ_I2KL(I2_OFFSET);
    case I2_TWOS: DQ_I2KL(I2_TWOS);
    default: DQ_FAIL("int2 gemm: unknown code convention %d", convention);
  }
#undef DQ_I2KL
#undef DQ_I2K
}

}  // namespace dq
