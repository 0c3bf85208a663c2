// MXFP4-weight x bf16 small batch (decode: up to 16 activation rows per pass) on gfx950: activations resident in
// registers, weights and block scales streamed once.
//
// Replaces the kernel of examples/dequantize_gemm/example_dequant_gemm_bf16_mxfp4_cdna4.py:201-244 (formats and
// scales: example_dequant_gemm_bf16_mxfp4_hopper.py:56-110,272-330) where M is a decode batch.  The tiled GEMM gives
// such a problem N / 256 workgroups with all of K behind each (N = K = 8192 at 1 to 128 rows: 60 us for 35 MB); here
// the matrix is cut by weight rows over all CUs and by K over the waves of a workgroup, as in dq_regres_i2.hip:
//
//   * one workgroup of eight waves per CU; a wave owns an eighth of K (which one turns with the workgroup): a run of
//     128-k chunks, at most eight (K <= 8192; more in slices, see below; K % 128 == 64 leaves the last chunk half
//     empty), and keeps the activations of its slice as operands of v_mfma_f32_16x16x32_bf16 in registers for the
//     whole kernel (16 rows x 1024 k: 128 registers per lane);
//   * the workgroups walk the blocks of 16 weight rows.  With K % 256 == 0 the runs are whole pairs of chunks and a
//     load takes 8 rows x 128 bytes (whole cache lines; lane l: piece l % 8 of row l / 8), two DPP moves sort a pair
//     of loads (rows 0 .. 7, rows 8 .. 15) into the even and the odd chunk; otherwise a load is a chunk of 16 rows x
//     64 bytes.  One ds_bpermute_b32 per dword then hands lane (g, r) piece g of row r of the chunk.  Dword s of a
//     lane feeds step s, contraction index k = 128 chunk + 32 g + 8 s + e for both operands: a lane's 32 codes are
//     ONE scale block, so the lane applies one E8M0 byte per chunk (byte g of the row's dword of scale bytes for the
//     chunk; 8 or 16 bytes of them per load) through the scale operand of the fp4 -> bf16 conversion;
//   * two sets of weight registers.  The workgroup's first block is asked for ahead of the activations and its
//     second behind them (loads come back in the order they went out); after that every chunk's registers are asked
//     for again, for the block after the next, as soon as the chunk's arithmetic is out.  The eight partial sums of
//     a block meet in LDS in fp32 (two buffers, one barrier per block) and 64 threads add them in slice order (the
//     same order every run), add the bias, round to bf16 and store.
//
// K beyond 8192 (K % 128 == 0): slices of at most 6144 k, the kernel's body once per slice with a prologue of its own,
// the running fp32 sums of the workgroup's blocks kept in LDS between slices (N <= 65536).
//
// Every load is unconditional and the last blocks have their own copies of the code, so that the compiler's count of
// loads in flight is exact (see dq_regres_i2.hip).  A wave whose run is shorter than the longest loads its last chunk
// (pair) again against activations of zero.  More than 16 rows: gridDim.y passes of 16, each streaming the weights
// again.
#include <type_traits>

#include "dq_common.h"
#include "dq_fp4_codes.h"

namespace dq {

namespace {

constexpr int kWaves = 8;              // K slices
constexpr int kMaxChunks = 8;          // 128-k chunks per wave
constexpr int kPartial = 16 * 16 * 4;  // one wave's 16 x 16 sums
constexpr int kLds = kWaves * 4096;    // the prologue's parking areas; the two buffers of partial sums reuse them
// With eight chunks per wave the activations (128 registers), two sets of weights and scales (80) and the arithmetic
// do not fit 256 registers: the fragments of the wave's last three chunks (four where the scale bytes are loaded one
// by one: eight more addresses) stay parked in LDS, 4 KiB per wave and chunk behind the areas above, and are read
// again for every block.
constexpr int parked_chunks(int ncw, int lines) { return ncw == 8 ? (lines ? 3 : 4) : 0; }

typedef float float4v __attribute__((ext_vector_type(4)));

// what a lane applies to its 32 codes of one chunk: the block's power of two as the conversion's scale operand, or,
// for the "simple" format, the exponent to add to both halves of a dword
struct LaneScale {
  float f;
  uint32_t add;
};
template <int FMT>
__device__ __forceinline__ LaneScale lane_scale(uint32_t e, int off) {
  LaneScale s;
  if constexpr (FMT == FP4_SIMPLE) {
    int ex = 126 + (int)e + off - 127;
    ex = ex < 0 ? 0 : (ex > 252 ? 252 : ex);  // E adds up to 3
    s.add = ((uint32_t)ex << 7) * 0x00010001u;
    s.f = 0.f;
  } else {
    s.f = scale_to_f32((int)e, off);
    s.add = 0;
  }
  return s;
}
template <int FMT>
__device__ __forceinline__ bf16x8_t decode8(uint32_t w, const LaneScale& s) {
  if constexpr (FMT == FP4_E2M1) return cvt_e2m1x8(w, s.f);
  else if constexpr (FMT == FP4_TWIDDLING) return cvt_e2m1x8(twiddled_to_plain(w), s.f);
  else return __builtin_bit_cast(bf16x8_t, simple_fp4x8<7>(w, s.add));
}

// LINES: 0: K % 64 == 0, a load per chunk of 16 rows x 64 bytes and a byte of scale per chunk and lane; 1: K % 256 == 0,
// the waves' runs are whole pairs of chunks, weights fetched as whole 128-byte lines and scales 8 bytes (a pair) at a
// time; 2: K % 4096 == 0, every run starts on a multiple of four chunks and is as long: scales 16 bytes at a time.
template <int FMT, bool HAS_BIAS, int NCW, int LINES, bool HALF, bool LONGK>
__global__ __launch_bounds__(64 * kWaves, 1) void mx_regres_kernel(const bf16_t* __restrict__ A_all, const uint8_t* __restrict__ B,
                                                                   const uint8_t* __restrict__ S, const bf16_t* __restrict__ Bias_all,
                                                                   bf16_t* __restrict__ C_all, int M_all, int N, int K, int exp_off) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int m_first = 16 * blockIdx.y;
  const bf16_t* const A = A_all + (size_t)m_first * K;
  bf16_t* const C = C_all + (size_t)m_first * N;
  const bf16_t* const Bias = HAS_BIAS ? Bias_all + (size_t)m_first * N : nullptr;
  const int M = min(M_all - m_first, 16);
  constexpr bool PAIR = LINES >= 1, SVEC = LINES == 2;
  static_assert(!PAIR || (NCW % 2 == 0 && !HALF), "whole pairs of whole chunks");
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15;
  const int g = lane >> 4;

  // The wave's chunks: [c_lo, c_lo + ncw), ncw <= NCW.  HALF: K % 128 == 64, the last chunk has 64 k.  Its lanes of the
  // upper half (pieces 2, 3 of a weight row's 64 bytes, 8 .. 15 of an activation row's 256) read the lower half's
  // addresses instead, so that nothing is read beyond a row, and multiply activations of zero.
  const int nchunk = (K + 127) >> 7;
  constexpr bool half_last = HALF;  // a form of its own: its lane-dependent addresses cost registers
  // LONGK: K beyond what the registers hold goes in slices of at most 8 NCW chunks, equal up to a chunk: the kernel's
  // body once per slice, with a fresh prologue, the finishing threads' running fp32 sums of the workgroup's blocks in
  // LDS in between (slice order: the same sums every run).
  const int nslices = LONGK ? (nchunk + kWaves * NCW - 1) / (kWaves * NCW) : 1;
  const int row_blocks = (N + 15) >> 4;
  const int step = gridDim.x;  // at most the number of blocks: every workgroup has one
  const int mine = (row_blocks - (int)blockIdx.x + step - 1) / step;
  for (int slice = 0; slice < nslices; ++slice) {
  if (slice > 0) __syncthreads();  // the partial sums of the slice before are read: their place is free
  // (PAIR: slices and runs are cut in whole pairs of chunks)
  constexpr int U = PAIR ? 2 : 1;
  const int nunit = nchunk / U;
  const int sl_lo = slice * nunit / nslices;
  const int sl_n = (slice + 1) * nunit / nslices - sl_lo;
  // Which eighth of K a wave owns turns with the workgroup (the workgroups x, x + 8, ... share an XCD): with wave w on
  // slice w everywhere, every CU asked the same stretch of every weight row and of the activations at the same time
  // (N = K = 8192 at 16 rows: 16.0 -> 14.4 us).  The partial sums are still added in slice order.
  const int kw = (wave + (int)(blockIdx.x >> 3)) & (kWaves - 1);
  const int u_lo = sl_lo + kw * sl_n / kWaves;
  const int nuw = sl_lo + (kw + 1) * sl_n / kWaves - u_lo;
  const int c_lo = U * u_lo, ncw = U * nuw;
  // K < 1024: some waves have no chunk at all
  auto chunk_of = [&](int i) { return c_lo + U * min(i / U, max(nuw - 1, 0)) + i % U; };
  auto is_half = [&](int i) { return half_last && chunk_of(i) == nchunk - 1; };

  int nb = blockIdx.x;

  // ---- weights and scales of the block of 16 rows nb
  // (the chunk numbers are the same for every lane of the wave: scalar registers, not eight offsets per lane)
  const uint32_t w_row_bytes = (uint32_t)(K >> 1), s_row_bytes = (uint32_t)(K >> 5);
  // load_part(.., i): what chunk i's arithmetic leaves free.  Whole 128-byte lines where K allows (PAIR): a pair of
  // chunks of 8 rows per load (lane l: piece l % 8 of row l / 8), rows 0 .. 7 of the block into w[2 j], rows 8 .. 15
  // into w[2 j + 1]; do_block sorts them into chunks.  (16 rows x 64 bytes per load asks the L2 for every line twice
  // and costs the load unit 16 rows per KiB instead of 8.)  A lane's scale bytes of a block: the dword of every chunk
  // (byte g of it is the lane's), 8 bytes (a pair) or 16 bytes (four chunks, SVEC) per load; without PAIR the lane's own
  // byte.  Dword by dword the eight loads of a lane fetched the same 32 bytes eight times from the L2 (nontemporal
  // loads leave nothing in the L1): 12 of 48 us at N = 28672, K = 8192.
  struct RowPtrs {
    const uint8_t *w_lo, *w_hi, *s_row;
  };
  auto rows_of = [&](int blk) __attribute__((always_inline)) {
    RowPtrs p;
    if constexpr (PAIR) {
      p.w_lo = B + (size_t)min(16 * blk + (lane >> 3), N - 1) * w_row_bytes + (lane & 7) * 16;
      p.w_hi = B + (size_t)min(16 * blk + 8 + (lane >> 3), N - 1) * w_row_bytes + (lane & 7) * 16;
    } else {
      p.w_lo = p.w_hi = B + (size_t)min(16 * blk + (lane >> 2), N - 1) * w_row_bytes;
    }
    p.s_row = S + (size_t)min(16 * blk + r, N - 1) * s_row_bytes;
    return p;
  };
  auto load_part = [&](uint4_t (&w)[NCW], uint32_t (&sc)[NCW], const RowPtrs& p, int i) __attribute__((always_inline)) {
    if constexpr (PAIR) {
      if (i & 1) {
        w[i - 1] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(p.w_lo + chunk_of(i - 1) * 64));
        w[i] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(p.w_hi + chunk_of(i - 1) * 64));
        if constexpr (!SVEC) {
          typedef uint32_t uint2v __attribute__((ext_vector_type(2)));
          const uint2v v = __builtin_nontemporal_load(reinterpret_cast<const uint2v*>(p.s_row + chunk_of(i - 1) * 4));
          sc[i - 1] = v[0], sc[i] = v[1];
        }
      }
      if constexpr (SVEC) {
        if ((i & 3) == 3) {
          const uint4_t v = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(p.s_row + c_lo * 4 + (i - 3) * 4));
          sc[i - 3] = v[0], sc[i - 2] = v[1], sc[i - 1] = v[2], sc[i] = v[3];
        }
      }
    } else {
      w[i] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(p.w_lo + chunk_of(i) * 64 + ((lane & 3) & (is_half(i) ? 1 : 3)) * 16));
      sc[i] = p.s_row[chunk_of(i) * 4 + (g & (is_half(i) ? 1 : 3))];  // the lane's own byte
    }
  };
  auto load_w = [&](uint4_t (&w)[NCW], uint32_t (&sc)[NCW], int blk) __attribute__((always_inline)) {
    const RowPtrs p = rows_of(blk);
#pragma unroll
    for (int i = 0; i < NCW; ++i) load_part(w, sc, p, i);
    // the loads go out here, ahead of what follows: left to itself the scheduler sinks them to save registers
    __builtin_amdgcn_sched_barrier(0);
  };
  uint4_t w0[NCW], w1[NCW];
  uint32_t sc0[NCW], sc1[NCW];
  // ---- activations: fragment (chunk i, step s): lane (g, r) holds k = 128 chunk + 32 g + 8 s .. + 7 of row r.  Read as
  // whole lines (instruction j: rows 4 j .. 4 j + 3, lane l the 16-byte piece l % 16 of row 4 j + l / 16 of the
  // chunk's 256 bytes), parked in the wave's 4 KiB of LDS (piece q of row m at position q ^ m), read back in operand
  // order: fetched in that order a load instruction would touch 32 cache lines for 32 bytes each.
  constexpr int PARK = parked_chunks(NCW, LINES), NR = NCW - PARK;
  unsigned char* const kept = smem + kLds + wave * (PARK * 4096);  // chunk NR + q at kept + 4096 q, laid out as `park`
  const int kept_rd = r * 256;                                      // piece p of the lane's row: kept_rd + ((p ^ r) << 4)
  bf16x8_t af[NR][4];
  // The workgroup's first two blocks of weights are asked for in the prologue as well (most matrices give a workgroup
  // two to four blocks, too few for a pipeline that starts one deep).  Loads come back in the order they went out, and
  // the first block's arithmetic needs the first block and the activations: so the second block goes out behind the
  // activations, and their fragments are parked and read back while it is still on its way.
  {
    load_w(w0, sc0, nb);
    const unsigned char* const a_base = reinterpret_cast<const unsigned char*>(A);
    uint4_t line[NCW][4];
#pragma unroll
    for (int i = 0; i < NCW; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        line[i][j] = *reinterpret_cast<const uint4_t*>(a_base + ((size_t)min(4 * j + (lane >> 4), M - 1) * K + 128 * chunk_of(i)) * 2 +
                                                       16 * ((lane & 15) & (is_half(i) ? 7 : 15)));
    __builtin_amdgcn_sched_barrier(0);
    if (mine > 1) load_w(w1, sc1, nb + step);
#pragma unroll
    for (int i = 0; i < NCW; ++i) {
      unsigned char* const park = i < NR ? smem + wave * 4096 : kept + (i - NR) * 4096;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int row = 4 * j + (lane >> 4);
        // a chunk beyond the wave's slice: zeros
        const bool there = i < ncw && !(is_half(i) && (lane & 15) >= 8);
        *reinterpret_cast<uint4_t*>(park + row * 256 + (((lane & 15) ^ row) << 4)) = there ? line[i][j] : uint4_t{0u, 0u, 0u, 0u};
      }
      // a wave's LDS operations are carried out in the order they were issued
      if (i < NR) {
#pragma unroll
        for (int s = 0; s < 4; ++s)
          af[i < NR ? i : 0][s] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const uint4_t*>(park + kept_rd + (((4 * g + s) ^ r) << 4)));
      }
    }
    __syncthreads();  // the parking areas are where the partial sums go
  }

  // lane (g, r) of the regrouped register takes lane 4 r + g.  PAIR: the loaded pair X (rows 0 .. 7), Y (rows 8 .. 15)
  // becomes the even chunk, X with the upper four lanes of every eight taken from Y's lower four, and the odd chunk, X
  // with the lower four taken from Y's upper four: row r % 8 + 8 j sits in lanes 8 (r % 8) + 4 j .. + 3 of the even
  // chunk and in lanes 8 (r % 8) + 4 (1 - j) .. + 3 of the odd one.
  const int w_from = PAIR ? ((r & 7) * 8 + (r >> 3) * 4 + g) * 4 : ((lane & 15) * 4 + (lane >> 4)) * 4;
  // the thread's share of the final sum: activation row tid / 4, weight rows 4 (tid % 4) .. + 3 of the block
  const int out_m = tid >> 2, out_p = tid & 3;
  const bool finisher = tid < 64 && out_m < M;

  // next_tag: whether the set takes the workgroup's block after the next (blk + 2 step) as this one is consumed: every
  // chunk's registers are asked for again as soon as its arithmetic is out, not when the whole block is done (with two
  // sets of registers that is what keeps close to two blocks per CU in flight).
  auto do_block = [&](uint4_t (&w)[NCW], uint32_t (&sc)[NCW], int blk, int it, auto next_tag) __attribute__((always_inline)) {
    constexpr bool reload = decltype(next_tag)::value;
    const RowPtrs nxt = rows_of(reload ? blk + 2 * step : blk);
    float4v acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < NCW; ++i) {
      uint4_t x = w[i];
      if constexpr (PAIR) {
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const int lo8 = (int)w[i & ~1][d], hi8 = (int)w[i | 1][d];
          // row_shr:4 into lanes 4 .. 7, 12 .. 15 of every 16; row_shl:4 into lanes 0 .. 3, 8 .. 11
          const int sorted = (i & 1) ? __builtin_amdgcn_update_dpp(lo8, hi8, 0x104, 0xF, 0x5, false)
                                     : __builtin_amdgcn_update_dpp(lo8, hi8, 0x114, 0xF, 0xA, false);
          x[d] = (uint32_t)__builtin_amdgcn_ds_bpermute((i & 1) ? (w_from ^ 16) : w_from, sorted);
        }
      } else {
#pragma unroll
        for (int d = 0; d < 4; ++d) x[d] = (uint32_t)__builtin_amdgcn_ds_bpermute(w_from, (int)x[d]);
      }
      const LaneScale ls = lane_scale<FMT>(PAIR ? (sc[i] >> (8 * g)) & 0xFFu : sc[i], exp_off);
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        bf16x8_t a;
        if (i < NR) a = af[i < NR ? i : 0][s];
        else a = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const uint4_t*>(kept + (i - NR) * 4096 + kept_rd + (((4 * g + s) ^ r) << 4)));
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(decode8<FMT>(x[s], ls), a, acc, 0, 0, 0);
      }
      if constexpr (reload) {
        __builtin_amdgcn_sched_barrier(0);
        load_part(w, sc, nxt, i);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // lane (g, r) holds the weight rows 4 g .. 4 g + 3 of activation row r.  A wave's sums in LDS: [16 activation
    // rows][4 pieces of 4 weight rows], piece p of row m at position p ^ (m & 3).
    unsigned char* const buf = smem + ((slice * mine + it) & 1) * (kWaves * kPartial);
    if (r < M) *reinterpret_cast<float4v*>(buf + kw * kPartial + r * 64 + ((g ^ (r & 3)) << 4)) = acc;
    // One barrier per block: the buffer written here is read below and written again two blocks later, after the next
    // block's barrier, which no thread passes before it has finished reading here.
    __syncthreads();
    if (finisher) {
      const int m = out_m, p = out_p;
      float4v sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w8 = 0; w8 < kWaves; ++w8) sum += *reinterpret_cast<const float4v*>(buf + w8 * kPartial + m * 64 + ((p ^ (m & 3)) << 4));
      if constexpr (LONGK) {  // this thread's four outputs of the workgroup's block number `it`, behind everything else
        float4v* const running = reinterpret_cast<float4v*>(smem + kLds + kWaves * PARK * 4096 + it * kPartial + m * 64 + p * 16);
        if (slice > 0) sum += *running;
        if (slice + 1 < nslices) *running = sum;
      }
      const int n = 16 * blk + 4 * p;
      if (slice + 1 == nslices && n < N) {
        bf16_t o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float v = sum[e];
          // reference: C = bf16(float(acc) + float(Bias))
          if constexpr (HAS_BIAS) {
            if (n + e < N) v += (float)Bias[(size_t)m * N + n + e];
          }
          o[e] = (bf16_t)v;
        }
        bf16_t* const dst = C + (size_t)m * N + n;
        if ((N & 3) == 0) {
          typedef bf16_t bf16x4_t __attribute__((ext_vector_type(4)));
          *reinterpret_cast<bf16x4_t*>(dst) = bf16x4_t{o[0], o[1], o[2], o[3]};
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < N) dst[e] = o[e];
        }
      }
    }
  };

  // w0 holds the workgroup's block k, w1 block k + 1.  The loop over pairs of blocks that both have a successor has no
  // exit in its body, and the last one to three blocks follow it in copies of their own: a load under a condition, or
  // an exit that shares its way out with the loop's way round, would make the compiler count the loads in flight for a
  // path that does not have them, and wait for everything at the top of the loop.
  constexpr std::true_type more{};
  constexpr std::false_type last{};
  int k = 0;
  for (; k + 4 <= mine; k += 2) {
    do_block(w0, sc0, nb, k, more);
    do_block(w1, sc1, nb + step, k + 1, more);
    nb += 2 * step;
  }
  const int left = mine - k;
  if (left == 1) {
    do_block(w0, sc0, nb, k, last);
  } else if (left == 2) {
    do_block(w0, sc0, nb, k, last);
    do_block(w1, sc1, nb + step, k + 1, last);
  } else {
    do_block(w0, sc0, nb, k, more);
    do_block(w1, sc1, nb + step, k + 1, last);
    do_block(w0, sc0, nb + 2 * step, k + 2, last);
  }
  }  // slices of K
}

template <int FMT, bool HAS_BIAS, int NCW, int LINES, bool HALF, bool LONGK>
int launch_mx_regres(const void* A, const void* B, const void* S, const void* Bias, void* C, int M, int N, int K, int exp_off,
                     hipStream_t stream) {
  auto kern = mx_regres_kernel<FMT, HAS_BIAS, NCW, LINES, HALF, LONGK>;
  static bool raised[kMaxDevices] = {};
  constexpr int kMaxRunning = 16;  // blocks of a workgroup whose running sums fit (N <= 65536)
  constexpr int kLdsFixed = kLds + kWaves * parked_chunks(NCW, LINES) * 4096;
  if (raise_lds_limit<kLdsFixed + (LONGK ? kMaxRunning * kPartial : 0)>(kern, raised)) return -1;
  static int cus_of[kMaxDevices] = {};
  int device = 0;
  DQ_CHECK_HIP(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices) DQ_FAIL("device index %d is beyond the %d this library keeps state for", device, kMaxDevices);
  if (!cus_of[device]) DQ_CHECK_HIP(hipDeviceGetAttribute(&cus_of[device], hipDeviceAttributeMultiprocessorCount, device));
  const int row_blocks = (N + 15) / 16;
  const int grid = row_blocks < cus_of[device] ? row_blocks : cus_of[device];
  const int mine = (row_blocks + grid - 1) / grid;
  if (LONGK && mine > kMaxRunning) return 1;
  const int kLdsAll = kLdsFixed + (LONGK ? mine * kPartial : 0);
  hipLaunchKernelGGL(kern, dim3(grid, (M + 15) / 16), dim3(64 * kWaves), kLdsAll, stream, (const bf16_t*)A, (const uint8_t*)B,
                     (const uint8_t*)S, (const bf16_t*)Bias, (bf16_t*)C, M, N, K, exp_off);
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

// ---- one activation row: a dot-product kernel (the memory-bound decode GEMV; no matrix instruction) --------------------
// A wave owns whole weight rows.  Lane l of step s holds the 32 codes k = 2048 s + 32 l .. + 31 of a row: 16 bytes, ONE
// scale block, so a wave's load instruction reads 1 KiB contiguous and a lane applies one E8M0 byte per load through
// the conversion's scale operand.  The lane's 32 activations of every step stay in registers for the whole kernel
// (16 per step), the products are summed in fp32 with v_dot2c_f32_bf16, a row's 64 partial sums by a butterfly over
// the lanes (fixed order).  kGemvRows rows are in flight per wave, and as many waves per SIMD as the registers allow
// hide the rest of the latency; the waves walk the batches of rows with a stride of the whole grid.  K % 64 == 0 up to
// 2048 STEPS: the lanes beyond a row's end read its last 16 bytes again against activations of zero.
constexpr int kGemvRows = 4;

template <int FMT, bool HAS_BIAS, int STEPS>
__global__ __launch_bounds__(256) void mx_gemv_kernel(const bf16_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                      const uint8_t* __restrict__ S, const bf16_t* __restrict__ Bias,
                                                      bf16_t* __restrict__ C, int N, int K, int exp_off) {
  const int lane = threadIdx.x & 63;
  const int gw = blockIdx.x * 4 + (threadIdx.x >> 6), nwaves = gridDim.x * 4;
  const int nblk = K >> 5;  // scale blocks (16 bytes of codes) per row
  const uint32_t w_row_bytes = (uint32_t)(K >> 1), s_row_bytes = (uint32_t)nblk;
  // the lane's block of every step, and its activations (zeros beyond the row's end)
  uint32_t blk[STEPS];
  uint4_t a[STEPS][4];
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    const int c = s * 64 + lane;
    blk[s] = (uint32_t)min(c, nblk - 1);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const uint4_t v = *reinterpret_cast<const uint4_t*>(reinterpret_cast<const unsigned char*>(A) + (size_t)blk[s] * 64 + q * 16);
      a[s][q] = c < nblk ? v : uint4_t{0u, 0u, 0u, 0u};
    }
  }
  const int nbatch = (N + kGemvRows - 1) / kGemvRows;
  for (int b = gw; b < nbatch; b += nwaves) {
    uint4_t w[kGemvRows][STEPS];
    uint32_t sc[kGemvRows][STEPS];
#pragma unroll
    for (int j = 0; j < kGemvRows; ++j) {
      const int n = min(b * kGemvRows + j, N - 1);
      const uint8_t* const w_row = B + (size_t)n * w_row_bytes;
      const uint8_t* const s_row = S + (size_t)n * s_row_bytes;
#pragma unroll
      for (int s = 0; s < STEPS; ++s) {
        w[j][s] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(w_row + blk[s] * 16));
        sc[j][s] = __builtin_nontemporal_load(s_row + blk[s]);
      }
    }
    float sum[kGemvRows];
#pragma unroll
    for (int j = 0; j < kGemvRows; ++j) {
      float acc = 0.f;
#pragma unroll
      for (int s = 0; s < STEPS; ++s) {
        const LaneScale ls = lane_scale<FMT>(sc[j][s], exp_off);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const bf16x8_t wv = decode8<FMT>(w[j][s][q], ls);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const uint32_t pair = a[s][q][e];  // a value first: a bit cast of the element expression itself reads element 0
            acc = __builtin_amdgcn_fdot2_f32_bf16(bf16x2_t{wv[2 * e], wv[2 * e + 1]}, __builtin_bit_cast(bf16x2_t, pair), acc, false);
          }
        }
      }
      sum[j] = acc;
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1)
#pragma unroll
      for (int j = 0; j < kGemvRows; ++j) sum[j] += __shfl_xor(sum[j], off);
    // lane j of the first kGemvRows stores row j of the batch
    float mine = sum[0];
#pragma unroll
    for (int j = 1; j < kGemvRows; ++j) mine = lane == j ? sum[j] : mine;
    const int n = b * kGemvRows + lane;
    if (lane < kGemvRows && n < N) {
      // reference: C = bf16(float(acc) + float(Bias))
      if constexpr (HAS_BIAS) mine += (float)Bias[n];
      C[n] = (bf16_t)mine;
    }
  }
}

template <int FMT, bool HAS_BIAS, int STEPS>
int launch_mx_gemv(const void* A, const void* B, const void* S, const void* Bias, void* C, int N, int K, int exp_off,
                   hipStream_t stream) {
  auto kern = mx_gemv_kernel<FMT, HAS_BIAS, STEPS>;
  static int cus_of[kMaxDevices] = {}, per_cu[kMaxDevices] = {};
  int device = 0;
  DQ_CHECK_HIP(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices) DQ_FAIL("device index %d is beyond the %d this library keeps state for", device, kMaxDevices);
  if (!cus_of[device]) {
    DQ_CHECK_HIP(hipDeviceGetAttribute(&cus_of[device], hipDeviceAttributeMultiprocessorCount, device));
    DQ_CHECK_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu[device], kern, 256, 0));
    if (per_cu[device] < 1) per_cu[device] = 1;
  }
  // every workgroup resident at once; no more waves than batches of rows
  const int nbatch = (N + kGemvRows - 1) / kGemvRows;
  const int want = (nbatch + 3) / 4, room = cus_of[device] * per_cu[device];
  hipLaunchKernelGGL(kern, dim3(want < room ? want : room), dim3(256), 0, stream, (const bf16_t*)A, (const uint8_t*)B,
                     (const uint8_t*)S, (const bf16_t*)Bias, (bf16_t*)C, N, K, exp_off);
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

// ---- two activation rows (the kernel takes up to four): the same dot-product kernel with the activations in LDS -----------
// MR rows of 32 activations per lane and step would not fit the registers beside the weights in flight: the workgroup
// copies the rows to LDS once ([row][step][piece of 16 bytes][lane]: a wave's read is 1 KiB contiguous), and a step's
// fragments of all rows are read once per batch of kGemvRows weight rows; every weight dword is converted once and
// multiplied into all rows.  The MR x kGemvRows sums of a batch are added over the lanes by the halving reduction
// (RowReduce over each 16 lanes, then two butterflies): lane 4 m + j ends up with row m of the batch's weight row j.
template <int FMT, bool HAS_BIAS, int STEPS, int MR>
__global__ __launch_bounds__(256) void mx_gemv_rows_kernel(const bf16_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                           const uint8_t* __restrict__ S, const bf16_t* __restrict__ Bias,
                                                           bf16_t* __restrict__ C, int M, int N, int K, int exp_off) {
  static_assert(MR * kGemvRows <= 16, "one value per lane of a DPP row");
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int gw = blockIdx.x * 4 + (tid >> 6), nwaves = gridDim.x * 4;
  const int nblk = K >> 5;  // scale blocks (16 bytes of codes, 64 bytes of activations) per row
  const uint32_t w_row_bytes = (uint32_t)(K >> 1), s_row_bytes = (uint32_t)nblk;
  for (int p = tid; p < MR * STEPS * 256; p += 256) {  // source order: piece q of block 64 s + l of row m at p = ((m STEPS + s) 64 + l) 4 + q
    const int q = p & 3, l = (p >> 2) & 63, ms = p >> 8;
    const int m = ms / STEPS, c = (ms % STEPS) * 64 + l;
    uint4_t v = {0u, 0u, 0u, 0u};  // rows beyond M, blocks beyond the row's end
    if (m < M && c < nblk) v = *reinterpret_cast<const uint4_t*>(reinterpret_cast<const unsigned char*>(A) + (size_t)m * K * 2 + (size_t)c * 64 + q * 16);
    *reinterpret_cast<uint4_t*>(smem + ((ms * 4 + q) * 64 + l) * 16) = v;
  }
  __syncthreads();
  uint32_t blk[STEPS];
#pragma unroll
  for (int s = 0; s < STEPS; ++s) blk[s] = (uint32_t)min(s * 64 + lane, nblk - 1);
  const int nbatch = (N + kGemvRows - 1) / kGemvRows;
  for (int b = gw; b < nbatch; b += nwaves) {
    uint4_t w[kGemvRows][STEPS];
    uint32_t sc[kGemvRows][STEPS];
#pragma unroll
    for (int j = 0; j < kGemvRows; ++j) {
      const int n = min(b * kGemvRows + j, N - 1);
      const uint8_t* const w_row = B + (size_t)n * w_row_bytes;
      const uint8_t* const s_row = S + (size_t)n * s_row_bytes;
#pragma unroll
      for (int s = 0; s < STEPS; ++s) {
        w[j][s] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(w_row + blk[s] * 16));
        sc[j][s] = __builtin_nontemporal_load(s_row + blk[s]);
      }
    }
    float acc[16];  // [m][j]
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      uint4_t af[MR][4];
#pragma unroll
      for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int q = 0; q < 4; ++q) af[m][q] = *reinterpret_cast<const uint4_t*>(smem + (((m * STEPS + s) * 4 + q) * 64 + lane) * 16);
#pragma unroll
      for (int j = 0; j < kGemvRows; ++j) {
        const LaneScale ls = lane_scale<FMT>(sc[j][s], exp_off);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const bf16x8_t wv = decode8<FMT>(w[j][s][q], ls);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const bf16x2_t wp = {wv[2 * e], wv[2 * e + 1]};
#pragma unroll
            for (int m = 0; m < MR; ++m) {
              const uint32_t pair = af[m][q][e];  // a value first (see mx_gemv_kernel)
              acc[m * kGemvRows + j] = __builtin_amdgcn_fdot2_f32_bf16(wp, __builtin_bit_cast(bf16x2_t, pair), acc[m * kGemvRows + j], false);
            }
          }
        }
      }
      // a step's fragments are read when the step before is done: hoisted, the fragments of all steps are live at once
      __builtin_amdgcn_sched_barrier(0);
    }
    float t = RowReduce<16, 0>::run(acc, lane);
    t += __shfl_xor(t, 16);
    t += __shfl_xor(t, 32);
    const int m = (lane >> 2) & 3, n = b * kGemvRows + (lane & 3);
    if (lane < 16 && m < M && n < N) {
      // reference: C = bf16(float(acc) + float(Bias))
      if constexpr (HAS_BIAS) t += (float)Bias[(size_t)m * N + n];
      C[(size_t)m * N + n] = (bf16_t)t;
    }
  }
}

template <int FMT, bool HAS_BIAS, int STEPS, int MR>
int launch_mx_gemv_rows(const void* A, const void* B, const void* S, const void* Bias, void* C, int M, int N, int K,
                        int exp_off, hipStream_t stream) {
  auto kern = mx_gemv_rows_kernel<FMT, HAS_BIAS, STEPS, MR>;
  constexpr int kLdsA = MR * STEPS * 4096;
  static bool raised[kMaxDevices] = {};
  if (raise_lds_limit<kLdsA>(kern, raised)) return -1;
  static int cus_of[kMaxDevices] = {}, per_cu[kMaxDevices] = {};
  int device = 0;
  DQ_CHECK_HIP(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices) DQ_FAIL("device index %d is beyond the %d this library keeps state for", device, kMaxDevices);
  if (!cus_of[device]) {
    DQ_CHECK_HIP(hipDeviceGetAttribute(&cus_of[device], hipDeviceAttributeMultiprocessorCount, device));
    DQ_CHECK_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu[device], kern, 256, kLdsA));
    if (per_cu[device] < 1) per_cu[device] = 1;
  }
  const int nbatch = (N + kGemvRows - 1) / kGemvRows;
  const int want = (nbatch + 3) / 4, room = cus_of[device] * per_cu[device];
  hipLaunchKernelGGL(kern, dim3(want < room ? want : room), dim3(256), kLdsA, stream, (const bf16_t*)A, (const uint8_t*)B,
                     (const uint8_t*)S, (const bf16_t*)Bias, (bf16_t*)C, M, N, K, exp_off);
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

// ---- one and two activation rows with K beyond 8192: the dot-product kernel over chunks of four steps ---------------------
// As mx_gemv_rows_kernel (activations in LDS, padded with zeros to whole chunks), the loop over K in chunks of four
// steps (8192 k): a chunk's 16 loads of a batch of four weight rows are asked for, waited for and multiplied, the
// sums carried from chunk to chunk; the other waves of the SIMD cover the wait.
template <int FMT, bool HAS_BIAS, int MR>
__global__ __launch_bounds__(256) void mx_gemv_long_kernel(const bf16_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                           const uint8_t* __restrict__ S, const bf16_t* __restrict__ Bias,
                                                           bf16_t* __restrict__ C, int M, int N, int K, int exp_off) {
  static_assert(MR * kGemvRows <= 16, "one value per lane of a DPP row");
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int gw = blockIdx.x * 4 + (tid >> 6), nwaves = gridDim.x * 4;
  const int nblk = K >> 5;
  const int nchunk = (nblk + 255) >> 8, nsteps = 4 * nchunk;  // steps of 64 blocks, padded to whole chunks
  const uint32_t w_row_bytes = (uint32_t)(K >> 1), s_row_bytes = (uint32_t)nblk;
  for (int p = tid; p < MR * nsteps * 256; p += 256) {  // piece q of block 64 s + l of row m at p = ((m nsteps + s) 64 + l) 4 + q
    const int q = p & 3, l = (p >> 2) & 63, ms = p >> 8;
    const int m = ms / nsteps, c = (ms % nsteps) * 64 + l;
    uint4_t v = {0u, 0u, 0u, 0u};  // rows beyond M, blocks beyond the row's end
    if (m < M && c < nblk) v = *reinterpret_cast<const uint4_t*>(reinterpret_cast<const unsigned char*>(A) + (size_t)m * K * 2 + (size_t)c * 64 + q * 16);
    *reinterpret_cast<uint4_t*>(smem + ((ms * 4 + q) * 64 + l) * 16) = v;
  }
  __syncthreads();
  const int nbatch = (N + kGemvRows - 1) / kGemvRows;
  for (int b = gw; b < nbatch; b += nwaves) {
    float acc[16];  // [m][j]
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
    for (int ch = 0; ch < nchunk; ++ch) {
      uint4_t w[kGemvRows][4];
      uint32_t sc[kGemvRows][4];
#pragma unroll
      for (int j = 0; j < kGemvRows; ++j) {
        const int n = min(b * kGemvRows + j, N - 1);
        const uint8_t* const w_row = B + (size_t)n * w_row_bytes;
        const uint8_t* const s_row = S + (size_t)n * s_row_bytes;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const uint32_t blk = (uint32_t)min((4 * ch + s) * 64 + lane, nblk - 1);
          w[j][s] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(w_row + blk * 16));
          sc[j][s] = __builtin_nontemporal_load(s_row + blk);
        }
      }
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        uint4_t af[MR][4];
#pragma unroll
        for (int m = 0; m < MR; ++m)
#pragma unroll
          for (int q = 0; q < 4; ++q) af[m][q] = *reinterpret_cast<const uint4_t*>(smem + (((m * nsteps + 4 * ch + s) * 4 + q) * 64 + lane) * 16);
#pragma unroll
        for (int j = 0; j < kGemvRows; ++j) {
          const LaneScale ls = lane_scale<FMT>(sc[j][s], exp_off);
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const bf16x8_t wv = decode8<FMT>(w[j][s][q], ls);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const bf16x2_t wp = {wv[2 * e], wv[2 * e + 1]};
#pragma unroll
              for (int m = 0; m < MR; ++m) {
                const uint32_t pair = af[m][q][e];  // a value first (see mx_gemv_kernel)
                acc[m * kGemvRows + j] = __builtin_amdgcn_fdot2_f32_bf16(wp, __builtin_bit_cast(bf16x2_t, pair), acc[m * kGemvRows + j], false);
              }
            }
          }
        }
        __builtin_amdgcn_sched_barrier(0);  // a step's fragments are read when the step before is done
      }
    }
    float t = RowReduce<16, 0>::run(acc, lane);
    t += __shfl_xor(t, 16);
    t += __shfl_xor(t, 32);
    const int m = (lane >> 2) & 3, n = b * kGemvRows + (lane & 3);
    if (lane < 16 && m < M && n < N) {
      // reference: C = bf16(float(acc) + float(Bias))
      if constexpr (HAS_BIAS) t += (float)Bias[(size_t)m * N + n];
      C[(size_t)m * N + n] = (bf16_t)t;
    }
  }
}

constexpr int kGemvLongMaxK = 32768;  // two rows of activations: 128 KiB of LDS

template <int FMT, bool HAS_BIAS, int MR>
int launch_mx_gemv_long(const void* A, const void* B, const void* S, const void* Bias, void* C, int M, int N, int K,
                        int exp_off, hipStream_t stream) {
  auto kern = mx_gemv_long_kernel<FMT, HAS_BIAS, MR>;
  static bool raised[kMaxDevices] = {};
  if (raise_lds_limit<MR * (kGemvLongMaxK / 2048) * 4096>(kern, raised)) return -1;
  const int nchunk = ((K >> 5) + 255) >> 8;
  const int lds = MR * 4 * nchunk * 4096;
  static int cus_of[kMaxDevices] = {};
  int device = 0;
  DQ_CHECK_HIP(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices) DQ_FAIL("device index %d is beyond the %d this library keeps state for", device, kMaxDevices);
  if (!cus_of[device]) DQ_CHECK_HIP(hipDeviceGetAttribute(&cus_of[device], hipDeviceAttributeMultiprocessorCount, device));
  // workgroups per CU: depends on K through the LDS a workgroup takes (asked once per device and chunk count)
  static int per_cu_of[kMaxDevices][kGemvLongMaxK / 8192 + 1] = {};
  int& per_cu = per_cu_of[device][nchunk];
  if (!per_cu) {
    DQ_CHECK_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kern, 256, lds));
    if (per_cu < 1) per_cu = 1;
  }
  const int nbatch = (N + kGemvRows - 1) / kGemvRows;
  const int want = (nbatch + 3) / 4, room = cus_of[device] * per_cu;
  hipLaunchKernelGGL(kern, dim3(want < room ? want : room), dim3(256), lds, stream, (const bf16_t*)A, (const uint8_t*)B,
                     (const uint8_t*)S, (const bf16_t*)Bias, (bf16_t*)C, M, N, K, exp_off);
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

}  // namespace

// 0: launched; 1: this shape is not the kernel's (the caller goes on to the tiled GEMM); -1: error.
// max_rows: the most activation rows to take (passes of 16, each streaming the weights again).
int mxfp4_gemm_regres(const void* A, const void* B, const void* S, const void* Bias, void* C, int M, int N, int K, int fmt,
                      int scale_bias, int max_rows, hipStream_t stream) {
  // 128-k chunks (the last one may be half: K % 128 == 64), at most eight per wave
  const bool longk = K > kWaves * kMaxChunks * 128;
  if (M < 1 || M > max_rows || K % 64 != 0 || (longk && K % 128 != 0)) return 1;
  // More than 16 rows run as passes of 16, each streaming the weights again: worth it while that stays ahead of the
  // tiled kernel, whose time up to 128 rows is one round of workgroups with all of K behind each (60 us at K = 8192,
  // 92 us from N = 16384 on).  Here the passes' workgroups come in rounds of one per CU, and a workgroup takes its
  // prologue (2 us + 2.5 us per 8192 k, once per slice of K) and 0.3 us + 2.8 us per 8192 k for every block of 16
  // weight rows it visits (measured at K = 8192: N = 8192 at 16 / 32 / 48 rows 13 / 24 / 35 us, N = 28672 at 16 rows
  // 26.6 us; N = K = 2880, where the passes share a round, 16 / 32 / 64 / 128 rows 6.7 / 11 / 16 / 29 us against 24.6 us).
  if (M > 16) {
    const double kfrac = (double)K / 8192.0;
    const int nslices = longk ? ((K >> 7) + kWaves * 6 - 1) / (kWaves * 6) : 1;
    const long grid = (N + 15) / 16 < 256 ? (N + 15) / 16 : 256, blocks_each = ((N + 15) / 16 + grid - 1) / grid;
    const long rounds = (grid * ((M + 15) / 16) + 255) / 256;
    const double t_here = 2.0 + 1.1 * (double)rounds * (2.0 * nslices + 2.5 * kfrac + (double)blocks_each * (0.3 * nslices + 2.8 * kfrac));
    const double t_tiled = (N > 16384 ? 92.0 : 60.0) * kfrac + 3.0;
    if (t_here > 0.9 * t_tiled) return 1;
  }
  const int exp_off = 127 - scale_bias;
  if (M == 1 && K <= 8192) {  // one row: the dot-product kernel
#define DQ_MXV(FMT_, STEPS_)                                                                                  \
  do {                                                                                                        \
    if (Bias) return launch_mx_gemv<FMT_, true, STEPS_>(A, B, S, Bias, C, N, K, exp_off, stream);             \
    return launch_mx_gemv<FMT_, false, STEPS_>(A, B, S, nullptr, C, N, K, exp_off, stream);                   \
  } while (0)
#define DQ_MXVN(FMT_)                 \
  do {                                \
    switch ((K + 2047) / 2048) {      \
      case 1: DQ_MXV(FMT_, 1);        \
      case 2: DQ_MXV(FMT_, 2);        \
      case 3: DQ_MXV(FMT_, 3);        \
      default: DQ_MXV(FMT_, 4);       \
    }                                 \
  } while (0)
    switch (fmt) {
      case FP4_E2M1: DQ_MXVN(FP4_E2M1);
      case FP4_SIMPLE: DQ_MXVN(FP4_SIMPLE);
      case FP4_TWIDDLING: DQ_MXVN(FP4_TWIDDLING);
      default: DQ_FAIL("mxfp4 gemm: unknown weight format %d", fmt);
    }
#undef DQ_MXVN
#undef DQ_MXV
  }
  // Two rows: the dot-product kernel with the activations in LDS (N = K = 8192: 10.1 against 12.7 us; N = 28672: level).
  // With four rows its 64 dot products per 16 bytes of weights are what binds (N = 28672, K = 8192: 31 against 25.5 us):
  // three and more rows go to the matrix-instruction kernel below.
  if (M == 2 && K <= 8192) {
#define DQ_MXW(FMT_, STEPS_)                                                                                   \
  do {                                                                                                         \
    if (Bias) return launch_mx_gemv_rows<FMT_, true, STEPS_, 2>(A, B, S, Bias, C, M, N, K, exp_off, stream);   \
    return launch_mx_gemv_rows<FMT_, false, STEPS_, 2>(A, B, S, nullptr, C, M, N, K, exp_off, stream);         \
  } while (0)
#define DQ_MXWN(FMT_)                 \
  do {                                \
    switch ((K + 2047) / 2048) {      \
      case 1: DQ_MXW(FMT_, 1);        \
      case 2: DQ_MXW(FMT_, 2);        \
      case 3: DQ_MXW(FMT_, 3);        \
      default: DQ_MXW(FMT_, 4);       \
    }                                 \
  } while (0)
    switch (fmt) {
      case FP4_E2M1: DQ_MXWN(FP4_E2M1);
      case FP4_SIMPLE: DQ_MXWN(FP4_SIMPLE);
      case FP4_TWIDDLING: DQ_MXWN(FP4_TWIDDLING);
      default: DQ_FAIL("mxfp4 gemm: unknown weight format %d", fmt);
    }
#undef DQ_MXWN
#undef DQ_MXW
  }
  if (M <= 2 && K > 8192 && K <= kGemvLongMaxK) {  // one and two rows, long K: the dot-product kernel over chunks of K
#define DQ_MXL(FMT_)                                                                                               \
  do {                                                                                                             \
    if (M == 1) {                                                                                                  \
      if (Bias) return launch_mx_gemv_long<FMT_, true, 1>(A, B, S, Bias, C, M, N, K, exp_off, stream);             \
      return launch_mx_gemv_long<FMT_, false, 1>(A, B, S, nullptr, C, M, N, K, exp_off, stream);                   \
    }                                                                                                              \
    if (Bias) return launch_mx_gemv_long<FMT_, true, 2>(A, B, S, Bias, C, M, N, K, exp_off, stream);               \
    return launch_mx_gemv_long<FMT_, false, 2>(A, B, S, nullptr, C, M, N, K, exp_off, stream);                     \
  } while (0)
    switch (fmt) {
      case FP4_E2M1: DQ_MXL(FP4_E2M1);
      case FP4_SIMPLE: DQ_MXL(FP4_SIMPLE);
      case FP4_TWIDDLING: DQ_MXL(FP4_TWIDDLING);
      default: DQ_FAIL("mxfp4 gemm: unknown weight format %d", fmt);
    }
#undef DQ_MXL
  }
  const bool half = K % 128 != 0;
  const int lines = K % 4096 == 0 ? 2 : (K % 256 == 0 ? 1 : 0);
  // chunks per wave: the longest run (with lines, whole pairs)
  const int nchunk = (K + 127) >> 7;
  const int ncw = lines ? 2 * ((nchunk / 2 + kWaves - 1) / kWaves) : (nchunk + kWaves - 1) / kWaves;
  if (half && ncw > 6) return 1;  // the half chunk's form with eight chunks per wave does not fit the registers
#define DQ_MXR(FMT_, NCW_, LINES_, HALF_, LONGK_)                                                                            \
  do {                                                                                                                       \
    if (Bias) return launch_mx_regres<FMT_, true, NCW_, LINES_, HALF_, LONGK_>(A, B, S, Bias, C, M, N, K, exp_off, stream); \
    return launch_mx_regres<FMT_, false, NCW_, LINES_, HALF_, LONGK_>(A, B, S, nullptr, C, M, N, K, exp_off, stream);       \
  } while (0)
#define DQ_MXRN(FMT_)                                                                                          \
  do {                                                                                                         \
    if (longk) { /* slices of at most 6144 k: six chunks per wave leave the registers the slice loop needs */ \
      if (lines) DQ_MXR(FMT_, 6, 1, false, true);                                                              \
      DQ_MXR(FMT_, 6, 0, false, true);                                                                         \
    }                                                                                                          \
    if (lines == 2 && ncw == 4) DQ_MXR(FMT_, 4, 2, false, false);                                              \
    if (lines == 2 && ncw == 8) DQ_MXR(FMT_, 8, 2, false, false);                                              \
    if (lines) {                                                                                               \
      if (ncw <= 2) DQ_MXR(FMT_, 2, 1, false, false);                                                          \
      if (ncw <= 4) DQ_MXR(FMT_, 4, 1, false, false);                                                          \
      if (ncw <= 6) DQ_MXR(FMT_, 6, 1, false, false);                                                          \
      DQ_MXR(FMT_, 8, 1, false, false);                                                                        \
    }                                                                                                          \
    if (half) {                                                                                                \
      if (ncw <= 2) DQ_MXR(FMT_, 2, 0, true, false);                                                           \
      if (ncw <= 4) DQ_MXR(FMT_, 4, 0, true, false);                                                           \
      DQ_MXR(FMT_, 6, 0, true, false);                                                                         \
    }                                                                                                          \
    if (ncw <= 2) DQ_MXR(FMT_, 2, 0, false, false);                                                            \
    if (ncw <= 4) DQ_MXR(FMT_, 4, 0, false, false);                                                            \
    if (ncw <= 6) DQ_MXR(FMT_, 6, 0, false, false);                                                            \
    DQ_MXR(FMT_, 8, 0, false, false);                                                                          \
  } while (0)
  switch (fmt) {
    case FP4_E2M1: DQ_MXRN(FP4_E2M1);
    case FP4_SIMPLE: DQ_MXRN(FP4_SIMPLE);
    case FP4_TWIDDLING: DQ_MXRN(FP4_TWIDDLING);
    default: DQ_FAIL("mxfp4 gemm: unknown weight format %d", fmt);
  }
#undef DQ_MXRN
#undef DQ_MXR
}

}  // namespace dq
