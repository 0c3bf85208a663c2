// BitNet W2A8 small batch (4 .. 32 activation rows; to 128 on matrices of few rows) on gfx950: activations resident in registers, weights streamed once.
//
// Replaces the batched use of the decode kernel of
// examples/bitnet-1.58b/kernel_benchmark/tilelang_bitnet_158_int8xint2_decode.py:66-176 (decoder
// decode_i2{u,s}_to_i8s, examples/dequantize_gemm/quantize/lop3.py:950-997; epilogue
// examples/bitnet-1.58b/utils_quant.py:165-170).  With a few dozen rows the problem is the weight stream: N x K / 4
// bytes that are used once.  The kernels built for hundreds of rows pull the activations through LDS again for every
// tile of weight rows, which costs the load unit several times the weight bytes; here nothing but weights moves
// after the prologue:
//
//   * one workgroup of eight waves per CU; wave w owns an eighth of K (a run of whole pairs of 128-k blocks, at most
//     four pairs: K <= 8192) and keeps the activations of its slice, in the matrix instruction's operand order, in
//     registers for the whole kernel: 32 rows x 1024 k = 128 registers per lane.  A longer K goes in chunks of at
//     most 6144, the kernel's body once per chunk, the finishing threads' running sums in LDS in between;
//   * the workgroups walk the blocks of 32 weight rows (block b, b + gridDim.x, ...).  Per block a wave loads its
//     slice of the 32 rows (eight 16-byte loads per lane at K = 8192), one block ahead of the arithmetic in a second
//     set of registers, decodes (7 instructions per 16 weights) and issues 32 matrix instructions of 32 x 32 x 32
//     against the resident activations;
//   * the eight partial sums of a block meet in LDS (4 KiB per wave, two buffers, one barrier per block); half the
//     threads add them in integer arithmetic (any order is exact), finish with the epilogue and store.
//
// Row-major weights: a load covers 16 rows x 64 bytes (lane l: row l / 4, piece l % 4: whole 64-byte runs) and two of
// them are regrouped into the operands of the pair's two blocks with one ds_bpermute_b32 per dword and one
// v_permlane16_swap_b32 per dword pair.  Fragment order (B[(N + 31) / 32][K / 128][64 lanes][16 bytes]): a load is
// 1 KiB contiguous and is the operand as it lands.  Every load is unconditional, so that the compiler's counting of
// outstanding loads stays exact: a wave whose slice has one pair fewer than the longest loads its last pair twice
// against activations of zero.
//
// Rows beyond N are read as the last row (row-major) or are the zeros of the padding (fragments); rows beyond M are
// read as row M - 1; neither is stored.
#include <type_traits>

#include "dq_common.h"
#include "dq_i2_codes.h"

namespace dq {

namespace {

constexpr int kWaves = 8;             // K slices
constexpr int kMaxPairs = 4;          // pairs of 128-k blocks per wave
constexpr int kChunkPairs = 3;        // the same when K goes in chunks
constexpr int kPartial = 32 * 32 * 4; // one wave's 32 x 32 sums
constexpr int kLds = 2 * kWaves * kPartial;
constexpr int kMaxRunning = 8;       // blocks of a workgroup whose running sums fit behind them (N <= 65536)

template <int CONV, bool FRAG, int NPW, bool CHUNKED, class FIN>
__global__ __launch_bounds__(64 * kWaves, 1) void i2_regres_kernel(const int8_t* __restrict__ A_all, const uint8_t* __restrict__ B,
                                                                   typename FIN::out_t* __restrict__ C_all, int M_all, int N, int K,
                                                                   int interleaved, FIN fin) {
  extern __shared__ __align__(16) unsigned char smem[];
  // more than 32 activation rows (small matrices only, see the launcher): workgroup row blockIdx.y takes rows
  // 32 blockIdx.y .. + 31 over all of the weights
  const int m_first = 32 * blockIdx.y;
  const int8_t* const A = A_all + (size_t)m_first * K;
  typename FIN::out_t* const C = C_all + (size_t)m_first * N;
  const int M = min(M_all - m_first, 32);
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 31;
  const int h = lane >> 5;

  // the thread's share of the final sum: activation row tid / 8, weight rows 4 (tid % 8) .. + 3 of the block.  (What
  // the epilogue needs of the row is fetched here, ahead of the activations: a load that could still be in flight
  // when the loop over the blocks begins would have the compiler wait for the blocks ahead at its first use.)
  const int out_m = tid >> 3, out_p = tid & 7;
  const bool finisher = tid < 256 && out_m < M;
  const typename FIN::row_t out_row = fin.row(finisher ? m_first + out_m : 0);

  // K beyond what the registers hold (8192): the kernel runs once per chunk of K, chunks of equal length up to a
  // pair; the finishing threads keep the running sums of the workgroup's blocks in LDS between the chunks.
  const int npair_all = K >> 8;
  const int nchunks = CHUNKED ? (npair_all + kWaves * NPW - 1) / (kWaves * NPW) : 1;
  const int row_blocks = (N + 31) >> 5;
  const int step = gridDim.x;  // at most the number of blocks: every workgroup has one
  int it = 0;
  for (int chunk = 0; chunk < nchunks; ++chunk) {
  const int it0 = it;
  if (chunk > 0) __syncthreads();  // the partial sums of the chunk before are read: their place is free
  // the wave's pairs of blocks: [p_lo, p_lo + npw), npw = NPW or NPW - 1
  const int c_lo = chunk * npair_all / nchunks;
  const int npair = (chunk + 1) * npair_all / nchunks - c_lo;
  const int p_lo = c_lo + wave * npair / kWaves;
  const int npw = c_lo + (wave + 1) * npair / kWaves - p_lo;
  auto pair_of = [&](int i) { return p_lo + min(i, max(npw - 1, 0)); };  // K < 2048: some waves have no pair at all

  // ---- weights: load (pair i, o) of the block of 32 rows nb
  uint32_t w_off[NPW][2];
#pragma unroll
  for (int i = 0; i < NPW; ++i)
#pragma unroll
    for (int o = 0; o < 2; ++o)
      w_off[i][o] = FRAG ? (uint32_t)((2 * pair_of(i) + o) * 1024 + lane * 16) : (uint32_t)(pair_of(i) * 64 + (lane & 3) * 16);
  const uint32_t row_bytes = (uint32_t)(K >> 2);
  auto load_w = [&](uint4_t (&w)[NPW][2], int nb) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < NPW; ++i)
#pragma unroll
      for (int o = 0; o < 2; ++o) {
        const uint8_t* src;
        if constexpr (FRAG) src = B + (size_t)nb * (size_t)(K >> 7) * 1024 + w_off[i][o];
        else src = B + (size_t)min(32 * nb + 16 * o + (lane >> 2), N - 1) * row_bytes + w_off[i][o];
        w[i][o] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(src));
      }
    // the loads go out here, ahead of the arithmetic of the block before: left to itself the scheduler sinks them
    // behind it to save registers, and the block ahead is then waited for right after it was asked for
    __builtin_amdgcn_sched_barrier(0);
  };
  // the first block's weights are asked for before the activations: the memory's first answer takes as long as the
  // prologue
  uint4_t w0[NPW][2], w1[NPW][2];
  int nb = blockIdx.x;
  load_w(w0, nb);

  // ---- activations: fragment (pair i, block b, step s): lane (r, h) holds k = 256 pair + 128 b + 64 h + 16 s .. + 15 of row r.
  // Fetched in that order a load instruction would touch 64 different cache lines for 16 bytes each, and the address
  // path of the CU's load unit (a line per cycle) made the prologue 7 us at 32 rows.  So a pair's 32 rows x 256 bytes
  // are loaded as whole lines (instruction j: rows 4 j .. 4 j + 3, lane l the 16-byte piece l % 16 of row 4 j + l / 16),
  // parked in 8 KiB of LDS of the wave's own (piece q of row m at position q ^ (m & 15)) and read back as fragments.
  // Up to 12 rows the lines are few either way (rows beyond M repeat row M - 1) and the direct form is the shorter
  // one: 18.9 against 19.4 us at 8 rows of N = 28672, K = 8192, 23.8 against 20.2 us at 32.
  int4_t af[NPW][2][4];
  if (M <= 12) {
    const int8_t* const a_row = A + (size_t)min(r, M - 1) * K + 64 * h;
    uint4_t raw[NPW][2][4];  // every load issued before the first is waited for
#pragma unroll
    for (int i = 0; i < NPW; ++i)
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int s = 0; s < 4; ++s) raw[i][b][s] = *reinterpret_cast<const uint4_t*>(a_row + 256 * pair_of(i) + 128 * b + 16 * s);
#pragma unroll
    for (int i = 0; i < NPW; ++i)
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const uint4_t a = interleaved ? raw[i][b][s] : transpose4x4_bytes(raw[i][b][s]);
          af[i][b][s] = __builtin_bit_cast(int4_t, i < npw ? a : uint4_t{0u, 0u, 0u, 0u});
        }
  } else {
    const int8_t* const a_lane = A + 16 * (lane & 15);
    uint4_t line[NPW][8];  // every load issued before the first is waited for
#pragma unroll
    for (int i = 0; i < NPW; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j)
        line[i][j] = *reinterpret_cast<const uint4_t*>(a_lane + (size_t)min(4 * j + (lane >> 4), M - 1) * K + 256 * pair_of(i));
    unsigned char* const park = smem + wave * 8192;
#pragma unroll
    for (int i = 0; i < NPW; ++i) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int row = 4 * j + (lane >> 4);
        *reinterpret_cast<uint4_t*>(park + row * 256 + (((lane & 15) ^ (row & 15)) << 4)) = line[i][j];
      }
      // a wave's LDS operations are carried out in the order they were issued: the reads below see the writes above,
      // and the next pair's writes come after them
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          uint4_t a = *reinterpret_cast<const uint4_t*>(park + r * 256 + (((8 * b + 4 * h + s) ^ (r & 15)) << 4));
          // plain packing: the decoder's dword j holds elements j, 4 + j, 8 + j, 12 + j of a fragment
          if (!interleaved) a = transpose4x4_bytes(a);
          af[i][b][s] = __builtin_bit_cast(int4_t, i < npw ? a : uint4_t{0u, 0u, 0u, 0u});
        }
    }
    __syncthreads();  // the parking areas are where the partial sums go
  }

  // lane (h, b, j) = 32 h + 16 b + j of the regrouped register takes lane 4 j + 2 b + h of the loaded one; afterwards
  // w[i][b] is the operand of block b of the pair: lane (r, h) holds k = 64 h .. 64 h + 63 of row r
  const int w_from = ((lane & 15) * 4 + ((lane >> 4) & 1) * 2 + (lane >> 5)) * 4;

  auto do_block = [&](uint4_t (&w)[NPW][2], int nb, int it) __attribute__((always_inline)) {
    int16_t_ acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0;
#pragma unroll
    for (int i = 0; i < NPW; ++i) {
      uint4_t x = w[i][0], y = w[i][1];
      if constexpr (!FRAG) {
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const uint32_t xd = (uint32_t)__builtin_amdgcn_ds_bpermute(w_from, (int)x[d]);
          const uint32_t yd = (uint32_t)__builtin_amdgcn_ds_bpermute(w_from, (int)y[d]);
          const auto sw = __builtin_amdgcn_permlane16_swap(xd, yd, false, false);
          x[d] = sw[0];
          y[d] = sw[1];
        }
      }
#pragma unroll
      for (int s = 0; s < 4; ++s) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(decode16<CONV>(x[s]), af[i][0][s], acc, 0, 0, 0);
#pragma unroll
      for (int s = 0; s < 4; ++s) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(decode16<CONV>(y[s]), af[i][1][s], acc, 0, 0, 0);
    }
    // Register group vg of lane (r, h) holds the weight rows 8 vg + 4 h .. + 3 of activation row r.  A wave's sums in
    // LDS: [32 activation rows][8 pieces of 4 weight rows], piece p of row m at position p ^ (m & 7).
    unsigned char* const buf = smem + (it & 1) * (kWaves * kPartial);
    if (r < M) {
#pragma unroll
      for (int vg = 0; vg < 4; ++vg) {
        const int4_t v = {acc[4 * vg], acc[4 * vg + 1], acc[4 * vg + 2], acc[4 * vg + 3]};
        *reinterpret_cast<int4_t*>(buf + wave * kPartial + r * 128 + (((2 * vg + h) ^ (r & 7)) << 4)) = v;
      }
    }
    // One barrier per block: the buffer written here is read below and written again two blocks later, after the next
    // block's barrier, which no thread passes before it has finished reading here.
    __syncthreads();
    const int m = out_m, p = out_p;
    if (finisher) {
      int4_t sum = {0, 0, 0, 0};
#pragma unroll
      for (int w8 = 0; w8 < kWaves; ++w8) sum += *reinterpret_cast<const int4_t*>(buf + w8 * kPartial + m * 128 + ((p ^ (m & 7)) << 4));
      // the running sum of this thread's four outputs of the workgroup's block number it - it0, behind the buffers
      int4_t* const running = reinterpret_cast<int4_t*>(smem + kLds + (it - it0) * kPartial + m * 128 + p * 16);
      if (chunk > 0) sum += *running;
      if (chunk + 1 < nchunks) *running = sum;
      using out_t = typename FIN::out_t;
      constexpr int kShift = Codes<CONV>::kShift;
      const int n = 32 * nb + 4 * p;
      if (chunk + 1 == nchunks && n < N) {
        out_t o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = fin.finish(sum[e] >> kShift, out_row);
        out_t* const dst = C + (size_t)m * N + n;
        if ((N & 3) == 0) {
          typedef out_t out4_t __attribute__((ext_vector_type(4)));
          *reinterpret_cast<out4_t*>(dst) = out4_t{o[0], o[1], o[2], o[3]};
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < N) dst[e] = o[e];
        }
      }
    }
  };

  // Two sets of weight registers, a block ahead: the loads of block nb + gridDim.x are issued before block nb is waited
  // for.  The last block of a workgroup has its own copy of the code: a load under a condition would make the compiler
  // count the loads in flight for the path without it, and wait for the block ahead before it computes.
  // (Asking for block nb + 2 gridDim.x pair by pair as block nb's registers come free needs copies of them that no
  // longer fit the 256 registers: the kernel then spills.)
  for (;;) {
    if (nb + step >= row_blocks) {
      do_block(w0, nb, it);
      break;
    }
    load_w(w1, nb + step);
    do_block(w0, nb, it);
    nb += step;
    ++it;
    if (nb + step >= row_blocks) {
      do_block(w1, nb, it);
      break;
    }
    load_w(w0, nb + step);
    do_block(w1, nb, it);
    nb += step;
    ++it;
  }
  ++it;  // the last block's
  }  // chunks of K
}

// ---- up to 16 activation rows -------------------------------------------------------------------------------------
// The same kernel on the 16 x 16 x 64 matrix instruction: blocks of 16 weight rows (N = 28672 is 1792 blocks, seven
// per workgroup, where blocks of 32 are three and a half), the activations of a wave's eighth of K in 64 registers,
// and the registers that frees hold four blocks of weights instead of two: three blocks (96 KiB per CU) are asked for
// ahead of the one being decoded.  A pair of 128-k blocks of 16 rows is 1 KiB: one load per lane.  Row-major: lane l
// reads piece l % 4 of row l / 4 (whole 64-byte runs) and one ds_bpermute_b32 per dword hands lane (g, r) piece g of
// row r; fragment order: lane (g, r) reads entry (block 2 pair + g / 2, lane 32 (g % 2) + 16 (nb % 2) + r) of the
// 32-row fragment block nb / 2, which is that piece.  Dword s of a lane feeds step s: contraction index
// k = 256 pair + 64 g + 16 s + e for both operands.
// The loads of the last three blocks' turns have nothing left to ask for and read block 0 instead (the same 32 KiB
// for every workgroup, from L2, never used): a load under a condition would make the compiler wait for more than
// the block it needs.
constexpr int kDepth16 = 4;               // sets of weight registers
constexpr int kPartial16 = 16 * 16 * 4;   // one wave's 16 x 16 sums
constexpr int kLds16 = kWaves * 4096;     // the prologue's parking areas; the two buffers of partial sums reuse them

template <int CONV, bool FRAG, int NPW, class FIN>
__global__ __launch_bounds__(64 * kWaves, 1) void i2_regres16_kernel(const int8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                                     typename FIN::out_t* __restrict__ C, int M, int N, int K,
                                                                     int interleaved, FIN fin) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15;
  const int g = lane >> 4;

  const int npair = K >> 8;
  const int p_lo = wave * npair / kWaves;
  const int npw = (wave + 1) * npair / kWaves - p_lo;
  auto pair_of = [&](int i) { return p_lo + min(i, max(npw - 1, 0)); };

  const int row_blocks = (N + 15) >> 4;
  const int step = gridDim.x;  // at most the number of blocks: every workgroup has one
  const int nb0 = blockIdx.x;
  const int mine = (row_blocks - nb0 + step - 1) / step;

  uint32_t w_off[NPW];
#pragma unroll
  for (int i = 0; i < NPW; ++i)
    w_off[i] = FRAG ? (uint32_t)((2 * pair_of(i) + (g >> 1)) * 1024 + (32 * (g & 1) + r) * 16) : (uint32_t)(pair_of(i) * 64 + (lane & 3) * 16);
  const uint32_t row_bytes = (uint32_t)(K >> 2);
  auto load_w = [&](uint4_t (&w)[NPW], int nb_asked, bool real) __attribute__((always_inline)) {
    const int nb = real ? nb_asked : 0;
    const uint8_t* base;
    if constexpr (FRAG) base = B + (size_t)(nb >> 1) * (size_t)(K >> 7) * 1024 + (nb & 1) * 256;
    else base = B + (size_t)min(16 * nb + (lane >> 2), N - 1) * row_bytes;
#pragma unroll
    for (int i = 0; i < NPW; ++i) w[i] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(base + w_off[i]));
    __builtin_amdgcn_sched_barrier(0);  // the loads go out here, see load_w of the kernel above
  };
  // the thread's share of the final sum: activation row tid / 4, weight rows 4 (tid % 4) .. + 3 of the block (fetched
  // ahead of the activations, see the kernel above)
  const int out_m = tid >> 2, out_p = tid & 3;
  const bool finisher = tid < 64 && out_m < M;
  const typename FIN::row_t out_row = fin.row(finisher ? out_m : 0);
  uint4_t w[kDepth16][NPW];
  // Loads come back in the order they went out, and the first block's arithmetic needs the first block and the
  // activations: the two blocks ahead go out behind the activations.
  load_w(w[0], nb0, true);

  // ---- activations: fragment (pair i, step s): lane (g, r) holds k = 256 pair + 64 g + 16 s .. + 15 of row r; read as
  // whole lines (instruction j: rows 4 j .. 4 j + 3, lane l the piece l % 16 of row 4 j + l / 16), parked in the
  // wave's 4 KiB of LDS (piece q of row m at position q ^ m) and read back in operand order
  int4_t af[NPW][4];
  {
    const int8_t* const a_lane = A + 16 * (lane & 15);
    uint4_t line[NPW][4];
#pragma unroll
    for (int i = 0; i < NPW; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        line[i][j] = *reinterpret_cast<const uint4_t*>(a_lane + (size_t)min(4 * j + (lane >> 4), M - 1) * K + 256 * pair_of(i));
    __builtin_amdgcn_sched_barrier(0);
    load_w(w[1], nb0 + step, mine > 1);
    load_w(w[2], nb0 + 2 * step, mine > 2);
    unsigned char* const park = smem + wave * 4096;
#pragma unroll
    for (int i = 0; i < NPW; ++i) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int row = 4 * j + (lane >> 4);
        *reinterpret_cast<uint4_t*>(park + row * 256 + (((lane & 15) ^ row) << 4)) = line[i][j];
      }
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        uint4_t a = *reinterpret_cast<const uint4_t*>(park + r * 256 + (((4 * g + s) ^ r) << 4));
        if (!interleaved) a = transpose4x4_bytes(a);  // plain packing: the decoder's dword j holds elements j, 4 + j, 8 + j, 12 + j
        af[i][s] = __builtin_bit_cast(int4_t, i < npw ? a : uint4_t{0u, 0u, 0u, 0u});
      }
    }
    __syncthreads();  // the parking areas are where the partial sums go
  }

  const int w_from = ((lane & 15) * 4 + (lane >> 4)) * 4;  // lane (g, r) of the regrouped register takes lane 4 r + g

  auto do_block = [&](auto q_tag, int k) __attribute__((always_inline)) {
    constexpr int q = decltype(q_tag)::value;
    const int nb = nb0 + k * step;
    load_w(w[(q + 3) % kDepth16], nb + 3 * step, k + 3 < mine);
    int4_t acc = {0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < NPW; ++i) {
      uint4_t x = w[q][i];
      if constexpr (!FRAG) {
#pragma unroll
        for (int d = 0; d < 4; ++d) x[d] = (uint32_t)__builtin_amdgcn_ds_bpermute(w_from, (int)x[d]);
      }
#pragma unroll
      for (int s = 0; s < 4; ++s) acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(decode16<CONV>(x[s]), af[i][s], acc, 0, 0, 0);
    }
    // lane (g, r) holds the weight rows 4 g .. 4 g + 3 of activation row r.  A wave's sums in LDS: [16 activation
    // rows][4 pieces of 4 weight rows], piece p of row m at position p ^ (m & 3).
    unsigned char* const buf = smem + (k & 1) * (kWaves * kPartial16);
    if (r < M) *reinterpret_cast<int4_t*>(buf + wave * kPartial16 + r * 64 + ((g ^ (r & 3)) << 4)) = acc;
    __syncthreads();  // one per block, see the kernel above
    if (finisher) {
      const int m = out_m, p = out_p;
      int4_t sum = {0, 0, 0, 0};
#pragma unroll
      for (int w8 = 0; w8 < kWaves; ++w8) sum += *reinterpret_cast<const int4_t*>(buf + w8 * kPartial16 + m * 64 + ((p ^ (m & 3)) << 4));
      using out_t = typename FIN::out_t;
      constexpr int kShift = Codes<CONV>::kShift;
      const int n = 16 * nb + 4 * p;
      if (n < N) {
        out_t o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = fin.finish(sum[e] >> kShift, out_row);
        out_t* const dst = C + (size_t)m * N + n;
        if ((N & 3) == 0) {
          typedef out_t out4_t __attribute__((ext_vector_type(4)));
          *reinterpret_cast<out4_t*>(dst) = out4_t{o[0], o[1], o[2], o[3]};
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < N) dst[e] = o[e];
        }
      }
    }
  };
  // Whole turns of the four register sets in a loop without an exit in its body, the last one to three blocks after
  // it: an exit between two blocks would share its way out with the loop's way round, and the compiler would count
  // the loads in flight at the top of the loop as if it could have come from there.
  int k = 0;
  for (; k + kDepth16 <= mine; k += kDepth16) {
    do_block(std::integral_constant<int, 0>{}, k);
    do_block(std::integral_constant<int, 1>{}, k + 1);
    do_block(std::integral_constant<int, 2>{}, k + 2);
    do_block(std::integral_constant<int, 3>{}, k + 3);
  }
  if (k < mine) {
    do_block(std::integral_constant<int, 0>{}, k);
    if (k + 1 < mine) {
      do_block(std::integral_constant<int, 1>{}, k + 1);
      if (k + 2 < mine) do_block(std::integral_constant<int, 2>{}, k + 2);
    }
  }
}

template <int CONV, bool FRAG, int NPW, class FIN>
int launch_i2_regres16(const void* A, const void* B, void* C, int M, int N, int K, int interleaved, FIN fin, hipStream_t stream) {
  auto kern = i2_regres16_kernel<CONV, FRAG, NPW, FIN>;
  static bool raised[kMaxDevices] = {};
  if (raise_lds_limit<kLds16>(kern, raised)) return -1;
  static int cus_of[kMaxDevices] = {};
  int device = 0;
  DQ_CHECK_HIP(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices) DQ_FAIL("device index %d is beyond the %d this library keeps state for", device, kMaxDevices);
  if (!cus_of[device]) DQ_CHECK_HIP(hipDeviceGetAttribute(&cus_of[device], hipDeviceAttributeMultiprocessorCount, device));
  const int row_blocks = (N + 15) / 16;
  const int grid = row_blocks < cus_of[device] ? row_blocks : cus_of[device];
  hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * kWaves), kLds16, stream, (const int8_t*)A, (const uint8_t*)B,
                     (typename FIN::out_t*)C, M, N, K, interleaved, fin);
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

template <int CONV, bool FRAG, int NPW, bool CHUNKED, class FIN>
int launch_i2_regres(const void* A, const void* B, void* C, int M, int N, int K, int interleaved, FIN fin, hipStream_t stream) {
  auto kern = i2_regres_kernel<CONV, FRAG, NPW, CHUNKED, FIN>;
  static bool raised[kMaxDevices] = {};
  if (raise_lds_limit<kLds + kMaxRunning * kPartial>(kern, raised)) return -1;
  static int cus_of[kMaxDevices] = {};
  int device = 0;
  DQ_CHECK_HIP(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices) DQ_FAIL("device index %d is beyond the %d this library keeps state for", device, kMaxDevices);
  if (!cus_of[device]) DQ_CHECK_HIP(hipDeviceGetAttribute(&cus_of[device], hipDeviceAttributeMultiprocessorCount, device));
  const int cus = cus_of[device];
  const int row_blocks = (N + 31) / 32;
  const int passes = (M + 31) / 32;
  // see i2_gemm_regres: one round of workgroups, or one and a half when K is short enough for one chunk (N = 3072,
  // K = 8192 at 128 rows: 17.6 us against 24.6 us of the K-sliced kernel; N = 8192, K = 28672 at 64 rows, two full
  // rounds of chunked work: 67 against 58 us)
  if (passes > 1 && (long)row_blocks * passes > (CHUNKED ? 2L : 3L) * cus / 2) return 1;
  const int grid = row_blocks < cus ? row_blocks : cus;
  // K in chunks: the running sums of a workgroup's blocks live behind the two buffers of partial sums
  const int mine = (row_blocks + grid - 1) / grid;
  if (CHUNKED && mine > kMaxRunning) return 1;
  const int lds = kLds + (CHUNKED ? mine * kPartial : 0);
  hipLaunchKernelGGL(kern, dim3(grid, passes), dim3(64 * kWaves), lds, stream, (const int8_t*)A, (const uint8_t*)B,
                     (typename FIN::out_t*)C, M, N, K, interleaved, fin);
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

}  // namespace

// 0: launched; 1: this shape is not the kernel's (the caller goes on to the kernels for more rows); -1: error.
int i2_gemm_regres(const void* A, const void* B, void* C, int M, int N, int K, int convention, int layout, const void* s_a,
                   float s_w, int bitnet_epilogue, hipStream_t stream) {
  // whole pairs of 128-k blocks, at most four per wave; the rows of one block of the matrix instruction
  // More than 32 rows: every 32 of them stream the weights again, which pays while the whole of it is about one
  // round of workgroups, i.e. on matrices of few rows, where the kernels for hundreds of activation rows have a
  // handful of tiles (N = 4096, K = 4096 at 64 rows: 14.9 us there, 6.5 us here); the launcher returns 1 beyond that.
  if (M < 1 || M > 128 || K % 256 != 0) return 1;
  if ((uint64_t)(N + 32) * (uint64_t)(K >> 2) >= (1ull << 32)) return 1;  // 32-bit lane offsets inside a row block's loads
  // Up to K = 8192 the activations of all of K stay in registers (one to four pairs of blocks per wave).  Beyond, K
  // goes in chunks of at most 6144, equal up to a pair: three pairs per wave leave the registers that the chunk loop
  // needs (with four the compiler spilled).
  const int npair = K >> 8;
  const bool chunked = npair > kWaves * kMaxPairs;
  const int npw = chunked ? kChunkPairs : (npair + kWaves - 1) / kWaves;
  const int il = (layout & ~LAYOUT_FRAGMENTS) == LAYOUT_INTERLEAVED;
  const bool frag = (layout & LAYOUT_FRAGMENTS) != 0;
  // Up to 16 rows the form on blocks of 16 weight rows: it divides the matrix over more workgroups and holds three
  // blocks in flight (N = 28672, K = 8192: 15.8 against 19.0 us; N = K = 8192 at 16 rows 9.1 against 10.5 us; N = 2048,
  // K = 8192: 7.6 against 9.8 us; N = K = 4096: 5.3 against 6.6 us).  With K below 4096 only where a workgroup has more
  // than four of them: its longer prologue shows (N = 8192, K = 2048 at 4 and 8 rows: 4.8 against 4.5 us).
  const bool rows16 = M <= 16 && (K >= 4096 || (N + 15) / 16 > 4 * 256);
#define DQ_I2R(CONV_, FRAG_, NPW_, CH_)                                                                                        \
  do {                                                                                                                         \
    if (bitnet_epilogue)                                                                                                       \
      return launch_i2_regres<CONV_, FRAG_, NPW_, CH_>(A, B, C, M, N, K, il, BitnetFinish{(const float*)s_a, s_w}, stream);    \
    return launch_i2_regres<CONV_, FRAG_, NPW_, CH_>(A, B, C, M, N, K, il, Int32Finish{}, stream);                             \
  } while (0)
#define DQ_I2R16(CONV_, FRAG_, NPW_)                                                                                     \
  do {                                                                                                                   \
    if (bitnet_epilogue)                                                                                                 \
      return launch_i2_regres16<CONV_, FRAG_, NPW_>(A, B, C, M, N, K, il, BitnetFinish{(const float*)s_a, s_w}, stream); \
    return launch_i2_regres16<CONV_, FRAG_, NPW_>(A, B, C, M, N, K, il, Int32Finish{}, stream);                          \
  } while (0)
#define DQ_I2RN(CONV_, FRAG_)                           \
  do {                                                  \
    if (chunked) DQ_I2R(CONV_, FRAG_, kChunkPairs, true); \
    if (rows16) {                                       \
      switch (npw) {                                    \
        case 1: DQ_I2R16(CONV_, FRAG_, 1);              \
        case 2: DQ_I2R16(CONV_, FRAG_, 2);              \
        case 3: DQ_I2R16(CONV_, FRAG_, 3);              \
        default: DQ_I2R16(CONV_, FRAG_, 4);             \
      }                                                 \
    }                                                   \
    switch (npw) {                                      \
      case 1: DQ_I2R(CONV_, FRAG_, 1, false);           \
      case 2: DQ_I2R(CONV_, FRAG_, 2, false);           \
      case 3: DQ_I2R(CONV_, FRAG_, 3, false);           \
      default: DQ_I2R(CONV_, FRAG_, 4, false);          \
    }                                                   \
  } while (0)
#define DQ_I2RL(CONV_)                  \
  do {                                  \
    if (frag) DQ_I2RN(CONV_, true);     \
    DQ_I2RN(CONV_, false);              \
  } while (0)
  switch (convention) {
    case I2_UNSIGNED: DQ_I2RL(I2_UNSIGNED);
    case I2_OFFSET: DQ_I2RL(I2_OFFSET);
    case I2_TWOS: DQ_I2RL(I2_TWOS);
    default: DQ_FAIL("int2 gemm: unknown code convention %d", convention);
  }
#undef DQ_I2RL
#undef DQ_I2RN
#undef DQ_I2R16
#undef DQ_I2R
}

}  // namespace dq
