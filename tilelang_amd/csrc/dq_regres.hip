// W4A16 decode kernel for 2 <= M <= 16 activation rows on gfx950: activations resident in REGISTERS.
//
// Replaces the batched use (up to 16 tokens) of the kernel generated from
// examples/dequantize_gemm/example_dequant_gemv_fp16xint4.py:83-153 with the group scales / zeros
// of examples/dequantize_gemm/quantize/lop3.py:41-81,136-176.  16 activation rows of K = 8192 are
// 256 KiB: too much for the LDS of a CU, but half of its register file.  So a workgroup is 16 waves
// (1024 threads, one workgroup per CU), wave w keeps the activations of its K/16 slice in MFMA
// operand registers for the whole kernel, and only weights, scales and zeros cross the memory
// system, with the access pattern and the occupancy of the M = 1 GEMV:
//
//   * the workgroup walks blocks of 16 weight rows; the 16 waves together read each row of a block
//     contiguously (wave w: K/32 bytes at offset w K/32), lane (g = lane / 16, r = lane % 16)
//     loading 16 bytes = 32 consecutive k of row r per 128-k chunk; a lane's registers are
//     refilled with the next block's weights as soon as they are consumed;
//   * each dword is decoded to the exact fp16 tile values (decode_w4) and is the 16 x 32 operand
//     of one v_mfma_f32_16x16x32_f16 against the resident activation operand (lanes with r >= M
//     hold copies of the last row; their output columns are never stored);
//   * the 16 K-slice partials of a row block are summed through LDS in a fixed order, one barrier
//     per row block (double-buffered): results are bit-identical from run to run.
#include "dq_common.h"

#include <type_traits>

namespace dq {

namespace {

// NC consecutive fp16 values (the scales of a wave's chunks) with one load.
template <int NC>
__device__ __forceinline__ uint2_t load_halves(const half_t* p) {
  if constexpr (NC == 4) return *reinterpret_cast<const uint2_t*>(p);
  else if constexpr (NC == 2) return uint2_t{*reinterpret_cast<const uint32_t*>(p), 0u};
  else return uint2_t{(uint32_t) * reinterpret_cast<const unsigned short*>(p), 0u};
}
__device__ __forceinline__ half_t pick_half(uint2_t v, int c) {
  const half2_t h = as_half2(c < 2 ? v[0] : v[1]);
  return (c & 1) ? h[1] : h[0];
}

// NC: 128-k chunks per wave (K = 2048 NC).  64 NC activation bytes per lane stay in registers.
template <int NC, int MODE, bool APERM>
__global__ __launch_bounds__(1024) void w4a16_regres_kernel(const half_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                             const half_t* __restrict__ S, const half_t* __restrict__ Z,
                                                             half_t* __restrict__ C, int M, int N, int K, int rbn) {
  __shared__ float red[2][16][256];  // [buffer][wave][lane * 4 + i]
  constexpr bool kScale = MODE >= W4_SCALE;
  constexpr bool kZeros = MODE >= W4_ZEROS_ORIGINAL;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int g = lane >> 4;
  const int r = lane & 15;
  const int nrb = (N + 15) >> 4;
  const int rb0 = blockIdx.x * rbn;
  const int nrb_wg = min(rbn, nrb - rb0);  // > 0 by construction of the grid
  const uint32_t row_bytes = (uint32_t)(K >> 1);
  const int groups_per_row = K >> 7;
  const int chunk0 = wave * NC;  // first 128-k chunk (= scale group) of this wave

  uint4_t bq[NC];
  uint2_t sc = {0u, 0u}, zp = {0u, 0u}, sc_next = {0u, 0u}, zp_next = {0u, 0u};  // NC scales / zeros of a row block
  // 32-bit byte offsets of this lane's row of the current / next row block from the (uniform) bases; N is
  // a multiple of 16 here, so every row of a block exists
  uint32_t w_off = (uint32_t)(rb0 * 16 + r) * row_bytes + (uint32_t)chunk0 * 64u + (uint32_t)g * 16u;
  uint32_t s_off = ((uint32_t)(rb0 * 16 + r) * (uint32_t)groups_per_row + (uint32_t)chunk0) * 2u;
  const unsigned char* Sb = reinterpret_cast<const unsigned char*>(S);
  const unsigned char* Zb = reinterpret_cast<const unsigned char*>(Z);
  auto load_chunk = [&](int c) {  // chunk c of the row block that w_off / s_off point at
    bq[c] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(B + w_off + c * 64));
    if (c == 0) {  // the block's scales travel with its first chunk
      if constexpr (kScale) sc_next = load_halves<NC>(reinterpret_cast<const half_t*>(Sb + s_off));
      if constexpr (kZeros) zp_next = load_halves<NC>(reinterpret_cast<const half_t*>(Zb + s_off));
    }
  };
  // the first block's weights go out before the activations are fetched
#pragma unroll
  for (int c = 0; c < NC; ++c) load_chunk(c);
  w_off += 16u * row_bytes;  // from here on they point at the next row block
  s_off += 32u * (uint32_t)groups_per_row;

  // resident activations: y[c][j] is the operand of MFMA step j of chunk c
  uint4_t y[NC][4];
  {
    const half_t* ap = A + (size_t)min(r, M - 1) * K + (size_t)chunk0 * 128 + g * 32;
#pragma unroll
    for (int c = 0; c < NC; ++c)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint4_t d = *reinterpret_cast<const uint4_t*>(ap + c * 128 + j * 8);
        y[c][j] = APERM ? permute_k8_16bit(d) : d;
      }
  }

  for (int rb = 0; rb < nrb_wg; ++rb) {
    float4_t acc = {0.f, 0.f, 0.f, 0.f};
    sc = sc_next;
    zp = zp_next;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const half_t s = kScale ? pick_half(sc, c) : (half_t)1.f;
      const half_t z = kZeros ? pick_half(zp, c) : (half_t)0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const half8_t x = decode_w4<MODE>(bq[c][j], s, z);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(x, __builtin_bit_cast(half8_t, y[c][j]), acc, 0, 0, 0);
      }
      // this chunk's registers are free: refill them with the next row block (kept behind the
      // arithmetic above and ahead of the next chunk's by the scheduling barriers)
      if (rb + 1 < nrb_wg) {
        __builtin_amdgcn_sched_barrier(0);
        load_chunk(c);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    w_off += 16u * row_bytes;
    s_off += 32u * (uint32_t)groups_per_row;
    // acc[i] = partial C[m = r][(rb0 + rb) * 16 + g * 4 + i] over this wave's K slice
    float* buf = &red[rb & 1][0][0];
    *reinterpret_cast<float4_t*>(buf + wave * 256 + lane * 4) = acc;
    __syncthreads();  // the other buffer is rewritten only after the next barrier
    if (tid < 256) {
      float v = buf[tid];
#pragma unroll
      for (int w = 1; w < 16; ++w) v += buf[w * 256 + tid];
      const int src_lane = tid >> 2, i = tid & 3;
      const int m = src_lane & 15;
      const int n = (rb0 + rb) * 16 + (src_lane >> 4) * 4 + i;
      if (m < M && n < N) C[(size_t)m * N + n] = (half_t)v;
    }
  }
}

// ---- the same kernel with the scale applied per 128-k group in fp32 ------------------------------------------
// The exact decoder above spends 17 to 21 VALU instructions per packed dword on reproducing the fp16 rounding of
// every weight; here a dword costs 7: every nibble becomes the exact fp16 value 64 + q ((x & 0x00F000F0) | 0x5400
// after the nibble is shifted to bits 4..7), the matrix instruction multiplies the activations with 64 + q, a
// 128-k group (one chunk of a wave) gets an accumulator of its own, and
//     s * (sum_k a_k (64 + q_k) - (64 + z) * sum_k a_k)  =  sum_k a_k (q_k - z) s
// is formed once per group and output in fp32 (two FMAs).  sum_k a_k over a wave's chunk comes out of the same
// matrix instruction against an operand of ones, once, in exactly the output layout.  The result is the fp32 dot
// product of A with the exact (q - z) * s; the per-weight fp16 rounding of the reference's tile (relative 2^-11)
// is not reproduced, as in the M <= 4 GEMV.  Operand roles are swapped against the kernel above (activations
// first), so that lane (g, r) ends up with outputs of weight row r: its scale and zero are the ones it loaded.
// Modes: everything of the form (q' - z) * s with q' = q or q ^ 8; "rescale" stays on the exact kernels.
template <bool FLIP>
__device__ __forceinline__ half8_t decode_w4_bias64(uint32_t w) {
  if constexpr (FLIP) w ^= 0x88888888u;
  uint32_t m = 0x00F000F0u;
  asm("" : "+v"(m));  // keep the mask in a VGPR: (x & m) | k is then one v_and_or_b32
  uint4_t t;
  t[0] = ((w << 4) & m) | 0x54005400u;  // (n0, n4)
  t[1] = (w & m) | 0x54005400u;         // (n1, n5)
  t[2] = ((w >> 4) & m) | 0x54005400u;  // (n2, n6)
  t[3] = ((w >> 8) & m) | 0x54005400u;  // (n3, n7)
  return __builtin_bit_cast(half8_t, t);
}

// NC consecutive fp16 values (NC = 1, 2, 4 or 8) with one load.
// NC consecutive fp16 values (NC = 1, 2, 4 or 8) with one buffer load; a range check that fails returns zeros.
template <int NC>
struct Halves {
  uint32_t w[(NC + 1) / 2];
};
template <int NC>
__device__ __forceinline__ Halves<NC> load_halves_n(__amdgpu_buffer_rsrc_t rsrc, uint32_t voff, uint32_t soff) {
  Halves<NC> h;
  if constexpr (NC == 8) {
    const uint4_t v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff, soff, 0);
    h.w[0] = v[0]; h.w[1] = v[1]; h.w[2] = v[2]; h.w[3] = v[3];
  } else if constexpr (NC == 4) {
    const uint2_t v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, voff, soff, 0);
    h.w[0] = v[0]; h.w[1] = v[1];
  } else if constexpr (NC == 2) {
    h.w[0] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, voff, soff, 0);
  } else {
    h.w[0] = __builtin_amdgcn_raw_buffer_load_b16(rsrc, voff, soff, 0);
  }
  return h;
}
template <int NC>
__device__ __forceinline__ float half_at(const Halves<NC>& h, int c) {
  const half2_t v = as_half2(h.w[c >> 1]);
  return (float)((c & 1) ? v[1] : v[0]);
}

constexpr uint32_t kBufferFlags = 0x00020000u;  // raw buffer of 32-bit data, the range check on
constexpr uint32_t kOutOfRange = 0xFFFFF000u;   // an offset no matrix of this kernel reaches

// WAVES waves (8 or 16) share K: wave w owns the NC chunks of 128 k from chunk w NC on (K = 128 NC WAVES) and keeps
// their activations in 16 NC registers.  DEPTH row blocks of weights (1 or 2) are in flight per lane.
// PARK: the activations of the wave's last PARK chunks live in LDS instead of registers (16 registers per chunk
// freed for weights in flight; a parked operand is read back with one 16-byte LDS read per matrix instruction).
//
// Every load of the main loop is a buffer load issued unconditionally: a row block past the workgroup's last one
// is asked for at an offset beyond the buffer, which returns zeros without touching memory.  The loop body is
// therefore straight-line code, and the waits the compiler places in front of each chunk count exactly the loads
// that were issued after that chunk's (a load behind a branch makes it wait for all of them at the loop's end,
// which exposes the whole memory latency once per row block).
//
// TR (one block in flight): the weights are fetched row-contiguously -- an instruction reads 1024 / S rows x S bytes,
// S = 64 NC the bytes of a row in the wave's K slice (4 rows x 256 bytes at K = 8192) -- which streams at 6.0 TB/s
// where the matrix instruction's own operand layout (16 rows x 64 bytes per instruction) streams at 4.8 TB/s, and a
// block is transposed into that layout through a 16 S-byte LDS area of the wave's own: 16-byte writes as loaded,
// 16-byte reads as multiplied, the pieces of row r XOR-swizzled with r so that neither side has bank conflicts.
// LDS operations of one wave execute in order, so no barrier and no second area is needed.
// FRAG: the weights were re-ordered offline into the matrix instruction's operand order (quantize.prepack_w4_fragments:
// [N / 16][K / 128][64 lanes][16 bytes], lane 16 g + r holding piece g of row r of the chunk), so an instruction reads
// 1 KiB contiguous straight into the operand layout and nothing is transposed.
template <int WAVES, int NC, int DEPTH, int PARK, bool TR, bool FRAG, bool HAS_SCALE, bool HAS_ZEROS, bool FLIP, bool APERM>
__global__ __launch_bounds__(64 * WAVES) void w4a16_regres_fast_kernel(const half_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                                        const half_t* __restrict__ S, const half_t* __restrict__ Z,
                                                                        half_t* __restrict__ C, int M, int N, int K, int rbn,
                                                                        float zconst) {
  __shared__ float red[2][WAVES][256];  // [buffer][wave][lane * 4 + i]
  // per wave, chunk and lane group: the sums over the chunk's 128 k of activation rows m = 4 g + i
  __shared__ float4_t asum_lds[WAVES][NC][4];
  __shared__ uint4_t ypark[WAVES][PARK > 0 ? PARK : 1][4][64];
  // group scales and zeros of a row block, staged by the whole workgroup: [slot][scales, zeros][row]; a row is its
  // K / 128 fp16 values (at most 128 bytes) plus 8 bytes that spread the rows over the banks
  constexpr int kSzRow = 136;
  __shared__ __align__(16) unsigned char sz_lds[2][2][16 * kSzRow + 16];  // + a word that idle threads write to
  constexpr int NR = NC - PARK;  // chunks whose activations stay in registers
  static_assert(!TR || DEPTH == 1, "the transposing form keeps one block in flight");
  static_assert(!(TR && FRAG), "fragment-ordered weights need no transposition");
  constexpr int LPR = 4 * NC;    // TR: lanes (16-byte pieces) per row of the wave's slice
  constexpr int RPI = 64 / LPR;  // TR: rows per load instruction
  __shared__ uint4_t wstage[(TR || FRAG) ? WAVES : 1][(TR || FRAG) ? 256 : 1];  // 16 rows x up to 256 bytes per wave
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int g = lane >> 4;
  const int r = lane & 15;
  const int nrb = (N + 15) >> 4;
  const int rb0 = blockIdx.x * rbn;
  const int nrb_wg = min(rbn, nrb - rb0);
  const uint32_t row_bytes = (uint32_t)(K >> 1);
  const uint32_t groups_per_row = (uint32_t)(K >> 7);
  // which slice of K a wave owns turns with the workgroup (x, x + 8, ... share an XCD), so that the CUs do not all ask
  // for the same stretch of the activations and of their weight rows at the same time; sums stay in slice order
  const int kw = (wave + (int)(blockIdx.x >> 3)) & (WAVES - 1);
  const int chunk0 = kw * NC;

  const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)B, 0, (uint32_t)N * row_bytes, kBufferFlags);
  const __amdgpu_buffer_rsrc_t s_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)S, 0, HAS_SCALE ? (uint32_t)N * groups_per_row * 2u : 0u, kBufferFlags);
  const __amdgpu_buffer_rsrc_t z_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)Z, 0, HAS_ZEROS ? (uint32_t)N * groups_per_row * 2u : 0u, kBufferFlags);

  uint4_t bq[DEPTH][NC];
  // Scales and zeros: asked for per lane (8 bytes of row r's line by every lane group of every wave) they cost
  // the L2 half as many requests again as the weights themselves, for 3 % of the bytes each.  So the workgroup
  // fetches a row block's 16 lines once, thread t the t-th dword of the block's contiguous 16 K / 128 values (one
  // block ahead, into a register), parks them in LDS in front of the block's barrier, and every lane reads its
  // row's NC values from there.
  uint32_t s_stage = 0, z_stage = 0;
  Halves<NC> sc, zp;
  // per-lane byte offsets inside a row block (N is a multiple of 16 here); the block's own offset is uniform
  constexpr uint32_t kChunkStep = FRAG ? 1024u : 64u;  // bytes from one 128-k chunk of a block to the next
  const uint32_t w_voff = TR ? (uint32_t)(lane / LPR) * row_bytes + (uint32_t)chunk0 * 64u + (uint32_t)(lane % LPR) * 16u
                             : (FRAG ? (uint32_t)chunk0 * 1024u + (uint32_t)lane * 16u
                                     : (uint32_t)r * row_bytes + (uint32_t)chunk0 * 64u + (uint32_t)g * 16u);
  const uint32_t sz_dwords = 8u * groups_per_row;  // dwords of scales of one row block
  const uint32_t s_voff = (uint32_t)tid < sz_dwords ? (uint32_t)tid * 4u : kOutOfRange;
  const int sz_shift = 31 - __builtin_clz(groups_per_row >> 1);  // log2(dwords of scales per row); K / 256 is a power of two here
  const uint32_t sz_read = (uint32_t)r * kSzRow + (uint32_t)chunk0 * 2u;
  auto w_soff = [&](int rb) { return rb < nrb_wg ? (uint32_t)(rb0 + rb) * 16u * row_bytes : kOutOfRange; };
  auto s_soff = [&](int rb) { return rb < nrb_wg ? (uint32_t)(rb0 + rb) * 32u * groups_per_row : 0u; };
  auto load_chunk = [&](int d, int c, int rb) {
    if constexpr (TR) {  // load instruction c of the block: rows c RPI .. c RPI + RPI - 1
      const uint32_t so = rb < nrb_wg ? (uint32_t)((rb0 + rb) * 16 + c * RPI) * row_bytes : kOutOfRange;
      bq[d][c] = __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, w_voff, so, 2 /* nt */);
    } else {
      bq[d][c] = __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, w_voff + (uint32_t)c * kChunkStep, w_soff(rb), 2 /* nt */);
    }
  };
  // TR: where load instruction i's 16 bytes go, and where chunk c's operand words of lane (g, r) are
  auto stage_widx = [&](int i) {
    const int row = i * RPI + lane / LPR, piece = lane % LPR;
    return row * LPR + (piece ^ (row & (LPR - 1)));
  };
  auto stage_ridx = [&](int c) { return r * LPR + ((c * 4 + g) ^ (r & (LPR - 1))); };
  auto load_scales = [&](int rb) {  // into the staging registers (zeros past the buffer or past the block's values)
    if constexpr (HAS_SCALE) s_stage = __builtin_amdgcn_raw_buffer_load_b32(s_rsrc, s_voff, s_soff(rb), 0);
    if constexpr (HAS_ZEROS) z_stage = __builtin_amdgcn_raw_buffer_load_b32(z_rsrc, s_voff, s_soff(rb), 0);
  };
  auto park_scales = [&](int rb) {  // staging registers -> LDS slot of block rb
    // recomputed from the thread index each time: a few instructions instead of a register held across the loop;
    // threads without a dword write to a spare word behind the rows (no branch: see the note on loads above)
    uint32_t sz_store = ((uint32_t)tid >> sz_shift) * kSzRow + ((uint32_t)tid & ((1u << sz_shift) - 1u)) * 4u;
    sz_store = (uint32_t)tid < sz_dwords ? sz_store : 16u * kSzRow;
    if constexpr (HAS_SCALE) *reinterpret_cast<uint32_t*>(&sz_lds[rb & 1][0][sz_store]) = s_stage;
    if constexpr (HAS_ZEROS) *reinterpret_cast<uint32_t*>(&sz_lds[rb & 1][1][sz_store]) = z_stage;
  };
  auto read_scales = [&](int rb) {
    if constexpr (HAS_SCALE) __builtin_memcpy(&sc, &sz_lds[rb & 1][0][sz_read], sizeof(sc));
    if constexpr (HAS_ZEROS) __builtin_memcpy(&zp, &sz_lds[rb & 1][1][sz_read], sizeof(zp));
  };
  // the first DEPTH blocks of weights go out before the activations are fetched
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) {
#pragma unroll
    for (int c = 0; c < NC; ++c) load_chunk(d, c, d);
  }
  load_scales(0);

  uint4_t y[NR > 0 ? NR : 1][4];
  {
    // rows beyond M: an offset beyond the buffer, i.e. a zero operand and nothing fetched
    const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)A, 0, (uint32_t)M * (uint32_t)K * 2u, kBufferFlags);
    const uint32_t a_voff = r < M ? ((uint32_t)r * (uint32_t)K + (uint32_t)chunk0 * 128u + (uint32_t)g * 32u) * 2u : kOutOfRange;
    const half_t one = (half_t)1.f;
    const half8_t ones = {one, one, one, one, one, one, one, one};
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      float4_t sum = {0.f, 0.f, 0.f, 0.f};
      uint4_t dd[4];
      if constexpr (TR || FRAG) {
        // the chunk's 16 rows x 256 bytes are fetched row-contiguously too (an instruction reads 4 rows x 256 bytes
        // instead of 16-byte pieces of 32 cache lines) and transposed through the wave's LDS area
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int row = i * 4 + (lane >> 4);
          const uint32_t vo = row < M ? ((uint32_t)row * (uint32_t)K + (uint32_t)chunk0 * 128u) * 2u + (uint32_t)(lane & 15) * 16u : kOutOfRange;
          dd[i] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, vo + (uint32_t)(c * 256), 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int row = i * 4 + (lane >> 4);
          wstage[wave][row * 16 + ((lane & 15) ^ row)] = dd[i];
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) dd[j] = wstage[wave][r * 16 + ((g * 4 + j) ^ r)];
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) dd[j] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, a_voff + (uint32_t)(c * 256 + j * 16), 0, 0);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        uint4_t d = dd[j];
        if constexpr (APERM) d = permute_k8_16bit(d);
        if (c < NR) y[c < NR ? c : 0][j] = d;
        else ypark[wave][c - NR][j][lane] = d;
        sum = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, d), ones, sum, 0, 0, 0);
      }
      // all 16 output columns of the ones-product are equal: lane (g, 0) stores the four sums of its rows
      if (r == 0) asum_lds[wave][c][g] = sum;
    }
  }
  park_scales(0);
  __syncthreads();  // also orders each wave's own asum / parked activations


  auto process = [&](auto d_tag, int rb) {
    constexpr int d = decltype(d_tag)::value;
    float4_t total = {0.f, 0.f, 0.f, 0.f};
    // The group epilogue of chunk c - 1 sits behind the matrix instructions of chunk c (their result is not
    // waited for), and scheduling barriers keep that order: two group accumulators are live, not NC.
    float4_t acc_prev = {0.f, 0.f, 0.f, 0.f};
    auto finish_group = [&](int c, const float4_t& acc) {
      const float s = HAS_SCALE ? half_at<NC>(sc, c) : 1.f;
      const float nz = -(64.f + (HAS_ZEROS ? half_at<NC>(zp, c) : zconst));
      const float4_t asum = asum_lds[wave][c][g];
#pragma unroll
      for (int i = 0; i < 4; ++i) total[i] = __builtin_fmaf(s, __builtin_fmaf(nz, asum[i], acc[i]), total[i]);
    };
    read_scales(rb);
    if constexpr (TR) {
      // the block as loaded goes to the wave's LDS area, and its registers take the next block at once
#pragma unroll
      for (int i = 0; i < NC; ++i) wstage[wave][stage_widx(i)] = bq[0][i];
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < NC; ++i) {
        load_chunk(0, i, rb + 1);
        if (i == 0) load_scales(rb + 1);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      float4_t acc = {0.f, 0.f, 0.f, 0.f};
      uint4_t wq;
      if constexpr (TR) wq = wstage[wave][stage_ridx(c)];
      else wq = bq[d][c];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint4_t a = c < NR ? y[c < NR ? c : 0][j] : ypark[wave][c < NR ? 0 : c - NR][j][lane];
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), decode_w4_bias64<FLIP>(wq[j]), acc, 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      if (c > 0) finish_group(c - 1, acc_prev);
      if constexpr (!TR) {
        // this chunk's registers are free: the same chunk, DEPTH blocks on (zeros from beyond the buffer after the
        // workgroup's last block); the next block's scales and zeros travel behind the first chunk
        load_chunk(d, c, rb + DEPTH);
        if (c == 0) load_scales(rb + 1);
      }
      __builtin_amdgcn_sched_barrier(0);
      acc_prev = acc;
    }
    finish_group(NC - 1, acc_prev);
    park_scales(rb + 1);
    // total[i] = partial C[m = 4 g + i][(rb0 + rb) * 16 + r] over this wave's K slice
    float* buf = &red[rb & 1][0][0];
    *reinterpret_cast<float4_t*>(buf + kw * 256 + lane * 4) = total;
    __syncthreads();  // the other buffer is rewritten only after the next barrier
    if (tid < 256 && rb < nrb_wg) {
      float v = buf[tid];
#pragma unroll
      for (int w = 1; w < WAVES; ++w) v += buf[w * 256 + tid];
      // tid = 4 * source lane + i: output row m = 4 (source lane / 16) + i, column 16 (rb0 + rb) + source lane % 16;
      // M * N fits 32 bits (M <= 16)
      const int out_m = ((tid >> 6) & 3) * 4 + (tid & 3);
      const uint32_t out_idx = (uint32_t)out_m * (uint32_t)N + (uint32_t)(rb0 + rb) * 16u + (uint32_t)((tid >> 2) & 15);
      if (out_m < M) C[out_idx] = (half_t)v;
    }
  };
  // blocks go DEPTH at a time without a branch between them; a block past the last one multiplies zeros and stores
  // nothing
  for (int rb = 0; rb < nrb_wg; rb += DEPTH) {
    process(std::integral_constant<int, 0>{}, rb);
    if constexpr (DEPTH == 2) process(std::integral_constant<int, 1>{}, rb + 1);
  }
}

template <int WAVES, int NC, int DEPTH, int PARK, bool TR, bool FRAG = false>
int launch_regres_fast(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int mode,
                       int layout, hipStream_t stream) {
  const int nrb = (N + 15) / 16;
  const int rbn = (nrb + 255) / 256;
  const dim3 grid((nrb + rbn - 1) / rbn), block(64 * WAVES);
  const bool plain = layout == LAYOUT_PLAIN;
#define DQ_FAST2(HS, HZ, FL, AP, ZC)                                                                                        \
  hipLaunchKernelGGL((w4a16_regres_fast_kernel<WAVES, NC, DEPTH, PARK, TR, FRAG, HS, HZ, FL, AP>), grid, block, 0, stream, (const half_t*)A, \
                     (const uint8_t*)B, (const half_t*)S, (const half_t*)Z, (half_t*)C, M, N, K, rbn, ZC)
#define DQ_FAST(HS, HZ, FL, ZC)                  \
  do {                                           \
    if (plain) DQ_FAST2(HS, HZ, FL, true, ZC);   \
    else DQ_FAST2(HS, HZ, FL, false, ZC);        \
  } while (0)
  switch (mode) {
    case W4_UNSIGNED: DQ_FAST(false, false, false, 0.f); break;
    case W4_SIGNED: DQ_FAST(false, false, true, 8.f); break;  // sext4(q) = (q ^ 8) - 8
    case W4_OFFSET8: DQ_FAST(false, false, false, 8.f); break;
    case W4_SCALE: DQ_FAST(true, false, false, 8.f); break;
    case W4_USCALE: DQ_FAST(true, false, false, 0.f); break;
    case W4_ZEROS_ORIGINAL: DQ_FAST(true, true, false, 0.f); break;
    default: return 1;  // "rescale" rounds at the magnitude of z: the exact kernels
  }
#undef DQ_FAST
#undef DQ_FAST2
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

template <int NC>
int launch_regres(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int mode,
                  int layout, hipStream_t stream) {
  const int nrb = (N + 15) / 16;
  const int rbn = (nrb + 255) / 256;  // one workgroup per CU, all resident at once
  const dim3 grid((nrb + rbn - 1) / rbn), block(1024);
#define DQ_LAUNCH2(MODE_, APERM_)                                                                                    \
  hipLaunchKernelGGL((w4a16_regres_kernel<NC, MODE_, APERM_>), grid, block, 0, stream, (const half_t*)A,             \
                     (const uint8_t*)B, (const half_t*)S, (const half_t*)Z, (half_t*)C, M, N, K, rbn)
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

// Returns 1 when the shape is not covered: needs M <= 16, N a multiple of 16, K = 2048, 4096 or 8192 (whole
// 128-k chunks per wave, activations within the register budget) and group 128 when the mode reads scales
// (one scale per chunk).
// `fast`: the variant that applies scale and zero point per group in fp32 (not for "rescale"); 4: the same for weights
// in fragment order (no other kernel reads that order).
int w4a16_regres(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int group,
                 int mode, int layout, int fast, hipStream_t stream) {
  if (M < 1 || M > 16 || N < 16 || N % 16 != 0) return 1;
  if (mode >= W4_SCALE && group != 128) return 1;
  if ((size_t)N * K / 2 >= (1ull << 32) - 8192) return 1;  // 32-bit offsets, and room for the out-of-range marker
  if (fast == 4 && mode == W4_ZEROS_RESCALE) return 1;  // the exact kernels read the row-major order only
  if (fast && mode != W4_ZEROS_RESCALE) {
    // fast = 1 (default): sixteen waves, row-contiguous loads transposed through LDS (at K = 2048 a wave's slice of a
    // row is 64 bytes and the matrix instruction's own layout is already row-contiguous); 3: sixteen waves, loads in
    // the matrix instruction's layout; 2: eight waves of 256 registers with two row blocks in flight, same layout
    if (fast == 4) {  // fragment-ordered weights
      if (K == 8192) return launch_regres_fast<16, 4, 1, 0, false, true>(A, B, S, Z, C, M, N, K, mode, layout, stream);
      if (K == 4096) return launch_regres_fast<16, 2, 1, 0, false, true>(A, B, S, Z, C, M, N, K, mode, layout, stream);
      if (K == 2048) return launch_regres_fast<16, 1, 1, 0, false, true>(A, B, S, Z, C, M, N, K, mode, layout, stream);
      return 1;
    }
    if (fast == 1) {
      if (K == 8192) return launch_regres_fast<16, 4, 1, 0, true>(A, B, S, Z, C, M, N, K, mode, layout, stream);
      if (K == 4096) return launch_regres_fast<16, 2, 1, 0, true>(A, B, S, Z, C, M, N, K, mode, layout, stream);
    }
    if (fast != 2) {
      if (K == 8192) return launch_regres_fast<16, 4, 1, 1, false>(A, B, S, Z, C, M, N, K, mode, layout, stream);
      if (K == 4096) return launch_regres_fast<16, 2, 1, 0, false>(A, B, S, Z, C, M, N, K, mode, layout, stream);
      if (K == 2048) return launch_regres_fast<16, 1, 1, 0, false>(A, B, S, Z, C, M, N, K, mode, layout, stream);
      return 1;
    }
    if (K == 8192) return launch_regres_fast<8, 8, 2, 3, false>(A, B, S, Z, C, M, N, K, mode, layout, stream);
    if (K == 4096) return launch_regres_fast<8, 4, 2, 0, false>(A, B, S, Z, C, M, N, K, mode, layout, stream);
    if (K == 2048) return launch_regres_fast<8, 2, 2, 0, false>(A, B, S, Z, C, M, N, K, mode, layout, stream);
    return 1;
  }
  if (K == 8192) return launch_regres<4>(A, B, S, Z, C, M, N, K, mode, layout, stream);
  if (K == 4096) return launch_regres<2>(A, B, S, Z, C, M, N, K, mode, layout, stream);
  if (K == 2048) return launch_regres<1>(A, B, S, Z, C, M, N, K, mode, layout, stream);
  return 1;
}

}  // namespace dq
