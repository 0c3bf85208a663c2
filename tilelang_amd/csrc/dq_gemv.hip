// W4A16 decode GEMV for M <= 4 on gfx950: the memory-bound M=1 path.
//
// Replaces the kernel generated from
// examples/dequantize_gemm/example_dequant_gemv_fp16xint4.py:83-153 (4 outputs per 128-thread
// block, 32-bit weight loads, 32-lane all-reduce).  Mapping chosen from measured HBM behaviour
// of the chip: a wave instruction reads 1 KiB of ONE weight row (64 lanes x 16 B, non-temporal),
// the 4 waves of a workgroup read 4 consecutive KiB of that row, and a workgroup issues the
// loads of all its R rows before it touches the data.
//
//   * thread t owns the 32 k-values of 16-byte chunk (pass * TPR + t % TPR) of every row; its
//     slice of the activations stays in registers for the whole kernel, pre-paired to the
//     order the nibble decoder produces ((k, k+4) pairs for the plain layout);
//   * nibbles are turned into fp16 by OR-ing them into the mantissa of 1024.0 / 64.0
//     (bias + q, exact) and fed to v_dot2_f32_f16; the bias, the zero point and the group
//     scale are applied once per 32 weights in fp32:
//         sum_k a_k (q_k - z) s  =  s * (dot - sum_k a_k bias_k - z * sum_k a_k)
//     so the result is the fp32 dot product of A with the exact (q - z) * s values (the fp16
//     rounding of each weight, relative 2^-11, is not reproduced; the MFMA kernel does);
//   * K is reduced over the lanes with DPP row operations and over the waves of a row through
//     LDS in a fixed order: no atomics, bit-identical from run to run.
#include "dq_common.h"

#include <type_traits>

namespace dq {

namespace {

constexpr int kMaxRowsPerWg = 128;  // also bounds nb * R (partial sums kept in LDS)

// 256 threads.  A weight row is spread over tpr = 32..256 threads (16 bytes each per pass), so
// a pass of the workgroup covers rpp = 256 / tpr rows; R row groups are in flight per thread
// and a workgroup walks nb batches of R groups, re-issuing a group's loads for the next batch
// as soon as its registers are consumed.  WIDE: tpr = 256 (one row per pass), which makes every
// row address uniform (scalar base + per-thread offset).
template <int MROWS, int NP, int R, bool HAS_SCALE, bool HAS_ZEROS, bool G128, bool FLIP, bool WIDE>
__global__ __launch_bounds__(256) void w4a16_gemv_kernel(const half_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                          const half_t* __restrict__ S, const half_t* __restrict__ Z,
                                                          half_t* __restrict__ C, int M, int N, int K, int group,
                                                          int tpr_shift_arg, int nb, float zsub_const, int interleaved) {
  constexpr int NV = R * MROWS;  // values reduced together per batch
  static_assert(NV <= 16, "at most 16 values per lane row");
  // partial sums: [batch][16-lane row of the workgroup (16)][value]
  __shared__ float red[kMaxRowsPerWg * 16 * MROWS];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int tpr_shift = WIDE ? 8 : tpr_shift_arg;
  const int tpr = 1 << tpr_shift;            // threads per row
  const int rpp = 256 >> tpr_shift;          // rows per pass
  const int slot = WIDE ? 0 : (tid >> tpr_shift);
  const int ct = tid & (tpr - 1);            // chunk within the pass
  const int c16 = K >> 5;                    // 16-byte chunks per row
  const int rows_per_batch = R * rpp;
  const int rows_per_wg = nb * rows_per_batch;
  const int row0 = blockIdx.x * rows_per_wg;
  const uint32_t row_bytes = (uint32_t)(K >> 1);
  const int groups_per_row = K / group;
  const int gshift = (group == K) ? 31 : (31 - __builtin_clz(group));

  // per-thread offsets from the (uniform) first row of a row group
  uint32_t boff[NP], goff[NP];
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int chunk = min(p * tpr + ct, c16 - 1);  // clamped: its activations are zeroed below
    boff[p] = (uint32_t)slot * row_bytes + (uint32_t)chunk * 16u;
    goff[p] = (uint32_t)(slot * groups_per_row + (G128 ? (chunk >> 2) : ((chunk << 5) >> gshift))) * 2u;
  }

  // One row per pass, four row groups, group size 128: the four lanes of a quad share their scale
  // group, so lane l fetches the scale (zero) of row (l & 3) of the batch for all four of them and
  // the batch needs one scale load per lane instead of four.
  constexpr bool kPack = WIDE && R == 4 && G128 && HAS_SCALE;
  uint32_t pack_off[NP];
#pragma unroll
  for (int p = 0; p < NP; ++p) pack_off[p] = (uint32_t)(min(p * tpr + ct, c16 - 1) >> 2) * 2u;
  unsigned short sc_pack[NP], zp_pack[NP];

  uint4_t bq[R][NP];
  half_t sc[R][NP], zp[R][NP];
  auto issue_pack = [&](int b) {
    const int row = min(row0 + b * R + (lane & 3), N - 1);
    const uint8_t* sp = reinterpret_cast<const uint8_t*>(S) + (size_t)row * groups_per_row * 2;
    const uint8_t* zq = reinterpret_cast<const uint8_t*>(Z) + (size_t)row * groups_per_row * 2;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      sc_pack[p] = *reinterpret_cast<const unsigned short*>(sp + pack_off[p]);
      if constexpr (HAS_ZEROS) zp_pack[p] = *reinterpret_cast<const unsigned short*>(zq + pack_off[p]);
    }
  };
  auto issue_group = [&](int u, int b) {
    // groups past N (N is a multiple of rpp) are clamped to the last one and dropped at the store
    const int rb = min(row0 + (b * R + u) * rpp, N - rpp);
    const uint8_t* bp = B + (size_t)rb * row_bytes;
    const uint8_t* sp = reinterpret_cast<const uint8_t*>(S) + (size_t)rb * groups_per_row * 2;
    const uint8_t* zq = reinterpret_cast<const uint8_t*>(Z) + (size_t)rb * groups_per_row * 2;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      bq[u][p] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(bp + boff[p]));
      if constexpr (HAS_SCALE && !kPack) sc[u][p] = *reinterpret_cast<const half_t*>(sp + goff[p]);
      if constexpr (HAS_ZEROS && !kPack) zp[u][p] = *reinterpret_cast<const half_t*>(zq + goff[p]);
    }
    if constexpr (kPack) {
      if (u == 0) issue_pack(b);
    }
  };

  // ---- first batch of weight / scale / zero loads goes out before anything else ----------
#pragma unroll
  for (int u = 0; u < R; ++u) issue_group(u, 0);

  // ---- this thread's activations, paired in decoder order ------------------------------
  uint32_t a[NP][MROWS][16];
  float abias[NP][MROWS], asum[NP][MROWS];
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int chunk = p * tpr + ct;
    const bool valid = chunk < c16;
#pragma unroll
    for (int m = 0; m < MROWS; ++m) {
      const half_t* ap = A + (size_t)min(m, M - 1) * K + (size_t)min(chunk, c16 - 1) * 32;
      float s_even = 0.f, s_odd = 0.f;  // sums over the pairs decoded with bias 1024 / bias 64
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        uint4_t d = *reinterpret_cast<const uint4_t*>(ap + j * 8);
        if (!valid) d = uint4_t{0u, 0u, 0u, 0u};
        if (!interleaved) d = permute_k8_16bit(d);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          a[p][m][j * 4 + i] = d[i];
          const half2_t one2 = {(half_t)1.f, (half_t)1.f};
          if (i & 1) s_odd = __builtin_amdgcn_fdot2(as_half2(d[i]), one2, s_odd, false);
          else s_even = __builtin_amdgcn_fdot2(as_half2(d[i]), one2, s_even, false);
        }
      }
      asum[p][m] = s_even + s_odd;
      // without per-group zeros the whole correction is one constant per thread
      abias[p][m] = 1024.f * s_even + 64.f * s_odd + (HAS_ZEROS ? 0.f : zsub_const * asum[p][m]);
    }
  }

  const bool writer = (lane & 15) < NV;
  float* red_w = red + (tid >> 4) * NV + (lane & (NV - 1));

  // ---- stream the batches ----------------------------------------------------------------
  auto process_batch = [&](int b, auto refill_tag) {
    constexpr bool kRefill = decltype(refill_tag)::value;
    float acc[NV];
    if constexpr (kPack) {
      // hand every lane of a quad the scale of each of the four rows (quad_perm broadcast of lane u)
#pragma unroll
      for (int p = 0; p < NP; ++p) {
        const int s32 = sc_pack[p], z32 = HAS_ZEROS ? zp_pack[p] : 0;
        const int sb[4] = {__builtin_amdgcn_update_dpp(0, s32, 0x00, 0xF, 0xF, true), __builtin_amdgcn_update_dpp(0, s32, 0x55, 0xF, 0xF, true),
                           __builtin_amdgcn_update_dpp(0, s32, 0xAA, 0xF, 0xF, true), __builtin_amdgcn_update_dpp(0, s32, 0xFF, 0xF, 0xF, true)};
#pragma unroll
        for (int u = 0; u < R; ++u) sc[u][p] = __builtin_bit_cast(half_t, (unsigned short)sb[u & 3]);
        if constexpr (HAS_ZEROS) {
          const int zb[4] = {__builtin_amdgcn_update_dpp(0, z32, 0x00, 0xF, 0xF, true), __builtin_amdgcn_update_dpp(0, z32, 0x55, 0xF, 0xF, true),
                             __builtin_amdgcn_update_dpp(0, z32, 0xAA, 0xF, 0xF, true), __builtin_amdgcn_update_dpp(0, z32, 0xFF, 0xF, 0xF, true)};
#pragma unroll
          for (int u = 0; u < R; ++u) zp[u][p] = __builtin_bit_cast(half_t, (unsigned short)zb[u & 3]);
        }
      }
    }
#pragma unroll
    for (int u = 0; u < R; ++u) {
#pragma unroll
      for (int m = 0; m < MROWS; ++m) acc[u * MROWS + m] = 0.f;
#pragma unroll
      for (int p = 0; p < NP; ++p) {
        float dot[MROWS][2];
#pragma unroll
        for (int m = 0; m < MROWS; ++m) dot[m][0] = dot[m][1] = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          uint32_t t[4];
          u4x8_to_biased_half(FLIP ? (bq[u][p][j] ^ 0x88888888u) : bq[u][p][j], t);
#pragma unroll
          for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int m = 0; m < MROWS; ++m)
              dot[m][i & 1] = __builtin_amdgcn_fdot2(as_half2(t[i]), as_half2(a[p][m][j * 4 + i]), dot[m][i & 1], false);
        }
        const float s = HAS_SCALE ? (float)sc[u][p] : 1.f;
#pragma unroll
        for (int m = 0; m < MROWS; ++m) {
          float d = (dot[m][0] + dot[m][1]) - abias[p][m];
          if constexpr (HAS_ZEROS) d -= (float)zp[u][p] * asum[p][m];
          acc[u * MROWS + m] += s * d;
        }
      }
      // this group's registers are free again: refill them with the same group of the next
      // batch.  The scheduling barriers keep the refill behind this group's arithmetic (no
      // second register set) and ahead of the next group's.
      if constexpr (kRefill) {
        __builtin_amdgcn_sched_barrier(0);
        issue_group(u, b + 1);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    const float v = RowReduce<NV, 0>::run(acc, lane);
    if (writer) red_w[b * 16 * NV] = v;
  };
  for (int b = 0; b + 1 < nb; ++b) process_batch(b, std::true_type{});
  process_batch(nb - 1, std::false_type{});
  __syncthreads();

  // ---- fixed-order sum of the 16-lane partials of each output ----------------------------
  const int parts = tpr >> 4;  // 16-lane rows per weight row
  for (int o = tid; o < rows_per_wg * MROWS; o += 256) {
    const int rl = o / MROWS, m = o - rl * MROWS;
    const int b = rl / rows_per_batch, within = rl - b * rows_per_batch;
    const int u = within >> (8 - tpr_shift), sl = within & (rpp - 1);
    const float* src = red + (b * 16 + sl * parts) * NV + u * MROWS + m;
    float v = src[0];
    for (int j = 1; j < parts; ++j) v += src[j * NV];
    const int row = row0 + rl;
    if (row < N && m < M) C[(size_t)m * N + row] = (half_t)v;
  }
}

template <int MROWS, int NP, int R, bool WIDE>
int launch_gemv(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int group,
                int mode, int layout, int tpr_shift, int nb, hipStream_t stream) {
  const int rpp = 256 >> tpr_shift;
  const int rows_per_wg = nb * R * rpp;
  if (rows_per_wg > kMaxRowsPerWg || nb * R > kMaxRowsPerWg)
    DQ_FAIL("w4a16 gemv: %d rows per workgroup exceed %d", rows_per_wg, kMaxRowsPerWg);
  if (N % rpp != 0 || N < rpp) DQ_FAIL("w4a16 gemv: N=%d must be a multiple of %d for K=%d", N, rpp, K);
  if (WIDE != (tpr_shift == 8)) DQ_FAIL("w4a16 gemv: internal dispatch error (tpr_shift %d)", tpr_shift);
  const dim3 grid((N + rows_per_wg - 1) / rows_per_wg), block(256);
  float zsub = 0.f;
  bool has_scale = false, has_zeros = false, flip = false;
  switch (mode) {
    case W4_UNSIGNED: break;
    case W4_SIGNED: flip = true; zsub = 8.f; break;
    case W4_OFFSET8: zsub = 8.f; break;
    case W4_SCALE: zsub = 8.f; has_scale = true; break;
    case W4_USCALE: has_scale = true; break;
    case W4_ZEROS_ORIGINAL: has_scale = has_zeros = true; break;
    default: DQ_FAIL("w4a16 gemv: unknown mode %d", mode);
  }
  const int il = layout == LAYOUT_INTERLEAVED;
#define DQ_GEMV(HS, HZ, G, FL)                                                                                   \
  hipLaunchKernelGGL((w4a16_gemv_kernel<MROWS, NP, R, HS, HZ, G, FL, WIDE>), grid, block, 0, stream,              \
                     (const half_t*)A, (const uint8_t*)B, (const half_t*)S, (const half_t*)Z, (half_t*)C, M, N, K, \
                     group, tpr_shift, nb, zsub, il)
  const bool g128 = group == 128;
  if (!has_scale) { if (flip) DQ_GEMV(false, false, false, true); else DQ_GEMV(false, false, false, false); }
  else if (!has_zeros) { if (g128) DQ_GEMV(true, false, true, false); else DQ_GEMV(true, false, false, false); }
  else { if (g128) DQ_GEMV(true, true, true, false); else DQ_GEMV(true, true, false, false); }
#undef DQ_GEMV
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

}  // namespace

// Returns 1 when this kernel does not cover the shape (caller falls through to the MFMA kernel).
int w4a16_gemv_dot2(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int group,
                    int mode, int layout, int rows_hint, hipStream_t stream) {
  if (M > 4 || K % 32 != 0) return 1;
  // q*s - z rounds to fp16 at the magnitude of z, far coarser than q*s: that tile rounding is
  // part of the result, so this mode goes to the kernel that materialises the fp16 tile.
  if (mode == W4_ZEROS_RESCALE) return 1;
  const int c16 = K / 32;
  int tpr_shift = 5;
  while ((1 << tpr_shift) < c16 && tpr_shift < 8) ++tpr_shift;
  const int np_needed = (c16 + (1 << tpr_shift) - 1) >> tpr_shift;
  const int np = np_needed <= 1 ? 1 : (np_needed <= 2 ? 2 : 4);
  if (np_needed > 4) return 1;
  const int mrows = M == 1 ? 1 : (M == 2 ? 2 : 4);
  if (np * mrows > 4) return 1;
  const int rpp = 256 >> tpr_shift;
  if (N % rpp != 0 || N < rpp) return 1;
  // rows_hint = r + 16 * nb (0 = choose here).  r row groups in flight per thread; nb batches
  // per workgroup so that the grid is about one resident wave of workgroups on a large matrix.
  int r = rows_hint & 15, nb = rows_hint >> 4;
  // a matrix that gives about 512 workgroups of four row groups and two rows per pass (N = K = 4096): one
  // workgroup per CU walking two batches measured 3.9 us against 4.1-4.2 us for the other shapes of the grid
  const long groups4 = (long)N / (4 * rpp);
  if (r == 0 && nb == 0 && np == 1 && mrows == 1 && rpp == 2 && groups4 >= 384 && groups4 <= 640) {
    r = 4;
    nb = 2;
  }
  if (r == 0) r = (groups4 >= 1024 ? 4 : 2);
  if (r != 2 && r != 4) r = 2;
  if (r * np * mrows > 16) r = 2;  // keep registers bounded
  if (r * mrows > 16) return 1;
  if (nb == 0) {
    const long wgs1 = ((long)N + r * rpp - 1) / (r * rpp);
    nb = (int)((wgs1 + 1791) / 1792);
    // long rows on a short matrix (N = 4096, K = 11008: 7.3 us with 1024 workgroups of one batch, 6.7 us with
    // 512 of two): let a workgroup overlap its second batch's loads with the first one's arithmetic
    if (np >= 2 && wgs1 >= 512 && wgs1 <= 1024) nb = 2;
  }
  while (nb > 1 && (nb * r * rpp > kMaxRowsPerWg || nb * r > kMaxRowsPerWg)) --nb;
  if (nb < 1) nb = 1;
#define DQ_R(MR, NP_, W)                                                                                              \
  do {                                                                                                                \
    if (r == 4) return launch_gemv<MR, NP_, 4, W>(A, B, S, Z, C, M, N, K, group, mode, layout, tpr_shift, nb, stream); \
    return launch_gemv<MR, NP_, 2, W>(A, B, S, Z, C, M, N, K, group, mode, layout, tpr_shift, nb, stream);            \
  } while (0)
  if (tpr_shift == 8) {
    if (mrows == 1 && np == 1) DQ_R(1, 1, true);
    if (mrows == 1 && np == 2) DQ_R(1, 2, true);
    if (mrows == 1 && np == 4) { r = 2; DQ_R(1, 4, true); }
    if (mrows == 2 && np == 1) DQ_R(2, 1, true);
    if (mrows == 2 && np == 2) { r = 2; DQ_R(2, 2, true); }
    if (mrows == 4 && np == 1) DQ_R(4, 1, true);
  } else {
    if (mrows == 1) DQ_R(1, 1, false);
    if (mrows == 2) DQ_R(2, 1, false);
    if (mrows == 4) DQ_R(4, 1, false);
  }
#undef DQ_R
  return 1;
}

}  // namespace dq
