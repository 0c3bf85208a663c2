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

// Sum over each 32-lane half of the wave; lane 31 and lane 63 receive the two totals.
__device__ __forceinline__ float wave_half_reduce(float v) {
  // quad_perm(1,0,3,2), quad_perm(2,3,0,1), row_half_mirror, row_mirror: all 16 lanes of a
  // DPP row then hold the row total
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));
  // row_bcast:15 into rows 1 and 3: lanes 16..31 += lane 15, lanes 48..63 += lane 47
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x142, 0xA, 0xF, false));
  return v;
}

constexpr int kMaxRowsPerWg = 128;

// R rows (per row slot) are in flight per thread; a workgroup walks NB batches of R rows and
// re-issues the load of a row's successor as soon as that row's registers are consumed, so
// the same R * NP loads stay in flight from the first instruction to the last batch.
template <int MROWS, int NP, int R, bool HAS_SCALE, bool HAS_ZEROS, bool G128>
__global__ __launch_bounds__(256) void w4a16_gemv_kernel(const half_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                          const half_t* __restrict__ S, const half_t* __restrict__ Z,
                                                          half_t* __restrict__ C, int M, int N, int K, int group,
                                                          int tpr_shift, int nb, uint32_t flip_mask, float zsub_const,
                                                          int interleaved) {
  __shared__ float red[kMaxRowsPerWg * 4 * MROWS];  // [row in workgroup][wave of the row][m]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int tpr = 1 << tpr_shift;            // threads per row: 32, 64, 128 or 256
  const int rpp = 256 >> tpr_shift;          // rows per pass
  const int slot = tid >> tpr_shift;         // which row of the pass
  const int ct = tid & (tpr - 1);            // chunk within the pass
  const int wave_in_row = ct >> 6;
  const int c16 = K >> 5;                    // 16-byte chunks per row
  const int rows_per_batch = R * rpp;
  const int rows_per_wg = nb * rows_per_batch;
  const int row0 = blockIdx.x * rows_per_wg;
  const size_t row_bytes = (size_t)(K >> 1);
  const int groups_per_row = K / group;
  const int gshift = (group == K) ? 31 : (31 - __builtin_clz(group));

  // per-pass byte offsets inside a row (chunk clamped: its activations are zeroed below)
  int boff[NP], goff[NP];
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int chunk = min(p * tpr + ct, c16 - 1);
    boff[p] = chunk * 16;
    goff[p] = G128 ? (chunk >> 2) : ((chunk << 5) >> gshift);
  }

  uint4_t bq[R][NP];
  half_t sc[R][NP], zp[R][NP];
  auto issue_row = [&](int u, int b) {
    // rows past N are clamped to a valid row and masked at the store
    const int row = min(row0 + b * rows_per_batch + u * rpp + slot, N - 1);
    const uint8_t* bp = B + (size_t)row * row_bytes;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      bq[u][p] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(bp + boff[p]));
      if constexpr (HAS_SCALE) sc[u][p] = S[(size_t)row * groups_per_row + goff[p]];
      if constexpr (HAS_ZEROS) zp[u][p] = Z[(size_t)row * groups_per_row + goff[p]];
    }
  };

  // ---- first batch of weight / scale / zero loads goes out before anything else ----------
#pragma unroll
  for (int u = 0; u < R; ++u) issue_row(u, 0);

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
      abias[p][m] = 1024.f * s_even + 64.f * s_odd;
      asum[p][m] = s_even + s_odd;
    }
  }

  // ---- stream the batches ----------------------------------------------------------------
  auto process_batch = [&](int b, auto refill_tag) {
    constexpr bool kRefill = decltype(refill_tag)::value;
    float acc[R][MROWS];
#pragma unroll
    for (int u = 0; u < R; ++u) {
#pragma unroll
      for (int m = 0; m < MROWS; ++m) acc[u][m] = 0.f;
#pragma unroll
      for (int p = 0; p < NP; ++p) {
        float dot[MROWS];
#pragma unroll
        for (int m = 0; m < MROWS; ++m) dot[m] = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          uint32_t t[4];
          u4x8_to_biased_half(bq[u][p][j] ^ flip_mask, t);
#pragma unroll
          for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int m = 0; m < MROWS; ++m)
              dot[m] = __builtin_amdgcn_fdot2(as_half2(t[i]), as_half2(a[p][m][j * 4 + i]), dot[m], false);
        }
        const float s = HAS_SCALE ? (float)sc[u][p] : 1.f;
        const float zsub = HAS_ZEROS ? (float)zp[u][p] : zsub_const;
#pragma unroll
        for (int m = 0; m < MROWS; ++m) acc[u][m] += s * (dot[m] - abias[p][m] - zsub * asum[p][m]);
      }
      // this row's registers are free again: refill them with the same row of the next batch.
      // The scheduling barriers keep the refill behind this row's arithmetic (no second register
      // set) and ahead of the next row's.
      if constexpr (kRefill) {
        __builtin_amdgcn_sched_barrier(0);
        issue_row(u, b + 1);
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    // reduce over the threads of each row; the chains of the R rows are independent
#pragma unroll
    for (int u = 0; u < R; ++u) {
      const int rl = b * rows_per_batch + u * rpp + slot;
#pragma unroll
      for (int m = 0; m < MROWS; ++m) {
        float v = wave_half_reduce(acc[u][m]);
        if (tpr >= 64) {
          // lane 63 += lane 31 (row_bcast:31 into rows 2 and 3)
          v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x143, 0xC, 0xF, false));
          if (lane == 63) red[(rl * 4 + wave_in_row) * MROWS + m] = v;
        } else {
          // two rows per wave: lane 31 carries the even slot, lane 63 the odd one
          if ((lane & 31) == 31) red[(rl * 4 + 0) * MROWS + m] = v;
        }
      }
    }
  };
  for (int b = 0; b + 1 < nb; ++b) process_batch(b, std::true_type{});
  process_batch(nb - 1, std::false_type{});
  __syncthreads();
  const int waves_per_row = tpr >= 64 ? (tpr >> 6) : 1;
  for (int o = tid; o < rows_per_wg * MROWS; o += 256) {
    const int rl = o / MROWS, m = o - rl * MROWS;
    float v = red[(rl * 4 + 0) * MROWS + m];
    for (int w = 1; w < waves_per_row; ++w) v += red[(rl * 4 + w) * MROWS + m];
    const int row = row0 + rl;
    if (row < N && m < M) C[(size_t)m * N + row] = (half_t)v;
  }
}

template <int MROWS, int NP, int R>
int launch_gemv(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int group,
                int mode, int layout, int tpr_shift, int nb, hipStream_t stream) {
  const int rows_per_wg = nb * R * (256 >> tpr_shift);
  if (rows_per_wg > kMaxRowsPerWg) DQ_FAIL("w4a16 gemv: %d rows per workgroup exceed %d", rows_per_wg, kMaxRowsPerWg);
  const dim3 grid((N + rows_per_wg - 1) / rows_per_wg), block(256);
  uint32_t flip = 0;
  float zsub = 0.f;
  bool has_scale = false, has_zeros = false;
  switch (mode) {
    case W4_UNSIGNED: break;
    case W4_SIGNED: flip = 0x88888888u; zsub = 8.f; break;
    case W4_OFFSET8: zsub = 8.f; break;
    case W4_SCALE: zsub = 8.f; has_scale = true; break;
    case W4_USCALE: has_scale = true; break;
    case W4_ZEROS_ORIGINAL: has_scale = has_zeros = true; break;
    default: DQ_FAIL("w4a16 gemv: unknown mode %d", mode);
  }
  const int il = layout == LAYOUT_INTERLEAVED;
#define DQ_GEMV(HS, HZ, G)                                                                                       \
  hipLaunchKernelGGL((w4a16_gemv_kernel<MROWS, NP, R, HS, HZ, G>), grid, block, 0, stream, (const half_t*)A,      \
                     (const uint8_t*)B, (const half_t*)S, (const half_t*)Z, (half_t*)C, M, N, K, group, tpr_shift, \
                     nb, flip, zsub, il)
  const bool g128 = group == 128;
  if (!has_scale) DQ_GEMV(false, false, false);
  else if (!has_zeros) { if (g128) DQ_GEMV(true, false, true); else DQ_GEMV(true, false, false); }
  else { if (g128) DQ_GEMV(true, true, true); else DQ_GEMV(true, true, false); }
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
  // rows_hint = r + 16 * nb (0 = choose here).  r rows in flight per thread (4 by default,
  // fewer when the grid would be small); nb batches per workgroup so that the whole grid is
  // resident at once (7 workgroups per CU) when the matrix is large enough.
  const int rpp = 256 >> tpr_shift;
  int r = rows_hint & 15, nb = rows_hint >> 4;
  if (r == 0) r = (((long)N / (4 * rpp)) >= 1024 ? 4 : 2);
  if (np * r > 8) r = 8 / np;  // keep registers bounded
  if (r != 2 && r != 4 && r != 8) r = 2;
  if (nb == 0) {
    const long wgs1 = ((long)N + r * rpp - 1) / (r * rpp);
    nb = (int)((wgs1 + 1791) / 1792);
  }
  while (nb > 1 && nb * r * rpp > 128) --nb;
  if (nb < 1) nb = 1;
#define DQ_R(MR, NP_)                                                                                            \
  do {                                                                                                           \
    if (r == 8) return launch_gemv<MR, NP_, 8>(A, B, S, Z, C, M, N, K, group, mode, layout, tpr_shift, nb, stream); \
    if (r == 4) return launch_gemv<MR, NP_, 4>(A, B, S, Z, C, M, N, K, group, mode, layout, tpr_shift, nb, stream); \
    return launch_gemv<MR, NP_, 2>(A, B, S, Z, C, M, N, K, group, mode, layout, tpr_shift, nb, stream);          \
  } while (0)
  if (mrows == 1 && np == 1) DQ_R(1, 1);
  if (mrows == 1 && np == 2) DQ_R(1, 2);
  if (mrows == 1 && np == 4) DQ_R(1, 4);
  if (mrows == 2 && np == 1) DQ_R(2, 1);
  if (mrows == 2 && np == 2) DQ_R(2, 2);
  if (mrows == 4 && np == 1) DQ_R(4, 1);
#undef DQ_R
  return 1;
}

}  // namespace dq
