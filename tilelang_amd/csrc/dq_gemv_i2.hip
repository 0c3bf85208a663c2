// BitNet W2A8 decode GEMV for M <= 4 on gfx950: C[M,N] = A[M,K] int8 . decode(B[N,K/4])^T, exact int32.
//
// Replaces the kernel generated from examples/bitnet-1.58b/kernel_benchmark/
// tilelang_bitnet_158_int8xint2_decode.py:93-173 (4 outputs per 128-thread block, 32-bit weight
// loads, dp4a, 32-lane all-reduce).  Same streaming shape as the W4A16 GEMV: a thread owns one
// 16-byte chunk (64 codes) of every weight row of its workgroup, the threads of a row read
// consecutive chunks, all loads of a batch are issued before the data is touched.
//
//   * (w >> 2i) & 0x03030303 puts codes 4b+i of packed byte b into byte b of dword i; the
//     thread's activations are held in that same order (a 4x4 byte transpose per 16 values, done
//     once), so each dword goes straight into v_dot4_i32_i8;
//   * the zero point is applied per thread as  sum a (c - 2) = sum a c - 2 sum a  (exact in
//     integers); two's-complement codes are handled as (c ^ 2) - 2;
//   * K is reduced over the lanes with DPP row operations and over the waves of a row through
//     LDS; integer sums, so the result is exact whatever the order.
#include "dq_common.h"

namespace dq {

namespace {

__device__ __forceinline__ int wave_half_reduce_i32(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, true);   // quad_perm(1,0,3,2)
  v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, true);   // quad_perm(2,3,0,1)
  v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, true);  // row_half_mirror
  v += __builtin_amdgcn_update_dpp(0, v, 0x140, 0xF, 0xF, true);  // row_mirror
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xA, 0xF, false); // row_bcast:15 -> lanes 31 / 63 hold 32-lane sums
  return v;
}

constexpr int kMaxRowsPerWg = 128;

template <int MROWS, int NP, int R>
__global__ __launch_bounds__(256) void i2_gemv_kernel(const int8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                       void* __restrict__ C, const float* __restrict__ s_a, float s_w,
                                                       int out_kind, int M, int N, int K, int tpr_shift, int nb,
                                                       uint32_t flip_mask, int zsub, int interleaved) {
  __shared__ int red[kMaxRowsPerWg * 4 * MROWS];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int tpr = 1 << tpr_shift;
  const int rpp = 256 >> tpr_shift;
  const int slot = tid >> tpr_shift;
  const int ct = tid & (tpr - 1);
  const int wave_in_row = ct >> 6;
  const int c16 = K >> 6;  // 16-byte chunks (64 codes) per row
  const int rows_per_batch = R * rpp;
  const int rows_per_wg = nb * rows_per_batch;
  const int row0 = blockIdx.x * rows_per_wg;
  const size_t row_bytes = (size_t)(K >> 2);

  int boff[NP];
#pragma unroll
  for (int p = 0; p < NP; ++p) boff[p] = min(p * tpr + ct, c16 - 1) * 16;

  uint4_t bq[R][NP];
  auto issue_row = [&](int u, int b) {
    const int row = min(row0 + b * rows_per_batch + u * rpp + slot, N - 1);
    const uint8_t* bp = B + (size_t)row * row_bytes;
#pragma unroll
    for (int p = 0; p < NP; ++p)
      bq[u][p] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(bp + boff[p]));
  };
#pragma unroll
  for (int u = 0; u < R; ++u) issue_row(u, 0);

  // activations of this thread's chunk(s), transposed to decoder order; asum for the zero point
  uint32_t a[NP][MROWS][16];
  int asum[NP][MROWS];
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int chunk = p * tpr + ct;
    const bool valid = chunk < c16;
#pragma unroll
    for (int m = 0; m < MROWS; ++m) {
      const int8_t* ap = A + (size_t)min(m, M - 1) * K + (size_t)min(chunk, c16 - 1) * 64;
      int s = 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        uint4_t d = *reinterpret_cast<const uint4_t*>(ap + j * 16);
        if (!valid) d = uint4_t{0u, 0u, 0u, 0u};
        if (!interleaved) d = transpose4x4_bytes(d);  // interleaved words decode to natural order
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          a[p][m][j * 4 + i] = d[i];
          s = __builtin_amdgcn_sdot4((int)d[i], 0x01010101, s, false);
        }
      }
      asum[p][m] = s;
    }
  }

  for (int b = 0; b < nb; ++b) {
    int acc[R][MROWS];
#pragma unroll
    for (int u = 0; u < R; ++u) {
#pragma unroll
      for (int m = 0; m < MROWS; ++m) acc[u][m] = 0;
#pragma unroll
      for (int p = 0; p < NP; ++p) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t w = bq[u][p][j] ^ flip_mask;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int d = (int)((w >> (2 * i)) & 0x03030303u);
#pragma unroll
            for (int m = 0; m < MROWS; ++m) acc[u][m] = __builtin_amdgcn_sdot4((int)a[p][m][j * 4 + i], d, acc[u][m], false);
          }
        }
#pragma unroll
        for (int m = 0; m < MROWS; ++m) acc[u][m] -= zsub * asum[p][m];
      }
    }
    // every row of the batch is consumed: refill all of them (wave-uniform branch)
    if (b + 1 < nb) {
#pragma unroll
      for (int u = 0; u < R; ++u) issue_row(u, b + 1);
    }
#pragma unroll
    for (int u = 0; u < R; ++u) {
      const int rl = b * rows_per_batch + u * rpp + slot;
#pragma unroll
      for (int m = 0; m < MROWS; ++m) {
        int v = wave_half_reduce_i32(acc[u][m]);
        if (tpr >= 64) {
          v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xC, 0xF, false);  // row_bcast:31
          if (lane == 63) red[(rl * 4 + wave_in_row) * MROWS + m] = v;
        } else {
          if ((lane & 31) == 31) red[(rl * 4 + 0) * MROWS + m] = v;
        }
      }
    }
  }
  __syncthreads();
  const int waves_per_row = tpr >= 64 ? (tpr >> 6) : 1;
  for (int o = tid; o < rows_per_wg * MROWS; o += 256) {
    const int rl = o / MROWS, m = o - rl * MROWS;
    int v = red[(rl * 4 + 0) * MROWS + m];
    for (int w = 1; w < waves_per_row; ++w) v += red[(rl * 4 + w) * MROWS + m];
    const int row = row0 + rl;
    if (row < N && m < M) {
      if (out_kind == 0) {
        ((int32_t*)C)[(size_t)m * N + row] = v;
      } else {
        // BitLinear epilogue: (float(acc) / s_a[m]) / s_w -> fp16
        float f = (float)v;
        f = f / s_a[m];
        f = f / s_w;
        ((half_t*)C)[(size_t)m * N + row] = (half_t)f;
      }
    }
  }
}

template <int MROWS, int NP>
int launch_i2_gemv(const void* A, const void* B, void* C, const void* s_a, float s_w, int out_kind, int M, int N, int K,
                   int tpr_shift, uint32_t flip, int zsub, int interleaved, hipStream_t stream) {
  constexpr int R = 4 / NP;
  const int rpp = 256 >> tpr_shift;
  const long wgs1 = ((long)N + R * rpp - 1) / (R * rpp);
  // about two workgroups per CU, each walking several batches: at N = K = 8192 one batch per workgroup (1024
  // workgroups) measured 7.4 us, two 6.3 us, four 6.2 us, eight 8.6 us
  int nb = (int)((wgs1 + 511) / 512);
  while (nb > 1 && nb * R * rpp > kMaxRowsPerWg) --nb;
  if (nb < 1) nb = 1;
  const int rows_per_wg = nb * R * rpp;
  hipLaunchKernelGGL((i2_gemv_kernel<MROWS, NP, R>), dim3((N + rows_per_wg - 1) / rows_per_wg), dim3(256), 0, stream,
                     (const int8_t*)A, (const uint8_t*)B, C, (const float*)s_a, s_w, out_kind, M, N, K, tpr_shift, nb,
                     flip, zsub, interleaved);
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

}  // namespace

// Returns 1 when this kernel does not cover the shape (caller uses the MFMA GEMM).
int i2_gemv(const void* A, const void* B, void* C, int M, int N, int K, int convention, int layout, const void* s_a,
            float s_w, int out_kind, hipStream_t stream) {
  const int interleaved = layout == LAYOUT_INTERLEAVED;
  if (M > 4 || K % 64 != 0) return 1;
  const int c16 = K / 64;
  int tpr_shift = 5;
  while ((1 << tpr_shift) < c16 && tpr_shift < 8) ++tpr_shift;
  const int np_needed = (c16 + (1 << tpr_shift) - 1) >> tpr_shift;
  if (np_needed > 2) return 1;
  const int np = np_needed;
  const int mrows = M == 1 ? 1 : (M == 2 ? 2 : 4);
  if (np * mrows > 4) return 1;
  uint32_t flip = 0;
  int zsub = 0;
  if (convention == I2_OFFSET) zsub = 2;
  else if (convention == I2_TWOS) { flip = 0xAAAAAAAAu; zsub = 2; }
  if (mrows == 1 && np == 1) return launch_i2_gemv<1, 1>(A, B, C, s_a, s_w, out_kind, M, N, K, tpr_shift, flip, zsub, interleaved, stream);
  if (mrows == 1 && np == 2) return launch_i2_gemv<1, 2>(A, B, C, s_a, s_w, out_kind, M, N, K, tpr_shift, flip, zsub, interleaved, stream);
  if (mrows == 2 && np == 1) return launch_i2_gemv<2, 1>(A, B, C, s_a, s_w, out_kind, M, N, K, tpr_shift, flip, zsub, interleaved, stream);
  if (mrows == 2 && np == 2) return launch_i2_gemv<2, 2>(A, B, C, s_a, s_w, out_kind, M, N, K, tpr_shift, flip, zsub, interleaved, stream);
  if (mrows == 4 && np == 1) return launch_i2_gemv<4, 1>(A, B, C, s_a, s_w, out_kind, M, N, K, tpr_shift, flip, zsub, interleaved, stream);
  return 1;
}

}  // namespace dq
