// W2A16 decode GEMV on gfx950: C[M,N] fp16 = A[M,K] fp16 . decode(B[N,K/4])^T, fp32 accumulation.
//
// The num_bits = 2 case of examples/dequantize_gemm/example_dequant_gemv_fp16xint4.py:11-155
// (B_shape = (N, K / 8 * num_bits), slow path `_tir_packed_int_to_int_convert`, :121-124) with the
// decoders of examples/dequantize_gemm/quantize/lop3.py:424-463 (unsigned `c`, signed `c - 2`) and
// :465-500 (the same times one fp16 scale per group).
//
// Streaming shape of the other GEMVs of this library: a thread owns one 16-byte chunk (64 codes)
// of every weight row of its workgroup, the threads of a row read consecutive chunks, the loads of
// a whole batch of rows are in flight before any of it is decoded.
//
//   * a packed dword holds 16 codes; w & 0x33333333 and (w >> 2) & 0x33333333 leave one code in every
//     nibble, and a 2-bit code c read as an e2m1 nibble is c / 2, so v_cvt_scalef32_pk_f16_fp4 with the
//     scale 2 turns each byte into the exact fp16 pair (c_lo, c_hi): eleven instructions decode a
//     dword, eight v_dot2_f32_f16 consume it, and the fp32 sum sees only exact products;
//   * the thread's 64 activations are arranged once, in registers, as the pairs that decode
//     produces: (4j, 4j + 2) and (4j + 1, 4j + 3) for byte j of the plain packing; for words passed
//     through interleave_weight(qw, 2, "float16") (bytes e0 e2 e4 e6 | e1 e3 e5 e7 | e8.. | e9..) the
//     pairs (e, e + 4);
//   * the zero point is applied per chunk as  sum a (c - 2) = sum a c - 2 sum a;  two's-complement
//     codes are (c ^ 2) - 2; a group scale multiplies the fp32 sum of the thread's chunk (a chunk of
//     64 k never straddles a group: group % 64 == 0).  With the signed codes (c - 2) * s is exact in
//     fp16, so this equals the per-weight fp16 rounding of the reference's scaled decoder; with
//     unsigned codes 3 * s is the one product that the reference rounds and this kernel does not;
//   * K is reduced over the lanes with DPP row operations and over the waves of a row through LDS,
//     in a fixed order: results are bit-identical from run to run.
#include "dq_common.h"

namespace dq {

namespace {

template <int CTRL, int ROW_MASK, bool BOUND>
__device__ __forceinline__ float dpp_add(float v) {
  const int y = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, BOUND);
  return v + __builtin_bit_cast(float, y);
}

// lanes 31 and 63 end up with the sums of lanes 0..31 and 32..63
__device__ __forceinline__ float wave_half_reduce_f32(float v) {
  v = dpp_add<0xB1, 0xF, true>(v);    // quad_perm(1,0,3,2)
  v = dpp_add<0x4E, 0xF, true>(v);    // quad_perm(2,3,0,1)
  v = dpp_add<0x141, 0xF, true>(v);   // row_half_mirror
  v = dpp_add<0x140, 0xF, true>(v);   // row_mirror
  v = dpp_add<0x142, 0xA, false>(v);  // row_bcast:15
  return v;
}

constexpr int kMaxRowsPerWg = 128;

// decode one packed dword into eight fp16 pairs of codes: pair 2j + t holds fields t and t + 2 of byte j
__device__ __forceinline__ void decode_w2_dword(uint32_t w, half2_t (&out)[8]) {
  const uint32_t d0 = w & 0x33333333u;
  const uint32_t d1 = (w >> 2) & 0x33333333u;
  out[0] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(d0, 2.0f, 0);
  out[1] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(d1, 2.0f, 0);
  out[2] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(d0, 2.0f, 1);
  out[3] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(d1, 2.0f, 1);
  out[4] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(d0, 2.0f, 2);
  out[5] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(d1, 2.0f, 2);
  out[6] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(d0, 2.0f, 3);
  out[7] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(d1, 2.0f, 3);
}

template <int MROWS, int NP, int R, bool IL, bool HAS_SCALE>
__global__ __launch_bounds__(256) void w2a16_gemv_kernel(const half_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                          const half_t* __restrict__ Scale, half_t* __restrict__ C,
                                                          int M, int N, int K, int group, int tpr_shift, int nb,
                                                          uint32_t flip_mask, int zsub) {
  __shared__ float red[kMaxRowsPerWg * 4 * MROWS];

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
  const int groups = K / group;

  int boff[NP], goff[NP];
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int chunk = min(p * tpr + ct, c16 - 1);
    boff[p] = chunk * 16;
    goff[p] = (chunk * 64) / group;
  }

  uint4_t bq[R][NP];
  half_t sq[R][NP];
  auto issue_row = [&](int u, int b) {
    const int row = min(row0 + b * rows_per_batch + u * rpp + slot, N - 1);
    const uint8_t* bp = B + (size_t)row * row_bytes;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      bq[u][p] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(bp + boff[p]));
      if constexpr (HAS_SCALE) sq[u][p] = Scale[(size_t)row * groups + goff[p]];
    }
  };
#pragma unroll
  for (int u = 0; u < R; ++u) issue_row(u, 0);

  // the thread's activations, paired as the decoder pairs the codes
  uint32_t a[NP][MROWS][32];
  float zasum[NP][MROWS];  // zero point times the sum of the chunk's activations
  const half2_t one2 = {(half_t)1.f, (half_t)1.f};
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int chunk = p * tpr + ct;
    const bool valid = chunk < c16;
#pragma unroll
    for (int m = 0; m < MROWS; ++m) {
      const half_t* ap = A + (size_t)min(m, M - 1) * K + (size_t)min(chunk, c16 - 1) * 64;
      float asum = 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {  // packed dword j: k = 16 j .. 16 j + 15, natural registers n[0..7]
        uint4_t lo = *reinterpret_cast<const uint4_t*>(ap + j * 16);
        uint4_t hi = *reinterpret_cast<const uint4_t*>(ap + j * 16 + 8);
        if (!valid) {
          lo = uint4_t{0u, 0u, 0u, 0u};
          hi = uint4_t{0u, 0u, 0u, 0u};
        }
        const uint32_t n[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
#pragma unroll
        for (int q = 0; q < 8; ++q) {
          const int bj = q >> 1, t = q & 1;  // byte of the packed dword, first field of the pair
          uint32_t v;
          if constexpr (IL) {
            // byte bj holds e[8 (bj / 2) + (bj % 2) + 2 f] in field f: the pair is (e, e + 4)
            const int i = 4 * (bj >> 1) + t;
            v = __builtin_amdgcn_perm(n[i + 2], n[i], (bj & 1) ? 0x07060302u : 0x05040100u);
          } else {
            // byte bj holds e[4 bj + f] in field f: the pair is (4 bj + t, 4 bj + t + 2)
            v = __builtin_amdgcn_perm(n[2 * bj + 1], n[2 * bj], t ? 0x07060302u : 0x05040100u);
          }
          a[p][m][j * 8 + q] = v;
          asum = __builtin_amdgcn_fdot2(as_half2(v), one2, asum, false);
        }
      }
      zasum[p][m] = (float)zsub * asum;
    }
  }

  for (int b = 0; b < nb; ++b) {
    float acc[R][MROWS];
#pragma unroll
    for (int u = 0; u < R; ++u) {
#pragma unroll
      for (int m = 0; m < MROWS; ++m) acc[u][m] = 0.f;
#pragma unroll
      for (int p = 0; p < NP; ++p) {
        float part[MROWS];
#pragma unroll
        for (int m = 0; m < MROWS; ++m) part[m] = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          half2_t wv[8];
          decode_w2_dword(bq[u][p][j] ^ flip_mask, wv);
#pragma unroll
          for (int q = 0; q < 8; ++q) {
#pragma unroll
            for (int m = 0; m < MROWS; ++m)
              part[m] = __builtin_amdgcn_fdot2(as_half2(a[p][m][j * 8 + q]), wv[q], part[m], false);
          }
        }
#pragma unroll
        for (int m = 0; m < MROWS; ++m) {
          if constexpr (HAS_SCALE) acc[u][m] = __builtin_fmaf((float)sq[u][p], part[m] - zasum[p][m], acc[u][m]);
          else acc[u][m] += part[m] - zasum[p][m];
        }
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
        float v = wave_half_reduce_f32(acc[u][m]);
        if (tpr >= 64) {
          v = dpp_add<0x143, 0xC, false>(v);  // row_bcast:31: lane 63 holds the wave's sum
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
    float v = red[(rl * 4 + 0) * MROWS + m];
    for (int w = 1; w < waves_per_row; ++w) v += red[(rl * 4 + w) * MROWS + m];
    const int row = row0 + rl;
    if (row < N && m < M) C[(size_t)m * N + row] = (half_t)v;
  }
}

template <int MROWS, int NP, bool IL, bool HAS_SCALE>
int launch_w2(const void* A, const void* B, const void* Scale, void* C, int M, int N, int K, int group, int tpr_shift,
              uint32_t flip, int zsub, hipStream_t stream) {
  constexpr int R = 4 / NP;
  const int rpp = 256 >> tpr_shift;
  const long wgs1 = ((long)N + R * rpp - 1) / (R * rpp);
  // about two workgroups per CU, each walking several batches of rows
  int nb = (int)((wgs1 + 511) / 512);
  while (nb > 1 && nb * R * rpp > kMaxRowsPerWg) --nb;
  if (nb < 1) nb = 1;
  const int rows_per_wg = nb * R * rpp;
  hipLaunchKernelGGL((w2a16_gemv_kernel<MROWS, NP, R, IL, HAS_SCALE>), dim3((N + rows_per_wg - 1) / rows_per_wg),
                     dim3(256), 0, stream, (const half_t*)A, (const uint8_t*)B, (const half_t*)Scale, (half_t*)C, M, N, K,
                     group, tpr_shift, nb, flip, zsub);
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

template <int MROWS, int NP>
int dispatch_w2(bool il, bool has_scale, const void* A, const void* B, const void* Scale, void* C, int M, int N, int K,
                int group, int tpr_shift, uint32_t flip, int zsub, hipStream_t stream) {
  if (il) {
    if (has_scale) return launch_w2<MROWS, NP, true, true>(A, B, Scale, C, M, N, K, group, tpr_shift, flip, zsub, stream);
    return launch_w2<MROWS, NP, true, false>(A, B, Scale, C, M, N, K, group, tpr_shift, flip, zsub, stream);
  }
  if (has_scale) return launch_w2<MROWS, NP, false, true>(A, B, Scale, C, M, N, K, group, tpr_shift, flip, zsub, stream);
  return launch_w2<MROWS, NP, false, false>(A, B, Scale, C, M, N, K, group, tpr_shift, flip, zsub, stream);
}

}  // namespace

// Activation rows go through the kernel two at a time (the weights are streamed once per pair).
// Returns 1 when the shape is not covered (K beyond 32768).
int w2a16_gemv(const void* A, const void* B, const void* Scale, void* C, int M, int N, int K, int group, int convention,
               int layout, hipStream_t stream) {
  const int c16 = K / 64;
  int tpr_shift = 5;
  while ((1 << tpr_shift) < c16 && tpr_shift < 8) ++tpr_shift;
  const int np = (c16 + (1 << tpr_shift) - 1) >> tpr_shift;
  if (np > 2) return 1;
  uint32_t flip = 0;
  int zsub = 0;
  if (convention == I2_OFFSET) zsub = 2;
  else if (convention == I2_TWOS) { flip = 0xAAAAAAAAu; zsub = 2; }
  const bool il = layout == LAYOUT_INTERLEAVED;
  const bool has_scale = Scale != nullptr;
  for (int m0 = 0; m0 < M; m0 += 2) {
    const int mm = M - m0 >= 2 ? 2 : 1;
    const half_t* a = (const half_t*)A + (size_t)m0 * K;
    half_t* c = (half_t*)C + (size_t)m0 * N;
    int rc;
    if (mm == 1 && np == 1) rc = dispatch_w2<1, 1>(il, has_scale, a, B, Scale, c, mm, N, K, group, tpr_shift, flip, zsub, stream);
    else if (mm == 1) rc = dispatch_w2<1, 2>(il, has_scale, a, B, Scale, c, mm, N, K, group, tpr_shift, flip, zsub, stream);
    else if (np == 1) rc = dispatch_w2<2, 1>(il, has_scale, a, B, Scale, c, mm, N, K, group, tpr_shift, flip, zsub, stream);
    else rc = dispatch_w2<2, 2>(il, has_scale, a, B, Scale, c, mm, N, K, group, tpr_shift, flip, zsub, stream);
    if (rc) return rc;
  }
  return 0;
}

}  // namespace dq
