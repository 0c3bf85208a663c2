// fp16 x 2-bit and fp16 x 1-bit decode GEMV on gfx950:
// C[M,N] fp16 = A[M,K] fp16 . decode(B[N, K * bits / 8])^T, fp32 accumulation.
//
// The num_bits = 2 and num_bits = 1 cases of examples/dequantize_gemm/example_dequant_gemv_fp16xint4.py:11-155
// (B_shape = (N, K / 8 * num_bits), slow path `_tir_packed_int_to_int_convert`, :121-124) with the
// decoders of examples/dequantize_gemm/quantize/lop3.py:424-463 and :679-746 (unsigned `c`; signed
// `c - 2` for two bits, `2 c - 1` for one), their scaled forms (:465-500, :748-810) and the zero-point
// forms "original" `(w - z) * s` and "rescale" `w * s - z` (:564-636, :812-891).
//
// Streaming shape of the other GEMVs of this library: a thread owns one 16-byte chunk (64 or 128
// codes) of every weight row of its workgroup, the threads of a row read consecutive chunks, the
// loads of a whole batch of rows are in flight before any of it is decoded.
//
//   * (w >> t) & 0x33333333 (t = 0, 2) or & 0x11111111 (t = 0..3) leaves one code in every nibble,
//     and a code read as an e2m1 nibble is c / 2, so v_cvt_scalef32_pk_f16_fp4 with the scale 2
//     turns each byte into the exact fp16 pair (c_lo, c_hi); the products with the activations are
//     exact in fp32 and are summed on the matrix pipe (see the loop), so the VALU only decodes;
//   * the thread's activations are arranged once, in registers, as the pairs that decode produces;
//     which two elements meet in a byte follows from the packing (plain, or the words of
//     interleave_weight(qw, bits, "float16"), examples/dequantize_gemm/quantize/utils.py:71-123) and
//     is worked out at compile time (elem_at_bit);
//   * every decoder is affine in the code, w = alpha c + beta, so a chunk contributes
//     alpha sum(a c) + beta sum(a); two's-complement 2-bit codes are (c ^ 2) - 2, two's-complement
//     1-bit codes are -c.  A group scale and zero point act on the chunk's fp32 sums (a chunk never
//     straddles a group).  For the signed 2-bit codes (c - 2) * s is exact in fp16, so this equals the
//     per-weight fp16 rounding of the reference's scaled decoder; elsewhere the reference rounds each
//     weight to fp16 and this kernel does not (far inside the 1e-2 tolerance);
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

// Bit of a packed 32-bit word at which element e of the word starts.
constexpr int bit_of_elem(int bits, bool interleaved, int e) {
  if (!interleaved) return bits * e;
  // interleave_weight(.., bits, "float16"): even elements fill the low halfword, odd ones the high
  const int p = (e % 2) * 16 + (e / 2) * bits;
  if (bits == 2) {
    const int bytemap[4] = {0, 2, 1, 3};  // bytes 1 and 2 change places
    return 8 * bytemap[p / 8] + p % 8;
  }
  const int nibmap[8] = {0, 2, 4, 6, 1, 3, 5, 7};  // one bit: nibbles 1..6 are shuffled as well
  return 4 * nibmap[p / 4] + p % 4;
}

constexpr int elem_at_bit(int bits, bool interleaved, int bit) {
  for (int e = 0; e < 32 / bits; ++e)
    if (bit_of_elem(bits, interleaved, e) == bit) return e;
  return -1;
}

// Pair q of a packed dword (the codes at bits 8 j + BITS t and 8 j + 4 + BITS t, q = NT j + t):
// the v_perm_b32 selector that builds (a[e_lo], a[e_hi]) from the natural registers, and those registers.
template <int BITS, bool IL, int Q>
struct PairOf {
  static constexpr int NT = 4 / BITS;
  static constexpr int e_lo = elem_at_bit(BITS, IL, 8 * (Q / NT) + BITS * (Q % NT));
  static constexpr int e_hi = elem_at_bit(BITS, IL, 8 * (Q / NT) + 4 + BITS * (Q % NT));
  static_assert(e_lo >= 0 && e_hi >= 0, "every bit position holds an element");
  static constexpr uint32_t sel = ((e_lo & 1) ? 0x0302u : 0x0100u) | (((e_hi & 1) ? 0x0706u : 0x0504u) << 16);
};

template <int BITS, bool IL, int Q, int PAIRS>
__device__ __forceinline__ void pair_activations(const uint32_t (&n)[PAIRS], uint32_t* out, float& sum) {
  if constexpr (Q < PAIRS) {
    using P = PairOf<BITS, IL, Q>;
    const uint32_t v = __builtin_amdgcn_perm(n[P::e_hi >> 1], n[P::e_lo >> 1], P::sel);
    out[Q] = v;
    const half2_t one2 = {(half_t)1.f, (half_t)1.f};
    sum = __builtin_amdgcn_fdot2(as_half2(v), one2, sum, false);
    pair_activations<BITS, IL, Q + 1, PAIRS>(n, out, sum);
  }
}

template <int BYTE>
__device__ __forceinline__ half2_t cvt_codes(uint32_t d) {
  return __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(d, 2.0f, BYTE);
}

// one packed dword -> 16 / BITS fp16 pairs of codes, pair NT j + t from byte j of (w >> BITS t) & mask
template <int BITS>
__device__ __forceinline__ void decode_codes(uint32_t w, half2_t (&out)[16 / BITS]) {
  constexpr int NT = 4 / BITS;
  constexpr uint32_t kMask = BITS == 2 ? 0x33333333u : 0x11111111u;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const uint32_t d = (w >> (BITS * t)) & kMask;
    out[0 * NT + t] = cvt_codes<0>(d);
    out[1 * NT + t] = cvt_codes<1>(d);
    out[2 * NT + t] = cvt_codes<2>(d);
    out[3 * NT + t] = cvt_codes<3>(d);
  }
}

enum ZeroMode : int { Z_NONE = 0, Z_ORIGINAL = 1, Z_RESCALE = 2 };

// SZ: 0 no scale, 1 group scales, 2 group scales and zero points (zmode: original or rescale)
template <int BITS, int MROWS, int NP, int R, bool IL, int SZ>
__global__ __launch_bounds__(256) void wlow_gemv_kernel(const half_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                         const half_t* __restrict__ Scale, const half_t* __restrict__ Zeros,
                                                         half_t* __restrict__ C, int M, int N, int K, int group,
                                                         int tpr_shift, int nb, uint32_t flip_mask, float alpha, float beta,
                                                         int zmode) {
  constexpr int CPD = 32 / BITS;  // codes per packed dword
  constexpr int CHUNK = 4 * CPD;  // codes per 16-byte chunk
  constexpr int PAIRS = CPD / 2;  // fp16 pairs per packed dword
  __shared__ float red[kMaxRowsPerWg * 4 * MROWS];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int tpr = 1 << tpr_shift;
  const int rpp = 256 >> tpr_shift;
  const int slot = tid >> tpr_shift;
  const int ct = tid & (tpr - 1);
  const int wave_in_row = ct >> 6;
  const int c16 = K / CHUNK;  // 16-byte chunks per row
  const int rows_per_batch = R * rpp;
  const int rows_per_wg = nb * rows_per_batch;
  const int row0 = blockIdx.x * rows_per_wg;
  const size_t row_bytes = (size_t)c16 * 16;
  const int groups = K / group;

  int boff[NP], goff[NP];
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int chunk = min(p * tpr + ct, c16 - 1);
    boff[p] = chunk * 16;
    goff[p] = (chunk * CHUNK) / group;
  }

  uint4_t bq[R][NP];
  half_t sq[R][NP], zq[R][NP];
  auto issue_row = [&](int u, int b) {
    const int row = min(row0 + b * rows_per_batch + u * rpp + slot, N - 1);
    const uint8_t* bp = B + (size_t)row * row_bytes;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      bq[u][p] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(bp + boff[p]));
      if constexpr (SZ >= 1) sq[u][p] = Scale[(size_t)row * groups + goff[p]];
      if constexpr (SZ == 2) zq[u][p] = Zeros[(size_t)row * groups + goff[p]];
    }
  };
#pragma unroll
  for (int u = 0; u < R; ++u) issue_row(u, 0);

  // the thread's activations, paired as the decoder pairs the codes, and their sum per chunk
  uint32_t a[NP][MROWS][4 * PAIRS];
  float asum[NP][MROWS];
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int chunk = p * tpr + ct;
    const bool valid = chunk < c16;
#pragma unroll
    for (int m = 0; m < MROWS; ++m) {
      const half_t* ap = A + (size_t)min(m, M - 1) * K + (size_t)min(chunk, c16 - 1) * CHUNK;
      float s = 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {  // packed dword j: elements CPD j .. CPD j + CPD - 1 in natural registers n[]
        uint32_t n[PAIRS];
#pragma unroll
        for (int i = 0; i < PAIRS / 4; ++i) {
          uint4_t d = *reinterpret_cast<const uint4_t*>(ap + j * CPD + i * 8);
          if (!valid) d = uint4_t{0u, 0u, 0u, 0u};
          n[4 * i + 0] = d[0];
          n[4 * i + 1] = d[1];
          n[4 * i + 2] = d[2];
          n[4 * i + 3] = d[3];
        }
        pair_activations<BITS, IL, 0, PAIRS>(n, &a[p][m][j * PAIRS], s);
      }
      asum[p][m] = s;
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
        // Four k per lane and instruction on the matrix pipe: v_mfma_f32_4x4x4_16B_f16 multiplies, in each
        // group of four lanes, the four weight vectors with the four activation vectors of those lanes; the
        // diagonal (lane i: register i) is the lane's own dot product, the other twelve products are unused.
        // The conversions above it stay on the VALU, so the two pipes overlap.
        float4_t part4[MROWS];
#pragma unroll
        for (int m = 0; m < MROWS; ++m) part4[m] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          half2_t wv[PAIRS];
          decode_codes<BITS>(bq[u][p][j] ^ flip_mask, wv);
#pragma unroll
          for (int q = 0; q < PAIRS; q += 2) {
            const half4_t w4 = {wv[q][0], wv[q][1], wv[q + 1][0], wv[q + 1][1]};
#pragma unroll
            for (int m = 0; m < MROWS; ++m) {
              const half2_t a0 = as_half2(a[p][m][j * PAIRS + q]), a1 = as_half2(a[p][m][j * PAIRS + q + 1]);
              const half4_t a4 = {a0[0], a0[1], a1[0], a1[1]};
              part4[m] = __builtin_amdgcn_mfma_f32_4x4x4f16(w4, a4, part4[m], 0, 0, 0);
            }
          }
        }
        float part[MROWS];
#pragma unroll
        for (int m = 0; m < MROWS; ++m) {
          const float p01 = (lane & 1) ? part4[m][1] : part4[m][0];
          const float p23 = (lane & 1) ? part4[m][3] : part4[m][2];
          part[m] = (lane & 2) ? p23 : p01;
        }
#pragma unroll
        for (int m = 0; m < MROWS; ++m) {
          // w = alpha c + beta; alpha is 1 for two bits
          const float ac = BITS == 1 ? alpha * part[m] : part[m];
          if constexpr (SZ == 2) {
            // original: (w - z) s;  rescale: w s - z
            const float z = (float)zq[u][p];
            const float b_eff = zmode == Z_ORIGINAL ? beta - z : beta;
            const float sub = zmode == Z_RESCALE ? z * asum[p][m] : 0.f;
            const float lin = __builtin_fmaf(b_eff, asum[p][m], ac);
            acc[u][m] += __builtin_fmaf((float)sq[u][p], lin, -sub);
          } else if constexpr (SZ == 1) {
            acc[u][m] = __builtin_fmaf((float)sq[u][p], __builtin_fmaf(beta, asum[p][m], ac), acc[u][m]);
          } else {
            acc[u][m] += __builtin_fmaf(beta, asum[p][m], ac);
          }
        }
      }
      // the row's registers are free: its place in the next batch is requested while the other rows are
      // worked on (wave-uniform branch)
      if (b + 1 < nb) issue_row(u, b + 1);
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

struct LowArgs {
  const void *A, *B, *Scale, *Zeros;
  void* C;
  int M, N, K, group, tpr_shift;
  uint32_t flip;
  float alpha, beta;
  int zmode;
  hipStream_t stream;
};

template <int BITS, int MROWS, int NP, bool IL, int SZ>
int launch_low(const LowArgs& g) {
  constexpr int R = 4 / NP;  // rows in flight per thread (eight measured slower)
  const int rpp = 256 >> g.tpr_shift;
  const long wgs1 = ((long)g.N + R * rpp - 1) / (R * rpp);
  // about two workgroups per CU, each walking several batches of rows
  // (measured at N = 28672, K = 8192: 512 workgroups 15.8 us, 1024 17.5 us, one batch each 20.7 us)
  int nb = (int)((wgs1 + 511) / 512);
  while (nb > 1 && nb * R * rpp > kMaxRowsPerWg) --nb;
  if (nb < 1) nb = 1;
  const int rows_per_wg = nb * R * rpp;
  hipLaunchKernelGGL((wlow_gemv_kernel<BITS, MROWS, NP, R, IL, SZ>), dim3((g.N + rows_per_wg - 1) / rows_per_wg),
                     dim3(256), 0, g.stream, (const half_t*)g.A, (const uint8_t*)g.B, (const half_t*)g.Scale,
                     (const half_t*)g.Zeros, (half_t*)g.C, g.M, g.N, g.K, g.group, g.tpr_shift, nb, g.flip, g.alpha, g.beta,
                     g.zmode);
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

template <int BITS, int MROWS, int NP>
int dispatch_low(const LowArgs& g, bool il) {
  const int sz = g.Scale ? (g.Zeros ? 2 : 1) : 0;
  if (il) {
    if (sz == 2) return launch_low<BITS, MROWS, NP, true, 2>(g);
    return sz == 1 ? launch_low<BITS, MROWS, NP, true, 1>(g) : launch_low<BITS, MROWS, NP, true, 0>(g);
  }
  if (sz == 2) return launch_low<BITS, MROWS, NP, false, 2>(g);
  return sz == 1 ? launch_low<BITS, MROWS, NP, false, 1>(g) : launch_low<BITS, MROWS, NP, false, 0>(g);
}

}  // namespace

// `convention`: I2_UNSIGNED c, I2_OFFSET the signed fast decoder (c - 2; one bit: 2 c - 1), I2_TWOS two's
// complement of the field.  Activation rows go through the kernel two at a time (the weights are streamed once
// per pair).  Returns 1 when the shape is not covered.
int wlow_gemv(const void* A, const void* B, const void* Scale, const void* Zeros, void* C, int M, int N, int K, int group,
              int bits, int convention, int layout, int zeros_rescale, hipStream_t stream) {
  const int chunk = bits == 2 ? 64 : 128;
  if (K % chunk != 0) return 1;
  const int c16 = K / chunk;
  int tpr_shift = 5;
  while ((1 << tpr_shift) < c16 && tpr_shift < 8) ++tpr_shift;
  const int np = (c16 + (1 << tpr_shift) - 1) >> tpr_shift;
  if (np > (bits == 2 ? 2 : 1)) return 1;
  LowArgs g{};
  g.B = B;
  g.Scale = Scale;
  g.Zeros = Zeros;
  g.N = N;
  g.K = K;
  g.group = group;
  g.tpr_shift = tpr_shift;
  g.stream = stream;
  g.flip = 0;
  g.alpha = 1.f;
  g.beta = 0.f;
  if (bits == 2) {
    if (convention == I2_OFFSET) g.beta = -2.f;
    else if (convention == I2_TWOS) { g.flip = 0xAAAAAAAAu; g.beta = -2.f; }
  } else {
    if (convention == I2_OFFSET) { g.alpha = 2.f; g.beta = -1.f; }
    else if (convention == I2_TWOS) g.alpha = -1.f;
  }
  g.zmode = Zeros ? (zeros_rescale ? Z_RESCALE : Z_ORIGINAL) : Z_NONE;
  const bool il = layout == LAYOUT_INTERLEAVED;
  for (int m0 = 0; m0 < M; m0 += 2) {
    const int mm = M - m0 >= 2 ? 2 : 1;
    g.A = (const half_t*)A + (size_t)m0 * K;
    g.C = (half_t*)C + (size_t)m0 * N;
    g.M = mm;
    int rc;
    if (bits == 2) {
      if (mm == 1 && np == 1) rc = dispatch_low<2, 1, 1>(g, il);
      else if (mm == 1) rc = dispatch_low<2, 1, 2>(g, il);
      else if (np == 1) rc = dispatch_low<2, 2, 1>(g, il);
      else rc = dispatch_low<2, 2, 2>(g, il);
    } else {
      rc = mm == 1 ? dispatch_low<1, 1, 1>(g, il) : dispatch_low<1, 2, 1>(g, il);
    }
    if (rc) return rc;
  }
  return 0;
}

}  // namespace dq
