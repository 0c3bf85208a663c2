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
//   * K is reduced over each 16-lane row with DPP operations (the values of a batch of rows together, so
//     that most steps halve their number) and over the 16-lane rows of a weight row through LDS, in a fixed
//     order: results are bit-identical from run to run;
//   * when a weight row takes a whole wave or more, the row's address lives in scalar registers and the
//     loads add the lane's offset themselves; the matrix instruction writes ordinary vector registers
//     (the file is compiled with -amdgpu-mfma-vgpr-form), so its diagonal is picked without register copies.
#include "dq_common.h"

#include <type_traits>

namespace dq {

namespace {

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
// (`flip` turns two's-complement fields into offset ones; it is zero otherwise and costs nothing either way)
template <int BITS>
__device__ __forceinline__ void decode_codes(uint32_t w, uint32_t flip, half2_t (&out)[16 / BITS]) {
  constexpr int NT = 4 / BITS;
  constexpr uint32_t kMask = BITS == 2 ? 0x33333333u : 0x11111111u;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    // (x ^ f) & mask in one instruction
    const uint32_t d = __builtin_amdgcn_bitop3_b32(w >> (BITS * t), flip >> (BITS * t), kMask, 0x28);
    out[0 * NT + t] = cvt_codes<0>(d);
    out[1 * NT + t] = cvt_codes<1>(d);
    out[2 * NT + t] = cvt_codes<2>(d);
    out[3 * NT + t] = cvt_codes<3>(d);
  }
}

// Global-memory pointer (the address space is spelled out so that an address rebuilt from integers still loads
// through the global path).
typedef const __attribute__((address_space(1))) uint8_t* gptr_t;

// A pointer that is the same in every lane, pinned to scalar registers: the loads then take it as their scalar
// base and add the lane's 32-bit offset themselves.
template <bool UNIFORM>
__device__ __forceinline__ gptr_t uniform_if(const uint8_t* p) {
  if constexpr (UNIFORM) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (gptr_t)(((uint64_t)hi << 32) | lo);
  } else {
    return (gptr_t)p;
  }
}

enum ZeroMode : int { Z_NONE = 0, Z_ORIGINAL = 1, Z_RESCALE = 2 };

// SZ: 0 no scale, 1 group scales, 2 group scales and zero points (zmode: original or rescale).
// WIDE: a row takes at least a whole wave (tpr >= 64), so the row a wave works on is the same for its 64 lanes
// and its address is kept in scalar registers (the loads take a scalar base and a per-lane offset).
template <int BITS, int MROWS, int NP, int R, bool IL, int SZ, bool WIDE>
__global__ __launch_bounds__(256) void wlow_gemv_kernel(const half_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                         const half_t* __restrict__ Scale, const half_t* __restrict__ Zeros,
                                                         half_t* __restrict__ C, int M, int N, int K, int group,
                                                         int tpr_shift, int rows_quot, int rows_rem, uint32_t flip_mask,
                                                         float alpha, float beta, int zmode) {
  constexpr int CPD = 32 / BITS;  // codes per packed dword
  constexpr int CHUNK = 4 * CPD;  // codes per 16-byte chunk
  constexpr int PAIRS = CPD / 2;  // fp16 pairs per packed dword
  constexpr int NV = R * MROWS;   // values reduced together per batch
  static_assert(NV <= 16, "at most 16 values per lane row");
  // partial sums: [batch][16-lane row of the workgroup (16)][value]
  __shared__ float red[kMaxRowsPerWg * 16 * MROWS];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int tpr = 1 << tpr_shift;
  const int rpp = 256 >> tpr_shift;
  const int slot = WIDE ? __builtin_amdgcn_readfirstlane(tid >> tpr_shift) : (tid >> tpr_shift);
  const int ct = tid & (tpr - 1);
  const int c16 = K / CHUNK;  // 16-byte chunks per row
  const int rows_per_batch = R * rpp;
  // The grid splits the rows evenly, whatever its size: with N = G quot + rem, workgroup i owns the rows from
  // i quot + min(i, rem) up to the next workgroup's first, both bounds rounded down to whole passes, and walks them
  // in batches.  Past the end of its range the last batch works on the range's last row again (loads and
  // arithmetic stay free of branches; those results are never read).
  const int wg = blockIdx.x;
  const int row0 = (wg * rows_quot + min(wg, rows_rem)) & ~(rpp - 1);
  const int row1 = wg + 1 == (int)gridDim.x ? N : ((wg + 1) * rows_quot + min(wg + 1, rows_rem)) & ~(rpp - 1);
  const int rows_per_wg = row1 - row0;  // the host sizes the grid so that nb * rows_per_batch <= kMaxRowsPerWg
  const int nb = (rows_per_wg + rows_per_batch - 1) / rows_per_batch;
  const int row_last = max(min(row1, N) - 1, 0);
  const uint32_t row_bytes = (uint32_t)c16 * 16u;
  const int groups = K / group;

  uint32_t boff[NP], goff[NP];
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int chunk = min(p * tpr + ct, c16 - 1);
    boff[p] = (uint32_t)chunk * 16u;
    goff[p] = (uint32_t)((chunk * CHUNK) / group) * 2u;
  }

  uint4_t bq[R][NP];
  half_t sq[R][NP], zq[R][NP];
  auto issue_row = [&](int u, int b) {
    const int row = min(row0 + b * rows_per_batch + u * rpp + slot, row_last);
    const gptr_t bp = uniform_if<WIDE>(B + (size_t)row * row_bytes);
    const gptr_t sp = uniform_if<WIDE>(reinterpret_cast<const uint8_t*>(Scale) + (size_t)row * groups * 2);
    const gptr_t zp = uniform_if<WIDE>(reinterpret_cast<const uint8_t*>(Zeros) + (size_t)row * groups * 2);
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      bq[u][p] = __builtin_nontemporal_load((const __attribute__((address_space(1))) uint4_t*)(bp + boff[p]));
      if constexpr (SZ >= 1) sq[u][p] = *(const __attribute__((address_space(1))) half_t*)(sp + goff[p]);
      if constexpr (SZ == 2) zq[u][p] = *(const __attribute__((address_space(1))) half_t*)(zp + goff[p]);
    }
  };
#pragma unroll
  for (int u = 0; u < R; ++u) issue_row(u, 0);

  // The thread's activations, paired as the decoder pairs the codes, and their sum per chunk (requested behind
  // the first weight rows: ahead of them measured 0.6 us slower).
  uint32_t a[NP][MROWS][4 * PAIRS];
  float asum[NP][MROWS];
  auto load_activations = [&](int p, int m, uint32_t (&raw)[4][PAIRS]) {
    const int chunk = p * tpr + ct;
    const bool valid = chunk < c16;
    const half_t* ap = A + (size_t)min(m, M - 1) * K + (size_t)min(chunk, c16 - 1) * CHUNK;
#pragma unroll
    for (int j = 0; j < 4; ++j)  // packed dword j: elements CPD j .. CPD j + CPD - 1 in natural order
#pragma unroll
      for (int i = 0; i < PAIRS / 4; ++i) {
        uint4_t d = *reinterpret_cast<const uint4_t*>(ap + j * CPD + i * 8);
        if (!valid) d = uint4_t{0u, 0u, 0u, 0u};
        raw[j][4 * i + 0] = d[0];
        raw[j][4 * i + 1] = d[1];
        raw[j][4 * i + 2] = d[2];
        raw[j][4 * i + 3] = d[3];
      }
  };
  auto pair_up = [&](int p, int m, const uint32_t (&raw)[4][PAIRS]) {
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) pair_activations<BITS, IL, 0, PAIRS>(raw[j], &a[p][m][j * PAIRS], s);
    asum[p][m] = s;
  };
#pragma unroll
  for (int p = 0; p < NP; ++p)
#pragma unroll
    for (int m = 0; m < MROWS; ++m) {
      uint32_t raw[4][PAIRS];
      load_activations(p, m, raw);
      pair_up(p, m, raw);
    }

  // After the row reduction lane l of a 16-lane row holds the row's total of value l & (NV - 1).
  const bool writer = (lane & 15) < NV;
  float* red_w = red + (tid >> 4) * NV + (lane & (NV - 1));

  auto process_batch = [&](int b, auto refill_tag) {
    constexpr bool kRefill = decltype(refill_tag)::value;
    float acc[NV];
#pragma unroll
    for (int u = 0; u < R; ++u) {
#pragma unroll
      for (int m = 0; m < MROWS; ++m) acc[u * MROWS + m] = 0.f;
      // the last batch may be partly empty (the same for every thread; no loads are issued in it)
      if (!kRefill && b * rows_per_batch + u * rpp >= rows_per_wg) continue;
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
          decode_codes<BITS>(bq[u][p][j], flip_mask, wv);
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
          float& dst = acc[u * MROWS + m];
          if constexpr (SZ == 2) {
            // original: (w - z) s;  rescale: w s - z
            const float z = (float)zq[u][p];
            const float b_eff = zmode == Z_ORIGINAL ? beta - z : beta;
            const float sub = zmode == Z_RESCALE ? z * asum[p][m] : 0.f;
            const float lin = __builtin_fmaf(b_eff, asum[p][m], ac);
            dst += __builtin_fmaf((float)sq[u][p], lin, -sub);
          } else if constexpr (SZ == 1) {
            dst = __builtin_fmaf((float)sq[u][p], __builtin_fmaf(beta, asum[p][m], ac), dst);
          } else {
            dst += __builtin_fmaf(beta, asum[p][m], ac);
          }
        }
      }
      // the row's registers are free: its place in the next batch is requested while the other rows are
      // worked on
      if constexpr (kRefill) issue_row(u, b + 1);
    }
    const float v = RowReduce<NV, 0>::run(acc, lane);
    if (writer) red_w[b * 16 * NV] = v;
  };
  for (int b = 0; b + 1 < nb; ++b) process_batch(b, std::true_type{});
  if (nb > 0) process_batch(nb - 1, std::false_type{});
  __syncthreads();

  // fixed-order sum of the 16-lane partials of each output
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

struct LowArgs {
  const void *A, *B, *Scale, *Zeros;
  void* C;
  int M, N, K, group, tpr_shift;
  uint32_t flip;
  float alpha, beta;
  int zmode;
  hipStream_t stream;
};

template <int BITS, int MROWS, int NP, bool IL, int SZ, bool WIDE>
int launch_low(const LowArgs& g) {
  constexpr int R = 4 / NP;  // rows in flight per thread (eight: no faster)
  const int rpp = 256 >> g.tpr_shift;
  // Two workgroups per CU, each walking several batches of rows: every workgroup arranges the activations for
  // itself before its first batch (as many instructions as a batch takes) and fills its pipeline once, so a finer
  // grid costs more than its extra loads in flight bring (N = 28672, K = 8192: 512 workgroups 15.0 us, 768 15.5 us,
  // 1024 16.1 us, 1792 16.7 us, 256 19.2 us).  Never fewer rows than one batch per workgroup, never more than the
  // partial sums in LDS hold.
  const long batches = ((long)g.N + R * rpp - 1) / (R * rpp);
  long wgs = 512;
  if (wgs > batches) wgs = batches;
  const long rows_max = kMaxRowsPerWg - R * rpp - rpp;  // leaves room for the rounding of the bounds and of nb
  const long wgs_min = ((long)g.N + rows_max - 1) / rows_max;
  if (wgs < wgs_min) wgs = wgs_min;
  hipLaunchKernelGGL((wlow_gemv_kernel<BITS, MROWS, NP, R, IL, SZ, WIDE>), dim3((unsigned)wgs), dim3(256), 0, g.stream,
                     (const half_t*)g.A, (const uint8_t*)g.B, (const half_t*)g.Scale, (const half_t*)g.Zeros,
                     (half_t*)g.C, g.M, g.N, g.K, g.group, g.tpr_shift, (int)(g.N / wgs), (int)(g.N % wgs), g.flip,
                     g.alpha, g.beta, g.zmode);
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

template <int BITS, int MROWS, int NP, bool IL, int SZ>
int launch_low_w(const LowArgs& g) {
  if constexpr (NP > 1) return launch_low<BITS, MROWS, NP, IL, SZ, true>(g);  // more than one chunk: 256 threads a row
  if (g.tpr_shift >= 6) return launch_low<BITS, MROWS, NP, IL, SZ, true>(g);
  return launch_low<BITS, MROWS, NP, IL, SZ, false>(g);
}

template <int BITS, int MROWS, int NP>
int dispatch_low(const LowArgs& g, bool il) {
  const int sz = g.Scale ? (g.Zeros ? 2 : 1) : 0;
  if (il) {
    if (sz == 2) return launch_low_w<BITS, MROWS, NP, true, 2>(g);
    return sz == 1 ? launch_low_w<BITS, MROWS, NP, true, 1>(g) : launch_low_w<BITS, MROWS, NP, true, 0>(g);
  }
  if (sz == 2) return launch_low_w<BITS, MROWS, NP, false, 2>(g);
  return sz == 1 ? launch_low_w<BITS, MROWS, NP, false, 1>(g) : launch_low_w<BITS, MROWS, NP, false, 0>(g);
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
