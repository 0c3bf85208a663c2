// Integer decode GEMV for M <= 4 on gfx950: C[M,N] = A[M,K] int8 . decode(B[N, K BITS / 8])^T, exact int32, for
// 4-bit, 2-bit and 1-bit weights.
//
// Replaces the integer branch (`use_dp4a`) of the kernel generated from
// examples/dequantize_gemm/example_dequant_gemv_fp16xint4.py:47-54,126-133 (16 int8 per lane, T.dp4a, 32-lane
// all-reduce) with the decoders decode_i{4,2,1}{s,u}_to_i8s of examples/dequantize_gemm/quantize/lop3.py:893-1047,
// and, for two bits, the kernel of examples/bitnet-1.58b/kernel_benchmark/
// tilelang_bitnet_158_int8xint2_decode.py:93-173.  Same streaming shape as the W4A16 GEMV: a thread owns one
// 16-byte chunk (128 / BITS codes) of every weight row of its workgroup, the threads of a row read consecutive
// chunks, all loads of a batch are issued before the data is touched.
//
//   * (w >> BITS i) & mask puts code (8 / BITS) b + i of packed byte b into byte b of dword i; the thread's
//     activations are held in that same order (a byte shuffle per chunk, done once, that depends on BITS and on the
//     word layout), so each dword goes straight into v_dot4_i32_i8;
//   * every decoder is  w = mul c' - zsub  with c' = c ^ flip:  sum a w = mul sum a c' - zsub sum a  (exact in
//     integers).  Unsigned: (1, 0, 0).  Two's complement: sext(c) = (c ^ top) - top.  The signed fast decoders:
//     c - 7 (four bits: the constant of decode_i4s_to_i8s), c - 2 (two bits), 2 c - 1 (one bit);
//   * K is reduced over each 16-lane row with DPP row operations, all values of a batch of rows together (most levels
//     halve the number of values), and over the 16-lane rows of a weight row through LDS; integer sums, so the result
//     is exact whatever the order.
#include "dq_common.h"

namespace dq {

namespace {

constexpr int kMaxRowsPerWg = 128;

// The activations that go with one 16-byte chunk of weights (128 / BITS int8 = 2, 4 or 8 loads of 16 bytes),
// shuffled into the order in which (w >> BITS i) & mask yields the codes of each of the chunk's four words:
// out[j * (8 / BITS) + i] goes with dword i of word j.
template <int BITS>
__device__ __forceinline__ void load_activations(const int8_t* ap, bool valid, bool interleaved, uint32_t* out) {
  constexpr int kLoads = 8 / BITS;  // 16-byte loads per chunk
  uint4_t d[kLoads];
#pragma unroll
  for (int l = 0; l < kLoads; ++l) {
    d[l] = *reinterpret_cast<const uint4_t*>(ap + l * 16);
    if (!valid) d[l] = uint4_t{0u, 0u, 0u, 0u};
  }
  if constexpr (BITS == 4) {
    // a word holds 8 codes = half a load.  Plain: dword 0 / 1 of a word = its even / odd nibbles.  Interleaved
    // (interleave_weight(., 4, "int8"): element e at byte e % 4, nibble e / 4): low / high nibbles = elements
    // 0..3 / 4..7, the order the activations are in.
#pragma unroll
    for (int l = 0; l < kLoads; ++l) {
      const uint4_t t = interleaved ? d[l] : split_even_odd_bytes(d[l]);
#pragma unroll
      for (int i = 0; i < 4; ++i) out[l * 4 + i] = t[i];
    }
  } else if constexpr (BITS == 2) {
    // a word holds 16 codes = one load.  Plain: dword i = codes (i, 4 + i, 8 + i, 12 + i).  Interleaved
    // (interleave_weight(., 2, "int8")): natural order.
#pragma unroll
    for (int l = 0; l < kLoads; ++l) {
      const uint4_t t = interleaved ? d[l] : transpose4x4_bytes(d[l]);
#pragma unroll
      for (int i = 0; i < 4; ++i) out[l * 4 + i] = t[i];
    }
  } else {
    // a word holds 32 codes = two loads x0 = d[2 j], x1 = d[2 j + 1].  Plain: dword i = codes (i, 8 + i, 16 + i,
    // 24 + i): a 4 x 4 byte transpose of (x0[0], x0[2], x1[0], x1[2]) gives dwords 0..3, of (x0[1], x0[3], x1[1],
    // x1[3]) dwords 4..7.  Interleaved (interleave_weight(., 1, "int8"), made for the reference's 16-bit decoder:
    // bit i of byte b of a halfword is element 4 (i % 4) + 2 (i / 4) + b): dword i < 4 = elements (4 i, 4 i + 1,
    // 16 + 4 i, 17 + 4 i), dword 4 + i = elements (4 i + 2, 4 i + 3, 18 + 4 i, 19 + 4 i).
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint4_t x0 = d[2 * j], x1 = d[2 * j + 1];
      if (interleaved) {
        const uint32_t lo[4] = {x0[0], x0[1], x0[2], x0[3]}, hi[4] = {x1[0], x1[1], x1[2], x1[3]};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          out[j * 8 + i] = __builtin_amdgcn_perm(hi[i], lo[i], 0x05040100u);
          out[j * 8 + 4 + i] = __builtin_amdgcn_perm(hi[i], lo[i], 0x07060302u);
        }
      } else {
        const uint4_t e = transpose4x4_bytes(uint4_t{x0[0], x0[2], x1[0], x1[2]});
        const uint4_t o = transpose4x4_bytes(uint4_t{x0[1], x0[3], x1[1], x1[3]});
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          out[j * 8 + i] = e[i];
          out[j * 8 + 4 + i] = o[i];
        }
      }
    }
  }
}

template <int BITS, int MROWS, int NP, int R>
__global__ __launch_bounds__(256) void int_gemv_kernel(const int8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                        void* __restrict__ C, const float* __restrict__ s_a, float s_w,
                                                        int out_kind, int M, int N, int K, int tpr_shift, int nb,
                                                        uint32_t flip_mask, int mul, int zsub, int interleaved) {
  constexpr int kCodes = 128 / BITS;       // codes (and activations) per 16-byte chunk
  constexpr int kDwords = kCodes / 4;      // activation dwords per chunk
  constexpr int kPerWord = 8 / BITS;       // dwords a 32-bit word of weights decodes into
  constexpr uint32_t kMask = BITS == 4 ? 0x0F0F0F0Fu : (BITS == 2 ? 0x03030303u : 0x01010101u);
  constexpr int NV = R * MROWS;  // values reduced together per batch
  static_assert(NV <= 16 && (NV & (NV - 1)) == 0, "a power of two of at most 16 values per lane row");
  // partial sums: [batch][16-lane row of the workgroup (16)][value]
  __shared__ int red[kMaxRowsPerWg * 16 * MROWS];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int tpr = 1 << tpr_shift;
  const int rpp = 256 >> tpr_shift;
  const int slot = tid >> tpr_shift;
  const int ct = tid & (tpr - 1);
  const int c16 = K / kCodes;  // 16-byte chunks per row
  const int rows_per_batch = R * rpp;
  const int rows_per_wg = nb * rows_per_batch;
  const int row0 = blockIdx.x * rows_per_wg;
  const size_t row_bytes = (size_t)K * BITS / 8;

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

  // activations of this thread's chunk(s) in decoder order; their sum for the zero point
  uint32_t a[NP][MROWS][kDwords];
  int asum[NP][MROWS];
#pragma unroll
  for (int p = 0; p < NP; ++p) {
    const int chunk = p * tpr + ct;
    const bool valid = chunk < c16;  // a clamped chunk is read (in bounds) and zeroed
#pragma unroll
    for (int m = 0; m < MROWS; ++m) {
      const int8_t* ap = A + (size_t)min(m, M - 1) * K + (size_t)min(chunk, c16 - 1) * kCodes;
      load_activations<BITS>(ap, valid, interleaved != 0, a[p][m]);
      int s = 0;
#pragma unroll
      for (int i = 0; i < kDwords; ++i) s = __builtin_amdgcn_sdot4((int)a[p][m][i], 0x01010101, s, false);
      asum[p][m] = s;
    }
  }

  const bool writer = (lane & 15) < NV;
  int* red_w = red + (tid >> 4) * NV + (lane & (NV - 1));

  for (int b = 0; b < nb; ++b) {
    int acc[NV];
#pragma unroll
    for (int u = 0; u < R; ++u) {
      int dot[MROWS];
#pragma unroll
      for (int m = 0; m < MROWS; ++m) dot[m] = 0;
#pragma unroll
      for (int p = 0; p < NP; ++p) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t w = bq[u][p][j] ^ flip_mask;
#pragma unroll
          for (int i = 0; i < kPerWord; ++i) {
            const int d = (int)((w >> (BITS * i)) & kMask);
#pragma unroll
            for (int m = 0; m < MROWS; ++m) dot[m] = __builtin_amdgcn_sdot4((int)a[p][m][j * kPerWord + i], d, dot[m], false);
          }
        }
      }
#pragma unroll
      for (int m = 0; m < MROWS; ++m) {
        int zs = 0;
#pragma unroll
        for (int p = 0; p < NP; ++p) zs += asum[p][m];
        acc[u * MROWS + m] = mul * dot[m] - zsub * zs;
      }
    }
    // every row of the batch is consumed: refill all of them (wave-uniform branch)
    if (b + 1 < nb) {
#pragma unroll
      for (int u = 0; u < R; ++u) issue_row(u, b + 1);
    }
    // the batch's R x MROWS values are summed over each 16-lane row together; lane l then holds value l % NV
    const int v = RowReduce<NV, 0, int>::run(acc, lane);
    if (writer) red_w[b * 16 * NV] = v;
  }
  __syncthreads();

  // ---- sum of the 16-lane partials of each output (integers: exact whatever the order) ----------------
  const int parts = tpr >> 4;  // 16-lane rows per weight row
  for (int o = tid; o < rows_per_wg * MROWS; o += 256) {
    const int rl = o / MROWS, m = o - rl * MROWS;
    const int b = rl / rows_per_batch, within = rl - b * rows_per_batch;
    const int u = within >> (8 - tpr_shift), sl = within & (rpp - 1);
    const int* src = red + (b * 16 + sl * parts) * NV + u * MROWS + m;
    int v = src[0];
    for (int j = 1; j < parts; ++j) v += src[j * NV];
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

struct Decoder {
  uint32_t flip;
  int mul, zsub;
};

template <int BITS, int MROWS, int NP>
int launch_int_gemv(const void* A, const void* B, void* C, const void* s_a, float s_w, int out_kind, int M, int N, int K,
                    int tpr_shift, Decoder dec, int interleaved, hipStream_t stream) {
  constexpr int R = NP >= 4 ? 1 : 4 / NP;
  const int rpp = 256 >> tpr_shift;
  const long wgs1 = ((long)N + R * rpp - 1) / (R * rpp);
  // about two workgroups per CU, each walking several batches: at N = K = 8192 with two bits one batch per
  // workgroup (1024 workgroups) measured 7.4 us, two 6.3 us, four 6.2 us, eight 8.6 us
  int nb = (int)((wgs1 + 511) / 512);
  while (nb > 1 && nb * R * rpp > kMaxRowsPerWg) --nb;
  if (nb < 1) nb = 1;
  const int rows_per_wg = nb * R * rpp;
  hipLaunchKernelGGL((int_gemv_kernel<BITS, MROWS, NP, R>), dim3((N + rows_per_wg - 1) / rows_per_wg), dim3(256), 0,
                     stream, (const int8_t*)A, (const uint8_t*)B, C, (const float*)s_a, s_w, out_kind, M, N, K, tpr_shift,
                     nb, dec.flip, dec.mul, dec.zsub, interleaved);
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

// Returns 1 when the kernel does not cover the shape.  kMaxRegs bounds NP * MROWS * (activation dwords per chunk).
template <int BITS>
int int_gemv(const void* A, const void* B, void* C, int M, int N, int K, Decoder dec, int interleaved, const void* s_a,
             float s_w, int out_kind, hipStream_t stream) {
  constexpr int kCodes = 128 / BITS;
  if (M < 1 || M > 4 || K % kCodes != 0) return 1;
  const int c16 = K / kCodes;
  int tpr_shift = 5;
  while ((1 << tpr_shift) < c16 && tpr_shift < 8) ++tpr_shift;
  const int np = (c16 + (1 << tpr_shift) - 1) >> tpr_shift;
  const int mrows = M == 1 ? 1 : (M == 2 ? 2 : 4);
  // activation registers per thread: np * mrows * 32 / BITS dwords, kept to 64
  if (np > 2 || np * mrows * (32 / BITS) > 64) return 1;
#define DQ_GO(MR_, NP_) \
  return launch_int_gemv<BITS, MR_, NP_>(A, B, C, s_a, s_w, out_kind, M, N, K, tpr_shift, dec, interleaved, stream)
  if (mrows == 1 && np == 1) DQ_GO(1, 1);
  if (mrows == 1 && np == 2) DQ_GO(1, 2);
  if (mrows == 2 && np == 1) DQ_GO(2, 1);
  if constexpr (BITS >= 2) {
    if (mrows == 2 && np == 2) DQ_GO(2, 2);
    if (mrows == 4 && np == 1) DQ_GO(4, 1);
  }
  if constexpr (BITS == 4) {
    if (mrows == 4 && np == 2) DQ_GO(4, 2);
  }
#undef DQ_GO
  return 1;
}

// ---- two-bit weights in fragment order (prepack_i2_fragments) ------------------------------------------------
// B[(N + 31) / 32][K / 128][64 lanes][16 bytes]: lane 32 h + r of block (nb, kb) holds the 64 codes
// k = 128 kb + 64 h .. + 63 of row 32 nb + r.  In that order the pieces of one K chunk of 32 consecutive rows are
// contiguous, so here a wave instruction reads one block (1 KiB) and the rows run over the lanes: lane (h, r) adds up
// row r's products over the wave's K blocks.  Its activations change from block to block, so they live in LDS, staged
// once per workgroup in decoder order, and every read of them is a broadcast (the 32 lanes of a half share a chunk).
// A workgroup is 16 waves; wave w takes blocks kb = w, w + 16, ... of a row block, the 32 partial sums of a row (16
// waves x 2 halves) meet in LDS.  Integer sums: exact in any order.
constexpr int kFragWaves = 16;
constexpr int kFragActBytes = 32768;  // staged activations: MROWS * K bytes

template <int MROWS, int NP>
__global__ __launch_bounds__(64 * kFragWaves) void i2_gemv_frag_kernel(const int8_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                                       void* __restrict__ C, const float* __restrict__ s_a,
                                                                       float s_w, int out_kind, int M, int N, int K,
                                                                       uint32_t flip_mask, int mul, int zsub, int interleaved) {
  __shared__ __align__(16) int8_t act[kFragActBytes];
  __shared__ int red[kFragWaves * 64 * MROWS];
  __shared__ int asum[MROWS];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h = lane >> 5;
  const int KB = K >> 7;                 // blocks of 128 k per row
  const int row_blocks = (N + 31) >> 5;

  // ---- the first row block's weights go out before anything else ---------------------------------------------
  uint4_t wq[NP];
  auto issue = [&](int nb) {
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int kb = min(wave + kFragWaves * p, KB - 1);  // past the end: the last block again, unused
      wq[p] = __builtin_nontemporal_load(reinterpret_cast<const uint4_t*>(B + ((size_t)nb * KB + kb) * 1024 + lane * 16));
    }
  };
  int nb = blockIdx.x;
  if (nb < row_blocks) issue(nb);

  // ---- activations into LDS in decoder order, and their sums ---------------------------------------------------
  if (tid < MROWS) asum[tid] = 0;
  __syncthreads();
  const int pieces = K >> 4;  // 16-byte pieces per activation row
#pragma unroll
  for (int m = 0; m < MROWS; ++m) {
    const int8_t* ap = A + (size_t)min(m, M - 1) * K;
    int s = 0;
    for (int q = tid; q < pieces; q += 64 * kFragWaves) {
      uint4_t d = *reinterpret_cast<const uint4_t*>(ap + q * 16);
      if (!interleaved) d = transpose4x4_bytes(d);  // plain words decode to elements (i, 4 + i, 8 + i, 12 + i)
      *reinterpret_cast<uint4_t*>(act + m * K + q * 16) = d;
#pragma unroll
      for (int i = 0; i < 4; ++i) s = __builtin_amdgcn_sdot4((int)d[i], 0x01010101, s, false);
    }
    const int one[1] = {s};
    s = RowReduce<1, 0, int>::run(one, lane);
    if ((lane & 15) == 0 && s != 0) atomicAdd(&asum[m], s);
  }
  __syncthreads();

  for (; nb < row_blocks; nb += gridDim.x) {
    int acc[MROWS];
#pragma unroll
    for (int m = 0; m < MROWS; ++m) acc[m] = 0;
#pragma unroll
    for (int p = 0; p < NP; ++p) {
      const int kb = wave + kFragWaves * p;
      if (kb < KB) {  // wave-uniform
        const int8_t* chunk = act + (2 * kb + h) * 64;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t w = wq[p][j] ^ flip_mask;
          uint4_t a[MROWS];
#pragma unroll
          for (int m = 0; m < MROWS; ++m) a[m] = *reinterpret_cast<const uint4_t*>(chunk + m * K + j * 16);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int d = (int)((w >> (2 * i)) & 0x03030303u);
#pragma unroll
            for (int m = 0; m < MROWS; ++m) acc[m] = __builtin_amdgcn_sdot4((int)a[m][i], d, acc[m], false);
          }
        }
      }
    }
    // the next row block's weights travel while this one's sums meet
    const int nb_next = nb + gridDim.x;
    if (nb_next < row_blocks) issue(nb_next);
#pragma unroll
    for (int m = 0; m < MROWS; ++m) red[(wave * 64 + lane) * MROWS + m] = acc[m];
    __syncthreads();
    if (tid < 32 * MROWS) {
      const int r = tid / MROWS, m = tid - r * MROWS;
      int v = 0;
#pragma unroll
      for (int w = 0; w < kFragWaves; ++w) v += red[(w * 64 + r) * MROWS + m] + red[(w * 64 + 32 + r) * MROWS + m];
      v = mul * v - zsub * asum[m];
      const int row = nb * 32 + r;
      if (row < N && m < M) {
        if (out_kind == 0) {
          ((int32_t*)C)[(size_t)m * N + row] = v;
        } else {
          float f = (float)v;
          f = f / s_a[m];
          f = f / s_w;
          ((half_t*)C)[(size_t)m * N + row] = (half_t)f;
        }
      }
    }
    __syncthreads();  // the sums are read: the next round may overwrite them
  }
}

template <int MROWS, int NP>
int launch_i2_gemv_frag(const void* A, const void* B, void* C, const void* s_a, float s_w, int out_kind, int M, int N, int K,
                        Decoder dec, int interleaved, hipStream_t stream) {
  const int row_blocks = (N + 31) / 32;
  const int grid = row_blocks < 512 ? row_blocks : 512;
  hipLaunchKernelGGL((i2_gemv_frag_kernel<MROWS, NP>), dim3(grid), dim3(64 * kFragWaves), 0, stream, (const int8_t*)A,
                     (const uint8_t*)B, C, (const float*)s_a, s_w, out_kind, M, N, K, dec.flip, dec.mul, dec.zsub, interleaved);
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

}  // namespace

// Each returns 1 when the streaming kernel does not cover the shape (the caller then uses the MFMA GEMM): M <= 4,
// K a multiple of the codes in 16 bytes and at most 512 chunks of 16 bytes per row (less where the activations of
// more rows would not fit the registers).

int i2_gemv(const void* A, const void* B, void* C, int M, int N, int K, int convention, int layout, const void* s_a,
            float s_w, int out_kind, hipStream_t stream) {
  Decoder dec{0u, 1, 0};
  if (convention == I2_OFFSET) dec = Decoder{0u, 1, 2};
  else if (convention == I2_TWOS) dec = Decoder{0xAAAAAAAAu, 1, 2};  // sext2(c) = (c ^ 2) - 2
  const int interleaved = (layout & ~LAYOUT_FRAGMENTS) == LAYOUT_INTERLEAVED;
  if (layout & LAYOUT_FRAGMENTS) {
    // the activations of the batch stay in LDS; a wave walks up to eight blocks of 128 k
    if (M < 1 || M > 4 || K % 128 != 0) return 1;
    const int mrows = M == 1 ? 1 : (M == 2 ? 2 : 4);
    const int np = ((K >> 7) + kFragWaves - 1) / kFragWaves;
    if ((size_t)mrows * K > (size_t)kFragActBytes || np > 8) return 1;
    if ((size_t)((N + 31) / 32) * (size_t)(K >> 7) * 1024 >= (1ull << 40)) return 1;
#define DQ_GO(MR_, NP_) return launch_i2_gemv_frag<MR_, NP_>(A, B, C, s_a, s_w, out_kind, M, N, K, dec, interleaved, stream)
#define DQ_NP(MR_)              \
  do {                          \
    if (np <= 1) DQ_GO(MR_, 1); \
    if (np <= 2) DQ_GO(MR_, 2); \
    if (np <= 4) DQ_GO(MR_, 4); \
    DQ_GO(MR_, 8);              \
  } while (0)
    if (mrows == 1) DQ_NP(1);
    if (mrows == 2) DQ_NP(2);
    DQ_NP(4);
#undef DQ_NP
#undef DQ_GO
  }
  return int_gemv<2>(A, B, C, M, N, K, dec, interleaved, s_a, s_w, out_kind, stream);
}

// decode: the values of call_gemm_int8xint4 (0 unsigned nibbles, 1 two's complement, 2 / 3 the words of
// interleave_weight(., 4, "int8") as decode_i4u_to_i8s / decode_i4s_to_i8s read them: w = q / w = q - 7).
int i4_gemv(const void* A, const void* B, void* C, int M, int N, int K, int decode, hipStream_t stream) {
  Decoder dec{0u, 1, 0};
  if (decode == 1) dec = Decoder{0x88888888u, 1, 8};  // sext4(q) = (q ^ 8) - 8
  else if (decode == 3) dec = Decoder{0u, 1, 7};
  else if (decode != 0 && decode != 2) return 1;
  return int_gemv<4>(A, B, C, M, N, K, dec, decode >= 2, nullptr, 1.f, 0, stream);
}

// convention: I2Convention read for one bit: unsigned w = c; offset w = 2 c - 1 (decode_i1s_to_i8s); two's
// complement w = -c (the sign extension of a one-bit field).
int i1_gemv(const void* A, const void* B, void* C, int M, int N, int K, int convention, int layout, hipStream_t stream) {
  Decoder dec{0u, 1, 0};
  if (convention == I2_OFFSET) dec = Decoder{0u, 2, 1};
  else if (convention == I2_TWOS) dec = Decoder{0u, -1, 0};
  return int_gemv<1>(A, B, C, M, N, K, dec, layout == LAYOUT_INTERLEAVED, nullptr, 1.f, 0, stream);
}

}  // namespace dq
