// W4A16 batch kernel for 17..64 activation rows on gfx950: one workgroup per CU, K sliced over its four waves.
//
// Replaces the batched use of the kernel generated from
// examples/dequantize_gemm/example_dequant_gemv_fp16xint4.py:83-153 (group scales / zeros as in
// examples/dequantize_gemm/quantize/lop3.py:41-81,136-176) for batches that are too large to keep the activations
// in registers and too small for a tiled GEMM to fill 256 CUs.
//
// With N = 28672 a CU owns 112 weight rows, seven blocks of 16.  What limits such a tile is how often an activation
// fragment is re-read per matrix instruction, so all RB row blocks of the workgroup go to every wave and the four
// waves (one per SIMD, 512 registers each) split K instead: wave w owns k in [w K/4, (w+1) K/4) and walks it in
// slabs of 256 k.  Per 32-k step a wave reads MB activation fragments once and multiplies them with RB weight
// fragments (RB x MB matrix instructions); the partial sums of the four waves meet once, through LDS, at the end.
//
//   * Weights are fetched row-contiguously, one slab (128 bytes) of 8 rows per instruction, a whole slab ahead, and
//     are transposed into the matrix instruction's layout through an LDS area of the wave's own (16-byte writes as
//     loaded, 4-byte reads as multiplied, pieces XOR-swizzled so that neither side has bank conflicts).  LDS
//     operations of one wave execute in order and no other wave touches the area, so the main loop has no barrier.
//   * Activations are fetched straight into the matrix instruction's layout (an instruction reads 16 rows x 64
//     contiguous bytes, from the L2 after the first workgroup touched them), into a ring of eight 32-k steps: the
//     registers of step kb are refilled for the next slab as soon as step kb has been multiplied.
//   * Loads return in order, so both streams are issued the same distance (one slab, 1/32 of the kernel) ahead of
//     their use; every load is a buffer load issued unconditionally (past the end: an out-of-range offset, which
//     returns zeros and moves nothing), so the loop body is straight-line code and the waits count exactly.
//   * A weight keeps the reference's rounding: RNE16(RNE16(q - z) s) etc., formed per packed dword with 5 bit
//     operations (fp16 1024 + q or 64 + q by masking) and two packed fp16 operations per pair.  (q - z) comes out of
//     ONE exact subtraction of bias + z when z is a non-negative integer (then bias + z and the difference are
//     exact); a workgroup whose zeros are not all of that kind runs a copy of the loop with the two subtractions.
//   * Group scales and zeros of the workgroup's rows are staged in LDS once, before the loop.
#include <type_traits>
#include <utility>

#include "dq_common.h"

namespace dq {

namespace {

constexpr uint32_t kBufferFlags = 0x00020000u;  // raw buffer of 32-bit data, the range check on
constexpr uint32_t kOutOfRange = 0xFFFFF000u;   // an offset no operand of this kernel reaches

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop whose index is a constant expression
template <int... I, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

constexpr int kSzRow = 208;  // LDS bytes per row of scales (K / 64 <= 192 of them used): 52 dwords spread 16 rows over all banks

// Packed constants of one row's group for the decoder: s2 = (s, s); nb_lo / nb_hi = -(1024 + z'), -(64 + z') twice,
// z' the part of the zero point that folds into the bias; nz2 = (-z, -z) where it does not.
struct RowGroup {
  uint32_t s2, nb_lo, nb_hi, nz2;
};

// Eight nibbles -> eight fp16 weights, element pair i = (n_i, n_{i+4}).  FOLD: the zero point is inside nb_lo/nb_hi.
template <int MODE, bool FOLD>
__device__ __forceinline__ half8_t decode_row_scaled(uint32_t w, const RowGroup& c) {
  if constexpr (MODE == W4_SIGNED) w ^= 0x88888888u;  // sext4(q) = (q ^ 8) - 8
  uint32_t t[4];
  u4x8_to_biased_half(w, t);
  uint4_t o;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    half2_t q = as_half2(t[i]) + as_half2((i & 1) ? c.nb_hi : c.nb_lo);  // exact
    if constexpr (MODE == W4_SCALE || MODE == W4_USCALE) {
      q = q * as_half2(c.s2);
    } else if constexpr (MODE == W4_ZEROS_ORIGINAL) {
      if constexpr (!FOLD) q = q + as_half2(c.nz2);
      q = q * as_half2(c.s2);
    } else if constexpr (MODE == W4_ZEROS_RESCALE) {
      q = __builtin_elementwise_fma(q, as_half2(c.s2), as_half2(c.nz2));
    }
    o[i] = as_u32(q);
  }
  return __builtin_bit_cast(half8_t, o);
}

template <int MB, int RB, int MODE, bool APERM>
__global__ __launch_bounds__(256) void w4a16_kslice_kernel(const half_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                           const half_t* __restrict__ S, const half_t* __restrict__ Z,
                                                           half_t* __restrict__ C, int M, int N, int K) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr bool kScale = MODE >= W4_SCALE;
  constexpr bool kZeros = MODE >= W4_ZEROS_ORIGINAL;
  constexpr int kSlabBytes = RB * 2048;        // one slab of the wave's weights: RB blocks x 16 rows x 128 bytes
  constexpr int kWaveStage = 2 * kSlabBytes;   // the slab being multiplied and the one being written
  constexpr int kStageBytes = 4 * kWaveStage;
  static_assert(RB * MB * 1024 <= kWaveStage, "a wave's partial sums fit its own staging area");

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = lane >> 4;
  const int r = lane & 15;
  const int nrb = N >> 4;
  const int rb0 = blockIdx.x * RB;
  const int nrb_wg = min(RB, nrb - rb0);
  const uint32_t row_bytes = (uint32_t)(K >> 1);
  const int kslice = K >> 2;       // k of one wave
  const int nslab = kslice >> 8;
  unsigned char* const wst = smem + wave * kWaveStage;
  unsigned char* const s_lds = smem + kStageBytes;
  unsigned char* const z_lds = s_lds + RB * 16 * kSzRow;

  const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)B, 0, (uint32_t)N * row_bytes, kBufferFlags);
  const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)A, 0, (uint32_t)M * (uint32_t)K * 2u, kBufferFlags);

  // ---- weights: raw loads and the transposing LDS area ---------------------------------------------------------
  // instruction i of a block: lane l fetches piece l % 8 (16 bytes, 32 k) of row 8 i + l / 8
  uint4_t raw[RB][2];
  const uint32_t w_voff = (uint32_t)(lane >> 3) * row_bytes + (uint32_t)(lane & 7) * 16u;
  const uint32_t w_sbase = (uint32_t)rb0 * 16u * row_bytes + (uint32_t)wave * (uint32_t)(kslice >> 1);
  auto load_raw = [&](auto rb_tag, int slab) {
    constexpr int rb = decltype(rb_tag)::value;
    const uint32_t vo = (slab < nslab && rb < nrb_wg) ? w_voff : kOutOfRange;
#pragma unroll
    for (int i = 0; i < 2; ++i)
      raw[rb][i] = __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, vo, w_sbase + (uint32_t)(rb * 16 + i * 8) * row_bytes + (uint32_t)slab * 128u, 2 /* nt */);
  };
  // piece p of row n sits at position p ^ ((n >> 1) & 7) of the row's eight
  uint32_t w_wr[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int row = i * 8 + (lane >> 3), piece = lane & 7;
    w_wr[i] = (uint32_t)(row * 8 + (piece ^ ((row >> 1) & 7))) * 16u;
  }
  auto park_raw = [&](auto rb_tag, int buf) {  // registers -> LDS, in the layout they were loaded in
    constexpr int rb = decltype(rb_tag)::value;
#pragma unroll
    for (int i = 0; i < 2; ++i) *reinterpret_cast<uint4_t*>(wst + buf * kSlabBytes + rb * 2048 + w_wr[i]) = raw[rb][i];
  };
  // Steps come in pairs that share 64 k, i.e. one 128-byte line of every activation row: lane (g, r) owns
  // k = 64 (kb / 2) + 16 g + 8 (kb % 2) .. + 7 in step kb, so that the two activation loads of a pair, issued back
  // to back, use the whole line while it is in the L1 (steps of 32 consecutive k use half a line each, a step apart,
  // and with 64 rows the line is gone by then: every line would come from the L2 twice).
  // The dword of step kb for lane (g, r):
  uint32_t w_rd[8];
#pragma unroll
  for (int kb = 0; kb < 8; ++kb)
    w_rd[kb] = (uint32_t)r * 128u + (uint32_t)((((kb >> 1) * 2 + (g >> 1)) ^ ((r >> 1) & 7)) << 4) + (uint32_t)((g & 1) * 8 + (kb & 1) * 4);

  // ---- activations: ring of eight steps, in the matrix instruction's layout --------------------------------------
  // NY steps deep: four when MB = 4 (the ring, the weights in flight and 112 accumulators must leave the decoder
  // room in 512 registers), else eight
  constexpr int NY = MB == 4 ? 4 : 8;
  uint4_t y[NY][MB];
  uint32_t a_voff[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int m = mb * 16 + r;
    a_voff[mb] = m < M ? ((uint32_t)m * (uint32_t)K + (uint32_t)g * 16u) * 2u : kOutOfRange;
  }
  const uint32_t a_sbase = (uint32_t)wave * (uint32_t)kslice * 2u;
  auto load_y = [&](int kb, int slab, const uint32_t (&vo)[MB]) {  // step kb of the slab, into its place in the ring
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
      y[kb % NY][mb] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, vo[mb], a_sbase + (uint32_t)slab * 512u + (uint32_t)((kb >> 1) * 128 + (kb & 1) * 16), 0);
  };

  // ---- prologue: slab 0 of the weights, the scales, slab 0 of the activations ------------------------------------
  static_for<RB>([&](auto rb) { load_raw(rb, 0); });

  bool fold = true;  // every zero point of the workgroup's rows is an integer in [0, 1024]
  if constexpr (kScale) {
    const uint32_t ppr = (uint32_t)K >> 10;  // 16-byte pieces per row of scales
    const uint32_t pieces = (uint32_t)RB * 16u * ppr;
    const uint32_t sz_bytes = (uint32_t)N * (uint32_t)(K >> 6);
    const __amdgpu_buffer_rsrc_t s_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)S, 0, sz_bytes, kBufferFlags);
    const __amdgpu_buffer_rsrc_t z_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)Z, 0, kZeros ? sz_bytes : 0u, kBufferFlags);
    for (uint32_t p = (uint32_t)tid; p < pieces; p += 256u) {
      const uint32_t row = p / ppr, piece = p - row * ppr;
      const uint32_t src = ((uint32_t)rb0 * 16u + row) * (uint32_t)(K >> 6) + piece * 16u;
      const uint32_t dst = row * kSzRow + piece * 16u;
      *reinterpret_cast<uint4_t*>(s_lds + dst) = __builtin_amdgcn_raw_buffer_load_b128(s_rsrc, src, 0, 0);
      if constexpr (kZeros) {
        const uint4_t zz = __builtin_amdgcn_raw_buffer_load_b128(z_rsrc, src, 0, 0);
        *reinterpret_cast<uint4_t*>(z_lds + dst) = zz;
        if constexpr (MODE == W4_ZEROS_ORIGINAL) {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const half2_t h = as_half2(zz[e]);
#pragma unroll
            for (int j = 0; j < 2; ++j) {
              const float v = (float)h[j];
              fold = fold && v >= 0.f && v <= 1024.f && v == __builtin_truncf(v);
            }
          }
        }
      }
    }
  }
  {
    uint32_t vo[MB];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) vo[mb] = a_voff[mb];
#pragma unroll
    for (int kb = 0; kb < NY; ++kb) load_y(kb, 0, vo);
  }
  static_for<RB>([&](auto rb) { park_raw(rb, 0); });
  static_for<RB>([&](auto rb) { load_raw(rb, 1); });
  if constexpr (MODE == W4_ZEROS_ORIGINAL) fold = __syncthreads_and(fold);
  else __syncthreads();

  float4_t acc[RB][MB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[rb][mb] = float4_t{0.f, 0.f, 0.f, 0.f};

  // ---- main loop -------------------------------------------------------------------------------------------
  auto run = [&](auto fold_tag) {
    constexpr bool kFold = decltype(fold_tag)::value;
    const uint32_t sz_rd = (uint32_t)r * kSzRow + (uint32_t)wave * (uint32_t)(kslice >> 6);  // + 4 slab: the slab's two groups
    uint32_t wd[2][RB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) wd[0][rb] = *reinterpret_cast<const uint32_t*>(wst + rb * 2048 + w_rd[0]);
    for (int slab = 0; slab < nslab; ++slab) {
      const int cur = slab & 1;
      const unsigned char* const w_cur = wst + cur * kSlabBytes;
      const unsigned char* const w_nxt = wst + (cur ^ 1) * kSlabBytes;
      uint32_t a_vo[MB];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) a_vo[mb] = slab + 1 < nslab ? a_voff[mb] : kOutOfRange;
      RowGroup rg[RB];
      static_for<8>([&](auto kb_tag) {
        constexpr int kb = decltype(kb_tag)::value;
        if constexpr ((kb & 3) == 0) {
          // the decoder's constants of this 128-k group
          const uint32_t sel = kb == 0 ? 0x01000100u : 0x03020302u;  // (lo, lo) / (hi, hi) of the slab's two values
          uint32_t s_raw[RB], z_raw[RB];
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) {
            s_raw[rb] = kScale ? *reinterpret_cast<const uint32_t*>(s_lds + rb * 16 * kSzRow + sz_rd + slab * 4) : 0u;
            z_raw[rb] = kZeros ? *reinterpret_cast<const uint32_t*>(z_lds + rb * 16 * kSzRow + sz_rd + slab * 4) : 0u;
          }
          const half2_t n1024 = {(half_t)-1024.f, (half_t)-1024.f}, n64 = {(half_t)-64.f, (half_t)-64.f};
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) {
            rg[rb].s2 = __builtin_amdgcn_perm(s_raw[rb], s_raw[rb], sel);
            half2_t zf = {(half_t)0.f, (half_t)0.f};  // folded into the bias
            rg[rb].nz2 = 0u;
            if constexpr (MODE == W4_SCALE || MODE == W4_OFFSET8 || MODE == W4_SIGNED) {
              zf = half2_t{(half_t)8.f, (half_t)8.f};
            } else if constexpr (kZeros) {
              const half2_t z2 = as_half2(__builtin_amdgcn_perm(z_raw[rb], z_raw[rb], sel));
              if constexpr (MODE == W4_ZEROS_ORIGINAL && kFold) zf = z2;
              else rg[rb].nz2 = as_u32(-z2);
            }
            rg[rb].nb_lo = as_u32(n1024 - zf);
            rg[rb].nb_hi = as_u32(n64 - zf);
          }
        }
        // next step's weight dwords (the next slab's first step reads the other area, complete since step 6)
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
          wd[(kb + 1) & 1][rb] = *reinterpret_cast<const uint32_t*>((kb < 7 ? w_cur : w_nxt) + rb * 2048 + w_rd[(kb + 1) & 7]);
        uint4_t ya[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) ya[mb] = APERM ? permute_k8_16bit(y[kb % NY][mb]) : y[kb % NY][mb];
        // one wave per SIMD: the decoder of block rb + 1 is issued between the matrix instructions of block rb
        half8_t xw[2];
        xw[0] = decode_row_scaled<MODE, kFold>(wd[kb & 1][0], rg[0]);
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) {
          if (rb + 1 < RB) xw[(rb + 1) & 1] = decode_row_scaled<MODE, kFold>(wd[kb & 1][rb + 1], rg[rb + 1]);
#pragma unroll
          for (int mb = 0; mb < MB; ++mb)
            acc[rb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xw[rb & 1], __builtin_bit_cast(half8_t, ya[mb]), acc[rb][mb], 0, 0, 0);
        }
        if constexpr (kb & 1) {  // the pair NY steps on: both halves of its lines, back to back
          if constexpr (kb + NY < 8) {
            load_y(kb - 1 + NY, slab, a_voff);
            load_y(kb + NY, slab, a_voff);
          } else {
            load_y(kb - 1 + NY - 8, slab + 1, a_vo);
            load_y(kb + NY - 8, slab + 1, a_vo);
          }
        }
        if constexpr (kb < RB) {  // block kb of the slab after next takes the registers of block kb of the next one
          park_raw(kb_tag, cur ^ 1);
          load_raw(kb_tag, slab + 2);
        }
      });
    }
  };
  if constexpr (MODE == W4_ZEROS_ORIGINAL) {
    if (fold) run(std::true_type{});
    else run(std::false_type{});
  } else {
    run(std::true_type{});
  }

  // ---- the four partial sums meet: every wave parks its own in its staging area -----------------------------------
  float4_t* const red = reinterpret_cast<float4_t*>(smem);
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) red[wave * (kWaveStage / 16) + (rb * MB + mb) * 64 + lane] = acc[rb][mb];
  __syncthreads();
  // acc[rb][mb][i] = C[mb * 16 + r][(rb0 + rb) * 16 + 4 g + i]
  for (int p = wave; p < RB * MB; p += 4) {
    float4_t v = red[p * 64 + lane];
#pragma unroll
    for (int w = 1; w < 4; ++w) {
      const float4_t o = red[w * (kWaveStage / 16) + p * 64 + lane];
      v = float4_t{v[0] + o[0], v[1] + o[1], v[2] + o[2], v[3] + o[3]};
    }
    const int rb = p / MB, mb = p - rb * MB;
    const int m = mb * 16 + r;
    if (m < M && rb < nrb_wg) {
      const half4_t o = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
      *reinterpret_cast<half4_t*>(C + (size_t)m * N + (size_t)(rb0 + rb) * 16 + g * 4) = o;
    }
  }
}

template <int MB, int RB>
int launch_kslice(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int mode,
                  int layout, hipStream_t stream) {
  constexpr int kLds = 4 * 2 * RB * 2048 + 2 * RB * 16 * kSzRow;
  static_assert(kLds <= 160 * 1024, "LDS budget");
  const int nrb = N / 16;
  const dim3 grid((nrb + RB - 1) / RB), block(256);
#define DQ_LAUNCH2(MODE_, APERM_)                                                                                 \
  do {                                                                                                            \
    auto kern = w4a16_kslice_kernel<MB, RB, MODE_, APERM_>;                                                       \
    static bool lds_limit_raised[kMaxDevices];                                                                    \
    if (raise_lds_limit<kLds>(kern, lds_limit_raised)) return -1;                                                 \
    hipLaunchKernelGGL(kern, grid, block, kLds, stream, (const half_t*)A, (const uint8_t*)B, (const half_t*)S,    \
                       (const half_t*)Z, (half_t*)C, M, N, K);                                                    \
  } while (0)
#define DQ_LAUNCH_MODE(MODE_)                             \
  do {                                                    \
    if (layout == LAYOUT_PLAIN) DQ_LAUNCH2(MODE_, true);  \
    else DQ_LAUNCH2(MODE_, false);                        \
  } while (0)
  switch (mode) {
    case W4_SCALE: DQ_LAUNCH_MODE(W4_SCALE); break;
    case W4_USCALE: DQ_LAUNCH_MODE(W4_USCALE); break;
    case W4_ZEROS_ORIGINAL: DQ_LAUNCH_MODE(W4_ZEROS_ORIGINAL); break;
    case W4_ZEROS_RESCALE: DQ_LAUNCH_MODE(W4_ZEROS_RESCALE); break;
    default: return 1;
  }
#undef DQ_LAUNCH_MODE
#undef DQ_LAUNCH2
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

}  // namespace

// Returns 1 when the shape is not covered (the caller falls back to a kernel without these restrictions): needs
// M <= 64, N a multiple of 16 with enough row blocks for every CU, K a multiple of 1024 (whole 256-k slabs per wave)
// up to 12288 (the workgroup's scales fit the LDS), group 128, a mode with scales, and operands below 4 GiB.
int w4a16_kslice(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int group,
                 int mode, int layout, hipStream_t stream) {
  if (M < 1 || M > 64 || N < 16 || N % 16 != 0) return 1;
  if (K % 1024 != 0 || K > 12288 || K < 2048) return 1;  // at least two slabs per wave
  if (mode < W4_SCALE || group != 128) return 1;
  if ((size_t)N * K / 2 >= (1ull << 32) - 8192) return 1;  // 32-bit offsets, and room for the out-of-range marker
  const int nrb = N / 16;
  if (nrb < 7 * 200) return 1;  // fewer than 200 workgroups of seven row blocks
  const int mb = (M + 15) / 16;
  switch (mb) {
    case 1: return 1;
    case 2: return launch_kslice<2, 7>(A, B, S, Z, C, M, N, K, mode, layout, stream);
    case 3: return launch_kslice<3, 7>(A, B, S, Z, C, M, N, K, mode, layout, stream);
    default: return launch_kslice<4, 7>(A, B, S, Z, C, M, N, K, mode, layout, stream);
  }
}

}  // namespace dq
