// W4A16 batch kernel for 17..64 activation rows on gfx950: one workgroup of eight waves per CU, K sliced over them.
//
// Replaces the batched use of the kernel generated from
// examples/dequantize_gemm/example_dequant_gemv_fp16xint4.py:83-153 (group scales / zeros as in
// examples/dequantize_gemm/quantize/lop3.py:41-81,136-176) for batches that are too large to keep the activations
// in registers and too small for a tiled GEMM to fill 256 CUs.
//
// With N = 28672 a CU owns 112 weight rows, seven blocks of 16.  A tile that flat re-reads every activation fragment
// once per block of rows, so the rows stay together and K is what the waves share out: wave (ks, rgp) owns the K
// quarter ks and the row blocks 4 rgp .. (four for rgp = 0, three for rgp = 1), and walks its quarter in slabs of
// 256 k, each four pairs of 32-k steps.  The two waves of a K quarter sit on one SIMD and share the quarter's
// activations; the eight partial sums meet once, through LDS, at the end.
//
//   * Weights are fetched row-contiguously, one slab (128 bytes) of 8 rows per instruction, a whole slab ahead, and
//     are transposed into the matrix instruction's layout through an LDS area of the wave's own (16-byte writes as
//     loaded, 4-byte reads as multiplied, pieces XOR-swizzled so that neither side has bank conflicts).  LDS
//     operations of one wave execute in order and no other wave touches that area.
//   * Activations are fetched row-contiguously too, a pair of steps (64 k, one 128-byte line per row) at a time, each
//     of the quarter's two waves half of the rows, and go through a double-buffered LDS area of the quarter; one
//     workgroup barrier per pair publishes them.  (Fetched in the matrix instruction's own layout, sixteen different
//     rows land in adjacent lanes and the load unit handles a cache line per four lanes: with 64 rows that alone
//     took as long as the weight stream.)
//   * Loads return in order, so both streams are issued well ahead of their use; every load is a buffer load issued
//     unconditionally (past the end: an out-of-range offset, which returns zeros and moves nothing), so the loop
//     body is straight-line code and the waits count exactly.
//   * A weight keeps the reference's rounding: RNE16(RNE16(q - z) s) etc., formed per packed dword with 5 bit
//     operations (fp16 1024 + q or 64 + q by masking) and two packed fp16 operations per pair.  (q - z) comes out of
//     ONE exact subtraction of bias + z when z is a non-negative integer (then bias + z and the difference are
//     exact); a workgroup whose zeros are not all of that kind runs a copy of the loop with the two subtractions.
//   * Group scales and zeros of the workgroup's rows are staged in LDS once, before the loop.
//
// Where the time goes (M = 64, N = 28672, K = 8192, 51 us; with every load redirected to lines that stay in the
// cache it is 42 us, so memory is not what binds): per 32-k step a SIMD issues about 130 VALU instructions (91 of them
// the decoder: 13 per packed dword, of which a dword feeds only M / 16 = 4 matrix instructions), 28 matrix
// instructions and some 40 LDS / memory / scalar ones.  Measured on this chip a VALU instruction costs 2.1 ns of a
// SIMD's issue time and a 16x16x32 matrix instruction 3.3 ns on top of whatever VALU work it overlaps (at most
// 1.5 VALU instructions each), which puts the floor of this instruction mix near 27 us; the LDS moves 62 KB per step
// and CU on top.  Against the streaming kernel (dq_stream.hip) this one is 11-18 % faster at M = 32 and 48 and equal
// at M = 64.
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

constexpr int kRB = 7;           // row blocks of 16 weight rows per workgroup: four for waves 0..3, three for waves 4..7
constexpr int kAStage = 8192;    // one pair of steps of activations: up to 64 rows x 128 bytes
constexpr int kWStage = 8192;    // a wave's slab of weights: up to 4 blocks x 16 rows x 128 bytes
constexpr int kStages = 4 * 2 * kAStage + 8 * kWStage;

// One wave's share of the workgroup's tile: K quarter ks = wave % 4, row blocks 4 rgp .. 4 rgp + RBW - 1 with
// rgp = wave / 4.  Leaves its partial sums in LDS.
template <int MB, int NP, int MODE, bool APERM, int RBW, bool FOLD>
__device__ __forceinline__ void kslice_wave(const half_t* __restrict__ A, const uint8_t* __restrict__ B, int M, int N, int K) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr bool kScale = MODE >= W4_SCALE;
  constexpr bool kZeros = MODE >= W4_ZEROS_ORIGINAL;
  static_assert(NP == 1 || NP == 2 || NP == 4, "pairs in flight divide the four pairs of a slab");

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int ks = wave & 3;
  const int rgp = wave >> 2;
  const int rbw0 = rgp * 4;
  const int g = lane >> 4;
  const int r = lane & 15;
  const int nrb = N >> 4;
  const int rb0 = blockIdx.x * kRB;
  const int nrb_wg = min(kRB, nrb - rb0);
  const uint32_t row_bytes = (uint32_t)(K >> 1);
  const int kslice = K >> 2;
  const int nslab = kslice >> 8;
  const int npair = nslab * 4;
  const uint32_t szrow = (uint32_t)(K >> 6) + 8u;
  unsigned char* const ast = smem + ks * (2 * kAStage);
  unsigned char* const wst = smem + 4 * 2 * kAStage + wave * kWStage;
  const unsigned char* const s_lds = smem + kStages;
  const unsigned char* const z_lds = s_lds + kRB * 16 * szrow;

  const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)B, 0, (uint32_t)N * row_bytes, kBufferFlags);
  const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)A, 0, (uint32_t)M * (uint32_t)K * 2u, kBufferFlags);

  // In the activation and weight areas 16-byte piece p of row n sits at position p ^ ((n >> 1) & 7) of the row's
  // eight: sixteen lanes that write two whole rows, or read one piece of sixteen rows, then cover all banks.
  // Row-contiguous instruction i covers rows 8 i .. 8 i + 7: lane l has piece l % 8 of row 8 i + l / 8, whose swizzle
  // is (4 i + l / 16) & 7, so even and odd i differ by 4.
  uint32_t rc_wr[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) rc_wr[i] = (uint32_t)((lane >> 3) * 8 + ((lane & 7) ^ ((4 * i + (lane >> 4)) & 7))) * 16u;

  // ---- activations: the two waves of a K quarter fetch alternate instructions of a pair ---------------------------
  // A load in the matrix instruction's own layout puts sixteen different rows into adjacent lanes, which the texture
  // addresser handles a cache line per lane group of four; row-contiguous it is 64 bytes per group.  Instruction
  // i = 2 ii + rgp of a pair: rows 8 i .. 8 i + 7, 128 bytes (64 k) each.
  uint4_t y_raw[NP][MB];
  uint32_t a_voff[MB];
#pragma unroll
  for (int ii = 0; ii < MB; ++ii) {
    const int m = (2 * ii + rgp) * 8 + (lane >> 3);
    a_voff[ii] = m < M ? (uint32_t)m * (uint32_t)K * 2u + (uint32_t)(lane & 7) * 16u : kOutOfRange;
  }
  const uint32_t a_sbase = (uint32_t)ks * (uint32_t)kslice * 2u;
  auto load_pair = [&](int q, int pair) {  // past the last pair: that pair again (L2 hits, results unused)
    const uint32_t so = a_sbase + (uint32_t)min(pair, npair - 1) * 128u;
#pragma unroll
    for (int ii = 0; ii < MB; ++ii) y_raw[q][ii] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, a_voff[ii], so, 0);
  };
  const uint32_t a_wr = (uint32_t)rgp * 1024u + (rgp ? rc_wr[1] : rc_wr[0]);
  auto park_pair = [&](int q, int buf) {  // a piece is the eight values of one fragment: permuted here, once
#pragma unroll
    for (int ii = 0; ii < MB; ++ii)
      *reinterpret_cast<uint4_t*>(ast + buf * kAStage + ii * 2048 + a_wr) = APERM ? permute_k8_16bit(y_raw[q][ii]) : y_raw[q][ii];
  };
  // Steps come in pairs that share 64 k, one 128-byte line of every activation row: in step j of a pair lane (g, r)
  // owns k = 16 g + 8 j .. + 7 of the pair, i.e. piece 2 g + j of activation row 16 mb + r
  uint32_t a_rd[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) a_rd[j] = (uint32_t)r * 128u + (uint32_t)(((2 * g + j) ^ ((r >> 1) & 7)) << 4);
  // ... and dword 2 (g % 2) + j of piece 2 p + g / 2 of weight row r in pair p of a slab
  uint32_t w_rd[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) w_rd[p] = (uint32_t)r * 128u + (uint32_t)(((p * 2 + (g >> 1)) ^ ((r >> 1) & 7)) << 4) + (uint32_t)((g & 1) * 8);

  // ---- weights: row-contiguous loads a slab ahead; instruction i of a block: lane l has piece l % 8 of row 8 i + l / 8
  uint4_t raw[RBW][2];
  const uint32_t w_voff = (uint32_t)(lane >> 3) * row_bytes + (uint32_t)(lane & 7) * 16u;
  const uint32_t w_sbase = (uint32_t)(rb0 + rbw0) * 16u * row_bytes + (uint32_t)ks * (uint32_t)(kslice >> 1);
  auto load_raw = [&](auto rb_tag, int slab) {
    constexpr int rb = decltype(rb_tag)::value;
    const uint32_t vo = (slab < nslab && rbw0 + rb < nrb_wg) ? w_voff : kOutOfRange;
#pragma unroll
    for (int i = 0; i < 2; ++i)
      raw[rb][i] = __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, vo, w_sbase + (uint32_t)(rb * 16 + i * 8) * row_bytes + (uint32_t)slab * 128u, 2 /* nt */);
  };
  auto park_raw = [&](auto rb_tag) {
    constexpr int rb = decltype(rb_tag)::value;
#pragma unroll
    for (int i = 0; i < 2; ++i) *reinterpret_cast<uint4_t*>(wst + rb * 2048 + i * 1024 + rc_wr[i]) = raw[rb][i];
  };

  // ---- prologue: slab 0 of the weights and the first pairs of activations ------------------------------------------
  static_for<RBW>([&](auto rb) { load_raw(rb, 0); });
#pragma unroll
  for (int q = 0; q < NP; ++q) load_pair(q, q);
  static_for<RBW>([&](auto rb) { park_raw(rb); });
  static_for<RBW>([&](auto rb) { load_raw(rb, 1); });
  park_pair(0, 0);
  load_pair(0, NP);
  __syncthreads();

  float4_t acc[RBW][MB];
#pragma unroll
  for (int rb = 0; rb < RBW; ++rb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[rb][mb] = float4_t{0.f, 0.f, 0.f, 0.f};

  // ---- main loop ---------------------------------------------------------------------------------------------
  // Step kb = 2 p + j of a slab is step j of pair p.  The operands of a step are read from LDS during the step
  // before; a pair's one barrier stands between its two steps:
  //   step 0 of pair P: the wave's share of pair P + 1 goes into activation area (P + 1) % 2 -- its last readers
  //                     (step 1 of pair P - 1, read during step 0 of pair P - 1) are behind the barrier of pair P - 1
  //                     -- and step 1's fragments are read from area P % 2;
  //   barrier;
  //   step 1 of pair P: the fragments of step 0 of pair P + 1 are read from area (P + 1) % 2, now complete.
  // The weight area is the wave's own: at step 7 its dwords of that step are already in registers, so the next
  // slab (in registers since the last such moment) replaces this one there and its registers take the slab after.
  const uint32_t sz_rd = (uint32_t)(rbw0 * 16 + r) * szrow + (uint32_t)ks * (uint32_t)(kslice >> 6);  // + 4 slab: the slab's two groups
  uint32_t wd_c[RBW], wd_n[RBW];
  uint4_t yf_c[MB], yf_n[MB];
#pragma unroll
  for (int rb = 0; rb < RBW; ++rb) wd_c[rb] = *reinterpret_cast<const uint32_t*>(wst + rb * 2048 + w_rd[0]);
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) yf_c[mb] = *reinterpret_cast<const uint4_t*>(ast + mb * 2048 + a_rd[0]);
  for (int slab = 0; slab < nslab; ++slab) {
    RowGroup rg[RBW];
    static_for<8>([&](auto kb_tag) {
      constexpr int kb = decltype(kb_tag)::value;
      constexpr int p = kb >> 1, j = kb & 1;
      if constexpr (j == 1) __syncthreads();
      if constexpr (kb == 7) {
        static_for<RBW>([&](auto rb) { park_raw(rb); });
        static_for<RBW>([&](auto rb) { load_raw(rb, slab + 2); });
      }
      // the next step's operands
#pragma unroll
      for (int rb = 0; rb < RBW; ++rb)
        wd_n[rb] = *reinterpret_cast<const uint32_t*>(wst + rb * 2048 + w_rd[((kb + 1) & 7) >> 1] + ((kb + 1) & 1) * 4);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
        yf_n[mb] = *reinterpret_cast<const uint4_t*>(ast + ((j == 0 ? p : p + 1) & 1) * kAStage + mb * 2048 + a_rd[j ^ 1]);
      if constexpr (j == 0) {
        park_pair((p + 1) % NP, (p + 1) & 1);
        load_pair((p + 1) % NP, slab * 4 + p + 1 + NP);
      }
      if constexpr ((kb & 3) == 0) {
        // the decoder's constants of this 128-k group
        const uint32_t sel = kb == 0 ? 0x01000100u : 0x03020302u;  // (lo, lo) / (hi, hi) of the slab's two values
        const half2_t n1024 = {(half_t)-1024.f, (half_t)-1024.f}, n64 = {(half_t)-64.f, (half_t)-64.f};
#pragma unroll
        for (int rb = 0; rb < RBW; ++rb) {
          const uint32_t s_raw = kScale ? *reinterpret_cast<const uint32_t*>(s_lds + (uint32_t)(rb * 16) * szrow + sz_rd + slab * 4) : 0u;
          rg[rb].s2 = __builtin_amdgcn_perm(s_raw, s_raw, sel);
          half2_t zf = {(half_t)0.f, (half_t)0.f};  // folded into the bias
          rg[rb].nz2 = 0u;
          if constexpr (MODE == W4_SCALE || MODE == W4_OFFSET8 || MODE == W4_SIGNED) {
            zf = half2_t{(half_t)8.f, (half_t)8.f};
          } else if constexpr (kZeros) {
            const uint32_t z_raw = *reinterpret_cast<const uint32_t*>(z_lds + (uint32_t)(rb * 16) * szrow + sz_rd + slab * 4);
            const half2_t z2 = as_half2(__builtin_amdgcn_perm(z_raw, z_raw, sel));
            if constexpr (MODE == W4_ZEROS_ORIGINAL && FOLD) zf = z2;
            else rg[rb].nz2 = as_u32(-z2);
          }
          rg[rb].nb_lo = as_u32(n1024 - zf);
          rg[rb].nb_hi = as_u32(n64 - zf);
        }
      }
#pragma unroll
      for (int rb = 0; rb < RBW; ++rb) {
        const half8_t xw = decode_row_scaled<MODE, FOLD>(wd_c[rb], rg[rb]);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          acc[rb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xw, __builtin_bit_cast(half8_t, yf_c[mb]), acc[rb][mb], 0, 0, 0);
      }
#pragma unroll
      for (int rb = 0; rb < RBW; ++rb) wd_c[rb] = wd_n[rb];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) yf_c[mb] = yf_n[mb];
    });
  }

  // ---- the partial sums go where the kernel adds the four K quarters up ----------------------------------------
  __syncthreads();  // other waves may still read their last operands where the sums go
  float4_t* const red = reinterpret_cast<float4_t*>(smem);
#pragma unroll
  for (int rb = 0; rb < RBW; ++rb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) red[(wave * 4 * MB + rb * MB + mb) * 64 + lane] = acc[rb][mb];
}

template <int MB, int NP, int MODE, bool APERM>
__global__ __launch_bounds__(512) void w4a16_kslice_kernel(const half_t* __restrict__ A, const uint8_t* __restrict__ B,
                                                           const half_t* __restrict__ S, const half_t* __restrict__ Z,
                                                           half_t* __restrict__ C, int M, int N, int K) {
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr bool kScale = MODE >= W4_SCALE;
  constexpr bool kZeros = MODE >= W4_ZEROS_ORIGINAL;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nrb = N >> 4;
  const int rb0 = blockIdx.x * kRB;
  const int nrb_wg = min(kRB, nrb - rb0);

  // ---- group scales and zeros of the workgroup's rows: staged once, [row][K / 128 values + 8 bytes] ------------------
  // The 8 bytes spread the rows over the banks.  A zero point that is a non-negative integer folds into the
  // decoder's bias; the check runs over what is staged.
  bool fold = true;
  if constexpr (kScale) {
    const uint32_t szrow = (uint32_t)(K >> 6) + 8u;
    unsigned char* const s_lds = smem + kStages;
    unsigned char* const z_lds = s_lds + kRB * 16 * szrow;
    const uint32_t ppr = (uint32_t)K >> 10;  // 16-byte pieces per row of scales
    const uint32_t pieces = (uint32_t)kRB * 16u * ppr;
    const uint32_t sz_bytes = (uint32_t)N * (uint32_t)(K >> 6);
    const __amdgpu_buffer_rsrc_t s_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)S, 0, sz_bytes, kBufferFlags);
    const __amdgpu_buffer_rsrc_t z_rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)Z, 0, kZeros ? sz_bytes : 0u, kBufferFlags);
    for (uint32_t p = (uint32_t)tid; p < pieces; p += 512u) {
      const uint32_t row = p / ppr, piece = p - row * ppr;
      const uint32_t src = ((uint32_t)rb0 * 16u + row) * (uint32_t)(K >> 6) + piece * 16u;
      const uint32_t dst = row * szrow + piece * 16u;
      const uint4_t ss = __builtin_amdgcn_raw_buffer_load_b128(s_rsrc, src, 0, 0);
      reinterpret_cast<uint2_t*>(s_lds + dst)[0] = uint2_t{ss[0], ss[1]};  // rows are 8-byte aligned
      reinterpret_cast<uint2_t*>(s_lds + dst)[1] = uint2_t{ss[2], ss[3]};
      if constexpr (kZeros) {
        const uint4_t zz = __builtin_amdgcn_raw_buffer_load_b128(z_rsrc, src, 0, 0);
        reinterpret_cast<uint2_t*>(z_lds + dst)[0] = uint2_t{zz[0], zz[1]};
        reinterpret_cast<uint2_t*>(z_lds + dst)[1] = uint2_t{zz[2], zz[3]};
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
    if constexpr (MODE == W4_ZEROS_ORIGINAL) fold = __syncthreads_and(fold);
  }

  if (wave < 4) {
    if constexpr (MODE == W4_ZEROS_ORIGINAL) {
      if (fold) kslice_wave<MB, NP, MODE, APERM, 4, true>(A, B, M, N, K);
      else kslice_wave<MB, NP, MODE, APERM, 4, false>(A, B, M, N, K);
    } else {
      kslice_wave<MB, NP, MODE, APERM, 4, true>(A, B, M, N, K);
    }
  } else {
    if constexpr (MODE == W4_ZEROS_ORIGINAL) {
      if (fold) kslice_wave<MB, NP, MODE, APERM, 3, true>(A, B, M, N, K);
      else kslice_wave<MB, NP, MODE, APERM, 3, false>(A, B, M, N, K);
    } else {
      kslice_wave<MB, NP, MODE, APERM, 3, true>(A, B, M, N, K);
    }
  }
  __syncthreads();
  // acc[rb][mb][i] of wave (ks, rgp) = partial C[mb * 16 + r][(rb0 + 4 rgp + rb) * 16 + 4 g + i]
  const int g = lane >> 4, r = lane & 15;
  const float4_t* const red = reinterpret_cast<const float4_t*>(smem);
  for (int p = wave; p < kRB * MB; p += 8) {
    const int rbg = p / MB, mb = p - rbg * MB;
    const int wv = (rbg >> 2) * 4, rbl = rbg & 3;
    float4_t v = red[(wv * 4 * MB + rbl * MB + mb) * 64 + lane];
#pragma unroll
    for (int w = 1; w < 4; ++w) {
      const float4_t o = red[((wv + w) * 4 * MB + rbl * MB + mb) * 64 + lane];
      v = float4_t{v[0] + o[0], v[1] + o[1], v[2] + o[2], v[3] + o[3]};
    }
    const int m = mb * 16 + r;
    if (m < M && rbg < nrb_wg) {
      const half4_t o = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
      *reinterpret_cast<half4_t*>(C + (size_t)m * N + (size_t)(rb0 + rbg) * 16 + g * 4) = o;
    }
  }
}

template <int MB, int NP>
int launch_kslice(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int mode,
                  int layout, hipStream_t stream) {
  constexpr int kLdsMax = 159 * 1024;  // the voting barrier of the zero-point check has a word of its own
  const int lds = kStages + 2 * kRB * 16 * (K / 64 + 8);
  if (lds > kLdsMax) return 1;
  const int nrb = N / 16;
  const dim3 grid((nrb + kRB - 1) / kRB), block(512);
#define DQ_LAUNCH2(MODE_, APERM_)                                                                                 \
  do {                                                                                                            \
    auto kern = w4a16_kslice_kernel<MB, NP, MODE_, APERM_>;                                                       \
    static bool lds_limit_raised[kMaxDevices];                                                                    \
    if (raise_lds_limit<kLdsMax>(kern, lds_limit_raised)) return -1;                                              \
    hipLaunchKernelGGL(kern, grid, block, lds, stream, (const half_t*)A, (const uint8_t*)B, (const half_t*)S,     \
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
// M <= 64, N a multiple of 16 with enough row blocks for every CU, K a multiple of 1024 (whole 256-k slabs per K
// quarter) from 2048 to 8192 (the workgroup's scales fit the LDS), group 128, a mode with scales, and operands below
// 4 GiB.  `deep`: four pairs of activation loads in flight per wave instead of two.
int w4a16_kslice(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int group,
                 int mode, int layout, int deep, hipStream_t stream) {
  if (M < 1 || M > 64 || N < 16 || N % 16 != 0) return 1;
  if (K % 1024 != 0 || K > 8192 || K < 2048) return 1;
  if (mode < W4_SCALE || group != 128) return 1;
  if ((size_t)N * K / 2 >= (1ull << 32) - 8192) return 1;  // 32-bit offsets, and room for the out-of-range marker
  const int nrb = N / 16;
  if (nrb < kRB * 200) return 1;  // fewer than 200 workgroups of seven row blocks
  const int mb = (M + 15) / 16;
  switch (mb) {
    case 1: return 1;
    case 2: return deep ? launch_kslice<2, 4>(A, B, S, Z, C, M, N, K, mode, layout, stream) : launch_kslice<2, 2>(A, B, S, Z, C, M, N, K, mode, layout, stream);
    case 3: return deep ? launch_kslice<3, 4>(A, B, S, Z, C, M, N, K, mode, layout, stream) : launch_kslice<3, 2>(A, B, S, Z, C, M, N, K, mode, layout, stream);
    default: return deep ? launch_kslice<4, 1>(A, B, S, Z, C, M, N, K, mode, layout, stream) : launch_kslice<4, 2>(A, B, S, Z, C, M, N, K, mode, layout, stream);
  }
}

}  // namespace dq
