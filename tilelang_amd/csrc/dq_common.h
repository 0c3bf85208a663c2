// Shared device helpers for the gfx950 dequantize-GEMM kernels: vector types,
// bit-exact weight decoders, and the host-side error buffer of the C-ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

namespace dq {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16_t;
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef int int4_t __attribute__((ext_vector_type(4)));
typedef int int16_t_ __attribute__((ext_vector_type(16)));
typedef unsigned int uint2_t __attribute__((ext_vector_type(2)));
typedef unsigned int uint4_t __attribute__((ext_vector_type(4)));

// ---- host side: error reporting shared by every entry point ----------------------
constexpr int kErrorBufSize = 1024;
char* error_buf();  // static 1024-byte buffer, as in the reference adapter's generated host stub

#define DQ_FAIL(...)                                        \
  do {                                                      \
    snprintf(::dq::error_buf(), ::dq::kErrorBufSize, __VA_ARGS__); \
    return -1;                                              \
  } while (0)

#define DQ_CHECK_HIP(expr)                                                        \
  do {                                                                            \
    hipError_t e__ = (expr);                                                      \
    if (e__ != hipSuccess) DQ_FAIL("%s failed: %s", #expr, hipGetErrorString(e__)); \
  } while (0)

// ---- host side: dynamic LDS requests ------------------------------------------------------------------
// A kernel that asks for more than 64 KiB of dynamic LDS needs its limit raised with hipFuncSetAttribute, once
// per kernel and per device (the attribute belongs to the kernel's code object on that device).  Every launcher
// does so through raise_lds_limit<BYTES>; instantiating it also enters BYTES into a table that is filled while
// the library loads, so init() can compare the largest request of any kernel built into the library with what
// the device offers before anything is launched.
constexpr int kMaxDevices = 64;
int register_lds_request(int bytes);  // returns bytes
int largest_lds_request();

template <int BYTES>
struct LdsRequest {
  static inline const int registered = register_lds_request(BYTES);
};

template <int BYTES, class Kernel>
int raise_lds_limit(Kernel kern, bool (&raised)[kMaxDevices]) {
  (void)LdsRequest<BYTES>::registered;  // forces the load-time registration of this instantiation
  int device = 0;
  DQ_CHECK_HIP(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices) DQ_FAIL("device index %d is beyond the %d this library keeps state for", device, kMaxDevices);
  if (!raised[device]) {  // afterwards the launch makes no attribute call: legal under stream capture
    DQ_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, BYTES));
    raised[device] = true;
  }
  return 0;
}

// ---- weight formats / modes (values are part of the C-ABI, see include/dqgemm.h) --
enum W4Mode : int {
  W4_UNSIGNED = 0,        // w = q
  W4_SIGNED = 1,          // w = sext4(q)  (two's complement)
  W4_OFFSET8 = 2,         // w = q - 8
  W4_SCALE = 3,           // w = RNE16((q - 8) * s)
  W4_USCALE = 4,          // w = RNE16(q * s)
  W4_ZEROS_ORIGINAL = 5,  // w = RNE16(RNE16(q - z) * s)
  W4_ZEROS_RESCALE = 6,   // w = RNE16(fma(q, s, -z))
  W4_ZEROS_FOLDED = 7,    // w = RNE16(fma(q, s, -RNE16(z * s))): (q - z) * s with the zero point folded into one
                          // fused multiply-add; differs from W4_ZEROS_ORIGINAL by the rounding of z * s
  W4_MODE_COUNT = 8,
};

enum W4Layout : int {
  LAYOUT_PLAIN = 0,        // nibble e of a 32-bit word is element e
  LAYOUT_INTERLEAVED = 1,  // word already permuted for the fast 16-bit decoder (elements 0,2,4,6,1,3,5,7)
  LAYOUT_FRAGMENTS = 2,    // flag, added to one of the above: 16-byte pieces re-ordered offline into the matrix
                           // instruction's operand order, [N / 16][K / 128][64 lanes][16 bytes] (uint4, decode GEMV only)
  DECODER_CONVERTER = 4,   // flag of call_dequantize_w4 only: dump the tile with the fp8-converter decoder
};

enum Fp4Format : int {
  FP4_E2M1 = 0,       // OCP e2m1, plain low-first nibbles
  FP4_SIMPLE = 1,     // 2^(E-1) * (1 + m/2) for every E (no zero, no subnormal)
  FP4_TWIDDLING = 2,  // e2m1 in the 16-bit "twiddled" bit layout
};

enum I2Convention : int {
  I2_UNSIGNED = 0,  // w = c
  I2_OFFSET = 1,    // w = c - 2
  I2_TWOS = 2,      // w = sext2(c)
};

// ---- device decoders ---------------------------------------------------------------

__device__ __forceinline__ half2_t as_half2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }
__device__ __forceinline__ uint32_t as_u32(half2_t h) { return __builtin_bit_cast(uint32_t, h); }

// One 32-bit word of eight 4-bit fields -> four half2 holding the raw integer values
// plus a bias: out[i] = (bias_i + n_i, bias_i + n_{i+4}) where n_e is nibble e and
// bias_0 = bias_2 = 1024, bias_1 = bias_3 = 64.  (0x6400 | n) is the fp16 1024 + n,
// (0x5400 | n << 4) is the fp16 64 + n; both are exact.
__device__ __forceinline__ void u4x8_to_biased_half(uint32_t w, uint32_t out[4]) {
  // The two masks live in VGPRs (opaque to the optimiser) so that each (w & mask) | magic
  // is a single v_and_or_b32: a VOP3 on gfx9 may read only one SGPR and no literal.
  uint32_t mlo = 0x000F000Fu, mhi = 0x00F000F0u;
  asm("" : "+v"(mlo));
  asm("" : "+v"(mhi));
  const uint32_t w2 = w >> 8;
  out[0] = (w & mlo) | 0x64006400u;
  out[1] = (w & mhi) | 0x54005400u;
  out[2] = (w2 & mlo) | 0x64006400u;
  out[3] = (w2 & mhi) | 0x54005400u;
}

// Decode one word of eight uint4 weights into fp16 with the rounding order of the
// reference's device snippets.  Result order: element pair i is (n_i, n_{i+4}), i.e.
// fragment element e holds nibble {0,4,1,5,2,6,3,7}[e].  For an interleaved word that
// is the natural element order.
template <int MODE>
__device__ __forceinline__ half8_t decode_w4(uint32_t w, half_t s, half_t z) {
  uint32_t t[4];
  u4x8_to_biased_half(w, t);
  half2_t r[4];
  const half2_t s2 = {s, s};
  const half2_t zero2 = {(half_t)0.f, (half_t)0.f};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const half_t bias = (i & 1) ? (half_t)64.f : (half_t)1024.f;
    half2_t x = as_half2(t[i]);
    if constexpr (MODE == W4_UNSIGNED) {
      const half2_t b2 = {bias, bias};
      r[i] = x - b2;
    } else if constexpr (MODE == W4_SIGNED) {
      // sext4(q) = ((q ^ 8) - 8): flip bit 3 of the nibble inside the mantissa, then
      // subtract bias + 8; all steps exact.
      const uint32_t flip = (i & 1) ? 0x00800080u : 0x00080008u;
      x = as_half2(t[i] ^ flip);
      const half2_t b2 = {(half_t)(bias + (half_t)8.f), (half_t)(bias + (half_t)8.f)};
      r[i] = x - b2;
    } else if constexpr (MODE == W4_OFFSET8) {
      const half2_t b2 = {(half_t)(bias + (half_t)8.f), (half_t)(bias + (half_t)8.f)};
      r[i] = x - b2;
    } else if constexpr (MODE == W4_SCALE) {
      const half2_t b2 = {(half_t)(bias + (half_t)8.f), (half_t)(bias + (half_t)8.f)};
      r[i] = __builtin_elementwise_fma(x - b2, s2, zero2);
    } else if constexpr (MODE == W4_USCALE) {
      const half2_t b2 = {bias, bias};
      r[i] = __builtin_elementwise_fma(x - b2, s2, zero2);
    } else if constexpr (MODE == W4_ZEROS_ORIGINAL) {
      const half2_t b2 = {bias, bias};
      const half2_t z2 = {z, z};
      r[i] = __builtin_elementwise_fma((x - b2) - z2, s2, zero2);
    } else if constexpr (MODE == W4_ZEROS_FOLDED) {
      const half2_t b2 = {bias, bias};
      const half_t nzs = (half_t)(-(z * s));
      const half2_t nzs2 = {nzs, nzs};
      r[i] = __builtin_elementwise_fma(x - b2, s2, nzs2);
    } else {  // W4_ZEROS_RESCALE
      const half2_t b2 = {bias, bias};
      const half2_t nz2 = {(half_t)(-z), (half_t)(-z)};
      r[i] = __builtin_elementwise_fma(x - b2, s2, nz2);
    }
  }
  half8_t o;
  o[0] = r[0][0]; o[1] = r[0][1]; o[2] = r[1][0]; o[3] = r[1][1];
  o[4] = r[2][0]; o[5] = r[2][1]; o[6] = r[3][0]; o[7] = r[3][1];
  return o;
}

// ---- uint4 -> fp16 through the fp8 converter ------------------------------------------------------------
// A byte 0x0q read as OCP e4m3 is q * 2^-9 for every q in 0..15 (q < 8 is subnormal, q >= 8 sits in the first
// binade: together one linear range).  v_cvt_scalef32_pk_f16_fp8 multiplies by the power of two of its scale
// operand (the scale's mantissa is ignored by the hardware), so with scale 512 two bytes become the exact
// integers as an fp16 pair: eight weights cost 3 bit operations and 4 conversions.  The even nibbles of a word
// land in one source dword and the odd ones in another; NATURAL spends two v_perm_b32 on the bytes so that the
// result is in element order 0..7 for either word layout (the activations then need no permutation).  Without
// NATURAL a plain word yields elements (0 2 4 6 1 3 5 7) and an interleaved word (0 4 1 5 2 6 3 7).
template <bool INTERLEAVED, bool NATURAL>
__device__ __forceinline__ void u4x8_to_half_cvt(uint32_t w, half2_t out[4]) {
  const uint32_t even = w & 0x0F0F0F0Fu, odd = (w >> 4) & 0x0F0F0F0Fu;
  uint32_t x = even, y = odd;
  if constexpr (NATURAL) {
    // plain: even = (n0 n2 n4 n6), odd = (n1 n3 n5 n7); interleaved: even = (e0 e4 e1 e5), odd = (e2 e6 e3 e7)
    x = __builtin_amdgcn_perm(odd, even, INTERLEAVED ? 0x06040200u : 0x05010400u);
    y = __builtin_amdgcn_perm(odd, even, INTERLEAVED ? 0x07050301u : 0x07030602u);
  }
  out[0] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(x, 512.0f, false);
  out[1] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(x, 512.0f, true);
  out[2] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(y, 512.0f, false);
  out[3] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(y, 512.0f, true);
}

// The second operand of decode_w4_cvt for a (row, group): computed once and used for every word of the group.
template <int MODE>
__device__ __forceinline__ half_t w4_cvt_addend(half_t s, half_t z) {
  if constexpr (MODE == W4_SCALE) return (half_t)((half_t)-8.f * s);       // exact: a power of two times s
  else if constexpr (MODE == W4_ZEROS_FOLDED) return (half_t)(-(z * s));   // one rounding
  else if constexpr (MODE == W4_ZEROS_ORIGINAL || MODE == W4_ZEROS_RESCALE) return (half_t)(-z);
  else return (half_t)0.f;
}

// Decode one word of eight uint4 weights with the converter above.  Same values, bit for bit, as decode_w4<MODE>
// in every mode of the C-ABI: (q - 8) * s is one fused multiply-add with the exact addend -8 s, (q - z) * s is an
// addition (the reference's first rounding) and a multiplication (its second), fma(q, s, -z) is itself.
template <int MODE, bool INTERLEAVED, bool NATURAL>
__device__ __forceinline__ half8_t decode_w4_cvt(uint32_t w, half_t s, half_t addend) {
  half2_t r[4];
  u4x8_to_half_cvt<INTERLEAVED, NATURAL>(MODE == W4_SIGNED ? (w ^ 0x88888888u) : w, r);
  const half2_t s2 = {s, s}, a2 = {addend, addend};
  const half2_t m8 = {(half_t)-8.f, (half_t)-8.f}, zero2 = {(half_t)0.f, (half_t)0.f};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if constexpr (MODE == W4_SIGNED || MODE == W4_OFFSET8) r[i] = r[i] + m8;  // sext4(q) = (q ^ 8) - 8
    // the reference multiplies with fma(x, s, +0): a zero product comes out as +0 whatever the sign of s
    else if constexpr (MODE == W4_USCALE) r[i] = __builtin_elementwise_fma(r[i], s2, zero2);
    else if constexpr (MODE == W4_ZEROS_ORIGINAL) r[i] = __builtin_elementwise_fma(r[i] + a2, s2, zero2);
    else if constexpr (MODE != W4_UNSIGNED) r[i] = __builtin_elementwise_fma(r[i], s2, a2);  // SCALE, RESCALE, FOLDED
  }
  half8_t o;
  o[0] = r[0][0]; o[1] = r[0][1]; o[2] = r[1][0]; o[3] = r[1][1];
  o[4] = r[2][0]; o[5] = r[2][1]; o[6] = r[3][0]; o[7] = r[3][1];
  return o;
}

// Permute eight consecutive 16-bit activations a0..a7 (two per register) into the
// order the plain-layout decoder produces: (a0,a4) (a1,a5) (a2,a6) (a3,a7).
__device__ __forceinline__ uint4_t permute_k8_16bit(uint4_t d) {
  uint4_t o;
  // __builtin_amdgcn_perm(hi_src, lo_src, sel): byte i of the result is byte sel[i] of {hi_src:lo_src}
  o[0] = __builtin_amdgcn_perm(d[2], d[0], 0x05040100u);  // (d0.lo, d2.lo)
  o[1] = __builtin_amdgcn_perm(d[2], d[0], 0x07060302u);  // (d0.hi, d2.hi)
  o[2] = __builtin_amdgcn_perm(d[3], d[1], 0x05040100u);  // (d1.lo, d3.lo)
  o[3] = __builtin_amdgcn_perm(d[3], d[1], 0x07060302u);  // (d1.hi, d3.hi)
  return o;
}

// 16 consecutive int8 (a0..a15) -> dword i = (a[i], a[4+i], a[8+i], a[12+i]): the element order
// of the 2-bit decoder, whose dword i holds the codes at bit 2i of each packed byte.
__device__ __forceinline__ uint4_t transpose4x4_bytes(uint4_t d) {
  const uint32_t t01_lo = __builtin_amdgcn_perm(d[1], d[0], 0x05010400u);  // d0.b0 d1.b0 d0.b1 d1.b1
  const uint32_t t01_hi = __builtin_amdgcn_perm(d[1], d[0], 0x07030602u);  // d0.b2 d1.b2 d0.b3 d1.b3
  const uint32_t t23_lo = __builtin_amdgcn_perm(d[3], d[2], 0x05010400u);
  const uint32_t t23_hi = __builtin_amdgcn_perm(d[3], d[2], 0x07030602u);
  uint4_t o;
  o[0] = __builtin_amdgcn_perm(t23_lo, t01_lo, 0x05040100u);
  o[1] = __builtin_amdgcn_perm(t23_lo, t01_lo, 0x07060302u);
  o[2] = __builtin_amdgcn_perm(t23_hi, t01_hi, 0x05040100u);
  o[3] = __builtin_amdgcn_perm(t23_hi, t01_hi, 0x07060302u);
  return o;
}

// 16 consecutive int8 -> (a0 a2 a4 a6) (a1 a3 a5 a7) (a8 a10 a12 a14) (a9 a11 a13 a15): the element
// order of the nibble decoder, whose dwords hold the even / odd nibbles of one packed word.
__device__ __forceinline__ uint4_t split_even_odd_bytes(uint4_t d) {
  uint4_t o;
  o[0] = __builtin_amdgcn_perm(d[1], d[0], 0x06040200u);
  o[1] = __builtin_amdgcn_perm(d[1], d[0], 0x07050301u);
  o[2] = __builtin_amdgcn_perm(d[3], d[2], 0x06040200u);
  o[3] = __builtin_amdgcn_perm(d[3], d[2], 0x07050301u);
  return o;
}

template <int CTRL, class T>
__device__ __forceinline__ T dpp_move(T x) {
  static_assert(sizeof(T) == 4, "one register");
  return __builtin_bit_cast(T, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, true));
}

// Sums N per-lane values (float or int) over each DPP row of 16 lanes at once.  While more than one value is
// left, a level lets a lane keep the value its lane bit selects and add the partner lane's copy
// of it, which halves the number of values; afterwards a level is a plain add.  Levels: xor 1,
// xor 2 (quad_perm), rotate by 4, rotate by 8 (row_ror).  On return lane l holds the row total
// of value (l & (N - 1)).  N values cost about 3 (N - 1) + 4 instructions instead of 4 N.
template <int N, int LEVEL, class T = float>
struct RowReduce {
  static __device__ __forceinline__ T run(const T* v, int lane) {
    if constexpr (LEVEL == 4) {
      return v[0];
    } else {
      constexpr int kCtrl = LEVEL == 0 ? 0xB1 : (LEVEL == 1 ? 0x4E : (LEVEL == 2 ? 0x124 : 0x128));
      if constexpr (N == 1) {
        const T t[1] = {v[0] + dpp_move<kCtrl>(v[0])};
        return RowReduce<1, LEVEL + 1, T>::run(t, lane);
      } else {
        const bool bit = (lane >> LEVEL) & 1;
        T t[N / 2];
#pragma unroll
        for (int i = 0; i < N / 2; ++i) {
          const T keep = bit ? v[2 * i + 1] : v[2 * i];
          const T give = bit ? v[2 * i] : v[2 * i + 1];
          t[i] = keep + dpp_move<kCtrl>(give);
        }
        return RowReduce<N / 2, LEVEL + 1, T>::run(t, lane);
      }
    }
  }
};

}  // namespace dq
