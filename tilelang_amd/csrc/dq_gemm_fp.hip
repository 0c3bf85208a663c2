// 16-bit operand policies of the LDS-staged dequantize GEMM (dq_gemm_core.h): MXFP4 x bf16, fp4 x bf16 and
// "simple" fp4 x fp16 (uint4 x fp16: dq_gemm_w4.hip).
#include "dq_fp4_codes.h"
#include "dq_gemm_core.h"

namespace dq {

namespace {

using gemm::Params;

struct Bf16Mfma {
  static constexpr int kKPerBlock = 64;
  using frag_t = bf16x8_t;
  using acc_t = float16_t;
  __device__ static __forceinline__ acc_t mfma(frag_t a, frag_t b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};

struct F16Mfma {
  static constexpr int kKPerBlock = 64;
  using frag_t = half8_t;
  using acc_t = float16_t;
  __device__ static __forceinline__ acc_t mfma(frag_t a, frag_t b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

// ---- MXFP4 x bf16 -------------------------------------------------------------------------------
// Scale[N, K/32] uint8, p.p0 = 127 - scale_bias.  Lane group g owns one 32-k scale block per tile.
template <int FMT, bool HAS_BIAS>
struct MxPolicy : Bf16Mfma, gemm::PlainA {
  static constexpr int kBRowBytes = 32;
  static constexpr bool kTransposed = false;
  using out_t = bf16_t;
  using ScaleRaw = int;
  static constexpr int kScaleDma = 1;  // one scale byte per 32 k travels by DMA in the direct-to-LDS kernel
  static bool dma_ok(const Params&) { return true; }
  struct Scale { float f; uint32_t add; };
  __device__ static __forceinline__ ScaleRaw fetch_scale(const Params& p, int row, int kb, int g) {
    return ((const uint8_t*)p.S)[(size_t)row * (p.K >> 5) + kb * 2 + g];
  }
  __device__ static __forceinline__ Scale prep_scale(ScaleRaw e, const Params& p) {
    Scale s;
    if constexpr (FMT == FP4_SIMPLE) {
      int ex = 126 + e + p.p0 - 127;
      ex = ex < 0 ? 0 : (ex > 252 ? 252 : ex);  // E adds up to 3
      s.add = ((uint32_t)ex << 7) * 0x00010001u;
      s.f = 0.f;
    } else {
      s.f = scale_to_f32(e, p.p0);
      s.add = 0;
    }
    return s;
  }
  __device__ static __forceinline__ frag_t decode(const uint32_t* w, int j, const Scale& s) {
    if constexpr (FMT == FP4_E2M1) return cvt_e2m1x8(w[j], s.f);
    else if constexpr (FMT == FP4_TWIDDLING) return cvt_e2m1x8(twiddled_to_plain(w[j]), s.f);
    else return __builtin_bit_cast(frag_t, simple_fp4x8<7>(w[j], s.add));
  }
  __device__ static __forceinline__ out_t finish(uint32_t raw, const Params& p, int m, int n) {
    float v = __builtin_bit_cast(float, raw);
    // reference: C = bf16(float(acc) + float(Bias))
    if constexpr (HAS_BIAS) v += (float)((const bf16_t*)p.Bias)[(size_t)m * p.N + n];
    return (bf16_t)v;
  }
};

// ---- fp4 x bf16 without block scales (examples/dequantize_gemm/example_dequant_gemm_bf16_fp4_hopper.py) ------------
// The same three nibble formats as above with the exponent offset at zero: the twiddled layout of the example's
// fast_dequant=True (:113-118) and the "simple" conversion of fast_dequant=False (:222-262: exponent E + 126).
template <int FMT>
struct Bf16Fp4Policy : Bf16Mfma, gemm::PlainA, gemm::NoScale {
  static constexpr int kBRowBytes = 32;
  static constexpr bool kTransposed = false;
  using out_t = bf16_t;
  __device__ static __forceinline__ Scale prep_scale(int, const Params&) { return {}; }
  using gemm::NoScale::prep_scale;
  __device__ static __forceinline__ frag_t decode(const uint32_t* w, int j, const Scale&) {
    if constexpr (FMT == FP4_E2M1) return cvt_e2m1x8(w[j], 1.f);
    else if constexpr (FMT == FP4_TWIDDLING) return cvt_e2m1x8(twiddled_to_plain(w[j]), 1.f);
    else return __builtin_bit_cast(frag_t, simple_fp4x8<7>(w[j], 0x3F003F00u));  // (E + 126) << 7
  }
  __device__ static __forceinline__ out_t finish(uint32_t raw, const Params&, int, int) {
    return (bf16_t)__builtin_bit_cast(float, raw);
  }
};

// ---- "simple" fp4 x fp16 (examples/dequantize_gemm/example_dequant_gemm_fp4_hopper.py) ------------
template <bool TRANSPOSED>
struct Fp16Fp4Policy : F16Mfma, gemm::PlainA, gemm::NoScale {
  static constexpr int kBRowBytes = 32;
  __device__ static __forceinline__ Scale prep_scale(int, const Params&) { return {}; }
  using gemm::NoScale::prep_scale;
  static constexpr bool kTransposed = TRANSPOSED;
  using out_t = half_t;
  __device__ static __forceinline__ frag_t decode(const uint32_t* w, int j, const Scale&) {
    return __builtin_bit_cast(frag_t, simple_fp4x8<10>(w[j], 0x38003800u));  // (E + 14) << 10
  }
  __device__ static __forceinline__ out_t finish(uint32_t raw, const Params&, int, int) {
    return (half_t)__builtin_bit_cast(float, raw);
  }
};

}  // namespace

int mxfp4_gemm(const void* A, const void* B, const void* S, const void* Bias, void* C, int M, int N, int K, int fmt,
               int scale_bias, hipStream_t stream) {
  Params p = gemm::make_params(A, B, S, nullptr, Bias, C, M, N, K);
  p.p0 = 127 - scale_bias;
#define DQ_MX(FMT_)                                                        \
  do {                                                                     \
    if (Bias) return gemm::launch_best<MxPolicy<FMT_, true>>(p, stream);   \
    return gemm::launch_best<MxPolicy<FMT_, false>>(p, stream);            \
  } while (0)
  switch (fmt) {
    case FP4_E2M1: DQ_MX(FP4_E2M1);
    case FP4_SIMPLE: DQ_MX(FP4_SIMPLE);
    case FP4_TWIDDLING: DQ_MX(FP4_TWIDDLING);
    default: DQ_FAIL("mxfp4 gemm: unknown weight format %d", fmt);
  }
#undef DQ_MX
}

int bf16_fp4_gemm(const void* A, const void* B, void* C, int M, int N, int K, int fmt, hipStream_t stream) {
  Params p = gemm::make_params(A, B, nullptr, nullptr, nullptr, C, M, N, K);
#define DQ_F4(FMT_) return gemm::launch_best<Bf16Fp4Policy<FMT_>>(p, stream)
  switch (fmt) {
    case FP4_E2M1: DQ_F4(FP4_E2M1);
    case FP4_SIMPLE: DQ_F4(FP4_SIMPLE);
    case FP4_TWIDDLING: DQ_F4(FP4_TWIDDLING);
    default: DQ_FAIL("bf16 x fp4 gemm: unknown weight format %d", fmt);
  }
#undef DQ_F4
}

int fp16_fp4_gemm(const void* A, const void* B, void* C, int M, int N, int K, int transposed, hipStream_t stream) {
  Params p = gemm::make_params(A, B, nullptr, nullptr, nullptr, C, M, N, K);
  if (transposed) return gemm::launch_best<Fp16Fp4Policy<true>>(p, stream);
  return gemm::launch_best<Fp16Fp4Policy<false>>(p, stream);
}

namespace {

// Second kernel of the split-K form (examples/dequantize_gemm/example_dequant_gemm_fp4_hopper.py:168-175): the
// partial results are fp16 and are added in fp16, slice 0 first, as the reference's `acc += SplitC[k]` does.
__global__ __launch_bounds__(256) void splitk_sum_f16_kernel(const half_t* __restrict__ parts, half_t* __restrict__ out,
                                                             size_t count, int split) {
  const size_t i8 = ((size_t)blockIdx.x * 256 + threadIdx.x) * 8;
  if (i8 + 8 <= count) {
    half8_t acc = *reinterpret_cast<const half8_t*>(parts + i8);
    for (int z = 1; z < split; ++z) acc = acc + *reinterpret_cast<const half8_t*>(parts + (size_t)z * count + i8);
    *reinterpret_cast<half8_t*>(out + i8) = acc;
  } else {
    for (size_t i = i8; i < count; ++i) {
      half_t acc = parts[i];
      for (int z = 1; z < split; ++z) acc = acc + parts[(size_t)z * count + i];
      out[i] = acc;
    }
  }
}

}  // namespace

// K cut into `split` slices, each multiplied by its own workgroups into parts[z] (M x N, or N x M when transposed,
// fp16), then summed.  Worth it when M x N alone gives the 256 CUs too few tiles.
int fp16_fp4_gemm_splitk(const void* A, const void* B, void* parts, void* C, int M, int N, int K, int split,
                         int transposed, hipStream_t stream) {
  Params p = gemm::make_params(A, B, nullptr, nullptr, nullptr, parts, M, N, K / split);
  p.ldk = K;
  p.split = split;
  const int rc = transposed ? gemm::launch_best<Fp16Fp4Policy<true>>(p, stream) : gemm::launch_best<Fp16Fp4Policy<false>>(p, stream);
  if (rc) return rc;
  const size_t count = (size_t)M * N;
  // the partial results are 16-byte aligned slice by slice only when M x N is a multiple of 8
  if (count % 8 != 0) DQ_FAIL("fp16 x fp4 split-K gemm: M * N = %zu must be a multiple of 8", count);
  const unsigned blocks = (unsigned)((count + 2047) / 2048);
  hipLaunchKernelGGL(splitk_sum_f16_kernel, dim3(blocks), dim3(256), 0, stream, (const half_t*)parts, (half_t*)C, count, split);
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}


}  // namespace dq
