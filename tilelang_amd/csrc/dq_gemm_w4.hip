// uint4 x fp16 policy of the LDS-staged dequantize GEMM (dq_gemm_core.h): the fine-grained example and W4A16 at large M.
#include "dq_gemm_core.h"

namespace dq {

namespace {

using gemm::Params;

struct F16Mfma {
  static constexpr int kKPerBlock = 64;
  using frag_t = half8_t;
  using acc_t = float16_t;
  __device__ static __forceinline__ acc_t mfma(frag_t a, frag_t b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

// ---- uint4 x fp16 with the integer decoders (fine-grained example, W4A16 at large M) ---------------
// Scale / Zeros fp16 [N, K/group], p.p0 = log2(group) (31 when group == K), p.p1 = K / group.
template <int MODE, bool INTERLEAVED>
struct W4F16Policy : F16Mfma {
  static constexpr int kBRowBytes = 32;
  static constexpr bool kTransposed = false;
  static constexpr bool kAPacked = false;
  // 9 to 17 vector instructions per decoded operand: with two rows of waves a lone wave's instruction issue is
  // busier than its matrix pipe (fp16 x uint4 at M = 4096, N = K = 8192: 467 us; 427 us with the waves side by side)
  static constexpr bool kTallWaves = true;
  using out_t = half_t;
  struct ScaleRaw { half_t s, z; };
  struct Scale { half_t s, addend; };  // what the decoder multiplies by and adds (w4_cvt_addend)
  // direct-to-LDS kernel: the fp16 scales (and zeros) of groups of 32 .. 4096 k travel by DMA, a dword per row (two
  // groups: four tiles of 64 k at group 128) at a time; (groups of 32 k on the 128 x 256 tile only); one group per row
  // and odd group counts stay on the register-staged kernel
  static constexpr int kScaleDma = MODE >= W4_ZEROS_ORIGINAL ? 3 : (MODE >= W4_SCALE ? 2 : 0);
  static bool dma_ok(const Params& p) { return kScaleDma == 0 || (p.p0 >= 5 && p.p0 <= 12 && p.K % (2 << p.p0) == 0); }
  __device__ static __forceinline__ Scale ring_scale(const unsigned char* s_at, const unsigned char* z_at) {
    ScaleRaw r{(half_t)1.f, (half_t)0.f};
    r.s = *reinterpret_cast<const half_t*>(s_at);
    if constexpr (kScaleDma == 3) r.z = *reinterpret_cast<const half_t*>(z_at);
    return Scale{r.s, w4_cvt_addend<MODE>(r.s, r.z)};
  }
  __device__ static __forceinline__ Scale prep_scale(int, const Params&) { return Scale{(half_t)1.f, (half_t)0.f}; }
  // the decoder emits the eight weights of a word in element order for either word layout: the activations go to
  // LDS and into the matrix instruction untouched
  __device__ static __forceinline__ uint4_t stage_a(uint4_t v) { return v; }
  __device__ static __forceinline__ frag_t fix_a(frag_t f) { return f; }
  __device__ static __forceinline__ void expand_a(uint4_t, uint4_t&, uint4_t&) {}
  __device__ static __forceinline__ ScaleRaw fetch_scale(const Params& p, int row, int kb, int g) {
    ScaleRaw r{(half_t)1.f, (half_t)0.f};
    const size_t idx = (size_t)row * p.p1 + ((kb * 64 + g * 32) >> p.p0);
    if constexpr (MODE >= W4_SCALE) r.s = ((const half_t*)p.S)[idx];
    if constexpr (MODE >= W4_ZEROS_ORIGINAL) r.z = ((const half_t*)p.Z)[idx];
    return r;
  }
  __device__ static __forceinline__ Scale prep_scale(ScaleRaw r, const Params&) {
    return Scale{r.s, w4_cvt_addend<MODE>(r.s, r.z)};
  }
  __device__ static __forceinline__ frag_t decode(const uint32_t* w, int j, const Scale& s) {
    return decode_w4_cvt<MODE, INTERLEAVED, true>(w[j], s.s, s.addend);
  }
  __device__ static __forceinline__ out_t finish(uint32_t raw, const Params&, int, int) {
    return (half_t)__builtin_bit_cast(float, raw);
  }
};

}  // namespace

int w4_f16_gemm(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int group,
                int mode, int layout, hipStream_t stream) {
  Params p = gemm::make_params(A, B, S, Z, nullptr, C, M, N, K);
  p.p0 = (group == K) ? 31 : (31 - __builtin_clz(group));
  p.p1 = K / group;
#define DQ_W4(MODE_)                                                                                \
  do {                                                                                              \
    if (layout == LAYOUT_PLAIN) return gemm::launch_best<W4F16Policy<MODE_, false>>(p, stream);     \
    return gemm::launch_best<W4F16Policy<MODE_, true>>(p, stream);                                  \
  } while (0)
  switch (mode) {
    case W4_UNSIGNED: DQ_W4(W4_UNSIGNED);
    case W4_SIGNED: DQ_W4(W4_SIGNED);
    case W4_OFFSET8: DQ_W4(W4_OFFSET8);
    case W4_SCALE: DQ_W4(W4_SCALE);
    case W4_USCALE: DQ_W4(W4_USCALE);
    case W4_ZEROS_ORIGINAL: DQ_W4(W4_ZEROS_ORIGINAL);
    case W4_ZEROS_RESCALE: DQ_W4(W4_ZEROS_RESCALE);
    case W4_ZEROS_FOLDED: DQ_W4(W4_ZEROS_FOLDED);
    default: DQ_FAIL("w4 fp16 gemm: unknown mode %d", mode);
  }
#undef DQ_W4
}

}  // namespace dq
