// BitNet W2A8 (int8 x 2-bit) tiled GEMM: the entry point, which picks the translation unit that holds the word
// layout and epilogue asked for (dq_gemm_i2.h).
#include "dq_gemm_i2.h"

namespace dq {

int i2_gemm(const void* A, const void* B, void* C, int M, int N, int K, int convention, int layout, const void* s_a,
            float s_w, int bitnet_epilogue, hipStream_t stream) {
  gemm::Params p = gemm::make_params(A, B, s_a, nullptr, nullptr, C, M, N, K);
  p.f0 = s_w;
  const bool interleaved = (layout & ~LAYOUT_FRAGMENTS) == LAYOUT_INTERLEAVED;
  if (layout & LAYOUT_FRAGMENTS) return i2_gemm_fragments(p, convention, interleaved, bitnet_epilogue != 0, stream);
  if (interleaved) {
    return bitnet_epilogue ? i2_gemm_interleaved_bitnet(p, convention, stream) : i2_gemm_interleaved_int32(p, convention, stream);
  }
  return bitnet_epilogue ? i2_gemm_rowmajor_bitnet(p, convention, stream) : i2_gemm_rowmajor_int32(p, convention, stream);
}

}  // namespace dq
