// BitNet W2A8 (int8 x 2-bit) tiled GEMM: the kernels for fragment-ordered weights (direct-to-LDS kernel only) (dq_gemm_i2.h).
#include "dq_gemm_i2.h"

namespace dq {

int i2_gemm_fragments(const gemm::Params& p, int convention, bool interleaved, bool bitnet_epilogue, hipStream_t stream) {
  if (interleaved) {
    return bitnet_epilogue ? i2_gemm_part<true, true, true>(p, convention, stream) : i2_gemm_part<true, false, true>(p, convention, stream);
  }
  return bitnet_epilogue ? i2_gemm_part<false, true, true>(p, convention, stream) : i2_gemm_part<false, false, true>(p, convention, stream);
}

}  // namespace dq
