// BitNet W2A8 (int8 x 2-bit) tiled GEMM: the kernels for row-major words and the int32 epilogue (dq_gemm_i2.h).
#include "dq_gemm_i2.h"

namespace dq {

int i2_gemm_rowmajor_int32(const gemm::Params& p, int convention, hipStream_t stream) {
  return i2_gemm_part<false, false, false>(p, convention, stream);
}

}  // namespace dq
