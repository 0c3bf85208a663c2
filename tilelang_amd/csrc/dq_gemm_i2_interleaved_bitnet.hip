// BitNet W2A8 (int8 x 2-bit) tiled GEMM: the kernels for interleaved words and the BitLinear fp16 epilogue (dq_gemm_i2.h).
#include "dq_gemm_i2.h"

namespace dq {

int i2_gemm_interleaved_bitnet(const gemm::Params& p, int convention, hipStream_t stream) {
  return i2_gemm_part<true, true, false>(p, convention, stream);
}

}  // namespace dq
