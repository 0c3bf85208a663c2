// Plain GEMM on the LDS-staged skeleton of the dequantize GEMMs (dq_gemm_core.h): both operands already at
// the compute type, so the policy's "decoder" hands the packed-B words to the matrix instruction unchanged.
//
// Stands where T.gemm without a dequantise step stands in the reference
// (testing/python/kernel/test_tilelang_kernel_gemm.py:5-105: matmul(M, N, K, ..., trans_A, trans_B, in_dtype,
// out_dtype, accum_dtype), f16 / bf16 / int8, nn / nt / tn / tt; testing/python/amd/test_tilelang_test_amd.py:7-157
// for the ROCm shapes).  Its use here is to pin the shared tile -- A staging and swizzle, fragment layout, MFMA,
// raster, epilogue -- without any decoder whose own permutation could cancel a layout mistake.
//
// The skeleton multiplies A[M,K] by B[N,K]^T ("nt", the layout of every dequantize kernel).  The other three
// operand layouts are brought to it by a tiled transpose of the operand that is stored the other way round, into
// a workspace the caller passes.
#include "dq_gemm_core.h"

namespace dq {

namespace {

using gemm::Params;

struct PlainBf16 {
  static constexpr int kKPerBlock = 64;
  using frag_t = bf16x8_t;
  using acc_t = float16_t;
  __device__ static __forceinline__ acc_t mfma(frag_t a, frag_t b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};

struct PlainF16 {
  static constexpr int kKPerBlock = 64;
  using frag_t = half8_t;
  using acc_t = float16_t;
  __device__ static __forceinline__ acc_t mfma(frag_t a, frag_t b, acc_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

struct PlainI8 {
  static constexpr int kKPerBlock = 128;
  using frag_t = int4_t;
  using acc_t = int16_t_;
  __device__ static __forceinline__ acc_t mfma(frag_t a, frag_t b, acc_t c) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
  }
};

// B rows are 128 bytes per k-block, like A rows: lane group g owns pieces 4g .. 4g+3 of its row and piece
// 4g + j is the operand of MFMA step j, exactly the k range of the A fragment of that step.
template <class MFMA, class OUT>
struct PlainPolicy : MFMA, gemm::PlainA, gemm::NoScale {
  static constexpr int kBRowBytes = 128;
  static constexpr bool kTransposed = false;
  using out_t = OUT;
  using frag_t = typename MFMA::frag_t;
  __device__ static __forceinline__ Scale prep_scale(int, const Params&) { return {}; }
  using gemm::NoScale::prep_scale;
  __device__ static __forceinline__ frag_t decode(const uint32_t* w, int j, const Scale&) {
    const uint4_t v = {w[4 * j], w[4 * j + 1], w[4 * j + 2], w[4 * j + 3]};
    return __builtin_bit_cast(frag_t, v);
  }
  __device__ static __forceinline__ out_t finish(uint32_t raw, const Params&, int, int) {
    if constexpr (std::is_same<OUT, int32_t>::value) return (int32_t)raw;
    else return (OUT)__builtin_bit_cast(float, raw);
  }
};

// out[c][r] = in[r][c] for a rows x cols matrix of T (1 or 2 bytes), 64 x 64 tiles through LDS.
template <class T>
__global__ __launch_bounds__(256) void transpose_kernel(const T* __restrict__ in, T* __restrict__ out, int rows, int cols) {
  __shared__ T tile[64][64 + 2];
  const int c0 = blockIdx.x * 64, r0 = blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int i = ty; i < 64; i += 4) {
    const int r = r0 + i, c = c0 + tx;
    if (r < rows && c < cols) tile[i][tx] = in[(size_t)r * cols + c];
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    const int c = c0 + i, r = r0 + tx;
    if (c < cols && r < rows) out[(size_t)c * rows + r] = tile[tx][i];
  }
}

template <class T>
int transpose(const void* in, void* out, int rows, int cols, hipStream_t stream) {
  const dim3 grid((cols + 63) / 64, (rows + 63) / 64);
  hipLaunchKernelGGL(transpose_kernel<T>, grid, dim3(256), 0, stream, (const T*)in, (T*)out, rows, cols);
  DQ_CHECK_HIP(hipGetLastError());
  return 0;
}

// 128-byte B rows take 64 KiB of LDS per stage at 256 x 256: the plain policy runs the 128 x 128 and 128 x 64
// tiles of the register-staged kernel only.
template <class P>
int launch_plain(const Params& p, hipStream_t stream) {
  const long tiles = (long)((p.M + 127) / 128) * ((p.N + 127) / 128);
  if (tiles >= 192) return gemm::launch<P, 2, 2>(p, stream);
  return gemm::launch<P, 2, 1>(p, stream);
}

}  // namespace

// in_dtype / out_dtype: 0 fp16, 1 bf16, 2 int8, 3 fp32, 4 int32 (DQ_DT_* of the header).
int plain_gemm(const void* A, const void* B, void* C, void* workspace, int M, int N, int K, int in_dtype, int out_dtype,
               int trans_A, int trans_B, hipStream_t stream) {
  const size_t esz = in_dtype == 2 ? 1 : 2;
  unsigned char* ws = (unsigned char*)workspace;
  if (trans_A) {  // A is stored [K, M]
    const int rc = esz == 1 ? transpose<uint8_t>(A, ws, K, M, stream) : transpose<uint16_t>(A, ws, K, M, stream);
    if (rc) return rc;
    A = ws;
    ws += (((size_t)M * K * esz + 255) & ~(size_t)255);
  }
  if (!trans_B) {  // B is stored [K, N]
    const int rc = esz == 1 ? transpose<uint8_t>(B, ws, K, N, stream) : transpose<uint16_t>(B, ws, K, N, stream);
    if (rc) return rc;
    B = ws;
  }
  Params p = gemm::make_params(A, B, nullptr, nullptr, nullptr, C, M, N, K);
  if (in_dtype == 0 && out_dtype == 0) return launch_plain<PlainPolicy<PlainF16, half_t>>(p, stream);
  if (in_dtype == 0 && out_dtype == 3) return launch_plain<PlainPolicy<PlainF16, float>>(p, stream);
  if (in_dtype == 1 && out_dtype == 1) return launch_plain<PlainPolicy<PlainBf16, bf16_t>>(p, stream);
  if (in_dtype == 1 && out_dtype == 3) return launch_plain<PlainPolicy<PlainBf16, float>>(p, stream);
  if (in_dtype == 2 && out_dtype == 4) return launch_plain<PlainPolicy<PlainI8, int32_t>>(p, stream);
  DQ_FAIL("plain gemm: unsupported dtype combination in=%d out=%d", in_dtype, out_dtype);
}

}  // namespace dq
