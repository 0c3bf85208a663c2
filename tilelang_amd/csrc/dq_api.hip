// extern "C" entry points of libdqgemm.so (declared in include/dqgemm.h).
//
// Same shape as the host stub the reference's adapter generates around every JIT kernel
// (tilelang/jit/adapter/wrapper.py:59-85): init / get_last_error / call, raw pointers and
// sizes in, 0 or -1 out, message in a static buffer.  Argument checks run before any
// launch so a bad call never reaches the GPU.
#include "../../include/dqgemm.h"
#include "dq_common.h"

namespace dq {

static char g_error_buf[kErrorBufSize];
char* error_buf() { return g_error_buf; }

// Filled by the initialisers of LdsRequest<BYTES>::registered while the library loads (zero-initialised
// before any of them runs).
static int g_largest_lds_request;
int register_lds_request(int bytes) {
  if (bytes > g_largest_lds_request) g_largest_lds_request = bytes;
  return bytes;
}
int largest_lds_request() { return g_largest_lds_request; }

// kernels (defined in the .hip files next to this one)
int w4a16_regres(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int group,
                 int mode, int layout, int fast, hipStream_t stream);
int w4a16_stream(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int group,
                 int mode, int layout, int config, int split, void* parts, hipStream_t stream);
int w4a16_skinny(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int group,
                 int mode, int layout, int variant, hipStream_t stream);
int w4_dequant(const void* B, const void* S, const void* Z, void* W, int N, int K, int group, int mode, int layout,
               hipStream_t stream);
int w4a16_gemv_dot2(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int group,
                    int mode, int layout, int rows_hint, hipStream_t stream);

int mxfp4_gemm(const void* A, const void* B, const void* S, const void* Bias, void* C, int M, int N, int K, int fmt,
               int scale_bias, hipStream_t stream);

int mxfp4_gemm_regres(const void* A, const void* B, const void* S, const void* Bias, void* C, int M, int N, int K, int fmt,
                      int scale_bias, int max_rows, hipStream_t stream);
int bf16_fp4_gemm(const void* A, const void* B, void* C, int M, int N, int K, int fmt, hipStream_t stream);
int fp16_fp4_gemm(const void* A, const void* B, void* C, int M, int N, int K, int transposed, hipStream_t stream);
int w4_f16_gemm(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int group,
                int mode, int layout, hipStream_t stream);
int i2_gemm(const void* A, const void* B, void* C, int M, int N, int K, int convention, int layout, const void* s_a,
            float s_w, int bitnet_epilogue, hipStream_t stream);
int wlow_gemv(const void* A, const void* B, const void* Scale, const void* Zeros, void* C, int M, int N, int K, int group,
              int bits, int convention, int layout, int zeros_rescale, hipStream_t stream);
int i2_gemm_kslice(const void* A, const void* B, void* C, int M, int N, int K, int convention, int layout, const void* s_a,
                   float s_w, int bitnet_epilogue, int force, hipStream_t stream);
int i2_gemm_regres(const void* A, const void* B, void* C, int M, int N, int K, int convention, int layout, const void* s_a,
                   float s_w, int bitnet_epilogue, hipStream_t stream);
int i2_gemv(const void* A, const void* B, void* C, int M, int N, int K, int convention, int layout, const void* s_a,
            float s_w, int out_kind, hipStream_t stream);
int i4_gemv(const void* A, const void* B, void* C, int M, int N, int K, int decode, hipStream_t stream);
int i1_gemv(const void* A, const void* B, void* C, int M, int N, int K, int convention, int layout, hipStream_t stream);
int activation_quant(const void* X, void* Q, void* S, int M, int K, hipStream_t stream);
int mxfp4_quant(const void* W, void* B, void* S, int N, int K, int scale_bias, hipStream_t stream);
int fp16_fp4_gemm_splitk(const void* A, const void* B, void* parts, void* C, int M, int N, int K, int split,
                         int transposed, hipStream_t stream);
int mxfp4_mxfp4_gemm(const void* A, const void* SA, const void* B, const void* SB, const void* Bias, void* C, int M,
                     int N, int K, hipStream_t stream);
int i4_gemm(const void* A, const void* B, void* C, int M, int N, int K, int decode, int a_packed, int transposed,
            hipStream_t stream);

int unpack_qzeros(const void* QZ, void* Z, int N, int groups, int packed, hipStream_t stream);
int mfma_rate(const void* operands, void* out, int dtype, int workgroups, int iters, hipStream_t stream);
int plain_gemm(const void* A, const void* B, void* C, void* workspace, int M, int N, int K, int in_dtype, int out_dtype,
               int trans_A, int trans_B, hipStream_t stream);

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
static int variant_bits(int transposed) { return transposed & ~1; }

// ---- device-resident scratch of the entry point that allocates nothing ---------------------------------
// One copy per GPU, held from the moment the library's code object is loaded on that GPU until the process
// ends.  Host code never uses the array's name as an address: the name is a host-side stand-in, the device
// address comes from hipGetSymbolAddress, once per device with that device current.
constexpr size_t kStaticScratchBytes = DQ_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static void* g_scratch_ptr[kMaxDevices];

// `stream`: when not the null stream, it must belong to the current device (the scratch buffer handed out is the
// current device's copy, the kernels run where the stream lives).
static int scratch_of_current_device(const char* fn, hipStream_t stream, void** out) {
  int device = -1;
  DQ_CHECK_HIP(hipGetDevice(&device));
  if (device < 0 || device >= kMaxDevices) DQ_FAIL("%s: device index %d is beyond the %d this library tracks", fn, device, kMaxDevices);
  if (stream) {
    hipDevice_t stream_device = -1;
    DQ_CHECK_HIP(hipStreamGetDevice(stream, &stream_device));
    if ((int)stream_device != device)
      DQ_FAIL("%s: the stream belongs to device %d but device %d is current; make the stream's device current first", fn,
              (int)stream_device, device);
  }
  if (!g_scratch_ptr[device]) {
    void* ptr = nullptr;
    DQ_CHECK_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (!ptr) DQ_FAIL("%s: the static scratch buffer has no address on device %d", fn, device);
    g_scratch_ptr[device] = ptr;
  }
  *out = g_scratch_ptr[device];
  return 0;
}

static int check_w4_args(const char* fn, const void* B, const void* S, const void* Z, int N, int K, int group, int mode,
                         int layout) {
  if (!B) DQ_FAIL("%s: B is expected to have non-NULL data pointer", fn);
  if (N <= 0 || K <= 0) DQ_FAIL("%s: N and K must be positive (got N=%d K=%d)", fn, N, K);
  if (mode < W4_UNSIGNED || mode >= W4_MODE_COUNT) DQ_FAIL("%s: unknown mode %d", fn, mode);
  if (layout != LAYOUT_PLAIN && layout != LAYOUT_INTERLEAVED) DQ_FAIL("%s: unknown layout %d", fn, layout);
  if (group <= 0 || group % 32 != 0) DQ_FAIL("%s: group must be a positive multiple of 32 (got %d)", fn, group);
  if (K % group != 0) DQ_FAIL("%s: K=%d is not a multiple of group=%d", fn, K, group);
  if (group != K && (group & (group - 1)) != 0)
    DQ_FAIL("%s: group=%d must be a power of two or equal to K", fn, group);
  if (mode >= W4_SCALE && !S) DQ_FAIL("%s: Scale is expected to have non-NULL data pointer for mode %d", fn, mode);
  if (mode >= W4_ZEROS_ORIGINAL && !Z) DQ_FAIL("%s: Zeros is expected to have non-NULL data pointer for mode %d", fn, mode);
  if (!aligned16(B)) DQ_FAIL("%s: B must be 16-byte aligned", fn);
  return 0;
}

}  // namespace dq

using namespace dq;

extern "C" const char* get_last_error(void) { return g_error_buf; }

extern "C" int init(void) {
  g_error_buf[0] = '\0';
  int device = 0;
  DQ_CHECK_HIP(hipGetDevice(&device));
  hipDeviceProp_t prop;
  DQ_CHECK_HIP(hipGetDeviceProperties(&prop, device));
  if (__builtin_strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    DQ_FAIL("init: device %d is %s; this library is built for gfx950 only", device, prop.gcnArchName);
  int max_lds = 0;
  DQ_CHECK_HIP(hipDeviceGetAttribute(&max_lds, hipDeviceAttributeMaxSharedMemoryPerBlock, device));
  if (largest_lds_request() > max_lds)
    DQ_FAIL("Requested dynamic shared memory %d exceeds device limit %d", largest_lds_request(), max_lds);
  void* scratch_ptr = nullptr;
  if (scratch_of_current_device("init", nullptr, &scratch_ptr)) return -1;
  return 0;
}

// ---- the streaming small-batch kernel's default configuration and K split ------------------------------
// Which configuration the default dispatch runs at M rows (see w4a16_stream for the numbering).
static int w4a16_stream_config(int M, int N) {
  // up to 16 rows: 64 weight rows per workgroup and a ring of four stages, whatever N and the group size (N = 28672,
  // K = 6144, 4 rows: 22.8 us against 23.8 with 128 weight rows and six stages, which has no room for the scale
  // slots of groups of 32; K = 8192, group 256: 26.9 against 28.9)
  if (M <= 16) return 3;
  // 128 weight rows per workgroup when that still gives every CU a workgroup, else 64
  const bool wide = N >= 128 * 200;
  // 33 to 48 rows: three blocks of 16 activation rows (40.9 us at N = 28672, K = 8192 against 45.3 us with four)
  return M <= 32 ? (wide ? 1 : 4) : (M <= 48 ? 7 : 6);
}

// Into how many slices of K the streaming kernel's workgroups are split when the matrix has too few rows to give
// every CU a workgroup (N = 4096: 64 workgroups of 64 rows for 256 CUs) and the caller brought a workspace: the
// count that fills the last round of workgroups best, every slice at least 1024 k long.  1: no split.
static int w4a16_stream_split(int M, int N, int K, int group, int mode, int config) {
  if (K % 256 != 0 || ((size_t)M * N) % 4 != 0) return 1;
  const int rows = (config >= 3 && config <= 5) ? 64 : 128;
  const int pass = (config == 0 || config == 3 || config == 5) ? 16 : (config == 1 || config == 4) ? 32 : (config == 7 ? 48 : 64);
  const long wgs = (long)((N + rows - 1) / rows) * ((M + pass - 1) / pass);
  constexpr int kCus = 256;
  if (wgs >= kCus * 5 / 8) return 1;
  // slices start where a chunk of scales (16 bytes of a row: eight groups) starts
  const int steps = K / 256;
  const int unit = (mode >= W4_SCALE && group != K && K / group >= 8 && group > 32) ? group / 32 : 1;
  const int units = (steps + unit - 1) / unit;
  int best = 1;
  double best_fill = (double)wgs / kCus;
  for (int split = 2; split <= 16 && split <= units && steps / split >= 4; ++split) {
    const long total = wgs * split;
    const double fill = (double)total / (double)(kCus * ((total + kCus - 1) / kCus));
    if (fill > best_fill * 1.04) best = split, best_fill = fill;
  }
  return best;
}

// A few hundred activation rows against a matrix that gives the tiled GEMM at most 64 tiles of 256 x 256: the GEMM
// then runs one round of workgroups on a quarter of the CUs at the latency of its ring (about 12 ns per k: N = 4096,
// K = 14336 takes 171 us from 129 to 512 rows), and the streaming kernel in passes of 64 rows is ahead of it (58 us at
// 256 rows, 42 us with K cut in two; N = 8192, K = 8192 at 512 rows: 81 against 114 us; the two meet near 128 tiles).
static bool w4a16_few_tiles(int M, int N, int K) {
  return M <= 1024 && K % 256 == 0 && (long)((M + 255) / 256) * ((N + 255) / 256) <= 64;
}

extern "C" size_t dq_w4a16_workspace_bytes(int M, int N, int K, int group, int mode) {
  if (M < 2 || N <= 0 || K <= 0 || group <= 0 || (M > 128 && !w4a16_few_tiles(M, N, K))) return 0;
  const int split = w4a16_stream_split(M, N, K, group, mode, w4a16_stream_config(M, N));
  return split > 1 ? (size_t)split * M * N * sizeof(float) : 0;
}

static int gemv_w4a16(const char* fn, const void* A, const void* B, const void* Scale, const void* Zeros, void* C, int M, int N,
                      int K, int group, int mode, int layout, int variant, void* workspace, size_t workspace_bytes,
                      dq_stream_t stream) {
  if (!A) DQ_FAIL("%s: A is expected to have non-NULL data pointer", fn);
  if (!C) DQ_FAIL("%s: C is expected to have non-NULL data pointer", fn);
  if (M <= 0) DQ_FAIL("%s: M must be positive (got %d)", fn, M);
  if (check_w4_args(fn, B, Scale, Zeros, N, K, group, mode, layout & ~LAYOUT_FRAGMENTS)) return -1;
  if (K % 128 != 0) DQ_FAIL("%s: K=%d must be a multiple of 128", fn, K);
  if (!aligned16(A) || !aligned16(C)) DQ_FAIL("%s: A and C must be 16-byte aligned", fn);
  // "folded" differs from "original" in the rounding of z * s only; the kernels below that have no folded decoder
  // of their own run "original" for it (tile-exact or fp32 arithmetic, either way inside the folded form's error)
  const int asked_mode = mode;
  if (mode == W4_ZEROS_FOLDED) mode = W4_ZEROS_ORIGINAL;
  if (layout & LAYOUT_FRAGMENTS) {
    // weights re-ordered offline into the matrix instruction's operand order: read by the register-resident
    // small-batch kernel only
    const int rc = (variant < 0 || variant == 44) && M <= 16
                       ? w4a16_regres(A, B, Scale, Zeros, C, M, N, K, group, mode, layout & 1, 4, (hipStream_t)stream)
                       : 1;
    if (rc > 0)
      DQ_FAIL("%s: fragment-ordered weights are read at M <= 16, N %% 16 == 0, K = 2048 / 4096 / 8192, group 128 and every mode "
              "but \"rescale\" only (got M=%d N=%d K=%d group=%d mode=%d)", fn, M, N, K, group, mode);
    return rc;
  }
  // prefill-sized M: the tiled MFMA GEMM (same tile-exact decoders); up to 128 rows, and beyond that against a
  // matrix of few tiles, the streaming kernel below (passes of 64 rows over the weights) is still the faster one.
  // 50: the GEMM whatever M.
  if ((variant == -1 && M > 128 && !w4a16_few_tiles(M, N, K)) || variant == 50) return w4_f16_gemm(A, B, Scale, Zeros, C, M, N, K, group, asked_mode, layout, (hipStream_t)stream);
  // variant < 0: heuristic.  100 + r: the dot2 GEMV kernel with r rows in flight per thread (r = 0: its own
  // choice).  30..37: a configuration of the direct-to-LDS small-batch kernel.  40: the kernel with
  // register-resident activations (M <= 16).  0, 4, 5, 10: a configuration of the tiled MFMA fallback kernel
  // (covers every shape).
  if ((variant >= 40 && variant <= 43) || (variant < 0 && M >= 2 && M <= 16)) {
    // a handful of rows: activations resident in registers (shapes it does not cover fall through).  40: the form
    // that reproduces the fp16 rounding of every weight; 41 and the default: scale and zero point applied per
    // group in fp32, weights fetched row-contiguously and transposed through LDS; 43: the same with the weights
    // fetched in the matrix instruction's layout; 42: that on eight waves with two row blocks in flight
    // ("rescale" always runs the exact form)
    const int rc = w4a16_regres(A, B, Scale, Zeros, C, M, N, K, group, mode, layout, variant == 40 ? 0 : (variant >= 42 ? variant - 40 : 1), (hipStream_t)stream);
    if (rc <= 0) return rc;
    if (variant >= 40) DQ_FAIL("%s: the register-resident kernel does not cover M=%d N=%d K=%d group=%d", fn, M, N, K, group);
  }
  // 70..77: as 30..37 with the zero point folded into one fused multiply-add per weight pair (only "original"
  // differs from the tile-exact form: RNE16(q s - RNE16(z s)) instead of RNE16(RNE16(q - z) s)); the default
  // above 16 rows
  const int folded_mode = mode == W4_ZEROS_ORIGINAL ? W4_ZEROS_FOLDED : mode;
  if (variant >= 70 && variant < 80) {
    const int rc = w4a16_stream(A, B, Scale, Zeros, C, M, N, K, group, folded_mode, layout, variant - 70, 1, nullptr, (hipStream_t)stream);
    if (rc > 0) DQ_FAIL("%s: the streaming small-batch kernel does not cover N=%d K=%d group=%d", fn, N, K, group);
    return rc;
  }
  if (variant >= 30 && variant < 40) {
    const int rc = w4a16_stream(A, B, Scale, Zeros, C, M, N, K, group, asked_mode, layout, variant - 30, 1, nullptr, (hipStream_t)stream);
    if (rc > 0) DQ_FAIL("%s: the streaming small-batch kernel does not cover N=%d K=%d group=%d", fn, N, K, group);
    return rc;
  }
  // one and two rows: the dot2 GEMV (it takes up to four, but from three rows on the streaming kernel below is ahead
  // of it: N = 13824, K = 5120 at 4 rows 13.0 against 19.4 us; N = 28672, K = 6144 22.8 against 32.3)
  if ((variant < 0 && M <= 2) || variant >= 100) {
    const int rc = w4a16_gemv_dot2(A, B, Scale, Zeros, C, M, N, K, group, mode, layout,
                                   variant >= 100 ? variant - 100 : 0, (hipStream_t)stream);
    if (rc <= 0) return rc;
    if (variant >= 100) DQ_FAIL("%s: the dot2 GEMV kernel does not cover M=%d K=%d", fn, M, K);
  }
  if (variant < 0 && M >= 2) {
    const int config = w4a16_stream_config(M, N);
    // the folded zero point shares one rounding of z * s among a group's weights: up to 128 k per group the sum stays
    // well inside the tolerance around the reference's tile, with groups of thousands it need not
    const int stream_mode = group <= 128 ? folded_mode : asked_mode;
    // with a workspace: K split over workgroups where the rows alone leave CUs idle
    // (variant -2, -3, ...: that many slices whatever the heuristic says, for measurements and tests)
    int split = !workspace ? 1 : (variant <= -2 ? -variant : w4a16_stream_split(M, N, K, group, mode, config));
    while (split > 1 && (size_t)split * M * N * sizeof(float) > workspace_bytes) --split;
    const int rc = w4a16_stream(A, B, Scale, Zeros, C, M, N, K, group, stream_mode, layout, config, split, workspace, (hipStream_t)stream);
    if (rc <= 0) return rc;
    // a shape the streaming kernel does not take (K % 256, a group size that is no power of two ...): from 64 rows on
    // the tiled GEMM is ahead of the general fallback (N = 28672, K = 8192, group 64: 142 against 285 us at M = 128)
    if (M >= 64 && K % 64 == 0) return w4_f16_gemm(A, B, Scale, Zeros, C, M, N, K, group, asked_mode, layout, (hipStream_t)stream);
  }
  if (variant < 0 && M > 2 && M <= 4) {  // three and four rows of a shape the streaming kernel does not take
    const int rc = w4a16_gemv_dot2(A, B, Scale, Zeros, C, M, N, K, group, mode, layout, 0, (hipStream_t)stream);
    if (rc <= 0) return rc;
  }
  return w4a16_skinny(A, B, Scale, Zeros, C, M, N, K, group, mode, layout, variant, (hipStream_t)stream);
}

extern "C" int call_dequantize_gemv_w4a16(const void* A, const void* B, const void* Scale, const void* Zeros, void* C,
                                          int M, int N, int K, int group, int mode, int layout, int variant,
                                          dq_stream_t stream) {
  return gemv_w4a16("call_dequantize_gemv_w4a16", A, B, Scale, Zeros, C, M, N, K, group, mode, layout, variant, nullptr, 0, stream);
}

extern "C" int call_dequantize_gemv_w4a16_ws(const void* A, const void* B, const void* Scale, const void* Zeros, void* C,
                                             void* Workspace, size_t workspace_bytes, int M, int N, int K, int group,
                                             int mode, int layout, int variant, dq_stream_t stream) {
  const char* fn = "call_dequantize_gemv_w4a16_ws";
  if (workspace_bytes && !Workspace) DQ_FAIL("%s: Workspace is expected to have non-NULL data pointer", fn);
  if (Workspace && !aligned16(Workspace)) DQ_FAIL("%s: Workspace must be 16-byte aligned", fn);
  return gemv_w4a16(fn, A, B, Scale, Zeros, C, M, N, K, group, mode, layout, variant, workspace_bytes ? Workspace : nullptr,
                    workspace_bytes, stream);
}

extern "C" int call_dequantize_gemv_lowbit(const void* A, const void* B, const void* Scale, const void* Zeros, void* C,
                                           int M, int N, int K, int group, int bits, int convention, int layout,
                                           int zeros_rescale, dq_stream_t stream) {
  const char* fn = "call_dequantize_gemv_lowbit";
  if (!A) DQ_FAIL("%s: A is expected to have non-NULL data pointer", fn);
  if (!B) DQ_FAIL("%s: B is expected to have non-NULL data pointer", fn);
  if (!C) DQ_FAIL("%s: C is expected to have non-NULL data pointer", fn);
  if (bits != 1 && bits != 2) DQ_FAIL("%s: bits must be 1 or 2 (got %d)", fn, bits);
  if (M <= 0 || N <= 0 || K <= 0) DQ_FAIL("%s: M, N, K must be positive (got %d %d %d)", fn, M, N, K);
  if (M > 64) DQ_FAIL("%s: M=%d is beyond the decode batch this kernel is built for (64)", fn, M);
  const int chunk = 128 / bits;  // codes in 16 bytes
  if (K % chunk != 0) DQ_FAIL("%s: K=%d must be a multiple of %d", fn, K, chunk);
  if (K > 32768) DQ_FAIL("%s: K=%d is beyond the 32768 this kernel is built for", fn, K);
  if (convention < I2_UNSIGNED || convention > I2_TWOS) DQ_FAIL("%s: unknown code convention %d", fn, convention);
  if (layout != LAYOUT_PLAIN && layout != LAYOUT_INTERLEAVED) DQ_FAIL("%s: unknown weight layout %d", fn, layout);
  if (Zeros && !Scale) DQ_FAIL("%s: Zeros without Scale", fn);
  if (Scale) {
    if (group <= 0 || group % chunk != 0 || K % group != 0)
      DQ_FAIL("%s: group=%d must be a multiple of %d that divides K=%d", fn, group, chunk, K);
  } else {
    group = K;
  }
  if (!aligned16(A) || !aligned16(B)) DQ_FAIL("%s: A and B must be 16-byte aligned", fn);
  const int rc = wlow_gemv(A, B, Scale, Zeros, C, M, N, K, group, bits, convention, layout, zeros_rescale, (hipStream_t)stream);
  if (rc > 0) DQ_FAIL("%s: shape M=%d N=%d K=%d is not covered", fn, M, N, K);
  return rc;
}

extern "C" int call_dequantize_w4(const void* B, const void* Scale, const void* Zeros, void* W, int N, int K, int group,
                                  int mode, int layout, dq_stream_t stream) {
  const char* fn = "call_dequantize_w4";
  if (!W) DQ_FAIL("%s: W is expected to have non-NULL data pointer", fn);
  if (check_w4_args(fn, B, Scale, Zeros, N, K, group, mode, layout & ~DECODER_CONVERTER)) return -1;
  if (K % 8 != 0) DQ_FAIL("%s: K=%d must be a multiple of 8", fn, K);
  if (!aligned16(W)) DQ_FAIL("%s: W must be 16-byte aligned", fn);
  return w4_dequant(B, Scale, Zeros, W, N, K, group, mode, layout, (hipStream_t)stream);
}

extern "C" int call_unpack_qzeros(const void* QZeros, void* Zeros, int N, int groups, int format, dq_stream_t stream) {
  const char* fn = "call_unpack_qzeros";
  if (!QZeros) DQ_FAIL("%s: QZeros is expected to have non-NULL data pointer", fn);
  if (!Zeros) DQ_FAIL("%s: Zeros is expected to have non-NULL data pointer", fn);
  if (N <= 0 || groups <= 0) DQ_FAIL("%s: N and groups must be positive (got %d, %d)", fn, N, groups);
  if (format != DQ_QZEROS_INT16 && format != DQ_QZEROS_PACKED4) DQ_FAIL("%s: unknown qzeros format %d", fn, format);
  if (format == DQ_QZEROS_INT16 && ((uintptr_t)QZeros & 1) != 0) DQ_FAIL("%s: int16 QZeros must be 2-byte aligned", fn);
  if (((uintptr_t)Zeros & 1) != 0) DQ_FAIL("%s: Zeros must be 2-byte aligned", fn);
  return unpack_qzeros(QZeros, Zeros, N, groups, format == DQ_QZEROS_PACKED4, (hipStream_t)stream);
}

extern "C" int call_dequant_gemm_bf16_mxfp4(const void* A, const void* B, const void* Scale, const void* Bias, void* C,
                                            int M, int N, int K, int scale_size, int fp4_format, int scale_bias,
                                            dq_stream_t stream) {
  const char* fn = "call_dequant_gemm_bf16_mxfp4";
  if (!A) DQ_FAIL("%s: A is expected to have non-NULL data pointer", fn);
  if (!B) DQ_FAIL("%s: B is expected to have non-NULL data pointer", fn);
  if (!Scale) DQ_FAIL("%s: Scale is expected to have non-NULL data pointer", fn);
  if (!C) DQ_FAIL("%s: C is expected to have non-NULL data pointer", fn);
  if (M <= 0 || N <= 0 || K <= 0) DQ_FAIL("%s: M, N, K must be positive (got %d %d %d)", fn, M, N, K);
  if (scale_size != 32) DQ_FAIL("%s: scale_size must be 32 (got %d)", fn, scale_size);
  if (K % 64 != 0) DQ_FAIL("%s: K=%d must be a multiple of 64", fn, K);
  if (fp4_format < FP4_E2M1 || fp4_format > FP4_TWIDDLING) DQ_FAIL("%s: unknown fp4 format %d", fn, fp4_format);
  if (scale_bias < 0 || scale_bias > 255) DQ_FAIL("%s: scale_bias must be in 0..255 (got %d)", fn, scale_bias);
  if (!aligned16(A) || !aligned16(B) || !aligned16(C) || (Bias && !aligned16(Bias)))
    DQ_FAIL("%s: A, B, Bias and C must be 16-byte aligned", fn);
  // a decode batch: activations resident in registers, the weights streamed once per 16 rows (K % 64 == 0, beyond 8192 K % 128 == 0;
  // beyond 16 rows while the passes stay ahead of the tiled kernel: the kernel's launcher decides)
  if (M <= 128) {
    const int rc = mxfp4_gemm_regres(A, B, Scale, Bias, C, M, N, K, fp4_format, scale_bias, 128, (hipStream_t)stream);
    if (rc <= 0) return rc;
  }
  return mxfp4_gemm(A, B, Scale, Bias, C, M, N, K, fp4_format, scale_bias, (hipStream_t)stream);
}

static int check_gemm_args(const char* fn, const void* A, const void* B, const void* C, int M, int N, int K, int kmult) {
  if (!A) DQ_FAIL("%s: A is expected to have non-NULL data pointer", fn);
  if (!B) DQ_FAIL("%s: B is expected to have non-NULL data pointer", fn);
  if (!C) DQ_FAIL("%s: C is expected to have non-NULL data pointer", fn);
  if (M <= 0 || N <= 0 || K <= 0) DQ_FAIL("%s: M, N, K must be positive (got %d %d %d)", fn, M, N, K);
  if (K % kmult != 0) DQ_FAIL("%s: K=%d must be a multiple of %d", fn, K, kmult);
  if (!aligned16(A) || !aligned16(B) || !aligned16(C)) DQ_FAIL("%s: A, B and C must be 16-byte aligned", fn);
  return 0;
}

extern "C" int call_dequant_gemm_bf16_fp4(const void* A, const void* B, void* C, int M, int N, int K, int fp4_format,
                                         dq_stream_t stream) {
  const char* fn = "call_dequant_gemm_bf16_fp4";
  if (!A) DQ_FAIL("%s: A is expected to have non-NULL data pointer", fn);
  if (!B) DQ_FAIL("%s: B is expected to have non-NULL data pointer", fn);
  if (!C) DQ_FAIL("%s: C is expected to have non-NULL data pointer", fn);
  if (M <= 0 || N <= 0 || K <= 0) DQ_FAIL("%s: M, N, K must be positive (got %d %d %d)", fn, M, N, K);
  if (K % 64 != 0) DQ_FAIL("%s: K=%d must be a multiple of 64", fn, K);
  if (fp4_format < FP4_E2M1 || fp4_format > FP4_TWIDDLING) DQ_FAIL("%s: unknown fp4 format %d", fn, fp4_format);
  if (!aligned16(A) || !aligned16(B) || !aligned16(C)) DQ_FAIL("%s: A, B and C must be 16-byte aligned", fn);
  return bf16_fp4_gemm(A, B, C, M, N, K, fp4_format, (hipStream_t)stream);
}

extern "C" int call_dequant_gemm_fp16_fp4(const void* A, const void* B, void* C, int M, int N, int K, int transposed,
                                          dq_stream_t stream) {
  if (check_gemm_args("call_dequant_gemm_fp16_fp4", A, B, C, M, N, K, 64)) return -1;
  return fp16_fp4_gemm(A, B, C, M, N, K, transposed, (hipStream_t)stream);
}

extern "C" int call_dequant_gemm_fp16_fp4_splitk(const void* A, const void* B, void* SplitC, void* C, int M, int N, int K,
                                                 int split, int transposed, dq_stream_t stream) {
  const char* fn = "call_dequant_gemm_fp16_fp4_splitk";
  if (check_gemm_args(fn, A, B, C, M, N, K, 64)) return -1;
  if (split < 1 || split > 64) DQ_FAIL("%s: split=%d must be in 1..64", fn, split);
  if (K % (64 * split) != 0) DQ_FAIL("%s: K=%d must be a multiple of 64 * split (split=%d)", fn, K, split);
  if (split == 1) return fp16_fp4_gemm(A, B, C, M, N, K, transposed, (hipStream_t)stream);
  if (!SplitC) DQ_FAIL("%s: SplitC is expected to have non-NULL data pointer", fn);
  if (!aligned16(SplitC)) DQ_FAIL("%s: SplitC must be 16-byte aligned", fn);
  if (((size_t)M * N) % 8 != 0) DQ_FAIL("%s: M * N must be a multiple of 8 when split > 1 (got %d x %d)", fn, M, N);
  return fp16_fp4_gemm_splitk(A, B, SplitC, C, M, N, K, split, transposed, (hipStream_t)stream);
}

extern "C" int call_dequant_gemm_fp16_fp4_splitk_static(const void* A, const void* B, void* C, int M, int N, int K,
                                                        int split, int transposed, dq_stream_t stream) {
  const char* fn = "call_dequant_gemm_fp16_fp4_splitk_static";
  if (check_gemm_args(fn, A, B, C, M, N, K, 64)) return -1;
  if (split < 1 || split > 64) DQ_FAIL("%s: split=%d must be in 1..64", fn, split);
  if (K % (64 * split) != 0) DQ_FAIL("%s: K=%d must be a multiple of 64 * split (split=%d)", fn, K, split);
  if (split == 1) return fp16_fp4_gemm(A, B, C, M, N, K, transposed, (hipStream_t)stream);
  if (((size_t)M * N) % 8 != 0) DQ_FAIL("%s: M * N must be a multiple of 8 when split > 1 (got %d x %d)", fn, M, N);
  const size_t need = (size_t)split * (size_t)M * (size_t)N * sizeof(half_t);
  if (need > kStaticScratchBytes)
    DQ_FAIL("%s: split * M * N fp16 partial results need %zu bytes, the static scratch buffer holds %zu; use "
            "call_dequant_gemm_fp16_fp4_splitk with a buffer of your own", fn, need, kStaticScratchBytes);
  void* parts = nullptr;
  if (scratch_of_current_device(fn, (hipStream_t)stream, &parts)) return -1;
  // every partial result the summing kernel reads is written by its slice's workgroups first, in stream order:
  // nothing has to start at zero, whatever the last call left behind
  return fp16_fp4_gemm_splitk(A, B, parts, C, M, N, K, split, transposed, (hipStream_t)stream);
}

extern "C" int call_dequant_gemm_w4_fp16(const void* A, const void* B, const void* Scale, const void* Zeros, void* C,
                                         int M, int N, int K, int group, int mode, int layout, dq_stream_t stream) {
  const char* fn = "call_dequant_gemm_w4_fp16";
  if (check_gemm_args(fn, A, B, C, M, N, K, 64)) return -1;
  if (check_w4_args(fn, B, Scale, Zeros, N, K, group, mode, layout)) return -1;
  return w4_f16_gemm(A, B, Scale, Zeros, C, M, N, K, group, mode, layout, (hipStream_t)stream);
}

extern "C" int call_gemm_int8xint2(const void* A, const void* B, void* C, int M, int N, int K, int convention,
                                   int layout, const void* s_a, float s_w, int out_kind, dq_stream_t stream) {
  const char* fn = "call_gemm_int8xint2";
  if (check_gemm_args(fn, A, B, C, M, N, K, 128)) return -1;
  if (convention < I2_UNSIGNED || convention > I2_TWOS) DQ_FAIL("%s: unknown code convention %d", fn, convention);
  const int word_layout = layout & ~LAYOUT_FRAGMENTS;
  if (word_layout != LAYOUT_PLAIN && word_layout != LAYOUT_INTERLEAVED) DQ_FAIL("%s: unknown weight layout %d", fn, layout);
  // bits 4 and 5 of out_kind name a kernel (tests and measurements): K sliced over the waves / the tiled GEMM
  constexpr int kChoices = DQ_I2_KERNEL_KSLICED | DQ_I2_KERNEL_TILED | DQ_I2_KERNEL_RESIDENT;
  int kernel_choice = out_kind & kChoices;
  out_kind &= ~kChoices;
  if (out_kind != 0 && out_kind != 1) DQ_FAIL("%s: out_kind must be 0 (int32) or 1 (fp16 BitLinear epilogue)", fn);
  if (kernel_choice & (kernel_choice - 1)) DQ_FAIL("%s: out_kind names two kernels", fn);
  if (out_kind == 1 && !s_a) DQ_FAIL("%s: s_a is expected to have non-NULL data pointer", fn);
  if (out_kind == 1 && !(s_w != 0.f)) DQ_FAIL("%s: s_w must be non-zero", fn);
  const bool frag = (layout & LAYOUT_FRAGMENTS) != 0;
  if (kernel_choice == DQ_I2_KERNEL_KSLICED) {
    const int rc = i2_gemm_kslice(A, B, C, M, N, K, convention, layout, s_a, s_w, out_kind, 1, (hipStream_t)stream);
    if (rc > 0) DQ_FAIL("%s: the K-sliced kernel needs K %% 2048 == 0, K < 131072 and operands below 4 GiB (got M=%d N=%d K=%d)", fn, M, N, K);
    return rc;
  }
  if (kernel_choice == DQ_I2_KERNEL_RESIDENT) {
    const int rc = i2_gemm_regres(A, B, C, M, N, K, convention, layout, s_a, s_w, out_kind, (hipStream_t)stream);
    if (rc > 0) DQ_FAIL("%s: the register-resident kernel needs M <= 32 (on matrices of few rows M <= 128) and K %% 256 == 0 (got M=%d N=%d K=%d)", fn, M, N, K);
    return rc;
  }
  // 4 to 32 rows: activations resident in registers, weights streamed once (at 4 rows ahead of the dot-product kernel
  // on fragment-ordered weights, N = 28672, K = 8192: 14.8 against 25.2 us, and on row-major ones from about 6000
  // weight rows on: N = 11008, K = 4096 7.3 against 8.7 us, N = 3072, K = 8192 8.6 against 7.1)
  const bool four_rows_resident = frag || N >= 6144 || (size_t)M * K > 32768;
  if ((M > 4 || (M == 4 && four_rows_resident)) && M <= 128 && !kernel_choice) {  // beyond 32 rows: on small matrices only (the kernel says which)
    const int rc = i2_gemm_regres(A, B, C, M, N, K, convention, layout, s_a, s_w, out_kind, (hipStream_t)stream);
    if (rc <= 0) return rc;
  }
  if (M <= 4 && !kernel_choice) {  // decode: the streaming dot4 kernel (row-major or fragment-ordered weights)
    const int rc = i2_gemv(A, B, C, M, N, K, convention, layout, s_a, s_w, out_kind, (hipStream_t)stream);
    if (rc <= 0) return rc;
  }
  if (M <= 4 && !kernel_choice) {  // one to four rows of a shape the dot-product kernel does not take
    const int rc = i2_gemm_regres(A, B, C, M, N, K, convention, layout, s_a, s_w, out_kind, (hipStream_t)stream);
    if (rc <= 0) return rc;
  }
  if (!kernel_choice) {  // a few hundred rows: K sliced over the waves of a workgroup
    const int rc = i2_gemm_kslice(A, B, C, M, N, K, convention, layout, s_a, s_w, out_kind, 0, (hipStream_t)stream);
    if (rc <= 0) return rc;
  }
  const int rc = i2_gemm(A, B, C, M, N, K, convention, layout, s_a, s_w, out_kind, (hipStream_t)stream);
  if (rc <= 0 || !frag) return rc;
  // Fragment-ordered weights are read by the decode kernel, the K-sliced kernel and the direct-to-LDS tiled kernel;
  // a shape the tiled one does not take (too few tiles) goes to the K-sliced kernel whatever its size.
  if (kernel_choice == DQ_I2_KERNEL_TILED)
    DQ_FAIL("%s: the tiled kernel reads fragment-ordered weights from 160 tiles of 128 x 256 on and K %% 256 == 0 (got M=%d N=%d K=%d)", fn, M, N, K);
  const int rck = i2_gemm_kslice(A, B, C, M, N, K, convention, layout, s_a, s_w, out_kind, 1, (hipStream_t)stream);
  if (rck > 0)
    DQ_FAIL("%s: fragment-ordered weights: no kernel takes M=%d N=%d K=%d (decode: M <= 4 and M * K <= 32768; register-resident: "
            "M <= 32, or 128 on a matrix of few rows, and K %% 256 == 0; K-sliced: K %% 2048 == 0; tiled: 160 tiles of "
            "128 x 256 and K %% 256 == 0)", fn, M, N, K);
  return rck;
}

extern "C" int call_bitnet_activation_quant(const void* X, void* Q, void* S, int M, int K, dq_stream_t stream) {
  const char* fn = "call_bitnet_activation_quant";
  if (!X) DQ_FAIL("%s: X is expected to have non-NULL data pointer", fn);
  if (!Q) DQ_FAIL("%s: Q is expected to have non-NULL data pointer", fn);
  if (!S) DQ_FAIL("%s: S is expected to have non-NULL data pointer", fn);
  if (M <= 0 || K <= 0) DQ_FAIL("%s: M and K must be positive (got %d, %d)", fn, M, K);
  if (K % 8 != 0) DQ_FAIL("%s: K=%d must be a multiple of 8", fn, K);
  if (!aligned16(X) || ((uintptr_t)Q & 7) != 0) DQ_FAIL("%s: X must be 16-byte and Q 8-byte aligned", fn);
  return activation_quant(X, Q, S, M, K, (hipStream_t)stream);
}

extern "C" int call_quantize_bf16_mxfp4(const void* W, void* B, void* Scale, int N, int K, int scale_bias,
                                        dq_stream_t stream) {
  const char* fn = "call_quantize_bf16_mxfp4";
  if (!W) DQ_FAIL("%s: W is expected to have non-NULL data pointer", fn);
  if (!B) DQ_FAIL("%s: B is expected to have non-NULL data pointer", fn);
  if (!Scale) DQ_FAIL("%s: Scale is expected to have non-NULL data pointer", fn);
  if (N <= 0 || K <= 0) DQ_FAIL("%s: N and K must be positive (got %d, %d)", fn, N, K);
  if (K % 32 != 0) DQ_FAIL("%s: K=%d must be a multiple of 32 (one scale per 32 elements)", fn, K);
  if (scale_bias < 0 || scale_bias > 254) DQ_FAIL("%s: scale_bias=%d must be in 0..254", fn, scale_bias);
  if (!aligned16(W) || ((uintptr_t)B & 3) != 0) DQ_FAIL("%s: W must be 16-byte and B 4-byte aligned", fn);
  return mxfp4_quant(W, B, Scale, N, K, scale_bias, (hipStream_t)stream);
}

extern "C" int call_gemm_mxfp4_mxfp4(const void* A, const void* B, const void* ScaleA, const void* ScaleB,
                                     const void* Bias, void* C, int M, int N, int K, dq_stream_t stream) {
  const char* fn = "call_gemm_mxfp4_mxfp4";
  if (!A) DQ_FAIL("%s: A is expected to have non-NULL data pointer", fn);
  if (!ScaleA) DQ_FAIL("%s: ScaleA is expected to have non-NULL data pointer", fn);
  if (!B) DQ_FAIL("%s: B is expected to have non-NULL data pointer", fn);
  if (!ScaleB) DQ_FAIL("%s: ScaleB is expected to have non-NULL data pointer", fn);
  if (!C) DQ_FAIL("%s: C is expected to have non-NULL data pointer", fn);
  if (M <= 0 || N <= 0 || K <= 0) DQ_FAIL("%s: M, N, K must be positive (got %d %d %d)", fn, M, N, K);
  if (!aligned16(A) || !aligned16(B) || !aligned16(C) || (Bias && !aligned16(Bias)))
    DQ_FAIL("%s: A, B, Bias and C must be 16-byte aligned", fn);
  if (((uintptr_t)ScaleA & 3) != 0 || ((uintptr_t)ScaleB & 3) != 0) DQ_FAIL("%s: ScaleA and ScaleB must be 4-byte aligned", fn);
  return mxfp4_mxfp4_gemm(A, ScaleA, B, ScaleB, Bias, C, M, N, K, (hipStream_t)stream);
}

extern "C" int call_gemm_plain(const void* A, const void* B, void* C, void* Workspace, int M, int N, int K, int in_dtype,
                               int out_dtype, int trans_A, int trans_B, dq_stream_t stream) {
  const char* fn = "call_gemm_plain";
  if (in_dtype != DQ_DT_F16 && in_dtype != DQ_DT_BF16 && in_dtype != DQ_DT_I8)
    DQ_FAIL("%s: in_dtype must be DQ_DT_F16, DQ_DT_BF16 or DQ_DT_I8 (got %d)", fn, in_dtype);
  const bool ok_out = in_dtype == DQ_DT_I8 ? out_dtype == DQ_DT_I32 : (out_dtype == in_dtype || out_dtype == DQ_DT_F32);
  if (!ok_out) DQ_FAIL("%s: out_dtype %d does not go with in_dtype %d (int8 -> int32; fp16 / bf16 -> the same or fp32)", fn, out_dtype, in_dtype);
  if (check_gemm_args(fn, A, B, C, M, N, K, in_dtype == DQ_DT_I8 ? 128 : 64)) return -1;
  if ((trans_A || !trans_B) && !Workspace) DQ_FAIL("%s: Workspace is expected to have non-NULL data pointer when trans_A or not trans_B", fn);
  if (Workspace && !aligned16(Workspace)) DQ_FAIL("%s: Workspace must be 16-byte aligned", fn);
  return plain_gemm(A, B, C, Workspace, M, N, K, in_dtype, out_dtype, trans_A != 0, trans_B != 0, (hipStream_t)stream);
}

extern "C" int call_mfma_rate(const void* Operands, void* Out, int in_dtype, int workgroups, int iters, dq_stream_t stream) {
  const char* fn = "call_mfma_rate";
  if (!Operands || !Out) DQ_FAIL("%s: Operands and Out are expected to have non-NULL data pointers", fn);
  if (!aligned16(Operands) || !aligned16(Out)) DQ_FAIL("%s: Operands and Out must be 16-byte aligned", fn);
  if (in_dtype != DQ_DT_F16 && in_dtype != DQ_DT_BF16 && in_dtype != DQ_DT_I8 && in_dtype != DQ_DT_FP4)
    DQ_FAIL("%s: in_dtype must be DQ_DT_F16, DQ_DT_BF16, DQ_DT_I8 or DQ_DT_FP4 (got %d)", fn, in_dtype);
  if (workgroups < 1 || workgroups > 65536 || iters < 1) DQ_FAIL("%s: workgroups=%d (1..65536) and iters=%d (>= 1) out of range", fn, workgroups, iters);
  return mfma_rate(Operands, Out, in_dtype, workgroups, iters, (hipStream_t)stream);
}

extern "C" int call_gemm_int8xint4(const void* A, const void* B, void* C, int M, int N, int K, int decode,
                                   int a_packed, int transposed, dq_stream_t stream) {
  const char* fn = "call_gemm_int8xint4";
  if (check_gemm_args(fn, A, B, C, M, N, K, 128)) return -1;
  if (decode < DQ_I4_UNSIGNED || decode > DQ_I2_TO_I4) DQ_FAIL("%s: unknown decode %d", fn, decode);
  if (decode == DQ_I2_TO_I4 && !a_packed) DQ_FAIL("%s: decode DQ_I2_TO_I4 (2-bit codes to int4) goes with a packed int4 A", fn);
  if (a_packed && decode != DQ_I4_TWOS && decode != DQ_I2_TO_I4)
    DQ_FAIL("%s: a packed A goes with decode DQ_I4_TWOS or DQ_I2_TO_I4 only (got %d)", fn, decode);
  if (a_packed && K >= 131072) DQ_FAIL("%s: K=%d is beyond the 131071 that keep the int32 accumulation of a packed A exact", fn, K);
  // decode batches: the streaming dot-product kernel (Ct[N,1] and C[1,N] are the same bytes)
  if (!a_packed && M <= 4 && (!transposed || M == 1) && !(variant_bits(transposed) & DQ_I4_KERNEL_TILED)) {
    const int rc = i4_gemv(A, B, C, M, N, K, decode, (hipStream_t)stream);
    if (rc <= 0) return rc;
  }
  return i4_gemm(A, B, C, M, N, K, decode, a_packed, transposed & 1, (hipStream_t)stream);
}

extern "C" int call_gemv_int8xint1(const void* A, const void* B, void* C, int M, int N, int K, int convention, int layout,
                                   dq_stream_t stream) {
  const char* fn = "call_gemv_int8xint1";
  if (check_gemm_args(fn, A, B, C, M, N, K, 128)) return -1;
  if (convention < I2_UNSIGNED || convention > I2_TWOS) DQ_FAIL("%s: unknown code convention %d", fn, convention);
  if (layout != LAYOUT_PLAIN && layout != LAYOUT_INTERLEAVED) DQ_FAIL("%s: unknown weight layout %d", fn, layout);
  if (M > 4) DQ_FAIL("%s: M=%d is beyond the decode batch (4) this kernel is built for", fn, M);
  if (K > 65536) DQ_FAIL("%s: K=%d is beyond the 65536 this kernel is built for", fn, K);
  // the activations of two rows at a time fit a thread's registers
  for (int m0 = 0; m0 < M; m0 += 2) {
    const int rows = M - m0 < 2 ? M - m0 : 2;
    const int rc = i1_gemv((const int8_t*)A + (size_t)m0 * K, B, (int32_t*)C + (size_t)m0 * N, rows, N, K, convention, layout,
                           (hipStream_t)stream);
    if (rc > 0) DQ_FAIL("%s: shape M=%d N=%d K=%d is not covered", fn, M, N, K);
    if (rc < 0) return rc;
  }
  return 0;
}
