/* C-ABI of libdqgemm.so: hand-written gfx950 kernels for the dequantize-GEMM path.
 *
 * Convention (the one the reference's kernel adapter generates for every JIT kernel,
 * tilelang/jit/adapter/wrapper.py:59-85,719-736): plain device pointers, explicit sizes,
 * the HIP stream as the last argument, return 0 on success and -1 on error with the
 * message available from get_last_error().  Launches are asynchronous on `stream`; no
 * entry point allocates, frees or synchronises.  The caller owns every buffer.
 *
 * All matrices are row-major and contiguous.  Packed weights keep the examples' layout:
 * B[N, K*bits/8] bytes, low field = lowest k.
 */
#ifndef DQGEMM_H_
#define DQGEMM_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* dq_stream_t; /* hipStream_t */

/* ---- library ------------------------------------------------------------------------ */

/* Replaces `int init()` of the generated host stub (tilelang/jit/adapter/wrapper.py:75-85,
 * :33-57): clears the error buffer, checks a gfx950 device is current and that the
 * largest dynamic-LDS request of any kernel fits the device limit. */
int init(void);

/* Replaces `const char* get_last_error()` (tilelang/jit/adapter/wrapper.py:71-73):
 * static 1024-byte buffer, not thread safe. */
const char* get_last_error(void);

/* ---- enums (int arguments below) ------------------------------------------------------ */

/* file names below are under examples/dequantize_gemm/quantize/ */
enum dq_w4_mode {
  DQ_W4_UNSIGNED = 0,       /* w = q                      quantization.py:310-318, lop3.py:35-39 (i4u) */
  DQ_W4_SIGNED = 1,         /* w = sext4(q)               quantization.py:333-343                      */
  DQ_W4_OFFSET8 = 2,        /* w = q - 8                  quantization.py:298-307, lop3.py:29-33 (i4s) */
  DQ_W4_SCALE = 3,          /* w = rne16((q-8)*s)         lop3.py:41-75 (i4s_scale)                    */
  DQ_W4_USCALE = 4,         /* w = rne16(q*s)             lop3.py:77-81 (i4u_scale)                    */
  DQ_W4_ZEROS_ORIGINAL = 5, /* w = rne16(rne16(q-z)*s)    lop3.py:136-176, quantization.py:321-330     */
  DQ_W4_ZEROS_RESCALE = 6,  /* w = rne16(fma(q,s,-z))     lop3.py:233-271                              */
  DQ_W4_ZEROS_FOLDED = 7    /* w = rne16(fma(q,s,-rne16(z*s))): the "original" formula (q-z)*s with the zero point
                               folded into one fused multiply-add per weight.  No counterpart in the reference: it
                               differs from DQ_W4_ZEROS_ORIGINAL by the rounding of z*s (relative 2^-11 of z*s, shared
                               by the weights of a group) and saves four instructions per packed word.  The batch
                               kernels of call_dequantize_gemv_w4a16 above 16 rows use it for DQ_W4_ZEROS_ORIGINAL
                               when `variant` < 0 (results stay inside rtol = atol = 1e-2 of the reference); the tiled
                               GEMM and call_dequantize_w4 use it only when asked for by this value.             */
};

enum dq_w4_layout {
  DQ_LAYOUT_PLAIN = 0,      /* nibble e of each 32-bit word is element e                         */
  DQ_LAYOUT_INTERLEAVED = 1, /* words pre-permuted by interleave_weight (.., 4, "float16") for uint4,
                               (.., 2, "int8") for 2-bit codes,
                               examples/dequantize_gemm/quantize/utils.py:71-125              */
  DQ_LAYOUT_FRAGMENTS = 2    /* flag, added to one of the two above (call_dequantize_gemv_w4a16 only, M <= 16): the
                               16-byte pieces of B re-ordered offline into the matrix instruction's operand order,
                               B[N/16][K/128][64][16 bytes], entry 16 g + r of a 128-k chunk = bytes 16 g .. 16 g + 15
                               of that chunk of row r of the block.  The role of the weight transform of
                               examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:136-354
                               (B[N/16][K/16][16][8], micro-tiles of the NVIDIA instruction), for this chip's 16x16x32
                               instruction; its BitBLAS permutation inside a tile is third-party and not reproduced.
                               call_gemm_int8xint2 takes the flag too, with the order of the 32x32x32 int8 instruction:
                               B[(N+31)/32][K/128][64][16 bytes], entry 32 h + r of a 128-k chunk = bytes 16 h .. + 15
                               of that chunk (32 bytes) of row r of the block of 32, rows past N zero; read by the
                               decode kernel (M <= 4, M * K <= 32768), the K-sliced kernel (K % 2048 == 0) and the
                               direct-to-LDS tiled kernel (from 160 tiles of 128 x 256 on).                          */
};

/* Flag for the `layout` of call_dequantize_w4 only: decode with the fp8-converter decoder (a nibble in a byte read as
 * OCP e4m3 is q * 2^-9; the streaming batch kernel and the tiled W4 GEMM decode this way) instead of the mantissa-mask
 * decoder of the other kernels.  The two produce the same bits in every mode; the flag exists so that a test can
 * see both. */
#define DQ_DECODER_CONVERTER 4

/* ---- W4A16 ---------------------------------------------------------------------------- */

/* C[M,N] fp16 = A[M,K] fp16 . dequant(B[N,K/2], Scale[N,K/group], Zeros[N,K/group])^T,
 * fp32 accumulation.  Replaces `call(A, B, C, stream)` of the kernel generated from
 * examples/dequantize_gemm/example_dequant_gemv_fp16xint4.py:83-153 (M = 1) and its
 * batched use (decode kernels up to M = 128; larger M goes to the tiled GEMM of call_dequant_gemm_w4_fp16).
 * Requires K % 128 == 0, group % 32 == 0, K % group == 0 (group = K when there is one
 * scale per row).  Scale / Zeros may be NULL for modes that do not read them.
 * `variant` < 0 selects the kernel configuration heuristically. */
int call_dequantize_gemv_w4a16(const void* A, const void* B, const void* Scale, const void* Zeros, void* C, int M,
                               int N, int K, int group, int mode, int layout, int variant, dq_stream_t stream);

/* The same product with a workspace the kernels may use for partial sums.  The reference's counterpart is the
 * split-K form of its dequantize GEMM (examples/dequantize_gemm/example_dequant_gemm_fp4_hopper.py:130-186, SplitC
 * allocated inside the kernel function); here the caller brings the buffer.  A matrix with few rows and a long K
 * (N = 4096, K = 14336: 64 workgroups of 64 rows for 256 CUs) leaves most of the chip idle at 2 <= M <= 128; with a
 * workspace of dq_w4a16_workspace_bytes(M, N, K, group, mode) bytes the default dispatch (`variant` < 0) cuts K into
 * up to 16 slices, one workgroup each, writes their fp32 sums to the workspace and adds them in slice order in a
 * second kernel: results do not depend on timing and stay within rounding of the unsplit kernel's.  A smaller
 * workspace lowers the slice count, NULL / 0 bytes is call_dequantize_gemv_w4a16.  Workspace: 16-byte aligned,
 * contents undefined afterwards, not to be shared by calls that overlap in time. */
size_t dq_w4a16_workspace_bytes(int M, int N, int K, int group, int mode);
int call_dequantize_gemv_w4a16_ws(const void* A, const void* B, const void* Scale, const void* Zeros, void* C,
                                  void* Workspace, size_t workspace_bytes, int M, int N, int K, int group, int mode,
                                  int layout, int variant, dq_stream_t stream);

/* W[N,K] fp16 = dequant(B, Scale, Zeros): the dequantised weight tile with the same
 * device decoder the GEMV/GEMM kernels use.  Replaces the `_convert_test`-style kernels
 * of the examples (examples/dequantize_gemm/example_dequant_gemm_w4a8.py:36-65). */
int call_dequantize_w4(const void* B, const void* Scale, const void* Zeros, void* W, int N, int K, int group,
                       int mode, int layout, dq_stream_t stream);

enum dq_qzeros_format {
  DQ_QZEROS_INT16 = 0,  /* QZeros[N, groups] int16, one zero point per group: what decode_i4u_to_f16_scale_zeros_quantized
                           reads (`int16_t zero_r`, examples/dequantize_gemm/quantize/lop3.py:339-341).  The reference
                           folds it as `0xe400 | zero_r`, which means -(1024 + qz) for 0 <= qz <= 1023 only: that is the
                           range with reference parity.  Values outside it are taken as the integers they are (the
                           reference gives them no meaning).                                                            */
  DQ_QZEROS_PACKED4 = 1 /* QZeros[N, ceil(groups / 2)] bytes, 4-bit zero points, group g in bits 4 (g % 2) of byte g / 2.
                           The tensor shape and the order of the groups inside a row are THIS LIBRARY'S convention: the
                           reference shows only the device-side extraction `(qzeros >> (group_offset * 4)) & 0xf` from
                           two storage words (the _offset variant, lop3.py:367-390) and defines no host-side tensor.    */
};

/* Zeros[N, groups] fp16 = the integer zero points of the "quantized" zeros mode.  The reference's decoder computes
 * (q - qz) exactly in fp16 by folding qz into its magic number and multiplies by the scale once
 * (examples/dequantize_gemm/quantize/lop3.py:326-363, 367-420); DQ_W4_ZEROS_ORIGINAL fed with the fp16 copy of qz
 * returns the same bits, because fp16(qz) and q - fp16(qz) are exact.  So a caller with integer zero points converts
 * them with this call (once for static weights, or per call) and uses DQ_W4_ZEROS_ORIGINAL. */
int call_unpack_qzeros(const void* QZeros, void* Zeros, int N, int groups, int format, dq_stream_t stream);

/* ---- MXFP4 x bf16 ------------------------------------------------------------------------ */

enum dq_fp4_format {
  DQ_FP4_E2M1 = 0,     /* OCP e2m1, plain low-first nibbles: examples/dequantize_gemm/quantize/nvfp4.py:17-34,
                          quantize/mxfp.py:136-157, src/tl_templates/hip/hip_fp4.h:18-57                         */
  DQ_FP4_SIMPLE = 1,   /* bf16 bits (s<<15)|((E+126)<<7)|(m<<6) for every E: examples/dequantize_gemm/
                          dequantize_utils.py:57-84, example_dequant_gemm_bf16_mxfp4_cdna4.py:26-41             */
  DQ_FP4_TWIDDLING = 2 /* e2m1 in the 16-bit twiddled layout: dequantize_utils.py:4-54, quantize/mxfp.py:67-131  */
};

/* C[M,N] bf16 = A[M,K] bf16 . (fp4(B[N,K/2]) * 2^(Scale[N,K/32] - scale_bias))^T (+ Bias[M,N] bf16),
 * fp32 accumulation.  Replaces `call(A, B, Scale, Bias, C, stream)` of the kernel generated from
 * examples/dequantize_gemm/example_dequant_gemm_bf16_mxfp4_cdna4.py:201-244.  The reference
 * multiplies by 2^Scale with the raw byte (:254-267): scale_bias = 0; an E8M0 scale is
 * scale_bias = 127.  Bias may be NULL.  Requires K % 64 == 0, scale_size == 32.
 * The library picks the kernel by shape (one and two rows up to K = 32768: a dot-product kernel on whole weight
 * rows; up to 16 rows, more while passes of 16 stay ahead: the activations resident in registers and the weights
 * streamed once; else the tiled GEMM).  Each adds the same products in fp32 in an order of its own: a row computed
 * in a small batch and in a large one may differ in the last bf16 bit; every call of one shape returns the same bits. */
int call_dequant_gemm_bf16_mxfp4(const void* A, const void* B, const void* Scale, const void* Bias, void* C, int M,
                                 int N, int K, int scale_size, int fp4_format, int scale_bias, dq_stream_t stream);

/* ---- further dequantize GEMMs (same 256x256 MFMA kernel, different decoders) ------------------ */

/* bf16 x fp4 without block scales: C[M,N] bf16 = A[M,K] bf16 . bf16(fp4(B[N,K/2]))^T, fp32 accumulation.
 * Replaces `kernel(A, qB)` of examples/dequantize_gemm/example_dequant_gemm_bf16_fp4_hopper.py:46-346
 * (ref_program_twiddling / ref_program_simple, :348-386).  fp4_format as above: DQ_FP4_TWIDDLING is the example's
 * fast_dequant=True layout, DQ_FP4_SIMPLE its fast_dequant=False conversion (exponent E + 126).  Requires K % 64 == 0. */
int call_dequant_gemm_bf16_fp4(const void* A, const void* B, void* C, int M, int N, int K, int fp4_format,
                               dq_stream_t stream);

/* fp16 x "simple" fp4: C[M,N] (transposed = 0) or Ct[N,M] (transposed = 1) fp16 =
 * A[M,K] fp16 . fp16bits((s<<15)|((E+14)<<10)|(m<<9))(B[N,K/2])^T, fp32 accumulation.  Replaces
 * `call(A, B, Ct, stream)` of examples/dequantize_gemm/example_dequant_gemm_fp4_hopper.py:179-215.
 * Requires K % 64 == 0. */
int call_dequant_gemm_fp16_fp4(const void* A, const void* B, void* C, int M, int N, int K, int transposed,
                               dq_stream_t stream);

/* The same product with K cut into `split` slices: slice z is multiplied by its own workgroups into
 * SplitC[z] (M x N, or N x M when transposed, fp16) and a second kernel adds the slices in fp16, slice 0 first.
 * Replaces `call(A, B, Ct, stream)` of the kernel built from `main_split`,
 * examples/dequantize_gemm/example_dequant_gemm_fp4_hopper.py:136-175, whose SplitC is an internal buffer: here the
 * caller passes it (split * M * N fp16; NULL allowed when split == 1), since no entry point allocates.
 * Requires K % (64 * split) == 0, split in 1..64, M * N % 8 == 0 when split > 1. */
int call_dequant_gemm_fp16_fp4_splitk(const void* A, const void* B, void* SplitC, void* C, int M, int N, int K,
                                      int split, int transposed, dq_stream_t stream);

/* The same split-K product for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference, whose SplitC is allocated
 * inside the kernel function.  The partial results live in a buffer of DQ_STATIC_SCRATCH_BYTES that the library
 * holds in device memory, one per GPU, from the moment it is loaded there until the process ends; the call
 * allocates and frees nothing.  Fails with a message when split * M * N * 2 bytes exceed the buffer.  Every
 * call on a GPU shares that GPU's buffer: calls that overlap in time on one GPU (two streams, two threads) race
 * on it; calls in one stream's order do not.  The current device must be the one `stream` belongs to.
 * Other requirements and results as call_dequant_gemm_fp16_fp4_splitk (bit-identical to it). */
#define DQ_STATIC_SCRATCH_BYTES (16u << 20)
int call_dequant_gemm_fp16_fp4_splitk_static(const void* A, const void* B, void* C, int M, int N, int K, int split,
                                             int transposed, dq_stream_t stream);

/* The 2-bit and 1-bit cases of the same example (`num_bits`: B[N, K * bits / 8], 16 or 32 codes per 32-bit word):
 * C[M,N] fp16 = A[M,K] fp16 . dequant(B, Scale[N, K/group], Zeros[N, K/group])^T, fp32 accumulation.
 * `convention` is a DQ_I2_* value: DQ_I2_TWOS is the example's slow path (`_tir_packed_int_to_int_convert`,
 * examples/dequantize_gemm/example_dequant_gemv_fp16xint4.py:121-124); DQ_I2_UNSIGNED is decode_i2u_to_f16 /
 * decode_i1u_to_f16 (w = c); DQ_I2_OFFSET is decode_i2s_to_f16 (w = c - 2) / decode_i1s_to_f16 (w = 2 c - 1)
 * (examples/dequantize_gemm/quantize/lop3.py:424-463, 679-746).  With Scale: w * s (lop3.py:465-500, 748-810); with
 * Zeros as well: (w - z) * s, or w * s - z when `zeros_rescale` is non-zero (lop3.py:564-636, 812-891).
 * DQ_LAYOUT_INTERLEAVED: words passed through interleave_weight(qw, bits, "float16")
 * (examples/dequantize_gemm/quantize/utils.py:71-123).  Scale and Zeros may be NULL.  Decode batches only: M <= 64
 * (rows go through the kernel two at a time).  Requires K % (128 / bits) == 0, K <= 32768, group % (128 / bits) == 0. */
int call_dequantize_gemv_lowbit(const void* A, const void* B, const void* Scale, const void* Zeros, void* C, int M, int N,
                                int K, int group, int bits, int convention, int layout, int zeros_rescale,
                                dq_stream_t stream);

/* fp16 x uint4 with the integer decoders: C[M,N] fp16 = A[M,K] fp16 . dequant(B, Scale, Zeros)^T with
 * the dequantised tile rounded to fp16 exactly as call_dequantize_w4 does.  Replaces `call(A, B, C)` of
 * examples/dequantize_gemm/example_dequant_gemm_fine_grained.py:45-88 (mode DQ_W4_UNSIGNED) and serves
 * W4A16 at M > 128.  Requires K % 64 == 0; group rules as for call_dequantize_gemv_w4a16. */
int call_dequant_gemm_w4_fp16(const void* A, const void* B, const void* Scale, const void* Zeros, void* C, int M,
                              int N, int K, int group, int mode, int layout, dq_stream_t stream);

enum dq_i2_convention {
  DQ_I2_UNSIGNED = 0, /* w = c       decode_i2u_to_i8s, examples/dequantize_gemm/quantize/lop3.py:975-997 */
  DQ_I2_OFFSET = 1,   /* w = c - 2   decode_i2s_to_i8s, lop3.py:950-973                                   */
  DQ_I2_TWOS = 2      /* w = sext2(c) quantization.py:333-343                                             */
};

/* int8 x 2-bit: C[M,N] = A[M,K] int8 . decode(B[N,K/4])^T, exact int32 accumulation.  out_kind 0: C is
 * int32.  out_kind 1: C is fp16 = (float(acc) / s_a[m]) / s_w, the BitLinear epilogue
 * (examples/bitnet-1.58b/utils_quant.py:165-170), s_a fp32 [M].  layout DQ_LAYOUT_PLAIN: byte j holds
 * codes 4j..4j+3 at bits 0,2,4,6; DQ_LAYOUT_INTERLEAVED: every 32-bit word pre-permuted by
 * interleave_weight(qw, 2, "int8"), which is what the reference's kernels are fed
 * (examples/bitnet-1.58b/kernel_benchmark/tilelang_bitnet_158_int8xint2_decode.py:196-234,249-251).
 * Replaces `call(A, B, C, stream)` of tilelang_bitnet_158_int8xint2_prefill.py:188-296 and
 * tilelang_bitnet_158_int8xint2_decode.py:66-175.  Requires K % 128 == 0.
 * The library picks the kernel by shape (M <= 4: a streaming dot-product kernel; up to 32 rows with K % 256 == 0: the
 * activations resident in registers and the weights streamed once; a few hundred rows on a long K:
 * K sliced over the waves of a workgroup; else the tiled GEMM).  All four read DQ_LAYOUT_FRAGMENTS; where the
 * tiled GEMM does not take a fragment-ordered problem (too few tiles) the K-sliced kernel runs it whatever its size.  For tests and measurements out_kind may carry one
 * of the flags below, which names the kernel instead; all kernels return the same bits. */
enum dq_i2_kernel {
  DQ_I2_KERNEL_KSLICED = 16, /* needs K % 2048 == 0, K < 131072; -1 where it cannot run */
  DQ_I2_KERNEL_TILED = 32,
  DQ_I2_KERNEL_RESIDENT = 64 /* activations resident in registers: M <= 32 (128 on matrices of few rows), K % 256 == 0 */
};
int call_gemm_int8xint2(const void* A, const void* B, void* C, int M, int N, int K, int convention, int layout,
                        const void* s_a, float s_w, int out_kind, dq_stream_t stream);

/* BitLinear activation quantiser (the caller-side step before call_gemm_int8xint2): per row of X[M,K] fp16,
 * S[m] = (1 / max(max_k |x|, 1e-5)) * 127 in fp32 (torch's `Qp / tensor` = reciprocal, then product) and Q[m,k] = clamp(round_half_even(float(x) * S[m]), -128, 127) int8,
 * bit-identical to BitLinearBitBLAS.activation_quant (examples/bitnet-1.58b/utils_quant.py:156-163), which it
 * replaces.  Requires K % 8 == 0. */
int call_bitnet_activation_quant(const void* X, void* Q, void* S, int M, int K, dq_stream_t stream);

/* MXFP4 weight quantiser (the producer of call_dequant_gemm_bf16_mxfp4's B and Scale, which the reference's
 * example draws at random, examples/dequantize_gemm/example_dequant_gemm_bf16_mxfp4_cdna4.py:99-103,286-290):
 * W[N,K] bf16 -> B[N,K/2] e2m1 codes, two per byte, even k in the low nibble, and Scale[N,K/32] one byte per 32 k.
 * Per block: e = max(floor(log2(max|w|)) - 2, -127), Scale = clamp(e + scale_bias, 0, 255), codes =
 * encode_fp4_e2m1_values(w / 2^(Scale - scale_bias)) of examples/dequantize_gemm/quantize/nvfp4.py:120-138
 * (thresholds 0.25 .. 5.0, a value on a threshold goes up, saturation at 6, no negative zero).
 * scale_bias as in call_dequant_gemm_bf16_mxfp4 (127: E8M0).  Requires K % 32 == 0. */
int call_quantize_bf16_mxfp4(const void* W, void* B, void* Scale, int N, int K, int scale_bias, dq_stream_t stream);

/* Block-scaled MXFP4 x MXFP4: C[M,N] bf16 = (e2m1(A[M,K/2]) * 2^(ScaleA[M,K/32] - 127)) .
 * (e2m1(B[N,K/2]) * 2^(ScaleB[N,K/32] - 127))^T (+ Bias[M,N] bf16), fp32 accumulation, on the gfx950 scaled matrix
 * instruction: codes and E8M0 scale bytes go to the instruction as they lie in memory (the layout
 * call_quantize_bf16_mxfp4 writes with scale_bias = 127, for either operand).  The arithmetic is that of
 * blockscaled_gemm_ref, examples/blockscaled_gemm_sm100/gemm_mxfp8_blockscaled_1d1d.py:575-620; it stands where the
 * reference's block-scaled kernels stand on NVIDIA parts (`C = kernel(A, B, SFA, SFB)` of :17-170 and of
 * examples/gemm_sm120/sm120_nvfp4_blockscaled_gemm.py:58-148), with plain row-major scales.  A scale byte of 255 is
 * NaN.  Requires K % 128 == 0, K >= 256. */
int call_gemm_mxfp4_mxfp4(const void* A, const void* B, const void* ScaleA, const void* ScaleB, const void* Bias,
                          void* C, int M, int N, int K, dq_stream_t stream);

enum dq_i4_decode {
  DQ_I4_UNSIGNED = 0,      /* w = q, plain nibbles (example_dequant_gemm_fine_grained.py int8 path)                     */
  DQ_I4_TWOS = 1,          /* w = sext4(q), plain nibbles (example_dequant_gemm_w4a8.py:10-21)                          */
  DQ_I4U_INTERLEAVED = 2,  /* w = q, words through interleave_weight(qB, 4, "int8"): decode_i4u_to_i8s,
                              examples/dequantize_gemm/quantize/lop3.py:1027-1047                                      */
  DQ_I4S_INTERLEAVED = 3,  /* w = q - 7 (the decoder's MEDIAN_NUM is 0x07070707), same words: decode_i4s_to_i8s,
                              lop3.py:999-1025                                                                         */
  DQ_I2_TO_I4 = 4          /* B[N,K/4] holds 2-bit codes, w = c: decode_i2u_to_i4s / decode_i2s_to_i4s, lop3.py:1049-1089
                              (the 2-bit operand of the int4 x int4 matrix instruction; the signed decoder's adjustment
                              is commented out in the reference, so both are w = c).  With a_packed = 1 only.          */
};

/* flag for `transposed` (tests and measurements): run the tiled GEMM also where the decode kernel would be taken */
#define DQ_I4_KERNEL_TILED 32

/* int8 x 4-bit, exact int32: C[M,N] or Ct[N,M] (transposed = 1) = A . decode(B[N,K/2])^T, `decode` a DQ_I4_* value.
 * Replaces `call(A, B, Ct)` of examples/dequantize_gemm/example_dequant_gemm_w4a8.py:109-147 (DQ_I4_TWOS), the int8
 * path of example_dequant_gemm_fine_grained.py (DQ_I4_UNSIGNED) and the int8 branch (`use_dp4a`) of
 * example_dequant_gemv_fp16xint4.py:47-54,113-133: its slow path (DQ_I4_TWOS) and, with fast_decoding, the two
 * interleaved decoders.  M <= 4 runs as a streaming dot-product kernel (K <= 16384; 16 bytes of B per lane,
 * v_dot4_i32_i8, the decoder's constant applied through the sum of the activations), larger M on the tiled GEMM.
 * a_packed 1: A is packed int4 too, A[M,K/2] (examples/gemm_int4/example_tilelang_gemm_int4.py:17-38), DQ_I4_TWOS
 * or DQ_I2_TO_I4, K < 131072 (the operands carry a factor 16 in the int32 accumulator).  Requires K % 128 == 0. */
int call_gemm_int8xint4(const void* A, const void* B, void* C, int M, int N, int K, int decode, int a_packed,
                        int transposed, dq_stream_t stream);

/* int8 x 1-bit decode GEMV, exact int32: C[M,N] = A[M,K] int8 . decode(B[N,K/8])^T for M <= 4, K <= 65536,
 * K % 128 == 0.  `convention` (a dq_i2_convention value read for one bit): DQ_I2_UNSIGNED w = c (decode_i1u_to_i8s),
 * DQ_I2_OFFSET w = 2 c - 1 (decode_i1s_to_i8s), DQ_I2_TWOS w = -c (the sign extension of a one-bit field, the int8
 * branch's slow path, quantization.py:333-343).  `layout`: DQ_LAYOUT_PLAIN (bit e of a byte is code e) or
 * DQ_LAYOUT_INTERLEAVED (32-bit words through interleave_weight(qB, 1, "int8"), utils.py:102-109, the order the
 * reference's 16-bit decoder expects).  Replaces the int8 branch of
 * examples/dequantize_gemm/example_dequant_gemv_fp16xint4.py:47-54,126-133 at num_bits = 1 with the decoders of
 * examples/dequantize_gemm/quantize/lop3.py:893-948. */
int call_gemv_int8xint1(const void* A, const void* B, void* C, int M, int N, int K, int convention, int layout,
                        dq_stream_t stream);

/* ---- plain GEMM on the same MFMA tile (no dequantise step) ----------------------------------------- */

enum dq_dtype { DQ_DT_F16 = 0, DQ_DT_BF16 = 1, DQ_DT_I8 = 2, DQ_DT_F32 = 3, DQ_DT_I32 = 4,
                DQ_DT_FP4 = 5 /* packed e2m1 codes: call_mfma_rate only */ };

/* C[M,N] = op(A) . op(B), both operands at the compute type, fp32 / int32 accumulation on the tile the dequantize
 * GEMMs share.  Replaces `call(A, B, C, stream)` of the kernel built by `matmul(M, N, K, ..., trans_A, trans_B,
 * in_dtype, out_dtype, accum_dtype)` of testing/python/kernel/test_tilelang_kernel_gemm.py:5-49 (and
 * testing/python/amd/test_tilelang_test_amd.py:7-55): A is [M,K], or [K,M] when trans_A; B is [N,K] when trans_B
 * (the layout of every dequantize kernel), else [K,N].  in_dtype DQ_DT_F16 / DQ_DT_BF16 with out_dtype the same or
 * DQ_DT_F32; DQ_DT_I8 with DQ_DT_I32 (exact).  An operand stored the other way round is transposed first into
 * Workspace, which the caller passes: (trans_A ? M*K : 0) + (trans_B ? 0 : N*K) elements of in_dtype, each part rounded
 * up to 256 bytes; NULL allowed for trans_A = 0, trans_B = 1.  Requires K % 64 == 0 (K % 128 == 0 for int8). */
int call_gemm_plain(const void* A, const void* B, void* C, void* Workspace, int M, int N, int K, int in_dtype,
                    int out_dtype, int trans_A, int trans_B, dq_stream_t stream);

/* ---- diagnostics ------------------------------------------------------------------------------------- */

/* The rate the matrix pipe sustains on the caller's operands, with no memory, LDS or decode work beside it: every
 * wave of `workgroups` workgroups of four loads four A and four B fragments from Operands (64 KiB, read as they
 * are: fill them with random values of `in_dtype`) and issues `iters` rounds of the 16 matrix instructions of a
 * 128 x 128 wave tile (32x32x16 for DQ_DT_F16 / DQ_DT_BF16, 32x32x32 for DQ_DT_I8, the block-scaled 32x32x64 for
 * DQ_DT_FP4 with both scales 1.0); Out takes workgroups * 256 floats that mean nothing.  Operations = workgroups * 4 *
 * iters * 16 * 2 * 32 * 32 * (16, 32 or 64); time it with
 * events.  It has no counterpart in the reference: bench.py reports it beside the GEMM rows, because random
 * operands hold this chip below the clock its published peak assumes, and the figure says by how much. */
int call_mfma_rate(const void* Operands, void* Out, int in_dtype, int workgroups, int iters, dq_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* DQGEMM_H_ */
