// W4A16 small-batch kernel for gfx950 (blocks of up to 64 activation rows), direct-to-LDS streaming.
//
// Replaces the batched use of the kernel generated from
// examples/dequantize_gemm/example_dequant_gemv_fp16xint4.py:83-153 (group scales / zeros as in
// examples/dequantize_gemm/quantize/lop3.py:41-81,136-176).  The path is HBM-bound, so the
// kernel is built around keeping many bytes in flight with the access pattern the memory system
// likes, at no register cost:
//
//   * a workgroup owns 64 or 128 weight rows (4 waves x 1 or 2 blocks of 16 rows) and walks K in
//     steps of 256; the packed weights (rows x 128 B) and the activations (16 MB rows x 512 B) travel
//     global -> LDS with global_load_lds_dwordx4 into a ring of NST stages, NST - 1 steps ahead of the
//     arithmetic; every weight DMA instruction reads 8 rows x 128 contiguous bytes; the group scales / zeros
//     travel the same way, 16 bytes (four steps) per row at a time, into a small ring of their own;
//   * a lane's bytes land at LDS base + lane * 16 whatever its source address, so the
//     bank-conflict swizzles are applied by permuting the SOURCE addresses: 16-byte piece p of
//     weight row n sits at position p ^ ((n >> 1) & 7), piece p of activation row m at
//     (p & 16) | ((p ^ m) & 15);
//   * lane (g = lane / 16, r = lane % 16) of a wave reads one 16-byte piece of weight row r per
//     128-k chunk; each of its four dwords is decoded in registers (exact fp16 tile values,
//     decode_w4) and is the 16 x 32 operand of one v_mfma_f32_16x16x32_f16, contraction index
//     labelled k = chunk + g * 32 + j * 8 + {0,4,1,5,2,6,3,7}[e]; the matching activation
//     operand is one ds_read_b128 plus, for the plain layout, four v_perm_b32;
//   * all vector-memory loads of the loop are these DMA instructions, issued from inline assembly
//     and tracked by hand with s_waitcnt vmcnt; one workgroup barrier per step;
//   * the LDS reads, the decode and the MFMAs of consecutive 32-k sub-steps are software-pipelined
//     (two sub-steps deep, across the step boundary), so that a wave's MFMAs issue among the VALU work
//     of its next sub-step.
//
// Every wave owns its output tile.  Asked for by the launcher (matrices with too few rows to give every CU a
// workgroup), K is cut into gridDim.z slices whose fp32 sums a second kernel adds in slice order: with or without
// the split no atomics, and results bit-identical from run to run.
#include <type_traits>

#include "dq_common.h"

namespace dq {

namespace {

// M0 is set inside each statement right before the one instruction that reads it and is not on the clobber list
// (clang treats M0 as reserved there and promises nothing for it); nothing else in this kernel depends on M0 across
// the statements: no other LDS-direct load, no GWS / sendmsg, no indirect register indexing.
__device__ __forceinline__ void dma16(unsigned lds_addr, unsigned voff, const void* sbase) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2\n\t" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
}
__device__ __forceinline__ void dma4(unsigned lds_addr, unsigned voff, const void* sbase) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2\n\t" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
}

constexpr int kStepK = 256;

// RBW blocks of 16 weight rows per wave: a workgroup owns 64 RBW rows.
template <int MB, int RBW>
struct StreamGeom {
  static constexpr int kRowsPerWg = 64 * RBW;
  static constexpr int kWBytes = kRowsPerWg * (kStepK / 2);  // packed weights of a stage
  static constexpr int kABytes = MB * 16 * (kStepK * 2);     // activations of a stage
  static constexpr int kStage = kWBytes + kABytes;
  // Scales and zeros live in a ring of their own behind the stages: one slot = the 16 bytes (8 groups of 128 k =
  // 4 steps) of 128 rows of scales, then the same of zeros.
  static constexpr int kScaleSlot = 2 * 128 * 16;
};

// KSPLIT = 2: eight waves, two per SIMD; waves 4..7 own the same rows as waves 0..3 and take the second
// 128-k half of every step (the two partial sums meet once, through LDS, after the K loop).  The
// LDS traffic and the decode work per workgroup are those of KSPLIT = 1; what the second wave per
// SIMD buys is that one wave's MFMAs run under the other's decode and waits.
template <int MB, int RBW, int NST, int KSPLIT, int MODE, bool APERM>
__global__ __launch_bounds__(256 * KSPLIT) void w4a16_stream_kernel(const half_t* __restrict__ A_all,
                                                                     const uint8_t* __restrict__ B_all,
                                                                     const half_t* __restrict__ S,
                                                                     const half_t* __restrict__ Z, half_t* __restrict__ C,
                                                                     float* __restrict__ Parts, int M, int N, int K, int gshift,
                                                                     int pshift, int scale_slot_mask) {
  extern __shared__ __align__(16) unsigned char smem[];
  using G = StreamGeom<MB, RBW>;
  static_assert(KSPLIT == 1 || KSPLIT == 2, "one or two waves per SIMD");
  static_assert((2 * RBW) % KSPLIT == 0 && (2 * MB) % KSPLIT == 0, "whole DMA instructions per wave");
  constexpr int kRowsPerWg = G::kRowsPerWg;
  constexpr int kWBytes = G::kWBytes;
  constexpr int kWOps = 2 * RBW / KSPLIT;               // weight DMA instructions per wave per stage
  constexpr bool kScale = MODE >= W4_SCALE;
  constexpr bool kZeros = MODE >= W4_ZEROS_ORIGINAL;
  constexpr int kAOps = 2 * MB / KSPLIT;                // activation DMA instructions per wave per stage
  // DMA instructions per wave per stage; every fourth stage carries one more, the scales / zeros of four steps,
  // which the waits below do not count (they then wait for one instruction more than they must)
  constexpr int kOps = kWOps + kAOps;
  constexpr int kRing = NST * G::kStage;
  constexpr int kWaitOps = (NST - 2) * kOps;            // younger instructions when the next stage must have landed
  static_assert((NST - 1) * kOps <= 63, "vmcnt is a 6-bit counter");
  constexpr int kU = 2 / KSPLIT;                        // 128-k halves of a step per wave
  constexpr int kSub = 4 * kU;                          // sub-steps (32 k) of a step per wave

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wn = wave & 3;                              // which rows
  const int kh = wave >> 2;                             // which half of a step (KSPLIT = 2)
  const int g = lane >> 4;
  const int r = lane & 15;
  const int n0 = blockIdx.x * kRowsPerWg;
  const int m0 = blockIdx.y * (16 * MB);
  const int mrows = min(M - m0, 16 * MB);
  // K split across workgroups (gridDim.z slices): slice z takes a run of whole steps that starts where a chunk of
  // scales starts, and leaves its fp32 sums in Parts[z][M][N]; w4a16_splitk_sum_kernel adds the slices up in a fixed
  // order.  For matrices with too few rows to give every CU a workgroup.
  int s0 = 0, KS = K / kStepK;
  if (gridDim.z > 1) {
    const int unit = (K >> gshift) < 8 ? 1 : (1 << pshift);  // steps per chunk of scales (short rows: one chunk for all)
    const int units = (KS + unit - 1) / unit;
    const int u0 = units * (int)blockIdx.z / (int)gridDim.z, u1 = units * ((int)blockIdx.z + 1) / (int)gridDim.z;
    s0 = u0 * unit;
    KS = min(u1 * unit, KS) - s0;
  }
  const int k0 = s0 * kStepK;
  const half_t* const A = A_all + k0;
  const uint8_t* const B = B_all + (k0 >> 1);
  // Group size 2^gshift (32 .. K): a row's 16 bytes of scales (eight groups) cover 2^pshift steps of 256 k, travel
  // once per that many steps and live in a ring of scale_slot_mask + 1 slots (the launcher sizes it).
  const int groups_per_row = max(K >> gshift, 1);  // one group per row: any shift that maps every k to group 0
  const unsigned lds0 = (unsigned)(size_t)smem;

  // ---- per-lane source offsets of the DMA instructions ------------------------------------------
  unsigned w_voff[kWOps], a_voff[kAOps];
#pragma unroll
  for (int i = 0; i < kWOps; ++i) {
    const int c = (wave * kWOps + i) * 64 + lane;  // LDS piece: row c / 8, position c % 8
    const int row = c >> 3, pos = c & 7;
    w_voff[i] = (unsigned)min(n0 + row, N - 1) * (unsigned)(K >> 1) + (unsigned)((pos ^ ((row >> 1) & 7)) << 4);
  }
#pragma unroll
  for (int i = 0; i < kAOps; ++i) {
    const int c = (wave * kAOps + i) * 64 + lane;  // LDS piece: row c / 32, position c % 32
    const int row = c >> 5, pos = c & 31;
    a_voff[i] = (unsigned)(m0 + min(row, mrows - 1)) * (unsigned)(K * 2) + (unsigned)((pos ^ (row & 15)) << 4);
  }
  // waves 0, 1: scales of rows 0..63 / 64..127 from the workgroup's first row; waves 2, 3: zeros (or,
  // without zeros, the scales again); waves 4..7 repeat 0..3.  Every wave issues the same number of
  // DMA instructions; with 64 rows per workgroup the second half is simply not read.
  // A dword of scales per row and step would ask for 64 different cache lines per instruction, and for the same
  // line 32 steps in a row: instead a row's 16 bytes (four steps) travel at once, every fourth step.
  const int row_bytes = groups_per_row * 2;
  // Rows of fewer than eight groups (row_bytes < 16; the launcher then made the period cover all of K): the 16 bytes
  // of a row start at the row's first scale and run into the next rows', except at the end of the array, where
  // they end with it; lane_shift() is how far behind their start a row's own scales then lie.
  const bool short_rows = row_bytes < 16;
  auto chunk_start = [&](int n) { return short_rows ? min(n * row_bytes, N * row_bytes - 16) : n * row_bytes; };
  const int s_row = min(n0 + (wn & 1) * 64 + lane, N - 1);
  const unsigned s_voff = (unsigned)chunk_start(s_row);
  const unsigned char* s_src = reinterpret_cast<const unsigned char*>((wn >= 2 && kZeros) ? Z : S);
  // the last chunk of a row whose scales are not a multiple of 16 bytes reads the row's last 16 bytes instead of
  // running past its end, and the readers shift their offset by the same amount
  // (positions inside a row count from the row's first scale, wherever the workgroup's K slice starts)
  const int slice_off = (k0 >> gshift) << 1;
  auto scale_src_off = [&](int g4) { return short_rows ? 0 : min(slice_off + g4 * 16, row_bytes - 16); };
  auto scale_base = [&](int step) -> const unsigned char* {
    const int g4 = step >> pshift;
    return smem + kRing + (g4 & scale_slot_mask) * G::kScaleSlot + ((((k0 + step * 256) >> gshift) << 1) - scale_src_off(g4));
  };

  // DMA instruction `op` of the stage of `step`, into ring slot `slot`: the weights, the activations, and (op == kOps,
  // every fourth step) the scales / zeros of four steps
  auto issue_op = [&](int op, int step, int slot) __attribute__((always_inline)) {
    const unsigned sb = lds0 + slot * G::kStage;
    if (op < kWOps) {
      dma16(sb + (wave * kWOps + op) * 1024, w_voff[op], B + (size_t)step * (kStepK / 2));
    } else if (op < kOps) {
      const int i = op - kWOps;
      dma16(sb + kWBytes + (wave * kAOps + i) * 1024, a_voff[i],
            reinterpret_cast<const unsigned char*>(A) + (size_t)step * (kStepK * 2));
    } else if constexpr (kScale) {
      if ((step & ((1 << pshift) - 1)) == 0) {
        const int g4 = step >> pshift;
        dma16(lds0 + kRing + (g4 & scale_slot_mask) * G::kScaleSlot + (wn >= 2 ? 2048 : 0) + (wn & 1) * 1024, s_voff,
              s_src + scale_src_off(g4));
      }
    }
  };
  auto issue_stage = [&](int step, int slot) __attribute__((always_inline)) {
#pragma unroll
    for (int op = 0; op <= kOps; ++op) issue_op(op, step, slot);
  };

  // ---- fragment read offsets inside a stage (ui: the wave's ui-th half of a step) -----------------
  int w_off[RBW][kU], sc_off[RBW][kU], y_off[kU][4];
#pragma unroll
  for (int ui = 0; ui < kU; ++ui) {
    const int u = KSPLIT == 2 ? kh : ui;
#pragma unroll
    for (int rb = 0; rb < RBW; ++rb) {
      const int row = wn * (16 * RBW) + rb * 16 + r;
      // from scale_base(step): the row's 16 bytes, the group of this lane's 32 k inside the step, and for short rows
      // the distance of the row's scales from the start of its 16 bytes
      const int n_abs = min(n0 + row, N - 1);
      sc_off[rb][ui] = row * 16 + ((((u << 7) + (g << 5)) >> gshift) << 1) + (n_abs * row_bytes - chunk_start(n_abs));
      w_off[rb][ui] = row * 128 + ((((u << 2) + g) ^ ((row >> 1) & 7)) << 4);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) y_off[ui][j] = kWBytes + r * 512 + (u << 8) + ((((g << 2) + j) ^ r) << 4);
  }

  float4_t acc[RBW][MB];
#pragma unroll
  for (int rb = 0; rb < RBW; ++rb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[rb][mb] = float4_t{0.f, 0.f, 0.f, 0.f};

  // ---- software pipeline over the sub-steps (32 k each) of every step -----------------------------
  // Sub-step t goes through R(t): its LDS reads are requested, D(t): the weight dwords are decoded and,
  // for the plain layout, one operand is permuted to the other's element order (whichever of the two
  // takes fewer v_perm_b32), M(t): the RBW x MB MFMAs.  Slot t of the instruction stream holds
  // R(t+2), D(t+1) and M(t) between two scheduling barriers, so the MFMAs of one sub-step issue among
  // the independent VALU work of the next and no operand is waited for right after it was requested.
  // The pipeline runs across steps: the last two slots of a step read from the NEXT stage, so the
  // workgroup barrier that publishes that stage (and releases the current one for the DMA engine)
  // sits in front of them.
  uint4_t w_c[kU][RBW], w_n[kU][RBW], yraw[2][MB];
  half_t sc_c[kU][RBW], zp_c[kU][RBW], sc_n[kU][RBW], zp_n[kU][RBW];
  half8_t x_m[RBW], y_m[MB], x_d[RBW], y_d[MB];
  const unsigned char* sc_nxt = scale_base(0);  // scales of the step whose weights read_weights fetches next
  auto read_weights = [&](const unsigned char* sb) {
#pragma unroll
    for (int ui = 0; ui < kU; ++ui)
#pragma unroll
      for (int rb = 0; rb < RBW; ++rb) {
        w_n[ui][rb] = *reinterpret_cast<const uint4_t*>(sb + w_off[rb][ui]);
        sc_n[ui][rb] = kScale ? *reinterpret_cast<const half_t*>(sc_nxt + sc_off[rb][ui]) : (half_t)1.f;
        const half_t z = kZeros ? *reinterpret_cast<const half_t*>(sc_nxt + sc_off[rb][ui] + 2048) : (half_t)0.f;
        zp_n[ui][rb] = w4_cvt_addend<MODE>(sc_n[ui][rb], z);  // what the decoder adds: -8 s, -z or -(z s)
      }
  };
  // element order 0..7 for either word layout: the activations are used as they come out of LDS
  auto decode = [&](uint32_t w, half_t sc, half_t addend) -> half8_t {
    return decode_w4_cvt<MODE, !APERM, true>(w, sc, addend);
  };
  // slots s_begin .. s_end-1 of a step whose stage is sb_cur; kCur: the step exists (false only
  // while the pipeline fills before step 0), kNext: so does the next one, staged at sb_nxt
  // dma_tag: the slots also carry the DMA instructions of stage dma_step (ring slot dma_slot), which the barrier in
  // front of slot kSub - 2 has released: kOpsPerSlot a slot, from that slot on round to slot kSub - 3 of the next
  // step, so that all of them are out before the next step's wait and the waits count as if a stage went out at once
  constexpr int kOpsPerSlot = (kOps + 1 + kSub - 1) / kSub;
  auto run_slots = [&](auto s_begin, auto s_end, const unsigned char* sb_cur, const unsigned char* sb_nxt, auto cur_tag,
                       auto next_tag, auto dma_tag, int dma_step, int dma_slot) __attribute__((always_inline)) {
    constexpr bool kCur = decltype(cur_tag)::value, kNext = decltype(next_tag)::value, kDma = decltype(dma_tag)::value;
#pragma unroll
    for (int s = decltype(s_begin)::value; s < decltype(s_end)::value; ++s) {
      const int s2 = s + 2, s1 = s + 1;
      if constexpr (kDma) {
        const int rel = s >= kSub - 2 ? s - (kSub - 2) : s + 2;  // slots since the barrier that released the stage
#pragma unroll
        for (int o = 0; o < kOpsPerSlot; ++o)
          if (rel * kOpsPerSlot + o <= kOps) issue_op(rel * kOpsPerSlot + o, dma_step, dma_slot);
      }
      if (s2 < kSub) {  // R(t+2)
        if constexpr (kCur) {
#pragma unroll
          for (int mb = 0; mb < MB; ++mb)
            yraw[s & 1][mb] = *reinterpret_cast<const uint4_t*>(sb_cur + y_off[s2 >> 2][s2 & 3] + mb * (16 * 512));
        }
      } else if constexpr (kNext) {
        if (s2 == kSub) read_weights(sb_nxt);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          yraw[s & 1][mb] = *reinterpret_cast<const uint4_t*>(sb_nxt + y_off[0][s2 - kSub] + mb * (16 * 512));
      }
      if (s1 < kSub ? kCur : kNext) {  // D(t+1)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          y_d[mb] = __builtin_bit_cast(half8_t, yraw[s1 & 1][mb]);
#pragma unroll
        for (int rb = 0; rb < RBW; ++rb) {
          if (s1 < kSub) x_d[rb] = decode(w_c[(s1 >> 2) % kU][rb][s1 & 3], sc_c[(s1 >> 2) % kU][rb], zp_c[(s1 >> 2) % kU][rb]);
          else x_d[rb] = decode(w_n[0][rb][0], sc_n[0][rb], zp_n[0][rb]);
        }
      }
      if constexpr (kCur) {  // M(t)
#pragma unroll
        for (int rb = 0; rb < RBW; ++rb)
#pragma unroll
          for (int mb = 0; mb < MB; ++mb)
            acc[rb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(x_m[rb], y_m[mb], acc[rb][mb], 0, 0, 0);
      }
#ifndef DQ_STREAM_SPREAD
#define DQ_STREAM_SPREAD 4
#endif
      if constexpr (DQ_STREAM_SPREAD > 0) {
        // one matrix instruction, at most one LDS read, a few vector instructions, RBW x MB times: left to itself
        // the scheduler issues the slot's matrix instructions back to back and the decode in one piece
#pragma unroll
        for (int i = 0; i < RBW * MB; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x002, DQ_STREAM_SPREAD, 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int rb = 0; rb < RBW; ++rb) x_m[rb] = x_d[rb];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) y_m[mb] = y_d[mb];
    }
  };
  auto next_weights_become_current = [&]() {
#pragma unroll
    for (int ui = 0; ui < kU; ++ui)
#pragma unroll
      for (int rb = 0; rb < RBW; ++rb) {
        w_c[ui][rb] = w_n[ui][rb];
        sc_c[ui][rb] = sc_n[ui][rb];
        zp_c[ui][rb] = zp_n[ui][rb];
      }
  };
  using SlotFirst = std::integral_constant<int, 0>;
  using SlotNext = std::integral_constant<int, kSub - 2>;  // first slot that reads the next stage
  using SlotEnd = std::integral_constant<int, kSub>;

  // ---- prologue: stages 0 .. NST-1 in flight, stage 0 landed, pipeline filled -----------------------
#pragma unroll
  for (int st = 0; st < NST; ++st)
    if (st < KS) issue_stage(st, st);
  if (KS >= NST) asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NST - 1) * kOps) : "memory");
  else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  using T = std::true_type;
  using F = std::false_type;
  run_slots(SlotNext{}, SlotEnd{}, smem, smem, F{}, T{}, F{}, 0, 0);
  next_weights_become_current();

  // Step `step` multiplies out of slot step % NST.  Before its last two slots the next stage must
  // have landed: the stages younger than it are the NST - 2 issued last (kWaitOps instructions), or, in
  // the tail where fewer are in flight, the wave simply drains its counter.  After the barrier no wave
  // reads stage `step` any more (the barrier also waits for the LDS reads in flight), so the DMA of
  // step + NST goes there: spread over the slots from there to the next step's wait.
  int slot = 0;
  auto one_step = [&](int step, auto dma_before_tag, auto dma_after_tag) __attribute__((always_inline)) {
    const int slot1 = slot + 1 == NST ? 0 : slot + 1;
    const int slot_prev = slot == 0 ? NST - 1 : slot - 1;
    const unsigned char* sb_cur = smem + slot * G::kStage;
    run_slots(SlotFirst{}, SlotNext{}, sb_cur, sb_cur, T{}, T{}, dma_before_tag, step - 1 + NST, slot_prev);
    if (step + NST - 1 < KS) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kWaitOps) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    sc_nxt = scale_base(step + 1);
    run_slots(SlotNext{}, SlotEnd{}, sb_cur, smem + slot1 * G::kStage, T{}, T{}, dma_after_tag, step + NST, slot);
    next_weights_become_current();
    slot = slot1;
  };
  // steps whose stage step + NST exists; then the tail, which only finishes the stage begun in the step before it
  int step = 0;
  if (KS > NST) {
    one_step(0, F{}, T{});
    for (step = 1; step + NST < KS; ++step) one_step(step, T{}, T{});
    one_step(step, T{}, F{});
    ++step;
  }
  for (; step + 1 < KS; ++step) one_step(step, F{}, F{});
  run_slots(SlotFirst{}, SlotEnd{}, smem + slot * G::kStage, smem, T{}, F{}, F{}, 0, 0);

  if constexpr (KSPLIT == 2) {
    // waves 4..7 hand their half of the K sum to waves 0..3: [wn][rb][mb][lane] float4
    __syncthreads();  // every wave is done with the stages
    float4_t* red = reinterpret_cast<float4_t*>(smem) + wn * (RBW * MB * 64) + lane;
    if (kh == 1) {
#pragma unroll
      for (int rb = 0; rb < RBW; ++rb)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) red[(rb * MB + mb) * 64] = acc[rb][mb];
    }
    __syncthreads();
    if (kh == 1) return;
#pragma unroll
    for (int rb = 0; rb < RBW; ++rb)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const float4_t o = red[(rb * MB + mb) * 64];
        acc[rb][mb] = float4_t{acc[rb][mb][0] + o[0], acc[rb][mb][1] + o[1], acc[rb][mb][2] + o[2], acc[rb][mb][3] + o[3]};
      }
  }

  // acc[rb][mb][i] = C[m0 + mb*16 + r][n0 + wn*16*RBW + rb*16 + g*4 + i]
#pragma unroll
  for (int rb = 0; rb < RBW; ++rb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int m = mb * 16 + r;
      const int n = n0 + wn * (16 * RBW) + rb * 16 + g * 4;
      if (m >= mrows || n >= N) continue;
      const float4_t v = acc[rb][mb];
      if (gridDim.z > 1) {  // a K slice: fp32, summed up afterwards
        float* dst = Parts + ((size_t)blockIdx.z * M + (m0 + m)) * N + n;
        if (((N & 3) == 0) && n + 3 < N) {
          *reinterpret_cast<float4_t*>(dst) = v;
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (n + i < N) dst[i] = v[i];
        }
        continue;
      }
      half_t* dst = C + (size_t)(m0 + m) * N + n;
      if (((N & 3) == 0) && n + 3 < N) {
        typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
        const half4_t o = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
        *reinterpret_cast<half4_t*>(dst) = o;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < N) dst[i] = (half_t)v[i];
      }
    }
}

// C[i] = fp16(Parts[0][i] + Parts[1][i] + ...), in that order
__global__ __launch_bounds__(256) void w4a16_splitk_sum_kernel(const float* __restrict__ parts, half_t* __restrict__ C, size_t count,
                                                                int split) {
  const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i + 3 < count) {
    float4_t v = *reinterpret_cast<const float4_t*>(parts + i);
    for (int z = 1; z < split; ++z) v = v + *reinterpret_cast<const float4_t*>(parts + (size_t)z * count + i);
    typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
    const half4_t o = {(half_t)v[0], (half_t)v[1], (half_t)v[2], (half_t)v[3]};
    *reinterpret_cast<half4_t*>(C + i) = o;
  } else {
    for (size_t j = i; j < count; ++j) {
      float v = parts[j];
      for (int z = 1; z < split; ++z) v += parts[(size_t)z * count + j];
      C[j] = (half_t)v;
    }
  }
}

template <int MB, int RBW, int NST, int KSPLIT>
int launch_stream(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int group, int mode,
                  int layout, int split, void* parts, hipStream_t stream) {
  constexpr int kRingBytes = NST * StreamGeom<MB, RBW>::kStage;
  constexpr int kRowsPerWg = StreamGeom<MB, RBW>::kRowsPerWg;
  constexpr int kMaxLds = 160 * 1024;
  static_assert(kRingBytes + 2 * StreamGeom<MB, RBW>::kScaleSlot <= kMaxLds, "LDS budget");
  // Scales: 16 bytes of a row (eight groups) cover `period` steps of 256 k; a chunk is issued with the first stage it
  // serves, NST - 1 steps ahead, and read until the last: ceil((NST + period - 1) / period) chunks are alive at a
  // time; the ring takes the next power of two.  Rows of fewer than eight groups: one chunk for the whole of K.
  int gshift = 7, pshift = 2, mask = 1;
  if (mode >= W4_SCALE) {
    gshift = group == K ? 32 - __builtin_clz((unsigned)(K - 1)) : 31 - __builtin_clz((unsigned)group);
    pshift = gshift - 5;
    if (K / group < 8) {  // short rows: one chunk, issued with stage 0, serves every step
      if ((size_t)N * (K / group) * 2 < 16) return 1;
      while ((K / kStepK) > (1 << pshift)) ++pshift;
    }
    const int period = 1 << pshift;
    const int alive = (NST + period - 1 + period - 1) / period;
    int slots = 2;
    while (slots < alive) slots *= 2;
    if (kRingBytes + slots * StreamGeom<MB, RBW>::kScaleSlot > kMaxLds) return 1;
    mask = slots - 1;
  }
  const int lds = kRingBytes + (mask + 1) * StreamGeom<MB, RBW>::kScaleSlot;
  const dim3 grid((N + kRowsPerWg - 1) / kRowsPerWg, (M + 16 * MB - 1) / (16 * MB), split);
  const dim3 block(256 * KSPLIT);
  if (split > 1) {  // every slice needs a step, and a slice's 4-element rows of fp32 must be 16-byte aligned
    const int unit = (K >> gshift) < 8 ? 1 : (1 << pshift);  // as the kernel cuts K
    if ((K / kStepK + unit - 1) / unit < split || ((size_t)M * N) % 4 != 0 || !parts) return 1;
  }
#define DQ_LAUNCH2(MODE_, APERM_)                                                                                    \
  do {                                                                                                               \
    auto kern = w4a16_stream_kernel<MB, RBW, NST, KSPLIT, MODE_, APERM_>;                                            \
    static bool lds_limit_raised[kMaxDevices];                                                                       \
    if (raise_lds_limit<kMaxLds>(kern, lds_limit_raised)) return -1;                                                 \
    hipLaunchKernelGGL(kern, grid, block, lds, stream, (const half_t*)A, (const uint8_t*)B, (const half_t*)S,        \
                       (const half_t*)Z, (half_t*)C, (float*)parts, M, N, K, gshift, pshift, mask);                                         \
  } while (0)
#define DQ_LAUNCH_MODE(MODE_)                              \
  do {                                                     \
    if (layout == LAYOUT_PLAIN) DQ_LAUNCH2(MODE_, true);   \
    else DQ_LAUNCH2(MODE_, false);                         \
  } while (0)
  switch (mode) {
    case W4_UNSIGNED: DQ_LAUNCH_MODE(W4_UNSIGNED); break;
    case W4_SIGNED: DQ_LAUNCH_MODE(W4_SIGNED); break;
    case W4_OFFSET8: DQ_LAUNCH_MODE(W4_OFFSET8); break;
    case W4_SCALE: DQ_LAUNCH_MODE(W4_SCALE); break;
    case W4_USCALE: DQ_LAUNCH_MODE(W4_USCALE); break;
    case W4_ZEROS_ORIGINAL: DQ_LAUNCH_MODE(W4_ZEROS_ORIGINAL); break;
    case W4_ZEROS_RESCALE: DQ_LAUNCH_MODE(W4_ZEROS_RESCALE); break;
    case W4_ZEROS_FOLDED: DQ_LAUNCH_MODE(W4_ZEROS_FOLDED); break;
    default: DQ_FAIL("w4a16: unknown mode %d", mode);
  }
#undef DQ_LAUNCH_MODE
#undef DQ_LAUNCH2
  DQ_CHECK_HIP(hipGetLastError());
  if (split > 1) {
    const size_t count = (size_t)M * N;
    hipLaunchKernelGGL(w4a16_splitk_sum_kernel, dim3((unsigned)((count + 1023) / 1024)), dim3(256), 0, stream, (const float*)parts,
                       (half_t*)C, count, split);
    DQ_CHECK_HIP(hipGetLastError());
  }
  return 0;
}

}  // namespace

// config 0, 1, 2: 16, 32, 64 activation rows and 128 weight rows per workgroup; 3, 4, 5: 16, 32, 16
// activation rows and 64 weight rows; 6: as 2 with eight waves (measured at N = 28672, K = 8192, M = 64:
// 60 us against 63 us; the eight-wave forms of 0 and 1 were slower than the four-wave ones and are
// not built); 7: as 6 on three blocks of 16 activation rows.  `split` > 1: K in that many slices, fp32 partial
// sums in parts[split][M][N].  Returns 1 when the shape is not covered (the caller falls back to a kernel without
// these restrictions): the group size must be a power of two from 32 on or K when the mode reads scales, K a
// multiple of 256, every operand below 4 GiB (32-bit lane offsets), every slice at least a chunk of scales long.
int w4a16_stream(const void* A, const void* B, const void* S, const void* Z, void* C, int M, int N, int K, int group,
                 int mode, int layout, int config, int split, void* parts, hipStream_t stream) {
  if (K % kStepK != 0 || N < 1 || M < 1) return 1;
  // scales travel 16 bytes of a row at a time: group sizes 32, 64, ... (powers of two that divide K), or one group per row
  if (mode >= W4_SCALE && group != K && (group < 32 || group > K || (group & (group - 1)) != 0 || K % group != 0)) return 1;
  if ((size_t)N * K / 2 >= (1ull << 32) || (size_t)M * K * 2 >= (1ull << 32)) return 1;
  switch (config) {
    case 0: return launch_stream<1, 2, 6, 1>(A, B, S, Z, C, M, N, K, group, mode, layout, split, parts, stream);
    case 1: return launch_stream<2, 2, 4, 1>(A, B, S, Z, C, M, N, K, group, mode, layout, split, parts, stream);
    case 2: return launch_stream<4, 2, 3, 1>(A, B, S, Z, C, M, N, K, group, mode, layout, split, parts, stream);
    case 3: return launch_stream<1, 1, 4, 1>(A, B, S, Z, C, M, N, K, group, mode, layout, split, parts, stream);
    case 4: return launch_stream<2, 1, 3, 1>(A, B, S, Z, C, M, N, K, group, mode, layout, split, parts, stream);
    case 5: return launch_stream<1, 1, 6, 1>(A, B, S, Z, C, M, N, K, group, mode, layout, split, parts, stream);
    case 6: return launch_stream<4, 2, 3, 2>(A, B, S, Z, C, M, N, K, group, mode, layout, split, parts, stream);
    case 7: return launch_stream<3, 2, 3, 2>(A, B, S, Z, C, M, N, K, group, mode, layout, split, parts, stream);
    default: DQ_FAIL("w4a16 stream kernel: unknown configuration %d", config);
  }
}

}  // namespace dq
