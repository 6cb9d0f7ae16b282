// Weight-streaming FP4 GEMM on packed operands for at most 128 activation rows (MXFP4; NVFP4 with the
// operands dequantized in registers to exact fp16, as in the NVFP4 tile kernel).
//
// With so few rows the time is the one pass over the weights (31 MB for the Llama-3-8B up/gate
// projection: 3.9 us at 8 TB/s), so the kernel is built around bytes in flight, not around tiles:
//   * a workgroup owns ONE 32-row weight tile and a range of K; nothing is staged through LDS:
//     in the packed layout one operand of one 32x32x64 matrix instruction is one contiguous
//     kilobyte, lane by lane, so a wave loads it straight into the registers the instruction reads;
//   * the four waves take the 256-K blocks of the range in turn (wave w: blocks w, w + 4, ...) and
//     every wave issues the loads of up to DB blocks before its first matrix instruction, so for
//     K = 4096 and 32 rows the whole weight tile is requested at once;
//   * activations (at most four 32-row tiles, padded rows are zero) are re-read by every workgroup
//     and come from the L2;
//   * the four partial tiles meet in LDS and are summed in the fixed order (w0 + w2) + (w1 + w3), every
//     wave a quarter of each tile; the rounded tile goes through LDS once more so that a store writes 64
//     contiguous bytes per row, and the four waves share the stores.
// Shapes with few weight tiles (N = 4096: 128 workgroups for 256 CUs) or long K also split K
// ACROSS workgroups: each stores its fp32 partial tile into a workspace, a per-tile counter tells
// the last one to arrive, and that one adds the partials of all splits in split order (its own
// included, read back from the workspace), so the result does not depend on the arrival order.
// Counters are left at zero for the next launch.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <type_traits>

#include "../../include/fpq.h"
#include "fpq_device.h"
#include "fpq_gemm_epilogue.h"

namespace fpq {

typedef unsigned v4u_s __attribute__((ext_vector_type(4)));

constexpr int kStreamCounters = 4096;                        // one per weight tile group
constexpr int64_t kStreamCounterBytes = kStreamCounters * 4;  // they open the workspace
constexpr int kStreamMaxRows = 128;

// Dynamic LDS of a workgroup with more than four output tiles (0: the kernel's own arrays hold them)
constexpr int stream_dynamic_lds(int nt, int mt) {
  return nt * mt > 4 ? 4 * nt * mt * 3 * 64 * 16 + nt * mt * 32 * 20 * 4 : 0;
}

// NT weight row tiles per workgroup, MT activation row tiles (exactly ceil(M / 32)), DB 256-K blocks
// of loads in flight per wave, NW waves.  Every workgroup re-reads all activations (NT = 2 halves
// that, at a register cost that stream_plan explains).  Two weight tiles per workgroup are compiled for
// two workgroups per CU (at most 256 registers).
// NV: NVFP4 operands (two E4M3 scale bytes per lane and K step, 512-byte scale blocks): a lane's dword s
// of a 64-K unit, times its group's scale, is its fp16 operand of the s-th 32x32x16 matrix instruction
// of the unit on both sides, so the K order is permuted consistently and the sum is complete.
template <int NT, int MT, int DB, int NW, bool NV = false>
__global__ __launch_bounds__(64 * NW, NT == 2 && NT * MT <= 4 ? 2 : 1) void gemm_fp4_stream_kernel(
    const uint8_t* __restrict__ xq_all, const uint8_t* __restrict__ xs_all, const uint8_t* __restrict__ wq,
    const uint8_t* __restrict__ ws, const float* __restrict__ alpha_p, const uint16_t* __restrict__ bias,
    const uint16_t* residual_all, uint16_t* y, int M_all, int N, int K, int bps, int ksplit,
    float* partial, unsigned* counters, const OutSegments seg) {
  static_assert(NW == 4, "a wave owns a quarter of every tile");
  // More than 32 MT activation rows: blockIdx.z numbers slabs of 32 MT rows, each a product of its own
  // (the last may have fewer rows, even fewer row tiles).
  const int slab = blockIdx.z, m0 = slab * (MT * 32);
  const int M = min(M_all - m0, MT * 32);
  const uint8_t* xq = xq_all + (size_t)slab * MT * (K >> 6) * 1024;
  const uint8_t* xs = xs_all + (size_t)slab * MT * (K >> 8) * (NV ? 512 : 256);
  const uint16_t* residual = residual_all ? residual_all + (size_t)m0 * N : nullptr;
  const int tile_id = slab * gridDim.x + blockIdx.x;   // numbers the output tile groups for the K split
  constexpr int kStageRow = 20;             // dwords: 16 of a row's 32 bf16 + 4, rows stay 16-byte aligned
  constexpr int kStageTile = 32 * kStageRow;
  // part: [owning wave][tile][the other waves in order][lane]; stage: the rounded tiles on their way out.  More
  // than four tiles per workgroup need more than the 64 KB a kernel may declare: those take them from the
  // launch's dynamic LDS.
  typedef v4f PartOf[NT * MT][3][64];
  typedef uint32_t StageOf[kStageTile];
  constexpr bool kDynLds = stream_dynamic_lds(NT, MT) > 0;
  __shared__ v4f part_fixed[kDynLds ? 1 : 4][kDynLds ? 1 : NT * MT][3][64];
  __shared__ __attribute__((aligned(16))) uint32_t stage_fixed[kDynLds ? 1 : NT * MT][kStageTile];
  extern __shared__ __attribute__((aligned(16))) uint8_t lds_dynamic[];
  PartOf* const part = kDynLds ? (PartOf*)lds_dynamic : (PartOf*)part_fixed;
  StageOf* const stage = kDynLds ? (StageOf*)(lds_dynamic + 4 * sizeof(PartOf)) : (StageOf*)stage_fixed;
  __shared__ unsigned arrival;
  constexpr int kSB = NV ? 512 : 256;    // scale bytes per row tile and 256-K block
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int nu = K >> 6, nkb = K >> 8;
  const int rtg = blockIdx.x, split = blockIdx.y;
  const float alpha = *alpha_p;   // asked for now: the epilogue, on the critical path of every workgroup, finds it there
  const int rt_n = (N + 31) >> 5;
  const int kb_begin = split * bps, kb_end = min(nkb, kb_begin + bps);
  const int first = kb_begin + wave;                                   // this wave: first, first + NW, ...
  const int nblk = kb_end > first ? (kb_end - first + NW - 1) / NW : 0;

  // A weight tile past the last one (odd tile count, NT = 2) re-reads the last: nothing of it is stored.
  const uint8_t* wcode[NT];
  const uint8_t* wscale[NT];
#pragma unroll
  for (int i = 0; i < NT; ++i) {
    const int rt = min(rtg * NT + i, rt_n - 1);
    wcode[i] = wq + (size_t)rt * nu * 1024 + lane * 16;
    wscale[i] = ws + (size_t)rt * nkb * kSB + lane * (kSB / 64);
  }
  // Lanes whose activation row lies past M read what the lane of row 0 in their K half reads: no further
  // cache line is touched for rows that are never stored.  A row tile past the last one (a short last
  // slab) re-reads the last: the operand ends there.
  const uint8_t* xcode[MT];
  const uint8_t* xscale[MT];
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    const int l = (lane & 31) < M - 32 * j ? lane : (lane & 32);
    const int jt = min(j, (M - 1) >> 5);
    xcode[j] = xq + (size_t)jt * nu * 1024 + l * 16;
    xscale[j] = xs + (size_t)jt * nkb * kSB + l * (kSB / 64);
  }

  v16f acc[NT * MT];
#pragma unroll
  for (int j = 0; j < NT * MT; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[j][v] = 0.f;

  // A ring of DB blocks in registers.  Every load is unconditional (a block index past the wave's
  // last one is clamped to it and its matrix instructions are skipped): with loads under branches
  // the compiler can no longer count which of them are still in flight and waits for all.
  uint4 a[DB][4][NT], b[DB][4][MT];
  uint2 sa[DB][NT], sb[DB][MT];   // MXFP4 uses .x only
  const int t_last = nblk > 0 ? nblk - 1 : 0;
  // (the lambdas must be inlined whatever their size: a call would pin the register arrays they capture
  // to memory)
  auto load_block = [&](auto slot, int t) __attribute__((always_inline)) {
    constexpr int s = decltype(slot)::value;
    const int kb = min(first + NW * min(t, t_last), nkb - 1);
#pragma unroll
    for (int i = 0; i < NT; ++i) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const v4u_s ld = __builtin_nontemporal_load((const v4u_s*)(wcode[i] + (size_t)(kb * 4 + u) * 1024));
        a[s][u][i] = make_uint4(ld.x, ld.y, ld.z, ld.w);
      }
      if constexpr (NV) sa[s][i] = *(const uint2*)(wscale[i] + (size_t)kb * kSB);
      else sa[s][i].x = *(const uint32_t*)(wscale[i] + (size_t)kb * kSB);
    }
#pragma unroll
    for (int j = 0; j < MT; ++j) {
#pragma unroll
      for (int u = 0; u < 4; ++u) b[s][u][j] = *(const uint4*)(xcode[j] + (size_t)(kb * 4 + u) * 1024);
      if constexpr (NV) sb[s][j] = *(const uint2*)(xscale[j] + (size_t)kb * kSB);
      else sb[s][j].x = *(const uint32_t*)(xscale[j] + (size_t)kb * kSB);
    }
  };
  // NVFP4: activation row tiles whose fp16 operands are held at a time (four tiles: two and two, the
  // weight operand is converted once more; all four at once left the register file)
  constexpr int kJB = (MT == 4) ? 2 : MT;
  auto compute_block = [&](auto slot) __attribute__((always_inline)) {
    constexpr int s = decltype(slot)::value;
#define FPQ_STREAM_STEP(U)                                                                              \
  if constexpr (NV) {                                                                                   \
    _Pragma("unroll") for (int j0 = 0; j0 < MT; j0 += kJB) {                                            \
      v8h bh[kJB][4];                                                                                   \
      _Pragma("unroll") for (int j = 0; j < kJB; ++j) {                                                 \
        const uint4 bq = b[s][U][j0 + j];                                                               \
        const uint32_t bw[4] = {bq.x, bq.y, bq.z, bq.w};                                                \
        const uint32_t bsc = (U) < 2 ? sb[s][j0 + j].x : sb[s][j0 + j].y;                               \
        const _Float16 bsh[2] = {e4m3_byte_f16(bsc, 2 * ((U) & 1)), e4m3_byte_f16(bsc, 2 * ((U) & 1) + 1)};   \
        _Pragma("unroll") for (int s4 = 0; s4 < 4; ++s4)                                                \
          bh[j][s4] = dequant8_f16_h(bw[s4], bsh[s4 >> 1]);                                             \
      }                                                                                                 \
      _Pragma("unroll") for (int i = 0; i < NT; ++i) {                                                  \
        const uint4 aq = a[s][U][i];                                                                    \
        const uint32_t aw[4] = {aq.x, aq.y, aq.z, aq.w};                                                \
        const uint32_t asc = (U) < 2 ? sa[s][i].x : sa[s][i].y;                                         \
        const _Float16 ash[2] = {e4m3_byte_f16(asc, 2 * ((U) & 1)), e4m3_byte_f16(asc, 2 * ((U) & 1) + 1)};   \
        _Pragma("unroll") for (int s4 = 0; s4 < 4; ++s4) {                                              \
          const v8h ah = dequant8_f16_h(aw[s4], ash[s4 >> 1]);                                          \
          _Pragma("unroll") for (int j = 0; j < kJB; ++j)                                               \
            acc[i * MT + j0 + j] =                                                                      \
                __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bh[j][s4], acc[i * MT + j0 + j], 0, 0, 0);   \
        }                                                                                               \
      }                                                                                                 \
    }                                                                                                   \
  } else {                                                                                              \
    _Pragma("unroll") for (int i = 0; i < NT; ++i) {                                                    \
      const uint4 aq = a[s][U][i];                                                                      \
      const v8i av = v8i{(int)aq.x, (int)aq.y, (int)aq.z, (int)aq.w, 0, 0, 0, 0};                       \
      _Pragma("unroll") for (int j = 0; j < MT; ++j) {                                                  \
        const uint4 bq = b[s][U][j];                                                                    \
        const v8i bv = v8i{(int)bq.x, (int)bq.y, (int)bq.z, (int)bq.w, 0, 0, 0, 0};                     \
        acc[i * MT + j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(                              \
            av, bv, acc[i * MT + j], 4, 4, U, (int)sa[s][i].x, U, (int)sb[s][j].x);                     \
      }                                                                                                 \
    }                                                                                                   \
  }
    FPQ_STREAM_STEP(0)
    FPQ_STREAM_STEP(1)
    FPQ_STREAM_STEP(2)
    FPQ_STREAM_STEP(3)
#undef FPQ_STREAM_STEP
  };
  // NVFP4 with three activation row tiles: the 16 K steps of a block (one 32x32x16 matrix instruction per output
  // tile each) as a software pipeline -- while the matrix instructions of step t issue, the operands of step
  // t + 1 are converted, and the instruction order is pinned to one matrix instruction followed by its share of
  // the conversions.  Only a step's operands are held as fp16 (32 registers, not the 48 of a whole unit's
  // activations), which brings the kernel under 256 registers: two workgroups per CU, whose waves fill each
  // other's gaps (a wave alone on its SIMD issues a conversion every 8 cycles, measured).  96 rows, K = 4096,
  // weights from HBM: N = 14336 22.5 -> 20.5 us, N = 24576 33.7 -> 28.9, N = 28672 44.7 -> 36.0.  One, two and
  // four row tiles measured the same or up to 5 % slower this way and keep the unit-by-unit order above.
  constexpr bool kPipelined = NV && MT == 3;
  auto a_op = [&](auto slot, int t, int i) __attribute__((always_inline)) {
    constexpr int s = decltype(slot)::value;
    const int U = t >> 2, s4 = t & 3;
    const uint4 q = a[s][U][i];
    const uint32_t cd = s4 == 0 ? q.x : s4 == 1 ? q.y : s4 == 2 ? q.z : q.w;
    return dequant8_f16_h(cd, e4m3_byte_f16(U < 2 ? sa[s][i].x : sa[s][i].y, 2 * (U & 1) + (s4 >> 1)));
  };
  auto b_op = [&](auto slot, int t, int j) __attribute__((always_inline)) {
    constexpr int s = decltype(slot)::value;
    const int U = t >> 2, s4 = t & 3;
    const uint4 q = b[s][U][j];
    const uint32_t cd = s4 == 0 ? q.x : s4 == 1 ? q.y : s4 == 2 ? q.z : q.w;
    return dequant8_f16_h(cd, e4m3_byte_f16(U < 2 ? sb[s][j].x : sb[s][j].y, 2 * (U & 1) + (s4 >> 1)));
  };
  auto compute_block_nv = [&](auto slot) __attribute__((always_inline)) {
    v8h ah[NT], bh[MT];
#pragma unroll
    for (int i = 0; i < NT; ++i) ah[i] = a_op(slot, 0, i);
#pragma unroll
    for (int j = 0; j < MT; ++j) bh[j] = b_op(slot, 0, j);
#pragma unroll
    for (int t = 0; t < 16; ++t) {
      v8h an[NT], bn[MT];
      if (t < 15) {
#pragma unroll
        for (int i = 0; i < NT; ++i) an[i] = a_op(slot, t + 1, i);
#pragma unroll
        for (int j = 0; j < MT; ++j) bn[j] = b_op(slot, t + 1, j);
      }
#pragma unroll
      for (int i = 0; i < NT; ++i)
#pragma unroll
        for (int j = 0; j < MT; ++j)
          acc[i * MT + j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah[i], bh[j], acc[i * MT + j], 0, 0, 0);
      constexpr int kValu = ((NT + MT) * 9 + NT * MT - 1) / (NT * MT);   // 8 conversions + the scale's share, per operand
#pragma unroll
      for (int m = 0; m < NT * MT; ++m) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, kValu, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      if (t < 15) {
#pragma unroll
        for (int i = 0; i < NT; ++i) ah[i] = an[i];
#pragma unroll
        for (int j = 0; j < MT; ++j) bh[j] = bn[j];
      }
    }
  };
  auto run_block = [&](auto slot) __attribute__((always_inline)) {
    if constexpr (kPipelined) compute_block_nv(slot);
    else compute_block(slot);
  };
  auto for_slots = [&](auto&& f) __attribute__((always_inline)) {
    f(std::integral_constant<int, 0>{});
    if constexpr (DB > 1) f(std::integral_constant<int, 1>{});
    if constexpr (DB > 2) f(std::integral_constant<int, 2>{});
    if constexpr (DB > 3) f(std::integral_constant<int, 3>{});
  };
  static_assert(DB >= 1 && DB <= 4, "at most four blocks in flight");

  // With a ring of two or more blocks the loads of a slot and the matrix instructions of the next must stay
  // in program order: left alone, the instruction scheduler groups the loads of all slots (weights first,
  // then scales and activations), and since loads complete in order the wait for one slot's last operand
  // then covers the other slots' weights as well -- the ring degenerates into load everything, wait for
  // everything, compute everything (M = 1, N = 14336: 8.4 against 7.8 us from HBM; it also takes 40 registers
  // more).  With three or four activation row tiles the effect is within +-4 % either way; only four tiles
  // of NVFP4 gain throughout (128 rows, N = 4096: 15.1 -> 14.6 us).  One block in flight has nothing to order.
  constexpr bool kOrdered = NT == 1 && DB >= 2 && (MT <= 2 || (NV && MT == 4));
  for_slots([&](auto slot) {
    load_block(slot, decltype(slot)::value);
    if constexpr (kOrdered) __builtin_amdgcn_sched_barrier(0);
  });
  // Where the epilogue will store, worked out while the first loads are in flight (after the reduction
  // every instruction delays the workgroup's end).  The epilogue's lane layout: 8 consecutive columns
  // (16 bytes) of row lane / 4 and of that row + 16.  16-byte accesses need the whole tile inside N and
  // aligned rows and bases (a residual never comes with segments: one output, its rows N long).
  const int row16 = lane >> 2, c = lane & 3;
  int res_rows = __builtin_amdgcn_readfirstlane(residual && (N & 7) == 0 && ((uintptr_t)residual & 15) == 0);
  const uint16_t* res_src = residual + (size_t)row16 * N + rtg * NT * 32 + 8 * c;
  uint16_t* out_dst[NT];
  int out_ld[NT], out_whole[NT];
#pragma unroll
  for (int i = 0; i < NT; ++i) {
    const int tn0 = (rtg * NT + i) * 32;
    const OutView out = out_view(seg, y, nullptr, tn0, N);   // the matrix this tile's columns go to (unused past N)
    out_ld[i] = __builtin_amdgcn_readfirstlane(out.N);
    out_dst[i] = out.y + (size_t)(m0 + row16) * out.N + out.n0 + 8 * c;
    out_whole[i] = __builtin_amdgcn_readfirstlane(tn0 + 32 <= N && (out.N & 7) == 0 && ((uintptr_t)out.y & 15) == 0 &&
                                                  (!residual || res_rows));
    // (values the compiler may not look through: it would otherwise move their computation, kernel
    // argument loads included, to their first use behind the reduction)
    if constexpr (NT == 1) asm volatile("" : "+s"(out_ld[i]), "+s"(out_whole[i]), "+v"(out_dst[i]));
  }
  if constexpr (NT == 1) asm volatile("" : "+s"(res_rows), "+v"(res_src));
  int t0 = 0;
  for (; t0 + 2 * DB <= nblk; t0 += DB) {   // steady state: the block DB ahead exists
    for_slots([&](auto slot) {
      run_block(slot);
      if constexpr (kOrdered) __builtin_amdgcn_sched_barrier(0);
      load_block(slot, t0 + DB + decltype(slot)::value);
      if constexpr (kOrdered) __builtin_amdgcn_sched_barrier(0);
    });
  }
  for_slots([&](auto slot) {                // the ring's last full or partial content
    if (t0 + decltype(slot)::value < nblk) run_block(slot);
    if constexpr (kOrdered) __builtin_amdgcn_sched_barrier(0);
  });
  if (nblk - t0 > DB) {                     // up to DB - 1 blocks more
    for_slots([&](auto slot) { load_block(slot, t0 + DB + decltype(slot)::value); });
    for_slots([&](auto slot) {
      if (t0 + DB + decltype(slot)::value < nblk) run_block(slot);
    });
  }

  // ---- the four K parts of the workgroup, summed in the fixed order (w0 + w2) + (w1 + w3).
  // Whatever follows the last matrix instruction delays the workgroup's end, so all four waves share it:
  // wave g owns quarter g of every tile (registers 4g .. 4g + 3: columns 8g .. 8g + 7), gets that
  // quarter from the three others through LDS and carries it through the rest of the kernel.
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    if (g == wave) continue;
    const int from = wave < g ? wave : wave - 1;
#pragma unroll
    for (int t = 0; t < NT * MT; ++t)
      part[g][t][from][lane] = v4f{acc[t][4 * g], acc[t][4 * g + 1], acc[t][4 * g + 2], acc[t][4 * g + 3]};
  }
  // The rows of the residual this wave will add are asked for now: they arrive during the reduction.
  // (Store pass 2 t + p -- rows 16 p .. 16 p + 15 of tile t -- belongs to wave (2 t + p) % 4.)
  uint4 rv[(2 * NT * MT + 3) / 4];
  if (res_rows) {
#pragma unroll
    for (int pass = 0; pass < 2 * NT * MT; ++pass) {
      if ((pass & 3) != wave) continue;
      const int i = (pass >> 1) / MT, j = (pass >> 1) % MT, p = pass & 1;
      const int m = j * 32 + 16 * p + row16, n = (rtg * NT + i) * 32 + 8 * c;
      rv[pass >> 2] = m < M && n < N ? *(const uint4*)(res_src + (size_t)(j * 32 + 16 * p) * N + 32 * i)
                                     : make_uint4(0, 0, 0, 0);
    }
  }
  __syncthreads();
  v4f sum[NT * MT];
#pragma unroll
  for (int g = 0; g < 4; ++g) {
    if (g != wave) continue;
#pragma unroll
    for (int t = 0; t < NT * MT; ++t) {
      v4f k[4];   // the quarter as each wave computed it
#pragma unroll
      for (int w = 0; w < 4; ++w)
        k[w] = w == g ? v4f{acc[t][4 * g], acc[t][4 * g + 1], acc[t][4 * g + 2], acc[t][4 * g + 3]}
                      : part[g][t][w < g ? w : w - 1][lane];
#pragma unroll
      for (int q = 0; q < 4; ++q) sum[t][q] = (k[0][q] + k[2][q]) + (k[1][q] + k[3][q]);
    }
  }

  // ---- K split across workgroups: partial tiles through the workspace, last arrival finishes
  if (ksplit > 1) {
    // The parts of a tile run on different XCDs, whose L2 caches are not coherent with each other
    // for ordinary accesses.  Device-scope fences would write back and invalidate whole caches
    // (measured: 55 us for a 6 us kernel); instead every access to the workspace is a relaxed
    // device-scope atomic, which the hardware performs at the point all XCDs agree on, and every
    // wave waits for its stores to be acknowledged before the workgroup moves the counter.
    constexpr int kTile = NT * MT * 16 * 64;  // floats per partial: register v of tile t at (16 t + v) * 64 + lane
    float* mine = partial + ((size_t)tile_id * ksplit + split) * kTile + wave * 256 + lane;
#pragma unroll
    for (int t = 0; t < NT * MT; ++t)
#pragma unroll
      for (int q = 0; q < 4; ++q)
        __hip_atomic_store(mine + (t * 16 + q) * 64, sum[t][q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();   // (ksplit is the same for the whole grid: every wave of the workgroup is here)
    // One arrival per workgroup: a counter that every wave moved made the exchange 1.5 us slower (its
    // updates from different XCDs are served one after the other).
    if (threadIdx.x == 0)
      arrival = __hip_atomic_fetch_add(counters + tile_id, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    // (one value for the workgroup: all its waves leave or all stay for the barrier further down)
    if (__builtin_amdgcn_readfirstlane(arrival) != (unsigned)(ksplit - 1)) return;
    const float* all = partial + (size_t)tile_id * ksplit * kTile + wave * 256 + lane;
    for (int s = 0; s < ksplit; ++s) {
#pragma unroll
      for (int t = 0; t < NT * MT; ++t)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float p = __hip_atomic_load(all + (size_t)s * kTile + (t * 16 + q) * 64, __ATOMIC_RELAXED,
                                            __HIP_MEMORY_SCOPE_AGENT);
          sum[t][q] = s == 0 ? p : sum[t][q] + p;
        }
    }
    if (threadIdx.x == 0) __hip_atomic_store(counters + tile_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }

  // ---- y[m][n] = bf16(alpha * sum) (+ bias) (+ residual, a further bf16 add): element q of this wave's
  // quarter of tile (i, j) is m = 32 j + lane % 32, n = 32 (NT rtg + i) + 8 wave + 4 (lane / 32) + q.
  // Stored from there, an instruction would write 16 bytes into each of 32 rows; so many small pieces
  // cost 5-8 % of the whole kernel (M = 16, N = 14336: 8.0 -> 7.6 us; M = 64: 11.3 -> 10.4 us).  The
  // rounded tile goes through LDS instead and comes back with a lane holding 8 consecutive columns: 64
  // contiguous bytes per row and store.
  const int r32 = lane & 31, kh = lane >> 5;
  uint32_t* lane_stage = &stage[0][r32 * kStageRow + 4 * wave + 2 * kh];
  if (!bias) {   // (a code path of its own rather than a select after the additions)
#pragma unroll
    for (int t = 0; t < NT * MT; ++t)
      *(uint2*)(lane_stage + t * kStageTile) = make_uint2(pack_bf16x2(sum[t][0] * alpha, sum[t][1] * alpha),
                                                          pack_bf16x2(sum[t][2] * alpha, sum[t][3] * alpha));
  } else {
#pragma unroll
    for (int i = 0; i < NT; ++i) {
      const int n = (rtg * NT + i) * 32 + 8 * wave + 4 * kh;   // bias is indexed by the product's column
      float bv[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) bv[q] = n + q < N ? __uint_as_float((uint32_t)bias[n + q] << 16) : 0.f;
#pragma unroll
      for (int j = 0; j < MT; ++j) {
        const v4f& t = sum[i * MT + j];
        const uint32_t lo = pack_bf16x2(t[0] * alpha, t[1] * alpha), hi = pack_bf16x2(t[2] * alpha, t[3] * alpha);
        *(uint2*)(lane_stage + (i * MT + j) * kStageTile) =
            make_uint2(pack_bf16x2(__uint_as_float(lo << 16) + bv[0], __uint_as_float(lo & 0xffff0000u) + bv[1]),
                       pack_bf16x2(__uint_as_float(hi << 16) + bv[2], __uint_as_float(hi & 0xffff0000u) + bv[3]));
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int pass = 0; pass < 2 * NT * MT; ++pass) {
    if ((pass & 3) != wave) continue;
    const int i = (pass >> 1) / MT, j = (pass >> 1) % MT, p = pass & 1;
    const int n = (rtg * NT + i) * 32 + 8 * c, m = j * 32 + 16 * p + row16;
    if (m >= M || n >= N) continue;
    const uint4 v = *(const uint4*)&stage[pass >> 1][(16 * p + row16) * kStageRow + 4 * c];
    uint32_t w[4] = {v.x, v.y, v.z, v.w};
    uint16_t* dst = out_dst[i] + (size_t)(j * 32 + 16 * p) * out_ld[i];
    if (out_whole[i]) {   // the same for every lane
      if (residual) {
        const uint32_t r[4] = {rv[pass >> 2].x, rv[pass >> 2].y, rv[pass >> 2].z, rv[pass >> 2].w};
#pragma unroll
        for (int q = 0; q < 4; ++q)
          w[q] = pack_bf16x2(__uint_as_float(w[q] << 16) + __uint_as_float(r[q] << 16),
                             __uint_as_float(w[q] & 0xffff0000u) + __uint_as_float(r[q] & 0xffff0000u));
      }
      *(uint4*)dst = make_uint4(w[0], w[1], w[2], w[3]);
      continue;
    }
#pragma unroll
    for (int q = 0; q < 8; ++q) {   // N's last tile, or an unaligned output: element by element
      if (n + q >= N) continue;
      uint32_t h = (w[q >> 1] >> (16 * (q & 1))) & 0xffffu;
      if (residual)
        h = pack_bf16x2(__uint_as_float(h << 16) + __uint_as_float((uint32_t)residual[(size_t)m * N + n + q] << 16), 0.0f) & 0xffffu;
      dst[q] = (uint16_t)h;
    }
  }
}

struct StreamPlan {
  bool use;    // false: the tile kernels of fpq_gemm_packed.hip serve the shape better
  int nt;      // weight row tiles per workgroup
  int ksplit;  // K parts (workgroups per group of weight tiles)
  int bps;     // 256-K blocks per part
};

// Which shapes run here and how (all thresholds are measured break-even points on Llama-3-8B and
// Qwen3-8B layer shapes).  Up to 64 activation rows: always, one weight tile per workgroup.  More
// rows: up to a number of weight tiles beyond which the 128x128 tile kernel, which shares activations
// through LDS, is faster -- 65-96 rows: 512 tiles for MXFP4, one round of this kernel's workgroups (with the
// weights from HBM, this kernel against the tiles: N = 14336 12.0 / 12.3 us, N = 16384 12.5 / 12.5, N = 18432
// 15.6 / 14.3, N = 24576 17.1 / 15.3, N = 28672 20.7 / 16.5, N = 32768 21.9 / 18.0), any number for NVFP4 (N = 14336: 22.1
// against 35.9 us, N = 128256: 165 against 215); 97-128 rows (276-346 registers, one workgroup per
// CU): one round of the 256 CUs for both formats (NVFP4 took two until its tile kernels ran eight waves per
// workgroup: N = 8192 15.0 against 22.9 us for the tiles, N = 10240 26.7 against 22.7, N = 16384 27.7 against 23.9).  (Two weight tiles per workgroup halve what the L2 has to
// deliver for 33-64 rows, but need so many registers that one workgroup fills a CU; one tile per
// workgroup with two blocks in flight, two workgroups per CU, measured 5-13 % faster -- except from
// 768 weight tiles on, where two tiles per workgroup with ONE block in flight, held to 256 registers,
// are 12-16 % faster: MXFP4, N = 28672 at 64 rows 20.1 -> 17.0 us, N = 128256 73.5 -> 61.6 us; NVFP4 -- where the
// two weight tiles also share the activations' conversion to fp16 -- N = 28672 26.2 -> 22.6 us, N = 57344 45.6 -> 40.8, and already from 384 tiles on 1-4 %.)
// K is split across workgroups when the weight tiles leave at least half of the CUs idle and every
// part keeps at least 4096 of K (the exchange of partial tiles through the workspace costs about as
// much as streaming 16 blocks); fewer parts if the workspace is small.  (While one wave did the
// exchange alone the split paid for at most 32 rows; shared by the four waves it pays at every row
// count: N = 4096, K = 14336: 64 rows 14.4 -> 11.7 us, 128 rows 19.8 -> 15.4 us, NVFP4 39.0 -> 24.6 us.)
static StreamPlan stream_plan(int64_t M, int64_t N, int64_t K, int64_t workspace_bytes, bool nv = false) {
  StreamPlan plan{false, 1, 1, 0};
  if (M < 1 || M > kStreamMaxRows || N < 1 || K < 256 || K % 256 != 0) return plan;
  const int64_t rt_m = (M + 31) / 32, tiles = (N + 31) / 32, nkb = K / 256;
  // (weight-tile counts in units of the device's compute units: 256 on the part the figures above were measured on)
  const int64_t cus = device_cus();
  if (rt_m == 3 && !nv && tiles > 2 * cus) return plan;
  if (rt_m == 4 && tiles > cus) return plan;
  plan.use = true;
  if (rt_m == 2 && tiles >= (nv ? 3 * cus / 2 : 3 * cus)) plan.nt = 2;
  // NVFP4, 33-64 rows, between two and three weight tiles per CU: three per workgroup, one workgroup per CU in
  // a single round instead of a round and a half of pairs (N = 24576: K = 4096 22.2 -> 21.2 us, K = 12288 56.0 ->
  // 48.0; N = 20480 21.0 -> 19.7; four tiles per workgroup for the next range measured 4 % slower than pairs).
  // With one workgroup per CU anyway it keeps two blocks in flight per wave (N = 24576: 20.9 -> 20.1 us, K = 12288
  // 48.2 -> 45.2; N = 20480 19.8 -> 18.8; three measured 15-20 % slower).
  if (nv && rt_m == 2 && tiles > 2 * cus && tiles <= 3 * cus) plan.nt = 3;
  const int64_t groups = (tiles + plan.nt - 1) / plan.nt;
  int64_t ksplit = 1;
  if (workspace_bytes > kStreamCounterBytes && groups <= kStreamCounters) {
    ksplit = cus / groups;
    if (ksplit > nkb / 16) ksplit = nkb / 16;
    if (ksplit < 1) ksplit = 1;
    while (ksplit > 1 && kStreamCounterBytes + ksplit * groups * plan.nt * rt_m * 4096 > workspace_bytes) --ksplit;
  }
  const int64_t bps = (nkb + ksplit - 1) / ksplit;
  plan.ksplit = (int)((nkb + bps - 1) / bps);  // no empty part
  plan.bps = (int)bps;
  return plan;
}

bool stream_eligible(bool nv, int64_t M, int64_t N, int64_t K) { return stream_plan(M, N, K, 0, nv).use; }

int64_t gemm_mxf4_stream_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  const StreamPlan plan = stream_plan(M, N, K, (int64_t)1 << 62);
  if (!plan.use || plan.ksplit <= 1) return 0;
  const int64_t groups = ((N + 31) / 32 + plan.nt - 1) / plan.nt;
  return kStreamCounterBytes + (int64_t)plan.ksplit * groups * plan.nt * ((M + 31) / 32) * 4096;
}

// Arguments are validated by the caller (gemm_packed); `workspace` is null or 256-byte aligned with
// its first kStreamCounterBytes zero.  NV: NVFP4 operands.  slab_rows > 0 (a multiple of 32, at most 128):
// M exceeds what one workgroup takes and is cut into slabs of that many rows, one grid plane each, K whole.
template <bool NV>
static int launch_stream(const void* xq, const void* xs, const void* wq, const void* ws, const float* alpha,
                         const void* bias, const void* residual, void* y, int64_t M, int64_t N, int64_t K,
                         void* workspace, int64_t workspace_bytes, const OutSegments& seg, hipStream_t stream,
                         int64_t slab_rows = 0) {
  if (slab_rows) workspace = nullptr;
  const int64_t rows = slab_rows ? slab_rows : M;   // what one workgroup sees
  const StreamPlan plan = stream_plan(rows, N, K, workspace ? workspace_bytes : 0, NV);
  if (!plan.use) return FPQ_E_UNSUPPORTED;
  const dim3 grid((unsigned)(((N + 31) / 32 + plan.nt - 1) / plan.nt), (unsigned)plan.ksplit,
                  (unsigned)(slab_rows ? (M + slab_rows - 1) / slab_rows : 1));
  unsigned* counters = (unsigned*)workspace;
  float* partial = workspace ? (float*)((uint8_t*)workspace + kStreamCounterBytes) : nullptr;
#define FPQ_STREAM(NTT, MTT, DBB)                                                                       \
  hipLaunchKernelGGL((gemm_fp4_stream_kernel<NTT, MTT, DBB, 4, NV>), grid, dim3(256), 0, stream,        \
                     (const uint8_t*)xq, (const uint8_t*)xs, (const uint8_t*)wq, (const uint8_t*)ws, alpha, \
                     (const uint16_t*)bias, (const uint16_t*)residual, (uint16_t*)y, (int)M, (int)N,    \
                     (int)K, plan.bps, plan.ksplit, partial, counters, seg)
  const int mt = (int)((rows + 31) / 32);
#define FPQ_STREAM_BIG(NTT, MTT, DBB)                                                                   \
  {                                                                                                     \
    constexpr int kLds = stream_dynamic_lds(NTT, MTT);                                                  \
    static LdsLimitOnce lds_limit;                                                                      \
    if (const int st = lds_limit.ensure((const void*)gemm_fp4_stream_kernel<NTT, MTT, DBB, 4, NV>, kLds)) return st; \
    hipLaunchKernelGGL((gemm_fp4_stream_kernel<NTT, MTT, DBB, 4, NV>), grid, dim3(256), kLds, stream,   \
                       (const uint8_t*)xq, (const uint8_t*)xs, (const uint8_t*)wq, (const uint8_t*)ws, alpha, \
                       (const uint16_t*)bias, (const uint16_t*)residual, (uint16_t*)y, (int)M, (int)N,  \
                       (int)K, plan.bps, plan.ksplit, partial, counters, seg);                          \
    return (int)hipGetLastError();                                                                      \
  }
  if constexpr (NV) {
    if (plan.nt == 3 && mt == 2) FPQ_STREAM_BIG(3, 2, 2)
  }
#undef FPQ_STREAM_BIG
  if (plan.nt > 2) return FPQ_E_UNSUPPORTED;
  if (plan.nt == 2) {   // 33-64 rows only
    if (mt != 2) return FPQ_E_UNSUPPORTED;
    FPQ_STREAM(2, 2, 1);
    return (int)hipGetLastError();
  }
  switch (mt) {
    case 1:
      // enough workgroups for three per CU: two blocks in flight per wave beat four by 3-5 %; with fewer
      // workgroups the deeper ring of each wave is what keeps the memory system busy
      if ((int64_t)grid.x * grid.y * grid.z >= 3 * device_cus() / 2) FPQ_STREAM(1, 1, 2);
      else FPQ_STREAM(1, 1, 4);
      break;
    case 2: FPQ_STREAM(1, 2, 2); break;
    // (65-128 rows: one block in flight per wave, which fits two workgroups into a CU, measured 1-2 %
    // slower for MXFP4 and 6-12 % slower for NVFP4 than two blocks -- 96 rows of NVFP4, N = 4096:
    // K = 4096 12.4 against 11.5 us, K = 14336 33.7 against 29.5 us)
    case 3: FPQ_STREAM(1, 3, 2); break;
    default: FPQ_STREAM(1, 4, 2); break;
  }
#undef FPQ_STREAM
  return (int)hipGetLastError();
}

int gemm_fp4_stream(bool nv, const void* xq, const void* xs, const void* wq, const void* ws, const float* alpha,
                    const void* bias, const void* residual, void* y, int64_t M, int64_t N, int64_t K,
                    void* workspace, int64_t workspace_bytes, const OutSegments& seg, hipStream_t stream) {
  return nv ? launch_stream<true>(xq, xs, wq, ws, alpha, bias, residual, y, M, N, K, workspace, workspace_bytes, seg,
                                  stream)
            : launch_stream<false>(xq, xs, wq, ws, alpha, bias, residual, y, M, N, K, workspace, workspace_bytes, seg,
                                   stream);
}

// M rows in slabs of slab_rows (a multiple of 32 for which stream_eligible holds), all in one launch.
int gemm_fp4_stream_slabs(bool nv, const void* xq, const void* xs, const void* wq, const void* ws,
                          const float* alpha, const void* bias, const void* residual, void* y, int64_t M, int64_t N,
                          int64_t K, int64_t slab_rows, const OutSegments& seg, hipStream_t stream) {
  if (slab_rows < 32 || slab_rows > kStreamMaxRows || slab_rows % 32 != 0 || M <= slab_rows) return FPQ_E_UNSUPPORTED;
  return nv ? launch_stream<true>(xq, xs, wq, ws, alpha, bias, residual, y, M, N, K, nullptr, 0, seg, stream, slab_rows)
            : launch_stream<false>(xq, xs, wq, ws, alpha, bias, residual, y, M, N, K, nullptr, 0, seg, stream, slab_rows);
}


// ---- the entry point that allocates nothing -------------------------------------------------------
// Counters and partial tiles of a split K live in this file-scope array instead of a caller-provided
// workspace.  Every GPU the library runs on holds its own copy at its own address until the process
// ends; the array's name is only a host-side handle, the device address comes from
// hipGetSymbolAddress, once per device, and that address is what kernels and host code use.
// A split needs at most 1024 partial tiles of 4 KB on a device of 256 compute units (stream_plan: parts x
// weight tiles <= compute units, times up to four activation row tiles).
constexpr int64_t kScratchBytes = kStreamCounterBytes + 1024 * 4096;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kMaxDevices = 64;
static std::atomic<void*> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device (looked up on the first call per device; two
// threads racing on that first call store the same address).
int scratch_address(void** out) {   // also called by fpq_prepare_device (fpq_capi.hip)
  int device = -1;
  hipError_t err = hipGetDevice(&device);
  if (err != hipSuccess) return (int)err;
  if (device < 0 || device >= kMaxDevices) return FPQ_E_UNSUPPORTED;
  void* ptr = g_scratch_ptr[device].load(std::memory_order_acquire);
  if (!ptr) {
    err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess) return (int)err;
    if (!ptr) return FPQ_E_UNSUPPORTED;
    g_scratch_ptr[device].store(ptr, std::memory_order_release);
  }
  *out = ptr;
  return FPQ_OK;
}

// fpq_gemm_packed.hip: argument checks and dispatch shared with fpq_gemm_mxf4_packed_splitk
int gemm_mxf4_packed_any(const void* xq, const void* xs, const void* wq, const void* ws, const float* alpha,
                         const void* bias, const void* residual, void* y, int64_t M, int64_t N, int64_t K,
                         void* workspace, int64_t workspace_bytes, void* stream);

}  // namespace fpq

extern "C" int64_t fpq_gemm_mxf4_packed_noalloc_max_rows(void) { return fpq::kStreamMaxRows; }

extern "C" int fpq_gemm_mxf4_packed_noalloc(const void* xq, const void* xs, const void* wq, const void* ws,
                                            const float* alpha, const void* bias, const void* residual,
                                            void* y, int64_t M, int64_t N, int64_t K, void* stream) {
  if (M > fpq::kStreamMaxRows) return FPQ_E_LIMIT;
  // (a shape that could use more than the array holds -- none on a device of 256 compute units -- splits K
  // into as many parts as fit: stream_plan sizes the split to the workspace it is given)
  void* ptr = nullptr;
  const int st = fpq::scratch_address(&ptr);
  if (st != FPQ_OK) return st;
  return fpq::gemm_mxf4_packed_any(xq, xs, wq, ws, alpha, bias, residual, y, M, N, K, ptr, fpq::kScratchBytes,
                                   stream);
}

// Test hook: the split-K counters at the head of the current device's scratch array (16 KB), copied to
// `out` (device memory) in stream order; they must read zero between calls.
extern "C" int fpq_test_noalloc_counters(void* out, int64_t bytes, void* stream) {
  if (!out) return FPQ_E_NULL;
  if (bytes < 0 || bytes > fpq::kStreamCounterBytes) return FPQ_E_SHAPE;
  void* ptr = nullptr;
  const int st = fpq::scratch_address(&ptr);
  if (st != FPQ_OK) return st;
  if (bytes == 0) return FPQ_OK;
  return (int)hipMemcpyAsync(out, ptr, (size_t)bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream);
}
