// MXFP4 GEMM on operands re-tiled into the order the 32x32x64 block-scaled MFMA consumes them.
//
// Why a second layout.  With row-major codes a K slice of a 256x256 output tile is 512 separate
// 128-byte row segments; the texture path of a CU moves such segments at about half the rate of
// contiguous kilobytes, which makes operand fetch, not the matrix pipe, the limit of the
// row-major kernel.  Here every 32-row x 64-K operand of one MFMA is one contiguous kilobyte in
// memory, laid out lane by lane, so that
//   * one direct global->LDS load instruction fetches exactly one operand (contiguous 1 KB),
//   * the LDS image needs no swizzle: lane L reads its 16 bytes at block + 16 L (conflict-free),
//   * any K granularity can be staged: the kernel keeps a ring of eight 64-K units in flight,
//     enough to cover memory latency without stalling the matrix pipe.
//
// Packed codes   : block (rt, ks) = rows [32 rt, 32 rt + 32) x K [64 ks, 64 ks + 64) at byte
//                  ((rt * K/64) + ks) * 1024; inside it lane L = 32 kh + r holds the 16 bytes
//                  (32 codes) of row 32 rt + r, K [64 ks + 32 kh, +32)  -- one MX group.
// Packed scales  : block (rt, kb) = the same rows x K [256 kb, 256 kb + 256) at byte
//                  ((rt * K/256) + kb) * 256; lane L holds one dword whose byte q is the E8M0
//                  scale of row 32 rt + r, group 8 kb + 2 q + kh  -- what MFMA number q of the
//                  block takes through op_sel.
// Rows are padded to a multiple of 32 with zero codes.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/fpq.h"
#include "fpq_device.h"
#include "fpq_gemm_epilogue.h"

namespace fpq {

// ---------------------------------------------------------------------------------------------
// Row-major -> packed.  One workgroup re-tiles 32 rows x 256 K: reads are 128-byte row segments,
// writes cover 4 KB of codes and 256 B of scales contiguously.
template <bool NV>
__global__ __launch_bounds__(256) void pack_fp4_kernel(const uint8_t* __restrict__ codes,
                                                        const uint8_t* __restrict__ scales,
                                                        int64_t scale_stride, int rows, int K,
                                                        uint8_t* __restrict__ pcodes,
                                                        uint8_t* __restrict__ pscales) {
  const int kb = blockIdx.x, rt = blockIdx.y;
  const int t = threadIdx.x;
  const int r = t >> 3, c = t & 7;  // row in the tile, 16-byte chunk of the 128-byte segment
  const int row = rt * 32 + r;
  uint4 v = make_uint4(0u, 0u, 0u, 0u);
  if (row < rows) v = *(const uint4*)(codes + (size_t)row * (K >> 1) + kb * 128 + c * 16);
  const int ks = kb * 4 + (c >> 1), kh = c & 1;
  *(uint4*)(pcodes + (((size_t)rt * (K >> 6) + ks) * 64 + kh * 32 + r) * 16) = v;
  if (t < 64) {
    const int sr = t & 31, skh = t >> 5;
    const int srow = rt * 32 + sr;
    if (NV) {
      // 16 E4M3 bytes per row and 256 K; K step q, half kh uses bytes 4q + 2kh and 4q + 2kh + 1
      uint32_t lo = 0u, hi = 0u;
      if (srow < rows) {
        const uint8_t* sp = scales + (size_t)srow * scale_stride + kb * 16 + 2 * skh;
        lo = (uint32_t)sp[0] | ((uint32_t)sp[1] << 8) | ((uint32_t)sp[4] << 16) | ((uint32_t)sp[5] << 24);
        hi = (uint32_t)sp[8] | ((uint32_t)sp[9] << 8) | ((uint32_t)sp[12] << 16) | ((uint32_t)sp[13] << 24);
      }
      *(uint2*)(pscales + (((size_t)rt * (K >> 8) + kb) * 64 + t) * 8) = make_uint2(lo, hi);
    } else {
      uint32_t out = 0u;
      if (srow < rows) {
        const uint8_t* sp = scales + (size_t)srow * scale_stride + kb * 8 + skh;
        out = (uint32_t)sp[0] | ((uint32_t)sp[2] << 8) | ((uint32_t)sp[4] << 16) | ((uint32_t)sp[6] << 24);
      }
      *(uint32_t*)(pscales + (((size_t)rt * (K >> 8) + kb) * 64 + t) * 4) = out;
    }
  }
}

// Packed -> row-major, the inverse of pack_fp4_kernel on the rows that exist: what a layer that keeps
// only its packed weights hands to state_dict().
template <bool NV>
__global__ __launch_bounds__(256) void unpack_fp4_kernel(const uint8_t* __restrict__ pcodes,
                                                         const uint8_t* __restrict__ pscales, int rows, int K,
                                                         uint8_t* __restrict__ codes, uint8_t* __restrict__ scales,
                                                         int64_t scale_stride) {
  const int kb = blockIdx.x, rt = blockIdx.y;
  const int t = threadIdx.x;
  const int r = t >> 3, c = t & 7;
  const int row = rt * 32 + r;
  const int ks = kb * 4 + (c >> 1), kh = c & 1;
  const uint4 v = *(const uint4*)(pcodes + (((size_t)rt * (K >> 6) + ks) * 64 + kh * 32 + r) * 16);
  if (row < rows) *(uint4*)(codes + (size_t)row * (K >> 1) + kb * 128 + c * 16) = v;
  if (t < 64) {
    const int sr = t & 31, skh = t >> 5;
    const int srow = rt * 32 + sr;
    if (NV) {
      const uint2 in = *(const uint2*)(pscales + (((size_t)rt * (K >> 8) + kb) * 64 + t) * 8);
      if (srow < rows) {
        uint8_t* sp = scales + (size_t)srow * scale_stride + kb * 16 + 2 * skh;
        sp[0] = (uint8_t)in.x;
        sp[1] = (uint8_t)(in.x >> 8);
        sp[4] = (uint8_t)(in.x >> 16);
        sp[5] = (uint8_t)(in.x >> 24);
        sp[8] = (uint8_t)in.y;
        sp[9] = (uint8_t)(in.y >> 8);
        sp[12] = (uint8_t)(in.y >> 16);
        sp[13] = (uint8_t)(in.y >> 24);
      }
    } else {
      const uint32_t in = *(const uint32_t*)(pscales + (((size_t)rt * (K >> 8) + kb) * 64 + t) * 4);
      if (srow < rows) {
        uint8_t* sp = scales + (size_t)srow * scale_stride + kb * 8 + skh;
        sp[0] = (uint8_t)in;
        sp[2] = (uint8_t)(in >> 8);
        sp[4] = (uint8_t)(in >> 16);
        sp[6] = (uint8_t)(in >> 24);
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
constexpr int kTileCounters = 4096;                          // as the weight-streaming kernel's: they open the workspace
constexpr int64_t kTileCounterBytes = kTileCounters * 4;
#ifndef FPQ_TILE_SPLIT_MIN_BLOCKS
#define FPQ_TILE_SPLIT_MIN_BLOCKS 16     // a part of a K split keeps at least this many 256-K blocks
#endif
#ifndef FPQ_TILE_SPLIT_OVER_SLABS
#define FPQ_TILE_SPLIT_OVER_SLABS 1      // a tile kernel that splits K comes before row slabs of the streaming kernel
#endif
constexpr int kRing = 8;                 // 64-K units resident or in flight
// Scales of a 256-K block: 256 bytes per row tile for MXFP4 (one E8M0 byte per lane and K step), 512
// for NVFP4 (two E4M3 bytes per lane and K step).  They travel with the first unit of their block,
// issued eight units ahead, and are read into registers one unit before the block starts, so the
// slot a block lands in was last read several hand-overs (barriers) earlier: 2 slots would do.
constexpr int kScaleSlots = 4;
constexpr int scale_block_bytes(bool nv) { return nv ? 512 : 256; }
// (one kilobyte piece per load instruction, the same number of loads for each of the four waves: with six
// pieces -- NVFP4, 256 x 128 tiles -- two each, the last two kilobytes copies that are never read)
constexpr int scale_loads_per_wave(int blocks, bool nv) { return (blocks * scale_block_bytes(nv) / 1024 + 3) / 4; }
constexpr int scale_slot_bytes(int blocks, bool nv) {
  return (scale_loads_per_wave(blocks, nv) > 1 ? scale_loads_per_wave(blocks, nv) : 1) * 4096;
}
constexpr int scale_slots(bool nv, int groups = 1) { return nv || groups > 1 ? 2 : kScaleSlots; }
// LDS of a group of four waves whose unit holds `blocks` operand kilobytes (weight + activation row tiles)
constexpr int packed_lds_bytes(int blocks, bool nv = false, int ring = kRing, int groups = 1) {
  return ring * blocks * 1024 + scale_slots(nv, groups) * scale_slot_bytes(blocks, nv);
}
// ... and what is allocated: at least the epilogue's staging area (four waves, each WT_M rows of
// WT_N bf16 + 16 bytes)
constexpr int packed_lds_alloc(int blocks, bool nv, int ring, int wt_n, int wt_m, int groups = 1) {
  const int rings = groups * packed_lds_bytes(blocks, nv, ring, groups), staging = 4 * wt_m * (wt_n * 2 + 16);
  const int exchange = groups > 1 ? 4 * (wt_n / 32) * (wt_m / 32) * 4096 : 0;   // four waves' accumulators
  const int most = rings > staging ? rings : staging;
  return most > exchange ? most : exchange;
}

template <int N>
__device__ __forceinline__ void wait_vmem_le() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
// Workgroup barrier that orders LDS traffic only: this wave's LDS reads and writes are complete,
// its outstanding global->LDS loads are NOT waited for (that is what wait_vmem_le is for).
__device__ __forceinline__ void barrier_lds() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}
// The same with this wave's N newest LDS reads left outstanding (LDS operations complete in order).
template <int N>
__device__ __forceinline__ void barrier_lds_but() {
  asm volatile("s_waitcnt lgkmcnt(%0)\n\ts_barrier" ::"n"(N) : "memory");
}

// One workgroup of four waves (WN x WM) computes a tile of NT*32 weight rows (n) x MT*32 activation
// rows (m); a wave owns TN x TM accumulator tiles of 32 x 32.  A unit holds KW >= NT weight and MT
// activation operand blocks (KW, MT multiples of 4 so that loads and scale pieces split evenly).
//   <8, 8, 4, 2, 2>  256 x 128 tile, waves 128 x 64, ring of 4 units, 68 KB of LDS and 193 registers:
//                    two workgroups per CU.  Large M, MXFP4: while one workgroup stores its tile
//                    the other keeps the matrix pipes busy, which is worth more than the 1.5x
//                    operand traffic costs (62.4 us against 66.1 us at M = 2048, N = 14336)
//   <8, 8, 8, 2, 2>  256 x 256 tile, waves 128 x 128, one workgroup per CU: large M, NVFP4 (whose
//                    limit is the register dequantization), where whole rounds of them cost less than
//                    the 256 x 128 tiles' finer rounds (tile_plan)
//   <2, 4, 4, 2, 2>  64 x 128 tile (weight rows x activation rows), waves 32 x 64: when even the 128 x 128
//                    tiles would fill at most half of the CUs
//   <4, 4, 4, 2, 2>  128 x 128 tile, waves 64 x 64, 80 KB of LDS: two workgroups per CU; used when
//                    the big tiles would leave most CUs idle (M of a few hundred rows).  Its time
//                    has a floor of about 12 us at K = 4096; two K steps per hand-over and a ring
//                    twice as deep were both built and measured the same, so neither is kept.
// (<7, 8, 8, 1, 4>, 224 x 256 tiles that fill two whole rounds of 256 CUs at N = 14336, works and
// measured the same time as 256 x 256: the kernel runs at the matrix pipes' power limit, not at
// their issue limit, so fuller rounds buy nothing.  <7, 8, 4, 1, 4>, 224 x 128 tiles with two workgroups per CU --
// 1024 tiles, two whole rounds -- measured 3 % slower than 256 x 128: 62.0 against 60.3 us.)
// NV = true: NVFP4 operands (same packed codes; E4M3 scales, two bytes per lane and K step, 512-byte
// scale blocks): codes are dequantized in registers to exact fp16 and fed to the fp16 MFMA; a lane's
// dword s of a block goes to MFMA s of the unit on both operands, so the K order is permuted
// consistently and the sum is complete.
// GR = 2 (the 64 x 128 and 128 x 128 tiles when every workgroup has a CU to itself): a workgroup of eight
// waves in two groups of four, each group the kernel described above on one half of K with a ring of its
// own; the second group hands its accumulators to the first through LDS after the loop.  A wave of these
// small tiles spends most of a unit waiting -- for its loads, for the barrier, for its two or four matrix
// instructions to drain -- and alone on its SIMD nothing fills that time; with a second wave there, working
// on the other half of K, something does, and each group's loop is half as long.
template <int NT, int KW, int MT, int WN, int WM, bool NV = false, int RING = kRing, int GR = 1>
__global__ __launch_bounds__(256 * GR, (NT * MT <= 32 && GR == 1 ? 2 : 1)) void gemm_fp4_packed_kernel(
    const uint8_t* __restrict__ xq, const uint8_t* __restrict__ xs, const uint8_t* __restrict__ wq,
    const uint8_t* __restrict__ ws, const float* __restrict__ alpha_p,
    const uint16_t* __restrict__ bias, uint16_t* __restrict__ y, int M, int N, int K, int tiles_m,
    const uint16_t* __restrict__ residual, const OutSegments seg, int ksplit, int bps, float* partial,
    unsigned* counters) {
  constexpr int BN = NT * 32, BM = MT * 32;
  constexpr int NW = WN * WM;           // waves
  static_assert(NW == 4 && NT <= KW && KW % 4 == 0 && MT % 4 == 0 && NT % WN == 0 && MT % WM == 0,
                "unsupported tile / wave arrangement");
  constexpr int TN = NT / WN, TM = MT / WM;  // 32x32 MFMA tiles per wave along n and m
  constexpr int kBlocks = KW + MT;      // operand kilobytes per unit
  constexpr int kPer = kBlocks / NW;    // code loads per wave per unit
  constexpr int kSB = scale_block_bytes(NV);            // scale bytes per row tile and 256-K block
  constexpr int kRpp = 1024 / kSB;                      // row tiles per 1 KB scale piece
  constexpr int kPieces = kBlocks / kRpp;               // scale pieces per 256-K block
  constexpr int kScLoads = kPieces >= NW ? (kPieces + NW - 1) / NW : 1;  // scale loads per wave per block
  constexpr int kSlots = scale_slots(NV, GR), kSlotBytes = scale_slot_bytes(kBlocks, NV);
  constexpr int kUnitBytes = kBlocks * 1024;
  static_assert(RING == 4 || RING == 8, "the ring holds one or two 256-K blocks");
  constexpr int kPackedLds = packed_lds_bytes(kBlocks, NV, RING, GR);
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem_all[];
  static_assert(GR == 1 || GR == 2, "one or two groups of four waves");
  const int grp = GR > 1 ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 8) : 0;
  uint8_t* const smem = smem_all + grp * kPackedLds;   // this group's ring and scale slots
  const uint32_t smem_base = (uint32_t)(uintptr_t)smem;
  constexpr int kScaleBase = RING * kUnitBytes;
  static_assert(kScaleBase + kSlots * kSlotBytes == kPackedLds, "LDS map does not match the allocation");

  const int wave = __builtin_amdgcn_readfirstlane((threadIdx.x >> 6) & 3), lane = threadIdx.x & 63;
  // (One workgroup per tile: a persistent variant that walked several tiles per CU measured slower, the
  // hardware's own dispatch balances the XCDs better.)
  int tile_m, tile_n;
  const int logical = banded_tile<BM>(tiles_m, tile_m, tile_n);
  const int n_blk = tile_n * BN, m_blk = tile_m * BM;
  const int wn = wave % WN, wm = wave / WN;
  const int nu = K >> 6, nkb_all = K >> 8;      // units, scale blocks of a whole row tile
  // K split across workgroups (ksplit > 1, grid plane blockIdx.y): this one multiplies the 256-K blocks
  // [kb_begin, kb_begin + nkb) only, and the parts of a tile meet in the workspace after the loop.
  // Only the kernels for few tiles are ever launched that way (the large tiles have no register to spare).
  constexpr bool kCanSplit = NT * MT <= 16;
  static_assert(GR == 1 || kCanSplit, "groups split K");
  const int kb_begin = kCanSplit ? (blockIdx.y * GR + grp) * bps : 0;   // (GR = 2: both halves hold bps blocks)
  const int nkb = kCanSplit ? min(nkb_all - kb_begin, bps) : nkb_all;
  const int rt_n = (N + 31) >> 5, rt_m = (M + 31) >> 5;

  // ---- loads.  Operand b of a unit: b < KW weight row tile tile_n*NT + b % NT, else activation row tile
  // tile_m*MT + b - KW (clamped at the edge: those rows are never stored).  The slots past NT are loaded
  // and not used, which keeps every wave's load count the same; they repeat the tile's own rows, which
  // the caches serve -- the next tile's rows there doubled what the 64 x 128 tiles fetch from memory
  // (weights from HBM: N = 14336, K = 4096, 128 rows 13.0 -> 12.0 us; N = 4096, K = 14336, 384 / 512 rows
  // 32.3 -> 28.7 / 29.1; N = 8192, K = 8192, 256 rows 21.6 -> 19.2).
  // Wave w loads operands w*kPer .. w*kPer + kPer - 1.
  const uint8_t* op_base[kPer];
#pragma unroll
  for (int j = 0; j < kPer; ++j) {
    const int b = wave * kPer + j;
    if (b < KW) {
      const int rt = min(tile_n * NT + b % NT, rt_n - 1);
      op_base[j] = wq + ((size_t)rt * nu + kb_begin * 4) * 1024;
    } else {
      const int rt = min(tile_m * MT + b - KW, rt_m - 1);
      op_base[j] = xq + ((size_t)rt * nu + kb_begin * 4) * 1024;
    }
  }
  // Scale piece p of a block: one load instruction for kRpp row tiles (unit operand order), lane L
  // fetches 16 bytes of row tile L / (64 / kRpp).  Wave w loads pieces (w*kScLoads + j) % kPieces
  // into kilobyte w*kScLoads + j of the slot (with fewer pieces than waves the copies in the upper
  // kilobytes are never read: every wave issues the same instructions, no branch).
  const uint8_t* sc_base[kScLoads];
  uint32_t sc_off[kScLoads];
#pragma unroll
  for (int j = 0; j < kScLoads; ++j) {
    const int fb = ((wave * kScLoads + j) % kPieces) * kRpp;   // first operand block of the piece
    const bool is_w = fb < KW;
    constexpr int kLpr = 64 / kRpp;                            // lanes per row tile
    const int rt = min(is_w ? tile_n * NT + (fb + (int)(lane / kLpr)) % NT : tile_m * MT + fb - KW + (int)(lane / kLpr),
                       (is_w ? rt_n : rt_m) - 1);
    sc_base[j] = (is_w ? ws : xs) + (size_t)kb_begin * kSB;
    sc_off[j] = (uint32_t)rt * (uint32_t)nkb_all * (uint32_t)kSB + (lane % kLpr) * 16;
  }
  const uint32_t lane16 = lane * 16;

  // Unit u into its ring slot; with every fourth unit travel the scales of the block it opens,
  // issued first so that they have landed whenever the unit has.
  auto issue_unit = [&](int u, bool with_scales) {
    if (with_scales) {
      const int blk = u >> 2;
#pragma unroll
      for (int j = 0; j < kScLoads; ++j)
        lds_dma16(sc_base[j] + (size_t)blk * kSB, sc_off[j],
                  smem_base + kScaleBase + (blk % kSlots) * kSlotBytes + (wave * kScLoads + j) * 1024);
    }
    const uint32_t dst = smem_base + (u % RING) * kUnitBytes + wave * kPer * 1024;
#pragma unroll
    for (int j = 0; j < kPer; ++j) lds_dma16(op_base[j] + (size_t)u * 1024, lane16, dst + j * 1024);
  };

  v16f acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  // operand registers of the current and the next unit; scales of the current block and, read
  // ahead, of the next one.
  // kDeep (one row of MFMAs per unit, MXFP4): a wave has only TM matrix instructions per unit to cover the
  // LDS reads of the next one, the wait for them and the barrier, which left the matrix pipes idle three
  // quarters of the time.  There the registers run TWO units ahead (four sets, indexed by the unit's place in
  // its 256-K block): at the hand-over of unit u the reads of unit u + 2 are issued, those of unit u + 1 may
  // stay outstanding across the barrier, and the matrix instructions of unit u follow at once (64 x 128
  // tiles, N = 4096, K = 14336: 384 / 512 rows 28.9 / 29.0 -> 26.5 / 26.8 us; N = 14336, K = 4096, 128 rows
  // 10.1 -> 9.7 us, 14.0 -> 13.4 with the weights streamed from HBM; a ring of sixteen units instead of eight
  // changed nothing from the caches and cost 3 % from HBM, and with every load, LDS read
  // and barrier compiled out the matrix instructions alone take 16.3 us at 512 rows).  NVFP4 and the tiles
  // with two rows of matrix instructions per unit measured slower that way and keep one unit ahead.
#ifndef FPQ_DEEP_SMALL
#define FPQ_DEEP_SMALL 1
#endif
  constexpr bool kDeep = FPQ_DEEP_SMALL && TN == 1 && !NV;
  constexpr int kSets = kDeep ? 4 : 2;
  uint4 aq[kSets][TN], bq[kSets][TM];
  uint2 sa[TN], sb[TM], sa_next[TN], sb_next[TM];   // MXFP4 uses .x only
  const int a_off = (wn * TN) * 1024 + lane * 16, b_off = (KW + wm * TM) * 1024 + lane * 16;
  const int sa_off = kScaleBase + (wn * TN) * kSB + lane * (kSB / 64);
  const int sb_off = kScaleBase + (KW + wm * TM) * kSB + lane * (kSB / 64);
  auto read_unit = [&](int u, int set) {
    const uint8_t* base = smem + (u % RING) * kUnitBytes;
#pragma unroll
    for (int j = 0; j < TM; ++j) bq[set][j] = *(const uint4*)(base + b_off + j * 1024);
#pragma unroll
    for (int i = 0; i < TN; ++i) aq[set][i] = *(const uint4*)(base + a_off + i * 1024);
  };
  auto read_scales = [&](int blk) {
    const uint8_t* base = smem + (blk % kSlots) * kSlotBytes;
    if (NV) {
#pragma unroll
      for (int j = 0; j < TM; ++j) sb_next[j] = *(const uint2*)(base + sb_off + j * kSB);
#pragma unroll
      for (int i = 0; i < TN; ++i) sa_next[i] = *(const uint2*)(base + sa_off + i * kSB);
    } else {
#pragma unroll
      for (int j = 0; j < TM; ++j) sb_next[j].x = *(const uint32_t*)(base + sb_off + j * kSB);
#pragma unroll
      for (int i = 0; i < TN; ++i) sa_next[i].x = *(const uint32_t*)(base + sa_off + i * kSB);
    }
  };

  // ---- prologue: the first RING units (scales of blocks 0 and 1 with units 0 and 4)
  const int n_pro = min(nkb * 4, RING);
  for (int u = 0; u < n_pro; ++u) issue_unit(u, (u & 3) == 0);
  // Loads complete in order: unit 0 and scale block 0 have landed once at most the loads of the
  // younger units are outstanding (a wave issues kPer per unit, one more with scales).
  if (n_pro == RING) wait_vmem_le<(RING - (kDeep ? 2 : 1)) * kPer>();
  else wait_vmem();
  barrier_lds();
  read_unit(0, 0);
  if constexpr (kDeep) read_unit(1, 1);   // (a K range holds at least four units)
  read_scales(0);
  if constexpr (kDeep) {   // (the first block's scales move into place here, the others' behind the block before)
#pragma unroll
    for (int i = 0; i < TN; ++i) sa[i] = sa_next[i];
#pragma unroll
    for (int j = 0; j < TM; ++j) sb[j] = sb_next[j];
  }

  // One 64-K unit: 16 MFMAs per wave.  After the first row of MFMAs comes the hand-over: every
  // wave holds unit u in registers, so its ring slot is free for unit u + RING, and unit u + 1
  // must have landed for everyone before it is read into the other register set.  The code
  // between two hand-overs is branch-free (the compiler must not move MFMAs across them).
#define FPQ_MFMA_ROW(Q, I)                                                                          \
  if constexpr (NV) {                                                                               \
    const uint4 av = aq[(Q) & 1][I];                                                                \
    const uint32_t aw[4] = {av.x, av.y, av.z, av.w};                                                \
    const uint32_t asc = (Q) < 2 ? sa[I].x : sa[I].y;                                               \
    _Pragma("unroll") for (int s4 = 0; s4 < 4; ++s4) {                                              \
      const v8h ah = dequant8_f16_h(aw[s4], e4m3_byte_f16(asc, 2 * ((Q) & 1) + (s4 >> 1)));         \
      _Pragma("unroll") for (int j = 0; j < TM; ++j)                                                \
        acc[I][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bh[j][s4], acc[I][j], 0, 0, 0);      \
    }                                                                                               \
    __builtin_amdgcn_sched_barrier(0);                                                              \
  } else {                                                                                          \
    const uint4 av = aq[(Q) & (kSets - 1)][I];                                                      \
    const v8i a = v8i{(int)av.x, (int)av.y, (int)av.z, (int)av.w, 0, 0, 0, 0};                      \
    _Pragma("unroll") for (int j = 0; j < TM; ++j) {                                                \
      const uint4 bv = bq[(Q) & (kSets - 1)][j];                                                    \
      const v8i b = v8i{(int)bv.x, (int)bv.y, (int)bv.z, (int)bv.w, 0, 0, 0, 0};                    \
      acc[I][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc[I][j], 4, 4, Q,        \
                                                                  (int)sa[I].x, Q, (int)sb[j].x);   \
    }                                                                                               \
    __builtin_amdgcn_sched_barrier(0);                                                              \
  }
  // NVFP4: the activation operands of the unit, dequantized once for all rows of MFMAs
  v8h bh[NV ? TM : 1][4];
  // NVFP4 on the large tiles (four rows of matrix instructions per wave): a software pipeline over the K steps of 16
  // instead -- while the matrix instructions of step (unit, s4) issue, row by row, the operands of the next step
  // are converted (row i: weight tile i and its share of the activation tiles' halves), and the instruction
  // order is pinned to one matrix instruction followed by its share of the conversions.  The step after a
  // unit's last one belongs to the next unit, whose registers were read at this unit's hand-over (the next
  // block's scales with them); after the last unit of all the conversions run on stale registers and nothing
  // consumes them.  Against converting a unit's activation operands in one block ahead of its matrix instructions
  // (K = 4096, weights from HBM): 256 x 256 tiles, 4096 x 24576 618 -> 570 us (the row-major kernel: 610), 2048 x
  // 14336 197 -> 178; 256 x 128 tiles 52-55 -> 44-48; 128 x 128 tiles with eight waves 2-5 % (640-1024 rows, N =
  // 4096: 30.4-35.4 -> 29.2-34.8); the 64 x 128 tiles measured 1-2 % slower this way and keep the block.
  constexpr bool kNvPipe = NV && TN >= 2 && (2 * TM) % TN == 0;
  constexpr int kHpr = kNvPipe ? 2 * TM / TN : 1;   // halves of activation tiles converted per row
  // conversion instructions behind each matrix instruction of a row (a row converts 9 + 4.5 kHpr for its TM; one
  // more or less measured 1-3 % slower)
  constexpr int kPinValu = TN == 4 ? (TM == 4 ? 5 : 6) : 8;
  v8h ah_c[kNvPipe ? TN : 1], ah_n[kNvPipe ? TN : 1];
  v4h bh_c[kNvPipe ? TM : 1][2], bh_n[kNvPipe ? TM : 1][2];
  auto nv_scale = [&](const uint2& cur, const uint2& next, int qn, int sn, bool nxt) __attribute__((always_inline)) {
    const uint2 sc = nxt ? next : cur;
    return e4m3_byte_f16(qn < 2 ? sc.x : sc.y, 2 * (qn & 1) + (sn >> 1));
  };
  auto nv_dword = [&](const uint4& c, int sn) __attribute__((always_inline)) {
    return sn == 0 ? c.x : sn == 1 ? c.y : sn == 2 ? c.z : c.w;
  };
  auto nv_a = [&](int qn, int sn, int i, bool nxt) __attribute__((always_inline)) {
    return dequant8_f16_h(nv_dword(aq[qn & 1][i], sn), nv_scale(sa[i], sa_next[i], qn, sn, nxt));
  };
  auto nv_b = [&](int qn, int sn, int j, int part, bool nxt) __attribute__((always_inline)) {
    return dequant4_f16_h(nv_dword(bq[qn & 1][j], sn), nv_scale(sb[j], sb_next[j], qn, sn, nxt), part);
  };
  if constexpr (kNvPipe) {   // the first step's operands (block 0's scales are still where they were read ahead)
#pragma unroll
    for (int i = 0; i < TN; ++i) ah_c[i] = nv_a(0, 0, i, true);
#pragma unroll
    for (int j = 0; j < TM; ++j) {
      bh_c[j][0] = nv_b(0, 0, j, 0, true);
      bh_c[j][1] = nv_b(0, 0, j, 1, true);
    }
  }
#define FPQ_PREP_B(Q)                                                                               \
  if constexpr (NV) {                                                                               \
    _Pragma("unroll") for (int j = 0; j < TM; ++j) {                                                \
      const uint4 bv = bq[(Q) & 1][j];                                                              \
      const uint32_t bw[4] = {bv.x, bv.y, bv.z, bv.w};                                              \
      const uint32_t bsc = (Q) < 2 ? sb[j].x : sb[j].y;                                             \
      _Pragma("unroll") for (int s4 = 0; s4 < 4; ++s4)                                              \
        bh[j][s4] = dequant8_f16_h(bw[s4], e4m3_byte_f16(bsc, 2 * ((Q) & 1) + (s4 >> 1)));          \
    }                                                                                               \
  }
  constexpr int kHand = (TM >= 4 || TN <= 2) ? 1 : 2;  // rows of MFMAs ahead of the hand-over
  // ALLOWED: loads of this wave that may still be outstanding while unit u + 1 is complete; READ / READ2: unit
  // u + 1 / u + 2 exists; NEXT_BLOCK: so does the 256-K block after this unit's, whose scales are read into
  // registers at the block's last hand-over (kDeep: at the one before, so that the reads of unit u + 1 are
  // the newest at the start of a block and taking the scales does not wait for them)
#define FPQ_UNIT(Q, U, ALLOWED, ISSUE, READ, NEXT_BLOCK, READ2)                                     \
  if constexpr (kDeep) {                                                                            \
    wait_vmem_le<((ALLOWED) >= kPer ? (ALLOWED) - kPer : 0)>();   /* unit u + 2 is complete */     \
    barrier_lds_but<TN + TM>();                                                                     \
    if (ISSUE) issue_unit((U) + RING, (Q) == 0);                                                   \
    if ((Q) == 2 && (NEXT_BLOCK)) read_scales(((U) + 2) >> 2);                                      \
    if (READ2) read_unit((U) + 2, ((Q) + 2) & 3);                                                   \
    __builtin_amdgcn_sched_barrier(0);                                                              \
    _Pragma("unroll") for (int i1 = 0; i1 < TN; ++i1) FPQ_MFMA_ROW(Q, i1)                           \
  } else if constexpr (kNvPipe) {                                                                   \
    _Pragma("unroll") for (int s4 = 0; s4 < 4; ++s4) {                                              \
      const int qn = s4 == 3 ? ((Q) + 1) & 3 : (Q), sn = s4 == 3 ? 0 : s4 + 1;                      \
      const bool nxt = s4 == 3 && (Q) == 3;   /* the next block's scales */                         \
      _Pragma("unroll") for (int i = 0; i < TN; ++i) {                                              \
        ah_n[i] = nv_a(qn, sn, i, nxt);                                                             \
        _Pragma("unroll") for (int h = i * kHpr; h < (i + 1) * kHpr; ++h)                           \
          bh_n[h >> 1][h & 1] = nv_b(qn, sn, h >> 1, h & 1, nxt);                                   \
        _Pragma("unroll") for (int j = 0; j < TM; ++j)                                              \
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(                                       \
              ah_c[i], __builtin_shufflevector(bh_c[j][0], bh_c[j][1], 0, 1, 2, 3, 4, 5, 6, 7), acc[i][j], 0, 0, 0); \
        _Pragma("unroll") for (int j = 0; j < TM; ++j) {                                            \
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                        \
          __builtin_amdgcn_sched_group_barrier(0x002, kPinValu, 0);                                 \
        }                                                                                           \
        __builtin_amdgcn_sched_barrier(0);                                                          \
      }                                                                                             \
      if (s4 == 0) {                                                                                \
        wait_vmem_le<(ALLOWED)>();                                                                  \
        barrier_lds();                                                                              \
        if (ISSUE) issue_unit((U) + RING, (Q) == 0);                                               \
        if (READ) read_unit((U) + 1, ((Q) + 1) & 1);                                                \
        if ((Q) == 3 && (NEXT_BLOCK)) read_scales(((U) + 1) >> 2);                                  \
        __builtin_amdgcn_sched_barrier(0);                                                          \
      }                                                                                             \
      _Pragma("unroll") for (int i = 0; i < TN; ++i) ah_c[i] = ah_n[i];                             \
      _Pragma("unroll") for (int j = 0; j < TM; ++j) {                                              \
        bh_c[j][0] = bh_n[j][0];                                                                    \
        bh_c[j][1] = bh_n[j][1];                                                                    \
      }                                                                                             \
    }                                                                                               \
  } else {                                                                                          \
    FPQ_PREP_B(Q)                                                                                   \
    _Pragma("unroll") for (int i0 = 0; i0 < kHand; ++i0) FPQ_MFMA_ROW(Q, i0)                        \
    wait_vmem_le<(ALLOWED)>();                                                                      \
    barrier_lds();                                                                                  \
    if (ISSUE) issue_unit((U) + RING, (Q) == 0);                                                   \
    if (READ) read_unit((U) + 1, ((Q) + 1) & 1);                                                    \
    if ((Q) == 3 && (NEXT_BLOCK)) read_scales(((U) + 1) >> 2);                                      \
    __builtin_amdgcn_sched_barrier(0);                                                              \
    _Pragma("unroll") for (int i1 = kHand; i1 < TN; ++i1) FPQ_MFMA_ROW(Q, i1)                       \
  }
#define FPQ_TAKE_SCALES_NOW()                                                                       \
  {                                                                                                 \
    _Pragma("unroll") for (int i = 0; i < TN; ++i) sa[i] = sa_next[i];                              \
    _Pragma("unroll") for (int j = 0; j < TM; ++j) sb[j] = sb_next[j];                              \
  }
  // The scales of a block move into place at its start; kDeep: at the end of the block before (behind its last
  // matrix instructions, in straight-line code, where the compiler sees that only the operand reads issued
  // since may still be outstanding: at the head of the loop it waits for every LDS read instead)
#define FPQ_TAKE_SCALES()                                                                           \
  if constexpr (!kDeep) FPQ_TAKE_SCALES_NOW()
#define FPQ_TAKE_SCALES_AFTER()                                                                     \
  if constexpr (kDeep) {   /* (moves the compiler may not turn into copies at the head of the loop) */ \
    _Pragma("unroll") for (int i = 0; i < TN; ++i)                                                  \
      asm volatile("v_mov_b32 %0, %1" : "=v"(sa[i].x) : "v"(sa_next[i].x));                         \
    _Pragma("unroll") for (int j = 0; j < TM; ++j)                                                  \
      asm volatile("v_mov_b32 %0, %1" : "=v"(sb[j].x) : "v"(sb_next[j].x));                         \
  }

  // steady state: every unit of these blocks still has a unit RING ahead of it to issue
  constexpr int kDrain = RING / 4;   // blocks in the last ring of units
  const int kb_tail = max(nkb - kDrain, 0);
  for (int kb = 0; kb < kb_tail; ++kb) {
    const int u0 = kb * 4;
    FPQ_TAKE_SCALES()
    FPQ_UNIT(0, u0 + 0, (RING - 2) * kPer, true, true, true, true)
    FPQ_UNIT(1, u0 + 1, (RING - 2) * kPer, true, true, true, true)
    FPQ_UNIT(2, u0 + 2, (RING - 2) * kPer, true, true, true, true)
    FPQ_UNIT(3, u0 + 3, (RING - 2) * kPer, true, true, true, true)
    FPQ_TAKE_SCALES_AFTER()
  }
  // drain: the last ring of units (fewer if K is short); nothing is issued any more, and with t
  // units to go after unit u + 1 exactly t * kPer loads may stay outstanding.  Block D of the kDrain last ones:
#define FPQ_DRAIN_BLOCK(D)                                                                          \
  if constexpr (kDrain > (D)) {                                                                     \
    constexpr int kLeft = 4 * (kDrain - 1 - (D));   /* units behind this block */                   \
    if (kLeft == 0 || nkb >= kDrain - (D)) {   /* (the last block always exists) */                 \
      const int u0 = (nkb - (kDrain - (D))) * 4;                                                    \
      FPQ_TAKE_SCALES()                                                                             \
      FPQ_UNIT(0, u0 + 0, (kLeft + 2) * kPer, false, true, kLeft > 0, true)                         \
      FPQ_UNIT(1, u0 + 1, (kLeft + 1) * kPer, false, true, kLeft > 0, true)                         \
      FPQ_UNIT(2, u0 + 2, kLeft * kPer, false, true, kLeft > 0, kLeft > 0)                          \
      FPQ_UNIT(3, u0 + 3, (kLeft > 0 ? kLeft - 1 : 0) * kPer, false, kLeft > 0, kLeft > 0, kLeft > 0) \
      if constexpr (kLeft > 0) FPQ_TAKE_SCALES_AFTER()                                              \
    }                                                                                               \
  }
  FPQ_DRAIN_BLOCK(0)
  FPQ_DRAIN_BLOCK(1)
  FPQ_DRAIN_BLOCK(2)
  FPQ_DRAIN_BLOCK(3)
#undef FPQ_DRAIN_BLOCK
#undef FPQ_UNIT
#undef FPQ_PREP_B
#undef FPQ_MFMA_ROW
#undef FPQ_TAKE_SCALES
#undef FPQ_TAKE_SCALES_NOW
#undef FPQ_TAKE_SCALES_AFTER

  if constexpr (GR == 2) {
    // The second group's accumulators go to the first through LDS (the rings are idle: every wave has waited
    // for its last loads and read its last unit), added in a fixed order; then the second group only keeps
    // the first company at the one barrier of the epilogue.  (Launched with K whole per workgroup: ksplit = 1.)
    __syncthreads();
    float* xch = (float*)smem_all + wave * (TN * TM * 16 * 64) + lane;
    if (grp == 1) {
#pragma unroll
      for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
          for (int v = 0; v < 16; ++v) xch[((i * TM + j) * 16 + v) * 64] = acc[i][j][v];
    }
    __syncthreads();
    if (grp == 1) {
      __syncthreads();
      return;
    }
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
      for (int j = 0; j < TM; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] += xch[((i * TM + j) * 16 + v) * 64];
  }
  if (GR == 1 && kCanSplit && ksplit > 1) {
    // The parts of a tile run on different XCDs, whose L2 caches are not coherent with each other for
    // ordinary accesses: every access to the workspace is a relaxed device-scope atomic, every wave waits
    // for its stores to be acknowledged before the workgroup moves the tile's counter, and the workgroup
    // that arrives last adds all parts in part order (its own read back like the others), so the sum does
    // not depend on the order of arrival.  Register v of accumulator tile t of wave w: float
    // ((w * TN * TM + t) * 16 + v) * 64 + lane of the part.  The counter is left at zero.  (Sixteen-byte
    // accesses with the same cache policy measured no faster than these four-byte ones: the exchange is
    // bound by its volume, M x N x 4 bytes per part written and read.)
    constexpr int kPart = NW * TN * TM * 16 * 64;   // floats per part
    float* mine = partial + ((size_t)logical * ksplit + blockIdx.y) * kPart + wave * (TN * TM * 16 * 64) + lane;
#pragma unroll
    for (int i = 0; i < TN; ++i)
#pragma unroll
      for (int j = 0; j < TM; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v)
          __hip_atomic_store(mine + ((i * TM + j) * 16 + v) * 64, acc[i][j][v], __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();   // (every wave is past its last LDS read as well: the first word may be reused)
    unsigned* arrival = (unsigned*)smem;
    if (threadIdx.x == 0)
      *arrival = __hip_atomic_fetch_add(counters + logical, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    // (one value for the workgroup: all its waves leave or all stay for the barriers of the epilogue)
    if (__builtin_amdgcn_readfirstlane(*arrival) != (unsigned)(ksplit - 1)) return;
    const float* all = partial + (size_t)logical * ksplit * kPart + wave * (TN * TM * 16 * 64) + lane;
    for (int part = 0; part < ksplit; ++part) {
#pragma unroll
      for (int i = 0; i < TN; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const float p = __hip_atomic_load(all + (size_t)part * kPart + ((i * TM + j) * 16 + v) * 64,
                                              __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            acc[i][j][v] = part == 0 ? p : acc[i][j][v] + p;
          }
    }
    if (threadIdx.x == 0) __hip_atomic_store(counters + logical, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }

  const OutView out = out_view(seg, y, bias, n_blk + wn * TN * 32, N);
  wave_tile_store<TN, TM, packed_lds_alloc(kBlocks, NV, RING, TN * 32, TM * 32, GR), NW>(
      acc, smem_all, out.y, out.bias, alpha_p, out.n0, m_blk + wm * TM * 32, wave, lane, M, out.N, residual);
}

}  // namespace fpq

#ifndef FPQ_NV_STREAM_ROWS
#define FPQ_NV_STREAM_ROWS 128  // NVFP4: up to this many rows the weight-streaming kernel (where its plan applies)
#endif
#ifndef FPQ_PACKED_HALF_TILES
#define FPQ_PACKED_HALF_TILES 1  // large M: 1 = 256x128 tiles for MXFP4, 2 = for NVFP4 too, 0 = 256x256
#endif
// Shape thresholds that stand for a share of the chip are multiples of the device's compute-unit count
// (measured on the 256 CUs of an MI355X, where they come to the figures in the comments):
//   row slabs of the streaming kernel x weight tiles: at most one workgroup per CU (256)
//   up to CUs / 2 tiles of 128 x 128 (128): 64 x 128 tiles instead
//   up to CUs tiles of 128 x 128 (256): those; beyond, tiles of 256 x 128 or (NVFP4, by round counts) 256 x 256
static inline int64_t slab_workgroups(int cus) { return cus; }
static inline int64_t narrow_below(int cus) { return cus / 2; }

namespace fpq {
// A K split of a tile kernel (ksplit > 1): `workspace` = kStreamCounterBytes of counters, all zero, then
// one fp32 part of the workgroup tile per (tile, split).
struct TileSplit {
  int ksplit = 1;   // parts of K, one grid plane each
  int bps = 0;      // 256-K blocks per part (the last part may have fewer, never none)
};

template <int NT, int KW, int MT, int WN, int WM, bool NV, int RING = kRing, int GR = 1>
static int launch_packed(const void* xq, const void* xs, const void* wq, const void* ws, const float* alpha,
                         const void* bias, void* y, int64_t M, int64_t N, int64_t K, hipStream_t stream,
                         const void* residual, const OutSegments& seg, TileSplit split = TileSplit{},
                         void* workspace = nullptr) {
  constexpr int kLds = packed_lds_alloc(KW + MT, NV, RING, NT / WN * 32, MT / WM * 32, GR);
  static_assert(kLds <= 160 * 1024, "more LDS than a CU has");
  const int tiles_m = (int)((M + MT * 32 - 1) / (MT * 32)), tiles_n = (int)((N + NT * 32 - 1) / (NT * 32));
  if (split.ksplit <= 1 || !workspace || NT * MT > 16 || GR > 1) split = TileSplit{1, (int)(K / 256)};
  if (GR > 1) {   // the two groups of a workgroup take one half of K each (the caller checked that K / 256 is even)
    if ((K / 256) % GR != 0) return FPQ_E_UNSUPPORTED;
    split.bps = (int)(K / 256) / GR;
  }
  static LdsLimitOnce lds_limit;
  if (const int st = lds_limit.ensure((const void*)gemm_fp4_packed_kernel<NT, KW, MT, WN, WM, NV, RING, GR>, kLds)) return st;
  hipLaunchKernelGGL((gemm_fp4_packed_kernel<NT, KW, MT, WN, WM, NV, RING, GR>),
                     dim3((unsigned)(tiles_m * tiles_n), (unsigned)split.ksplit), dim3(256 * GR), kLds, stream,
                     (const uint8_t*)xq, (const uint8_t*)xs, (const uint8_t*)wq, (const uint8_t*)ws, alpha,
                     (const uint16_t*)bias, (uint16_t*)y, (int)M, (int)N, (int)K, tiles_m,
                     (const uint16_t*)residual, seg, split.ksplit, split.bps,
                     workspace ? (float*)((uint8_t*)workspace + kTileCounterBytes) : nullptr, (unsigned*)workspace);
  return (int)hipGetLastError();
}

// Which shapes split K in the tile kernels, and how.  Shapes of a few hundred rows on few weight rows and a
// long K (a down-projection at 257-512 rows: 64-256 workgroups, each walking all of K, against a few
// microseconds of arithmetic) get up to two workgroups per CU by cutting K, every part keeping at least
// kTileSplitMinBlocks blocks of 256; fewer parts if the workspace is small.  `part_bytes`: one fp32 part of the
// kernel's workgroup tile.  The exchange moves M x N x 4 bytes per part each way, about as much as the
// operands themselves, so the split only pays where the main loop is slow for other reasons -- NVFP4, whose
// loop is bound by the in-register dequantization (N = 4096: K = 14336, 384 rows 79.6 -> 69.8 us; K = 12288,
// 512 rows 69.2 -> 65.2).  MXFP4 measured slower with it (N = 4096, K = 14336: 256 rows 19.5 -> 21.5 us,
// 512 rows 29.0 -> 29.8; doubling the workgroups and halving their K left the time where it was: these tiles
// are bound by what a CU can have in flight from the L2, not by the length of a workgroup's loop) and does not split.
constexpr int64_t kTileSplitMinBlocks = FPQ_TILE_SPLIT_MIN_BLOCKS;
static TileSplit tile_split_plan(int64_t tiles, int64_t K, int64_t part_bytes, int64_t workspace_bytes, int cus) {
  TileSplit plan{1, (int)(K / 256)};
  const int64_t nkb = K / 256;
  if (tiles < 1 || tiles > kTileCounters || tiles > cus) return plan;
  int64_t ksplit = 2 * (int64_t)cus / tiles;
  if (ksplit > nkb / kTileSplitMinBlocks) ksplit = nkb / kTileSplitMinBlocks;
  while (ksplit > 1 && kTileCounterBytes + ksplit * tiles * part_bytes > workspace_bytes) --ksplit;
  if (ksplit <= 1) return plan;
  const int64_t bps = (nkb + ksplit - 1) / ksplit;
  plan.ksplit = (int)((nkb + bps - 1) / bps);   // no empty part
  plan.bps = (int)bps;
  return plan;
}

// The tile kernel a shape beyond the weight-streaming kernel's reach runs, and its K split.
struct TilePlan {
  int kind;          // 0: 64 x 128 tiles, 1: 128 x 128, 2: 256 x 128 (MXFP4), 3: 256 x 256
  int64_t tiles;
  int64_t part_bytes;
  TileSplit split;
  int groups;        // 2: workgroups of eight waves, K halved inside the workgroup (no K split across workgroups then)
};
template <bool NV>
static TilePlan tile_plan(int64_t M, int64_t N, int64_t K, int64_t workspace_bytes, int cus) {
  TilePlan plan{};
  plan.groups = 1;
  const int64_t big_tiles = ((M + 255) / 256) * ((N + 255) / 256);
  const int64_t tiles128 = ((M + 127) / 128) * ((N + 127) / 128);
  const bool ragged = ((M + 127) / 128) % 2 == 1;   // the last 256 activation rows of the large tiles would be half empty
  if (((M + 127) / 128) * ((N + 127) / 128) <= narrow_below(cus)) {
    plan.kind = 0;
    plan.tiles = ((M + 127) / 128) * ((N + 63) / 64);
    plan.part_bytes = 4 * 64 * 32 * 4;     // four waves of 32 x 64: two accumulator tiles per lane
  } else if (tiles128 <= cus) {
    // MXFP4: 128 x 128 tiles while every workgroup has a CU to itself -- two of them on a CU wait on its LDS, and
    // with the weights from HBM the 256 x 128 tiles are faster from there on (us, K = 4096: 256 rows, N = 20480 /
    // 24576 23.0 / 23.9 -> 20.3 / 21.2; 512 rows, N = 12288 22.0 -> 20.0; 768 rows, N = 8192 21.4 -> 19.0; 1024 rows,
    // N = 6144 21.1 -> 19.4; at exactly one tile per CU the small tiles win: 1024 rows, N = 4096 13.6 against 18.6).
    // NVFP4 likewise (the small tiles ran up to 400 of them before): K = 4096, 512 rows, N = 12288 60.3 -> 56.2 us;
    // 768 rows, N = 8192 59.9 -> 54.9; 256 rows, N = 24576 61.1 -> 55.9; K = 12288, 512 rows, N = 12288 170 -> 153.
    plan.kind = 1;
    plan.tiles = ((M + 127) / 128) * ((N + 127) / 128);
    plan.part_bytes = 4 * 64 * 64 * 4;     // four waves of 64 x 64
  } else {
    // MXFP4: 256 x 128 tiles.  NVFP4: 256 x 256 tiles (one workgroup per CU) do a given amount of work 4 % faster,
    // 256 x 128 tiles (two per CU; alone on a CU one takes 0.54 of a large tile's time) waste less of the last
    // round and of a row count that is an odd number of 128s -- whichever the round counts favour (K = 4096:
    // 4096 rows, N = 6144 197 -> 164 us; 128 rows, N = 28672 97 -> 41, now 128 x 128 tiles; 384 rows, N = 14336
    // 96 -> 54; 896 rows, N = 8192 98 -> 57; 4096 rows, N = 24576 633 / 625 and K = 12288, N = 4096 302 / 314
    // stay with the large tiles).
    const int64_t half_tiles = ((M + 127) / 128) * ((N + 255) / 256);
    const int64_t rounds = half_tiles / (2 * cus), rest = half_tiles % (2 * cus);
    const int64_t cost_half = rounds * 104 + (rest == 0 ? 0 : rest <= cus ? 54 : 104);
    const int64_t cost_large = (big_tiles + cus - 1) / cus * 100;
    const bool half = !NV || FPQ_PACKED_HALF_TILES > 1 || cost_half + (ragged ? 0 : 4) <= cost_large;
    plan.kind = half && FPQ_PACKED_HALF_TILES ? 2 : 3;
    plan.split = TileSplit{1, (int)(K / 256)};
    return plan;
  }
  plan.split = TileSplit{1, (int)(K / 256)};
  // NVFP4 with at most one workgroup per CU: two groups of four waves per workgroup, one half of K each (the
  // in-register conversions of one wave overlap the matrix instructions of the other on its SIMD, and the halves
  // meet in LDS): 300-512 rows, N = 4096, K = 4096 25.9 -> 23.4 us; 640-1024 rows 34.9-37.3 -> 32.2-35.6;
  // N = 12288, 129-256 rows 35.1 -> 32.9; K = 12288, 384 / 512 rows 69 / 70 -> 59.3 / 62.7 (a K split across two
  // workgroups through the caller's workspace: 61.1 / 65.3).  MXFP4, whose waves wait on what the CU receives
  // from the L2, measured the same with 64 x 128 tiles and 8 % slower with 128 x 128: it keeps four waves.
  if (NV && plan.tiles <= cus && (K / 256) % 2 == 0 && K >= 2048) {
    plan.groups = 2;
    return plan;
  }
  // (NVFP4 beyond the 256 rows that two passes of the weight-streaming kernel serve better)
  if (NV && M > 2 * FPQ_NV_STREAM_ROWS) plan.split = tile_split_plan(plan.tiles, K, plan.part_bytes, workspace_bytes, cus);
  return plan;
}

// fpq_gemm_stream.hip: the weight-streaming kernel for at most 128 activation rows
bool stream_eligible(bool nv, int64_t M, int64_t N, int64_t K);
int64_t gemm_mxf4_stream_workspace_bytes(int64_t M, int64_t N, int64_t K);
int gemm_fp4_stream(bool nv, const void* xq, const void* xs, const void* wq, const void* ws, const float* alpha,
                    const void* bias, const void* residual, void* y, int64_t M, int64_t N, int64_t K,
                    void* workspace, int64_t workspace_bytes, const OutSegments& seg, hipStream_t stream);
int gemm_fp4_stream_slabs(bool nv, const void* xq, const void* xs, const void* wq, const void* ws,
                          const float* alpha, const void* bias, const void* residual, void* y, int64_t M, int64_t N,
                          int64_t K, int64_t slab_rows, const OutSegments& seg, hipStream_t stream);

template <bool NV>
static int gemm_packed(const void* xq, const void* xs, const void* wq, const void* ws, const float* alpha,
                       const void* bias, void* y, int64_t M, int64_t N, int64_t K, void* stream,
                       const void* residual = nullptr, void* workspace = nullptr, int64_t workspace_bytes = 0,
                       const OutSegments& seg = OutSegments{});

template <bool NV>
static int pack_operand(const void* codes, const void* scales, int64_t scale_stride, int64_t rows, int64_t K,
                        void* packed_codes, void* packed_scales, void* stream) {
  constexpr int GROUP = NV ? 16 : 32;
  if (rows < 0 || K < 0) return FPQ_E_SHAPE;
  if (rows == 0) return FPQ_OK;
  if (!codes || !scales || !packed_codes || !packed_scales) return FPQ_E_NULL;
  if (K == 0 || K % 256 != 0 || scale_stride < K / GROUP) return FPQ_E_SHAPE;
  if (rows > (1 << 24) || K > (1 << 24)) return FPQ_E_SHAPE;
  if (((uintptr_t)codes & 15u) || ((uintptr_t)packed_codes & 15u) || ((uintptr_t)packed_scales & 7u))
    return FPQ_E_ALIGN;
  const dim3 grid((unsigned)(K / 256), (unsigned)((rows + 31) / 32));
  hipLaunchKernelGGL(pack_fp4_kernel<NV>, grid, dim3(256), 0, (hipStream_t)stream, (const uint8_t*)codes,
                     (const uint8_t*)scales, scale_stride, (int)rows, (int)K, (uint8_t*)packed_codes,
                     (uint8_t*)packed_scales);
  return (int)hipGetLastError();
}
}  // namespace fpq

namespace fpq {
template <bool NV>
static int gemm_packed(const void* xq, const void* xs, const void* wq, const void* ws, const float* alpha,
                       const void* bias, void* y, int64_t M, int64_t N, int64_t K, void* stream,
                       const void* residual, void* workspace, int64_t workspace_bytes, const OutSegments& seg) {
  if (M < 0 || N < 0 || K < 0 || workspace_bytes < 0) return FPQ_E_SHAPE;
  if (M == 0 || N == 0) return FPQ_OK;
  if (!xq || !xs || !wq || !ws || !alpha || !y) return FPQ_E_NULL;
  if (K == 0 || K % 256 != 0) return FPQ_E_SHAPE;
  if (M > (1 << 24) || N > (1 << 24) || K > (1 << 24)) return FPQ_E_SHAPE;
  // scale offsets inside one operand are 32-bit
  const int64_t sdiv = NV ? 16 : 32;
  if (((M + 31) / 32) * 32 * (K / sdiv) >= ((int64_t)1 << 32) || ((N + 31) / 32) * 32 * (K / sdiv) >= ((int64_t)1 << 32))
    return FPQ_E_SHAPE;
  if (((uintptr_t)xq & 15u) || ((uintptr_t)wq & 15u) || ((uintptr_t)xs & 15u) || ((uintptr_t)ws & 15u) ||
      ((uintptr_t)y & 15u) || ((uintptr_t)residual & 15u))
    return FPQ_E_ALIGN;
  if ((uintptr_t)workspace & 255u) return FPQ_E_ALIGN;
  // Few weight tiles: the rows are cut into slabs, one grid plane of the weight-streaming kernel each, as low as
  // keeps slabs x weight tiles within one round of the 256 CUs -- more workgroups that each hold fewer
  // activation row tiles (fewer registers, less to re-read per weight tile, a shorter tail) and that, unlike
  // the tile kernels', share nothing through LDS and meet at no barrier in their K loop.  Slabs of 32 / 64 /
  // 96 / 128 rows measured best exactly where they are the lowest that fit (us, K = 4096, against one
  // workgroup per weight tile or the tile kernels): N = 4096: 64 rows 6.3 -> 5.3, 128 rows 8.0 -> 6.2, 256
  // rows 9.9 -> 8.0; N = 2048: 128 rows 7.8 -> 5.1, 256 rows 7.6 -> 6.0 (tiles: 9.5), 384 rows 9.6 -> 6.9;
  // N = 1024: 512 rows 9.5 -> 5.5; NVFP4 N = 4096: 128 rows 14.1 -> 9.3, 256 rows 28 -> 14.1; K = 14336, 256
  // rows: 32 -> 19.  (More slabs than one round -- two or three workgroups per CU -- measured slower.)  K
  // stays whole in slabs, so a shape whose K the caller's workspace lets split keeps the split up to 96 rows
  // (N = 4096, K = 14336: 64 rows 11.7 split / 11.9 us in slabs, 96 rows 13.9 / 13.9, 128 rows 15.4 / 14.1).
  const int cus = device_cus();
  // A tile kernel that splits K through the caller's workspace comes before the row slabs.
  const TilePlan plan = tile_plan<NV>(M, N, K, workspace ? workspace_bytes : 0, cus);
  const bool tile_splits = FPQ_TILE_SPLIT_OVER_SLABS && plan.split.ksplit > 1;
  {
    const int64_t tiles = (N + 31) / 32;
    const bool splits = tile_splits || (workspace && workspace_bytes > 16384 && M <= 96 &&
                                        gemm_mxf4_stream_workspace_bytes(M, N, K) > 0);
    for (int64_t cap = 32; cap <= 128 && !splits; cap += 32) {
      const int64_t slabs = (M + cap - 1) / cap;
      if (slabs * tiles > slab_workgroups(cus)) continue;
      const int64_t rows = ((M + slabs - 1) / slabs + 31) / 32 * 32;   // rows of a slab, whole 32-row tiles
      if (slabs > 1 && rows < M && stream_eligible(NV, rows, N, K))
        return gemm_fp4_stream_slabs(NV, xq, xs, wq, ws, alpha, bias, residual, y, M, N, K, rows, seg,
                                     (hipStream_t)stream);
      break;   // one slab, or a shape the kernel does not take: the paths below
    }
  }
  if (stream_eligible(NV, M, N, K) && (!NV || M <= FPQ_NV_STREAM_ROWS))
    return gemm_fp4_stream(NV, xq, xs, wq, ws, alpha, bias, residual, y, M, N, K, workspace, workspace_bytes,
                           seg, (hipStream_t)stream);
  if constexpr (NV) {
    // 129-256 rows of NVFP4 at up to 256 weight tiles (N <= 8192): the 128x128 tile kernel fills at most
    // half of the 256 CUs with workgroups that take 34 us for K = 4096, so two passes of the weight-streaming
    // kernel over one half of the rows each are faster although the second re-reads the weights (from the
    // last-level cache): N = 6144, K = 4096: 192 rows 35.2 -> 23.1 us, 256 rows 34.8 -> 28.6; N = 4096, K =
    // 12288: 97 -> 52 / 68 us.  (The tile kernel's time stays at one round up to N = 16384, where two passes
    // take 44-55 us; three passes for more rows measured slower than the tiles as well.)  Where the tile
    // kernels halve K inside their workgroups they take 23 us for K = 4096 at any of these row counts and the
    // two passes are ahead up to 192 rows only (weights from HBM; N = 6144: 144 rows 22.5 two passes / 25.8 us
    // tiles, 192 rows 23.7 / 23.6, 224 rows 26.7 / 23.5, 256 rows 28.7 / 22.9; N = 8192, K = 8192: 35.7 / 43.4,
    // 39.5 / 42.6, 45.5 / 43.1, 49.7 / 42.8).
    const int64_t half = ((M + 1) / 2 + 31) / 32 * 32;   // rows of the first pass, whole 32-row tiles
    const int64_t two_pass_rows = plan.groups == 2 ? 192 : 2 * FPQ_NV_STREAM_ROWS;
    if (!tile_splits && M > FPQ_NV_STREAM_ROWS && M <= two_pass_rows && (N + 31) / 32 <= cus &&
        stream_eligible(true, half, N, K)) {
      // (both passes may split K through the caller's workspace: they run one after the other on the stream)
      const int rc = gemm_fp4_stream(true, xq, xs, wq, ws, alpha, bias, residual, y, half, N, K, workspace,
                                     workspace_bytes, seg, (hipStream_t)stream);
      if (rc != FPQ_OK) return rc;
      OutSegments rest = seg;
      for (int i = 0; i < seg.count; ++i)
        rest.y[i] = seg.y[i] + (size_t)half * (seg.end[i] - (i ? seg.end[i - 1] : 0));
      return gemm_fp4_stream(true, (const uint8_t*)xq + (size_t)half * (K / 2), (const uint8_t*)xs + (size_t)half * (K / 16),
                             wq, ws, alpha, bias, residual ? (const uint16_t*)residual + (size_t)half * N : nullptr,
                             (uint16_t*)y + (size_t)half * N, M - half, N, K, workspace, workspace_bytes, rest,
                             (hipStream_t)stream);
    }
  }
  // At most 128 tiles of 128 x 128 would leave half of the CUs idle: 64 x 128 tiles (twice the workgroups, the
  // same accumulation order and bits) take 25 instead of 34.5 us for NVFP4 at 257-512 rows, N = 4096, K = 4096
  // (K = 12288: 69 instead of 97 us) and 4-7 % less for MXFP4; with more tiles they measured 14 % slower.
  // Either of these two kernels splits K through the caller's workspace where that fills the CUs (tile_split_plan).
  if constexpr (NV) {
    if (plan.groups == 2 && plan.kind == 0)
      return launch_packed<2, 4, 4, 2, 2, true, kRing, 2>(xq, xs, wq, ws, alpha, bias, y, M, N, K, (hipStream_t)stream,
                                                          residual, seg);
    if (plan.groups == 2 && plan.kind == 1)
      return launch_packed<4, 4, 4, 2, 2, true, kRing, 2>(xq, xs, wq, ws, alpha, bias, y, M, N, K, (hipStream_t)stream,
                                                          residual, seg);
  }
  if (plan.kind == 0)
    return launch_packed<2, 4, 4, 2, 2, NV>(xq, xs, wq, ws, alpha, bias, y, M, N, K, (hipStream_t)stream, residual, seg,
                                            plan.split, workspace);
  if (plan.kind == 1)
    return launch_packed<4, 4, 4, 2, 2, NV>(xq, xs, wq, ws, alpha, bias, y, M, N, K, (hipStream_t)stream, residual, seg,
                                            plan.split, workspace);
  // 256 x 128 tiles that have a CU to themselves and a long K: a ring of eight units.  Four units are 48 KB in
  // flight per CU, less than the weights' way from HBM takes at the rate one workgroup consumes them (two
  // workgroups per CU have 96 KB); weights from HBM, N = 4096, K = 14336: 1280 rows 59.6 -> 56.4 us, 1536 rows
  // 58.1 -> 53.6; N = 8192, K = 8192, 640 rows 35.3 -> 32.8 (from the caches 4-10 % slower; K = 4096 and NVFP4
  // measured the same either way and keep four).
  if constexpr (!NV) {
    if (plan.kind == 2 && K >= 8192 && ((M + 127) / 128) * ((N + 255) / 256) <= cus)
      return launch_packed<8, 8, 4, 2, 2, false, 8>(xq, xs, wq, ws, alpha, bias, y, M, N, K, (hipStream_t)stream,
                                                    residual, seg);
  }
  if (plan.kind == 2)
    return launch_packed<8, 8, 4, 2, 2, NV, 4>(xq, xs, wq, ws, alpha, bias, y, M, N, K, (hipStream_t)stream, residual, seg);
  return launch_packed<8, 8, 8, 2, 2, NV>(xq, xs, wq, ws, alpha, bias, y, M, N, K, (hipStream_t)stream, residual, seg);
}
}  // namespace fpq

extern "C" int64_t fpq_packed_codes_bytes(int64_t rows, int64_t K) {
  return ((rows + 31) / 32) * 32 * (K / 2);
}

extern "C" int64_t fpq_packed_scales_bytes(int64_t rows, int64_t K) {
  return ((rows + 31) / 32) * 32 * (K / 32);
}

extern "C" int64_t fpq_packed_scales_bytes_nv(int64_t rows, int64_t K) {
  return ((rows + 31) / 32) * 32 * (K / 16);
}

extern "C" int fpq_pack_mxf4(const void* codes, const void* scales, int64_t scale_stride, int64_t rows,
                             int64_t K, void* packed_codes, void* packed_scales, void* stream) {
  return fpq::pack_operand<false>(codes, scales, scale_stride, rows, K, packed_codes, packed_scales, stream);
}

namespace fpq {
template <bool NV>
static int unpack_operand(const void* packed_codes, const void* packed_scales, int64_t rows, int64_t K, void* codes,
                          void* scales, int64_t scale_stride, void* stream) {
  constexpr int GROUP = NV ? 16 : 32;
  if (rows < 0 || K < 0) return FPQ_E_SHAPE;
  if (rows == 0) return FPQ_OK;
  if (!codes || !scales || !packed_codes || !packed_scales) return FPQ_E_NULL;
  if (K == 0 || K % 256 != 0 || scale_stride < K / GROUP) return FPQ_E_SHAPE;
  if (rows > (1 << 24) || K > (1 << 24)) return FPQ_E_SHAPE;
  if (((uintptr_t)codes & 15u) || ((uintptr_t)packed_codes & 15u) || ((uintptr_t)packed_scales & (NV ? 7u : 3u)))
    return FPQ_E_ALIGN;
  const dim3 grid((unsigned)(K / 256), (unsigned)((rows + 31) / 32));
  hipLaunchKernelGGL(unpack_fp4_kernel<NV>, grid, dim3(256), 0, (hipStream_t)stream, (const uint8_t*)packed_codes,
                     (const uint8_t*)packed_scales, (int)rows, (int)K, (uint8_t*)codes, (uint8_t*)scales,
                     scale_stride);
  return (int)hipGetLastError();
}
}  // namespace fpq

extern "C" int fpq_unpack_mxf4(const void* packed_codes, const void* packed_scales, int64_t rows, int64_t K,
                               void* codes, void* scales, int64_t scale_stride, void* stream) {
  return fpq::unpack_operand<false>(packed_codes, packed_scales, rows, K, codes, scales, scale_stride, stream);
}

extern "C" int fpq_unpack_nvf4(const void* packed_codes, const void* packed_scales, int64_t rows, int64_t K,
                               void* codes, void* scales, int64_t scale_stride, void* stream) {
  return fpq::unpack_operand<true>(packed_codes, packed_scales, rows, K, codes, scales, scale_stride, stream);
}

extern "C" int fpq_pack_nvf4(const void* codes, const void* scales, int64_t scale_stride, int64_t rows,
                             int64_t K, void* packed_codes, void* packed_scales, void* stream) {
  return fpq::pack_operand<true>(codes, scales, scale_stride, rows, K, packed_codes, packed_scales, stream);
}

extern "C" int fpq_gemm_mxf4_packed(const void* xq, const void* xs, const void* wq, const void* ws,
                                    const float* alpha, const void* bias, void* y, int64_t M,
                                    int64_t N, int64_t K, void* stream) {
  return fpq::gemm_packed<false>(xq, xs, wq, ws, alpha, bias, y, M, N, K, stream);
}

extern "C" int fpq_gemm_mxf4_packed_residual(const void* xq, const void* xs, const void* wq, const void* ws,
                                             const float* alpha, const void* bias, const void* residual, void* y,
                                             int64_t M, int64_t N, int64_t K, void* stream) {
  if (!residual) return FPQ_E_NULL;
  return fpq::gemm_packed<false>(xq, xs, wq, ws, alpha, bias, y, M, N, K, stream, residual);
}

namespace fpq {
int gemm_mxf4_packed_any(const void* xq, const void* xs, const void* wq, const void* ws, const float* alpha,
                         const void* bias, const void* residual, void* y, int64_t M, int64_t N, int64_t K,
                         void* workspace, int64_t workspace_bytes, void* stream) {
  return gemm_packed<false>(xq, xs, wq, ws, alpha, bias, y, M, N, K, stream, residual, workspace,
                            workspace ? workspace_bytes : 0);
}
}  // namespace fpq

extern "C" int64_t fpq_gemm_mxf4_packed_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  return fpq::gemm_mxf4_stream_workspace_bytes(M, N, K);
}

extern "C" int64_t fpq_gemm_nvf4_packed_workspace_bytes(int64_t M, int64_t N, int64_t K) {
  if (M < 1 || N < 1 || K < 256 || K % 256 != 0) return 0;
  int64_t need = 0;
  if (M <= FPQ_NV_STREAM_ROWS) {
    need = fpq::gemm_mxf4_stream_workspace_bytes(M, N, K);
  } else if (M <= 2 * FPQ_NV_STREAM_ROWS) {   // two passes, the first over `half` rows
    need = fpq::gemm_mxf4_stream_workspace_bytes(((M + 1) / 2 + 31) / 32 * 32, N, K);
  }
  // a tile kernel: what its K split, if it makes one, exchanges
  const fpq::TilePlan plan = fpq::tile_plan<true>(M, N, K, (int64_t)1 << 62, fpq::device_cus());
  const int64_t tile = plan.split.ksplit > 1
                           ? fpq::kTileCounterBytes + plan.split.ksplit * plan.tiles * plan.part_bytes : 0;
  return tile > need ? tile : need;
}

extern "C" int fpq_gemm_mxf4_packed_splitk(const void* xq, const void* xs, const void* wq, const void* ws,
                                           const float* alpha, const void* bias, const void* residual, void* y,
                                           int64_t M, int64_t N, int64_t K, void* workspace,
                                           int64_t workspace_bytes, void* stream) {
  return fpq::gemm_mxf4_packed_any(xq, xs, wq, ws, alpha, bias, residual, y, M, N, K, workspace, workspace_bytes,
                                   stream);
}

extern "C" int fpq_gemm_nvf4_packed_splitk(const void* xq, const void* xs, const void* wq, const void* ws,
                                           const float* alpha, const void* bias, const void* residual, void* y,
                                           int64_t M, int64_t N, int64_t K, void* workspace,
                                           int64_t workspace_bytes, void* stream) {
  return fpq::gemm_packed<true>(xq, xs, wq, ws, alpha, bias, y, M, N, K, stream, residual, workspace,
                                workspace ? workspace_bytes : 0);
}

namespace fpq {
template <bool NV>
static int gemm_packed_multi(const void* xq, const void* xs, const void* wq, const void* ws, const float* alpha,
                             const void* bias, void* const* ys, const int64_t* ns, int64_t count, int64_t M,
                             int64_t K, void* stream) {
  if (count < 1 || count > kMaxSegments) return FPQ_E_SHAPE;
  if (!ys || !ns) return FPQ_E_NULL;
  OutSegments seg{};
  int64_t N = 0;
  for (int64_t i = 0; i < count; ++i) {
    if (ns[i] < 1 || ns[i] % kSegmentAlign != 0 || N + ns[i] > (1 << 24)) return FPQ_E_SHAPE;
    if (M > 0 && !ys[i]) return FPQ_E_NULL;
    if ((uintptr_t)ys[i] & 15u) return FPQ_E_ALIGN;
    N += ns[i];
    seg.end[i] = (int)N;
    seg.y[i] = (uint16_t*)ys[i];
  }
  seg.count = (int)count;
  return gemm_packed<NV>(xq, xs, wq, ws, alpha, bias, ys[0], M, N, K, stream, nullptr, nullptr, 0, seg);
}
}  // namespace fpq

extern "C" int fpq_gemm_mxf4_packed_multi(const void* xq, const void* xs, const void* wq, const void* ws,
                                          const float* alpha, const void* bias, void* const* ys,
                                          const int64_t* ns, int64_t count, int64_t M, int64_t K, void* stream) {
  return fpq::gemm_packed_multi<false>(xq, xs, wq, ws, alpha, bias, ys, ns, count, M, K, stream);
}

extern "C" int fpq_gemm_nvf4_packed_multi(const void* xq, const void* xs, const void* wq, const void* ws,
                                          const float* alpha, const void* bias, void* const* ys,
                                          const int64_t* ns, int64_t count, int64_t M, int64_t K, void* stream) {
  return fpq::gemm_packed_multi<true>(xq, xs, wq, ws, alpha, bias, ys, ns, count, M, K, stream);
}

extern "C" int fpq_gemm_nvf4_packed(const void* xq, const void* xs, const void* wq, const void* ws,
                                    const float* alpha, const void* bias, void* y, int64_t M,
                                    int64_t N, int64_t K, void* stream) {
  return fpq::gemm_packed<true>(xq, xs, wq, ws, alpha, bias, y, M, N, K, stream);
}

extern "C" int fpq_gemm_nvf4_packed_residual(const void* xq, const void* xs, const void* wq, const void* ws,
                                             const float* alpha, const void* bias, const void* residual, void* y,
                                             int64_t M, int64_t N, int64_t K, void* stream) {
  if (!residual) return FPQ_E_NULL;
  return fpq::gemm_packed<true>(xq, xs, wq, ws, alpha, bias, y, M, N, K, stream, residual);
}
