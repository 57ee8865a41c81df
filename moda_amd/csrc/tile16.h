// MFMA 16x16x32 building blocks.  On gfx950 the matrix pipe is power limited, and on random operands
// the 16x16x32 shape sustains about 16 % more FLOP/s than 32x32x16 at the same operand traffic (it moves
// a quarter of the accumulator bits per multiply-add), so the backward kernels and the 256-wide forward kernel
// are built on it (the narrower forward kernel is bound by its vector work and stays on 32x32x16).
//
// Register layouts, lane l = (n, q) with n = l & 15, q = l >> 4:
//   A (16 x 32):  row n,    k slots 8q .. 8q+7
//   B (32 x 16):  column n, k slots 8q .. 8q+7
//   C (16 x 16):  column n, rows 4q + i, i = 0..3
// The k slots are a summation index: any assignment of real k values to slots is fine as long as A and
// B agree.  The kernels produce scores with the stationary side on N, so that a lane's accumulator
// registers of two vertically adjacent 16-row blocks (rows 4q+i of each) ARE its eight k slots of the
// next product's B operand; the transposed LDS read below delivers the A operand in that same order.
//
// Which tile row sits on row m of a 16-row A block is free as well.  The blocks here carry tile row
// slot_base(m >> 2) + (m & 3) on row m, so that lane group q holds tile rows slot_base(q) .. +3 of a
// block, with slot_base = {0, 8, 12, 4}.  That order keeps both LDS read patterns free of bank conflicts
// under the tile swizzle (measured with SQ_LDS_BANK_CONFLICT; the plain order 0, 4, 8, 12 doubles the
// cost of both):
//  - the transposed 64-bit read is served 32 lanes at a time (lane groups q = 0,1, then 2,3), each group
//    touching four rows of one 32-byte column pair: the two groups of a pass must differ in row bit 3;
//  - the 128-bit row read is served 16 lanes at a time in the order {0-3, 12-15, 20-23, 24-27},
//    {4-7, 8-11, 16-19, 28-31} (+32 for the upper half): the four quads of a pass read two adjacent
//    chunks of four different row groups, which must land on four different chunk residues.
#pragma once
#include "tile.h"

namespace moda {

template <typename T>
__device__ __forceinline__ f32x4 mfma16(i32x4 a, i32x4 b, f32x4 c);
template <>
__device__ __forceinline__ f32x4 mfma16<BF16>(i32x4 a, i32x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0,
                                                 0, 0);
}
template <>
__device__ __forceinline__ f32x4 mfma16<FP16>(i32x4 a, i32x4 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0,
                                                0);
}

// First tile row (within a 16-row block) of the four that lane group q holds in an accumulator block.
__host__ __device__ __forceinline__ constexpr int slot_base(int q) { return (0x4C80 >> (4 * q)) & 15; }

// Two accumulator blocks (rows 4q+i of each) -> the eight k slots of a B operand, rounded to 16 bits.
template <typename T>
__device__ __forceinline__ i32x4 pack_slots(const f32x4& lo, const f32x4& hi) {
  i32x4 r;
  r[0] = pack2<T>(lo[0], lo[1]);
  r[1] = pack2<T>(lo[2], lo[3]);
  r[2] = pack2<T>(hi[0], hi[1]);
  r[3] = pack2<T>(hi[2], hi[3]);
  return r;
}

// Reductions over the four lanes (q = 0..3) that share a column n.
__device__ __forceinline__ float quad_max(float x) {
  x = fmaxf(x, __shfl_xor(x, 16, 64));
  return pair_max(x);
}
__device__ __forceinline__ float quad_sum(float x) {
  x += __shfl_xor(x, 16, 64);
  return pair_sum(x);
}

// Per-lane LDS offsets of the two operand read patterns of a swizzled tile (see Tile<HD>), computed
// once.  Tile rows are only ever offset by multiples of 16, which leaves a row's swizzle unchanged.
//
// Row operand: lane (n, q) gets elements [32*ks + 8q, +8) of tile row row0 + slot_base(n >> 2) + (n & 3):
// MFMA A with M = tile rows and K = head dim.
//
// Transposed operand for head-dim block mb (columns 16*mb .. +15) and the 32 tile rows starting at rb:
// lane (n, q) gets column 16*mb + n of rows rb + slot_base(q) + {0..3} (k slots 0..3) and 16 rows further
// down (k slots 4..7).  Two LDS transpose reads: within a 16-lane group source lane s supplies the address
// of 4 consecutive elements (row slot_base(q) + s/4, columns 16*mb + 4*(s%4) ..), result lane i receives
// element (i & 3) of source lanes 4j + (i >> 2), j = 0..3.
template <int HD>
struct Operand16 {
  static constexpr int KS = HD / 32, MB = HD / 16;
  int row[KS];
  int tr[MB];

  __device__ __forceinline__ void init(int lane) {
    const int n = lane & 15, q = lane >> 4;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) row[ks] = Tile<HD>::off(slot_base(n >> 2) + (n & 3), 4 * ks + q);
#pragma unroll
    for (int mb = 0; mb < MB; mb++) {
      const int r = slot_base(q) + (n >> 2);
      const int dcol = 16 * mb + 4 * (n & 3);
      tr[mb] = Tile<HD>::off(r, dcol >> 3) + (dcol & 7);
    }
  }
  // row0 must be a multiple of 16
  __device__ __forceinline__ i32x4 row_operand(lds_cptr tile, int row0, int ks) const {
    return *reinterpret_cast<MODA_LDS const i32x4*>(tile + row[ks] + row0 * HD);
  }
  // rb must be a multiple of 16
  __device__ __forceinline__ i32x4 tr_operand(lds_cptr tile, int rb, int mb) const {
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((MODA_LDS s16x4*)(tile + tr[mb] + rb * HD));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((MODA_LDS s16x4*)(tile + tr[mb] + (rb + 16) * HD));
    i32x2 l2 = __builtin_bit_cast(i32x2, lo);
    i32x2 h2 = __builtin_bit_cast(i32x2, hi);
    i32x4 r;
    r[0] = l2[0];
    r[1] = l2[1];
    r[2] = h2[0];
    r[3] = h2[1];
    return r;
  }
};

// Software-pipelined MFMA sequences (see the 32x32 versions in tile.h for the why): DEPTH operand reads
// in flight ahead of the matrix pipe, order pinned with scheduling barriers, hook(j) after step j.
// One LDS operand feeds NB MFMAs (one per register operand); consecutive steps use different accumulators.

// acc[mb][nb] = sum_ks rows(tile, 16*mb + n, ks) x breg[nb][ks]     (ACCUMULATE: += instead, acc preset)
template <typename T, int HD, int MBLK, int NB, int DEPTH, bool ACCUMULATE = false, typename Hook = NoHook>
__device__ __forceinline__ void mfma16_rows(const Operand16<HD>& oa, lds_cptr tile, const i32x4 (&breg)[NB][HD / 32],
                                            f32x4 (&acc)[MBLK][NB], Hook&& hook = Hook{}) {
  constexpr int KS = HD / 32, N = MBLK * KS;
  i32x4 ops[N];
#pragma unroll
  for (int j = 0; j < DEPTH && j < N; j++) ops[j] = oa.row_operand(tile, 16 * (j % MBLK), j / MBLK);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int j = 0; j < N; j++) {
    if (j + DEPTH < N) ops[j + DEPTH] = oa.row_operand(tile, 16 * ((j + DEPTH) % MBLK), (j + DEPTH) / MBLK);
    const int mb = j % MBLK, ks = j / MBLK;
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
      f32x4 z = {0.f, 0.f, 0.f, 0.f};
      acc[mb][nb] = mfma16<T>(ops[j], breg[nb][ks], (ks == 0 && !ACCUMULATE) ? z : acc[mb][nb]);
    }
    __builtin_amdgcn_sched_barrier(0);
    hook(j);
  }
}

// Two tiles against two register operand sets in one pipeline:
// acc0[mb][nb] = rows(tile0) x breg0[nb], acc1[mb][nb] = init1[nb] + rows(tile1) x breg1[nb].
// REG_A: the register operands go on the A side instead (the products come out transposed: lane n then holds the
// tile row of its row operand, registers i the rows 4q + i of the register operand's block).
template <typename T, int HD, int MBLK, int NB, int DEPTH, bool REG_A = false, typename Hook = NoHook>
__device__ __forceinline__ void mfma16_rows2(const Operand16<HD>& oa, lds_cptr tile0,
                                             const i32x4 (&breg0)[NB][HD / 32], f32x4 (&acc0)[MBLK][NB],
                                             lds_cptr tile1, const i32x4 (&breg1)[NB][HD / 32],
                                             f32x4 (&acc1)[MBLK][NB], const f32x4 (&init1)[NB], Hook&& hook = Hook{}) {
  constexpr int KS = HD / 32, N = 2 * MBLK * KS;
  i32x4 ops[N];
  // step j: which = j & 1, mb = (j >> 1) % MBLK, ks = (j >> 1) / MBLK
#pragma unroll
  for (int j = 0; j < DEPTH && j < N; j++)
    ops[j] = oa.row_operand((j & 1) ? tile1 : tile0, 16 * ((j >> 1) % MBLK), (j >> 1) / MBLK);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int j = 0; j < N; j++) {
    if (j + DEPTH < N) {
      const int jn = j + DEPTH;
      ops[jn] = oa.row_operand((jn & 1) ? tile1 : tile0, 16 * ((jn >> 1) % MBLK), (jn >> 1) / MBLK);
    }
    const int mb = (j >> 1) % MBLK, ks = (j >> 1) / MBLK;
    const f32x4 z = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
      if (j & 1)
        acc1[mb][nb] = mfma16<T>(REG_A ? breg1[nb][ks] : ops[j], REG_A ? ops[j] : breg1[nb][ks], ks == 0 ? init1[nb] : acc1[mb][nb]);
      else
        acc0[mb][nb] = mfma16<T>(REG_A ? breg0[nb][ks] : ops[j], REG_A ? ops[j] : breg0[nb][ks], ks == 0 ? z : acc0[mb][nb]);
    }
    __builtin_amdgcn_sched_barrier(0);
    hook(j);
  }
}

// acc[mb][nb] += tr(tile, 32*ks, mb) x breg[ks][nb]  for ks < NKS, mb < HD/16.  prefetch() may be called
// early (before the code that produces breg) to have the first operands waiting.
template <typename T, int HD, int NKS, int NB, int DEPTH>
struct TrPipe16 {
  static constexpr int MB = HD / 16, N = NKS * MB;
  i32x4 ops[N];
  __device__ __forceinline__ void prefetch(const Operand16<HD>& oa, lds_cptr tile) {
#pragma unroll
    for (int j = 0; j < DEPTH && j < N; j++) ops[j] = oa.tr_operand(tile, 32 * (j / MB), j % MB);
    __builtin_amdgcn_sched_barrier(0);
  }
  template <typename Hook = NoHook>
  __device__ __forceinline__ void run(const Operand16<HD>& oa, lds_cptr tile, const i32x4 (&breg)[NKS][NB],
                                      f32x4 (&acc)[MB][NB], Hook&& hook = Hook{}) {
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < N; j++) {
      if (j + DEPTH < N) ops[j + DEPTH] = oa.tr_operand(tile, 32 * ((j + DEPTH) / MB), (j + DEPTH) % MB);
#pragma unroll
      for (int nb = 0; nb < NB; nb++) acc[j % MB][nb] = mfma16<T>(ops[j], breg[j / MB][nb], acc[j % MB][nb]);
      __builtin_amdgcn_sched_barrier(0);
      hook(j);
    }
  }
};

}  // namespace moda
