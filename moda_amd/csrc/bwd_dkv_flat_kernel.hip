// Backward, key side, sequence keys of fixed-length launches on the 64-wide tiles: the same products as dkv_kernel
// (moda_v14.py:874-1248, fla/ops/attn/parallel.py:299-440) without the split into two roles.
//
// A workgroup of FOUR waves owns 128 key columns of one (batch, kv head), a wave 32 of them with K AND V in
// registers and BOTH accumulators, dK^T and dV^T; the query rows come by in tiles of 32 (one summation step of the
// 16x16x32 instruction):
//   S = Q K^T, dP - delta = dO V^T (accumulators preset with -delta), P = exp2(S c - lse), dS = P (dP - delta),
//   dV^T += dO^T P, dK^T += Q^T dS.
// P stays in fp32 until dS is formed (one rounding on the dK path) and nothing travels between waves.  With 26 KB of
// LDS and no mailbox, three workgroups share a compute unit where dkv_kernel fits one: a launch of a few hundred
// column tiles of a short sequence (a vision model's 197 tokens) runs in one round of workgroups instead of three,
// and a launch with many column tiles keeps twelve waves per compute unit busy instead of eight.  A launch of few
// tiles over a long sequence is bound by its heaviest tile, where the eight waves of dkv_kernel are faster; on the
// 128-wide tiles this structure spills.  geometry.h: takes_dkv_flat says which launches come here.
#include <type_traits>

#include "geometry.h"
#include "kargs.h"
#include "tile.h"
#include "tile16.h"

namespace moda {

// VARLEN: packed variable-length batch (a workgroup enters its sequence; column tiles past its end leave at once)
template <typename T, int HD, bool VARLEN>
__global__ __launch_bounds__(256, 3) void dkv_flat_kernel(const KArgs a_in) {
  constexpr int NB = 2, BM = 32, MBLK = BM / 16, BN = 4 * 16 * NB, KS = HD / 32, MB = HD / 16, NST = 3, DIST = 2;
  constexpr int SP = 64;  // floats per statistic and stage (one wave-wide load each)
  extern __shared__ __align__(16) unsigned char smem_raw[];
  lds_ptr ring = (lds_ptr)smem_raw;                                      // [NST]: Q tile, dO tile
  MODA_LDS float* stat = (MODA_LDS float*)(ring + NST * 2 * BM * HD);    // [NST][2][SP]: lse, minus delta

  const int tid = threadIdx.x, lane = tid & 63, n = lane & 15, q4 = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int BHk = a_in.B * a_in.Hkv;
  const int bh = blockIdx.x % BHk;
  const int ct = blockIdx.x / BHk;
  int b = bh / a_in.Hkv;
  const int hkv = bh % a_in.Hkv;
  SeqArgs<VARLEN> seq(a_in, b);
  const KArgs& a = seq.a;
  const ColTilePlan plan = col_tile_plan(a_in, a, ct, BN, BM, VARLEN, 1);
  if (VARLEN && !plan.active) return;  // a tile beyond this sequence of a variable-length batch
  int c[NB];
  bool valid[NB];
#pragma unroll
  for (int nb = 0; nb < NB; nb++) {
    c[nb] = plan.c_first + wave * (16 * NB) + 16 * nb + n;
    valid[nb] = c[nb] < a.T;
  }
  i32x4 Kr[NB][KS], Vr[NB][KS];
  {
    const uint16_t* kp = a.k + b * a.sk.b + hkv * a.sk.h + 8 * q4;
    const uint16_t* vp = a.v + b * a.sv.b + hkv * a.sv.h + 8 * q4;
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        i32x4 z = {0, 0, 0, 0};
        Kr[nb][ks] = (valid[nb] && 32 * ks + 8 * q4 < a.D) ? *reinterpret_cast<const i32x4*>(kp + (int64_t)c[nb] * a.sk.t + 32 * ks) : z;
        Vr[nb][ks] = (valid[nb] && 32 * ks + 8 * q4 < a.Dv) ? *reinterpret_cast<const i32x4*>(vp + (int64_t)c[nb] * a.sv.t + 32 * ks) : z;
      }
  }
  // No wait here: K and V travel together with the first query tiles.  The compiler waits for all loads it knows
  // of before the first product, which (loads returning in order) also covers nothing it does not know of.

  int qlo[NB], qhi[NB];
#pragma unroll
  for (int nb = 0; nb < NB; nb++) {
    qlo[nb] = qhi[nb] = 0;
    if (valid[nb]) q_interval(a, false, c[nb], qlo[nb], qhi[nb]);
  }
  const int qt0 = plan.qt0, nqt = plan.nqt;

  typedef AsyncTileLoader<HD, BM, 256> Loader;
  constexpr int LPT = 2 * Loader::N + 1;  // vector-memory loads one wave issues per tile: Q, dO and one statistic
  Loader ld;
  ld.init(tid);
  const uint16_t* qb = a.q + b * a.sq.b + hkv * a.sq.h;
  const uint16_t* dob = a.d_o + b * a.sdo.b + hkv * a.sdo.h;
  // even waves fetch lse ([B, Tq, Hq]: one dword every Hq), odd waves minus delta ([B, Hq, Tq]: contiguous); the two
  // waves of a kind write the same values to the same place, which keeps every wave's load count per tile equal
  const bool st_lse = (wave & 1) == 0;
  const char* stb = st_lse ? (const char*)(a.lse + (int64_t)b * a.Tq * a.Hq + hkv) : (const char*)(a.delta + ((int64_t)b * a.Hq + hkv) * (VARLEN ? a.delta_pitch : a.Tq));
  const uint32_t st_row = st_lse ? (uint32_t)a.Hq * 4u : 4u;
  const int voff_stat = lane * (int)st_row;
  int ld_st = 0;
  auto issue = [&](int it) {  // trip `it` consumes query tile nqt - 1 - it
    const int f_q0 = (qt0 + nqt - 1 - it) * BM;
    lds_ptr Qt = ring + ld_st * 2 * BM * HD;
    ld.load(Qt, qb, a.sq.t, f_q0, a.Tq, a.D);
    ld.load(Qt + BM * HD, dob, a.sdo.t, f_q0, a.Tq, a.Dv);
    const int rows = imax(imin(a.Tq - f_q0, BM), 0);
    const i32x4 rs = rsrc_words(stb + (int64_t)f_q0 * st_row, rows > 0 ? (uint32_t)(rows - 1) * st_row + 4u : 0u);
    lds_dma<4>(rs, (uint32_t)(uintptr_t)(stat + ld_st * 2 * SP + (st_lse ? 0 : SP)), voff_stat, 0);
    ld_st = (ld_st + 1 == NST) ? 0 : ld_st + 1;
  };
  auto wait_tile = [&](int next) {
    if (next + 1 < nqt)
      Loader::template wait_but<LPT>();
    else
      Loader::wait_all();
  };

  f32x4 dk[MB][NB], dv[MB][NB];
#pragma unroll
  for (int d = 0; d < MB; d++)
#pragma unroll
    for (int nb = 0; nb < NB; nb++) dk[d][nb] = dv[d][nb] = f32x4{0.f, 0.f, 0.f, 0.f};
  const float sc = a.scale * kLog2e;
  Operand16<HD> oa;
  oa.init(lane);

#pragma unroll
  for (int j = 0; j < DIST; j++)
    if (j < nqt) issue(j);
  wait_tile(0);
  __syncthreads();

  auto tile = [&](auto masked, int st, int q0) {
    constexpr bool MASKED = decltype(masked)::value;
    lds_cptr Qs = ring + st * 2 * BM * HD;
    lds_cptr dOs = Qs + BM * HD;
    MODA_LDS const float* lse_s = stat + st * 2 * SP;
    MODA_LDS const float* del_s = lse_s + SP;
    f32x4 s[MBLK][NB], dp[MBLK][NB];
#pragma unroll
    for (int m = 0; m < MBLK; m++) {
      const f32x4 dl = *reinterpret_cast<MODA_LDS const f32x4*>(del_s + 16 * m + slot_base(q4));
#pragma unroll
      for (int nb = 0; nb < NB; nb++) dp[m][nb] = dl;
    }
    {  // S and dP in one pipeline, two operand reads ahead of the matrix pipe
      constexpr int N = 2 * MBLK * KS, DEPTH = 2;
      i32x4 ops[N];
      auto rd = [&](int j) { return oa.row_operand((j & 1) ? dOs : Qs, 16 * ((j >> 1) % MBLK), (j >> 1) / MBLK); };
#pragma unroll
      for (int j = 0; j < DEPTH; j++) ops[j] = rd(j);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < N; j++) {
        if (j + DEPTH < N) ops[j + DEPTH] = rd(j + DEPTH);
        const int m = (j >> 1) % MBLK, ks = (j >> 1) / MBLK;
        const f32x4 z = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
          if (j & 1)
            dp[m][nb] = mfma16<T>(ops[j], Vr[nb][ks], dp[m][nb]);
          else
            s[m][nb] = mfma16<T>(ops[j], Kr[nb][ks], ks == 0 ? z : s[m][nb]);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    TrPipe16<T, HD, 1, NB, 3> pv;
    pv.prefetch(oa, dOs);
#pragma unroll
    for (int m = 0; m < MBLK; m++) {
      const f32x4 lv = *reinterpret_cast<MODA_LDS const f32x4*>(lse_s + 16 * m + slot_base(q4));
#pragma unroll
      for (int nb = 0; nb < NB; nb++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
          float p = fast_exp2(__builtin_fmaf(s[m][nb][j], sc, -lv[j]));
          if (MASKED) {
            const int qr = q0 + 16 * m + slot_base(q4) + j;
            p = (qr >= qlo[nb] && qr < qhi[nb]) ? p : 0.f;
          }
          s[m][nb][j] = p;
          dp[m][nb][j] *= p;
        }
    }
    i32x4 P[1][NB], DS[1][NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
      P[0][nb] = pack_slots<T>(s[0][nb], s[1][nb]);
      DS[0][nb] = pack_slots<T>(dp[0][nb], dp[1][nb]);
    }
    pv.run(oa, dOs, P, dv);
    TrPipe16<T, HD, 1, NB, 3> pk;
    pk.prefetch(oa, Qs);
    pk.run(oa, Qs, DS, dk);
  };

  // query tiles whose rows all see all 128 columns need no masking: for causal keys those at or past the last
  // column's first visible row (padding rows past Tq carry zero Q, dO, lse, delta and contribute nothing)
  const int first_free_qt = a.causal ? ((imin(a.T, plan.c_first + BN) - 1) * a.Gf + BM - 1) / BM - qt0 : 0;
  int it = 0, c_st = 0;
  for (; it < nqt && nqt - 1 - it >= first_free_qt; it++) {
    if (it + DIST < nqt) issue(it + DIST);
    tile(std::false_type{}, c_st, (qt0 + nqt - 1 - it) * BM);
    c_st = (c_st + 1 == NST) ? 0 : c_st + 1;
    wait_tile(it + 1);
    __syncthreads();
  }
  for (; it < nqt; it++) {
    if (it + DIST < nqt) issue(it + DIST);
    tile(std::true_type{}, c_st, (qt0 + nqt - 1 - it) * BM);
    c_st = (c_st + 1 == NST) ? 0 : c_st + 1;
    wait_tile(it + 1);
    __syncthreads();
  }

#pragma unroll
  for (int nb = 0; nb < NB; nb++)
    if (valid[nb]) {
      uint16_t* dkp = a.dk + b * a.sdk.b + hkv * a.sdk.h + (int64_t)c[nb] * a.sdk.t + 4 * q4;
      uint16_t* dvp = a.dv + b * a.sdv.b + hkv * a.sdv.h + (int64_t)c[nb] * a.sdv.t + 4 * q4;
#pragma unroll
      for (int d = 0; d < MB; d++) {
        i32x2 w;
        w[0] = pack2<T>(dk[d][nb][0] * a.scale, dk[d][nb][1] * a.scale);
        w[1] = pack2<T>(dk[d][nb][2] * a.scale, dk[d][nb][3] * a.scale);
        if (16 * d + 4 * q4 < a.D) *reinterpret_cast<i32x2*>(dkp + 16 * d) = w;
        w[0] = pack2<T>(dv[d][nb][0], dv[d][nb][1]);
        w[1] = pack2<T>(dv[d][nb][2], dv[d][nb][3]);
        if (16 * d + 4 * q4 < a.Dv) *reinterpret_cast<i32x2*>(dvp + 16 * d) = w;
      }
    }
}

template <typename T, int HD, bool VARLEN>
hipError_t launch_dkv_flat_t(const KArgs& a, hipStream_t stream) {
  constexpr size_t smem = (size_t)3 * 2 * 32 * HD * sizeof(uint16_t) + 3 * 2 * 64 * sizeof(float);
  static LdsAttrState attr;
  const hipError_t ea = allow_dynamic_lds(attr, reinterpret_cast<const void*>(&dkv_flat_kernel<T, HD, VARLEN>), smem);
  if (ea != hipSuccess) return ea;
  const int64_t nblk = dkv_flat_blocks(a);
  if (nblk == 0) return hipSuccess;
  if (nblk >= (1ll << 31)) return hipErrorInvalidValue;
  hipLaunchKernelGGL((dkv_flat_kernel<T, HD, VARLEN>), dim3((unsigned)nblk), dim3(256), smem, stream, a);
  return hipGetLastError();
}

// dtype: 0 bf16, 1 fp16; 64-wide tiles only (the caller asks takes_dkv_flat first)
hipError_t launch_dkv_flat(const KArgs& a, int dtype, hipStream_t stream) {
  if (a.cu) return dtype == 0 ? launch_dkv_flat_t<BF16, 64, true>(a, stream) : launch_dkv_flat_t<FP16, 64, true>(a, stream);
  return dtype == 0 ? launch_dkv_flat_t<BF16, 64, false>(a, stream) : launch_dkv_flat_t<FP16, 64, false>(a, stream);
}

}  // namespace moda
