// Backward, key side: dK/dV of the sequence stream and of the depth stream
// (moda_v14.py:874-1248 and :1251-1454, moda_v16.py:1223-1425 and :1632-1834,
// fda_v12.py:646-860, fla/ops/attn/parallel.py:299-440).
//
// A workgroup (eight waves) owns 128 key columns of one (batch, kv head) --
// sequence keys or flattened depth slots -- as four 32-column blocks; the products
// run on the 16x16x32 matrix instruction (less power per multiply-add than 32x32x16
// on a power-limited matrix pipe), a block being two 16-column halves with lane
// (n, q) on columns 16*nb + n.  It streams 64-row query tiles (Q, dO, LSE, delta) through a
// three-stage LDS ring (one tile in flight while each role consumes one), from
// the last tile down to its
// diagonal (workgroups that run together then read the same tiles at the same
// time and share them in L2), over exactly the query rows that can see its columns:
// all later tokens for a causal sequence key, the owner token's G rows (or the
// rest of its chunk) for a depth slot.  Two waves share each column block and
// split the work by ROLE so that each stays under 256 registers and the two
// instruction streams overlap matrix and vector work on their SIMD:
//   role A: S = Q K^T, P = exp2(S*c - lse), dV^T += dO^T P    (K in registers)
//   role B: dP = dO V^T, dS = P (dP - delta), dK^T += Q^T dS  (V in registers)
// P travels from A to B through a lane-private LDS mailbox in the 16-bit input
// format; B runs one tile behind A, so one barrier per tile orders everything.
// All G folded rows, and in head-dim GQA all G query heads, are reduced in
// registers: every output row has one writer, no atomics, no partial buffers.
#include <type_traits>

#include "geometry.h"
#include "kargs.h"
#include "tile.h"
#include "tile16.h"

namespace moda {

// SPLIT: the launch cuts the query rows of every sequence column tile into a.dkv_split segments (a variant of
// its own: the extra index arithmetic costs the long-sequence instantiation scalar registers it cannot spare)
template <typename T, int HD, bool VARLEN, bool SPLIT = false>
__global__ __launch_bounds__(512) void dkv_kernel(const KArgs a_in) {
  static_assert(!(VARLEN && SPLIT), "packed batches are not split");
  // 16-column halves per wave, query rows per streamed tile: halved for the 256-wide tiles, whose operands and
  // accumulators would not fit the register file (and whose three-stage ring would not fit the LDS) otherwise
  constexpr int NB = HD > 128 ? 1 : 2, BM = HD > 128 ? 32 : 64, MBLK = BM / 16;
  constexpr int BN = 4 * 16 * NB, KS = HD / 32, MB = HD / 16, NST = 3;
  constexpr int NP = (MBLK / 2) * NB;  // B operands of P per lane in the mailbox
  constexpr int SP = 64;               // floats per statistic and stage (one wave-wide load each)
  extern __shared__ __align__(16) unsigned char smem_raw[];
  lds_ptr smem = (lds_ptr)smem_raw;
  // ring of NST stages, each: Q tile, dO tile; then the P mailbox; then lse/delta per stage
  lds_ptr ring = smem;
  MODA_LDS i32x4* mbox = (MODA_LDS i32x4*)(smem + NST * 2 * BM * HD);      // [2 parities][4 blocks][NP][64 lanes]
  MODA_LDS float* stat = (MODA_LDS float*)(mbox + 2 * 4 * NP * 64);        // [NST][2][SP]

  // lane (n, q4) owns columns 16*nb + n (nb < NB) of the wave's block
  const int tid = threadIdx.x, lane = tid & 63, n = lane & 15, q4 = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kblk = wave & 3;
  const bool role_b = wave >= 4;
  const int BHk = a_in.B * a_in.Hkv;
  const int bh = blockIdx.x % BHk;
  const int ct = blockIdx.x / BHk;
  int b = bh / a_in.Hkv;
  const int hkv = bh % a_in.Hkv;
  SeqArgs<VARLEN> seq(a_in, b);
  const KArgs& a = seq.a;
  // sequence tiles come `nseg` workgroups each (row segments of one column tile are neighbours in the grid, the
  // heaviest column tile first), then the depth tiles
  const int nseg = SPLIT ? a.dkv_split : 1;
  const ColTilePlan plan = col_tile_plan(a_in, a, ct, BN, BM, VARLEN, nseg);
  if (VARLEN && !plan.active) return;  // a tile beyond this sequence of a variable-length batch
  const bool dep = plan.dep;
  const int ncols = plan.ncols, seg = plan.seg, c_first = plan.c_first;
  int c[NB];
  bool valid[NB];
#pragma unroll
  for (int nb = 0; nb < NB; nb++) {
    c[nb] = c_first + kblk * (16 * NB) + 16 * nb + n;
    valid[nb] = c[nb] < ncols;
  }
  // the column's row in its tensor: the key's row, or the depth slot's (depth columns are counted on the compact
  // axis of the slots that hold data); computed where it is used, at both ends of the kernel, not kept in between
  auto column_row = [&](int nb) -> int64_t { return dep ? depth_row_of(a, c[nb]) : (int64_t)c[nb]; };

  // stationary operand of this wave's role: K rows (A) or V rows (B)
  i32x4 Sr[NB][KS];
  {
    const uint16_t* src = role_b ? (dep ? a.vd + b * a.svd.b + hkv * a.svd.h : a.v + b * a.sv.b + hkv * a.sv.h)
                                 : (dep ? a.kd + b * a.skd.b + hkv * a.skd.h : a.k + b * a.sk.b + hkv * a.sk.h);
    const int64_t st = role_b ? (dep ? a.svd.t : a.sv.t) : (dep ? a.skd.t : a.sk.t);
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
      const int64_t crow = column_row(nb);
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        i32x4 z = {0, 0, 0, 0};
        Sr[nb][ks] = (valid[nb] && 32 * ks + 8 * q4 < (role_b ? a.Dv : a.D))
                         ? *reinterpret_cast<const i32x4*>(src + crow * st + 32 * ks + 8 * q4)
                         : z;
      }
    }
  }

  // The register operands above must have arrived before the tile loads start: those are issued
  // behind the compiler's back, and a load it still believes pending would cost a vmcnt(0) in every
  // trip of the main loop.
  asm volatile("" ::: "memory");  // keep the loads above this point
  __builtin_amdgcn_s_waitcnt(0x0F70);
  asm volatile("" ::: "memory");

  // visible query-row interval of this lane's columns
  int qlo[NB], qhi[NB];
#pragma unroll
  for (int nb = 0; nb < NB; nb++) {
    qlo[nb] = qhi[nb] = 0;
    if (valid[nb]) q_interval(a, dep, c[nb], qlo[nb], qhi[nb]);
  }
  const int qt0 = plan.qt0, nqt = plan.nqt;
  const int niter = nqt * a.hdiv;

  using Loader = AsyncTileLoader<HD, BM, 512>;
  Loader ld;
  ld.init(tid);
  // Producer.  The global -> LDS loads of one tile are NOT issued back to back: forty wave-wide
  // loads arriving at once queue up in the CU's address unit and every wave would sit on its issue
  // for hundreds of cycles.  prep() fixes the descriptors of the next tile (wave-uniform, scalar
  // registers only); part(k), k < kParts, issues one load; the tile bodies slip the parts between
  // the MFMAs of their first phase, early enough for the tile to land within the trip.
  constexpr int kParts = 2 * Loader::N + 1;
  // The cursor is kept as running byte pointers (row f_q0 of the current query head in Q, dO and this
  // wave's statistic) that step down one tile per call: the scalar unit then has a few adds per trip
  // instead of a dozen dependent 64-bit multiplies.
  const uint32_t q_row_bytes = (uint32_t)a.sq.t * 2u, do_row_bytes = (uint32_t)a.sdo.t * 2u;
  const int voff_q = ld.lane_offset((int)q_row_bytes, a.D);
  const int voff_do = ld.lane_offset((int)do_row_bytes, a.Dv);
  // wave 0 fetches lse ([B, Tq, Hq]: one dword every Hq), wave 1 delta ([B, Hq, Tq]: contiguous)
  const int voff_stat = wave == 0 ? lane * a.Hq * 4 : lane * 4;
  const uint32_t stat_row_bytes = wave == 0 ? (uint32_t)a.Hq * 4u : 4u;
  const char *q_ptr = nullptr, *do_ptr = nullptr, *st_ptr = nullptr;
  int f_q0 = 0, f_left = 0, ld_gh = 0, ld_st = 0;
  auto seek_head = [&]() {  // top tile of query head ld_gh
    const int hq = hkv * a.hdiv + ld_gh;
    f_q0 = (qt0 + nqt - 1) * BM;
    f_left = nqt;
    q_ptr = (const char*)(a.q + b * a.sq.b + hq * a.sq.h + (int64_t)f_q0 * a.sq.t);
    do_ptr = (const char*)(a.d_o + b * a.sdo.b + hq * a.sdo.h + (int64_t)f_q0 * a.sdo.t);
    st_ptr = wave == 0 ? (const char*)(a.lse + ((int64_t)b * a.Tq + f_q0) * a.Hq + hq)
                       : (const char*)(a.delta + ((int64_t)b * a.Hq + hq) * (VARLEN ? a.delta_pitch : a.Tq) + f_q0);
    ld_gh++;
  };
  i32x4 rs_q, rs_do, rs_stat;
  uint32_t lds_q, lds_stat;
  auto prep = [&]() {
    if (f_left == 0) seek_head();
    const uint32_t rows = (uint32_t)query_tile_rows(a, f_q0, BM);  // only a head's top tile can be short
    rs_q = rsrc_words(q_ptr, rows * q_row_bytes);
    rs_do = rsrc_words(do_ptr, rows * do_row_bytes);
    rs_stat = rsrc_words(st_ptr, rows > 0 ? (rows - 1) * stat_row_bytes + 4u : 0u);
    lds_q = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_addr(ring + ld_st * 2 * BM * HD + wave * 512));
    lds_stat = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uintptr_t)(stat + ld_st * 2 * SP + (wave == 0 ? 0 : SP)));
    q_ptr -= (int64_t)BM * q_row_bytes;
    do_ptr -= (int64_t)BM * do_row_bytes;
    st_ptr -= (int64_t)BM * stat_row_bytes;
    f_q0 -= BM;
    f_left--;
    ld_st = (ld_st + 1 == NST) ? 0 : ld_st + 1;
  };
  bool feeding = false;  // this trip has a tile to fetch
  auto part = [&](int k) {
    if (!feeding) return;
    __builtin_amdgcn_sched_barrier(0);
    if (k < Loader::N)
      lds_dma<16>(rs_q, lds_q + k * 8 * 1024, voff_q, k * 8 * Loader::RPW * (int)q_row_bytes);
    else if (k < 2 * Loader::N)
      lds_dma<16>(rs_do, lds_q + BM * HD * 2 + (k - Loader::N) * 8 * 1024, voff_do,
                  (k - Loader::N) * 8 * Loader::RPW * (int)do_row_bytes);
    else if (wave < 2)
      lds_dma<4>(rs_stat, lds_stat, voff_stat, 0);
    __builtin_amdgcn_sched_barrier(0);
  };
  // hook for the first MFMA phase of a tile body: one part after every third MFMA (every second one when
  // the phase is short)
  auto feed = [&](int j) {
    constexpr int every = HD == 64 ? 2 : 3;
    if (j % every == 1 && j / every < kParts) part(j / every);
  };

  f32x4 acc[MB][NB];  // dV^T (role A) or dK^T (role B): head-dim block x column block
#pragma unroll
  for (int d = 0; d < MB; d++)
#pragma unroll
    for (int nb = 0; nb < NB; nb++) acc[d][nb] = f32x4{0.f, 0.f, 0.f, 0.f};
  const float sc = a.scale * kLog2e;
  Operand16<HD> oa;
  oa.init(lane);

  feeding = niter > 0;
  if (feeding) prep();
#pragma unroll
  for (int k = 0; k < kParts; k++) part(k);
  Loader::wait_all();
  __syncthreads();

  // Query tiles whose rows ALL see ALL 128 columns of this workgroup need no masking and no
  // visibility test: for a causal sequence tile those are the tiles at or past the last column's
  // first visible row (padding rows past Tq carry zero Q, dO, lse, delta and contribute nothing);
  // non-causal sequence tiles are all of that kind; depth tiles never are.
  int first_free_qt;  // query tiles (relative to qt0) below this index take the masked body
  if (dep)
    first_free_qt = nqt;
  else if (a.causal)
    first_free_qt = ((min(ncols, c_first + BN) - 1) * a.Gf + BM - 1) / BM - qt0;
  else
    first_free_qt = 0;
  if (SPLIT) first_free_qt = max(first_free_qt, 0);  // an upper row segment starts past the diagonal
  // the last sequence tile may hold padding columns: their K, V are zero, their results unused

  // role A, one tile: S = Q K^T, P = exp2(S c - lse) -> mailbox, dV^T += dO^T P
  auto tile_a = [&](bool masked, lds_cptr Qs, lds_cptr dOs, MODA_LDS const float* lse_s, MODA_LDS i32x4* mb, int q0) {
    f32x4 s[MBLK][NB];
    mfma16_rows<T, HD, MBLK, NB, 4>(oa, Qs, Sr, s, feed);
    TrPipe16<T, HD, MBLK / 2, NB, 2> dvp;
    dvp.prefetch(oa, dOs);
#pragma unroll
    for (int m = 0; m < MBLK; m++) {
      const f32x4 lv = *reinterpret_cast<MODA_LDS const f32x4*>(lse_s + 16 * m + slot_base(q4));
#pragma unroll
      for (int nb = 0; nb < NB; nb++)
#pragma unroll
        for (int j = 0; j < 4; j++) s[m][nb][j] = fast_exp2(__builtin_fmaf(s[m][nb][j], sc, -lv[j]));
    }
    if (masked) {  // wave-uniform; touches only s, so the accumulators stay where they are
#pragma unroll
      for (int m = 0; m < MBLK; m++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
          for (int j = 0; j < 4; j++) {
            const int qr = q0 + 16 * m + slot_base(q4) + j;
            s[m][nb][j] = (qr >= qlo[nb] && qr < qhi[nb]) ? s[m][nb][j] : 0.f;
          }
    }
    i32x4 P[MBLK / 2][NB];
#pragma unroll
    for (int ks = 0; ks < MBLK / 2; ks++)
#pragma unroll
      for (int nb = 0; nb < NB; nb++) {
        P[ks][nb] = pack_slots<T>(s[2 * ks][nb], s[2 * ks + 1][nb]);
        mb[(NB * ks + nb) * 64] = P[ks][nb];
      }
    dvp.run(oa, dOs, P, acc);
  };
  // role B, one tile: dP - delta = dO V^T with the accumulators preset to -delta (the workspace holds
  // minus delta), dS = P (dP - delta), dK^T += Q^T dS
  auto tile_b = [&](lds_cptr Qs, lds_cptr dOs, MODA_LDS const float* del_s, MODA_LDS const i32x4* mb) {
    f32x4 dp[MBLK][NB];
#pragma unroll
    for (int m = 0; m < MBLK; m++) {
      const f32x4 dv = *reinterpret_cast<MODA_LDS const f32x4*>(del_s + 16 * m + slot_base(q4));
#pragma unroll
      for (int nb = 0; nb < NB; nb++) dp[m][nb] = dv;
    }
    mfma16_rows<T, HD, MBLK, NB, 4, true>(oa, dOs, Sr, dp, feed);
    TrPipe16<T, HD, MBLK / 2, NB, 2> dkp;
    dkp.prefetch(oa, Qs);
    i32x4 DS[MBLK / 2][NB];
#pragma unroll
    for (int ks = 0; ks < MBLK / 2; ks++)
#pragma unroll
      for (int nb = 0; nb < NB; nb++) {
        const i32x4 pw = mb[(NB * ks + nb) * 64];
        float p[8];
#pragma unroll
        for (int w = 0; w < 4; w++) unpack2<T>(pw[w], p[2 * w], p[2 * w + 1]);
        DS[ks][nb][0] = pack2<T>(p[0] * dp[2 * ks][nb][0], p[1] * dp[2 * ks][nb][1]);
        DS[ks][nb][1] = pack2<T>(p[2] * dp[2 * ks][nb][2], p[3] * dp[2 * ks][nb][3]);
        DS[ks][nb][2] = pack2<T>(p[4] * dp[2 * ks + 1][nb][0], p[5] * dp[2 * ks + 1][nb][1]);
        DS[ks][nb][3] = pack2<T>(p[6] * dp[2 * ks + 1][nb][2], p[7] * dp[2 * ks + 1][nb][3]);
      }
    dkp.run(oa, Qs, DS, acc);
  };

  // Role A handles tile `it` in trip `it`, role B tile `it - 1` (B idles in the first trip, A in the
  // last).  Each role runs its own copy of the loop nest, and the tiles that need no masking get a
  // loop whose body is unconditional, so the accumulators are updated in place (a tile body behind a
  // branch costs a register-to-register copy of all 64 of them per trip).  Both copies execute
  // niter + 1 barriers.
  auto role_loop = [&](auto is_b) {
    constexpr bool ROLE_B = decltype(is_b)::value;
    int it = 0, c_st = 0, c_par = 0;  // trip, ring stage and mailbox parity of the tile being consumed
    auto begin_trip = [&]() {
      feeding = it + 1 < niter;
      if (feeding) prep();
    };
    auto end_trip = [&]() {
      Loader::wait_all();
      __syncthreads();
      it++;
    };
    auto idle_trip = [&]() {
      begin_trip();
#pragma unroll
      for (int k = 0; k < kParts; k++) part(k);
      end_trip();
    };
    // `stage_tag`: the ring stage as a compile-time constant (the tile's LDS offset then rides in the
    // immediate field of every operand read) or -1 = take it from c_st
    auto body = [&](auto masked_tag, auto stage_tag, int rel_qt) {
      constexpr bool MASKED = decltype(masked_tag)::value;
      constexpr int STAGE = decltype(stage_tag)::value;
      const int q0 = (qt0 + rel_qt) * BM;
      const int st = STAGE >= 0 ? STAGE : c_st;
      lds_cptr Qs = ring + st * 2 * BM * HD;
      lds_cptr dOs = Qs + BM * HD;
      MODA_LDS i32x4* mb = mbox + (c_par * 4 + kblk) * NP * 64 + lane;
      MODA_LDS const float* st_s = stat + st * 2 * SP;
      bool run = true;
      if (MASKED) {
        bool touches = false;
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
          touches = touches || ((qhi[nb] > q0) && (qlo[nb] < q0 + BM) && (qhi[nb] > qlo[nb]));
        run = __any(touches);
        if (!run) {
#pragma unroll
          for (int k = 0; k < kParts; k++) part(k);
        }
      }
      if (run) {
        if constexpr (ROLE_B)
          tile_b(Qs, dOs, st_s + SP, mb);
        else
          tile_a(MASKED, Qs, dOs, st_s, mb, q0);
      }
      c_st = (c_st + 1 == NST) ? 0 : c_st + 1;
      c_par ^= 1;
    };
    using dyn = std::integral_constant<int, -1>;
    if (ROLE_B) idle_trip();
    for (int gh = 0; gh < a.hdiv; gh++) {
      int rel_qt = nqt - 1;
      auto free_trip = [&](auto stage_tag) {
        begin_trip();
        body(std::false_type{}, stage_tag, rel_qt);
        end_trip();
        rel_qt--;
      };
      // unmasked tiles: reach ring stage 0, then three trips per round with the stage known at compile time
      while (rel_qt >= first_free_qt && c_st != 0) free_trip(dyn{});
      while (rel_qt - (NST - 1) >= first_free_qt) {
        free_trip(std::integral_constant<int, 0>{});
        free_trip(std::integral_constant<int, 1>{});
        free_trip(std::integral_constant<int, 2>{});
      }
      while (rel_qt >= first_free_qt) free_trip(dyn{});
      for (; rel_qt >= 0; rel_qt--) {
        begin_trip();
        body(std::true_type{}, dyn{}, rel_qt);
        end_trip();
      }
    }
    if (!ROLE_B) idle_trip();
  };
  if (!role_b)
    role_loop(std::false_type{});
  else
    role_loop(std::true_type{});

  if (SPLIT && !dep) {
    // a row segment: fp32 partial sums, added up by dkv_reduce_kernel
    const int64_t plane = (int64_t)a.B * a.Hkv * a.T * HD;
    const float mul = role_b ? a.scale : 1.f;
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
      if (valid[nb]) {
        float* outp = a.dkv_part + ((int64_t)(role_b ? 0 : 1) * nseg + seg) * plane +
                      (((int64_t)b * a.Hkv + hkv) * a.T + c[nb]) * HD;
#pragma unroll
        for (int d = 0; d < MB; d++) *reinterpret_cast<f32x4*>(outp + 16 * d + 4 * q4) = acc[d][nb] * mul;
      }
    return;
  }
#pragma unroll
  for (int nb = 0; nb < NB; nb++)
    if (valid[nb]) {
      uint16_t* outp;
      float mul;
      const int64_t crow = column_row(nb);
      const int width = role_b ? a.D : a.Dv;  // head dim of the gradient this role writes
      if (!role_b) {  // dV
        outp = dep ? a.dvd + b * a.sdvd.b + hkv * a.sdvd.h + crow * a.sdvd.t
                   : a.dv + b * a.sdv.b + hkv * a.sdv.h + crow * a.sdv.t;
        mul = 1.f;
      } else {  // dK
        outp = dep ? a.dkd + b * a.sdkd.b + hkv * a.sdkd.h + crow * a.sdkd.t
                   : a.dk + b * a.sdk.b + hkv * a.sdk.h + crow * a.sdk.t;
        mul = a.scale;
      }
      if (dep && a.accum_depth) {
        // add to what the row holds (this lane is its only writer).  One 8-byte piece at a time, in order: with the
        // old values of all pieces fetched up front the kernel would not fit its registers
#pragma unroll
        for (int d = 0; d < MB; d++) {
          if (16 * d + 4 * q4 < width) {
            i32x2* dst = reinterpret_cast<i32x2*>(outp + 16 * d + 4 * q4);
            const i32x2 old = *dst;
            float o0, o1, o2, o3;
            unpack2<T>(old[0], o0, o1);
            unpack2<T>(old[1], o2, o3);
            i32x2 w;
            w[0] = pack2<T>(acc[d][nb][0] * mul + o0, acc[d][nb][1] * mul + o1);
            w[1] = pack2<T>(acc[d][nb][2] * mul + o2, acc[d][nb][3] * mul + o3);
            *dst = w;
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
#pragma unroll
        for (int d = 0; d < MB; d++) {
          i32x2 w;
          w[0] = pack2<T>(acc[d][nb][0] * mul, acc[d][nb][1] * mul);
          w[1] = pack2<T>(acc[d][nb][2] * mul, acc[d][nb][3] * mul);
          if (16 * d + 4 * q4 < width) *reinterpret_cast<i32x2*>(outp + 16 * d + 4 * q4) = w;
        }
      }
    }
}

// Depth columns in chunk-visible mode when a chunk's query rows fit one 64-row tile (the reference's only
// shipped geometry: 64 rows per chunk, moda_v16.py:581-585, 1632-1834).  A depth slot is then seen by rows of ONE
// query tile only, so the column-tile kernel above would run a single trip per workgroup and spend its time on
// start-up latency.  Here a workgroup of four waves owns a whole CHUNK: the chunk's Q, dO, lse and delta are
// staged once, then every wave takes 32-column blocks of the chunk's depth slots and does both halves of the
// work itself -- S, P, dV^T with the slots' K rows in registers, then dP, dS, dK^T with their V rows -- with P kept
// in registers in between (no mailbox, no barrier after the staging).  The slots' K/V rows come in and the
// gradient rows go out through a wave-private 32-row tile, so that every global access covers whole rows
// (operand-shaped accesses straight to global memory touch 32 rows per instruction and are bound by the
// request rate).  Two workgroups share a compute unit.
template <typename T, int HD, bool VARLEN>
__global__ __launch_bounds__(256, 2) void chunk_depth_kernel(const KArgs a_in) {
  constexpr int BM = 64, KK = HD / 16, DB = HD / 32;
  constexpr int CH = HD / 8, RPW = 64 / CH, NPASS = 32 / RPW;  // 16-byte chunks per row, rows per wave-wide access
  extern __shared__ __align__(16) unsigned char smem_raw[];
  lds_ptr Qs = (lds_ptr)smem_raw;
  lds_ptr dOs = Qs + BM * HD;
  const int tid = threadIdx.x, lane = tid & 63, n = lane & 31, g = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  lds_ptr wt = dOs + BM * HD + wave * (32 * HD);                           // this wave's private tile
  MODA_LDS float* stat = (MODA_LDS float*)(dOs + BM * HD + 4 * 32 * HD);    // lse[BM], then minus delta[BM]

  const int BHk = a_in.B * a_in.Hkv;
  const int bh = blockIdx.x % BHk;
  const int chunk = blockIdx.x / BHk;
  int b = bh / a_in.Hkv;
  const int hkv = bh % a_in.Hkv;
  SeqArgs<VARLEN> seq(a_in, b);
  const KArgs& a = seq.a;
  const int t0 = chunk * a.Cb;
  if (t0 >= a.T) return;  // a chunk beyond this sequence of a variable-length batch
  const int t1 = min(a.T, t0 + a.Cb);
  const int r0 = t0 * a.Gf, r_end = t1 * a.Gf;  // the chunk's query rows (at most BM)

  using Loader = AsyncTileLoader<HD, BM, 256>;
  Loader ld;
  ld.init(tid);
  ld.load(Qs, a.q + b * a.sq.b + hkv * a.sq.h, a.sq.t, r0, r_end, a.D);
  ld.load(dOs, a.d_o + b * a.sdo.b + hkv * a.sdo.h, a.sdo.t, r0, r_end, a.Dv);
  if (tid < BM) {
    const int r = r0 + tid;
    const bool in = r < r_end;
    stat[tid] = in ? a.lse[((int64_t)b * a.Tq + r) * a.Hq + hkv] : 0.f;
    stat[BM + tid] = in ? a.delta[((int64_t)b * a.Hq + hkv) * (VARLEN ? a.delta_pitch : a.Tq) + r] : 0.f;
  }
  Loader::wait_all();
  __syncthreads();

  const float sc = a.scale * kLog2e;
  OperandAddr<HD> oa;
  oa.init(lane);
  const int c_end = t1 * a.Lv;  // depth columns on the compact axis of the slots that hold data
  const uint16_t* kdp = a.kd + b * a.skd.b + hkv * a.skd.h;
  const uint16_t* vdp = a.vd + b * a.svd.b + hkv * a.svd.h;
  const int prow = lane / CH, pch = lane % CH;  // this lane's row within a pass over the private tile, its physical chunk
  WaveTileLoader<HD> own;
  own.init(lane);
  // columns [cb, cb + 32) of a depth tensor of head dim d -> the private tile (rows past the chunk's last column
  // arrive as zeros)
  const bool partial = a.Lv != a.L;
  auto fetch = [&](const uint16_t* base, int64_t stride, int cb, int d) {
    if (partial)
      own.fetch_mapped(wt, base, stride, cb, min(32, c_end - cb), (int64_t)a.T * a.L, a.L, a.Lv, d);
    else
      own.fetch(wt, base, stride, cb, min(32, c_end - cb), d);
  };
  auto landed = [&]() {
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
    asm volatile("" ::: "memory");
  };
  auto reads_done = [&]() {  // every LDS read of this wave has returned: the tile may be overwritten
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    asm volatile("" ::: "memory");
  };
  // 32 gradient rows from the accumulators (one column per lane) through the private tile to global memory
  auto store = [&](const f32x16 (&acc)[DB], uint16_t* base, int64_t stride, int cb, float mul, int width) {
    reads_done();
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        i32x2 w;
        w[0] = pack2<T>(acc[d][4 * i4 + 0] * mul, acc[d][4 * i4 + 1] * mul);
        w[1] = pack2<T>(acc[d][4 * i4 + 2] * mul, acc[d][4 * i4 + 3] * mul);
        *reinterpret_cast<MODA_LDS i32x2*>(wt + Tile<HD>::off(n, 4 * d + i4) + 4 * g) = w;
      }
#pragma unroll
    for (int i = 0; i < NPASS; i++) {
      const int row = i * RPW + prow;
      i32x4 val = *reinterpret_cast<MODA_LDS const i32x4*>(wt + i * 512 + lane * 8);
      const int lch = pch ^ Tile<HD>::swz(row);
      if (cb + row < c_end && lch * 8 < width) {
        i32x4* dst = reinterpret_cast<i32x4*>(base + depth_row_of(a, cb + row) * stride + lch * 8);
        if (a.accum_depth) {  // add to what the row holds (this lane is the only writer of its 16 bytes)
          const i32x4 old = *dst;
#pragma unroll
          for (int w = 0; w < 4; w++) {
            float x0, x1, y0, y1;
            unpack2<T>(val[w], x0, x1);
            unpack2<T>(old[w], y0, y1);
            val[w] = pack2<T>(x0 + y0, x1 + y1);
          }
        }
        __builtin_nontemporal_store(val, dst);  // next read by another launch
      }
    }
  };

  for (int cb = t0 * a.Lv + wave * 32; cb < c_end; cb += 128) {
    const int c = cb + n;
    // the column's visible rows: from its owner token's first row to the end of the chunk
    const int qlo = c < c_end ? (c / a.Lv) * a.Gf : r_end;
    reads_done();
    fetch(kdp, a.skd.t, cb, a.D);
    landed();
    i32x4 Sr[KK];
#pragma unroll
    for (int kk = 0; kk < KK; kk++) Sr[kk] = oa.row_operand(wt, 0, kk);
    reads_done();
    fetch(vdp, a.svd.t, cb, a.Dv);  // the V rows travel while the probabilities are computed
    // S = Q K^T, P = exp2(S c - lse) on the visible rows
    f32x16 s[2];
    mfma_rows<T, HD, 2, 4>(oa, Qs, Sr, s);
#pragma unroll
    for (int bb = 0; bb < 2; bb++)
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        const f32x4 lv = *reinterpret_cast<MODA_LDS const f32x4*>(stat + 32 * bb + 8 * i4 + 4 * g);
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const int qr = r0 + 32 * bb + 8 * i4 + 4 * g + j;
          const float p = fast_exp2(__builtin_fmaf(s[bb][4 * i4 + j], sc, -lv[j]));
          s[bb][4 * i4 + j] = (qr >= qlo && qr < r_end) ? p : 0.f;
        }
      }
    i32x4 P[4];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) P[ks] = pack8<T>(s[ks >> 1], (ks & 1) * 8);
    landed();
    i32x4 Vr[KK];
#pragma unroll
    for (int kk = 0; kk < KK; kk++) Vr[kk] = oa.row_operand(wt, 0, kk);
    {  // dV^T = dO^T P
      f32x16 acc[DB];
#pragma unroll
      for (int d = 0; d < DB; d++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[d][i] = 0.f;
      TrPipe<T, HD, 4, 2> dvp;
      dvp.prefetch(oa, dOs);
      dvp.run(oa, dOs, P, acc);
      store(acc, a.dvd + b * a.sdvd.b + hkv * a.sdvd.h, a.sdvd.t, cb, 1.f, a.Dv);
    }
    {  // dP - delta = dO V^T (accumulators start from minus delta), dS = P (dP - delta), dK^T = Q^T dS
      f32x16 dp[2];
#pragma unroll
      for (int bb = 0; bb < 2; bb++)
#pragma unroll
        for (int i4 = 0; i4 < 4; i4++) {
          const f32x4 dl = *reinterpret_cast<MODA_LDS const f32x4*>(stat + BM + 32 * bb + 8 * i4 + 4 * g);
#pragma unroll
          for (int j = 0; j < 4; j++) dp[bb][4 * i4 + j] = dl[j];
        }
      mfma_rows_acc<T, HD, 2, 4>(oa, dOs, Vr, dp);
      i32x4 DS[4];
#pragma unroll
      for (int ks = 0; ks < 4; ks++) {
        const int bb = ks >> 1;
        float p[8];
#pragma unroll
        for (int w = 0; w < 4; w++) unpack2<T>(P[ks][w], p[2 * w], p[2 * w + 1]);
#pragma unroll
        for (int w = 0; w < 4; w++)
          DS[ks][w] = pack2<T>(p[2 * w] * dp[bb][8 * (ks & 1) + 2 * w], p[2 * w + 1] * dp[bb][8 * (ks & 1) + 2 * w + 1]);
      }
      f32x16 acc[DB];
#pragma unroll
      for (int d = 0; d < DB; d++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[d][i] = 0.f;
      TrPipe<T, HD, 4, 2> dkp;
      dkp.prefetch(oa, Qs);
      dkp.run(oa, Qs, DS, acc);
      store(acc, a.dkd + b * a.sdkd.b + hkv * a.sdkd.h, a.sdkd.t, cb, a.scale, a.D);
    }
  }
}

// Depth columns outside chunk-visible mode (moda_v14.py:1251-1454, fda_v12.py:646-860): a depth slot is seen
// by the G query rows of its own token only, so its gradients are 2*G dot products and 2*G scaled row
// additions of length D -- far too little to fill a 64 x 128 MFMA tile, and on short sequences the
// matrix kernel's per-workgroup latency dominated it.  Here HD/8 lanes share a column (16 bytes of the
// head dim each), a wave covers 8 (D = 64) or 4 (D = 128) consecutive columns, everything stays in
// registers and the kernel streams kd, vd in and dkd, dvd out once: it is bound by HBM.
// P and dS are rounded to the input type before they are used, as in the matrix kernels.
// Sum over the LPC (8, 16 or 32) consecutive lanes that share a column, result in every one of them.  The first
// four steps are data-parallel-primitive moves inside the vector ALU (two quad permutes leave every lane of a quad
// with the quad's sum, mirroring half a row, then the row, brings in the other quads' sums); only the step across
// two rows of 16 lanes goes through the LDS crossbar.
template <int LPC>
__device__ __forceinline__ float group_sum(float x) {
  static_assert(LPC == 8 || LPC == 16 || LPC == 32, "8, 16 or 32 lanes per column");
#if defined(__HIP_DEVICE_COMPILE__)
  auto dpp = [](float v, auto ctrl) {
    const int i = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(i, i, decltype(ctrl)::value, 0xf, 0xf, false));
  };
  x += dpp(x, std::integral_constant<int, 0xB1>{});   // quad_perm [1,0,3,2]
  x += dpp(x, std::integral_constant<int, 0x4E>{});   // quad_perm [2,3,0,1]
  x += dpp(x, std::integral_constant<int, 0x141>{});  // row_half_mirror
  if (LPC >= 16) x += dpp(x, std::integral_constant<int, 0x140>{});  // row_mirror
  if (LPC == 32) x += __shfl_xor(x, 16, 64);
#endif
  return x;
}

template <typename T, int HD>
__global__ __launch_bounds__(256) void depth_cols_kernel(const KArgs a_in) {
  constexpr int LPC = HD / 8, CPW = 64 / LPC, CPB = 4 * CPW;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int sub = lane % LPC;
  KArgs a = a_in;
  const int BHk = a.B * a.Hkv;
  const int bh = blockIdx.x % BHk;
  int b = bh / a.Hkv;
  const int hkv = bh % a.Hkv;
  enter_sequence(a, b);
  const int64_t c = (int64_t)(blockIdx.x / BHk) * CPB + wave * CPW + lane / LPC;
  if (c >= (int64_t)a.T * a.L) return;  // whole lane groups leave together
  const int w = (int)(c / a.L), slot = (int)(c - (int64_t)w * a.L);
  uint16_t* dk_out = a.dkd + b * a.sdkd.b + hkv * a.sdkd.h + c * a.sdkd.t + 8 * sub;
  uint16_t* dv_out = a.dvd + b * a.sdvd.b + hkv * a.sdvd.h + c * a.sdvd.t + 8 * sub;
  // lanes past a tensor's head dim carry zeros and store nothing (keys and values may differ in width)
  const bool in_k = 8 * sub < a.D, in_v = 8 * sub < a.Dv;
  if (slot >= a.Lv) {  // a slot without data: zero gradient, or (accumulating) somebody else's sum to leave alone
    if (a.accum_depth) return;
    const i32x4 z = {0, 0, 0, 0};
    if (in_k) *reinterpret_cast<i32x4*>(dk_out) = z;
    if (in_v) *reinterpret_cast<i32x4*>(dv_out) = z;
    return;
  }
  auto load8 = [&](const uint16_t* p, float (&f)[8], bool in_dim) {
    const i32x4 zero = {0, 0, 0, 0};
    const i32x4 v = in_dim ? *reinterpret_cast<const i32x4*>(p) : zero;
#pragma unroll
    for (int i = 0; i < 4; i++) unpack2<T>(v[i], f[2 * i], f[2 * i + 1]);
  };
  float kf[8], vf[8], dk[8], dv[8];
  load8(a.kd + b * a.skd.b + hkv * a.skd.h + c * a.skd.t + 8 * sub, kf, in_k);
  load8(a.vd + b * a.svd.b + hkv * a.svd.h + c * a.svd.t + 8 * sub, vf, in_v);
#pragma unroll
  for (int i = 0; i < 8; i++) dk[i] = dv[i] = 0.f;
  const float sc = a.scale * kLog2e;
  const uint16_t* qb = a.q + b * a.sq.b + hkv * a.sq.h + 8 * sub;
  const uint16_t* dob = a.d_o + b * a.sdo.b + hkv * a.sdo.h + 8 * sub;
  for (int gq = 0; gq < a.Gf; gq++) {
    const int64_t r = (int64_t)w * a.Gf + gq;
    float qf[8], dof[8];
    load8(qb + r * a.sq.t, qf, in_k);
    load8(dob + r * a.sdo.t, dof, in_v);
    float s = 0.f, dp = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      s = __builtin_fmaf(qf[i], kf[i], s);
      dp = __builtin_fmaf(dof[i], vf[i], dp);
    }
    s = group_sum<LPC>(s);
    dp = group_sum<LPC>(dp);
    const float lse = a.lse[((int64_t)b * a.Tq + r) * a.Hq + hkv];
    const float neg_delta = a.delta[((int64_t)b * a.Hq + hkv) * a.delta_pitch + r];
    float p = fast_exp2(__builtin_fmaf(s, sc, -lse));
    float ds = p * (dp + neg_delta);
    unpack2<T>(pack2<T>(p, ds), p, ds);  // the rounding the matrix kernels apply before the second product
#pragma unroll
    for (int i = 0; i < 8; i++) {
      dv[i] = __builtin_fmaf(p, dof[i], dv[i]);
      dk[i] = __builtin_fmaf(ds, qf[i], dk[i]);
    }
  }
#pragma unroll
  for (int i = 0; i < 8; i++) dk[i] *= a.scale;
  if (a.accum_depth) {  // add to what the row holds (this thread is its only writer), one rounding per call
    float ok_old[8], ov_old[8];
    load8(dk_out, ok_old, in_k);
    load8(dv_out, ov_old, in_v);
#pragma unroll
    for (int i = 0; i < 8; i++) {
      dk[i] += ok_old[i];
      dv[i] += ov_old[i];
    }
  }
  i32x4 ok, ov;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    ok[i] = pack2<T>(dk[2 * i], dk[2 * i + 1]);
    ov[i] = pack2<T>(dv[2 * i], dv[2 * i + 1]);
  }
  if (in_k) *reinterpret_cast<i32x4*>(dk_out) = ok;
  if (in_v) *reinterpret_cast<i32x4*>(dv_out) = ov;
}

// The same columns when the dQ kernel has left its rounded P and dS of every (query row, slot) pair in the workspace
// (KArgs::depth_p, depth_ds): no kd, vd, no scores -- per column G scalar pairs and the G rows of q and do, which the
// L columns of a token share through the caches.  The launch moves the gradient rows out and little else.
template <typename T, int HD>
__global__ __launch_bounds__(256) void depth_cols_handed_kernel(const KArgs a_in) {
  constexpr int LPC = HD / 8, CPW = 64 / LPC, CPB = 4 * CPW;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int sub = lane % LPC;
  KArgs a = a_in;
  const int BHk = a.B * a.Hkv;
  const int bh = blockIdx.x % BHk;
  int b = bh / a.Hkv;
  const int hkv = bh % a.Hkv;
  enter_sequence(a, b);
  const int64_t c = (int64_t)(blockIdx.x / BHk) * CPB + wave * CPW + lane / LPC;
  if (c >= (int64_t)a.T * a.L) return;  // whole lane groups leave together
  const int w = (int)(c / a.L), slot = (int)(c - (int64_t)w * a.L);
  uint16_t* dk_out = a.dkd + b * a.sdkd.b + hkv * a.sdkd.h + c * a.sdkd.t + 8 * sub;
  uint16_t* dv_out = a.dvd + b * a.sdvd.b + hkv * a.sdvd.h + c * a.sdvd.t + 8 * sub;
  const bool in_k = 8 * sub < a.D, in_v = 8 * sub < a.Dv;
  if (slot >= a.Lv) {  // a slot without data: zero gradient, or (accumulating) somebody else's sum to leave alone
    if (a.accum_depth) return;
    const i32x4 z = {0, 0, 0, 0};
    if (in_k) *reinterpret_cast<i32x4*>(dk_out) = z;
    if (in_v) *reinterpret_cast<i32x4*>(dv_out) = z;
    return;
  }
  auto load8 = [&](const uint16_t* p, float (&f)[8], bool in_dim) {
    const i32x4 zero = {0, 0, 0, 0};
    const i32x4 v = in_dim ? *reinterpret_cast<const i32x4*>(p) : zero;
#pragma unroll
    for (int i = 0; i < 4; i++) unpack2<T>(v[i], f[2 * i], f[2 * i + 1]);
  };
  float dk[8], dv[8];
#pragma unroll
  for (int i = 0; i < 8; i++) dk[i] = dv[i] = 0.f;
  const uint16_t* qb = a.q + b * a.sq.b + hkv * a.sq.h + 8 * sub;
  const uint16_t* dob = a.d_o + b * a.sdo.b + hkv * a.sdo.h + 8 * sub;
  const int64_t head = ((int64_t)b * a.Hq + hkv) * a.delta_pitch;
  for (int gq = 0; gq < a.Gf; gq++) {
    const int64_t r = (int64_t)w * a.Gf + gq;
    float qf[8], dof[8];
    load8(qb + r * a.sq.t, qf, in_k);
    load8(dob + r * a.sdo.t, dof, in_v);
    float p, ds, unused;
    const int64_t at = (head + (int64_t)w * a.Gf) * a.Lv + (int64_t)slot * a.Gf + gq;
    unpack2<T>((int)a.depth_p[at], p, unused);
    unpack2<T>((int)a.depth_ds[at], ds, unused);
#pragma unroll
    for (int i = 0; i < 8; i++) {
      dv[i] = __builtin_fmaf(p, dof[i], dv[i]);
      dk[i] = __builtin_fmaf(ds, qf[i], dk[i]);
    }
  }
#pragma unroll
  for (int i = 0; i < 8; i++) dk[i] *= a.scale;
  if (a.accum_depth) {  // add to what the row holds (this thread is its only writer), one rounding per call
    float ok_old[8], ov_old[8];
    load8(dk_out, ok_old, in_k);
    load8(dv_out, ov_old, in_v);
#pragma unroll
    for (int i = 0; i < 8; i++) {
      dk[i] += ok_old[i];
      dv[i] += ov_old[i];
    }
  }
  i32x4 ok, ov;
#pragma unroll
  for (int i = 0; i < 4; i++) {
    ok[i] = pack2<T>(dk[2 * i], dk[2 * i + 1]);
    ov[i] = pack2<T>(dv[2 * i], dv[2 * i + 1]);
  }
  if (in_k) *reinterpret_cast<i32x4*>(dk_out) = ok;
  if (in_v) *reinterpret_cast<i32x4*>(dv_out) = ov;
}

// The same for query groups of up to four rows, organised by token: the lanes that share a token (16 bytes of the head
// dim each) keep the token's rows of q and do in registers and walk its slots, so that q and do are read once per
// token instead of once per slot and the launch is little more than the stream of gradient rows going out.
template <typename T, int HD>
__global__ __launch_bounds__(256) void depth_token_handed_kernel(const KArgs a_in) {
  constexpr int LPT = HD / 8, TPW = 64 / LPT, TPB = 4 * TPW, GMAX = 4;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int sub = lane % LPT;
  KArgs a = a_in;
  const int BHk = a.B * a.Hkv;
  const int bh = blockIdx.x % BHk;
  int b = bh / a.Hkv;
  const int hkv = bh % a.Hkv;
  enter_sequence(a, b);
  const int w = (blockIdx.x / BHk) * TPB + wave * TPW + lane / LPT;
  if (w >= a.T) return;  // whole lane groups leave together
  const bool in_k = 8 * sub < a.D, in_v = 8 * sub < a.Dv;
  auto load8 = [&](const uint16_t* p, float (&f)[8], bool in_dim) {
    const i32x4 zero = {0, 0, 0, 0};
    const i32x4 v = in_dim ? *reinterpret_cast<const i32x4*>(p) : zero;
#pragma unroll
    for (int i = 0; i < 4; i++) unpack2<T>(v[i], f[2 * i], f[2 * i + 1]);
  };
  float qf[GMAX][8], dof[GMAX][8];
  const uint16_t* qb = a.q + b * a.sq.b + hkv * a.sq.h + 8 * sub;
  const uint16_t* dob = a.d_o + b * a.sdo.b + hkv * a.sdo.h + 8 * sub;
#pragma unroll
  for (int g = 0; g < GMAX; g++) {
    const int64_t r = (int64_t)w * a.Gf + g;
    load8(qb + r * a.sq.t, qf[g], in_k && g < a.Gf);
    load8(dob + r * a.sdo.t, dof[g], in_v && g < a.Gf);
  }
  const int64_t block = (((int64_t)b * a.Hq + hkv) * a.delta_pitch + (int64_t)w * a.Gf) * a.Lv;
  uint16_t* dk_out = a.dkd + b * a.sdkd.b + hkv * a.sdkd.h + (int64_t)w * a.L * a.sdkd.t + 8 * sub;
  uint16_t* dv_out = a.dvd + b * a.sdvd.b + hkv * a.sdvd.h + (int64_t)w * a.L * a.sdvd.t + 8 * sub;
  for (int slot = 0; slot < a.L; slot++, dk_out += a.sdkd.t, dv_out += a.sdvd.t) {
    float dk[8], dv[8];
#pragma unroll
    for (int i = 0; i < 8; i++) dk[i] = dv[i] = 0.f;
    if (slot >= a.Lv) {  // a slot without data: zero gradient, or (accumulating) somebody else's sum to leave alone
      if (a.accum_depth) continue;
    } else {
#pragma unroll
      for (int g = 0; g < GMAX; g++) {
        float p = 0.f, ds = 0.f, unused;
        if (g < a.Gf) {
          unpack2<T>((int)a.depth_p[block + (int64_t)slot * a.Gf + g], p, unused);
          unpack2<T>((int)a.depth_ds[block + (int64_t)slot * a.Gf + g], ds, unused);
        }
#pragma unroll
        for (int i = 0; i < 8; i++) {
          dv[i] = __builtin_fmaf(p, dof[g][i], dv[i]);
          dk[i] = __builtin_fmaf(ds, qf[g][i], dk[i]);
        }
      }
#pragma unroll
      for (int i = 0; i < 8; i++) dk[i] *= a.scale;
      if (a.accum_depth) {  // add to what the row holds (this thread is its only writer), one rounding per call
        float ok_old[8], ov_old[8];
        load8(dk_out, ok_old, in_k);
        load8(dv_out, ov_old, in_v);
#pragma unroll
        for (int i = 0; i < 8; i++) {
          dk[i] += ok_old[i];
          dv[i] += ov_old[i];
        }
      }
    }
    i32x4 ok, ov;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      ok[i] = pack2<T>(dk[2 * i], dk[2 * i + 1]);
      ov[i] = pack2<T>(dv[2 * i], dv[2 * i + 1]);
    }
    // written once here and next read by another launch: past the caches
    if (in_k) __builtin_nontemporal_store(ok, reinterpret_cast<i32x4*>(dk_out));
    if (in_v) __builtin_nontemporal_store(ov, reinterpret_cast<i32x4*>(dv_out));
  }
}

// A partially filled depth stream, not accumulating: the chunk-visible kernels above, and the dQ kernel where it
// forms the depth gradients itself, only visit the slots that hold data, so the gradient rows of the other slots
// are written here (zeros).  One thread per 16 bytes of a
// depth row; `rows`: depth rows per batch entry of the tensors (the whole packed axis for a packed batch).
template <int HD>
__global__ __launch_bounds__(256) void zero_unfilled_slots_kernel(const KArgs a, int64_t rows, int batches) {
  constexpr int TPR = HD / 8;
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int sub = (int)(gid % TPR);
  int64_t rest = gid / TPR;
  const int h = (int)(rest % a.Hkv);
  rest /= a.Hkv;
  const int64_t row = rest % rows;
  const int64_t b = rest / rows;
  if (b >= batches || (int)(row % a.L) < a.Lv) return;
  const i32x4 z = {0, 0, 0, 0};
  if (8 * sub < a.D) *reinterpret_cast<i32x4*>(a.dkd + b * a.sdkd.b + h * a.sdkd.h + row * a.sdkd.t + 8 * sub) = z;
  if (8 * sub < a.Dv) *reinterpret_cast<i32x4*>(a.dvd + b * a.sdvd.b + h * a.sdvd.h + row * a.sdvd.t + 8 * sub) = z;
}

// Adds the fp32 partial sums of the row segments (in segment order: the result does not depend on which
// workgroup finished first) and writes dk, dv in the tensor type.  One thread per 8 head-dim elements.
template <typename T, int HD>
__global__ __launch_bounds__(256) void dkv_reduce_kernel(const KArgs a) {
  constexpr int TPR = HD / 8;
  const int64_t rows = (int64_t)a.B * a.Hkv * a.T;
  const int64_t gid = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t row = gid / TPR;
  if (row >= rows) return;
  const int sub = (int)(gid % TPR);
  const int c = (int)(row % a.T);
  const int bh = (int)(row / a.T);
  const int b = bh / a.Hkv, hkv = bh % a.Hkv;
  const int64_t plane = rows * HD;
#pragma unroll
  for (int which = 0; which < 2; which++) {  // 0: dk, 1: dv
    const float* src = a.dkv_part + (int64_t)which * a.dkv_split * plane + row * HD + 8 * sub;
    float s[8];
#pragma unroll
    for (int i = 0; i < 8; i++) s[i] = 0.f;
    for (int sg = 0; sg < a.dkv_split; sg++) {
      const f32x4 lo = *reinterpret_cast<const f32x4*>(src + sg * plane);
      const f32x4 hi = *reinterpret_cast<const f32x4*>(src + sg * plane + 4);
#pragma unroll
      for (int i = 0; i < 4; i++) {
        s[i] += lo[i];
        s[4 + i] += hi[i];
      }
    }
    i32x4 w;
#pragma unroll
    for (int i = 0; i < 4; i++) w[i] = pack2<T>(s[2 * i], s[2 * i + 1]);
    uint16_t* outp = which == 0 ? a.dk + b * a.sdk.b + hkv * a.sdk.h + (int64_t)c * a.sdk.t
                                : a.dv + b * a.sdv.b + hkv * a.sdv.h + (int64_t)c * a.sdv.t;
    if (8 * sub < (which == 0 ? a.D : a.Dv)) *reinterpret_cast<i32x4*>(outp + 8 * sub) = w;
  }
}

hipError_t launch_dkv_flat(const KArgs& a, int dtype, hipStream_t stream);  // bwd_dkv_flat_kernel.hip

template <typename T, int HD>
hipError_t launch_dkv_t(const KArgs& a, hipStream_t stream) {
  constexpr int NB = HD > 128 ? 1 : 2, BM = HD > 128 ? 32 : 64, BN = 64 * NB;  // as in dkv_kernel
  constexpr size_t smem = 3 * 2 * BM * HD * sizeof(uint16_t) + 2 * 4 * (BM / 32) * NB * 64 * 16 + 3 * 2 * 64 * sizeof(float);
  static LdsAttrState attr;
  static LdsAttrState attr_packed;
  static LdsAttrState attr_split;
  const int nseg = a.cu ? 1 : a.dkv_split;
  const hipError_t ea =
      a.cu       ? allow_dynamic_lds(attr_packed, reinterpret_cast<const void*>(&dkv_kernel<T, HD, true>), smem)
      : nseg > 1 ? allow_dynamic_lds(attr_split, reinterpret_cast<const void*>(&dkv_kernel<T, HD, false, true>), smem)
                 : allow_dynamic_lds(attr, reinterpret_cast<const void*>(&dkv_kernel<T, HD, false>), smem);
  if (ea != hipSuccess) return ea;
  // depth columns: vector kernel, except in chunk-visible mode where a column has up to G*Cb visible rows
  const bool in_dq = depth_grads_in_dq(a, HD);  // the dQ launch has formed the depth slots' dK and dV already
  const bool depth_by_columns = a.L > 0 && !a.chunk && !in_dq;
  const int64_t n_seq_tiles = a.has_seq ? (a.T + BN - 1) / BN : 0;
  const bool depth_by_chunks = moda::depth_by_chunks(a, HD);
  const int64_t nblk = col_kernel_blocks(a, HD, BN, nseg);
  if (nblk >= (1ll << 31)) return hipErrorInvalidValue;
  if (nblk > 0 && takes_dkv_flat(a, HD, nseg)) {
    const hipError_t e = launch_dkv_flat(a, std::is_same<T, FP16>::value ? 1 : 0, stream);
    if (e != hipSuccess) return e;
  } else if (nblk > 0) {
    if (a.cu)
      hipLaunchKernelGGL((dkv_kernel<T, HD, true>), dim3((unsigned)nblk), dim3(512), smem, stream, a);
    else if (nseg > 1)
      hipLaunchKernelGGL((dkv_kernel<T, HD, false, true>), dim3((unsigned)nblk), dim3(512), smem, stream, a);
    else
      hipLaunchKernelGGL((dkv_kernel<T, HD, false>), dim3((unsigned)nblk), dim3(512), smem, stream, a);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (nseg > 1 && n_seq_tiles > 0) {
      const int64_t nthreads = (int64_t)a.B * a.Hkv * a.T * (HD / 8);
      hipLaunchKernelGGL((dkv_reduce_kernel<T, HD>), dim3((unsigned)((nthreads + 255) / 256)), dim3(256), 0, stream, a);
      const hipError_t er = hipGetLastError();
      if (er != hipSuccess) return er;
    }
  }
  if (a.L > 0 && (a.chunk || in_dq) && a.Lv != a.L && !a.accum_depth && (int64_t)a.B * a.T > 0) {
    // packed batch: one row axis of all sequences (its length is the row-sum pitch / G), else B x T * L rows
    const int64_t rows = a.cu ? (int64_t)(a.delta_pitch / a.Gf) * a.L : (int64_t)a.T * a.L;
    const int batches = a.cu ? 1 : a.B;
    const int64_t nthreads = rows * batches * a.Hkv * (HD / 8);
    if ((nthreads + 255) / 256 >= (1ll << 31)) return hipErrorInvalidValue;
    hipLaunchKernelGGL((zero_unfilled_slots_kernel<HD>), dim3((unsigned)((nthreads + 255) / 256)), dim3(256), 0, stream, a,
                       rows, batches);
    const hipError_t ez = hipGetLastError();
    if (ez != hipSuccess) return ez;
  }
  if constexpr (HD <= 128) if (depth_by_chunks && (int64_t)a.B * a.T > 0) {
    constexpr size_t csmem = (2 * 64 + 4 * 32) * HD * sizeof(uint16_t) + 2 * 64 * sizeof(float);
    const int64_t nx = (((int64_t)a.T + a.Cb - 1) / a.Cb) * a.B * a.Hkv;
    if (nx >= (1ll << 31)) return hipErrorInvalidValue;
    static LdsAttrState cattr, cattr_packed;
    const hipError_t ec =
        a.cu ? allow_dynamic_lds(cattr_packed, reinterpret_cast<const void*>(&chunk_depth_kernel<T, HD, true>), csmem)
             : allow_dynamic_lds(cattr, reinterpret_cast<const void*>(&chunk_depth_kernel<T, HD, false>), csmem);
    if (ec != hipSuccess) return ec;
    if (a.cu)
      hipLaunchKernelGGL((chunk_depth_kernel<T, HD, true>), dim3((unsigned)nx), dim3(256), csmem, stream, a);
    else
      hipLaunchKernelGGL((chunk_depth_kernel<T, HD, false>), dim3((unsigned)nx), dim3(256), csmem, stream, a);
  }
  if (depth_by_columns && (int64_t)a.B * a.T > 0) {
    constexpr int CPB = 4 * (64 / (HD / 8));
    const int64_t nx = (((int64_t)a.T * a.L + CPB - 1) / CPB) * a.B * a.Hkv;
    if (nx >= (1ll << 31)) return hipErrorInvalidValue;
    if constexpr (HD <= 128) {
      if (a.depth_p && a.Gf <= 4) {
        constexpr int TPB = 4 * (64 / (HD / 8));
        const int64_t nt = (((int64_t)a.T + TPB - 1) / TPB) * a.B * a.Hkv;
        hipLaunchKernelGGL((depth_token_handed_kernel<T, HD>), dim3((unsigned)nt), dim3(256), 0, stream, a);
      } else if (a.depth_p)
        hipLaunchKernelGGL((depth_cols_handed_kernel<T, HD>), dim3((unsigned)nx), dim3(256), 0, stream, a);
      else
        hipLaunchKernelGGL((depth_cols_kernel<T, HD>), dim3((unsigned)nx), dim3(256), 0, stream, a);
    } else {
      hipLaunchKernelGGL((depth_cols_kernel<T, HD>), dim3((unsigned)nx), dim3(256), 0, stream, a);
    }
  }
  return hipGetLastError();
}

template __global__ void depth_cols_kernel<BF16, 128>(const KArgs);
template __global__ void depth_cols_kernel<BF16, 64>(const KArgs);
template __global__ void depth_cols_kernel<FP16, 128>(const KArgs);
template __global__ void depth_cols_kernel<FP16, 64>(const KArgs);
template __global__ void dkv_kernel<BF16, 128, false, true>(const KArgs);
template __global__ void dkv_kernel<BF16, 64, false, true>(const KArgs);
template __global__ void dkv_kernel<FP16, 128, false, true>(const KArgs);
template __global__ void dkv_kernel<FP16, 64, false, true>(const KArgs);
template __global__ void dkv_kernel<BF16, 128, false>(const KArgs);
template __global__ void dkv_kernel<BF16, 128, true>(const KArgs);
template __global__ void dkv_kernel<BF16, 64, false>(const KArgs);
template __global__ void dkv_kernel<BF16, 64, true>(const KArgs);
template __global__ void dkv_kernel<FP16, 128, false>(const KArgs);
template __global__ void dkv_kernel<FP16, 128, true>(const KArgs);
template __global__ void dkv_kernel<FP16, 64, false>(const KArgs);
template __global__ void dkv_kernel<FP16, 64, true>(const KArgs);

hipError_t launch_dkv(const KArgs& a, int dtype, int hd, hipStream_t stream) {
  if (dtype == 0 && hd == 128) return launch_dkv_t<BF16, 128>(a, stream);
  if (dtype == 0 && hd == 64) return launch_dkv_t<BF16, 64>(a, stream);
  if (dtype == 1 && hd == 128) return launch_dkv_t<FP16, 128>(a, stream);
  if (dtype == 1 && hd == 64) return launch_dkv_t<FP16, 64>(a, stream);
  if (dtype == 0 && hd == 256) return launch_dkv_t<BF16, 256>(a, stream);
  if (dtype == 1 && hd == 256) return launch_dkv_t<FP16, 256>(a, stream);
  return hipErrorInvalidValue;
}

}  // namespace moda
