// Forward kernel: one online softmax over the visible sequence keys and the
// query's depth-KV slots (the computation of moda_v14.py:45-378,
// moda_v16.py:39-352, fda_v12.py:44-253 and fla/ops/attn/parallel.py:18-143).
//
// Work split: one workgroup = 32 query rows per wave of one (batch, query
// head).  Scores are produced transposed, S^T = K * Q^T, so each lane owns ONE
// query row: row statistics need a single half-wave exchange and P^T is already
// laid out as the B operand of O^T += V^T * P^T.  K and V tiles (64 columns)
// travel global -> LDS without touching registers, a ring of stages keeps the
// loads ahead of the math, V is read with the LDS transpose load.  Depth
// columns are extra column tiles with a different per-row visible interval.
//
// Vector-ALU instructions do not overlap with MFMA on this hardware, so the
// loop over column tiles is split in two: tiles every row of the workgroup sees
// completely run a body without any masking or visibility tests; boundary and
// depth tiles run the masked body.
#include <algorithm>
#include <type_traits>

#include "geometry.h"
#include "kargs.h"
#include "tile.h"
#include "tile16.h"
#include "tuning.h"

namespace moda {

// launch shape of the forward kernel for all but small problems
using FwdLarge = RowLargePP;

// ADDR bit 0: a (batch, head) slice is wider than 2 GiB (descriptors anchored per tile instead of 32-bit
// offsets inside the slice); bit 1: packed variable-length batch; bit 2: no depth stream; bit 3: partially filled
// depth stream (only Lv of a token's L slots hold data: depth tiles are loaded through the slot mapping)
template <typename T, int HD, typename Shape, int ADDR>
__global__ __launch_bounds__(64 * Shape::W, 2) void fwd_kernel(const KArgs a_in) {
  constexpr int BM = 32 * Shape::W, BN = 64, KK = HD / 16, DB = HD / 32, NT = 64 * Shape::W, NST = Shape::NST,
                DIST = Shape::DIST;
  constexpr bool PP = Shape::PP;
  // on the 64-wide tiles the waves' own depth columns go through two sets of private tiles (see the end of the kernel)
  constexpr bool TWO_OWN_SETS = HD <= 64;
  static_assert(NST >= DIST + 1 + (PP ? 1 : 0) && DIST >= 1 && DIST <= 2,
                "ring must hold the tile in use, the tiles in flight and (ping-pong) the previous tile");
  static_assert(2 * NST >= Shape::W, "the ring must be large enough for one 32-column K tile and V tile per wave");
  extern __shared__ __align__(16) unsigned char smem_raw[];
  lds_ptr smem = (lds_ptr)smem_raw;  // ring stage st: K tile at smem + st * 2*BN*HD, V tile right behind it

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n = lane & 31, g = lane >> 5;
  constexpr bool WIDE = (ADDR & 1) != 0, VARLEN = (ADDR & 2) != 0;
  // bit 2: launched without a depth stream (the plain and sequence-only calls): the depth code is compiled out,
  // so that it cannot disturb the register allocation of their main loop
  constexpr bool NODEPTH = (ADDR & 4) != 0, PARTIAL = (ADDR & 8) != 0;
  static_assert(!(NODEPTH && PARTIAL), "a partially filled depth stream is a depth stream");
  const int BH = a_in.B * a_in.Hq;
  const int bh = blockIdx.x % BH;
  int b = bh / a_in.Hq;
  const int hq = bh % a_in.Hq, hkv = hq / a_in.hdiv;
  SeqArgs<VARLEN> seq(a_in, b);
  const KArgs& a = seq.a;
  const int Ld = NODEPTH ? 0 : a.L;  // depth slots per token
  const int nqt = (a.Tq + BM - 1) / BM;
  // heavy (late) tiles first; the positions a shorter sequence of a variable-length batch does not have are dropped
  const int qt = query_tile_of(blockIdx.x, BH, BM, VARLEN ? a_in.Tq : a.Tq);
  if (VARLEN && qt >= nqt) return;
  const int r = qt * BM + wave * 32 + n;
  const bool valid = r < a.Tq;
  const int t = r / a.Gf;

  i32x4 Qr[KK];
  {
    const uint16_t* qp = a.q + b * a.sq.b + hq * a.sq.h + (int64_t)r * a.sq.t + 8 * g;
#pragma unroll
    for (int kk = 0; kk < KK; kk++) {
      i32x4 z = {0, 0, 0, 0};
      Qr[kk] = (valid && 16 * kk + 8 * g < a.D) ? *reinterpret_cast<const i32x4*>(qp + 16 * kk) : z;
    }
  }

  // The register operands above must have arrived before the tile loads start: those are issued
  // behind the compiler's back, and a load it still believes pending would cost a vmcnt(0) in every
  // trip of the main loop.
  asm volatile("" ::: "memory");  // keep the loads above this point
  __builtin_amdgcn_s_waitcnt(0x0F70);
  asm volatile("" ::: "memory");

  // per-row visible column intervals [lo, hi) for the two phases
  const RowVis vis = row_visibility(a, r, Ld);
  const int shi = vis.shi, dlo = vis.dlo, dhi = vis.dhi;
  // Depth columns a wave alone can see are not streamed through the workgroup's ring: each wave fetches its own
  // rows' span after the sequence tiles (see the end of the kernel).
  const bool own_depth = waves_own_depth(a, Ld);
  const RowTilePlan plan = row_tile_plan(a, qt, BM, BN, Ld > 0 && !own_depth);
  int n_seq = plan.n_seq, n_full = plan.n_full, dep0 = plan.dep0;
  const int n_dep = plan.n_dep;
  // wave-uniform by construction, but computed with vector divisions: the explicit hint keeps the
  // loop control in scalar registers
  n_seq = __builtin_amdgcn_readfirstlane(n_seq);
  n_full = __builtin_amdgcn_readfirstlane(n_full);
  dep0 = __builtin_amdgcn_readfirstlane(dep0);
  const int ntiles = __builtin_amdgcn_readfirstlane(n_seq + n_dep);

  typedef AsyncTileLoader<HD, BN, NT> Loader;
  constexpr int LPT = 2 * Loader::N;  // vector-memory loads one wave issues per tile (K + V)
  Loader ld;
  ld.init(tid);
  // the two sources being streamed: sequence K/V first, swapped for the depth K/V when the
  // producer reaches the first depth tile
  typename Loader::Source srcK, srcV;
  if (a.has_seq && n_seq > 0) {
    srcK = ld.source(a.k + b * a.sk.b + hkv * a.sk.h, a.sk.t, 0, a.T, a.D);
    srcV = ld.source(a.v + b * a.sv.b + hkv * a.sv.h, a.sv.t, 0, a.T, a.Dv);
  }
  int ld_st = 0;  // ring stage the next issued tile goes to
  auto issue = [&](int it) {
    lds_ptr Kt = smem + ld_st * 2 * BN * HD;
    if (!NODEPTH && it == n_seq) {
      srcK = ld.source(a.kd + b * a.skd.b + hkv * a.skd.h, a.skd.t, dep0, a.T * a.L, a.D);
      srcV = ld.source(a.vd + b * a.svd.b + hkv * a.svd.h, a.svd.t, dep0, a.T * a.L, a.Dv);
    }
    const int row0 = it < n_seq ? it * BN : dep0 + (it - n_seq) * BN;
    if (PARTIAL && it >= n_seq) {  // depth tile of a partially filled stream: rows through the slot mapping
      ld.load_mapped(Kt, a.kd + b * a.skd.b + hkv * a.skd.h, a.skd.t, row0, (int64_t)a.T * a.L, a.L, a.Lv, a.D);
      ld.load_mapped(Kt + BN * HD, a.vd + b * a.svd.b + hkv * a.svd.h, a.svd.t, row0, (int64_t)a.T * a.L, a.L, a.Lv,
                     a.Dv);
    } else if (WIDE) {  // some slice spans more than 2 GiB: a descriptor anchored at this tile
      const bool dep = !NODEPTH && it >= n_seq;
      const int row_end = dep ? a.T * a.L : a.T;
      ld.load(Kt, dep ? a.kd + b * a.skd.b + hkv * a.skd.h : a.k + b * a.sk.b + hkv * a.sk.h, dep ? a.skd.t : a.sk.t,
              row0, row_end, a.D);
      ld.load(Kt + BN * HD, dep ? a.vd + b * a.svd.b + hkv * a.svd.h : a.v + b * a.sv.b + hkv * a.sv.h,
              dep ? a.svd.t : a.sv.t, row0, row_end, a.Dv);
    } else {
      ld.load_from(Kt, srcK, row0);
      ld.load_from(Kt + BN * HD, srcV, row0);
    }
    ld_st = (ld_st + 1 == NST) ? 0 : ld_st + 1;
  };
  // wait until tile `next` has landed; tiles next+1 .. next+DIST-1 may still be in flight
  auto wait_tile = [&](int next) {
    if (DIST == 2 && next + 1 < ntiles)
      Loader::template wait_but<LPT>();
    else
      Loader::wait_all();
  };

  f32x16 o[DB];
#pragma unroll
  for (int d = 0; d < DB; d++)
#pragma unroll
    for (int i = 0; i < 16; i++) o[d][i] = 0.f;
  float m = kNegInf, l = 0.f;
  const float sc = a.scale * kLog2e;
  OperandAddr<HD> oa;
  oa.init(lane);

#pragma unroll
  for (int j = 0; j < DIST; j++)
    if (j < ntiles) issue(j);
  wait_tile(0);
  __syncthreads();
  int c_st = 0;  // ring stage of the tile being consumed

  // One column tile in two halves.  front: S^T = K Q^T and the online softmax, leaving the rounded
  // probabilities in P; back: O^T += V^T P^T.
  i32x4 P[4];
  TrPipe<T, HD, 4, 2> pv;
  const std::integral_constant<int, 2> two{};
  auto front = [&](auto masked, auto nblk, lds_cptr Kc, int col0, int lo, int hi, auto&& after_scores) {
    constexpr bool MASKED = decltype(masked)::value;
    constexpr int NBLK = decltype(nblk)::value;  // 32-column blocks of the tile
    f32x16 s[NBLK];
    mfma_rows<T, HD, NBLK, 4>(oa, Kc, Qr, s);
    after_scores();
    // row maximum of the raw scores (scale > 0, so it commutes with the max)
    float mx = kNegInf;
#pragma unroll
    for (int bb = 0; bb < NBLK; bb++)
#pragma unroll
      for (int i = 0; i < 16; i++) {
        if (MASKED) {
          const int c = col0 + 32 * bb + acc_row(i, g);
          mx = fmaxf(mx, (c >= lo && c < hi) ? s[bb][i] : kNegInf);
        } else {
          mx = fmaxf(mx, s[bb][i]);
        }
      }
    mx = pair_max(mx) * sc;
    // The exponent reference m only moves when some row's maximum outgrows it by more than 2^8:
    // p stays <= 256, exact in fp32 accumulation and harmless in the 16-bit P, and the
    // rescale of O is skipped on almost every tile.
    if (__any(mx > m + 8.f)) {
      const float m_new = fmaxf(m, mx);
      const float alpha = fast_exp2(m - ((m_new == kNegInf) ? 0.f : m_new));
      l *= alpha;
      m = m_new;
#pragma unroll
      for (int d = 0; d < DB; d++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[d][i] *= alpha;
    }
    const float neg_m = (m == kNegInf) ? 0.f : -m;
    float rs0 = 0.f, rs1 = 0.f;  // fp32 row sum of the unrounded probabilities, as the reference keeps it
#pragma unroll
    for (int bb = 0; bb < NBLK; bb++)
#pragma unroll
      for (int i = 0; i < 16; i++) {
        float p = fast_exp2(__builtin_fmaf(s[bb][i], sc, neg_m));
        if (MASKED) {
          const int c = col0 + 32 * bb + acc_row(i, g);
          p = (c >= lo && c < hi) ? p : 0.f;
        }
        s[bb][i] = p;
        if (i & 1)
          rs1 += p;
        else
          rs0 += p;
      }
#pragma unroll
    for (int ks = 0; ks < 2 * NBLK; ks++) P[ks] = pack8<T>(s[ks >> 1], (ks & 1) * 8);
    l += pair_sum(rs0 + rs1);
  };
  // the whole tile at once: the first V^T operands start travelling while the softmax runs
  auto tile = [&](auto masked, lds_cptr Kc, lds_cptr Vc, int col0, int lo, int hi) {
    front(masked, two, Kc, col0, lo, hi, [&]() { pv.prefetch(oa, Vc); });
    pv.run(oa, Vc, P, o);
  };
  auto back = [&](lds_cptr Vc) {
    pv.prefetch(oa, Vc);
    pv.run(oa, Vc, P, o);
  };
  auto stage_k = [&](int st) { return smem + st * 2 * BN * HD; };

  // Ping-pong: the two waves of a SIMD (wave w and w + W/2) would otherwise run the same phase at the
  // same time -- matrix pipe contended during the MFMA phases, idle during both softmaxes.  The upper
  // half of the workgroup therefore runs half a tile behind: between two barriers it first finishes the
  // previous tile (V product), then does scores and softmax of the current one, so its softmax overlaps
  // the lower half's V product and its V product the lower half's scores.  The previous tile's V must
  // survive one more barrier interval, hence the extra ring stage.
  const bool late = PP && __builtin_amdgcn_readfirstlane(wave) >= Shape::W / 2;
  int it = 0;
  if (!late) {
    // phase 1: tiles fully visible to every row -- no masks, no visibility tests.  The loop is unrolled
    // over the ring stages so that each copy reads its tile at a compile-time LDS offset (the stage
    // offset then rides in the instructions' immediate field instead of costing an address add per
    // operand read); the remainder runs the same body with the stage in a register.
    auto full_tile = [&](lds_cptr Kc) {
      if (it + DIST < ntiles) issue(it + DIST);
      tile(std::false_type{}, Kc, Kc + BN * HD, it * BN, 0, 0);
      wait_tile(it + 1);
      __syncthreads();
      it++;
    };
    for (; it + NST <= n_full;) {
      full_tile(smem);
      full_tile(smem + 1 * 2 * BN * HD);
      if (NST > 2) full_tile(smem + 2 * 2 * BN * HD);
      if (NST > 3) full_tile(smem + 3 * 2 * BN * HD);
    }
    c_st = 0;
    for (; it < n_full;) {
      full_tile(stage_k(c_st));
      c_st = (c_st + 1 == NST) ? 0 : c_st + 1;
    }
    // phase 2: boundary sequence tiles and depth tiles
    for (; it < ntiles; it++) {
      if (it + DIST < ntiles) issue(it + DIST);
      const bool dep = !NODEPTH && it >= n_seq;
      const int col0 = dep ? dep0 + (it - n_seq) * BN : it * BN;
      const int lo = dep ? dlo : 0;
      const int hi = dep ? dhi : shi;
      const bool touches = (hi > col0) && (lo < col0 + BN) && (hi > lo);
      if (__any(touches)) {
        lds_cptr Kc = stage_k(c_st);
        tile(std::true_type{}, Kc, Kc + BN * HD, col0, lo, hi);
      }
      c_st = (c_st + 1 == NST) ? 0 : c_st + 1;
      wait_tile(it + 1);
      __syncthreads();
    }
  } else {
    // the late half: [V product of the previous tile] [scores + softmax of this tile] [barrier]
    if (n_full > 0) {  // first tile: nothing to finish yet
      if (DIST < ntiles) issue(DIST);
      front(std::false_type{}, two, smem, 0, 0, 0, []() {});
      wait_tile(1);
      __syncthreads();
      it = 1;
    }
    // `Vp`: V tile of the previous tile, `Kc`: K tile of this one
    auto full_tile = [&](lds_cptr Vp, lds_cptr Kc) {
      if (it + DIST < ntiles) issue(it + DIST);
      back(Vp);
      front(std::false_type{}, two, Kc, it * BN, 0, 0, []() {});
      wait_tile(it + 1);
      __syncthreads();
      it++;
    };
    if (NST == 4) {
      // it % NST == 1 here (or no full tile at all): copies with compile-time stages
      for (; it + NST <= n_full;) {
        full_tile(smem + BN * HD, smem + 1 * 2 * BN * HD);
        full_tile(smem + 1 * 2 * BN * HD + BN * HD, smem + 2 * 2 * BN * HD);
        full_tile(smem + 2 * 2 * BN * HD + BN * HD, smem + 3 * 2 * BN * HD);
        full_tile(smem + 3 * 2 * BN * HD + BN * HD, smem);
      }
    }
    c_st = it % NST;
    for (; it < n_full;) {
      const int prev = (c_st == 0) ? NST - 1 : c_st - 1;
      full_tile(stage_k(prev) + BN * HD, stage_k(c_st));
      c_st = (c_st + 1 == NST) ? 0 : c_st + 1;
    }
    bool pending = it > 0;  // a tile whose V product is still to do
    int p_st = (c_st == 0) ? NST - 1 : c_st - 1;
    for (; it < ntiles; it++) {
      if (it + DIST < ntiles) issue(it + DIST);
      if (pending) back(stage_k(p_st) + BN * HD);
      pending = false;
      const bool dep = !NODEPTH && it >= n_seq;
      const int col0 = dep ? dep0 + (it - n_seq) * BN : it * BN;
      const int lo = dep ? dlo : 0;
      const int hi = dep ? dhi : shi;
      const bool touches = (hi > col0) && (lo < col0 + BN) && (hi > lo);
      if (__any(touches)) {
        front(std::true_type{}, two, stage_k(c_st), col0, lo, hi, []() {});
        pending = true;
        p_st = c_st;
      }
      c_st = (c_st + 1 == NST) ? 0 : c_st + 1;
      wait_tile(it + 1);
      __syncthreads();
    }
    if (pending) back(stage_k(p_st) + BN * HD);
  }

  if (own_depth) {
    // The wave's own depth columns, 32 at a time through a wave-private K tile and V tile cut out of the ring
    // (no workgroup barrier after the one that retires the ring).  The next K tile is fetched as soon as the
    // scores are out, the next V tile once the V product is.
    __syncthreads();
    typedef WaveTileLoader<HD> Own;
    const int wv = __builtin_amdgcn_readfirstlane(wave);
    lds_ptr Kt = smem + wv * (2 * 32 * HD), Vt = Kt + 32 * HD;
    const int rw0 = qt * BM + wv * 32;
    if (rw0 < a.Tq) {
      const DepthSpan span = own_depth_span(a, rw0, 32);
      const int c_beg = __builtin_amdgcn_readfirstlane(span.c_beg);
      const int c_end = __builtin_amdgcn_readfirstlane(span.c_end);
      const int nh = (c_end - c_beg + 31) / 32;
      const uint16_t* kdp = a.kd + b * a.skd.b + hkv * a.skd.h;
      const uint16_t* vdp = a.vd + b * a.svd.b + hkv * a.svd.h;
      Own own;
      own.init(lane);
      // rows [col0, col0 + 32) of the span (short at its end) into a private tile; d: the tensor's head dim
      auto fetch = [&](lds_ptr tile, const uint16_t* slice, int64_t stride, int col0, int d) {
        const int nrows = min(32, c_end - col0);
        if (PARTIAL)
          own.fetch_mapped(tile, slice, stride, col0, nrows, (int64_t)a.T * a.L, a.L, a.Lv, d);
        else
          own.fetch(tile, slice, stride, col0, nrows, d);
      };
      fetch(Kt, kdp, a.skd.t, c_beg, a.D);
      fetch(Vt, vdp, a.svd.t, c_beg, a.Dv);
      const std::integral_constant<int, 1> one{};
      if constexpr (TWO_OWN_SETS) {
        // room for two sets of private tiles: the rows of tile j + 1 travel while tile j is worked on
        constexpr int SET = Shape::W * 2 * 32 * HD;
        for (int j = 0; j < nh; j++) {
          const int col0 = c_beg + 32 * j;
          lds_ptr Kc = Kt + (j & 1) * SET, Vc = Vt + (j & 1) * SET;
          Own::template wait_but<0>();
          if (j + 1 < nh) {
            fetch(Kt + ((j + 1) & 1) * SET, kdp, a.skd.t, col0 + 32, a.D);
            fetch(Vt + ((j + 1) & 1) * SET, vdp, a.svd.t, col0 + 32, a.Dv);
          }
          front(std::true_type{}, one, Kc, col0, dlo, dhi, []() {});
          TrPipe<T, HD, 2, 2> pv1;
          const i32x4 P1[2] = {P[0], P[1]};
          pv1.prefetch(oa, Vc);
          pv1.run(oa, Vc, P1, o);
          Own::reads_done();  // this set may be loaded over in the next trip
        }
      } else {
      for (int j = 0; j < nh; j++) {
        const int col0 = c_beg + 32 * j;
        const bool more = j + 1 < nh;
        Own::template wait_but<Own::N>();  // K landed, V may still be on its way
        front(std::true_type{}, one, Kt, col0, dlo, dhi, []() {});
        Own::reads_done();
        if (more) fetch(Kt, kdp, a.skd.t, col0 + 32, a.D);
        if (more)
          Own::template wait_but<Own::N>();  // V landed, the next K on its way
        else
          Own::template wait_but<0>();
        TrPipe<T, HD, 2, 2> pv1;
        const i32x4 P1[2] = {P[0], P[1]};
        pv1.prefetch(oa, Vt);
        pv1.run(oa, Vt, P1, o);
        Own::reads_done();
        if (more) fetch(Vt, vdp, a.svd.t, col0 + 32, a.Dv);
      }
      }
    }
  }

  if (valid) {
    const float inv = l > 0.f ? 1.f / l : 0.f;
    uint16_t* op = a.out_o + b * a.so.b + hq * a.so.h + (int64_t)r * a.so.t;
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        i32x2 w;
        w[0] = pack2<T>(o[d][4 * i4 + 0] * inv, o[d][4 * i4 + 1] * inv);
        w[1] = pack2<T>(o[d][4 * i4 + 2] * inv, o[d][4 * i4 + 3] * inv);
        if (32 * d + 8 * i4 + 4 * g < a.Dv) *reinterpret_cast<i32x2*>(op + 32 * d + 8 * i4 + 4 * g) = w;
      }
    if (g == 0) a.lse[((int64_t)b * a.Tq + r) * a.Hq + hq] = (l > 0.f) ? m + log2f(l) : kNegInf;
  }
}

// The forward kernel for the 256-wide tiles (head dims above 128), on the 16x16x32 matrix instruction: a wave
// owns 16 * NB query rows (NB = 1 here: Q and the 256-wide O accumulator of 32 rows would not fit the register
// file), lane (n, q) owns rows 16*nb + n and, inside a 16-column score block, columns slot_base(q) .. +3; four
// lanes share a row, their shares of the row sum are added at the end.  Same streaming structure and the same
// arithmetic as fwd_kernel (which stays on 32x32x16: on the narrower tiles it is the faster of the two); depth
// columns always stream through the workgroup's ring.
template <typename T, int HD, typename Shape, int ADDR>
__global__ __launch_bounds__(64 * Shape::W, 2) void fwd_wide_kernel(const KArgs a_in) {
  constexpr int NB = Shape::NB, WR = 16 * NB, BM = WR * Shape::W, BN = 64, KS = HD / 32, MB = HD / 16, NT = 64 * Shape::W, NST = Shape::NST,
                DIST = Shape::DIST;
  static_assert(!Shape::PP, "no ping-pong schedule here");
  static_assert(NST >= DIST + 1 && DIST >= 1 && DIST <= 2, "ring must hold the tile in use plus the tiles in flight");
  extern __shared__ __align__(16) unsigned char smem_raw[];
  lds_ptr smem = (lds_ptr)smem_raw;  // ring stage st: K tile at smem + st * 2*BN*HD, V tile right behind it

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n = lane & 15, q4 = lane >> 4;
  constexpr bool WIDE = (ADDR & 1) != 0, VARLEN = (ADDR & 2) != 0, PARTIAL = (ADDR & 8) != 0;
  const int BH = a_in.B * a_in.Hq;
  const int bh = blockIdx.x % BH;
  int b = bh / a_in.Hq;
  const int hq = bh % a_in.Hq, hkv = hq / a_in.hdiv;
  SeqArgs<VARLEN> seq(a_in, b);
  const KArgs& a = seq.a;
  const int nqt = (a.Tq + BM - 1) / BM;
  // heavy (late) tiles first; the positions a shorter sequence of a variable-length batch does not have are dropped
  const int qt = query_tile_of(blockIdx.x, BH, BM, VARLEN ? a_in.Tq : a.Tq);
  if (VARLEN && qt >= nqt) return;
  i32x4 Qr[NB][KS];
  int shi[NB], dlo[NB], dhi[NB];  // per-row visible column intervals [lo, hi) for the two phases
#pragma unroll
  for (int nb = 0; nb < NB; nb++) {
    const int r = qt * BM + wave * WR + 16 * nb + n;
    const bool valid = r < a.Tq;
    const uint16_t* qp = a.q + b * a.sq.b + hq * a.sq.h + (int64_t)r * a.sq.t + 8 * q4;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      i32x4 z = {0, 0, 0, 0};
      Qr[nb][ks] = (valid && 32 * ks + 8 * q4 < a.D) ? *reinterpret_cast<const i32x4*>(qp + 32 * ks) : z;
    }
    const RowVis vis = row_visibility(a, r, a.L);
    shi[nb] = vis.shi;
    dlo[nb] = vis.dlo;
    dhi[nb] = vis.dhi;
  }

  // The register operands above must have arrived before the tile loads start: those are issued
  // behind the compiler's back, and a load it still believes pending would cost a vmcnt(0) in every
  // trip of the main loop.
  asm volatile("" ::: "memory");  // keep the loads above this point
  __builtin_amdgcn_s_waitcnt(0x0F70);
  asm volatile("" ::: "memory");

  // the workgroup's column tiles: depth columns always stream through the ring here
  const RowTilePlan plan = row_tile_plan(a, qt, BM, BN, a.L > 0);
  int n_seq = plan.n_seq, n_full = plan.n_full, dep0 = plan.dep0;
  const int n_dep = plan.n_dep;
  // wave-uniform by construction, but computed with vector divisions: the explicit hint keeps the
  // loop control in scalar registers
  n_seq = __builtin_amdgcn_readfirstlane(n_seq);
  n_full = __builtin_amdgcn_readfirstlane(n_full);
  dep0 = __builtin_amdgcn_readfirstlane(dep0);
  const int ntiles = __builtin_amdgcn_readfirstlane(n_seq + n_dep);

  typedef AsyncTileLoader<HD, BN, NT> Loader;
  constexpr int LPT = 2 * Loader::N;  // vector-memory loads one wave issues per tile (K + V)
  Loader ld;
  ld.init(tid);
  // the two sources being streamed: sequence K/V first, swapped for the depth K/V when the
  // producer reaches the first depth tile
  typename Loader::Source srcK, srcV;
  if (a.has_seq && n_seq > 0) {
    srcK = ld.source(a.k + b * a.sk.b + hkv * a.sk.h, a.sk.t, 0, a.T, a.D);
    srcV = ld.source(a.v + b * a.sv.b + hkv * a.sv.h, a.sv.t, 0, a.T, a.Dv);
  }
  int ld_st = 0;  // ring stage the next issued tile goes to
  auto issue = [&](int it) {
    lds_ptr Kt = smem + ld_st * 2 * BN * HD;
    if (it == n_seq) {
      srcK = ld.source(a.kd + b * a.skd.b + hkv * a.skd.h, a.skd.t, dep0, a.T * a.L, a.D);
      srcV = ld.source(a.vd + b * a.svd.b + hkv * a.svd.h, a.svd.t, dep0, a.T * a.L, a.Dv);
    }
    const int row0 = it < n_seq ? it * BN : dep0 + (it - n_seq) * BN;
    if (PARTIAL && it >= n_seq) {  // depth tile of a partially filled stream: rows through the slot mapping
      ld.load_mapped(Kt, a.kd + b * a.skd.b + hkv * a.skd.h, a.skd.t, row0, (int64_t)a.T * a.L, a.L, a.Lv, a.D);
      ld.load_mapped(Kt + BN * HD, a.vd + b * a.svd.b + hkv * a.svd.h, a.svd.t, row0, (int64_t)a.T * a.L, a.L, a.Lv,
                     a.Dv);
    } else if (WIDE) {  // some slice spans more than 2 GiB: a descriptor anchored at this tile
      const bool dep = it >= n_seq;
      const int row_end = dep ? a.T * a.L : a.T;
      ld.load(Kt, dep ? a.kd + b * a.skd.b + hkv * a.skd.h : a.k + b * a.sk.b + hkv * a.sk.h, dep ? a.skd.t : a.sk.t,
              row0, row_end, a.D);
      ld.load(Kt + BN * HD, dep ? a.vd + b * a.svd.b + hkv * a.svd.h : a.v + b * a.sv.b + hkv * a.sv.h,
              dep ? a.svd.t : a.sv.t, row0, row_end, a.Dv);
    } else {
      ld.load_from(Kt, srcK, row0);
      ld.load_from(Kt + BN * HD, srcV, row0);
    }
    ld_st = (ld_st + 1 == NST) ? 0 : ld_st + 1;
  };
  // wait until tile `next` has landed; tiles next+1 .. next+DIST-1 may still be in flight
  auto wait_tile = [&](int next) {
    if (DIST == 2 && next + 1 < ntiles)
      Loader::template wait_but<LPT>();
    else
      Loader::wait_all();
  };

  f32x4 o[MB][NB];
#pragma unroll
  for (int d = 0; d < MB; d++)
#pragma unroll
    for (int nb = 0; nb < NB; nb++) o[d][nb] = f32x4{0.f, 0.f, 0.f, 0.f};
  // exponent reference (shared by the four lanes of a row) and this lane's share of the row sum
  float m[NB], l[NB];
#pragma unroll
  for (int nb = 0; nb < NB; nb++) {
    m[nb] = kNegInf;
    l[nb] = 0.f;
  }
  const float sc = a.scale * kLog2e;
  Operand16<HD> oa;
  oa.init(lane);

#pragma unroll
  for (int j = 0; j < DIST; j++)
    if (j < ntiles) issue(j);
  wait_tile(0);
  __syncthreads();
  int c_st = 0;  // ring stage of the tile being consumed

  // One column tile in two halves.  front: S^T = K Q^T and the online softmax, leaving the rounded
  // probabilities in P; back: O^T += V^T P^T.
  i32x4 P[2][NB];
  TrPipe16<T, HD, 2, NB, 2> pv;
  auto front = [&](auto masked, lds_cptr Kc, int col0, const int (&lo)[NB], const int (&hi)[NB], auto&& after_scores) {
    constexpr bool MASKED = decltype(masked)::value;
    f32x4 s[4][NB];
    mfma16_rows<T, HD, 4, NB, 4>(oa, Kc, Qr, s);
    after_scores();
    // this lane's maximum of the raw scores of each row (scale > 0, so it commutes with the max)
    float mx[NB];
#pragma unroll
    for (int nb = 0; nb < NB; nb++) mx[nb] = kNegInf;
#pragma unroll
    for (int mb = 0; mb < 4; mb++)
#pragma unroll
      for (int nb = 0; nb < NB; nb++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
          if (MASKED) {
            const int c = col0 + 16 * mb + slot_base(q4) + i;
            mx[nb] = fmaxf(mx[nb], (c >= lo[nb] && c < hi[nb]) ? s[mb][nb][i] : kNegInf);
          } else {
            mx[nb] = fmaxf(mx[nb], s[mb][nb][i]);
          }
        }
    bool grows = false;
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
      mx[nb] *= sc;
      grows = grows || mx[nb] > m[nb] + 8.f;
    }
    // The exponent reference m only moves when some score outgrows it by more than 2^8:
    // p stays <= 256, exact in fp32 accumulation and harmless in the 16-bit P, and the row-wide
    // maximum and the rescale of O are skipped on almost every tile.
    if (__any(grows)) {
#pragma unroll
      for (int nb = 0; nb < NB; nb++) {
        const float m_new = fmaxf(m[nb], quad_max(mx[nb]));
        const float alpha = fast_exp2(m[nb] - ((m_new == kNegInf) ? 0.f : m_new));
        l[nb] *= alpha;
        m[nb] = m_new;
#pragma unroll
        for (int d = 0; d < MB; d++) o[d][nb] *= alpha;
      }
    }
    float rs[NB][2];  // fp32 row sum of the unrounded probabilities, as the reference keeps it
#pragma unroll
    for (int nb = 0; nb < NB; nb++) rs[nb][0] = rs[nb][1] = 0.f;
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
      const float neg_m = (m[nb] == kNegInf) ? 0.f : -m[nb];
#pragma unroll
      for (int mb = 0; mb < 4; mb++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
          float p = fast_exp2(__builtin_fmaf(s[mb][nb][i], sc, neg_m));
          if (MASKED) {
            const int c = col0 + 16 * mb + slot_base(q4) + i;
            p = (c >= lo[nb] && c < hi[nb]) ? p : 0.f;
          }
          s[mb][nb][i] = p;
          rs[nb][i & 1] += p;
        }
    }
#pragma unroll
    for (int ks = 0; ks < 2; ks++)
#pragma unroll
      for (int nb = 0; nb < NB; nb++) P[ks][nb] = pack_slots<T>(s[2 * ks][nb], s[2 * ks + 1][nb]);
#pragma unroll
    for (int nb = 0; nb < NB; nb++) l[nb] += rs[nb][0] + rs[nb][1];
  };
  // the whole tile at once: the first V^T operands start travelling while the softmax runs
  auto tile = [&](auto masked, lds_cptr Kc, lds_cptr Vc, int col0, const int (&lo)[NB], const int (&hi)[NB]) {
    front(masked, Kc, col0, lo, hi, [&]() { pv.prefetch(oa, Vc); });
    pv.run(oa, Vc, P, o);
  };
  auto stage_k = [&](int st) { return smem + st * 2 * BN * HD; };

  int none[NB];
#pragma unroll
  for (int nb = 0; nb < NB; nb++) none[nb] = 0;
  // phase 1: tiles fully visible to every row -- no masks, no visibility tests
  int it = 0;
  for (; it < n_full; it++) {
    if (it + DIST < ntiles) issue(it + DIST);
    lds_cptr Kc = stage_k(c_st);
    tile(std::false_type{}, Kc, Kc + BN * HD, it * BN, none, none);
    c_st = (c_st + 1 == NST) ? 0 : c_st + 1;
    wait_tile(it + 1);
    __syncthreads();
  }
  // phase 2: boundary sequence tiles and depth tiles
  for (; it < ntiles; it++) {
    if (it + DIST < ntiles) issue(it + DIST);
    const bool dep = it >= n_seq;
    const int col0 = dep ? dep0 + (it - n_seq) * BN : it * BN;
    int lo[NB], hi[NB];
    bool touches = false;
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
      lo[nb] = dep ? dlo[nb] : 0;
      hi[nb] = dep ? dhi[nb] : shi[nb];
      touches = touches || ((hi[nb] > col0) && (lo[nb] < col0 + BN) && (hi[nb] > lo[nb]));
    }
    if (__any(touches)) {
      lds_cptr Kc = stage_k(c_st);
      tile(std::true_type{}, Kc, Kc + BN * HD, col0, lo, hi);
    }
    c_st = (c_st + 1 == NST) ? 0 : c_st + 1;
    wait_tile(it + 1);
    __syncthreads();
  }

#pragma unroll
  for (int nb = 0; nb < NB; nb++) {
    const int r = qt * BM + wave * WR + 16 * nb + n;
    const float lsum = quad_sum(l[nb]);
    if (r < a.Tq) {
      const float inv = lsum > 0.f ? 1.f / lsum : 0.f;
      uint16_t* op = a.out_o + b * a.so.b + hq * a.so.h + (int64_t)r * a.so.t;
#pragma unroll
      for (int d = 0; d < MB; d++) {
        i32x2 w;
        w[0] = pack2<T>(o[d][nb][0] * inv, o[d][nb][1] * inv);
        w[1] = pack2<T>(o[d][nb][2] * inv, o[d][nb][3] * inv);
        if (16 * d + 4 * q4 < a.Dv) *reinterpret_cast<i32x2*>(op + 16 * d + 4 * q4) = w;
      }
      if (q4 == 0) a.lse[((int64_t)b * a.Tq + r) * a.Hq + hq] = (lsum > 0.f) ? m[nb] + log2f(lsum) : kNegInf;
    }
  }
}

template <typename T, int HD, typename Shape, int ADDR>
hipError_t launch_fwd_t_shape(const KArgs& a, hipStream_t stream) {
  // the ring, or (64-wide tiles) two sets of a private 32-column K tile and V tile per wave, whichever is larger
  constexpr size_t ring = (size_t)Shape::NST * 2 * 64 * HD * sizeof(uint16_t);
  constexpr size_t own = HD <= 64 ? (size_t)2 * Shape::W * 2 * 32 * HD * sizeof(uint16_t) : 0;
  constexpr size_t smem = ring > own ? ring : own;
  static LdsAttrState attr;
  const hipError_t ea = allow_dynamic_lds(attr, reinterpret_cast<const void*>(&fwd_kernel<T, HD, Shape, ADDR>), smem);
  if (ea != hipSuccess) return ea;
  const int64_t nblk = row_kernel_blocks(a, 32 * Shape::W);
  if (nblk == 0) return hipSuccess;
  if (nblk >= (1ll << 31)) return hipErrorInvalidValue;
  hipLaunchKernelGGL((fwd_kernel<T, HD, Shape, ADDR>), dim3((unsigned)nblk), dim3(64 * Shape::W), smem, stream, a);
  return hipGetLastError();
}

template <typename T, int HD, int ADDR>
hipError_t launch_fwd_wide(const KArgs& a, hipStream_t stream) {
  typedef RowWide Shape;
  constexpr size_t smem = (size_t)Shape::NST * 2 * 64 * HD * sizeof(uint16_t);
  static LdsAttrState attr;
  const hipError_t ea =
      allow_dynamic_lds(attr, reinterpret_cast<const void*>(&fwd_wide_kernel<T, HD, Shape, ADDR>), smem);
  if (ea != hipSuccess) return ea;
  constexpr int rows = 16 * Shape::NB * Shape::W;
  const int64_t nblk = row_kernel_blocks(a, rows);
  if (nblk == 0) return hipSuccess;
  if (nblk >= (1ll << 31)) return hipErrorInvalidValue;
  hipLaunchKernelGGL((fwd_wide_kernel<T, HD, Shape, ADDR>), dim3((unsigned)nblk), dim3(64 * Shape::W), smem, stream, a);
  return hipGetLastError();
}

template <typename T, int HD, int ADDR>
hipError_t launch_fwd_t_addr(const KArgs& a, bool small, hipStream_t stream) {
  if constexpr (HD > 128) return launch_fwd_wide<T, HD, ADDR & 11>(a, stream);
  else {
    if (ADDR & 1) return launch_fwd_t_shape<T, HD, FwdLarge, ADDR>(a, stream);  // slices wider than 2 GiB: never a small launch
    if (small) return launch_fwd_t_shape<T, HD, RowSmall<HD>, ADDR>(a, stream);
    return launch_fwd_t_shape<T, HD, FwdLarge, ADDR>(a, stream);
  }
}

template <typename T, int HD>
hipError_t launch_fwd_t(const KArgs& a, hipStream_t stream) {
  // byte span of the widest streamed (batch, head) slice
  const int64_t span = 2 * std::max(std::max((int64_t)a.T * a.sk.t, (int64_t)a.T * a.sv.t),
                                    std::max((int64_t)a.T * a.L * a.skd.t, (int64_t)a.T * a.L * a.svd.t));
  const bool wide = span > 0x7fffffffll;
  const bool small = use_small_rows(a.Tq, (long long)a.B * a.Hq, a.compute_units);
  switch ((wide ? 1 : 0) | (a.cu ? 2 : 0) | (a.L == 0 ? 4 : 0) | (a.L > 0 && a.Lv != a.L ? 8 : 0)) {
    case 0: return launch_fwd_t_addr<T, HD, 0>(a, small, stream);
    case 1: return launch_fwd_t_addr<T, HD, 1>(a, small, stream);
    case 2: return launch_fwd_t_addr<T, HD, 2>(a, small, stream);
    case 3: return launch_fwd_t_addr<T, HD, 3>(a, small, stream);
    case 4: return launch_fwd_t_addr<T, HD, 4>(a, small, stream);
    case 5: return launch_fwd_t_addr<T, HD, 5>(a, small, stream);
    case 6: return launch_fwd_t_addr<T, HD, 6>(a, small, stream);
    case 7: return launch_fwd_t_addr<T, HD, 7>(a, small, stream);
    case 8: return launch_fwd_t_addr<T, HD, 8>(a, small, stream);
    case 9: return launch_fwd_t_addr<T, HD, 9>(a, small, stream);
    case 10: return launch_fwd_t_addr<T, HD, 10>(a, small, stream);
    default: return launch_fwd_t_addr<T, HD, 11>(a, small, stream);
  }
}

hipError_t launch_fwd(const KArgs& a, int dtype, int hd, hipStream_t stream) {
  if (dtype == 0 && hd == 128) return launch_fwd_t<BF16, 128>(a, stream);
  if (dtype == 0 && hd == 64) return launch_fwd_t<BF16, 64>(a, stream);
  if (dtype == 1 && hd == 128) return launch_fwd_t<FP16, 128>(a, stream);
  if (dtype == 1 && hd == 64) return launch_fwd_t<FP16, 64>(a, stream);
  if (dtype == 0 && hd == 256) return launch_fwd_t<BF16, 256>(a, stream);
  if (dtype == 1 && hd == 256) return launch_fwd_t<FP16, 256>(a, stream);
  return hipErrorInvalidValue;
}

}  // namespace moda
