// Backward, query side: the preprocess kernel (-delta = -rowsum(o * do), moda_v14.py:525-539) and the
// dQ kernel (moda_v14.py:542-871, moda_v16.py:936-1220, fda_v12.py:432-638,
// fla/ops/attn/parallel.py:165-296).
//
// Same streaming structure as the forward kernel: a workgroup owns 32 query rows per wave
// (256 in the throughput launch shape, 64 or 128 in the small one) and streams 64-column K/V tiles
// (sequence keys, then the rows' depth slots) through an LDS ring.  The products run on the 16x16x32
// matrix instruction, which moves a quarter of the accumulator bits per multiply-add of the 32x32x16
// one and draws less power on a matrix pipe whose clock the power limit sets (measured on the
// long-sequence workload: about 9 % less time for the same tiles).  A wave's 32 rows are two 16-row
// blocks; lane (n, q) owns rows 16*nb + n and, inside a 16-column score block, columns slot_base(q) .. +3.
// P^T is recomputed from the saved base-2 LSE, dS^T = P^T * (dP^T - delta) is packed straight into the
// B operand of dQ^T += K^T * dS^T, K^T coming from the LDS transpose read of the K tile.
#include <algorithm>
#include <type_traits>

#include "geometry.h"
#include "kargs.h"
#include "tile.h"
#include "tile16.h"
#include "tuning.h"

namespace moda {

template <typename T, int HD>
__global__ __launch_bounds__(256) void delta_kernel(const KArgs a_in) {
  constexpr int TPR = HD / 8;         // threads per row
  constexpr int RPB = 256 / TPR;      // rows per block
  const int tid = threadIdx.x;
  // one-dimensional grid (row blocks of the longest sequence x batch*heads): the y extent of a grid stops at 65535
  const int nrb = (a_in.Tq + RPB - 1) / RPB;
  const int bh = blockIdx.x / nrb;
  const int rb = blockIdx.x - bh * nrb;
  KArgs a = a_in;
  int b = bh / a.Hq;
  const int hq = bh % a.Hq;
  enter_sequence(a, b);
  const int r = rb * RPB + tid / TPR;
  const int c = (tid % TPR) * 8;
  float acc = 0.f;
  if (r < a.Tq && c < a.Dv) {
    const uint16_t* op = a.o + b * a.so.b + hq * a.so.h + (int64_t)r * a.so.t + c;
    const uint16_t* dp = a.d_o + b * a.sdo.b + hq * a.sdo.h + (int64_t)r * a.sdo.t + c;
    const typename T::vec8 ov = *reinterpret_cast<const typename T::vec8*>(op);
    const typename T::vec8 dv = *reinterpret_cast<const typename T::vec8*>(dp);
#pragma unroll
    for (int i = 0; i < 8; i++) acc += (float)ov[i] * (float)dv[i];
  }
#pragma unroll
  for (int s = TPR / 2; s > 0; s >>= 1) acc += __shfl_xor(acc, s, 64);
  if (r < a.Tq && (tid % TPR) == 0) a.delta[((int64_t)b * a.Hq + hq) * a.delta_pitch + r] = -acc;
}

// ADDR bit 0: a (batch, head) slice is wider than 2 GiB (descriptors anchored per tile instead of 32-bit
// offsets inside the slice); bit 1: packed variable-length batch; bit 2: no depth stream; bit 3: partially filled
// depth stream (only Lv of a token's L slots hold data: depth tiles are loaded through the slot mapping)
template <typename T, int HD, typename Shape, int ADDR>
__global__ __launch_bounds__(64 * Shape::W, 2) void dq_kernel(const KArgs a_in) {
  constexpr int NB = Shape::NB, WR = 16 * NB, BM = WR * Shape::W, BN = 64, KS = HD / 32, MB = HD / 16, NT = 64 * Shape::W, NST = Shape::NST, DIST = Shape::DIST;
  static_assert(NST >= DIST + 1 && DIST >= 1 && DIST <= 2, "ring must hold the tile in use plus the tiles in flight");
  extern __shared__ __align__(16) unsigned char smem_raw[];
  lds_ptr smem = (lds_ptr)smem_raw;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n = lane & 15, q4 = lane >> 4;
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
  const int qt = query_tile_of(blockIdx.x, BH, BM, VARLEN ? a_in.Tq : a.Tq);
  if (VARLEN && qt >= nqt) return;

  i32x4 Qr[NB][KS], dOr[NB][KS];
  float lse[NB], delta[NB];
  int shi[NB], dlo[NB], dhi[NB];
#pragma unroll
  for (int nb = 0; nb < NB; nb++) {
    const int r = qt * BM + wave * WR + 16 * nb + n;
    const bool valid = r < a.Tq;
    const uint16_t* qp = a.q + b * a.sq.b + hq * a.sq.h + (int64_t)r * a.sq.t + 8 * q4;
    const uint16_t* dop = a.d_o + b * a.sdo.b + hq * a.sdo.h + (int64_t)r * a.sdo.t + 8 * q4;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      i32x4 z = {0, 0, 0, 0};
      Qr[nb][ks] = (valid && 32 * ks + 8 * q4 < a.D) ? *reinterpret_cast<const i32x4*>(qp + 32 * ks) : z;
      dOr[nb][ks] = (valid && 32 * ks + 8 * q4 < a.Dv) ? *reinterpret_cast<const i32x4*>(dop + 32 * ks) : z;
    }
    lse[nb] = 0.f;
    delta[nb] = 0.f;
    if (valid) lse[nb] = a.lse[((int64_t)b * a.Tq + r) * a.Hq + hq];
    float* drow = a.delta + ((int64_t)b * a.Hq + hq) * (VARLEN ? a.delta_pitch : a.Tq) + r;
    if (a.own_delta) {
      // minus rowsum(o * do) (moda_v14.py:525-539) from the dO pieces this lane holds anyway and the same pieces of
      // o; the four lanes of a row add their shares and the first one leaves the sum for the kernels that follow
      const uint16_t* orow = a.o + b * a.so.b + hq * a.so.h + (int64_t)r * a.so.t + 8 * q4;
      float acc = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        i32x4 z = {0, 0, 0, 0};
        const i32x4 ov = (valid && 32 * ks + 8 * q4 < a.Dv) ? *reinterpret_cast<const i32x4*>(orow + 32 * ks) : z;
#pragma unroll
        for (int w = 0; w < 4; w++) {
          float x0, x1, y0, y1;
          unpack2<T>(ov[w], x0, x1);
          unpack2<T>(dOr[nb][ks][w], y0, y1);
          acc = __builtin_fmaf(x0, y0, acc);
          acc = __builtin_fmaf(x1, y1, acc);
        }
      }
      acc = quad_sum(acc);
      delta[nb] = valid ? -acc : 0.f;
      if (valid && q4 == 0) *drow = -acc;
    } else if (valid) {
      delta[nb] = *drow;
    }
    const RowVis vis = row_visibility(a, r, Ld);
    shi[nb] = vis.shi;
    dlo[nb] = vis.dlo;
    dhi[nb] = vis.dhi;
  }
  // the register operands must have arrived before the tile loads (issued behind the compiler's back) start
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(0x0F70);
  asm volatile("" ::: "memory");

  // Depth columns a wave alone can see are not streamed through the workgroup's ring: each wave fetches its own
  // rows' span after the sequence tiles (see the end of the kernel), when a 32-column K and V tile per wave fit.
  constexpr bool OWN_FITS = Shape::W * 64 * HD * 2 <= 128 * 1024;
  const bool own_depth = OWN_FITS && waves_own_depth(a, Ld);
  const RowTilePlan plan = row_tile_plan(a, qt, BM, BN, Ld > 0 && !own_depth);
  int n_seq = plan.n_seq, n_full = plan.n_full, dep0 = plan.dep0;
  const int n_dep = plan.n_dep;
  n_seq = __builtin_amdgcn_readfirstlane(n_seq);
  n_full = __builtin_amdgcn_readfirstlane(n_full);
  dep0 = __builtin_amdgcn_readfirstlane(dep0);
  const int ntiles = __builtin_amdgcn_readfirstlane(n_seq + n_dep);

  constexpr int DMA_NOP = MODA_DMA_NOP;
  typedef AsyncTileLoader<HD, BN, NT, DMA_NOP> Loader;
  constexpr int LPT = 2 * Loader::N;
  Loader ld;
  ld.init(tid);
  typename Loader::Source srcK, srcV;
  if (a.has_seq && n_seq > 0) {
    srcK = ld.source(a.k + b * a.sk.b + hkv * a.sk.h, a.sk.t, 0, a.T, a.D);
    srcV = ld.source(a.v + b * a.sv.b + hkv * a.sv.h, a.sv.t, 0, a.T, a.Dv);
  }
  int ld_st = 0;
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
    } else if (WIDE) {
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
  auto wait_tile = [&](int next) {
    if (DIST == 2 && next + 1 < ntiles)
      Loader::template wait_but<LPT>();
    else
      Loader::wait_all();
  };

  f32x4 dq[MB][NB];
#pragma unroll
  for (int d = 0; d < MB; d++)
#pragma unroll
    for (int nb = 0; nb < NB; nb++) dq[d][nb] = f32x4{0.f, 0.f, 0.f, 0.f};
  const float sc = a.scale * kLog2e;
  Operand16<HD> oa;
  oa.init(lane);

#pragma unroll
  for (int j = 0; j < DIST; j++)
    if (j < ntiles) issue(j);
  wait_tile(0);
  __syncthreads();
  int c_st = 0;

  f32x4 dp_init[NB];
#pragma unroll
  for (int nb = 0; nb < NB; nb++) dp_init[nb] = f32x4{delta[nb], delta[nb], delta[nb], delta[nb]};
  // `nblk`: 16-column blocks of the tile (4, or 2 for a wave's own depth tiles); `scored` runs once K and V
  // have been read for the scores (V is not needed after that)
  // `emit(mb, nb, p, ds)`: called with the probabilities and the dS of every 4-column piece (the wave's own depth
  // tiles use it to hand them to the depth-gradient kernel)
  auto tile = [&](auto masked, auto nblk, lds_cptr Kc, lds_cptr Vc, int col0, const int (&lo)[NB], const int (&hi)[NB],
                  auto&& scored, auto&& emit) {
    constexpr bool MASKED = decltype(masked)::value;
    constexpr int MBLK = decltype(nblk)::value;
    f32x4 s[MBLK][NB], dp[MBLK][NB];
    mfma16_rows2<T, HD, MBLK, NB, 2>(oa, Kc, Qr, s, Vc, dOr, dp, dp_init);
    scored();
    TrPipe16<T, HD, MBLK / 2, NB, 3> kt;
    kt.prefetch(oa, Kc);
#pragma unroll
    for (int mb = 0; mb < MBLK; mb++)
#pragma unroll
      for (int nb = 0; nb < NB; nb++) {
        f32x4 pr;
#pragma unroll
        for (int i = 0; i < 4; i++) {
          float p = fast_exp2(__builtin_fmaf(s[mb][nb][i], sc, -lse[nb]));
          if (MASKED) {
            const int c = col0 + 16 * mb + slot_base(q4) + i;
            p = (c >= lo[nb] && c < hi[nb]) ? p : 0.f;
          }
          pr[i] = p;
          s[mb][nb][i] = p * dp[mb][nb][i];
        }
        emit(mb, nb, pr, s[mb][nb]);
      }
    i32x4 DS[MBLK / 2][NB];
#pragma unroll
    for (int ks = 0; ks < MBLK / 2; ks++)
#pragma unroll
      for (int nb = 0; nb < NB; nb++) DS[ks][nb] = pack_slots<T>(s[2 * ks][nb], s[2 * ks + 1][nb]);
    kt.run(oa, Kc, DS, dq);
  };

  int it = 0;
  int none[NB];
#pragma unroll
  for (int nb = 0; nb < NB; nb++) none[nb] = 0;
  const std::integral_constant<int, 4> four{};
  for (; it < n_full; it++) {
    if (it + DIST < ntiles) issue(it + DIST);
    lds_cptr Kc = smem + c_st * 2 * BN * HD;
    tile(std::false_type{}, four, Kc, Kc + BN * HD, it * BN, none, none, []() {}, [](int, int, const f32x4&, const f32x4&) {});
    c_st = (c_st + 1 == NST) ? 0 : c_st + 1;
    wait_tile(it + 1);
    __syncthreads();
  }
  for (; it < ntiles; it++) {
    if (it + DIST < ntiles) issue(it + DIST);
    const bool dep = !NODEPTH && it >= n_seq;
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
      lds_cptr Kc = smem + c_st * 2 * BN * HD;
      tile(std::true_type{}, four, Kc, Kc + BN * HD, col0, lo, hi, []() {}, [](int, int, const f32x4&, const f32x4&) {});
    }
    c_st = (c_st + 1 == NST) ? 0 : c_st + 1;
    wait_tile(it + 1);
    __syncthreads();
  }

  // Outside chunk-visible mode (when a token's rows never straddle waves) the pass over the wave's own depth
  // columns also forms their dK and dV: see the second block below.
  bool fused_depth = false;
  constexpr bool FUSABLE = !NODEPTH && OWN_FITS && HD <= kDepthGradsInDqMaxWidth;
  if constexpr (FUSABLE) fused_depth = depth_grads_in_dq(a, HD);
  if (own_depth && !fused_depth) {
    // The wave's own depth columns, 32 at a time through a wave-private K tile and V tile cut out of the ring
    // (no workgroup barrier after the one that retires the ring).  The next V tile is fetched as soon as the
    // scores are out, the next K tile once dQ has its share.
    __syncthreads();
    typedef WaveTileLoader<HD, DMA_NOP> Own;
    const int wv = __builtin_amdgcn_readfirstlane(wave);
    lds_ptr Kt = smem + wv * (2 * 32 * HD), Vt = Kt + 32 * HD;
    const int rw0 = qt * BM + wv * WR;
    if (rw0 < a.Tq) {
      const DepthSpan span = own_depth_span(a, rw0, WR);
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
      const std::integral_constant<int, 2> two{};
      // where the depth-gradient kernel takes P and dS from here: this lane's rows of the two arrays
      const bool hand_over = a.depth_p != nullptr;
      uint16_t *hp[NB], *hds[NB];
#pragma unroll
      for (int nb = 0; nb < NB; nb++) {
        const int r = rw0 + 16 * nb + n, t = r / a.Gf;  // slot l of row r: element l * Gf + (r - t * Gf) of token t's block
        const int64_t at = (((int64_t)b * a.Hq + hq) * (VARLEN ? a.delta_pitch : a.Tq) + (int64_t)t * a.Gf) * a.Lv + (r - t * a.Gf);
        hp[nb] = a.depth_p + at;
        hds[nb] = a.depth_ds + at;
      }
      for (int j = 0; j < nh; j++) {
        const int col0 = c_beg + 32 * j;
        const bool more = j + 1 < nh;
        Own::template wait_but<0>();
        tile(std::true_type{}, two, Kt, Vt, col0, dlo, dhi,
             [&]() {
               Own::reads_done();
               if (more) fetch(Vt, vdp, a.svd.t, col0 + 32, a.Dv);
             },
             [&](int mb, int nb, const f32x4& p, const f32x4& ds) {
               if (!hand_over) return;
               // rounded as the matrix products take them; slot of column c within its row: c - dlo
               const int w0 = pack2<T>(p[0], p[1]), w1 = pack2<T>(p[2], p[3]);
               const int x0 = pack2<T>(ds[0], ds[1]), x1 = pack2<T>(ds[2], ds[3]);
#pragma unroll
               for (int i = 0; i < 4; i++) {
                 const int c = col0 + 16 * mb + slot_base(q4) + i;
                 if (c >= dlo[nb] && c < dhi[nb]) {
                   const int pw = (i < 2) ? w0 : w1, dw = (i < 2) ? x0 : x1;
                   hp[nb][(c - dlo[nb]) * a.Gf] = (uint16_t)((i & 1) ? ((unsigned)pw >> 16) : ((unsigned)pw & 0xffffu));
                   hds[nb][(c - dlo[nb]) * a.Gf] = (uint16_t)((i & 1) ? ((unsigned)dw >> 16) : ((unsigned)dw & 0xffffu));
                 }
               }
             });
        Own::reads_done();
        if (more) fetch(Kt, kdp, a.skd.t, col0 + 32, a.D);
      }
    }
  }

  // The wave's own depth columns when no other wave sees them (moda_v14.py:1251-1454, fda_v12.py:646-860 for
  // their dK/dV): the products run the other way round here, S = Q Kd^T with the query rows on the accumulator
  // registers (rows 4q + i of each 16-row block) and the depth column on the lane.  P and dS of the wave's 32 rows,
  // rounded and packed, then ARE the operands (summation index = query row) of dVd^T = dO^T P and
  // dKd^T = Q^T dS: one matrix instruction per 16 columns x 16 head-dim elements, nothing to accumulate across
  // tiles.  Q^T and dO^T in that slot order are read once, through the private tiles before the first fetch.
  // dQ needs dS with the columns as summation index: the rounded dS block crosses over through a small LDS block
  // of the wave, which afterwards stages the gradient rows on their way out.
  if constexpr (FUSABLE) {
    if (fused_depth) {
      static_assert(NB == 2, "the wave's 32 query rows are the 32 summation slots of one matrix instruction");
      __syncthreads();
      typedef WaveTileLoader<HD, DMA_NOP> Own;
      const int wv = __builtin_amdgcn_readfirstlane(wave);
      // two sets of a private K tile and V tile (the next tile's rows travel while this one is worked on), then
      // the staging block: 16 rows of HD, or 32 x 32 for the dS block
      lds_ptr Kt = smem + wv * (2 * 32 * HD), Vt = Kt + 32 * HD;
      constexpr int SET = Shape::W * 64 * HD;
      lds_ptr stage = smem + 2 * SET + wv * (16 * HD);
      const int rw0 = qt * BM + wv * WR;
      if (rw0 < a.Tq) {
        // Query row 16*nb + n goes to the tile row its lane reads as a row operand, slot_base(n >> 2) + (n & 3):
        // the transposed read then delivers rows 4q + j and 16 + 4q + j as lane group q's eight summation slots,
        // the order of the packed accumulators.
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
          for (int ks = 0; ks < KS; ks++) {
            *reinterpret_cast<MODA_LDS i32x4*>(Kt + oa.row[ks] + 16 * nb * HD) = Qr[nb][ks];
            *reinterpret_cast<MODA_LDS i32x4*>(Vt + oa.row[ks] + 16 * nb * HD) = dOr[nb][ks];
          }
        Own::reads_done();  // (the counter covers LDS writes as well)
        i32x4 QT[MB], dOT[MB];
#pragma unroll
        for (int mb = 0; mb < MB; mb++) {
          QT[mb] = oa.tr_operand(Kt, 0, mb);
          dOT[mb] = oa.tr_operand(Vt, 0, mb);
        }
        Own::reads_done();
        // per accumulator register: base-2 LSE and minus delta of query row 16*nb + 4*q4 + i, from the lanes that
        // hold those rows (lane n of the first sixteen holds row 16*nb + n; rows past the end carry zeros)
        f32x4 lse4[NB], del4[NB];
        const int rq = rw0 + 4 * q4;
#pragma unroll
        for (int nb = 0; nb < NB; nb++)
#pragma unroll
          for (int i = 0; i < 4; i++) {
            lse4[nb][i] = __shfl(lse[nb], 4 * q4 + i, 64);
            del4[nb][i] = __shfl(delta[nb], 4 * q4 + i, 64);
          }
        const int gshift = __builtin_ctz(a.Gf);  // Gf divides 32: a power of two
        const DepthSpan span = own_depth_span(a, rw0, WR);
        const int c_beg = __builtin_amdgcn_readfirstlane(span.c_beg);
        const int c_end = __builtin_amdgcn_readfirstlane(span.c_end);
        const int nh = (c_end - c_beg + 31) / 32;
        const uint16_t* kdp = a.kd + b * a.skd.b + hkv * a.skd.h;
        const uint16_t* vdp = a.vd + b * a.svd.b + hkv * a.svd.h;
        uint16_t* dkdp = a.dkd + b * a.sdkd.b + hkv * a.sdkd.h;
        uint16_t* dvdp = a.dvd + b * a.sdvd.b + hkv * a.sdvd.h;
        Own own;
        own.init(lane);
        auto fetch = [&](lds_ptr tile, const uint16_t* slice, int64_t stride, int col0, int d) {
          const int nrows = min(32, c_end - col0);
          if (PARTIAL)
            own.fetch_mapped(tile, slice, stride, col0, nrows, (int64_t)a.T * a.L, a.L, a.Lv, d);
          else
            own.fetch(tile, slice, stride, col0, nrows, d);
        };
        const int lrow = slot_base(n >> 2) + (n & 3);  // tile row (of a 16-row block) whose column this lane holds
        // 16 gradient rows (the columns cbase .. cbase + 15) leave through the staging block: the accumulators
        // hold 8-byte pieces of 16 different rows per register, which the memory pipeline would take as 16 partial
        // lines per store; written to LDS and read back by rows, every store covers whole rows.
        constexpr int RPW = Own::RPW, NPASS = 16 / RPW;
        auto stage_put = [&](int mb, const f32x4& x, float mul) {
          i32x2 w;
          w[0] = pack2<T>(x[0] * mul, x[1] * mul);
          w[1] = pack2<T>(x[2] * mul, x[3] * mul);
          *reinterpret_cast<MODA_LDS i32x2*>(stage + Tile<HD>::off(lrow, 2 * mb + (q4 >> 1)) + 4 * (q4 & 1)) = w;
        };
        auto flush = [&](uint16_t* base, int64_t stride, int cbase, int width) {
          Own::reads_done();  // the block is written
#pragma unroll
          for (int i = 0; i < NPASS; i++) {
            const int row = i * RPW + own.prow;
            i32x4 val = *reinterpret_cast<MODA_LDS const i32x4*>(stage + i * 512 + lane * 8);
            const int lch = own.pch ^ Tile<HD>::swz(row);
            const int c = cbase + row;
            if (c < c_end && lch * 8 < width) {
              i32x4* dst = reinterpret_cast<i32x4*>(base + depth_row_of(a, c) * stride + lch * 8);
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
          Own::reads_done();  // the block may be overwritten
        };
        fetch(Kt, kdp, a.skd.t, c_beg, a.D);
        fetch(Vt, vdp, a.svd.t, c_beg, a.Dv);
        MODA_LDS uint16_t* xs = (MODA_LDS uint16_t*)stage;  // dS block: [32 query rows][32 column slots]
        // the gradient rows of one tile's columns from its packed P and dS
        auto gradients = [&](const i32x4 (&PA)[2], const i32x4 (&DSA)[2], int col0) {
          const f32x4 z = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int cb = 0; cb < 2; cb++)
            if (col0 + 16 * cb < c_end) {
#pragma unroll
              for (int mb = 0; mb < MB; mb++) stage_put(mb, mfma16<T>(dOT[mb], PA[cb], z), 1.f);
              flush(dvdp, a.sdvd.t, col0 + 16 * cb, a.Dv);
#pragma unroll
              for (int mb = 0; mb < MB; mb++) stage_put(mb, mfma16<T>(QT[mb], DSA[cb], z), a.scale);
              flush(dkdp, a.sdkd.t, col0 + 16 * cb, a.D);
            }
        };
        // Tile j: wait for its rows, send for tile j + 1 (other set), write out the gradient rows of tile j - 1, then
        // scores, dS and dQ of tile j.  The stores of a tile are thus issued a whole tile before the next wait
        // (the wave's memory counter covers loads and stores alike), the loads one tile ahead of their use.
        i32x4 PA[2], DSA[2];
        for (int j = 0; j < nh; j++) {
          const int col0 = c_beg + 32 * j;
          lds_ptr Kc = Kt + (j & 1) * SET, Vc = Vt + (j & 1) * SET;
          Own::template wait_but<0>();
          if (j + 1 < nh) {
            fetch(Kt + ((j + 1) & 1) * SET, kdp, a.skd.t, col0 + 32, a.D);
            fetch(Vt + ((j + 1) & 1) * SET, vdp, a.svd.t, col0 + 32, a.Dv);
          }
          if (j > 0) gradients(PA, DSA, col0 - 32);
          f32x4 s[2][NB], dp[2][NB];
          mfma16_rows2<T, HD, 2, NB, 2, true>(oa, Kc, Qr, s, Vc, dOr, dp, del4);
#pragma unroll
          for (int cb = 0; cb < 2; cb++) {
            const int c = col0 + 16 * cb + lrow;
            const int tokc = c < c_end ? c / a.Lv : -2;
            f32x4 p[NB], ds[NB];
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
#pragma unroll
              for (int i = 0; i < 4; i++) {
                const int r = rq + 16 * nb + i;
                float pv = fast_exp2(__builtin_fmaf(s[cb][nb][i], sc, -lse4[nb][i]));
                pv = (r < a.Tq && (r >> gshift) == tokc) ? pv : 0.f;
                p[nb][i] = pv;
                ds[nb][i] = pv * dp[cb][nb][i];
              }
            PA[cb] = pack_slots<T>(p[0], p[1]);
            DSA[cb] = pack_slots<T>(ds[0], ds[1]);
            // the rounded dS block to LDS, a query row per 64-byte line, the column of tile row
            // 16*cb + slot_base(g) + j in slot 8g + 4*cb + j: lane group g of the dQ product then reads its eight
            // summation slots (tile rows slot_base(g) + j and 16 + slot_base(g) + j) as one 16-byte piece
            const int slot = 8 * (n >> 2) + 4 * cb + (n & 3);
#pragma unroll
            for (int nb = 0; nb < NB; nb++)
#pragma unroll
              for (int i = 0; i < 4; i++) {
                const int w = DSA[cb][2 * nb + (i >> 1)];
                xs[(16 * nb + 4 * q4 + i) * 32 + slot] = (uint16_t)((i & 1) ? ((unsigned)w >> 16) : ((unsigned)w & 0xffffu));
              }
          }
          Own::reads_done();
          i32x4 DS[1][NB];
#pragma unroll
          for (int nb = 0; nb < NB; nb++) DS[0][nb] = *reinterpret_cast<MODA_LDS const i32x4*>(xs + (16 * nb + n) * 32 + 8 * q4);
          TrPipe16<T, HD, 1, NB, 3> kt;
          kt.prefetch(oa, Kc);
          kt.run(oa, Kc, DS, dq);
          Own::reads_done();  // this set and the staging block are free again
        }
        if (nh > 0) gradients(PA, DSA, c_beg + 32 * (nh - 1));
      }
    }
  }

#pragma unroll
  for (int nb = 0; nb < NB; nb++) {
    const int r = qt * BM + wave * WR + 16 * nb + n;
    if (r < a.Tq) {
      uint16_t* op = a.dq + b * a.sdq.b + hq * a.sdq.h + (int64_t)r * a.sdq.t;
#pragma unroll
      for (int d = 0; d < MB; d++) {
        i32x2 w;
        w[0] = pack2<T>(dq[d][nb][0] * a.scale, dq[d][nb][1] * a.scale);
        w[1] = pack2<T>(dq[d][nb][2] * a.scale, dq[d][nb][3] * a.scale);
        if (16 * d + 4 * q4 < a.D) {
          i32x2* dst = reinterpret_cast<i32x2*>(op + 16 * d + 4 * q4);
          // the narrow tiles serve HBM-bound shapes whose depth stream can stay in the memory-side cache between
          // launches if results written once do not displace it
          if (HD <= 64)
            __builtin_nontemporal_store(w, dst);
          else
            *dst = w;
        }
      }
    }
  }
}

template <typename T, int HD>
hipError_t launch_delta_t(const KArgs& a, hipStream_t stream) {
  if (a.Tq == 0 || a.B * a.Hq == 0) return hipSuccess;
  constexpr int RPB = 256 / (HD / 8);
  const int64_t nblk = delta_kernel_blocks(a, RPB);
  if (nblk >= (1ll << 31)) return hipErrorInvalidValue;
  hipLaunchKernelGGL((delta_kernel<T, HD>), dim3((unsigned)nblk), dim3(256), 0, stream, a);
  return hipGetLastError();
}

template <typename T, int HD, typename Shape, int ADDR>
hipError_t launch_dq_t_shape(const KArgs& a, hipStream_t stream) {
  // the ring, or one 32-column K tile and V tile per wave for the waves' own depth columns
  // ... and, where the kernel forms the depth gradients, a second set of those and a 16-row block per wave through
  // which the gradients leave
  constexpr size_t ring = (size_t)Shape::NST * 2 * 64 * HD * sizeof(uint16_t),
                   own = (size_t)Shape::W * (HD <= kDepthGradsInDqMaxWidth ? 2 * 64 + 16 : 64) * HD * sizeof(uint16_t);
  constexpr size_t smem = (size_t)Shape::W * 64 * HD * sizeof(uint16_t) <= 128 * 1024 ? std::max(ring, own) : ring;
  static LdsAttrState attr;
  const hipError_t ea = allow_dynamic_lds(attr, reinterpret_cast<const void*>(&dq_kernel<T, HD, Shape, ADDR>), smem);
  if (ea != hipSuccess) return ea;
  constexpr int rows = 16 * Shape::NB * Shape::W;
  const int64_t nblk = row_kernel_blocks(a, rows);
  if (nblk == 0) return hipSuccess;
  if (nblk >= (1ll << 31)) return hipErrorInvalidValue;
  hipLaunchKernelGGL((dq_kernel<T, HD, Shape, ADDR>), dim3((unsigned)nblk), dim3(64 * Shape::W), smem, stream, a);
  return hipGetLastError();
}

template <typename T, int HD, int ADDR>
hipError_t launch_dq_t_addr(const KArgs& a, bool small, hipStream_t stream) {
  if constexpr (HD > 128) return launch_dq_t_shape<T, HD, RowWide, ADDR>(a, stream);  // one shape for the wide tiles
  else {
    if (ADDR & 1) return launch_dq_t_shape<T, HD, RowLarge, ADDR>(a, stream);  // slices wider than 2 GiB: never a small launch
    if (small) return launch_dq_t_shape<T, HD, RowSmall<HD>, ADDR>(a, stream);
    return launch_dq_t_shape<T, HD, RowLarge, ADDR>(a, stream);
  }
}

template <typename T, int HD>
hipError_t launch_dq_t(const KArgs& a, hipStream_t stream) {
  // byte span of the widest streamed (batch, head) slice
  const int64_t span = 2 * std::max(std::max((int64_t)a.T * a.sk.t, (int64_t)a.T * a.sv.t),
                                    std::max((int64_t)a.T * a.L * a.skd.t, (int64_t)a.T * a.L * a.svd.t));
  const bool wide = span > 0x7fffffffll;
  const bool small = use_small_rows(a.Tq, (long long)a.B * a.Hq, a.compute_units);
  switch ((wide ? 1 : 0) | (a.cu ? 2 : 0) | (a.L == 0 ? 4 : 0) | (a.L > 0 && a.Lv != a.L ? 8 : 0)) {
    case 0: return launch_dq_t_addr<T, HD, 0>(a, small, stream);
    case 1: return launch_dq_t_addr<T, HD, 1>(a, small, stream);
    case 2: return launch_dq_t_addr<T, HD, 2>(a, small, stream);
    case 3: return launch_dq_t_addr<T, HD, 3>(a, small, stream);
    case 4: return launch_dq_t_addr<T, HD, 4>(a, small, stream);
    case 5: return launch_dq_t_addr<T, HD, 5>(a, small, stream);
    case 6: return launch_dq_t_addr<T, HD, 6>(a, small, stream);
    case 7: return launch_dq_t_addr<T, HD, 7>(a, small, stream);
    case 8: return launch_dq_t_addr<T, HD, 8>(a, small, stream);
    case 9: return launch_dq_t_addr<T, HD, 9>(a, small, stream);
    case 10: return launch_dq_t_addr<T, HD, 10>(a, small, stream);
    default: return launch_dq_t_addr<T, HD, 11>(a, small, stream);
  }
}

hipError_t launch_delta(const KArgs& a, int dtype, int hd, hipStream_t stream) {
  if (dtype == 0 && hd == 128) return launch_delta_t<BF16, 128>(a, stream);
  if (dtype == 0 && hd == 64) return launch_delta_t<BF16, 64>(a, stream);
  if (dtype == 1 && hd == 128) return launch_delta_t<FP16, 128>(a, stream);
  if (dtype == 1 && hd == 64) return launch_delta_t<FP16, 64>(a, stream);
  if (dtype == 0 && hd == 256) return launch_delta_t<BF16, 256>(a, stream);
  if (dtype == 1 && hd == 256) return launch_delta_t<FP16, 256>(a, stream);
  return hipErrorInvalidValue;
}

hipError_t launch_dq(const KArgs& a, int dtype, int hd, hipStream_t stream) {
  if (dtype == 0 && hd == 128) return launch_dq_t<BF16, 128>(a, stream);
  if (dtype == 0 && hd == 64) return launch_dq_t<BF16, 64>(a, stream);
  if (dtype == 1 && hd == 128) return launch_dq_t<FP16, 128>(a, stream);
  if (dtype == 1 && hd == 64) return launch_dq_t<FP16, 64>(a, stream);
  if (dtype == 0 && hd == 256) return launch_dq_t<BF16, 256>(a, stream);
  if (dtype == 1 && hd == 256) return launch_dq_t<FP16, 256>(a, stream);
  return hipErrorInvalidValue;
}

}  // namespace moda
