// Backward, query side: the preprocess kernel (-delta = -rowsum(o * do), moda_v14.py:525-539) and the
// dQ kernel (moda_v14.py:542-871, moda_v16.py:936-1220, fda_v12.py:432-638,
// fla/ops/attn/parallel.py:165-296).
//
// Same decomposition as the forward kernel: a workgroup owns 32 query rows per wave
// (256 in the throughput launch shape, 64 or 128 in the small one),
// one row per lane pair, and streams 64-column K/V tiles (sequence keys, then
// the rows' depth slots).  P^T is recomputed from the saved base-2 LSE,
// dS^T = P^T * (dP^T - delta) is packed straight into the B operand of
// dQ^T += K^T * dS^T, K^T coming from the LDS transpose read of the K tile.
#include <algorithm>
#include <type_traits>

#include "kargs.h"
#include "tile.h"
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
  if (r < a.Tq && c < a.D) {
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
// offsets inside the slice); bit 1: packed variable-length batch
template <typename T, int HD, typename Shape, int ADDR>
__global__ __launch_bounds__(64 * Shape::W, 2) void dq_kernel(const KArgs a_in) {
  constexpr int BM = 32 * Shape::W, BN = 64, KK = HD / 16, DB = HD / 32, NT = 64 * Shape::W, NST = Shape::NST, DIST = Shape::DIST;
  static_assert(NST >= DIST + 1 && DIST >= 1 && DIST <= 2, "ring must hold the tile in use plus the tiles in flight");
  extern __shared__ __align__(16) unsigned char smem_raw[];
  lds_ptr smem = (lds_ptr)smem_raw;
  // ring stage st: K tile at smem + st * 2*BN*HD, V tile right behind it

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n = lane & 31, g = lane >> 5;
  constexpr bool WIDE = (ADDR & 1) != 0, VARLEN = (ADDR & 2) != 0;
  const int BH = a_in.B * a_in.Hq;
  const int bh = blockIdx.x % BH;
  int b = bh / a_in.Hq;
  const int hq = bh % a_in.Hq, hkv = hq / a_in.hdiv;
  SeqArgs<VARLEN> seq(a_in, b);
  const KArgs& a = seq.a;
  const int nqt = (a.Tq + BM - 1) / BM;
  // Heavy (late) tiles first.  In a variable-length batch the grid counts tiles from the end of the longest
  // sequence, so that tiles of equal cost (equal row position) of all sequences are dispatched together and the
  // heaviest of the whole batch first; the positions a shorter sequence does not have are dropped.
  const int qt = (VARLEN ? (a_in.Tq + BM - 1) / BM : nqt) - 1 - blockIdx.x / BH;
  if (VARLEN && qt >= nqt) return;
  const int r = qt * BM + wave * 32 + n;
  const bool valid = r < a.Tq;
  const int t = r / a.Gf;

  i32x4 Qr[KK], dOr[KK];
  float lse = 0.f, delta = 0.f;
  {
    const uint16_t* qp = a.q + b * a.sq.b + hq * a.sq.h + (int64_t)r * a.sq.t + 8 * g;
    const uint16_t* dop = a.d_o + b * a.sdo.b + hq * a.sdo.h + (int64_t)r * a.sdo.t + 8 * g;
#pragma unroll
    for (int kk = 0; kk < KK; kk++) {
      i32x4 z = {0, 0, 0, 0};
      const bool in = valid && 16 * kk + 8 * g < a.D;
      Qr[kk] = in ? *reinterpret_cast<const i32x4*>(qp + 16 * kk) : z;
      dOr[kk] = in ? *reinterpret_cast<const i32x4*>(dop + 16 * kk) : z;
    }
    if (valid) {
      lse = a.lse[((int64_t)b * a.Tq + r) * a.Hq + hq];
      delta = a.delta[((int64_t)b * a.Hq + hq) * (VARLEN ? a.delta_pitch : a.Tq) + r];
    }
  }

  // The register operands above must have arrived before the tile loads start: those are issued
  // behind the compiler's back, and a load it still believes pending would cost a vmcnt(0) in every
  // trip of the main loop.
  asm volatile("" ::: "memory");  // keep the loads above this point
  __builtin_amdgcn_s_waitcnt(0x0F70);
  asm volatile("" ::: "memory");

  int shi = 0, dlo = 0, dhi = 0;
  if (valid) {
    if (a.has_seq) shi = a.causal ? t + 1 : a.T;
    if (a.L > 0) {
      const int lo_t = a.chunk ? (t / a.Cb) * a.Cb : t;
      dlo = lo_t * a.L;
      dhi = a.chunk ? (t + 1) * a.L : dlo + a.Lv;  // the token's filled slots
    }
  }
  const int r_first = qt * BM;
  const int r_last = min(a.Tq, r_first + BM) - 1;
  const int t_first = r_first / a.Gf, t_last = r_last / a.Gf;
  int n_seq = 0, n_full = 0;
  if (a.has_seq) {
    n_seq = ((a.causal ? t_last + 1 : a.T) + BN - 1) / BN;
    // leading sequence tiles every row of the workgroup sees completely (padding rows of the last
    // workgroup carry zero queries and zero dO there and are never stored)
    n_full = min(n_seq, (a.causal ? t_first + 1 : a.T) / BN);
  }
  int dep0 = 0, n_dep = 0;
  if (a.L > 0) {
    const int lo_t = a.chunk ? (t_first / a.Cb) * a.Cb : t_first;
    dep0 = lo_t * a.L;
    n_dep = ((t_last + 1) * a.L - dep0 + BN - 1) / BN;
  }
  // wave-uniform by construction, but computed with vector divisions: the explicit hint keeps the
  // loop control in scalar registers
  n_seq = __builtin_amdgcn_readfirstlane(n_seq);
  n_full = __builtin_amdgcn_readfirstlane(n_full);
  dep0 = __builtin_amdgcn_readfirstlane(dep0);
  const int ntiles = __builtin_amdgcn_readfirstlane(n_seq + n_dep);

  typedef AsyncTileLoader<HD, BN, NT> Loader;
  constexpr int LPT = 2 * Loader::N;  // vector-memory loads one wave issues per tile (K + V)
  Loader ld;
  ld.init(tid, a.D);
  // the two sources being streamed: sequence K/V first, swapped for the depth K/V when the
  // producer reaches the first depth tile
  typename Loader::Source srcK, srcV;
  if (a.has_seq && n_seq > 0) {
    srcK = ld.source(a.k + b * a.sk.b + hkv * a.sk.h, a.sk.t, 0, a.T);
    srcV = ld.source(a.v + b * a.sv.b + hkv * a.sv.h, a.sv.t, 0, a.T);
  }
  int ld_st = 0;  // ring stage the next issued tile goes to
  auto issue = [&](int it) {
    lds_ptr Kt = smem + ld_st * 2 * BN * HD;
    if (it == n_seq) {
      srcK = ld.source(a.kd + b * a.skd.b + hkv * a.skd.h, a.skd.t, dep0, a.T * a.L);
      srcV = ld.source(a.vd + b * a.svd.b + hkv * a.svd.h, a.svd.t, dep0, a.T * a.L);
    }
    const int row0 = it < n_seq ? it * BN : dep0 + (it - n_seq) * BN;
    if (WIDE) {  // some slice spans more than 2 GiB: a descriptor anchored at this tile
      const bool dep = it >= n_seq;
      const int row_end = dep ? a.T * a.L : a.T;
      ld.load(Kt, dep ? a.kd + b * a.skd.b + hkv * a.skd.h : a.k + b * a.sk.b + hkv * a.sk.h, dep ? a.skd.t : a.sk.t,
              row0, row_end);
      ld.load(Kt + BN * HD, dep ? a.vd + b * a.svd.b + hkv * a.svd.h : a.v + b * a.sv.b + hkv * a.sv.h,
              dep ? a.svd.t : a.sv.t, row0, row_end);
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

  f32x16 dq[DB];
#pragma unroll
  for (int d = 0; d < DB; d++)
#pragma unroll
    for (int i = 0; i < 16; i++) dq[d][i] = 0.f;
  const float sc = a.scale * kLog2e;
  OperandAddr<HD> oa;
  oa.init(lane);

#pragma unroll
  for (int j = 0; j < DIST; j++)
    if (j < ntiles) issue(j);
  wait_tile(0);
  __syncthreads();
  int c_st = 0;  // ring stage of the tile being consumed

  // start value of every dP^T accumulator block: this lane's row constant -rowsum(o * do), so that the
  // subtraction costs no instruction per element
  f32x16 dp_init;
#pragma unroll
  for (int i = 0; i < 16; i++) dp_init[i] = delta;
  // one column tile: S^T = K Q^T and dP^T = V dO^T in one MFMA pipeline, dS^T, dQ^T += K^T dS^T
  auto tile = [&](auto masked, lds_cptr Kc, lds_cptr Vc, int col0, int lo, int hi) {
    constexpr bool MASKED = decltype(masked)::value;
    f32x16 s[2], dp[2];
    mfma_rows2<T, HD, 2, 4>(oa, Kc, Qr, s, Vc, dOr, dp, dp_init);
    TrPipe<T, HD, 4, 2> kt;
    kt.prefetch(oa, Kc);
#pragma unroll
    for (int bb = 0; bb < 2; bb++)
#pragma unroll
      for (int i = 0; i < 16; i++) {
        float p = fast_exp2(__builtin_fmaf(s[bb][i], sc, -lse));
        if (MASKED) {
          const int c = col0 + 32 * bb + acc_row(i, g);
          p = (c >= lo && c < hi) ? p : 0.f;
        }
        s[bb][i] = p * dp[bb][i];  // dp started from minus rowsum(o * do)
      }
    i32x4 DS[4];
#pragma unroll
    for (int ks = 0; ks < 4; ks++) DS[ks] = pack8<T>(s[ks >> 1], (ks & 1) * 8);
    kt.run(oa, Kc, DS, dq);
  };

  // phase 1: tiles fully visible to every row -- no masks, no visibility tests.  (Not unrolled over the
  // ring stages like the forward loop: this kernel has no registers left for a second set of operand
  // addresses.)
  int it = 0;
  for (; it < n_full; it++) {
    if (it + DIST < ntiles) issue(it + DIST);
    lds_cptr Kc = smem + c_st * 2 * BN * HD;
    tile(std::false_type{}, Kc, Kc + BN * HD, it * BN, 0, 0);
    c_st = (c_st + 1 == NST) ? 0 : c_st + 1;
    wait_tile(it + 1);
    __syncthreads();
  }
  // phase 2: boundary sequence tiles and depth tiles
  for (; it < ntiles; it++) {
    if (it + DIST < ntiles) issue(it + DIST);
    const bool dep = it >= n_seq;
    const int col0 = dep ? dep0 + (it - n_seq) * BN : it * BN;
    const int lo = dep ? dlo : 0;
    const int hi = dep ? dhi : shi;
    const bool touches = (hi > col0) && (lo < col0 + BN) && (hi > lo);
    if (__any(touches)) {
      lds_cptr Kc = smem + c_st * 2 * BN * HD;
      tile(std::true_type{}, Kc, Kc + BN * HD, col0, lo, hi);
    }
    c_st = (c_st + 1 == NST) ? 0 : c_st + 1;
    wait_tile(it + 1);
    __syncthreads();
  }

  if (valid) {
    uint16_t* op = a.dq + b * a.sdq.b + hq * a.sdq.h + (int64_t)r * a.sdq.t;
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        i32x2 w;
        w[0] = pack2<T>(dq[d][4 * i4 + 0] * a.scale, dq[d][4 * i4 + 1] * a.scale);
        w[1] = pack2<T>(dq[d][4 * i4 + 2] * a.scale, dq[d][4 * i4 + 3] * a.scale);
        if (32 * d + 8 * i4 + 4 * g < a.D) *reinterpret_cast<i32x2*>(op + 32 * d + 8 * i4 + 4 * g) = w;
      }
  }
}

template <typename T, int HD>
hipError_t launch_delta_t(const KArgs& a, hipStream_t stream) {
  if (a.Tq == 0 || a.B * a.Hq == 0) return hipSuccess;
  constexpr int RPB = 256 / (HD / 8);
  const int64_t nblk = (int64_t)((a.Tq + RPB - 1) / RPB) * a.B * a.Hq;
  if (nblk >= (1ll << 31)) return hipErrorInvalidValue;
  hipLaunchKernelGGL((delta_kernel<T, HD>), dim3((unsigned)nblk), dim3(256), 0, stream, a);
  return hipGetLastError();
}

template <typename T, int HD, typename Shape, int ADDR>
hipError_t launch_dq_t_shape(const KArgs& a, hipStream_t stream) {
  constexpr size_t smem = (size_t)Shape::NST * 2 * 64 * HD * sizeof(uint16_t);
  static LdsAttrState attr;
  const hipError_t ea = allow_dynamic_lds(attr, reinterpret_cast<const void*>(&dq_kernel<T, HD, Shape, ADDR>), smem);
  if (ea != hipSuccess) return ea;
  const int64_t nblk = (int64_t)((a.Tq + 32 * Shape::W - 1) / (32 * Shape::W)) * a.B * a.Hq;
  if (nblk == 0) return hipSuccess;
  if (nblk >= (1ll << 31)) return hipErrorInvalidValue;
  hipLaunchKernelGGL((dq_kernel<T, HD, Shape, ADDR>), dim3((unsigned)nblk), dim3(64 * Shape::W), smem, stream, a);
  return hipGetLastError();
}

template <typename T, int HD>
hipError_t launch_dq_t(const KArgs& a, hipStream_t stream) {
  // byte span of the widest streamed (batch, head) slice
  const int64_t span = 2 * std::max(std::max((int64_t)a.T * a.sk.t, (int64_t)a.T * a.sv.t),
                                    std::max((int64_t)a.T * a.L * a.skd.t, (int64_t)a.T * a.L * a.svd.t));
  const bool wide = span > 0x7fffffffll;
  const bool small = use_small_rows(a.Tq, (long long)a.B * a.Hq, a.compute_units);
  if (a.cu) {
    if (wide) return launch_dq_t_shape<T, HD, RowLarge, 3>(a, stream);
    if (small) return launch_dq_t_shape<T, HD, RowSmall<HD>, 2>(a, stream);
    return launch_dq_t_shape<T, HD, RowLarge, 2>(a, stream);
  }
  if (wide) return launch_dq_t_shape<T, HD, RowLarge, 1>(a, stream);
  if (small) return launch_dq_t_shape<T, HD, RowSmall<HD>, 0>(a, stream);
  return launch_dq_t_shape<T, HD, RowLarge, 0>(a, stream);
}

template __global__ void dq_kernel<BF16, 128, RowLarge, 0>(const KArgs);
template __global__ void dq_kernel<BF16, 64, RowLarge, 0>(const KArgs);
template __global__ void dq_kernel<FP16, 128, RowLarge, 0>(const KArgs);
template __global__ void dq_kernel<FP16, 64, RowLarge, 0>(const KArgs);
template __global__ void dq_kernel<BF16, 128, RowLarge, 1>(const KArgs);
template __global__ void dq_kernel<BF16, 64, RowLarge, 1>(const KArgs);
template __global__ void dq_kernel<FP16, 128, RowLarge, 1>(const KArgs);
template __global__ void dq_kernel<FP16, 64, RowLarge, 1>(const KArgs);
template __global__ void dq_kernel<BF16, 128, RowSmall<128>, 0>(const KArgs);
template __global__ void dq_kernel<BF16, 64, RowSmall<64>, 0>(const KArgs);
template __global__ void dq_kernel<FP16, 128, RowSmall<128>, 0>(const KArgs);
template __global__ void dq_kernel<FP16, 64, RowSmall<64>, 0>(const KArgs);
template __global__ void dq_kernel<BF16, 128, RowLarge, 2>(const KArgs);
template __global__ void dq_kernel<BF16, 128, RowLarge, 3>(const KArgs);
template __global__ void dq_kernel<BF16, 128, RowSmall<128>, 2>(const KArgs);
template __global__ void dq_kernel<BF16, 64, RowLarge, 2>(const KArgs);
template __global__ void dq_kernel<BF16, 64, RowLarge, 3>(const KArgs);
template __global__ void dq_kernel<BF16, 64, RowSmall<64>, 2>(const KArgs);
template __global__ void dq_kernel<FP16, 128, RowLarge, 2>(const KArgs);
template __global__ void dq_kernel<FP16, 128, RowLarge, 3>(const KArgs);
template __global__ void dq_kernel<FP16, 128, RowSmall<128>, 2>(const KArgs);
template __global__ void dq_kernel<FP16, 64, RowLarge, 2>(const KArgs);
template __global__ void dq_kernel<FP16, 64, RowLarge, 3>(const KArgs);
template __global__ void dq_kernel<FP16, 64, RowSmall<64>, 2>(const KArgs);

hipError_t launch_delta(const KArgs& a, int dtype, int hd, hipStream_t stream) {
  if (dtype == 0 && hd == 128) return launch_delta_t<BF16, 128>(a, stream);
  if (dtype == 0 && hd == 64) return launch_delta_t<BF16, 64>(a, stream);
  if (dtype == 1 && hd == 128) return launch_delta_t<FP16, 128>(a, stream);
  if (dtype == 1 && hd == 64) return launch_delta_t<FP16, 64>(a, stream);
  return hipErrorInvalidValue;
}

hipError_t launch_dq(const KArgs& a, int dtype, int hd, hipStream_t stream) {
  if (dtype == 0 && hd == 128) return launch_dq_t<BF16, 128>(a, stream);
  if (dtype == 0 && hd == 64) return launch_dq_t<BF16, 64>(a, stream);
  if (dtype == 1 && hd == 128) return launch_dq_t<FP16, 128>(a, stream);
  if (dtype == 1 && hd == 64) return launch_dq_t<FP16, 64>(a, stream);
  return hipErrorInvalidValue;
}

}  // namespace moda
