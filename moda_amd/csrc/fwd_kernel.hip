// Forward kernel: one online softmax over the visible sequence keys and the
// query's depth-KV slots (the computation of moda_v14.py:45-378,
// moda_v16.py:39-352, fda_v12.py:44-253 and fla/ops/attn/parallel.py:18-143).
//
// Work split: one workgroup = 128 query rows of one (batch, query head), four
// 64-lane waves of 32 rows each.  Scores are produced transposed,
// S^T = K * Q^T, so each lane owns ONE query row: row statistics need a single
// cross-lane exchange and P^T is already laid out as the B operand of
// O^T += V^T * P^T.  K and V tiles (64 columns) are staged through LDS, V is
// read with the LDS transpose load.  Depth columns are extra column tiles with
// a different per-row visible interval.
#include "kargs.h"
#include "tile.h"

namespace moda {

template <typename T, int HD>
__global__ __launch_bounds__(256, 2) void fwd_kernel(const KArgs a) {
  constexpr int BM = 128, BN = 64, KK = HD / 16, DB = HD / 32;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  lds_ptr smem = (lds_ptr)smem_raw;
  lds_ptr Ks[2] = {smem, smem + BN * HD};
  lds_ptr Vs[2] = {smem + 2 * BN * HD, smem + 3 * BN * HD};

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n = lane & 31, g = lane >> 5;
  const int BH = a.B * a.Hq;
  const int bh = blockIdx.x % BH;
  const int qt = a.nqt - 1 - blockIdx.x / BH;  // heavy (late) tiles first
  const int b = bh / a.Hq, hq = bh % a.Hq, hkv = hq / a.hdiv;
  const int r = qt * BM + wave * 32 + n;
  const bool valid = r < a.Tq;
  const int t = r / a.Gf;

  i32x4 Qr[KK];
  {
    const uint16_t* qp = a.q + b * a.sq.b + hq * a.sq.h + (int64_t)r * a.sq.t + 8 * g;
#pragma unroll
    for (int kk = 0; kk < KK; kk++) {
      i32x4 z = {0, 0, 0, 0};
      Qr[kk] = valid ? *reinterpret_cast<const i32x4*>(qp + 16 * kk) : z;
    }
  }

  // per-row visible column intervals [lo, hi) for the two phases
  int shi = 0, dlo = 0, dhi = 0;
  if (valid) {
    if (a.has_seq) shi = a.causal ? t + 1 : a.T;
    if (a.L > 0) {
      const int lo_t = a.chunk ? (t / a.Cb) * a.Cb : t;
      dlo = lo_t * a.L;
      dhi = (t + 1) * a.L;
    }
  }
  // workgroup column ranges
  const int r_first = qt * BM;
  const int r_last = min(a.Tq, r_first + BM) - 1;
  const int t_first = r_first / a.Gf, t_last = r_last / a.Gf;
  int n_seq = 0;
  if (a.has_seq) n_seq = ((a.causal ? t_last + 1 : a.T) + BN - 1) / BN;
  int dep0 = 0, n_dep = 0;
  if (a.L > 0) {
    const int lo_t = a.chunk ? (t_first / a.Cb) * a.Cb : t_first;
    dep0 = lo_t * a.L;
    n_dep = ((t_last + 1) * a.L - dep0 + BN - 1) / BN;
  }
  const int ntiles = n_seq + n_dep;

  const uint16_t* kb = a.has_seq ? a.k + b * a.sk.b + hkv * a.sk.h : nullptr;
  const uint16_t* vb = a.has_seq ? a.v + b * a.sv.b + hkv * a.sv.h : nullptr;
  const uint16_t* kdb = a.L > 0 ? a.kd + b * a.skd.b + hkv * a.skd.h : nullptr;
  const uint16_t* vdb = a.L > 0 ? a.vd + b * a.svd.b + hkv * a.svd.h : nullptr;
  const int TL = a.T * a.L;

  AsyncTileLoader<HD, BN, 256> ld;
  ld.init(tid);
  auto issue = [&](int it) {
    const int st = it & 1;
    if (it < n_seq) {
      ld.load(Ks[st], kb, a.sk.t, it * BN, a.T);
      ld.load(Vs[st], vb, a.sv.t, it * BN, a.T);
    } else {
      const int c0 = dep0 + (it - n_seq) * BN;
      ld.load(Ks[st], kdb, a.skd.t, c0, TL);
      ld.load(Vs[st], vdb, a.svd.t, c0, TL);
    }
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

  if (ntiles > 0) issue(0);
  ld.wait_all();
  __syncthreads();

  for (int it = 0; it < ntiles; it++) {
    const int cur = it & 1;
    if (it + 1 < ntiles) issue(it + 1);

    const bool dep = it >= n_seq;
    const int col0 = dep ? dep0 + (it - n_seq) * BN : it * BN;
    const int lo = dep ? dlo : 0;
    const int hi = dep ? dhi : shi;
    const bool touches = (hi > col0) && (lo < col0 + BN) && (hi > lo);
    if (__any(touches)) {
      const bool full = (lo <= col0) && (hi >= col0 + BN);
      const bool need_mask = !__all(full);
      f32x16 s[2];
      mfma_rows<T, HD, 2, 4>(oa, Ks[cur], Qr, s);
      // first V^T operands start travelling while the softmax runs
      TrPipe<T, HD, 4, 4> pv;
      pv.prefetch(oa, Vs[cur]);
      // row maximum of the raw scores (scale > 0, so it commutes with the max)
      float mx = kNegInf;
      if (need_mask) {
#pragma unroll
        for (int bb = 0; bb < 2; bb++)
#pragma unroll
          for (int i = 0; i < 16; i++) {
            const int c = col0 + 32 * bb + acc_row(i, g);
            mx = fmaxf(mx, (c >= lo && c < hi) ? s[bb][i] : kNegInf);
          }
      } else {
#pragma unroll
        for (int bb = 0; bb < 2; bb++)
#pragma unroll
          for (int i = 0; i < 16; i++) mx = fmaxf(mx, s[bb][i]);
      }
      mx = fmaxf(mx, xor32(mx)) * sc;
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
      float rs = 0.f;
      i32x4 P[4];
      if (need_mask) {
#pragma unroll
        for (int bb = 0; bb < 2; bb++)
#pragma unroll
          for (int i = 0; i < 16; i++) {
            const int c = col0 + 32 * bb + acc_row(i, g);
            const float p = (c >= lo && c < hi) ? fast_exp2(__builtin_fmaf(s[bb][i], sc, neg_m)) : 0.f;
            s[bb][i] = p;
            rs += p;
          }
      } else {
#pragma unroll
        for (int bb = 0; bb < 2; bb++)
#pragma unroll
          for (int i = 0; i < 16; i++) {
            const float p = fast_exp2(__builtin_fmaf(s[bb][i], sc, neg_m));
            s[bb][i] = p;
            rs += p;
          }
      }
#pragma unroll
      for (int ks = 0; ks < 4; ks++) P[ks] = pack8<T>(s[ks >> 1], (ks & 1) * 8);
      rs += xor32(rs);
      l += rs;
      pv.run(oa, Vs[cur], P, o);
    }

    ld.wait_all();
    __syncthreads();
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
        *reinterpret_cast<i32x2*>(op + 32 * d + 8 * i4 + 4 * g) = w;
      }
    if (g == 0) a.lse[((int64_t)b * a.Tq + r) * a.Hq + hq] = (l > 0.f) ? m + log2f(l) : kNegInf;
  }
}

template <typename T, int HD>
hipError_t launch_fwd_t(const KArgs& a, hipStream_t stream) {
  constexpr size_t smem = 4 * 64 * HD * sizeof(uint16_t);
  static bool attr_done = false;
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&fwd_kernel<T, HD>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
    attr_done = true;
  }
  const int64_t nblk = (int64_t)a.nqt * a.B * a.Hq;
  if (nblk == 0) return hipSuccess;
  hipLaunchKernelGGL((fwd_kernel<T, HD>), dim3((unsigned)nblk), dim3(256), smem, stream, a);
  return hipGetLastError();
}

hipError_t launch_fwd(const KArgs& a, int dtype, int hd, hipStream_t stream) {
  if (dtype == 0 && hd == 128) return launch_fwd_t<BF16, 128>(a, stream);
  if (dtype == 0 && hd == 64) return launch_fwd_t<BF16, 64>(a, stream);
  if (dtype == 1 && hd == 128) return launch_fwd_t<FP16, 128>(a, stream);
  if (dtype == 1 && hd == 64) return launch_fwd_t<FP16, 64>(a, stream);
  return hipErrorInvalidValue;
}

}  // namespace moda
