// Backward, key side: dK/dV of the sequence stream and of the depth stream
// (moda_v14.py:874-1248 and :1251-1454, moda_v16.py:1223-1425 and :1632-1834,
// fda_v12.py:646-860, fla/ops/attn/parallel.py:299-440).
//
// A workgroup owns 128 key columns of one (batch, kv head) -- sequence keys or
// flattened depth slots -- one column per lane pair, K and V rows held in
// registers as MFMA B operands.  It streams 64-row query tiles (Q, dO, LSE,
// delta) through LDS over exactly the query rows that can see its columns:
// all later tokens for a causal sequence key, the owner token's G rows (or the
// rest of its chunk) for a depth slot.  All G folded rows, and in head-dim GQA
// all G query heads, are reduced in registers, so every output row has one
// writer and no atomics or partial buffers are needed.
#include "kargs.h"
#include "tile.h"

namespace moda {

template <typename T, int HD>
__global__ __launch_bounds__(256) void dkv_kernel(const KArgs a) {
  constexpr int BN = 128, BM = 64, KK = HD / 16, DB = HD / 32;
  extern __shared__ __align__(16) unsigned char smem_raw[];
  lds_ptr smem = (lds_ptr)smem_raw;
  lds_ptr Qs[2] = {smem, smem + BM * HD};
  lds_ptr dOs[2] = {smem + 2 * BM * HD, smem + 3 * BM * HD};
  MODA_LDS float* stat = (MODA_LDS float*)(smem + 4 * BM * HD);  // [2][2][BM]: lse, delta per stage

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, n = lane & 31, g = lane >> 5;
  const int BHk = a.B * a.Hkv;
  const int bh = blockIdx.x % BHk;
  const int ct = blockIdx.x / BHk;
  const int b = bh / a.Hkv, hkv = bh % a.Hkv;
  const int n_seq_tiles = a.has_seq ? (a.T + BN - 1) / BN : 0;
  const bool dep = ct >= n_seq_tiles;
  const int ncols = dep ? a.T * a.L : a.T;
  const int c_first = (dep ? ct - n_seq_tiles : ct) * BN;
  const int c = c_first + wave * 32 + n;
  const bool valid = c < ncols;

  const uint16_t* ksrc = dep ? a.kd + b * a.skd.b + hkv * a.skd.h : a.k + b * a.sk.b + hkv * a.sk.h;
  const uint16_t* vsrc = dep ? a.vd + b * a.svd.b + hkv * a.svd.h : a.v + b * a.sv.b + hkv * a.sv.h;
  const int64_t kst = dep ? a.skd.t : a.sk.t, vst = dep ? a.svd.t : a.sv.t;
  i32x4 Kr[KK], Vr[KK];
#pragma unroll
  for (int kk = 0; kk < KK; kk++) {
    i32x4 z = {0, 0, 0, 0};
    Kr[kk] = valid ? *reinterpret_cast<const i32x4*>(ksrc + (int64_t)c * kst + 16 * kk + 8 * g) : z;
    Vr[kk] = valid ? *reinterpret_cast<const i32x4*>(vsrc + (int64_t)c * vst + 16 * kk + 8 * g) : z;
  }

  // visible query-row interval of a column
  auto q_interval = [&](int col, int& lo, int& hi) {
    if (!dep) {
      lo = a.causal ? col * a.Gf : 0;
      hi = a.Tq;
    } else {
      const int w = col / a.L;
      lo = w * a.Gf;
      hi = a.chunk ? min(a.T, (w / a.Cb + 1) * a.Cb) * a.Gf : (w + 1) * a.Gf;
    }
  };
  int qlo = 0, qhi = 0;
  if (valid) q_interval(c, qlo, qhi);
  int wg_lo, wg_hi, tmp;
  q_interval(c_first, wg_lo, tmp);
  q_interval(min(ncols, c_first + BN) - 1, tmp, wg_hi);
  const int qt0 = wg_lo / BM;
  const int nqt = (wg_hi + BM - 1) / BM - qt0;
  const int niter = nqt * a.hdiv;

  TileLoader<HD, BM, 256> ldq, ldo;
  ldq.init(tid);
  ldo.init(tid);
  float st_reg = 0.f;
  auto issue = [&](int it) {
    const int gh = it / nqt;
    const int q0 = (qt0 + it % nqt) * BM;
    const int hq = hkv * a.hdiv + gh;
    ldq.load(a.q + b * a.sq.b + hq * a.sq.h, a.sq.t, q0, a.Tq, tid);
    ldo.load(a.d_o + b * a.sdo.b + hq * a.sdo.h, a.sdo.t, q0, a.Tq, tid);
    if (tid < 2 * BM) {
      const int row = q0 + (tid & (BM - 1));
      st_reg = 0.f;
      if (row < a.Tq)
        st_reg = tid < BM ? a.lse[((int64_t)b * a.Tq + row) * a.Hq + hq]
                          : a.delta[((int64_t)b * a.Hq + hq) * a.Tq + row];
    }
  };
  auto commit = [&](int stage) {
    ldq.store(Qs[stage]);
    ldo.store(dOs[stage]);
    if (tid < 2 * BM) stat[stage * 2 * BM + tid] = st_reg;
  };

  f32x16 dk[DB], dv[DB];
#pragma unroll
  for (int d = 0; d < DB; d++)
#pragma unroll
    for (int i = 0; i < 16; i++) {
      dk[d][i] = 0.f;
      dv[d][i] = 0.f;
    }
  const float sc = a.scale * kLog2e;

  if (niter > 0) {
    issue(0);
    commit(0);
  }
  __syncthreads();

  for (int it = 0; it < niter; it++) {
    const int cur = it & 1;
    if (it + 1 < niter) issue(it + 1);
    const int q0 = (qt0 + it % nqt) * BM;
    const bool touches = (qhi > q0) && (qlo < q0 + BM) && (qhi > qlo);
    if (__any(touches)) {
      const bool full = (qlo <= q0) && (qhi >= q0 + BM);
      const bool need_mask = !__all(full);
      MODA_LDS const float* lse_s = stat + cur * 2 * BM;
      MODA_LDS const float* del_s = lse_s + BM;
      // two 32-row halves of the query tile, one after the other: only one half's scores are live
#pragma unroll
      for (int bb = 0; bb < 2; bb++) {
        f32x16 s, dp;
#pragma unroll
        for (int i = 0; i < 16; i++) {
          s[i] = 0.f;
          dp[i] = 0.f;
        }
#pragma unroll
        for (int kk = 0; kk < KK; kk++) {
          s = mfma32<T>(lds_row_operand<HD>(Qs[cur], 32 * bb, kk, lane), Kr[kk], s);
          dp = mfma32<T>(lds_row_operand<HD>(dOs[cur], 32 * bb, kk, lane), Vr[kk], dp);
        }
#pragma unroll
        for (int i4 = 0; i4 < 4; i4++) {
          const int row0 = 32 * bb + 8 * i4 + 4 * g;
          const f32x4 lv = *reinterpret_cast<MODA_LDS const f32x4*>(lse_s + row0);
          const f32x4 dl = *reinterpret_cast<MODA_LDS const f32x4*>(del_s + row0);
#pragma unroll
          for (int j = 0; j < 4; j++) {
            const int i = 4 * i4 + j;
            float p = fast_exp2(__builtin_fmaf(s[i], sc, -lv[j]));
            if (need_mask) {
              const int qr = q0 + row0 + j;
              p = (qr >= qlo && qr < qhi) ? p : 0.f;
            }
            s[i] = p;
            dp[i] = p * (dp[i] - dl[j]);
          }
        }
        i32x4 P[2], DS[2];
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
          P[ks] = pack8<T>(s, ks * 8);
          DS[ks] = pack8<T>(dp, ks * 8);
        }
#pragma unroll
        for (int d = 0; d < DB; d++)
#pragma unroll
          for (int ks = 0; ks < 2; ks++) {
            dv[d] = mfma32<T>(lds_tr_operand<HD>(dOs[cur], 32 * bb + 16 * ks, d, lane), P[ks], dv[d]);
            dk[d] = mfma32<T>(lds_tr_operand<HD>(Qs[cur], 32 * bb + 16 * ks, d, lane), DS[ks], dk[d]);
          }
      }
    }
    if (it + 1 < niter) commit(cur ^ 1);
    __syncthreads();
  }

  if (valid) {
    uint16_t* dkp = dep ? a.dkd + b * a.sdkd.b + hkv * a.sdkd.h + (int64_t)c * a.sdkd.t
                        : a.dk + b * a.sdk.b + hkv * a.sdk.h + (int64_t)c * a.sdk.t;
    uint16_t* dvp = dep ? a.dvd + b * a.sdvd.b + hkv * a.sdvd.h + (int64_t)c * a.sdvd.t
                        : a.dv + b * a.sdv.b + hkv * a.sdv.h + (int64_t)c * a.sdv.t;
#pragma unroll
    for (int d = 0; d < DB; d++)
#pragma unroll
      for (int i4 = 0; i4 < 4; i4++) {
        i32x2 w;
        w[0] = pack2<T>(dk[d][4 * i4 + 0] * a.scale, dk[d][4 * i4 + 1] * a.scale);
        w[1] = pack2<T>(dk[d][4 * i4 + 2] * a.scale, dk[d][4 * i4 + 3] * a.scale);
        *reinterpret_cast<i32x2*>(dkp + 32 * d + 8 * i4 + 4 * g) = w;
        w[0] = pack2<T>(dv[d][4 * i4 + 0], dv[d][4 * i4 + 1]);
        w[1] = pack2<T>(dv[d][4 * i4 + 2], dv[d][4 * i4 + 3]);
        *reinterpret_cast<i32x2*>(dvp + 32 * d + 8 * i4 + 4 * g) = w;
      }
  }
}

template <typename T, int HD>
hipError_t launch_dkv_t(const KArgs& a, hipStream_t stream) {
  constexpr size_t smem = 4 * 64 * HD * sizeof(uint16_t) + 2 * 2 * 64 * sizeof(float);
  static bool attr_done = false;
  if (!attr_done) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&dkv_kernel<T, HD>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) return e;
    attr_done = true;
  }
  const int64_t n_seq_tiles = a.has_seq ? (a.T + 127) / 128 : 0;
  const int64_t n_dep_tiles = a.L > 0 ? ((int64_t)a.T * a.L + 127) / 128 : 0;
  const int64_t nblk = (n_seq_tiles + n_dep_tiles) * a.B * a.Hkv;
  if (nblk == 0) return hipSuccess;
  hipLaunchKernelGGL((dkv_kernel<T, HD>), dim3((unsigned)nblk), dim3(256), smem, stream, a);
  return hipGetLastError();
}

hipError_t launch_dkv(const KArgs& a, int dtype, int hd, hipStream_t stream) {
  if (dtype == 0 && hd == 128) return launch_dkv_t<BF16, 128>(a, stream);
  if (dtype == 0 && hd == 64) return launch_dkv_t<BF16, 64>(a, stream);
  if (dtype == 1 && hd == 128) return launch_dkv_t<FP16, 128>(a, stream);
  if (dtype == 1 && hd == 64) return launch_dkv_t<FP16, 64>(a, stream);
  return hipErrorInvalidValue;
}

}  // namespace moda
