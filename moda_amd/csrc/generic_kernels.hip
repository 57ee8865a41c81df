// Reference-grade kernels for everything the MFMA kernels do not cover: fp32
// tensors, head dims other than 64/128 (any D <= 256, D % 4 == 0) and a value
// head dim Dv that differs from the key head dim D.  Same
// math, same visible sets and the same base-2 conventions as the MFMA kernels,
// all arithmetic in fp32 on the vector ALU; one 64-lane wave per query row
// (forward, dQ) or per key / depth column (dK, dV).  Not tuned: meant for small
// problems such as the reference's fp32 self-test shapes (moda_v14.py:2917).
#include "kargs.h"
#include "tile.h"

namespace moda {

template <typename E>
__device__ __forceinline__ float ld(const void* base, int64_t idx) {
  return (float)reinterpret_cast<const E*>(base)[idx];
}
template <typename E>
__device__ __forceinline__ void st(void* base, int64_t idx, float v) {
  reinterpret_cast<E*>(base)[idx] = (E)v;
}

__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
  for (int s = 32; s > 0; s >>= 1) x = fmaxf(x, __shfl_xor(x, s, 64));
  return x;
}
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int s = 32; s > 0; s >>= 1) x += __shfl_xor(x, s, 64);
  return x;
}

constexpr int kMaxD = 256;
constexpr int kDR = kMaxD / 64;

struct RowGeom {
  int b, hq, hkv, r, t;
  int shi, dlo, dhi;
};

// `a` arrives as launched and leaves rebased on the row's sequence (variable-length batches)
template <typename E>
__device__ __forceinline__ bool row_geom(KArgs& a, int64_t gid, RowGeom& g) {
  const int64_t total = (int64_t)a.B * a.Hq * a.Tq;
  if (gid >= total) return false;
  g.r = (int)(gid % a.Tq);
  const int bh = (int)(gid / a.Tq);
  g.b = bh / a.Hq;
  g.hq = bh % a.Hq;
  enter_sequence(a, g.b, sizeof(E) / 2);
  if (g.r >= a.Tq) return false;  // a row beyond this sequence
  g.hkv = g.hq / a.hdiv;
  g.t = g.r / a.Gf;
  g.shi = a.has_seq ? (a.causal ? g.t + 1 : a.T) : 0;
  g.dlo = g.dhi = 0;
  if (a.L > 0) {
    const int lo_t = a.chunk ? (g.t / a.Cb) * a.Cb : g.t;
    g.dlo = lo_t * a.L;
    g.dhi = a.chunk ? (g.t + 1) * a.L : g.dlo + a.Lv;  // the token's filled slots
  }
  return true;
}

// MODE 0: forward (o, lse).  MODE 1: dq (needs lse; delta computed inline).
template <typename E, int MODE>
__global__ __launch_bounds__(256) void generic_row_kernel(const KArgs a_in, const int D, const int Dv) {
  __shared__ float qs[4][kMaxD];
  __shared__ float dos[4][kMaxD];
  __shared__ float pb[4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  RowGeom g;
  KArgs a = a_in;
  if (!row_geom<E>(a, (int64_t)blockIdx.x * 4 + wave, g)) return;  // whole wave exits together
  const int64_t qoff = g.b * a.sq.b + g.hq * a.sq.h + (int64_t)g.r * a.sq.t;
  const int64_t dooff = g.b * a.sdo.b + g.hq * a.sdo.h + (int64_t)g.r * a.sdo.t;
  const int64_t ooff = g.b * a.so.b + g.hq * a.so.h + (int64_t)g.r * a.so.t;
  float delta = 0.f, lse = 0.f;
  for (int d = lane; d < D; d += 64) qs[wave][d] = ld<E>(a.q, qoff + d);
  if (MODE == 1) {
    for (int d = lane; d < Dv; d += 64) {
      const float dov = ld<E>(a.d_o, dooff + d);
      dos[wave][d] = dov;
      delta += dov * ld<E>(a.o, ooff + d);
    }
  }
  if (MODE == 1) {
    delta = wave_sum(delta);
    lse = a.lse[((int64_t)g.b * a.Tq + g.r) * a.Hq + g.hq];
  }
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");

  float acc[kDR];
#pragma unroll
  for (int i = 0; i < kDR; i++) acc[i] = 0.f;
  float m = kNegInf, l = 0.f;
  const float sc = a.scale * kLog2e;

  for (int phase = 0; phase < 2; phase++) {
    const int lo = phase == 0 ? 0 : g.dlo;
    const int hi = phase == 0 ? g.shi : g.dhi;
    if (hi <= lo) continue;
    const void* kp = phase == 0 ? (const void*)a.k : (const void*)a.kd;
    const void* vp = phase == 0 ? (const void*)a.v : (const void*)a.vd;
    const Str3 ks = phase == 0 ? a.sk : a.skd;
    const Str3 vs = phase == 0 ? a.sv : a.svd;
    const int64_t kb = g.b * ks.b + g.hkv * ks.h, vb = g.b * vs.b + g.hkv * vs.h;
    for (int c0 = lo; c0 < hi; c0 += 64) {
      const int col = c0 + lane;
      // chunk-visible depth columns span several tokens: the slots without data among them are skipped
      const bool vis = col < hi && !(phase == 1 && a.chunk && (col % a.L) >= a.Lv);
      float s = 0.f, dp = 0.f;
      if (vis) {
        for (int d = 0; d < D; d++) s += qs[wave][d] * ld<E>(kp, kb + (int64_t)col * ks.t + d);
        if (MODE == 1)
          for (int d = 0; d < Dv; d++) dp += dos[wave][d] * ld<E>(vp, vb + (int64_t)col * vs.t + d);
      }
      const float s2 = vis ? s * sc : kNegInf;
      float w;  // weight applied to the value / key row of this column
      float alpha = 1.f;
      if (MODE == 0) {
        const float m_new = fmaxf(m, wave_max(s2));
        alpha = exp2f(m - m_new);
        w = exp2f(s2 - m_new);
        l = l * alpha + wave_sum(w);
        m = m_new;
      } else {
        const float p = vis ? exp2f(s2 - lse) : 0.f;
        w = p * (dp - delta);
      }
      pb[wave][lane] = w;
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      const int nc = min(64, hi - c0);
      const void* xp = MODE == 0 ? vp : kp;
      const int64_t xb = MODE == 0 ? vb : kb;
      const int64_t xs = MODE == 0 ? vs.t : ks.t;
      const int Dx = MODE == 0 ? Dv : D;  // width of the rows being accumulated: values (o) or keys (dq)
#pragma unroll
      for (int i = 0; i < kDR; i++) {
        const int d = lane + 64 * i;
        if (d < Dx) {
          float x = acc[i] * alpha;
          for (int j = 0; j < nc; j++) {
            const float wj = pb[wave][j];  // the same in every lane; rows of weight zero (invisible columns) are not read
            if (wj != 0.f) x += wj * ld<E>(xp, xb + (int64_t)(c0 + j) * xs + d);
          }
          acc[i] = x;
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }
  }
  if (MODE == 0) {
    const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
    for (int i = 0; i < kDR; i++) {
      const int d = lane + 64 * i;
      if (d < Dv) st<E>(a.out_o, ooff + d, acc[i] * inv);
    }
    if (lane == 0) a.lse[((int64_t)g.b * a.Tq + g.r) * a.Hq + g.hq] = l > 0.f ? m + log2f(l) : kNegInf;
  } else {
    const int64_t dqoff = g.b * a.sdq.b + g.hq * a.sdq.h + (int64_t)g.r * a.sdq.t;
#pragma unroll
    for (int i = 0; i < kDR; i++) {
      const int d = lane + 64 * i;
      if (d < D) st<E>(a.dq, dqoff + d, acc[i] * a.scale);
    }
  }
}

// dK/dV: one wave per column (sequence key or depth slot) of one (batch, kv head).
template <typename E>
__global__ __launch_bounds__(256) void generic_col_kernel(const KArgs a_in, const int D, const int Dv) {
  __shared__ float kc[4][kMaxD];
  __shared__ float vc[4][kMaxD];
  __shared__ float pb[4][64];
  __shared__ float dsb[4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  KArgs a = a_in;
  const int n_seq = a.has_seq ? a.T : 0;
  const int ncol = n_seq + a.T * a.L;
  const int64_t gid = (int64_t)blockIdx.x * 4 + wave;
  if (gid >= (int64_t)a.B * a.Hkv * ncol) return;
  const int cidx = (int)(gid % ncol);
  const int bh = (int)(gid / ncol);
  int b = bh / a.Hkv;
  const int hkv = bh % a.Hkv;
  enter_sequence(a, b, sizeof(E) / 2);
  const bool dep = cidx >= n_seq;
  const int col = dep ? cidx - n_seq : cidx;
  if (col >= (dep ? a.T * a.L : a.T)) return;  // a column beyond this sequence
  const void* kp = dep ? (const void*)a.kd : (const void*)a.k;
  const void* vp = dep ? (const void*)a.vd : (const void*)a.v;
  const Str3 ks = dep ? a.skd : a.sk, vs = dep ? a.svd : a.sv;
  const int64_t koff = b * ks.b + hkv * ks.h + (int64_t)col * ks.t;
  const int64_t voff = b * vs.b + hkv * vs.h + (int64_t)col * vs.t;
  for (int d = lane; d < D; d += 64) kc[wave][d] = ld<E>(kp, koff + d);
  for (int d = lane; d < Dv; d += 64) vc[wave][d] = ld<E>(vp, voff + d);
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  int qlo, qhi;
  if (!dep) {
    qlo = a.causal ? col * a.Gf : 0;
    qhi = a.Tq;
  } else {
    const int w = col / a.L;
    qlo = w * a.Gf;
    qhi = a.chunk ? min(a.T, (w / a.Cb + 1) * a.Cb) * a.Gf : (w + 1) * a.Gf;
    if (col - w * a.L >= a.Lv) {  // a slot without data: no row sees it
      if (a.accum_depth) return;  // accumulating: the row holds somebody else's sum
      qhi = qlo;                  // its gradients are zero
    }
  }
  float dk[kDR], dv[kDR];
#pragma unroll
  for (int i = 0; i < kDR; i++) dk[i] = dv[i] = 0.f;
  const float sc = a.scale * kLog2e;
  for (int gh = 0; gh < a.hdiv; gh++) {
    const int hq = hkv * a.hdiv + gh;
    const int64_t qb = b * a.sq.b + hq * a.sq.h, dob = b * a.sdo.b + hq * a.sdo.h, ob = b * a.so.b + hq * a.so.h;
    for (int r0 = qlo; r0 < qhi; r0 += 64) {
      const int r = r0 + lane;
      float p = 0.f, ds = 0.f;
      if (r < qhi) {
        float s = 0.f, dp = 0.f, delta = 0.f;
        for (int d = 0; d < D; d++) s += kc[wave][d] * ld<E>(a.q, qb + (int64_t)r * a.sq.t + d);
        for (int d = 0; d < Dv; d++) {
          const float dov = ld<E>(a.d_o, dob + (int64_t)r * a.sdo.t + d);
          dp += vc[wave][d] * dov;
          delta += dov * ld<E>(a.o, ob + (int64_t)r * a.so.t + d);
        }
        p = exp2f(s * sc - a.lse[((int64_t)b * a.Tq + r) * a.Hq + hq]);
        ds = p * (dp - delta);
      }
      pb[wave][lane] = p;
      dsb[wave][lane] = ds;
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      const int nr = min(64, qhi - r0);
#pragma unroll
      for (int i = 0; i < kDR; i++) {
        const int d = lane + 64 * i;
        if (d < D) {
          float xk = dk[i];
          for (int j = 0; j < nr; j++) xk += dsb[wave][j] * ld<E>(a.q, qb + (int64_t)(r0 + j) * a.sq.t + d);
          dk[i] = xk;
        }
        if (d < Dv) {
          float xv = dv[i];
          for (int j = 0; j < nr; j++) xv += pb[wave][j] * ld<E>(a.d_o, dob + (int64_t)(r0 + j) * a.sdo.t + d);
          dv[i] = xv;
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }
  }
  void* dkp = dep ? (void*)a.dkd : (void*)a.dk;
  void* dvp = dep ? (void*)a.dvd : (void*)a.dv;
  const Str3 dks = dep ? a.sdkd : a.sdk, dvs = dep ? a.sdvd : a.sdv;
  const int64_t dkoff = b * dks.b + hkv * dks.h + (int64_t)col * dks.t;
  const int64_t dvoff = b * dvs.b + hkv * dvs.h + (int64_t)col * dvs.t;
#pragma unroll
  for (int i = 0; i < kDR; i++) {
    const int d = lane + 64 * i;
    const bool add = dep && a.accum_depth;  // this wave is the row's only writer
    if (d < D) st<E>(dkp, dkoff + d, dk[i] * a.scale + (add ? ld<E>(dkp, dkoff + d) : 0.f));
    if (d < Dv) st<E>(dvp, dvoff + d, dv[i] + (add ? ld<E>(dvp, dvoff + d) : 0.f));
  }
}

template <typename E>
hipError_t launch_generic_t(const KArgs& a, int D, int Dv, int which, hipStream_t stream) {
  if (which == 0 || which == 1) {
    const int64_t rows = (int64_t)a.B * a.Hq * a.Tq;
    if (rows == 0) return hipSuccess;
    if ((rows + 3) / 4 >= (1ll << 31)) return hipErrorInvalidValue;
    const unsigned nblk = (unsigned)((rows + 3) / 4);
    if (which == 0)
      hipLaunchKernelGGL((generic_row_kernel<E, 0>), dim3(nblk), dim3(256), 0, stream, a, D, Dv);
    else
      hipLaunchKernelGGL((generic_row_kernel<E, 1>), dim3(nblk), dim3(256), 0, stream, a, D, Dv);
  } else {
    const int64_t ncol = (int64_t)(a.has_seq ? a.T : 0) + (int64_t)a.T * a.L;
    const int64_t cols = ncol * a.B * a.Hkv;
    if (cols == 0) return hipSuccess;
    if ((cols + 3) / 4 >= (1ll << 31)) return hipErrorInvalidValue;
    hipLaunchKernelGGL((generic_col_kernel<E>), dim3((unsigned)((cols + 3) / 4)), dim3(256), 0, stream, a, D, Dv);
  }
  return hipGetLastError();
}

// which: 0 forward, 1 dq, 2 dk/dv
hipError_t launch_generic(const KArgs& a, int dtype, int D, int Dv, int which, hipStream_t stream) {
  if (dtype == 0) return launch_generic_t<__bf16>(a, D, Dv, which, stream);
  if (dtype == 1) return launch_generic_t<_Float16>(a, D, Dv, which, stream);
  if (dtype == 2) return launch_generic_t<float>(a, D, Dv, which, stream);
  return hipErrorInvalidValue;
}

}  // namespace moda
