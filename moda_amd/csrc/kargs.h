// Kernel argument block shared by the host launchers and the device kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace moda {

struct Str3 {
  int64_t b, t, h;
};

struct KArgs {
  const uint16_t *q, *k, *v, *kd, *vd, *o, *d_o;
  uint16_t *out_o, *dq, *dk, *dv, *dkd, *dvd;
  float* lse;          // [B, Tq, Hq]   (written by forward, read by backward)
  float* delta;        // [B, Hq, delta_pitch]   workspace: MINUS rowsum(o * do)
  Str3 sq, sk, sv, skd, svd, so, sdo, sdq, sdk, sdv, sdkd, sdvd;
  int B, T, Hkv;
  int D;     // head dim of q, k, kd and their gradients; the matrix kernels run it zero-padded to their tile width
  int Dv;    // head dim of v, vd, o, do and their gradients (same tile width)
  int Tq;    // query rows per (batch, query head)
  int Gf;    // query rows per token (fold factor)
  int Hq;    // query-head programs per batch
  int hdiv;  // kv head = hq / hdiv
  int L;     // depth slots per token in the depth tensors (row t*L + l = slot l of token t)
  int Lv;    // slots per token that hold data, 1 <= Lv <= L: slots l >= Lv are invisible
  int Cb;    // chunk-visible: tokens per chunk
  int has_seq, causal, chunk;
  int accum_depth;  // dkd, dvd += (slots l >= Lv untouched) instead of = (slots l >= Lv zeroed)
  int own_delta;    // the dQ kernel forms the row sums of o * do itself and leaves them in `delta` for the later kernels
  // Outside chunk-visible mode a query row sees the Lv depth slots of its own token only.  When the dQ kernel walks
  // them (its waves' own depth columns) it leaves the rounded P and dS of those (row, slot) pairs here,
  // [B, Hq, delta_pitch / Gf tokens, Lv, Gf] each (a token's block starts at the `delta` index of its first row
  // times Lv; inside it slot-major, the token's Gf rows side by side), and the depth-gradient kernel forms dkd, dvd
  // from them and the rows of q, do without reading kd, vd again.  Null: no room in the workspace, or another route.
  uint16_t *depth_p, *depth_ds;
  // Sequence dK/dV of launches too small to fill the device: the query rows of every column tile are cut into
  // `dkv_split` segments, one workgroup each, which leave fp32 partial sums in `dkv_part`
  // ([2 (dk, dv)][dkv_split][B][Hkv][T][D]); a second kernel adds them in segment order.  1 = no split.
  int dkv_split;
  float* dkv_part;
  int nqt;   // query tiles per (batch, query head)
  float scale;
  int compute_units;  // of the device the launch goes to (host-side launch-shape decisions)
  // Packed variable-length batch: cu[b] .. cu[b+1] are the base tokens of sequence b on a row axis all
  // sequences share (the tensors have no batch axis then); T, Tq above are those of the longest sequence.
  const int32_t* cu;
  int delta_pitch;  // query rows per head in `delta`: Tq, or the packed total
};

// Variable-length batches: rebases every tensor on the first row of sequence `b` and shrinks T / Tq to the
// sequence's length, so that the code after it addresses the sequence as batch 0 of a fixed-length problem.
// The launch grid is sized for the longest sequence: callers drop the tiles beyond their own sequence.
// `units`: 16-bit units per tensor element (the data pointers are typed for 16-bit elements).
__host__ __device__ __forceinline__ void enter_sequence(KArgs& a, int& b, int units = 1) {
  if (a.cu == nullptr) return;
  const int t0 = a.cu[b];
  const int T = a.cu[b + 1] - t0;
  const int64_t r0 = (int64_t)t0 * a.Gf * units, c0 = (int64_t)t0 * a.L * units, k0 = (int64_t)t0 * units;
  a.q += r0 * a.sq.t;
  a.o += r0 * a.so.t;
  a.d_o += r0 * a.sdo.t;
  a.out_o += r0 * a.so.t;
  a.dq += r0 * a.sdq.t;
  a.k += k0 * a.sk.t;
  a.v += k0 * a.sv.t;
  a.dk += k0 * a.sdk.t;
  a.dv += k0 * a.sdv.t;
  a.kd += c0 * a.skd.t;
  a.vd += c0 * a.svd.t;
  a.dkd += c0 * a.sdkd.t;
  a.dvd += c0 * a.sdvd.t;
  a.lse += (int64_t)t0 * a.Gf * a.Hq;
  a.delta += (int64_t)t0 * a.Gf;
  if (a.depth_p) {
    a.depth_p += (int64_t)t0 * a.Gf * a.Lv;
    a.depth_ds += (int64_t)t0 * a.Gf * a.Lv;
  }
  a.T = T;
  a.Tq = T * a.Gf;
  b = 0;
}

// The argument block a kernel body works on: the launch's own (fixed-length instantiations, no copy)
// or a copy rebased on the workgroup's sequence.
template <bool VARLEN>
struct SeqArgs;
template <>
struct SeqArgs<false> {
  const KArgs& a;
  __device__ __forceinline__ SeqArgs(const KArgs& in, int&) : a(in) {}
};
template <>
struct SeqArgs<true> {
  KArgs a;
  __device__ __forceinline__ SeqArgs(const KArgs& in, int& b) : a(in) { enter_sequence(a, b); }
};

}  // namespace moda
