// C ABI of libmoda_hip.so (see include/moda_hip.h): descriptor validation and
// dispatch to the gfx950 kernels.  No tensor-library types cross this file.
#include <hip/hip_runtime.h>

#include <atomic>
#include <string.h>

#include "../../include/moda_hip.h"
#include "geometry.h"
#include "kargs.h"

namespace moda {
hipError_t launch_fwd(const KArgs& a, int dtype, int hd, hipStream_t stream);
hipError_t launch_delta(const KArgs& a, int dtype, int hd, hipStream_t stream);
hipError_t launch_dq(const KArgs& a, int dtype, int hd, hipStream_t stream);
hipError_t launch_dkv(const KArgs& a, int dtype, int hd, hipStream_t stream);
hipError_t launch_generic(const KArgs& a, int dtype, int D, int Dv, int which, hipStream_t stream);
hipError_t launch_reorg(void* const* layers, int64_t n_layers, int64_t slot0, int64_t L_total, int64_t n_tokens,
                        int64_t row_bytes, void* cache, bool to_cache, hipStream_t stream);
}  // namespace moda

using moda::KArgs;
using moda::Str3;

namespace {

int elem_size(int dtype) { return dtype == MODA_HIP_FP32 ? 4 : 2; }

Str3 cvt(const moda_hip_strides& s) { return Str3{s.b, s.t, s.h}; }

// The MFMA kernels move rows with 16-byte accesses; the vector-ALU kernels load element by element and
// need element alignment only.
bool aligned(const void* p, const moda_hip_strides& s, int esize, bool vec16) {
  if (!vec16) return (uintptr_t)p % esize == 0;
  const int64_t m = 16 / esize;
  return ((uintptr_t)p % 16 == 0) && (s.b % m == 0) && (s.t % m == 0) && (s.h % m == 0);
}

// The streaming kernels address rows inside a tile with 32-bit byte offsets: a row stride must stay
// below 16 MiB (tiles have at most 64 rows per pass).
bool row_stride_ok(const moda_hip_strides& s, int esize) { return s.t >= 0 && s.t * esize < (1ll << 24); }

// A partially filled depth stream is read through one descriptor per tile, anchored at the first column's token:
// the byte offsets of a tile's 64 columns from that anchor -- up to 64 / Lv + 2 tokens of L rows -- must fit 31 bits.
bool mapped_span_ok(const KArgs& a, const moda_hip_strides& s, int esize) {
  if (a.L == 0 || a.Lv == a.L) return true;
  return (int64_t)(64 / a.Lv + 2) * a.L * s.t * esize < (1ll << 31);
}

int value_dim(const moda_hip_desc* d) { return (int)(d->Dv > 0 ? d->Dv : d->D); }

// The matrix-core kernels exist for tile widths 64, 128 and 256; any 16-bit head dim that is a multiple of 8 (whole
// 16-byte chunks) up to 256 runs on the next width, zero-padded inside the kernels.
bool mfma_shape(const moda_hip_desc* d) {
  return (d->dtype == MODA_HIP_BF16 || d->dtype == MODA_HIP_FP16) && d->D % 8 == 0 && d->D <= 256 &&
         value_dim(d) % 8 == 0 && value_dim(d) <= 256;
}
// Packed variable-length batches with head dims above 128 do not run the packed instantiations of the 256-wide
// kernels: that combination (with chunk-visible mode) once ended in a GPU memory fault whose cause was never
// found, so those instantiations stay switched off.  With a host copy of the offsets the batch runs as one launch
// per sequence on the fixed-length 256-wide kernels (per_sequence below); without it, on the vector-ALU kernels.
int widest_dim(const moda_hip_desc* d) { return (int)(d->D > value_dim(d) ? d->D : value_dim(d)); }
bool packed_wide(const moda_hip_desc* d) { return widest_dim(d) > 128 && d->cu_seqlens; }
bool per_sequence(const moda_hip_desc* d) { return mfma_shape(d) && packed_wide(d) && d->cu_seqlens_host; }
bool use_mfma(const moda_hip_desc* d) { return mfma_shape(d) && !packed_wide(d); }
// keys and values share one tile width: that of the wider of the two head dims
int tile_width(const moda_hip_desc* d) { return widest_dim(d) <= 64 ? 64 : widest_dim(d) <= 128 ? 128 : 256; }

// Validates the descriptor and fills the geometry part of KArgs.
int fill_geometry(const moda_hip_desc* d, KArgs& a) {
  if (!d || d->struct_size != (int32_t)sizeof(moda_hip_desc)) return MODA_HIP_EINVAL;
  if (d->dtype < MODA_HIP_BF16 || d->dtype > MODA_HIP_FP32) return MODA_HIP_EINVAL;
  if (d->mode < MODA_HIP_CAUSAL || d->mode > MODA_HIP_PLAIN_GQA) return MODA_HIP_EINVAL;
  if (d->B < 0 || d->T < 0 || d->H <= 0 || d->G <= 0 || d->D <= 0 || d->L < 0) return MODA_HIP_EINVAL;
  if (d->D > 256 || d->D % 4 != 0) return MODA_HIP_EUNSUPPORTED;
  if (d->Dv < 0) return MODA_HIP_EINVAL;
  if (d->Dv > 256 || d->Dv % 4 != 0) return MODA_HIP_EUNSUPPORTED;
  if (d->mode == MODA_HIP_PLAIN_GQA && d->L != 0) return MODA_HIP_EINVAL;
  if (d->mode == MODA_HIP_DEPTH_ONLY && d->L == 0) return MODA_HIP_EINVAL;
  if (d->mode == MODA_HIP_CHUNK_VISIBLE && d->L > 0 && d->chunk_tokens <= 0) return MODA_HIP_EINVAL;
  if (d->L_valid < 0 || d->L_valid > d->L) return MODA_HIP_EINVAL;
  if (d->flags & ~(int32_t)MODA_HIP_FLAG_ACCUMULATE_DEPTH_GRADS) return MODA_HIP_EINVAL;
  // 32-bit index space used for rows and flattened depth columns inside the kernels
  if (d->T * d->G >= (1ll << 30) || d->T * (d->L > 0 ? d->L : 1) >= (1ll << 30) || d->B * d->H * d->G >= (1ll << 20))
    return MODA_HIP_EUNSUPPORTED;
  memset(&a, 0, sizeof(a));
  const bool plain = d->mode == MODA_HIP_PLAIN_GQA;
  a.B = (int)d->B;
  a.T = (int)d->T;
  a.Hkv = (int)d->H;
  a.D = (int)d->D;
  a.Dv = value_dim(d);
  a.Tq = plain ? (int)d->T : (int)(d->T * d->G);
  a.Gf = plain ? 1 : (int)d->G;
  a.Hq = plain ? (int)(d->H * d->G) : (int)d->H;
  a.hdiv = plain ? (int)d->G : 1;
  a.L = (int)d->L;
  a.Lv = d->L_valid > 0 ? (int)d->L_valid : (int)d->L;
  if (a.Lv == 0) a.Lv = a.L = 0;
  a.Cb = d->mode == MODA_HIP_CHUNK_VISIBLE ? (int)(d->chunk_tokens > 0 ? d->chunk_tokens : 1) : 1;
  a.has_seq = d->mode != MODA_HIP_DEPTH_ONLY;
  a.causal = d->mode == MODA_HIP_CAUSAL || d->mode == MODA_HIP_CHUNK_VISIBLE || plain;
  a.chunk = d->mode == MODA_HIP_CHUNK_VISIBLE;
  a.accum_depth = (d->flags & MODA_HIP_FLAG_ACCUMULATE_DEPTH_GRADS) ? 1 : 0;
  a.nqt = (a.Tq + 127) / 128;
  a.scale = d->scale;
  a.delta_pitch = a.Tq;
  a.dkv_split = 1;
  if (d->cu_seqlens) {
    // packed batch: T is the longest sequence, the row axes hold total_tokens tokens
    if (d->total_tokens < d->T || ((uintptr_t)d->cu_seqlens % 4) != 0) return MODA_HIP_EINVAL;
    if (d->total_tokens * d->G >= (1ll << 30) || d->total_tokens * (d->L > 0 ? d->L : 1) >= (1ll << 30))
      return MODA_HIP_EUNSUPPORTED;
    if (d->cu_seqlens_host) {  // the host copy can be checked: offsets start at 0, do not decrease, fit T and total
      const int32_t* h = d->cu_seqlens_host;
      if (h[0] != 0 || h[d->B] != d->total_tokens) return MODA_HIP_EINVAL;
      for (int64_t i = 0; i < d->B; i++)
        if (h[i + 1] < h[i] || h[i + 1] - h[i] > d->T) return MODA_HIP_EINVAL;
    }
    a.cu = d->cu_seqlens;
    a.delta_pitch = (int)(plain ? d->total_tokens : d->total_tokens * d->G);
  } else if (d->cu_seqlens_host) {
    return MODA_HIP_EINVAL;
  }
  return MODA_HIP_OK;
}

// Bytes of the row-sum part of the backward workspace, rounded up so that what follows stays aligned.
size_t delta_bytes_exact(const KArgs& a) {
  const size_t n = (a.cu ? (size_t)1 : (size_t)a.B) * a.Hq * a.delta_pitch * sizeof(float);
  return n ? n : sizeof(float);
}
size_t delta_bytes(const KArgs& a) { return (delta_bytes_exact(a) + 255) / 256 * 256; }

// Row segments per column tile of the sequence dK/dV kernel (see KArgs::dkv_split).  A launch whose column
// tiles cannot give every compute unit two workgroups is cut further along the query rows, as long as a
// segment keeps at least 16 query tiles.  Sized for the 256 compute units of a whole MI355X whatever the
// partition mode, so that the workspace size depends on the descriptor alone.
int desired_dkv_split(const moda_hip_desc* d, const KArgs& a) {
  if (!use_mfma(d) || a.cu || !a.has_seq || a.T == 0) return 1;
  const int cols = widest_dim(d) > 128 ? 64 : 128, rows = widest_dim(d) > 128 ? 32 : 64;  // the kernel's column tile and query tile
  const int64_t tiles = (int64_t)((a.T + cols - 1) / cols) * a.B * a.Hkv;
  const int64_t query_tiles = (a.Tq + rows - 1) / rows;
  int s = 1;
  while (tiles * s < 512 && s < 8 && query_tiles / (2 * s) >= 16) s *= 2;
  return s;
}

// P and dS of the (query row, depth slot) pairs, handed from the dQ kernel to the depth-gradient kernel (see
// KArgs::depth_p): two 16-bit arrays indexed like the row sums, times the slots that hold data.
size_t depth_handover_bytes(const moda_hip_desc* d, const KArgs& a) {
  if (!use_mfma(d) || !moda::depth_scores_from_dq(a, tile_width(d))) return 0;
  const size_t n = (a.cu ? (size_t)1 : (size_t)a.B) * a.Hq * a.delta_pitch * a.Lv * sizeof(uint16_t);
  return 2 * ((n + 255) / 256 * 256);
}

size_t dkv_part_bytes(const moda_hip_desc* d, const KArgs& a, int split) {
  return split > 1 ? (size_t)2 * split * a.B * a.Hkv * a.T * tile_width(d) * sizeof(float) : 0;
}

// The current device must be a gfx950; reports its compute-unit count.  One entry per device is cached.
int check_device(int* compute_units = nullptr) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return MODA_HIP_EDEVICE;
  struct Entry {
    std::atomic<int> state{0};  // 0 unknown, 1 gfx950, -1 something else
    int cus = 0;
  };
  static Entry cache[64];
  Entry local;
  Entry& e = (dev >= 0 && dev < 64) ? cache[dev] : local;
  int st = e.state.load(std::memory_order_acquire);
  if (st == 0) {
    hipDeviceProp_t p;
    if (hipGetDeviceProperties(&p, dev) != hipSuccess) return MODA_HIP_EDEVICE;
    e.cus = p.multiProcessorCount;
    st = strncmp(p.gcnArchName, "gfx950", 6) == 0 ? 1 : -1;
    e.state.store(st, std::memory_order_release);
  }
  if (compute_units) *compute_units = e.cus;
  return st == 1 ? MODA_HIP_OK : MODA_HIP_EDEVICE;
}

// Workspace of moda_hip_bwd_static: lives in the code object, one copy per device the library is loaded on, for as
// long as the process runs.  In host code the array's name is only a handle for hipGetSymbolAddress; the
// device address is looked up once per device and kept.
static __device__ __align__(256) unsigned char scratch[MODA_HIP_STATIC_WORKSPACE_BYTES];

int static_workspace(void** out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return MODA_HIP_EDEVICE;
  static std::atomic<void*> table[64];
  if (dev < 0 || dev >= 64) return MODA_HIP_EDEVICE;
  void* p = table[dev].load(std::memory_order_acquire);
  if (!p) {
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return MODA_HIP_ELAUNCH;
    table[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return MODA_HIP_OK;
}


// Sequence i of a packed batch as a fixed-length problem of batch size 1: the descriptor, and the element offsets
// of its first query row, key row and depth row on the packed row axes.
struct SeqView {
  moda_hip_desc d;
  int64_t q_row, k_row, d_row;
};
SeqView sequence_view(const moda_hip_desc* d, int64_t i) {
  SeqView v;
  v.d = *d;
  const int64_t t0 = d->cu_seqlens_host[i];
  v.d.B = 1;
  v.d.T = d->cu_seqlens_host[i + 1] - t0;
  v.d.cu_seqlens = nullptr;
  v.d.cu_seqlens_host = nullptr;
  v.d.total_tokens = 0;
  v.q_row = d->mode == MODA_HIP_PLAIN_GQA ? t0 : t0 * d->G;
  v.k_row = t0;
  v.d_row = t0 * d->L;
  return v;
}
const void* at(const void* p, int64_t row, int64_t stride, int esize) {
  return p ? (const char*)p + row * stride * esize : nullptr;
}
void* at(void* p, int64_t row, int64_t stride, int esize) { return p ? (char*)p + row * stride * esize : nullptr; }

#define MODA_REQ_PTR(p) \
  if (!(p)) return MODA_HIP_EINVAL
#define MODA_REQ_ALIGN(p, s)                                    \
  if (!aligned((p), (s), es, vec16)) return MODA_HIP_EALIGN; \
  if (vec16 && !row_stride_ok((s), es)) return MODA_HIP_EUNSUPPORTED

}  // namespace

extern "C" {

int moda_hip_fwd(const moda_hip_desc* d, const void* q, const void* k, const void* v, const void* kd,
                 const void* vd, void* o, float* lse, void* stream) {
  KArgs a;
  int rc = fill_geometry(d, a);
  if (rc) return rc;
  if ((int64_t)a.B * a.Tq * a.Hq == 0) return MODA_HIP_OK;
  const int es = elem_size(d->dtype);
  if (per_sequence(d)) {
    MODA_REQ_PTR(lse);
    for (int64_t i = 0; i < d->B; i++) {
      const SeqView s = sequence_view(d, i);
      if (s.d.T == 0) continue;
      rc = moda_hip_fwd(&s.d, at(q, s.q_row, d->q.t, es), at(k, s.k_row, d->k.t, es), at(v, s.k_row, d->v.t, es),
                        at(kd, s.d_row, d->kd.t, es), at(vd, s.d_row, d->vd.t, es), at(o, s.q_row, d->o.t, es),
                        lse + s.q_row * a.Hq, stream);
      if (rc) return rc;
    }
    return MODA_HIP_OK;
  }
  const bool vec16 = use_mfma(d);
  MODA_REQ_PTR(q);
  MODA_REQ_PTR(o);
  MODA_REQ_PTR(lse);
  MODA_REQ_ALIGN(q, d->q);
  MODA_REQ_ALIGN(o, d->o);
  if (a.has_seq) {
    MODA_REQ_PTR(k);
    MODA_REQ_PTR(v);
    MODA_REQ_ALIGN(k, d->k);
    MODA_REQ_ALIGN(v, d->v);
  }
  if (a.L > 0) {
    MODA_REQ_PTR(kd);
    MODA_REQ_PTR(vd);
    MODA_REQ_ALIGN(kd, d->kd);
    MODA_REQ_ALIGN(vd, d->vd);
    if (vec16 && !(mapped_span_ok(a, d->kd, es) && mapped_span_ok(a, d->vd, es))) return MODA_HIP_EUNSUPPORTED;
  }
  if ((rc = check_device(&a.compute_units))) return rc;
  a.q = (const uint16_t*)q;
  a.k = (const uint16_t*)k;
  a.v = (const uint16_t*)v;
  a.kd = (const uint16_t*)kd;
  a.vd = (const uint16_t*)vd;
  a.out_o = (uint16_t*)o;
  a.lse = lse;
  a.sq = cvt(d->q);
  a.sk = cvt(d->k);
  a.sv = cvt(d->v);
  a.skd = cvt(d->kd);
  a.svd = cvt(d->vd);
  a.so = cvt(d->o);
  hipError_t e = use_mfma(d) ? moda::launch_fwd(a, d->dtype, tile_width(d), (hipStream_t)stream)
                             : moda::launch_generic(a, d->dtype, (int)d->D, value_dim(d), 0, (hipStream_t)stream);
  return e == hipSuccess ? MODA_HIP_OK : MODA_HIP_ELAUNCH;
}

size_t moda_hip_bwd_workspace_bytes(const moda_hip_desc* d) {
  KArgs a;
  if (fill_geometry(d, a)) return 0;
  const size_t part = dkv_part_bytes(d, a, desired_dkv_split(d, a));
  const size_t hand = depth_handover_bytes(d, a);
  // the row sums, then (each optional) the handed-over depth scores and the partial sums of the row split
  return (part || hand) ? delta_bytes(a) + hand + part : delta_bytes_exact(a);
}

int moda_hip_bwd(const moda_hip_desc* d, const void* q, const void* k, const void* v, const void* kd,
                 const void* vd, const void* o, const float* lse, const void* d_o, void* dq, void* dk, void* dv,
                 void* dkd, void* dvd, void* workspace, size_t workspace_bytes, void* stream) {
  return moda_hip_bwd_stages(d, q, k, v, kd, vd, o, lse, d_o, dq, dk, dv, dkd, dvd, workspace, workspace_bytes,
                             MODA_HIP_STAGE_ALL, stream);
}

int moda_hip_bwd_static(const moda_hip_desc* d, const void* q, const void* k, const void* v, const void* kd,
                        const void* vd, const void* o, const float* lse, const void* d_o, void* dq, void* dk,
                        void* dv, void* dkd, void* dvd, void* stream) {
  KArgs g;
  const int grc = fill_geometry(d, g);
  if (grc) return grc;
  if (delta_bytes_exact(g) > (size_t)MODA_HIP_STATIC_WORKSPACE_BYTES) return MODA_HIP_ESTATIC;
  void* ws = nullptr;
  const int rc = static_workspace(&ws);
  if (rc) return rc;
  return moda_hip_bwd_stages(d, q, k, v, kd, vd, o, lse, d_o, dq, dk, dv, dkd, dvd, ws,
                             (size_t)MODA_HIP_STATIC_WORKSPACE_BYTES, MODA_HIP_STAGE_ALL, stream);
}

int moda_hip_bwd_stages(const moda_hip_desc* d, const void* q, const void* k, const void* v, const void* kd,
                        const void* vd, const void* o, const float* lse, const void* d_o, void* dq, void* dk,
                        void* dv, void* dkd, void* dvd, void* workspace, size_t workspace_bytes, int stages,
                        void* stream) {
  KArgs a;
  int rc = fill_geometry(d, a);
  if (rc) return rc;
  if (stages < 0 || stages > MODA_HIP_STAGE_ALL) return MODA_HIP_EINVAL;
  const int es = elem_size(d->dtype);
  if (per_sequence(d) && (int64_t)a.B * a.Tq * a.Hq > 0) {
    MODA_REQ_PTR(lse);
    if (!workspace || workspace_bytes < delta_bytes_exact(a)) return MODA_HIP_EWORKSPACE;
    for (int64_t i = 0; i < d->B; i++) {
      const SeqView s = sequence_view(d, i);
      if (s.d.T == 0) continue;
      // every sequence keeps its own part of the row-sum workspace ([heads][its query rows]), so the stages of
      // one backward may still be issued as separate calls
      const size_t ws_off = (size_t)a.Hq * s.q_row * sizeof(float);
      const size_t ws_len = (size_t)a.Hq * (d->mode == MODA_HIP_PLAIN_GQA ? s.d.T : s.d.T * d->G) * sizeof(float);
      rc = moda_hip_bwd_stages(&s.d, at(q, s.q_row, d->q.t, es), at(k, s.k_row, d->k.t, es),
                               at(v, s.k_row, d->v.t, es), at(kd, s.d_row, d->kd.t, es), at(vd, s.d_row, d->vd.t, es),
                               at(o, s.q_row, d->o.t, es), lse + s.q_row * a.Hq, at(d_o, s.q_row, d->d_o.t, es),
                               at(dq, s.q_row, d->dq.t, es), at(dk, s.k_row, d->dk.t, es), at(dv, s.k_row, d->dv.t, es),
                               at(dkd, s.d_row, d->dkd.t, es), at(dvd, s.d_row, d->dvd.t, es),
                               (char*)workspace + ws_off, ws_len, stages, stream);
      if (rc) return rc;
    }
    return MODA_HIP_OK;
  }
  const bool vec16 = use_mfma(d);
  const bool have_rows = (int64_t)a.B * a.Tq * a.Hq > 0;
  if (have_rows) {
    MODA_REQ_PTR(q);
    MODA_REQ_PTR(o);
    MODA_REQ_PTR(lse);
    MODA_REQ_PTR(d_o);
    MODA_REQ_PTR(dq);
    MODA_REQ_ALIGN(q, d->q);
    MODA_REQ_ALIGN(o, d->o);
    MODA_REQ_ALIGN(d_o, d->d_o);
    MODA_REQ_ALIGN(dq, d->dq);
    if (a.has_seq) {
      MODA_REQ_PTR(k);
      MODA_REQ_PTR(v);
      MODA_REQ_PTR(dk);
      MODA_REQ_PTR(dv);
      MODA_REQ_ALIGN(k, d->k);
      MODA_REQ_ALIGN(v, d->v);
      MODA_REQ_ALIGN(dk, d->dk);
      MODA_REQ_ALIGN(dv, d->dv);
    }
    if (a.L > 0) {
      MODA_REQ_PTR(kd);
      MODA_REQ_PTR(vd);
      MODA_REQ_PTR(dkd);
      MODA_REQ_PTR(dvd);
      MODA_REQ_ALIGN(kd, d->kd);
      MODA_REQ_ALIGN(vd, d->vd);
      MODA_REQ_ALIGN(dkd, d->dkd);
      MODA_REQ_ALIGN(dvd, d->dvd);
      if (vec16 && !(mapped_span_ok(a, d->kd, es) && mapped_span_ok(a, d->vd, es))) return MODA_HIP_EUNSUPPORTED;
    }
    if (!workspace || workspace_bytes < delta_bytes_exact(a)) return MODA_HIP_EWORKSPACE;
    if ((uintptr_t)workspace % sizeof(float) != 0) return MODA_HIP_EALIGN;
    // the row split of light launches uses what the workspace offers beyond the row sums: a caller that gives
    // less than moda_hip_bwd_workspace_bytes asks for (moda_hip_bwd_static) gets fewer segments or none
    // ... and likewise the hand-over of the depth scores from the dQ kernel to the depth-gradient kernel, which sits
    // between the row sums and the partial sums
    size_t hand = depth_handover_bytes(d, a);
    if (delta_bytes(a) + hand > workspace_bytes) hand = 0;
    int split = desired_dkv_split(d, a);
    while (split > 1 && delta_bytes(a) + hand + dkv_part_bytes(d, a, split) > workspace_bytes) split /= 2;
    if ((uintptr_t)workspace % 16 != 0) split = 1;  // the partial sums are written and read 16 bytes at a time
    a.dkv_split = split;
    a.dkv_part = (float*)((char*)workspace + delta_bytes(a) + hand);
    if (hand) {
      a.depth_p = (uint16_t*)((char*)workspace + delta_bytes(a));
      a.depth_ds = (uint16_t*)((char*)workspace + delta_bytes(a) + hand / 2);
    }
  } else {
    return MODA_HIP_OK;
  }
  if ((rc = check_device(&a.compute_units))) return rc;
  a.q = (const uint16_t*)q;
  a.k = (const uint16_t*)k;
  a.v = (const uint16_t*)v;
  a.kd = (const uint16_t*)kd;
  a.vd = (const uint16_t*)vd;
  a.o = (const uint16_t*)o;
  a.d_o = (const uint16_t*)d_o;
  a.lse = const_cast<float*>(lse);
  a.delta = (float*)workspace;
  a.dq = (uint16_t*)dq;
  a.dk = (uint16_t*)dk;
  a.dv = (uint16_t*)dv;
  a.dkd = (uint16_t*)dkd;
  a.dvd = (uint16_t*)dvd;
  a.sq = cvt(d->q);
  a.sk = cvt(d->k);
  a.sv = cvt(d->v);
  a.skd = cvt(d->kd);
  a.svd = cvt(d->vd);
  a.so = cvt(d->o);
  a.sdo = cvt(d->d_o);
  a.sdq = cvt(d->dq);
  a.sdk = cvt(d->dk);
  a.sdv = cvt(d->dv);
  a.sdkd = cvt(d->dkd);
  a.sdvd = cvt(d->dvd);
  hipStream_t s = (hipStream_t)stream;
  hipError_t e = hipSuccess;
  if (use_mfma(d)) {
    // with both stages asked for, the dQ kernel forms the row sums itself (one launch and one pass over o, do less)
    a.own_delta = (stages & MODA_HIP_STAGE_DELTA) && (stages & MODA_HIP_STAGE_DQ) ? 1 : 0;
    if ((stages & MODA_HIP_STAGE_DELTA) && !a.own_delta) e = moda::launch_delta(a, d->dtype, tile_width(d), s);
    if (e == hipSuccess && (stages & MODA_HIP_STAGE_DQ)) e = moda::launch_dq(a, d->dtype, tile_width(d), s);
    if (e == hipSuccess && (stages & MODA_HIP_STAGE_DKV)) e = moda::launch_dkv(a, d->dtype, tile_width(d), s);
  } else {
    // the generic kernels recompute delta inline; the DELTA stage is a no-op for them
    if (stages & MODA_HIP_STAGE_DQ) e = moda::launch_generic(a, d->dtype, (int)d->D, value_dim(d), 1, s);
    if (e == hipSuccess && (stages & MODA_HIP_STAGE_DKV)) e = moda::launch_generic(a, d->dtype, (int)d->D, value_dim(d), 2, s);
  }
  return e == hipSuccess ? MODA_HIP_OK : MODA_HIP_ELAUNCH;
}

int moda_hip_depth_reorg_fwd(const void* const* layers, int64_t n_layers, int64_t slot0, int64_t L_total, int64_t B,
                             int64_t T, int64_t H, int64_t D, int32_t dtype, void* cache, void* stream) {
  if (n_layers < 0 || slot0 < 0 || slot0 + n_layers > L_total || B < 0 || T < 0 || H <= 0 || D <= 0)
    return MODA_HIP_EINVAL;
  if (dtype < MODA_HIP_BF16 || dtype > MODA_HIP_FP32) return MODA_HIP_EINVAL;
  if (B * T == 0 || n_layers == 0) return MODA_HIP_OK;
  if (!layers || !cache) return MODA_HIP_EINVAL;
  for (int64_t i = 0; i < n_layers; i++)
    if (!layers[i]) return MODA_HIP_EINVAL;
  if (B * T >= (1ll << 31)) return MODA_HIP_EUNSUPPORTED;
  hipError_t e = moda::launch_reorg(const_cast<void* const*>(layers), n_layers, slot0, L_total, B * T,
                                    H * D * elem_size(dtype), cache, true, (hipStream_t)stream);
  return e == hipSuccess ? MODA_HIP_OK : MODA_HIP_ELAUNCH;
}

int moda_hip_depth_reorg_bwd(const void* d_cache, int64_t n_layers, int64_t slot0, int64_t L_total, int64_t B,
                             int64_t T, int64_t H, int64_t D, int32_t dtype, void* const* d_layers, void* stream) {
  if (n_layers < 0 || slot0 < 0 || slot0 + n_layers > L_total || B < 0 || T < 0 || H <= 0 || D <= 0)
    return MODA_HIP_EINVAL;
  if (dtype < MODA_HIP_BF16 || dtype > MODA_HIP_FP32) return MODA_HIP_EINVAL;
  if (B * T == 0 || n_layers == 0) return MODA_HIP_OK;
  if (!d_layers || !d_cache) return MODA_HIP_EINVAL;
  for (int64_t i = 0; i < n_layers; i++)
    if (!d_layers[i]) return MODA_HIP_EINVAL;
  if (B * T >= (1ll << 31)) return MODA_HIP_EUNSUPPORTED;
  hipError_t e = moda::launch_reorg(d_layers, n_layers, slot0, L_total, B * T, H * D * elem_size(dtype),
                                    const_cast<void*>(d_cache), false, (hipStream_t)stream);
  return e == hipSuccess ? MODA_HIP_OK : MODA_HIP_ELAUNCH;
}

int moda_hip_uses_matrix_cores(const moda_hip_desc* d) {
  KArgs a;
  const int rc = fill_geometry(d, a);
  if (rc) return rc;
  return (use_mfma(d) || per_sequence(d)) ? 1 : 0;
}

const char* moda_hip_strerror(int code) {
  switch (code) {
    case MODA_HIP_OK: return "ok";
    case MODA_HIP_EINVAL: return "invalid descriptor field or missing tensor pointer";
    case MODA_HIP_EUNSUPPORTED: return "unsupported head dim / dtype / size";
    case MODA_HIP_EALIGN: return "tensor pointer or stride is not 16-byte aligned";
    case MODA_HIP_EWORKSPACE: return "workspace missing or too small";
    case MODA_HIP_ELAUNCH: return "HIP kernel launch failed";
    case MODA_HIP_EDEVICE: return "current device is not an MI355X-class (gfx950) GPU";
    case MODA_HIP_ESTATIC: return "problem needs more than the MODA_HIP_STATIC_WORKSPACE_BYTES of moda_hip_bwd_static";
    default: return "unknown error";
  }
}

int moda_hip_version(void) { return MODA_HIP_VERSION; }

}  // extern "C"
