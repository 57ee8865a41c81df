/*
 * moda_hip.h -- C ABI of libmoda_hip.so: fused sequence+depth attention
 * (MoDA) for AMD MI355X (gfx950), forward and backward, plus the depth-KV
 * cache reorganisation.
 *
 * Every pointer that names tensor data is a DEVICE pointer.  Strides are in
 * elements; the innermost (head-dim) stride is always 1.  For the matrix-core
 * kernels (bf16/fp16, head dims D and Dv multiples of 8 up to 256) every row must be 16-byte
 * aligned (base pointer and all strides multiples of 8 elements) and a row
 * stride must stay below 16 MiB; every other combination runs on vector-ALU
 * kernels that need element alignment only.  All work is enqueued on the hipStream_t passed
 * as `stream` (NULL = the legacy default stream); nothing synchronises the
 * host.  The library keeps no mutable state except where a function says so,
 * apart from one flag per kernel variant and device: the first launch of a
 * variant raises that kernel's dynamic-LDS limit (hipFuncSetAttribute), which is
 * not a stream operation -- under stream capture (HIP graphs) make one ordinary
 * call with the same descriptor first, then capture.
 * Every function returns 0 on success or a negative MODA_HIP_E* code; no
 * function throws.
 *
 * Geometry (symbols as in the reference's docstrings):
 *   folded layouts (modes CAUSAL, NONCAUSAL, CHUNK_VISIBLE, DEPTH_ONLY)
 *     q, o, do, dq : [B, T*G, H, D]   query row r belongs to token r / G
 *     k, v, dk, dv : [B, T,   H, D]
 *     kd, vd, dkd, dvd : [B, T*L, H, D]   depth row t*L + l = slot l of token t
 *     lse          : [B, T*G, H] fp32, base-2 log-sum-exp, contiguous
 *   head-dim GQA layout (mode PLAIN_GQA, causal, no depth stream)
 *     q, o, do, dq : [B, T, H*G, D]   query head hq reads kv head hq / G
 *     lse          : [B, T, H*G]
 *
 * Partially filled depth stream (no counterpart in the reference, which rebuilds a
 * compact [B, T*L, H, D] cache for every layer, vision_tasks/deit/models.py:361-390):
 * with 0 < L_valid < L the depth tensors keep their L slots per token but only
 * slots l < L_valid are visible; results equal those for the compacted tensors
 * [B, T*L_valid, H, D], and dkd, dvd are written as zeros in the other slots.
 * The invisible slots of kd, vd are never read: they may hold anything, bit patterns of
 * NaN or Inf included (an uninitialised cache).  Every mode with a depth stream takes it.
 * On the matrix-core kernels the rows of 64 / L_valid + 2 tokens of a depth tensor
 * ((64 / L_valid + 2) * L * row stride bytes) must span less than 2 GiB
 * (MODA_HIP_EUNSUPPORTED otherwise).
 *
 * Packed variable-length batch (the reference carries a cu_seqlens argument but asserts
 * it away, moda_v14.py:83-101, 2672-2673): with cu_seqlens != NULL the tensors have no
 * batch axis (batch strides are ignored); sequence i of the B sequences owns base tokens
 * [cu_seqlens[i], cu_seqlens[i+1]) of one packed token axis of total_tokens tokens, i.e.
 * query rows cu*G .., key rows cu .., depth rows cu*L .. of q [total*G, H, D],
 * k [total, H, D], kd [total*L, H, D], lse [total*G, H].  Offsets count BASE TOKENS
 * (equal to query rows when G == 1), start at 0 and do not decrease; T is the length of
 * the longest sequence.  Sequences attend only within themselves; chunks of
 * CHUNK_VISIBLE are counted from each sequence's first token.  The offsets are read on
 * the device only: the host cannot check them, rows outside [0, total_tokens) named by
 * them are out-of-bounds accesses.  A caller that also has the offsets in host memory may pass them as
 * cu_seqlens_host: they are then validated, and packed batches with head dims above 128 run on the matrix cores
 * as one launch per sequence (the fixed-length 256-wide kernels on each sequence's rows; the result is the same
 * as one call per sequence); without the host copy that combination runs on the vector-ALU kernels.
 */
#ifndef MODA_HIP_H_
#define MODA_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MODA_HIP_VERSION 105

enum moda_hip_dtype { MODA_HIP_BF16 = 0, MODA_HIP_FP16 = 1, MODA_HIP_FP32 = 2 };

enum moda_hip_mode {
  MODA_HIP_CAUSAL = 0,        /* moda_v14.py:45-378 with IS_CAUSAL=True            */
  MODA_HIP_NONCAUSAL = 1,     /* moda_v14.py:259-300 (IS_CAUSAL=False)             */
  MODA_HIP_CHUNK_VISIBLE = 2, /* moda_v16.py:39-352 (CHUNK_VISIBLE)                */
  MODA_HIP_DEPTH_ONLY = 3,    /* fda_v12.py:44-253 (k, v are NULL)                 */
  MODA_HIP_PLAIN_GQA = 4      /* fla/ops/attn/parallel.py:18-143 (kd, vd are NULL) */
};

enum moda_hip_error {
  MODA_HIP_OK = 0,
  MODA_HIP_EINVAL = -1,      /* bad descriptor field or NULL where data is required */
  MODA_HIP_EUNSUPPORTED = -2,/* head dim / dtype combination without a kernel       */
  MODA_HIP_EALIGN = -3,      /* pointer or stride not 16-byte aligned               */
  MODA_HIP_EWORKSPACE = -4,  /* workspace too small                                 */
  MODA_HIP_ELAUNCH = -5,     /* hipGetLastError() reported a launch failure         */
  MODA_HIP_EDEVICE = -6,     /* current device is not gfx950                        */
  MODA_HIP_ESTATIC = -7      /* moda_hip_bwd_static: problem exceeds the built-in workspace */
};

enum moda_hip_flag {
  /*
   * Backward adds the depth-stream gradients to what dkd, dvd already hold (one rounding to the
   * tensor type per call) instead of overwriting them, and leaves the slots l >= L_valid untouched.
   * With one preallocated depth cache per model and one gradient buffer of the same shape, the
   * backward of layer n (L_valid = n) then adds its share to slots < n, and a layer's K/V gradient is
   * a slice of that buffer: no per-layer rebuild of the cache and no scatter of its gradient
   * (vision_tasks/deit/models.py:361-390 does both for every layer).  Still one writer per row and
   * no atomics.  Every mode with a depth stream takes it.
   */
  MODA_HIP_FLAG_ACCUMULATE_DEPTH_GRADS = 1
};

typedef struct moda_hip_strides {
  int64_t b; /* batch stride   */
  int64_t t; /* row stride     */
  int64_t h; /* head stride    */
} moda_hip_strides;

typedef struct moda_hip_desc {
  int32_t struct_size;  /* sizeof(moda_hip_desc), checked                         */
  int32_t dtype;        /* moda_hip_dtype of q,k,v,kd,vd,o,do and all gradients    */
  int32_t mode;         /* moda_hip_mode                                           */
  int32_t L_valid;      /* depth slots per token that hold data; 0 = all L (see below)          */
  int64_t B;            /* batch                                                   */
  int64_t T;            /* tokens (key rows)                                       */
  int64_t H;            /* kv heads                                                */
  int64_t G;            /* moda_group_num (folded) or query heads per kv head      */
  int64_t D;            /* head dim of q, k, kd (and of v, vd, o unless Dv says otherwise) */
  int64_t L;            /* depth slots per token, 0 = no depth stream              */
  int64_t chunk_tokens; /* CHUNK_VISIBLE: base tokens per chunk (C / G), else 0    */
  float scale;          /* logits = scale * <q, key>                               */
  int32_t flags;        /* OR of moda_hip_flag values, 0 = none                    */
  moda_hip_strides q, k, v, kd, vd, o, d_o, dq, dk, dv, dkd, dvd;
  const int32_t* cu_seqlens; /* packed variable-length batch (see above): DEVICE array of B + 1 offsets, else NULL */
  int64_t total_tokens;      /* with cu_seqlens: cu_seqlens[B], the length of the packed token axis              */
  int64_t Dv;                /* head dim of v, vd, o, do, dv, dvd; 0 = D (the reference takes any K, V <= 256,
                                moda_v14.py:423-437) */
  const int32_t* cu_seqlens_host; /* optional HOST copy of the B + 1 offsets of cu_seqlens (checked against T and
                                     total_tokens), else NULL; see "Packed variable-length batch" above */
} moda_hip_desc;

/*
 * Forward.  Replaces parallel_moda_fwd + parallel_moda_fwd_kernel
 * (moda_v14.py:381-522, 45-378), parallel_moda_chunk_visible_fwd
 * (moda_v16.py:498-633), parallel_fda_fwd (fda_v12.py:261-400) and
 * parallel_attn_fwd (fla/ops/attn/parallel.py:443-503).
 * Writes o (dtype) and lse (fp32, base 2).  k, v NULL iff DEPTH_ONLY;
 * kd, vd NULL iff L == 0.
 */
int moda_hip_fwd(const moda_hip_desc* desc, const void* q, const void* k, const void* v,
                 const void* kd, const void* vd, void* o, float* lse, void* stream);

/*
 * Bytes of device workspace moda_hip_bwd asks for: one fp32 per query row and head (the row sum of
 * o * do of moda_v14.py:525-539, kept in a form private to the library) and, for launches whose key
 * tiles alone would leave compute units idle, fp32 partial sums of dk, dv per row segment (the role of
 * the reference's dk_grouped / dv_grouped buffers, moda_v14.py:1715-1752; added up in a fixed order).
 * Outside chunk-visible mode (head dims up to 128) it also holds the rounded probabilities and dS of every
 * (query row, depth slot) pair, 2 * 2 bytes each, which the dQ kernel leaves for the launch that forms dkd, dvd.
 * A smaller workspace is accepted down to the row sums alone (B * H * G * T * 4 bytes; packed batch:
 * H * G * total_tokens * 4): the backward then uses fewer row segments or none, which changes the fp32
 * summation order of dk, dv, and recomputes the depth scores in the depth-gradient launch (fp32 dot products
 * in place of the matrix products: the same values up to fp32 rounding).  Returns 0 for an invalid descriptor.
 */
size_t moda_hip_bwd_workspace_bytes(const moda_hip_desc* desc);
/* `workspace` below must be 4-byte aligned (MODA_HIP_EALIGN otherwise); the row segments are only used when it is
 * 16-byte aligned as well. */

/*
 * Backward.  Replaces parallel_moda_bwd and its kernels (moda_v14.py:1470-1842,
 * 525-539, 542-871, 874-1248, 1251-1454), parallel_moda_chunk_visible_bwd
 * (moda_v16.py:2099-2343), parallel_fda_bwd (fda_v12.py:881-1135) and
 * parallel_attn_bwd (fla/ops/attn/parallel.py:522-629).
 * Writes every element of dq, dk, dv, dkd, dvd (no pre-zeroing needed; nothing
 * is accumulated with atomics, results are run-to-run identical).
 * dk, dv NULL iff DEPTH_ONLY; dkd, dvd NULL iff L == 0.
 */
int moda_hip_bwd(const moda_hip_desc* desc, const void* q, const void* k, const void* v,
                 const void* kd, const void* vd, const void* o, const float* lse, const void* d_o,
                 void* dq, void* dk, void* dv, void* dkd, void* dvd,
                 void* workspace, size_t workspace_bytes, void* stream);

/*
 * moda_hip_bwd restricted to the stages named in `stages` (an OR of the values
 * below); the stages of one backward must run in the order DELTA, DQ, DKV on
 * one stream (DQ and DKV read the workspace DELTA writes).  Lets a caller skip
 * dK/dV when only dQ is needed, or time the stages separately.  The reference
 * launches the same three steps one after another (moda_v14.py:1609, 1658,
 * 1698-1801).  Which of DQ and DKV writes the depth gradients depends on the
 * shape (outside chunk-visible mode the dQ kernel forms them itself for head
 * dims up to 64 when G divides 32): dkd and dvd are complete once both have run.
 */
enum moda_hip_bwd_stage {
  MODA_HIP_STAGE_DELTA = 1, /* row sums of o * do into the workspace (asked for together with DQ, the dQ kernel forms them) */
  MODA_HIP_STAGE_DQ = 2,    /* dq (and, for some shapes, dkd and dvd: see below) */
  MODA_HIP_STAGE_DKV = 4,   /* dk, dv and, with a depth stream, what is left of dkd, dvd */
  MODA_HIP_STAGE_ALL = 7
};
int moda_hip_bwd_stages(const moda_hip_desc* desc, const void* q, const void* k, const void* v,
                        const void* kd, const void* vd, const void* o, const float* lse, const void* d_o,
                        void* dq, void* dk, void* dv, void* dkd, void* dvd,
                        void* workspace, size_t workspace_bytes, int stages, void* stream);

/*
 * moda_hip_bwd without a workspace argument and without any allocation.  No counterpart in the
 * reference (whose launcher allocates its buffers with torch, moda_v14.py:1609-1652, 1715-1716); it is
 * for callers that cannot allocate device memory: code under stream capture, serving loops and
 * harnesses that forbid hipMalloc.  The row sums of o * do go to a workspace of
 * MODA_HIP_STATIC_WORKSPACE_BYTES that is part of the library's device image (one copy per GPU, held
 * until the process ends): problems with B * H * G * T fp32 values (packed batch: H * G * total_tokens)
 * beyond that size are rejected with MODA_HIP_ESTATIC.  Same kernels as moda_hip_bwd and the same results
 * whenever moda_hip_bwd_workspace_bytes fits the built-in workspace (otherwise dk, dv are summed over fewer
 * row segments, see there).
 * All calls on one GPU share the workspace: calls that may overlap on one GPU (different streams,
 * different host threads) race; serialise them or use moda_hip_bwd with private workspaces.  The first
 * call on a device looks the workspace address up (hipGetSymbolAddress, not a stream operation): under
 * stream capture make one ordinary call first, as for the kernel attribute setup described above.
 */
#define MODA_HIP_STATIC_WORKSPACE_BYTES (8u << 20)
int moda_hip_bwd_static(const moda_hip_desc* desc, const void* q, const void* k, const void* v,
                        const void* kd, const void* vd, const void* o, const float* lse, const void* d_o,
                        void* dq, void* dk, void* dv, void* dkd, void* dvd, void* stream);

/*
 * Depth-KV reorganisation.  Replaces the caller-side
 * torch.stack(dim=2).reshape(B, T*L, H, D).contiguous() of
 * vision_tasks/deit/models.py:361-375 (one call per tensor, K or V).
 * `layers` is a HOST array of n_layers device pointers, each a contiguous
 * [B, T, H, D] tensor; they are written to slots [slot0, slot0 + n_layers) of
 * the token-major cache [B, T*L_total, H, D].  With n_layers == 1 this is the
 * in-place append of one layer's K (or V) into a preallocated cache.
 */
int moda_hip_depth_reorg_fwd(const void* const* layers, int64_t n_layers, int64_t slot0, int64_t L_total,
                             int64_t B, int64_t T, int64_t H, int64_t D, int32_t dtype,
                             void* cache, void* stream);

/*
 * Transpose of the above (the scatter autograd performs for the stack/reshape):
 * splits d_cache [B, T*L_total, H, D] slots [slot0, slot0 + n_layers) into the
 * per-layer gradients d_layers[i] ([B, T, H, D], contiguous, overwritten).
 */
int moda_hip_depth_reorg_bwd(const void* d_cache, int64_t n_layers, int64_t slot0, int64_t L_total,
                             int64_t B, int64_t T, int64_t H, int64_t D, int32_t dtype,
                             void* const* d_layers, void* stream);

/*
 * Which kernels a descriptor runs on: 1 = the matrix-core kernels (tensor rows must then be 16-byte aligned, see
 * the top of this file), 0 = the vector-ALU kernels (element alignment), negative = the descriptor's error code.
 * No counterpart in the reference; lets a host wrapper decide whether an input needs a contiguous copy without
 * repeating the library's rule.  Touches no device.
 */
int moda_hip_uses_matrix_cores(const moda_hip_desc* desc);

/* Human-readable text for an error code (static storage). */
const char* moda_hip_strerror(int code);

/* MODA_HIP_VERSION the library was built with. */
int moda_hip_version(void);

#ifdef __cplusplus
}
#endif
#endif /* MODA_HIP_H_ */
