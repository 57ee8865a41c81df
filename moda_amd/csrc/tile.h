// Device-side building blocks shared by the gfx950 attention kernels:
// 16-bit element types, MFMA 32x32x16 wrappers, the swizzled LDS tile layout
// and its two read patterns (row operand, transposed operand).
#pragma once
#include <hip/hip_runtime.h>

#include <atomic>
#include <stdint.h>

namespace moda {

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

struct BF16 {
  typedef bf16x8 vec8;
  typedef bf16x4 vec4;
  typedef __bf16 elem;
};
struct FP16 {
  typedef f16x8 vec8;
  typedef f16x4 vec4;
  typedef _Float16 elem;
};

#define MODA_LDS __attribute__((address_space(3)))
typedef MODA_LDS uint16_t* lds_ptr;        // LDS tile pointer (32-bit, address space 3)
typedef MODA_LDS const uint16_t* lds_cptr;

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kNegInf = -__builtin_huge_valf();

// D(32x32) += A(32x16) * B(16x32).  Operand layout per lane l (n = l & 31,
// g = l >> 5): A holds row n, k = 8g..8g+7; B holds column n, k = 8g..8g+7;
// the accumulator holds column n, rows (i/4)*8 + 4g + (i%4) for i = 0..15.
template <typename T>
__device__ __forceinline__ f32x16 mfma32(i32x4 a, i32x4 b, f32x16 c);
template <>
__device__ __forceinline__ f32x16 mfma32<BF16>(i32x4 a, i32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0,
                                                 0, 0);
}
template <>
__device__ __forceinline__ f32x16 mfma32<FP16>(i32x4 a, i32x4 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0,
                                                0);
}

// Row index inside a 32-row accumulator block that register i of lane-half g holds.
__device__ __forceinline__ constexpr int acc_row(int i, int g) { return (i >> 2) * 8 + g * 4 + (i & 3); }

// fp32 -> 16-bit packs (round to nearest even).
template <typename T>
__device__ __forceinline__ int pack2(float a, float b);
template <>
__device__ __forceinline__ int pack2<BF16>(float a, float b) {
  bf16x2 v;
  v[0] = (__bf16)a;
  v[1] = (__bf16)b;
  return __builtin_bit_cast(int, v);
}
template <>
__device__ __forceinline__ int pack2<FP16>(float a, float b) {
  f16x2 v;
  v[0] = (_Float16)a;
  v[1] = (_Float16)b;
  return __builtin_bit_cast(int, v);
}

// One packed pair of 16-bit values -> fp32.
template <typename T>
__device__ __forceinline__ void unpack2(int w, float& lo, float& hi);
template <>
__device__ __forceinline__ void unpack2<BF16>(int w, float& lo, float& hi) {
  lo = __builtin_bit_cast(float, w << 16);
  hi = __builtin_bit_cast(float, w & 0xffff0000);
}
template <>
__device__ __forceinline__ void unpack2<FP16>(int w, float& lo, float& hi) {
  const f16x2 v = __builtin_bit_cast(f16x2, w);
  lo = (float)v[0];
  hi = (float)v[1];
}

// Eight consecutive accumulator registers -> one MFMA B operand (k slots 0..7).
template <typename T>
__device__ __forceinline__ i32x4 pack8(const f32x16& x, int first) {
  i32x4 r;
  r[0] = pack2<T>(x[first + 0], x[first + 1]);
  r[1] = pack2<T>(x[first + 2], x[first + 3]);
  r[2] = pack2<T>(x[first + 4], x[first + 5]);
  r[3] = pack2<T>(x[first + 6], x[first + 7]);
  return r;
}

template <typename T>
__device__ __forceinline__ float to_float(typename T::elem x) {
  return (float)x;
}

// ---------------------------------------------------------------------------
// LDS tile: ROWS x HD 16-bit elements, row-major, 16-byte chunks XOR-swizzled
// so that (a) 16 consecutive rows at one logical chunk and (b) 4 consecutive
// rows x 4 adjacent chunks both spread over all banks.
// ---------------------------------------------------------------------------
template <int HD>
struct Tile {
  static constexpr int CH = HD / 8;  // 16-byte chunks per row
  // Rows of 256 bytes and more start at bank 0 each, so all four low row bits go into the chunk index.  A 128-byte
  // row (HD = 64) covers half the banks and odd rows the other half: there row bits 1..3 choose among the eight
  // chunks, bit 1 on top so that rows r and r + 2 of a four-row, four-chunk transposed read land in different
  // halves of the row.  (Measured with SQ_LDS_BANK_CONFLICT on all four operand read patterns: 0 for HD = 64,
  // 128 and 256; the first formula cut to three bits cost HD = 64 a second pass on every read.)
  __host__ __device__ __forceinline__ static int swz(int row) {
    return CH == 8 ? ((((row >> 1) & 1) << 2) | ((row >> 2) & 3)) : ((((row & 3) << 2) | ((row >> 2) & 3)) & (CH - 1));
  }
  // element offset of logical (row, chunk)
  __host__ __device__ __forceinline__ static int off(int row, int chunk) { return row * HD + ((chunk ^ swz(row)) << 3); }
};

// Per-lane LDS offsets of the two operand read patterns, computed once.  Tile
// rows are only ever offset by multiples of 16, which leaves the swizzle of a
// lane's row unchanged, so every read is `tile + precomputed + compile-time constant`.
//
// Row operand: lane (n, g) gets elements [16*kk + 8g, +8) of tile row (row0 + n).
// Serves as MFMA A (M = tile rows) or B (N = tile rows) with K = head dim.
//
// Transposed operand: lane (n, g) gets, for head-dim column d = 32*dblk + n,
// tile rows rb + 4g + {0,1,2,3} (k slots 0..3) and rb + 8 + 4g + {0,1,2,3}
// (k slots 4..7) -- exactly the rows that accumulator registers 8s..8s+7 of a
// 32-row block hold, so a packed accumulator can be the other operand.
// Uses the gfx950 LDS transpose read: within each 16-lane group, source lane
// r supplies the address of 4 consecutive elements; result lane i receives
// element (i & 3) of source lanes 4j + (i >> 2), j = 0..3.
template <int HD>
struct OperandAddr {
  static constexpr int KK = HD / 16, DB = HD / 32;
  int row[KK];
  int tr[2][DB];

  __device__ __forceinline__ void init(int lane) {
    const int n = lane & 31, g = lane >> 5, r16 = lane & 15;
#pragma unroll
    for (int kk = 0; kk < KK; kk++) row[kk] = Tile<HD>::off(n, 2 * kk + g);
#pragma unroll
    for (int hi = 0; hi < 2; hi++)
#pragma unroll
      for (int d = 0; d < DB; d++) {
        const int r = 4 * g + (r16 >> 2) + 8 * hi;
        const int dcol = 32 * d + ((lane >> 4) & 1) * 16 + (r16 & 3) * 4;
        tr[hi][d] = Tile<HD>::off(r, dcol >> 3) + (dcol & 7);
      }
  }
  // row0 must be a multiple of 16
  __device__ __forceinline__ i32x4 row_operand(lds_cptr tile, int row0, int kk) const {
    return *reinterpret_cast<MODA_LDS const i32x4*>(tile + row[kk] + row0 * HD);
  }
  // rb must be a multiple of 16
  __device__ __forceinline__ i32x4 tr_operand(lds_cptr tile, int rb, int dblk) const {
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((MODA_LDS s16x4*)(tile + tr[0][dblk] + rb * HD));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((MODA_LDS s16x4*)(tile + tr[1][dblk] + rb * HD));
    i32x2 l2 = __builtin_bit_cast(i32x2, lo);
    i32x2 h2 = __builtin_bit_cast(i32x2, hi);
    i32x4 r;
    r[0] = l2[0];
    r[1] = l2[1];
    r[2] = h2[0];
    r[3] = h2[1];
    return r;
  }
};

// Software-pipelined MFMA sequences.  The compiler, left alone, issues each LDS
// operand read immediately before the MFMA that consumes it and so exposes the
// full LDS latency once per MFMA; these helpers keep DEPTH operand reads in
// flight ahead of the matrix pipe and pin that order with scheduling barriers.
// Consecutive MFMAs always target different accumulators.

// Every helper takes an optional hook, called as hook(j) right after the j-th MFMA has been issued
// (j is a constant after unrolling): a place to slip other instructions -- the next tile's
// global -> LDS loads -- into the stream at a fixed position.
struct NoHook {
  __device__ __forceinline__ void operator()(int) const {}
};

// acc[bb] = sum_kk rows(tile, 32*bb + n, kk) x breg[kk]   (accumulators start at zero)
template <typename T, int HD, int NB, int DEPTH, typename Hook = NoHook>
__device__ __forceinline__ void mfma_rows(const OperandAddr<HD>& oa, lds_cptr tile, const i32x4 (&breg)[HD / 16],
                                          f32x16 (&acc)[NB], Hook&& hook = Hook{}) {
  constexpr int KK = HD / 16, N = NB * KK;
  i32x4 ops[N];
#pragma unroll
  for (int j = 0; j < DEPTH && j < N; j++) ops[j] = oa.row_operand(tile, 32 * (j % NB), j / NB);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int j = 0; j < N; j++) {
    if (j + DEPTH < N) ops[j + DEPTH] = oa.row_operand(tile, 32 * ((j + DEPTH) % NB), (j + DEPTH) / NB);
    const int bb = j % NB, kk = j / NB;
    if (kk == 0) {
      f32x16 z;
#pragma unroll
      for (int i = 0; i < 16; i++) z[i] = 0.f;
      acc[bb] = mfma32<T>(ops[j], breg[kk], z);
    } else {
      acc[bb] = mfma32<T>(ops[j], breg[kk], acc[bb]);
    }
    __builtin_amdgcn_sched_barrier(0);
    hook(j);
  }
}

// acc[bb] += sum_kk rows(tile, 32*bb + n, kk) x breg[kk]   (accumulators preset by the caller)
template <typename T, int HD, int NB, int DEPTH, typename Hook = NoHook>
__device__ __forceinline__ void mfma_rows_acc(const OperandAddr<HD>& oa, lds_cptr tile, const i32x4 (&breg)[HD / 16],
                                              f32x16 (&acc)[NB], Hook&& hook = Hook{}) {
  constexpr int KK = HD / 16, N = NB * KK;
  i32x4 ops[N];
#pragma unroll
  for (int j = 0; j < DEPTH && j < N; j++) ops[j] = oa.row_operand(tile, 32 * (j % NB), j / NB);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int j = 0; j < N; j++) {
    if (j + DEPTH < N) ops[j + DEPTH] = oa.row_operand(tile, 32 * ((j + DEPTH) % NB), (j + DEPTH) / NB);
    acc[j % NB] = mfma32<T>(ops[j], breg[j / NB], acc[j % NB]);
    __builtin_amdgcn_sched_barrier(0);
    hook(j);
  }
}

// acc[d] += tr(tile, 16*ks, d) x breg[ks]  for ks < NKS, d < HD/32.  prefetch() may be
// called early (before the code that produces breg) to have the first operands waiting.
template <typename T, int HD, int NKS, int DEPTH>
struct TrPipe {
  static constexpr int DB = HD / 32, N = NKS * DB;
  i32x4 ops[N];
  __device__ __forceinline__ void prefetch(const OperandAddr<HD>& oa, lds_cptr tile) {
#pragma unroll
    for (int j = 0; j < DEPTH && j < N; j++) ops[j] = oa.tr_operand(tile, 16 * (j / DB), j % DB);
    __builtin_amdgcn_sched_barrier(0);
  }
  template <typename Hook = NoHook>
  __device__ __forceinline__ void run(const OperandAddr<HD>& oa, lds_cptr tile, const i32x4 (&breg)[NKS],
                                      f32x16 (&acc)[DB], Hook&& hook = Hook{}) {
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < N; j++) {
      if (j + DEPTH < N) ops[j + DEPTH] = oa.tr_operand(tile, 16 * ((j + DEPTH) / DB), (j + DEPTH) % DB);
      acc[j % DB] = mfma32<T>(ops[j], breg[j / DB], acc[j % DB]);
      __builtin_amdgcn_sched_barrier(0);
      hook(j);
    }
  }
};

// Host side: raise a kernel's dynamic-LDS limit, once per device (the attribute belongs to the device's
// copy of the kernel, so a process that drives several GPUs needs it on each of them).  `state` is a
// static of the calling launcher, one per kernel instantiation.
struct LdsAttrState {
  std::atomic<uint64_t> devices{0};
};
inline hipError_t allow_dynamic_lds(LdsAttrState& state, const void* kernel, size_t bytes) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  const bool tracked = dev >= 0 && dev < 64;
  const uint64_t bit = tracked ? (1ull << dev) : 0;
  if (tracked && (state.devices.load(std::memory_order_acquire) & bit)) return hipSuccess;
  e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  if (e == hipSuccess && tracked) state.devices.fetch_or(bit, std::memory_order_release);
  return e;
}

// One wave-wide direct global -> LDS load: lane l's BYTES bytes (16 or 4) land at lds_byte_addr +
// l * BYTES; the global side is a raw buffer (descriptor rsrc, per-lane byte offset voff, scalar
// byte offset soff) whose range check zero-fills lanes past the end.  Issued as inline assembly on
// purpose: the compiler's wait-count pass does not see these loads, so it does not stall every
// later LDS read (in particular the transpose reads) on vmcnt(0) while the NEXT tiles are still in
// flight.  Completion is the caller's business: s_waitcnt vmcnt via wait_all()/wait_but<>() and a
// workgroup barrier before any wave reads the tile.  The compiler's own vmcnt waits stay correct
// because vector-memory loads return in order and an unseen younger load only makes them stricter.
// The compiler's hazard pass does not look inside inline assembly either: a vector-memory instruction
// that reads a scalar register written by a vector-ALU instruction (v_readfirstlane, v_readlane of a
// spilled scalar) fewer than five wait states earlier sees the register's OLD value.  The compiler places
// such writes right in front of the block when scalar registers are short (the forward kernels: dozens of sites),
// so the block brings its own wait states: s_mov (1) + s_nop 3 (4), which also covers the one wait state m0 needs.
// NOP = 0 (the loaders' last template argument, or MODA_DMA_NOP defined as 0 before this header) leaves only the
// one wait state m0 needs and is for experiments: whether the compiled code keeps its distance by itself changes
// with unrelated edits (one more spilled scalar somewhere), so every kernel of the library keeps the wait states
// -- about 0.3 % of the long-sequence step -- and tests/test_inline_asm_hazards_cpu.py checks every tile load of
// every kernel in the compiler's output.
#ifndef MODA_DMA_NOP
#define MODA_DMA_NOP 3
#endif
template <int BYTES, int NOP = MODA_DMA_NOP>
__device__ __forceinline__ void lds_dma(i32x4 rsrc, uint32_t lds_byte_addr, int voff, int soff) {
  static_assert(BYTES == 16 || BYTES == 4, "dwordx4 or dword");
  static_assert(NOP == 0 || NOP == 3, "one wait state for m0, or five for scalars written by the vector ALU");
  // The scalar operands are wave-uniform by contract.  Under scalar-register pressure the compiler may
  // park such a value in a vector register and would then hand that register to the "s" operands
  // below; reading it back through readfirstlane (free when the value already sits in a scalar
  // register) keeps the operands legal.
  const uint32_t m0v = (uint32_t)__builtin_amdgcn_readfirstlane((int)lds_byte_addr);
  const int so = __builtin_amdgcn_readfirstlane(soff);
  i32x4 rs;
  rs[0] = __builtin_amdgcn_readfirstlane(rsrc[0]);
  rs[1] = __builtin_amdgcn_readfirstlane(rsrc[1]);
  rs[2] = __builtin_amdgcn_readfirstlane(rsrc[2]);
  rs[3] = __builtin_amdgcn_readfirstlane(rsrc[3]);
  if (BYTES == 16 && NOP == 3)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(m0v), "v"(voff), "s"(rs), "s"(so)
                 : "memory", "m0");
  else if (BYTES == 16)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(m0v), "v"(voff), "s"(rs), "s"(so)
                 : "memory", "m0");
  else if (NOP == 3)
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 3\n\tbuffer_load_dword %1, %2, %3 offen lds"
                 :
                 : "s"(m0v), "v"(voff), "s"(rs), "s"(so)
                 : "memory", "m0");
  else
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds"
                 :
                 : "s"(m0v), "v"(voff), "s"(rs), "s"(so)
                 : "memory", "m0");
}

// The four descriptor words of a raw buffer over `nbytes` bytes at `base` (wave-uniform).
__device__ __forceinline__ i32x4 rsrc_words(const void* base, uint32_t nbytes) {
  const uint64_t p = (uint64_t)base;
  i32x4 r;
  r[0] = __builtin_amdgcn_readfirstlane((int)(uint32_t)p);
  r[1] = __builtin_amdgcn_readfirstlane((int)((uint32_t)(p >> 32) & 0xffffu));
  r[2] = __builtin_amdgcn_readfirstlane((int)nbytes);
  r[3] = 0x00020000;
  return r;
}

__device__ __forceinline__ uint32_t lds_addr(lds_cptr p) { return (uint32_t)(uintptr_t)p; }

// Global -> LDS staging without registers: gfx950 `buffer_load_dwordx4 ... lds`.
// One wave-wide load fills 64 consecutive 16-byte LDS slots (lane l -> slot l);
// the XOR swizzle is therefore applied on the GLOBAL side: the lane that owns
// physical chunk p of a row fetches logical chunk p ^ swz(row).  Rows past the
// end of the source are zero-filled by the buffer range check.  The loads are
// asynchronous: call wait_all() before the barrier that publishes the tile.
// Byte offset of a lane whose chunk lies beyond the tensor's head dim (head dims below the tile width run
// zero-padded): past the end of every descriptor, so the range check fills the chunk with zeros.
constexpr int kPadOffset = 0x7ffffff0;

// Depth tiles when only Lv of a token's L slots hold data: the tile's columns are counted on the compact axis
// (column c = token * Lv + slot, see geometry.h) and lie in rows token * L + slot of the tensor.  The loaders anchor
// one descriptor at slot 0 of the first column's token; this is the row, relative to that anchor, of the tile's
// row `rho`, given the first column's slot l0.
__host__ __device__ __forceinline__ int mapped_row(int l0, int rho, int L, int Lv) {
  const int l = l0 + rho, dw = l / Lv;
  return dw * L + (l - dw * Lv);
}
// bytes the anchored descriptor covers: from the anchor row to the end of the slice (rows_total rows), capped
__host__ __device__ __forceinline__ uint32_t mapped_bytes(int64_t anchor_row, int64_t rows_total, uint32_t stride_bytes) {
  const int64_t left = (rows_total - anchor_row) * (int64_t)stride_bytes;
  return left <= 0 ? 0u : left > 0x7fffffffll ? 0x7fffffffu : (uint32_t)left;
}

template <int HD, int ROWS, int NT, int NOP = MODA_DMA_NOP>
struct AsyncTileLoader {
  static constexpr int CH = HD / 8;            // 16-byte chunks per row
  static constexpr int NW = NT / 64;           // waves
  static constexpr int RPW = 64 / CH;          // rows per wave-wide load
  static constexpr int N = ROWS / (RPW * NW);  // loads per wave
  static_assert(ROWS % (RPW * NW) == 0 && (RPW * NW) % 16 == 0, "tile must divide evenly");
  int row_in_pass;  // row of this lane within one pass over the tile
  int gchunk;       // logical chunk this lane fetches
  int wave;

  __host__ __device__ __forceinline__ void init(int tid) {
    const int lane = tid & 63;
#if defined(__HIP_DEVICE_COMPILE__)
    wave = __builtin_amdgcn_readfirstlane(tid >> 6);
#else
    wave = tid >> 6;
#endif
    row_in_pass = wave * RPW + lane / CH;
    gchunk = (lane % CH) ^ Tile<HD>::swz(row_in_pass);
  }
  // whether this lane's chunk lies past a tensor's head dim `d` (a multiple of 8 not above HD): such lanes fetch
  // out of range and receive zeros
  __host__ __device__ __forceinline__ bool pads(int d) const { return gchunk * 8 >= d; }
  // this lane's byte offset inside a tile of a tensor of head dim `d` whose rows are `stride_bytes` apart
  __host__ __device__ __forceinline__ int lane_offset(int stride_bytes, int d) const {
    return pads(d) ? kPadOffset : row_in_pass * stride_bytes + gchunk * 16;
  }
  // the i-th of a wave's N loads of a tile: element offset of the 64 LDS slots it fills, tile rows it skips
  __host__ __device__ __forceinline__ int lds_elems(int i) const { return (i * NW + wave) * 512; }
  __host__ __device__ __forceinline__ static constexpr int rows_before(int i) { return i * NW * RPW; }
  // A source of rows: fixed descriptor over rows [row_base, row_end) of a (batch, head) slice whose
  // byte span fits 31 bits (kernels that may meet wider slices use load() below, which anchors a
  // descriptor at every tile at the price of 64-bit address arithmetic per tile).
  struct Source {
    const uint16_t* base;  // row `row_base` of the slice
    uint32_t nbytes;       // bytes from there to the end of the slice
    int voff;              // this lane's byte offset inside a tile
    int stride_bytes;
    int row_base;
  };
  __host__ __device__ __forceinline__ Source source(const uint16_t* slice, int64_t row_stride, int row_base, int row_end,
                                                    int d) const {
    Source s;
    s.stride_bytes = (int)row_stride * 2;
    s.row_base = row_base;
    const int64_t nbytes = (int64_t)(row_end > row_base ? row_end - row_base : 0) * s.stride_bytes;
    s.base = slice + (int64_t)row_base * row_stride;
    s.nbytes = nbytes > 0x7fffffffll ? 0x7fffffffu : (uint32_t)nbytes;
    s.voff = lane_offset(s.stride_bytes, d);
    return s;
  }
  // rows [row0, row0 + ROWS) of the source into `tile`; rows past the source's end arrive as zeros
  // scalar byte offset of load i of the tile that starts at row `row0` of the source
  __host__ __device__ __forceinline__ static int source_soffset(const Source& s, int row0, int i) {
    return (row0 - s.row_base + rows_before(i)) * s.stride_bytes;
  }
  __device__ __forceinline__ void load_from(lds_ptr tile, const Source& s, int row0) const {
    const i32x4 rs = rsrc_words(s.base, s.nbytes);
#pragma unroll
    for (int i = 0; i < N; i++) lds_dma<16, NOP>(rs, lds_addr(tile + lds_elems(i)), s.voff, source_soffset(s, row0, i));
  }
  // bytes covered by the descriptor load() anchors at row `row0` of a slice that ends at row `row_end`
  __host__ __device__ __forceinline__ static uint32_t anchored_bytes(int64_t row_stride, int row0, int row_end) {
    const int rows_left = row_end - row0;
    const uint32_t stride_bytes = (uint32_t)row_stride * 2u;
    return rows_left <= 0 ? 0u : (uint32_t)(rows_left < ROWS ? rows_left : ROWS) * stride_bytes;
  }
  __device__ __forceinline__ void load(lds_ptr tile, const uint16_t* src, int64_t row_stride, int row0, int row_end,
                                       int d) const {
    const uint32_t stride_bytes = (uint32_t)row_stride * 2u;
    const i32x4 rs = rsrc_words(src + (int64_t)row0 * row_stride, anchored_bytes(row_stride, row0, row_end));
    const int voff = lane_offset((int)stride_bytes, d);
#pragma unroll
    for (int i = 0; i < N; i++) lds_dma<16, NOP>(rs, lds_addr(tile + lds_elems(i)), voff, rows_before(i) * (int)stride_bytes);
  }
  // this lane's byte offset, relative to the anchor, in load i of a mapped depth tile (see mapped_row)
  __host__ __device__ __forceinline__ int mapped_offset(int i, int l0, int L, int Lv, int stride_bytes, int d) const {
    return pads(d) ? kPadOffset : mapped_row(l0, rows_before(i) + row_in_pass, L, Lv) * stride_bytes + gchunk * 16;
  }
  // compact depth columns [col0, col0 + ROWS) of a slice of rows_total rows with L slots per token, Lv of them filled
  __device__ __forceinline__ void load_mapped(lds_ptr tile, const uint16_t* slice, int64_t row_stride, int col0,
                                              int64_t rows_total, int L, int Lv, int d) const {
    const int w0 = __builtin_amdgcn_readfirstlane(col0 / Lv), l0 = col0 - w0 * Lv;
    const uint32_t stride_bytes = (uint32_t)row_stride * 2u;
    const int64_t anchor = (int64_t)w0 * L;
    const i32x4 rs = rsrc_words(slice + anchor * row_stride, mapped_bytes(anchor, rows_total, stride_bytes));
#pragma unroll
    for (int i = 0; i < N; i++)
      lds_dma<16, NOP>(rs, lds_addr(tile + lds_elems(i)), mapped_offset(i, l0, L, Lv, (int)stride_bytes, d), 0);
  }
  // s_waitcnt vmcnt(0): every outstanding vector-memory load of this wave has landed
  __device__ __forceinline__ static void wait_all() { __builtin_amdgcn_s_waitcnt(0x0F70); }
  // s_waitcnt vmcnt(K): at most K of this wave's vector-memory loads (the youngest ones) still in flight
  template <int K>
  __device__ __forceinline__ static void wait_but() {
    static_assert(K >= 0 && K < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (K & 15) | ((K >> 4) << 14));
  }
};

// A 32-row tile that ONE wave stages for itself (same swizzled layout, same zero fill past the end of the
// source and past the tensors' head dim).  Nothing but the wave's own counters orders these loads: wait for
// vmcnt before reading the tile, and for lgkmcnt(0) -- all LDS reads returned -- before loading over it.
template <int HD, int NOP = MODA_DMA_NOP>
struct WaveTileLoader {
  static constexpr int CH = HD / 8, RPW = 64 / CH, N = 32 / RPW;  // chunks per row, rows per load, loads per tile
  int prow, pch;
  __host__ __device__ __forceinline__ void init(int lane) {
    prow = lane / CH;
    pch = lane % CH;
  }
  // this lane's byte offset in load i of a tile (rows `stride_bytes` apart, head dim `d`): its tile row is i * RPW + prow
  __host__ __device__ __forceinline__ int lane_offset(int i, int stride_bytes, int d) const {
    const int row = i * RPW + prow;
    const int lch = pch ^ Tile<HD>::swz(row);
    return lch * 8 < d ? row * stride_bytes + lch * 16 : kPadOffset;
  }
  // rows [row0, row0 + nrows) of the slice at `base` (nrows <= 32; the rest of the tile arrives as zeros)
  __device__ __forceinline__ void fetch(lds_ptr tile, const uint16_t* base, int64_t row_stride, int64_t row0, int nrows,
                                        int d) const {
    const uint32_t stride_bytes = (uint32_t)row_stride * 2u;
    const i32x4 rs = rsrc_words(base + row0 * row_stride, nrows > 0 ? (uint32_t)nrows * stride_bytes : 0u);
#pragma unroll
    for (int i = 0; i < N; i++) lds_dma<16, NOP>(rs, lds_addr(tile + i * 512), lane_offset(i, (int)stride_bytes, d), 0);
  }
  // the same for a mapped depth tile (see mapped_row): offset relative to the anchor, rows >= nrows padded
  __host__ __device__ __forceinline__ int mapped_offset(int i, int l0, int L, int Lv, int nrows, int stride_bytes, int d) const {
    const int row = i * RPW + prow;
    const int lch = pch ^ Tile<HD>::swz(row);
    return (lch * 8 < d && row < nrows) ? mapped_row(l0, row, L, Lv) * stride_bytes + lch * 16 : kPadOffset;
  }
  // compact depth columns [col0, col0 + nrows) of a slice of rows_total rows, L slots per token, Lv of them filled
  __device__ __forceinline__ void fetch_mapped(lds_ptr tile, const uint16_t* slice, int64_t row_stride, int col0,
                                               int nrows, int64_t rows_total, int L, int Lv, int d) const {
    const int w0 = __builtin_amdgcn_readfirstlane(col0 / Lv), l0 = col0 - w0 * Lv;
    const uint32_t stride_bytes = (uint32_t)row_stride * 2u;
    const int64_t anchor = (int64_t)w0 * L;
    const i32x4 rs = rsrc_words(slice + anchor * row_stride, nrows > 0 ? mapped_bytes(anchor, rows_total, stride_bytes) : 0u);
#pragma unroll
    for (int i = 0; i < N; i++)
      lds_dma<16, NOP>(rs, lds_addr(tile + i * 512), mapped_offset(i, l0, L, Lv, nrows, (int)stride_bytes, d), 0);
  }
  // at most K of this wave's vector-memory loads (the youngest) still in flight
  template <int K>
  __device__ __forceinline__ static void wait_but() {
    static_assert(K >= 0 && K < 64, "vmcnt is a 6-bit counter");
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0x0F70 | (K & 15) | ((K >> 4) << 14));
    asm volatile("" ::: "memory");
  }
  // every LDS read of this wave has returned
  __device__ __forceinline__ static void reads_done() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0xC07F);
    asm volatile("" ::: "memory");
  }
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Combine a value with the one held by lane ^ 32 (the other half of the lane pair that shares a
// row or column) using the gfx950 half-wave swap: {r0, r1} = {x[lane], x[lane ^ 32]} in every lane.
__device__ __forceinline__ float pair_max(float x) {
#if defined(__HIP_DEVICE_COMPILE__)
  const int xi = __builtin_bit_cast(int, x);
  auto r = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);
  return fmaxf(__builtin_bit_cast(float, (int)r[0]), __builtin_bit_cast(float, (int)r[1]));
#else
  return x;  // host pass of the single-source compile: never executed
#endif
}
__device__ __forceinline__ float pair_sum(float x) {
#if defined(__HIP_DEVICE_COMPILE__)
  const int xi = __builtin_bit_cast(int, x);
  auto r = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);
  return __builtin_bit_cast(float, (int)r[0]) + __builtin_bit_cast(float, (int)r[1]);
#else
  return x;  // host pass of the single-source compile: never executed
#endif
}

}  // namespace moda
