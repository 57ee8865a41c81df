// Index arithmetic of the attention kernels: which rows and columns a workgroup, a wave and a lane touch.
// Everything here is plain integer code marked for host and device, shared by the kernels, their host
// launchers and the host-side address walker of the test suite (tests/address_walker.cpp), which replays
// every descriptor, load and store of a launch on the CPU and checks them against the tensor extents.
#pragma once
#include "kargs.h"

#define MODA_HD __host__ __device__ __forceinline__

namespace moda {

MODA_HD int imin(int a, int b) { return a < b ? a : b; }
MODA_HD int imax(int a, int b) { return a > b ? a : b; }

// Depth columns.  A depth tensor holds L slots per token (row t * L + l = slot l of token t) of which the first
// Lv hold data.  The kernels count depth columns on the COMPACT axis of the slots that hold data: column
// c = t * Lv + l; slots l >= Lv are never read.  With Lv == L (every slot filled) the compact axis is the row axis.
MODA_HD int64_t depth_row_of(const KArgs& a, int c) {
  if (a.Lv == a.L) return c;
  const int t = c / a.Lv;
  return (int64_t)t * a.L + (c - t * a.Lv);
}

// ---------------------------------------------------------------------------------------------------
// Query-row kernels (forward, dQ): a workgroup owns BM consecutive query rows of one (batch, query head)
// and streams BN-column tiles: the sequence keys, then (when they go through the workgroup's ring) the
// depth columns its rows can see.
// ---------------------------------------------------------------------------------------------------

// Query tile of workgroup `block` (heavy, late tiles first).  In a variable-length batch the grid counts tiles
// from the end of the longest sequence (Tq_longest), so that tiles of equal cost of all sequences are dispatched
// together; a result >= the sequence's own tile count means the workgroup has nothing to do.
MODA_HD int query_tile_of(int block, int BH, int BM, int Tq_grid) { return (Tq_grid + BM - 1) / BM - 1 - block / BH; }

// Visible column intervals [0, shi) of the sequence keys and [dlo, dhi) of the depth columns (compact axis) for
// query row r (all zero for a row past the end).  Ld: depth slots per token, 0 when the launch has no depth stream.
struct RowVis {
  int shi, dlo, dhi;
};
MODA_HD RowVis row_visibility(const KArgs& a, int r, int Ld) {
  RowVis v = {0, 0, 0};
  if (r < a.Tq) {
    const int t = r / a.Gf;
    if (a.has_seq) v.shi = a.causal ? t + 1 : a.T;
    if (Ld > 0) {
      const int lo_t = a.chunk ? (t / a.Cb) * a.Cb : t;
      v.dlo = lo_t * a.Lv;
      v.dhi = (t + 1) * a.Lv;
    }
  }
  return v;
}

// Depth columns a wave alone can see (always outside chunk-visible mode, and in it when a chunk's rows fit a
// wave pair) are not streamed through the workgroup's ring: each wave fetches its own rows' span.
MODA_HD bool waves_own_depth(const KArgs& a, int Ld) { return Ld > 0 && (!a.chunk || a.Cb * a.Gf <= 64); }

// Outside chunk-visible mode a depth slot is seen by the Gf query rows of its own token only.  When those rows
// always sit in one wave of the dQ kernel (32 rows per wave, Gf divides 32) the dQ kernel can form the slots' dK
// and dV while their K and V rows are in its LDS tiles: no other wave contributes to them, and the depth stream is
// read once per backward instead of twice.  Done for the 64-wide tiles only -- there the extra operands (Q^T and
// dO^T of the wave's rows) fit the register file next to the dQ accumulators, and the shapes that use them are
// bound by memory traffic; on the 128-wide tiles the same code spills and was measured slower than the separate
// depth-column kernel, which every other case runs from the dK/dV launch.
constexpr int kDepthGradsInDqMaxWidth = 64;
MODA_HD bool depth_grads_in_dq(const KArgs& a, int HD) {
  return a.L > 0 && !a.chunk && HD <= kDepthGradsInDqMaxWidth && 32 % a.Gf == 0;
}

// ... and where the dQ kernel's waves walk their own depth columns without forming the gradients (the 128-wide tiles,
// or a query group that does not divide a wave), they can at least hand their rounded P and dS of the (row, slot)
// pairs to the depth-column kernel through the workspace (KArgs::depth_p), which then skips reading kd, vd and
// recomputing the scores.
MODA_HD bool depth_scores_from_dq(const KArgs& a, int HD) {
  return a.L > 0 && !a.chunk && HD <= 128 && !depth_grads_in_dq(a, HD);
}

// The column tiles of query tile qt: n_seq sequence tiles, of which the first n_full are seen completely by every
// row of the workgroup, then n_dep depth tiles starting at flattened depth column dep0 (ring_depth: the depth
// columns go through the ring at all).
struct RowTilePlan {
  int n_seq, n_full, dep0, n_dep;
};
MODA_HD RowTilePlan row_tile_plan(const KArgs& a, int qt, int BM, int BN, bool ring_depth) {
  RowTilePlan p = {0, 0, 0, 0};
  const int r_first = qt * BM;
  const int r_last = imin(a.Tq, r_first + BM) - 1;
  const int t_first = r_first / a.Gf, t_last = r_last / a.Gf;
  if (a.has_seq) {
    p.n_seq = ((a.causal ? t_last + 1 : a.T) + BN - 1) / BN;
    // padding rows of the last workgroup compute on zero queries in the full tiles and are never stored
    p.n_full = imin(p.n_seq, (a.causal ? t_first + 1 : a.T) / BN);
  }
  if (ring_depth) {
    const int lo_t = a.chunk ? (t_first / a.Cb) * a.Cb : t_first;
    p.dep0 = lo_t * a.Lv;
    p.n_dep = ((t_last + 1) * a.Lv - p.dep0 + BN - 1) / BN;
  }
  return p;
}
// first row (sequence key or flattened depth column) of ring tile `it`
MODA_HD int ring_tile_row0(const RowTilePlan& p, int it, int BN) {
  return it < p.n_seq ? it * BN : p.dep0 + (it - p.n_seq) * BN;
}

// Depth columns [c_beg, c_end) that the `rows` query rows starting at rw0 (< Tq) can see.
struct DepthSpan {
  int c_beg, c_end;
};
MODA_HD DepthSpan own_depth_span(const KArgs& a, int rw0, int rows) {
  const int tw0 = rw0 / a.Gf, tw1 = (imin(a.Tq, rw0 + rows) - 1) / a.Gf;
  DepthSpan s;
  s.c_beg = (a.chunk ? (tw0 / a.Cb) * a.Cb : tw0) * a.Lv;
  s.c_end = (tw1 + 1) * a.Lv;
  return s;
}

// ---------------------------------------------------------------------------------------------------
// Column kernel (dK/dV): a workgroup owns BN columns -- sequence keys or flattened depth columns -- of one
// (batch, kv head) and streams BM-row query tiles from the last visible one down.
// ---------------------------------------------------------------------------------------------------

// visible query-row interval [lo, hi) of a column
MODA_HD void q_interval(const KArgs& a, bool dep, int col, int& lo, int& hi) {
  if (!dep) {
    lo = a.causal ? col * a.Gf : 0;
    hi = a.Tq;
  } else {
    const int w = col / a.Lv;
    lo = w * a.Gf;
    hi = a.chunk ? imin(a.T, (w / a.Cb + 1) * a.Cb) * a.Gf : (w + 1) * a.Gf;
  }
}

// What column-tile workgroup `ct` of a (batch, kv head) does.  `grid`: the launch's argument block (T of the
// longest sequence), `a`: the one rebased on the workgroup's sequence; nseg: row segments per sequence tile.
struct ColTilePlan {
  bool active;  // false: a tile beyond this sequence of a variable-length batch
  bool dep;     // depth columns (else sequence keys)
  int ncols;    // columns of the (batch, head): T or T * L
  int seg;      // row segment of a split sequence tile
  int c_first;  // first column
  int qt0, nqt; // query tiles qt0 .. qt0 + nqt - 1 (BM rows each), streamed from the last one down
};
MODA_HD ColTilePlan col_tile_plan(const KArgs& grid, const KArgs& a, int ct, int BN, int BM, bool varlen, int nseg) {
  ColTilePlan p;
  // the grid holds the sequence tiles of the longest sequence (nseg workgroups each: the row segments of one
  // column tile are neighbours in the grid), then, when launched with them, the depth tiles
  const int n_seq_tiles = grid.has_seq ? (grid.T + BN - 1) / BN : 0;
  p.active = true;
  p.dep = ct >= n_seq_tiles * nseg;
  p.ncols = p.dep ? a.T * a.Lv : a.T;
  p.seg = p.dep ? 0 : ct % nseg;
  int tile = p.dep ? ct - n_seq_tiles * nseg : ct / nseg;
  if (varlen && !p.dep && a.causal) {
    // a causal sequence tile costs what lies behind it: count the grid's tiles from the end of the sequence, so
    // that tiles of equal cost of all sequences are dispatched together, the heaviest of the whole batch first
    tile -= n_seq_tiles - (a.T + BN - 1) / BN;
    if (tile < 0) p.active = false;
  }
  p.c_first = tile * BN;
  if (varlen && p.c_first >= p.ncols) p.active = false;
  p.qt0 = p.nqt = 0;
  if (!p.active) return p;
  int wg_lo, wg_hi, tmp;
  q_interval(a, p.dep, p.c_first, wg_lo, tmp);
  q_interval(a, p.dep, imin(p.ncols, p.c_first + BN) - 1, tmp, wg_hi);
  p.qt0 = wg_lo / BM;
  p.nqt = (wg_hi + BM - 1) / BM - p.qt0;
  if (nseg > 1 && !p.dep) {  // this workgroup's share of the column tile's query tiles
    const int lo = (int)((int64_t)p.nqt * p.seg / nseg), hi = (int)((int64_t)p.nqt * (p.seg + 1) / nseg);
    p.qt0 += lo;
    p.nqt = hi - lo;
  }
  return p;
}

// rows of query tile starting at row f_q0 that exist (only a head's top tile can be short)
MODA_HD int query_tile_rows(const KArgs& a, int f_q0, int BM) { return imax(imin(a.Tq - f_q0, BM), 0); }

// ---------------------------------------------------------------------------------------------------
// Launch grids (host side), one place for the launchers and the walker.
// ---------------------------------------------------------------------------------------------------
inline int64_t row_kernel_blocks(const KArgs& a, int rows_per_block) {
  return (int64_t)((a.Tq + rows_per_block - 1) / rows_per_block) * a.B * a.Hq;
}
// chunk-visible depth columns: by whole chunks when a chunk's rows fit one 64-row query tile (tile widths up to 128:
// the chunk kernel's registers and LDS do not stretch to 256), else as column tiles of the dK/dV kernel
inline bool depth_by_chunks(const KArgs& a, int HD) { return HD <= 128 && a.L > 0 && a.chunk && (int64_t)a.Cb * a.Gf <= 64; }
inline int64_t col_kernel_blocks(const KArgs& a, int HD, int BN, int nseg) {
  const int64_t n_seq_tiles = a.has_seq ? (a.T + BN - 1) / BN : 0;
  const int64_t n_dep_tiles = (a.L > 0 && a.chunk && !depth_by_chunks(a, HD)) ? ((int64_t)a.T * a.Lv + BN - 1) / BN : 0;
  return (n_seq_tiles * nseg + n_dep_tiles) * a.B * a.Hkv;
}
// Sequence dK/dV on the 64-wide tiles: dkv_flat_kernel (three workgroups per compute unit, where dkv_kernel fits
// one) takes a launch of sequence-key column tiles -- kv head = query head, no row segments -- when the
// tiles see few query rows each (the launch waits for memory, not for the matrix pipe) or when there are enough of
// them to fill every compute unit's three places (measured: 18-35 % faster from 768 tiles up, at any sequence
// length; 16-25 % slower at 512 tiles of 16 K rows, where the heaviest tile's trips set the time).
constexpr int kDkvFlatMaxRows = 512;
inline int64_t dkv_flat_blocks(const KArgs& a) { return a.has_seq ? (int64_t)((a.T + 127) / 128) * a.B * a.Hkv : 0; }
inline bool takes_dkv_flat(const KArgs& a, int HD, int nseg) {
  return HD == 64 && a.has_seq && a.hdiv == 1 && nseg == 1 && a.compute_units > 0 &&
         col_kernel_blocks(a, HD, 128, 1) == dkv_flat_blocks(a) &&
         (a.Tq <= kDkvFlatMaxRows || dkv_flat_blocks(a) >= 3ll * a.compute_units);
}
inline int64_t delta_kernel_blocks(const KArgs& a, int rows_per_block) {
  return (int64_t)((a.Tq + rows_per_block - 1) / rows_per_block) * a.B * a.Hq;
}

}  // namespace moda
