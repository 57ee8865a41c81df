// Compile-time launch shapes of the streaming (query-row) kernels: forward and dQ.
#pragma once

namespace moda {

// Waves per workgroup (16 * NB query rows each; NB matters to the 16x16x32 kernels only), LDS ring stages of one 64-column K tile + V tile, and how
// many tiles ahead the global->LDS loads run.
//
// RowLarge is the throughput shape: 256 query rows share every K/V tile.  RowSmall is for problems
// with few query rows per (batch, head), where the large shape leaves compute units without a
// workgroup and makes every wave sit through the barriers of depth tiles that only other waves of
// its workgroup touch: fewer rows per workgroup mean more workgroups and a depth range that is
// mostly the wave's own.  Its wave count is the smallest one whose tile loader covers a multiple
// of 16 rows per pass (the LDS swizzle repeats every 16 rows).
struct RowLarge {
  static constexpr int W = 8, NST = 3, DIST = 2, NB = 2;
  static constexpr bool PP = false;
};
// RowLarge with the upper half of the workgroup running half a tile behind the lower half (see the
// forward kernel); one more ring stage keeps the previous tile's V alive for it.
struct RowLargePP {
  static constexpr int W = 8, NST = 4, DIST = 2, NB = 2;
  static constexpr bool PP = true;
};
template <int HD>
struct RowSmall;
template <>
struct RowSmall<64> {
  static constexpr int W = 2, NST = 3, DIST = 2, NB = 2;  // 48 KB of LDS: three workgroups per compute unit
  static constexpr bool PP = false;
};
template <>
struct RowSmall<128> {
  static constexpr int W = 4, NST = 2, DIST = 1, NB = 2;  // 64 KB of LDS: two workgroups per compute unit
  static constexpr bool PP = false;
};

// Head dims above 128 (tile width 256, 16x16x32 kernels only): 16 query rows per wave, so that the wave's Q (and
// dO) operands and its 256-wide accumulator still fit the register file; two ring stages of 64 KB.
struct RowWide {
  static constexpr int W = 8, NST = 2, DIST = 1, NB = 1;
  static constexpr bool PP = false;
};

// Host side: the small shape is used when the large one would not even give every compute unit
// two workgroups.
inline bool use_small_rows(long long rows_per_head, long long heads, int compute_units) {
  const long long large_blocks = (rows_per_head + 32 * RowLarge::W - 1) / (32 * RowLarge::W) * heads;
  return large_blocks < 2ll * compute_units;
}

}  // namespace moda
