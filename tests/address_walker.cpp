// Host-side address walker for the matrix-core attention kernels (test infrastructure, built and run by
// tests/test_address_model_cpu.py; needs no GPU).
//
// For one problem description it replays, on the CPU, every global-memory access the kernels of a forward and a
// backward launch would make -- per workgroup, wave, lane and trip: the register operand loads, every buffer
// descriptor of the global->LDS tile loads with each lane's vector and scalar offset, the row statistics, and all
// stores -- and checks each one against the extent of the tensor it belongs to.  The index arithmetic is not
// restated here: it is the kernels' own (moda_amd/csrc/geometry.h, kargs.h: enter_sequence, tile.h: Tile,
// AsyncTileLoader, WaveTileLoader, tile16.h: slot_base, tuning.h), compiled for the host; what this file adds is
// the kernels' control flow around it (which tile is issued when, which lanes are guarded by what).
//
// Checked per access:
//   * register loads and stores: [address, address + bytes) inside the tensor;
//   * tile loads: the descriptor's base inside the tensor and every lane the range check lets through inside it
//     (lanes whose offset + 16 exceeds num_records receive zeros and touch no memory); the lane's offset
//     voffset + soffset does not wrap 32 bits (the range check the kernels rely on compares that sum with
//     num_records); a lane whose chunk lies past the tensors' head dim is out of range; the 64 LDS slots the load
//     fills lie inside the launch's dynamic LDS allocation;
//   * coverage: every element of o, lse, dq, dk, dv, dkd, dvd and of the row-sum workspace is written exactly once.
//
// usage: address_walker HD D Dv H G L Lv mode(0..4) chunk_tokens row_segments packed B_or_n len0 [len1 ...]
//   packed = 0: a fixed-length batch of B sequences of len0 tokens; packed = 1: n sequences on one packed axis.
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "../moda_amd/csrc/geometry.h"
#include "../moda_amd/csrc/kargs.h"
#include "../moda_amd/csrc/tile.h"
#include "../moda_amd/csrc/tile16.h"
#include "../moda_amd/csrc/tuning.h"

using namespace moda;

namespace {

struct Region {
  std::string name;
  uint64_t base = 0, bytes = 0;
  std::vector<uint8_t> writes;  // per 2-byte (or 4-byte for fp32 regions) unit: number of writes
  int unit = 2;
  bool track = false;
};

std::map<std::string, Region> g_regions;
long long g_checked = 0, g_dma_in = 0, g_dma_out = 0;
std::string g_ctx;

[[noreturn]] void fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  fprintf(stdout, "VIOLATION [%s] ", g_ctx.c_str());
  vfprintf(stdout, fmt, ap);
  fprintf(stdout, "\n");
  va_end(ap);
  exit(1);
}

Region& region(const char* name) { return g_regions.at(name); }

const uint16_t* add_region(const char* name, int idx, uint64_t bytes, int unit, bool track) {
  // self-test hook: WALKER_SHRINK=<tensor>:<bytes> makes one tensor smaller than the kernels are told, which the
  // walk must report
  if (const char* e = getenv("WALKER_SHRINK")) {
    const char* colon = strchr(e, ':');
    if (colon && std::string(e, colon - e) == name) {
      const uint64_t cut = strtoull(colon + 1, nullptr, 10);
      bytes = bytes > cut ? bytes - cut : 0;
      track = false;
    }
  }
  Region r;
  r.name = name;
  r.base = ((uint64_t)(idx + 1)) << 40;  // far apart: an offset error cannot land in a neighbour
  r.bytes = bytes;
  r.unit = unit;
  r.track = track;
  if (track) r.writes.assign(bytes / unit, 0);
  g_regions[name] = r;
  return (const uint16_t*)r.base;
}

void check_access(const char* name, const void* p, uint64_t n, bool write) {
  Region& r = region(name);
  const uint64_t a = (uint64_t)p;
  g_checked++;
  if (a < r.base || a + n > r.base + r.bytes)
    fail("%s of %llu bytes at %s%+lld (tensor holds %llu bytes)", write ? "store" : "load", (unsigned long long)n, name,
         (long long)(a - r.base), (unsigned long long)r.bytes);
  if (write && r.track)
    for (uint64_t i = (a - r.base) / r.unit; i < (a - r.base + n) / r.unit; i++)
      if (++r.writes[i] > 1) fail("%s unit %llu written twice", name, (unsigned long long)i);
}

// one lane of a global->LDS load
void check_dma(const char* name, const void* desc_base, uint32_t num_records, int voff, int soff, int bytes,
               uint32_t lds_byte, uint32_t lds_limit, bool lane_is_pad) {
  Region& r = region(name);
  const uint64_t b = (uint64_t)desc_base;
  g_checked++;
  // The descriptor of a (batch, head) slice starts at the slice's first row and covers whole row strides, so behind
  // the tensor's last row it may reach into the other heads' share of one more stride; no lane offset does (each
  // in-range lane is checked against the tensor below).  The base itself must lie inside the tensor.
  if (num_records > 0 && (b < r.base || b >= r.base + r.bytes))
    fail("descriptor of %s: base %+lld, %u bytes (tensor holds %llu)", name, (long long)(b - r.base), num_records,
         (unsigned long long)r.bytes);
  if (voff < 0 || soff < 0) fail("negative offset into %s: voffset %d soffset %d", name, voff, soff);
  const uint64_t off = (uint64_t)(uint32_t)voff + (uint64_t)(uint32_t)soff;
  if (off + bytes > 0xffffffffull) fail("offset into %s wraps 32 bits: voffset %d soffset %d", name, voff, soff);
  const bool in_range = off + bytes <= num_records;
  if (lane_is_pad && in_range) fail("padding lane of %s in range: voffset %d soffset %d records %u", name, voff, soff, num_records);
  if (in_range) {
    g_dma_in++;
    check_access(name, (const char*)desc_base + off, bytes, false);
  } else {
    g_dma_out++;
  }
  if ((uint64_t)lds_byte + 64ull * bytes > lds_limit)
    fail("LDS target %u (+%d) beyond the %u bytes of dynamic LDS", lds_byte, 64 * bytes, lds_limit);
}

struct Case {
  int HD, D, Dv, H, G, L, Lv, mode, cb, packed, nseq;
  std::vector<int> len;
  std::vector<int32_t> cu;
  int total, Tmax;
};

KArgs make_args(const Case& c) {
  KArgs a;
  memset(&a, 0, sizeof(a));
  const bool plain = c.mode == 4;
  const int Bt = c.packed ? 1 : c.nseq;  // batch extent of the tensors
  const int T = c.packed ? c.total : c.Tmax;
  a.B = c.nseq;
  a.T = c.Tmax;
  a.Hkv = c.H;
  a.D = c.D;
  a.Dv = c.Dv;
  a.Tq = plain ? c.Tmax : c.Tmax * c.G;
  a.Gf = plain ? 1 : c.G;
  a.Hq = plain ? c.H * c.G : c.H;
  a.hdiv = plain ? c.G : 1;
  a.L = c.L;
  a.Lv = c.Lv > 0 ? c.Lv : c.L;
  a.Cb = c.mode == 2 ? (c.cb > 0 ? c.cb : 1) : 1;
  a.has_seq = c.mode != 3;
  a.causal = c.mode == 0 || c.mode == 2 || plain;
  a.chunk = c.mode == 2;
  a.scale = 1.f;
  a.dkv_split = 1;
  a.compute_units = 256;
  const int64_t qrows = plain ? T : (int64_t)T * c.G;
  a.delta_pitch = c.packed ? (int)qrows : a.Tq;
  a.own_delta = 1;  // a whole backward: the dQ kernel forms the row sums (the delta kernel is walked as well)
  auto strides = [&](int64_t rows, int heads, int dim) { return Str3{rows * heads * dim, (int64_t)heads * dim, (int64_t)dim}; };
  // bytes of a dense [Bt, rows, heads, dim] tensor of 16-bit elements
  auto bytes = [&](int64_t rows, int heads, int dim) { return (uint64_t)Bt * rows * heads * dim * 2; };
  int idx = 0;
  a.q = add_region("q", idx++, bytes(qrows, a.Hq, c.D), 2, false);
  a.o = add_region("o", idx++, bytes(qrows, a.Hq, c.Dv), 2, true);
  a.out_o = (uint16_t*)a.o;
  a.d_o = add_region("do", idx++, bytes(qrows, a.Hq, c.Dv), 2, false);
  a.dq = (uint16_t*)add_region("dq", idx++, bytes(qrows, a.Hq, c.D), 2, true);
  a.k = add_region("k", idx++, bytes(T, c.H, c.D), 2, false);
  a.v = add_region("v", idx++, bytes(T, c.H, c.Dv), 2, false);
  a.dk = (uint16_t*)add_region("dk", idx++, bytes(T, c.H, c.D), 2, true);
  a.dv = (uint16_t*)add_region("dv", idx++, bytes(T, c.H, c.Dv), 2, true);
  a.kd = add_region("kd", idx++, bytes((int64_t)T * c.L, c.H, c.D), 2, false);
  a.vd = add_region("vd", idx++, bytes((int64_t)T * c.L, c.H, c.Dv), 2, false);
  a.dkd = (uint16_t*)add_region("dkd", idx++, bytes((int64_t)T * c.L, c.H, c.D), 2, true);
  a.dvd = (uint16_t*)add_region("dvd", idx++, bytes((int64_t)T * c.L, c.H, c.Dv), 2, true);
  a.lse = (float*)add_region("lse", idx++, (uint64_t)Bt * qrows * a.Hq * 4, 4, true);
  a.delta = (float*)add_region("delta", idx++, (uint64_t)(c.packed ? 1 : c.nseq) * a.Hq * a.delta_pitch * 4, 4, true);
  if (depth_scores_from_dq(a, c.HD)) {  // P and dS of the (query row, slot) pairs, handed from dQ to the depth-gradient kernel
    const uint64_t n = (uint64_t)(c.packed ? 1 : c.nseq) * a.Hq * a.delta_pitch * a.Lv * 2;
    a.depth_p = (uint16_t*)add_region("hand_p", idx++, n, 2, true);
    a.depth_ds = (uint16_t*)add_region("hand_ds", idx++, n, 2, true);
  }
  a.sq = a.sdq = strides(qrows, a.Hq, c.D);
  a.so = a.sdo = strides(qrows, a.Hq, c.Dv);
  a.sk = a.sdk = strides(T, c.H, c.D);
  a.sv = a.sdv = strides(T, c.H, c.Dv);
  a.skd = a.sdkd = strides((int64_t)T * c.L, c.H, c.D);
  a.svd = a.sdvd = strides((int64_t)T * c.L, c.H, c.Dv);
  if (c.packed) a.cu = c.cu.data();
  return a;
}

// argument block of the workgroup: rebased on its sequence for a packed batch
KArgs seq_args(const KArgs& in, int& b) {
  KArgs a = in;
  enter_sequence(a, b);
  return a;
}

void ctx(const char* kernel, int block, int wave, int lane, const char* what) {
  char buf[256];
  snprintf(buf, sizeof(buf), "%s block %d wave %d lane %d: %s", kernel, block, wave, lane, what);
  g_ctx = buf;
}

// ---------------------------------------------------------------------------------------------------------------
// forward / dQ: the ring of K+V tiles and the waves' own depth tiles.  `dq`: also dO, lse, delta reads, dq stores.
// ROWS_PER_WAVE: 32 (forward on 32x32x16) or 16 * NB.
// ---------------------------------------------------------------------------------------------------------------
template <int HD, typename Shape, bool WIDE_ADDR>
void walk_row_kernel(const KArgs& a_in, bool dq, int rows_per_wave, bool own_possible, uint32_t lds_bytes,
                     const char* kname) {
  constexpr int BN = 64, NT = 64 * Shape::W, NST = Shape::NST, DIST = Shape::DIST;
  const int BM = rows_per_wave * Shape::W;
  const bool varlen = a_in.cu != nullptr;
  const int BH = a_in.B * a_in.Hq;
  const int64_t nblk = row_kernel_blocks(a_in, BM);
  typedef AsyncTileLoader<HD, BN, NT> Loader;
  for (int64_t block = 0; block < nblk; block++) {
    const int bh = (int)(block % BH);
    int b = bh / a_in.Hq;
    const int hq = bh % a_in.Hq, hkv = hq / a_in.hdiv;
    const KArgs a = seq_args(a_in, b);
    const int Ld = a.L;
    const int nqt = (a.Tq + BM - 1) / BM;
    const int qt = query_tile_of((int)block, BH, BM, varlen ? a_in.Tq : a.Tq);
    if (varlen && qt >= nqt) continue;
    if (qt < 0 || qt >= nqt) fail("%s: query tile %d of %d", kname, qt, nqt);
    const bool own_depth = own_possible && waves_own_depth(a, Ld);
    const RowTilePlan plan = row_tile_plan(a, qt, BM, BN, Ld > 0 && !own_depth);
    const int ntiles = plan.n_seq + plan.n_dep;
    for (int tid = 0; tid < NT; tid++) {
      const int lane = tid & 63, wave = tid >> 6;
      // register operands, statistics, stores: lane owns row(s) r, 16-byte pieces of the head dim
      const int rpl = rows_per_wave == 32 ? 1 : rows_per_wave / 16;  // rows per lane
      for (int nb = 0; nb < rpl; nb++) {
        const int r = rows_per_wave == 32 ? qt * BM + wave * 32 + (lane & 31) : qt * BM + wave * rows_per_wave + 16 * nb + (lane & 15);
        if (r >= a.Tq) continue;
        const int piece = rows_per_wave == 32 ? 8 * (lane >> 5) : 8 * (lane >> 4);  // first element of this lane's pieces
        const int step = rows_per_wave == 32 ? 16 : 32;
        ctx(kname, (int)block, wave, lane, "Q / dO register rows");
        for (int e = piece; e < HD; e += step) {
          if (e < a.D) check_access("q", a.q + b * a.sq.b + hq * a.sq.h + (int64_t)r * a.sq.t + e, 16, false);
          if (dq && e < a.Dv) check_access("do", a.d_o + b * a.sdo.b + hq * a.sdo.h + (int64_t)r * a.sdo.t + e, 16, false);
          if (dq && a.own_delta && e < a.Dv) check_access("o", a.o + b * a.so.b + hq * a.so.h + (int64_t)r * a.so.t + e, 16, false);
        }
        const bool stat_lane = rows_per_wave == 32 ? (lane >> 5) == 0 : (lane >> 4) == 0;
        ctx(kname, (int)block, wave, lane, "row statistics and result rows");
        if (dq) {
          check_access("lse", a.lse + ((int64_t)b * a.Tq + r) * a.Hq + hq, 4, false);
          // the row sum: read, or formed here and left for the later kernels by the first of the row's four lanes
          if (!a.own_delta || stat_lane)
            check_access("delta", a.delta + ((int64_t)b * a.Hq + hq) * (varlen ? a.delta_pitch : a.Tq) + r, 4, a.own_delta != 0);
        } else if (stat_lane) {
          check_access("lse", a.lse + ((int64_t)b * a.Tq + r) * a.Hq + hq, 4, true);
        }
        // result row: 8-byte stores, lane group g / q4 owns elements 4g + 8j (32x32) or 4q + 16j (16x16)
        const int first = rows_per_wave == 32 ? 4 * (lane >> 5) : 4 * (lane >> 4), stride = rows_per_wave == 32 ? 8 : 16;
        for (int e = first; e < HD; e += stride) {
          if (dq && e < a.D) check_access("dq", a.dq + b * a.sdq.b + hq * a.sdq.h + (int64_t)r * a.sdq.t + e, 8, true);
          if (!dq && e < a.Dv) check_access("o", a.out_o + b * a.so.b + hq * a.so.h + (int64_t)r * a.so.t + e, 8, true);
        }
      }
      // ring tiles: every tile 0 .. ntiles-1 is issued once, stages in turn
      Loader ld;
      ld.init(tid);
      typename Loader::Source srcK{}, srcV{};
      if (a.has_seq && plan.n_seq > 0) {
        srcK = ld.source(a.k + b * a.sk.b + hkv * a.sk.h, a.sk.t, 0, a.T, a.D);
        srcV = ld.source(a.v + b * a.sv.b + hkv * a.sv.h, a.sv.t, 0, a.T, a.Dv);
      }
      for (int it = 0; it < ntiles; it++) {
        const int st = it % NST;
        const uint32_t kt = (uint32_t)st * 2 * BN * HD * 2;
        const bool dep = it >= plan.n_seq;
        if (Ld > 0 && it == plan.n_seq) {
          srcK = ld.source(a.kd + b * a.skd.b + hkv * a.skd.h, a.skd.t, plan.dep0, a.T * a.L, a.D);
          srcV = ld.source(a.vd + b * a.svd.b + hkv * a.svd.h, a.svd.t, plan.dep0, a.T * a.L, a.Dv);
        }
        const int row0 = ring_tile_row0(plan, it, BN);
        ctx(kname, (int)block, wave, lane, dep ? "ring depth tile" : "ring sequence tile");
        for (int i = 0; i < Loader::N; i++) {
          const uint32_t ldsK = kt + (uint32_t)ld.lds_elems(i) * 2, ldsV = ldsK + BN * HD * 2;
          if (dep && a.Lv != a.L) {  // partially filled stream: one descriptor anchored at the first column's token
            const int w0 = row0 / a.Lv, l0 = row0 - w0 * a.Lv;
            const int64_t anchor = (int64_t)w0 * a.L, rows_total = (int64_t)a.T * a.L;
            check_dma("kd", a.kd + b * a.skd.b + hkv * a.skd.h + anchor * a.skd.t,
                      mapped_bytes(anchor, rows_total, (uint32_t)a.skd.t * 2u),
                      ld.mapped_offset(i, l0, a.L, a.Lv, (int)a.skd.t * 2, a.D), 0, 16, ldsK, lds_bytes, ld.pads(a.D));
            check_dma("vd", a.vd + b * a.svd.b + hkv * a.svd.h + anchor * a.svd.t,
                      mapped_bytes(anchor, rows_total, (uint32_t)a.svd.t * 2u),
                      ld.mapped_offset(i, l0, a.L, a.Lv, (int)a.svd.t * 2, a.Dv), 0, 16, ldsV, lds_bytes, ld.pads(a.Dv));
            // a lane in range must have fetched a slot that holds data
            const int rel = mapped_row(l0, Loader::rows_before(i) + ld.row_in_pass, a.L, a.Lv);
            if ((anchor + rel) % a.L >= a.Lv) fail("mapped depth tile reads slot %d of %d filled", (int)((anchor + rel) % a.L), a.Lv);
          } else if (WIDE_ADDR) {
            const int row_end = dep ? a.T * a.L : a.T;
            const uint16_t* kb = dep ? a.kd + b * a.skd.b + hkv * a.skd.h : a.k + b * a.sk.b + hkv * a.sk.h;
            const uint16_t* vb = dep ? a.vd + b * a.svd.b + hkv * a.svd.h : a.v + b * a.sv.b + hkv * a.sv.h;
            const int64_t ks = dep ? a.skd.t : a.sk.t, vs = dep ? a.svd.t : a.sv.t;
            check_dma(dep ? "kd" : "k", kb + (int64_t)row0 * ks, Loader::anchored_bytes(ks, row0, row_end),
                      ld.lane_offset((int)ks * 2, a.D), Loader::rows_before(i) * (int)ks * 2, 16, ldsK, lds_bytes, ld.pads(a.D));
            check_dma(dep ? "vd" : "v", vb + (int64_t)row0 * vs, Loader::anchored_bytes(vs, row0, row_end),
                      ld.lane_offset((int)vs * 2, a.Dv), Loader::rows_before(i) * (int)vs * 2, 16, ldsV, lds_bytes, ld.pads(a.Dv));
          } else {
            check_dma(dep ? "kd" : "k", srcK.base, srcK.nbytes, srcK.voff, Loader::source_soffset(srcK, row0, i), 16, ldsK,
                      lds_bytes, ld.pads(a.D));
            check_dma(dep ? "vd" : "v", srcV.base, srcV.nbytes, srcV.voff, Loader::source_soffset(srcV, row0, i), 16, ldsV,
                      lds_bytes, ld.pads(a.Dv));
          }
        }
      }
      // the wave's own depth columns, 32 at a time through a private K tile and V tile
      if (own_depth) {
        typedef WaveTileLoader<HD> Own;
        const uint32_t kt = (uint32_t)wave * (2 * 32 * HD) * 2, vt = kt + 32 * HD * 2;
        const int rw0 = qt * BM + wave * rows_per_wave;
        if (rw0 < a.Tq) {
          const DepthSpan span = own_depth_span(a, rw0, rows_per_wave);
          const int nh = (span.c_end - span.c_beg + 31) / 32;
          Own own;
          own.init(lane);
          ctx(kname, (int)block, wave, lane, "own depth tile");
          for (int j = 0; j < nh; j++) {
            const int col0 = span.c_beg + 32 * j;
            const int nrows = imin(32, span.c_end - col0);
            // where the dQ kernel forms the depth gradients it alternates between two sets of private tiles
            // ... and so does the forward kernel on the 64-wide tiles
            const uint32_t set = ((dq && depth_grads_in_dq(a, HD)) || (!dq && HD <= 64)) ? (uint32_t)(j & 1) * Shape::W * 64 * HD * 2 : 0u;
            for (int i = 0; i < Own::N; i++) {
              if (a.Lv != a.L) {
                const int w0 = col0 / a.Lv, l0 = col0 - w0 * a.Lv;
                const int64_t anchor = (int64_t)w0 * a.L, rows_total = (int64_t)a.T * a.L;
                const int vk = own.mapped_offset(i, l0, a.L, a.Lv, nrows, (int)a.skd.t * 2, a.D);
                const int vv = own.mapped_offset(i, l0, a.L, a.Lv, nrows, (int)a.svd.t * 2, a.Dv);
                check_dma("kd", a.kd + b * a.skd.b + hkv * a.skd.h + anchor * a.skd.t,
                          nrows > 0 ? mapped_bytes(anchor, rows_total, (uint32_t)a.skd.t * 2u) : 0u, vk, 0, 16, kt + set + i * 1024,
                          lds_bytes, vk == kPadOffset);
                check_dma("vd", a.vd + b * a.svd.b + hkv * a.svd.h + anchor * a.svd.t,
                          nrows > 0 ? mapped_bytes(anchor, rows_total, (uint32_t)a.svd.t * 2u) : 0u, vv, 0, 16, vt + set + i * 1024,
                          lds_bytes, vv == kPadOffset);
                continue;
              }
              const int voffk = own.lane_offset(i, (int)a.skd.t * 2, a.D), voffv = own.lane_offset(i, (int)a.svd.t * 2, a.Dv);
              check_dma("kd", a.kd + b * a.skd.b + hkv * a.skd.h + (int64_t)col0 * a.skd.t,
                        nrows > 0 ? (uint32_t)nrows * (uint32_t)a.skd.t * 2u : 0u, voffk, 0, 16, kt + set + i * 1024, lds_bytes,
                        voffk == kPadOffset);
              check_dma("vd", a.vd + b * a.svd.b + hkv * a.svd.h + (int64_t)col0 * a.svd.t,
                        nrows > 0 ? (uint32_t)nrows * (uint32_t)a.svd.t * 2u : 0u, voffv, 0, 16, vt + set + i * 1024, lds_bytes,
                        voffv == kPadOffset);
            }
          }
          // dQ kernel handing P and dS of its rows' visible depth columns to the depth-gradient kernel: lane (n, q4)
          // holds, per 16-column block, the columns slot_base(q4) .. +3 of rows 16*nb + n
          if (dq && a.depth_p && !depth_grads_in_dq(a, HD)) {
            const int n = lane & 15, q4 = lane >> 4;
            ctx(kname, (int)block, wave, lane, "depth scores for the depth-gradient kernel");
            for (int nb = 0; nb < rows_per_wave / 16; nb++) {
              const int r = rw0 + 16 * nb + n;
              const RowVis vis = row_visibility(a, r, Ld);
              const int t = r / a.Gf;  // slot l of row r: element l * Gf + (r - t * Gf) of token t's block
              const int64_t at = (((int64_t)b * a.Hq + hq) * (varlen ? a.delta_pitch : a.Tq) + (int64_t)t * a.Gf) * a.Lv + (r - t * a.Gf);
              for (int j = 0; j < nh; j++)
                for (int mb = 0; mb < 2; mb++)
                  for (int i = 0; i < 4; i++) {
                    const int c = span.c_beg + 32 * j + 16 * mb + slot_base(q4) + i;
                    if (c < vis.dlo || c >= vis.dhi) continue;
                    check_access("hand_p", a.depth_p + at + (int64_t)(c - vis.dlo) * a.Gf, 2, true);
                    check_access("hand_ds", a.depth_ds + at + (int64_t)(c - vis.dlo) * a.Gf, 2, true);
                  }
            }
          }
          // dQ kernel outside chunk-visible mode: the same pass forms dK and dV of the wave's own depth columns.
          // The gradient rows leave 16 at a time through a staging block behind the private tiles, 16 bytes per lane
          // (WaveTileLoader's row / chunk split).
          if (dq && depth_grads_in_dq(a, HD)) {
            if (rows_per_wave != 32) fail("%s: depth gradients need 32 rows per wave", kname);
            const uint32_t stage = 2u * Shape::W * 64 * HD * 2 + (uint32_t)wave * 16 * HD * 2;
            if (stage + 16 * HD * 2 > lds_bytes) fail("%s: staging block past the LDS allocation", kname);
            ctx(kname, (int)block, wave, lane, "own depth gradients");
            constexpr int RPW = Own::RPW, NPASS = 16 / RPW;
            for (int j = 0; j < nh; j++)
              for (int cb = 0; cb < 2; cb++) {
                const int cbase = span.c_beg + 32 * j + 16 * cb;
                if (cbase >= span.c_end) continue;
                for (int i = 0; i < NPASS; i++) {
                  const int row = i * RPW + own.prow;
                  const int lch = own.pch ^ Tile<HD>::swz(row);
                  const int c = cbase + row;
                  if (c >= span.c_end) continue;
                  if (c / a.Lv >= a.T) fail("%s: depth column %d outside the stream", kname, c);
                  const int64_t prow = depth_row_of(a, c);
                  if (lch * 8 < a.Dv) check_access("dvd", a.dvd + b * a.sdvd.b + hkv * a.sdvd.h + prow * a.sdvd.t + lch * 8, 16, true);
                  if (lch * 8 < a.D) check_access("dkd", a.dkd + b * a.sdkd.b + hkv * a.sdkd.h + prow * a.sdkd.t + lch * 8, 16, true);
                }
              }
          }
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// row sums: o * do -> workspace
// ---------------------------------------------------------------------------------------------------------------
template <int HD>
void walk_delta(const KArgs& a_in) {
  constexpr int TPR = HD / 8, RPB = 256 / TPR;
  const int nrb = (a_in.Tq + RPB - 1) / RPB;
  const int64_t nblk = delta_kernel_blocks(a_in, RPB);
  for (int64_t block = 0; block < nblk; block++)
    for (int tid = 0; tid < 256; tid++) {
      const int bh = (int)(block / nrb), rb = (int)(block - (int64_t)bh * nrb);
      int b = bh / a_in.Hq;
      const int hq = bh % a_in.Hq;
      const KArgs a = seq_args(a_in, b);
      const int r = rb * RPB + tid / TPR, c = (tid % TPR) * 8;
      ctx("delta_kernel", (int)block, tid >> 6, tid & 63, "o, do rows and the row sum");
      if (r < a.Tq && c < a.Dv) {
        check_access("o", a.o + b * a.so.b + hq * a.so.h + (int64_t)r * a.so.t + c, 16, false);
        check_access("do", a.d_o + b * a.sdo.b + hq * a.sdo.h + (int64_t)r * a.sdo.t + c, 16, false);
      }
      if (r < a.Tq && (tid % TPR) == 0)
        check_access("delta", a.delta + ((int64_t)b * a.Hq + hq) * a.delta_pitch + r, 4, true);
    }
}

// ---------------------------------------------------------------------------------------------------------------
// dK/dV column tiles (sequence keys, and depth columns in chunk-visible mode when not done by whole chunks)
// ---------------------------------------------------------------------------------------------------------------
template <int HD>
void walk_dkv(const KArgs& a_in) {
  constexpr int NB = HD > 128 ? 1 : 2, BM = HD > 128 ? 32 : 64, MBLK = BM / 16, BN = 4 * 16 * NB, KS = HD / 32, MB = HD / 16,
                NST = 3, NP = (MBLK / 2) * NB, SP = 64;
  const uint32_t lds_bytes = 3 * 2 * BM * HD * 2 + 2 * 4 * (BM / 32) * NB * 64 * 16 + 3 * 2 * 64 * 4;
  const uint32_t stat_byte = NST * 2 * BM * HD * 2 + 2 * 4 * NP * 64 * 16;
  const bool varlen = a_in.cu != nullptr;
  const int nseg = varlen ? 1 : a_in.dkv_split;
  const int BHk = a_in.B * a_in.Hkv;
  const int64_t nblk = col_kernel_blocks(a_in, HD, BN, nseg);
  typedef AsyncTileLoader<HD, BM, 512> Loader;
  for (int64_t block = 0; block < nblk; block++) {
    const int bh = (int)(block % BHk), ct = (int)(block / BHk);
    int b = bh / a_in.Hkv;
    const int hkv = bh % a_in.Hkv;
    const KArgs a = seq_args(a_in, b);
    const ColTilePlan plan = col_tile_plan(a_in, a, ct, BN, BM, varlen, nseg);
    if (!plan.active) {
      if (!varlen) fail("dkv_kernel: inactive column tile in a fixed-length launch");
      continue;
    }
    const bool dep = plan.dep;
    for (int tid = 0; tid < 512; tid++) {
      const int lane = tid & 63, n = lane & 15, q4 = lane >> 4, wave = tid >> 6, kblk = wave & 3;
      const bool role_b = wave >= 4;
      for (int nb = 0; nb < NB; nb++) {
        const int c = plan.c_first + kblk * (16 * NB) + 16 * nb + n;
        const bool valid = c < plan.ncols;
        const int64_t crow = dep ? depth_row_of(a, c) : c;
        ctx("dkv_kernel", (int)block, wave, lane, "stationary K / V rows");
        const uint16_t* src = role_b ? (dep ? a.vd + b * a.svd.b + hkv * a.svd.h : a.v + b * a.sv.b + hkv * a.sv.h)
                                     : (dep ? a.kd + b * a.skd.b + hkv * a.skd.h : a.k + b * a.sk.b + hkv * a.sk.h);
        const int64_t st = role_b ? (dep ? a.svd.t : a.sv.t) : (dep ? a.skd.t : a.sk.t);
        const char* sname = role_b ? (dep ? "vd" : "v") : (dep ? "kd" : "k");
        for (int ks = 0; ks < KS; ks++)
          if (valid && 32 * ks + 8 * q4 < (role_b ? a.Dv : a.D)) check_access(sname, src + crow * st + 32 * ks + 8 * q4, 16, false);
        if (!valid) continue;
        ctx("dkv_kernel", (int)block, wave, lane, "gradient rows");
        if (nseg > 1 && !dep) {  // a row segment: fp32 partial sums, all HD columns of the tile width
          const int64_t plane = (int64_t)a.B * a.Hkv * a.T * HD;
          float* pp = a.dkv_part + ((int64_t)(role_b ? 0 : 1) * nseg + plan.seg) * plane +
                      (((int64_t)b * a.Hkv + hkv) * a.T + c) * HD;
          for (int d = 0; d < MB; d++) check_access("part", pp + 16 * d + 4 * q4, 16, true);
          continue;
        }
        const char* oname = role_b ? (dep ? "dkd" : "dk") : (dep ? "dvd" : "dv");
        uint16_t* outp = !role_b ? (dep ? a.dvd + b * a.sdvd.b + hkv * a.sdvd.h + crow * a.sdvd.t
                                        : a.dv + b * a.sdv.b + hkv * a.sdv.h + crow * a.sdv.t)
                                 : (dep ? a.dkd + b * a.sdkd.b + hkv * a.sdkd.h + crow * a.sdkd.t
                                        : a.dk + b * a.sdk.b + hkv * a.sdk.h + crow * a.sdk.t);
        for (int d = 0; d < MB; d++)
          if (16 * d + 4 * q4 < (role_b ? a.D : a.Dv)) check_access(oname, outp + 16 * d + 4 * q4, 8, true);
      }
      // the streamed query tiles: per query head, from the top tile down, stages in turn
      Loader ld;
      ld.init(tid);
      const uint32_t q_row_bytes = (uint32_t)a.sq.t * 2u, do_row_bytes = (uint32_t)a.sdo.t * 2u;
      const int voff_q = ld.lane_offset((int)q_row_bytes, a.D), voff_do = ld.lane_offset((int)do_row_bytes, a.Dv);
      const int voff_stat = wave == 0 ? lane * a.Hq * 4 : lane * 4;
      const uint32_t stat_row_bytes = wave == 0 ? (uint32_t)a.Hq * 4u : 4u;
      int ld_st = 0;
      for (int gh = 0; gh < a.hdiv; gh++) {
        const int hq = hkv * a.hdiv + gh;
        int f_q0 = (plan.qt0 + plan.nqt - 1) * BM;
        for (int t = 0; t < plan.nqt; t++, f_q0 -= BM) {
          if (f_q0 < 0) fail("dkv_kernel: query tile row %d", f_q0);
          const uint32_t rows = (uint32_t)query_tile_rows(a, f_q0, BM);
          if (rows == 0) fail("dkv_kernel: empty query tile at row %d (Tq %d)", f_q0, a.Tq);
          const uint16_t* qp = a.q + b * a.sq.b + hq * a.sq.h + (int64_t)f_q0 * a.sq.t;
          const uint16_t* dop = a.d_o + b * a.sdo.b + hq * a.sdo.h + (int64_t)f_q0 * a.sdo.t;
          const uint32_t lds_q = (uint32_t)(ld_st * 2 * BM * HD + wave * 512) * 2;
          ctx("dkv_kernel", (int)block, wave, lane, "query tile (Q, dO)");
          for (int k = 0; k < Loader::N; k++) {
            check_dma("q", qp, rows * q_row_bytes, voff_q, k * 8 * Loader::RPW * (int)q_row_bytes, 16, lds_q + k * 8 * 1024,
                      lds_bytes, ld.pads(a.D));
            check_dma("do", dop, rows * do_row_bytes, voff_do, k * 8 * Loader::RPW * (int)do_row_bytes, 16,
                      lds_q + BM * HD * 2 + k * 8 * 1024, lds_bytes, ld.pads(a.Dv));
          }
          if (wave < 2) {
            ctx("dkv_kernel", (int)block, wave, lane, wave == 0 ? "query tile lse" : "query tile row sums");
            const float* sp = wave == 0 ? a.lse + ((int64_t)b * a.Tq + f_q0) * a.Hq + hq
                                        : a.delta + ((int64_t)b * a.Hq + hq) * (varlen ? a.delta_pitch : a.Tq) + f_q0;
            check_dma(wave == 0 ? "lse" : "delta", sp, (rows - 1) * stat_row_bytes + 4u, voff_stat, 0, 4,
                      stat_byte + (uint32_t)(ld_st * 2 * SP + (wave == 0 ? 0 : SP)) * 4, lds_bytes, false);
          }
          ld_st = (ld_st + 1) % NST;
        }
      }
    }
  }
}

// dkv_flat_kernel: four waves, a wave's 32 columns with K and V in registers, query tiles of 32 rows
template <int HD>
void walk_dkv_flat(const KArgs& a_in) {
  constexpr int NB = 2, BM = 32, BN = 4 * 16 * NB, KS = HD / 32, MB = HD / 16, NST = 3, SP = 64;
  const uint32_t lds_bytes = 3 * 2 * 32 * HD * 2 + 3 * 2 * 64 * 4;
  const uint32_t stat_byte = NST * 2 * BM * HD * 2;
  const bool varlen = a_in.cu != nullptr;
  const int BHk = a_in.B * a_in.Hkv;
  const int64_t nblk = dkv_flat_blocks(a_in);
  typedef AsyncTileLoader<HD, BM, 256> Loader;
  for (int64_t block = 0; block < nblk; block++) {
    const int bh = (int)(block % BHk), ct = (int)(block / BHk);
    int b = bh / a_in.Hkv;
    const int hkv = bh % a_in.Hkv;
    const KArgs a = seq_args(a_in, b);
    const ColTilePlan plan = col_tile_plan(a_in, a, ct, BN, BM, varlen, 1);
    if (!plan.active) {
      if (!varlen) fail("dkv_flat_kernel: inactive column tile in a fixed-length launch");
      continue;
    }
    if (plan.dep) fail("dkv_flat_kernel: column tile %d is not a sequence tile", ct);
    for (int tid = 0; tid < 256; tid++) {
      const int lane = tid & 63, n = lane & 15, q4 = lane >> 4, wave = tid >> 6;
      for (int nb = 0; nb < NB; nb++) {
        const int c = plan.c_first + wave * (16 * NB) + 16 * nb + n;
        if (c >= a.T) continue;
        ctx("dkv_flat_kernel", (int)block, wave, lane, "stationary K and V rows");
        for (int ks = 0; ks < KS; ks++) {
          if (32 * ks + 8 * q4 < a.D) check_access("k", a.k + b * a.sk.b + hkv * a.sk.h + 8 * q4 + (int64_t)c * a.sk.t + 32 * ks, 16, false);
          if (32 * ks + 8 * q4 < a.Dv) check_access("v", a.v + b * a.sv.b + hkv * a.sv.h + 8 * q4 + (int64_t)c * a.sv.t + 32 * ks, 16, false);
        }
        ctx("dkv_flat_kernel", (int)block, wave, lane, "gradient rows");
        uint16_t* dkp = a.dk + b * a.sdk.b + hkv * a.sdk.h + (int64_t)c * a.sdk.t + 4 * q4;
        uint16_t* dvp = a.dv + b * a.sdv.b + hkv * a.sdv.h + (int64_t)c * a.sdv.t + 4 * q4;
        for (int d = 0; d < MB; d++) {
          if (16 * d + 4 * q4 < a.D) check_access("dk", dkp + 16 * d, 8, true);
          if (16 * d + 4 * q4 < a.Dv) check_access("dv", dvp + 16 * d, 8, true);
        }
      }
      Loader ld;
      ld.init(tid);
      const bool st_lse = (wave & 1) == 0;
      const char* stb = st_lse ? (const char*)(a.lse + (int64_t)b * a.Tq * a.Hq + hkv) : (const char*)(a.delta + ((int64_t)b * a.Hq + hkv) * (varlen ? a.delta_pitch : a.Tq));
      const uint32_t st_row = st_lse ? (uint32_t)a.Hq * 4u : 4u;
      int ld_st = 0;
      for (int it = 0; it < plan.nqt; it++) {
        const int f_q0 = (plan.qt0 + plan.nqt - 1 - it) * BM;
        if (f_q0 < 0) fail("dkv_flat_kernel: query tile row %d", f_q0);
        const uint32_t Qt = (uint32_t)(ld_st * 2 * BM * HD) * 2;
        ctx("dkv_flat_kernel", (int)block, wave, lane, "query tile (Q, dO)");
        for (int i = 0; i < Loader::N; i++) {
          check_dma("q", a.q + b * a.sq.b + hkv * a.sq.h + (int64_t)f_q0 * a.sq.t, Loader::anchored_bytes(a.sq.t, f_q0, a.Tq),
                    ld.lane_offset((int)a.sq.t * 2, a.D), Loader::rows_before(i) * (int)a.sq.t * 2, 16,
                    Qt + (uint32_t)ld.lds_elems(i) * 2, lds_bytes, ld.pads(a.D));
          check_dma("do", a.d_o + b * a.sdo.b + hkv * a.sdo.h + (int64_t)f_q0 * a.sdo.t, Loader::anchored_bytes(a.sdo.t, f_q0, a.Tq),
                    ld.lane_offset((int)a.sdo.t * 2, a.Dv), Loader::rows_before(i) * (int)a.sdo.t * 2, 16,
                    Qt + (uint32_t)(BM * HD + ld.lds_elems(i)) * 2, lds_bytes, ld.pads(a.Dv));
        }
        const int rows = imax(imin(a.Tq - f_q0, BM), 0);
        if (rows == 0) fail("dkv_flat_kernel: empty query tile at row %d (Tq %d)", f_q0, a.Tq);
        ctx("dkv_flat_kernel", (int)block, wave, lane, st_lse ? "query tile lse" : "query tile row sums");
        check_dma(st_lse ? "lse" : "delta", stb + (int64_t)f_q0 * st_row, (uint32_t)(rows - 1) * st_row + 4u, lane * (int)st_row, 0, 4,
                  stat_byte + (uint32_t)(ld_st * 2 * SP + (st_lse ? 0 : SP)) * 4, lds_bytes, false);
        ld_st = (ld_st + 1) % NST;
      }
    }
  }
}

// the partial sums of the row segments -> dk, dv
template <int HD>
void walk_reduce(const KArgs& a) {
  constexpr int TPR = HD / 8;
  const int64_t rows = (int64_t)a.B * a.Hkv * a.T, plane = rows * HD;
  const int64_t nthreads = rows * TPR;
  for (int64_t gid = 0; gid < (nthreads + 255) / 256 * 256; gid++) {
    const int64_t row = gid / TPR;
    if (row >= rows) continue;
    const int sub = (int)(gid % TPR), c = (int)(row % a.T), bh = (int)(row / a.T), b = bh / a.Hkv, hkv = bh % a.Hkv;
    ctx("dkv_reduce_kernel", (int)(gid / 256), (int)(gid % 256) >> 6, (int)(gid & 63), "partial sums and dk, dv rows");
    for (int which = 0; which < 2; which++) {
      const float* src = a.dkv_part + (int64_t)which * a.dkv_split * plane + row * HD + 8 * sub;
      for (int sg = 0; sg < a.dkv_split; sg++) check_access("part", src + sg * plane, 32, false);
      uint16_t* outp = which == 0 ? a.dk + b * a.sdk.b + hkv * a.sdk.h + (int64_t)c * a.sdk.t
                                  : a.dv + b * a.sdv.b + hkv * a.sdv.h + (int64_t)c * a.sdv.t;
      if (8 * sub < (which == 0 ? a.D : a.Dv)) check_access(which == 0 ? "dk" : "dv", outp + 8 * sub, 16, true);
    }
  }
}

// chunk-visible depth columns by whole chunks (tile widths up to 128)
template <int HD>
void walk_chunk_depth(const KArgs& a_in) {
  constexpr int BM = 64, CH = HD / 8, RPW = 64 / CH, NPASS = 32 / RPW;
  const uint32_t lds_bytes = (2 * 64 + 4 * 32) * HD * 2 + 2 * 64 * 4;
  const bool varlen = a_in.cu != nullptr;
  const int BHk = a_in.B * a_in.Hkv;
  const int64_t nx = (((int64_t)a_in.T + a_in.Cb - 1) / a_in.Cb) * BHk;
  typedef AsyncTileLoader<HD, BM, 256> Loader;
  for (int64_t block = 0; block < nx; block++) {
    const int bh = (int)(block % BHk), chunk = (int)(block / BHk);
    int b = bh / a_in.Hkv;
    const int hkv = bh % a_in.Hkv;
    const KArgs a = seq_args(a_in, b);
    const int t0 = chunk * a.Cb;
    if (t0 >= a.T) continue;
    const int t1 = imin(a.T, t0 + a.Cb), r0 = t0 * a.Gf, r_end = t1 * a.Gf, c_end = t1 * a.Lv;
    if (r_end - r0 > BM) fail("chunk_depth_kernel: a chunk of %d query rows", r_end - r0);
    for (int tid = 0; tid < 256; tid++) {
      const int lane = tid & 63, wave = tid >> 6;
      Loader ld;
      ld.init(tid);
      ctx("chunk_depth_kernel", (int)block, wave, lane, "the chunk's Q, dO, lse, row sums");
      for (int i = 0; i < Loader::N; i++) {
        check_dma("q", a.q + b * a.sq.b + hkv * a.sq.h + (int64_t)r0 * a.sq.t, Loader::anchored_bytes(a.sq.t, r0, r_end),
                  ld.lane_offset((int)a.sq.t * 2, a.D), Loader::rows_before(i) * (int)a.sq.t * 2, 16, (uint32_t)ld.lds_elems(i) * 2,
                  lds_bytes, ld.pads(a.D));
        check_dma("do", a.d_o + b * a.sdo.b + hkv * a.sdo.h + (int64_t)r0 * a.sdo.t, Loader::anchored_bytes(a.sdo.t, r0, r_end),
                  ld.lane_offset((int)a.sdo.t * 2, a.Dv), Loader::rows_before(i) * (int)a.sdo.t * 2, 16,
                  (uint32_t)(BM * HD + ld.lds_elems(i)) * 2, lds_bytes, ld.pads(a.Dv));
      }
      if (tid < BM && r0 + tid < r_end) {
        check_access("lse", a.lse + ((int64_t)b * a.Tq + r0 + tid) * a.Hq + hkv, 4, false);
        check_access("delta", a.delta + ((int64_t)b * a.Hq + hkv) * (varlen ? a.delta_pitch : a.Tq) + r0 + tid, 4, false);
      }
      const int prow = lane / CH, pch = lane % CH;
      const uint32_t wt = (uint32_t)(2 * BM * HD + wave * 32 * HD) * 2;
      WaveTileLoader<HD> own;
      own.init(lane);
      for (int cb = t0 * a.Lv + wave * 32; cb < c_end; cb += 128) {
        const int nrows = imin(32, c_end - cb);
        for (int i = 0; i < NPASS; i++) {
          const int row = i * RPW + prow, lch = pch ^ Tile<HD>::swz(row);
          const bool pad_k = !(lch * 8 < a.D), pad_v = !(lch * 8 < a.Dv);
          ctx("chunk_depth_kernel", (int)block, wave, lane, "depth K / V rows");
          if (a.Lv != a.L) {
            const int w0 = cb / a.Lv, l0 = cb - w0 * a.Lv;
            const int64_t anchor = (int64_t)w0 * a.L, rows_total = (int64_t)a.T * a.L;
            const int vk = own.mapped_offset(i, l0, a.L, a.Lv, nrows, (int)a.skd.t * 2, a.D);
            const int vv = own.mapped_offset(i, l0, a.L, a.Lv, nrows, (int)a.svd.t * 2, a.Dv);
            check_dma("kd", a.kd + b * a.skd.b + hkv * a.skd.h + anchor * a.skd.t,
                      mapped_bytes(anchor, rows_total, (uint32_t)a.skd.t * 2u), vk, 0, 16, wt + i * 1024, lds_bytes, vk == kPadOffset);
            check_dma("vd", a.vd + b * a.svd.b + hkv * a.svd.h + anchor * a.svd.t,
                      mapped_bytes(anchor, rows_total, (uint32_t)a.svd.t * 2u), vv, 0, 16, wt + i * 1024, lds_bytes, vv == kPadOffset);
          } else {
            const int vk = own.lane_offset(i, (int)a.skd.t * 2, a.D), vv = own.lane_offset(i, (int)a.svd.t * 2, a.Dv);
            check_dma("kd", a.kd + b * a.skd.b + hkv * a.skd.h + (int64_t)cb * a.skd.t, (uint32_t)nrows * (uint32_t)a.skd.t * 2u,
                      vk, 0, 16, wt + i * 1024, lds_bytes, pad_k);
            check_dma("vd", a.vd + b * a.svd.b + hkv * a.svd.h + (int64_t)cb * a.svd.t, (uint32_t)nrows * (uint32_t)a.svd.t * 2u,
                      vv, 0, 16, wt + i * 1024, lds_bytes, pad_v);
          }
          ctx("chunk_depth_kernel", (int)block, wave, lane, "depth gradient rows");
          if (cb + row < c_end) {
            const int64_t prow_t = depth_row_of(a, cb + row);
            if (!pad_k) check_access("dkd", a.dkd + b * a.sdkd.b + hkv * a.sdkd.h + prow_t * a.sdkd.t + lch * 8, 16, true);
            if (!pad_v) check_access("dvd", a.dvd + b * a.sdvd.b + hkv * a.sdvd.h + prow_t * a.sdvd.t + lch * 8, 16, true);
          }
        }
      }
    }
  }
}

// the gradient rows of the slots without data of a partially filled stream (launched where the kernels that form
// the depth gradients only visit the slots that hold data)
template <int HD>
void walk_zero_unfilled(const KArgs& a) {
  constexpr int TPR = HD / 8;
  const int64_t rows = a.cu ? (int64_t)(a.delta_pitch / a.Gf) * a.L : (int64_t)a.T * a.L;
  const int batches = a.cu ? 1 : a.B;
  const int64_t nthreads = rows * batches * a.Hkv * TPR;
  for (int64_t gid = 0; gid < (nthreads + 255) / 256 * 256; gid++) {
    const int sub = (int)(gid % TPR);
    int64_t rest = gid / TPR;
    const int h = (int)(rest % a.Hkv);
    rest /= a.Hkv;
    const int64_t row = rest % rows, b = rest / rows;
    if (b >= batches || (int)(row % a.L) < a.Lv) continue;
    ctx("zero_unfilled_slots_kernel", (int)(gid / 256), (int)(gid % 256) >> 6, (int)(gid & 63), "gradient rows of empty slots");
    if (8 * sub < a.D) check_access("dkd", a.dkd + b * a.sdkd.b + h * a.sdkd.h + row * a.sdkd.t + 8 * sub, 16, true);
    if (8 * sub < a.Dv) check_access("dvd", a.dvd + b * a.sdvd.b + h * a.sdvd.h + row * a.sdvd.t + 8 * sub, 16, true);
  }
}

// depth columns outside chunk-visible mode: one column per HD/8 lanes
template <int HD>
void walk_depth_cols(const KArgs& a_in) {
  constexpr int LPC = HD / 8, CPW = 64 / LPC, CPB = 4 * CPW;
  const int BHk = a_in.B * a_in.Hkv;
  const int64_t nx = (((int64_t)a_in.T * a_in.L + CPB - 1) / CPB) * BHk;
  for (int64_t block = 0; block < nx; block++)
    for (int tid = 0; tid < 256; tid++) {
      const int lane = tid & 63, wave = tid >> 6, sub = lane % LPC;
      const int bh = (int)(block % BHk);
      int b = bh / a_in.Hkv;
      const int hkv = bh % a_in.Hkv;
      const KArgs a = seq_args(a_in, b);
      const int64_t c = (int64_t)(block / BHk) * CPB + wave * CPW + lane / LPC;
      if (c >= (int64_t)a.T * a.L) continue;
      const int w = (int)(c / a.L), slot = (int)(c - (int64_t)w * a.L);
      const bool in_k = 8 * sub < a.D, in_v = 8 * sub < a.Dv;
      ctx("depth_cols_kernel", (int)block, wave, lane, "depth column");
      uint16_t* dk_out = a.dkd + b * a.sdkd.b + hkv * a.sdkd.h + c * a.sdkd.t + 8 * sub;
      uint16_t* dv_out = a.dvd + b * a.sdvd.b + hkv * a.sdvd.h + c * a.sdvd.t + 8 * sub;
      if (slot >= a.Lv) {
        if (!a.accum_depth) {
          if (in_k) check_access("dkd", dk_out, 16, true);
          if (in_v) check_access("dvd", dv_out, 16, true);
        }
        continue;
      }
      const bool handed = a.depth_p != nullptr;  // depth_cols_handed_kernel: P and dS from the dQ kernel, no kd, vd, statistics
      if (!handed && in_k) check_access("kd", a.kd + b * a.skd.b + hkv * a.skd.h + c * a.skd.t + 8 * sub, 16, false);
      if (!handed && in_v) check_access("vd", a.vd + b * a.svd.b + hkv * a.svd.h + c * a.svd.t + 8 * sub, 16, false);
      for (int gq = 0; gq < a.Gf; gq++) {
        const int64_t r = (int64_t)w * a.Gf + gq;
        if (in_k) check_access("q", a.q + b * a.sq.b + hkv * a.sq.h + 8 * sub + r * a.sq.t, 16, false);
        if (in_v) check_access("do", a.d_o + b * a.sdo.b + hkv * a.sdo.h + 8 * sub + r * a.sdo.t, 16, false);
        if (handed) {
          const int64_t at = (((int64_t)b * a.Hq + hkv) * a.delta_pitch + (int64_t)w * a.Gf) * a.Lv + (int64_t)slot * a.Gf + gq;
          check_access("hand_p", a.depth_p + at, 2, false);
          check_access("hand_ds", a.depth_ds + at, 2, false);
          continue;
        }
        check_access("lse", a.lse + ((int64_t)b * a.Tq + r) * a.Hq + hkv, 4, false);
        check_access("delta", a.delta + ((int64_t)b * a.Hq + hkv) * a.delta_pitch + r, 4, false);
      }
      if (in_k) check_access("dkd", dk_out, 16, true);
      if (in_v) check_access("dvd", dv_out, 16, true);
    }
}

// the same organised by token (query groups of up to four rows with the depth scores handed over by the dQ kernel)
template <int HD>
void walk_depth_tokens(const KArgs& a_in) {
  constexpr int LPT = HD / 8, TPW = 64 / LPT, TPB = 4 * TPW;
  const int BHk = a_in.B * a_in.Hkv;
  const int64_t nt = (((int64_t)a_in.T + TPB - 1) / TPB) * BHk;
  for (int64_t block = 0; block < nt; block++)
    for (int tid = 0; tid < 256; tid++) {
      const int lane = tid & 63, wave = tid >> 6, sub = lane % LPT;
      const int bh = (int)(block % BHk);
      int b = bh / a_in.Hkv;
      const int hkv = bh % a_in.Hkv;
      const KArgs a = seq_args(a_in, b);
      const int w = (int)(block / BHk) * TPB + wave * TPW + lane / LPT;
      if (w >= a.T) continue;
      const bool in_k = 8 * sub < a.D, in_v = 8 * sub < a.Dv;
      ctx("depth_token_handed_kernel", (int)block, wave, lane, "token");
      for (int g = 0; g < a.Gf; g++) {
        const int64_t r = (int64_t)w * a.Gf + g;
        if (in_k) check_access("q", a.q + b * a.sq.b + hkv * a.sq.h + 8 * sub + r * a.sq.t, 16, false);
        if (in_v) check_access("do", a.d_o + b * a.sdo.b + hkv * a.sdo.h + 8 * sub + r * a.sdo.t, 16, false);
      }
      const int64_t blk = (((int64_t)b * a.Hq + hkv) * a.delta_pitch + (int64_t)w * a.Gf) * a.Lv;
      for (int slot = 0; slot < a.L; slot++) {
        if (slot >= a.Lv && a.accum_depth) continue;
        if (slot < a.Lv)
          for (int g = 0; g < a.Gf; g++) {
            check_access("hand_p", a.depth_p + blk + (int64_t)slot * a.Gf + g, 2, false);
            check_access("hand_ds", a.depth_ds + blk + (int64_t)slot * a.Gf + g, 2, false);
          }
        const int64_t c = (int64_t)w * a.L + slot;
        if (in_k) check_access("dkd", a.dkd + b * a.sdkd.b + hkv * a.sdkd.h + c * a.sdkd.t + 8 * sub, 16, true);
        if (in_v) check_access("dvd", a.dvd + b * a.sdvd.b + hkv * a.sdvd.h + c * a.sdvd.t + 8 * sub, 16, true);
      }
    }
}

void reset_writes(const char* name) {
  Region& r = region(name);
  std::fill(r.writes.begin(), r.writes.end(), 0);
}
// every element of the rows that exist must have been written exactly once (elements of a row past the head dim do
// not exist: the regions are dense [rows, heads, D])
void require_full(const char* name) {
  Region& r = region(name);
  if (!r.track) return;
  for (size_t i = 0; i < r.writes.size(); i++)
    if (r.writes[i] != 1) fail("%s unit %zu written %d times after the launch", name, i, (int)r.writes[i]);
}

template <int HD>
void walk_all(const Case& c, const KArgs& a) {
  const bool packed = a.cu != nullptr;
  // byte span of the widest streamed (batch, head) slice decides the addressing variant (as the launchers do)
  const int64_t span = 2 * std::max(std::max((int64_t)a.T * a.sk.t, (int64_t)a.T * a.sv.t),
                                    std::max((int64_t)a.T * a.L * a.skd.t, (int64_t)a.T * a.L * a.svd.t));
  const bool wide_addr = span > 0x7fffffffll;
  if (wide_addr) fail("slices beyond 2 GiB are not walked (the fake tensors would not fit the walker's write maps)");
  const bool small = use_small_rows(a.Tq, (long long)a.B * a.Hq, a.compute_units);
  // ---- forward
  g_ctx = "forward";
  auto fwd_lds = [&](int W, int NST) {  // the ring, or (64-wide tiles) two sets of private tiles per wave
    const uint32_t ring = (uint32_t)NST * 2 * 64 * HD * 2, own = HD <= 64 ? 2u * W * 2 * 32 * HD * 2 : 0u;
    return std::max(ring, own);
  };
  if constexpr (HD > 128) {
    walk_row_kernel<HD, RowWide, false>(a, false, 16, false, RowWide::NST * 2 * 64 * HD * 2, "fwd_wide_kernel");
  } else {
    if (small)
      walk_row_kernel<HD, RowSmall<HD>, false>(a, false, 32, true, fwd_lds(RowSmall<HD>::W, RowSmall<HD>::NST), "fwd_kernel(small)");
    else
      walk_row_kernel<HD, RowLargePP, false>(a, false, 32, true, fwd_lds(RowLargePP::W, RowLargePP::NST), "fwd_kernel");
  }
  require_full("o");
  require_full("lse");
  // ---- backward
  // the row sums: by the delta kernel when that stage is run alone, else inside the dQ kernel
  walk_delta<HD>(a);
  require_full("delta");
  reset_writes("delta");
  auto ring_or_own = [&](int W, int NST) {
    const uint32_t ring = (uint32_t)NST * 2 * 64 * HD * 2, own = (uint32_t)W * (HD <= kDepthGradsInDqMaxWidth ? 2 * 64 + 16 : 64) * HD * 2;
    return (uint32_t)W * 64 * HD * 2 <= 128 * 1024 ? std::max(ring, own) : ring;
  };
  if constexpr (HD > 128) {
    walk_row_kernel<HD, RowWide, false>(a, true, 16, false, ring_or_own(RowWide::W, RowWide::NST), "dq_kernel(wide)");
  } else {
    if (small)
      walk_row_kernel<HD, RowSmall<HD>, false>(a, true, 32, true, ring_or_own(RowSmall<HD>::W, RowSmall<HD>::NST), "dq_kernel(small)");
    else
      walk_row_kernel<HD, RowLarge, false>(a, true, 32, true, ring_or_own(RowLarge::W, RowLarge::NST), "dq_kernel");
  }
  require_full("dq");
  require_full("delta");
  if (a.depth_p) {
    require_full("hand_p");
    require_full("hand_ds");
  }
  if (takes_dkv_flat(a, HD, a.cu ? 1 : a.dkv_split)) {
    if constexpr (HD == 64) walk_dkv_flat<HD>(a);
  } else {
    walk_dkv<HD>(a);
  }
  if (a.dkv_split > 1 && a.has_seq) {
    require_full("part");
    walk_reduce<HD>(a);
  }
  if (a.has_seq) {
    require_full("dk");
    require_full("dv");
  }
  if (a.L > 0) {
    if ((a.chunk || depth_grads_in_dq(a, HD)) && a.Lv != a.L) walk_zero_unfilled<HD>(a);
    if (a.chunk) {
      if constexpr (HD <= 128) {
        if (depth_by_chunks(a, HD)) walk_chunk_depth<HD>(a);
      }
    } else if (!depth_grads_in_dq(a, HD)) {
      if (a.depth_p && a.Gf <= 4)
        walk_depth_tokens<HD>(a);
      else
        walk_depth_cols<HD>(a);
    }
    require_full("dkd");
    require_full("dvd");
  }
  (void)packed;
  (void)c;
}

}  // namespace

int main(int argc, char** argv) {
  if (argc < 14) {
    fprintf(stderr, "usage: %s HD D Dv H G L Lv mode chunk_tokens split packed n len0 [len1 ...]\n", argv[0]);
    return 2;
  }
  Case c;
  int i = 1;
  c.HD = atoi(argv[i++]);
  c.D = atoi(argv[i++]);
  c.Dv = atoi(argv[i++]);
  c.H = atoi(argv[i++]);
  c.G = atoi(argv[i++]);
  c.L = atoi(argv[i++]);
  c.Lv = atoi(argv[i++]);
  c.mode = atoi(argv[i++]);
  c.cb = atoi(argv[i++]);
  const int split = atoi(argv[i++]);
  c.packed = atoi(argv[i++]);
  c.nseq = atoi(argv[i++]);
  for (; i < argc; i++) c.len.push_back(atoi(argv[i]));
  c.cu.push_back(0);
  c.Tmax = 0;
  if (c.packed) {
    if ((int)c.len.size() != c.nseq) return 2;
    for (int n : c.len) {
      c.cu.push_back(c.cu.back() + n);
      c.Tmax = std::max(c.Tmax, n);
    }
    c.total = c.cu.back();
  } else {
    c.Tmax = c.len[0];
    c.total = c.Tmax;
  }
  KArgs a = make_args(c);
  a.dkv_split = split > 0 && !c.packed ? split : 1;
  if (a.dkv_split > 1)
    a.dkv_part = (float*)add_region("part", 20, (uint64_t)2 * a.dkv_split * a.B * a.Hkv * a.T * c.HD * 4, 4, true);
  switch (c.HD) {
    case 64: walk_all<64>(c, a); break;
    case 128: walk_all<128>(c, a); break;
    case 256: walk_all<256>(c, a); break;
    default: return 2;
  }
  printf("OK checked=%lld dma_in_range=%lld dma_zero_filled=%lld\n", g_checked, g_dma_in, g_dma_out);
  return 0;
}
