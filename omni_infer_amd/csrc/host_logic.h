// The integer logic of the library that needs no GPU to run: kernel choice and workspace sizes, the numbering of
// the tile kernel's tiles, the weight rules of row blocks, the workspace layout of the whole-layer entry, the
// bookkeeping of the arrival counters and the placement tables.
//
// This header is plain C++17.  The .hip sources include it (after the HIP runtime header, so that the functions
// the kernels call are compiled for both sides); a host build with g++ includes it alone and runs the same code
// under the address and undefined-behaviour sanitizers (tests/host/host_logic_test.cpp).
#pragma once
#include <stddef.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <mutex>
#include <unordered_map>
#include <vector>

#include "../../include/omni_moe_hip.h"

#if defined(__HIPCC__)
#define OMNI_HD __host__ __device__ __forceinline__
#else
#define OMNI_HD inline
#endif

void omni_set_error(const char* fmt, ...);
#ifndef OMNI_FAIL
#define OMNI_FAIL(code, ...)        \
  do {                              \
    omni_set_error(__VA_ARGS__);    \
    return (code);                  \
  } while (0)
#endif

namespace omni_host {

inline size_t align256(size_t v) { return (v + 255) / 256 * 256; }

template <typename T>
OMNI_HD T imin(T a, T b) { return a < b ? a : b; }

// ------------------------------------------------------------------------------------------------
// Row blocks by weight.  A group's last block is light when it has at most light_max rows -- except in a group of
// exactly one full block and a few rows more: there the small block stays next to the full one, whose weight
// panel it shares (deferred to the end it would fetch that panel a second time, and with one full block per
// group that doubles the traffic).
// ------------------------------------------------------------------------------------------------
OMNI_HD bool last_block_is_light(int c, int BM, int light_max) {
  return (c % BM) > 0 && (c % BM) <= light_max && c / BM != 1;
}
OMNI_HD int heavy_blocks(int c, int BM, int light_max) {
  return c / BM + ((c % BM) > 0 && !last_block_is_light(c, BM, light_max));
}
OMNI_HD int light_blocks(int c, int BM, int light_max) { return last_block_is_light(c, BM, light_max); }

// ------------------------------------------------------------------------------------------------
// Which tile a block id of the tile kernel names.
// Real tiles (row blocks that exist x column tiles) get the ids [0, n_real): first the tiles of the heavy row
// blocks, then those of the light ones; the last `left` real tiles (a last partial round of at most half the
// chip) are each split `split` ways along the reduction, the helper shares have the ids [n_real, total).
// ------------------------------------------------------------------------------------------------
struct TileGeom {
  int gx;         // column tiles
  int pc;         // column tiles of a patch (divides gx)
  int slots;      // blocks the chip runs at once (0: no split tiles)
  int split_max;  // most shares of a split tile
  bool tail;      // scratch for split tiles is there
};
struct TileCount { int n_heavy, n_real, left, split, total; };
struct TileSel { int bx, by, share, tail_tile; bool light; };
constexpr int TILE_LIGHT_MAX = 96;
constexpr int TILE_PR = 4;  // row blocks of a patch

// nk_units: the pieces a reduction can be cut into (k-steps, or pairs of k-steps in the line layout)
OMNI_HD TileCount tile_count(const TileGeom& g, int total_h, int total_l, int nk_units) {
  TileCount t;
  t.n_heavy = total_h * g.gx;
  t.n_real = (total_h + total_l) * g.gx;
  t.left = 0;
  t.split = 1;
  if (g.tail && g.slots > 0) {
    t.left = t.n_real % g.slots;
    if (t.left > 0 && 2 * t.left <= g.slots) t.split = imin(imin(g.split_max, g.slots / t.left), nk_units);
    if (t.split < 2) { t.split = 1; t.left = 0; }
  }
  t.total = t.n_real + t.left * (t.split - 1);
  return t;
}

// false: the id names no work.  Each set (heavy, light) is numbered in three runs:
//   A: whole patches of TILE_PR row blocks x pc column tiles, in rounds of 8 dealt to the 8 XCDs (the tiles of a
//      patch are 8 ids apart: one XCD runs them all);
//   B: the whole patches that do not fill a round of 8, one after the other;
//   C: the row blocks past the last whole patch row, row by row.
OMNI_HD bool tile_select(const TileGeom& g, const TileCount& tc, int total_h, int total_l, int id, TileSel& s) {
  const int gx = g.gx, pc = g.pc, npc = gx / pc, per_patch = TILE_PR * pc;
  s.share = 0;
  s.tail_tile = -1;
  s.bx = s.by = 0;
  s.light = false;
  if (id < 0) return false;
  if (id >= tc.n_real) {
    const int h = id - tc.n_real;
    if (tc.split == 1 || h >= tc.left * (tc.split - 1)) return false;
    s.tail_tile = h / (tc.split - 1);
    s.share = 1 + h % (tc.split - 1);
    id = tc.n_real - tc.left + s.tail_tile;
  } else if (tc.split > 1 && id >= tc.n_real - tc.left) {
    s.tail_tile = id - (tc.n_real - tc.left);
  }
  s.light = id >= tc.n_heavy;
  const int t = s.light ? id - tc.n_heavy : id;   // id inside the set
  const int RB = s.light ? total_l : total_h;     // row blocks of the set
  const int bulk_rows = RB / TILE_PR * TILE_PR;
  const int patches = bulk_rows / TILE_PR * npc, patches8 = patches / 8 * 8;
  const int nA = patches8 * per_patch, nB = (patches - patches8) * per_patch;
  if (t < nA + nB) {
    int patch, q;
    if (t < nA) {
      const int j = t >> 3;
      patch = (j / per_patch) * 8 + (t & 7);
      q = j % per_patch;
    } else {
      patch = patches8 + (t - nA) / per_patch;
      q = (t - nA) % per_patch;
    }
    s.by = (patch / npc) * TILE_PR + q / pc;
    s.bx = (patch % npc) * pc + q % pc;
  } else {
    s.by = bulk_rows + (t - nA - nB) / gx;
    s.bx = (t - nA - nB) % gx;
  }
  return true;
}

// k-steps [k_first, k_end) of share `share` of a tile split `split` ways; a reduction of nk k-steps is cut in
// units of ku k-steps (2 in the line layout, whose stages hold two k-steps).  split == 1: the whole reduction.
OMNI_HD void tile_share_k_range(int nk, int ku, int split, int share, int& k_first, int& k_end) {
  k_first = share * (nk / ku) / split * ku;
  k_end = (share + 1) * (nk / ku) / split * ku;
  if (share == split - 1) k_end = nk;
}

// ------------------------------------------------------------------------------------------------
// Block numbering of the weight-streaming kernel when the whole launch is resident at once
// A compute unit draws at most about 30 GB/s from memory, a ninth above its share of what the chip delivers
// when every unit pulls (27 GB/s of 6.97 TB/s); blocks stay where the dispatcher puts them.  A launch of
// q * cus + r blocks therefore leaves r units with q + 1 blocks and runs as long as those take: 33 x 32 blocks of
// the decode GEMM1 read at 6.45 TB/s where 32 x 32 read at 6.95 (measured with a kernel that only reads).
// So the last r blocks ("overflow") are each cut `split` ways along the reduction: the block itself takes the
// first share, helper blocks with the ids [n_real, n_real + r * (split - 1)) the others, every unit ends up
// with q blocks and a few shares, and whoever arrives last at an overflow block's counter adds up the partial
// sums (integers: any order) and runs the epilogue.
// ------------------------------------------------------------------------------------------------
// arrival counters of the overflow blocks: one word each, GEMM1's and GEMM2's apart (one clearing serves both)
constexpr int STREAM_BAL_CNT_WORDS = 256;   // per kind of GEMM; a launch with more overflow blocks is not split
struct StreamBalance { int cap, n_over, split, total; };  // ids [0, cap) whole blocks; n_over overflow blocks; all ids
struct StreamSel { int task, share, over; };              // block of the launch, its k share, overflow index or -1

// Whether the cut pays, and how many shares: in units of the time a busy compute unit takes for one block, the
// launch takes q + 1 without the cut; with `sp` shares per overflow block it takes what the fullest unit then holds,
// q + ceil(r sp / cus) / sp, but no less than 1.08 times the mean load q + r / cus (a unit alone draws about a
// tenth more than its share of the chip's rate), plus what a share costs on top of its bytes (its first loads, the
// hand-over of its partial sums: 2.7 us measured, which a busy unit streams 83 KB in) for every share a unit gets.
// The cut is made when the best `sp` saves at least 2 % of a block's time.  The two constants were set on the
// DeepSeek-V3 GEMM1 (917 KB blocks, 256 units) and give the sign of all sixteen measured cases: layer time with 2 /
// 4 shares against uncut at 1 token (9 x 32 blocks) -7.0 / -10.0 us, 2 tokens (14 x 32) +6.6 / +5.2, 4 tokens (21 x 32)
// +5.8 / +5.8, 8 tokens (31 x 32) +4.9 / +11.4, 16 tokens (33 x 32) -7.0 / -9.1, 32 tokens -5.5 / -5.6, 64 tokens
// (34 x 32) -7.2 / -6.1, 96 tokens (36 x 32) -3.7 / +2.4.
// n_real: blocks with rows; resident: blocks a unit holds at once; nchunks: chunks of 4 k-steps of the reduction;
// dc: chunks a wavefront keeps in flight; share_cap: shares the partial-sum scratch holds (0: no scratch);
// block_kb: weight bytes a block streams, in KiB
OMNI_HD StreamBalance stream_balance(int n_real, int cus, int resident, int nchunks, int dc, int share_cap, int block_kb) {
  StreamBalance b{n_real, 0, 1, n_real};
  if (cus <= 0 || n_real <= cus || share_cap <= 0 || block_kb <= 0) return b;
  const int q = n_real / cus, r = n_real % cus;
  if (r == 0 || q + 1 > resident) return b;           // even already, or more than one round: the dispatcher evens out
  if (r > STREAM_BAL_CNT_WORDS) return b;
  // everything in thousandths of a block's time
  const long long whole = 1000LL * (q + 1);
  const long long mean_floor = 1080LL * n_real / cus;
  long long best = whole - 20;
  int split = 0;
  for (int sp = 2; sp <= 4; sp += 2) {
    if (nchunks % sp != 0 || nchunks / sp < 2 * dc || r * sp > share_cap) continue;
    const long long shares_per_unit = ((long long)r * sp + cus - 1) / cus;
    const long long fullest = 1000LL * q + 1000LL * shares_per_unit / sp;
    const long long cost = (fullest > mean_floor ? fullest : mean_floor) + 83LL * 1000 * r * sp / ((long long)cus * block_kb);
    if (cost < best) { best = cost; split = sp; }
  }
  if (split == 0) return b;
  b.cap = n_real - r;
  b.n_over = r;
  b.split = split;
  b.total = n_real + r * (split - 1);
  return b;
}
OMNI_HD bool stream_select(const StreamBalance& b, int n_real, int id, StreamSel& s) {
  s.task = id;
  s.share = 0;
  s.over = -1;
  if (id < 0 || id >= b.total) return false;
  if (id >= n_real) {
    const int h = id - n_real;            // helper: consecutive ids serve different overflow blocks
    s.over = h % b.n_over;
    s.share = 1 + h / b.n_over;
    s.task = b.cap + s.over;
  } else if (id >= b.cap) {
    s.over = id - b.cap;
  }
  return true;
}
// most helper blocks a launch can need
OMNI_HD int stream_balance_max_helpers(int cus) { return cus > 1 ? (cus - 1) * 3 : 0; }

// ------------------------------------------------------------------------------------------------
// Kernel choice of the grouped GEMMs and what follows from it
// ------------------------------------------------------------------------------------------------
// Tuning aids, read from the environment once (the first GEMM call of the process) and never again:
//   OMNI_MOE_FORCE_KERNEL  1 stream kernel, 2 tile kernel, whatever the row counts
//   OMNI_MOE_G1 / _G2      "mt,nt,d[,S]" of the stream kernel of GEMM1 / GEMM2; a combination that is not
//                          compiled in is refused here, with a message, and the default is used
//   OMNI_MOE_TILE_WN       2: tile kernel of 256 x 128 instead of 256 x 256
//   OMNI_MOE_TILE_LINES    0: the 256 x 256 tile kernel keeps the fragment layout of the activation operand
//   OMNI_MOE_TILE_MFMA16   0: the line-layout tile kernel multiplies with v_mfma_i32_32x32x32_i8 instead of 16x16x64
//   OMNI_MOE_TILE_TAIL     0: tiles of the last partial round are not split along k
//   OMNI_MOE_TILE_SPLIT    most shares of such a tile (default 4)
//   OMNI_MOE_ROWQ          threads per row of swiglu_quant_rows
//   OMNI_MOE_TILE_FROM      "g1,g2": expected rows per routed group above which GEMM1 / GEMM2 run the tile kernel
//   OMNI_MOE_STREAM_BALANCE 0: the overflow blocks of a resident stream launch are not split along k
//   OMNI_MOE_EQUAL_PROGRESS bit 0: the stream kernel of GEMM1 lowers the issue priority of its wavefronts as they
//                          advance (default 1), bit 1: that of GEMM2 too (measured slower in every geometry)
struct Tuning {
  int force_kernel = 0, tile_wn = 4, tile_tail = 1, tile_split = 4, rowq = 0, equal_progress = 1, tile_lines = 1;
  int tile_mfma16 = 1;
  int stream_balance = 1;
  int tile_from[3] = {0, 48, 56};  // expected rows per routed group above which GEMM1 / GEMM2 run the tile kernel
  bool have[3] = {false, false, false};
  int mt[3] = {0, 0, 0}, nt[3] = {0, 0, 0}, d[3] = {0, 0, 0}, S[3] = {0, 0, 0};
};

// the compiled (KIND, MT, NT, D) combinations of gemm_stream
#define OMNI_STREAM_VARIANTS(X)                                                        \
  X(1, 1, 1, 4) X(1, 2, 1, 4) X(1, 4, 1, 4) X(1, 1, 1, 8) X(1, 2, 1, 8)                \
  X(1, 1, 2, 4) X(1, 2, 2, 4) X(1, 4, 2, 4) X(1, 2, 2, 8)                              \
  X(2, 1, 1, 4) X(2, 2, 1, 4) X(2, 4, 1, 4) X(2, 1, 2, 4) X(2, 2, 2, 4) X(2, 4, 2, 4)  \
  X(2, 1, 4, 4) X(2, 2, 4, 4) X(2, 2, 2, 8) X(2, 1, 2, 8) X(2, 2, 1, 8)
inline bool stream_variant_exists(int kind, int mt, int nt, int d) {
#define OMNI_HAS_VARIANT(K_, MT_, NT_, D_) if (kind == K_ && mt == MT_ && nt == NT_ && d == D_) return true;
  OMNI_STREAM_VARIANTS(OMNI_HAS_VARIANT)
#undef OMNI_HAS_VARIANT
  return false;
}

inline Tuning read_tuning() {
  Tuning r;
  auto geti = [](const char* name, int dflt) {
    const char* v = getenv(name);
    return v ? atoi(v) : dflt;
  };
  r.force_kernel = geti("OMNI_MOE_FORCE_KERNEL", 0);
  r.tile_wn = geti("OMNI_MOE_TILE_WN", 4);
  r.tile_tail = geti("OMNI_MOE_TILE_TAIL", 1);
  r.tile_mfma16 = geti("OMNI_MOE_TILE_MFMA16", 1);
  r.tile_split = geti("OMNI_MOE_TILE_SPLIT", 4);
  r.rowq = geti("OMNI_MOE_ROWQ", 0);
  r.equal_progress = geti("OMNI_MOE_EQUAL_PROGRESS", 1);
  r.tile_lines = geti("OMNI_MOE_TILE_LINES", 1);
  r.stream_balance = geti("OMNI_MOE_STREAM_BALANCE", 1);
  if (const char* e = getenv("OMNI_MOE_TILE_FROM")) {
    int g1 = 0, g2 = 0;
    if (sscanf(e, "%d,%d", &g1, &g2) == 2 && g1 > 0 && g2 > 0) { r.tile_from[1] = g1; r.tile_from[2] = g2; }
  }
  for (int kind = 1; kind <= 2; ++kind) {
    const char* name = kind == 1 ? "OMNI_MOE_G1" : "OMNI_MOE_G2";
    const char* e = getenv(name);
    if (!e) continue;
    int mt = 0, nt = 0, d = 0, S = 0;
    if (sscanf(e, "%d,%d,%d,%d", &mt, &nt, &d, &S) >= 3 && stream_variant_exists(kind, mt, nt, d)) {
      r.have[kind] = true;
      r.mt[kind] = mt; r.nt[kind] = nt; r.d[kind] = d; r.S[kind] = S;
    } else {
      fprintf(stderr, "omni_moe: %s=\"%s\" names no compiled stream kernel; ignored\n", name, e);
    }
  }
  return r;
}
// read at the first GEMM call of the process; omni_moe_reload_tuning() reads the environment again
inline Tuning& tuning_store() {
  static Tuning t = read_tuning();
  return t;
}
inline const Tuning& tuning() { return tuning_store(); }

struct Plan {
  bool tile;
  int mt, nt, d;  // stream kernel parameters
  int S;          // k splits (GEMM1 stream kernel only)
  int64_t per;    // expected rows of a busy group
};

// Decides the kernel from what the host knows: the expected rows of a busy group.  The stream kernel covers a
// group with blocks of 16*mt rows.  kind 1: GEMM1 (N = 2I channels, Kdim = H), kind 2: GEMM2 (T = M_cap, K = 1).
inline Plan make_plan(int kind, int T, int K, int G, int extra_rows, int Kdim, int N) {
  const int units = (kind == 1) ? N / 32 : N / 16;  // kind 1: (gate, up) strip pairs; kind 2: strips
  // expected rows of a routed group (uniform routing); the shared group, when there is one, has T rows
  int64_t avg = (G > 0) ? ((int64_t)T * K + G - 1) / G : 0;
  if (avg > (int64_t)T) avg = T;
  const int64_t per = (G > 0) ? avg : extra_rows;
  Plan p{};
  p.per = per;
  // Measured on the DeepSeek-V3 shape (32 routed groups + the shared one): the stream kernel wins GEMM1 up to 48
  // expected rows per routed group and GEMM2 up to 56 (row blocks of 64 rows from 25 expected rows on, so that
  // nearly every group is one block and its weights are read once; past 48 too many groups spill into a second
  // block and the launch into a second round: 200 tokens 365 us against 336 us with tiles); above that the tile
  // kernel does.
  const Tuning& tn = tuning();
  p.tile = (G > 0) ? per > tn.tile_from[kind] : per > 128;
  const int force = tn.force_kernel;
  if (force == 1) p.tile = false;
  if (force == 2) p.tile = true;
  const bool tile_ok = units % ((kind == 1) ? 4 : 8) == 0;  // the tile kernel takes 64 / 128 channels at least
  if (p.tile && !tile_ok) p.tile = false;
  // the stream kernel walks the reduction in chunks of 256: other lengths go to the tile kernel
  if (!p.tile && Kdim % 256 != 0 && tile_ok && force != 1) p.tile = true;
  p.mt = per <= 10 ? 1 : (per <= 24 ? 2 : 4);
  p.S = 1;
  p.nt = 1;
  p.d = 4;
  int s_env = 0;
  if (tn.have[kind]) { p.mt = tn.mt[kind]; p.nt = tn.nt[kind]; p.d = tn.d[kind]; s_env = tn.S[kind]; }
  if (Kdim % (64 * p.d) != 0) p.d = 4;
  if (kind == 1 && !p.tile && Kdim % 256 == 0 && units % (4 * p.nt) == 0) {
    // measured on MI355X: extra k splits cost more in block start-up than they win back in the
    // tail of the launch, so the default is one share (the tuning aid OMNI_MOE_G1 can ask for more)
    const int nchunks = Kdim / 256, dc = p.d / 4;
    const int want = s_env > 0 ? s_env : 1;
    int best = 1;
    for (int sdiv = 1; sdiv <= nchunks; ++sdiv) {
      if (nchunks % sdiv != 0 || (nchunks / sdiv) % dc != 0 || nchunks / sdiv < 2 * dc) continue;
      if (sdiv <= want) best = sdiv;
    }
    p.S = best;
  }
  return p;
}

// the line layout of the activation operand needs whole super-steps of 128 (OMNI_MOE_TILE_LINES=0: never)
inline bool tile_lines(int Kdim) { return tuning().tile_lines && Kdim % 128 == 0; }

// wavefront columns of the large tile: 4 (256 channels per block) when the channel count allows, else 2
inline int tile_wn(int kind, int units) {
  const int wide = (kind == 1) ? 8 : 16;  // units per 256-channel block
  return (tuning().tile_wn == 4 && units % wide == 0) ? 4 : 2;
}

// Scratch of the split tiles of a launch: arrival counters, then one slot of partial accumulators per
// share.  At most `tile_slots` shares exist (splits x split tiles <= slots), a slot is the 256 x 64*WN
// int32 tile of a block, and the slot count is capped so that the area has one size for every shape.
// (the counters of GEMM1 and of GEMM2 are different words, so that one clearing in front of both launches serves)
constexpr int TILE_TAIL_CNT_WORDS = 1024;                                  // per kind of GEMM
constexpr size_t TILE_TAIL_CNT_BYTES = 2 * TILE_TAIL_CNT_WORDS * sizeof(int32_t);
constexpr size_t TILE_TAIL_PART_BYTES = (size_t)64 << 20;
constexpr size_t TILE_TAIL_BYTES = TILE_TAIL_CNT_BYTES + TILE_TAIL_PART_BYTES;
// the entry on the library's static scratch refuses every shape that selects the tile kernel by size alone
static_assert(TILE_TAIL_BYTES > (size_t)OMNI_STATIC_SCRATCH_BYTES, "a tile-kernel call must not fit the static scratch");

// Scratch of the overflow blocks of a stream launch (stream_balance): the counter words of GEMM1 and of GEMM2,
// then room for the partial sums of the k shares.  It ends the GEMM1 workspace of a stream plan with one k share.
constexpr size_t STREAM_BAL_PART_BYTES = (size_t)8 << 20;
constexpr size_t STREAM_BAL_CNT_BYTES = 2 * STREAM_BAL_CNT_WORDS * sizeof(int32_t);
constexpr size_t STREAM_BAL_BYTES = STREAM_BAL_CNT_BYTES + STREAM_BAL_PART_BYTES;
inline size_t gemm1_stream_sums_bytes(const Plan& p, int64_t M_cap, int I) {
  return (size_t)p.S * M_cap * 2 * I * sizeof(int32_t) + 256;
}
// byte offset of that scratch in the GEMM1 workspace, or 0 when the plan has none
inline size_t gemm1_stream_bal_at(const Plan& p, int64_t M_cap, int I) {
  return (!p.tile && p.S == 1) ? align256(gemm1_stream_sums_bytes(p, M_cap, I)) : 0;
}
inline size_t gemm1_ws_bytes(const Plan& p, int64_t M_cap, int I) {
  if (p.tile) {
    // y = silu(gate) * up before the row quantiser, then the scratch of the split tiles
    return align256((size_t)M_cap * I * sizeof(float) + 256) + TILE_TAIL_BYTES;
  }
  const size_t at = gemm1_stream_bal_at(p, M_cap, I);
  return at ? at + STREAM_BAL_BYTES : gemm1_stream_sums_bytes(p, M_cap, I);
}
inline size_t gemm1_workspace_bytes(int T, int K, int G, int extra_rows, int64_t M_cap, int H, int I) {
  if (M_cap < 0 || I <= 0 || H <= 0 || T < 0 || K <= 0 || G < 0) return 0;
  return gemm1_ws_bytes(make_plan(1, T, K, G, extra_rows, H, 2 * I), M_cap, I);
}
inline size_t gemm2_workspace_bytes(int G, int extra_rows, int64_t M_cap, int H, int I) {
  if (M_cap < 0 || I <= 0 || H <= 0 || G < 0) return 0;
  return make_plan(2, (int)M_cap, 1, G, extra_rows, I, H).tile ? TILE_TAIL_BYTES : 0;
}

// ------------------------------------------------------------------------------------------------
// The sort by expert: sizes of its paths
// ------------------------------------------------------------------------------------------------
constexpr int PERM_GMAX = 256;             // local experts per call
constexpr int PERM_NB = PERM_GMAX + 1;     // buckets incl. the dropped one
constexpr int PERM_CH_MULTI = 1024;        // assignments per block in the multi-block path
constexpr int PERM_CH_SINGLE = 4096;       // largest input of the single-block path
inline size_t permute_workspace_bytes(int T, int K) {
  const int64_t n = (int64_t)T * K;
  if (n <= PERM_CH_SINGLE) return 256;
  const int64_t nblk = (n + PERM_CH_MULTI - 1) / PERM_CH_MULTI;
  return (size_t)((nblk + 1) * PERM_NB * sizeof(int32_t));
}

// ------------------------------------------------------------------------------------------------
// Workspace of the whole-layer entry: byte offsets of its parts, each 256-byte aligned
// ------------------------------------------------------------------------------------------------
struct LayerWs {
  size_t x_q, x_s, sorted_src, src_to_dst, counts, offsets, perm_ws, h_q, h_s, g1_ws, rows, total;
  size_t perm_bytes, g1_bytes;
  int64_t M_cap;
  int rows_dtype;
};
// rows_dtype: the caller's choice for the expert rows between GEMM2 and the combine, fp32 (the
// numerics of the fused GEMM2+finalize operator) or bf16 (those of the separate GEMM2 and finalize
// operators, half the bytes of the largest intermediate).
inline LayerWs layer_layout(int T, int K, int G, int H, int I, int with_shared, int rows_dtype) {
  LayerWs L{};
  L.M_cap = (int64_t)T * K + (with_shared ? T : 0);
  size_t o = 0;
  auto take = [&](size_t bytes) { size_t at = o; o += align256(bytes); return at; };
  L.x_q = take((size_t)T * H);
  L.x_s = take((size_t)T * 4);
  L.sorted_src = take((size_t)T * K * 4);
  L.src_to_dst = take((size_t)T * K * 4);
  L.counts = take((size_t)G * 4);
  L.offsets = take((size_t)(G + 1) * 4);
  L.perm_bytes = permute_workspace_bytes(T, K);
  L.perm_ws = take(L.perm_bytes);
  L.h_q = take((size_t)L.M_cap * I);
  L.h_s = take((size_t)L.M_cap * 4);
  L.g1_bytes = gemm1_workspace_bytes(T, K, G, with_shared ? T : 0, L.M_cap, H, I);
  const size_t g2_bytes = gemm2_workspace_bytes(G, with_shared ? T : 0, L.M_cap, H, I);
  if (g2_bytes > L.g1_bytes) L.g1_bytes = g2_bytes;
  L.g1_ws = take(L.g1_bytes);
  L.rows_dtype = rows_dtype;
  L.rows = take((size_t)L.M_cap * H * (L.rows_dtype == OMNI_DT_F32 ? 4 : 2));
  L.total = o;
  return L;
}

// ------------------------------------------------------------------------------------------------
// Arrival counters of the launch that routes, quantises and sorts: which word of a device's counter array a
// call uses.  Every launch needs a word that is zero when it starts and leaves it at zero when it ends, so two
// launches may share a word exactly when they cannot overlap in time.
//   Eager calls take the words [0, EAGER_SLOTS) in turn: calls on one stream are ordered, and calls on different
//   streams get different words as long as fewer than EAGER_SLOTS of them are in flight.
//   A call recorded into a stream capture keeps its word for every replay of the graph, so it gets one from a
//   pool that eager calls never touch: one word per (capture, stream) pair.  The launches that one stream
//   records into one capture are ordered among themselves in every replay, and a graph cannot run concurrently
//   with itself, so they can share the word; another capture, or another stream of the same capture, gets
//   another word.  When the pool is used up, take() says so (-1) and the caller runs the launches that need no
//   counter instead.
// ------------------------------------------------------------------------------------------------
class ArriveBook {
 public:
  static constexpr int EAGER_SLOTS = 256;
  static constexpr int CAPTURE_SLOTS = 3840;
  static constexpr int TOTAL_SLOTS = EAGER_SLOTS + CAPTURE_SLOTS;

  // capture_id 0: the call is not being captured
  int take(unsigned long long capture_id, uintptr_t stream) {
    std::lock_guard<std::mutex> lock(mu_);
    if (capture_id == 0) {
      const int s = (int)(next_eager_ % EAGER_SLOTS);
      ++next_eager_;
      return s;
    }
    const Key key{capture_id, stream};
    auto it = capture_slot_.find(key);
    if (it != capture_slot_.end()) return it->second;
    if (used_capture_ >= CAPTURE_SLOTS) return -1;
    const int s = EAGER_SLOTS + used_capture_++;
    capture_slot_.emplace(key, s);
    return s;
  }
  int capture_slots_used() {
    std::lock_guard<std::mutex> lock(mu_);
    return used_capture_;
  }

 private:
  struct Key {
    unsigned long long id;
    uintptr_t stream;
    bool operator==(const Key& o) const { return id == o.id && stream == o.stream; }
  };
  struct KeyHash {
    size_t operator()(const Key& k) const { return (size_t)(k.id * 0x9E3779B97F4A7C15ull) ^ (size_t)(k.stream >> 4); }
  };
  std::mutex mu_;
  unsigned next_eager_ = 0;
  int used_capture_ = 0;
  std::unordered_map<Key, int, KeyHash> capture_slot_;
};

// ------------------------------------------------------------------------------------------------
// Placement tables (host arrays): see omni_placement_tables in the public header
// ------------------------------------------------------------------------------------------------
inline int placement_tables(const int32_t* pattern, int world, int layers, int experts, int rank, int devices_per_host,
                            int num_deploy, int32_t* position_to_expert, int32_t* selector) {
  if (!pattern || !selector) OMNI_FAIL(OMNI_E_INVALID, "placement_tables: null pointer");
  if (world < 1 || layers < 1 || experts < 1 || devices_per_host < 1)
    OMNI_FAIL(OMNI_E_INVALID, "placement_tables: bad sizes world=%d layers=%d experts=%d devices_per_host=%d", world, layers, experts, devices_per_host);
  if (rank < 0 || rank >= world) OMNI_FAIL(OMNI_E_INVALID, "placement_tables: rank %d outside [0,%d)", rank, world);
  if (num_deploy < experts || num_deploy % world != 0)
    OMNI_FAIL(OMNI_E_INVALID, "placement_tables: %d deployed positions for %d experts on %d devices", num_deploy, experts, world);
  const int per_device = num_deploy / world;
  // positions: device r owns [r*per_device, (r+1)*per_device); its deployed experts take them in id order
  std::vector<int32_t> pos((size_t)layers * num_deploy, -1);
  for (int l = 0; l < layers; ++l)
    for (int r = 0; r < world; ++r) {
      int local = 0;
      for (int e = 0; e < experts; ++e) {
        const int32_t v = pattern[((size_t)r * layers + l) * experts + e];
        if (v != 0 && v != 1) OMNI_FAIL(OMNI_E_INVALID, "placement_tables: pattern[%d][%d][%d] = %d is neither 0 nor 1", r, l, e, v);
        if (v == 0) continue;
        if (local >= per_device)
          OMNI_FAIL(OMNI_E_INVALID, "placement_tables: device %d deploys more than %d experts in layer %d", r, per_device, l);
        pos[(size_t)l * num_deploy + (size_t)r * per_device + local] = e;
        ++local;
      }
    }
  // selector: for each logical expert the position this rank sends its tokens to: the copy on the rank itself, else
  // one of the copies on the rank's host, else one of the others, each set shared out by rank modulo its size
  const int my_host = rank / devices_per_host;
  std::vector<int32_t> same, far;
  for (int l = 0; l < layers; ++l)
    for (int e = 0; e < experts; ++e) {
      same.clear();
      far.clear();
      int32_t own = -1;
      for (int p = 0; p < num_deploy; ++p) {
        if (pos[(size_t)l * num_deploy + p] != e) continue;
        const int dev = p / per_device;
        if (dev == rank) { if (own < 0) own = p; }
        else if (dev / devices_per_host == my_host) same.push_back(p);
        else far.push_back(p);
      }
      int32_t s = 0;  // an expert that is deployed nowhere keeps position 0, as in the reference's zero-filled table
      if (own >= 0) s = own;
      else if (!same.empty()) s = same[rank % same.size()];
      else if (!far.empty()) s = far[rank % far.size()];
      selector[(size_t)l * experts + e] = s;
    }
  if (position_to_expert)
    for (size_t i = 0; i < pos.size(); ++i) position_to_expert[i] = pos[i];
  return OMNI_OK;
}

}  // namespace omni_host
