// Host build of the library's integer logic (omni_infer_amd/csrc/host_logic.h), run under the address and
// undefined-behaviour sanitizers: g++ -std=c++17 -O1 -g -fsanitize=address,undefined -fno-sanitize-recover=all.
//
// What is checked (random inputs from a fixed seed, and small cases exhaustively):
//   * tile numbering of the tile kernel: over all block ids of a launch every (row block, column tile) is named
//     exactly once, the shares of a split tile cut its reduction into disjoint pieces that cover it, ids past
//     the work name nothing, and the launch grid the host sizes for the worst case holds every id;
//   * the row-block lookup of the kernels (the wavefront-wide scan of the device code restated with a loop over
//     the 64 lanes): every row of every group lies in exactly one block, heavy blocks first;
//   * the workspace layout of the whole-layer entry: parts aligned, disjoint, inside the total, large enough;
//   * kernel choice: the chosen stream-kernel variant is one that is compiled;
//   * the bookkeeping of the arrival counters; the placement tables.
#include <assert.h>
#include <stdarg.h>

#include <algorithm>
#include <map>
#include <random>
#include <set>
#include <thread>

#include "../../omni_infer_amd/csrc/host_logic.h"

static char g_err[512];
void omni_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

#define CHECK(...)                                                                   \
  do {                                                                               \
    if (!(__VA_ARGS__)) {                                                                 \
      fprintf(stderr, "CHECK failed at %s:%d: %s\n", __FILE__, __LINE__, #__VA_ARGS__);    \
      abort();                                                                       \
    }                                                                                \
  } while (0)

using namespace omni_host;
constexpr int WAVE = 64;

struct RowBlock { int group, row0, nrows; };

// ---- the device's row-block lookups with the lane loops written out.  Lane l owns group l (up to 64 groups) or
// the `per` consecutive groups from l * per on; prefix sums over the lanes; the lane whose range holds block b
// answers.  (csrc/common.h: row_blocks_scan / row_blocks_find and row_block_kinds_scan / row_block_kinds_find.)
static int group_rows(const std::vector<int>& offsets, int G, int extra_rows, int g) {
  return g < G ? offsets[g + 1] - offsets[g] : extra_rows;
}
static bool rows_find(const std::vector<int>& offsets, int G, int extra_rows, int BM, int b, RowBlock& rb, int& total) {
  const int Gt = G + (extra_rows > 0 ? 1 : 0);
  const int per = Gt <= WAVE ? 1 : (Gt + WAVE - 1) / WAVE;
  int incl[WAVE], nb[WAVE];
  int run = 0;
  for (int lane = 0; lane < WAVE; ++lane) {
    int mine = 0;
    for (int j = 0; j < per; ++j) {
      const int g = lane * per + j;
      if (g < Gt) mine += (group_rows(offsets, G, extra_rows, g) + BM - 1) / BM;
    }
    nb[lane] = mine;
    run += mine;
    incl[lane] = run;
  }
  total = incl[WAVE - 1];
  if (b < 0 || b >= total) return false;
  int owner = -1;
  for (int lane = 0; lane < WAVE; ++lane)
    if (b >= incl[lane] - nb[lane] && b < incl[lane]) { owner = lane; break; }
  CHECK(owner >= 0);
  int acc = incl[owner] - nb[owner];
  for (int j = 0; j < per; ++j) {
    const int g = owner * per + j;
    if (g >= Gt) break;
    const int start = offsets[g < G ? g : G];
    const int c = group_rows(offsets, G, extra_rows, g);
    const int n = (c + BM - 1) / BM;
    if (b < acc + n) {
      rb.group = g;
      rb.row0 = start + (b - acc) * BM;
      rb.nrows = std::min(BM, c - (b - acc) * BM);
      return true;
    }
    acc += n;
  }
  CHECK(false);
  return false;
}
struct Kinds { int total_h, total_l; };
static Kinds kinds_scan(const std::vector<int>& offsets, int G, int extra_rows, int BM, int light_max) {
  const int Gt = G + (extra_rows > 0 ? 1 : 0);
  Kinds k{0, 0};
  for (int g = 0; g < Gt; ++g) {
    const int c = group_rows(offsets, G, extra_rows, g);
    k.total_h += heavy_blocks(c, BM, light_max);
    k.total_l += light_blocks(c, BM, light_max);
  }
  return k;
}
static void kinds_find(const std::vector<int>& offsets, int G, int extra_rows, int BM, int light_max, bool light, int b,
                       RowBlock& rb) {
  const int Gt = G + (extra_rows > 0 ? 1 : 0);
  const int per = Gt <= WAVE ? 1 : (Gt + WAVE - 1) / WAVE;
  int incl[WAVE], n_of[WAVE];
  int run = 0;
  for (int lane = 0; lane < WAVE; ++lane) {
    int mine = 0;
    for (int j = 0; j < per; ++j) {
      const int g = lane * per + j;
      if (g < Gt) {
        const int c = group_rows(offsets, G, extra_rows, g);
        mine += light ? light_blocks(c, BM, light_max) : heavy_blocks(c, BM, light_max);
      }
    }
    n_of[lane] = mine;
    run += mine;
    incl[lane] = run;
  }
  int owner = -1;
  for (int lane = 0; lane < WAVE; ++lane)
    if (b >= incl[lane] - n_of[lane] && b < incl[lane]) { owner = lane; break; }
  CHECK(owner >= 0);
  int acc = incl[owner] - n_of[owner];
  for (int j = 0; j < per; ++j) {
    const int g = owner * per + j;
    CHECK(g < Gt);
    const int start = offsets[g < G ? g : G];
    const int c = group_rows(offsets, G, extra_rows, g);
    const int n = light ? light_blocks(c, BM, light_max) : heavy_blocks(c, BM, light_max);
    if (b < acc + n) {
      const int first = light ? c / BM * BM : (b - acc) * BM;
      rb.group = g;
      rb.row0 = start + first;
      rb.nrows = std::min(BM, c - first);
      return;
    }
    acc += n;
  }
  CHECK(false);
}

static std::vector<int> random_offsets(std::mt19937& rng, int G, int max_rows, double p_empty) {
  std::vector<int> off(G + 1, 0);
  std::uniform_int_distribution<int> rows(0, max_rows);
  std::uniform_real_distribution<double> u(0, 1);
  for (int g = 0; g < G; ++g) off[g + 1] = off[g] + (u(rng) < p_empty ? 0 : rows(rng));
  return off;
}

// ---- stream kernels: blocks of BM rows, group by group
static void test_row_blocks(std::mt19937& rng) {
  for (int it = 0; it < 400; ++it) {
    const int G = 1 + rng() % 200;
    const int BM = 16 << (rng() % 3);
    const int extra = (rng() % 2) ? rng() % 300 : 0;
    const std::vector<int> off = random_offsets(rng, G, 3 * BM, 0.2);
    const int64_t M_cap = off[G] + extra;
    std::vector<int> hits(M_cap, 0);
    int total = 0;
    RowBlock rb;
    rows_find(off, G, extra, BM, 0, rb, total);
    const int Gt = G + (extra > 0 ? 1 : 0);
    CHECK(total <= (M_cap + BM - 1) / BM + Gt);   // the grid the host launches (launch_stream)
    for (int b = 0; b < total; ++b) {
      int t2;
      CHECK(rows_find(off, G, extra, BM, b, rb, t2));
      CHECK(rb.nrows >= 1 && rb.nrows <= BM);
      const int start = off[rb.group < G ? rb.group : G];
      CHECK(rb.row0 >= start && rb.row0 + rb.nrows <= start + group_rows(off, G, extra, rb.group));
      for (int r = 0; r < rb.nrows; ++r) hits[rb.row0 + r]++;
    }
    int t3;
    CHECK(!rows_find(off, G, extra, BM, total, rb, t3));
    for (int64_t m = 0; m < M_cap; ++m) CHECK(hits[m] == 1);
  }
}

// ---- tile kernel: every (row block, column tile) exactly once, split tiles cover their reduction
static void check_tiles(const std::vector<int>& off, int G, int extra, int gx, int slots, int split_max, bool tail, int nk, int ku) {
  const int BM = 256, LM = TILE_LIGHT_MAX;
  const Kinds k = kinds_scan(off, G, extra, BM, LM);
  int pc = 1;
  for (int c = 1; c <= 8; ++c)
    if (gx % c == 0) pc = c;
  const TileGeom geom{gx, pc, tail ? slots : 0, split_max, tail};
  const TileCount tc = tile_count(geom, k.total_h, k.total_l, nk / ku);
  CHECK(tc.split >= 1 && tc.split <= std::max(1, split_max));
  CHECK(tc.total == tc.n_real + tc.left * (tc.split - 1));
  if (tc.split > 1) CHECK(tc.left * tc.split <= slots && tc.left <= tc.n_real);
  const int64_t M_cap = off[G] + extra;
  const int Gt = G + (extra > 0 ? 1 : 0);
  const int64_t grid = ((M_cap + BM - 1) / BM + Gt) * gx + (tail ? slots : 0);   // launch_tile
  CHECK(tc.total <= grid);
  // (row0, bx) -> covered k-steps
  std::map<std::pair<int, int>, std::vector<int>> cover;
  std::set<std::pair<int, int>> share_seen;
  for (int64_t id = 0; id < grid; ++id) {
    TileSel s;
    const bool ok = tile_select(geom, tc, k.total_h, k.total_l, (int)id, s);
    CHECK(ok == (id < tc.total));
    if (!ok) continue;
    CHECK(s.bx >= 0 && s.bx < gx);
    CHECK(s.by >= 0 && s.by < (s.light ? k.total_l : k.total_h));
    RowBlock rb;
    kinds_find(off, G, extra, BM, LM, s.light, s.by, rb);
    CHECK(rb.nrows >= 1 && rb.nrows <= BM);
    if (s.light) CHECK(rb.nrows <= LM);
    int k0 = 0, k1 = nk;
    if (s.tail_tile >= 0) {
      CHECK(tc.split > 1 && s.tail_tile < tc.left && s.share >= 0 && s.share < tc.split);
      CHECK(share_seen.insert({s.tail_tile, s.share}).second);
      tile_share_k_range(nk, ku, tc.split, s.share, k0, k1);
      CHECK(k1 > k0 && k0 % ku == 0);
    } else {
      CHECK(s.share == 0);
    }
    auto& v = cover[{rb.row0, s.bx}];
    if (v.empty()) v.assign(nk, 0);
    for (int kk = k0; kk < k1; ++kk) v[kk]++;
  }
  // every row of every group in exactly one row block, every tile's reduction covered once
  std::vector<int> hits(M_cap, 0);
  std::set<int> row0s;
  for (auto& kv : cover) {
    for (int c : kv.second) CHECK(c == 1);
    row0s.insert(kv.first.first);
  }
  CHECK((int64_t)cover.size() == (int64_t)row0s.size() * gx);
  CHECK((int)row0s.size() == k.total_h + k.total_l);
  for (int set = 0; set < 2; ++set)
    for (int b = 0; b < (set ? k.total_l : k.total_h); ++b) {
      RowBlock rb;
      kinds_find(off, G, extra, BM, LM, set == 1, b, rb);
      CHECK(row0s.count(rb.row0) == 1);
      for (int r = 0; r < rb.nrows; ++r) hits[rb.row0 + r]++;
    }
  for (int64_t m = 0; m < M_cap; ++m) CHECK(hits[m] == 1);
}

static void test_tiles(std::mt19937& rng) {
  const int gxs[] = {1, 2, 7, 8, 16, 28, 30};
  for (int it = 0; it < 300; ++it) {
    const int G = 1 + rng() % ((it % 5 == 0) ? 200 : 40);
    const int extra = (rng() % 2) ? rng() % 1500 : 0;
    const int max_rows = (it % 3 == 0) ? 120 : 700;
    const std::vector<int> off = random_offsets(rng, G, max_rows, 0.15);
    const int gx = gxs[rng() % 7];
    const int slots = (rng() % 2) ? 256 : 64 + rng() % 512;
    const int nk = 2 * (1 + rng() % 60);
    check_tiles(off, G, extra, gx, slots, 1 + rng() % 6, rng() % 4 != 0, nk, (rng() % 2) ? 2 : 1);
  }
  // the benchmark shapes: 32 groups of 2048 rows + 8192 shared rows; 16 / 28 column tiles; 256 slots
  std::vector<int> off(33, 0);
  for (int g = 0; g < 32; ++g) off[g + 1] = off[g] + 2048;
  check_tiles(off, 32, 8192, 16, 256, 4, true, 112, 2);
  check_tiles(off, 32, 8192, 28, 256, 4, true, 32, 2);
  // small cases, exhaustively: up to 3 groups of 0..600 rows in steps that hit every rule of the weight classes
  const int sizes[] = {0, 1, 96, 97, 255, 256, 257, 352, 353, 512, 600};
  for (int a : sizes)
    for (int b : sizes)
      for (int c : sizes) {
        std::vector<int> o = {0, a, a + b, a + b + c};
        for (int slots : {8, 256})
          for (int gx : {1, 8}) check_tiles(o, 3, (a + b) % 2 ? 300 : 0, gx, slots, 4, true, 8, 2);
      }
}

// Balanced numbering of the weight-streaming kernel: every block of the launch is covered by exactly the k-steps
// of its reduction, once; helper ids stay inside the grid the host launches; the overflow blocks fit the counter
// words and the partial-sum scratch; after the split no unit is more than a quarter block above the mean.
static void test_stream_balance(std::mt19937& rng) {
  for (int it = 0; it < 20000; ++it) {
    const int cus = (it % 3 == 0) ? 256 : 1 + (int)(rng() % 320);
    const int n_real = (it % 5 == 0) ? 1024 + (int)(rng() % 300) : (int)(rng() % 4000);
    const int resident = 1 + (int)(rng() % 8), dc = 1 + (int)(rng() % 2);
    const int nchunks = dc * (1 + (int)(rng() % 28));
    const int share_cap = (rng() % 4 == 0) ? 0 : (int)(rng() % 2000);
    const int block_kb = 1 + (int)(rng() % 2000);
    const StreamBalance b = stream_balance(n_real, cus, resident, nchunks, dc, share_cap, block_kb);
    CHECK(b.split == 1 || b.split == 2 || b.split == 4);
    CHECK(b.cap + b.n_over == n_real);
    CHECK(b.total == n_real + b.n_over * (b.split - 1));
    CHECK(b.total - n_real <= stream_balance_max_helpers(cus));
    if (b.split > 1) {
      CHECK(b.n_over > 0 && b.n_over < cus && b.n_over <= STREAM_BAL_CNT_WORDS);
      CHECK(b.n_over * b.split <= share_cap);
      CHECK(nchunks % b.split == 0 && nchunks / b.split >= 2 * dc);
      CHECK(b.cap % cus == 0 && b.cap / cus + 1 <= resident);
    } else {
      CHECK(b.n_over == 0);
    }
    std::vector<int> covered(n_real, 0);   // k shares seen per block, as a bit mask
    for (int id = -1; id < b.total + 3; ++id) {
      StreamSel s;
      const bool ok = stream_select(b, n_real, id, s);
      CHECK(ok == (id >= 0 && id < b.total));
      if (!ok) continue;
      CHECK(s.task >= 0 && s.task < n_real);
      if (s.task < b.cap) {
        CHECK(s.over == -1 && s.share == 0);
        covered[s.task] |= 0xf;
      } else {
        CHECK(s.over == s.task - b.cap && s.share >= 0 && s.share < b.split);
        CHECK(!(covered[s.task] & (1 << s.share)));
        covered[s.task] |= 1 << s.share;
      }
    }
    for (int t = 0; t < n_real; ++t) CHECK(covered[t] == (t < b.cap ? 0xf : (1 << b.split) - 1));
  }
  // GEMM1 of the DeepSeek-V3 shape (blocks of 917 KB, 28 chunks) on 256 units that hold 5 blocks each
  const StreamBalance d = stream_balance(1088, 256, 5, 28, 1, 1024, 896);   // 64 tokens: 34 row blocks x 32
  CHECK(d.cap == 1024 && d.n_over == 64 && d.split == 2 && d.total == 1088 + 64);
  CHECK(stream_balance(1056, 256, 5, 28, 1, 1024, 896).split == 4);   // 16 and 32 tokens
  CHECK(stream_balance(288, 256, 7, 28, 1, 1024, 896).split == 4);    // 1 token
  CHECK(stream_balance(448, 256, 7, 28, 1, 1024, 896).split == 1);    // 2, 4 and 8 tokens: the chip's rate is reached
  CHECK(stream_balance(672, 256, 7, 28, 1, 1024, 896).split == 1);    //   uncut, or the shares cost more than they save
  CHECK(stream_balance(992, 256, 7, 28, 1, 1024, 896).split == 1);
  CHECK(stream_balance(1152, 256, 5, 28, 1, 1024, 896).split == 2);   // 96 tokens: halves pay, quarters do not
  CHECK(stream_balance(1216, 256, 5, 28, 1, 1024, 896).split == 1);   // the fullest unit is near the mean
  CHECK(stream_balance(1024, 256, 5, 28, 1, 1024, 896).split == 1);   // even already
  CHECK(stream_balance(1280 + 64, 256, 5, 28, 1, 1024, 896).split == 1);   // a second round: left to the dispatcher
  CHECK(stream_balance(1088, 256, 5, 28, 1, 100, 896).split == 1);    // scratch too small for 64 x 2 shares
  CHECK(stream_balance(1056, 256, 5, 28, 1, 100, 896).split == 2);    // room for 32 x 2 shares, not for 32 x 4
  CHECK(stream_balance(1088, 256, 5, 28, 1, 1024, 16).split == 1);    // tiny blocks: a share costs more than it saves
}

static void test_layout(std::mt19937& rng) {
  for (int it = 0; it < 2000; ++it) {
    const int T = 1 + rng() % ((it % 10 == 0) ? 20000 : 600);
    const int K = 1 + rng() % 8, G = 1 + rng() % 256;
    const int H = 64 * (1 + rng() % 128), I = 64 * (1 + rng() % 64);
    const int with_shared = rng() % 2, rd = (rng() % 2) ? OMNI_DT_F32 : OMNI_DT_BF16;
    const LayerWs L = layer_layout(T, K, G, H, I, with_shared, rd);
    const int64_t M_cap = (int64_t)T * K + (with_shared ? T : 0);
    CHECK(L.M_cap == M_cap);
    struct Part { size_t at, bytes; };
    const Part parts[] = {
        {L.x_q, (size_t)T * H}, {L.x_s, (size_t)T * 4}, {L.sorted_src, (size_t)T * K * 4}, {L.src_to_dst, (size_t)T * K * 4},
        {L.counts, (size_t)G * 4}, {L.offsets, (size_t)(G + 1) * 4}, {L.perm_ws, L.perm_bytes}, {L.h_q, (size_t)M_cap * I},
        {L.h_s, (size_t)M_cap * 4}, {L.g1_ws, L.g1_bytes}, {L.rows, (size_t)M_cap * H * (rd == OMNI_DT_F32 ? 4 : 2)}};
    size_t end = 0;
    for (const Part& p : parts) {
      CHECK(p.at % 256 == 0);
      CHECK(p.at >= end);          // in order, disjoint
      end = p.at + p.bytes;
    }
    CHECK(end <= L.total);
    CHECK(L.perm_bytes == permute_workspace_bytes(T, K));
    CHECK(L.g1_bytes >= gemm1_workspace_bytes(T, K, G, with_shared ? T : 0, M_cap, H, I));
    CHECK(L.g1_bytes >= gemm2_workspace_bytes(G, with_shared ? T : 0, M_cap, H, I));
    // what the GEMM1 paths put into their workspace
    const Plan p1 = make_plan(1, T, K, G, with_shared ? T : 0, H, 2 * I);
    if (p1.tile) CHECK(L.g1_bytes >= (size_t)M_cap * I * 4 + TILE_TAIL_BYTES);
    else CHECK(L.g1_bytes >= (size_t)p1.S * M_cap * 2 * I * 4);
    if (!p1.tile && p1.S == 1) {   // the scratch of the overflow blocks ends the workspace, past the sums, aligned
      const size_t at = gemm1_stream_bal_at(p1, M_cap, I);
      CHECK(at % 256 == 0 && at >= (size_t)M_cap * 2 * I * 4 && at + STREAM_BAL_BYTES <= L.g1_bytes);
    } else {
      CHECK(gemm1_stream_bal_at(p1, M_cap, I) == 0);
    }
    if (!p1.tile) CHECK(stream_variant_exists(1, p1.mt, p1.nt, p1.d));
    const Plan p2 = make_plan(2, (int)M_cap, 1, G, with_shared ? T : 0, I, H);
    if (!p2.tile) CHECK(stream_variant_exists(2, p2.mt, p2.nt, p2.d));
    if (p1.tile) CHECK(L.total > (size_t)OMNI_STATIC_SCRATCH_BYTES);   // the static entry refuses it by size
  }
  // the sort's workspace holds the block table and the bucket bases of its three-launch path
  for (int n : {4097, 5000, 65536, 1 << 20}) {
    const int nblk = (n + PERM_CH_MULTI - 1) / PERM_CH_MULTI;
    CHECK(permute_workspace_bytes(n, 1) >= (size_t)(nblk + 1) * PERM_NB * 4);
  }
}

static void test_arrive_book() {
  ArriveBook book;
  // eager calls: the first pool in turn, never a word of the capture pool
  for (int i = 0; i < 3 * ArriveBook::EAGER_SLOTS; ++i) CHECK(book.take(0, 0x1000 + i) == i % ArriveBook::EAGER_SLOTS);
  // captured calls: one word per (capture, stream), kept, never shared, never from the eager pool
  std::map<std::pair<unsigned long long, uintptr_t>, int> seen;
  std::set<int> used;
  for (unsigned long long id = 1; id <= 60; ++id)
    for (uintptr_t st = 0x100; st < 0x100 + 64 * 16; st += 16) {
      const int s = book.take(id, st);
      CHECK(s >= ArriveBook::EAGER_SLOTS && s < ArriveBook::TOTAL_SLOTS);
      CHECK(used.insert(s).second);
      seen[{id, st}] = s;
    }
  CHECK((int)used.size() == ArriveBook::CAPTURE_SLOTS && book.capture_slots_used() == ArriveBook::CAPTURE_SLOTS);
  for (auto& kv : seen) CHECK(book.take(kv.first.first, kv.first.second) == kv.second);   // replays of a capture
  CHECK(book.take(61, 0x100) == -1);                                                     // pool used up
  CHECK(book.take(1, 0x100) == seen[{1, 0x100}]);                                         // known pairs still served
  CHECK(book.take(0, 0) >= 0 && book.take(0, 0) < ArriveBook::EAGER_SLOTS);
  // from several threads at once: no word handed to two pairs
  ArriveBook b2;
  std::vector<std::vector<int>> got(8);
  std::vector<std::thread> th;
  for (int t = 0; t < 8; ++t)
    th.emplace_back([&, t] {
      for (int i = 0; i < 200; ++i) got[t].push_back(b2.take(1 + t, 0x10 * (1 + i)));
    });
  for (auto& x : th) x.join();
  std::set<int> all;
  for (auto& v : got)
    for (int s : v) CHECK(s >= ArriveBook::EAGER_SLOTS && all.insert(s).second);
}

static void test_placement(std::mt19937& rng) {
  for (int it = 0; it < 200; ++it) {
    const int world = 1 + rng() % 8, layers = 1 + rng() % 3, experts = world * (1 + rng() % 8);
    const int per = experts / world + rng() % 3, num_deploy = per * world, dph = 1 + rng() % 4;
    std::vector<int32_t> pat((size_t)world * layers * experts, 0);
    for (int l = 0; l < layers; ++l) {
      std::vector<int> load(world, 0);
      for (int e = 0; e < experts; ++e) {   // every expert once, then spare positions filled with copies
        int r = e % world;
        pat[((size_t)r * layers + l) * experts + e] = 1;
        load[r]++;
      }
      for (int r = 0; r < world; ++r)
        for (int tries = 0; load[r] < per && tries < 50; ++tries) {
          const int e = rng() % experts;
          int32_t& v = pat[((size_t)r * layers + l) * experts + e];
          if (!v) { v = 1; load[r]++; }
        }
    }
    const int rank = rng() % world;
    std::vector<int32_t> pos((size_t)layers * num_deploy), sel((size_t)layers * experts);
    CHECK(placement_tables(pat.data(), world, layers, experts, rank, dph, num_deploy, pos.data(), sel.data()) == OMNI_OK);
    for (int l = 0; l < layers; ++l)
      for (int e = 0; e < experts; ++e) {
        const int p = sel[(size_t)l * experts + e];
        CHECK(p >= 0 && p < num_deploy && pos[(size_t)l * num_deploy + p] == e);   // the position holds the expert
        if (pat[((size_t)rank * layers + l) * experts + e]) CHECK(p / per == rank);   // an own copy wins
      }
  }
  int32_t bad[4] = {1, 2, 0, 1}, sel[2];
  CHECK(placement_tables(bad, 2, 1, 2, 0, 1, 2, nullptr, sel) == OMNI_E_INVALID);
  CHECK(placement_tables(bad, 2, 1, 2, 5, 1, 2, nullptr, sel) == OMNI_E_INVALID);
}

int main() {
  std::mt19937 rng(12345);
  test_row_blocks(rng);
  test_tiles(rng);
  test_stream_balance(rng);
  test_layout(rng);
  test_arrive_book();
  test_placement(rng);
  printf("host logic: all checks passed\n");
  return 0;
}
