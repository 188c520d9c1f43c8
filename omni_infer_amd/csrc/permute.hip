// Stable counting sort of the (token, k) assignments by local expert id.
//
// Assignments are numbered p = n*K + k.  Bucket e < G is local expert lo + e, bucket G collects
// the assignments whose expert is outside [lo, hi) ("dropped"); the dropped bucket sorts last.
// A block of four wavefronts ranks a chunk of assignments: each wavefront walks its part of the
// chunk 64 assignments at a time, finds the lanes that hold the same bucket with one ballot per
// bucket-id bit, and keeps a running per-bucket count in an LDS histogram (one per wavefront).
// An exclusive prefix over wavefronts, blocks and buckets then gives every assignment its slot.
// Small inputs (<= 4096 assignments) are sorted by one block in one launch: four wavefronts up to 1024
// assignments (a block of four starts sooner than one of sixteen: measured better up to 128 tokens of 8), sixteen
// wavefronts above; either way a wavefront has at most four dependent passes.  Larger inputs take a count launch,
// a one-block scan launch and a scatter launch.
#include <stdlib.h>
#include <mutex>
#include "common.h"
#include "quant_rows.h"
#include "route_body.h"

namespace {

constexpr int GMAX = omni_host::PERM_GMAX;            // local experts per call
constexpr int NB = omni_host::PERM_NB;                // buckets incl. the dropped one
constexpr int CH_MULTI = omni_host::PERM_CH_MULTI;    // assignments per block in the multi-block path
constexpr int CH_SINGLE = omni_host::PERM_CH_SINGLE;  // largest input of the single-block path
constexpr int NW_SMALL_MAX_N = 1024;  // up to this many assignments the single block has 4 wavefronts, above 16

struct PermArgs {
  const int32_t* ids;
  int n, T, K, lo, G, idx_mode;
  int32_t* sorted_src;
  int32_t* src_to_dst;
  int32_t* counts;
  int32_t* offsets;
  int32_t* blk_hist;  // [nblk][NB] counts, then (after the scan) exclusive block bases
  int nblk;
  int32_t* zero_words;  // cleared by the single-block kernel of the call (null: nothing to clear)
  int zero_n;
};

__device__ __forceinline__ void clear_words(const PermArgs& a) {
  for (int i = threadIdx.x; i < a.zero_n; i += blockDim.x) a.zero_words[i] = 0;
}

__device__ __forceinline__ int bucket_of(int id, int lo, int G) {
  int e = id - lo;
  return (e >= 0 && e < G) ? e : G;
}

// The buckets of a thread's assignments of the chunk, all requested at once (the passes below depend on each
// other through the histogram, so loads inside them would be paid one latency at a time): bk[j] is the bucket of
// assignment (w * passes + j) * 64 + lane, -1 past the end.  MP bounds the passes of a chunk.
template <int MP>
__device__ __forceinline__ void load_buckets(const PermArgs& a, int base, int len, int passes, int (&bk)[MP]) {
  const int w = threadIdx.x / WAVE, lane = threadIdx.x & (WAVE - 1);
#pragma unroll
  for (int j = 0; j < MP; ++j) {
    const int i = (w * passes + j) * WAVE + lane;
    bk[j] = (j < passes && i < len) ? bucket_of(a.ids[base + i], a.lo, a.G) : -1;
  }
}

// Ranks the chunk [base, base+len): lrank[i] = number of earlier assignments of the same bucket
// inside the same wavefront's part; whist[w][b] = count of bucket b in wavefront w's part.
template <int MP, int NW = 4>
__device__ __forceinline__ void rank_chunk(const PermArgs& a, int len, int passes, int (*whist)[NB], int* lrank,
                                           const int (&bk)[MP]) {
  const int w = threadIdx.x / WAVE, lane = threadIdx.x & (WAVE - 1);
  for (int i = threadIdx.x; i < NW * NB; i += NW * WAVE) (&whist[0][0])[i] = 0;
  __syncthreads();
  const int nbits = 32 - __clz(a.G);
  const uint64_t lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
#pragma unroll
  for (int j = 0; j < MP; ++j) {
    if (j >= passes) break;
    int i = (w * passes + j) * WAVE + lane;
    bool valid = bk[j] >= 0;
    int b = valid ? bk[j] : 0;
    uint64_t peers = __ballot(valid);
    for (int bit = 0; bit < nbits; ++bit) {
      uint64_t m = __ballot((b >> bit) & 1);
      peers &= ((b >> bit) & 1) ? m : ~m;
    }
    if (valid) {
      // lanes of one wavefront run these two LDS accesses in program order: every peer reads
      // the running count before the first peer replaces it
      volatile int* cnt = &whist[w][b];
      int r = __popcll(peers & lt);
      int start = *cnt;
      lrank[i] = start + r;
      if (r == 0) *cnt = start + __popcll(peers);
    }
  }
  __syncthreads();
}

__device__ __forceinline__ int src_index(const PermArgs& a, int p) {
  if (a.idx_mode == OMNI_IDX_TOKEN_MAJOR) return p;
  int n = p / a.K, k = p - n * a.K;
  return k * a.T + n;
}

// Scatter of the chunk, given for every bucket the slot of the chunk's first assignment of it.
template <int MP>
__device__ __forceinline__ void scatter_chunk(const PermArgs& a, int base, int passes, int (*whist)[NB],
                                              const int* lrank, const int* bucket_slot0, const int (&bk)[MP]) {
  const int w = threadIdx.x / WAVE, lane = threadIdx.x & (WAVE - 1);
#pragma unroll
  for (int j = 0; j < MP; ++j) {
    if (j >= passes) break;
    int i = (w * passes + j) * WAVE + lane;
    if (bk[j] >= 0) {
      int b = bk[j];
      int slot = bucket_slot0[b] + lrank[i];
      for (int ww = 0; ww < w; ++ww) slot += whist[ww][b];
      int src = src_index(a, base + i);
      a.sorted_src[slot] = src;
      a.src_to_dst[src] = (b < a.G) ? slot : -1;
    }
  }
}

// exclusive scan of tot[0..nb) by wavefront 0 into off[0..nb]; off[nb] = grand total
__device__ __forceinline__ void wave0_excl_scan(const int* tot, int* off, int nb) {
  if (threadIdx.x < WAVE) {
    const int lane = threadIdx.x;
    const int per = (nb + WAVE - 1) / WAVE;
    int mine = 0;
    for (int j = 0; j < per; ++j) {
      int b = lane * per + j;
      if (b < nb) mine += tot[b];
    }
    int incl = wave_incl_scan_i(mine, lane);
    int run = incl - mine;
    for (int j = 0; j < per; ++j) {
      int b = lane * per + j;
      if (b < nb) {
        off[b] = run;
        run += tot[b];
      }
    }
    if (lane == WAVE - 1) off[nb] = incl;
  }
}

// The whole sort by one block of NW wavefronts.  After the ranking a thread per bucket turns the
// wavefronts' counts of its bucket into their exclusive prefix (and the bucket's total), so that an assignment's
// slot is three LDS reads: the bucket's base, its wavefront's prefix, its rank inside the wavefront.
template <int NW>
__device__ __forceinline__ void permute_single_body(const PermArgs& a) {
  constexpr int NT = NW * WAVE, MP = (NW == 4 ? NW_SMALL_MAX_N : CH_SINGLE) / NT;  // passes of a wavefront at most
  __shared__ int whist[NW][NB];
  __shared__ int lrank[CH_SINGLE];
  __shared__ int tot[NB];
  __shared__ int off[NB + 1];
  const int passes = (a.n + NT - 1) / NT;
  int bk[MP];
  load_buckets(a, 0, a.n, passes, bk);
  clear_words(a);
  rank_chunk<MP, NW>(a, a.n, passes, whist, lrank, bk);
  const int nb = a.G + 1;
  for (int b = threadIdx.x; b < nb; b += NT) {
    int c[NW];
#pragma unroll
    for (int ww = 0; ww < NW; ++ww) c[ww] = whist[ww][b];
    int run = 0;
#pragma unroll
    for (int ww = 0; ww < NW; ++ww) {
      whist[ww][b] = run;
      run += c[ww];
    }
    tot[b] = run;
  }
  __syncthreads();
  wave0_excl_scan(tot, off, nb);
  __syncthreads();
  for (int b = threadIdx.x; b < a.G; b += NT) {
    a.counts[b] = tot[b];
    a.offsets[b] = off[b];
  }
  if (threadIdx.x == 0) a.offsets[a.G] = off[a.G];
  const int w = threadIdx.x / WAVE, lane = threadIdx.x & (WAVE - 1);
#pragma unroll
  for (int j = 0; j < MP; ++j) {
    if (j >= passes) break;
    const int i = (w * passes + j) * WAVE + lane;
    if (bk[j] >= 0) {
      const int b = bk[j];
      const int slot = off[b] + whist[w][b] + lrank[i];
      const int src = src_index(a, i);
      a.sorted_src[slot] = src;
      a.src_to_dst[src] = (b < a.G) ? slot : -1;
    }
  }
}

template <int NW>
__global__ __launch_bounds__(NW * WAVE) void permute_single(PermArgs a) { permute_single_body<NW>(a); }

// NW / 4 token rows of a block of NW wavefronts, four wavefronts a row: the row body of quant_rows.h with the
// block barrier shared by the rows (rows past the end take part in it and touch no memory).
template <int MAXV>
__device__ __forceinline__ void quant_block_rows(const void* __restrict__ xv, int64_t r0, int64_t rows, int cols,
                                                int8_t* __restrict__ q, float* __restrict__ scale, float* red) {
  const int tid = threadIdx.x & 255, qd = threadIdx.x >> 8;
  const int64_t r = r0 + qd;
  const bool live = r < rows;
  const uint16_t* x = (const uint16_t*)xv + (live ? r : 0) * (int64_t)cols;
  const int nvec = cols / 8;
  float v[MAXV][8];
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    const int vi = tid + i * 256;
    if (live && vi < nvec) {
      const v4i raw = __builtin_nontemporal_load((const v4i*)(x + (size_t)vi * 8));  // the row is read once here
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint32_t u = (uint32_t)raw[j];
        v[i][2 * j] = bf16_to_f32((uint16_t)(u & 0xffffu));
        v[i][2 * j + 1] = bf16_to_f32((uint16_t)(u >> 16));
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[i][j]));
    }
  }
  amax = wave_allmax_f(amax);
  if ((threadIdx.x & (WAVE - 1)) == 0) red[threadIdx.x / WAVE] = amax;
  __syncthreads();
  amax = fmaxf(fmaxf(red[4 * qd], red[4 * qd + 1]), fmaxf(red[4 * qd + 2], red[4 * qd + 3]));
  if (!live) return;  // (a block of four wavefronts has one row, qd = 0)
  const float s = amax / 127.0f;
  if (tid == 0) scale[r] = s;
  int8_t* qr = q + r * (int64_t)cols;
#pragma unroll
  for (int i = 0; i < MAXV; ++i) {
    const int vi = tid + i * 256;
    if (vi < nvec) {
      uint32_t w0 = 0, w1 = 0;
      if (s > 0.0f) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          w0 |= ((uint32_t)(quant_i8(v[i][j], s) & 0xff)) << (8 * j);
          w1 |= ((uint32_t)(quant_i8(v[i][4 + j], s) & 0xff)) << (8 * j);
        }
      }
      const v2i o = {(int)w0, (int)w1};
      *(v2i*)(qr + (size_t)vi * 8) = o;
    }
  }
}

// One launch for the two independent first steps of a small layer call: blocks [0, ceil(rows / (NW/4))) quantise
// NW / 4 bf16 token rows each, the last block sorts the assignments.
template <int MAXV, int NW>
__global__ __launch_bounds__(NW * WAVE) void quant_permute_small(const void* __restrict__ x, int64_t rows, int cols,
                                                                 int8_t* __restrict__ q, float* __restrict__ scale,
                                                                 PermArgs a) {
  constexpr int RPB = NW / 4;
  __shared__ float red[NW];
  const int quant_blocks = (int)((rows + RPB - 1) / RPB);
  if ((int)blockIdx.x < quant_blocks) quant_block_rows<MAXV>(x, (int64_t)blockIdx.x * RPB, rows, cols, q, scale, red);
  else permute_single_body<NW>(a);
}

// One launch for the three first steps of a small layer call: blocks [0, ceil(T/NW)) route NW tokens each
// (one per wavefront), the next ceil(T/(NW/4)) blocks quantise NW/4 bf16 token rows each, and the routing block that
// finishes last sorts the assignments.  `arrive` counts the routing blocks that are done.  It is zero when the
// kernel starts and the sorting block sets it back to zero, so no launch ever has to clear it.  The hand-over is
// the one of the split tiles of the grouped GEMM: every wavefront waits for its stores, the block meets at a
// barrier, one thread counts in with a device-scope acquire-release add (the release half makes the block's stores
// visible to the device, the acquire half of the last add makes everybody else's visible to the sorting block).
// No block waits for another.
// FOLD: the logits come as partial sums of the gate projection (RouteArgs::partials): a routing block takes one
// token, its four wavefronts add the parts up together and the first one routes (blocks [0, T) route).
// rows == 0: the tokens are quantised already and the launch has no quantising blocks.
template <int MAXV, int V, int NW, bool FOLD>
__global__ __launch_bounds__(NW * WAVE) void route_quant_permute_small(const void* __restrict__ x, int64_t rows,
                                                                       int cols, int8_t* __restrict__ q,
                                                                       float* __restrict__ scale, RouteArgs r,
                                                                       PermArgs a, int* arrive) {
  static_assert(!FOLD || NW == 4, "the block-wide fold is written for four wavefronts");
  constexpr int RPB = NW / 4;
  __shared__ float red[NW];
  __shared__ int s_last;
  const int route_blocks = FOLD ? r.T : (r.T + NW - 1) / NW;
  if ((int)blockIdx.x >= route_blocks) {
    quant_block_rows<MAXV>(x, ((int64_t)blockIdx.x - route_blocks) * RPB, rows, cols, q, scale, red);
    return;
  }
  const int lane = threadIdx.x & (WAVE - 1);
  if constexpr (FOLD) {
    __shared__ float s_q[FOLD_MAX_GROUPS][WAVE * V];
    const int t = (int)blockIdx.x, wv = threadIdx.x / WAVE;
    float s[V], bias[V], tot[V];
    bool in[V];
    route_load_bias<V>(r, lane, bias);
#pragma unroll
    for (int j = 0; j < V; ++j) in[j] = lane * V + j < r.E;
    if (route_fold_block<V>(r, t, lane, wv, in, tot, s_q)) {
      route_finish_logits<V>(r, t, lane, in, tot, s);
      route_token<V>(r, t, lane, s, in, bias);
    }
  } else {
    const int t = (int)blockIdx.x * NW + threadIdx.x / WAVE;
    if (t < r.T) {  // the same for a whole wavefront
      float s[V], bias[V];
      bool in[V];
      route_load_bias<V>(r, lane, bias);
      route_load_logits<V>(r, t, lane, s, in);
      route_token<V>(r, t, lane, s, in, bias);
    }
  }
  __builtin_amdgcn_s_waitcnt(0);  // this wavefront's stores are acknowledged before it meets the block
  __syncthreads();
  if (threadIdx.x == 0) {
    s_last = (__hip_atomic_fetch_add(arrive, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT) == route_blocks - 1);
    if (s_last) __hip_atomic_store(arrive, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if (!s_last) return;
  permute_single_body<NW>(a);
}

__global__ __launch_bounds__(256) void permute_count(PermArgs a) {
  __shared__ int whist[4][NB];
  __shared__ int lrank[CH_MULTI];
  const int base = blockIdx.x * CH_MULTI;
  const int len = min(CH_MULTI, a.n - base);
  int bk[CH_MULTI / 256];
  load_buckets(a, base, len, CH_MULTI / 256, bk);
  rank_chunk(a, len, CH_MULTI / 256, whist, lrank, bk);
  for (int b = threadIdx.x; b <= a.G; b += 256)
    a.blk_hist[(size_t)blockIdx.x * NB + b] = whist[0][b] + whist[1][b] + whist[2][b] + whist[3][b];
}

// one block: per bucket exclusive prefix over blocks (in place), then the prefix over buckets
__global__ __launch_bounds__(256) void permute_scan(PermArgs a) {
  __shared__ int tot[NB];
  __shared__ int off[NB + 1];
  const int nb = a.G + 1;
  clear_words(a);
  for (int b = threadIdx.x; b < nb; b += 256) {
    int run = 0;
    // eight blocks' counts are requested together before their prefixes are written back
    for (int k0 = 0; k0 < a.nblk; k0 += 8) {
      int c[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) c[u] = (k0 + u < a.nblk) ? a.blk_hist[(size_t)(k0 + u) * NB + b] : 0;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        if (k0 + u < a.nblk) a.blk_hist[(size_t)(k0 + u) * NB + b] = run;
        run += c[u];
      }
    }
    tot[b] = run;
  }
  __syncthreads();
  wave0_excl_scan(tot, off, nb);
  __syncthreads();
  for (int b = threadIdx.x; b < a.G; b += 256) {
    a.counts[b] = tot[b];
    a.offsets[b] = off[b];
  }
  if (threadIdx.x == 0) a.offsets[a.G] = off[a.G];
  // bucket bases for the scatter launch live after the block table
  for (int b = threadIdx.x; b < nb; b += 256) a.blk_hist[(size_t)a.nblk * NB + b] = off[b];
}

__global__ __launch_bounds__(256) void permute_scatter(PermArgs a) {
  __shared__ int whist[4][NB];
  __shared__ int lrank[CH_MULTI];
  __shared__ int slot0[NB];
  const int base = blockIdx.x * CH_MULTI;
  const int len = min(CH_MULTI, a.n - base);
  int bk[CH_MULTI / 256];
  load_buckets(a, base, len, CH_MULTI / 256, bk);
  rank_chunk(a, len, CH_MULTI / 256, whist, lrank, bk);
  for (int b = threadIdx.x; b <= a.G; b += 256)
    slot0[b] = a.blk_hist[(size_t)a.nblk * NB + b] + a.blk_hist[(size_t)blockIdx.x * NB + b];
  __syncthreads();
  scatter_chunk(a, base, CH_MULTI / 256, whist, lrank, slot0, bk);
}

struct GatherArgs {
  const uint8_t* x;
  int64_t row_bytes;
  const float* x_scale;
  const int32_t* sorted_src;
  const int32_t* offsets;
  int n_local, T, K, idx_mode;
  uint8_t* rows_out;
  float* scale_out;
};

// one block per sorted slot; slots past the kept total copy nothing
__global__ __launch_bounds__(256) void gather_rows_kernel(GatherArgs g) {
  const int m = blockIdx.x;
  if (m >= g.offsets[g.n_local]) return;
  const int src = g.sorted_src[m];
  const int tok = (g.idx_mode == OMNI_IDX_TOKEN_MAJOR) ? src / g.K : src % g.T;
  const uint8_t* s = g.x + (size_t)tok * g.row_bytes;
  uint8_t* d = g.rows_out + (size_t)m * g.row_bytes;
  if ((g.row_bytes % 16 == 0) && ((uintptr_t)g.x % 16 == 0) && ((uintptr_t)g.rows_out % 16 == 0)) {
    for (int64_t i = threadIdx.x; i < g.row_bytes / 16; i += 256) ((v4i*)d)[i] = ((const v4i*)s)[i];
  } else {
    for (int64_t i = threadIdx.x; i < g.row_bytes; i += 256) d[i] = s[i];
  }
  if (threadIdx.x == 0 && g.x_scale && g.scale_out) g.scale_out[m] = g.x_scale[tok];
}

}  // namespace

namespace {
// wavefronts of the block that sorts a small input (and of the launch it is part of); OMNI_MOE_SORT_WAVES = 4 or
// 16 overrides the choice (a tuning aid, read once)
int sort_waves(int n) {
  static const int forced = [] {
    const char* e = getenv("OMNI_MOE_SORT_WAVES");
    const int v = e ? atoi(e) : 0;
    return (v == 4 || v == 16) ? v : 0;
  }();
  if (n > NW_SMALL_MAX_N) return 16;  // four wavefronts hold no more
  return forced ? forced : 4;
}
}  // namespace

extern "C" size_t omni_moe_permute_workspace_bytes(int T, int K, int n_local) {
  (void)n_local;
  return omni_host::permute_workspace_bytes(T, K);
}

extern "C" int omni_moe_permute(const int32_t* topk_ids, int T, int K, int lo, int hi, int idx_mode,
                                int32_t* sorted_src, int32_t* src_to_dst, int32_t* counts, int32_t* offsets,
                                void* workspace, size_t ws_bytes, void* stream) {
  return omni_moe_permute_clearing(topk_ids, T, K, lo, hi, idx_mode, sorted_src, src_to_dst, counts, offsets, workspace,
                                   ws_bytes, nullptr, 0, stream);
}

int omni_moe_permute_clearing(const int32_t* topk_ids, int T, int K, int lo, int hi, int idx_mode, int32_t* sorted_src,
                              int32_t* src_to_dst, int32_t* counts, int32_t* offsets, void* workspace, size_t ws_bytes,
                              int32_t* zero_words, int zero_n, void* stream) {
  if (T < 0 || K <= 0 || hi <= lo) OMNI_FAIL(OMNI_E_INVALID, "permute: bad sizes T=%d K=%d range=[%d,%d)", T, K, lo, hi);
  const int G = hi - lo;
  if (G > GMAX) OMNI_FAIL(OMNI_E_UNSUPPORTED, "permute: %d local experts > %d", G, GMAX);
  if ((int64_t)T * K > 0x7fffffffLL) OMNI_FAIL(OMNI_E_UNSUPPORTED, "permute: T*K overflows int32");
  if (!counts || !offsets) OMNI_FAIL(OMNI_E_INVALID, "permute: null pointer");
  if (idx_mode != OMNI_IDX_TOKEN_MAJOR && idx_mode != OMNI_IDX_K_MAJOR) OMNI_FAIL(OMNI_E_INVALID, "permute: bad idx_mode %d", idx_mode);
  if (T > 0 && (!topk_ids || !sorted_src || !src_to_dst)) OMNI_FAIL(OMNI_E_INVALID, "permute: null pointer");
  const int n = T * K;
  if (ws_bytes < omni_moe_permute_workspace_bytes(T, K, G)) OMNI_FAIL(OMNI_E_WORKSPACE, "permute: workspace %zu < %zu", ws_bytes, omni_moe_permute_workspace_bytes(T, K, G));
  hipStream_t st = (hipStream_t)stream;
  PermArgs a{topk_ids, n, T, K, lo, G, idx_mode, sorted_src, src_to_dst, counts, offsets, (int32_t*)workspace, 0,
             zero_words, zero_words ? zero_n : 0};
  if (n <= CH_SINGLE) {
    if (sort_waves(n) == 4) hipLaunchKernelGGL(permute_single<4>, dim3(1), dim3(4 * WAVE), 0, st, a);
    else hipLaunchKernelGGL(permute_single<16>, dim3(1), dim3(16 * WAVE), 0, st, a);
    OMNI_CHECK_LAUNCH("permute_single");
    return OMNI_OK;
  }
  if (!workspace) OMNI_FAIL(OMNI_E_WORKSPACE, "permute: workspace is null");
  a.nblk = (n + CH_MULTI - 1) / CH_MULTI;
  hipLaunchKernelGGL(permute_count, dim3(a.nblk), dim3(256), 0, st, a);
  hipLaunchKernelGGL(permute_scan, dim3(1), dim3(256), 0, st, a);
  hipLaunchKernelGGL(permute_scatter, dim3(a.nblk), dim3(256), 0, st, a);
  OMNI_CHECK_LAUNCH("permute");
  return OMNI_OK;
}

// Internal to the library (the whole-layer entry uses it): quantise bf16 rows and sort the
// assignments in one launch.  Returns 1 without launching when the shapes do not fit that kernel.
int omni_quant_permute_fused(const void* x_bf16, int T, int H, int8_t* q, float* scale, const int32_t* topk_ids, int K,
                             int lo, int hi, int idx_mode, int32_t* sorted_src, int32_t* src_to_dst, int32_t* counts,
                             int32_t* offsets, int32_t* zero_words, int zero_n, void* stream) {
  const int G = hi - lo;
  const int64_t n = (int64_t)T * K;
  if (T <= 0 || n > CH_SINGLE || G > GMAX || H % 8 != 0 || H > 8 * 256 * 4) return 1;
  if (((uintptr_t)x_bf16 % 16) || ((uintptr_t)q % 8) || ((size_t)H * 2) % 16 != 0) return 1;
  PermArgs a{topk_ids, (int)n, T, K, lo, G, idx_mode, sorted_src, src_to_dst, counts, offsets, nullptr, 0,
             zero_words, zero_words ? zero_n : 0};
  const int nw = sort_waves((int)n), rpb = nw / 4;
  dim3 grid((unsigned)((T + rpb - 1) / rpb + 1)), block(nw * WAVE);
  hipStream_t st = (hipStream_t)stream;
  const int MV = H <= 8 * 256 ? 1 : (H <= 8 * 256 * 2 ? 2 : 4);
#define QP_LAUNCH(MAXV, NW_) hipLaunchKernelGGL((quant_permute_small<MAXV, NW_>), grid, block, 0, st, x_bf16, (int64_t)T, H, q, scale, a)
#define QP_NW(MAXV)             \
  do {                          \
    if (nw == 4) QP_LAUNCH(MAXV, 4); \
    else QP_LAUNCH(MAXV, 16);   \
  } while (0)
  if (MV == 1) QP_NW(1);
  else if (MV == 2) QP_NW(2);
  else QP_NW(4);
#undef QP_NW
#undef QP_LAUNCH
  OMNI_CHECK_LAUNCH("quant_permute");
  return OMNI_OK;
}

// ---- arrival counters of the kernel that routes, quantises and sorts
// A file-scope device array, zero when the module is loaded; every GPU holds its own copy at its own address (the
// array's name is only a host-side handle: the device address is asked for once per device).  Every launch leaves
// its counter at zero.  Which word a call uses is decided by omni_host::ArriveBook (host_logic.h): eager calls take
// the first 256 words in turn, a call under stream capture gets a word of its (capture, stream) pair from the
// rest, and when those are used up the call is told so and runs the launches that need no counter.
namespace {
constexpr int ARRIVE_SLOTS = omni_host::ArriveBook::TOTAL_SLOTS;
static __device__ int arrive_counters[ARRIVE_SLOTS];
constexpr int ARRIVE_MAX_DEVICES = 64;
int* g_arrive_ptr[ARRIVE_MAX_DEVICES];
omni_host::ArriveBook g_arrive_book[ARRIVE_MAX_DEVICES];
std::mutex g_arrive_mutex;

// OMNI_OK with *out set; 1 when the call is being captured and the capture pool is used up (or the device's
// array cannot be looked up during a capture): the caller then takes the path without a counter
int next_arrive_counter(hipStream_t st, int** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= ARRIVE_MAX_DEVICES)
    OMNI_FAIL(OMNI_E_LAUNCH, "route_quant_permute: no current device (or device index >= %d)", ARRIVE_MAX_DEVICES);
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  unsigned long long capture_id = 0;
  if (hipStreamGetCaptureInfo(st, &status, &capture_id) != hipSuccess) {
    (void)hipGetLastError();
    status = hipStreamCaptureStatusNone;
  }
  const bool capturing = status == hipStreamCaptureStatusActive;
  int* base;
  {
    std::lock_guard<std::mutex> lock(g_arrive_mutex);
    if (g_arrive_ptr[dev] == nullptr) {
      if (capturing) return 1;  // the symbol look-up is not a call to make inside a capture
      void* ptr = nullptr;
      const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(arrive_counters));
      if (e != hipSuccess || ptr == nullptr)
        OMNI_FAIL(OMNI_E_LAUNCH, "route_quant_permute: hipGetSymbolAddress(arrive_counters): %s", hipGetErrorString(e));
      g_arrive_ptr[dev] = (int*)ptr;
    }
    base = g_arrive_ptr[dev];
  }
  // capture ids start at 1; 0 stands for "not captured" in the book
  const int slot = g_arrive_book[dev].take(capturing ? (capture_id ? capture_id : ~0ull) : 0ull, (uintptr_t)st);
  if (slot < 0) return 1;
  *out = base + slot;
  return OMNI_OK;
}
}  // namespace

// Internal to the library (the whole-layer entry uses it): route, quantise bf16 rows and sort the assignments in
// one launch.  Returns 1 without launching when the shapes do not fit that kernel.  The routing arguments have
// been checked by the caller (omni_route_check).
int omni_route_quant_permute_fused(const OmniRouteParams* rp, const void* x_bf16, int T, int H, int8_t* q, float* scale,
                                   int K, int lo, int hi, int32_t* sorted_src, int32_t* src_to_dst, int32_t* counts,
                                   int32_t* offsets, int32_t* zero_words, int zero_n, void* stream) {
  const int G = hi - lo;
  const int64_t n = (int64_t)T * K;
  if (T <= 0 || n > CH_SINGLE || G > GMAX) return 1;
  // x_bf16 == null: the tokens are quantised already, the launch routes and sorts only
  const int64_t qrows = x_bf16 ? T : 0;
  if (x_bf16 && (H % 8 != 0 || H > 8 * 256 * 4)) return 1;
  if (x_bf16 && (((uintptr_t)x_bf16 % 16) || ((uintptr_t)q % 8) || ((size_t)H * 2) % 16 != 0)) return 1;
  const bool fold = rp->partials != nullptr;
  if (fold) {
    // a routing block per token, four wavefronts: up to 1024 assignments and 16 groups of partial sums
    const int n_groups = (rp->n_parts + rp->group_len - 1) / rp->group_len;
    if (n > NW_SMALL_MAX_N || n_groups > OMNI_FOLD_MAX_GROUPS || rp->group_len > 8) return 1;
  }
  hipStream_t st = (hipStream_t)stream;
  int* arrive = nullptr;
  const int rc = next_arrive_counter(st, &arrive);
  if (rc) return rc;  // 1: no counter to be had (capture pool used up): the caller launches router and sort apart
  RouteArgs r{rp->logits, rp->partials, rp->n_parts, rp->group_len, fold ? 1 : 0, rp->logits_out, rp->round_logits_bf16,
              rp->bias, T, rp->E, rp->n_group, rp->topk_group, K, rp->score_fn, rp->group_mode, rp->masked_fill_zero,
              rp->weight_from_c, rp->renorm, rp->scale, rp->eps, rp->topk_w, rp->topk_ids};
  PermArgs a{rp->topk_ids, (int)n, T, K, lo, G, OMNI_IDX_TOKEN_MAJOR, sorted_src, src_to_dst, counts, offsets, nullptr, 0,
             zero_words, zero_words ? zero_n : 0};
  const int nw = fold ? 4 : sort_waves((int)n), rpb = nw / 4;
  const int route_blocks = fold ? T : (T + nw - 1) / nw;
  dim3 grid((unsigned)(route_blocks + (qrows + rpb - 1) / rpb)), block(nw * WAVE);
  const int V = (rp->E + 63) / 64;
  const int MV = H <= 8 * 256 ? 1 : (H <= 8 * 256 * 2 ? 2 : 4);
#define RQP_LAUNCH(MAXV, VV)                                                                                                  \
  do {                                                                                                                        \
    if (fold) hipLaunchKernelGGL((route_quant_permute_small<MAXV, VV, 4, true>), grid, block, 0, st, x_bf16, qrows, H, q, scale, r, a, arrive); \
    else if (nw == 4) hipLaunchKernelGGL((route_quant_permute_small<MAXV, VV, 4, false>), grid, block, 0, st, x_bf16, qrows, H, q, scale, r, a, arrive); \
    else hipLaunchKernelGGL((route_quant_permute_small<MAXV, VV, 16, false>), grid, block, 0, st, x_bf16, qrows, H, q, scale, r, a, arrive);       \
  } while (0)
#define RQP_V(MAXV)                      \
  do {                                   \
    if (V <= 1) RQP_LAUNCH(MAXV, 1);     \
    else if (V <= 2) RQP_LAUNCH(MAXV, 2); \
    else if (V <= 4) RQP_LAUNCH(MAXV, 4); \
    else RQP_LAUNCH(MAXV, 8);            \
  } while (0)
  if (MV == 1) RQP_V(1);
  else if (MV == 2) RQP_V(2);
  else RQP_V(4);
#undef RQP_V
#undef RQP_LAUNCH
  OMNI_CHECK_LAUNCH("route_quant_permute");
  return OMNI_OK;
}

// ---- group offsets from group sizes: one block, a thread per group, the prefix over the lanes of a wavefront
// with data-parallel moves and over the wavefronts through LDS
namespace {
__global__ __launch_bounds__(GMAX) void group_offsets_kernel(const void* __restrict__ counts, int wide, int G,
                                                            int32_t* __restrict__ offsets) {
  __shared__ int wave_tot[GMAX / WAVE];
  const int g = threadIdx.x, lane = g & (WAVE - 1), wv = g / WAVE;
  int c = 0;
  if (g < G) c = wide ? (int)((const int64_t*)counts)[g] : ((const int32_t*)counts)[g];
  const int incl = wave_incl_scan_dpp_i(c);
  if (lane == WAVE - 1) wave_tot[wv] = incl;
  __syncthreads();
  int base = 0;
  for (int i = 0; i < wv; ++i) base += wave_tot[i];
  if (g < G) offsets[g + 1] = base + incl;
  if (g == 0) offsets[0] = 0;
}
}  // namespace

extern "C" int omni_moe_group_offsets(const void* counts, int counts_are_int64, int G, int32_t* offsets, void* stream) {
  if (G < 0) OMNI_FAIL(OMNI_E_INVALID, "group_offsets: bad size G=%d", G);
  if (G > GMAX) OMNI_FAIL(OMNI_E_UNSUPPORTED, "group_offsets: %d groups > %d", G, GMAX);
  if (!offsets || (G > 0 && !counts)) OMNI_FAIL(OMNI_E_INVALID, "group_offsets: null pointer");
  hipLaunchKernelGGL(group_offsets_kernel, dim3(1), dim3(GMAX), 0, (hipStream_t)stream, counts, counts_are_int64 ? 1 : 0, G,
                     offsets);
  OMNI_CHECK_LAUNCH("group_offsets");
  return OMNI_OK;
}

extern "C" int omni_moe_gather_rows(const void* x, int elem_bytes, int H, const float* x_scale,
                                    const int32_t* sorted_src, const int32_t* offsets, int n_local, int T, int K,
                                    int idx_mode, void* rows_out, float* scale_out, void* stream) {
  if (T < 0 || K <= 0 || H <= 0 || elem_bytes <= 0 || n_local <= 0) OMNI_FAIL(OMNI_E_INVALID, "gather_rows: bad sizes");
  if (T == 0) return OMNI_OK;
  if (!x || !sorted_src || !offsets || !rows_out) OMNI_FAIL(OMNI_E_INVALID, "gather_rows: null pointer");
  GatherArgs g{(const uint8_t*)x, (int64_t)H * elem_bytes, x_scale, sorted_src, offsets, n_local, T, K, idx_mode,
               (uint8_t*)rows_out, scale_out};
  hipLaunchKernelGGL(gather_rows_kernel, dim3((unsigned)((int64_t)T * K)), dim3(256), 0, (hipStream_t)stream, g);
  OMNI_CHECK_LAUNCH("gather_rows");
  return OMNI_OK;
}
