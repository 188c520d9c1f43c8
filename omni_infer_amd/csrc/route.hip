// Grouped top-k router: one wavefront per token.
//
// Lane l owns the V = ceil(E/64) consecutive experts [V*l, V*l + V).  Scores, group scores and
// the K selection rounds are all wave-level reductions (DPP inside a row of 16 lanes, bpermute
// across rows); nothing goes through LDS or global memory between the logits load and the
// K (weight, id) stores.
//
// The same kernel also finishes the gate projection: when it is given partial sums of the logits
// (gate_partial_kernel below) it adds them up in the stated order before it routes, so the logits
// never make a round trip of their own and the two launches of this file are the whole
// gate + router.
//
// Gate projection: logits[t][e] = sum_k x[t][k] * w[e][k] on the fp32 matrix cores with a fixed order.
//   v_mfma_f32_32x32x1_2b_f32 is a rank-1 update, one fused multiply-add (a single rounding) per
//   output element; a run of them over ascending k is therefore an exactly specified chain
//       acc = fma(x[t][k], w[e][k], acc),  acc = +0 at the start of a slice.
//   The reduction is cut into slices of 128 elements and groups of 8 slices:
//       P_s = fma chain over slice s;  Q_g = P_8g + P_8g+1 + ... (left to right, fp32 adds);
//       logits = Q_0 + Q_1 + ... (left to right).
//   How the slices are dealt to wavefronts (one slice each for small batches, one group each for
//   large ones) does not change a bit of the result.
#include <stdlib.h>
#include "common.h"
#include "route_body.h"

namespace {

constexpr int GATE_SLICE = 128;  // reduction elements of one fma chain (GATE_GROUP of them make a group: route_body.h)

template <int V>
__global__ __launch_bounds__(256) void route_kernel(RouteArgs a) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int wv = threadIdx.x / WAVE;
  // one token per wavefront; with fold_block one token per block: its four wavefronts add up the partial
  // sums of the gate projection together (one round of loads), then the first one routes
  const int t = a.fold_block ? (int)blockIdx.x : (int)blockIdx.x * (blockDim.x / WAVE) + wv;
  if (t >= a.T) return;  // whole wave leaves together

  float s[V];  // score
  bool in[V];
  float bias[V];
  route_load_bias<V>(a, lane, bias);
#pragma unroll
  for (int j = 0; j < V; ++j) in[j] = lane * V + j < a.E;
  if (a.partials == nullptr) {
    const float* row = a.logits + (size_t)t * a.E;
#pragma unroll
    for (int j = 0; j < V; ++j) s[j] = in[j] ? row[lane * V + j] : NEG_INF;
  } else {
    // finish the gate projection: groups of `group_len` parts left to right, then the groups left to right
    float tot[V];
    if (a.fold_block) {
      __shared__ float s_q[FOLD_MAX_GROUPS][WAVE * V];
      if (!route_fold_block<V>(a, t, lane, wv, in, tot, s_q)) return;
    } else {
      route_fold_wave<V>(a, t, lane, in, tot);
    }
    route_finish_logits<V>(a, t, lane, in, tot, s);
    if (a.K == 0) return;  // the logits were all that was asked for
  }
  route_token<V>(a, t, lane, s, in, bias);
}


// ---------------------------------------------------------------- gate projection, partial sums
struct GateArgs {
  const void* x;   // [T, H] bf16 or fp32
  const void* w;   // [E, H] fp32 or bf16
  int T, H, E;
  int slices_per_task;  // 1 or GATE_GROUP
  int n_parts;          // H / 128 / slices_per_task, rounded up
  int n_tt, n_et;       // token tiles of 64, expert tiles of 32
  float* partials;      // [n_parts][T][E]
};

typedef float v32f __attribute__((ext_vector_type(32)));

// 32 consecutive reduction elements of one row as floats, loaded with 16-byte loads
template <int DT>
struct Chunk32;
template <>
struct Chunk32<OMNI_DT_F32> {
  v4f r[8];
  __device__ __forceinline__ void load(const void* row, int k) {
    const v4f* p = (const v4f*)((const float*)row + k);
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = p[i];
  }
  __device__ __forceinline__ float at(int k) const { return r[k >> 2][k & 3]; }
};
template <>
struct Chunk32<OMNI_DT_BF16> {
  v4i r[4];
  __device__ __forceinline__ void load(const void* row, int k) {
    const v4i* p = (const v4i*)((const uint16_t*)row + k);
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = p[i];
  }
  __device__ __forceinline__ float at(int k) const {
    const uint32_t word = (uint32_t)r[k >> 3][(k >> 1) & 3];
    return __uint_as_float((k & 1) ? (word & 0xffff0000u) : (word << 16));
  }
};

// One wavefront per task: 64 tokens x 32 experts x `slices_per_task` slices of 128 reduction elements.
// Lane l supplies token t0 + l (the matrix instruction's two 32-row blocks are the two halves of the token
// tile) and expert e0 + l % 32.  The whole first slice is requested before the first multiply; while a chunk
// of 32 elements is multiplied, the same chunk of the next slice is requested into the registers just used,
// so the loads run a full slice (128 matrix instructions) ahead and one wavefront per SIMD keeps the matrix
// pipe fed.  Output element (token t0 + 32 b + 8 (j/4) + 4 (l/32) + j%4, expert e0 + l%32) sits in
// accumulator register 16 b + j of lane l.
template <int XDT, int WDT>
__global__ __launch_bounds__(64) void gate_partial_kernel(GateArgs a) {
  const int lane = threadIdx.x;
  int id = blockIdx.x;
  const int tt = id % a.n_tt; id /= a.n_tt;
  const int et = id % a.n_et; id /= a.n_et;
  const int part = id;
  const int n_slices = a.H / GATE_SLICE;
  const int s_first = part * a.slices_per_task;
  const int s_end = min(n_slices, s_first + a.slices_per_task);
  const int tok = min(tt * 64 + lane, a.T - 1);           // rows past the end alias the last row; not stored
  const int exp = min(et * 32 + (lane & 31), a.E - 1);
  const size_t xes = (XDT == OMNI_DT_F32) ? 4 : 2, wes = (WDT == OMNI_DT_F32) ? 4 : 2;
  const char* xrow = (const char*)a.x + (size_t)tok * a.H * xes;
  const char* wrow = (const char*)a.w + (size_t)exp * a.H * wes;

  Chunk32<XDT> xb[4];
  Chunk32<WDT> wb[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    xb[c].load(xrow, s_first * GATE_SLICE + c * 32);
    wb[c].load(wrow, s_first * GATE_SLICE + c * 32);
  }
  __builtin_amdgcn_sched_barrier(0);  // the loads stay where they are written: ahead of the multiplies
  v32f acc, q;
#pragma unroll
  for (int i = 0; i < 32; ++i) { acc[i] = 0.0f; q[i] = 0.0f; }
  for (int s = s_first; s < s_end; ++s) {
    const int s_next = min(s + 1, s_end - 1);  // the last slice is requested once more instead of a branch
#pragma unroll
    for (int c = 0; c < 4; ++c) {
#pragma unroll
      for (int k = 0; k < 32; ++k) acc = __builtin_amdgcn_mfma_f32_32x32x1f32(xb[c].at(k), wb[c].at(k), acc, 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      xb[c].load(xrow, s_next * GATE_SLICE + c * 32);
      wb[c].load(wrow, s_next * GATE_SLICE + c * 32);
      __builtin_amdgcn_sched_barrier(0);
    }
    // the slice's chain is complete: add it to the group's sum (the first slice starts it)
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      q[i] = (s == s_first) ? acc[i] : q[i] + acc[i];
      acc[i] = 0.0f;
    }
  }
  float* out = a.partials + (size_t)part * a.T * a.E;
  const int e = et * 32 + (lane & 31);
  if (e < a.E) {
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      const int t = tt * 64 + 32 * (i >> 4) + 8 * ((i & 15) >> 2) + 4 * (lane >> 5) + (i & 3);
      if (t < a.T) out[(size_t)t * a.E + e] = q[i];
    }
  }
}

// ---------------------------------------------------------------- gate projection, large batches
// Block of four wavefronts: 128 tokens x 64 experts x one group of 8 slices, a wavefront 64 x 32 as above.
// The operands pass through LDS: every 16-byte global load covers consecutive bytes of one row (the one-
// wavefront kernel asks for 64 different cache lines per load instruction, which is what limits it once the
// batch is large), each wavefront then reads "its" row per lane (token 64 (w&1) + l, expert 32 (w>>1) + l%32)
// with 16-byte LDS reads; rows are padded by 16 bytes, so the 16 lanes that LDS serves together hit 16
// different groups of four banks.  Stages of 32 reduction elements, two LDS buffers, the global loads of the
// next stage are in flight while the current one is multiplied; one barrier per stage; three blocks per CU.
// The order of the multiply-adds and of the sums is that of the one-wavefront kernel: the same bits.
// (Two chains per wavefront against the same tokens, alternating so that no matrix instruction directly
// follows the one it accumulates onto, was measured and is not faster.)
constexpr int GT_TOK = 128, GT_EXP = 64, GT_KS = 32;

template <int DT>
struct LdsChunk16;  // 16 consecutive reduction elements of one LDS row
template <>
struct LdsChunk16<OMNI_DT_F32> {
  v4f r[4];
  __device__ __forceinline__ void load(const unsigned char* row, int k) {
    const v4f* p = (const v4f*)(row + k * 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) r[i] = p[i];
  }
  __device__ __forceinline__ float at(int k) const { return r[k >> 2][k & 3]; }
};
template <>
struct LdsChunk16<OMNI_DT_BF16> {
  v4i r[2];
  __device__ __forceinline__ void load(const unsigned char* row, int k) {
    const v4i* p = (const v4i*)(row + k * 2);
#pragma unroll
    for (int i = 0; i < 2; ++i) r[i] = p[i];
  }
  __device__ __forceinline__ float at(int k) const {
    const uint32_t word = (uint32_t)r[k >> 3][(k >> 1) & 3];
    return __uint_as_float((k & 1) ? (word & 0xffff0000u) : (word << 16));
  }
};

template <int XDT, int WDT>
__global__ __launch_bounds__(256, (XDT == OMNI_DT_F32 && WDT == OMNI_DT_F32) ? 2 : 3) void gate_tile_kernel(GateArgs a) {
  constexpr int XES = (XDT == OMNI_DT_F32) ? 4 : 2, WES = (WDT == OMNI_DT_F32) ? 4 : 2;
  constexpr int XROW = GT_KS * XES + 16, WROW = GT_KS * WES + 16;  // bytes of a padded LDS row
  constexpr int XBUF = GT_TOK * XROW, WBUF = GT_EXP * WROW;
  constexpr int XCPR = GT_KS * XES / 16, WCPR = GT_KS * WES / 16;  // 16-byte pieces of a row's stage
  constexpr int XN = GT_TOK * XCPR / 256, WN = GT_EXP * WCPR / 256;  // pieces per thread
  constexpr int SPS = GATE_SLICE / GT_KS;                           // stages per slice
  static_assert(XN >= 1 && WN >= 1 && GT_KS % 16 == 0, "stage too small for 256 threads");
  __shared__ __align__(16) unsigned char lds[2 * (XBUF + WBUF)];

  const int tid = threadIdx.x, lane = tid & (WAVE - 1), wv = tid / WAVE;
  int id = blockIdx.x;
  const int tt = id % a.n_tt; id /= a.n_tt;
  const int et = id % a.n_et; id /= a.n_et;
  const int part = id;
  const int n_slices = a.H / GATE_SLICE;
  const int s_first = part * GATE_GROUP;
  const int s_end = min(n_slices, s_first + GATE_GROUP);
  const int n_st = (s_end - s_first) * SPS;
  const size_t k_first = (size_t)s_first * GATE_SLICE;

  // what this thread carries from global memory to LDS (rows past the end alias the last row; not stored)
  const char* xsrc[XN];
  const char* wsrc[WN];
  int xdst[XN], wdst[WN];
#pragma unroll
  for (int i = 0; i < XN; ++i) {
    const int c = i * 256 + tid, row = c / XCPR, col = c % XCPR;
    xsrc[i] = (const char*)a.x + ((size_t)min(tt * GT_TOK + row, a.T - 1) * a.H + k_first) * XES + col * 16;
    xdst[i] = row * XROW + col * 16;
  }
#pragma unroll
  for (int i = 0; i < WN; ++i) {
    const int c = i * 256 + tid, row = c / WCPR, col = c % WCPR;
    wsrc[i] = (const char*)a.w + ((size_t)min(et * GT_EXP + row, a.E - 1) * a.H + k_first) * WES + col * 16;
    wdst[i] = XBUF + row * WROW + col * 16;
  }
  v4i xg[XN], wg[WN];
#pragma unroll
  for (int i = 0; i < XN; ++i) xg[i] = *(const v4i*)xsrc[i];
#pragma unroll
  for (int i = 0; i < WN; ++i) wg[i] = *(const v4i*)wsrc[i];
#pragma unroll
  for (int i = 0; i < XN; ++i) *(v4i*)(lds + xdst[i]) = xg[i];
#pragma unroll
  for (int i = 0; i < WN; ++i) *(v4i*)(lds + wdst[i]) = wg[i];
  __syncthreads();

  const int xrow_off = ((wv & 1) * 64 + lane) * XROW;
  const int wrow_off = XBUF + ((wv >> 1) * 32 + (lane & 31)) * WROW;
  v32f acc, q;
#pragma unroll
  for (int i = 0; i < 32; ++i) { acc[i] = 0.0f; q[i] = 0.0f; }
  for (int st = 0; st < n_st; ++st) {
    const int st_next = min(st + 1, n_st - 1);  // the last stage is requested once more instead of a branch
#pragma unroll
    for (int i = 0; i < XN; ++i) xg[i] = *(const v4i*)(xsrc[i] + (size_t)st_next * GT_KS * XES);
#pragma unroll
    for (int i = 0; i < WN; ++i) wg[i] = *(const v4i*)(wsrc[i] + (size_t)st_next * GT_KS * WES);
    const unsigned char* buf = lds + (st & 1) * (XBUF + WBUF);
    LdsChunk16<XDT> xc[2];
    LdsChunk16<WDT> wc[2];
    xc[0].load(buf + xrow_off, 0);
    wc[0].load(buf + wrow_off, 0);
    // the scheduling barriers keep the requests where they are written: the global loads a whole stage, the
    // LDS reads sixteen steps ahead of their use
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < GT_KS / 16; ++j) {
      if (j + 1 < GT_KS / 16) {
        xc[(j + 1) & 1].load(buf + xrow_off, (j + 1) * 16);
        wc[(j + 1) & 1].load(buf + wrow_off, (j + 1) * 16);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int k = 0; k < 16; ++k)
        acc = __builtin_amdgcn_mfma_f32_32x32x1f32(xc[j & 1].at(k), wc[j & 1].at(k), acc, 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    unsigned char* nbuf = lds + ((st + 1) & 1) * (XBUF + WBUF);
#pragma unroll
    for (int i = 0; i < XN; ++i) *(v4i*)(nbuf + xdst[i]) = xg[i];
#pragma unroll
    for (int i = 0; i < WN; ++i) *(v4i*)(nbuf + wdst[i]) = wg[i];
    __syncthreads();
    if ((st & (SPS - 1)) == SPS - 1) {
      // the slice's chain is complete: add it to the group's sum (the first slice starts it)
#pragma unroll
      for (int i = 0; i < 32; ++i) {
        q[i] = (st < SPS) ? acc[i] : q[i] + acc[i];
        acc[i] = 0.0f;
      }
    }
  }
  float* out = a.partials + (size_t)part * a.T * a.E;
  const int e = et * GT_EXP + (wv >> 1) * 32 + (lane & 31);
  if (e < a.E) {
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      const int t = tt * GT_TOK + (wv & 1) * 64 + 32 * (i >> 4) + 8 * ((i & 15) >> 2) + 4 * (lane >> 5) + (i & 3);
      if (t < a.T) out[(size_t)t * a.E + e] = q[i];
    }
  }
}

// Tuning aids, read from the environment once.
struct GateTuning {
  int group_tasks;  // from this many (64 tokens x 32 experts x group) tasks on, a task is a whole group of slices
  int tile_from;    // from this many tokens on, the block kernel that passes the operands through LDS
};
const GateTuning& gate_tuning() {
  static const GateTuning t = [] {
    GateTuning g{400, 1024};
    if (const char* e = getenv("OMNI_MOE_GATE_GROUP_TASKS")) { const int v = atoi(e); if (v > 0) g.group_tasks = v; }
    if (const char* e = getenv("OMNI_MOE_GATE_TILE_FROM")) { const int v = atoi(e); if (v > 0) g.tile_from = v; }
    return g;
  }();
  return t;
}

// small batches: one slice per wavefront (many short tasks); large ones: a group of 8 slices each
int gate_slices_per_task(int T, int H, int E) {
  const int n_tt = (T + 63) / 64, n_et = (E + 31) / 32;
  const int n_groups = (H / GATE_SLICE + GATE_GROUP - 1) / GATE_GROUP;
  return ((int64_t)n_tt * n_et * n_groups >= gate_tuning().group_tasks) ? GATE_GROUP : 1;
}

void launch_route(const RouteArgs& a, hipStream_t st) {
  dim3 grid(a.fold_block ? a.T : (a.T + 3) / 4), block(256);
  const int V = (a.E + 63) / 64;
  if (V <= 1) hipLaunchKernelGGL(route_kernel<1>, grid, block, 0, st, a);
  else if (V <= 2) hipLaunchKernelGGL(route_kernel<2>, grid, block, 0, st, a);
  else if (V <= 4) hipLaunchKernelGGL(route_kernel<4>, grid, block, 0, st, a);
  else hipLaunchKernelGGL(route_kernel<8>, grid, block, 0, st, a);
}

int check_route_args(const char* what, int T, int E, int n_group, int topk_group, int K, int score_fn) {
  if (E > 512) OMNI_FAIL(OMNI_E_UNSUPPORTED, "%s: E=%d > 512", what, E);
  if (K > 64 || K > E) OMNI_FAIL(OMNI_E_UNSUPPORTED, "%s: K=%d must be <= min(64, E=%d)", what, K, E);
  if (score_fn != OMNI_SCORE_SOFTMAX && score_fn != OMNI_SCORE_SIGMOID)
    OMNI_FAIL(OMNI_E_INVALID, "%s: unknown score_fn %d", what, score_fn);
  if (n_group > 1) {
    if (n_group > 64 || E % n_group != 0) OMNI_FAIL(OMNI_E_UNSUPPORTED, "%s: n_group=%d must divide E=%d and be <= 64", what, n_group, E);
    if (topk_group < 1 || topk_group > n_group) OMNI_FAIL(OMNI_E_INVALID, "%s: topk_group=%d out of range", what, topk_group);
  }
  (void)T;
  return OMNI_OK;
}

}  // namespace

int omni_route_check(const char* what, int T, int E, int n_group, int topk_group, int K, int score_fn) {
  return check_route_args(what, T, E, n_group, topk_group, K, score_fn);
}

int omni_route_launch(const OmniRouteParams* rp, int T, int K, void* stream) {
  // few tokens: a block per token adds the parts up with its four wavefronts (the latency of one round of
  // loads instead of one per group); many tokens: a wavefront per token keeps every wavefront routing
  const int n_groups = rp->partials ? (rp->n_parts + rp->group_len - 1) / rp->group_len : 0;
  const int fold_block = (rp->partials && T <= 2048 && n_groups <= FOLD_MAX_GROUPS) ? 1 : 0;
  RouteArgs a{rp->logits, rp->partials, rp->n_parts, rp->group_len, fold_block, rp->logits_out, rp->round_logits_bf16,
              rp->bias, T, rp->E, rp->n_group, rp->topk_group, K, rp->score_fn, rp->group_mode, rp->masked_fill_zero,
              rp->weight_from_c, rp->renorm, rp->scale, rp->eps, rp->topk_w, rp->topk_ids};
  launch_route(a, (hipStream_t)stream);
  OMNI_CHECK_LAUNCH("route");
  return OMNI_OK;
}

int omni_gate_partials(const void* x, int x_dtype, const void* gate_w, int w_dtype, int T, int H, int E, void* partials,
                       size_t partials_bytes, int* n_parts, int* group_len, void* stream) {
  if (!x || !gate_w) OMNI_FAIL(OMNI_E_INVALID, "gate: null pointer");
  if ((x_dtype != OMNI_DT_BF16 && x_dtype != OMNI_DT_F32) || (w_dtype != OMNI_DT_BF16 && w_dtype != OMNI_DT_F32))
    OMNI_FAIL(OMNI_E_INVALID, "gate: tokens and gate weights must be bf16 or fp32");
  if (H % GATE_SLICE != 0) OMNI_FAIL(OMNI_E_UNSUPPORTED, "gate: H=%d must be a multiple of %d", H, GATE_SLICE);
  if (((uintptr_t)x % 16) || ((uintptr_t)gate_w % 16)) OMNI_FAIL(OMNI_E_INVALID, "gate: pointers must be 16-byte aligned");
  if (E > 512) OMNI_FAIL(OMNI_E_UNSUPPORTED, "gate: E=%d > 512", E);
  const size_t need = omni_moe_gate_route_workspace_bytes(T, H, E);
  if (!partials || partials_bytes < need) OMNI_FAIL(OMNI_E_WORKSPACE, "gate: workspace %zu < %zu", partials_bytes, need);
  if ((uintptr_t)partials % 16) OMNI_FAIL(OMNI_E_INVALID, "gate: workspace must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  GateArgs g{};
  g.x = x; g.w = gate_w; g.T = T; g.H = H; g.E = E;
  g.slices_per_task = gate_slices_per_task(T, H, E);
  g.n_parts = (H / GATE_SLICE + g.slices_per_task - 1) / g.slices_per_task;
  const bool tile = g.slices_per_task == GATE_GROUP && T >= gate_tuning().tile_from;
  g.n_tt = tile ? (T + GT_TOK - 1) / GT_TOK : (T + 63) / 64;
  g.n_et = tile ? (E + GT_EXP - 1) / GT_EXP : (E + 31) / 32;
  g.partials = (float*)partials;
  const int64_t tasks = (int64_t)g.n_parts * g.n_et * g.n_tt;
  if (tasks > 0x7fffffffLL) OMNI_FAIL(OMNI_E_UNSUPPORTED, "gate: too many tasks");
  dim3 grid((unsigned)tasks), block(tile ? 256 : 64);
#define GATE_LAUNCH(KERNEL)                                                                                   \
  do {                                                                                                        \
    if (x_dtype == OMNI_DT_BF16 && w_dtype == OMNI_DT_F32) hipLaunchKernelGGL((KERNEL<OMNI_DT_BF16, OMNI_DT_F32>), grid, block, 0, st, g); \
    else if (x_dtype == OMNI_DT_BF16) hipLaunchKernelGGL((KERNEL<OMNI_DT_BF16, OMNI_DT_BF16>), grid, block, 0, st, g);  \
    else if (w_dtype == OMNI_DT_F32) hipLaunchKernelGGL((KERNEL<OMNI_DT_F32, OMNI_DT_F32>), grid, block, 0, st, g);     \
    else hipLaunchKernelGGL((KERNEL<OMNI_DT_F32, OMNI_DT_BF16>), grid, block, 0, st, g);                               \
  } while (0)
  if (tile) GATE_LAUNCH(gate_tile_kernel);
  else GATE_LAUNCH(gate_partial_kernel);
#undef GATE_LAUNCH
  OMNI_CHECK_LAUNCH("gate_partial");
  *n_parts = g.n_parts;
  *group_len = g.slices_per_task == 1 ? GATE_GROUP : 1;
  return OMNI_OK;
}

extern "C" int omni_moe_route(const float* logits, const float* bias, int T, int E, int n_group, int topk_group,
                              int K, int score_fn, int group_mode, int masked_fill_zero, int weight_from_c,
                              int renorm, float scale, float eps, float* topk_w, int32_t* topk_ids, void* stream) {
  if (T < 0 || E <= 0 || K <= 0) OMNI_FAIL(OMNI_E_INVALID, "route: bad sizes T=%d E=%d K=%d", T, E, K);
  if (T == 0) return OMNI_OK;
  if (!logits || !topk_w || !topk_ids) OMNI_FAIL(OMNI_E_INVALID, "route: null pointer");
  const int rc = check_route_args("route", T, E, n_group, topk_group, K, score_fn);
  if (rc) return rc;
  OmniRouteParams rp{logits, bias, E, n_group, topk_group, score_fn, group_mode, masked_fill_zero, weight_from_c, renorm,
                     scale, eps, topk_w, topk_ids};
  return omni_route_launch(&rp, T, K, stream);
}

extern "C" size_t omni_moe_gate_route_workspace_bytes(int T, int H, int E) {
  if (T <= 0 || H <= 0 || E <= 0 || H % GATE_SLICE != 0) return 0;
  const int spt = gate_slices_per_task(T, H, E);
  const int n_parts = (H / GATE_SLICE + spt - 1) / spt;
  return align256((size_t)n_parts * T * E * sizeof(float));
}

extern "C" int omni_moe_gate_route(const void* x, int x_dtype, const void* gate_w, int w_dtype, const float* bias, int T,
                                   int H, int E, int n_group, int topk_group, int K, int score_fn, int group_mode,
                                   int masked_fill_zero, int weight_from_c, int renorm, float scale, float eps,
                                   int round_logits_bf16, float* logits_out, float* topk_w, int32_t* topk_ids,
                                   void* workspace, size_t ws_bytes, void* stream) {
  if (T < 0 || H <= 0 || E <= 0 || K < 0) OMNI_FAIL(OMNI_E_INVALID, "gate_route: bad sizes T=%d H=%d E=%d K=%d", T, H, E, K);
  if (T == 0) return OMNI_OK;
  if (!x || !gate_w) OMNI_FAIL(OMNI_E_INVALID, "gate_route: null pointer");
  if (K == 0 && !logits_out) OMNI_FAIL(OMNI_E_INVALID, "gate_route: nothing to compute (K = 0 and no logits_out)");
  if (K > 0 && (!topk_w || !topk_ids)) OMNI_FAIL(OMNI_E_INVALID, "gate_route: null pointer");
  if (K > 0) {
    const int rc = check_route_args("gate_route", T, E, n_group, topk_group, K, score_fn);
    if (rc) return rc;
  }
  OmniRouteParams rp{nullptr, bias, E, n_group, topk_group, score_fn, group_mode, masked_fill_zero, weight_from_c, renorm,
                     scale, eps, topk_w, topk_ids};
  int rc = omni_gate_partials(x, x_dtype, gate_w, w_dtype, T, H, E, workspace, ws_bytes, &rp.n_parts, &rp.group_len, stream);
  if (rc) return rc;
  rp.partials = (const float*)workspace;
  rp.round_logits_bf16 = round_logits_bf16;
  rp.logits_out = logits_out;
  return omni_route_launch(&rp, T, K, stream);
}
