// Grouped top-k router: one wavefront per token.
//
// Lane l owns the V = ceil(E/64) consecutive experts [V*l, V*l + V).  Scores, group scores and
// the K selection rounds are all wave-level reductions (DPP inside a row of 16 lanes, bpermute
// across rows); nothing goes through LDS or global memory between the logits load and the
// K (weight, id) stores.
#include "common.h"

namespace {

struct RouteArgs {
  const float* logits;
  const float* bias;
  int T, E, n_group, topk_group, K;
  int score_fn, group_mode, masked_fill_zero, weight_from_c, renorm;
  float scale, eps;
  float* topk_w;
  int32_t* topk_ids;
};

constexpr float NEG_INF = -__builtin_inff();

template <int V>
__global__ __launch_bounds__(256) void route_kernel(RouteArgs a) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int t = blockIdx.x * (blockDim.x / WAVE) + (threadIdx.x / WAVE);
  if (t >= a.T) return;  // whole wave leaves together
  const float* row = a.logits + (size_t)t * a.E;

  float s[V];  // score
  float c[V];  // selection score
  bool in[V];
#pragma unroll
  for (int j = 0; j < V; ++j) {
    int e = lane * V + j;
    in[j] = e < a.E;
    s[j] = in[j] ? row[e] : NEG_INF;
  }
  if (a.score_fn == OMNI_SCORE_SIGMOID) {
#pragma unroll
    for (int j = 0; j < V; ++j) s[j] = in[j] ? sigmoid_spec(s[j]) : 0.0f;
  } else {
    float m = NEG_INF;
#pragma unroll
    for (int j = 0; j < V; ++j) m = fmaxf(m, s[j]);
    m = wave_allmax_f(m);
    float part = 0.0f;
#pragma unroll
    for (int j = 0; j < V; ++j) {
      s[j] = in[j] ? exp_spec(s[j] - m) : 0.0f;
      part = (j == 0) ? s[0] : part + s[j];
    }
    float tot = wave_allsum_f(part);
#pragma unroll
    for (int j = 0; j < V; ++j) s[j] = s[j] / tot;
  }
#pragma unroll
  for (int j = 0; j < V; ++j) {
    float b = (a.bias != nullptr && in[j]) ? a.bias[lane * V + j] : 0.0f;
    c[j] = in[j] ? (a.bias != nullptr ? s[j] + b : s[j]) : NEG_INF;
  }

  // ---- group limiting
  if (a.n_group > 1) {
    const int gsz = a.E / a.n_group;
    int ge[V];  // group of each owned expert
#pragma unroll
    for (int j = 0; j < V; ++j) ge[j] = (lane * V + j) / gsz;
    float my_gs = NEG_INF;  // lane g keeps the score of group g
#define MERGE2(S)                                         \
  {                                                       \
    float b1 = xchg_f<S>(a1), b2 = xchg_f<S>(a2);         \
    float n1 = fmaxf(a1, b1);                             \
    float n2 = fmaxf(fminf(a1, b1), fmaxf(a2, b2));       \
    a1 = n1; a2 = n2;                                     \
  }
    const int L = gsz / V;  // lanes per group when a group is a whole power-of-two run of lanes
    if (gsz % V == 0 && (L & (L - 1)) == 0 && a.E == WAVE * V) {
      // every group at once: (largest, second largest) merged inside each run of L lanes
      float a1 = NEG_INF, a2 = NEG_INF;
#pragma unroll
      for (int j = 0; j < V; ++j) {
        float v = c[j];
        if (v > a1) { a2 = a1; a1 = v; }
        else if (v > a2) { a2 = v; }
      }
      if (L > 1) MERGE2(1)
      if (L > 2) MERGE2(2)
      if (L > 4) MERGE2(4)
      if (L > 8) MERGE2(8)
      if (L > 16) MERGE2(16)
      if (L > 32) MERGE2(32)
      float gs = (a.group_mode == OMNI_GROUP_TOP2SUM) ? a1 + a2 : a1;
      my_gs = __shfl(gs, (lane < a.n_group) ? lane * L : 0, WAVE);
    } else {
      for (int g = 0; g < a.n_group; ++g) {
        float a1 = NEG_INF, a2 = NEG_INF;
#pragma unroll
        for (int j = 0; j < V; ++j) {
          if (in[j] && ge[j] == g) {
            float v = c[j];
            if (v > a1) { a2 = a1; a1 = v; }
            else if (v > a2) { a2 = v; }
          }
        }
        MERGE2(1) MERGE2(2) MERGE2(4) MERGE2(8) MERGE2(16) MERGE2(32)
        float gs = (a.group_mode == OMNI_GROUP_TOP2SUM) ? a1 + a2 : a1;
        if (lane == g) my_gs = gs;
      }
    }
#undef MERGE2
    // a group is kept when fewer than topk_group groups beat it (higher score, or the same score
    // and a lower index): the same set as topk_group rounds of arg-max
    const uint32_t gkey = f32_order_key(my_gs);
    int beaten = 0;
    for (int g = 0; g < a.n_group; ++g) {
      uint32_t ok = (uint32_t)__builtin_amdgcn_readlane((int)gkey, g);
      beaten += (ok > gkey || (ok == gkey && g < lane)) ? 1 : 0;
    }
    const uint64_t kept = __ballot(lane < a.n_group && beaten < a.topk_group);
#pragma unroll
    for (int j = 0; j < V; ++j) {
      if (in[j] && !((kept >> ge[j]) & 1ull)) c[j] = a.masked_fill_zero ? 0.0f : NEG_INF;
    }
  }

  // ---- K rounds of wave arg-max; ties go to the lower expert id.  A round: each lane's best
  // remaining key, the wave maximum, then the lowest lane holding it (lanes own ascending ids).
  uint32_t ck[V];  // order keys of the remaining candidates; 0 once taken (real keys are > 0)
#pragma unroll
  for (int j = 0; j < V; ++j) ck[j] = in[j] ? f32_order_key(c[j]) : 0u;
  float my_w = 0.0f;
  int my_id = 0;
  float denom = 0.0f;
  for (int k = 0; k < a.K; ++k) {
    uint32_t best = ck[0];
    int bj = 0;
#pragma unroll
    for (int j = 1; j < V; ++j) {
      if (ck[j] > best) { best = ck[j]; bj = j; }
    }
    const uint32_t top = wave_allmax_u32(best);
    const uint64_t holders = __ballot(best == top && best != 0u);
    const int owner = __ffsll((unsigned long long)holders) - 1;
    float wv = 0.0f;
#pragma unroll
    for (int j = 0; j < V; ++j) {
      if (bj == j) wv = a.weight_from_c ? c[j] : s[j];
    }
    if (lane == owner) {
#pragma unroll
      for (int j = 0; j < V; ++j) {
        if (bj == j) ck[j] = 0u;
      }
    }
    const int id = owner * V + __builtin_amdgcn_readlane(bj, owner);
    wv = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wv), owner));
    denom = (k == 0) ? wv : denom + wv;
    if (lane == k) { my_w = wv; my_id = id; }
  }
  if (lane < a.K) {
    float w = my_w;
    if (a.renorm) w = w / (denom + a.eps);
    w = w * a.scale;
    a.topk_w[(size_t)t * a.K + lane] = w;
    a.topk_ids[(size_t)t * a.K + lane] = my_id;
  }
}

}  // namespace

extern "C" int omni_moe_route(const float* logits, const float* bias, int T, int E, int n_group, int topk_group,
                              int K, int score_fn, int group_mode, int masked_fill_zero, int weight_from_c,
                              int renorm, float scale, float eps, float* topk_w, int32_t* topk_ids, void* stream) {
  if (T < 0 || E <= 0 || K <= 0) OMNI_FAIL(OMNI_E_INVALID, "route: bad sizes T=%d E=%d K=%d", T, E, K);
  if (T == 0) return OMNI_OK;
  if (!logits || !topk_w || !topk_ids) OMNI_FAIL(OMNI_E_INVALID, "route: null pointer");
  if (E > 512) OMNI_FAIL(OMNI_E_UNSUPPORTED, "route: E=%d > 512", E);
  if (K > 64 || K > E) OMNI_FAIL(OMNI_E_UNSUPPORTED, "route: K=%d must be <= min(64, E=%d)", K, E);
  if (score_fn != OMNI_SCORE_SOFTMAX && score_fn != OMNI_SCORE_SIGMOID)
    OMNI_FAIL(OMNI_E_INVALID, "route: unknown score_fn %d", score_fn);
  if (n_group > 1) {
    if (n_group > 64 || E % n_group != 0) OMNI_FAIL(OMNI_E_UNSUPPORTED, "route: n_group=%d must divide E=%d and be <= 64", n_group, E);
    if (topk_group < 1 || topk_group > n_group) OMNI_FAIL(OMNI_E_INVALID, "route: topk_group=%d out of range", topk_group);
  }
  RouteArgs a{logits, bias, T, E, n_group, topk_group, K, score_fn, group_mode, masked_fill_zero, weight_from_c, renorm,
              scale, eps, topk_w, topk_ids};
  dim3 grid((T + 3) / 4), block(256);
  hipStream_t st = (hipStream_t)stream;
  int V = (E + 63) / 64;
  if (V <= 1) hipLaunchKernelGGL(route_kernel<1>, grid, block, 0, st, a);
  else if (V <= 2) hipLaunchKernelGGL(route_kernel<2>, grid, block, 0, st, a);
  else if (V <= 4) hipLaunchKernelGGL(route_kernel<4>, grid, block, 0, st, a);
  else hipLaunchKernelGGL(route_kernel<8>, grid, block, 0, st, a);
  OMNI_CHECK_LAUNCH("route");
  return OMNI_OK;
}
