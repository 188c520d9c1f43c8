// The router's arguments and its per-token body, shared by the routing kernel and by the kernel that routes,
// quantises and sorts in one launch.
#pragma once
#include "common.h"

namespace {

struct RouteArgs {
  const float* logits;
  // partial sums of the logits instead of the logits: [n_parts][T][E]; parts are slices (group_len 8) or
  // whole groups (group_len 1)
  const float* partials;
  int n_parts, group_len;
  int fold_block;        // the four wavefronts of a block add up one token's parts together
  float* logits_out;     // nullable: the finished logits
  int round_logits_bf16; // round the finished logits to bf16 (the bf16 gate of deepseek_v3_a2.py:607-613)
  const float* bias;
  int T, E, n_group, topk_group, K;
  int score_fn, group_mode, masked_fill_zero, weight_from_c, renorm;
  float scale, eps;
  float* topk_w;
  int32_t* topk_ids;
};

constexpr float NEG_INF = -__builtin_inff();

// The selection bias of the lane's V experts (0 without a bias).  Asked for before the scores are computed, so
// that its latency is not paid after them.
template <int V>
__device__ __forceinline__ void route_load_bias(const RouteArgs& a, int lane, float (&b)[V]) {
#pragma unroll
  for (int j = 0; j < V; ++j) b[j] = (a.bias != nullptr && lane * V + j < a.E) ? a.bias[lane * V + j] : 0.0f;
}

// Routes token t with one wavefront: s[] holds the logits of the lane's V experts (NEG_INF where in[] is
// false) and is overwritten, bias[] their selection bias; the K weights and ids are stored by lanes 0..K-1.
template <int V>
__device__ __forceinline__ void route_token(const RouteArgs& a, int t, int lane, float (&s)[V], const bool (&in)[V],
                                            const float (&bias)[V]) {
  float c[V];  // selection score
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
    c[j] = in[j] ? (a.bias != nullptr ? s[j] + bias[j] : s[j]) : NEG_INF;
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

// ---- finishing the gate projection from its partial sums (route.hip describes the order): groups of `group_len`
// parts are added left to right, then the groups left to right.
constexpr int GATE_GROUP = 8;        // slices added up before the groups are
constexpr int FOLD_MAX_GROUPS = OMNI_FOLD_MAX_GROUPS;  // groups of partial sums the block-wide fold takes (H <= 16384)

__device__ __forceinline__ int route_fold_groups(const RouteArgs& a) { return (a.n_parts + a.group_len - 1) / a.group_len; }

// parts of group g of token t for the lane's V experts, all requested before the first add; returns their number
template <int V>
__device__ __forceinline__ int route_load_group(const RouteArgs& a, int t, int lane, const bool (&in)[V], int g,
                                                float (&part)[GATE_GROUP][V]) {
  const size_t plane = (size_t)a.T * a.E;
  const float* p0 = a.partials + (size_t)t * a.E + lane * V;
  const int g0 = g * a.group_len;
  const int gl = (g < route_fold_groups(a)) ? min(a.group_len, a.n_parts - g0) : 0;
#pragma unroll
  for (int u = 0; u < GATE_GROUP; ++u)
#pragma unroll
    for (int j = 0; j < V; ++j) part[u][j] = (u < gl && in[j]) ? p0[(size_t)(g0 + u) * plane + j] : 0.0f;
  return gl;
}
template <int V>
__device__ __forceinline__ void route_fold_group(const float (&part)[GATE_GROUP][V], int gl, float (&q)[V]) {
#pragma unroll
  for (int j = 0; j < V; ++j) q[j] = part[0][j];
#pragma unroll
  for (int u = 1; u < GATE_GROUP; ++u)
    if (u < gl) {
#pragma unroll
      for (int j = 0; j < V; ++j) q[j] = q[j] + part[u][j];
    }
}
// One wavefront adds up everything of token t (one round of loads per group).
template <int V>
__device__ __forceinline__ void route_fold_wave(const RouteArgs& a, int t, int lane, const bool (&in)[V], float (&tot)[V]) {
  const int n_groups = route_fold_groups(a);
  for (int g = 0; g < n_groups; ++g) {
    float part[GATE_GROUP][V], q[V];
    const int gl = route_load_group<V>(a, t, lane, in, g, part);
    route_fold_group<V>(part, gl, q);
#pragma unroll
    for (int j = 0; j < V; ++j) tot[j] = (g == 0) ? q[j] : tot[j] + q[j];
  }
}
// The four wavefronts of a block add up token t together: wavefront wv takes groups wv, wv + 4, ..., two of them
// loaded before either is added up, the group sums meet in s_q and wavefront 0 adds them left to right.  All four
// wavefronts call this (block barrier inside); true for wavefront 0, whose tot[] then holds the sums.
template <int V>
__device__ __forceinline__ bool route_fold_block(const RouteArgs& a, int t, int lane, int wv, const bool (&in)[V],
                                                 float (&tot)[V], float (*s_q)[WAVE * V]) {
  const int n_groups = route_fold_groups(a);
  for (int base = 0; base < n_groups; base += 8) {
    float pa[GATE_GROUP][V], pb[GATE_GROUP][V], q[V];
    const int ga = base + wv, gb = base + 4 + wv;
    const int la = route_load_group<V>(a, t, lane, in, ga, pa);
    const int lb = route_load_group<V>(a, t, lane, in, gb, pb);
    if (la > 0) {
      route_fold_group<V>(pa, la, q);
#pragma unroll
      for (int j = 0; j < V; ++j) s_q[ga][lane * V + j] = q[j];
    }
    if (lb > 0) {
      route_fold_group<V>(pb, lb, q);
#pragma unroll
      for (int j = 0; j < V; ++j) s_q[gb][lane * V + j] = q[j];
    }
  }
  __syncthreads();
  if (wv != 0) return false;
#pragma unroll
  for (int j = 0; j < V; ++j) tot[j] = s_q[0][lane * V + j];
  for (int g = 1; g < n_groups; ++g)
#pragma unroll
    for (int j = 0; j < V; ++j) tot[j] = tot[j] + s_q[g][lane * V + j];
  return true;
}
// The finished sums become the logits the router reads: rounded to bf16 when asked, written out when asked.
template <int V>
__device__ __forceinline__ void route_finish_logits(const RouteArgs& a, int t, int lane, const bool (&in)[V],
                                                    float (&tot)[V], float (&s)[V]) {
#pragma unroll
  for (int j = 0; j < V; ++j) {
    if (a.round_logits_bf16) tot[j] = round_bf16(tot[j]);
    s[j] = in[j] ? tot[j] : NEG_INF;
    if (a.logits_out != nullptr && in[j]) a.logits_out[(size_t)t * a.E + lane * V + j] = tot[j];
  }
}

// The lane's V logits of token t from a.logits.
template <int V>
__device__ __forceinline__ void route_load_logits(const RouteArgs& a, int t, int lane, float (&s)[V], bool (&in)[V]) {
  const float* row = a.logits + (size_t)t * a.E;
#pragma unroll
  for (int j = 0; j < V; ++j) {
    in[j] = lane * V + j < a.E;
    s[j] = in[j] ? row[lane * V + j] : NEG_INF;
  }
}

}  // namespace
