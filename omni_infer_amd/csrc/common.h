// Shared device helpers for the gfx950 MoE kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/omni_moe_hip.h"
#include "../../include/omni_moe_diag.h"

// Every floating-point operation below is meant to round once: no contraction into FMA.
#pragma clang fp contract(off)

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));

#define WAVE 64

// ---------------------------------------------------------------- host side error state, host-side integer logic
// (omni_set_error, OMNI_FAIL, align256, kernel choice, tile numbering, workspace layout: host_logic.h)
#include "host_logic.h"
using omni_host::align256;
#define OMNI_CHECK_LAUNCH(what)                                                            \
  do {                                                                                     \
    hipError_t e__ = hipGetLastError();                                                    \
    if (e__ != hipSuccess) OMNI_FAIL(OMNI_E_LAUNCH, "%s: %s", what, hipGetErrorString(e__)); \
  } while (0)

// library-internal: bf16 row quantisation and assignment sort in one launch (permute.hip); 1 = not applicable.
// zero_words (may be null) are cleared by the sorting block: the whole-layer entry has the arrival counters of
// the later tile launches cleared here instead of by a launch of their own.
int omni_quant_permute_fused(const void* x_bf16, int T, int H, int8_t* q, float* scale, const int32_t* topk_ids, int K,
                             int lo, int hi, int idx_mode, int32_t* sorted_src, int32_t* src_to_dst, int32_t* counts,
                             int32_t* offsets, int32_t* zero_words, int zero_n, void* stream);
// library-internal: the router's arguments as the whole-layer entry hands them on; topk_w and topk_ids are outputs
struct OmniRouteParams {
  const float* logits;
  const float* bias;
  int E, n_group, topk_group, score_fn, group_mode, masked_fill_zero, weight_from_c, renorm;
  float scale, eps;
  float* topk_w;
  int32_t* topk_ids;
  // instead of the logits: the partial sums of the gate projection [n_parts][T][E] (omni_gate_partials), added
  // up in groups of group_len, and what is done with the finished logits
  const float* partials = nullptr;
  int n_parts = 0, group_len = 1, round_logits_bf16 = 0;
  float* logits_out = nullptr;
};
// library-internal: the argument checks of omni_moe_route (route.hip)
int omni_route_check(const char* what, int T, int E, int n_group, int topk_group, int K, int score_fn);
// library-internal (route.hip): the router as a launch of its own, on the logits or on the partial sums of rp
int omni_route_launch(const OmniRouteParams* rp, int T, int K, void* stream);
// library-internal (route.hip): the partial sums of the gate projection of omni_moe_gate_route into `partials`
// (omni_moe_gate_route_workspace_bytes(T, H, E) bytes); how many parts there are and how they are grouped
int omni_gate_partials(const void* x, int x_dtype, const void* gate_w, int w_dtype, int T, int H, int E, void* partials,
                       size_t partials_bytes, int* n_parts, int* group_len, void* stream);
// library-internal: most groups of partial sums the launch that also routes, quantises and sorts takes
constexpr int OMNI_FOLD_MAX_GROUPS = 16;
// library-internal: routing, bf16 row quantisation and assignment sort in one launch (permute.hip); 1 = not
// applicable.  zero_words as above.
int omni_route_quant_permute_fused(const OmniRouteParams* rp, const void* x_bf16, int T, int H, int8_t* q, float* scale,
                                   int K, int lo, int hi, int32_t* sorted_src, int32_t* src_to_dst, int32_t* counts,
                                   int32_t* offsets, int32_t* zero_words, int zero_n, void* stream);
// library-internal: omni_moe_permute that also clears zero_words (in its single-block kernel)
int omni_moe_permute_clearing(const int32_t* topk_ids, int T, int K, int lo, int hi, int idx_mode, int32_t* sorted_src,
                              int32_t* src_to_dst, int32_t* counts, int32_t* offsets, void* workspace, size_t ws_bytes,
                              int32_t* zero_words, int zero_n, void* stream);
// library-internal (gemm.hip): the scratch of split tiles inside a GEMM1 workspace when both grouped GEMMs of a layer
// call of this shape run the tile kernel (else null), with the number of counter words at its start that must be
// zero before the first of the two launches; and the two GEMM entries with the promise that they are.
// The same promise covers the counter words of the weight-streaming kernel's overflow blocks
// (omni_host::gemm1_stream_bal_at: where they sit in a GEMM1 workspace).
void* omni_tile_tail_area(int T, int K, int G, int extra_rows, int64_t M_cap, int H, int I, void* gemm1_ws,
                          size_t gemm1_ws_bytes, int* counter_words, size_t* tail_bytes);
int omni_gemm1_swiglu_quant_impl(const int8_t* x_q, const float* x_scale, const int32_t* sorted_src, int idx_mode, int T,
                                 int K, const int8_t* w13_packed, const float* w13_scale, const int8_t* w13_extra,
                                 const float* w13_extra_scale, int extra_rows, const int32_t* offsets, int G, int H, int I,
                                 int64_t M_cap, int flags, const float* quant_scale, int8_t* h_q, float* h_scale,
                                 int32_t* acc_dbg, void* workspace, size_t ws_bytes, bool counters_clean, void* stream);
int omni_gemm2_dequant_impl(const int8_t* h_q, const float* h_scale, const int8_t* w2_packed, const float* w2_scale,
                            const int8_t* w2_extra, const float* w2_extra_scale, int extra_rows, const int32_t* offsets,
                            int G, int H, int I, int64_t M_cap, int out_dtype, void* rows_out, int32_t* acc_dbg,
                            void* workspace, size_t ws_bytes, bool counters_clean, bool extra_rows_bf16, void* stream);

// ---------------------------------------------------------------- specified transcendental
// exp with a fixed operation sequence: clamp to [-87, 87], Cody-Waite reduction by ln2 split in
// two constants, the Cephes expf polynomial by Horner, scaling by 2^n through the exponent field.
// One rounding per operation (this file is compiled with contraction off).
__device__ __forceinline__ float exp_spec(float x) {
  x = fminf(fmaxf(x, -87.0f), 87.0f);
  float n = rintf(x * 1.44269504088896341f);
  float r = x - n * 0.693359375f;
  r = r - n * -2.12194440e-4f;
  float p = 1.9875691500e-4f;
  p = p * r;
  p = p + 1.3981999507e-3f;
  p = p * r;
  p = p + 8.3334519073e-3f;
  p = p * r;
  p = p + 4.1665795894e-2f;
  p = p * r;
  p = p + 1.6666665459e-1f;
  p = p * r;
  p = p + 5.0000001201e-1f;
  float y = p * (r * r);
  y = y + r;
  y = y + 1.0f;
  int ni = (int)n;
  return y * __int_as_float((ni + 127) << 23);
}
__device__ __forceinline__ float sigmoid_spec(float x) { return 1.0f / (1.0f + exp_spec(-x)); }
__device__ __forceinline__ float silu_spec(float x) { return x / (1.0f + exp_spec(-x)); }

// ---------------------------------------------------------------- bf16 <-> fp32
__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }
// round to nearest even; NaN stays NaN
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
// two values at once with the hardware conversion (round to nearest even): low half = a, high half = b
typedef float omni_f2 __attribute__((ext_vector_type(2)));
typedef __bf16 omni_bf2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t f32x2_to_bf16x2(float a, float b) {
  omni_f2 v = {a, b};
  omni_bf2 r = __builtin_convertvector(v, omni_bf2);
  uint32_t u;
  __builtin_memcpy(&u, &r, 4);
  return u;
}
__device__ __forceinline__ float round_bf16(float f) { return bf16_to_f32(f32_to_bf16(f)); }
__device__ __forceinline__ float f16_to_f32(uint16_t h) {
  _Float16 v;
  __builtin_memcpy(&v, &h, 2);
  return (float)v;
}

// ---------------------------------------------------------------- cross-lane exchange
// DPP inside a row of 16 lanes, ds_bpermute across rows.  xchg<S>(v) returns the value held by
// the partner lane of a butterfly step over 2*S lanes; every lane of a 2*S cluster that already
// agrees on a cluster value receives the other half's value, which is all an all-reduce needs.
template <int S>
__device__ __forceinline__ int xchg_i(int v) {
  if constexpr (S == 1) return __builtin_amdgcn_update_dpp(v, v, 0xB1, 0xf, 0xf, false);       // quad_perm [1,0,3,2]
  else if constexpr (S == 2) return __builtin_amdgcn_update_dpp(v, v, 0x4E, 0xf, 0xf, false);  // quad_perm [2,3,0,1]
  else if constexpr (S == 4) return __builtin_amdgcn_update_dpp(v, v, 0x141, 0xf, 0xf, false); // row_half_mirror
  else if constexpr (S == 8) return __builtin_amdgcn_update_dpp(v, v, 0x140, 0xf, 0xf, false); // row_mirror
  else return __shfl_xor(v, S, WAVE);
}
template <int S>
__device__ __forceinline__ float xchg_f(float v) { return __int_as_float(xchg_i<S>(__float_as_int(v))); }
template <int S>
__device__ __forceinline__ uint64_t xchg_u64(uint64_t v) {
  uint32_t lo = (uint32_t)xchg_i<S>((int)(uint32_t)v);
  uint32_t hi = (uint32_t)xchg_i<S>((int)(uint32_t)(v >> 32));
  return ((uint64_t)hi << 32) | lo;
}

__device__ __forceinline__ float wave_allmax_f(float v) {
  v = fmaxf(v, xchg_f<1>(v));
  v = fmaxf(v, xchg_f<2>(v));
  v = fmaxf(v, xchg_f<4>(v));
  v = fmaxf(v, xchg_f<8>(v));
  v = fmaxf(v, xchg_f<16>(v));
  v = fmaxf(v, xchg_f<32>(v));
  return v;
}
// butterfly sum, pairing order 1,2,4,8,16,32 (the order the checker states)
__device__ __forceinline__ float wave_allsum_f(float v) {
  v = v + xchg_f<1>(v);
  v = v + xchg_f<2>(v);
  v = v + xchg_f<4>(v);
  v = v + xchg_f<8>(v);
  v = v + xchg_f<16>(v);
  v = v + xchg_f<32>(v);
  return v;
}
__device__ __forceinline__ uint64_t wave_allmax_u64(uint64_t v) {
  uint64_t o;
  o = xchg_u64<1>(v); v = o > v ? o : v;
  o = xchg_u64<2>(v); v = o > v ? o : v;
  o = xchg_u64<4>(v); v = o > v ? o : v;
  o = xchg_u64<8>(v); v = o > v ? o : v;
  o = xchg_u64<16>(v); v = o > v ? o : v;
  o = xchg_u64<32>(v); v = o > v ? o : v;
  return v;
}
// wave-wide max of unsigned keys: four DPP steps inside each row of 16 lanes, then the four row
// results are read through scalar registers (no LDS-crossbar permutes)
__device__ __forceinline__ uint32_t wave_allmax_u32(uint32_t v) {
  uint32_t o;
  o = (uint32_t)xchg_i<1>((int)v); v = o > v ? o : v;
  o = (uint32_t)xchg_i<2>((int)v); v = o > v ? o : v;
  o = (uint32_t)xchg_i<4>((int)v); v = o > v ? o : v;
  o = (uint32_t)xchg_i<8>((int)v); v = o > v ? o : v;
  uint32_t r0 = (uint32_t)__builtin_amdgcn_readlane((int)v, 0), r1 = (uint32_t)__builtin_amdgcn_readlane((int)v, 16);
  uint32_t r2 = (uint32_t)__builtin_amdgcn_readlane((int)v, 32), r3 = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
  r0 = r0 > r1 ? r0 : r1;
  r2 = r2 > r3 ? r2 : r3;
  return r0 > r2 ? r0 : r2;
}
// max over the 16 lanes of a DPP row
__device__ __forceinline__ float row16_allmax_f(float v) {
  v = fmaxf(v, xchg_f<1>(v));
  v = fmaxf(v, xchg_f<2>(v));
  v = fmaxf(v, xchg_f<4>(v));
  v = fmaxf(v, xchg_f<8>(v));
  return v;
}
__device__ __forceinline__ int wave_incl_scan_i(int v, int lane) {
#pragma unroll
  for (int s = 1; s < WAVE; s <<= 1) {
    int o = __shfl_up(v, s, WAVE);
    if (lane >= s) v += o;
  }
  return v;
}

// inclusive prefix sum over the 64 lanes with data-parallel-primitive moves only: shifts by 1, 2, 4, 8
// inside each row of 16 lanes (lanes without a source add 0), then the last lane of row 0 / row 2 is
// added to rows 1 / 3, then lane 31 to rows 2 and 3
__device__ __forceinline__ int wave_incl_scan_dpp_i(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);  // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);  // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);  // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);  // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1 and 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2 and 3
  return v;
}

// floats to unsigned keys with the same order
__device__ __forceinline__ uint32_t f32_order_key(float f) {
  uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// ---------------------------------------------------------------- quantisation of one value
__device__ __forceinline__ int quant_i8(float x, float s) {
  float q = rintf(x / s);
  q = fminf(fmaxf(q, -128.0f), 127.0f);
  return (int)q;
}

// ---------------------------------------------------------------- grouped row-block lookup
// Row blocks of BM rows are numbered group by group (a group with c rows has ceil(c/BM) of them).
// Finds the group and the first row of block `b`; returns false when b is past the last block.
// offsets[0..G] is the exclusive prefix of the regular groups; an extra group of extra_rows rows
// follows at offsets[G].  Every lane of the calling wave gets the same answer.
struct RowBlock {
  int group;
  int row0;
  int nrows;
};
// Row blocks of BM rows, group by group (the extra group last).  The scan is done once per
// wavefront (every lane takes part); any number of lookups can follow.
struct RowBlockScan {
  int start, c, incl, nb;  // Gt <= 64: this lane's group (first row, rows, inclusive block prefix, blocks)
  int total;               // row blocks over all groups
  bool small;              // one group per lane
};
__device__ __forceinline__ RowBlockScan row_blocks_scan(const int32_t* __restrict__ offsets, int G, int extra_rows, int BM) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int Gt = G + (extra_rows > 0 ? 1 : 0);
  RowBlockScan s{};
  s.small = Gt <= WAVE;
  if (s.small) {
    // one group per lane: everything a lookup needs stays in registers after one round of loads
    if (lane < Gt) {
      s.start = offsets[lane < G ? lane : G];
      s.c = (lane < G) ? (offsets[lane + 1] - s.start) : extra_rows;
    }
    s.nb = (s.c + BM - 1) / BM;
    s.incl = wave_incl_scan_dpp_i(s.nb);
    s.total = __builtin_amdgcn_readlane(s.incl, WAVE - 1);
    return s;
  }
  const int per = (Gt + WAVE - 1) / WAVE;
  const int g0 = lane * per;
  int mine = 0;
  for (int j = 0; j < per; ++j) {
    int g = g0 + j;
    if (g < Gt) {
      int c = (g < G) ? (offsets[g + 1] - offsets[g]) : extra_rows;
      mine += (c + BM - 1) / BM;
    }
  }
  s.nb = mine;
  s.incl = wave_incl_scan_dpp_i(mine);
  s.total = __builtin_amdgcn_readlane(s.incl, WAVE - 1);
  return s;
}
__device__ __forceinline__ bool row_blocks_find(const RowBlockScan& s, const int32_t* __restrict__ offsets, int G,
                                                int extra_rows, int BM, int b, RowBlock& rb) {
  if (b < 0 || b >= s.total) return false;
  const int lane = threadIdx.x & (WAVE - 1);
  const int excl = s.incl - s.nb;
  const uint64_t owner_mask = __ballot(b >= excl && b < s.incl);
  const int owner = __ffsll((unsigned long long)owner_mask) - 1;
  if (s.small) {
    const int o_start = __builtin_amdgcn_readlane(s.start, owner);
    const int o_c = __builtin_amdgcn_readlane(s.c, owner);
    const int o_excl = __builtin_amdgcn_readlane(excl, owner);
    rb.group = owner;
    rb.row0 = o_start + (b - o_excl) * BM;
    rb.nrows = min(BM, o_c - (b - o_excl) * BM);
    return true;
  }
  const int Gt = G + (extra_rows > 0 ? 1 : 0);
  const int per = (Gt + WAVE - 1) / WAVE;
  const int g0 = lane * per;
  int grp = -1, row0 = 0, nrows = 0;
  if (lane == owner) {
    int acc = excl;
    for (int j = 0; j < per; ++j) {
      int g = g0 + j;
      if (g >= Gt) break;
      int start = offsets[g < G ? g : G];
      int c = (g < G) ? (offsets[g + 1] - start) : extra_rows;
      int nb = (c + BM - 1) / BM;
      if (b < acc + nb) {
        grp = g;
        row0 = start + (b - acc) * BM;
        nrows = min(BM, c - (b - acc) * BM);
        break;
      }
      acc += nb;
    }
  }
  rb.group = __builtin_amdgcn_readlane(grp, owner);
  rb.row0 = __builtin_amdgcn_readlane(row0, owner);
  rb.nrows = __builtin_amdgcn_readlane(nrows, owner);
  return true;
}
// The same row blocks numbered by weight: first the heavy blocks of all groups in group order (full blocks, and
// last blocks that are not light, see last_block_is_light), then the light last blocks of the groups that have one.  A
// kernel whose blocks cost the same from light_max + 1 rows on can then deal out equal work first and keep the
// cheap blocks for the end.
struct RowBlockKinds {
  int start, c;              // Gt <= 64: this lane's group (first row, rows)
  int incl_h, nh;            // inclusive prefix and count of the heavy blocks of this lane's group(s)
  int incl_l, nl;            // same for the light blocks
  int total_h, total_l;
  bool small;
};
using omni_host::heavy_blocks;
using omni_host::last_block_is_light;
using omni_host::light_blocks;
__device__ __forceinline__ RowBlockKinds row_block_kinds_scan(const int32_t* __restrict__ offsets, int G, int extra_rows,
                                                              int BM, int light_max) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int Gt = G + (extra_rows > 0 ? 1 : 0);
  RowBlockKinds s{};
  s.small = Gt <= WAVE;
  if (s.small) {
    if (lane < Gt) {
      s.start = offsets[lane < G ? lane : G];
      s.c = (lane < G) ? (offsets[lane + 1] - s.start) : extra_rows;
    }
    s.nh = heavy_blocks(s.c, BM, light_max);
    s.nl = light_blocks(s.c, BM, light_max);
  } else {
    const int per = (Gt + WAVE - 1) / WAVE;
    for (int j = 0; j < per; ++j) {
      const int g = lane * per + j;
      if (g < Gt) {
        const int c = (g < G) ? (offsets[g + 1] - offsets[g]) : extra_rows;
        s.nh += heavy_blocks(c, BM, light_max);
        s.nl += light_blocks(c, BM, light_max);
      }
    }
  }
  s.incl_h = wave_incl_scan_dpp_i(s.nh);
  s.incl_l = wave_incl_scan_dpp_i(s.nl);
  s.total_h = __builtin_amdgcn_readlane(s.incl_h, WAVE - 1);
  s.total_l = __builtin_amdgcn_readlane(s.incl_l, WAVE - 1);
  return s;
}
// heavy block b (light == false) or light block b; b must be in range
__device__ __forceinline__ void row_block_kinds_find(const RowBlockKinds& s, const int32_t* __restrict__ offsets, int G,
                                                     int extra_rows, int BM, int light_max, bool light, int b, RowBlock& rb) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int incl = light ? s.incl_l : s.incl_h;
  const int excl = incl - (light ? s.nl : s.nh);
  const uint64_t owner_mask = __ballot(b >= excl && b < incl);
  const int owner = __ffsll((unsigned long long)owner_mask) - 1;
  if (s.small) {
    const int o_start = __builtin_amdgcn_readlane(s.start, owner);
    const int o_c = __builtin_amdgcn_readlane(s.c, owner);
    const int o_excl = __builtin_amdgcn_readlane(excl, owner);
    rb.group = owner;
    const int first = light ? o_c / BM * BM : (b - o_excl) * BM;  // row of the group the block starts at
    rb.row0 = o_start + first;
    rb.nrows = min(BM, o_c - first);
    return;
  }
  const int Gt = G + (extra_rows > 0 ? 1 : 0);
  const int per = (Gt + WAVE - 1) / WAVE;
  int grp = -1, row0 = 0, nrows = 0;
  if (lane == owner) {
    int acc = excl;
    for (int j = 0; j < per; ++j) {
      const int g = lane * per + j;
      if (g >= Gt) break;
      const int start = offsets[g < G ? g : G];
      const int c = (g < G) ? (offsets[g + 1] - start) : extra_rows;
      const int n = light ? light_blocks(c, BM, light_max) : heavy_blocks(c, BM, light_max);
      if (b < acc + n) {
        const int first = light ? c / BM * BM : (b - acc) * BM;
        grp = g;
        row0 = start + first;
        nrows = min(BM, c - first);
        break;
      }
      acc += n;
    }
  }
  rb.group = __builtin_amdgcn_readlane(grp, owner);
  rb.row0 = __builtin_amdgcn_readlane(row0, owner);
  rb.nrows = __builtin_amdgcn_readlane(nrows, owner);
}
__device__ __forceinline__ bool find_row_block(const int32_t* __restrict__ offsets, int G, int extra_rows, int BM,
                                               int b, RowBlock& rb) {
  const RowBlockScan s = row_blocks_scan(offsets, G, extra_rows, BM);
  return row_blocks_find(s, offsets, G, extra_rows, BM, b, rb);
}
