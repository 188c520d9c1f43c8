// Weighted un-permute (finalize routing), the library's error state and the whole-layer entry.
//
// combine: grid (token, column chunk of 1024).  The block first lists the token's kept
// assignments (slot, weight) in LDS, ordered by slot or by k as asked, then every thread
// accumulates four consecutive columns in fp32, one multiply and one add per row, in that order.
#include "common.h"

#include <string.h>

#include <mutex>

// ---------------------------------------------------------------- error state
static thread_local char g_err[512] = "";
void omni_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}
extern "C" const char* omni_moe_last_error(void) { return g_err; }
extern "C" int omni_moe_abi_version(void) { return 7; }

namespace {

constexpr int KMAX = 64;

struct CombineArgs {
  const void* rows;
  int rows_dtype;
  const float* topk_w;
  const int32_t* src_to_dst;
  int idx_mode, order, T, K, H;
  const uint16_t* init;
  const void* post_add;
  const int32_t* post_add_row0;
  // the added rows are bf16 rows of H values packed from row *post_add_row0 of an fp32 row buffer on (what
  // GEMM2 writes for the extra group when the whole-layer entry asks for it); rows_dtype is fp32 then
  int post_add_bf16;
  uint16_t* out;
};

// VEC columns of one row as floats: 16 bytes per lane (4 fp32 or 8 bf16), element by element at a ragged end.
// STREAM: the row is read once and not again (expert rows), so it need not stay in the caches
template <int DT, bool STREAM, int VEC>
__device__ __forceinline__ void load_vec(const void* base, size_t row, int H, int c, int ncol, bool vec, float* v) {
  if constexpr (DT == OMNI_DT_F32) {
    static_assert(VEC == 4, "16 bytes of fp32");
    const float* p = (const float*)base + row * H + c;
    if (ncol == VEC && vec) {
      v4f t = STREAM ? __builtin_nontemporal_load((const v4f*)p) : *(const v4f*)p;
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = t[j];
    } else {
      for (int j = 0; j < VEC; ++j) v[j] = j < ncol ? p[j] : 0.0f;
    }
  } else {
    static_assert(VEC == 8, "16 bytes of bf16");
    const uint16_t* p = (const uint16_t*)base + row * H + c;
    if (ncol == VEC && vec) {
      v4i t = STREAM ? __builtin_nontemporal_load((const v4i*)p) : *(const v4i*)p;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[2 * j] = bf16_to_f32((uint16_t)((uint32_t)t[j] & 0xffffu));
        v[2 * j + 1] = bf16_to_f32((uint16_t)((uint32_t)t[j] >> 16));
      }
    } else {
      for (int j = 0; j < VEC; ++j) v[j] = j < ncol ? bf16_to_f32(p[j]) : 0.0f;
    }
  }
}

template <int DT>
__global__ __launch_bounds__(256) void combine_kernel(CombineArgs a) {
  constexpr int VEC = (DT == OMNI_DT_F32) ? 4 : 8;   // columns per thread and step
  __shared__ int s_slot[KMAX], s_raw[KMAX];
  __shared__ float s_w[KMAX];
  const int n = blockIdx.x;
  // thread k fetches assignment k; its place in the list is the number of kept assignments that
  // come before it (lower slot, or lower k, as the order asks)
  int slot = -1;
  float wv = 0.0f;
  if (threadIdx.x < a.K) {
    const int k = threadIdx.x;
    const int idx = (a.idx_mode == OMNI_IDX_TOKEN_MAJOR) ? n * a.K + k : k * a.T + n;
    slot = a.src_to_dst[idx];
    wv = a.topk_w[(size_t)n * a.K + k];
    s_raw[k] = slot;
  }
  __syncthreads();
  int cnt = 0;
  {
    int pos = 0;
    for (int j = 0; j < a.K; ++j) {
      const int sj = s_raw[j];
      if (sj < 0) continue;
      ++cnt;
      if (a.order == OMNI_ORDER_SLOT ? (sj < slot) : (j < (int)threadIdx.x)) ++pos;
    }
    if (threadIdx.x < a.K && slot >= 0) {
      s_slot[pos] = slot;
      s_w[pos] = wv;
    }
  }
  __syncthreads();
  const size_t post_row = (size_t)n + ((a.post_add && a.post_add_row0) ? (size_t)*a.post_add_row0 : 0);
  const bool vec = (a.H % VEC) == 0;  // every row then starts on a 16-byte boundary
  // a block walks the column chunks blockIdx.y, blockIdx.y + gridDim.y, ... of its token
  for (int c = (blockIdx.y * 256 + threadIdx.x) * VEC; c < a.H; c += gridDim.y * 256 * VEC) {
    const int ncol = min(VEC, a.H - c);
    float acc[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc[i] = 0.0f;
    if (a.init) {
      const uint16_t* ip = a.init + (size_t)n * a.H + c;
      for (int j = 0; j < ncol; ++j) acc[j] = bf16_to_f32(ip[j]);
    }
    // the row added after the rounding is requested with the first batch
    float pv[VEC];
    if (a.post_add) {
      if (DT == OMNI_DT_F32 && a.post_add_bf16) {
        // bf16 row n of the packed rows begins 2 * row0 + n rows of H bf16 values into the buffer
        const uint16_t* p = (const uint16_t*)a.post_add + (post_row + (size_t)*a.post_add_row0) * a.H + c;
        if (ncol == VEC && vec) {
          const v2i t = *(const v2i*)p;
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            pv[2 * j] = bf16_to_f32((uint16_t)((uint32_t)t[j] & 0xffffu));
            pv[2 * j + 1] = bf16_to_f32((uint16_t)((uint32_t)t[j] >> 16));
          }
        } else {
          for (int j = 0; j < VEC; ++j) pv[j] = j < ncol ? bf16_to_f32(p[j]) : 0.0f;
        }
      } else {
        load_vec<DT, false, VEC>(a.post_add, post_row, a.H, c, ncol, vec, pv);
      }
    }
    // eight rows are requested together, then added in list order (one multiply, one add per row)
    for (int j0 = 0; j0 < cnt; j0 += 8) {
      float v[8][VEC];
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (j0 + u < cnt) load_vec<DT, true, VEC>(a.rows, (size_t)s_slot[j0 + u], a.H, c, ncol, vec, v[u]);
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        if (j0 + u < cnt) {
          const float wu = s_w[j0 + u];
#pragma unroll
          for (int i = 0; i < VEC; ++i) {
            float prod = wu * v[u][i];
            acc[i] = acc[i] + prod;
          }
        }
      }
    }
    uint16_t o[VEC];
#pragma unroll
    for (int i = 0; i < VEC; ++i) o[i] = f32_to_bf16(acc[i]);
    if (a.post_add) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) o[i] = f32_to_bf16(bf16_to_f32(o[i]) + round_bf16(pv[i]));
    }
    uint16_t* op = a.out + (size_t)n * a.H + c;
    if (ncol == VEC && vec) {
      if constexpr (VEC == 4) {
        v2i t = {(int)((uint32_t)o[0] | ((uint32_t)o[1] << 16)), (int)((uint32_t)o[2] | ((uint32_t)o[3] << 16))};
        *(v2i*)op = t;
      } else {
        v4i t;
#pragma unroll
        for (int j = 0; j < 4; ++j) t[j] = (int)((uint32_t)o[2 * j] | ((uint32_t)o[2 * j + 1] << 16));
        *(v4i*)op = t;
      }
    } else {
      for (int j = 0; j < ncol; ++j) op[j] = o[j];
    }
  }
}


}  // namespace

namespace {
int combine_impl(const void* rows, int rows_dtype, const float* topk_w, const int32_t* src_to_dst, int idx_mode,
                 int order, int T, int K, int H, const void* init_bf16, const void* post_add,
                 const int32_t* post_add_row0, int post_add_bf16, void* out_bf16, void* stream) {
  if (T < 0 || K <= 0 || H <= 0) OMNI_FAIL(OMNI_E_INVALID, "combine: bad sizes T=%d K=%d H=%d", T, K, H);
  if (T == 0) return OMNI_OK;
  if (K > KMAX) OMNI_FAIL(OMNI_E_UNSUPPORTED, "combine: K=%d > %d", K, KMAX);
  if (!rows || !topk_w || !src_to_dst || !out_bf16) OMNI_FAIL(OMNI_E_INVALID, "combine: null pointer");
  if (rows_dtype != OMNI_DT_F32 && rows_dtype != OMNI_DT_BF16) OMNI_FAIL(OMNI_E_INVALID, "combine: rows_dtype %d", rows_dtype);
  if (H % 4 != 0) OMNI_FAIL(OMNI_E_UNSUPPORTED, "combine: H=%d must be a multiple of 4", H);
  // a thread moves 16 bytes of a row at a time: 4 fp32 or 8 bf16 columns in, as many bf16 columns out
  const uintptr_t out_align = (rows_dtype == OMNI_DT_BF16) ? 16 : 8;
  if (((uintptr_t)rows % 16) || ((uintptr_t)out_bf16 % out_align) || ((uintptr_t)post_add % 16))
    OMNI_FAIL(OMNI_E_INVALID, "combine: misaligned pointer");
  if (post_add_bf16 && (rows_dtype != OMNI_DT_F32 || !post_add || !post_add_row0))
    OMNI_FAIL(OMNI_E_INVALID, "combine: packed bf16 rows need fp32 rows and the extra group's first row");
  CombineArgs a{rows, rows_dtype, topk_w, src_to_dst, idx_mode, order, T, K, H, (const uint16_t*)init_bf16, post_add,
                post_add_row0, post_add_bf16, (uint16_t*)out_bf16};
  // few tokens: one block per (token, chunk of 256 x 16 bytes) for parallelism; many tokens: one block
  // per token walks all chunks, so that a row's bytes are requested close together in time
  const int chunk_cols = 256 * ((rows_dtype == OMNI_DT_BF16) ? 8 : 4);
  const unsigned chunks = (unsigned)((H + chunk_cols - 1) / chunk_cols);
  dim3 grid((unsigned)T, T >= 2048 ? 1u : chunks), block(256);
  hipStream_t st = (hipStream_t)stream;
  if (rows_dtype == OMNI_DT_F32) hipLaunchKernelGGL(combine_kernel<OMNI_DT_F32>, grid, block, 0, st, a);
  else hipLaunchKernelGGL(combine_kernel<OMNI_DT_BF16>, grid, block, 0, st, a);
  OMNI_CHECK_LAUNCH("combine");
  return OMNI_OK;
}
}  // namespace

extern "C" int omni_moe_combine(const void* rows, int rows_dtype, const float* topk_w, const int32_t* src_to_dst,
                                int idx_mode, int order, int T, int K, int H, const void* init_bf16,
                                const void* post_add, const int32_t* post_add_row0, void* out_bf16, void* stream) {
  return combine_impl(rows, rows_dtype, topk_w, src_to_dst, idx_mode, order, T, K, H, init_bf16, post_add, post_add_row0,
                      0, out_bf16, stream);
}

// ---------------------------------------------------------------- whole layer
// byte offsets of the parts of the caller's workspace: omni_host::layer_layout (host_logic.h)
using omni_host::LayerWs;
using omni_host::layer_layout;

extern "C" size_t omni_moe_w8a8_layer_workspace_bytes(int T, int K, int n_local, int H, int I, int with_shared,
                                                      int rows_dtype) {
  if (T < 0 || K <= 0 || n_local <= 0 || H <= 0 || I <= 0) return 0;
  if (rows_dtype != OMNI_DT_F32 && rows_dtype != OMNI_DT_BF16) return 0;
  return layer_layout(T, K, n_local, H, I, with_shared, rows_dtype).total;
}

namespace {
// The layer.  With `route` the routing is part of the call: topk_w and topk_ids are route's outputs, written before
// anything reads them (by the first launch when the call is small enough for the kernel that routes, quantises
// and sorts at once, by a routing launch of its own otherwise).
int layer_impl(const void* x, int x_dtype, const float* x_scale_in, const float* topk_w, const int32_t* topk_ids,
               const OmniRouteParams* route, int T, int K, int lo, int hi, const int8_t* w13_packed,
               const float* w13_scale, const int8_t* w2_packed, const float* w2_scale, const int8_t* sh13_packed,
               const float* sh13_scale, const int8_t* sh2_packed, const float* sh2_scale, int H, int I, int rows_dtype,
               void* out_bf16, void* workspace, size_t ws_bytes, void* stream, const float* quant_scale = nullptr) {
  if (T < 0 || K <= 0 || hi <= lo || H <= 0 || I <= 0) OMNI_FAIL(OMNI_E_INVALID, "layer: bad sizes");
  if (rows_dtype != OMNI_DT_F32 && rows_dtype != OMNI_DT_BF16) OMNI_FAIL(OMNI_E_INVALID, "layer: rows_dtype %d", rows_dtype);
  if (T == 0) return OMNI_OK;
  if (!x || !topk_w || !topk_ids || !out_bf16 || !workspace) OMNI_FAIL(OMNI_E_INVALID, "layer: null pointer");
  if (x_dtype == -1 && !x_scale_in) OMNI_FAIL(OMNI_E_INVALID, "layer: int8 input without scales");
  const int G = hi - lo;
  const int with_shared = sh13_packed != nullptr;
  if (with_shared && (!sh13_scale || !sh2_packed || !sh2_scale)) OMNI_FAIL(OMNI_E_INVALID, "layer: incomplete shared expert");
  if ((uintptr_t)workspace % 256) OMNI_FAIL(OMNI_E_INVALID, "layer: workspace must be 256-byte aligned");
  LayerWs L = layer_layout(T, K, G, H, I, with_shared, rows_dtype);
  if (ws_bytes < L.total) OMNI_FAIL(OMNI_E_WORKSPACE, "layer: workspace %zu < %zu", ws_bytes, L.total);
  char* ws = (char*)workspace;
  const int8_t* xq = (const int8_t*)x;
  const float* xs = x_scale_in;
  int rc;
  int32_t* sorted_src = (int32_t*)(ws + L.sorted_src);
  int32_t* src_to_dst = (int32_t*)(ws + L.src_to_dst);
  int32_t* offsets = (int32_t*)(ws + L.offsets);
  bool sorted = false;
  const int extra = with_shared ? T : 0;
  // When both grouped GEMMs run the tile kernel, the arrival counters of their split tiles are cleared by the
  // sorting kernel below (the first kernel to run that has a single-block part), not by two launches of their own.
  int cnt_words = 0;
  size_t tail_bytes = 0;
  void* const tail = omni_tile_tail_area(T, K, G, extra, L.M_cap, H, I, ws + L.g1_ws, L.g1_bytes, &cnt_words, &tail_bytes);
  // When GEMM1 runs the streaming kernel, the same kernel clears the arrival counters of its overflow blocks instead.
  const omni_host::Plan p1 = omni_host::make_plan(1, T, K, G, extra, H, 2 * I);
  const size_t bal_at = omni_host::gemm1_stream_bal_at(p1, L.M_cap, I);
  int32_t* zero_words = (int32_t*)tail;
  int zero_n = cnt_words;
  if (!tail && bal_at != 0) {
    zero_words = (int32_t*)(ws + L.g1_ws + bal_at);
    zero_n = 2 * omni_host::STREAM_BAL_CNT_WORDS;
  }
  const bool counters_clean = zero_words != nullptr;
  bool routed = route == nullptr;
  if (route != nullptr && (x_dtype == OMNI_DT_BF16 || x_dtype == -1)) {
    // routing, quantisation (of bf16 tokens) and sort in one launch when the call is small
    const bool quantise = x_dtype == OMNI_DT_BF16;
    rc = omni_route_quant_permute_fused(route, quantise ? x : nullptr, T, H, (int8_t*)(ws + L.x_q), (float*)(ws + L.x_s), K,
                                        lo, hi, sorted_src, src_to_dst, (int32_t*)(ws + L.counts), offsets, zero_words,
                                        zero_n, stream);
    if (rc < 0) return rc;
    routed = sorted = rc == 0;
    if (sorted && quantise) {
      xq = (const int8_t*)(ws + L.x_q);
      xs = (const float*)(ws + L.x_s);
    }
  }
  if (!routed) {
    rc = omni_route_launch(route, T, K, stream);
    if (rc) return rc;
  }
  if (x_dtype != -1 && !sorted) {
    // the quantisation and the sort do not depend on each other: one launch when both are small
    rc = 1;
    if (x_dtype == OMNI_DT_BF16)
      rc = omni_quant_permute_fused(x, T, H, (int8_t*)(ws + L.x_q), (float*)(ws + L.x_s), topk_ids, K, lo, hi,
                                    OMNI_IDX_TOKEN_MAJOR, sorted_src, src_to_dst, (int32_t*)(ws + L.counts), offsets,
                                    zero_words, zero_n, stream);
    if (rc < 0) return rc;
    sorted = rc == 0;
    if (!sorted) {
      rc = omni_dynamic_quant(x, x_dtype, T, H, H, (int8_t*)(ws + L.x_q), (float*)(ws + L.x_s), stream);
      if (rc) return rc;
    }
    xq = (const int8_t*)(ws + L.x_q);
    xs = (const float*)(ws + L.x_s);
  }
  if (!sorted) {
    rc = omni_moe_permute_clearing(topk_ids, T, K, lo, hi, OMNI_IDX_TOKEN_MAJOR, sorted_src, src_to_dst,
                                   (int32_t*)(ws + L.counts), offsets, ws + L.perm_ws, L.perm_bytes, zero_words,
                                   zero_n, stream);
    if (rc) return rc;
  }
  rc = omni_gemm1_swiglu_quant_impl(xq, xs, sorted_src, OMNI_IDX_TOKEN_MAJOR, T, K, w13_packed, w13_scale, sh13_packed,
                                    sh13_scale, extra, offsets, G, H, I, L.M_cap, 0, quant_scale, (int8_t*)(ws + L.h_q),
                                    (float*)(ws + L.h_s), nullptr, ws + L.g1_ws, L.g1_bytes, counters_clean, stream);
  if (rc) return rc;
  // The weighted sum rounds the shared expert's row to bf16 before it adds it to the rounded sum of the routed rows,
  // so with fp32 rows GEMM2 writes that group's rows as bf16 straight away (into the first half of the space their
  // fp32 form would take): the same bits, half the bytes written and read.  Only where GEMM2 runs the tile kernel,
  // whose epilogue stores whole lines either way; the streaming kernel stores an element per lane, and 2-byte
  // elements cost its few shared rows more than their bytes save (measured at 64 tokens: +0.5 us).
  const bool shared_rows_bf16 = with_shared && L.rows_dtype == OMNI_DT_F32 && tail != nullptr;
  // GEMM1's scratch is free again once its row quantiser has run: GEMM2 takes it over (with cleared counters: the
  // split-tile scratch of GEMM1, whose counter words for GEMM2 nobody has touched since the sorting kernel)
  rc = omni_gemm2_dequant_impl((const int8_t*)(ws + L.h_q), (const float*)(ws + L.h_s), w2_packed, w2_scale, sh2_packed,
                               sh2_scale, extra, offsets, G, H, I, L.M_cap, L.rows_dtype, ws + L.rows, nullptr,
                               tail ? tail : (void*)(ws + L.g1_ws), tail ? tail_bytes : L.g1_bytes, tail != nullptr,
                               shared_rows_bf16, stream);
  if (rc) return rc;
  return combine_impl(ws + L.rows, L.rows_dtype, topk_w, src_to_dst, OMNI_IDX_TOKEN_MAJOR, OMNI_ORDER_SLOT, T, K, H,
                      nullptr, with_shared ? ws + L.rows : nullptr, with_shared ? offsets + G : nullptr,
                      shared_rows_bf16 ? 1 : 0, out_bf16, stream);
}
}  // namespace

extern "C" int omni_moe_w8a8_layer(const void* x, int x_dtype, const float* x_scale_in, const float* topk_w,
                                   const int32_t* topk_ids, int T, int K, int lo, int hi, const int8_t* w13_packed,
                                   const float* w13_scale, const int8_t* w2_packed, const float* w2_scale,
                                   const int8_t* sh13_packed, const float* sh13_scale, const int8_t* sh2_packed,
                                   const float* sh2_scale, const float* quant_scale, int H, int I, int rows_dtype,
                                   void* out_bf16, void* workspace, size_t ws_bytes, void* stream) {
  return layer_impl(x, x_dtype, x_scale_in, topk_w, topk_ids, nullptr, T, K, lo, hi, w13_packed, w13_scale, w2_packed,
                    w2_scale, sh13_packed, sh13_scale, sh2_packed, sh2_scale, H, I, rows_dtype, out_bf16, workspace,
                    ws_bytes, stream, quant_scale);
}

extern "C" int omni_moe_w8a8_layer_routed(const void* x, int x_dtype, const float* x_scale_in, const float* logits,
                                          const float* bias, int E, int n_group, int topk_group, int score_fn,
                                          int group_mode, int masked_fill_zero, int weight_from_c, int renorm,
                                          float scale, float eps, float* topk_w, int32_t* topk_ids, int T, int K, int lo,
                                          int hi, const int8_t* w13_packed, const float* w13_scale,
                                          const int8_t* w2_packed, const float* w2_scale, const int8_t* sh13_packed,
                                          const float* sh13_scale, const int8_t* sh2_packed, const float* sh2_scale,
                                          int H, int I, int rows_dtype, void* out_bf16, void* workspace, size_t ws_bytes,
                                          void* stream) {
  if (T < 0 || E <= 0 || K <= 0) OMNI_FAIL(OMNI_E_INVALID, "layer_routed: bad sizes T=%d E=%d K=%d", T, E, K);
  if (T == 0) return OMNI_OK;
  if (!logits || !topk_w || !topk_ids) OMNI_FAIL(OMNI_E_INVALID, "layer_routed: null pointer");
  const int rc = omni_route_check("layer_routed", T, E, n_group, topk_group, K, score_fn);
  if (rc) return rc;
  const OmniRouteParams rp{logits, bias, E, n_group, topk_group, score_fn, group_mode, masked_fill_zero, weight_from_c,
                           renorm, scale, eps, topk_w, topk_ids};
  return layer_impl(x, x_dtype, x_scale_in, topk_w, topk_ids, &rp, T, K, lo, hi, w13_packed, w13_scale, w2_packed,
                    w2_scale, sh13_packed, sh13_scale, sh2_packed, sh2_scale, H, I, rows_dtype, out_bf16, workspace,
                    ws_bytes, stream);
}

// ---------------------------------------------------------------- the whole block: gate, router, layer
extern "C" size_t omni_moe_w8a8_block_workspace_bytes(int T, int K, int n_local, int H, int I, int E, int with_shared,
                                                      int rows_dtype) {
  const size_t layer = omni_moe_w8a8_layer_workspace_bytes(T, K, n_local, H, I, with_shared, rows_dtype);
  const size_t gate = omni_moe_gate_route_workspace_bytes(T, H, E);
  if (layer == 0 || (gate == 0 && T > 0)) return 0;
  return align256(layer) + gate;
}

extern "C" int omni_moe_w8a8_block(const void* x, int x_dtype, const int8_t* x_q, const float* x_scale, const void* gate_w,
                                   int gate_w_dtype, const float* bias, int E, int n_group, int topk_group, int score_fn,
                                   int group_mode, int masked_fill_zero, int weight_from_c, int renorm, float scale,
                                   float eps, int round_logits_bf16, float* topk_w, int32_t* topk_ids, int T, int K, int lo,
                                   int hi, const int8_t* w13_packed, const float* w13_scale, const int8_t* w2_packed,
                                   const float* w2_scale, const int8_t* sh13_packed, const float* sh13_scale,
                                   const int8_t* sh2_packed, const float* sh2_scale, int H, int I, int rows_dtype,
                                   void* out_bf16, void* workspace, size_t ws_bytes, void* stream) {
  if (T < 0 || E <= 0 || K <= 0 || H <= 0 || I <= 0 || hi <= lo) OMNI_FAIL(OMNI_E_INVALID, "block: bad sizes T=%d E=%d K=%d", T, E, K);
  if (T == 0) return OMNI_OK;
  if (!x || !gate_w || !topk_w || !topk_ids || !workspace) OMNI_FAIL(OMNI_E_INVALID, "block: null pointer");
  if ((x_q == nullptr) != (x_scale == nullptr)) OMNI_FAIL(OMNI_E_INVALID, "block: quantised tokens and their scales come together");
  if (x_q == nullptr && x_dtype != OMNI_DT_BF16) OMNI_FAIL(OMNI_E_UNSUPPORTED, "block: tokens that are not quantised yet must be bf16");
  if (rows_dtype != OMNI_DT_F32 && rows_dtype != OMNI_DT_BF16) OMNI_FAIL(OMNI_E_INVALID, "block: rows_dtype %d", rows_dtype);
  int rc = omni_route_check("block", T, E, n_group, topk_group, K, score_fn);
  if (rc) return rc;
  const int with_shared = sh13_packed != nullptr;
  const size_t layer_bytes = align256(omni_moe_w8a8_layer_workspace_bytes(T, K, hi - lo, H, I, with_shared, rows_dtype));
  const size_t gate_bytes = omni_moe_gate_route_workspace_bytes(T, H, E);
  if (gate_bytes == 0) OMNI_FAIL(OMNI_E_UNSUPPORTED, "block: the gate projection needs H %% 128 == 0 (H=%d)", H);
  if (ws_bytes < layer_bytes + gate_bytes) OMNI_FAIL(OMNI_E_WORKSPACE, "block: workspace %zu < %zu", ws_bytes, layer_bytes + gate_bytes);
  if ((uintptr_t)workspace % 256) OMNI_FAIL(OMNI_E_INVALID, "block: workspace must be 256-byte aligned");
  char* gate_ws = (char*)workspace + layer_bytes;
  OmniRouteParams rp{nullptr, bias, E, n_group, topk_group, score_fn, group_mode, masked_fill_zero, weight_from_c, renorm,
                     scale, eps, topk_w, topk_ids};
  rc = omni_gate_partials(x, x_dtype, gate_w, gate_w_dtype, T, H, E, gate_ws, gate_bytes, &rp.n_parts, &rp.group_len, stream);
  if (rc) return rc;
  rp.partials = (const float*)gate_ws;
  rp.round_logits_bf16 = round_logits_bf16;
  return layer_impl(x_q ? (const void*)x_q : x, x_q ? -1 : x_dtype, x_scale, topk_w, topk_ids, &rp, T, K, lo, hi, w13_packed,
                    w13_scale, w2_packed, w2_scale, sh13_packed, sh13_scale, sh2_packed, sh2_scale, H, I, rows_dtype, out_bf16,
                    workspace, layer_bytes, stream);
}

// ---------------------------------------------------------------- whole layer on the library's own scratch
// The same layer for callers that must not allocate and have no workspace to pass (code under HIP graph
// capture, tight serving loops).  The scratch is a file-scope device array: every GPU the library runs on
// holds one copy of it, at an address of its own, until the process ends.  The array's name is only a
// host-side handle; the device address is asked for once per device and used from then on.
namespace {
static __device__ __align__(256) unsigned char scratch[OMNI_STATIC_SCRATCH_BYTES];
constexpr int MAX_DEVICES = 64;
void* g_scratch_ptr[MAX_DEVICES];
std::mutex g_scratch_mutex;

// device address of this device's copy of `scratch` (resolved on the first call with that device current)
int static_scratch_ptr(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MAX_DEVICES)
    OMNI_FAIL(OMNI_E_LAUNCH, "layer_static: no current device (or device index >= %d)", MAX_DEVICES);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr)
      OMNI_FAIL(OMNI_E_LAUNCH, "layer_static: hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return OMNI_OK;
}
}  // namespace

extern "C" int omni_moe_w8a8_layer_static(const void* x, int x_dtype, const float* x_scale_in, const float* topk_w,
                                          const int32_t* topk_ids, int T, int K, int lo, int hi,
                                          const int8_t* w13_packed, const float* w13_scale, const int8_t* w2_packed,
                                          const float* w2_scale, const int8_t* sh13_packed, const float* sh13_scale,
                                          const int8_t* sh2_packed, const float* sh2_scale, int H, int I,
                                          int rows_dtype, void* out_bf16, void* stream) {
  if (T < 0 || K <= 0 || hi <= lo || H <= 0 || I <= 0) OMNI_FAIL(OMNI_E_INVALID, "layer_static: bad sizes");
  if (rows_dtype != OMNI_DT_F32 && rows_dtype != OMNI_DT_BF16) OMNI_FAIL(OMNI_E_INVALID, "layer_static: rows_dtype %d", rows_dtype);
  const size_t need = layer_layout(T, K, hi - lo, H, I, sh13_packed != nullptr, rows_dtype).total;
  if (need > (size_t)OMNI_STATIC_SCRATCH_BYTES)
    OMNI_FAIL(OMNI_E_WORKSPACE,
              "layer_static: this call needs %zu bytes of scratch, the library's static scratch holds %zu; "
              "use omni_moe_w8a8_layer with a workspace for calls of this size",
              need, (size_t)OMNI_STATIC_SCRATCH_BYTES);
  void* ptr = nullptr;
  const int rc = static_scratch_ptr(&ptr);
  if (rc) return rc;
  // nothing in the scratch has to start at zero except the arrival counters of split tiles, and those are cleared
  // by a kernel of the call itself (the sorting kernel, or a fill kernel in front of the tile launch); everything
  // else is written before it is read
  return omni_moe_w8a8_layer(x, x_dtype, x_scale_in, topk_w, topk_ids, T, K, lo, hi, w13_packed, w13_scale, w2_packed,
                             w2_scale, sh13_packed, sh13_scale, sh2_packed, sh2_scale, nullptr, H, I, rows_dtype, out_bf16,
                             ptr, (size_t)OMNI_STATIC_SCRATCH_BYTES, stream);
}
