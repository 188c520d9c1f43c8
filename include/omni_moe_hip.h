/*
 * omni_moe_hip.h -- C ABI of libomni_moe_hip.so: the gfx950 (MI355X) operator set
 * behind omni-infer's W8A8 dynamic-quant fused-MoE layer.
 *
 * The reference reaches its device arithmetic through `torch_npu.npu_*` Python
 * operators (closed CANN kernels).  Each entry point below replaces one such
 * operator family; the reference call sites are cited per function (paths are
 * relative to the reference tree).  All pointers are device pointers unless
 * stated, all sizes are explicit, `stream` is a hipStream_t passed as void*.
 *
 * Conventions
 *  - every function returns 0 on success and a negative OMNI_E_* code on a
 *    rejected argument; omni_moe_last_error() then describes it (thread local);
 *  - nothing here allocates device memory, synchronises the device or copies to
 *    the host: all work is enqueued on `stream`, data dependent sizes (rows per
 *    expert) stay in device memory, so a call sequence can be captured in a HIP
 *    graph;
 *  - the library keeps no results between calls.  It does hold two static device
 *    arrays on every GPU it runs on, from the first call that needs them until the
 *    process ends: 16 KiB of arrival counters, zero between launches (see
 *    omni_moe_w8a8_layer_routed), and the 64 MiB scratch of
 *    omni_moe_w8a8_layer_static (resident whether that entry is used or not);
 *  - measurement helpers (kernel names, hardware-rate probes, the tuning re-read)
 *    are declared in omni_moe_diag.h, not here.
 *
 * Packed weight layout ("frag16"), produced by omni_moe_pack_weight
 *  A logical matrix B[Kdim][N] (Kdim = reduction dim, N = output channels) is
 *  stored as tiles of 16 output channels x 64 reduction elements, 1024 bytes each:
 *      offset(k, n) = (((n/16) * (Kdim/64) + k/64) * 64 + (n%16) + 16*((k%64)/16)) * 16 + k%16
 *  so that lane l of a wavefront reads its 16-byte operand of
 *  v_mfma_i32_16x16x64_i8 at tile_base + 16*l, and a 16-channel strip is
 *  contiguous along k.  Requires Kdim % 64 == 0 and N % 16 == 0.
 */
#ifndef OMNI_MOE_HIP_H
#define OMNI_MOE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define OMNI_OK 0
#define OMNI_E_INVALID (-1)      /* null pointer, negative size, inconsistent arguments */
#define OMNI_E_UNSUPPORTED (-2)  /* shape outside what the kernels are built for */
#define OMNI_E_WORKSPACE (-3)    /* workspace too small */
#define OMNI_E_LAUNCH (-4)       /* the HIP runtime refused a launch */

/* dtype codes of activations / row buffers */
#define OMNI_DT_BF16 0
#define OMNI_DT_F32 1
#define OMNI_DT_F16 2

/* omni_moe_route: score_fn */
#define OMNI_SCORE_SOFTMAX 0
#define OMNI_SCORE_SIGMOID 1
/* omni_moe_route: group_mode */
#define OMNI_GROUP_MAX 0
#define OMNI_GROUP_TOP2SUM 1

/* gemm flags */
#define OMNI_GEMM1_BF16_INTERMEDIATE 1 /* round the dequantised gate/up and the SwiGLU product to bf16
                                          (numerics of the non-EP pipeline, compressed_tensors_moe.py:242-247) */
#define OMNI_GEMM1_NO_REQUANT 4   /* stop after the GEMM kernel: its result (int32 accumulators or fp32 y)
                                     stays in the workspace, h_q / h_scale are not written.  The call is then
                                     exactly one kernel launch, which is how the benchmark times that kernel
                                     alone. */
#define OMNI_GEMM1_WS_ZEROED 8    /* the caller has filled the workspace with zeros once and nothing but calls of this
                                     entry with this flag and the same sizes have written to it since: the entry then
                                     skips the launch that clears its arrival counters (it leaves them at zero) */
/* combine: how src_to_dst is indexed */
#define OMNI_IDX_TOKEN_MAJOR 0 /* n*K + k  (npu_moe_init_routing_v2 row_idx_type=1; finalize drop_pad_mode=2) */
#define OMNI_IDX_K_MAJOR 1     /* k*T + n  (npu_moe_init_routing; finalize drop_pad_mode=0) */
/* combine: order in which a token's rows are added */
#define OMNI_ORDER_SLOT 0 /* ascending sorted slot  (npu_grouped_matmul_finalize_routing) */
#define OMNI_ORDER_K 1    /* ascending k            (npu_moe_finalize_routing) */

/* Last error message of the calling thread ("" if none). */
const char* omni_moe_last_error(void);
/* ABI version of this header (bumped on incompatible change). */
int omni_moe_abi_version(void);

/*
 * Router.  Replaces torch_npu.npu_moe_gating_top_k
 * (omni/models/common/layers/moe/fused_moe/layer.py:341-351), the torch
 * grouped_topk (omni/models/common/layers/moe/fused_moe/fused_moe.py:38-84) and
 * torch_npu.npu_moe_gating_top_k_softmax (fused_moe.py:29).
 *   logits [T,E] fp32, bias [E] fp32 or NULL.
 *   score s = softmax(logits) or sigmoid(logits); c = s + bias.
 *   n_group > 1: group score = max c (GROUP_MAX) or sum of the two largest c
 *   (GROUP_TOP2SUM); the topk_group best groups are kept; other experts take part
 *   with score -inf (masked_fill_zero = 0) or 0.0 (masked_fill_zero = 1).
 *   top-K by c, descending, ties to the lower id.
 *   weight = s[id] (weight_from_c = 0) or the selection score (weight_from_c = 1);
 *   renorm != 0: weight /= (sum of the K weights in output order + eps);
 *   weight *= scale.
 * Outputs topk_w [T,K] fp32, topk_ids [T,K] int32.  E <= 512, K <= 64, n_group <= 64.
 */
int omni_moe_route(const float* logits, const float* bias, int T, int E, int n_group, int topk_group, int K,
                   int score_fn, int group_mode, int masked_fill_zero, int weight_from_c, int renorm, float scale,
                   float eps, float* topk_w, int32_t* topk_ids, void* stream);

/*
 * Gate projection + router in two launches.  Replaces self.gate.forward(hidden_states.float()) followed by
 * FusedMoE.select_experts (omni/models/common/layers/moe/deepseek_moe.py:147-152,253-256,329; the bf16 gate
 * of omni/models/deepseek/deepseek_v3_a2.py:607-613 with w_dtype BF16 and round_logits_bf16 = 1).
 *   x [T,H] bf16 or fp32 (x_dtype), gate_w [E,H] fp32 or bf16 (w_dtype), H % 128 == 0, E <= 512.
 *   logits[t][e] = sum_k x[t][k] * gate_w[e][k] on the fp32 matrix cores in a fixed order: the reduction is cut
 *   into slices of 128 elements, each summed as a chain of fused multiply-adds over ascending k starting from
 *   +0 (v_mfma_f32_32x32x1_2b_f32 is one fma per output element); 8 consecutive slices are added left to right
 *   into a group sum, and the group sums left to right into the logit.  The result does not depend on T.
 *   The logits are then routed exactly as omni_moe_route routes them (same arguments); they are written to
 *   logits_out when it is not NULL; K = 0 computes the logits only (topk_* may be NULL).
 *   workspace: omni_moe_gate_route_workspace_bytes(T, H, E) (partial sums), 16-byte aligned.
 */
int omni_moe_gate_route(const void* x, int x_dtype, const void* gate_w, int w_dtype, const float* bias, int T, int H,
                        int E, int n_group, int topk_group, int K, int score_fn, int group_mode, int masked_fill_zero,
                        int weight_from_c, int renorm, float scale, float eps, int round_logits_bf16, float* logits_out,
                        float* topk_w, int32_t* topk_ids, void* workspace, size_t ws_bytes, void* stream);
size_t omni_moe_gate_route_workspace_bytes(int T, int H, int E);

/*
 * Per-row dynamic int8 quantisation.  Replaces torch_npu.npu_dynamic_quant
 * (omni/models/common/layers/moe/deepseek_moe.py:247,323,612;
 * omni/quantization/compressed_tensors/compressed_tensors_moe.py:241,247;
 * fused_moe.py:668; schemes/compressed_tensors_w8a8_int8.py:97).
 *   x [rows, cols] of in_dtype with row stride ld (elements);
 *   scale[r] = max|x[r,:]| / 127; q = clamp(rint(x / scale), -128, 127); a zero row gives 0, 0.
 */
int omni_dynamic_quant(const void* x, int in_dtype, int64_t rows, int cols, int64_t ld, int8_t* q, float* scale,
                       void* stream);

/*
 * Residual add + RMSNorm (+ per-token dynamic quantisation of the result) in one pass: the producer
 * in front of the MoE block.  Replaces RMSNorm.forward (omni/models/common/layers/layernorm.py:13-32):
 * npu_add_rms_norm(x, residual, weight, eps) followed, under quant_symbol, by npu_dynamic_quant
 * (:21-25; call sites deepseek_v3.py:219-220,233-235); residual == NULL gives npu_rms_norm (:28-32).
 * x, residual, weight, residual_out, y: bf16; rows x H row-major, H % 8 == 0, H <= 8192.
 *   s = float(x) + float(residual); residual_out = bf16(s);
 *   y = bf16((s / sqrt(mean(s*s) + eps)) * weight)     (fixed summation order, see csrc/norm.hip)
 *   scale = max|y| / 127, q = rint(y / scale)           (q/scale optional, together)
 * Any of residual_out, y, q may be NULL (at least one output).  residual_out may be residual itself.
 */
int omni_add_rms_norm_quant(const void* x_bf16, const void* residual_bf16, const void* weight_bf16, int64_t rows,
                            int H, float eps, void* residual_out_bf16, void* y_bf16, int8_t* q, float* scale,
                            void* stream);

/*
 * Sort (token, k) assignments by expert.  Replaces torch_npu.npu_moe_init_routing +
 * npu_moe_compute_expert_tokens (compressed_tensors_moe.py:235-237) and
 * npu_moe_init_routing_v2 with active_expert_range (fused_moe.py:514-515, :607-618).
 *   topk_ids [T,K] int32; entries with lo <= id < hi are kept.
 *   idx_mode selects how an assignment is numbered ("source index"): n*K+k or k*T+n.
 *   Stable by expert id; inside an expert ascending n*K+k.
 *   sorted_src [T*K]: source index of every sorted slot (dropped assignments follow the kept
 *   ones, in their original order); src_to_dst [T*K]: slot of every source index, -1 if dropped;
 *   counts [hi-lo]; offsets [hi-lo+1] (exclusive prefix, offsets[hi-lo] = kept total).
 *   workspace: omni_moe_permute_workspace_bytes(T, K, hi-lo).
 */
int omni_moe_permute(const int32_t* topk_ids, int T, int K, int lo, int hi, int idx_mode, int32_t* sorted_src,
                     int32_t* src_to_dst, int32_t* counts, int32_t* offsets, void* workspace, size_t ws_bytes,
                     void* stream);
size_t omni_moe_permute_workspace_bytes(int T, int K, int n_local);

/*
 * Row offsets of the groups from their sizes: offsets[0] = 0, offsets[g+1] = offsets[g] + counts[g].  The grouped
 * GEMM entries below take offsets; the reference hands its operators the sizes themselves
 * (`group_list=expert_tokens, group_list_type=1`, fused_moe.py:531-536, :552-574, :670-685) and they add them up
 * inside.  counts: int32 or int64 (counts_are_int64), G <= 256.
 */
int omni_moe_group_offsets(const void* counts, int counts_are_int64, int G, int32_t* offsets, void* stream);

/*
 * Materialise the sorted rows (the expanded_x / dynamic_quant_scale outputs of
 * npu_moe_init_routing(_v2), fused_moe.py:514-515).  row m < offsets[n_local] is a copy of
 * source row token(sorted_src[m]); elem_bytes is the byte size of a row element.
 */
int omni_moe_gather_rows(const void* x, int elem_bytes, int H, const float* x_scale, const int32_t* sorted_src,
                         const int32_t* offsets, int n_local, int T, int K, int idx_mode, void* rows_out,
                         float* scale_out, void* stream);

/*
 * One-off weight re-layout into the frag16 format (the analogue of
 * torch_npu.npu_format_cast(w, 29), compressed_tensors_moe.py:97-99).
 *   src_layout 0: w is [G, Kdim, N] (after process_weights_after_loading's transpose,
 *   compressed_tensors_moe.py:95-96); 1: w is [G, N, Kdim] (as create_weights declares it, :44-60).
 */
int omni_moe_pack_weight(const int8_t* w, int src_layout, int G, int Kdim, int N, int8_t* packed, void* stream);

/*
 * GEMM1 + dequant + SwiGLU + per-row requant.  Replaces
 * npu_grouped_matmul(output_dtype=int32) + npu_dequant_swiglu_quant
 * (fused_moe.py:531-534, :552-561, :670-677; deepseek_moe.py:465-471; activation.py:15-27),
 * and with OMNI_GEMM1_BF16_INTERMEDIATE npu_grouped_matmul(bf16) + npu_swiglu + npu_dynamic_quant
 * (compressed_tensors_moe.py:242-247).
 *   Rows are grouped: group g owns rows [offsets[g], offsets[g+1]); an optional extra group
 *   (w13_extra != NULL) owns rows [offsets[G], offsets[G] + extra_rows) and maps row r to source
 *   row r - offsets[G] (the shared expert on every token).
 *   Row m of a regular group reads x_q[sorted_src[m] / K] (idx_mode TOKEN_MAJOR) or
 *   x_q[sorted_src[m] % T] (K_MAJOR); sorted_src NULL: row m reads x_q[m].
 *   acc = x_q[row] . W13[g]  (int32, exact);  d = (float(acc) * w13_scale[g][n]) * x_scale[row];
 *   y = silu(d[:I]) * d[I:];  y *= quant_scale[g][n] when quant_scale is given ([G][I] fp32, the smooth_scale of
 *   fused_experts_w8a8_allgather_ep_a2, fused_moe.py:907; regular groups only);
 *   h_scale[m] = max|y| / 127;  h_q = rint(y / h_scale).
 *   w13 packed: G matrices of Kdim = H, N = 2I (gate channels first).
 *   acc_dbg (nullable) [M_cap, 2I] receives the int32 accumulators.
 *   workspace: omni_moe_gemm1_workspace_bytes(T, K, G, extra_rows, M_cap, H, I) (same arguments as the call).
 */
int omni_moe_gemm1_swiglu_quant(const int8_t* x_q, const float* x_scale, const int32_t* sorted_src, int idx_mode,
                                int T, int K, const int8_t* w13_packed, const float* w13_scale,
                                const int8_t* w13_extra, const float* w13_extra_scale, int extra_rows,
                                const int32_t* offsets, int G, int H, int I, int64_t M_cap, int flags,
                                const float* quant_scale, int8_t* h_q, float* h_scale, int32_t* acc_dbg, void* workspace,
                                size_t ws_bytes, void* stream);
size_t omni_moe_gemm1_workspace_bytes(int T, int K, int G, int extra_rows, int64_t M_cap, int H, int I);

/*
 * GEMM2 + dequant.  Replaces npu_grouped_matmul(scale=, per_token_scale=, output_dtype=bf16)
 * (fused_moe.py:570-574, :681-685; deepseek_moe.py:473-477; compressed_tensors_moe.py:249-251)
 * and npu_quant_matmul(pertoken_scale=) (schemes/compressed_tensors_w8a8_int8.py:105-109).
 *   rows_out[m, :] = cast((float(h_q[m] . W2[g]) * w2_scale[g][:]) * h_scale[m]), out_dtype BF16 or F32.
 *   w2 packed: G matrices of Kdim = I, N = H.  Grouping as in GEMM1.
 *   workspace (omni_moe_gemm2_workspace_bytes, 256-byte aligned) is scratch for tiles whose reduction is
 *   shared between blocks; NULL is accepted (such tiles then run unsplit, the results are the same).
 */
int omni_moe_gemm2_dequant(const int8_t* h_q, const float* h_scale, const int8_t* w2_packed, const float* w2_scale,
                           const int8_t* w2_extra, const float* w2_extra_scale, int extra_rows,
                           const int32_t* offsets, int G, int H, int I, int64_t M_cap, int out_dtype, void* rows_out,
                           int32_t* acc_dbg, void* workspace, size_t ws_bytes, void* stream);
size_t omni_moe_gemm2_workspace_bytes(int G, int extra_rows, int64_t M_cap, int H, int I);

/*
 * Expert placement (redundant copies of experts over the devices of an EP group).
 *
 * omni_placement_tables is HOST code on HOST pointers: from a placement pattern [world][layers][experts] of 0/1
 * (1: that device deploys that expert in that layer) it writes
 *   position_to_expert [layers][num_deploy] (may be NULL): device r owns the positions [r*P, (r+1)*P),
 *       P = num_deploy / world, and its deployed experts take them in ascending expert id; unused positions
 *       hold -1 (omni/accelerators/placement/omni_planner/cpp/placement_mapping.cpp:223-257);
 *   selector [layers][experts]: the position that `rank` routes a logical expert to: its own copy, else one of
 *       the copies on its host (devices_per_host devices per host), else one of the others, each set shared
 *       out by rank modulo the size of the set, in ascending position order; an expert without any copy keeps 0
 *       (placement_mapping.cpp:374-427).
 * A pattern entry other than 0/1 or a device with more than P experts is rejected.
 *
 * omni_moe_remap_ids: out[i] = map[ids[i]] for 0 <= ids[i] < n_map, other ids are copied; `map` is one layer's
 * row of the selector in device memory.  Replaces OmniPlanner.plan (omni_planner.py:244-274, the lookup at :273),
 * called from FusedMoE.apply_expert_load_balance (omni/models/common/layers/moe/fused_moe/layer.py:273-286).
 * out may be ids.
 *
 * omni_moe_record_activation: counts[e] = (counts[e] + tokens_per_expert[e]) mod modulus for the n deployed
 * experts of the rank (int64 counters of one layer, int32 token counts as omni_moe_permute writes them).
 * Replaces OmniPlanner.record_activation (omni_planner.py:337-343; called at fused_moe.py:652,746).
 */
int omni_placement_tables(const int32_t* pattern, int world, int layers, int experts, int rank,
                          int devices_per_host, int num_deploy, int32_t* position_to_expert, int32_t* selector);
int omni_moe_remap_ids(const int32_t* ids, int64_t n, const int32_t* map, int n_map, int32_t* out, void* stream);
int omni_moe_record_activation(int64_t* counts, const int32_t* tokens_per_expert, int n, int64_t modulus,
                               void* stream);

/*
 * Weighted un-permute.  Replaces the routing half of npu_grouped_matmul_finalize_routing
 * (fused_moe.py:536), npu_moe_finalize_routing (compressed_tensors_moe.py:253;
 * deepseek_moe.py:292-301) and the shared-expert add (deepseek_moe.py:303,366).
 *   acc = init ? float(init[n]) : 0;  for each kept assignment of token n, in `order`:
 *   acc += topk_w[n,k] * float(rows[src_to_dst[idx(n,k)]]);  out = bf16(acc);
 *   if post_add != NULL: out = bf16(float(out) + float(bf16(post_add_row n)))   (post_add has rows_dtype,
 *   row n of it is added; pass rows + offsets_total*H to add the extra group's rows).
 */
int omni_moe_combine(const void* rows, int rows_dtype, const float* topk_w, const int32_t* src_to_dst, int idx_mode,
                     int order, int T, int K, int H, const void* init_bf16, const void* post_add,
                     const int32_t* post_add_row0, void* out_bf16, void* stream);

/*
 * The whole layer in one call: quant (if x is bf16) -> permute -> GEMM1 epilogue -> GEMM2 -> combine,
 * the sequence of fused_experts_w8a8_allgather_ep (fused_moe.py:489-538) with the shared expert
 * (deepseek_moe.py:64-118,244,303) carried as an extra group.  Routing weights and ids are inputs
 * (omni_moe_route makes them).  x_dtype BF16: x is quantised first; x_dtype -1: x is int8 and
 * x_scale is given.  Returns bf16 [T,H].
 *   rows_dtype is the caller's choice of how the expert rows travel from GEMM2 to the weighted sum:
 *   OMNI_DT_F32  the rows stay fp32 and are rounded once, after the sum: the numerics of
 *                npu_grouped_matmul_finalize_routing (fused_moe.py:536); 4*H bytes per row of workspace;
 *   OMNI_DT_BF16 every row is rounded to bf16 first: the numerics of a bf16 npu_grouped_matmul followed by
 *                npu_moe_finalize_routing (fused_moe.py:570-574 + deepseek_moe.py:292-301); half the bytes.
 *   The same value must be given to omni_moe_w8a8_layer_workspace_bytes.
 *   quant_scale (nullable, [hi-lo][I] fp32): as for omni_moe_gemm1_swiglu_quant; with it the call is
 *   fused_experts_w8a8_allgather_ep_a2 (fused_moe.py:844-937) in its default form.
 */
int omni_moe_w8a8_layer(const void* x, int x_dtype, const float* x_scale_in, const float* topk_w,
                        const int32_t* topk_ids, int T, int K, int lo, int hi, const int8_t* w13_packed,
                        const float* w13_scale, const int8_t* w2_packed, const float* w2_scale,
                        const int8_t* sh13_packed, const float* sh13_scale, const int8_t* sh2_packed,
                        const float* sh2_scale, const float* quant_scale, int H, int I, int rows_dtype, void* out_bf16,
                        void* workspace, size_t ws_bytes, void* stream);
size_t omni_moe_w8a8_layer_workspace_bytes(int T, int K, int n_local, int H, int I, int with_shared, int rows_dtype);

/*
 * Router and layer in one call: FusedMoE.select_experts followed by the quant method's apply, the two steps
 * of a MoE block between the gate projection and the sum with the shared expert (deepseek_moe.py:253-263,
 * 329-339; layer.py:301-365).  The results are those of omni_moe_route followed by omni_moe_w8a8_layer, bit
 * for bit: the routing arguments (logits .. eps) mean what they mean for omni_moe_route, topk_w [T,K] fp32 and
 * topk_ids [T,K] int32 are outputs here and hold the routing when the call's work is done, everything else is
 * as for omni_moe_w8a8_layer, workspace size included.  Small calls (bf16 tokens, T*K <= 4096, H <= 8192) route,
 * quantise and sort in a single launch; other calls run the router's own launch first.
 *   The single launch counts its finished routing blocks in an arrival counter, a word of a static device array
 *   (16 KiB per GPU, zero when the library is loaded; every launch leaves its word at zero).  Eager calls take the
 *   first 256 words in turn: nothing is asked of the caller as long as fewer than 256 such calls are in flight on
 *   one GPU at a time.  A call recorded into a stream capture keeps its word for every replay, so it gets one that
 *   eager calls never use: one word per (capture, stream) pair, shared by the calls that stream records into that
 *   capture (they are ordered in every replay; a graph does not run concurrently with itself).  3840 such words
 *   exist; when they are used up, or when the first such call on a device happens inside a capture (the look-up
 *   of the device's copy of the array is not made there), the call records the separate launches instead: same
 *   results, one launch more.
 */
int omni_moe_w8a8_layer_routed(const void* x, int x_dtype, const float* x_scale_in, const float* logits,
                               const float* bias, int E, int n_group, int topk_group, int score_fn, int group_mode,
                               int masked_fill_zero, int weight_from_c, int renorm, float scale, float eps,
                               float* topk_w, int32_t* topk_ids, int T, int K, int lo, int hi,
                               const int8_t* w13_packed, const float* w13_scale, const int8_t* w2_packed,
                               const float* w2_scale, const int8_t* sh13_packed, const float* sh13_scale,
                               const int8_t* sh2_packed, const float* sh2_scale, int H, int I, int rows_dtype,
                               void* out_bf16, void* workspace, size_t ws_bytes, void* stream);

/*
 * The whole MoE block in one call: gate projection, router and layer, i.e. self.gate.forward(hidden_states.float())
 * + FusedMoE.select_experts + the quant method's apply + the sum with the shared expert
 * (omni/models/common/layers/moe/deepseek_moe.py:147-152, 244-263, 303, 323-339, 366).  The results are those of
 * omni_moe_gate_route followed by omni_moe_w8a8_layer, bit for bit.
 *   x [T,H] is what the gate reads (x_dtype BF16 or F32); gate_w [E,H] fp32 or bf16 (gate_w_dtype); the routing
 *   arguments, round_logits_bf16, topk_w / topk_ids (outputs) as for omni_moe_gate_route.
 *   x_q / x_scale (both or neither): the tokens already quantised (the producer in front of the block can make
 *   them, omni_add_rms_norm_quant); without them x must be bf16 and is quantised here.
 *   Everything from T on as for omni_moe_w8a8_layer.  workspace: omni_moe_w8a8_block_workspace_bytes.
 * Two launches stand in front of the GEMMs for small calls (at most 1024 assignments): the partial sums of the
 * gate projection, then one launch that adds them up, routes, quantises and sorts (its arrival counter: see
 * omni_moe_w8a8_layer_routed); larger calls run the router, the quantiser and the sort as launches of their own.
 */
int omni_moe_w8a8_block(const void* x, int x_dtype, const int8_t* x_q, const float* x_scale, const void* gate_w,
                        int gate_w_dtype, const float* bias, int E, int n_group, int topk_group, int score_fn,
                        int group_mode, int masked_fill_zero, int weight_from_c, int renorm, float scale, float eps,
                        int round_logits_bf16, float* topk_w, int32_t* topk_ids, int T, int K, int lo, int hi,
                        const int8_t* w13_packed, const float* w13_scale, const int8_t* w2_packed, const float* w2_scale,
                        const int8_t* sh13_packed, const float* sh13_scale, const int8_t* sh2_packed,
                        const float* sh2_scale, int H, int I, int rows_dtype, void* out_bf16, void* workspace,
                        size_t ws_bytes, void* stream);
size_t omni_moe_w8a8_block_workspace_bytes(int T, int K, int n_local, int H, int I, int E, int with_shared,
                                           int rows_dtype);

/*
 * The same layer on the library's own scratch.  No counterpart in the reference: it is for callers
 * that cannot allocate device memory or hold a workspace (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  Arguments and results are those of omni_moe_w8a8_layer
 * without the workspace; the scratch is a static device array of OMNI_STATIC_SCRATCH_BYTES that every
 * GPU the library runs on holds until the process ends.  A call that would need more scratch (at the
 * DeepSeek-V3 shape with 32 local experts, a shared expert and fp32 rows: more than about 128 tokens, and
 * any shape whose row counts select the large-tile GEMM kernel) is refused with OMNI_E_WORKSPACE.
 * The call allocates nothing and frees nothing.  Its first call on a device looks up that device's copy
 * of the array (make that call outside a stream capture).  All calls on one GPU share the array, so two
 * calls that overlap in time on one GPU (different streams) race; calls on one stream are safe.
 */
#define OMNI_STATIC_SCRATCH_BYTES 67108864 /* 64 MiB */
int omni_moe_w8a8_layer_static(const void* x, int x_dtype, const float* x_scale_in, const float* topk_w,
                               const int32_t* topk_ids, int T, int K, int lo, int hi, const int8_t* w13_packed,
                               const float* w13_scale, const int8_t* w2_packed, const float* w2_scale,
                               const int8_t* sh13_packed, const float* sh13_scale, const int8_t* sh2_packed,
                               const float* sh2_scale, int H, int I, int rows_dtype, void* out_bf16, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* OMNI_MOE_HIP_H */
