"""Operator boundary: torch-tensor wrappers over the C ABI of libomni_moe_hip.so.

Each function stands where the reference calls a ``torch_npu.npu_*`` operator on the MoE
path and keeps that operator's argument meaning; the arithmetic is done by the gfx950 HIP
kernels.  torch is used for device memory and the current stream only.  Nothing here has a
CPU or eager fallback: tensors must live on the GPU and the library must be built.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib as L


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _need_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("omni_infer_amd operators run on the GPU only (got a CPU tensor)")


_DT = {torch.bfloat16: L.OMNI_DT_BF16, torch.float32: L.OMNI_DT_F32, torch.float16: L.OMNI_DT_F16}


# ----------------------------------------------------------------------------- routing
def moe_route(logits: torch.Tensor, bias: Optional[torch.Tensor], top_k: int, n_group: int, topk_group: int,
              score_fn: str, group_mode: int, masked_fill_zero: bool, weight_from_c: bool, renorm: bool,
              scale: float, eps: float) -> Tuple[torch.Tensor, torch.Tensor]:
    _need_gpu(logits, bias)
    if logits.dim() != 2:
        raise ValueError("router logits must be [T, E]")
    logits = logits.float().contiguous()
    T, E = logits.shape
    if bias is not None:
        bias = bias.float().contiguous()
        if bias.numel() != E:
            raise ValueError("bias must have one entry per expert")
    w = torch.empty(T, top_k, dtype=torch.float32, device=logits.device)
    ids = torch.empty(T, top_k, dtype=torch.int32, device=logits.device)
    fn = {"softmax": L.OMNI_SCORE_SOFTMAX, "sigmoid": L.OMNI_SCORE_SIGMOID}.get(score_fn)
    if fn is None:
        raise ValueError(f"Unsupported scoring function: {score_fn}")
    rc = L.lib().omni_moe_route(_ptr(logits), _ptr(bias), T, E, int(n_group), int(topk_group), int(top_k), fn,
                                int(group_mode), int(masked_fill_zero), int(weight_from_c), int(renorm),
                                float(scale), float(eps), _ptr(w), _ptr(ids), _stream())
    L.check(rc, "omni_moe_route")
    return w, ids


_GATE_WS = {}


def moe_gate_route(x: torch.Tensor, gate_w: torch.Tensor, bias: Optional[torch.Tensor], top_k: int, n_group: int,
                   topk_group: int, score_fn: str, group_mode: int, masked_fill_zero: bool, weight_from_c: bool,
                   renorm: bool, scale: float, eps: float, want_logits: bool = False, round_logits_bf16: bool = False):
    """Gate projection and router in one library call: ``self.gate.forward(hidden_states.float())`` +
    ``FusedMoE.select_experts`` (deepseek_moe.py:147-152,253-256).  ``x`` [T,H] bf16 or fp32 is read as it
    is (no fp32 copy), ``gate_w`` [E,H] fp32 or bf16.  ``top_k`` = 0 computes the logits only.
    Returns (topk_w, topk_ids, logits or None)."""
    _need_gpu(x, gate_w, bias)
    if x.dim() != 2 or gate_w.dim() != 2 or x.shape[1] != gate_w.shape[1]:
        raise ValueError("gate: x must be [T, H] and the gate weight [E, H]")
    if x.dtype not in (torch.bfloat16, torch.float32) or gate_w.dtype not in (torch.bfloat16, torch.float32):
        raise ValueError("gate: tokens and gate weight must be bf16 or fp32")
    x = x.contiguous()
    gate_w = gate_w.contiguous()
    T, H = x.shape
    E = gate_w.shape[0]
    dev = x.device
    if bias is not None:
        bias = bias.float().contiguous()
        if bias.numel() != E:
            raise ValueError("bias must have one entry per expert")
    fn = {"softmax": L.OMNI_SCORE_SOFTMAX, "sigmoid": L.OMNI_SCORE_SIGMOID}.get(score_fn)
    if fn is None:
        raise ValueError(f"Unsupported scoring function: {score_fn}")
    need = L.lib().omni_moe_gate_route_workspace_bytes(T, H, E)
    key = str(dev)
    ws = _GATE_WS.get(key)   # one scratch per device, grown on demand; calls on one stream are ordered
    if ws is None or ws.numel() < need:
        ws = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
        _GATE_WS[key] = ws
    w = torch.empty(T, top_k, dtype=torch.float32, device=dev) if top_k > 0 else None
    ids = torch.empty(T, top_k, dtype=torch.int32, device=dev) if top_k > 0 else None
    logits = torch.empty(T, E, dtype=torch.float32, device=dev) if (want_logits or top_k == 0) else None
    rc = L.lib().omni_moe_gate_route(_ptr(x), _DT[x.dtype], _ptr(gate_w), _DT[gate_w.dtype], _ptr(bias), T, H, E,
                                     int(n_group), int(topk_group), int(top_k), fn, int(group_mode),
                                     int(masked_fill_zero), int(weight_from_c), int(renorm), float(scale), float(eps),
                                     int(round_logits_bf16), _ptr(logits), _ptr(w), _ptr(ids), _ptr(ws), ws.numel(),
                                     _stream())
    L.check(rc, "omni_moe_gate_route")
    return w, ids, logits


def gate_logits(x: torch.Tensor, gate_w: torch.Tensor, round_logits_bf16: bool = False) -> torch.Tensor:
    """``ReplicatedLinear.forward`` of the gate (deepseek_moe.py:147-152): fp32 logits [T, E] in the
    library's fixed summation order."""
    return moe_gate_route(x, gate_w, None, 0, 1, 1, "softmax", L.OMNI_GROUP_MAX, False, False, False, 1.0, 0.0,
                          round_logits_bf16=round_logits_bf16)[2]


_ROW_IDX = {}


def _row_idx(T: int, K: int, device) -> torch.Tensor:
    """row_idx[n, k] = k*T + n (fused_moe.py:80-81, layer.py:352-353).  A constant of (T, K): made once per
    shape and device, so that the routing wrappers launch nothing but the router."""
    key = (int(T), int(K), str(device))
    t = _ROW_IDX.get(key)
    if t is None:
        if len(_ROW_IDX) > 256:
            _ROW_IDX.clear()
        t = torch.arange(T * K, device=device, dtype=torch.int32).view(K, T).transpose(0, 1)
        _ROW_IDX[key] = t
    return t


def npu_moe_gating_top_k(x: torch.Tensor, k: int, bias: Optional[torch.Tensor], k_group: int, group_count: int,
                         group_select_mode: int = 1, renorm: int = 0, norm_type: int = 1,
                         routed_scaling_factor: float = 1.0, eps: float = 1e-20):
    """Stands in for ``torch_npu.npu_moe_gating_top_k`` as called at
    omni/models/common/layers/moe/fused_moe/layer.py:341-351."""
    if renorm != 0:
        raise ValueError("npu_moe_gating_top_k: only renorm=0 (score, then top-k) is supported")
    w, ids = moe_route(x, bias, k, group_count, k_group, "sigmoid" if norm_type == 1 else "softmax",
                       L.OMNI_GROUP_TOP2SUM if group_select_mode == 1 else L.OMNI_GROUP_MAX,
                       masked_fill_zero=False, weight_from_c=False, renorm=True,
                       scale=routed_scaling_factor, eps=eps)
    return w, ids, None


def npu_moe_gating_top_k_softmax(x: torch.Tensor, k: int):
    """Stands in for ``torch_npu.npu_moe_gating_top_k_softmax`` (fused_moe.py:29)."""
    w, ids = moe_route(x, None, k, 1, 1, "softmax", L.OMNI_GROUP_MAX, False, False, False, 1.0, 0.0)
    return w, ids, _row_idx(x.shape[0], k, x.device)


# ----------------------------------------------------------------------------- quant
def npu_dynamic_quant(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Stands in for ``torch_npu.npu_dynamic_quant`` (deepseek_moe.py:247,323;
    compressed_tensors_moe.py:241,247; schemes/compressed_tensors_w8a8_int8.py:97)."""
    _need_gpu(x)
    if x.dtype not in _DT:
        raise ValueError(f"npu_dynamic_quant: unsupported dtype {x.dtype}")
    shape = x.shape
    x2 = x.reshape(-1, shape[-1])
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    rows, cols = x2.shape
    q = torch.empty(rows, cols, dtype=torch.int8, device=x.device)
    s = torch.empty(rows, dtype=torch.float32, device=x.device)
    rc = L.lib().omni_dynamic_quant(_ptr(x2), _DT[x.dtype], rows, cols, x2.stride(0) if rows > 1 else cols,
                                    _ptr(q), _ptr(s), _stream())
    L.check(rc, "omni_dynamic_quant")
    return q.view(shape), s.view(shape[:-1])


def add_rms_norm_quant(x: torch.Tensor, residual: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                       want_y: bool = True, want_quant: bool = False, inplace_residual: bool = False):
    """Stands in for ``npu_add_rms_norm`` / ``npu_rms_norm`` and, with ``want_quant``, the
    ``npu_dynamic_quant`` that follows it (omni/models/common/layers/layernorm.py:13-32).
    Returns (y or None, residual_out or None, x_int8 or None, pertoken_scale or None)."""
    _need_gpu(x, weight)
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16 or (residual is not None and residual.dtype != torch.bfloat16):
        raise ValueError("add_rms_norm_quant: bf16 tensors only")
    shape = x.shape
    H = shape[-1]
    x2 = x.reshape(-1, H).contiguous()
    rows = x2.shape[0]
    r2 = residual.reshape(-1, H).contiguous() if residual is not None else None
    res_out = None
    if r2 is not None:
        res_out = r2 if inplace_residual else torch.empty_like(r2)
    y = torch.empty_like(x2) if want_y else None
    q = torch.empty(rows, H, dtype=torch.int8, device=x.device) if want_quant else None
    sc = torch.empty(rows, dtype=torch.float32, device=x.device) if want_quant else None
    rc = L.lib().omni_add_rms_norm_quant(_ptr(x2), _ptr(r2), _ptr(weight.contiguous()), rows, H, float(eps),
                                         _ptr(res_out), _ptr(y), _ptr(q), _ptr(sc), _stream())
    L.check(rc, "omni_add_rms_norm_quant")
    return (y.view(shape) if y is not None else None, res_out.view(shape) if res_out is not None else None,
            q.view(shape) if q is not None else None, sc.view(shape[:-1]) if sc is not None else None)


# ----------------------------------------------------------------------------- permutation
class Permutation:
    """Result of sorting the (token, k) assignments by local expert."""
    __slots__ = ("sorted_src", "src_to_dst", "counts", "offsets", "T", "K", "n_local", "idx_mode")


def moe_permute(topk_ids: torch.Tensor, lo: int, hi: int, idx_mode: int = L.OMNI_IDX_TOKEN_MAJOR) -> Permutation:
    _need_gpu(topk_ids)
    if topk_ids.dtype != torch.int32:
        topk_ids = topk_ids.to(torch.int32)
    topk_ids = topk_ids.contiguous()
    T, K = topk_ids.shape
    G = hi - lo
    dev = topk_ids.device
    p = Permutation()
    p.T, p.K, p.n_local, p.idx_mode = T, K, G, idx_mode
    p.sorted_src = torch.empty(max(T * K, 1), dtype=torch.int32, device=dev)
    p.src_to_dst = torch.empty(max(T * K, 1), dtype=torch.int32, device=dev)
    p.counts = torch.empty(G, dtype=torch.int32, device=dev)
    p.offsets = torch.empty(G + 1, dtype=torch.int32, device=dev)
    ws_bytes = L.lib().omni_moe_permute_workspace_bytes(T, K, G)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    rc = L.lib().omni_moe_permute(_ptr(topk_ids), T, K, lo, hi, idx_mode, _ptr(p.sorted_src), _ptr(p.src_to_dst),
                                  _ptr(p.counts), _ptr(p.offsets), _ptr(ws), ws_bytes, _stream())
    L.check(rc, "omni_moe_permute")
    return p


def moe_gather_rows(x: torch.Tensor, x_scale: Optional[torch.Tensor], p: Permutation):
    _need_gpu(x)
    x = x.contiguous()
    T, H = x.shape
    rows = torch.zeros(T * p.K, H, dtype=x.dtype, device=x.device)
    sc = torch.zeros(T * p.K, dtype=torch.float32, device=x.device) if x_scale is not None else None
    rc = L.lib().omni_moe_gather_rows(_ptr(x), x.element_size(), H, _ptr(x_scale), _ptr(p.sorted_src),
                                      _ptr(p.offsets), p.n_local, T, p.K, p.idx_mode, _ptr(rows), _ptr(sc), _stream())
    L.check(rc, "omni_moe_gather_rows")
    return rows, sc


def npu_moe_init_routing_v2(x: torch.Tensor, expert_idx: torch.Tensor, scale: Optional[torch.Tensor] = None,
                            active_expert_range=None, expert_num: int = 0, **_unused):
    """Stands in for ``torch_npu.npu_moe_init_routing_v2`` with ``row_idx_type=1``,
    ``expert_tokens_num_type=1``, ``quant_mode=-1`` (fused_moe.py:514-515): returns
    (sorted rows, expanded_x_idx, per-expert counts int64, gathered scale)."""
    lo, hi = active_expert_range if active_expert_range is not None else (0, expert_num)
    p = moe_permute(expert_idx, lo, hi, L.OMNI_IDX_TOKEN_MAJOR)
    rows, sc = moe_gather_rows(x, scale, p)
    return rows, p.sorted_src, p.counts.to(torch.int64), sc


def npu_moe_init_routing(x: torch.Tensor, row_idx: torch.Tensor, expert_idx: torch.Tensor, active_num: int,
                         num_experts: int = 256):
    """Stands in for ``torch_npu.npu_moe_init_routing`` (compressed_tensors_moe.py:235-236):
    returns (sorted rows, expanded_src_to_dst_row indexed by k*T+n, sorted expert ids).
    ``row_idx`` must be the reference's k*T+n numbering (the only one it ever builds,
    compressed_tensors_moe.py:186-187); ``num_experts`` bounds the expert ids (no host sync)."""
    T, K = expert_idx.shape
    p = moe_permute(expert_idx, 0, num_experts, L.OMNI_IDX_K_MAJOR)
    rows, _ = moe_gather_rows(x, None, p)
    sorted_ids = torch.repeat_interleave(torch.arange(p.n_local, device=x.device, dtype=torch.int32),
                                         p.counts.to(torch.int64), output_size=T * K)
    return rows, p.src_to_dst, sorted_ids


def group_offsets(counts: torch.Tensor) -> torch.Tensor:
    """int32 [G+1] row offsets of the groups from their sizes (int32 or int64 [G]): what the reference's grouped
    operators make of ``group_list`` with ``group_list_type=1`` inside (fused_moe.py:531-536)."""
    _need_gpu(counts)
    if counts.dtype not in (torch.int32, torch.int64):
        counts = counts.to(torch.int64)
    counts = counts.contiguous()
    G = counts.numel()
    offsets = torch.empty(G + 1, dtype=torch.int32, device=counts.device)
    rc = L.lib().omni_moe_group_offsets(_ptr(counts), int(counts.dtype == torch.int64), G, _ptr(offsets), _stream())
    L.check(rc, "omni_moe_group_offsets")
    return offsets


def npu_moe_compute_expert_tokens(sorted_expert_idx: torch.Tensor, num_experts: int) -> torch.Tensor:
    """Stands in for ``torch_npu.npu_moe_compute_expert_tokens`` (compressed_tensors_moe.py:237):
    cumulative number of rows up to and including each expert."""
    return group_offsets(torch.bincount(sorted_expert_idx.to(torch.int64), minlength=num_experts))[1:]


_DENSE_OFFSETS = {}


def dense_offsets(M: int, device) -> torch.Tensor:
    """[0, M] int32 on the device: the row grouping of a dense (one group) GEMM.  Cached so that
    the steady state issues no host-to-device copy."""
    key = (int(M), str(device))
    t = _DENSE_OFFSETS.get(key)
    if t is None:
        t = torch.tensor([0, int(M)], dtype=torch.int32, device=device)
        _DENSE_OFFSETS[key] = t
    return t


# ----------------------------------------------------------------------------- weights
def pack_weight(w: torch.Tensor, src_layout: int) -> torch.Tensor:
    """One-off re-layout of int8 weights into the frag16 format the GEMM kernels stream
    (the analogue of ``npu_format_cast(w, 29)``, compressed_tensors_moe.py:97-99).
    src_layout 0: w is [G, Kdim, N]; 1: w is [G, N, Kdim]."""
    _need_gpu(w)
    if w.dtype != torch.int8:
        raise ValueError("pack_weight expects int8 weights")
    if w.dim() == 2:
        w = w.unsqueeze(0)
    w = w.contiguous()
    G = w.shape[0]
    Kdim, N = (w.shape[1], w.shape[2]) if src_layout == 0 else (w.shape[2], w.shape[1])
    out = torch.empty(G, Kdim * N, dtype=torch.int8, device=w.device)
    rc = L.lib().omni_moe_pack_weight(_ptr(w), src_layout, G, Kdim, N, _ptr(out), _stream())
    L.check(rc, "omni_moe_pack_weight")
    return out


# ----------------------------------------------------------------------------- GEMMs
def _quant_scale(quant_scale: Optional[torch.Tensor], G: int, I: int) -> Optional[torch.Tensor]:
    """The ``quant_scale`` of ``npu_dequant_swiglu_quant`` as the library takes it: contiguous fp32 [G, I]."""
    if quant_scale is None:
        return None
    _need_gpu(quant_scale)
    if tuple(quant_scale.shape) != (G, I):
        raise ValueError(f"quant_scale must be [{G}, {I}] (one factor per expert and intermediate channel)")
    return quant_scale.float().contiguous()


def grouped_gemm1_swiglu_quant(x_q: torch.Tensor, x_scale: torch.Tensor, sorted_src: Optional[torch.Tensor],
                               idx_mode: int, K: int, w13_packed: torch.Tensor, w13_scale: torch.Tensor,
                               offsets: torch.Tensor, H: int, I: int, M_cap: int,
                               extra: Optional[Tuple[torch.Tensor, torch.Tensor]] = None, extra_rows: int = 0,
                               bf16_intermediate: bool = False, want_acc: bool = False, flags: int = 0,
                               workspace: Optional[torch.Tensor] = None, out=None,
                               quant_scale: Optional[torch.Tensor] = None):
    """GEMM1 + dequant + SwiGLU + requant: ``npu_grouped_matmul(int32)`` +
    ``npu_dequant_swiglu_quant`` (fused_moe.py:531-534, :670-677).  Returns (h_q, h_scale, acc)."""
    _need_gpu(x_q, x_scale, w13_packed, w13_scale, offsets)
    dev = x_q.device
    T = x_q.shape[0]
    G = offsets.numel() - 1
    if out is None:
        h_q = torch.empty(M_cap, I, dtype=torch.int8, device=dev)
        h_s = torch.empty(M_cap, dtype=torch.float32, device=dev)
    else:
        h_q, h_s = out
    acc = torch.zeros(M_cap, 2 * I, dtype=torch.int32, device=dev) if want_acc else None
    ws_bytes = L.lib().omni_moe_gemm1_workspace_bytes(T, K, G, extra_rows, M_cap, H, I)
    ws = workspace if workspace is not None else torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    ew, es = extra if extra is not None else (None, None)
    quant_scale = _quant_scale(quant_scale, G, I)
    rc = L.lib().omni_moe_gemm1_swiglu_quant(
        _ptr(x_q), _ptr(x_scale), _ptr(sorted_src), idx_mode, T, K, _ptr(w13_packed), _ptr(w13_scale), _ptr(ew),
        _ptr(es), extra_rows, _ptr(offsets), G, H, I, M_cap,
        flags | (L.OMNI_GEMM1_BF16_INTERMEDIATE if bf16_intermediate else 0), _ptr(quant_scale),
        _ptr(h_q), _ptr(h_s), _ptr(acc), _ptr(ws), ws_bytes, _stream())
    L.check(rc, "omni_moe_gemm1_swiglu_quant")
    return h_q, h_s, acc


def grouped_gemm2_dequant(h_q: torch.Tensor, h_scale: torch.Tensor, w2_packed: torch.Tensor, w2_scale: torch.Tensor,
                          offsets: torch.Tensor, H: int, I: int, out_dtype: torch.dtype = torch.bfloat16,
                          extra: Optional[Tuple[torch.Tensor, torch.Tensor]] = None, extra_rows: int = 0,
                          want_acc: bool = False, out: Optional[torch.Tensor] = None,
                          workspace: Optional[torch.Tensor] = None):
    """GEMM2 + dequant: ``npu_grouped_matmul(scale=, per_token_scale=, output_dtype=bf16)``
    (fused_moe.py:570-574, :681-685).  Returns (rows [M_cap, H], acc)."""
    _need_gpu(h_q, h_scale, w2_packed, w2_scale, offsets)
    dev = h_q.device
    M_cap = h_q.shape[0]
    G = offsets.numel() - 1
    # rows past the kept total are never written and never read by a consumer that goes by the offsets
    rows = out if out is not None else torch.empty(M_cap, H, dtype=out_dtype, device=dev)
    acc = torch.zeros(M_cap, H, dtype=torch.int32, device=dev) if want_acc else None
    ew, es = extra if extra is not None else (None, None)
    need = L.lib().omni_moe_gemm2_workspace_bytes(G, extra_rows, M_cap, H, I)
    if workspace is None and need:
        workspace = torch.empty(need, dtype=torch.uint8, device=dev)
    rc = L.lib().omni_moe_gemm2_dequant(_ptr(h_q), _ptr(h_scale), _ptr(w2_packed), _ptr(w2_scale), _ptr(ew), _ptr(es),
                                        extra_rows, _ptr(offsets), G, H, I, M_cap, _DT[out_dtype], _ptr(rows),
                                        _ptr(acc), _ptr(workspace), workspace.numel() if workspace is not None else 0,
                                        _stream())
    L.check(rc, "omni_moe_gemm2_dequant")
    return rows, acc


def gemm_kernel_name(kind: int, T: int, K: int, G: int, extra_rows: int, M_cap: int, H: int, I: int) -> str:
    """Template name of the GEMM kernel the library launches for a call of these sizes (diagnostic)."""
    import ctypes
    buf = ctypes.create_string_buffer(64)
    rc = L.lib().omni_moe_gemm_kernel_name(kind, T, K, G, extra_rows, M_cap, H, I, ctypes.addressof(buf), 64)
    L.check(rc, "omni_moe_gemm_kernel_name")
    return buf.value.decode()


def moe_combine(rows: torch.Tensor, topk_w: torch.Tensor, src_to_dst: torch.Tensor, idx_mode: int, order: int,
                init: Optional[torch.Tensor] = None, post_add: Optional[torch.Tensor] = None,
                post_add_row0: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Weighted un-permute: ``npu_moe_finalize_routing`` (compressed_tensors_moe.py:253;
    deepseek_moe.py:292-301) and the routing half of ``npu_grouped_matmul_finalize_routing``
    (fused_moe.py:536).  Returns bf16 [T, H]."""
    _need_gpu(rows, topk_w, src_to_dst)
    T, K = topk_w.shape
    H = rows.shape[1]
    topk_w = topk_w.float().contiguous()
    if init is not None:
        init = init.to(torch.bfloat16).contiguous()
    out = torch.empty(T, H, dtype=torch.bfloat16, device=rows.device)
    rc = L.lib().omni_moe_combine(_ptr(rows), _DT[rows.dtype], _ptr(topk_w), _ptr(src_to_dst), idx_mode, order, T, K, H,
                                  _ptr(init), _ptr(post_add), _ptr(post_add_row0), _ptr(out), _stream())
    L.check(rc, "omni_moe_combine")
    return out


def moe_w8a8_layer(x: torch.Tensor, x_scale: Optional[torch.Tensor], topk_w: torch.Tensor, topk_ids: torch.Tensor,
                   lo: int, hi: int, w13_packed, w13_scale, w2_packed, w2_scale, shared=None, H: int = 0, I: int = 0,
                   workspace: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                   rows_dtype: torch.dtype = torch.float32, quant_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The whole local-share layer in one library call (quant if x is bf16, permute, GEMM1
    epilogue, GEMM2, combine), the shared expert carried as an extra group.

    ``rows_dtype`` is how the expert rows travel from GEMM2 to the weighted sum.  ``torch.float32``
    (default) keeps them fp32 and rounds once after the sum: the numerics of
    ``npu_grouped_matmul_finalize_routing`` (fused_moe.py:536).  ``torch.bfloat16`` rounds every row
    first: the numerics of the bf16 ``npu_grouped_matmul`` + ``npu_moe_finalize_routing`` pair
    (fused_moe.py:570-574, deepseek_moe.py:292-301), half the bytes of the largest intermediate."""
    _need_gpu(x, topk_w, topk_ids)
    T, K = topk_ids.shape
    dev = x.device
    x = x.contiguous()
    topk_w = topk_w.float().contiguous()
    topk_ids = topk_ids.to(torch.int32).contiguous()
    x_dtype = -1 if x.dtype == torch.int8 else _DT[x.dtype]
    sh = shared if shared is not None else (None, None, None, None)
    if rows_dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("rows_dtype must be torch.float32 or torch.bfloat16")
    need = L.lib().omni_moe_w8a8_layer_workspace_bytes(T, K, hi - lo, H, I, int(shared is not None), _DT[rows_dtype])
    if workspace is None or workspace.numel() < need:
        workspace = torch.empty(need, dtype=torch.uint8, device=dev)
    if out is None:
        out = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
    quant_scale = _quant_scale(quant_scale, hi - lo, I)
    rc = L.lib().omni_moe_w8a8_layer(_ptr(x), x_dtype, _ptr(x_scale), _ptr(topk_w), _ptr(topk_ids), T, K, lo, hi,
                                     _ptr(w13_packed), _ptr(w13_scale), _ptr(w2_packed), _ptr(w2_scale), _ptr(sh[0]),
                                     _ptr(sh[1]), _ptr(sh[2]), _ptr(sh[3]), _ptr(quant_scale), H, I, _DT[rows_dtype],
                                     _ptr(out), _ptr(workspace), workspace.numel(), _stream())
    L.check(rc, "omni_moe_w8a8_layer")
    return out


def moe_w8a8_layer_routed(x: torch.Tensor, x_scale: Optional[torch.Tensor], logits: torch.Tensor,
                          bias: Optional[torch.Tensor], top_k: int, n_group: int, topk_group: int, score_fn: str,
                          group_mode: int, masked_fill_zero: bool, weight_from_c: bool, renorm: bool, scale: float,
                          eps: float, lo: int, hi: int, w13_packed, w13_scale, w2_packed, w2_scale, shared=None,
                          H: int = 0, I: int = 0, workspace: Optional[torch.Tensor] = None,
                          out: Optional[torch.Tensor] = None, rows_dtype: torch.dtype = torch.float32,
                          topk_w: Optional[torch.Tensor] = None, topk_ids: Optional[torch.Tensor] = None):
    """``moe_route`` followed by ``moe_w8a8_layer`` in one library call (``FusedMoE.select_experts`` and the
    quant method's ``apply``: deepseek_moe.py:253-263; layer.py:301-365), the same bits as the two calls.  Small
    calls route, quantise and sort in a single launch.  Returns (out, topk_w, topk_ids)."""
    _need_gpu(x, logits, bias)
    if logits.dim() != 2:
        raise ValueError("router logits must be [T, E]")
    logits = logits.float().contiguous()
    T, E = logits.shape
    if x.shape[0] != T:
        raise ValueError("one row of logits per token")
    if bias is not None:
        bias = bias.float().contiguous()
        if bias.numel() != E:
            raise ValueError("bias must have one entry per expert")
    fn = {"softmax": L.OMNI_SCORE_SOFTMAX, "sigmoid": L.OMNI_SCORE_SIGMOID}.get(score_fn)
    if fn is None:
        raise ValueError(f"Unsupported scoring function: {score_fn}")
    if rows_dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("rows_dtype must be torch.float32 or torch.bfloat16")
    dev = x.device
    x = x.contiguous()
    K = int(top_k)
    if topk_w is None:
        topk_w = torch.empty(T, K, dtype=torch.float32, device=dev)
    if topk_ids is None:
        topk_ids = torch.empty(T, K, dtype=torch.int32, device=dev)
    if (topk_w.dtype != torch.float32 or topk_ids.dtype != torch.int32 or tuple(topk_w.shape) != (T, K) or
            tuple(topk_ids.shape) != (T, K) or not topk_w.is_contiguous() or not topk_ids.is_contiguous()):
        raise ValueError("topk_w must be a contiguous fp32 [T, K] tensor and topk_ids a contiguous int32 one")
    x_dtype = -1 if x.dtype == torch.int8 else _DT[x.dtype]
    sh = shared if shared is not None else (None, None, None, None)
    need = L.lib().omni_moe_w8a8_layer_workspace_bytes(T, K, hi - lo, H, I, int(shared is not None), _DT[rows_dtype])
    if workspace is None or workspace.numel() < need:
        workspace = torch.empty(need, dtype=torch.uint8, device=dev)
    if out is None:
        out = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
    rc = L.lib().omni_moe_w8a8_layer_routed(_ptr(x), x_dtype, _ptr(x_scale), _ptr(logits), _ptr(bias), E, int(n_group),
                                            int(topk_group), fn, int(group_mode), int(masked_fill_zero),
                                            int(weight_from_c), int(renorm), float(scale), float(eps), _ptr(topk_w),
                                            _ptr(topk_ids), T, K, lo, hi, _ptr(w13_packed), _ptr(w13_scale),
                                            _ptr(w2_packed), _ptr(w2_scale), _ptr(sh[0]), _ptr(sh[1]), _ptr(sh[2]),
                                            _ptr(sh[3]), H, I, _DT[rows_dtype], _ptr(out), _ptr(workspace),
                                            workspace.numel(), _stream())
    L.check(rc, "omni_moe_w8a8_layer_routed")
    return out, topk_w, topk_ids


def moe_w8a8_block(x: torch.Tensor, gate_w: torch.Tensor, bias: Optional[torch.Tensor], top_k: int, n_group: int,
                   topk_group: int, score_fn: str, group_mode: int, masked_fill_zero: bool, weight_from_c: bool,
                   renorm: bool, scale: float, eps: float, lo: int, hi: int, w13_packed, w13_scale, w2_packed, w2_scale,
                   shared=None, H: int = 0, I: int = 0, x_int8: Optional[torch.Tensor] = None,
                   pertoken_scale: Optional[torch.Tensor] = None, round_logits_bf16: bool = False,
                   workspace: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None,
                   rows_dtype: torch.dtype = torch.float32, topk_w: Optional[torch.Tensor] = None,
                   topk_ids: Optional[torch.Tensor] = None):
    """The whole block in one library call: ``self.gate.forward(hidden_states.float())``, ``FusedMoE.select_experts``,
    the quant method's ``apply`` and the sum with the shared expert (deepseek_moe.py:147-152, 244-263, 303).  The same
    bits as ``moe_gate_route`` followed by ``moe_w8a8_layer``.  ``x`` [T,H] bf16 (or fp32 together with ``x_int8`` /
    ``pertoken_scale``, the tokens already quantised).  Returns (out, topk_w, topk_ids)."""
    _need_gpu(x, gate_w, bias, x_int8, pertoken_scale)
    if x.dim() != 2 or gate_w.dim() != 2 or x.shape[1] != gate_w.shape[1]:
        raise ValueError("block: x must be [T, H] and the gate weight [E, H]")
    if x.dtype not in (torch.bfloat16, torch.float32) or gate_w.dtype not in (torch.bfloat16, torch.float32):
        raise ValueError("block: tokens and gate weight must be bf16 or fp32")
    if (x_int8 is None) != (pertoken_scale is None):
        raise ValueError("block: quantised tokens and their scales come together")
    x = x.contiguous()
    gate_w = gate_w.contiguous()
    T, E, K, dev = x.shape[0], gate_w.shape[0], int(top_k), x.device
    if x_int8 is not None:
        x_int8 = x_int8.contiguous()
        pertoken_scale = pertoken_scale.float().reshape(-1).contiguous()
    if bias is not None:
        bias = bias.float().contiguous()
        if bias.numel() != E:
            raise ValueError("bias must have one entry per expert")
    fn = {"softmax": L.OMNI_SCORE_SOFTMAX, "sigmoid": L.OMNI_SCORE_SIGMOID}.get(score_fn)
    if fn is None:
        raise ValueError(f"Unsupported scoring function: {score_fn}")
    if rows_dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("rows_dtype must be torch.float32 or torch.bfloat16")
    if topk_w is None:
        topk_w = torch.empty(T, K, dtype=torch.float32, device=dev)
    if topk_ids is None:
        topk_ids = torch.empty(T, K, dtype=torch.int32, device=dev)
    sh = shared if shared is not None else (None, None, None, None)
    need = L.lib().omni_moe_w8a8_block_workspace_bytes(T, K, hi - lo, H, I, E, int(shared is not None), _DT[rows_dtype])
    if workspace is None or workspace.numel() < need:
        workspace = torch.empty(max(need, 1), dtype=torch.uint8, device=dev)
    if out is None:
        out = torch.empty(T, H, dtype=torch.bfloat16, device=dev)
    rc = L.lib().omni_moe_w8a8_block(_ptr(x), _DT[x.dtype], _ptr(x_int8), _ptr(pertoken_scale), _ptr(gate_w),
                                     _DT[gate_w.dtype], _ptr(bias), E, int(n_group), int(topk_group), fn, int(group_mode),
                                     int(masked_fill_zero), int(weight_from_c), int(renorm), float(scale), float(eps),
                                     int(round_logits_bf16), _ptr(topk_w), _ptr(topk_ids), T, K, lo, hi, _ptr(w13_packed),
                                     _ptr(w13_scale), _ptr(w2_packed), _ptr(w2_scale), _ptr(sh[0]), _ptr(sh[1]), _ptr(sh[2]),
                                     _ptr(sh[3]), H, I, _DT[rows_dtype], _ptr(out), _ptr(workspace), workspace.numel(),
                                     _stream())
    L.check(rc, "omni_moe_w8a8_block")
    return out, topk_w, topk_ids


def moe_w8a8_layer_static(x: torch.Tensor, x_scale: Optional[torch.Tensor], topk_w: torch.Tensor, topk_ids: torch.Tensor,
                          lo: int, hi: int, w13_packed, w13_scale, w2_packed, w2_scale, shared=None, H: int = 0,
                          I: int = 0, out: Optional[torch.Tensor] = None,
                          rows_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """``moe_w8a8_layer`` on the library's static scratch: the call allocates nothing on the device
    when ``out`` is given and the inputs are already fp32 / int32 / contiguous.  Sizes that need more
    than ``OMNI_STATIC_SCRATCH_BYTES`` of scratch raise RuntimeError.  Calls that overlap in time on
    one GPU share the scratch and race; calls on one stream are safe."""
    _need_gpu(x, topk_w, topk_ids)
    T, K = topk_ids.shape
    if not (x.is_contiguous() and topk_w.is_contiguous() and topk_ids.is_contiguous() and
            topk_w.dtype == torch.float32 and topk_ids.dtype == torch.int32):
        raise ValueError("moe_w8a8_layer_static: contiguous inputs, fp32 weights and int32 ids only (no conversion "
                         "copies are made here)")
    if rows_dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("rows_dtype must be torch.float32 or torch.bfloat16")
    x_dtype = -1 if x.dtype == torch.int8 else _DT[x.dtype]
    sh = shared if shared is not None else (None, None, None, None)
    if out is None:
        out = torch.empty(T, H, dtype=torch.bfloat16, device=x.device)
    rc = L.lib().omni_moe_w8a8_layer_static(_ptr(x), x_dtype, _ptr(x_scale), _ptr(topk_w), _ptr(topk_ids), T, K, lo, hi,
                                            _ptr(w13_packed), _ptr(w13_scale), _ptr(w2_packed), _ptr(w2_scale),
                                            _ptr(sh[0]), _ptr(sh[1]), _ptr(sh[2]), _ptr(sh[3]), H, I, _DT[rows_dtype],
                                            _ptr(out), _stream())
    L.check(rc, "omni_moe_w8a8_layer_static")
    return out


# ----------------------------------------------------------------------------- expert placement
def placement_tables(pattern: torch.Tensor, rank: int, devices_per_host: int, num_deploy: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Host tables of a placement pattern [world, layers, experts] (0/1, CPU): ``position_to_expert``
    [layers, num_deploy] (-1: unused position) and ``selector`` [layers, experts], the position ``rank`` routes
    each logical expert to (placement_mapping.cpp:223-257, :374-427).  Both are CPU int32 tensors."""
    if pattern.is_cuda or pattern.dim() != 3:
        raise ValueError("placement pattern must be a CPU tensor [world, layers, experts]")
    pat = pattern.to(torch.int32).contiguous()
    world, layers, experts = pat.shape
    pos = torch.empty(layers, max(int(num_deploy), 0), dtype=torch.int32)
    sel = torch.empty(layers, experts, dtype=torch.int32)
    rc = L.lib().omni_placement_tables(pat.data_ptr(), world, layers, experts, int(rank), int(devices_per_host),
                                       int(num_deploy), pos.data_ptr(), sel.data_ptr())
    L.check(rc, "omni_placement_tables")
    return pos, sel


def remap_ids(ids: torch.Tensor, expert_map: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``embedding(ids, expert_map).squeeze(-1)`` of OmniPlanner.plan (omni_planner.py:273): every id becomes
    ``expert_map[id]``; int32 in, int32 out (``out`` may be ``ids``)."""
    _need_gpu(ids, expert_map)
    if ids.dtype != torch.int32:
        ids = ids.to(torch.int32)
    ids = ids.contiguous()
    expert_map = expert_map.reshape(-1)
    if expert_map.dtype != torch.int32 or not expert_map.is_contiguous():
        expert_map = expert_map.to(torch.int32).contiguous()
    if out is None:
        out = torch.empty_like(ids)
    elif out.dtype != torch.int32 or not out.is_contiguous() or out.numel() != ids.numel():
        raise ValueError("remap_ids: out must be a contiguous int32 tensor of the ids' size")
    rc = L.lib().omni_moe_remap_ids(_ptr(ids), ids.numel(), _ptr(expert_map), expert_map.numel(), _ptr(out), _stream())
    L.check(rc, "omni_moe_remap_ids")
    return out


def record_activation(counts: torch.Tensor, tokens_per_expert: torch.Tensor, modulus: int) -> torch.Tensor:
    """``counts = (counts + tokens_per_expert) % modulus`` in place (omni_planner.py:337-343): int64 counters of
    one layer, int32 token counts of the rank's deployed experts."""
    _need_gpu(counts, tokens_per_expert)
    if counts.dtype != torch.int64 or not counts.is_contiguous():
        raise ValueError("record_activation: counts must be a contiguous int64 tensor (it is updated in place)")
    n = counts.numel()
    if tokens_per_expert.numel() != n:
        raise ValueError("record_activation: one token count per counter")
    if tokens_per_expert.dtype != torch.int32 or not tokens_per_expert.is_contiguous():
        tokens_per_expert = tokens_per_expert.to(torch.int32).contiguous()
    rc = L.lib().omni_moe_record_activation(_ptr(counts), _ptr(tokens_per_expert), n, int(modulus), _stream())
    L.check(rc, "omni_moe_record_activation")
    return counts
