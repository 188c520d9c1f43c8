"""ctypes binding of libomni_moe_hip.so (the C ABI declared in include/omni_moe_hip.h).

The library is the only implementation of the operators: if it is missing or a symbol is
absent the import of this module's ``lib()`` fails loudly; there is no fallback path.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libomni_moe_hip.so")

P = c_void_p
I = c_int
# name -> (restype, argtypes); mirrors include/omni_moe_hip.h one to one
SIGNATURES = {
    "omni_moe_last_error": (c_char_p, []),
    "omni_moe_abi_version": (I, []),
    "omni_moe_route": (I, [P, P, I, I, I, I, I, I, I, I, I, I, c_float, c_float, P, P, P]),
    "omni_moe_gate_route": (I, [P, I, P, I, P, I, I, I, I, I, I, I, I, I, I, I, c_float, c_float, I, P, P, P, P, c_size_t, P]),
    "omni_moe_gate_route_workspace_bytes": (c_size_t, [I, I, I]),
    "omni_dynamic_quant": (I, [P, I, c_int64, I, c_int64, P, P, P]),
    "omni_add_rms_norm_quant": (I, [P, P, P, c_int64, I, c_float, P, P, P, P, P]),
    "omni_moe_permute": (I, [P, I, I, I, I, I, P, P, P, P, P, c_size_t, P]),
    "omni_moe_permute_workspace_bytes": (c_size_t, [I, I, I]),
    "omni_moe_group_offsets": (I, [P, I, I, P, P]),
    "omni_moe_gather_rows": (I, [P, I, I, P, P, P, I, I, I, I, P, P, P]),
    "omni_moe_pack_weight": (I, [P, I, I, I, I, P, P]),
    "omni_moe_gemm1_swiglu_quant": (I, [P, P, P, I, I, I, P, P, P, P, I, P, I, I, I, c_int64, I, P, P, P, P, P, c_size_t, P]),
    "omni_moe_gemm1_workspace_bytes": (c_size_t, [I, I, I, I, c_int64, I, I]),
    "omni_moe_gemm2_dequant": (I, [P, P, P, P, P, P, I, P, I, I, I, c_int64, I, P, P, P, c_size_t, P]),
    "omni_moe_gemm2_workspace_bytes": (c_size_t, [I, I, c_int64, I, I]),
    "omni_moe_gemm_kernel_name": (I, [I, I, I, I, I, c_int64, I, I, P, c_size_t]),
    "omni_placement_tables": (I, [P, I, I, I, I, I, I, P, P]),
    "omni_moe_remap_ids": (I, [P, c_int64, P, I, P, P]),
    "omni_moe_record_activation": (I, [P, P, I, c_int64, P]),
    "omni_moe_reload_tuning": (None, []),
    "omni_diag_mfma_i8_rate": (I, [P, c_size_t, I, I, P, P]),
    "omni_diag_hbm_read_rate": (I, [P, c_size_t, I, P, P]),
    "omni_diag_mfma_i8_tile_rate": (I, [P, c_size_t, I, I, I, P, P]),
    "omni_moe_combine": (I, [P, I, P, P, I, I, I, I, I, P, P, P, P, P]),
    "omni_moe_w8a8_layer": (I, [P, I, P, P, P, I, I, I, I, P, P, P, P, P, P, P, P, P, I, I, I, P, P, c_size_t, P]),
    "omni_moe_w8a8_layer_workspace_bytes": (c_size_t, [I, I, I, I, I, I, I]),
    "omni_moe_w8a8_layer_routed": (I, [P, I, P, P, P, I, I, I, I, I, I, I, I, c_float, c_float, P, P, I, I, I, I,
                                       P, P, P, P, P, P, P, P, I, I, I, P, P, c_size_t, P]),
    "omni_moe_w8a8_block": (I, [P, I, P, P, P, I, P, I, I, I, I, I, I, I, I, c_float, c_float, I, P, P, I, I, I, I,
                                P, P, P, P, P, P, P, P, I, I, I, P, P, c_size_t, P]),
    "omni_moe_w8a8_block_workspace_bytes": (c_size_t, [I, I, I, I, I, I, I, I]),
    "omni_moe_w8a8_layer_static": (I, [P, I, P, P, P, I, I, I, I, P, P, P, P, P, P, P, P, I, I, I, P, P]),
}

OMNI_DT_BF16, OMNI_DT_F32, OMNI_DT_F16 = 0, 1, 2
OMNI_SCORE_SOFTMAX, OMNI_SCORE_SIGMOID = 0, 1
OMNI_GROUP_MAX, OMNI_GROUP_TOP2SUM = 0, 1
OMNI_GEMM1_BF16_INTERMEDIATE, OMNI_GEMM1_NO_REQUANT, OMNI_GEMM1_WS_ZEROED = 1, 4, 8
OMNI_IDX_TOKEN_MAJOR, OMNI_IDX_K_MAJOR = 0, 1
OMNI_ORDER_SLOT, OMNI_ORDER_K = 0, 1

OMNI_STATIC_SCRATCH_BYTES = 64 << 20
ABI_VERSION = 7   # omni_moe_abi_version() of the header these signatures were written from

_lib = None


class OmniMoeError(RuntimeError):
    pass


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise OmniMoeError(
                f"{LIB_PATH} is missing: build it with `python -m omni_infer_amd._build` "
                "(hipcc --offload-arch=gfx950); there is no fallback implementation")
        # torch ships its own HIP runtime (same soname as /opt/rocm's).  The library must bind to
        # the runtime torch initialised, or its launches would see another runtime's streams and
        # devices: make sure torch is loaded first.
        import torch  # noqa: F401
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)  # AttributeError if the library does not export it
            fn.restype = res
            fn.argtypes = args
        have = handle.omni_moe_abi_version()
        if have != ABI_VERSION:
            raise OmniMoeError(f"{LIB_PATH} has ABI version {have}, this package binds version {ABI_VERSION}: "
                               "rebuild it with `python -m omni_infer_amd._build`")
        _lib = handle
    return _lib


def check(rc: int, what: str) -> None:
    """Map a negative return code to the exception type the reference raises for the same
    condition: invalid argument -> ValueError, unsupported / workspace / launch -> RuntimeError."""
    if rc == 0:
        return
    msg = lib().omni_moe_last_error().decode("utf-8", "replace")
    if rc == -1:
        raise ValueError(f"{what}: {msg}")
    raise OmniMoeError(f"{what}: {msg} (code {rc})")
