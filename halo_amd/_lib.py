"""ctypes binding of ``libhalo_moe.so`` (``include/halo_moe.h``).

The library is the only compute path for device tensors: if it is missing or fails to load, an op on a device tensor
raises; there is no fallback for it.  (CPU tensors take plain torch operations, as they do in the reference:
``halo_amd/kernels/_cpu.py``.)  Torch supplies device memory and the current HIP stream, nothing else.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p

import torch

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libhalo_moe.so")

HMOE_F32, HMOE_BF16 = 0, 1
_DTYPES = {torch.float32: HMOE_F32, torch.bfloat16: HMOE_BF16}

P, I, L, F = c_void_p, c_int, c_int64, c_float

# name -> (restype, argtypes); must list every symbol include/halo_moe.h declares
SIGNATURES = {
    "hmoe_abi_version": (I, []),
    "hmoe_status_string": (c_char_p, [I]),
    "hmoe_route_sort_workspace_bytes": (L, [L, I, I]),
    "hmoe_route_sort": (I, [P, I, P, I, L, I, I, L, P, P, P, P, P, P, P, P, P]),
    "hmoe_route_sort_static": (I, [P, I, P, I, L, I, I, L, P, P, P, P, P, P, P, P]),
    "hmoe_route_sort_bwd": (I, [P, P, L, L, I, P, P]),
    "hmoe_bincount": (I, [P, P, L, L, I, P, P]),
    "hmoe_gather_rows": (I, [P, L, P, L, L, I, P, P]),
    "hmoe_gather_reduce": (I, [P, P, P, L, I, L, L, I, P, P]),
    "hmoe_gather_reduce_add": (I, [P, P, P, L, I, L, L, I, P, L, P, P, P]),
    "hmoe_unpermute_bwd": (I, [P, L, P, P, P, L, L, I, P, P, P]),
    "hmoe_expert_colsum_workspace_bytes": (L, [L, L, I]),
    "hmoe_expert_colsum": (I, [P, P, L, L, I, I, P, P, P]),
    "hmoe_glu_fwd": (I, [P, P, L, L, L, L, I, I, F, F, I, I, P, P]),
    "hmoe_glu_bwd": (I, [P, P, L, L, P, L, L, I, I, F, F, I, I, P, P, L, L, P]),
    "hmoe_glu_fwd_weighted": (I, [P, P, L, L, P, I, L, L, I, I, F, F, I, I, P, P]),
    "hmoe_glu_bwd_weighted": (I, [P, P, L, L, P, P, I, L, L, I, I, F, F, I, I, P, P, L, L, P, P]),
    "hmoe_router_topk_fwd": (I, [P, I, L, I, I, I, I, F, P, P, P]),
    "hmoe_router_topk_bwd": (I, [P, I, P, P, L, I, I, I, I, F, P, P]),
    "hmoe_probe_mfma_bf16": (L, [L, I, I, P, P]),
    "hmoe_probe_hbm_read": (L, [P, L, P, P]),
    "hmoe_row_gate_fwd": (I, [P, L, P, L, I, I, P, P]),
    "hmoe_row_gate_bwd_workspace_bytes": (L, [L, I]),
    "hmoe_row_gate_bwd": (I, [P, L, P, P, P, L, I, I, P, L, P, P, P]),
    "hmoe_set_gemm_tile": (I, [I]),
    "hmoe_grouped_gemm_mx_fits": (I, [L, L, L, L, L, I]),
    "hmoe_grouped_gemm_fwd": (I, [P, L, P, P, L, I, L, L, I, P, L, P]),
    "hmoe_grouped_gemm_fwd_bias": (I, [P, L, P, P, P, L, I, L, L, I, P, L, P]),
    "hmoe_grouped_gemm_fwd_addto": (I, [P, L, P, P, L, I, L, L, I, P, L, F, P, L, P]),
    "hmoe_grouped_gemm_dgrad": (I, [P, L, P, P, L, I, L, L, I, P, L, P]),
    "hmoe_grouped_gemm_dgrad_addto": (I, [P, L, P, P, L, I, L, L, I, P, L, P, L, P]),
    "hmoe_grouped_gemm_wgrad": (I, [P, L, P, L, P, L, I, L, L, I, P, P]),
    "hmoe_grouped_gemm_fwd_gather": (I, [P, L, L, P, P, P, L, I, L, L, I, P, L, P]),
    "hmoe_grouped_gemm_fwd_gather_bias": (I, [P, L, L, P, P, P, P, L, I, L, L, I, P, L, P]),
    "hmoe_grouped_gemm_wgrad_gather": (I, [P, L, L, P, P, L, P, L, I, L, L, I, P, P]),
    "hmoe_grouped_gemm_dgrad_gather": (I, [P, L, L, P, P, P, L, I, L, L, I, P, L, P]),
    "hmoe_grouped_gemm_wgrad_gather_grad": (I, [P, L, P, L, L, P, P, L, I, L, L, I, P, P]),
    "hmoe_quantize_block_fp8": (I, [P, I, L, L, L, P, P, P]),
    "hmoe_dequantize_block_fp8": (I, [P, P, L, L, L, I, P, P]),
    "hmoe_grouped_gemm_fwd_fp8w": (I, [P, L, P, P, P, L, I, L, L, P, L, P]),
    "hmoe_quantize_rows_fp8": (I, [P, L, P, L, L, L, P, P, L, P]),
    "hmoe_glu_fwd_quant_fp8": (I, [P, P, L, L, L, L, I, F, F, I, I, P, P, L, P]),
    "hmoe_grouped_gemm_fwd_fp8": (I, [P, P, L, P, P, P, L, I, L, L, P, L, P]),
    "hmoe_quantize_rows_mxfp8": (I, [P, I, L, P, L, L, L, P, P, L, P]),
    "hmoe_dequantize_rows_mxfp8": (I, [P, P, L, L, L, P, L, P]),
    "hmoe_quantize_weight_mxfp8": (I, [P, I, L, L, L, P, P, P, P]),
    "hmoe_grouped_gemm_fwd_mxfp8": (I, [P, P, L, P, P, P, L, I, L, L, P, L, P]),
    "hmoe_mxfp4_rows": (I, [P, I, L, P, L, L, L, P, P, P, L, P]),
    "hmoe_mxfp4_weight": (I, [P, I, L, L, L, P, P, P, P]),
    "hmoe_mxfp4_dequantize_rows": (I, [P, P, L, L, P, L, P]),
    "hmoe_mxfp4_rows_panels": (I, [P, I, L, P, L, L, L, P, P, L, P]),
    "hmoe_mxfp4_weight_panels": (I, [P, I, L, L, L, P, P, P, P]),
    "hmoe_mxfp4_dequantize_panels": (I, [P, P, L, L, L, P, L, P]),
    "hmoe_grouped_gemm_fwd_mxfp4": (I, [P, P, L, P, P, P, L, I, L, L, P, L, P]),
    "hmoe_grouped_gemm_fwd_mxfp8_bias": (I, [P, P, L, P, P, P, P, L, I, L, L, P, L, P]),
    "hmoe_grouped_gemm_fwd_mxfp4_bias": (I, [P, P, L, P, P, P, P, L, I, L, L, P, L, P]),
    "hmoe_nvfp4_rows": (I, [P, I, L, P, L, L, L, P, P, P, P, L, P, P]),
    "hmoe_nvfp4_weight": (I, [P, I, L, L, L, P, P, P, P, P, P]),
    "hmoe_nvfp4_dequantize_rows": (I, [P, P, P, L, L, P, L, P]),
}

_lib = None


def load() -> ctypes.CDLL:
    """The loaded library; raises when it has not been built (``python -m halo_amd.build``)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: the HIP extension is the only compute path of halo_amd. "
                f"Build it with `python -m halo_amd.build` (hipcc, gfx950)."
            )
        lib = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = restype, argtypes
        _lib = lib
    return _lib


def dtype_id(dtype: torch.dtype) -> int:
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise TypeError(f"halo_amd kernels take float32 or bfloat16 tensors, got {dtype}") from None


def require_device(*tensors: torch.Tensor) -> torch.device:
    """All tensors on one GPU; a CPU tensor among device tensors is refused."""
    device = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError(
                "halo_amd kernels run on MI355X device tensors only; got a tensor on "
                f"{t.device} among the operands of a device call"
            )
        if device is None:
            device = t.device
        elif t.device != device:
            raise RuntimeError(f"tensors on different devices: {device} and {t.device}")
    return device


def ptr(t: torch.Tensor | None):
    return None if t is None else t.data_ptr()


def stream_ptr(device: torch.device | None = None):
    return torch.cuda.current_stream(device).cuda_stream


def call(name: str, *args) -> None:
    """Calls ``name`` and raises with the status text on a negative return."""
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise RuntimeError(f"{name} failed: {lib.hmoe_status_string(rc).decode()} (status {rc})")


class _NullGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NULL_GUARD = _NullGuard()


def on_device(device: torch.device):
    """Context making ``device`` current for the launch (kernels start on the current device)."""
    if device is None or device.index is None or device.index == torch.cuda.current_device():
        return _NULL_GUARD
    return torch.cuda.device(device)
