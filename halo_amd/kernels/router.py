"""Fused router gate: softmax / top-k / renormalise / cast in one HIP kernel per direction (``csrc/router.hip``).

The reference calls a third-party router module for this step (transformers' ``Qwen3MoeTopKRouter`` and
``GptOssTopKRouter``; call sites ``halo/distributed/expert_parallel/moe_layer/shared_experts_layer.py:44-56`` and
``families/gpt_oss.py:108``) and restates its gate weights in ``moe_layer/routing.py:110-122`` and
``families/gpt_oss.py:82-84``.  Selection order here: descending score, equal scores to the lower expert index.
"""

from __future__ import annotations

import torch

from halo_amd import _lib
from halo_amd.kernels import _cpu

SOFTMAX_ALL = 0  # softmax over every expert, gather the picks, optionally renormalise by (sum + eps)
SOFTMAX_TOPK = 1  # softmax over the k selected logits


class _FusedTopKGate(torch.autograd.Function):
    @staticmethod
    def forward(ctx, logits: torch.Tensor, top_k: int, mode: int, normalize: bool, eps: float):
        device = _lib.require_device(logits)
        if logits.dim() != 2:
            raise ValueError(f"expected logits [tokens, experts], got {tuple(logits.shape)}")
        logits = logits.contiguous()
        n_tokens, num_experts = logits.shape
        indices = torch.empty((n_tokens, top_k), dtype=torch.long, device=device)
        weights = torch.empty((n_tokens, top_k), dtype=torch.float32, device=device)
        with _lib.on_device(device):
            _lib.call("hmoe_router_topk_fwd", _lib.ptr(logits), _lib.dtype_id(logits.dtype), n_tokens, num_experts,
                      top_k, mode, int(normalize), float(eps), _lib.ptr(indices), _lib.ptr(weights),
                      _lib.stream_ptr(device))
        ctx.save_for_backward(logits, indices)
        ctx.args = (top_k, mode, int(normalize), float(eps))
        ctx.mark_non_differentiable(indices)
        ctx.set_materialize_grads(False)  # no zero tensor made for the indices' gradient on the way back
        return indices, weights

    @staticmethod
    def backward(ctx, _grad_indices, grad_weights):
        logits, indices = ctx.saved_tensors
        if grad_weights is None:
            return None, None, None, None, None
        top_k, mode, normalize, eps = ctx.args
        device = logits.device
        grad_weights = grad_weights.float().contiguous()
        grad_logits = torch.empty_like(logits)
        n_tokens, num_experts = logits.shape
        with _lib.on_device(device):
            _lib.call("hmoe_router_topk_bwd", _lib.ptr(logits), _lib.dtype_id(logits.dtype), _lib.ptr(indices),
                      _lib.ptr(grad_weights), n_tokens, num_experts, top_k, mode, normalize, eps,
                      _lib.ptr(grad_logits), _lib.stream_ptr(device))
        return grad_logits, None, None, None, None


def fused_topk_gate(logits: torch.Tensor, top_k: int, *, mode: int = SOFTMAX_ALL, normalize: bool = True,
                    eps: float = 0.0) -> tuple[torch.Tensor, torch.Tensor]:
    """``(indices i64[T, k], weights f32[T, k])``: the router's picks and gate weights, the weights rounded to the
    logits' dtype and held in fp32 (what the layer gets after the router's cast and its own ``.float()``)."""
    if not logits.is_cuda:
        return _cpu.topk_gate(logits, top_k, mode == SOFTMAX_TOPK, normalize, eps)
    return _FusedTopKGate.apply(logits, top_k, mode, normalize, eps)
