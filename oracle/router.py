"""Oracle (test infrastructure): softmax / top-k / renormalise routing on the CPU.

The reference calls a third-party router module for this step (transformers 5.20.2 ``Qwen3MoeTopKRouter.forward``
and ``GptOssTopKRouter.forward``; call sites ``halo/distributed/expert_parallel/moe_layer/shared_experts_layer.py:44-56``
and ``halo/distributed/expert_parallel/families/gpt_oss.py:108``) and restates its weights in
``halo/distributed/expert_parallel/moe_layer/routing.py:110-122`` (softmax over all experts in fp32, gather, optional
renormalisation by ``sum + eps``, cast to the logits' dtype) and ``families/gpt_oss.py:82-84`` (softmax over the k
selected logits in fp32).

Selection rule of this build: the k largest scores in descending order, and of equal scores the lower expert index
first.  ``torch.topk`` leaves that order unspecified, so the reference's own order on tied rows is parity unpinned;
on rows without a tie at or above the k-th score both agree.  Softmax is monotone, so the selection is read off the
logits, which compare exactly on every device.
"""

from __future__ import annotations

import torch

SOFTMAX_ALL = 0  # Qwen3 family: softmax over every expert, gather, optional renorm
SOFTMAX_TOPK = 1  # gpt-oss: softmax over the k selected logits


def select_topk(logits: torch.Tensor, top_k: int) -> torch.Tensor:
    """Indices ``[T, k]`` int64: descending logit, ties to the lower index (a stable descending sort)."""
    order = torch.sort(logits.float(), dim=-1, descending=True, stable=True).indices
    return order[:, :top_k].contiguous()


def gate_weights(logits: torch.Tensor, indices: torch.Tensor, mode: int, normalize: bool, eps: float) -> torch.Tensor:
    """Gate weights at ``indices`` in the logits' dtype (``routing.py:110-122``; ``families/gpt_oss.py:82-84``)."""
    if mode == SOFTMAX_TOPK:
        return torch.softmax(logits.float().gather(-1, indices), dim=-1).to(logits.dtype)
    probs = torch.softmax(logits, dtype=torch.float, dim=-1)
    weights = probs.gather(-1, indices)
    if normalize:
        weights = weights / (weights.sum(dim=-1, keepdim=True) + eps)
    return weights.to(logits.dtype)


def route(logits: torch.Tensor, top_k: int, mode: int = SOFTMAX_ALL, normalize: bool = True, eps: float = 0.0):
    """``(indices i64[T,k], weights fp32[T,k])`` as the layer hands them on: the router's weights in the logits' dtype,
    then ``.float()`` (``shared_experts_layer.py:26-27``)."""
    indices = select_topk(logits, top_k)
    return indices, gate_weights(logits, indices, mode, normalize, eps).float()


def route_backward(logits: torch.Tensor, indices: torch.Tensor, grad_weights: torch.Tensor, mode: int = SOFTMAX_ALL,
                   normalize: bool = True, eps: float = 0.0) -> torch.Tensor:
    """Gradient of the gate weights with respect to the logits by autograd through :func:`gate_weights` computed in
    fp64 (the cast to the logits' dtype passes its gradient through)."""
    leaf = logits.detach().double().requires_grad_(True)
    if mode == SOFTMAX_TOPK:
        weights = torch.softmax(leaf.gather(-1, indices), dim=-1)
    else:
        weights = torch.softmax(leaf, dim=-1).gather(-1, indices)
        if normalize:
            weights = weights / (weights.sum(dim=-1, keepdim=True) + eps)
    (grad,) = torch.autograd.grad(weights, leaf, grad_weights.double())
    return grad.to(logits.dtype)
