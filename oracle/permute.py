"""Oracle (test infrastructure): token permute / weighted unpermute / expert-bias gather on the CPU.

Follows ``halo/kernels/moe_permute.py``.  The reference's device kernel multiplies and accumulates in fp32 and rounds
the sum once (``:17-41``, docstring ``:144-147``); its CPU twin rounds each weighted row first (``:115-120``).  The
target here is the device kernel's: accumulate wide, round once.  The accumulator is fp64, so a result in fp32 or
bf16 is the exact sum rounded once.
"""

from __future__ import annotations

import torch


def gather_rows(tokens: torch.Tensor, sorted_token_idx: torch.Tensor) -> torch.Tensor:
    """``MoEGatherPermute.forward`` (``halo/kernels/moe_permute.py:133-136``)."""
    return tokens.index_select(0, sorted_token_idx.long())


def gather_reduce(src: torch.Tensor, inv_map: torch.Tensor, weight: torch.Tensor | None = None,
                  out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """``out[r] = sum_k w[j] * src[j]`` over ``j = inv_map[r, k] < len(src)`` (``halo/kernels/moe_permute.py:17-41``):
    the permute's backward without a weight, the weighted unpermute's forward with one."""
    n_src = src.shape[0]
    wide = src.double()
    if weight is not None:
        wide = wide * weight.double().unsqueeze(-1)
    wide = torch.cat([wide, wide.new_zeros(1, src.shape[1])], 0)
    index = inv_map.long().clamp(max=n_src)
    out = wide[index].sum(dim=1)
    return out.to(out_dtype if out_dtype is not None else src.dtype)


def weighted_unpermute_backward(grad_out: torch.Tensor, expert_out: torch.Tensor | None, weights: torch.Tensor,
                                sorted_token_idx: torch.Tensor):
    """``grad_expert[j] = w[j] * grad_out[tok[j]]`` in ``grad_out``'s dtype and ``grad_w[j] = <grad_out[tok[j]],
    expert_out[j]>`` accumulated wide, cast to ``weights``' dtype (``halo/kernels/moe_permute.py:44-72, 158-189``).
    ``expert_out`` None skips the weight gradient."""
    gathered = grad_out.index_select(0, sorted_token_idx.long()).double()
    grad_expert = (gathered * weights.double().unsqueeze(-1)).to(grad_out.dtype)
    if expert_out is None:
        return grad_expert, None
    grad_weights = (gathered * expert_out.double()).sum(-1)
    return grad_expert, grad_weights.to(weights.dtype)


def bias_gather(bias: torch.Tensor, eids: torch.Tensor) -> torch.Tensor:
    """``MoEExpertBiasGather.forward`` (``halo/kernels/moe_permute.py:197-200``)."""
    return bias.index_select(0, eids.long())


def bias_gather_backward(grad_out: torch.Tensor, eids: torch.Tensor, num_experts: int) -> torch.Tensor:
    """Per-expert column sums of ``grad_out`` (``halo/kernels/moe_permute.py:202-208``), accumulated wide and rounded
    once to ``grad_out``'s dtype."""
    sums = torch.zeros(num_experts, grad_out.shape[1], dtype=torch.float64)
    sums.index_add_(0, eids.long(), grad_out.double())
    return sums.to(grad_out.dtype)
