"""What the ``halo_amd.kernels`` operators do with CPU tensors: plain torch operations, with autograd's own gradients.

The reference's operators take CPU tensors as well (``halo/kernels/moe_route_sort.py:201-243`` sorts with a stable
argsort, ``moe_permute.py:115-127`` sums padded gathers, ``fused_glu.py:352-361`` multiplies eagerly, ``histogram.py``
scatter-adds), which is what its own CPU tests run on.  This module is that contract for this package.  It is reached
only for tensors that live on the CPU: a device tensor always takes the HIP library and raises when the library is
missing, so nothing here is a fallback for the GPU path.  The arithmetic follows the kernels' (products and sums in
fp32, or in fp64 for fp64 inputs, one rounding to the inputs' dtype) rather than the reference's CPU twins where the
two differ in the position of a rounding.
"""

from __future__ import annotations

import torch


def _acc_dtype(dtype: torch.dtype) -> torch.dtype:
    return torch.float64 if dtype == torch.float64 else torch.float32


# --------------------------------------------------------------------------------------------------- histogram

def bincount(indices: torch.Tensor, size: int, dtype: torch.dtype, weights: torch.Tensor | None) -> torch.Tensor:
    flat = indices.reshape(-1).long()
    inside = (flat >= 0) & (flat < size)
    native = torch.int64 if (weights is None and not dtype.is_floating_point) else torch.float32
    out = torch.zeros(size, dtype=native)
    ones = torch.ones_like(flat, dtype=native) if weights is None else weights.reshape(-1).to(native)
    out.scatter_add_(0, flat.clamp(0, max(size - 1, 0)), torch.where(inside, ones, torch.zeros_like(ones)))
    return out.to(dtype)


# ------------------------------------------------------------------------------------------------ routing sort

def sort_routing(experts: torch.Tensor, weights: torch.Tensor, num_local_experts: int,
                 counts: tuple[int, ...] | None, wrong_total: str, foreign_id: str):
    """Stable sort of the local slots by expert; only ``weights`` carries a gradient (through the indexing)."""
    from halo_amd.kernels.moe_permute import build_inv_map

    rows, top_k = experts.shape
    slot_expert = experts.reshape(-1)
    local = (slot_expert >= 0) & (slot_expert < num_local_experts)
    n_local = int(local.sum())
    if counts is None:
        if n_local != slot_expert.numel():
            raise RuntimeError(foreign_id)
    elif n_local != sum(counts):
        raise RuntimeError(wrong_total)
    slots = torch.nonzero(local).squeeze(1)  # ascending, so a stable sort by expert keeps slot order inside an expert
    order = slots[torch.argsort(slot_expert[slots], stable=True)]
    sorted_expert_ids = slot_expert[order]
    sorted_token_idx = torch.div(order, top_k, rounding_mode="floor")
    per_expert = bincount(sorted_expert_ids, num_local_experts, torch.int64, None)
    offs = per_expert.cumsum(0).to(torch.int32)
    return (sorted_token_idx, weights.reshape(-1)[order], sorted_expert_ids, offs,
            build_inv_map(sorted_token_idx, rows, top_k))


# ----------------------------------------------------------------------------------------- permute and combine

def gather_reduce(src: torch.Tensor, inv_map: torch.Tensor, weight: torch.Tensor | None, addend: torch.Tensor | None,
                  addend_scale: torch.Tensor | None) -> torch.Tensor:
    n_src = src.shape[0]
    acc = _acc_dtype(src.dtype)
    rows = src.to(acc)
    if weight is not None:
        rows = rows * weight.to(src.dtype).to(acc).unsqueeze(-1)
    padded = torch.cat([rows, rows.new_zeros(1, src.shape[1])], 0)
    out = padded[inv_map.long().clamp(max=n_src)].sum(dim=1).to(src.dtype)
    if addend is not None:
        out = out + (addend if addend_scale is None else addend_scale.reshape(-1, 1).to(src.dtype) * addend)
    return out


def unpermute_backward(grad_out, expert_out, weights, sorted_token_idx, weight_grad: bool):
    acc = _acc_dtype(grad_out.dtype)
    by_row = grad_out.index_select(0, sorted_token_idx.long()).to(acc)
    grad_expert = (by_row * weights.to(grad_out.dtype).to(acc).unsqueeze(-1)).to(grad_out.dtype)
    grad_weights = None
    if weight_grad:
        grad_weights = (by_row * expert_out.to(grad_out.dtype).to(acc)).sum(-1).to(weights.dtype)
    return grad_expert, grad_weights


def expert_bias_grad(grad_out: torch.Tensor, eids: torch.Tensor, num_experts: int) -> torch.Tensor:
    acc = _acc_dtype(grad_out.dtype)
    sums = torch.zeros((num_experts, grad_out.shape[1]), dtype=acc)
    return sums.index_add_(0, eids.long(), grad_out.to(acc)).to(grad_out.dtype)


# ------------------------------------------------------------------------------------------------ grouped GEMM

def _group_bounds(offs: torch.Tensor | None, groups: int, rows: int) -> list[tuple[int, int]]:
    if offs is None:
        return [(0, rows)]
    ends = [min(max(int(e), 0), rows) for e in offs.tolist()]
    starts = [0] + ends[:-1]
    return [(s, max(s, e)) for s, e in zip(starts, ends)][:groups]


def grouped_forward(mat_a: torch.Tensor, mat_b: torch.Tensor, offs: torch.Tensor | None) -> torch.Tensor:
    acc = _acc_dtype(mat_a.dtype)
    out = mat_a.new_zeros((mat_a.shape[0], mat_b.shape[2]))
    for g, (s, e) in enumerate(_group_bounds(offs, mat_b.shape[0], mat_a.shape[0])):
        if e > s:
            out[s:e] = (mat_a[s:e].to(acc) @ mat_b[g].to(acc)).to(mat_a.dtype)
    return out


def grouped_dgrad(grad_output: torch.Tensor, mat_b: torch.Tensor, offs: torch.Tensor | None) -> torch.Tensor:
    return grouped_forward(grad_output, mat_b.transpose(-2, -1), offs)


def grouped_wgrad(mat_a: torch.Tensor, grad_output: torch.Tensor, offs: torch.Tensor | None, groups: int):
    acc = _acc_dtype(mat_a.dtype)
    out = mat_a.new_zeros((groups, mat_a.shape[1], grad_output.shape[1]))
    for g, (s, e) in enumerate(_group_bounds(offs, groups, mat_a.shape[0])):
        if e > s:
            out[g] = (mat_a[s:e].to(acc).t() @ grad_output[s:e].to(acc)).to(mat_a.dtype)
    return out


# ------------------------------------------------------------------------------------------------------ router

def topk_gate(logits: torch.Tensor, top_k: int, softmax_over_picks: bool, normalize: bool, eps: float):
    """Descending score, equal scores to the lower index (a stable descending sort); weights in fp32 softmax arithmetic,
    rounded to the logits' dtype and handed on as fp32.  Differentiable in the logits."""
    picks = torch.sort(logits.detach().float(), dim=-1, descending=True, stable=True).indices[:, :top_k].contiguous()
    if softmax_over_picks:
        weights = torch.softmax(logits.float().gather(-1, picks), dim=-1)
    else:
        weights = torch.softmax(logits, dtype=torch.float, dim=-1).gather(-1, picks)
        if normalize:
            weights = weights / (weights.sum(dim=-1, keepdim=True) + eps)
    return picks, weights.to(logits.dtype).float()
