"""Atomic-free token permute/unpermute and per-expert bias gather for the grouped-GEMM MoE expert compute.  Both
directions reduce through ``inv_map`` in fp32 and round once.

Mirrors the reference's ``halo/kernels/moe_permute.py`` (``build_inv_map`` ``:75-89``, ``gather_reduce_rows``
``:123-127``, ``MoEGatherPermute`` ``:130-141``, ``MoEWeightedUnpermute`` ``:144-189``, ``MoEExpertBiasGather``
``:192-208``); the kernels are ``csrc/permute.hip``.
"""

from __future__ import annotations

import torch

from halo_amd import _lib
from halo_amd.kernels import _cpu
from halo_amd.kernels.histogram import sync_free_bincount


def _gather_rows(src: torch.Tensor, index: torch.Tensor) -> torch.Tensor:
    """``src[index]`` for a 2-D ``src`` whose rows may be strided (a ``[:, :H]`` view of a padded buffer)."""
    if src.dim() != 2:
        raise ValueError(f"expected [rows, hidden], got {tuple(src.shape)}")
    if not src.is_cuda:
        return src.index_select(0, index.long())
    device = _lib.require_device(src, index)
    if src.stride(1) != 1:
        src = src.contiguous()
    index = index.long().contiguous()
    hidden = src.shape[1]
    out = torch.empty((index.shape[0], hidden), dtype=src.dtype, device=device)
    if out.numel():
        with _lib.on_device(device):
            _lib.call("hmoe_gather_rows", _lib.ptr(src), src.stride(0), _lib.ptr(index), index.shape[0], hidden,
                      _lib.dtype_id(src.dtype), _lib.ptr(out), _lib.stream_ptr(device))
    return out


def gather_reduce_rows(src: torch.Tensor, inv_map: torch.Tensor, weight: torch.Tensor | None = None, *,
                       addend: torch.Tensor | None = None, addend_scale: torch.Tensor | None = None) -> torch.Tensor:
    """``out[r] = sum_k w[j] * src[j]`` over ``j = inv_map[r, k] < len(src)``; ``w = 1`` without a weight.  The sum is
    taken in fp32 and rounded once to ``src``'s dtype.  With ``addend [len(out), hidden]`` (and ``addend_scale
    [len(out)]``) the same pass returns ``out + addend_scale[:, None] * addend`` with that expression's roundings."""
    if not src.is_cuda:
        return _cpu.gather_reduce(src, inv_map, weight, addend, addend_scale)
    device = _lib.require_device(src, inv_map, weight, addend, addend_scale)
    n_out, top_k = inv_map.shape
    hidden = src.shape[-1]
    out = torch.empty((n_out, hidden), device=device, dtype=src.dtype)
    if n_out == 0 or hidden == 0:
        return out
    src = src.contiguous()
    if weight is not None:
        weight = weight.to(src.dtype).contiguous()
    inv_map = inv_map.long().contiguous()
    if addend is not None:
        if addend.shape != out.shape or addend.dtype != src.dtype:
            raise ValueError(f"addend must be {tuple(out.shape)} {src.dtype}, got {tuple(addend.shape)} {addend.dtype}")
        if addend.stride(-1) != 1:
            addend = addend.contiguous()
        if addend_scale is not None:
            addend_scale = addend_scale.reshape(-1).to(src.dtype).contiguous()
            if addend_scale.shape[0] != n_out:
                raise ValueError(f"addend_scale must hold {n_out} values, got {addend_scale.shape[0]}")
    elif addend_scale is not None:
        raise ValueError("addend_scale without an addend")
    with _lib.on_device(device):
        _lib.call("hmoe_gather_reduce_add", _lib.ptr(src), _lib.ptr(weight), _lib.ptr(inv_map), n_out, top_k,
                  src.shape[0], hidden, _lib.dtype_id(src.dtype), _lib.ptr(addend),
                  addend.stride(0) if addend is not None else 0, _lib.ptr(addend_scale), _lib.ptr(out),
                  _lib.stream_ptr(device))
    return out


def padded_gather_reduce(src: torch.Tensor, inv_map: torch.Tensor, weight: torch.Tensor | None = None) -> torch.Tensor:
    """The reference keeps this name for its CPU twin (``moe_permute.py:115-120``); here it is the same operator (the
    kernel for device tensors, the padded gather-sum in fp32 for CPU tensors)."""
    return gather_reduce_rows(src, inv_map, weight)


def build_inv_map(sorted_token_idx: torch.Tensor, recv_N: int, width: int) -> torch.Tensor:
    """``inv_map[r, j]`` = the j-th sorted position whose recv token is ``r``, padded to ``width`` columns with the
    sentinel ``len(sorted_token_idx)``.  Auxiliary: the routing sort already returns this map, so the expert path
    never calls this; it serves callers holding only ``sorted_token_idx`` and is a handful of device-side torch ops
    with no host readback (stable argsort, counts, exclusive cumsum, one scatter)."""
    device = sorted_token_idx.device
    token_of = sorted_token_idx.to(torch.int64)
    rows = token_of.numel()
    result = token_of.new_full((recv_N, width), rows)  # every slot the sentinel until a row claims it
    if rows:
        # sorted positions grouped by token, ascending inside a token (stable), then each position's rank inside its
        # token: its index in the grouped order minus the index at which its token's run begins
        by_token = torch.argsort(token_of, stable=True)
        owner = token_of[by_token]
        # torch.bincount sizes its output from the largest index and reads it back to the host; this one does not
        per_token = sync_free_bincount(token_of, recv_N, dtype=torch.int64)
        run_start = per_token.cumsum(0) - per_token
        rank = torch.arange(rows, device=device) - run_start[owner]
        result[owner, rank] = by_token
    return result


class MoEGatherPermute(torch.autograd.Function):
    """The permute by expert: row j of the result is ``tokens[sorted_token_idx[j]]``.  Backward sums, per token, the
    gradient rows of its sorted positions (``inv_map``) in fp32 without atomics."""

    @staticmethod
    def forward(ctx, tokens: torch.Tensor, sorted_token_idx: torch.Tensor, inv_map: torch.Tensor):
        ctx.save_for_backward(inv_map)
        return _gather_rows(tokens, sorted_token_idx)

    @staticmethod
    def backward(ctx, grad_sorted):
        (inv_map,) = ctx.saved_tensors
        return gather_reduce_rows(grad_sorted, inv_map), None, None


class MoEWeightedUnpermute(torch.autograd.Function):
    """``out[r] = sum_k w[j] * expert_out[j]`` for ``j = inv_map[r, k]``, the weighted rows summed in fp32 without an
    intermediate rounding.  ``expert_out`` is saved only when ``weights`` needs a gradient, the one gradient that
    reads it."""

    @staticmethod
    def forward(ctx, expert_out, weights, sorted_token_idx, inv_map):
        rows, gates = expert_out.contiguous(), weights.contiguous()
        ctx.weight_grad = bool(ctx.needs_input_grad[1])
        # the rows are read again only by the gate weights' gradient: kept only when that gradient is wanted
        ctx.save_for_backward(rows if ctx.weight_grad else None, gates, sorted_token_idx.contiguous())
        return gather_reduce_rows(rows, inv_map, gates)

    @staticmethod
    def backward(ctx, grad_out):
        expert_out, weights, sorted_token_idx = ctx.saved_tensors
        grad_expert, grad_weights = _unpermute_backward(grad_out, expert_out, weights, sorted_token_idx,
                                                        ctx.weight_grad)
        return grad_expert, grad_weights, None, None


def _unpermute_backward(grad_out, expert_out, weights, sorted_token_idx, weight_grad: bool):
    """``(w[j] * grad_out[tok[j]], <grad_out[tok[j]], expert_out[j]>)``; the second only when ``weight_grad``."""
    if not grad_out.is_cuda:
        return _cpu.unpermute_backward(grad_out, expert_out, weights, sorted_token_idx, weight_grad)
    device = _lib.require_device(grad_out, weights, sorted_token_idx)
    n_sorted, hidden = sorted_token_idx.shape[0], grad_out.shape[-1]
    # Under EP the gradient arrives as a row-strided view of the padded transport buffer, read in place.
    if grad_out.stride(-1) != 1:
        grad_out = grad_out.contiguous()
    grad_expert = torch.empty((n_sorted, hidden), device=device, dtype=grad_out.dtype)
    grad_weights = torch.empty(n_sorted if weight_grad else 0, device=device, dtype=torch.float32)
    if n_sorted:
        w = weights if weights.dtype == grad_out.dtype else weights.to(grad_out.dtype)
        y = None
        if weight_grad:
            y = expert_out if expert_out.dtype == grad_out.dtype else expert_out.to(grad_out.dtype)
        with _lib.on_device(device):
            _lib.call("hmoe_unpermute_bwd", _lib.ptr(grad_out), grad_out.stride(0), _lib.ptr(y), _lib.ptr(w),
                      _lib.ptr(sorted_token_idx), n_sorted, hidden, _lib.dtype_id(grad_out.dtype),
                      _lib.ptr(grad_expert), _lib.ptr(grad_weights) if weight_grad else None,
                      _lib.stream_ptr(device))
    return grad_expert, grad_weights.to(weights.dtype) if weight_grad else None


class MoEWeightedUnpermuteAdd(torch.autograd.Function):
    """``MoEWeightedUnpermute.apply(expert_out, weights, sorted_token_idx, inv_map) + scale[:, None] * addend`` in the
    combine's own pass (``scale`` may be None): the routed output plus the shared expert's, which the reference adds
    as a separate tensor operation (``expert_parallel/layer.py:270-299``; Qwen3.5's sigmoid gate on the shared expert,
    ``families/qwen3_5.py:41-42``).  The forward rounds where those operations round, so it returns their bits; the
    gradients are theirs as well, except that the gradient of ``scale`` is a dot product accumulated in fp32 and
    rounded once where autograd would round every product first."""

    @staticmethod
    def forward(ctx, expert_out, weights, sorted_token_idx, inv_map, addend, scale):
        expert_out, weights = expert_out.contiguous(), weights.contiguous()
        ctx.weight_grad = ctx.needs_input_grad[1]
        ctx.scaled = scale is not None
        ctx.scale_shape = scale.shape if ctx.scaled else None
        ctx.save_for_backward(expert_out if ctx.weight_grad else None, weights, sorted_token_idx.contiguous(),
                              addend if ctx.scaled and ctx.needs_input_grad[5] else None, scale)
        return gather_reduce_rows(expert_out, inv_map, weights, addend=addend, addend_scale=scale)

    @staticmethod
    def backward(ctx, grad_out):
        expert_out, weights, sorted_token_idx, addend, scale = ctx.saved_tensors
        grad_expert, grad_weights = _unpermute_backward(grad_out, expert_out, weights, sorted_token_idx,
                                                        ctx.weight_grad)
        grad_addend = grad_scale = None
        if not ctx.scaled:
            grad_addend = grad_out if ctx.needs_input_grad[4] else None
        elif ctx.needs_input_grad[4] or ctx.needs_input_grad[5]:
            # the same kernel with every row its own token: scale[r] * grad_out[r] and <grad_out[r], addend[r]>
            rows = torch.arange(grad_out.shape[0], device=grad_out.device)
            want_scale = ctx.needs_input_grad[5]
            grad_addend, grad_scale = _unpermute_backward(grad_out, addend, scale.reshape(-1), rows, want_scale)
            if want_scale:
                grad_scale = grad_scale.to(scale.dtype).view(ctx.scale_shape)
        return grad_expert, grad_weights, None, None, grad_addend, grad_scale


def expert_bias_grad(grad_out: torch.Tensor, eids: torch.Tensor, num_experts: int) -> torch.Tensor:
    """``[num_experts, width]``: per expert, the sum of the rows of ``grad_out`` that belong to it (``eids`` sorted),
    accumulated in fp32 in a fixed order and rounded once; an expert without rows gets exact zeros.  What the
    reference computes as ``onehot(eids)^T @ grad_out`` (``moe_permute.py:202-208``)."""
    if not grad_out.is_cuda:
        return _cpu.expert_bias_grad(grad_out, eids, num_experts)
    device = _lib.require_device(grad_out, eids)
    grad_out = grad_out.contiguous()
    eids = eids.long().contiguous()
    grad_bias = torch.empty((num_experts, grad_out.shape[1]), dtype=grad_out.dtype, device=device)
    lib = _lib.load()
    ws_bytes = lib.hmoe_expert_colsum_workspace_bytes(grad_out.shape[0], grad_out.shape[1], num_experts)
    workspace = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=device)
    with _lib.on_device(device):
        _lib.call("hmoe_expert_colsum", _lib.ptr(grad_out), _lib.ptr(eids), grad_out.shape[0], grad_out.shape[1],
                  num_experts, _lib.dtype_id(grad_out.dtype), _lib.ptr(grad_bias), _lib.ptr(workspace),
                  _lib.stream_ptr(device))
    return grad_bias


class MoEExpertBiasGather(torch.autograd.Function):
    """``bias[eids]`` to expert-sorted tokens; ``grad_bias`` is the per-expert column sum of the incoming gradient,
    accumulated in fp32 in row order (no atomics).  ``eids`` must be non-decreasing, as the routing sort emits them."""

    @staticmethod
    def forward(ctx, bias: torch.Tensor, eids: torch.Tensor):
        ctx.save_for_backward(eids)
        ctx.num_experts = bias.shape[0]
        return _gather_rows(bias, eids)

    @staticmethod
    def backward(ctx, grad_out):
        (eids,) = ctx.saved_tensors
        return expert_bias_grad(grad_out, eids, ctx.num_experts), None


def warm_permute_kernels(num_tokens: int, hidden: int, top_k: int, device: torch.device, dtype: torch.dtype) -> None:
    """Ahead-of-time binaries need no warm-up; kept for API parity (``moe_permute.py:211-227``)."""
    _lib.load()
