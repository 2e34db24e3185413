"""Expert-sorted routing for the grouped-GEMM MoE compute: a stable counting sort in three HIP launches, sized by the
dispatch's host-side receive counts or, at ``ep_size`` 1, by every slot.  Nothing is read back from the device.

Mirrors the reference's ``halo/kernels/moe_route_sort.py`` (``sort_routing_by_expert`` ``:230-243``,
``_CountingSort`` ``:128-189``); the kernels are ``csrc/route_sort.hip``.
"""

from __future__ import annotations

import torch

from halo_amd import _lib

RECEIVE_COUNTS_DISAGREE = "DeepEP receive counts disagree with the received expert ids"
# At ep_size 1 no dispatch pads, so an id outside the local range came from the routing itself.
NONLOCAL_EXPERT_ID_MESSAGE = (
    "An expert id outside the local experts at ep_size 1, where the routing hands over only local ids"
)

_ID_BYTES = {torch.int64: 8, torch.int32: 4}


def counting_sort_raw(experts: torch.Tensor, weights: torch.Tensor, num_local_experts: int, n_valid: int):
    """The three launches.  Returns ``(sorted_token_idx, sorted_weights, sorted_expert_ids, offs, inv_map, dest, ok)``;
    ``ok`` is an int32 device flag, 1 when the number of local slots equals ``n_valid``.  With ``ok == 0`` the sorted
    outputs are left unwritten."""
    device = _lib.require_device(experts, weights)
    if experts.dim() != 2 or weights.shape != experts.shape:
        raise ValueError(f"experts and weights must both be [rows, top_k], got {tuple(experts.shape)} and "
                         f"{tuple(weights.shape)}")
    if experts.dtype not in _ID_BYTES:
        raise TypeError(f"expert ids must be int64 or int32, got {experts.dtype}")
    if weights.element_size() not in (2, 4, 8):
        raise TypeError(f"unsupported gate-weight dtype {weights.dtype}")
    n_rows, top_k = experts.shape
    experts, weights = experts.contiguous(), weights.contiguous()
    lib = _lib.load()
    ws_bytes = lib.hmoe_route_sort_workspace_bytes(n_rows, top_k, num_local_experts)
    if ws_bytes < 0:
        raise ValueError(f"bad routing shape: rows={n_rows} top_k={top_k} experts={num_local_experts}")
    workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=device)
    offs = torch.empty(num_local_experts, dtype=torch.int32, device=device)
    ok = torch.empty(1, dtype=torch.int32, device=device)
    dest = torch.empty(n_rows * top_k, dtype=torch.int32, device=device)
    sorted_token_idx = torch.empty(n_valid, dtype=torch.long, device=device)
    sorted_weights = torch.empty(n_valid, dtype=weights.dtype, device=device)
    sorted_expert_ids = torch.empty(n_valid, dtype=experts.dtype, device=device)
    inv_map = torch.empty((n_rows, top_k), dtype=torch.long, device=device)
    with _lib.on_device(device):
        _lib.call(
            "hmoe_route_sort", _lib.ptr(experts), _ID_BYTES[experts.dtype], _lib.ptr(weights), weights.element_size(),
            n_rows, top_k, num_local_experts, n_valid, _lib.ptr(sorted_token_idx), _lib.ptr(sorted_weights),
            _lib.ptr(sorted_expert_ids), _lib.ptr(offs), _lib.ptr(inv_map), _lib.ptr(dest), _lib.ptr(ok),
            _lib.ptr(workspace), _lib.stream_ptr(device),
        )
    return sorted_token_idx, sorted_weights, sorted_expert_ids, offs, inv_map, dest, ok


class _CountingSort(torch.autograd.Function):
    """Only the gate weights carry a gradient, each slot's read back at its sorted position."""

    @staticmethod
    def forward(ctx, weights: torch.Tensor, experts: torch.Tensor, num_local_experts: int,
                counts: tuple[int, ...] | None):
        n_rows, top_k = experts.shape
        n_valid = n_rows * top_k if counts is None else sum(counts)
        sorted_token_idx, sorted_weights, sorted_expert_ids, offs, inv_map, dest, ok = counting_sort_raw(
            experts, weights, num_local_experts, n_valid
        )
        # Device-side, no readback: a wrong total would have written past the outputs the counts sized.
        torch._assert_async(ok, NONLOCAL_EXPERT_ID_MESSAGE if counts is None else RECEIVE_COUNTS_DISAGREE)
        ctx.save_for_backward(dest)
        ctx.weights_shape = weights.shape
        ctx.n_valid = n_valid
        ctx.mark_non_differentiable(sorted_token_idx, sorted_expert_ids, offs, inv_map)
        # The integer outputs take no gradient; materialized, each would cost a zero-fill in every backward.
        ctx.set_materialize_grads(False)
        return sorted_token_idx, sorted_weights, sorted_expert_ids, offs, inv_map

    @staticmethod
    def backward(ctx, _token_grad, sorted_weights_grad, _expert_grad, _offs_grad, _inv_map_grad):
        if sorted_weights_grad is None:
            return None, None, None, None
        (dest,) = ctx.saved_tensors
        grad_sorted = sorted_weights_grad.contiguous()
        grad = torch.empty(ctx.weights_shape, dtype=grad_sorted.dtype, device=grad_sorted.device)
        with _lib.on_device(grad.device):
            _lib.call("hmoe_route_sort_bwd", _lib.ptr(grad_sorted), _lib.ptr(dest), dest.numel(), ctx.n_valid,
                      grad_sorted.element_size(), _lib.ptr(grad), _lib.stream_ptr(grad.device))
        return grad, None, None, None


def sort_routing_by_expert(
    experts: torch.Tensor, weights: torch.Tensor, num_local_experts: int, counts: tuple[int, ...] | None
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Each local expert's slots in slot order, ids outside ``[0, num_local_experts)`` (the dispatch's ``-1``)
    dropped: ``(sorted_token_idx i64[R], sorted_weights[R], sorted_expert_ids[R], offs i32[E], inv_map i64[N, k])``.
    ``counts[e]`` is the host-side slot count of expert ``e``, None when every id is local; a size that disagrees with
    the ids trips a device-side assert.  Same signature and outputs as the reference's
    ``halo.kernels.moe_route_sort.sort_routing_by_expert``."""
    if counts is not None and len(counts) != num_local_experts:
        raise ValueError(f"{len(counts)} receive counts for {num_local_experts} local experts")
    return _CountingSort.apply(weights, experts, num_local_experts, counts)


def warm_route_sort_kernels(top_k: int, num_local_experts: int, device: torch.device) -> None:
    """The kernels are compiled ahead of time and one binary serves every receive size; kept for API parity with the
    reference (``moe_route_sort.py:246-254``), it only forces the library to load."""
    _lib.load()
