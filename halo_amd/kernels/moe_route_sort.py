"""Expert-sorted routing for the grouped-GEMM MoE compute: a stable counting sort in three HIP launches, sized by the
dispatch's host-side receive counts or, at ``ep_size`` 1, by every slot.  Nothing is read back from the device.

Mirrors the reference's ``halo/kernels/moe_route_sort.py`` (``sort_routing_by_expert`` ``:230-243``,
``_CountingSort`` ``:128-189``); the kernels are ``csrc/route_sort.hip``.
"""

from __future__ import annotations

import torch

from halo_amd import _lib
from halo_amd.kernels import _cpu

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
    rows, k = experts.shape
    ids, gates = experts.contiguous(), weights.contiguous()
    ws_bytes = _lib.load().hmoe_route_sort_workspace_bytes(rows, k, num_local_experts)
    if ws_bytes < 0:
        raise ValueError(f"bad routing shape: rows={rows} top_k={k} experts={num_local_experts}")

    def buffer(shape, dtype):
        return torch.empty(shape, dtype=dtype, device=device)

    workspace = buffer(ws_bytes, torch.uint8)
    out = {
        "sorted_token_idx": buffer(n_valid, torch.int64),
        "sorted_weights": buffer(n_valid, gates.dtype),
        "sorted_expert_ids": buffer(n_valid, ids.dtype),
        "offs": buffer(num_local_experts, torch.int32),
        "inv_map": buffer((rows, k), torch.int64),
        "dest": buffer(rows * k, torch.int32),
        "ok": buffer(1, torch.int32),
    }
    with _lib.on_device(device):
        _lib.call("hmoe_route_sort", _lib.ptr(ids), _ID_BYTES[ids.dtype], _lib.ptr(gates), gates.element_size(), rows,
                  k, num_local_experts, n_valid, *(_lib.ptr(t) for t in out.values()), _lib.ptr(workspace),
                  _lib.stream_ptr(device))
    return tuple(out.values())


class _CountingSort(torch.autograd.Function):
    """Only the gate weights carry a gradient, each slot's read back at its sorted position."""

    @staticmethod
    def forward(ctx, weights: torch.Tensor, experts: torch.Tensor, num_local_experts: int,
                counts: tuple[int, ...] | None):
        n_valid = experts.numel() if counts is None else sum(counts)
        token_idx, gates, expert_ids, offs, inv_map, dest, ok = counting_sort_raw(experts, weights,
                                                                                   num_local_experts, n_valid)
        # Checked on the device, nothing read back: with a wrong total the sort leaves the outputs unwritten.
        torch._assert_async(ok, RECEIVE_COUNTS_DISAGREE if counts is not None else NONLOCAL_EXPERT_ID_MESSAGE)
        ctx.n_valid, ctx.weights_shape = n_valid, weights.shape
        ctx.save_for_backward(dest)
        # Only ``gates`` is differentiable; without materialised gradients backward is not handed a zero tensor for
        # each of the integer outputs.
        ctx.mark_non_differentiable(token_idx, expert_ids, offs, inv_map)
        ctx.set_materialize_grads(False)
        return token_idx, gates, expert_ids, offs, inv_map

    @staticmethod
    def backward(ctx, _token_grad, sorted_weights_grad, _expert_grad, _offs_grad, _inv_map_grad):
        if sorted_weights_grad is not None:
            (dest,) = ctx.saved_tensors
            grad_sorted = sorted_weights_grad.contiguous()
            grad = grad_sorted.new_empty(ctx.weights_shape)
            with _lib.on_device(grad.device):
                _lib.call("hmoe_route_sort_bwd", _lib.ptr(grad_sorted), _lib.ptr(dest), dest.numel(), ctx.n_valid,
                          grad_sorted.element_size(), _lib.ptr(grad), _lib.stream_ptr(grad.device))
            return grad, None, None, None
        return (None,) * 4


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
    if not experts.is_cuda:  # CPU tensors: a stable argsort, as the reference's _argsort_routing (:201-227)
        return _cpu.sort_routing(experts, weights, num_local_experts, counts, RECEIVE_COUNTS_DISAGREE,
                                 NONLOCAL_EXPERT_ID_MESSAGE)
    return _CountingSort.apply(weights, experts, num_local_experts, counts)


def warm_route_sort_kernels(top_k: int, num_local_experts: int, device: torch.device) -> None:
    """The kernels are compiled ahead of time and one binary serves every receive size; kept for API parity with the
    reference (``moe_route_sort.py:246-254``), it only forces the library to load."""
    _lib.load()
