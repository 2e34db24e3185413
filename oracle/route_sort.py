"""Oracle (test infrastructure): expert-sorted routing in numpy.

Follows the torch construction the reference runs off CUDA, ``halo/kernels/moe_route_sort.py:201-227``
(``_argsort_routing``), and ``halo/kernels/moe_permute.py:75-89`` (``build_inv_map``).  Slot = ``row * top_k + k``;
a slot is valid when ``0 <= expert < num_local_experts``; the valid slots are ordered by expert, then by slot.
"""

from __future__ import annotations

import numpy as np

RECEIVE_COUNTS_DISAGREE = "DeepEP receive counts disagree with the received expert ids"
NONLOCAL_EXPERT_ID_MESSAGE = (
    "An expert id outside the local experts at ep_size 1, where the routing hands over only local ids"
)


def build_inv_map(sorted_token_idx: np.ndarray, n_rows: int, width: int) -> np.ndarray:
    """``inv_map[r, j]`` = the j-th (ascending) sorted position whose token is ``r``; rows shorter than ``width`` are
    padded with the sentinel ``len(sorted_token_idx)``.  (``halo/kernels/moe_permute.py:75-89``.)"""
    sorted_token_idx = np.asarray(sorted_token_idx, dtype=np.int64)
    n_sorted = sorted_token_idx.shape[0]
    inv_map = np.full((n_rows, width), n_sorted, dtype=np.int64)
    if n_sorted == 0:
        return inv_map
    order = np.argsort(sorted_token_idx, kind="stable")
    tokens = sorted_token_idx[order]
    counts = np.bincount(sorted_token_idx, minlength=n_rows)
    starts = np.cumsum(counts) - counts
    column = np.arange(n_sorted) - starts[tokens]
    inv_map[tokens, column] = order
    return inv_map


def argsort_routing(experts: np.ndarray, weights: np.ndarray, num_local_experts: int, counts=None):
    """Returns ``(sorted_token_idx i64[R], sorted_weights[R], sorted_expert_ids[R], offs i32[E], inv_map i64[N,k],
    dest i32[N*k])``.

    The first five are the reference's outputs (``halo/kernels/moe_route_sort.py:201-227``); ``dest`` is the tensor
    its counting sort saves for backward (``:119, 181-189``): each slot's sorted position, ``R`` for a dropped slot.
    ``counts`` (host-side per-expert slot counts) only sizes the outputs through its sum (``:141``); a sum that
    disagrees with the ids raises, as does an id outside the range when ``counts`` is None (``:209-216``).
    """
    experts = np.asarray(experts)
    weights = np.asarray(weights)
    if counts is not None and len(counts) != num_local_experts:
        raise ValueError(f"{len(counts)} receive counts for {num_local_experts} local experts")
    n_rows, top_k = experts.shape
    flat_experts = experts.reshape(-1)
    flat_weights = weights.reshape(-1)
    valid = (flat_experts >= 0) & (flat_experts < num_local_experts)
    n_valid = int(valid.sum())
    if counts is None:
        if n_valid != flat_experts.size:
            raise RuntimeError(NONLOCAL_EXPERT_ID_MESSAGE)
    elif n_valid != int(sum(counts)):
        raise RuntimeError(RECEIVE_COUNTS_DISAGREE)
    slots = np.nonzero(valid)[0]
    order = slots[np.argsort(flat_experts[slots], kind="stable")]
    sorted_expert_ids = flat_experts[order].astype(experts.dtype)
    sorted_token_idx = (order // max(top_k, 1)).astype(np.int64)
    sorted_weights = flat_weights[order]
    offs = np.cumsum(np.bincount(sorted_expert_ids.astype(np.int64), minlength=num_local_experts)).astype(np.int32)
    inv_map = build_inv_map(sorted_token_idx, n_rows, top_k)
    dest = np.full(n_rows * top_k, n_valid, dtype=np.int32)
    dest[order] = np.arange(n_valid, dtype=np.int32)
    return sorted_token_idx, sorted_weights, sorted_expert_ids, offs, inv_map, dest


def sort_backward(sorted_weights_grad: np.ndarray, dest: np.ndarray, shape) -> np.ndarray:
    """Gate-weight gradient: each slot reads its sorted position's gradient, a dropped slot reads zero
    (``halo/kernels/moe_route_sort.py:181-189``)."""
    padded = np.concatenate([np.asarray(sorted_weights_grad), np.zeros(1, dtype=sorted_weights_grad.dtype)])
    return padded[dest].reshape(shape)


def bincount(indices: np.ndarray, size: int, dtype=np.float32, weights=None) -> np.ndarray:
    """``halo/kernels/histogram.py:9-18``: histogram of in-range indices, optionally weighted."""
    flat = np.asarray(indices).reshape(-1).astype(np.int64)
    out = np.zeros(size, dtype=dtype)
    np.add.at(out, flat, 1 if weights is None else np.asarray(weights).reshape(-1).astype(dtype))
    return out
