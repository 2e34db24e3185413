"""Per-expert load counting for bias-update balancing: the part of the reference's balancing state that sits on the
expert path.

Mirrors ``halo/distributed/expert_parallel/moe_layer/balancing_bias.py:200-207`` (``_record_expert_load``) and the
token-weight scope of ``halo/models/moe/balancing.py:253-274``.  The bias itself (adoption of a family's native slot,
the sign update, its checkpointing) belongs to the trainer side and is not part of this package: a caller that runs
bias-update balancing attaches ``balancing_biases`` to the layer, and from then on every training forward adds its
selection counts to ``expert_load_counter`` with the sync-free histogram kernel.
"""

from __future__ import annotations

from collections.abc import Iterator
from contextlib import contextmanager
from contextvars import ContextVar

import torch

from halo_amd.kernels.histogram import accumulate_bincount

BALANCING_BIASES_ATTR = "balancing_biases"

class _LoadWeightScope:
    """The per-token load weights of the innermost open :func:`expert_load_token_weights` block of this context (a
    thread or an asyncio task keeps its own), as a stack so that blocks nest."""

    _stack: ContextVar[tuple] = ContextVar("halo_amd_expert_load_weights", default=())

    @classmethod
    def current(cls) -> torch.Tensor | None:
        stack = cls._stack.get()
        return stack[-1] if stack else None

    @classmethod
    @contextmanager
    def opened(cls, weights: torch.Tensor | None) -> Iterator[None]:
        restore = cls._stack.set(cls._stack.get() + (weights,))
        try:
            yield
        finally:
            cls._stack.reset(restore)


def expert_load_token_weights(weights: torch.Tensor | None):
    """A context manager: inside it, token ``i`` of every forward counts ``weights[i]`` times toward expert load (a
    packed row that computes a shared prefix once for several examples).  None switches the weighting off for the
    block.  Same contract as ``halo/models/moe/balancing.py:253-262`` of the reference."""
    return _LoadWeightScope.opened(weights)


def resolve_expert_load_weights(indices: torch.Tensor) -> torch.Tensor | None:
    """One weight per routed slot of ``indices [..., top_k]`` (each token's weight repeated over its picks), or None
    when no weighting block is open.  The weights must name exactly the tokens of this forward
    (``balancing.py:265-274`` of the reference, whose message this raises)."""
    per_token = _LoadWeightScope.current()
    if per_token is None:
        return None
    token_shape = indices.shape[:-1]
    routed_tokens = 1
    for extent in token_shape:
        routed_tokens *= int(extent)
    if per_token.numel() != routed_tokens:
        raise ValueError(f"expert-load token weights cover {per_token.numel()} tokens but the router selected for "
                         f"{routed_tokens}: the weights do not describe this forward.")
    per_slot = per_token.to(device=indices.device).reshape(*token_shape, 1)
    return per_slot.expand(*token_shape, indices.shape[-1])


def counts_toward_expert_load() -> bool:
    """A grad-enabled pass counts; a frozen reference forward would skew the balance.  (The reference also tells a
    checkpoint's recomputation from its original pass; this package runs no recompute scopes.)"""
    return torch.is_grad_enabled()


class ExpertLoadMixin:
    """``expert_load_counter`` (fp32 ``[num_experts]``, None until the first counted forward) on a MoE layer."""

    num_experts: int
    training: bool
    expert_load_counter: torch.Tensor | None = None

    def _balancing_attached(self) -> bool:
        return getattr(self, BALANCING_BIASES_ATTR, None) is not None

    def _record_expert_load(self, indices: torch.Tensor) -> None:
        """Called once per forward with the router's picks.  When bias-update balancing is attached to the layer, the
        layer is in training mode and the pass counts (:func:`counts_toward_expert_load`), the picks are histogrammed
        on the device (no host readback) and added into ``expert_load_counter``
        (``moe_layer/balancing_bias.py:200-207`` of the reference)."""
        counted = self._balancing_attached() and self.training and counts_toward_expert_load()
        if not counted:
            return
        slot_weights = resolve_expert_load_weights(indices)
        with torch.no_grad():
            self.expert_load_counter = accumulate_bincount(self.expert_load_counter, indices, self.num_experts,
                                                           weights=slot_weights)
