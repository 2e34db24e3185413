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

_expert_load_weights: ContextVar[torch.Tensor | None] = ContextVar("expert_load_weights", default=None)


@contextmanager
def expert_load_token_weights(weights: torch.Tensor | None) -> Iterator[None]:
    """Inside the block, token ``i`` of every forward counts ``weights[i]`` times toward expert load (a packed row
    that computes a shared prefix once for several examples)."""
    token = _expert_load_weights.set(weights)
    try:
        yield
    finally:
        _expert_load_weights.reset(token)


def resolve_expert_load_weights(indices: torch.Tensor) -> torch.Tensor | None:
    """The active token weights broadcast over ``indices [..., top_k]``, None outside a weighting scope."""
    weights = _expert_load_weights.get()
    if weights is None:
        return None
    tokens = indices[..., 0].numel()
    if weights.numel() != tokens:
        raise ValueError(f"expert-load token weights cover {weights.numel()} tokens but the router selected for "
                         f"{tokens}: the weights do not describe this forward.")
    return weights.to(indices.device).reshape(indices.shape[:-1]).unsqueeze(-1).expand_as(indices)


def counts_toward_expert_load() -> bool:
    """A grad-enabled pass counts; a frozen reference forward would skew the balance.  (The reference also tells a
    checkpoint's recomputation from its original pass; this package runs no recompute scopes.)"""
    return torch.is_grad_enabled()


class ExpertLoadMixin:
    """``expert_load_counter`` (fp32 ``[num_experts]``, None until the first counted forward) on a MoE layer."""

    num_experts: int
    training: bool
    expert_load_counter: torch.Tensor | None = None

    def _record_expert_load(self, indices: torch.Tensor) -> None:
        """Adds this forward's per-expert selection counts while training, once bias-update balancing is attached."""
        if getattr(self, BALANCING_BIASES_ATTR, None) is None or not self.training or not counts_toward_expert_load():
            return
        with torch.no_grad():
            self.expert_load_counter = accumulate_bincount(
                self.expert_load_counter, indices, self.num_experts, weights=resolve_expert_load_weights(indices))
