"""Grouped LoRA on the expert weights, the part of it that lies on one GPU's compute path: a stored expert weight
``W [E, K, N]`` gains ``<name>_lora_A [E, K, r]`` and ``<name>_lora_B [E, r, N]``, its base is frozen, and the expert
projection becomes ``x @ W + scaling * (dropout(x) @ A) @ B`` with both adapter products on the grouped GEMM kernels.

Mirrors the reference's recipe (``halo/models/moe/expert_lora_spec.py:24-41``: ``scaling = alpha / r``, or
``alpha / sqrt(r)`` with rsLoRA; which weight roots count as gate / up / down ``:9-16``), its adapter construction
(``halo/distributed/expert_parallel/moe_layer/expert_lora.py:40-72``: A uniform in ``+-1/sqrt(K)``, B zero, the rank a
multiple of 8) and the projection of ``moe_layer/compute.py:283-294``.  Gathering and loading adapter checkpoints across
the ranks of an expert-parallel group (``expert_lora.py:92-172``) is collective work and not part of this build.
"""

from __future__ import annotations

import contextlib
import math
from dataclasses import dataclass, field

import torch
import torch.nn as nn

from halo_amd.kernels.grouped_mm import GROUPED_MM_STRIDE_ALIGNMENT_BYTES

# which of the FFN's projections each stored weight root carries
LORA_PROJECTION_COVERAGE: dict[str, frozenset[str]] = {
    "gate_up_proj": frozenset({"gate", "up"}),
    "gate_proj": frozenset({"gate"}),
    "gate_proj_gmm": frozenset({"gate"}),
    "up_proj": frozenset({"up"}),
    "up_proj_gmm": frozenset({"up"}),
    "down_proj": frozenset({"down"}),
}
EXPERT_PROJECTIONS: frozenset[str] = frozenset({"gate", "up", "down"})
EXPERT_LORA_SUFFIXES: tuple[str, str] = ("_lora_A", "_lora_B")
# The adapter products run in the activation dtype, bf16 at the narrowest, and the rank is a row length of one of
# their operands: it has to span whole 16-byte rows.
EXPERT_LORA_RANK_MULTIPLE = GROUPED_MM_STRIDE_ALIGNMENT_BYTES // 2


@dataclass(frozen=True)
class ExpertLoraSpec:
    r: int
    alpha: float
    dropout: float = 0.0
    projections: frozenset[str] = field(default_factory=lambda: EXPERT_PROJECTIONS)
    use_rslora: bool = False

    @property
    def scaling(self) -> float:
        return self.alpha / (math.sqrt(self.r) if self.use_rslora else self.r)

    def adapts(self, weight_attr: str) -> bool:
        return bool(LORA_PROJECTION_COVERAGE.get(weight_attr, frozenset()) & self.projections)


def expert_lora_delta(lora_a: torch.Tensor, lora_b: torch.Tensor, scaling: float) -> torch.Tensor:
    """``scaling * A @ B`` per expert in fp32: what merging the adapters adds to the weight."""
    return torch.bmm(lora_a.float(), lora_b.float()) * scaling


def init_expert_lora(layer, spec: ExpertLoraSpec | None) -> None:
    """Builds the adapters the spec asks for on ``layer``'s 3-D expert weights (initial delta zero) and freezes those
    weights.  A rank that is not a multiple of 8 is refused with the reference's wording."""
    layer._expert_lora_attrs = frozenset()
    layer._expert_adapters_enabled = True
    if spec is None:
        return
    layer.expert_lora_scaling = spec.scaling
    layer.expert_lora_dropout = nn.Dropout(spec.dropout) if spec.dropout > 0 else nn.Identity()
    taken = []
    for name, weight in layer.expert_named_params():
        if not isinstance(weight, torch.Tensor) or weight.dim() != 3 or not spec.adapts(name):
            continue
        if spec.r % EXPERT_LORA_RANK_MULTIPLE:
            raise ValueError(
                f"lora_r={spec.r} cannot adapt the expert weight {name!r}: the grouped GEMM contracts over the "
                f"adapter's rank dimension and reads it as a stride spanning a multiple of "
                f"{GROUPED_MM_STRIDE_ALIGNMENT_BYTES} bytes at the bf16 the adapters run in at the narrowest — "
                f"use a multiple of {EXPERT_LORA_RANK_MULTIPLE}."
            )
        experts, k, n = weight.shape
        bound = 1.0 / math.sqrt(k)  # PEFT's kaiming_uniform_(a=sqrt(5)) on a [r, K] matrix: the fan-in is K, not K*r
        lora_a = torch.empty(experts, k, spec.r, dtype=weight.dtype, device=weight.device).uniform_(-bound, bound)
        lora_b = torch.zeros(experts, spec.r, n, dtype=weight.dtype, device=weight.device)
        setattr(layer, name + EXPERT_LORA_SUFFIXES[0], nn.Parameter(lora_a))
        setattr(layer, name + EXPERT_LORA_SUFFIXES[1], nn.Parameter(lora_b))
        weight.requires_grad_(False)
        taken.append(name)
    layer._expert_lora_attrs = frozenset(taken)


def expert_lora_layers(model: nn.Module) -> list:
    return [(name, m) for name, m in model.named_modules() if getattr(m, "has_expert_lora", False)]


def model_has_expert_lora(model: nn.Module) -> bool:
    return bool(expert_lora_layers(model))


@contextlib.contextmanager
def disable_expert_adapters(model: nn.Module):
    """The expert half of ``PeftModel.disable_adapter()``: inside the block every layer of ``model`` computes with its
    frozen base weights alone."""
    layers = [layer for _, layer in expert_lora_layers(model)]
    before = [layer._expert_adapters_enabled for layer in layers]
    try:
        for layer in layers:
            layer._expert_adapters_enabled = False
        yield
    finally:
        for layer, state in zip(layers, before):
            layer._expert_adapters_enabled = state
