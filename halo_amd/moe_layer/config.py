"""Expert-parallel configuration as the MoE block reads it, in its one-GPU shapes.

Mirrors the attributes the reference's layer takes off its ``EPConfig``
(``halo/distributed/expert_parallel/config.py:28-161``; read at ``moe_layer/layer.py:122-152``) and the
single-process shape of ``tests/common/parallelism.py:130-146``.  No process group is ever created here: ``ep_size``
above 1 only describes which slice of the experts this GPU holds, for running one GPU's share of an EP layer on rows
a dispatch has already delivered.
"""

from __future__ import annotations

from dataclasses import dataclass


@dataclass
class EPConfig:
    ep_size: int = 1
    ep_rank: int = 0
    expert_tp_size: int = 1
    expert_tp_rank: int = 0
    expert_tp_group: object | None = None
    use_grouped_gemm: bool = True
    fp32_router: bool = False
    fp32_experts: bool = False
    experts_fsdp_managed: bool = False
    num_experts: int | None = None
    experts_per_rank: int | None = None
    expert_start_idx: int | None = None
    expert_end_idx: int | None = None
    expert_lora: object | None = None  # an ExpertLoraSpec (moe_layer/expert_lora.py): grouped adapters on the experts

    def __post_init__(self):
        if self.expert_tp_size != 1:
            raise NotImplementedError("expert tensor parallelism needs a process group; this build runs one GPU")
        if not 0 <= self.ep_rank < self.ep_size:
            raise ValueError(f"ep_rank {self.ep_rank} outside ep_size {self.ep_size}")
        if self.num_experts is not None:
            self.finalize_expert_assignment(self.num_experts)

    @property
    def grouped_gemm_enabled(self) -> bool:
        """The grouped kernels are this build's only expert compute."""
        return self.use_grouped_gemm

    def finalize_expert_assignment(self, num_experts: int) -> None:
        """Contiguous equal ranges: rank ``r`` owns ``[r * E/ep, (r+1) * E/ep)``."""
        if num_experts % self.ep_size:
            raise ValueError(f"{num_experts} experts do not divide over ep_size {self.ep_size}")
        self.num_experts = num_experts
        self.experts_per_rank = num_experts // self.ep_size
        self.expert_start_idx = self.ep_rank * self.experts_per_rank
        self.expert_end_idx = self.expert_start_idx + self.experts_per_rank


def single_process_ep_config(num_experts: int | None = None, **overrides) -> EPConfig:
    """Every expert on this GPU, nothing dispatched."""
    return EPConfig(**{"ep_size": 1, "num_experts": num_experts, **overrides})


@dataclass(frozen=True)
class MoEFamilySpec:
    """The layout facts of a family the block reads: where the HF block keeps its experts and shared expert, and how
    the expert weights are stored at run time (``fused`` ``gate_up_proj``, ``separate_glu`` halves, or gpt-oss's
    ``interleaved_glu`` with biases)."""

    name: str
    expert_layout: str = "fused"
    experts_container_attrs: tuple[str, ...] = ("experts",)
    shared_expert_attrs: tuple[str, ...] = ()
    expert_weight_roots: tuple[str, ...] = ("gate_up_proj", "gate_proj", "up_proj", "down_proj")


QWEN3 = MoEFamilySpec("qwen3_moe", expert_layout="separate_glu")
QWEN3_5 = MoEFamilySpec("qwen3_5_moe", expert_layout="fused", shared_expert_attrs=("shared_expert",))
# Gemma-4: the wrapped HF module is the expert container itself; its router is a sibling module of the decoder layer
GEMMA4 = MoEFamilySpec("gemma4", expert_layout="fused", experts_container_attrs=())
GPT_OSS = MoEFamilySpec(
    "gpt_oss",
    expert_layout="interleaved_glu",
    expert_weight_roots=(
        "gate_up_proj", "gate_proj", "up_proj", "down_proj", "gate_up_proj_bias", "gate_proj_gmm", "up_proj_gmm",
        "gate_proj_gmm_bias", "up_proj_gmm_bias", "gate_proj_bias", "up_proj_bias", "down_proj_bias",
    ),
)
