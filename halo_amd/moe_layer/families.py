"""Per-family glue over :class:`EPMoELayerBase`: Qwen3 (gate and up stored apart), Qwen3.5 / Qwen3.6 (fused experts and
a sigmoid-gated shared expert), gpt-oss (interleaved fused experts with biases, clamped SwiGLU, logit-space router
bias) and Gemma-4 (the experts alone: the routing decision arrives with the call).

Mirrors the reference's ``halo/distributed/expert_parallel/families/qwen3.py``, ``qwen3_5.py``, ``gpt_oss.py`` and
``gemma4.py``.
"""

from __future__ import annotations

import torch
import torch.nn as nn

from halo_amd.kernels.fused_glu import GluCombine, fused_glu_enabled
from halo_amd.kernels.grouped_mm import bias_fusable, grouped_mm_bias
from halo_amd.kernels.moe_permute import MoEExpertBiasGather
from halo_amd.kernels.router import SOFTMAX_TOPK, fused_topk_gate
from halo_amd.moe_layer.config import GEMMA4, GPT_OSS, QWEN3, QWEN3_5
from halo_amd.moe_layer.layer import EPMoELayerBase, EPSharedExpertsMoELayerBase, sigmoid_row_gate


def split_interleaved_gate_up(interleaved: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """gpt-oss stores ``[g0, u0, g1, u1, ...]`` along the last axis (``halo/models/moe/expert_layout.py:87-88``)."""
    return interleaved[..., ::2], interleaved[..., 1::2]


class EPQwen3MoELayer(EPSharedExpertsMoELayerBase):
    """``Qwen3MoeSparseMoeBlock``: fused HF experts split into matmul-convention halves, three grouped GEMMs."""

    HF_MODULE_NAMES = ("Qwen3MoeSparseMoeBlock",)
    FAMILY = QWEN3
    # ``Qwen3MoeTopKRouter`` renormalises with no floor.
    _TOPK_WEIGHT_NORM_EPS = 0.0

    def _normalizes_topk(self) -> bool:
        """The router's configurable ``norm_topk_prob``, read live."""
        return bool(getattr(self.gate, "norm_topk_prob", True))


class EPQwen3_5MoELayer(EPSharedExpertsMoELayerBase):
    """``Qwen3_5MoeSparseMoeBlock``: fused ``gate_up_proj`` (two grouped GEMMs and the packed GLU), a router that
    always renormalises, and a shared expert scaled by ``sigmoid(x @ w_gate^T)``."""

    HF_MODULE_NAMES = ("Qwen3_5MoeSparseMoeBlock",)
    FAMILY = QWEN3_5
    _TOPK_WEIGHT_NORM_EPS = 0.0

    def _adopt_shared_experts(self, original_layer: nn.Module) -> None:
        super()._adopt_shared_experts(original_layer)
        self.shared_expert_gate = original_layer.shared_expert_gate

    def _shared_expert_parts(self, hidden_states: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor | None]:
        rows, _ = super()._shared_expert_parts(hidden_states)
        gate = getattr(self, "shared_expert_gate", None)
        if gate is None:
            return rows, None
        x = hidden_states.reshape(-1, hidden_states.shape[-1])
        # a [T, 1] projection is below the GEMM kernels' 16-byte row granularity: a kernel of its own
        return rows, sigmoid_row_gate(x, gate.weight)

    def replicated_named_params(self) -> list:
        extra = [] if getattr(self, "shared_expert_gate", None) is None else [
            (f"shared_expert_gate.{n}", p) for n, p in self.shared_expert_gate.named_parameters()]
        return super().replicated_named_params() + extra


class EPGptOssMoELayer(EPMoELayerBase):
    """``GptOssMLP``: the interleaved ``gate_up_proj`` is stored de-interleaved for the grouped GEMMs
    (``gate_proj_gmm`` / ``up_proj_gmm`` ``[E, H, F]``), each projection adds its expert bias through
    :class:`MoEExpertBiasGather`, the combine is the clamped SwiGLU ``(clamp(u)+1) * g' * sigmoid(alpha g')``, and the
    router picks on bias-inclusive logits then takes a softmax over the picks.  ``forward`` returns
    ``(out [B, S, H], logits)``."""

    HF_MODULE_NAMES = ("GptOssMLP",)
    FAMILY = GPT_OSS
    _ROUTER_ATTR = "router"

    def _adopt_expert_compute(self, original_layer: nn.Module, experts: nn.Module) -> None:
        self._gptoss_glu = GluCombine.gptoss(experts.alpha, experts.limit)
        self._fused_glu_mul = self._gptoss_glu

    def _adopt_expert_params(self, experts: nn.Module, weights_already_sharded: bool = False) -> None:
        self._require_fused_experts(experts)
        local = slice(*self._local_expert_range(weights_already_sharded))

        def own(tensor: torch.Tensor) -> nn.Parameter:  # this rank's experts, as a dense parameter of its own
            return nn.Parameter(tensor.contiguous().clone() if tensor.is_contiguous() else tensor.contiguous())

        # HF keeps gate and up interleaved column by column in one [E, H, 2F] weight (and one [E, 2F] bias); the
        # grouped GEMMs take them apart
        for source, suffix in (("gate_up_proj", ""), ("gate_up_proj_bias", "_bias")):
            packed = getattr(experts, source, None)
            if packed is None:
                continue
            gate_half, up_half = split_interleaved_gate_up(packed.data[local])
            setattr(self, f"gate_proj_gmm{suffix}", own(gate_half))
            setattr(self, f"up_proj_gmm{suffix}", own(up_half))
        for source in ("down_proj", "down_proj_bias"):
            tensor = getattr(experts, source, None)
            if tensor is not None:
                setattr(self, source, own(tensor.data[local]))

    @classmethod
    def from_weights(cls, *, alpha: float = 1.702, limit: float = 7.0, router_bias: torch.Tensor | None = None,
                     **kwargs):
        self = super().from_weights(**kwargs)
        self._gptoss_glu = GluCombine.gptoss(alpha, limit)
        self._fused_glu_mul = self._gptoss_glu
        if router_bias is not None:
            self.router.bias = nn.Parameter(router_bias)
        return self

    def _glu_combine_name(self) -> str:
        return self._gptoss_glu.name if fused_glu_enabled() else "eager"

    def forward(self, hidden_states: torch.Tensor, **kwargs) -> tuple[torch.Tensor, torch.Tensor]:
        shape = hidden_states.shape
        input_dtype = hidden_states.dtype
        flat = hidden_states.reshape(-1, shape[-1])
        logits = self._linear_router_logits(flat)
        experts, weights = fused_topk_gate(logits, self.top_k, mode=SOFTMAX_TOPK, normalize=False)
        result = self._dispatch_compute_combine(flat, experts, weights.float(), input_dtype)
        return result.view(shape), logits.to(input_dtype)

    def _gate_up_attrs(self) -> tuple[str, str]:
        return ("gate_proj_gmm", "up_proj_gmm") if hasattr(self, "gate_proj_gmm") else ("gate_proj", "up_proj")

    def _grouped_expert_ffn(self, sorted_tokens, offs, sorted_expert_ids, output_dtype):
        """Three grouped GEMMs (gate, up, down) on de-interleaved weights, each plus its expert bias."""
        def project(x, weight_attr):
            return self._grouped_proj_with_bias(x, weight_attr, offs, output_dtype, sorted_expert_ids)

        gate, up = self._project_gate_up(sorted_tokens, offs, output_dtype, sorted_expert_ids, project, with_bias=True)
        return project(self._gptoss_glu(gate, up).to(output_dtype), "down_proj")

    def _grouped_proj_with_bias(self, x, weight_attr, offs, out_dtype, eids):
        bias = getattr(self, f"{weight_attr}_bias", None)
        weight = getattr(self, weight_attr)
        if (bias is not None and getattr(self, "fuse_bias_into_gemm", True) and self._lowp_quant_format is None
                and not self._adapted(weight_attr)
                and isinstance(weight, torch.Tensor) and isinstance(x, torch.Tensor)):
            weight, bias_cast = weight.to(out_dtype), bias.to(out_dtype)
            if bias_fusable(x, weight, bias_cast):  # the projection and its bias in one kernel, the same bits
                return grouped_mm_bias(x, weight, bias_cast, offs=offs, eids=eids)
        if (bias is not None and getattr(self, "fuse_bias_into_gemm", True)
                and self._lowp_quant_format in ("mxfp8", "mxfp4") and not self._adapted(weight_attr)
                and isinstance(weight, torch.Tensor) and out_dtype == torch.bfloat16):
            # the MX products add the bias row in their epilogue too, with the roundings of the two tensor operations
            from halo_amd.kernels.expert_gemm import expert_gemm

            return expert_gemm(x, weight.to(out_dtype), offs=offs, quant_format=self._lowp_quant_format,
                               weight_cacheable=self._lowp_weight_cacheable, bias=bias.to(out_dtype), eids=eids)
        out = self._expert_proj(x, weight_attr, offs, out_dtype)
        return out if bias is None else out + MoEExpertBiasGather.apply(bias.to(out_dtype), eids)


class EPGemma4MoELayer(EPMoELayerBase):
    """``Gemma4TextExperts``: Gemma-4 computes its router in the decoder layer, so only the expert container is
    replaced and ``forward`` takes the routing decision as made: ``(hidden [T, H], top_k_index [T, k], top_k_weights
    [T, k])``, tokens already flat, the result ``[T, H]`` (``families/gemma4.py:12-39`` of the reference).  The
    experts-only seam: sort, two grouped GEMMs around the fused tanh-GELU combine, weighted combine; the gate weights
    carry a gradient back to the caller's router."""

    HF_MODULE_NAMES = ("Gemma4TextExperts",)
    FAMILY = GEMMA4
    _ROUTER_ATTR = None  # the router is a sibling module of the decoder layer

    @classmethod
    def _find_experts_container(cls, layer: nn.Module) -> nn.Module:
        return layer  # the wrapped module holds gate_up_proj / down_proj itself

    def _adopt_routing(self, original_layer: nn.Module) -> None:
        """Nothing to adopt: indices and weights come with every call."""
        self.top_k = None

    @classmethod
    def from_weights(cls, *, gelu: bool = True, **kwargs):
        self = super().from_weights(router_weight=None, top_k=kwargs.pop("top_k", None), **kwargs)
        if gelu:  # Gemma-4's hidden activation, gelu_pytorch_tanh
            self._fused_glu_mul = GluCombine.gelu_tanh()
        return self

    def forward(self, hidden_states: torch.Tensor, top_k_index: torch.Tensor,  # type: ignore[override]
                top_k_weights: torch.Tensor) -> torch.Tensor:
        return self._dispatch_compute_combine(hidden_states, top_k_index.long(), top_k_weights.float(),
                                              hidden_states.dtype)


MOE_LAYER_MAP = {name: cls for cls in (EPQwen3MoELayer, EPQwen3_5MoELayer, EPGptOssMoELayer, EPGemma4MoELayer)
                 for name in cls.HF_MODULE_NAMES}


def apply_ep_layers(model: nn.Module, ep_config) -> int:
    """Swaps every HF MoE block whose class name a family claims for this package's block, in place; returns how many
    were swapped (the module swap of the reference's ``expert_parallel/parallelize.py:22-69`` at one GPU)."""
    import copy

    swapped = 0
    for parent in list(model.modules()):
        for child_name, child in list(parent.named_children()):
            cls = MOE_LAYER_MAP.get(type(child).__name__)
            if cls is not None:
                setattr(parent, child_name, cls(child, copy.copy(ep_config)))
                swapped += 1
    return swapped
