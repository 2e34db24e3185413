"""The MoE block (route, sort, grouped GLU FFN, combine, shared expert) on one GPU."""

from halo_amd.moe_layer.balancing import expert_load_token_weights  # noqa: F401
from halo_amd.moe_layer.config import EPConfig, single_process_ep_config  # noqa: F401
from halo_amd.moe_layer.families import (  # noqa: F401
    MOE_LAYER_MAP,
    EPGemma4MoELayer,
    EPGptOssMoELayer,
    EPQwen3_5MoELayer,
    EPQwen3MoELayer,
    apply_ep_layers,
)
from halo_amd.moe_layer.expert_lora import (  # noqa: F401
    ExpertLoraSpec,
    disable_expert_adapters,
    expert_lora_delta,
    expert_lora_layers,
    model_has_expert_lora,
)
from halo_amd.moe_layer.layer import EPMoELayerBase, EPSharedExpertsMoELayerBase  # noqa: F401
