"""Host-side logic that needs no GPU: the expert-LoRA recipe."""

import torch


def test_expert_lora_spec_scaling_and_coverage():
    """The recipe of the reference's spec (``expert_lora_spec.py:24-41``): alpha / r, alpha / sqrt(r) with rsLoRA; a
    stored weight is adapted when it carries one of the projections asked for."""
    from halo_amd.moe_layer.expert_lora import EXPERT_LORA_RANK_MULTIPLE, ExpertLoraSpec, expert_lora_delta

    assert ExpertLoraSpec(16, 32.0).scaling == 2.0
    assert abs(ExpertLoraSpec(16, 32.0, use_rslora=True).scaling - 8.0) < 1e-12
    gate_only = ExpertLoraSpec(8, 8.0, projections=frozenset({"gate"}))
    assert gate_only.adapts("gate_up_proj") and gate_only.adapts("gate_proj_gmm") and gate_only.adapts("gate_proj")
    assert not gate_only.adapts("down_proj") and not gate_only.adapts("up_proj") and not gate_only.adapts("router")
    assert EXPERT_LORA_RANK_MULTIPLE == 8
    a, b = torch.randn(3, 5, 8), torch.randn(3, 8, 7)
    assert torch.allclose(expert_lora_delta(a, b, 0.5), 0.5 * torch.einsum("ekr,ern->ekn", a, b), atol=1e-6)
