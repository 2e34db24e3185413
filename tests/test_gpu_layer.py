"""GPU parity tests of the whole MoE block: forward and every gradient against the CPU oracle's per-expert loop
(fp32 math on the same input bits), routing bit for bit, and the blocks as drop-ins for the Hugging Face MoE modules
they wrap.

Tolerances (BASELINE.json): routing indices / offsets bit-exact; bf16 outputs and gradients max-rel <= 2e-2 and cosine
>= 0.9999 against the fp32 result; fp32 runs max-rel <= 1e-4.
"""

import pytest
import torch

from tests.cases import CONFIG1, CONFIG2_SMALL, CONFIG4_SMALL, make_layer_inputs

pytestmark = pytest.mark.gpu


def max_rel(actual, reference):
    a, r = actual.detach().double().cpu(), reference.detach().double().cpu()
    return ((a - r).abs().max() / r.abs().max().clamp(min=1e-30)).item()


def cosine(actual, reference):
    a, r = actual.detach().double().cpu().flatten(), reference.detach().double().cpu().flatten()
    return (torch.dot(a, r) / (a.norm() * r.norm())).item()


def _check(name, got, want, tol):
    assert torch.isfinite(got).all(), name
    err, cos = max_rel(got, want), cosine(got, want)
    assert err <= tol, f"{name}: max-rel {err:.3e} > {tol}"
    assert cos >= 0.9999, f"{name}: cosine {cos:.6f}"


def _build_layer(cfg, inputs, device):
    from halo_amd.moe_layer import EPGptOssMoELayer, EPQwen3_5MoELayer, EPQwen3MoELayer

    params = {k: v.to(device) for k, v in inputs["params"].items()}
    if cfg.router == "softmax_topk":
        renamed = {}
        for k, v in params.items():
            renamed[k.replace("gate_proj", "gate_proj_gmm").replace("up_proj", "up_proj_gmm")] = v
        return EPGptOssMoELayer.from_weights(router_weight=inputs["router_weight"].to(device), top_k=cfg.top_k,
                                             router_bias=inputs.get("router_bias", torch.zeros(cfg.experts)).to(device),
                                             **renamed)
    cls = EPQwen3_5MoELayer if cfg.fused else EPQwen3MoELayer
    return cls.from_weights(router_weight=inputs["router_weight"].to(device), top_k=cfg.top_k, **params)


def _oracle_run(cfg, inputs, indices):
    """fp32 per-expert loop on the CPU over the same input bits, with the device's selection."""
    from oracle import moe_layer as oracle
    from oracle import router as router_oracle

    f = lambda t: t.float().requires_grad_(True)
    x, wr = f(inputs["x"]), f(inputs["router_weight"])
    params = {k: f(v) for k, v in inputs["params"].items()}
    bias = f(inputs["router_bias"]) if "router_bias" in inputs else None
    glu = oracle.Glu("gptoss", 1.702, 7.0) if cfg.glu == "gptoss" else oracle.Glu(cfg.glu)
    mode = router_oracle.SOFTMAX_TOPK if cfg.router == "softmax_topk" else router_oracle.SOFTMAX_ALL
    out, logits, idx, w = oracle.moe_layer_forward(x, wr, params, glu, cfg.top_k, router_bias=bias, mode=mode,
                                                   normalize=True, eps=0.0, indices=indices)
    out.backward(inputs["grad_out"].float())
    grads = {"x": x.grad, "router_weight": wr.grad, **{k: v.grad for k, v in params.items()}}
    if bias is not None:
        grads["router_bias"] = bias.grad
    return out.detach(), logits.detach(), grads


@pytest.mark.parametrize("cfg", (CONFIG1, CONFIG2_SMALL, CONFIG4_SMALL), ids=lambda c: c.name)
def test_layer_forward_backward_matches_the_cpu_loop(device, cfg):
    from halo_amd.kernels.router import SOFTMAX_ALL, SOFTMAX_TOPK, fused_topk_gate
    from oracle import router as router_oracle

    skew = dict(zipf_alpha=1.2, empty_experts=3) if cfg.router == "softmax_topk" else {}
    inputs = make_layer_inputs(cfg, **skew)
    layer = _build_layer(cfg, inputs, device)
    x = inputs["x"].to(device).requires_grad_(True)
    result = layer(x)
    out = result[0] if isinstance(result, tuple) else result
    out.backward(inputs["grad_out"].to(device))
    assert out.dtype == cfg.dtype and out.shape == x.shape

    # routing: the device's picks equal the oracle's rule on the device's own logits, bit for bit
    with torch.no_grad():
        logits = layer._linear_router_logits(x.detach())
        mode = SOFTMAX_TOPK if cfg.router == "softmax_topk" else SOFTMAX_ALL
        idx, gates = fused_topk_gate(logits, cfg.top_k, mode=mode, normalize=True, eps=0.0)
    want_idx = router_oracle.select_topk(logits.cpu(), cfg.top_k)
    assert torch.equal(idx.cpu(), want_idx)
    if skew:
        counts = torch.bincount(idx.cpu().flatten(), minlength=cfg.experts)
        assert (counts == 0).sum() >= 3, "the skewed case should leave experts without tokens"
        assert counts.max() > 4 * counts[counts > 0].float().median()

    want_out, want_logits, want_grads = _oracle_run(cfg, inputs, idx.cpu())
    tol = 1e-4 if cfg.dtype == torch.float32 else 2e-2
    _check("logits", logits, want_logits, tol)
    _check("out", out, want_out, tol)
    _check("grad x", x.grad, want_grads["x"], tol)
    router = getattr(layer, layer._ROUTER_ATTR)
    _check("grad router_weight", router.weight.grad, want_grads["router_weight"], tol)
    for name in inputs["params"]:
        attr = name.replace("gate_proj", "gate_proj_gmm").replace("up_proj", "up_proj_gmm") \
            if cfg.router == "softmax_topk" else name
        got = getattr(layer, attr).grad
        _check(f"grad {name}", got, want_grads[name], tol)
        if got.dim() == 3 and skew:
            empty = (torch.bincount(idx.cpu().flatten(), minlength=cfg.experts) == 0).nonzero().flatten()
            assert not got[empty.to(device)].any(), "an expert without tokens must get an exact-zero weight gradient"
    if "router_bias" in want_grads:
        _check("grad router_bias", router.bias.grad, want_grads["router_bias"], tol)


def test_layer_is_bit_reproducible(device):
    cfg = CONFIG2_SMALL
    inputs = make_layer_inputs(cfg)
    runs = []
    for _ in range(2):
        layer = _build_layer(cfg, inputs, device)
        x = inputs["x"].to(device).requires_grad_(True)
        out = layer(x)
        out.backward(inputs["grad_out"].to(device))
        runs.append([out.detach(), x.grad, layer.gate.weight.grad, layer.gate_up_proj.grad, layer.down_proj.grad])
    assert all(torch.equal(a, b) for a, b in zip(*runs))


@pytest.mark.parametrize("cfg", (CONFIG1, CONFIG2_SMALL, CONFIG2_SMALL._replace(name="cfg2_small_apart", fused=False),
                                 CONFIG4_SMALL), ids=lambda c: c.name)
def test_permute_folded_into_the_first_projection_changes_no_bit(device, cfg, monkeypatch):
    """By default the first expert projection fetches its rows through the sort's index instead of reading a permuted
    copy; the output and every gradient must equal the permute-then-GEMM path's bit for bit (the products and their
    summation order are the same, only the addressing differs).  Where gate and up are stored apart (Qwen3; gpt-oss,
    with biases) the two projections run as one node that also sums their two input gradients in the second one's
    epilogue, where autograd adds them as tensors.  The fp32 configuration does not qualify for the gathering kernels
    and takes the copy either way."""
    from halo_amd.kernels import grouped_mm as gmm

    pairs = []
    real_pair = gmm.gather_grouped_mm_pair
    monkeypatch.setattr(gmm, "gather_grouped_mm_pair", lambda *a, **k: pairs.append(1) or real_pair(*a, **k))
    inputs = make_layer_inputs(cfg)
    runs = []
    for fuse in (True, False):
        layer = _build_layer(cfg, inputs, device)
        assert layer.fuse_permute_into_gemm
        layer.fuse_permute_into_gemm = fuse
        x = inputs["x"].to(device).requires_grad_(True)
        out = layer(x)
        out = out[0] if isinstance(out, tuple) else out
        out.backward(inputs["grad_out"].to(device))
        runs.append([out.detach(), x.grad] + [p.grad for _, p in sorted(layer.named_parameters())])
    assert len(runs[0]) >= 4 and all(g is not None for g in runs[0])
    assert all(torch.equal(a, b) for a, b in zip(*runs))
    assert len(pairs) == (0 if cfg.fused or cfg.dtype != torch.bfloat16 else 1)


def test_gate_weight_folded_into_the_glu_stays_inside_the_tolerance(device):
    """By default the fused-GLU bf16 layer multiplies the gate weights into the GLU's output and sums the down
    projection's rows unweighted (no gradient of the expert outputs is written in backward).  That moves roundings
    relative to the reference's order (weight applied behind the down projection), so it is checked twice: both
    orders against the fp32 CPU loop within BASELINE's tolerance (output and every gradient, the router's included,
    which carries the gate weights' gradient), and against each other."""
    from halo_amd.kernels.router import fused_topk_gate

    cfg = CONFIG2_SMALL
    inputs = make_layer_inputs(cfg)
    runs = {}
    for fold in (True, False):
        layer = _build_layer(cfg, inputs, device)
        assert layer.fold_gate_weight_into_glu
        layer.fold_gate_weight_into_glu = fold
        x = inputs["x"].to(device).requires_grad_(True)
        out = layer(x)
        out.backward(inputs["grad_out"].to(device))
        runs[fold] = {"out": out.detach(), "x": x.grad, "router_weight": layer.gate.weight.grad,
                      "gate_up_proj": layer.gate_up_proj.grad, "down_proj": layer.down_proj.grad}
    with torch.no_grad():
        idx, _ = fused_topk_gate(layer._linear_router_logits(x.detach()), cfg.top_k, normalize=True, eps=0.0)
    want_out, _, want = _oracle_run(cfg, inputs, idx.cpu())
    want["out"] = want_out
    for fold, got in runs.items():
        for name, value in got.items():
            _check(f"{name} (fold={fold})", value, want[name], 2e-2)
    for name in runs[True]:
        assert max_rel(runs[True][name], runs[False][name]) < 2e-2, name
    assert not torch.equal(runs[True]["out"], runs[False]["out"])  # the two orders do round differently


def test_one_gpus_share_of_an_ep_layer(device):
    """Local ids with -1 for other ranks' picks plus host-side receive counts (an EP8 shard's shape, scaled down):
    ``_compute_experts`` against the dense formula over the valid slots, and the count checks."""
    from halo_amd.moe_layer import EPConfig, EPQwen3_5MoELayer
    from oracle import moe_layer as oracle

    g = torch.Generator().manual_seed(2)
    local, ep, top_k, hidden, ffn, rows = 8, 8, 8, 256, 128, 700
    picks = torch.rand(rows, local * ep, generator=g).argsort(dim=1)[:, :top_k]
    experts = torch.where(picks < local, picks, -1)
    experts = experts[(experts >= 0).any(dim=1)]  # a dispatch sends a token only where it has a local pick
    n = experts.shape[0]
    counts = tuple(torch.bincount(experts[experts >= 0], minlength=local).tolist())
    weights = torch.rand(n, top_k, generator=g)
    x = torch.randn(n, hidden, generator=g).bfloat16()
    params = {"gate_up_proj": (torch.randn(local, hidden, 2 * ffn, generator=g) * 0.02).bfloat16(),
              "down_proj": (torch.randn(local, ffn, hidden, generator=g) * 0.02).bfloat16()}
    layer = EPQwen3_5MoELayer.from_weights(router_weight=None, top_k=top_k, ep_config=EPConfig(ep_size=ep, ep_rank=0),
                                           **{k: v.to(device) for k, v in params.items()})
    assert layer.experts_per_rank == local and layer.num_experts == local * ep
    out = layer._compute_experts(x.to(device), experts.to(device), weights.to(device), torch.bfloat16,
                                 recv_counts=counts)
    want = oracle.compute_experts_loop(x.float(), experts, weights.bfloat16().float(),
                                       {k: v.float() for k, v in params.items()}, oracle.Glu(), local)
    _check("shard out", out, want, 2e-2)
    with pytest.raises(RuntimeError, match="needs the dispatch's per-local-expert receive counts"):
        layer._compute_experts(x.to(device), experts.to(device), weights.to(device), torch.bfloat16, recv_counts=None)
    with pytest.raises(RuntimeError, match="needs the dispatch's per-local-expert receive counts"):
        layer._compute_experts(x.to(device), experts.to(device), weights.to(device), torch.bfloat16,
                               recv_counts=counts[:-1])
    empty = layer._compute_experts(x[:0].to(device), experts[:0].to(device), weights[:0].to(device), torch.bfloat16,
                                   recv_counts=(0,) * local)
    assert empty.shape == (0, hidden)


def test_quantised_weight_forward(device):
    """Block-fp8 expert weights (BASELINE config 5, scaled down): forward only, against the dequantised-bf16 path."""
    from halo_amd.kernels.expert_gemm import BlockFp8Weight
    from halo_amd.kernels.lowp.block_fp8 import dequantize_block_fp8, quantize_block_fp8
    from halo_amd.moe_layer import EPConfig, EPQwen3_5MoELayer

    g = torch.Generator().manual_seed(4)
    local, top_k, hidden, ffn, rows = 8, 8, 384, 256, 900
    picks = torch.rand(rows, local * 8, generator=g).argsort(dim=1)[:, :top_k]
    experts = torch.where(picks < local, picks, -1)
    experts = experts[(experts >= 0).any(dim=1)]
    counts = tuple(torch.bincount(experts[experts >= 0], minlength=local).tolist())
    weights = torch.rand(experts.shape, generator=g)
    x = torch.randn(experts.shape[0], hidden, generator=g).bfloat16().to(device)
    w1 = (torch.randn(local, hidden, 2 * ffn, generator=g) * 0.02).to(device)
    w2 = (torch.randn(local, ffn, hidden, generator=g) * 0.02).to(device)
    q1, q2 = quantize_block_fp8(w1), quantize_block_fp8(w2)
    cfg = EPConfig(ep_size=8, ep_rank=0)
    lowp = EPQwen3_5MoELayer.from_weights(router_weight=None, top_k=top_k, ep_config=cfg,
                                          gate_up_proj=BlockFp8Weight(*q1), down_proj=BlockFp8Weight(*q2))
    ref = EPQwen3_5MoELayer.from_weights(router_weight=None, top_k=top_k, ep_config=EPConfig(ep_size=8, ep_rank=0),
                                         gate_up_proj=dequantize_block_fp8(*q1), down_proj=dequantize_block_fp8(*q2))
    ref.fold_gate_weight_into_glu = False  # the order of operations the quantised-weight route keeps
    with torch.no_grad():
        got = lowp._compute_experts(x, experts.to(device), weights.to(device), torch.bfloat16, recv_counts=counts)
        want = ref._compute_experts(x, experts.to(device), weights.to(device), torch.bfloat16, recv_counts=counts)
    assert torch.equal(got, want)  # the dequantisation is exact, inside the kernel or ahead of it
    lowp._lowp_weight_cacheable = False  # weights that may change under the layer: the fp8-reading kernel every time
    with torch.no_grad():
        again = lowp._compute_experts(x, experts.to(device), weights.to(device), torch.bfloat16, recv_counts=counts)
    assert torch.equal(again, want)
    # activations quantised too (per row and 128 values), both products on the e4m3 MFMA: the result moves by the
    # activations' e4m3 rounding, twice over (layer input and GLU output), and by nothing systematic
    lowp._lowp_fp8_activations = True
    with torch.no_grad():
        fp8 = lowp._compute_experts(x, experts.to(device), weights.to(device), torch.bfloat16, recv_counts=counts)
    rel = ((fp8.double() - want.double()).norm() / want.double().norm()).item()
    assert 0.005 < rel < 0.07, rel
    assert cosine(fp8, want) > 0.997
    assert abs(((fp8.double() - want.double()).mean() / want.double().abs().mean()).item()) < 5e-3
    lowp.fuse_glu_quantise = False  # the SwiGLU output through bf16 and the row quantiser: the same bits
    with torch.no_grad():
        two_step = lowp._compute_experts(x, experts.to(device), weights.to(device), torch.bfloat16, recv_counts=counts)
    assert torch.equal(two_step, fp8)


def test_quantised_weight_layer_against_the_cpu_loop_over_oracle_dequantised_weights(device):
    """BASELINE config 5, scaled down, against the oracle end to end: the oracle quantises the fp32 weights
    (numpy, ``oracle.block_fp8``), dequantises them, and runs the fp32 per-expert loop over them; the layer quantises
    the same weights with the HIP quantiser and runs its W8A16 forward.  Bit-equal codes and scales first, then the
    output within the bf16 tolerance; with quantised activations within the band stated for that route."""
    import numpy as np

    from halo_amd.kernels.expert_gemm import BlockFp8Weight
    from halo_amd.kernels.lowp.block_fp8 import quantize_block_fp8
    from halo_amd.moe_layer import EPConfig, EPQwen3_5MoELayer
    from oracle import block_fp8 as fp8_oracle
    from oracle import moe_layer as oracle

    g = torch.Generator().manual_seed(4)
    local, top_k, hidden, ffn, rows = 8, 8, 384, 256, 900
    picks = torch.rand(rows, local * 8, generator=g).argsort(dim=1)[:, :top_k]
    experts = torch.where(picks < local, picks, -1)
    experts = experts[(experts >= 0).any(dim=1)]
    counts = tuple(torch.bincount(experts[experts >= 0], minlength=local).tolist())
    weights = torch.rand(experts.shape, generator=g)
    x = torch.randn(experts.shape[0], hidden, generator=g).bfloat16()
    w1 = torch.randn(local, hidden, 2 * ffn, generator=g) * 0.02
    w2 = torch.randn(local, ffn, hidden, generator=g) * 0.02
    device_q, oracle_params = {}, {}
    for name, w in (("gate_up_proj", w1), ("down_proj", w2)):
        q, scale = quantize_block_fp8(w.to(device))
        want_q, want_scale = fp8_oracle.quantize_block_fp8(w.numpy())
        assert np.array_equal(q.view(torch.uint8).cpu().numpy(), want_q), name
        assert np.array_equal(scale.cpu().numpy(), want_scale), name
        device_q[name] = BlockFp8Weight(q, scale)
        # the reference's dequantised-bf16 path: q * scale in fp32, rounded once to bf16 (exact here)
        oracle_params[name] = torch.from_numpy(fp8_oracle.dequantize_block_fp8(want_q, want_scale)).bfloat16().float()
    layer = EPQwen3_5MoELayer.from_weights(router_weight=None, top_k=top_k, ep_config=EPConfig(ep_size=8, ep_rank=0),
                                           **device_q)
    want = oracle.compute_experts_loop(x.float(), experts, weights.bfloat16().float(), oracle_params, oracle.Glu(),
                                       local)
    with torch.no_grad():
        got = layer._compute_experts(x.to(device), experts.to(device), weights.to(device), torch.bfloat16,
                                     recv_counts=counts)
        _check("W8A16 layer", got, want, 2e-2)
        layer._lowp_fp8_activations = True
        fp8 = layer._compute_experts(x.to(device), experts.to(device), weights.to(device), torch.bfloat16,
                                     recv_counts=counts)
    rel = ((fp8.double().cpu() - want.double()).norm() / want.double().norm()).item()
    assert 0.005 < rel < 0.07, rel
    assert cosine(fp8, want) > 0.997


# ------------------------------------------------------------------------------ drop-ins for the Hugging Face blocks

def _hf_config(model_type, **kw):
    import transformers

    return getattr(transformers, model_type)(**kw)


def test_drop_in_for_hf_qwen3_moe_block(device):
    from transformers.models.qwen3_moe.modeling_qwen3_moe import Qwen3MoeSparseMoeBlock

    from halo_amd.moe_layer import EPQwen3MoELayer, apply_ep_layers, single_process_ep_config

    cfg = _hf_config("Qwen3MoeConfig", hidden_size=256, moe_intermediate_size=128, num_experts=16,
                     num_experts_per_tok=4, norm_topk_prob=True, hidden_act="silu")
    torch.manual_seed(0)
    block = Qwen3MoeSparseMoeBlock(cfg)
    for p in block.parameters():
        torch.nn.init.normal_(p, std=0.05)
    x = torch.randn(2, 48, 256)
    want = block(x)
    want.sum().backward()
    holder = torch.nn.Sequential(torch.nn.Identity(), block.to(device))
    assert apply_ep_layers(holder, single_process_ep_config()) == 1
    layer = holder[1]
    assert isinstance(layer, EPQwen3MoELayer) and hasattr(layer, "gate_proj") and not hasattr(layer, "gate_up_proj")
    assert layer.gate_proj.shape == (16, 256, 128) and layer.down_proj.shape == (16, 128, 256)
    xd = x.to(device).requires_grad_(True)
    got = layer(xd)
    got.sum().backward()
    _check("qwen3 out", got, want, 1e-4)
    assert max_rel(layer.gate.weight.grad, block.gate.weight.grad.cpu()) < 1e-3
    assert {n for n, _ in layer.expert_named_params()} == {"gate_proj", "up_proj", "down_proj"}


def test_drop_in_for_hf_gpt_oss_block(device):
    from transformers.models.gpt_oss.modeling_gpt_oss import GptOssMLP

    from halo_amd.moe_layer import EPGptOssMoELayer, single_process_ep_config

    cfg = _hf_config("GptOssConfig", hidden_size=256, intermediate_size=128, num_local_experts=8,
                     num_experts_per_tok=2)
    torch.manual_seed(1)
    block = GptOssMLP(cfg)
    for p in block.parameters():
        torch.nn.init.normal_(p, std=0.05)
    x = torch.randn(1, 40, 256)
    result = block(x)
    want = result[0] if isinstance(result, tuple) else result
    layer = EPGptOssMoELayer(block.to(device), single_process_ep_config())
    got, logits = layer(x.to(device))
    _check("gpt-oss out", got.view(want.shape), want, 1e-4)
    assert logits.shape == (40, 8) and layer._glu_combine_name() == "gptoss"


def test_drop_in_for_hf_gemma4_experts(device):
    """The experts-only entry (``families/gemma4.py:30-39``): routing decided outside, ``forward(hidden, top_k_index,
    top_k_weights)``.  bf16 on the device against transformers' ``Gemma4TextExperts`` in fp32 on the CPU: output,
    input gradient and the gate weights' gradient within BASELINE's tolerance."""
    from transformers.models.gemma4.configuration_gemma4 import Gemma4TextConfig
    from transformers.models.gemma4.modeling_gemma4 import Gemma4TextExperts

    from halo_amd.moe_layer import EPGemma4MoELayer, single_process_ep_config

    torch.manual_seed(2)
    config = Gemma4TextConfig(hidden_size=256, moe_intermediate_size=88, num_experts=16, top_k_experts=4,
                              hidden_activation="gelu_pytorch_tanh", num_hidden_layers=1)
    hf = Gemma4TextExperts(config)
    with torch.no_grad():
        hf.gate_up_proj.normal_(0, 0.05)
        hf.down_proj.normal_(0, 0.05)
    x = torch.randn(300, 256).bfloat16().float().requires_grad_(True)
    probs, idx = torch.topk(torch.softmax(torch.randn(300, 16), -1), 4, dim=-1)
    w = (probs / probs.sum(-1, keepdim=True)).bfloat16().float().requires_grad_(True)
    upstream = torch.randn(300, 256).bfloat16().float()
    for p in (hf.gate_up_proj, hf.down_proj):
        p.data = p.data.bfloat16().float()
    want = hf(x, idx, w)
    want_gx, want_gw = torch.autograd.grad(want, (x, w), upstream)
    layer = EPGemma4MoELayer(hf.to(device).to(torch.bfloat16), single_process_ep_config())
    assert layer._glu_combine_name() == "gelu_tanh"
    xd = x.detach().bfloat16().to(device).requires_grad_(True)
    wd = w.detach().to(device).requires_grad_(True)
    got = layer(xd, idx.to(device), wd)
    assert got.dtype == torch.bfloat16 and got.shape == (300, 256)
    got_gx, got_gw = torch.autograd.grad(got, (xd, wd), upstream.bfloat16().to(device))
    _check("gemma4 out", got, want, 2e-2)
    _check("gemma4 grad x", got_gx, want_gx, 2e-2)
    _check("gemma4 grad gate weights", got_gw, want_gw, 2e-2)


def test_router_projection_gradients_at_a_token_count_that_splits_the_wgrad(device):
    """The router's weight gradient goes through the grouped wgrad kernel in 32 token slices once there are enough
    tokens; the layer configurations above are too small to take that path.  Checked against the fp64 product over
    the same bf16 inputs (BASELINE tolerance), and for run-to-run bit equality."""
    from halo_amd.moe_layer.layer import _DenseLinear

    tokens, hidden, experts = 4096, 512, 128
    assert tokens >= _DenseLinear._MIN_TOKENS and tokens % _DenseLinear._SPLITS == 0
    g = torch.Generator().manual_seed(7)
    x = torch.randn(tokens, hidden, generator=g).bfloat16()
    w = (torch.randn(experts, hidden, generator=g) * 0.05).bfloat16()
    dlogits = torch.randn(tokens, experts, generator=g).bfloat16()
    results = []
    for _ in range(2):
        xd, wd = x.to(device).requires_grad_(True), w.to(device).requires_grad_(True)
        logits = _DenseLinear.apply(xd, wd)
        logits.backward(dlogits.to(device))
        results.append((logits.detach(), xd.grad, wd.grad))
    logits, dx, dw = results[0]
    _check("logits", logits, x.double() @ w.double().t(), 2e-2)
    _check("dx", dx, dlogits.double() @ w.double(), 2e-2)
    _check("dw", dw, dlogits.double().t() @ x.double(), 2e-2)
    assert all(torch.equal(a, b) for a, b in zip(results[0], results[1]))


def test_router_projection_with_an_expert_count_the_grouped_kernel_does_not_take(device):
    """60 experts: the logits' rows are not 16-byte multiples, so neither the grouped kernels nor the sliced weight
    gradient apply and the library's dense product takes over."""
    from halo_amd.moe_layer.layer import _DenseLinear

    tokens, hidden, experts = 2048, 256, 60
    g = torch.Generator().manual_seed(9)
    x = torch.randn(tokens, hidden, generator=g).bfloat16()
    w = (torch.randn(experts, hidden, generator=g) * 0.05).bfloat16()
    dlogits = torch.randn(tokens, experts, generator=g).bfloat16()
    xd, wd = x.to(device).requires_grad_(True), w.to(device).requires_grad_(True)
    assert not _DenseLinear._sliced_wgrad_usable(dlogits.to(device), xd)
    _DenseLinear.apply(xd, wd).backward(dlogits.to(device))
    _check("dw", wd.grad, dlogits.double().t() @ x.double(), 2e-2)
    _check("dx", xd.grad, dlogits.double() @ w.double(), 2e-2)


@pytest.mark.parametrize(("tokens", "width", "hidden"), ((8192, 512, 2048), (4096, 2048, 512), (2048, 264, 1000)))
def test_dense_projection_weight_gradient_in_token_slices(device, tokens, width, hidden):
    """``dense_mm`` (the shared expert's projections): forward and input gradient on the grouped kernels with one
    group, the weight gradient summed from token slices on the grouped kernel (16, 16 and 32 of them here).  Against
    the fp64 products over the same bf16 inputs (BASELINE tolerance) and for run-to-run bit equality."""
    from halo_amd.moe_layer.layer import _DenseLinear, dense_mm

    g = torch.Generator().manual_seed(17)
    x = torch.randn(tokens, hidden, generator=g).bfloat16()
    w = (torch.randn(width, hidden, generator=g) * hidden ** -0.5).bfloat16()
    dout = torch.randn(tokens, width, generator=g).bfloat16()
    assert _DenseLinear._sliced_wgrad_usable(dout.to(device), x.to(device))
    results = []
    for _ in range(2):
        xd, wd = x.to(device).requires_grad_(True), w.to(device).requires_grad_(True)
        out = dense_mm(xd, wd)
        out.backward(dout.to(device))
        results.append((out.detach(), xd.grad, wd.grad))
    out, dx, dw = results[0]
    _check("out", out, x.double() @ w.double().t(), 2e-2)
    _check("dx", dx, dout.double() @ w.double(), 2e-2)
    _check("dw", dw, dout.double().t() @ x.double(), 2e-2)
    assert all(torch.equal(a, b) for a, b in zip(results[0], results[1]))


def test_sliced_weight_gradient_rounding_against_the_fp32_accumulated_gradient(device):
    """The token slices' partial gradients are rounded to bf16 before they are summed (fp32 accumulation, one more
    rounding), where a dense product accumulates every token in fp32 and rounds once.  On ordinary data the partials
    add in quadrature and the result stays at the single-rounding floor (Frobenius error within 1.5x of rounding the
    fp32-accumulated gradient once).  When the slices cancel (the second half of the tokens repeats the first with the
    output gradient negated, plus a small remainder) the error is bounded by the partials, not by the result: at most
    splits x 2^-9 x the largest partial magnitude per element."""
    from halo_amd.moe_layer.layer import _DenseLinear, dense_mm

    tokens, width, hidden = 8192, 512, 2048
    g = torch.Generator().manual_seed(23)
    x = torch.randn(tokens, hidden, generator=g).bfloat16()
    w = (torch.randn(width, hidden, generator=g) * hidden ** -0.5).bfloat16()
    dout = torch.randn(tokens, width, generator=g).bfloat16()
    splits = _DenseLinear._splits_for(dout.to(device), x.to(device))
    assert _DenseLinear._sliced_wgrad_usable(dout.to(device), x.to(device)) and splits >= 4

    def sliced_gradient(rows, grads):
        wd = w.to(device).requires_grad_(True)
        dense_mm(rows.to(device), wd).backward(grads.to(device))
        return wd.grad.double().cpu()

    # ordinary data: at the floor of one bf16 rounding of the exact gradient
    exact = dout.double().t() @ x.double()
    floor = (exact.float().bfloat16().double() - exact).norm()
    err = (sliced_gradient(x, dout) - exact).norm()
    assert err <= 1.5 * floor, f"Frobenius error {err:.4e} against a rounding floor of {floor:.4e}"

    # cancelling slices: tokens [half:] repeat tokens [:half] with the gradient negated, plus a remainder 2^-6 the size
    half = tokens // 2
    x2 = torch.cat([x[:half], x[:half]])
    small = (torch.randn(half, width, generator=g) * 2.0 ** -6).bfloat16()
    dout2 = torch.cat([dout[:half], (-dout[:half].float() + small.float()).bfloat16()])
    exact2 = dout2.double().t() @ x2.double()
    step = tokens // splits
    largest_partial = max((dout2[i:i + step].double().t() @ x2[i:i + step].double()).abs().max().item()
                          for i in range(0, tokens, step))
    worst = (sliced_gradient(x2, dout2) - exact2).abs().max().item()
    bound = splits * 2.0 ** -9 * largest_partial + 2.0 ** -8 * exact2.abs().max().item()
    assert worst <= bound, f"largest error {worst:.4e} against the bound {bound:.4e}"


@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float32), ids=("bf16", "fp32"))
@pytest.mark.parametrize(("tokens", "hidden", "pitch"), ((8192, 2048, 2048), (1027, 264, 264), (45, 512, 640), (3, 64, 64)))
def test_sigmoid_row_gate_against_the_tensor_operations(device, dtype, tokens, hidden, pitch):
    """``sigmoid_row_gate`` (the shared expert's per-token output gate, one kernel per direction) against
    ``sigmoid(x @ w^T)`` and its autograd in fp64 over the same inputs: the gate within one rounding of the dtype, the
    gradients within the BASELINE tolerance (fp32: 1e-5); row counts that do not fill a workgroup's share, a hidden
    size of 33 chunks, rows read from a wider buffer; two runs bit-equal."""
    from halo_amd.moe_layer.layer import _SigmoidRowGate, sigmoid_row_gate

    g = torch.Generator().manual_seed(31)
    x = torch.randn(tokens, pitch, generator=g).to(dtype)
    w = (torch.randn(1, hidden, generator=g) * hidden ** -0.5 * 2).to(dtype)
    grad = torch.randn(tokens, generator=g).to(dtype)
    results = []
    for _ in range(2):
        xd = x.to(device)[:, :hidden].requires_grad_(True)
        wd = w.to(device).requires_grad_(True)
        gate = sigmoid_row_gate(xd, wd)
        assert isinstance(gate.grad_fn, _SigmoidRowGate._backward_cls)
        gate.backward(grad.to(device))
        results.append((gate.detach().clone(), xd.grad.clone(), wd.grad.clone()))
    assert all(torch.equal(a, b) for a, b in zip(results[0], results[1]))
    gate, gx, gw = (t.double().cpu() for t in results[0])
    xr = x[:, :hidden].double().requires_grad_(True)
    wr = w.double().requires_grad_(True)
    want = torch.sigmoid(xr @ wr.t()).view(-1)
    want.backward(grad.double())
    # the logit is rounded to the dtype before the sigmoid (the linear's output): |d sigmoid| <= |d logit| / 4; in fp32
    # the dot product's own accumulation error (hidden terms) is what is left
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -23 * hidden ** 0.5
    logit = (xr @ wr.t()).view(-1).detach()
    assert ((gate - want.detach()).abs() <= ulp * (want.detach() + logit.abs() / 4 + 1e-3)).all()
    tol = 2e-2 if dtype == torch.bfloat16 else 1e-5
    _check("grad x", gx, xr.grad, tol)
    _check("grad w", gw, wr.grad, tol)


def test_sigmoid_row_gate_roundings_are_the_tensor_operations(device):
    """Given the same gate values, ``grad_x`` is the tensor operations' bit for bit: sigmoid's backward in fp32 rounded
    to bf16, then one product per element rounded once (an outer product has no summation order)."""
    from halo_amd.moe_layer.layer import sigmoid_row_gate

    g = torch.Generator().manual_seed(33)
    x = torch.randn(4096, 1024, generator=g).bfloat16().to(device).requires_grad_(True)
    w = (torch.randn(1, 1024, generator=g) * 0.05).bfloat16().to(device).requires_grad_(True)
    grad = torch.randn(4096, generator=g).bfloat16().to(device)
    gate = sigmoid_row_gate(x, w)
    gate.backward(grad)
    y = gate.detach().float()
    scaled = (grad.float() * (1.0 - y) * y).bfloat16()
    assert torch.equal(x.grad, (scaled.float()[:, None] * w.detach().float()).bfloat16())


class _SharedMlp(torch.nn.Module):
    def __init__(self, hidden, width, dtype, generator):
        super().__init__()
        for name, shape in (("gate_proj", (width, hidden)), ("up_proj", (width, hidden)), ("down_proj", (hidden, width))):
            linear = torch.nn.Linear(shape[1], shape[0], bias=False, dtype=dtype)
            linear.weight.data = (torch.randn(shape, generator=generator) * shape[1] ** -0.5).to(dtype)
            setattr(self, name, linear)


def _layer_with_shared_expert(cfg, inputs, device, gated, fuse):
    g = torch.Generator().manual_seed(21)
    layer = _build_layer(cfg, inputs, device)
    layer.shared_expert = _SharedMlp(cfg.hidden, 64, cfg.dtype, g).to(device)
    layer._shared_expert_attr = "shared_expert"
    if gated:
        gate = torch.nn.Linear(cfg.hidden, 1, bias=False, dtype=cfg.dtype)
        gate.weight.data = (torch.randn(1, cfg.hidden, generator=g) * cfg.hidden ** -0.5).to(cfg.dtype)
        layer.shared_expert_gate = gate.to(device)
    layer.fuse_shared_into_combine = fuse
    return layer


@pytest.mark.parametrize("gated", (False, True), ids=("plain", "sigmoid_gated"))
@pytest.mark.parametrize("cfg", (CONFIG1, CONFIG2_SMALL), ids=lambda c: c.name)
def test_shared_expert_added_in_the_combine_kernel(device, cfg, gated):
    """A layer with a shared expert (Qwen3.5's carries a sigmoid gate): the sum ``routed + shared`` taken by the
    combine kernel gives the output of the tensor addition bit for bit, and the gradients of everything that does not
    pass through the gate's dot product bit for bit; the output and input gradient also match the fp32 loop with the
    same selection."""
    from halo_amd.moe_layer import EPQwen3_5MoELayer
    from oracle import moe_layer as oracle

    if not cfg.fused:
        pytest.skip("the sigmoid-gated shared expert belongs to the fused-GLU family")
    inputs = make_layer_inputs(cfg)
    results = []
    for fuse in (False, True):
        layer = _layer_with_shared_expert(cfg, inputs, device, gated, fuse)
        assert isinstance(layer, EPQwen3_5MoELayer)
        x = inputs["x"].to(device).requires_grad_(True)
        out = layer(x)
        out.backward(inputs["grad_out"].to(device))
        grads = {n: p.grad.clone() for n, p in layer.named_parameters() if p.grad is not None}
        results.append((out.detach(), x.grad.clone(), grads))
    (out_a, gx_a, grads_a), (out_b, gx_b, grads_b) = results
    assert torch.equal(out_a, out_b)
    assert set(grads_a) == set(grads_b) and any(n.startswith("shared_expert.") for n in grads_a)
    tol = 1e-5 if cfg.dtype == torch.float32 else 2e-2
    for name in grads_a:
        if name.startswith("shared_expert_gate"):
            assert max_rel(grads_b[name], grads_a[name]) < tol, name
        else:
            assert torch.equal(grads_a[name], grads_b[name]), name
    if gated:
        assert max_rel(gx_b, gx_a) < tol
    else:
        assert torch.equal(gx_a, gx_b)

    # against the fp32 loop: selection taken from the device
    from halo_amd.kernels.router import fused_topk_gate
    with torch.no_grad():
        idx, _ = fused_topk_gate(layer._linear_router_logits(x.detach()), cfg.top_k, normalize=True, eps=0.0)
    f = lambda t: t.detach().float().cpu().requires_grad_(True)
    xs, wr = f(inputs["x"]), f(inputs["router_weight"])
    params = {k: f(v) for k, v in inputs["params"].items()}
    shared = {n: f(getattr(layer.shared_expert, n).weight) for n in ("gate_proj", "up_proj", "down_proj")}
    if gated:
        shared["shared_expert_gate"] = f(layer.shared_expert_gate.weight)
    want, _, _, _ = oracle.moe_layer_forward(xs, wr, params, oracle.Glu(cfg.glu), cfg.top_k, normalize=True, eps=0.0,
                                             indices=idx.cpu(), shared=shared)
    want.backward(inputs["grad_out"].float())
    check_tol = 1e-4 if cfg.dtype == torch.float32 else 2e-2
    _check("out with shared expert", out_b, want.detach(), check_tol)
    _check("grad x with shared expert", gx_b, xs.grad, check_tol)
    _check("grad shared down_proj", grads_b["shared_expert.down_proj.weight"], shared["down_proj"].grad, check_tol)


def test_shared_expert_gate_and_up_as_one_product_keeps_the_forward_bits(device):
    """The shared expert's gate and up projections as one product over the two weights side by side against two
    products: the same dot products, so the layer's output is equal bit for bit; the input gradient is summed over both
    in fp32 instead of two rounded products and an addition, so gradients agree within the bf16 tolerance."""
    cfg = CONFIG2_SMALL
    inputs = make_layer_inputs(cfg)
    results = []
    for one_product in (False, True):
        layer = _layer_with_shared_expert(cfg, inputs, device, gated=True, fuse=True)
        layer.fuse_shared_gate_up = one_product
        x = inputs["x"].to(device).requires_grad_(True)
        out = layer(x)
        out.backward(inputs["grad_out"].to(device))
        grads = {n: p.grad.clone() for n, p in layer.named_parameters() if p.grad is not None}
        results.append((out.detach(), x.grad.clone(), grads))
    (out_a, gx_a, grads_a), (out_b, gx_b, grads_b) = results
    assert torch.equal(out_a, out_b)
    assert max_rel(gx_b, gx_a) < 2e-2
    assert set(grads_a) == set(grads_b)
    for name in grads_a:
        assert max_rel(grads_b[name], grads_a[name]) < 2e-2, name
        # the same contraction per element (at this size the weight gradient is one product, not token slices)
        if name.startswith(("shared_expert.gate_proj", "shared_expert.up_proj")):
            assert torch.equal(grads_a[name], grads_b[name]), name


@pytest.mark.parametrize("fuse", (False, True), ids=("tensor_add", "in_combine"))
def test_shared_expert_on_a_side_stream_changes_no_bit(device, fuse, monkeypatch):
    """``HALO_EP_SHARED_OVERLAP``: the shared expert runs on a second stream beside the routed path and is joined
    ahead of the sum.  Same kernels on the same data: output and every gradient equal the single-stream run bit for
    bit, three steps in a row (a missing join would show as a stale or half-written shared output)."""
    from halo_amd.moe_layer import layer as layer_module

    cfg = CONFIG2_SMALL
    inputs = make_layer_inputs(cfg)
    runs = {}
    for overlap in (False, True):
        monkeypatch.setattr(layer_module, "_SHARED_OVERLAP_ENABLED", overlap)
        layer = _layer_with_shared_expert(cfg, inputs, device, gated=True, fuse=fuse)
        steps = []
        for _ in range(3):
            for p in layer.parameters():
                p.grad = None
            x = inputs["x"].to(device).requires_grad_(True)
            out = layer(x)
            out.backward(inputs["grad_out"].to(device))
            torch.cuda.synchronize()
            steps.append([out.detach(), x.grad] + [p.grad.clone() for _, p in sorted(layer.named_parameters())])
        assert all(torch.equal(a, b) for later in steps[1:] for a, b in zip(steps[0], later))
        runs[overlap] = steps[0]
    assert len(layer_module._shared_overlap_streams) == 1
    assert all(torch.equal(a, b) for a, b in zip(runs[False], runs[True]))


def test_expert_load_counter(device):
    """``_record_expert_load`` (reference ``balancing_bias.py:200-207``): once ``balancing_biases`` is attached, every
    grad-enabled training forward adds the router's selection counts to ``expert_load_counter``; evaluation, a
    ``no_grad`` forward and a layer without the bias leave it alone; a token-weight scope counts tokens by weight."""
    from halo_amd.kernels.router import fused_topk_gate
    from halo_amd.moe_layer import expert_load_token_weights

    cfg = CONFIG2_SMALL
    inputs = make_layer_inputs(cfg)
    layer = _build_layer(cfg, inputs, device)
    x = inputs["x"].to(device)
    layer.train()
    layer(x)
    assert layer.expert_load_counter is None  # no balancing bias attached: nothing is counted
    layer.balancing_biases = torch.zeros(cfg.experts, device=device)
    with torch.no_grad():
        idx, _ = fused_topk_gate(layer._linear_router_logits(x), cfg.top_k, normalize=True, eps=0.0)
    want = torch.bincount(idx.flatten().cpu(), minlength=cfg.experts).float()
    layer(x)
    layer(x)
    assert torch.equal(layer.expert_load_counter.cpu(), 2 * want)
    with torch.no_grad():
        layer(x)
    layer.eval()
    layer(x)
    assert torch.equal(layer.expert_load_counter.cpu(), 2 * want)
    layer.train()
    token_weights = torch.arange(cfg.tokens, dtype=torch.float32) % 3
    with expert_load_token_weights(token_weights):
        layer(x)
    weighted = torch.zeros(cfg.experts).index_add_(0, idx.flatten().cpu(), token_weights.repeat_interleave(cfg.top_k))
    assert torch.allclose(layer.expert_load_counter.cpu(), 2 * want + weighted, rtol=1e-6)
    with pytest.raises(ValueError, match="do not describe this forward"), expert_load_token_weights(token_weights[:5]):
        layer(x)


# ------------------------------------------------------------------------------------------------- expert LoRA

@pytest.mark.parametrize("cfg", (CONFIG2_SMALL, CONFIG4_SMALL), ids=lambda c: c.name)
def test_expert_lora_equals_the_layer_with_merged_weights(device, cfg):
    """``x @ W + s (x @ A) @ B`` is ``x @ (W + s A B)``: the oracle runs the fp32 loop over the merged weights (the
    adapters as its leaves, so their gradients come out of the same graph), the layer runs the three grouped products.
    The base weights are frozen, the adapters' initial delta is zero, and ``disable_expert_adapters`` gives the base
    layer back."""
    from halo_amd.kernels.router import SOFTMAX_ALL, SOFTMAX_TOPK, fused_topk_gate
    from halo_amd.moe_layer import ExpertLoraSpec, disable_expert_adapters, expert_lora_delta
    from halo_amd.moe_layer.config import EPConfig
    from oracle import moe_layer as oracle
    from oracle import router as router_oracle

    inputs = make_layer_inputs(cfg)
    base = _build_layer(cfg, inputs, device)
    base.fold_gate_weight_into_glu = False  # a layer with adapters keeps the reference's order of operations
    spec = ExpertLoraSpec(r=16, alpha=32.0)
    # the same construction with adapters asked for
    from halo_amd.moe_layer import EPGptOssMoELayer, EPQwen3_5MoELayer, EPQwen3MoELayer
    params = {k: v.to(device) for k, v in inputs["params"].items()}
    ep = EPConfig(expert_lora=spec)
    if cfg.router == "softmax_topk":
        params = {k.replace("gate_proj", "gate_proj_gmm").replace("up_proj", "up_proj_gmm"): v for k, v in params.items()}
        layer = EPGptOssMoELayer.from_weights(router_weight=inputs["router_weight"].to(device), top_k=cfg.top_k,
                                              router_bias=inputs.get("router_bias", torch.zeros(cfg.experts)).to(device),
                                              ep_config=ep, **params)
    else:
        cls = EPQwen3_5MoELayer if cfg.fused else EPQwen3MoELayer
        layer = cls.from_weights(router_weight=inputs["router_weight"].to(device), top_k=cfg.top_k, ep_config=ep, **params)
    assert layer.has_expert_lora and len(layer.expert_lora_named_params()) == 2 * len(layer._expert_lora_attrs)
    for attr in layer._expert_lora_attrs:
        assert not getattr(layer, attr).requires_grad and getattr(layer, attr + "_lora_A").requires_grad
        assert not getattr(layer, attr + "_lora_B").any()
    x = inputs["x"].to(device)

    def run(module, inp):
        result = module(inp)
        return result[0] if isinstance(result, tuple) else result

    with torch.no_grad():
        start = run(layer, x)
        assert torch.equal(start, run(base, x))  # B = 0: the delta is an exact zero
        g = torch.Generator().manual_seed(5)
        for attr in layer._expert_lora_attrs:  # a delta comparable to the weights themselves
            b = getattr(layer, attr + "_lora_B")
            b.copy_((torch.randn(b.shape, generator=g) * 0.05).to(b.dtype))
        assert not torch.equal(run(layer, x), start)
        holder = torch.nn.Sequential(layer)
        with disable_expert_adapters(holder):
            assert torch.equal(run(layer, x), start)

    xd = x.clone().requires_grad_(True)
    out = run(layer, xd)
    out.backward(inputs["grad_out"].to(device))

    with torch.no_grad():
        logits = layer._linear_router_logits(x)
        mode = SOFTMAX_TOPK if cfg.router == "softmax_topk" else SOFTMAX_ALL
        idx, _ = fused_topk_gate(logits, cfg.top_k, mode=mode, normalize=True, eps=0.0)
    f = lambda t: t.detach().float().cpu().requires_grad_(True)
    xr, wr = f(inputs["x"]), f(inputs["router_weight"])
    leaves, merged = {}, {}
    for name, value in inputs["params"].items():
        attr = name.replace("gate_proj", "gate_proj_gmm").replace("up_proj", "up_proj_gmm") \
            if cfg.router == "softmax_topk" else name
        if attr in layer._expert_lora_attrs:
            a, b = f(getattr(layer, attr + "_lora_A")), f(getattr(layer, attr + "_lora_B"))
            leaves[attr + "_lora_A"], leaves[attr + "_lora_B"] = a, b
            merged[name] = value.float() + expert_lora_delta(a, b, spec.scaling)
        else:
            merged[name] = value.float()
    bias = inputs["router_bias"].float() if "router_bias" in inputs else None
    glu = oracle.Glu("gptoss", 1.702, 7.0) if cfg.glu == "gptoss" else oracle.Glu(cfg.glu)
    ref_mode = router_oracle.SOFTMAX_TOPK if cfg.router == "softmax_topk" else router_oracle.SOFTMAX_ALL
    want, _, _, _ = oracle.moe_layer_forward(xr, wr, merged, glu, cfg.top_k, router_bias=bias, mode=ref_mode,
                                             normalize=True, eps=0.0, indices=idx.cpu())
    want.backward(inputs["grad_out"].float())
    _check("out", out, want.detach(), 2e-2)
    _check("grad x", xd.grad, xr.grad, 2e-2)
    for name, leaf in leaves.items():
        _check(f"grad {name}", getattr(layer, name).grad, leaf.grad, 2e-2)
    for attr in layer._expert_lora_attrs:
        assert getattr(layer, attr).grad is None


@pytest.mark.parametrize("cfg", (CONFIG2_SMALL, CONFIG4_SMALL), ids=lambda c: c.name)
def test_expert_lora_delta_added_in_the_gemm_epilogue_changes_no_bit(device, cfg):
    """With adapters the projection's low-rank delta is added by the second adapter product's epilogue, and on a
    fused-GLU layer both readers of the token rows fetch them through the sort's index.  Output and every gradient
    equal the three-products-and-two-tensor-operations form bit for bit."""
    from halo_amd.moe_layer import EPGptOssMoELayer, EPQwen3_5MoELayer, ExpertLoraSpec
    from halo_amd.moe_layer.config import EPConfig

    inputs = make_layer_inputs(cfg)
    runs = []
    for fuse in (False, True):
        params = {k: v.to(device) for k, v in inputs["params"].items()}
        ep = EPConfig(expert_lora=ExpertLoraSpec(r=16, alpha=24.0))
        if cfg.router == "softmax_topk":
            params = {k.replace("gate_proj", "gate_proj_gmm").replace("up_proj", "up_proj_gmm"): v
                      for k, v in params.items()}
            layer = EPGptOssMoELayer.from_weights(
                router_weight=inputs["router_weight"].to(device), top_k=cfg.top_k, ep_config=ep,
                router_bias=inputs.get("router_bias", torch.zeros(cfg.experts)).to(device), **params)
        else:
            layer = EPQwen3_5MoELayer.from_weights(router_weight=inputs["router_weight"].to(device), top_k=cfg.top_k,
                                                   ep_config=ep, **params)
        g = torch.Generator().manual_seed(5)
        with torch.no_grad():
            for attr in sorted(layer._expert_lora_attrs):
                for suffix in ("_lora_A", "_lora_B"):
                    p = getattr(layer, attr + suffix)
                    p.copy_((torch.randn(p.shape, generator=g) * 0.05).to(p.dtype))
        layer.fuse_lora_into_gemm = fuse
        x = inputs["x"].to(device).requires_grad_(True)
        out = layer(x)
        out = out[0] if isinstance(out, tuple) else out
        out.backward(inputs["grad_out"].to(device))
        grads = {name: p.grad for name, p in layer.named_parameters() if p.grad is not None}
        runs.append({"out": out.detach(), "grad_x": x.grad, **grads})
    assert runs[0].keys() == runs[1].keys() and len(runs[0]) >= 6
    assert [name for name in runs[0] if not torch.equal(runs[0][name], runs[1][name])] == []


def test_expert_lora_rank_must_span_whole_rows(device):
    from halo_amd.moe_layer import EPQwen3_5MoELayer, ExpertLoraSpec
    from halo_amd.moe_layer.config import EPConfig

    w1 = torch.zeros(4, 64, 128, dtype=torch.bfloat16, device=device)
    w2 = torch.zeros(4, 64, 64, dtype=torch.bfloat16, device=device)
    with pytest.raises(ValueError, match="use a multiple of 8"):
        EPQwen3_5MoELayer.from_weights(router_weight=None, top_k=2, ep_config=EPConfig(expert_lora=ExpertLoraSpec(12, 24.0)),
                                       gate_up_proj=w1, down_proj=w2)
    only_down = EPQwen3_5MoELayer.from_weights(
        router_weight=None, top_k=2, gate_up_proj=w1, down_proj=w2,
        ep_config=EPConfig(expert_lora=ExpertLoraSpec(8, 16.0, projections=frozenset({"down"}), use_rslora=True)))
    assert only_down._expert_lora_attrs == frozenset({"down_proj"}) and only_down.gate_up_proj.requires_grad
    assert abs(only_down.expert_lora_scaling - 16.0 / 8 ** 0.5) < 1e-12


@pytest.mark.parametrize("frozen", ("weight", "x"))
def test_sigmoid_row_gate_with_one_side_frozen(device, frozen):
    """A frozen gate weight (adapter fine-tuning) or a frozen input: the gradient that is asked for keeps the bits of
    the run that asks for both, and the other one is not produced."""
    from halo_amd.moe_layer.layer import sigmoid_row_gate

    g = torch.Generator().manual_seed(35)
    x = torch.randn(777, 512, generator=g).bfloat16().to(device)
    w = (torch.randn(1, 512, generator=g) * 0.05).bfloat16().to(device)
    grad = torch.randn(777, generator=g).bfloat16().to(device)
    xa, wa = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    sigmoid_row_gate(xa, wa).backward(grad)
    xb, wb = x.clone().requires_grad_(frozen != "x"), w.clone().requires_grad_(frozen != "weight")
    gate = sigmoid_row_gate(xb, wb)
    gate.backward(grad)
    if frozen == "weight":
        assert wb.grad is None and torch.equal(xb.grad, xa.grad)
    else:
        assert xb.grad is None and torch.equal(wb.grad, wa.grad)
