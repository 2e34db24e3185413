"""The ``halo_amd.kernels`` operators on CPU tensors (plain torch operations, ``halo_amd/kernels/_cpu.py``) against the
oracle: the reference's operators take CPU tensors too (``halo/kernels/moe_route_sort.py:201-243``,
``moe_permute.py:115-127``, ``fused_glu.py:352-361``), which is what a checkout that swaps the imports runs its own
CPU tests on.  Integer outputs bit for bit, floating point to fp32 rounding."""

import numpy as np
import pytest
import torch

from tests.cases import ROUTING_CASES, make_receive


@pytest.mark.parametrize("case", ROUTING_CASES, ids=lambda c: c.name)
def test_cpu_route_sort_matches_the_oracle_bit_for_bit(case):
    from halo_amd.kernels.moe_route_sort import sort_routing_by_expert
    from oracle import route_sort as oracle

    experts, weights, counts = make_receive(case, seed=ROUTING_CASES.index(case))
    weights = weights.clone().requires_grad_(True)
    got = sort_routing_by_expert(experts, weights, case.local_experts, counts)
    want = oracle.argsort_routing(experts.numpy(), weights.detach().numpy(), case.local_experts, counts)
    for name, g, w in zip(("sorted_token_idx", "sorted_weights", "sorted_expert_ids", "offs", "inv_map"), got, want):
        assert g.dtype == torch.from_numpy(np.asarray(w)).dtype, name
        assert np.array_equal(g.detach().numpy(), w), name
    # only the gate weights carry a gradient: each slot's, read back at its sorted position
    upstream = torch.arange(1, got[1].numel() + 1, dtype=torch.float32)
    if got[1].numel():
        got[1].backward(upstream)
        assert np.array_equal(weights.grad.numpy(), oracle.sort_backward(upstream.numpy(), want[5], weights.shape))


def test_cpu_route_sort_literal_and_disagreeing_counts():
    from halo_amd.kernels.moe_route_sort import RECEIVE_COUNTS_DISAGREE, NONLOCAL_EXPERT_ID_MESSAGE, sort_routing_by_expert

    experts = torch.tensor([[0, -1, 2], [2, 0, 3], [-1, 3, -1], [-1, -1, 0]])
    weights = torch.arange(12, dtype=torch.float32).view(4, 3)
    tok, w, eids, offs, inv_map = sort_routing_by_expert(experts, weights, 4, (3, 0, 2, 2))
    assert tok.tolist() == [0, 1, 3, 0, 1, 1, 2] and eids.tolist() == [0, 0, 0, 2, 2, 3, 3]
    assert offs.tolist() == [3, 3, 5, 7] and offs.dtype == torch.int32
    assert w.tolist() == [0.0, 4.0, 11.0, 2.0, 3.0, 5.0, 7.0]
    assert inv_map.tolist() == [[0, 3, 7], [1, 4, 5], [6, 7, 7], [2, 7, 7]]
    with pytest.raises(RuntimeError, match=RECEIVE_COUNTS_DISAGREE):
        sort_routing_by_expert(experts, weights, 4, (3, 0, 2, 1))
    with pytest.raises(RuntimeError, match="outside the local experts"):
        sort_routing_by_expert(experts, weights, 4, None)
    assert NONLOCAL_EXPERT_ID_MESSAGE.startswith("An expert id outside")


def test_cpu_histogram_and_inv_map():
    from halo_amd.kernels.histogram import accumulate_bincount, sync_free_bincount
    from halo_amd.kernels.moe_permute import build_inv_map
    from oracle import route_sort as oracle

    g = torch.Generator().manual_seed(0)
    idx = torch.randint(-2, 40, (500,), generator=g)
    w = torch.rand(500, generator=g)
    inside = (idx >= 0) & (idx < 32)  # the reference leaves out-of-range values to its caller; here they are ignored
    assert np.array_equal(sync_free_bincount(idx, 32, dtype=torch.long).numpy(),
                          oracle.bincount(idx[inside].numpy(), 32, dtype=np.int64))
    torch.testing.assert_close(sync_free_bincount(idx, 32, weights=w),
                               torch.from_numpy(oracle.bincount(idx[inside].numpy(), 32, weights=w[inside].numpy())))
    counter = accumulate_bincount(None, idx, 32)
    assert torch.equal(accumulate_bincount(counter, idx, 32), 2 * sync_free_bincount(idx, 32))
    tok = torch.tensor([3, 0, 3, 1, 0, 3])
    assert np.array_equal(build_inv_map(tok, 5, 3).numpy(), oracle.build_inv_map(tok.numpy(), 5, 3))
    assert build_inv_map(torch.zeros(0, dtype=torch.long), 3, 2).tolist() == [[0, 0]] * 3


@pytest.mark.parametrize("dtype", (torch.float32, torch.bfloat16, torch.float64), ids=("fp32", "bf16", "fp64"))
def test_cpu_permute_and_combine_match_the_oracle(dtype):
    from halo_amd.kernels.moe_permute import (MoEExpertBiasGather, MoEGatherPermute, MoEWeightedUnpermute,
                                              gather_reduce_rows, padded_gather_reduce)
    from halo_amd.kernels.moe_route_sort import sort_routing_by_expert
    from oracle import permute as oracle

    case = ROUTING_CASES[1]
    experts, gates, counts = make_receive(case, seed=5)
    tok, w, eids, offs, inv_map = sort_routing_by_expert(experts, gates, case.local_experts, counts)
    g = torch.Generator().manual_seed(1)
    hidden = 48
    tokens = torch.randn(case.rows, hidden, generator=g).to(dtype).requires_grad_(True)
    rows = MoEGatherPermute.apply(tokens, tok, inv_map)
    assert torch.equal(rows, oracle.gather_rows(tokens.detach(), tok))
    y = torch.randn(tok.numel(), hidden, generator=g).to(dtype).requires_grad_(True)
    wd = w.to(dtype).detach().requires_grad_(True)
    out = MoEWeightedUnpermute.apply(y, wd, tok, inv_map)
    tol = dict(rtol=2e-2, atol=2e-2) if dtype == torch.bfloat16 else dict(rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(out, oracle.gather_reduce(y.detach(), inv_map, wd.detach()), **tol)
    dout = torch.randn(case.rows, hidden, generator=g).to(dtype)
    (out.float().mul(dout.float()).sum() + rows.float().mul(y.detach().float()).sum()).backward()
    want_dy, want_dw = oracle.weighted_unpermute_backward(dout, y.detach(), wd.detach(), tok)
    torch.testing.assert_close(y.grad, want_dy, **tol)
    torch.testing.assert_close(wd.grad, want_dw.to(dtype), **tol)
    torch.testing.assert_close(tokens.grad, oracle.gather_reduce(y.detach(), inv_map), **tol)
    # the sentinel example of the reference's test: positions at or past len(src) add nothing
    src = torch.arange(1.0, 7.0).view(6, 1)
    assert gather_reduce_rows(src, torch.tensor([[0, 3], [5, 6], [6, 6]])).view(-1).tolist() == [5.0, 6.0, 0.0]
    assert torch.equal(padded_gather_reduce(src, torch.tensor([[1, 6]])), torch.tensor([[2.0]]))
    bias = torch.randn(case.local_experts, hidden, generator=g).to(dtype).requires_grad_(True)
    gathered = MoEExpertBiasGather.apply(bias, eids)
    assert torch.equal(gathered, oracle.bias_gather(bias.detach(), eids))
    gathered.backward(y.detach())
    torch.testing.assert_close(bias.grad, oracle.bias_gather_backward(y.detach(), eids, case.local_experts), **tol)


@pytest.mark.parametrize("counts", ((7, 33, 0, 1, 64, 0), (0, 0, 0, 0, 105, 0), (5,)))
def test_cpu_grouped_mm_matches_the_per_group_loop(counts):
    from halo_amd.kernels.grouped_mm import grouped_mm
    from oracle import grouped_mm as oracle

    g = torch.Generator().manual_seed(sum(counts))
    k, n, total = 24, 40, sum(counts)
    a = torch.randn(total, k, generator=g, requires_grad=True)
    b = torch.randn(len(counts), k, n, generator=g, requires_grad=True)
    dout = torch.randn(total, n, generator=g)
    offs = torch.tensor(np.cumsum(counts), dtype=torch.int32)
    out = grouped_mm(a, b, offs=offs)
    out.backward(dout)
    ends = np.cumsum(counts).astype(np.int32)
    torch.testing.assert_close(out, oracle.grouped_mm(a.detach(), b.detach(), ends))
    torch.testing.assert_close(a.grad, oracle.grouped_mm_dgrad(dout, b.detach(), ends))
    torch.testing.assert_close(b.grad, oracle.grouped_mm_wgrad(a.detach(), dout, ends))
    for e, c in enumerate(counts):
        assert (c == 0) == (not b.grad[e].any())
    a16, b16 = a.detach().bfloat16(), b.detach().bfloat16()
    bf = grouped_mm(a16, b16, offs=offs)
    assert bf.dtype == torch.bfloat16  # fp32 accumulation, one rounding
    assert torch.equal(bf, oracle.grouped_mm(a16.float(), b16.float(), ends).bfloat16())


@pytest.mark.parametrize("name", ("silu", "gelu_tanh", "clamped_silu", "silu_then_clamp", "gptoss"))
def test_cpu_glu_is_the_eager_form_and_matches_the_oracle(name):
    from halo_amd.kernels.fused_glu import _ACTIVATION_PROBE_INPUT, GluCombine
    from oracle import glu as oracle

    combine = {"silu": GluCombine.silu(), "gelu_tanh": GluCombine.gelu_tanh(),
               "clamped_silu": GluCombine.clamped_silu(7.0), "silu_then_clamp": GluCombine.clamped_silu(7.0, clamp_activated=True),
               "gptoss": GluCombine.gptoss(1.702, 7.0)}[name]
    probe = torch.tensor(_ACTIVATION_PROBE_INPUT)
    gate = probe.repeat(len(probe), 1).clone().requires_grad_(True)
    up = probe.repeat(len(probe), 1).t().contiguous().requires_grad_(True)
    args = (combine.activation, combine.alpha, combine.limit, combine.clamp_activated, combine.up_plus_one)
    out = combine(gate, up)
    torch.testing.assert_close(out, oracle.glu_forward(gate.detach(), up.detach(), *args), rtol=1e-5, atol=1e-6)
    packed = torch.cat([gate.detach(), up.detach()], dim=-1).requires_grad_(True)
    torch.testing.assert_close(combine.packed(packed), out, rtol=1e-6, atol=1e-30)  # strided halves: last-bit only
    weight = torch.linspace(0.1, 1.1, len(probe))
    torch.testing.assert_close(combine.packed_weighted(packed, weight), out * weight[:, None])
    out.backward(torch.ones_like(out))
    want_dg, want_du = oracle.glu_backward(gate.detach(), up.detach(), torch.ones_like(out), *args)
    # away from the clamp bounds (autograd's clamp has its own sub-gradient convention at the bound itself)
    inside = (gate.detach().abs() != 7.0) & (up.detach().abs() != 7.0)
    torch.testing.assert_close(gate.grad[inside], want_dg[inside], rtol=1e-4, atol=1e-6)
    torch.testing.assert_close(up.grad[inside], want_du[inside], rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("mode", (0, 1))
@pytest.mark.parametrize("dtype", (torch.float32, torch.bfloat16), ids=("fp32", "bf16"))
def test_cpu_router_gate_matches_the_oracle_with_ties_to_the_lower_index(mode, dtype):
    from halo_amd.kernels.router import fused_topk_gate
    from oracle import router as oracle

    g = torch.Generator().manual_seed(3)
    logits = (torch.randn(64, 32, generator=g) * 0.5).to(dtype)  # bf16: ties are common
    logits[0] = 0.0
    leaf = logits.clone().requires_grad_(True)
    idx, w = fused_topk_gate(leaf, 4, mode=mode, normalize=True, eps=1e-20)
    want_idx, want_w = oracle.route(logits, 4, mode, True, 1e-20)
    assert torch.equal(idx, want_idx) and idx[0].tolist() == [0, 1, 2, 3]
    assert w.dtype == torch.float32 and torch.equal(w, want_w)
    upstream = torch.randn(w.shape, generator=g)
    w.backward(upstream)
    want = oracle.route_backward(logits, idx, upstream, mode, True, 1e-20)
    torch.testing.assert_close(leaf.grad.float(), want.float(), rtol=2e-2, atol=2e-3)


@pytest.mark.parametrize("cfg_name", ("CONFIG1", "CONFIG2_SMALL", "CONFIG4_SMALL"))
def test_cpu_layer_forward_backward_matches_the_per_expert_loop(cfg_name):
    """The MoE block on CPU tensors (the operators above under the layer's orchestration, grouped path) against the
    oracle's per-expert loop with the same selection: forward and every gradient, BASELINE's tolerances."""
    import tests.cases as cases
    from halo_amd.kernels.router import SOFTMAX_ALL, SOFTMAX_TOPK, fused_topk_gate
    from tests.test_gpu_layer import _build_layer, _check, _oracle_run

    cfg = getattr(cases, cfg_name)
    skew = dict(zipf_alpha=1.2, empty_experts=3) if cfg.router == "softmax_topk" else {}
    inputs = cases.make_layer_inputs(cfg, **skew)
    layer = _build_layer(cfg, inputs, torch.device("cpu"))
    x = inputs["x"].clone().requires_grad_(True)
    result = layer(x)
    out = result[0] if isinstance(result, tuple) else result
    out.backward(inputs["grad_out"])
    with torch.no_grad():
        logits = layer._linear_router_logits(x.detach())
        mode = SOFTMAX_TOPK if cfg.router == "softmax_topk" else SOFTMAX_ALL
        idx, _ = fused_topk_gate(logits, cfg.top_k, mode=mode, normalize=True, eps=0.0)
    want_out, _, want_grads = _oracle_run(cfg, inputs, idx)
    tol = 1e-4 if cfg.dtype == torch.float32 else 2e-2
    _check("out", out, want_out, tol)
    _check("grad x", x.grad, want_grads["x"], tol)
    _check("grad router_weight", getattr(layer, layer._ROUTER_ATTR).weight.grad, want_grads["router_weight"], tol)
    for name in inputs["params"]:
        attr = name.replace("gate_proj", "gate_proj_gmm").replace("up_proj", "up_proj_gmm") \
            if cfg.router == "softmax_topk" else name
        _check(f"grad {name}", getattr(layer, attr).grad, want_grads[name], tol)


@pytest.mark.parametrize("fuse_gate_up", (True, False), ids=("gate_up_as_one_product", "gate_and_up_apart"))
def test_cpu_layer_with_a_gated_shared_expert_matches_the_oracle(fuse_gate_up):
    """Qwen3.5's block with its sigmoid-gated shared expert on CPU tensors: the shared expert's gate and up projections
    as one product over the two weights side by side (the default) or as two, the gate through ``sigmoid_row_gate``'s
    tensor-operation form; output and gradients against the oracle's loop with the same selection."""
    import tests.cases as cases
    from halo_amd.kernels.router import fused_topk_gate
    from halo_amd.moe_layer.layer import sigmoid_row_gate
    from oracle import moe_layer as oracle
    from tests.test_gpu_layer import _check, _layer_with_shared_expert

    cfg = cases.CONFIG2_SMALL
    inputs = cases.make_layer_inputs(cfg)
    cpu = torch.device("cpu")
    layer = _layer_with_shared_expert(cfg, inputs, cpu, gated=True, fuse=True)
    layer.fuse_shared_gate_up = fuse_gate_up
    x = inputs["x"].clone().requires_grad_(True)
    out = layer(x)
    out.backward(inputs["grad_out"])
    with torch.no_grad():
        idx, _ = fused_topk_gate(layer._linear_router_logits(x.detach()), cfg.top_k, normalize=True, eps=0.0)
    f = lambda t: t.detach().float().requires_grad_(True)
    xs, wr = f(inputs["x"]), f(inputs["router_weight"])
    params = {k: f(v) for k, v in inputs["params"].items()}
    shared = {n: f(getattr(layer.shared_expert, n).weight) for n in ("gate_proj", "up_proj", "down_proj")}
    shared["shared_expert_gate"] = f(layer.shared_expert_gate.weight)
    want, _, _, _ = oracle.moe_layer_forward(xs, wr, params, oracle.Glu(cfg.glu), cfg.top_k, normalize=True, eps=0.0,
                                             indices=idx, shared=shared)
    want.backward(inputs["grad_out"].float())
    tol = 1e-4 if cfg.dtype == torch.float32 else 2e-2
    _check("out", out, want.detach(), tol)
    _check("grad x", x.grad, xs.grad, tol)
    for name in ("gate_proj", "up_proj", "down_proj"):
        _check(f"grad shared {name}", getattr(layer.shared_expert, name).weight.grad, shared[name].grad, tol)
    _check("grad shared gate", layer.shared_expert_gate.weight.grad, shared["shared_expert_gate"].grad, tol)
    # the gate helper on CPU tensors is the tensor operations themselves
    g = torch.Generator().manual_seed(5)
    rows, w = torch.randn(33, 24, generator=g), torch.randn(1, 24, generator=g)
    assert torch.equal(sigmoid_row_gate(rows, w), torch.sigmoid(rows @ w.t()).view(-1))


def test_cpu_gemma4_experts_drop_in_matches_the_hf_module():
    """``EPGemma4MoELayer`` wraps transformers' ``Gemma4TextExperts`` (experts only, routing handed in) and returns its
    output and gradients, the gate weights' included, in fp32 on the CPU."""
    from transformers.models.gemma4.configuration_gemma4 import Gemma4TextConfig
    from transformers.models.gemma4.modeling_gemma4 import Gemma4TextExperts

    from halo_amd.moe_layer import MOE_LAYER_MAP, EPGemma4MoELayer, single_process_ep_config

    torch.manual_seed(0)
    config = Gemma4TextConfig(hidden_size=64, moe_intermediate_size=48, num_experts=8, top_k_experts=2,
                              hidden_activation="gelu_pytorch_tanh", num_hidden_layers=1)
    hf = Gemma4TextExperts(config)
    with torch.no_grad():
        hf.gate_up_proj.normal_(0, 0.1)
        hf.down_proj.normal_(0, 0.1)
    assert MOE_LAYER_MAP["Gemma4TextExperts"] is EPGemma4MoELayer
    layer = EPGemma4MoELayer(hf, single_process_ep_config())
    assert layer._glu_combine_name() == "gelu_tanh" and layer.gate_up_proj.shape == (8, 64, 96)
    assert {n for n, _ in layer.expert_named_params()} == {"gate_up_proj", "down_proj"}
    x = torch.randn(40, 64, requires_grad=True)
    probs, idx = torch.topk(torch.softmax(torch.randn(40, 8), -1), 2, dim=-1)
    w = (probs / probs.sum(-1, keepdim=True)).requires_grad_()
    out, want = layer(x, idx, w), hf(x, idx, w)
    torch.testing.assert_close(out, want, rtol=1e-5, atol=1e-6)
    upstream = torch.randn_like(out)
    for got, ref in zip(torch.autograd.grad(out, (x, w), upstream), torch.autograd.grad(want, (x, w), upstream)):
        torch.testing.assert_close(got, ref, rtol=1e-4, atol=1e-6)
