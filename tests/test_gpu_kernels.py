"""GPU parity tests, op by op: every HIP kernel through the C ABI (via the ``halo_amd.kernels`` ops) against the CPU
oracle on the same seeded inputs.  Integer outputs are compared bit for bit; floating-point outputs within the
tolerance written next to each check."""

import json
import os

import numpy as np
import pytest
import torch

from tests.cases import ROUTING_CASES, make_receive

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def max_rel(actual, reference):
    """Largest elementwise error relative to the reference's peak."""
    a, r = actual.detach().double().cpu(), reference.detach().double().cpu()
    return ((a - r).abs().max() / r.abs().max().clamp(min=1e-30)).item()


def fro_rel(actual, reference):
    a, r = actual.detach().double().cpu(), reference.detach().double().cpu()
    return ((a - r).norm() / r.norm()).item()


def cosine(actual, reference):
    a, r = actual.detach().double().cpu().flatten(), reference.detach().double().cpu().flatten()
    return (torch.dot(a, r) / (a.norm() * r.norm())).item()


# ------------------------------------------------------------------------------------------------- routing sort

@pytest.mark.parametrize("case", ROUTING_CASES, ids=lambda c: c.name)
def test_route_sort_matches_oracle_bit_for_bit(device, case):
    from halo_amd.kernels.moe_route_sort import sort_routing_by_expert
    from oracle import route_sort as oracle

    experts, weights, counts = make_receive(case, seed=ROUTING_CASES.index(case))
    want = oracle.argsort_routing(experts.numpy(), weights.numpy(), case.local_experts, counts)
    leaf = weights.to(device).requires_grad_(True)
    got = sort_routing_by_expert(experts.to(device), leaf, case.local_experts, counts)
    names = ("sorted_token_idx", "sorted_weights", "sorted_expert_ids", "offs", "inv_map")
    for name, g, w in zip(names, got, want):
        g = g.detach().cpu().numpy()
        assert g.dtype == w.dtype and g.shape == w.shape, f"{case.name}: {name} {g.dtype}{g.shape} vs {w.dtype}{w.shape}"
        if g.dtype == np.float32:
            g, w = g.view(np.int32), w.view(np.int32)
        assert np.array_equal(g, w), f"{case.name}: {name}"
    # gate-weight gradient: each slot reads its sorted position's gradient, dropped slots read zero
    upstream = torch.randn(got[1].shape, generator=torch.Generator().manual_seed(1))
    (grad,) = torch.autograd.grad(got[1], leaf, upstream.to(device))
    want_grad = oracle.sort_backward(upstream.numpy(), want[5], tuple(experts.shape))
    assert np.array_equal(grad.cpu().numpy().view(np.int32), want_grad.view(np.int32))


def test_route_sort_literal_known_answer(device):
    from halo_amd.kernels.moe_route_sort import sort_routing_by_expert

    with open(os.path.join(GOLDEN, "route_sort_literal.json")) as f:
        gold = json.load(f)
    experts = torch.tensor(gold["experts"], device=device)
    weights = torch.tensor(gold["weights"], device=device)
    got = sort_routing_by_expert(experts, weights, gold["num_local_experts"], tuple(gold["counts"]))
    for name, g in zip(("sorted_token_idx", "sorted_weights", "sorted_expert_ids", "offs", "inv_map"), got):
        assert g.cpu().tolist() == gold[name], name


def test_route_sort_count_flag_and_int32_ids_and_bf16_weights(device):
    """The device flag the async assert reads: 1 when the local slots number the host count (only the sum is read),
    0 when they do not -- checked on the flag itself, so no assert ever fires on the GPU."""
    from halo_amd.kernels.moe_route_sort import counting_sort_raw, sort_routing_by_expert
    from oracle import route_sort as oracle

    case = ROUTING_CASES[1]
    experts, weights, counts = make_receive(case, seed=1)
    e, w = experts.to(device), weights.to(device)
    for n_valid, expect in ((sum(counts), 1), (sum(counts) - 1, 0), (sum(counts) + 1, 0)):
        *_, ok = counting_sort_raw(e, w, case.local_experts, n_valid)
        assert int(ok.item()) == expect
    moved = (counts[0] - 1, counts[1] + 1, *counts[2:])
    a = sort_routing_by_expert(e, w, case.local_experts, moved)
    b = sort_routing_by_expert(e, w, case.local_experts, counts)
    assert all(torch.equal(x, y) for x, y in zip(a, b))
    with pytest.raises(ValueError, match="2 receive counts for 4 local experts"):
        sort_routing_by_expert(torch.zeros(2, 2, dtype=torch.long, device=device),
                               torch.rand(2, 2, device=device), 4, (3, 1))
    # int32 ids and bf16 weights are copied bit for bit too
    want = oracle.argsort_routing(experts.numpy().astype(np.int32), weights.bfloat16().view(torch.int16).numpy(),
                                  case.local_experts, counts)
    got = sort_routing_by_expert(e.int(), w.bfloat16(), case.local_experts, counts)
    assert got[2].dtype == torch.int32 and got[1].dtype == torch.bfloat16
    assert np.array_equal(got[1].view(torch.int16).cpu().numpy(), want[1])
    assert np.array_equal(got[2].cpu().numpy(), want[2])


def test_route_sort_is_bit_reproducible(device):
    from halo_amd.kernels.moe_route_sort import sort_routing_by_expert

    case = ROUTING_CASES[-1]
    experts, weights, counts = make_receive(case, seed=5)
    e, w = experts.to(device), weights.to(device)
    first = sort_routing_by_expert(e, w, case.local_experts, counts)
    for _ in range(3):
        again = sort_routing_by_expert(e, w, case.local_experts, counts)
        assert all(torch.equal(x, y) for x, y in zip(first, again))


def test_bincount(device):
    from halo_amd.kernels.histogram import accumulate_bincount, sync_free_bincount

    g = torch.Generator().manual_seed(0)
    idx = torch.randint(0, 128, (8192, 8), generator=g)
    want = torch.bincount(idx.flatten(), minlength=128)
    assert torch.equal(sync_free_bincount(idx.to(device), 128, dtype=torch.long).cpu(), want)
    got = sync_free_bincount(idx.to(device), 128)
    assert got.dtype == torch.float32 and torch.equal(got.cpu(), want.float())
    w = torch.rand(idx.shape, generator=g)
    want_w = torch.zeros(128, dtype=torch.float64).scatter_add_(0, idx.flatten(), w.flatten().double())
    got_w = sync_free_bincount(idx.to(device), 128, weights=w.to(device))
    assert max_rel(got_w, want_w) < 1e-5  # fp32 sums of ~512 terms each, order not fixed
    counter = accumulate_bincount(None, idx.to(device), 128)
    counter = accumulate_bincount(counter, idx.to(device), 128)
    assert torch.equal(counter.cpu(), 2 * want.float())


@pytest.mark.parametrize(("n", "size"), ((500_000, 128), (70_000, 8192), (300_000, 65_536), (1000, 100_000),
                                         (0, 9000)))
def test_bincount_with_many_indices_and_many_bins(device, n, size):
    """Beyond one workgroup's reach (65536 indices, 8192 bins) the histogram takes many workgroups: exact counts in
    int64 and fp32, weighted sums to fp32 rounding, out-of-range indices ignored.  The reference calls it with a
    token count as ``size`` (``moe_permute.py:75-89``)."""
    from halo_amd.kernels.histogram import sync_free_bincount
    from oracle import route_sort as oracle

    g = torch.Generator().manual_seed(n + size)
    idx = torch.randint(-3, size + 3, (n,), generator=g)  # a few values either side of the range
    inside = idx[(idx >= 0) & (idx < size)]
    want = torch.from_numpy(oracle.bincount(inside.numpy(), size, np.int64))
    got = sync_free_bincount(idx.to(device), size, dtype=torch.long)
    assert got.dtype == torch.int64 and torch.equal(got.cpu(), want)
    assert torch.equal(sync_free_bincount(idx.to(device), size).cpu(), want.float())
    w = torch.rand(n, generator=g)
    want_w = torch.zeros(size, dtype=torch.float64).scatter_add_(0, inside, w[(idx >= 0) & (idx < size)].double())
    got_w = sync_free_bincount(idx.to(device), size, weights=w.to(device))
    assert torch.allclose(got_w.cpu().double(), want_w, rtol=1e-4, atol=1e-4)


def test_expert_path_and_inv_map_never_synchronise_the_host(device):
    """With torch's sync debug mode at ``error`` (the reference's ``cuda_syncs_are_errors``,
    ``tests/common/harness.py:118-126``) an op that makes the host wait for the device raises.  A layer's forward and
    backward, ``build_inv_map`` and the histograms run under it; a known synchronising op is checked first, so that a
    torch build which does not honour the mode fails this test's premise rather than passing it silently."""
    from halo_amd.kernels.histogram import sync_free_bincount
    from halo_amd.kernels.moe_permute import build_inv_map
    from halo_amd.moe_layer import EPQwen3_5MoELayer

    g = torch.Generator().manual_seed(8)
    tokens, hidden, experts, top_k, ffn = 512, 256, 16, 4, 128
    x = torch.randn(tokens, hidden, generator=g).bfloat16().to(device).requires_grad_(True)
    layer = EPQwen3_5MoELayer.from_weights(
        router_weight=(torch.randn(experts, hidden, generator=g) * 0.02).bfloat16().to(device), top_k=top_k,
        gate_up_proj=(torch.randn(experts, hidden, 2 * ffn, generator=g) * 0.02).bfloat16().to(device),
        down_proj=(torch.randn(experts, ffn, hidden, generator=g) * 0.02).bfloat16().to(device))
    grad = torch.randn(tokens, hidden, generator=g).bfloat16().to(device)
    sorted_tokens = torch.randint(0, tokens, (3000,), generator=g).to(device)
    layer(x).backward(grad)  # once outside: allocator warm-up and the library load are not the subject
    torch.cuda.synchronize()
    torch.cuda.set_sync_debug_mode("error")
    try:
        with pytest.raises(RuntimeError):
            sorted_tokens.sum().item()  # the premise: a readback is an error in this mode
        x.grad = None
        out = layer(x)
        out.backward(grad)
        inv_map = build_inv_map(sorted_tokens, tokens, 16)
        counts = sync_free_bincount(sorted_tokens, 100_000, dtype=torch.long)
    finally:
        torch.cuda.set_sync_debug_mode("default")
    assert out.shape == x.shape and x.grad is not None
    assert inv_map.shape == (tokens, 16) and int(counts.sum()) == 3000


# -------------------------------------------------------------------------------------------- permute / combine

DTYPE_TOLS = ((torch.float32, 1e-5), (torch.bfloat16, 2e-2))
# top_k 2, 4 and 8 take the kernels with the slot count fixed at compile time, 3 and 6 the runtime-count loop
ROUTINGS = ((517, 8, 2816, 0.5), (64, 4, 100, 1.0), (33, 8, 1025, 0.1), (300, 8, 2048, 1.0), (96, 2, 520, 0.7),
            (50, 6, 512, 0.6), (40, 3, 264, 0.8), (200, 4, 768, 0.4))


def _routing(n_tokens, top_k, n_sorted, seed):
    from oracle import route_sort as oracle

    g = torch.Generator().manual_seed(seed)
    slots = torch.arange(n_tokens).repeat_interleave(top_k)
    token_idx = slots[torch.randperm(slots.numel(), generator=g)[:n_sorted]]
    return token_idx, torch.from_numpy(oracle.build_inv_map(token_idx.numpy(), n_tokens, top_k))


@pytest.mark.parametrize(("dtype", "tol"), DTYPE_TOLS, ids=("fp32", "bf16"))
@pytest.mark.parametrize(("n_tokens", "top_k", "hidden", "fill"), ROUTINGS)
def test_weighted_unpermute_and_permute_match_oracle(device, dtype, tol, n_tokens, top_k, hidden, fill):
    from halo_amd.kernels.moe_permute import MoEGatherPermute, MoEWeightedUnpermute
    from oracle import permute as oracle

    n_sorted = int(n_tokens * top_k * fill)
    token_idx, inv_map = _routing(n_tokens, top_k, n_sorted, seed=n_tokens)
    g = torch.Generator().manual_seed(n_tokens + 1)
    y = torch.randn(n_sorted, hidden, generator=g).to(dtype)
    w = torch.rand(n_sorted, generator=g).to(dtype)
    grad = torch.randn(n_tokens, hidden, generator=g).to(dtype)
    yd, wd = y.to(device).requires_grad_(True), w.to(device).requires_grad_(True)
    out = MoEWeightedUnpermute.apply(yd, wd, token_idx.to(device), inv_map.to(device))
    out.backward(grad.to(device))
    want_out = oracle.gather_reduce(y, inv_map, w, out_dtype=torch.float64)
    want_gy, want_gw = oracle.weighted_unpermute_backward(grad.double(), y.double(), w.double(), token_idx)
    for name, got, want in (("out", out, want_out), ("grad_expert", yd.grad, want_gy), ("grad_w", wd.grad, want_gw)):
        assert got.dtype == dtype
        assert max_rel(got, want) < tol, f"{name}: {max_rel(got, want):.3e}"
        if dtype == torch.bfloat16:
            # a result accumulated in fp32 is the exact result rounded once: within 1.1x of the bf16 rounding floor
            floor = fro_rel(want.to(torch.bfloat16), want)
            assert fro_rel(got, want) <= 1.1 * floor + 1e-12, (name, fro_rel(got, want), floor)
    # permute forward (bit copy) and backward (unweighted gather-sum)
    tokens = torch.randn(n_tokens, hidden, generator=g).to(dtype)
    td = tokens.to(device).requires_grad_(True)
    sorted_tokens = MoEGatherPermute.apply(td, token_idx.to(device), inv_map.to(device))
    assert torch.equal(sorted_tokens.cpu(), oracle.gather_rows(tokens, token_idx))
    gs = torch.randn(n_sorted, hidden, generator=g).to(dtype)
    sorted_tokens.backward(gs.to(device))
    want_b = oracle.gather_reduce(gs, inv_map, out_dtype=torch.float64)
    assert max_rel(td.grad, want_b) < tol
    if dtype == torch.bfloat16:
        assert torch.equal(td.grad.cpu(), want_b.to(torch.bfloat16))  # sums of <= 8 bf16 values: fp32 is exact


def test_gather_reduce_sentinel_known_answer_and_strided_inputs(device):
    from halo_amd.kernels.moe_permute import MoEGatherPermute, MoEWeightedUnpermute, gather_reduce_rows
    from oracle import permute as oracle

    src = torch.arange(1, 7, device=device, dtype=torch.float32).unsqueeze(-1).expand(6, 3).contiguous()
    inv_map = torch.tensor([[0, 3], [5, 6], [6, 6]], device=device)  # 6 == len(src): sentinel
    assert gather_reduce_rows(src, inv_map)[:, 0].tolist() == [5.0, 6.0, 0.0]
    # strided operands: expert_out / weights as views, grad_out and tokens as [:, :H] views of padded buffers
    n_tokens, top_k, hidden = 257, 8, 704
    n_sorted = n_tokens * top_k // 2
    token_idx, inv_map = _routing(n_tokens, top_k, n_sorted, seed=0)
    g = torch.Generator().manual_seed(0)
    wide_out = torch.randn(n_sorted, 2 * hidden, generator=g)
    wide_w = torch.rand(n_sorted, 2, generator=g)
    wide_grad = torch.randn(n_tokens, hidden + 64, generator=g)
    yd = wide_out.to(device).requires_grad_(True)
    wd = wide_w.to(device).requires_grad_(True)
    y_view, w_view = yd[:, :hidden], wd[:, 0]
    grad_view = wide_grad.to(device)[:, :hidden]
    assert not y_view.is_contiguous() and grad_view.stride() == (hidden + 64, 1)
    out = MoEWeightedUnpermute.apply(y_view, w_view, token_idx.to(device), inv_map.to(device))
    out.backward(grad_view)
    y, w, grad = wide_out[:, :hidden], wide_w[:, 0], wide_grad[:, :hidden]
    assert max_rel(out, oracle.gather_reduce(y, inv_map, w, out_dtype=torch.float64)) < 1e-5
    want_gy, want_gw = oracle.weighted_unpermute_backward(grad.double(), y.double(), w.double(), token_idx)
    assert max_rel(yd.grad[:, :hidden], want_gy) < 1e-5 and max_rel(wd.grad[:, 0], want_gw) < 1e-5
    padded = torch.randn(n_tokens, 768, generator=g).bfloat16().to(device)  # 704 columns of a 768-wide buffer
    got = MoEGatherPermute.apply(padded[:, :hidden], token_idx.to(device), inv_map.to(device))
    assert torch.equal(got, padded[:, :hidden][token_idx.to(device)])


def test_empty_dispatch_and_no_weight_grad(device):
    from halo_amd.kernels.moe_permute import MoEWeightedUnpermute, build_inv_map

    out = MoEWeightedUnpermute.apply(torch.zeros(0, 16, device=device), torch.zeros(0, device=device),
                                     torch.zeros(0, dtype=torch.long, device=device),
                                     torch.zeros(0, 8, dtype=torch.long, device=device))
    assert out.shape == (0, 16)
    inv = build_inv_map(torch.empty(0, dtype=torch.long, device=device), 8, 4)
    assert inv.shape == (8, 4) and bool((inv == 0).all())
    got = MoEWeightedUnpermute.apply(torch.empty(0, 5, device=device), torch.empty(0, device=device),
                                     torch.empty(0, dtype=torch.long, device=device), inv)
    assert got.shape == (8, 5) and not got.any()
    # weights needing no gradient: expert_out is not kept, the expert gradient is the same bit for bit
    token_idx, inv_map = _routing(129, 8, 516, seed=1)
    g = torch.Generator().manual_seed(2)
    y = torch.randn(516, 1100, generator=g).bfloat16().to(device)
    w = torch.rand(516, generator=g).bfloat16().to(device)
    grad = torch.randn(129, 1100, generator=g).bfloat16().to(device)
    grads = {}
    for need in (True, False):
        yy, ww = y.clone().requires_grad_(True), w.clone().requires_grad_(need)
        saved = []
        with torch.autograd.graph.saved_tensors_hooks(lambda t: saved.append(t) or t, lambda t: t):
            o = MoEWeightedUnpermute.apply(yy, ww, token_idx.to(device), inv_map.to(device))
        o.backward(grad)
        grads[need] = yy.grad
        assert any(t.shape == y.shape for t in saved) == need
    assert torch.equal(grads[True], grads[False])


def test_build_inv_map_matches_oracle(device):
    from halo_amd.kernels.moe_permute import build_inv_map
    from oracle import route_sort as oracle

    token_idx, inv_map = _routing(2000, 8, 9000, seed=7)
    assert torch.equal(build_inv_map(token_idx.to(device), 2000, 8).cpu(), inv_map)


@pytest.mark.parametrize(("rows", "width", "skew"), ((5000, 2880, 0), (20000, 360, 3), (700, 100, 0), (9, 64, 0)),
                         ids=("even", "one_expert_holds_most", "unaligned_width", "tiny"))
def test_expert_bias_gather(device, rows, width, skew):
    from halo_amd.kernels.moe_permute import MoEExpertBiasGather
    from oracle import permute as oracle

    g = torch.Generator().manual_seed(3)
    for dtype, tol in DTYPE_TOLS:
        ids = torch.randint(0, 32, (rows,), generator=g)
        if skew:  # four rows in five go to one expert
            ids = torch.where(torch.rand(rows, generator=g) < 0.8, torch.full_like(ids, skew), ids)
        eids = torch.sort(ids).values
        eids = eids[(eids != 7) & (eids != 31)]  # two idle experts, one of them last
        bias = torch.randn(32, width, generator=g).to(dtype)
        grad = torch.randn(eids.numel(), width, generator=g).to(dtype)
        bd = bias.to(device).requires_grad_(True)
        out = MoEExpertBiasGather.apply(bd, eids.to(device))
        assert torch.equal(out.cpu(), oracle.bias_gather(bias, eids))
        out.backward(grad.to(device))
        want = oracle.bias_gather_backward(grad.double(), eids, 32)
        assert max_rel(bd.grad, want) < tol
        assert not bd.grad[7].any() and not bd.grad[31].any()
        # the same sums without a workspace (one workgroup per expert and column chunk), through the C-ABI
        plain = _colsum_without_workspace(grad.to(device), eids.to(device), 32)
        assert max_rel(plain, want) < tol
        assert not plain[7].any() and not plain[31].any()


def _colsum_without_workspace(grad, eids, num_experts):
    from halo_amd import _lib

    out = torch.empty((num_experts, grad.shape[1]), dtype=grad.dtype, device=grad.device)
    with _lib.on_device(grad.device):
        _lib.call("hmoe_expert_colsum", _lib.ptr(grad), _lib.ptr(eids), grad.shape[0], grad.shape[1], num_experts,
                  _lib.dtype_id(grad.dtype), _lib.ptr(out), None, _lib.stream_ptr(grad.device))
    return out


def test_expert_bias_gradient_in_row_blocks(device):
    """The blocked column sums: expert boundaries on and off the 512-row block edges, an expert spanning many blocks,
    many experts inside one block, idle experts first, in the middle and last; twice the same bits."""
    from halo_amd.kernels.moe_permute import MoEExpertBiasGather
    from oracle import permute as oracle

    counts = [0, 512, 512, 0, 0, 1, 3000, 7, 0, 505, 1024, 1, 1, 1, 0, 2, 600, 0]
    eids = torch.repeat_interleave(torch.arange(len(counts)), torch.tensor(counts))
    g = torch.Generator().manual_seed(11)
    for dtype, tol in DTYPE_TOLS:
        for width in (64, 2880, 72):
            grad = torch.randn(eids.numel(), width, generator=g).to(dtype)
            bias = torch.zeros(len(counts), width, dtype=dtype, device=device, requires_grad=True)
            results = []
            for _ in range(2):
                bias.grad = None
                MoEExpertBiasGather.apply(bias, eids.to(device)).backward(grad.to(device))
                results.append(bias.grad.clone())
            assert torch.equal(results[0], results[1])
            want = oracle.bias_gather_backward(grad.double(), eids, len(counts))
            assert max_rel(results[0], want) < tol
            for e, n in enumerate(counts):
                if n == 0:
                    assert not results[0][e].any()
                elif n == 1:  # a single row comes through untouched
                    row = int(sum(counts[:e]))
                    assert torch.equal(results[0][e].cpu(), grad[row])


# ---------------------------------------------------------------------------------------------------- fused GLU

def _combines():
    from halo_amd.kernels.fused_glu import GluCombine

    return {
        "silu": GluCombine.silu(),
        "gelu_tanh": GluCombine.gelu_tanh(),
        "clamped_silu": GluCombine.clamped_silu(2.5),
        "silu_then_clamp": GluCombine.clamped_silu(2.5, clamp_activated=True),
        "gptoss": GluCombine.gptoss(1.702, 7.0),
    }


@pytest.mark.parametrize("name", ("silu", "gelu_tanh", "clamped_silu", "silu_then_clamp", "gptoss"))
@pytest.mark.parametrize(("dtype", "tol"), ((torch.float32, 1e-5), (torch.bfloat16, 2e-2)), ids=("fp32", "bf16"))
@pytest.mark.parametrize(("rows", "width"), ((300, 768), (17, 100), (64, 2880), (5, 1025)))
def test_glu_matches_oracle_packed_and_separate(device, name, dtype, tol, rows, width):
    from oracle import glu as oracle

    combine = _combines()[name]
    kw = dict(activation=combine.activation, alpha=combine.alpha, limit=combine.limit,
              clamp_activated=combine.clamp_activated, up_plus_one=combine.up_plus_one)
    g = torch.Generator().manual_seed(rows * 7 + width)
    gate_up = (torch.randn(rows, 2 * width, generator=g) * 3).to(dtype)
    dout = torch.randn(rows, width, generator=g).to(dtype)
    gate, up = gate_up[:, :width], gate_up[:, width:]
    want = oracle.glu_forward(gate.double(), up.double(), **kw)
    want_dg, want_du = oracle.glu_backward(gate.double(), up.double(), dout.double(), **kw)
    # separate operands
    gd, ud = gate.contiguous().to(device).requires_grad_(True), up.contiguous().to(device).requires_grad_(True)
    out = combine(gd, ud)
    out.backward(dout.to(device))
    assert out.dtype == dtype
    assert max_rel(out, want) < tol and max_rel(gd.grad, want_dg) < tol and max_rel(ud.grad, want_du) < tol
    # packed [gate | up], read in place; the gradient comes back as one buffer and equals the separate form's bits
    pd = gate_up.to(device).requires_grad_(True)
    out_p = combine.packed(pd)
    out_p.backward(dout.to(device))
    assert torch.equal(out_p, out)
    assert torch.equal(pd.grad[:, :width], gd.grad) and torch.equal(pd.grad[:, width:], ud.grad)


@pytest.mark.parametrize("name", ("silu", "gelu_tanh", "gptoss"))
@pytest.mark.parametrize(("dtype", "tol"), ((torch.float32, 1e-5), (torch.bfloat16, 2e-2)), ids=("fp32", "bf16"))
@pytest.mark.parametrize(("rows", "width"), ((300, 768), (64, 512), (129, 360), (17, 100), (5, 1025)))
def test_glu_with_the_gate_weight_folded_in_matches_oracle(device, name, dtype, tol, rows, width):
    """``w[r] * combine(gate, up)[r]`` and its gradients against the oracle's closed forms in fp64 composed with the
    product rule: ``d(gate, up) = glu_backward(gate, up, w * dout)`` and ``dw[r] = <dout[r], combine(gate, up)[r]>``.
    The widths take the three lanes-per-row forms of the backward kernel and the scalar fallback."""
    from oracle import glu as oracle

    combine = _combines()[name]
    kw = dict(activation=combine.activation, alpha=combine.alpha, limit=combine.limit,
              clamp_activated=combine.clamp_activated, up_plus_one=combine.up_plus_one)
    g = torch.Generator().manual_seed(rows * 11 + width)
    gate_up = (torch.randn(rows, 2 * width, generator=g) * 3).to(dtype)
    weight = torch.rand(rows, generator=g).to(dtype)
    dout = torch.randn(rows, width, generator=g).to(dtype)
    gate, up, w64 = gate_up[:, :width].double(), gate_up[:, width:].double(), weight.double().unsqueeze(1)
    act = oracle.glu_forward(gate, up, **kw)
    want = w64 * act
    want_dg, want_du = oracle.glu_backward(gate, up, w64 * dout.double(), **kw)
    want_dw = (dout.double() * act).sum(dim=1)
    pd = gate_up.to(device).requires_grad_(True)
    wd = weight.to(device).requires_grad_(True)
    out = combine.packed_weighted(pd, wd)
    out.backward(dout.to(device))
    assert out.dtype == dtype and wd.grad.dtype == dtype and out.shape == (rows, width)
    assert max_rel(out, want) < tol
    assert max_rel(pd.grad[:, :width], want_dg) < tol and max_rel(pd.grad[:, width:], want_du) < tol
    assert max_rel(wd.grad, want_dw) < tol
    if dtype == torch.bfloat16:  # one rounding of the fp32 product w * act, not a product of two rounded values
        exact = (weight.float().unsqueeze(1).to(device)
                 * oracle.glu_forward(gate_up[:, :width].float(), gate_up[:, width:].float(), **kw).to(device))
        assert fro_rel(out, exact) < 3e-3
    # a weight of one changes nothing: the plain kernel's bits
    ones = torch.ones(rows, dtype=dtype, device=device)
    assert torch.equal(combine.packed_weighted(pd.detach(), ones), combine.packed(pd.detach()))


def test_glu_subgradient_at_the_clamp_bound_and_probe_vector(device):
    from halo_amd.kernels.fused_glu import (GluCombine, is_gelu_tanh_activation, is_silu_activation,
                                            resolve_clamped_glu_mul, resolve_fused_glu_mul)
    from oracle import glu as oracle

    limit = 2.0
    gate = torch.tensor([[limit, limit, -limit, 0.5, limit + 1e-3, 0.0, 0.0, 0.0]], device=device)
    up = torch.tensor([[limit, -limit, limit, limit, 1.0, limit + 1e-3, -limit - 1e-3, 1.0]], device=device)
    gd, ud = gate.clone().requires_grad_(True), up.clone().requires_grad_(True)
    GluCombine.clamped_silu(limit)(gd, ud).backward(torch.ones_like(gate))
    want_dg, want_du = oracle.glu_backward(gate.cpu().double(), up.cpu().double(), torch.ones(1, 8).double(),
                                           oracle.CLAMPED_SILU, limit=limit)
    assert ((gd.grad.cpu() != 0) == (want_dg != 0)).all() and ((ud.grad.cpu() != 0) == (want_du != 0)).all()
    assert bool((gd.grad[0, :4] != 0).all()) and gd.grad[0, 4] == 0  # at the bound passes, past it is cut
    assert ud.grad[0, 5] == 0 and ud.grad[0, 6] == 0
    probe = torch.tensor([[-64.0, -8.0, -1.0, -0.5, -1e-3, 0.0, 1e-3, 0.5, 1.0, 8.0, 64.0, 0.0]], device=device)
    out = GluCombine.silu()(probe, torch.ones_like(probe))
    assert torch.isfinite(out).all() and max_rel(out, torch.nn.functional.silu(probe.cpu().double())) < 1e-6
    assert is_silu_activation(torch.nn.SiLU()) and not is_silu_activation(torch.nn.GELU())
    assert is_gelu_tanh_activation(torch.nn.GELU(approximate="tanh")) and not is_gelu_tanh_activation(torch.nn.GELU())
    assert resolve_fused_glu_mul(torch.nn.functional.silu) == GluCombine.silu()
    assert resolve_fused_glu_mul(torch.relu) is None
    assert resolve_clamped_glu_mul(torch.nn.functional.silu, 3.0, clamp_activated=True) == \
        GluCombine.clamped_silu(3.0, clamp_activated=True)
    assert [c.name for c in _combines().values()] == list(_combines())


# ------------------------------------------------------------------------------------------------------- router

@pytest.mark.parametrize(("tokens", "experts", "top_k"), ((512, 8, 2), (2048, 128, 8), (300, 32, 4), (64, 512, 10),
                                                         (100, 1000, 8), (7, 64, 64)))
@pytest.mark.parametrize("dtype", (torch.float32, torch.bfloat16), ids=("fp32", "bf16"))
def test_router_selection_is_bit_exact_and_weights_close(device, tokens, experts, top_k, dtype):
    from halo_amd.kernels.router import SOFTMAX_ALL, SOFTMAX_TOPK, fused_topk_gate
    from oracle import router as oracle

    g = torch.Generator().manual_seed(tokens + experts)
    logits = (torch.randn(tokens, experts, generator=g) * 0.9).to(dtype)
    if dtype == torch.bfloat16:
        assert (logits.float().sort(-1).values.diff(dim=-1) == 0).any(), "bf16 logits should tie"
    for mode, normalize, eps in ((SOFTMAX_ALL, True, 0.0), (SOFTMAX_ALL, False, 0.0), (SOFTMAX_ALL, True, 1e-20),
                                 (SOFTMAX_TOPK, False, 0.0)):
        want_idx, want_w = oracle.route(logits, top_k, mode, normalize, eps)
        ld = logits.to(device).requires_grad_(True)
        idx, w = fused_topk_gate(ld, top_k, mode=mode, normalize=normalize, eps=eps)
        assert idx.dtype == torch.int64 and w.dtype == torch.float32
        assert torch.equal(idx.cpu(), want_idx), f"selection differs (mode {mode})"
        # weights: fp32 math (a few fp32 ulps from the oracle's), then one rounding to the logits' dtype, which can
        # land on the neighbouring bf16 value: at most one bf16 ulp (2^-7 relative) there, 1e-6 relative in fp32
        ulp = 2.0 ** -7 if dtype == torch.bfloat16 else 1e-6
        assert ((w.detach().cpu() - want_w).abs() <= ulp * want_w.abs() + 1e-30).all()
        if dtype == torch.bfloat16:
            assert torch.equal(w, w.bfloat16().float())
        gw = torch.randn(tokens, top_k, generator=g)
        (grad,) = torch.autograd.grad(w, ld, gw.to(device))
        want_grad = oracle.route_backward(logits.double(), want_idx, gw, mode, normalize, eps)
        assert grad.dtype == dtype
        assert max_rel(grad, want_grad) < (2e-2 if dtype == torch.bfloat16 else 1e-5)


def test_router_ties_go_to_the_lower_index(device):
    from halo_amd.kernels.router import fused_topk_gate

    logits = torch.tensor([[1.0, 1.0, 0.5, 1.0], [0.0, 2.0, 2.0, -1.0], [3.0, 3.0, 3.0, 3.0]], device=device)
    assert fused_topk_gate(logits, 2)[0].tolist() == [[0, 1], [1, 2], [0, 1]]
    assert fused_topk_gate(logits, 3)[0].tolist() == [[0, 1, 3], [1, 2, 0], [0, 1, 2]]
    wide = torch.zeros(2, 200, device=device)  # every score equal, experts spread over several lanes and registers
    assert fused_topk_gate(wide, 5)[0].tolist() == [[0, 1, 2, 3, 4]] * 2
    wide[0, 130], wide[0, 65], wide[0, 199] = 1.0, 1.0, 1.0
    assert fused_topk_gate(wide, 5)[0][0].tolist() == [65, 130, 199, 0, 1]


# ------------------------------------------------------------------------------------------------- grouped GEMM

def _offsets(counts, device):
    return torch.cumsum(torch.tensor(counts), 0).to(torch.int32).to(device)


@pytest.fixture(params=("mono", "duo", "small"))
def tile(request, device):
    """Runs a test once per tile configuration of the bf16 grouped GEMM (fp32 products ignore it)."""
    from halo_amd.kernels.grouped_mm import gemm_tile

    with gemm_tile(request.param):
        yield request.param


GEMM_CASES = (
    # counts per group, K, N
    ((7, 33, 0, 1, 64, 0), 128, 96),       # the reference's empty-group roster
    ((0, 0, 0, 0, 105, 0), 128, 96),       # one live expert
    ((130, 1, 255, 128, 129), 256, 384),   # ragged around half a row tile
    ((300, 0, 45), 2880, 360),             # widths off the tile size (2880 = 11.25 x 256)
    ((64,) * 16, 512, 1536),
    ((255, 256, 257, 0, 513, 31), 200, 264),  # ragged around the 256-row tile; K and N off the 64 / 256 steps
    (tuple((37 * i * i + 11 * i) % 91 for i in range(150)), 320, 256),  # many small and empty groups
    ((300,) * 36 + (7,), 256, 1024),       # more tiles than workgroups: every workgroup walks several
)


@pytest.mark.parametrize(("counts", "k", "n"), GEMM_CASES)
@pytest.mark.parametrize(("dtype", "tol"), ((torch.bfloat16, 2e-2), (torch.float32, 1e-5)), ids=("bf16", "fp32"))
def test_grouped_mm_forward_and_gradients_match_oracle(device, counts, k, n, dtype, tol, tile):
    from halo_amd.kernels.grouped_mm import grouped_mm
    from oracle import grouped_mm as oracle

    g = torch.Generator().manual_seed(sum(counts) + k)
    total = sum(counts)
    x = (torch.randn(total, k, generator=g) * 0.5).to(dtype)
    w = (torch.randn(len(counts), k, n, generator=g) * 0.05).to(dtype)
    dout = torch.randn(total, n, generator=g).to(dtype)
    offs = np.cumsum(counts).astype(np.int32)
    xd, wd = x.to(device).requires_grad_(True), w.to(device).requires_grad_(True)
    out = grouped_mm(xd, wd, offs=_offsets(counts, device))
    out.backward(dout.to(device))
    assert out.dtype == dtype and out.shape == (total, n) and wd.grad.shape == w.shape
    kw = dict(acc_dtype=torch.float64)
    want = oracle.grouped_mm(x.double(), w.double(), offs, **kw)
    want_dx = oracle.grouped_mm_dgrad(dout.double(), w.double(), offs, **kw)
    want_dw = oracle.grouped_mm_wgrad(x.double(), dout.double(), offs, **kw)
    for name, got, ref in (("out", out, want), ("dx", xd.grad, want_dx), ("dw", wd.grad, want_dw)):
        assert torch.isfinite(got).all(), name
        assert max_rel(got, ref) < tol, f"{name}: {max_rel(got, ref):.3e}"
        assert cosine(got, ref) > 0.9999, f"{name}: cosine {cosine(got, ref)}"
        if dtype == torch.bfloat16:
            # fp32 accumulation, one rounding: the error sits at the bf16 rounding floor of the exact result
            floor = fro_rel(ref.to(torch.bfloat16), ref)
            assert fro_rel(got, ref) <= 1.05 * floor + 1e-12, (name, fro_rel(got, ref), floor)
    for e, c in enumerate(counts):
        assert (c == 0) == (not wd.grad[e].any()), f"expert {e}: an empty group's weight gradient must be exact zeros"


def test_grouped_mm_takes_int64_offsets_transposed_weights_and_strided_rows(device, tile):
    from halo_amd.kernels.grouped_mm import grouped_mm
    from oracle import grouped_mm as oracle

    counts = (40, 0, 200, 16)
    g = torch.Generator().manual_seed(0)
    total, k, n = sum(counts), 192, 320
    wide = (torch.randn(total, 2 * k, generator=g) * 0.5).bfloat16()
    w_nk = (torch.randn(len(counts), n, k, generator=g) * 0.05).bfloat16()  # [G, N, K] storage, used as its transpose
    dout = torch.randn(total, n, generator=g).bfloat16()
    offs = np.cumsum(counts).astype(np.int32)
    x = wide[:, :k]
    xd = wide.to(device)[:, :k].detach().requires_grad_(True)
    wd = w_nk.to(device).requires_grad_(True)
    out = grouped_mm(xd, wd.transpose(1, 2), offs=torch.from_numpy(offs).long().to(device))
    out.backward(dout.to(device))
    w_kn = w_nk.transpose(1, 2).contiguous()
    kw = dict(acc_dtype=torch.float64)
    assert max_rel(out, oracle.grouped_mm(x.double(), w_kn.double(), offs, **kw)) < 2e-2
    assert max_rel(xd.grad, oracle.grouped_mm_dgrad(dout.double(), w_kn.double(), offs, **kw)) < 2e-2
    want_dw = oracle.grouped_mm_wgrad(x.double(), dout.double(), offs, **kw).transpose(1, 2)
    assert wd.grad.shape == w_nk.shape and max_rel(wd.grad, want_dw) < 2e-2


def test_grouped_mm_is_bit_reproducible_and_zero_rows(device, tile):
    from halo_amd.kernels.grouped_mm import grouped_mm

    counts = (100, 3, 0, 500, 77)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(sum(counts), 256, generator=g).bfloat16().to(device)
    w = (torch.randn(5, 256, 512, generator=g) * 0.05).bfloat16().to(device)
    dout = torch.randn(sum(counts), 512, generator=g).bfloat16().to(device)
    results = []
    for _ in range(3):
        xd, wd = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
        out = grouped_mm(xd, wd, offs=_offsets(counts, device))
        out.backward(dout)
        results.append((out.detach(), xd.grad, wd.grad))
    for other in results[1:]:
        assert all(torch.equal(a, b) for a, b in zip(results[0], other))
    empty = grouped_mm(torch.zeros(0, 256, device=device, dtype=torch.bfloat16, requires_grad=True), w,
                       offs=torch.zeros(5, dtype=torch.int32, device=device))
    assert empty.shape == (0, 512)
    empty.sum().backward()


@pytest.mark.parametrize(("counts", "k", "n"), (((255, 256, 257, 0, 513, 31, 128, 129, 1), 200, 264),
                                                 ((300, 0, 45), 2880, 360), ((700,), 96, 1000)))
def test_both_tile_configurations_give_the_same_bits(device, counts, k, n):
    """The 256 x 256, 128 x 256 and 128 x 128 tiles sum every contraction in the same order (sixteen values at a time, in
    sequence), so the plain and the gathered products and all their gradients are bit-equal between them, and the
    choice by size (``auto``) is one of them."""
    from halo_amd.kernels.grouped_mm import gather_grouped_mm, gemm_tile, grouped_mm
    from halo_amd.kernels.moe_permute import build_inv_map

    g = torch.Generator().manual_seed(11)
    rows, n_tokens = sum(counts), max(8, sum(counts) // 3)
    row_index = torch.randint(0, n_tokens, (rows,), generator=g).to(device)
    inv_map = build_inv_map(row_index, n_tokens, int(torch.bincount(row_index.cpu(), minlength=n_tokens).max()))
    tokens = torch.randn(n_tokens, k, generator=g).bfloat16().to(device)
    x = torch.randn(rows, k, generator=g).bfloat16().to(device)
    w = (torch.randn(len(counts), k, n, generator=g) * 0.05).bfloat16().to(device)
    dout = torch.randn(rows, n, generator=g).bfloat16().to(device)
    offs = _offsets(counts, device)
    results = {}
    for name in ("mono", "duo", "small", "auto"):
        with gemm_tile(name):
            xd, t, wd, wg = (v.clone().requires_grad_(True) for v in (x, tokens, w, w))
            out = grouped_mm(xd, wd, offs=offs)
            out.backward(dout)
            gathered = gather_grouped_mm(t, row_index, inv_map, wg, offs=offs)
            gathered.backward(dout)
            results[name] = (out.detach(), xd.grad, wd.grad, gathered.detach(), t.grad, wg.grad)
    for other in ("duo", "small", "auto"):
        for i, (a, b) in enumerate(zip(results["mono"], results[other])):
            assert torch.equal(a, b), (other, i)
    assert gemm_tile.set("auto") == "auto"  # the context managers restored the default


# ---------------------------------------------------------------------------------------------------- block fp8

@pytest.mark.parametrize("shape", [(128, 128), (256, 384), (200, 130), (5, 7), (3, 130, 129)])
def test_block_fp8_quantiser_is_bit_exact(device, shape):
    from halo_amd.kernels.lowp.block_fp8 import dequantize_block_fp8, quantize_block_fp8
    from oracle import block_fp8 as oracle

    torch.manual_seed(0)
    weight = (torch.randn(shape) * torch.rand(shape).mul(4)).bfloat16()
    q, scale = quantize_block_fp8(weight.to(device))
    want_q, want_scale = oracle.quantize_block_fp8(weight.float().numpy())
    assert q.dtype == torch.float8_e4m3fn and scale.dtype == torch.float32
    assert np.array_equal(scale.cpu().numpy(), want_scale)
    got_bits = q.view(torch.uint8).cpu().numpy()
    nonzero = (want_q & 0x7F) != 0
    assert np.array_equal(got_bits[nonzero], want_q[nonzero]) and not (got_bits[~nonzero] & 0x7F).any()
    restored = dequantize_block_fp8(q, scale)
    want_restored = torch.from_numpy(oracle.dequantize_block_fp8(want_q, want_scale)).bfloat16()
    assert torch.equal(restored.cpu(), want_restored)


def test_block_fp8_boundary_and_zero_block(device):
    from halo_amd.kernels.lowp.block_fp8 import quantize_block_fp8

    w = torch.zeros(128, 256)
    w[0, 0] = 448.0 * 4
    w[0, 128] = 448.0 * 4 * 1.0001
    _, scale = quantize_block_fp8(w.to(device))
    assert scale.tolist() == [[4.0, 8.0]]
    q0, s0 = quantize_block_fp8(torch.zeros(128, 128, device=device))
    assert torch.isfinite(s0).all() and bool((s0 > 0).all()) and not q0.float().any()


def test_fp8_weight_grouped_gemm_equals_the_dequantised_bf16_path(device):
    """bf16 activations times block-fp8 weights: every e4m3 value times its power-of-two scale is a bf16 value, so the
    kernel must equal the bf16 grouped GEMM over the dequantised weights bit for bit; against the oracle's fp64
    product it sits at the bf16 rounding floor."""
    from halo_amd.kernels.expert_gemm import BlockFp8Weight, expert_gemm
    from halo_amd.kernels.grouped_mm import grouped_mm
    from halo_amd.kernels.lowp.block_fp8 import dequantize_block_fp8, quantize_block_fp8
    from oracle import block_fp8 as fp8_oracle
    from oracle import grouped_mm as oracle

    counts = (130, 0, 257, 64)
    g = torch.Generator().manual_seed(4)
    k, n = 384, 640
    x = torch.randn(sum(counts), k, generator=g).bfloat16()
    w = (torch.randn(len(counts), k, n, generator=g) * 0.02)
    q, scale = quantize_block_fp8(w.to(device))
    offs = _offsets(counts, device)
    weight = BlockFp8Weight(q, scale)
    out = expert_gemm(x.to(device), weight, offs=offs, weight_cacheable=False)  # the kernel that reads the fp8 bytes
    deq = dequantize_block_fp8(q, scale)
    assert torch.equal(out, grouped_mm(x.to(device), deq, offs=offs))
    # the route over a dequantised copy kept with the weight (taken from 64 rows per expert on) gives the same bits
    assert weight._bf16 is None
    assert torch.equal(expert_gemm(x.to(device), weight, offs=offs), out) and weight._bf16 is not None
    few = x[:100].to(device)  # too few rows per expert: the fp8 kernel again
    few_offs = _offsets((30, 0, 50, 20), device)
    assert torch.equal(expert_gemm(few, BlockFp8Weight(q, scale), offs=few_offs), grouped_mm(few, deq, offs=few_offs))
    want_q, want_scale = fp8_oracle.quantize_block_fp8(w.numpy())
    w_ref = torch.from_numpy(fp8_oracle.dequantize_block_fp8(want_q, want_scale)).bfloat16()
    want = oracle.grouped_mm(x.double(), w_ref.double(), np.cumsum(counts).astype(np.int32), acc_dtype=torch.float64)
    assert max_rel(out, want) < 2e-2 and cosine(out, want) > 0.9999


@pytest.mark.parametrize(("rows", "k"), ((5, 128), (300, 1024), (1000, 3072)))
def test_activation_row_quantiser_is_bit_exact(device, rows, k):
    """e4m3 values and scale exponents equal the oracle's bit for bit, over magnitudes from subnormal bf16 to 1e30,
    with all-zero blocks and blocks whose maximum sits on either side of a scale boundary."""
    from halo_amd.kernels.lowp.block_fp8 import quantize_rows_fp8
    from oracle import block_fp8 as oracle

    g = torch.Generator().manual_seed(rows + k)
    x = torch.randn(rows, k, generator=g) * torch.exp2(torch.randint(-20, 20, (rows, k // 128), generator=g)
                                                       .repeat_interleave(128, dim=1).float())
    x[0, :128] = 0
    x[1, :128] = 0
    x[1, 5] = 448.0
    x[2, :128] = 0
    x[2, 7] = -450.0
    x[3, :128] = 1e-40
    x[4, :128] = 0
    x[4, 100] = 1e30
    x = x.bfloat16()
    q, exps = quantize_rows_fp8(x.to(device))
    want_q, want_exps = oracle.quantize_rows_fp8(x.float().numpy())
    assert q.dtype == torch.float8_e4m3fn and exps.dtype == torch.uint8 and exps.shape == (k // 128, rows)
    assert q.shape == (k // 64, rows, 64)  # panels of 64 values
    assert np.array_equal(exps.cpu().numpy(), want_exps)
    got_bits = q.view(torch.uint8).permute(1, 0, 2).reshape(rows, k).cpu().numpy()
    nonzero = (want_q & 0x7F) != 0
    assert np.array_equal(got_bits[nonzero], want_q[nonzero]) and not (got_bits[~nonzero] & 0x7F).any()
    assert exps[0, 0] == 0 and exps[0, 1] == 127 and exps[0, 2] == 128
    # rows fetched through an index on the way equal the rows quantised after a gather; an index outside the source
    # gives a row of zeros
    index = torch.randint(0, rows, (2 * rows + 3,), generator=g)
    index[1], index[-1] = -1, rows
    gq, gexps = quantize_rows_fp8(x.to(device), index.to(device))
    picked = x[index.clamp(0, rows - 1)]
    picked[1], picked[-1] = 0, 0
    pq, pexps = quantize_rows_fp8(picked.to(device))
    assert torch.equal(gq.view(torch.uint8), pq.view(torch.uint8)) and torch.equal(gexps, pexps)


@pytest.mark.parametrize("kind", ("silu", "gelu_tanh", "gptoss", "clamped"))
def test_glu_writing_e4m3_panels_equals_glu_then_row_quantiser(device, kind):
    from halo_amd.kernels.fused_glu import GluCombine
    from halo_amd.kernels.lowp.block_fp8 import quantize_rows_fp8

    combine = {"silu": GluCombine.silu(), "gelu_tanh": GluCombine.gelu_tanh(), "gptoss": GluCombine.gptoss(1.702, 7.0),
               "clamped": GluCombine.clamped_silu(5.0, clamp_activated=True)}[kind]
    g = torch.Generator().manual_seed(9)
    for rows, half in ((77, 128), (300, 1024)):
        gate_up = (torch.randn(rows, 2 * half, generator=g) * 3).bfloat16().to(device)
        gate_up[3, :half] = 0
        fused = combine.packed_quantized(gate_up)
        q, exps = quantize_rows_fp8(combine.packed(gate_up))
        assert fused.shape == (rows, half)
        assert torch.equal(fused.q.view(torch.uint8), q.view(torch.uint8))
        assert torch.equal(fused.scale_exponents, exps)
    assert combine.packed_quantized(gate_up[:, : 2 * 96]) is None  # a half width off the block size
    assert combine.packed_quantized(gate_up.float()) is None


@pytest.mark.parametrize("mantissas", (False, True))
@pytest.mark.parametrize(("counts", "k", "n"), (((130, 0, 257, 64), 128, 256), ((300, 1, 0, 255, 256, 700), 1024, 520),
                                                 ((64,) * 16, 384, 1536), ((1000,), 3072, 128)))
def test_fp8_mfma_grouped_gemm_equals_the_exact_products(device, counts, k, n, mantissas):
    """Both operands e4m3 on the scaled MFMA: against the float64 product of the same quantised values and scales
    (every term exact there) the result sits at the bf16 rounding floor.  ``mantissas``: weight scales that are not
    powers of two, whose mantissas the kernel carries in its accumulators."""
    from halo_amd.kernels.expert_gemm import BlockFp8Weight, expert_gemm
    from halo_amd.kernels.lowp.block_fp8 import quantize_block_fp8, quantize_rows_fp8
    from oracle import block_fp8 as oracle

    g = torch.Generator().manual_seed(len(counts) + k)
    x = (torch.randn(sum(counts), k, generator=g) * torch.exp2(torch.randint(-3, 4, (sum(counts), 1), generator=g)
                                                               .float())).bfloat16()
    w = torch.randn(len(counts), k, n, generator=g) * 0.02
    q, scale = quantize_block_fp8(w.to(device))
    if mantissas:
        scale = scale * (1 + torch.rand(scale.shape, generator=g)).to(device)
        scale[0, 0, 0] = 0.0  # a block switched off
    offs = _offsets(counts, device)
    out = expert_gemm(x.to(device), BlockFp8Weight(q, scale), offs=offs, fp8_activations=True)
    a_q, a_exps = quantize_rows_fp8(x.to(device))
    want = oracle.fp8_grouped_mm(a_q.view(torch.uint8).permute(1, 0, 2).reshape(-1, k).cpu().numpy(), a_exps.cpu().numpy(),
                                 q.view(torch.uint8).cpu().numpy(), scale.cpu().numpy(),
                                 np.cumsum(counts).astype(np.int32))
    want = torch.from_numpy(want)
    assert out.dtype == torch.bfloat16 and out.shape == want.shape
    err = (out.double().cpu() - want).abs().max() / want.abs().max()
    assert err < 4e-3, err
    assert cosine(out, want) > 0.99999


def test_fp8_mfma_path_against_the_dequantised_bf16_path(device):
    """The quantised-weight configuration scaled down (8 experts, hidden 1024, FFN projection 512): with the
    activations at e4m3 too the product differs from the bf16-activation path by the activations' quantisation
    error, 2-3 % of the result's norm for three mantissa bits, and by nothing systematic."""
    from halo_amd.kernels.expert_gemm import BlockFp8Weight, expert_gemm
    from halo_amd.kernels.lowp.block_fp8 import quantize_block_fp8

    g = torch.Generator().manual_seed(4)
    counts = (700, 512, 3, 0, 1300, 256, 257, 1068)
    x = torch.randn(sum(counts), 1024, generator=g).bfloat16().to(device)
    w = (torch.randn(len(counts), 1024, 512, generator=g) * 0.02).to(device)
    weight = BlockFp8Weight(*quantize_block_fp8(w))
    offs = _offsets(counts, device)
    got = expert_gemm(x, weight, offs=offs, fp8_activations=True).double()
    ref = expert_gemm(x, weight, offs=offs).double()
    rel = ((got - ref).norm() / ref.norm()).item()
    assert 0.005 < rel < 0.04, rel
    assert cosine(got, ref) > 0.999
    assert abs(((got - ref).mean() / ref.abs().mean()).item()) < 2e-3


@pytest.mark.parametrize(("counts", "k", "n"), (((255, 256, 257, 0, 513, 31), 200, 264), ((64,) * 16, 512, 1536),
                                                 (tuple((37 * i * i + 11 * i) % 91 for i in range(150)), 320, 256)))
def test_gather_grouped_mm_equals_permute_then_grouped_mm(device, counts, k, n, tile):
    """The GEMM that gathers its A rows through the sorted token index does the same arithmetic in the same order as
    the permute followed by the plain GEMM: outputs and all gradients are bit-equal.  Tokens are drawn so that rows
    repeat (top-k) and some tokens are never picked."""
    from halo_amd.kernels.grouped_mm import gather_fusable, gather_grouped_mm, grouped_mm
    from halo_amd.kernels.moe_permute import MoEGatherPermute, build_inv_map

    g = torch.Generator().manual_seed(3)
    rows, n_tokens = sum(counts), max(8, sum(counts) // 3)
    row_index = torch.randint(0, n_tokens, (rows,), generator=g).to(device)
    width = int(torch.bincount(row_index.cpu(), minlength=n_tokens).max())
    inv_map = build_inv_map(row_index, n_tokens, width)
    tokens = torch.randn(n_tokens, k, generator=g).bfloat16().to(device)
    w = (torch.randn(len(counts), k, n, generator=g) * 0.05).bfloat16().to(device)
    dout = torch.randn(rows, n, generator=g).bfloat16().to(device)
    offs = _offsets(counts, device)
    assert gather_fusable(tokens, w)
    results = []
    for fused in (False, True):
        t, wd = tokens.clone().requires_grad_(True), w.clone().requires_grad_(True)
        if fused:
            out = gather_grouped_mm(t, row_index, inv_map, wd, offs=offs)
        else:
            out = grouped_mm(MoEGatherPermute.apply(t, row_index, inv_map), wd, offs=offs)
        out.backward(dout)
        results.append((out.detach(), t.grad, wd.grad))
    for name, a, b in zip(("out", "grad_tokens", "grad_weight"), *results):
        assert torch.equal(a, b), name


@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float32), ids=("bf16", "fp32"))
@pytest.mark.parametrize(("counts", "k", "n"), (((255, 256, 257, 0, 513, 31), 200, 264), ((64,) * 16, 512, 1536),
                                                 ((0, 0, 700, 1, 0), 2880, 2880), ((5,), 64, 8)))
def test_grouped_mm_with_the_bias_in_its_epilogue_equals_the_two_operations(device, dtype, counts, k, n, tile):
    """``grouped_mm_bias`` = ``grouped_mm`` followed by ``+ MoEExpertBiasGather.apply(bias, eids)``: the product is
    rounded, the bias row of the row's expert is added, the sum is rounded again.  Output and the three gradients
    are bit-equal to the two-operation path; the output also matches the fp64 loop."""
    from halo_amd.kernels.grouped_mm import bias_fusable, grouped_mm, grouped_mm_bias
    from halo_amd.kernels.moe_permute import MoEExpertBiasGather

    g = torch.Generator().manual_seed(5)
    rows, groups = sum(counts), len(counts)
    x = torch.randn(rows, k, generator=g).to(dtype).to(device)
    w = (torch.randn(groups, k, n, generator=g) * 0.05).to(dtype).to(device)
    bias = torch.randn(groups, n, generator=g).to(dtype).to(device)
    dout = torch.randn(rows, n, generator=g).to(dtype).to(device)
    offs = _offsets(counts, device)
    eids = torch.repeat_interleave(torch.arange(groups), torch.tensor(counts)).to(device)
    assert bias_fusable(x, w, bias)
    results = []
    for fused in (False, True):
        xd, wd, bd = (t.clone().requires_grad_(True) for t in (x, w, bias))
        if fused:
            out = grouped_mm_bias(xd, wd, bd, offs=offs, eids=eids)
        else:
            out = grouped_mm(xd, wd, offs=offs) + MoEExpertBiasGather.apply(bd, eids)
        out.backward(dout)
        results.append((out.detach(), xd.grad, wd.grad, bd.grad))
    for name, a, b in zip(("out", "grad_x", "grad_weight", "grad_bias"), *results):
        assert torch.equal(a, b), name
    want = torch.cat([x[s:e].double() @ w[i].double() + bias[i].double()
                      for i, (s, e) in enumerate(zip([0] + list(np.cumsum(counts)[:-1]), np.cumsum(counts)))])
    tol = 2e-2 if dtype == torch.bfloat16 else 1e-4
    assert max_rel(results[1][0], want) < tol


@pytest.mark.parametrize("scaled", (False, True), ids=("plain", "scaled"))
@pytest.mark.parametrize(("dtype", "top_k", "hidden"), ((torch.bfloat16, 8, 2048), (torch.bfloat16, 3, 264),
                                                         (torch.float32, 4, 256), (torch.bfloat16, 2, 100)))
def test_combine_with_an_added_term_equals_the_tensor_operations(device, dtype, top_k, hidden, scaled):
    """``gather_reduce_rows(..., addend=a, addend_scale=s)`` returns the bits of ``gather_reduce_rows(...) + s * a``:
    the reduction is rounded, the scaled term is rounded, the sum is rounded.  Rows without a valid slot and a
    row-strided addend included."""
    from halo_amd.kernels.moe_permute import gather_reduce_rows

    g = torch.Generator().manual_seed(13)
    n_tokens = 300
    token_idx, inv_map = _routing(n_tokens, top_k, n_tokens * top_k * 2 // 3, seed=4)
    n_sorted = token_idx.numel()
    src = torch.randn(n_sorted, hidden, generator=g).to(dtype).to(device)
    w = torch.rand(n_sorted, generator=g).to(dtype).to(device)
    padded = torch.randn(n_tokens, hidden + 24, generator=g).to(dtype).to(device)
    addend = padded[:, :hidden]  # rows 24 elements apart from dense
    scale = torch.rand(n_tokens, generator=g).to(dtype).to(device) if scaled else None
    inv_map[5] = inv_map[77] = n_sorted  # two tokens that no expert row belongs to: their output is the added term
    inv = inv_map.to(device)
    got = gather_reduce_rows(src, inv, w, addend=addend, addend_scale=scale)
    combined = gather_reduce_rows(src, inv, w)
    want = combined + (addend if scale is None else scale[:, None] * addend)
    assert torch.equal(got, want)
    assert torch.equal(got[5], want[5]) and combined[5].count_nonzero() == 0


@pytest.mark.parametrize(("counts", "k", "n"), (((255, 256, 257, 0, 513, 31), 200, 264), ((64,) * 16, 512, 1536),
                                                 ((0, 0, 700, 1), 768, 2048),
                                                 (tuple((37 * i * i + 11 * i) % 91 for i in range(150)), 320, 256)))
def test_down_projection_with_the_plain_combine_equals_the_separate_operations(device, counts, k, n, tile):
    """``grouped_mm_combine``: the product's rows summed per token in one autograd node, its backward fetching the
    token gradient's rows through the index.  Same arithmetic in the same order as ``grouped_mm`` followed by the
    unweighted gather-reduce, whose backward materialises ``grad_out[row_index]``: output and both gradients are
    bit-equal, with and without an added term, for contiguous and row-strided token gradients."""
    from halo_amd.kernels.grouped_mm import combine_fusable, grouped_mm, grouped_mm_combine
    from halo_amd.kernels.moe_permute import build_inv_map, gather_reduce_rows

    g = torch.Generator().manual_seed(5)
    rows, n_tokens = sum(counts), max(8, sum(counts) // 3)
    row_index = torch.randint(0, n_tokens, (rows,), generator=g).to(device)
    width = int(torch.bincount(row_index.cpu(), minlength=n_tokens).max())
    inv_map = build_inv_map(row_index, n_tokens, width)
    a = torch.randn(rows, k, generator=g).bfloat16().to(device)
    w = (torch.randn(len(counts), k, n, generator=g) * 0.05).bfloat16().to(device)
    addend = torch.randn(n_tokens, n, generator=g).bfloat16().to(device)
    padded = torch.zeros(n_tokens, n + 24, dtype=torch.bfloat16, device=device)
    padded[:, :n] = torch.randn(n_tokens, n, generator=g).bfloat16().to(device)
    offs = _offsets(counts, device)
    assert combine_fusable(a, w, torch.bfloat16)
    for with_addend in (False, True):
        for dout in (padded[:, :n].contiguous(), padded[:, :n]):
            results = []
            for fused in (False, True):
                ad, wd = a.clone().requires_grad_(True), w.clone().requires_grad_(True)
                extra = addend.clone().requires_grad_(True) if with_addend else None
                if fused:
                    out = grouped_mm_combine(ad, wd, offs=offs, row_index=row_index, inv_map=inv_map, addend=extra)
                else:
                    product = grouped_mm(ad, wd, offs=offs)
                    out = _PlainCombine.apply(product, row_index, inv_map)
                    if with_addend:
                        out = out + extra
                out.backward(dout)
                results.append((out.detach(), ad.grad, wd.grad) + ((extra.grad,) if with_addend else ()))
            for name, x, y in zip(("out", "grad_a", "grad_b", "grad_addend"), *results):
                assert torch.equal(x, y), (name, with_addend, dout.is_contiguous())
            # the gradients themselves against fp64 products of the same bf16 values
            gathered = dout.double()[row_index].cpu()
            ends = [0] + offs.cpu().tolist()
            for e, (lo, hi) in enumerate(zip(ends[:-1], ends[1:])):
                if hi > lo:
                    want = a[lo:hi].double().cpu().t() @ gathered[lo:hi]
                    assert max_rel(results[1][2][e], want) < 2e-2
                else:
                    assert not results[1][2][e].any()


class _PlainCombine(torch.autograd.Function):
    """Unweighted gather-reduce whose backward copies ``grad_out[row_index]`` out: the two-operation reference of the
    test above."""

    @staticmethod
    def forward(ctx, rows, row_index, inv_map):
        from halo_amd.kernels.moe_permute import gather_reduce_rows

        ctx.save_for_backward(row_index)
        return gather_reduce_rows(rows, inv_map)

    @staticmethod
    def backward(ctx, grad_out):
        (row_index,) = ctx.saved_tensors
        return grad_out[row_index].contiguous(), None, None


@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float32), ids=("bf16", "fp32"))
@pytest.mark.parametrize(("counts", "k", "n"), (((255, 256, 257, 0, 513, 31), 16, 264), ((64,) * 16, 64, 1536),
                                                 ((300, 0, 41), 8, 520)))
def test_grouped_mm_added_to_a_tensor_equals_the_tensor_operations(device, dtype, counts, k, n, tile):
    """``grouped_mm_addto``: ``addend + scale * grouped_mm(a, b)`` with the product scaled and added in the GEMM's
    epilogue.  The roundings sit where the tensor operations have them, so the output and all three gradients equal
    the unfused expression bit for bit; the contraction lengths are adapter ranks."""
    from halo_amd.kernels.grouped_mm import addto_fusable, grouped_mm, grouped_mm_addto

    g = torch.Generator().manual_seed(17)
    rows, scale = sum(counts), 32.0 / 24.0  # a scale that is not a power of two: its rounding shows
    a = torch.randn(rows, k, generator=g).to(dtype).to(device)
    b = (torch.randn(len(counts), k, n, generator=g) * 0.2).to(dtype).to(device)
    base = torch.randn(rows, n, generator=g).to(dtype).to(device)
    dout = torch.randn(rows, n, generator=g).to(dtype).to(device)
    offs = _offsets(counts, device)
    assert addto_fusable(a, b, base)
    results = []
    for fused in (False, True):
        ad, bd, cd = (t.clone().requires_grad_(True) for t in (a, b, base))
        out = grouped_mm_addto(ad, bd, cd, scale, offs=offs) if fused else cd + scale * grouped_mm(ad, bd, offs=offs)
        out.backward(dout)
        results.append((out.detach(), ad.grad, bd.grad, cd.grad))
    for name, x, y in zip(("out", "grad_a", "grad_b", "grad_addend"), *results):
        assert torch.equal(x, y), name


@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float32), ids=("bf16", "fp32"))
@pytest.mark.parametrize(("counts", "k", "n"), (((255, 256, 257, 0, 513, 31), 200, 264), ((64,) * 16, 1536, 512),
                                                 ((0, 0, 700, 1, 0), 2880, 2880), ((5,), 8, 64)))
def test_input_gradient_added_into_a_tensor_equals_the_two_operations(device, dtype, counts, k, n, tile):
    """``hmoe_grouped_gemm_dgrad_addto`` returns the bits of ``addend + grad @ W^T``: the product rounded, then the
    sum, as the tensor addition of two input gradients rounds.  A row-strided addend, and the output written over the
    addend itself."""
    from halo_amd import _lib
    from halo_amd.kernels.grouped_mm import grouped_mm_grads

    g = torch.Generator().manual_seed(21)
    rows, groups = sum(counts), len(counts)
    grad = torch.randn(rows, n, generator=g).to(dtype).to(device)
    w = (torch.randn(groups, k, n, generator=g) * 0.05).to(dtype).to(device)
    padded = torch.randn(rows, k + 16, generator=g).to(dtype).to(device)
    addend = padded[:, :k]
    offs = _offsets(counts, device)
    shape_only = grad.new_empty((1, k)).expand(rows, k)
    product, _ = grouped_mm_grads(shape_only, w, grad, offs, True, False)
    want = addend + product

    def run(base, out):
        with _lib.on_device(device):
            _lib.call("hmoe_grouped_gemm_dgrad_addto", _lib.ptr(grad), grad.stride(0), _lib.ptr(w), _lib.ptr(offs), rows,
                      groups, k, n, _lib.dtype_id(dtype), _lib.ptr(base), base.stride(0), _lib.ptr(out), out.stride(0),
                      _lib.stream_ptr(device))
        return out

    assert torch.equal(run(addend, torch.empty(rows, k, dtype=dtype, device=device)), want)
    in_place = addend.contiguous()
    assert torch.equal(run(in_place, in_place), want)


@pytest.mark.parametrize("biased", (True, False), ids=("biased", "plain"))
@pytest.mark.parametrize(("counts", "k", "n"), (((255, 256, 257, 0, 513, 31), 200, 264), ((64,) * 16, 512, 768),
                                                 (tuple((37 * i * i + 11 * i) % 91 for i in range(150)), 320, 256)))
def test_two_projections_of_gathered_rows_as_one_node_equal_the_separate_operations(device, counts, k, n, biased, tile):
    """``gather_grouped_mm_pair`` = the permute followed by two (biased) grouped products: both outputs, the token
    gradient (the two input gradients added, then scattered back), both weight gradients and both bias gradients are
    bit-equal to the operations the reference runs one by one."""
    from halo_amd.kernels.grouped_mm import gather_grouped_mm_pair, grouped_mm, pair_fusable
    from halo_amd.kernels.moe_permute import MoEExpertBiasGather, MoEGatherPermute, build_inv_map

    g = torch.Generator().manual_seed(23)
    rows, groups, n_tokens = sum(counts), len(counts), max(8, sum(counts) // 3)
    row_index = torch.randint(0, n_tokens, (rows,), generator=g).to(device)
    width = int(torch.bincount(row_index.cpu(), minlength=n_tokens).max())
    inv_map = build_inv_map(row_index, n_tokens, width)
    tokens = torch.randn(n_tokens, k, generator=g).bfloat16().to(device)
    w1, w2 = ((torch.randn(groups, k, n, generator=g) * 0.05).bfloat16().to(device) for _ in range(2))
    b1, b2 = (torch.randn(groups, n, generator=g).bfloat16().to(device) if biased else None for _ in range(2))
    d1, d2 = (torch.randn(rows, n, generator=g).bfloat16().to(device) for _ in range(2))
    offs = _offsets(counts, device)
    eids = torch.repeat_interleave(torch.arange(groups), torch.tensor(counts)).to(device)
    assert pair_fusable(tokens, w1, b1, w2, b2)
    results = []
    for fused in (False, True):
        leaves = [t.clone().requires_grad_(True) for t in (tokens, w1, w2)]
        biases = [b.clone().requires_grad_(True) for b in (b1, b2)] if biased else [None, None]
        t, wa, wb = leaves
        if fused:
            out1, out2 = gather_grouped_mm_pair(t, row_index, inv_map, wa, biases[0], wb, biases[1], offs=offs, eids=eids)
        else:
            permuted = MoEGatherPermute.apply(t, row_index, inv_map)
            out1, out2 = grouped_mm(permuted, wa, offs=offs), grouped_mm(permuted, wb, offs=offs)
            if biased:
                out1 = out1 + MoEExpertBiasGather.apply(biases[0], eids)
                out2 = out2 + MoEExpertBiasGather.apply(biases[1], eids)
        torch.autograd.backward([out1, out2], [d1, d2])
        results.append([out1.detach(), out2.detach(), *(leaf.grad for leaf in leaves),
                        *(b.grad for b in biases if b is not None)])
    names = ("out1", "out2", "grad_tokens", "grad_w1", "grad_w2", "grad_b1", "grad_b2")
    for name, a, b in zip(names, *results):
        assert torch.equal(a, b), name
