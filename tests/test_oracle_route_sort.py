"""Pins ``oracle.route_sort`` and ``oracle.permute``: hand-derived known answers, brute force on tiny inputs, the
invariants the reference's tests state, and library routines in fp64."""

import json
import os

import numpy as np
import pytest
import torch

from oracle import permute as permute_oracle
from oracle import route_sort as oracle
from tests.cases import ROUTING_CASES, brute_force_sort, make_receive

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
NAMES = ("sorted_token_idx", "sorted_weights", "sorted_expert_ids", "offs", "inv_map", "dest")


def test_literal_receive_known_answer():
    with open(os.path.join(GOLDEN, "route_sort_literal.json")) as f:
        gold = json.load(f)
    experts = np.array(gold["experts"], dtype=np.int64)
    weights = np.array(gold["weights"], dtype=np.float32)
    got = oracle.argsort_routing(experts, weights, gold["num_local_experts"], tuple(gold["counts"]))
    for name, value in zip(NAMES, got):
        assert value.tolist() == gold[name], name
    assert got[3].dtype == np.int32 and got[0].dtype == np.int64 and got[4].dtype == np.int64


@pytest.mark.parametrize("case", [c for c in ROUTING_CASES if c.rows * c.top_k <= 4096], ids=lambda c: c.name)
def test_matches_brute_force(case):
    experts, weights, counts = make_receive(case, seed=ROUTING_CASES.index(case))
    got = oracle.argsort_routing(experts.numpy(), weights.numpy(), case.local_experts, counts)
    want = brute_force_sort(experts.numpy(), weights.numpy(), case.local_experts)
    for name, g, w in zip(NAMES, got, want):
        assert g.dtype == w.dtype and g.shape == w.shape, name
        assert np.array_equal(g, w), f"{case.name}: {name}"


@pytest.mark.parametrize("case", ROUTING_CASES, ids=lambda c: c.name)
def test_invariants(case):
    experts, weights, counts = make_receive(case, seed=ROUTING_CASES.index(case))
    e, w = experts.numpy(), weights.numpy()
    tok, sw, eid, offs, inv_map, dest = oracle.argsort_routing(e, w, case.local_experts, counts)
    n_valid = tok.shape[0]
    assert n_valid == int(((e >= 0) & (e < case.local_experts)).sum())
    assert np.all(np.diff(eid) >= 0)
    assert offs[-1] == n_valid and np.all(np.diff(np.concatenate([[0], offs])) >= 0)
    starts = np.concatenate([[0], offs[:-1]])
    for g in range(case.local_experts):
        assert np.all(eid[starts[g]:offs[g]] == g)
        assert np.all(np.diff(tok[starts[g]:offs[g]]) >= 0)  # stable: slot order within an expert
    valid = inv_map[inv_map != n_valid]
    assert np.array_equal(np.sort(valid), np.arange(n_valid))
    for r in range(case.rows):
        row = inv_map[r]
        assert np.all(np.diff(row) >= 0)
        assert np.all(tok[row[row != n_valid]] == r)
    flat_valid = ((e >= 0) & (e < case.local_experts)).reshape(-1)
    assert np.all(dest[~flat_valid] == n_valid)
    assert np.array_equal(sw[dest[flat_valid]], w.reshape(-1)[flat_valid])
    if case.idle_expert is not None:
        g = case.idle_expert
        assert offs[g] == starts[g]


def test_count_checks_and_errors():
    case = ROUTING_CASES[1]
    experts, weights, counts = make_receive(case, seed=1)
    e, w = experts.numpy(), weights.numpy()
    want = oracle.argsort_routing(e, w, case.local_experts, counts)
    moved = (counts[0] - 1, counts[1] + 1, *counts[2:])  # only the sum is read
    got = oracle.argsort_routing(e, w, case.local_experts, moved)
    assert all(np.array_equal(a, b) for a, b in zip(got, want))
    for bad in ((counts[0] - 1, *counts[1:]), (counts[0] + 1, *counts[1:])):
        with pytest.raises(RuntimeError, match="receive counts disagree"):
            oracle.argsort_routing(e, w, case.local_experts, bad)
    with pytest.raises(ValueError, match="2 receive counts for 4 local experts"):
        oracle.argsort_routing(np.zeros((2, 2), dtype=np.int64), np.zeros((2, 2), dtype=np.float32), 4, (3, 1))
    ep1 = np.array([[0, 1], [2, -1]])
    with pytest.raises(RuntimeError, match="outside the local experts"):
        oracle.argsort_routing(ep1, np.zeros((2, 2), dtype=np.float32), 3, None)


def test_sort_backward_reads_sorted_positions():
    experts, weights, counts = make_receive(ROUTING_CASES[0], seed=0)
    e, w = experts.numpy(), weights.numpy()
    *_, dest = oracle.argsort_routing(e, w, 4, counts)
    upstream = np.random.default_rng(0).standard_normal(sum(counts)).astype(np.float32)
    grad = oracle.sort_backward(upstream, dest, e.shape)
    # autograd through the gather that defines sorted_weights
    leaf = weights.clone().requires_grad_(True)
    valid = ((experts >= 0) & (experts < 4)).reshape(-1)
    order = torch.argsort(torch.where(valid, experts.reshape(-1), 10**6), stable=True)[: sum(counts)]
    leaf.reshape(-1)[order].backward(torch.from_numpy(upstream))
    assert np.array_equal(grad, leaf.grad.numpy())


def test_build_inv_map_empty_and_full_width():
    inv = oracle.build_inv_map(np.zeros(0, dtype=np.int64), 8, 4)
    assert inv.shape == (8, 4) and np.all(inv == 0)
    inv = oracle.build_inv_map(np.array([0, 0, 0, 0]), 2, 4)
    assert inv[0].tolist() == [0, 1, 2, 3] and np.all(inv[1] == 4)


def test_bincount():
    idx = np.array([[0, 2], [2, 2]])
    assert oracle.bincount(idx, 4).tolist() == [1.0, 0.0, 3.0, 0.0]
    assert oracle.bincount(idx, 4, np.int64).dtype == np.int64
    assert oracle.bincount(idx, 3, weights=np.array([0.5, 1.0, 2.0, 4.0])).tolist() == [0.5, 0.0, 7.0]


# ---------------------------------------------------------------- permute / unpermute against fp64 library routines


def _routing(n_tokens, top_k, n_sorted, seed):
    g = torch.Generator().manual_seed(seed)
    slots = torch.arange(n_tokens).repeat_interleave(top_k)
    token_idx = slots[torch.randperm(slots.numel(), generator=g)[:n_sorted]]
    return token_idx, torch.from_numpy(oracle.build_inv_map(token_idx.numpy(), n_tokens, top_k))


def test_gather_reduce_sentinel_known_answer():
    # tests/gpu/kernels/test_moe_permute.py:93-97 of the reference
    src = torch.arange(1, 7, dtype=torch.float32).unsqueeze(-1).expand(6, 3).contiguous()
    inv_map = torch.tensor([[0, 3], [5, 6], [6, 6]])
    out = permute_oracle.gather_reduce(src, inv_map)
    assert out[:, 0].tolist() == [5.0, 6.0, 0.0]


@pytest.mark.parametrize(("n_tokens", "top_k", "hidden", "fill"), ((64, 8, 16, 0.5), (33, 4, 7, 1.0), (50, 2, 6, 0.1)))
def test_permute_matches_index_add(n_tokens, top_k, hidden, fill):
    n_sorted = int(n_tokens * top_k * fill)
    token_idx, inv_map = _routing(n_tokens, top_k, n_sorted, seed=n_tokens)
    g = torch.Generator().manual_seed(1)
    y = torch.randn(n_sorted, hidden, dtype=torch.float64, generator=g)
    w = torch.rand(n_sorted, dtype=torch.float64, generator=g)
    grad = torch.randn(n_tokens, hidden, dtype=torch.float64, generator=g)
    ref_y, ref_w = y.clone().requires_grad_(True), w.clone().requires_grad_(True)
    want = torch.zeros(n_tokens, hidden, dtype=torch.float64).index_add(0, token_idx, ref_y * ref_w[:, None])
    want.backward(grad)
    got = permute_oracle.gather_reduce(y, inv_map, w)
    gy, gw = permute_oracle.weighted_unpermute_backward(grad, y, w, token_idx)
    assert torch.allclose(got, want.detach(), rtol=0, atol=1e-12)
    assert torch.allclose(gy, ref_y.grad, rtol=0, atol=1e-12)
    assert torch.allclose(gw, ref_w.grad, rtol=0, atol=1e-12)
    # permute forward / backward
    tokens = torch.randn(n_tokens, hidden, dtype=torch.float64, generator=g)
    assert torch.equal(permute_oracle.gather_rows(tokens, token_idx), tokens[token_idx])
    gs = torch.randn(n_sorted, hidden, dtype=torch.float64, generator=g)
    want_b = torch.zeros(n_tokens, hidden, dtype=torch.float64).index_add_(0, token_idx, gs)
    assert torch.allclose(permute_oracle.gather_reduce(gs, inv_map), want_b, rtol=0, atol=1e-12)


def test_bf16_result_is_the_exact_sum_rounded_once():
    token_idx, inv_map = _routing(40, 8, 200, seed=3)
    g = torch.Generator().manual_seed(4)
    y = torch.randn(200, 32, generator=g).bfloat16()
    w = torch.rand(200, generator=g).bfloat16()
    exact = torch.zeros(40, 32, dtype=torch.float64).index_add(0, token_idx, y.double() * w.double()[:, None])
    assert torch.equal(permute_oracle.gather_reduce(y, inv_map, w), exact.bfloat16())


def test_bias_gather_backward_is_per_expert_column_sums():
    g = torch.Generator().manual_seed(5)
    eids = torch.sort(torch.randint(0, 6, (50,), generator=g)).values
    eids = eids[eids != 2]  # expert 2 idle
    grad = torch.randn(eids.numel(), 9, dtype=torch.float64, generator=g)
    bias = torch.randn(6, 9, dtype=torch.float64, generator=g).requires_grad_(True)
    bias.index_select(0, eids).backward(grad)
    got = permute_oracle.bias_gather_backward(grad, eids, 6)
    assert torch.allclose(got, bias.grad, rtol=0, atol=1e-12) and not got[2].any()
    assert torch.equal(permute_oracle.bias_gather(bias.detach(), eids), bias.detach()[eids])
