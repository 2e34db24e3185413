"""The allocation-free routing sort (``hmoe_route_sort_static``) against ``hmoe_route_sort``, both called straight
through the C ABI: every output bit for bit, on two calls in a row, the second with a smaller routing (the library's
array then still holds the first call's table), and the size limit refused as a status code."""

import pytest
import torch

from halo_amd import _lib
from tests.cases import ROUTING_CASES, make_receive

pytestmark = pytest.mark.gpu


def _sort(entry, experts, weights, local_experts, n_valid, device):
    rows, k = experts.shape
    out = [
        torch.full((n_valid,), -7, dtype=torch.int64, device=device),       # sorted_token_idx
        torch.full((n_valid,), -7.0, dtype=weights.dtype, device=device),   # sorted_weights
        torch.full((n_valid,), -7, dtype=experts.dtype, device=device),     # sorted_expert_ids
        torch.full((local_experts,), -7, dtype=torch.int32, device=device),  # offs
        torch.full((rows, k), -7, dtype=torch.int64, device=device),        # inv_map
        torch.full((rows * k,), -7, dtype=torch.int32, device=device),      # dest
        torch.full((1,), -7, dtype=torch.int32, device=device),             # ok
    ]
    args = [_lib.ptr(experts), experts.element_size(), _lib.ptr(weights), weights.element_size(), rows, k,
            local_experts, n_valid, *(_lib.ptr(t) for t in out)]
    if entry == "hmoe_route_sort":
        bytes_needed = _lib.load().hmoe_route_sort_workspace_bytes(rows, k, local_experts)
        workspace = torch.empty(bytes_needed, dtype=torch.uint8, device=device)
        args.append(_lib.ptr(workspace))
    args.append(_lib.stream_ptr(device))
    _lib.call(entry, *args)
    torch.cuda.synchronize(device)
    return out


def _routing(rows, top_k, local_experts, seed, device):
    g = torch.Generator().manual_seed(seed)
    # a fifth of the slots belong to other ranks (-1), the rest spread over the local experts
    experts = torch.randint(0, local_experts, (rows, top_k), generator=g)
    experts[torch.rand(rows, top_k, generator=g) < 0.2] = -1
    weights = torch.rand(rows, top_k, generator=g)
    n_valid = int((experts >= 0).sum())
    return experts.to(device), weights.to(device), n_valid


def test_static_sort_equals_workspace_sort_on_two_calls_in_a_row(device):
    # first a large routing (many sort blocks), then a smaller one that reuses the start of the same array
    for rows, top_k, local_experts, seed in ((8192, 8, 128, 11), (777, 4, 32, 12)):
        experts, weights, n_valid = _routing(rows, top_k, local_experts, seed, device)
        want = _sort("hmoe_route_sort", experts, weights, local_experts, n_valid, device)
        got = _sort("hmoe_route_sort_static", experts, weights, local_experts, n_valid, device)
        assert int(want[-1].item()) == 1
        for name, g, w in zip(("sorted_token_idx", "sorted_weights", "sorted_expert_ids", "offs", "inv_map", "dest",
                               "ok"), got, want):
            assert torch.equal(g, w), f"rows={rows}: {name}"


def test_static_sort_matches_the_oracle_on_the_reference_held_cases(device):
    import numpy as np

    from oracle import route_sort as oracle

    for index, case in enumerate(ROUTING_CASES[:4]):
        experts, weights, counts = make_receive(case, seed=index)
        n_valid = experts.numel() if counts is None else sum(counts)
        want = oracle.argsort_routing(experts.numpy(), weights.numpy(), case.local_experts, counts)
        got = _sort("hmoe_route_sort_static", experts.to(device), weights.to(device), case.local_experts, n_valid,
                    device)
        for g, w in zip(got[:5], want[:5]):
            g = g.cpu().numpy()
            if g.dtype == np.float32:
                g, w = g.view(np.int32), w.view(np.int32)
            assert np.array_equal(g, w), case.name


def test_static_sort_refuses_a_table_beyond_its_array(device):
    lib = _lib.load()
    rows, top_k, local_experts = 1 << 20, 8, 1024  # 8192 sort blocks x 1024 experts x 4 bytes = 32 MiB
    assert lib.hmoe_route_sort_workspace_bytes(rows, top_k, local_experts) > 4 << 20
    one = torch.zeros(1, dtype=torch.int64, device=device)
    rc = lib.hmoe_route_sort_static(_lib.ptr(one), 8, _lib.ptr(one), 4, rows, top_k, local_experts, 0, None, None,
                                    None, _lib.ptr(one), _lib.ptr(one), _lib.ptr(one), _lib.ptr(one),
                                    _lib.stream_ptr(device))
    assert rc == -2 and b"unsupported" in lib.hmoe_status_string(rc)
