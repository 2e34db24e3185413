"""Seeded inputs shared by the CPU (oracle) tests and the GPU parity tests.

The routing roster mirrors the shapes the reference's own sort test runs (``tests/common/route_sort_reference.py:46-59``:
rows, top_k, local experts, ep_size, rows with no local slot, an idle expert); inputs are generated on the CPU from a
seeded ``torch.Generator`` so the oracle and the device see identical bits.
"""

from __future__ import annotations

from typing import NamedTuple

import numpy as np
import torch


class RoutingCase(NamedTuple):
    name: str
    rows: int
    top_k: int
    local_experts: int
    ep_size: int  # 1: every id local, no receive counts
    empty_rows: int = 0
    idle_expert: int | None = None


ROUTING_CASES = (
    RoutingCase("gpt_oss_ep8", 600, 4, 4, 8),
    RoutingCase("qwen3_5_ep8", 300, 8, 32, 8, empty_rows=17),
    RoutingCase("top6_ep4", 400, 6, 16, 4, idle_expert=5),
    RoutingCase("qwen3_next_ep8", 260, 10, 64, 8),
    RoutingCase("ep2_128_local", 200, 8, 128, 2, idle_expert=127),
    RoutingCase("one_local_expert", 300, 4, 1, 32),
    RoutingCase("top1_ep2", 50, 1, 3, 2),
    RoutingCase("no_local_slot", 40, 4, 4, 8, empty_rows=40),
    RoutingCase("zero_tokens", 0, 8, 32, 8),
    RoutingCase("qwen3_5_ep1", 300, 8, 256, 1),
    RoutingCase("qwen3_next_ep1", 120, 10, 512, 1),
    RoutingCase("top1_ep1", 50, 1, 3, 1, idle_expert=2),
    # beyond the reference's roster: several sort blocks, odd top_k, many rows
    RoutingCase("many_blocks_ep1", 5000, 8, 128, 1),
    RoutingCase("many_blocks_ep8", 7001, 7, 24, 8, empty_rows=100, idle_expert=3),
)


def make_receive(case: RoutingCase, seed: int):
    """``(experts i64[rows,k], weights f32[rows,k], counts tuple|None)``: distinct picks per row over the global
    expert set, other ranks' picks as ``-1``, and at ep_size > 1 one slot of every fourth row holding an id just
    past the local range (dropped like a ``-1``)."""
    g = torch.Generator().manual_seed(seed)
    total = case.local_experts * case.ep_size
    picks = torch.rand(case.rows, total, generator=g).argsort(dim=1)[:, : case.top_k]
    if case.idle_expert is not None:
        spare = case.local_experts if case.ep_size > 1 else 0
        picks = torch.where(picks == case.idle_expert, spare, picks)
    experts = torch.where(picks < case.local_experts, picks, -1)
    experts[: case.empty_rows] = -1
    if case.ep_size > 1 and case.rows:
        first = experts[1::4, 0]
        experts[1::4, 0] = torch.where(first < 0, case.local_experts, first)
    weights = torch.rand(experts.shape, generator=g)
    counts = None
    if case.ep_size > 1:
        local = experts[(experts >= 0) & (experts < case.local_experts)]
        counts = tuple(torch.bincount(local, minlength=case.local_experts).tolist())
    return experts, weights, counts


def brute_force_sort(experts: np.ndarray, weights: np.ndarray, num_local_experts: int):
    """The sort's specification slot by slot in pure Python (tiny inputs only)."""
    n_rows, top_k = experts.shape
    entries = []
    for row in range(n_rows):
        for k in range(top_k):
            e = int(experts[row, k])
            if 0 <= e < num_local_experts:
                entries.append((e, row * top_k + k, row, weights[row, k]))
    entries.sort(key=lambda item: (item[0], item[1]))
    n_valid = len(entries)
    offs, running = [], 0
    for e in range(num_local_experts):
        running += sum(1 for item in entries if item[0] == e)
        offs.append(running)
    inv_map = [[n_valid] * top_k for _ in range(n_rows)]
    fill = [0] * n_rows
    dest = [n_valid] * (n_rows * top_k)
    for pos, (_, slot, row, _) in enumerate(entries):
        inv_map[row][fill[row]] = pos
        fill[row] += 1
        dest[slot] = pos
    return (
        np.array([item[2] for item in entries], dtype=np.int64),
        np.array([item[3] for item in entries], dtype=weights.dtype),
        np.array([item[0] for item in entries], dtype=experts.dtype),
        np.array(offs, dtype=np.int32),
        np.array(inv_map, dtype=np.int64).reshape(n_rows, top_k),
        np.array(dest, dtype=np.int32),
    )


class LayerConfig(NamedTuple):
    """One BASELINE.json configuration (or a scaled-down copy for the oracle-speed parity tests)."""

    name: str
    tokens: int
    hidden: int
    experts: int
    top_k: int
    ffn: int
    dtype: torch.dtype
    seed: int
    glu: str = "silu"
    fused: bool = True  # gate_up_proj fused [E,H,2F] vs gate_proj/up_proj apart
    biases: bool = False
    router: str = "softmax_all"  # or "softmax_topk" (gpt-oss)


CONFIG1 = LayerConfig("cfg1_plumbing", 512, 256, 8, 2, 512, torch.float32, 0)
CONFIG2 = LayerConfig("cfg2_qwen3", 8192, 2048, 128, 8, 768, torch.bfloat16, 1)
CONFIG2_SMALL = LayerConfig("cfg2_small", 1024, 512, 32, 8, 256, torch.bfloat16, 1)
CONFIG4 = LayerConfig("cfg4_gptoss", 16384, 2880, 32, 4, 2880, torch.bfloat16, 3, glu="gptoss", fused=False,
                      biases=True, router="softmax_topk")
CONFIG4_SMALL = LayerConfig("cfg4_small", 1024, 360, 16, 4, 360, torch.bfloat16, 3, glu="gptoss", fused=False,
                            biases=True, router="softmax_topk")


def make_layer_inputs(cfg: LayerConfig, *, zipf_alpha: float | None = None, empty_experts: int = 0):
    """Weights ~ N(0, 0.02), x and upstream gradient ~ N(0, 1), generated in fp32 on the CPU and rounded to
    ``cfg.dtype``.  With ``zipf_alpha`` the router bias makes expert popularity follow a Zipf law and forces
    ``empty_experts`` experts to receive nothing (BASELINE config 4)."""
    g = torch.Generator().manual_seed(cfg.seed)
    dt = cfg.dtype

    def normal(*shape, std=1.0):
        return (torch.randn(*shape, generator=g) * std).to(dt)

    inputs = {
        "x": normal(cfg.tokens, cfg.hidden),
        "router_weight": normal(cfg.experts, cfg.hidden, std=0.02),
        "grad_out": normal(cfg.tokens, cfg.hidden),
    }
    params = {}
    if cfg.fused:
        params["gate_up_proj"] = normal(cfg.experts, cfg.hidden, 2 * cfg.ffn, std=0.02)
    else:
        params["gate_proj"] = normal(cfg.experts, cfg.hidden, cfg.ffn, std=0.02)
        params["up_proj"] = normal(cfg.experts, cfg.hidden, cfg.ffn, std=0.02)
    params["down_proj"] = normal(cfg.experts, cfg.ffn, cfg.hidden, std=0.02)
    if cfg.biases:
        for name in [n for n in params]:
            params[name + "_bias"] = normal(cfg.experts, params[name].shape[-1], std=0.02)
    inputs["params"] = params
    if zipf_alpha is not None:
        rank = torch.arange(1, cfg.experts + 1, dtype=torch.float32)
        bias = -zipf_alpha * torch.log(rank)
        bias = bias[torch.randperm(cfg.experts, generator=g)]
        if empty_experts:
            bias[torch.randperm(cfg.experts, generator=g)[:empty_experts]] = -1e9
        inputs["router_bias"] = bias.to(dt)
    return inputs
