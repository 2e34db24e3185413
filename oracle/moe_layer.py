"""Oracle (test infrastructure): one MoE layer on the CPU, the op sequence the reference runs for CPU tensors.

Without CUDA the reference's layer takes the per-expert loop (``supports_grouped_mm()`` is False,
``halo/hardware.py:35-41``): ``halo/distributed/expert_parallel/moe_layer/compute.py:314-347`` -- per expert, the
slots routed to it, ``x[idx] @ W`` through the GLU FFN (``:357-361``; gpt-oss: ``families/gpt_oss.py:121-137``), the
outputs weighted and ``index_add_``-ed.  The layer shell follows ``moe_layer/shared_experts_layer.py:20-28`` and
``layer.py:270-299`` (routed plus shared expert; Qwen3.5's shared expert is sigmoid-gated,
``families/qwen3_5.py:41-42``).  Everything is torch on the CPU and differentiable, so ``torch.autograd`` gives the
reference gradients.  :func:`dense_formula` is an independent statement of the same result
(``tests/cpu/parallelism/test_moe_permute_equivalence.py:190-196``) used to pin the loop.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch
import torch.nn.functional as F

from oracle import router as router_oracle


@dataclass(frozen=True)
class Glu:
    """Which combine: ``kind`` in silu / gelu_tanh / clamped_silu / silu_then_clamp / gptoss."""

    kind: str = "silu"
    alpha: float = 1.0
    limit: float = 0.0

    def __call__(self, gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
        # halo/kernels/fused_glu.py:66-87
        if self.kind == "silu":
            return F.silu(gate) * up
        if self.kind == "gelu_tanh":
            return F.gelu(gate, approximate="tanh") * up
        if self.kind == "gptoss":
            gate = gate.clamp(max=self.limit)
            up = up.clamp(min=-self.limit, max=self.limit)
            return (up + 1) * (gate * torch.sigmoid(gate * self.alpha))
        if self.kind == "clamped_silu":
            return F.silu(gate.clamp(max=self.limit)) * up.clamp(min=-self.limit, max=self.limit)
        if self.kind == "silu_then_clamp":
            return F.silu(gate).clamp(max=self.limit) * up.clamp(min=-self.limit, max=self.limit)
        raise ValueError(self.kind)


def expert_ffn(x: torch.Tensor, params: dict, e: int, glu: Glu, quant=None) -> torch.Tensor:
    """One expert's GLU FFN on either stored layout (``compute.py:357-361``; ``families/gpt_oss.py:121-137``).
    ``params`` holds ``gate_up_proj [E,H,2F]`` + ``down_proj [E,F,H]`` or ``gate_proj``/``up_proj [E,H,F]`` +
    ``down_proj``, each with an optional ``<name>_bias [E, width]``.  ``quant(t, axis)``, when given, is applied to both
    operands of every product along its contraction axis, which is what the grouped path's low-precision dispatch does
    (``compute.py:306-312`` into ``expert_gemm.py:33-38``: activations along their last axis, ``[E, K, N]`` weights
    along axis 1; a block lies inside one row or one expert's column, so per expert is the same)."""

    def proj(t, name):
        weight = params[name][e]
        out = t @ weight if quant is None else quant(t, -1) @ quant(weight, 0)
        bias = params.get(name + "_bias")
        return out if bias is None else out + bias[e]

    if "gate_up_proj" in params:
        gate, up = proj(x, "gate_up_proj").chunk(2, dim=-1)
    else:
        gate, up = proj(x, "gate_proj"), proj(x, "up_proj")
    return proj(glu(gate, up), "down_proj")


def compute_experts_loop(tokens: torch.Tensor, experts: torch.Tensor, weights: torch.Tensor, params: dict, glu: Glu,
                         num_local_experts: int, quant=None) -> torch.Tensor:
    """``_compute_experts_loop`` (``compute.py:314-347``): ids outside ``[0, E)`` (the dispatch's ``-1``) take no
    part."""
    output = torch.zeros_like(tokens)
    for e in range(num_local_experts):
        top_k_pos, token_idx = torch.where((experts == e).t())
        if token_idx.numel() == 0:
            continue
        out = expert_ffn(tokens.index_select(0, token_idx), params, e, glu, quant)
        output = output.index_add(0, token_idx, out * weights[token_idx, top_k_pos].unsqueeze(-1).to(out.dtype))
    return output


class _CpuGroupedMM(torch.autograd.Function):
    """``F.grouped_mm`` on CPU tensors with the gradients the reference's wrapper takes
    (``halo/kernels/grouped_mm.py:16-47``): both are grouped products again, over a gradient made dense first
    (torch's own backward refuses a broadcast one)."""

    @staticmethod
    def forward(ctx, a, b, offs):
        ctx.save_for_backward(a, b, offs)
        return F.grouped_mm(a, b, offs=offs)

    @staticmethod
    def backward(ctx, grad):
        a, b, offs = ctx.saved_tensors
        grad = grad.contiguous() if grad.numel() else grad.new_empty(grad.shape)
        grad_a = F.grouped_mm(grad, b.transpose(-2, -1), offs=offs) if ctx.needs_input_grad[0] else None
        grad_b = F.grouped_mm(a.transpose(-2, -1), grad, offs=offs) if ctx.needs_input_grad[1] else None
        return grad_a, grad_b, None


def compute_experts_grouped(tokens: torch.Tensor, experts: torch.Tensor, weights: torch.Tensor, params: dict,
                            glu: Glu, num_local_experts: int) -> torch.Tensor:
    """``_compute_experts_grouped`` (``compute.py:222-242``) as it would run on CPU tensors: stable sort of the valid
    slots by expert (``moe_route_sort.py:201-227``), ``index_select`` (``moe_permute.py:133-136``),
    ``F.grouped_mm`` for the fused gate/up and the down projection (``compute.py:357-361``), and the weighted rows
    summed back per token (``moe_permute.py:115-120``).  fp32 only (the reference does not take this path without
    CUDA: it is timed beside the loop for completeness); fused ``gate_up_proj`` layout, no biases."""
    top_k = experts.shape[1]
    flat = experts.reshape(-1)
    slots = torch.nonzero((flat >= 0) & (flat < num_local_experts)).flatten()
    order = slots[torch.argsort(flat[slots], stable=True)]
    token_of = order // top_k
    offs = torch.bincount(flat[order], minlength=num_local_experts).cumsum(0).to(torch.int32)
    rows = tokens.index_select(0, token_of)
    gate, up = _CpuGroupedMM.apply(rows, params["gate_up_proj"], offs).chunk(2, dim=-1)
    out = _CpuGroupedMM.apply(glu(gate, up), params["down_proj"], offs)
    gates = weights.reshape(-1)[order].to(out.dtype)
    return torch.zeros_like(tokens).index_add(0, token_of, out * gates.unsqueeze(-1))


def dense_formula(tokens, experts, weights, params, glu, num_local_experts):
    """``out[t] = sum over valid slots of w[t,k] * FFN_{e[t,k]}(x[t])``, slot by slot."""
    out = torch.zeros_like(tokens)
    for t in range(tokens.shape[0]):
        for k in range(experts.shape[1]):
            e = int(experts[t, k])
            if 0 <= e < num_local_experts:
                out[t] = out[t] + weights[t, k] * expert_ffn(tokens[t : t + 1], params, e, glu)[0]
    return out


def shared_expert(x: torch.Tensor, shared: dict, glu: Glu) -> torch.Tensor:
    """Dense GLU MLP ``down(act(gate(x)) * up(x))`` in ``F.linear`` convention (weights ``[out, in]``), times
    ``sigmoid(x @ gate_w^T)`` when ``shared`` carries ``shared_expert_gate`` (``families/qwen3_5.py:41-42``)."""
    out = F.linear(glu(F.linear(x, shared["gate_proj"]), F.linear(x, shared["up_proj"])), shared["down_proj"])
    if "shared_expert_gate" in shared:
        out = out * torch.sigmoid(F.linear(x, shared["shared_expert_gate"]))
    return out


def moe_layer_forward(x: torch.Tensor, router_weight: torch.Tensor, params: dict, glu: Glu, top_k: int, *,
                      router_bias: torch.Tensor | None = None, mode: int = router_oracle.SOFTMAX_ALL,
                      normalize: bool = True, eps: float = 0.0, indices: torch.Tensor | None = None,
                      shared: dict | None = None, quant=None):
    """Router -> per-expert loop -> (+ shared expert).  ``indices`` overrides the selection (used to compare an fp32
    run against a bf16 run that selected on bf16 logits); ``quant`` as in :func:`expert_ffn` (the routed experts'
    products only).  Returns ``(out, logits, indices, weights)``."""
    logits = F.linear(x, router_weight, router_bias)
    if indices is None:
        indices = router_oracle.select_topk(logits.detach(), top_k)
    weights = router_oracle.gate_weights(logits, indices, mode, normalize, eps).float()
    num_experts = router_weight.shape[0]
    out = compute_experts_loop(x, indices, weights.to(x.dtype), params, glu, num_experts, quant)
    if shared is not None:
        out = out + shared_expert(x, shared, glu)
    return out, logits, indices, weights
