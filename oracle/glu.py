"""Oracle (test infrastructure): the GLU combines and their gradients on the CPU.

Follows ``halo/kernels/fused_glu.py``: eager forms ``:66-87``, kernel gradient forms ``:155-205``.  Math runs in the
input promoted to at least fp32 (fp64 stays fp64); callers wanting an exact reference pass fp64.
"""

from __future__ import annotations

import math

import torch

SILU, GELU_TANH, CLAMPED_SILU = 0, 1, 2
_SQRT_2_OVER_PI = math.sqrt(2.0 / math.pi)
_GELU_COEFF = 0.044715


def _wide(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.promote_types(t.dtype, torch.float32))


def _clamped_terms(gate, up, alpha, limit, clamp_activated, up_plus_one):
    # halo/kernels/fused_glu.py:104-113
    up_g = up.clamp(min=-limit, max=limit)
    if up_plus_one:
        up_g = up_g + 1.0
    gate_a = gate if clamp_activated else gate.clamp(max=limit)
    s = torch.sigmoid(gate_a * alpha)
    glu = gate_a * s
    activated = glu.clamp(max=limit) if clamp_activated else glu
    return activated, up_g, gate_a, s, glu


def glu_forward(gate: torch.Tensor, up: torch.Tensor, activation: int, alpha: float = 1.0, limit: float = 0.0,
                clamp_activated: bool = False, up_plus_one: bool = False) -> torch.Tensor:
    """``act(gate) * up`` for the five combines (``halo/kernels/fused_glu.py:66-87, 118-152``)."""
    g, u = _wide(gate), _wide(up)
    if activation == SILU:
        out = g * torch.sigmoid(g) * u
    elif activation == GELU_TANH:
        out = 0.5 * g * (1.0 + torch.tanh(_SQRT_2_OVER_PI * (g + _GELU_COEFF * g * g * g))) * u
    else:
        activated, up_g, _, _, _ = _clamped_terms(g, u, alpha, limit, clamp_activated, up_plus_one)
        out = activated * up_g
    return out.to(gate.dtype)


def glu_backward(gate: torch.Tensor, up: torch.Tensor, grad_out: torch.Tensor, activation: int, alpha: float = 1.0,
                 limit: float = 0.0, clamp_activated: bool = False, up_plus_one: bool = False):
    """``(dgate, dup)`` in the closed forms of ``halo/kernels/fused_glu.py:177-203``; a clamp passes its gradient
    through on the closed interval, bounds included."""
    g, u, d = _wide(gate), _wide(up), _wide(grad_out)
    if activation == SILU:
        s = torch.sigmoid(g)
        dgate = d * u * (s * (1.0 + g * (1.0 - s)))
        dup = d * (g * s)
    elif activation == GELU_TANH:
        t = torch.tanh(_SQRT_2_OVER_PI * (g + _GELU_COEFF * g * g * g))
        inner = _SQRT_2_OVER_PI * (1.0 + 3.0 * _GELU_COEFF * g * g)
        dgate = d * u * (0.5 * (1.0 + t) + 0.5 * g * (1.0 - t * t) * inner)
        dup = d * (0.5 * g * (1.0 + t))
    else:
        activated, up_g, gate_a, s, glu = _clamped_terms(g, u, alpha, limit, clamp_activated, up_plus_one)
        dglu = s + gate_a * alpha * s * (1.0 - s)
        up_in = ((u >= -limit) & (u <= limit)).to(g.dtype)
        gate_in = ((glu <= limit) if clamp_activated else (g <= limit)).to(g.dtype)
        dgate = d * up_g * dglu * gate_in
        dup = d * activated * up_in
    return dgate.to(gate.dtype), dup.to(up.dtype)
