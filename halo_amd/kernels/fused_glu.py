"""Fused GLU combines for MoE expert compute: one row-strided HIP kernel pair serves SiLU, tanh-GELU and the clamped
SwiGLU family.  :meth:`GluCombine.packed` reads a fused ``[gate | up]`` projection in place and returns its gradient
as one buffer, so the expert path copies on neither side of the activation.

Mirrors the reference's ``halo/kernels/fused_glu.py`` (``GluCombine`` ``:306-361``, autograd functions ``:259-299``,
resolvers ``:364-384``, activation probes ``:36-63``); the kernels are ``csrc/glu.hip``.
"""

from __future__ import annotations

import logging
import os
from collections.abc import Callable
from dataclasses import dataclass

import torch

from halo_amd import _lib

logger = logging.getLogger(__name__)


def _env_flag(name: str, default: bool) -> bool:
    value = os.environ.get(name)
    if value is None:
        return default
    return value.strip().lower() not in ("0", "false", "no", "off", "")


# ``HALO_FUSED_GLU=0`` runs every combine as eager torch ops on the device, the reference's escape hatch.
_FUSED_GLU_ENABLED = _env_flag("HALO_FUSED_GLU", True)

_SILU = 0
_GELU_TANH = 1
_CLAMPED_SILU = 2  # alpha-scaled SiLU with the clamps of the GptOss/DeepSeek-V4/Step-3.7 family

# Both saturating tails, both signs, zero and near-zero; it separates every registered activation.
_ACTIVATION_PROBE_INPUT = (-64.0, -8.0, -1.0, -0.5, -1e-3, 0.0, 1e-3, 0.5, 1.0, 8.0, 64.0)


def _computes_exactly(act_fn: object, reference_fn: Callable[[torch.Tensor], torch.Tensor], name: str) -> bool:
    """Bit for bit over the probe vector on the host; behavioural, since an activation module need not be
    ``F.silu`` itself.  Callers latch the result at construction."""
    if not callable(act_fn):
        return False
    try:
        probe = torch.tensor(_ACTIVATION_PROBE_INPUT, dtype=torch.float32, device="cpu")
        expected = reference_fn(probe)
        with torch.no_grad():
            out = act_fn(probe)
        return (
            isinstance(out, torch.Tensor)
            and out.shape == expected.shape
            and out.dtype == expected.dtype
            and torch.equal(out, expected)
        )
    except Exception:
        logger.warning(f"Activation {act_fn!r} could not be probed against {name}; treating it as non-{name}.")
        return False


def is_silu_activation(act_fn: object) -> bool:
    return _computes_exactly(act_fn, torch.nn.functional.silu, "F.silu")


def is_gelu_tanh_activation(act_fn: object) -> bool:
    return _computes_exactly(act_fn, lambda x: torch.nn.functional.gelu(x, approximate="tanh"), "tanh-GELU")


# Eager forms: plain torch ops on whatever device the operands live on (``HALO_FUSED_GLU=0``).
def silu_mul_eager(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    return torch.nn.functional.silu(gate) * up


def gelu_tanh_mul_eager(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    return torch.nn.functional.gelu(gate, approximate="tanh") * up


def gptoss_glu_eager(gate: torch.Tensor, up: torch.Tensor, alpha: float, limit: float) -> torch.Tensor:
    gate = gate.clamp(max=limit)
    up = up.clamp(min=-limit, max=limit)
    return (up + 1) * (gate * torch.sigmoid(gate * alpha))


def clamped_silu_mul_eager(gate: torch.Tensor, up: torch.Tensor, limit: float) -> torch.Tensor:
    return torch.nn.functional.silu(gate.clamp(max=limit)) * up.clamp(min=-limit, max=limit)


def silu_then_clamp_mul_eager(gate: torch.Tensor, up: torch.Tensor, limit: float) -> torch.Tensor:
    return torch.nn.functional.silu(gate).clamp(max=limit) * up.clamp(min=-limit, max=limit)


def _as_rows(t: torch.Tensor) -> torch.Tensor:
    if t.stride(-1) != 1:
        t = t.contiguous()
    return t.reshape(-1, t.shape[-1])


def _glu_forward(gate: torch.Tensor, up: torch.Tensor, combine: "GluCombine") -> torch.Tensor:
    device = _lib.require_device(gate, up)
    n_rows, width = gate.shape
    out = torch.empty((n_rows, width), device=device, dtype=gate.dtype)
    if out.numel():
        with _lib.on_device(device):
            _lib.call("hmoe_glu_fwd", _lib.ptr(gate), _lib.ptr(up), gate.stride(0), up.stride(0), n_rows, width,
                      _lib.dtype_id(gate.dtype), combine.activation, combine.alpha, combine.limit,
                      int(combine.clamp_activated), int(combine.up_plus_one), _lib.ptr(out), _lib.stream_ptr(device))
    return out


def _glu_backward(gate, up, grad_out, dgate, dup, combine: "GluCombine") -> None:
    device = _lib.require_device(gate, up, grad_out, dgate, dup)
    n_rows, width = gate.shape
    if n_rows == 0 or width == 0:
        return
    grad_out = grad_out.contiguous().view(n_rows, width)
    with _lib.on_device(device):
        _lib.call("hmoe_glu_bwd", _lib.ptr(gate), _lib.ptr(up), gate.stride(0), up.stride(0), _lib.ptr(grad_out),
                  n_rows, width, _lib.dtype_id(gate.dtype), combine.activation, combine.alpha, combine.limit,
                  int(combine.clamp_activated), int(combine.up_plus_one), _lib.ptr(dgate), _lib.ptr(dup),
                  dgate.stride(0), dup.stride(0), _lib.stream_ptr(device))


class _FusedGLU(torch.autograd.Function):
    @staticmethod
    def forward(ctx, gate: torch.Tensor, up: torch.Tensor, combine: "GluCombine") -> torch.Tensor:
        shape = gate.shape
        gate2d, up2d = _as_rows(gate), _as_rows(up)
        ctx.save_for_backward(gate2d, up2d)
        ctx.combine, ctx.shape = combine, shape
        return _glu_forward(gate2d, up2d, combine).view(shape)

    @staticmethod
    def backward(ctx, grad_out: torch.Tensor):
        gate, up = ctx.saved_tensors
        dgate = torch.empty(gate.shape, dtype=gate.dtype, device=gate.device)
        dup = torch.empty(up.shape, dtype=up.dtype, device=up.device)
        _glu_backward(gate, up, grad_out, dgate, dup, ctx.combine)
        return dgate.view(ctx.shape), dup.view(ctx.shape), None


class _FusedPackedGLU(torch.autograd.Function):
    """Over a ``[..., 2M]`` ``[gate | up]`` output, read in place with the gradient written as one buffer."""

    @staticmethod
    def forward(ctx, gate_up: torch.Tensor, combine: "GluCombine") -> torch.Tensor:
        shape = gate_up.shape
        rows2d = _as_rows(gate_up)
        width = shape[-1] // 2
        ctx.save_for_backward(rows2d)
        ctx.combine, ctx.shape = combine, shape
        out = _glu_forward(rows2d[:, :width], rows2d[:, width:], combine)
        return out.view(*shape[:-1], width)

    @staticmethod
    def backward(ctx, grad_out: torch.Tensor):
        (rows2d,) = ctx.saved_tensors
        width = rows2d.shape[-1] // 2
        grad = torch.empty(rows2d.shape, device=rows2d.device, dtype=rows2d.dtype)
        _glu_backward(rows2d[:, :width], rows2d[:, width:], grad_out, grad[:, :width], grad[:, width:], ctx.combine)
        return grad.view(ctx.shape), None


def fused_glu_enabled() -> bool:
    return _FUSED_GLU_ENABLED


@dataclass(frozen=True)
class GluCombine:
    """``alpha`` and ``limit`` are runtime kernel arguments; the activation and the two clamp flags pick one of the
    ahead-of-time kernel instances."""

    activation: int
    alpha: float = 1.0
    limit: float = 0.0
    clamp_activated: bool = False
    up_plus_one: bool = False

    @classmethod
    def silu(cls) -> "GluCombine":
        return cls(_SILU)

    @classmethod
    def gelu_tanh(cls) -> "GluCombine":
        return cls(_GELU_TANH)

    @classmethod
    def clamped_silu(cls, limit: float, *, clamp_activated: bool = False) -> "GluCombine":
        """The gate clamped before SiLU (DeepSeek-V4, GLM-5 Next) or, with ``clamp_activated``, after (Step-3.7)."""
        return cls(_CLAMPED_SILU, limit=float(limit), clamp_activated=clamp_activated)

    @classmethod
    def gptoss(cls, alpha: float, limit: float) -> "GluCombine":
        return cls(_CLAMPED_SILU, alpha=float(alpha), limit=float(limit), up_plus_one=True)

    @property
    def name(self) -> str:
        if self.activation != _CLAMPED_SILU:
            return "silu" if self.activation == _SILU else "gelu_tanh"
        if self.up_plus_one:
            return "gptoss"
        return "silu_then_clamp" if self.clamp_activated else "clamped_silu"

    def __call__(self, gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
        if fused_glu_enabled():
            return _FusedGLU.apply(gate, up, self)
        return self._eager(gate, up)

    def packed(self, gate_up: torch.Tensor) -> torch.Tensor:
        if fused_glu_enabled():
            return _FusedPackedGLU.apply(gate_up, self)
        return self._eager(*gate_up.chunk(2, dim=-1))

    def _eager(self, gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
        if self.activation == _SILU:
            return silu_mul_eager(gate, up)
        if self.activation == _GELU_TANH:
            return gelu_tanh_mul_eager(gate, up)
        if self.up_plus_one:
            return gptoss_glu_eager(gate, up, self.alpha, self.limit)
        if self.clamp_activated:
            return silu_then_clamp_mul_eager(gate, up, self.limit)
        return clamped_silu_mul_eager(gate, up, self.limit)


def resolve_fused_glu_mul(act_fn: object) -> GluCombine | None:
    """The fused combine computing ``act_fn(gate) * up``, or None for the eager ``act_fn`` combine."""
    if is_silu_activation(act_fn):
        return GluCombine.silu()
    if is_gelu_tanh_activation(act_fn):
        return GluCombine.gelu_tanh()
    return None


def resolve_clamped_glu_mul(
    act_fn: object, limit: float, *, clamp_activated: bool
) -> Callable[[torch.Tensor, torch.Tensor], torch.Tensor]:
    """Fused for a SiLU gate; any other activation runs the same clamps eagerly."""
    if is_silu_activation(act_fn):
        return GluCombine.clamped_silu(limit, clamp_activated=clamp_activated)

    def clamped_glu_mul_eager(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
        activated = act_fn(gate).clamp(max=limit) if clamp_activated else act_fn(gate.clamp(max=limit))
        return activated * up.clamp(min=-limit, max=limit)

    return clamped_glu_mul_eager
