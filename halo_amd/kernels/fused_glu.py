"""Fused GLU combines for MoE expert compute: one row-strided HIP kernel pair serves SiLU, tanh-GELU and the clamped
SwiGLU family.  :meth:`GluCombine.packed` reads a fused ``[gate | up]`` projection in place and returns its gradient
as one buffer, so the expert path copies on neither side of the activation.

Same public surface as the reference's ``halo/kernels/fused_glu.py`` (``GluCombine`` ``:306-361``, its resolvers
``:364-384``, the activation probes ``:36-63``, the eager forms ``:66-87``, ``HALO_FUSED_GLU`` ``:21``); the kernels are
``csrc/glu.hip`` and take the combine as (kind, alpha, limit, two flags).
"""

from __future__ import annotations

import logging
import os
from collections.abc import Callable
from dataclasses import dataclass

import torch
import torch.nn.functional as F

from halo_amd import _lib

logger = logging.getLogger(__name__)

# kernel-side activation kinds (csrc/glu.hip)
_SILU, _GELU_TANH, _CLAMPED_SILU = 0, 1, 2

# ``HALO_FUSED_GLU=0`` (or false/no/off/empty) runs every combine as eager torch ops on the device.
_FUSED_GLU_ENABLED = os.environ.get("HALO_FUSED_GLU", "1").strip().lower() not in ("0", "false", "no", "off", "")


def fused_glu_enabled() -> bool:
    return _FUSED_GLU_ENABLED


# ------------------------------------------------------------------------------------------------- eager forms

def _clip_up(up: torch.Tensor, limit: float) -> torch.Tensor:
    return torch.clamp(up, -limit, limit)


def silu_mul_eager(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    return F.silu(gate) * up


def gelu_tanh_mul_eager(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    return F.gelu(gate, approximate="tanh") * up


def clamped_silu_mul_eager(gate: torch.Tensor, up: torch.Tensor, limit: float) -> torch.Tensor:
    """The gate is cut off at ``limit`` before the SiLU, ``up`` is held within ``±limit``."""
    return F.silu(torch.clamp(gate, max=limit)) * _clip_up(up, limit)


def silu_then_clamp_mul_eager(gate: torch.Tensor, up: torch.Tensor, limit: float) -> torch.Tensor:
    """As above with the cut-off applied to the SiLU's result instead of its argument."""
    return torch.clamp(F.silu(gate), max=limit) * _clip_up(up, limit)


def gptoss_glu_eager(gate: torch.Tensor, up: torch.Tensor, alpha: float, limit: float) -> torch.Tensor:
    """gpt-oss: ``(clip(up) + 1) * g * sigmoid(alpha * g)`` with ``g = min(gate, limit)``."""
    g = torch.clamp(gate, max=limit)
    return (g * torch.sigmoid(alpha * g)) * (_clip_up(up, limit) + 1)


# ------------------------------------------------------------------------------------------- activation probes

# Both saturating tails, both signs, zero and values next to it: no two registered activations agree on all of them.
_ACTIVATION_PROBE_INPUT = (-64.0, -8.0, -1.0, -0.5, -1e-3, 0.0, 1e-3, 0.5, 1.0, 8.0, 64.0)


def _computes_exactly(act_fn: object, reference_fn: Callable[[torch.Tensor], torch.Tensor], name: str) -> bool:
    """Whether ``act_fn`` returns ``reference_fn``'s bits on the probe vector (fp32, CPU).  Anything that is not
    callable, raises, or returns another shape or dtype is taken not to be that activation."""
    if not callable(act_fn):
        return False
    points = torch.tensor(_ACTIVATION_PROBE_INPUT, dtype=torch.float32)
    want = reference_fn(points)
    try:
        with torch.no_grad():
            got = act_fn(points)
    except Exception:
        logger.warning(f"Activation {act_fn!r} could not be probed against {name}; treating it as non-{name}.")
        return False
    if not isinstance(got, torch.Tensor) or got.dtype != want.dtype or got.shape != want.shape:
        return False
    return bool(torch.equal(got, want))


def is_silu_activation(act_fn: object) -> bool:
    return _computes_exactly(act_fn, F.silu, "F.silu")


def is_gelu_tanh_activation(act_fn: object) -> bool:
    return _computes_exactly(act_fn, lambda x: F.gelu(x, approximate="tanh"), "tanh-GELU")


# -------------------------------------------------------------------------------------------------- launchers

def _as_rows(t: torch.Tensor) -> torch.Tensor:
    """``[rows, width]`` with unit stride along the width (the kernels take any row stride)."""
    return (t if t.stride(-1) == 1 else t.contiguous()).reshape(-1, t.shape[-1])


def _kernel_args(combine: "GluCombine") -> tuple:
    return (combine.activation, combine.alpha, combine.limit, int(combine.clamp_activated), int(combine.up_plus_one))


def _glu_forward(gate: torch.Tensor, up: torch.Tensor, combine: "GluCombine") -> torch.Tensor:
    device = _lib.require_device(gate, up)
    rows, width = gate.shape
    out = gate.new_empty((rows, width))
    if rows and width:
        with _lib.on_device(device):
            _lib.call("hmoe_glu_fwd", _lib.ptr(gate), _lib.ptr(up), gate.stride(0), up.stride(0), rows, width,
                      _lib.dtype_id(gate.dtype), *_kernel_args(combine), _lib.ptr(out), _lib.stream_ptr(device))
    return out


def _glu_backward(gate, up, grad_out, dgate, dup, combine: "GluCombine") -> None:
    """Writes the gradients into ``dgate`` / ``dup`` (any row stride: the halves of one packed buffer, or two)."""
    device = _lib.require_device(gate, up, grad_out, dgate, dup)
    rows, width = gate.shape
    if rows and width:
        grad_out = grad_out.contiguous().view(rows, width)
        with _lib.on_device(device):
            _lib.call("hmoe_glu_bwd", _lib.ptr(gate), _lib.ptr(up), gate.stride(0), up.stride(0), _lib.ptr(grad_out),
                      rows, width, _lib.dtype_id(gate.dtype), *_kernel_args(combine), _lib.ptr(dgate), _lib.ptr(dup),
                      dgate.stride(0), dup.stride(0), _lib.stream_ptr(device))


class _FusedGLU(torch.autograd.Function):
    """``combine(gate, up)`` over two tensors of one shape."""

    @staticmethod
    def forward(ctx, gate: torch.Tensor, up: torch.Tensor, combine: "GluCombine") -> torch.Tensor:
        g, u = _as_rows(gate), _as_rows(up)
        ctx.combine, ctx.shape = combine, gate.shape
        ctx.save_for_backward(g, u)
        return _glu_forward(g, u, combine).view(gate.shape)

    @staticmethod
    def backward(ctx, grad_out: torch.Tensor):
        g, u = ctx.saved_tensors
        dgate, dup = torch.empty_like(g), torch.empty_like(u)
        _glu_backward(g, u, grad_out, dgate, dup, ctx.combine)
        return dgate.view(ctx.shape), dup.view(ctx.shape), None


class _FusedPackedGLU(torch.autograd.Function):
    """``combine`` over the two halves of a ``[..., 2 M]`` ``[gate | up]`` tensor, read where they lie; the gradient
    comes back as one ``[..., 2 M]`` buffer whose halves the kernel fills."""

    @staticmethod
    def forward(ctx, gate_up: torch.Tensor, combine: "GluCombine") -> torch.Tensor:
        packed = _as_rows(gate_up)
        half = packed.shape[1] // 2
        ctx.combine, ctx.shape = combine, gate_up.shape
        ctx.save_for_backward(packed)
        return _glu_forward(packed[:, :half], packed[:, half:], combine).view(*gate_up.shape[:-1], half)

    @staticmethod
    def backward(ctx, grad_out: torch.Tensor):
        (packed,) = ctx.saved_tensors
        half = packed.shape[1] // 2
        grad = torch.empty_like(packed, memory_format=torch.contiguous_format)
        _glu_backward(packed[:, :half], packed[:, half:], grad_out, grad[:, :half], grad[:, half:], ctx.combine)
        return grad.view(ctx.shape), None


class _WeightedPackedGLU(torch.autograd.Function):
    """``row_weight[:, None] * combine(gate, up)`` over the halves of a packed ``[R, 2 M]`` tensor, the product taken
    in fp32 and rounded once: the MoE combine's gate weight applied ahead of the down projection instead of behind it
    (``sum_k w_k (act_k @ W) = sum_k (w_k act_k) @ W``).  Backward returns the packed gradient and the weights'
    gradient ``<grad_out[r], combine(gate, up)[r]>`` (fp32 sum, cast to the weights' dtype): what the reference's
    weighted unpermute computes as ``<grad_out[token], expert_out[r]>`` (``moe_permute.py:44-72``), without the
    expert outputs."""

    @staticmethod
    def forward(ctx, gate_up: torch.Tensor, row_weight: torch.Tensor, combine: "GluCombine") -> torch.Tensor:
        device = _lib.require_device(gate_up, row_weight)
        packed = _as_rows(gate_up)
        rows, half = packed.shape[0], packed.shape[1] // 2
        # fp32 weights beside bf16 rows go in as they are: the kernel rounds them to bf16 on the way in and their
        # gradient on the way out, the bits of casting first, without the cast launches (one forward, two backward)
        ctx.weight_f32 = row_weight.dtype == torch.float32 and packed.dtype == torch.bfloat16
        weight = row_weight.contiguous() if ctx.weight_f32 else row_weight.to(packed.dtype).contiguous()
        ctx.combine, ctx.shape, ctx.weight_dtype = combine, gate_up.shape, row_weight.dtype
        ctx.save_for_backward(packed, weight)
        out = packed.new_empty((rows, half))
        if rows and half:
            gate, up = packed[:, :half], packed[:, half:]
            with _lib.on_device(device):
                _lib.call("hmoe_glu_fwd_weighted", _lib.ptr(gate), _lib.ptr(up), gate.stride(0), up.stride(0),
                          _lib.ptr(weight), _lib.dtype_id(weight.dtype), rows, half, _lib.dtype_id(packed.dtype),
                          *_kernel_args(combine), _lib.ptr(out), _lib.stream_ptr(device))
        return out

    @staticmethod
    def backward(ctx, grad_out: torch.Tensor):
        packed, weight = ctx.saved_tensors
        device = packed.device
        rows, half = packed.shape[0], packed.shape[1] // 2
        grad = torch.empty_like(packed, memory_format=torch.contiguous_format)
        grad_weight = torch.empty(rows, dtype=torch.float32, device=device)
        if rows and half:
            grad_out = grad_out.contiguous().view(rows, half)
            gate, up = packed[:, :half], packed[:, half:]
            dgate, dup = grad[:, :half], grad[:, half:]
            with _lib.on_device(device):
                _lib.call("hmoe_glu_bwd_weighted", _lib.ptr(gate), _lib.ptr(up), gate.stride(0), up.stride(0),
                          _lib.ptr(grad_out), _lib.ptr(weight), _lib.dtype_id(weight.dtype), rows, half,
                          _lib.dtype_id(packed.dtype),
                          *_kernel_args(ctx.combine), _lib.ptr(dgate), _lib.ptr(dup), dgate.stride(0), dup.stride(0),
                          _lib.ptr(grad_weight), _lib.stream_ptr(device))
        else:
            grad_weight.zero_()
        return (grad.view(ctx.shape), grad_weight.to(ctx.weight_dtype) if ctx.needs_input_grad[1] else None, None)


# ---------------------------------------------------------------------------------------------------- combine

@dataclass(frozen=True)
class GluCombine:
    """One of the fused ``activation(gate) * up`` forms; frozen, so two combines with the same numbers are equal and a
    combine can key a cache.  Calling it (or ``packed``) runs the HIP kernel pair, or the eager form when
    ``HALO_FUSED_GLU`` turns the kernels off or the tensors live on the CPU (``fused_glu.py:352-361`` of the
    reference)."""

    activation: int
    alpha: float = 1.0
    limit: float = 0.0
    clamp_activated: bool = False
    up_plus_one: bool = False

    # constructors -----------------------------------------------------------------------------------------
    @classmethod
    def silu(cls) -> "GluCombine":
        return cls(activation=_SILU)

    @classmethod
    def gelu_tanh(cls) -> "GluCombine":
        return cls(activation=_GELU_TANH)

    @classmethod
    def clamped_silu(cls, limit: float, *, clamp_activated: bool = False) -> "GluCombine":
        """SiLU with the gate cut off at ``limit`` before the activation, or after it with ``clamp_activated``;
        ``up`` within ``±limit`` either way."""
        return cls(activation=_CLAMPED_SILU, limit=float(limit), clamp_activated=bool(clamp_activated))

    @classmethod
    def gptoss(cls, alpha: float, limit: float) -> "GluCombine":
        return cls(activation=_CLAMPED_SILU, alpha=float(alpha), limit=float(limit), up_plus_one=True)

    # use --------------------------------------------------------------------------------------------------
    @property
    def name(self) -> str:
        if self.activation == _CLAMPED_SILU:
            if self.up_plus_one:
                return "gptoss"
            return ("clamped_silu", "silu_then_clamp")[self.clamp_activated]
        return ("silu", "gelu_tanh")[self.activation == _GELU_TANH]

    def __call__(self, gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
        return _FusedGLU.apply(gate, up, self) if _FUSED_GLU_ENABLED and gate.is_cuda else self._eager(gate, up)

    def packed(self, gate_up: torch.Tensor) -> torch.Tensor:
        if _FUSED_GLU_ENABLED and gate_up.is_cuda:
            return _FusedPackedGLU.apply(gate_up, self)
        gate, up = gate_up.chunk(2, dim=-1)
        return self._eager(gate, up)

    def packed_weighted(self, gate_up: torch.Tensor, row_weight: torch.Tensor) -> torch.Tensor:
        """``row_weight[:, None] * packed(gate_up)`` with one rounding (:class:`_WeightedPackedGLU`); ``gate_up`` is
        ``[R, 2 M]``, ``row_weight`` ``[R]``."""
        if _FUSED_GLU_ENABLED and gate_up.is_cuda:
            return _WeightedPackedGLU.apply(gate_up, row_weight, self)
        gate, up = gate_up.chunk(2, dim=-1)
        weight = row_weight.to(gate_up.dtype).float()  # the rounding the kernel gives fp32 weights beside bf16 rows
        return (self._eager(gate, up).float() * weight.unsqueeze(-1)).to(gate_up.dtype)

    def packed_quantized(self, gate_up: torch.Tensor):
        """``packed`` with its output as e4m3 panels and scale exponents for the fp8 expert GEMM
        (:class:`halo_amd.kernels.lowp.block_fp8.QuantizedRows`): the bits ``quantize_rows_fp8(self.packed(gate_up))``
        gives, without the bf16 output being written.  Forward only.  None where the kernel does not apply (kernels
        switched off, not bf16, a half width that is not a multiple of 128, rows that are not 16-byte aligned)."""
        from halo_amd.kernels.lowp.block_fp8 import QuantizedRows

        if not _FUSED_GLU_ENABLED or not gate_up.is_cuda or gate_up.dtype != torch.bfloat16 or gate_up.dim() != 2:
            return None
        if gate_up.requires_grad and torch.is_grad_enabled():
            return None
        packed = _as_rows(gate_up)
        rows, half = packed.shape[0], packed.shape[1] // 2
        if half == 0 or half % 128 or packed.stride(0) % 8 or packed.data_ptr() % 16:
            return None
        device = _lib.require_device(packed)
        q = torch.empty((half // 64, rows, 64), dtype=torch.uint8, device=device)
        scale = torch.empty((half // 128, rows), dtype=torch.uint8, device=device)
        if rows:
            gate, up = packed[:, :half], packed[:, half:]
            with _lib.on_device(device):
                _lib.call("hmoe_glu_fwd_quant_fp8", _lib.ptr(gate), _lib.ptr(up), gate.stride(0), up.stride(0), rows,
                          half, *_kernel_args(self), _lib.ptr(q), _lib.ptr(scale), rows, _lib.stream_ptr(device))
        return QuantizedRows(q.view(torch.float8_e4m3fn), scale)

    def _eager(self, gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
        kind = self.name
        if kind == "silu":
            return silu_mul_eager(gate, up)
        if kind == "gelu_tanh":
            return gelu_tanh_mul_eager(gate, up)
        if kind == "gptoss":
            return gptoss_glu_eager(gate, up, self.alpha, self.limit)
        if kind == "silu_then_clamp":
            return silu_then_clamp_mul_eager(gate, up, self.limit)
        return clamped_silu_mul_eager(gate, up, self.limit)


def resolve_fused_glu_mul(act_fn: object) -> GluCombine | None:
    """The fused combine that computes ``act_fn(gate) * up``; None when ``act_fn`` is neither SiLU nor tanh-GELU (the
    caller then multiplies eagerly)."""
    for probe, make in ((is_silu_activation, GluCombine.silu), (is_gelu_tanh_activation, GluCombine.gelu_tanh)):
        if probe(act_fn):
            return make()
    return None


def resolve_clamped_glu_mul(act_fn: object, limit: float, *,
                            clamp_activated: bool) -> Callable[[torch.Tensor, torch.Tensor], torch.Tensor]:
    """The clamped combine for ``act_fn``: fused when it is SiLU, else the same clamps around ``act_fn`` in torch."""
    if is_silu_activation(act_fn):
        return GluCombine.clamped_silu(limit, clamp_activated=clamp_activated)

    def clamped_glu_mul_eager(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
        if clamp_activated:
            head = torch.clamp(act_fn(gate), max=limit)
        else:
            head = act_fn(torch.clamp(gate, max=limit))
        return head * _clip_up(up, limit)

    return clamped_glu_mul_eager
