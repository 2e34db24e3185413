"""The MoE block on one GPU: route, sort by expert, grouped GLU FFN, weighted combine, plus the shared expert.

Mirrors the parts of the reference's EP MoE layer that run at ``ep_size`` 1 or on one rank's received rows:
``halo/distributed/expert_parallel/moe_layer/compute.py`` (``_compute_experts`` ``:207-220``,
``_compute_experts_grouped`` ``:222-242``, ``_sort_tokens_for_grouped_mm`` ``:263-281``, ``_expert_proj`` ``:283-294``,
``_glu_ffn`` ``:357-361``, ``_init_fused_glu_params`` ``:77-88``), ``moe_layer/layer.py`` (construction order ``:67-80``,
``_dispatch_compute_combine{,_shared}`` ``:270-342``), ``moe_layer/routing.py`` (``_softmax_gate_weights_at``
``:110-119``) and ``moe_layer/shared_experts_layer.py`` (``forward`` ``:20-28``).  Every tensor op on the path is a HIP
kernel of this package; grouped expert LoRA is in as far as it computes (``moe_layer/expert_lora.py``); the
dispatch/combine exchange, balancing bias, routing replay and expert TP of the reference are not part of it.
"""

from __future__ import annotations

import logging
import os
from abc import ABC, abstractmethod
from collections.abc import Callable
from typing import ClassVar

import torch
import torch.nn as nn

from halo_amd import _lib
from halo_amd.kernels.expert_gemm import BlockFp8Weight, expert_gemm, fp8_mfma_usable
from halo_amd.kernels.fused_glu import GluCombine, fused_glu_enabled, resolve_fused_glu_mul
from halo_amd.kernels.grouped_mm import (GatheredRows, addto_fusable, grouped_mm_addto, grouped_mm_combine,
                                         grouped_mm_forward, grouped_wgrad)
from halo_amd.kernels.moe_permute import (MoEGatherPermute, MoEWeightedUnpermute, MoEWeightedUnpermuteAdd,
                                          warm_permute_kernels)
from halo_amd.kernels.moe_route_sort import sort_routing_by_expert, warm_route_sort_kernels
from halo_amd.kernels.router import SOFTMAX_ALL, fused_topk_gate
from halo_amd.moe_layer.balancing import ExpertLoadMixin
from halo_amd.moe_layer.config import EPConfig, MoEFamilySpec
from halo_amd.moe_layer.expert_lora import EXPERT_LORA_SUFFIXES, init_expert_lora

logger = logging.getLogger(__name__)

ROUTER_TOPK_FIELDS = ("top_k", "num_experts_per_tok", "num_experts_per_token")

# Opt-in: the shared expert's FFN on a second stream (of the same, default priority) beside the routed path, joined
# before the sum; one stream per device.  The reference's HALO_EP_SHARED_OVERLAP (layer.py:31-33, 284-296).
_SHARED_OVERLAP_ENABLED = os.environ.get("HALO_EP_SHARED_OVERLAP", "").strip().lower() in ("1", "true", "yes", "on")
_shared_overlap_streams: dict[int, torch.cuda.Stream] = {}


class _DenseLinear(torch.autograd.Function):
    """``F.linear(x, weight)`` for a dense projection of all tokens (the router's logits ``[T, E]``, the shared expert's
    three projections, ``nn.Linear`` modules in the reference: ``families/qwen3_5.py:41-42``) on this build's grouped
    GEMM kernels with one group.

    Forward ``x @ weight^T`` is the input-gradient kernel's form (both operands contraction-contiguous), the input
    gradient ``grad_out @ weight`` the forward kernel's; each launch takes the largest of the kernels' three tile
    configurations that still gives every compute unit a tile (``csrc/grouped_gemm.hip``: 8192 tokens x 512 columns
    are 64 tiles of 256 x 256 but 256 of 128 x 128).  The weight gradient ``grad_out^T @ x`` is an ``[out, in]`` output
    contracted over all T tokens, a handful of output tiles however small the tile: the tokens are cut into slices
    that the weight-gradient kernel takes as groups, one partial ``[out, in]`` each (rounded to the operands' dtype),
    as many as bring the launch to about one tile per compute unit; the partials are summed in fp32 in a fixed order
    and rounded once, so the result stays deterministic.  Operands the kernels do not take (fp32 under
    ``fp32_router``, rows that are not 16-byte multiples, unaligned views) use the library's dense product."""

    _SPLITS = 32  # at most
    _MIN_TOKENS = 2048
    _slice_ends: ClassVar[dict] = {}  # (device, tokens, splits) -> the slices' row ends; a handful of shapes at most
    _SLICE_ENDS_KEPT = 16

    @staticmethod
    def _slice_ends_for(device: torch.device, tokens: int, splits: int) -> torch.Tensor:
        cache = _DenseLinear._slice_ends
        offs = cache.get((device, tokens, splits))
        if offs is None:
            if len(cache) >= _DenseLinear._SLICE_ENDS_KEPT:  # varying sequence lengths: start over, never grow
                cache.clear()
            offs = torch.arange(1, splits + 1, device=device, dtype=torch.int32) * (tokens // splits)
            cache[(device, tokens, splits)] = offs
        return offs

    @staticmethod
    def _kernel_usable(*operands: torch.Tensor) -> bool:
        """What the grouped kernels ask of their operands: bf16, 16-byte rows, 16-byte aligned."""
        return all(t.dtype == torch.bfloat16 and t.dim() == 2 and t.shape[0] > 0 and t.shape[1] % 8 == 0
                   and t.stride(-1) == 1 and t.stride(0) % 8 == 0 and t.data_ptr() % 16 == 0 for t in operands)

    @staticmethod
    def forward(ctx, x, weight):
        ctx.save_for_backward(x, weight)
        if _DenseLinear._kernel_usable(x, weight) and weight.is_contiguous() and weight.shape[0] % 8 == 0:
            return grouped_mm_forward(x, weight.t().unsqueeze(0), None)  # a transposed view: the kernel reads [out, in]
        return torch.nn.functional.linear(x, weight)

    @staticmethod
    def _splits_for(grad_out: torch.Tensor, x: torch.Tensor) -> int:
        """How many token slices the weight gradient is cut into: the power of two that brings the launch nearest to
        256 output tiles of 256 x 256 without passing it, at most 32, slices of equal whole numbers of tokens."""
        tiles = -(-grad_out.shape[1] // 256) * -(-x.shape[1] // 256)
        splits = _DenseLinear._SPLITS
        while splits > 1 and (splits * tiles > 256 or x.shape[0] % splits):
            splits //= 2
        return splits

    @staticmethod
    def _sliced_wgrad_usable(grad_out: torch.Tensor, x: torch.Tensor) -> bool:
        return (_DenseLinear._kernel_usable(grad_out, x) and x.shape[0] >= _DenseLinear._MIN_TOKENS
                and _DenseLinear._splits_for(grad_out, x) >= 4)

    @staticmethod
    def backward(ctx, grad_out):
        x, weight = ctx.saved_tensors
        grad_x = grad_weight = None
        if ctx.needs_input_grad[0]:
            if _DenseLinear._kernel_usable(grad_out, weight) and weight.is_contiguous():
                grad_x = grouped_mm_forward(grad_out, weight.unsqueeze(0), None)
            else:
                grad_x = grad_out @ weight
        if ctx.needs_input_grad[1]:
            if _DenseLinear._sliced_wgrad_usable(grad_out, x):
                splits = _DenseLinear._splits_for(grad_out, x)
                offs = _DenseLinear._slice_ends_for(x.device, x.shape[0], splits)
                partial = grouped_wgrad(grad_out, x, offs, splits)
                grad_weight = partial.sum(dim=0)  # the reduction accumulates in fp32 and rounds once
            else:
                grad_weight = grad_out.t() @ x
        return grad_x, grad_weight


def dense_mm(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """``x @ weight^T`` for an ``F.linear``-convention ``weight [out, in]`` (the shared expert's projections);
    differentiable in both operands.  See :class:`_DenseLinear`."""
    if not x.is_cuda:
        return torch.nn.functional.linear(x, weight)
    if x.dim() == 2 and weight.dim() == 2 and x.dtype == weight.dtype == torch.bfloat16:
        return _DenseLinear.apply(x, weight)
    return torch.nn.functional.linear(x, weight)


class _SigmoidRowGate(torch.autograd.Function):
    """``sigmoid(x @ weight^T).view(-1)`` for ``weight [1, H]``: the shared expert's per-token output gate
    (``families/qwen3_5.py:41-42`` of the reference: ``torch.sigmoid(self.shared_expert_gate(hidden_states))``), one
    kernel forward and one (plus a small reduction) backward in place of the library's matrix-vector products, the
    sigmoid and their autograd; rounded where those tensor operations round (``csrc/row_gate.hip``)."""

    @staticmethod
    def forward(ctx, x, weight):
        device = _lib.require_device(x, weight)
        gate = torch.empty(x.shape[0], dtype=x.dtype, device=device)
        with _lib.on_device(device):
            _lib.call("hmoe_row_gate_fwd", _lib.ptr(x), x.stride(0), _lib.ptr(weight), x.shape[0], x.shape[1],
                      _lib.dtype_id(x.dtype), _lib.ptr(gate), _lib.stream_ptr(device))
        ctx.save_for_backward(x, weight, gate)
        return gate

    @staticmethod
    def backward(ctx, grad_gate):
        x, weight, gate = ctx.saved_tensors
        device = x.device
        need_x, need_w = ctx.needs_input_grad
        if not (need_x or need_w):
            return None, None
        grad_gate = grad_gate.to(x.dtype).contiguous()
        grad_x = torch.empty_like(x, memory_format=torch.contiguous_format) if need_x else None
        grad_w = torch.empty_like(weight, memory_format=torch.contiguous_format) if need_w else None
        workspace = None
        if need_w:
            nbytes = _lib.load().hmoe_row_gate_bwd_workspace_bytes(x.shape[0], x.shape[1])
            workspace = torch.empty(max(int(nbytes), 4) // 4, dtype=torch.float32, device=device)
        with _lib.on_device(device):
            _lib.call("hmoe_row_gate_bwd", _lib.ptr(x), x.stride(0), _lib.ptr(weight), _lib.ptr(gate),
                      _lib.ptr(grad_gate), x.shape[0], x.shape[1], _lib.dtype_id(x.dtype), _lib.ptr(grad_x),
                      grad_x.stride(0) if need_x else 0, _lib.ptr(grad_w), _lib.ptr(workspace),
                      _lib.stream_ptr(device))
        return grad_x, grad_w


class _ScaleRows(torch.autograd.Function):
    """``rows * scale[:, None]`` (the shared expert's output times its per-token gate, where the sum with the routed
    output is not taken by the combine kernel: under expert parallelism the routed rows come back through the
    exchange first).  Forward is the tensor multiplication; backward is one pass of the combine-backward kernel with
    every row its own token, ``scale * grad`` and ``<grad, rows>`` together, in place of two multiplications and a row
    sum (the dot product accumulated in fp32 and rounded once, where autograd rounds every product first)."""

    @staticmethod
    def forward(ctx, rows, scale):
        ctx.save_for_backward(rows, scale)
        return rows * scale.unsqueeze(-1)

    @staticmethod
    def backward(ctx, grad_out):
        from halo_amd.kernels.moe_permute import _unpermute_backward

        rows, scale = ctx.saved_tensors
        own = torch.arange(rows.shape[0], device=rows.device)
        grad_rows, grad_scale = _unpermute_backward(grad_out, rows, scale, own, ctx.needs_input_grad[1])
        return (grad_rows if ctx.needs_input_grad[0] else None), grad_scale


def sigmoid_row_gate(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """``sigmoid(F.linear(x, weight)).view(-1)`` for ``x [T, H]`` and an ``nn.Linear(H, 1)`` weight ``[1, H]``;
    differentiable in both.  Device tensors whose rows are 16-byte multiples take :class:`_SigmoidRowGate`; CPU
    tensors and other shapes the tensor operations."""
    weight = weight.to(x.dtype)
    row_bytes_ok = x.dim() == 2 and (x.shape[1] * x.element_size()) % 16 == 0 and x.stride(1) == 1 \
        and (x.stride(0) * x.element_size()) % 16 == 0 and x.data_ptr() % 16 == 0
    if (x.is_cuda and row_bytes_ok and x.dtype in (torch.bfloat16, torch.float32) and weight.shape == (1, x.shape[1])
            and weight.is_contiguous() and weight.data_ptr() % 16 == 0 and x.shape[0] > 0):
        return _SigmoidRowGate.apply(x, weight)
    return torch.sigmoid(torch.nn.functional.linear(x, weight)).view(-1)


class EPMoELayerBase(ExpertLoadMixin, nn.Module, ABC):
    """Base class of the per-family MoE blocks.  A family fills in the declarations below, implements ``forward`` and
    overrides the ``_adopt_*`` hooks its expert layout needs.  Built from an HF MoE block
    (``cls(original_layer, ep_config)``, what the reference's ``apply_ep_layers`` does), or directly from tensors with
    :meth:`from_weights`."""

    FAMILY: ClassVar[MoEFamilySpec]
    # HF class name(s) of the MoE block this layer replaces.
    HF_MODULE_NAMES: tuple[str, ...] = ()
    _shared_expert_attr: str = "shared_experts"
    # Attribute the router hangs off, on the wrapped HF block and on this layer.
    _ROUTER_ATTR: str | None = "gate"
    # The floor the family's router adds to a top-k weight sum before renormalising by it.
    _TOPK_WEIGHT_NORM_EPS: float = 1e-20

    def __init__(self, original_layer: nn.Module, ep_config: EPConfig, weights_already_sharded: bool = False):
        # what the HF block holds, found before nn.Module's own state exists
        experts = self._find_experts_container(original_layer)
        router = self._declared_router(original_layer)
        if ep_config.num_experts is None:  # the expert range of this rank follows from the block's expert count
            ep_config.finalize_expert_assignment(self.detect_num_experts(original_layer))
        hidden = self._detect_hidden_dim(router, experts)
        self._init_ep_state(ep_config, hidden)
        # the hooks a family overrides, in the reference's order: router, routing fields, shared expert, activation,
        # expert weights, dtype fix-ups
        if router is not None:
            self.add_module(self._ROUTER_ATTR, router)
        for adopt in (self._adopt_routing, self._adopt_shared_experts):
            adopt(original_layer)
        self._adopt_expert_compute(original_layer, experts)
        self._adopt_expert_params(experts, weights_already_sharded=weights_already_sharded)
        self._finalize_expert_init()
        init_expert_lora(self, ep_config.expert_lora)

    # ---------------------------------------------------------------------------------------------- construction

    @classmethod
    def detect_num_experts(cls, layer: nn.Module) -> int:
        container = cls._find_experts_container(layer)
        if isinstance(container, nn.ModuleList):  # one module per expert
            return len(container)
        return int(container.num_experts)

    @classmethod
    def _declared_router(cls, layer: nn.Module) -> nn.Module | None:
        name = cls._ROUTER_ATTR
        if name is None:  # a family whose router lives outside the block
            return None
        found = getattr(layer, name, None)
        if found is not None:
            return found
        raise AttributeError(f"{cls.__name__} declares _ROUTER_ATTR='{name}', but {type(layer).__name__} has no such "
                             f"attribute")

    @classmethod
    def _find_experts_container(cls, layer: nn.Module) -> nn.Module:
        candidates = cls.FAMILY.experts_container_attrs
        present = [name for name in candidates if hasattr(layer, name)]
        if not present:
            raise AttributeError(f"{cls.__name__}: {type(layer).__name__} carries none of {candidates}")
        return getattr(layer, present[0])

    @classmethod
    def _detect_hidden_dim(cls, router: nn.Module | None, experts: nn.Module) -> int:
        weight = getattr(router, "weight", None)
        if weight is not None:  # [E, H]
            return int(weight.shape[1])
        return int(cls._require_fused_experts(experts).gate_up_proj.shape[2])  # HF layout [E, 2F, H]

    @staticmethod
    def _require_fused_experts(experts: nn.Module) -> nn.Module:
        absent = [name for name in ("gate_up_proj", "down_proj") if getattr(experts, name, None) is None]
        if not absent:
            return experts
        raise AttributeError(f"Expected fused-GLU experts carrying gate_up_proj and down_proj, but "
                             f"{type(experts).__name__} carries no {absent}")

    def _init_ep_state(self, ep_config: EPConfig, hidden_dim: int) -> None:
        if not ep_config.grouped_gemm_enabled:
            raise NotImplementedError("the per-expert loop is the reference's CPU path; this block runs the grouped "
                                      "kernels only (use_grouped_gemm=True)")
        super().__init__()
        self.ep_config, self.hidden_dim = ep_config, hidden_dim
        # the fields the reference's block exposes, copied off the config
        for field, source in (("num_experts", "num_experts"), ("experts_per_rank", "experts_per_rank"),
                              ("ep_rank", "ep_rank"), ("ep_size", "ep_size"), ("expert_start", "expert_start_idx"),
                              ("expert_end", "expert_end_idx"), ("expert_tp_size", "expert_tp_size"),
                              ("expert_tp_rank", "expert_tp_rank"), ("fp32_router", "fp32_router"),
                              ("fp32_experts", "fp32_experts")):
            setattr(self, field, getattr(ep_config, source))
        self._use_grouped_mm = True
        self._expert_kernels_warmed = False
        self._lowp_quant_format = None
        self._lowp_weight_cacheable = True
        # quantised weights only: quantise the activations too and multiply on the e4m3 MFMA
        self._lowp_fp8_activations = False
        # with it: the SwiGLU kernel writes the down projection's e4m3 operand itself
        self.fuse_glu_quantise = True
        # the first expert projection gathers its rows by index instead of reading a permuted copy of the tokens
        self.fuse_permute_into_gemm = True
        # the shared expert's output joins the routed one in the combine kernel instead of a tensor addition
        self.fuse_shared_into_combine = True
        self.fuse_shared_gate_up = True
        # an adapted projection adds its low-rank delta in the second adapter product's epilogue
        self.fuse_lora_into_gemm = True
        # the gate weights multiply the GLU's output instead of the down projection's: the combine becomes a plain
        # sum and its backward writes no [R, H] gradient (see _compute_experts_weight_folded)
        self.fold_gate_weight_into_glu = True
        self._fused_glu_mul: Callable | None = None
        # labels the dispatch / expert-compute / combine spans at no device cost (swappable, as in the reference)
        self._perf = torch.profiler.record_function

    def _adopt_routing(self, original_layer: nn.Module) -> None:
        self.top_k = self._find_top_k(original_layer)

    @classmethod
    def _find_top_k(cls, layer: nn.Module) -> int:
        router = getattr(layer, cls._ROUTER_ATTR, None) if cls._ROUTER_ATTR else None
        for source in (layer, router, getattr(layer, "config", None)):
            for attr in ROUTER_TOPK_FIELDS:
                if source is not None and hasattr(source, attr):
                    return int(getattr(source, attr))
        raise AttributeError(f"Cannot determine top_k from {type(layer).__name__}: none of {ROUTER_TOPK_FIELDS}")

    def _adopt_shared_experts(self, original_layer: nn.Module) -> None:
        for attr in self.FAMILY.shared_expert_attrs:
            if getattr(original_layer, attr, None) is not None:
                self._shared_expert_attr = attr
                setattr(self, attr, getattr(original_layer, attr))
                return
        if self.FAMILY.shared_expert_attrs:
            raise AttributeError(f"{type(self).__name__} declares shared experts {self.FAMILY.shared_expert_attrs}, "
                                 f"but {type(original_layer).__name__} carries none")

    def _adopt_expert_compute(self, original_layer: nn.Module, experts: nn.Module) -> None:
        act_fn = getattr(experts, "act_fn", None)
        if act_fn is None:
            raise AttributeError(f"{type(self).__name__}: {type(experts).__name__}.act_fn does not name the expert "
                                 f"activation")
        self.act_fn = act_fn
        self._fused_glu_mul = resolve_fused_glu_mul(act_fn)
        if self._fused_glu_mul is None:
            raise NotImplementedError(f"expert activation {act_fn!r} has no fused combine (SiLU and tanh-GELU do)")

    def _local_expert_range(self, weights_already_sharded: bool) -> tuple[int, int]:
        return (0, self.experts_per_rank) if weights_already_sharded else (self.expert_start, self.expert_end)

    def _adopt_expert_params(self, experts: nn.Module, weights_already_sharded: bool = False) -> None:
        """HF ``gate_up_proj [E, 2F, H]`` / ``down_proj [E, H, F]`` to the matmul convention ``[E, K, N]``: fused
        ``gate_up_proj [E, H, 2F]`` (columns ``[gate | up]``) + ``down_proj [E, F, H]``, or gate and up apart on a
        ``separate_glu`` family."""
        self._require_fused_experts(experts)
        start, end = self._local_expert_range(weights_already_sharded)
        def to_matmul_layout(weight: torch.Tensor) -> nn.Parameter:  # [E, out, in] -> [E, in, out], dense
            return nn.Parameter(weight.transpose(1, 2).contiguous())

        local = slice(start, end)
        fused = experts.gate_up_proj.data[local]
        if self.FAMILY.expert_layout != "separate_glu":
            self.gate_up_proj = to_matmul_layout(fused)
        else:
            halves = fused.chunk(2, dim=1)  # rows [gate ; up] of the HF weight
            self.gate_proj, self.up_proj = to_matmul_layout(halves[0]), to_matmul_layout(halves[1])
        self.down_proj = to_matmul_layout(experts.down_proj.data[local])

    def _finalize_expert_init(self) -> None:
        router_name = self._ROUTER_ATTR
        if router_name is not None and self.fp32_router:
            getattr(self, router_name).float()  # nn.Module.float() converts in place
        if not self.fp32_experts:
            return
        for name, weight in self.expert_named_params():
            upcast = nn.Parameter(weight.data.to(torch.float32), requires_grad=weight.requires_grad)
            setattr(self, name, upcast)

    def expert_named_params(self) -> list:
        held = (root for root in self.FAMILY.expert_weight_roots if hasattr(self, root))
        return [(root, getattr(self, root)) for root in held]

    def replicated_named_params(self) -> list:
        shared = getattr(self, self._shared_expert_attr, None)
        return [] if shared is None else [(f"{self._shared_expert_attr}.{n}", p) for n, p in shared.named_parameters()]

    @abstractmethod
    def forward(self, hidden_states: torch.Tensor, **kwargs): ...

    # -------------------------------------------------------------------------------------------- expert compute

    def _warm_expert_kernels(self, device: torch.device, dtype: torch.dtype, hidden: int, top_k: int) -> None:
        """Ahead-of-time binaries: nothing compiles or loads lazily on first launch.  Kept so callers of the
        reference's hook find it; it loads the library once."""
        if self._expert_kernels_warmed:
            return
        self._expert_kernels_warmed = True
        warm_route_sort_kernels(top_k, self.experts_per_rank, device)
        warm_permute_kernels(16, hidden, top_k, device, dtype)

    def _compute_experts(self, tokens: torch.Tensor, experts: torch.Tensor, weights: torch.Tensor,
                         output_dtype: torch.dtype, *, recv_counts: tuple[int, ...] | None,
                         addend: tuple[torch.Tensor, torch.Tensor | None] | None = None,
                         addend_ready: "torch.cuda.Stream | None" = None) -> torch.Tensor:
        """``experts``/``weights`` are ``[T, top_k]`` local ids (``-1`` = not this rank's) and gate weights;
        ``recv_counts`` counts per local expert, None at ``ep_size`` 1.  ``addend = (rows [T, H], scale [T] or None)``
        (not in the reference's signature) is added to the result, ``scale[:, None] * rows``, by the combine kernel;
        ``addend_ready`` is the stream that produces it, waited for right ahead of that kernel."""
        if tokens.shape[0] == 0:
            return torch.zeros((0, tokens.shape[-1]), device=tokens.device, dtype=output_dtype)
        return self._compute_experts_grouped(tokens, experts, weights, output_dtype, recv_counts=recv_counts,
                                             addend=addend, addend_ready=addend_ready)

    def _compute_experts_grouped(self, tokens, experts, weights, output_dtype, *, recv_counts, addend=None,
                                 addend_ready=None):
        """Sort -> grouped GLU FFN -> weighted unpermute."""
        sorted_tokens, offs, sorted_token_idx, sorted_weights, sorted_expert_ids, inv_map = (
            self._sort_tokens_for_grouped_mm(tokens, experts, weights, recv_counts=recv_counts)
        )
        if self._folds_gate_weight(sorted_tokens, output_dtype):
            return self._compute_experts_weight_folded(sorted_tokens, offs, sorted_token_idx, sorted_weights, inv_map,
                                                       output_dtype, addend, addend_ready)
        expert_out = self._grouped_expert_ffn(sorted_tokens.to(output_dtype), offs, sorted_expert_ids, output_dtype)
        if addend_ready is not None:
            torch.cuda.current_stream(tokens.device).wait_stream(addend_ready)
        if addend is not None:
            rows, scale = addend
            return MoEWeightedUnpermuteAdd.apply(
                expert_out.to(output_dtype).contiguous(), sorted_weights.to(output_dtype), sorted_token_idx, inv_map,
                rows.to(output_dtype), None if scale is None else scale.to(output_dtype))
        return MoEWeightedUnpermute.apply(
            expert_out.to(output_dtype).contiguous(), sorted_weights.to(output_dtype), sorted_token_idx, inv_map
        )

    def _folds_gate_weight(self, sorted_tokens, output_dtype: torch.dtype) -> bool:
        """Whether the layer takes :meth:`_compute_experts_weight_folded`: bf16, gate and up stored fused, a fused
        combine, a plain bf16 down projection without a bias (``(w act) @ W + w b`` is not ``w (act @ W + b)``'s
        kernel), no adapters and no low-precision route."""
        down = getattr(self, "down_proj", None)
        if not (self.fold_gate_weight_into_glu and self._stores_fused_glu and fused_glu_enabled()
                and isinstance(self._fused_glu_mul, GluCombine) and self._lowp_quant_format is None
                and not self.has_expert_lora and getattr(self, "down_proj_bias", None) is None
                and isinstance(self.gate_up_proj, torch.Tensor) and isinstance(down, torch.Tensor)):
            return False
        # what combine_fusable asks of the operands, read off the parameter without casting it
        return (sorted_tokens.dtype == torch.bfloat16 and output_dtype == torch.bfloat16 and down.is_cuda
                and down.dim() == 3 and (down.dtype != output_dtype or down.is_contiguous())
                and down.shape[1] % 8 == 0 and down.shape[2] % 8 == 0)

    def _compute_experts_weight_folded(self, sorted_tokens, offs, sorted_token_idx, sorted_weights, inv_map,
                                       output_dtype, addend, addend_ready=None):
        """The same layer with the gate weight moved ahead of the down projection:
        ``sum_k w_k (act_k @ W_down) = sum_k (w_k act_k) @ W_down``.  The GLU kernel writes ``round(w * act)`` (one
        rounding, where the reference rounds ``act`` and applies ``w`` in the combine, ``compute.py:222-242`` +
        ``moe_permute.py:33-41``), the down projection runs on those rows, and the combine is a plain sum per token.
        In backward the down projection's two gradients fetch ``grad_out[token of row]`` through the sort's index, so
        the ``[R, H]`` gradient of the expert outputs (``moe_permute.py:44-72``) is never written or re-read, the
        expert outputs are not kept, and the gate weights' gradient ``<grad_out[token], y_row>`` comes out of the
        GLU's backward as ``<grad_out[token] @ W_down^T, act_row>``, the same number."""
        gate_up = self._expert_proj(sorted_tokens.to(output_dtype), "gate_up_proj", offs, output_dtype)
        # the fp32 gate weights go in uncast: the kernel rounds them to the output dtype (sorted_weights.to(dt) of
        # compute.py:241) and their gradient back through it
        weighted = self._fused_glu_mul.packed_weighted(gate_up, sorted_weights)
        rows, scale = addend if addend is not None else (None, None)
        if addend_ready is not None:
            # the join: the down projection runs ahead of the sum in the same node, so it waits with it (the gate_up
            # projection and the GLU have overlapped with the shared expert by now)
            torch.cuda.current_stream(weighted.device).wait_stream(addend_ready)
        return grouped_mm_combine(
            weighted, self._cast_weight("down_proj", output_dtype), offs=offs, row_index=sorted_token_idx,
            inv_map=inv_map, addend=None if rows is None else rows.to(output_dtype),
            scale=None if scale is None else scale.to(output_dtype))

    def _require_recv_counts(self, recv_counts: tuple[int, ...] | None) -> tuple[int, ...]:
        if recv_counts is not None and len(recv_counts) == self.experts_per_rank:
            return recv_counts
        raise RuntimeError(f"{type(self).__name__}: the expert compute at ep_size={self.ep_size} needs the dispatch's "
                           f"per-local-expert receive counts ({self.experts_per_rank} of them), got {recv_counts!r}.")

    def _sort_tokens_for_grouped_mm(self, tokens, experts, weights, *, recv_counts):
        """``(sorted_tokens, offs, sorted_token_idx, sorted_weights, sorted_expert_ids, inv_map)`` over the valid local
        assignments; the dispatch's -1 padding is dropped.  At ``ep_size > 1`` the host-side counts size the sort."""
        counts = self._require_recv_counts(recv_counts) if self.ep_size > 1 else None
        sorted_token_idx, sorted_weights, sorted_expert_ids, offs, inv_map = sort_routing_by_expert(
            experts, weights, self.experts_per_rank, counts
        )
        # The permuted copy is left to the first expert projection, whose loader can fetch the rows through the index
        # (one pass over the tokens saved each way); a projection that cannot asks for the copy.  Only where one node
        # reads the rows (gate and up stored fused, or apart and run as a pair): two nodes would each scatter a
        # gradient back.
        fuse = self.fuse_permute_into_gemm and (self._stores_fused_glu or self._pairs_gate_up())
        sorted_tokens = (GatheredRows(tokens, sorted_token_idx, inv_map) if fuse
                         else MoEGatherPermute.apply(tokens, sorted_token_idx, inv_map))
        return sorted_tokens, offs, sorted_token_idx, sorted_weights, sorted_expert_ids, inv_map

    def _grouped_expert_ffn(self, sorted_tokens, offs, sorted_expert_ids, output_dtype):
        def proj(x, attr):
            return self._expert_proj(x, attr, offs, output_dtype)

        if self._stores_fused_glu:
            return self._glu_ffn(sorted_tokens, proj)
        gate, up = self._project_gate_up(sorted_tokens, offs, output_dtype, None, proj, with_bias=False)
        return proj(self._glu_combine(gate, up), "down_proj")

    def _gate_up_attrs(self) -> tuple[str, str] | None:
        """The attribute names of the gate and up weights where the layer stores them apart."""
        return None if self._stores_fused_glu else ("gate_proj", "up_proj")

    def _pairs_gate_up(self) -> bool:
        """Whether gate and up, stored apart, run as one node over rows fetched through the sort's index
        (``GatheredRows.grouped_mm_pair``): plain weights, no adapters on either, no low-precision route, and a bias
        only where the GEMM's epilogue adds it."""
        attrs = self._gate_up_attrs()
        if attrs is None or self._lowp_quant_format is not None:
            return False
        for attr in attrs:
            if self._adapted(attr) or not isinstance(getattr(self, attr, None), torch.Tensor):
                return False
            if getattr(self, f"{attr}_bias", None) is not None and not getattr(self, "fuse_bias_into_gemm", True):
                return False
        return True

    def _project_gate_up(self, x, offs, out_dtype, eids, proj, *, with_bias: bool):
        """``(gate, up)`` of rows ``x``.  Rows nobody has copied yet go through the pair node when the operands
        qualify (both projections fetch them by index, their two input gradients are summed in the second one's
        epilogue); otherwise the rows are copied once and ``proj`` runs twice, as the reference has it
        (``compute.py:222-242``, ``families/gpt_oss.py:139-152``)."""
        gate_attr, up_attr = self._gate_up_attrs()
        if isinstance(x, GatheredRows):
            pair = None
            if self._pairs_gate_up():
                def operand(name):
                    tensor = getattr(self, name, None)
                    return None if tensor is None else tensor.to(out_dtype)

                biases = [operand(f"{attr}_bias") if with_bias else None for attr in (gate_attr, up_attr)]
                pair = x.grouped_mm_pair(operand(gate_attr), biases[0], operand(up_attr), biases[1], offs=offs,
                                         eids=eids)
            if pair is not None:
                return pair
            x = x.materialize()
        return proj(x, gate_attr), proj(x, up_attr)

    @property
    def has_expert_lora(self) -> bool:
        return bool(getattr(self, "_expert_lora_attrs", None))

    def expert_lora_named_params(self) -> list:
        names = [attr + suffix for attr in sorted(self._expert_lora_attrs) for suffix in EXPERT_LORA_SUFFIXES]
        return [(name, getattr(self, name)) for name in names]

    def _adapted(self, weight_attr: str) -> bool:
        return self.has_expert_lora and self._expert_adapters_enabled and weight_attr in self._expert_lora_attrs

    def _expert_proj(self, x: torch.Tensor, weight_attr: str, offs: torch.Tensor, out_dtype: torch.dtype):
        if self._adapted(weight_attr):
            # x @ W + scaling * (dropout(x) @ A) @ B, the adapter products in the activation dtype whatever the
            # base weight is stored in (a scale block along a rank of 8-64 means nothing)
            lora_a = getattr(self, weight_attr + EXPERT_LORA_SUFFIXES[0]).to(out_dtype)
            lora_b = getattr(self, weight_attr + EXPERT_LORA_SUFFIXES[1]).to(out_dtype)
            weight = self._cast_weight(weight_attr, out_dtype)
            base = low = None
            drops = isinstance(self.expert_lora_dropout, nn.Dropout) and self.training and self.expert_lora_dropout.p > 0
            if isinstance(x, GatheredRows) and not drops and self._lowp_quant_format is None:
                # both readers of the rows fetch them through the sort's index: no permuted copy for the adapters
                base, low = x.grouped_mm(weight, offs=offs), x.grouped_mm(lora_a, offs=offs)
            if base is None or low is None:
                rows = x.materialize() if isinstance(x, GatheredRows) else x
                base = self._grouped_mm(rows, weight, offs=offs)
                low = self._grouped_mm(self.expert_lora_dropout(rows), lora_a, offs=offs, lowp=False)
            if self.fuse_lora_into_gemm and addto_fusable(low, lora_b, base):
                # the delta joins the base projection in the second adapter product's epilogue: the same bits
                return grouped_mm_addto(low, lora_b, base, self.expert_lora_scaling, offs=offs)
            return base + self.expert_lora_scaling * self._grouped_mm(low, lora_b, offs=offs, lowp=False)
        weight = self._cast_weight(weight_attr, out_dtype)
        if isinstance(x, GatheredRows):
            if (isinstance(weight, BlockFp8Weight) and self._lowp_fp8_activations and x.dtype == torch.bfloat16
                    and fp8_mfma_usable(weight.shape[1], weight.shape[2])):
                return self._grouped_mm(x, weight, offs=offs)  # the row quantiser fetches the rows itself
            if self._lowp_quant_format is not None and isinstance(weight, torch.Tensor):
                return self._grouped_mm(x, weight, offs=offs)  # as above: quantised as they are fetched
            fused = x.grouped_mm(weight, offs=offs) if self._lowp_quant_format is None else None
            if fused is not None:
                return fused
            x = x.materialize()
        return self._grouped_mm(x, weight, offs=offs)

    def set_lowp_compute(self, quant_format, *, weight_cacheable: bool) -> bool:
        """Set this layer's expert-compute quantisation format (``"mxfp8"``); returns whether it applies (always: the
        layer runs on the grouped kernels only).  ``weight_cacheable=False`` re-quantises the weights on every call,
        for parameters whose version counter does not track the optimizer step.  Reference ``compute.py:53-58``."""
        if quant_format is not None:
            from halo_amd.kernels.lowp.spec import require_implemented

            require_implemented(quant_format)
        self._lowp_quant_format = quant_format
        self._lowp_weight_cacheable = weight_cacheable
        return self._use_grouped_mm

    def _cast_weight(self, weight_attr: str, out_dtype: torch.dtype):
        weight = getattr(self, weight_attr)
        return weight.to(out_dtype) if isinstance(weight, torch.Tensor) else weight

    def _grouped_mm(self, mat_a, mat_b, *, offs=None, lowp: bool = True):
        return expert_gemm(mat_a, mat_b, offs=offs, quant_format=self._lowp_quant_format if lowp else None,
                           weight_cacheable=self._lowp_weight_cacheable,
                           fp8_activations=lowp and getattr(self, "_lowp_fp8_activations", False))

    @property
    def _stores_fused_glu(self) -> bool:
        return hasattr(self, "gate_up_proj")

    def _glu_ffn(self, x: torch.Tensor, proj: Callable[[torch.Tensor, str], torch.Tensor]) -> torch.Tensor:
        if self._stores_fused_glu:  # one projection to [gate | up], combined where it lies
            gate_up = proj(x, "gate_up_proj")
            hidden = self._glu_combine_quantized(gate_up)
            if hidden is None:
                hidden = self._glu_combine_packed(gate_up)
        else:
            hidden = self._glu_combine(proj(x, "gate_proj"), proj(x, "up_proj"))
        return proj(hidden, "down_proj")

    def _glu_combine(self, gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
        return self._fused_glu_mul(gate, up)

    def _glu_combine_quantized(self, gate_up: torch.Tensor):
        """The combine writing the down projection's e4m3 operand directly, where that projection runs on the e4m3
        MFMA (quantised weights with ``_lowp_fp8_activations``); None otherwise."""
        down = getattr(self, "down_proj", None)
        combine = self._fused_glu_mul
        if self._adapted("down_proj"):  # the adapter products take the bf16 rows
            return None
        if not (self._lowp_fp8_activations and self.fuse_glu_quantise and isinstance(down, BlockFp8Weight)
                and isinstance(combine, GluCombine) and isinstance(gate_up, torch.Tensor)
                and fp8_mfma_usable(down.shape[1], down.shape[2])):
            return None
        return combine.packed_quantized(gate_up)

    def _glu_combine_packed(self, gate_up: torch.Tensor) -> torch.Tensor:
        combine = self._fused_glu_mul
        if not isinstance(combine, GluCombine):  # an eager callable: it takes the halves as two tensors
            return self._glu_combine(*gate_up.chunk(2, dim=-1))
        return combine.packed(gate_up)

    def _glu_combine_name(self) -> str:
        combine = self._fused_glu_mul
        if fused_glu_enabled() and combine is not None:
            if isinstance(combine, GluCombine):
                return combine.name
            return getattr(combine, "__name__", "eager")
        return "eager"

    # ------------------------------------------------------------------------------------------------- routing

    def _router_input(self, hidden: torch.Tensor) -> torch.Tensor:
        router = getattr(self, self._ROUTER_ATTR) if self._ROUTER_ATTR else None
        weight = getattr(router, "weight", None)
        upcast = self.fp32_router and weight is not None and weight.dtype == torch.float32
        return hidden.float() if upcast else hidden

    def _linear_router_logits(self, flat: torch.Tensor) -> torch.Tensor:
        """The router's logits at the input dtype (fp32 under ``fp32_router``), fp32 accumulation, one rounding."""
        router = getattr(self, self._ROUTER_ATTR)
        x = self._router_input(flat)
        logits = _DenseLinear.apply(x, router.weight.to(x.dtype))
        bias = getattr(router, "bias", None)
        return logits if bias is None else logits + bias.to(logits.dtype)

    # ------------------------------------------------------------------------------- dispatch / compute / combine

    def _dispatch_compute_combine(self, flat: torch.Tensor, experts: torch.Tensor, weights: torch.Tensor,
                                  input_dtype: torch.dtype, addend=None, addend_ready=None) -> torch.Tensor:
        """At ``ep_size`` 1 dispatch and combine are the identity; the spans keep the reference's names."""
        if self.ep_size > 1:
            raise NotImplementedError(
                "forward() at ep_size > 1 needs the dispatch/combine exchange, which is outside this build; hand the "
                "received rows to _compute_experts(recv_x, recv_topk_idx, recv_topk_weights, dtype, recv_counts=...)"
            )
        self._warm_expert_kernels(flat.device, input_dtype, flat.shape[-1], experts.shape[1])
        self._record_expert_load(experts)
        with self._perf("ep.dispatch"):
            recv_x, recv_topk_idx, recv_topk_weights, recv_counts = flat, experts, weights, None
        with self._perf("ep.expert_compute"):
            output = self._compute_experts(recv_x, recv_topk_idx, recv_topk_weights, input_dtype,
                                           recv_counts=recv_counts, addend=addend, addend_ready=addend_ready)
        with self._perf("ep.combine"):
            combined = output
        return combined

    def _dispatch_compute_combine_shared(self, flat, experts, weights, input_dtype, orig_shape, shared_fn,
                                         shared_parts_fn=None):
        """``routed + shared``.  With ``shared_parts_fn`` (the shared expert's output as ``(rows [T, H], scale [T] or
        None)``, ``shared = scale[:, None] * rows``) and tokens to route, the sum is taken by the combine kernel.
        Under ``HALO_EP_SHARED_OVERLAP`` the shared expert runs on a side stream beside the routed path and the two
        are joined before the sum (``layer.py:284-296`` of the reference)."""
        fused = shared_parts_fn is not None and self.fuse_shared_into_combine and flat.shape[0] > 0
        if shared_fn is not None and _SHARED_OVERLAP_ENABLED and flat.is_cuda:
            index = flat.device.index if flat.device.index is not None else torch.cuda.current_device()
            side = _shared_overlap_streams.get(index)
            if side is None:
                side = _shared_overlap_streams[index] = torch.cuda.Stream(device=index)  # default priority
            current = torch.cuda.current_stream(flat.device)
            side.wait_stream(current)
            with torch.cuda.stream(side):
                shared = shared_parts_fn() if fused else shared_fn()
            if not fused:
                routed = self._dispatch_compute_combine(flat, experts, weights, input_dtype).view(*orig_shape)
                current.wait_stream(side)
                shared.record_stream(current)  # the side stream's tensor stays alive for the sum
                return routed + shared
            # the combine kernel takes the shared rows: everything ahead of it overlaps, the join sits in front of it
            for part in shared:
                if part is not None:
                    part.record_stream(current)
            return self._dispatch_compute_combine(flat, experts, weights, input_dtype, addend=shared,
                                                  addend_ready=side).view(*orig_shape)
        if fused:
            return self._dispatch_compute_combine(flat, experts, weights, input_dtype,
                                                  addend=shared_parts_fn()).view(*orig_shape)
        routed = self._dispatch_compute_combine(flat, experts, weights, input_dtype).view(*orig_shape)
        return routed if shared_fn is None else routed + shared_fn()

    # ---------------------------------------------------------------------------------- construction from tensors

    @classmethod
    def from_weights(cls, *, router_weight: torch.Tensor | None, top_k: int, ep_config: EPConfig | None = None,
                     **expert_tensors: torch.Tensor):
        """A layer built straight from tensors in the runtime layout (``gate_up_proj [E,H,2F]`` + ``down_proj [E,F,H]``,
        or ``gate_proj``/``up_proj [E,H,F]``; optional ``*_bias``), for benches and tests that have no HF block."""
        self = cls.__new__(cls)
        down = expert_tensors["down_proj"]
        local_experts = down.shape[0]
        if ep_config is None:
            ep_config = EPConfig(num_experts=local_experts)
        elif ep_config.num_experts is None:
            ep_config.finalize_expert_assignment(local_experts * ep_config.ep_size)
        self._init_ep_state(ep_config, down.shape[2])
        self.top_k = top_k
        if router_weight is not None and cls._ROUTER_ATTR is not None:
            router = nn.Module()
            router.weight = nn.Parameter(router_weight)
            router.top_k = top_k
            router.norm_topk_prob = True
            setattr(self, cls._ROUTER_ATTR, router)
        for name, tensor in expert_tensors.items():
            # a BlockFp8Weight (quantised serving weights) is held as it is
            setattr(self, name, nn.Parameter(tensor) if isinstance(tensor, torch.Tensor) else tensor)
        self._fused_glu_mul = GluCombine.silu()
        init_expert_lora(self, ep_config.expert_lora)
        return self


class EPSharedExpertsMoELayerBase(EPMoELayerBase):
    """``forward`` routes the flattened tokens, then adds the shared expert, which reads the layer input."""

    _ROUTER_MODE: int = SOFTMAX_ALL

    def forward(self, hidden_states: torch.Tensor, **kwargs) -> torch.Tensor:
        orig_shape = hidden_states.shape
        flat = hidden_states.reshape(-1, orig_shape[-1])
        topk_indices, topk_weights = self._route_hidden_states(flat, **kwargs)
        shared = getattr(self, self._shared_expert_attr, None)
        shared_fn = (lambda: self._shared_expert_output(hidden_states)) if shared is not None else None
        parts_fn = (lambda: self._shared_expert_parts(hidden_states)) if shared is not None else None
        return self._dispatch_compute_combine_shared(
            flat, topk_indices.long(), topk_weights.float(), hidden_states.dtype, orig_shape, shared_fn, parts_fn
        )

    def _normalizes_topk(self) -> bool:
        return True

    def _route_hidden_states(self, flat: torch.Tensor, **kwargs) -> tuple[torch.Tensor, torch.Tensor]:
        """Logits projection, then the fused softmax / top-k / renormalise / cast kernel."""
        logits = self._linear_router_logits(flat)
        return fused_topk_gate(logits, self.top_k, mode=self._ROUTER_MODE, normalize=self._normalizes_topk(),
                               eps=self._TOPK_WEIGHT_NORM_EPS)

    def _shared_expert_output(self, hidden_states: torch.Tensor) -> torch.Tensor:
        """Dense GLU MLP ``down(act(gate(x)) * up(x))`` through the same GEMM and GLU kernels."""
        rows, scale = self._shared_expert_parts(hidden_states)
        if scale is None:
            return rows.view(hidden_states.shape)
        if rows.is_cuda and rows.dim() == 2 and rows.dtype == scale.dtype and rows.shape[0] > 0:
            return _ScaleRows.apply(rows, scale.reshape(-1)).view(hidden_states.shape)
        return rows.view(hidden_states.shape) * scale.view(*hidden_states.shape[:-1], 1)

    def _shared_expert_parts(self, hidden_states: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor | None]:
        """The shared expert's output as ``(rows [T, H], scale [T] or None)``: ``rows`` the MLP's output, ``scale`` a
        per-token factor on it (none here; Qwen3.5's sigmoid gate)."""
        shared = getattr(self, self._shared_expert_attr)
        x = hidden_states.reshape(-1, hidden_states.shape[-1])
        dtype = x.dtype
        gate_w, up_w = shared.gate_proj.weight.to(dtype), shared.up_proj.weight.to(dtype)
        packable = getattr(self._fused_glu_mul, "packed", None)
        if getattr(self, "fuse_shared_gate_up", True) and packable is not None and gate_w.shape == up_w.shape:
            # gate and up as one product over the two weights side by side (HF keeps them apart): one launch per
            # direction, the input gradient summed over both in fp32 instead of two rounded products and an addition,
            # and the SwiGLU in its packed form.  The same dot products: the forward's bits do not change.
            gate_up = dense_mm(x, torch.cat((gate_w, up_w), dim=0))
            return dense_mm(packable(gate_up), shared.down_proj.weight.to(dtype)), None
        gate = dense_mm(x, gate_w)
        up = dense_mm(x, up_w)
        return dense_mm(self._fused_glu_mul(gate, up), shared.down_proj.weight.to(dtype)), None
