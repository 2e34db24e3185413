"""Grouped GEMM for MoE expert FFNs, by format: bf16/fp32 (the training path), the MXFP8 and MXFP4
quantisation-aware formats (both operands block-scaled along the contraction, straight-through backward), or block-fp8
weights (the quantised-weight serving configuration, forward only).

Mirrors the dispatch seam of the reference's ``halo/kernels/expert_gemm.py:14-38``.  Of its ``quant_format`` values
``"mxfp8"`` and ``"mxfp4"`` run on the scaled matrix instruction (e4m3 / e2m1 operands with an e8m0 exponent per 32
values); ``"nvfp4"`` (e4m3 scales, which the instruction cannot take) is the bf16 product of the two round-tripped
operands, the reference's own formulation.
"""

from __future__ import annotations

import torch

from halo_amd import _lib
from halo_amd.kernels.grouped_mm import GatheredRows, _forward, _offs_arg, _rows, grouped_mm, grouped_mm_grads
from halo_amd.kernels.lowp.spec import require_implemented


# rows per expert (on average) from which the dequantised-copy route is taken
_CACHED_MIN_ROWS = 64


class BlockFp8Weight:
    """Expert weights ``[G, K, N]`` as float8_e4m3fn with one fp32 power-of-two scale per 128x128 block
    (``halo_amd.kernels.lowp.block_fp8.quantize_block_fp8`` of the matmul-convention weight)."""

    def __init__(self, q: torch.Tensor, scale_inv: torch.Tensor):
        if q.dim() != 3 or scale_inv.dim() != 3:
            raise ValueError("expected q [G, K, N] and scale_inv [G, ceil(K/128), ceil(N/128)]")
        g, k, n = q.shape
        if tuple(scale_inv.shape) != (g, -(-k // 128), -(-n // 128)):
            raise ValueError(f"scale grid {tuple(scale_inv.shape)} does not match weight {tuple(q.shape)}")
        self.q = q.contiguous()
        self.scale_inv = scale_inv.float().contiguous()
        self._bf16 = None
        self._panels = None

    @property
    def shape(self):
        return self.q.shape

    def dequantized(self) -> torch.Tensor:
        """The weights as bf16 ``[G, K, N]`` (``q * scale`` per block, exact: the scales are powers of two), made once
        and kept: twice the fp8 bytes again in device memory, for the bf16 kernel's speed on compute-bound batches."""
        if self._bf16 is None:
            from halo_amd.kernels.lowp.block_fp8 import dequantize_block_fp8

            self._bf16 = dequantize_block_fp8(self.q, self.scale_inv)
        return self._bf16


    def panels(self) -> torch.Tensor:
        """The e4m3 bytes as ``[G, K / 64, N, 64]``: the contraction contiguous within a panel of 64 values and a
        tile's columns of one panel in one run, which is how the fp8 MFMA kernel loads them.  Made once and kept: the
        fp8 bytes once more in device memory."""
        if self._panels is None:
            g, k, n = self.q.shape
            self._panels = self.q.view(torch.uint8).view(g, k // 64, 64, n).permute(0, 1, 3, 2).contiguous()
        return self._panels


def expert_gemm(
    mat_a: torch.Tensor,
    mat_b,
    *,
    offs: torch.Tensor | None = None,
    quant_format=None,
    weight_cacheable: bool = True,
    fp8_activations: bool = False,
    bias: torch.Tensor | None = None,
    eids: torch.Tensor | None = None,
) -> torch.Tensor:
    """``[total_tokens, K]`` activations stacked by expert times ``[num_experts, K, N]`` weights.  ``mat_b`` may be a
    :class:`BlockFp8Weight` (or ``quant_format == "block_fp8"`` with ``mat_b = (q, scale_inv)``): bf16 activations
    against fp8 weights dequantised on their way into the MFMA tiles, forward only.  ``fp8_activations=True``
    quantises the activations too (per row and 128 values, power-of-two scales) and multiplies on the e4m3 MFMA:
    twice the bf16 rate and half the bytes, at e4m3 precision on both sides instead of one.  ``bias [G, N]`` with
    ``eids`` (the sorted expert id of every row), for the MX formats: ``+ bias[eids]`` joins the product in the
    kernel's epilogue, rounded as the two tensor operations round (reference ``families/gpt_oss.py:153-159``)."""
    if bias is not None and (quant_format not in ("mxfp8", "mxfp4") or eids is None):
        raise ValueError("bias is taken with quant_format 'mxfp8' or 'mxfp4' and needs eids")
    if isinstance(mat_b, BlockFp8Weight) or quant_format == "block_fp8":
        weight = mat_b if isinstance(mat_b, BlockFp8Weight) else BlockFp8Weight(*mat_b)
        if fp8_activations:
            return _fp8_mfma_forward(mat_a, weight, offs)
        # Two routes with bit-identical results (the dequantisation is exact).  The kernel that reads the fp8 bytes
        # moves half the weight traffic, which is what counts while a batch is small; once an expert sees enough rows
        # to be compute-bound the bf16 kernel over a dequantised copy kept with the weight is faster (configuration 5:
        # 1.1 PFLOP/s against 0.65).  ``weight_cacheable=False`` (weights that change under the caller) always takes
        # the first.
        if weight_cacheable and isinstance(mat_b, BlockFp8Weight) and mat_a.shape[0] >= _CACHED_MIN_ROWS * weight.shape[0]:
            if mat_a.requires_grad and torch.is_grad_enabled():
                raise RuntimeError("the block-fp8 expert GEMM is forward only")
            with torch.no_grad():
                return grouped_mm(mat_a, weight.dequantized(), offs=offs)
        return _fp8w_forward(mat_a, weight, offs)
    if quant_format is not None:
        require_implemented(quant_format)
        gathered = isinstance(mat_a, GatheredRows)  # the row quantiser fetches the rows itself
        source, row_index, inv_map = (mat_a.tokens, mat_a.row_index, mat_a.inv_map) if gathered else (mat_a, None, None)
        if quant_format == "nvfp4":
            # one scale for the whole activation tensor: the rows are gathered first, then round-tripped as one tensor
            return _RoundTripExpertGemm.apply(mat_a.materialize() if gathered else mat_a, mat_b, offs, weight_cacheable,
                                              quant_format)
        node = _Mxfp4ExpertGemm if quant_format == "mxfp4" else _MxFp8ExpertGemm
        return node.apply(source, mat_b, offs, weight_cacheable, row_index, inv_map, bias, eids)
    return grouped_mm(mat_a, mat_b, offs=offs)


def mxfp8_mfma_usable(mat_a_dtype: torch.dtype, mat_b_dtype: torch.dtype, k: int, n: int, rows: int = 0) -> bool:
    """Whether the scaled e4m3 MFMA kernel takes the product: bf16 operands, whole panels of 64 values along K,
    16-byte output rows, and ``rows`` activation rows whose operands the kernel can address (activations and output of
    any size; one expert's weights and the rows' exponent bytes below 2 GiB: the library's own check,
    ``hmoe_grouped_gemm_mx_fits``).  Anything else multiplies the two
    round-tripped operands on the bf16 / fp32 kernel, which is the reference's own formulation."""
    return (mat_a_dtype == torch.bfloat16 and mat_b_dtype == torch.bfloat16 and k > 0 and k % 64 == 0
            and n % 8 == 0 and bool(_lib.load().hmoe_grouped_gemm_mx_fits(rows, rows, k, n, n, 64)))


def _plus_bias(out: torch.Tensor, bias, eids) -> torch.Tensor:
    """``out + bias[eids]`` as two tensor operations, for the routes whose kernel has no bias epilogue."""
    return out if bias is None else out + bias.to(out.dtype).index_select(0, eids.long())


def _bias_grad(ctx, grad_output: torch.Tensor, position: int):
    """The bias gradient of an MX node: per expert, the column sums of the rows' gradient."""
    if ctx.eids is None or not ctx.needs_input_grad[position]:
        return None
    from halo_amd.kernels.moe_permute import expert_bias_grad

    return expert_bias_grad(grad_output, ctx.eids, ctx.groups).to(ctx.bias_dtype)


class _SharedRows:
    """The last activation tensor quantised (forward) and the last e4m3 rows dequantised (backward), each with its
    result: projections that read the same rows (gate and up stored apart) quantise them once and rebuild them once.
    An entry is tied to the tensor object by a weak reference, to its version counter, its storage address and its
    shape, and dies with the tensor; the slot is read and written under a lock (autograd's backward thread shares it
    with the forward thread).  What the key cannot see is a write that leaves the version counter alone (``.data``
    assignments into the same storage, a kernel writing through a raw pointer): such writes between two projections
    of the same rows are not supported."""

    def __init__(self):
        import threading

        self._ref, self._key, self._value, self._hold = None, None, None, None
        self._lock = threading.Lock()

    @staticmethod
    def _full_key(tensor: torch.Tensor, key: tuple) -> tuple:
        return (key, tensor.data_ptr(), tuple(tensor.shape), tuple(tensor.stride()))

    def get(self, tensor: torch.Tensor, key: tuple):
        with self._lock:
            if self._ref is not None and self._ref() is tensor and self._key == self._full_key(tensor, key):
                return self._value
        return None

    def put(self, tensor: torch.Tensor, key: tuple, value, hold=None) -> None:
        """``hold``: an object the key names by ``id`` (the row index); kept alive with the entry, so that the id
        cannot pass to another object while the entry can still be hit."""
        import weakref

        def drop(ref, self=self):
            with self._lock:
                if self._ref is ref:
                    self._ref, self._key, self._value, self._hold = None, None, None, None

        with self._lock:
            self._ref, self._key, self._value, self._hold = (weakref.ref(tensor, drop), self._full_key(tensor, key),
                                                             value, hold)


_quantised_rows = _SharedRows()
_dequantised_rows = _SharedRows()


class _MxFp8ExpertGemm(torch.autograd.Function):
    """``grouped_mm(fake_quant(mat_a, "mxfp8", axis=-1), cached_fake_quant(mat_b, "mxfp8", axis=1), offs)`` of the
    reference (``expert_gemm.py:33-38``) as one node.  Forward: the rows are quantised to e4m3 with an e8m0 scale per
    32 values (one launch, which also fetches them through ``row_index`` when the permuted copy was never made), the
    weights once per optimizer step, and the product runs on the scaled e4m3 matrix instruction: the same products of
    dequantised values the reference's bf16 GEMM sums, accumulated in fp32, at twice the bf16 rate and half the
    operand bytes.  Backward is the fake-quant's straight-through estimator around ``grouped_mm``'s own gradients
    (``quantization.py:350-360``, ``grouped_mm.py:16-27``): ``grad_a = dO @ fq(B)^T``, ``grad_b = fq(A)^T @ dO`` with
    the round-tripped operands in bf16, ``fq(A)`` rebuilt from the saved e4m3 rows (half the bytes of a bf16 copy)."""

    @staticmethod
    def forward(ctx, mat_a, mat_b, offs, weight_cacheable, row_index, inv_map, bias=None, eids=None):
        from halo_amd.kernels.lowp.quantization import (MxRows, dequantize_rows_mxfp8, expert_weight_operand,
                                                        quantize_rows_mxfp8)

        device = _lib.require_device(mat_a, mat_b, offs, row_index, inv_map, bias, eids)
        ctx.eids, ctx.groups, ctx.bias_dtype = eids, mat_b.shape[0], None if bias is None else bias.dtype
        if mat_a.dim() != 2 or mat_b.dim() != 3 or mat_a.shape[1] != mat_b.shape[1]:
            raise ValueError(f"expected [R, K] x [G, K, N], got {tuple(mat_a.shape)} x {tuple(mat_b.shape)}")
        groups, k, n = mat_b.shape
        offs32 = _offs_arg(offs, groups)
        weight = expert_weight_operand(mat_b, weight_cacheable)
        key = (mat_a._version, None if row_index is None else (id(row_index), row_index._version))
        rows_q = _quantised_rows.get(mat_a, key)
        if rows_q is None:
            rows_q = quantize_rows_mxfp8(mat_a, row_index)
            _quantised_rows.put(mat_a, key, rows_q, hold=row_index)
        rows = rows_q.rows
        ctx.k, ctx.dtype, ctx.gathered = k, mat_a.dtype, row_index is not None
        # the e4m3 rows ride on the node itself: projections that share them must see one object, and they are no
        # input or output of this node
        ctx.rows_q = rows_q
        ctx.save_for_backward(weight.dequant, offs32, inv_map)
        if not mxfp8_mfma_usable(mat_a.dtype, mat_b.dtype, k, n, rows):
            return _plus_bias(_forward(dequantize_rows_mxfp8(rows_q).to(mat_a.dtype), weight.dequant.to(mat_a.dtype),
                                       offs32), bias, eids)
        out = torch.empty((rows, n), dtype=torch.bfloat16, device=device)
        if rows and n:
            with _lib.on_device(device):
                if bias is None:
                    _lib.call("hmoe_grouped_gemm_fwd_mxfp8", _lib.ptr(rows_q.q), _lib.ptr(rows_q.scales), rows,
                              _lib.ptr(weight.q), _lib.ptr(weight.scales), _lib.ptr(offs32), rows, groups, k, n,
                              _lib.ptr(out), out.stride(0), _lib.stream_ptr(device))
                else:
                    bias16 = bias.to(torch.bfloat16).contiguous()
                    _lib.call("hmoe_grouped_gemm_fwd_mxfp8_bias", _lib.ptr(rows_q.q), _lib.ptr(rows_q.scales), rows,
                              _lib.ptr(weight.q), _lib.ptr(weight.scales), _lib.ptr(bias16), _lib.ptr(offs32), rows,
                              groups, k, n, _lib.ptr(out), out.stride(0), _lib.stream_ptr(device))
        return out

    @staticmethod
    def backward(ctx, grad_output):
        from halo_amd.kernels.lowp.quantization import MxRows, dequantize_rows_mxfp8
        from halo_amd.kernels.moe_permute import gather_reduce_rows

        w_dq, offs32, inv_map = ctx.saved_tensors
        q, scales = ctx.rows_q.q, ctx.rows_q.scales
        grad_a = grad_b = None
        if ctx.needs_input_grad[0] or ctx.needs_input_grad[1]:
            if ctx.needs_input_grad[1]:
                a_dq = _dequantised_rows.get(q, (q._version, ctx.dtype))
                if a_dq is None:
                    a_dq = dequantize_rows_mxfp8(MxRows(q, scales, ctx.k)).to(ctx.dtype)
                    _dequantised_rows.put(q, (q._version, ctx.dtype), a_dq)
            else:  # the input gradient reads the rows' shape and dtype only
                a_dq = grad_output.new_empty((1, ctx.k)).expand(q.shape[1], ctx.k).to(ctx.dtype)
            grad_a, grad_b = grouped_mm_grads(a_dq, w_dq.to(ctx.dtype), grad_output.to(ctx.dtype), offs32,
                                              ctx.needs_input_grad[0], ctx.needs_input_grad[1])
            if ctx.gathered and grad_a is not None:
                grad_a = gather_reduce_rows(grad_a, inv_map)
        return grad_a, grad_b, None, None, None, None, _bias_grad(ctx, grad_output, 6), None


class _RoundTripExpertGemm(torch.autograd.Function):
    """``grouped_mm(fake_quant(mat_a, fmt, axis=-1), cached_fake_quant(mat_b, fmt, axis=1), offs)`` of the reference
    (``expert_gemm.py:33-38``) as one node, for a format the matrix instruction has no operand type for (NVFP4): both
    operands through their round trip (the weights' kept per optimizer step), the product and, straight through
    (``quantization.py:350-360``), the gradients on the bf16 / fp32 grouped kernels."""

    @staticmethod
    def forward(ctx, mat_a, mat_b, offs, weight_cacheable, fmt):
        from halo_amd.kernels.lowp.quantization import _round_trip, expert_weight_round_trip

        _lib.require_device(mat_a, mat_b, offs)
        if mat_a.dim() != 2 or mat_b.dim() != 3 or mat_a.shape[1] != mat_b.shape[1]:
            raise ValueError(f"expected [R, K] x [G, K, N], got {tuple(mat_a.shape)} x {tuple(mat_b.shape)}")
        offs32 = _offs_arg(offs, mat_b.shape[0])
        w_rt = expert_weight_round_trip(mat_b, fmt, weight_cacheable).to(mat_a.dtype)
        key = (mat_a._version, fmt)
        a_rt = _round_tripped_rows.get(mat_a, key)
        if a_rt is None:
            a_rt = _round_trip(mat_a.detach(), fmt, -1).to(mat_a.dtype)
            _round_tripped_rows.put(mat_a, key, a_rt)
        ctx.save_for_backward(a_rt, w_rt, offs32)
        return _forward(a_rt, w_rt, offs32)

    @staticmethod
    def backward(ctx, grad_output):
        a_rt, w_rt, offs32 = ctx.saved_tensors
        grad_a = grad_b = None
        if ctx.needs_input_grad[0] or ctx.needs_input_grad[1]:
            grad_a, grad_b = grouped_mm_grads(a_rt, w_rt, grad_output.to(a_rt.dtype), offs32, ctx.needs_input_grad[0],
                                              ctx.needs_input_grad[1])
        return grad_a, grad_b, None, None, None


def mxfp4_mfma_usable(mat_a_dtype: torch.dtype, mat_b_dtype: torch.dtype, k: int, n: int, rows: int = 0) -> bool:
    """Whether the scaled matrix instruction takes the MXFP4 product: bf16 operands, 16-byte output rows, and ``rows``
    activation rows whose quantised panels and output the kernel can address (``hmoe_grouped_gemm_mx_fits``).  Anything
    else multiplies the two round-tripped operands on the bf16 / fp32 kernel, the reference's own formulation."""
    return (mat_a_dtype == torch.bfloat16 and mat_b_dtype == torch.bfloat16 and k > 0 and k % 32 == 0 and n % 8 == 0
            and bool(_lib.load().hmoe_grouped_gemm_mx_fits(rows, rows, k, n, n, 128)))


_round_tripped_rows = _SharedRows()
_quantised_rows4 = _SharedRows()
_dequantised_rows4 = _SharedRows()


class _Mxfp4ExpertGemm(torch.autograd.Function):
    """``grouped_mm(fake_quant(mat_a, "mxfp4", axis=-1), cached_fake_quant(mat_b, "mxfp4", axis=1), offs)`` of the
    reference (``expert_gemm.py:33-38``) as one node.  Forward: the rows are quantised to e2m1 with an e8m0 scale per 32
    values (one launch, which also fetches them through ``row_index`` when the permuted copy was never made), the
    weights once per optimizer step, and the product runs on the scaled matrix instruction with e2m1 operands: the
    same products of dequantised values the reference's bf16 GEMM sums, accumulated in fp32.  fp32 operands go through
    the round trip in one launch each and the fp32 grouped GEMM.  Backward is the straight-through estimator around ``grouped_mm``'s own gradients
    (``quantization.py:350-360``, ``grouped_mm.py:16-27``) with the round-tripped operands, the rows' rebuilt from the
    saved e2m1 codes (a quarter of the bytes of a bf16 copy)."""

    @staticmethod
    def forward(ctx, mat_a, mat_b, offs, weight_cacheable, row_index, inv_map, bias=None, eids=None):
        from halo_amd.kernels.lowp.quantization import (expert_weight_operand, expert_weight_round_trip, mxfp4_rows,
                                                        quantize_rows_mxfp4)

        device = _lib.require_device(mat_a, mat_b, offs, row_index, inv_map, bias, eids)
        ctx.eids, ctx.groups, ctx.bias_dtype = eids, mat_b.shape[0], None if bias is None else bias.dtype
        if mat_a.dim() != 2 or mat_b.dim() != 3 or mat_a.shape[1] != mat_b.shape[1]:
            raise ValueError(f"expected [R, K] x [G, K, N], got {tuple(mat_a.shape)} x {tuple(mat_b.shape)}")
        groups, k, n = mat_b.shape
        offs32 = _offs_arg(offs, groups)
        key = (mat_a._version, None if row_index is None else (id(row_index), row_index._version))
        ctx.gathered, ctx.k, ctx.dtype = row_index is not None, k, mat_a.dtype
        ctx.native = mxfp4_mfma_usable(mat_a.dtype, mat_b.dtype, k, n,
                                       mat_a.shape[0] if row_index is None else row_index.shape[0])
        if not ctx.native:
            w_rt = expert_weight_round_trip(mat_b, "mxfp4", weight_cacheable).to(mat_a.dtype)
            a_rt = _round_tripped_rows.get(mat_a, key)
            if a_rt is None:
                a_rt = mxfp4_rows(mat_a, row_index, codes=False, round_trip=True)[2].to(mat_a.dtype)
                _round_tripped_rows.put(mat_a, key, a_rt, hold=row_index)
            ctx.save_for_backward(a_rt, w_rt, offs32, inv_map)
            return _plus_bias(_forward(a_rt, w_rt, offs32), bias, eids)
        weight = expert_weight_operand(mat_b, weight_cacheable, "mxfp4")
        rows_q = _quantised_rows4.get(mat_a, key)
        if rows_q is None:
            rows_q = quantize_rows_mxfp4(mat_a, row_index)
            _quantised_rows4.put(mat_a, key, rows_q, hold=row_index)
        rows = rows_q.rows
        ctx.rows_q = rows_q  # projections that share the rows must see one object
        ctx.save_for_backward(weight.dequant, offs32, inv_map)
        out = torch.empty((rows, n), dtype=torch.bfloat16, device=device)
        if rows and n:
            with _lib.on_device(device):
                if bias is None:
                    _lib.call("hmoe_grouped_gemm_fwd_mxfp4", _lib.ptr(rows_q.q), _lib.ptr(rows_q.scales), rows,
                              _lib.ptr(weight.q), _lib.ptr(weight.scales), _lib.ptr(offs32), rows, groups, k, n,
                              _lib.ptr(out), out.stride(0), _lib.stream_ptr(device))
                else:
                    bias16 = bias.to(torch.bfloat16).contiguous()
                    _lib.call("hmoe_grouped_gemm_fwd_mxfp4_bias", _lib.ptr(rows_q.q), _lib.ptr(rows_q.scales), rows,
                              _lib.ptr(weight.q), _lib.ptr(weight.scales), _lib.ptr(bias16), _lib.ptr(offs32), rows,
                              groups, k, n, _lib.ptr(out), out.stride(0), _lib.stream_ptr(device))
        return out

    @staticmethod
    def backward(ctx, grad_output):
        from halo_amd.kernels.lowp.quantization import dequantize_rows_mxfp4
        from halo_amd.kernels.moe_permute import gather_reduce_rows

        grad_a = grad_b = None
        grad_bias = _bias_grad(ctx, grad_output, 6)
        if not (ctx.needs_input_grad[0] or ctx.needs_input_grad[1]):
            return None, None, None, None, None, None, grad_bias, None
        if ctx.native:
            w_rt, offs32, inv_map = ctx.saved_tensors
            q = ctx.rows_q.q
            if ctx.needs_input_grad[1]:
                a_rt = _dequantised_rows4.get(q, (q._version,))
                if a_rt is None:
                    a_rt = dequantize_rows_mxfp4(ctx.rows_q)
                    _dequantised_rows4.put(q, (q._version,), a_rt)
            else:  # the input gradient reads the rows' shape and dtype only
                a_rt = grad_output.new_empty((1, ctx.k)).expand(q.shape[1], ctx.k).to(torch.bfloat16)
        else:
            a_rt, w_rt, offs32, inv_map = ctx.saved_tensors
        grad_a, grad_b = grouped_mm_grads(a_rt, w_rt, grad_output.to(a_rt.dtype), offs32,
                                          ctx.needs_input_grad[0], ctx.needs_input_grad[1])
        if ctx.gathered and grad_a is not None:
            grad_a = gather_reduce_rows(grad_a, inv_map)
        return grad_a, grad_b, None, None, None, None, grad_bias, None


def _fp8w_forward(mat_a: torch.Tensor, weight: BlockFp8Weight, offs: torch.Tensor | None) -> torch.Tensor:
    device = _lib.require_device(mat_a, weight.q, weight.scale_inv, offs)
    if mat_a.dtype != torch.bfloat16:
        raise TypeError(f"block-fp8 expert GEMM takes bf16 activations, got {mat_a.dtype}")
    if mat_a.requires_grad and torch.is_grad_enabled():
        raise RuntimeError("the block-fp8 expert GEMM is forward only")
    groups, k, n = weight.shape
    rows = mat_a.shape[0]
    out = torch.empty((rows, n), dtype=torch.bfloat16, device=device)
    if rows == 0 or n == 0:
        return out
    mat_a = _rows(mat_a)
    offs32 = _offs_arg(offs, groups)
    q = weight.q.view(torch.uint8)
    with _lib.on_device(device):
        _lib.call("hmoe_grouped_gemm_fwd_fp8w", _lib.ptr(mat_a), mat_a.stride(0), _lib.ptr(q),
                  _lib.ptr(weight.scale_inv), _lib.ptr(offs32), rows, groups, k, n, _lib.ptr(out), out.stride(0),
                  _lib.stream_ptr(device))
    return out


def fp8_mfma_usable(k: int, n: int) -> bool:
    """Whether the e4m3 MFMA kernel takes a ``[*, K] x [G, K, N]`` product: whole 128-value scale blocks along K,
    16-byte output rows."""
    return k > 0 and k % 128 == 0 and n % 8 == 0


def _fp8_mfma_forward(mat_a: torch.Tensor, weight: BlockFp8Weight, offs: torch.Tensor | None) -> torch.Tensor:
    """Activations to e4m3 (one launch, which also fetches the rows when ``mat_a`` is a :class:`GatheredRows`: the
    permuted bf16 copy is never written; none at all when ``mat_a`` already is a ``QuantizedRows``), then the grouped GEMM on the scaled e4m3 MFMA against the weight's bytes in
    panels and its fp32 block scales."""
    from halo_amd.kernels.lowp.block_fp8 import QuantizedRows, quantize_rows_fp8

    gathered = isinstance(mat_a, GatheredRows)
    quantized = isinstance(mat_a, QuantizedRows)
    source = mat_a.tokens if gathered else (mat_a.q if quantized else mat_a)
    device = _lib.require_device(source, weight.q, weight.scale_inv, offs)
    if quantized:
        source = mat_a  # its dtype and gradient flag stand for the bf16 rows it was made from
    if source.dtype != torch.bfloat16:
        raise TypeError(f"block-fp8 expert GEMM takes bf16 activations, got {source.dtype}")
    if source.requires_grad and torch.is_grad_enabled():
        raise RuntimeError("the block-fp8 expert GEMM is forward only")
    groups, k, n = weight.shape
    if len(mat_a.shape) != 2 or mat_a.shape[1] != k:
        raise ValueError(f"expected [R, {k}] activations, got {tuple(mat_a.shape)}")
    if not fp8_mfma_usable(k, n):
        raise ValueError(f"the fp8 MFMA product needs K % 128 == 0 and N % 8 == 0, got K = {k}, N = {n}")
    rows = mat_a.shape[0]
    out = torch.empty((rows, n), dtype=torch.bfloat16, device=device)
    if rows == 0 or n == 0:
        return out
    offs32 = _offs_arg(offs, groups)
    if quantized:
        a_q, a_scale = mat_a.q, mat_a.scale_exponents
    else:
        a_q, a_scale = quantize_rows_fp8(source, mat_a.row_index if gathered else None)
    w_panels = weight.panels()
    with _lib.on_device(device):
        _lib.call("hmoe_grouped_gemm_fwd_fp8", _lib.ptr(a_q), _lib.ptr(a_scale), rows, _lib.ptr(w_panels),
                  _lib.ptr(weight.scale_inv), _lib.ptr(offs32), rows, groups, k, n, _lib.ptr(out), out.stride(0),
                  _lib.stream_ptr(device))
    return out
