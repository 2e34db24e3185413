"""Oracle (test infrastructure): grouped GEMM as a per-expert loop on the CPU.

The reference's arithmetic for this op lives in torch's ``aten::_grouped_mm`` (torch 2.11.0+cu130, third party, not
in the reference tree); its call sites are ``halo/kernels/grouped_mm.py:25-26, 39``.  The published contract is the
per-group matrix product: ``out[s:e] = A[s:e] @ B[g]`` with ``offs`` the int32 inclusive group ends, and the two
gradients ``dA[s:e] = dO[s:e] @ B[g]^T`` and ``dB[g] = A[s:e]^T @ dO[s:e]`` (an empty group gives exact zeros).  The
reference's own tests check it against exactly this loop (``tests/gpu/kernels/test_expert_gemm.py:19-25``,
``tests/gpu/kernels/test_grouped_mm_empty_groups.py:28-35``).  Products accumulate in ``acc_dtype`` (fp32 by default,
fp64 for an exact reference) and are rounded once to ``A``'s dtype.
"""

from __future__ import annotations

import torch


def _bounds(offs) -> list[tuple[int, int]]:
    ends = [int(v) for v in offs]
    return list(zip([0] + ends[:-1], ends))


def grouped_mm(a: torch.Tensor, b: torch.Tensor, offs, acc_dtype=torch.float32) -> torch.Tensor:
    out = torch.zeros(a.shape[0], b.shape[-1], dtype=acc_dtype)
    for g, (s, e) in enumerate(_bounds(offs)):
        if e > s:
            out[s:e] = a[s:e].to(acc_dtype) @ b[g].to(acc_dtype)
    return out.to(a.dtype)


def grouped_mm_dgrad(grad_out: torch.Tensor, b: torch.Tensor, offs, acc_dtype=torch.float32) -> torch.Tensor:
    out = torch.zeros(grad_out.shape[0], b.shape[1], dtype=acc_dtype)
    for g, (s, e) in enumerate(_bounds(offs)):
        if e > s:
            out[s:e] = grad_out[s:e].to(acc_dtype) @ b[g].to(acc_dtype).t()
    return out.to(grad_out.dtype)


def grouped_mm_wgrad(a: torch.Tensor, grad_out: torch.Tensor, offs, acc_dtype=torch.float32) -> torch.Tensor:
    groups = len(offs)
    out = torch.zeros(groups, a.shape[1], grad_out.shape[1], dtype=acc_dtype)
    for g, (s, e) in enumerate(_bounds(offs)):
        if e > s:
            out[g] = a[s:e].to(acc_dtype).t() @ grad_out[s:e].to(acc_dtype)
    return out.to(a.dtype)
