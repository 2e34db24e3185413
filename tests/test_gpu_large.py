"""Operands past 2**31 elements or 2 GiB: the sizes at which a 32-bit element index or byte offset wraps.  The
reference addresses rows in 64 bits and tests its GLU at 746000 x 2880 (``tests/gpu/kernels/test_fused_glu.py:286-291``);
here one case per kernel family, each checked on sampled rows (or whole small outputs) against fp32 arithmetic on the
device.  Inputs are generated on the device; every tensor is dropped before the next case."""

import pytest
import torch

pytestmark = pytest.mark.gpu


def _close(got, want, tol=2e-2):
    err = float((got.float() - want).abs().max() / want.abs().max())
    cos = float(torch.nn.functional.cosine_similarity(got.float().flatten(), want.flatten(), dim=0))
    assert err <= tol and cos >= 0.9999, (err, cos)


def _sample(n, count, generator, device):
    head_tail = torch.tensor([0, 1, n - 2, n - 1], device=device)
    return torch.cat([head_tail, torch.randint(0, n, (count,), generator=generator, device=device)])


def test_glu_past_two_to_the_31_elements(device):
    from halo_amd.kernels.fused_glu import GluCombine

    rows, width = 746_000, 2880
    assert rows * width > 2**31
    g = torch.Generator(device=device).manual_seed(1)
    gate_up = torch.randn(rows, 2 * width, generator=g, device=device, dtype=torch.bfloat16)
    weight = torch.rand(rows, generator=g, device=device).bfloat16()
    pick = _sample(rows, 60, g, device)
    want = torch.nn.functional.silu(gate_up[pick, :width].float()) * gate_up[pick, width:].float()
    with torch.no_grad():
        out = GluCombine.silu().packed(gate_up)
        _close(out[pick], want)
        del out
        out = GluCombine.silu().packed_weighted(gate_up, weight)
        _close(out[pick], want * weight[pick].float().unsqueeze(1))
    # backward at the same size: the packed gradient is as large as the input
    dout = torch.randn(rows, width, generator=g, device=device, dtype=torch.bfloat16)
    leaf = gate_up.requires_grad_(True)
    GluCombine.silu().packed(leaf).backward(dout)
    gate, up = gate_up.detach()[pick, :width].float(), gate_up.detach()[pick, width:].float()
    sig = torch.sigmoid(gate)
    _close(leaf.grad[pick, :width], dout[pick].float() * up * sig * (1 + gate * (1 - sig)))
    _close(leaf.grad[pick, width:], dout[pick].float() * gate * sig)


def test_permute_and_combine_past_two_to_the_31_elements(device):
    from halo_amd.kernels.moe_permute import _gather_rows, gather_reduce_rows

    rows, hidden, tokens, top_k = 600_000, 4096, 150_000, 4
    assert rows * hidden > 2**31
    g = torch.Generator(device=device).manual_seed(2)
    src = torch.randn(rows, hidden, generator=g, device=device, dtype=torch.bfloat16)
    # rows from the far end of the source land at the near end of the output and the other way round
    index = torch.arange(rows - 1, -1, -1, device=device)
    out = _gather_rows(src, index)
    pick = _sample(rows, 60, g, device)
    assert torch.equal(out[pick], src[index[pick]])
    del out
    inv_map = index.view(tokens, top_k).contiguous()  # token t sums sorted rows R-1-4t .. R-4-4t
    weight = torch.rand(rows, generator=g, device=device).bfloat16()
    out = gather_reduce_rows(src, inv_map, weight)
    tok = _sample(tokens, 60, g, device)
    want = (src[inv_map[tok]].float() * weight[inv_map[tok]].float().unsqueeze(-1)).sum(dim=1)
    _close(out[tok], want)


def test_grouped_gemm_with_operands_past_two_gib(device):
    """Activations of 2.3 GB with one group holding 97 % of the rows: forward rows, the input gradient (an output of
    2.3 GB) and the weight gradient (a contraction that walks past 2 GiB inside one group), plain and gathered."""
    from halo_amd.kernels.grouped_mm import grouped_mm, grouped_mm_combine, grouped_mm_grads
    from halo_amd.kernels.moe_permute import build_inv_map

    rows, k, n = 400_000, 2880, 512
    assert rows * k * 2 > 2**31
    counts = (5_000, 390_000, 0, 5_000)
    offs = torch.tensor(counts, device=device).cumsum(0).int()
    g = torch.Generator(device=device).manual_seed(3)
    a = torch.randn(rows, k, generator=g, device=device, dtype=torch.bfloat16)
    w = (torch.randn(len(counts), k, n, generator=g, device=device) * 0.02).bfloat16()
    dout = torch.randn(rows, n, generator=g, device=device, dtype=torch.bfloat16)
    group_of = torch.repeat_interleave(torch.arange(len(counts), device=device), torch.tensor(counts, device=device))
    pick = torch.cat([_sample(rows, 80, g, device), torch.tensor([4_999, 5_000, 394_999, 395_000], device=device)])
    with torch.no_grad():
        out = grouped_mm(a, w, offs=offs)
        want = torch.stack([a[r].float() @ w[group_of[r]].float() for r in pick.tolist()])
        _close(out[pick], want)
        del out
        grad_a, grad_w = grouped_mm_grads(a, w, dout, offs, True, True)
        want = torch.stack([dout[r].float() @ w[group_of[r]].float().t() for r in pick.tolist()])
        _close(grad_a[pick], want)
        del grad_a
        ends = [0] + offs.tolist()
        for e, (lo, hi) in enumerate(zip(ends[:-1], ends[1:])):
            if hi > lo:
                _close(grad_w[e], a[lo:hi].float().t() @ dout[lo:hi].float())
            else:
                assert not grad_w[e].any()
    # the down projection's pair: the product summed per token, its gradients fetching the token gradient by index
    tokens = rows // 4
    row_index = torch.arange(rows, device=device) % tokens
    inv_map = build_inv_map(row_index, tokens, 4)
    token_grad = torch.randn(tokens, n, generator=g, device=device, dtype=torch.bfloat16)
    a_leaf, w_leaf = a.requires_grad_(True), w.requires_grad_(True)
    out = grouped_mm_combine(a_leaf, w_leaf, offs=offs, row_index=row_index, inv_map=inv_map)
    out.backward(token_grad)
    with torch.no_grad():
        want = torch.stack([token_grad[row_index[r]].float() @ w[group_of[r]].float().t() for r in pick.tolist()])
        _close(a_leaf.grad[pick], want)
        lo, hi = ends[1], ends[2]
        _close(w_leaf.grad[1], a.detach()[lo:hi].float().t() @ token_grad[row_index[lo:hi]].float())


@pytest.mark.parametrize(("k", "n"), ((256, 1536), (3072, 256)), ids=("output_past_2gib", "panels_past_2gib"))
@pytest.mark.parametrize("fmt", ("mxfp8", "mxfp4"))
def test_mx_expert_gemm_past_two_gib_on_the_scaled_kernel(device, fmt, k, n):
    """720 000 rows: with 1536 columns the output passes 2 GiB, with a contraction of 3072 the quantised activations'
    panels do (MXFP8; the e2m1 panels hold half as many bytes).  The scaled-MFMA kernel rebases its descriptors per
    stage and per tile, so the product stays native: sampled rows of every group, the first and the last rows among
    them, against the fp32 product of the round-tripped operands (the same products summed in another order, then one
    bf16 rounding: within 2^-7 of the row's largest output); the input gradient is the straight-through one."""
    from halo_amd.kernels.expert_gemm import expert_gemm, mxfp4_mfma_usable, mxfp8_mfma_usable
    from halo_amd.kernels.grouped_mm import grouped_mm_grads
    from halo_amd.kernels.lowp.quantization import fake_quant

    rows, groups = 720_000, 3
    usable = mxfp8_mfma_usable if fmt == "mxfp8" else mxfp4_mfma_usable
    assert max(rows * n * 2, rows * k) >= 2**31 and usable(torch.bfloat16, torch.bfloat16, k, n, rows)
    g = torch.Generator(device=device).manual_seed(7)
    a = torch.randn(rows, k, generator=g, device=device, dtype=torch.bfloat16).requires_grad_(True)
    w = (torch.randn(groups, k, n, generator=g, device=device) * 0.05).bfloat16()
    ends = [5, rows - 300, rows]
    offs = torch.tensor(ends, dtype=torch.int32, device=device)
    out = expert_gemm(a, w, offs=offs, quant_format=fmt)
    a_rt, w_rt = fake_quant(a.detach(), fmt, axis=-1), fake_quant(w, fmt, axis=1)
    pick = torch.cat([_sample(rows, 200, g, device), torch.arange(0, 8, device=device),
                      torch.arange(rows - 600, rows, device=device)])
    group_of = torch.bucketize(pick, offs.long(), right=True)
    for grp in range(groups):
        sel = pick[group_of == grp]
        want = a_rt[sel].float() @ w_rt[grp].float()
        bound = 2.0 ** -7 * want.abs().amax(dim=1, keepdim=True).clamp_min(1e-6)
        assert ((out[sel].float() - want).abs() <= bound).all(), (fmt, grp)
    dout = torch.randn(rows, n, generator=g, device=device, dtype=torch.bfloat16)
    out.backward(dout)
    want_da, _ = grouped_mm_grads(a_rt, w_rt, dout, offs, True, False)
    assert torch.equal(a.grad[pick], want_da[pick])
