"""GPU parity tests for the MXFP4 expert path: the quantiser, dequantiser and fused round trip bit for bit against
``oracle.mxfp4`` (a restatement of the reference's eager ``quantize_mxfp4`` / ``dequantize``), the known answers the
reference's own tests hold, ``expert_gemm(quant_format="mxfp4")`` on the scaled matrix instruction with e2m1 operands
against the float64 product of the oracle's round-tripped operands, the straight-through backward, and the layer with
``set_lowp_compute("mxfp4")`` against the CPU loop over fake-quantised products."""

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _edge_rows(rows, k, seed, dtype=torch.bfloat16):
    """Values over 40 binades plus the blocks the scale and rounding rules turn on: all zero, amax exactly 6 with every
    level and every tie beside it, the bf16 neighbours of 6, below 6 * 2^-127, one holding an inf, one holding a NaN,
    negative zeros, values that round to zero from below."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, k, generator=g) * torch.exp2(
        torch.randint(-20, 20, (rows, k // 32), generator=g).repeat_interleave(32, dim=1).float())
    x = x.to(dtype).float()
    x[0, :32] = 0
    x[1, :32] = torch.tensor([6.0, 0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, -0.5, -6.0, 0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0,
                              -0.25, -0.75, -1.25, -1.75, -2.5, -3.5, -5.0, 0.7, 0.8, 2.4, 2.6, -0.0, -0.1, 0.2, 5.5])
    x[2, :32] = 0; x[2, 3] = -6.03125  # the next bf16 magnitude above 6: scale 2
    x[3, :32] = 0; x[3, 3] = 5.96875   # the next below: scale 1
    sign = torch.where(torch.rand(32, generator=g) < 0.5, -1.0, 1.0)
    x[4, :32] = (torch.rand(32, generator=g) * 0.5 + 0.5) * 3e-38 * sign
    x[5, :32] = torch.exp2(torch.rand(32, generator=g) * 19 + 108) * sign
    x[5, 0] = float("inf")
    x[6, 40] = float("nan")
    x[7, :32] = x[1, :32] * 2.0 ** -40  # the same levels and ties under another scale
    return x.to(dtype)


def _equal_with_nan(got: torch.Tensor, want: np.ndarray):
    assert torch.equal(got.float().cpu().nan_to_num(nan=7.0), torch.from_numpy(want).nan_to_num(nan=7.0))


@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float32), ids=("bf16", "fp32"))
@pytest.mark.parametrize("k", (256, 96))
def test_row_quantiser_dequantiser_and_round_trip_equal_the_oracle_bit_for_bit(device, dtype, k):
    from halo_amd.kernels.lowp.quantization import dequantize, fake_quant, quantize_mxfp4
    from oracle import mxfp4 as oracle

    x = _edge_rows(70, k, seed=31, dtype=dtype)
    if dtype == torch.float32:  # values with full fp32 mantissas: the exponent rule is exact arithmetic on both sides
        x[8:] = x[8:] * (1 + torch.rand(x[8:].shape, generator=torch.Generator().manual_seed(2)) * 2 ** -9)
    want_data, want_scales = oracle.quantize_mxfp4(x.float().numpy())
    q = quantize_mxfp4(x.to(device))
    assert q.data.dtype == torch.uint8 and q.data.shape == (70, k // 2)
    assert q.scales.dtype == torch.uint8 and q.scales.shape == (70, k // 32)
    assert q.block_size == 32 and q.axis == 1 and q.packed and q.pow2_scale and q.global_scale is None
    assert np.array_equal(q.scales.cpu().numpy(), want_scales)
    assert want_scales[0, 0] == 0 and want_scales[1, 0] == 127 and want_scales[2, 0] == 128 and want_scales[3, 0] == 127
    assert want_scales[4, 0] == 0 and want_scales[5, 0] == 254 and want_scales[6, 1] == 255 and want_scales[7, 0] == 87
    assert np.array_equal(q.data.cpu().numpy(), want_data)
    # the reference's known answers (tests/cpu/kernels/test_block_scale_oracle.py:60-94,
    # tests/cpu/kernels/test_quantization.py:99-113) on the device: levels keep their codes, ties go to the even code
    codes = oracle.unpack_codes(q.data.cpu().numpy())[1, :28].tolist()
    assert codes == [7, 0, 1, 2, 3, 4, 5, 6, 9, 15, 0, 2, 2, 4, 4, 6, 6, 8, 10, 10, 12, 12, 14, 14, 1, 2, 4, 5]
    restored = dequantize(q)
    assert restored.dtype == torch.bfloat16 and restored.shape == x.shape
    want = oracle.dequantize_mxfp4(want_data, want_scales)
    _equal_with_nan(restored, want)
    fused = fake_quant(x.to(device), "mxfp4")  # one launch, no codes written
    assert fused.dtype == dtype
    _equal_with_nan(fused, want)


@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float32), ids=("bf16", "fp32"))
def test_negative_values_that_the_scaling_rounds_to_zero_take_the_code_of_zero(device, dtype):
    """A negative value whose scaled fp32 product underflows (beside an inf, or more than 150 binades below its block's
    largest magnitude) is -0.0 by then, which the reference's ``scaled < 0`` does not count as negative: code 0, not 8
    (``quantization.py:166-177, 191-198``).  Rows and weights, against the oracle's codes."""
    from halo_amd.kernels.lowp.quantization import quantize_mxfp4
    from oracle import mxfp4 as oracle

    g = torch.Generator().manual_seed(12)
    x = torch.randn(6, 64, generator=g)
    x[0, :32] = -torch.rand(32, generator=g) * 1e-11
    x[0, 5] = float("inf")                                   # scale 254: everything finite underflows
    x[1, :32] = -torch.rand(32, generator=g) * 1e-20
    x[1, 9] = 1e30                                           # 166 binades above the rest
    x[2, 32:] = torch.rand(32, generator=g) * 1e-20 * torch.where(torch.rand(32, generator=g) < 0.5, -1.0, 1.0)
    x[2, 40] = -3e29
    x[3, :32] = -torch.rand(32, generator=g) * 2.0 ** -20    # a span that does not underflow: the sign stays
    x[3, 0] = 2.0 ** 100
    x = x.to(dtype)
    want_data, want_scales = oracle.quantize_mxfp4(x.float().numpy())
    codes = oracle.unpack_codes(want_data)
    assert (codes[0, :32] == 0).sum() == 31 and (codes[1, :32] == 0).sum() == 31 and (codes[3, 1:32] == 8).all()
    q = quantize_mxfp4(x.to(device))
    assert np.array_equal(q.scales.cpu().numpy(), want_scales) and np.array_equal(q.data.cpu().numpy(), want_data)
    w = x.t().contiguous().view(1, 64, 6).repeat(2, 1, 1)    # the same blocks down the columns of a weight
    want_data, want_scales = oracle.quantize_mxfp4(w.float().numpy(), axis=1)
    q = quantize_mxfp4(w.to(device), axis=1)
    assert np.array_equal(q.scales.cpu().numpy(), want_scales) and np.array_equal(q.data.cpu().numpy(), want_data)


def test_row_round_trip_fetches_rows_through_an_index(device):
    from halo_amd.kernels.lowp.quantization import mxfp4_rows

    g = torch.Generator().manual_seed(5)
    x = torch.randn(50, 192, generator=g).bfloat16().to(device)
    index = torch.randint(0, 50, (333,), generator=g).to(device)
    index[7], index[200] = -1, 50  # outside the array: rows of zeros
    inside = ((index >= 0) & (index < 50)).unsqueeze(1)
    rows = torch.where(inside, x[index.clamp(0, 49)], torch.zeros((), device=device, dtype=x.dtype))
    direct = mxfp4_rows(rows, round_trip=True)
    gathered = mxfp4_rows(x, index, round_trip=True)
    assert all(torch.equal(d, f) for d, f in zip(direct, gathered))
    assert gathered[2].shape == (333, 192) and not gathered[2][7].any() and not gathered[0][200].any()
    only = mxfp4_rows(x, index, codes=False, round_trip=True)
    assert only[0] is None and only[1] is None and torch.equal(only[2], gathered[2])
    with pytest.raises(ValueError, match="nothing to compute"):
        mxfp4_rows(x, codes=False)


@pytest.mark.parametrize(("groups", "k", "n", "dtype"), ((3, 96, 136, torch.bfloat16), (2, 128, 130, torch.bfloat16),
                                                         (2, 64, 264, torch.float32)))
def test_weight_quantiser_equals_the_oracle_bit_for_bit(device, groups, k, n, dtype):
    """``quantize_mxfp4(w, axis=1)`` of an ``[E, K, N]`` weight: codes, scales and the round trip; a contraction that
    ends in half a tile, a column count that is no multiple of eight (element loads), fp32 masters."""
    from halo_amd.kernels.lowp.quantization import dequantize, fake_quant, quantize_mxfp4
    from oracle import mxfp4 as oracle

    g = torch.Generator().manual_seed(9)
    w = (torch.randn(groups, k, n, generator=g) * torch.exp2(torch.randint(-12, 4, (groups, 1, n), generator=g).float()))
    w = w.to(dtype)
    w[0, :32, 0] = 0
    w[0, 32:64, 1] = 0
    w[0, 40, 1] = 6.0
    w[0, 41:45, 1] = torch.tensor([0.75, -1.75, 2.5, 3.5]).to(dtype)
    w[1, :32, 5] = float("nan")
    want_data, want_scales = oracle.quantize_mxfp4(w.float().numpy(), axis=1)
    q = quantize_mxfp4(w.to(device), axis=1)
    assert q.data.shape == (groups, k // 2, n) and q.scales.shape == (groups, k // 32, n) and q.axis == 1 and q.packed
    assert np.array_equal(q.scales.cpu().numpy(), want_scales)
    assert np.array_equal(q.data.cpu().numpy(), want_data)
    want = oracle.dequantize_mxfp4(want_data, want_scales, axis=1)
    _equal_with_nan(dequantize(q), want)
    round_trip = fake_quant(w.to(device), "mxfp4", axis=1)
    assert round_trip.dtype == dtype
    _equal_with_nan(round_trip, want)
    # an axis that is neither the last nor the one before it
    moved = quantize_mxfp4(w.to(device).permute(1, 0, 2).contiguous(), axis=0)
    assert moved.data.shape == (k // 2, groups, n) and torch.equal(moved.data.permute(1, 0, 2), q.data)
    _equal_with_nan(dequantize(moved).permute(1, 0, 2), want)


def test_fake_quant_api_as_the_reference_tests_state_it(device):
    """``tests/cpu/kernels/test_quantization.py`` of the reference, on the device: storage shapes and dtypes (:48-55),
    round trip inside the format's tolerance with mxfp8 the more accurate (:58-71), zeros (:82-89), midpoints to the
    even code (:99-113), the divisibility guard (:127-135), the straight-through backward (:138-146), the input dtype
    kept (:149-151), the weight cache (:154-183); and of ``tests/cpu/kernels/test_block_scale_oracle.py``: the error
    independent of the magnitude (:118-137), a shard quantised alone equal to its slice of the bank (:157-172), an inf
    or a NaN never absorbed and finite inputs never non-finite (:175-196)."""
    from halo_amd.kernels.lowp.quantization import (QUANTIZERS, cached_fake_quant, dequantize, fake_quant,
                                                    quantize_mxfp4, quantize_mxfp8)

    def fro(a, b):
        return ((a.double() - b.double()).norm() / b.double().norm()).item()

    assert {"mxfp4", "mxfp8"} <= set(QUANTIZERS)
    torch.manual_seed(0)
    x = (torch.randn(64, 256) * 0.5).to(device)
    q = quantize_mxfp4(x, axis=-1)
    assert q.data.shape == (64, 128) and q.data.dtype == torch.uint8
    assert q.scales.shape == (64, 8) and q.scales.dtype == torch.uint8 and q.packed and q.pow2_scale
    recon = dequantize(q)
    assert recon.dtype == torch.bfloat16 and fro(dequantize(quantize_mxfp8(x)), x) < fro(recon, x) < 0.25
    zeros = dequantize(quantize_mxfp4(torch.zeros(32, 64, device=device)))
    assert torch.isfinite(zeros).all() and zeros.abs().max().item() == 0.0
    block = torch.zeros(1, 32)
    block[0, :7] = torch.tensor([6.0, 0.75, 1.75, 3.5, -0.75, 0.7, 0.8])
    assert dequantize(quantize_mxfp4(block.to(device)))[0, :7].tolist() == [6.0, 1.0, 2.0, 4.0, -1.0, 0.5, 1.0]
    with pytest.raises(ValueError, match="not divisible"):
        quantize_mxfp4(torch.randn(8, 30, device=device))
    with pytest.raises(ValueError, match="unknown block-scaled format"):
        fake_quant(x, "fp3")
    base = torch.randn(128, 256).double()
    errs = []
    for exponent in range(4, -32, -4):
        scaled = (base * 10.0 ** exponent).float().to(device)
        errs.append(fro(dequantize(quantize_mxfp4(scaled)), scaled))
    assert max(errs) - min(errs) < 0.02 and 0.05 < errs[0] < 0.25
    bank = torch.randn(8, 64, 256) * 0.02
    bank[0] *= 1e-3
    bank = bank.to(device)
    gathered = dequantize(quantize_mxfp4(bank, axis=-1))
    sharded = torch.cat([dequantize(quantize_mxfp4(s, axis=-1)) for s in bank.chunk(4, dim=0)], dim=0)
    assert torch.equal(sharded, gathered)
    for poison in (float("nan"), float("inf"), float("-inf")):
        bad = torch.randn(4, 64) * 0.3
        bad[1, 7] = poison
        recon = dequantize(quantize_mxfp4(bad.to(device)))
        assert not torch.isfinite(recon[1, :32]).all() and torch.isfinite(recon[1, 32:]).all()
        assert torch.isfinite(recon[0]).all()
    outlier = torch.randn(4, 64) * 0.3
    outlier[0, 0] = 5e4
    outlier[2, :] = 0.0
    assert torch.isfinite(dequantize(quantize_mxfp4(outlier.to(device)))).all()

    leaf = (torch.randn(64, 256) * 0.3).to(device).requires_grad_(True)
    y = fake_quant(leaf, "mxfp4", axis=-1)
    assert fro(y.detach(), leaf.detach()) < 0.25
    assert torch.equal(y.detach().bfloat16(), dequantize(quantize_mxfp4(leaf.detach())))
    (y * 2.0).sum().backward()
    assert torch.equal(leaf.grad, torch.full_like(leaf.grad, 2.0))
    assert fake_quant((torch.randn(32, 64) * 0.2).bfloat16().to(device), "mxfp4").dtype == torch.bfloat16
    w = torch.nn.Parameter((torch.randn(8, 64) * 0.3).to(device))
    cached = cached_fake_quant(w, "mxfp4", axis=-1)
    assert torch.equal(cached.detach(), fake_quant(w.detach(), "mxfp4", axis=-1))
    first = cached.detach().clone()
    assert torch.equal(first, cached_fake_quant(w, "mxfp4", axis=-1).detach())
    with torch.no_grad():
        w.add_(1.0)
    after = cached_fake_quant(w, "mxfp4", axis=-1).detach()
    assert not torch.equal(first, after) and fro(after, w.detach()) < 0.25
    (cached_fake_quant(w, "mxfp4", axis=-1) * 3.0).sum().backward()
    assert torch.equal(w.grad, torch.full_like(w.grad, 3.0))


def test_panel_quantisers_hold_the_same_codes_in_the_matrix_kernels_layout(device):
    """The operands of the e2m1 matrix kernel are the quantiser's codes and exponents in panels of 128 contraction
    values: unfolded they equal ``quantize_mxfp4``'s bit for bit, the last panel is zeros past K, the rows can be
    fetched through an index, and the dequantiser gives the round trip back."""
    from halo_amd.kernels.lowp.quantization import (dequantize, dequantize_rows_mxfp4, quantize_mxfp4,
                                                    quantize_rows_mxfp4, quantize_weight_mxfp4)

    for k in (192, 256, 96):
        x = _edge_rows(70, k, seed=33).to(device)
        logical = quantize_mxfp4(x)
        rows = quantize_rows_mxfp4(x)
        panels = -(-k // 128)
        assert rows.q.shape == (panels, 70, 64) and rows.scales.shape == (panels, 70, 4) and rows.rows == 70
        codes = rows.q.permute(1, 0, 2).reshape(70, panels * 64)
        scales = rows.scales.permute(1, 0, 2).reshape(70, panels * 4)
        assert torch.equal(codes[:, :k // 2], logical.data) and not codes[:, k // 2:].any()
        assert torch.equal(scales[:, :k // 32], logical.scales) and not scales[:, k // 32:].any()
        want = dequantize(logical)
        assert torch.equal(dequantize_rows_mxfp4(rows).nan_to_num(nan=7.0), want.nan_to_num(nan=7.0))
        index = (torch.arange(101, device=device) * 7) % 70
        index[5] = -1
        fetched = quantize_rows_mxfp4(x, index)
        assert torch.equal(fetched.q[:, 6], rows.q[:, 42]) and not fetched.q[:, 5].any() and not fetched.scales[:, 5].any()
    g = torch.Generator().manual_seed(11)
    for groups, k, n, dtype in ((3, 96, 136, torch.bfloat16), (2, 320, 130, torch.bfloat16), (2, 128, 264, torch.float32)):
        w = (torch.randn(groups, k, n, generator=g) * torch.exp2(torch.randint(-12, 4, (groups, 1, n), generator=g).float()))
        w = w.to(dtype).to(device)
        logical = quantize_mxfp4(w, axis=1)
        weight = quantize_weight_mxfp4(w, with_dequant=True)
        panels = -(-k // 128)
        assert weight.q.shape == (groups, panels, n, 64) and weight.scales.shape == (groups, panels, n, 4)
        codes = weight.q.permute(0, 1, 3, 2).reshape(groups, panels * 64, n)
        scales = weight.scales.permute(0, 1, 3, 2).reshape(groups, panels * 4, n)
        assert torch.equal(codes[:, :k // 2], logical.data) and not codes[:, k // 2:].any()
        assert torch.equal(scales[:, :k // 32], logical.scales) and not scales[:, k // 32:].any()
        assert torch.equal(weight.dequant, dequantize(logical))


GEMM_CASES = (
    # counts, K, N
    ((255, 256, 257, 0, 513, 31), 192, 264),   # row tiles that end inside a tile, an empty group, half a panel at the end
    ((64,) * 16, 128, 1536),                   # one contraction step
    ((64,) * 4, 32, 64),                       # a quarter of a panel
    ((1, 0, 0, 700, 3), 2880, 136),            # 22 panels and a half, tiny groups beside a large one
    ((300, 41), 256, 8),                       # one 16-byte output row
)


@pytest.mark.parametrize(("counts", "k", "n"), GEMM_CASES)
def test_mxfp4_expert_gemm_against_the_oracle_product(device, counts, k, n):
    """``expert_gemm(quant_format="mxfp4")`` on the scaled matrix instruction with e2m1 operands against the float64
    product of the oracle's round-tripped operands.  Every term is exact in either; the kernel accumulates in fp32 and
    rounds once to bf16, so the error is bf16's half ulp (2^-9 relative) plus the accumulation's, bounded here by 2^-8
    of the element or 2^-8 of the root-sum-square of its terms' scale.  Row scales that differ from block to block and
    from row to row, so that a block's exponent applied to the wrong values shows."""
    from halo_amd.kernels.expert_gemm import expert_gemm
    from oracle import mxfp4 as oracle

    g = torch.Generator().manual_seed(41)
    rows = sum(counts)
    a = (torch.randn(rows, k, generator=g) * torch.exp2(torch.randint(-6, 3, (rows, k // 32), generator=g)
                                                         .repeat_interleave(32, dim=1).float())).bfloat16()
    b = (torch.randn(len(counts), k, n, generator=g) * 0.05 * torch.exp2(
        torch.randint(-3, 3, (len(counts), k // 32, n), generator=g).repeat_interleave(32, dim=1).float())).bfloat16()
    offs = torch.tensor(counts).cumsum(0).int()
    want = oracle.expert_gemm_mxfp4(a.float().numpy(), b.float().numpy(), offs.numpy())
    got = expert_gemm(a.to(device), b.to(device), offs=offs.to(device), quant_format="mxfp4", weight_cacheable=False)
    assert got.dtype == torch.bfloat16 and got.shape == (rows, n)
    err = np.abs(got.float().cpu().numpy().astype(np.float64) - want)
    group_of = np.repeat(np.arange(len(counts)), counts)
    aq, bq = oracle.fake_quant_mxfp4(a.float().numpy()), oracle.fake_quant_mxfp4(b.float().numpy(), 1)
    spread = np.linalg.norm(aq, axis=1)[:, None] * np.linalg.norm(bq, axis=1)[group_of]
    assert (err <= 2.0 ** -8 * np.abs(want) + 2.0 ** -8 * spread / np.sqrt(k)).all()
    plain = np.zeros_like(want)
    start = 0
    for e, end in enumerate(offs.tolist()):
        plain[start:end] = a[start:end].double().numpy() @ b[e].double().numpy()
        start = end
    shift = np.linalg.norm(want - plain) / np.linalg.norm(plain)
    assert 0.04 < shift < 0.25, shift  # the quantisation took place, and at the format's size


def test_mxfp4_expert_gemm_outside_the_matrix_kernel_is_the_product_of_the_round_tripped_operands(device):
    """fp32 operands take the reference's own formulation (``expert_gemm.py:33-38``): bit-equal to ``grouped_mm`` over the two ``fake_quant`` results, forward and both
    gradients; within the kernel's bound of the oracle's float64 product; an empty group leaves exact zeros in the weight
    gradient; fp32 operands stay fp32."""
    from halo_amd.kernels.expert_gemm import expert_gemm
    from halo_amd.kernels.grouped_mm import grouped_mm, grouped_mm_grads
    from halo_amd.kernels.lowp.quantization import fake_quant
    from oracle import mxfp4 as oracle

    g = torch.Generator().manual_seed(43)
    counts = (255, 0, 257, 40, 513, 31)
    offs = torch.tensor(counts).cumsum(0).int()
    for dtype, k, n in ((torch.float32, 96, 72), (torch.float32, 160, 36)):
        a = (torch.randn(sum(counts), k, generator=g) * torch.exp2(torch.randint(-6, 3, (sum(counts), 1), generator=g)
                                                                   .float())).to(dtype)
        b = (torch.randn(len(counts), k, n, generator=g) * 0.05).to(dtype)
        want = oracle.expert_gemm_mxfp4(a.float().numpy(), b.float().numpy(), offs.numpy())
        al, bl = a.to(device).requires_grad_(True), b.to(device).requires_grad_(True)
        dev_offs = offs.to(device)
        got = expert_gemm(al, bl, offs=dev_offs, quant_format="mxfp4", weight_cacheable=False)
        assert got.dtype == dtype and got.shape == (sum(counts), n)
        upstream = torch.randn(got.shape, generator=g).to(dtype).to(device)
        got.backward(upstream)
        with torch.no_grad():
            aq, bq = fake_quant(al.detach(), "mxfp4", -1), fake_quant(bl.detach(), "mxfp4", 1)
            assert torch.equal(got, grouped_mm(aq, bq, offs=dev_offs))
            grad_a, grad_b = grouped_mm_grads(aq, bq, upstream, dev_offs, True, True)
            assert torch.equal(al.grad, grad_a) and torch.equal(bl.grad, grad_b) and not bl.grad[1].any()
        tol = 2.0 ** -7 if dtype == torch.bfloat16 else 1e-5
        assert np.abs(got.detach().float().cpu().numpy() - want).max() <= tol * np.abs(want).max()


def test_mxfp4_expert_gemm_at_the_reference_band_shape_with_its_backward(device):
    """The reference's banded check (``tests/gpu/kernels/test_expert_gemm.py:55-74``: E = 8, M = 256, K = N = 2880,
    the relative error against the bf16 product inside the 4-bit band 0.04-0.25, finite gradients) and its dispatch
    contract (``:77-106``: every implemented format returns ``[E * M, N]``); then the straight-through backward bit for
    bit: the gradients are ``grouped_mm``'s own over the two round-tripped operands, and the forward is the bf16
    kernel's product of those within its rounding."""
    from halo_amd.kernels.expert_gemm import expert_gemm
    from halo_amd.kernels.grouped_mm import grouped_mm, grouped_mm_grads
    from halo_amd.kernels.lowp.quantization import fake_quant

    torch.manual_seed(0)
    e, m, k, n = 8, 256, 2880, 2880
    x = (torch.randn(e * m, k, device=device, dtype=torch.bfloat16) * 0.3).requires_grad_(True)
    w = (torch.randn(e, k, n, device=device, dtype=torch.bfloat16) * 0.02).requires_grad_(True)
    offs = torch.arange(m, e * m + 1, m, device=device, dtype=torch.int32)
    out = expert_gemm(x, w, offs=offs, quant_format="mxfp4")
    assert out.shape == (e * m, n) and out.dtype == torch.bfloat16
    upstream = torch.randn_like(out)
    (out * upstream).sum().backward()
    with torch.no_grad():
        plain = grouped_mm(x, w, offs=offs)
        rel = ((out.double() - plain.double()).norm() / plain.double().norm()).item()
        assert 0.04 < rel < 0.25, rel
        assert torch.isfinite(x.grad).all() and torch.isfinite(w.grad).all()
        xq, wq = fake_quant(x.detach(), "mxfp4", -1), fake_quant(w.detach(), "mxfp4", 1)
        simulated = grouped_mm(xq, wq, offs=offs)  # the reference's formulation: the same terms on the bf16 kernel
        assert ((out.double() - simulated.double()).norm() / simulated.double().norm()).item() < 2e-3
        grad_x, grad_w = grouped_mm_grads(xq, wq, upstream, offs, True, True)
        assert torch.equal(x.grad, grad_x) and torch.equal(w.grad, grad_w)
    with pytest.raises(ValueError, match="unknown block-scaled format"):
        expert_gemm(x, w, offs=offs, quant_format="fp3")


def test_mxfp4_rows_fetched_through_the_sorts_index_and_shared_between_projections(device, monkeypatch):
    """Rows fetched through the sort's index give the same bits as rows gathered first, and their gradient is summed
    back per token; gate and up stored apart read the same rows, quantise them once and rebuild them once in backward;
    the weights' operand is kept until the parameter changes."""
    from halo_amd.kernels import expert_gemm as eg
    from halo_amd.kernels.grouped_mm import GatheredRows
    from halo_amd.kernels.lowp import quantization
    from halo_amd.kernels.moe_permute import build_inv_map

    calls = {"rows": 0, "weight": 0, "back": 0}

    def counting(name, real):
        def wrapper(*args, **kwargs):
            calls[name] += 1
            return real(*args, **kwargs)
        return wrapper

    monkeypatch.setattr(quantization, "quantize_rows_mxfp4", counting("rows", quantization.quantize_rows_mxfp4))
    monkeypatch.setattr(quantization, "quantize_weight_mxfp4", counting("weight", quantization.quantize_weight_mxfp4))
    monkeypatch.setattr(quantization, "dequantize_rows_mxfp4", counting("back", quantization.dequantize_rows_mxfp4))
    g = torch.Generator().manual_seed(47)
    offs = torch.tensor([40, 40, 110, 128], dtype=torch.int32, device=device)
    tokens = torch.randn(40, 128, generator=g).bfloat16().to(device).requires_grad_(True)
    w_gate = torch.nn.Parameter((torch.randn(4, 128, 64, generator=g) * 0.05).bfloat16().to(device))
    w_up = torch.nn.Parameter((torch.randn(4, 128, 64, generator=g) * 0.05).bfloat16().to(device))
    row_index = torch.arange(128, device=device) % 40
    inv_map = build_inv_map(row_index, 40, 4)
    upstream = torch.randn(128, 64, generator=g).bfloat16().to(device)
    rows = GatheredRows(tokens, row_index, inv_map)
    gate = eg.expert_gemm(rows, w_gate, offs=offs, quant_format="mxfp4")
    up = eg.expert_gemm(rows, w_up, offs=offs, quant_format="mxfp4")
    assert calls == {"rows": 1, "weight": 2, "back": 0}
    grad_fetched, _, _ = torch.autograd.grad(gate + up, (tokens, w_gate, w_up), upstream)
    assert calls["back"] == 1
    copied = tokens[row_index]
    gate2 = eg.expert_gemm(copied, w_gate, offs=offs, quant_format="mxfp4")
    up2 = eg.expert_gemm(copied, w_up, offs=offs, quant_format="mxfp4")
    assert calls["rows"] == 2 and calls["weight"] == 2  # other rows; the weights are those of the step
    (grad_copied,) = torch.autograd.grad(gate2 + up2, tokens, upstream)
    assert torch.equal(gate, gate2) and torch.equal(up, up2)
    assert ((grad_fetched.double() - grad_copied.double()).norm() / grad_copied.double().norm()).item() < 5e-3
    with torch.no_grad():
        w_gate.mul_(0.5)  # an optimizer step: exactly half, so the codes stay and every exponent drops by one
    again = eg.expert_gemm(copied, w_gate, offs=offs, quant_format="mxfp4")
    assert calls["weight"] == 3 and torch.equal(again, gate2 * 0.5)
    eg.expert_gemm(copied, w_gate, offs=offs, quant_format="mxfp4", weight_cacheable=False)
    assert calls["weight"] == 4


@pytest.mark.parametrize("fmt", ("mxfp8", "mxfp4"))
def test_expert_bias_joins_the_mx_products_in_the_epilogue(device, fmt):
    """``expert_gemm(..., bias=, eids=)`` for the MX formats (reference ``families/gpt_oss.py:153-159``: the projection,
    then ``+ bias[eids]``): bit-equal to the product followed by the tensor addition, a partial column tile and an empty
    group included; the bias gradient is the per-expert column sum of the rows' gradient (exact zeros for the empty
    group), the other gradients are unchanged; fp32 operands (outside the matrix kernel) take the addition unfused."""
    from halo_amd.kernels.expert_gemm import expert_gemm

    g = torch.Generator().manual_seed(53)
    counts = (255, 0, 257, 40, 513, 31)
    offs = torch.tensor(counts).cumsum(0).int().to(device)
    eids = torch.repeat_interleave(torch.arange(len(counts)), torch.tensor(counts)).to(device)
    for dtype, k, n in ((torch.bfloat16, 192, 264), (torch.bfloat16, 2880, 136), (torch.float32, 96, 72)):
        a = (torch.randn(sum(counts), k, generator=g) * 0.5).to(dtype).to(device).requires_grad_(True)
        b = (torch.randn(len(counts), k, n, generator=g) * 0.05).to(dtype).to(device).requires_grad_(True)
        bias = torch.randn(len(counts), n, generator=g).to(dtype).to(device).requires_grad_(True)
        upstream = torch.randn(sum(counts), n, generator=g).to(dtype).to(device)
        fused = expert_gemm(a, b, offs=offs, quant_format=fmt, weight_cacheable=False, bias=bias, eids=eids)
        grads_fused = torch.autograd.grad(fused, (a, b, bias), upstream)
        plain = expert_gemm(a, b, offs=offs, quant_format=fmt, weight_cacheable=False) + bias[eids]
        grads_plain = torch.autograd.grad(plain, (a, b, bias), upstream)
        assert fused.dtype == dtype and torch.equal(fused, plain)
        assert torch.equal(grads_fused[0], grads_plain[0]) and torch.equal(grads_fused[1], grads_plain[1])
        want = torch.zeros(len(counts), n, dtype=torch.float64, device=device).index_add_(0, eids, upstream.double())
        assert not grads_fused[2][1].any()
        tol = 2.0 ** -8 if dtype == torch.bfloat16 else 1e-5
        assert ((grads_fused[2].double() - want).abs() <= tol * want.abs() + tol).all()
    with pytest.raises(ValueError, match="bias is taken"):
        expert_gemm(a, b, offs=offs, bias=bias, eids=eids)


@pytest.mark.parametrize("name", ("cfg2_small", "cfg4_small"))
def test_layer_with_mxfp4_experts_against_the_cpu_loop_over_fake_quantised_products(device, name):
    """``set_lowp_compute("mxfp4")`` on the layer (reference ``compute.py:53-58, 306-312``): forward and every
    gradient against the oracle's per-expert loop with both operands of each product round-tripped (straight-through
    backward).  Stored fused (rows fetched through the sort's index by the round trip) and stored apart with biases.

    Tolerance: the layer keeps its intermediate tensors in bf16 and the oracle in fp32, and a 4-bit quantiser sits
    behind them: a bf16 rounding (2^-9 relative) moves well under 1 % of the GLU outputs across an e2m1 rounding
    boundary (the levels lie 25-50 % apart), but each of those moves by a whole level, a third of its value on average,
    which is 2-3 % of relative RMS error in the down projection's operand before any kernel error.  Hence a relative
    Frobenius error of 6 % and a cosine of 0.998 here; the products themselves are held to 2^-8 in the GEMM tests
    above."""
    from halo_amd.kernels.router import SOFTMAX_ALL, SOFTMAX_TOPK, fused_topk_gate
    from oracle import moe_layer as oracle
    from oracle import mxfp4 as mx_oracle
    from oracle import router as router_oracle
    from tests import cases
    from tests.test_gpu_layer import _build_layer, cosine

    def _check(what, got, ref, tol):
        assert torch.isfinite(got).all(), what
        err = ((got.double().cpu() - ref.double()).norm() / ref.double().norm()).item()
        assert err <= tol and cosine(got, ref) >= 0.998, (what, err, cosine(got, ref))

    cfg = {"cfg2_small": cases.CONFIG2_SMALL, "cfg4_small": cases.CONFIG4_SMALL._replace(hidden=384, ffn=352)}[name]
    inputs = cases.make_layer_inputs(cfg)
    layer = _build_layer(cfg, inputs, device)
    assert layer.set_lowp_compute("mxfp4", weight_cacheable=True) is True
    x = inputs["x"].to(device).requires_grad_(True)
    result = layer(x)
    out = result[0] if isinstance(result, tuple) else result
    out.backward(inputs["grad_out"].to(device))
    with torch.no_grad():
        again = layer(x.detach())
    again = again[0] if isinstance(again, tuple) else again
    assert torch.equal(again, out.detach())

    with torch.no_grad():
        logits = layer._linear_router_logits(x.detach())
        mode = SOFTMAX_TOPK if cfg.router == "softmax_topk" else SOFTMAX_ALL
        idx, _ = fused_topk_gate(logits, cfg.top_k, mode=mode, normalize=True, eps=0.0)
    f = lambda t: t.float().requires_grad_(True)
    rx, wr = f(inputs["x"]), f(inputs["router_weight"])
    params = {k: f(v) for k, v in inputs["params"].items()}
    bias = f(inputs["router_bias"]) if "router_bias" in inputs else None
    glu = oracle.Glu("gptoss", 1.702, 7.0) if cfg.glu == "gptoss" else oracle.Glu(cfg.glu)
    ref_mode = router_oracle.SOFTMAX_TOPK if cfg.router == "softmax_topk" else router_oracle.SOFTMAX_ALL
    want, _, _, _ = oracle.moe_layer_forward(rx, wr, params, glu, cfg.top_k, router_bias=bias, mode=ref_mode,
                                             normalize=True, eps=0.0, indices=idx.cpu(), quant=mx_oracle.fake_quant_ste)
    want.backward(inputs["grad_out"].float())
    tol = 6e-2
    _check("out", out, want.detach(), tol)
    _check("grad x", x.grad, rx.grad, tol)
    _check("grad router_weight", getattr(layer, layer._ROUTER_ATTR).weight.grad, wr.grad, tol)
    for pname in inputs["params"]:
        attr = pname.replace("gate_proj", "gate_proj_gmm").replace("up_proj", "up_proj_gmm") \
            if cfg.router == "softmax_topk" else pname
        _check(f"grad {pname}", getattr(layer, attr).grad, params[pname].grad, tol)
    with torch.no_grad():
        plain, _, _, _ = oracle.moe_layer_forward(rx.detach(), wr.detach(), {k: v.detach() for k, v in params.items()},
                                                  glu, cfg.top_k, router_bias=None if bias is None else bias.detach(),
                                                  mode=ref_mode, normalize=True, eps=0.0, indices=idx.cpu())
    rel = ((out.detach().double().cpu() - plain.double()).norm() / plain.double().norm()).item()
    assert 0.05 < rel < 0.4, rel
