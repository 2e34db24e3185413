"""GPU parity tests for the MXFP8 expert path: the quantisers and dequantisers bit for bit against ``oracle.mxfp8`` (a
restatement of the reference's eager ``quantize_mxfp8`` / ``dequantize``), the product on the scaled e4m3 matrix
instruction against the float64 product of the oracle's round-tripped operands, the straight-through backward, and the
layer with ``set_lowp_compute("mxfp8")`` against the CPU loop over fake-quantised products."""

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _edge_rows(rows, k, seed, dtype=torch.bfloat16):
    """Values over 40 binades plus the blocks the scale rule turns on: all zero, exactly 448, the bf16 neighbours of
    448, below 448 * 2^-127, one holding an inf, one holding a NaN."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, k, generator=g) * torch.exp2(
        torch.randint(-20, 20, (rows, k // 32), generator=g).repeat_interleave(32, dim=1).float())
    x = x.to(dtype).float()
    x[0, :32] = 0
    x[1, :32] = 0; x[1, 3] = 448.0
    x[2, :32] = 0; x[2, 3] = -452.0
    x[3, :32] = 0; x[3, 3] = 446.0
    sign = torch.where(torch.rand(32, generator=g) < 0.5, -1.0, 1.0)
    x[4, :32] = (torch.rand(32, generator=g) * 0.5 + 0.5) * 3e-38 * sign
    x[5, :32] = torch.exp2(torch.rand(32, generator=g) * 19 + 108) * sign
    x[5, 0] = float("inf")
    x[6, 40] = float("nan")
    return x.to(dtype)


def _same_codes(got: np.ndarray, want: np.ndarray, scales_want: np.ndarray, axis: int):
    """Equal e4m3 codes; a zero may carry either sign, and inside a NaN block only NaN-ness is compared."""
    nan_block = np.repeat(scales_want == 255, 32, axis=axis)
    both_zero = ((got & 0x7F) == 0) & ((want & 0x7F) == 0)
    both_nan = nan_block & ((got & 0x7F) == 0x7F) & ((want & 0x7F) == 0x7F)
    assert ((got == want) | both_zero | both_nan).all()


@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float32), ids=("bf16", "fp32"))
@pytest.mark.parametrize("k", (256, 96))
def test_row_quantiser_and_dequantiser_equal_the_oracle_bit_for_bit(device, dtype, k):
    from halo_amd.kernels.lowp.quantization import dequantize, quantize_mxfp8
    from oracle import mxfp8 as oracle

    x = _edge_rows(70, k, seed=31, dtype=dtype)
    if dtype == torch.float32:  # values with full fp32 mantissas: the exponent rule is exact arithmetic on both sides
        x[8:] = x[8:] * (1 + torch.rand(x[8:].shape, generator=torch.Generator().manual_seed(2)) * 2 ** -9)
    want_data, want_scales = oracle.quantize_mxfp8(x.float().numpy())
    q = quantize_mxfp8(x.to(device))
    assert q.data.dtype == torch.float8_e4m3fn and q.data.shape == x.shape
    assert q.scales.dtype == torch.uint8 and q.scales.shape == (70, k // 32)
    assert q.block_size == 32 and q.axis == 1 and not q.packed and q.pow2_scale and q.global_scale is None
    assert np.array_equal(q.scales.cpu().numpy(), want_scales)
    assert want_scales[0, 0] == 0 and want_scales[1, 0] == 127 and want_scales[2, 0] == 128 and want_scales[4, 0] == 0
    assert want_scales[5, 0] == 254 and want_scales[6, 1] == 255
    _same_codes(q.data.view(torch.uint8).cpu().numpy(), want_data, want_scales, axis=1)
    restored = dequantize(q)
    assert restored.dtype == torch.bfloat16
    want = torch.from_numpy(oracle.dequantize_mxfp8(want_data, want_scales))
    assert torch.equal(restored.float().cpu().nan_to_num(nan=7.0), want.nan_to_num(nan=7.0))


def test_row_quantiser_fetches_rows_through_an_index(device):
    from halo_amd.kernels.lowp.quantization import dequantize_rows_mxfp8, quantize_rows_mxfp8

    g = torch.Generator().manual_seed(5)
    x = torch.randn(50, 192, generator=g).bfloat16().to(device)
    index = torch.randint(0, 50, (333,), generator=g).to(device)
    index[7], index[200] = -1, 50  # outside the array: rows of zeros
    inside = ((index >= 0) & (index < 50)).unsqueeze(1)
    direct = quantize_rows_mxfp8(torch.where(inside, x[index.clamp(0, 49)], torch.zeros((), device=device, dtype=x.dtype)))
    gathered = quantize_rows_mxfp8(x, index)
    assert torch.equal(direct.q, gathered.q) and torch.equal(direct.scales, gathered.scales)
    assert not dequantize_rows_mxfp8(gathered)[7].any()


@pytest.mark.parametrize(("groups", "k", "n", "dtype"), ((3, 96, 136, torch.bfloat16), (2, 128, 130, torch.bfloat16),
                                                         (2, 64, 264, torch.float32)))
def test_weight_quantiser_equals_the_oracle_bit_for_bit(device, groups, k, n, dtype):
    """``quantize_mxfp8(w, axis=1)`` of an ``[E, K, N]`` weight, codes, scales and the round trip; a contraction that
    ends in half a panel, a column count that is no multiple of eight (element loads), fp32 masters."""
    from halo_amd.kernels.lowp.quantization import dequantize, fake_quant, quantize_mxfp8
    from oracle import mxfp8 as oracle

    g = torch.Generator().manual_seed(9)
    w = (torch.randn(groups, k, n, generator=g) * torch.exp2(torch.randint(-12, 4, (groups, 1, n), generator=g).float()))
    w = w.to(dtype)
    w[0, :32, 0] = 0
    w[0, 32:64, 1] = 0
    w[0, 40, 1] = 448.0
    w[1, :32, 5] = float("nan")
    want_data, want_scales = oracle.quantize_mxfp8(w.float().numpy(), axis=1)
    q = quantize_mxfp8(w.to(device), axis=1)
    assert q.data.shape == w.shape and q.scales.shape == (groups, k // 32, n) and q.axis == 1
    assert np.array_equal(q.scales.cpu().numpy(), want_scales)
    _same_codes(q.data.view(torch.uint8).cpu().numpy(), want_data, want_scales, axis=1)
    want = torch.from_numpy(oracle.dequantize_mxfp8(want_data, want_scales, axis=1)).nan_to_num(nan=7.0)
    assert torch.equal(dequantize(q).float().cpu().nan_to_num(nan=7.0), want)
    round_trip = fake_quant(w.to(device), "mxfp8", axis=1)
    assert round_trip.dtype == dtype and torch.equal(round_trip.float().cpu().nan_to_num(nan=7.0), want)


def test_fake_quant_api_as_the_reference_tests_state_it(device):
    """``tests/cpu/kernels/test_quantization.py`` of the reference, on the device: storage shapes and dtypes (:29-35),
    round trip inside the format's tolerance (:57-64), axis 0 (:77-82), zeros (:87-93), scale order (:96-101), the
    divisibility guard (:127-135), the straight-through backward (:138-146), the input dtype kept (:149-151), and the
    weight cache: equal to the uncached result, reused until the version moves, straight-through (:154-183)."""
    from halo_amd.kernels.lowp.quantization import (cached_fake_quant, dequantize, fake_quant, quantize_mxfp8,
                                                    _weight_dequant_cache)

    def fro(a, b):
        return ((a.double() - b.double()).norm() / b.double().norm()).item()

    torch.manual_seed(0)
    x = (torch.randn(64, 256) * 0.5).to(device)
    q = quantize_mxfp8(x, axis=-1)
    assert q.data.shape == x.shape and q.data.dtype == torch.float8_e4m3fn
    assert q.scales.shape == (64, 256 // 32) and q.scales.dtype == torch.uint8
    recon = dequantize(q)
    assert recon.dtype == torch.bfloat16 and fro(recon, x) < 0.05
    x0 = (torch.randn(128, 96) * 0.3).to(device)
    q0 = quantize_mxfp8(x0, axis=0)
    assert q0.scales.shape == (128 // 32, 96) and fro(dequantize(q0), x0) < 0.05
    zeros = dequantize(quantize_mxfp8(torch.zeros(32, 64, device=device)))
    assert torch.isfinite(zeros).all() and zeros.abs().max().item() == 0.0
    small = quantize_mxfp8(torch.full((1, 32), 0.01, device=device)).scales.item()
    large = quantize_mxfp8(torch.full((1, 32), 100.0, device=device)).scales.item()
    assert large > small and large == 125
    with pytest.raises(ValueError, match="not divisible"):
        quantize_mxfp8(torch.randn(8, 30, device=device))
    with pytest.raises(ValueError, match="unknown block-scaled format"):
        fake_quant(x, "fp3")
    leaf = (torch.randn(64, 256) * 0.3).to(device).requires_grad_(True)
    y = fake_quant(leaf, "mxfp8", axis=-1)
    assert fro(y.detach(), leaf.detach()) < 0.05
    (y * 2.0).sum().backward()
    assert torch.equal(leaf.grad, torch.full_like(leaf.grad, 2.0))
    assert fake_quant((torch.randn(32, 64) * 0.2).bfloat16().to(device), "mxfp8").dtype == torch.bfloat16
    # a 3-D activation quantises along its last axis like the flattened rows
    x3 = torch.randn(4, 6, 64, device=device)
    assert torch.equal(fake_quant(x3, "mxfp8"), fake_quant(x3.reshape(24, 64), "mxfp8").reshape(4, 6, 64))

    w = torch.nn.Parameter((torch.randn(8, 64) * 0.3).to(device))
    cached = cached_fake_quant(w, "mxfp8", axis=-1)
    assert torch.equal(cached.detach(), fake_quant(w.detach(), "mxfp8", axis=-1))
    first = cached.detach().clone()
    entries = len(_weight_dequant_cache)
    assert torch.equal(first, cached_fake_quant(w, "mxfp8", axis=-1).detach()) and len(_weight_dequant_cache) == entries
    with torch.no_grad():
        w.add_(1.0)
    after = cached_fake_quant(w, "mxfp8", axis=-1).detach()
    assert not torch.equal(first, after) and fro(after, w.detach()) < 0.05
    w.grad = None
    (cached_fake_quant(w, "mxfp8", axis=-1) * 3.0).sum().backward()
    assert torch.equal(w.grad, torch.full_like(w.grad, 3.0))


GEMM_CASES = (
    # counts, K, N
    ((255, 256, 257, 0, 513, 31), 192, 264),   # row tiles that end inside a tile, an empty group, a partial column tile
    ((64,) * 16, 64, 1536),                    # one contraction step
    ((1, 0, 0, 700, 3), 2880, 136),            # 45 steps, tiny groups beside a large one
    ((300, 41), 256, 8),                       # one 16-byte output row
)


@pytest.mark.parametrize(("counts", "k", "n"), GEMM_CASES)
def test_mxfp8_expert_gemm_against_the_oracle_product(device, counts, k, n):
    """``expert_gemm(quant_format="mxfp8")`` on the scaled e4m3 matrix instruction against the float64 product of the
    oracle's round-tripped operands.  Every term is exact in either; the kernel accumulates in fp32 and rounds once to
    bf16, so the error is bf16's half ulp (2^-9 relative) plus the accumulation's, bounded here by 2^-8 of the
    element or 2^-8 of the root-sum-square of its terms' scale."""
    from halo_amd.kernels.expert_gemm import expert_gemm
    from oracle import mxfp8 as oracle

    g = torch.Generator().manual_seed(41)
    rows = sum(counts)
    a = (torch.randn(rows, k, generator=g) * torch.exp2(torch.randint(-6, 3, (rows, 1), generator=g).float())).bfloat16()
    b = (torch.randn(len(counts), k, n, generator=g) * 0.05).bfloat16()
    offs = torch.tensor(counts).cumsum(0).int()
    want = oracle.expert_gemm_mxfp8(a.float().numpy(), b.float().numpy(), offs.numpy())
    got = expert_gemm(a.to(device), b.to(device), offs=offs.to(device), quant_format="mxfp8", weight_cacheable=False)
    assert got.dtype == torch.bfloat16 and got.shape == (rows, n)
    err = np.abs(got.float().cpu().numpy().astype(np.float64) - want)
    group_of = np.repeat(np.arange(len(counts)), counts)
    spread = np.linalg.norm(a.float().numpy(), axis=1)[:, None] * np.linalg.norm(b.float().numpy(), axis=1)[group_of]
    assert (err <= 2.0 ** -8 * np.abs(want) + 2.0 ** -8 * spread / np.sqrt(k)).all()
    # the quantisation shows: against the unquantised product the error is the format's, not zero
    plain = np.zeros_like(want)
    start = 0
    for e, end in enumerate(offs.tolist()):
        plain[start:end] = a[start:end].double().numpy() @ b[e].double().numpy()
        start = end
    rel = np.linalg.norm(got.float().cpu().numpy() - plain) / np.linalg.norm(plain)
    assert 0.01 < rel < 0.08, rel


def test_mxfp8_expert_gemm_at_the_reference_band_shape_with_its_backward(device):
    """The reference's banded check (``tests/gpu/kernels/test_expert_gemm.py:55-74``: E = 8, M = 256, K = N = 2880,
    relative error against the bf16 product between 0.01 and 0.08, about 0.038 measured there; finite gradients), then
    the straight-through backward bit for bit: the gradients are ``grouped_mm``'s own over the two round-tripped
    operands."""
    from halo_amd.kernels.expert_gemm import expert_gemm
    from halo_amd.kernels.grouped_mm import grouped_mm, grouped_mm_grads
    from halo_amd.kernels.lowp.quantization import fake_quant

    torch.manual_seed(0)
    e, m, k, n = 8, 256, 2880, 2880
    x = (torch.randn(e * m, k, device=device, dtype=torch.bfloat16) * 0.3).requires_grad_(True)
    w = (torch.randn(e, k, n, device=device, dtype=torch.bfloat16) * 0.02).requires_grad_(True)
    offs = torch.arange(m, e * m + 1, m, device=device, dtype=torch.int32)
    out = expert_gemm(x, w, offs=offs, quant_format="mxfp8")
    upstream = torch.randn_like(out)
    (out * upstream).sum().backward()
    with torch.no_grad():
        plain = grouped_mm(x, w, offs=offs)
        rel = ((out.double() - plain.double()).norm() / plain.double().norm()).item()
        assert 0.03 < rel < 0.045, rel
        assert torch.isfinite(x.grad).all() and torch.isfinite(w.grad).all()
        xq, wq = fake_quant(x.detach(), "mxfp8", -1), fake_quant(w.detach(), "mxfp8", 1)
        simulated = grouped_mm(xq, wq, offs=offs)  # the reference's formulation: the same terms on the bf16 kernel
        assert ((out.double() - simulated.double()).norm() / simulated.double().norm()).item() < 2e-3
        grad_x, grad_w = grouped_mm_grads(xq, wq, upstream, offs, True, True)
        assert torch.equal(x.grad, grad_x) and torch.equal(w.grad, grad_w)


def test_mxfp8_expert_gemm_outside_the_matrix_kernel(device):
    """A contraction that ends in half a panel (K = 96) and fp32 operands take the reference's own formulation, the
    product of the two round-tripped operands on the bf16 / fp32 kernel; empty groups leave exact zeros in the weight
    gradient (``tests/gpu/kernels/test_grouped_mm_empty_groups.py:115-137``); rows fetched through the sort's index
    give the same bits as rows gathered first, and their gradient is summed back per token."""
    from halo_amd.kernels.expert_gemm import expert_gemm
    from halo_amd.kernels.grouped_mm import GatheredRows
    from halo_amd.kernels.moe_permute import build_inv_map
    from oracle import mxfp8 as oracle

    g = torch.Generator().manual_seed(43)
    counts = (40, 0, 70, 18)
    offs = torch.tensor(counts).cumsum(0).int()
    for dtype, k in ((torch.bfloat16, 96), (torch.float32, 128)):
        a = (torch.randn(sum(counts), k, generator=g) * 0.3).to(dtype)
        b = (torch.randn(len(counts), k, 72, generator=g) * 0.05).to(dtype)
        want = oracle.expert_gemm_mxfp8(a.float().numpy(), b.float().numpy(), offs.numpy())
        al, bl = a.to(device).requires_grad_(True), b.to(device).requires_grad_(True)
        got = expert_gemm(al, bl, offs=offs.to(device), quant_format="mxfp8")
        assert got.dtype == dtype
        tol = 2.0 ** -7 if dtype == torch.bfloat16 else 1e-5
        assert np.abs(got.detach().float().cpu().numpy() - want).max() <= tol * np.abs(want).max()
        (got * torch.randn(got.shape, generator=g).to(device)).sum().backward()
        assert torch.isfinite(al.grad).all() and torch.isfinite(bl.grad).all() and not bl.grad[1].any()
    tokens = torch.randn(40, 128, generator=g).bfloat16().to(device).requires_grad_(True)
    w = (torch.randn(4, 128, 64, generator=g) * 0.05).bfloat16().to(device)
    row_index = torch.arange(128, device=device) % 40
    inv_map = build_inv_map(row_index, 40, 4)
    dev_offs = offs.to(device)
    upstream = torch.randn(128, 64, generator=g).bfloat16().to(device)
    fetched = expert_gemm(GatheredRows(tokens, row_index, inv_map), w, offs=dev_offs, quant_format="mxfp8")
    (grad_fetched,) = torch.autograd.grad(fetched, tokens, upstream)
    copied = expert_gemm(tokens[row_index], w, offs=dev_offs, quant_format="mxfp8")
    (grad_copied,) = torch.autograd.grad(copied, tokens, upstream)
    assert torch.equal(fetched, copied)
    assert ((grad_fetched.double() - grad_copied.double()).norm() / grad_copied.double().norm()).item() < 5e-3


def test_projections_reading_the_same_rows_quantise_them_once(device, monkeypatch):
    """Gate and up stored apart read the same sorted rows: the second product takes the first one's e4m3 rows, and in
    backward the second weight gradient takes the first one's dequantised rows.  A change of the tensor in place (its
    version moves) or another tensor quantises again; the results equal the unshared ones bit for bit."""
    from halo_amd.kernels import expert_gemm as eg
    from halo_amd.kernels.lowp import quantization

    calls = {"quantise": 0, "dequantise": 0}
    real_q, real_d = quantization.quantize_rows_mxfp8, quantization.dequantize_rows_mxfp8

    def counting_q(*args, **kwargs):
        calls["quantise"] += 1
        return real_q(*args, **kwargs)

    def counting_d(*args, **kwargs):
        calls["dequantise"] += 1
        return real_d(*args, **kwargs)

    monkeypatch.setattr(quantization, "quantize_rows_mxfp8", counting_q)
    monkeypatch.setattr(quantization, "dequantize_rows_mxfp8", counting_d)
    g = torch.Generator().manual_seed(7)
    x = torch.randn(192, 128, generator=g).bfloat16().to(device).requires_grad_(True)
    w_gate = (torch.randn(3, 128, 64, generator=g) * 0.05).bfloat16().to(device).requires_grad_(True)
    w_up = (torch.randn(3, 128, 64, generator=g) * 0.05).bfloat16().to(device).requires_grad_(True)
    offs = torch.tensor([64, 64, 192], dtype=torch.int32, device=device)
    gate = eg.expert_gemm(x, w_gate, offs=offs, quant_format="mxfp8")
    up = eg.expert_gemm(x, w_up, offs=offs, quant_format="mxfp8")
    assert calls["quantise"] == 1
    (gate * up).sum().backward()
    assert calls["dequantise"] == 1
    shared = (gate.detach().clone(), up.detach().clone(), x.grad.clone(), w_gate.grad.clone(), w_up.grad.clone())
    with torch.no_grad():
        x.mul_(1.0)  # same values, the version counter moves
    again = eg.expert_gemm(x, w_up, offs=offs, quant_format="mxfp8")
    other = eg.expert_gemm(x.detach().clone(), w_up, offs=offs, quant_format="mxfp8")
    assert calls["quantise"] == 3 and torch.equal(again, up) and torch.equal(other, up)
    # unshared: every product on a tensor of its own
    x.grad = w_gate.grad = w_up.grad = None
    xa, xb = x.detach().clone().requires_grad_(True), x.detach().clone().requires_grad_(True)
    gate2 = eg.expert_gemm(xa, w_gate, offs=offs, quant_format="mxfp8")
    up2 = eg.expert_gemm(xb, w_up, offs=offs, quant_format="mxfp8")
    (gate2 * up2).sum().backward()
    assert torch.equal(gate2, shared[0]) and torch.equal(up2, shared[1]) and torch.equal(xa.grad + xb.grad, shared[2])
    assert torch.equal(w_gate.grad, shared[3]) and torch.equal(w_up.grad, shared[4])


@pytest.mark.parametrize("name", ("cfg2_small", "cfg4_small"))
def test_layer_with_mxfp8_experts_against_the_cpu_loop_over_fake_quantised_products(device, name):
    """``set_lowp_compute("mxfp8")`` on the layer (reference ``compute.py:53-58, 306-312``): forward and every
    gradient against the oracle's per-expert loop with both operands of each product round-tripped (straight-through
    backward); the weights are quantised once until they change.  Stored fused (rows fetched through the sort's index
    by the quantiser) and stored apart with biases.

    Tolerance: the layer keeps its intermediate tensors in bf16 and the oracle in fp32, and a quantiser sits behind
    them: a bf16 rounding (2^-9 relative) moves about 2 % of the GLU outputs across an e4m3 rounding boundary (spacing
    2^-3..2^-4 of the value), each by one step of about 9 %, which is 1.3 % of relative RMS error in the down
    projection's operand before any kernel error.  Hence a relative Frobenius error of 3 % and a cosine of 0.9995
    here, against 2 % elementwise and 0.9999 in the bf16 layer tests; the products themselves are held to 2^-8 in the
    GEMM tests above."""
    from halo_amd.kernels.lowp import quantization
    from halo_amd.kernels.router import SOFTMAX_ALL, SOFTMAX_TOPK, fused_topk_gate
    from oracle import moe_layer as oracle
    from oracle import mxfp8 as mx_oracle
    from oracle import router as router_oracle
    from tests import cases
    from tests.test_gpu_layer import _build_layer, cosine

    def _check(what, got, ref, tol):
        assert torch.isfinite(got).all(), what
        err = ((got.double().cpu() - ref.double()).norm() / ref.double().norm()).item()
        assert err <= tol and cosine(got, ref) >= 0.9995, (what, err, cosine(got, ref))

    # the gpt-oss shape with widths that are multiples of 32: 384 (whole panels, the matrix kernel) into 352 (half a
    # panel at the end: the down projection multiplies the round-tripped operands on the bf16 kernel)
    cfg = {"cfg2_small": cases.CONFIG2_SMALL, "cfg4_small": cases.CONFIG4_SMALL._replace(hidden=384, ffn=352)}[name]
    inputs = cases.make_layer_inputs(cfg)
    layer = _build_layer(cfg, inputs, device)
    assert layer.set_lowp_compute("mxfp8", weight_cacheable=True) is True
    with pytest.raises(ValueError, match="unknown block-scaled format"):
        layer.set_lowp_compute("fp3", weight_cacheable=True)
    x = inputs["x"].to(device).requires_grad_(True)
    result = layer(x)
    out = result[0] if isinstance(result, tuple) else result
    cached = len(quantization._weight_operand_cache)
    out.backward(inputs["grad_out"].to(device))
    with torch.no_grad():
        again = layer(x.detach())
    again = again[0] if isinstance(again, tuple) else again
    assert torch.equal(again, out.detach()) and len(quantization._weight_operand_cache) == cached >= 2

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
    tol = 3e-2
    _check("out", out, want.detach(), tol)
    _check("grad x", x.grad, rx.grad, tol)
    _check("grad router_weight", getattr(layer, layer._ROUTER_ATTR).weight.grad, wr.grad, tol)
    for pname in inputs["params"]:
        attr = pname.replace("gate_proj", "gate_proj_gmm").replace("up_proj", "up_proj_gmm") \
            if cfg.router == "softmax_topk" else pname
        _check(f"grad {pname}", getattr(layer, attr).grad, params[pname].grad, tol)
    # and the quantisation took place: the unquantised loop differs by the format's error
    with torch.no_grad():
        plain, _, _, _ = oracle.moe_layer_forward(rx.detach(), wr.detach(), {k: v.detach() for k, v in params.items()},
                                                  glu, cfg.top_k, router_bias=None if bias is None else bias.detach(),
                                                  mode=ref_mode, normalize=True, eps=0.0, indices=idx.cpu())
    rel = ((out.detach().double().cpu() - plain.double()).norm() / plain.double().norm()).item()
    assert 0.01 < rel < 0.1, rel
