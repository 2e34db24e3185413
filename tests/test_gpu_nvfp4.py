"""GPU parity tests for the NVFP4 expert path: the quantiser, dequantiser and fused round trip bit for bit against
``oracle.nvfp4`` (a restatement of the reference's eager ``quantize_nvfp4`` / ``dequantize``), the known answers the
reference's own tests hold, ``expert_gemm(quant_format="nvfp4")`` as the bf16 product of the two round-tripped operands
with the straight-through backward, and the layer with ``set_lowp_compute("nvfp4")`` against the CPU loop over
fake-quantised products."""

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _rows(rows, k, seed, dtype=torch.bfloat16):
    """Values over six binades (one scale per tensor: a wider spread only zeroes the small blocks) plus the blocks the
    rules turn on: all zero, the reference's amax-30 block, every level and tie of a block whose divisor is 1,
    negative zeros, a block far below the rest (its e4m3 scale underflows)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, k, generator=g) * torch.exp2(
        torch.randint(-3, 3, (rows, k // 16), generator=g).repeat_interleave(16, dim=1).float())
    x = x.to(dtype).float()
    x[0, :16] = 0
    x[1, :16] = 0; x[1, 0] = 30.0
    x[2, :16] = torch.tensor([6.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, -6.0, 0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, -0.0])
    x[3, :16] = torch.tensor([-6.0, -0.25, -0.75, -1.25, -1.75, -2.5, -3.5, -5.0, 0.7, 0.8, 2.4, 2.6, -0.1, 0.2, 5.5, 0.0])
    x[4, :16] = x[2, :16] * 2.0 ** -30
    return x.to(dtype)


def _equal_with_nan(got: torch.Tensor, want: np.ndarray):
    assert torch.equal(got.float().cpu().nan_to_num(nan=7.0), torch.from_numpy(want).nan_to_num(nan=7.0))


@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float32), ids=("bf16", "fp32"))
@pytest.mark.parametrize("k", (256, 48))
def test_row_quantiser_dequantiser_and_round_trip_equal_the_oracle_bit_for_bit(device, dtype, k):
    from halo_amd.kernels.lowp.quantization import dequantize, fake_quant, quantize_nvfp4
    from oracle import nvfp4 as oracle

    x = _rows(70, k, seed=31, dtype=dtype)
    if dtype == torch.float32:  # full fp32 mantissas: the divisions round as the reference's do
        x[8:] = x[8:] * (1 + torch.rand(x[8:].shape, generator=torch.Generator().manual_seed(2)) * 2 ** -9)
    want_data, want_scales, want_global = oracle.quantize_nvfp4(x.float().numpy())
    q = quantize_nvfp4(x.to(device))
    assert q.data.dtype == torch.uint8 and q.data.shape == (70, k // 2)
    assert q.scales.dtype == torch.float8_e4m3fn and q.scales.shape == (70, k // 16)
    assert q.block_size == 16 and q.axis == 1 and q.packed and not q.pow2_scale
    assert q.global_scale.dtype == torch.float32 and q.global_scale.numel() == 1
    assert float(q.global_scale) == float(want_global)
    assert np.array_equal(q.scales.view(torch.uint8).cpu().numpy(), want_scales)
    assert np.array_equal(q.data.cpu().numpy(), want_data)
    assert want_scales[0, 0] == 0 and want_scales[4, 0] == 0  # the zero block and the block that underflows e4m3
    restored = dequantize(q)
    assert restored.dtype == torch.bfloat16 and restored.shape == x.shape
    want = oracle.dequantize_nvfp4(want_data, want_scales, want_global)
    _equal_with_nan(restored, want)
    fused = fake_quant(x.to(device), "nvfp4")
    assert fused.dtype == dtype
    _equal_with_nan(fused, want)
    # a block whose divisor is exactly 1: the levels keep their codes and the ties go to the even code
    unit = torch.zeros(2, 16)
    unit[0] = _rows(8, 16, 1).float()[2]
    unit[1] = _rows(8, 16, 1).float()[3]
    unit = torch.cat([unit, torch.full((1, 16), 2688.0)])  # pins the tensor's scale at 1
    qu = quantize_nvfp4(unit.to(device))
    assert float(qu.global_scale) == 1.0 and qu.scales.float()[:2, 0].tolist() == [1.0, 1.0]
    codes = oracle.unpack_codes(qu.data.cpu().numpy())
    assert codes[0].tolist() == [7, 1, 2, 3, 4, 5, 6, 15, 0, 2, 2, 4, 4, 6, 6, 0]
    assert codes[1].tolist() == [15, 8, 10, 10, 12, 12, 14, 14, 1, 2, 4, 5, 8, 0, 7, 0]


@pytest.mark.parametrize(("groups", "k", "n", "dtype"), ((3, 96, 136, torch.bfloat16), (2, 128, 130, torch.bfloat16),
                                                         (2, 48, 264, torch.float32)))
def test_weight_quantiser_equals_the_oracle_bit_for_bit(device, groups, k, n, dtype):
    """``quantize_nvfp4(w, axis=1)`` of an ``[E, K, N]`` bank under one scale: codes, scales, the tensor's scale and the
    round trip; a contraction that ends inside a tile, a column count that is no multiple of eight, fp32 masters."""
    from halo_amd.kernels.lowp.quantization import dequantize, fake_quant, quantize_nvfp4
    from oracle import nvfp4 as oracle

    g = torch.Generator().manual_seed(9)
    w = (torch.randn(groups, k, n, generator=g) * torch.exp2(torch.randint(-4, 2, (groups, 1, n), generator=g).float()))
    w = w.to(dtype)
    w[0, :16, 0] = 0
    w[0, 16:32, 1] = 0
    w[0, 20, 1] = 6.0
    want_data, want_scales, want_global = oracle.quantize_nvfp4(w.float().numpy(), axis=1)
    q = quantize_nvfp4(w.to(device), axis=1)
    assert q.data.shape == (groups, k // 2, n) and q.scales.shape == (groups, k // 16, n) and q.axis == 1 and q.packed
    assert float(q.global_scale) == float(want_global)
    assert np.array_equal(q.scales.view(torch.uint8).cpu().numpy(), want_scales)
    assert np.array_equal(q.data.cpu().numpy(), want_data)
    want = oracle.dequantize_nvfp4(want_data, want_scales, want_global, axis=1)
    _equal_with_nan(dequantize(q), want)
    round_trip = fake_quant(w.to(device), "nvfp4", axis=1)
    assert round_trip.dtype == dtype
    _equal_with_nan(round_trip, want)
    moved = quantize_nvfp4(w.to(device).permute(1, 0, 2).contiguous(), axis=0)
    assert moved.data.shape == (k // 2, groups, n) and torch.equal(moved.data.permute(1, 0, 2), q.data)
    _equal_with_nan(dequantize(moved).permute(1, 0, 2), want)


def test_fake_quant_api_as_the_reference_tests_state_it(device):
    """``tests/cpu/kernels/test_quantization.py`` of the reference, on the device: storage shapes and dtypes (:37-45),
    round trip inside the format's tolerance with mxfp8 the more accurate (:58-71), zeros (:82-89), an outlier above
    6 * 448 kept finite (:116-124), the divisibility guard (:127-135), the straight-through backward (:138-146), the
    input dtype kept (:149-151), the weight cache (:154-183); and of ``tests/cpu/kernels/test_block_scale_oracle.py``:
    the two-level scale (:97-116), the error independent of the magnitude (:118-137), a shard quantised alone equal to
    its slice of the bank (:157-172), an inf or a NaN never absorbed and finite inputs never non-finite (:175-196)."""
    import math

    from halo_amd.kernels.lowp.quantization import (QUANTIZERS, cached_fake_quant, dequantize, fake_quant,
                                                    quantize_mxfp8, quantize_nvfp4)

    def fro(a, b):
        return ((a.double() - b.double()).norm() / b.double().norm()).item()

    assert sorted(QUANTIZERS) == ["mxfp4", "mxfp8", "nvfp4"]
    torch.manual_seed(0)
    x = (torch.randn(64, 256) * 0.5).to(device)
    q = quantize_nvfp4(x, axis=-1)
    assert q.data.shape == (64, 128) and q.data.dtype == torch.uint8
    assert q.scales.shape == (64, 16) and q.scales.dtype == torch.float8_e4m3fn and q.packed and not q.pow2_scale
    assert q.global_scale is not None and q.global_scale.numel() == 1 and q.global_scale.dtype == torch.float32
    recon = dequantize(q)
    assert recon.dtype == torch.bfloat16 and fro(dequantize(quantize_mxfp8(x)), x) < fro(recon, x) < 0.25
    zeros = dequantize(quantize_nvfp4(torch.zeros(32, 64, device=device)))
    assert torch.isfinite(zeros).all() and zeros.abs().max().item() == 0.0
    block = torch.zeros(16)
    block[0] = 30.0
    b = quantize_nvfp4(block.to(device))
    assert b.global_scale.item() == 2.0 ** math.ceil(math.log2(30.0 / (448.0 * 6.0))) and b.scales.float().item() == 320.0
    assert abs(float(dequantize(b)[0]) - 30.0) < 1e-3
    outlier = torch.randn(16, 64) * 0.1
    outlier[0, 0] = 5000.0
    qo = quantize_nvfp4(outlier.to(device))
    assert torch.isfinite(qo.scales.float()).all() and torch.isfinite(dequantize(qo)).all()
    with pytest.raises(ValueError, match="not divisible"):
        quantize_nvfp4(torch.randn(8, 24, device=device))
    base = torch.randn(128, 256).double()
    errs = []
    for exponent in range(4, -32, -4):
        scaled = (base * 10.0 ** exponent).float().to(device)
        errs.append(fro(dequantize(quantize_nvfp4(scaled)), scaled))
    assert max(errs) - min(errs) < 0.02 and 0.04 < errs[0] < 0.25
    bank = torch.randn(8, 64, 256) * 0.02
    bank[0] *= 1e-3
    bank = bank.to(device)
    gathered = dequantize(quantize_nvfp4(bank, axis=-1))
    sharded = torch.cat([dequantize(quantize_nvfp4(s, axis=-1)) for s in bank.chunk(4, dim=0)], dim=0)
    assert torch.equal(sharded, gathered)
    for poison in (float("nan"), float("inf"), float("-inf")):
        bad = torch.randn(4, 64) * 0.3
        bad[1, 7] = poison
        assert not torch.isfinite(dequantize(quantize_nvfp4(bad.to(device)))).all()
    fine = torch.randn(4, 64) * 0.3
    fine[0, 0] = 5e4
    fine[2, :] = 0.0
    assert torch.isfinite(dequantize(quantize_nvfp4(fine.to(device)))).all()

    leaf = (torch.randn(64, 256) * 0.3).to(device).requires_grad_(True)
    y = fake_quant(leaf, "nvfp4", axis=-1)
    assert fro(y.detach(), leaf.detach()) < 0.25
    assert torch.equal(y.detach().bfloat16(), dequantize(quantize_nvfp4(leaf.detach())))
    (y * 2.0).sum().backward()
    assert torch.equal(leaf.grad, torch.full_like(leaf.grad, 2.0))
    assert fake_quant((torch.randn(32, 64) * 0.2).bfloat16().to(device), "nvfp4").dtype == torch.bfloat16
    w = torch.nn.Parameter((torch.randn(8, 64) * 0.3).to(device))
    cached = cached_fake_quant(w, "nvfp4", axis=-1)
    assert torch.equal(cached.detach(), fake_quant(w.detach(), "nvfp4", axis=-1))
    first = cached.detach().clone()
    assert torch.equal(first, cached_fake_quant(w, "nvfp4", axis=-1).detach())
    with torch.no_grad():
        w.add_(1.0)
    after = cached_fake_quant(w, "nvfp4", axis=-1).detach()
    assert not torch.equal(first, after) and fro(after, w.detach()) < 0.25
    (cached_fake_quant(w, "nvfp4", axis=-1) * 3.0).sum().backward()
    assert torch.equal(w.grad, torch.full_like(w.grad, 3.0))


def test_nvfp4_expert_gemm_is_the_product_of_the_round_tripped_operands(device):
    """``expert_gemm(quant_format="nvfp4")`` (reference ``expert_gemm.py:33-38``): bit-equal to ``grouped_mm`` over the
    two ``fake_quant`` results, forward and both gradients (the straight-through estimator hands ``grouped_mm``'s own
    gradients through); within the kernel's bound of the oracle's float64 product; an empty group leaves exact zeros in
    the weight gradient; rows handed over as (tokens, index) give the bits of the gathered copy; at the reference's band
    shape the error against the bf16 product lies in its band for this format, 0.04-0.25
    (``tests/gpu/kernels/test_expert_gemm.py:55-74``)."""
    from halo_amd.kernels.expert_gemm import expert_gemm
    from halo_amd.kernels.grouped_mm import GatheredRows, grouped_mm, grouped_mm_grads
    from halo_amd.kernels.lowp.quantization import fake_quant
    from halo_amd.kernels.moe_permute import build_inv_map
    from oracle import nvfp4 as oracle

    g = torch.Generator().manual_seed(43)
    counts = (255, 0, 257, 40, 513, 31)
    offs = torch.tensor(counts).cumsum(0).int()
    for dtype, k, n in ((torch.bfloat16, 192, 264), (torch.float32, 96, 72)):
        a = (torch.randn(sum(counts), k, generator=g) * 0.5).to(dtype)
        b = (torch.randn(len(counts), k, n, generator=g) * 0.05).to(dtype)
        want = oracle.expert_gemm_nvfp4(a.float().numpy(), b.float().numpy(), offs.numpy())
        al, bl = a.to(device).requires_grad_(True), b.to(device).requires_grad_(True)
        dev_offs = offs.to(device)
        got = expert_gemm(al, bl, offs=dev_offs, quant_format="nvfp4", weight_cacheable=False)
        assert got.dtype == dtype and got.shape == (sum(counts), n)
        upstream = torch.randn(got.shape, generator=g).to(dtype).to(device)
        got.backward(upstream)
        with torch.no_grad():
            aq, bq = fake_quant(al.detach(), "nvfp4", -1), fake_quant(bl.detach(), "nvfp4", 1)
            assert torch.equal(got, grouped_mm(aq, bq, offs=dev_offs))
            grad_a, grad_b = grouped_mm_grads(aq, bq, upstream, dev_offs, True, True)
            assert torch.equal(al.grad, grad_a) and torch.equal(bl.grad, grad_b) and not bl.grad[1].any()
        tol = 2.0 ** -7 if dtype == torch.bfloat16 else 1e-5
        assert np.abs(got.detach().float().cpu().numpy() - want).max() <= tol * np.abs(want).max()
    tokens = torch.randn(40, 128, generator=g).bfloat16().to(device).requires_grad_(True)
    w = (torch.randn(4, 128, 64, generator=g) * 0.05).bfloat16().to(device)
    row_index = torch.arange(128, device=device) % 40
    inv_map = build_inv_map(row_index, 40, 4)
    small_offs = torch.tensor([40, 40, 110, 128], dtype=torch.int32, device=device)
    fetched = expert_gemm(GatheredRows(tokens, row_index, inv_map), w, offs=small_offs, quant_format="nvfp4")
    copied = expert_gemm(tokens[row_index], w, offs=small_offs, quant_format="nvfp4")
    assert torch.equal(fetched, copied)
    torch.manual_seed(0)
    e, m, k, n = 8, 256, 2880, 2880
    x = (torch.randn(e * m, k, device=device, dtype=torch.bfloat16) * 0.3).requires_grad_(True)
    wb = (torch.randn(e, k, n, device=device, dtype=torch.bfloat16) * 0.02).requires_grad_(True)
    band_offs = torch.arange(m, e * m + 1, m, device=device, dtype=torch.int32)
    out = expert_gemm(x, wb, offs=band_offs, quant_format="nvfp4")
    (out * torch.randn_like(out)).sum().backward()
    with torch.no_grad():
        plain = grouped_mm(x, wb, offs=band_offs)
        rel = ((out.double() - plain.double()).norm() / plain.double().norm()).item()
    assert 0.04 < rel < 0.25, rel
    assert torch.isfinite(x.grad).all() and torch.isfinite(wb.grad).all()


@pytest.mark.parametrize("name", ("cfg2_small", "cfg4_small"))
def test_layer_with_nvfp4_experts_against_the_cpu_loop_over_fake_quantised_products(device, name):
    """``set_lowp_compute("nvfp4")`` on the layer (reference ``compute.py:53-58, 306-312``): forward and every gradient
    against the oracle's per-expert loop with both operands of each product round-tripped (straight-through backward).
    The loop quantises an expert's rows on their own and the layer all sorted rows as one tensor; the two agree
    because the tensor's scale is a power of two, under which the e4m3 block scales do not move (the property the
    reference tests for expert shards).  Tolerance as for MXFP4 (a 4-bit quantiser behind bf16 intermediates): 6 %
    Frobenius, cosine 0.998."""
    from halo_amd.kernels.router import SOFTMAX_ALL, SOFTMAX_TOPK, fused_topk_gate
    from oracle import moe_layer as oracle
    from oracle import nvfp4 as nv_oracle
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
    assert layer.set_lowp_compute("nvfp4", weight_cacheable=True) is True
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
                                             normalize=True, eps=0.0, indices=idx.cpu(), quant=nv_oracle.fake_quant_ste)
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
