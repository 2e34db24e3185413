"""Pins ``oracle.glu``, ``oracle.grouped_mm``, ``oracle.router``, ``oracle.block_fp8``, ``oracle.mxfp8``,
``oracle.mxfp4``, ``oracle.nvfp4`` and ``oracle.moe_layer`` against
library routines (torch autograd, matmul, softmax, topk, the float8 cast), identities and brute force."""

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import block_fp8, glu, grouped_mm, moe_layer, mxfp4, mxfp8, nvfp4, router

PROBE = (-64.0, -8.0, -1.0, -0.5, -1e-3, 0.0, 1e-3, 0.5, 1.0, 8.0, 64.0)  # fused_glu.py:33 of the reference

VARIANTS = {
    "silu": (dict(activation=glu.SILU), lambda g, u: F.silu(g) * u),
    "gelu_tanh": (dict(activation=glu.GELU_TANH), lambda g, u: F.gelu(g, approximate="tanh") * u),
    "clamped_silu": (dict(activation=glu.CLAMPED_SILU, limit=2.5),
                     lambda g, u: F.silu(g.clamp(max=2.5)) * u.clamp(-2.5, 2.5)),
    "silu_then_clamp": (dict(activation=glu.CLAMPED_SILU, limit=2.5, clamp_activated=True),
                        lambda g, u: F.silu(g).clamp(max=2.5) * u.clamp(-2.5, 2.5)),
    "gptoss": (dict(activation=glu.CLAMPED_SILU, alpha=1.702, limit=7.0, up_plus_one=True),
               lambda g, u: (u.clamp(-7, 7) + 1) * (g.clamp(max=7) * torch.sigmoid(g.clamp(max=7) * 1.702))),
}


@pytest.mark.parametrize("name", VARIANTS)
def test_glu_forward_and_gradients_match_autograd(name):
    kwargs, eager = VARIANTS[name]
    g = torch.Generator().manual_seed(0)
    gate = torch.cat([torch.randn(500, generator=g) * 4, torch.tensor(PROBE)]).double()
    up = torch.cat([torch.randn(500, generator=g) * 4, torch.tensor(PROBE[::-1])]).double()
    dout = torch.randn(gate.shape, generator=g).double()
    gl, ul = gate.clone().requires_grad_(True), up.clone().requires_grad_(True)
    want = eager(gl, ul)
    want.backward(dout)
    assert torch.allclose(glu.glu_forward(gate, up, **kwargs), want.detach(), rtol=1e-13, atol=1e-13)
    dgate, dup = glu.glu_backward(gate, up, dout, **kwargs)
    assert torch.allclose(dgate, gl.grad, rtol=1e-12, atol=1e-12)
    assert torch.allclose(dup, ul.grad, rtol=1e-12, atol=1e-12)


def test_glu_clamp_gradient_passes_at_the_bound():
    # torch's clamp passes the gradient on the closed interval; so must the closed forms
    limit = 2.0
    gate = torch.tensor([limit, limit, -limit, 0.5], dtype=torch.float64)
    up = torch.tensor([limit, -limit, limit, limit], dtype=torch.float64)
    dout = torch.ones(4, dtype=torch.float64)
    dgate, dup = glu.glu_backward(gate, up, dout, glu.CLAMPED_SILU, limit=limit)
    assert (dgate != 0).all() and (dup != 0).all()
    dgate_hi, dup_hi = glu.glu_backward(gate + 1e-9, up * (1 + 1e-9), dout, glu.CLAMPED_SILU, limit=limit)
    assert dgate_hi[0] == 0 and dup_hi[0] == 0  # just past the bound the gradient is cut


def test_glu_identity_gptoss_alpha1_minus_clamped_silu_is_silu_of_clamped_gate():
    g = torch.Generator().manual_seed(1)
    gate, up = torch.randn(300, generator=g).double() * 5, torch.randn(300, generator=g).double() * 5
    a = glu.glu_forward(gate, up, glu.CLAMPED_SILU, alpha=1.0, limit=3.0, up_plus_one=True)
    b = glu.glu_forward(gate, up, glu.CLAMPED_SILU, limit=3.0)
    assert torch.allclose(a - b, F.silu(gate.clamp(max=3.0)), atol=1e-12)


def test_glu_bf16_is_fp32_math_rounded_once():
    g = torch.Generator().manual_seed(2)
    gate, up = torch.randn(256, generator=g).bfloat16(), torch.randn(256, generator=g).bfloat16()
    want = (F.silu(gate.float()) * up.float()).bfloat16()
    assert torch.equal(glu.glu_forward(gate, up, glu.SILU), want)


# ------------------------------------------------------------------------------------------------ grouped GEMM

@pytest.mark.parametrize("counts", ((7, 33, 0, 1, 64, 0), (0, 0, 0, 0, 105, 0), (5, 5, 5)))
def test_grouped_mm_matches_matmul_and_autograd(counts):
    torch.manual_seed(0)
    total, k, n = sum(counts), 24, 20
    a = torch.randn(total, k, dtype=torch.float64, requires_grad=True)
    b = torch.randn(len(counts), k, n, dtype=torch.float64, requires_grad=True)
    offs = np.cumsum(counts).astype(np.int32)
    pieces, start = [], 0
    for e, c in enumerate(counts):
        pieces.append(a[start:start + c] @ b[e])
        start += c
    want = torch.cat(pieces)
    dout = torch.randn(total, n, dtype=torch.float64)
    want.backward(dout)
    kw = dict(acc_dtype=torch.float64)
    assert torch.allclose(grouped_mm.grouped_mm(a.detach(), b.detach(), offs, **kw), want.detach(), atol=1e-12)
    assert torch.allclose(grouped_mm.grouped_mm_dgrad(dout, b.detach(), offs, **kw), a.grad, atol=1e-12)
    wgrad = grouped_mm.grouped_mm_wgrad(a.detach(), dout, offs, **kw)
    assert torch.allclose(wgrad, b.grad, atol=1e-12)
    for e, c in enumerate(counts):
        assert (c == 0) == (not wgrad[e].any())


# ------------------------------------------------------------------------------------------------------ router

def test_router_selection_ties_go_to_the_lower_index():
    logits = torch.tensor([[1.0, 1.0, 0.5, 1.0], [0.0, 2.0, 2.0, -1.0], [3.0, 3.0, 3.0, 3.0]])
    assert router.select_topk(logits, 2).tolist() == [[0, 1], [1, 2], [0, 1]]
    assert router.select_topk(logits, 3).tolist() == [[0, 1, 3], [1, 2, 0], [0, 1, 2]]


def test_router_matches_torch_topk_on_tie_free_rows_and_in_bf16_ties():
    g = torch.Generator().manual_seed(0)
    logits = torch.randn(512, 64, generator=g)
    idx, w = router.route(logits, 8, router.SOFTMAX_ALL, normalize=True, eps=0.0)
    probs = torch.softmax(logits, dtype=torch.float, dim=-1)
    top_v, top_i = torch.topk(probs, 8, dim=-1)
    assert torch.equal(idx, top_i)
    assert torch.equal(w, top_v / top_v.sum(-1, keepdim=True))
    # bf16 logits tie often: selection must still be descending, lower index first among equals
    lb = (torch.randn(2048, 128, generator=g) * 0.9).bfloat16()
    idx_b, w_b = router.route(lb, 8)
    picked = lb.float().gather(-1, idx_b)
    assert (picked[:, :-1] >= picked[:, 1:]).all()
    same = picked[:, :-1] == picked[:, 1:]
    assert same.any(), "the case should contain ties"
    assert (idx_b[:, :-1][same] < idx_b[:, 1:][same]).all()
    kth = picked[:, -1:]
    rest = lb.float().scatter(-1, idx_b, float("-inf"))
    assert (rest <= kth).all()
    tied_out = (rest == kth)
    cols = torch.arange(128).expand_as(rest)
    last_in = torch.where(picked == kth, idx_b, -1).max(-1, keepdim=True).values
    assert (cols[tied_out] > last_in.expand_as(rest)[tied_out]).all()  # an excluded equal score sits at a higher index
    assert w_b.dtype == torch.float32 and torch.equal(w_b, w_b.bfloat16().float())  # bf16 values stored in fp32


def test_router_gptoss_mode_and_backward():
    g = torch.Generator().manual_seed(1)
    logits = torch.randn(64, 32, generator=g)
    idx, w = router.route(logits, 4, router.SOFTMAX_TOPK)
    top_v, top_i = torch.topk(logits, 4, dim=-1)
    assert torch.equal(idx, top_i) and torch.allclose(w, torch.softmax(top_v, dim=-1))
    gw = torch.randn(64, 4, generator=g)
    for mode, norm in ((router.SOFTMAX_ALL, True), (router.SOFTMAX_ALL, False), (router.SOFTMAX_TOPK, False)):
        leaf = logits.clone().requires_grad_(True)
        if mode == router.SOFTMAX_TOPK:
            ww = torch.softmax(leaf.gather(-1, idx), dim=-1)
        else:
            ww = torch.softmax(leaf, dim=-1).gather(-1, idx)
            if norm:
                ww = ww / ww.sum(-1, keepdim=True)
        ww.backward(gw)
        got = router.route_backward(logits, idx, gw, mode, norm, 0.0)
        assert torch.allclose(got, leaf.grad, rtol=1e-4, atol=1e-6)


# ------------------------------------------------------------------------------------------------- block fp8

def test_e4m3_encoder_matches_torch_cast_on_every_code_and_on_random_values():
    codes = np.arange(256, dtype=np.uint8)
    finite = (codes & 0x7F) != 0x7F
    decoded = block_fp8.decode_e4m3fn(codes[finite])
    want = torch.from_numpy(codes[finite]).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(decoded, want)
    assert np.array_equal(block_fp8.encode_e4m3fn(decoded) & 0x7F, codes[finite] & 0x7F)
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(20000, generator=g) * torch.rand(20000, generator=g) * 300).clamp(-448, 448)
    x = torch.cat([x, torch.tensor([0.0, 2.0**-9, 2.0**-10, 3 * 2.0**-10, 448.0, -448.0, 0.0009765625 * 1.5])])
    got = block_fp8.encode_e4m3fn(x.numpy())
    want = x.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    nz = (want & 0x7F) != 0
    assert np.array_equal(got[nz], want[nz]) and not (got[~nz] & 0x7F).any()


def _diagnostic(w):
    # the formula the reference's own test holds (tests/cpu/weight_sync/test_block_fp8.py:13-21)
    n, k = w.shape
    x = F.pad(w.float(), (0, (-k) % 128, 0, (-n) % 128))
    xb = x.reshape(x.shape[0] // 128, 128, x.shape[1] // 128, 128)
    amax = xb.abs().amax(dim=(1, 3), keepdim=True).clamp_min(1e-12)
    scale = torch.exp2(torch.ceil(torch.log2(amax / 448.0)))
    q = (xb / scale).clamp(-448, 448).to(torch.float8_e4m3fn).reshape(x.shape)[:n, :k].contiguous()
    return q.view(torch.uint8).numpy(), scale[:, 0, :, 0].numpy()


@pytest.mark.parametrize("shape", [(128, 128), (256, 384), (200, 130), (5, 7), (512, 64)])
def test_block_quantiser_matches_the_diagnostic_formula(shape):
    torch.manual_seed(0)
    weight = (torch.randn(shape) * torch.rand(shape).mul(4)).bfloat16()
    q, scale = block_fp8.quantize_block_fp8(weight.float().numpy())
    ref_q, ref_scale = _diagnostic(weight)
    assert np.array_equal(scale, ref_scale)
    same = (q & 0x7F) == (ref_q & 0x7F)
    assert same.all() and np.array_equal(q[(q & 0x7F) != 0], ref_q[(q & 0x7F) != 0])


def test_block_quantiser_boundary_zero_block_and_leading_dims():
    w = np.zeros((128, 256), dtype=np.float32)
    w[0, 0] = 448.0 * 4
    w[0, 128] = 448.0 * 4 * 1.0001
    q, scale = block_fp8.quantize_block_fp8(w)
    assert scale.tolist() == [[4.0, 8.0]]
    q0, s0 = block_fp8.quantize_block_fp8(np.zeros((128, 128), dtype=np.float32))
    assert np.isfinite(s0).all() and (s0 > 0).all() and not (q0 & 0x7F).any()
    rng = np.random.default_rng(2)
    bank = rng.standard_normal((3, 130, 129)).astype(np.float32)
    qb, sb = block_fp8.quantize_block_fp8(bank)
    assert qb.shape == bank.shape and sb.shape == (3, 2, 2)
    for e in range(3):
        q1, s1 = block_fp8.quantize_block_fp8(bank[e])
        assert np.array_equal(qb[e], q1) and np.array_equal(sb[e], s1)
    restored = block_fp8.dequantize_block_fp8(qb, sb)
    assert (np.abs(restored - bank) <= np.abs(bank) * 0.0625 + sb.max() * 2.0**-9).all()


# --------------------------------------------------------------------------------------------------- MoE layer

@pytest.mark.parametrize("fused", (True, False))
@pytest.mark.parametrize("kind", ("silu", "gptoss"))
def test_layer_loop_matches_the_dense_formula(fused, kind):
    g = torch.Generator().manual_seed(3)
    T, H, E, K, Fw = 11, 8, 3, 2, 6
    x = torch.randn(T, H, dtype=torch.float64, generator=g)
    experts = torch.randint(-1, 5, (T, K), generator=g)  # -1 padding, 3..4 not local
    weights = torch.rand(T, K, dtype=torch.float64, generator=g)
    params = {"down_proj": torch.randn(E, Fw, H, dtype=torch.float64, generator=g)}
    if fused:
        params["gate_up_proj"] = torch.randn(E, H, 2 * Fw, dtype=torch.float64, generator=g)
    else:
        params["gate_proj"] = torch.randn(E, H, Fw, dtype=torch.float64, generator=g)
        params["up_proj"] = torch.randn(E, H, Fw, dtype=torch.float64, generator=g)
        params["gate_proj_bias"] = torch.randn(E, Fw, dtype=torch.float64, generator=g)
        params["down_proj_bias"] = torch.randn(E, H, dtype=torch.float64, generator=g)
    combine = moe_layer.Glu(kind, 1.702, 7.0) if kind == "gptoss" else moe_layer.Glu(kind)
    got = moe_layer.compute_experts_loop(x, experts, weights, params, combine, E)
    want = moe_layer.dense_formula(x, experts, weights, params, combine, E)
    assert torch.allclose(got, want, atol=1e-10)


def test_layer_grouped_on_cpu_matches_the_loop_and_the_dense_formula():
    """The grouped-on-CPU variant (sort, ``F.grouped_mm``, weighted sum) against the per-expert loop and the slot-by-
    slot formula: output and every gradient, with -1 padding, a non-local id and an expert without rows."""
    g = torch.Generator().manual_seed(6)
    T, H, E, K, Fw = 24, 16, 4, 3, 8
    experts = torch.randint(-1, 4, (T, K), generator=g)
    experts[experts == 2] = 5  # expert 2 gets nothing; 5 is not local
    weights = torch.rand(T, K, generator=g)
    base = {"x": torch.randn(T, H, generator=g), "gate_up_proj": torch.randn(E, H, 2 * Fw, generator=g) * 0.3,
            "down_proj": torch.randn(E, Fw, H, generator=g) * 0.3}
    upstream = torch.randn(T, H, generator=g)
    runs = []
    for fn in (moe_layer.compute_experts_grouped, moe_layer.compute_experts_loop):
        leaves = {k: v.clone().requires_grad_(True) for k, v in base.items()}
        params = {k: v for k, v in leaves.items() if k != "x"}
        out = fn(leaves["x"], experts, weights, params, moe_layer.Glu(), E)
        out.backward(upstream)
        runs.append([out.detach()] + [leaves[k].grad for k in ("x", "gate_up_proj", "down_proj")])
    for a, b in zip(*runs):
        assert torch.allclose(a, b, atol=1e-5, rtol=1e-5)
    assert not runs[0][3][2].any()  # the idle expert's weight gradient is exact zeros
    want = moe_layer.dense_formula(base["x"], experts, weights, {k: v for k, v in base.items() if k != "x"},
                                   moe_layer.Glu(), E)
    assert torch.allclose(runs[0][0], want, atol=1e-5)


def test_layer_forward_routes_and_adds_the_shared_expert():
    g = torch.Generator().manual_seed(4)
    T, H, E, K, Fw = 16, 8, 4, 2, 6
    x = torch.randn(T, H, generator=g)
    wr = torch.randn(E, H, generator=g)
    params = {"gate_up_proj": torch.randn(E, H, 2 * Fw, generator=g) * 0.1,
              "down_proj": torch.randn(E, Fw, H, generator=g) * 0.1}
    shared = {"gate_proj": torch.randn(Fw, H, generator=g), "up_proj": torch.randn(Fw, H, generator=g),
              "down_proj": torch.randn(H, Fw, generator=g), "shared_expert_gate": torch.randn(1, H, generator=g)}
    out, logits, idx, w = moe_layer.moe_layer_forward(x, wr, params, moe_layer.Glu(), K, shared=shared)
    routed, *_ = moe_layer.moe_layer_forward(x, wr, params, moe_layer.Glu(), K)
    mlp = F.linear(F.silu(F.linear(x, shared["gate_proj"])) * F.linear(x, shared["up_proj"]), shared["down_proj"])
    assert torch.allclose(out - routed, mlp * torch.sigmoid(x @ shared["shared_expert_gate"].t()), atol=1e-5)
    assert torch.equal(idx, torch.topk(torch.softmax(logits, -1), K).indices)
    assert torch.allclose(w.sum(-1), torch.ones(T))


def test_row_quantiser_picks_the_smallest_power_of_two_that_fits_and_keeps_e4m3_precision():
    """Pins ``quantize_rows_fp8`` by what defines it rather than by its formula: the scale is a power of two under
    which the block's largest magnitude is at most 448 and above 224 (one step smaller would overflow), the codes are
    what torch's own float8_e4m3fn cast gives for the scaled values, and ``q * scale`` is within half an e4m3 step
    (2^-4 relative for normal values) of ``x``."""
    g = torch.Generator().manual_seed(11)
    x = (torch.randn(64, 512, generator=g) * torch.exp2(torch.randint(-12, 12, (64, 4), generator=g)
                                                        .repeat_interleave(128, dim=1).float())).bfloat16().float()
    x[0, :128] = 0
    x[1, :128] = 0
    x[1, 3] = 448.0  # exactly at the top of the range: scale 1
    x[2, :128] = 0
    x[2, 3] = 449.0  # bf16 rounds this to 448 too
    x[3, :128] = 0
    x[3, 3] = 452.0  # the next bf16 value above 448: scale 2
    q, exps_t = block_fp8.quantize_rows_fp8(x.numpy())
    exps = exps_t.T.astype(np.int64)
    assert exps_t.shape == (4, 64) and exps[0, 0] == 0 and exps[1, 0] == 127 and exps[3, 0] == 128
    amax = x.abs().reshape(64, 4, 128).amax(dim=2).double().numpy()
    scale = np.ldexp(1.0, exps - 127)
    live = amax > 0
    assert (amax[live] / scale[live] <= 448).all() and (amax[live] / scale[live] > 224).all()
    scaled = (x.double().reshape(64, 4, 128) / torch.from_numpy(scale)[:, :, None]).reshape(64, 512).float()
    torch_bits = scaled.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    nonzero = (q & 0x7F) != 0
    assert np.array_equal(q[nonzero], torch_bits[nonzero]) and not (torch_bits[~nonzero] & 0x7F).any()
    restored = block_fp8.dequantize_rows_fp8(q, exps_t)
    step = np.repeat(scale, 128, axis=1) * 2.0 ** -9  # half the subnormal spacing (2^-9) in the block's scale
    assert (np.abs(restored - x.double().numpy()) <= np.maximum(np.abs(x.double().numpy()) * 2.0 ** -4, step)).all()


def test_fp8_product_of_the_oracle_is_the_product_of_its_dequantised_operands():
    """``fp8_grouped_mm`` against a per-element restatement on a tiny case (two experts, K = 256): the sum over k of
    code value times row scale times code value times block scale, term by term in Python floats."""
    g = torch.Generator().manual_seed(12)
    x = torch.randn(5, 256, generator=g).bfloat16().float().numpy()
    w = (torch.randn(2, 256, 136, generator=g) * 0.02).numpy()
    q, exps_t = block_fp8.quantize_rows_fp8(x)
    wq, ws = block_fp8.quantize_block_fp8(w)
    ws = ws * np.float32(1.25)
    got = block_fp8.fp8_grouped_mm(q, exps_t, wq, ws, np.array([2, 5], dtype=np.int32))
    qa, qw = block_fp8.decode_e4m3fn(q).astype(float), block_fp8.decode_e4m3fn(wq).astype(float)
    for r, c in ((0, 0), (1, 135), (2, 7), (4, 130)):
        expert = 0 if r < 2 else 1
        total = 0.0
        for kk in range(256):
            total += qa[r, kk] * 2.0 ** (int(exps_t[kk // 128, r]) - 127) * qw[expert, kk, c] * float(ws[expert, kk // 128, c // 128])
        assert abs(got[r, c] - total) <= 1e-12 * max(1.0, abs(total))


# ----------------------------------------------------------------------------------------------------------- mxfp8
def _mx_blocks(seed=21):
    """bf16-valued blocks over 40 binades, with the boundary cases of the scale rule in the first rows."""
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(96, 256, generator=g) * torch.exp2(torch.randint(-20, 20, (96, 8), generator=g)
                                                        .repeat_interleave(32, dim=1).float())).bfloat16().float()
    x[0, :32] = 0                                        # an all-zero block
    x[1, :32] = 0; x[1, 3] = 448.0                       # exactly the format's maximum: scale 1
    x[2, :32] = 0; x[2, 3] = -452.0                      # the next bf16 magnitude above: scale 2
    x[3, :32] = 0; x[3, 3] = 446.0                       # the next below: scale 1
    x[4, :32] = 0; x[4, 3] = 448.0 * 2.0 ** -30          # a power-of-two multiple of the maximum, far down
    x[5, :32] = 0; x[5, 0] = 100.0; x[5, 5] = -12.5      # the reference's own first-principles case
    return x


def test_mxfp8_block_exponent_is_the_smallest_power_of_two_that_fits():
    """Pins ``e8m0_exponent`` by its defining inequality in exact rational arithmetic, 2^(e-1) < amax / 448 <= 2^e,
    and by the known answers the reference's tests hold: ``ceil(log2(100 / 448)) + 127`` for a block whose amax is 100
    (``tests/cpu/kernels/test_block_scale_oracle.py:19-23, 40-48``), code 0 for an all-zero block and for one below
    448 * 2^-127, 254 for a block holding an inf (``tests/cpu/kernels/test_quantization.py:268-301``) and 0xFF for a
    NaN block (``quantization.py:36``)."""
    import math
    from fractions import Fraction

    x = _mx_blocks()
    amax = x.abs().reshape(96, 8, 32).amax(dim=2).numpy()
    e, biased = mxfp8.e8m0_exponent(amax)
    assert biased.dtype == np.uint8 and np.array_equal(biased.astype(np.int64), e + 127)
    for a, ee in zip(amax.reshape(-1).tolist(), e.reshape(-1).tolist()):
        if a == 0:
            assert ee == -127
            continue
        ratio = Fraction(a) / 448
        assert ratio <= Fraction(2) ** ee and (ee == -127 or ratio > Fraction(2) ** (ee - 1)), (a, ee)
    assert biased[0, 0] == 0 and biased[1, 0] == 127 and biased[2, 0] == 128 and biased[3, 0] == 127
    assert biased[4, 0] == 97 and biased[5, 0] == math.ceil(math.log2(100.0 / 448.0)) + 127 == 125
    edge = np.array([3e-38, 1e-36, np.inf, np.nan, 448.0 * 2.0 ** 119, 3.0e38], dtype=np.float32)
    assert mxfp8.e8m0_exponent(edge)[1].tolist() == [0, 0, 254, 255, 246, 247]


def test_mxfp8_codes_are_torchs_e4m3_cast_of_the_scaled_block_and_round_trip_to_e4m3_precision():
    """Pins ``quantize_mxfp8`` / ``dequantize_mxfp8``: the codes equal torch's own float8_e4m3fn cast of the block
    divided (exactly, in float64) by its power-of-two scale; ``code * scale`` is within half an e4m3 step of the value
    (2^-4 relative for normals, 2^-10 of the scale below); shapes and dtypes as the reference's tests state them
    (``tests/cpu/kernels/test_quantization.py:29-35, 77-82``), along the last axis and along axis 0."""
    x = _mx_blocks()
    data, scales = mxfp8.quantize_mxfp8(x.numpy())
    assert data.shape == (96, 256) and data.dtype == np.uint8 and scales.shape == (96, 8) and scales.dtype == np.uint8
    scale = np.ldexp(1.0, scales.astype(np.int64) - 127)
    scaled = (x.double().reshape(96, 8, 32) / torch.from_numpy(scale)[:, :, None]).reshape(96, 256)
    assert float(scaled.abs().max()) <= 448
    want = scaled.float().to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    nonzero = (data & 0x7F) != 0
    assert np.array_equal(data[nonzero], want[nonzero]) and not (want[~nonzero] & 0x7F).any()
    restored = mxfp8.dequantize_mxfp8(data, scales)
    assert np.array_equal(restored, torch.from_numpy(restored).bfloat16().float().numpy())  # bf16 values
    xd = x.double().numpy()
    step = np.repeat(scale, 32, axis=1) * 2.0 ** -10
    assert (np.abs(restored - xd) <= np.maximum(np.abs(xd) * 2.0 ** -4, step)).all()
    # axis 0: the same blocks taken down the columns
    d0, s0 = mxfp8.quantize_mxfp8(x.numpy().T.copy(), axis=0)
    assert d0.shape == (256, 96) and s0.shape == (8, 96)
    assert np.array_equal(d0, data.T) and np.array_equal(s0, scales.T)
    with pytest.raises(ValueError, match="not divisible"):
        mxfp8.quantize_mxfp8(np.zeros((8, 30), dtype=np.float32))


def test_mxfp8_extreme_blocks_keep_their_codes():
    """The edges the reference tests (``tests/cpu/kernels/test_quantization.py:87-93, 268-301``): an all-zero tensor
    round-trips to exact zeros; a block below 448 * 2^-127 clamps to exponent -127 and one holding an inf reaches 127,
    and both keep nonzero codes (they are scaled by normal powers of two); a NaN poisons its own block only."""
    zeros = mxfp8.fake_quant_mxfp8(np.zeros((32, 64), dtype=np.float32))
    assert np.isfinite(zeros).all() and not zeros.any()
    g = torch.Generator().manual_seed(0)
    x = torch.randn(4, 64, generator=g)
    sign = torch.where(torch.rand(32, generator=g) < 0.5, -1.0, 1.0)
    x[1, :32] = (torch.rand(32, generator=g) * 0.5 + 0.5) * 3e-38 * sign
    x[2, :32] = torch.exp2(torch.rand(32, generator=g) * 19 + 108) * sign
    x[2, 0] = float("inf")
    x[3, 40] = float("nan")
    data, scales = mxfp8.quantize_mxfp8(x.numpy())
    assert scales[1, 0] == 0 and scales[2, 0] == 254 and scales[3, 1] == 255 and scales[3, 0] != 255
    assert (data[1, :32] & 0x7F).max() > 0 and (data[2, 1:16] & 0x7F).max() > 0
    assert data[2, 0] == 0x7E  # the inf itself saturates at 448
    # 3e-38 * 2^127 = 5.1: every element of the tiny block is a normal e4m3 value after scaling
    want = (x[1, :32].double() * 2.0 ** 127).float().to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(data[1, :32], want)
    restored = mxfp8.dequantize_mxfp8(data, scales)
    assert np.isnan(restored[3, 32:]).all() and np.isfinite(restored[3, :32]).all() and np.isfinite(restored[0]).all()


def test_mxfp8_round_trip_and_expert_product_sit_in_the_reference_error_bands():
    """The reference's tolerance for the round trip (relative Frobenius error below 0.05 on ``randn(64, 256) * 0.5``,
    ``tests/cpu/kernels/test_quantization.py:24, 57-64``) and its band for the fake-quantised expert product against
    the bf16 one (between 0.01 and 0.08, about 0.038 measured, ``tests/gpu/kernels/test_expert_gemm.py:55-74``: zero
    would mean nothing was quantised).  The product is also checked term by term on sampled outputs."""
    torch.manual_seed(0)
    x = torch.randn(64, 256) * 0.5
    recon = mxfp8.fake_quant_mxfp8(x.numpy())
    assert np.linalg.norm(recon - x.numpy()) / np.linalg.norm(x.numpy()) < 0.05
    g = torch.Generator().manual_seed(3)
    counts = (40, 0, 70, 18)
    a = (torch.randn(sum(counts), 320, generator=g) * 0.3).bfloat16().float().numpy()
    b = (torch.randn(len(counts), 320, 96, generator=g) * 0.02).bfloat16().float().numpy()
    offs = np.cumsum(counts)
    got = mxfp8.expert_gemm_mxfp8(a, b, offs)
    plain = np.zeros_like(got)
    start = 0
    for e, end in enumerate(offs.tolist()):
        plain[start:end] = a[start:end].astype(np.float64) @ b[e].astype(np.float64)
        start = end
    rel = np.linalg.norm(got - plain) / np.linalg.norm(plain)
    assert 0.01 < rel < 0.08, rel
    da, sa = mxfp8.quantize_mxfp8(a, -1)
    db, sb = mxfp8.quantize_mxfp8(b, 1)
    va, vb = block_fp8.decode_e4m3fn(da).astype(float), block_fp8.decode_e4m3fn(db).astype(float)
    for r, c in ((0, 0), (39, 95), (40, 3), (127, 50)):
        e = int(np.searchsorted(offs, r, side="right"))
        total = sum(va[r, k] * 2.0 ** (int(sa[r, k // 32]) - 127) * vb[e, k, c] * 2.0 ** (int(sb[e, k // 32, c]) - 127)
                    for k in range(320))
        assert abs(got[r, c] - total) <= 1e-12 * max(1.0, abs(total))


# ----------------------------------------------------------------------------------------------------------- mxfp4
def test_mxfp4_block_exponent_is_the_smallest_power_of_two_that_fits():
    """Pins ``mxfp4.e8m0_exponent`` by its defining inequality in exact rational arithmetic, 2^(e-1) < amax / 6 <= 2^e,
    and by the known answers the reference's tests hold: exponent 0 (code 127) for a block whose amax is 6
    (``tests/cpu/kernels/test_block_scale_oracle.py:60-70``), code 0 for a block below 6 * 2^-127 and 254 for one
    holding an inf (``tests/cpu/kernels/test_quantization.py:248-280``), 0xFF for a NaN block."""
    from fractions import Fraction

    x = _mx_blocks()
    amax = x.abs().reshape(96, 8, 32).amax(dim=2).numpy()
    e, biased = mxfp4.e8m0_exponent(amax)
    assert biased.dtype == np.uint8 and np.array_equal(biased.astype(np.int64), e + 127)
    for a, ee in zip(amax.reshape(-1).tolist(), e.reshape(-1).tolist()):
        if a == 0:
            assert ee == -127
            continue
        ratio = Fraction(a) / 6
        assert ratio <= Fraction(2) ** ee and (ee == -127 or ratio > Fraction(2) ** (ee - 1)), (a, ee)
    edge = np.array([6.0, 6.03125, 5.96875, 3.0, 3e-38, np.inf, np.nan, 3.0e38, 0.0], dtype=np.float32)
    assert mxfp4.e8m0_exponent(edge)[1].tolist() == [127, 128, 127, 126, 0, 254, 255, 127 + 126, 0]


def test_mxfp4_codes_are_the_nearest_level_with_ties_to_the_even_code():
    """Pins ``e2m1_round`` / ``quantize_mxfp4`` / ``dequantize_mxfp4``: the reference's known answers -- with amax 6 the
    scale is 1 and the levels map to their own codes (``tests/cpu/kernels/test_block_scale_oracle.py:60-78``); 2.5 goes
    down to 2.0, 2.6 up, 2.4 down (``:81-94``); 0.75, 1.75, 3.5 and -0.75 go up to 1, 2, 4 and -1, 0.7 and 0.8 to their
    nearest (``tests/cpu/kernels/test_quantization.py:99-113``) -- and, for every value of a dense grid, brute force:
    the chosen level is a nearest one, and on an exact tie it is the one whose code is even."""
    block = np.zeros(32, dtype=np.float32)
    vals = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.5, -6.0]
    block[:len(vals)] = vals
    data, scales = mxfp4.quantize_mxfp4(block)
    assert data.shape == (16,) and data.dtype == np.uint8 and scales.shape == (1,) and int(scales[0]) == 127
    assert mxfp4.unpack_codes(data)[:len(vals)].tolist() == [0, 1, 2, 3, 4, 5, 6, 7, 9, 15]
    assert data[0] == 0x10 and data[4] == 0xF9  # the even element sits in the low nibble
    block = np.zeros(32, dtype=np.float32)
    block[:4] = [6.0, 2.5, 2.6, 2.4]
    assert mxfp4.unpack_codes(mxfp4.quantize_mxfp4(block)[0])[1:4].tolist() == [4, 5, 4]
    block = np.zeros((1, 32), dtype=np.float32)
    block[0, :7] = [6.0, 0.75, 1.75, 3.5, -0.75, 0.7, 0.8]
    assert mxfp4.fake_quant_mxfp4(block)[0, :7].tolist() == [6.0, 1.0, 2.0, 4.0, -1.0, 0.5, 1.0]
    grid = np.arange(-7 * 64, 7 * 64 + 1, dtype=np.float32) / 64  # every multiple of 1/64 in [-7, 7]: holds every tie
    codes = mxfp4.e2m1_round(grid)
    levels = mxfp4.E2M1_LEVELS.astype(np.float64)
    for v, c in zip(grid.tolist(), codes.tolist()):
        mag = min(abs(v), 6.0)
        dist = np.abs(levels - mag)
        nearest = np.flatnonzero(dist == dist.min())
        want = nearest[0] if len(nearest) == 1 else next(i for i in nearest if i % 2 == 0)
        assert c & 7 == want and (c >> 3) == (1 if v < 0 else 0), (v, c)
    # shapes along the last axis and along axis 0 (``tests/cpu/kernels/test_quantization.py:48-55``)
    torch.manual_seed(0)
    x = (torch.randn(64, 256) * 0.5).numpy()
    data, scales = mxfp4.quantize_mxfp4(x)
    assert data.shape == (64, 128) and scales.shape == (64, 8) and data.dtype == scales.dtype == np.uint8
    d0, s0 = mxfp4.quantize_mxfp4(x.T.copy(), axis=0)
    assert d0.shape == (128, 64) and s0.shape == (8, 64) and np.array_equal(d0, data.T) and np.array_equal(s0, scales.T)
    # code * scale is within half a level gap of the value: at most a quarter of the block's scale below 2 * scale,
    # half of it up to 4, one above
    restored = mxfp4.dequantize_mxfp4(data, scales)
    scale = np.repeat(np.ldexp(1.0, scales.astype(np.int64) - 127), 32, axis=1)
    ratio = np.abs(x.astype(np.float64)) / scale
    bound = np.where(ratio <= 2, 0.25, np.where(ratio <= 4, 0.5, 1.0)) * scale
    assert (np.abs(restored - x) <= bound * (1 + 2.0 ** -8)).all()  # 2^-8: the bf16 rounding of the result
    with pytest.raises(ValueError, match="not divisible"):
        mxfp4.quantize_mxfp4(np.zeros((8, 30), dtype=np.float32))


def test_mxfp4_extreme_blocks_keep_their_codes():
    """The edges the reference tests (``tests/cpu/kernels/test_quantization.py:82-89, 248-280``;
    ``tests/cpu/kernels/test_block_scale_oracle.py:175-196``): zeros round-trip to zeros; a block below 6 * 2^-127
    clamps to exponent -127 and one holding an inf reaches 127, both keeping nonzero codes; an inf or a NaN makes its
    own block non-finite and no other; a large finite outlier never produces a NaN."""
    zeros = mxfp4.fake_quant_mxfp4(np.zeros((32, 64), dtype=np.float32))
    assert np.isfinite(zeros).all() and not zeros.any()
    g = torch.Generator().manual_seed(0)
    x = torch.randn(4, 64, generator=g)
    sign = torch.where(torch.rand(32, generator=g) < 0.5, -1.0, 1.0)
    x[1, :32] = (torch.rand(32, generator=g) * 0.5 + 0.5) * 3e-38 * sign
    x[2, :32] = torch.exp2(torch.rand(32, generator=g) * 19 + 108) * sign
    x[2, 0] = float("inf")
    x[3, 40] = float("nan")
    x[0, 0] = 5e4
    data, scales = mxfp4.quantize_mxfp4(x.numpy())
    assert scales[1, 0] == 0 and scales[2, 0] == 254 and scales[3, 1] == 255 and scales[3, 0] != 255
    codes = mxfp4.unpack_codes(data)
    assert (codes[1, :32] & 7).max() > 0 and (codes[2, 1:32] & 7).max() > 0 and codes[2, 0] == 7
    # 3e-38 * 2^127 = 5.1: the tiny block's codes are those of its values times 2^127
    assert np.array_equal(codes[1, :32], mxfp4.e2m1_round((x[1, :32].double() * 2.0 ** 127).float().numpy()))
    restored = mxfp4.dequantize_mxfp4(data, scales)
    assert np.isnan(restored[3, 32:]).all() and np.isfinite(restored[3, :32]).all() and np.isfinite(restored[0]).all()
    assert not np.isfinite(restored[2, :32]).all() and np.isfinite(restored[2, 32:]).all()


def test_mxfp4_round_trip_and_expert_product_sit_in_the_format_error_bands():
    """The reference's tolerance for the round trip (relative Frobenius error below 0.25 on ``randn(64, 256) * 0.5``,
    ``tests/cpu/kernels/test_quantization.py:24, 57-64``) with mxfp8 the more accurate of the two (``:67-70`` states it
    for fp8 against fp4), the error independent of the magnitude over 32 decades
    (``tests/cpu/kernels/test_block_scale_oracle.py:118-137``), and the product checked term by term on sampled
    outputs."""
    torch.manual_seed(0)
    x = (torch.randn(64, 256) * 0.5).numpy()
    err4 = np.linalg.norm(mxfp4.fake_quant_mxfp4(x) - x) / np.linalg.norm(x)
    err8 = np.linalg.norm(mxfp8.fake_quant_mxfp8(x) - x) / np.linalg.norm(x)
    assert err8 < err4 < 0.25 and err4 > 0.05
    base = torch.randn(128, 256).double().numpy()
    errs = []
    for exponent in range(4, -32, -4):
        scaled = (base * 10.0 ** exponent).astype(np.float32)
        recon = mxfp4.fake_quant_mxfp4(scaled).astype(np.float64)
        errs.append(np.linalg.norm(recon - scaled) / np.linalg.norm(scaled.astype(np.float64)))
    assert max(errs) - min(errs) < 0.02
    g = torch.Generator().manual_seed(3)
    counts = (40, 0, 70, 18)
    a = (torch.randn(sum(counts), 320, generator=g) * 0.3).bfloat16().float().numpy()
    b = (torch.randn(len(counts), 320, 96, generator=g) * 0.02).bfloat16().float().numpy()
    offs = np.cumsum(counts)
    got = mxfp4.expert_gemm_mxfp4(a, b, offs)
    ca, sa = mxfp4.unpack_codes(mxfp4.quantize_mxfp4(a, -1)[0]), mxfp4.quantize_mxfp4(a, -1)[1]
    cb, sb = mxfp4.unpack_codes(mxfp4.quantize_mxfp4(b, 1)[0], 1), mxfp4.quantize_mxfp4(b, 1)[1]
    level = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    value = lambda c: level[c & 7] * (-1.0 if c & 8 else 1.0)
    for r, c in ((0, 0), (39, 95), (40, 3), (127, 50)):
        e = int(np.searchsorted(offs, r, side="right"))
        total = sum(value(int(ca[r, k])) * 2.0 ** (int(sa[r, k // 32]) - 127) *
                    value(int(cb[e, k, c])) * 2.0 ** (int(sb[e, k // 32, c]) - 127) for k in range(320))
        assert abs(got[r, c] - total) <= 1e-12 * max(1.0, abs(total))


# ----------------------------------------------------------------------------------------------------------- nvfp4
def test_nvfp4_global_scale_is_the_smallest_power_of_two_that_lifts_the_amax_into_range():
    """Pins ``nvfp4.global_scale`` by its defining inequality in exact rational arithmetic, 2^(e-1) < amax / 2688 <=
    2^e, and by the reference's known answer: amax 30 gives 2^ceil(log2(30 / 2688)) = 2^-6, the block's e4m3 scale is
    then 30 / 6 / 2^-6 = 320 exactly, and the value comes back as 30
    (``tests/cpu/kernels/test_block_scale_oracle.py:97-116``)."""
    import math
    from fractions import Fraction

    g = torch.Generator().manual_seed(5)
    values = (torch.rand(200, generator=g) + 0.5) * torch.exp2(torch.randint(-100, 100, (200,), generator=g).float())
    for a in values.tolist() + [2688.0, 2688.0 * 2.0 ** -20, 2689.0, 2687.0, 1e-38, 3e38]:
        e = int(math.log2(float(nvfp4.global_scale(a))))
        assert float(nvfp4.global_scale(a)) == 2.0 ** e
        ratio = Fraction(max(np.float32(a).item(), float(np.finfo(np.float32).tiny))) / 2688
        assert ratio <= Fraction(2) ** e and ratio > Fraction(2) ** (e - 1), (a, e)
    assert nvfp4.global_scale(0.0) == np.float32(2.0 ** -137) and np.isnan(nvfp4.global_scale(np.nan))
    block = np.zeros(16, dtype=np.float32)
    block[0] = 30.0
    data, scales, gs = nvfp4.quantize_nvfp4(block)
    assert gs == 2.0 ** math.ceil(math.log2(30.0 / 2688.0)) == 2.0 ** -6
    assert block_fp8.decode_e4m3fn(scales)[0] == 320.0 and scales.dtype == np.uint8 and scales.shape == (1,)
    assert data.shape == (8,) and data[0] == 7 and not data[1:].any()
    assert nvfp4.dequantize_nvfp4(data, scales, gs)[0] == 30.0


def test_nvfp4_scales_are_torchs_e4m3_cast_and_codes_the_nearest_level_of_the_fp32_quotient():
    """Pins ``quantize_nvfp4`` / ``dequantize_nvfp4`` by library routines and brute force: the block scales equal
    torch's own float8_e4m3fn cast of ``amax / 6 / global`` (fp32 operations, as the reference's); every code is a
    level nearest to the fp32 quotient ``value / (scale * global)``, the even code on a tie; the round trip is within
    half a level gap of the value in units of the block's scale; storage shapes as the reference's tests state them
    (``tests/cpu/kernels/test_quantization.py:37-45``), along the last axis and along axis 0."""
    x = _mx_blocks().numpy()[6:]  # finite rows over 40 binades
    data, scales, gs = nvfp4.quantize_nvfp4(x)
    rows = x.shape[0]
    assert data.shape == (rows, 128) and scales.shape == (rows, 16) and data.dtype == scales.dtype == np.uint8
    xt = torch.from_numpy(x)
    amax = xt.abs().reshape(rows, 16, 16).amax(dim=2)
    want_scales = (amax / 6.0 / float(gs)).clamp(max=448.0).to(torch.float8_e4m3fn)
    assert np.array_equal(scales, want_scales.view(torch.uint8).numpy())
    divisor = want_scales.float() * float(gs)
    divisor = torch.where(divisor == 0, torch.ones_like(divisor), divisor)
    quotient = (xt.reshape(rows, 16, 16) / divisor[:, :, None]).reshape(rows, 256).double().numpy()
    codes = mxfp4.unpack_codes(data)
    levels = mxfp4.E2M1_LEVELS.astype(np.float64)
    mag = np.minimum(np.abs(quotient), 6.0)
    dist = np.abs(mag[..., None] - levels)
    chosen = np.take_along_axis(dist, (codes & 7)[..., None].astype(np.int64), axis=-1)[..., 0]
    assert (chosen == dist.min(axis=-1)).all()
    tie = (dist == dist.min(axis=-1, keepdims=True)).sum(axis=-1) > 1
    assert tie.any() and ((codes & 7)[tie] % 2 == 0).all()
    assert np.array_equal(codes >> 3, (quotient < 0).astype(np.uint8))
    restored = nvfp4.dequantize_nvfp4(data, scales, gs)
    assert np.array_equal(restored, torch.from_numpy(restored).bfloat16().float().numpy())
    # within half a level gap in units of the block's scale; a quotient above 6 (the e4m3 scale was rounded down)
    # saturates at 6 scales exactly, and a block whose scale underflows e4m3 (the tensor spans 40 binades under one
    # global scale) comes back as zeros: the format's own behaviour, asserted as such
    unit = np.repeat((want_scales.float() * float(gs)).double().numpy(), 16, axis=1)
    bound = np.where(mag <= 2, 0.25, np.where(mag <= 4, 0.5, 1.0)) * unit
    inside, dead = (np.abs(quotient) <= 6) & (unit > 0), unit == 0
    assert inside.sum() > 5000 and dead.any() and (~inside & ~dead).any()
    assert (np.abs(restored - x)[inside] <= (bound * (1 + 2.0 ** -8))[inside]).all()
    assert np.array_equal(np.abs(restored)[~inside & ~dead], (6 * unit)[~inside & ~dead].astype(np.float32))
    assert not restored[dead].any()
    d0, s0, g0 = nvfp4.quantize_nvfp4(x.T.copy(), axis=0)
    assert d0.shape == (128, rows) and s0.shape == (16, rows) and g0 == gs
    assert np.array_equal(d0, data.T) and np.array_equal(s0, scales.T)
    with pytest.raises(ValueError, match="not divisible"):
        nvfp4.quantize_nvfp4(np.zeros((8, 24), dtype=np.float32))


def test_nvfp4_edges_and_error_bands_as_the_reference_tests_state_them():
    """Zeros round-trip to zeros (``tests/cpu/kernels/test_quantization.py:82-89``); an outlier above 6 * 448 keeps every
    scale and value finite (``:116-124``); the round trip is inside 0.25 and worse than MXFP8's (``:58-71``); the error
    does not depend on the magnitude over 32 decades (``tests/cpu/kernels/test_block_scale_oracle.py:118-137``); a shard
    quantised alone equals its slice of the bank although their global scales differ (``:157-172``); an inf or a NaN is
    never absorbed and finite input never gives a NaN (``:175-196``); the product term by term on sampled outputs."""
    zeros = nvfp4.fake_quant_nvfp4(np.zeros((32, 64), dtype=np.float32))
    assert np.isfinite(zeros).all() and not zeros.any()
    torch.manual_seed(0)
    x = (torch.randn(16, 64) * 0.1).numpy()
    x[0, 0] = 5000.0
    data, scales, gs = nvfp4.quantize_nvfp4(x)
    assert np.isfinite(block_fp8.decode_e4m3fn(scales)).all() and ((scales & 0x7F) != 0x7F).all()
    assert np.isfinite(nvfp4.dequantize_nvfp4(data, scales, gs)).all()
    torch.manual_seed(0)
    x = (torch.randn(64, 256) * 0.5).numpy()
    err4 = np.linalg.norm(nvfp4.fake_quant_nvfp4(x) - x) / np.linalg.norm(x)
    err8 = np.linalg.norm(mxfp8.fake_quant_mxfp8(x) - x) / np.linalg.norm(x)
    assert err8 < err4 < 0.25 and err4 > 0.04
    base = torch.randn(128, 256).double().numpy()
    errs = []
    for exponent in range(4, -32, -4):
        scaled = (base * 10.0 ** exponent).astype(np.float32)
        recon = nvfp4.fake_quant_nvfp4(scaled).astype(np.float64)
        errs.append(np.linalg.norm(recon - scaled) / np.linalg.norm(scaled.astype(np.float64)))
    assert max(errs) - min(errs) < 0.02
    bank = (torch.randn(8, 64, 256) * 0.02).numpy()
    bank[0] *= 1e-3
    whole = nvfp4.fake_quant_nvfp4(bank)
    assert nvfp4.quantize_nvfp4(bank[:1])[2] != nvfp4.quantize_nvfp4(bank)[2]  # the small expert alone scales lower
    for lo in range(0, 8, 2):
        assert np.array_equal(nvfp4.fake_quant_nvfp4(bank[lo:lo + 2]), whole[lo:lo + 2])
    for poison in (np.nan, np.inf, -np.inf):
        bad = (torch.randn(4, 64) * 0.3).numpy()
        bad[1, 7] = poison
        assert not np.isfinite(nvfp4.fake_quant_nvfp4(bad)).all()
    fine = (torch.randn(4, 64) * 0.3).numpy()
    fine[0, 0] = 5e4
    fine[2, :] = 0.0
    assert np.isfinite(nvfp4.fake_quant_nvfp4(fine)).all()
    g = torch.Generator().manual_seed(3)
    counts = (40, 0, 70, 18)
    a = (torch.randn(sum(counts), 320, generator=g) * 0.3).bfloat16().float().numpy()
    b = (torch.randn(len(counts), 320, 96, generator=g) * 0.02).bfloat16().float().numpy()
    offs = np.cumsum(counts)
    got = nvfp4.expert_gemm_nvfp4(a, b, offs)
    da, sa, ga = nvfp4.quantize_nvfp4(a, -1)
    db, sb, gb = nvfp4.quantize_nvfp4(b, 1)
    ca, cb = mxfp4.unpack_codes(da), mxfp4.unpack_codes(db, 1)
    va, vb = block_fp8.decode_e4m3fn(sa).astype(float) * float(ga), block_fp8.decode_e4m3fn(sb).astype(float) * float(gb)
    level = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    value = lambda c: level[c & 7] * (-1.0 if c & 8 else 1.0)
    for r, c in ((0, 0), (39, 95), (40, 3), (127, 50)):
        e = int(np.searchsorted(offs, r, side="right"))
        total = sum(value(int(ca[r, k])) * va[r, k // 16] * value(int(cb[e, k, c])) * vb[e, k // 16, c] for k in range(320))
        assert abs(got[r, c] - total) <= 1e-12 * max(1.0, abs(total))
    plain = np.zeros_like(got)
    start = 0
    for e, end in enumerate(offs.tolist()):
        plain[start:end] = a[start:end].astype(np.float64) @ b[e].astype(np.float64)
        start = end
    rel = np.linalg.norm(got - plain) / np.linalg.norm(plain)
    assert 0.04 < rel < 0.25, rel  # the reference's band for this format (tests/gpu/kernels/test_expert_gemm.py:55-74)
