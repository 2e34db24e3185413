"""The C-ABI library builds into the tree, loads without a GPU, and exports exactly the symbols the header declares.
No compute is called here."""

import ctypes
import os
import re

import pytest
import torch

from halo_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "halo_moe.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hmoe_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    if not os.path.exists(_lib.LIB_PATH):
        from halo_amd.build import build

        build(verbose=False)
    lib = ctypes.CDLL(_lib.LIB_PATH)
    declared = _declared()
    assert len(declared) >= 20
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in include/halo_moe.h but not exported"
    assert sorted(_lib.SIGNATURES) == declared, "the ctypes table and the header disagree"


def test_status_strings_and_version():
    lib = _lib.load()
    assert lib.hmoe_abi_version() == 1
    assert lib.hmoe_status_string(0) == b"ok"
    assert b"unsupported" in lib.hmoe_status_string(-2)


def test_header_is_plain_c():
    """The header compiles as C: plain pointers and sizes, no C++ or torch types."""
    import subprocess
    import tempfile

    with tempfile.TemporaryDirectory() as tmp:
        src = os.path.join(tmp, "t.c")
        with open(src, "w") as f:
            f.write('#include "halo_moe.h"\nint main(void) { return hmoe_abi_version() == 0; }\n')
        subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-fsyntax-only", f"-I{ROOT}/include", src], check=True)


def test_a_cpu_tensor_among_device_operands_is_refused_and_bad_counts_raise():
    """CPU tensors take the operators' torch path (tests/test_cpu_ops.py); what is refused is a device call that is
    handed a CPU tensor (there is no GPU here, so the check is exercised on the helper itself)."""
    from halo_amd.kernels.moe_route_sort import sort_routing_by_expert

    with pytest.raises(RuntimeError, match="device tensors only"):
        _lib.require_device(torch.zeros(2))
    with pytest.raises(ValueError, match="2 receive counts for 4 local experts"):
        sort_routing_by_expert(torch.zeros(2, 2, dtype=torch.long), torch.rand(2, 2), 4, (3, 1))


def test_product_never_imports_the_oracle():
    for dirpath, _, files in os.walk(os.path.join(ROOT, "halo_amd")):
        for name in files:
            if name.endswith(".py"):
                text = open(os.path.join(dirpath, name)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M), f"{name} imports the oracle"


def test_bad_arguments_come_back_as_status_codes_before_any_launch():
    """Every entry point checks its arguments first and reports through its return value; none of these calls reaches
    a kernel launch (there is no GPU here), and an empty problem is a success that launches nothing."""
    lib = _lib.load()
    invalid, unsupported = -1, -2
    assert lib.hmoe_status_string(invalid) != lib.hmoe_status_string(unsupported)
    bf16, f32 = _lib.dtype_id(torch.bfloat16), _lib.dtype_id(torch.float32)
    fake = 0x10000  # a non-null, 16-byte aligned address that is never dereferenced on these paths

    # grouped GEMM: negative sizes, several groups without offsets, rows not 16-byte multiples, too many groups
    gemm = lib.hmoe_grouped_gemm_fwd
    assert gemm(fake, 64, fake, fake, -1, 4, 64, 64, bf16, fake, 64, None) == invalid
    assert gemm(fake, 64, fake, None, 8, 4, 64, 64, bf16, fake, 64, None) == invalid
    assert gemm(fake, 60, fake, fake, 8, 4, 60, 64, bf16, fake, 64, None) == unsupported
    assert gemm(fake, 64, fake, fake, 8, 5000, 64, 64, bf16, fake, 64, None) == unsupported
    assert gemm(fake, 64, fake, fake, 8, 4, 64, 64, 77, fake, 64, None) == unsupported
    assert gemm(None, 64, fake, fake, 8, 4, 64, 64, bf16, fake, 64, None) == invalid
    assert gemm(fake, 32, fake, fake, 8, 4, 64, 64, bf16, fake, 64, None) == invalid  # row stride below the row length
    assert gemm(None, 64, None, None, 0, 1, 64, 64, bf16, None, 64, None) == 0  # no rows: nothing to do
    assert lib.hmoe_grouped_gemm_fwd_bias(fake, 64, fake, None, fake, 8, 4, 64, 64, bf16, fake, 64, None) == invalid
    assert lib.hmoe_grouped_gemm_fwd_gather(fake, 64, 8, fake, fake, fake, 8, 4, 64, 64, f32, fake, 64, None) == unsupported
    addto = lib.hmoe_grouped_gemm_fwd_addto
    assert addto(fake, 64, fake, fake, 8, 4, 64, 64, bf16, None, 64, 2.0, fake, 64, None) == invalid  # no addend
    assert addto(fake, 64, fake, fake, 8, 4, 64, 64, bf16, fake, 32, 2.0, fake, 64, None) == invalid  # addend rows overlap
    assert addto(fake, 64, fake, fake, 8, 4, 64, 64, bf16, fake, 68, 2.0, fake, 64, None) == unsupported  # 136-byte rows
    assert addto(fake, 64, fake, fake, 8, 4, 64, 64, bf16, fake + 2, 64, 2.0, fake, 64, None) == unsupported
    assert lib.hmoe_grouped_gemm_fwd_gather(fake, 64, -3, fake, fake, fake, 8, 4, 64, 64, bf16, fake, 64, None) == invalid
    gather_bias = lib.hmoe_grouped_gemm_fwd_gather_bias
    assert gather_bias(fake, 64, 8, fake, fake, None, fake, 8, 4, 64, 64, bf16, fake, 64, None) == invalid  # no bias
    assert gather_bias(fake, 64, 8, fake, fake, fake, fake, 8, 4, 64, 64, f32, fake, 64, None) == unsupported
    assert gather_bias(fake, 64, 8, fake, fake, fake + 4, fake, 8, 4, 64, 64, bf16, fake, 64, None) == unsupported
    assert gather_bias(None, 64, 8, None, None, None, None, 0, 1, 64, 64, bf16, None, 64, None) == 0
    dgrad_addto = lib.hmoe_grouped_gemm_dgrad_addto
    assert dgrad_addto(fake, 64, fake, fake, 8, 4, 64, 64, bf16, None, 64, fake, 64, None) == invalid  # no addend
    assert dgrad_addto(fake, 64, fake, fake, 8, 4, 64, 64, bf16, fake, 32, fake, 64, None) == invalid  # addend rows overlap
    assert dgrad_addto(fake, 64, fake, fake, 8, 4, 64, 64, bf16, fake, 68, fake, 64, None) == unsupported
    assert dgrad_addto(fake, 64, fake, fake, 8, 4, 64, 64, bf16, fake + 2, 64, fake, 64, None) == unsupported
    assert dgrad_addto(None, 64, None, None, 0, 1, 64, 64, bf16, None, 64, None, 64, None) == 0

    # what must stay below 2 GiB: an array gathered from by row index, one expert's weight, 512 rows of the widest
    # operand -- and nothing else (activations and outputs of any size are addressed tile by tile)
    big_rows = (1 << 31) // (2880 * 2) + 1000  # 2880-wide bf16 rows past 2 GiB
    gather = lib.hmoe_grouped_gemm_fwd_gather
    assert gather(fake, 2880, big_rows, fake, fake, fake, 64, 4, 2880, 64, bf16, fake, 64, None) == unsupported
    assert lib.hmoe_grouped_gemm_dgrad_gather(fake, 2880, big_rows, fake, fake, fake, 64, 4, 64, 2880, bf16, fake, 64,
                                              None) == unsupported
    assert lib.hmoe_grouped_gemm_wgrad_gather_grad(fake, 64, fake, 2880, big_rows, fake, fake, 64, 4, 64, 2880, bf16,
                                                   fake, None) == unsupported
    assert gemm(fake, 40000, fake, fake, 8, 4, 40000, 40000, bf16, fake, 40000, None) == unsupported  # 3 GB per expert
    assert gemm(fake, 1 << 22, fake, fake, 8, 4, 64, 64, bf16, fake, 64, None) == unsupported  # 8 MiB between rows
    assert lib.hmoe_grouped_gemm_fwd_fp8w(fake, 2880, fake, fake, fake, big_rows, 4, 2880, 64, fake, 64, None) == unsupported

    # fp8 MFMA product: whole scale blocks along K, 16-byte output rows, a scale row for every row
    fp8 = lib.hmoe_grouped_gemm_fwd_fp8
    assert fp8(fake, fake, 8, fake, fake, fake, 8, 4, 200, 128, fake, 128, None) == unsupported
    assert fp8(fake, fake, 8, fake, fake, fake, 8, 4, 256, 100, fake, 128, None) == unsupported
    assert fp8(fake, fake, 8, fake, fake, fake, 8, 4, 256, 128, fake, 100, None) == unsupported
    assert fp8(fake, fake, 4, fake, fake, fake, 8, 4, 256, 128, fake, 128, None) == unsupported
    assert fp8(fake, fake, 8, fake, fake, fake, -1, 4, 256, 128, fake, 128, None) == invalid

    # MXFP8: blocks of 32 along the contraction for the quantisers, whole panels of 64 for the product
    rows_mx = lib.hmoe_quantize_rows_mxfp8
    assert rows_mx(fake, bf16, 64, None, 8, 8, 48, fake, fake, 8, None) == unsupported      # K % 32
    assert rows_mx(fake, 77, 64, None, 8, 8, 64, fake, fake, 8, None) == unsupported        # dtype
    assert rows_mx(fake, bf16, 64, None, 9, 8, 64, fake, fake, 8, None) == invalid          # no index: x_rows == rows
    assert rows_mx(fake, bf16, 64, None, 8, 8, 64, fake, fake, 4, None) == unsupported      # out_rows < rows
    assert rows_mx(fake, bf16, 64, None, 8, 8, 64, None, fake, 8, None) == invalid
    assert rows_mx(None, bf16, 64, None, 0, 0, 64, None, None, 0, None) == 0
    assert lib.hmoe_dequantize_rows_mxfp8(fake, fake, 4, 8, 64, fake, 64, None) == invalid  # fewer rows than asked for
    assert lib.hmoe_dequantize_rows_mxfp8(fake, fake, 8, 8, 48, fake, 64, None) == unsupported
    weight_mx = lib.hmoe_quantize_weight_mxfp8
    assert weight_mx(fake, bf16, 4, 48, 64, fake, fake, None, None) == unsupported
    assert weight_mx(fake, bf16, 4, 64, 64, None, fake, None, None) == invalid
    assert weight_mx(fake, bf16, 0, 64, 64, None, None, None, None) == 0
    mx = lib.hmoe_grouped_gemm_fwd_mxfp8
    assert mx(fake, fake, 8, fake, fake, fake, 8, 4, 96, 128, fake, 128, None) == unsupported   # half a panel
    assert mx(fake, fake, 8, fake, fake, fake, 8, 4, 128, 100, fake, 128, None) == unsupported
    assert mx(fake, fake, 4, fake, fake, fake, 8, 4, 128, 128, fake, 128, None) == unsupported  # scale rows < rows
    assert mx(fake, fake, 8, fake, fake, None, 8, 4, 128, 128, fake, 128, None) == invalid      # groups without ends
    assert mx(fake, fake, 8, fake, None, fake, 8, 4, 128, 128, fake, 128, None) == invalid
    assert mx(None, None, 0, None, None, None, 0, 1, 128, 128, None, 128, None) == 0

    # MXFP4: blocks of 32 along the contraction, at least one output, the scales with the codes
    rows4 = lib.hmoe_mxfp4_rows
    assert rows4(fake, bf16, 64, None, 8, 8, 48, fake, fake, None, 64, None) == unsupported   # K % 32
    assert rows4(fake, 77, 64, None, 8, 8, 64, fake, fake, None, 64, None) == unsupported     # dtype
    assert rows4(fake, bf16, 64, None, 9, 8, 64, fake, fake, None, 64, None) == invalid       # no index: x_rows == rows
    assert rows4(fake, bf16, 64, None, 8, 8, 64, None, None, None, 64, None) == invalid       # no output
    assert rows4(fake, bf16, 64, None, 8, 8, 64, fake, None, None, 64, None) == invalid       # codes without scales
    assert rows4(fake, bf16, 64, None, 8, 8, 64, None, None, fake, 60, None) == unsupported   # rows that overlap
    assert rows4(None, bf16, 64, None, 0, 0, 64, None, None, None, 64, None) == 0
    weight4 = lib.hmoe_mxfp4_weight
    assert weight4(fake, bf16, 4, 48, 64, fake, fake, None, None) == unsupported
    assert weight4(fake, bf16, 4, 64, 64, None, None, None, None) == invalid
    assert weight4(fake, bf16, 4, 64, 64, fake, None, None, None) == invalid
    assert weight4(fake, bf16, 0, 64, 64, None, None, None, None) == 0
    assert lib.hmoe_mxfp4_dequantize_rows(fake, fake, 8, 48, fake, 64, None) == unsupported
    assert lib.hmoe_mxfp4_dequantize_rows(fake, None, 8, 64, fake, 64, None) == invalid
    assert lib.hmoe_mxfp4_dequantize_rows(None, None, 0, 64, None, 64, None) == 0
    assert lib.hmoe_mxfp4_rows_panels(fake, bf16, 64, None, 8, 8, 64, fake, fake, 4, None) == unsupported  # out_rows < rows
    assert lib.hmoe_mxfp4_rows_panels(fake, bf16, 64, None, 8, 8, 64, None, fake, 8, None) == invalid
    assert lib.hmoe_mxfp4_rows_panels(None, bf16, 64, None, 0, 0, 64, None, None, 0, None) == 0
    assert lib.hmoe_mxfp4_weight_panels(fake, bf16, 4, 64, 64, None, fake, fake, None) == invalid          # no codes
    assert lib.hmoe_mxfp4_weight_panels(fake, bf16, 4, 48, 64, fake, fake, None, None) == unsupported
    assert lib.hmoe_mxfp4_dequantize_panels(fake, fake, 4, 8, 64, fake, 64, None) == invalid  # fewer rows than asked for
    mx4 = lib.hmoe_grouped_gemm_fwd_mxfp4
    assert mx4(fake, fake, 8, fake, fake, fake, 8, 4, 48, 128, fake, 128, None) == unsupported    # K % 32
    assert mx4(fake, fake, 8, fake, fake, fake, 8, 4, 128, 100, fake, 128, None) == unsupported
    assert mx4(fake, fake, 4, fake, fake, fake, 8, 4, 128, 128, fake, 128, None) == unsupported   # scale rows < rows
    assert mx4(fake, fake, 8, fake, fake, None, 8, 4, 128, 128, fake, 128, None) == invalid       # groups without ends
    assert mx4(fake, fake, 8, fake, None, fake, 8, 4, 128, 128, fake, 128, None) == invalid
    assert mx4(None, None, 0, None, None, None, 0, 1, 128, 128, None, 128, None) == 0
    # NVFP4: blocks of 16, the tensor's amax required, at least one output, the scales with the codes
    nv = lib.hmoe_nvfp4_rows
    assert nv(fake, bf16, 64, None, 8, 8, 40, fake, fake, fake, None, 64, None, None) == unsupported   # K % 16
    assert nv(fake, bf16, 64, None, 8, 8, 64, None, fake, fake, None, 64, None, None) == invalid       # no amax
    assert nv(fake, bf16, 64, None, 8, 8, 64, fake, None, None, None, 64, None, None) == invalid       # no output
    assert nv(fake, bf16, 64, None, 8, 8, 64, fake, fake, None, None, 64, None, None) == invalid       # codes, no scales
    assert nv(None, bf16, 64, None, 0, 0, 64, None, None, None, None, 64, None, None) == 0
    assert lib.hmoe_nvfp4_weight(fake, bf16, 4, 40, 64, fake, fake, fake, None, None, None) == unsupported
    assert lib.hmoe_nvfp4_weight(fake, bf16, 4, 64, 64, None, fake, fake, None, None, None) == invalid
    assert lib.hmoe_nvfp4_weight(fake, bf16, 0, 64, 64, None, None, None, None, None, None) == 0
    assert lib.hmoe_nvfp4_dequantize_rows(fake, fake, None, 8, 64, fake, 64, None) == invalid
    assert lib.hmoe_nvfp4_dequantize_rows(fake, fake, fake, 8, 40, fake, 64, None) == unsupported
    for with_bias in (lib.hmoe_grouped_gemm_fwd_mxfp8_bias, lib.hmoe_grouped_gemm_fwd_mxfp4_bias):
        assert with_bias(fake, fake, 8, fake, fake, None, fake, 8, 4, 128, 128, fake, 128, None) == invalid  # no bias
        assert with_bias(fake, fake, 8, fake, fake, fake + 2, fake, 8, 4, 128, 128, fake, 128, None) == unsupported
        assert with_bias(fake, fake, 8, fake, fake, fake, fake, 8, 4, 128, 100, fake, 128, None) == unsupported
        assert with_bias(None, None, 0, None, None, None, None, 0, 1, 128, 128, None, 128, None) == 0
    assert fp8(fake, None, 8, fake, fake, fake, 8, 4, 256, 128, fake, 128, None) == invalid
    assert fp8(None, None, 0, None, None, None, 0, 1, 256, 128, None, 128, None) == 0
    assert lib.hmoe_quantize_rows_fp8(fake, 200, None, 8, 8, 200, fake, fake, 8, None) == unsupported
    assert lib.hmoe_quantize_rows_fp8(fake, 256, None, 8, 8, 256, fake, fake, 4, None) == unsupported
    assert lib.hmoe_quantize_rows_fp8(fake, 256, None, 8, 8, 256, fake, None, 8, None) == invalid
    assert lib.hmoe_quantize_rows_fp8(fake, 256, None, 9, 8, 256, fake, fake, 8, None) == invalid  # no index, other rows
    assert lib.hmoe_quantize_rows_fp8(None, 256, None, 0, 0, 256, None, None, 0, None) == 0
    glu_q = lib.hmoe_glu_fwd_quant_fp8
    assert glu_q(fake, fake, 512, 512, 8, 200, 0, 1.0, 0.0, 0, 0, fake, fake, 8, None) == unsupported  # 200 % 128
    assert glu_q(fake, fake, 512, 512, 8, 256, 0, 1.0, 0.0, 0, 0, fake, fake, 4, None) == unsupported  # out_rows < rows
    assert glu_q(fake, fake, 512, 512, 8, 256, 0, 1.0, 0.0, 0, 0, None, fake, 8, None) == invalid
    assert glu_q(fake, fake, 512, 512, 8, 256, 9, 1.0, 0.0, 0, 0, fake, fake, 8, None) == invalid  # no such activation
    assert glu_q(None, None, 512, 512, 0, 256, 0, 1.0, 0.0, 0, 0, None, None, 0, None) == 0

    # row movers
    assert lib.hmoe_gather_rows(fake, 64, fake, -1, 64, bf16, fake, None) == invalid
    assert lib.hmoe_gather_rows(None, 64, None, 0, 64, bf16, None, None) == 0
    assert lib.hmoe_gather_reduce(fake, None, None, 4, 2, 8, 64, bf16, fake, None) == invalid  # slots without a map
    assert lib.hmoe_gather_reduce_add(fake, None, fake, 4, 2, 8, 64, bf16, None, 0, fake, fake, None) == invalid
    assert lib.hmoe_gather_reduce_add(fake, None, fake, 4, 2, 8, 64, bf16, fake, 32, None, fake, None) == invalid
    assert lib.hmoe_unpermute_bwd(fake, 64, fake, fake, fake, 4, 64, bf16, fake, None, None) == invalid
    assert lib.hmoe_expert_colsum(None, None, 4, 64, 2, bf16, fake, None, None) == invalid
    assert lib.hmoe_expert_colsum(None, None, 0, 64, 0, bf16, None, None, None) == 0
    assert lib.hmoe_expert_colsum_workspace_bytes(1000, 64, 3) == (8 + 3) * 64 * 4
    assert lib.hmoe_expert_colsum_workspace_bytes(-1, 64, 3) == 0

    # routing sort
    assert lib.hmoe_route_sort_workspace_bytes(-1, 2, 4) < 0
    assert lib.hmoe_route_sort_workspace_bytes(16, 2, 4) > 0


def test_mx_size_check_is_the_entry_points_own_and_the_predicates_follow_it():
    """The MX products' scaled-MFMA kernel rebases the activations' descriptor per stage and the output's per tile, so
    neither has a size limit; one expert's quantised weights, the rows' exponent bytes (counted as four per row and
    panel) and a tile's 256 output rows must stay below 2 GiB.  ``hmoe_grouped_gemm_mx_fits`` is the check the entry
    points run; the Python predicates that route an oversized product to the round trip on the bf16 kernels call it,
    so the two cannot disagree.  Both sides of each boundary."""
    from halo_amd.kernels.expert_gemm import mxfp4_mfma_usable, mxfp8_mfma_usable

    lib = _lib.load()
    two_gib = 2**31
    k, n = 2048, 1536
    assert lib.hmoe_grouped_gemm_mx_fits(4_000_000, 4_000_000, k, n, n, 64) == 1  # 12 GB of output, 8 GB of panels
    scale_limit = -(-two_gib // (4 * (k // 64)))  # rows at which the exponent bytes reach 2 GiB
    assert lib.hmoe_grouped_gemm_mx_fits(scale_limit - 1, scale_limit - 1, k, 8, 8, 64) == 1
    assert lib.hmoe_grouped_gemm_mx_fits(scale_limit, scale_limit, k, 8, 8, 64) == 0
    assert lib.hmoe_grouped_gemm_mx_fits(2 * scale_limit - 1, 2 * scale_limit - 1, k, 8, 8, 128) == 1  # half the panels
    assert lib.hmoe_grouped_gemm_mx_fits(2 * scale_limit, 2 * scale_limit, k, 8, 8, 128) == 0
    assert lib.hmoe_grouped_gemm_mx_fits(16, 16, 32768, 65536, 65536, 64) == 0  # one expert's weights at 2 GiB
    assert lib.hmoe_grouped_gemm_mx_fits(16, 16, 32768, 65528, 65528, 64) == 1
    wide = two_gib // (2 * 256)             # an output pitch at which 256 rows reach 2 GiB
    assert lib.hmoe_grouped_gemm_mx_fits(16, 16, 64, 8, wide - 8, 64) == 1
    assert lib.hmoe_grouped_gemm_mx_fits(16, 16, 64, 8, wide, 64) == 0
    assert lib.hmoe_grouped_gemm_mx_fits(-1, 0, k, n, n, 64) == 0 and lib.hmoe_grouped_gemm_mx_fits(1, 1, k, n, n, 32) == 0
    bf16 = torch.bfloat16
    for rows in (scale_limit - 1, scale_limit, 10 * scale_limit):
        fits = rows < scale_limit
        assert mxfp8_mfma_usable(bf16, bf16, k, n, rows) == fits
        assert mxfp4_mfma_usable(bf16, bf16, k, n, rows) == (rows < 2 * scale_limit)
    # the entry point itself refuses what the check refuses, before any launch
    fake = 4096  # a non-null, 16-byte aligned address that is never dereferenced on the host
    rc = lib.hmoe_grouped_gemm_fwd_mxfp8(fake, fake, scale_limit, fake, fake, None, scale_limit, 1, k, n, fake, n, None)
    assert rc == -2
