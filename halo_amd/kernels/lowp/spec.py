"""The low-precision vocabulary of the expert path.

Mirrors ``halo/kernels/lowp/spec.py:9-11`` of the reference: ``QuantFormat`` names a block-scaled operand format of
the expert GEMM.  Of the reference's three (mxfp8 = e4m3 + e8m0 / 32, mxfp4 = e2m1 + e8m0 / 32, nvfp4 = e2m1 +
e4m3 / 16) mxfp8 and mxfp4 run on the scaled matrix instruction (e4m3 and e2m1 operands); nvfp4, whose e4m3 scales
the instruction cannot take, runs as the reference's default does: the bf16 product of the two round-tripped operands.
"""

from __future__ import annotations

from typing import Literal

QuantFormat = Literal["mxfp8", "mxfp4", "nvfp4"]

# Elements per shared scale along the contraction axis (``halo/kernels/lowp/quantization.py:47``).
FORMAT_BLOCK_SIZE: dict[str, int] = {"mxfp8": 32, "mxfp4": 32, "nvfp4": 16}


def require_implemented(fmt: str) -> None:
    if fmt not in FORMAT_BLOCK_SIZE:
        raise ValueError(f"unknown block-scaled format {fmt!r} (expected one of {sorted(FORMAT_BLOCK_SIZE)})")
