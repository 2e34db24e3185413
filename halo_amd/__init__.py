"""MI355X-native single-GPU MoE expert path: router top-k, atomic-free permute by expert, grouped SwiGLU expert GEMMs
and the weighted unpermute/combine, forward and backward, behind the Python API of the reference's ``halo.kernels``
ops and MoE block.  Compute lives in hand-written HIP kernels for gfx950 (``csrc/``) reached through a C ABI
(``include/halo_moe.h``)."""

__version__ = "0.1.0"
