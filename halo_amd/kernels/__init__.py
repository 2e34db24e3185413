"""The ops of the reference's ``halo.kernels`` package that sit on the MoE expert path, on HIP kernels for gfx950."""
