"""Low-precision formats on the expert path: block fp8 served weights and the MXFP8 quantisation-aware format."""
