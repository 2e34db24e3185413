"""Low-precision weight formats on the expert path (block fp8)."""
