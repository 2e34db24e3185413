"""CPU oracle for the single-GPU MoE expert path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``halo_amd/`` imports this package; only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` do, and there only as the checker or as the
timed CPU baseline, never as the product.

Every function restates, on the CPU in numpy (integer work) or torch fp32/fp64 (floating point), what the reference
computes for this path, and cites the reference file:line it follows (paths relative to the reference checkout).

How each function is pinned (tests/test_oracle_*.py):

* ``route_sort.argsort_routing`` / ``build_inv_map`` -- brute-force slot-by-slot sort on tiny inputs, the literal
  receive ``[[0,-1,2],[2,0,3],[-1,3,-1],[-1,-1,0]]`` of ``tests/cpu/parallelism/test_ep_receive_counts.py:65-70``,
  the twelve routing cases of ``tests/common/route_sort_reference.py:46-59`` through their invariants, and the
  ``inv_map`` invariants of ``tests/cpu/parallelism/test_moe_permute_equivalence.py:79-106``.
* ``permute.*`` -- fp64 ``index_select`` / ``index_add`` (library routines) and the literal sentinel example of
  ``tests/gpu/kernels/test_moe_permute.py:93-97``.
* ``glu.*`` -- torch autograd through ``F.silu`` / ``F.gelu`` / ``clamp`` in fp64 (library routines), the identity
  ``gptoss(alpha=1) - clamped_silu = silu(min(g, L))`` and bound sub-gradients.
* ``grouped_mm.*`` -- ``torch.matmul`` per group with autograd, and the empty-group counts ``(7,33,0,1,64,0)`` and
  ``(0,0,0,0,105,0)`` of ``tests/gpu/kernels/test_grouped_mm_empty_groups.py``.
* ``router.*`` -- ``torch.softmax`` / ``torch.topk`` on tie-free rows, autograd for the backward, and the tie rule
  (lower expert index wins) by brute force.  The order ``torch.topk`` gives tied scores is implementation-defined in
  the reference's third-party router: for tied rows the reference's own order is "parity unpinned"; this build fixes
  it to the lower index.
* ``block_fp8.*`` -- the ``exp2(ceil(log2(amax/448)))`` diagnostic formula, the ``448*4`` boundary case, padded
  shapes and the zero block of ``tests/cpu/weight_sync/test_block_fp8.py``.
* ``mxfp8.*`` -- the block exponent by its defining inequality ``2^(e-1) < amax/448 <= 2^e`` in exact rational
  arithmetic; the codes by torch's own ``float8_e4m3fn`` cast of the exactly scaled blocks; ``code * scale`` within half
  an e4m3 step of the value; the known answers the reference's tests hold (amax 100 -> code 125 of
  ``tests/cpu/kernels/test_block_scale_oracle.py:40-48``; zero, sub-2^-127, inf and NaN blocks and the round-trip bound of
  ``tests/cpu/kernels/test_quantization.py:57-93, 268-301``; the expert product's error band of
  ``tests/gpu/kernels/test_expert_gemm.py:55-74``) and the product term by term on sampled outputs.  For fp32 inputs
  whose amax / 448 lies within an ulp of a power of two the reference's exponent depends on the rounding of its
  ``log2``: "parity unpinned" there (bf16 inputs are never that close).
* ``mxfp4.*`` -- the block exponent by ``2^(e-1) < amax/6 <= 2^e`` in exact rational arithmetic; the e2m1 rounding by brute
  force over every multiple of 1/64 in [-7, 7] (a nearest level, the even code on a tie); the known answers the
  reference's tests hold (amax 6 -> scale 1 and every level its own code, 2.5 down / 2.6 up / 2.4 down of
  ``tests/cpu/kernels/test_block_scale_oracle.py:60-94``; 0.75, 1.75, 3.5, -0.75 -> 1, 2, 4, -1 and the storage shapes
  of ``tests/cpu/kernels/test_quantization.py:48-55, 99-113``; zero, sub-2^-127, inf and NaN blocks, the 0.25 round-trip
  bound, the magnitude independence of ``test_block_scale_oracle.py:118-137``) and the product term by term on sampled
  outputs.  The same fp32 ``log2`` caveat as ``mxfp8`` at power-of-two multiples of 6: "parity unpinned" there.
* ``nvfp4.*`` -- the global scale by ``2^(e-1) < amax/2688 <= 2^e`` in exact rational arithmetic; the block scales by
  torch's own ``float8_e4m3fn`` cast of ``amax / 6 / global``; the codes by brute force (a nearest level of the fp32
  quotient, the even code on a tie); the known answers the reference's tests hold (amax 30 -> global 2^-6, scale 320,
  value 30 of ``tests/cpu/kernels/test_block_scale_oracle.py:97-116``; the storage shapes, the outlier of 5000, the
  0.25 bound and "fp8 beats fp4" of ``tests/cpu/kernels/test_quantization.py:37-45, 58-71, 116-124``; magnitude
  independence, shard against bank, non-finite inputs of ``test_block_scale_oracle.py:118-196``) and the product term by
  term.  A tensor whose amax / 2688 lies within an ulp of a power of two: "parity unpinned" (``log2`` rounding).
* ``moe_layer.*`` -- the dense formula ``out[t] = sum_k w[t,k] * FFN_e(x[t])`` over valid slots.
"""
