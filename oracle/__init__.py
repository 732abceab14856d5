"""CPU oracle for the quantized-linear hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package may import this
directory: it is the checker used by ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py``.  The product path must fail
loudly when its HIP library is missing rather than fall back to this code.

Each module restates, with numpy / CPU torch only, what the reference's
operators on this path are defined to compute; each function cites the
reference file:line it follows.

Pinning status (what independent evidence each function is checked against is
in ``tests/test_oracle_*.py``):

* ``w4.gptq_unpack_*``, ``w4.awq_unpack_*``, ``w4.ref_halfgroup_*``:
  hand-derived known-answer words, pack/unpack inverses over all 16 nibble
  values, brute-force scalar loops on tiny matrices.
* ``w4.w4a16_gemm``: exact special cases (power-of-two scales, small-integer
  activations), GEMV reduction row by row in float64.
* ``w8a8.*``: int64 brute force, float64 closed forms.
* ``fp8.*``: float64 decode tables for e4m3fn, closed-form scales.
* ``moe.topk_softmax`` / ``moe.grouped_topk`` / ``moe.moe_align_block_size``:
  brute force on tiny inputs, the upstream docstring known-answer case for
  align, structural invariants.
* The vendor GEMM kernels the reference forwards to are closed source and no
  test in the reference pins any quantized-GEMM result, so the floating-point
  GEMM results are "parity unpinned" with respect to the reference's device
  output; they are pinned to the stated definition (CPU dequantize + matmul
  with fp32 accumulation) only.
"""
