"""CPU oracle for the expert-specialized grouped-GEMM path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
directory: it is the checker that the HIP kernels are compared against (from
``tests/``, from the smoke check and from the CPU-baseline leg of the
benchmark), never the thing measured or shipped.

Every function restates, in numpy (torch CPU only for the big fp32 matmul), the
arithmetic that the reference defines for this path and cites the reference
file:line it follows.

Parity status per function (what pins it is in ``tests/test_oracle_*.py``):

* ``fp8.e4m3fn_decode / e4m3fn_encode_rne``  pinned: exhaustive against torch's
  ``float8_e4m3fn`` cast over all 2^16 bf16 patterns and against the OCP table.
* ``fp8_blockwise.quant_act_1x128 / quant_weight_128x128``  pinned: closed-form
  invariants (argmax element maps to +-448, zero block scale 1e-4/448,
  transpose equivalence) and an independent torch restatement.
* ``fp8_blockwise.grouped_mm``  pinned: C brute-force triple loop, fp64
  evaluation, exact integer cases, one-hot rows, power-of-two scale shifts.
* ``mxfp8.quant_rows``  pinned for everything except one hardware-dependent
  tie: at amax == 448 * 2^j the reference result depends on the last bit of
  NVIDIA's ``rcp.approx.ftz.f32(448)``; the oracle uses the correctly rounded
  reciprocal.  That single case is PARITY UNPINNED (no golden vectors exist in
  the reference and it cannot be executed here).
* ``mxfp8.sf_offset``  pinned: literal enumeration of the CuTe layout
  ``((32,4),4):((16,4),1)`` tiled K-fastest.
* ``mxfp8.grouped_mm``  pinned: same exact-case set as ``fp8_blockwise.grouped_mm``.
* ``torch_path.scaled_mm / mx_scaled_mm``  (the benchmark's CPU baseline: the reference's
  torch path in stock torch ops)  pinned: against the two ``grouped_mm`` above and an
  exact small-integer case.
"""
