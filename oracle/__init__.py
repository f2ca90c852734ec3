"""CPU oracle for the quantized dot_general hot path of aqt.jax.v2.

TEST INFRASTRUCTURE ONLY.  This package is a from-scratch numpy restatement of
the reference's algorithm (google/aqt, `aqt/jax/v2/*`).  It exists to check the
HIP path: only `tests/`, `__graft_entry__.smoke()` and the `cpu_baseline` leg of
`bench.py` may import it.  Nothing under `aqt_amd/` imports it, and the product
path never falls back to it.

Semantics restated here are the reference's *strict, op-by-op* ones (what an
eager JAX run does): every jnp/lax op rounds its result to the op's result
dtype, so with bf16 operands the scale, its reciprocal, the scaled value and the
noisy value are each rounded to bf16 (see `numerics.py`).

Pin status of each part (what fixes it without importing JAX):
  * threefry2x32 block function ........ Random123 known-answer vectors
  * jax.random split/bits/uniform, non-partitionable layout
        ................................ published JAX values (PRNGKey(0) split
                                         and uniform) -- see tests/test_oracle_prng.py
  * jax.random partitionable layout .... PARITY UNPINNED (no JAX available; the
                                         layout is restated from upstream JAX)
  * int numerics / abs-max scales ...... closed forms + reference known-answer
                                         tests (aqt_dot_general_test.py:1079-1209)
  * fp8 RTNE casts ..................... reference golden arrays
                                         (numerics/fp8_numerics_test.py:50-110,221-242)
                                         + torch.float8 casts (library routine)
  * bf16 rounding ...................... torch.bfloat16 casts (library routine)
  * int8 GEMM .......................... exact integer arithmetic (brute force)
  * fwd/bwd dimension numbers .......... float dot_general + hand gradients
  * tiling / LocalAqt .................. reference known-answer tests
  * fp8 SR (fp_mantissa_round) ......... closed form on bit patterns; the random
                                         bits feeding it inherit the PRNG pins
  * order of float32 sums (over tiles, over LocalAqt shards, inside an fp8
    contraction) ....................... PARITY UNPINNED (XLA-internal); sums here
                                         run in index order, fp8 dots are exact in
                                         float64 and rounded once
  * dequant with scales of different dtypes
        ................................ jnp promotion rule, product by product
                                         (bf16*bf16 -> bf16, anything with f32 -> f32)
"""
