"""CPU oracle for the chunked delta-rule scan -- TEST INFRASTRUCTURE ONLY.

Nothing in ``linearnexus_amd`` may import this package.  It is the checker the
HIP kernels are compared against (tests, the smoke entry point and the
``cpu_baseline`` leg of the benchmark), never a fallback for them.

Modules
-------
recurrent   token-by-token forms and single steps (the ground truth),
            restated from the reference's ``*_recurrent`` / ``*_step`` ops.
chunkwise   the reference's chunk algorithms (explicit inverse for DeltaNet,
            16x16-blocked M/Aqk + forward substitution for Gated/KDA), a
            second, independent restatement.
adjoint     token-level reverse recurrence = gradient of the recurrent form.
staged      chunk-level forward and backward split exactly the way the HIP
            kernels are split, exposing every intermediate tensor.
inputs      shared synthetic-input generator (numpy ``default_rng``).

Pinning status (see the tests under ``tests/test_oracle_*.py``): every
function is pinned by closed forms, brute-force matrix products on tiny
inputs, reductions between the variants, central finite differences (fp64)
and ``torch.autograd`` on an independent torch restatement.  The reference
holds no golden vectors for this path, and its JAX code cannot run in this
environment (jax is not installed), so no value here was produced by the
reference itself.
"""
