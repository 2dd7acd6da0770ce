"""CPU oracle for the KV-cache compression hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
directory: it exists so that tests, the smoke check and the benchmark's
CPU-baseline leg can compare the HIP kernels against an independent numpy / C
restatement of the reference algorithms.  Every function cites the reference
file:line it restates (paths relative to the VeloxQuant-MLX source tree).

Parity pinning status (which external facts each function is checked against
lives in tests/test_oracle_*.py):

* group quantisation, packing, dequantisation, decode attention, causal
  prefill attention, attention from codebook indices with its sliding-window
  mask, cache frontier arithmetic, the Kitty channel ranking / mixed round trip /
  accounting, the AgeTieredKV tiers / windows / bytes: pinned (hand-computed known answers, the reference tests' own seeded
  cases, closed forms, invariants, brute force, library SDPA).
* ``quantize_vq`` on exact fp32 near-ties: PARITY UNPINNED against MLX's
  ``mx.sum`` reduction order and ``mx.argmin`` tie order (MLX is not
  installable here).  The oracle fixes the order the reference's Metal twin
  uses: separately rounded squares, left-to-right fp32 sum, strict ``<``
  (lowest index wins).
* Kitty's channel ranking between channels whose float32 variances differ only in
  the last bits: PARITY UNPINNED (the reduction order of ``mx.var`` is not
  reproducible without MLX); parity inputs keep the channel spreads apart.
* default random codebooks drawn from ``mx.random``: PARITY UNPINNED (MLX's
  RNG stream is not reproducible without MLX); all parity inputs pass
  explicit codebooks.
"""
