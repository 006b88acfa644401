"""CPU oracle for the attention column-mean path.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package imports this directory.  It is used by the tests, by the
smoke check and by the CPU-baseline leg of the benchmark, always as the checker or the
reported baseline and never as the thing under test.

Contents
  naive_colsum.py   eager-torch restatement of the reference oracle
                    (reference: flash_colsum/baselines.py:13-78) plus a memory-bounded
                    exact variant for shapes whose score matrix does not fit in RAM.
  colsum_ref.c      plain-C float64 restatement (triple loop, no BLAS, no torch),
                    built by oracle/Makefile into oracle/libcolsum_ref.so.
  c_ref.py          ctypes loader for that library.

Parity pins (all in tests/test_oracle.py, none of them re-types the formula):
  * brute-force pure-Python float64 loops on tiny shapes,
  * closed forms: uniform rows (Q = 0) and the harmonic-sum profile of the aligned
    causal mask,
  * torch.nn.functional.scaled_dot_product_attention with V = I (and the library's own
    lower-right causal bias) as an independent implementation,
  * invariances (key shift, scale/Q trade, key/head/row permutations) and the one-hot
    limit at very large scale,
  * committed golden vectors under tests/golden/ written by the pure-Python brute force.
`colsum_ext_exact` / `colsum_ref_ext` (grouped key heads, batched causal calls, causal calls
restricted to their first rows, explicit k_past, S_q != S_k) go beyond the reference operator's
domain; they are pinned by their own brute-force vectors (tests/golden/colsum_ext_golden.npz),
by scaled_dot_product_attention with enable_gqa, by the harmonic closed form with an explicit
k_past and by reduction to the pinned functions above when the extension is not used.
The reference ships no golden vectors or known-answer values for this path.
"""
from .naive_colsum import naive_colsum, colsum_exact, colsum_ext_exact, visible  # noqa: F401
