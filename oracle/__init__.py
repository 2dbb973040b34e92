"""CPU oracle for the quantized-linear hot path.

THIS PACKAGE IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It restates, in plain
numpy (and in plain C under ``oracle/c`` for timing), the arithmetic that the
reference framework performs on this path, so that the HIP kernels can be
checked against it.  Only the test-suite, the smoke check and the
``cpu_baseline`` leg of the benchmark may import it; nothing under
``minit_amd/`` does, and the product path raises when its HIP library is
missing instead of falling back to anything in here.

How each function is pinned (the reference ships no tests or golden vectors,
so none of this is pinned by the reference's own fixtures):

* ``gptq.unpack``      closed-form shift/mask; cross-checked against a second,
                       independent restatement of the reference's view algebra
                       (byte reinterpretation on a little-endian host) and
                       against known-answer words such as 0x76543210.
* ``gptq.dequantize``  closed form; special cases (q == z+1 -> 0, scale == 1 ->
                       integers), float64 evaluation rounded once.
* ``gptq.matmul``      reduces to a float64 library matmul; one-hot rows pick
                       rows of the dequantized matrix; linearity.
* ``int8.gemm_i32``    exact integer arithmetic; brute-force loops on tiny
                       shapes and an int64 library matmul.
* ``special.*``        closed forms in float64; invariants (rows of softmax sum
                       to one, RoPE at position 0 is the identity and composes
                       additively, RMSNorm of a constant row is sign * weight,
                       the sum of ones is the row length).
* ``decode.*``         a known-answer decode step computed scalar by scalar
                       with python floats (two layers, grouped heads, rows at
                       different positions) held bit for bit, and constructed
                       models whose logits the mathematics fixes (zeroed o and
                       down projections, one visible cache entry, a zero norm
                       weight, batch-row permutations); seeded slips in the
                       operator order fail them.

The checks live in ``tests/test_oracle_*.py``; no function here is left
unpinned.
"""
