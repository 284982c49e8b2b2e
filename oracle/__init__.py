"""CPU oracle for the fused elementwise / reduction / flex16 path.

TEST INFRASTRUCTURE ONLY.  Nothing in the product package imports this
directory; only tests/, __graft_entry__.smoke() and the cpu_baseline leg of
bench.py do, and only as the checker.  Each module restates, in NumPy, what the
reference's CPU transformer (ngraph/transformers/cputransform.py) or its flex
device code (ngraph/transformers/gpu/float_ew2.py) computes, citing the lines
it follows.

Pinning status (what checks each restatement beyond itself):
  numpy_ops.py      closed forms: each entry IS the NumPy ufunc call the CPU
                    transformer emits; tests/test_cabi_fused_gpu.py and
                    tests/test_execution.py check them against float64 references
                    and NumPy expressions written in each test.  Its integer ops
                    (int32 / uint32 operands) are pinned against arithmetic on
                    Python integers modulo 2^32 in tests/test_oracle_integer_ops.py.
  configs.py        BatchNorm / Adam / LSTM pinned against independent float64
                    restatements of the reference's own test references
                    (neon/tests/test_batchnorm_layer.py:35-58,
                    test_optimizer.py:103-135, lstm_ref.py) in tests/.
  flex_model.py     rounding / saturation / maxabs given scales: pinned by
                    brute force over all int16 values and by the reference's
                    known-answer vectors (tests/golden/flex_vectors.json).
                    Exponent policy (next_dec): the reference delegates it to
                    the private `autoflex` package, which is not in the tree;
                    PARITY UNPINNED at source level, pinned at the boundary by
                    all 154 vectors the reference itself enables (the 9 it
                    disables are flagged inside the fixture).
  cpu_transformer.py evaluates op graphs op by op with numpy_ops; pinned by the
                    NumPy expressions written in each test, as the reference's
                    own tests do.
"""
