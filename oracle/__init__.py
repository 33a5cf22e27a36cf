"""CPU oracle for the GEMM -> dense-layer -> row-primitive path.  TEST INFRASTRUCTURE ONLY.

This package restates, in NumPy, the semantics of the reference's Spiral sources
(ml/matmul/kernel.spi, ml/layers.spi, ml/primitives.spi, corecuda/random.spi).  It exists to
check the HIP library; it is never a fallback.  Only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py may import it.

Pinning status of each function (what checks it besides its own formula):

  philox.philox4x32_10 / curand_uniform   pinned: replays every sampled index stored in the
                                           reference's golden outputs (tests/test_oracle_golden.py)
                                           and the Random123 known-answer vectors
  row_ops.softmax / masked_softmax        pinned: golden output_softmax*.txt, output_masked_softmax.txt
  row_ops.ln_l2                           pinned: golden output_ln.txt
  row_ops.argmax                          pinned: golden output_argmax.txt
  row_ops.inclusive_scan_sum              pinned: golden output_softmax_scan.txt (2nd component)
  row_ops.exclusive_scan                  pinned: golden output_sum_exclusive.txt (exact, integer)
  row_ops.masked_regret_matching          pinned: golden test3 output_op_map.txt (incl. sum==0 branch)
  row_ops.regret_matching                 pinned: equals masked_regret_matching with a full mask + closed forms
  row_ops.discrete_sampling               pinned: golden output_sampling*.txt, output_sample_reduce.txt
  row_ops.reduce_sum                      pinned: golden test6 (closed form 134209536)
  row_ops.transpose_inner                 pinned: golden test5 transpose.txt
  row_ops.l1_normalize                    PARITY UNPINNED against the reference (no output of it is stored);
                                           pinned mathematically: rows under the threshold come back as their
                                           absolute values, rows above it sum to the threshold and keep their
                                           proportions, a negative entry comes back positive, the l2 norm is not
                                           what is clamped (tests/test_oracle_math.py)
  row_ops.reduce_all                      NumPy's own sum / prod / max / min over the flattened tensor (library
                                           routines); the u64 sum reproduces golden test6
  gemm.gemm_abt                           PARITY UNPINNED against the reference (it stores no GEMM
                                           vectors; its self-test only prints a max-abs-diff,
                                           ml/matmul/run.spi:54-58).  Pinned mathematically instead:
                                           brute-force triple loop, identity operand, exactly
                                           representable integer inputs, alpha/beta algebra, f64 bound
  layers.mlp_forward                      PARITY UNPINNED end to end (the reference's layer goldens
                                           hold inputs truncated to 100 values).  It is a composition
                                           of gemm_abt and the pinned row ops; checked by closed forms
"""
from . import philox, row_ops, gemm, layers  # noqa: F401
