"""CPU oracle for the hot path: TEST INFRASTRUCTURE ONLY.

A plain-numpy restatement of what the reference computes for this path when it runs under
TRITON_INTERPRET=1 (python/triton/runtime/interpreter.py), plus closed forms that pin it.
Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may import this
package, and only as the checker.  Nothing under triton_amd/ imports it: the product path
is the HIP library and fails loudly without it.

Parity status per function (what pins it):
  formats.*            closed forms, cross-checked three ways (reference format table
                       test_conversions.py:295-303, its up-cast emulation :178-209, the restated
                       interpreter up-cast interpreter.py:130-191, torch's fp8 views)    PINNED
  gemm.matmul_tiled    against gemm.matmul_closed_form (fp64) and exact small-integer KATs
                       (test_cublas.py:28-49 construction); pid mapping by brute force      PINNED
  attention.*_tiled    against attention.*_closed_form (fp64 softmax / analytic gradients),
                       invariants (row sums, M = logsumexp/ln2, causal O[0] = V[0])          PINNED
  mx.*                 e2m1 / e8m0 tables and mx_matmul: the reference snapshot has no MX code
                       at all, so these are pinned only by the OCP MX v1.0 closed forms and
                       exactness KATs                               PARITY UNPINNED by the reference
"""
