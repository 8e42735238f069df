"""TEST INFRASTRUCTURE ONLY.

CPU oracle for the submanifold-conv hot path: a restatement of the reference's algorithms
(`subm_ref.c` for the integer tables, `explicit_gemm.py` for the explicit gather-GEMM) plus
independent definition-level builders (`definitions.py`) used to pin the restatement.

Only tests/, the smoke check and the bench's cpu_baseline leg may import this package, and
only as the checker.  The shipped package (`flexgemm_amd`, `flex_gemm`) never does.
"""
