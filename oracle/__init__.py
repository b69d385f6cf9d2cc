"""CPU oracle for the conv_nd / max_pool path.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package (``mygrad_amd``) may import from here; only the
tests, the smoke check and the CPU-baseline leg of the benchmark use it, and
only as the checker.

Modules
-------
np_oracle   NumPy restatement of the reference algorithm (same library calls
            in the same order: pad -> strided window view -> tensordot ->
            col2im loop; reshape -> argmax -> add.at).
brute       Independent definition-level loops for tiny inputs (pins np_oracle).
direct      ctypes binding of ``direct_ref.c``: definition-level loops in C with
            OpenMP, usable at the full benchmark sizes.
"""
