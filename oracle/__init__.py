"""CPU oracle for the quantized-weight matmul path (test infrastructure only).

Two independent restatements of the same documented algorithm live here:
``cref`` binds the C library built from ``gllmq_oracle.c`` and ``npref`` is a
vectorised numpy formulation written element-wise instead of loop-wise.  Tests,
the smoke check and the CPU-baseline leg of the benchmark are the only callers;
nothing under ``gllm_amd`` imports this package.
"""
