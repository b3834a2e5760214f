"""CPU restatements of the three operators, used only to check the HIP kernels.

TEST INFRASTRUCTURE, NOT PRODUCT. Nothing on the product path (the HIP sources, the C-ABI
library, the workspace ``ModelNew`` classes) imports, links or falls back to this package;
only the tests, the smoke entry and the CPU-baseline leg of the benchmark do.

The reference repository holds no implementation of these operators (its only operator is
``alpha*a+b``, agent_workdir/model.py:15-16), so each function restates the operator's
definition from the workload specification and is pinned by closed forms, brute force,
library special cases and golden fixtures instead of by reference vectors; every module's
header lists what pins it.
"""
