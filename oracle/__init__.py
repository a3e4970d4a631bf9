"""TEST INFRASTRUCTURE -- not part of the product.

CPU checkers for the FluidML hot path:
  oracle.kernels      ctypes door onto liboracle_kernels.so (kernels.c: the reference's loop nests in C)
  oracle.memory_plan  Python restatement of the reference's greedy / linear memory planner
  oracle.ref_memory   ctypes door onto _ref/libref_memory.so (the reference's own planner sources, compiled)

Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py import this package.
"""
