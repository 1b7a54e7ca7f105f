"""MI355X-native CSR SpMV / SpMM behind the AlphaSparse generic API.

The product is the shared library ``libalphasparse_amd.so`` (HIP kernels + C-ABI + the C++
``alphasparseSpMV`` / ``alphasparseSpMM`` entry points).  This Python package only holds the
build recipe, a ctypes view of the C-ABI used by tests and the benchmark, and the synthetic
workload generators.
"""
