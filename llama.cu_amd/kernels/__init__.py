"""The native libraries: building, loading, and the kernels as Python functions."""
