"""HIP kernels and their Python entry points."""
