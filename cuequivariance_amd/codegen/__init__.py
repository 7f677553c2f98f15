"""Build-time generators of descriptor-specialised HIP kernels."""
