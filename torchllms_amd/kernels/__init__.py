"""Python side of the HIP kernels: build, load, and call."""
