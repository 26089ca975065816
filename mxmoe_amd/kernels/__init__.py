"""Python side of the kernel generator: the same module names as the reference's `mxmoe/kernels` package."""
