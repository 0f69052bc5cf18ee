"""Plain-torch baselines the harness times and verifies the HIP kernels against (GPU or CPU tensors)."""
