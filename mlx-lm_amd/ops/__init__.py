"""HIP kernels of the engine: building, loading and launching them."""
