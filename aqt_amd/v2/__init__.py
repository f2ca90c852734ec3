"""Mirror of the aqt.jax.v2 quantized dot_general API on torch tensors + HIP kernels."""
