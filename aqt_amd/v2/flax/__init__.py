"""Module-level callers of the quantized dot_general (counterparts of aqt/jax/v2/flax)."""
