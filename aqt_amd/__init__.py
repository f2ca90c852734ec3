"""aqt_amd: MI355X (gfx950) kernels behind the aqt.jax.v2 quantized dot_general API."""
__version__ = '0.1.0'
