"""JAX-ROCm binding of libgla_hip.so through XLA FFI custom calls: source only (see gla_jax.py)."""
