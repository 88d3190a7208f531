"""Fusion-IR graphs used by the parity tests (the benchmark configurations live in helium_amd.configs)."""
from helium_amd.configs import c3_chain  # noqa: F401
