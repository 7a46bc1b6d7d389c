"""Utilities: seeded synthetic workloads."""
from . import synthetic  # noqa: F401
