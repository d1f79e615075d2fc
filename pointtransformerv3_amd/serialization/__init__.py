"""Curve codes with the call signature of the reference's serialization package
(serialization/default.py:8-24); the arithmetic runs in the fused HIP encode kernel."""
from .default import ORDERS, encode

__all__ = ["encode", "ORDERS"]
