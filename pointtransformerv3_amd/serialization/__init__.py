"""Curve codes with the call signatures of the reference's serialization package
(serialization/__init__.py:1-8, default.py:8-60); the arithmetic runs in the HIP encode / decode kernels."""
from .default import ORDERS, decode, encode, hilbert_decode, hilbert_encode, z_order_decode, z_order_encode

__all__ = ["encode", "decode", "z_order_encode", "z_order_decode", "hilbert_encode", "hilbert_decode", "ORDERS"]
