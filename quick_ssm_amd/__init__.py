"""quick_ssm on MI355X: the gated linear scan as hand-written HIP kernels for gfx950.

Public surface is the reference's (quick_ssm/__init__.py:1-4): `scan`, `SSM`, `RMSNorm`, plus
`scan_chunk`, the same scan with the state carried in and out (chunked prefill, generation).
"""
from .scan_interface import scan, scan_chunk
from .layers import SSM, RMSNorm

__all__ = ["scan", "scan_chunk", "SSM", "RMSNorm"]
__version__ = "0.2.0"
