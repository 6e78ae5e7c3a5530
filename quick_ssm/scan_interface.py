"""`quick_ssm.scan_interface` import path of the reference, served by quick_ssm_amd."""
from quick_ssm_amd.scan_interface import (  # noqa: F401
    _HipScanFunction,
    _TritonScanFunction,
    _chunk_ranges,
    _torch_scan,
    honor_tiles,
    scan,
    scan_chunk,
)

__all__ = ["scan"]
