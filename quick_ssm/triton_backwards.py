"""Legacy module name: the device backward is a HIP kernel now; the entry point keeps its name."""
from quick_ssm_amd.hip_scan import block_scan_backward_3d  # noqa: F401
