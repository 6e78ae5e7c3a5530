"""Legacy module name: the device forward is a HIP kernel now; the entry point keeps its name."""
from quick_ssm_amd.hip_scan import block_scan_forward_3d  # noqa: F401
