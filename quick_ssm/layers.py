"""`quick_ssm.layers` import path of the reference, served by quick_ssm_amd."""
from quick_ssm_amd.layers import RMSNorm, SSM  # noqa: F401

__all__ = ["SSM", "RMSNorm"]
