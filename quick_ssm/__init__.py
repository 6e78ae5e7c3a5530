"""Drop-in import path: `import quick_ssm` resolves to the MI355X implementation in quick_ssm_amd."""
from quick_ssm_amd import RMSNorm, SSM, scan

__all__ = ["scan", "SSM", "RMSNorm"]
