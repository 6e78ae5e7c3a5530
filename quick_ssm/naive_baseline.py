"""`quick_ssm.naive_baseline` import path of the reference, served by quick_ssm_amd."""
from quick_ssm_amd.naive_baseline import naive_backward_3d, naive_forward_3d, naive_full_3d  # noqa: F401
