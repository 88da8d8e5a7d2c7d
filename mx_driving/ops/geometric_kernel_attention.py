"""Module path of the reference's operator file (mx_driving/ops/geometric_kernel_attention.py:29-57)."""
from drivingsdk_amd.ops.geometric_kernel_attention import (  # noqa: F401
    GeometricKernelAttentionFunc,
    geometric_kernel_attention,
)
