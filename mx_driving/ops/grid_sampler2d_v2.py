"""Module path of the reference's operator file (mx_driving/ops/grid_sampler2d_v2.py:18-73)."""
from drivingsdk_amd.ops.grid_sampler2d_v2 import GridSampler2dV2Function, grid_sampler2d_v2  # noqa: F401
