"""``mx_driving._C`` -- the module path of the reference's compiled binding (mx_driving/csrc/pybind.cpp,
mx_driving/_C/__init__.pyi), so that the reference's own operator files, which do ``import mx_driving._C``
(mx_driving/ops/multi_scale_deformable_attn.py:15,38), resolve here.  Every function is the one of
``drivingsdk_amd._C`` (ctypes over libmxd_msda.so); the names are those the reference binds
(pybind.cpp:110-111 multi-scale deformable attention, :121-122 deformable aggregation, :131-132 geometric kernel
attention, :205-208 grid sampler)."""
from drivingsdk_amd._C import (  # noqa: F401
    deformable_aggregation,
    deformable_aggregation_backward,
    geometric_kernel_attention_backward,
    geometric_kernel_attention_forward,
    grid_sampler2d_v2,
    grid_sampler2d_v2_backward,
    msda_fused_backward,
    msda_fused_forward,
    multi_scale_deformable_attn,
    multi_scale_deformable_attn_backward,
)

# the names under which the reference exports deformable aggregation (pybind.cpp:121-122)
npu_deformable_aggregation = deformable_aggregation
npu_deformable_aggregation_backward = deformable_aggregation_backward
