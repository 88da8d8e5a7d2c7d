"""Module path of the reference's patcher for the one patch this repository provides
(reference: mx_driving/patcher/mmcv_patch.py:36-69)."""
from drivingsdk_amd.patcher import (  # noqa: F401
    APPLIED,
    FAILED,
    SKIPPED,
    AtomicPatch,
    MultiScaleDeformableAttention,
    apply_patches,
)

__all__ = ["AtomicPatch", "MultiScaleDeformableAttention", "apply_patches", "APPLIED", "SKIPPED", "FAILED"]
