"""mmcv entry point of multi-scale deformable attention: swap this library's kernels in.

Models written against mmcv call ``mmcv.ops.multi_scale_deform_attn.MultiScaleDeformableAttnFunction``
with one extra positional argument (``im2col_step``) and expect one gradient per forward argument.
The reference SDK adapts its own Function to that calling convention with two wrappers and swaps
them into mmcv at import time (mx_driving/patcher/mmcv_patch.py:36-69: ``forward`` drops
``im2col_step``, ``backward`` appends ``None`` for it).  This module is the same adaptation for the
HIP operator, with a deliberately small patch mechanism:

    from mx_driving.patcher import MultiScaleDeformableAttention, apply_patches
    apply_patches(MultiScaleDeformableAttention.patches())      # no-op when mmcv is not installed

``AtomicPatch(target, replacement, replacement_wrapper=None)`` replaces one attribute named by a
dotted path (module path followed by attribute path).  ``apply()`` reports ``"applied"``,
``"skipped"`` (the target module or attribute does not exist) or ``"failed"``; ``restore()``
puts the original back.  Only what this one operator needs is provided; the reference's
registry/legacy patch kinds, import skipping and reporting are not part of the hot path.
"""
import importlib
from typing import Callable, List, Optional, Tuple

__all__ = ["AtomicPatch", "MultiScaleDeformableAttention", "apply_patches", "APPLIED", "SKIPPED", "FAILED"]

APPLIED, SKIPPED, FAILED = "applied", "skipped", "failed"


def _resolve(path: str) -> Tuple[object, str, object]:
    """(parent object, attribute name, current value) of a dotted path whose leading part is the
    longest importable module name.  Raises ImportError / AttributeError when it does not exist."""
    parts = path.split(".")
    if len(parts) < 2:
        raise AttributeError(f"'{path}' names no attribute of a module")
    module, err = None, None
    for cut in range(len(parts) - 1, 0, -1):
        try:
            module = importlib.import_module(".".join(parts[:cut]))
            break
        except ImportError as e:  # try a shorter module path
            err = e
    if module is None:
        raise ImportError(f"no importable module in '{path}'") from err
    parent = module
    for name in parts[cut:-1]:
        parent = getattr(parent, name)
    return parent, parts[-1], getattr(parent, parts[-1])


class AtomicPatch:
    """Replace the attribute ``target`` by ``replacement`` (an object or a dotted path to one),
    passed through ``replacement_wrapper`` first when given."""

    def __init__(self, target: str, replacement, replacement_wrapper: Optional[Callable] = None):
        self.target = target
        self.replacement = replacement
        self._replacement_wrapper = replacement_wrapper
        self._undo = None
        self.status = None
        self.reason = ""

    @property
    def name(self) -> str:
        return self.target

    def apply(self) -> str:
        try:
            parent, attr, original = _resolve(self.target)
        except (ImportError, AttributeError) as e:
            self.status, self.reason = SKIPPED, str(e)
            return self.status
        try:
            new = _resolve(self.replacement)[2] if isinstance(self.replacement, str) else self.replacement
            if self._replacement_wrapper is not None:
                new = self._replacement_wrapper(new)
            setattr(parent, attr, new)
        except Exception as e:  # replacement missing or the target refuses assignment
            self.status, self.reason = FAILED, f"{type(e).__name__}: {e}"
            return self.status
        self._undo = (parent, attr, original)
        self.status, self.reason = APPLIED, ""
        return self.status

    def restore(self) -> None:
        if self._undo is not None:
            parent, attr, original = self._undo
            setattr(parent, attr, original)
            self._undo = None
            self.status = None


class MultiScaleDeformableAttention:
    """The mmcv patch of the operator (same name, legacy name and targets as the reference's)."""

    name = "multi_scale_deformable_attention"
    legacy_name = "msda"
    target_module = "mmcv"

    @classmethod
    def patches(cls, options=None) -> List[AtomicPatch]:
        base = "mmcv.ops.multi_scale_deform_attn.MultiScaleDeformableAttnFunction"
        ours = "mx_driving.MultiScaleDeformableAttnFunction"

        def forward_wrapper(our_forward):
            # mmcv passes im2col_step (a CUDA batching knob); it has no meaning here
            def forward(ctx, value, spatial_shapes, level_start_index, sampling_locations, attention_weights,
                        im2col_step=None):
                return our_forward(ctx, value, spatial_shapes, level_start_index, sampling_locations,
                                   attention_weights)
            return forward

        def backward_wrapper(our_backward):
            # one more None: the gradient slot of im2col_step
            def backward(ctx, grad_output):
                return (*our_backward(ctx, grad_output), None)
            return backward

        return [
            AtomicPatch(f"{base}.forward", f"{ours}.forward", replacement_wrapper=forward_wrapper),
            AtomicPatch(f"{base}.backward", f"{ours}.backward", replacement_wrapper=backward_wrapper),
        ]


def apply_patches(patches: List[AtomicPatch]) -> List[Tuple[str, str]]:
    """Apply every patch; returns [(target, status)].  Missing targets are skipped, not errors."""
    return [(p.target, p.apply()) for p in patches]
