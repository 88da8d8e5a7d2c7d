"""Loader for libmxd_msda.so, the C-ABI library declared in include/mxd_msda.h.

The library is built in-tree (``drivingsdk_amd/lib/libmxd_msda.so``) by
``drivingsdk_amd.build.build()`` / ``make -C drivingsdk_amd/csrc``.  There is no other
implementation behind this package: if the library is missing, loading fails loudly.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libmxd_msda.so")

DTYPE_F32, DTYPE_F16, DTYPE_BF16 = 0, 1, 2
BWD_ACCUMULATE = 1
META_I64 = 0x100  # OR into a dtype code: level metadata tensors hold int64 elements

EXPORTS = (
    "mxd_msda_version",
    "mxd_msda_last_error",
    "mxd_msda_init",
    "mxd_msda_reload_tuning",
    "mxd_msda_make_plan",
    "mxd_msda_decode_block",
    "mxd_msda_forward",
    "mxd_msda_fused_forward",
    "mxd_msda_fused_backward_workspace_bytes",
    "mxd_msda_fused_backward",
    "mxd_msda_backward_workspace_bytes",
    "mxd_msda_backward",
    "mxd_msda_backward_static_limit",
    "mxd_msda_backward_static",
    "mxd_dagg_forward",
    "mxd_dagg_backward_workspace_bytes",
    "mxd_dagg_backward",
    "mxd_gka_forward",
    "mxd_gka_backward_workspace_bytes",
    "mxd_gka_backward",
    "mxd_grid_sampler2d_forward",
    "mxd_grid_sampler2d_backward_workspace_bytes",
    "mxd_grid_sampler2d_backward",
)


class Plan(ctypes.Structure):
    """Mirror of ``mxd_msda_plan`` (include/mxd_msda.h)."""

    _fields_ = [(n, ctypes.c_int32) for n in (
        "vec", "lanes_per_row", "npass", "units_per_wave", "waves_per_block", "iters", "tile_q", "ntiles",
        "xcd_mode", "heads_per_xcd", "xcds_per_head", "tiles_per_part")] + [
        (n, ctypes.c_uint32) for n in ("grid", "block", "lds_bytes")]

    def as_dict(self):
        return {n: getattr(self, n) for n, _ in self._fields_}


_lib = None


def load():
    """Return the ctypes handle of the library, loading it on first use."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: the HIP library has not been built "
            "(run `python -c 'import __graft_entry__ as g; g.build()'` or `make -C drivingsdk_amd/csrc`). "
            "This package has no CPU or eager fallback.")
    lib = ctypes.CDLL(LIB_PATH)
    i64, p, ci = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int
    lib.mxd_msda_version.restype = ci
    lib.mxd_msda_version.argtypes = []
    lib.mxd_msda_last_error.restype = ctypes.c_char_p
    lib.mxd_msda_last_error.argtypes = []
    lib.mxd_msda_init.restype = ci
    lib.mxd_msda_init.argtypes = []
    lib.mxd_msda_reload_tuning.restype = None
    lib.mxd_msda_reload_tuning.argtypes = []
    lib.mxd_msda_make_plan.restype = ci
    lib.mxd_msda_make_plan.argtypes = [ci, ci] + [i64] * 8 + [ci, ctypes.POINTER(Plan)]
    lib.mxd_msda_decode_block.restype = ci
    lib.mxd_msda_decode_block.argtypes = [ctypes.POINTER(Plan), ctypes.c_uint32, i64, i64, i64,
                                          ctypes.POINTER(ctypes.c_int32 * 4)]
    lib.mxd_msda_forward.restype = ci
    lib.mxd_msda_forward.argtypes = [p] * 6 + [ci] + [i64] * 8 + [p]
    lib.mxd_msda_fused_forward.restype = ci
    lib.mxd_msda_fused_forward.argtypes = [p] * 4 + [ci] + [p] * 3 + [ci] + [i64] * 7 + [p]
    lib.mxd_msda_fused_backward_workspace_bytes.restype = ctypes.c_size_t
    lib.mxd_msda_fused_backward_workspace_bytes.argtypes = [ci] + [i64] * 7 + [ci, ci]
    lib.mxd_msda_fused_backward.restype = ci
    lib.mxd_msda_fused_backward.argtypes = [p] * 4 + [ci] + [p] * 9 + [ctypes.c_size_t, ci] + [i64] * 7 + [ci, p]
    lib.mxd_msda_backward_workspace_bytes.restype = ctypes.c_size_t
    lib.mxd_msda_backward_workspace_bytes.argtypes = [ci] + [i64] * 8
    lib.mxd_msda_backward.restype = ci
    lib.mxd_msda_backward.argtypes = [p] * 10 + [ctypes.c_size_t, ci] + [i64] * 8 + [ci, p]
    lib.mxd_msda_backward_static_limit.restype = ctypes.c_size_t
    lib.mxd_msda_backward_static_limit.argtypes = []
    lib.mxd_msda_backward_static.restype = ci
    lib.mxd_msda_backward_static.argtypes = [p] * 9 + [ci] + [i64] * 8 + [ci, p]
    lib.mxd_dagg_forward.restype = ci
    lib.mxd_dagg_forward.argtypes = [p] * 6 + [ci] + [i64] * 8 + [p]
    lib.mxd_dagg_backward_workspace_bytes.restype = ctypes.c_size_t
    lib.mxd_dagg_backward_workspace_bytes.argtypes = [ci] + [i64] * 8
    lib.mxd_dagg_backward.restype = ci
    lib.mxd_dagg_backward.argtypes = [p] * 10 + [ctypes.c_size_t, ci] + [i64] * 8 + [p]
    lib.mxd_gka_forward.restype = ci
    lib.mxd_gka_forward.argtypes = [p] * 6 + [ci] + [i64] * 7 + [p]
    lib.mxd_gka_backward_workspace_bytes.restype = ctypes.c_size_t
    lib.mxd_gka_backward_workspace_bytes.argtypes = [ci] + [i64] * 7
    lib.mxd_gka_backward.restype = ci
    lib.mxd_gka_backward.argtypes = [p] * 9 + [ctypes.c_size_t, ci] + [i64] * 7 + [p]
    lib.mxd_grid_sampler2d_forward.restype = ci
    lib.mxd_grid_sampler2d_forward.argtypes = [p] * 3 + [ci] + [i64] * 6 + [ci] * 3 + [p]
    lib.mxd_grid_sampler2d_backward_workspace_bytes.restype = ctypes.c_size_t
    lib.mxd_grid_sampler2d_backward_workspace_bytes.argtypes = [ci] + [i64] * 6
    lib.mxd_grid_sampler2d_backward.restype = ci
    lib.mxd_grid_sampler2d_backward.argtypes = [p] * 6 + [ctypes.c_size_t, ci] + [i64] * 6 + [ci] * 3 + [p]
    _lib = lib
    return lib


def reload_tuning():
    """Have the library read its MXD_MSDA_* environment variables again (they are read once per process)."""
    load().mxd_msda_reload_tuning()


def last_error():
    return load().mxd_msda_last_error().decode("utf-8", "replace")


def make_plan(backward, dtype_code, bs, nk, nh, hd, nl, nl_attn, nq, npts, align_bytes=16):
    """Launch geometry for a problem (no GPU needed).  Raises RuntimeError on bad sizes."""
    plan = Plan()
    rc = load().mxd_msda_make_plan(int(bool(backward)), dtype_code, bs, nk, nh, hd, nl, nl_attn, nq, npts,
                                   align_bytes, ctypes.byref(plan))
    if rc != 0:
        raise RuntimeError(last_error())
    return plan
