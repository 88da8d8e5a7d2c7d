"""Host-side checks that need no GPU: the C-ABI library loads and exports what the header
declares, argument checking, launch geometry, and the error behaviour of the Python layer."""
import ctypes
import os
import re

import pytest
import torch

import drivingsdk_amd
import mx_driving
from conftest import ROOT
from drivingsdk_amd import _C, _lib, workloads


def test_library_exports_every_declared_symbol():
    with open(os.path.join(ROOT, "include", "mxd_msda.h")) as f:
        header = f.read()
    declared = set(re.findall(r"\b(mxd_(?:msda|dagg|gka|grid_sampler2d)_[a-z_]+)\s*\(", header))
    declared.discard("mxd_msda_plan")
    assert declared == set(_lib.EXPORTS)
    lib = _lib.load()
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.mxd_msda_version() == 103


def test_public_names_match_the_reference_module():
    for mod in (mx_driving, drivingsdk_amd):
        assert mod.multi_scale_deformable_attn == mod.MultiScaleDeformableAttnFunction.apply
        assert callable(mod.npu_multi_scale_deformable_attn_function)
    assert mx_driving._C.multi_scale_deformable_attn is _C.multi_scale_deformable_attn
    assert mx_driving._C.multi_scale_deformable_attn_backward is _C.multi_scale_deformable_attn_backward


@pytest.mark.parametrize("backward", [0, 1])
@pytest.mark.parametrize("dims", [
    # bs, nk, nh, hd, nl, nl_attn, nq, np
    (2, 19947, 8, 32, 4, 4, 19947, 4),
    (6, 30825, 8, 32, 4, 4, 9675, 8),
    (1, 19947, 8, 128, 4, 4, 19947, 4),
    (1, 2400, 5, 16, 3, 3, 27216, 1),
    (3, 2400, 4, 37, 5, 5, 301, 3),
    (1, 2400, 7, 147, 3, 3, 1450, 21),
    (2, 100, 16, 8, 1, 2, 33, 2),
    (1, 100, 1, 256, 1, 1, 1, 1),
    (2, 100, 2, 64, 2, 2, 1000, 4),
])
def test_plan_covers_every_unit_exactly_once(backward, dims):
    bs, nk, nh, hd, nl, nl_attn, nq, npts = dims
    lib = _lib.load()
    for dtype in (0, 1, 2):
        plan = _lib.make_plan(backward, dtype, *dims)
        assert plan.lanes_per_row * plan.units_per_wave == 64
        assert plan.vec * plan.lanes_per_row * plan.npass >= hd
        assert hd % plan.vec == 0
        assert plan.block == 64 * plan.waves_per_block
        if plan.block == 1024:
            # the forward's one-workgroup-per-CU form: a workgroup takes a whole CU's LDS and any multiple of
            # units_per_wave queries, its wavefronts taking groups of units_per_wave in turn
            assert not backward and plan.lds_bytes == 160 * 1024
            assert plan.tile_q % plan.units_per_wave == 0
            assert plan.tile_q <= plan.units_per_wave * plan.waves_per_block * plan.iters
        else:
            # the backward's first kernel gives queries of 25 to 32 samples two units each (16 samples per unit)
            # when its workgroups make one pass
            split = 2 if backward and 24 < nl * npts <= 32 and plan.iters == 1 and plan.units_per_wave >= 2 else 1
            assert plan.tile_q * split == plan.units_per_wave * plan.waves_per_block * plan.iters
            # two workgroups per CU (forward), the default dynamic LDS limit (backward)
            assert plan.lds_bytes <= (64 if backward else 80) * 1024
        seen = {}
        work = (ctypes.c_int32 * 4)()
        for bid in range(plan.grid):
            if not lib.mxd_msda_decode_block(ctypes.byref(plan), bid, bs, nh, nq, ctypes.byref(work)):
                continue
            b, h, q0, q1 = work
            assert 0 <= b < bs and 0 <= h < nh and 0 <= q0 < q1 <= nq and q1 - q0 <= plan.tile_q
            if plan.xcd_mode == 1:
                assert h // plan.heads_per_xcd == bid % 8   # a head never leaves its XCD
            elif plan.xcd_mode == 2:
                assert h == (bid % 8) % nh
            assert (b, h, q0) not in seen
            seen[(b, h, q0)] = q1
        covered = sum(q1 - q0 for (_, _, q0), q1 in seen.items())
        assert covered == bs * nh * nq
        assert len(seen) == bs * nh * plan.ntiles


def test_plan_vector_width_follows_alignment_and_head_dim():
    assert _lib.make_plan(0, 0, 1, 10, 1, 32, 1, 1, 1, 1, 16).vec == 4
    assert _lib.make_plan(0, 0, 1, 10, 1, 32, 1, 1, 1, 1, 8).vec == 2
    assert _lib.make_plan(0, 0, 1, 10, 1, 32, 1, 1, 1, 1, 4).vec == 1
    assert _lib.make_plan(0, 1, 1, 10, 1, 32, 1, 1, 1, 1, 16).vec == 8
    assert _lib.make_plan(0, 0, 1, 10, 1, 37, 1, 1, 1, 1, 16).vec == 1
    assert _lib.make_plan(0, 0, 1, 10, 1, 147, 1, 1, 1, 1, 16).npass == 4
    assert _lib.make_plan(0, 1, 1, 10, 1, 250, 1, 1, 1, 1, 16).vec == 2


@pytest.mark.parametrize("dims,fragment", [
    ((1, 10, 1, 257, 1, 1, 1, 1), "less than or equal to 256"),
    ((1, 10, 1, 32, 65, 65, 1, 1), "levels"),
    ((1, 10, 1, 32, 2, 1, 1, 1), "levels"),
    ((0, 10, 1, 32, 1, 1, 1, 1), "empty"),
    ((1, 1 << 22, 8, 32, 1, 1, 1, 1), "2 GiB"),
])
def test_c_abi_rejects_bad_sizes(dims, fragment):
    with pytest.raises(RuntimeError) as e:
        _lib.make_plan(0, 0, *dims)
    assert fragment in str(e.value)
    plan = _lib.Plan()
    assert _lib.load().mxd_msda_make_plan(0, 7, 1, 10, 1, 32, 1, 1, 1, 1, 16, ctypes.byref(plan)) == -1
    assert _lib.load().mxd_msda_make_plan(0, 0, 1, 10, 1, 32, 1, 1, 1, 1, 16, None) == -3


def test_workspace_size():
    lib = _lib.load()
    # bs 2, nk 100, nh 8, hd 32, nl 4, nq 50, np 3.  The first backward kernel runs 32-query workgroups for rows
    # of more than 32 bytes (eight units per wavefront: two workgroups per (batch, head) here) and 64-query ones
    # for shorter rows (sixteen units: one); a workgroup's slab holds two pair records (12 B) per sample (the
    # record area is padded to 256 bytes); the run
    # table has one column per possible tile (nk // 512 + nl) plus one per workgroup, padded to 256 bytes
    def expect(tile_q):
        nwg = -(-50 // tile_q)
        table = -(-(2 * 8 * nwg * (100 // 512 + 4 + 1) * 4) // 256) * 256
        return table + -(-(2 * 8 * nwg * (2 * tile_q * 4 * 3) * 12) // 256) * 256
    image = 2 * 100 * 8 * 32 * 4
    assert lib.mxd_msda_backward_workspace_bytes(0, 2, 100, 8, 32, 4, 4, 50, 3) == expect(32)
    assert lib.mxd_msda_backward_workspace_bytes(1, 2, 100, 8, 32, 4, 4, 50, 3) == expect(32) + image
    assert lib.mxd_msda_backward_workspace_bytes(2, 2, 100, 8, 32, 4, 4, 50, 3) == expect(32) + image
    image16 = 2 * 100 * 8 * 16 * 4
    assert lib.mxd_msda_backward_workspace_bytes(1, 2, 100, 8, 16, 4, 4, 50, 3) == expect(64) + image16
    assert lib.mxd_msda_backward_workspace_bytes(0, 2, 100, 8, 300, 4, 4, 50, 3) == 0  # invalid sizes


def _cpu_inputs(dtype=torch.float32):
    return workloads.reference_test_inputs([1, 7, 8, 2, 2, 3], dtype=dtype)


def test_binding_dtype_checks_raise_before_any_launch():
    inp = _cpu_inputs()
    sh, ls = inp.spatial_shapes.int(), inp.level_start_index.int()
    with pytest.raises(RuntimeError, match="value: float16, bfloat16 or float32"):
        _C.multi_scale_deformable_attn(inp.value.double(), sh, ls, inp.sampling_locations, inp.attention_weights)
    with pytest.raises(RuntimeError, match="value_spatial_shapes: int32 or int64"):
        _C.multi_scale_deformable_attn(inp.value, inp.spatial_shapes.float(), ls, inp.sampling_locations,
                                       inp.attention_weights)
    # int32 and int64 metadata are both taken, but not one of each
    with pytest.raises(RuntimeError, match="value_level_start_index: torch.int64 tensor"):
        _C.multi_scale_deformable_attn(inp.value, inp.spatial_shapes, ls, inp.sampling_locations,
                                       inp.attention_weights)
    with pytest.raises(RuntimeError, match="value_level_start_index: torch.int32 tensor"):
        _C.multi_scale_deformable_attn(inp.value, sh, inp.level_start_index, inp.sampling_locations,
                                       inp.attention_weights)
    with pytest.raises(RuntimeError, match="sampling_locations: float16"):
        _C.multi_scale_deformable_attn(inp.value, sh, ls, inp.sampling_locations.double(), inp.attention_weights)
    with pytest.raises(RuntimeError, match="attention_weights: float16"):
        _C.multi_scale_deformable_attn(inp.value, sh, ls, inp.sampling_locations, inp.attention_weights.long())
    big = torch.zeros(1, 4, 1, 257)
    with pytest.raises(RuntimeError, match="less than or equal to 256"):
        _C.multi_scale_deformable_attn(big, sh, ls, inp.sampling_locations, inp.attention_weights)
    with pytest.raises(RuntimeError, match="grad_output: float16"):
        _C.multi_scale_deformable_attn_backward(inp.value, sh, ls, inp.sampling_locations, inp.attention_weights,
                                                inp.grad_output.double())


def test_cpu_tensors_are_refused_not_silently_computed():
    inp = _cpu_inputs()
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        mx_driving.multi_scale_deformable_attn(inp.value, inp.spatial_shapes, inp.level_start_index,
                                               inp.sampling_locations, inp.attention_weights)


def test_empty_tensors_raise_plain_exception_like_the_reference():
    inp = _cpu_inputs()
    with pytest.raises(Exception, match="can not be a empty Tensor"):
        mx_driving.multi_scale_deformable_attn(inp.value[:0], inp.spatial_shapes, inp.level_start_index,
                                               inp.sampling_locations, inp.attention_weights)


def test_deprecated_alias_warns():
    inp = _cpu_inputs()
    with pytest.warns(DeprecationWarning):
        with pytest.raises(RuntimeError):
            mx_driving.npu_multi_scale_deformable_attn_function(
                inp.value, inp.spatial_shapes, inp.level_start_index, inp.sampling_locations, inp.attention_weights)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libmxd_msda.so"))
    with pytest.raises(ImportError, match="no CPU or eager fallback"):
        _lib.load()


def test_algorithmic_bytes_match_the_published_table():
    """Compulsory HBM bytes per call of the five workloads (decimal MB)."""
    mb = lambda name, dt=torch.float32, bwd=False: workloads.algorithmic_bytes(
        workloads.make_inputs(name, dtype=dt, scale_queries=1.0), backward=bwd) / 1e6
    assert abs(mb("tiny") - 4.87) < 0.01
    assert abs(mb("detr_encoder") - 142.98) < 0.01
    assert abs(mb("detr_encoder_bwd", bwd=True) - 245.11) < 0.01
    assert abs(mb("head_dim_128", torch.float16) - 97.02) < 0.01
    assert abs(mb("bevformer_sca") - 427.16) < 0.01
    assert abs(mb("bevformer_sca", torch.float16) - 213.58) < 0.01


def test_bench_refuses_more_than_one_gpu():
    """This build runs on one GPU: bench.py --gpus N (N > 1) says so and exits before touching a device."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 2 and "one GPU" in r.stderr and r.stdout.strip() == ""


def test_fused_backward_workspace_adds_the_reference_point_partials():
    lib = _lib.load()
    args = (0, 2, 19947, 8, 32, 4, 19947, 4)
    plain = lib.mxd_msda_backward_workspace_bytes(0, 2, 19947, 8, 32, 4, 4, 19947, 4)
    assert lib.mxd_msda_fused_backward_workspace_bytes(*args, 2, 0) == plain
    assert lib.mxd_msda_fused_backward_workspace_bytes(*args, 2, 1) == plain + 8 * 2 * 19947 * 4 * 2 * 4
    assert lib.mxd_msda_fused_backward_workspace_bytes(*args, 4, 1) == plain + 8 * 2 * 19947 * 4 * 4 * 4
    assert lib.mxd_msda_fused_backward_workspace_bytes(*args, 3, 1) == 0


def test_reference_module_paths_below_the_package_root():
    """The reference's operator files do ``import mx_driving._C`` (mx_driving/ops/multi_scale_deformable_attn.py:15,38)
    and its package re-exports from ``.ops.<operator>`` (mx_driving/__init__.py:106-113): both paths resolve, to the
    same objects, and ``_C`` carries the names the reference binds (mx_driving/csrc/pybind.cpp:110-111,121-122,131-132,
    205-208)."""
    import importlib
    c = importlib.import_module("mx_driving._C")
    for name in ("multi_scale_deformable_attn", "multi_scale_deformable_attn_backward", "npu_deformable_aggregation",
                 "npu_deformable_aggregation_backward", "geometric_kernel_attention_forward",
                 "geometric_kernel_attention_backward", "grid_sampler2d_v2", "grid_sampler2d_v2_backward"):
        assert callable(getattr(c, name)), name
    assert c.multi_scale_deformable_attn is _C.multi_scale_deformable_attn
    assert c.npu_deformable_aggregation is _C.deformable_aggregation
    m = importlib.import_module("mx_driving.ops.multi_scale_deformable_attn")
    assert m.MultiScaleDeformableAttnFunction is mx_driving.MultiScaleDeformableAttnFunction
    assert m.multi_scale_deformable_attn is mx_driving.multi_scale_deformable_attn
    assert importlib.import_module("mx_driving.ops.npu_deformable_aggregation").npu_deformable_aggregation \
        is mx_driving.npu_deformable_aggregation
    assert importlib.import_module("mx_driving.ops.geometric_kernel_attention").geometric_kernel_attention \
        is mx_driving.geometric_kernel_attention
    assert importlib.import_module("mx_driving.ops.grid_sampler2d_v2").grid_sampler2d_v2 is mx_driving.grid_sampler2d_v2


C_PROGRAM = r"""
/* A C99 host: the header compiles as C, the library links, and the entry points that need no GPU behave. */
#include <stdio.h>
#include <string.h>
#include "mxd_msda.h"

int main(void)
{
    mxd_msda_plan plan;
    int32_t work[4];
    int rc;
    if (mxd_msda_version() != MXD_MSDA_VERSION) return 1;
    if (strcmp(mxd_msda_last_error(), "") != 0) return 2;
    rc = mxd_msda_make_plan(0, MXD_DTYPE_F32, 2, 19947, 8, 32, 4, 4, 19947, 4, 16, &plan);
    if (rc != MXD_OK || plan.vec != 4 || plan.lanes_per_row != 8 || plan.grid == 0) return 3;
    if (!mxd_msda_decode_block(&plan, 0, 2, 8, 19947, work) || work[0] != 0 || work[2] != 0) return 4;
    if (mxd_msda_make_plan(0, 7, 1, 10, 1, 32, 1, 1, 1, 1, 16, &plan) != MXD_E_DTYPE) return 5;
    if (mxd_msda_make_plan(0, MXD_DTYPE_F16, 1, 10, 1, 257, 1, 1, 1, 1, 16, &plan) != MXD_E_SHAPE) return 6;
    if (strstr(mxd_msda_last_error(), "256") == NULL) return 7;
    if (mxd_msda_make_plan(0, MXD_DTYPE_F32, 1, 10, 1, 32, 1, 1, 1, 1, 16, NULL) != MXD_E_NULL) return 8;
    if (mxd_msda_forward(NULL, NULL, NULL, NULL, NULL, NULL, MXD_DTYPE_F32, 1, 10, 1, 32, 1, 1, 1, 1, NULL) != MXD_E_NULL)
        return 9;
    if (mxd_msda_backward_workspace_bytes(MXD_DTYPE_F32 | MXD_META_I64, 2, 100, 8, 32, 4, 4, 50, 3) == 0) return 10;
    if (mxd_msda_backward_workspace_bytes(MXD_DTYPE_F32, 2, 100, 8, 300, 4, 4, 50, 3) != 0) return 11;
    if (mxd_msda_backward_static_limit() != MXD_MSDA_STATIC_SCRATCH_BYTES) return 12;
    printf("ok %d\n", mxd_msda_version());
    return 0;
}
"""


def test_header_compiles_as_c99_and_the_library_links(tmp_path):
    """include/mxd_msda.h through a C compiler (not C++), linked against the built library, run."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    src = tmp_path / "host.c"
    src.write_text(C_PROGRAM)
    exe = tmp_path / "host"
    libdir = os.path.dirname(_lib.LIB_PATH)
    subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(ROOT, "include"),
                    str(src), "-o", str(exe), "-L", libdir, "-lmxd_msda", f"-Wl,-rpath,{libdir}",
                    "-Wl,-rpath,/opt/rocm/lib"], check=True, capture_output=True, text=True)
    res = subprocess.run([str(exe)], capture_output=True, text=True)
    assert res.returncode == 0, (res.returncode, res.stdout, res.stderr)
    assert res.stdout.startswith("ok 103")


def test_backward_runs_every_fallible_step_before_its_first_launch(monkeypatch):
    """A problem that passes the size checks and the workspace check but whose grad_value pass would need more
    workgroups than a launch can have: the call must fail with MXD_E_SHAPE having enqueued nothing.  Without a GPU a
    launch attempted first would have surfaced as MXD_E_LAUNCH instead.  (No pointer is dereferenced on the host.)"""
    if torch.cuda.is_available():
        pytest.skip("meant for a box without a GPU: the sizes describe terabytes of (never touched) memory")
    from util import set_tuning
    set_tuning(monkeypatch, MXD_MSDA_TILE_TARGET=128)   # (small work items: 259 per (batch, head) here)
    lib = _lib.load()
    dims = (1 << 20, 64, 8, 32, 1, 1, 32, 512)   # bs, nk, nh, hd, nl, nl_attn, nq, np
    need = lib.mxd_msda_backward_workspace_bytes(0, *dims)
    assert need > 0
    fake = 4096   # a non-NULL, 16-byte aligned value standing for device pointers that are never used
    rc = lib.mxd_msda_backward(fake, fake, fake, fake, fake, fake, fake, fake, fake, fake, need, 0, *dims, 0, None)
    assert rc == -2, (rc, _lib.last_error())
    assert "workgroups" in _lib.last_error()


def test_backward_plans_stay_inside_the_default_lds_limit():
    """The first backward kernel does not opt in to more than 64 KiB of LDS: for every row size and up to the largest
    key count a call accepts its plan must fit, the launcher falling back to the one-kernel form (no tile counters in
    LDS) where the tile bookkeeping would not."""
    for dtype in (0, 1, 2):
        for hd in (1, 4, 8, 16, 32, 64, 128, 256):
            es = 4 if dtype == 0 else 2
            for nh in (1, 8):
                limit = ((1 << 31) - 1) // (nh * hd * 4)
                for nk in (1000, 500_000, 1_800_000, 2_090_000, 16_000_000, limit):
                    if nk > limit:
                        continue
                    for nl in (1, 4):
                        plan = _lib.make_plan(1, dtype, 1, nk, nh, hd, nl, nl, 1000, 4)
                        assert plan.lds_bytes <= 64 * 1024, (dtype, hd, nh, nk, nl, plan.lds_bytes, es)


@pytest.mark.parametrize("forced", [None, 1])
def test_forward_cu_form_is_refused_beyond_its_index_arithmetic(monkeypatch, forced):
    """The forward's one-workgroup-per-CU form multiplies pixel indices and pixel strides as 24-bit integers and
    addresses the locations, weights and results of a batch element with 32-bit byte offsets: problems beyond that must
    get the general kernel's plan (block != 1024), also when the environment forces the form on
    (reference: the same class of overflow is flagged in kernels/multi_scale_deformable_attn/op_kernel/msda.h:428)."""
    from util import set_tuning
    if forced is not None:
        set_tuning(monkeypatch, MXD_MSDA_FWD_CU=forced)
    # bs, nk, nh, hd, nl, nl_attn, nq, np -- each just beyond one of the limits, all inside what a call accepts
    beyond = [
        (1, (1 << 23) + 1, 8, 4, 4, 4, 300_000, 4),          # key count: 24-bit pixel index
        (2, 19947, 8, 32, 4, 4, 1 << 21, 4),                  # locations of a batch element: 2^21*8*16*8 B = 2 GiB
        (2, 19947, 8, 32, 4, 4, (1 << 21) + 1, 1),            # results of a batch element: > 2 GiB
    ]
    for dtype in (0, 1, 2):
        es = 4 if dtype == 0 else 2
        for dims in beyond:
            bs, nk, nh, hd, nl, nla, nq, npts = dims
            if nk * nh * hd * 4 >= 1 << 31:
                continue
            plan = _lib.make_plan(0, dtype, *dims)
            over_loc = nq * nh * nla * npts * 2 * es >= 1 << 31
            over_out = nq * nh * hd * es >= 1 << 31
            if nk >= 1 << 23 or over_loc or over_out:
                assert plan.block != 1024, (dtype, dims, plan.as_dict())
    # the form is still what the benchmark shape gets (forced or by default)
    assert _lib.make_plan(0, 0, 2, 19947, 8, 32, 4, 4, 19947, 4).block == 1024
    # distance between neighbouring pixels of 2^23 bytes and more (fp32, forced form): general kernel
    if forced:
        plan = _lib.make_plan(0, 0, 1, 60, 32768, 64, 1, 1, 1 << 16, 16)
        assert plan.block != 1024, plan.as_dict()
