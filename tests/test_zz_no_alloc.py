"""mxd_msda_backward_static: the backward pass for callers that cannot allocate (its scratch is a static device array
of the library).  Through the C ABI, against mxd_msda_backward on the same inputs, two calls in a row -- the second with
a smaller input, so that the first call's leftovers in the shared scratch are in its way."""
import pytest
import torch

from drivingsdk_amd import _lib, workloads
from util import rel_err, to_device

pytestmark = pytest.mark.gpu


def _call(d, static, dtype_code=0):
    """One raw backward call on device inputs d; returns (grad_value, grad_loc, grad_attn)."""
    lib = _lib.load()
    shapes, lsi = d.spatial_shapes.int().contiguous(), d.level_start_index.int().contiguous()
    bs, nk, nh, hd = d.value.shape
    _, nq, _, nl, npts, _ = d.sampling_locations.shape
    dims = (bs, nk, nh, hd, nl, nl, nq, npts)
    gv, gl, ga = torch.empty_like(d.value), torch.empty_like(d.sampling_locations), torch.empty_like(d.attention_weights)
    stream = torch.cuda.current_stream().cuda_stream
    ins = (d.value.data_ptr(), shapes.data_ptr(), lsi.data_ptr(), d.sampling_locations.data_ptr(),
           d.attention_weights.data_ptr(), d.grad_output.data_ptr(), gv.data_ptr(), gl.data_ptr(), ga.data_ptr())
    if static:
        rc = lib.mxd_msda_backward_static(*ins, dtype_code, *dims, 0, stream)
    else:
        nbytes = lib.mxd_msda_backward_workspace_bytes(dtype_code, *dims)
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=d.value.device)
        rc = lib.mxd_msda_backward(*ins, ws.data_ptr(), nbytes, dtype_code, *dims, 0, stream)
    assert rc == 0, _lib.last_error()
    torch.cuda.synchronize()
    return gv, gl, ga


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_static_backward_matches_the_workspace_backward_twice_in_a_row(gpu_device, dtype):
    code = {torch.float32: 0, torch.float16: 1}[dtype]
    # float32: the encoder shape with a tenth of its queries (about 16 MiB of scratch), then the tiny workload (5 MiB);
    # float16 (the scratch also holds the fp32 image of grad_value): a shape of the reference's test with fewer
    # queries (22 MiB), then the tiny workload
    first = workloads.make_inputs("detr_encoder_bwd", with_grad_output=True, scale_queries=0.1) if dtype == torch.float32 \
        else workloads.reference_test_inputs([2, 3000, 32, 8, 2, 4], dtype=dtype, seed=17)
    second = workloads.make_inputs("tiny", dtype=dtype, with_grad_output=True)
    for name, inp in (("first", first), ("second, smaller", second)):
        d = to_device(inp, gpu_device)
        want = _call(d, static=False, dtype_code=code)
        got = _call(d, static=True, dtype_code=code)
        assert torch.equal(got[1], want[1]) and torch.equal(got[2], want[2]), name
        # (grad_value: the order of its sums varies from run to run, also between two calls of one entry point)
        tol = 1e-6 if dtype == torch.float32 else 2e-3
        assert rel_err(got[0].double().cpu().numpy(), want[0].double().cpu().numpy()) <= tol, name


def test_static_backward_refuses_what_does_not_fit(gpu_device):
    lib = _lib.load()
    assert lib.mxd_msda_backward_static_limit() == 32 << 20
    d = to_device(workloads.make_inputs("tiny", with_grad_output=True), gpu_device)
    shapes, lsi = d.spatial_shapes.int().contiguous(), d.level_start_index.int().contiguous()
    p = d.value.data_ptr()
    # the full encoder shape needs about 163 MB: refused before anything is launched (the pointers are never used)
    dims = (2, 19947, 8, 32, 4, 4, 19947, 4)
    assert lib.mxd_msda_backward_workspace_bytes(0, *dims) > (32 << 20)
    rc = lib.mxd_msda_backward_static(p, shapes.data_ptr(), lsi.data_ptr(), p, p, p, p, p, p, 0, *dims, 0,
                                      torch.cuda.current_stream().cuda_stream)
    assert rc == -4 and "static" in _lib.last_error()
