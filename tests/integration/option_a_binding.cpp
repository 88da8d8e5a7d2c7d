// The reference's compiled binding for this path (mx_driving/csrc/MultiScaleDeformableAttn.cpp:28-118: checks,
// allocation of the outputs, one launch per function) rewritten over the C ABI of libmxd_msda.so, as a maintainer of a
// PyTorch-ROCm build of mx_driving._C would write it: the two EXEC_NPU_CMD(aclnnMultiScaleDeformableAttn[Grad], ...)
// calls become mxd_msda_forward / mxd_msda_backward on the current HIP stream, and the float16 up-cast blocks go (the
// library reads 16-bit tensors as they are).  pybind registration as in mx_driving/csrc/pybind.cpp:110-111.
// tests/test_host.py compiles this file against the installed torch headers; nothing in the package uses it.
// (PyTorch-ROCm presents its devices as "cuda": the guard and stream types that go with that are these)
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/extension.h>

#include <tuple>

#include "mxd_msda.h"

namespace {

int dtype_code(at::ScalarType t)
{
    TORCH_CHECK(t == at::kFloat || t == at::kHalf || t == at::kBFloat16, "value: float32, float16 or bfloat16 expected");
    return t == at::kFloat ? MXD_DTYPE_F32 : t == at::kHalf ? MXD_DTYPE_F16 : MXD_DTYPE_BF16;
}

// spatial_shapes / level_start_index as the library takes them: int32, or int64 with MXD_META_I64
int meta_flag(const at::Tensor& shapes, const at::Tensor& lsi)
{
    TORCH_CHECK(shapes.scalar_type() == lsi.scalar_type() && (shapes.scalar_type() == at::kInt || shapes.scalar_type() == at::kLong),
                "spatial_shapes and level_start_index: both int32 or both int64");
    return shapes.scalar_type() == at::kLong ? MXD_META_I64 : 0;
}

}  // namespace

at::Tensor multi_scale_deformable_attn(const at::Tensor& value, const at::Tensor& value_spatial_shapes,
                                       const at::Tensor& value_level_start_index, const at::Tensor& sampling_locations,
                                       const at::Tensor& attention_weights)
{
    TORCH_CHECK(value.dim() == 4 && sampling_locations.dim() == 6 && attention_weights.dim() == 5, "unexpected ranks");
    TORCH_CHECK(value.size(3) <= 256, "The number of embedding dimensions should be less than or equal to 256");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(value.device());
    const at::Tensor v = value.contiguous(), s = value_spatial_shapes.contiguous(), l = value_level_start_index.contiguous();
    const at::Tensor loc = sampling_locations.to(v.scalar_type()).contiguous();
    const at::Tensor attn = attention_weights.to(v.scalar_type()).contiguous();
    at::Tensor out = at::empty({loc.size(0), loc.size(1), v.size(2) * v.size(3)}, v.options());
    const int rc = mxd_msda_forward(v.data_ptr(), static_cast<const int32_t*>(s.data_ptr()), static_cast<const int32_t*>(l.data_ptr()),
                                    loc.data_ptr(), attn.data_ptr(), out.data_ptr(), dtype_code(v.scalar_type()) | meta_flag(s, l),
                                    v.size(0), v.size(1), v.size(2), v.size(3), s.size(0), attn.size(3), loc.size(1), loc.size(4),
                                    c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream());
    TORCH_CHECK(rc == MXD_OK, mxd_msda_last_error());
    return out;
}

std::tuple<at::Tensor, at::Tensor, at::Tensor> multi_scale_deformable_attn_backward(
    const at::Tensor& value, const at::Tensor& value_spatial_shapes, const at::Tensor& value_level_start_index,
    const at::Tensor& sampling_locations, const at::Tensor& attention_weights, const at::Tensor& grad_output)
{
    TORCH_CHECK(value.dim() == 4 && sampling_locations.dim() == 6 && attention_weights.dim() == 5, "unexpected ranks");
    c10::hip::HIPGuardMasqueradingAsCUDA guard(value.device());
    const at::Tensor v = value.contiguous(), s = value_spatial_shapes.contiguous(), l = value_level_start_index.contiguous();
    const at::Tensor loc = sampling_locations.to(v.scalar_type()).contiguous();
    const at::Tensor attn = attention_weights.to(v.scalar_type()).contiguous();
    const at::Tensor go = grad_output.to(v.scalar_type()).contiguous();
    // (the library zero-fills what it accumulates into and writes every element of the other two)
    at::Tensor grad_value = at::empty_like(v), grad_loc = at::empty_like(loc), grad_attn = at::empty_like(attn);
    const int code = dtype_code(v.scalar_type()) | meta_flag(s, l);
    const int64_t bs = v.size(0), nk = v.size(1), nh = v.size(2), hd = v.size(3), nl = s.size(0), nl_attn = attn.size(3),
                  nq = loc.size(1), np = loc.size(4);
    const size_t bytes = mxd_msda_backward_workspace_bytes(code, bs, nk, nh, hd, nl, nl_attn, nq, np);
    at::Tensor workspace = at::empty({static_cast<int64_t>(bytes > 16 ? bytes : 16)}, v.options().dtype(at::kByte));
    const int rc = mxd_msda_backward(v.data_ptr(), static_cast<const int32_t*>(s.data_ptr()), static_cast<const int32_t*>(l.data_ptr()),
                                     loc.data_ptr(), attn.data_ptr(), go.data_ptr(), grad_value.data_ptr(), grad_loc.data_ptr(),
                                     grad_attn.data_ptr(), workspace.data_ptr(), bytes, code, bs, nk, nh, hd, nl, nl_attn, nq, np,
                                     /*flags=*/0, c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream());
    TORCH_CHECK(rc == MXD_OK, mxd_msda_last_error());
    return std::make_tuple(grad_value, grad_loc, grad_attn);
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    m.def("multi_scale_deformable_attn", &multi_scale_deformable_attn);
    m.def("multi_scale_deformable_attn_backward", &multi_scale_deformable_attn_backward);
}
