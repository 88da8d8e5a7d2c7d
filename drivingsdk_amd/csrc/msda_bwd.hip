// Backward pass of multi-scale deformable attention for gfx950: the helper kernels on the launch stream (zero-fill of the
// fp32 image, rounding passes, sum over heads) and the dispatch of the first kernel by dtype.  The kernel itself
// (msda_bwd_kernel.h) is instantiated in one translation unit per dtype (msda_bwd_f32.hip, msda_bwd_f16.hip,
// msda_bwd_bf16.hip), so that they compile side by side.
#include "msda_device.h"

namespace mxd {

// ---- helpers on the same stream: zero-fill of the fp32 image, rounding pass ------------------
__global__ __launch_bounds__(256) void msda_fill_zero_kernel(float* p, size_t n, int head)
{
    // [0, head) scalar up to the first 16-byte boundary, then 16-byte stores, then the tail
    f32x4* body = reinterpret_cast<f32x4*>(p + head);
    const size_t n4 = (n - head) / 4;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    const f32x4 z = {0.f, 0.f, 0.f, 0.f};
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += stride) body[i] = z;
    if (blockIdx.x == 0) {
        if ((int)threadIdx.x < head) p[threadIdx.x] = 0.f;
        const size_t t = head + n4 * 4 + threadIdx.x;
        if (threadIdx.x < 4 && t < n) p[t] = 0.f;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void msda_round_kernel(const float* src, T* dst, size_t n)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = from_f32<T>(src[i]);
}

// 16-bit dtypes, sparse image: rounds the rows of the fp32 image that received atomic additions into the caller's
// tensor (the other rows were stored there by the tile pass).  One workgroup per piece of a tile of a batch element.
template <typename T>
__global__ __launch_bounds__(256) void msda_round_rows_kernel(const KArgs a)
{
    // the levels through LDS, one per thread: evaluated straight from memory the two tests below are a chain of scalar
    // loads, one level after the other, in front of a workgroup that moves a few kilobytes
    __shared__ i32x4 lv[kMaxLevels];
    if ((int)threadIdx.x < a.nl) lv[threadIdx.x] = load_level(a, (int)threadIdx.x);
    __syncthreads();
    auto level = [&](int l) { return lv[l]; };
    const int32_t tiles = a.tbl_stride - 1;
    const uint32_t row4 = (uint32_t)(a.nh * a.hd) / 4;
    typedef T t4 __attribute__((ext_vector_type(4)));
    if (!levels_tile_the_keys_of(a, level)) {
        // every row went through the fp32 image: the workgroups round it between them
        const uint64_t n4 = (uint64_t)a.bs * a.nk * row4, per = (n4 + gridDim.x - 1) / gridDim.x;
        const uint64_t lo = (uint64_t)blockIdx.x * per, hi = lo + per < n4 ? lo + per : n4;
        const f32x4* src = reinterpret_cast<const f32x4*>(a.grad_value);
        t4* dst = reinterpret_cast<t4*>(a.grad_value_t);
        for (uint64_t i = lo + threadIdx.x; i < hi; i += blockDim.x) {
            const f32x4 v = __builtin_nontemporal_load(src + i);  // (read once, written once)
            __builtin_nontemporal_store(t4{from_f32<T>(v[0]), from_f32<T>(v[1]), from_f32<T>(v[2]), from_f32<T>(v[3])}, dst + i);
        }
        return;
    }
    const int32_t b = (int32_t)(blockIdx.x / (uint32_t)(tiles * kRowParts)), r = (int32_t)(blockIdx.x % (uint32_t)(tiles * kRowParts));
    int32_t r0, r1;
    if (b >= a.bs || !atomic_rows_of_part_of(a, level, r / kRowParts, r % kRowParts, &r0, &r1)) return;
    const f32x4* src = reinterpret_cast<const f32x4*>(a.grad_value) + ((size_t)b * a.nk + r0) * row4;
    t4* dst = reinterpret_cast<t4*>(a.grad_value_t) + ((size_t)b * a.nk + r0) * row4;
    const uint32_t n4 = (uint32_t)(r1 - r0) * row4;
    for (uint32_t i = threadIdx.x; i < n4; i += blockDim.x) {
        const f32x4 v = __builtin_nontemporal_load(src + i);
        __builtin_nontemporal_store(t4{from_f32<T>(v[0]), from_f32<T>(v[1]), from_f32<T>(v[2]), from_f32<T>(v[3])}, dst + i);
    }
}

hipError_t launch_round_rows(int dtype, const KArgs& a, hipStream_t stream)
{
    const int64_t grid = (int64_t)a.bs * (a.tbl_stride - 1) * kRowParts;
    if (grid <= 0 || grid >= (int64_t(1) << 31)) return hipErrorInvalidConfiguration;
    if (dtype == MXD_DTYPE_F16)
        hipLaunchKernelGGL(msda_round_rows_kernel<f16_t>, dim3((unsigned)grid), dim3(256), 0, stream, a);
    else if (dtype == MXD_DTYPE_BF16)
        hipLaunchKernelGGL(msda_round_rows_kernel<bf16_t>, dim3((unsigned)grid), dim3(256), 0, stream, a);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

// deformable aggregation: grad_location[i] = sum over heads of the per-head partial images
template <typename T>
__global__ __launch_bounds__(256) void dagg_sum_heads_kernel(const float* part, T* dst, size_t n, int nh)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        float s = 0.0f;
        for (int h = 0; h < nh; ++h) s += part[(size_t)h * n + i];
        dst[i] = from_f32<T>(s);
    }
}

hipError_t launch_sum_heads(int dtype, const float* part, void* dst, size_t n, int nh, hipStream_t stream)
{
    if (n == 0) return hipSuccess;
    size_t blocks = (n + 255) / 256;
    if (blocks > 256 * 16) blocks = 256 * 16;
    const dim3 grid((unsigned)blocks), block(256);
    if (dtype == MXD_DTYPE_F32)
        hipLaunchKernelGGL(dagg_sum_heads_kernel<float>, grid, block, 0, stream, part, static_cast<float*>(dst), n, nh);
    else if (dtype == MXD_DTYPE_F16)
        hipLaunchKernelGGL(dagg_sum_heads_kernel<f16_t>, grid, block, 0, stream, part, static_cast<f16_t*>(dst), n, nh);
    else if (dtype == MXD_DTYPE_BF16)
        hipLaunchKernelGGL(dagg_sum_heads_kernel<bf16_t>, grid, block, 0, stream, part, static_cast<bf16_t*>(dst), n, nh);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

hipError_t launch_fill_zero(float* p, size_t n, hipStream_t stream)
{
    if (n == 0) return hipSuccess;
    size_t head = ((16 - (reinterpret_cast<uintptr_t>(p) & 15)) & 15) / 4;
    if (head > n) head = n;
    size_t blocks = ((n - head) / 4 + 255) / 256;
    if (blocks > 256 * 16) blocks = 256 * 16;
    if (blocks == 0) blocks = 1;
    hipLaunchKernelGGL(msda_fill_zero_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, p, n, (int)head);
    return hipGetLastError();
}

hipError_t launch_round(int dtype, const float* src, void* dst, size_t n, hipStream_t stream)
{
    if (n == 0) return hipSuccess;
    size_t blocks = (n + 255) / 256;
    if (blocks > 256 * 16) blocks = 256 * 16;
    if (dtype == MXD_DTYPE_F16)
        hipLaunchKernelGGL(msda_round_kernel<f16_t>, dim3((unsigned)blocks), dim3(256), 0, stream, src,
                           static_cast<f16_t*>(dst), n);
    else if (dtype == MXD_DTYPE_BF16)
        hipLaunchKernelGGL(msda_round_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, stream, src,
                           static_cast<bf16_t*>(dst), n);
    else
        return hipErrorInvalidValue;
    return hipGetLastError();
}

hipError_t launch_backward_f32(const KArgs& a, bool scatter, hipStream_t stream);
hipError_t launch_backward_f16(const KArgs& a, bool scatter, hipStream_t stream);
hipError_t launch_backward_bf16(const KArgs& a, bool scatter, hipStream_t stream);

// scatter = true: one kernel does everything (grad_value through global atomics);
// scatter = false: grad_attn / grad_loc only, grad_value is left to the tile kernel.
hipError_t launch_backward(int dtype, const KArgs& a, bool scatter, hipStream_t stream)
{
    switch (dtype) {
        case MXD_DTYPE_F32: return launch_backward_f32(a, scatter, stream);
        case MXD_DTYPE_F16: return launch_backward_f16(a, scatter, stream);
        case MXD_DTYPE_BF16: return launch_backward_bf16(a, scatter, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace mxd
