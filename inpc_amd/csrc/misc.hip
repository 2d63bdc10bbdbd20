// misc.hip — the element-wise steps on either side of the appearance field, between the sampler's output and
// the rasterizer's input:
//   spherical contraction of the sample positions   (B/misc/src/misc_kernels.cu:49-66)
//   raw density feature -> opacity and its gradient  (feature_to_opacity / TruncExp, utils.py:13-33)
#include <algorithm>

#include "common.hpp"

namespace inpc {
namespace {

constexpr int kBlock = 256;

__global__ void __launch_bounds__(kBlock) k_spherical_contraction(const float* __restrict__ positions,
                                                                  float* __restrict__ contracted, uint32_t n_points) {
    const uint32_t stride = gridDim.x * kBlock;
    for (uint32_t i = blockIdx.x * kBlock + threadIdx.x; i < n_points; i += stride) {
        const float x = positions[3 * (size_t)i], y = positions[3 * (size_t)i + 1], z = positions[3 * (size_t)i + 2];
        const float length_sq = fmaxf((x * x + y * y) + z * z, 1.0f);
        const float scale = (sqrtf(length_sq) * 2.0f - 1.0f) / length_sq * 0.25f;
        contracted[3 * (size_t)i] = __saturatef(scale * x + 0.5f);
        contracted[3 * (size_t)i + 1] = __saturatef(scale * y + 0.5f);
        contracted[3 * (size_t)i + 2] = __saturatef(scale * z + 0.5f);
    }
}

// opacity = -expm1(-exp(x))
__global__ void __launch_bounds__(kBlock) k_opacity_forward(const float* __restrict__ raw, float* __restrict__ opacity,
                                                            size_t n) {
    const size_t stride = (size_t)gridDim.x * kBlock;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) opacity[i] = -expm1f(-expf(raw[i]));
}

// d opacity / d x = exp(-exp(x)) * exp(clamp(x, -15, 15)): the inner exponential's gradient is the truncated one
__global__ void __launch_bounds__(kBlock) k_opacity_backward(const float* __restrict__ grad, const float* __restrict__ raw,
                                                             float* __restrict__ grad_raw, size_t n) {
    const size_t stride = (size_t)gridDim.x * kBlock;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
        const float x = raw[i];
        grad_raw[i] = (grad[i] * expf(-expf(x))) * expf(fminf(fmaxf(x, -15.0f), 15.0f));
    }
}

uint32_t grid_for(size_t n) { return (uint32_t)std::min<size_t>((n + kBlock - 1) / kBlock, 8192); }

}  // namespace
}  // namespace inpc

extern "C" {

int inpc_spherical_contraction(const float* positions, float* contracted, uint32_t n_points, void* stream) {
    using namespace inpc;
    if (n_points == 0) return INPC_OK;
    if (!positions || !contracted) return fail(INPC_E_INVALID_ARGUMENT, "spherical_contraction: null pointer");
    INPC_LAUNCH("spherical_contraction", k_spherical_contraction, dim3(grid_for(n_points)), dim3(kBlock),
                (hipStream_t)stream, positions, contracted, n_points);
    return INPC_OK;
}

int inpc_opacity_forward(const float* raw, float* opacity, size_t n, void* stream) {
    using namespace inpc;
    if (n == 0) return INPC_OK;
    if (!raw || !opacity) return fail(INPC_E_INVALID_ARGUMENT, "opacity_forward: null pointer");
    INPC_LAUNCH("opacity_forward", k_opacity_forward, dim3(grid_for(n)), dim3(kBlock), (hipStream_t)stream, raw, opacity, n);
    return INPC_OK;
}

int inpc_opacity_backward(const float* grad_opacity, const float* raw, float* grad_raw, size_t n, void* stream) {
    using namespace inpc;
    if (n == 0) return INPC_OK;
    if (!grad_opacity || !raw || !grad_raw) return fail(INPC_E_INVALID_ARGUMENT, "opacity_backward: null pointer");
    INPC_LAUNCH("opacity_backward", k_opacity_backward, dim3(grid_for(n)), dim3(kBlock), (hipStream_t)stream, grad_opacity,
                raw, grad_raw, n);
    return INPC_OK;
}

}  // extern "C"
