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

// Weight decay of the multi-resolution hash grid, normalised per level: grad = 0.1 * 2 / (entries of the level)
// * weight; the level of a weight follows from its position in the flat parameter vector, and the weights in
// front of 6144 (the dense coarsest levels) are not decayed (B/misc/src/misc_kernels.cu:6-47).
template <bool ADD>
__global__ void __launch_bounds__(kBlock) k_weight_decay_grads(const float* __restrict__ weights, float* __restrict__ grads,
                                                               uint32_t n_weights) {
    constexpr float f0 = 0.1f * 2.0f / float(210917376 - 177362944);
    constexpr float f1 = 0.1f * 2.0f / float(177362944 - 143808512);
    constexpr float f2 = 0.1f * 2.0f / float(143808512 - 110254080);
    constexpr float f3 = 0.1f * 2.0f / float(110254080 - 76699648);
    constexpr float f4 = 0.1f * 2.0f / float(76699648 - 43145216);
    constexpr float f5 = 0.1f * 2.0f / float(43145216 - 9590784);
    constexpr float f6 = 0.1f * 2.0f / float(9590784 - 1202176);
    constexpr float f7 = 0.1f * 2.0f / float(1202176 - 153600);
    constexpr float f8 = 0.1f * 2.0f / float(153600 - 22528);
    constexpr float f9 = 0.1f * 2.0f / float(22528 - 6144);
    const uint32_t stride = gridDim.x * kBlock;
    for (uint32_t i = blockIdx.x * kBlock + threadIdx.x; i < n_weights; i += stride) {
        float factor = 0.0f;
        if (i >= 177362944u) factor = f0;
        else if (i >= 143808512u) factor = f1;
        else if (i >= 110254080u) factor = f2;
        else if (i >= 76699648u) factor = f3;
        else if (i >= 43145216u) factor = f4;
        else if (i >= 9590784u) factor = f5;
        else if (i >= 1202176u) factor = f6;
        else if (i >= 153600u) factor = f7;
        else if (i >= 22528u) factor = f8;
        else if (i >= 6144u) factor = f9;
        const float g = factor * weights[i];
        grads[i] = ADD ? grads[i] + g : g;
    }
}

// Cauchy loss, element-wise part: log1p(12.5 d^2) / n (B/misc/src/misc_kernels.cu:68-79)
__global__ void __launch_bounds__(kBlock) k_cauchy_loss(const float* __restrict__ input, const float* __restrict__ target,
                                                        float* __restrict__ loss, uint32_t n) {
    const uint32_t stride = gridDim.x * kBlock;
    for (uint32_t i = blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
        const float diff = input[i] - target[i];
        loss[i] = log1pf(diff * diff * 12.5f) / (float)n;
    }
}

// and its gradient (B/misc/src/misc_kernels.cu:81-94)
__global__ void __launch_bounds__(kBlock) k_cauchy_loss_backward(const float* __restrict__ grad, const float* __restrict__ input,
                                                                 const float* __restrict__ target, float* __restrict__ grad_input,
                                                                 uint32_t n) {
    const uint32_t stride = gridDim.x * kBlock;
    const float g = grad[0];
    for (uint32_t i = blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
        const float diff = input[i] - target[i];
        const float denominator = (float)n * (12.5f * diff * diff + 1.0f);
        grad_input[i] = 25.0f * diff / fmaxf(denominator, 1.0e-12f) * g;
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

int inpc_weight_decay_grads(const float* weights, float* grads, uint32_t n_weights, int add, void* stream) {
    using namespace inpc;
    if (n_weights == 0) return INPC_OK;
    if (!weights || !grads) return fail(INPC_E_INVALID_ARGUMENT, "weight_decay_grads: null pointer");
    if (add) {
        INPC_LAUNCH("weight_decay_grads_add", k_weight_decay_grads<true>, dim3(grid_for(n_weights)), dim3(kBlock),
                    (hipStream_t)stream, weights, grads, n_weights);
    } else {
        INPC_LAUNCH("weight_decay_grads", k_weight_decay_grads<false>, dim3(grid_for(n_weights)), dim3(kBlock),
                    (hipStream_t)stream, weights, grads, n_weights);
    }
    return INPC_OK;
}

int inpc_cauchy_loss(const float* input, const float* target, float* elementwise_loss, uint32_t n, void* stream) {
    using namespace inpc;
    if (n == 0) return INPC_OK;
    if (!input || !target || !elementwise_loss) return fail(INPC_E_INVALID_ARGUMENT, "cauchy_loss: null pointer");
    INPC_LAUNCH("cauchy_loss", k_cauchy_loss, dim3(grid_for(n)), dim3(kBlock), (hipStream_t)stream, input, target,
                elementwise_loss, n);
    return INPC_OK;
}

int inpc_cauchy_loss_backward(const float* grad, const float* input, const float* target, float* grad_input, uint32_t n,
                              void* stream) {
    using namespace inpc;
    if (n == 0) return INPC_OK;
    if (!grad || !input || !target || !grad_input) return fail(INPC_E_INVALID_ARGUMENT, "cauchy_loss_backward: null pointer");
    INPC_LAUNCH("cauchy_loss_backward", k_cauchy_loss_backward, dim3(grid_for(n)), dim3(kBlock), (hipStream_t)stream, grad,
                input, target, grad_input, n);
    return INPC_OK;
}

}  // extern "C"
