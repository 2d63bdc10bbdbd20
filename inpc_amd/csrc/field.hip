// field.hip — per-iteration update of the octree probability field from the samples a frame used
// (the reference's ProbabilityField.update, Modules/ProbabilityField.py:146-157):
//   leaf_weights *= decay; scores *= decay
//   max_sampled / min_sampled = per leaf maximum / minimum of the blending weights of its samples (0 for a leaf
//                               without samples: scatter_reduce amax / amin with include_self = False)
//   leaf_weights = max(leaf_weights, max_sampled)
//   scores       = max(scores, clamp(max_sampled - min_sampled, 0, 1))
// Maximum and minimum do not depend on the order of the samples, so the result is bit-identical to a
// sequential evaluation. Floats are compared through an order-preserving map to unsigned integers, which
// makes one integer atomic per sample and extremum enough for any sign.
#include <algorithm>

#include "common.hpp"

namespace inpc {
namespace {

constexpr int kBlock = 256;

__device__ __forceinline__ uint32_t ordered_key(float f) {
    const uint32_t b = __float_as_uint(f);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

__device__ __forceinline__ float ordered_value(uint32_t k) {
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7FFFFFFFu) : ~k);
}

constexpr uint32_t kNoMax = 0u;           // below the key of every float
constexpr uint32_t kNoMin = 0xFFFFFFFFu;  // above the key of every float

__global__ void __launch_bounds__(kBlock) k_field_reset(uint32_t* __restrict__ max_key, uint32_t* __restrict__ min_key,
                                                        uint32_t n_leaves) {
    const uint32_t stride = gridDim.x * kBlock;
    for (uint32_t i = blockIdx.x * kBlock + threadIdx.x; i < n_leaves; i += stride) {
        max_key[i] = kNoMax;
        min_key[i] = kNoMin;
    }
}

__global__ void __launch_bounds__(kBlock) k_field_scatter(const int64_t* __restrict__ indices,
                                                          const float* __restrict__ weights, uint32_t n_samples,
                                                          uint32_t* max_key, uint32_t* min_key, uint32_t n_leaves,
                                                          uint32_t* error_flag) {
    const uint32_t stride = gridDim.x * kBlock;
    for (uint32_t i = blockIdx.x * kBlock + threadIdx.x; i < n_samples; i += stride) {
        const int64_t leaf = indices[i];
        if (leaf < 0 || leaf >= (int64_t)n_leaves) {  // the reference's scatter_reduce_ raises for these
            atomicOr(error_flag, 1u);
            continue;
        }
        const uint32_t key = ordered_key(weights[i]);
        // most samples of a leaf do not change its extrema: look before paying for the atomic
        if (key > __hip_atomic_load(&max_key[leaf], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) atomicMax(&max_key[leaf], key);
        if (key < __hip_atomic_load(&min_key[leaf], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) atomicMin(&min_key[leaf], key);
    }
}

__global__ void __launch_bounds__(kBlock) k_field_finish(const uint32_t* __restrict__ max_key,
                                                         const uint32_t* __restrict__ min_key, float* __restrict__ leaf_weights,
                                                         float* __restrict__ leaf_scores, uint32_t n_leaves, float decay) {
    const uint32_t stride = gridDim.x * kBlock;
    for (uint32_t i = blockIdx.x * kBlock + threadIdx.x; i < n_leaves; i += stride) {
        const uint32_t kmax = max_key[i], kmin = min_key[i];
        const float max_sampled = kmax == kNoMax ? 0.0f : ordered_value(kmax);
        const float min_sampled = kmin == kNoMin ? 0.0f : ordered_value(kmin);
        leaf_weights[i] = fmaxf(leaf_weights[i] * decay, max_sampled);
        leaf_scores[i] = fmaxf(leaf_scores[i] * decay, fminf(fmaxf(max_sampled - min_sampled, 0.0f), 1.0f));
    }
}

}  // namespace
}  // namespace inpc

extern "C" {

size_t inpc_field_update_workspace_bytes(uint32_t n_leaves) { return (size_t)n_leaves * 8 + 256; }

int inpc_field_update(const int64_t* indices, const float* weights, uint32_t n_samples, float* leaf_weights,
                      float* leaf_scores, uint32_t n_leaves, float decay, void* workspace, size_t workspace_bytes,
                      void* stream_) {
    using namespace inpc;
    hipStream_t stream = (hipStream_t)stream_;
    if (n_leaves == 0) return INPC_OK;
    if (!leaf_weights || !leaf_scores) return fail(INPC_E_INVALID_ARGUMENT, "field_update: null leaf arrays");
    if (n_samples > 0 && (!indices || !weights)) return fail(INPC_E_INVALID_ARGUMENT, "field_update: null samples");
    if (!workspace || workspace_bytes < inpc_field_update_workspace_bytes(n_leaves))
        return fail(INPC_E_WORKSPACE, "field_update: workspace too small");
    if (((uintptr_t)workspace & 3u) != 0) return fail(INPC_E_WORKSPACE, "field_update: workspace must be 4-byte aligned");
    uint32_t* error_flag = (uint32_t*)workspace;
    uint32_t* max_key = (uint32_t*)workspace + 64;
    uint32_t* min_key = max_key + n_leaves;
    int rc = fill_u32(error_flag, 0u, 1, stream);
    if (rc != INPC_OK) return rc;
    const uint32_t leaf_blocks = std::min<uint32_t>(div_up(n_leaves, kBlock), 4096u);
    INPC_LAUNCH("field_reset", k_field_reset, dim3(leaf_blocks), dim3(kBlock), stream, max_key, min_key, n_leaves);
    if (n_samples > 0) {
        INPC_LAUNCH("field_scatter", k_field_scatter, dim3(std::min<uint32_t>(div_up(n_samples, kBlock), 8192u)),
                    dim3(kBlock), stream, indices, weights, n_samples, max_key, min_key, n_leaves, error_flag);
    }
    INPC_LAUNCH("field_finish", k_field_finish, dim3(leaf_blocks), dim3(kBlock), stream, (const uint32_t*)max_key,
                (const uint32_t*)min_key, leaf_weights, leaf_scores, n_leaves, decay);
    return INPC_OK;
}

int inpc_field_update_check(const void* workspace, void* stream_) {
    using namespace inpc;
    hipStream_t stream = (hipStream_t)stream_;
    uint32_t flag = 0;
    INPC_HIP_CHECK(hipMemcpyAsync(&flag, workspace, 4, hipMemcpyDeviceToHost, stream));
    INPC_HIP_CHECK(hipStreamSynchronize(stream));
    if (flag) return fail(INPC_E_INVALID_ARGUMENT, "field_update: a sample index lies outside [0, n_leaves)");
    return INPC_OK;
}

}  // extern "C"
