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

// keys[leaf] = {key of the maximum, key of the minimum}: one 8-byte word, so that the look before the atomics is
// one gather (a divergent load costs the same whatever its width).
__global__ void __launch_bounds__(kBlock) k_field_reset(uint2* __restrict__ keys, uint32_t n_leaves) {
    const uint32_t stride = gridDim.x * kBlock;
    for (uint32_t i = blockIdx.x * kBlock + threadIdx.x; i < n_leaves; i += stride) keys[i] = make_uint2(kNoMax, kNoMin);
}

__global__ void __launch_bounds__(kBlock) k_field_scatter(const int64_t* __restrict__ indices,
                                                          const float* __restrict__ weights, uint32_t n_samples,
                                                          uint2* keys, uint32_t n_leaves, uint32_t* error_flag) {
    const uint32_t stride = gridDim.x * kBlock;
    for (uint32_t i = blockIdx.x * kBlock + threadIdx.x; i < n_samples; i += stride) {
        const int64_t leaf = indices[i];
        if (leaf < 0 || leaf >= (int64_t)n_leaves) {  // the reference's scatter_reduce_ raises for these
            atomicOr(error_flag, 1u);
            continue;
        }
        const uint32_t key = ordered_key(weights[i]);
        // most samples of a leaf do not change its extrema: look before paying for the atomics. The look may see
        // an older value of either half; the atomics decide.
        unsigned long long* word = (unsigned long long*)(keys + leaf);
        const unsigned long long seen = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (key > (uint32_t)seen) atomicMax(&keys[leaf].x, key);
        if (key < (uint32_t)(seen >> 32)) atomicMin(&keys[leaf].y, key);
    }
}

__global__ void __launch_bounds__(kBlock) k_field_finish(const uint2* __restrict__ keys, float* __restrict__ leaf_weights,
                                                         float* __restrict__ leaf_scores, uint32_t n_leaves, float decay) {
    const uint32_t stride = gridDim.x * kBlock;
    for (uint32_t i = blockIdx.x * kBlock + threadIdx.x; i < n_leaves; i += stride) {
        const uint2 k = keys[i];
        const float max_sampled = k.x == kNoMax ? 0.0f : ordered_value(k.x);
        const float min_sampled = k.y == kNoMin ? 0.0f : ordered_value(k.y);
        leaf_weights[i] = fmaxf(leaf_weights[i] * decay, max_sampled);
        leaf_scores[i] = fmaxf(leaf_scores[i] * decay, fminf(fmaxf(max_sampled - min_sampled, 0.0f), 1.0f));
    }
}


// ---- prune / subdivide (Modules/ProbabilityField.py:159-165, 217-257) -----------------------------------------------
// Both are ordered selections over the leaves: prune keeps the leaves whose weight exceeds a threshold, in
// order; subdivide keeps the leaves that are not split, in order, and appends eight children per split leaf,
// parents in order, children in the order x, y, z of the sign of their offset. A leaf is selected when
// value > threshold and (levels == nullptr or level < max_level).
//   k_select_count   per block of kSelectTile leaves: number of selected leaves
//   k_select_scan    one block: exclusive scan of the block counts, total to counts[0]
//   k_prune_apply / k_subdivide_apply   recompute the flags, rank inside the block by ballots, write
constexpr int kSelectItems = 4;
constexpr int kSelectTile = kBlock * kSelectItems;

__device__ __forceinline__ bool leaf_selected(const float* __restrict__ values, const int32_t* __restrict__ levels,
                                              uint32_t i, float threshold, int max_level) {
    return values[i] > threshold && (levels == nullptr || levels[i] < max_level);
}

// Exclusive rank of this thread's flag among the flags of the block in thread order; `total` = their number.
__device__ __forceinline__ uint32_t block_rank(bool flag, uint32_t* s_wave /* kBlock / kWave */, uint32_t& total) {
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint64_t ballot = __ballot(flag);
    if (lane == 0) s_wave[wave] = (uint32_t)__popcll(ballot);
    __syncthreads();
    uint32_t before = 0;
    total = 0;
#pragma unroll
    for (int w = 0; w < kBlock / kWave; ++w) {
        const uint32_t c = s_wave[w];
        if ((uint32_t)w < wave) before += c;
        total += c;
    }
    __syncthreads();
    return before + mask_rank(ballot);
}

__global__ void __launch_bounds__(kBlock) k_select_count(const float* __restrict__ values, const int32_t* __restrict__ levels,
                                                         uint32_t n, float threshold, int max_level,
                                                         uint32_t* __restrict__ block_counts) {
    __shared__ uint32_t s_count;
    if (threadIdx.x == 0) s_count = 0u;
    __syncthreads();
    uint32_t mine = 0;
#pragma unroll
    for (int j = 0; j < kSelectItems; ++j) {
        const uint32_t i = blockIdx.x * kSelectTile + j * kBlock + threadIdx.x;
        if (i < n && leaf_selected(values, levels, i, threshold, max_level)) ++mine;
    }
    for (int sh = 32; sh > 0; sh >>= 1) mine += __shfl_down(mine, sh, 64);
    if ((threadIdx.x & 63u) == 0u && mine) atomicAdd(&s_count, mine);
    __syncthreads();
    if (threadIdx.x == 0) block_counts[blockIdx.x] = s_count;
}

__global__ void __launch_bounds__(kBlock) k_select_scan(uint32_t* block_counts, uint32_t n_blocks, uint32_t* counts) {
    __shared__ uint32_t s_wave[kBlock / kWave];
    __shared__ uint32_t s_carry;
    if (threadIdx.x == 0) s_carry = 0u;
    __syncthreads();
    for (uint32_t base = 0; base < n_blocks; base += kBlock) {
        const uint32_t i = base + threadIdx.x, lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
        const uint32_t v = i < n_blocks ? block_counts[i] : 0u;
        uint32_t incl = v;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t up = __shfl_up(incl, d, 64);
            if (lane >= (uint32_t)d) incl += up;
        }
        if (lane == 63) s_wave[wave] = incl;
        __syncthreads();
        uint32_t before = s_carry, all = 0;
#pragma unroll
        for (int w = 0; w < kBlock / kWave; ++w) {
            const uint32_t c = s_wave[w];
            if ((uint32_t)w < wave) before += c;
            all += c;
        }
        if (i < n_blocks) block_counts[i] = before + incl - v;
        __syncthreads();
        if (threadIdx.x == 0) s_carry += all;
        __syncthreads();
    }
    if (threadIdx.x == 0) counts[0] = s_carry;
}

struct LeafArrays {
    const float* centers;
    const int32_t* levels;
    const float* weights;
    const float* scores;
};

struct LeafOutputs {
    float* centers;
    int32_t* levels;
    float* weights;
    float* scores;
};

__global__ void __launch_bounds__(kBlock) k_prune_apply(LeafArrays in, LeafOutputs out, uint32_t n, float threshold,
                                                        const uint32_t* __restrict__ block_offsets) {
    __shared__ uint32_t s_wave[kBlock / kWave];
    uint32_t base = block_offsets[blockIdx.x];
#pragma unroll
    for (int j = 0; j < kSelectItems; ++j) {
        const uint32_t i = blockIdx.x * kSelectTile + j * kBlock + threadIdx.x;
        const bool keep = i < n && leaf_selected(in.weights, nullptr, i, threshold, 0);
        uint32_t total;
        const uint32_t slot = base + block_rank(keep, s_wave, total);
        base += total;
        if (keep) {
            out.centers[3 * (size_t)slot] = in.centers[3 * (size_t)i];
            out.centers[3 * (size_t)slot + 1] = in.centers[3 * (size_t)i + 1];
            out.centers[3 * (size_t)slot + 2] = in.centers[3 * (size_t)i + 2];
            out.levels[slot] = in.levels[i];
            out.weights[slot] = in.weights[i];
            out.scores[slot] = in.scores[i];
        }
    }
}

// Split leaf number r (in order) becomes the children n_kept + 8 r .. + 7; child j sits at
// centre -/+ initial_size / 2^(level + 2) per axis, + in x for odd j, in y for j % 4 >= 2, in z for j >= 4
// (ProbabilityField.py:233-250); its level is level + 1, its weight the parent's, its score 0.
__global__ void __launch_bounds__(kBlock) k_subdivide_apply(LeafArrays in, LeafOutputs out, uint32_t n, float threshold,
                                                            int max_level, float size_x, float size_y, float size_z,
                                                            const uint32_t* __restrict__ block_offsets,
                                                            const uint32_t* __restrict__ counts) {
    __shared__ uint32_t s_wave[kBlock / kWave];
    const uint32_t n_split = counts[0], n_kept = n - n_split;
    uint32_t split_base = block_offsets[blockIdx.x];
#pragma unroll
    for (int j = 0; j < kSelectItems; ++j) {
        const uint32_t i = blockIdx.x * kSelectTile + j * kBlock + threadIdx.x;
        const bool live = i < n;
        const bool split = live && leaf_selected(in.scores, in.levels, i, threshold, max_level);
        uint32_t total;
        const uint32_t rank = block_rank(split, s_wave, total);
        if (live) {
            const float cx = in.centers[3 * (size_t)i], cy = in.centers[3 * (size_t)i + 1], cz = in.centers[3 * (size_t)i + 2];
            const int32_t level = in.levels[i];
            const float weight = in.weights[i];
            if (!split) {
                const uint32_t slot = i - (split_base + rank);   // kept leaves in front of this one
                out.centers[3 * (size_t)slot] = cx;
                out.centers[3 * (size_t)slot + 1] = cy;
                out.centers[3 * (size_t)slot + 2] = cz;
                out.levels[slot] = level;
                out.weights[slot] = weight;
                out.scores[slot] = in.scores[i];
            } else {
                const size_t first = (size_t)n_kept + 8u * (size_t)(split_base + rank);
                const float ox = ldexpf(size_x, -(level + 2)), oy = ldexpf(size_y, -(level + 2)), oz = ldexpf(size_z, -(level + 2));
#pragma unroll
                for (int c = 0; c < 8; ++c) {
                    out.centers[3 * (first + c)] = (c & 1) ? cx + ox : cx - ox;
                    out.centers[3 * (first + c) + 1] = (c & 2) ? cy + oy : cy - oy;
                    out.centers[3 * (first + c) + 2] = (c & 4) ? cz + oz : cz - oz;
                    out.levels[first + c] = level + 1;
                    out.weights[first + c] = weight;
                    out.scores[first + c] = 0.0f;
                }
            }
        }
        split_base += total;
    }
}


// ---- quasi-random positions from per-leaf sample counts (Modules/ProbabilityField.py:131-140, utils.py:36-64) -------
// Sample s belongs to the leaf whose run [first[leaf], first[leaf + 1]) of the exclusive sum of the counts
// holds s (arange.repeat_interleave(counts)); with h = s - first[leaf] its position is
//   centre - size / 2 + halton(h + 1) * size,  size = initial_size / 2^level,
// or the centre itself when the leaf has a single sample. halton(i) = radical inverse of i in the bases 2, 3, 5,
// accumulated in double precision exactly as the reference's Python loop does and rounded to float once.
__global__ void __launch_bounds__(kBlock) k_count_block_sums(const int64_t* __restrict__ counts, uint32_t n,
                                                             uint32_t* __restrict__ block_sums, uint32_t* error_flag) {
    __shared__ uint32_t s_sum;
    if (threadIdx.x == 0) s_sum = 0u;
    __syncthreads();
    uint32_t mine = 0;
#pragma unroll
    for (int j = 0; j < kSelectItems; ++j) {
        const uint32_t i = blockIdx.x * kSelectTile + j * kBlock + threadIdx.x;
        if (i < n) {
            const int64_t c = counts[i];
            if (c < 0 || c > 0x7FFFFFFF) atomicOr(error_flag, 1u);
            else mine += (uint32_t)c;
        }
    }
    for (int sh = 32; sh > 0; sh >>= 1) mine += __shfl_down(mine, sh, 64);
    if ((threadIdx.x & 63u) == 0u && mine) atomicAdd(&s_sum, mine);
    __syncthreads();
    if (threadIdx.x == 0) block_sums[blockIdx.x] = s_sum;
}

// first[i] = sum of counts[0 .. i), i = 0 .. n (block_first: the scanned block sums)
__global__ void __launch_bounds__(kBlock) k_count_offsets(const int64_t* __restrict__ counts, uint32_t n,
                                                          const uint32_t* __restrict__ block_first,
                                                          uint32_t* __restrict__ first) {
    __shared__ uint32_t s_wave[kBlock / kWave];
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    uint32_t run = block_first[blockIdx.x];
#pragma unroll
    for (int j = 0; j < kSelectItems; ++j) {
        const uint32_t i = blockIdx.x * kSelectTile + j * kBlock + threadIdx.x;
        const uint32_t v = i < n ? (uint32_t)counts[i] : 0u;
        uint32_t incl = v;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t up = __shfl_up(incl, d, 64);
            if (lane >= (uint32_t)d) incl += up;
        }
        if (lane == 63) s_wave[wave] = incl;
        __syncthreads();
        uint32_t before = run, all = 0;
#pragma unroll
        for (int w = 0; w < kBlock / kWave; ++w) {
            const uint32_t c = s_wave[w];
            if ((uint32_t)w < wave) before += c;
            all += c;
        }
        if (i < n) {
            first[i] = before + incl - v;
            if (i == n - 1) first[n] = before + incl;
        }
        run += all;
        __syncthreads();
    }
}

__device__ __forceinline__ float halton(uint32_t index, uint32_t base) {   // utils.py:36-45
    double result = 0.0, f = 1.0 / (double)base;
    for (uint32_t i = index; i > 0; i /= base) {
        result += f * (double)(i % base);
        f /= (double)base;
    }
    return (float)result;
}

__global__ void __launch_bounds__(kBlock) k_extract_global(const float* __restrict__ centers, const int32_t* __restrict__ levels,
                                                           const uint32_t* __restrict__ first, uint32_t n_leaves,
                                                           float size_x, float size_y, float size_z,
                                                           float* __restrict__ positions, uint32_t n_samples) {
    const uint32_t s = blockIdx.x * kBlock + threadIdx.x;
    if (s >= n_samples) return;
    // last leaf with first[leaf] <= s (leaves without samples have empty runs and are never that leaf)
    uint32_t lo = 0, hi = n_leaves;
    while (hi - lo > 1) {
        const uint32_t mid = (lo + hi) >> 1;
        if (first[mid] <= s) lo = mid;
        else hi = mid;
    }
    const uint32_t leaf = lo, begin = first[leaf], count = first[leaf + 1] - begin;
    float x = centers[3 * (size_t)leaf], y = centers[3 * (size_t)leaf + 1], z = centers[3 * (size_t)leaf + 2];
    if (count != 1u) {
        const uint32_t h = s - begin + 1u;
        const int level = levels[leaf];
        const float sx = ldexpf(size_x, -level), sy = ldexpf(size_y, -level), sz = ldexpf(size_z, -level);
        x = (x - sx / 2.0f) + halton(h, 2u) * sx;
        y = (y - sy / 2.0f) + halton(h, 3u) * sy;
        z = (z - sz / 2.0f) + halton(h, 5u) * sz;
    }
    positions[3 * (size_t)s] = x;
    positions[3 * (size_t)s + 1] = y;
    positions[3 * (size_t)s + 2] = z;
}

// ---- Morton codes ------------------------------------------------------------------------------------
// bounds[0..2] = ordered keys of the per-axis minima, bounds[3..5] of the maxima (set to kNoMin / kNoMax before).
__global__ void __launch_bounds__(kBlock) k_morton_bounds(const float* __restrict__ positions, uint32_t n,
                                                          uint32_t* __restrict__ bounds) {
    uint32_t lo[3] = {kNoMin, kNoMin, kNoMin}, hi[3] = {kNoMax, kNoMax, kNoMax};
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
#pragma unroll
        for (int a = 0; a < 3; ++a) {
            const uint32_t k = ordered_key(positions[3 * i + a]);
            lo[a] = min(lo[a], k);
            hi[a] = max(hi[a], k);
        }
    }
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        for (int s = 32; s > 0; s >>= 1) {
            lo[a] = min(lo[a], (uint32_t)__shfl_xor(lo[a], s, 64));
            hi[a] = max(hi[a], (uint32_t)__shfl_xor(hi[a], s, 64));
        }
    }
    if (lane_id() == 0) {
#pragma unroll
        for (int a = 0; a < 3; ++a) {
            atomicMin(bounds + a, lo[a]);
            atomicMax(bounds + 3 + a, hi[a]);
        }
    }
}

// Bit k of v goes to bit 3 k (v < 2^21).
__device__ __forceinline__ uint64_t spread3(uint32_t v) {
    uint64_t x = v;
    x = (x | (x << 32)) & 0x001F00000000FFFFull;
    x = (x | (x << 16)) & 0x001F0000FF0000FFull;
    x = (x | (x << 8)) & 0x100F00F00F00F00Full;
    x = (x | (x << 4)) & 0x10C30C30C30C30C3ull;
    x = (x | (x << 2)) & 0x1249249249249249ull;
    return x;
}

constexpr uint32_t kMortonCells = 1u << 21;   // per axis: 63 bits in all

__global__ void __launch_bounds__(kBlock) k_morton_encode(const float* __restrict__ positions, uint32_t n,
                                                          const uint32_t* __restrict__ bounds,
                                                          int64_t* __restrict__ codes) {
    const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    const float lx = ordered_value(bounds[0]), ly = ordered_value(bounds[1]), lz = ordered_value(bounds[2]);
    const float extent = fmaxf(fmaxf(ordered_value(bounds[3]) - lx, ordered_value(bounds[4]) - ly),
                               ordered_value(bounds[5]) - lz);
    const float scale = extent > 0.0f ? (float)kMortonCells / extent : 0.0f;
    const float lo[3] = {lx, ly, lz};
    uint64_t code = 0;
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        const float q = (positions[3 * (size_t)i + a] - lo[a]) * scale;
        const uint32_t cell = min((uint32_t)q, kMortonCells - 1u);   // q >= 0; the maximum lands on 2^21
        code |= spread3(cell) << a;
    }
    codes[i] = (int64_t)code;
}

int select_offsets(const float* values, const int32_t* levels, uint32_t n, float threshold, int max_level,
                   uint32_t* block_offsets, uint32_t* counts, hipStream_t stream) {
    const uint32_t blocks = div_up(n, kSelectTile);
    INPC_LAUNCH("field_select_count", k_select_count, dim3(blocks), dim3(kBlock), stream, values, levels, n, threshold,
                max_level, block_offsets);
    INPC_LAUNCH("field_select_scan", k_select_scan, dim3(1), dim3(kBlock), stream, block_offsets, blocks, counts);
    return INPC_OK;
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
    if (((uintptr_t)workspace & 7u) != 0) return fail(INPC_E_WORKSPACE, "field_update: workspace must be 8-byte aligned");
    uint32_t* error_flag = (uint32_t*)workspace;
    uint2* keys = (uint2*)((uint32_t*)workspace + 64);
    int rc = fill_u32(error_flag, 0u, 1, stream);
    if (rc != INPC_OK) return rc;
    const uint32_t leaf_blocks = std::min<uint32_t>(div_up(n_leaves, kBlock), 4096u);
    INPC_LAUNCH("field_reset", k_field_reset, dim3(leaf_blocks), dim3(kBlock), stream, keys, n_leaves);
    if (n_samples > 0)
        INPC_LAUNCH("field_scatter", k_field_scatter, dim3(std::min<uint32_t>(div_up(n_samples, kBlock), 8192u)),
                    dim3(kBlock), stream, indices, weights, n_samples, keys, n_leaves, error_flag);
    INPC_LAUNCH("field_finish", k_field_finish, dim3(leaf_blocks), dim3(kBlock), stream, (const uint2*)keys, leaf_weights,
                leaf_scores, n_leaves, decay);
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


size_t inpc_field_select_workspace_bytes(uint32_t n_leaves) {
    return (size_t)inpc::div_up(std::max(n_leaves, 1u), (uint32_t)inpc::kSelectTile) * 4 + 256;
}

int inpc_field_select_count(const float* values, const int32_t* levels, uint32_t n_leaves, float threshold, int max_level,
                            uint32_t* count_out, void* workspace, size_t workspace_bytes, void* stream) {
    using namespace inpc;
    if (!count_out) return fail(INPC_E_INVALID_ARGUMENT, "field_select_count: null count");
    if (n_leaves == 0) return fill_u32(count_out, 0u, 1, (hipStream_t)stream);
    if (!values) return fail(INPC_E_INVALID_ARGUMENT, "field_select_count: null values");
    if (!workspace || workspace_bytes < inpc_field_select_workspace_bytes(n_leaves))
        return fail(INPC_E_WORKSPACE, "field_select_count: workspace too small");
    return select_offsets(values, levels, n_leaves, threshold, max_level, (uint32_t*)workspace, count_out, (hipStream_t)stream);
}

int inpc_field_prune(const float* centers, const int32_t* levels, const float* weights, const float* scores,
                     uint32_t n_leaves, float threshold, float* centers_out, int32_t* levels_out, float* weights_out,
                     float* scores_out, uint32_t* count_out, void* workspace, size_t workspace_bytes, void* stream_) {
    using namespace inpc;
    hipStream_t stream = (hipStream_t)stream_;
    if (!count_out) return fail(INPC_E_INVALID_ARGUMENT, "field_prune: null count");
    if (n_leaves == 0) return fill_u32(count_out, 0u, 1, stream);
    if (!centers || !levels || !weights || !scores || !centers_out || !levels_out || !weights_out || !scores_out)
        return fail(INPC_E_INVALID_ARGUMENT, "field_prune: null pointer");
    if (!workspace || workspace_bytes < inpc_field_select_workspace_bytes(n_leaves))
        return fail(INPC_E_WORKSPACE, "field_prune: workspace too small");
    uint32_t* offsets = (uint32_t*)workspace;
    const int rc = select_offsets(weights, nullptr, n_leaves, threshold, 0, offsets, count_out, stream);
    if (rc != INPC_OK) return rc;
    INPC_LAUNCH("field_prune", k_prune_apply, dim3(div_up(n_leaves, kSelectTile)), dim3(kBlock), stream,
                (LeafArrays{centers, levels, weights, scores}), (LeafOutputs{centers_out, levels_out, weights_out, scores_out}),
                n_leaves, threshold, (const uint32_t*)offsets);
    return INPC_OK;
}

int inpc_field_subdivide(const float* centers, const int32_t* levels, const float* weights, const float* scores,
                         uint32_t n_leaves, float threshold, int max_level, const float initial_size[3],
                         float* centers_out, int32_t* levels_out, float* weights_out, float* scores_out,
                         uint32_t* count_out, void* workspace, size_t workspace_bytes, void* stream_) {
    using namespace inpc;
    hipStream_t stream = (hipStream_t)stream_;
    if (!count_out) return fail(INPC_E_INVALID_ARGUMENT, "field_subdivide: null count");
    if (n_leaves == 0) return fill_u32(count_out, 0u, 1, stream);
    if (!centers || !levels || !weights || !scores || !centers_out || !levels_out || !weights_out || !scores_out ||
        !initial_size)
        return fail(INPC_E_INVALID_ARGUMENT, "field_subdivide: null pointer");
    if (!workspace || workspace_bytes < inpc_field_select_workspace_bytes(n_leaves))
        return fail(INPC_E_WORKSPACE, "field_subdivide: workspace too small");
    uint32_t* offsets = (uint32_t*)workspace;
    const int rc = select_offsets(scores, levels, n_leaves, threshold, max_level, offsets, count_out, stream);
    if (rc != INPC_OK) return rc;
    INPC_LAUNCH("field_subdivide", k_subdivide_apply, dim3(div_up(n_leaves, kSelectTile)), dim3(kBlock), stream,
                (LeafArrays{centers, levels, weights, scores}), (LeafOutputs{centers_out, levels_out, weights_out, scores_out}),
                n_leaves, threshold, max_level, initial_size[0], initial_size[1], initial_size[2], (const uint32_t*)offsets,
                (const uint32_t*)count_out);
    return INPC_OK;
}


size_t inpc_extract_global_workspace_bytes(uint32_t n_leaves) {
    const size_t blocks = inpc::div_up(std::max(n_leaves, 1u), (uint32_t)inpc::kSelectTile);
    return 256 + inpc::align_up(blocks * 4, 256) + ((size_t)n_leaves + 1) * 4;
}

int inpc_extract_global(const float* centers, const int32_t* levels, const int64_t* counts, uint32_t n_leaves,
                        const float initial_size[3], float* positions_out, uint32_t n_samples, void* workspace,
                        size_t workspace_bytes, void* stream_) {
    using namespace inpc;
    hipStream_t stream = (hipStream_t)stream_;
    if (!workspace || workspace_bytes < inpc_extract_global_workspace_bytes(n_leaves))
        return fail(INPC_E_WORKSPACE, "extract_global: workspace too small");
    uint32_t* head = (uint32_t*)workspace;   // [0] total of the counts, [1] error flag
    int rc = fill_u32(head, 0u, 2, stream);
    if (rc != INPC_OK) return rc;
    if (n_leaves == 0 || n_samples == 0) return INPC_OK;
    if (!centers || !levels || !counts || !initial_size || !positions_out)
        return fail(INPC_E_INVALID_ARGUMENT, "extract_global: null pointer");
    const uint32_t blocks = div_up(n_leaves, kSelectTile);
    uint32_t* block_sums = head + 64;
    uint32_t* first = (uint32_t*)((char*)workspace + 256 + align_up((size_t)blocks * 4, 256));
    INPC_LAUNCH("global_count_sums", k_count_block_sums, dim3(blocks), dim3(kBlock), stream, counts, n_leaves, block_sums,
                head + 1);
    INPC_LAUNCH("field_select_scan", k_select_scan, dim3(1), dim3(kBlock), stream, block_sums, blocks, head);
    INPC_LAUNCH("global_count_offsets", k_count_offsets, dim3(blocks), dim3(kBlock), stream, counts, n_leaves,
                (const uint32_t*)block_sums, first);
    INPC_LAUNCH("extract_global", k_extract_global, dim3(div_up(n_samples, kBlock)), dim3(kBlock), stream, centers, levels,
                (const uint32_t*)first, n_leaves, initial_size[0], initial_size[1], initial_size[2], positions_out,
                n_samples);
    return INPC_OK;
}

int inpc_extract_global_check(const void* workspace, uint32_t n_samples, void* stream_) {
    using namespace inpc;
    hipStream_t stream = (hipStream_t)stream_;
    uint32_t head[2] = {0, 0};
    INPC_HIP_CHECK(hipMemcpyAsync(head, workspace, 8, hipMemcpyDeviceToHost, stream));
    INPC_HIP_CHECK(hipStreamSynchronize(stream));
    if (head[1]) return fail(INPC_E_INVALID_ARGUMENT, "extract_global: a count is negative or above 2^31 - 1");
    if (head[0] != n_samples)
        return fail(INPC_E_INVALID_ARGUMENT, "extract_global: the counts add up to %u, not to the %u samples asked for",
                    head[0], n_samples);
    return INPC_OK;
}

size_t inpc_morton_workspace_bytes(void) { return 256; }

int inpc_morton_encode(const float* positions, uint32_t n, int64_t* codes_out, void* workspace, size_t workspace_bytes,
                       void* stream_) {
    using namespace inpc;
    hipStream_t stream = (hipStream_t)stream_;
    if (n == 0) return INPC_OK;
    if (!positions || !codes_out) return fail(INPC_E_INVALID_ARGUMENT, "morton_encode: null pointer");
    if (!workspace || workspace_bytes < inpc_morton_workspace_bytes())
        return fail(INPC_E_WORKSPACE, "morton_encode: workspace too small");
    uint32_t* bounds = (uint32_t*)workspace;
    int rc = fill_u32(bounds, kNoMin, 3, stream);
    if (rc != INPC_OK) return rc;
    rc = fill_u32(bounds + 3, kNoMax, 3, stream);
    if (rc != INPC_OK) return rc;
    INPC_LAUNCH("morton_bounds", k_morton_bounds, dim3(std::min(div_up(n, kBlock), 2048u)), dim3(kBlock), stream,
                positions, n, bounds);
    INPC_LAUNCH("morton_encode", k_morton_encode, dim3(div_up(n, kBlock)), dim3(kBlock), stream, positions, n,
                (const uint32_t*)bounds, codes_out);
    return INPC_OK;
}

}  // extern "C"
