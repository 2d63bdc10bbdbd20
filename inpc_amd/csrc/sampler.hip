// sampler.hip — view-dependent point sampling from the octree probability field (gfx950).
//
//   k_leaf_weights        per-leaf visibility + weight   (B/sampling/src/sampling_kernels.cu:9-64)
//   k_tile_totals / k_cdf_scan_tiles / k_cdf_finish
//                         normalise + float CDF with a fixed association order (chunks of 64,
//                         left to right, recursively) and the top of the search tree, in three
//                         launches                         (B/sampling/src/sampling.cu:150-186)
//   k_sample              multinomial leaf pick + jitter  (B/sampling/src/sampling_kernels.cu:128-150)
//   k_sample_cull         the same draw, frustum test, ordered stream compaction
//                                                         (B/sampling/src/sampling_kernels.cu:77-126)
//   k_tile_totals + k_expected_counts / k_repeat_interleave / k_expected_samples
//                                                         (B/sampling/src/sampling_kernels.cu:152-205)
//
// Candidate k always uses the sampler's generator advanced by 4*k draws. A thread walks candidates
// 256 apart, so it pays one O(log k) jump at the start and one constant affine step per candidate.
#include <algorithm>
#include <mutex>

#include "common.hpp"

namespace inpc {

namespace {

constexpr float kFltEps = 1e-8f;
constexpr int kBlock = 256;
constexpr int kChunk = 64;
constexpr int kChunksPerBlock = 64;                      // one wave scans 64 chunks
constexpr int kChunkTile = kChunk * kChunksPerBlock;     // 4096 floats per block
constexpr int kSampleItems = 8;                          // candidates per thread
constexpr int kSampleTile = kBlock * kSampleItems;       // candidates per block (expected-count sampler)
constexpr int kDrawBlock = 512;                          // threads per block of the sampling kernels that search the CDF
constexpr int kDrawTile = kDrawBlock * kSampleItems;     // candidates per block of those

struct Rows {
    float4 r1, r2, r3;
};

__device__ __forceinline__ Rows load_rows(const float* w2c) {
    Rows r;
    r.r1 = make_float4(w2c[0], w2c[1], w2c[2], w2c[3]);
    r.r2 = make_float4(w2c[4], w2c[5], w2c[6], w2c[7]);
    r.r3 = make_float4(w2c[8], w2c[9], w2c[10], w2c[11]);
    return r;
}

// Conjunction of "inside" comparisons (NaN is not visible), sampling_kernels.cu:31-36.
__device__ __forceinline__ bool leaf_point_visible(const Rows& m, float x, float y, float z, const Camera& cam) {
    const float vz = affine_row(m.r3, x, y, z);
    const float inv_z = 1.0f / (vz + kFltEps);
    const float sx = affine_row(m.r1, x, y, z) * inv_z * cam.fx + cam.cx;
    const float sy = affine_row(m.r2, x, y, z) * inv_z * cam.fy + cam.cy;
    return (vz >= cam.near_plane) & (vz <= cam.far_plane) & (sx >= 0.0f) & (sx < cam.width) & (sy >= 0.0f) &
           (sy < cam.height);
}

// Sequence of "outside" rejections (NaN is not rejected), sampling_kernels.cu:110-119.
__device__ __forceinline__ bool sample_accepted(const Rows& m, float x, float y, float z, const Camera& cam) {
    const float vz = affine_row(m.r3, x, y, z);
    if (vz < cam.near_plane || vz > cam.far_plane) return false;
    const float inv_z = 1.0f / (vz + kFltEps);
    const float sx = affine_row(m.r1, x, y, z) * inv_z * cam.fx + cam.cx;
    if (sx < 0.0f || sx >= cam.width) return false;
    const float sy = affine_row(m.r2, x, y, z) * inv_z * cam.fy + cam.cy;
    if (sy < 0.0f || sy >= cam.height) return false;
    return true;
}

__global__ void __launch_bounds__(kBlock) k_leaf_weights(const float* __restrict__ centers,
                                                         const int32_t* __restrict__ levels,
                                                         const float* __restrict__ weights,
                                                         const float* __restrict__ w2c, float* __restrict__ out,
                                                         float4* __restrict__ boxes, uint32_t n_leaves, Camera cam,
                                                         float initial_size) {
    const uint32_t l = blockIdx.x * kBlock + threadIdx.x;
    if (l >= n_leaves) return;
    const Rows m = load_rows(w2c);
    const float cx = centers[3 * (size_t)l], cy = centers[3 * (size_t)l + 1], cz = centers[3 * (size_t)l + 2];
    const int level = levels[l];
    // centre and edge length in one 16-byte word: the sampling kernels fetch it with one gather instead of four
    if (boxes) boxes[l] = make_float4(cx, cy, cz, ldexpf(1.0f, -level) * initial_size);
    const float z = affine_row(m.r3, cx, cy, cz);
    bool valid = leaf_point_visible(m, cx, cy, cz, cam);
    if (!valid) {
        const float half = ldexpf(initial_size, -(level + 1));
        for (int corner = 0; corner < 8; ++corner) {
            const float ox = (corner & 4) ? half : -half;
            const float oy = (corner & 2) ? half : -half;
            const float oz = (corner & 1) ? half : -half;
            valid = valid | leaf_point_visible(m, cx + ox, cy + oy, cz + oz, cam);
        }
    }
    float wgt = 0.0f;
    if (valid) {
        const float depth_scale = fmaxf(fabsf(z - cam.near_plane) / cam.far_plane, kFltEps);
        const float size_scale = ldexpf((level & 1) ? 1.41421356f : 1.0f, level >> 1);
        wgt = 1.0f / (depth_scale * size_scale) * weights[l];
    }
    out[l] = wgt;
}

// ---- sums and scans in the fixed association order ------------------------------------------------------------------
// Left to right inside chunks of 64 values, the chunk totals combined the same way one level up, recursively; a scanned
// element is its chunk's local scan plus the final scanned total of the chunks in front (B/sampling/src/sampling.cu:
// 150-186 leaves the order to cub; this one is the library's own, so that a CPU restatement can follow it bit for
// bit). A block of one wave takes a tile of 64 chunks, which is one chunk of the level above.

// Stages the tile's 64 rows of 64 floats in LDS (row stride 65: lane c then walks row c without bank conflicts).
// `scale` multiplies every element on the way in.
__device__ __forceinline__ void stage_tile(float* tile, const float* data, size_t base, uint32_t n, float scale,
                                           uint32_t lane) {
    // the loads of sixteen rows are issued together (one row at a time left the wave waiting on every load)
    for (int r0 = 0; r0 < kChunksPerBlock; r0 += 16) {
        float v[16];
#pragma unroll
        for (int k = 0; k < 16; ++k) {
            const size_t i = base + (size_t)(r0 + k) * kChunk + lane;
            v[k] = i < n ? data[i] : 0.0f;
        }
#pragma unroll
        for (int k = 0; k < 16; ++k) tile[(r0 + k) * (kChunk + 1) + lane] = v[k] * scale;
    }
}

// values[0] + values[1] + ... + values[len - 1], left to right; 1 <= len <= 64. All 64 values are fetched before the
// first addition (the storage behind `values` holds a whole chunk; what lies behind `len` is not used).
__device__ __forceinline__ float chunk_sum(const float* values, uint32_t len) {
    float v[kChunk];
#pragma unroll
    for (int i = 0; i < kChunk; ++i) v[i] = values[i];
    float s = v[0];
#pragma unroll
    for (int i = 1; i < kChunk; ++i)
        if ((uint32_t)i < len) s += v[i];
    return s;
}

// The same additions with every partial sum written back: values[i] = values[0] + ... + values[i] for i < len; returns
// the last one. One round of loads, the additions in registers, one round of stores (a load and a store per step kept
// the chain waiting on LDS 64 times).
__device__ __forceinline__ float chunk_scan(float* values, uint32_t len) {
    float v[kChunk];
#pragma unroll
    for (int i = 0; i < kChunk; ++i) v[i] = values[i];
    float s = v[0];
#pragma unroll
    for (int i = 1; i < kChunk; ++i)
        if ((uint32_t)i < len) {
            s += v[i];
            values[i] = s;
        }
    return s;
}

// The totals of `m` values one and two levels up, by one wave: s_a[k] = total of chunk k of `values` (k < ceil(m / 64)
// <= 4096), s_b[k] = total of chunk k of s_a. Ends with the LDS of the wave in order.
constexpr uint32_t kMaxUpperValues = 1u << 18;   // values of the level that tops a tile: 2^30 leaves
constexpr uint32_t kMaxCdfLeaves = 1u << 30;
__device__ __forceinline__ void upper_totals(const float* values, uint32_t m, float* s_a, float* s_b, uint32_t lane) {
    const uint32_t m_a = (m + kChunk - 1) / kChunk, m_b = (m_a + kChunk - 1) / kChunk;
    for (uint32_t k = lane; k < m_a; k += kWave) s_a[k] = chunk_sum(values + (size_t)k * kChunk, min((uint32_t)kChunk, m - k * kChunk));
    wave_sync();
    if (lane < m_b) s_b[lane] = chunk_sum(s_a + lane * kChunk, min((uint32_t)kChunk, m_a - lane * kChunk));
    wave_sync();
}

// Total of the `m` values (m <= kMaxUpperValues) behind upper_totals; the same in every lane.
__device__ __forceinline__ float blocked_total(uint32_t m, const float* s_b) {
    const uint32_t m_a = (m + kChunk - 1) / kChunk, m_b = (m_a + kChunk - 1) / kChunk;
    return chunk_sum(s_b, m_b);
}

// Element j of the inclusive scan of the `m` values, behind upper_totals.
__device__ __forceinline__ float blocked_scan_at(const float* values, uint32_t j, const float* s_a, const float* s_b) {
    const uint32_t c0 = j / kChunk;
    const float local0 = chunk_sum(values + (size_t)c0 * kChunk, j - c0 * kChunk + 1u);
    if (c0 == 0u) return local0;
    const uint32_t ja = c0 - 1u, ca = ja / kChunk;
    const float local_a = chunk_sum(s_a + ca * kChunk, ja - ca * kChunk + 1u);
    if (ca == 0u) return local_a + local0;
    const float final_b = chunk_sum(s_b, ca);   // scan of s_b at ca - 1: s_b is a single chunk
    return (final_b + local_a) + local0;
}

// Level 1 and 2 of a sum: tile_totals[b] = total of tile b's chunk totals. Totals only, `data` is not written.
// `clear` (n_clear floats, or null) is set to zero, a slice per block.
__global__ void __launch_bounds__(kWave) k_tile_totals(const float* __restrict__ data, uint32_t n,
                                                       float* __restrict__ tile_totals, float* __restrict__ clear,
                                                       uint32_t n_clear) {
    __shared__ float tile[kChunksPerBlock * (kChunk + 1)];
    __shared__ float s_chunk[kChunk];
    const uint32_t lane = threadIdx.x;
    const size_t base = (size_t)blockIdx.x * kChunkTile;
    if (clear) {
        const uint32_t per_block = (n_clear + gridDim.x - 1u) / gridDim.x, first = blockIdx.x * per_block;
        for (uint32_t i = first + lane; i < min(first + per_block, n_clear); i += kWave) clear[i] = 0.0f;
    }
    stage_tile(tile, data, base, n, 1.0f, lane);
    __syncthreads();
    const size_t chunk_base = base + (size_t)lane * kChunk;
    float s = 0.0f;
    if (chunk_base < n) {
        const int len = (int)min((size_t)kChunk, (size_t)n - chunk_base);
        s = chunk_sum(tile + lane * (kChunk + 1), (uint32_t)len);
    }
    s_chunk[lane] = s;
    wave_sync();
    const uint32_t n_chunks = min((uint32_t)kChunksPerBlock, (uint32_t)(((size_t)n - base + kChunk - 1) / kChunk));
    const float total = chunk_sum(s_chunk, n_chunks);
    if (lane == 0u) tile_totals[blockIdx.x] = total;
}

// The total on top of k_tile_totals (every block computes it: at most 2^18 values, 64 for 262,144 leaves), then the
// tile's elements times 1 / total, scanned inside their chunks in place; scanned_chunk_totals[c] = the scan of the
// tile's chunk totals inside the tile (level 1, local), tile_totals_out[b] = its last element (level 2). head[0] = the
// total; when that is not positive nothing else is written.
__global__ void __launch_bounds__(kWave) k_cdf_scan_tiles(float* data, uint32_t n, const float* __restrict__ raw_tile_totals,
                                                          float* __restrict__ scanned_chunk_totals,
                                                          float* __restrict__ tile_totals_out, float* __restrict__ head) {
    __shared__ float tile[kChunksPerBlock * (kChunk + 1)];   // first the totals one level above the tile totals
    __shared__ float s_b[kChunk];
    __shared__ float s_chunk[kChunk];
    static_assert(kMaxUpperValues / kChunk <= kChunksPerBlock * (kChunk + 1), "the upper totals fit the tile's LDS");
    const uint32_t lane = threadIdx.x;
    const uint32_t n_tiles = gridDim.x;
    upper_totals(raw_tile_totals, n_tiles, tile, s_b, lane);
    const float sum = blocked_total(n_tiles, s_b);
    if (blockIdx.x == 0u && lane == 0u) head[0] = sum;
    if (!(sum > 0.0f)) return;
    const float norm = 1.0f / sum;
    const size_t base = (size_t)blockIdx.x * kChunkTile;
    wave_sync();   // the upper totals have been read
    stage_tile(tile, data, base, n, norm, lane);
    __syncthreads();
    const size_t chunk_base = base + (size_t)lane * kChunk;
    float s = 0.0f;
    if (chunk_base < n) {
        const int len = (int)min((size_t)kChunk, (size_t)n - chunk_base);
        s = chunk_scan(tile + lane * (kChunk + 1), (uint32_t)len);
    }
    s_chunk[lane] = s;
    __syncthreads();
#pragma unroll 16
    for (int r = 0; r < kChunksPerBlock; ++r) {
        const size_t i = base + (size_t)r * kChunk + lane;
        if (i < n) data[i] = tile[r * (kChunk + 1) + lane];
    }
    // the chunk totals scanned left to right; lane c keeps element c
    const uint32_t n_chunks = min((uint32_t)kChunksPerBlock, (uint32_t)(((size_t)n - base + kChunk - 1) / kChunk));
    float v[kChunk];
#pragma unroll
    for (int i = 0; i < kChunk; ++i) v[i] = s_chunk[i];
    float run = v[0], mine = v[0];
#pragma unroll
    for (int i = 1; i < kChunk; ++i) {
        if ((uint32_t)i < n_chunks) run += v[i];
        if ((uint32_t)i == lane) mine = run;
    }
    if (lane < n_chunks) scanned_chunk_totals[(size_t)blockIdx.x * kChunksPerBlock + lane] = mine;
    if (lane == 0u) tile_totals_out[blockIdx.x] = run;
}

// The leaf of a sample is std::lower_bound over the CDF with the probe sequence of
// B/sampling/include/sampling_utils.h:49-69:
//     first = 0, count = n;  while (count > 0) { step = count / 2; it = first + step;
//         if (cdf[it] < sample) { first = it + 1; count -= step + 1; } else count = step; }
//     leaf = min(first, n - 1)
// draw_candidates below makes exactly these probes, level by level for all candidates of a thread.
//
// The top of the decision tree of that search lives in LDS. Which element the k-th probe reads depends only on
// the outcomes of the probes before it, so the first kTreeDepth probes can only touch 2^kTreeDepth - 1 fixed
// elements. inpc_build_cdf leaves those, in heap order (node 1 = first probe, node 2n / 2n + 1 = the probe after
// going left / right), behind the total in the CDF head; a block copies them into LDS and reads the CDF itself
// only below that depth. The comparisons are exactly those of the sequence above, so the result is the same even
// where rounding leaves the CDF not perfectly monotone; for 262,144 leaves 14 of the 18 dependent cache round
// trips of a sample become LDS reads and the other four fall into one 64-byte stretch. The tree takes 64 KB of LDS,
// shared by the 512 threads of a block (two blocks per CU); every probe that still reads the CDF itself is a load
// whose 64 lanes touch 64 different lines and costs the kernel as much as all its arithmetic (13 levels for 256
// threads: cull kernel 0.32 instead of 0.27 ms).
constexpr uint32_t kFetch = 16;   // elements of a search that four lanes fetch together
constexpr int kTreeDepth = 14;
constexpr uint32_t kTreeNodes = 1u << kTreeDepth;  // heap indices 1 .. kTreeNodes - 1; index 0 of the head: the total
static_assert(kTreeNodes == INPC_CDF_HEAD_MIN_FLOATS, "the CDF head holds the total and the search tree");
static_assert(kSampleItems * (kDrawBlock / kWave) <= kWave, "one wave scans the (round, wave) counts of a tile");

// Levels of the tree for n leaves: at least kTreeDepth (the part a block keeps in LDS), and as many as leave a search
// with at most kFetch elements (every level halves what is left). The levels below kTreeDepth are read from the head
// in memory: for 2,097,152 leaves three levels, 448 KB that stay in the second-level cache, where probes of the CDF
// itself fetch a 128-byte line from memory for every 4-byte element (12.9 GB for 33,554,432 samples).
constexpr int kMaxTreeDepth = 24;
__host__ __device__ __forceinline__ int tree_levels(uint32_t n_leaves) {
    int levels = kTreeDepth;
    while (levels < kMaxTreeDepth && (n_leaves >> levels) > kFetch) ++levels;
    return levels;
}

// Last step of the CDF: the scanned totals of the chunks in front are added to every element, and the elements that
// the first `levels` probes of the search can read go to the head. Which node of the decision tree probes element i
// follows from i alone: the search for position i is replayed on the indices (no memory access) until it probes i
// itself; every element is probed by exactly one node. Nodes that no search reaches (fewer leaves than the tree has
// nodes) keep the zero they got from k_tile_totals.
constexpr int kFinishItems = 8;
constexpr int kFinishTile = kBlock * kFinishItems;   // elements per block: a whole number of chunks, a divisor of a tile
static_assert(kFinishTile % kChunk == 0 && kChunkTile % kFinishTile == 0, "a block's elements lie in one tile");
__global__ void __launch_bounds__(kBlock) k_cdf_finish(float* data, uint32_t n, const float* __restrict__ scanned_chunk_totals,
                                                       const float* __restrict__ tile_totals, uint32_t n_tiles,
                                                       float* __restrict__ head, int levels) {
    __shared__ float s_a[kMaxUpperValues / kChunk];
    __shared__ float s_b[kChunk];
    __shared__ float s_front[2];                      // scan of the tile totals at tile - 1 and tile - 2
    __shared__ float s_prefix[kFinishTile / kChunk];  // what is added to the block's chunks
    if (!(head[0] > 0.0f)) return;
    const uint32_t tid = threadIdx.x;
    const uint32_t first = blockIdx.x * (uint32_t)kFinishTile;
    const uint32_t tile = first / (uint32_t)kChunkTile;
    // final scanned total (level 1) of the chunk in front of chunk c is
    //   scanned_chunk_totals[c - 1] + the scan of the tile totals (level 2) at tile(c - 1) - 1
    if (tid < (uint32_t)kWave && tile > 0u) {
        upper_totals(tile_totals, tile, s_a, s_b, tid);   // only the tiles in front matter
        if (tid < 2u && tile > tid) s_front[tid] = blocked_scan_at(tile_totals, tile - 1u - tid, s_a, s_b);
    }
    __syncthreads();
    if (tid < (uint32_t)(kFinishTile / kChunk)) {
        const uint32_t c = first / (uint32_t)kChunk + tid;
        float prefix = 0.0f;
        if (c > 0u && (size_t)c * kChunk < n) {
            const uint32_t before = c - 1u, its_tile = before / (uint32_t)kChunksPerBlock;
            prefix = scanned_chunk_totals[before];
            if (its_tile > 0u) prefix = s_front[tile - its_tile] + prefix;
        }
        s_prefix[tid] = prefix;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kFinishItems; ++k) {
        const uint32_t offset = (uint32_t)k * kBlock + tid, i = first + offset;
        if (i >= n) continue;
        float v = data[i];
        if (i >= (uint32_t)kChunk) {
            v = s_prefix[offset / (uint32_t)kChunk] + v;
            data[i] = v;
        }
        uint32_t lo = 0u, count = n, node = 1u;
        for (int depth = 0; depth < levels; ++depth) {
            const uint32_t step = count >> 1, it = lo + step;
            if (it == i) {
                head[node] = v;
                break;
            }
            if (it < i) {
                lo = it + 1u;
                count -= step + 1u;
                node = 2u * node + 1u;
            } else {
                count = step;
                node = 2u * node;
            }
        }
    }
}

// Every thread of the block must call it; ends with a barrier. s_tree[0] (the total) is not used.
__device__ __forceinline__ void load_search_tree(float* s_tree, const float* __restrict__ head) {
    const float4* src = (const float4*)head;
    float4* dst = (float4*)s_tree;
    for (uint32_t i = threadIdx.x; i < kTreeNodes / 4; i += blockDim.x) dst[i] = src[i];
    __syncthreads();
}

struct Candidate {
    uint32_t leaf;
    float x, y, z;
};

// A candidate k takes draws 4k .. 4k + 3 of the stream: u picks the leaf (lower_bound over the CDF, the probe
// sequence above with the first kTreeDepth probes read from the tree), the other three place the
// point in the leaf's cell; boxes[leaf] = {centre, edge length} (B/sampling/src/sampling_kernels.cu:141-147:
// centre + (u - 0.5) * initial_size / 2^level).

// ---- the kSampleItems candidates of a thread, side by side ---------------------------------------------------------
// One candidate is a chain of dependent steps (four generator steps, up to 19 probes of the CDF, the box of the
// leaf); a thread that takes its candidates one after the other spends its time waiting for the next link. Here the
// chains of all its candidates advance together: every generator state comes from the thread's first one by a jump
// of its own, and the part of the searches that reads the tree in LDS runs level by level for all candidates, without
// branches, so that the probes of one level are in flight together. The values and comparisons are those of the
// sequential form.
__device__ __forceinline__ float pcg_float_of(uint64_t state) {   // the output of the generator standing at `state`
    const uint32_t xs = (uint32_t)(((state >> 18u) ^ state) >> 27u);
    const uint32_t rot = (uint32_t)(state >> 59u);
    const uint32_t v = (xs >> rot) | (xs << ((~rot + 1u) & 31u));
    return __uint_as_float((v >> 9) | 0x3f800000u) - 1.0f;
}

struct TileJumps {
    PcgJump row[kSampleItems];   // from the thread's first candidate of a tile to its j-th: 4 * kDrawBlock * j draws
    PcgJump draw[3];             // from a candidate's first draw to its second, third and fourth
};

__device__ __forceinline__ TileJumps make_tile_jumps(uint64_t inc) {
    TileJumps t;
#pragma unroll
    for (int j = 0; j < kSampleItems; ++j) t.row[j] = pcg_jump(inc, 4ull * kDrawBlock * (uint64_t)j);
#pragma unroll
    for (int d = 0; d < 3; ++d) t.draw[d] = pcg_jump(inc, (uint64_t)d + 1u);
    return t;
}

// `state0`: the generator at the first draw of the thread's first candidate; live[j]: candidate j exists.
__device__ __forceinline__ void draw_candidates(uint64_t state0, const TileJumps& jumps, const bool (&live)[kSampleItems],
                                                const float4* __restrict__ boxes, const float* __restrict__ cdf,
                                                const float* __restrict__ head, const float* s_tree,
                                                uint32_t n_leaves, Candidate (&c)[kSampleItems]) {
    float u[kSampleItems], ox[kSampleItems], oy[kSampleItems], oz[kSampleItems];
#pragma unroll
    for (int j = 0; j < kSampleItems; ++j) {
        const uint64_t s = pcg_apply(jumps.row[j], state0);
        u[j] = pcg_float_of(s);
        ox[j] = pcg_float_of(pcg_apply(jumps.draw[0], s));
        oy[j] = pcg_float_of(pcg_apply(jumps.draw[1], s));
        oz[j] = pcg_float_of(pcg_apply(jumps.draw[2], s));
    }
    uint32_t first[kSampleItems], count[kSampleItems], node[kSampleItems];
#pragma unroll
    for (int j = 0; j < kSampleItems; ++j) {
        first[j] = 0u;
        count[j] = live[j] ? n_leaves : 0u;
        node[j] = 1u;
    }
    // the probes whose element lies in the tree (a finished search keeps its node and reads it again)
    if (n_leaves >= (4u << kTreeDepth)) {
        // no search ends inside the tree (every level leaves at least half of the elements minus one); a candidate
        // that does not exist goes left all the way with nothing to search
#pragma unroll
        for (int j = 0; j < kSampleItems; ++j) u[j] = live[j] ? u[j] : -1.0f;
#pragma unroll 1
        for (int level = 0; level < kTreeDepth; ++level) {
#pragma unroll
            for (int j = 0; j < kSampleItems; ++j) {
                const uint32_t step = count[j] >> 1;
                const bool right = s_tree[node[j]] < u[j];
                first[j] += right ? step + 1u : 0u;
                count[j] = right ? count[j] - (step + 1u) : step;
                node[j] = 2u * node[j] + (right ? 1u : 0u);
            }
        }
    } else {
#pragma unroll 1
        for (int level = 0; level < kTreeDepth; ++level) {
#pragma unroll
            for (int j = 0; j < kSampleItems; ++j) {
                const bool active = count[j] > 0u;
                const uint32_t step = count[j] >> 1;
                const bool right = s_tree[node[j]] < u[j];
                first[j] = active && right ? first[j] + step + 1u : first[j];
                count[j] = !active ? 0u : right ? count[j] - (step + 1u) : step;
                node[j] = active ? 2u * node[j] + (right ? 1u : 0u) : node[j];
            }
        }
    }
    // the levels of the tree below that are read from the head in memory, all eight searches level by level again
    const int levels = tree_levels(n_leaves);
#pragma unroll 1
    for (int level = kTreeDepth; level < levels; ++level) {
        float key[kSampleItems];
#pragma unroll
        for (int j = 0; j < kSampleItems; ++j) key[j] = head[node[j]];
#pragma unroll
        for (int j = 0; j < kSampleItems; ++j) {
            const bool active = count[j] > 0u;
            const uint32_t step = count[j] >> 1;
            const bool right = key[j] < u[j];
            first[j] = active && right ? first[j] + step + 1u : first[j];
            count[j] = !active ? 0u : right ? count[j] - (step + 1u) : step;
            node[j] = active ? 2u * node[j] + (right ? 1u : 0u) : node[j];
        }
    }
    // What is left of a search (at most kFetch elements, see tree_levels) reads the CDF itself. A probe is a load whose
    // 64 lanes read 64 different lines, and what it costs goes with the lines it looks up: so four neighbouring lanes
    // fetch the kFetch elements from the search's first one on, 16 bytes each (one or two lines per search instead of
    // one per probe and lane), compare them with the sample, and the search's own lane makes the remaining probes of
    // the reference's sequence on these sixteen outcomes. (The CDF is not monotone everywhere: where a chunk of the
    // blocked scan ends an element can be an ulp above the next one, so the probe sequence itself is kept.)
    // (Measured with 8,388,608 samples: -6 % for 131,072 leaves, -13 % for 262,144.)
    const bool wide = n_leaves >= kFetch;
#pragma unroll
    for (int j = 0; j < kSampleItems; ++j) {
        while (count[j] > (wide ? kFetch : 0u)) {
            const uint32_t step = count[j] >> 1;
            const uint32_t it = first[j] + step;
            if (cdf[it] < u[j]) {
                first[j] = it + 1u;
                count[j] -= step + 1u;
            } else {
                count[j] = step;
            }
        }
    }
    if (wide) {
        const uint32_t lane = lane_id(), group = lane >> 2, part = lane & 3u;
#pragma unroll
        for (int j = 0; j < kSampleItems; ++j) {
            uint32_t below = 0u;   // bit i: element base + i is below the sample
#pragma unroll
            for (uint32_t r = 0; r < 4u; ++r) {
                // this sub-round serves the searches of lanes 16 r .. 16 r + 15; the lane helps with that of `owner`
                const uint32_t owner = r * 16u + group;
                const uint32_t f = (uint32_t)__shfl((int)first[j], (int)owner, 64);
                const float sample = __shfl(u[j], (int)owner, 64);
                const uint32_t base = min(f, n_leaves - kFetch);   // the fetch stays inside the array
                float e[4];
                __builtin_memcpy(e, cdf + base + 4u * part, 16);   // 4-byte aligned
                uint32_t mine = 0u;
#pragma unroll
                for (uint32_t k = 0; k < 4u; ++k) mine |= (e[k] < sample ? 1u : 0u) << (4u * part + k);
                mine |= (uint32_t)__shfl_xor((int)mine, 1, 64);
                mine |= (uint32_t)__shfl_xor((int)mine, 2, 64);
                const uint32_t got = (uint32_t)__shfl((int)mine, (int)((lane & 15u) * 4u), 64);
                if ((lane >> 4) == r) below = got;
            }
            const uint32_t base = min(first[j], n_leaves - kFetch);
#pragma unroll
            for (int probe = 0; probe < 5; ++probe) {   // 16 elements: at most five probes
                const bool active = count[j] > 0u;
                const uint32_t step = count[j] >> 1;
                const uint32_t it = first[j] + step;
                const bool right = ((below >> ((it - base) & 31u)) & 1u) != 0u;
                first[j] = active && right ? it + 1u : first[j];
                count[j] = !active ? 0u : right ? count[j] - (step + 1u) : step;
            }
        }
    }
    float4 box[kSampleItems];
#pragma unroll
    for (int j = 0; j < kSampleItems; ++j) {
        c[j].leaf = min(first[j], n_leaves - 1u);
        box[j] = boxes[c[j].leaf];
    }
#pragma unroll
    for (int j = 0; j < kSampleItems; ++j) {
        c[j].x = box[j].x + (ox[j] - 0.5f) * box[j].w;
        c[j].y = box[j].y + (oy[j] - 0.5f) * box[j].w;
        c[j].z = box[j].z + (oz[j] - 0.5f) * box[j].w;
    }
}

// Generator of the first candidate of this thread: tile start (uniform jump) then 4*tid draws.
__device__ __forceinline__ Pcg32 thread_generator(const uint64_t* rng_dev, uint64_t first_candidate_of_block) {
    Pcg32 r{rng_dev[0], rng_dev[1]};
    r.state = pcg_apply(pcg_jump(r.inc, 4ull * first_candidate_of_block), r.state);
    r.state = pcg_apply(pcg_jump(r.inc, 4ull * threadIdx.x), r.state);
    return r;
}

__global__ void __launch_bounds__(kDrawBlock) k_sample(const float4* __restrict__ boxes, const float* __restrict__ cdf,
                                                   const float* __restrict__ sum_dev, float* __restrict__ positions,
                                                   int32_t* __restrict__ leaf_ids, uint32_t n_samples, uint32_t n_leaves,
                                                   const uint64_t* __restrict__ rng_dev) {
    __shared__ __align__(16) float s_tree[kTreeNodes];
    if (!(*sum_dev > 0.0f)) return;
    load_search_tree(s_tree, sum_dev);
    const uint64_t tile_first = (uint64_t)blockIdx.x * kDrawTile;
    const Pcg32 r = thread_generator(rng_dev, tile_first);
    const TileJumps jumps = make_tile_jumps(r.inc);
    bool live[kSampleItems];
#pragma unroll
    for (int j = 0; j < kSampleItems; ++j) live[j] = tile_first + (uint64_t)j * kDrawBlock + threadIdx.x < n_samples;
    Candidate c[kSampleItems];
    draw_candidates(r.state, jumps, live, boxes, cdf, sum_dev, s_tree, n_leaves, c);
#pragma unroll
    for (int j = 0; j < kSampleItems; ++j) {
        const uint64_t k = tile_first + (uint64_t)j * kDrawBlock + threadIdx.x;
        if (live[j]) {
            positions[3 * k] = c[j].x;
            positions[3 * k + 1] = c[j].y;
            positions[3 * k + 2] = c[j].z;
            if (leaf_ids) leaf_ids[k] = (int32_t)c[j].leaf;
        }
    }
}

// Advance the device generator by `mult * (*count_ptr or count)` draws, guarded by sum > 0.
__global__ void k_rng_advance(uint64_t* rng_dev, const float* sum_dev, uint64_t draws) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    if (sum_dev && !(*sum_dev > 0.0f)) return;
    rng_dev[0] = pcg_apply(pcg_jump(rng_dev[1], draws), rng_dev[0]);
}

// ---- training sampler round ---------------------------------------------------------------------------
struct CullState {
    uint32_t accepted;   // samples accepted so far in this draw (a lower bound once `consumed` is set)
    uint32_t consumed;   // candidates consumed when the capacity-th sample was accepted, else 0
    uint32_t error;      // look-back gave up
    uint32_t ticket;     // next tile of the round that is running (cleared with the round's status words)
    uint32_t pad[12];
};
constexpr size_t kCullHeaderWords = sizeof(CullState) / 4;
constexpr int kTileJumpBits = 20;   // a round has fewer than 2^20 tiles (candidate indices stay below 2^30)

// Id: the type the caller wants the leaf indices in (int32_t, or the int64_t of the Python API's tensors,
// B/sampling/src/sampling_api.cu:71: written here directly instead of widened by a pass of its own).
template <typename Id>
__global__ void __launch_bounds__(kDrawBlock)
    k_sample_cull(const float4* __restrict__ boxes, const float* __restrict__ cdf, const float* __restrict__ sum_dev,
                  const float* __restrict__ w2c, float* __restrict__ positions, Id* __restrict__ leaf_ids,
                  uint32_t capacity, uint32_t k0, uint32_t n_candidates, uint32_t n_blocks, uint32_t n_leaves, Camera cam,
                  const uint64_t* __restrict__ rng_dev, CullState* st, uint32_t* status) {
    __shared__ uint32_t s_accepted0, s_exclusive, s_done, s_bid;
    __shared__ PcgJump s_tile_jump[kTileJumpBits];   // generator step over 2^b tiles
    __shared__ uint32_t s_count[kSampleItems * (kDrawBlock / kWave)];
    __shared__ __align__(16) float s_tree[kTreeNodes];
    if (!(*sum_dev > 0.0f)) return;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    // `accepted` keeps its value from the rounds before until the last tile of this round has its total, and
    // that needs the count of every tile in front of it
    if (tid == 0) s_accepted0 = __hip_atomic_load(&st->accepted, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    load_search_tree(s_tree, sum_dev);
    const Rows m = load_rows(w2c);
    // The generator of a thread's first candidate of a tile = the tile's (start of the draw + 4 * first candidate of
    // the tile) advanced by 4 * tid draws. The O(log) jumps are made once: by 4 * tid, from a candidate to the
    // thread's j-th one of a tile, and from a tile of this block to its next one; per tile a few multiply-adds are left.
    const uint64_t rng_inc = rng_dev[1];
    const PcgJump jump_thread = pcg_jump(rng_inc, 4ull * tid);
    const TileJumps jumps = make_tile_jumps(rng_inc);
    if (tid < (uint32_t)kTileJumpBits) s_tile_jump[tid] = pcg_jump(rng_inc, (4ull * kDrawTile) << tid);
    uint64_t tile_state = pcg_apply(pcg_jump(rng_inc, 4ull * (uint64_t)k0), rng_dev[0]);   // of tile `at`
    uint32_t at = 0;
    // A block takes its tiles from a ticket counter, in order: a tile waits (look-back) only for tiles in front of
    // it, and each of those was taken by a block that was running then. Nothing ever waits for a block that has
    // not started, whatever else occupies the GPU.
    for (;;) {
        if (tid == 0) s_bid = atomicAdd(&st->ticket, 1u);
        __syncthreads();   // also: s_tile_jump is complete
        const uint32_t bid = s_bid;
        if (bid >= n_blocks) break;
        for (uint32_t step = bid - at, b = 0; step != 0u; step >>= 1, ++b)
            if (step & 1u) tile_state = pcg_apply(s_tile_jump[b], tile_state);
        at = bid;
        const uint64_t state0 = pcg_apply(jump_thread, tile_state);
        if (tid == 0) {
            const uint32_t done = __hip_atomic_load(&st->consumed, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u;
            s_done = done;
            if (done) {
                // The draw is already complete: tell later tiles that everything is taken.
                status_store(status + bid, kFlagInclusive | min(capacity, kValueMask));
                if (bid == n_blocks - 1) st->accepted = max(s_accepted0, capacity);
            }
        }
        __syncthreads();
        if (s_done) {   // uniform
            __syncthreads();   // s_done is rewritten by the next tile
            continue;
        }
        const uint64_t tile_first = (uint64_t)bid * kDrawTile;  // relative to k0

        Candidate cand[kSampleItems];
        uint32_t rank[kSampleItems];
        bool keep[kSampleItems];
#pragma unroll
        for (int j = 0; j < kSampleItems; ++j) keep[j] = tile_first + (uint64_t)j * kDrawBlock + tid < n_candidates;
        draw_candidates(state0, jumps, keep, boxes, cdf, sum_dev, s_tree, n_leaves, cand);
#pragma unroll
        for (int j = 0; j < kSampleItems; ++j) {
            keep[j] = keep[j] && sample_accepted(m, cand[j].x, cand[j].y, cand[j].z, cam);
            const uint64_t ballot = __ballot(keep[j]);
            rank[j] = mask_rank(ballot);
            if (lane == 0) s_count[j * (kDrawBlock / kWave) + wave] = (uint32_t)__popcll(ballot);
        }
        __syncthreads();
        if (wave == 0) {
            // exclusive scan of the 32 (round, wave) counts by the first lanes, then the block-level look-back
            uint32_t c = lane < (uint32_t)(kSampleItems * (kDrawBlock / kWave)) ? s_count[lane] : 0u;
            uint32_t incl = c;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const uint32_t up = __shfl_up(incl, d, 64);
                if (lane >= (uint32_t)d) incl += up;
            }
            if (lane < (uint32_t)(kSampleItems * (kDrawBlock / kWave))) s_count[lane] = incl - c;
            const uint32_t run = __shfl(incl, 63, 64);
            const uint32_t exclusive = lookback_exclusive_wave(status, bid, run, &st->error);
            if (lane == 0) {
                s_exclusive = exclusive;
                if (bid == n_blocks - 1) st->accepted = s_accepted0 + exclusive + run;
            }
        }
        __syncthreads();
        const uint64_t base = (uint64_t)s_accepted0 + s_exclusive;
#pragma unroll
        for (int j = 0; j < kSampleItems; ++j) {
            if (!keep[j]) continue;
            const uint64_t slot = base + s_count[j * (kDrawBlock / kWave) + wave] + rank[j];
            if (slot >= capacity) continue;
            positions[3 * slot] = cand[j].x;
            positions[3 * slot + 1] = cand[j].y;
            positions[3 * slot + 2] = cand[j].z;
            leaf_ids[slot] = (Id)cand[j].leaf;
            if (slot + 1 == capacity) {
                const uint64_t rel = tile_first + (uint64_t)j * kDrawBlock + tid;
                __hip_atomic_store(&st->consumed, (uint32_t)(k0 + rel + 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        __syncthreads();   // s_count, s_exclusive, s_done and s_bid are reused by the next tile
    }
}

// Clears the status words of a round; the first round of a draw (k0 = 0) clears the whole state in front of them too.
__global__ void k_cull_round_reset(uint32_t* status, uint32_t n_blocks, CullState* st, bool new_draw) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n_blocks) status[i] = 0u;
    if (new_draw && i < (uint32_t)kCullHeaderWords) ((uint32_t*)st)[i] = 0u;
    if (!new_draw && i == 0) st->ticket = 0u;
}

// End of a draw. A positive weight sum: the generator moves on by four draws per consumed candidate. Otherwise: the
// failure pattern of B/sampling/src/sampling.cu:107-111 in the outputs (a small grid, so that the usual case costs
// next to nothing) and the generator stays where it is.
template <typename Id>
__global__ void __launch_bounds__(kBlock) k_cull_finish(const float* __restrict__ sum_dev, uint64_t* rng_dev,
                                                        const CullState* st, float* positions, Id* leaf_ids,
                                                        uint32_t capacity, uint32_t total_candidates) {
    if (*sum_dev > 0.0f) {
        if (blockIdx.x == 0 && threadIdx.x == 0) {
            const uint32_t consumed = st->consumed != 0u ? st->consumed : total_candidates;
            // INPC_CULL_IF_COMPLETE: a draw that has not reached its capacity is left as it is
            if (consumed != INPC_CULL_IF_COMPLETE)
                rng_dev[0] = pcg_apply(pcg_jump(rng_dev[1], 4ull * consumed), rng_dev[0]);
        }
        return;
    }
    if (!positions || !leaf_ids) return;
    const uint32_t stride = gridDim.x * kBlock;
    for (uint32_t i = blockIdx.x * kBlock + threadIdx.x; i < capacity; i += stride) {
        positions[3 * (size_t)i] = 0.0f;
        positions[3 * (size_t)i + 1] = 0.0f;
        positions[3 * (size_t)i + 2] = 0.0f;
        leaf_ids[i] = (Id)-1;
    }
}

__global__ void __launch_bounds__(kBlock) k_widen_ids(const int32_t* __restrict__ ids, int64_t* __restrict__ out,
                                                      uint32_t n) {
    const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
    if (i < n) out[i] = (int64_t)ids[i];
}

// ---- expected-count sampler -------------------------------------------------------------------------
constexpr int kCountItems = 4;
constexpr int kCountTile = kBlock * kCountItems;

struct ScanState {
    uint32_t ticket;
    uint32_t error;
    uint32_t pad[14];
};
constexpr size_t kScanHeaderWords = sizeof(ScanState) / 4;

// Block-wide exclusive scan of one value per thread (256 threads); returns the block total in `total`.
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t v, uint32_t* s_wave /*4*/, uint32_t& total) {
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    uint32_t incl = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const uint32_t up = __shfl_up(incl, d, 64);
        if (lane >= (uint32_t)d) incl += up;
    }
    if (lane == 63) s_wave[wave] = incl;
    __syncthreads();
    uint32_t wave_base = 0, t = 0;
#pragma unroll
    for (int w = 0; w < kBlock / kWave; ++w) {
        const uint32_t c = s_wave[w];
        if ((uint32_t)w < wave) wave_base += c;
        t += c;
    }
    total = t;
    __syncthreads();
    return wave_base + incl - v;
}

// counts + inclusive integer scan in one pass (thread owns 4 consecutive leaves). The sum of the weights is what
// k_tile_totals left, added up by every block itself (64 values for 262,144 leaves: less than a launch costs);
// *sum_out receives it. A sum that is not positive leaves all offsets at zero.
__global__ void __launch_bounds__(kBlock)
    k_expected_counts(const float* __restrict__ weights, const float* __restrict__ raw_tile_totals, uint32_t n_tiles,
                      float* __restrict__ sum_out, int32_t* __restrict__ offsets, uint32_t n_samples, uint32_t n_leaves,
                      ScanState* st, uint32_t* status) {
    __shared__ float s_a[kMaxUpperValues / kChunk];
    __shared__ float s_b[kChunk];
    __shared__ float s_sum;
    __shared__ uint32_t s_bid, s_exclusive;
    __shared__ uint32_t s_wave[kBlock / kWave];
    if (threadIdx.x < (uint32_t)kWave) {
        upper_totals(raw_tile_totals, n_tiles, s_a, s_b, threadIdx.x);
        const float total = blocked_total(n_tiles, s_b);
        if (threadIdx.x == 0) s_sum = total;
    }
    __syncthreads();
    const float sum = s_sum;
    if (blockIdx.x == 0 && threadIdx.x == 0) *sum_out = sum;
    if (!(sum > 0.0f)) {
        for (int j = 0; j < kCountItems; ++j) {
            const size_t l = (size_t)blockIdx.x * kCountTile + (size_t)j * kBlock + threadIdx.x;
            if (l < n_leaves) offsets[l] = 0;
        }
        return;
    }
    if (threadIdx.x == 0) s_bid = atomicAdd(&st->ticket, 1u);
    __syncthreads();
    const uint32_t bid = s_bid;
    const size_t first = (size_t)bid * kCountTile + (size_t)threadIdx.x * kCountItems;
    const float norm = 1.0f / sum;
    uint32_t count[kCountItems];
    uint32_t mine = 0;
#pragma unroll
    for (int j = 0; j < kCountItems; ++j) {
        count[j] = 0;
        const size_t l = first + j;
        if (l < n_leaves) {
            const float w = weights[l];
            if (w > 0.0f) count[j] = (uint32_t)max(__float2int_rn(w * norm * (float)n_samples), 1);
        }
        mine += count[j];
    }
    uint32_t total;
    const uint32_t local = block_exclusive_scan(mine, s_wave, total);
    if (threadIdx.x < 64) {
        const uint32_t exclusive = lookback_exclusive_wave(status, bid, total, &st->error);
        if (threadIdx.x == 0) s_exclusive = exclusive;
    }
    __syncthreads();
    uint32_t run = s_exclusive + local;
#pragma unroll
    for (int j = 0; j < kCountItems; ++j) {
        const size_t l = first + j;
        run += count[j];
        if (l < n_leaves) offsets[l] = (int32_t)run;
    }
}

// ids[offsets[l-1] .. offsets[l]) = l; one wave per 64 leaves, lanes stride over each leaf's run. The wave fetches its
// 64 offsets with one load and hands them round (two dependent loads per leaf made the walk a chain of 128 round trips).
__global__ void __launch_bounds__(kBlock) k_repeat_interleave(const int32_t* __restrict__ offsets,
                                                              int32_t* __restrict__ ids, uint32_t n_leaves) {
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave_global = (blockIdx.x * kBlock + threadIdx.x) >> 6;
    const uint32_t l0 = wave_global * 64u;
    if (l0 >= n_leaves) return;   // the whole wave
    const uint32_t n_here = min(64u, n_leaves - l0);
    const int32_t mine = offsets[min(l0 + lane, n_leaves - 1u)];
    const int32_t front = l0 == 0u ? 0 : offsets[l0 - 1u];
    int32_t b = front;
    for (uint32_t k = 0; k < n_here; ++k) {
        const int32_t e = __shfl(mine, (int)k, 64);
        for (int32_t i = b + (int32_t)lane; i < e; i += 64) ids[i] = (int32_t)(l0 + k);
        b = e;
    }
}

__global__ void __launch_bounds__(kBlock)
    k_expected_samples(const float* __restrict__ centers, const int32_t* __restrict__ levels,
                       const int32_t* __restrict__ ids, float* __restrict__ positions, uint32_t n_total,
                       uint32_t n_created, float initial_size, const uint64_t* __restrict__ rng_dev) {
    const uint64_t tile_first = (uint64_t)blockIdx.x * kSampleTile;
    Pcg32 r{rng_dev[0], rng_dev[1]};
    r.state = pcg_apply(pcg_jump(r.inc, 3ull * tile_first), r.state);
    r.state = pcg_apply(pcg_jump(r.inc, 3ull * threadIdx.x), r.state);
    const PcgJump step = pcg_jump(r.inc, 3ull * kBlock - 3ull);
    for (int j = 0; j < kSampleItems; ++j) {
        const uint64_t s = tile_first + (uint64_t)j * kBlock + threadIdx.x;
        if (s < n_total) {
            const int32_t leaf = ids[s % n_created];
            const float ox = pcg_float(r), oy = pcg_float(r), oz = pcg_float(r);
            const float scale = ldexpf(1.0f, -levels[leaf]) * initial_size;
            positions[3 * s] = centers[3 * (size_t)leaf] + (ox - 0.5f) * scale;
            positions[3 * s + 1] = centers[3 * (size_t)leaf + 1] + (oy - 0.5f) * scale;
            positions[3 * s + 2] = centers[3 * (size_t)leaf + 2] + (oz - 0.5f) * scale;
            r.state = pcg_apply(step, r.state);
        }
    }
}

// Scratch of the CDF passes for n leaves, in floats: the raw tile totals, the tile totals of the normalised weights
// (each padded to whole chunks: the kernels fetch whole chunks) and the scanned chunk totals.
struct CdfScratch {
    uint32_t n_tiles;
    size_t raw_tile_totals, tile_totals, scanned_chunk_totals;   // offsets in floats
    size_t total_floats;
};

CdfScratch plan_cdf(uint32_t n) {
    CdfScratch p{};
    p.n_tiles = div_up(n, kChunkTile);
    p.raw_tile_totals = 0;
    p.tile_totals = align_up(p.n_tiles, kChunk);
    p.scanned_chunk_totals = 2 * align_up(p.n_tiles, kChunk);
    p.total_floats = p.scanned_chunk_totals + (size_t)p.n_tiles * kChunksPerBlock;
    return p;
}

// Sum, normalisation and inclusive scan of the n leaf weights in place; the head of the CDF into sum_out.
// `scratch` holds plan_cdf(n).total_floats floats; every element that is read has been written by an earlier launch
// of the same call (or is not used), so it needs no clearing.
int launch_build_cdf(float* w, float* sum_out, float* scratch, uint32_t n_leaves, hipStream_t stream) {
    const CdfScratch plan = plan_cdf(n_leaves);
    const int levels = tree_levels(n_leaves);
    const uint32_t n_nodes = 1u << levels;
    float* raw = scratch + plan.raw_tile_totals;
    float* tile_totals = scratch + plan.tile_totals;
    float* scanned = scratch + plan.scanned_chunk_totals;
    INPC_LAUNCH("cdf_tile_totals", k_tile_totals, dim3(plan.n_tiles), dim3(kWave), stream, (const float*)w, n_leaves, raw,
                sum_out + 1, n_nodes - 1u);
    INPC_LAUNCH("cdf_scan_tiles", k_cdf_scan_tiles, dim3(plan.n_tiles), dim3(kWave), stream, w, n_leaves,
                (const float*)raw, scanned, tile_totals, sum_out);
    INPC_LAUNCH("cdf_finish", k_cdf_finish, dim3(div_up(n_leaves, kFinishTile)), dim3(kBlock), stream, w, n_leaves,
                (const float*)scanned, (const float*)tile_totals, plan.n_tiles, sum_out, levels);
    return INPC_OK;
}

// ---- built-in scratch of inpc_build_cdf_static ------------------------------------------------------------------
// Scratch of the CDF passes for up to INPC_BUILD_CDF_STATIC_MAX_LEAVES leaves (1024 tiles: two arrays of 1024 tile
// totals and 65536 scanned chunk totals). The
// array's name is only a handle in host code: the address kernels can use comes from hipGetSymbolAddress,
// once per device (every device holds its own copy).
constexpr size_t kStaticTotalsFloats = 65536 + 1024 + 1024;
__device__ __align__(256) float g_static_totals[kStaticTotalsFloats];

constexpr int kMaxDevices = 64;
std::mutex g_static_mutex;
float* g_static_totals_ptr[kMaxDevices] = {};

int static_totals(float*& out) {
    int device = 0;
    INPC_HIP_CHECK(hipGetDevice(&device));
    if (device < 0 || device >= kMaxDevices) return fail(INPC_E_UNSUPPORTED, "device index %d out of range", device);
    std::lock_guard<std::mutex> lock(g_static_mutex);
    if (!g_static_totals_ptr[device]) {
        void* p = nullptr;
        INPC_HIP_CHECK(hipGetSymbolAddress(&p, HIP_SYMBOL(g_static_totals)));
        if (!p) return fail(INPC_E_HIP, "hipGetSymbolAddress returned a null address for the built-in scratch");
        g_static_totals_ptr[device] = (float*)p;
    }
    out = g_static_totals_ptr[device];
    return INPC_OK;
}

}  // namespace

// Floats at the start of the workspace: the CDF passes and the expected-count sampler's sum share them.
size_t sampler_scratch_floats(uint32_t n_leaves) { return plan_cdf(std::max(n_leaves, 1u)).total_floats; }

size_t sampler_workspace_bytes(uint32_t n_leaves) {
    const size_t floats = sampler_scratch_floats(n_leaves);
    const uint32_t scan_blocks = div_up(std::max(n_leaves, 1u), kCountTile);
    return align_up(floats * 4, 256) + align_up((kScanHeaderWords + scan_blocks) * 4, 256) + 256;
}

}  // namespace inpc

using namespace inpc;

extern "C" {

int inpc_leaf_weights(const float* centers, const int32_t* levels, const float* weights, const float* w2c,
                      float* out, float* boxes_out, uint32_t n_leaves, const inpc_camera* cam, float initial_size,
                      void* stream) {
    if (!cam) return fail(INPC_E_INVALID_ARGUMENT, "inpc_leaf_weights: camera is null");
    if (n_leaves == 0) return INPC_OK;
    if (!centers || !levels || !weights || !w2c || !out)
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_leaf_weights: null pointer");
    if (((uintptr_t)boxes_out & 15u) != 0)
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_leaf_weights: boxes_out must be 16-byte aligned");
    INPC_LAUNCH("leaf_weights", k_leaf_weights, dim3(div_up(n_leaves, kBlock)), dim3(kBlock), (hipStream_t)stream,
                centers, levels, weights, w2c, out, (float4*)boxes_out, n_leaves, to_device_camera(*cam), initial_size);
    return INPC_OK;
}

size_t inpc_sampler_workspace_bytes(uint32_t n_leaves) { return sampler_workspace_bytes(n_leaves); }

size_t inpc_cdf_head_floats(uint32_t n_leaves) { return (size_t)1 << tree_levels(n_leaves); }

// The head of a CDF for n_leaves leaves holds inpc_cdf_head_floats(n_leaves) floats: the kernels write and read that many.
static int check_head(const char* who, size_t head_floats, uint32_t n_leaves) {
    const size_t need = (size_t)1 << tree_levels(n_leaves);
    if (head_floats < need)
        return fail(INPC_E_WORKSPACE, "%s: the CDF head has %zu floats, %u leaves need %zu (inpc_cdf_head_floats)", who,
                    head_floats, n_leaves, need);
    return INPC_OK;
}

int inpc_build_cdf(float* w, float* sum_out, size_t head_floats, void* workspace, size_t workspace_bytes,
                   uint32_t n_leaves, void* stream_) {
    if (n_leaves == 0) return fail(INPC_E_INVALID_ARGUMENT, "inpc_build_cdf: no leaves");
    if (!w || !sum_out || !workspace) return fail(INPC_E_INVALID_ARGUMENT, "inpc_build_cdf: null pointer");
    if (n_leaves > kMaxCdfLeaves)
        return fail(INPC_E_UNSUPPORTED, "inpc_build_cdf: %u leaves exceed the %u the scan's levels hold", n_leaves,
                    kMaxCdfLeaves);
    if (const int rc = check_head("inpc_build_cdf", head_floats, n_leaves); rc != INPC_OK) return rc;
    if (workspace_bytes < sampler_workspace_bytes(n_leaves))
        return fail(INPC_E_WORKSPACE, "inpc_build_cdf: workspace has %zu bytes, needs %zu", workspace_bytes,
                    sampler_workspace_bytes(n_leaves));
    return launch_build_cdf(w, sum_out, (float*)workspace, n_leaves, (hipStream_t)stream_);
}

int inpc_build_cdf_static(float* w, float* sum_out, size_t head_floats, uint32_t n_leaves, void* stream_) {
    if (n_leaves == 0) return fail(INPC_E_INVALID_ARGUMENT, "inpc_build_cdf_static: no leaves");
    if (!w || !sum_out) return fail(INPC_E_INVALID_ARGUMENT, "inpc_build_cdf_static: null pointer");
    if (n_leaves > INPC_BUILD_CDF_STATIC_MAX_LEAVES)
        return fail(INPC_E_UNSUPPORTED, "inpc_build_cdf_static: %u leaves exceed the %u the built-in scratch holds",
                    n_leaves, (unsigned)INPC_BUILD_CDF_STATIC_MAX_LEAVES);
    if (plan_cdf(n_leaves).total_floats > kStaticTotalsFloats)
        return fail(INPC_E_UNSUPPORTED, "inpc_build_cdf_static: the built-in scratch is too small for %u leaves", n_leaves);
    if (const int rc = check_head("inpc_build_cdf_static", head_floats, n_leaves); rc != INPC_OK) return rc;
    float* totals = nullptr;
    const int rc = static_totals(totals);
    if (rc != INPC_OK) return rc;
    return launch_build_cdf(w, sum_out, totals, n_leaves, (hipStream_t)stream_);
}

int inpc_sample(const float* boxes, const float* cdf, const float* sum_dev, size_t head_floats, float* positions_out,
                int32_t* leaf_ids_out, uint32_t n_samples, uint32_t n_leaves, uint64_t* rng_dev, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    if (n_samples == 0) return INPC_OK;
    if (n_samples >= (1u << 30)) return fail(INPC_E_UNSUPPORTED, "inpc_sample: n_samples must be below 2^30");
    if (n_leaves == 0 || !boxes || !cdf || !sum_dev || !positions_out || !rng_dev)
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_sample: null pointer or no leaves");
    if (((uintptr_t)boxes & 15u) != 0) return fail(INPC_E_INVALID_ARGUMENT, "inpc_sample: boxes must be 16-byte aligned");
    if (const int rc = check_head("inpc_sample", head_floats, n_leaves); rc != INPC_OK) return rc;
    INPC_LAUNCH("sample", k_sample, dim3(div_up(n_samples, kDrawTile)), dim3(kDrawBlock), stream, (const float4*)boxes, cdf,
                sum_dev, positions_out, leaf_ids_out, n_samples, n_leaves, (const uint64_t*)rng_dev);
    INPC_LAUNCH("rng_advance", k_rng_advance, dim3(1), dim3(64), stream, rng_dev, sum_dev, 4ull * n_samples);
    return INPC_OK;
}

size_t inpc_cull_workspace_bytes(uint32_t n_candidates) {
    return align_up((kCullHeaderWords + div_up(std::max(n_candidates, 1u), kDrawTile)) * 4, 256);
}

int inpc_cull_begin(void* workspace, size_t workspace_bytes, void* stream) {
    if (!workspace || workspace_bytes < sizeof(CullState))
        return fail(INPC_E_WORKSPACE, "inpc_cull_begin: workspace too small");
    return fill_u32(workspace, 0u, kCullHeaderWords, (hipStream_t)stream);
}

int inpc_sample_cull_compact(const float* boxes, const float* cdf, const float* sum_dev, size_t head_floats,
                             const float* w2c, float* positions_out, void* leaf_ids_out, int ids_int64, uint32_t capacity,
                             uint32_t k0, uint32_t n_candidates, uint32_t n_leaves, const inpc_camera* cam,
                             const uint64_t* rng_dev, void* workspace, size_t workspace_bytes, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    if (n_candidates == 0) {   // nothing to draw; a new draw still starts from a cleared state
        if (k0 == 0u && workspace && workspace_bytes >= sizeof(CullState))
            return fill_u32(workspace, 0u, kCullHeaderWords, stream);
        return INPC_OK;
    }
    if (!cam || n_leaves == 0 || !boxes || !cdf || !sum_dev || !w2c || !positions_out || !leaf_ids_out || !rng_dev ||
        !workspace)
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_sample_cull_compact: null pointer or no leaves");
    if (((uintptr_t)boxes & 15u) != 0)
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_sample_cull_compact: boxes must be 16-byte aligned");
    if ((uint64_t)k0 + n_candidates >= (1ull << 30))
        return fail(INPC_E_UNSUPPORTED, "inpc_sample_cull_compact: candidate index must stay below 2^30");
    if (const int rc = check_head("inpc_sample_cull_compact", head_floats, n_leaves); rc != INPC_OK) return rc;
    if (workspace_bytes < inpc_cull_workspace_bytes(n_candidates))
        return fail(INPC_E_WORKSPACE, "inpc_sample_cull_compact: workspace has %zu bytes, needs %zu", workspace_bytes,
                    inpc_cull_workspace_bytes(n_candidates));
    CullState* st = (CullState*)workspace;
    uint32_t* status = (uint32_t*)workspace + kCullHeaderWords;
    const uint32_t n_blocks = div_up(n_candidates, kDrawTile);
    INPC_LAUNCH("cull_round_reset", k_cull_round_reset, dim3(div_up(std::max(n_blocks, (uint32_t)kCullHeaderWords), kBlock)),
                dim3(kBlock), stream, status, n_blocks, st, k0 == 0u);
    // as many blocks as the GPU holds at once; each takes tiles until none is left
    uint32_t resident = 0;
    const int rc = resident_blocks(ids_int64 ? (const void*)k_sample_cull<int64_t> : (const void*)k_sample_cull<int32_t>,
                                   kDrawBlock, resident);
    if (rc != INPC_OK) return rc;
    if (ids_int64) {
        INPC_LAUNCH("sample_cull_compact", k_sample_cull<int64_t>, dim3(std::min(n_blocks, resident)), dim3(kDrawBlock),
                    stream, (const float4*)boxes, cdf, sum_dev, w2c, positions_out, (int64_t*)leaf_ids_out, capacity, k0,
                    n_candidates, n_blocks, n_leaves, to_device_camera(*cam), rng_dev, st, status);
    } else {
        INPC_LAUNCH("sample_cull_compact", k_sample_cull<int32_t>, dim3(std::min(n_blocks, resident)), dim3(kDrawBlock),
                    stream, (const float4*)boxes, cdf, sum_dev, w2c, positions_out, (int32_t*)leaf_ids_out, capacity, k0,
                    n_candidates, n_blocks, n_leaves, to_device_camera(*cam), rng_dev, st, status);
    }
    return INPC_OK;
}

int inpc_cull_read_counts(const void* workspace, uint32_t* accepted_host, uint32_t* consumed_host, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    uint32_t host[3] = {0, 0, 0};
    INPC_HIP_CHECK(hipMemcpyAsync(host, workspace, sizeof(host), hipMemcpyDeviceToHost, stream));
    INPC_HIP_CHECK(hipStreamSynchronize(stream));
    if (accepted_host) *accepted_host = host[0];
    if (consumed_host) *consumed_host = host[1];
    if (host[2]) return fail(INPC_E_DEVICE, "sampler look-back gave up waiting (device error flag set)");
    return INPC_OK;
}

int inpc_cull_finish(const float* sum_dev, float* positions_out, void* leaf_ids_out, int ids_int64, uint32_t capacity,
                     uint32_t total_candidates, uint64_t* rng_dev, void* workspace, size_t workspace_bytes,
                     void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    if (!sum_dev || !rng_dev || !workspace || workspace_bytes < sizeof(CullState))
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_cull_finish: null pointer");
    const dim3 grid(std::max(std::min(div_up(capacity, kBlock), 1024u), 1u));
    if (ids_int64) {
        INPC_LAUNCH("cull_finish", k_cull_finish<int64_t>, grid, dim3(kBlock), stream, sum_dev, rng_dev,
                    (const CullState*)workspace, positions_out, (int64_t*)leaf_ids_out, capacity, total_candidates);
    } else {
        INPC_LAUNCH("cull_finish", k_cull_finish<int32_t>, grid, dim3(kBlock), stream, sum_dev, rng_dev,
                    (const CullState*)workspace, positions_out, (int32_t*)leaf_ids_out, capacity, total_candidates);
    }
    return INPC_OK;
}

int inpc_widen_ids(const int32_t* ids, int64_t* out, uint32_t n, void* stream) {
    if (n == 0) return INPC_OK;
    INPC_LAUNCH("widen_ids", k_widen_ids, dim3(div_up(n, kBlock)), dim3(kBlock), (hipStream_t)stream, ids, out, n);
    return INPC_OK;
}

int inpc_expected_counts(const float* weights, float* sum_out, int32_t* offsets_out, uint32_t n_samples,
                         void* workspace, size_t workspace_bytes, uint32_t n_leaves, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    if (n_leaves == 0 || !weights || !sum_out || !offsets_out || !workspace)
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_expected_counts: null pointer or no leaves");
    if (n_leaves > kMaxCdfLeaves)
        return fail(INPC_E_UNSUPPORTED, "inpc_expected_counts: %u leaves exceed the %u the sum's levels hold", n_leaves,
                    kMaxCdfLeaves);
    if (workspace_bytes < sampler_workspace_bytes(n_leaves))
        return fail(INPC_E_WORKSPACE, "inpc_expected_counts: workspace too small");
    const CdfScratch plan = plan_cdf(n_leaves);
    float* raw = (float*)workspace + plan.raw_tile_totals;
    uint32_t* scan = (uint32_t*)((char*)workspace + align_up(plan.total_floats * 4, 256));
    const uint32_t n_blocks = div_up(n_leaves, kCountTile);
    // the tile totals of the weights, and the state of the scan cleared on the way
    INPC_LAUNCH("tile_totals", k_tile_totals, dim3(plan.n_tiles), dim3(kWave), stream, weights, n_leaves, raw,
                (float*)scan, (uint32_t)kScanHeaderWords + n_blocks);
    INPC_LAUNCH("expected_counts", k_expected_counts, dim3(n_blocks), dim3(kBlock), stream, weights, (const float*)raw,
                plan.n_tiles, sum_out, offsets_out, n_samples, n_leaves, (ScanState*)scan, scan + kScanHeaderWords);
    return INPC_OK;
}

int inpc_expected_samples(const float* centers, const int32_t* levels, const int32_t* offsets,
                          int32_t* leaf_ids_scratch, float* positions_out, uint32_t n_created, uint32_t n_multi,
                          uint32_t n_leaves, float initial_size, uint64_t* rng_dev, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    const uint64_t total64 = (uint64_t)n_created * n_multi;
    if (total64 == 0) return INPC_OK;
    if (total64 >= (1ull << 30)) return fail(INPC_E_UNSUPPORTED, "inpc_expected_samples: too many samples");
    if (!centers || !levels || !offsets || !leaf_ids_scratch || !positions_out || !rng_dev)
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_expected_samples: null pointer");
    const uint32_t n_total = (uint32_t)total64;
    INPC_LAUNCH("repeat_interleave", k_repeat_interleave, dim3(div_up(div_up(n_leaves, 64u) * 64u, kBlock)),
                dim3(kBlock), stream, offsets, leaf_ids_scratch, n_leaves);
    INPC_LAUNCH("expected_samples", k_expected_samples, dim3(div_up(n_total, kSampleTile)), dim3(kBlock), stream,
                centers, levels, (const int32_t*)leaf_ids_scratch, positions_out, n_total, n_created, initial_size,
                (const uint64_t*)rng_dev);
    INPC_LAUNCH("rng_advance", k_rng_advance, dim3(1), dim3(64), stream, rng_dev, (const float*)nullptr,
                3ull * n_total);
    return INPC_OK;
}

}  // extern "C"
