// raster.hip — tile-based differentiable bilinear point rasterizer for gfx950.
//
// Pipeline (on the caller's stream but for k_records; counts stay on the device):
//   k_bin_count      project every point; per chunk of points count the instances (point, touched tile) per tile
//   k_bin_offsets    per tile: exclusive prefix of the counts over the chunks
//   k_bin_scan       exclusive scan over the tiles: [begin, end) of every tile's instances
//                    (B/rasterization/src/bilinear/kernels.cu:222-239); decides whether they fit the buffers
//                    and the schedule of the per-tile blocks: tiles with the longest instance lists first
//   k_bin_fill       project, cull, tile bounds, depth key: a (depth key, point) pair per instance into the bin of
//                    its tile (kernels.cu:11-84,198-220)
//   k_records        (on a second stream, beside the tile sort) the blend record of a drawn point:
//                    footprint weights, opacity, view features, at the point's place in the record array
//                    (kernels.cu:11-84,106-184)
//   tilesort.hpp     one block per tile sorts its bin by (depth key, point index) inside LDS: the order the
//                    reference gets from its two device-wide sorts (forward.cu:91-141)
//   blend.hpp        k_blend_forward: front-to-back bilinear 2x2 splat blend, one block per tile
//                    (kernels.cu:241-313,422-495); k_blend_backward: replay of the blend with the saved
//                    final image (kernels.cu:315-420)
//   k_sh_backward    view-space feature gradient -> 36 fp16 SH coefficient gradients
//                    (kernels.cu:86-104, sh_utils.cuh:44-62)
#include <algorithm>
#include <atomic>
#include <chrono>
#include <cmath>
#include <random>
#include <cstring>
#include <type_traits>

#include "common.hpp"

#include <hip/hip_fp16.h>

namespace inpc {

namespace {

constexpr int kBlock = 256;
constexpr float kTransmittanceThreshold = 1e-4f;  // bilinear/config.h:16
constexpr float kOneMinusAlphaEps = 1e-8f;        // bilinear/config.h:17

// counters (u32) at the head of the workspace
enum Counter : int {
    kCntVisible = 0,
    kCntInstances = 1,
    kCntError = 2,
    kCntSplit = 3,         // drawn points that touch more than one tile
    kCntKept = 4,          // Gaussian footprint: instances that are sorted and drawn (0 when they do not fit)
    kCntOverflow = 5,      // the instances (or the gradient rows) do not fit the buffers: nothing is drawn
    kCntInstances64 = 6,   // Gaussian footprint: u64 at words 6, 7: exact instance count
    kCntMulti = 8,         // Gaussian footprint: drawn points that touch more than one tile
    kCntRows = 10,         // instances of the points that touch more than one tile
    kCntWords = 16
};

#include "geometry.hpp"

inline uint32_t record_stride(int channels, bool half_features) {
    return (uint32_t)align_up(kRecordHeader + (size_t)channels * (half_features ? 2 : 4), 32);
}


// ---- SH degree 2 (sh_utils.cuh:6-23) ---------------------------------------------------------------------
struct ShBasis {
    float b[9];
};

__device__ __forceinline__ ShBasis sh_basis(float px, float py, float pz, const float* __restrict__ cam) {
    const float dx = px - cam[0], dy = py - cam[1], dz = pz - cam[2];
    const float inv = rsqrtf((dx * dx + dy * dy) + dz * dz);
    const float x = dx * inv, y = dy * inv, z = dz * inv;
    ShBasis s;
    s.b[0] = 0.28209479177387814f;
    s.b[1] = -0.48860251190291987f * y;
    s.b[2] = 0.48860251190291987f * z;
    s.b[3] = -0.48860251190291987f * x;
    s.b[4] = 1.0925484305920792f * (x * y);
    s.b[5] = -1.0925484305920792f * (y * z);
    s.b[6] = 0.94617469575755997f * (z * z) - 0.31539156525251999f;
    s.b[7] = -1.0925484305920792f * (x * z);
    s.b[8] = 0.54627421529603959f * (x * x) - 0.54627421529603959f * (y * y);
    return s;
}

__device__ __forceinline__ float4 sh_to_view(const ShBasis& s, const __half* __restrict__ coeffs) {
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k = 0; k < 9; ++k) {
#pragma unroll
        for (int ch = 0; ch < 4; ++ch) {
            const float f = __half2float(coeffs[4 * k + ch]);
            acc[ch] = k == 0 ? s.b[0] * f : acc[ch] + s.b[k] * f;
        }
    }
    return make_float4(acc[0], acc[1], acc[2], acc[3]);
}

// The same for 36 coefficients that start on an 8-byte boundary: nine 8-byte loads (word k = the four channels of
// coefficient k) instead of 36 two-byte ones.
__device__ __forceinline__ float4 sh_to_view_aligned(const ShBasis& s, const __half* __restrict__ coeffs) {
    const uint2* src = (const uint2*)coeffs;
    uint2 w[9];
#pragma unroll
    for (int k = 0; k < 9; ++k) w[k] = src[k];
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k = 0; k < 9; ++k) {
        const __half2 lo = *reinterpret_cast<const __half2*>(&w[k].x), hi = *reinterpret_cast<const __half2*>(&w[k].y);
        const float f[4] = {__low2float(lo), __high2float(lo), __low2float(hi), __high2float(hi)};
#pragma unroll
        for (int ch = 0; ch < 4; ++ch) acc[ch] = k == 0 ? s.b[0] * f[ch] : acc[ch] + s.b[k] * f[ch];
    }
    return make_float4(acc[0], acc[1], acc[2], acc[3]);
}

// ---- instance bins ----------------------------------------------------------------------------------------------
// The points are cut into kBinBlocks contiguous chunks, one per block, the same way in k_bin_count,
// k_bin_fill and k_records. k_bin_count leaves, per (chunk, tile), the number of instances the chunk's points have in the
// tile; k_bin_offsets turns that table into the exclusive prefix over the chunks of every tile and k_bin_scan
// into the start of every tile's bin. k_bin_fill then hands out bin slots from LDS cursors seeded with
// bin_start[tile] + prefix[chunk][tile]: no global atomic anywhere (they run at about 10 G/s on this machine,
// far below what 8M points need).
//
// Up to kMaxLdsTiles tiles a block keeps its per-tile counters / cursors as 32-bit words in LDS. Beyond that (the
// reference's 8x8 tiles on large images, up to the 65536 tiles of its 16-bit tile key, kernels.cu:204,214)
// k_bin_count counts in 16-bit halves of LDS words, which a chunk of at most kWideChunk points cannot overflow (its
// WIDE variant: one block of 1024 threads per CU, the counters fill the LDS), and k_bin_fill is launched once per
// window of kMaxLdsTiles tiles.
constexpr int kBinBlocks = 512, kBinBlocksWide = 1024;   // chunks: normally; for many tiles and many points
constexpr int kBinThreads = 512, kBinThreadsWide = 1024;
constexpr uint32_t kMaxLdsTiles = 16384;  // 64 KiB of 32-bit counters
constexpr uint32_t kWideChunk = 65024;    // points per chunk with 16-bit counters (a multiple of kBinThreads)

__host__ __device__ inline uint32_t bin_chunk_size(uint32_t n, uint32_t n_chunks) {
    const uint32_t per = (n + n_chunks - 1) / n_chunks;
    return (per + kBinThreads - 1) / kBinThreads * kBinThreads;
}

// 16-bit counters, two per LDS word: add one to the counter of `tile`, return its value before.
__device__ __forceinline__ uint32_t packed_counter_next(uint32_t* counters, uint32_t tile) {
    const uint32_t shift = (tile & 1u) * 16u;
    return (atomicAdd(&counters[tile >> 1], 1u << shift) >> shift) & 0xFFFFu;
}

template <int T, bool WIDE>
__global__ void __launch_bounds__(WIDE ? kBinThreadsWide : kBinThreads) k_bin_count(const float* __restrict__ positions,
                                                           const float* __restrict__ w2c, uint32_t* __restrict__ table,
                                                           uint2* __restrict__ split_count, Geometry g) {
    constexpr int kThreads = WIDE ? kBinThreadsWide : kBinThreads;
    INPC_DYNAMIC_LDS(uint32_t, s_count);
    __shared__ uint32_t s_split, s_rows;   // the chunk's points that touch several tiles, and their instances
    const uint32_t n_words = WIDE ? (g.n_tiles + 1u) / 2u : g.n_tiles;
    for (uint32_t t = threadIdx.x; t < n_words; t += kThreads) s_count[t] = 0u;
    if (threadIdx.x == 0) s_split = s_rows = 0u;
    __syncthreads();
    uint32_t my_split = 0, my_rows = 0;
    const ViewRows m = load_view_rows(w2c);
    const uint32_t chunk = bin_chunk_size(g.n, g.n_chunks);
    const uint32_t begin = min(blockIdx.x * chunk, g.n), end = min(begin + chunk, g.n);
    constexpr int kUnroll = 4;   // points per thread and round, their loads issued together
    for (uint32_t base = begin; base < end; base += kUnroll * kThreads) {
        float px[kUnroll], py[kUnroll], pz[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const uint32_t at = base + u * kThreads + threadIdx.x;
            const size_t i = at < end ? at : begin;
            px[u] = positions[3 * i];
            py[u] = positions[3 * i + 1];
            pz[u] = positions[3 * i + 2];
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            if (base + u * kThreads + threadIdx.x >= end) continue;
            const Projected p = project_point<T>(m, g, px[u], py[u], pz[u]);
            if (p.info)
                for_each_tile(p.info, g.gw, [&](uint32_t tile) {
                    if (WIDE) packed_counter_next(s_count, tile);
                    else atomicAdd(&s_count[tile], 1u);
                });
            if (p.touched > 1u) {
                my_split += 1u;
                my_rows += p.touched;
            }
        }
    }
    for (int sh = 32; sh > 0; sh >>= 1) {
        my_split += __shfl_down(my_split, sh, 64);
        my_rows += __shfl_down(my_rows, sh, 64);
    }
    if ((threadIdx.x & 63u) == 0u && my_split) {
        atomicAdd(&s_split, my_split);
        atomicAdd(&s_rows, my_rows);
    }
    __syncthreads();
    uint32_t* row = table + (size_t)blockIdx.x * g.n_tiles;
    for (uint32_t t = threadIdx.x; t < g.n_tiles; t += kThreads)
        row[t] = WIDE ? (s_count[t >> 1] >> ((t & 1u) * 16u)) & 0xFFFFu : s_count[t];
    if (threadIdx.x == 0) split_count[blockIdx.x] = make_uint2(s_split, s_rows);
}

// table[c][t] <- sum of table[c'][t] over c' < c; total[t] <- sum over all chunks.
// A block owns 64 tiles (lane = tile); each of its 16 waves takes a run of consecutive chunks, keeps them in
// registers, and gets the sum of the runs in front of it through LDS.
constexpr int kOffsetWaves = 16;
template <int ROWS>
__global__ void __launch_bounds__(kOffsetWaves * kWave) k_bin_offsets(uint32_t* __restrict__ table,
                                                                       uint32_t* __restrict__ total, uint32_t n_tiles) {
    constexpr int kOffsetRun = ROWS / kOffsetWaves;
    __shared__ uint32_t s_run[kOffsetWaves][kWave];
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uint32_t t = blockIdx.x * kWave + lane;
    const bool valid = t < n_tiles;
    uint32_t v[kOffsetRun];
    uint32_t sum = 0;
    uint32_t* column = table + (size_t)wave * kOffsetRun * n_tiles + t;
#pragma unroll
    for (int c = 0; c < kOffsetRun; ++c) {
        v[c] = valid ? column[(size_t)c * n_tiles] : 0u;
        sum += v[c];
    }
    s_run[wave][lane] = sum;
    __syncthreads();
    uint32_t run = 0, all = 0;
#pragma unroll
    for (int w = 0; w < kOffsetWaves; ++w) {
        const uint32_t r = s_run[w][lane];
        if ((uint32_t)w < wave) run += r;
        all += r;
    }
    if (valid) {
#pragma unroll
        for (int c = 0; c < kOffsetRun; ++c) {
            column[(size_t)c * n_tiles] = run;
            run += v[c];
        }
        if (wave == 0) total[t] = all;
    }
}

// One block. bin_start[t] = number of instances in the bins before t (n_tiles + 1 entries) and the tiles'
// [begin, end) ranges, (0, 0) for a tile without instances as the reference's cleared buffer leaves it
// (forward.cu:52). split_base[c] = {points that touch several tiles, their instances} in the chunks before c.
// When the instances or the gradient rows exceed the buffers, every bin is left empty and the overflow counter set:
// the later kernels then draw nothing.
// order[] = the schedule of the per-tile blocks of the sort and blend kernels: longest instance list first, so that
// the few very long tiles do not start last and run on alone. The order only affects scheduling, not results (tiles
// are independent); ties inside a bucket of 64 instances are in no particular order.
// The tiles go through LDS in segments of kScanSegment, so that every access to memory is coalesced and the time
// does not grow with the serial part of a thread (65,536 tiles are 16 segments).
constexpr int kScanBlock = 1024;
constexpr int kScanPer = 4;                            // consecutive tiles of a thread in a segment
constexpr int kScanSegment = kScanBlock * kScanPer;
constexpr int kOrderBuckets = 4096;
static_assert(kBinBlocksWide <= kScanBlock, "one thread per chunk in k_bin_scan");

// bucket 0 holds the longest lists
__device__ __forceinline__ uint32_t order_bucket(uint32_t count) {
    return (uint32_t)(kOrderBuckets - 1) - min(count >> 6, (uint32_t)(kOrderBuckets - 1));
}

// Exclusive prefix of `v` over the threads of a kScanBlock block, in thread order; `total` = the block's sum.
// s_wave: kScanBlock / kWave words. Two block barriers; may be called again right away.
__device__ __forceinline__ uint32_t scan_block_exclusive(uint32_t v, uint32_t* s_wave, uint32_t& total) {
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    uint32_t incl = v;
#pragma unroll
    for (int s = 1; s < 64; s <<= 1) {
        const uint32_t up = __shfl_up(incl, s, 64);
        if (lane >= (uint32_t)s) incl += up;
    }
    __syncthreads();   // s_wave is free again
    if (lane == 63u) s_wave[wave] = incl;
    __syncthreads();
    uint32_t before = incl - v;
    total = 0u;
#pragma unroll
    for (uint32_t w = 0; w < (uint32_t)(kScanBlock / kWave); ++w) {
        const uint32_t c = s_wave[w];
        if (w < wave) before += c;
        total += c;
    }
    return before;
}

// GAUSSIAN: the counters of the Gaussian footprint's pipeline. Its exact instance count (a point touches any number
// of tiles: the 32-bit sums may wrap around) has been added up by its preprocess pass, and it steps `generation`, the
// stamp the backward pass marks its gradient rows with: a new one per forward pass *execution* (a full-period
// congruential step in the workspace, increment from the host's per-call seed), so that a captured graph, whose
// kernel arguments never change, still gets a new stamp on every replay.
template <bool GAUSSIAN>
__global__ void __launch_bounds__(kScanBlock)
    k_bin_scan(const uint32_t* __restrict__ bin_count, uint32_t* __restrict__ bin_start, uint2* ranges,
               const uint2* __restrict__ split_count, uint2* __restrict__ split_base, uint32_t* __restrict__ order,
               uint32_t* counters, uint32_t n_tiles, uint32_t n_chunks, uint32_t capacity, uint32_t row_capacity,
               unsigned long long* generation, unsigned long long seed) {
    __shared__ uint32_t s_count[kScanSegment], s_start[kScanSegment];
    __shared__ uint32_t s_bucket[kOrderBuckets];
    __shared__ uint32_t s_wave[kScanBlock / kWave];
    const uint32_t tid = threadIdx.x;
    // totals first: they decide whether anything is drawn
    uint32_t mine = 0u;
    constexpr int kAhead = 8;   // loads of a thread in flight together: a single block has little else to hide them behind
    for (uint32_t first = 0; first < n_tiles; first += kAhead * kScanBlock) {
        uint32_t v[kAhead];
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            const uint32_t t = first + u * kScanBlock + tid;
            v[u] = t < n_tiles ? bin_count[t] : 0u;
        }
#pragma unroll
        for (int u = 0; u < kAhead; ++u) mine += v[u];
    }
    uint2 split = make_uint2(0u, 0u);
    if (tid < n_chunks) split = split_count[tid];
    uint32_t n_instances, n_split, n_rows;
    (void)scan_block_exclusive(mine, s_wave, n_instances);
    const uint32_t split_before = scan_block_exclusive(split.x, s_wave, n_split);
    const uint32_t rows_before = scan_block_exclusive(split.y, s_wave, n_rows);
    bool overflow = n_instances > capacity || n_rows > row_capacity;
    if (GAUSSIAN) overflow = *(const unsigned long long*)(counters + kCntInstances64) > (unsigned long long)capacity;
    if (tid < n_chunks) split_base[tid] = make_uint2(split_before, rows_before);
    for (int i = tid; i < kOrderBuckets; i += kScanBlock) s_bucket[i] = 0u;
    uint32_t carry = 0u;
    for (uint32_t first = 0; first < n_tiles; first += kScanSegment) {
        __syncthreads();   // the segment buffers are free (and, the first time, the buckets are cleared)
#pragma unroll
        for (int k = 0; k < kScanPer; ++k) {
            const uint32_t i = k * kScanBlock + tid, t = first + i;
            s_count[i] = t < n_tiles && !overflow ? bin_count[t] : 0u;
        }
        __syncthreads();
        uint32_t c[kScanPer], sum = 0u;
#pragma unroll
        for (int j = 0; j < kScanPer; ++j) {
            c[j] = s_count[tid * kScanPer + j];
            sum += c[j];
        }
        uint32_t segment_total;
        uint32_t run = carry + scan_block_exclusive(sum, s_wave, segment_total);
#pragma unroll
        for (int j = 0; j < kScanPer; ++j) {
            s_start[tid * kScanPer + j] = run;
            run += c[j];
        }
        carry += segment_total;
        __syncthreads();
#pragma unroll
        for (int k = 0; k < kScanPer; ++k) {
            const uint32_t i = k * kScanBlock + tid, t = first + i;
            if (t < n_tiles) {
                const uint32_t count = s_count[i], start = s_start[i];
                bin_start[t] = overflow ? 0u : start;
                ranges[t] = count ? make_uint2(start, start + count) : make_uint2(0u, 0u);
                atomicAdd(&s_bucket[order_bucket(count)], 1u);
            }
        }
    }
    __syncthreads();
    // the buckets' first places in the schedule, then every tile takes the next place of its bucket
    constexpr int kPer = kOrderBuckets / kScanBlock;
    uint32_t in_buckets = 0u;
#pragma unroll
    for (int i = 0; i < kPer; ++i) in_buckets += s_bucket[tid * kPer + i];
    uint32_t all;
    uint32_t place = scan_block_exclusive(in_buckets, s_wave, all);
#pragma unroll
    for (int i = 0; i < kPer; ++i) {
        const uint32_t c = s_bucket[tid * kPer + i];
        s_bucket[tid * kPer + i] = place;
        place += c;
    }
    __syncthreads();   // also: the ranges written above are visible to the whole block
    for (uint32_t first = 0; first < n_tiles; first += kAhead * kScanBlock) {
        uint2 r[kAhead];
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            const uint32_t t = first + u * kScanBlock + tid;
            r[u] = t < n_tiles ? ranges[t] : make_uint2(0u, 0u);
        }
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            const uint32_t t = first + u * kScanBlock + tid;
            if (t < n_tiles) order[atomicAdd(&s_bucket[order_bucket(r[u].y - r[u].x)], 1u)] = t;
        }
    }
    if (tid == 0) {
        bin_start[n_tiles] = overflow ? 0u : n_instances;
        if (GAUSSIAN) {
            const unsigned long long total = *(const unsigned long long*)(counters + kCntInstances64);
            counters[kCntKept] = overflow ? 0u : (uint32_t)total;
            counters[kCntInstances] = total > 0xFFFFFFFFull ? 0xFFFFFFFFu : (uint32_t)total;
            counters[kCntMulti] = overflow ? 0u : n_split;
            if (generation) *generation = *generation * 6364136223846793005ull + (seed | 1ull);
        } else {
            counters[kCntVisible] = 0u;   // counted by k_bin_fill
            counters[kCntError] = 0u;
            counters[kCntInstances] = n_instances;
            counters[kCntSplit] = overflow ? 0u : n_split;   // no list entry is written when nothing is drawn
            counters[kCntRows] = n_rows;
            counters[kCntOverflow] = overflow ? 1u : 0u;
        }
    }
}

// ---- preprocess -------------------------------------------------------------------------------------------
// Size of a record in 16-byte words, per feature mode and channel count (record_stride() / 16).
template <int FMODE, int C>
struct PreprocessShape {
    static constexpr bool kHalf = FMODE == INPC_FEAT_DIRECT_F16;
    static constexpr bool kDirect = FMODE == INPC_FEAT_DIRECT_F32 || kHalf;
    static constexpr uint32_t kBytes = kRecordHeader + (kDirect ? C * (kHalf ? 2 : 4) : 16);
    static constexpr uint32_t kStrideWords = (kBytes + 31u) / 32u * 2u;
    static constexpr size_t stage_bytes(int threads) { return (size_t)threads * (kStrideWords + 1) * 16; }   // padded rows
};

// What a training configuration keeps of the points that touch several tiles: a list entry
// {point | touched tiles << 28, first gradient row} per such point, and a flag byte per gradient row.
struct SplitOut {
    const uint2* base;      // per chunk: {such points, their instances} in the chunks before
    uint2* list;
    uint8_t* row_flags;
};

// Preprocess is two kernels that do not depend on each other: k_bin_fill drops the (depth key, point) pairs into
// the tiles' bins, which is all the tile sort needs; k_records writes the blend records. The host runs the second
// beside the first and the tile sort (which leaves the memory system idle) on a stream of its own.
// One launch fills the bins of the tiles [tile_first, tile_first + tile_count), at most kMaxLdsTiles of them, so that a
// block keeps a 32-bit cursor per tile in LDS; with more tiles the host launches it once per window of tiles (the
// points are projected again in every launch, which costs less than taking each slot's base from the tables in
// memory: 1.0 against 1.6 ms for 33,554,432 points and 63,860 tiles).
template <int T>
__global__ void __launch_bounds__(kBinThreads)
    k_bin_fill(const float* __restrict__ positions, const float* __restrict__ w2c, const uint32_t* __restrict__ table,
               const uint32_t* __restrict__ bin_start, uint64_t* __restrict__ pairs, uint32_t* counters,
               uint32_t tile_first, uint32_t tile_count, Geometry g) {
    constexpr int kThreads = kBinThreads;
    INPC_DYNAMIC_LDS(uint32_t, s_cursor);   // tile_count
    __shared__ uint32_t s_visible;
    const bool overflow = counters[kCntOverflow] != 0u;   // written by k_bin_scan: then no instance is stored
    const uint32_t* row = table + (size_t)blockIdx.x * g.n_tiles;   // instances of the chunks before, per tile
    for (uint32_t t = threadIdx.x; t < tile_count; t += kThreads) s_cursor[t] = bin_start[tile_first + t] + row[tile_first + t];
    if (threadIdx.x == 0) s_visible = 0u;
    __syncthreads();
    const ViewRows m = load_view_rows(w2c);
    uint32_t my_visible = 0;
    const uint32_t chunk = bin_chunk_size(g.n, g.n_chunks);
    const uint32_t begin = min(blockIdx.x * chunk, g.n), end = min(begin + chunk, g.n);
    constexpr int kUnroll = 4;   // points per thread and round, their loads issued together
    for (uint32_t base = begin; base < end; base += kUnroll * kThreads) {
        float px[kUnroll], py[kUnroll], pz[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            // a thread behind the end reads the chunk's first point and drops it
            const uint32_t at = base + u * kThreads + threadIdx.x;
            const size_t i = at < end ? at : begin;
            px[u] = positions[3 * i];
            py[u] = positions[3 * i + 1];
            pz[u] = positions[3 * i + 2];
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const uint32_t i = base + u * kThreads + threadIdx.x;
            if (i >= end) continue;
            const Projected p = project_point<T>(m, g, px[u], py[u], pz[u]);
            if (p.info == 0u) continue;
            my_visible += 1u;
            const uint64_t pair = ((uint64_t)depth_key(p.depth, g.key_bias) << 32) | (uint64_t)i;
            if (!overflow)
                for_each_tile(p.info, g.gw, [&](uint32_t tile) {
                    const uint32_t local = tile - tile_first;   // wraps around for a tile in front of the window
                    if (local < tile_count) pairs[atomicAdd(&s_cursor[local], 1u)] = pair;
                });
        }
    }
    if (tile_first != 0u) return;   // the drawn points are counted by the first launch
    // block total -> one global atomic
    for (int s = 32; s > 0; s >>= 1) my_visible += __shfl_down(my_visible, s, 64);
    if ((threadIdx.x & 63u) == 0u) atomicAdd(&s_visible, my_visible);
    __syncthreads();
    if (threadIdx.x == 0 && s_visible) atomicAdd(&counters[kCntVisible], s_visible);
}

constexpr int kRecordThreads = kBinThreads;

template <int T, int FMODE, int C>
__global__ void __launch_bounds__(kRecordThreads)
    k_records(const float* __restrict__ positions, const void* __restrict__ features,
              const float* __restrict__ opacities, const float* __restrict__ w2c,
              const float* __restrict__ cam_position, char* __restrict__ records,
              float* __restrict__ blending_weights, SplitOut split, float4* __restrict__ debug_geometry,
              const uint32_t* __restrict__ counters, Geometry g) {
    constexpr int kThreads = kRecordThreads;
    INPC_DYNAMIC_LDS(uint32_t, s_dyn);
    float4* s_stage = (float4*)s_dyn;      // record staging, 64 rows per wave
    __shared__ uint32_t s_split, s_rows;   // next list entry / gradient row for a point of this chunk
    const bool overflow = counters[kCntOverflow] != 0u;   // written by k_bin_scan: then nothing is drawn
    if (threadIdx.x == 0) {
        const uint2 first = split.base ? split.base[blockIdx.x] : make_uint2(0u, 0u);
        s_split = first.x;
        s_rows = first.y;
    }
    __syncthreads();
    const ViewRows m = load_view_rows(w2c);
    const uint32_t chunk = bin_chunk_size(g.n, g.n_chunks);
    const uint32_t begin = min(blockIdx.x * chunk, g.n), end = min(begin + chunk, g.n);
    // kUnroll points per thread and round, their loads issued together. A record leaves the block through LDS:
    // every lane assembles its record in the wave's staging rows, then neighbouring lanes write the 16-byte
    // words of one record, so that a store instruction covers a contiguous stretch of the record array
    // instead of one word of 64 different records.
    constexpr bool kDirect = FMODE == INPC_FEAT_DIRECT_F32 || FMODE == INPC_FEAT_DIRECT_F16;
    constexpr int kUnroll = kDirect ? 4 : 2;
    using Word = std::conditional_t<FMODE == INPC_FEAT_DIRECT_F16, uint2, uint4>;  // four channels
    constexpr int kWords = kDirect ? C / 4 : 1;
    constexpr int kPer = sizeof(Word) / 4;   // 32-bit registers per word
    constexpr uint32_t kStrideWords = PreprocessShape<FMODE, C>::kStrideWords, kRow = kStrideWords + 1;  // padded row
    const uint32_t lane = threadIdx.x & 63u;
    float4* stage = s_stage + (threadIdx.x >> 6) * (64u * kRow);
    for (uint32_t base = begin; base < end; base += kUnroll * kThreads) {
        float px[kUnroll], py[kUnroll], pz[kUnroll], op[kUnroll];
        uint32_t fw[kUnroll][kWords * kPer];   // plain registers (an array of vector types ends up in scratch memory)
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            // a thread behind the end reads the chunk's first point and drops it
            const uint32_t at = base + u * kThreads + threadIdx.x;
            const size_t i = at < end ? at : begin;
            px[u] = positions[3 * i];
            py[u] = positions[3 * i + 1];
            pz[u] = positions[3 * i + 2];
            op[u] = FMODE == INPC_FEAT_RAW37_F16 ? 0.0f : opacities[i];
            if (kDirect) {
                const Word* src = (const Word*)features + i * kWords;
#pragma unroll
                for (int q = 0; q < kWords; ++q) {
                    const Word v = src[q];
                    fw[u][q * kPer] = v.x;
                    fw[u][q * kPer + 1] = v.y;
                    if constexpr (kPer == 4) {
                        fw[u][q * kPer + 2] = v.z;
                        fw[u][q * kPer + 3] = v.w;
                    }
                }
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const uint32_t i = base + u * kThreads + threadIdx.x;
            bool drawn = false;
            if (i < end) {
                const Projected p = project_point<T>(m, g, px[u], py[u], pz[u]);
                drawn = p.info != 0u;
                if (drawn) {
                    float4* rec = stage + lane * kRow;
                    float opacity = op[u];
#pragma unroll
                    for (uint32_t w = 2; w < kStrideWords; ++w) rec[w] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                    if (kDirect) {
                        Word* dst = (Word*)(rec + 2);
#pragma unroll
                        for (int q = 0; q < kWords; ++q) {
                            Word v;
                            v.x = fw[u][q * kPer];
                            v.y = fw[u][q * kPer + 1];
                            if constexpr (kPer == 4) {
                                v.z = fw[u][q * kPer + 2];
                                v.w = fw[u][q * kPer + 3];
                            }
                            dst[q] = v;
                        }
                    } else {
                        const ShBasis sb = sh_basis(px[u], py[u], pz[u], cam_position);
                        if (FMODE == INPC_FEAT_SH36_F16) {
                            rec[2] = sh_to_view_aligned(sb, (const __half*)features + 36 * (size_t)i);
                        } else {
                            const __half* raw = (const __half*)features + 37 * (size_t)i;
                            rec[2] = sh_to_view(sb, raw + 1);
                            opacity = 1.0f - expf(-expf(__half2float(raw[0])));  // kernels.cu:142
                        }
                    }
                    uint32_t tag = i | (((p.info >> 16) & 3u) << 29);
                    uint32_t extra = __float_as_uint(p.depth);
                    if (split.list) {   // training configurations
                        extra = 0u;
                        if (p.touched > 1u && !overflow) {
                            tag |= kRecordMulti;
                            extra = atomicAdd(&s_rows, p.touched);
                            split.list[atomicAdd(&s_split, 1u)] = make_uint2(i | (p.touched << 28), extra);
                            for (uint32_t r = 0; r < p.touched; ++r) split.row_flags[extra + r] = 0;
                        }
                    }
                    const AxisWeights ax = axis_weights(p.sx), ay = axis_weights(p.sy);
                    rec[0] = make_float4(ax.w0, ax.w1, ay.w0, ay.w1);
                    rec[1] = make_float4(opacity, __uint_as_float(tag),
                                         __uint_as_float((uint32_t)(ax.left + 1) | ((uint32_t)(ay.left + 1) << 16)),
                                         __uint_as_float(extra));
                }
                if (blending_weights) blending_weights[i] = 0.0f;
                if (debug_geometry) debug_geometry[i] = make_float4(p.sx, p.sy, p.depth, __uint_as_float(p.info));
            }
            wave_sync();
            // the wave's 64 points are consecutive: their records are one contiguous stretch
            const uint32_t wave_first = base + u * kThreads + (threadIdx.x & ~63u);
            const uint64_t drawn_lanes = __ballot(drawn);
            float4* out = (float4*)(records + (size_t)wave_first * g.stride);
#pragma unroll
            for (uint32_t k = 0; k < kStrideWords; ++k) {
                const uint32_t flat = k * 64u + lane, r = flat / kStrideWords, w = flat % kStrideWords;
                if ((drawn_lanes >> r) & 1ull) out[flat] = stage[r * kRow + w];
            }
            wave_sync();
        }
    }
}

// ---- blend: helpers shared with blend.hpp ---------------------------------------------------------------------

// View features of a record (they follow the 32-byte header), as C floats.
template <int C, bool HALF>
__device__ __forceinline__ void load_record_features(float* dst, const char* __restrict__ record) {
    if (!HALF) {
        const float4* src = (const float4*)(record + kRecordHeader);
#pragma unroll
        for (int q = 0; q < C / 4; ++q) {
            const float4 f = src[q];
            dst[4 * q] = f.x;
            dst[4 * q + 1] = f.y;
            dst[4 * q + 2] = f.z;
            dst[4 * q + 3] = f.w;
        }
    } else {
        const uint2* src = (const uint2*)(record + kRecordHeader);
#pragma unroll
        for (int q = 0; q < C / 4; ++q) {
            const uint2 v = src[q];
            const __half2 lo = *reinterpret_cast<const __half2*>(&v.x), hi = *reinterpret_cast<const __half2*>(&v.y);
            dst[4 * q] = __low2float(lo);
            dst[4 * q + 1] = __high2float(lo);
            dst[4 * q + 2] = __low2float(hi);
            dst[4 * q + 3] = __high2float(hi);
        }
    }
}

#include "blend.hpp"
#include "tilesort.hpp"
#include "gaussian.hpp"

// view-space feature gradient -> (N,36) fp16; a point that was not drawn has a zero view gradient and
// gets zeros (kernels.cu:95). A point's 72 bytes are nine 8-byte words (word k = the four channels of coefficient
// k); the wave's 64 points leave through LDS as one contiguous run.
__global__ void __launch_bounds__(kBlock)
    k_sh_backward(const float* __restrict__ positions, const float* __restrict__ cam_position,
                  const float4* __restrict__ grad_view, __half* __restrict__ grad_features, uint32_t n) {
    __shared__ uint2 s_out[kBlock * 9];
    const uint32_t i = blockIdx.x * kBlock + threadIdx.x, lane = threadIdx.x & 63u;
    uint2* stage = s_out + (threadIdx.x >> 6) * (64u * 9u);
    uint2 word[9];
#pragma unroll
    for (int k = 0; k < 9; ++k) word[k] = make_uint2(0u, 0u);
    if (i < n) {
        const float4 g = grad_view[i];
        if (!(g.x == 0.0f && g.y == 0.0f && g.z == 0.0f && g.w == 0.0f)) {
            const ShBasis s = sh_basis(positions[3 * (size_t)i], positions[3 * (size_t)i + 1], positions[3 * (size_t)i + 2],
                                       cam_position);
#pragma unroll
            for (int k = 0; k < 9; ++k) {
                const __half2 lo = __halves2half2(__float2half_rn(s.b[k] * g.x), __float2half_rn(s.b[k] * g.y));
                const __half2 hi = __halves2half2(__float2half_rn(s.b[k] * g.z), __float2half_rn(s.b[k] * g.w));
                word[k] = make_uint2(*reinterpret_cast<const uint32_t*>(&lo), *reinterpret_cast<const uint32_t*>(&hi));
            }
        }
    }
#pragma unroll
    for (int k = 0; k < 9; ++k) stage[lane * 9u + k] = word[k];
    wave_sync();
    const uint32_t wave_first = i - lane;
    uint2* out = (uint2*)grad_features + (size_t)wave_first * 9;
#pragma unroll
    for (uint32_t r = 0; r < 9; ++r) {
        const uint32_t flat = r * 64u + lane;
        if (wave_first + flat / 9u < n) out[flat] = stage[flat];
    }
}

__global__ void __launch_bounds__(kBlock) k_float_to_half(const float* __restrict__ src, __half* __restrict__ dst,
                                                          size_t n) {
    const size_t stride = (size_t)gridDim.x * kBlock;
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) dst[i] = __float2half_rn(src[i]);
}

// ---- host: workspace layout ---------------------------------------------------------------------------------
struct Layout {
    inpc_raster_layout pub;
    Geometry geo;
    int T, C, fmode, key_bits;
    bool inference, sh, half_features;
    bool wide;   // more tiles than a block keeps 32-bit counters for
    // private offsets
    size_t bin_table, bin_total, tile_order, split_count, split_base;
    size_t pairs, pairs_scratch;
    size_t split_list, row_flags, row_features, row_opacities;   // points that straddle tiles (0: no backward pass)
    size_t ordered_records, tile_end;                            // 0: the configuration has no backward pass
};

uint32_t float_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

template <typename Tp>
Tp* at(void* ws, size_t off) {
    return (Tp*)((char*)ws + off);
}

int make_layout(const inpc_raster_config* cfg, Layout& L) {
    if (!cfg) return fail(INPC_E_INVALID_ARGUMENT, "raster: config is null");
    const inpc_camera& cam = cfg->cam;
    if (cfg->tile != 8 && cfg->tile != 16) return fail(INPC_E_INVALID_ARGUMENT, "raster: tile must be 8 or 16");
    if (cam.width <= 0 || cam.height <= 0) return fail(INPC_E_INVALID_ARGUMENT, "raster: empty image");
    if (cfg->n_points >= (1u << 28)) return fail(INPC_E_UNSUPPORTED, "raster: n_points must be below 2^28");
    L.T = cfg->tile;
    L.fmode = cfg->feature_mode;
    if (L.fmode < 0 || L.fmode > 3) return fail(INPC_E_UNSUPPORTED, "raster: unknown feature mode %d", L.fmode);
    L.sh = L.fmode == INPC_FEAT_SH36_F16 || L.fmode == INPC_FEAT_RAW37_F16;
    L.half_features = L.fmode == INPC_FEAT_DIRECT_F16;
    L.C = L.sh ? 4 : cfg->channels;
    if (L.C != 4 && L.C != 8 && L.C != 16) return fail(INPC_E_INVALID_ARGUMENT, "raster: channels must be 4, 8 or 16");
    L.inference = (cfg->flags & INPC_RASTER_INFERENCE) != 0;
    const bool training = !L.inference && L.fmode != INPC_FEAT_RAW37_F16;   // configurations with a backward pass
    const bool debug = (cfg->flags & INPC_RASTER_KEEP_GEOMETRY) != 0;
    Geometry& g = L.geo;
    g.n = cfg->n_points;
    g.W = cam.width;
    g.H = cam.height;
    g.gw = (uint32_t)((cam.width + L.T - 1) / L.T);
    g.gh = (uint32_t)((cam.height + L.T - 1) / L.T);
    g.n_tiles = g.gw * g.gh;
    g.tile_shift = L.T == 16 ? 4u : 3u;
    if (cam.width > 65000 || cam.height > 65000)
        return fail(INPC_E_UNSUPPORTED, "raster: images beyond 65000 pixels per side are not supported");
    if (g.n_tiles > 65536u)
        return fail(INPC_E_UNSUPPORTED, "raster: %u tiles exceed the 16-bit tile key (65536)", g.n_tiles);
    L.wide = g.n_tiles > kMaxLdsTiles;
    g.n_chunks = kBinBlocks;
    if (L.wide && bin_chunk_size(g.n, kBinBlocks) > kWideChunk) g.n_chunks = kBinBlocksWide;
    if (L.wide && bin_chunk_size(g.n, g.n_chunks) > kWideChunk)
        return fail(INPC_E_UNSUPPORTED, "raster: more than %u points with more than %u tiles are not supported",
                    kBinBlocksWide * kWideChunk, kMaxLdsTiles);
    g.cam = to_device_camera(cam);
    g.stride = record_stride(L.C, L.half_features);
    // depth keys of drawn points lie in [bits(near), bits(far)] when 0 < near <= far: sort on the offset
    L.key_bits = 32;
    g.key_bias = 0u;
    if (cam.near_plane > 0.0f && cam.far_plane >= cam.near_plane && cam.far_plane < INFINITY) {
        g.key_bias = float_bits(cam.near_plane);
        L.key_bits = std::max(1, bit_length(float_bits(cam.far_plane) - g.key_bias));
    }
    const int end_bit = bit_length(g.n_tiles - 1);

    // A point has at most four instances; evenly spread points have (1 + 1 / tile)^2 on average, which the default
    // capacity covers with a margin. k_bin_scan decides on the device whether a call fits.
    const size_t n = std::max<size_t>(g.n, 1);
    const uint64_t most = 4ull * g.n;
    uint64_t capacity = cfg->max_instances;
    if (capacity == 0) {
        const double per_point = (1.0 + 1.0 / L.T) * (1.0 + 1.0 / L.T);
        capacity = (uint64_t)std::ceil((double)g.n * per_point * 1.0625) + 65536ull;
    }
    capacity = std::max<uint64_t>(std::min(capacity, most), 1);
    g.capacity = (uint32_t)capacity;
    // gradient rows: the instances of the points that touch several tiles. With every point drawn they are at most twice
    // the instances beyond one per point, but when part of the points is culled the rest may all touch several tiles:
    // as many rows as instances, so that a call whose instances fit never fails for its rows
    g.row_capacity = 0xFFFFFFFFu;
    if (training) g.row_capacity = (uint32_t)capacity;

    size_t off = 0;
    auto take = [&](size_t bytes) {
        const size_t o = off;
        off += align_up(bytes, 256);
        return o;
    };
    inpc_raster_layout& P = L.pub;
    memset(&P, 0, sizeof(P));
    P.counters = take(kCntWords * 4);
    P.tile_ranges = take((size_t)g.n_tiles * 8);
    L.bin_table = take((size_t)g.n_chunks * g.n_tiles * 4);
    L.bin_total = take((size_t)g.n_tiles * 4);
    L.tile_order = take((size_t)g.n_tiles * 4);
    P.bin_start = take((size_t)(g.n_tiles + 1) * 4);
    L.split_count = take(kBinBlocksWide * 8);
    L.split_base = take(kBinBlocksWide * 8);
    P.point_record = take(n * g.stride);
    L.pairs = take(capacity * 8);
    P.instance_points = take(capacity * 4);
    L.split_list = L.row_flags = L.row_features = L.row_opacities = L.ordered_records = L.tile_end = 0;
    if (training) {
        const size_t rows = std::max<size_t>(g.row_capacity, 1);
        L.split_list = take((rows / 2 + 1) * 8);
        L.row_flags = take(rows);
        L.row_features = take(rows * L.C * 4);
        L.row_opacities = take(rows * 4);
        // the records once more, per instance and in the order of the tiles' lists, left by the forward blend for
        // the backward blend; how far each tile's reach. Until the forward blend runs the block is free and the
        // merges of the tile sort use it.
        L.ordered_records = take(capacity * (2 + (size_t)L.C / 4) * 16);
        L.tile_end = take((size_t)g.n_tiles * 4);
        L.pairs_scratch = L.ordered_records;
    } else {
        L.pairs_scratch = take(capacity * 8);
    }
    P.debug_geometry = debug ? take(n * 16) : 0;
    P.total_bytes = off;
    P.record_stride = g.stride;
    P.grid_width = g.gw;
    P.grid_height = g.gh;
    P.n_tiles = g.n_tiles;
    P.end_bit = (uint32_t)end_bit;
    P.depth_key_bias = g.key_bias;
    P.max_instances = g.capacity;
    return INPC_OK;
}

// Launch with `lds_bytes` of dynamic LDS; above 64 KiB the kernel has to be told once.
#define INPC_LAUNCH_LDS(name, kernel, grid, block, lds_bytes, stream, ...)                                   \
    do {                                                                                                     \
        if ((lds_bytes) > 48 * 1024) {                                                                       \
            hipError_t _a = hipFuncSetAttribute(reinterpret_cast<const void*>(&kernel),                      \
                                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)(lds_bytes)); \
            if (_a != hipSuccess)                                                                            \
                return fail(INPC_E_HIP, "%s: cannot reserve %zu bytes of LDS: %s", name, (size_t)(lds_bytes), \
                            hipGetErrorString(_a));                                                          \
        }                                                                                                    \
        ::inpc::timing_begin(name, stream);                                                                  \
        hipLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, __VA_ARGS__);                             \
        ::inpc::timing_end(stream);                                                                          \
        hipError_t _e = hipGetLastError();                                                                   \
        if (_e != hipSuccess) return fail(INPC_E_HIP, "launch of %s failed: %s", name, hipGetErrorString(_e)); \
    } while (0)

template <int T>
int launch_bin_count(const Layout& L, const float* positions, const float* w2c, void* ws, hipStream_t stream) {
    if (L.wide) {
        const size_t lds = (size_t)(L.geo.n_tiles + 1) / 2 * 4;
        INPC_LAUNCH_LDS("raster_bin_count", (k_bin_count<T, true>), dim3(L.geo.n_chunks), dim3(kBinThreadsWide), lds, stream,
                        positions, w2c, at<uint32_t>(ws, L.bin_table), at<uint2>(ws, L.split_count), L.geo);
    } else {
        const size_t lds = (size_t)L.geo.n_tiles * 4;
        INPC_LAUNCH_LDS("raster_bin_count", (k_bin_count<T, false>), dim3(L.geo.n_chunks), dim3(kBinThreads), lds, stream,
                        positions, w2c, at<uint32_t>(ws, L.bin_table), at<uint2>(ws, L.split_count), L.geo);
    }
    return INPC_OK;
}

// One block per tile and launch; blocks of kSmallThreads threads sort the tiles of at most tilesort::kSmallTile
// instances, blocks of kLargeThreads threads the others; a block whose tile belongs to the other launch ends at once.
struct TileSortBuffers {
    const uint2* ranges;
    const uint32_t* order;
    uint64_t* pairs;
    uint64_t* scratch;
    uint32_t* points;
    uint32_t n_tiles;
    int key_bits;
};

template <int THREADS>
int launch_tile_sort(const char* name, const TileSortBuffers& b, hipStream_t stream) {
    INPC_LAUNCH_LDS(name, tilesort::k_tile_sort<THREADS>, dim3(b.n_tiles), dim3(THREADS),
                    sizeof(tilesort::Shared<THREADS>), stream, b.ranges, b.order, b.pairs, b.scratch, b.points, b.key_bits);
    return INPC_OK;
}

template <int T>
int launch_bin_fill(const Layout& L, const float* positions, const float* w2c, void* ws, hipStream_t stream) {
    const uint32_t* table = at<uint32_t>(ws, L.bin_table);
    const uint32_t* bin_start = at<uint32_t>(ws, L.pub.bin_start);
    for (uint32_t first = 0; first < L.geo.n_tiles; first += kMaxLdsTiles) {
        const uint32_t count = std::min(kMaxLdsTiles, L.geo.n_tiles - first);
        const size_t lds = (size_t)count * 4;
        INPC_LAUNCH_LDS("raster_bin_fill", (k_bin_fill<T>), dim3(L.geo.n_chunks), dim3(kBinThreads), lds, stream, positions,
                        w2c, table, bin_start, at<uint64_t>(ws, L.pairs), at<uint32_t>(ws, L.pub.counters), first, count,
                        L.geo);
    }
    return INPC_OK;
}

template <int T, int FMODE, int C>
int launch_records(const Layout& L, const float* positions, const void* features, const float* opacities,
                   const float* w2c, const float* cam_position, float* blending_weights, void* ws, hipStream_t stream) {
    if (L.pub.record_stride != PreprocessShape<FMODE, C>::kStrideWords * 16u)
        return fail(INPC_E_UNSUPPORTED, "record stride %u does not match the record kernel", L.pub.record_stride);
    SplitOut split{nullptr, nullptr, nullptr};
    if (L.split_list) split = SplitOut{at<uint2>(ws, L.split_base), at<uint2>(ws, L.split_list), at<uint8_t>(ws, L.row_flags)};
    char* records = at<char>(ws, L.pub.point_record);
    float4* debug = L.pub.debug_geometry ? at<float4>(ws, L.pub.debug_geometry) : (float4*)nullptr;
    const size_t lds = PreprocessShape<FMODE, C>::stage_bytes(kRecordThreads);
    INPC_LAUNCH_LDS("raster_records", (k_records<T, FMODE, C>), dim3(L.geo.n_chunks), dim3(kRecordThreads), lds, stream,
                    positions, features, opacities, w2c, cam_position, records, blending_weights, split, debug,
                    (const uint32_t*)at<uint32_t>(ws, L.pub.counters), L.geo);
    return INPC_OK;
}

template <int T, int C, bool HALF>
int launch_blend_forward(const Layout& L, float* image, float* alpha, float* blending_weights, float* depth_image,
                         void* ws, hipStream_t stream) {
    const uint2* ranges = at<uint2>(ws, L.pub.tile_ranges);
    const uint32_t* order = at<uint32_t>(ws, L.tile_order);
    const uint32_t* inst = at<uint32_t>(ws, L.pub.instance_points);
    const char* records = at<char>(ws, L.pub.point_record);
    if (L.inference) {
        INPC_LAUNCH("raster_blend_inference", (blend::k_blend_forward<T, C, HALF, true>), dim3(L.geo.n_tiles), dim3(T * T),
                    stream, ranges, order, inst, records, L.geo.stride, image, alpha, (float*)nullptr, depth_image,
                    (float4*)nullptr, (uint32_t*)nullptr, L.geo.W, L.geo.H, L.geo.gw);
    } else {
        INPC_LAUNCH("raster_blend_forward", (blend::k_blend_forward<T, C, HALF, false>), dim3(L.geo.n_tiles), dim3(T * T),
                    stream, ranges, order, inst, records, L.geo.stride, image, alpha, blending_weights, (float*)nullptr,
                    L.ordered_records ? at<float4>(ws, L.ordered_records) : (float4*)nullptr,
                    L.tile_end ? at<uint32_t>(ws, L.tile_end) : (uint32_t*)nullptr, L.geo.W, L.geo.H, L.geo.gw);
    }
    return INPC_OK;
}

template <int T, int C, bool HALF>
int launch_blend_backward(const Layout& L, const float* grad_image, const float* grad_alpha, const float* image,
                          const float* alpha, float* grad_view, float* grad_opacities, void* ws, hipStream_t stream) {
    const blend::SplitRows rows{at<float>(ws, L.row_features), at<float>(ws, L.row_opacities),
                                at<uint8_t>(ws, L.row_flags), (const uint2*)at<uint2>(ws, L.split_list),
                                (const uint32_t*)at<uint32_t>(ws, L.pub.counters) + kCntSplit};
    INPC_LAUNCH("raster_blend_backward", (blend::k_blend_backward<T, C, HALF>), dim3(L.geo.n_tiles), dim3(T * T), stream,
                at<uint2>(ws, L.pub.tile_ranges), (const uint32_t*)at<uint32_t>(ws, L.tile_order),
                (const float4*)at<float4>(ws, L.ordered_records), (const uint32_t*)at<uint32_t>(ws, L.tile_end), grad_image,
                grad_alpha, image, alpha, grad_view,
                grad_opacities, rows, L.geo.W, L.geo.H, L.geo.gw);
    INPC_LAUNCH("raster_grad_reduce", blend::k_grad_reduce<C>, dim3(std::min(div_up(L.geo.n, 256u), 4096u)), dim3(256),
                stream, rows, grad_view, grad_opacities);
    return INPC_OK;
}

// dispatch on (tile, channels, storage)
#define INPC_DISPATCH_TCH(CALL)                                                   \
    do {                                                                          \
        const bool h = L.half_features;                                           \
        if (L.T == 8 && L.C == 4) return h ? CALL(8, 4, true) : CALL(8, 4, false);       \
        if (L.T == 8 && L.C == 8) return h ? CALL(8, 8, true) : CALL(8, 8, false);       \
        if (L.T == 8 && L.C == 16) return h ? CALL(8, 16, true) : CALL(8, 16, false);    \
        if (L.T == 16 && L.C == 4) return h ? CALL(16, 4, true) : CALL(16, 4, false);    \
        if (L.T == 16 && L.C == 8) return h ? CALL(16, 8, true) : CALL(16, 8, false);    \
        if (L.T == 16 && L.C == 16) return h ? CALL(16, 16, true) : CALL(16, 16, false); \
    } while (0)

int dispatch_blend_forward(const Layout& L, float* image, float* alpha, float* bw, float* depth_image, void* ws,
                           hipStream_t stream) {
#define CALL_FWD(T_, C_, H_) launch_blend_forward<T_, C_, H_>(L, image, alpha, bw, depth_image, ws, stream)
    INPC_DISPATCH_TCH(CALL_FWD);
#undef CALL_FWD
    return fail(INPC_E_UNSUPPORTED, "raster: unsupported blend configuration");
}

int dispatch_blend_backward(const Layout& L, const float* grad_image, const float* grad_alpha, const float* image,
                            const float* alpha, float* grad_view, float* grad_opacities, void* ws, hipStream_t stream) {
#define CALL_BWD(T_, C_, H_) \
    launch_blend_backward<T_, C_, H_>(L, grad_image, grad_alpha, image, alpha, grad_view, grad_opacities, ws, stream)
    INPC_DISPATCH_TCH(CALL_BWD);
#undef CALL_BWD
    return fail(INPC_E_UNSUPPORTED, "raster: unsupported backward configuration");
}

int dispatch_records(const Layout& L, const float* positions, const void* features, const float* opacities,
                     const float* w2c, const float* cam_position, float* bw, void* ws, hipStream_t stream) {
#define CALL_PRE(T_, FM_, C_) \
    launch_records<T_, FM_, C_>(L, positions, features, opacities, w2c, cam_position, bw, ws, stream)
#define CALL_PRE_C(T_, FM_)                    \
    do {                                       \
        if (L.C == 4) return CALL_PRE(T_, FM_, 4);   \
        if (L.C == 8) return CALL_PRE(T_, FM_, 8);   \
        if (L.C == 16) return CALL_PRE(T_, FM_, 16); \
    } while (0)
    switch (L.fmode) {
        case INPC_FEAT_SH36_F16:
            return L.T == 8 ? CALL_PRE(8, INPC_FEAT_SH36_F16, 4) : CALL_PRE(16, INPC_FEAT_SH36_F16, 4);
        case INPC_FEAT_RAW37_F16:
            return L.T == 8 ? CALL_PRE(8, INPC_FEAT_RAW37_F16, 4) : CALL_PRE(16, INPC_FEAT_RAW37_F16, 4);
        case INPC_FEAT_DIRECT_F32:
            if (L.T == 8) CALL_PRE_C(8, INPC_FEAT_DIRECT_F32);
            else CALL_PRE_C(16, INPC_FEAT_DIRECT_F32);
            break;
        case INPC_FEAT_DIRECT_F16:
            if (L.T == 8) CALL_PRE_C(8, INPC_FEAT_DIRECT_F16);
            else CALL_PRE_C(16, INPC_FEAT_DIRECT_F16);
            break;
    }
#undef CALL_PRE_C
#undef CALL_PRE
    return fail(INPC_E_UNSUPPORTED, "raster: unsupported record configuration");
}

// ---- Gaussian footprint: workspace layout and launches --------------------------------------------------------
struct GaussianLayout {
    inpc_gaussian_layout pub;
    Geometry geo;   // geo.n_chunks: chunks of points of the binning kernels
    gaussian::Params prm;
    int T, C, fmode, key_bits;
    bool inference, sh;
    size_t bin_table, bin_total, bin_start, tile_order, split_count, split_base;
    size_t pairs, pairs_scratch;
    size_t multi_list, grad_rows, generation;
};

int make_gaussian_layout(const inpc_gaussian_config* gcfg, GaussianLayout& L) {
    if (!gcfg) return fail(INPC_E_INVALID_ARGUMENT, "gaussian: config is null");
    const inpc_raster_config* cfg = &gcfg->base;
    const inpc_camera& cam = cfg->cam;
    if (cfg->tile != 8 && cfg->tile != 16) return fail(INPC_E_INVALID_ARGUMENT, "gaussian: tile must be 8 or 16");
    if (cam.width <= 0 || cam.height <= 0) return fail(INPC_E_INVALID_ARGUMENT, "gaussian: empty image");
    if (cfg->n_points >= (1u << 28)) return fail(INPC_E_UNSUPPORTED, "gaussian: n_points must be below 2^28");
    L.T = cfg->tile;
    L.fmode = cfg->feature_mode;
    if (L.fmode < 0 || L.fmode > 3) return fail(INPC_E_UNSUPPORTED, "gaussian: unknown feature mode %d", L.fmode);
    L.sh = L.fmode == INPC_FEAT_SH36_F16 || L.fmode == INPC_FEAT_RAW37_F16;
    L.C = L.sh ? 4 : cfg->channels;
    if (L.C != 4 && L.C != 8 && L.C != 16) return fail(INPC_E_INVALID_ARGUMENT, "gaussian: channels must be 4, 8 or 16");
    L.inference = (cfg->flags & INPC_RASTER_INFERENCE) != 0;
    if (L.fmode == INPC_FEAT_RAW37_F16 && !L.inference)
        return fail(INPC_E_INVALID_ARGUMENT, "gaussian: raw (N,37) features are an inference input");
    gaussian::Params& prm = L.prm;
    if (L.inference) {
        if (!(gcfg->sigma_cutoff > 0.0f) || !(gcfg->sigma_cutoff < 64.0f) || !(gcfg->sigma_world >= 0.0f) ||
            !(gcfg->sigma_world < INFINITY))
            return fail(INPC_E_INVALID_ARGUMENT, "gaussian: sigma_world must be >= 0 and sigma_cutoff in (0, 64)");
        prm.variance = gcfg->sigma_world * gcfg->sigma_world;                // kernels.cu:166
        prm.cutoff = gcfg->sigma_cutoff;                                     // kernels.cu:186-187
        prm.threshold = expf(-0.5f * gcfg->sigma_cutoff * gcfg->sigma_cutoff);  // inference.cu:171
    } else {
        constexpr float numerator = 0.3f * 0.3f * 0.5f * 0.5f;               // kernels.cu:57-59
        prm.variance = numerator / (cam.focal_x * cam.focal_y);
        prm.cutoff = gaussian::kTrainCutoff;
        prm.threshold = gaussian::kTrainThreshold;
    }
    prm.reach2 = -2.0f * logf(prm.threshold);
    Geometry& g = L.geo;
    g.n = cfg->n_points;
    g.W = cam.width;
    g.H = cam.height;
    g.gw = (uint32_t)((cam.width + L.T - 1) / L.T);
    g.gh = (uint32_t)((cam.height + L.T - 1) / L.T);
    g.n_tiles = g.gw * g.gh;
    if (g.n_tiles > 65536u)
        return fail(INPC_E_UNSUPPORTED, "gaussian: %u tiles exceed the 16-bit tile key (65536)", g.n_tiles);
    g.cam = to_device_camera(cam);
    g.stride = gaussian::record_stride(L.C);
    int depth_bits = 32;
    g.key_bias = 0u;
    if (cam.near_plane > 0.0f && cam.far_plane >= cam.near_plane && cam.far_plane < INFINITY) {
        g.key_bias = float_bits(cam.near_plane);
        depth_bits = std::max(1, bit_length(float_bits(cam.far_plane) - g.key_bias));
    }
    L.key_bits = depth_bits;
    const int end_bit = bit_length(g.n_tiles - 1);
    const size_t n = std::max<size_t>(g.n, 1);
    uint64_t capacity = gcfg->max_instances ? gcfg->max_instances : 4ull * g.n + 65536ull;
    if (capacity >= (1ull << 31)) return fail(INPC_E_UNSUPPORTED, "gaussian: max_instances must be below 2^31");
    prm.capacity = (uint32_t)capacity;
    g.n_chunks = kBinBlocks;

    size_t off = 0;
    auto take = [&](size_t bytes) {
        const size_t o = off;
        off += align_up(bytes, 256);
        return o;
    };
    inpc_gaussian_layout& P = L.pub;
    memset(&P, 0, sizeof(P));
    P.counters = take(kCntWords * 4);   // cleared by the forward pass: the preprocess pass adds its counts up there
    P.tile_ranges = take((size_t)g.n_tiles * 8);
    L.bin_table = take((size_t)g.n_chunks * g.n_tiles * 4);
    L.bin_total = take((size_t)g.n_tiles * 4);
    L.bin_start = take((size_t)(g.n_tiles + 1) * 4);
    L.tile_order = take((size_t)g.n_tiles * 4);
    L.split_count = take(kBinBlocksWide * 8);
    L.split_base = take(kBinBlocksWide * 8);
    P.point_touched = take(n * 4);
    P.point_bounds = take(n * 8);
    P.depth_keys = take(n * 4);
    L.multi_list = L.grad_rows = L.generation = 0;
    if (!L.inference) {   // configurations with a backward pass
        L.generation = take(8);   // never cleared: the stamp of the gradient rows carries on from call to call
        L.multi_list = take(n * 16);
        L.grad_rows = take(capacity * gaussian::GradRows::words(L.C) * 4);
    }
    P.point_record = take(n * g.stride);
    L.pairs = take(capacity * 8);
    L.pairs_scratch = take(capacity * 8);
    P.instance_points = take(capacity * 4);
    P.total_bytes = off;
    P.record_stride = g.stride;
    P.grid_width = g.gw;
    P.grid_height = g.gh;
    P.n_tiles = g.n_tiles;
    P.end_bit = (uint32_t)end_bit;
    P.depth_key_bias = g.key_bias;
    P.max_instances = prm.capacity;
    return INPC_OK;
}

template <int FMODE, int C>
int launch_gaussian_preprocess(const GaussianLayout& L, const float* positions, const void* features,
                               const float* opacities, const float* scales, const float* w2c, const float* cam_position,
                               float* blending_weights, void* ws, hipStream_t stream) {
    INPC_LAUNCH("gaussian_preprocess", (gaussian::k_preprocess<FMODE, C>), dim3(std::min(div_up(L.geo.n, kBlock), 2048u)), dim3(kBlock),
                stream, positions, features, opacities, scales, w2c, cam_position, at<char>(ws, L.pub.point_record),
                at<uint32_t>(ws, L.pub.point_touched), at<uint2>(ws, L.pub.point_bounds),
                at<uint32_t>(ws, L.pub.depth_keys), blending_weights, at<uint32_t>(ws, L.pub.counters), L.geo, L.prm,
                (float)L.T);
    return INPC_OK;
}

int dispatch_gaussian_preprocess(const GaussianLayout& L, const float* positions, const void* features,
                                 const float* opacities, const float* scales, const float* w2c,
                                 const float* cam_position, float* bw, void* ws, hipStream_t stream) {
#define CALL_GPRE(FM_, C_) \
    launch_gaussian_preprocess<FM_, C_>(L, positions, features, opacities, scales, w2c, cam_position, bw, ws, stream)
    switch (L.fmode) {
        case INPC_FEAT_SH36_F16: return CALL_GPRE(INPC_FEAT_SH36_F16, 4);
        case INPC_FEAT_RAW37_F16: return CALL_GPRE(INPC_FEAT_RAW37_F16, 4);
        case INPC_FEAT_DIRECT_F32:
            if (L.C == 4) return CALL_GPRE(INPC_FEAT_DIRECT_F32, 4);
            if (L.C == 8) return CALL_GPRE(INPC_FEAT_DIRECT_F32, 8);
            if (L.C == 16) return CALL_GPRE(INPC_FEAT_DIRECT_F32, 16);
            break;
        case INPC_FEAT_DIRECT_F16:
            if (L.C == 4) return CALL_GPRE(INPC_FEAT_DIRECT_F16, 4);
            if (L.C == 8) return CALL_GPRE(INPC_FEAT_DIRECT_F16, 8);
            if (L.C == 16) return CALL_GPRE(INPC_FEAT_DIRECT_F16, 16);
            break;
    }
#undef CALL_GPRE
    return fail(INPC_E_UNSUPPORTED, "gaussian: unsupported preprocess configuration");
}

template <int T, int C>
int launch_gaussian_blend_forward(const GaussianLayout& L, float* image, float* alpha, float* blending_weights,
                                  float* depth_image, void* ws, hipStream_t stream) {
    const uint2* ranges = at<uint2>(ws, L.pub.tile_ranges);
    const uint32_t* order = at<uint32_t>(ws, L.tile_order);
    const uint32_t* inst = at<uint32_t>(ws, L.pub.instance_points);
    const char* records = at<char>(ws, L.pub.point_record);
    if (L.inference) {
        INPC_LAUNCH("gaussian_blend_inference", (gaussian::k_blend_forward<T, C, true>), dim3(L.geo.n_tiles), dim3(T * T),
                    stream, ranges, order, inst, records, L.geo.stride, image, alpha, (float*)nullptr, depth_image,
                    L.geo.W, L.geo.H, L.geo.gw, L.prm.threshold, L.prm.reach2);
    } else {
        INPC_LAUNCH("gaussian_blend_forward", (gaussian::k_blend_forward<T, C, false>), dim3(L.geo.n_tiles), dim3(T * T),
                    stream, ranges, order, inst, records, L.geo.stride, image, alpha, blending_weights, (float*)nullptr,
                    L.geo.W, L.geo.H, L.geo.gw, L.prm.threshold, L.prm.reach2);
    }
    return INPC_OK;
}

// A 64-bit value no other forward call of this or another process is likely to have used: a counter above a
// start value drawn once per process. It seeds the step of the workspace's gradient-row stamp.
uint64_t next_stamp() {
    static std::atomic<uint64_t> counter{[] {
        std::random_device rd;
        return ((uint64_t)rd() << 32) ^ ((uint64_t)rd() << 11) ^ (uint64_t)std::chrono::steady_clock::now().time_since_epoch().count();
    }()};
    return counter.fetch_add(0x9E3779B97F4A7C15ull) + 1u;
}

template <int T, int C>
int launch_gaussian_blend_backward(const GaussianLayout& L, const float* grad_image, const float* grad_alpha,
                                   const float* image, const float* alpha, float* grad_view, float* grad_opacities,
                                   void* ws, hipStream_t stream) {
    const gaussian::GradRows rows{at<float>(ws, L.grad_rows), (const uint2*)at<uint2>(ws, L.pub.point_bounds),
                                  (const uint2*)at<uint2>(ws, L.generation)};
    INPC_LAUNCH("gaussian_blend_backward", (gaussian::k_blend_backward<T, C>), dim3(L.geo.n_tiles), dim3(T * T), stream,
                at<uint2>(ws, L.pub.tile_ranges), (const uint32_t*)at<uint32_t>(ws, L.tile_order),
                (const uint32_t*)at<uint32_t>(ws, L.pub.instance_points), (const char*)at<char>(ws, L.pub.point_record),
                L.geo.stride, grad_image, grad_alpha, image, alpha, grad_view, grad_opacities, rows, L.geo.W, L.geo.H,
                L.geo.gw, L.prm.threshold, L.prm.reach2);
    INPC_LAUNCH("gaussian_grad_reduce", gaussian::k_grad_reduce<C>, dim3(std::min(div_up(L.geo.n, kBlock), 4096u)),
                dim3(kBlock), stream, (const uint4*)at<uint4>(ws, L.multi_list),
                (const uint32_t*)at<uint32_t>(ws, L.pub.counters), rows, grad_view, grad_opacities);
    return INPC_OK;
}

#define INPC_DISPATCH_TC(CALL)                       \
    do {                                             \
        if (L.T == 8 && L.C == 4) return CALL(8, 4);    \
        if (L.T == 8 && L.C == 8) return CALL(8, 8);    \
        if (L.T == 8 && L.C == 16) return CALL(8, 16);  \
        if (L.T == 16 && L.C == 4) return CALL(16, 4);  \
        if (L.T == 16 && L.C == 8) return CALL(16, 8);  \
        if (L.T == 16 && L.C == 16) return CALL(16, 16); \
    } while (0)

int dispatch_gaussian_blend_forward(const GaussianLayout& L, float* image, float* alpha, float* bw, float* depth_image,
                                    void* ws, hipStream_t stream) {
#define CALL_GFWD(T_, C_) launch_gaussian_blend_forward<T_, C_>(L, image, alpha, bw, depth_image, ws, stream)
    INPC_DISPATCH_TC(CALL_GFWD);
#undef CALL_GFWD
    return fail(INPC_E_UNSUPPORTED, "gaussian: unsupported blend configuration");
}

int dispatch_gaussian_blend_backward(const GaussianLayout& L, const float* grad_image, const float* grad_alpha,
                                     const float* image, const float* alpha, float* grad_view, float* grad_opacities,
                                     void* ws, hipStream_t stream) {
#define CALL_GBWD(T_, C_) \
    launch_gaussian_blend_backward<T_, C_>(L, grad_image, grad_alpha, image, alpha, grad_view, grad_opacities, ws, stream)
    INPC_DISPATCH_TC(CALL_GBWD);
#undef CALL_GBWD
    return fail(INPC_E_UNSUPPORTED, "gaussian: unsupported backward configuration");
}

}  // namespace
}  // namespace inpc

using namespace inpc;

extern "C" {

int inpc_raster_layout_query(const inpc_raster_config* cfg, inpc_raster_layout* out) {
    Layout L;
    const int rc = make_layout(cfg, L);
    if (rc != INPC_OK) return rc;
    if (out) *out = L.pub;
    return INPC_OK;
}

int inpc_raster_forward(const inpc_raster_config* cfg, const float* positions, const void* features,
                        const float* opacities, const float* w2c, const float* cam_position, float* image,
                        float* alpha, float* blending_weights, float* depth_image, void* ws, size_t ws_bytes,
                        void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    Layout L;
    int rc = make_layout(cfg, L);
    if (rc != INPC_OK) return rc;
    if (!ws || ws_bytes < L.pub.total_bytes)
        return fail(INPC_E_WORKSPACE, "inpc_raster_forward: workspace has %zu bytes, needs %zu", ws_bytes,
                    L.pub.total_bytes);
    if (((uintptr_t)ws & 255u) != 0) return fail(INPC_E_WORKSPACE, "inpc_raster_forward: workspace must be 256-byte aligned");
    if (!w2c || !image || !alpha) return fail(INPC_E_INVALID_ARGUMENT, "inpc_raster_forward: null pointer");
    if (L.geo.n > 0 && (!positions || !features)) return fail(INPC_E_INVALID_ARGUMENT, "inpc_raster_forward: null input");
    if (L.fmode != INPC_FEAT_RAW37_F16 && L.geo.n > 0 && !opacities)
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_raster_forward: opacities are null");
    if (L.sh && !cam_position) return fail(INPC_E_INVALID_ARGUMENT, "inpc_raster_forward: cam_position is null");
    if (L.inference && !depth_image) return fail(INPC_E_INVALID_ARGUMENT, "inpc_raster_forward: depth image is null");
    if (!L.inference && L.geo.n > 0 && !blending_weights)
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_raster_forward: blending weights are null");
    if (L.fmode == INPC_FEAT_DIRECT_F32 && ((uintptr_t)features & 15u) != 0)
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_raster_forward: fp32 features must be 16-byte aligned");
    if ((L.fmode == INPC_FEAT_DIRECT_F16 || L.fmode == INPC_FEAT_SH36_F16) && ((uintptr_t)features & 7u) != 0)
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_raster_forward: fp16 features must be 8-byte aligned");

    uint32_t* counters = at<uint32_t>(ws, L.pub.counters);
    if (L.geo.n > 0) {
        rc = L.T == 8 ? launch_bin_count<8>(L, positions, w2c, ws, stream) : launch_bin_count<16>(L, positions, w2c, ws, stream);
        if (rc != INPC_OK) return rc;
        if (L.geo.n_chunks == (uint32_t)kBinBlocks) {
            INPC_LAUNCH("raster_bin_offsets", k_bin_offsets<kBinBlocks>, dim3(div_up(L.geo.n_tiles, kWave)),
                        dim3(kOffsetWaves * kWave), stream, at<uint32_t>(ws, L.bin_table), at<uint32_t>(ws, L.bin_total),
                        L.geo.n_tiles);
        } else {
            INPC_LAUNCH("raster_bin_offsets", k_bin_offsets<kBinBlocksWide>, dim3(div_up(L.geo.n_tiles, kWave)),
                        dim3(kOffsetWaves * kWave), stream, at<uint32_t>(ws, L.bin_table), at<uint32_t>(ws, L.bin_total),
                        L.geo.n_tiles);
        }
    } else {
        rc = fill_u32(at<uint32_t>(ws, L.bin_total), 0u, L.geo.n_tiles, stream);
        if (rc != INPC_OK) return rc;
        rc = fill_u32(at<uint32_t>(ws, L.split_count), 0u, 2 * kBinBlocksWide, stream);
        if (rc != INPC_OK) return rc;
    }
    INPC_LAUNCH("raster_bin_scan", k_bin_scan<false>, dim3(1), dim3(kScanBlock), stream,
                (const uint32_t*)at<uint32_t>(ws, L.bin_total), at<uint32_t>(ws, L.pub.bin_start),
                at<uint2>(ws, L.pub.tile_ranges), (const uint2*)at<uint2>(ws, L.split_count),
                at<uint2>(ws, L.split_base), at<uint32_t>(ws, L.tile_order), counters, L.geo.n_tiles, L.geo.n_chunks,
                L.geo.capacity, L.geo.row_capacity, (unsigned long long*)nullptr, 0ull);
    if (L.geo.n > 0) {
        rc = L.T == 8 ? launch_bin_fill<8>(L, positions, w2c, ws, stream) : launch_bin_fill<16>(L, positions, w2c, ws, stream);
        if (rc != INPC_OK) return rc;
        // The records are not needed before the blend, and writing them is bound by memory while the tile sort hardly
        // touches memory: they are written on the device's second stream, beside the tile sort (not beside
        // k_bin_fill, which is bound by memory itself). With the
        // per-launch timing on, everything stays on the caller's stream, so that each duration is that of a kernel
        // that has the device to itself.
        // A stream that is being captured into a graph takes its lane along (fork and join become edges of the graph);
        // a lane is never created during a capture, and a stream whose capture state cannot be told gets none.
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        const bool capture_known = hipStreamIsCapturing(stream, &capture) == hipSuccess;
        if (!capture_known) (void)hipGetLastError();
        SideLane* lane = nullptr;
        if (!timing_enabled() && capture_known) lane = side_lane(stream, capture != hipStreamCaptureStatusNone);
        hipStream_t record_stream = stream;
        if (lane) {
            std::lock_guard<std::mutex> lock(lane->mutex);
            if (hipEventRecord(lane->fork, stream) == hipSuccess &&
                hipStreamWaitEvent(lane->stream, lane->fork, 0) == hipSuccess) {
                record_stream = lane->stream;
            } else {
                (void)hipGetLastError();
                lane = nullptr;
            }
        }
        // the sort of the large tiles goes first (the blocks of the longest tiles are the ones to start early), then
        // the records beside it
        const TileSortBuffers sort{at<uint2>(ws, L.pub.tile_ranges), at<uint32_t>(ws, L.tile_order), at<uint64_t>(ws, L.pairs),
                                   at<uint64_t>(ws, L.pairs_scratch), at<uint32_t>(ws, L.pub.instance_points),
                                   L.geo.n_tiles, L.key_bits};
        const int rc_sort = launch_tile_sort<tilesort::kLargeThreads>("raster_tile_sort", sort, stream);
        rc = dispatch_records(L, positions, features, opacities, w2c, cam_position,
                              L.inference ? nullptr : blending_weights, ws, record_stream);
        if (rc == INPC_OK) rc = rc_sort;
        // the two launches of the tile sort touch different tiles. Where most tiles are large (going by the mean number
        // of instances per tile) the sort of the small ones runs behind the records, beside the sort of the large ones;
        // where most are small, the few large ones would only start late that way
        const bool small_beside = (uint64_t)L.geo.n * 5u / 4u > (uint64_t)L.geo.n_tiles * (tilesort::kSmallTile / 2u);
        if (rc == INPC_OK && small_beside)
            rc = launch_tile_sort<tilesort::kSmallThreads>("raster_tile_sort", sort, record_stream);
        // the caller's stream takes the second stream's work in again behind the tile sort, or wherever this
        // function is left before
        struct Join {
            hipStream_t stream;
            SideLane* lane;
            ~Join() {
                if (lane) (void)hipStreamWaitEvent(stream, lane->join, 0);
            }
        } join{stream, lane};
        if (lane && hipEventRecord(lane->join, lane->stream) != hipSuccess) {
            join.lane = nullptr;
            (void)hipStreamSynchronize(lane->stream);   // no event to wait for: wait on the host
            return fail(INPC_E_HIP, "inpc_raster_forward: cannot record on the record stream: %s",
                        hipGetErrorString(hipGetLastError()));
        }
        if (rc == INPC_OK && !small_beside) rc = launch_tile_sort<tilesort::kSmallThreads>("raster_tile_sort", sort, stream);
        if (rc != INPC_OK) return rc;
    }
    return dispatch_blend_forward(L, image, alpha, blending_weights, depth_image, ws, stream);
}

int inpc_raster_backward(const inpc_raster_config* cfg, const float* grad_image, const float* grad_alpha,
                         const float* image, const float* alpha, const float* positions, const float* cam_position,
                         void* grad_features, float* grad_opacities, float* grad_view_scratch, void* ws,
                         size_t ws_bytes, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    Layout L;
    int rc = make_layout(cfg, L);
    if (rc != INPC_OK) return rc;
    if (L.inference || L.fmode == INPC_FEAT_RAW37_F16)
        return fail(INPC_E_UNSUPPORTED, "inpc_raster_backward: inference configurations have no backward pass");
    if (!ws || ws_bytes < L.pub.total_bytes) return fail(INPC_E_WORKSPACE, "inpc_raster_backward: workspace too small");
    if (L.geo.n == 0) return INPC_OK;
    if (!grad_image || !grad_alpha || !image || !alpha || !grad_features || !grad_opacities)
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_raster_backward: null pointer");
    const bool direct32 = L.fmode == INPC_FEAT_DIRECT_F32;
    float* grad_view = direct32 ? (float*)grad_features : grad_view_scratch;
    if (!grad_view) return fail(INPC_E_INVALID_ARGUMENT, "inpc_raster_backward: this feature mode needs grad_view_scratch");
    if (((uintptr_t)grad_view & 15u) != 0)
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_raster_backward: the fp32 gradient buffer must be 16-byte aligned");
    if (L.sh && (!cam_position || !positions))
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_raster_backward: positions / cam_position are null");
    if (L.fmode == INPC_FEAT_SH36_F16 && ((uintptr_t)grad_features & 7u) != 0)
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_raster_backward: the fp16 gradient buffer must be 8-byte aligned");
    rc = fill_u32(grad_view, 0u, (size_t)L.geo.n * L.C, stream);
    if (rc != INPC_OK) return rc;
    rc = fill_u32(grad_opacities, 0u, L.geo.n, stream);
    if (rc != INPC_OK) return rc;
    rc = dispatch_blend_backward(L, grad_image, grad_alpha, image, alpha, grad_view, grad_opacities, ws, stream);
    if (rc != INPC_OK) return rc;
    if (L.fmode == INPC_FEAT_SH36_F16) {
        INPC_LAUNCH("raster_sh_backward", k_sh_backward, dim3(div_up(L.geo.n, kBlock)), dim3(kBlock), stream, positions,
                    cam_position, (const float4*)grad_view, (__half*)grad_features, L.geo.n);
    } else if (L.fmode == INPC_FEAT_DIRECT_F16) {
        const size_t total = (size_t)L.geo.n * L.C;
        INPC_LAUNCH("raster_grad_to_half", k_float_to_half, dim3((uint32_t)std::min<size_t>((total + 255) / 256, 8192)),
                    dim3(kBlock), stream, (const float*)grad_view, (__half*)grad_features, total);
    }
    return INPC_OK;
}

int inpc_raster_read_counters(const inpc_raster_config* cfg, const void* ws, uint32_t counters_host[3], void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    Layout L;
    const int rc = make_layout(cfg, L);
    if (rc != INPC_OK) return rc;
    uint32_t host[kCntWords] = {};
    INPC_HIP_CHECK(hipMemcpyAsync(host, (const char*)ws + L.pub.counters, sizeof(host), hipMemcpyDeviceToHost, stream));
    INPC_HIP_CHECK(hipStreamSynchronize(stream));
    if (counters_host) {
        counters_host[0] = host[kCntVisible];
        counters_host[1] = host[kCntInstances];
        counters_host[2] = host[kCntError];
    }
    if (host[kCntError]) return fail(INPC_E_DEVICE, "rasterizer raised its device error flag");
    if (host[kCntOverflow])
        return fail(INPC_E_WORKSPACE,
                    "raster: %u instances (%u of them of points that touch several tiles) do not fit max_instances = %u "
                    "(%u of those); nothing was drawn",
                    host[kCntInstances], host[kCntRows], L.geo.capacity, L.geo.row_capacity);
    return INPC_OK;
}

int inpc_gaussian_layout_query(const inpc_gaussian_config* cfg, inpc_gaussian_layout* out) {
    GaussianLayout L;
    const int rc = make_gaussian_layout(cfg, L);
    if (rc != INPC_OK) return rc;
    if (out) *out = L.pub;
    return INPC_OK;
}

int inpc_gaussian_forward(const inpc_gaussian_config* cfg, const float* positions, const void* features,
                          const float* opacities, const float* scales, const float* w2c, const float* cam_position,
                          float* image, float* alpha, float* blending_weights, float* depth_image, void* ws,
                          size_t ws_bytes, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    GaussianLayout L;
    int rc = make_gaussian_layout(cfg, L);
    if (rc != INPC_OK) return rc;
    if (!ws || ws_bytes < L.pub.total_bytes)
        return fail(INPC_E_WORKSPACE, "inpc_gaussian_forward: workspace has %zu bytes, needs %zu", ws_bytes,
                    L.pub.total_bytes);
    if (((uintptr_t)ws & 255u) != 0)
        return fail(INPC_E_WORKSPACE, "inpc_gaussian_forward: workspace must be 256-byte aligned");
    if (!w2c || !image || !alpha) return fail(INPC_E_INVALID_ARGUMENT, "inpc_gaussian_forward: null pointer");
    if (L.geo.n > 0 && (!positions || !features)) return fail(INPC_E_INVALID_ARGUMENT, "inpc_gaussian_forward: null input");
    if (L.fmode != INPC_FEAT_RAW37_F16 && L.geo.n > 0 && !opacities)
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_gaussian_forward: opacities are null");
    if (L.sh && !cam_position) return fail(INPC_E_INVALID_ARGUMENT, "inpc_gaussian_forward: cam_position is null");
    if (L.inference && !depth_image) return fail(INPC_E_INVALID_ARGUMENT, "inpc_gaussian_forward: depth image is null");
    if (!L.inference && L.geo.n > 0 && !blending_weights)
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_gaussian_forward: blending weights are null");
    if (!L.inference && scales)
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_gaussian_forward: per-point scales are an inference input");
    if (L.fmode == INPC_FEAT_DIRECT_F32 && ((uintptr_t)features & 15u) != 0)
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_gaussian_forward: fp32 features must be 16-byte aligned");
    if (L.fmode == INPC_FEAT_SH36_F16 && ((uintptr_t)features & 7u) != 0)
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_gaussian_forward: fp16 features must be 8-byte aligned");

    uint32_t* counters = at<uint32_t>(ws, L.pub.counters);
    rc = fill_u32(counters, 0u, kCntWords, stream);
    if (rc != INPC_OK) return rc;
    const uint32_t* touched = at<uint32_t>(ws, L.pub.point_touched);
    const uint2* bounds = at<uint2>(ws, L.pub.point_bounds);
    uint32_t* table = at<uint32_t>(ws, L.bin_table);
    const bool big = L.geo.n_tiles > kMaxLdsTiles;
    const uint32_t window = big ? 2u * kMaxLdsTiles : kMaxLdsTiles;
    if (L.geo.n > 0) {
        rc = dispatch_gaussian_preprocess(L, positions, features, opacities, scales, w2c, cam_position,
                                          L.inference ? nullptr : blending_weights, ws, stream);
        if (rc != INPC_OK) return rc;
        // a block keeps a 32-bit counter per tile in LDS: one launch per window of tiles (16,384 with two blocks of
        // 512 threads per CU; with more tiles than that 32,768 with one block of 1024 threads)
        for (uint32_t first = 0; first < L.geo.n_tiles; first += window) {
            const uint32_t count = std::min(window, L.geo.n_tiles - first);
            if (big) {
                INPC_LAUNCH_LDS("gaussian_bin_count", gaussian::k_bin_count<1024>, dim3(L.geo.n_chunks), dim3(1024),
                                (size_t)count * 4, stream, touched, bounds, table, at<uint2>(ws, L.split_count), first,
                                count, L.geo.n, L.geo.n_chunks, L.geo.n_tiles, L.geo.gw);
            } else {
                INPC_LAUNCH_LDS("gaussian_bin_count", gaussian::k_bin_count<kBinThreads>, dim3(L.geo.n_chunks),
                                dim3(kBinThreads), (size_t)count * 4, stream, touched, bounds, table,
                                at<uint2>(ws, L.split_count), first, count, L.geo.n, L.geo.n_chunks, L.geo.n_tiles,
                                L.geo.gw);
            }
        }
        INPC_LAUNCH("raster_bin_offsets", k_bin_offsets<kBinBlocks>, dim3(div_up(L.geo.n_tiles, kWave)),
                    dim3(kOffsetWaves * kWave), stream, table, at<uint32_t>(ws, L.bin_total), L.geo.n_tiles);
    } else {
        rc = fill_u32(at<uint32_t>(ws, L.bin_total), 0u, L.geo.n_tiles, stream);
        if (rc != INPC_OK) return rc;
        rc = fill_u32(at<uint32_t>(ws, L.split_count), 0u, 2 * kBinBlocksWide, stream);
        if (rc != INPC_OK) return rc;
    }
    INPC_LAUNCH("gaussian_bin_scan", k_bin_scan<true>, dim3(1), dim3(kScanBlock), stream,
                (const uint32_t*)at<uint32_t>(ws, L.bin_total), at<uint32_t>(ws, L.bin_start),
                at<uint2>(ws, L.pub.tile_ranges), (const uint2*)at<uint2>(ws, L.split_count),
                at<uint2>(ws, L.split_base), at<uint32_t>(ws, L.tile_order), counters, L.geo.n_tiles, L.geo.n_chunks,
                L.prm.capacity, L.prm.capacity,
                L.inference ? (unsigned long long*)nullptr : at<unsigned long long>(ws, L.generation),
                (unsigned long long)next_stamp());
    if (L.geo.n > 0) {
        for (uint32_t first = 0; first < L.geo.n_tiles; first += window) {
            const uint32_t count = std::min(window, L.geo.n_tiles - first);
#define INPC_GAUSSIAN_FILL(THREADS_)                                                                                  \
    INPC_LAUNCH_LDS("gaussian_bin_fill", gaussian::k_bin_fill<THREADS_>, dim3(L.geo.n_chunks), dim3(THREADS_),        \
                    (size_t)count * 4, stream, touched, bounds, (const uint32_t*)at<uint32_t>(ws, L.pub.depth_keys), \
                    (const uint32_t*)table, (const uint32_t*)at<uint32_t>(ws, L.bin_start), at<uint64_t>(ws, L.pairs), \
                    (const uint2*)at<uint2>(ws, L.split_base),                                                        \
                    L.inference ? (uint4*)nullptr : at<uint4>(ws, L.multi_list), at<char>(ws, L.pub.point_record),    \
                    L.geo.stride, (const uint32_t*)counters, first, count, L.geo.n, L.geo.n_chunks, L.geo.n_tiles,    \
                    L.geo.gw)
            if (big) INPC_GAUSSIAN_FILL(1024);
            else INPC_GAUSSIAN_FILL(kBinThreads);
#undef INPC_GAUSSIAN_FILL
        }
        // the tiles with the most instances first (large blocks), then the others with small blocks
        const TileSortBuffers sort{at<uint2>(ws, L.pub.tile_ranges), at<uint32_t>(ws, L.tile_order), at<uint64_t>(ws, L.pairs),
                                   at<uint64_t>(ws, L.pairs_scratch), at<uint32_t>(ws, L.pub.instance_points),
                                   L.geo.n_tiles, L.key_bits};
        rc = launch_tile_sort<tilesort::kLargeThreads>("gaussian_tile_sort", sort, stream);
        if (rc == INPC_OK) rc = launch_tile_sort<tilesort::kSmallThreads>("gaussian_tile_sort", sort, stream);
        if (rc != INPC_OK) return rc;
    }
    return dispatch_gaussian_blend_forward(L, image, alpha, blending_weights, depth_image, ws, stream);
}

int inpc_gaussian_backward(const inpc_gaussian_config* cfg, const float* grad_image, const float* grad_alpha,
                           const float* image, const float* alpha, const float* positions, const float* cam_position,
                           void* grad_features, float* grad_opacities, float* grad_view_scratch, void* ws,
                           size_t ws_bytes, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    GaussianLayout L;
    int rc = make_gaussian_layout(cfg, L);
    if (rc != INPC_OK) return rc;
    if (L.inference) return fail(INPC_E_UNSUPPORTED, "inpc_gaussian_backward: inference configurations have no backward pass");
    if (!ws || ws_bytes < L.pub.total_bytes) return fail(INPC_E_WORKSPACE, "inpc_gaussian_backward: workspace too small");
    if (L.geo.n == 0) return INPC_OK;
    if (!grad_image || !grad_alpha || !image || !alpha || !grad_features || !grad_opacities)
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_gaussian_backward: null pointer");
    const bool direct32 = L.fmode == INPC_FEAT_DIRECT_F32;
    float* grad_view = direct32 ? (float*)grad_features : grad_view_scratch;
    if (!grad_view) return fail(INPC_E_INVALID_ARGUMENT, "inpc_gaussian_backward: this feature mode needs grad_view_scratch");
    if (((uintptr_t)grad_view & 15u) != 0)
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_gaussian_backward: the fp32 gradient buffer must be 16-byte aligned");
    if (L.sh && (!cam_position || !positions))
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_gaussian_backward: positions / cam_position are null");
    if (L.fmode == INPC_FEAT_SH36_F16 && ((uintptr_t)grad_features & 7u) != 0)
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_gaussian_backward: the fp16 gradient buffer must be 8-byte aligned");
    rc = fill_u32(grad_view, 0u, (size_t)L.geo.n * L.C, stream);
    if (rc != INPC_OK) return rc;
    rc = fill_u32(grad_opacities, 0u, L.geo.n, stream);
    if (rc != INPC_OK) return rc;
    rc = dispatch_gaussian_blend_backward(L, grad_image, grad_alpha, image, alpha, grad_view, grad_opacities, ws, stream);
    if (rc != INPC_OK) return rc;
    if (L.fmode == INPC_FEAT_SH36_F16) {
        INPC_LAUNCH("raster_sh_backward", k_sh_backward, dim3(div_up(L.geo.n, kBlock)), dim3(kBlock), stream, positions,
                    cam_position, (const float4*)grad_view, (__half*)grad_features, L.geo.n);
    } else if (L.fmode == INPC_FEAT_DIRECT_F16) {
        const size_t total = (size_t)L.geo.n * L.C;
        INPC_LAUNCH("raster_grad_to_half", k_float_to_half, dim3((uint32_t)std::min<size_t>((total + 255) / 256, 8192)),
                    dim3(kBlock), stream, (const float*)grad_view, (__half*)grad_features, total);
    }
    return INPC_OK;
}

int inpc_gaussian_read_counters(const inpc_gaussian_config* cfg, const void* ws, uint32_t counters_host[4],
                                void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    GaussianLayout L;
    const int rc = make_gaussian_layout(cfg, L);
    if (rc != INPC_OK) return rc;
    uint32_t host[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    INPC_HIP_CHECK(hipMemcpyAsync(host, (const char*)ws + L.pub.counters, sizeof(host), hipMemcpyDeviceToHost, stream));
    INPC_HIP_CHECK(hipStreamSynchronize(stream));
    if (counters_host) {
        counters_host[0] = host[kCntVisible];
        counters_host[1] = host[kCntInstances];
        counters_host[2] = host[kCntError];
        counters_host[3] = host[kCntKept];
    }
    if (host[kCntError]) return fail(INPC_E_DEVICE, "rasterizer raised its device error flag");
    if (host[kCntInstances] > L.prm.capacity)
        return fail(INPC_E_WORKSPACE, "gaussian: %u instances do not fit max_instances = %u; nothing was drawn",
                    host[kCntInstances], L.prm.capacity);
    return INPC_OK;
}

}  // extern "C"
