// gaussian.hpp — the rasterizer's Gaussian footprint (RasterizerMode.GAUSSIAN; B/rasterization/src/gaussian/).
// Included by raster.hip after blend.hpp; shares the projection, SH and sort helpers with the bilinear path.
//
// A point is drawn as a screen-space Gaussian and touches any number of tiles. Per-point records in point order;
// the per-tile instance lists of the reference (depth sort, instances expanded in depth order, stable tile sort,
// ranges: B/rasterization/src/gaussian/forward.cu:12-172) come from per-tile bins sorted in LDS, as for the bilinear
// footprint.
//   k_preprocess        project, covariance -> conic, tile bounds, record, depth key (kernels.cu:11-324)
//   k_bin_count         per (chunk of points, tile): instances; a rectangle of many tiles is taken by the whole block,
//                       so a point that covers the screen costs no more per instance than one that covers a tile
//   k_bin_offsets, k_bin_scan (raster.hip)   prefix over the chunks; tile ranges, schedule, "do the instances fit"
//   k_bin_fill          a (depth key, point) pair per instance into the bin of its tile; gradient rows of the points
//                       that touch several tiles (kernels.cu:358-380)
//   tilesort.hpp        every bin sorted by (depth key, point index): the order of forward.cu:92-141
//   k_blend_*           one block per tile, one thread per pixel, a wave owns an 8 x 8 pixel block; per batch of
//                       T*T staged instances and 64 instances at a time, every lane first collects the instances
//                       whose pixel box contains its pixel (a few integer operations each) and then evaluates only
//                       those, each lane its own list in depth order (kernels.cu:401-660)
#pragma once

namespace gaussian {

constexpr float kDilation = 0.16f;                  // gaussian/config.h:19
constexpr float kTrainThreshold = 0.01110899653f;   // kernels.cu:452
constexpr float kTrainCutoff = 3.0f;                // kernels.cu:80-81
// Last header word of a record: point id (n < 2^28), then min(tile columns, 7), then "touches more than one tile".
constexpr uint32_t kMultiTile = 1u << 31;
constexpr uint32_t kPointMask = (1u << 28) - 1u;
constexpr int kColumnsShift = 28;
constexpr uint32_t kManyColumns = 7u;               // 7 or more tile columns: the count is looked up
constexpr uint32_t kNoKey = 0xFFFFFFFFu;            // depth key of a point that is not drawn

inline uint32_t record_stride(int channels) { return (uint32_t)align_up(32 + (size_t)channels * 4, 32); }

struct Params {
    float variance;    // world-space variance of a point without a scale of its own
    float cutoff;      // the tile bounds reach cutoff * sigma - 0.5 pixels
    float threshold;   // smallest footprint value that is drawn
    float reach2;      // -2 ln(threshold): |dx| <= sqrt(reach2 * cov_x) wherever the footprint passes the threshold
    uint32_t capacity; // instances the buffers hold
};

// ---- preprocess (kernels.cu:11-324) -------------------------------------------------------------------------------
template <int FMODE, int C>
__global__ void __launch_bounds__(kBlock)
    k_preprocess(const float* __restrict__ positions, const void* __restrict__ features,
                 const float* __restrict__ opacities, const float* __restrict__ scales, const float* __restrict__ w2c,
                 const float* __restrict__ cam_position, char* __restrict__ records, uint32_t* __restrict__ touched_out,
                 uint2* __restrict__ bounds_out, uint32_t* __restrict__ keys,
                 float* __restrict__ blending_weights, uint32_t* counters, Geometry g, Params prm, float tile_edge) {
    // A record leaves the block through LDS: every lane assembles its record in the wave's staging rows, then the
    // wave writes its 64 records, which are neighbours in memory, as one contiguous run of 16-byte words (a lane
    // storing its own record would put 16 bytes into each of 64 different lines per instruction).
    constexpr uint32_t kWords = (32u + 4u * C + 31u) / 32u * 2u, kRow = kWords + 1u;   // 16-byte words per record; padded row
    __shared__ float4 s_stage[kBlock * kRow];
    __shared__ uint32_t s_visible;
    __shared__ unsigned long long s_instances;
    if (threadIdx.x == 0) {
        s_visible = 0u;
        s_instances = 0ull;
    }
    __syncthreads();
    const uint32_t lane = threadIdx.x & 63u;
    float4* stage = s_stage + (threadIdx.x >> 6) * (64u * kRow);
    const ViewRows m = load_view_rows(w2c);
    uint32_t my_visible = 0u;
    unsigned long long my_instances = 0ull;
    // the grid is a few blocks per CU and walks over the points: the counts leave a block once
    for (uint32_t first = blockIdx.x * kBlock; first < g.n; first += gridDim.x * kBlock) {
    const uint32_t i = first + threadIdx.x;
#pragma unroll
    for (uint32_t w = 0; w < kWords; ++w) stage[lane * kRow + w] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    uint32_t touched = 0u;
    if (i < g.n) {
        uint32_t key = kNoKey;
        const float px = positions[3 * (size_t)i], py = positions[3 * (size_t)i + 1], pz = positions[3 * (size_t)i + 2];
        const float depth = affine_row(m.r3, px, py, pz);
        if (!(depth < g.cam.near_plane || depth > g.cam.far_plane)) {
            const float x = affine_row(m.r1, px, py, pz) / depth;
            const float y = affine_row(m.r2, px, py, pz) / depth;
            const float sx = x * g.cam.fx + g.cam.cx;
            const float sy = y * g.cam.fy + g.cam.cy;
            float variance = prm.variance;
            if (scales) variance = scales[i] * scales[i];
            const float j00 = g.cam.fx / depth;
            const float j02 = -j00 * fmaxf(-1.3f * g.cam.cx / g.cam.fx, fminf(x, 1.3f * g.cam.cx / g.cam.fx));
            const float j11 = g.cam.fy / depth;
            const float j12 = -j11 * fmaxf(-1.3f * g.cam.cy / g.cam.fy, fminf(y, 1.3f * g.cam.cy / g.cam.fy));
            float cov_x = variance * (j00 * j00 + j02 * j02);
            const float cov_y = variance * (j02 * j12);
            float cov_z = variance * (j11 * j11 + j12 * j12);
            cov_x += kDilation;
            cov_z += kDilation;
            const float det = cov_x * cov_z - cov_y * cov_y;
            if (det != 0.0f) {
                const float rcp = 1.0f / det;
                const float conic_x = cov_z * rcp, conic_y = -cov_y * rcp, conic_z = cov_x * rcp;
                const float reach_x = prm.cutoff * sqrtf(cov_x) - 0.5f;
                const float reach_y = prm.cutoff * sqrtf(cov_z) - 0.5f;
                const float fgw = (float)g.gw, fgh = (float)g.gh;
                const uint32_t x0 = (uint32_t)fminf(fgw, fmaxf(0.0f, floorf((sx - reach_x) / tile_edge)));
                const uint32_t x1 = (uint32_t)fminf(fgw, fmaxf(0.0f, ceilf((sx + reach_x) / tile_edge)));
                const uint32_t y0 = (uint32_t)fminf(fgh, fmaxf(0.0f, floorf((sy - reach_y) / tile_edge)));
                const uint32_t y1 = (uint32_t)fminf(fgh, fmaxf(0.0f, ceilf((sy + reach_y) / tile_edge)));
                if (x1 > x0 && y1 > y0) {
                    touched = (x1 - x0) * (y1 - y0);
                    bounds_out[i] = make_uint2(x0 | (x1 << 16), y0 | (y1 << 16));
                    float opacity = FMODE == INPC_FEAT_RAW37_F16 ? 0.0f : opacities[i];
                    float4* rec = stage + lane * kRow;
                    if (FMODE == INPC_FEAT_DIRECT_F32) {
                        const float4* src = (const float4*)features + (size_t)i * (C / 4);
#pragma unroll
                        for (int q = 0; q < C / 4; ++q) rec[2 + q] = src[q];
                    } else if (FMODE == INPC_FEAT_DIRECT_F16) {
                        const __half* src = (const __half*)features + (size_t)i * C;
#pragma unroll
                        for (int q = 0; q < C / 4; ++q)
                            rec[2 + q] = make_float4(__half2float(src[4 * q]), __half2float(src[4 * q + 1]),
                                                     __half2float(src[4 * q + 2]), __half2float(src[4 * q + 3]));
                    } else {
                        const ShBasis sb = sh_basis(px, py, pz, cam_position);
                        if (FMODE == INPC_FEAT_SH36_F16) {
                            rec[2] = sh_to_view_aligned(sb, (const __half*)features + 36 * (size_t)i);
                        } else {
                            const __half* raw = (const __half*)features + 37 * (size_t)i;
                            rec[2] = sh_to_view(sb, raw + 1);
                            opacity = 1.0f - expf(-expf(__half2float(raw[0])));  // kernels.cu:154
                        }
                    }
                    rec[0] = make_float4(sx, sy, opacity, conic_x);
                    rec[1] = make_float4(conic_y, conic_z, depth,
                                         __uint_as_float(i | (min(x1 - x0, kManyColumns) << kColumnsShift) | (touched > 1u ? kMultiTile : 0u)));
                    key = __float_as_uint(depth) - g.key_bias;
                }
            }
        }
        touched_out[i] = touched;
        keys[i] = key;
        if (blending_weights) blending_weights[i] = 0.0f;
    }
    wave_sync();
    {
        const uint32_t wave_first = i - lane;   // first point of this wave
        float4* out = (float4*)(records + (size_t)wave_first * g.stride);
#pragma unroll
        for (uint32_t k = 0; k < kWords; ++k) {
            const uint32_t flat = k * 64u + lane, r = flat / kWords, w = flat % kWords;
            if (wave_first + r < g.n) out[flat] = stage[r * kRow + w];
        }
    }
    wave_sync();   // the staging rows are reused by the next round
    my_visible += touched != 0u ? 1u : 0u;
    my_instances += touched;
    }
    for (int s = 32; s > 0; s >>= 1) {
        my_visible += __shfl_down(my_visible, s, 64);
        my_instances += __shfl_down(my_instances, s, 64);
    }
    if ((threadIdx.x & 63u) == 0u) {
        if (my_visible) atomicAdd(&s_visible, my_visible);
        if (my_instances) atomicAdd(&s_instances, my_instances);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        if (s_visible) atomicAdd(&counters[kCntVisible], s_visible);
        if (s_instances) atomicAdd((unsigned long long*)(counters + kCntInstances64), s_instances);
    }
}

// ---- instance bins (kernels.cu:346-399, forward.cu:87-160) --------------------------------------------------------
// The reference sorts the drawn points by depth, expands them into (tile, point) instances and sorts those by tile
// with a second stable device-wide sort: per tile the instances end up ordered by (depth key, point index). Here, as
// for the bilinear footprint, the instances are counted per (chunk of points, tile), every tile gets its range, a
// (depth key, point) pair per instance is dropped into the bin of its tile and one block per tile sorts its bin in LDS
// (tilesort.hpp): the same lists, without any device-wide sort. A point touches any number of tiles: the owner thread
// walks over a rectangle of up to kOwnTiles tiles itself, larger ones are queued and taken by the whole block.
constexpr uint32_t kOwnTiles = 64;
constexpr int kQueue = 512;   // queued points per block; further ones are walked by their owner after all

// Calls point(i, touched, bounds) once for every drawn point of the block's points [begin, end) and then
// visit(i, key, tile) for the tiles of its rectangle in the rows that the window [tile_first, tile_first + tile_count)
// of tile ids reaches into (the first and the last of these rows may lie partly outside the window: visit checks).
// `keys` may be null (key 0). A thread takes kUnroll points per round, their loads issued together.
template <int THREADS, typename Point, typename Visit>
__device__ __forceinline__ void for_each_instance(const uint32_t* __restrict__ touched, const uint2* __restrict__ bounds,
                                                  const uint32_t* __restrict__ keys, uint32_t begin, uint32_t end,
                                                  uint32_t gw, uint32_t tile_first, uint32_t tile_count,
                                                  uint32_t* s_queue, uint32_t* s_queued, Point point, Visit visit) {
    constexpr uint32_t kThreads = THREADS;
    constexpr int kUnroll = 8;
    const uint32_t band_y0 = tile_first / gw, band_y1 = (tile_first + tile_count + gw - 1u) / gw;
    if (threadIdx.x == 0) *s_queued = 0u;
    __syncthreads();
    for (uint32_t base = begin; base < end; base += kUnroll * kThreads) {
        uint32_t count[kUnroll], key[kUnroll];
        uint2 b[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            // a thread behind the end reads the chunk's first point and drops it
            const uint32_t at = base + u * kThreads + threadIdx.x;
            const uint32_t i = at < end ? at : begin;
            count[u] = touched[i];
            b[u] = bounds[i];
            key[u] = keys ? keys[i] : 0u;
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const uint32_t i = base + u * kThreads + threadIdx.x;
            if (i >= end || count[u] == 0u) continue;
            point(i, count[u], b[u]);
            const uint32_t x0 = b[u].x & 0xFFFFu, x1 = b[u].x >> 16;
            const uint32_t y0 = max(b[u].y & 0xFFFFu, band_y0), y1 = min(b[u].y >> 16, band_y1);
            if (y0 >= y1) continue;
            if ((x1 - x0) * (y1 - y0) > kOwnTiles) {
                const uint32_t slot = atomicAdd(s_queued, 1u);
                if (slot < (uint32_t)kQueue) {
                    s_queue[slot] = i;
                    continue;
                }
            }
            for (uint32_t ty = y0; ty < y1; ++ty)
                for (uint32_t tx = x0; tx < x1; ++tx) visit(i, key[u], ty * gw + tx);
        }
    }
    __syncthreads();
    const uint32_t queued = min(*s_queued, (uint32_t)kQueue);
    for (uint32_t q = 0; q < queued; ++q) {
        const uint32_t i = s_queue[q];
        const uint2 b = bounds[i];
        const uint32_t key = keys ? keys[i] : 0u;
        const uint32_t x0 = b.x & 0xFFFFu, nx = (b.x >> 16) - x0;
        const uint32_t y0 = max(b.y & 0xFFFFu, band_y0), ny = min(b.y >> 16, band_y1) - y0;
        for (uint32_t r = threadIdx.x; r < nx * ny; r += kThreads) visit(i, key, (y0 + r / nx) * gw + x0 + r % nx);
    }
}

// Per chunk of points and tile of the window: number of instances; per chunk (first window only): the points that
// touch several tiles and their instances.
template <int THREADS>
__global__ void __launch_bounds__(THREADS)
    k_bin_count(const uint32_t* __restrict__ touched, const uint2* __restrict__ bounds, uint32_t* __restrict__ table,
                uint2* __restrict__ split_count, uint32_t tile_first, uint32_t tile_count, uint32_t n, uint32_t n_chunks,
                uint32_t n_tiles, uint32_t gw) {
    INPC_DYNAMIC_LDS(uint32_t, s_count);   // tile_count
    __shared__ uint32_t s_queue[kQueue];
    __shared__ uint32_t s_queued, s_split, s_rows;
    for (uint32_t t = threadIdx.x; t < tile_count; t += THREADS) s_count[t] = 0u;
    if (threadIdx.x == 0) s_split = s_rows = 0u;
    const uint32_t chunk = bin_chunk_size(n, n_chunks);
    const uint32_t begin = min(blockIdx.x * chunk, n), end = min(begin + chunk, n);
    uint32_t my_split = 0u, my_rows = 0u;
    for_each_instance<THREADS>(
        touched, bounds, (const uint32_t*)nullptr, begin, end, gw, tile_first, tile_count, s_queue, &s_queued,
        [&](uint32_t, uint32_t count, uint2) {
            if (count > 1u) {
                my_split += 1u;
                my_rows += count;
            }
        },
        [&](uint32_t, uint32_t, uint32_t tile) {
            const uint32_t local = tile - tile_first;   // wraps around for a tile in front of the window
            if (local < tile_count) atomicAdd(&s_count[local], 1u);
        });
    if (my_split) {
        atomicAdd(&s_split, my_split);
        atomicAdd(&s_rows, my_rows);
    }
    __syncthreads();
    uint32_t* row = table + (size_t)blockIdx.x * n_tiles + tile_first;
    for (uint32_t t = threadIdx.x; t < tile_count; t += THREADS) row[t] = s_count[t];
    if (threadIdx.x == 0 && tile_first == 0u) split_count[blockIdx.x] = make_uint2(s_split, s_rows);
}

// Drops the pair (depth key, point) of every instance into the bin of its tile (window by window, like the counts).
// First window only, training configurations: a point that touches several tiles gets its gradient rows, one per
// tile in row-major order of its rectangle: the instance of tile (tx, ty) has row origin + ty * columns + tx, and the
// origin (modulo 2^32) replaces the depth in the point's record, which only the inference blend reads. The points go
// on a list {first row, rows, point} for the pass that adds the rows up.
template <int THREADS>
__global__ void __launch_bounds__(THREADS)
    k_bin_fill(const uint32_t* __restrict__ touched, const uint2* __restrict__ bounds, const uint32_t* __restrict__ keys,
               const uint32_t* __restrict__ table, const uint32_t* __restrict__ bin_start, uint64_t* __restrict__ pairs,
               const uint2* __restrict__ split_base, uint4* __restrict__ multi_list, char* __restrict__ records,
               uint32_t stride, const uint32_t* __restrict__ counters, uint32_t tile_first, uint32_t tile_count,
               uint32_t n, uint32_t n_chunks, uint32_t n_tiles, uint32_t gw) {
    INPC_DYNAMIC_LDS(uint32_t, s_cursor);   // tile_count
    __shared__ uint32_t s_queue[kQueue];
    __shared__ uint32_t s_queued, s_split, s_rows;
    if (counters[kCntKept] == 0u) return;   // nothing is drawn (no instances, or more than the buffers hold)
    const uint32_t* row = table + (size_t)blockIdx.x * n_tiles + tile_first;
    for (uint32_t t = threadIdx.x; t < tile_count; t += THREADS) s_cursor[t] = bin_start[tile_first + t] + row[t];
    const bool lists = multi_list != nullptr && tile_first == 0u;
    if (threadIdx.x == 0) {
        const uint2 first = lists ? split_base[blockIdx.x] : make_uint2(0u, 0u);
        s_split = first.x;
        s_rows = first.y;
    }
    const uint32_t chunk = bin_chunk_size(n, n_chunks);
    const uint32_t begin = min(blockIdx.x * chunk, n), end = min(begin + chunk, n);
    for_each_instance<THREADS>(
        touched, bounds, keys, begin, end, gw, tile_first, tile_count, s_queue, &s_queued,
        [&](uint32_t i, uint32_t count, uint2 b) {
            if (lists && count > 1u) {
                const uint32_t first_row = atomicAdd(&s_rows, count);
                const uint32_t x0 = b.x & 0xFFFFu, nx = (b.x >> 16) - x0, y0 = b.y & 0xFFFFu;
                ((uint32_t*)(records + (size_t)i * stride))[6] = first_row - y0 * nx - x0;
                multi_list[atomicAdd(&s_split, 1u)] = make_uint4(first_row, count, i, 0u);
            }
        },
        [&](uint32_t i, uint32_t key, uint32_t tile) {
            const uint32_t local = tile - tile_first;
            if (local < tile_count) pairs[atomicAdd(&s_cursor[local], 1u)] = ((uint64_t)key << 32) | (uint64_t)i;
        });
}

// ---- blend -----------------------------------------------------------------------------------------------------------
// An instance whose pixel box has at most kSlots pixels owns one slot per pixel of the box. The instance's own thread
// fills the slots with the footprint values (0: pixel skipped) when the instance is staged, so that the per-pixel
// walk, which is sequential where many points pile up on a few pixels, only has the blend itself left to do. A pixel
// that has blended the instance replaces the value (positive) by minus its contribution (forward: G * blending
// weight; backward: the blending weight, next to the opacity gradient in a second array); after the batch the
// instance's thread adds up the negative slots, in slot order: no atomics.
// Larger boxes (points close to the camera) have no slots. A training configuration takes such an instance through the
// whole block at once, at its place in the depth order: every pixel of its box evaluates the footprint and blends it,
// the waves add their pixels' contributions up (DPP sums, a fixed order), a block barrier, and the instance's own
// thread adds the waves' sums in wave order: no atomics either, and the same bits on every run. The inference blend
// has nothing to hand back to the instance and lets every pixel walk over such instances on its own.
constexpr int kSlots = 9;
constexpr int kSlotStride = kSlots;   // odd: rows of neighbouring instances spread over the LDS banks

// A staged instance: header words, features, and the pixel box (tile-local, conservative) its footprint can reach.
template <int T, int C>
struct Stage {
    static constexpr int TT = T * T;
    float4 head0[TT];   // sx, sy, opacity, conic.x
    float4 head1[TT];   // conic.y, conic.z, depth (or row origin), point id with the column and several-tiles bits
    float4 feat[TT * (C / 4)];
    uint32_t box[TT];   // bits 0-15: columns of the tile the footprint can reach, bits 16-31: rows
    float value[TT][kSlotStride];   // footprint value per pixel of the box (boxes of at most kSlots pixels)
};

// The record of this thread's instance of a coming batch, requested a batch ahead so that the gather (a line from
// anywhere in the point records per instance) is under way while the current batch is blended; `after` is the point
// of the thread's instance one batch further on.
template <int C>
struct Ahead {
    float4 h0, h1, f[C / 4];
    uint32_t after;
    __device__ __forceinline__ void request(const char* __restrict__ record) {
        const float4* src = (const float4*)record;
        h0 = src[0];
        h1 = src[1];
#pragma unroll
        for (int q = 0; q < C / 4; ++q) f[q] = src[2 + q];
    }
    // first batch and the point of the second
    __device__ __forceinline__ void start(const uint32_t* __restrict__ inst_points, const char* __restrict__ records,
                                          uint32_t stride, uint2 range, uint32_t block) {
        h0 = h1 = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
        for (int q = 0; q < C / 4; ++q) f[q] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        after = 0u;
        const uint32_t at = range.x + threadIdx.x;
        if (at < range.y) request(records + (size_t)inst_points[at] * stride);
        if (at + block < range.y) after = inst_points[at + block];
    }
};

// Thread `slot` stages instance `slot` of the batch.
template <int T, int C>
__device__ __forceinline__ void stage_instance(Stage<T, C>& st, uint32_t slot, const float4 h0, const float4 h1,
                                               const float4 (&feat)[C / 4], int tile_x0, int tile_y0, float reach2,
                                               float threshold) {
    st.head0[slot] = h0;
    st.head1[slot] = h1;
#pragma unroll
    for (int q = 0; q < C / 4; ++q) st.feat[slot * (C / 4) + q] = feat[q];
    // cov = conic^-1; the footprint passes the threshold only where |dx| <= sqrt(reach2 * cov_x) (same in y).
    // Taken a little wider; anything odd (non-positive determinant, non-finite values) selects the whole tile.
    const float det = h0.w * h1.y - h1.x * h1.x;
    float x_lo = 0.0f, x_hi = (float)T, y_lo = 0.0f, y_hi = (float)T;
    if (det > 0.0f) {
        // hardware reciprocal and square root (1 ulp) are plenty for a bound that is widened by a percent
        const float scale = reach2 * __builtin_amdgcn_rcpf(det);
        const float rx = __builtin_amdgcn_sqrtf(scale * h1.y) * 1.01f + 0.01f;
        const float ry = __builtin_amdgcn_sqrtf(scale * h0.w) * 1.01f + 0.01f;
        if (rx < 1e6f && ry < 1e6f) {
            x_lo = fminf(fmaxf(ceilf(h0.x - rx - 0.5f) - (float)tile_x0, 0.0f), (float)T);
            x_hi = fminf(fmaxf(floorf(h0.x + rx - 0.5f) + 1.0f - (float)tile_x0, 0.0f), (float)T);
            y_lo = fminf(fmaxf(ceilf(h0.y - ry - 0.5f) - (float)tile_y0, 0.0f), (float)T);
            y_hi = fminf(fmaxf(floorf(h0.y + ry - 0.5f) + 1.0f - (float)tile_y0, 0.0f), (float)T);
        }
    }
    // columns and rows of the tile as bit masks
    const uint32_t cols = ((1u << (uint32_t)x_hi) - 1u) & ~((1u << (uint32_t)x_lo) - 1u);
    const uint32_t rows = ((1u << (uint32_t)y_hi) - 1u) & ~((1u << (uint32_t)y_lo) - 1u);
    st.box[slot] = cols | (rows << 16);
    const int w = __popc(cols), h = __popc(rows);
    if (w * h <= kSlots) {
        const int px0 = tile_x0 + __ffs(cols) - 1, py0 = tile_y0 + __ffs(rows) - 1;
        int k = 0;
        for (int yy = 0; yy < h; ++yy) {
            for (int xx = 0; xx < w; ++xx, ++k) {
                float G;
                const bool hit = footprint_value(h0, h1, (float)(px0 + xx) + 0.5f, (float)(py0 + yy) + 0.5f, threshold, G);
                st.value[slot][k] = hit ? G : 0.0f;
            }
        }
    }
}

__device__ __forceinline__ bool has_slots(uint32_t box) { return __popc(box & 0xFFFFu) * __popc(box >> 16) <= kSlots; }

// Slot of tile-local pixel (lx, ly), which lies in the box, of a box that has slots.
__device__ __forceinline__ int slot_in(uint32_t box, int lx, int ly) {
    const uint32_t cols = box & 0xFFFFu, rows = box >> 16;
    return (ly - (__ffs(rows) - 1)) * __popc(cols) + (lx - (__ffs(cols) - 1));
}

// Slot of tile-local pixel (lx, ly), which lies in the box; -1 when the box has no slots.
__device__ __forceinline__ int slot_of(uint32_t box, int lx, int ly) {
    const uint32_t cols = box & 0xFFFFu, rows = box >> 16;
    const int w = __popc(cols), h = __popc(rows);
    if (w * h > kSlots) return -1;
    return (ly - (__ffs(rows) - 1)) * w + (lx - (__ffs(cols) - 1));
}

struct Pixel {
    int x, y;       // image coordinates
    int lx, ly;     // tile-local coordinates
    int qx0, qy0;   // tile-local origin of the wave's pixel block
    bool inside;
};

template <int T>
__device__ __forceinline__ Pixel pixel_of_thread(uint32_t tile, uint32_t gw, int W, int H) {
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    Pixel p;
    p.qx0 = T == 16 ? (int)(wave & 1u) * 8 : 0;
    p.qy0 = T == 16 ? (int)(wave >> 1) * 8 : 0;
    p.lx = p.qx0 + (int)(lane & 7u);
    p.ly = p.qy0 + (int)(lane >> 3);
    p.x = (int)(tile % gw) * T + p.lx;
    p.y = (int)(tile / gw) * T + p.ly;
    p.inside = p.x < W && p.y < H;
    return p;
}

// Does the box reach the wave's 8 x 8 pixel block?
__device__ __forceinline__ bool box_reaches(uint32_t box, const Pixel& p) {
    return (box & (0xFFu << p.qx0)) != 0u && (box & (0xFF0000u << p.qy0)) != 0u;
}

// Lane k holds row k of a 64 x 64 bit matrix; afterwards lane k holds column k (bit p of the result = bit k of lane
// p's input). Six exchange steps: in step j the two off-diagonal j x j blocks of every 2j x 2j block change places.
__device__ __forceinline__ uint64_t wave_transpose_bits(uint64_t x) {
    const uint32_t lane = lane_id();
    uint64_t keep = 0x00000000FFFFFFFFull;   // bit positions p with (p & j) == 0
#pragma unroll
    for (int j = 32; j > 0; j >>= 1) {
        const uint64_t other = __shfl_xor((unsigned long long)x, j, 64);
        x = (lane & (uint32_t)j) == 0u ? (x & keep) | ((other & keep) << j) : (x & ~keep) | ((other & ~keep) >> j);
        keep ^= keep << (j >> 1);
    }
    return x;
}

// Per lane: of the instances first + k (lane k looks at instance first + k, `box` is its box word, 0 for none), the
// ones whose box contains this lane's pixel, as a bit mask over k. Every lane marks the pixels of the wave's 8 x 8
// block that its instance's box covers (lane l owns pixel l of the block), and a bit transpose hands every pixel its
// column.
__device__ __forceinline__ uint64_t instances_over_pixel(uint32_t box, const Pixel& p) {
    const uint32_t cols = (box >> p.qx0) & 0xFFu, rows = (box >> (16 + p.qy0)) & 0xFFu;
    // byte r of a half = cols when row r is in the box: the row bits spread to one per byte, times cols
    const uint32_t lo = (((rows & 15u) * 0x00204081u) & 0x01010101u) * cols;
    const uint32_t hi = (((rows >> 4) * 0x00204081u) & 0x01010101u) * cols;
    return wave_transpose_bits((uint64_t)lo | ((uint64_t)hi << 32));
}


template <int T, int C, bool INFERENCE>
__global__ void __launch_bounds__(T * T)
    k_blend_forward(const uint2* __restrict__ ranges, const uint32_t* __restrict__ order,
                    const uint32_t* __restrict__ inst_points, const char* __restrict__ records, uint32_t stride,
                    float* __restrict__ image, float* __restrict__ alpha_image, float* blending_weights,
                    float* __restrict__ depth_image, int W, int H, uint32_t gw, float threshold, float reach2) {
    constexpr int TT = T * T;
    __shared__ Stage<T, C> st;
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t tile = order[blockIdx.x];
    const Pixel px = pixel_of_thread<T>(tile, gw, W, H);
    const int tile_x0 = (int)(tile % gw) * T, tile_y0 = (int)(tile / gw) * T;
    const float cx = (float)px.x + 0.5f, cy = (float)px.y + 0.5f;
    float acc[C];
#pragma unroll
    for (int c = 0; c < C; ++c) acc[c] = 0.0f;
    float depth_acc = 0.0f, tr = 1.0f;
    bool done = !px.inside;
    // per wave: what its pixels add to the blending weight of the instance without slots that the block is at; two
    // sets, so that the next such instance does not overwrite what the thread of this one is still reading
    __shared__ float s_big[2][TT / 64];
    uint32_t big_parity = 0u;
    const uint2 range = ranges[tile];
    Ahead<C> ahead;
    ahead.start(inst_points, records, stride, range, TT);
    for (uint32_t base = range.x; base < range.y; base += TT) {
        if (__syncthreads_count(done) == TT) break;
        const uint32_t count = min((uint32_t)TT, range.y - base);
        {
            const float4 h0 = ahead.h0, h1 = ahead.h1;
            float4 feat[C / 4];
#pragma unroll
            for (int q = 0; q < C / 4; ++q) feat[q] = ahead.f[q];
            if (base + TT + tid < range.y) ahead.request(records + (size_t)ahead.after * stride);
            if (base + 2u * TT + tid < range.y) ahead.after = inst_points[base + 2u * TT + tid];
            if (tid < count) stage_instance<T, C>(st, tid, h0, h1, feat, tile_x0, tile_y0, reach2, threshold);
        }
        __syncthreads();
        {
            const bool wave_live = __ballot(!done) != 0ull;
            for (uint32_t first = 0; first < count; first += 64u) {
                const uint32_t at = first + lane;
                const uint32_t my_box = at < count ? st.box[at] : 0u;
                // the instances without slots of these 64, the same mask in every wave of the block
                const uint64_t big = INFERENCE ? 0ull : __ballot(!has_slots(my_box));
                if (!wave_live && big == 0ull) continue;
                const uint64_t reach = __ballot(box_reaches(my_box, px));
                const bool all_slots = __ballot(box_reaches(my_box, px) && !has_slots(my_box)) == 0ull;
                uint64_t over = reach != 0ull ? instances_over_pixel(my_box, px) : 0ull;
                if (done) over = 0ull;
                uint64_t now = 0ull;   // the part of `over` a walk is going through
                // blend instance j, whose footprint value at this pixel is G; returns G * blending weight
                auto blend = [&](uint32_t j, float G) {
                    const float a = st.head0[j].z * G;
                    const float bw = tr * a;
#pragma unroll
                    for (int q = 0; q < C / 4; ++q) {
                        const float4 f = st.feat[j * (C / 4) + q];
                        acc[4 * q] += bw * f.x;
                        acc[4 * q + 1] += bw * f.y;
                        acc[4 * q + 2] += bw * f.z;
                        acc[4 * q + 3] += bw * f.w;
                    }
                    if (INFERENCE) depth_acc += bw * st.head1[j].z;
                    tr *= 1.0f - a;
                    if (tr < kTransmittanceThreshold) {
                        done = true;
                        over = 0ull;
                        now = 0ull;
                    }
                    return bw > 0.0f ? G * bw : 0.0f;
                };
                // every lane its own instances of `now`, all of which have slots
                auto walk_slots = [&]() {
                    while (__ballot(now != 0ull) != 0ull) {
                        if (now != 0ull) {
                            const uint32_t j = first + (uint32_t)__builtin_ctzll(now);
                            now &= now - 1ull;
                            const int slot = slot_in(st.box[j], px.lx, px.ly);
                            const float G = st.value[j][slot];
                            if (G != 0.0f) {
                                const float part = blend(j, G);
                                if (!INFERENCE) st.value[j][slot] = -part;
                            }
                        }
                    }
                };
                if (all_slots && big == 0ull) {   // the usual case
                    now = over;
                    walk_slots();
                } else if (INFERENCE) {   // nothing goes back to the instances: every lane on its own
                    now = over;
                    while (__ballot(now != 0ull) != 0ull) {
                        if (now == 0ull) continue;
                        const uint32_t j = first + (uint32_t)__builtin_ctzll(now);
                        now &= now - 1ull;
                        const int slot = slot_of(st.box[j], px.lx, px.ly);
                        float G;
                        if (slot >= 0) {
                            G = st.value[j][slot];
                            if (G == 0.0f) continue;
                        } else if (!footprint_value(st.head0[j], st.head1[j], cx, cy, threshold, G)) {
                            continue;
                        }
                        (void)blend(j, G);
                    }
                } else {
                    // in depth order: the instances with slots up to the next one without, lane by lane, then that
                    // one by the whole block
                    uint64_t big_left = big;
                    for (;;) {
                        const uint32_t kb = big_left != 0ull ? (uint32_t)__builtin_ctzll(big_left) : 64u;
                        now = kb == 64u ? over : over & ((1ull << kb) - 1ull);
                        over &= ~now;
                        walk_slots();
                        if (kb == 64u) break;
                        big_left &= big_left - 1ull;
                        const uint32_t j = first + kb;
                        float part = 0.0f, G;
                        if (((over >> kb) & 1ull) != 0ull &&
                            footprint_value(st.head0[j], st.head1[j], cx, cy, threshold, G))
                            part = blend(j, G);
                        over &= ~(1ull << kb);
                        const float wave_part = blend::wave_sum(part);
                        if (lane == 0u) s_big[big_parity][tid >> 6] = wave_part;
                        __syncthreads();
                        if (tid == j) {   // the instance's thread: its blending weight in this tile
                            float w = 0.0f;
#pragma unroll
                            for (int q = 0; q < TT / 64; ++q) w += s_big[big_parity][q];
                            st.value[j][0] = w;
                        }
                        big_parity ^= 1u;
                    }
                }
            }
        }
        if (!INFERENCE) {
            __syncthreads();
            if (tid < count) {
                float w = 0.0f;
                const uint32_t box = st.box[tid];
                const int used = __popc(box & 0xFFFFu) * __popc(box >> 16);
                if (used <= kSlots) {
#pragma unroll
                    for (int k = 0; k < kSlots; ++k) {
                        const float v = st.value[tid][k];
                        if (k < used && v < 0.0f) w -= v;   // slots no pixel has blended still hold the footprint value
                    }
                } else {
                    w = st.value[tid][0];   // an instance without slots: added up when the block went through it
                }
                if (w != 0.0f) {
                    const uint32_t word = __float_as_uint(st.head1[tid].w);
                    if (word & kMultiTile) atomicAdd(&blending_weights[word & kPointMask], w);
                    else blending_weights[word & kPointMask] = w;   // the point's only instance
                }
            }
        }
    }
    if (px.inside) {
        const size_t n_pixels = (size_t)W * H, pix = (size_t)px.y * W + px.x;
#pragma unroll
        for (int c = 0; c < C; ++c) image[c * n_pixels + pix] = acc[c];
        const float alpha_px = 1.0f - tr;
        alpha_image[pix] = tr < kTransmittanceThreshold ? 1.0f : alpha_px;
        if (INFERENCE) depth_image[pix] = alpha_px > 0.0f ? depth_acc / alpha_px : 0.0f;
    }
}

// Gradient rows of the points that touch several tiles: one row per instance, a point's rows one after the other in
// the row-major order of its tiles: C + 1 values, then the two words of the call's stamp, padded
// to whole 16-byte words. A block that ends early (every pixel saturated) leaves the rows of its remaining instances
// unwritten: a row counts when it carries the stamp of the forward pass the rows were laid out by (64 bits, a new
// value per execution of k_bin_scan, kept in the workspace), so nothing has to be cleared. Backward passes of one
// forward pass share the stamp: they write the same rows.
struct GradRows {
    float* values;
    const uint2* bounds;   // per point: tile bounds (looked up for points with kManyColumns or more tile columns)
    const uint2* stamp;    // the workspace's current stamp
    __host__ __device__ static constexpr uint32_t words(int channels) { return (uint32_t)(channels + 6) / 4u * 4u; }
};

// Gradient of a point that touches several tiles = sum of its rows, in row order. A group of neighbouring lanes
// takes one such point, lane j the j-th 16-byte word of every row, so that a wave reads whole rows of neighbouring
// points with each load (one lane per point walked its rows 16 bytes at a time and fetched every line three times:
// 0.89 GB for 0.28 GB of rows). The last word of a row carries the opacity gradient and the stamp.
template <int C>
__global__ void __launch_bounds__(kBlock)
    k_grad_reduce(const uint4* __restrict__ multi_list, const uint32_t* __restrict__ counters, GradRows rows,
                  float* __restrict__ grad_features, float* __restrict__ grad_opacities) {
    constexpr uint32_t kWords = GradRows::words(C) / 4u;                   // 16-byte words per row: C / 4 + 1
    constexpr uint32_t kGroup = kWords <= 2u ? 2u : kWords <= 4u ? 4u : 8u;  // lanes per point
    static_assert(kWords == (uint32_t)C / 4u + 1u && kWords <= kGroup, "row layout");
    if (counters[kCntKept] == 0u) return;
    const uint32_t n_multi = counters[kCntMulti];
    const uint2 stamp = *rows.stamp;
    const uint32_t gtid = blockIdx.x * kBlock + threadIdx.x, lane = threadIdx.x & 63u;
    const uint32_t word = gtid % kGroup, tail_lane = (lane & ~(kGroup - 1u)) + kWords - 1u;
    const uint32_t stride = gridDim.x * kBlock / kGroup;
    uint32_t m = gtid / kGroup;
    uint4 next = m < n_multi ? multi_list[m] : make_uint4(0u, 0u, 0u, 0u);
    for (; m < n_multi; m += stride) {   // the lanes of a group stay together
        const uint4 entry = next;
        if (m + stride < n_multi) next = multi_list[m + stride];
        const uint32_t first = entry.x, end = entry.x + entry.y, point = entry.z;
        float4 sum = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        for (uint32_t base = first; base < end; base += 4u) {   // four rows in flight: most points have two or four
            float4 v[4];
#pragma unroll
            for (uint32_t k = 0; k < 4u; ++k) {
                v[k] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                if (base + k < end && word < kWords)
                    v[k] = ((const float4*)(rows.values + (size_t)(base + k) * GradRows::words(C)))[word];
            }
#pragma unroll
            for (uint32_t k = 0; k < 4u; ++k) {
                const bool mine = base + k < end && __float_as_uint(v[k].y) == stamp.x && __float_as_uint(v[k].z) == stamp.y;
                if (!__shfl((int)mine, (int)tail_lane, 64)) continue;   // no such row, or one this pass has not written
                sum.x += v[k].x;
                sum.y += v[k].y;
                sum.z += v[k].z;
                sum.w += v[k].w;
            }
        }
        if (word < kWords - 1u) ((float4*)(grad_features + (size_t)point * C))[word] = sum;
        else if (word == kWords - 1u) grad_opacities[point] = sum.x;
    }
}

// Backward: the same walk with the saved final image (kernels.cu:476-579). A pixel leaves its blending weight and
// opacity gradient in the instance's slot; after the batch the instance's thread multiplies the weights with the
// pixels' image gradients (kept in LDS) and adds everything up: a plain store for a point with a single
// instance, a stamped row for k_grad_reduce otherwise.
template <int T, int C>
__global__ void __launch_bounds__(T * T)
    k_blend_backward(const uint2* __restrict__ ranges, const uint32_t* __restrict__ order,
                     const uint32_t* __restrict__ inst_points, const char* __restrict__ records, uint32_t stride,
                     const float* __restrict__ grad_image, const float* __restrict__ grad_alpha,
                     const float* __restrict__ image, const float* __restrict__ alpha_image, float* grad_features,
                     float* grad_opacities, GradRows grad_rows, int W, int H, uint32_t gw, float threshold, float reach2) {
    constexpr int TT = T * T;
    __shared__ Stage<T, C> st;
    __shared__ float s_d_opacity[TT][kSlotStride];   // per staged instance and box pixel: d loss / d opacity
    __shared__ float s_grad_px[TT][C + 1];       // image gradient of every pixel of the tile (padded rows)
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    const uint32_t tile = order[blockIdx.x];
    const Pixel px = pixel_of_thread<T>(tile, gw, W, H);
    const int tile_x0 = (int)(tile % gw) * T, tile_y0 = (int)(tile / gw) * T;
    const float cx = (float)px.x + 0.5f, cy = (float)px.y + 0.5f;
    // With s = features . grad of an instance, R the running sum of blending weight x s of the pixel and S its final
    // value, the reference's dot(T f + (F_running - F_final) / (1 - a), grad) + grad_alpha (1 - alpha_final) / (1 - a)
    // is T s + (R - S + grad_alpha (1 - alpha_final)) / (1 - a): the walk carries two scalars, not 2C.
    float g[C];
    float offset = 0.0f;   // grad_alpha (1 - alpha_final) - S
#pragma unroll
    for (int c = 0; c < C; ++c) g[c] = 0.0f;
    if (px.inside) {
        const size_t n_pixels = (size_t)W * H, pix = (size_t)px.y * W + px.x;
        float final_dot = 0.0f;
#pragma unroll
        for (int c = 0; c < C; ++c) {
            g[c] = grad_image[c * n_pixels + pix];
            final_dot = fmaf(image[c * n_pixels + pix], g[c], final_dot);
        }
        offset = grad_alpha[pix] * (1.0f - alpha_image[pix]) - final_dot;
    }
    float running = 0.0f;
    const uint2 stamp = *grad_rows.stamp;
    // per wave: what its pixels add to the gradient of the instance without slots that the block is at (C feature
    // gradients and the opacity gradient); two sets, so that the next such instance does not overwrite what the thread
    // of this one is still reading
    static_assert(C + 1 <= 2 * kSlots, "the sums of an instance without slots are kept in its two slot rows");
    __shared__ float s_big[2][TT / 64][C + 1];
    uint32_t big_parity = 0u;
#pragma unroll
    for (int c = 0; c < C; ++c) s_grad_px[px.ly * T + px.lx][c] = g[c];
    float tr = 1.0f;
    bool done = !px.inside;
    const uint2 range = ranges[tile];
    Ahead<C> ahead;
    ahead.start(inst_points, records, stride, range, TT);
    for (uint32_t base = range.x; base < range.y; base += TT) {
        if (__syncthreads_count(done) == TT) break;
        const uint32_t count = min((uint32_t)TT, range.y - base);
        uint32_t my_row = 0u;
        {
            const float4 h0 = ahead.h0, h1 = ahead.h1;
            float4 feat[C / 4];
#pragma unroll
            for (int q = 0; q < C / 4; ++q) feat[q] = ahead.f[q];
            if (base + TT + tid < range.y) ahead.request(records + (size_t)ahead.after * stride);
            if (base + 2u * TT + tid < range.y) ahead.after = inst_points[base + 2u * TT + tid];
            if (tid < count) {
                // the row of a point that touches several tiles is looked up now, long before it is needed: its
                // instances were created row-major over its tile bounds
                const uint32_t word = __float_as_uint(h1.w);
                if (word & kMultiTile) {
                    uint32_t columns = (word >> kColumnsShift) & kManyColumns;
                    if (columns == kManyColumns) {
                        const uint2 b = grad_rows.bounds[word & kPointMask];
                        columns = (b.x >> 16) - (b.x & 0xFFFFu);
                    }
                    my_row = __float_as_uint(h1.z) + (tile / gw) * columns + tile % gw;
                }
                stage_instance<T, C>(st, tid, h0, h1, feat, tile_x0, tile_y0, reach2, threshold);
            }
        }
        __syncthreads();
        {
            const bool wave_live = __ballot(!done) != 0ull;
            for (uint32_t first = 0; first < count; first += 64u) {
                const uint32_t at = first + lane;
                const uint32_t my_box = at < count ? st.box[at] : 0u;
                // the instances without slots of these 64, the same mask in every wave of the block
                const uint64_t big = __ballot(!has_slots(my_box));
                if (!wave_live && big == 0ull) continue;
                const uint64_t reach = __ballot(box_reaches(my_box, px));
                uint64_t over = reach != 0ull ? instances_over_pixel(my_box, px) : 0ull;
                if (done) over = 0ull;
                uint64_t now = 0ull;   // the part of `over` a walk is going through
                // blend instance j, whose footprint value at this pixel is G: blending weight and d loss / d opacity
                auto blend = [&](uint32_t j, float G, float& weight, float& d_opacity) {
                    const float a = st.head0[j].z * G;
                    const float bw = tr * a;
                    const float one_minus_a = 1.0f - a;
                    // hardware reciprocal (1 ulp): the gradients are compared to 1e-4, not to the bit
                    const float rcp = __builtin_amdgcn_rcpf(fmaxf(one_minus_a, kOneMinusAlphaEps));
                    float sd = 0.0f;
#pragma unroll
                    for (int q = 0; q < C / 4; ++q) {
                        const float4 f = st.feat[j * (C / 4) + q];
                        sd = fmaf(f.x, g[4 * q], sd);
                        sd = fmaf(f.y, g[4 * q + 1], sd);
                        sd = fmaf(f.z, g[4 * q + 2], sd);
                        sd = fmaf(f.w, g[4 * q + 3], sd);
                    }
                    running = fmaf(bw, sd, running);
                    const float d_alpha = fmaf(tr, sd, (running + offset) * rcp);
                    d_opacity = d_alpha * G;
                    weight = bw > 0.0f ? bw : 0.0f;
                    tr *= one_minus_a;
                    if (tr < kTransmittanceThreshold) {
                        done = true;
                        over = 0ull;
                        now = 0ull;
                    }
                };
                // in depth order: the instances with slots up to the next one without, lane by lane, then that one by
                // the whole block (the usual case has none of those and is a single walk)
                uint64_t big_left = big;
                for (;;) {
                    const uint32_t kb = big_left != 0ull ? (uint32_t)__builtin_ctzll(big_left) : 64u;
                    now = kb == 64u ? over : over & ((1ull << kb) - 1ull);
                    over &= ~now;
                    while (__ballot(now != 0ull) != 0ull) {
                        if (now != 0ull) {
                            const uint32_t j = first + (uint32_t)__builtin_ctzll(now);
                            now &= now - 1ull;
                            const int slot = slot_in(st.box[j], px.lx, px.ly);
                            const float G = st.value[j][slot];
                            if (G != 0.0f) {
                                float weight, d_opacity;
                                blend(j, G, weight, d_opacity);
                                st.value[j][slot] = -weight;
                                s_d_opacity[j][slot] = d_opacity;
                            }
                        }
                    }
                    if (kb == 64u) break;
                    big_left &= big_left - 1ull;
                    const uint32_t j = first + kb;
                    float weight = 0.0f, d_opacity = 0.0f, G;
                    if (((over >> kb) & 1ull) != 0ull && footprint_value(st.head0[j], st.head1[j], cx, cy, threshold, G))
                        blend(j, G, weight, d_opacity);
                    over &= ~(1ull << kb);
                    // what this wave's pixels add to the instance's gradient
#pragma unroll
                    for (int c = 0; c < C; ++c) {
                        const float wave_part = blend::wave_sum(weight * g[c]);
                        if (lane == 0u) s_big[big_parity][tid >> 6][c] = wave_part;
                    }
                    {
                        const float wave_part = blend::wave_sum(d_opacity);
                        if (lane == 0u) s_big[big_parity][tid >> 6][C] = wave_part;
                    }
                    __syncthreads();
                    if (tid == j) {   // the instance's thread: the waves' sums in wave order, kept in its unused slot rows
#pragma unroll
                        for (int c = 0; c <= C; ++c) {
                            float sum = 0.0f;
#pragma unroll
                            for (int q = 0; q < TT / 64; ++q) sum += s_big[big_parity][q][c];
                            if (c < kSlots) st.value[j][c] = sum;
                            else s_d_opacity[j][c - kSlots] = sum;
                        }
                    }
                    big_parity ^= 1u;
                }
            }
        }
        __syncthreads();
        if (tid < count) {
            const uint32_t box = st.box[tid];
            const uint32_t cols = box & 0xFFFFu, rows = box >> 16;
            const int w = __popc(cols), h = __popc(rows), x_lo = __ffs(cols) - 1, y_lo = __ffs(rows) - 1;
            if (w * h > 0) {
                float sum[C + 1];
#pragma unroll
                for (int c = 0; c <= C; ++c) sum[c] = 0.0f;
                if (w * h <= kSlots) {
                    int slot = 0;
                    for (int yy = 0; yy < h; ++yy) {
                        for (int xx = 0; xx < w; ++xx, ++slot) {
                            const float v = st.value[tid][slot];
                            if (!(__float_as_uint(v) >> 31)) continue;   // no pixel has blended it: still the footprint value
                            const float weight = -v;
                            const float* gp = s_grad_px[(y_lo + yy) * T + x_lo + xx];
#pragma unroll
                            for (int c = 0; c < C; ++c) sum[c] = fmaf(weight, gp[c], sum[c]);
                            sum[C] += s_d_opacity[tid][slot];
                        }
                    }
                } else {   // an instance without slots: added up when the block went through it
#pragma unroll
                    for (int c = 0; c <= C; ++c) sum[c] = c < kSlots ? st.value[tid][c] : s_d_opacity[tid][c - kSlots];
                }
                const uint32_t word = __float_as_uint(st.head1[tid].w);
                const uint32_t point = word & kPointMask;
                float* gf = grad_features + (size_t)point * C;
                if (word & kMultiTile) {
                    float4* out = (float4*)(grad_rows.values + (size_t)my_row * GradRows::words(C));
#pragma unroll
                    for (int q = 0; q < C / 4; ++q)
                        out[q] = make_float4(sum[4 * q], sum[4 * q + 1], sum[4 * q + 2], sum[4 * q + 3]);
                    out[C / 4] = make_float4(sum[C], __uint_as_float(stamp.x), __uint_as_float(stamp.y), 0.0f);
                } else {
#pragma unroll
                    for (int q = 0; q < C / 4; ++q)   // the rows are 16-byte aligned (checked by the host)
                        ((float4*)gf)[q] = make_float4(sum[4 * q], sum[4 * q + 1], sum[4 * q + 2], sum[4 * q + 3]);
                    grad_opacities[point] = sum[C];
                }
            }
        }
    }
}

}  // namespace gaussian
