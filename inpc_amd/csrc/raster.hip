// raster.hip — tile-based differentiable bilinear point rasterizer for gfx950.
//
// Pipeline (all on the caller's stream, counts stay on the device):
//   k_preprocess     project, cull, tile bounds, blend record, depth key, depth-digit histograms
//                    (B/rasterization/src/bilinear/kernels.cu:11-84,106-184)
//   radix sort       stable sort of the visible points by depth key; the first pass drops the
//                    culled points, in ascending point id (forward.cu:91-98)
//   k_expand         per depth-sorted point: instance offsets (single-pass scan) and one
//                    (tile, point) instance per touched tile, row-major; tile-digit histograms
//                    (kernels.cu:186-220, forward.cu:101-130)
//   radix sort       stable sort of the instances by tile id (forward.cu:132-139)
//   k_tile_ranges    [begin, end) of every tile (kernels.cu:222-239)
//   k_blend_forward  front-to-back bilinear 2x2 splat blend, one block per tile
//                    (kernels.cu:241-313,422-495)
//   k_blend_backward replay of the blend with the saved final image (kernels.cu:315-420)
//   k_sh_backward    view-space feature gradient -> 36 fp16 SH coefficient gradients
//                    (kernels.cu:86-104, sh_utils.cuh:44-62)
//
// The blend kernels do not test every pixel against every instance. For a batch of instances staged
// in LDS, each wave builds, with one ballot per tile column and per tile row, 64-bit masks of the
// instances whose footprint covers that column / row (the exact float test of the reference). A pixel
// ANDs its column and row mask and walks the set bits, i.e. exactly its own hits, in depth order.
#include <algorithm>
#include <cmath>
#include <cstring>

#include "common.hpp"
#include "radix.hpp"

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
    kCntTicketDepth = 4,   // 4 words
    kCntTicketTile = 8,    // 4 words
    kCntTicketExpand = 12,
    kCntWords = 16
};

// tileinfo word of the blend record
constexpr uint32_t kInfoValid = 1u << 18;
__device__ __forceinline__ uint32_t info_tile0(uint32_t info) { return info & 0xFFFFu; }
__device__ __forceinline__ uint32_t info_nx(uint32_t info) { return ((info >> 16) & 1u) + 1u; }
__device__ __forceinline__ uint32_t info_ny(uint32_t info) { return ((info >> 17) & 1u) + 1u; }
__device__ __forceinline__ uint32_t info_count(uint32_t info) {
    return (info & kInfoValid) ? info_nx(info) * info_ny(info) : 0u;
}

struct Geometry {
    uint32_t n;
    int W, H;
    uint32_t gw, gh, n_tiles;
    Camera cam;
    uint32_t key_bias;  // depth key = float bits - key_bias
};

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

// ---- preprocess -------------------------------------------------------------------------------------------
template <int T, int FMODE>
__global__ void __launch_bounds__(kBlock)
    k_preprocess(const float* __restrict__ positions, const void* __restrict__ features,
                 const float* __restrict__ opacities, const float* __restrict__ w2c,
                 const float* __restrict__ cam_position, float4* __restrict__ rec, float* __restrict__ depth_out,
                 float4* __restrict__ features_view, uint32_t* __restrict__ keys, float* __restrict__ blending_weights,
                 uint32_t* counters, uint32_t* g_hist, Geometry g, radix::DevicePlan plan) {
    __shared__ uint32_t s_hist[radix::kMaxPasses * radix::kRadix];
    __shared__ uint32_t s_visible, s_instances;
    for (int i = threadIdx.x; i < plan.n_passes * radix::kRadix; i += kBlock) s_hist[i] = 0u;
    if (threadIdx.x == 0) {
        s_visible = 0u;
        s_instances = 0u;
    }
    __syncthreads();
    const float4 r1 = make_float4(w2c[0], w2c[1], w2c[2], w2c[3]);
    const float4 r2 = make_float4(w2c[4], w2c[5], w2c[6], w2c[7]);
    const float4 r3 = make_float4(w2c[8], w2c[9], w2c[10], w2c[11]);
    const float fT = (float)T, fgw = (float)g.gw, fgh = (float)g.gh;
    uint32_t my_visible = 0, my_instances = 0;
    const uint32_t stride = gridDim.x * kBlock;
    for (uint32_t i = blockIdx.x * kBlock + threadIdx.x; i < g.n; i += stride) {
        const float px = positions[3 * (size_t)i], py = positions[3 * (size_t)i + 1], pz = positions[3 * (size_t)i + 2];
        const float depth = affine_row(r3, px, py, pz);
        uint32_t info = 0u, key = radix::kInvalidKey;
        float sx = 0.0f, sy = 0.0f, opacity = 0.0f;
        if (!(depth < g.cam.near_plane || depth > g.cam.far_plane)) {
            const float x = affine_row(r1, px, py, pz) / depth;
            const float y = affine_row(r2, px, py, pz) / depth;
            sx = x * g.cam.fx + g.cam.cx;
            sy = y * g.cam.fy + g.cam.cy;
            const uint32_t x0 = (uint32_t)fminf(fgw, fmaxf(0.0f, floorf((sx - 0.5f) / fT)));
            const uint32_t x1 = (uint32_t)fminf(fgw, fmaxf(0.0f, ceilf((sx + 0.5f) / fT)));
            const uint32_t y0 = (uint32_t)fminf(fgh, fmaxf(0.0f, floorf((sy - 0.5f) / fT)));
            const uint32_t y1 = (uint32_t)fminf(fgh, fmaxf(0.0f, ceilf((sy + 0.5f) / fT)));
            const uint32_t touched = (x1 - x0) * (y1 - y0);
            if (touched != 0u) {
                info = (y0 * g.gw + x0) | ((x1 - x0 - 1u) << 16) | ((y1 - y0 - 1u) << 17) | kInfoValid;
                key = __float_as_uint(depth) - g.key_bias;
                my_visible += 1u;
                my_instances += touched;
                radix::hist_add(s_hist, plan, key);
                if (FMODE == INPC_FEAT_SH36_F16) {
                    const ShBasis s = sh_basis(px, py, pz, cam_position);
                    features_view[i] = sh_to_view(s, (const __half*)features + 36 * (size_t)i);
                    opacity = opacities[i];
                } else if (FMODE == INPC_FEAT_RAW37_F16) {
                    const __half* raw = (const __half*)features + 37 * (size_t)i;
                    const ShBasis s = sh_basis(px, py, pz, cam_position);
                    features_view[i] = sh_to_view(s, raw + 1);
                    opacity = 1.0f - expf(-expf(__half2float(raw[0])));
                } else {
                    opacity = opacities[i];
                }
            }
        }
        rec[i] = make_float4(sx, sy, opacity, __uint_as_float(info));
        depth_out[i] = depth;
        keys[i] = key;
        if (blending_weights) blending_weights[i] = 0.0f;
    }
    // block totals -> one global atomic each
    for (int s = 32; s > 0; s >>= 1) {
        my_visible += __shfl_down(my_visible, s, 64);
        my_instances += __shfl_down(my_instances, s, 64);
    }
    if ((threadIdx.x & 63u) == 0u) {
        atomicAdd(&s_visible, my_visible);
        atomicAdd(&s_instances, my_instances);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        if (s_visible) atomicAdd(&counters[kCntVisible], s_visible);
        if (s_instances) atomicAdd(&counters[kCntInstances], s_instances);
    }
    radix::hist_flush(s_hist, plan, g_hist);
}

// ---- instance expansion -----------------------------------------------------------------------------------
constexpr int kExpandItems = 4;
constexpr int kExpandTile = kBlock * kExpandItems;

__global__ void __launch_bounds__(kBlock)
    k_expand(const uint32_t* __restrict__ depth_order, const float4* __restrict__ rec, uint16_t* __restrict__ inst_keys,
             uint32_t* __restrict__ inst_points, uint32_t* counters, uint32_t* status, uint32_t* g_hist, uint32_t gw,
             radix::DevicePlan plan) {
    __shared__ uint32_t s_hist[radix::kMaxPasses * radix::kRadix];
    __shared__ uint32_t s_wave[kBlock / kWave];
    __shared__ uint32_t s_bid, s_exclusive;
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    for (int i = tid; i < plan.n_passes * radix::kRadix; i += kBlock) s_hist[i] = 0u;
    if (tid == 0) s_bid = atomicAdd(&counters[kCntTicketExpand], 1u);
    __syncthreads();
    const uint32_t bid = s_bid;
    const uint32_t n_visible = counters[kCntVisible];
    const uint64_t first = (uint64_t)bid * kExpandTile + (uint64_t)tid * kExpandItems;
    if ((uint64_t)bid * kExpandTile >= n_visible) return;

    uint32_t point[kExpandItems], info[kExpandItems];
    uint32_t mine = 0;
#pragma unroll
    for (int j = 0; j < kExpandItems; ++j) {
        point[j] = 0u;
        info[j] = 0u;
        if (first + j < n_visible) {
            point[j] = depth_order[first + j];
            info[j] = __float_as_uint(rec[point[j]].w);
        }
        mine += info_count(info[j]);
    }
    // block exclusive scan of `mine`
    uint32_t incl = mine;
#pragma unroll
    for (int s = 1; s < 64; s <<= 1) {
        const uint32_t up = __shfl_up(incl, s, 64);
        if (lane >= (uint32_t)s) incl += up;
    }
    if (lane == 63) s_wave[wave] = incl;
    __syncthreads();
    uint32_t wave_off = 0, block_total = 0;
#pragma unroll
    for (int w = 0; w < kBlock / kWave; ++w) {
        const uint32_t c = s_wave[w];
        if ((uint32_t)w < wave) wave_off += c;
        block_total += c;
    }
    if (tid == 0) s_exclusive = lookback_exclusive(status, 1u, bid, block_total, &counters[kCntError]);
    __syncthreads();
    uint32_t offset = s_exclusive + wave_off + incl - mine;
#pragma unroll
    for (int j = 0; j < kExpandItems; ++j) {
        if (!(info[j] & kInfoValid)) continue;
        const uint32_t tile0 = info_tile0(info[j]), nx = info_nx(info[j]), ny = info_ny(info[j]);
        for (uint32_t dy = 0; dy < ny; ++dy)
            for (uint32_t dx = 0; dx < nx; ++dx) {
                const uint32_t tile = tile0 + dy * gw + dx;
                inst_keys[offset] = (uint16_t)tile;
                inst_points[offset] = point[j];
                radix::hist_add(s_hist, plan, tile);
                ++offset;
            }
    }
    __syncthreads();
    radix::hist_flush(s_hist, plan, g_hist);
}

// ---- tile ranges (kernels.cu:222-239) ------------------------------------------------------------------------
__global__ void __launch_bounds__(kBlock) k_tile_ranges(const uint16_t* __restrict__ inst_keys, uint2* ranges,
                                                        const uint32_t* __restrict__ counters, uint32_t n_max) {
    const uint32_t n = min(counters[kCntInstances], n_max);
    const uint32_t stride = gridDim.x * kBlock;
    for (uint32_t i = blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) {
        const uint32_t t = inst_keys[i];
        if (i == 0) {
            ranges[t].x = 0u;
        } else {
            const uint32_t prev = inst_keys[i - 1];
            if (prev != t) {
                ranges[prev].y = i;
                ranges[t].x = i;
            }
        }
        if (i == n - 1) ranges[t].y = n;
    }
}

// ---- blend -------------------------------------------------------------------------------------------------
constexpr int kBatch = 256;            // instances staged per round
constexpr int kWords = kBatch / kWave; // 64-bit mask words per column / row

template <int FMODE, int C>
__device__ __forceinline__ void load_features(float* dst, const void* __restrict__ features,
                                              const float4* __restrict__ features_view, uint32_t point) {
    if (FMODE == INPC_FEAT_SH36_F16 || FMODE == INPC_FEAT_RAW37_F16) {
        const float4 f = features_view[point];
        dst[0] = f.x;
        dst[1] = f.y;
        dst[2] = f.z;
        dst[3] = f.w;
    } else if (FMODE == INPC_FEAT_DIRECT_F32) {
        const float4* src = (const float4*)features + (size_t)point * (C / 4);
#pragma unroll
        for (int q = 0; q < C / 4; ++q) {
            const float4 f = src[q];
            dst[4 * q] = f.x;
            dst[4 * q + 1] = f.y;
            dst[4 * q + 2] = f.z;
            dst[4 * q + 3] = f.w;
        }
    } else {
        const __half* src = (const __half*)features + (size_t)point * C;
#pragma unroll
        for (int c = 0; c < C; ++c) dst[c] = __half2float(src[c]);
    }
}

// Pixel of thread `tid` inside a T x T tile: a wave always covers an 8x8 quad.
template <int T>
__device__ __forceinline__ void pixel_of_thread(uint32_t tid, int& lx, int& ly) {
    const uint32_t lane = tid & 63u, wave = tid >> 6;
    lx = (int)(lane & 7u);
    ly = (int)(lane >> 3);
    if (T == 16) {
        lx += (int)(wave & 1u) * 8;
        ly += (int)(wave >> 1) * 8;
    }
}

// Stage one batch: records and features into LDS, then the column / row coverage masks.
template <int T, int C, int FMODE, bool NEED_DEPTH>
__device__ __forceinline__ void stage_batch(uint32_t begin, uint32_t count, const uint32_t* __restrict__ inst_points,
                                            const float4* __restrict__ rec, const void* __restrict__ features,
                                            const float4* __restrict__ features_view,
                                            const float* __restrict__ depth, int tile_x0, int tile_y0,
                                            uint32_t* s_point, float2* s_xy, float* s_opacity, uint32_t* s_multi,
                                            float* s_feat, float* s_depth, uint64_t (*s_col)[kWords],
                                            uint64_t (*s_row)[kWords]) {
    constexpr int TT = T * T;
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    for (uint32_t j = tid; j < (uint32_t)kBatch; j += TT) {
        float sx = 0.0f, sy = 0.0f;
        const bool valid = j < count;
        if (valid) {
            const uint32_t p = inst_points[begin + j];
            const float4 r = rec[p];
            sx = r.x;
            sy = r.y;
            s_point[j] = p;
            s_xy[j] = make_float2(sx, sy);
            s_opacity[j] = r.z;
            const uint32_t info = __float_as_uint(r.w);
            s_multi[j] = (info >> 16) & 3u;
            float f[C];
            load_features<FMODE, C>(f, features, features_view, p);
#pragma unroll
            for (int c = 0; c < C; ++c) s_feat[j * C + c] = f[c];
            if (NEED_DEPTH) s_depth[j] = depth[p];
        }
        // j / 64 is uniform over the wave: one mask word per ballot
        const uint32_t word = j >> 6;
        uint64_t mine = 0;
#pragma unroll
        for (int x = 0; x < T; ++x) {
            const float d = fabsf(sx - ((float)(tile_x0 + x) + 0.5f));
            const uint64_t m = __ballot(valid && !(d >= 1.0f));
            if (lane == (uint32_t)x) mine = m;
        }
#pragma unroll
        for (int y = 0; y < T; ++y) {
            const float d = fabsf(sy - ((float)(tile_y0 + y) + 0.5f));
            const uint64_t m = __ballot(valid && !(d >= 1.0f));
            if (lane == (uint32_t)(32 + y)) mine = m;
        }
        if (lane < (uint32_t)T) s_col[lane][word] = mine;
        if (lane >= 32u && lane < (uint32_t)(32 + T)) s_row[lane - 32u][word] = mine;
    }
}

template <int T, int C, int FMODE, bool INFERENCE>
__global__ void __launch_bounds__(T* T)
    k_blend_forward(const uint2* __restrict__ ranges, const uint32_t* __restrict__ inst_points,
                    const float4* __restrict__ rec, const void* __restrict__ features,
                    const float4* __restrict__ features_view, const float* __restrict__ depth,
                    float* __restrict__ image, float* __restrict__ alpha_image, float* blending_weights,
                    float* __restrict__ depth_image, int W, int H, uint32_t gw) {
    constexpr int TT = T * T;
    __shared__ uint32_t s_point[kBatch];
    __shared__ float2 s_xy[kBatch];
    __shared__ float s_opacity[kBatch];
    __shared__ uint32_t s_multi[kBatch];
    __shared__ float s_feat[kBatch * C];
    __shared__ float s_depth[INFERENCE ? kBatch : 1];
    __shared__ float s_acc[INFERENCE ? 1 : kBatch];
    __shared__ uint64_t s_col[T][kWords];
    __shared__ uint64_t s_row[T][kWords];

    const uint32_t tid = threadIdx.x;
    const uint32_t tile = blockIdx.x;
    const int tile_x0 = (int)(tile % gw) * T, tile_y0 = (int)(tile / gw) * T;
    int lx, ly;
    pixel_of_thread<T>(tid, lx, ly);
    const int px = tile_x0 + lx, py = tile_y0 + ly;
    const bool inside = px < W && py < H;
    const float pcx = (float)px + 0.5f, pcy = (float)py + 0.5f;

    float F[C];
#pragma unroll
    for (int c = 0; c < C; ++c) F[c] = 0.0f;
    float D = 0.0f, Tr = 1.0f;
    bool done = !inside;

    const uint2 range = ranges[tile];
    for (uint32_t begin = range.x; begin < range.y; begin += kBatch) {
        const uint32_t count = min((uint32_t)kBatch, range.y - begin);
        if (!INFERENCE)
            for (uint32_t j = tid; j < (uint32_t)kBatch; j += TT) s_acc[j] = 0.0f;
        stage_batch<T, C, FMODE, INFERENCE>(begin, count, inst_points, rec, features, features_view, depth, tile_x0,
                                            tile_y0, s_point, s_xy, s_opacity, s_multi, s_feat, s_depth, s_col, s_row);
        __syncthreads();
        if (!done) {
            const uint32_t n_words = (count + 63u) >> 6;
            for (uint32_t w = 0; w < n_words && !done; ++w) {
                uint64_t m = s_col[lx][w] & s_row[ly][w];
                while (m) {
                    const uint32_t j = (w << 6) + (uint32_t)__builtin_ctzll(m);
                    m &= m - 1;
                    const float2 xy = s_xy[j];
                    const float dx = fabsf(xy.x - pcx), dy = fabsf(xy.y - pcy);
                    const float wgt = __saturatef(1.0f - dx) * __saturatef(1.0f - dy);
                    const float a = s_opacity[j] * wgt;
                    const float bw = Tr * a;
                    if (!INFERENCE) {
                        if (bw > 0.0f) atomicAdd(&s_acc[j], bw * wgt);
                    }
#pragma unroll
                    for (int c = 0; c < C; ++c) F[c] = fmaf(bw, s_feat[j * C + c], F[c]);
                    if (INFERENCE) D = fmaf(bw, s_depth[j], D);
                    Tr *= 1.0f - a;
                    if (Tr < kTransmittanceThreshold) {
                        done = true;
                        break;
                    }
                }
            }
        }
        __syncthreads();
        if (!INFERENCE) {
            for (uint32_t j = tid; j < count; j += TT) {
                const float v = s_acc[j];
                if (v != 0.0f) {
                    if (s_multi[j]) atomicAdd(&blending_weights[s_point[j]], v);
                    else blending_weights[s_point[j]] = v;
                }
            }
        }
        if (__syncthreads_and(done)) break;
    }
    if (inside) {
        const size_t n_pixels = (size_t)W * H, pix = (size_t)py * W + px;
#pragma unroll
        for (int c = 0; c < C; ++c) image[c * n_pixels + pix] = F[c];
        const float alpha_px = 1.0f - Tr;
        alpha_image[pix] = Tr < kTransmittanceThreshold ? 1.0f : alpha_px;
        if (INFERENCE) depth_image[pix] = alpha_px > 0.0f ? D / alpha_px : 0.0f;
    }
}

template <int T, int C, int FMODE>
__global__ void __launch_bounds__(T* T)
    k_blend_backward(const uint2* __restrict__ ranges, const uint32_t* __restrict__ inst_points,
                     const float4* __restrict__ rec, const void* __restrict__ features,
                     const float4* __restrict__ features_view, const float* __restrict__ grad_image,
                     const float* __restrict__ grad_alpha, const float* __restrict__ image,
                     const float* __restrict__ alpha_image, float* grad_view, float* grad_opacities, int W, int H,
                     uint32_t gw) {
    constexpr int TT = T * T;
    __shared__ uint32_t s_point[kBatch];
    __shared__ float2 s_xy[kBatch];
    __shared__ float s_opacity[kBatch];
    __shared__ uint32_t s_multi[kBatch];
    __shared__ float s_feat[kBatch * C];
    __shared__ float s_gfeat[kBatch * C];
    __shared__ float s_gop[kBatch];
    __shared__ uint64_t s_col[T][kWords];
    __shared__ uint64_t s_row[T][kWords];

    const uint32_t tid = threadIdx.x;
    const uint32_t tile = blockIdx.x;
    const int tile_x0 = (int)(tile % gw) * T, tile_y0 = (int)(tile / gw) * T;
    int lx, ly;
    pixel_of_thread<T>(tid, lx, ly);
    const int px = tile_x0 + lx, py = tile_y0 + ly;
    const bool inside = px < W && py < H;
    const float pcx = (float)px + 0.5f, pcy = (float)py + 0.5f;

    float G[C], Ffin[C], Fnew[C];
    float common = 0.0f;
#pragma unroll
    for (int c = 0; c < C; ++c) {
        G[c] = 0.0f;
        Ffin[c] = 0.0f;
        Fnew[c] = 0.0f;
    }
    if (inside) {
        const size_t n_pixels = (size_t)W * H, pix = (size_t)py * W + px;
#pragma unroll
        for (int c = 0; c < C; ++c) {
            G[c] = grad_image[c * n_pixels + pix];
            Ffin[c] = image[c * n_pixels + pix];
        }
        common = grad_alpha[pix] * (1.0f - alpha_image[pix]);
    }
    float Tr = 1.0f;
    bool done = !inside;

    const uint2 range = ranges[tile];
    for (uint32_t begin = range.x; begin < range.y; begin += kBatch) {
        const uint32_t count = min((uint32_t)kBatch, range.y - begin);
        for (uint32_t j = tid; j < (uint32_t)kBatch; j += TT) s_gop[j] = 0.0f;
        for (uint32_t j = tid; j < (uint32_t)(kBatch * C); j += TT) s_gfeat[j] = 0.0f;
        stage_batch<T, C, FMODE, false>(begin, count, inst_points, rec, features, features_view, nullptr, tile_x0,
                                        tile_y0, s_point, s_xy, s_opacity, s_multi, s_feat, nullptr, s_col, s_row);
        __syncthreads();
        if (!done) {
            const uint32_t n_words = (count + 63u) >> 6;
            for (uint32_t w = 0; w < n_words && !done; ++w) {
                uint64_t m = s_col[lx][w] & s_row[ly][w];
                while (m) {
                    const uint32_t j = (w << 6) + (uint32_t)__builtin_ctzll(m);
                    m &= m - 1;
                    const float2 xy = s_xy[j];
                    const float dx = fabsf(xy.x - pcx), dy = fabsf(xy.y - pcy);
                    const float wgt = __saturatef(1.0f - dx) * __saturatef(1.0f - dy);
                    const float a = s_opacity[j] * wgt;
                    const float bw = Tr * a;
                    const float one_minus_a = 1.0f - a;
                    const float rcp = 1.0f / fmaxf(one_minus_a, kOneMinusAlphaEps);
                    float dot = 0.0f;
#pragma unroll
                    for (int c = 0; c < C; ++c) {
                        const float f = s_feat[j * C + c];
                        if (bw > 0.0f) atomicAdd(&s_gfeat[j * C + c], bw * G[c]);
                        Fnew[c] = fmaf(bw, f, Fnew[c]);
                        dot = fmaf(fmaf(Tr, f, (Fnew[c] - Ffin[c]) * rcp), G[c], dot);
                    }
                    const float d_alpha = fmaf(common, rcp, dot);
                    const float d_op = d_alpha * wgt;
                    if (d_op != 0.0f) atomicAdd(&s_gop[j], d_op);
                    Tr *= one_minus_a;
                    if (Tr < kTransmittanceThreshold) {
                        done = true;
                        break;
                    }
                }
            }
        }
        __syncthreads();
        for (uint32_t e = tid; e < count * C; e += TT) {
            const uint32_t j = e / C, c = e % C;
            const float v = s_gfeat[e];
            if (v != 0.0f) {
                float* dst = grad_view + (size_t)s_point[j] * C + c;
                if (s_multi[j]) atomicAdd(dst, v);
                else *dst = v;
            }
        }
        for (uint32_t j = tid; j < count; j += TT) {
            const float v = s_gop[j];
            if (v != 0.0f) {
                if (s_multi[j]) atomicAdd(&grad_opacities[s_point[j]], v);
                else grad_opacities[s_point[j]] = v;
            }
        }
        if (__syncthreads_and(done)) break;
    }
}

// view-space feature gradient -> (N,36) fp16, zero where the point was not drawn
__global__ void __launch_bounds__(kBlock)
    k_sh_backward(const float* __restrict__ positions, const float* __restrict__ cam_position,
                  const float4* __restrict__ rec, const float4* __restrict__ grad_view, __half* __restrict__ grad_features,
                  uint32_t n) {
    const uint32_t i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    __half* out = grad_features + 36 * (size_t)i;
    const uint32_t info = __float_as_uint(rec[i].w);
    if (!(info & kInfoValid)) {
#pragma unroll
        for (int k = 0; k < 36; ++k) out[k] = __float2half_rn(0.0f);
        return;
    }
    const ShBasis s = sh_basis(positions[3 * (size_t)i], positions[3 * (size_t)i + 1], positions[3 * (size_t)i + 2],
                               cam_position);
    const float4 g = grad_view[i];
#pragma unroll
    for (int k = 0; k < 9; ++k) {
        out[4 * k + 0] = __float2half_rn(s.b[k] * g.x);
        out[4 * k + 1] = __float2half_rn(s.b[k] * g.y);
        out[4 * k + 2] = __float2half_rn(s.b[k] * g.z);
        out[4 * k + 3] = __float2half_rn(s.b[k] * g.w);
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
    radix::PassPlan depth_plan, tile_plan;
    int T, C, fmode;
    bool inference, sh;
    // private offsets
    size_t zero_begin, zero_words;  // region cleared at the start of every forward
    size_t hist_depth, hist_tile, bases_depth, bases_tile;
    size_t status_depth, status_tile, status_expand;
    size_t keys_a, keys_b, vals_a, vals_b;
    size_t inst_keys_a, inst_keys_b, inst_vals_a, inst_vals_b;
};

uint32_t float_bits(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
}

int make_layout(const inpc_raster_config* cfg, Layout& L) {
    if (!cfg) return fail(INPC_E_INVALID_ARGUMENT, "raster: config is null");
    const inpc_camera& cam = cfg->cam;
    if (cfg->tile != 8 && cfg->tile != 16) return fail(INPC_E_INVALID_ARGUMENT, "raster: tile must be 8 or 16");
    if (cam.width <= 0 || cam.height <= 0) return fail(INPC_E_INVALID_ARGUMENT, "raster: empty image");
    if (cfg->n_points >= (1u << 28)) return fail(INPC_E_UNSUPPORTED, "raster: n_points must be below 2^28");
    L.T = cfg->tile;
    L.fmode = cfg->feature_mode;
    L.sh = L.fmode == INPC_FEAT_SH36_F16 || L.fmode == INPC_FEAT_RAW37_F16;
    if (L.fmode < 0 || L.fmode > 3) return fail(INPC_E_UNSUPPORTED, "raster: unknown feature mode %d", L.fmode);
    L.C = L.sh ? 4 : cfg->channels;
    if (L.C != 4 && L.C != 8 && L.C != 16) return fail(INPC_E_INVALID_ARGUMENT, "raster: channels must be 4, 8 or 16");
    L.inference = (cfg->flags & INPC_RASTER_INFERENCE) != 0;
    Geometry& g = L.geo;
    g.n = cfg->n_points;
    g.W = cam.width;
    g.H = cam.height;
    g.gw = (uint32_t)((cam.width + L.T - 1) / L.T);
    g.gh = (uint32_t)((cam.height + L.T - 1) / L.T);
    g.n_tiles = g.gw * g.gh;
    if (g.n_tiles > 65536u)
        return fail(INPC_E_UNSUPPORTED, "raster: %u tiles exceed the 16-bit tile key (65536)", g.n_tiles);
    g.cam = to_device_camera(cam);
    // depth keys of drawn points lie in [bits(near), bits(far)] when 0 < near <= far: sort on the offset
    int depth_bits = 32;
    g.key_bias = 0u;
    if (cam.near_plane > 0.0f && cam.far_plane >= cam.near_plane && cam.far_plane < INFINITY) {
        g.key_bias = float_bits(cam.near_plane);
        depth_bits = std::max(1, bit_length(float_bits(cam.far_plane) - g.key_bias));
    }
    L.depth_plan = radix::make_plan(depth_bits);
    const int end_bit = bit_length(g.n_tiles - 1);
    L.tile_plan = radix::make_plan(std::max(end_bit, 1));

    const size_t n = std::max<size_t>(g.n, 1), ni = 4 * n;
    size_t off = 0;
    auto take = [&](size_t bytes) {
        const size_t o = off;
        off += align_up(bytes, 256);
        return o;
    };
    inpc_raster_layout& P = L.pub;
    memset(&P, 0, sizeof(P));
    // zeroed region: counters, histograms, look-back status, tile ranges
    L.zero_begin = off;
    P.counters = take(kCntWords * 4);
    L.hist_depth = take(radix::kMaxPasses * radix::kRadix * 4);
    L.hist_tile = take(radix::kMaxPasses * radix::kRadix * 4);
    L.status_depth = take(L.depth_plan.n_passes * radix::status_words(g.n) * 4);
    L.status_tile = take(L.tile_plan.n_passes * radix::status_words((uint32_t)std::min<size_t>(ni, 0xFFFFFFFFu)) * 4);
    L.status_expand = take((size_t)div_up(g.n, kExpandTile) * 4 + 4);
    P.tile_ranges = take((size_t)g.n_tiles * 8);
    L.zero_words = (off - L.zero_begin) / 4;
    L.bases_depth = take(radix::kMaxPasses * radix::kRadix * 4);
    L.bases_tile = take(radix::kMaxPasses * radix::kRadix * 4);
    P.point_record = take(n * 16);
    P.point_depth = take(n * 4);
    P.features_view = L.sh ? take(n * 16) : 0;
    L.keys_a = take(n * 4);
    L.keys_b = take(n * 4);
    L.vals_a = take(n * 4);
    L.vals_b = take(n * 4);
    L.inst_keys_a = take(ni * 2);
    L.inst_keys_b = take(ni * 2);
    L.inst_vals_a = take(ni * 4);
    L.inst_vals_b = take(ni * 4);
    const bool depth_in_a = (L.depth_plan.n_passes % 2) == 0;
    P.depth_keys = depth_in_a ? L.keys_a : L.keys_b;
    P.depth_order = depth_in_a ? L.vals_a : L.vals_b;
    const bool tile_in_a = (L.tile_plan.n_passes % 2) == 0;
    P.instance_keys = tile_in_a ? L.inst_keys_a : L.inst_keys_b;
    P.instance_points = tile_in_a ? L.inst_vals_a : L.inst_vals_b;
    P.total_bytes = off;
    P.grid_width = g.gw;
    P.grid_height = g.gh;
    P.n_tiles = g.n_tiles;
    P.end_bit = (uint32_t)end_bit;
    P.depth_key_bias = g.key_bias;
    return INPC_OK;
}

template <typename Tp>
Tp* at(void* ws, size_t off) {
    return (Tp*)((char*)ws + off);
}

template <int T, int FMODE>
int launch_preprocess(const Layout& L, const float* positions, const void* features, const float* opacities,
                      const float* w2c, const float* cam_position, float* blending_weights, void* ws,
                      hipStream_t stream) {
    const uint32_t blocks = std::min<uint32_t>(div_up(L.geo.n, kBlock), 2048u);
    INPC_LAUNCH("raster_preprocess", (k_preprocess<T, FMODE>), dim3(blocks), dim3(kBlock), stream, positions, features,
                opacities, w2c, cam_position, at<float4>(ws, L.pub.point_record), at<float>(ws, L.pub.point_depth),
                L.sh ? at<float4>(ws, L.pub.features_view) : (float4*)nullptr, at<uint32_t>(ws, L.keys_a),
                blending_weights, at<uint32_t>(ws, L.pub.counters), at<uint32_t>(ws, L.hist_depth), L.geo,
                radix::to_device_plan(L.depth_plan));
    return INPC_OK;
}

template <int T, int C, int FMODE>
int launch_blend_forward(const Layout& L, const void* features, float* image, float* alpha, float* blending_weights,
                         float* depth_image, void* ws, hipStream_t stream) {
    const uint2* ranges = at<uint2>(ws, L.pub.tile_ranges);
    const uint32_t* inst = at<uint32_t>(ws, L.pub.instance_points);
    const float4* rec = at<float4>(ws, L.pub.point_record);
    const float4* fview = L.sh ? at<float4>(ws, L.pub.features_view) : (const float4*)nullptr;
    const float* depth = at<float>(ws, L.pub.point_depth);
    if (L.inference) {
        INPC_LAUNCH("raster_blend_inference", (k_blend_forward<T, C, FMODE, true>), dim3(L.geo.n_tiles), dim3(T * T),
                    stream, ranges, inst, rec, features, fview, depth, image, alpha, (float*)nullptr, depth_image,
                    L.geo.W, L.geo.H, L.geo.gw);
    } else {
        INPC_LAUNCH("raster_blend_forward", (k_blend_forward<T, C, FMODE, false>), dim3(L.geo.n_tiles), dim3(T * T),
                    stream, ranges, inst, rec, features, fview, depth, image, alpha, blending_weights,
                    (float*)nullptr, L.geo.W, L.geo.H, L.geo.gw);
    }
    return INPC_OK;
}

template <int T, int C, int FMODE>
int launch_blend_backward(const Layout& L, const void* features, const float* grad_image, const float* grad_alpha,
                          const float* image, const float* alpha, float* grad_view, float* grad_opacities, void* ws,
                          hipStream_t stream) {
    INPC_LAUNCH("raster_blend_backward", (k_blend_backward<T, C, FMODE>), dim3(L.geo.n_tiles), dim3(T * T), stream,
                at<uint2>(ws, L.pub.tile_ranges), at<uint32_t>(ws, L.pub.instance_points),
                at<float4>(ws, L.pub.point_record), features,
                L.sh ? at<float4>(ws, L.pub.features_view) : (const float4*)nullptr, grad_image, grad_alpha, image,
                alpha, grad_view, grad_opacities, L.geo.W, L.geo.H, L.geo.gw);
    return INPC_OK;
}

// dispatch on (tile, channels, feature mode)
#define INPC_DISPATCH_TC(FM, CALL)                                        \
    do {                                                                  \
        if (L.T == 8 && L.C == 4) return CALL(8, 4, FM);                  \
        if (L.T == 8 && L.C == 8) return CALL(8, 8, FM);                  \
        if (L.T == 8 && L.C == 16) return CALL(8, 16, FM);                \
        if (L.T == 16 && L.C == 4) return CALL(16, 4, FM);                \
        if (L.T == 16 && L.C == 8) return CALL(16, 8, FM);                \
        if (L.T == 16 && L.C == 16) return CALL(16, 16, FM);              \
    } while (0)

int dispatch_blend_forward(const Layout& L, const void* features, float* image, float* alpha, float* bw,
                           float* depth_image, void* ws, hipStream_t stream) {
#define CALL_FWD(T_, C_, FM_) launch_blend_forward<T_, C_, FM_>(L, features, image, alpha, bw, depth_image, ws, stream)
    switch (L.fmode) {
        case INPC_FEAT_SH36_F16:
            if (L.T == 8) return CALL_FWD(8, 4, INPC_FEAT_SH36_F16);
            return CALL_FWD(16, 4, INPC_FEAT_SH36_F16);
        case INPC_FEAT_RAW37_F16:
            if (L.T == 8) return CALL_FWD(8, 4, INPC_FEAT_RAW37_F16);
            return CALL_FWD(16, 4, INPC_FEAT_RAW37_F16);
        case INPC_FEAT_DIRECT_F32:
            INPC_DISPATCH_TC(INPC_FEAT_DIRECT_F32, CALL_FWD);
            break;
        case INPC_FEAT_DIRECT_F16:
            INPC_DISPATCH_TC(INPC_FEAT_DIRECT_F16, CALL_FWD);
            break;
    }
#undef CALL_FWD
    return fail(INPC_E_UNSUPPORTED, "raster: unsupported blend configuration");
}

int dispatch_blend_backward(const Layout& L, const void* features, const float* grad_image, const float* grad_alpha,
                            const float* image, const float* alpha, float* grad_view, float* grad_opacities, void* ws,
                            hipStream_t stream) {
#define CALL_BWD(T_, C_, FM_) \
    launch_blend_backward<T_, C_, FM_>(L, features, grad_image, grad_alpha, image, alpha, grad_view, grad_opacities, ws, stream)
    switch (L.fmode) {
        case INPC_FEAT_SH36_F16:
            if (L.T == 8) return CALL_BWD(8, 4, INPC_FEAT_SH36_F16);
            return CALL_BWD(16, 4, INPC_FEAT_SH36_F16);
        case INPC_FEAT_DIRECT_F32:
            INPC_DISPATCH_TC(INPC_FEAT_DIRECT_F32, CALL_BWD);
            break;
        case INPC_FEAT_DIRECT_F16:
            INPC_DISPATCH_TC(INPC_FEAT_DIRECT_F16, CALL_BWD);
            break;
    }
#undef CALL_BWD
    return fail(INPC_E_UNSUPPORTED, "raster: unsupported backward configuration");
}

int dispatch_preprocess(const Layout& L, const float* positions, const void* features, const float* opacities,
                        const float* w2c, const float* cam_position, float* bw, void* ws, hipStream_t stream) {
#define CALL_PRE(T_, FM_) launch_preprocess<T_, FM_>(L, positions, features, opacities, w2c, cam_position, bw, ws, stream)
    switch (L.fmode) {
        case INPC_FEAT_SH36_F16:
            return L.T == 8 ? CALL_PRE(8, INPC_FEAT_SH36_F16) : CALL_PRE(16, INPC_FEAT_SH36_F16);
        case INPC_FEAT_RAW37_F16:
            return L.T == 8 ? CALL_PRE(8, INPC_FEAT_RAW37_F16) : CALL_PRE(16, INPC_FEAT_RAW37_F16);
        default:
            // the direct modes do not touch the features here
            return L.T == 8 ? CALL_PRE(8, INPC_FEAT_DIRECT_F32) : CALL_PRE(16, INPC_FEAT_DIRECT_F32);
    }
#undef CALL_PRE
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

    rc = fill_u32(at<uint32_t>(ws, L.zero_begin), 0u, L.zero_words, stream);
    if (rc != INPC_OK) return rc;
    uint32_t* counters = at<uint32_t>(ws, L.pub.counters);
    if (L.geo.n > 0) {
        rc = dispatch_preprocess(L, positions, features, opacities, w2c, cam_position,
                                 L.inference ? nullptr : blending_weights, ws, stream);
        if (rc != INPC_OK) return rc;
        rc = radix::sort_pairs<uint32_t>(L.depth_plan, true, at<uint32_t>(ws, L.keys_a), at<uint32_t>(ws, L.vals_a),
                                         at<uint32_t>(ws, L.keys_b), at<uint32_t>(ws, L.vals_b),
                                         counters + kCntVisible, L.geo.n, at<uint32_t>(ws, L.hist_depth),
                                         at<uint32_t>(ws, L.bases_depth), at<uint32_t>(ws, L.status_depth),
                                         counters + kCntTicketDepth, counters + kCntError, stream, "raster_depth_sort");
        if (rc != INPC_OK) return rc;
        INPC_LAUNCH("raster_expand", k_expand, dim3(div_up(L.geo.n, kExpandTile)), dim3(kBlock), stream,
                    (const uint32_t*)at<uint32_t>(ws, L.pub.depth_order), (const float4*)at<float4>(ws, L.pub.point_record),
                    at<uint16_t>(ws, L.inst_keys_a), at<uint32_t>(ws, L.inst_vals_a), counters,
                    at<uint32_t>(ws, L.status_expand), at<uint32_t>(ws, L.hist_tile), L.geo.gw,
                    radix::to_device_plan(L.tile_plan));
        const uint32_t ni = 4u * L.geo.n;
        rc = radix::sort_pairs<uint16_t>(L.tile_plan, false, at<uint16_t>(ws, L.inst_keys_a),
                                         at<uint32_t>(ws, L.inst_vals_a), at<uint16_t>(ws, L.inst_keys_b),
                                         at<uint32_t>(ws, L.inst_vals_b), counters + kCntInstances, ni,
                                         at<uint32_t>(ws, L.hist_tile), at<uint32_t>(ws, L.bases_tile),
                                         at<uint32_t>(ws, L.status_tile), counters + kCntTicketTile,
                                         counters + kCntError, stream, "raster_tile_sort");
        if (rc != INPC_OK) return rc;
        INPC_LAUNCH("raster_tile_ranges", k_tile_ranges, dim3(std::min<uint32_t>(div_up(ni, kBlock), 4096u)),
                    dim3(kBlock), stream, (const uint16_t*)at<uint16_t>(ws, L.pub.instance_keys),
                    at<uint2>(ws, L.pub.tile_ranges), (const uint32_t*)counters, ni);
    }
    return dispatch_blend_forward(L, features, image, alpha, blending_weights, depth_image, ws, stream);
}

int inpc_raster_backward(const inpc_raster_config* cfg, const float* grad_image, const float* grad_alpha,
                         const float* image, const float* alpha, const float* positions, const void* features,
                         const float* opacities, const float* cam_position, void* grad_features,
                         float* grad_opacities, float* grad_view_scratch, void* ws, size_t ws_bytes, void* stream_) {
    hipStream_t stream = (hipStream_t)stream_;
    (void)opacities;
    Layout L;
    int rc = make_layout(cfg, L);
    if (rc != INPC_OK) return rc;
    if (L.inference || L.fmode == INPC_FEAT_RAW37_F16)
        return fail(INPC_E_UNSUPPORTED, "inpc_raster_backward: inference configurations have no backward pass");
    if (!ws || ws_bytes < L.pub.total_bytes) return fail(INPC_E_WORKSPACE, "inpc_raster_backward: workspace too small");
    if (L.geo.n == 0) return INPC_OK;
    if (!grad_image || !grad_alpha || !image || !alpha || !positions || !grad_features || !grad_opacities)
        return fail(INPC_E_INVALID_ARGUMENT, "inpc_raster_backward: null pointer");
    if (!L.sh && !features) return fail(INPC_E_INVALID_ARGUMENT, "inpc_raster_backward: features are null");
    const bool direct32 = L.fmode == INPC_FEAT_DIRECT_F32;
    float* grad_view = direct32 ? (float*)grad_features : grad_view_scratch;
    if (!grad_view) return fail(INPC_E_INVALID_ARGUMENT, "inpc_raster_backward: this feature mode needs grad_view_scratch");
    if (L.sh && !cam_position) return fail(INPC_E_INVALID_ARGUMENT, "inpc_raster_backward: cam_position is null");
    rc = fill_u32(grad_view, 0u, (size_t)L.geo.n * L.C, stream);
    if (rc != INPC_OK) return rc;
    rc = fill_u32(grad_opacities, 0u, L.geo.n, stream);
    if (rc != INPC_OK) return rc;
    rc = dispatch_blend_backward(L, features, grad_image, grad_alpha, image, alpha, grad_view, grad_opacities, ws, stream);
    if (rc != INPC_OK) return rc;
    if (L.fmode == INPC_FEAT_SH36_F16) {
        INPC_LAUNCH("raster_sh_backward", k_sh_backward, dim3(div_up(L.geo.n, kBlock)), dim3(kBlock), stream, positions,
                    cam_position, (const float4*)at<float4>(ws, L.pub.point_record), (const float4*)grad_view,
                    (__half*)grad_features, L.geo.n);
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
    uint32_t host[3] = {0, 0, 0};
    INPC_HIP_CHECK(hipMemcpyAsync(host, (const char*)ws + L.pub.counters, sizeof(host), hipMemcpyDeviceToHost, stream));
    INPC_HIP_CHECK(hipStreamSynchronize(stream));
    if (counters_host) memcpy(counters_host, host, sizeof(host));
    if (host[2]) return fail(INPC_E_DEVICE, "rasterizer look-back gave up waiting (device error flag set)");
    return INPC_OK;
}

}  // extern "C"
