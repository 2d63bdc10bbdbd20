// Test infrastructure: the rasterizer's per-point arithmetic (inpc_amd/csrc/geometry.hpp: the very functions the
// kernels call on the device) compiled for the host, so that tests can run it on a CPU, without a GPU, against
// independent restatements and the oracle. Built by tests/host_build/build.py with hipcc (host code only runs).
#include <cstdint>

#include "../../inpc_amd/csrc/common.hpp"

namespace inpc {
namespace {
#include "../../inpc_amd/csrc/geometry.hpp"
}  // namespace
}  // namespace inpc

using namespace inpc;

namespace {

Geometry geometry_of(int tile, const inpc_camera* cam) {
    Geometry g{};
    g.W = cam->width;
    g.H = cam->height;
    g.gw = (uint32_t)((cam->width + tile - 1) / tile);
    g.gh = (uint32_t)((cam->height + tile - 1) / tile);
    g.n_tiles = g.gw * g.gh;
    g.cam = to_device_camera(*cam);
    g.key_bias = float_bits_of(cam->near_plane);
    g.tile_shift = tile == 16 ? 4u : 3u;
    return g;
}

template <int T>
void project_all(const Geometry& g, const float* w2c, const float* positions, uint32_t n, float* sx, float* sy,
                 float* depth, uint32_t* info, uint32_t* touched, uint32_t* key) {
    const ViewRows m = load_view_rows(w2c);
    for (uint32_t i = 0; i < n; ++i) {
        const Projected p = project_point<T>(m, g, positions[3 * i], positions[3 * i + 1], positions[3 * i + 2]);
        sx[i] = p.sx;
        sy[i] = p.sy;
        depth[i] = p.depth;
        info[i] = p.info;
        touched[i] = p.touched;
        key[i] = p.info ? depth_key(p.depth, g.key_bias) : 0xFFFFFFFFu;
    }
}

// The record header of a point at screen position (sx, sy), as the records kernel writes it.
blend::Header header_of(float sx, float sy, uint32_t info) {
    const AxisWeights ax = axis_weights(sx), ay = axis_weights(sy);
    blend::Header h{};
    h.wx0 = ax.w0;
    h.wx1 = ax.w1;
    h.wy0 = ay.w0;
    h.wy1 = ay.w1;
    h.opacity = 1.0f;
    h.tag = ((info >> 16) & 3u) << 29;
    h.cell = (uint32_t)(ax.left + 1) | ((uint32_t)(ay.left + 1) << 16);
    h.extra = 0u;
    return h;
}

}  // namespace

extern "C" {

// project_point, tile bounds and depth key of n points (key 0xFFFFFFFF: not drawn); info = first tile | spans | valid
void host_project(int tile, const inpc_camera* cam, const float* w2c, const float* positions, uint32_t n, float* sx,
                  float* sy, float* depth, uint32_t* info, uint32_t* touched, uint32_t* key) {
    const Geometry g = geometry_of(tile, cam);
    if (tile == 16) project_all<16>(g, w2c, positions, n, sx, sy, depth, info, touched, key);
    else project_all<8>(g, w2c, positions, n, sx, sy, depth, info, touched, key);
}

void host_axis_weights(const float* s, uint32_t n, int32_t* left, float* w0, float* w1) {
    for (uint32_t i = 0; i < n; ++i) {
        const AxisWeights a = axis_weights(s[i]);
        left[i] = a.left;
        w0[i] = a.w0;
        w1[i] = a.w1;
    }
}

// The four fragment slots of the point at (sx, sy) in the tile with origin (tile_x0, tile_y0): weight[4], pixel[4]
// (pixel in the owning wave's 8 x 8 grid, 255: no fragment).
void host_fragment_slots(int tile, float sx, float sy, int tile_x0, int tile_y0, float* weight, uint32_t* pixel) {
    const blend::Header h = header_of(sx, sy, 0u);
    float w[4];
    uint32_t p[4];
    if (tile == 16) blend::fragment_slots<16>(h, tile_x0, tile_y0, w, p);
    else blend::fragment_slots<8>(h, tile_x0, tile_y0, w, p);
    for (int c = 0; c < 4; ++c) {
        weight[c] = w[c];
        pixel[c] = p[c];
    }
}

// For every drawn point: its tiles in the order the instances are created in (tiles[i][0..3], 0xFFFFFFFF: none) and the
// gradient row instance_row() gives each of them above a first row of 1000.
void host_instance_rows(int tile, const inpc_camera* cam, const float* w2c, const float* positions, uint32_t n,
                        uint32_t* tiles, uint32_t* rows) {
    const Geometry g = geometry_of(tile, cam);
    const ViewRows m = load_view_rows(w2c);
    for (uint32_t i = 0; i < n; ++i) {
        for (int k = 0; k < 4; ++k) tiles[4 * i + k] = rows[4 * i + k] = 0xFFFFFFFFu;
        const Projected p = tile == 16 ? project_point<16>(m, g, positions[3 * i], positions[3 * i + 1], positions[3 * i + 2])
                                       : project_point<8>(m, g, positions[3 * i], positions[3 * i + 1], positions[3 * i + 2]);
        if (!p.info) continue;
        blend::Header h = header_of(p.sx, p.sy, p.info);
        h.extra = 1000u;
        int k = 0;
        for_each_tile(p.info, g.gw, [&](uint32_t t) {
            const int tile_x0 = (int)(t % g.gw) * tile, tile_y0 = (int)(t / g.gw) * tile;
            const int lx = blend::local_left(h.cell & 0xFFFFu, tile_x0), ly = blend::local_left(h.cell >> 16, tile_y0);
            tiles[4 * i + k] = t;
            rows[4 * i + k] = blend::instance_row(h.extra, h.tag, lx, ly, tile_x0, tile_y0);
            ++k;
        });
    }
}

void host_footprint_exp(const float* x, uint32_t n, float* out) {
    for (uint32_t i = 0; i < n; ++i) out[i] = gaussian::footprint_exp(x[i]);
}

// footprint_value for n pixel centres of one instance {sx, sy, conic}: G[i], drawn[i]
void host_footprint_value(float sx, float sy, float conic_x, float conic_y, float conic_z, float threshold, const float* cx,
                          const float* cy, uint32_t n, float* G, uint8_t* drawn) {
    const float4 h0 = make_float4(sx, sy, 1.0f, conic_x), h1 = make_float4(conic_y, conic_z, 0.0f, 0.0f);
    for (uint32_t i = 0; i < n; ++i) drawn[i] = gaussian::footprint_value(h0, h1, cx[i], cy[i], threshold, G[i]) ? 1 : 0;
}

}  // extern "C"
