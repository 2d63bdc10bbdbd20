// geometry.hpp — the per-point arithmetic of the bilinear rasterizer as plain functions: projection, tile bounds,
// footprint weights, the fragment slots of a point in a tile, the gradient row of an instance
// (B/rasterization/src/bilinear/kernels.cu:11-84,198-220,281-287). Included by raster.hip inside its namespace, where the
// kernels call them on the device; the same functions compile for the host (INPC_HD), so that the tests can run them on
// a CPU, without a GPU, against restatements of the reference. Nothing here touches memory or knows about waves.
#pragma once

// tile info word of a projected point: first tile id, spans, valid
constexpr uint32_t kInfoValid = 1u << 18;
INPC_HD uint32_t info_tile0(uint32_t info) { return info & 0xFFFFu; }
INPC_HD uint32_t info_nx(uint32_t info) { return ((info >> 16) & 1u) + 1u; }
INPC_HD uint32_t info_ny(uint32_t info) { return ((info >> 17) & 1u) + 1u; }

// Blend record of a drawn point, at the point's index in the record array: a 32-byte header followed by the view
// features, padded to a multiple of 32 bytes (64 bytes for every configuration but 16 fp32 channels).
//   header: float wx0, wx1, wy0, wy1   interpolation weights of the two candidate pixel columns Lx, Lx + 1 and rows
//                                      Ly, Ly + 1 (L = floor(s - 0.5)); 0 where the pixel centre is 1 or more away
//                                      (kernels.cu:284-287)
//           float opacity
//           u32   point index | kRecordMulti when the point touches several tiles | span bits
//           u32   (Lx + 1) | (Ly + 1) << 16
//           u32   training: first gradient row of a point that touches several tiles; inference: depth
constexpr uint32_t kRecordHeader = 32;
constexpr uint32_t kRecordIdMask = (1u << 28) - 1u;
constexpr uint32_t kRecordMulti = 1u << 28, kRecordSpanX = 1u << 29;   // bit 30: two tiles in y
struct Geometry {
    uint32_t n;
    int W, H;
    uint32_t gw, gh, n_tiles;
    Camera cam;
    uint32_t key_bias;      // depth key = float bits - key_bias
    uint32_t stride;        // record stride in bytes
    uint32_t capacity;      // instances the buffers hold
    uint32_t row_capacity;  // gradient rows (instances of points that touch several tiles)
    uint32_t tile_shift;    // log2 of the tile size
    uint32_t n_chunks;      // contiguous chunks the points are cut into for binning (one block each)
};

// ---- projection (kernels.cu:40-64) ---------------------------------------------------------------------------
struct Projected {
    float sx, sy, depth;
    uint32_t info;     // 0 when the point is not drawn
    uint32_t touched;  // number of tiles
};

struct ViewRows {
    float4 r1, r2, r3;
};

INPC_HD ViewRows load_view_rows(const float* __restrict__ w2c) {
    ViewRows m;
    m.r1 = make_float4(w2c[0], w2c[1], w2c[2], w2c[3]);
    m.r2 = make_float4(w2c[4], w2c[5], w2c[6], w2c[7]);
    m.r3 = make_float4(w2c[8], w2c[9], w2c[10], w2c[11]);
    return m;
}

template <int T>
INPC_HD Projected project_point(const ViewRows& m, const Geometry& g, float px, float py, float pz) {
    Projected o;
    o.sx = 0.0f;
    o.sy = 0.0f;
    o.info = 0u;
    o.touched = 0u;
    o.depth = affine_row(m.r3, px, py, pz);
    if (o.depth < g.cam.near_plane || o.depth > g.cam.far_plane) return o;
    const float fT = (float)T, fgw = (float)g.gw, fgh = (float)g.gh;
    const float x = affine_row(m.r1, px, py, pz) / o.depth;
    const float y = affine_row(m.r2, px, py, pz) / o.depth;
    o.sx = x * g.cam.fx + g.cam.cx;
    o.sy = y * g.cam.fy + g.cam.cy;
    const uint32_t x0 = (uint32_t)fminf(fgw, fmaxf(0.0f, floorf((o.sx - 0.5f) / fT)));
    const uint32_t x1 = (uint32_t)fminf(fgw, fmaxf(0.0f, ceilf((o.sx + 0.5f) / fT)));
    const uint32_t y0 = (uint32_t)fminf(fgh, fmaxf(0.0f, floorf((o.sy - 0.5f) / fT)));
    const uint32_t y1 = (uint32_t)fminf(fgh, fmaxf(0.0f, ceilf((o.sy + 0.5f) / fT)));
    o.touched = (x1 - x0) * (y1 - y0);
    if (o.touched != 0u) o.info = (y0 * g.gw + x0) | ((x1 - x0 - 1u) << 16) | ((y1 - y0 - 1u) << 17) | kInfoValid;
    return o;
}

// The two pixels of one axis that can lie closer than 1 to screen coordinate s: L = floor(s - 0.5) and L + 1.
// Their interpolation weights as the reference's blend computes them per pixel (kernels.cu:284-287):
// d = |s - (pixel + 0.5)|, skipped when d >= 1 (weight 0 here), else saturate(1 - d).
struct AxisWeights {
    int left;         // L, clamped to [-1, 65534]
    float w0, w1;
};

INPC_HD AxisWeights axis_weights(float s) {
    AxisWeights a;
    a.left = (int)fminf(fmaxf(floorf(s - 0.5f), -1.0f), 65534.0f);
    const float d0 = fabsf(s - ((float)a.left + 0.5f));
    const float d1 = fabsf(s - ((float)(a.left + 1) + 0.5f));
    a.w0 = !(d0 >= 1.0f) ? saturate01(1.0f - d0) : 0.0f;
    a.w1 = !(d1 >= 1.0f) ? saturate01(1.0f - d1) : 0.0f;
    return a;
}

// Depth key of a drawn point: its depth's float bits above those of the near plane (positive floats order like their
// bits), so that the tile sort only has to look at the bits that can differ (kernels.cu:66-84).
INPC_HD uint32_t depth_key(float depth, uint32_t key_bias) { return float_bits_of(depth) - key_bias; }

// For every touched tile of a projected point, in the row-major order of the reference's create_instances_cu
// (kernels.cu:208-217).
template <typename F>
INPC_HD void for_each_tile(uint32_t info, uint32_t gw, F f) {
    const uint32_t tile0 = info_tile0(info);
    f(tile0);
    if (info & (1u << 16)) f(tile0 + 1u);
    if (info & (1u << 17)) {
        f(tile0 + gw);
        if (info & (1u << 16)) f(tile0 + gw + 1u);
    }
}

namespace blend {

// Fragment field of a staged instance (16 bits per slot), 0 until the slot's wave places the fragment in its
// list: bits 0-5 the pixel in the owning wave's grid (row * 8 + column), bit 7: placed, bits 8-15: where.
constexpr uint32_t kPixelMask = 63u, kPlaced = 0x80u;
constexpr uint32_t kNoPixel = 0xFFu;

// The record header as the kernels use it.
struct Header {
    float wx0, wx1, wy0, wy1;   // weights of the candidate columns Lx, Lx + 1 and rows Ly, Ly + 1
    float opacity;
    uint32_t tag;     // point index | kRecordMulti | span bits (kept as the raw word until the write phase: a
                      // flag derived at the load would make the gather wait for its own first reply)
    uint32_t cell;    // (Lx + 1) | (Ly + 1) << 16
    uint32_t extra;   // first gradient row (training, points that touch several tiles) or depth bits (inference)
    INPC_HD bool multi() const { return (tag & kRecordMulti) != 0u; }
    INPC_HD uint32_t point() const { return tag & kRecordIdMask; }
};

INPC_HD Header make_header(const float4 h0, const float4 h1) {
    Header h;
    h.wx0 = h0.x;
    h.wx1 = h0.y;
    h.wy0 = h0.z;
    h.wy1 = h0.w;
    h.opacity = h1.x;
    h.tag = float_bits_of(h1.y);
    h.cell = float_bits_of(h1.z);
    h.extra = float_bits_of(h1.w);
    return h;
}

// Tile-local index of the left / top candidate pixel of a record.
INPC_HD int local_left(uint32_t cell_half, int tile_origin) { return (int)cell_half - 1 - tile_origin; }

// The candidate (0: L, 1: L + 1) of one axis whose tile-local index has the parity `odd` (tiles start at even pixels).
INPC_HD int candidate_of_parity(int left, uint32_t odd) { return (left ^ (int)odd) & 1; }

// The four fragment slots of a point in a tile. 16x16 tiles: slot = parity class (x parity | y parity << 1) of the
// candidate pixel, i.e. the wave that owns it; 8x8 tiles: slot = candidate (kx | ky << 1). Per slot: the
// interpolation weight (whether the fragment exists or not) and the pixel in the owning wave's 8 x 8 grid, kNoPixel
// when the candidate lies outside the tile or a pixel centre is 1 or more away (B/rasterization/src/bilinear/
// kernels.cu:284-285: weight 0).
template <int T>
INPC_HD void fragment_slots(const Header& h, int tile_x0, int tile_y0, float (&weight)[4],
                                               uint32_t (&pixel)[4]) {
    // plain scalars: a choice between two members of the record would otherwise be made through memory
    const float wx0 = h.wx0, wx1 = h.wx1, wy0 = h.wy0, wy1 = h.wy1;
    const int lx = local_left(h.cell & 0xFFFFu, tile_x0), ly = local_left(h.cell >> 16, tile_y0);
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const int kx = T == 16 ? candidate_of_parity(lx, c & 1) : (c & 1);
        const int ky = T == 16 ? candidate_of_parity(ly, c >> 1) : (c >> 1);
        const int cx = lx + kx, cy = ly + ky;
        const float wx = kx ? wx1 : wx0, wy = ky ? wy1 : wy0;
        weight[c] = wx * wy;
        const bool hit = (uint32_t)(cx | cy) < (uint32_t)T && weight[c] > 0.0f;
        const uint32_t pix = T == 16 ? (uint32_t)((cy >> 1) * 8 + (cx >> 1)) : (uint32_t)(cy * 8 + cx);
        pixel[c] = hit ? (pix & kPixelMask) : kNoPixel;
    }
}

// The gradient row of an instance of a point that touches several tiles: the point's first row plus the place of this
// tile among the point's tiles, row-major (kernels.cu:208-217 creates the instances in that order). The tile is the
// second of its row / column exactly when the point's left / top candidate pixel lies in the tile in front (and there
// is one: a candidate left of the image belongs to no tile). lx, ly: tile-local index of the left / top candidate pixel.
INPC_HD uint32_t instance_row(uint32_t first_row, uint32_t tag, int lx, int ly, int tile_x0, int tile_y0) {
    return first_row + (lx < 0 && tile_x0 > 0 ? 1u : 0u) + (ly < 0 && tile_y0 > 0 ? ((tag & kRecordSpanX) ? 2u : 1u) : 0u);
}

}  // namespace blend

namespace gaussian {

// exp(x) for x <= 0 by one fixed sequence of fp32 operations (the reference calls expf / __expf, kernels.cu:451,
// 548,634): n = rint(x log2 e), r = x - n ln 2 in two parts, a degree-7 polynomial (Cephes' expf coefficients),
// scaling by 2^n. Within one ulp of exp on [-87, 0], 0 below; a CPU evaluates the same sequence to the same bits,
// so the cut at the footprint's threshold falls on the same pixels.
INPC_HD float footprint_exp(float x) {
    if (!(x >= -87.0f)) return 0.0f;
    const float n = __builtin_rintf(x * 1.44269504088896341f);
    const float r = (x - n * 0.693359375f) - n * -2.12194440e-4f;
    float p = 1.9875691500e-4f;
    p = p * r + 1.3981999507e-3f;
    p = p * r + 8.3334519073e-3f;
    p = p * r + 4.1665795894e-2f;
    p = p * r + 1.6666665459e-1f;
    p = p * r + 5.0000001201e-1f;
    const float y = (p * (r * r) + r) + 1.0f;
    return ldexpf(y, (int)n);
}

// Footprint value of a staged instance at the pixel centre (kernels.cu:447-452); false when the pixel is skipped.
// Without branches, so that the values of several instances are computed side by side.
INPC_HD bool footprint_value(const float4 h0, const float4 h1, float cx, float cy, float threshold, float& G) {
    const float dx = h0.x - cx, dy = h0.y - cy;
    const float exponent = -0.5f * (h0.w * dx * dx + h1.y * dy * dy) - h1.x * dx * dy;
    const bool positive = exponent > 0.0f;
    G = footprint_exp(positive ? 0.0f : exponent);   // a NaN exponent stays NaN and gives 0: skipped, as in the reference
    return !positive && !(G < threshold);
}

}  // namespace gaussian
