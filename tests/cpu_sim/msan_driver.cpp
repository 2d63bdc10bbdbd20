// msan_driver.cpp — the library's entry points on buffers that nobody has initialised, under MemorySanitizer.
//
// The library's contract is that a caller's workspace needs no clearing and that every output element is written.
// This program checks it at the level of single bytes: built by tests/cpu_sim/build.py with clang++ -fsanitize=memory
// from the library's own sources and the simulator (a standalone executable, because MemorySanitizer needs the whole
// program instrumented), it gives every call freshly allocated, uninitialised workspaces and outputs, and
// MemorySanitizer ends it at the first branch, address or output that depends on a byte nothing has written.
// The outputs are then checked to be initialised in full. TEST INFRASTRUCTURE ONLY.
#include <sanitizer/msan_interface.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>

#include "../../include/inpc_hip.h"

namespace {

void* fresh(size_t bytes) {   // uninitialised, 256-byte aligned like device memory
    void* p = nullptr;
    if (posix_memalign(&p, 256, bytes ? bytes : 1) != 0) std::abort();
    return p;
}

// The workspace of the Gaussian footprint is the one exception to "nothing reads what nothing has written", by design:
// its backward pass tells the gradient rows of this pass from stale ones by a 64-bit stamp that every forward pass
// takes from the workspace and steps by one, so the first stamp of a workspace and the rows it is compared with are
// whatever the memory held (a stale row passes for a fresh one only if 64 arbitrary bits equal the stamp). That
// workspace is therefore handed over filled with a byte pattern, which MemorySanitizer takes for initialised.
void* filled(size_t bytes) {
    void* p = fresh(bytes);
    std::memset(p, 0xA7, bytes);
    return p;
}

#define CHECK(call)                                                                 \
    do {                                                                            \
        const int rc_ = (call);                                                     \
        if (rc_ != 0) {                                                             \
            std::printf("%s -> %d: %s\n", #call, rc_, inpc_last_error());           \
            return 1;                                                               \
        }                                                                           \
    } while (0)

std::mt19937 g_gen(1);
float uniform(float lo, float hi) { return std::uniform_real_distribution<float>(lo, hi)(g_gen); }

const float kW2c[16] = {1, 0, 0, 0, 0, 1, 0, 0, 0, 0, 1, 2.5f, 0, 0, 0, 1};   // camera at (0, 0, -2.5) looking along +z
const float kCamPosition[3] = {0, 0, -2.5f};

int sampler() {
    const uint32_t n_leaves = 70001, n = 50000;
    float* centers = (float*)fresh(n_leaves * 12);
    int32_t* levels = (int32_t*)fresh(n_leaves * 4);
    float* weights = (float*)fresh(n_leaves * 4);
    for (uint32_t i = 0; i < n_leaves; ++i) {
        for (int k = 0; k < 3; ++k) centers[3 * i + k] = uniform(-2.f, 2.f);
        levels[i] = 5 + (int)(i % 4);
        weights[i] = (i % 7 == 0) ? 0.0f : std::exp(uniform(-1.f, 1.f));
    }
    float* w2c = (float*)fresh(64);
    std::memcpy(w2c, kW2c, 64);
    const inpc_camera cam{320, 200, 260.f, 260.f, 160.f, 100.f, 0.01f, 100.f};
    float* view_weights = (float*)fresh(n_leaves * 4);
    float* boxes = (float*)fresh(n_leaves * 16);
    CHECK(inpc_leaf_weights(centers, levels, weights, w2c, view_weights, boxes, n_leaves, &cam, 4.0f, nullptr));
    const size_t head_floats = inpc_cdf_head_floats(n_leaves);
    float* head = (float*)fresh(head_floats * 4);
    const size_t ws_bytes = inpc_sampler_workspace_bytes(n_leaves);
    void* ws = fresh(ws_bytes);
    // the expected-count sampler on the un-normalised weights first
    float* total = (float*)fresh(4);
    int32_t* offsets = (int32_t*)fresh(n_leaves * 4);
    CHECK(inpc_expected_counts(view_weights, total, offsets, 40000, ws, ws_bytes, n_leaves, nullptr));
    __msan_check_mem_is_initialized(offsets, n_leaves * 4);
    __msan_check_mem_is_initialized(total, 4);
    const uint32_t n_created = (uint32_t)offsets[n_leaves - 1];
    uint64_t* rng = (uint64_t*)fresh(16);
    inpc_pcg32_seed(rng, 7, 1);
    int32_t* ids32 = (int32_t*)fresh((size_t)n_created * 4);
    float* expected = (float*)fresh((size_t)n_created * 2 * 12);
    CHECK(inpc_expected_samples(centers, levels, offsets, ids32, expected, n_created, 2, n_leaves, 4.0f, rng, nullptr));
    __msan_check_mem_is_initialized(expected, (size_t)n_created * 2 * 12);
    // the CDF and a training draw
    CHECK(inpc_build_cdf(view_weights, head, head_floats, ws, ws_bytes, n_leaves, nullptr));
    __msan_check_mem_is_initialized(view_weights, n_leaves * 4);
    __msan_check_mem_is_initialized(head, head_floats * 4);
    float* positions = (float*)fresh(n * 12);
    int64_t* ids = (int64_t*)fresh(n * 8);
    const size_t cull_bytes = inpc_cull_workspace_bytes(n + 4096);
    void* cull_ws = fresh(cull_bytes);
    CHECK(inpc_sample_cull_compact(boxes, view_weights, head, head_floats, w2c, positions, ids, 1, n, 0, n + 4096, n_leaves,
                                   &cam, rng, cull_ws, cull_bytes, nullptr));
    CHECK(inpc_cull_finish(head, positions, ids, 1, n, INPC_CULL_IF_COMPLETE, rng, cull_ws, cull_bytes, nullptr));
    uint32_t accepted = 0, consumed = 0;
    CHECK(inpc_cull_read_counts(cull_ws, &accepted, &consumed, nullptr));
    __msan_check_mem_is_initialized(positions, (size_t)accepted * 12);
    __msan_check_mem_is_initialized(ids, (size_t)accepted * 8);
    float* plain = (float*)fresh(n * 12);
    int32_t* plain_ids = (int32_t*)fresh(n * 4);
    CHECK(inpc_sample(boxes, view_weights, head, head_floats, plain, plain_ids, n, n_leaves, rng, nullptr));
    __msan_check_mem_is_initialized(plain, n * 12);
    __msan_check_mem_is_initialized(plain_ids, n * 4);
    // the probability field's update from these samples
    float* leaf_weights = (float*)fresh(n_leaves * 4);
    float* leaf_scores = (float*)fresh(n_leaves * 4);
    float* sample_weights = (float*)fresh(n * 4);
    for (uint32_t i = 0; i < n_leaves; ++i) leaf_weights[i] = uniform(0.f, 1.f), leaf_scores[i] = uniform(0.f, 1.f);
    for (uint32_t i = 0; i < n; ++i) sample_weights[i] = uniform(0.f, 1.f);
    const size_t field_bytes = inpc_field_update_workspace_bytes(n_leaves);
    void* field_ws = fresh(field_bytes);
    CHECK(inpc_field_update(ids, sample_weights, accepted, leaf_weights, leaf_scores, n_leaves, 0.99f, field_ws, field_bytes,
                            nullptr));
    CHECK(inpc_field_update_check(field_ws, nullptr));
    __msan_check_mem_is_initialized(leaf_weights, n_leaves * 4);
    __msan_check_mem_is_initialized(leaf_scores, n_leaves * 4);
    (void)consumed;
    std::printf("sampler, expected counts, field update: %u samples accepted, %u expected samples\n", accepted, n_created);
    return 0;
}

struct Scene {
    uint32_t n;
    float* positions;
    float* features;
    float* opacities;
    float* w2c;
    float* cam_position;
};

Scene make_scene(uint32_t n, int channels) {
    Scene s{n, (float*)fresh(n * 12), (float*)fresh((size_t)n * channels * 4), (float*)fresh(n * 4), (float*)fresh(64),
            (float*)fresh(12)};
    for (uint32_t i = 0; i < n; ++i) {
        for (int k = 0; k < 3; ++k) s.positions[3 * i + k] = uniform(-0.9f, 0.9f);
        if (i % 50 == 0) s.positions[3 * i + 2] = -2.45f;      // next to the camera: a Gaussian footprint of many tiles
        if (i % 97 == 0) s.positions[3 * i] = NAN;            // never drawn
        if (i % 11 == 0 && i > 0) std::memcpy(s.positions + 3 * i, s.positions + 3 * (i - 1), 12);   // equal depth keys
        for (int c = 0; c < channels; ++c) s.features[(size_t)i * channels + c] = uniform(-1.f, 1.f);
        s.opacities[i] = uniform(0.f, 1.f);
    }
    std::memcpy(s.w2c, kW2c, 64);
    std::memcpy(s.cam_position, kCamPosition, 12);
    return s;
}

int rasterizer(int tile, int channels, bool gaussian) {
    const uint32_t n = 30000;
    const int width = 203, height = 131;
    const Scene s = make_scene(n, channels);
    const inpc_camera cam{width, height, 180.f, 180.f, width / 2.f, height / 2.f, 0.01f, 100.f};
    const size_t pixels = (size_t)width * height;
    float* image = (float*)fresh(pixels * channels * 4);
    float* alpha = (float*)fresh(pixels * 4);
    float* blending_weights = (float*)fresh(n * 4);
    float* grad_image = (float*)fresh(pixels * channels * 4);
    float* grad_alpha = (float*)fresh(pixels * 4);
    for (size_t i = 0; i < pixels * channels; ++i) grad_image[i] = uniform(-0.01f, 0.01f);
    for (size_t i = 0; i < pixels; ++i) grad_alpha[i] = uniform(-0.01f, 0.01f);
    float* grad_features = (float*)fresh((size_t)n * channels * 4);
    float* grad_opacities = (float*)fresh(n * 4);
    inpc_raster_config cfg{n, tile, channels, INPC_FEAT_DIRECT_F32, 0u, cam, 0u};
    uint32_t visible = 0, instances = 0;
    for (int pass = 0; pass < 2; ++pass) {   // two passes on one workspace: the second finds what the first left
        static void* ws = nullptr;
        static size_t ws_bytes = 0;
        if (pass == 0) {
            if (gaussian) {
                inpc_gaussian_config g{cfg, 0.0f, 3.0f, 40u * n, 0u};
                inpc_gaussian_layout layout;
                CHECK(inpc_gaussian_layout_query(&g, &layout));
                ws_bytes = layout.total_bytes;
            } else {
                inpc_raster_layout layout;
                CHECK(inpc_raster_layout_query(&cfg, &layout));
                ws_bytes = layout.total_bytes;
            }
            ws = gaussian ? filled(ws_bytes) : fresh(ws_bytes);
        }
        if (gaussian) {
            inpc_gaussian_config g{cfg, 0.0f, 3.0f, 40u * n, 0u};
            CHECK(inpc_gaussian_forward(&g, s.positions, s.features, s.opacities, nullptr, s.w2c, s.cam_position, image, alpha,
                                        blending_weights, nullptr, ws, ws_bytes, nullptr));
            uint32_t counters[4];
            CHECK(inpc_gaussian_read_counters(&g, ws, counters, nullptr));
            visible = counters[0], instances = counters[1];
            CHECK(inpc_gaussian_backward(&g, grad_image, grad_alpha, image, alpha, s.positions, s.cam_position, grad_features,
                                         grad_opacities, nullptr, ws, ws_bytes, nullptr));
        } else {
            CHECK(inpc_raster_forward(&cfg, s.positions, s.features, s.opacities, s.w2c, s.cam_position, image, alpha,
                                      blending_weights, nullptr, ws, ws_bytes, nullptr));
            uint32_t counters[3];
            CHECK(inpc_raster_read_counters(&cfg, ws, counters, nullptr));
            visible = counters[0], instances = counters[1];
            CHECK(inpc_raster_backward(&cfg, grad_image, grad_alpha, image, alpha, s.positions, s.cam_position, grad_features,
                                       grad_opacities, nullptr, ws, ws_bytes, nullptr));
        }
        __msan_check_mem_is_initialized(image, pixels * channels * 4);
        __msan_check_mem_is_initialized(alpha, pixels * 4);
        __msan_check_mem_is_initialized(blending_weights, n * 4);
        __msan_check_mem_is_initialized(grad_features, (size_t)n * channels * 4);
        __msan_check_mem_is_initialized(grad_opacities, n * 4);
    }
    // inference on the same points: depth image instead of blending weights
    float* depth = (float*)fresh(pixels * 4);
    cfg.flags = INPC_RASTER_INFERENCE;
    if (gaussian) {
        inpc_gaussian_config g{cfg, 0.004f, 2.5f, 40u * n, 0u};
        inpc_gaussian_layout layout;
        CHECK(inpc_gaussian_layout_query(&g, &layout));
        void* ws = filled(layout.total_bytes);
        CHECK(inpc_gaussian_forward(&g, s.positions, s.features, s.opacities, nullptr, s.w2c, s.cam_position, image, alpha,
                                    nullptr, depth, ws, layout.total_bytes, nullptr));
    } else {
        inpc_raster_layout layout;
        CHECK(inpc_raster_layout_query(&cfg, &layout));
        void* ws = fresh(layout.total_bytes);
        CHECK(inpc_raster_forward(&cfg, s.positions, s.features, s.opacities, s.w2c, s.cam_position, image, alpha, nullptr, depth,
                                  ws, layout.total_bytes, nullptr));
    }
    __msan_check_mem_is_initialized(image, pixels * channels * 4);
    __msan_check_mem_is_initialized(depth, pixels * 4);
    std::printf("%s footprint, %dx%d tiles, %d channels: %u of %u points drawn, %u instances\n",
                gaussian ? "Gaussian" : "bilinear", tile, tile, channels, visible, n, instances);
    return 0;
}

// The bookkeeping of the probability field (selections, extraction of a global cloud, Morton codes) and the
// element-wise operators.
int field_and_misc() {
    const uint32_t n = 33333;
    float* centers = (float*)fresh(n * 12);
    int32_t* levels = (int32_t*)fresh(n * 4);
    float* weights = (float*)fresh(n * 4);
    float* scores = (float*)fresh(n * 4);
    int64_t* counts = (int64_t*)fresh(n * 8);
    uint32_t n_samples = 0;
    for (uint32_t i = 0; i < n; ++i) {
        for (int k = 0; k < 3; ++k) centers[3 * i + k] = uniform(-2.f, 2.f);
        levels[i] = 3 + (int)(i % 5);
        weights[i] = uniform(0.f, 1.f);
        scores[i] = uniform(0.f, 1.f);
        counts[i] = (int64_t)(i % 4);
        n_samples += (uint32_t)counts[i];
    }
    const float initial_size[3] = {4.f, 4.f, 4.f};
    const size_t select_bytes = inpc_field_select_workspace_bytes(n);
    void* select_ws = fresh(select_bytes);
    uint32_t* count = (uint32_t*)fresh(4);
    CHECK(inpc_field_select_count(scores, levels, n, 0.5f, 7, count, select_ws, select_bytes, nullptr));
    __msan_check_mem_is_initialized(count, 4);
    const uint32_t split = *count, n_out = n + 7u * split;
    float* centers_out = (float*)fresh((size_t)n_out * 12);
    int32_t* levels_out = (int32_t*)fresh((size_t)n_out * 4);
    float* weights_out = (float*)fresh((size_t)n_out * 4);
    float* scores_out = (float*)fresh((size_t)n_out * 4);
    CHECK(inpc_field_subdivide(centers, levels, weights, scores, n, 0.5f, 7, initial_size, centers_out, levels_out, weights_out,
                               scores_out, count, select_ws, select_bytes, nullptr));
    __msan_check_mem_is_initialized(centers_out, (size_t)n_out * 12);
    __msan_check_mem_is_initialized(levels_out, (size_t)n_out * 4);
    __msan_check_mem_is_initialized(weights_out, (size_t)n_out * 4);
    __msan_check_mem_is_initialized(scores_out, (size_t)n_out * 4);
    CHECK(inpc_field_prune(centers, levels, weights, scores, n, 0.3f, centers_out, levels_out, weights_out, scores_out, count,
                           select_ws, select_bytes, nullptr));
    __msan_check_mem_is_initialized(count, 4);
    __msan_check_mem_is_initialized(centers_out, (size_t)*count * 12);
    __msan_check_mem_is_initialized(scores_out, (size_t)*count * 4);
    const size_t extract_bytes = inpc_extract_global_workspace_bytes(n);
    void* extract_ws = fresh(extract_bytes);
    float* cloud = (float*)fresh((size_t)n_samples * 12);
    CHECK(inpc_extract_global(centers, levels, counts, n, initial_size, cloud, n_samples, extract_ws, extract_bytes, nullptr));
    CHECK(inpc_extract_global_check(extract_ws, n_samples, nullptr));
    __msan_check_mem_is_initialized(cloud, (size_t)n_samples * 12);
    int64_t* codes = (int64_t*)fresh((size_t)n_samples * 8);
    void* morton_ws = fresh(inpc_morton_workspace_bytes());
    CHECK(inpc_morton_encode(cloud, n_samples, codes, morton_ws, inpc_morton_workspace_bytes(), nullptr));
    __msan_check_mem_is_initialized(codes, (size_t)n_samples * 8);
    float* contracted = (float*)fresh((size_t)n_samples * 12);
    CHECK(inpc_spherical_contraction(cloud, contracted, n_samples, nullptr));
    __msan_check_mem_is_initialized(contracted, (size_t)n_samples * 12);
    float* out_a = (float*)fresh(n * 4);
    float* out_b = (float*)fresh(n * 4);
    CHECK(inpc_opacity_forward(scores, out_a, n, nullptr));
    CHECK(inpc_opacity_backward(weights, scores, out_b, n, nullptr));
    __msan_check_mem_is_initialized(out_a, n * 4);
    __msan_check_mem_is_initialized(out_b, n * 4);
    CHECK(inpc_weight_decay_grads(weights, out_a, n, 0, nullptr));
    CHECK(inpc_weight_decay_grads(weights, out_a, n, 1, nullptr));
    CHECK(inpc_cauchy_loss(weights, scores, out_b, n, nullptr));
    __msan_check_mem_is_initialized(out_a, n * 4);
    __msan_check_mem_is_initialized(out_b, n * 4);
    float* upstream = (float*)fresh(4);
    *upstream = 1.5f;
    CHECK(inpc_cauchy_loss_backward(upstream, weights, scores, out_a, n, nullptr));
    __msan_check_mem_is_initialized(out_a, n * 4);
    std::printf("field bookkeeping and element-wise operators: %u leaves split, %u samples extracted\n", split, n_samples);
    return 0;
}

// fp16 bits of a float of ordinary size (no rounding needed for the tests: truncation)
uint16_t half_bits(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    const uint32_t sign = (u >> 16) & 0x8000u;
    const int32_t exponent = (int32_t)((u >> 23) & 0xFF) - 127 + 15;
    if (exponent <= 0) return (uint16_t)sign;
    if (exponent >= 31) return (uint16_t)(sign | 0x7BFFu);
    return (uint16_t)(sign | ((uint32_t)exponent << 10) | ((u >> 13) & 0x3FFu));
}

// The spherical-harmonics modes: training on (N,36) fp16 coefficients (the gradient comes back as fp16 through a
// scratch array) and inference on the raw (N,37) fp16 output of the appearance field.
int rasterizer_sh(bool gaussian) {
    const uint32_t n = 20000;
    const int width = 157, height = 101, tile = 16;
    const Scene s = make_scene(n, 4);
    const inpc_camera cam{width, height, 140.f, 140.f, width / 2.f, height / 2.f, 0.01f, 100.f};
    const size_t pixels = (size_t)width * height;
    uint16_t* sh = (uint16_t*)fresh((size_t)n * 36 * 2);
    uint16_t* raw = (uint16_t*)fresh((size_t)n * 37 * 2);
    for (size_t i = 0; i < (size_t)n * 36; ++i) sh[i] = half_bits(uniform(-0.5f, 0.5f));
    for (size_t i = 0; i < (size_t)n * 37; ++i) raw[i] = half_bits(uniform(-0.5f, 0.5f));
    float* image = (float*)fresh(pixels * 4 * 4);
    float* alpha = (float*)fresh(pixels * 4);
    float* depth = (float*)fresh(pixels * 4);
    float* blending_weights = (float*)fresh(n * 4);
    float* grad_image = (float*)fresh(pixels * 4 * 4);
    float* grad_alpha = (float*)fresh(pixels * 4);
    for (size_t i = 0; i < pixels * 4; ++i) grad_image[i] = uniform(-0.01f, 0.01f);
    for (size_t i = 0; i < pixels; ++i) grad_alpha[i] = uniform(-0.01f, 0.01f);
    uint16_t* grad_sh = (uint16_t*)fresh((size_t)n * 36 * 2);
    float* grad_opacities = (float*)fresh(n * 4);
    float* scratch = (float*)fresh((size_t)n * 4 * 4);
    inpc_raster_config cfg{n, tile, 4, INPC_FEAT_SH36_F16, 0u, cam, 0u};
    inpc_raster_config raw_cfg{n, tile, 4, INPC_FEAT_RAW37_F16, INPC_RASTER_INFERENCE, cam, 0u};
    if (gaussian) {
        inpc_gaussian_config g{cfg, 0.0f, 3.0f, 40u * n, 0u};
        inpc_gaussian_layout layout;
        CHECK(inpc_gaussian_layout_query(&g, &layout));
        void* ws = filled(layout.total_bytes);
        CHECK(inpc_gaussian_forward(&g, s.positions, sh, s.opacities, nullptr, s.w2c, s.cam_position, image, alpha,
                                    blending_weights, nullptr, ws, layout.total_bytes, nullptr));
        CHECK(inpc_gaussian_backward(&g, grad_image, grad_alpha, image, alpha, s.positions, s.cam_position, grad_sh,
                                     grad_opacities, scratch, ws, layout.total_bytes, nullptr));
    } else {
        inpc_raster_layout layout;
        CHECK(inpc_raster_layout_query(&cfg, &layout));
        void* ws = fresh(layout.total_bytes);
        CHECK(inpc_raster_forward(&cfg, s.positions, sh, s.opacities, s.w2c, s.cam_position, image, alpha, blending_weights,
                                  nullptr, ws, layout.total_bytes, nullptr));
        CHECK(inpc_raster_backward(&cfg, grad_image, grad_alpha, image, alpha, s.positions, s.cam_position, grad_sh,
                                   grad_opacities, scratch, ws, layout.total_bytes, nullptr));
    }
    __msan_check_mem_is_initialized(image, pixels * 4 * 4);
    __msan_check_mem_is_initialized(alpha, pixels * 4);
    __msan_check_mem_is_initialized(blending_weights, n * 4);
    __msan_check_mem_is_initialized(grad_sh, (size_t)n * 36 * 2);
    __msan_check_mem_is_initialized(grad_opacities, n * 4);
    if (gaussian) {
        inpc_gaussian_config g{raw_cfg, 0.004f, 2.5f, 40u * n, 0u};
        inpc_gaussian_layout layout;
        CHECK(inpc_gaussian_layout_query(&g, &layout));
        void* ws = filled(layout.total_bytes);
        CHECK(inpc_gaussian_forward(&g, s.positions, raw, nullptr, nullptr, s.w2c, s.cam_position, image, alpha, nullptr, depth,
                                    ws, layout.total_bytes, nullptr));
    } else {
        inpc_raster_layout layout;
        CHECK(inpc_raster_layout_query(&raw_cfg, &layout));
        void* ws = fresh(layout.total_bytes);
        CHECK(inpc_raster_forward(&raw_cfg, s.positions, raw, nullptr, s.w2c, s.cam_position, image, alpha, nullptr, depth, ws,
                                  layout.total_bytes, nullptr));
    }
    __msan_check_mem_is_initialized(image, pixels * 4 * 4);
    __msan_check_mem_is_initialized(alpha, pixels * 4);
    __msan_check_mem_is_initialized(depth, pixels * 4);
    std::printf("%s footprint, spherical harmonics: training on (N,36) fp16, inference on raw (N,37) fp16\n",
                gaussian ? "Gaussian" : "bilinear");
    return 0;
}

}  // namespace

int main() {
    if (sampler() != 0) return 1;
    if (field_and_misc() != 0) return 1;
    for (const bool gaussian : {false, true})
        for (const int tile : {16, 8})
            if (rasterizer(tile, tile == 16 ? 8 : 4, gaussian) != 0) return 1;
    for (const bool gaussian : {false, true})
        if (rasterizer_sh(gaussian) != 0) return 1;
    std::printf("no use of uninitialised memory\n");
    return 0;
}
