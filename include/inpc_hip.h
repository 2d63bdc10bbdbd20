/*
 * inpc_hip.h — C ABI of libinpc_hip.so, the MI355X (gfx950) implementation of the
 * INPCCudaBackend hot path: view-dependent octree point sampling and the tile-based
 * differentiable point rasterizer (forward, backward, inference; bilinear and Gaussian footprint).
 *
 * Conventions
 *   - every pointer marked "dev" is a device pointer on the current HIP device;
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *   - every function returns 0 on success and a negative INPC_E_* code on failure,
 *     never throws; inpc_last_error() returns a thread-local message for the last failure;
 *   - the library never allocates or frees device memory: the caller provides the
 *     workspace whose size inpc_*_workspace_bytes() reports (sized for the worst case,
 *     so no count has to travel back to the host between kernels; the Gaussian footprint,
 *     whose worst case has no useful bound, takes a capacity and reports when it is exceeded);
 *   - all kernels are enqueued on `stream`; no call synchronises the host unless its
 *     comment says so.
 *
 * Each entry point names the reference interface it replaces (paths relative to the
 * reference repository, B/ = INPCCudaBackend/INPCCudaBackend/).
 */
#ifndef INPC_HIP_H
#define INPC_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- status codes -------------------------------------------------------------------- */
#define INPC_OK 0
#define INPC_E_INVALID_ARGUMENT (-1) /* bad size, tile, channel count, null pointer, ...   */
#define INPC_E_WORKSPACE (-2)        /* workspace too small or misaligned                   */
#define INPC_E_UNSUPPORTED (-3)      /* e.g. more than 65536 tiles, unknown feature mode    */
#define INPC_E_HIP (-4)              /* a HIP runtime call failed (message has the detail)  */
#define INPC_E_DEVICE (-5)           /* a kernel raised its device-side error flag          */

/* ---- pinhole camera: the scalars B/torch_bindings/sampling.py:20-33 and
 *      B/torch_bindings/rasterization.py:116-128 unpack from a View ---------------------- */
typedef struct inpc_camera {
    int32_t width;
    int32_t height;
    float focal_x;
    float focal_y;
    float center_x;
    float center_y;
    float near_plane;
    float far_plane;
} inpc_camera;

/* ---- how the per-point features are stored ------------------------------------------- */
#define INPC_FEAT_SH36_F16 0   /* (N,36) fp16, 9 SH coefficients x 4 channels -> 4 channels
                                  (B/rasterization/include/sh_utils.cuh:6-23)              */
#define INPC_FEAT_DIRECT_F32 1 /* (N,C) fp32, C in {4,8,16}, used as they are              */
#define INPC_FEAT_DIRECT_F16 2 /* (N,C) fp16 stored, fp32 accumulated                      */
#define INPC_FEAT_RAW37_F16 3  /* (N,37) fp16: [0] raw opacity, [1..36] SH coefficients
                                  (B/rasterization/src/bilinear/kernels.cu:106-184)        */

/* ---- rasterizer flags ------------------------------------------------------------------ */
#define INPC_RASTER_INFERENCE 1u     /* write a depth image, no blending weights
                                        (B/rasterization/src/bilinear/kernels.cu:422-495)  */
#define INPC_RASTER_KEEP_GEOMETRY 2u /* bilinear footprint: also keep every point's screen position, depth
                                        and tile bounds in the workspace (layout field debug_geometry),
                                        for callers that want to inspect the projection             */

const char* inpc_last_error(void);
int inpc_abi_version(void);

/* =========================================================================================
 * PCG32 host helpers (B/sampling/include/pcg32.h:42-201). `rng` is {state, inc}.
 * The sampler keeps its generator in device memory (two uint64) so that a call whose
 * consumption is data dependent needs no host read-back; these helpers build and step the
 * same generator on the host.
 * ======================================================================================= */
void inpc_pcg32_seed(uint64_t rng[2], uint64_t initstate, uint64_t initseq);
uint32_t inpc_pcg32_next_uint(uint64_t rng[2]);
float inpc_pcg32_next_float(uint64_t rng[2]);
void inpc_pcg32_advance(uint64_t rng[2], int64_t delta);

/* =========================================================================================
 * Sampler
 * ======================================================================================= */

/* Per-leaf view-dependent weight.
 * Replaces compute_viewpoint_weights_wrapper (B/sampling/src/sampling_api.cu:10-47) and
 * kernel compute_viewpoint_weights_cu (B/sampling/src/sampling_kernels.cu:9-64).
 * centers (L,3) f32, levels (L,) i32, weights (L,) f32, w2c (4,4) f32 row-major (rows 0..2
 * are read), out (L,) f32; all dev. boxes_out (L,4) f32 dev, 16-byte aligned, or NULL: receives
 * {centre, initial_size / 2^level} per leaf, the form in which the sampling calls below take the
 * octree (one 16-byte gather per sample instead of four). */
int inpc_leaf_weights(const float* centers, const int32_t* levels, const float* weights,
                      const float* w2c, float* out, float* boxes_out, uint32_t n_leaves,
                      const inpc_camera* cam, float initial_size, void* stream);

/* Bytes of scratch the CDF / counting passes need for n_leaves leaves. */
size_t inpc_sampler_workspace_bytes(uint32_t n_leaves);

/* Floats in the head of a CDF: the total and the top levels of the search tree (the binary search
 * of B/sampling/include/sampling_utils.h:49-69): 14 levels, which the sampling kernels keep in LDS,
 * and for an octree of more than 278,527 leaves as many more as leave a search with at most sixteen
 * elements (they are read from memory in place of the CDF itself). inpc_cdf_head_floats gives the
 * size of the head for n_leaves leaves: INPC_CDF_HEAD_MIN_FLOATS = 2^14 up to 278,527 leaves, the
 * next powers of two beyond (2^17 for 2,097,152 leaves). Every call that takes the head also takes
 * the number of floats the caller's buffer holds (`head_floats`) and returns INPC_E_WORKSPACE, before
 * anything is launched, when that is less than inpc_cdf_head_floats(n_leaves). */
#define INPC_CDF_HEAD_MIN_FLOATS 16384
size_t inpc_cdf_head_floats(uint32_t n_leaves);

/* Normalise the leaf weights and turn them into an inclusive CDF, in place.
 * Replaces compute_cdf (B/sampling/src/sampling.cu:150-186): cub::DeviceReduce::Sum, the
 * reciprocal-multiply normalisation (B/sampling/src/sampling_kernels.cu:66-75) and
 * cub::DeviceScan::InclusiveSum. The float association order is fixed: left-to-right inside
 * chunks of 64, chunk totals combined the same way one level up, recursively.
 * `sum_out` (dev, head_floats >= inpc_cdf_head_floats(n_leaves) floats, 16-byte aligned) is the head of
 * the CDF: [0]
 * receives the un-normalised total; when it is <= 0 the weights are left un-normalised and later
 * sampling kernels take the failure path themselves. [1 .. INPC_CDF_HEAD_MIN_FLOATS - 1] receive
 * the CDF elements that the first 14 probes of the binary search of B/sampling/src/
 * sampling_kernels.cu:101-126 can read, in heap order, and behind them those of the further
 * levels. Every later call that takes `sum_dev` takes this buffer. No host synchronisation.
 * Three launches whatever the size; at most 2^30 leaves (INPC_E_UNSUPPORTED beyond). */
int inpc_build_cdf(float* weights_inout, float* sum_out, size_t head_floats, void* workspace,
                   size_t workspace_bytes, uint32_t n_leaves, void* stream);

/* The same as inpc_build_cdf without a workspace argument: the chunk totals live in a scratch array
 * built into the library (264 KB of device memory per GPU the library runs on, held until the
 * process ends), so the call allocates nothing and takes nothing but inputs and outputs. It has no
 * counterpart in the reference; it is for callers that cannot allocate device memory or size a
 * workspace (code under HIP graph capture, tight serving loops, harnesses that forbid allocation).
 * At most INPC_BUILD_CDF_STATIC_MAX_LEAVES leaves (INPC_E_UNSUPPORTED beyond). All calls on one GPU
 * share the one scratch array: calls that overlap on one GPU (different streams or threads) race;
 * calls ordered on one stream do not. Nothing in the scratch has to be cleared between calls.
 * The first call of a process on a device looks the array's device address up (the runtime may load
 * the library's code object then): make one call outside any graph capture before capturing one. */
#define INPC_BUILD_CDF_STATIC_MAX_LEAVES 4194304u
int inpc_build_cdf_static(float* weights_inout, float* sum_out, size_t head_floats, uint32_t n_leaves,
                          void* stream);

/* Multinomial leaf pick + uniform in-leaf jitter, no culling.
 * Replaces create_samples (B/sampling/src/sampling.cu:188-209) and create_samples_cu
 * (B/sampling/src/sampling_kernels.cu:128-150). Sample i uses the generator `rng_dev`
 * advanced by 4*i draws; afterwards the device generator is advanced by 4*n_samples.
 * boxes (L,4) f32 as written by inpc_leaf_weights; positions_out (n,3) f32; leaf_ids_out (n,) i32
 * or NULL. If *sum_dev <= 0 nothing is written and the generator is left untouched. */
int inpc_sample(const float* boxes, const float* cdf, const float* sum_dev, size_t head_floats,
                float* positions_out, int32_t* leaf_ids_out, uint32_t n_samples, uint32_t n_leaves,
                uint64_t* rng_dev, void* stream);

/* Bytes of scratch for inpc_sample_cull_compact over up to n_candidates per round. */
size_t inpc_cull_workspace_bytes(uint32_t n_candidates);

/* Zero the round state (accepted count, consumed count) kept at the head of a cull
 * workspace: the zero-initialised sample_counter tensor of B/sampling/src/sampling_api.cu:72.
 * A round with k0 = 0 does the same by itself, so the call is only needed for a draw whose
 * first round starts at another candidate. */
int inpc_cull_begin(void* workspace, size_t workspace_bytes, void* stream);

/* One round of the training sampler: candidates k0 .. k0+n_candidates-1 of the counter-based
 * stream (candidate k uses the generator advanced by 4*k draws) are generated as in
 * inpc_sample, tested against the frustum, and the accepted ones appended, in ascending k,
 * to positions_out / leaf_ids_out behind the `accepted` count held in the workspace, up to
 * `capacity` entries.
 * Replaces create_training_samples_cu (B/sampling/src/sampling_kernels.cu:77-126); its
 * scheduling-dependent atomic slot order is replaced by ascending candidate order.
 * The workspace records, once `capacity` entries exist, how many candidates were consumed
 * (index of the last accepted candidate + 1). The generator is NOT advanced here; see
 * inpc_cull_finish. k0 = 0 starts a new draw: the state in the workspace is cleared first.
 * leaf_ids_out holds `capacity` int32 values, or int64 values when ids_int64 is not 0 (the dtype of
 * the tensor the reference returns, B/sampling/src/sampling_api.cu:71: written directly). */
int inpc_sample_cull_compact(const float* boxes, const float* cdf, const float* sum_dev,
                             size_t head_floats, const float* w2c, float* positions_out,
                             void* leaf_ids_out, int ids_int64, uint32_t capacity, uint32_t k0,
                             uint32_t n_candidates, uint32_t n_leaves, const inpc_camera* cam,
                             const uint64_t* rng_dev, void* workspace, size_t workspace_bytes,
                             void* stream);

/* Copy {accepted, consumed} of the current draw to host memory. Synchronises `stream`.
 * The one host read-back of a training draw; it stands where the reference reads the weight
 * sum back (B/sampling/src/sampling.cu:106-107) before launching its single sampling kernel. */
int inpc_cull_read_counts(const void* workspace, uint32_t* accepted_host, uint32_t* consumed_host,
                          void* stream);

/* End of a draw: advance the device generator by 4*consumed draws (4*total_candidates when
 * fewer than `capacity` samples were accepted), mirroring the host-side rng.advance of
 * B/sampling/src/sampling.cu:208. When *sum_dev <= 0 the outputs are filled with the
 * failure pattern of B/sampling/src/sampling.cu:107-111 (positions 0, ids -1).
 * total_candidates = INPC_CULL_IF_COMPLETE: the generator only moves if `capacity` samples were
 * accepted; a caller can enqueue this behind a round before it has read the counts back, and
 * makes the call again with the real number only if the draw needed more rounds. */
#define INPC_CULL_IF_COMPLETE 0xFFFFFFFFu
int inpc_cull_finish(const float* sum_dev, float* positions_out, void* leaf_ids_out, int ids_int64,
                     uint32_t capacity, uint32_t total_candidates, uint64_t* rng_dev,
                     void* workspace, size_t workspace_bytes, void* stream);

/* Widen int32 leaf ids to the int64 the Python API returns (B/sampling/src/sampling_api.cu:71),
 * for callers that drew int32 ids; inpc_sample_cull_compact writes int64 ids itself on request. */
int inpc_widen_ids(const int32_t* ids, int64_t* out, uint32_t n, void* stream);

/* Expected-count sampler, step 1: count[l] = w>0 ? max(1, rint(w*(1/sum)*n_samples)) : 0 and
 * its inclusive integer prefix sum. Replaces compute_sample_distribution
 * (B/sampling/src/sampling.cu:211-253), compute_sample_counts_cu
 * (B/sampling/src/sampling_kernels.cu:152-169). `weights` are the un-normalised leaf
 * weights; sum_out (dev) gets their total; offsets_out (L,) i32 dev gets the inclusive sums
 * (last entry = number of samples created). No host synchronisation. */
int inpc_expected_counts(const float* weights, float* sum_out, int32_t* offsets_out,
                         uint32_t n_samples, void* workspace, size_t workspace_bytes,
                         uint32_t n_leaves, void* stream);

/* Expected-count sampler, step 2: sample j (of n_created*n_multi) lies in leaf
 * ids[j mod n_created], where ids is the repeat-interleave of the counts, with three
 * jitters from the generator advanced by 3*j draws; afterwards the device generator is
 * advanced by 3*n_total. Replaces create_expected_samples (B/sampling/src/sampling.cu:255-287),
 * repeat_interleave_indices_cu and create_expected_samples_cu
 * (B/sampling/src/sampling_kernels.cu:171-205). leaf_ids_scratch (n_created,) i32 dev. */
int inpc_expected_samples(const float* centers, const int32_t* levels, const int32_t* offsets,
                          int32_t* leaf_ids_scratch, float* positions_out, uint32_t n_created,
                          uint32_t n_multi, uint32_t n_leaves, float initial_size,
                          uint64_t* rng_dev, void* stream);

/* =========================================================================================
 * Rasterizer
 * ======================================================================================= */

/* Geometry of a rasterizer call; fills the derived fields. */
typedef struct inpc_raster_config {
    uint32_t n_points;
    int32_t tile;         /* 8 (reference, B/rasterization/include/bilinear/config.h:23-25) or 16 */
    int32_t channels;     /* 4, 8 or 16 (4 for the SH modes)                                       */
    int32_t feature_mode; /* INPC_FEAT_*                                                           */
    uint32_t flags;       /* INPC_RASTER_*                                                         */
    inpc_camera cam;
    uint32_t max_instances; /* bilinear footprint: (point, touched tile) pairs the workspace holds; 0: about
                               1.06 (1 + 1/tile)^2 per point + 65536, what evenly spread points need with a
                               margin; 4 * n_points can never be exceeded. Ignored by the Gaussian footprint,
                               which takes its own (inpc_gaussian_config)                              */
} inpc_raster_config;

/* Offsets (bytes from the workspace base) of the buffers a caller may want to inspect.
 * The layout is private otherwise. Counts live in device memory.
 *
 * A drawn point owns the blend record at its own index in the record array (record_stride bytes):
 *   float wx0, wx1, wy0, wy1: interpolation weights of the pixel columns Lx, Lx + 1 and rows Ly, Ly + 1 that
 *     can lie closer than 1 to the point's screen position (L = floor(s - 0.5)), 0 where a pixel centre is 1
 *     or more away; float opacity; u32 point index | bit 28: touches several tiles | bit 29 / 30: two tiles in
 *     x / y; u32 (Lx + 1) | (Ly + 1) << 16; u32 first gradient row (training) or float depth (inference);
 *     then the view features (fp32, or fp16 for INPC_FEAT_DIRECT_F16).
 * The instances (point, touched tile) of tile t are instance_points[bin_start[t] .. bin_start[t + 1] - 1], in
 * (depth bits, point index) order. */
typedef struct inpc_raster_layout {
    size_t total_bytes;
    size_t counters;        /* u32[16]: [0] n_visible, [1] n_instances, [2] error flag,
                               [5] the instances do not fit max_instances: nothing was drawn      */
    size_t bin_start;       /* u32[n_tiles + 1]: first instance of every tile                      */
    size_t point_record;    /* (N) records of record_stride bytes, valid for drawn points          */
    size_t instance_points; /* (max_instances) u32: point index per instance in final order        */
    size_t tile_ranges;     /* (n_tiles) {u32 begin, end}; {0, 0} for a tile without instances      */
    size_t debug_geometry;  /* (N) {float sx, sy, depth; u32 tile info} with INPC_RASTER_KEEP_GEOMETRY,
                               else 0. tile info: bits 0-15 first tile, bit 16 / 17: two tiles in x / y,
                               bit 18: drawn                                                        */
    uint32_t record_stride;
    uint32_t grid_width;
    uint32_t grid_height;
    uint32_t n_tiles;
    uint32_t end_bit;       /* bit length of n_tiles-1
                               (B/rasterization/include/rasterization_utils.h:3-13)             */
    uint32_t depth_key_bias; /* instances are ordered by (float bits of the depth) - depth_key_bias */
    uint32_t max_instances; /* the capacity in effect                                            */
    uint32_t reserved;
} inpc_raster_layout;

/* Workspace size and layout for a configuration. Replaces the three growable blobs of
 * B/rasterization/include/bilinear/buffer_utils.h:24-115 and the resize callbacks of
 * B/rasterization/include/torch_utils.h:6-12 with one caller-owned worst-case buffer
 * (visible points <= N, instances <= 4N). */
int inpc_raster_layout_query(const inpc_raster_config* cfg, inpc_raster_layout* out);

/* Forward pass: project, cull, sort by (tile, depth, id), per-tile ranges, front-to-back
 * bilinear 2x2 splat blend.
 * Replaces forward_wrapper / inference_wrapper / inference_preextracted_wrapper
 * (B/rasterization/src/rasterization_api.cu:23-107,192-374) and bilinear::forward /
 * inference / inference_preextracted (B/rasterization/src/bilinear/forward.cu:12-170,
 * inference.cu:11-167, inference_preextracted.cu:11-168).
 *   positions (N,3) f32; features per cfg->feature_mode; opacities (N,) f32 (unused for
 *   INPC_FEAT_RAW37_F16); w2c (4,4) f32; cam_position (3,) f32 (SH modes only);
 *   image (C,H,W) f32; alpha (1,H,W) f32;
 *   blending_weights (N,) f32 (training) or NULL; depth_image (1,H,W) f32 (inference) or NULL.
 * The workspace is the saved state the backward pass needs. No host synchronisation. Everything is enqueued on
 * `stream` except the kernel that writes the blend records, which runs beside the tile sort on a second stream that
 * belongs to `stream` alone (created by the library the first time `stream` is used outside a graph capture, default
 * priority, kept until the process ends); `stream` waits for it before the blend, so to the caller the call is
 * ordered on `stream` like any other, and calls on different streams share nothing. A capture of `stream` takes its
 * second stream into the graph; a stream that is first seen while it is being captured gets none and runs
 * everything on itself (inpc_side_stream_policy). */
int inpc_raster_forward(const inpc_raster_config* cfg, const float* positions, const void* features,
                        const float* opacities, const float* w2c, const float* cam_position,
                        float* image, float* alpha, float* blending_weights, float* depth_image,
                        void* workspace, size_t workspace_bytes, void* stream);

/* The rule by which inpc_raster_forward decides about the second stream of a caller's stream, as a pure function
 * of what it finds (no GPU call): existing = a second stream for this (device, stream) exists; stream_is_capturing =
 * the caller's stream is being captured; second_is_capturing = the second stream is; n_kept = second streams the
 * process keeps. Returns 0: use the existing one, 1: create one, 2: none, everything runs on the caller's stream
 * (first seen during a capture; 256 kept already; or the second stream is still inside a capture its owner has
 * left, which happens when a capture was abandoned half-way). Library plumbing without a counterpart in the
 * reference, which has a single stream. */
int inpc_side_stream_policy(int existing, int stream_is_capturing, int second_is_capturing, int n_kept);

/* Backward pass: replays the blend front to back with the saved final image.
 * Replaces backward_wrapper (B/rasterization/src/rasterization_api.cu:109-190),
 * bilinear::backward (B/rasterization/src/bilinear/backward.cu:9-67), blend_backward_cu and
 * preprocess_backward_cu (B/rasterization/src/bilinear/kernels.cu:86-104,315-420).
 *   grad_image (C,H,W), grad_alpha (1,H,W), image, alpha: f32, as produced by forward;
 *   positions, cam_position: as in forward (read by the SH mode only, may be NULL otherwise);
 *   grad_features: (N,36) fp16 for INPC_FEAT_SH36_F16, (N,C) f32 for INPC_FEAT_DIRECT_F32,
 *                  (N,C) fp16 for INPC_FEAT_DIRECT_F16; fully written (zeros where a point
 *                  was not drawn);
 *   grad_opacities (N,) f32, fully written;
 *   grad_view_scratch: (N,C) f32 scratch for the SH and fp16 modes, else NULL.
 * The features and opacities themselves are not needed: the workspace holds what the blend used. */
int inpc_raster_backward(const inpc_raster_config* cfg, const float* grad_image,
                         const float* grad_alpha, const float* image, const float* alpha,
                         const float* positions, const float* cam_position, void* grad_features,
                         float* grad_opacities, float* grad_view_scratch, void* workspace,
                         size_t workspace_bytes, void* stream);

/* Copy the rasterizer counters {n_visible, n_instances, error flag} to the host.
 * Synchronises `stream`. Returns INPC_E_DEVICE if the error flag is set and INPC_E_WORKSPACE if the
 * instances did not fit max_instances (the images of that call show the background: call again
 * with a larger capacity; the reference reads the count back and resizes on every call,
 * B/rasterization/src/bilinear/forward.cu:86-89,118-119). */
int inpc_raster_read_counters(const inpc_raster_config* cfg, const void* workspace,
                              uint32_t counters_host[3], void* stream);

/* =========================================================================================
 * Rasterizer, Gaussian footprint (RasterizerMode.GAUSSIAN of
 * B/torch_bindings/rasterization.py:15-18; B/rasterization/src/gaussian/)
 * ======================================================================================= */

/* A point is drawn as a screen-space Gaussian: covariance from an isotropic world-space variance
 * through the Jacobian of the projection plus a dilation of 0.16, cut where it falls below a
 * threshold (B/rasterization/src/gaussian/kernels.cu:57-91, include/gaussian/config.h:19).
 *   training (base.flags without INPC_RASTER_INFERENCE): variance (0.3 * 0.5)^2 / (fx * fy),
 *     3-sigma tile bounds, threshold 0.01110899653 (kernels.cu:57-60,80-81,452); sigma_world and
 *     sigma_cutoff are ignored;
 *   inference: variance sigma_world^2, or scales[i]^2 when a scales array is passed; tile bounds
 *     sigma_cutoff * sigma - 0.5, threshold exp(-sigma_cutoff^2 / 2)
 *     (kernels.cu:166,186-187,268-273; inference.cu:170-171).
 * A point touches any number of tiles, so the instance buffers have a capacity the caller
 * chooses: max_instances (0: 4 * n_points + 65536). */
typedef struct inpc_gaussian_config {
    inpc_raster_config base;
    float sigma_world;
    float sigma_cutoff;
    uint32_t max_instances;
    uint32_t reserved;
} inpc_gaussian_config;

/* Offsets (bytes from the workspace base) of the buffers a caller may want to inspect. */
typedef struct inpc_gaussian_layout {
    size_t total_bytes;
    size_t counters;         /* u32[16]: [0] n_visible, [1] n_instances, [2] error flag,
                                [4] instances drawn (n_instances, or 0 when they do not fit)   */
    size_t point_touched;    /* (N) u32: tiles a point touches, 0 when it is not drawn          */
    size_t point_bounds;     /* (N) 4 x u16: x_min, x_max, y_min, y_max in tiles, half open     */
    size_t point_record;     /* (N) records of record_stride bytes, in point order:
                                float sx, sy, opacity, conic.x, conic.y, conic.z, depth (training
                                configurations, points that touch several tiles: u32 origin of
                                the point's gradient rows instead), u32 (bits 0-27 point id,
                                28-30 min(tile columns, 7), 31: touches more than one tile);
                                then the view features as fp32                                  */
    size_t depth_keys;       /* (N) u32, in point order: (float bits of the depth) - depth_key_bias,
                                0xFFFFFFFF for a point that is not drawn                        */
    size_t instance_points;  /* (max_instances) u32 point id per instance: the instances of tile
                                t are [tile_ranges[t].begin, .end), in (depth key, point id) order */
    size_t tile_ranges;      /* (n_tiles) {u32 begin, end}; {0, 0} for a tile without instances  */
    uint32_t record_stride;
    uint32_t grid_width;
    uint32_t grid_height;
    uint32_t n_tiles;
    uint32_t end_bit;
    uint32_t depth_key_bias;
    uint32_t max_instances;  /* the capacity in effect                                          */
    uint32_t reserved;
} inpc_gaussian_layout;

/* Workspace size and layout. Replaces the growable blobs of
 * B/rasterization/include/gaussian/buffer_utils.h:24-117 with one caller-owned buffer.
 * The workspace needs no clearing, whatever it held before. (Its backward pass tells the gradient
 * rows of the current pass from older ones by a 64-bit number that every forward pass takes from
 * the workspace and steps by one; in a workspace never used before, that number and the rows are
 * whatever the memory held, and an unwritten row passes for a written one only if 64 arbitrary
 * bits equal it.) */
int inpc_gaussian_layout_query(const inpc_gaussian_config* cfg, inpc_gaussian_layout* out);

/* Forward pass with the Gaussian footprint. Replaces the gaussian branches of forward_wrapper /
 * inference_wrapper / inference_preextracted_wrapper
 * (B/rasterization/src/rasterization_api.cu:79-100,248-269,336-360), gaussian::forward /
 * inference / inference_preextracted (B/rasterization/src/gaussian/forward.cu:12-172,
 * inference.cu:12-175, inference_preextracted.cu:11-177) and the kernels of
 * B/rasterization/src/gaussian/kernels.cu:11-324,346-474,581-660.
 *   Arguments as for inpc_raster_forward; scales (N,) f32 or NULL (inference only).
 *   blending_weights receive sum over pixels of G * blending weight (kernels.cu:456).
 * When the points touch more tiles than max_instances, counter [1] exceeds the capacity, no
 * instance is drawn (the images show the background) and inpc_gaussian_read_counters reports
 * it. No host synchronisation. */
int inpc_gaussian_forward(const inpc_gaussian_config* cfg, const float* positions,
                          const void* features, const float* opacities, const float* scales,
                          const float* w2c, const float* cam_position, float* image, float* alpha,
                          float* blending_weights, float* depth_image, void* workspace,
                          size_t workspace_bytes, void* stream);

/* Backward pass of the Gaussian footprint. Replaces the gaussian branch of backward_wrapper
 * (B/rasterization/src/rasterization_api.cu:165-184), gaussian::backward
 * (B/rasterization/src/gaussian/backward.cu:9-68), blend_backward_cu and preprocess_backward_cu
 * (B/rasterization/src/gaussian/kernels.cu:326-344,476-579). Arguments as for
 * inpc_raster_backward. The gradient of a point that touches several tiles is the sum of
 * per-instance rows in the workspace, taken in a fixed order, and an instance's row is a sum
 * in a fixed order as well (also for footprints of many pixels): no float atomics, the same
 * bits on every run (the reference adds with atomics, kernels.cu:548-571).
 * The workspace must be the one the forward pass of the same inputs has filled. Like the
 * forward pass it only enqueues kernels, so forward + backward can be captured in a graph
 * and replayed with new inputs written in place. */
int inpc_gaussian_backward(const inpc_gaussian_config* cfg, const float* grad_image,
                           const float* grad_alpha, const float* image, const float* alpha,
                           const float* positions, const float* cam_position, void* grad_features,
                           float* grad_opacities, float* grad_view_scratch, void* workspace,
                           size_t workspace_bytes, void* stream);

/* Copy {n_visible, n_instances, error flag, instances drawn} to the host; synchronises `stream`.
 * Returns INPC_E_DEVICE if the error flag is set and INPC_E_WORKSPACE if n_instances exceeds
 * max_instances (the images of that call are incomplete: call again with a larger capacity; the
 * reference reads the count back and resizes, B/rasterization/src/gaussian/forward.cu:87-90,118-119). */
int inpc_gaussian_read_counters(const inpc_gaussian_config* cfg, const void* workspace,
                                uint32_t counters_host[4], void* stream);

/* =========================================================================================
 * Probability-field statistics (the consumer of the sampler's leaf indices and the
 * rasterizer's blending weights, once per training iteration)
 * ======================================================================================= */

/* Bytes of scratch for inpc_field_update over n_leaves leaves. */
size_t inpc_field_update_workspace_bytes(uint32_t n_leaves);

/* leaf_weights *= decay; leaf_scores *= decay; then, with max_s / min_s the per-leaf maximum /
 * minimum of `weights` over the samples whose index names the leaf (0 for a leaf without
 * samples), leaf_weights = max(leaf_weights, max_s) and
 * leaf_scores = max(leaf_scores, clamp(max_s - min_s, 0, 1)), all in place.
 * Replaces ProbabilityField.update (Modules/ProbabilityField.py:146-157): two mul_, two
 * scatter_reduce_ (amax / amin, include_self=False) and two torch.maximum.
 * indices (n,) i64 dev (the leaf indices generate_training_samples returned), weights (n,) f32
 * dev (blending weights), leaf_weights / leaf_scores (L,) f32 dev. An index outside [0, L) is
 * skipped and recorded; inpc_field_update_check reports it. No host synchronisation. */
int inpc_field_update(const int64_t* indices, const float* weights, uint32_t n_samples,
                      float* leaf_weights, float* leaf_scores, uint32_t n_leaves, float decay,
                      void* workspace, size_t workspace_bytes, void* stream);

/* INPC_E_INVALID_ARGUMENT if the last inpc_field_update on this workspace met an index outside
 * [0, n_leaves) (the reference's scatter_reduce_ raises for those). Synchronises `stream`. */
int inpc_field_update_check(const void* workspace, void* stream);

/* =========================================================================================
 * Element-wise steps between the sampler and the rasterizer
 * ======================================================================================= */

/* contracted = saturate(scale * p + 0.5), scale = (2 sqrt(L) - 1) / L / 4, L = max(|p|^2, 1):
 * the unit ball maps linearly into [0.25, 0.75]^3, everything outside into the rest of the unit
 * cube. Replaces spherical_contraction_cu (B/misc/src/misc_kernels.cu:49-66) behind
 * spherical_contraction (B/torch_bindings/misc.py:17-18). positions, contracted (n,3) f32 dev. */
int inpc_spherical_contraction(const float* positions, float* contracted, uint32_t n_points,
                               void* stream);

/* opacity = -expm1(-exp(raw)), element-wise: feature_to_opacity (utils.py:31-33) with the
 * forward of TruncExp (utils.py:13-22). raw, opacity (n,) f32 dev. */
int inpc_opacity_forward(const float* raw, float* opacity, size_t n, void* stream);

/* grad_raw = grad_opacity * exp(-exp(raw)) * exp(clamp(raw, -15, 15)): the backward of the same
 * expression, the truncated exponential's gradient as in TruncExp.backward (utils.py:24-28). */
int inpc_opacity_backward(const float* grad_opacity, const float* raw, float* grad_raw, size_t n,
                          void* stream);

/* Ordered selections over the leaves of the probability field. A leaf is selected when
 * values[i] > threshold and (levels == NULL or levels[i] < max_level).
 * inpc_field_select_workspace_bytes: scratch for n_leaves leaves.
 * inpc_field_select_count: count_out (1 u32 dev) = number of selected leaves; replaces the mask sums
 * `valid_mask.sum()` (Modules/ProbabilityField.py:222) and the shape of `self.leaf_weights[mask]`
 * (:161): the caller reads it to size the outputs of the two calls below. */
size_t inpc_field_select_workspace_bytes(uint32_t n_leaves);
int inpc_field_select_count(const float* values, const int32_t* levels, uint32_t n_leaves,
                            float threshold, int max_level, uint32_t* count_out, void* workspace,
                            size_t workspace_bytes, void* stream);

/* Keeps the leaves with weights[i] > threshold, in order. Replaces ProbabilityField.prune
 * (Modules/ProbabilityField.py:159-165). Outputs hold at least the selected count (n_leaves
 * always suffices); count_out (1 u32 dev) receives it. centers (n,3) f32, levels (n,) i32. */
int inpc_field_prune(const float* centers, const int32_t* levels, const float* weights,
                     const float* scores, uint32_t n_leaves, float threshold, float* centers_out,
                     int32_t* levels_out, float* weights_out, float* scores_out,
                     uint32_t* count_out, void* workspace, size_t workspace_bytes, void* stream);

/* Splits the leaves with scores[i] > threshold and levels[i] < max_level into eight children
 * each. Replaces the array part of ProbabilityField.subdivide
 * (Modules/ProbabilityField.py:217-257): outputs = the other leaves in order, then the children,
 * parents in order, child j
 * at centre -/+ initial_size / 2^(level + 2) per axis (+ in x for odd j, in y for j % 4 >= 2, in
 * z for j >= 4), level + 1, the parent's weight, score 0. count_out (1 u32 dev) receives the
 * number s of split leaves; outputs must hold n_leaves + 7 s leaves (s from
 * inpc_field_select_count with the same arguments). The reference's size limit (:223-224) is
 * the caller's decision between the two calls. initial_size: 3 floats on the host. */
int inpc_field_subdivide(const float* centers, const int32_t* levels, const float* weights,
                         const float* scores, uint32_t n_leaves, float threshold, int max_level,
                         const float initial_size[3], float* centers_out, int32_t* levels_out,
                         float* weights_out, float* scores_out, uint32_t* count_out,
                         void* workspace, size_t workspace_bytes, void* stream);

/* Quasi-random positions from per-leaf sample counts: the deterministic part of
 * ProbabilityField.extract_global (Modules/ProbabilityField.py:131-140) with compute_halton_coords /
 * generate_halton_sequence / halton_base (utils.py:36-64). Sample s lies in the leaf whose run of
 * the exclusive sum of `counts` holds it; with h its 0-based number in that run, its position is
 * centre - size / 2 + halton(h + 1; 2, 3, 5) * size, size = initial_size / 2^level, or the centre
 * when the leaf has one sample. The radical inverses are accumulated in double precision as in
 * the reference's Python loop and rounded to float once, so the positions are bit-identical.
 * counts (L,) i64 dev as torch.bincount returns them; positions_out (n_samples, 3) f32 dev;
 * initial_size: 3 floats on the host. The multinomial draw in front (:130) stays with the caller;
 * inpc_morton_encode gives the codes of the optional order behind (:141-143).
 * inpc_extract_global_check synchronises and fails unless the counts are in range and add
 * up to n_samples. */
size_t inpc_extract_global_workspace_bytes(uint32_t n_leaves);
int inpc_extract_global(const float* centers, const int32_t* levels, const int64_t* counts,
                        uint32_t n_leaves, const float initial_size[3], float* positions_out,
                        uint32_t n_samples, void* workspace, size_t workspace_bytes, void* stream);
int inpc_extract_global_check(const void* workspace, uint32_t n_samples, void* stream);

/* codes_out[i] = 63-bit Morton code of positions[i] in the bounding cube of all positions: with lo
 * the per-axis minimum and e the largest per-axis extent, cell_a = min(uint((p_a - lo_a) *
 * (2^21 / e)), 2^21 - 1) in fp32 (all cells 0 when e = 0), and bit k of cell_x / cell_y / cell_z
 * is bit 3k / 3k + 1 / 3k + 2 of the code. Sorting by the code (torch.argsort, as the caller does)
 * gives the order ProbabilityField.extract_global asks for with use_morton_order
 * (Modules/ProbabilityField.py:141-143). The reference takes the codes from
 * CudaUtils.MortonEncoding.morton_encode, an extension of its framework whose source is not part
 * of the reference tree: this is the textbook Z-order code, equal to the reference's only as far
 * as both are Morton orders of the same points. positions (n, 3) f32 dev, codes_out (n,) i64 dev,
 * workspace: inpc_morton_workspace_bytes() bytes. No host synchronisation. */
size_t inpc_morton_workspace_bytes(void);
int inpc_morton_encode(const float* positions, uint32_t n, int64_t* codes_out, void* workspace,
                       size_t workspace_bytes, void* stream);

/* grads (= or +=, `add` != 0) factor(i) * weights[i], factor = 0.1 * 2 / (entries of the hash-grid
 * level that holds flat index i), 0 in front of index 6144. Replaces
 * compute_normalized_weight_decay_grads_cu<add> (B/misc/src/misc_kernels.cu:6-47) behind
 * compute_normalized_weight_decay_grads / add_normalized_weight_decay_grads
 * (B/torch_bindings/misc.py:9-14). weights, grads (n,) f32 dev. */
int inpc_weight_decay_grads(const float* weights, float* grads, uint32_t n_weights, int add,
                            void* stream);

/* elementwise_loss[i] = log1p(12.5 (input[i] - target[i])^2) / n. Replaces cauchy_loss_cu
 * (B/misc/src/misc_kernels.cu:68-79); the caller sums (B/misc/src/misc_api.cu:51-65). */
int inpc_cauchy_loss(const float* input, const float* target, float* elementwise_loss, uint32_t n,
                     void* stream);

/* grad_input[i] = 25 d / max(n (12.5 d^2 + 1), 1e-12) * grad[0], d = input[i] - target[i].
 * Replaces cauchy_loss_backward_cu (B/misc/src/misc_kernels.cu:81-94). grad: 1 f32 dev. */
int inpc_cauchy_loss_backward(const float* grad, const float* input, const float* target,
                              float* grad_input, uint32_t n, void* stream);

/* Per-kernel timing hooks for benchmarks: when enabled, every launch made by the calling
 * thread is bracketed by HIP events on its stream; inpc_timing_collect synchronises and
 * returns the number of records written as {name, milliseconds}. */
typedef struct inpc_timing_record {
    const char* name;
    float ms;
} inpc_timing_record;
void inpc_timing_enable(int on);
int inpc_timing_collect(inpc_timing_record* out, int capacity);

/* Plain device-to-device copy kernel (reads `bytes`, writes `bytes`; both dev, 16-byte
 * aligned, bytes a multiple of 16). It exists so that a profiler's memory counters can be
 * scaled by what they read for a kernel whose traffic is known; no counterpart in the
 * reference. */
int inpc_calibration_copy(const void* src, void* dst, size_t bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* INPC_HIP_H */
