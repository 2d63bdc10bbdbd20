// blend.hpp — front-to-back alpha blending of the sorted instance lists, forward and backward
// (B/rasterization/src/bilinear/kernels.cu:241-495). Included by raster.hip after the record helpers.
//
// One block per tile, one thread per pixel. A wave owns 64 pixels on an 8 x 8 grid: the whole tile for 8x8
// tiles; for 16x16 tiles the pixels of one parity class (x odd / even, y odd / even), so that the 2 x 2
// footprint of a point gives every wave exactly one fragment and a cluster of points on one spot loads the
// four waves evenly. Per batch of T*T instances:
//   stage    thread t gathers the record of instance t into LDS, finds the waves ("quads") in which it covers a
//            pixel that is still open, and appends t, in depth order, to the list of each such quad;
//   consume  every wave walks its own list, 64 instances at a time, with wave-level
//            synchronisation only: coverage bit masks per pixel column / row -> per-pixel fragment lists
//            in depth order -> the sequential transmittance chain per pixel (short lists) or a wave-wide
//            product scan (long lists) -> per-instance results into LDS;
//   write    thread t writes the result of instance t: a plain store when the point lies in one tile only,
//            atomics when it straddles tiles.
// Two block barriers per batch; the record gather runs two batches ahead of the blend.
#pragma once

namespace blend {

constexpr int kQuad = 8;             // a wave's pixel quad is 8 x 8
#ifndef INPC_LONG_LIST
#define INPC_LONG_LIST 12
#endif
constexpr uint32_t kLongList = INPC_LONG_LIST;  // lists longer than this are evaluated by the whole wave

__device__ __forceinline__ uint64_t lanes_below() {
    const uint32_t lane = __lane_id();
    return lane == 0u ? 0ull : (~0ull >> (64u - lane));
}

// ---- wave-wide scans and sums through DPP (no LDS round trips) -------------------------------------------------
// update_dpp(old, src, ctrl, row_mask, bank_mask, bound_ctrl): a lane whose source lane does not exist, or whose
// row is masked out, keeps `old`; passing the operation's identity as `old` makes every step unconditional.
constexpr int kDppRowShr1 = 0x111, kDppRowShr2 = 0x112, kDppRowShr4 = 0x114, kDppRowShr8 = 0x118;
constexpr int kDppRowBcast15 = 0x142, kDppRowBcast31 = 0x143, kDppWaveShr1 = 0x138;

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_take(float old, float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(old), __float_as_int(v), CTRL, ROW_MASK, 0xf, false));
}

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_take(uint32_t old, uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp((int)old, (int)v, CTRL, ROW_MASK, 0xf, false);
}

// T_i = (...((t_in * m_0) * m_1)...) * m_i for the lanes i < n, multiplied strictly left to right: the result is
// bit-identical to a sequential walk, which the early-out test against the transmittance threshold needs
// (a product taken in tree order may land on the other side of the threshold). Every step, every lane takes
// its left neighbour's value (lane 0: t_in) times its own factor: after step s the lanes 0..s hold their final
// value, and computing a final value again from a final neighbour reproduces it. One multiply per step, no LDS.
// (Steps beyond n only recompute final values, so the loop runs in unrolled groups of eight.)
__device__ __forceinline__ float wave_sequential_product(float m, float t_in, uint32_t n) {
    float x = m;
    for (uint32_t s = 0; s < n; s += 8u) {
#pragma unroll
        for (int u = 0; u < 8; ++u) x = dpp_take<kDppWaveShr1, 0xf>(t_in, x) * m;
    }
    return x;
}

__device__ __forceinline__ float wave_inclusive_sum(float v) {
    v += dpp_take<kDppRowShr1, 0xf>(0.0f, v);
    v += dpp_take<kDppRowShr2, 0xf>(0.0f, v);
    v += dpp_take<kDppRowShr4, 0xf>(0.0f, v);
    v += dpp_take<kDppRowShr8, 0xf>(0.0f, v);
    v += dpp_take<kDppRowBcast15, 0xa>(0.0f, v);
    v += dpp_take<kDppRowBcast31, 0xc>(0.0f, v);
    return v;
}

// Value of the lane in front (lane 0: `first`).
__device__ __forceinline__ float wave_previous(float v, float first) { return dpp_take<kDppWaveShr1, 0xf>(first, v); }

// Sum over all 64 lanes, the same value in every lane.
__device__ __forceinline__ float wave_sum(float v) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wave_inclusive_sum(v)), 63));
}

__device__ __forceinline__ uint32_t wave_exclusive_sum(uint32_t v, uint32_t& total) {
    uint32_t incl = v;
    incl += dpp_take<kDppRowShr1, 0xf>(0u, incl);
    incl += dpp_take<kDppRowShr2, 0xf>(0u, incl);
    incl += dpp_take<kDppRowShr4, 0xf>(0u, incl);
    incl += dpp_take<kDppRowShr8, 0xf>(0u, incl);
    incl += dpp_take<kDppRowBcast15, 0xa>(0u, incl);
    incl += dpp_take<kDppRowBcast31, 0xc>(0u, incl);
    total = (uint32_t)__builtin_amdgcn_readlane((int)incl, 63);
    return incl - v;
}

// Per-block staging area of one batch.
//   NQ  waves ("quads") per tile
//   NF  fragments one instance can have inside one wave's pixel grid: 4 (8x8 tiles: the whole 2 x 2 footprint),
//       1 (16x16 tiles: one pixel per parity class)
template <int T, int C, bool WITH_DEPTH>
struct Stage {
    static constexpr int TT = T * T;
    static constexpr int NQ = TT / 64;
    static constexpr int NF = T == 16 ? 1 : 4;
    float opacity[TT];
    float4 feat[TT * (C / 4)];
    float depth[WITH_DEPTH ? TT : 1];
    float weight[NQ][NF][TT];   // interpolation weight of the fragment
    uint8_t pixel[NQ][NF][TT];  // its pixel in the wave's grid (row * 8 + column), kNoPixel: no fragment
    float2 result[NQ][NF][TT];  // what the blend made of the fragment (written by the quad's wave, else {0, 0})
    uint8_t list[NQ][NQ][64];   // [quad][source wave][rank]: staged instances with an open pixel in the quad
    uint8_t count[NQ][NQ];
    uint64_t done[NQ];          // per quad: pixels that are finished
};
constexpr uint32_t kNoPixel = 0xFFu;

// Per-wave scratch of the consume phase. A fragment entry is {alpha, x} on the way in and {blending weight, y}
// on the way out; forward: x = staged instance; backward: x = features . grad, y = d loss / d alpha.
template <int NF>
struct QuadScratch {
    uint64_t hits[64];          // per pixel: lanes (instances of the sub-batch) that hit it
    float2 fragment[64 * NF];   // per fragment, pixel by pixel, in depth order
};

// The record header as the kernels use it.
struct Header {
    float sx, sy, opacity;
    uint32_t point;
    uint32_t tiles;  // raw word; see multi()
    float depth;
    // the point touches more than one tile (kept as the raw word until the write phase: a flag derived
    // at the load would make the gather wait for its own first reply)
    __device__ __forceinline__ bool multi() const { return ((tiles >> 16) & 3u) != 0u; }
};

// Makes the value available here: the wait for an outstanding load that produces it lands at this point and not
// at a later first use.
__device__ __forceinline__ void arrive(float& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void arrive(uint32_t& v) { asm volatile("" : "+v"(v)); }

__device__ __forceinline__ Header read_header(const char* __restrict__ record) {
    const float4 h0 = ((const float4*)record)[0];
    const float4 h1 = ((const float4*)record)[1];
    Header h;
    h.sx = h0.x;
    h.sy = h0.y;
    h.opacity = h0.z;
    h.point = __float_as_uint(h0.w);
    h.tiles = __float_as_uint(h1.x);
    h.depth = h1.y;
    return h;
}

// Stage instance `t` (thread t): features and opacity, the fragment it has in every quad (pixel + weight), and
// its entry, in depth order, in the list of each quad where it covers an open pixel. `valid` is false for the
// threads behind the end of the batch. Must be followed by a block barrier.
template <int T, int C, bool WITH_DEPTH>
__device__ __forceinline__ void stage_instance(Stage<T, C, WITH_DEPTH>& st, bool valid, const Header& h,
                                               const float (&f)[C], int tile_x0, int tile_y0) {
    constexpr int NQ = T * T / 64;
    const uint32_t t = threadIdx.x, lane = t & 63u, wave = t >> 6;
    bool in_quad[NQ];
#pragma unroll
    for (int q = 0; q < NQ; ++q) in_quad[q] = false;
    if (valid) {
        st.opacity[t] = h.opacity;
#pragma unroll
        for (int q4 = 0; q4 < C / 4; ++q4) st.feat[t * (C / 4) + q4] = make_float4(f[4 * q4], f[4 * q4 + 1], f[4 * q4 + 2], f[4 * q4 + 3]);
        if (WITH_DEPTH) st.depth[t] = h.depth;
        // the float test of B/rasterization/src/bilinear/kernels.cu:284-287 for the 2 x 2 candidate pixels
        const AxisCover ax = cover_axis<T>(h.sx, tile_x0), ay = cover_axis<T>(h.sy, tile_y0);
#pragma unroll
        for (int ky = 0; ky < 2; ++ky)
#pragma unroll
            for (int kx = 0; kx < 2; ++kx) {
                const bool hit = ax.hit[kx] && ay.hit[ky];
                const int cx = ax.first + kx, cy = ay.first + ky;
                if (T == 16) {
                    // quad = parity class of the pixel; every class has exactly one of the four candidates
                    const int q = (cy & 1) * 2 + (cx & 1);
                    const int pix = hit ? (cy >> 1) * 8 + (cx >> 1) : 0;
                    const bool open = hit && ((st.done[q] >> pix) & 1ull) == 0ull;
                    st.pixel[q][0][t] = hit ? (uint8_t)pix : (uint8_t)kNoPixel;
                    st.weight[q][0][t] = ax.weight[kx] * ay.weight[ky];
#pragma unroll
                    for (int qq = 0; qq < NQ; ++qq)
                        if (qq == q && open) in_quad[qq] = true;
                } else {
                    const int pix = hit ? cy * 8 + cx : 0;
                    const bool open = hit && ((st.done[0] >> pix) & 1ull) == 0ull;
                    st.pixel[0][ky * 2 + kx][t] = hit ? (uint8_t)pix : (uint8_t)kNoPixel;
                    st.weight[0][ky * 2 + kx][t] = ax.weight[kx] * ay.weight[ky];
                    if (open) in_quad[0] = true;
                }
            }
    }
#pragma unroll
    for (int q = 0; q < NQ; ++q)
#pragma unroll
        for (int k = 0; k < Stage<T, C, WITH_DEPTH>::NF; ++k) st.result[q][k][t] = make_float2(0.0f, 0.0f);
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
        const uint64_t members = __ballot(in_quad[q]);
        if (in_quad[q]) st.list[q][wave][mask_rank(members)] = (uint8_t)t;
        if (lane == 0u) st.count[q][wave] = (uint8_t)__popcll(members);
    }
}

// A quad's list is the concatenation, in wave order, of the pieces the NQ source waves wrote. ListIndex holds
// the piece boundaries of one batch (the same in every lane).
template <int NQ>
struct ListIndex {
    uint32_t end[NQ];  // end[s]: entries in the pieces 0..s; end[NQ - 1] is the length of the list
};

template <int T, int C, bool WITH_DEPTH>
__device__ __forceinline__ ListIndex<T * T / 64> list_index(const Stage<T, C, WITH_DEPTH>& st, uint32_t q) {
    constexpr int NQ = T * T / 64;
    ListIndex<NQ> li;
    uint32_t run = 0;
#pragma unroll
    for (int s = 0; s < NQ; ++s) {
        run += st.count[q][s];
        li.end[s] = (uint32_t)__builtin_amdgcn_readfirstlane((int)run);
    }
    return li;
}

// The idx-th staged instance of quad q's list, idx < li.end[NQ - 1].
template <int T, int C, bool WITH_DEPTH>
__device__ __forceinline__ uint32_t list_entry(const Stage<T, C, WITH_DEPTH>& st, const ListIndex<T * T / 64>& li,
                                               uint32_t q, uint32_t idx) {
    constexpr int NQ = T * T / 64;
    uint32_t w = 0, first = 0;
#pragma unroll
    for (int s = 0; s < NQ - 1; ++s)
        if (idx >= li.end[s]) {
            w = s + 1;
            first = li.end[s];
        }
    return st.list[q][w][idx - first];
}

// Fragments of one sub-batch lane: the (at most NF) pixels staged instance j covers in this wave's grid.
template <int NF>
struct LaneFragments {
    uint32_t pixel[NF];  // kNoPixel: none, or the pixel is finished
    float weight[NF];
    uint32_t where[NF];  // position in the fragment list (valid when pixel != kNoPixel)
};

// Per-pixel fragment lists of one sub-batch. In: every lane's fragments (pixel, weight), the alpha factor
// `opacity`, and payload(q), the second word of fragment q's entry. Out: every pixel lane's list
// [my_start, my_start + my_count) of {alpha, payload} in depth order in qs.fragment, and `where` for every
// fragment. Every lane of the wave must call it.
template <int NF, typename Payload>
__device__ __forceinline__ void build_fragment_lists(QuadScratch<NF>& qs, float opacity, LaneFragments<NF>& lf,
                                                     uint32_t& my_start, uint32_t& my_count, uint32_t& n_fragments,
                                                     Payload payload) {
    const uint32_t lane = __lane_id();
    qs.hits[lane] = 0ull;
    wave_sync();
    const unsigned long long bit = 1ull << lane;
#pragma unroll
    for (int q = 0; q < NF; ++q)
        if (lf.pixel[q] != kNoPixel) atomicOr((unsigned long long*)&qs.hits[lf.pixel[q]], bit);
    wave_sync();
    my_count = (uint32_t)__popcll(qs.hits[lane]);
    my_start = wave_exclusive_sum(my_count, n_fragments);
    if (n_fragments == 0u) return;
    const uint64_t below = lanes_below();
#pragma unroll
    for (int q = 0; q < NF; ++q) {
        const bool hit = lf.pixel[q] != kNoPixel;
        const uint32_t pix = hit ? lf.pixel[q] : 0u;
        const uint32_t start = __shfl(my_start, pix, 64);  // every lane takes part in the exchange
        if (hit) {
            const uint32_t pos = start + (uint32_t)__popcll(qs.hits[pix] & below);
            lf.where[q] = pos;
            qs.fragment[pos] = make_float2(opacity * lf.weight[q], payload(q));
        }
    }
    wave_sync();
}

// Lane l of a sub-batch: its staged instance and fragments (pixels that finished since staging are dropped).
template <int T, int C, bool WITH_DEPTH>
__device__ __forceinline__ void load_lane_fragments(const Stage<T, C, WITH_DEPTH>& st, uint32_t quad, bool live,
                                                    uint32_t j, uint64_t finished,
                                                    LaneFragments<Stage<T, C, WITH_DEPTH>::NF>& lf) {
    constexpr int NF = Stage<T, C, WITH_DEPTH>::NF;
#pragma unroll
    for (int q = 0; q < NF; ++q) {
        uint32_t pix = live ? (uint32_t)st.pixel[quad][q][j] : kNoPixel;
        if (pix != kNoPixel && ((finished >> pix) & 1ull)) pix = kNoPixel;
        lf.pixel[q] = pix;
        lf.weight[q] = st.weight[quad][q][j];
        lf.where[q] = 0u;
    }
}

// ---- the record gather, two batches ahead -------------------------------------------------------------------------
// Per thread: the record of the batch being staged, the record of the batch after it (requested one batch
// earlier, still in flight or arrived) and the slot of the batch after that.
template <int C>
struct Gather {
    Header h;
    float f[C];
    Header h_next;
    float f_next[C];
    uint32_t next_slot;
};

template <int T, int C, bool HALF>
__device__ __forceinline__ void start_gather(Gather<C>& g, const uint32_t* __restrict__ inst_slots,
                                             const char* __restrict__ records, uint32_t stride, uint2 range) {
    constexpr uint32_t TT = T * T;
    const uint32_t at = range.x + threadIdx.x;
    g.h = Header{};
    g.h_next = Header{};
#pragma unroll
    for (int c = 0; c < C; ++c) g.f[c] = g.f_next[c] = 0.0f;
    g.next_slot = 0u;
    uint32_t slot0 = 0u, slot1 = 0u;
    if (at < range.y) slot0 = inst_slots[at];
    if (at + TT < range.y) slot1 = inst_slots[at + TT];
    if (at + 2u * TT < range.y) g.next_slot = inst_slots[at + 2u * TT];
    if (at < range.y) {
        const char* record = records + (size_t)slot0 * stride;
        g.h = read_header(record);
        load_record_features<C, HALF>(g.f, record);
    }
    if (at + TT < range.y) {
        const char* record = records + (size_t)slot1 * stride;
        g.h_next = read_header(record);
        load_record_features<C, HALF>(g.f_next, record);
    }
}

// Called at the end of the batch that starts at `begin`, in front of the stores of its write phase, so that
// waiting for the gather never waits for those stores: takes the record of the next batch (requested a whole
// batch ago) and requests the record of the batch after it and the slot of the one after that.
template <int T, int C, bool HALF>
__device__ __forceinline__ void advance_gather(Gather<C>& g, const uint32_t* __restrict__ inst_slots,
                                               const char* __restrict__ records, uint32_t stride, uint32_t begin,
                                               uint32_t end) {
    constexpr uint32_t TT = T * T;
    const uint32_t at = begin + threadIdx.x;
    arrive(g.h_next.sx);
    arrive(g.h_next.sy);
    arrive(g.h_next.opacity);
    arrive(g.h_next.point);
    arrive(g.h_next.tiles);
    arrive(g.h_next.depth);
#pragma unroll
    for (int c = 0; c < C; ++c) arrive(g.f_next[c]);
    arrive(g.next_slot);
    g.h = g.h_next;
#pragma unroll
    for (int c = 0; c < C; ++c) g.f[c] = g.f_next[c];
    if (at + 2u * TT < end) {
        const char* record = records + (size_t)g.next_slot * stride;
        g.h_next = read_header(record);
        load_record_features<C, HALF>(g.f_next, record);
    }
    if (at + 3u * TT < end) g.next_slot = inst_slots[at + 3u * TT];
}

// ---- forward ------------------------------------------------------------------------------------------------------
template <int T, int C, bool HALF, bool INFERENCE>
__global__ void __launch_bounds__(T* T)
    k_blend_forward(const uint2* __restrict__ ranges, const uint32_t* __restrict__ tile_order,
                    const uint32_t* __restrict__ inst_slots,
                    const char* __restrict__ records, uint32_t stride, float* __restrict__ image,
                    float* __restrict__ alpha_image, float* blending_weights, float* __restrict__ depth_image, int W,
                    int H, uint32_t gw) {
    constexpr int TT = T * T;
    constexpr int NQ = TT / 64;
    constexpr int NF = Stage<T, C, INFERENCE>::NF;
    __shared__ Stage<T, C, INFERENCE> st;
    __shared__ QuadScratch<NF> s_quad[NQ];

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t tile = tile_order[blockIdx.x];
    const int tile_x0 = (int)(tile % gw) * T, tile_y0 = (int)(tile / gw) * T;
    const int px = tile_x0 + (T == 16 ? 2 * (int)(lane & 7u) + (int)(wave & 1u) : (int)(lane & 7u));
    const int py = tile_y0 + (T == 16 ? 2 * (int)(lane >> 3) + (int)(wave >> 1) : (int)(lane >> 3));
    const bool inside = px < W && py < H;
    QuadScratch<NF>& qs = s_quad[wave];

    float F[C];
#pragma unroll
    for (int c = 0; c < C; ++c) F[c] = 0.0f;
    float D = 0.0f, Tr = 1.0f;
    bool done = !inside;
    {
        const uint64_t finished = __ballot(done);
        if (lane == 0u) st.done[wave] = finished;
    }
    __syncthreads();

    const uint2 range = ranges[tile];
#ifdef INPC_PROFILE_BACKWARD
#define FWD_MARK(i)
#else
    INPC_PROF_DECL;
#define FWD_MARK(i) INPC_PROF_MARK(i)
#endif
    Gather<C> g;
    start_gather<T, C, HALF>(g, inst_slots, records, stride, range);
    for (uint32_t begin = range.x; begin < range.y; begin += TT) {
        const uint32_t count = min((uint32_t)TT, range.y - begin);
        const bool valid = tid < count;
        stage_instance<T, C, INFERENCE>(st, valid, g.h, g.f, tile_x0, tile_y0);
        FWD_MARK(0);
        __syncthreads();
        FWD_MARK(1);

        // ---- consume: this wave's list
        const ListIndex<NQ> li = list_index<T, C, INFERENCE>(st, wave);
        const uint32_t total = li.end[NQ - 1];
        for (uint32_t sub = 0; sub < total; sub += 64u) {
            const bool live = sub + lane < total;
            const uint32_t j = live ? list_entry<T, C, INFERENCE>(st, li, wave, sub + lane) : 0u;
            LaneFragments<NF> lf;
            load_lane_fragments<T, C, INFERENCE>(st, wave, live, j, __ballot(done), lf);
            uint32_t my_start, my_count, n_fragments;
            build_fragment_lists<NF>(qs, st.opacity[j], lf, my_start, my_count, n_fragments,
                                     [&](int) { return __uint_as_float(j); });
            FWD_MARK(2);
            if (n_fragments == 0u) continue;
            // ---- pixels with short lists: the reference's sequential walk (kernels.cu:281-299)
            if (my_count <= kLongList) {
                for (uint32_t i = 0; i < my_count; ++i) {
                    const uint32_t pos = my_start + i;
                    const float2 e = qs.fragment[pos];
                    const float a = done ? 0.0f : e.x;
                    const uint32_t jj = __float_as_uint(e.y);
                    const float bw = Tr * a;
                    qs.fragment[pos].x = bw;
#pragma unroll
                    for (int q4 = 0; q4 < C / 4; ++q4) {
                        const float4 v = st.feat[jj * (C / 4) + q4];
                        F[4 * q4] = fmaf(bw, v.x, F[4 * q4]);
                        F[4 * q4 + 1] = fmaf(bw, v.y, F[4 * q4 + 1]);
                        F[4 * q4 + 2] = fmaf(bw, v.z, F[4 * q4 + 2]);
                        F[4 * q4 + 3] = fmaf(bw, v.w, F[4 * q4 + 3]);
                    }
                    if (INFERENCE) D = fmaf(bw, st.depth[jj], D);
                    Tr *= 1.0f - a;
                    done = done || Tr < kTransmittanceThreshold;
                }
            }
            FWD_MARK(3);
            // ---- pixels with long lists, one after the other, 64 fragments at a time over the wave
            uint64_t long_pixels = __ballot(my_count > kLongList);
            while (long_pixels) {
                const int p = __builtin_ctzll(long_pixels);
                long_pixels &= long_pixels - 1ull;
                const uint32_t p_start = __shfl(my_start, p, 64), p_count = __shfl(my_count, p, 64);
                float p_T = __shfl(Tr, p, 64);
                float part[C];
#pragma unroll
                for (int c = 0; c < C; ++c) part[c] = 0.0f;
                float dpart = 0.0f;
                for (uint32_t base = 0; base < p_count && !(p_T < kTransmittanceThreshold); base += 64u) {
                    const bool here = base + lane < p_count;
                    const uint32_t pos = p_start + base + lane;
                    float2 e = make_float2(0.0f, 0.0f);
                    if (here) e = qs.fragment[pos];
                    const float a = e.x;
                    const float t_after = wave_sequential_product(1.0f - a, p_T, min(64u, p_count - base));
                    const float t_before = wave_previous(t_after, p_T);
                    const bool reached = here && !(t_before < kTransmittanceThreshold);
                    const float bw = reached ? t_before * a : 0.0f;
                    if (here) qs.fragment[pos].x = bw;
                    if (reached) {
                        const uint32_t jj = __float_as_uint(e.y);
#pragma unroll
                        for (int q4 = 0; q4 < C / 4; ++q4) {
                            const float4 v = st.feat[jj * (C / 4) + q4];
                            part[4 * q4] = fmaf(bw, v.x, part[4 * q4]);
                            part[4 * q4 + 1] = fmaf(bw, v.y, part[4 * q4 + 1]);
                            part[4 * q4 + 2] = fmaf(bw, v.z, part[4 * q4 + 2]);
                            part[4 * q4 + 3] = fmaf(bw, v.w, part[4 * q4 + 3]);
                        }
                        if (INFERENCE) dpart = fmaf(bw, st.depth[jj], dpart);
                    }
                    // transmittance behind the last fragment that was reached
                    const uint64_t reached_lanes = __ballot(reached);
                    const int last = 63 - __builtin_clzll(reached_lanes | 1ull);
                    p_T = __shfl(t_after, last, 64);
                    // a walk that ended inside this round leaves the rest of the list untouched: weights 0
                    if (p_T < kTransmittanceThreshold)
                        for (uint32_t rest = base + 64u + lane; rest < p_count; rest += 64u) qs.fragment[p_start + rest].x = 0.0f;
                }
#pragma unroll
                for (int c = 0; c < C; ++c) {
                    const float sum = wave_sum(part[c]);
                    if ((int)lane == p) F[c] += sum;
                }
                if (INFERENCE) {
                    const float sum = wave_sum(dpart);
                    if ((int)lane == p) D += sum;
                }
                if ((int)lane == p) {
                    Tr = p_T;
                    done = Tr < kTransmittanceThreshold;
                }
            }
            wave_sync();
            FWD_MARK(4);
            // ---- instances: hand the blending weights of the fragments to the thread that owns the instance
            if (!INFERENCE) {
#pragma unroll
                for (int q = 0; q < NF; ++q)
                    if (lf.pixel[q] != kNoPixel) st.result[wave][q][j] = qs.fragment[lf.where[q]];
            }
        }
        {
            const uint64_t finished = __ballot(done);
            if (lane == 0u) st.done[wave] = finished;
        }
        FWD_MARK(2);
        const bool all_done = __syncthreads_and(done) != 0;
        FWD_MARK(5);
#if defined(INPC_BLEND_PROFILE) && !defined(INPC_PROFILE_BACKWARD)
        ++prof_batches;
#endif
        // ---- the gather moves on in front of the stores of the write phase
        const uint32_t point = g.h.point;
        const bool multi = g.h.multi();
        advance_gather<T, C, HALF>(g, inst_slots, records, stride, begin, range.y);
        // ---- write: thread t owns staged instance t (kernels.cu:291-295)
        if (!INFERENCE && valid) {
            float w = 0.0f;
#pragma unroll
            for (int q = 0; q < NQ; ++q)
#pragma unroll
                for (int k = 0; k < NF; ++k) {
                    const float bw = st.result[q][k][tid].x;
                    if (bw > 0.0f) w = fmaf(bw, st.weight[q][k][tid], w);
                }
            if (w > 0.0f) {
                if (multi) atomicAdd(&blending_weights[point], w);
                else blending_weights[point] = w;
            }
        }
        if (all_done) break;
    }
#ifndef INPC_PROFILE_BACKWARD
    INPC_PROF_FLUSH;
#endif
#undef FWD_MARK
    if (inside) {
        const size_t n_pixels = (size_t)W * H, pix = (size_t)py * W + px;
#pragma unroll
        for (int c = 0; c < C; ++c) image[c * n_pixels + pix] = F[c];
        const float alpha_px = 1.0f - Tr;
        alpha_image[pix] = Tr < kTransmittanceThreshold ? 1.0f : alpha_px;
        if (INFERENCE) depth_image[pix] = alpha_px > 0.0f ? D / alpha_px : 0.0f;
    }
}

// ---- backward -----------------------------------------------------------------------------------------------------
// With s = features . grad of a fragment, R the running sum of weight x s of a pixel and S its final value
// image . grad, the opacity gradient of the reference (kernels.cu:405-413),
//   dot(T f + (F_running - F_final) / (1 - a), grad) + grad_alpha (1 - alpha_final) / (1 - a),
// is T s + (R - S + grad_alpha (1 - alpha_final)) / (1 - a): the pixel walk carries two scalars, not 2C.
template <int T, int C, bool HALF>
__global__ void __launch_bounds__(T* T)
    k_blend_backward(const uint2* __restrict__ ranges, const uint32_t* __restrict__ tile_order,
                     const uint32_t* __restrict__ inst_slots, const char* __restrict__ records, uint32_t stride,
                     const float* __restrict__ grad_image, const float* __restrict__ grad_alpha,
                     const float* __restrict__ image, const float* __restrict__ alpha_image, float* grad_view,
                     float* grad_opacities, int W, int H, uint32_t gw) {
    constexpr int TT = T * T;
    constexpr int NQ = TT / 64;
    constexpr int NF = Stage<T, C, false>::NF;
    __shared__ Stage<T, C, false> st;
    __shared__ QuadScratch<NF> s_quad[NQ];
    __shared__ float4 s_grad[NQ][64][C / 4];   // upstream gradient of every wave's pixels (0 outside the image)

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t tile = tile_order[blockIdx.x];
    const int tile_x0 = (int)(tile % gw) * T, tile_y0 = (int)(tile / gw) * T;
    const int px = tile_x0 + (T == 16 ? 2 * (int)(lane & 7u) + (int)(wave & 1u) : (int)(lane & 7u));
    const int py = tile_y0 + (T == 16 ? 2 * (int)(lane >> 3) + (int)(wave >> 1) : (int)(lane >> 3));
    const bool inside = px < W && py < H;
    QuadScratch<NF>& qs = s_quad[wave];

    float final_dot = 0.0f, common = 0.0f;
    {
        // all loads of the pixel in one go (a pixel outside the image reads pixel 0 and drops it)
        const size_t n_pixels = (size_t)W * H, pix = inside ? (size_t)py * W + px : 0;
        float g[C], v[C];
#pragma unroll
        for (int c = 0; c < C; ++c) {
            g[c] = grad_image[c * n_pixels + pix];
            v[c] = image[c * n_pixels + pix];
        }
        const float ga = grad_alpha[pix], av = alpha_image[pix];
#pragma unroll
        for (int c = 0; c < C; ++c) {
            if (!inside) g[c] = 0.0f;
            if (inside) final_dot = fmaf(v[c], g[c], final_dot);
        }
#pragma unroll
        for (int q4 = 0; q4 < C / 4; ++q4) s_grad[wave][lane][q4] = make_float4(g[4 * q4], g[4 * q4 + 1], g[4 * q4 + 2], g[4 * q4 + 3]);
        if (inside) common = ga * (1.0f - av);
    }
    const float offset = common - final_dot;
    float Tr = 1.0f, running = 0.0f;
    bool done = !inside;
    {
        const uint64_t finished = __ballot(done);
        if (lane == 0u) st.done[wave] = finished;
    }
    __syncthreads();

    const uint2 range = ranges[tile];
#ifdef INPC_PROFILE_BACKWARD
    INPC_PROF_DECL;
#define BWD_MARK(i) INPC_PROF_MARK(i)
#else
#define BWD_MARK(i)
#endif
    Gather<C> g;
    start_gather<T, C, HALF>(g, inst_slots, records, stride, range);
    for (uint32_t begin = range.x; begin < range.y; begin += TT) {
        const uint32_t count = min((uint32_t)TT, range.y - begin);
        const bool valid = tid < count;
        stage_instance<T, C, false>(st, valid, g.h, g.f, tile_x0, tile_y0);
        BWD_MARK(0);
        __syncthreads();
        BWD_MARK(1);

        // ---- consume: this wave's list
        const ListIndex<NQ> li = list_index<T, C, false>(st, wave);
        const uint32_t total = li.end[NQ - 1];
        for (uint32_t sub = 0; sub < total; sub += 64u) {
            const bool live = sub + lane < total;
            const uint32_t j = live ? list_entry<T, C, false>(st, li, wave, sub + lane) : 0u;
            LaneFragments<NF> lf;
            load_lane_fragments<T, C, false>(st, wave, live, j, __ballot(done), lf);
            float feat[C];
#pragma unroll
            for (int q4 = 0; q4 < C / 4; ++q4) {
                const float4 v = st.feat[j * (C / 4) + q4];
                feat[4 * q4] = v.x;
                feat[4 * q4 + 1] = v.y;
                feat[4 * q4 + 2] = v.z;
                feat[4 * q4 + 3] = v.w;
            }
            uint32_t my_start, my_count, n_fragments;
            build_fragment_lists<NF>(qs, st.opacity[j], lf, my_start, my_count, n_fragments, [&](int q) {
                float d = 0.0f;  // features . grad of the fragment's pixel
#pragma unroll
                for (int q4 = 0; q4 < C / 4; ++q4) {
                    const float4 gr = s_grad[wave][lf.pixel[q]][q4];
                    d = fmaf(feat[4 * q4], gr.x, d);
                    d = fmaf(feat[4 * q4 + 1], gr.y, d);
                    d = fmaf(feat[4 * q4 + 2], gr.z, d);
                    d = fmaf(feat[4 * q4 + 3], gr.w, d);
                }
                return d;
            });
            BWD_MARK(2);
            if (n_fragments == 0u) continue;
            // ---- pixels with short lists: the sequential walk (kernels.cu:383-417)
            if (my_count <= kLongList) {
                for (uint32_t i = 0; i < my_count; ++i) {
                    const uint32_t pos = my_start + i;
                    const float2 e = qs.fragment[pos];
                    const float a = done ? 0.0f : e.x, sd = e.y;
                    const float bw = Tr * a;
                    const float one_minus_a = 1.0f - a;
                    const float rcp = __frcp_rn(fmaxf(one_minus_a, kOneMinusAlphaEps));
                    running = fmaf(bw, sd, running);
                    const float dalpha = done ? 0.0f : fmaf(Tr, sd, (running + offset) * rcp);
                    qs.fragment[pos] = make_float2(bw, dalpha);
                    Tr *= one_minus_a;
                    done = done || Tr < kTransmittanceThreshold;
                }
            }
            BWD_MARK(3);
            // ---- pixels with long lists, one after the other, 64 fragments at a time over the wave
            uint64_t long_pixels = __ballot(my_count > kLongList);
            while (long_pixels) {
                const int p = __builtin_ctzll(long_pixels);
                long_pixels &= long_pixels - 1ull;
                const uint32_t p_start = __shfl(my_start, p, 64), p_count = __shfl(my_count, p, 64);
                float p_T = __shfl(Tr, p, 64), p_R = __shfl(running, p, 64);
                const float p_offset = __shfl(offset, p, 64);
                for (uint32_t base = 0; base < p_count && !(p_T < kTransmittanceThreshold); base += 64u) {
                    const bool here = base + lane < p_count;
                    const uint32_t pos = p_start + base + lane;
                    float2 e = make_float2(0.0f, 0.0f);
                    if (here) e = qs.fragment[pos];
                    const float a = e.x, sd = e.y;
                    const float t_after = wave_sequential_product(1.0f - a, p_T, min(64u, p_count - base));
                    const float t_before = wave_previous(t_after, p_T);
                    const bool reached = here && !(t_before < kTransmittanceThreshold);
                    const float bw = reached ? t_before * a : 0.0f;
                    const float run = p_R + wave_inclusive_sum(bw * sd);
                    const float rcp = __frcp_rn(fmaxf(1.0f - a, kOneMinusAlphaEps));
                    const float dalpha = reached ? fmaf(t_before, sd, (run + p_offset) * rcp) : 0.0f;
                    if (here) qs.fragment[pos] = make_float2(bw, dalpha);
                    const uint64_t reached_lanes = __ballot(reached);
                    const int last = 63 - __builtin_clzll(reached_lanes | 1ull);
                    p_T = __shfl(t_after, last, 64);
                    p_R = __shfl(run, last, 64);
                    if (p_T < kTransmittanceThreshold)
                        for (uint32_t rest = base + 64u + lane; rest < p_count; rest += 64u)
                            qs.fragment[p_start + rest] = make_float2(0.0f, 0.0f);
                }
                if ((int)lane == p) {
                    Tr = p_T;
                    running = p_R;
                    done = Tr < kTransmittanceThreshold;
                }
            }
            wave_sync();
            BWD_MARK(4);
            // ---- instances: hand {blending weight, d loss / d alpha} of the fragments to the instance's thread
#pragma unroll
            for (int q = 0; q < NF; ++q)
                if (lf.pixel[q] != kNoPixel) st.result[wave][q][j] = qs.fragment[lf.where[q]];
        }
        {
            const uint64_t finished = __ballot(done);
            if (lane == 0u) st.done[wave] = finished;
        }
        BWD_MARK(2);
        const bool all_done = __syncthreads_and(done) != 0;
        BWD_MARK(5);
#if defined(INPC_PROFILE_BACKWARD) && defined(INPC_BLEND_PROFILE)
        ++prof_batches;
#endif
        // ---- the gather moves on before the stores of the write phase (see the forward kernel)
        const uint32_t point = g.h.point;
        const bool multi = g.h.multi();
        advance_gather<T, C, HALF>(g, inst_slots, records, stride, begin, range.y);
        // ---- write: thread t owns staged instance t: gradient of the point from its fragments in all quads
        if (valid) {
            float gf[C];
#pragma unroll
            for (int c = 0; c < C; ++c) gf[c] = 0.0f;
            float gop = 0.0f;
            bool any_weight = false;
#pragma unroll
            for (int q = 0; q < NQ; ++q)
#pragma unroll
                for (int k = 0; k < NF; ++k) {
                    const float2 e = st.result[q][k][tid];
                    gop = fmaf(e.y, st.weight[q][k][tid], gop);
                    if (e.x > 0.0f) {
                        any_weight = true;
                        const uint32_t pix = st.pixel[q][k][tid];
#pragma unroll
                        for (int q4 = 0; q4 < C / 4; ++q4) {
                            const float4 gr = s_grad[q][pix][q4];
                            gf[4 * q4] = fmaf(e.x, gr.x, gf[4 * q4]);
                            gf[4 * q4 + 1] = fmaf(e.x, gr.y, gf[4 * q4 + 1]);
                            gf[4 * q4 + 2] = fmaf(e.x, gr.z, gf[4 * q4 + 2]);
                            gf[4 * q4 + 3] = fmaf(e.x, gr.w, gf[4 * q4 + 3]);
                        }
                    }
                }
            if (any_weight || gop != 0.0f) {
                float* dst = grad_view + (size_t)point * C;
                if (multi) {
#pragma unroll
                    for (int c = 0; c < C; ++c)
                        if (gf[c] != 0.0f) atomicAdd(dst + c, gf[c]);
                    if (gop != 0.0f) atomicAdd(&grad_opacities[point], gop);
                } else {
#pragma unroll
                    for (int q4 = 0; q4 < C / 4; ++q4)
                        ((float4*)dst)[q4] = make_float4(gf[4 * q4], gf[4 * q4 + 1], gf[4 * q4 + 2], gf[4 * q4 + 3]);
                    grad_opacities[point] = gop;
                }
            }
        }
        if (all_done) break;
    }
#ifdef INPC_PROFILE_BACKWARD
    INPC_PROF_FLUSH;
#endif
#undef BWD_MARK
}

}  // namespace blend
