// blend.hpp — front-to-back alpha blending of the sorted instance lists, forward and backward
// (B/rasterization/src/bilinear/kernels.cu:241-495). Included by raster.hip after the record helpers.
//
// One block per tile, one thread per pixel. A wave owns 64 pixels on an 8 x 8 grid: the whole tile for 8x8
// tiles; for 16x16 tiles the pixels of one parity class (x odd / even, y odd / even), so that the 2 x 2
// footprint of a point gives every wave exactly one fragment and a cluster of points on one spot loads the
// four waves evenly. Per batch of T*T instances:
//   stage    thread t puts the record of instance t into LDS: screen position, opacity, features;
//   consume  every wave goes over the whole batch (up to four instances per lane) and derives, for each
//            instance, the one fragment that falls into its parity class (8x8 tiles: all four fragments), with
//            wave-level synchronisation only: hit masks per pixel -> per-pixel fragment lists in depth order -> the
//            sequential transmittance chain per pixel (short lists) or a wave-wide product scan (long
//            lists); the results stay in the fragment list;
//   write    thread t collects the results of instance t's fragments: a plain store when the point lies in
//            one tile only, rows of its own when it straddles tiles (forward: atomics).
// Two block barriers per batch. The forward pass gathers the records by point index, two batches ahead of the blend,
// and (configurations with a backward pass) writes each record once more where its instance stands in the tile's
// list; the backward pass reads those ordered records in contiguous runs, one batch ahead.
// A record carries the footprint of its point as preprocess computed it: the left / top candidate pixel and the
// interpolation weights of the two candidate columns and rows, so a wave finds the fragment of an instance with a
// few integer operations.
#pragma once

namespace blend {

constexpr int kQuad = 8;             // a wave's pixel quad is 8 x 8
constexpr uint32_t kLongList = 32;   // lists longer than this are evaluated by the whole wave

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
// (a product taken in tree order may land on the other side of the threshold). Every step, every lane takes its left neighbour's value (lane 0: t_in) times
// its own factor: after step s the lanes 0..s hold their final value, and computing a final value again from a
// final neighbour reproduces it. One multiply per step, no LDS. (Steps beyond n only recompute final values, so
// the loop runs in unrolled groups of eight.)
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

// Shape of the work per tile size.
//   NQ  waves ("quads") per tile
//   NF  fragments one instance can have inside one wave's pixel grid: 4 (8x8 tiles: the whole 2 x 2 footprint),
//       1 (16x16 tiles: one pixel per parity class)
//   K   list entries a lane takes per batch: a quad's list has up to T*T = 64 K entries
// Either way an instance has four fragment slots in the tile (slot = quad for 16x16 tiles, = candidate pixel
// ky * 2 + kx for 8x8 tiles) and a wave handles up to 256 fragments per batch.
template <int T>
struct Shape {
    static constexpr int TT = T * T;
    static constexpr int NQ = TT / 64;
    static constexpr int NF = T == 16 ? 1 : 4;
    static constexpr int K = T == 16 ? 4 : 1;
};

// Per-block staging area of one batch.
template <int T, int C, bool WITH_DEPTH>
struct Stage {
    static constexpr int TT = T * T;
    static constexpr int NQ = TT / 64;
    float4 feat[TT * (C / 4)];
    float depth[WITH_DEPTH ? TT : 1];
    float4 alpha[T == 16 ? TT : 1];     // per fragment slot of the staged instance: opacity * interpolation weight
    uint32_t pixel[T == 16 ? TT : 1];   // per slot, one byte: pixel in the owning wave's grid, kNoPixel: no fragment
    alignas(8) uint16_t frag[TT][4];    // per slot: the fragment field, written by the wave that placed the fragment
};

// Per-wave scratch of the consume phase. A fragment entry is {alpha, x} on the way in and {blending weight, y}
// on the way out; forward: x = staged instance; backward: x = features . grad, y = d loss / d alpha.
template <int T>
struct QuadScratch {
    uint64_t hits[Shape<T>::K][64];  // per entry round and pixel: lanes whose entry hits the pixel (round-major:
                                     // the lanes of an access are a round's, their pixels spread over the banks)
    float2 fragment[256];            // per fragment, pixel by pixel, in depth order
};

// Block barrier that also tells whether `done` holds for every thread of the block. The waves leave their verdicts
// in the first hit mask of their scratch, which is idle between the list building of one batch and that of the next
// (the block barrier in front of the next list building separates the reads here from its clearing). The library's
// __syncthreads_and keeps LDS of its own, which kept the fourth block of the 16-channel inference kernel off a CU.
template <int T>
__device__ __forceinline__ bool barrier_all_done(QuadScratch<T>* s_quad, bool done) {
    constexpr int NQ = Shape<T>::NQ;
    const bool wave_done = __ballot(done) == ~0ull;   // every wave of the block is full
    if (__lane_id() == 0u) s_quad[threadIdx.x >> 6].hits[0][0] = wave_done ? 1ull : 0ull;
    __syncthreads();
    bool all = true;
#pragma unroll
    for (int q = 0; q < NQ; ++q) all = all && s_quad[q].hits[0][0] != 0ull;
    return all;
}

// Makes the value available here: the wait for an outstanding load that produces it lands at this point and not
// at a later first use.
#if defined(__AMDGCN__)
__device__ __forceinline__ void arrive(float& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void arrive(uint32_t& v) { asm volatile("" : "+v"(v)); }
#else   // only the device has loads in flight to wait for
__device__ __forceinline__ void arrive(float&) {}
__device__ __forceinline__ void arrive(uint32_t&) {}
#endif

__device__ __forceinline__ void arrive(Header& h) {
    arrive(h.wx0);
    arrive(h.wx1);
    arrive(h.wy0);
    arrive(h.wy1);
    arrive(h.opacity);
    arrive(h.tag);
    arrive(h.cell);
    arrive(h.extra);
}

__device__ __forceinline__ Header read_header(const char* __restrict__ record) {
    return make_header(((const float4*)record)[0], ((const float4*)record)[1]);
}

// Stage instance `t` (thread t): features, and per fragment slot the blend's alpha and the pixel, so that the waves
// only look their fragments up. `weight` receives the slots' interpolation weights (for the write phase of the same
// thread). `valid` is false for the threads behind the end of the batch. Must be followed by a block barrier.
template <int T, int C, bool WITH_DEPTH>
__device__ __forceinline__ void stage_instance(Stage<T, C, WITH_DEPTH>& st, bool valid, const Header& h,
                                               const float (&f)[C], int tile_x0, int tile_y0, float (&weight)[4],
                                               uint32_t (&pixel)[4]) {
    const uint32_t t = threadIdx.x;
    fragment_slots<T>(h, tile_x0, tile_y0, weight, pixel);
    if (!valid) return;
#pragma unroll
    for (int q4 = 0; q4 < C / 4; ++q4) st.feat[t * (C / 4) + q4] = make_float4(f[4 * q4], f[4 * q4 + 1], f[4 * q4 + 2], f[4 * q4 + 3]);
    if (WITH_DEPTH) st.depth[t] = __uint_as_float(h.extra);
    if (T == 16) {   // 8x8 tiles: the staging thread's wave is the only consumer and takes them from its registers
        st.alpha[t] = make_float4(h.opacity * weight[0], h.opacity * weight[1], h.opacity * weight[2], h.opacity * weight[3]);
        st.pixel[t] = pixel[0] | (pixel[1] << 8) | (pixel[2] << 16) | (pixel[3] << 24);
    }
    if (!WITH_DEPTH) {   // the write phase that reads the fields only exists in training configurations
        const uint2 nothing_placed = make_uint2(0u, 0u);
        __builtin_memcpy(st.frag[t], &nothing_placed, 8);
    }
}

// The instances of one lane: entry k is staged instance k * 64 + lane; its (at most NF) fragments in this
// wave's grid. Depth order is the order of (k, lane).
template <int T>
struct Entries {
    static constexpr int K = Shape<T>::K, NF = Shape<T>::NF;
    uint32_t j[K];           // staged instance
    uint32_t pixel[K][NF];   // kNoPixel: no fragment in this wave's grid, or the pixel is finished
    float alpha[K][NF];
};

// `count`: staged instances of the batch; `finished`: this wave's pixels that are done. 16x16 tiles: the wave looks
// up slot `quad` of all staged instances; 8x8 tiles: lane l staged instance l itself and passes its slots
// (`opacity`, `weight`, `pixel`).
template <int T, int C, bool WITH_DEPTH>
__device__ __forceinline__ void load_entries(const Stage<T, C, WITH_DEPTH>& st, uint32_t count, uint32_t quad,
                                             uint64_t finished, float opacity, const float (&weight)[4],
                                             const uint32_t (&pixel)[4], Entries<T>& e) {
    constexpr int K = Shape<T>::K, NF = Shape<T>::NF;
    const uint32_t lane = __lane_id();
    if (T == 16) {
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const uint32_t j = k * 64u + lane;
            const bool live = j < count;
            e.j[k] = j;
            const uint32_t at = live ? j : 0u;
            const uint32_t pix = ((const uint8_t*)&st.pixel[at])[quad];
            const bool open = live && pix != kNoPixel && ((finished >> (pix & kPixelMask)) & 1ull) == 0ull;
            e.pixel[k][0] = open ? pix : kNoPixel;
            e.alpha[k][0] = ((const float*)&st.alpha[at])[quad];
        }
    } else {
        const bool live = lane < count;
        e.j[0] = lane;
#pragma unroll
        for (int q = 0; q < NF; ++q) {
            const bool open = live && pixel[q] != kNoPixel && ((finished >> (pixel[q] & kPixelMask)) & 1ull) == 0ull;
            e.pixel[0][q] = open ? pixel[q] : kNoPixel;
            e.alpha[0][q] = opacity * weight[q];
        }
    }
}

// Per-pixel fragment lists of one batch. In: the lane's entries and payload(k, q), the second word of a
// fragment's entry. Out: every pixel lane's list [my_start, my_start + my_count) of {alpha, payload} in depth
// order in qs.fragment, and in the stage, for every fragment placed, where it is. Every lane of the wave
// must call it.
template <int T, int C, bool WITH_DEPTH, typename Payload>
__device__ __forceinline__ void build_fragment_lists(QuadScratch<T>& qs, Stage<T, C, WITH_DEPTH>& st, uint32_t quad,
                                                     const Entries<T>& e, uint32_t& my_start, uint32_t& my_count,
                                                     uint32_t& n_fragments, Payload payload) {
    constexpr int K = Shape<T>::K, NF = Shape<T>::NF;
    const uint32_t lane = __lane_id();
#pragma unroll
    for (int k = 0; k < K; ++k) qs.hits[k][lane] = 0ull;
    wave_sync();
    const unsigned long long bit = 1ull << lane;
#pragma unroll
    for (int k = 0; k < K; ++k)
#pragma unroll
        for (int q = 0; q < NF; ++q)
            if (e.pixel[k][q] != kNoPixel) atomicOr((unsigned long long*)&qs.hits[k][e.pixel[k][q]], bit);
    wave_sync();
    // where the fragments of entry round k start in this lane's pixel's list: behind those of the rounds before
    uint32_t round_start[K];
    my_count = 0u;
#pragma unroll
    for (int k = 0; k < K; ++k) {
        round_start[k] = my_count;
        my_count += (uint32_t)__popcll(qs.hits[k][lane]);
    }
    my_start = wave_exclusive_sum(my_count, n_fragments);
    if (n_fragments == 0u) return;
    const uint64_t below = lanes_below();
#pragma unroll
    for (int k = 0; k < K; ++k) {
        round_start[k] += my_start;
#pragma unroll
        for (int q = 0; q < NF; ++q) {
            const bool hit = e.pixel[k][q] != kNoPixel;
            const uint32_t pix = hit ? e.pixel[k][q] : 0u;
            const uint32_t start = __shfl(round_start[k], pix, 64);  // every lane takes part in the exchange
            if (hit) {
                const uint32_t pos = start + (uint32_t)__popcll(qs.hits[k][pix] & below);
                qs.fragment[pos] = make_float2(e.alpha[k][q], payload(k, q));
                if (!WITH_DEPTH) st.frag[e.j[k]][T == 16 ? quad : q] = (uint16_t)((pos << 8) | pix | kPlaced);
            }
        }
    }
    wave_sync();
}

// Fragment fields of staged instance t, one per slot.
template <int T, int C, bool WITH_DEPTH>
__device__ __forceinline__ void load_fields(const Stage<T, C, WITH_DEPTH>& st, uint32_t t, uint32_t (&field)[4]) {
    uint2 fields;
    __builtin_memcpy(&fields, st.frag[t], 8);
    field[0] = fields.x & 0xFFFFu;
    field[1] = fields.x >> 16;
    field[2] = fields.y & 0xFFFFu;
    field[3] = fields.y >> 16;
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
__device__ __forceinline__ void start_gather(Gather<C>& g, const uint32_t* __restrict__ inst_points,
                                             const char* __restrict__ records, uint32_t stride, uint2 range) {
    constexpr uint32_t TT = T * T;
    const uint32_t at = range.x + threadIdx.x;
    g.h = Header{};
    g.h_next = Header{};
#pragma unroll
    for (int c = 0; c < C; ++c) g.f[c] = g.f_next[c] = 0.0f;
    g.next_slot = 0u;
    uint32_t slot0 = 0u, slot1 = 0u;
    if (at < range.y) slot0 = inst_points[at];
    if (at + TT < range.y) slot1 = inst_points[at + TT];
    if (at + 2u * TT < range.y) g.next_slot = inst_points[at + 2u * TT];

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
__device__ __forceinline__ void advance_gather(Gather<C>& g, const uint32_t* __restrict__ inst_points,
                                               const char* __restrict__ records, uint32_t stride, uint32_t begin,
                                               uint32_t end) {
    constexpr uint32_t TT = T * T;
    const uint32_t at = begin + threadIdx.x;
    arrive(g.h_next);
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
    if (at + 3u * TT < end) g.next_slot = inst_points[at + 3u * TT];
}

// ---- ordered records: what the forward blend leaves for the backward blend ------------------------------------------
// One record per staged instance (2 + C / 4 words of 16 bytes), where the instance stands in its tile's list, with a
// header that is the instance's, not the point's: what the forward blend has worked out of the point's record for
// this tile, so that the backward blend stages an instance with a handful of instructions.
//   float weight[4]   interpolation weights of the four fragment slots
//   float opacity
//   u32   tag         as in the point's record (point index | kRecordMulti | span bits)
//   u32   pixels      per slot one byte: pixel in the owning wave's grid, kNoPixel: no fragment
//   u32   row         gradient row of this instance (points that touch several tiles)
// Within a batch the words are stored one after the other, word w of all the batch's instances in a row, so that a wave
// writes and reads 1 KB runs (a thread that writes its own 64-byte record costs the forward blend 0.11 ms, more than
// the backward blend gains). The batch that starts at instance `begin` and holds `count` instances occupies words
// [begin * kWords, (begin + count) * kWords).
struct InstanceHeader {
    float weight[4];
    float opacity;
    uint32_t tag, pixels, row;
    __device__ __forceinline__ bool multi() const { return (tag & kRecordMulti) != 0u; }
    __device__ __forceinline__ uint32_t point() const { return tag & kRecordIdMask; }
};

__device__ __forceinline__ void arrive(InstanceHeader& h) {
#pragma unroll
    for (int c = 0; c < 4; ++c) arrive(h.weight[c]);
    arrive(h.opacity);
    arrive(h.tag);
    arrive(h.pixels);
    arrive(h.row);
}

template <int C>
struct Ordered {
    static constexpr uint32_t kWords = 2u + (uint32_t)C / 4u;
    __device__ static __forceinline__ size_t word(uint32_t begin, uint32_t count, uint32_t w) {
        return (size_t)begin * kWords + (size_t)w * count + threadIdx.x;
    }
    __device__ static __forceinline__ void store(float4* __restrict__ ordered, uint32_t begin, uint32_t count,
                                                 const float (&weight)[4], float opacity, uint32_t tag, uint32_t pixels,
                                                 uint32_t row, const float (&f)[C]) {
        ordered[word(begin, count, 0)] = make_float4(weight[0], weight[1], weight[2], weight[3]);
        ordered[word(begin, count, 1)] = make_float4(opacity, __uint_as_float(tag), __uint_as_float(pixels),
                                                     __uint_as_float(row));
#pragma unroll
        for (int q = 0; q < C / 4; ++q)
            ordered[word(begin, count, 2 + q)] = make_float4(f[4 * q], f[4 * q + 1], f[4 * q + 2], f[4 * q + 3]);
    }
    // this thread's instance of the batch that starts at `begin`, if the batch has one for it
    __device__ static __forceinline__ void load(const float4* __restrict__ ordered, uint32_t begin, uint32_t end,
                                                InstanceHeader& h, float (&f)[C]) {
        if (begin >= end) return;
        const uint32_t count = min((uint32_t)blockDim.x, end - begin);
        if (threadIdx.x >= count) return;
        const float4 h0 = ordered[word(begin, count, 0)], h1 = ordered[word(begin, count, 1)];
        h.weight[0] = h0.x;
        h.weight[1] = h0.y;
        h.weight[2] = h0.z;
        h.weight[3] = h0.w;
        h.opacity = h1.x;
        h.tag = __float_as_uint(h1.y);
        h.pixels = __float_as_uint(h1.z);
        h.row = __float_as_uint(h1.w);
#pragma unroll
        for (int q = 0; q < C / 4; ++q) {
            const float4 v = ordered[word(begin, count, 2 + q)];
            f[4 * q] = v.x;
            f[4 * q + 1] = v.y;
            f[4 * q + 2] = v.z;
            f[4 * q + 3] = v.w;
        }
    }
};

// The ordered record of the batch being staged and the one of the batch after it (requested a batch earlier).
template <int C>
struct OrderedAhead {
    InstanceHeader h, h_next;
    float f[C], f_next[C];
};

template <int T, int C>
__device__ __forceinline__ void start_ordered(OrderedAhead<C>& g, const float4* __restrict__ ordered, uint2 range) {
    g.h = InstanceHeader{};
    g.h_next = InstanceHeader{};
    g.h.pixels = g.h_next.pixels = 0xFFFFFFFFu;   // no fragment in any slot
#pragma unroll
    for (int c = 0; c < C; ++c) g.f[c] = g.f_next[c] = 0.0f;
    Ordered<C>::load(ordered, range.x, range.y, g.h, g.f);
    Ordered<C>::load(ordered, range.x + T * T, range.y, g.h_next, g.f_next);
}

// At the end of the batch that starts at `begin`: takes the next batch's record, requests the one after it.
template <int T, int C>
__device__ __forceinline__ void advance_ordered(OrderedAhead<C>& g, const float4* __restrict__ ordered, uint32_t begin,
                                                uint32_t end) {
    arrive(g.h_next);
#pragma unroll
    for (int c = 0; c < C; ++c) arrive(g.f_next[c]);
    g.h = g.h_next;
#pragma unroll
    for (int c = 0; c < C; ++c) g.f[c] = g.f_next[c];
    Ordered<C>::load(ordered, begin + 2u * T * T, end, g.h_next, g.f_next);
}

// Stage instance `t` (thread t) of the backward blend from its ordered record; see stage_instance.
template <int T, int C>
__device__ __forceinline__ void stage_ordered(Stage<T, C, false>& st, bool valid, const InstanceHeader& h,
                                              const float (&f)[C], float (&weight)[4], uint32_t (&pixel)[4]) {
    const uint32_t t = threadIdx.x;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        weight[c] = h.weight[c];
        pixel[c] = (h.pixels >> (8 * c)) & 0xFFu;
    }
    if (!valid) return;
#pragma unroll
    for (int q4 = 0; q4 < C / 4; ++q4) st.feat[t * (C / 4) + q4] = make_float4(f[4 * q4], f[4 * q4 + 1], f[4 * q4 + 2], f[4 * q4 + 3]);
    if (T == 16) {
        st.alpha[t] = make_float4(h.opacity * weight[0], h.opacity * weight[1], h.opacity * weight[2], h.opacity * weight[3]);
        st.pixel[t] = h.pixels;
    }
    const uint2 nothing_placed = make_uint2(0u, 0u);
    __builtin_memcpy(st.frag[t], &nothing_placed, 8);
}

// ---- forward ------------------------------------------------------------------------------------------------------
template <int T, int C, bool HALF, bool INFERENCE>
__global__ void __launch_bounds__(T* T)
    k_blend_forward(const uint2* __restrict__ ranges, const uint32_t* __restrict__ tile_order,
                    const uint32_t* __restrict__ inst_points,
                    const char* __restrict__ records, uint32_t stride, float* __restrict__ image,
                    float* __restrict__ alpha_image, float* blending_weights, float* __restrict__ depth_image,
                    float4* __restrict__ ordered_records, uint32_t* __restrict__ tile_end, int W, int H, uint32_t gw) {
    constexpr int TT = T * T;
    constexpr int NQ = TT / 64;
    __shared__ Stage<T, C, INFERENCE> st;
    __shared__ QuadScratch<T> s_quad[NQ];

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t tile = tile_order[blockIdx.x];
    const int tile_x0 = (int)(tile % gw) * T, tile_y0 = (int)(tile / gw) * T;
    const int px = tile_x0 + (T == 16 ? 2 * (int)(lane & 7u) + (int)(wave & 1u) : (int)(lane & 7u));
    const int py = tile_y0 + (T == 16 ? 2 * (int)(lane >> 3) + (int)(wave >> 1) : (int)(lane >> 3));
    const bool inside = px < W && py < H;
    QuadScratch<T>& qs = s_quad[wave];

    float F[C];
#pragma unroll
    for (int c = 0; c < C; ++c) F[c] = 0.0f;
    float D = 0.0f, Tr = 1.0f;
    bool done = !inside;

    const uint2 range = ranges[tile];
    Gather<C> g;
    start_gather<T, C, HALF>(g, inst_points, records, stride, range);
    uint32_t staged_end = range.x;   // the tile's instances in front of this one have been staged
    for (uint32_t begin = range.x; begin < range.y; begin += TT) {
        const uint32_t count = min((uint32_t)TT, range.y - begin);
        const bool valid = tid < count;
        staged_end = begin + count;
        float weight[4];   // of this thread's staged instance, per fragment slot
        uint32_t slot_pixel[4];
        stage_instance<T, C, INFERENCE>(st, valid, g.h, g.f, tile_x0, tile_y0, weight, slot_pixel);
        __syncthreads();

        // ---- consume: this wave's list
        uint32_t my_start = 0, my_count = 0, n_fragments = 0;
        {
            Entries<T> e;
            load_entries<T, C, INFERENCE>(st, count, wave, __ballot(done), g.h.opacity, weight, slot_pixel, e);
            build_fragment_lists<T, C, INFERENCE>(qs, st, wave, e, my_start, my_count, n_fragments,
                                                  [&](int k, int) { return __uint_as_float(e.j[k]); });
        }
        if (n_fragments != 0u) {
            // ---- pixels with short lists: the reference's sequential walk (kernels.cu:281-299)
            if (my_count <= kLongList) {
                for (uint32_t i = 0; i < my_count; ++i) {
                    const uint32_t pos = my_start + i;
                    const float2 e = qs.fragment[pos];
                    const float a = done ? 0.0f : e.x;
                    const uint32_t jj = __float_as_uint(e.y);
                    const float bw = Tr * a;
                    if (!INFERENCE) qs.fragment[pos].x = bw;
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
                    if (!INFERENCE && here) qs.fragment[pos].x = bw;
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
                    if (!INFERENCE && p_T < kTransmittanceThreshold)
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
        }
        const bool all_done = barrier_all_done<T>(s_quad, done);
        // ---- the gather moves on in front of the stores of the write phase
        const Header mine = g.h;
        // the backward pass reads the records of this batch in runs (a gather pulls a 128-byte line per
        // 64-byte record and was 0.13 ms of the backward blend)
        if (!INFERENCE && ordered_records && valid) {
            uint32_t row = 0u;
            if (g.h.multi()) {
                const int lx = local_left(g.h.cell & 0xFFFFu, tile_x0), ly = local_left(g.h.cell >> 16, tile_y0);
                row = instance_row(g.h.extra, g.h.tag, lx, ly, tile_x0, tile_y0);
            }
            const uint32_t pixels = slot_pixel[0] | (slot_pixel[1] << 8) | (slot_pixel[2] << 16) | (slot_pixel[3] << 24);
            Ordered<C>::store(ordered_records, begin, count, weight, g.h.opacity, g.h.tag, pixels, row, g.f);
        }
        advance_gather<T, C, HALF>(g, inst_points, records, stride, begin, range.y);
        // ---- write: thread t owns staged instance t (kernels.cu:291-295): its blending weight is the sum over
        // the fragments the waves placed
        if (!INFERENCE && valid) {
            uint32_t field[4];
            load_fields<T, C, INFERENCE>(st, tid, field);
            float w = 0.0f;
#pragma unroll
            for (int c = 0; c < 4; ++c)
                if (field[c] & kPlaced) {
                    const float bw = s_quad[T == 16 ? c : 0].fragment[field[c] >> 8].x;
                    if (bw > 0.0f) w = fmaf(bw, weight[c], w);
                }
            if (w > 0.0f) {
                if (mine.multi()) atomicAdd(&blending_weights[mine.point()], w);
                else blending_weights[mine.point()] = w;
            }
        }
        if (all_done) break;
    }
    // how far the ordered records of the tile reach: the backward pass goes no further
    if (!INFERENCE && tile_end && tid == 0) tile_end[tile] = staged_end;
    if (inside) {
        const size_t n_pixels = (size_t)W * H, pix = (size_t)py * W + px;
#pragma unroll
        for (int c = 0; c < C; ++c) image[c * n_pixels + pix] = F[c];
        const float alpha_px = 1.0f - Tr;
        alpha_image[pix] = Tr < kTransmittanceThreshold ? 1.0f : alpha_px;
        if (INFERENCE) depth_image[pix] = alpha_px > 0.0f ? D / alpha_px : 0.0f;
    }
}

// ---- gradients of points that straddle tiles --------------------------------------------------------------------
// A point that touches several tiles has a list entry {point | touched tiles << 28, first row} and one gradient row
// per touched tile, in the row-major order of its tiles: features[row][C], opacities[row], and a flag byte per
// row: the row has been written. The flags are zero after the forward pass and after k_grad_reduce.
struct SplitRows {
    float* features;
    float* opacities;
    uint8_t* flags;
    const uint2* list;
    const uint32_t* count;    // number of list entries
};

// gradient of the point = sum of its rows that were written, in row order (the gradient buffers are zero before). A
// group of kGroup neighbouring lanes takes one point, lane j the j-th 16-byte word of each feature row (the last lane
// of the group also the opacity gradients), so that a wave reads the rows of neighbouring points in whole lines; one
// lane per point walked its rows 16 bytes at a time and fetched every line several times. All rows are read whether
// written or not (stale rows are dropped by their flag): the reads are dense and independent.
template <int C>
__global__ void __launch_bounds__(256) k_grad_reduce(SplitRows rows, float* __restrict__ grad_view,
                                                     float* __restrict__ grad_opacities) {
    constexpr uint32_t kGroup = C / 4;   // 1, 2 or 4 lanes per point
    const uint32_t n = *rows.count;
    const uint32_t gtid = blockIdx.x * 256u + threadIdx.x, word = gtid % kGroup;
    const uint32_t stride = gridDim.x * 256u / kGroup;
    for (uint32_t s = gtid / kGroup; s < n; s += stride) {   // the lanes of a group stay together
        const uint2 entry = rows.list[s];
        const uint32_t i = entry.x & kRecordIdMask, touched = entry.x >> 28, first = entry.y;
        const float4* row = (const float4*)(rows.features + (size_t)first * C) + word;
        float4 part[4];
        float part_opacity[4];
        bool written[4];
        bool any = false;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const bool exists = (uint32_t)p < touched;
            written[p] = exists && rows.flags[first + (exists ? p : 0)] != 0;
            any = any || written[p];
            part[p] = exists ? row[p * (C / 4)] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            part_opacity[p] = exists && word == kGroup - 1u ? rows.opacities[first + p] : 0.0f;
        }
        if (!any) continue;   // the same for all lanes of the group
        float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        float opacity = 0.0f;
#pragma unroll
        for (int p = 0; p < 4; ++p)
            if (written[p]) {
                acc.x += part[p].x;
                acc.y += part[p].y;
                acc.z += part[p].z;
                acc.w += part[p].w;
                opacity += part_opacity[p];
            }
        ((float4*)(grad_view + (size_t)i * C))[word] = acc;
        if (word == kGroup - 1u) grad_opacities[i] = opacity;
        // the flags go back to zero for the next pass, once the other lanes of the group have read them (same wave,
        // same control flow: their loads are complete behind this point)
        wave_sync();
        if (word == 0u) {
#pragma unroll
            for (int p = 0; p < 4; ++p)
                if (written[p]) rows.flags[first + p] = 0;
        }
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
                     const float4* __restrict__ ordered_records, const uint32_t* __restrict__ tile_end,
                     const float* __restrict__ grad_image, const float* __restrict__ grad_alpha,
                     const float* __restrict__ image, const float* __restrict__ alpha_image, float* grad_view,
                     float* grad_opacities, SplitRows rows, int W, int H, uint32_t gw) {
    constexpr int TT = T * T;
    constexpr int NQ = TT / 64;
    constexpr int K = Shape<T>::K, NF = Shape<T>::NF;
    __shared__ Stage<T, C, false> st;
    __shared__ QuadScratch<T> s_quad[NQ];
    __shared__ float4 s_grad[NQ][C / 4][64];   // upstream gradient of every wave's pixels (0 outside the image)

    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    const uint32_t tile = tile_order[blockIdx.x];
    const int tile_x0 = (int)(tile % gw) * T, tile_y0 = (int)(tile / gw) * T;
    const int px = tile_x0 + (T == 16 ? 2 * (int)(lane & 7u) + (int)(wave & 1u) : (int)(lane & 7u));
    const int py = tile_y0 + (T == 16 ? 2 * (int)(lane >> 3) + (int)(wave >> 1) : (int)(lane >> 3));
    const bool inside = px < W && py < H;
    QuadScratch<T>& qs = s_quad[wave];

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
        for (int q4 = 0; q4 < C / 4; ++q4) s_grad[wave][q4][lane] = make_float4(g[4 * q4], g[4 * q4 + 1], g[4 * q4 + 2], g[4 * q4 + 3]);
        if (inside) common = ga * (1.0f - av);
    }
    const float offset = common - final_dot;
    float Tr = 1.0f, running = 0.0f;
    bool done = !inside;

    // the records as the forward pass staged them, in the order of the tile's list; only as far as it got
    uint2 range = ranges[tile];
    range.y = min(range.y, tile_end[tile]);
    OrderedAhead<C> g;
    start_ordered<T, C>(g, ordered_records, range);
    for (uint32_t begin = range.x; begin < range.y; begin += TT) {
        const uint32_t count = min((uint32_t)TT, range.y - begin);
        const bool valid = tid < count;
        float weight[4];   // of this thread's staged instance, per fragment slot
        uint32_t slot_pixel[4];
        stage_ordered<T, C>(st, valid, g.h, g.f, weight, slot_pixel);
        __syncthreads();

        // ---- consume: this wave's list
        uint32_t my_start = 0, my_count = 0, n_fragments = 0;
        {
            Entries<T> e;
            load_entries<T, C, false>(st, count, wave, __ballot(done), g.h.opacity, weight, slot_pixel, e);
            float dots[K][NF];   // features . grad of the fragment's pixel
#pragma unroll
            for (int k = 0; k < K; ++k) {
                float4 feat[C / 4];
#pragma unroll
                for (int q4 = 0; q4 < C / 4; ++q4) feat[q4] = st.feat[e.j[k] * (C / 4) + q4];
#pragma unroll
                for (int q = 0; q < NF; ++q) {
                    const uint32_t pix = e.pixel[k][q] != kNoPixel ? e.pixel[k][q] : 0u;
                    float d = 0.0f;
#pragma unroll
                    for (int q4 = 0; q4 < C / 4; ++q4) {
                        const float4 gr = s_grad[wave][q4][pix];
                        d = fmaf(feat[q4].x, gr.x, d);
                        d = fmaf(feat[q4].y, gr.y, d);
                        d = fmaf(feat[q4].z, gr.z, d);
                        d = fmaf(feat[q4].w, gr.w, d);
                    }
                    arrive(d);   // computed here, not where it is used: the loaded values are not kept alive
                    dots[k][q] = d;
                }
            }
            build_fragment_lists<T, C, false>(qs, st, wave, e, my_start, my_count, n_fragments,
                                              [&](int k, int q) { return dots[k][q]; });
        }
        if (n_fragments != 0u) {
            // ---- pixels with short lists: the sequential walk (kernels.cu:383-417)
            if (my_count <= kLongList) {
                for (uint32_t i = 0; i < my_count; ++i) {
                    const uint32_t pos = my_start + i;
                    const float2 e = qs.fragment[pos];
                    const float a = done ? 0.0f : e.x, sd = e.y;
                    const float bw = Tr * a;
                    const float one_minus_a = 1.0f - a;
                    // the hardware reciprocal (1 ulp) instead of an IEEE division (ten instructions): the gradient
                    // is compared to 1e-4
                    const float rcp = __builtin_amdgcn_rcpf(fmaxf(one_minus_a, kOneMinusAlphaEps));
                    running = fmaf(bw, sd, running);
                    const float dalpha = done ? 0.0f : fmaf(Tr, sd, (running + offset) * rcp);
                    qs.fragment[pos] = make_float2(bw, dalpha);
                    Tr *= one_minus_a;
                    done = done || Tr < kTransmittanceThreshold;
                }
            }
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
                    const float rcp = __builtin_amdgcn_rcpf(fmaxf(1.0f - a, kOneMinusAlphaEps));
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
        }
        const bool all_done = barrier_all_done<T>(s_quad, done);
        // ---- the gather moves on in front of the stores of the write phase (see the forward kernel)
        const uint32_t mine_tag = g.h.tag, mine_row = g.h.row;
        advance_ordered<T, C>(g, ordered_records, begin, range.y);
        // ---- write: thread t owns staged instance t: gradient of the point from the fragments the waves placed
        if (valid) {
            uint32_t field[4];
            load_fields<T, C, false>(st, tid, field);
            float gf[C];
#pragma unroll
            for (int c = 0; c < C; ++c) gf[c] = 0.0f;
            float gop = 0.0f;
            bool any_weight = false;
#pragma unroll
            for (int c = 0; c < 4; ++c)
                if (field[c] & kPlaced) {
                    const int q = T == 16 ? c : 0;
                    const float2 e = s_quad[q].fragment[field[c] >> 8];   // {blending weight, d loss / d alpha}
                    gop = fmaf(e.y, weight[c], gop);
                    if (e.x > 0.0f) {
                        any_weight = true;
                        const uint32_t pix = field[c] & kPixelMask;
#pragma unroll
                        for (int q4 = 0; q4 < C / 4; ++q4) {
                            const float4 gr = s_grad[q][q4][pix];
                            gf[4 * q4] = fmaf(e.x, gr.x, gf[4 * q4]);
                            gf[4 * q4 + 1] = fmaf(e.x, gr.y, gf[4 * q4 + 1]);
                            gf[4 * q4 + 2] = fmaf(e.x, gr.z, gf[4 * q4 + 2]);
                            gf[4 * q4 + 3] = fmaf(e.x, gr.w, gf[4 * q4 + 3]);
                        }
                    }
                }
            if (any_weight || gop != 0.0f) {
                // a point that straddles tiles gets its gradient from up to four blocks: each writes a row of
                // its own (summed up by k_grad_reduce); no atomics, and the sum has a fixed order
                const uint32_t point = mine_tag & kRecordIdMask;
                float* dst = grad_view + (size_t)point * C;
                float* dst_opacity = grad_opacities + point;
                if (mine_tag & kRecordMulti) {
                    dst = rows.features + (size_t)mine_row * C;
                    dst_opacity = rows.opacities + mine_row;
                    rows.flags[mine_row] = 1;
                }
#pragma unroll
                for (int q4 = 0; q4 < C / 4; ++q4)
                    ((float4*)dst)[q4] = make_float4(gf[4 * q4], gf[4 * q4 + 1], gf[4 * q4 + 2], gf[4 * q4 + 3]);
                *dst_opacity = gop;
            }
        }
        if (all_done) break;
    }
}

}  // namespace blend
