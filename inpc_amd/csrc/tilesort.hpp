// tilesort.hpp — per-tile depth sort of the binned instances, inside LDS. Included by raster.hip.
//
// The reference sorts all drawn points by depth with one device-wide radix sort, expands them into
// (tile, point) instances and sorts those by tile with a second, stable device-wide sort
// (B/rasterization/src/bilinear/forward.cu:91-141): the result is, for every tile, its instances ordered by
// (depth bits, compaction order). With points compacted in ascending point index that is the order
// (tile, depth bits, point index), and it can be had without any device-wide sort: the preprocess pass drops a
// (depth key, point index) pair per instance into the bin of its tile, and one block per tile sorts its bin.
//
//   elements   u64 = depth key << 32 | point index: the order wanted is plain ascending u64 order
//   in LDS     least-significant-digit radix sort, 4-bit digits, over the key bits. A thread owns up to 15
//              consecutive elements, holds them in registers during a pass (so the pass works in place) and
//              counts their digits in sixteen 4-bit fields of one 64-bit register; the 16 x threads counts are
//              scanned in digit-major order, which is a stable ranking. Digits that are the same for all
//              elements of the tile are skipped (the depths of one tile mostly share their leading bits).
//   ties       elements with equal keys come out in the order they were binned, which is arbitrary: short runs
//              of equal keys are put right in place (rank by point index inside the run); a tile with a long
//              run is sorted again over all 64 bits.
//   big tiles  more elements than fit LDS: runs of kCap elements are sorted as above and written back, then
//              merged pairwise through global memory (rank of an element = its place in its own run + the
//              number of smaller elements in the partner run, by binary search on the full 64 bits).
#pragma once

namespace tilesort {

constexpr int kMaxPer = 15;                 // elements per thread: 3, 7, 11 or 15 (odd: conflict-free LDS rows; at
                                            // most 15: a thread's digit counts fit 4-bit fields)
constexpr int kDigits = 16;
constexpr uint32_t kShortRun = 16;          // ties are fixed in place while no run of equal keys reaches further than
                                            // this from any of its elements
constexpr uint64_t kPad = ~0ull;            // sorts behind every element
constexpr int kLargeThreads = 512, kSmallThreads = 128;   // block sizes of the two kernels
constexpr uint32_t kSmallTile = kSmallThreads * kMaxPer;  // tiles up to this size go to the small blocks

// LDS of a block of THREADS threads.
template <int THREADS>
struct Shared {
    static constexpr int kCap = THREADS * kMaxPer;        // elements sorted in LDS at a time
    uint64_t buf[kCap];
    alignas(16) uint16_t count[kDigits * THREADS];        // [digit][thread], scanned in this order
    uint32_t wave_sum[THREADS / kWave];
    uint32_t bits_or[2], bits_and[2];                     // over the tile's elements: [0] point index, [1] key
    static_assert(kCap <= kDigits * THREADS && kCap <= 65536, "count[] also holds one 16-bit place per element");
};

__device__ __forceinline__ uint32_t hi32(uint64_t v) { return (uint32_t)(v >> 32); }
__device__ __forceinline__ uint32_t lo32(uint64_t v) { return (uint32_t)v; }

__device__ __forceinline__ uint32_t wave_inclusive_u32(uint32_t v) {
    v += blend::dpp_take<blend::kDppRowShr1, 0xf>(0u, v);
    v += blend::dpp_take<blend::kDppRowShr2, 0xf>(0u, v);
    v += blend::dpp_take<blend::kDppRowShr4, 0xf>(0u, v);
    v += blend::dpp_take<blend::kDppRowShr8, 0xf>(0u, v);
    v += blend::dpp_take<blend::kDppRowBcast15, 0xa>(0u, v);
    v += blend::dpp_take<blend::kDppRowBcast31, 0xc>(0u, v);
    return v;
}

// The 4-bit digit at bit `shift` (a multiple of 4) of a 64-bit element.
__device__ __forceinline__ uint32_t digit_of(uint64_t v, int shift) {
    const uint32_t word = shift >= 32 ? hi32(v) : lo32(v);
    return (word >> (shift & 31)) & 15u;
}

// One stable counting pass, in place, on the 4-bit digit at bit `shift`. The first `active` threads (a multiple
// of 64) own kPer consecutive elements each; every thread of the block calls it (the others only meet the
// barriers). All elements are in registers before the first one is stored, so one buffer suffices.
template <int THREADS, int kPer>
__device__ __forceinline__ void digit_pass(Shared<THREADS>& sh, uint32_t t, uint32_t active, int shift) {
    const uint32_t lane = t & 63u, wave = t >> 6;
    const bool on = t < active;
    uint64_t v[kPer];
    uint64_t fields = 0ull;   // sixteen 4-bit counters: kPer <= 15 elements per thread cannot overflow one
    if (on) {
#pragma unroll
        for (int e = 0; e < kPer; ++e) {
            v[e] = sh.buf[t * kPer + e];
            fields += 1ull << (4u * digit_of(v[e], shift));
        }
#pragma unroll
        for (int d = 0; d < kDigits; ++d) sh.count[d * active + t] = (uint16_t)((fields >> (4 * d)) & 15ull);
    }
    __syncthreads();
    // exclusive scan of the 16 * active counts in storage order; thread t owns entries [16 t, 16 t + 16)
    uint32_t w[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};   // two counts per word
    uint32_t sum = 0, incl = 0;
    uint4* mine = (uint4*)(sh.count + 16u * t);
    if (on) {
        const uint4 a = mine[0], b = mine[1];
        w[0] = a.x, w[1] = a.y, w[2] = a.z, w[3] = a.w, w[4] = b.x, w[5] = b.y, w[6] = b.z, w[7] = b.w;
#pragma unroll
        for (int i = 0; i < 8; ++i) sum += (w[i] & 0xFFFFu) + (w[i] >> 16);
        incl = wave_inclusive_u32(sum);
        if (lane == 63u) sh.wave_sum[wave] = incl;
    }
    __syncthreads();
    if (on) {
        uint32_t run = incl - sum;
#pragma unroll
        for (int k = 0; k < THREADS / kWave; ++k) run += (uint32_t)k < wave ? sh.wave_sum[k] : 0u;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t c0 = w[i] & 0xFFFFu, c1 = w[i] >> 16;
            w[i] = run | ((run + c0) << 16);
            run += c0 + c1;
        }
        mine[0] = make_uint4(w[0], w[1], w[2], w[3]);
        mine[1] = make_uint4(w[4], w[5], w[6], w[7]);
    }
    __syncthreads();
    if (on) {
        uint64_t seen = 0ull;     // how many of this thread's earlier elements had the same digit
#pragma unroll
        for (int e = 0; e < kPer; ++e) {
            const uint32_t d = digit_of(v[e], shift);
            const uint32_t at = (uint32_t)sh.count[d * active + t] + (uint32_t)((seen >> (4u * d)) & 15ull);
            seen += 1ull << (4u * d);
            sh.buf[at] = v[e];
        }
    }
    __syncthreads();
}

// Sorts the n <= kPer * active elements in sh.buf ascending as u64 (the slots behind them, up to
// kPer * active, hold kPad). All threads of the block call it.
template <int THREADS, int kPer>
__device__ void sort_run(Shared<THREADS>& sh, uint32_t n, uint32_t active, int key_bits) {
    // the thread index as a value of this function's own: the compiler otherwise computes the element addresses of
    // all four instantiations (kPer = 3, 7, 11, 15) at the top of the kernel and keeps them in registers throughout
    uint32_t t = threadIdx.x;
    blend::arrive(t);
    const uint32_t lane = t & 63u;
    const bool on = t < active;
    // bits that differ between the elements
    {
        uint32_t or_lo = 0u, or_hi = 0u, and_lo = ~0u, and_hi = ~0u;
#pragma unroll
        for (int e = 0; e < kPer; ++e) {
            const uint32_t p = t * kPer + e;
            if (on && p < n) {
                const uint64_t v = sh.buf[p];
                or_lo |= lo32(v);
                or_hi |= hi32(v);
                and_lo &= lo32(v);
                and_hi &= hi32(v);
            }
        }
        for (int s = 32; s > 0; s >>= 1) {
            or_lo |= __shfl_xor(or_lo, s, 64);
            or_hi |= __shfl_xor(or_hi, s, 64);
            and_lo &= __shfl_xor(and_lo, s, 64);
            and_hi &= __shfl_xor(and_hi, s, 64);
        }
        if (t < 2) {
            sh.bits_or[t] = 0u;
            sh.bits_and[t] = ~0u;
        }
        __syncthreads();
        if (lane == 0u && on) {
            atomicOr(&sh.bits_or[0], or_lo);
            atomicOr(&sh.bits_or[1], or_hi);
            atomicAnd(&sh.bits_and[0], and_lo);
            atomicAnd(&sh.bits_and[1], and_hi);
        }
        __syncthreads();
    }
    const uint32_t vary_lo = sh.bits_or[0] ^ sh.bits_and[0], vary_hi = sh.bits_or[1] ^ sh.bits_and[1];
    auto key_passes = [&]() {
        for (int shift = 0; shift < key_bits; shift += 4)
            if ((vary_hi >> shift) & 15u) digit_pass<THREADS, kPer>(sh, t, active, 32 + shift);
    };
    key_passes();
    // elements with equal keys stand in the order they were binned; the order wanted is by point index
    bool tied[kPer];
    bool any = false;
#pragma unroll
    for (int e = 0; e < kPer; ++e) {
        const uint32_t p = t * kPer + e;
        tied[e] = false;
        if (on && p < n) {
            const uint32_t key = hi32(sh.buf[p]);
            tied[e] = (p > 0u && hi32(sh.buf[p - 1u]) == key) || (p + 1u < n && hi32(sh.buf[p + 1u]) == key);
        }
        any = any || tied[e];
    }
    if (__syncthreads_or(any) == 0) return;
    // Runs of equal keys are mostly short, however many there are: every tied element looks along its run, up to
    // kShortRun elements to either side, and takes the place its point index gives it inside the run. The places go
    // to sh.count (free between the passes; a place is below kCap <= 65536 / 8), so that no thread keeps a table
    // of them in registers; then all tied elements are read before the first one is stored. A longer run anywhere
    // in the tile sends the tile to the sort over all 64 bits below (nothing has been stored by then).
    {
        bool long_run = false;
#pragma unroll
        for (int e = 0; e < kPer; ++e) {
            if (!tied[e]) continue;
            const uint32_t p = t * kPer + e;
            const uint64_t own = sh.buf[p];
            const uint32_t key = hi32(own), mine = lo32(own);
            uint32_t first = p, last = p + 1u, smaller = 0u;
            for (uint32_t step = 0; first > 0u; ++step) {
                const uint64_t w = sh.buf[first - 1u];
                if (hi32(w) != key) break;
                if (step == kShortRun) {
                    long_run = true;
                    break;
                }
                --first;
                smaller += lo32(w) < mine ? 1u : 0u;
            }
            for (uint32_t step = 0; last < n; ++step) {
                const uint64_t w = sh.buf[last];
                if (hi32(w) != key) break;
                if (step == kShortRun) {
                    long_run = true;
                    break;
                }
                ++last;
                smaller += lo32(w) < mine ? 1u : 0u;
            }
            sh.count[p] = (uint16_t)(first + smaller);
        }
        if (__syncthreads_or(long_run) == 0) {
            uint64_t v[kPer];
#pragma unroll
            for (int e = 0; e < kPer; ++e)
                if (tied[e]) v[e] = sh.buf[t * kPer + e];
            __syncthreads();
#pragma unroll
            for (int e = 0; e < kPer; ++e)
                if (tied[e]) sh.buf[sh.count[t * kPer + e]] = v[e];
            __syncthreads();
            return;
        }
    }
    // many ties: sort over all 64 bits, least significant digit first
    for (int shift = 0; shift < 32; shift += 4)
        if ((vary_lo >> shift) & 15u) digit_pass<THREADS, kPer>(sh, t, active, shift);
    key_passes();
}

// Loads `n` <= THREADS * kMaxPer elements from `src` into sh.buf and sorts them there.
template <int THREADS>
__device__ __forceinline__ void load_and_sort(Shared<THREADS>& sh, const uint64_t* __restrict__ src, uint32_t n, int key_bits) {
    const uint32_t t = threadIdx.x;
    // as few threads as hold the elements with at most kMaxPer each: the per-thread cost of a pass does not
    // depend on the number of its elements
    uint32_t active = kWave;
    while (active < (uint32_t)THREADS && active * kMaxPer < n) active <<= 1;
    const uint32_t need = (n + active - 1u) / active;
    const uint32_t per = need <= 3u ? 3u : need <= 7u ? 7u : need <= 11u ? 11u : 15u;
    for (uint32_t p = t; p < per * active; p += THREADS) sh.buf[p] = p < n ? src[p] : kPad;
    __syncthreads();
    if (per == 3u) sort_run<THREADS, 3>(sh, n, active, key_bits);
    else if (per == 7u) sort_run<THREADS, 7>(sh, n, active, key_bits);
    else if (per == 11u) sort_run<THREADS, 11>(sh, n, active, key_bits);
    else sort_run<THREADS, 15>(sh, n, active, key_bits);
}

// One block per tile, longest bins first. pairs[begin .. end) of a tile are its elements in no particular order;
// afterwards points[begin .. end) holds their point indices in ascending element order. `pairs` and `scratch`
// (same size) are clobbered for tiles with more than THREADS * kMaxPer elements. Two launches cover the tiles:
// blocks of kSmallThreads threads take the tiles of at most kSmallTile elements (many blocks per CU), blocks of
// kLargeThreads threads the others; a block whose tile belongs to the other launch ends at once.
template <int THREADS>
__global__ void __launch_bounds__(THREADS, 4)   // four waves per SIMD: 128 registers
    k_tile_sort(const uint2* __restrict__ ranges, const uint32_t* __restrict__ tile_order, uint64_t* pairs,
                uint64_t* scratch, uint32_t* __restrict__ points, int key_bits) {
    INPC_DYNAMIC_LDS(unsigned char, s_raw);
    Shared<THREADS>& sh = *reinterpret_cast<Shared<THREADS>*>(s_raw);
    constexpr uint32_t kThreads = THREADS, kCap = Shared<THREADS>::kCap;
    const uint32_t t = threadIdx.x;
    const uint2 range = ranges[tile_order[blockIdx.x]];
    const uint32_t begin = range.x, n = range.y - range.x;
    if (n == 0u || (n <= kSmallTile) != (THREADS == kSmallThreads)) return;
    if (n <= kCap) {
        load_and_sort<THREADS>(sh, pairs + begin, n, key_bits);
        for (uint32_t p = t; p < n; p += kThreads) points[begin + p] = lo32(sh.buf[p]);
        return;
    }
    // runs of kCap elements, each sorted in LDS and written back in place
    for (uint32_t first = 0; first < n; first += kCap) {
        const uint32_t len = min((uint32_t)kCap, n - first);
        load_and_sort<THREADS>(sh, pairs + begin + first, len, key_bits);
        for (uint32_t p = t; p < len; p += kThreads) pairs[begin + first + p] = sh.buf[p];
        __syncthreads();
    }
    // pairwise merges; the global stores of a level are visible to the whole block behind the barrier
    uint64_t* from = pairs + begin;
    uint64_t* to = scratch + begin;
    for (uint32_t width = kCap; width < n; width <<= 1) {
        constexpr int kAhead = 8;   // independent searches per thread
        for (uint32_t base = 0; base < n; base += kAhead * kThreads) {
            uint64_t v[kAhead];
            uint32_t lo[kAhead], hi[kAhead];   // the part of the partner run still searched
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                const uint32_t p = base + u * kThreads + t;
                lo[u] = hi[u] = 0u;
                v[u] = 0ull;
                if (p < n) {
                    v[u] = from[p];
                    const uint32_t run = p / width, left = (run & ~1u) * width;
                    const uint32_t mid = min(left + width, n), right_end = min(left + 2u * width, n);
                    lo[u] = (run & 1u) ? left : mid;
                    hi[u] = (run & 1u) ? mid : right_end;
                }
            }
            bool busy = true;
            while (busy) {
                busy = false;
#pragma unroll
                for (int u = 0; u < kAhead; ++u)
                    if (lo[u] < hi[u]) {
                        const uint32_t mid = (lo[u] + hi[u]) >> 1;
                        if (from[mid] < v[u]) lo[u] = mid + 1u;
                        else hi[u] = mid;
                        busy = busy || lo[u] < hi[u];
                    }
            }
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                const uint32_t p = base + u * kThreads + t;
                if (p < n) {
                    const uint32_t run = p / width, left = (run & ~1u) * width;
                    const uint32_t mid = min(left + width, n);
                    // lo[u]: first element of the partner run that is not smaller than v
                    const uint32_t smaller = (run & 1u) ? lo[u] - left : lo[u] - mid;
                    const uint32_t own = (run & 1u) ? p - mid : p - left;
                    to[left + own + smaller] = v[u];
                }
            }
        }
        __syncthreads();
        uint64_t* swap = from;
        from = to;
        to = swap;
    }
    for (uint32_t p = t; p < n; p += kThreads) points[begin + p] = lo32(from[p]);
}

}  // namespace tilesort
